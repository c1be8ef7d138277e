"""Hybrid decoders: a stack whose layers each pick one mixer -- chunk-masked attention over the
paged cache, latent attention over a cache of compressed rows, minGRU, gated linear attention or
mLSTM -- around an fp32 residual stream.

Four designs are served, told apart by ``architecture`` in ``config.json`` (``DESIGNS``); the file lists
the layers (``layers[i].type``, ``.mixer`` sizes, ``.mlp``), and every size and constant comes from
there or from a tensor's shape.

Gizilorn (pre-norm, a residual of several parallel streams):

* ``e = rms_norm(embed[token]) * w_e``; the residual is ``streams`` copies x_1 .. x_S of e. A sublayer reads
  ``u = sum_s in[s] x_s`` through its RMS norm and writes all streams at once from the old ones,
  ``x_t <- sum_s mix[s, t] x_s + out[t] y`` (``hc1`` for the mixer, ``hc2`` for the feed-forward); the model's
  output is ``head . rms_norm(sum_s x_s)``;
* ``attention``: biased q / k / v projections; q and k turn over their first ``rot.dims`` coordinates (i with
  i + dims / 2), the values over their WHOLE width by their own position and are cached so; scores are scaled,
  then capped (``softcap * tanh(s / softcap)``); a window of ``mask.size`` positions; a softmax whose denominator carries
  an extra 1 (a sink); the heads' weights are mixed by ``talk`` [H, H] before they meet the values of the head's own
  group; each head's result turns back by the row's position; ``W_o``;
* ``latent_attention``: a query head is [dim plain | rot_dim turned] coordinates; the cached row per token is the
  RMS-normed compressed row (``kv_rank``) beside ONE turned key part (``rot_dim``, neighbouring pairs) that all
  heads share; keys and values are linear maps of the compressed row (moved to the query and the output side as
  for Telurax); a window; a plain softmax; the heads' results are gated coordinate by coordinate with
  ``sigmoid(W_g h)``; ``kv_from: j`` reads layer j's cached rows (no down-projection of its own);
* feed-forward: ``down(xielu(up h + b) ) + b`` with xIELU ``softplus(p) z^2 + z/2`` above zero and
  ``(1/2 + softplus(q)) (exp(z) - 1 - z) + z/2`` below.

Surevik (pre-norm, Dynamic Tanh norms):

* ``x = embed[token] * embedding.scale``; a layer computes ``x += m * mixer(n1(x))`` and, if it has a
  feed-forward, ``x += m * ff(n2(x))`` with ``m = residual_mult`` and ``n(x) = tanh(alpha x) * w + b``
  (no mean, no variance; a scalar ``alpha``, vectors ``w``, ``b``); logits are ``embed . n_final(x)``, the
  embedding table itself without its scale;
* ``loop``: the layers ``start .. stop - 1`` run ``times`` times in a row with the same weights, every pass
  over cache planes of its own; each pass begins with ``x <- W_in [x; x0]`` (``x0``: the embedding output);
* ``attention``: ``q = W_q h``, ``k = W_k h``, no biases, no norms, and no value projection: the values
  are the keys as projected. q and k (not the values) rotate in neighbouring coordinate pairs (2i, 2i + 1)
  over the first ``rot.dims`` coordinates of each head; softmax over the last ``mask.size`` positions
  (the row's own included); grouped key/value heads;
* feed-forward: a routed mixture whose router scores are ``sigmoid(W_r h)``; the ``top`` best experts
  are taken with their scores as weights (not renormalised), and the weight multiplies the expert's
  INPUT; an expert is ``down(g * sigmoid(1.702 g) * (u + 1))`` with ``g = min(gate h, limit)``,
  ``u = clamp(up h, -limit, limit)``; a shared expert of the same form runs for every token, scaled by
  ``sigmoid(W_sg h)``.

Telurax (pre-norm):

* ``x = embed[token] * embedding.scale`` plus a sinusoidal position vector (entry 2i: sin, 2i+1: cos of
  ``p * 10000^(-2i/width)``); a layer computes ``x += mixer(n1(x))`` and, if it has a feed-forward,
  ``x += ff(n2(x))`` with ``n(x) = x / sqrt(mean(x^2) + eps) * (1 + w)``; logits are
  ``head . n_final(x) * logit_scale``;
* ``latent_attention``: queries ``W_q h`` per head; ONE compressed row per token, the RMS-normed
  ``W_dkv h`` (plain weight), is cached, and every head's keys and values are linear maps of it
  (``W_uk``, ``W_uv``). The maps are moved to the query and to the output side (scores
  ``(W_uk_h^T q_h) . c_j``, output ``W_uv_h sum_j p_j c_j``), so attention runs over the cached rows
  themselves: H query heads, one key/value head of the latent's width, causal softmax, no positions.
  Each head's output is scaled by ``sigmoid(W_g h)_h`` before ``W_o``;
* ``mlstm``: per head a matrix memory ``S <- a S + b k v^T`` with a normaliser ``n <- a n + b k``,
  ``a = exp(f + m' - m)``, ``b = exp(i - m)``, ``m = max(f + m', i)`` (m' the previous maximum, 0 at
  the start), soft-capped gate logits; read out ``S^T q / (max(|n.q|, exp(-m)) + 1e-6)``, unit RMS
  per head, a weight over all heads, an output gate ``sigmoid(W_g h)``, ``W_o``;
* feed-forwards: ``down(relu(gate h) * up h)``, or a routed mixture (softmax router, bias-corrected
  group-limited top-k choice, identity experts that return their input, a shared expert; experts are
  ``down(relu(up h)^2)``).

Nidozen (norms on the sublayer outputs):

* a layer computes ``x += norm1(mixer(x))`` and, if it has a feed-forward, ``x += norm2(ff(x))``:
  the sublayers read the stream itself and the norm (RMS with ONE gain for all coordinates) sits
  on their output;
* ``attention``: biased q/k/v/o projections, an RMS norm over the whole query (key) projection
  before the heads are split, rotary positions on the first ``rot.dims`` coordinates of each head,
  value heads scaled to unit RMS, grouped key/value heads of widths ``dim`` / ``vdim``, softmax over
  the keys of the row's own chunk of ``mask.size`` positions; ``kv_from: j`` reads layer j's cache;
* ``mingru``: S <- (1 - z) S + z c with gates that read only the current token;
* ``gla``: per head S <- diag(a) S + k v^T, read out with q, normed per head and gated;
* feed-forward: down(relu(up(x))^2).

The residual stream, norms, scores, recurrences and their states are fp32 whatever the activation
type (``dtype``: bf16 products with fp32 accumulation, or fp32 throughout). Keys / values live in
the paged pool the engine's KV manager hands out blocks of; recurrent states live in per-sequence
slots of the same manager (``HybridCache``). The step description is the engine's ``AttnMeta``
with its ``layout`` (row ranges, row -> sequence, state slots, block tables of ALL sequences of
the step, prompt portions and single decoded tokens alike).
"""
from __future__ import annotations

import json
import zlib
from dataclasses import dataclass, field
from pathlib import Path
from typing import Dict, List, Optional, Tuple

import torch

from .. import ops

ARCHITECTURE = "Nidozen"


@dataclass(frozen=True)
class Design:
    """What a design fixes for all of its models."""

    name: str
    mixers: Tuple[str, ...]
    pre_norm: bool = False          # norms with a weight per coordinate on the sublayer INPUTS (else: one-gain norms on the outputs)
    norm_offset: float = 0.0        # stored norm weights are offsets from this value
    pos_base: float = 0.0           # > 0: a sinusoidal position vector of this base is added to the embedding
    dense_ff: str = "relu2"         # dense feed-forward: down(relu(up x)^2) | "glu_relu": down(relu(gate x) * up x) |
                                    # "xielu": down(xielu(up x + b)) + b with the activation's two numbers in ``mlp.act`` | "": none
    norm: str = "rms"               # "dyt": Dynamic Tanh, tanh(alpha x) * w + b (tensors <name>, <name>.b, <name>.alpha)
    tied_head: bool = False         # logits from the embedding table (no ``head`` tensor)
    attention: str = "normed"       # what the ``attention`` mixer is: "normed" (biases, whole-projection q / k norms,
                                    # rotate-half pairs, unit-RMS values, ``mask.size`` = chunk) | "keys_as_values" (no
                                    # biases or norms, values = the un-rotated keys, neighbouring pairs, ``mask.size`` = window)
                                    # | "talking" (biased q / k / v, rotate-half pairs on q and k, values turned by their own
                                    # position, capped scores, ``mask.size`` = window, a sink in the softmax, the heads'
                                    # weights mixed by a matrix)
    latent: str = "plain"           # latent attention: "plain" (no positions, all earlier rows, a gate per head) | "rotary" (a
                                    # turned key part shared by all heads beside the compressed row, a window, a gate per
                                    # output coordinate, ``kv_from``)
    embed_norm: bool = False        # an RMS norm (tensor ``embed.norm``) on the embedding rows
    hyper: bool = False             # the residual is ``streams`` parallel streams (tensors ``<layer>.hc<q>.{in,out,mix}``)
    routed_ff: str = "grouped_relu2"    # "sigmoid_clamped": sigmoid scores, weight on the expert's input, clamped gated experts | "": none
    # constants of the clamped gated unit g * sigmoid(slope g) * (u + shift)
    glu_slope: float = 1.702
    glu_shift: float = 1.0


DESIGNS: Dict[str, Design] = {
    "Nidozen": Design("Nidozen", ("attention", "mingru", "gla")),
    "Telurax": Design("Telurax", ("latent_attention", "mlstm"), pre_norm=True, norm_offset=1.0, pos_base=10000.0,
                      dense_ff="glu_relu"),
    "Surevik": Design("Surevik", ("attention",), pre_norm=True, dense_ff="", norm="dyt", tied_head=True,
                      attention="keys_as_values", routed_ff="sigmoid_clamped"),
    "Gizilorn": Design("Gizilorn", ("attention", "latent_attention"), pre_norm=True, dense_ff="xielu", attention="talking",
                       latent="rotary", embed_norm=True, hyper=True, routed_ff=""),
}
MIXERS = tuple(dict.fromkeys(m for d in DESIGNS.values() for m in d.mixers))


@dataclass(frozen=True)
class MoESpec:
    """A routed feed-forward: ``experts`` small relu^2 feed-forwards of width ``ff`` plus ``identity``
    experts without tensors; the router's ``experts + identity`` outputs form ``groups`` equal runs of
    neighbours of which the ``keep`` best stay eligible; ``top`` are chosen per token, weighted by their
    softmax score times ``scale``; ``shared_ff`` > 0: a shared expert of that width runs for every token.

    ``unit`` "clamped_glu" (with ``score`` "sigmoid"): experts are down(g * sigmoid(slope g) * (u + shift)) with
    g = min(gate x, limit), u = clamp(up x, -limit, limit); the weight multiplies the expert's input; the
    shared expert has a limit of its own and a sigmoid gate, one number per token."""

    experts: int
    ff: int
    top: int
    identity: int = 0
    groups: int = 1
    keep: int = 1
    scale: float = 1.0
    shared_ff: int = 0
    score: str = "softmax"
    unit: str = "relu2"
    limit: float = 0.0
    shared_limit: float = 0.0

    @property
    def clamped(self) -> bool:
        return self.unit == "clamped_glu"

    @property
    def outputs(self) -> int:
        return self.experts + self.identity


@dataclass(frozen=True)
class LayerSpec:
    type: str
    # attention / gla
    heads: int = 0
    kv_heads: int = 0
    dim: int = 0
    vdim: int = 0
    scale: float = 0.0
    chunk: int = 0               # keys visible only inside the row's chunk of this many positions (0: all)
    window: int = 0              # keys visible only this far back (0: all)
    rot_dims: int = 0
    rot_base: float = 10000.0
    kv_from: int = -1            # attention / latent attention: read this layer's cached rows (-1: own)
    values_are_keys: bool = False    # attention: no norms, biases or value projection; neighbouring rotary pairs
    # attention whose heads' weights are mixed: score cap (0: none), a softmax whose denominator carries an extra 1,
    # values turned by their own position over their whole width (and the result turned back)
    talk: bool = False
    softcap: float = 0.0
    sink: bool = False
    rotate_values: bool = False
    # gla
    tau: float = 1.0
    rank: int = 0                # width of the decay's low-rank bottleneck (from the tensor's shape)
    # mingru
    width: int = 0
    # latent attention: width of the cached compressed row; width of the turned key part cached beside it (0: none),
    # which is also the turned part of every query head; a gate per output coordinate instead of one per head
    kv_rank: int = 0
    rot_dim: int = 0
    gate_full: bool = False
    # mlstm: soft cap of the gate logits (0: none)
    gate_cap: float = 0.0
    # feed-forward (0: none); ``moe``: a routed one instead of the dense one
    ff: int = 0
    moe: Optional[MoESpec] = None

    @property
    def owns_kv(self) -> bool:
        return self.type == "attention" and self.kv_from < 0

    @property
    def owns_latent(self) -> bool:
        return self.type == "latent_attention" and self.kv_from < 0

    @property
    def has_ff(self) -> bool:
        return self.ff > 0 or self.moe is not None

    def state_size(self) -> int:
        """fp32 numbers of recurrent state per sequence."""
        if self.type == "mingru":
            return self.width
        if self.type == "gla":
            return self.heads * self.dim * self.vdim
        if self.type == "mlstm":          # S with the normaliser as an extra column, then the running maxima
            return self.heads * self.dim * (self.vdim + 1) + self.heads
        return 0

    def cache_elems(self) -> int:
        """Cached elements per token."""
        if self.owns_kv and self.values_are_keys:     # rotated keys, and the un-rotated ones unless nothing rotates
            return self.kv_heads * self.dim * (2 if self.rot_dims else 1)
        if self.owns_kv:
            return self.kv_heads * (self.dim + self.vdim)
        return self.kv_rank + self.rot_dim if self.owns_latent else 0


@dataclass(frozen=True)
class HybridConfig:
    name: str
    vocab_size: int
    hidden_size: int
    rms_eps: float
    layers: Tuple[LayerSpec, ...]
    max_position: int = 1 << 20
    model_type: str = "nidozen"
    architecture: str = ARCHITECTURE
    embed_scale: float = 1.0
    logit_scale: float = 1.0
    residual_mult: float = 1.0      # every sublayer output is scaled by this before it joins the stream
    loop: Tuple[int, int, int] = (0, 0, 1)      # layers [start, stop) run ``times`` times in a row (times 1: no loop)
    streams: int = 0                # parallel residual streams (designs with hyper-connections)

    @property
    def design(self) -> Design:
        return DESIGNS[self.architecture]

    @property
    def looped(self) -> bool:
        return self.loop[1] > self.loop[0]          # (an empty range loops over nothing, whatever its count)

    @property
    def runs(self) -> Tuple[Tuple[int, bool], ...]:
        """The layer runs of one forward pass in order: (layer, whether the stream is re-injected before
        it). Run r has cache / state planes of its own: a looped layer has one set per pass."""
        start, stop, times = self.loop
        if not self.looped:
            return tuple((i, False) for i in range(len(self.layers)))
        out = [(i, False) for i in range(start)]
        for _ in range(times):
            out += [(i, i == start) for i in range(start, stop)]
        return tuple(out + [(i, False) for i in range(stop, len(self.layers))])

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @property
    def has_state(self) -> bool:
        return any(l.state_size() for l in self.layers)

    @property
    def num_heads(self) -> int:
        return max([l.heads for l in self.layers if l.type in ("attention", "latent_attention")] or [1])

    @property
    def num_kv_heads(self) -> int:
        return max([l.kv_heads for l in self.layers if l.type == "attention"] or [1])

    def kv_elems_per_token(self) -> int:
        return sum(self.layers[i].cache_elems() for i, _ in self.runs)

    def kv_bytes_per_token(self, bytes_per_elem: int = 2) -> int:
        return self.kv_elems_per_token() * bytes_per_elem

    def state_floats(self) -> int:
        return sum(self.layers[i].state_size() for i, _ in self.runs)

    def param_count(self) -> int:
        return sum(_numel(s) for s in param_shapes(self).values())

    def weight_bytes(self, bytes_per_param: int = 2) -> int:
        return self.param_count() * bytes_per_param

    def validate(self) -> None:
        if self.vocab_size <= 0 or self.hidden_size <= 0 or not self.layers:
            raise ValueError(f"{self.name}: vocab, width and at least one layer are needed")
        if self.architecture not in DESIGNS:
            raise ValueError(f"{self.name}: unknown design {self.architecture!r} (known: {', '.join(DESIGNS)})")
        known = self.design.mixers
        start, stop, times = self.loop
        if self.looped:
            if not (0 <= start and stop <= len(self.layers)) or times < 1:
                raise ValueError(f"{self.name}: loop: 0 <= start, stop <= layers and times >= 1 are needed")
            if any(l.kv_from >= 0 for l in self.layers):
                raise ValueError(f"{self.name}: looped layers and shared keys (kv_from) do not combine")
        if self.design.pos_base > 0 and self.hidden_size % 2:
            raise ValueError(f"{self.name}: a sinusoidal position vector needs an even width")
        if self.design.hyper and (not 1 <= self.streams <= ops.MAX_STREAMS or self.looped):
            raise ValueError(f"{self.name}: 1..{ops.MAX_STREAMS} residual streams are needed, and no loop")
        for i, l in enumerate(self.layers):
            if l.type not in known:
                raise ValueError(f"{self.name}: layer {i}: unknown mixer {l.type!r} (known: {', '.join(known)})")
            if l.type in ("latent_attention", "mlstm") and (l.heads <= 0 or l.dim <= 0 or l.vdim <= 0):
                raise ValueError(f"{self.name}: layer {i}: heads, dim and vdim are needed")
            if l.type == "latent_attention" and (l.kv_rank <= 0 or l.kv_rank > 512):
                raise ValueError(f"{self.name}: layer {i}: the attention kernels take a latent width of 1..512")
            if l.type == "latent_attention" and (l.rot_dim % 2 or l.rot_dim < 0 or l.rot_dims != l.rot_dim or l.window < 0):
                raise ValueError(f"{self.name}: layer {i}: the turned key part has an even width, and rot.dims equals it")
            if l.type == "latent_attention" and l.kv_from >= 0:
                src = self.layers[l.kv_from] if l.kv_from < i else None
                if src is None or not src.owns_latent:
                    raise ValueError(f"{self.name}: layer {i}: kv_from must name an earlier latent-attention layer with a "
                                     f"down-projection of its own")
                if (src.kv_rank, src.rot_dim, src.rot_base) != (l.kv_rank, l.rot_dim, l.rot_base):
                    raise ValueError(f"{self.name}: layer {i}: kv_from layer {l.kv_from} has another latent width or rotation")
            if l.type == "mlstm" and (l.dim > 256 or l.gate_cap < 0):
                raise ValueError(f"{self.name}: layer {i}: mLSTM takes dim <= 256 and a gate cap >= 0")
            if l.moe is not None:
                m = l.moe
                if m.clamped and (m.score != "sigmoid" or m.identity or not m.limit > 0 or (m.shared_ff and not m.shared_limit > 0)):
                    raise ValueError(f"{self.name}: layer {i}: clamped gated experts take sigmoid scores, positive limits "
                                     f"and no identity experts")
                if m.experts <= 0 or m.ff <= 0 or m.identity < 0 or m.top <= 0 or m.groups <= 0 or m.outputs % m.groups:
                    raise ValueError(f"{self.name}: layer {i}: experts, their width and `top` are needed, and the groups "
                                     f"must divide experts + identity")
                if not 1 <= m.keep <= m.groups or m.top > m.keep * (m.outputs // m.groups) or m.top > 32:
                    raise ValueError(f"{self.name}: layer {i}: the kept groups must hold `top` (at most 32) router outputs")
            if l.type == "mingru" and l.width <= 0:
                raise ValueError(f"{self.name}: layer {i}: minGRU needs a width")
            if l.type in ("attention", "gla") and (l.heads <= 0 or l.dim <= 0 or l.vdim <= 0):
                raise ValueError(f"{self.name}: layer {i}: heads, dim and vdim are needed")
            if l.type == "gla" and (l.dim > 256 or not l.tau > 0):
                raise ValueError(f"{self.name}: layer {i}: gated linear attention takes dim <= 256 and tau > 0")
            if l.type == "attention":
                if l.kv_heads <= 0 or l.heads % l.kv_heads:
                    raise ValueError(f"{self.name}: layer {i}: heads must be a multiple of kv_heads")
                if l.rot_dims % 2 or l.rot_dims > l.dim:
                    raise ValueError(f"{self.name}: layer {i}: rot.dims must be even and at most dim")
                if l.vdim > 256:
                    raise ValueError(f"{self.name}: layer {i}: the attention kernel takes vdim <= 256")
                if l.talk and (l.kv_from >= 0 or l.chunk or l.softcap < 0 or l.window < 0 or (l.rotate_values and l.vdim % 2)):
                    raise ValueError(f"{self.name}: layer {i}: mixed heads take keys of their own, a cap >= 0, and values "
                                     f"of even width when they turn")
                if l.values_are_keys and (l.vdim != l.dim or l.kv_from >= 0 or l.chunk):
                    raise ValueError(f"{self.name}: layer {i}: values that are the keys have the keys' width (vdim = dim)")
                if l.kv_from >= 0:
                    src = self.layers[l.kv_from] if l.kv_from < i else None
                    if src is None or not src.owns_kv:
                        raise ValueError(f"{self.name}: layer {i}: kv_from must name an earlier attention layer "
                                         f"with keys of its own")
                    if (src.kv_heads, src.dim, src.vdim) != (l.kv_heads, l.dim, l.vdim):
                        raise ValueError(f"{self.name}: layer {i}: kv_from layer {l.kv_from} has other head sizes")


def _numel(shape) -> int:
    n = 1
    for s in shape:
        n *= s
    return n


def _mlp_of(name: str, i: int, mlp: Optional[dict], design: Design):
    """(ff, MoESpec or None) of a layer's ``mlp`` entry."""
    if mlp is None:
        return 0, None
    kind = mlp.get("kind", "dense")
    if kind == "dense" and not design.dense_ff:
        raise ValueError(f"{name}: layer {i}: {design.name} has no dense feed-forward")
    if kind == "dense":
        return int(mlp["ff"]), None
    if kind != "moe" or not design.pre_norm or not design.routed_ff:
        raise ValueError(f"{name}: layer {i}: feed-forward kind {kind!r} is not supported")
    r, g = mlp["router"], mlp["router"].get("groups") or {}
    shared = mlp.get("shared") or {}
    if design.routed_ff == "sigmoid_clamped":
        return 0, MoESpec(experts=int(r["experts"]), ff=int(mlp["expert"]["ff"]), top=int(r["top"]),
                          shared_ff=int(shared.get("ff", 0)), score="sigmoid", unit="clamped_glu",
                          limit=float(mlp["expert"]["limit"]), shared_limit=float(shared.get("limit", 0.0)))
    return 0, MoESpec(experts=int(r["experts"]), ff=int(mlp["expert"]["ff"]), top=int(r["top"]),
                      identity=int(r.get("identity", 0)), groups=int(g.get("count", 1)), keep=int(g.get("keep", g.get("count", 1))),
                      scale=float(r.get("scale", 1.0)), shared_ff=int(shared.get("ff", 0)))


def _loop_of(loop: Optional[dict]) -> Tuple[int, int, int]:
    if not loop:
        return (0, 0, 1)
    return (int(loop["start"]), int(loop["stop"]), int(loop.get("times", 1)))


def config_from_dict(c: dict, name: str = "hybrid", tensor_shapes: Optional[Dict[str, tuple]] = None) -> HybridConfig:
    """Parses the ``config.json`` of a hybrid design. ``tensor_shapes`` (name -> shape of the checkpoint's
    tensors) supplies the sizes the configuration leaves to the tensors."""
    arch = c.get("architecture")
    if arch not in DESIGNS:
        raise ValueError(f"{name}: architecture {arch!r} is not one of {', '.join(DESIGNS)}")
    design = DESIGNS[arch]
    layers = []
    for i, L in enumerate(c["layers"]):
        t, m = L["type"], L.get("mixer") or {}
        if t not in design.mixers:
            raise ValueError(f"{name}: layer {i}: unknown mixer {t!r} (known: {', '.join(design.mixers)})")
        ff, moe = _mlp_of(name, i, L.get("mlp"), design)
        if t == "attention" and design.attention == "keys_as_values":
            mask, rot = m.get("mask") or {}, m.get("rot") or {}
            layers.append(LayerSpec(t, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])),
                                    dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])), scale=float(m["scale"]),
                                    window=int(mask.get("size", 0)), rot_dims=int(rot.get("dims", 0)),
                                    rot_base=float(rot.get("base", 10000.0)), values_are_keys=True, ff=ff, moe=moe))
        elif t == "attention" and design.attention == "talking":
            mask, rot = m.get("mask") or {}, m.get("rot") or {}
            layers.append(LayerSpec(t, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])),
                                    dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                                    scale=float(m.get("scale", int(m["dim"]) ** -0.5)),
                                    window=int(mask.get("size", 0)), rot_dims=int(rot.get("dims", 0)),
                                    rot_base=float(rot.get("base", 10000.0)), talk=True, softcap=float(m.get("softcap", 0.0)),
                                    sink=True, rotate_values=True, ff=ff))
        elif t == "latent_attention" and design.latent == "rotary":
            mask, rot = m.get("mask") or {}, m.get("rot") or {}
            kvf = m.get("kv_from")
            layers.append(LayerSpec(t, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                                    kv_rank=int(m["kv_rank"]), rot_dim=int(m.get("rot_dim", 0)),
                                    scale=float(m.get("scale", (int(m["dim"]) + int(m.get("rot_dim", 0))) ** -0.5)),
                                    window=int(mask.get("size", 0)), rot_dims=int(rot.get("dims", m.get("rot_dim", 0))),
                                    rot_base=float(rot.get("base", 10000.0)), kv_from=-1 if kvf is None else int(kvf),
                                    gate_full=True, ff=ff))
        elif t == "attention":
            mask, rot = m.get("mask") or {}, m.get("rot") or {}
            kvf = m.get("kv_from")
            layers.append(LayerSpec(t, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])),
                                    dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])), scale=float(m["scale"]),
                                    chunk=int(mask.get("size", 0)), window=int(mask.get("window", 0)),
                                    rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)),
                                    kv_from=-1 if kvf is None else int(kvf), ff=ff))
        elif t == "mingru":
            layers.append(LayerSpec(t, width=int(m["width"]), ff=ff))
        elif t == "gla":
            rank = int(m.get("rank", 0))
            if tensor_shapes is not None and f"l{i}.mix.a1" in tensor_shapes:
                rank = int(tensor_shapes[f"l{i}.mix.a1"][0])
            layers.append(LayerSpec(t, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                                    tau=float(m["tau"]), rank=rank or 16, ff=ff))
        elif t == "latent_attention":
            layers.append(LayerSpec(t, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                                    kv_rank=int(m["kv_rank"]), scale=float(m.get("scale", int(m["dim"]) ** -0.5)),
                                    ff=ff, moe=moe))
        else:
            layers.append(LayerSpec(t, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                                    gate_cap=float(m.get("gate_cap", 0.0)), ff=ff, moe=moe))
    cfg = HybridConfig(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]),
                       rms_eps=float(c["norm"]["eps"]), layers=tuple(layers),
                       max_position=int(c.get("max_position", 1 << 20)), model_type=arch.lower(), architecture=arch,
                       embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)),
                       logit_scale=float(c.get("logit_scale", 1.0)), residual_mult=float(c.get("residual_mult", 1.0)),
                       loop=_loop_of(c.get("loop")), streams=int(c.get("streams", 1)) if design.hyper else 0)
    cfg.validate()
    return cfg


def config_to_dict(cfg: HybridConfig) -> dict:
    layers = []
    for l in cfg.layers:
        if l.type == "attention" and l.values_are_keys:
            m = {"heads": l.heads, "kv_heads": l.kv_heads, "dim": l.dim, "vdim": l.vdim, "scale": l.scale,
                 "mask": {"size": l.window}, "rot": {"dims": l.rot_dims, "base": l.rot_base}}
        elif l.type == "attention" and l.talk:
            m = {"heads": l.heads, "kv_heads": l.kv_heads, "dim": l.dim, "vdim": l.vdim, "scale": l.scale,
                 "softcap": l.softcap, "mask": {"size": l.window}, "rot": {"dims": l.rot_dims, "base": l.rot_base}}
        elif l.type == "latent_attention" and l.gate_full:
            m = {"heads": l.heads, "dim": l.dim, "rot_dim": l.rot_dim, "vdim": l.vdim, "kv_rank": l.kv_rank, "scale": l.scale,
                 "mask": {"size": l.window}, "rot": {"dims": l.rot_dims, "base": l.rot_base}}
            if l.kv_from >= 0:
                m["kv_from"] = l.kv_from
        elif l.type == "attention":
            m = {"heads": l.heads, "kv_heads": l.kv_heads, "dim": l.dim, "vdim": l.vdim, "scale": l.scale,
                 "mask": {"size": l.chunk} if not l.window else {"size": l.chunk, "window": l.window},
                 "rot": {"dims": l.rot_dims, "base": l.rot_base}}
            if l.kv_from >= 0:
                m["kv_from"] = l.kv_from
        elif l.type == "mingru":
            m = {"width": l.width}
        elif l.type == "gla":
            m = {"heads": l.heads, "dim": l.dim, "vdim": l.vdim, "tau": l.tau, "rank": l.rank}
        elif l.type == "latent_attention":
            m = {"heads": l.heads, "dim": l.dim, "vdim": l.vdim, "kv_rank": l.kv_rank, "scale": l.scale}
        else:
            m = {"heads": l.heads, "dim": l.dim, "vdim": l.vdim, "gate_cap": l.gate_cap}
        mlp = {"kind": "dense", "ff": l.ff} if l.ff else None
        if l.moe is not None and l.moe.clamped:
            e = l.moe
            mlp = {"kind": "moe", "expert": {"ff": e.ff, "limit": e.limit}, "router": {"experts": e.experts, "top": e.top},
                   "shared": {"ff": e.shared_ff, "limit": e.shared_limit} if e.shared_ff else None}
        elif l.moe is not None:
            e = l.moe
            mlp = {"kind": "moe", "expert": {"ff": e.ff},
                   "router": {"experts": e.experts, "identity": e.identity, "top": e.top, "scale": e.scale,
                              "groups": {"count": e.groups, "keep": e.keep}},
                   "shared": {"ff": e.shared_ff} if e.shared_ff else None}
        layers.append({"type": l.type, "mixer": m, "mlp": mlp})
    out = {"architecture": cfg.architecture, "vocab": cfg.vocab_size, "width": cfg.hidden_size,
           "norm": {"eps": cfg.rms_eps}, "layers": layers}
    if cfg.design.hyper:
        out["streams"] = cfg.streams
        return out
    if cfg.design.pre_norm:
        out["embedding"] = {"scale": cfg.embed_scale}
    if cfg.design.pre_norm and not cfg.design.tied_head:
        out["logit_scale"] = cfg.logit_scale
    if cfg.design.norm == "dyt":
        out["residual_mult"] = cfg.residual_mult
    if cfg.looped:
        out["loop"] = {"start": cfg.loop[0], "stop": cfg.loop[1], "times": cfg.loop[2]}
    return out


def config_from_path(path: str) -> HybridConfig:
    p = Path(path)
    d = p if p.is_dir() else p.parent
    c = json.loads((d / "config.json").read_text())
    shapes = None
    st = d / "model.safetensors"
    if st.exists():
        from safetensors import safe_open

        with safe_open(str(st), framework="pt", device="cpu") as h:
            shapes = {k: tuple(h.get_slice(k).get_shape()) for k in h.keys()}
    return config_from_dict(c, name=d.name, tensor_shapes=shapes)


def param_shapes(cfg: HybridConfig) -> Dict[str, tuple]:
    """Checkpoint tensor names -> shapes (linear weights are [out, in])."""
    d = cfg.hidden_size
    norm = (d,) if cfg.design.pre_norm else ()
    out: Dict[str, tuple] = {"embed": (cfg.vocab_size, d)}
    dyt = cfg.design.norm == "dyt"

    def norm_tensors(name: str) -> None:
        out[name] = norm
        if dyt:
            out[name + ".b"], out[name + ".alpha"] = (d,), ()
    if cfg.looped:
        out["loop.in"] = (d, 2 * d)
    if cfg.design.embed_norm:
        out["embed.norm"] = (d,)
    for i, l in enumerate(cfg.layers):
        p = f"l{i}."
        norm_tensors(p + "norm1")
        if l.has_ff:
            norm_tensors(p + "norm2")
        if cfg.design.hyper:
            for q in ("hc1.", "hc2.") if l.has_ff else ("hc1.",):
                out[p + q + "in"], out[p + q + "out"], out[p + q + "mix"] = (cfg.streams,), (cfg.streams,), (cfg.streams, cfg.streams)
        m = p + "mix."
        if l.type == "attention" and l.talk:
            out[m + "q"], out[m + "q.b"] = (l.heads * l.dim, d), (l.heads * l.dim,)
            out[m + "k"], out[m + "k.b"] = (l.kv_heads * l.dim, d), (l.kv_heads * l.dim,)
            out[m + "v"], out[m + "v.b"] = (l.kv_heads * l.vdim, d), (l.kv_heads * l.vdim,)
            out[m + "talk"], out[m + "o"] = (l.heads, l.heads), (d, l.heads * l.vdim)
        elif l.type == "latent_attention" and l.gate_full:
            out[m + "q"] = (l.heads * (l.dim + l.rot_dim), d)
            if l.owns_latent:
                out[m + "dkv"], out[m + "dkv.norm"] = (l.kv_rank + l.rot_dim, d), (l.kv_rank,)
            out[m + "uk"], out[m + "uv"] = (l.heads * l.dim, l.kv_rank), (l.heads * l.vdim, l.kv_rank)
            out[m + "g"], out[m + "o"] = (l.heads * l.vdim, d), (d, l.heads * l.vdim)
        elif l.type == "attention" and l.values_are_keys:
            out[m + "q"], out[m + "k"] = (l.heads * l.dim, d), (l.kv_heads * l.dim, d)
            out[m + "o"] = (d, l.heads * l.vdim)
        elif l.type == "attention":
            out[m + "q"], out[m + "q.b"], out[m + "q.norm"] = (l.heads * l.dim, d), (l.heads * l.dim,), (l.heads * l.dim,)
            if l.owns_kv:
                out[m + "k"], out[m + "k.b"] = (l.kv_heads * l.dim, d), (l.kv_heads * l.dim,)
                out[m + "k.norm"] = (l.kv_heads * l.dim,)
                out[m + "v"], out[m + "v.b"] = (l.kv_heads * l.vdim, d), (l.kv_heads * l.vdim,)
            out[m + "o"], out[m + "o.b"] = (d, l.heads * l.vdim), (d,)
        elif l.type == "mingru":
            for n in ("z", "x", "g"):
                out[m + n] = (l.width, d)
            out[m + "z.b"], out[m + "x.b"] = (l.width,), (l.width,)
            out[m + "o"] = (d, l.width)
        elif l.type == "gla":
            out[m + "q"], out[m + "k"] = (l.heads * l.dim, d), (l.heads * l.dim, d)
            out[m + "v"], out[m + "g"] = (l.heads * l.vdim, d), (l.heads * l.vdim, d)
            out[m + "a1"], out[m + "a2"], out[m + "a2.b"] = (l.rank, d), (l.heads * l.dim, l.rank), (l.heads * l.dim,)
            out[m + "norm"] = (l.vdim,)
            out[m + "o"] = (d, l.heads * l.vdim)
        elif l.type == "latent_attention":
            out[m + "q"] = (l.heads * l.dim, d)
            out[m + "dkv"], out[m + "dkv.norm"] = (l.kv_rank, d), (l.kv_rank,)
            out[m + "uk"], out[m + "uv"] = (l.heads * l.dim, l.kv_rank), (l.heads * l.vdim, l.kv_rank)
            out[m + "g"] = (l.heads, d)
            out[m + "o"] = (d, l.heads * l.vdim)
        else:
            out[m + "q"], out[m + "k"] = (l.heads * l.dim, d), (l.heads * l.dim, d)
            out[m + "v"], out[m + "g"] = (l.heads * l.vdim, d), (l.heads * l.vdim, d)
            out[m + "o"], out[m + "norm"] = (d, l.heads * l.vdim), (l.heads * l.vdim,)
            for n in ("i", "f"):
                out[m + n], out[m + n + ".b"] = (l.heads, d), (l.heads,)
        f = p + "mlp."
        if l.moe is not None:
            e = l.moe
            for j in range(e.experts):
                if e.clamped:
                    out[f + f"e{j}.gate"] = (e.ff, d)
                out[f + f"e{j}.up"], out[f + f"e{j}.down"] = (e.ff, d), (d, e.ff)
            out[f + "router"] = (e.outputs, d)
            if not e.clamped:
                out[f + "correction"] = (e.outputs,)
            if e.shared_ff:
                if e.clamped:
                    out[f + "shared.gate"], out[f + "shared.sg"] = (e.shared_ff, d), (1, d)
                out[f + "shared.up"], out[f + "shared.down"] = (e.shared_ff, d), (d, e.shared_ff)
        elif l.ff:
            if cfg.design.dense_ff == "glu_relu":
                out[f + "gate"] = (l.ff, d)
            out[f + "up"], out[f + "down"] = (l.ff, d), (d, l.ff)
            if cfg.design.dense_ff == "xielu":
                out[f + "up.b"], out[f + "down.b"], out[f + "act"] = (l.ff,), (d,), (2,)
    norm_tensors("final.norm")
    if not cfg.design.tied_head:
        out["head"] = (cfg.vocab_size, d)
    return out


@dataclass
class StepLayout:
    """All sequences of a step, prompt portions first, single decoded tokens behind them
    (device tensors, int32)."""

    cu_q: torch.Tensor                      # [B+1] row ranges
    row_seq: torch.Tensor                   # [T] sequence of each row (< 0: padding row)
    block_tables: torch.Tensor              # [B, max_blocks]
    state_slots: Optional[torch.Tensor]     # [B] (< 0: padding row), None for models without state


class HybridCache:
    """Paged keys / values of the attention layers that own any, the paged compressed rows of the
    latent-attention layers that own any, and the fp32 state slots of the recurrent layers, in ONE pool. Key
    planes are [blocks, G, BS, dim], value planes [blocks, G, BS, vdim], latent planes
    [blocks, 1, BS, kv_rank + rot_dim] (keys; their first kv_rank columns are the values) in the model's activation type; a state
    plane is [slots, size] fp32. Planes belong to layer RUNS (``HybridConfig.runs``): a layer that a
    loop runs several times has a set per pass; without a loop run r is layer r."""

    def __init__(self, cfg: HybridConfig, num_blocks: int, block_size: int, num_slots: int, device,
                 dtype: torch.dtype, alloc=None):
        self.cfg, self.num_blocks, self.block_size, self.num_slots = cfg, num_blocks, block_size, num_slots
        es = 4 if dtype == torch.float32 else 2
        plan, off = [], 0

        def take(nbytes: int) -> int:
            nonlocal off
            at = off
            off = (off + nbytes + 255) // 256 * 256
            return at
        for i, (li, _) in enumerate(cfg.runs):
            l = cfg.layers[li]
            if l.owns_kv:
                plan.append(("k", i, take(num_blocks * l.kv_heads * block_size * l.dim * es)))
                if not (l.values_are_keys and l.rot_dims == 0):      # (un-rotated keys that are the values: one plane)
                    plan.append(("v", i, take(num_blocks * l.kv_heads * block_size * l.vdim * es)))
            elif l.owns_latent:
                plan.append(("c", i, take(num_blocks * block_size * (l.kv_rank + l.rot_dim) * es)))
            elif l.state_size():
                plan.append(("s", i, take(max(1, num_slots) * l.state_size() * 4)))
        total = max(off, 256)
        if alloc is None:
            self.pool = torch.zeros(total // 2, dtype=torch.bfloat16, device=device)
        else:
            self.pool = alloc(total // 2)
            ops.zero_(self.pool)
        raw = self.pool.view(torch.uint8)
        self._k: Dict[int, torch.Tensor] = {}
        self._v: Dict[int, torch.Tensor] = {}
        self._s: Dict[int, torch.Tensor] = {}
        for kind, i, at in plan:
            l = cfg.layers[cfg.runs[i][0]]
            if kind == "k":
                n = num_blocks * l.kv_heads * block_size * l.dim * es
                self._k[i] = raw[at:at + n].view(dtype).view(num_blocks, l.kv_heads, block_size, l.dim)
                if l.values_are_keys and l.rot_dims == 0:
                    self._v[i] = self._k[i]
            elif kind == "v":
                n = num_blocks * l.kv_heads * block_size * l.vdim * es
                self._v[i] = raw[at:at + n].view(dtype).view(num_blocks, l.kv_heads, block_size, l.vdim)
            elif kind == "c":
                w = l.kv_rank + l.rot_dim
                n = num_blocks * block_size * w * es
                self._k[i] = raw[at:at + n].view(dtype).view(num_blocks, 1, block_size, w)
                self._v[i] = self._k[i][..., :l.kv_rank]     # (the compressed row: the first columns of the same rows)
            else:
                n = max(1, num_slots) * l.state_size() * 4
                self._s[i] = raw[at:at + n].view(torch.float32).view(max(1, num_slots), l.state_size())

    def k(self, run: int) -> torch.Tensor:
        return self._k[run]

    def v(self, run: int) -> torch.Tensor:
        return self._v[run]

    def state(self, run: int) -> torch.Tensor:
        return self._s[run]

    def copy_blocks(self, src: torch.Tensor, dst: torch.Tensor) -> None:
        # sequences with a state slot are never forked (csrc/core/kv_manager.cpp), so no block is
        # ever shared and copied on write
        raise NotImplementedError("hybrid decoders serve one chain per request: no copy-on-write")

    @staticmethod
    def bytes_per_block(cfg: HybridConfig, block_size: int, dtype: torch.dtype) -> int:
        return max(1, cfg.kv_elems_per_token() * block_size * (4 if dtype == torch.float32 else 2))


@dataclass
class DyT:
    """A Dynamic Tanh norm: tanh(alpha x) * w + b."""

    alpha: float
    w: torch.Tensor                                 # fp32 [d]
    b: torch.Tensor                                 # fp32 [d]


@dataclass
class HybridLayer:
    spec: LayerSpec
    norm1: object                                   # fp32 [1] | fp32 [d] | DyT
    proj: ops.LinearWeight                          # fused input projections of the mixer
    out: ops.LinearWeight
    norm2: object = None
    up: Optional[ops.LinearWeight] = None
    down: Optional[ops.LinearWeight] = None
    q_norm: Optional[torch.Tensor] = None           # fp32 [H*D]
    k_norm: Optional[torch.Tensor] = None
    inv_freq: Optional[torch.Tensor] = None         # fp32 [rot_dims/2] (fp64 for neighbouring pairs)
    decay_up: Optional[ops.LinearWeight] = None     # gla: bottleneck -> decay logits
    head_norm: Optional[torch.Tensor] = None        # gla: fp32 [vdim]; mlstm: fp32 [H*vdim]
    gate_up: Optional[ops.LinearWeight] = None      # gated dense feed-forward: gate | up
    latent_norm: Optional[torch.Tensor] = None      # latent attention: fp32 [kv_rank]
    key_up_t: Optional[torch.Tensor] = None         # latent attention: [H, kv_rank, dim], head h's key map transposed
    value_up: Optional[torch.Tensor] = None         # latent attention: [H, vdim, kv_rank]
    router: Optional[ops.LinearWeight] = None       # routed feed-forward: [experts + identity, d]
    correction: Optional[torch.Tensor] = None       # fp32 [experts + identity]
    experts_up: object = None                       # [E, ff, d] ([E, 2 ff, d] = gate | up of clamped gated experts) row-major, or ops.ExpertWeights (packed for the MFMA kernels)
    experts_down: object = None                     # [E, d, ff]
    shared_up: Optional[ops.LinearWeight] = None
    shared_down: Optional[ops.LinearWeight] = None
    inv_freq_v: Optional[torch.Tensor] = None       # attention whose values turn: fp64 [vdim/2]
    talk: Optional[torch.Tensor] = None             # fp32 [H, H]: new head h's weights = sum_g talk[h, g] head g's
    act: Optional[Tuple[float, float]] = None       # xIELU: (softplus(p), 1/2 + softplus(q))
    hc1: Optional["StreamWeights"] = None           # parallel residual streams: the mixer's read / write weights
    hc2: Optional["StreamWeights"] = None           # the feed-forward's


@dataclass
class StreamWeights:
    """How one sublayer reads S parallel residual streams (``read`` [S]) and writes them (``mix`` [S, S] from -> to,
    ``write`` [S] shares of its result), fp32."""

    read: torch.Tensor
    write: torch.Tensor
    mix: torch.Tensor


class HybridModel:
    """One model of a hybrid design on one device. Same surface as ``TransformerModel`` towards the engine:
    ``forward`` (the residual stream of the step's rows), ``logits``, ``make_cache``."""

    tp_rank, tp_size, ep_size, comm = 0, 1, 1, None
    supports_embed = False          # pooled embeddings read bf16 final-normed rows; this stream is fp32
    wants_layout = True

    def __init__(self, cfg: HybridConfig, device, dtype: torch.dtype = torch.bfloat16) -> None:
        cfg.validate()
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"{cfg.name}: activation type {dtype}: bf16 or fp32")
        self.cfg, self.device, self.dtype = cfg, torch.device(device), dtype
        self.hq, self.hkv = cfg.num_heads, cfg.num_kv_heads
        self.embed: Optional[torch.Tensor] = None
        self.final_norm: Optional[torch.Tensor] = None
        self.lm_head: Optional[ops.LinearWeight] = None
        self.loop_in: Optional[ops.LinearWeight] = None     # [d, 2 d]: the stream's re-injection before every pass of a loop
        self.embed_norm: Optional[torch.Tensor] = None      # fp32 [d]: norm weight on the embedding rows
        self.stream_sum: Optional[torch.Tensor] = None      # fp32 [S] of ones: the model's output reads every stream once
        self.layers: List[HybridLayer] = []
        self._rows: Dict[int, Tuple[torch.Tensor, torch.Tensor]] = {}
        self._max_len = 1
        self._portions = (0, 0)
        self.pos_freq: Optional[torch.Tensor] = None    # fp64 [d/2]: frequencies of the sinusoidal position vector
        if cfg.design.pos_base > 0:
            half = cfg.hidden_size // 2
            f = torch.tensor([cfg.design.pos_base ** (-2.0 * j / cfg.hidden_size) for j in range(half)], dtype=torch.float64)
            self.pos_freq = f.to(self.device)

    # ------------------------------------------------------------------ construction
    def set_weights(self, get) -> None:
        """``get(name) -> tensor`` with the checkpoint's names. Shapes are checked against the
        configuration, by name, before anything is fused or packed."""
        c, dev, dt = self.cfg, self.device, self.dtype
        shapes = param_shapes(c)

        def load(name: str) -> torch.Tensor:
            t = get(name)
            t = t.to(torch.float32) if hasattr(t, "to") else torch.as_tensor(t, dtype=torch.float32)
            if tuple(t.shape) != tuple(shapes[name]):
                raise ValueError(f"{c.name}: tensor {name!r} has shape {tuple(t.shape)}, the configuration implies "
                                 f"{tuple(shapes[name])}")
            return t.to(dev)

        def lin(W: torch.Tensor, b: Optional[torch.Tensor] = None, pad: bool = False) -> ops.LinearWeight:
            # ``pad``: zero rows up to a multiple of 32 outputs, for fused projections whose consumers
            # address their columns anyway (products that split their depth reduce whole groups of 32 columns)
            extra = -W.shape[0] % 32 if pad else 0
            if extra:
                W = torch.cat([W, W.new_zeros(extra, W.shape[1])], 0)
                b = torch.cat([b, b.new_zeros(extra)], 0) if b is not None else None
            return ops.LinearWeight.from_dense(W, b, dev, dtype=dt, any_shape=True)

        def f32(t: torch.Tensor) -> torch.Tensor:
            return t.to(torch.float32).reshape(-1).contiguous()

        def norm_w(name: str, scale: float = 1.0):
            if c.design.norm == "dyt":
                return DyT(float(load(name + ".alpha").item()), (f32(load(name)) * scale).contiguous(),
                           (f32(load(name + ".b")) * scale).contiguous())
            # stored as an offset from the design's base value; the kernels multiply by the sum
            return ((f32(load(name)) + c.design.norm_offset) * scale).contiguous()
        self.embed = load("embed").to(dt).contiguous()
        # the logits' scale rides on the final norm's weight
        self.final_norm = norm_w("final.norm", c.logit_scale) if c.design.pre_norm else f32(load("final.norm"))
        # (a tied head is the embedding table once more, in the layout of the matrix products)
        self.lm_head = lin(load("embed" if c.design.tied_head else "head"))
        self.loop_in = lin(load("loop.in")) if c.looped else None
        self.embed_norm = f32(load("embed.norm")) if c.design.embed_norm else None
        self.stream_sum = torch.ones(c.streams, dtype=torch.float32, device=dev) if c.design.hyper else None

        def inv_freqs(base: float, dims: int) -> torch.Tensor:
            return torch.tensor([base ** (-2.0 * j / dims) for j in range(dims // 2)], dtype=torch.float64).to(dev)
        self.layers = []
        for i, l in enumerate(c.layers):
            p, m = f"l{i}.", f"l{i}.mix."
            kw = {}
            if c.design.hyper:
                for q in ("hc1", "hc2") if l.has_ff else ("hc1",):
                    kw[q] = StreamWeights(f32(load(p + q + ".in")), f32(load(p + q + ".out")), f32(load(p + q + ".mix")))
            if l.type == "attention" and l.talk:
                if l.rot_dims:
                    kw["inv_freq"] = inv_freqs(l.rot_base, l.rot_dims)
                if l.rotate_values:
                    kw["inv_freq_v"] = inv_freqs(l.rot_base, l.vdim)
                kw["talk"] = f32(load(m + "talk"))
                proj = lin(torch.cat([load(m + n) for n in ("q", "k", "v")], 0),
                           torch.cat([load(m + n + ".b") for n in ("q", "k", "v")], 0), pad=True)
                out = lin(load(m + "o"))
            elif l.type == "latent_attention" and l.gate_full:
                # queries (head by head: plain | turned part) | compressed row | shared key part | a gate logit per output
                names = ("q", "dkv", "g") if l.owns_latent else ("q", "g")
                proj = lin(torch.cat([load(m + n) for n in names], 0), pad=True)
                if l.owns_latent:
                    kw["latent_norm"] = f32(load(m + "dkv.norm"))
                if l.rot_dim:
                    kw["inv_freq"] = inv_freqs(l.rot_base, l.rot_dim)
                kw["key_up_t"] = load(m + "uk").view(l.heads, l.dim, l.kv_rank).transpose(1, 2).to(dt).contiguous()
                kw["value_up"] = load(m + "uv").view(l.heads, l.vdim, l.kv_rank).to(dt).contiguous()
                out = lin(load(m + "o"))
            elif l.type == "attention" and l.values_are_keys:
                half = l.rot_dims // 2
                if half:
                    kw["inv_freq"] = torch.tensor([l.rot_base ** (-2.0 * j / l.rot_dims) for j in range(half)],
                                                  dtype=torch.float64).to(dev)
                proj, out = lin(torch.cat([load(m + "q"), load(m + "k")], 0), pad=True), lin(load(m + "o"))
            elif l.type == "attention":
                Ws, bs = [load(m + "q")], [load(m + "q.b")]
                if l.owns_kv:
                    Ws += [load(m + "k"), load(m + "v")]
                    bs += [load(m + "k.b"), load(m + "v.b")]
                    kw["k_norm"] = f32(load(m + "k.norm"))
                kw["q_norm"] = f32(load(m + "q.norm"))
                half = l.rot_dims // 2
                inv = torch.tensor([l.rot_base ** (-2.0 * j / l.rot_dims) for j in range(half)] or [0.0],
                                   dtype=torch.float64)
                kw["inv_freq"] = inv.to(torch.float32).to(dev)
                proj, out = lin(torch.cat(Ws, 0), torch.cat(bs, 0)), lin(load(m + "o"), load(m + "o.b"))
            elif l.type == "mingru":
                bias = torch.cat([load(m + "z.b"), load(m + "x.b"), torch.zeros(l.width, device=dev)])
                proj = lin(torch.cat([load(m + "z"), load(m + "x"), load(m + "g")], 0), bias)
                out = lin(load(m + "o"))
            elif l.type == "gla":
                proj = lin(torch.cat([load(m + n) for n in ("q", "k", "v", "g", "a1")], 0))
                # the bottleneck's output is an fp32 column slice of the fused projection: the small
                # second product takes it as it is through the shape-agnostic kernel
                kw["decay_up"] = ops.LinearWeight.from_dense(load(m + "a2"), load(m + "a2.b"), dev, dtype=dt, plain=True)
                kw["head_norm"] = f32(load(m + "norm"))
                out = lin(load(m + "o"))
            elif l.type == "latent_attention":
                # queries | compressed row | one gate logit per head, in one product
                proj = lin(torch.cat([load(m + n) for n in ("q", "dkv", "g")], 0), pad=True)
                kw["latent_norm"] = f32(load(m + "dkv.norm"))
                kw["key_up_t"] = load(m + "uk").view(l.heads, l.dim, l.kv_rank).transpose(1, 2).to(dt).contiguous()
                kw["value_up"] = load(m + "uv").view(l.heads, l.vdim, l.kv_rank).to(dt).contiguous()
                out = lin(load(m + "o"))
            else:
                hd, hv = l.heads * l.dim, l.heads * l.vdim
                bias = torch.cat([torch.zeros(2 * hd + 2 * hv, device=dev), load(m + "i.b"), load(m + "f.b")])
                proj = lin(torch.cat([load(m + n) for n in ("q", "k", "v", "g", "i", "f")], 0), bias, pad=True)
                kw["head_norm"] = f32(load(m + "norm"))
                out = lin(load(m + "o"))
            f = p + "mlp."
            if l.moe is not None and l.moe.clamped:
                e = l.moe
                # one product for the router's logits (32-bit: fp32 accumulation of the operands) and, when there is a
                # shared expert, its gate | up units and its gate logit: gate | up | router | sg
                rows = [load(f + "router")]
                if e.shared_ff:
                    rows = [load(f + "shared.gate"), load(f + "shared.up")] + rows + [load(f + "shared.sg")]
                    kw["shared_down"] = lin(load(f + "shared.down"))
                kw["router"] = lin(torch.cat(rows, 0), pad=True)
                ups = torch.stack([torch.cat([load(f + f"e{j}.gate"), load(f + f"e{j}.up")], 0) for j in range(e.experts)])
                downs = torch.stack([load(f + f"e{j}.down") for j in range(e.experts)])
                if dt == torch.bfloat16 and c.hidden_size % 64 == 0 and e.ff % 64 == 0 and dev.type == "cuda":
                    # depths the MFMA kernels take: fragment order per expert, 16-row tiles alternating gate / up so
                    # that the gated unit is the product's epilogue
                    ups = torch.stack([ops.interleave_gate_up(load(f + f"e{j}.gate"), load(f + f"e{j}.up")) for j in range(e.experts)])
                    kw["experts_up"] = ops.ExpertWeights.from_dense(ups, dev, swiglu=True)
                    kw["experts_down"] = ops.ExpertWeights.from_dense(downs, dev)
                else:
                    kw["experts_up"], kw["experts_down"] = ups.to(dt).contiguous(), downs.to(dt).contiguous()
            elif l.moe is not None:
                e = l.moe
                # bf16 operands with fp32 accumulation give the router's logits in 32-bit either way
                # (and they ride behind the shared expert's up projection, one product for both, if there is one)
                if e.shared_ff:
                    kw.update(shared_up=lin(torch.cat([load(f + "shared.up"), load(f + "router")], 0), pad=True),
                              shared_down=lin(load(f + "shared.down")))
                else:
                    kw["router"] = lin(load(f + "router"))
                kw["correction"] = f32(load(f + "correction"))
                ups = torch.stack([load(f + f"e{j}.up") for j in range(e.experts)])
                downs = torch.stack([load(f + f"e{j}.down") for j in range(e.experts)])
                if dt == torch.bfloat16 and c.hidden_size % 64 == 0 and e.ff % 64 == 0:
                    # depths the MFMA kernels take: MFMA fragment order per expert
                    kw["experts_up"] = ops.ExpertWeights.from_dense(ups, dev)
                    kw["experts_down"] = ops.ExpertWeights.from_dense(downs, dev)
                else:
                    kw["experts_up"], kw["experts_down"] = ups.to(dt).contiguous(), downs.to(dt).contiguous()
            elif l.ff and c.design.dense_ff == "xielu":
                a = load(f + "act").double().cpu()
                sp = torch.nn.functional.softplus(a)
                kw.update(up=lin(load(f + "up"), load(f + "up.b")), down=lin(load(f + "down"), load(f + "down.b")),
                          act=(float(sp[0]), 0.5 + float(sp[1])))
            elif l.ff:
                if c.design.dense_ff == "glu_relu":
                    kw["gate_up"] = lin(torch.cat([load(f + "gate"), load(f + "up")], 0))
                else:
                    kw["up"] = lin(load(f + "up"))
                kw["down"] = lin(load(f + "down"))
            if c.design.pre_norm:
                n1 = norm_w(p + "norm1")
                if l.has_ff:
                    kw["norm2"] = norm_w(p + "norm2")
            else:
                n1 = f32(load(p + "norm1"))
                if l.has_ff:
                    kw["norm2"] = f32(load(p + "norm2"))
            self.layers.append(HybridLayer(l, n1, proj, out, **kw))

    @classmethod
    def random_init(cls, cfg: HybridConfig, device, seed: int = 0, dtype: torch.dtype = torch.bfloat16,
                    **_ignored) -> "HybridModel":
        """Random weights of the configured shapes (benchmarks, smoke tests): N(0, 1/fan_in)
        matrices, small biases, gains near one, decay biases that keep the states alive."""
        m = cls(cfg, device, dtype)
        shapes = param_shapes(cfg)
        gen = torch.Generator()

        def get(name: str) -> torch.Tensor:
            shape = shapes[name]
            gen.manual_seed((seed * 1000003 + zlib.crc32(name.encode())) & 0x7FFFFFFFFFFFFFFF)
            offset_norm = cfg.design.norm_offset != 0.0 and name.split(".")[-1] in ("norm1", "norm2") or \
                (cfg.design.norm_offset != 0.0 and name == "final.norm")
            if ".hc" in name:                                    # streams that neither die out nor blow up
                n = cfg.streams
                t = {"in": torch.full(shape, 1.0 / n), "out": torch.ones(shape), "mix": torch.eye(n)}[name.split(".")[-1]]
                t = t + 0.05 * torch.randn(shape, generator=gen)
            elif name.endswith("mix.talk"):
                t = torch.eye(shape[0]) + 0.1 * torch.randn(shape, generator=gen)
            elif name.endswith(".alpha"):
                t = 0.6 + 0.1 * torch.randn(shape, generator=gen)
            elif len(shape) == 2:
                scale = cfg.hidden_size ** -0.5 if cfg.design.tied_head else 1.0     # (the table is the head too)
                t = torch.randn(shape, generator=gen) * (scale if name == "embed" else shape[1] ** -0.5)
            elif offset_norm:
                t = 0.1 * torch.randn(shape, generator=gen)
            elif name.endswith("norm") or name.endswith("norm1") or name.endswith("norm2"):
                t = 1.0 + 0.1 * torch.randn(shape, generator=gen)
            elif name.endswith("a2.b") or name.endswith("mix.f.b"):
                t = 2.0 + torch.randn(shape, generator=gen)
            elif name.endswith("correction"):
                t = 0.02 * torch.randn(shape, generator=gen)
            else:
                t = 0.1 * torch.randn(shape, generator=gen)
            return t.to(torch.bfloat16)
        m.set_weights(get)
        return m

    def weight_bytes(self) -> int:
        n = self.embed.numel() * self.embed.element_size() + self.lm_head.nbytes()
        n += self.loop_in.nbytes() if self.loop_in is not None else 0
        for L in self.layers:
            for w in (L.proj, L.out, L.up, L.down, L.decay_up, L.gate_up, L.router, L.shared_up, L.shared_down):
                n += w.nbytes() if w is not None else 0
            for t in (L.key_up_t, L.value_up, L.experts_up, L.experts_down, L.talk):
                t = t.data if isinstance(t, ops.ExpertWeights) else t
                n += t.numel() * t.element_size() if t is not None else 0
        return n

    # ------------------------------------------------------------------ engine surface
    def make_cache(self, num_blocks: int, block_size: int, num_slots: int, alloc=None) -> HybridCache:
        return HybridCache(self.cfg, num_blocks, block_size, num_slots, self.device, self.dtype, alloc)

    def cache_bytes_per_block(self, block_size: int) -> int:
        return HybridCache.bytes_per_block(self.cfg, block_size, self.dtype)

    def state_slots_needed(self, max_seqs: int) -> int:
        return max_seqs if self.cfg.has_state else 0

    def decode_capturable(self, rows: int) -> bool:
        return True

    def _decode_layout(self, meta, B: int) -> StepLayout:
        """A pure decode step described the old way (one row per sequence): rows are sequences."""
        e = self._rows.get(B)
        if e is None:
            e = (torch.arange(B + 1, dtype=torch.int32, device=self.device),
                 torch.arange(B, dtype=torch.int32, device=self.device))
            self._rows[B] = e
        return StepLayout(e[0], e[1], meta.block_tables, None)

    # ------------------------------------------------------------------ forward
    def forward(self, token_ids: torch.Tensor, positions: torch.Tensor, slot_mapping: torch.Tensor, meta,
                cache: HybridCache, taps: Optional[list] = None) -> torch.Tensor:
        """The fp32 residual stream [T, d] after the last layer for the step's rows (``logits``
        applies the final norm). ``taps`` (a list) receives a copy of the stream after every layer."""
        c, dt, eps = self.cfg, self.dtype, self.cfg.rms_eps
        lay: StepLayout = getattr(meta, "layout", None) or self._decode_layout(meta, token_ids.numel())
        if c.has_state and lay.state_slots is None:
            raise ValueError(f"{c.name}: the step names no state slots (the engine's KV manager must be made with slots)")
        # the longest portion of the step: long ones are scanned in parallel segments
        self._max_len = max(1, int(meta.max_q_len)) if meta.is_prefill else 1
        # prompt portions come first (sequences and rows), single decoded tokens ride behind them
        T = token_ids.numel()
        self._portions = (meta.block_tables.shape[0], meta.prefill_tokens if meta.riders is not None else T) \
            if meta.is_prefill else (0, 0)
        if c.design.hyper:
            return self._forward_streams(token_ids, positions, slot_mapping, meta, lay, cache, taps)
        if c.design.pre_norm:
            return self._forward_pre_norm(token_ids, positions, slot_mapping, meta, lay, cache, taps)
        x, xa = ops.embed_rows(token_ids, self.embed, dt, meta.token_feed)
        for i, L in enumerate(self.layers):
            l = L.spec
            if l.type == "attention":
                y = self._attention(i, L, xa, positions, slot_mapping, lay, cache)
            elif l.type == "mingru":
                zxg = ops.linear(xa, L.proj, out_f32=True)
                y = ops.mingru_scan(zxg, cache.state(i), lay.cu_q, positions, lay.state_slots, dt, self._max_len)
                y = ops.linear(y, L.out, out_f32=True)
            else:
                y = self._gla(i, L, xa, positions, lay, cache)
            xa = ops.scalar_norm_add(x, y, L.norm1, eps, dt)
            if L.up is not None:
                xa = ops.scalar_norm_add(x, ops.linear(self._relu2_up(xa, L.up), L.down, out_f32=True), L.norm2, eps, dt)
            if taps is not None:
                taps.append(x.clone())
        return x

    def _relu2_up(self, xa: torch.Tensor, up: ops.LinearWeight) -> torch.Tensor:
        """relu(up x)^2 in the activation type: an epilogue of the shape-agnostic product, one more
        launch behind the packed MFMA product."""
        if up.is_packed or not xa.is_cuda:
            return ops.relu2(ops.linear(xa, up, out_f32=True), self.dtype)
        return ops.linear_any(xa, up, out_f32=self.dtype == torch.float32, epi_relu2=True)

    def _forward_pre_norm(self, token_ids, positions, slot_mapping, meta, lay: StepLayout, cache: HybridCache,
                          taps: Optional[list]) -> torch.Tensor:
        """Layers whose sublayers read the normed stream: every residual sum and the norm that feeds
        the next sublayer are one launch (``_residual_norm``). The layer runs come from the
        configuration's loop; a run that starts a pass replaces the stream by ``W_in [x; x0]``, whose input
        the residual step in front of it writes straight into the left half of a [T, 2 d] matrix (the
        right half holds the embedding output, written once per step)."""
        c, dt = self.cfg, self.dtype
        x, _ = ops.embed_rows(token_ids, self.embed, None, meta.token_feed, c.embed_scale,
                              positions if self.pos_freq is not None else None, self.pos_freq)
        runs, d = c.runs, c.hidden_size
        both = None
        if c.looped:
            both = torch.empty(x.shape[0], 2 * d, dtype=dt, device=x.device)
            ops.add_dyt(x, None, 1.0, 1.0, None, None, dt, out=both[:, d:])
            if runs[0][1]:
                ops.add_dyt(x, None, 1.0, 1.0, None, None, dt, out=both[:, :d])
        xa = None if runs[0][1] else self._residual_norm(x, None, self.layers[runs[0][0]].norm1)
        for r, (i, inject) in enumerate(runs):
            L = self.layers[i]
            l = L.spec
            if inject:
                x = ops.linear(both, self.loop_in, out_f32=True)
                xa = self._residual_norm(x, None, L.norm1)
            if l.type == "latent_attention":
                y = self._latent_attention(r, L, xa, positions, slot_mapping, lay, cache)
            elif l.type == "mlstm":
                y = self._mlstm(r, L, xa, positions, lay, cache)
            else:
                y = self._attention_kv(r, L, xa, positions, slot_mapping, lay, cache)
            if l.has_ff:
                xa = self._residual_norm(x, y, L.norm2)
                if l.moe is None:
                    y = self._dense_ff(L, xa)
                else:
                    y = self._clamped_ff(L, xa) if l.moe.clamped else self._routed_ff(L, xa)
            if r + 1 == len(runs):
                self._residual_norm(x, y, None)
            elif runs[r + 1][1]:
                self._residual_norm(x, y, None, out=both[:, :d])
            else:
                xa = self._residual_norm(x, y, self.layers[runs[r + 1][0]].norm1)
            if taps is not None:
                taps.append(x.clone())
        return x

    def _forward_streams(self, token_ids, positions, slot_mapping, meta, lay: StepLayout, cache: HybridCache,
                         taps: Optional[list]) -> torch.Tensor:
        """Layers around a residual of S parallel streams (fp32 [T, S, d]). One launch sits between two sublayers:
        it writes the first one's result into the streams (every new stream a mixture of the old ones plus its
        share), forms the second one's input from the new streams and norms it. The last launch of the step
        returns the sum of the streams, which is what ``logits`` norms."""
        c, dt, eps = self.cfg, self.dtype, self.cfg.rms_eps
        x0, _ = ops.embed_rows(token_ids, self.embed, None, meta.token_feed)
        xs = ops.hc_init(x0, self.embed_norm, eps, c.streams)
        runs = c.runs
        first = self.layers[runs[0][0]]
        xa = ops.hc_step(xs, None, None, None, first.hc1.read, first.norm1, eps, dt)
        x = None
        for r, (i, _) in enumerate(runs):
            L = self.layers[i]
            l, hc = L.spec, L.hc1
            if l.type == "latent_attention":
                y = self._latent_attention_rot(r, L, xa, positions, slot_mapping, lay, cache)
            else:
                y = self._attention_talk(r, L, xa, positions, slot_mapping, lay, cache)
            if l.has_ff:
                xa = ops.hc_step(xs, y, hc.mix, hc.write, L.hc2.read, L.norm2, eps, dt)
                y, hc = self._dense_ff(L, xa), L.hc2
            if r + 1 == len(runs):
                x = ops.hc_step(xs, y, hc.mix, hc.write, self.stream_sum, None, eps, None)
            else:
                nxt = self.layers[runs[r + 1][0]]
                xa = ops.hc_step(xs, y, hc.mix, hc.write, nxt.hc1.read, nxt.norm1, eps, dt)
            if taps is not None:
                taps.append(x.clone() if x is not None else ops.hc_step(xs, None, None, None, self.stream_sum, None, eps, None))
        return x

    def _residual_norm(self, x: torch.Tensor, y: Optional[torch.Tensor], norm, out: Optional[torch.Tensor] = None):
        """x += m * y (when y is given) and the design's norm of the new x in the activation type (when a
        norm is given; with ``out`` and no norm: the stream itself, cast, into that column block)."""
        c = self.cfg
        if c.design.norm == "dyt":
            if norm is None:
                return ops.add_dyt(x, y, c.residual_mult, 1.0, None, None, None, out=out)
            return ops.add_dyt(x, y, c.residual_mult, norm.alpha, norm.w, norm.b, self.dtype, out=out)
        xa = ops.add_rmsnorm(x, y, norm, c.rms_eps, self.dtype)
        if out is not None:                 # the start of a loop's pass: the stream itself, cast
            ops.add_dyt(x, None, 1.0, 1.0, None, None, None, out=out)
        return xa

    def _dense_ff(self, L: HybridLayer, xa: torch.Tensor) -> torch.Tensor:
        if L.act is not None:               # (biases ride in the products)
            return ops.linear(ops.xielu(ops.linear(xa, L.up, out_f32=True), L.act[0], L.act[1], self.dtype), L.down, out_f32=True)
        if L.gate_up is not None:
            return ops.linear(ops.glu(ops.linear(xa, L.gate_up, out_f32=True), self.dtype, "relu"), L.down, out_f32=True)
        return ops.linear(self._relu2_up(xa, L.up), L.down, out_f32=True)

    def _routed_ff(self, L: HybridLayer, xa: torch.Tensor) -> torch.Tensor:
        e = L.spec.moe
        shared = None
        if L.shared_up is not None:
            su = ops.linear(xa, L.shared_up, out_f32=True)          # shared expert's hidden units | router logits
            z = su[:, e.shared_ff:e.shared_ff + e.outputs]
            shared = ops.linear(ops.relu2(su[:, :e.shared_ff], self.dtype), L.shared_down, out_f32=True)
        else:
            z = ops.linear(xa, L.router, out_f32=True)
        ids, wts = ops.route_grouped(z, L.correction, e.top, e.groups, e.keep, e.scale)
        offsets, sorted_src, slot_of = ops.moe_sort(ids, e.outputs)
        rows = ids.numel()
        act = ops.grouped_linear(xa, sorted_src, offsets, L.experts_up, self.dtype, rows, relu2_epi=True)
        ye = ops.grouped_linear(act, None, offsets, L.experts_down, torch.float32, rows)
        return ops.moe_mix(ye, slot_of, ids, wts, xa, e.experts, shared)

    def _clamped_ff(self, L: HybridLayer, xa: torch.Tensor) -> torch.Tensor:
        """Routed feed-forward with sigmoid scores whose weight multiplies the expert's INPUT. The products are
        linear up to the clamps, so the expert's gate | up product runs on the un-weighted rows and the weight
        scales its fp32 result in the launch that clamps and gates it."""
        e, des = L.spec.moe, self.cfg.design
        sf = e.shared_ff
        su = ops.linear(xa, L.router, out_f32=True)                 # (shared gate | shared up |) router logits (| shared gate logit)
        z = su[:, 2 * sf:2 * sf + e.experts]
        shared = gate = None
        if sf:
            act = ops.glu_clamped(su, 0, sf, sf, e.shared_limit, self.dtype, slope=des.glu_slope, shift=des.glu_shift)
            shared = ops.linear(act, L.shared_down, out_f32=True)
            gate = su[:, 2 * sf + e.experts:2 * sf + e.experts + 1]
        ids, wts = ops.route_grouped(z, None, e.top, 1, 1, 1.0, score="sigmoid")
        rows = ids.numel()
        if isinstance(L.experts_up, ops.ExpertWeights):     # (bf16, MFMA depths: the gated unit is the product's epilogue)
            offsets, sorted_src, slot_of, sorted_wts = ops.moe_sort(ids, e.experts, wts)
            act = ops.grouped_linear(xa, sorted_src, offsets, L.experts_up, self.dtype, rows,
                                     glu_clamp=(sorted_wts, e.limit, des.glu_slope, des.glu_shift))
        else:
            offsets, sorted_src, slot_of = ops.moe_sort(ids, e.experts)
            gu = ops.grouped_linear(xa, sorted_src, offsets, L.experts_up, torch.float32, rows)
            act = ops.glu_clamped(gu, 0, e.ff, e.ff, e.limit, self.dtype, slot_of=slot_of.view(-1), wts=wts.view(-1),
                                  slope=des.glu_slope, shift=des.glu_shift)
        ye = ops.grouped_linear(act, None, offsets, L.experts_down, torch.float32, rows)
        return ops.moe_mix(ye, slot_of, ids, None, xa, e.experts, shared, gate)

    def _attention_kv(self, r: int, L: HybridLayer, xa, positions, slot_mapping, lay: StepLayout, cache: HybridCache):
        """Attention whose values are its un-rotated keys, under a sliding window."""
        l = L.spec
        kc = cache.k(r)
        vc = cache.v(r) if l.rot_dims else None
        qk = ops.linear(xa, L.proj, out_f32=True)
        q = ops.rope_pairs_write(qk, L.inv_freq, positions, slot_mapping, kc, vc, l.heads, l.kv_heads, l.dim, l.rot_dims)
        a = ops.attn_masked(q, kc, cache.v(r), lay.block_tables, lay.cu_q, lay.row_seq, positions, l.heads, l.kv_heads, l.dim,
                            l.vdim, l.scale, 0, l.window, self.dtype, n_portions=self._portions[0],
                            portion_rows=self._portions[1], max_len=self._max_len)
        return ops.linear(a, L.out, out_f32=True)

    def _attention_talk(self, r: int, L: HybridLayer, xa, positions, slot_mapping, lay: StepLayout, cache: HybridCache):
        """Attention whose heads' softmax weights are mixed before they meet the values. The mix is linear in the
        weights, so it is applied behind the weighted sums: the attention kernels give every head's weights on the
        values of EVERY key/value head (fp32), and one launch mixes those sums per head and turns the result back
        by the row's position (the values were cached turned by their own)."""
        l = L.spec
        kc, vc = cache.k(r), cache.v(r)
        qkv = ops.linear(xa, L.proj, out_f32=True)
        q = ops.rope_qkv_write(qkv, L.inv_freq, L.inv_freq_v, positions, slot_mapping, kc, vc, l.heads, l.kv_heads, l.dim,
                               l.vdim, l.rot_dims)
        o = ops.attn_masked(q, kc, vc, lay.block_tables, lay.cu_q, lay.row_seq, positions, l.heads, l.kv_heads, l.dim, l.vdim,
                            l.scale, 0, l.window, torch.float32, n_portions=self._portions[0], portion_rows=self._portions[1],
                            max_len=self._max_len, softcap=l.softcap, sink=l.sink, all_value_heads=True)
        a = ops.talk_mix(o, L.talk, positions, L.inv_freq_v, l.heads, l.kv_heads, l.vdim, self.dtype)
        return ops.linear(a, L.out, out_f32=True)

    def _latent_attention_rot(self, r: int, L: HybridLayer, xa, positions, slot_mapping, lay: StepLayout, cache: HybridCache):
        """Latent attention with a turned key part shared by all heads. The cached row is [compressed row | key part];
        the query of head h in the same coordinates is [U_h^T q_plain | turned q part], so that one dot product with
        the cached row is the head's score; the values are the first kv_rank columns of the same rows."""
        l = L.spec
        H, D, rd, R, Dv = l.heads, l.dim, l.rot_dim, l.kv_rank, l.vdim
        nq, W = H * (D + rd), R + rd
        own = l.owns_latent
        cc = cache.k(r if own else l.kv_from)
        proj = ops.linear(xa, L.proj, out_f32=True)                 # q | (compressed row | key part) | gate logits
        qlat = torch.empty(proj.shape[0], H * W, dtype=torch.float32, device=proj.device)
        ops.latent_rope_write(proj, nq, L.latent_norm, self.cfg.rms_eps, L.inv_freq, positions, slot_mapping,
                              cc if own else None, qlat, H, D, R, rd)
        ops.head_linear(proj, L.key_up_t, torch.float32, x_head_stride=D + rd, out=qlat, out_head_stride=W)
        a = ops.attn_masked(qlat, cc, cc[..., :R], lay.block_tables, lay.cu_q, lay.row_seq, positions, H, 1, W, R, l.scale,
                            0, l.window, torch.float32, n_portions=self._portions[0], portion_rows=self._portions[1],
                            max_len=self._max_len)
        g0 = nq + (W if own else 0)
        o = ops.head_linear(a, L.value_up, self.dtype, gate=proj[:, g0:g0 + H * Dv], gate_full=True)
        return ops.linear(o, L.out, out_f32=True)

    def _latent_attention(self, i: int, L: HybridLayer, xa, positions, slot_mapping, lay: StepLayout, cache: HybridCache):
        l = L.spec
        hd, R = l.heads * l.dim, l.kv_rank
        proj = ops.linear(xa, L.proj, out_f32=True)                 # q | compressed row | gate logits
        cc = cache.k(i)
        ops.latent_write(proj, hd, L.latent_norm, self.cfg.rms_eps, slot_mapping, cc)
        q = ops.head_linear(proj[:, :hd], L.key_up_t, torch.float32)        # queries in the latent's coordinates
        a = ops.attn_masked(q, cc, cc, lay.block_tables, lay.cu_q, lay.row_seq, positions, l.heads, 1, R, R, l.scale,
                            0, 0, self.dtype, n_portions=self._portions[0], portion_rows=self._portions[1],
                            max_len=self._max_len)
        o = ops.head_linear(a, L.value_up, self.dtype, gate=proj[:, hd + R:hd + R + l.heads])
        return ops.linear(o, L.out, out_f32=True)

    def _mlstm(self, i: int, L: HybridLayer, xa, positions, lay: StepLayout, cache: HybridCache):
        l = L.spec
        hd, hv = l.heads * l.dim, l.heads * l.vdim
        proj = ops.linear(xa, L.proj, out_f32=True)                 # q | k | v | gate | input gate | forget gate
        o, m = ops.mlstm_scan(proj, cache.state(i), lay.cu_q, positions, lay.state_slots, l.heads, l.dim, l.vdim,
                              l.gate_cap, self._max_len)
        y = ops.mlstm_out(o, m, L.head_norm, proj[:, 2 * hd + hv:2 * hd + 2 * hv], l.heads, l.vdim, self.cfg.rms_eps,
                          self.dtype)
        return ops.linear(y, L.out, out_f32=True)

    def _attention(self, i: int, L: HybridLayer, xa, positions, slot_mapping, lay: StepLayout, cache: HybridCache):
        l = L.spec
        src = i if l.owns_kv else l.kv_from
        kc, vc = cache.k(src), cache.v(src)
        qkv = ops.linear(xa, L.proj, out_f32=True)
        q = ops.qkv_prep(qkv, L.q_norm, L.k_norm, L.inv_freq, positions, slot_mapping, kc if l.owns_kv else None,
                         vc if l.owns_kv else None, l.heads, l.kv_heads, l.dim, l.vdim, l.rot_dims, l.rot_base,
                         self.cfg.rms_eps)
        a = ops.attn_masked(q, kc, vc, lay.block_tables, lay.cu_q, lay.row_seq, positions, l.heads, l.kv_heads, l.dim,
                            l.vdim, l.scale, l.chunk, l.window, self.dtype, n_portions=self._portions[0],
                            portion_rows=self._portions[1], max_len=self._max_len)
        return ops.linear(a, L.out, out_f32=True)

    def _gla(self, i: int, L: HybridLayer, xa, positions, lay: StepLayout, cache: HybridCache):
        l = L.spec
        hd, hv = l.heads * l.dim, l.heads * l.vdim
        proj = ops.linear(xa, L.proj, out_f32=True)                 # q | k | v | gate | bottleneck
        logits = ops.linear_any(proj[:, 2 * hd + 2 * hv:], L.decay_up)
        o = ops.gla_scan(proj, logits, cache.state(i), lay.cu_q, positions, lay.state_slots, l.heads, l.dim, l.vdim,
                         l.tau, self._max_len)
        y = ops.headnorm_gate(o, L.head_norm, proj[:, 2 * hd + hv:2 * hd + 2 * hv], l.vdim, self.cfg.rms_eps, self.dtype)
        return ops.linear(y, L.out, out_f32=True)

    def logits(self, hidden_rows: torch.Tensor) -> torch.Tensor:
        """fp32 logits [R, V] of the given rows of the residual stream (final norm, then the head)."""
        if self.cfg.design.pre_norm:
            xa = self._residual_norm(hidden_rows.contiguous(), None, self.final_norm)
        else:
            xa = ops.scalar_norm_add(hidden_rows, None, self.final_norm, self.cfg.rms_eps, self.dtype)
        return ops.linear(xa, self.lm_head, out_f32=True)

    def target_logprobs(self, hidden_rows: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
        return ops.logprob_gather(self.logits(hidden_rows), ids)

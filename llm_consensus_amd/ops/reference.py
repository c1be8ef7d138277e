"""Plain PyTorch (fp32 math) implementations of every op.

Two uses: (1) the numerics oracle each HIP kernel is tested against, (2) the CPU
plumbing backend, so the engine, the protocol drivers and the HTTP endpoint run end to
end on hosts without a GPU. They operate on the same data layouts as the kernels (paged
K / transposed-V cache, rotate-half RoPE tables) except that CPU weights stay row-major.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

MASK64 = (1 << 64) - 1


# ------------------------------------------------------------------ RNG (mirrors common.h)
def _mix64(z: int) -> int:
    z &= MASK64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK64
    return z ^ (z >> 31)


def rng_uniform(seed: int, step: int, counter: int = 0) -> float:
    z = _mix64((seed * 0x9E3779B97F4A7C15 + 0x632BE59BD9B4E019) & MASK64)
    z = _mix64(z ^ (((step & 0xFFFFFFFF) << 32) | (counter & 0xFFFFFFFF)))
    return ((z >> 40) + 0.5) * (1.0 / 16777216.0)


# ------------------------------------------------------------------ elementwise / norm
def embed(ids: torch.Tensor, E: torch.Tensor) -> torch.Tensor:
    return E[ids.long().clamp(0, E.shape[0] - 1)]


def rmsnorm(h: torch.Tensor, w: torch.Tensor, eps: float, delta: Optional[torch.Tensor] = None) -> torch.Tensor:
    if delta is not None:
        h.copy_((h.float() + delta.float()).to(h.dtype))
    x = h.float()
    y = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    return y.to(h.dtype)


def swiglu(gu: torch.Tensor) -> torch.Tensor:
    dff = gu.shape[-1] // 2
    g, u = gu[..., :dff].float(), gu[..., dff:].float()
    return (torch.nn.functional.silu(g) * u).to(gu.dtype)


def linear(x: torch.Tensor, W: torch.Tensor, bias: Optional[torch.Tensor] = None, out_dtype=None) -> torch.Tensor:
    y = x.float() @ W.float().t()
    if bias is not None:
        y = y + bias.float()
    return y.to(out_dtype or x.dtype)


# ------------------------------------------------------------------ RoPE + KV write
def rope_inv_freq(head_dim: int, theta: float, scaling: Optional[dict] = None) -> torch.Tensor:
    """Rotary inverse frequencies (float64, [head_dim/2]). ``scaling`` is a checkpoint's
    ``rope_scaling`` dict: ``llama3`` (Llama-3.1/3.2: wavelengths beyond the original context
    divided by ``factor``, a smooth blend between ``low_freq_factor`` and ``high_freq_factor``),
    ``linear`` (every frequency divided by ``factor``) or none/``default``. Anything else raises:
    a silently ignored scaling rule changes the logits at every position."""
    import math

    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))
    if not scaling:
        return inv
    kind = scaling.get("rope_type", scaling.get("type", "default"))
    if kind in (None, "default"):
        return inv
    if kind == "linear":
        return inv / float(scaling["factor"])
    if kind == "llama3":
        factor = float(scaling["factor"])
        lo, hi = float(scaling.get("low_freq_factor", 1.0)), float(scaling.get("high_freq_factor", 4.0))
        old = float(scaling["original_max_position_embeddings"])
        wavelen = 2 * math.pi / inv
        smooth = ((old / wavelen - lo) / (hi - lo)).clamp(0.0, 1.0)
        blended = (1 - smooth) * inv / factor + smooth * inv
        out = torch.where(wavelen > old / lo, inv / factor, torch.where(wavelen < old / hi, inv, blended))
        return out
    raise ValueError(f"rope_scaling type {kind!r} is not supported (supported: default, linear, llama3)")


def rope_tables(head_dim: int, max_pos: int, theta: float, device="cpu",
                scaling: Optional[dict] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    inv = rope_inv_freq(head_dim, theta, scaling)
    ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * inv[None, :]
    return ang.cos().float().to(device), ang.sin().float().to(device)


def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, slot_mapping: torch.Tensor, cos_t: torch.Tensor,
                  sin_t: torch.Tensor, k_cache: torch.Tensor, vt_cache: torch.Tensor, Hq: int, Hkv: int,
                  Dh: int) -> None:
    """qkv [T, (Hq+2Hkv)*Dh]: Q rotated in place; K rotated -> k_cache[blk, h, off, :];
    V -> vt_cache[blk, h, :, off]."""
    T = qkv.shape[0]
    BS = k_cache.shape[2]
    x = qkv.view(T, Hq + 2 * Hkv, Dh)
    pos = positions.long().clamp(0, cos_t.shape[0] - 1)
    c, s = cos_t[pos][:, None, :], sin_t[pos][:, None, :]  # [T,1,Dh/2]
    half = Dh // 2
    qk = x[:, : Hq + Hkv].float()
    a, b = qk[..., :half], qk[..., half:]
    ra = (a * c - b * s).to(qkv.dtype)   # round like the kernel: each half separately
    rb = (b * c + a * s).to(qkv.dtype)
    rot = torch.cat([ra, rb], dim=-1)
    x[:, :Hq] = rot[:, :Hq]
    slots = slot_mapping.long()
    ok = slots >= 0
    blk, off = slots[ok] // BS, slots[ok] % BS
    k_cache[blk, :, off, :] = rot[ok][:, Hq:]
    vt_cache[blk, :, :, off] = x[ok][:, Hq + Hkv:]


# ------------------------------------------------------------------ attention
def _gather_kv(k_cache, vt_cache, table, n):
    BS = k_cache.shape[2]
    nb = (n + BS - 1) // BS
    blocks = table[:nb].long()
    K = k_cache[blocks].permute(1, 0, 2, 3).reshape(k_cache.shape[1], nb * BS, -1)[:, :n]          # [Hkv, n, Dh]
    V = vt_cache[blocks].permute(1, 2, 0, 3).reshape(vt_cache.shape[1], vt_cache.shape[2], nb * BS)[..., :n]  # [Hkv, Dh, n]
    return K.float(), V.float()


def attn_prefill(q: torch.Tensor, k_cache, vt_cache, block_tables, cu_q, ctx_lens, Hq, Hkv, Dh, scale,
                 window: int = 0) -> torch.Tensor:
    """q [T, Hq*Dh] (may be a strided view into qkv). Causal over the paged context."""
    T = q.shape[0]
    out = torch.zeros(T, Hq * Dh, dtype=q.dtype, device=q.device)
    G = Hq // Hkv
    for s in range(len(ctx_lens)):
        q0, q1 = int(cu_q[s]), int(cu_q[s + 1])
        n, ql = int(ctx_lens[s]), q1 - q0
        if ql == 0:
            continue
        K, V = _gather_kv(k_cache, vt_cache, block_tables[s], n)
        Q = q[q0:q1].float().view(ql, Hkv, G, Dh)
        sc = torch.einsum("qhgd,hkd->hgqk", Q, K) * scale
        pos = torch.arange(n - ql, n, device=q.device)[:, None]
        key = torch.arange(n, device=q.device)[None, :]
        mask = key <= pos
        if window > 0:
            mask &= key > pos - window
        sc = sc.masked_fill(~mask[None, None], float("-inf"))
        p = torch.softmax(sc, dim=-1)
        o = torch.einsum("hgqk,hdk->qhgd", p, V)
        out[q0:q1] = o.reshape(ql, Hq * Dh).to(q.dtype)
    return out


def attn_decode(q: torch.Tensor, k_cache, vt_cache, block_tables, ctx_lens, Hq, Hkv, Dh, scale,
                window: int = 0) -> torch.Tensor:
    B = q.shape[0]
    cu = torch.arange(B + 1, dtype=torch.int32, device=q.device)
    return attn_prefill(q, k_cache, vt_cache, block_tables, cu, ctx_lens, Hq, Hkv, Dh, scale, window)


# ------------------------------------------------------------------ sampling
TOP_P_SEARCH_RANGE = 30.0     # the threshold search starts this far below the row maximum (logit / T units)
TOP_P_SEARCH_BINS = 12        # thresholds tried per refinement
TOP_P_SEARCH_PASSES = 4       # refinements: resolution 30 / 12^4 = 1.4e-3


def top_p_threshold(z: torch.Tensor, keep: torch.Tensor, p: float, floor: float = float("-inf")) -> float:
    """The nucleus cut as sampling.hip finds it: the kept set is {z >= thr}, and thr is the
    LARGEST threshold on a grid, refined TOP_P_SEARCH_PASSES times by a factor of
    TOP_P_SEARCH_BINS inside [max - TOP_P_SEARCH_RANGE, max], whose kept mass still reaches
    p * mass(keep). Against the exact top-p (sort, cumulative sum) this keeps, besides the exact
    nucleus, at most the entries within 30 / 12^4 = 1.4e-3 of the exact cut; on the flat
    distributions of a random-init model that is a few entries of ~1e-5 of the mass each. The
    definition is what both the kernel and this oracle implement, so their draws agree token for
    token (the arithmetic of the grid is done in fp32 here as there)."""
    import numpy as np

    f32 = np.float32
    zz = z.to(torch.float32).numpy()
    live = keep.numpy()
    zmax = f32(zz[live].max()) if live.any() else f32(0.0)
    mass = np.where(live, np.exp((zz - zmax).astype(np.float64)), 0.0)
    target = p * float(mass.sum())
    lo, hi = f32(max(f32(floor), zmax - f32(TOP_P_SEARCH_RANGE))), zmax
    thr = f32(floor)
    above, hi_is_max = 0.0, True
    for _ in range(TOP_P_SEARCH_PASSES):
        w = f32((hi - lo) * f32(1.0 / TOP_P_SEARCH_BINS))
        inv_w = f32(1.0) / w if w > 0 else f32(0.0)
        cand = live & (zz >= lo) & (np.ones_like(live) if hi_is_max else (zz < hi))
        b = np.minimum(((zz - lo) * inv_w).astype(np.int64), TOP_P_SEARCH_BINS - 1)
        bins = np.bincount(b[cand], weights=mass[cand], minlength=TOP_P_SEARCH_BINS)
        cum, best, above_best = above, -1, above
        for j in range(TOP_P_SEARCH_BINS - 1, -1, -1):
            before = cum
            cum += float(bins[j])
            if cum >= target:
                best, above_best = j, before
                break
        if best < 0:
            break
        nlo = f32(lo + w * f32(best))
        if best < TOP_P_SEARCH_BINS - 1:
            hi = f32(lo + w * f32(best + 1))
            hi_is_max = False
            above = above_best
        lo = nlo
        thr = lo
    return float(thr)


def sample(logits: torch.Tensor, temperature, top_p, top_k, seeds, steps, row_index=None):
    """Same definition as sampling.hip: scale by 1/T, keep the k largest, then the nucleus
    {z >= thr} with thr from ``top_p_threshold`` (relative to the mass that survived top-k), draw
    by inverse CDF in *index* order with u = rng_uniform(seed, step)."""
    R = len(temperature)
    toks = torch.zeros(R, dtype=torch.int32)
    lps = torch.zeros(R, dtype=torch.float32)
    for r in range(R):
        row = logits[int(row_index[r]) if row_index is not None else r].double().cpu()
        T = float(temperature[r])
        if not T > 0:
            lp = torch.log_softmax(row, -1)
            t = int(torch.argmax(row))
            toks[r], lps[r] = t, float(lp[t])
            continue
        z32 = (logits[int(row_index[r]) if row_index is not None else r].float().cpu()
               * torch.tensor(1.0 / T, dtype=torch.float32))
        z = row / T
        w = torch.exp(z - z.max())
        order = torch.argsort(w, descending=True, stable=True)
        keep = torch.ones_like(w, dtype=torch.bool)
        k = int(top_k[r]) if top_k is not None else 0
        floor = float("-inf")
        if 0 < k < w.numel():
            kth = w[order[k - 1]]
            keep &= w >= kth
            floor = float(z32[order[k - 1]])
        p = float(top_p[r]) if top_p is not None else 1.0
        if p < 1.0:
            keep &= z32 >= top_p_threshold(z32, keep, p, floor)
        wk = torch.where(keep, w, torch.zeros_like(w))
        u = rng_uniform(int(seeds[r]), int(steps[r]) if steps is not None else 0)
        csum = torch.cumsum(wk, 0)
        target = u * float(csum[-1])
        t = int(torch.searchsorted(csum, torch.tensor(target, dtype=csum.dtype), right=True).item())
        t = min(t, w.numel() - 1)
        while t > 0 and not bool(keep[t]):
            t -= 1
        toks[r] = t
        lps[r] = float(torch.log(wk[t] / csum[-1]))
    return toks.to(logits.device), lps.to(logits.device)


def logprob_gather(logits: torch.Tensor, ids: torch.Tensor, row_index=None) -> torch.Tensor:
    rows = logits if row_index is None else logits[row_index.long()]
    lp = torch.log_softmax(rows.float(), -1)
    ids = ids.long()
    if ids.dim() == 1:
        ids = ids[None, :].expand(rows.shape[0], -1)
    return torch.gather(lp, 1, ids.clamp(0, rows.shape[1] - 1))


# ------------------------------------------------------------------ MoE
def moe_router(x: torch.Tensor, Wr: torch.Tensor, topk: int):
    logits = (x.float() @ Wr.float().t()).to(x.dtype).float()  # HF rounds router logits to the model dtype
    p = torch.softmax(logits, -1)
    w, ids = torch.topk(p, topk, dim=-1)
    w = w / w.sum(-1, keepdim=True)
    return ids.int(), w.float(), logits


def embed_pool(hidden: torch.Tensor, cu: torch.Tensor, mode: int = 0) -> torch.Tensor:
    outs = []
    for s in range(len(cu) - 1):
        r0, r1 = int(cu[s]), int(cu[s + 1])
        if r1 <= r0:
            outs.append(torch.zeros(hidden.shape[1]))
            continue
        v = hidden[r1 - 1].float() if mode == 1 else hidden[r0:r1].float().mean(0)
        n = v.norm()
        outs.append(v / n if n > 0 else v)
    return torch.stack(outs).to(hidden.device)


# ------------------------------------------------------------------ hybrid decoders: fp32 residual stream
# Mixers of hybrid decoder designs (scalar-gain output norms on an fp32 residual stream, gated
# recurrences with per-sequence state slots, attention with separate key / value widths under a
# chunk or window mask). Sequences of a step are described by ``cu_q`` [B+1] (row ranges),
# ``positions`` [T] and ``slots`` [B] (state slot per sequence, < 0 = skip the sequence).
def scalar_norm_add(x: torch.Tensor, y: Optional[torch.Tensor], gain: torch.Tensor, eps: float, act_dtype):
    """x (fp32, in place) += y / sqrt(mean(y^2) + eps) * gain; without ``y`` the normed x itself is
    returned instead and x stays. Returns the result in ``act_dtype``."""
    if y is None:
        v = x.float()
        return (v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps) * gain.float()).to(act_dtype)
    v = y.float()
    x.add_(v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps) * gain.float())
    return x.to(act_dtype)


def relu2(y: torch.Tensor, act_dtype) -> torch.Tensor:
    return torch.relu(y.float()).pow(2).to(act_dtype)


def mingru_scan(zxg: torch.Tensor, state: torch.Tensor, cu_q, positions, slots, act_dtype) -> torch.Tensor:
    """zxg fp32 [T, 3w] = (update-gate logits, candidate pre-activations, output-gate logits).
    S <- (1 - z) S + z c with z = sigmoid(.), c = u + 1/2 for u >= 0 and sigmoid(u) below;
    returns S * silu(g) [T, w]. A sequence whose first row is at position 0 starts from zero."""
    T, w = zxg.shape[0], zxg.shape[1] // 3
    out = torch.zeros(T, w, dtype=torch.float32, device=zxg.device)
    z = torch.sigmoid(zxg[:, :w].float())
    u = zxg[:, w:2 * w].float()
    c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = zxg[:, 2 * w:].float()
    for b in range(len(slots)):
        r0, r1, slot = int(cu_q[b]), int(cu_q[b + 1]), int(slots[b])
        if slot < 0 or r1 <= r0:
            continue
        S = torch.zeros(w, dtype=torch.float32, device=zxg.device) if int(positions[r0]) == 0 else state[slot].clone()
        for t in range(r0, r1):
            S = (1 - z[t]) * S + z[t] * c[t]
            out[t] = S
        state[slot] = S
    return (out * g * torch.sigmoid(g)).to(act_dtype)


def gla_scan(proj: torch.Tensor, decay_logits: torch.Tensor, state: torch.Tensor, cu_q, positions, slots,
             H: int, D: int, Dv: int, tau: float) -> torch.Tensor:
    """proj fp32 [T, >= 2HD + HDv]: columns (q | k | v); decay_logits fp32 [T, HD].
    Per head S <- diag(a) S + k v^T with a = sigmoid(logit)^(1/tau), o = S^T (q / sqrt(D)).
    state [slots, H*D*Dv] fp32. Returns o fp32 [T, H*Dv]."""
    T = proj.shape[0]
    q = proj[:, :H * D].float().view(T, H, D) * (D ** -0.5)
    k = proj[:, H * D:2 * H * D].float().view(T, H, D)
    v = proj[:, 2 * H * D:2 * H * D + H * Dv].float().view(T, H, Dv)
    a = torch.exp(torch.nn.functional.logsigmoid(decay_logits.float()) / tau).view(T, H, D)
    out = torch.zeros(T, H, Dv, dtype=torch.float32, device=proj.device)
    for b in range(len(slots)):
        r0, r1, slot = int(cu_q[b]), int(cu_q[b + 1]), int(slots[b])
        if slot < 0 or r1 <= r0:
            continue
        S = state[slot].view(H, D, Dv).clone()
        if int(positions[r0]) == 0:
            S.zero_()
        for t in range(r0, r1):
            S = a[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
            out[t] = torch.einsum("hdv,hd->hv", S, q[t])
        state[slot] = S.reshape(-1)
    return out.view(T, H * Dv)


def headnorm_gate(o: torch.Tensor, w: torch.Tensor, gate: torch.Tensor, Dv: int, eps: float, act_dtype) -> torch.Tensor:
    """Per head of width Dv: o / sqrt(mean(o^2) + eps) * w, times silu(gate)."""
    T = o.shape[0]
    v = o.float().view(T, -1, Dv)
    v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    g = gate.float()
    return (v.view(T, -1) * g * torch.sigmoid(g)).to(act_dtype)


def rope_partial(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x fp32 [T, heads, D]: the first ``dims`` coordinates of each head rotate (coordinate i with
    i + dims/2, angle position * base^(-2i/dims)), the rest pass."""
    half = dims // 2
    if half == 0:
        return x
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64),
                  -2.0 * torch.arange(half, dtype=torch.float64) / dims).float().to(x.device)
    ang = positions.float()[:, None] * f[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def qkv_prep(qkv: torch.Tensor, q_norm: torch.Tensor, k_norm: Optional[torch.Tensor], positions, slot_mapping,
             k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor], H: int, G: int, D: int, Dv: int,
             rot_dims: int, rot_base: float, eps: float) -> torch.Tensor:
    """qkv fp32 [T, H*D (+ G*D + G*Dv)]. Queries (and keys) are RMS-normed over their WHOLE
    projection with a weight per coordinate, then rotated; each value head is scaled to unit RMS.
    Keys go to k_cache [blocks, G, BS, D], values to v_cache [blocks, G, BS, Dv] at the rows'
    slots (skipped when the layer has no keys of its own: ``k_cache`` None). Returns q fp32 [T, H*D]."""
    T = qkv.shape[0]
    q = qkv[:, :H * D].float()
    q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * q_norm.float()
    q = rope_partial(q.view(T, H, D), positions, rot_dims, rot_base).reshape(T, H * D)
    if k_cache is not None:
        k = qkv[:, H * D:(H + G) * D].float()
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * k_norm.float()
        k = rope_partial(k.view(T, G, D), positions, rot_dims, rot_base)
        v = qkv[:, (H + G) * D:(H + G) * D + G * Dv].float().view(T, G, Dv)
        v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
        BS = k_cache.shape[2]
        slots = slot_mapping.long()
        ok = slots >= 0
        blk, off = slots[ok] // BS, slots[ok] % BS
        k_cache[blk, :, off, :] = k[ok].to(k_cache.dtype)
        v_cache[blk, :, off, :] = v[ok].to(v_cache.dtype)
    return q.contiguous()


def attn_masked(q: torch.Tensor, k_cache, v_cache, block_tables, cu_q, positions, H: int, G: int, D: int, Dv: int,
                scale: float, chunk: int, window: int, act_dtype, softcap: float = 0.0, sink: bool = False,
                all_value_heads: bool = False) -> torch.Tensor:
    """q fp32 [T, H*D]; paged keys [blocks, G, BS, D] and values [blocks, G, BS, Dv]. The row at
    position p sees keys j <= p with j >= floor(p / chunk) * chunk (``chunk`` > 0) and
    j > p - window (``window`` > 0). Scores, softmax and the weighted sum in fp32. ``softcap`` > 0: scores
    become softcap * tanh(score / softcap); ``sink``: the softmax's denominator carries an extra 1 (an entry of
    score 0 without a value); ``all_value_heads``: every head's weights meet the values of all G value heads,
    result [T, H * G * Dv]."""
    T = q.shape[0]
    nv = G if all_value_heads else 1
    out = torch.zeros(T, H * nv * Dv, dtype=torch.float32, device=q.device)
    BS = k_cache.shape[2]
    rep = H // G
    for b in range(len(cu_q) - 1):
        r0, r1 = int(cu_q[b]), int(cu_q[b + 1])
        if r1 <= r0:
            continue
        pos = positions[r0:r1].long()
        n = int(pos.max()) + 1
        nb = (n + BS - 1) // BS
        blocks = block_tables[b, :nb].long()
        K = k_cache[blocks].permute(1, 0, 2, 3).reshape(G, nb * BS, D)[:, :n].float()
        V = v_cache[blocks].permute(1, 0, 2, 3).reshape(G, nb * BS, Dv)[:, :n].float()
        Q = q[r0:r1].float().view(r1 - r0, G, rep, D)
        sc = torch.einsum("qgrd,gkd->grqk", Q, K) * scale
        if softcap > 0:
            sc = softcap * torch.tanh(sc / softcap)
        key = torch.arange(n, device=q.device)[None, :]
        mask = key <= pos[:, None]
        if chunk > 0:
            mask &= key >= (pos[:, None] // chunk) * chunk
        if window > 0:
            mask &= key > pos[:, None] - window
        sc = sc.masked_fill(~mask[None, None], float("-inf"))
        if sink:
            m = sc.max(-1, keepdim=True).values.clamp_min(0.0)
            e = torch.exp(sc - m)
            w = e / (torch.exp(-m) + e.sum(-1, keepdim=True))
        else:
            w = torch.softmax(sc, dim=-1)
        if all_value_heads:
            out[r0:r1] = torch.einsum("grqk,ckv->qgrcv", w, V).reshape(r1 - r0, H * G * Dv)
        else:
            out[r0:r1] = torch.einsum("grqk,gkv->qgrv", w, V).reshape(r1 - r0, H * Dv)
    return out.to(act_dtype)


# ------------------------------------------------------------------ hybrid decoders: pre-norm designs, latent
# attention, mLSTM, routed feed-forwards
def sinusoid_rows(positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """fp32 [T, 2 * len(inv_freq)]: entry 2i = sin(p f_i), entry 2i + 1 = cos(p f_i); angles in fp64."""
    ang = positions.double()[:, None] * inv_freq.double()[None, :]
    return torch.stack([torch.sin(ang), torch.cos(ang)], -1).reshape(positions.numel(), -1).float()


def add_rmsnorm(x: torch.Tensor, y: Optional[torch.Tensor], w: Optional[torch.Tensor], eps: float, act_dtype):
    """x (fp32, in place) += y; returns x / sqrt(mean(x^2) + eps) * w in ``act_dtype`` (None without w)."""
    if y is not None:
        x.add_(y.float())
    if w is None:
        return None
    return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(act_dtype)


def latent_write(proj: torch.Tensor, col0: int, w: torch.Tensor, eps: float, slot_mapping, cache: torch.Tensor) -> None:
    """cache [blocks, 1, BS, R] at the rows' slots <- rms_norm(proj[:, col0:col0 + R]) * w."""
    R, BS = cache.shape[3], cache.shape[2]
    c = proj[:, col0:col0 + R].float()
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    slots = slot_mapping.long()
    ok = slots >= 0
    cache[slots[ok] // BS, 0, slots[ok] % BS, :] = c[ok].to(cache.dtype)


def head_linear(x: torch.Tensor, W: torch.Tensor, out_dtype, gate: Optional[torch.Tensor] = None,
                x_head_stride: Optional[int] = None, out: Optional[torch.Tensor] = None,
                out_head_stride: Optional[int] = None, gate_full: bool = False) -> torch.Tensor:
    """x [T, >= H*K], W [H, N, K] -> y with y[t, h] = W[h] x[t, h]; head h reads from column h * x_head_stride and
    writes from column h * out_head_stride (of ``out`` when given); ``gate`` [T, H]: y[t, h] *= sigmoid(gate[t, h]),
    or a logit per output, [T, H*N], with ``gate_full``."""
    H, N, K = W.shape
    T = x.shape[0]
    xs = K if x_head_stride is None else x_head_stride
    os_ = N if out_head_stride is None else out_head_stride
    xh = torch.stack([x[:, h * xs:h * xs + K].float() for h in range(H)], 1)
    y = torch.einsum("thk,hnk->thn", xh, W.float())
    if gate is not None:
        y = y * (torch.sigmoid(gate.float()).view(T, H, N) if gate_full else torch.sigmoid(gate.float())[:, :, None])
    if out is None:
        out = torch.zeros(T, (H - 1) * os_ + N, dtype=out_dtype, device=x.device)
    for h in range(H):
        out[:, h * os_:h * os_ + N] = y[:, h].to(out_dtype)
    return out


def capped(x: torch.Tensor, cap: float) -> torch.Tensor:
    return cap * torch.tanh(x / cap) if cap > 0 else x


def mlstm_scan(proj: torch.Tensor, state: torch.Tensor, cu_q, positions, slots, H: int, D: int, Dv: int, cap: float):
    """Matrix-memory recurrence with a running maximum. proj fp32 [T, >= 2HD + 2HDv + 2H]: columns
    q | k | v | (output gate) | input-gate logits | forget-gate logits. Per head, with
    i = cap tanh(. / cap), f = log sigmoid(cap tanh(. / cap)), m <- max(f + m, i):
    S <- exp(f + m' - m) S + exp(i - m) k [v, 1]^T (the extra column carries the normaliser n),
    read out with q / sqrt(D). state [slots, H*D*(Dv+1) + H] fp32 (S with n as its last column,
    then m). Returns (o fp32 [T, H*(Dv+1)] whose last column per head is n.q, m fp32 [T, H])."""
    T = proj.shape[0]
    hd, hv = H * D, H * Dv
    q = proj[:, :hd].float().view(T, H, D) * (D ** -0.5)
    k = proj[:, hd:2 * hd].float().view(T, H, D)
    v = torch.cat([proj[:, 2 * hd:2 * hd + hv].float().view(T, H, Dv), torch.ones(T, H, 1, device=proj.device)], -1)
    ig = capped(proj[:, 2 * hd + 2 * hv:2 * hd + 2 * hv + H].float(), cap)
    fg = torch.nn.functional.logsigmoid(capped(proj[:, 2 * hd + 2 * hv + H:2 * hd + 2 * hv + 2 * H].float(), cap))
    out = torch.zeros(T, H, Dv + 1, dtype=torch.float32, device=proj.device)
    ms = torch.zeros(T, H, dtype=torch.float32, device=proj.device)
    n_s = H * D * (Dv + 1)
    for b in range(len(slots)):
        r0, r1, slot = int(cu_q[b]), int(cu_q[b + 1]), int(slots[b])
        if slot < 0 or r1 <= r0:
            continue
        S = state[slot, :n_s].view(H, D, Dv + 1).clone()
        m = state[slot, n_s:].clone()
        if int(positions[r0]) == 0:
            S.zero_()
            m.zero_()
        for t in range(r0, r1):
            mn = torch.maximum(fg[t] + m, ig[t])
            a, bb = torch.exp(fg[t] + m - mn), torch.exp(ig[t] - mn)
            S = a[:, None, None] * S + (bb[:, None] * k[t])[:, :, None] * v[t][:, None, :]
            m = mn
            out[t] = torch.einsum("hdv,hd->hv", S, q[t])
            ms[t] = m
        state[slot, :n_s] = S.reshape(-1)
        state[slot, n_s:] = m
    return out.view(T, H * (Dv + 1)), ms


def mlstm_out(o: torch.Tensor, m: torch.Tensor, w: torch.Tensor, gate: torch.Tensor, H: int, Dv: int, eps: float,
              act_dtype) -> torch.Tensor:
    """o [T, H*(Dv+1)] from ``mlstm_scan``: per head h = o[:Dv] / (max(|o[Dv]|, exp(-m)) + 1e-6),
    h / sqrt(mean(h^2) + eps) * w (w [H*Dv]), times sigmoid(gate)."""
    T = o.shape[0]
    oo = o.float().view(T, H, Dv + 1)
    den = torch.maximum(oo[:, :, Dv].abs(), torch.exp(-m.float())) + 1e-6
    h = oo[:, :, :Dv] / den[:, :, None]
    h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + eps)
    return (h.reshape(T, H * Dv) * w.float() * torch.sigmoid(gate.float())).to(act_dtype)


def glu(y: torch.Tensor, act_dtype, kind: str = "relu") -> torch.Tensor:
    """y [T, 2n] = (gate | up) -> act(gate) * up."""
    n = y.shape[1] // 2
    g, u = y[:, :n].float(), y[:, n:].float()
    g = torch.relu(g) if kind == "relu" else g * torch.sigmoid(g)
    return (g * u).to(act_dtype)


def route_grouped(z: torch.Tensor, correction: Optional[torch.Tensor], top: int, groups: int, keep: int, scale: float,
                  score: str = "softmax"):
    """Router over fp32 logits z [T, n]: s = softmax(z) (or sigmoid(z), each output on its own); choice = s + correction; the n outputs form
    ``groups`` equal runs of neighbours, a run's score is its largest choice, only the ``keep`` best runs
    stay eligible; the ``top`` largest eligible choices are taken (ties: the lower index) with weights
    s * scale. Returns (ids int32 [T, top], weights fp32 [T, top])."""
    T, n = z.shape
    s = torch.softmax(z.float(), -1) if score == "softmax" else torch.sigmoid(z.float())
    ch = s + correction.float() if correction is not None else s.clone()
    if groups > 1 and keep < groups:
        gs = ch.view(T, groups, n // groups).max(-1).values
        order = torch.argsort(gs, dim=-1, descending=True, stable=True)[:, :keep]
        allow = torch.zeros(T, groups, dtype=torch.bool, device=z.device).scatter_(1, order, True)
        ch = ch.masked_fill(~allow.repeat_interleave(n // groups, 1), float("-inf"))
    ids = torch.argsort(ch, dim=-1, descending=True, stable=True)[:, :top]
    return ids.to(torch.int32), (s.gather(1, ids) * scale).float()


def grouped_linear(x: torch.Tensor, row_index: Optional[torch.Tensor], offsets: torch.Tensor, W: torch.Tensor,
                   out_dtype, rows: int, relu2_epi: bool = False) -> torch.Tensor:
    """Sorted position p in [offsets[e], offsets[e+1]) reads x[row_index[p]] (x[p] without an index) and
    gives W[e] x; W [E, N, K]. Positions of experts >= E (no tensors) stay zero."""
    E, N, K = W.shape
    y = torch.zeros(rows, N, dtype=torch.float32, device=x.device)
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi > lo:
            xe = x[row_index[lo:hi].long()] if row_index is not None else x[lo:hi]
            y[lo:hi] = xe.float() @ W[e].float().t()
    if relu2_epi:
        y = torch.relu(y).pow(2)
    return y.to(out_dtype)


def moe_mix(ye: torch.Tensor, slot_of: torch.Tensor, ids: torch.Tensor, wts: Optional[torch.Tensor], h: torch.Tensor, E: int,
            shared: Optional[torch.Tensor], shared_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 [T, d]: sum_k wts[t, k] * (ye[slot_of[t, k]] for ids < E, h[t] itself for the identity experts
    ids >= E) + shared[t] (times sigmoid(shared_gate[t]) when gate logits [T, 1] are given); no weights: 1."""
    T, top = ids.shape
    rows = ye[slot_of.long()].float().view(T, top, -1)
    rows = torch.where((ids >= E)[:, :, None], h.float()[:, None, :], rows)
    out = (rows * wts.float()[:, :, None]).sum(1) if wts is not None else rows.sum(1)
    if shared is None:
        return out
    return out + (shared.float() * torch.sigmoid(shared_gate.float().reshape(T, 1)) if shared_gate is not None else shared.float())


def add_dyt(x: torch.Tensor, y: Optional[torch.Tensor], mult: float, alpha: float, w: Optional[torch.Tensor],
            b: Optional[torch.Tensor], out: Optional[torch.Tensor]) -> None:
    """x (fp32, in place) += mult * y; ``out`` (a view, any type) <- tanh(alpha x) * w + b, or x itself without w."""
    if y is not None:
        x.add_(y.float(), alpha=mult)
    if out is not None:
        out.copy_((torch.tanh(alpha * x) * w.float() + b.float()) if w is not None else x)


def rope_pairs(x: torch.Tensor, positions: torch.Tensor, dims: int, inv_freq: torch.Tensor) -> torch.Tensor:
    """x fp32 [T, heads, D]: in the first ``dims`` coordinates of each head the neighbours (2i, 2i + 1) turn by
    position * inv_freq[i] (fp64 angles); the rest pass."""
    if dims == 0:
        return x
    ang = positions.double()[:, None] * inv_freq.double()[None, :]
    c, s = torch.cos(ang).float()[:, None, :], torch.sin(ang).float()[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    rot = torch.stack([u * c - v * s, v * c + u * s], -1).reshape(*x.shape[:-1], dims)
    return torch.cat([rot, x[..., dims:]], -1)


def rope_pairs_write(qk: torch.Tensor, inv_freq: Optional[torch.Tensor], positions, slot_mapping, k_cache: torch.Tensor,
                     v_cache: Optional[torch.Tensor], H: int, G: int, D: int, rot_dims: int) -> torch.Tensor:
    """qk fp32 [T, >= (H + G) D] = q | k. Rotated keys go to k_cache [blocks, G, BS, D], the keys as projected
    (before the rotation) to v_cache, the layer's values. Returns the rotated q fp32 [T, H*D]."""
    T = qk.shape[0]
    q = rope_pairs(qk[:, :H * D].float().view(T, H, D), positions, rot_dims, inv_freq).reshape(T, H * D)
    k = qk[:, H * D:(H + G) * D].float().view(T, G, D)
    BS = k_cache.shape[2]
    slots = slot_mapping.long()
    ok = slots >= 0
    blk, off = slots[ok] // BS, slots[ok] % BS
    k_cache[blk, :, off, :] = rope_pairs(k, positions, rot_dims, inv_freq)[ok].to(k_cache.dtype)
    if v_cache is not None:
        v_cache[blk, :, off, :] = k[ok].to(v_cache.dtype)
    return q.contiguous()


def glu_clamped(y: torch.Tensor, col_gate: int, col_up: int, n: int, limit: float, slope: float, shift: float,
                slot_of: Optional[torch.Tensor], wts: Optional[torch.Tensor], act_dtype, rows: int) -> torch.Tensor:
    """g = min(s gate, limit), u = clamp(s up, -limit, limit) -> g sigmoid(slope g) (u + shift); with a work list,
    entry r is row slot_of[r] scaled by s = wts[r] (rows no entry names stay zero)."""
    g, u = y[:, col_gate:col_gate + n].float(), y[:, col_up:col_up + n].float()
    if slot_of is None:
        s = 1.0
    else:
        s = torch.zeros(y.shape[0], 1, dtype=torch.float32, device=y.device)
        s[slot_of.long().reshape(-1)[:rows], 0] = wts.float().reshape(-1)[:rows] if wts is not None else 1.0
    g, u = torch.clamp(g * s, max=limit), torch.clamp(u * s, -limit, limit)
    return (g * torch.sigmoid(slope * g) * (u + shift)).to(act_dtype)


# ------------------------------------------------------------------ hybrid decoders: parallel residual streams, rotary
# values, mixed heads' weights, rotated latent keys, xIELU
def hc_init(x0: torch.Tensor, w: torch.Tensor, eps: float, streams: int) -> torch.Tensor:
    """fp32 [T, S, d]: every stream is rms_norm(x0) * w."""
    e = x0 * torch.rsqrt(x0.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    return e[:, None, :].repeat(1, streams, 1).contiguous()


def hc_step(xs: torch.Tensor, y, mix, out_w, in_w, norm_w, eps: float, act_dtype):
    """xs fp32 [T, S, d] in place: xs[:, j] <- sum_s mix[s, j] xs[:, s] + out_w[j] y (with y); then
    u = sum_s in_w[s] xs[:, s] (with in_w), returned normed times norm_w in ``act_dtype``, or as it is."""
    S = xs.shape[1]
    if y is not None:
        xs.copy_(torch.einsum("sj,tsd->tjd", mix.float().view(S, S), xs) + out_w.float()[None, :, None] * y.float()[:, None, :])
    if in_w is None:
        return None
    u = torch.einsum("s,tsd->td", in_w.float(), xs)
    if norm_w is None:
        return u
    return (u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()).to(act_dtype)


def rope_any(x: torch.Tensor, positions: torch.Tensor, dims: int, inv_freq: torch.Tensor, pairs: bool,
             sign: float = 1.0) -> torch.Tensor:
    """x fp32 [T, heads, D]: the first ``dims`` coordinates of each head turn by sign * position * inv_freq[i]
    (fp64 angles), neighbours together (``pairs``) or i with i + dims / 2; the rest pass."""
    if dims == 0:
        return x
    if pairs:
        return rope_pairs(x, positions if sign > 0 else -positions, dims, inv_freq)
    half = dims // 2
    ang = sign * positions.double()[:, None] * inv_freq.double()[None, :]
    c, s = torch.cos(ang).float()[:, None, :], torch.sin(ang).float()[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def rope_qkv_write(qkv: torch.Tensor, inv_freq, inv_freq_v, positions, slot_mapping, k_cache, v_cache, H: int, G: int,
                   D: int, Dv: int, rot_dims: int, pairs: bool, v_pairs: bool) -> torch.Tensor:
    """qkv fp32 [T, >= H D + G (D + Dv)] = q | k | v: q and k turn over their first rot_dims coordinates, v (with
    ``inv_freq_v``) over its whole width; keys and values go to the paged planes. Returns the turned q [T, H*D]."""
    T = qkv.shape[0]
    q = rope_any(qkv[:, :H * D].float().view(T, H, D), positions, rot_dims, inv_freq, pairs).reshape(T, H * D)
    if k_cache is not None:
        k = rope_any(qkv[:, H * D:(H + G) * D].float().view(T, G, D), positions, rot_dims, inv_freq, pairs)
        v = qkv[:, (H + G) * D:(H + G) * D + G * Dv].float().view(T, G, Dv)
        if inv_freq_v is not None:
            v = rope_any(v, positions, Dv, inv_freq_v, v_pairs)
        BS = k_cache.shape[2]
        slots = slot_mapping.long()
        ok = slots >= 0
        blk, off = slots[ok] // BS, slots[ok] % BS
        k_cache[blk, :, off, :] = k[ok].to(k_cache.dtype)
        v_cache[blk, :, off, :] = v[ok].to(v_cache.dtype)
    return q.contiguous()


def talk_mix(o: torch.Tensor, talk: torch.Tensor, positions, inv_freq_v, H: int, G: int, Dv: int, act_dtype,
             v_pairs: bool) -> torch.Tensor:
    """o fp32 [T, H * G * Dv] -> out[t, h] = sum_g talk[h, g] o[t, g, h / (H / G)], turned back by the row's position."""
    T = o.shape[0]
    o5 = o.float().view(T, H, G, Dv)
    kv = torch.arange(H, device=o.device) // (H // G)
    mixed = torch.einsum("hg,tghv->thv", talk.float().view(H, H), o5[:, :, kv, :])
    if inv_freq_v is not None:
        mixed = rope_any(mixed, positions, Dv, inv_freq_v, v_pairs, sign=-1.0)
    return mixed.reshape(T, H * Dv).to(act_dtype)


def latent_rope_write(proj: torch.Tensor, col_c: int, w, eps: float, inv_freq, positions, slot_mapping, cache, qlat,
                      H: int, D: int, R: int, rd: int, pairs: bool) -> None:
    """cache [blocks, 1, BS, R + rd] <- rms_norm(proj[:, col_c:+R]) * w | turned proj[:, col_c + R:+rd]; the turned
    query parts (columns D .. D + rd - 1 of each head's block of D + rd) go to columns R .. R + rd - 1 of each head's
    block of qlat [T, H * (R + rd)]."""
    T = proj.shape[0]
    if rd:
        qr = proj[:, :H * (D + rd)].float().view(T, H, D + rd)[:, :, D:]
        qlat.view(T, H, R + rd)[:, :, R:] = rope_any(qr, positions, rd, inv_freq, pairs)
    if cache is None:
        return
    BS = cache.shape[2]
    c = proj[:, col_c:col_c + R].float()
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    row = [c]
    if rd:
        row.append(rope_any(proj[:, col_c + R:col_c + R + rd].float().view(T, 1, rd), positions, rd, inv_freq, pairs)[:, 0])
    slots = slot_mapping.long()
    ok = slots >= 0
    cache[slots[ok] // BS, 0, slots[ok] % BS, :] = torch.cat(row, -1)[ok].to(cache.dtype)


def xielu(y: torch.Tensor, ap: float, an: float, act_dtype) -> torch.Tensor:
    z = y.float()
    return torch.where(z > 0, ap * z * z + 0.5 * z, an * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z).to(act_dtype)

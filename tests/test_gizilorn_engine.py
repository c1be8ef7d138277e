"""Gizilorn decoders through the engine (scheduler, paged cache, step function) against the plain
implementation in ``gizilorn_oracle.py``. Small configurations with random weights made here; every
test runs on the CPU ops and, marked ``gpu``, on the HIP kernels."""
import copy
import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import gizilorn_oracle as oracle
from llm_consensus_amd._native import core
from llm_consensus_amd.engine.engine import Engine
from llm_consensus_amd.models.hybrid import HybridModel, config_from_dict, config_to_dict

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, torch.bfloat16]
BS = 16
ROOT = Path(__file__).resolve().parents[1]
FF = {"kind": "dense", "ff": 56}


def attn(heads=4, kv=2, dim=12, vdim=10, window=21, rot=6, base=500.0, scale=0.3, cap=4.0, mlp=FF):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "softcap": cap, "mask": {"size": window},
         "rot": {"dims": rot, "base": base}}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def latent(heads=3, dim=10, rot_dim=6, vdim=14, rank=20, window=17, base=3000.0, scale=0.25, kv_from=None, mlp=FF):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale, "mask": {"size": window},
         "rot": {"dims": rot_dim, "base": base}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def config(layers, width=40, vocab=67, streams=3, eps=1e-5):
    return {"architecture": "Gizilorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "streams": streams,
            "layers": layers}


MIXED = config([latent(), attn(), latent(kv_from=0, heads=2, dim=8, vdim=6, window=9, mlp=None), attn(heads=3, kv=3, dim=8, vdim=8, window=40, rot=8, cap=30.0),
                latent(heads=4, dim=4, rot_dim=4, vdim=8, rank=12, window=33), latent(kv_from=0, window=5)])


def build(cfg, device, dtype=torch.float32, seed=0, blocks=24, slots=4, weights=None, **kw):
    W = weights if weights is not None else oracle.random_weights(cfg, seed)
    model = HybridModel(config_from_dict(cfg, "test", {k: tuple(v.shape) for k, v in W.items()}), device, dtype)
    model.set_weights(lambda n: W[n])
    eng = Engine(model, num_kv_blocks=blocks, block_size=BS, max_batch_seqs=kw.pop("max_batch_seqs", slots),
                 state_slots=slots, max_model_len=blocks * BS, enable_prefix_cache=False,
                 use_graphs=kw.pop("use_graphs", False), pipeline_decode=kw.pop("pipeline_decode", False), **kw)
    return eng, W


def tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def replay_alone(eng, toks, cuts):
    """One request fed in portions of the given sizes (the rest one token at a time); all logits."""
    rid, at, out = eng.replay_open(), 0, []
    sizes = list(cuts) + [1] * (len(toks) - sum(cuts))
    for n in sizes:
        out.append(eng.replay_step([(rid, toks[at:at + n], list(range(n)))]))
        at += n
    eng.replay_close(rid)
    return np.concatenate(out)


def rel_err(got, want):
    """Largest row error (mean taken off, RMS over the vocabulary, against the mean RMS of the wanted rows)."""
    want = want.numpy() if hasattr(want, "numpy") else want
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return float((np.sqrt((d ** 2).mean(-1)) / np.sqrt((w ** 2).mean(-1)).mean()).max())


def limit(dtype):
    return 2e-4 if dtype == torch.float32 else 6e-2


def _whole_prompt(cfg, device, dtype, name, cuts=None, seed=0, n=45):
    eng, W = build(cfg, device, dtype, seed=seed)
    toks = tokens(n if cuts is None else sum(cuts) + 3, cfg["vocab"], 3)
    got = replay_alone(eng, toks, cuts or [len(toks)])
    assert rel_err(got, oracle.forward(cfg, W, toks)) < limit(dtype), name


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,layers,streams", [
    ("attention: grouped heads, part of the head turns, values narrower than keys", [attn(), attn(heads=6, kv=3, dim=10, vdim=16, window=5, rot=4)], 3),
    ("attention: one key head; as many key heads as heads; the whole head turns", [attn(heads=4, kv=1, dim=16, vdim=16, window=30, rot=16),
                                                                                  attn(heads=3, kv=3, dim=8, vdim=4, window=19, rot=8)], 2),
    ("attention: widths of the matrix-core kernel, two and four value heads side by side", [attn(heads=4, kv=2, dim=16, vdim=32, window=25, rot=8),
                                                                                           attn(heads=8, kv=4, dim=32, vdim=16, window=44, rot=32)], 2),
    ("attention: nothing of q and k turns, one head, widths of 2", [attn(heads=1, kv=1, dim=7, vdim=2, window=12, rot=0), attn(heads=2, kv=1, dim=2, vdim=6, window=3, rot=2)], 3),
    ("attention: a window of one, longer than the prompt, a cap that always binds, one that never does", [attn(window=1), attn(window=500, cap=0.3), attn(cap=1e4)], 2),
    ("latent attention: own rows, another layer's rows twice, widths of the matrix-core kernel", [latent(rank=24, rot_dim=8, vdim=16, window=11), latent(kv_from=0, rank=24, rot_dim=8, heads=5, dim=6, vdim=4),
                                                                                                 attn(), latent(kv_from=0, rank=24, rot_dim=8, window=30)], 2),
    ("latent attention: one head, a turned part of two, wider than a wave", [latent(heads=1, rot_dim=2, rank=7), latent(heads=2, dim=70, rot_dim=80, vdim=66, rank=130, window=200)], 3),
    ("one stream", [attn(), latent()], 1),
    ("four streams, layers without a feed-forward", [latent(mlp=None), attn(mlp=None), attn(), latent(kv_from=0, mlp=None)], 4),
    ("eight streams", [attn(mlp={"kind": "dense", "ff": 9})], 8),
])
def test_each_mechanism_whole_prompt(device, dtype, name, layers, streams):
    _whole_prompt(config(layers, streams=streams), device, dtype, name)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_depths_the_mfma_products_take(device, dtype):
    """Widths of 64 / 128 with feed-forwards of 64 / 192 units: in bf16 on the GPU the projections go through the
    packed MFMA kernels (depths in multiples of 64, fp32 epilogues, biases)."""
    for width, ff in ((64, 64), (128, 192)):
        cfg = config([attn(heads=4, kv=2, dim=16, vdim=16, rot=8, mlp={"kind": "dense", "ff": ff}), latent(heads=4, dim=16, rot_dim=8, vdim=16, rank=24, mlp={"kind": "dense", "ff": ff}),
                      latent(kv_from=1, heads=4, dim=16, rot_dim=8, vdim=16, rank=24, mlp=None)], width=width, vocab=70, streams=2)
        _whole_prompt(cfg, device, dtype, f"mfma depths {width}", cuts=[40, 2, 17])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_deep_products_and_a_long_portion(device, dtype):
    """Width 1024 (the bf16 products of a few rows split their depth over workgroups), fused projection
    widths that are no multiple of 32, a portion of a few hundred rows, a short one, decoded tokens."""
    cfg = config([attn(heads=3, kv=1, dim=16, vdim=16, window=100, rot=8, mlp={"kind": "dense", "ff": 72}),
                  latent(heads=2, dim=24, rot_dim=8, vdim=16, rank=40, window=260, mlp=None)], width=1024, vocab=90, streams=2)
    eng, W = build(cfg, device, dtype, blocks=24)
    toks = tokens(300, cfg["vocab"], 3)
    assert rel_err(replay_alone(eng, toks, [270, 20]), oracle.forward(cfg, W, toks)) < limit(dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_constants_that_could_pass_for_one(device):
    """Score scales and caps of 1, one stream read and written with weights of exactly one, then other constants
    with the SAME tensors; norm weights and activation numbers far from their usual values; a large eps."""
    layers = [attn(scale=1.0, cap=1.0), latent(scale=1.0)]
    cfg = config(layers, streams=1, eps=1.0)
    W = oracle.random_weights(cfg, 4)
    for k in W:
        if ".hc" in k:
            W[k] = torch.ones_like(W[k])
        elif k.endswith(("norm1", "norm2", "final.norm", "embed.norm", "dkv.norm")):
            W[k] = (W[k].float() * 3 - 1.5).to(W[k].dtype)
        elif k.endswith("mlp.act"):
            W[k] = torch.tensor([1.7, -2.0]).to(W[k].dtype)
    eng, _ = build(cfg, device, weights=W)
    toks = tokens(30, cfg["vocab"], 9)
    base = oracle.forward(cfg, W, toks)
    assert rel_err(replay_alone(eng, toks, [17]), base) < 2e-4
    other = config([attn(scale=0.6, cap=2.5), latent(scale=0.4)], streams=1, eps=1e-3)
    for k in W:
        if ".hc" in k:
            W[k] = (0.7 * torch.ones_like(W[k].float())).to(W[k].dtype)
    eng2, _ = build(other, device, weights=W)
    want = oracle.forward(other, W, toks)
    assert rel_err(want.numpy(), base) > 0.05
    assert rel_err(replay_alone(eng2, toks, [17]), want) < 2e-4


@pytest.mark.parametrize("device", DEVICES)
def test_the_sink_takes_its_share_and_the_cap_binds(device):
    """Biases on the queries and keys (on coordinates that do not turn) and a negative scale put every score a few
    units below zero: the weights of a row sum to about a half, so an implementation without the extra entry in
    the denominator, which would make them sum to one, gives other logits. A second model whose raw scores lie far
    above the cap shows that the cap is applied before the softmax."""
    cfg = config([attn(heads=2, kv=1, dim=8, vdim=8, window=30, rot=4, scale=-0.3, cap=50.0, mlp=None)], streams=2)
    W = oracle.random_weights(cfg, 2)
    qb, kb = W["l0.mix.q.b"].float(), W["l0.mix.k.b"].float()
    qb[4:8] = qb[12:16] = kb[4:8] = 1.7
    W["l0.mix.q.b"], W["l0.mix.k.b"] = qb.to(torch.bfloat16), kb.to(torch.bfloat16)
    W["l0.mix.q"], W["l0.mix.k"] = (0.3 * W["l0.mix.q"].float()).to(torch.bfloat16), (0.3 * W["l0.mix.k"].float()).to(torch.bfloat16)
    eng, _ = build(cfg, device, weights=W)
    toks = tokens(40, cfg["vocab"], 13)
    Wd = {k: v.double() for k, v in W.items()}
    e = oracle.rms_norm(Wd["embed"][toks], Wd["embed.norm"], 1e-5)
    h = oracle.rms_norm(sum(Wd["l0.hc1.in"][s] * e for s in range(2)), Wd["l0.norm1"], 1e-5)
    _, wts = oracle.talking_attention(h, Wd, "l0.mix.", cfg["layers"][0]["mixer"], return_weights=True)
    sums = wts.sum(-1)
    assert 0.3 < float(sums.median()) < 0.7 and float(sums.max()) < 0.9      # the silent entry holds a real share of every row
    assert rel_err(replay_alone(eng, toks, [25]), oracle.forward(cfg, W, toks)) < 2e-4
    capped = config([attn(heads=2, kv=1, dim=8, vdim=8, window=30, rot=4, scale=3.0, cap=1.5, mlp=None)], streams=2)
    loose = copy.deepcopy(capped)
    loose["layers"][0]["mixer"]["softcap"] = 1e3
    assert rel_err(oracle.forward(capped, W, toks).numpy(), oracle.forward(loose, W, toks)) > 0.05
    eng2, _ = build(capped, device, weights=W)
    assert rel_err(replay_alone(eng2, toks, [25]), oracle.forward(capped, W, toks)) < 2e-4


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_heads_cross_the_groups(device):
    """A mixing matrix that gives every head ONLY another group's weights (a cyclic shift by the group size): a
    head's output is then built from its own group's values under weights computed with the other group's keys."""
    H, G = 4, 2
    cfg = config([attn(heads=H, kv=G, dim=8, vdim=6, window=20, rot=8, mlp=None)], streams=2)
    W = oracle.random_weights(cfg, 8)
    shift = torch.zeros(H, H)
    for h in range(H):
        shift[h, (h + H // G) % H] = 1.5
    W["l0.mix.talk"] = shift.to(torch.bfloat16)
    same = dict(W)
    same["l0.mix.talk"] = (1.5 * torch.eye(H)).to(torch.bfloat16)
    toks = tokens(35, cfg["vocab"], 6)
    want = oracle.forward(cfg, W, toks)
    assert rel_err(oracle.forward(cfg, same, toks).numpy(), want) > 0.05
    for cuts in ([35], [20]):
        eng, _ = build(cfg, device, weights=W)
        assert rel_err(replay_alone(eng, toks, cuts), want) < 2e-4


@pytest.mark.parametrize("device", DEVICES)
def test_residual_stream_after_every_layer(device):
    eng, W = build(MIXED, device)
    toks = tokens(20, MIXED["vocab"], 5)
    taps, rid = [], eng.replay_open()
    eng.replay_step([(rid, toks, [])], taps=taps)
    _, want = oracle.forward(MIXED, W, toks, return_layers=True)
    assert len(taps) == len(want) == 6
    for i, t in enumerate(taps):
        torch.testing.assert_close(t.cpu().double(), want[i], atol=2e-4, rtol=2e-4, msg=f"layer {i}")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cuts", [[], [1], [40], [2, 2, 3, 2, 17, 2], [11, 1, 1, 12, 13], [5, 7, 12, 16, 1, 15, 2]])
def test_portions_and_token_by_token_decoding(device, dtype, cuts):
    """The same logits whether the prompt comes whole, in portions down to two tokens (cut inside pages of 16
    and inside windows of 5, 9, 17, 21, 33 and 40), or one token at a time."""
    eng, W = build(MIXED, device, dtype)
    toks = tokens(70, MIXED["vocab"], 7)
    assert rel_err(replay_alone(eng, toks, cuts), oracle.forward(MIXED, W, toks)) < limit(dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_past_pages_and_windows(device):
    eng, W = build(MIXED, device)
    toks = tokens(120, MIXED["vocab"], 11)
    assert rel_err(replay_alone(eng, toks, [3]), oracle.forward(MIXED, W, toks)) < 2e-4


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_mixed_batches_reused_pages(device, dtype):
    """Up to four live requests, portions beside single tokens, in a pool too small for all of them at once:
    requests end, others take their pages."""
    eng, W = build(MIXED, device, dtype, blocks=12, slots=4)
    V = MIXED["vocab"]
    reqs = {n: tokens(L, V, 20 + i) for i, (n, L) in enumerate([("a", 50), ("b", 33), ("c", 1), ("d", 47), ("e", 40),
                                                                ("f", 18), ("g", 60)])}
    want = {n: oracle.forward(MIXED, W, t) for n, t in reqs.items()}
    sched = [[("a", 20), ("b", 2)], [("a", 1), ("b", 13), ("c", 1)], [("a", 1), ("b", 1), ("d", 30)],
             [("a", 28), ("d", 1)], [("b", 17), ("d", 16), ("e", 9)], [("e", 1)], [("e", 30), ("f", 18)],
             [("g", 33)], [("g", 1)], [("g", 26)]]
    at, rid, got = {n: 0 for n in reqs}, {}, {n: [] for n in reqs}
    free0 = eng.kvm.stats().blocks_free
    for step in sched:
        entries = []
        for n, k in step:
            if n not in rid:
                rid[n] = eng.replay_open()
            entries.append((rid[n], reqs[n][at[n]:at[n] + k], list(range(k))))
        lg = eng.replay_step(entries)
        o = 0
        for n, k in step:
            got[n].append(lg[o:o + k])
            o += k
            at[n] += k
            if at[n] == len(reqs[n]):
                eng.replay_close(rid[n])
    assert all(at[n] == len(reqs[n]) for n in reqs)
    assert eng.kvm.stats().blocks_free == free0
    for n in reqs:
        assert rel_err(np.concatenate(got[n]), want[n]) < limit(dtype), n


def _one_layer(kind, window):
    if kind == "attention":
        return attn(heads=2, kv=1, dim=8, vdim=8, window=window, rot=4, scale=0.05, mlp=None)
    return latent(heads=2, dim=8, rot_dim=4, vdim=8, rank=16, window=window, scale=0.05, mlp=None)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kind", ["attention", "latent_attention"])
@pytest.mark.parametrize("window", [5, 16, 21])
@pytest.mark.parametrize("decode_from", [0, 3, 30])
def test_the_windows_edge_at_every_place_and_page_border(device, kind, window, decode_from):
    """ONE mixer and nothing else (no other way for a token to reach a later row), a flat softmax: a changed
    token at place j moves the rows j .. j + window - 1 and no other, neither the rows before it nor the row at
    j + window, whether the rows run as a prompt or are decoded one by one. Pages of 16: the window's far edge
    crosses page borders as the rows go on."""
    cfg = config([_one_layer(kind, window)], streams=2)
    eng, W = build(cfg, device)
    toks = tokens(60, cfg["vocab"], 31)
    cuts = [decode_from] if decode_from else [len(toks)]
    base = replay_alone(eng, toks, cuts)
    assert rel_err(base, oracle.forward(cfg, W, toks)) < 2e-4
    for j in (0, 1, 10, 15, 16, 17, 31, 32, 38, 59):
        alt = list(toks)
        alt[j] = (alt[j] + 1) % cfg["vocab"]
        moved = np.abs(replay_alone(eng, alt, cuts) - base).max(-1)
        inside = np.zeros(len(toks), dtype=bool)
        inside[j:j + window] = True
        assert (moved[inside] > 2e-6).all() and (moved[~inside] < 1e-6).all(), (j, np.nonzero(moved > 1e-6)[0])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kind", ["attention", "latent_attention"])
def test_the_oldest_key_of_the_window_stands_out(device, kind):
    """The key at the window's far edge carries the answer: the first token's query / key input is made so that
    every row that still sees it gives it most of its weight, and the first row that does not falls back to the
    others. The oracle's own weights confirm the jump between the last row inside and the first row outside."""
    window = 23
    cfg = config([_one_layer(kind, window)], vocab=30, streams=1)
    cfg["layers"][0]["mixer"].update(scale=1.0, softcap=60.0)
    cfg["layers"][0]["mixer"]["rot"]["dims"] = 0 if kind == "attention" else 4
    W = oracle.random_weights(cfg, 6)
    d = cfg["width"]
    toks = [29] + tokens(50, 29, 3)                 # token 29 appears at place 0 only
    # Embedding coordinate 0 is large for token 29 and zero for every other token; coordinate 1 is the same positive
    # number for all. Every row's query has one plain coordinate that reads a constant; the key coordinate it meets
    # reads coordinate 0 of the mixer's input, so only the first token's key scores, and highly.
    E = W["embed"].float()
    E[:, 0], E[:, 1] = 0.0, 1.0
    E[29, 0] = 40.0
    W["embed"] = E.to(torch.bfloat16)
    for n in ("embed.norm", "l0.norm1"):
        W[n] = torch.ones(d, dtype=torch.bfloat16)
    W["l0.hc1.in"] = torch.ones(1, dtype=torch.bfloat16)
    if kind == "attention":
        qb, k = torch.zeros(16), torch.zeros(8, d)
        qb[0] = qb[8] = 1.0                         # both heads: query = first key coordinate, whatever the token
        k[0, 0] = 4.0
        W["l0.mix.q"], W["l0.mix.q.b"] = torch.zeros(16, d, dtype=torch.bfloat16), qb.to(torch.bfloat16)
        W["l0.mix.k"], W["l0.mix.k.b"] = k.to(torch.bfloat16), torch.zeros(8, dtype=torch.bfloat16)
    else:
        q, dkv, uk = torch.zeros(2 * 12, d), torch.zeros(20, d), torch.zeros(16, 16)
        q[0, 1] = q[12, 1] = 3.0                    # both heads: plain query coordinate 0 reads the constant coordinate
        dkv[0, 0] = 1.0                             # compressed coordinate 0 reads the marked coordinate
        dkv[1:16, 2:] = 0.05 * torch.randn(15, d - 2, generator=torch.Generator().manual_seed(1))
        uk[0, 0] = uk[8, 0] = 3.0                   # both heads: plain key coordinate 0 = compressed coordinate 0
        W["l0.mix.q"], W["l0.mix.dkv"], W["l0.mix.uk"] = q.to(torch.bfloat16), dkv.to(torch.bfloat16), uk.to(torch.bfloat16)
        W["l0.mix.dkv.norm"] = torch.ones(16, dtype=torch.bfloat16)
    Wd = {n: v.double() for n, v in W.items()}
    h = oracle.rms_norm(Wd["l0.hc1.in"][0] * oracle.rms_norm(Wd["embed"][toks], Wd["embed.norm"], 1e-5), Wd["l0.norm1"], 1e-5)
    m = cfg["layers"][0]["mixer"]
    if kind == "attention":
        _, wts = oracle.talking_attention(h, Wd, "l0.mix.", m, return_weights=True)
    else:
        _, wts = oracle.latent_attention(h, Wd, "l0.mix.", m, oracle.latent_rows(h, Wd, "l0.mix.", m, 1e-5), return_weights=True)
    assert float((wts[0, :, 0] > 0).sum()) == window          # the first key is seen by the first ``window`` rows only
    assert float(wts[0, 1:window, 0].min()) > 0.5             # and holds most of their weight
    for cuts in ([len(toks)], [window - 2], [2]):
        eng, _ = build(cfg, device, weights=W)
        assert rel_err(replay_alone(eng, toks, cuts), oracle.forward(cfg, W, toks)) < 2e-4, cuts


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kind", ["attention", "latent_attention"])
def test_a_far_key_that_stands_out(device, kind):
    """One key far back among hundreds carries the answer: with a large score scale single keys dominate the
    softmax rows, so dropping or misplacing one shows. The window holds 280 keys; the last rows are decoded."""
    layer = _one_layer(kind, 280)
    layer["mixer"].update(scale=5.0, softcap=80.0, heads=1)
    layer["mixer"]["rot"]["base"] = 1e5
    cfg = config([layer], vocab=50, streams=2)
    eng, W = build(cfg, device, blocks=24)
    toks = tokens(330, cfg["vocab"], 41)
    assert rel_err(replay_alone(eng, toks, [300]), oracle.forward(cfg, W, toks)) < 2e-4
    Wd = {k: v.double() for k, v in W.items()}
    e = oracle.rms_norm(Wd["embed"][toks], Wd["embed.norm"], 1e-5)
    h = oracle.rms_norm(sum(Wd["l0.hc1.in"][s] * e for s in range(2)), Wd["l0.norm1"], 1e-5)
    m = layer["mixer"]
    if kind == "attention":
        _, wts = oracle.talking_attention(h, Wd, "l0.mix.", m, return_weights=True)
    else:
        _, wts = oracle.latent_attention(h, Wd, "l0.mix.", m, oracle.latent_rows(h, Wd, "l0.mix.", m, 1e-5), return_weights=True)
    far = sum(int(float(wts[0, i].max()) > 0.5 and i - int(wts[0, i].argmax()) > 100) for i in range(300, len(toks)))
    assert far >= 3


@pytest.mark.parametrize("device", DEVICES)
def test_values_turn_with_their_own_position_and_back_with_the_rows(device):
    """A small rotary base and rows far from the start: the angles of the values and of the rows that read them are
    large and differ from row to row. What a row sums are values turned by their distance to it, so the turns do not
    cancel: the same weights under a base so large that nothing turns give other logits. The paged values hold the
    turned rows (the op that writes them, against the oracle's turn)."""
    from llm_consensus_amd import ops

    cfg = config([attn(heads=2, kv=2, dim=8, vdim=8, window=300, rot=0, base=3.0, mlp=None)], streams=2)
    eng, W = build(cfg, device, blocks=24)
    toks = tokens(200, cfg["vocab"], 17)
    want = oracle.forward(cfg, W, toks)
    still = copy.deepcopy(cfg)
    still["layers"][0]["mixer"]["rot"]["base"] = 1e30
    assert rel_err(oracle.forward(still, W, toks).numpy(), want) > 0.05
    assert rel_err(replay_alone(eng, toks, [150, 2, 30]), want) < 2e-4
    g = torch.Generator().manual_seed(1)
    T, G, D, Dv = 9, 2, 4, 6
    qkv = torch.randn(T, 3 * D + G * (D + Dv), generator=g)
    pos = torch.tensor([0, 1, 2, 50, 51, 700, 3, 4, 5], dtype=torch.int32)
    slots = torch.tensor([0, 1, 2, 9, 10, 20, 5, 6, 7], dtype=torch.int32)
    kc, vc = torch.zeros(3, G, 8, D), torch.zeros(3, G, 8, Dv)
    fv = torch.tensor([3.0 ** (-2.0 * j / Dv) for j in range(Dv // 2)], dtype=torch.float64)
    dev = torch.device(device)
    kd, vd = kc.to(dev), vc.to(dev)
    ops.rope_qkv_write(qkv.to(dev), None, fv.to(dev), pos.to(dev), slots.to(dev), kd, vd, 3, G, D, Dv, 0)
    v = qkv[:, 3 * D + G * D:].double().view(T, G, Dv)
    turned = oracle.turn(v, pos.tolist(), Dv, 3.0, "halves")
    got = vd.cpu().double().permute(0, 2, 1, 3).reshape(24, G, Dv)[slots.long()]
    torch.testing.assert_close(got, turned, atol=1e-5, rtol=1e-5)
    assert float((turned - v).abs().max()) > 0.5


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens_and_single_token_requests(device):
    eng, W = build(MIXED, device)
    for toks in ([7], [7, 7], tokens(3, MIXED["vocab"], 2)):
        assert rel_err(replay_alone(eng, toks, [len(toks)]), oracle.forward(MIXED, W, toks)) < 2e-4
        assert rel_err(replay_alone(eng, toks, []), oracle.forward(MIXED, W, toks)) < 2e-4


@pytest.mark.parametrize("device", DEVICES)
def test_pool_exhausted_is_an_error_and_leaves_the_engine_usable(device):
    cfg = config([attn(), latent()])
    eng, W = build(cfg, device, blocks=2, slots=4)
    a, b, c = eng.replay_open(), eng.replay_open(), eng.replay_open()
    eng.replay_step([(a, [1, 2], []), (b, [3], [])])
    with pytest.raises(RuntimeError):
        eng.replay_step([(c, [4], [])])
    eng.replay_close(a)
    lg = eng.replay_step([(c, [4, 5], [1])])
    assert rel_err(lg, oracle.forward(cfg, W, [4, 5])[1:]) < 2e-4


def _greedy_oracle(cfg, W, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(oracle.forward(cfg, W, toks)[-1].argmax()))
    return toks[len(prompt):]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_submit_and_the_scheduler(device, graphs):
    """More requests than the batch holds, prompts cut by the scheduler's token budget, decoding chains riding
    in the steps that prefill later prompts; recorded decode steps on the GPU."""
    if graphs and device == "cpu":
        pytest.skip("decode graphs are a GPU feature")
    eng, W = build(MIXED, device, blocks=40, slots=3, max_batch_seqs=3, max_prefill_tokens=24, use_graphs=graphs,
                   pipeline_decode=graphs)
    p = core.SamplingParams()
    p.temperature, p.max_new_tokens, p.ignore_eos = 0.0, 9, True
    prompts = [tokens(n, MIXED["vocab"], 50 + n) for n in (30, 5, 41, 1, 17)]
    rids = [eng.submit(pr, params=p) for pr in prompts]
    eng.run_until_done()
    for rid, pr in zip(rids, prompts):
        out = eng.pop_result(rid)
        assert out.token_ids[0] == _greedy_oracle(MIXED, W, pr, 9)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_serving_steps_launch_only_the_kernel_library(dtype):
    """Prompt portions, mixed steps, decode steps and replayed steps: PyTorch launches no kernel of its own in
    any of them (allocations, views and buffer copies aside)."""
    from llm_consensus_amd.utils.audit import AtenAudit

    cfg = config([latent(heads=4, dim=16, rot_dim=8, vdim=16, rank=24, mlp={"kind": "dense", "ff": 64}), attn(heads=4, kv=2, dim=16, vdim=16, rot=8),
                  latent(kv_from=0, heads=2, dim=8, rot_dim=8, vdim=8, rank=24, mlp=None), attn()], width=64, vocab=70, streams=2)
    eng, _ = build(cfg, "cuda:0", dtype, blocks=40, slots=3, max_batch_seqs=3, max_prefill_tokens=24)
    p = core.SamplingParams()
    p.temperature, p.max_new_tokens, p.ignore_eos = 0.7, 5, True

    def work():
        rids = [eng.submit(tokens(n, cfg["vocab"], n), params=p) for n in (30, 5, 41)]
        eng.run_until_done()
        rid = eng.replay_open()
        eng.replay_step([(rid, tokens(20, cfg["vocab"], 1), [0, 19])])
        eng.replay_step([(rid, [3], [0])])
        eng.replay_close(rid)
        return [eng.pop_result(r) for r in rids]

    work()
    torch.cuda.synchronize()
    with AtenAudit() as audit:
        outs = work()
        torch.cuda.synchronize()
    assert all(len(o.token_ids[0]) == 5 for o in outs)
    assert audit.kernels == {}, audit.kernels


def test_checkpoint_directory_through_the_registry_the_trace_tool_and_the_command_line(tmp_path, capsys):
    """A Gizilorn checkpoint directory is found by its config.json, loaded with the checkpoint's tensor names,
    replayed by ``bin/trace_run`` (two requests in one step, a request that ends and one that goes on) and
    answers a question through the command line."""
    from safetensors.torch import save_file

    from llm_consensus_amd import cli
    from llm_consensus_amd.models.loader import load_model
    from llm_consensus_amd.models.registry import resolve

    cfg = config([latent(), attn(heads=2, kv=1, dim=8, vdim=8, window=6, rot=8), latent(kv_from=0, mlp=None)], width=32, vocab=300, streams=2)
    W = oracle.random_weights(cfg, 3)
    ck = tmp_path / "gizilorn"
    ck.mkdir()
    (ck / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in W.items()}, str(ck / "model.safetensors"))
    assert resolve(str(ck)).name == "hybrid"
    m = load_model(str(ck), "cpu", dtype=torch.float32)
    back = config_to_dict(m.cfg)
    assert back["layers"] == cfg["layers"] and back["streams"] == cfg["streams"] and back["norm"] == cfg["norm"]
    a, b = tokens(21, 300, 1), tokens(9, 300, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": [0, 16]}, {"id": "b", "tokens": b[:2], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[17:18], "want": [0]}, {"id": "b", "tokens": b[2:], "want": [6]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[18:], "want": [2]}], "end": ["a"]}]
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(ck), "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "128", "--device", "cpu"], input="".join(json.dumps(s) + "\n" for s in steps),
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    la, lb = oracle.forward(cfg, W, a).numpy(), oracle.forward(cfg, W, b).numpy()
    got = [np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, 300) for i in range(3)]
    assert rel_err(got[0], la[[0, 16]]) < 2e-4
    assert rel_err(got[1], np.stack([la[17], lb[8]])) < 2e-4
    assert rel_err(got[2], la[[20]]) < 2e-4
    toml = tmp_path / "e.toml"
    toml.write_text(f"""strategy = "majority_vote"
decision_mode = "logprob"
choices = "ABCD"
[sampling]
temperature = 0.0
max_new_tokens = 4
[models.h]
path = "{ck}"
[[members]]
name = "hybrid"
model = "h"
""")
    q = tmp_path / "q.txt"
    q.write_text("Which? A. a B. b C. c D. d\n")
    assert cli.main(["--config", str(toml), "--questions", str(q), "--device", "cpu", "--no-warm-up"]) == 0
    assert capsys.readouterr().out.strip()[-1] in "ABCD"


def test_random_checkpoint_writer_and_random_init(tmp_path):
    """The family's checkpoint writer and ``random_init`` (benchmarks, stand-ins) know the design's tensors: what
    one writes the loader reads back, and both models answer the same."""
    from llm_consensus_amd.models.loader import load_model, write_random_hybrid_checkpoint

    cfg = config_from_dict(config([attn(), latent(), latent(kv_from=1, mlp=None)], width=24, vocab=80, streams=2))
    ck = write_random_hybrid_checkpoint(cfg, str(tmp_path / "ck"), seed=7)
    assert json.loads((ck / "config.json").read_text())["architecture"] == "Gizilorn"
    a = load_model(str(ck), "cpu", dtype=torch.float32)
    b = HybridModel.random_init(cfg, "cpu", seed=7, dtype=torch.float32)
    assert a.cfg.layers == b.cfg.layers and a.cfg.streams == b.cfg.streams == 2
    out = []
    for m in (a, b):
        eng = Engine(m, num_kv_blocks=8, block_size=BS, max_batch_seqs=2, state_slots=2, max_model_len=8 * BS,
                     enable_prefix_cache=False, use_graphs=False, pipeline_decode=False)
        out.append(replay_alone(eng, tokens(12, 80, 1), [7]))
    assert np.isfinite(out[0]).all() and np.abs(out[0]).max() > 0
    np.testing.assert_allclose(out[0], out[1], rtol=1e-6, atol=1e-6)


def test_configurations_the_design_does_not_have_are_refused():
    with pytest.raises(ValueError):
        config_from_dict(config([attn(vdim=5)]))                              # values that turn have an even width
    with pytest.raises(ValueError):
        config_from_dict(config([attn()], streams=9))
    with pytest.raises(ValueError):
        config_from_dict(config([latent(kv_from=0)]))                        # no earlier layer to read from
    with pytest.raises(ValueError):
        config_from_dict(config([latent(), latent(kv_from=0, rank=8)]))      # another latent width
    with pytest.raises(ValueError):
        config_from_dict(config([latent(), latent(kv_from=0), latent(kv_from=1)]))     # a layer without rows of its own
    with pytest.raises(ValueError):
        config_from_dict(config([attn(mlp={"kind": "moe"})]))
    with pytest.raises(ValueError):
        config_from_dict(config([{"type": "mingru", "mixer": {"width": 8}, "mlp": None}]))

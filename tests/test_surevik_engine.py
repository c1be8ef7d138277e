"""Surevik decoders through the engine (scheduler, paged cache, step function) against the plain
implementation in ``surevik_oracle.py``. Small configurations with random weights made here; every
test runs on the CPU ops and, marked ``gpu``, on the HIP kernels."""
import json
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import surevik_oracle as oracle
from llm_consensus_amd._native import core
from llm_consensus_amd.engine.engine import Engine
from llm_consensus_amd.models.hybrid import HybridModel, config_from_dict, config_to_dict

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, torch.bfloat16]
BS = 16
ROOT = Path(__file__).resolve().parents[1]


def moe(experts=6, top=2, ff=20, limit=0.7, shared=24, shared_limit=1.2):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top},
            "shared": {"ff": shared, "limit": shared_limit} if shared else None}


def attn(heads=4, kv=2, dim=12, window=21, rot=6, base=500.0, scale=0.3, mlp=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": scale, "mask": {"size": window} if window else None,
         "rot": {"dims": rot, "base": base} if rot is not None else None}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def config(layers, width=40, vocab=67, loop=None, mult=0.6, embed_scale=3.0):
    c = {"architecture": "Surevik", "vocab": vocab, "width": width, "norm": {"eps": 1e-6}, "embedding": {"scale": embed_scale},
         "residual_mult": mult, "layers": layers}
    if loop:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


MIXED = config([attn(mlp=moe()), attn(heads=4, kv=1, dim=16, window=9, rot=16), attn(heads=2, kv=2, dim=10, window=40, rot=4, mlp=moe(experts=5, top=1, shared=0)),
                attn(heads=3, kv=3, dim=8, window=17, rot=0, mlp=moe(experts=3, top=3, ff=9, shared=7))], loop=(1, 3, 2))


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


def rel_err(got, want, rows=None):
    """Largest row error (mean taken off, RMS over the vocabulary, against the mean RMS of the wanted
    rows) over the first ``rows`` rows (default: all)."""
    want = want.numpy() if hasattr(want, "numpy") else want
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    err = np.sqrt((d ** 2).mean(-1)) / np.sqrt((w ** 2).mean(-1)).mean()
    return float(err[:rows].max()) if len(err[:rows]) else 0.0


_ORACLE = {}


def plain(cfg, W, toks):
    """(logits, per-token margin of the closest routing choice) of the plain implementation, kept per case."""
    key = (json.dumps(cfg, sort_keys=True), float(sum(float(v.float().abs().sum()) for v in W.values())), tuple(toks))
    if key not in _ORACLE:
        _ORACLE[key] = oracle.forward(cfg, W, toks, return_margins=True)
    return _ORACLE[key]


def expected(cfg, W, toks, dtype, least=4):
    """(logits of the plain implementation, rows to compare). In bf16 a router whose candidates' scores lie within
    rounding of each other can choose the other one, and every later row that sees that token then differs for
    good: rows are compared up to the first token with such a close call (none is one in fp32)."""
    want, margins = plain(cfg, W, toks)
    if dtype == torch.float32:
        return want, len(toks)
    close = np.nonzero(margins.numpy() < 0.003)[0]
    rows = int(close[0]) if len(close) else len(toks)
    assert rows >= min(least, len(toks)), f"only {rows} rows before the first close call: take other tokens"
    return want, rows


def tokens_for(cfg, W, n, seed, dtype, least=4):
    """``tokens(n, vocab, seed)``; for bf16 the one of a few such sequences whose first close routing call comes latest."""
    if dtype == torch.float32:
        return tokens(n, cfg["vocab"], seed)
    best, rows = None, -1
    for k in range(8):
        toks = tokens(n, cfg["vocab"], seed + 1000 * k)
        close = np.nonzero(plain(cfg, W, toks)[1].numpy() < 0.003)[0]
        r = int(close[0]) if len(close) else n
        if r > rows:
            best, rows = toks, r
        if rows >= max(least, n // 2):
            break
    return best


def limit(dtype):
    return 2e-4 if dtype == torch.float32 else 6e-2


def _whole_prompt(cfg, device, dtype, name, cuts=None, seed=0, n=45):
    eng, W = build(cfg, device, dtype, seed=seed)
    toks = tokens_for(cfg, W, n if cuts is None else sum(cuts) + 3, 3, dtype)
    got = replay_alone(eng, toks, cuts or [len(toks)])
    assert rel_err(got, *expected(cfg, W, toks, dtype)) < limit(dtype), name


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,layers,loop", [
    ("attention: grouped heads, part of the head turns", [attn(), attn(heads=6, kv=3, dim=10, window=5, rot=4)], None),
    ("attention: one key head, the whole head turns, widths of the matrix-core kernel", [attn(heads=4, kv=1, dim=16, window=30, rot=16),
                                                                                         attn(heads=2, kv=2, dim=32, window=19, rot=8)], None),
    ("attention: nothing turns (one plane is keys and values), odd width", [attn(heads=2, kv=1, dim=7, window=12, rot=0), attn(heads=1, kv=1, dim=9, window=3, rot=None)], None),
    ("attention: a window of one, a window longer than the prompt, none", [attn(window=1), attn(window=500), attn(window=0)], None),
    ("routed feed-forward: two of six, a shared expert", [attn(mlp=moe())], None),
    ("routed feed-forward: one of seven, none shared; all of three", [attn(mlp=moe(experts=7, top=1, shared=0)), attn(mlp=moe(experts=3, top=3, ff=5))], None),
    ("routed feed-forward: more experts than a wave has lanes, limits that rarely bind", [attn(mlp=moe(experts=70, top=5, ff=4, limit=30.0, shared_limit=30.0))], None),
    ("layers without a feed-forward, looped from the first layer on", [attn(), attn(mlp=moe()), attn()], (0, 2, 3)),
    ("a loop that ends the stack", [attn(mlp=moe()), attn(), attn(mlp=moe(top=1))], (1, 3, 2)),
    ("a loop of one pass still re-injects", [attn(), attn(mlp=moe())], (1, 2, 1)),
])
def test_each_mechanism_whole_prompt(device, dtype, name, layers, loop):
    _whole_prompt(config(layers, loop=loop), device, dtype, name)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_depths_the_mfma_products_take(device, dtype):
    """Widths of 64 / 128 and experts of 64 / 128 units: in bf16 on the GPU the projections and the experts go
    through the packed MFMA kernels (depths in multiples of 64, fp32 epilogues)."""
    for width, ff in ((64, 64), (128, 128)):
        cfg = config([attn(heads=4, kv=2, dim=16, rot=8, mlp=moe(ff=ff, shared=64)), attn(heads=2, kv=1, dim=32, window=50, rot=32, mlp=moe(experts=9, top=3, ff=64, shared=0))],
                     width=width, vocab=70, loop=(0, 1, 2))
        _whole_prompt(cfg, device, dtype, f"mfma depths {width}", cuts=[40, 2, 17])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_deep_products_and_a_long_portion(device, dtype):
    """Width 1024 (the bf16 products of a few rows split their depth over workgroups), fused projection
    widths that are no multiple of 32, a portion of a few hundred rows, a short one, decoded tokens."""
    cfg = config([attn(heads=3, kv=1, dim=16, window=100, rot=8, mlp=moe(ff=64, shared=64)), attn(heads=2, kv=2, dim=24, window=260, rot=24)],
                 width=1024, vocab=90, loop=(1, 2, 2))
    eng, W = build(cfg, device, dtype, blocks=24)
    toks = tokens_for(cfg, W, 300, 3, dtype)
    got = replay_alone(eng, toks, [270, 20])
    assert rel_err(got, *expected(cfg, W, toks, dtype)) < limit(dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_constants_that_could_pass_for_one(device):
    """A residual multiplier, an embedding scale and score scale of 1 and then other values with the SAME
    weights; slopes, norm weights and biases far from 1 and 0: none is assumed."""
    layers = [attn(scale=1.0, mlp=moe(limit=1.0, shared_limit=1.0)), attn(mlp=moe(top=1))]
    cfg = config(layers, mult=1.0, embed_scale=1.0)
    W = oracle.random_weights(cfg, 4)
    for k in W:
        if k.endswith(".alpha"):
            W[k] = (W[k].float() * 0.3).to(W[k].dtype)
        elif k.endswith(("norm1", "norm2", "final.norm")):
            W[k] = (W[k].float() * 3 - 1.0).to(W[k].dtype)
        elif k.endswith(("norm1.b", "norm2.b", "final.norm.b")):
            W[k] = (W[k].float() * 4 + 0.5).to(W[k].dtype)
    eng, _ = build(cfg, device, weights=W)
    toks = tokens(30, cfg["vocab"], 9)
    base = oracle.forward(cfg, W, toks)
    assert rel_err(replay_alone(eng, toks, [17]), base) < 2e-4
    other = config(layers, mult=0.45, embed_scale=2.5)
    eng2, _ = build(other, device, weights=W)
    want = oracle.forward(other, W, toks)
    assert rel_err(want.numpy(), base) > 0.05
    assert rel_err(replay_alone(eng2, toks, [17]), want) < 2e-4


@pytest.mark.parametrize("device", DEVICES)
def test_the_weight_scales_the_experts_input(device):
    """Limits low enough that the clamps bind: scaling an expert's input is then not scaling its output. The
    oracle's two orders differ, and the engine follows the first; several experts per token are chosen."""
    mlp = moe(experts=5, top=2, limit=0.25, shared=0)
    cfg = config([attn(mlp=mlp)])
    eng, W = build(cfg, device, seed=5)
    toks = tokens(40, cfg["vocab"], 12)
    want = oracle.forward(cfg, W, toks)
    assert rel_err(replay_alone(eng, toks, [25]), want) < 2e-4
    Wd = {k: v.double() for k, v in W.items()}
    x = Wd["embed"][toks] * cfg["embedding"]["scale"]
    x = x + cfg["residual_mult"] * oracle.window_attention(oracle.tanh_norm(x, Wd, "l0.norm1"), Wd, "l0.mix.", cfg["layers"][0]["mixer"])
    h = oracle.tanh_norm(x, Wd, "l0.norm2")
    a, b = oracle.routed_ff(h, Wd, "l0.mlp.", mlp), oracle.routed_ff(h, Wd, "l0.mlp.", mlp, weight_on_output=True)
    assert float((a - b).abs().max()) > 0.05 * float(a.abs().max())
    ids, _ = oracle.choose(h, Wd, "l0.mlp.", mlp["router"])
    assert len(set(ids.reshape(-1).tolist())) == 5


@pytest.mark.parametrize("device", DEVICES)
def test_residual_stream_after_every_layer_run(device):
    eng, W = build(MIXED, device)
    toks = tokens(20, MIXED["vocab"], 5)
    taps, rid = [], eng.replay_open()
    eng.replay_step([(rid, toks, [])], taps=taps)
    _, want = oracle.forward(MIXED, W, toks, return_layers=True)
    assert len(taps) == len(want) == 6                # four layers, two of them twice
    for i, t in enumerate(taps):
        torch.testing.assert_close(t.cpu().double(), want[i], atol=2e-4, rtol=2e-4, msg=f"layer run {i}")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cuts", [[], [1], [40], [2, 2, 3, 2, 17, 2], [11, 1, 1, 12, 13], [5, 7, 12, 16, 1, 15, 2]])
def test_portions_and_token_by_token_decoding(device, dtype, cuts):
    """The same logits whether the prompt comes whole, in portions down to two tokens (cut inside pages of 16
    and inside windows of 9, 17, 21 and 40), or one token at a time."""
    eng, W = build(MIXED, device, dtype)
    toks = tokens_for(MIXED, W, 70, 7, dtype)
    assert rel_err(replay_alone(eng, toks, cuts), *expected(MIXED, W, toks, dtype)) < limit(dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_past_pages_and_windows(device):
    eng, W = build(MIXED, device)
    toks = tokens(120, MIXED["vocab"], 11)
    assert rel_err(replay_alone(eng, toks, [3]), oracle.forward(MIXED, W, toks)) < 2e-4


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_mixed_batches_reused_pages(device, dtype):
    """Up to four live requests, portions beside single tokens, in a pool too small for all of them at once:
    requests end, others take their pages (every pass of a looped layer has planes of its own in them)."""
    eng, W = build(MIXED, device, dtype, blocks=12, slots=4)
    V = MIXED["vocab"]
    reqs = {n: tokens(L, V, 20 + i) for i, (n, L) in enumerate([("a", 50), ("b", 33), ("c", 1), ("d", 47), ("e", 40),
                                                                ("f", 18), ("g", 60)])}
    want = {n: expected(MIXED, W, t, dtype, least=1) for n, t in reqs.items()}
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
        assert rel_err(np.concatenate(got[n]), *want[n]) < limit(dtype), n


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("window", [5, 16, 21])
@pytest.mark.parametrize("decode_from", [0, 3, 30])
def test_the_windows_edge_at_every_place_and_page_border(device, window, decode_from):
    """ONE attention layer and nothing else (no other way for a token to reach a later row), a flat softmax: a
    changed token at place j moves the rows j .. j + window - 1 and no other, neither the rows before it nor the
    row at j + window, whether the rows run as a prompt or are decoded one by one. Pages of 16: the window's far
    edge crosses page borders as the rows go on."""
    cfg = config([attn(heads=2, kv=1, dim=8, window=window, rot=4, scale=0.05)])
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
def test_the_oldest_key_of_the_window_stands_out(device):
    """The key at the window's far edge carries the answer: the first token's key is scaled up so that every row
    that still sees it gives it most of its weight, and the first row that does not falls back to the others.
    The oracle's own weights confirm the jump between the last row inside and the first row outside."""
    window = 23
    cfg = config([attn(heads=1, kv=1, dim=8, window=window, rot=0, scale=1.0)], vocab=30)
    W = oracle.random_weights(cfg, 6)
    toks = [29] + tokens(50, 29, 3)                 # token 29 appears at place 0 only
    # every query likes the direction e0 of the key space; only token 29's key points there, strongly
    W["l0.norm1"] = torch.zeros_like(W["l0.norm1"])
    W["l0.norm1.b"] = torch.ones_like(W["l0.norm1.b"])
    q = torch.zeros(8, cfg["width"])
    q[0] = 0.2
    W["l0.mix.q"] = q.to(torch.bfloat16)
    _, wts = oracle.window_attention(oracle.tanh_norm(W["embed"].double()[toks] * 3.0, {k: v.double() for k, v in W.items()}, "l0.norm1"),
                                     {k: v.double() for k, v in W.items()}, "l0.mix.", cfg["layers"][0]["mixer"], return_weights=True)
    assert float((wts[0, :, 0] > 0).sum()) == window          # the first key is seen by the first ``window`` rows only
    for cuts in ([len(toks)], [window - 2], [2]):
        eng, _ = build(cfg, device, weights=W)
        assert rel_err(replay_alone(eng, toks, cuts), oracle.forward(cfg, W, toks)) < 2e-4, cuts


@pytest.mark.parametrize("device", DEVICES)
def test_a_far_key_that_stands_out(device):
    """One key far back among hundreds carries the answer: with a large score scale single keys dominate the
    softmax rows, so dropping or misplacing one shows. The window holds 280 keys; the last rows are decoded."""
    cfg = config([attn(heads=1, kv=1, dim=16, window=280, rot=8, base=1e5, scale=5.0)], vocab=50)
    eng, W = build(cfg, device, blocks=24)
    toks = tokens(330, cfg["vocab"], 41)
    assert rel_err(replay_alone(eng, toks, [300]), oracle.forward(cfg, W, toks)) < 2e-4
    Wd = {k: v.double() for k, v in W.items()}
    h = oracle.tanh_norm(Wd["embed"][toks] * cfg["embedding"]["scale"], Wd, "l0.norm1")
    _, wts = oracle.window_attention(h, Wd, "l0.mix.", cfg["layers"][0]["mixer"], return_weights=True)
    far = sum(int(float(wts[0, i].max()) > 0.5 and i - int(wts[0, i].argmax()) > 100) for i in range(300, len(toks)))
    assert far >= 3


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens_and_single_token_requests(device):
    eng, W = build(MIXED, device)
    for toks in ([7], [7, 7], tokens(3, MIXED["vocab"], 2)):
        assert rel_err(replay_alone(eng, toks, [len(toks)]), oracle.forward(MIXED, W, toks)) < 2e-4
        assert rel_err(replay_alone(eng, toks, []), oracle.forward(MIXED, W, toks)) < 2e-4


@pytest.mark.parametrize("device", DEVICES)
def test_pool_exhausted_is_an_error_and_leaves_the_engine_usable(device):
    cfg = config([attn(mlp=moe())])
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

    cfg = config([attn(heads=4, kv=2, dim=16, rot=8, mlp=moe(ff=64, shared=64)), attn(), attn(heads=2, kv=1, dim=32, window=50, rot=32, mlp=moe(shared=0))],
                 width=64, vocab=70, loop=(1, 3, 2))
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
    """A Surevik checkpoint directory is found by its config.json, loaded with the checkpoint's tensor names,
    replayed by ``bin/trace_run`` (two requests in one step, a request that ends and one that goes on) and
    answers a question through the command line."""
    from safetensors.torch import save_file

    from llm_consensus_amd import cli
    from llm_consensus_amd.models.loader import load_model
    from llm_consensus_amd.models.registry import resolve

    cfg = config([attn(mlp=moe()), attn(heads=2, kv=1, dim=8, window=6, rot=8), attn(mlp=moe(top=1, shared=0))], width=32, vocab=300, loop=(0, 2, 2))
    W = oracle.random_weights(cfg, 3)
    ck = tmp_path / "surevik"
    ck.mkdir()
    (ck / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in W.items()}, str(ck / "model.safetensors"))
    assert resolve(str(ck)).name == "hybrid"
    m = load_model(str(ck), "cpu", dtype=torch.float32)
    assert [i for i, _ in m.cfg.runs] == [0, 1, 0, 1, 2] and [f for _, f in m.cfg.runs] == [True, False, True, False, False]
    back = config_to_dict(m.cfg)
    assert back["layers"] == cfg["layers"] and back["loop"] == cfg["loop"] and back["residual_mult"] == cfg["residual_mult"]
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

    cfg = config_from_dict(config([attn(mlp=moe(shared=0)), attn(), attn(mlp=moe())], width=24, vocab=80, loop=(1, 3, 2)))
    ck = write_random_hybrid_checkpoint(cfg, str(tmp_path / "ck"), seed=7)
    assert json.loads((ck / "config.json").read_text())["architecture"] == "Surevik"
    a = load_model(str(ck), "cpu", dtype=torch.float32)
    b = HybridModel.random_init(cfg, "cpu", seed=7, dtype=torch.float32)
    assert a.cfg.layers == b.cfg.layers and (a.cfg.loop, a.cfg.residual_mult) == (b.cfg.loop, b.cfg.residual_mult)
    out = []
    for m in (a, b):
        eng = Engine(m, num_kv_blocks=8, block_size=BS, max_batch_seqs=2, state_slots=2, max_model_len=8 * BS,
                     enable_prefix_cache=False, use_graphs=False, pipeline_decode=False)
        out.append(replay_alone(eng, tokens(12, 80, 1), [7]))
    assert np.isfinite(out[0]).all() and np.abs(out[0]).max() > 0
    np.testing.assert_allclose(out[0], out[1], rtol=1e-6, atol=1e-6)


def test_configurations_the_design_does_not_have_are_refused():
    bad = config([attn()])
    bad["layers"][0]["mixer"]["vdim"] = 5
    with pytest.raises(ValueError):
        config_from_dict(bad)
    with pytest.raises(ValueError):
        config_from_dict(config([attn(mlp={"kind": "dense", "ff": 8})]))
    with pytest.raises(ValueError):
        config_from_dict(config([attn(), attn()], loop=(1, 3, 2)))
    with pytest.raises(ValueError):
        config_from_dict(config([{"type": "mingru", "mixer": {"width": 8}, "mlp": None}]))

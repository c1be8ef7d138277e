"""Prefill and decode throughput of the hybrid decoders (Nidozen, Telurax, Surevik, Gizilorn) beside each other and a
Llama-shaped transformer of equal width, depth and head sizes (``bench.py --hybrid``,
``--hybrid-models gizilorn,surevik,telurax,nidozen,llama``). Random weights, synthetic tokens.

Per size: one prompt of ``prompt`` tokens goes through each engine as a single step (prefill
tokens/s), then ``batch`` requests decode ``new`` tokens each from recorded steps (decode tokens/s).
The hybrid stack repeats (attention, minGRU, attention on the first layer's keys, minGRU, gated
linear attention); the Telurax stack alternates mLSTM layers with a gated dense feed-forward and
latent-attention layers (compressed rows of width 128) with a routed feed-forward (32 experts of a
sixteenth of the dense width plus 4 identity experts in 4 groups of which 2 are kept, 4 chosen, a shared
expert of a quarter); the Surevik stack is window attention (the window is the others' chunk) with a routed
feed-forward of the same sizes in every layer (32 clamped gated experts of a sixteenth of the dense width, 4
chosen, a gated shared expert of a quarter), its second and third layer run twice, so that it has as many
layer runs as the others have layers; the Gizilorn stack repeats (attention with mixed heads' weights, the same,
latent attention with rows of its own, latent attention on those rows) over two residual streams, windows of the
others' chunk, compressed rows of width 128 beside a turned key part of 64, a dense xIELU feed-forward in every
layer; the transformer has full causal attention and a SwiGLU feed-forward. Prints one
JSON line. Per-kernel times come from running this under ``rocprofv3 --kernel-trace --stats``.
"""
from __future__ import annotations

import json
import time
from typing import Dict

import numpy as np
import torch

SIZES = {
    # width, layers, heads, kv heads, head dim, ff, chunk
    "1k": dict(width=1024, layers=5, heads=8, kv=2, dim=128, ff=4096, chunk=512, vocab=32000),
    "2k": dict(width=2048, layers=10, heads=16, kv=4, dim=128, ff=8192, chunk=1024, vocab=32000),
    "4k": dict(width=4096, layers=10, heads=32, kv=8, dim=128, ff=14336, chunk=1024, vocab=32000),
}


def hybrid_config(s: dict):
    from .models.hybrid import config_from_dict

    def attn(kv_from=None):
        m = {"heads": s["heads"], "kv_heads": s["kv"], "dim": s["dim"], "vdim": s["dim"], "scale": s["dim"] ** -0.5,
             "mask": {"size": s["chunk"]}, "rot": {"dims": s["dim"] // 2, "base": 10000.0}}
        if kv_from is not None:
            m["kv_from"] = kv_from
        return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": s["ff"]}}
    layers = []
    for i in range(s["layers"]):
        k = i % 5
        if k == 0:
            first = len(layers)
            layers.append(attn())
        elif k == 2:
            layers.append(attn(first))
        elif k in (1, 3):
            layers.append({"type": "mingru", "mixer": {"width": s["width"]}, "mlp": {"kind": "dense", "ff": s["ff"]}})
        else:
            layers.append({"type": "gla", "mixer": {"heads": s["heads"], "dim": s["dim"], "vdim": s["dim"], "tau": 16.0,
                                                     "rank": 64}, "mlp": {"kind": "dense", "ff": s["ff"]}})
    return config_from_dict({"architecture": "Nidozen", "vocab": s["vocab"], "width": s["width"],
                             "norm": {"eps": 1e-5}, "layers": layers}, name="nidozen-bench")


def telurax_config(s: dict):
    from .models.hybrid import config_from_dict

    layers = []
    for i in range(s["layers"]):
        if i % 2 == 0:
            layers.append({"type": "mlstm", "mixer": {"heads": s["heads"], "dim": s["dim"], "vdim": s["dim"], "gate_cap": 15.0},
                           "mlp": {"kind": "dense", "ff": s["ff"]}})
        else:
            layers.append({"type": "latent_attention",
                           "mixer": {"heads": s["heads"], "dim": s["dim"], "vdim": s["dim"], "kv_rank": 128,
                                     "scale": s["dim"] ** -0.5},
                           "mlp": {"kind": "moe", "expert": {"ff": s["ff"] // 16},
                                   "router": {"experts": 32, "identity": 4, "top": 4, "scale": 1.0,
                                              "groups": {"count": 4, "keep": 2}},
                                   "shared": {"ff": s["ff"] // 4}}})
    return config_from_dict({"architecture": "Telurax", "vocab": s["vocab"], "width": s["width"], "norm": {"eps": 1e-5},
                             "embedding": {"scale": 1.0}, "logit_scale": 1.0, "layers": layers}, name="telurax-bench")


def surevik_config(s: dict):
    from .models.hybrid import config_from_dict

    layer = {"type": "attention",
             "mixer": {"heads": s["heads"], "kv_heads": s["kv"], "dim": s["dim"], "vdim": s["dim"], "scale": s["dim"] ** -0.5,
                       "mask": {"size": s["chunk"]}, "rot": {"dims": s["dim"] // 2, "base": 10000.0}},
             "mlp": {"kind": "moe", "expert": {"ff": s["ff"] // 16, "limit": 7.0}, "router": {"experts": 32, "top": 4},
                     "shared": {"ff": s["ff"] // 4, "limit": 7.0}}}
    return config_from_dict({"architecture": "Surevik", "vocab": s["vocab"], "width": s["width"], "norm": {"eps": 1e-6},
                             "embedding": {"scale": s["width"] ** 0.5}, "residual_mult": 0.5,
                             "layers": [layer] * (s["layers"] - 2), "loop": {"start": 1, "stop": 3, "times": 2}},
                            name="surevik-bench")


def gizilorn_config(s: dict):
    from .models.hybrid import config_from_dict

    ff = {"kind": "dense", "ff": s["ff"]}
    attn = {"type": "attention",
            "mixer": {"heads": s["heads"], "kv_heads": s["kv"], "dim": s["dim"], "vdim": s["dim"], "scale": s["dim"] ** -0.5,
                      "softcap": 50.0, "mask": {"size": s["chunk"]}, "rot": {"dims": s["dim"] // 2, "base": 10000.0}}, "mlp": ff}

    def latent(kv_from=None):
        m = {"heads": s["heads"], "dim": s["dim"], "rot_dim": 64, "vdim": s["dim"], "kv_rank": 128,
             "scale": (s["dim"] + 64) ** -0.5, "mask": {"size": s["chunk"]}, "rot": {"dims": 64, "base": 1e6}}
        if kv_from is not None:
            m["kv_from"] = kv_from
        return {"type": "latent_attention", "mixer": m, "mlp": ff}
    layers = []
    for i in range(s["layers"]):
        k = i % 4
        if k == 2:
            own = i
        layers.append(attn if k < 2 else latent(None if k == 2 else own))
    return config_from_dict({"architecture": "Gizilorn", "vocab": s["vocab"], "width": s["width"], "norm": {"eps": 1e-5},
                             "streams": 2, "layers": layers}, name="gizilorn-bench")


def transformer_config(s: dict):
    from .models.config import ModelConfig

    return ModelConfig("llama-bench", s["vocab"], s["width"], s["layers"], s["heads"], s["kv"], s["dim"], s["ff"],
                       max_position=8192)


def _measure(model, prompt: int, batch: int, new: int, steps: int, warmup: int, phases=("prefill", "decode")) -> Dict[str, float]:
    from ._native import core
    from .engine.engine import Engine

    blocks = (prompt // 64 + 2) + batch * ((64 + new) // 64 + 2) + 8
    eng = Engine(model, num_kv_blocks=blocks, block_size=64, max_batch_seqs=max(batch, 4), max_model_len=8192,
                 enable_prefix_cache=False, name="bench")
    vocab = model.cfg.vocab_size
    rng = np.random.default_rng(0)
    times = []
    out: Dict[str, float] = {}
    for i in range(warmup + steps if "prefill" in phases else 0):
        toks = rng.integers(0, vocab, prompt).tolist()
        rid = eng.replay_open()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.replay_step([(rid, toks, [prompt - 1])])
        torch.cuda.synchronize()
        if i >= warmup:
            times.append(time.perf_counter() - t0)
        eng.replay_close(rid)
    if times:
        out = {"prefill_tokens_per_s": prompt / float(np.median(times)), "prefill_ms": 1e3 * float(np.median(times))}
    if "decode" not in phases:
        return out
    p = core.SamplingParams()
    p.temperature, p.max_new_tokens, p.ignore_eos = 0.8, new, True
    dec = []
    for i in range(2):          # the first pass records the decode graphs
        for b in range(batch):
            p.seed = 100 * i + b
            eng.submit(rng.integers(0, vocab, 64).tolist(), params=p)
        while eng.sched.num_running < batch and eng.step():
            pass
        torch.cuda.synchronize()
        t0, n0 = time.perf_counter(), eng.metrics.snapshot().get("decode.tokens", 0)
        eng.run_until_done()
        torch.cuda.synchronize()
        dec.append((eng.metrics.snapshot().get("decode.tokens", 0) - n0) / (time.perf_counter() - t0))
    out["decode_tokens_per_s"] = dec[-1]
    out["decode_ms_per_step"] = 1e3 * batch / dec[-1]
    return out


def run(a) -> int:
    from .models.hybrid import HybridModel
    from .models.transformer import TransformerModel

    dev = "cuda:0"
    torch.cuda.set_device(0)
    res = {"metric": "prefill / decode tokens per second, hybrid decoders beside a Llama-shaped transformer of equal size",
           "dtype": "bf16", "data": "synthetic tokens, random-init weights", "n_gpus": 1,
           "prompt": a.hybrid_prompt, "batch": a.hybrid_batch, "new_tokens": a.hybrid_new, "sizes": {}}
    for name in [n for n in a.hybrid_sizes.split(",") if n]:
        s = SIZES[name]
        row = {}
        phases = tuple(x for x in a.hybrid_phases.split(",") if x)
        for kind in [k for k in a.hybrid_models.split(",") if k]:
            if kind == "nidozen":
                model = HybridModel.random_init(hybrid_config(s), dev, seed=1)
            elif kind == "telurax":
                model = HybridModel.random_init(telurax_config(s), dev, seed=1)
            elif kind == "surevik":
                model = HybridModel.random_init(surevik_config(s), dev, seed=1)
            elif kind == "gizilorn":
                model = HybridModel.random_init(gizilorn_config(s), dev, seed=1)
            else:
                model = TransformerModel.random_init(transformer_config(s), dev, seed=1)
            row[kind] = _measure(model, a.hybrid_prompt, a.hybrid_batch, a.hybrid_new, a.steps, a.warmup, phases)
            row[kind]["weight_gb"] = model.weight_bytes() / 1e9
            del model
            torch.cuda.empty_cache()
        for ph in ("prefill", "decode"):
            k = ph + "_tokens_per_s"
            if all(k in row.get(m, {}) for m in ("nidozen", "llama")):
                row[ph + "_ratio"] = row["nidozen"][k] / row["llama"][k]
            for mine, others in (("telurax", ("nidozen", "llama")), ("surevik", ("telurax", "nidozen", "llama")),
                                 ("gizilorn", ("surevik", "telurax", "nidozen", "llama"))):
                for other in others:
                    if all(k in row.get(m, {}) for m in (mine, other)):
                        row[f"{ph}_{mine}_over_{other}"] = row[mine][k] / row[other][k]
        res["sizes"][name] = row
    print(json.dumps(res))
    if a.out:
        with open(a.out, "w") as f:
            f.write(json.dumps(res) + "\n")
    return 0

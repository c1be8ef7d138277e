"""Plain, slow implementation of the Surevik decoder, written from its equations.

One function per mechanism, float64 throughout, whole sequences at once, no cache and no batching.
The tests compare the engine against it; nothing here is imported by the package and nothing of
the package is imported here.

Weights come as a dict name -> tensor with the checkpoint's names: ``embed``, ``final.norm`` (with
``.b`` and ``.alpha``), ``loop.in`` when layers are looped, and per layer i ``l<i>.norm1``, ``l<i>.norm2``,
``l<i>.mix.{q,k,o}``, ``l<i>.mlp.{router, e<j>.{gate,up,down}, shared.{gate,up,down,sg}}``. The
configuration is the parsed ``config.json`` (a dict).
"""
import math

import torch

F = torch.float64
GATE_SLOPE = 1.702


def tanh_norm(x, W, name):
    """Dynamic Tanh: no statistics of x, a scalar slope inside the tanh, a weight and a bias outside."""
    return torch.tanh(W[name + ".alpha"] * x) * W[name] + W[name + ".b"]


def turn_pairs(x, dims, base):
    """x [T, heads, D]: coordinates (2i, 2i + 1), i < dims / 2, of the row at position p turn by the
    angle p * base^(-2i / dims); coordinates from ``dims`` on pass."""
    out = x.clone()
    for p in range(x.shape[0]):
        for i in range(dims // 2):
            a = p * base ** (-2.0 * i / dims)
            u, v = x[p, :, 2 * i], x[p, :, 2 * i + 1]
            out[p, :, 2 * i] = u * math.cos(a) - v * math.sin(a)
            out[p, :, 2 * i + 1] = v * math.cos(a) + u * math.sin(a)
    return out


def window_attention(h, W, p, m, return_weights=False):
    """Grouped heads; the values are the keys as projected (before they turn); row i sees the rows
    i - size + 1 .. i."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    rot = m.get("rot") or {}
    size = (m.get("mask") or {}).get("size", 0)
    q = (h @ W[p + "q"].T).view(T, H, D)
    k = (h @ W[p + "k"].T).view(T, G, D)
    v = k
    q, k = turn_pairs(q, rot.get("dims", 0), rot.get("base", 10000.0)), turn_pairs(k, rot.get("dims", 0), rot.get("base", 10000.0))
    out = torch.zeros(T, H, D, dtype=F)
    weights = torch.zeros(H, T, T, dtype=F)
    for i in range(T):
        lo = max(0, i - size + 1) if size else 0
        for hh in range(H):
            g = hh // (H // G)
            s = torch.softmax((k[lo:i + 1, g] @ q[i, hh]) * m["scale"], 0)
            out[i, hh] = s @ v[lo:i + 1, g]
            weights[hh, i, lo:i + 1] = s
    y = out.reshape(T, H * D) @ W[p + "o"].T
    return (y, weights) if return_weights else y


def gated_unit(h, W, p, limit):
    """One expert: the gate is capped from above only, the other branch from both sides."""
    g = torch.clamp(h @ W[p + "gate"].T, max=limit)
    u = torch.clamp(h @ W[p + "up"].T, -limit, limit)
    return (g * torch.sigmoid(GATE_SLOPE * g) * (u + 1.0)) @ W[p + "down"].T


def choose(h, W, p, r):
    """(chosen experts [T, top], their scores [T, top]): independent sigmoid scores, the largest win."""
    s = torch.sigmoid(h @ W[p + "router"].T)
    ids = torch.argsort(s, dim=-1, descending=True, stable=True)[:, :r["top"]]
    return ids, s.gather(1, ids)


def choice_margin(h, W, p, r):
    """Per token: how far the last chosen expert's score lies above the best one not chosen (inf when all are chosen)."""
    s = torch.sort(torch.sigmoid(h @ W[p + "router"].T), dim=-1, descending=True).values
    if r["top"] >= s.shape[1]:
        return torch.full((h.shape[0],), math.inf, dtype=F)
    return s[:, r["top"] - 1] - s[:, r["top"]]


def routed_ff(h, W, p, mlp, weight_on_output=False):
    """Every token runs its ``top`` best experts on ITS INPUT TIMES THE SCORE (``weight_on_output``: the
    other, wrong order, for tests that show the two differ), plus a shared expert under a scalar gate."""
    ids, sc = choose(h, W, p, mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(ids[t].tolist(), sc[t]):
            if weight_on_output:
                out[t] += w * gated_unit(h[t:t + 1], W, f"{p}e{e}.", mlp["expert"]["limit"])[0]
            else:
                out[t] += gated_unit(w * h[t:t + 1], W, f"{p}e{e}.", mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        out = out + torch.sigmoid(h @ W[p + "shared.sg"].T) * gated_unit(h, W, p + "shared.", mlp["shared"]["limit"])
    return out


def layer_runs(cfg):
    """[(layer, starts a pass of the loop)] in the order the layers run."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b = loop["start"], loop["stop"]
    runs = [(i, False) for i in range(a)]
    for _ in range(loop.get("times", 1)):
        runs += [(i, i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def forward(cfg, W, tokens, return_layers=False, return_margins=False):
    """Logits [T, vocab] (float64) of a whole sequence; with ``return_layers`` also the stream after every layer
    run; with ``return_margins`` also, per token, the smallest ``choice_margin`` of all routers it went through."""
    W = {k: v.to(F) for k, v in W.items()}
    mult = cfg.get("residual_mult", 1.0)
    x0 = W["embed"][torch.as_tensor(tokens, dtype=torch.long)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    x, taps = x0, []
    margins = torch.full((x0.shape[0],), math.inf, dtype=F)
    for i, first in layer_runs(cfg):
        L, p = cfg["layers"][i], f"l{i}."
        if first:
            x = torch.cat([x, x0], 1) @ W["loop.in"].T
        x = x + mult * window_attention(tanh_norm(x, W, p + "norm1"), W, p + "mix.", L["mixer"])
        if L.get("mlp") is not None:
            h = tanh_norm(x, W, p + "norm2")
            margins = torch.minimum(margins, choice_margin(h, W, p + "mlp.", L["mlp"]["router"]))
            x = x + mult * routed_ff(h, W, p + "mlp.", L["mlp"])
        taps.append(x)
    logits = tanh_norm(x, W, "final.norm") @ W["embed"].T
    if return_margins:
        return logits, margins
    return (logits, taps) if return_layers else logits


def random_weights(cfg, seed=0):
    """bf16 tensors under the checkpoint's names: matrices N(0, 1 / fan_in), norm weights near one with
    small biases, slopes near 0.7, an embedding whose rows have unit scale after ``embedding.scale``."""
    gen = torch.Generator().manual_seed(seed)
    d, V = cfg["width"], cfg["vocab"]
    W = {}

    def mat(n, k, s=1.0):
        return (torch.randn(n, k, generator=gen) * s * k ** -0.5).to(torch.bfloat16)

    def norm(name):
        W[name] = (1.0 + 0.2 * torch.randn(d, generator=gen)).to(torch.bfloat16)
        W[name + ".b"] = (0.1 * torch.randn(d, generator=gen)).to(torch.bfloat16)
        W[name + ".alpha"] = (0.7 + 0.1 * torch.randn((), generator=gen)).to(torch.bfloat16)
    W["embed"] = (torch.randn(V, d, generator=gen) / (cfg.get("embedding") or {}).get("scale", 1.0)).to(torch.bfloat16)
    if cfg.get("loop"):
        W["loop.in"] = mat(d, 2 * d, 1.4)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        norm(p + "norm1")
        W[p + "mix.q"], W[p + "mix.k"] = mat(m["heads"] * m["dim"], d, 2.0), mat(m["kv_heads"] * m["dim"], d, 2.0)
        W[p + "mix.o"] = mat(d, m["heads"] * m["dim"])
        mlp = L.get("mlp")
        if mlp is None:
            continue
        norm(p + "norm2")
        f = p + "mlp."
        W[f + "router"] = mat(mlp["router"]["experts"], d, 4.0)
        for e in range(mlp["router"]["experts"]):
            W[f + f"e{e}.gate"], W[f + f"e{e}.up"] = mat(mlp["expert"]["ff"], d, 2.0), mat(mlp["expert"]["ff"], d, 2.0)
            W[f + f"e{e}.down"] = mat(d, mlp["expert"]["ff"])
        if mlp.get("shared"):
            n = mlp["shared"]["ff"]
            W[f + "shared.gate"], W[f + "shared.up"], W[f + "shared.down"] = mat(n, d, 2.0), mat(n, d, 2.0), mat(d, n)
            W[f + "shared.sg"] = mat(1, d, 2.0)
    norm("final.norm")
    return W

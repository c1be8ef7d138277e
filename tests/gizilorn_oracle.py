"""Plain, slow implementation of the Gizilorn decoder, written from its equations.

One function per mechanism, float64 throughout, whole sequences at once, no cache and no batching.
The tests compare the engine against it; nothing here is imported by the package and nothing of
the package is imported here.

Weights come as a dict name -> tensor with the checkpoint's names: ``embed``, ``embed.norm``,
``final.norm``, ``head``, and per layer i ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.hc<q>.{in,out,mix}``,
``l<i>.mix.*`` (attention: q, k, v with ``.b``, talk, o; latent attention: q, dkv, dkv.norm, uk, uv,
g, o) and ``l<i>.mlp.{up,down}`` with ``.b`` and ``act``. The configuration is the parsed
``config.json`` (a dict).
"""
import math

import torch

F = torch.float64


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def turn(x, pos, dims, base, layout, sign=1.0):
    """x [T, heads, D]: the first ``dims`` coordinates of every head of row t turn by ``sign * pos[t]``
    times the pair's frequency base^(-2i / dims). Pairs: (i, i + dims/2) for ``halves``, (2i, 2i + 1) for
    ``pairs``; coordinates from ``dims`` on pass."""
    out = x.clone()
    for t in range(x.shape[0]):
        for i in range(dims // 2):
            a = sign * pos[t] * base ** (-2.0 * i / dims)
            ia, ib = (i, i + dims // 2) if layout == "halves" else (2 * i, 2 * i + 1)
            u, v = x[t, :, ia], x[t, :, ib]
            out[t, :, ia] = u * math.cos(a) - v * math.sin(a)
            out[t, :, ib] = v * math.cos(a) + u * math.sin(a)
    return out


def sink_softmax(s):
    """Softmax over the last axis with a silent extra entry of score zero: the weights sum to less than one."""
    m = torch.clamp(s.max(-1, keepdim=True).values, min=0.0)
    e = torch.exp(s - m)
    return e / (torch.exp(-m) + e.sum(-1, keepdim=True))


def talking_attention(h, W, p, m, return_weights=False):
    """Grouped heads with biased projections; keys and queries turn over their first rot.dims coordinates, the
    values over their whole width by their own position; capped scores; a window; a sink in the softmax; the
    heads' weights are mixed by a matrix before they meet the values; the result turns back by the row's position."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot, size, cap = m["rot"], m["mask"]["size"], m["softcap"]
    pos = list(range(T))
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, D)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, D)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).view(T, G, Dv)
    q, k = turn(q, pos, rot["dims"], rot["base"], "halves"), turn(k, pos, rot["dims"], rot["base"], "halves")
    v = turn(v, pos, Dv, rot["base"], "halves")
    weights = torch.zeros(H, T, T, dtype=F)
    for i in range(T):
        lo = max(0, i - size + 1)
        for hh in range(H):
            s = (k[lo:i + 1, hh // (H // G)] @ q[i, hh]) * m["scale"]
            weights[hh, i, lo:i + 1] = sink_softmax(cap * torch.tanh(s / cap))
    mixed = torch.einsum("hg,gij->hij", W[p + "talk"], weights)
    out = torch.zeros(T, H, Dv, dtype=F)
    for hh in range(H):
        out[:, hh] = mixed[hh] @ v[:, hh // (H // G)]
    out = turn(out, pos, Dv, rot["base"], "halves", sign=-1.0)
    y = out.reshape(T, H * Dv) @ W[p + "o"].T
    return (y, weights) if return_weights else y


def latent_rows(h, W, p, m, eps):
    """What a latent-attention layer with a down-projection of its own leaves for the keys: the normed compressed
    row [T, kv_rank] and the one turned key part [T, rot_dim] that all heads share."""
    R, rd = m["kv_rank"], m["rot_dim"]
    down = h @ W[p + "dkv"].T
    c = rms_norm(down[:, :R], W[p + "dkv.norm"], eps)
    kr = turn(down[:, R:].reshape(-1, 1, rd), list(range(h.shape[0])), m["rot"]["dims"], m["rot"]["base"], "pairs")
    return c, kr[:, 0]


def latent_attention(h, W, p, m, rows, return_weights=False):
    """Heads whose keys and values are linear maps of the compressed rows ``rows`` = (c, turned key part), this
    layer's own or another's; a query head is [dim plain | rot_dim turned]; a window; a plain softmax; the heads'
    outputs are gated coordinate by coordinate."""
    T = h.shape[0]
    H, D, rd, Dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    size = m["mask"]["size"]
    c, kr = rows
    q = (h @ W[p + "q"].T).view(T, H, D + rd)
    qr = turn(q[:, :, D:], list(range(T)), m["rot"]["dims"], m["rot"]["base"], "pairs")
    kn = (c @ W[p + "uk"].T).view(T, H, D)
    v = (c @ W[p + "uv"].T).view(T, H, Dv)
    out = torch.zeros(T, H, Dv, dtype=F)
    weights = torch.zeros(H, T, T, dtype=F)
    for i in range(T):
        lo = max(0, i - size + 1)
        for hh in range(H):
            s = (kn[lo:i + 1, hh] @ q[i, hh, :D] + kr[lo:i + 1] @ qr[i, hh]) * m["scale"]
            w = torch.softmax(s, 0)
            out[i, hh] = w @ v[lo:i + 1, hh]
            weights[hh, i, lo:i + 1] = w
    y = (out.reshape(T, H * Dv) * torch.sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T
    return (y, weights) if return_weights else y


def xielu(z, a):
    """Quadratic above zero, a saturating exponential below; both branches have the slope 1/2 at zero."""
    sp = torch.nn.functional.softplus
    pos = sp(a[0]) * z * z + z / 2
    neg = (0.5 + sp(a[1])) * (torch.expm1(torch.clamp(z, max=0.0)) - z) + z / 2
    return torch.where(z > 0, pos, neg)


def feed_forward(h, W, p):
    return xielu(h @ W[p + "up"].T + W[p + "up.b"], W[p + "act"]) @ W[p + "down"].T + W[p + "down.b"]


def forward(cfg, W, tokens, return_layers=False):
    """Logits [T, vocab] (float64) of a whole sequence; with ``return_layers`` also the sum of the streams after
    every layer."""
    W = {k: v.to(F) for k, v in W.items()}
    eps, S = cfg["norm"]["eps"], cfg["streams"]
    x0 = rms_norm(W["embed"][torch.as_tensor(tokens, dtype=torch.long)], W["embed.norm"], eps)
    xs = [x0.clone() for _ in range(S)]
    taps, kept = [], {}

    def sublayer(pre, norm, fn):
        """The streams are read through the weights ``in``, and written: every new stream is a mixture of the old
        ones (``mix[from, to]``) plus its own share (``out``) of the sublayer's result."""
        u = sum(W[pre + "in"][s] * xs[s] for s in range(S))
        y = fn(rms_norm(u, W[norm], eps))
        new = [sum(W[pre + "mix"][s, t] * xs[s] for s in range(S)) + W[pre + "out"][t] * y for t in range(S)]
        xs[:] = new
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        if L["type"] == "attention":
            sublayer(p + "hc1.", p + "norm1", lambda h: talking_attention(h, W, p + "mix.", m))
        else:
            def mixer(h):
                src = m.get("kv_from")
                if src is None:
                    kept[i] = latent_rows(h, W, p + "mix.", m, eps)
                return latent_attention(h, W, p + "mix.", m, kept[i if src is None else src])
            sublayer(p + "hc1.", p + "norm1", mixer)
        if L.get("mlp") is not None:
            sublayer(p + "hc2.", p + "norm2", lambda h: feed_forward(h, W, p + "mlp."))
        taps.append(sum(xs))
    logits = rms_norm(sum(xs), W["final.norm"], eps) @ W["head"].T
    return (logits, taps) if return_layers else logits


def random_weights(cfg, seed=0):
    """bf16 tensors under the checkpoint's names: matrices N(0, 1 / fan_in) (queries and keys larger, so that the
    softmax is not flat), norm weights near one, stream weights that keep the streams apart."""
    gen = torch.Generator().manual_seed(seed)
    d, V, S = cfg["width"], cfg["vocab"], cfg["streams"]
    W = {}

    def mat(n, k, s=1.0):
        return (torch.randn(n, k, generator=gen) * s * k ** -0.5).to(torch.bfloat16)

    def vec(n, mean=0.0, s=0.1):
        return (mean + s * torch.randn(n, generator=gen)).to(torch.bfloat16)
    W["embed"], W["embed.norm"] = mat(V, d, d ** 0.5), vec(d, 1.0, 0.2)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        subs = ["1"] + (["2"] if L.get("mlp") is not None else [])
        for q in subs:
            W[p + "norm" + q] = vec(d, 1.0, 0.2)
            W[p + f"hc{q}.in"] = vec(S, 1.0 / S, 0.3)
            W[p + f"hc{q}.out"] = vec(S, 0.8, 0.4)
            W[p + f"hc{q}.mix"] = (torch.eye(S) + 0.25 * torch.randn(S, S, generator=gen)).to(torch.bfloat16)
        x = p + "mix."
        if L["type"] == "attention":
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            W[x + "q"], W[x + "k"], W[x + "v"] = mat(H * D, d, 2.0), mat(G * D, d, 2.0), mat(G * Dv, d)
            W[x + "q.b"], W[x + "k.b"], W[x + "v.b"] = vec(H * D, s=0.3), vec(G * D, s=0.3), vec(G * Dv, s=0.3)
            W[x + "talk"] = (torch.eye(H) + 0.4 * torch.randn(H, H, generator=gen)).to(torch.bfloat16)
            W[x + "o"] = mat(d, H * Dv)
        else:
            H, D, rd, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            W[x + "q"] = mat(H * (D + rd), d, 2.0)
            if m.get("kv_from") is None:
                W[x + "dkv"], W[x + "dkv.norm"] = mat(R + rd, d, 2.0), vec(R, 1.0, 0.2)
            W[x + "uk"], W[x + "uv"] = mat(H * D, R, 2.0), mat(H * Dv, R)
            W[x + "g"], W[x + "o"] = mat(H * Dv, d, 2.0), mat(d, H * Dv)
        if L.get("mlp") is not None:
            f, n = p + "mlp.", L["mlp"]["ff"]
            W[f + "up"], W[f + "up.b"] = mat(n, d, 1.5), vec(n, s=0.3)
            W[f + "down"], W[f + "down.b"] = mat(d, n), vec(d, s=0.1)
            W[f + "act"] = vec(2, 0.3, 0.5)
    W["final.norm"], W["head"] = vec(d, 1.0, 0.2), mat(V, d)
    return W

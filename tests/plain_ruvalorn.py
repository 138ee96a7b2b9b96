"""Ruvalorn, plain and slow: float64, one function per mechanism, whole sequences at once.

Written from the design's equations and sharing nothing with the engine: no cache, no pages,
no batching.  ``weights`` maps tensor names to float64 tensors, ``cfg`` is the dictionary of
``config.json``.  Notation: ``n`` tokens, width ``w``; a linear map stored ``[out, in]`` is applied
as ``x @ W.T``.
"""
import torch


def unit_rms(x, eps):
    """``x / sqrt(mean(x^2) + eps)`` over the last axis."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def norm(x, weight, eps):
    """The weight is stored around zero: the scale is ``1 + weight``."""
    return unit_rms(x, eps) * (1.0 + weight)


def silu(z):
    return z * torch.sigmoid(z)


def rotate(x, positions, dims, base):
    """``x [n, heads, d]``: of every head the first ``dims`` channels turn, channel ``i`` with channel
    ``i + dims/2`` by the angle ``position * base^(-2i/dims)``; the rest is left alone."""
    if not dims:
        return x
    half = dims // 2
    out = x.clone()
    for i in range(half):
        angle = positions.double() * (float(base) ** (-2.0 * i / dims))
        c, s = torch.cos(angle)[:, None], torch.sin(angle)[:, None]
        u, v = x[..., i], x[..., i + half]
        out[..., i] = u * c - v * s
        out[..., i + half] = v * c + u * s
    return out


def gate_heads(out, gate_logits):
    """``out [n, heads, d]`` times one sigmoid per token and head."""
    return out * torch.sigmoid(gate_logits)[:, :, None]


def visible(i, j, window):
    """Whether the query at position i reads the key at position j."""
    return 0 <= i - j and (window is None or i - j < window)


def attention(h, weights, prefix, m):
    """The mixer: queries and keys with biases, the values are the keys as projected (before they
    turn), a window of ``mask.size`` positions, one sigmoid gate per head on the heads' outputs."""
    n = h.shape[0]
    heads, groups, d = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ weights[prefix + "q"].T + weights[prefix + "q.b"]).view(n, heads, d)
    k = (h @ weights[prefix + "k"].T + weights[prefix + "k.b"]).view(n, groups, d)
    values = k.clone()
    rot = m.get("rot") or {}
    positions = torch.arange(n)
    q = rotate(q, positions, rot.get("dims", 0), rot.get("base", 1.0))
    k = rotate(k, positions, rot.get("dims", 0), rot.get("base", 1.0))
    window = (m.get("mask") or {}).get("size")
    out = torch.zeros(n, heads, d, dtype=h.dtype)
    for head in range(heads):
        g = head // (heads // groups)
        for i in range(n):
            seen = [j for j in range(n) if visible(i, j, window)]
            scores = (k[seen, g] @ q[i, head]) * m["scale"]
            p = torch.softmax(scores, 0)
            out[i, head] = p @ values[seen, g]
    out = gate_heads(out, h @ weights[prefix + "g"].T)
    return out.reshape(n, heads * d) @ weights[prefix + "o"].T


def gated_ffn(h, weights, prefix):
    return (silu(h @ weights[prefix + "gate"].T) * (h @ weights[prefix + "up"].T)) @ weights[prefix + "down"].T


def route(h, weights, prefix, router):
    """Per token: the chosen outputs of the router and their weights.  Scores are a softmax over all
    outputs; the choice is made on score + correction, among the outputs of the ``keep`` groups of
    neighbours whose best choice value is largest; the weight is the score itself times a constant."""
    z = h @ weights[prefix + "router"].T
    s = torch.softmax(z, -1)
    choice = s + weights[prefix + "correction"]
    total = z.shape[-1]
    groups = router.get("groups") or {"count": 1, "keep": 1}
    per = total // groups["count"]
    picks = []
    for t in range(h.shape[0]):
        best = sorted(range(groups["count"]), key=lambda g: (-float(choice[t, g * per:(g + 1) * per].max()), g))
        allowed = [e for g in best[:groups["keep"]] for e in range(g * per, (g + 1) * per)]
        chosen = sorted(allowed, key=lambda e: (-float(choice[t, e]), e))[:router["top"]]
        picks.append([(e, s[t, e] * router["scale"]) for e in chosen])
    return picks


def mixture(h, weights, prefix, mlp):
    router = mlp["router"]
    real = router["experts"]
    out = torch.zeros_like(h)
    for t, chosen in enumerate(route(h, weights, prefix, router)):
        for e, weight in chosen:
            if e >= real:                       # the last outputs of the router stand for the input itself
                out[t] += weight * h[t]
            else:
                out[t] += weight * gated_ffn(h[t:t + 1], weights, f"{prefix}e{e}.")[0]
    if mlp.get("shared"):
        out = out + gated_ffn(h, weights, prefix + "shared.")
    return out


def layer_runs(cfg):
    """``(layer, pass or None)`` in the order they run: the layers ``start .. stop-1`` of the loop
    are run ``times`` times in a row."""
    loop = cfg.get("loop")
    n = len(cfg["layers"])
    if not loop:
        return [(i, None) for i in range(n)]
    runs = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(i, t) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, None) for i in range(loop["stop"], n)]


def forward(ids, weights, cfg, keep_layers=False):
    """Logits ``[n, vocab]`` (and the stream after every layer run)."""
    eps = cfg["norm"]["eps"]
    x = weights["embed"][torch.tensor(ids)]
    after = []
    loop = cfg.get("loop")
    started = set()
    for i, t in layer_runs(cfg):
        if t is not None and t not in started:          # once a pass, right before its first layer
            started.add(t)
            x = x + weights["loop.step"][t]
        layer, p = cfg["layers"][i], f"l{i}."
        assert layer["type"] == "attention"
        x = x + attention(norm(x, weights[p + "norm1"], eps), weights, p + "mix.", layer["mixer"])
        mlp = layer.get("mlp")
        if mlp is not None:
            h = norm(x, weights[p + "norm2"], eps)
            x = x + (gated_ffn(h, weights, p + "mlp.") if mlp["kind"] == "dense" else mixture(h, weights, p + "mlp.", mlp))
        after.append(x.clone())
    if loop and loop["start"] == loop["stop"]:
        raise ValueError("a loop over no layer")
    logits = norm(x, weights["final.norm"], eps) @ weights["head"].T
    return (logits, torch.stack(after)) if keep_layers else logits

"""A plain, slow implementation of the Vivevik decoder, one function per mechanism,
in float64 on the CPU.  It shares no code with the engine: tensors come as a
dictionary by file name, the configuration as the dictionary of ``config.json``.

Notation: ``h [T, W]`` the rows of one sequence, positions ``0 .. T-1``.
"""
from __future__ import annotations

import torch

F = torch.float64


def layer_norm(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def squared_relu_mlp(h, up, down):
    return (torch.relu(h @ up.T) ** 2) @ down.T


def gla_decay(h, a1, a2, a2_bias, tau):
    """Per key channel: ``sigmoid(z) ** (1 / tau)`` with ``z`` from a low-rank projection."""
    z = (h @ a1.T) @ a2.T + a2_bias
    return torch.sigmoid(z) ** (1.0 / tau)


def gla_recurrence(q, k, v, alpha, state=None):
    """``q, k, alpha [T, H, D]``, ``v [T, H, E]``; ``state [H, D, E]`` or None for zero.
    Token by token: ``S = alpha_t[:, None] * S + k_t v_t^T``, ``o_t = S^T q_t``.
    Returns ``o [T, H, E]`` and the state after the last token."""
    T, H, D = q.shape
    E = v.shape[-1]
    S = torch.zeros(H, D, E, dtype=q.dtype) if state is None else state.clone()
    out = torch.zeros(T, H, E, dtype=q.dtype)
    for t in range(T):
        S = alpha[t].unsqueeze(-1) * S + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        out[t] = torch.einsum("hde,hd->he", S, q[t])
    return out, S


def gla_mixer(h, p, sizes, eps, state=None):
    H, D, E, tau = sizes["heads"], sizes["dim"], sizes["vdim"], sizes["tau"]
    T = h.shape[0]
    q = (h @ p["q"].T).view(T, H, D) * D ** -0.5
    k = (h @ p["k"].T).view(T, H, D)
    v = (h @ p["v"].T).view(T, H, E)
    alpha = gla_decay(h, p["a1"], p["a2"], p["a2.b"], tau).view(T, H, D)
    o, S = gla_recurrence(q, k, v, alpha, state)
    o = rms_norm(o, p["norm"], eps).reshape(T, H * E)
    gate = h @ p["g"].T
    return (o * gate * torch.sigmoid(gate)) @ p["o"].T, S


def visible(i, j, size, keep_first):
    """Whether the query at position ``i`` sees the key at position ``j``."""
    return j <= i and (i - j < size or j < keep_first)


def sink_attention(q, k, v, sink, scale, size, keep_first, q_positions=None):
    """``q [T, H, D]``, ``k [S, G, D]``, ``v [S, G, E]``, ``sink [H]``.  The softmax's
    denominator holds ``exp(sink_h)`` beside the visible keys' terms; the sink has no value.
    ``q_positions``: positions of the queries among the keys (default: the last ``T``)."""
    T, H, D = q.shape
    S, G, E = v.shape
    if q_positions is None:
        q_positions = list(range(S - T, S))
    out = torch.zeros(T, H, E, dtype=q.dtype)
    for t, i in enumerate(q_positions):
        js = torch.tensor([j for j in range(S) if visible(i, j, size, keep_first)])
        for hd in range(H):
            g = hd // (H // G)
            s = (k[js, g] @ q[t, hd]) * scale
            m = torch.maximum(s.max(), sink[hd])
            e = torch.exp(s - m)
            den = e.sum() + torch.exp(sink[hd] - m)
            out[t, hd] = (e @ v[js, g]) / den
    return out


def attention_keys_values(h, p, sizes, eps):
    """The keys (after their norm over the whole projection) and values a layer keeps."""
    T = h.shape[0]
    G, D, E = sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    k = rms_norm(h @ p["k"].T, p["k.norm"], eps).view(T, G, D)
    v = (h @ p["v"].T).view(T, G, E)
    return k, v


def attention_mixer(h, p, sizes, eps, k, v):
    """``k, v``: all keys and values of the sequence so far (this layer's own or another's)."""
    T = h.shape[0]
    H, D, E = sizes["heads"], sizes["dim"], sizes["vdim"]
    q = rms_norm(h @ p["q"].T, p["q.norm"], eps).view(T, H, D)
    mask = sizes.get("mask") or {}
    size = mask.get("size", 1 << 60)
    o = sink_attention(q, k, v, p["sink"], sizes["scale"], size, mask.get("keep_first", 0))
    return o.reshape(T, H * E) @ p["o"].T


def _layer_tensors(tensors, i, part):
    prefix = f"l{i}.{part}."
    return {n[len(prefix):]: t.to(F) for n, t in tensors.items() if n.startswith(prefix)}


def forward(token_ids, tensors, config, memory=None, return_layers=False):
    """Logits ``[T, vocab]`` of ``token_ids`` that follow what ``memory`` holds (None: a new
    sequence).  ``memory`` is a dictionary the caller keeps between calls: per layer the
    recurrent state or the keys and values so far."""
    eps = config["norm"]["eps"]
    memory = {} if memory is None else memory
    x = tensors["embed"].to(F)[torch.as_tensor(token_ids, dtype=torch.long)]
    T = x.shape[0]
    layers_out = []
    for i, layer in enumerate(config["layers"]):
        sizes = layer["mixer"]
        p = _layer_tensors(tensors, i, "mix")
        if layer["type"] == "gla":
            y, memory[i] = gla_mixer(x, p, sizes, eps, memory.get(i))
        elif layer["type"] == "attention":
            src = sizes.get("kv_from")
            if src is None:
                k, v = attention_keys_values(x, p, sizes, eps)
                if i in memory:
                    k, v = torch.cat([memory[i][0], k]), torch.cat([memory[i][1], v])
                memory[i] = (k, v)
            else:
                k, v = memory[src]
            y = attention_mixer(x, p, sizes, eps, k, v)
        else:
            raise ValueError(f"unknown layer type {layer['type']}")
        x = x + layer_norm(y, tensors[f"l{i}.norm1"].to(F), eps)
        if layer.get("mlp") is not None:
            m = _layer_tensors(tensors, i, "mlp")
            x = x + layer_norm(squared_relu_mlp(x, m["up"], m["down"]), tensors[f"l{i}.norm2"].to(F), eps)
        layers_out.append(x.clone())
    logits = layer_norm(x, tensors["final.norm"].to(F), eps) @ tensors["embed"].to(F).T
    if return_layers:
        return logits, torch.stack(layers_out)
    return logits


def greedy_generate(prompt, n_new, tensors, config):
    memory, out = {}, []
    logits = forward(prompt, tensors, config, memory)
    for _ in range(n_new):
        out.append(int(logits[-1].argmax()))
        logits = forward([out[-1]], tensors, config, memory)
    return out

"""A plain, slow Sabezen decoder in float32 (or float64) torch on the CPU, one function per mechanism,
written from the design's equations.  It shares no code with hfee_amd: the tests compare the engine
with it.

Notation.  x: the residual stream [T, width] of one sequence whose first token sits at position 0.
`w`: a dict from tensor names to tensors (linear weights [out, in], applied as W x).  Every function
takes the whole sequence at once; the recurrent mixers walk over it token by token, so cutting a
sequence can change nothing here.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def layer_norm(x, weight, eps):
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * weight


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def xielu(z, p, q):
    pos = F.softplus(p) * z * z + z / 2
    neg = (0.5 + F.softplus(q)) * (torch.exp(torch.clamp(z, max=0.0)) - 1 - z) + z / 2
    return torch.where(z > 0, pos, neg)


def rotate_half(x, positions, dims, base):
    """x [T, heads, dim]: the first `dims` dims of each head are turned, pairs (i, i + dims/2)."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    ang = positions.to(torch.float64)[:, None] * freq[None, :]
    cos, sin = torch.cos(ang).to(x.dtype)[:, None, :], torch.sin(ang).to(x.dtype)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


def chunked_talking_attention(h, w, pre, m, eps):
    """Grouped attention whose values are the keys as projected; rotation, then a weightless RMS norm of
    q and k; the heads' scores are mixed by T; keys of the query's own chunk up to the query; a sink of
    score zero in the softmax."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    if m.get("vdim", D) != D:
        raise ValueError("the values are the keys: vdim must equal dim")
    pos = torch.arange(T)
    q = (h @ w[pre + "q"].T).view(T, H, D)
    k = (h @ w[pre + "k"].T).view(T, G, D)
    v = k
    rot = m.get("rot") or {"dims": 0, "base": 2.0}            # (no rotation named: none)
    q = rms(rotate_half(q, pos, rot["dims"], rot["base"]), eps)
    kr = rms(rotate_half(k, pos, rot["dims"], rot["base"]), eps)
    rep = H // G
    kh = kr.repeat_interleave(rep, dim=1)                                 # [T, H, D]
    vh = v.repeat_interleave(rep, dim=1)
    s = torch.einsum("ihd,jhd->hij", q, kh) * m["scale"]                  # [H, T, T]
    s = torch.einsum("hg,gij->hij", w[pre + "talk"].to(s.dtype), s)
    size = (m.get("mask") or {"size": T})["size"]             # (no mask named: every earlier position)
    seen = (pos[None, :] <= pos[:, None]) & ((pos[None, :] // size) == (pos[:, None] // size))
    e = torch.where(seen[None], torch.exp(s), torch.zeros_like(s))
    p = e / (1 + e.sum(-1, keepdim=True))
    o = torch.einsum("hij,jhd->ihd", p, vh).reshape(T, H * D)
    return o @ w[pre + "o"].T


def short_conv_silu(x, taps):
    """x [T, C], taps [C, K]: y_t = sum_j taps[:, K-1-j] x_{t-j}, zeros before the start; then silu."""
    T, C = x.shape
    K = taps.shape[1]
    padded = torch.cat([torch.zeros(K - 1, C, dtype=x.dtype), x], dim=0)
    y = torch.zeros_like(x)
    for j in range(K):
        y = y + padded[j:j + T] * taps[:, j]
    return F.silu(y)


def channel_delta(h, w, pre, m, eps):
    """The gated delta rule with one decay a key channel."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = short_conv_silu(h @ w[pre + "q"].T, w[pre + "q.conv"]).view(T, G, D)
    k = short_conv_silu(h @ w[pre + "k"].T, w[pre + "k.conv"]).view(T, G, D)
    v = short_conv_silu(h @ w[pre + "v"].T, w[pre + "v.conv"]).view(T, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[pre + "b"].T)                                                    # [T, H]
    dt = F.softplus((h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "dt_bias"]).view(T, H, D)
    g = torch.exp(-torch.exp(w[pre + "A_log"])[None, :, None] * dt)                             # [T, H, D]
    gate = torch.sigmoid((h @ w[pre + "g1"].T) @ w[pre + "g2"].T).view(T, H, V)
    out = torch.zeros(T, H, V, dtype=h.dtype)
    rep = H // G
    for hd in range(H):
        S = torch.zeros(D, V, dtype=h.dtype)
        for t in range(T):
            qt, kt = q[t, hd // rep], k[t, hd // rep]
            S = g[t, hd][:, None] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ kt)
            S = S + kt[:, None] * u[None, :]
            out[t, hd] = S.T @ qt
    out = rms(out, eps) * w[pre + "norm"] * gate
    return out.reshape(T, H * V) @ w[pre + "o"].T


def gla(h, w, pre, m, eps):
    """Gated linear attention with one decay a key channel, alpha = sigmoid(z)^(1/tau)."""
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ w[pre + "k"].T).view(T, H, D)
    v = (h @ w[pre + "v"].T).view(T, H, V)
    z = (h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "a2.b"]
    alpha = torch.exp(F.logsigmoid(z) / m["tau"]).view(T, H, D)
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for hd in range(H):
        S = torch.zeros(D, V, dtype=h.dtype)
        for t in range(T):
            S = alpha[t, hd][:, None] * S + k[t, hd][:, None] * v[t, hd][None, :]
            out[t, hd] = S.T @ q[t, hd]
    out = (rms(out, eps) * w[pre + "norm"]).reshape(T, H * V)
    return (out * F.silu(h @ w[pre + "g"].T)) @ w[pre + "o"].T


def dense_ff(h, w, pre):
    p, q = w[pre + "act"][0], w[pre + "act"][1]
    return xielu(h @ w[pre + "up"].T, p, q) @ w[pre + "down"].T


def table_moe(h, tokens, w, pre, mlp):
    """Every token id has `top` experts in a table; each counts 1/top."""
    top = mlp["router"]["top"]
    table = w[pre + "table"]
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(table[int(tokens[t]), j])
            a = F.silu(w[f"{pre}e{e}.gate"] @ h[t]) * (w[f"{pre}e{e}.up"] @ h[t])
            out[t] = out[t] + (w[f"{pre}e{e}.down"] @ a) / top
    return out


MIXERS = {"attention": chunked_talking_attention, "channel_delta": channel_delta, "gla": gla}


def forward(config: dict, weights: dict, tokens, dtype=torch.float32, layers_out=None):
    """Logits [T, vocab] of one sequence from its first token on.  layers_out: a list that gets the
    residual stream after every layer."""
    w = {k: (v if v.dtype in (torch.int32, torch.int64) else v.to(dtype)) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    tok = torch.as_tensor(tokens, dtype=torch.long)
    x = w["embed"][tok] * config["embedding"]["scale"]
    for i, layer in enumerate(config["layers"]):
        pre = f"l{i}."
        h = layer_norm(x, w[pre + "norm1"], eps)
        y = MIXERS[layer["type"]](h, w, pre + "mix.", layer["mixer"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            if mlp.get("kind", "dense") == "dense":
                y = y + dense_ff(h, w, pre + "mlp.")
            else:
                y = y + table_moe(h, tok, w, pre + "mlp.", mlp)
        x = x + y
        if layers_out is not None:
            layers_out.append(x.clone())
    return layer_norm(x, w["final.norm"], eps) @ w["head"].T

"""A plain, slow implementation of the Vofezen decoder: float64, whole sequences, no cache,
one function per mechanism.  It shares no code with the product path and is what the tests
compare the engine with.

Notation.  x: the residual stream [T, width].  A layer is
    x <- x + N1b(mixer(N1(x)));   x <- x + N2b(ff(N2(x)))
with N(y) = y / sqrt(mean(y^2) + eps) * (1 + w).  Two mixers:

  attention         H query heads over G key/value heads, key size Dk, value size Dv, rotation of
                    the first R dimensions of each q/k head (pairs (i, i + R/2)), frequencies
                    stretched for long contexts, a per-head sink in the softmax's denominator,
                    values blended with those of the first blending layer.
  latent_attention  queries and keys/values through low-rank latents with their own norms; per
                    head an unrotated part from the latent and one rotated key part shared by all
                    heads.

The feed-forward is down(relu(up(h) + b)^2) + b'.
"""
from __future__ import annotations

import json
import math
import os

import numpy as np


def read_safetensors(path: str) -> dict:
    """name -> float64 (or integer) numpy array."""
    with open(path, "rb") as f:
        n = int.from_bytes(f.read(8), "little")
        header = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, e in header.items():
        if name == "__metadata__":
            continue
        lo, hi = e["data_offsets"]
        raw = np.frombuffer(data[lo:hi], dtype=np.uint8)
        if e["dtype"] == "BF16":
            a = (raw.view(np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        elif e["dtype"] == "F32":
            a = raw.view(np.float32).astype(np.float64)
        elif e["dtype"] == "I32":
            a = raw.view(np.int32).copy()
        else:
            raise ValueError(f"{name}: dtype {e['dtype']}")
        out[name] = a.reshape(e["shape"])
    return out


# ---------------------------------------------------------------- mechanisms

def unit_rms(y, eps):
    return y / np.sqrt(np.mean(y * y, axis=-1, keepdims=True) + eps)


def offset_norm(y, w, eps):
    """The layer norm of this design: weight stored around zero."""
    return unit_rms(y, eps) * (1.0 + w)


def plain_norm(y, w, eps):
    """The latents' norm: weight as it is."""
    return unit_rms(y, eps) * w


def rotary_frequencies(dims: int, base: float, scaling=None):
    """(frequencies [dims/2], amplitude of cos and sin)."""
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def turn(t):          # the dimension whose wave makes t turns over the original context
        return dims * math.log(original / (2 * math.pi * t)) / (2 * math.log(base))
    lo = max(math.floor(turn(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turn(float(scaling["slow"]))), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(u, positions, freq, amplitude, dims):
    """u [T, heads, D]: the first `dims` of D are rotated, pairs (i, i + dims/2)."""
    a = positions[:, None].astype(np.float64) * freq[None, :]
    c, s = (np.cos(a) * amplitude)[:, None, :], (np.sin(a) * amplitude)[:, None, :]
    half = dims // 2
    lo, hi = u[..., :half], u[..., half:dims]
    return np.concatenate([lo * c - hi * s, hi * c + lo * s, u[..., dims:]], axis=-1)


def causal_softmax_mix(scores, values, sink=None):
    """scores [H, T, T] (already scaled), values [H, T, Dv]; row i sees columns j <= i; sink [H]
    joins the denominator only."""
    H, T, _ = scores.shape
    mask = np.tril(np.ones((T, T), dtype=bool))
    s = np.where(mask[None], scores, -np.inf)
    m = s.max(axis=-1, keepdims=True)
    if sink is not None:
        m = np.maximum(m, sink[:, None, None])
    e = np.exp(s - m)
    den = e.sum(axis=-1, keepdims=True)
    if sink is not None:
        den = den + np.exp(sink[:, None, None] - m)
    return (e / den) @ values


def attention_mixer(h, positions, w, m, v_first=None):
    """w: the mixer's tensors by short name; m: its config.  Returns (output, this layer's values
    before blending: what a first blending layer hands on)."""
    T = h.shape[0]
    H, G, Dk, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).reshape(T, H, Dk)
    k = (h @ w["k"].T).reshape(T, G, Dk)
    v = (h @ w["v"].T).reshape(T, G, Dv)
    rot = m["rot"]
    freq, amp = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
    q, k = rotate(q, positions, freq, amp, rot["dims"]), rotate(k, positions, freq, amp, rot["dims"])
    own = v
    if v_first is not None:
        lam = float(w["vmix"])
        v = (1.0 - lam) * v + lam * v_first
    kh = np.repeat(k, H // G, axis=1).transpose(1, 0, 2)          # head h reads key/value head h // (H/G)
    vh = np.repeat(v, H // G, axis=1).transpose(1, 0, 2)
    scores = np.einsum("thd,hsd->hts", q, kh) * m["scale"]
    o = causal_softmax_mix(scores, vh, w["sink"])                  # [H, T, Dv]
    return o.transpose(1, 0, 2).reshape(T, H * Dv) @ w["o"].T, own


def latent_attention_mixer(h, positions, w, m, eps):
    T = h.shape[0]
    H, Dn, Dr, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = plain_norm(h @ w["dq"].T, w["dq.norm"], eps)
    q = (cq @ w["uq"].T).reshape(T, H, Dn + Dr)
    dkv = h @ w["dkv"].T
    c = plain_norm(dkv[:, :R], w["dkv.norm"], eps)
    k_rot = dkv[:, R:].reshape(T, 1, Dr)
    k_un = (c @ w["uk"].T).reshape(T, H, Dn)
    v = (c @ w["uv"].T).reshape(T, H, Dv)
    rot = m["rot"]
    freq, amp = rotary_frequencies(Dr, rot["base"], rot.get("scaling"))
    q_rot = rotate(q[..., Dn:], positions, freq, amp, Dr)
    k_rot = rotate(k_rot, positions, freq, amp, Dr)
    scores = (np.einsum("thd,shd->hts", q[..., :Dn], k_un) +
              np.einsum("thd,sd->hts", q_rot, k_rot[:, 0])) * m["scale"]
    o = causal_softmax_mix(scores, v.transpose(1, 0, 2))
    return o.transpose(1, 0, 2).reshape(T, H * Dv) @ w["o"].T


def dense_feed_forward(h, w):
    a = np.maximum(h @ w["up"].T + w["up.b"], 0.0)
    return (a * a) @ w["down"].T + w["down.b"]


# ---------------------------------------------------------------- the model

class PlainVofezen:
    def __init__(self, folder: str = None, config: dict = None, tensors: dict = None):
        if folder is not None:
            with open(os.path.join(folder, "config.json")) as f:
                config = json.load(f)
            tensors = read_safetensors(os.path.join(folder, "model.safetensors"))
        self.config = config
        self.t = {k: np.asarray(v, dtype=np.float64) for k, v in tensors.items()}
        self.eps = float(config["norm"]["eps"])

    def _sub(self, prefix):
        return {k[len(prefix):]: v for k, v in self.t.items() if k.startswith(prefix)}

    def forward(self, tokens, layers_out=None):
        """Logits [T, vocab] of a whole sequence from position 0; layers_out, if a list, gets the
        stream after every layer."""
        t, eps = self.t, self.eps
        tokens = np.asarray(tokens, dtype=np.int64)
        positions = np.arange(len(tokens))
        x = t["embed"][tokens]
        v_first = None
        for i, layer in enumerate(self.config["layers"]):
            p = f"l{i}."
            h = offset_norm(x, t[p + "norm1"], eps)
            m = layer["mixer"]
            if layer["type"] == "attention":
                blend = bool(m.get("v_mix"))
                y, own = attention_mixer(h, positions, self._sub(p + "mix."), m, v_first if blend else None)
                if blend and v_first is None:
                    v_first = own
            elif layer["type"] == "latent_attention":
                y = latent_attention_mixer(h, positions, self._sub(p + "mix."), m, eps)
            else:
                raise ValueError(layer["type"])
            x = x + offset_norm(y, t[p + "norm1b"], eps)
            if layer.get("mlp") is not None:
                h = offset_norm(x, t[p + "norm2"], eps)
                y = dense_feed_forward(h, self._sub(p + "mlp."))
                x = x + offset_norm(y, t[p + "norm2b"], eps)
            if layers_out is not None:
                layers_out.append(x.copy())
        return offset_norm(x, t["final.norm"], eps) @ t["head"].T

    def greedy(self, prompt, count):
        tokens, out = list(prompt), []
        for _ in range(count):
            nxt = int(np.argmax(self.forward(tokens)[-1]))
            out.append(nxt)
            tokens.append(nxt)
        return out

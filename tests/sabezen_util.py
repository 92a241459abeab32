"""Small Sabezen configurations for the tests, and folders of random weights for them in which the
numbers that plain random weights would leave without effect (norm weights, the heads' mixing
matrix, decays, step sizes, the activation's two numbers) are large enough to show."""
import json
import os

import numpy as np
import torch


def attention(heads, kv_heads, dim, rot_dims, chunk, scale, base=10000.0):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale,
                                           "mask": {"size": chunk}, "rot": {"base": base, "dims": rot_dims}}}


def delta(heads, kv_heads, dim, vdim, conv, decay_rank, gate_rank):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
                                               "decay_rank": decay_rank, "gate_rank": gate_rank}}


def gla(heads, dim, vdim, tau, decay_rank):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "decay_rank": decay_rank}}


def dense(layer, ff):
    return dict(layer, mlp={"kind": "dense", "ff": ff})


def moe(layer, ff, experts, top):
    return dict(layer, mlp={"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}})


def bare(layer):
    return dict(layer, mlp=None)


def config(vocab, width, eps, scale, layers):
    return {"architecture": "Sabezen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale},
            "layers": layers}


# every mixer and feed-forward twice, two experts a token, two value heads a query/key head in the delta
# rule, a layer without a feed-forward, chunks that are no multiple of a page
S_A = config(131, 64, 1e-6, 3.0, [
    dense(attention(4, 2, 16, 8, 24, 0.3), 72),
    moe(delta(4, 2, 8, 16, 4, 8, 8), 24, 5, 2),
    bare(gla(2, 16, 8, 7.0, 8)),
    moe(attention(4, 2, 16, 8, 24, 0.3), 24, 5, 2),
    dense(delta(4, 2, 8, 16, 4, 8, 8), 40),
    moe(gla(2, 16, 8, 7.0, 8), 16, 3, 1),
])
# sizes that are multiples of nothing, the whole head rotated, as many key heads as heads, one query/key
# head under three value heads, two taps, every expert for every token, no scaling of the embedding
S_B = config(97, 72, 1e-5, 1.0, [
    moe(gla(3, 20, 12, 3.0, 6), 10, 4, 4),
    dense(attention(3, 3, 24, 24, 17, 0.2, base=500.0), 50),
    bare(delta(3, 1, 12, 20, 2, 5, 7)),
    dense(attention(3, 3, 24, 24, 17, 0.2, base=500.0), 33),
])
# no attention at all: a model without a paged cache, states only; one tap (no convolution state)
S_C = config(60, 48, 1e-6, 2.0, [
    dense(delta(2, 2, 16, 16, 1, 8, 8), 64),
    moe(gla(3, 8, 24, 16.0, 4), 32, 6, 3),
    bare(delta(2, 2, 16, 16, 5, 8, 8)),
])
# larger, for prompts of hundreds of tokens over many chunks; chunks longer than a tile of keys; experts of
# sizes that the grouped kernels take
S_D = config(500, 128, 1e-6, 8.0, [
    dense(attention(8, 2, 32, 16, 80, 0.15), 160),
    moe(delta(2, 2, 32, 64, 3, 16, 24), 64, 8, 1),
    dense(gla(4, 32, 32, 12.0, 16), 96),
    moe(attention(8, 2, 32, 16, 80, 0.15), 96, 8, 2),
])
CONFIGS = {"A": S_A, "B": S_B, "C": S_C, "D": S_D}

# one mechanism each
SINGLE = {
    "attention": config(50, 48, 1e-6, 2.0, [bare(attention(4, 2, 12, 6, 10, 0.4))]),
    "attention without chunks or rotation": config(50, 64, 1e-6, 2.0, [bare(
        {"type": "attention", "mixer": {"heads": 4, "kv_heads": 4, "dim": 32, "scale": 0.2}})]),
    "delta": config(50, 48, 1e-6, 2.0, [bare(delta(4, 2, 8, 12, 3, 6, 6))]),
    "gla": config(50, 48, 1e-6, 2.0, [bare(gla(3, 8, 12, 5.0, 6))]),
    "dense": config(50, 48, 1e-6, 2.0, [dense(gla(1, 4, 4, 5.0, 2), 40)]),
    "moe": config(50, 48, 1e-6, 2.0, [moe(gla(1, 4, 4, 5.0, 2), 20, 7, 3)]),
}


def make_tensors(config_json, seed, std=0.1):
    """name -> float32 (or int32) tensor."""
    import hfee_amd  # noqa: F401
    from hfee_amd.config import config_from_dict
    from hfee_amd.engine.model import declared_tensors
    from hfee_amd.weights.random_init import random_tensors
    cfg = config_from_dict(config_json)
    tensors = random_tensors(declared_tensors(cfg), seed, std, torch.float32, "cpu")
    g = torch.Generator().manual_seed(seed + 1)
    for name in list(tensors):
        t = tensors[name]
        if name.endswith(".table"):
            continue
        if name.endswith(".talk"):
            t = torch.eye(t.shape[0]) + torch.randn(t.shape, generator=g) * 0.3
        elif name.endswith(".norm") or ".norm1" in name:
            t = 1.0 + torch.randn(t.shape, generator=g) * 0.3
        elif name.endswith(".A_log") or name.endswith(".dt_bias"):
            t = torch.randn(t.shape, generator=g) * 0.5 - 1.0
        elif name.endswith(".a2.b"):
            t = torch.randn(t.shape, generator=g) + 2.0
        elif name.endswith(".act"):
            t = torch.randn(t.shape, generator=g)
        elif name.endswith(".conv"):
            t = torch.randn(t.shape, generator=g) * 0.5
        elif name.endswith(".a2") or name.endswith(".g2") or name.endswith(".b"):
            t = torch.randn(t.shape, generator=g) * 0.5
        tensors[name] = t
    return tensors


def make_folder(path, config_json, seed, dtype="float32", std=0.1, tensors=None):
    """config.json + model.safetensors with seeded weights; returns the folder.  The ranks of the low-rank
    projections are left to the tensors' shapes, as in a checkpoint of this design."""
    from hfee_amd.weights.safetensors_io import write_safetensors
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    tensors = make_tensors(config_json, seed, std) if tensors is None else tensors
    tensors = {n: (t if t.dtype == torch.int32 else t.to(dt)) for n, t in tensors.items()}
    os.makedirs(path, exist_ok=True)
    stripped = json.loads(json.dumps(config_json))
    for layer in stripped["layers"]:
        layer["mixer"].pop("decay_rank", None)
        layer["mixer"].pop("gate_rank", None)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(stripped, f)
    write_safetensors(os.path.join(str(path), "model.safetensors"), tensors, metadata={"format": "pt"})
    return str(path)


def load_plain(folder):
    """(config.json's keys, name -> tensor) of a folder, for the plain implementation."""
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as f:
        cj = json.load(f)
    return cj, load_file(os.path.join(folder, "model.safetensors"))


def rel(a, b):
    a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    return float(np.abs(a - b).max() / np.abs(b).max())

"""Small Vofezen configurations for the tests, and folders of random weights for them in which
the numbers that random weights would leave without effect (sinks, blend weights, norm weights,
biases) are large enough to show."""
import json
import os

import numpy as np
import torch


def attention(heads, kv_heads, dim, vdim, rot_dims, v_mix, scaling=True, base=10000.0, scale=None):
    rot = {"base": base, "dims": rot_dims}
    if scaling:
        rot["scaling"] = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                                           "scale": scale if scale is not None else 1.3 / dim ** 0.5, "v_mix": v_mix, "rot": rot}}


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, base=300000.0, scale=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                      "scale": scale if scale is not None else 0.9 / (dim + rot_dim) ** 0.5,
                      "rot": {"base": base, "dims": rot_dim}}}


def with_mlp(layer, ff):
    return dict(layer, mlp=None if ff is None else {"kind": "dense", "ff": ff})


def config(vocab, width, eps, layers):
    return {"architecture": "Vofezen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


# sizes in multiples of 16 (the matrix-core kernels in bfloat16); a layer without a feed-forward, an
# attention layer that blends nothing in front of the blending ones, 2 query heads a key/value head
V_A = config(211, 72, 1e-5, [
    with_mlp(attention(4, 2, 32, 16, 16, False), 100),
    with_mlp(attention(4, 2, 32, 16, 16, True), 96),
    with_mlp(latent(3, 16, 16, 16, 48, 32), None),
    with_mlp(attention(4, 2, 32, 16, 16, True), 100),
    with_mlp(latent(3, 16, 16, 16, 48, 32), 64),
    with_mlp(attention(4, 2, 32, 16, 16, True), 40),
])
# sizes that are no multiples of 16 (the plain kernel in both dtypes), as many key/value heads as
# heads, the whole head rotated, no stretching, values larger than keys, blending from layer 0 on
V_B = config(97, 58, 1e-6, [
    with_mlp(attention(3, 3, 24, 28, 24, True, scaling=False, base=500.0), 77),
    with_mlp(latent(2, 12, 8, 20, 30, 40, base=1000.0), 50),
    with_mlp(attention(3, 3, 24, 28, 24, True, scaling=False, base=500.0), 33),
])
# 20 query heads on one key/value head (more than a tile's 16 rows), values larger than keys, a wide
# latent, one head; for long sequences
V_C = config(300, 128, 1e-5, [
    with_mlp(attention(20, 1, 16, 48, 8, True), 128),
    with_mlp(latent(1, 32, 16, 48, 64, 96), 256),
    with_mlp(attention(20, 1, 16, 48, 8, True), 64),
])
# latent attention first, four query heads a key/value head and eight latent heads (the kernels that
# share key tiles through LDS), larger sizes, for prompts beyond a thousand tokens
V_D = config(1000, 256, 1e-6, [
    with_mlp(latent(8, 32, 32, 48, 96, 64), 384),
    with_mlp(attention(8, 2, 64, 32, 32, True, base=50000.0), 320),
    with_mlp(attention(8, 2, 64, 32, 32, False, base=50000.0), None),
    with_mlp(attention(8, 2, 64, 32, 32, True, base=50000.0), 384),
    with_mlp(latent(8, 32, 32, 48, 96, 64), 128),
])
CONFIGS = {"A": V_A, "B": V_B, "C": V_C, "D": V_D}


def make_folder(path, config_json, seed, dtype="float32", std=0.1):
    """config.json + model.safetensors with seeded weights; returns the folder."""
    import hfee_amd  # noqa: F401
    from hfee_amd.config import config_from_dict
    from hfee_amd.engine.model import declared_tensors
    from hfee_amd.weights.random_init import random_tensors
    from hfee_amd.weights.safetensors_io import write_safetensors
    cfg = config_from_dict(config_json)
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    specs = declared_tensors(cfg)
    tensors = random_tensors(specs, seed, std, torch.float32, "cpu")
    for sp in specs:          # (the numbers a layer does not use are in a checkpoint all the same)
        if sp.optional:
            tensors[sp.name] = torch.zeros(tuple(sp.shape))
    g = torch.Generator().manual_seed(seed + 1)
    for name in list(tensors):
        t = tensors[name]
        if name.endswith(".sink"):
            t = torch.randn(t.shape, generator=g) * 2.0 + 1.0
        elif name.endswith(".vmix"):
            t = torch.rand((), generator=g) * 0.6 + 0.2
        elif name.endswith(".b") or ".norm" in name and not name.endswith(".dq.norm") and not name.endswith(".dkv.norm"):
            t = torch.randn(t.shape, generator=g) * 0.3
        elif name.endswith(".dq.norm") or name.endswith(".dkv.norm"):
            t = 1.0 + torch.randn(t.shape, generator=g) * 0.3
        tensors[name] = t.to(dt)
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config_json, f)
    write_safetensors(os.path.join(str(path), "model.safetensors"), tensors, metadata={"format": "pt"})
    return str(path)


def rel(a, b):
    a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    return float(np.abs(a - b).max() / np.abs(b).max())

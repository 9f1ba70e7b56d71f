"""Small Saposun configurations for the tests, and folders of random weights for them in which the numbers
that plain random weights would leave without effect (norm weights, the routers' corrections, the taps of the
short convolutions) are large enough to show."""
import json
import os

import numpy as np
import torch


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, window=None, base=10000.0, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale,
         "rot": {"base": base, "dims": rot_dim}}
    if window:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m}


def retention(heads, dim, vdim, decay, rot_dims=None, base=10000.0):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
    return {"type": "retention", "mixer": m}


def attention(heads, kv_heads, dim, vdim, scale, window=None, pool=None, conv=None, softcap=None, rot_dims=None, base=10000.0):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
        if pool:
            m["mask"]["pool"] = pool
    if conv:
        m["conv"] = conv
    if softcap:
        m["softcap"] = softcap
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
    return {"type": "attention", "mixer": m}


def moe(layer, ff, experts, top):
    return dict(layer, mlp={"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}})


def bare(layer):
    return dict(layer, mlp=None)


def config(vocab, width, eps, mult, layers):
    return {"architecture": "Saposun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult,
            "layers": layers}


def every_expert(config_json):
    """The same model with every expert for every token (nothing is chosen: no near tie of a router)."""
    out = json.loads(json.dumps(config_json))
    for layer in out["layers"]:
        if layer["mlp"] is not None:
            layer["mlp"]["router"]["top"] = layer["mlp"]["router"]["experts"]
    return out


# every mixer twice, a layer that reads the first layer's keys, a layer without a feed-forward, windows and
# blocks that are no multiples of a page; sizes that the matrix-core kernels take
P_A = config(131, 64, 1e-6, 0.5, [
    moe(latent(4, 16, 16, 16, 24, 32, 0.2, window=21), 32, 6, 2),
    moe(retention(2, 16, 32, (0.9, 0.97), rot_dims=16), 32, 6, 2),
    moe(attention(4, 2, 32, 16, 0.2, window=19, pool=5, conv=3, softcap=4.0, rot_dims=16), 32, 6, 2),
    bare(latent(4, 16, 16, 16, 24, 32, 0.2, window=9, kv_from=0)),
    moe(retention(2, 16, 32, (0.5, 1.0), rot_dims=16), 32, 5, 1),
    moe(attention(4, 2, 32, 16, 0.2, window=40, pool=16, conv=2, rot_dims=32), 32, 6, 2),
])
# sizes that are multiples of nothing, as many key heads as heads, one head, a pool of one and a window of one, a
# pool longer than the window, four taps, no cap, the whole head rotated and nothing rotated, every expert for every
# token, no scaling of the layers' results
P_B = config(97, 72, 1e-5, 1.0, [
    moe(attention(3, 3, 10, 12, 0.3, window=7, pool=1, conv=4, rot_dims=10), 10, 4, 4),
    moe(latent(3, 6, 4, 10, 14, 18, 0.25, window=1, base=500.0), 20, 3, 3),
    bare(retention(3, 12, 20, (0.8, 0.99, 0.95))),
    moe(attention(1, 1, 20, 6, 0.2, window=5, pool=11, softcap=2.0), 33, 4, 4),
    moe(latent(2, 6, 4, 10, 10, 18, 0.25, base=500.0, kv_from=1), 20, 3, 3),
])
# no attention at all: a model without a paged cache, states only
P_C = config(60, 48, 1e-6, 0.7, [
    moe(retention(2, 16, 16, (0.9, 0.95), rot_dims=8), 32, 6, 3),
    bare(retention(3, 8, 24, (0.99, 0.5, 0.75), rot_dims=8)),
])
# larger, for prompts of hundreds of tokens: windows over several pages and tiles, hundreds of pooled blocks' worth of
# tokens, experts of sizes that the grouped kernels take
P_D = config(500, 128, 1e-6, 0.4, [
    moe(latent(8, 16, 16, 32, 48, 64, 0.15, window=70), 64, 8, 2),
    moe(retention(4, 32, 32, (0.95, 0.98, 0.99, 0.999), rot_dims=32), 64, 8, 2),
    moe(attention(8, 2, 64, 64, 0.12, window=100, pool=7, conv=4, softcap=20.0, rot_dims=64), 96, 8, 2),
    moe(latent(4, 16, 16, 32, 48, 64, 0.15, window=33, kv_from=0), 64, 8, 1),
    moe(attention(4, 4, 32, 32, 0.2, window=48, pool=16, conv=2, rot_dims=16), 64, 8, 2),
])
CONFIGS = {"A": P_A, "B": P_B, "C": P_C, "D": P_D, "A every expert": every_expert(P_A), "D every expert": every_expert(P_D)}

# one mechanism each
SINGLE = {
    "latent": config(50, 48, 1e-6, 0.5, [bare(latent(3, 8, 8, 12, 16, 20, 0.3, window=6))]),
    "latent without a window": config(50, 48, 1e-6, 1.0, [bare(latent(4, 16, 16, 16, 24, 32, 0.2))]),
    "retention": config(50, 48, 1e-6, 0.5, [bare(retention(3, 8, 12, (0.9, 0.6, 1.0), rot_dims=4))]),
    "attention": config(50, 48, 1e-6, 0.5, [bare(attention(4, 2, 12, 6, 0.4, window=10, pool=3, conv=3, softcap=3.0, rot_dims=6))]),
    "attention without anything": config(50, 64, 1e-6, 2.0, [bare(attention(4, 4, 32, 32, 0.2))]),
    "moe": config(50, 48, 1e-6, 0.5, [moe(retention(1, 4, 4, (0.5,)), 20, 7, 3)]),
    # a width that is a multiple of nothing, a convolution of one tap (no state), two layers so that the scaled sum
    # makes the next layer's norm
    "odd width": config(61, 58, 1e-6, 0.25, [moe(attention(2, 1, 14, 10, 0.3, window=9, pool=4, conv=1, rot_dims=14), 9, 3, 2),
                                              moe(latent(2, 5, 6, 7, 9, 11, 0.3, window=4), 9, 3, 3)]),
}


def make_tensors(config_json, seed, std=0.1):
    """name -> float32 tensor."""
    import hfee_amd  # noqa: F401
    from hfee_amd.config import config_from_dict
    from hfee_amd.engine.model import declared_tensors
    from hfee_amd.weights.random_init import random_tensors
    cfg = config_from_dict(config_json)
    tensors = random_tensors(declared_tensors(cfg), seed, std, torch.float32, "cpu")
    g = torch.Generator().manual_seed(seed + 1)
    for name in list(tensors):
        t = tensors[name]
        if name.endswith(".norm") or name.endswith(".norm1"):
            t = 1.0 + torch.randn(t.shape, generator=g) * 0.3
        elif name.endswith(".conv"):
            t = torch.randn(t.shape, generator=g) * 0.5
        elif name.endswith(".correction"):
            t = torch.randn(t.shape, generator=g) * 0.2
        elif name.endswith(".router"):
            t = torch.randn(t.shape, generator=g) * 0.3
        elif name.endswith("mix.g"):
            t = torch.randn(t.shape, generator=g) * 0.3
        tensors[name] = t
    return tensors


def make_folder(path, config_json, seed, dtype="float32", std=0.1, tensors=None):
    """config.json + model.safetensors with seeded weights; returns the folder."""
    from hfee_amd.weights.safetensors_io import write_safetensors
    dt = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    tensors = make_tensors(config_json, seed, std) if tensors is None else tensors
    tensors = {n: (t if t.dtype == torch.int32 else t.to(dt)) for n, t in tensors.items()}
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config_json, f)
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

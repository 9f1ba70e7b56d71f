"""Small Ronavik configurations for the tests, and folders of random weights for them in which the
numbers that plain random weights would leave without effect (norm weights, the heads' numbers, decays,
step sizes, biases, the router) are large enough to show."""
import json
import os

import numpy as np
import torch


def pair(heads, kv_heads, dim, vdim, scale, width, blocks, conv, q_temp=None, left_scale=1.0, right_scale=1.0):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if q_temp is not None:
        left["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return {"type": "parallel", "mixer": {"left": left, "right": {"width": width, "blocks": blocks, "conv": conv},
                                          "left_scale": left_scale, "right_scale": right_scale}}


def ssm(heads, vdim, state, groups, conv, norm_groups):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                        "norm_groups": norm_groups}}


def moe(layer, ff, experts, top):
    return dict(layer, mlp={"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}})


def bare(layer):
    return dict(layer, mlp=None)


def config(vocab, width, eps, positions, layers):
    return {"architecture": "Ronavik", "vocab": vocab, "width": width, "norm": {"eps": eps}, "max_positions": positions,
            "layers": layers}


# both mixers twice, a layer without a feed-forward, two experts a token and one; a temperature that steps
# every 8 positions; sizes that the matrix-core attention takes with two query heads a key head
R_A = config(131, 64, 1e-6, 512, [
    moe(pair(4, 2, 16, 32, 0.3, 48, 3, 4, q_temp=(0.5, 8), left_scale=0.7, right_scale=1.3), 24, 5, 2),
    moe(ssm(4, 8, 16, 2, 4, 4), 16, 3, 1),
    bare(pair(4, 2, 16, 32, 0.3, 48, 3, 4, q_temp=(0.5, 8), left_scale=0.7, right_scale=1.3)),
    moe(ssm(4, 8, 16, 2, 4, 4), 24, 5, 2),
])
# sizes that are multiples of nothing, as many key heads as heads, no temperature, no scales in the file, one
# block, two taps and one, one group, every expert for every token, the state-space layer first
R_B = config(97, 72, 1e-5, 300, [
    moe(ssm(3, 12, 10, 1, 1, 1), 10, 4, 4),
    bare(pair(3, 3, 20, 12, 0.2, 36, 1, 2)),
    moe(ssm(3, 12, 10, 3, 2, 9), 50, 2, 1),
    moe(pair(3, 3, 20, 12, 0.2, 36, 1, 2), 33, 70, 3),
])
# no attention at all: a model without a paged cache, states only; norm parts smaller than a head
R_C = config(60, 48, 1e-6, 256, [
    moe(ssm(2, 16, 8, 2, 5, 8), 32, 6, 3),
    bare(ssm(4, 4, 24, 1, 3, 2)),
])
# larger, for prompts of hundreds of tokens; four query heads a key head and sizes that the grouped experts
# and the matrix-core kernels take
R_D = config(500, 128, 1e-6, 1024, [
    moe(pair(8, 2, 32, 64, 0.15, 128, 4, 3, q_temp=(0.3, 64), left_scale=1.1, right_scale=0.8), 64, 8, 2),
    moe(ssm(4, 32, 32, 2, 3, 2), 96, 8, 1),
    moe(pair(8, 2, 32, 64, 0.15, 128, 4, 3, q_temp=(0.3, 64), left_scale=1.1, right_scale=0.8), 64, 8, 2),
])


def every_expert(cj):
    """The same configuration with routers that choose every expert for every token."""
    layers = [layer if layer["mlp"] is None else
              dict(layer, mlp=dict(layer["mlp"], router=dict(layer["mlp"]["router"], top=layer["mlp"]["router"]["experts"])))
              for layer in cj["layers"]]
    return dict(cj, layers=layers)


CONFIGS = {"A": R_A, "B": R_B, "C": R_C, "D": R_D, "A every expert": every_expert(R_A), "D every expert": every_expert(R_D)}

# one mechanism each (a pair with one of its scales zero is the other mixer alone)
SINGLE = {
    "sigmoid attention": config(50, 48, 1e-6, 128, [bare(pair(4, 2, 12, 20, 0.4, 16, 2, 2, q_temp=(0.8, 5), right_scale=0.0))]),
    "recurrent unit": config(50, 48, 1e-6, 128, [bare(pair(2, 1, 8, 8, 0.4, 40, 5, 3, left_scale=0.0))]),
    "state space": config(50, 48, 1e-6, 128, [bare(ssm(6, 4, 12, 3, 3, 2))]),
    "experts": config(50, 48, 1e-6, 128, [moe(ssm(1, 4, 4, 1, 2, 1), 20, 7, 3)]),
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
    rn = lambda t, s=1.0: torch.randn(t.shape, generator=g) * s          # noqa: E731
    for name in list(tensors):
        t = tensors[name]
        last = name.split(".")[-1]
        if last == "norm" or last.startswith("norm") or name.endswith(".D"):
            t = 1.0 + rn(t, 0.3)
        elif last == "pos":
            t = rn(t, 0.3)
        elif last == "pb":
            t = rn(t, 0.7) - 1.0
        elif last in ("A_log", "dt_bias"):
            t = rn(t, 0.5) - 1.0
        elif last == "lam":
            t = rn(t, 1.0) - 3.0
        elif last == "conv":
            t = rn(t, 0.5)
        elif last == "b":
            t = rn(t, 0.4)
        elif last in ("ra", "ri"):
            t = rn(t, 0.5)
        elif last == "router":
            t = rn(t, 0.6)
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

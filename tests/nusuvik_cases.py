"""Tiny Nusuvik configurations and weights for the tests, made here: sizes that differ in everything from each
other, and weights with gains near one, so that every mechanism moves the logits (the framework's own random
weights are N(0, 0.02): a mixer's fault would hardly show through them)."""
import json
from pathlib import Path

import numpy as np
import torch


def latent_layer(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, mlp, base=10000.0):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
                      "scale": scale, "rot": {"base": base, "dims": rot_dim}},
            "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, groups=None, keep=None):
    router = {"experts": experts, "top": top}
    if groups is not None:
        router["groups"] = {"count": groups, "keep": keep}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


# A: small odd sizes; every layer's mixer of other sizes (three page groups); a layer without feed-forward; the loop
# starts at the first layer and runs three times; groups of two experts of which two of three are kept
CONFIG_A = {"architecture": "Nusuvik", "vocab": 211, "width": 96, "norm": {"eps": 1e-5}, "logit_softcap": 9.0,
            "embedding": {"bigram": {"buckets": 97, "mul_prev": 5, "mul_cur": 3}},
            "loop": {"start": 0, "stop": 2, "times": 3},
            "layers": [latent_layer(3, 24, 8, 16, 40, 56, 0.2, dense(120)),
                       latent_layer(4, 16, 12, 20, 24, 36, 0.25, moe(6, 2, 40, 3, 2), base=500.0),
                       latent_layer(2, 10, 6, 30, 18, 20, 0.3, None)]}
# B: no loop, no cap, no groups in the router, ONE expert chosen in one layer and all of them in another; one head; both
# multipliers of the pair hash 1; buckets fewer than tokens
CONFIG_B = {"architecture": "Nusuvik", "vocab": 300, "width": 128, "norm": {"eps": 1e-6},
            "embedding": {"bigram": {"buckets": 31, "mul_prev": 1, "mul_cur": 1}},
            "layers": [latent_layer(1, 48, 16, 32, 64, 32, 0.12, moe(4, 1, 72)),
                       latent_layer(6, 16, 4, 16, 28, 48, 0.22, moe(3, 3, 48, 1, 1)),
                       latent_layer(5, 8, 24, 8, 8, 16, 0.18, dense(200))]}
# C: sizes that reach the matrix-core kernels (widths in multiples of 32, rows of the cache of 128 and 256 columns); the
# loop is the last layer alone, twice; one of four groups kept; groups of ONE expert in the other routed layer
CONFIG_C = {"architecture": "Nusuvik", "vocab": 384, "width": 256, "norm": {"eps": 1e-5}, "logit_softcap": 20.0,
            "embedding": {"bigram": {"buckets": 1021, "mul_prev": 1000003, "mul_cur": 77}},
            "loop": {"start": 2, "stop": 3, "times": 2},
            "layers": [latent_layer(4, 32, 64, 64, 64, 96, 0.1, moe(8, 2, 64, 4, 1)),
                       latent_layer(8, 64, 64, 32, 192, 64, 0.09, dense(512)),
                       latent_layer(4, 32, 64, 64, 64, 96, 0.1, moe(4, 2, 96, 4, 2))]}
# D: no pair table at all, a loop of one pass over the middle layers
CONFIG_D = {"architecture": "Nusuvik", "vocab": 64, "width": 48, "norm": {"eps": 1e-6}, "logit_softcap": 4.0,
            "loop": {"start": 1, "stop": 3, "times": 1},
            "layers": [latent_layer(2, 8, 8, 8, 16, 16, 0.25, dense(64)), latent_layer(2, 8, 8, 8, 16, 16, 0.25, None),
                       latent_layer(3, 12, 2, 4, 10, 6, 0.3, moe(2, 1, 24, 2, 1)), latent_layer(2, 8, 8, 8, 16, 16, 0.25, dense(32))]}
CASES = {"A": (CONFIG_A, 8, 31), "B": (CONFIG_B, 16, 32), "C": (CONFIG_C, 32, 33), "D": (CONFIG_D, 4, 34)}


def draw_weights(config, seed):
    """name -> float32 array for every tensor of the configuration's model, gains near one."""
    from litinfer_amd.config import lookup, architecture_name
    from litinfer_amd.engine.model import expected_params_of_spec
    arch = lookup(architecture_name(config))
    spec = arch.model_spec(arch.config_from_dict(config))
    rng = np.random.default_rng(seed)
    out = {}
    for name, p in sorted(expected_params_of_spec(spec).items()):
        shape, leaf = tuple(p.shape), name.split(".")[-1]
        if name.endswith(".norm") or leaf == "norm1":                  # norm weights
            a = rng.normal(1.0, 0.1, shape)
        elif leaf == "b":                                               # biases of norms and of the dense feed-forward
            a = rng.normal(0.0, 0.1, shape)
        elif leaf == "correction":
            a = rng.normal(0.0, 0.3, shape)
        elif leaf == "router":
            a = rng.normal(0.0, 3.0 / np.sqrt(shape[-1]), shape)
        elif name == "embed":
            a = rng.normal(0.0, 1.0, shape)
        elif name == "bigram":
            a = rng.normal(0.0, 0.7, shape)
        elif name == "loop.in":
            a = rng.normal(0.0, 1.4 / np.sqrt(shape[-1]), shape)
        elif leaf == "g":
            a = rng.normal(0.0, 2.0 / np.sqrt(shape[-1]), shape)
        else:                                                           # a matrix [out, in]
            a = rng.normal(0.0, 1.0 / np.sqrt(shape[-1]), shape)
        out[name] = a.astype(np.float32)
    return out


def write_model(folder, config, weights, dtype=torch.float32):
    """config.json and model.safetensors with these weights, stored in `dtype`."""
    from litinfer_amd.weights.safetensors_io import write_safetensors
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(config))
    write_safetensors(folder / "model.safetensors", ((n, torch.from_numpy(a).to(dtype)) for n, a in sorted(weights.items())),
                      metadata={"format": "pt"})
    return folder


def stored(weights, dtype):
    """The weights as a checkpoint of `dtype` holds them, float64."""
    return {n: torch.from_numpy(a).to(dtype).to(torch.float64).numpy() for n, a in weights.items()}


def random_config(seed):
    """A configuration drawn from a seed: every size, the order of layers, the loop and the routers' shapes vary."""
    rng = np.random.default_rng(seed)
    pick = lambda *xs: xs[int(rng.integers(0, len(xs)))]
    n = int(rng.integers(2, 6))
    width = pick(64, 72, 96, 160, 192, 256, 328, 384)
    kinds = []

    def mixer():
        heads, dim, rot = pick(1, 2, 3, 4, 6, 8, 16), pick(8, 16, 24, 32, 64, 128), pick(2, 8, 16, 32, 64)
        return dict(heads=heads, dim=dim, rot_dim=rot, vdim=pick(8, 16, 32, 48, 64, 128), kv_rank=pick(8, 24, 32, 64, 96, 128),
                    q_rank=pick(8, 16, 48, 64, 128, 192), scale=float(rng.uniform(0.5, 1.5)) / np.sqrt(dim + rot),
                    base=pick(100.0, 10000.0, 500000.0))
    shared = mixer()
    layers = []
    for i in range(n):
        m = shared if rng.random() < 0.6 else mixer()           # (equal mixers share a page group)
        kind = pick("dense", "moe", "moe", None)
        if kind == "dense":
            mlp = dense(pick(32, 100, 256, 520))
        elif kind == "moe":
            groups = pick(1, 2, 3, 4)
            per = pick(1, 2, 4) if groups > 1 else pick(2, 3, 8)
            keep = int(rng.integers(1, groups + 1))
            top = int(rng.integers(1, min(keep * per, 6) + 1))
            mlp = moe(groups * per, top, pick(16, 40, 64, 96), groups if rng.random() < 0.8 or groups > 1 else None, keep)
        else:
            mlp = None
        kinds.append(kind)
        layers.append(latent_layer(m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"], m["scale"], mlp, m["base"]))
    cfg = {"architecture": "Nusuvik", "vocab": pick(61, 200, 450, 515), "width": width, "norm": {"eps": pick(1e-6, 1e-5, 1e-3)}, "layers": layers}
    if rng.random() < 0.8:
        cfg["embedding"] = {"bigram": {"buckets": pick(7, 521, 4099), "mul_prev": pick(1, 37, 65537), "mul_cur": pick(1, 11, 1009)}}
    if rng.random() < 0.8:
        start = int(rng.integers(0, n))
        cfg["loop"] = {"start": start, "stop": int(rng.integers(start + 1, n + 1)), "times": int(rng.integers(1, 4))}
    if rng.random() < 0.7:
        cfg["logit_softcap"] = pick(5.0, 25.0, 50.0)
    return cfg

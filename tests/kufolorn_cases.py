"""Tiny Kufolorn configurations and weights for the tests, made here: sizes that differ in everything from each
other, and weights with gains near one, so that every mechanism moves the logits (the framework's own random
weights are N(0, 0.02): a mixer's fault would hardly show through them)."""
import json
from pathlib import Path

import numpy as np
import torch


def delta_layer(heads, kv_heads, dim, vdim, conv, mlp):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}, "mlp": mlp}


def rot(dims, base=10000.0, factor=None):
    r = {"base": base, "dims": dims}
    if factor is not None:
        r["scaling"] = {"factor": factor}
    return r


def parallel_layer(left, right, left_scale, right_scale, mlp):
    """left = (heads, kv_heads, dim, vdim, scale, rot); right = (heads, dim, vdim, decay list, rot)."""
    lh, lkv, ld, lv, ls, lr = left
    rh, rd, rv, decay, rr = right
    return {"type": "parallel",
            "mixer": {"left": {"heads": lh, "kv_heads": lkv, "dim": ld, "vdim": lv, "scale": ls, "rot": lr},
                      "right": {"heads": rh, "dim": rd, "vdim": rv, "decay": list(decay), "rot": rr},
                      "left_scale": left_scale, "right_scale": right_scale},
            "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, identity, top, ff, limit, groups=None, keep=None):
    router = {"experts": experts, "top": top, "identity": identity}
    if groups is not None:
        router["groups"] = {"count": groups, "keep": keep}
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": router}


# A: small odd sizes; four taps; three q/k heads for six heads; partial rotation with scaled frequencies; two identity
# experts among eight router outputs in four groups of which two are kept; a layer without feed-forward
CONFIG_A = {"architecture": "Kufolorn", "vocab": 211, "width": 96, "norm": {"eps": 1e-5}, "logit_softcap": 9.0,
            "layers": [delta_layer(6, 3, 24, 16, 4, dense(120)),
                       parallel_layer((4, 2, 24, 16, 0.2, rot(8, 500.0, 4.0)), (3, 12, 20, (0.9, 0.97, 0.995), rot(12)), 0.7, 0.4,
                                      moe(6, 2, 2, 40, 1.5, 4, 2)),
                       delta_layer(2, 2, 8, 40, 2, None),
                       parallel_layer((6, 6, 10, 30, 0.3, rot(10)), (1, 20, 8, (0.95,), rot(4, 100.0, 3.0)), 1.0, 1.0, dense(64))]}
# B: a parallel layer first; one kv head; no convolution in one delta layer (one tap); no identity experts, no groups,
# every expert chosen in one layer and ONE in the other; no cap of the logits; rotation of the whole head
CONFIG_B = {"architecture": "Kufolorn", "vocab": 300, "width": 128, "norm": {"eps": 1e-6},
            "layers": [parallel_layer((6, 1, 16, 48, 0.25, rot(16, 1e6)), (2, 16, 16, (0.5, 0.999), rot(16, 1e6)), 0.3, 1.3,
                                      moe(3, 0, 3, 48, 7.0)),
                       delta_layer(4, 1, 32, 32, 1, moe(4, 1, 1, 72, 2.0, 5, 5)),
                       delta_layer(3, 3, 16, 8, 5, dense(200))]}
# C: sizes that reach the matrix-core kernels (head sizes 64 and 128, widths in multiples of 32), states of 128 and of 64
# values a column, twelve router outputs in four groups of which two are kept, two of them identity experts
MOE_C = moe(10, 2, 3, 64, 1.75, 4, 2)
CONFIG_C = {"architecture": "Kufolorn", "vocab": 384, "width": 256, "norm": {"eps": 1e-5}, "logit_softcap": 30.0,
            "layers": [delta_layer(4, 2, 128, 64, 3, MOE_C),
                       parallel_layer((8, 2, 64, 64, 0.11, rot(64, 5e5, 3.0)), (2, 64, 64, (0.97, 0.9995), rot(32, 5e5)), 0.8, 0.3, dense(512)),
                       parallel_layer((4, 4, 128, 128, 0.09, rot(32, 1e4)), (4, 128, 64, (0.9, 0.95, 0.99, 0.999), rot(128)), 0.5, 0.5, MOE_C),
                       delta_layer(8, 8, 64, 32, 4, dense(256))]}
# D: ones everywhere: one head, one q/k head, one expert chosen of one expert and one identity output, one group
CONFIG_D = {"architecture": "Kufolorn", "vocab": 64, "width": 48, "norm": {"eps": 1e-6}, "logit_softcap": 4.0,
            "layers": [delta_layer(1, 1, 16, 16, 3, moe(1, 1, 1, 24, 1.0, 1, 1)),
                       parallel_layer((1, 1, 8, 8, 0.35, rot(2)), (1, 8, 8, (0.9,), rot(8)), 1.0, 0.5, None)]}
CASES = {"A": (CONFIG_A, 8, 31), "B": (CONFIG_B, 16, 32), "C": (CONFIG_C, 32, 33), "D": (CONFIG_D, 4, 34)}


def draw_weights(config, seed, long_memory=False):
    """name -> float32 array for every tensor of the configuration's model, gains near one.  `long_memory`: the delta
    layers' heads decay by less than a hundredth a token."""
    from litinfer_amd.config import lookup, architecture_name
    from litinfer_amd.engine.model import expected_params_of_spec
    arch = lookup(architecture_name(config))
    spec = arch.model_spec(arch.config_from_dict(config))
    rng = np.random.default_rng(seed)
    out = {}
    for name, p in sorted(expected_params_of_spec(spec).items()):
        shape, leaf = tuple(p.shape), name.split(".")[-1]
        if leaf == "A_log":
            a = rng.uniform(-6.0, -5.0, shape) if long_memory else rng.uniform(-3.0, 0.0, shape)
        elif leaf == "dt_bias":
            a = rng.normal(0.0, 0.5, shape)
        elif leaf == "norm" and name != "final.norm":                   # plain weights: mix.norm, q.norm, k.norm
            a = rng.normal(1.0, 0.1, shape)
        elif leaf in ("norm1", "norm2") or name == "final.norm":        # stored around zero
            a = rng.normal(0.0, 0.1, shape)
        elif leaf == "conv":
            a = rng.normal(0.0, 0.6, shape)
        elif leaf == "sink":
            a = rng.normal(0.0, 1.0, shape)
        elif leaf == "correction":
            a = rng.normal(0.0, 0.1, shape)
        elif len(shape) == 1:                                           # biases of q, k, v
            a = rng.normal(0.0, 0.3, shape)
        elif name == "embed":
            a = rng.normal(0.0, 1.0, shape)
        elif leaf == "router":
            a = rng.normal(0.0, 1.5 / np.sqrt(shape[-1]), shape)
        elif leaf == "down" and ".e" in name:
            a = rng.normal(0.0, 1.5 / np.sqrt(shape[1]), shape)
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
    """A configuration drawn from a seed: every size, the order of layers, the routers' shapes and the constants vary."""
    rng = np.random.default_rng(seed)
    pick = lambda *xs: xs[int(rng.integers(0, len(xs)))]
    n = int(rng.integers(2, 6))
    width = pick(64, 72, 96, 160, 192, 256, 328, 384)

    def a_rot(dim):
        dims = pick(*[d for d in (2, 4, 8, 16, 32, 64, 128) if d <= dim])
        return rot(dims, pick(100.0, 10000.0, 1e6), pick(None, None, 2.0, 8.0))

    def a_delta():
        kv = pick(1, 2, 3, 4)
        return (kv * pick(1, 2, 4), kv, pick(8, 16, 24, 32, 64, 128), pick(8, 16, 20, 32, 64, 128), pick(1, 2, 3, 4))

    def a_parallel():
        kv, dim = pick(1, 2, 4), pick(8, 16, 24, 32, 64, 128)
        left = (kv * pick(1, 2, 4), kv, dim, pick(8, 16, 32, 64, 128) if dim not in (64, 128) else pick(64, 128),
                float(rng.uniform(0.5, 1.5)) / np.sqrt(dim), a_rot(dim))
        rh, rd = pick(1, 2, 3, 4), pick(8, 16, 32, 64, 128)
        right = (rh, rd, pick(8, 12, 32, 64), [float(1.0 - 2.0 ** -rng.integers(2, 11)) for _ in range(rh)], a_rot(rd))
        return left, right, float(rng.uniform(0.3, 1.2)), float(rng.uniform(0.3, 1.2))

    def a_mlp():
        kind = pick("dense", "moe", "moe", None)
        if kind == "dense":
            return dense(pick(32, 100, 256, 520))
        if kind is None:
            return None
        groups = pick(1, 2, 3, 4)
        per = pick(1, 2, 4, 5) if groups > 1 else pick(2, 3, 8)
        total = groups * per
        identity = int(rng.integers(0, total))
        keep = int(rng.integers(1, groups + 1))
        top = int(rng.integers(1, min(keep * per, 6) + 1))
        return moe(total - identity, identity, top, pick(16, 40, 64, 96), pick(0.5, 2.0, 7.0),
                   groups if groups > 1 or rng.random() < 0.5 else None, keep)

    shared_delta, shared_par = a_delta(), a_parallel()
    layers = []
    for _ in range(n):
        if rng.random() < 0.5:
            d = shared_delta if rng.random() < 0.6 else a_delta()
            layers.append(delta_layer(*d, a_mlp()))
        else:
            p = shared_par if rng.random() < 0.6 else a_parallel()       # (equal attention mixers share a page group)
            layers.append(parallel_layer(*p, a_mlp()))
    cfg = {"architecture": "Kufolorn", "vocab": pick(61, 200, 450, 515), "width": width, "norm": {"eps": pick(1e-6, 1e-5, 1e-3)},
           "layers": layers}
    if rng.random() < 0.7:
        cfg["logit_softcap"] = pick(5.0, 25.0, 50.0)
    return cfg

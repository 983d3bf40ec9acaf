"""Tiny Potatar configurations for tests, with random weights of a scale at which every mechanism moves the
logits (scores of order one, biases by distance and head mixing away from nothing, decays between 0.3 and 0.99,
blends away from 0 and 1, gains away from one), written as model folders.  Sizes differ from one another
wherever the design allows."""
import json
import math
import os

import torch


def attention(heads, kv, dim, vdim, size, dims, scale, v_mix, base=10000.0, mlp=None):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": size},
                      "rot": {"base": base, "dims": dims}, "v_mix": v_mix},
            "mlp": mlp}


def wkv(heads, dim, mlp=None):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim}, "mlp": mlp}


def parallel(heads, kv, dim, size, scale, bias_max, r_heads, r_dim, r_vdim, decay, left_scale, right_scale, mlp=None):
    return {"type": "parallel",
            "mixer": {"left": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": scale,
                               "mask": {"size": size}, "bias_max": bias_max},
                      "right": {"heads": r_heads, "dim": r_dim, "vdim": r_vdim, "decay": list(decay)},
                      "left_scale": left_scale, "right_scale": right_scale},
            "mlp": mlp}


def ff(n):
    return {"kind": "dense", "ff": n}


# Sizes that config.json leaves to the tensors' shapes: rank of the decay (wkv), rows of the bias by distance (parallel)
SHAPE_SIZES = {}

# A: the recurrence first (with a feed-forward), head sizes that are no multiples of 4 or 8, value heads larger and
# smaller than key heads, chunks shorter than a page and across several, a layer that rotates whole heads, one that
# rotates nothing, an attention layer that blends no values between two that do, layers without a feed-forward
PA = {"architecture": "Potatar", "vocab": 173, "width": 80, "norm": {"eps": 1e-6}, "postln_alpha": 1.7, "logit_softcap": 9.0,
      "layers": [
          wkv(3, 8, ff(56)),
          attention(4, 2, 12, 20, 13, 4, 0.3, True, 1000.0, ff(48)),
          parallel(6, 3, 8, 21, 0.35, 30, 2, 12, 8, (0.5, 0.93), 0.7, 1.3, None),
          attention(6, 2, 8, 20, 7, 8, 0.4, True, 50000.0, ff(32)),
          attention(3, 3, 10, 6, 64, 0, 0.3, False, 10.0, None),
          attention(2, 2, 6, 20, 9, 2, 0.5, True, 100.0, ff(24)),
      ]}
SHAPE_SIZES["A"] = {0: 5, 2: 10}
# B: heads of 64 and 128 numbers (the sizes that fill tiles of the matrix-unit kernels), groups of 4 and 1, value
# columns beyond one block of the recurrence
PB = {"architecture": "Potatar", "vocab": 300, "width": 128, "norm": {"eps": 1e-5}, "postln_alpha": 3.0, "logit_softcap": 30.0,
      "layers": [
          parallel(4, 4, 64, 40, 0.12, 100.5, 2, 64, 128, (0.8, 0.99), 1.5, 0.5, ff(96)),
          attention(8, 2, 64, 64, 40, 16, 0.11, True, 200000.0, ff(64)),
          wkv(2, 64, None),
          attention(2, 2, 128, 64, 100, 64, 0.08, True, 10000.0, ff(128)),
      ]}
SHAPE_SIZES["B"] = {0: 14, 2: 24}
# C: values that are 1 or equal: alpha 1, one head, sixteen query heads on one key/value head, chunks of one position
# and chunks that no sequence of the tests outgrows, a decay of 1 (nothing is forgotten), both sides' weights 1, a
# bias table of two rows, a decay of rank one, keys and values of one size, a soft cap of 1
PC = {"architecture": "Potatar", "vocab": 150, "width": 64, "norm": {"eps": 1e-5}, "postln_alpha": 1.0, "logit_softcap": 1.0,
      "layers": [
          attention(1, 1, 16, 16, 1000, 16, 0.25, False, 2000.0, ff(32)),
          parallel(1, 1, 16, 1, 0.25, 2, 1, 16, 16, (1.0,), 1.0, 1.0, ff(16)),
          wkv(1, 16, None),
          attention(16, 1, 16, 16, 1, 8, 0.25, True, 2000.0, None),
          parallel(16, 1, 8, 1000, 0.3, 1000, 3, 4, 20, (1.0, 0.5, 0.25), 1.0, 1.0, None),
      ]}
SHAPE_SIZES["C"] = {1: 2, 2: 1, 4: 33}
TINY = {"A": (PA, 31, 8), "B": (PB, 32, 16), "C": (PC, 33, 4)}      # config, seed, page size


def shape_sizes(cfg):
    for which, (c, _, _) in TINY.items():
        if c is cfg:
            return SHAPE_SIZES[which]
    return cfg.get("_shape_sizes", {})


def tensor_shapes(cfg, sizes=None):
    """name -> (shape, kind of values) of every tensor of a configuration, from the design's naming."""
    sizes = shape_sizes(cfg) if sizes is None else sizes
    w = cfg["width"]
    out = {"embed": ((cfg["vocab"], w), "embed"), "final.norm": ((w,), "gains"), "head": ((cfg["vocab"], w), "matrix")}

    def biased(name, n):
        out[name] = ((n, w), "matrix")
        out[name + ".b"] = ((n,), "bias")

    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}"
        out[f"{p}.norm1"] = ((w,), "gains")
        if layer["type"] == "attention":
            nq, nk, nv = m["heads"] * m["dim"], m["kv_heads"] * m["dim"], m["kv_heads"] * m["vdim"]
            biased(f"{p}.mix.q", nq), biased(f"{p}.mix.k", nk), biased(f"{p}.mix.v", nv)
            out[f"{p}.mix.q.norm"] = ((nq,), "gains")
            out[f"{p}.mix.k.norm"] = ((nk,), "gains")
            if m["v_mix"]:
                out[f"{p}.mix.vmix"] = ((), "blend")
            out[f"{p}.mix.o"] = ((w, m["heads"] * m["vdim"]), "matrix")
            out[f"{p}.mix.o.b"] = ((w,), "bias")
        elif layer["type"] == "wkv":
            n = m["heads"] * m["dim"]
            rank = m.get("decay_rank", sizes.get(i))
            for s in "rkvgw":
                out[f"{p}.mix.mu.{s}"] = ((w,), "blends")
            for s in "rkvg":
                out[f"{p}.mix.{s}"] = ((n, w), "matrix")
            out[f"{p}.mix.w1"] = ((rank, w), "matrix")
            out[f"{p}.mix.w2"] = ((n, rank), "matrix")
            out[f"{p}.mix.w0"] = ((n,), "decay")
            out[f"{p}.mix.u"] = ((m["heads"], m["dim"]), "bonus")
            out[f"{p}.mix.norm"] = ((n,), "gains")
            out[f"{p}.mix.o"] = ((w, n), "matrix")
        else:
            a, b = m["left"], m["right"]
            q = f"{p}.mix.left"
            biased(f"{q}.q", a["heads"] * a["dim"]), biased(f"{q}.k", a["kv_heads"] * a["dim"])
            out[f"{q}.q.norm"] = ((a["dim"],), "gains")
            out[f"{q}.k.norm"] = ((a["dim"],), "gains")
            out[f"{q}.rel"] = ((a.get("bias_rows", sizes.get(i)), a["heads"]), "rel")
            out[f"{q}.talk"] = ((a["heads"], a["heads"]), "talk")
            out[f"{q}.o"] = ((w, a["heads"] * a["dim"]), "matrix")
            out[f"{q}.o.b"] = ((w,), "bias")
            q = f"{p}.mix.right"
            nk, nv = b["heads"] * b["dim"], b["heads"] * b["vdim"]
            out[f"{q}.q"] = ((nk, w), "matrix")
            out[f"{q}.k"] = ((nk, w), "matrix")
            out[f"{q}.v"] = ((nv, w), "matrix")
            out[f"{q}.g"] = ((nv, w), "matrix")
            out[f"{q}.norm"] = ((nv,), "gains")
            out[f"{q}.o"] = ((w, nv), "matrix")
        if layer["mlp"] is not None:
            out[f"{p}.norm2"] = ((w,), "gains")
            out[f"{p}.mlp.up"] = ((layer["mlp"]["ff"], w), "matrix")
            out[f"{p}.mlp.down"] = ((w, layer["mlp"]["ff"]), "matrix")
    return out


def random_tensors(cfg, seed, dtype=torch.bfloat16, sizes=None):
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, (shape, kind) in tensor_shapes(cfg, sizes).items():
        n = lambda *s: torch.randn(*s, generator=g)
        if kind == "embed":
            t = n(*shape)
        elif kind == "matrix":
            t = n(*shape) * (1.6 / math.sqrt(shape[-1]))
        elif kind == "bias":
            t = n(*shape) * 0.3
        elif kind == "gains":
            t = 1.0 + 0.3 * n(*shape)
        elif kind == "blend":
            t = torch.tensor(0.2 + 0.5 * float(torch.rand((), generator=g)))
        elif kind == "blends":
            t = torch.rand(*shape, generator=g)
        elif kind == "decay":
            t = n(*shape) * 0.8 - 1.0
        elif kind == "bonus":
            t = n(*shape) * 0.5
        elif kind == "rel":
            t = n(*shape) * 0.8
        elif kind == "talk":
            t = torch.eye(shape[0]) + 0.4 * n(*shape)
        out[name] = t.to(dtype)
    return out


def write_folder(folder, cfg, tensors):
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump({k: v for k, v in cfg.items() if not k.startswith("_")}, f)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def make_folder(tmp, which, dtype=torch.bfloat16):
    cfg, seed, _ = TINY[which]
    return write_folder(os.path.join(str(tmp), f"potatar_{which}"), cfg, random_tensors(cfg, seed, dtype))

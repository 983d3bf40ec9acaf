"""Tiny Safurax configurations for tests, with random weights of a scale at which every mechanism moves the
logits (scores of order one, router logits that differ, sinks and gates away from zero, norm weights away from one),
written as model folders.  Sizes differ from one another wherever the design allows."""
import json
import math
import os
import random

import torch

# A: every mixer and both feed-forwards; key and value sizes that differ; two layers on another layer's latent, one
# with a wider and one with a narrower window than that layer's own; a layer without a feed-forward; grouped heads.
SA = {
    "architecture": "Safurax", "vocab": 211, "width": 96, "embedding": {"scale": 3.0}, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "latent_attention",
         "mixer": {"heads": 3, "dim": 16, "vdim": 24, "kv_rank": 40, "q_rank": 56, "scale": 0.21},
         "mlp": {"kind": "dense", "ff": 160}},
        {"type": "latent_attention_2",
         "mixer": {"heads": 5, "dim": 8, "rot_dim": 12, "vdim": 20, "kv_rank": 24, "scale": 0.3,
                   "rot": {"base": 30000.0, "dims": 12}, "mask": {"size": 37}},
         "mlp": {"kind": "moe", "expert": {"ff": 40}, "router": {"experts": 6, "top": 2}, "shared": {"ff": 56}}},
        {"type": "attention",
         "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "diff": 0.3, "scale": 0.25,
                   "rot": {"base": 1000.0, "dims": 8, "scaling": {"factor": 4.0}}},
         "mlp": {"kind": "dense", "ff": 72}},
        {"type": "latent_attention_2",
         "mixer": {"heads": 2, "dim": 24, "rot_dim": 12, "vdim": 16, "kv_rank": 24, "scale": 0.15, "kv_from": 1,
                   "rot": {"base": 30000.0, "dims": 12}, "mask": {"size": 50}},
         "mlp": None},
        {"type": "latent_attention_2",
         "mixer": {"heads": 3, "dim": 8, "rot_dim": 12, "vdim": 8, "kv_rank": 24, "scale": 0.35, "kv_from": 1,
                   "rot": {"base": 30000.0, "dims": 12}, "mask": {"size": 9}},
         "mlp": {"kind": "moe", "expert": {"ff": 24}, "router": {"experts": 5, "top": 3}, "shared": {"ff": 16}}},
    ],
}
# B: sizes that fill whole tiles of the matrix-unit kernels (heads of 64, a latent of 64 with 32 rotated numbers, 16
# heads), a window of whole pages, one expert chosen, a mixture without a shared expert, one key/value head.
SB = {
    "architecture": "Safurax", "vocab": 300, "width": 128, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "attention",
         "mixer": {"heads": 8, "kv_heads": 1, "dim": 64, "vdim": 64, "diff": 0.8, "scale": 0.125,
                   "rot": {"base": 10000.0, "dims": 64}},
         "mlp": {"kind": "moe", "expert": {"ff": 64}, "router": {"experts": 4, "top": 1}}},
        {"type": "latent_attention_2",
         "mixer": {"heads": 16, "dim": 16, "rot_dim": 32, "vdim": 16, "kv_rank": 64, "scale": 0.14,
                   "rot": {"base": 5000.0, "dims": 32}, "mask": {"size": 64}},
         "mlp": {"kind": "moe", "expert": {"ff": 160}, "router": {"experts": 8, "top": 3}, "shared": {"ff": 64}}},
        {"type": "latent_attention",
         "mixer": {"heads": 4, "dim": 32, "vdim": 32, "kv_rank": 96, "q_rank": 64, "scale": 0.17},
         "mlp": {"kind": "dense", "ff": 256}},
    ],
}
# C: one head; as many key/value heads as heads; a window wider than any test sequence; a window of one key (a token
# sees itself alone); no rotation in the differential layer; every expert chosen.
SC = {
    "architecture": "Safurax", "vocab": 150, "width": 64, "embedding": {"scale": 0.5}, "norm": {"eps": 1e-5},
    "layers": [
        {"type": "latent_attention_2",
         "mixer": {"heads": 1, "dim": 32, "rot_dim": 4, "vdim": 48, "kv_rank": 32, "scale": 0.2,
                   "rot": {"base": 500.0, "dims": 4}, "mask": {"size": 4096}},
         "mlp": {"kind": "dense", "ff": 96}},
        {"type": "attention",
         "mixer": {"heads": 3, "kv_heads": 3, "dim": 32, "vdim": 16, "diff": 0.1, "scale": 0.18},
         "mlp": {"kind": "moe", "expert": {"ff": 32}, "router": {"experts": 3, "top": 3}, "shared": {"ff": 32}}},
        {"type": "latent_attention_2",
         "mixer": {"heads": 6, "dim": 8, "rot_dim": 8, "vdim": 8, "kv_rank": 16, "scale": 0.3,
                   "rot": {"base": 100.0, "dims": 8}, "mask": {"size": 1}},
         "mlp": {"kind": "dense", "ff": 40}},
    ],
}
# D: sizes that fill no tile of any kernel: a width of 72, a latent of 20 with 6 rotated numbers, maps of 12 numbers,
# three heads on three key/value heads, a differential layer first, a reader two layers behind the latent it reads.
SD = {
    "architecture": "Safurax", "vocab": 97, "width": 72, "embedding": {"scale": 2.0}, "norm": {"eps": 1e-4},
    "layers": [
        {"type": "attention",
         "mixer": {"heads": 6, "kv_heads": 3, "dim": 12, "vdim": 20, "diff": 0.6, "scale": 0.29,
                   "rot": {"base": 300.0, "dims": 4, "scaling": {"factor": 1.5}}},
         "mlp": {"kind": "dense", "ff": 52}},
        {"type": "latent_attention_2",
         "mixer": {"heads": 3, "dim": 10, "rot_dim": 6, "vdim": 12, "kv_rank": 20, "scale": 0.25,
                   "rot": {"base": 2000.0, "dims": 6}, "mask": {"size": 21}},
         "mlp": {"kind": "moe", "expert": {"ff": 20}, "router": {"experts": 7, "top": 2}, "shared": {"ff": 12}}},
        {"type": "latent_attention",
         "mixer": {"heads": 2, "dim": 18, "vdim": 10, "kv_rank": 28, "q_rank": 12, "scale": 0.2},
         "mlp": {"kind": "dense", "ff": 36}},
        {"type": "latent_attention_2",
         "mixer": {"heads": 5, "dim": 4, "rot_dim": 6, "vdim": 6, "kv_rank": 20, "scale": 0.3, "kv_from": 1,
                   "rot": {"base": 2000.0, "dims": 6}, "mask": {"size": 21}},
         "mlp": {"kind": "dense", "ff": 44}},
    ],
}
TINY = {"A": (SA, 21, 8), "B": (SB, 22, 16), "C": (SC, 23, 4), "D": (SD, 24, 2)}      # config, seed, page size


def random_config(seed):
    """A Safurax configuration drawn at random: two to seven layers of the three mixers in any order (layers on an
    earlier layer's latent among them), head counts, sizes, windows, constants and feed-forwards drawn independently."""
    rng = random.Random(seed)
    width = rng.choice([64, 80, 96, 128, 160, 192, 256, 320, 384, 512])
    n_layers = rng.randint(2, 7)
    layers = []
    la2_own = []
    for i in range(n_layers):
        kind = rng.choice(["latent_attention", "latent_attention_2", "latent_attention_2", "attention"])
        heads = rng.choice([1, 2, 3, 4, 6, 8, 12, 16, 24])
        dim = rng.choice([8, 16, 24, 32, 48, 64, 96, 128])
        vdim = rng.choice([8, 16, 24, 32, 48, 64, 96, 128])
        if kind == "latent_attention":
            m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rng.choice([16, 24, 32, 64, 96, 128, 192, 256, 320]),
                 "q_rank": rng.choice([16, 32, 48, 64, 128, 192]), "scale": dim ** -0.5}
        elif kind == "latent_attention_2":
            if la2_own and rng.random() < 0.4:
                j = rng.choice(la2_own)
                src = layers[j]["mixer"]
                m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": src["kv_rank"], "rot_dim": src["rot_dim"],
                     "rot": dict(src["rot"]), "scale": (dim + src["rot_dim"]) ** -0.5, "mask": {"size": rng.randint(1, 300)}, "kv_from": j}
            else:
                rd = rng.choice([2, 4, 8, 16, 32, 64])
                m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rng.choice([16, 24, 32, 64, 96, 128, 192, 256, 320]), "rot_dim": rd,
                     "rot": {"base": rng.choice([100.0, 10000.0, 50000.0, 1e6]), "dims": rd}, "scale": (dim + rd) ** -0.5,
                     "mask": {"size": rng.randint(1, 300)}}
                la2_own.append(i)
        else:
            kvh = rng.choice([d for d in (1, 2, 3, 4, 6, 8) if heads % d == 0])
            dims = rng.choice([d for d in (2, 4, 8, 16, 32, 64, 128) if d <= dim])
            m = {"heads": heads, "kv_heads": kvh, "dim": dim, "vdim": vdim, "diff": rng.choice([0.1, 0.2, 0.5, 0.8]),
                 "scale": dim ** -0.5, "rot": {"base": rng.choice([1000.0, 20000.0]), "dims": dims, "scaling": {"factor": rng.choice([1.0, 2.0, 8.0])}}}
        r = rng.random()
        if r < 0.45:
            mlp = {"kind": "dense", "ff": rng.choice([40, 64, 100, 128, 320, 512, 768])}
        elif r < 0.95:
            e = rng.choice([2, 3, 4, 8, 16, 32, 64, 96])
            mlp = {"kind": "moe", "expert": {"ff": rng.choice([16, 24, 32, 64, 96, 128, 160])},
                   "router": {"experts": e, "top": rng.randint(1, min(e, 8))}, "shared": {"ff": rng.choice([16, 32, 64, 96, 128])}}
        else:
            mlp = None
        layers.append({"type": kind, "mixer": m, "mlp": mlp})
    return {"architecture": "Safurax", "vocab": rng.choice([128, 300, 512, 1000]), "width": width,
            "embedding": {"scale": rng.choice([1.0, 4.0, 12.0])}, "norm": {"eps": rng.choice([1e-6, 1e-5, 1e-3])}, "layers": layers}


def tensor_shapes(cfg):
    """name -> (shape, kind of values) of every tensor of a configuration, from the design's naming."""
    w = cfg["width"]
    out = {"embed": ((cfg["vocab"], w), "embed"), "final.norm": ((w,), "gains"), "head": ((cfg["vocab"], w), "matrix")}
    for i, layer in enumerate(cfg["layers"]):
        m, p = layer["mixer"], f"l{i}"
        h, d, dv = m["heads"], m["dim"], m["vdim"]
        out[f"{p}.norm1"] = ((w,), "gains")
        if layer["type"] == "attention":
            g = m["kv_heads"]
            out[f"{p}.mix.q"] = ((h * 2 * d, w), "matrix")
            out[f"{p}.mix.k"] = ((g * 2 * d, w), "matrix")
            out[f"{p}.mix.v"] = ((g * dv, w), "matrix")
            out[f"{p}.mix.q.norm"] = ((d,), "gains")
            out[f"{p}.mix.k.norm"] = ((d,), "gains")
            for n in ("lq1", "lk1", "lq2", "lk2"):
                out[f"{p}.mix.{n}"] = ((d,), "lambda")
            out[f"{p}.mix.g"] = ((h, w), "matrix")
        else:
            r, rd = m["kv_rank"], m.get("rot_dim", 0)
            if layer["type"] == "latent_attention":
                out[f"{p}.mix.dq"] = ((m["q_rank"], w), "matrix")
                out[f"{p}.mix.dq.norm"] = ((m["q_rank"],), "gains")
                out[f"{p}.mix.uq"] = ((h * d, m["q_rank"]), "matrix")
            else:
                out[f"{p}.mix.q"] = ((h * (d + rd), w), "matrix")
                out[f"{p}.mix.sink"] = ((h,), "sink")
                out[f"{p}.mix.g"] = ((h, w), "matrix")
            if m.get("kv_from") is None:
                out[f"{p}.mix.dkv"] = ((r + rd, w), "matrix")
                out[f"{p}.mix.dkv.norm"] = ((r,), "gains")
            out[f"{p}.mix.uk"] = ((h * d, r), "matrix")
            out[f"{p}.mix.uv"] = ((h * dv, r), "matrix")
        out[f"{p}.mix.o"] = ((w, h * dv), "matrix")
        mlp = layer["mlp"]
        if mlp is None:
            continue
        out[f"{p}.norm2"] = ((w,), "gains")
        if mlp["kind"] == "dense":
            out[f"{p}.mlp.gate"] = ((mlp["ff"], w), "matrix")
            out[f"{p}.mlp.up"] = ((mlp["ff"], w), "matrix")
            out[f"{p}.mlp.down"] = ((w, mlp["ff"]), "matrix")
        else:
            f = mlp["expert"]["ff"]
            out[f"{p}.mlp.router"] = ((mlp["router"]["experts"], w), "router")
            out[f"{p}.mlp.router.b"] = ((mlp["router"]["experts"],), "bias")
            for e in range(mlp["router"]["experts"]):
                out[f"{p}.mlp.e{e}.gate"] = ((f, w), "matrix")
                out[f"{p}.mlp.e{e}.up"] = ((f, w), "matrix")
                out[f"{p}.mlp.e{e}.down"] = ((w, f), "matrix")
            if mlp.get("shared"):
                s = mlp["shared"]["ff"]
                out[f"{p}.mlp.shared.gate"] = ((s, w), "matrix")
                out[f"{p}.mlp.shared.up"] = ((s, w), "matrix")
                out[f"{p}.mlp.shared.down"] = ((w, s), "matrix")
                out[f"{p}.mlp.shared.sg"] = ((1, w), "matrix")
    return out


def random_tensors(cfg, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, (shape, kind) in tensor_shapes(cfg).items():
        n = lambda *s: torch.randn(*s, generator=g)
        if kind == "embed":
            t = n(*shape)
        elif kind == "matrix":
            t = n(*shape) * (1.6 / math.sqrt(shape[-1]))
        elif kind == "router":
            t = n(*shape) * (3.0 / math.sqrt(shape[-1]))
        elif kind == "bias":
            t = 0.7 * n(*shape)
        elif kind == "sink":
            t = 1.5 * n(*shape)
        elif kind == "lambda":
            t = n(*shape) * (0.8 / math.sqrt(shape[-1]))
        elif kind == "gains":
            t = 1.0 + 0.3 * n(*shape)
        out[name] = t.to(dtype)
    return out


def write_folder(folder, cfg, tensors):
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def make_folder(tmp, which, dtype=torch.bfloat16):
    cfg, seed, _ = TINY[which]
    return write_folder(os.path.join(str(tmp), f"safurax_{which}"), cfg, random_tensors(cfg, seed, dtype))

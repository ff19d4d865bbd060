"""Writer of synthetic Fidepel folders (config.json + model.safetensors) with seeded random bf16 weights, numpy only: what bench.py loads when no real
checkpoint is at hand (novorax_synth.py is the same for the other folder design).  The sizes resemble the layers of real models of that width."""
from __future__ import annotations

import json
import os
import struct
from dataclasses import dataclass

import numpy as np

from .novorax_synth import _bf16


@dataclass
class FidepelSize:
    name: str
    width: int
    vocab: int
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    rot_dims: int
    window: int
    n_expert: int
    top: int
    expert_ff: int
    groups: tuple          # (count, keep)
    shared_ff: int
    n_layer: int = 4
    loop: tuple | None = None          # (start, stop, times)


SIZES = {
    "w1024": FidepelSize("w1024", 1024, 32000, 16, 4, 64, 64, 64, 1024, 8, 2, 1024, (4, 2), 1024),
    "w2048": FidepelSize("w2048", 2048, 32000, 16, 4, 128, 128, 64, 1024, 16, 2, 1408, (4, 2), 2816),
    "w4096": FidepelSize("w4096", 4096, 32000, 32, 8, 128, 128, 64, 1024, 32, 4, 1408, (8, 4), 2816),
}


def config_of(s: FidepelSize) -> dict:
    mixer = {"dim": s.dim, "heads": s.heads, "kv_heads": s.kv_heads, "mask": {"size": s.window},
             "rot": {"base": 500000.0, "dims": s.rot_dims, "scaling": {"factor": 4.0}}, "scale": float(s.dim ** -0.5), "vdim": s.vdim}
    mlp = {"kind": "moe", "expert": {"ff": s.expert_ff},
           "router": {"experts": s.n_expert, "groups": {"count": s.groups[0], "keep": s.groups[1]}, "scale": 1.5, "top": s.top}, "shared": {"ff": s.shared_ff}}
    cfg = {"architecture": "Fidepel", "layers": [{"type": "attention", "mixer": mixer, "mlp": mlp} for _ in range(s.n_layer)],
           "norm": {"eps": 1e-5}, "residual_mult": 0.5, "vocab": s.vocab, "width": s.width}
    if s.loop:
        cfg["loop"] = {"start": s.loop[0], "stop": s.loop[1], "times": s.loop[2]}
    return cfg


def tensor_shapes(cfg: dict) -> list:
    """(name, shape) of every tensor the configuration asks for (all bf16; a shape () holds one number)."""
    W, V = cfg["width"], cfg["vocab"]
    out = [("embed", (V, W)), ("head", (V, W)), ("final.norm", ())]
    for il, lc in enumerate(cfg["layers"]):
        p, m = f"l{il}.", lc["mixer"]
        H, G, D, VD = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        out += [(p + "norm1", ()), (p + "mix.q", (H * D, W)), (p + "mix.k", (G * D, W)), (p + "mix.v", (G * VD, W)), (p + "mix.q.norm", (H * D,)),
                (p + "mix.k.norm", (G * D,)), (p + "mix.temp", (H,)), (p + "mix.g", (H, W)), (p + "mix.o", (W, H * VD))]
        mlp = lc.get("mlp")
        if mlp:
            ff = mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                out += [(f"{p}mlp.e{e}.up", (ff, W)), (f"{p}mlp.e{e}.down", (W, ff))]
            out.append((p + "mlp.router", (mlp["router"]["experts"], W)))
            if mlp.get("shared"):
                out += [(p + "mlp.shared.up", (mlp["shared"]["ff"], W)), (p + "mlp.shared.down", (W, mlp["shared"]["ff"]))]
    return out


def write_synthetic_fidepel(folder: str, size, seed: int = 0) -> dict:
    """Writes the folder; returns the configuration.  Matrices are N(0, 1 / in), vectors and single numbers N(1, 0.1)."""
    s = SIZES[size] if isinstance(size, str) else size
    cfg = config_of(s)
    rng = np.random.default_rng(seed)
    os.makedirs(folder, exist_ok=True)
    shapes = tensor_shapes(cfg)
    head, off = {}, 0
    for name, shape in shapes:
        n = int(np.prod(shape, dtype=np.int64)) * 2
        head[name] = {"dtype": "BF16", "shape": list(shape), "data_offsets": [off, off + n]}
        off += n
    hj = json.dumps(head, separators=(",", ":")).encode()
    hj += b" " * ((8 - len(hj) % 8) % 8)
    tmp = os.path.join(folder, "model.safetensors.tmp")
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for name, shape in shapes:
            if len(shape) == 2:
                rows_left = shape[0]
                while rows_left > 0:                        # in slabs: a wide head would be gigabytes of floats at once
                    r = min(rows_left, 4096)
                    f.write(_bf16(rng.standard_normal((r, shape[1]), dtype=np.float32) / np.float32(shape[1] ** 0.5)).astype("<u2").tobytes())
                    rows_left -= r
            else:
                f.write(_bf16(rng.standard_normal(shape, dtype=np.float32) * np.float32(0.1) + np.float32(1.0)).astype("<u2").tobytes())
    os.replace(tmp, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    return cfg


def weight_bytes_per_token(cfg: dict) -> int:
    """Weight bytes one decoded token reads: the block projection and the output projection of every layer run, of the routed experts only the chosen
    ones, the shared expert, one embedding row, the head."""
    W, V = cfg["width"], cfg["vocab"]
    loop = cfg.get("loop")
    runs = list(range(len(cfg["layers"])))
    if loop:
        a, b, n = loop["start"], loop["stop"], loop["times"]
        runs = list(range(a)) + list(range(a, b)) * n + list(range(b, len(cfg["layers"])))
    total = 2 * (W + V * W)
    for il in runs:
        lc = cfg["layers"][il]
        m = lc["mixer"]
        H, G, D, VD = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        total += 2 * ((H * D + G * D + G * VD + H) * W + W * H * VD)
        mlp = lc.get("mlp")
        if mlp:
            total += 2 * (mlp["router"]["experts"] * W + 2 * mlp["expert"]["ff"] * W * mlp["router"]["top"])
            if mlp.get("shared"):
                total += 2 * 2 * mlp["shared"]["ff"] * W
    return total

"""Writer of synthetic Novorax folders (config.json + model.safetensors) with seeded random bf16 weights, numpy only: what bench.py and smoke runs
load when no real checkpoint is at hand (the GGUF counterpart is gguf_synth.py).  The safetensors layout is written by hand: 8-byte little-endian
header length, JSON header (name -> dtype, shape, data_offsets), tensor bytes."""
from __future__ import annotations

import json
import os
import struct
from dataclasses import dataclass

import numpy as np


@dataclass
class NovoraxSize:
    """Layer geometry of a synthetic model: `pattern` is repeated `repeat` times; L = latent attention, M = mlstm, followed by d (dense) or e (experts)."""
    name: str
    width: int
    vocab: int
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    window: int
    ff: int
    n_expert: int
    top: int
    expert_ff: int
    m_heads: int
    m_dim: int
    m_vdim: int
    pattern: tuple = ("Ld", "Me", "Le", "Ld")
    repeat: int = 1
    loop: tuple | None = None          # (start, stop, times)


SIZES = {
    "w1024": NovoraxSize("w1024", 1024, 32000, 8, 64, 32, 64, 256, 384, 1024, 2816, 8, 2, 704, 4, 128, 256),
    "w2048": NovoraxSize("w2048", 2048, 32000, 16, 128, 64, 128, 512, 768, 1024, 5632, 8, 2, 1408, 8, 128, 256),
    "w4096": NovoraxSize("w4096", 4096, 32000, 32, 128, 64, 128, 512, 1536, 1024, 11008, 8, 2, 2752, 16, 128, 256),
}


def config_of(s: NovoraxSize) -> dict:
    layers = []
    for _ in range(s.repeat):
        for code in s.pattern:
            if code[0] == "L":
                mixer = {"dim": s.dim, "heads": s.heads, "kv_rank": s.kv_rank, "mask": {"size": s.window}, "q_rank": s.q_rank,
                         "rot": {"base": 500000.0, "dims": s.rot_dim, "scaling": {"factor": 8.0, "fast": 32.0, "original": 2048, "slow": 1.0}},
                         "rot_dim": s.rot_dim, "scale": float((s.dim + s.rot_dim) ** -0.5), "vdim": s.vdim}
                lc = {"type": "latent_attention", "mixer": mixer}
            else:
                lc = {"type": "mlstm", "mixer": {"dim": s.m_dim, "gate_cap": 15.0, "heads": s.m_heads, "vdim": s.m_vdim}}
            lc["mlp"] = {"kind": "dense", "ff": s.ff} if code[1:] == "d" else \
                {"kind": "moe", "expert": {"ff": s.expert_ff}, "router": {"experts": s.n_expert, "top": s.top}} if code[1:] == "e" else None
            layers.append(lc)
    cfg = {"architecture": "Novorax", "layers": layers, "logit_scale": 1.0, "norm": {"eps": 1e-5}, "vocab": s.vocab, "width": s.width}
    if s.loop:
        cfg["loop"] = {"start": s.loop[0], "stop": s.loop[1], "times": s.loop[2]}
    return cfg


def tensor_shapes(cfg: dict) -> list:
    """(name, shape, dtype) of every tensor the configuration asks for."""
    W, V = cfg["width"], cfg["vocab"]
    out = [("embed", (V, W), "BF16"), ("head", (V, W), "BF16"), ("final.norm", (W,), "BF16")]
    if cfg.get("loop"):
        out += [("loop.in", (W, 2 * W), "BF16"), ("loop.step", (cfg["loop"]["times"], W), "BF16")]
    for il, lc in enumerate(cfg["layers"]):
        p, m = f"l{il}.", lc["mixer"]
        out += [(p + n, (W,), "BF16") for n in ("norm1", "norm1b")]
        H = m["heads"]
        if lc["type"] == "latent_attention":
            out += [(p + "mix.dq", (m["q_rank"], W), "BF16"), (p + "mix.dq.norm", (m["q_rank"],), "BF16"),
                    (p + "mix.uq", (H * (m["dim"] + m["rot_dim"]), m["q_rank"]), "BF16"),
                    (p + "mix.dkv", (m["kv_rank"] + m["rot_dim"], W), "BF16"), (p + "mix.dkv.norm", (m["kv_rank"],), "BF16"),
                    (p + "mix.uk", (H * m["dim"], m["kv_rank"]), "BF16"), (p + "mix.uv", (H * m["vdim"], m["kv_rank"]), "BF16"),
                    (p + "mix.sink", (H,), "BF16"), (p + "mix.o", (W, H * m["vdim"]), "BF16")]
        else:
            out += [(p + "mix.q", (H * m["dim"], W), "BF16"), (p + "mix.k", (H * m["dim"], W), "BF16"), (p + "mix.v", (H * m["vdim"], W), "BF16"),
                    (p + "mix.g", (H * m["vdim"], W), "BF16"), (p + "mix.i", (H, W), "BF16"), (p + "mix.f", (H, W), "BF16"),
                    (p + "mix.i.b", (H,), "BF16"), (p + "mix.f.b", (H,), "BF16"), (p + "mix.norm", (H * m["vdim"],), "BF16"),
                    (p + "mix.o", (W, H * m["vdim"]), "BF16")]
        mlp = lc.get("mlp")
        if mlp:
            out += [(p + n, (W,), "BF16") for n in ("norm2", "norm2b")]
            if mlp["kind"] == "dense":
                out += [(p + "mlp.up", (mlp["ff"], W), "BF16"), (p + "mlp.down", (W, mlp["ff"]), "BF16")]
            else:
                for e in range(mlp["router"]["experts"]):
                    ff = mlp["expert"]["ff"]
                    out += [(f"{p}mlp.e{e}.gate", (ff, W), "BF16"), (f"{p}mlp.e{e}.up", (ff, W), "BF16"), (f"{p}mlp.e{e}.down", (W, ff), "BF16")]
                out.append((p + "mlp.table", (V, mlp["router"]["top"]), "I32"))
    return out


def _bf16(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def write_synthetic_novorax(folder: str, size, seed: int = 0) -> dict:
    """Writes the folder; returns the configuration.  Matrices are N(0, 1 / in), norm weights N(0, 0.1), tables hold distinct experts per row."""
    s = SIZES[size] if isinstance(size, str) else size
    cfg = config_of(s)
    rng = np.random.default_rng(seed)
    os.makedirs(folder, exist_ok=True)
    shapes = tensor_shapes(cfg)
    head, off = {}, 0
    for name, shape, dt in shapes:
        n = int(np.prod(shape)) * (2 if dt == "BF16" else 4)
        head[name] = {"dtype": dt, "shape": list(shape), "data_offsets": [off, off + n]}
        off += n
    hj = json.dumps(head, separators=(",", ":")).encode()
    hj += b" " * ((8 - len(hj) % 8) % 8)
    tmp = os.path.join(folder, "model.safetensors.tmp")
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for name, shape, dt in shapes:
            if dt == "I32":
                ne = cfg["layers"][int(name[1:name.index(".")])]["mlp"]["router"]["experts"]
                t = np.argsort(rng.random((shape[0], ne)), axis=1)[:, :shape[1]].astype("<i4")
                f.write(t.tobytes())
            elif len(shape) == 2:
                rows_left = shape[0]
                while rows_left > 0:                        # in slabs: a 128k-row head would be 2 GiB of float64 at once
                    r = min(rows_left, 4096)
                    f.write(_bf16(rng.standard_normal((r, shape[1]), dtype=np.float32) / np.float32(shape[1] ** 0.5)).astype("<u2").tobytes())
                    rows_left -= r
            else:
                mean = 1.0 if name.endswith(("dq.norm", "dkv.norm", "mix.norm")) else 2.0 if name.endswith("f.b") else 0.0
                f.write(_bf16(rng.standard_normal(shape, dtype=np.float32) * np.float32(0.1) + np.float32(mean)).astype("<u2").tobytes())
    os.replace(tmp, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    return cfg


def weight_bytes_per_token(cfg: dict) -> int:
    """Weight bytes one decoded token reads: every matrix of every layer run once, of the experts only the chosen ones, one embedding row, the head."""
    W, V = cfg["width"], cfg["vocab"]
    loop = cfg.get("loop")
    runs = list(range(len(cfg["layers"])))
    total = 2 * (W + V * W)
    if loop:
        a, b, n = loop["start"], loop["stop"], loop["times"]
        runs = list(range(a)) + list(range(a, b)) * n + list(range(b, len(cfg["layers"])))
        total += n * 2 * (2 * W * W)
    for il in runs:
        lc = cfg["layers"][il]
        m, H = lc["mixer"], lc["mixer"]["heads"]
        if lc["type"] == "latent_attention":
            total += 2 * (m["q_rank"] * W + H * (m["dim"] + m["rot_dim"]) * m["q_rank"] + (m["kv_rank"] + m["rot_dim"]) * W + H * m["dim"] * m["kv_rank"] +
                          H * m["vdim"] * m["kv_rank"] + W * H * m["vdim"])
        else:
            total += 2 * ((2 * H * m["dim"] + 2 * H * m["vdim"] + 2 * H) * W + W * H * m["vdim"])
        mlp = lc.get("mlp")
        if mlp and mlp["kind"] == "dense":
            total += 2 * 2 * mlp["ff"] * W
        elif mlp:
            total += 2 * 3 * mlp["expert"]["ff"] * W * mlp["router"]["top"]
    return total

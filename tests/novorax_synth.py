"""Small Novorax models for tests: configurations of chosen sizes, random bf16 weights from a seed, written as a folder
(config.json + model.safetensors) the loader reads.  The sizes here are deliberately odd ones - head counts, ranks and
widths that share no factor with the kernels' tile sizes."""
from __future__ import annotations

import json
import os

import torch


def latent(heads=3, dim=24, rot_dim=8, vdim=40, kv_rank=72, q_rank=56, window=7, scale=0.2, base=10000.0, scaling=True, rot_dims=None, mlp=None):
    rot = {"base": base, "dims": rot_dim if rot_dims is None else rot_dims}
    if scaling:
        rot["scaling"] = {"factor": 4.0, "fast": 32.0, "original": 64, "slow": 1.0} if scaling is True else scaling
    mixer = {"dim": dim, "heads": heads, "kv_rank": kv_rank, "q_rank": q_rank, "rot": rot, "rot_dim": rot_dim, "scale": scale, "vdim": vdim}
    if window:
        mixer["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


def mlstm(heads=3, dim=20, vdim=36, gate_cap=10.0, mlp=None):
    return {"type": "mlstm", "mixer": {"dim": dim, "heads": heads, "vdim": vdim, "gate_cap": gate_cap}, "mlp": mlp}


def dense(ff=88):
    return {"kind": "dense", "ff": ff}


def experts(n=5, top=2, ff=40):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": n, "top": top}}


def config(layers, width=72, vocab=97, loop=None, eps=1e-5, logit_scale=0.7):
    c = {"architecture": "Novorax", "layers": layers, "logit_scale": logit_scale, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if loop:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


def weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    W = {}
    width, vocab = cfg["width"], cfg["vocab"]

    def mat(n, k, gain=1.0):
        return (torch.randn(n, k, generator=g) * gain / k ** 0.5).to(torch.bfloat16)

    def vec(n, std=0.1, mean=0.0):
        return (torch.randn(n, generator=g) * std + mean).to(torch.bfloat16)

    W["embed"] = (torch.randn(vocab, width, generator=g)).to(torch.bfloat16)
    W["head"] = mat(vocab, width, 2.0)
    W["final.norm"] = vec(width)
    if cfg.get("loop"):
        W["loop.in"] = mat(width, 2 * width, 1.4)
        W["loop.step"] = (torch.randn(cfg["loop"]["times"], width, generator=g) * 0.5).to(torch.bfloat16)
    for il, lc in enumerate(cfg["layers"]):
        p, m = f"l{il}.", lc["mixer"]
        for n in ("norm1", "norm1b") + (("norm2", "norm2b") if lc.get("mlp") else ()):
            W[p + n] = vec(width)
        H = m["heads"]
        if lc["type"] == "latent_attention":
            W[p + "mix.dq"] = mat(m["q_rank"], width)
            W[p + "mix.dq.norm"] = vec(m["q_rank"], 0.2, 1.0)
            W[p + "mix.uq"] = mat(H * (m["dim"] + m["rot_dim"]), m["q_rank"], 2.0)
            W[p + "mix.dkv"] = mat(m["kv_rank"] + m["rot_dim"], width, 1.5)
            W[p + "mix.dkv.norm"] = vec(m["kv_rank"], 0.2, 1.0)
            W[p + "mix.uk"] = mat(H * m["dim"], m["kv_rank"], 2.0)
            W[p + "mix.uv"] = mat(H * m["vdim"], m["kv_rank"])
            W[p + "mix.sink"] = vec(H, 1.0)
            W[p + "mix.o"] = mat(width, H * m["vdim"])
        else:
            for n, rows in (("q", H * m["dim"]), ("k", H * m["dim"]), ("v", H * m["vdim"]), ("g", H * m["vdim"]), ("i", H), ("f", H)):
                W[p + "mix." + n] = mat(rows, width, 1.5)
            W[p + "mix.i.b"] = vec(H, 1.0)
            W[p + "mix.f.b"] = vec(H, 1.0, 2.0)
            W[p + "mix.norm"] = vec(H * m["vdim"], 0.2, 1.0)
            W[p + "mix.o"] = mat(width, H * m["vdim"])
        mlp = lc.get("mlp")
        if mlp and mlp["kind"] == "dense":
            W[p + "mlp.up"] = mat(mlp["ff"], width, 1.5)
            W[p + "mlp.down"] = mat(width, mlp["ff"])
        elif mlp:
            ne, top, ff = mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["ff"]
            for e in range(ne):
                W[f"{p}mlp.e{e}.gate"] = mat(ff, width, 1.5)
                W[f"{p}mlp.e{e}.up"] = mat(ff, width, 1.5)
                W[f"{p}mlp.e{e}.down"] = mat(width, ff)
            W[p + "mlp.table"] = torch.stack([torch.randperm(ne, generator=g)[:top] for _ in range(vocab)]).to(torch.int32)
    return W


def write(folder, cfg, W):
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(folder, "model.safetensors"))
    return str(folder)

"""Small Fidepel models for tests: configurations of chosen sizes, random bf16 weights from a seed, written as a folder
(config.json + model.safetensors) the loader reads.  The sizes are deliberately odd ones - head counts, head sizes and
widths that share no factor with the kernels' tile sizes."""
from __future__ import annotations

import json
import os

import torch


def moe(n=6, top=2, ff=40, groups=(3, 2), scale=1.5, shared=24):
    rt = {"experts": n, "top": top, "scale": scale}
    if groups:
        rt["groups"] = {"count": groups[0], "keep": groups[1]}
    out = {"kind": "moe", "expert": {"ff": ff}, "router": rt}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def attention(heads=6, kv_heads=2, dim=24, vdim=20, window=7, rot_dims=16, base=10000.0, factor=4.0, scale=0.2, mlp=None):
    mixer = {"dim": dim, "heads": heads, "kv_heads": kv_heads, "scale": scale, "vdim": vdim}
    if window:
        mixer["mask"] = {"size": window}
    if rot_dims:
        mixer["rot"] = {"base": base, "dims": rot_dims}
        if factor:
            mixer["rot"]["scaling"] = {"factor": factor}
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def config(layers, width=72, vocab=97, loop=None, eps=1e-5, residual_mult=0.8):
    c = {"architecture": "Fidepel", "layers": layers, "norm": {"eps": eps}, "residual_mult": residual_mult, "vocab": vocab, "width": width}
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

    def one(mean=1.0, std=0.2):
        return (torch.randn((), generator=g) * std + mean).to(torch.bfloat16)

    W["embed"] = torch.randn(vocab, width, generator=g).to(torch.bfloat16)
    W["head"] = mat(vocab, width, 2.0)
    W["final.norm"] = one()
    for il, lc in enumerate(cfg["layers"]):
        p, m = f"l{il}.", lc["mixer"]
        H, G, D, VD = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
        W[p + "norm1"] = one()
        W[p + "mix.q"] = mat(H * D, width, 1.5)
        W[p + "mix.k"] = mat(G * D, width, 1.5)
        W[p + "mix.v"] = mat(G * VD, width, 1.5)
        W[p + "mix.q.norm"] = vec(H * D, 0.3, 1.5)
        W[p + "mix.k.norm"] = vec(G * D, 0.3, 1.5)
        W[p + "mix.temp"] = vec(H, 0.3, 1.0)
        W[p + "mix.g"] = mat(H, width, 2.0)
        W[p + "mix.o"] = mat(width, H * VD)
        mlp = lc.get("mlp")
        if mlp:
            ne, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            for e in range(ne):
                W[f"{p}mlp.e{e}.up"] = mat(ff, width, 1.5)
                W[f"{p}mlp.e{e}.down"] = mat(width, ff)
            W[p + "mlp.router"] = mat(ne, width, 3.0)
            if mlp.get("shared"):
                W[p + "mlp.shared.up"] = mat(mlp["shared"]["ff"], width, 1.5)
                W[p + "mlp.shared.down"] = mat(width, mlp["shared"]["ff"])
    return W


def write(folder, cfg, W):
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(folder, "model.safetensors"))
    return str(folder)

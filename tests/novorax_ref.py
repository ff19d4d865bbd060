"""Plain, slow restatement of the Novorax design in float64 torch, one function per mechanism.

Test infrastructure only: it shares no code with the product path (cortex.llamacpp_amd/), runs on the CPU and
processes whole sequences at once - no cache, no state carried between calls, no batching.  Weights are a dict
name -> tensor, the configuration is the dict a model's config.json holds.

Notation: h [T, width] rows of one sequence, positions 0 .. T-1.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    """x divided by its root mean square over the last axis (eps under the root)."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_offset(x, w, eps):
    """RMS norm with a zero-centred weight: unit(x) * (1 + w)."""
    return rms_unit(x, eps) * (1.0 + w.to(F64))


def norm_plain(x, w, eps):
    return rms_unit(x, eps) * w.to(F64)


def rotary_tables(rot, positions):
    """cos / sin [T, dims / 2] of the interleaved rotary embedding, with the YaRN frequency blend when rot['scaling'] is given."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    i = torch.arange(half, dtype=F64)
    f = base ** (-2.0 * i / dims)
    mscale = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def corr(turns):
            return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

        lo = max(math.floor(corr(float(sc["fast"]))), 0)
        hi = min(math.ceil(corr(float(sc["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        mscale = 0.1 * math.log(factor) + 1.0
    ang = positions.to(F64)[:, None] * f[None, :]
    return torch.cos(ang) * mscale, torch.sin(ang) * mscale


def rotate_interleaved(x, cos, sin, dims):
    """x [T, ..., D]: pairs (2i, 2i + 1) of the first `dims` entries turn by the table's angle, the rest pass."""
    out = x.clone()
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = cos.reshape(shape), sin.reshape(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def latent_attention(h, W, p, cfg, eps):
    """Attention through low-rank latents: queries via a normed latent, keys / values from one normed latent per token plus one
    rotated key part shared by the heads; sliding window; a learned per-head logit joins the softmax denominator with neither key nor value behind it."""
    T = h.shape[0]
    H, D, R, VD, KR = int(cfg["heads"]), int(cfg["dim"]), int(cfg["rot_dim"]), int(cfg["vdim"]), int(cfg["kv_rank"])
    g = lambda n: W[p + n].to(F64)
    cq = norm_plain(h @ g("dq").T, g("dq.norm"), eps)
    q = (cq @ g("uq").T).reshape(T, H, D + R)
    q_n, q_r = q[..., :D], q[..., D:]
    dkv = h @ g("dkv").T
    c = norm_plain(dkv[:, :KR], g("dkv.norm"), eps)
    k_r = dkv[:, KR:KR + R]
    rot = cfg["rot"]
    cos, sin = rotary_tables(rot, torch.arange(T))
    q_r = rotate_interleaved(q_r, cos, sin, int(rot["dims"]))
    k_r = rotate_interleaved(k_r, cos, sin, int(rot["dims"]))
    k_n = (c @ g("uk").T).reshape(T, H, D)
    v = (c @ g("uv").T).reshape(T, H, VD)
    s = (torch.einsum("ihd,jhd->hij", q_n, k_n) + torch.einsum("ihr,jr->hij", q_r, k_r)) * float(cfg["scale"])
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    seen = (i - j >= 0)
    if cfg.get("mask") and cfg["mask"].get("size"):
        seen = seen & (i - j < int(cfg["mask"]["size"]))
    s = s.masked_fill(~seen[None], -math.inf)
    if p + "sink" in W:
        sink = g("sink").reshape(H, 1, 1).expand(H, T, 1)
        w = torch.softmax(torch.cat([s, sink], -1), -1)[..., :T]
    else:
        w = torch.softmax(s, -1)
    o = torch.einsum("hij,jhv->ihv", w, v).reshape(T, H * VD)
    return o @ g("o").T


def mlstm(h, W, p, cfg, eps):
    """Matrix-memory recurrence with exponential gating, stabilised by a running maximum that starts at 0."""
    T = h.shape[0]
    H, D, VD, cap = int(cfg["heads"]), int(cfg["dim"]), int(cfg["vdim"]), float(cfg["gate_cap"])
    g = lambda n: W[p + n].to(F64)
    q = (h @ g("q").T).reshape(T, H, D) * D ** -0.5
    k = (h @ g("k").T).reshape(T, H, D)
    v = (h @ g("v").T).reshape(T, H, VD)
    ig = cap * torch.tanh((h @ g("i").T + g("i.b")) / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ g("f").T + g("f.b")) / cap))
    S = torch.zeros(H, D, VD, dtype=F64)
    n = torch.zeros(H, D, dtype=F64)
    m = torch.zeros(H, dtype=F64)
    outs = []
    for t in range(T):
        m_new = torch.maximum(fg[t] + m, ig[t])
        a, b = torch.exp(fg[t] + m - m_new), torch.exp(ig[t] - m_new)
        S = a[:, None, None] * S + b[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = a[:, None] * n + b[:, None] * k[t]
        m = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        outs.append(num / den[:, None])
    o = torch.stack(outs)                                    # [T, H, VD]
    o = rms_unit(o, eps).reshape(T, H * VD) * g("norm")
    o = o * torch.sigmoid(h @ g("g").T)
    return o @ g("o").T


def ff_dense(h, W, p):
    up = h @ W[p + "up"].to(F64).T
    return (torch.relu(up) ** 2) @ W[p + "down"].to(F64).T


def ff_experts(h, tokens, W, p, cfg):
    """Experts chosen by a table indexed with the token id; every chosen expert weighs 1 / top."""
    top = int(cfg["router"]["top"])
    table = W[p + "table"].to(torch.int64)
    out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for e in table[int(tokens[t])].tolist()[:top]:
            q = f"{p}e{e}."
            a = torch.nn.functional.silu(h[t] @ W[q + "gate"].to(F64).T) * (h[t] @ W[q + "up"].to(F64).T)
            out[t] += (a @ W[q + "down"].to(F64).T) / top
    return out


def layer_runs(config):
    """The order in which layers run: (layer index, pass number or -1 outside the loop, first-of-pass flag)."""
    L = len(config["layers"])
    loop = config.get("loop")
    if not loop or int(loop.get("times", 1)) < 1 or int(loop["stop"]) <= int(loop["start"]):
        return [(i, -1, False) for i in range(L)]
    a, b, n = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, -1, False) for i in range(a)]
    for t in range(n):
        runs += [(i, t, i == a) for i in range(a, b)]
    return runs + [(i, -1, False) for i in range(b, L)]


def forward(tokens, W, config, want_layers=False):
    """Logits [T, vocab] of one sequence (float64); with want_layers also the residual stream after every layer run."""
    eps = float(config["norm"]["eps"])
    tokens = torch.as_tensor(tokens, dtype=torch.int64)
    x0 = W["embed"].to(F64)[tokens]
    x = x0
    taps = []
    for il, t, first in layer_runs(config):
        if first:
            x = torch.cat([x, x0], -1) @ W["loop.in"].to(F64).T + W["loop.step"].to(F64)[t]
        spec = config["layers"][il]
        p = f"l{il}."
        hin = norm_offset(x, W[p + "norm1"], eps)
        if spec["type"] == "latent_attention":
            y = latent_attention(hin, W, p + "mix.", spec["mixer"], eps)
        elif spec["type"] == "mlstm":
            y = mlstm(hin, W, p + "mix.", spec["mixer"], eps)
        else:
            raise ValueError(spec["type"])
        x = x + norm_offset(y, W[p + "norm1b"], eps)
        if spec.get("mlp"):
            hin = norm_offset(x, W[p + "norm2"], eps)
            if spec["mlp"]["kind"] == "dense":
                y = ff_dense(hin, W, p + "mlp.")
            else:
                y = ff_experts(hin, tokens, W, p + "mlp.", spec["mlp"])
            x = x + norm_offset(y, W[p + "norm2b"], eps)
        taps.append(x)
    logits = norm_offset(x, W["final.norm"], eps) @ W["head"].to(F64).T * float(config.get("logit_scale", 1.0))
    return (logits, torch.stack(taps)) if want_layers else logits

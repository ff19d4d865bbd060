"""Plain, slow restatement of the Fidepel design in float64 torch, one function per mechanism.

Test infrastructure only: it shares no code with the product path (cortex.llamacpp_amd/), runs on the CPU and
processes whole sequences at once - no cache, no batching.  Weights are a dict name -> tensor, the configuration
is the dict a model's config.json holds.

Notation: x [T, width] the residual stream of one sequence, positions 0 .. T-1; h its normed rows.
  block:      h = unit(x) * g                      (g ONE number per norm)
              x <- x + m * (attend(h) + experts(h) + shared(h))
  attend:     q = Wq h, k = Wk h, v = Wv h;  q <- unit(q) * wq, k <- unit(k) * wk over the WHOLE projection;
              the first `dims` entries of every q / k head turn, entry i with entry i + dims/2, by p * base^(-2i/dims) / factor;
              score(i, j) = q_i . k_j * scale * temp[head], j in (i - window, i];  softmax;  head output * sigmoid(Wg h)[head];  Wo
  experts:    s = softmax(Wr h);  groups of neighbours score as their best member, the `keep` best groups stay open;
              the `top` open experts with the largest s;  weights s / (sum + 1e-20) * scale;  expert = Wdown relu(Wup h)^2
"""
from __future__ import annotations

import torch

F64 = torch.float64


def unit(x, eps):
    """x over its root mean square along the last axis, eps under the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_number(x, g, eps):
    return unit(x, eps) * g.to(F64).reshape(())


def turn_half(x, positions, rot):
    """x [T, heads, D]: entry i < dims/2 of every head pairs with entry i + dims/2; the pair turns by position * frequency_i."""
    if not rot or not rot.get("dims"):
        return x
    dims = int(rot["dims"])
    half = dims // 2
    f = float(rot["base"]) ** (-2.0 * torch.arange(half, dtype=F64) / dims)
    if rot.get("scaling"):
        f = f / float(rot["scaling"]["factor"])
    ang = positions.to(F64)[:, None, None] * f[None, None, :]
    c, s = torch.cos(ang), torch.sin(ang)
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


def window_mask(T, window):
    """[T, T] bool: row i sees column j when 0 <= i - j < window (window 0 / None: every j <= i)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = j <= i
    if window:
        seen = seen & (i - j < window)
    return seen


def attend(h, W, p, mx, eps):
    T = h.shape[0]
    H, G, D, VD = mx["heads"], mx.get("kv_heads", mx["heads"]), mx["dim"], mx.get("vdim", mx["dim"])
    q = h @ W[p + "q"].to(F64).T
    k = h @ W[p + "k"].to(F64).T
    v = h @ W[p + "v"].to(F64).T
    q = unit(q, eps) * W[p + "q.norm"].to(F64)
    k = unit(k, eps) * W[p + "k.norm"].to(F64)
    pos = torch.arange(T)
    q = turn_half(q.reshape(T, H, D), pos, mx.get("rot"))
    k = turn_half(k.reshape(T, G, D), pos, mx.get("rot"))
    v = v.reshape(T, G, VD)
    seen = window_mask(T, (mx.get("mask") or {}).get("size"))
    gate = torch.sigmoid(h @ W[p + "g"].to(F64).T)
    temp = W[p + "temp"].to(F64)
    heads = []
    for a in range(H):
        b = a // (H // G)
        sc = (q[:, a] @ k[:, b].T) * float(mx["scale"]) * temp[a]
        sc = sc.masked_fill(~seen, float("-inf"))
        heads.append((torch.softmax(sc, -1) @ v[:, b]) * gate[:, a:a + 1])
    return torch.cat(heads, -1) @ W[p + "o"].to(F64).T


def route(h, W, p, rt):
    """ids [T, top] and weights [T, top]."""
    E, top = rt["experts"], rt["top"]
    s = torch.softmax(h @ W[p + "router"].to(F64).T, -1)
    T = s.shape[0]
    open_ = torch.ones(T, E, dtype=torch.bool)
    gr = rt.get("groups")
    if gr and gr["count"] > 1 and gr["keep"] < gr["count"]:
        per = E // gr["count"]
        best = s.reshape(T, gr["count"], per).amax(-1)
        kept = torch.topk(best, gr["keep"], dim=-1).indices
        og = torch.zeros(T, gr["count"], dtype=torch.bool)
        og.scatter_(1, kept, True)
        open_ = og.repeat_interleave(per, dim=1)
    ids = torch.topk(s.masked_fill(~open_, -1.0), top, dim=-1).indices
    w = s.gather(1, ids)
    w = w / (w.sum(-1, keepdim=True) + 1e-20) * float(rt.get("scale", 1.0))
    return ids, w


def relu2_expert(h, up, down):
    return (torch.relu(h @ up.to(F64).T) ** 2) @ down.to(F64).T


def experts(h, W, p, mlp):
    ids, w = route(h, W, p, mlp["router"])
    out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for j in range(ids.shape[1]):
            e = int(ids[t, j])
            out[t] += w[t, j] * relu2_expert(h[t:t + 1], W[f"{p}e{e}.up"], W[f"{p}e{e}.down"])[0]
    if mlp.get("shared"):
        out = out + relu2_expert(h, W[p + "shared.up"], W[p + "shared.down"])
    return out


def layer_order(cfg):
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp or lp["stop"] <= lp["start"] or lp["times"] < 1:
        return list(range(n))
    return list(range(lp["start"])) + list(range(lp["start"], lp["stop"])) * lp["times"] + list(range(lp["stop"], n))


def forward(tokens, W, cfg, layers=False):
    """logits [T, vocab] (and, with layers=True, the stream after every layer run [runs, T, width])."""
    eps, m = float(cfg["norm"]["eps"]), float(cfg.get("residual_mult", 1.0))
    x = W["embed"].to(F64)[torch.as_tensor(tokens)]
    taps = []
    for il in layer_order(cfg):
        lc, p = cfg["layers"][il], f"l{il}."
        h = norm_one_number(x, W[p + "norm1"], eps)
        y = attend(h, W, p + "mix.", lc["mixer"], eps)
        if lc.get("mlp"):
            y = y + experts(h, W, p + "mlp.", lc["mlp"])
        x = x + m * y
        taps.append(x)
    out = norm_one_number(x, W["final.norm"], eps) @ W["head"].to(F64).T
    return (out, torch.stack(taps)) if layers else out

"""Plain float64 implementations of the Fusasun decoder's mechanisms, written from its equations: loops over
tokens, heads and keys, whole sequences only, no cache, nothing shared with the package.

A model is ``(cfg, sd)``: the checkpoint's config dictionary and its tensors by checkpoint name.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def canon(h, w):
    """h [T, W] + causal per-channel convolution with w [W, taps] (last tap = the current token)."""
    T, taps = h.shape[0], w.shape[1]
    out = h.clone()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def llama3_freqs(rot: dict):
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if sc:
        factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
        out = []
        for x in f:
            wl = 2.0 * math.pi / x
            if wl < orig / high:
                out.append(x)
            elif wl > orig / low:
                out.append(x / factor)
            else:
                s = (orig / wl - low) / (high - low)
                out.append((1.0 - s) * x / factor + s * x)
        f = out
    return f, 1.0


def yarn_freqs(rot: dict):
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig, fast, slow = float(sc["factor"]), float(sc["original"]), float(sc["fast"]), float(sc["slow"])

    def dim_of(t):
        return dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(fast)), 0)
    hi = min(math.ceil(dim_of(slow)), dims - 1)
    out = []
    for i, x in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(x / factor * ramp + x * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate(x, pos: int, freqs, mag: float):
    """x [..., d]: the first 2 * len(freqs) dimensions rotated in adjacent pairs (2i, 2i + 1)."""
    y = x.clone()
    for i, f in enumerate(freqs):
        a = pos * f
        c, s = math.cos(a) * mag, math.sin(a) * mag
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        y[..., 2 * i] = u * c - v * s
        y[..., 2 * i + 1] = v * c + u * s
    return y


def softmax_rows(scores: list, values: list):
    m = max(scores)
    e = [math.exp(s - m) for s in scores]
    den = sum(e)
    out = torch.zeros_like(values[0])
    for w, v in zip(e, values):
        out += (w / den) * v
    return out


def pooled_window_attention(h, m: dict, sd: dict, p: str, round_cache=None):
    """Grouped-query attention under a sliding window plus one mean key / value per block of ``pool`` tokens
    that the window has left behind entirely.  ``round_cache``: how the cache rounds what it holds (None: exact)."""
    H, G, dim, vdim = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    size = int(m["mask"]["size"])
    P = int(m["mask"].get("pool") or 0)
    freqs, mag = llama3_freqs(m["rot"]) if m.get("rot") else ([], 1.0)
    T = h.shape[0]
    rc = round_cache or (lambda t: t)
    q = (h @ sd[p + "q"].T).view(T, H, dim)
    k = (h @ sd[p + "k"].T).view(T, G, dim)
    v = rc((h @ sd[p + "v"].T).view(T, G, vdim))
    q = torch.stack([rotate(q[t], t, freqs, mag) for t in range(T)])
    k = rc(torch.stack([rotate(k[t], t, freqs, mag) for t in range(T)]))
    nblk = T // P if P else 0
    pk = [rc(k[b * P:(b + 1) * P].mean(0)) for b in range(nblk)]
    pv = [rc(v[b * P:(b + 1) * P].mean(0)) for b in range(nblk)]
    out = torch.zeros(T, H, vdim, dtype=h.dtype)
    scale = float(m["scale"])
    for i in range(T):
        for hh in range(H):
            g = hh // (H // G)
            sc, vs = [], []
            for b in range(nblk):
                if b * P + P - 1 <= i - size:
                    sc.append(float(q[i, hh] @ pk[b][g]) * scale)
                    vs.append(pv[b][g])
            for j in range(max(0, i - size + 1), i + 1):
                sc.append(float(q[i, hh] @ k[j, g]) * scale)
                vs.append(v[j, g])
            out[i, hh] = softmax_rows(sc, vs)
    return out.reshape(T, H * vdim) @ sd[p + "o"].T


def latent_window_attention(h, m: dict, sd: dict, p: str, eps: float, round_cache=None):
    """Attention whose keys and values are expanded from a normed latent, with a rotated key segment common to
    the heads, under a sliding window, each head's output gated."""
    H, dim, rd, vdim, R = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    size = int(m["mask"]["size"])
    freqs, mag = yarn_freqs(m["rot"])
    T = h.shape[0]
    rc = round_cache or (lambda t: t)
    cq = rms(h @ sd[p + "dq"].T, eps) * sd[p + "dq.norm"]
    q = (cq @ sd[p + "uq"].T).view(T, H, dim + rd)
    ckv = h @ sd[p + "dkv"].T
    c = rms(ckv[:, :R], eps) * sd[p + "dkv.norm"]
    kr = torch.stack([rotate(ckv[t, R:], t, freqs, mag) for t in range(T)])
    kn = (c @ sd[p + "uk"].T).view(T, H, dim)
    v = rc((c @ sd[p + "uv"].T).view(T, H, vdim))
    k = rc(torch.cat([kn, kr[:, None, :].expand(T, H, rd)], -1))
    gate = torch.sigmoid(h @ sd[p + "g"].T)
    scale = float(m["scale"])
    out = torch.zeros(T, H, vdim, dtype=h.dtype)
    for i in range(T):
        for hh in range(H):
            qi = torch.cat([q[i, hh, :dim], rotate(q[i, hh, dim:], i, freqs, mag)])
            js = range(max(0, i - size + 1), i + 1)
            out[i, hh] = softmax_rows([float(qi @ k[j, hh]) * scale for j in js], [v[j, hh] for j in js]) * gate[i, hh]
    return out.reshape(T, H * vdim) @ sd[p + "o"].T


def table_moe(h, ids, mlp: dict, sd: dict, p: str):
    """Each token's experts are the row of its token id in an integer table; equal weights."""
    top = int(mlp["router"]["top"])
    out = torch.zeros(h.shape[0], sd[p + "e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for e in sd[p + "table"][int(ids[t])].tolist():
            g, u = sd[p + f"e{e}.gate"] @ h[t], sd[p + f"e{e}.up"] @ h[t]
            out[t] += (sd[p + f"e{e}.down"] @ (g * torch.sigmoid(g) * u)) / top
    return out


def forward(cfg: dict, sd: dict, ids, taps: list = None, round_cache=None):
    """Logits [T, vocab] (float64) of one whole sequence; ``taps`` receives the stream after every layer."""
    sd = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in sd.items()}
    eps = float(cfg["norm"]["eps"])
    x = sd["embed"][torch.as_tensor(ids, dtype=torch.long)] * float(cfg["embedding"]["scale"])
    for i, L in enumerate(cfg["layers"]):
        b = f"l{i}."
        h = rms(x, eps) * sd[b + "norm1"]
        gate = torch.sigmoid(h @ sd[b + "rg1"].T + sd[b + "rg1.b"])
        hc = canon(h, sd[b + "canon1"])
        if L["type"] == "attention":
            y = pooled_window_attention(hc, L["mixer"], sd, b + "mix.", round_cache)
        elif L["type"] == "latent_attention":
            y = latent_window_attention(hc, L["mixer"], sd, b + "mix.", eps, round_cache)
        else:
            raise ValueError(L["type"])
        x = x + rms(y * gate, eps) * sd[b + "norm1b"]
        if L.get("mlp"):
            h = rms(x, eps) * sd[b + "norm2"]
            gate = torch.sigmoid(h @ sd[b + "rg2"].T + sd[b + "rg2.b"])
            x = x + rms(table_moe(h, ids, L["mlp"], sd, b + "mlp.") * gate, eps) * sd[b + "norm2b"]
        if taps is not None:
            taps.append(x.clone())
    return (rms(x, eps) * sd["final.norm"]) @ sd["head"].T

"""Plain float64 implementation of the Lumedra decoder, written from its equations: whole sequences only, one
function per mechanism, loops over tokens and heads where a recurrence or a mask is involved.  It shares no
code with the package (not even its config reader): ``cfg`` is the checkpoint's ``config.json`` as a dict and
``sd`` a dict of tensors under the checkpoint names.

    x = embed[token]
    per layer:  x <- x + mixer(rms(x) w1) + ff(rms(x) w2)          (ff may be absent)
    logits = embed . (rms(x) w_f)                                   rms(v) = v / sqrt(mean(v^2) + eps)
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(v, w, eps):
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * w


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


def rotate_pairs(x, pos, dims, base):
    """x [T, n]: dimensions (2 i, 2 i + 1), i < dims / 2, turned by pos * base^(-2 i / dims); the rest unchanged."""
    out = x.clone()
    for i in range(dims // 2):
        a = pos.to(F64) * base ** (-2.0 * i / dims)
        u, v = x[:, 2 * i], x[:, 2 * i + 1]
        out[:, 2 * i] = u * torch.cos(a) - v * torch.sin(a)
        out[:, 2 * i + 1] = v * torch.cos(a) + u * torch.sin(a)
    return out


def softmax_rows(s, seen):
    """Rows of s over the columns where ``seen``; every row sees at least itself."""
    s = s.masked_fill(~seen, -math.inf)
    e = torch.exp(s - s.max(-1, keepdim=True).values)
    return e / e.sum(-1, keepdim=True)


def window_attention(h, m, w, v_first=None):
    """Grouped-query softmax attention without rotation: capped scores, a sliding window that also keeps the
    first tokens, values blended with ``v_first`` [T, G vdim].  Returns (output [T, W], this layer's unmixed v)."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    q = (h @ w["q"].T).view(T, H, d)
    k = (h @ w["k"].T).view(T, G, d)
    v_own = h @ w["v"].T
    v = v_own
    if v_first is not None:
        lam = w["vmix"].to(F64)
        v = (1.0 - lam) * v_own + lam * v_first
    v = v.view(T, G, dv)
    i = torch.arange(T).view(-1, 1)
    j = torch.arange(T).view(1, -1)
    seen = j <= i
    mask = m.get("mask")
    if mask:
        seen = seen & ((i - j < mask["size"]) | (j < mask.get("keep_first", 0)))
    cap = float(m.get("softcap") or 0.0)
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"]
        if cap > 0:
            s = cap * torch.tanh(s / cap)
        out[:, hd] = softmax_rows(s, seen) @ v[:, g]
    return out.reshape(T, H * dv) @ w["o"].T, v_own


def latent_attention(h, m, w, eps):
    """Causal softmax attention with queries and keys / values through normed low-rank latents, one rotated key
    part common to the heads, and an element-wise output gate."""
    T = h.shape[0]
    H, d, r, dv, kvr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    base = m["rot"]["base"]
    cq = rms(h @ w["dq"].T, w["dq.norm"], eps)
    q = (cq @ w["uq"].T).view(T, H, d + r)
    ckv = h @ w["dkv"].T
    c = rms(ckv[:, :kvr], w["dkv.norm"], eps)
    kr = rotate_pairs(ckv[:, kvr:], pos, r, base)
    ku = (c @ w["uk"].T).view(T, H, d)
    vv = (c @ w["uv"].T).view(T, H, dv)
    i = torch.arange(T).view(-1, 1)
    j = torch.arange(T).view(1, -1)
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        qr = rotate_pairs(q[:, hd, d:], pos, r, base)
        s = (q[:, hd, :d] @ ku[:, hd].T + qr @ kr.T) * m["scale"]
        out[:, hd] = softmax_rows(s, j <= i) @ vv[:, hd]
    return (out.reshape(T, H * dv) * sigmoid(h @ w["g"].T)) @ w["o"].T


def lightning(h, m, w, eps):
    """Linear attention with one decay per head: S <- decay S + k v^T, o = S^T q; all heads normed together."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w["q"].T).view(T, H, d)
    k = silu(h @ w["k"].T).view(T, H, d)
    v = silu(h @ w["v"].T).view(T, H, dv)
    o = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        S = torch.zeros(d, dv, dtype=F64)
        for t in range(T):
            S = m["decay"][hd] * S + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    y = rms(o.reshape(T, H * dv), w["norm"], eps) * sigmoid(h @ w["g"].T)
    return y @ w["o"].T


def dense_ff(h, mlp, w):
    lim = mlp["limit"]
    g = torch.clamp(h @ w["gate"].T, max=lim)
    u = torch.clamp(h @ w["up"].T, -lim, lim)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w["down"].T


def expert(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(z, r):
    """z [E] router logits -> (chosen experts, weights)."""
    E, top = r["experts"], r["top"]
    s = sigmoid(z)
    allowed = torch.ones(E, dtype=torch.bool)
    gr = r.get("groups")
    if gr:
        n = E // gr["count"]
        gs = torch.stack([s[a * n:(a + 1) * n].sort(descending=True).values[:2].sum() for a in range(gr["count"])])
        best = gs.sort(descending=True, stable=True).indices[:gr["keep"]]
        allowed[:] = False
        for a in best.tolist():
            allowed[a * n:(a + 1) * n] = True
    chosen = s.masked_fill(~allowed, -1.0).sort(descending=True, stable=True).indices[:top]
    wgt = s[chosen] / (s[chosen].sum() + 1e-20) * r.get("scale", 1.0)
    return chosen.tolist(), wgt


def moe_ff(h, mlp, w):
    T = h.shape[0]
    z = h @ w["router"].T
    out = torch.zeros(T, w["e0.down"].shape[0], dtype=F64)
    for t in range(T):
        chosen, wgt = route(z[t], mlp["router"])
        for e, a in zip(chosen, wgt):
            out[t] += a * expert(h[t:t + 1], w, f"e{e}.")[0]
    if mlp.get("shared"):
        out = out + expert(h, w, "shared.")
    return out


def forward(cfg: dict, sd: dict, tokens, return_streams: bool = False):
    """-> logits [T, vocab] float64 (and the stream after every layer)."""
    sd = {k: v.to(F64) for k, v in sd.items()}
    eps = cfg["norm"]["eps"]
    x = sd["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    streams, v_first = [], None
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        wm = {k[len(p) + 4:]: v for k, v in sd.items() if k.startswith(p + "mix.")}
        h = rms(x, sd[p + "norm1"], eps)
        m = L["mixer"]
        if L["type"] == "attention":
            mixes = bool(m.get("v_mix"))
            y, v_own = window_attention(h, m, wm, v_first if mixes else None)
            if mixes and v_first is None:
                v_first = v_own
        elif L["type"] == "latent_attention":
            y = latent_attention(h, m, wm, eps)
        elif L["type"] == "lightning":
            y = lightning(h, m, wm, eps)
        else:
            raise ValueError(L["type"])
        if L.get("mlp"):
            wf = {k[len(p) + 4:]: v for k, v in sd.items() if k.startswith(p + "mlp.")}
            h2 = rms(x, sd[p + "norm2"], eps)
            y = y + (dense_ff(h2, L["mlp"], wf) if L["mlp"]["kind"] == "dense" else moe_ff(h2, L["mlp"], wf))
        x = x + y
        streams.append(x.clone())
    logits = rms(x, sd["final.norm"], eps) @ sd["embed"].T
    return (logits, streams) if return_streams else logits

"""Entry points of the linear-state recurrences (``csrc/delta_scan.hip``): one scan kernel for the family

    S_t = diag(w_t) S_(t-1) - p_t (z_t^T S_(t-1)) + k_t v_t^T          o_t = S_t^T q_t

with an f32 state ``S [dk, dv]`` per head and sequence, and the token-parallel kernels that prepare its
operands in f32 for three members of the family:

* retention: ``w`` one constant per head, no removal term (``p = z = 0``);
* gated delta rule ``S <- g S; S <- S + k (beta (v - S^T k))^T``: ``w = g``, ``p = beta k``,
  ``z = g * k`` and the written value ``beta v`` (the removal then reads the old state);
* generalized delta rule: ``w`` and a removal rate ``a`` per key channel, ``p = a * u``, ``z = u`` with
  ``u`` the unit key.

GPU tensors go to the HIP kernels; CPU tensors to the torch implementations below, which keep the
kernels' layouts: sequences of a step are rows ``[cu[s], cu[s+1])`` with state slot ``slots[s]`` (< 0: a
padding row), a fresh state when ``positions[cu[s]] == 0``; state ``[slots, H, dk, dv]`` f32.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn.functional as F

from ._ext import lib, use_hip

__all__ = ["delta_scan", "delta_scan_supported", "gated_delta_prep", "general_delta_prep", "head_norm_gate", "tanh_"]

DELTA_MAX_DK = 256       # largest key size the scan kernel is built for
GATE_SILU, GATE_SIGMOID = 0, 1
UNIT_EPS = 1e-6          # inside the root of the unit-vector norms


def delta_scan_supported(dk: int, dv: int) -> bool:
    return 1 <= dk <= DELTA_MAX_DK and dv >= 1


def delta_scan(q, k, v, w, p, z, state, cu, slots, positions, H: int, Hk: int, dk: int, dv: int,
               w_head=None, k_scale: float = 1.0, max_len: int = 1, lanes: int = 0, act: bool = False):
    """o f32 [T, H * dv] of the recurrence in the module docstring, per sequence and head, the state read
    from / left in ``state[slot]``.  q, k: rows of ``Hk * dk`` (head h reads q/k head ``h // (H / Hk)``),
    v: rows of ``H * dv``; each in bf16 or f32 (k is multiplied by ``k_scale`` in f32).  ``w``: f32 rows of
    ``H * dk``, or None with ``w_head`` f32 [H] (one decay per head).  ``p``, ``z``: f32 rows of ``H * dk``,
    or both None (no removal term).  ``lanes``: 4 or 16 forces how many lanes of the GPU kernel share a state
    column (default: by the step's shape -- 16 while (sequence, head) pairs do not fill the chip).  ``act``: q, k
    and v are the silu (f32) of what the rows hold."""
    if use_hip(q):
        return lib().delta_scan(q, k, v, w, p, z, state, cu, slots, positions, H, Hk, dk, dv, w_head, float(k_scale), int(max_len),
                                int(lanes), bool(act))
    T = q.shape[0]
    o = torch.zeros(T, H * dv, dtype=torch.float32, device=q.device)
    cul, sl = cu.tolist(), slots.tolist()
    rep = H // Hk
    for s in range(len(cul) - 1):
        r0, r1 = cul[s], cul[s + 1]
        if sl[s] < 0 or r1 <= r0:
            continue
        S = state[sl[s]].clone() if int(positions[r0]) > 0 else torch.zeros_like(state[sl[s]])     # [H, dk, dv]
        f = F.silu if act else (lambda t: t)
        qq = f(q[r0:r1, : Hk * dk].float()).view(-1, Hk, dk).repeat_interleave(rep, 1)
        kk = (f(k[r0:r1, : Hk * dk].float()) * k_scale).view(-1, Hk, dk).repeat_interleave(rep, 1)
        vv = f(v[r0:r1, : H * dv].float()).view(-1, H, dv)
        ww = w[r0:r1, : H * dk].view(-1, H, dk) if w is not None else w_head.view(1, H, 1).expand(r1 - r0, H, dk)
        for t in range(r1 - r0):
            new = ww[t].unsqueeze(-1) * S + kk[t].unsqueeze(-1) * vv[t].unsqueeze(1)
            if p is not None:
                zs = torch.einsum("hi,hij->hj", z[r0 + t, : H * dk].view(H, dk), S)
                new = new - p[r0 + t, : H * dk].view(H, dk).unsqueeze(-1) * zs.unsqueeze(1)
            S = new
            o[r0 + t] = torch.einsum("hi,hij->hj", qq[t], S).reshape(-1)
        state[sl[s]] = S
    return o


def _unit(x):
    return x / torch.sqrt(x.pow(2).sum(-1, keepdim=True) + UNIT_EPS)


def gated_delta_prep(q, k, v, beta, dt, dt_bias, A_log, H: int, Hk: int, dk: int, dv: int):
    """Operands of the gated delta rule, all f32.  ``q``, ``k`` rows of ``Hk * dk`` and ``v`` rows of ``H * dv``
    after the short convolution and its activation; ``beta`` rows of H raw write strengths; ``dt`` rows of
    ``H * dk`` raw step sizes.  Returns (qn [T, Hk dk] unit vectors times dk^-1/2, kn [T, Hk dk] unit vectors,
    vb [T, H dv] = sigmoid(beta) v, g [T, H dk] = exp(-exp(A_log) softplus(dt + dt_bias)),
    p = sigmoid(beta) kn, z = g * kn per head)."""
    if use_hip(q):
        return tuple(lib().gated_delta_prep(q, k, v, beta, dt, dt_bias, A_log, H, Hk, dk, dv))
    T = q.shape[0]
    rep = H // Hk
    kn = _unit(k[:, : Hk * dk].float().view(T, Hk, dk))
    qn = _unit(q[:, : Hk * dk].float().view(T, Hk, dk)) * dk ** -0.5
    b = torch.sigmoid(beta[:, :H].float())
    vb = v[:, : H * dv].float().view(T, H, dv) * b.unsqueeze(-1)
    g = torch.exp(-torch.exp(A_log.float()).view(1, H, 1) * F.softplus(dt[:, : H * dk].float() + dt_bias, threshold=30.0).view(T, H, dk))
    kh = kn.repeat_interleave(rep, 1)
    return (qn.reshape(T, -1), kn.reshape(T, -1), vb.reshape(T, -1), g.reshape(T, -1), (b.unsqueeze(-1) * kh).reshape(T, -1),
            (g * kh).reshape(T, -1))


GENERAL_DELTA_DECAY = math.exp(-0.5)   # the design's fixed bound on the decay's exponent


def general_delta_prep(k, wraw, w0, araw, a_b, H: int, dk: int):
    """Operands of the generalized delta rule, all f32 rows of ``H * dk``: (w = exp(-e^(-1/2) sigmoid(wraw +
    w0)), p = sigmoid(araw + a_b) * u, z = u) with u the unit key of each head."""
    if use_hip(k):
        return tuple(lib().general_delta_prep(k, wraw, w0, araw, a_b, H, dk))
    T = k.shape[0]
    u = _unit(k[:, : H * dk].float().view(T, H, dk)).reshape(T, -1)
    w = torch.exp(-GENERAL_DELTA_DECAY * torch.sigmoid(wraw[:, : H * dk].float() + w0))
    a = torch.sigmoid(araw[:, : H * dk].float() + a_b)
    return w, a * u, u


def head_norm_gate(o, gate, w, H: int, eps: float, gate_kind: int, out_dtype):
    """``o`` f32 [T, H * dv]: each head divided by its RMS, times ``w`` f32 [H * dv] (None: ones), times
    silu or sigmoid of ``gate`` rows of ``H * dv``; result in ``out_dtype``."""
    if use_hip(o):
        return lib().head_norm_gate(o, gate, w, H, float(eps), int(gate_kind), out_dtype)
    T, n = o.shape
    x = o.view(T, H, n // H)
    x = (x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)).reshape(T, n)
    if w is not None:
        x = x * w
    g = gate[:, :n].float()
    return (x * (F.silu(g) if gate_kind == GATE_SILU else torch.sigmoid(g))).to(out_dtype)


def tanh_(x):
    """tanh in place on a (possibly strided) block of columns."""
    if use_hip(x):
        lib().tanh_(x)
        return x
    return x.copy_(torch.tanh(x.float()).to(x.dtype))

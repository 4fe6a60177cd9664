"""Entry points of the kernels behind parallel sublayers and routed experts (``csrc/parallel_ops.hip``, the
expert products of ``csrc/moe.hip``), with their CPU implementations:

* ``stream_parallel_norm`` -- the f32 stream takes the sum of a block's sublayer results (two dense rows and a
  token's weighted expert rows), and the next block's two norms of the same row come out of the same pass;
* ``router_topk``          -- f32 router logits, sigmoid scores, group-limited choice of the ``top`` experts and
  their normalised weights;
* ``routed_experts``       -- the chosen experts' feed-forwards, un-summed (the stream update weighs them);
* ``clamped_glu``          -- ``g sigmoid(alpha g) (u + 1)`` with ``g = min(gate, limit)``, ``u = clamp(up, +-limit)``;
* ``silu_``, ``sigmoid_mul_`` -- element-wise activations in place on a block of columns.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F

from ._ext import lib, use_hip

__all__ = ["stream_parallel_norm", "router_topk", "routed_experts", "clamped_glu", "silu_", "sigmoid_mul_"]

WEIGHT_SUM_FLOOR = 1e-20     # added to the sum of the chosen scores before the division


def stream_parallel_norm(x, a, b, y, y_w, w1, w2, eps: float, out_dtype=torch.bfloat16):
    """``x += a + b + sum_k y_w[t, k] * y[t * top + k]`` in place (f32; every term optional), then
    ``(rms(x) * w1, rms(x) * w2)`` in ``out_dtype`` (a weight None: no such output; rms(v) = v / sqrt(mean(v^2) +
    eps), one root for both).  ``a``, ``b`` [T, W] activations; ``y`` [T * top, W] with a token's rows adjacent and
    ``y_w`` f32 [T, top] their weights."""
    if use_hip(x):
        return tuple(lib().stream_parallel_norm(x, a, b, y, y_w, w1, w2, float(eps), out_dtype))
    T, W = x.shape
    d = None
    for t in (a, b):
        if t is not None:
            d = t.float() if d is None else d + t.float()
    if y is not None:
        e = (y.float().view(T, -1, W) * y_w.view(T, -1, 1)).sum(1)
        d = e if d is None else d + e
    if d is not None:
        x += d
    if w1 is None and w2 is None:
        return None, None
    n = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return tuple((n * w).to(out_dtype) if w is not None else None for w in (w1, w2))


def router_topk(h, w_router, top: int, groups: int = 1, keep: int = 1, scale: float = 1.0):
    """(experts int32 [T, top], weights f32 [T, top]) for rows ``h`` [T, W] and ``w_router`` f32 [E, W]:
    scores ``s = sigmoid(W_router h)`` from f32 logits (the sigmoid, sums and weights are evaluated in f64); the
    experts form ``groups`` equal groups of neighbours, a group's score is the sum of its two largest scores and
    only experts of the ``keep`` best groups can be chosen; the ``top`` largest scores among those; weights
    ``s / (sum of the chosen s + 1e-20) * scale``."""
    E = w_router.shape[0]
    if E % groups or not 1 <= keep <= groups or not 1 <= top <= (E // groups) * keep:
        raise ValueError(f"router: {top} of {E} experts in {keep} of {groups} groups")
    if use_hip(h):
        ex, wt = lib().router_topk(h, w_router, int(top), int(groups), int(keep), float(scale))
        return ex, wt
    # f32 logits; the sigmoid and the sums in f64 (an f32 sigmoid near 1 would tie logits that are clearly apart)
    s = torch.sigmoid((h.float() @ w_router.float().T).double())            # [T, E]
    T = s.shape[0]
    if groups > 1:
        per = E // groups
        gs = s.view(T, groups, per).topk(min(2, per), dim=-1).values.sum(-1)
        best = gs.sort(dim=-1, descending=True, stable=True).indices[:, :keep]     # ties: the lower index, as on the GPU
        ok = torch.zeros(T, groups, dtype=torch.bool, device=s.device).scatter_(1, best, True)
        sel = s.masked_fill(~ok.repeat_interleave(per, dim=1), -1.0)
    else:
        sel = s
    ex = sel.sort(dim=-1, descending=True, stable=True).indices[:, :top]
    sc = s.gather(1, ex)
    return ex.to(torch.int32), (sc / (sc.sum(-1, keepdim=True) + WEIGHT_SUM_FLOOR) * scale).float()


def routed_experts(h, experts, w_gate_up, w_down):
    """Token t runs the experts ``experts[t]`` (int32 [T, top]), each ``W_down (silu(W_gate h) * (W_up h))``.
    ``w_gate_up`` [E, 2 * ffp, W] (gate rows, then up rows, each padded with zero rows to ffp), ``w_down``
    [E, W, ffp].  Returns the experts' results un-summed, [T * top, W] in h's dtype with a token's ``top`` rows
    adjacent, for a consumer that weighs them in f32 (``stream_parallel_norm``)."""
    from .window import run_experts

    return run_experts(h, None, experts, w_gate_up, w_down, experts.shape[1])


def clamped_glu(gu, limit: float, alpha: float = 1.702):
    """[T, 2F] = [gate | up] -> ``g * sigmoid(alpha g) * (u + 1)`` with ``g = min(gate, limit)`` and
    ``u = clamp(up, -limit, limit)``, [T, F] in the same dtype (f32 arithmetic)."""
    if use_hip(gu):
        return lib().clamped_glu(gu, float(limit), float(alpha))
    F_ = gu.shape[1] // 2
    g = gu[:, :F_].float().clamp(max=limit)
    u = gu[:, F_:].float().clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gu.dtype)


def silu_(x):
    """silu in place on a (possibly strided) block of columns."""
    if use_hip(x):
        lib().silu_(x)
        return x
    return x.copy_(F.silu(x.float()).to(x.dtype))


def sigmoid_mul_(x, gate):
    """``x *= sigmoid(gate)`` in place, element by element (both possibly strided blocks of columns)."""
    if use_hip(x):
        lib().sigmoid_mul_(x, gate)
        return x
    return x.copy_((x.float() * torch.sigmoid(gate.float())).to(x.dtype))

"""Entry points of the kernels behind windowed attention with pooled blocks, latent attention and
table-routed experts (``csrc/window_ops.hip``, ``csrc/moe.hip``, the grouped form of the prefill GEMM in
``csrc/gemm.hip``), with their CPU implementations:

* ``stream_gated_norm``  -- gated, normed sublayer result added to the f32 stream + the next sublayer's norm;
* ``rms_cols``           -- RMS norm of a block of columns of a fused projection;
* ``rot_kv_write``       -- rotation of adjacent pairs with a frequency table (any scaling baked into the table,
  one magnitude for cos and sin), keys assembled from a per-head part and a part shared by the heads, K / V
  filed in the paged cache;
* ``pool_kv_write``      -- mean key / value of every block of P positions a step completes, filed at the
  block's index in a second cache pair addressed by the sequence's own block table;
* ``table_experts``      -- experts chosen per token by a [vocab, top] table, equal weights.

Layouts are those of ``ops.mixers``: K cache ``[blocks, G, BS, dim]``, V cache key-contiguous
``[blocks, G, vdim, BS]``.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from ._ext import lib, use_hip

# from this many (token, choice) pairs per expert on average the experts run on the dense GEMM's 256-row tiles
GROUPED_DENSE_MIN_ROWS = 128

__all__ = ["stream_gated_norm", "rms_cols", "rot_kv_write", "pool_kv_write", "table_experts", "run_experts", "moe_route"]


def stream_gated_norm(x, y, g, g_bias, w_post, w_next, eps: float, out_dtype=torch.bfloat16, parts: int = 1):
    """``x += rms(v) * w_post`` in place (f32) with ``v = mean over parts of y * sigmoid(g + g_bias)``, then
    ``rms(x) * w_next`` in ``out_dtype`` (``w_next`` None: nothing is returned).  ``y`` [T * parts, W]: the
    ``parts`` rows of a token are adjacent (partial results that are averaged, e.g. a token's experts);
    ``g`` [T, W] the raw gate, ``g_bias`` f32 [W].  rms(v) = v / sqrt(mean(v^2) + eps); all of it f32."""
    if use_hip(x):
        return lib().stream_gated_norm(x, y, int(parts), g, g_bias, w_post, w_next, float(eps), out_dtype)
    T, W = x.shape
    v = y.float().view(T, parts, W)
    v = v[:, 0] if parts == 1 else v.sum(1) * (1.0 / parts)
    v = v * torch.sigmoid(g.float() + g_bias)
    x += v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps) * w_post
    if w_next is None:
        return None
    return (x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w_next).to(out_dtype)


def rms_cols(u, col0: int, n: int, w, eps: float):
    """Columns [col0, col0 + n) of ``u`` divided by their root mean square (f32) times ``w`` f32 [n]; a new
    [T, n] tensor in u's dtype."""
    if use_hip(u):
        return lib().rms_cols(u, int(col0), int(n), w, float(eps))
    v = u[:, col0:col0 + n].float()
    return (v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps) * w).to(u.dtype)


def rot_kv_write(q, H: int, qdim: int, k, G: int, kdim: int, kshared, sdim: int, v, vdim: int, rot_off: int, rot: int, freq,
                 mag: float, positions, k_cache, v_cache, slots, v_other=None, v_blend: float = 0.0):
    """Rotate and file one step's queries and keys.

    ``q`` rows hold H heads of ``qdim`` columns (rotated in place); a key head is ``[k head part (kdim) |
    kshared (sdim, the same for all G heads) | zeros]`` up to the cache's head size; ``v`` rows hold G heads
    of ``vdim`` columns.  Dimensions ``rot_off + 2 i`` and ``rot_off + 2 i + 1`` (i < rot / 2) of every query and
    key head are rotated by the angle ``position * freq[i]`` (f32), cos and sin both times ``mag``.  Keys and values
    go to the paged cache at ``slots`` (< 0: nothing is cached).  With ``v_other`` (rows of G heads of ``vdim``
    columns, e.g. an earlier layer's values of the same tokens) the cached value is the f32 blend
    ``(1 - v_blend) * v + v_blend * v_other``."""
    if use_hip(q):
        lib().rot_kv_write(q, H, qdim, k, G, kdim, kshared, sdim, v, vdim, int(rot_off), int(rot), freq, float(mag), positions,
                           k_cache, v_cache, slots, v_other, float(v_blend))
        return q
    T = q.shape[0]
    half = rot // 2
    ang = positions[:T].float().view(T, 1, 1) * freq.float()[:half].view(1, 1, half)
    c, s = torch.cos(ang) * mag, torch.sin(ang) * mag

    def rot(x):
        a, b = x[..., rot_off:rot_off + 2 * half:2].clone(), x[..., rot_off + 1:rot_off + 2 * half:2].clone()
        x[..., rot_off:rot_off + 2 * half:2] = a * c - b * s
        x[..., rot_off + 1:rot_off + 2 * half:2] = b * c + a * s
        return x

    qq = q[:, : H * qdim].float().reshape(T, H, qdim).clone()
    if half:
        q[:, : H * qdim] = rot(qq).reshape(T, -1).to(q.dtype)
    kd = k_cache.shape[3]
    kk = torch.zeros(T, G, kd, dtype=torch.float32, device=q.device)
    kk[..., :kdim] = k[:, : G * kdim].float().reshape(T, G, kdim)
    if kshared is not None:
        kk[..., kdim:kdim + sdim] = kshared[:, :sdim].float().reshape(T, 1, sdim)
    if half:
        kk = rot(kk)
    vv = torch.zeros(T, G, v_cache.shape[2], dtype=torch.float32, device=q.device)
    vv[..., :vdim] = v[:, : G * vdim].float().reshape(T, G, vdim)
    if v_other is not None:
        vv[..., :vdim] = (1.0 - v_blend) * vv[..., :vdim] + v_blend * v_other[:, : G * vdim].float().reshape(T, G, vdim)
    BS = k_cache.shape[2]
    sl = slots[:T].long()
    ok = sl >= 0
    blk, off = sl[ok] // BS, sl[ok] % BS
    k_cache[blk, :, off, :] = kk[ok].to(k_cache.dtype)
    v_cache[blk, :, :, off] = vv[ok].to(v_cache.dtype)
    return q


def pool_kv_write(k_cache, v_cache, pk_cache, pv_cache, P: int, block_tables, ctx_lens, cu_q, slots, row0: int, max_len: int):
    """For every sequence of the step (``ctx_lens[s]`` cached tokens, of which the rows ``[cu_q[s],
    cu_q[s + 1])`` are new; ``cu_q`` None: one new row each) and every block b of ``P`` positions whose last
    position is new: the f32 mean of the block's P cached keys and of its values, filed in the pooled cache
    pair at the logical position b of the sequence's block table.  Sequence s is skipped when the slot of its
    first row, ``slots[row0 + first row]``, is negative (a padding row).  ``max_len``: the most new rows of a
    sequence."""
    if use_hip(k_cache):
        lib().pool_kv_write(k_cache, v_cache, pk_cache, pv_cache, int(P), block_tables, ctx_lens, cu_q, slots, int(row0),
                            int(max_len))
        return
    BS = k_cache.shape[2]
    cu = cu_q.tolist() if cu_q is not None else list(range(ctx_lens.numel() + 1))
    for s in range(len(cu) - 1):
        if int(slots[row0 + cu[s]]) < 0:
            continue
        ctx = int(ctx_lens[s])
        past = ctx - (cu[s + 1] - cu[s])
        bt = block_tables[s].long()
        for b in range(past // P, ctx // P):
            pos = torch.arange(b * P, b * P + P)
            blk, off = bt[pos // BS], pos % BS
            km = k_cache[blk, :, off, :].float().sum(0) * (1.0 / P)         # [G, dim]
            vm = v_cache[blk, :, :, off].float().sum(0) * (1.0 / P)         # [G, vdim]
            pk_cache[bt[b // BS], :, b % BS, :] = km.to(pk_cache.dtype)
            pv_cache[bt[b // BS], :, :, b % BS] = vm.to(pv_cache.dtype)


def moe_route(ids, table, experts: int):
    """(seg int32 [experts + 1], order int32 [T * top]): the (token, choice) pairs ``t * top + k`` sorted by
    their expert ``table[ids[t], k]`` (``ids`` None: ``table[t, k]``, a table with one row per token of the
    step); pairs ``order[seg[e] : seg[e + 1]]`` belong to expert e."""
    if use_hip(table):
        seg, order = lib().moe_route(ids, table, int(experts))
        return seg, order
    e = (table if ids is None else table[ids.long()]).reshape(-1).long()
    order = torch.sort(e, stable=True).indices.to(torch.int32)
    seg = torch.zeros(experts + 1, dtype=torch.int32)
    seg[1:] = torch.cumsum(torch.bincount(e, minlength=experts), 0)
    return seg, order


def table_experts(h, ids, table, w_gate_up, w_down, top: int):
    """Feed-forward of table-routed experts: token t runs the experts ``table[ids[t]]`` (int32 [vocab, top]),
    each ``W_down (silu(W_gate h) * (W_up h))``.  ``w_gate_up`` [E, 2 * ffp, W] (gate rows, then up rows, each
    padded with zero rows to ffp), ``w_down`` [E, W, ffp].  Returns the experts' results un-summed,
    [T * top, W] in h's dtype with a token's ``top`` rows adjacent: the consumer averages them in f32
    (``stream_gated_norm(parts=top)``)."""
    return run_experts(h, ids, table, w_gate_up, w_down, top)


def run_experts(h, ids, table, w_gate_up, w_down, top: int):
    """The expert products behind ``table_experts`` (``ids`` int32 [T] index the table's rows) and
    ``routed_experts`` (``ids`` None: ``table`` int32 [T, top] holds each row's own choice)."""
    T, W = h.shape
    E, ffp = w_gate_up.shape[0], w_down.shape[2]
    if use_hip(h):
        seg, order = moe_route(ids, table, E)
        if (h.dtype == torch.bfloat16 and T * top >= GROUPED_DENSE_MIN_ROWS * E and lib().gemm_grouped_supported(2 * ffp, W, True)
                and lib().gemm_grouped_supported(W, ffp, False)):
            # prompt-sized steps on the framework's dense GEMM tiles, one GEMM per expert inside one launch: the first
            # product reads each pair's token row in place, the second writes each result into its pair's row
            mid = lib().gemm_grouped(h, seg, w_gate_up, True, torch.div(order, top, rounding_mode="floor"), None)
            return lib().gemm_grouped(mid, seg, w_down, False, None, order)
        mid = lib().moe_gemm(h, order, seg, w_gate_up, int(top), True)          # [T * top, ffp], sorted-pair order
        return lib().moe_gemm(mid, order, seg, w_down, int(top), False)         # [T * top, W], pair order
    e = (table if ids is None else table[ids.long()]).long()                    # [T, top]
    out = torch.zeros(T * top, W, dtype=h.dtype, device=h.device)
    pair_e = e.reshape(-1)
    rows = torch.arange(T * top, device=h.device) // top
    for ex in pair_e.unique().tolist():
        sel = (pair_e == ex).nonzero().squeeze(1)
        gu = F.linear(h[rows[sel]], w_gate_up[ex])
        mid = (F.silu(gu[:, :ffp].float()) * gu[:, ffp:].float()).to(h.dtype)
        out[sel] = F.linear(mid, w_down[ex])
    return out

"""Entry points of the sequence-mixer kernels beside softmax attention: an f32 residual stream
(``csrc/stream_f32.hip``), sigmoid attention with a log-distance penalty over a paged cache
(``csrc/attn_sigmoid.hip``), a Mamba-2 style state-space mixer (``csrc/ssm.hip``), a post-norm f32
stream with layer norms (``csrc/stream_ln.hip``) and softmax attention with a sink under a causal / chunk /
window mask over the same paged cache (``csrc/attn_sink.hip``).  The linear-state scans are in ``ops.delta``.

GPU tensors go to the HIP kernels (bf16 or f32 activations); CPU tensors to the torch
implementations below, which keep the kernels' layouts and their split of what is 32-bit:

* K cache ``[blocks, G, BS, dim]``, V cache key-contiguous ``[blocks, G, vdim, BS]``;
* sequences of a step: rows ``[cu[s], cu[s+1])``, state slot ``slots[s]`` (< 0: padding row),
  fresh state when ``positions[cu[s]] == 0``;
* conv state ``[slots, taps - 1, C]`` (activation dtype), SSM state ``[slots, heads, P, N]`` f32.
"""
from __future__ import annotations

from typing import Optional, Sequence

import numpy as np
import torch
import torch.nn.functional as F

from ._ext import lib, use_hip

__all__ = ["embed_pos", "stream_rmsnorm", "softcap", "linear_swiglu_any", "unitnorm_kv_write", "sig_prefill_tiles", "sig_decode_splits",
           "sigmoid_attention_prefill", "sigmoid_attention_decode", "sigattn_supported", "conv_silu", "ssm_scan",
           "gated_group_rmsnorm", "embed_stream", "stream_layernorm", "gelu_tanh_mul", "dual_rmsnorm_mean", "normrope_kv_write",
           "sink_attention_prefill", "sink_attention_decode", "mask_first_key", "pooled_blocks_seen", "MASK_CAUSAL", "MASK_CHUNK",
           "MASK_WINDOW"]

SIG_TILE_ROWS = 16       # queries per wave of the prefill kernel
SIG_MAX_HEAD = 256       # largest per-head q/k or v size the kernels are built for


# ------------------------------------------------------------------ f32 residual stream
def embed_pos(ids, positions, tok, pos, keep_copy: bool = False):
    """x f32 [T, W] = tok[ids] + pos[positions]; with ``keep_copy`` a second tensor of the same
    values (for models that add the embedding output to the stream again)."""
    if use_hip(tok):
        r = lib().embed_pos(ids, positions, tok, pos, keep_copy)
        return (r[0], r[1]) if keep_copy else (r[0], None)
    x = tok[ids.long()].float() + pos[positions.long()].float()
    return x, (x.clone() if keep_copy else None)


def stream_rmsnorm(x, a=None, b=None, e=None, mult: float = 1.0, w=None, w_offset: float = 0.0, eps: float = 1e-5,
                   idx=None, out_dtype=torch.bfloat16, a_bias=None):
    """``x += mult * (a + a_bias + b) + e`` in place (f32), then ``x / sqrt(mean(x^2) + eps) *
    (w_offset + w)`` in ``out_dtype``.  With ``idx`` (int64 rows) only those rows are computed and
    ``x`` is left as it was.  ``a_bias`` (f32 [W]): the bias of the projection that produced ``a``,
    added here so that the projection itself runs on the bias-free GEMM kernels."""
    if use_hip(x):
        return lib().stream_rmsnorm(x, a, a_bias if a is not None else None, b, e, float(mult), w, float(w_offset),
                                    float(eps), idx, out_dtype)
    if a is not None and a_bias is not None:
        a = a.float() + a_bias
    v = x if idx is None else x.index_select(0, idx)
    sel = (lambda t: t) if idx is None else (lambda t: t.index_select(0, idx))
    d = None
    for t in (a, b):
        if t is not None:
            d = sel(t).float() if d is None else d + sel(t).float()
    if d is not None:
        v = v + mult * d
    if e is not None:
        v = v + sel(e)
    if idx is None and v is not x:
        x.copy_(v)
    h = v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps)
    if w is not None:
        h = h * (w_offset + w.float())
    return h.to(out_dtype)


def softcap(z, cap: float):
    """``cap * tanh(z / cap)`` as f32 (cap <= 0: a plain f32 copy)."""
    if use_hip(z):
        return lib().softcap(z, float(cap))
    zf = z.float()
    return cap * torch.tanh(zf / cap) if cap > 0 else zf


def linear_swiglu_any(x, w_gate_up):
    """silu(x Wg^T) * (x Wu^T) for a fused [Wg; Wu] weight in bf16 (the GEMM's SwiGLU epilogue) or,
    for f32 activations on the GPU, a true-f32 library product and an f32 activation kernel."""
    from . import _library, linear_swiglu

    if use_hip(x) and x.dtype == torch.float32:
        return lib().silu_mul_f32(_library(x, w_gate_up, None, None, (True, w_gate_up.shape[0], w_gate_up.shape[1], 1)))
    return linear_swiglu(x, w_gate_up)


# ------------------------------------------------------------------ sigmoid attention
def sigattn_supported(H: int, G: int, dim: int, vdim: int, block_size: int, dtype) -> bool:
    ev = 16 // torch.tensor([], dtype=dtype).element_size()
    return (H % G == 0 and dim % ev == 0 and vdim % ev == 0 and block_size % 16 == 0
            and max(dim, vdim) <= SIG_MAX_HEAD)


def unitnorm_kv_write(qkv, H: int, G: int, dim: int, vdim: int, eps: float, k_cache, v_cache, slots,
                      norm_dim: Optional[int] = None, bias=None):
    """Rows ``[q: H dim | k: G dim | v: G vdim]``: q and k become x / sqrt(mean(x^2) + eps) per head
    (f32 arithmetic; q in place, k into the cache), v goes into the cache.  Slots < 0 cache nothing.
    ``norm_dim``: the divisor of the mean when the heads carry zero padding columns (default dim).
    ``bias`` [row width]: the projection's bias, added first in f32 (the projection then runs bias-free)."""
    norm_dim = dim if norm_dim is None else int(norm_dim)
    if use_hip(qkv):
        lib().unitnorm_kv_write(qkv, H, G, dim, vdim, norm_dim, float(eps), k_cache, v_cache, slots, bias)
        return qkv
    T = qkv.shape[0]
    if bias is not None:
        qkv.copy_((qkv.float() + bias.float()).to(qkv.dtype))
    qk = qkv[:, : (H + G) * dim].float().view(T, H + G, dim)
    qk = qk / torch.sqrt(qk.pow(2).sum(-1, keepdim=True) / norm_dim + eps)
    qkv[:, : (H + G) * dim] = qk.reshape(T, -1).to(qkv.dtype)
    BS = k_cache.shape[2]
    sl = slots[:T].long()
    ok = sl >= 0
    blk, off = sl[ok] // BS, sl[ok] % BS
    k_cache[blk, :, off, :] = qkv[ok, H * dim:(H + G) * dim].view(-1, G, dim)
    v_cache[blk, :, :, off] = qkv[ok, (H + G) * dim:].view(-1, G, vdim)
    return qkv


def sig_prefill_tiles(q_lens: Sequence[int], ctx_lens: Optional[Sequence[int]] = None):
    """(tile_seq, tile_q0) int32: one entry per 16-query tile of each chunk, heaviest first -- a tile
    attends every key up to its last query, so its cost is its end position in the sequence."""
    tiles = []
    for b, n in enumerate(q_lens):
        past = (ctx_lens[b] - n) if ctx_lens is not None else 0
        tiles += [(past + s + SIG_TILE_ROWS, b, s) for s in range(0, n, SIG_TILE_ROWS)]
    tiles.sort(key=lambda t: -t[0])
    return (np.asarray([t[1] for t in tiles], dtype=np.int32), np.asarray([t[2] for t in tiles], dtype=np.int32))


def sig_decode_splits(B: int, G: int, rep: int, max_context: int) -> int:
    """Workgroups per (sequence, kv group) of the decode kernel: enough to give the chip about two
    workgroups per CU, never more than one per 128 keys (a workgroup's 4 waves take 32 keys each
    per round).  Static per (batch bucket, model, max context): safe to capture."""
    groups = max(1, B * G * ((rep + 15) // 16))
    return int(max(1, min(512 // groups, (max_context + 127) // 128)))


def _gather_kv(k_cache, v_cache, table, n):
    BS = k_cache.shape[2]
    nb = (n + BS - 1) // BS
    bt = table[:nb].long()
    k = k_cache[bt].permute(0, 2, 1, 3).reshape(nb * BS, k_cache.shape[1], -1)[:n]     # [n, G, dim]
    v = v_cache[bt].permute(0, 3, 1, 2).reshape(nb * BS, v_cache.shape[1], -1)[:n]     # [n, G, vdim]
    return k.float(), v.float()


def _sig_rows(q, k, v, qpos, scale, r1, r2, pb):
    """q f32 [S, H, dim] at positions qpos [S]; k/v f32 [n, G, *] at positions 0..n-1."""
    H, G = q.shape[1], k.shape[1]
    rep = H // G
    kk = k.repeat_interleave(rep, dim=1)
    vv = v.repeat_interleave(rep, dim=1)
    s = torch.einsum("ihd,jhd->hij", q, kk) * scale
    d = qpos.view(-1, 1) - torch.arange(k.shape[0], device=q.device).view(1, -1)
    pen = r1.view(-1, 1, 1) * torch.log(1.0 + r2.view(-1, 1, 1) * d.clamp(min=0).float()[None])
    wgt = torch.sigmoid(s - pen + pb.view(-1, 1, 1)) * (d >= 0)[None]
    return torch.einsum("hij,jhd->ihd", wgt, vv)


def sigmoid_attention_prefill(q, k_cache, v_cache, block_tables, cu_q, ctx_lens, H: int, G: int, dim: int, vdim: int,
                              scale: float, r1, r2, pb, out, tiles=None, q_lens_cpu=None):
    """Causal sigmoid attention of query chunks over their sequences' cached keys (the chunk's own
    keys included).  q: rows whose first H * dim columns are the unit-RMS queries; out [T, H * vdim]."""
    if use_hip(q):
        if tiles is None:
            ql = q_lens_cpu if q_lens_cpu is not None else (cu_q[1:] - cu_q[:-1]).tolist()
            ts, tq = sig_prefill_tiles(ql, ctx_lens.tolist())
            tiles = (torch.from_numpy(ts).to(q.device), torch.from_numpy(tq).to(q.device))
        lib().sigattn_prefill(q, k_cache, v_cache, block_tables, cu_q, ctx_lens, tiles[0], tiles[1], H, G, dim, vdim,
                              float(scale), r1, r2, pb, out)
        return out
    cu = cu_q.tolist()
    for b in range(len(cu) - 1):
        s0, s1 = cu[b], cu[b + 1]
        n = int(ctx_lens[b])
        k, v = _gather_kv(k_cache, v_cache, block_tables[b], n)
        qq = q[s0:s1, : H * dim].float().view(s1 - s0, H, dim)
        qpos = torch.arange(n - (s1 - s0), n, device=q.device)
        out[s0:s1, : H * vdim] = _sig_rows(qq, k, v, qpos, scale, r1, r2, pb).reshape(s1 - s0, H * vdim).to(out.dtype)
    return out


def sigmoid_attention_decode(q, k_cache, v_cache, block_tables, ctx_lens, H: int, G: int, dim: int, vdim: int,
                             scale: float, r1, r2, pb, out, splits: int = 1, part=None):
    """One query row per sequence at its last position (ctx - 1) over all its cached keys."""
    B = q.shape[0]
    if use_hip(q):
        if splits > 1 and part is None:
            part = torch.empty(B * H * splits * vdim, dtype=torch.float32, device=q.device)
        lib().sigattn_decode(q, k_cache, v_cache, block_tables, ctx_lens, int(splits), H, G, dim, vdim, float(scale),
                             r1, r2, pb, out, part)
        return out
    for b in range(B):
        n = int(ctx_lens[b])
        k, v = _gather_kv(k_cache, v_cache, block_tables[b], n)
        qq = q[b:b + 1, : H * dim].float().view(1, H, dim)
        qpos = torch.tensor([n - 1], device=q.device)
        out[b:b + 1, : H * vdim] = _sig_rows(qq, k, v, qpos, scale, r1, r2, pb).reshape(1, H * vdim).to(out.dtype)
    return out


# ------------------------------------------------------------------ state-space mixer
def conv_silu(u, col0: int, C: int, w, bias, state, cu, slots, positions, max_len: int, act: bool = True):
    """silu(causal depthwise conv + bias) of columns [col0, col0 + C) of ``u``, per sequence, reading
    the inputs before a chunk from ``state`` and leaving the sequence's last ``taps - 1`` inputs there.
    w f32 [C, taps] (last column = the current token), bias f32 [C] or None.  ``act`` False: the
    convolution alone, without the SiLU."""
    if use_hip(u):
        return lib().conv_silu(u, col0, C, w, bias, state, cu, slots, positions, int(max_len), bool(act))
    taps = w.shape[1]
    out = torch.zeros(u.shape[0], C, dtype=u.dtype, device=u.device)
    cul, sl = cu.tolist(), slots.tolist()
    for s in range(len(cul) - 1):
        r0, r1 = cul[s], cul[s + 1]
        if sl[s] < 0 or r1 <= r0:
            continue
        x = u[r0:r1, col0:col0 + C]
        if taps > 1:
            prev = state[sl[s]] if int(positions[r0]) > 0 else torch.zeros_like(state[sl[s]])
            full = torch.cat([prev, x], 0)                                    # [taps - 1 + n, C]
            state[sl[s]] = full[-(taps - 1):]
        else:
            full = x
        ff = full.float()
        acc = torch.zeros(r1 - r0, C, dtype=torch.float32, device=u.device)
        for k in range(taps):
            acc += ff[k:k + r1 - r0] * w[:, k]
        if bias is not None:
            acc += bias
        out[r0:r1] = (F.silu(acc) if act else acc).to(u.dtype)
    return out


def ssm_scan(xbc, dt, heads: int, P: int, N: int, groups: int, dt_bias, A_log, D, state, cu, slots, positions,
             max_len: int = 1):
    """y f32 [T, heads * P]: per head, S_t = exp(-exp(A_log) dt_t) S_{t-1} + dt_t B_t x_t^T and
    y_t = S_t^T C_t + D x_t with dt_t = softplus(dt_t + dt_bias); x | B | C are the columns of
    ``xbc``; the f32 state of each sequence is read from / left in ``state[slot]`` ([heads, P, N]).
    ``max_len``: the longest sequence of the step (from 8 rows on the GPU runs the chunked matrix
    form, below that the token-by-token kernel)."""
    if use_hip(xbc):
        return lib().ssm_scan(xbc, dt, heads, P, N, groups, dt_bias, A_log, D, state, cu, slots, positions, int(max_len))
    inner = heads * P
    y = torch.zeros(xbc.shape[0], inner, dtype=torch.float32, device=xbc.device)
    cul, sl = cu.tolist(), slots.tolist()
    nA = -torch.exp(A_log.float())
    hg = heads // groups
    for s in range(len(cul) - 1):
        r0, r1 = cul[s], cul[s + 1]
        if sl[s] < 0 or r1 <= r0:
            continue
        S = state[sl[s]].clone() if int(positions[r0]) > 0 else torch.zeros_like(state[sl[s]])   # [heads, P, N]
        rows = xbc[r0:r1].float()
        x = rows[:, :inner].view(-1, heads, P)
        Bm = rows[:, inner:inner + groups * N].view(-1, groups, N).repeat_interleave(hg, dim=1)
        Cm = rows[:, inner + groups * N:].view(-1, groups, N).repeat_interleave(hg, dim=1)
        dts = F.softplus(dt[r0:r1].float() + dt_bias, threshold=20.0)
        dA = torch.exp(nA * dts)
        for t in range(r1 - r0):
            S = dA[t].view(-1, 1, 1) * S + (dts[t].view(-1, 1) * x[t]).unsqueeze(-1) * Bm[t].unsqueeze(1)
            y[r0 + t] = (torch.einsum("hpn,hn->hp", S, Cm[t]) + D.view(-1, 1) * x[t]).reshape(-1)
        state[sl[s]] = S
    return y


def gated_group_rmsnorm(y, z, w, ngroups: int, eps: float):
    """(y * silu(z)) normalised to unit RMS within each of ``ngroups`` equal column groups, times w;
    y f32, z and the result in the activation dtype."""
    if use_hip(y):
        return lib().gated_group_rmsnorm(y, z, w, int(ngroups), float(eps))
    T, inner = y.shape
    v = (y * F.silu(z.float())).view(T, ngroups, inner // ngroups)
    v = v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps)
    return (v.reshape(T, inner) * w).to(z.dtype)


# ------------------------------------------------------------------ post-norm f32 stream
def embed_stream(ids, tok, out_dtype=torch.bfloat16, scale: float = 1.0):
    """(x f32 [T, W], h): the token rows times ``scale`` (an f32 product) as the f32 stream and as the
    activation-dtype copy the projections read (for f32 activations both are the same tensor)."""
    if use_hip(tok):
        x, h = lib().embed_stream(ids, tok, out_dtype, float(scale))
        return x, h
    x = tok[ids.long()].float()
    if scale != 1.0:
        x = x * scale
    return x, (x if out_dtype == torch.float32 else x.to(out_dtype))


def stream_layernorm(x, y, ls, alpha: float, w, b, eps: float, out_dtype=torch.bfloat16, idx=None):
    """Post-norm stream update ``x <- LN(alpha x + ls * y) * w + b`` in place (f32; mean and variance over
    the row, variance = mean squared deviation) and the activation-dtype copy of the new ``x`` that the
    next sublayer's projections read (the same tensor for f32 activations).  ``y`` None: a plain layer
    norm of ``x``.  With ``idx`` (int64 rows) only those rows are normed into a new tensor and ``x``
    stays as it was (the rows that feed the LM head)."""
    if use_hip(x):
        return lib().stream_layernorm(x, y, ls, float(alpha), w, b, float(eps), idx, out_dtype)
    v = x if idx is None else x.index_select(0, idx)
    if y is not None:
        yy = y if idx is None else y.index_select(0, idx)
        v = alpha * v + (yy.float() * ls if ls is not None else yy.float())
    mu = v.mean(-1, keepdim=True)
    d = v - mu
    r = d / torch.sqrt(d.pow(2).mean(-1, keepdim=True) + eps) * w + b
    if idx is not None:
        return r.to(out_dtype)
    x.copy_(r)
    return x if out_dtype == torch.float32 else x.to(out_dtype)


def gelu_tanh_mul(gu):
    """[T, 2F] = [gate | up] -> gelu_tanh(gate) * up, [T, F] in the same dtype."""
    if use_hip(gu):
        return lib().gelu_tanh_mul(gu)
    F_ = gu.shape[1] // 2
    g, u = gu[:, :F_].float(), gu[:, F_:].float()
    return (F.gelu(g, approximate="tanh") * u).to(gu.dtype)


def dual_rmsnorm_mean(a, wa, b, wb, eps: float):
    """f32 [T, W]: half the sum of ``a`` and ``b``, each first scaled to unit RMS over the row and
    multiplied by its weight (two branches that read the same input and share one stream update)."""
    if use_hip(a):
        return lib().dual_rmsnorm_mean(a, wa, b, wb, float(eps))
    af, bf = a.float(), b.float()
    na = af / torch.sqrt(af.pow(2).mean(-1, keepdim=True) + eps) * wa
    nb = bf / torch.sqrt(bf.pow(2).mean(-1, keepdim=True) + eps) * wb
    return 0.5 * (na + nb)


# ------------------------------------------------------------------ softmax attention with a sink, masked to chunks
MASK_CAUSAL, MASK_CHUNK, MASK_WINDOW = 0, 1, 2


def mask_first_key(qpos: int, mask_kind: int, mask_size: int) -> int:
    """First position a query at ``qpos`` sees: causal everything, chunk = the start of its chunk of
    ``mask_size`` positions (counted from position 0 of the sequence), window = the last ``mask_size``."""
    if mask_kind == MASK_CHUNK:
        return (qpos // mask_size) * mask_size
    if mask_kind == MASK_WINDOW:
        return max(0, qpos - mask_size + 1)
    return 0


def normrope_kv_write(qkv, H: int, G: int, dim: int, vdim: int, q_w, k_w, rot_dims: int, inv_freq, positions, eps: float,
                      k_cache, v_cache, slots, v_unit: bool = True, norm_dim: Optional[int] = None, norm_vdim: Optional[int] = None):
    """Rows ``[q: H dim | k: G dim | v: G vdim | ...]``: q and k are RMS-normed per head (f32) with the
    weights ``q_w`` / ``k_w`` [dim] shared by the heads, then their first ``rot_dims`` dimensions rotated
    by the row's position (dimension i pairs with i + rot_dims / 2, angle = position * inv_freq[i], f32);
    v is divided by its RMS per head when ``v_unit``.  q in place, k and v into the paged cache
    (K ``[blocks, G, BS, dim]``, V key-contiguous ``[blocks, G, vdim, BS]``); slots < 0 cache nothing.
    ``norm_dim`` / ``norm_vdim``: divisors of the means when heads carry zero padding columns."""
    norm_dim = dim if norm_dim is None else int(norm_dim)
    norm_vdim = vdim if norm_vdim is None else int(norm_vdim)
    if use_hip(qkv):
        lib().normrope_kv_write(qkv, H, G, dim, vdim, norm_dim, norm_vdim, q_w, k_w, int(rot_dims), inv_freq, positions, float(eps),
                                k_cache, v_cache, slots, bool(v_unit))
        return qkv
    T = qkv.shape[0]
    half = rot_dims // 2
    ang = positions[:T].float().view(T, 1, 1) * inv_freq.float()[:half].view(1, 1, half)
    c, s = torch.cos(ang), torch.sin(ang)

    def prep(x, w):
        x = x / torch.sqrt(x.pow(2).sum(-1, keepdim=True) / norm_dim + eps) * w
        u, v = x[..., :half].clone(), x[..., half:rot_dims].clone()
        x[..., :half] = u * c - v * s
        x[..., half:rot_dims] = v * c + u * s
        return x

    q = prep(qkv[:, : H * dim].float().view(T, H, dim), q_w)
    k = prep(qkv[:, H * dim:(H + G) * dim].float().view(T, G, dim), k_w)
    v = qkv[:, (H + G) * dim:(H + G) * dim + G * vdim].float().view(T, G, vdim)
    if v_unit:
        v = v / torch.sqrt(v.pow(2).sum(-1, keepdim=True) / norm_vdim + eps)
    qkv[:, : H * dim] = q.reshape(T, -1).to(qkv.dtype)
    BS = k_cache.shape[2]
    sl = slots[:T].long()
    ok = sl >= 0
    blk, off = sl[ok] // BS, sl[ok] % BS
    k_cache[blk, :, off, :] = k[ok].to(k_cache.dtype)
    v_cache[blk, :, :, off] = v[ok].to(v_cache.dtype)
    return qkv


def pooled_blocks_seen(qpos, mask_size: int, pool: int):
    """Number of leading blocks of ``pool`` positions that the window of ``mask_size`` positions ending at
    ``qpos`` has left behind entirely (block b is seen when b * pool + pool - 1 <= qpos - mask_size)."""
    if isinstance(qpos, torch.Tensor):
        return ((qpos - mask_size + 1).clamp(min=0)) // pool
    return max(0, qpos - mask_size + 1) // pool


def _sink_rows(q, k, v, qpos, hscale, mask_kind, mask_size, sink, pooled=None, keep_first=0, cap=0.0):
    """q f32 [S, H, dim] at positions qpos [S]; k/v f32 [n, G, *] at positions 0..n-1.  ``pooled`` = (pk, pv
    f32 [nb, G, *], pool): one more key / value per block of ``pool`` positions, seen by a query once the
    block is entirely behind its window, in the same softmax.  ``keep_first``: the first positions stay
    visible behind a window; ``cap`` > 0: scores become cap * tanh(score / cap)."""
    H, G = q.shape[1], k.shape[1]
    rep = H // G
    s = torch.einsum("ihd,jhd->hij", q, k.repeat_interleave(rep, dim=1)) * hscale.view(-1, 1, 1)
    if cap > 0:
        s = cap * torch.tanh(s / cap)
    j = torch.arange(k.shape[0], device=q.device).view(1, -1)
    i = qpos.view(-1, 1)
    if pooled is not None and pooled[0].shape[0]:
        pk, pv, pool = pooled
        sp = torch.einsum("ihd,jhd->hij", q, pk.repeat_interleave(rep, dim=1)) * hscale.view(-1, 1, 1)
        bj = torch.arange(pk.shape[0], device=q.device).view(1, -1)
        sp = sp.masked_fill(~(bj < pooled_blocks_seen(i, mask_size, pool))[None], float("-inf"))
        lo = (i - mask_size + 1).clamp(min=0)
        s = s.masked_fill(~((j <= i) & (j >= lo))[None], float("-inf"))
        s = torch.cat([sp, s], -1)
        m = s.amax(-1, keepdim=True)
        if sink:
            m = m.clamp(min=0.0)
        e = torch.exp(s - m)
        den = e.sum(-1, keepdim=True) + (torch.exp(-m) if sink else 0.0)
        vv = torch.cat([pv, v], 0).repeat_interleave(rep, dim=1)
        return torch.einsum("hij,jhd->ihd", e / den, vv)
    if mask_kind == MASK_CHUNK:
        lo = (i // mask_size) * mask_size
    elif mask_kind == MASK_WINDOW:
        lo = (i - mask_size + 1).clamp(min=0)
    else:
        lo = torch.zeros_like(i)
    seen = (j <= i) & ((j >= lo) | (j < keep_first))
    s = s.masked_fill(~seen[None], float("-inf"))
    m = s.amax(-1, keepdim=True)
    if sink:
        m = m.clamp(min=0.0)                             # the sink's score 0 bounds the maximum from below
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True) + (torch.exp(-m) if sink else 0.0)
    return torch.einsum("hij,jhd->ihd", e / den, v.repeat_interleave(rep, dim=1))


def _pooled_of(pool, table, n):
    """(pk, pv f32 [n // P, G, *], P) of a sequence of ``n`` cached tokens: pooled entry b lives at the
    logical position b of the sequence's own block table in the pooled cache pair."""
    if pool is None:
        return None
    pk_cache, pv_cache, P = pool
    nb = n // P
    if nb == 0:
        return (torch.zeros(0, pk_cache.shape[1], pk_cache.shape[3]), torch.zeros(0, pv_cache.shape[1], pv_cache.shape[2]), P)
    pk, pv = _gather_kv(pk_cache, pv_cache, table, nb)
    return pk, pv, P


def _check_mask_options(mask_kind, pool, keep_first):
    if pool is not None and mask_kind != MASK_WINDOW:
        raise ValueError("pooled blocks go with a sliding window")
    if keep_first and (mask_kind != MASK_WINDOW or pool is not None):
        raise ValueError("kept first positions go with a sliding window without pooled blocks")


def _gated(o, gate, r0, r1, gate_col, H, vdim, gate_elem):
    """o f32 [S, H, vdim] times the sigmoid of the gate rows [r0, r1): one column per head, or per element."""
    if gate is None:
        return o
    if gate_elem:
        return o * torch.sigmoid(gate[r0:r1, gate_col:gate_col + H * vdim].float()).view(-1, H, vdim)
    return o * torch.sigmoid(gate[r0:r1, gate_col:gate_col + H].float()).unsqueeze(-1)


def sink_attention_prefill(q, k_cache, v_cache, block_tables, cu_q, ctx_lens, H: int, G: int, dim: int, vdim: int, hscale,
                           mask_kind: int, mask_size: int, sink: bool, gate, gate_col: int, out, tiles=None, q_lens_cpu=None,
                           pool=None, keep_first: int = 0, softcap: float = 0.0, gate_elem: bool = False):
    """Softmax attention of query chunks over their sequences' cached keys inside the mask
    (``mask_first_key``), with ``sink``: one more term of score 0 and no value in the denominator.
    ``hscale`` f32 [H]: the score multiplier of each head.  ``gate`` (or None): rows aligned with ``q``
    whose columns ``gate_col + h`` hold the raw output gate of head h; the head's output is multiplied by
    its sigmoid.  q: rows whose first H * dim columns are the prepared queries; out [T, H * vdim].
    ``pool`` = (pooled K cache, pooled V cache, P), window masks only: beside its window a query sees one
    pooled key / value per block of P positions entirely behind the window (``pooled_blocks_seen``), filed by
    ``pool_kv_write`` at the logical position b of the same block table.
    ``keep_first`` (window masks, no pooling): positions below it stay visible to every later query.  ``softcap`` >
    0: a score s becomes softcap * tanh(s / softcap) before the softmax.  ``gate_elem``: the gate has one column
    per output element, ``gate_col + h * vdim + d``, instead of one per head."""
    _check_mask_options(mask_kind, pool, keep_first)
    if use_hip(q):
        if tiles is None:
            ql = q_lens_cpu if q_lens_cpu is not None else (cu_q[1:] - cu_q[:-1]).tolist()
            ts, tq = sig_prefill_tiles(ql, ctx_lens.tolist())
            tiles = (torch.from_numpy(ts).to(q.device), torch.from_numpy(tq).to(q.device))
        pk, pv, P = pool if pool is not None else (None, None, 0)
        lib().sinkattn_prefill(q, k_cache, v_cache, block_tables, cu_q, ctx_lens, tiles[0], tiles[1], H, G, dim, vdim, hscale,
                               int(mask_kind), int(mask_size), bool(sink), gate, int(gate_col), out, pk, pv, int(P),
                               int(keep_first), float(softcap), bool(gate_elem))
        return out
    cu = cu_q.tolist()
    for b in range(len(cu) - 1):
        s0, s1 = cu[b], cu[b + 1]
        n = int(ctx_lens[b])
        k, v = _gather_kv(k_cache, v_cache, block_tables[b], n)
        qq = q[s0:s1, : H * dim].float().view(s1 - s0, H, dim)
        qpos = torch.arange(n - (s1 - s0), n, device=q.device)
        o = _sink_rows(qq, k, v, qpos, hscale, mask_kind, mask_size, sink, _pooled_of(pool, block_tables[b], n), keep_first, softcap)
        out[s0:s1, : H * vdim] = _gated(o, gate, s0, s1, gate_col, H, vdim, gate_elem).reshape(s1 - s0, H * vdim).to(out.dtype)
    return out


def sink_attention_decode(q, k_cache, v_cache, block_tables, ctx_lens, H: int, G: int, dim: int, vdim: int, hscale,
                          mask_kind: int, mask_size: int, sink: bool, gate, gate_col: int, out, splits: int = 1, part=None,
                          pool=None, keep_first: int = 0, softcap: float = 0.0, gate_elem: bool = False):
    """One query row per sequence at its last position (ctx - 1) over its cached keys inside the mask
    (and the pooled blocks before it: see ``sink_attention_prefill``)."""
    B = q.shape[0]
    _check_mask_options(mask_kind, pool, keep_first)
    if use_hip(q):
        if splits > 1 and part is None:
            part = torch.empty(B * H * splits * (vdim + 2), dtype=torch.float32, device=q.device)
        pk, pv, P = pool if pool is not None else (None, None, 0)
        lib().sinkattn_decode(q, k_cache, v_cache, block_tables, ctx_lens, int(splits), H, G, dim, vdim, hscale, int(mask_kind),
                              int(mask_size), bool(sink), gate, int(gate_col), out, part, pk, pv, int(P), int(keep_first),
                              float(softcap), bool(gate_elem))
        return out
    for b in range(B):
        n = int(ctx_lens[b])
        k, v = _gather_kv(k_cache, v_cache, block_tables[b], n)
        qq = q[b:b + 1, : H * dim].float().view(1, H, dim)
        o = _sink_rows(qq, k, v, torch.tensor([n - 1], device=q.device), hscale, mask_kind, mask_size, sink,
                       _pooled_of(pool, block_tables[b], n), keep_first, softcap)
        out[b:b + 1, : H * vdim] = _gated(o, gate, b, b + 1, gate_col, H, vdim, gate_elem).reshape(1, H * vdim).to(out.dtype)
    return out

"""Sliding-window attention mixers over the engine's paged cache: grouped-query attention whose queries
also see one pooled (mean) key / value per block of positions that has left the window, grouped-query attention
with capped scores whose window keeps the first positions and whose values are blended across layers, and latent attention
(queries through a normed low-rank latent, keys and values expanded from a normed latent, a rotated key segment
common to the heads, gated heads).  Both rotate adjacent pairs of dimensions by a frequency table that carries
the scaling rule (``RotarySpec``), and both run on the masked softmax kernels of ``ops.sink_attention_*``
(window mask, no sink), so whole prompts, portions and decode rows are one code path.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import Optional

import torch

from .. import ops
from .attention import AttnMeta


@dataclass
class RotarySpec:
    """Rotation of adjacent pairs (2 i, 2 i + 1) by ``position * f_i``, ``f_i = base^(-2 i / dims)`` before
    scaling.  ``kind``: ``"none"``; ``"bands"`` -- frequencies whose wavelength is longer than
    ``original / low`` are divided by ``factor``, those shorter than ``original / high`` are kept, the band
    between is interpolated linearly in ``original / wavelength``; ``"ramp"`` -- a linear ramp over the pair
    index between the pairs that turn ``fast`` and ``slow`` times within ``original`` positions blends
    ``f_i`` (ramp 0) into ``f_i / factor`` (ramp 1), and cos / sin are multiplied by ``0.1 ln(factor) + 1``."""
    dims: int = 0
    base: float = 10000.0
    kind: str = "none"
    scaling: dict = field(default_factory=dict)

    @classmethod
    def from_dict(cls, rot: Optional[dict], kind: str) -> "RotarySpec":
        if not rot or not int(rot.get("dims", 0)):
            return cls()
        sc = dict(rot.get("scaling") or {})
        s = cls(int(rot["dims"]), float(rot.get("base", 10000.0)), kind if sc else "none", sc)
        if s.dims % 2:
            raise ValueError(f"rotated dimensions must be even: {rot}")
        return s

    def table(self):
        """(frequencies as float64 list [dims / 2], magnitude of cos and sin)."""
        d, sc = self.dims, self.scaling
        f = [self.base ** (-2.0 * i / d) for i in range(d // 2)]
        if self.kind == "bands":
            factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
            out = []
            for x in f:
                wl = 2.0 * math.pi / x
                if wl < orig / high:
                    out.append(x)
                elif wl > orig / low:
                    out.append(x / factor)
                else:
                    t = (orig / wl - low) / (high - low)
                    out.append((1.0 - t) * x / factor + t * x)
            return out, 1.0
        if self.kind == "ramp":
            factor, orig, fast, slow = float(sc["factor"]), float(sc["original"]), float(sc["fast"]), float(sc["slow"])

            def pair_of(turns):
                return d * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(self.base))

            lo, hi = max(math.floor(pair_of(fast)), 0), min(math.ceil(pair_of(slow)), d - 1)
            out = []
            for i, x in enumerate(f):
                r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
                out.append(x / factor * r + x * (1.0 - r))
            return out, 0.1 * math.log(factor) + 1.0
        return f, 1.0

    def freq_tensor(self, device) -> torch.Tensor:
        """f32 [max(dims / 2, 1)], rounded once from float64 (an unused 0 when nothing is rotated)."""
        f, _ = self.table()
        return torch.tensor(f or [0.0], dtype=torch.float64).to(torch.float32).to(device)

    @property
    def magnitude(self) -> float:
        return self.table()[1]


def _pad8(n: int) -> int:
    return -(-int(n) // 8) * 8


def _cache_pair(num_blocks, G, block_size, dim, vdim, dtype, device):
    return (torch.zeros(num_blocks, G, block_size, dim, dtype=dtype, device=device),
            torch.zeros(num_blocks, G, vdim, block_size, dtype=dtype, device=device))


@dataclass
class PooledWindowAttnSpec:
    """Grouped-query softmax attention: query i sees the ``window`` positions up to its own and, when
    ``pool`` > 0, the mean key / value of every block of ``pool`` positions that this window has left behind
    entirely, all in one softmax.  Head sizes here are the kernels' (multiples of 8); the checkpoint's may be
    smaller (zero weight rows / columns)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    pool: int = 0
    rot: RotarySpec = field(default_factory=RotarySpec)

    @classmethod
    def from_dict(cls, m: dict) -> "PooledWindowAttnSpec":
        mask = m.get("mask") or {}
        s = cls(int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m.get("vdim", m["dim"])),
                float(m.get("scale", int(m["dim"]) ** -0.5)), int(mask.get("size", 0)), int(mask.get("pool") or 0),
                RotarySpec.from_dict(m.get("rot"), "bands"))
        if s.heads % s.kv_heads or s.window < 1 or s.pool < 0 or s.rot.dims > s.dim:
            raise ValueError(f"unsupported attention sizes {m}")
        return s

    def padded(self) -> "PooledWindowAttnSpec":
        return PooledWindowAttnSpec(self.heads, self.kv_heads, _pad8(self.dim), _pad8(self.vdim), self.scale, self.window,
                                    self.pool, self.rot)

    def make_caches(self, num_blocks: int, block_size: int, dtype, device) -> tuple:
        """(K, V) and, with pooling, (pooled K, pooled V) of the same shapes: pooled entry b of a sequence
        sits at the logical position b of its block table."""
        c = _cache_pair(num_blocks, self.kv_heads, block_size, self.dim, self.vdim, dtype, device)
        if self.pool:
            c += _cache_pair(num_blocks, self.kv_heads, block_size, self.dim, self.vdim, dtype, device)
        return c

    def bytes_per_token(self, dtype) -> int:
        n = self.kv_heads * (self.dim + self.vdim) * torch.tensor([], dtype=dtype).element_size()
        return n * (2 if self.pool else 1)


def _attend(q, k_cache, v_cache, meta: AttnMeta, H, G, dim, vdim, hscale, window, gate, gate_col, out, pool, keep_first=0,
            softcap=0.0, gate_elem=False):
    """Prompt rows and decode rows of a step through the masked softmax kernels.  ``window`` 0: causal."""
    Tp, Bd = meta.num_prefill_tokens, meta.num_decode
    kind = ops.MASK_WINDOW if window > 0 else ops.MASK_CAUSAL
    opt = dict(pool=pool, keep_first=keep_first if window > 0 else 0, softcap=softcap, gate_elem=gate_elem)
    if Tp:
        if meta.sig_tiles is None and q.is_cuda:
            ts, tq = ops.sig_prefill_tiles(meta.q_lens_cpu, meta.ctx_lens_cpu)
            meta.sig_tiles = (torch.from_numpy(ts).to(q.device, non_blocking=True),
                              torch.from_numpy(tq).to(q.device, non_blocking=True))
        ops.sink_attention_prefill(q[:Tp], k_cache, v_cache, meta.block_tables_p, meta.cu_q, meta.ctx_lens_p, H, G, dim, vdim,
                                   hscale, kind, window, False, gate[:Tp] if gate is not None else None, gate_col,
                                   out[:Tp], tiles=meta.sig_tiles, **opt)
    if Bd:
        span = meta.block_tables_d.shape[1] * k_cache.shape[2]
        keys = (min(span, window + keep_first) if window > 0 else span) + (span // pool[2] if pool is not None else 0)
        Z = ops.sig_decode_splits(Bd, G, H // G, keys)
        ops.sink_attention_decode(q[Tp:Tp + Bd], k_cache, v_cache, meta.block_tables_d, meta.ctx_lens_d, H, G, dim, vdim,
                                  hscale, kind, window, False, gate[Tp:Tp + Bd] if gate is not None else None,
                                  gate_col, out[Tp:Tp + Bd], splits=Z, **opt)
    return out


def pooled_window_attention(qkv: torch.Tensor, caches, meta: AttnMeta, spec: PooledWindowAttnSpec, freq, hscale,
                            out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """qkv [T, q | k | v] straight from the fused projection (``spec``: the padded sizes).  One kernel rotates q
    in place and files rotated k and v in the paged cache; a second files the pooled key / value of every
    block this step completes; then prompt rows and decode rows attend through the cache.  [T, H vdim]."""
    H, G, dim, vdim = spec.heads, spec.kv_heads, spec.dim, spec.vdim
    T = qkv.shape[0]
    if out is None:
        out = torch.empty(T, H * vdim, dtype=qkv.dtype, device=qkv.device)
    k_cache, v_cache = caches[0], caches[1]
    kcol, vcol = H * dim, (H + G) * dim
    ops.rot_kv_write(qkv, H, dim, qkv[:, kcol:], G, dim, None, 0, qkv[:, vcol:], vdim, 0, spec.rot.dims, freq, spec.rot.magnitude,
                     meta.positions, k_cache, v_cache, meta.slots)
    pool = None
    if spec.pool:
        pool = (caches[2], caches[3], spec.pool)
        Tp, Bd = meta.num_prefill_tokens, meta.num_decode
        if Tp:
            ops.pool_kv_write(k_cache, v_cache, caches[2], caches[3], spec.pool, meta.block_tables_p, meta.ctx_lens_p, meta.cu_q,
                              meta.slots, 0, max(meta.q_lens_cpu))
        if Bd:
            ops.pool_kv_write(k_cache, v_cache, caches[2], caches[3], spec.pool, meta.block_tables_d, meta.ctx_lens_d, None,
                              meta.slots, Tp, 1)
    return _attend(qkv, k_cache, v_cache, meta, H, G, dim, vdim, hscale, spec.window, None, 0, out, pool)


@dataclass
class CappedWindowAttnSpec:
    """Grouped-query softmax attention without rotation: scores ``cap * tanh(scale q.k / cap)`` (``softcap`` 0:
    plain), query i sees j <= i with ``i - j < window`` or ``j < keep_first`` (``window`` 0: causal).  With
    ``v_mix`` the cached value is ``(1 - lambda) v + lambda v_first``, ``v_first`` the values that the model's
    first such layer projects for the same token (that layer itself caches its own).  Head sizes here are the
    kernels' (multiples of 8); the checkpoint's may be smaller (zero weight rows / columns)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0
    keep_first: int = 0
    softcap: float = 0.0
    v_mix: bool = False

    @classmethod
    def from_dict(cls, m: dict) -> "CappedWindowAttnSpec":
        mask = m.get("mask") or {}
        s = cls(int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m.get("vdim", m["dim"])),
                float(m.get("scale", int(m["dim"]) ** -0.5)), int(mask.get("size", 0)), int(mask.get("keep_first") or 0),
                float(m.get("softcap") or 0.0), bool(m.get("v_mix", False)))
        if s.heads % s.kv_heads or s.window < 0 or s.keep_first < 0 or s.softcap < 0:
            raise ValueError(f"unsupported attention sizes {m}")
        return s

    def padded(self) -> "CappedWindowAttnSpec":
        return CappedWindowAttnSpec(self.heads, self.kv_heads, _pad8(self.dim), _pad8(self.vdim), self.scale, self.window,
                                    self.keep_first, self.softcap, self.v_mix)

    def make_caches(self, num_blocks: int, block_size: int, dtype, device) -> tuple:
        return _cache_pair(num_blocks, self.kv_heads, block_size, self.dim, self.vdim, dtype, device)

    def bytes_per_token(self, dtype) -> int:
        return self.kv_heads * (self.dim + self.vdim) * torch.tensor([], dtype=dtype).element_size()


def capped_window_attention(qkv: torch.Tensor, caches, meta: AttnMeta, spec: CappedWindowAttnSpec, hscale, freq, v_first=None,
                            v_blend: float = 0.0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """qkv [T, q | k | v] straight from the fused projection (``spec``: the padded sizes).  One kernel files k and
    the (blended) v in the paged cache; then prompt rows and decode rows attend through the cache.  ``v_first``
    [T, G vdim]: the values to blend in with weight ``v_blend``.  ``freq``: an unused frequency table (nothing
    is rotated).  [T, H vdim]."""
    H, G, dim, vdim = spec.heads, spec.kv_heads, spec.dim, spec.vdim
    T = qkv.shape[0]
    if out is None:
        out = torch.empty(T, H * vdim, dtype=qkv.dtype, device=qkv.device)
    k_cache, v_cache = caches[0], caches[1]
    kcol, vcol = H * dim, (H + G) * dim
    ops.rot_kv_write(qkv, H, dim, qkv[:, kcol:], G, dim, None, 0, qkv[:, vcol:], vdim, 0, 0, freq, 1.0, meta.positions, k_cache, v_cache,
                     meta.slots, v_other=v_first, v_blend=v_blend)
    return _attend(qkv, k_cache, v_cache, meta, H, G, dim, vdim, hscale, spec.window, None, 0, out, None, spec.keep_first,
                   spec.softcap)


@dataclass
class LatentAttnSpec:
    """Latent attention: ``c_q = rms(W_dq h) w_q``, ``q = W_uq c_q`` (per head ``dim`` plain and ``rot_dim``
    rotated columns); ``W_dkv h`` = ``kv_rank`` latent columns (normed: c) and ``rot_dim`` columns of one
    rotated key segment common to the heads; per head key ``[W_uk c | common segment]``, value ``W_uv c``; sliding
    window (``window`` 0: causal); the output times ``sigmoid(W_g h)``, one gate per head or (``gate_elem``) one
    per output element.  The cache holds the expanded keys and values
    (``heads`` key / value heads): a sliding window bounds what a decoded token reads, and scores against
    the latent would cost ``kv_rank / dim`` times the products."""
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    window: int
    rot: RotarySpec = field(default_factory=RotarySpec)
    gate_elem: bool = False

    @classmethod
    def from_dict(cls, m: dict, gate_elem: bool = False, causal_ok: bool = False) -> "LatentAttnSpec":
        mask, rd = m.get("mask") or {}, int(m.get("rot_dim", 0))
        rot = dict(m.get("rot") or {})
        rot["dims"] = rd
        s = cls(int(m["heads"]), int(m["dim"]), rd, int(m.get("vdim", m["dim"])), int(m["q_rank"]), int(m["kv_rank"]),
                float(m.get("scale", (int(m["dim"]) + rd) ** -0.5)), int(mask.get("size", 0)), RotarySpec.from_dict(rot, "ramp"),
                gate_elem)
        if s.window < (0 if causal_ok else 1) or rd % 2:
            raise ValueError(f"unsupported latent attention sizes {m}")
        return s

    @property
    def gate_cols(self) -> int:
        """Columns of the gate projection: one per head, or one per (padded) output element."""
        return self.heads * self.vdim_p if self.gate_elem else self.heads

    @property
    def kdim(self) -> int:
        """Key head size in the cache (plain + rotated columns, padded to the kernels' fragments)."""
        return _pad8(self.dim + self.rot_dim)

    @property
    def vdim_p(self) -> int:
        return _pad8(self.vdim)

    def make_caches(self, num_blocks: int, block_size: int, dtype, device) -> tuple:
        return _cache_pair(num_blocks, self.heads, block_size, self.kdim, self.vdim_p, dtype, device)

    def bytes_per_token(self, dtype) -> int:
        return self.heads * (self.kdim + self.vdim_p) * torch.tensor([], dtype=dtype).element_size()


def latent_window_attention(u, rows, uv_col: int, w_uq, w_ukv, dq_norm, dkv_norm, caches, meta: AttnMeta, spec: LatentAttnSpec, freq, hscale,
                            eps: float, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """u [T, dq | dkv | g] = the fused down projections of the mixer's input (``rows``: their column layout).
    ``w_uq`` [H kdim, q_rank] (zero rows behind every head's dim + rot_dim), ``w_ukv`` = [W_uk ; W_uv] with
    the value rows starting at row ``uv_col`` (a multiple of 8)."""
    H, dim, rd, vdim = spec.heads, spec.dim, spec.rot_dim, spec.vdim
    kd, vd = spec.kdim, spec.vdim_p
    T = u.shape[0]
    if out is None:
        out = torch.empty(T, H * vd, dtype=u.dtype, device=u.device)
    cq = ops.rms_cols(u, rows.off["dq"], spec.q_rank, dq_norm, eps)
    q = ops.linear(cq, w_uq)                                            # [T, H kdim]
    c = ops.rms_cols(u, rows.off["dkv"], spec.kv_rank, dkv_norm, eps)
    kv = ops.linear(c, w_ukv)                                           # [T, H dim (padded to 8) | H vdim_p]
    k_cache, v_cache = caches[0], caches[1]
    ops.rot_kv_write(q, H, kd, kv, H, dim, u[:, rows.off["dkv"] + spec.kv_rank:], rd, kv[:, uv_col:], vd, dim, rd, freq,
                     spec.rot.magnitude, meta.positions, k_cache, v_cache, meta.slots)
    return _attend(q, k_cache, v_cache, meta, H, H, kd, vd, hscale, spec.window, u, rows.off["g"], out, None,
                   gate_elem=spec.gate_elem)

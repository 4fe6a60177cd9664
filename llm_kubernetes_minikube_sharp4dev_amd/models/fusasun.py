"""Fusasun: sliding-window attention layers with pooled blocks or latent keys, a short convolution in front
of every mixer, gated and twice-normed sublayers, experts chosen by the token id.

    x = embed[token] * embed_scale                                                     (f32 stream)
    per layer:  h = rms(x) w1;   x += rms(sigmoid(W_rg1 h + b1) * mixer(h + conv(h))) w1b
                h = rms(x) w2;   x += rms(sigmoid(W_rg2 h + b2) * experts(h, token)) w2b     (ff may be absent)
    logits = head(rms(x) w_f)                      rms(v) = v / sqrt(mean(v^2) + eps)

Mixers (``cfg.layers``, any order): ``attention`` -- ``models.window_attention.pooled_window_attention``;
``latent_attention`` -- ``models.window_attention.latent_window_attention``.  Feed-forward:
``ops.table_experts`` (each token's experts are a row of an integer table indexed by its id, equal weights).

MI355X layout decisions:
  * the stream is f32 and each sublayer costs one pass over it: gate, post-norm, residual add and the next
    sublayer's pre-norm (with its activation-dtype copy for the projections) are one kernel
    (``ops.stream_gated_norm``), which also averages a token's experts; the final norm runs only on the rows
    that feed the LM head;
  * ``h + conv(h)`` is one causal convolution whose last tap carries the identity (the +1 is folded into the
    f32 tap at load), over the state slots the recurrent designs use;
  * the gate projection and a mixer's input projections are one GEMM each; rotation, key assembly and the
    paged cache write are one kernel, the pooled keys of finished blocks a second;
  * the experts' three products run on grouped MFMA kernels over (token, choice) pairs sorted by expert on the
    device, so a step needs no host round trip and decode steps can be captured.

Checkpoint format: ``config.json`` (``FusasunConfig.from_json``) and ``model.safetensors`` with ``embed``,
``l<i>.norm1 | norm1b | norm2 | norm2b``, ``l<i>.canon1``, ``l<i>.rg1`` (+ ``.b``), ``l<i>.rg2`` (+ ``.b``),
``l<i>.mix.*``, ``l<i>.mlp.e<j>.gate | up | down``, ``l<i>.mlp.table``, ``final.norm``, ``head``; linear weights
[out, in].
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn

from .. import ops
from ..parallel.tp import SINGLE, TPGroup
from .attention import AttnMeta
from .configs import FusasunConfig, pad_vocab
from .linear_state import FusedRows, fused_mult
from .window_attention import LatentAttnSpec, PooledWindowAttnSpec, latent_window_attention, pooled_window_attention


def _p(*shape, **kw):
    return nn.Parameter(torch.zeros(*shape, **kw), requires_grad=False)


def _pad8(n: int) -> int:
    return -(-int(n) // 8) * 8


class _PooledAttention(nn.Module):
    """Weights of an ``attention`` mixer under checkpoint prefix ``mix.``."""

    def __init__(self, m: dict, W: int, e: dict, f: dict):
        super().__init__()
        t = self.true = PooledWindowAttnSpec.from_dict(m)       # the checkpoint's sizes
        s = self.spec = t.padded()                              # head sizes of the kernels (zero rows / columns)
        self.rows = FusedRows([("q", s.heads * s.dim), ("k", s.kv_heads * s.dim), ("v", s.kv_heads * s.vdim)], fused_mult(W))
        self.w_in = _p(self.rows.total, W, **e)
        self.o = _p(W, s.heads * s.vdim, **e)
        self.freq = _p(max(s.rot.dims // 2, 1), **f)
        self.hscale = _p(s.heads, **f)

    def init_constants(self):
        self.freq.copy_(self.spec.rot.freq_tensor(self.freq.device))
        self.hscale.fill_(self.spec.scale)


class _LatentAttention(nn.Module):
    """Weights of a ``latent_attention`` mixer under checkpoint prefix ``mix.``."""

    def __init__(self, m: dict, W: int, e: dict, f: dict):
        super().__init__()
        s = self.spec = LatentAttnSpec.from_dict(m)
        H = s.heads
        # down projections and the head gates in one GEMM; the two up projections of the latent in another
        self.rows = FusedRows([("dq", s.q_rank), ("dkv", s.kv_rank + s.rot_dim), ("g", H)], fused_mult(W))
        self.w_in = _p(self.rows.total, W, **e)
        self.up_rows = FusedRows([("uk", H * s.dim), ("uv", H * s.vdim_p)])
        self.w_uq = _p(H * s.kdim, s.q_rank, **e)
        self.w_ukv = _p(self.up_rows.total, s.kv_rank, **e)
        self.dq_norm, self.dkv_norm = _p(s.q_rank, **f), _p(s.kv_rank, **f)
        self.o = _p(W, H * s.vdim_p, **e)
        self.freq = _p(max(s.rot_dim // 2, 1), **f)
        self.hscale = _p(H, **f)

    def init_constants(self):
        self.freq.copy_(self.spec.rot.freq_tensor(self.freq.device))
        self.hscale.fill_(self.spec.scale)


class _TableExperts(nn.Module):
    """Weights of a table-routed feed-forward under checkpoint prefix ``mlp.``."""

    def __init__(self, mlp: dict, W: int, vocab: int, e: dict, device):
        super().__init__()
        self.experts, self.top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
        self.ff = int(mlp["expert"]["ff"])
        self.ffp = _pad8(self.ff)                               # zero gate / up rows and down columns behind ff
        if not 1 <= self.top <= self.experts:
            raise ValueError(f"top {self.top} of {self.experts} experts")
        self.gate_up = _p(self.experts, 2 * self.ffp, W, **e)
        self.down = _p(self.experts, W, self.ffp, **e)
        self.table = nn.Parameter(torch.zeros(vocab, self.top, dtype=torch.int32, device=device), requires_grad=False)


class FusasunLayer(nn.Module):
    def __init__(self, cfg: FusasunConfig, spec, dtype, device):
        super().__init__()
        W = cfg.hidden
        e = dict(dtype=dtype, device=device)
        f = dict(dtype=torch.float32, device=device)   # norms, gate biases and convolution taps stay f32
        self.type = spec.type
        self.norm1, self.norm1b = _p(W, **f), _p(W, **f)
        self.rg1, self.rg1_b = _p(W, W, **e), _p(W, **f)
        self.canon = _p(W, cfg.canon_taps, **f)        # last tap + 1: the convolution returns h + conv(h)
        self.mix = (_PooledAttention if spec.type == "attention" else _LatentAttention)(spec.mixer, W, e, f)
        self.mlp = _TableExperts(spec.mlp, W, cfg.vocab_size, e, device) if spec.mlp else None
        if self.mlp is not None:
            self.norm2, self.norm2b = _p(W, **f), _p(W, **f)
            self.rg2, self.rg2_b = _p(W, W, **e), _p(W, **f)


class FusasunModel(nn.Module):
    stateful = True            # the convolution's last inputs per sequence: no prefix reuse, chunks run as prompt portions

    def __init__(self, cfg: FusasunConfig, tp: TPGroup = SINGLE, dtype=torch.bfloat16, device="cpu"):
        super().__init__()
        if tp.enabled:
            raise NotImplementedError("the Fusasun decoder runs on one GPU (no tensor-parallel sharding)")
        self.cfg, self.tp, self.dtype, self.device = cfg, tp, dtype, torch.device(device)
        e = dict(dtype=dtype, device=device)
        f = dict(dtype=torch.float32, device=device)
        self.vocab_lo, self.vocab_local = 0, cfg.vocab_size
        self.embed = _p(cfg.vocab_size, cfg.hidden, **e)
        self.layers = nn.ModuleList([FusasunLayer(cfg, l, dtype, device) for l in cfg.layers])
        self.final_norm = _p(cfg.hidden, **f)
        # head rows padded (zero rows) so that logits rows start 32-byte aligned for the sampling kernels
        self.lm_head = _p(pad_vocab(cfg.vocab_size, 64), cfg.hidden, **e)
        specs = [L.mix.spec for L in self.layers]
        self.hq = max(s.heads for s in specs)
        self.hkv = max(getattr(s, "kv_heads", s.heads) for s in specs)
        self.D = max(max(getattr(s, "kdim", s.dim), getattr(s, "vdim_p", s.vdim)) for s in specs)

    # ------------------------------------------------------------------ weights
    def _finish(self):
        for L in self.layers:
            L.mix.init_constants()
        return self

    @torch.no_grad()
    def random_init(self, seed: int = 0):
        """Random weights of a scale that keeps every mechanism active, written through the checkpoint names
        so that padding stays zero."""
        return self.load_state_dict_native(random_state_dict(self.cfg, seed))

    @torch.no_grad()
    def load_state_dict_native(self, sd: dict):
        """Tensors named as in the checkpoint format (module docstring)."""
        cfg, W = self.cfg, self.cfg.hidden

        def get(name, *shape):
            t = sd[name]
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name}: checkpoint shape {tuple(t.shape)} != {tuple(shape)}")
            return t

        def put(p, name):
            p.copy_(get(name, *p.shape).to(p.dtype))

        def heads_in(dst, name, h, d, dp, cols):
            """[h * d, cols] checkpoint rows -> h heads of dp >= d rows each (zero rows behind d)."""
            dst.view(h, dp, cols)[:, :d].copy_(get(name, h * d, cols).view(h, d, cols).to(dst.dtype))

        put(self.embed, "embed")
        put(self.final_norm, "final.norm")
        self.lm_head.zero_()
        self.lm_head[:cfg.vocab_size].copy_(get("head", cfg.vocab_size, W).to(self.lm_head.dtype))
        for i, L in enumerate(self.layers):
            b, m = f"l{i}.", f"l{i}.mix."
            for p, n in ((L.norm1, "norm1"), (L.norm1b, "norm1b"), (L.rg1, "rg1"), (L.rg1_b, "rg1.b")):
                put(p, b + n)
            put(L.canon, b + "canon1")
            L.canon[:, -1] += 1.0
            M = L.mix
            M.w_in.zero_()
            M.o.zero_()
            if L.type == "attention":
                a, t = M.spec, M.true
                for seg, h, d, dp in (("q", a.heads, t.dim, a.dim), ("k", a.kv_heads, t.dim, a.dim), ("v", a.kv_heads, t.vdim, a.vdim)):
                    o = M.rows.off[seg]
                    heads_in(M.w_in[o:o + h * dp], m + seg, h, d, dp, W)
                M.o.view(W, a.heads, a.vdim)[:, :, :t.vdim].copy_(get(m + "o", W, a.heads * t.vdim).view(W, a.heads, t.vdim).to(M.o.dtype))
            else:
                s = M.spec
                H, qd = s.heads, s.dim + s.rot_dim
                for seg, n in (("dq", s.q_rank), ("dkv", s.kv_rank + s.rot_dim), ("g", H)):
                    o = M.rows.off[seg]
                    M.w_in[o:o + n].copy_(get(m + seg, n, W).to(M.w_in.dtype))
                M.w_uq.zero_()
                heads_in(M.w_uq, m + "uq", H, qd, s.kdim, s.q_rank)
                M.w_ukv.zero_()
                M.w_ukv[:H * s.dim].copy_(get(m + "uk", H * s.dim, s.kv_rank).to(M.w_ukv.dtype))
                o = M.up_rows.off["uv"]
                heads_in(M.w_ukv[o:o + H * s.vdim_p], m + "uv", H, s.vdim, s.vdim_p, s.kv_rank)
                put(M.dq_norm, m + "dq.norm")
                put(M.dkv_norm, m + "dkv.norm")
                M.o.view(W, H, s.vdim_p)[:, :, :s.vdim].copy_(get(m + "o", W, H * s.vdim).view(W, H, s.vdim).to(M.o.dtype))
            if L.mlp is not None:
                X = L.mlp
                X.gate_up.zero_()
                X.down.zero_()
                for j in range(X.experts):
                    p = f"{b}mlp.e{j}."
                    X.gate_up[j, :X.ff].copy_(get(p + "gate", X.ff, W).to(X.gate_up.dtype))
                    X.gate_up[j, X.ffp:X.ffp + X.ff].copy_(get(p + "up", X.ff, W).to(X.gate_up.dtype))
                    X.down[j, :, :X.ff].copy_(get(p + "down", W, X.ff).to(X.down.dtype))
                tab = get(b + "mlp.table", cfg.vocab_size, X.top)
                if int(tab.min()) < 0 or int(tab.max()) >= X.experts:
                    raise ValueError(f"{b}mlp.table names experts outside 0..{X.experts - 1}")
                X.table.copy_(tab.to(torch.int32))
                for p, n in ((L.norm2, "norm2"), (L.norm2b, "norm2b"), (L.rg2, "rg2"), (L.rg2_b, "rg2.b")):
                    put(p, b + n)
        return self._finish()

    def native_state_dict(self) -> dict:
        """The inverse of :meth:`load_state_dict_native` (tests, export)."""
        cfg, W = self.cfg, self.cfg.hidden
        sd = {"embed": self.embed, "final.norm": self.final_norm, "head": self.lm_head[:cfg.vocab_size]}

        def heads_out(src, h, d, dp, cols):
            return src.view(h, dp, cols)[:, :d].reshape(h * d, cols)

        for i, L in enumerate(self.layers):
            b, m = f"l{i}.", f"l{i}.mix."
            canon = L.canon.detach().clone()
            canon[:, -1] -= 1.0
            sd.update({b + "norm1": L.norm1, b + "norm1b": L.norm1b, b + "rg1": L.rg1, b + "rg1.b": L.rg1_b, b + "canon1": canon})
            M = L.mix
            if L.type == "attention":
                a, t = M.spec, M.true
                for seg, h, d, dp in (("q", a.heads, t.dim, a.dim), ("k", a.kv_heads, t.dim, a.dim), ("v", a.kv_heads, t.vdim, a.vdim)):
                    o = M.rows.off[seg]
                    sd[m + seg] = heads_out(M.w_in[o:o + h * dp], h, d, dp, W)
                sd[m + "o"] = M.o.view(W, a.heads, a.vdim)[:, :, :t.vdim].reshape(W, -1)
            else:
                s = M.spec
                H, qd = s.heads, s.dim + s.rot_dim
                for seg, n in (("dq", s.q_rank), ("dkv", s.kv_rank + s.rot_dim), ("g", H)):
                    o = M.rows.off[seg]
                    sd[m + seg] = M.w_in[o:o + n]
                o = M.up_rows.off["uv"]
                sd.update({m + "uq": heads_out(M.w_uq, H, qd, s.kdim, s.q_rank), m + "uk": M.w_ukv[:H * s.dim],
                           m + "uv": heads_out(M.w_ukv[o:o + H * s.vdim_p], H, s.vdim, s.vdim_p, s.kv_rank),
                           m + "dq.norm": M.dq_norm, m + "dkv.norm": M.dkv_norm,
                           m + "o": M.o.view(W, H, s.vdim_p)[:, :, :s.vdim].reshape(W, -1)})
            if L.mlp is not None:
                X = L.mlp
                for j in range(X.experts):
                    p = f"{b}mlp.e{j}."
                    sd.update({p + "gate": X.gate_up[j, :X.ff], p + "up": X.gate_up[j, X.ffp:X.ffp + X.ff], p + "down": X.down[j, :, :X.ff]})
                sd.update({b + "mlp.table": X.table, b + "norm2": L.norm2, b + "norm2b": L.norm2b, b + "rg2": L.rg2, b + "rg2.b": L.rg2_b})
        return {k: v.detach().clone().contiguous() for k, v in sd.items()}

    def decode_gemm_shapes(self):
        """(weight, swiglu) of the dense projections a decode step runs, one per distinct shape, for the
        engine's decode GEMM routing (ops.tune_decode)."""
        if self.dtype != torch.bfloat16:
            return []   # f32 activations run on the vendor library: nothing to route
        seen, out = set(), []
        for L in self.layers:
            M = L.mix
            ws = [L.rg1, M.w_in, M.o] + ([M.w_uq, M.w_ukv] if L.type == "latent_attention" else []) + ([L.rg2] if L.mlp is not None else [])
            for w in ws:
                if tuple(w.shape) not in seen:
                    seen.add(tuple(w.shape))
                    out.append((w, False))
        return [(w, sw) for w, sw in out + [(self.lm_head, False)] if w.numel() >= 1 << 20]

    # ------------------------------------------------------------------ caches
    def make_caches(self, num_blocks: int, block_size: int, num_slots: int) -> list:
        """One entry per layer: the mixer's paged caches (K, V and, with pooling, the pooled pair), then the
        convolution state ``[slots, taps - 1, W]``.  Zero-filled: a masked key or a padding column may be read
        (and multiplied by zero), never a NaN pattern left by the allocator."""
        caches = []
        W, taps = self.cfg.hidden, self.cfg.canon_taps
        for L in self.layers:
            s = L.mix.spec
            G = getattr(s, "kv_heads", s.heads)
            kd, vd = (s.kdim, s.vdim_p) if L.type == "latent_attention" else (s.dim, s.vdim)
            if not ops.sigattn_supported(s.heads, G, kd, vd, block_size, self.dtype):
                raise ValueError(f"attention kernels do not cover {s} with block size {block_size}")
            conv = torch.zeros(num_slots, max(taps - 1, 1), W, dtype=self.dtype, device=self.device)
            caches.append(s.make_caches(num_blocks, block_size, self.dtype, self.device) + (conv,))
        return caches

    def cache_block_bytes(self, block_size: int) -> int:
        return sum(L.mix.spec.bytes_per_token(self.dtype) for L in self.layers) * block_size

    def state_slot_bytes(self) -> int:
        esz = torch.tensor([], dtype=self.dtype).element_size()
        return len(self.layers) * max(self.cfg.canon_taps - 1, 1) * self.cfg.hidden * esz

    def kv_bytes_per_token(self) -> int:
        return self.cache_block_bytes(1)

    # ------------------------------------------------------------------ forward
    def _mixer(self, L: FusasunLayer, h, meta: AttnMeta, cache):
        W = self.cfg.hidden
        hc = ops.conv_silu(h, 0, W, L.canon, None, cache[-1], meta.seq_cu, meta.state_slots, meta.positions, meta.max_seq_len,
                           act=False)
        M = L.mix
        u = ops.linear(hc, M.w_in)
        if L.type == "attention":
            att = pooled_window_attention(u, cache, meta, M.spec, M.freq, M.hscale)
        else:
            att = latent_window_attention(u, M.rows, M.up_rows.off["uv"], M.w_uq, M.w_ukv, M.dq_norm, M.dkv_norm, cache, meta, M.spec, M.freq,
                                          M.hscale, self.cfg.norm_eps)
        return ops.linear(att, M.o)

    def forward(self, ids: torch.Tensor, meta: AttnMeta, caches, taps: list = None) -> torch.Tensor:
        """-> normed hidden rows [R, W] that feed the LM head (``meta.logits_idx``, or every row).
        ``taps``: a list that receives a copy of the f32 stream after every layer (debugging and tests)."""
        cfg = self.cfg
        eps = cfg.norm_eps
        x, _ = ops.embed_stream(ids, self.embed, self.dtype, cfg.embed_scale)
        h = ops.stream_rmsnorm(x, w=self.layers[0].norm1, eps=eps, out_dtype=self.dtype)
        n = len(self.layers)
        for i, L in enumerate(self.layers):
            g = ops.linear(h, L.rg1)
            y = self._mixer(L, h, meta, caches[i])
            nxt = L.norm2 if L.mlp is not None else (self.layers[i + 1].norm1 if i + 1 < n else None)
            h = ops.stream_gated_norm(x, y, g, L.rg1_b, L.norm1b, nxt, eps, self.dtype)
            if L.mlp is not None:
                X = L.mlp
                g = ops.linear(h, L.rg2)
                y = ops.table_experts(h, ids, X.table, X.gate_up, X.down, X.top)
                nxt = self.layers[i + 1].norm1 if i + 1 < n else None
                h = ops.stream_gated_norm(x, y, g, L.rg2_b, L.norm2b, nxt, eps, self.dtype, parts=X.top)
            if taps is not None:
                taps.append(x.clone())
        idx = meta.logits_idx
        if idx is None:
            idx = torch.arange(x.shape[0], dtype=torch.long, device=x.device)
        return ops.stream_rmsnorm(x, w=self.final_norm, eps=eps, idx=idx, out_dtype=self.dtype)

    def head(self, hidden):
        return ops.linear(hidden, self.lm_head)[:, : self.cfg.vocab_size]

    def logits(self, hidden, gather: bool = True, dtype=torch.float32):
        lg = self.head(hidden)
        return lg if dtype is None else lg.to(dtype)

    def greedy(self, hidden):
        return self.tp.greedy_ids(self.head(hidden), self.vocab_lo)


def random_state_dict(cfg: FusasunConfig, seed: int = 0) -> dict:
    """Random f32 tensors (int32 tables) under the checkpoint names for ``cfg`` (presets, benchmarks, tests)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg.hidden

    def rn(*shape, scale=1.0, shift=0.0):
        return torch.randn(*shape, generator=g) * scale + shift

    def lin(out, inp, gain=1.0):
        return rn(out, inp, scale=gain / math.sqrt(inp))

    sd = {"embed": rn(cfg.vocab_size, W), "final.norm": rn(W, scale=0.1, shift=1.0), "head": lin(cfg.vocab_size, W)}
    for i, l in enumerate(cfg.layers):
        b, m = f"l{i}.", f"l{i}.mix."
        sd.update({b + "norm1": rn(W, scale=0.1, shift=1.0), b + "norm1b": rn(W, scale=0.1, shift=1.0), b + "rg1": lin(W, W),
                   b + "rg1.b": rn(W, scale=0.5), b + "canon1": rn(W, cfg.canon_taps, scale=0.3)})
        if l.type == "attention":
            a = PooledWindowAttnSpec.from_dict(l.mixer)
            sd.update({m + "q": lin(a.heads * a.dim, W, 2.0), m + "k": lin(a.kv_heads * a.dim, W, 2.0), m + "v": lin(a.kv_heads * a.vdim, W),
                       m + "o": lin(W, a.heads * a.vdim)})
        else:
            s = LatentAttnSpec.from_dict(l.mixer)
            H = s.heads
            sd.update({m + "dq": lin(s.q_rank, W), m + "dq.norm": rn(s.q_rank, scale=0.1, shift=1.0),
                       m + "uq": lin(H * (s.dim + s.rot_dim), s.q_rank, 2.0), m + "dkv": lin(s.kv_rank + s.rot_dim, W, 2.0),
                       m + "dkv.norm": rn(s.kv_rank, scale=0.1, shift=1.0), m + "uk": lin(H * s.dim, s.kv_rank, 2.0),
                       m + "uv": lin(H * s.vdim, s.kv_rank), m + "g": lin(H, W), m + "o": lin(W, H * s.vdim)})
        if l.mlp:
            E, top, ff = int(l.mlp["router"]["experts"]), int(l.mlp["router"]["top"]), int(l.mlp["expert"]["ff"])
            for j in range(E):
                p = f"{b}mlp.e{j}."
                sd.update({p + "gate": lin(ff, W), p + "up": lin(ff, W), p + "down": lin(W, ff)})
            # a token's experts are distinct: the first `top` of a random permutation per row
            sd[b + "mlp.table"] = torch.rand(cfg.vocab_size, E, generator=g).argsort(1)[:, :top].to(torch.int32)
            sd.update({b + "norm2": rn(W, scale=0.1, shift=1.0), b + "norm2b": rn(W, scale=0.1, shift=1.0), b + "rg2": lin(W, W),
                       b + "rg2.b": rn(W, scale=0.5)})
    return sd

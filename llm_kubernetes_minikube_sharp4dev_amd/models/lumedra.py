"""Lumedra: parallel blocks -- a mixer and a feed-forward side by side on two norms of the same row -- over
capped-window attention, causal latent attention and lightning (decayed linear) attention, with dense or
routed-expert feed-forwards and the embedding table as LM head.

    x = embed[token]                                                                    (f32 stream)
    per layer:  x += mixer(rms(x) w1) + ff(rms(x) w2)                                   (ff may be absent)
    logits = embed . (rms(x) w_f)                      rms(v) = v / sqrt(mean(v^2) + eps)

Mixers (``cfg.layers``, any order): ``attention`` -- ``models.window_attention.capped_window_attention``;
``latent_attention`` -- ``models.window_attention.latent_window_attention`` (causal, one gate per output
element); ``lightning`` -- ``models.linear_state.lightning_mixer``.  Feed-forward: ``dense`` --
``W_down (g sigmoid(1.702 g) (u + 1))``, ``g = min(W_gate h, limit)``, ``u = clamp(W_up h, +-limit)``; ``moe`` --
``ops.router_topk`` + ``ops.routed_experts`` (+ a shared expert of the same form for every token).

MI355X layout decisions:
  * the stream is f32 and a block costs one pass over it: the sum of the block's results (mixer, dense or shared
    feed-forward, a token's weighted expert rows) and BOTH norms of the next block (one root, two weights, two
    activation-dtype copies for the projections) are one kernel (``ops.stream_parallel_norm``); the final norm runs
    only on the rows that feed the LM head;
  * a mixer's input projections are one GEMM; key / value filing (with the value blend across layers) is one
    kernel; masks, the score cap and the element gate live inside the masked attention kernels;
  * the lightning state is one f32 tensor per layer over the engine's state slots and runs on the scan kernel of
    the other linear-state mixers;
  * router logits, scores, the choice and the weights are one f32 kernel; the experts' products run on the
    grouped MFMA kernels over (token, choice) pairs sorted by expert on the device, so decode steps with experts
    can be captured.

Checkpoint format: ``config.json`` (``LumedraConfig.from_json``) and ``model.safetensors`` with ``embed``,
``l<i>.norm1 | norm2``, ``l<i>.mix.*``, ``l<i>.mlp.gate | up | down`` (dense) or ``l<i>.mlp.router``,
``l<i>.mlp.e<j>.gate | up | down``, ``l<i>.mlp.shared.gate | up | down`` (moe), ``final.norm``; linear weights
[out, in].
"""
from __future__ import annotations

import math

import torch
import torch.nn as nn

from .. import ops
from ..parallel.tp import SINGLE, TPGroup
from .attention import AttnMeta
from .configs import LumedraConfig, pad_vocab
from .linear_state import FusedRows, LightningSpec, fused_mult, lightning_mixer
from .window_attention import CappedWindowAttnSpec, LatentAttnSpec, capped_window_attention, latent_window_attention

GLU_ALPHA = 1.702      # the design's fixed slope inside the dense feed-forward's sigmoid


def _p(*shape, **kw):
    return nn.Parameter(torch.zeros(*shape, **kw), requires_grad=False)


def _pad8(n: int) -> int:
    return -(-int(n) // 8) * 8


class _CappedAttention(nn.Module):
    """Weights of an ``attention`` mixer under checkpoint prefix ``mix.``."""

    def __init__(self, m: dict, W: int, e: dict, f: dict):
        super().__init__()
        t = self.true = CappedWindowAttnSpec.from_dict(m)       # the checkpoint's sizes
        s = self.spec = t.padded()                              # head sizes of the kernels (zero rows / columns)
        self.rows = FusedRows([("q", s.heads * s.dim), ("k", s.kv_heads * s.dim), ("v", s.kv_heads * s.vdim)], fused_mult(W))
        self.w_in = _p(self.rows.total, W, **e)
        self.o = _p(W, s.heads * s.vdim, **e)
        self.hscale = _p(s.heads, **f)
        self.freq = _p(1, **f)                                  # nothing is rotated
        self.vmix = _p(1, **f)                                  # lambda of the value blend
        self.blend = 0.0                                        # its host copy, read once at load

    def init_constants(self):
        self.hscale.fill_(self.spec.scale)
        self.blend = float(self.vmix.item())


class _LatentAttention(nn.Module):
    """Weights of a ``latent_attention`` mixer under checkpoint prefix ``mix.``."""

    def __init__(self, m: dict, W: int, e: dict, f: dict):
        super().__init__()
        s = self.spec = LatentAttnSpec.from_dict(m, gate_elem=True, causal_ok=True)
        H = s.heads
        # down projections and the element gates in one GEMM; the two up projections of the latent in another
        self.rows = FusedRows([("dq", s.q_rank), ("dkv", s.kv_rank + s.rot_dim), ("g", s.gate_cols)], fused_mult(W))
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


class _Lightning(nn.Module):
    """Weights of a ``lightning`` mixer under checkpoint prefix ``mix.``."""

    def __init__(self, m: dict, W: int, e: dict, f: dict):
        super().__init__()
        s = self.spec = LightningSpec.from_dict(m)
        self.rows = s.rows(W)
        self.w_in = _p(self.rows.total, W, **e)
        self.decay = _p(s.heads, **f)
        self.norm = _p(s.heads * s.vdim, **f)
        self.o = _p(W, s.heads * s.vdim, **e)

    def init_constants(self):
        self.decay.copy_(torch.tensor(self.spec.decay, dtype=torch.float64).to(torch.float32))


class _DenseFF(nn.Module):
    """Weights of a dense feed-forward under checkpoint prefix ``mlp.``."""

    def __init__(self, mlp: dict, W: int, e: dict):
        super().__init__()
        self.ff, self.limit = int(mlp["ff"]), float(mlp["limit"])
        self.ffp = _pad8(self.ff)                               # zero gate / up rows and down columns behind ff
        self.gate_up = _p(2 * self.ffp, W, **e)
        self.down = _p(W, self.ffp, **e)


class _RoutedFF(nn.Module):
    """Weights of a mixture-of-experts feed-forward under checkpoint prefix ``mlp.``."""

    def __init__(self, mlp: dict, W: int, e: dict, f: dict):
        super().__init__()
        r = mlp["router"]
        gr = r.get("groups") or {}
        self.experts, self.top = int(r["experts"]), int(r["top"])
        self.groups, self.keep = int(gr.get("count", 1)), int(gr.get("keep", gr.get("count", 1)))
        self.scale = float(r.get("scale", 1.0))
        self.ff = int(mlp["expert"]["ff"])
        self.ffp = _pad8(self.ff)
        if self.experts % self.groups or not 1 <= self.keep <= self.groups or not 1 <= self.top <= self.experts // self.groups * self.keep:
            raise ValueError(f"router: {self.top} of {self.experts} experts in {self.keep} of {self.groups} groups")
        self.router = _p(self.experts, W, **f)                  # f32: the router's logits are 32-bit
        self.gate_up = _p(self.experts, 2 * self.ffp, W, **e)
        self.down = _p(self.experts, W, self.ffp, **e)
        sh = mlp.get("shared")
        self.sff = int(sh["ff"]) if sh else 0
        self.sffp = _pad8(self.sff)
        if self.sff:
            self.shared_gate_up = _p(2 * self.sffp, W, **e)
            self.shared_down = _p(W, self.sffp, **e)


class LumedraLayer(nn.Module):
    def __init__(self, cfg: LumedraConfig, spec, dtype, device):
        super().__init__()
        W = cfg.hidden
        e = dict(dtype=dtype, device=device)
        f = dict(dtype=torch.float32, device=device)   # norms, router and per-head constants stay f32
        self.type = spec.type
        self.norm1 = _p(W, **f)
        self.mix = {"attention": _CappedAttention, "latent_attention": _LatentAttention, "lightning": _Lightning}[spec.type](spec.mixer, W, e, f)
        self.kind = spec.mlp["kind"] if spec.mlp else None
        if self.kind is not None:
            self.norm2 = _p(W, **f)
            self.mlp = _DenseFF(spec.mlp, W, e) if self.kind == "dense" else _RoutedFF(spec.mlp, W, e, f)


class LumedraModel(nn.Module):
    stateful = True            # recurrent state per sequence: no prefix reuse, chunks run as prompt portions

    def __init__(self, cfg: LumedraConfig, tp: TPGroup = SINGLE, dtype=torch.bfloat16, device="cpu"):
        super().__init__()
        if tp.enabled:
            raise NotImplementedError("the Lumedra decoder runs on one GPU (no tensor-parallel sharding)")
        self.cfg, self.tp, self.dtype, self.device = cfg, tp, dtype, torch.device(device)
        e = dict(dtype=dtype, device=device)
        f = dict(dtype=torch.float32, device=device)
        self.vocab_lo, self.vocab_local = 0, cfg.vocab_size
        # the embedding table is the LM head: rows padded (zero rows) so that logits rows start 32-byte aligned
        self.embed = _p(pad_vocab(cfg.vocab_size, 64), cfg.hidden, **e)
        self.layers = nn.ModuleList([LumedraLayer(cfg, l, dtype, device) for l in cfg.layers])
        self.final_norm = _p(cfg.hidden, **f)
        att = [L.mix.spec for L in self.layers if L.type != "lightning"]
        self.hq = max((s.heads for s in att), default=1)
        self.hkv = max((getattr(s, "kv_heads", s.heads) for s in att), default=1)
        self.D = max((max(getattr(s, "kdim", s.dim), getattr(s, "vdim_p", s.vdim)) for s in att), default=16)
        # the first layer that blends values defines what the later ones blend in
        mixing = [L.mix.spec for L in self.layers if L.type == "attention" and L.mix.spec.v_mix]
        for s in mixing[1:]:
            if (s.kv_heads, s.vdim) != (mixing[0].kv_heads, mixing[0].vdim):
                raise ValueError("layers that blend values must share kv_heads and vdim")

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

        def glu_in(gate_up, down, prefix, ff, ffp):
            gate_up.zero_()
            down.zero_()
            gate_up[:ff].copy_(get(prefix + "gate", ff, W).to(gate_up.dtype))
            gate_up[ffp:ffp + ff].copy_(get(prefix + "up", ff, W).to(gate_up.dtype))
            down[:, :ff].copy_(get(prefix + "down", W, ff).to(down.dtype))

        self.embed.zero_()
        self.embed[:cfg.vocab_size].copy_(get("embed", cfg.vocab_size, W).to(self.embed.dtype))
        put(self.final_norm, "final.norm")
        for i, L in enumerate(self.layers):
            b, m = f"l{i}.", f"l{i}.mix."
            put(L.norm1, b + "norm1")
            M = L.mix
            M.w_in.zero_()
            M.o.zero_()
            if L.type == "attention":
                a, t = M.spec, M.true
                for seg, h, d, dp in (("q", a.heads, t.dim, a.dim), ("k", a.kv_heads, t.dim, a.dim), ("v", a.kv_heads, t.vdim, a.vdim)):
                    o = M.rows.off[seg]
                    heads_in(M.w_in[o:o + h * dp], m + seg, h, d, dp, W)
                M.o.view(W, a.heads, a.vdim)[:, :, :t.vdim].copy_(get(m + "o", W, a.heads * t.vdim).view(W, a.heads, t.vdim).to(M.o.dtype))
                M.vmix.fill_(float(get(m + "vmix").float()) if a.v_mix else 0.0)
            elif L.type == "latent_attention":
                s = M.spec
                H, qd = s.heads, s.dim + s.rot_dim
                for seg, n in (("dq", s.q_rank), ("dkv", s.kv_rank + s.rot_dim)):
                    o = M.rows.off[seg]
                    M.w_in[o:o + n].copy_(get(m + seg, n, W).to(M.w_in.dtype))
                o = M.rows.off["g"]
                heads_in(M.w_in[o:o + H * s.vdim_p], m + "g", H, s.vdim, s.vdim_p, W)
                M.w_uq.zero_()
                heads_in(M.w_uq, m + "uq", H, qd, s.kdim, s.q_rank)
                M.w_ukv.zero_()
                M.w_ukv[:H * s.dim].copy_(get(m + "uk", H * s.dim, s.kv_rank).to(M.w_ukv.dtype))
                o = M.up_rows.off["uv"]
                heads_in(M.w_ukv[o:o + H * s.vdim_p], m + "uv", H, s.vdim, s.vdim_p, s.kv_rank)
                put(M.dq_norm, m + "dq.norm")
                put(M.dkv_norm, m + "dkv.norm")
                M.o.view(W, H, s.vdim_p)[:, :, :s.vdim].copy_(get(m + "o", W, H * s.vdim).view(W, H, s.vdim).to(M.o.dtype))
            else:
                s = M.spec
                for seg, n in (("q", s.heads * s.dim), ("k", s.heads * s.dim), ("v", s.heads * s.vdim), ("g", s.heads * s.vdim)):
                    o = M.rows.off[seg]
                    M.w_in[o:o + n].copy_(get(m + seg, n, W).to(M.w_in.dtype))
                put(M.norm, m + "norm")
                put(M.o, m + "o")
            if L.kind is None:
                continue
            put(L.norm2, b + "norm2")
            X = L.mlp
            if L.kind == "dense":
                glu_in(X.gate_up, X.down, b + "mlp.", X.ff, X.ffp)
            else:
                put(X.router, b + "mlp.router")
                for j in range(X.experts):
                    glu_in(X.gate_up[j], X.down[j], f"{b}mlp.e{j}.", X.ff, X.ffp)
                if X.sff:
                    glu_in(X.shared_gate_up, X.shared_down, b + "mlp.shared.", X.sff, X.sffp)
        return self._finish()

    def native_state_dict(self) -> dict:
        """The inverse of :meth:`load_state_dict_native` (tests, export)."""
        cfg, W = self.cfg, self.cfg.hidden
        sd = {"embed": self.embed[:cfg.vocab_size], "final.norm": self.final_norm}

        def heads_out(src, h, d, dp, cols):
            return src.view(h, dp, cols)[:, :d].reshape(h * d, cols)

        def glu_out(gate_up, down, prefix, ff, ffp):
            sd.update({prefix + "gate": gate_up[:ff], prefix + "up": gate_up[ffp:ffp + ff], prefix + "down": down[:, :ff]})

        for i, L in enumerate(self.layers):
            b, m = f"l{i}.", f"l{i}.mix."
            sd[b + "norm1"] = L.norm1
            M = L.mix
            if L.type == "attention":
                a, t = M.spec, M.true
                for seg, h, d, dp in (("q", a.heads, t.dim, a.dim), ("k", a.kv_heads, t.dim, a.dim), ("v", a.kv_heads, t.vdim, a.vdim)):
                    o = M.rows.off[seg]
                    sd[m + seg] = heads_out(M.w_in[o:o + h * dp], h, d, dp, W)
                sd[m + "o"] = M.o.view(W, a.heads, a.vdim)[:, :, :t.vdim].reshape(W, -1)
                if a.v_mix:
                    sd[m + "vmix"] = M.vmix.reshape(())
            elif L.type == "latent_attention":
                s = M.spec
                H, qd = s.heads, s.dim + s.rot_dim
                for seg, n in (("dq", s.q_rank), ("dkv", s.kv_rank + s.rot_dim)):
                    o = M.rows.off[seg]
                    sd[m + seg] = M.w_in[o:o + n]
                o, ov = M.rows.off["g"], M.up_rows.off["uv"]
                sd.update({m + "g": heads_out(M.w_in[o:o + H * s.vdim_p], H, s.vdim, s.vdim_p, W),
                           m + "uq": heads_out(M.w_uq, H, qd, s.kdim, s.q_rank), m + "uk": M.w_ukv[:H * s.dim],
                           m + "uv": heads_out(M.w_ukv[ov:ov + H * s.vdim_p], H, s.vdim, s.vdim_p, s.kv_rank),
                           m + "dq.norm": M.dq_norm, m + "dkv.norm": M.dkv_norm,
                           m + "o": M.o.view(W, H, s.vdim_p)[:, :, :s.vdim].reshape(W, -1)})
            else:
                s = M.spec
                for seg, n in (("q", s.heads * s.dim), ("k", s.heads * s.dim), ("v", s.heads * s.vdim), ("g", s.heads * s.vdim)):
                    o = M.rows.off[seg]
                    sd[m + seg] = M.w_in[o:o + n]
                sd.update({m + "norm": M.norm, m + "o": M.o})
            if L.kind is None:
                continue
            sd[b + "norm2"] = L.norm2
            X = L.mlp
            if L.kind == "dense":
                glu_out(X.gate_up, X.down, b + "mlp.", X.ff, X.ffp)
            else:
                sd[b + "mlp.router"] = X.router
                for j in range(X.experts):
                    glu_out(X.gate_up[j], X.down[j], f"{b}mlp.e{j}.", X.ff, X.ffp)
                if X.sff:
                    glu_out(X.shared_gate_up, X.shared_down, b + "mlp.shared.", X.sff, X.sffp)
        return {k: v.detach().clone().contiguous() for k, v in sd.items()}

    def decode_gemm_shapes(self):
        """(weight, swiglu) of the dense projections a decode step runs, one per distinct shape, for the
        engine's decode GEMM routing (ops.tune_decode)."""
        if self.dtype != torch.bfloat16:
            return []   # f32 activations run on the vendor library: nothing to route
        seen, out = set(), []

        def add(w, sw=False):
            if (tuple(w.shape), sw) not in seen:
                seen.add((tuple(w.shape), sw))
                out.append((w, sw))

        for L in self.layers:
            M = L.mix
            for w in [M.w_in, M.o] + ([M.w_uq, M.w_ukv] if L.type == "latent_attention" else []):
                add(w)
            if L.kind == "dense":
                add(L.mlp.gate_up)
                add(L.mlp.down)
            elif L.kind == "moe" and L.mlp.sff:
                add(L.mlp.shared_gate_up, True)
                add(L.mlp.shared_down)
        add(self.embed)
        return [(w, sw) for w, sw in out if w.numel() >= 1 << 20]

    # ------------------------------------------------------------------ caches
    def make_caches(self, num_blocks: int, block_size: int, num_slots: int) -> list:
        """One entry per layer: an attention layer's paged (K, V) -- a latent layer caches the expanded keys and
        values per head -- or a lightning layer's f32 state ``[slots, heads, dim, vdim]``.  Zero-filled: a masked
        key or a padding column may be read (and multiplied by zero), never a NaN pattern left by the allocator."""
        caches = []
        for L in self.layers:
            s = L.mix.spec
            if L.type == "lightning":
                caches.append(s.make_state(num_slots, self.dtype, self.device))
                continue
            G = getattr(s, "kv_heads", s.heads)
            kd, vd = (s.kdim, s.vdim_p) if L.type == "latent_attention" else (s.dim, s.vdim)
            if not ops.sigattn_supported(s.heads, G, kd, vd, block_size, self.dtype):
                raise ValueError(f"attention kernels do not cover {s} with block size {block_size}")
            caches.append(s.make_caches(num_blocks, block_size, self.dtype, self.device))
        return caches

    def cache_block_bytes(self, block_size: int) -> int:
        return sum(L.mix.spec.bytes_per_token(self.dtype) for L in self.layers if L.type != "lightning") * block_size

    def state_slot_bytes(self) -> int:
        return sum(L.mix.spec.state_bytes(self.dtype) for L in self.layers if L.type == "lightning")

    def kv_bytes_per_token(self) -> int:
        return self.cache_block_bytes(1)

    # ------------------------------------------------------------------ forward
    def _mixer(self, L: LumedraLayer, h, meta: AttnMeta, cache, shared: dict):
        M = L.mix
        if L.type == "lightning":
            return lightning_mixer(h, M.w_in, M.rows, M.decay, M.norm, M.o, M.spec, self.cfg.norm_eps, cache, meta, self.dtype)
        u = ops.linear(h, M.w_in)
        if L.type == "attention":
            s = M.spec
            v_first, blend = None, 0.0
            if s.v_mix:
                if "v_first" in shared:
                    v_first, blend = shared["v_first"], M.blend
                else:     # the first blending layer: its own projected values are what the later ones blend in
                    vcol = M.rows.off["v"]
                    shared["v_first"] = u[:, vcol:vcol + s.kv_heads * s.vdim]
            att = capped_window_attention(u, cache, meta, s, M.hscale, M.freq, v_first, blend)
        else:
            att = latent_window_attention(u, M.rows, M.up_rows.off["uv"], M.w_uq, M.w_ukv, M.dq_norm, M.dkv_norm, cache, meta, M.spec, M.freq,
                                          M.hscale, self.cfg.norm_eps)
        return ops.linear(att, M.o)

    def _ff(self, L: LumedraLayer, h):
        """-> (dense rows [T, W] or None, expert rows [T * top, W] or None, their weights f32 [T, top] or None)."""
        X = L.mlp
        if L.kind == "dense":
            return ops.linear(ops.clamped_glu(ops.linear(h, X.gate_up), X.limit, GLU_ALPHA), X.down), None, None
        experts, weights = ops.router_topk(h, X.router, X.top, X.groups, X.keep, X.scale)
        y = ops.routed_experts(h, experts, X.gate_up, X.down)
        b = ops.linear(ops.linear_swiglu_any(h, X.shared_gate_up), X.shared_down) if X.sff else None
        return b, y, weights

    def forward(self, ids: torch.Tensor, meta: AttnMeta, caches, taps: list = None) -> torch.Tensor:
        """-> normed hidden rows [R, W] that feed the LM head (``meta.logits_idx``, or every row).
        ``taps``: a list that receives a copy of the f32 stream after every layer (debugging and tests)."""
        eps = self.cfg.norm_eps
        x, _ = ops.embed_stream(ids, self.embed, self.dtype)
        L0 = self.layers[0]
        h1, h2 = ops.stream_parallel_norm(x, None, None, None, None, L0.norm1, L0.norm2 if L0.kind else None, eps, self.dtype)
        n = len(self.layers)
        shared: dict = {}
        for i, L in enumerate(self.layers):
            a = self._mixer(L, h1, meta, caches[i], shared)
            b, y, yw = self._ff(L, h2) if L.kind else (None, None, None)
            nxt = self.layers[i + 1] if i + 1 < n else None
            w1 = nxt.norm1 if nxt is not None else None
            w2 = nxt.norm2 if nxt is not None and nxt.kind else None
            h1, h2 = ops.stream_parallel_norm(x, a, b, y, yw, w1, w2, eps, self.dtype)
            if taps is not None:
                taps.append(x.clone())
        idx = meta.logits_idx
        if idx is None:
            idx = torch.arange(x.shape[0], dtype=torch.long, device=x.device)
        return ops.stream_rmsnorm(x, w=self.final_norm, eps=eps, idx=idx, out_dtype=self.dtype)

    def head(self, hidden):
        return ops.linear(hidden, self.embed)[:, : self.cfg.vocab_size]

    def logits(self, hidden, gather: bool = True, dtype=torch.float32):
        lg = self.head(hidden)
        return lg if dtype is None else lg.to(dtype)

    def greedy(self, hidden):
        return self.tp.greedy_ids(self.head(hidden), self.vocab_lo)


def random_state_dict(cfg: LumedraConfig, seed: int = 0) -> dict:
    """Random f32 tensors under the checkpoint names for ``cfg`` (presets, benchmarks, tests)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg.hidden

    def rn(*shape, scale=1.0, shift=0.0):
        return torch.randn(*shape, generator=g) * scale + shift

    def lin(out, inp, gain=1.0):
        return rn(out, inp, scale=gain / math.sqrt(inp))

    def glu(prefix, ff):
        return {prefix + "gate": lin(ff, W), prefix + "up": lin(ff, W), prefix + "down": lin(W, ff)}

    sd = {"embed": rn(cfg.vocab_size, W), "final.norm": rn(W, scale=0.1, shift=1.0)}
    for i, l in enumerate(cfg.layers):
        b, m = f"l{i}.", f"l{i}.mix."
        sd[b + "norm1"] = rn(W, scale=0.1, shift=1.0)
        if l.type == "attention":
            a = CappedWindowAttnSpec.from_dict(l.mixer)
            sd.update({m + "q": lin(a.heads * a.dim, W, 2.0), m + "k": lin(a.kv_heads * a.dim, W, 2.0), m + "v": lin(a.kv_heads * a.vdim, W),
                       m + "o": lin(W, a.heads * a.vdim)})
            if a.v_mix:
                sd[m + "vmix"] = torch.rand((), generator=g) * 0.6 + 0.2
        elif l.type == "latent_attention":
            s = LatentAttnSpec.from_dict(l.mixer, gate_elem=True, causal_ok=True)
            H = s.heads
            sd.update({m + "dq": lin(s.q_rank, W), m + "dq.norm": rn(s.q_rank, scale=0.1, shift=1.0),
                       m + "uq": lin(H * (s.dim + s.rot_dim), s.q_rank, 2.0), m + "dkv": lin(s.kv_rank + s.rot_dim, W, 2.0),
                       m + "dkv.norm": rn(s.kv_rank, scale=0.1, shift=1.0), m + "uk": lin(H * s.dim, s.kv_rank, 2.0),
                       m + "uv": lin(H * s.vdim, s.kv_rank), m + "g": lin(H * s.vdim, W), m + "o": lin(W, H * s.vdim)})
        else:
            s = LightningSpec.from_dict(l.mixer)
            sd.update({m + "q": lin(s.heads * s.dim, W), m + "k": lin(s.heads * s.dim, W), m + "v": lin(s.heads * s.vdim, W),
                       m + "g": lin(s.heads * s.vdim, W), m + "norm": rn(s.heads * s.vdim, scale=0.1, shift=1.0),
                       m + "o": lin(W, s.heads * s.vdim)})
        if not l.mlp:
            continue
        sd[b + "norm2"] = rn(W, scale=0.1, shift=1.0)
        if l.mlp["kind"] == "dense":
            sd.update(glu(b + "mlp.", int(l.mlp["ff"])))
        else:
            E = int(l.mlp["router"]["experts"])
            sd[b + "mlp.router"] = lin(E, W, 2.0)
            for j in range(E):
                sd.update(glu(f"{b}mlp.e{j}.", int(l.mlp["expert"]["ff"])))
            if l.mlp.get("shared"):
                sd.update(glu(b + "mlp.shared.", int(l.mlp["shared"]["ff"])))
    return sd

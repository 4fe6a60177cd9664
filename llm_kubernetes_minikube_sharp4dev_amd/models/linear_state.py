"""Linear-state mixers over the engine's per-sequence state slots: retention, lightning attention (retention on
activated projections with one norm over all heads), the gated delta rule (with short causal convolutions on
q, k, v) and the generalized delta rule.  All are members of

    S_t = diag(w_t) S_(t-1) - p_t (z_t^T S_(t-1)) + k_t v_t^T,    o_t = S_t^T q_t

and share one scan kernel (``ops.delta_scan``); what differs is how the f32 operands are made from the
layer's projections.  A mixer layer owns one f32 state tensor ``[slots, H, dk, dv]`` (and, with
convolutions, their last ``taps - 1`` inputs), one row per state slot
(``engine.block_manager.StateSlotPool``); a step's sequences -- prompt portions of any length and
one-token decode rows alike -- are described by ``AttnMeta.seq_cu`` / ``state_slots``, and a sequence whose
first row sits at position 0 starts from a zero state.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch

from .. import ops


class FusedRows:
    """Row layout of several projections fused into one weight: every segment starts at a multiple of
    8 rows (16-byte aligned column blocks of the product, for any activation dtype), the total is padded
    to ``total_mult``; padding rows are zero."""

    def __init__(self, segments, total_mult: int = 8):
        self.off, self.size = {}, {}
        n = 0
        for name, rows in segments:
            self.off[name], self.size[name] = n, int(rows)
            n += -(-int(rows) // 8) * 8
        self.used = n
        self.total = -(-n // total_mult) * total_mult

    def cols(self, u, name: str, padded: bool = False):
        o, n = self.off[name], self.size[name]
        return u[:, o:o + (-(-n // 8) * 8 if padded else n)]

    def padded(self, name: str) -> int:
        return -(-self.size[name] // 8) * 8


def fused_mult(width: int) -> int:
    """Row multiple of a fused projection: the framework's GEMM kernels tile 256 output columns for prompt
    portions and 128 for decode-sized steps, and the latter need a contraction size that is a multiple of
    256; other widths run on kernels without that constraint."""
    return 256 if width % 256 == 0 else 8


@dataclass
class RetentionSpec:
    heads: int
    dim: int
    vdim: int
    decay: list = field(default_factory=list)      # one per head

    @classmethod
    def from_dict(cls, m: dict) -> "RetentionSpec":
        s = cls(int(m["heads"]), int(m["dim"]), int(m.get("vdim", m["dim"])), [float(d) for d in m["decay"]])
        if len(s.decay) != s.heads or not ops.delta_scan_supported(s.dim, s.vdim):
            raise ValueError(f"unsupported retention sizes {m}")
        return s

    def rows(self, width: int) -> FusedRows:
        return FusedRows([("q", self.heads * self.dim), ("k", self.heads * self.dim), ("v", self.heads * self.vdim),
                          ("g", self.heads * self.vdim)], fused_mult(width))

    def make_state(self, slots: int, dtype, device):
        return (torch.zeros(slots, self.heads, self.dim, self.vdim, dtype=torch.float32, device=device),)

    def state_bytes(self, dtype) -> int:
        return self.heads * self.dim * self.vdim * 4


def retention_mixer(h, w_in, rows: FusedRows, decay, w_out, spec: RetentionSpec, eps: float, state, meta, out_dtype):
    """h [T, W] -> [T, W]: q | k | v | g in one projection, the decayed scan (k scaled by dim^-1/2, f32
    state), per-head unit RMS times silu(g), output projection."""
    u = ops.linear(h, w_in)
    o = ops.delta_scan(rows.cols(u, "q"), rows.cols(u, "k"), rows.cols(u, "v"), None, None, None, state[0], meta.seq_cu,
                       meta.state_slots, meta.positions, spec.heads, spec.heads, spec.dim, spec.vdim, w_head=decay,
                       k_scale=spec.dim ** -0.5, max_len=meta.max_seq_len)
    g = ops.head_norm_gate(o, rows.cols(u, "g"), None, spec.heads, eps, ops.GATE_SILU, out_dtype)
    return ops.linear(g, w_out)


@dataclass
class LightningSpec:
    """Decayed linear attention on activated projections: q, k, v = silu of their projections, ``S <- decay_h S +
    k v^T``, ``o = S^T q`` with no other scale; the heads' outputs are RMS-normed together over the whole row
    with a weight, multiplied by ``sigmoid(W_g h)`` and projected."""
    heads: int
    dim: int
    vdim: int
    decay: list = field(default_factory=list)      # one per head

    @classmethod
    def from_dict(cls, m: dict) -> "LightningSpec":
        s = cls(int(m["heads"]), int(m["dim"]), int(m.get("vdim", m["dim"])), [float(d) for d in m["decay"]])
        if len(s.decay) != s.heads or not ops.delta_scan_supported(s.dim, s.vdim):
            raise ValueError(f"unsupported lightning sizes {m}")
        return s

    def rows(self, width: int) -> FusedRows:
        return FusedRows([("q", self.heads * self.dim), ("k", self.heads * self.dim), ("v", self.heads * self.vdim),
                          ("g", self.heads * self.vdim)], fused_mult(width))

    def make_state(self, slots: int, dtype, device):
        return (torch.zeros(slots, self.heads, self.dim, self.vdim, dtype=torch.float32, device=device),)

    def state_bytes(self, dtype) -> int:
        return self.heads * self.dim * self.vdim * 4


def lightning_mixer(h, w_in, rows: FusedRows, decay, norm_w, w_out, spec: LightningSpec, eps: float, state, meta, out_dtype):
    """h [T, W] -> [T, W]: q | k | v | g in one projection, the decayed scan on silu(q), silu(k), silu(v) (the
    activation is applied in f32 as the scan stages its operands; f32 state), one RMS norm over all heads times a
    weight times sigmoid(g), output projection."""
    u = ops.linear(h, w_in)
    o = ops.delta_scan(rows.cols(u, "q"), rows.cols(u, "k"), rows.cols(u, "v"), None, None, None, state[0], meta.seq_cu,
                       meta.state_slots, meta.positions, spec.heads, spec.heads, spec.dim, spec.vdim, w_head=decay,
                       max_len=meta.max_seq_len, act=True)
    g = ops.head_norm_gate(o, rows.cols(u, "g"), norm_w, 1, eps, ops.GATE_SIGMOID, out_dtype)
    return ops.linear(g, w_out)


@dataclass
class GeneralDeltaSpec:
    heads: int
    dim: int
    lora: int = 32          # rank of the decay's two-layer projection (a checkpoint's tensor shapes override it)

    @classmethod
    def from_dict(cls, m: dict) -> "GeneralDeltaSpec":
        s = cls(int(m["heads"]), int(m["dim"]), int(m.get("lora", 32)))
        if not ops.delta_scan_supported(s.dim, s.dim) or s.lora < 1:
            raise ValueError(f"unsupported delta-rule sizes {m}")
        return s

    @property
    def inner(self) -> int:
        return self.heads * self.dim

    def rows(self, width: int) -> FusedRows:
        n = self.inner
        return FusedRows([("r", n), ("k", n), ("v", n), ("g", n), ("a", n), ("w1", self.lora)], fused_mult(width))

    def make_state(self, slots: int, dtype, device):
        return (torch.zeros(slots, self.heads, self.dim, self.dim, dtype=torch.float32, device=device),)

    def state_bytes(self, dtype) -> int:
        return self.heads * self.dim * self.dim * 4


def general_delta_mixer(h, w_in, rows: FusedRows, w2, w0, a_b, norm_w, w_out, spec: GeneralDeltaSpec, eps: float, state, meta,
                        out_dtype):
    """h [T, W] -> [T, W]: r | k | v | g | a | w1 in one projection; decay = exp(-e^(-1/2) sigmoid(W2 tanh(w1) +
    w0)) and removal rate sigmoid(a + bias) per key channel (f32); the scan with the unit key; per-head
    unit RMS times a weight times sigmoid(g); output projection."""
    u = ops.linear(h, w_in)
    wraw = ops.linear(ops.tanh_(rows.cols(u, "w1", padded=True)), w2)
    w, p, z = ops.general_delta_prep(rows.cols(u, "k"), wraw, w0, rows.cols(u, "a"), a_b, spec.heads, spec.dim)
    o = ops.delta_scan(rows.cols(u, "r"), rows.cols(u, "k"), rows.cols(u, "v"), w, p, z, state[0], meta.seq_cu,
                       meta.state_slots, meta.positions, spec.heads, spec.heads, spec.dim, spec.dim, max_len=meta.max_seq_len)
    g = ops.head_norm_gate(o, rows.cols(u, "g"), norm_w, spec.heads, eps, ops.GATE_SIGMOID, out_dtype)
    return ops.linear(g, w_out)


@dataclass
class GatedDeltaSpec:
    heads: int
    kv_heads: int      # q / k heads (value head h reads q / k head h // (heads / kv_heads))
    dim: int
    vdim: int
    conv: int          # taps of the causal convolutions on q, k and v
    lora_a: int = 32   # ranks of the step-size and output-gate projections (a checkpoint's shapes override them)
    lora_g: int = 32

    @classmethod
    def from_dict(cls, m: dict) -> "GatedDeltaSpec":
        s = cls(int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m.get("vdim", m["dim"])),
                int(m.get("conv", 4)), int(m.get("lora_a", m.get("lora", 32))), int(m.get("lora_g", m.get("lora", 32))))
        if s.heads % s.kv_heads or not 1 <= s.conv <= 8 or not ops.delta_scan_supported(s.dim, s.vdim):
            raise ValueError(f"unsupported gated delta-rule sizes {m}")
        return s

    def rows(self, width: int) -> FusedRows:
        return FusedRows([("q", self.kv_heads * self.dim), ("k", self.kv_heads * self.dim), ("v", self.heads * self.vdim),
                          ("b", self.heads), ("a1", self.lora_a), ("g1", self.lora_g)], fused_mult(width))

    def conv_channels(self) -> int:
        """Columns the convolution runs over: the q, k and v segments with their alignment padding."""
        r = self.rows(8)
        return r.off["v"] + r.padded("v")

    def make_state(self, slots: int, dtype, device):
        """(conv state [slots, taps - 1, C] in the activation dtype, S f32 [slots, heads, dim, vdim])."""
        return (torch.zeros(slots, max(self.conv - 1, 1), self.conv_channels(), dtype=dtype, device=device),
                torch.zeros(slots, self.heads, self.dim, self.vdim, dtype=torch.float32, device=device))

    def state_bytes(self, dtype) -> int:
        esz = torch.tensor([], dtype=dtype).element_size()
        return max(self.conv - 1, 1) * self.conv_channels() * esz + self.heads * self.dim * self.vdim * 4


def gated_delta_mixer(h, w_in, rows: FusedRows, conv_w, a2, dt_bias, A_log, g2, norm_w, w_out, spec: GatedDeltaSpec, eps: float,
                      state, meta, out_dtype):
    """h [T, W] -> [T, W]: q | k | v | beta | a1 | g1 in one projection; causal conv + SiLU over q | k | v;
    unit q / k, write strength, per-channel decay in f32; the scan; per-head unit RMS times a weight times
    sigmoid(W_g2 g1); output projection.  ``state`` = (conv, S) of this layer."""
    conv_state, S = state
    u = ops.linear(h, w_in)
    C = spec.conv_channels()
    xc = ops.conv_silu(u, 0, C, conv_w, None, conv_state, meta.seq_cu, meta.state_slots, meta.positions, meta.max_seq_len)
    dt = ops.linear(rows.cols(u, "a1", padded=True), a2)
    graw = ops.linear(rows.cols(u, "g1", padded=True), g2)
    qn, kn, vb, g, p, z = ops.gated_delta_prep(rows.cols(xc, "q"), rows.cols(xc, "k"), rows.cols(xc, "v"), rows.cols(u, "b"), dt,
                                               dt_bias, A_log, spec.heads, spec.kv_heads, spec.dim, spec.vdim)
    o = ops.delta_scan(qn, kn, vb, g, p, z, S, meta.seq_cu, meta.state_slots, meta.positions, spec.heads, spec.kv_heads, spec.dim,
                       spec.vdim, max_len=meta.max_seq_len)
    y = ops.head_norm_gate(o, graw, norm_w, spec.heads, eps, ops.GATE_SIGMOID, out_dtype)
    return ops.linear(y, w_out)

// Softmax attention with a sink over a paged K/V cache, restricted by a position mask.
//
//   s(i, j)  = hscale_h * <q_i, k_j>                         for first(i) <= j <= i
//   p(i, j)  = exp(s(i, j)) / (sink + sum_j' exp(s(i, j')))  sink = 1: one more term of score 0 without a value
//   out_i    = sigmoid(gate_(i, h)) * sum_j p(i, j) v_j      (the gate is optional)
//
// first(i): 0 (causal), the start of i's chunk of `msize` positions (chunks counted from position 0 of
// the sequence), or i - msize + 1 (sliding window).  Positions are absolute, so a prompt cut into
// portions, a decode row and a whole prompt give the same sums; keys outside the mask are never read
// beyond the 32-key step that holds the first visible one.
//
// Pooled blocks (window masks, pool > 0): beside its window a query sees one more key / value per block of
// `pool` positions that the window has left behind entirely -- block b once b * pool + pool - 1 <= i - msize, i.e.
// the first max(0, i - msize + 1) / pool blocks -- in the same softmax.  The pooled keys and values live in a
// second cache pair of the same layout, entry b at the logical position b of the sequence's block table, so
// the pass over them is the pass over the window with other pointers and the bound "b < blocks seen".
//
// Kept first positions (window masks without pooling, keep > 0): positions below `keep` stay visible to every
// later query, at their true places; the ones the window has left are one more pass over the first cache pages.
// cap > 0: a score s enters the softmax as cap * tanh(s / cap).  The optional gate is one sigmoid per head or
// (gelem) one per output element.
//
// lk_normrope_kv_write prepares the operands in f32: q and k RMS-normed per head with a weight shared by
// the heads, their first `rot` dimensions rotated by the position (dimension i pairs with i + rot / 2),
// v divided by its RMS; q in place, k and v into the cache.
//
// Layouts and the wave's work are those of the sigmoid-attention kernels: K cache [blocks, G, BS, dim],
// V cache key-contiguous [blocks, G, vdim, BS]; a wave holds 16 columns (prefill: 16 consecutive queries
// of a head; decode: the query heads of a kv group) against 32-key steps,
//   S^T (keys x columns) = K . Q^T,   O^T (vdim x columns) += V^T . P^T
// with the same key permutation on both sides.  The softmax is the running-maximum form: per column a
// maximum m >= 0 when there is a sink (its score bounds the maximum from below, so exp(-m) <= 1 is its
// share of the denominator), the sum l of exp(s - m) and O^T scaled alike.  The four waves of a
// workgroup take every fourth step and are merged through LDS in wave order; decode splits the key range
// over workgroups as well and a second kernel merges the parts (m, l, O) and applies the gate.
#include "common.h"
#include "kernels.h"
#include "attn_frag.h"

namespace {

constexpr float kNegBig = -1e30f;

struct SinkParams {
  const void* q;   // rows of [H * dim] (+ anything behind them)
  long qs;
  const void* kc;
  const void* vc;
  const int* bt;
  int bt_stride;
  int H, G, dim, vdim, BS;
  const float* hscale;  // [H]
  int mkind, msize;     // 0 causal, 1 chunk, 2 window
  int sink;
  const void* gate;     // rows aligned with q; column gcol + h (null: no gate)
  long gs;
  int gcol;
  const void* pkc;      // pooled K / V caches (pool > 0)
  const void* pvc;
  int pool;
  int keep;             // window masks: positions below `keep` stay visible behind the window
  float cap;            // > 0: scores become cap * tanh(score / cap)
  int gelem;            // the gate has one column per output element (gcol + h * vdim + d) instead of one per head
};

LK_DEVICE int blocks_seen(int qpos, int msize, int pool) { return max(0, qpos - msize + 1) / pool; }

LK_DEVICE int first_key(int qpos, int mkind, int msize) {
  if (mkind == 1) return (qpos / msize) * msize;
  if (mkind == 2) return max(0, qpos - msize + 1);
  return 0;
}

template <bool EXACT>
LK_DEVICE float exp_f(float x) {
  if constexpr (EXACT) return expf(x);
  else return __expf(x);
}

// cap * tanh(s / cap); icap = 1 / cap
template <bool EXACT>
LK_DEVICE float cap_f(float s, float cap, float icap) {
  if constexpr (EXACT) return cap * tanhf(s * icap);
  else return cap * (1.f - 2.f * __builtin_amdgcn_rcpf(1.f + __expf(2.f * s * icap)));
}

// The columns of this wave against the 32-key steps step0, step0 + stride, ... of keys [k0, k1): k0 is a
// multiple of 32.  Column n = lane % 16 sits at position qpos and sees keys klo .. qpos.  m, l, o are the
// running maximum (equal in the four lane groups of a column), this lane group's share of the sum, and
// the O^T accumulators.  Key order inside a step: see attn_sigmoid.hip (lane group g holds the weights
// of the 8 consecutive keys 8g .. 8g + 7).
template <typename T, int PAD>
LK_DEVICE void sink_run(const SinkParams& p, const void* kcache, const void* vcache, const uint4_t (&qf)[PAD / (4 * El<T>::V)], int kvh,
                        const int* bt, int k0, int k1, int step0, int stride, bool cvalid, int qpos, int klo, float hs, float& m,
                        float& l, floatx4 (&o)[PAD / 16]) {
  constexpr int EV = El<T>::V, KS = PAD / (4 * EV), VT = PAD / 16;
  constexpr bool BF = sizeof(T) == 2;
  const int lane = threadIdx.x & 63, n16 = lane & 15, g = lane >> 4;
  const T* kc = reinterpret_cast<const T*>(kcache);
  const T* vc = reinterpret_cast<const T*>(vcache);
  const int krow = 8 * (n16 >> 2) + (n16 & 3);
  // bf16: the next step's K fragments are requested as soon as this step's Q.K products have consumed the
  // current ones, and this step's V fragments before the softmax arithmetic, so both fly under it
  auto load_k = [&](int kb, uint4_t (&kf)[2][KS]) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int key = min(kb + krow + 4 * t, k1 - 1);
      const T* kr = kc + (((long)bt[key / p.BS] * p.G + kvh) * p.BS + key % p.BS) * p.dim;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        const int d0 = s * 4 * EV + g * EV;
        kf[t][s] = d0 < p.dim ? ld16(kr + d0) : uint4_t{0u, 0u, 0u, 0u};
      }
    }
  };
  uint4_t kf[2][KS];
  int kb = k0 + 32 * step0;
  if (BF && kb < k1) load_k(kb, kf);
  for (; kb < k1; kb += 32 * stride) {
    if (!BF) load_k(kb, kf);
    floatx4 c[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      c[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < KS; ++s)
        if (s * 4 * EV < p.dim) c[t] = mma_qk<T>(kf[t][s], qf[s], c[t]);
    }
    const int vk = kb + 8 * g < k1 ? kb + 8 * g : ((k1 - 1) & ~7);
    const T* vrow = vc + ((long)bt[vk / p.BS] * p.G + kvh) * p.vdim * p.BS + vk % p.BS;
    uint4_t vf[BF ? VT : 1];
    if constexpr (BF) {
#pragma unroll
      for (int vt = 0; vt < VT; ++vt) {
        const int vd = vt * 16 + n16;
        vf[vt] = (vt * 16 < p.vdim && vd < p.vdim) ? ld16(vrow + (long)vd * p.BS) : uint4_t{0u, 0u, 0u, 0u};
      }
      const int kn = kb + 32 * stride;
      if (kn < k1) load_k(kn, kf);
    }
    float sc[2][4];
    bool ok[2][4];
    float mx = kNegBig;
    const float icap = p.cap > 0.f ? 1.f / p.cap : 0.f;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int key = kb + 8 * g + 4 * t + j;
        ok[t][j] = cvalid && key <= qpos && key >= klo && key < k1;
        sc[t][j] = c[t][j] * hs;
        if (p.cap > 0.f) sc[t][j] = cap_f<!BF>(sc[t][j], p.cap, icap);
        if (ok[t][j]) mx = fmaxf(mx, sc[t][j]);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float mn = fmaxf(m, mx);
    const float alpha = exp_f<!BF>(m - mn);   // m == mn == kNegBig (nothing seen yet, no sink): exp(0) on zeros
    m = mn;
    l *= alpha;
#pragma unroll
    for (int vt = 0; vt < VT; ++vt)
#pragma unroll
      for (int j = 0; j < 4; ++j) o[vt][j] *= alpha;
    float pw[2][4];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        pw[t][j] = ok[t][j] ? exp_f<!BF>(sc[t][j] - mn) : 0.f;
        l += pw[t][j];
      }
    if constexpr (BF) {
      short8 pbits;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        pbits[j] = (short)f2bf(pw[0][j]);
        pbits[4 + j] = (short)f2bf(pw[1][j]);
      }
#pragma unroll
      for (int vt = 0; vt < VT; ++vt)
        if (vt * 16 < p.vdim) o[vt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(short8, vf[vt]), pbits, o[vt], 0, 0, 0);
    } else {
#pragma unroll
      for (int vt = 0; vt < VT; ++vt) {
        if (vt * 16 < p.vdim) {
          const int vd = vt * 16 + n16;
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            floatx4 a = {0.f, 0.f, 0.f, 0.f};
            if (vd < p.vdim) a = *reinterpret_cast<const floatx4*>(vrow + (long)vd * p.BS + 4 * t);
#pragma unroll
            for (int j = 0; j < 4; ++j) o[vt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[j], pw[t][j], o[vt], 0, 0, 0);
          }
        }
      }
    }
  }
}

template <typename T, int PAD>
LK_DEVICE void load_q(const SinkParams& p, const T* qrow, bool cvalid, uint4_t (&qf)[PAD / (4 * El<T>::V)]) {
  constexpr int EV = El<T>::V, KS = PAD / (4 * EV);
  const int g = (threadIdx.x & 63) >> 4;
#pragma unroll
  for (int s = 0; s < KS; ++s) {
    const int d0 = s * 4 * EV + g * EV;
    qf[s] = (cvalid && d0 < p.dim) ? ld16(qrow + d0) : uint4_t{0u, 0u, 0u, 0u};
  }
}

// Merge of the 4 waves' (m, l, O^T) in wave order through LDS; afterwards wave 0 holds, per column, the
// maximum m, the whole sum l (all lane groups) and O^T relative to m.
template <bool EXACT, int VT>
LK_DEVICE void merge_waves(float& m, float& l, floatx4 (&o)[VT], float (&red)[3][VT][64][4], float (&ml)[3][64][2]) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (w > 0) {
    ml[w - 1][lane][0] = m;
    ml[w - 1][lane][1] = l;
#pragma unroll
    for (int vt = 0; vt < VT; ++vt)
#pragma unroll
      for (int j = 0; j < 4; ++j) red[w - 1][vt][lane][j] = o[vt][j];
  }
  __syncthreads();
  if (w == 0) {
    float M = m;
#pragma unroll
    for (int i = 0; i < 3; ++i) M = fmaxf(M, ml[i][lane][0]);
    float a0 = exp_f<EXACT>(m - M), a[3];
#pragma unroll
    for (int i = 0; i < 3; ++i) a[i] = exp_f<EXACT>(ml[i][lane][0] - M);
    l = ((l * a0 + ml[0][lane][1] * a[0]) + ml[1][lane][1] * a[1]) + ml[2][lane][1] * a[2];
#pragma unroll
    for (int vt = 0; vt < VT; ++vt)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        o[vt][j] = ((o[vt][j] * a0 + red[0][vt][lane][j] * a[0]) + red[1][vt][lane][j] * a[1]) + red[2][vt][lane][j] * a[2];
    m = M;
  }
}

// the head's gate (1 when there is none, or when the gate is per element)
template <typename T>
LK_DEVICE float gate_of(const SinkParams& p, long row, int head) {
  if (!p.gate || p.gelem) return 1.f;
  const float gv = El<T>::ld(reinterpret_cast<const T*>(p.gate) + row * p.gs + p.gcol + head);
  return 1.f / (1.f + expf(-gv));
}

// the gate of output element vd of a head (1 unless the gate is per element)
template <typename T>
LK_DEVICE float gate_el(const SinkParams& p, long row, int head, int vd) {
  if (!p.gate || !p.gelem) return 1.f;
  const float gv = El<T>::ld(reinterpret_cast<const T*>(p.gate) + row * p.gs + p.gcol + (long)head * p.vdim + vd);
  return 1.f / (1.f + expf(-gv));
}

// the positions below `keep` that lie behind the window of a query whose first visible key is klo
LK_DEVICE int kept_keys(const SinkParams& p, int klo) { return p.keep > 0 ? min(p.keep, klo) : 0; }

// ---- prefill: blockIdx.x = head, blockIdx.y walks the tile list (16 queries of one sequence each).
// WT = false: a workgroup owns one tile, its 4 waves take every fourth 32-key step and are merged (long key
// ranges: the chain of steps is what bounds the tile).  WT = true: each wave owns a tile of its own and
// walks all its steps (masks that bound a query's keys to a few steps: no merge and no barrier; the four
// tiles of a workgroup are neighbours in the cost-sorted tile list, so its waves finish together).
template <typename T, int PAD, bool WT>
__global__ __launch_bounds__(256) void sinkattn_prefill_kernel(SinkParams p, const int* __restrict__ cu_q,
                                                               const int* __restrict__ ctx_lens,
                                                               const int* __restrict__ tile_seq,
                                                               const int* __restrict__ tile_q0, int ntiles, T* __restrict__ out,
                                                               long os) {
  constexpr int VT = PAD / 16, NR = WT ? 1 : 3;
  constexpr bool EXACT = sizeof(T) == 4;
  __shared__ float red[NR][VT][64][4];
  __shared__ float ml[NR][64][2];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, n16 = lane & 15, g = lane >> 4;
  const int head = blockIdx.x;
  const int tile = WT ? blockIdx.y * 4 + w : blockIdx.y;
  if (WT && tile >= ntiles) return;   // wave-uniform; no barrier follows in this mode
  const int b = tile_seq[tile], q0 = tile_q0[tile];
  const int qbeg = cu_q[b], qlen = cu_q[b + 1] - qbeg, ctx = ctx_lens[b], past = ctx - qlen;
  const int qi = q0 + n16;
  const bool cvalid = qi < qlen;
  const int qpos = past + qi;
  const T* qrow = reinterpret_cast<const T*>(p.q) + (long)(qbeg + min(qi, qlen - 1)) * p.qs + (long)head * p.dim;
  uint4_t qf[PAD / (4 * El<T>::V)];
  load_q<T, PAD>(p, qrow, cvalid, qf);
  floatx4 o[VT];
#pragma unroll
  for (int vt = 0; vt < VT; ++vt) o[vt] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m = p.sink ? 0.f : kNegBig, l = 0.f;
  const int k1 = min(ctx, past + q0 + 16);
  const int k0 = first_key(past + q0, p.mkind, p.msize) & ~31;   // first(i) never decreases with i
  const int klo_q = first_key(qpos, p.mkind, p.msize);
  sink_run<T, PAD>(p, p.kc, p.vc, qf, head / (p.H / p.G), p.bt + (long)b * p.bt_stride, k0, k1, WT ? 0 : w, WT ? 1 : 4, cvalid, qpos, klo_q,
                   p.hscale[head], m, l, o);
  {
    // A second pass over what lies behind the window -- the pooled blocks it has left behind entirely, or (never both) the kept
    // first positions: entries [0, n1) of the pooled / the plain cache pair, bounded by the tile's last query (it sees the most
    // blocks and has the latest window) and per column by its own window.
    const bool pooled = p.pool > 0;
    const int n1 = pooled ? blocks_seen(k1 - 1, p.msize, p.pool) : kept_keys(p, first_key(k1 - 1, p.mkind, p.msize));
    const int vis = (pooled ? blocks_seen(qpos, p.msize, p.pool) : kept_keys(p, klo_q)) - 1;
    if (n1 > 0)
      sink_run<T, PAD>(p, pooled ? p.pkc : p.kc, pooled ? p.pvc : p.vc, qf, head / (p.H / p.G), p.bt + (long)b * p.bt_stride, 0, n1,
                       WT ? 0 : w, WT ? 1 : 4, cvalid, vis, 0, p.hscale[head], m, l, o);
  }
  if constexpr (WT) {
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
  } else {
    merge_waves<EXACT, VT>(m, l, o, red, ml);
  }
  if ((WT || w == 0) && cvalid) {
    const float den = l + (p.sink ? exp_f<EXACT>(-m) : 0.f);
    const float f = den > 0.f ? gate_of<T>(p, qbeg + qi, head) / den : 0.f;
    T* orow = out + (long)(qbeg + qi) * os + (long)head * p.vdim;
#pragma unroll
    for (int vt = 0; vt < VT; ++vt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int vd = vt * 16 + 4 * g + j;
        if (vd < p.vdim) El<T>::st(orow + vd, o[vt][j] * f * gate_el<T>(p, qbeg + qi, head, vd));
      }
  }
}

// ---- decode: workgroup = (sequence, up to 16 heads of one kv group, key split z) -----------------------
// part: [B, H, Z, vdim + 2] f32 = O^T relative to m, then m, l
template <typename T, int PAD>
__global__ __launch_bounds__(256) void sinkattn_decode_kernel(SinkParams p, const int* __restrict__ ctx_lens, int Z,
                                                              T* __restrict__ out, long os, float* __restrict__ part) {
  constexpr int VT = PAD / 16;
  constexpr bool EXACT = sizeof(T) == 4;
  __shared__ float red[3][VT][64][4];
  __shared__ float ml[3][64][2];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, n16 = lane & 15, g = lane >> 4;
  const int rep = p.H / p.G, ngr = (rep + 15) / 16;
  const int b = blockIdx.x, kvh = blockIdx.y / ngr, sub = blockIdx.y % ngr, z = blockIdx.z;
  const int ctx = ctx_lens[b];
  const int hn = sub * 16 + n16;
  const bool cvalid = hn < rep;
  const int head = kvh * rep + min(hn, rep - 1);
  const T* qrow = reinterpret_cast<const T*>(p.q) + (long)b * p.qs + (long)head * p.dim;
  uint4_t qf[PAD / (4 * El<T>::V)];
  load_q<T, PAD>(p, qrow, cvalid, qf);
  floatx4 o[VT];
#pragma unroll
  for (int vt = 0; vt < VT; ++vt) o[vt] = floatx4{0.f, 0.f, 0.f, 0.f};
  float m = p.sink ? 0.f : kNegBig, l = 0.f;
  const int klo = first_key(ctx - 1, p.mkind, p.msize), k0 = klo & ~31;
  // the key splits share the window's 32-key steps and, behind them, the steps over what lies behind the window: the pooled
  // blocks or (never both) the kept first positions, entries [0, n1) of the pooled / the plain cache pair
  const bool pooled = p.pool > 0;
  const int n1 = pooled ? blocks_seen(ctx - 1, p.msize, p.pool) : kept_keys(p, klo);
  const int nwin = (ctx - k0 + 31) / 32, nsteps = nwin + (n1 + 31) / 32, spz = (nsteps + Z - 1) / Z;
  const int s0 = z * spz, s1 = min(nsteps, s0 + spz);
  if (s0 < min(s1, nwin))
    sink_run<T, PAD>(p, p.kc, p.vc, qf, kvh, p.bt + (long)b * p.bt_stride, k0 + 32 * s0, min(ctx, k0 + 32 * min(s1, nwin)), w, 4, cvalid,
                     ctx - 1, klo, p.hscale[head], m, l, o);
  if (max(s0, nwin) < s1)
    sink_run<T, PAD>(p, pooled ? p.pkc : p.kc, pooled ? p.pvc : p.vc, qf, kvh, p.bt + (long)b * p.bt_stride, 32 * (max(s0, nwin) - nwin),
                     min(n1, 32 * (s1 - nwin)), w, 4, cvalid, n1 - 1, 0, p.hscale[head], m, l, o);
  merge_waves<EXACT, VT>(m, l, o, red, ml);
  if (w == 0 && cvalid) {
    if (Z == 1) {
      const float den = l + (p.sink ? exp_f<EXACT>(-m) : 0.f);
      const float f = den > 0.f ? gate_of<T>(p, b, head) / den : 0.f;
#pragma unroll
      for (int vt = 0; vt < VT; ++vt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int vd = vt * 16 + 4 * g + j;
          if (vd < p.vdim) El<T>::st(out + (long)b * os + (long)head * p.vdim + vd, o[vt][j] * f * gate_el<T>(p, b, head, vd));
        }
    } else {
      float* pp = part + (((long)b * p.H + head) * Z + z) * (p.vdim + 2);
#pragma unroll
      for (int vt = 0; vt < VT; ++vt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int vd = vt * 16 + 4 * g + j;
          if (vd < p.vdim) pp[vd] = o[vt][j];
        }
      if (g == 0) {
        pp[p.vdim] = m;
        pp[p.vdim + 1] = l;
      }
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void sinkattn_reduce_kernel(SinkParams p, const float* __restrict__ part, int Z,
                                                              T* __restrict__ out, long os) {
  constexpr bool EXACT = sizeof(T) == 4;
  const int b = blockIdx.x, head = blockIdx.y;
  const float* pp = part + ((long)b * p.H + head) * Z * (p.vdim + 2);
  float M = p.sink ? 0.f : kNegBig;
  for (int z = 0; z < Z; ++z) M = fmaxf(M, pp[(long)z * (p.vdim + 2) + p.vdim]);
  float den = p.sink ? exp_f<EXACT>(-M) : 0.f;
  for (int z = 0; z < Z; ++z) den += pp[(long)z * (p.vdim + 2) + p.vdim + 1] * exp_f<EXACT>(pp[(long)z * (p.vdim + 2) + p.vdim] - M);
  const float f = den > 0.f ? gate_of<T>(p, b, head) / den : 0.f;
  for (int vd = threadIdx.x; vd < p.vdim; vd += 256) {
    float s = 0.f;
    for (int z = 0; z < Z; ++z) s += pp[(long)z * (p.vdim + 2) + vd] * exp_f<EXACT>(pp[(long)z * (p.vdim + 2) + p.vdim] - M);
    El<T>::st(out + (long)b * os + (long)head * p.vdim + vd, s * f * gate_el<T>(p, b, head, vd));
  }
}

// ---- q / k norm + rotation, v norm, k and v into the paged cache ---------------------------------------
// One workgroup per token; its 4 waves take the H + 2G (head, kind) jobs in turn.  A head's elements are
// held in registers (own and rotation partner, up to 4 of each per lane) before anything is written, so
// the in-place q is safe.
template <typename T>
__global__ __launch_bounds__(256) void normrope_kv_write_kernel(T* __restrict__ qkv, long qs, int H, int G, int dim, int vdim,
                                                                int norm_dim, int norm_vdim, const float* __restrict__ qw,
                                                                const float* __restrict__ kw, int rot,
                                                                const float* __restrict__ inv_freq,
                                                                const int* __restrict__ positions, float eps,
                                                                T* __restrict__ kc, T* __restrict__ vc,
                                                                const int* __restrict__ slots, int BS, int v_unit) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int slot = slots[t];
  const float pos = (float)positions[t];
  T* row = qkv + t * qs;
  const long blk = slot >= 0 ? slot / BS : 0;
  const int off = slot >= 0 ? slot % BS : 0;
  const int half = rot / 2;
  for (int job = w; job < H + 2 * G; job += 4) {
    if (job < H + G) {
      const bool isq = job < H;
      const T* x = row + (long)job * dim;
      const float* wt = isq ? qw : kw;
      float own[4], par[4];
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = lane + 64 * i;
        own[i] = par[i] = 0.f;
        if (c < dim) {
          own[i] = El<T>::ld(x + c);
          ss += own[i] * own[i];
          if (c < rot) {
            const int pc = c < half ? c + half : c - half;
            par[i] = El<T>::ld(x + pc) * wt[pc];
          }
          own[i] *= wt[c];
        }
      }
      const float inv = 1.f / sqrtf(wave_sum(ss) / (float)norm_dim + eps);
      T* dst = isq ? row + (long)job * dim : (slot >= 0 ? kc + ((blk * G + (job - H)) * BS + off) * dim : nullptr);
      if (!dst) continue;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = lane + 64 * i;
        if (c < dim) {
          float y = own[i] * inv;
          if (c < rot) {
            float sn, cs;
            sincosf(pos * inv_freq[c < half ? c : c - half], &sn, &cs);
            const float pr = par[i] * inv;
            y = c < half ? y * cs - pr * sn : y * cs + pr * sn;
          }
          El<T>::st(dst + c, y);
        }
      }
    } else if (slot >= 0) {
      const int gh = job - H - G;
      const T* x = row + (long)(H + G) * dim + (long)gh * vdim;
      float own[4];
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = lane + 64 * i;
        own[i] = c < vdim ? El<T>::ld(x + c) : 0.f;
        ss += own[i] * own[i];
      }
      const float inv = v_unit ? 1.f / sqrtf(wave_sum(ss) / (float)norm_vdim + eps) : 1.f;
      T* dst = vc + (blk * G + gh) * (long)vdim * BS + off;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = lane + 64 * i;
        if (c < vdim) El<T>::st(dst + (long)c * BS, own[i] * inv);
      }
    }
  }
}

int pad_of(int dim, int vdim) {
  const int m = dim > vdim ? dim : vdim;
  return m <= 64 ? 64 : m <= 96 ? 96 : m <= 128 ? 128 : m <= 192 ? 192 : m <= 256 ? 256 : 0;
}

bool shape_ok(const SinkParams& p, int esz) {
  const int ev = 16 / esz;
  return p.H > 0 && p.G > 0 && p.H % p.G == 0 && p.dim > 0 && p.vdim > 0 && p.dim % ev == 0 && p.vdim % ev == 0 && p.BS % 16 == 0 &&
         pad_of(p.dim, p.vdim) != 0 && p.mkind >= 0 && p.mkind <= 2 && (p.mkind == 0 || p.msize >= 1) && p.pool >= 0 &&
         (p.pool == 0 || (p.mkind == 2 && p.pkc != nullptr && p.pvc != nullptr)) && p.keep >= 0 &&
         (p.keep == 0 || (p.mkind == 2 && p.pool == 0)) && p.cap >= 0.f;
}

template <typename T, int PAD>
int launch_prefill(const SinkParams& p, const int* cu_q, const int* ctx, const int* ts, const int* tq, int ntiles, void* out,
                   long os, hipStream_t st) {
  // a query that sees at most 512 keys (17 steps): one wave per tile.  Likewise when the step has (tile, head) pairs enough to
  // fill every SIMD of the chip several times with one wave each: splitting a tile's keys over a workgroup then only adds
  // the merge and leaves each wave a short chain of steps to hide its loads behind
  const bool wt = (p.mkind != 0 && p.msize <= 512) || (long)ntiles * p.H >= 2048;
  const int gy = wt ? (ntiles + 3) / 4 : ntiles;
  if (gy > 65535) return -2;
  if (wt) sinkattn_prefill_kernel<T, PAD, true><<<dim3(p.H, gy), 256, 0, st>>>(p, cu_q, ctx, ts, tq, ntiles, reinterpret_cast<T*>(out), os);
  else sinkattn_prefill_kernel<T, PAD, false><<<dim3(p.H, gy), 256, 0, st>>>(p, cu_q, ctx, ts, tq, ntiles, reinterpret_cast<T*>(out), os);
  LK_CHECK_LAUNCH();
  return 0;
}

template <typename T, int PAD>
int launch_decode(const SinkParams& p, const int* ctx, int B, int Z, void* out, long os, float* part, hipStream_t st) {
  const int rep = p.H / p.G;
  sinkattn_decode_kernel<T, PAD><<<dim3(B, p.G * ((rep + 15) / 16), Z), 256, 0, st>>>(p, ctx, Z, reinterpret_cast<T*>(out), os, part);
  LK_CHECK_LAUNCH();
  if (Z > 1) {
    sinkattn_reduce_kernel<T><<<dim3(B, p.H), 256, 0, st>>>(p, part, Z, reinterpret_cast<T*>(out), os);
    LK_CHECK_LAUNCH();
  }
  return 0;
}

#define LK_SINK_DISPATCH(FN, ...)                      \
  switch (pad_of(p.dim, p.vdim)) {                     \
    case 64: return FN<T, 64>(__VA_ARGS__);            \
    case 96: return FN<T, 96>(__VA_ARGS__);            \
    case 128: return FN<T, 128>(__VA_ARGS__);          \
    case 192: return FN<T, 192>(__VA_ARGS__);          \
    case 256: return FN<T, 256>(__VA_ARGS__);          \
    default: return -1;                                \
  }

template <typename T>
int prefill_t(const SinkParams& p, const int* cu_q, const int* ctx, const int* ts, const int* tq, int ntiles, void* out, long os,
              hipStream_t st) {
  LK_SINK_DISPATCH(launch_prefill, p, cu_q, ctx, ts, tq, ntiles, out, os, st)
}

template <typename T>
int decode_t(const SinkParams& p, const int* ctx, int B, int Z, void* out, long os, float* part, hipStream_t st) {
  LK_SINK_DISPATCH(launch_decode, p, ctx, B, Z, out, os, part, st)
}

SinkParams make_params(const void* q, long qs, const void* kc, const void* vc, const int* bt, int bt_stride, int H, int G, int dim,
                       int vdim, int BS, const float* hscale, int mkind, int msize, int sink, const void* gate, long gs, int gcol,
                       const void* pkc, const void* pvc, int pool, int keep, float cap, int gelem) {
  SinkParams p;
  p.q = q; p.qs = qs; p.kc = kc; p.vc = vc; p.bt = bt; p.bt_stride = bt_stride;
  p.H = H; p.G = G; p.dim = dim; p.vdim = vdim; p.BS = BS; p.hscale = hscale; p.mkind = mkind; p.msize = msize; p.sink = sink;
  p.gate = gate; p.gs = gs; p.gcol = gcol; p.pkc = pkc; p.pvc = pvc; p.pool = pool; p.keep = keep; p.cap = cap; p.gelem = gelem;
  return p;
}

}  // namespace

int lk_normrope_kv_write(void* qkv, long qs, long T, int H, int G, int dim, int vdim, int norm_dim, int norm_vdim, const float* qw,
                         const float* kw, int rot, const float* inv_freq, const int* positions, float eps, void* kc, void* vc,
                         const int* slots, int BS, int v_unit, int esz, hipStream_t st) {
  if (T <= 0) return 0;
  if (H < 1 || G < 1 || dim < 1 || vdim < 1 || dim > 256 || vdim > 256 || rot < 0 || rot % 2 || rot > dim || norm_dim < 1 ||
      norm_dim > dim || norm_vdim < 1 || norm_vdim > vdim || (rot > 0 && !inv_freq))
    return -1;
  if (esz == 2)
    normrope_kv_write_kernel<bf16_t><<<(unsigned)T, 256, 0, st>>>((bf16_t*)qkv, qs, H, G, dim, vdim, norm_dim, norm_vdim, qw, kw, rot,
                                                                  inv_freq, positions, eps, (bf16_t*)kc, (bf16_t*)vc, slots, BS, v_unit);
  else
    normrope_kv_write_kernel<float><<<(unsigned)T, 256, 0, st>>>((float*)qkv, qs, H, G, dim, vdim, norm_dim, norm_vdim, qw, kw, rot,
                                                                 inv_freq, positions, eps, (float*)kc, (float*)vc, slots, BS, v_unit);
  LK_CHECK_LAUNCH();
  return 0;
}

int lk_sinkattn_prefill(const void* q, long qs, const void* kc, const void* vc, const int* bt, int bt_stride, const int* cu_q,
                        const int* ctx_lens, const int* tile_seq, const int* tile_q0, int ntiles, int H, int G, int dim, int vdim,
                        int BS, const float* hscale, int mkind, int msize, int sink, const void* gate, long gs, int gcol, void* out,
                        long os, const void* pkc, const void* pvc, int pool, int keep, float cap, int gelem, int esz, hipStream_t st) {
  if (ntiles <= 0) return 0;
  const SinkParams p = make_params(q, qs, kc, vc, bt, bt_stride, H, G, dim, vdim, BS, hscale, mkind, msize, sink, gate, gs, gcol, pkc, pvc,
                                   pool, keep, cap, gelem);
  if (!shape_ok(p, esz)) return -1;
  return esz == 2 ? prefill_t<bf16_t>(p, cu_q, ctx_lens, tile_seq, tile_q0, ntiles, out, os, st)
                  : prefill_t<float>(p, cu_q, ctx_lens, tile_seq, tile_q0, ntiles, out, os, st);
}

int lk_sinkattn_decode(const void* q, long qs, const void* kc, const void* vc, const int* bt, int bt_stride, const int* ctx_lens,
                       int B, int Z, int H, int G, int dim, int vdim, int BS, const float* hscale, int mkind, int msize, int sink,
                       const void* gate, long gs, int gcol, void* out, long os, float* part, const void* pkc, const void* pvc,
                       int pool, int keep, float cap, int gelem, int esz, hipStream_t st) {
  if (B <= 0) return 0;
  const SinkParams p = make_params(q, qs, kc, vc, bt, bt_stride, H, G, dim, vdim, BS, hscale, mkind, msize, sink, gate, gs, gcol, pkc, pvc,
                                   pool, keep, cap, gelem);
  if (!shape_ok(p, esz) || Z < 1 || (Z > 1 && part == nullptr)) return -1;
  return esz == 2 ? decode_t<bf16_t>(p, ctx_lens, B, Z, out, os, part, st) : decode_t<float>(p, ctx_lens, B, Z, out, os, part, st);
}

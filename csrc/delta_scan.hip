// Linear-state recurrences with an f32 state S [dk, dv] per head and sequence:
//
//   S_t = diag(w_t) S_(t-1) - p_t (z_t^T S_(t-1)) + k_t v_t^T          o_t = S_t^T q_t
//
// w, p, z are f32 vectors over the key channels (made by the token-parallel kernels below); w may instead
// be one constant per head and the removal term may be absent (retention).  Both terms read the old
// state, so a gated delta rule  S <- g S; S <- S + k (beta (v - S^T k))^T  is w = g, p = beta k,
// z = g * k with the written value beta v.
//
// A batch is a list of sequences (prompt portions of any length, decode rows of length 1): rows
// [cu[s], cu[s+1]) belong to sequence s, whose state lives in slot slots[s] (< 0: a padding row, its
// output rows are zeroed) and starts from zero when its first row sits at position 0.
//
// Scan kernel: a workgroup owns (sequence, head, a block of state columns).  A state column is split
// over R adjacent lanes, each holding DKT of its rows in registers for the whole sequence; the two
// contractions over the rows (z^T S and q^T S) are finished with log2(R) cross-lane moves, so nothing but
// the tile staging needs a barrier.  The operands of a tile of tokens are staged in LDS as f32 (each row
// slice padded by 4 floats, so the R different 16-byte broadcasts of one read hit different banks).
#include <type_traits>

#include "common.h"
#include "kernels.h"

namespace {

template <typename T>
LK_DEVICE float ldf(const T* p);
template <>
LK_DEVICE float ldf<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <>
LK_DEVICE float ldf<float>(const float* p) { return *p; }
template <typename T>
LK_DEVICE void stf(T* p, float v);
template <>
LK_DEVICE void stf<bf16_t>(bf16_t* p, float v) { *p = f2bf(v); }
template <>
LK_DEVICE void stf<float>(float* p, float v) { *p = v; }

// silu of a staged operand: accurate exponential for f32 rows, the hardware one for bf16 rows (whose own rounding is 2^-9)
template <typename TQ>
LK_DEVICE float scan_act(float x, int act) {
  if (!act) return x;
  if constexpr (sizeof(TQ) == 4) return x / (1.f + expf(-x));
  else return x * __builtin_amdgcn_rcpf(1.f + __expf(-x));
}

struct ScanParams {
  const void* q;   // rows of Hk * dk
  const void* k;   // rows of Hk * dk
  const void* v;   // rows of H * dv
  long qs, ks, vs;
  const float* w;  // rows of H * dk, or null
  const float* p;  // rows of H * dk, or null (then z is null too)
  const float* z;
  long ws, ps, zs;
  const float* w_head;  // [H], used when w is null
  float k_scale;
  int act;       // 1: q, k and v are silu of what the rows hold (f32, applied as they are staged)
  float* state;  // [slots, H, dk, dv]
  const int* cu;
  const int* slots;
  const int* positions;
  float* o;  // rows of H * dv
  long os;
  int H, Hk, dk, dv;
};

// tokens per LDS tile: as many (16 at most, 4 at least) as keep the operands of a tile near 48 KB
template <int NOPS, int ROW>
constexpr int tile_tokens() {
  return NOPS * ROW * 4 * 16 <= 49152 ? 16 : NOPS * ROW * 4 * 8 <= 53248 ? 8 : 4;
}

// Sum over the R adjacent lanes that share a state column (R a power of two up to 16, groups aligned
// to R): data-parallel-primitive moves inside a row of 16 lanes, no LDS round trip.
template <int R>
LK_DEVICE float group_sum(float v) {
  auto dpp = [](float x, auto ctrl) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value, 0xf, 0xf, true));
  };
  if constexpr (R >= 2) v += dpp(v, std::integral_constant<int, 0xB1>{});    // quad_perm [1, 0, 3, 2]
  if constexpr (R >= 4) v += dpp(v, std::integral_constant<int, 0x4E>{});    // quad_perm [2, 3, 0, 1]
  if constexpr (R >= 8) v += dpp(v, std::integral_constant<int, 0x141>{});   // row_half_mirror: the other quad of 8
  if constexpr (R >= 16) v += dpp(v, std::integral_constant<int, 0x140>{});  // row_mirror: the other half of 16
  return v;
}

template <int DKT, int NOPS>
struct TokenOps {
  floatx4 v[NOPS][DKT / 4];
  float vj;
};

// FULL: w per channel and the removal term; !FULL: w_head, no removal.
template <typename TQ, int DKT, int R, bool FULL>
__global__ __launch_bounds__(256) void delta_scan_kernel(ScanParams a) {
  constexpr int ROW = R * (DKT + 4), NOPS = FULL ? 5 : 2, TT = tile_tokens<NOPS, ROW>();
  constexpr int OQ = 0, OK = 1, OW = 2, OP = 3, OZ = 4;
  constexpr bool PREFETCH = DKT <= 16;   // the next token's operands are read while this one is computed
  __shared__ __attribute__((aligned(16))) float ops[TT][NOPS][ROW];
  __shared__ float vs[TT][256 / R];
  const int s = blockIdx.x, h = blockIdx.y;
  constexpr int cols = 256 / R;  // state columns of this workgroup (256 threads)
  const int j0 = blockIdx.z * cols;
  const int r = threadIdx.x % R, jj = threadIdx.x / R, j = j0 + jj;
  const int row0 = a.cu[s], len = a.cu[s + 1] - row0, slot = a.slots[s];
  if (len <= 0) return;
  if (slot < 0) {
    if (r == 0 && j < a.dv)
      for (int t = 0; t < len; ++t) a.o[(long)(row0 + t) * a.os + (long)h * a.dv + j] = 0.f;
    return;
  }
  const int kh = h / (a.H / a.Hk);
  const bool live = j < a.dv;
  float* Sg = a.state + (((long)slot * a.H + h) * a.dk) * a.dv + j;
  float S[DKT];
  const bool fresh = a.positions[row0] == 0;
#pragma unroll
  for (int ii = 0; ii < DKT; ++ii) {
    const int i = r * DKT + ii;
    S[ii] = (!fresh && live && i < a.dk) ? Sg[(long)i * a.dv] : 0.f;
  }
  const float wh = FULL ? 0.f : a.w_head[h];
  const TQ* qg = reinterpret_cast<const TQ*>(a.q) + (long)kh * a.dk;
  const TQ* kg = reinterpret_cast<const TQ*>(a.k) + (long)kh * a.dk;
  const TQ* vg = reinterpret_cast<const TQ*>(a.v) + (long)h * a.dv;
  auto fetch = [&](int t, TokenOps<DKT, NOPS>& x) {
    const float* base = &ops[t][0][r * (DKT + 4)];
#pragma unroll
    for (int n = 0; n < NOPS; ++n)
#pragma unroll
      for (int c = 0; c < DKT / 4; ++c) x.v[n][c] = *reinterpret_cast<const floatx4*>(base + n * ROW + 4 * c);
    x.vj = vs[t][jj];
  };
  // The next tile's operands travel from global memory into registers while this tile is computed, and
  // into LDS once it has been consumed: the chain over the tokens never waits for a global load.
  // (Only where a column is split over 8 or more lanes, the launch for few sequences: with the chip full,
  // other waves cover the loads and the registers are worth more than the overlap.)
  constexpr bool TILE_PF = R >= 8;
  constexpr int CNT = TILE_PF ? TT * R * DKT / 256 : 1, CV = TILE_PF ? (TT * (256 / R) + 255) / 256 : 1;
  static_assert(TT * R * DKT % 256 == 0, "a tile's operands divide evenly over the 256 threads");
  float pf[CNT][NOPS], pv[CV];
  auto gload = [&](int t0) {
#pragma unroll
    for (int c = 0; c < CNT; ++c) {
      const int e = threadIdx.x + 256 * c, t = e / (R * DKT), i = e % (R * DKT);
      const long row = row0 + t0 + t;
      const bool in = i < a.dk && t0 + t < len;
      pf[c][OQ] = in ? scan_act<TQ>(ldf<TQ>(qg + row * a.qs + i), a.act) : 0.f;
      pf[c][OK] = in ? scan_act<TQ>(ldf<TQ>(kg + row * a.ks + i), a.act) * a.k_scale : 0.f;
      if constexpr (FULL) {
        pf[c][OW] = in ? a.w[row * a.ws + (long)h * a.dk + i] : 0.f;
        pf[c][OP] = in ? a.p[row * a.ps + (long)h * a.dk + i] : 0.f;
        pf[c][OZ] = in ? a.z[row * a.zs + (long)h * a.dk + i] : 0.f;
      }
    }
#pragma unroll
    for (int c = 0; c < CV; ++c) {
      const int e = threadIdx.x + 256 * c, t = e / cols, cc = e % cols;
      pv[c] = (t < TT && t0 + t < len && j0 + cc < a.dv) ? scan_act<TQ>(ldf<TQ>(vg + (long)(row0 + t0 + t) * a.vs + j0 + cc), a.act) : 0.f;
    }
  };
  if constexpr (TILE_PF) gload(0);
  for (int t0 = 0; t0 < len; t0 += TT) {
    const int nt = min(TT, len - t0);
    __syncthreads();  // the previous tile has been consumed
    if constexpr (TILE_PF) {
#pragma unroll
      for (int c = 0; c < CNT; ++c) {
        const int e = threadIdx.x + 256 * c, t = e / (R * DKT), i = e % (R * DKT), li = i + 4 * (i / DKT);
#pragma unroll
        for (int n = 0; n < NOPS; ++n) ops[t][n][li] = pf[c][n];
      }
#pragma unroll
      for (int c = 0; c < CV; ++c) {
        const int e = threadIdx.x + 256 * c, t = e / cols, cc = e % cols;
        if (t < TT) vs[t][cc] = pv[c];
      }
    } else {
      for (int e = threadIdx.x; e < nt * R * DKT; e += 256) {
        const int t = e / (R * DKT), i = e % (R * DKT), li = i + 4 * (i / DKT);
        const long row = row0 + t0 + t;
        const bool in = i < a.dk;
        ops[t][OQ][li] = in ? scan_act<TQ>(ldf<TQ>(qg + row * a.qs + i), a.act) : 0.f;
        ops[t][OK][li] = in ? scan_act<TQ>(ldf<TQ>(kg + row * a.ks + i), a.act) * a.k_scale : 0.f;
        if constexpr (FULL) {
          ops[t][OW][li] = in ? a.w[row * a.ws + (long)h * a.dk + i] : 0.f;
          ops[t][OP][li] = in ? a.p[row * a.ps + (long)h * a.dk + i] : 0.f;
          ops[t][OZ][li] = in ? a.z[row * a.zs + (long)h * a.dk + i] : 0.f;
        }
      }
      for (int e = threadIdx.x; e < nt * cols; e += 256) {
        const int t = e / cols, c = e % cols;
        vs[t][c] = j0 + c < a.dv ? scan_act<TQ>(ldf<TQ>(vg + (long)(row0 + t0 + t) * a.vs + j0 + c), a.act) : 0.f;
      }
    }
    __syncthreads();
    if constexpr (TILE_PF) {
      if (t0 + TT < len) gload(t0 + TT);
    }
    auto step = [&](const TokenOps<DKT, NOPS>& x, int t) {
      float zsum = 0.f;
      if constexpr (FULL) {
        float zp[4] = {0.f, 0.f, 0.f, 0.f};   // four partial sums: four short chains of multiply-adds
#pragma unroll
        for (int ii = 0; ii < DKT; ii += 4)
#pragma unroll
          for (int e = 0; e < 4; ++e) zp[e] += x.v[OZ][ii / 4][e] * S[ii + e];
        zsum = group_sum<R>((zp[0] + zp[1]) + (zp[2] + zp[3]));
      }
      float ap[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ii = 0; ii < DKT; ii += 4) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if constexpr (FULL) S[ii + e] = x.v[OW][ii / 4][e] * S[ii + e] - x.v[OP][ii / 4][e] * zsum + x.v[OK][ii / 4][e] * x.vj;
          else S[ii + e] = wh * S[ii + e] + x.v[OK][ii / 4][e] * x.vj;
          ap[e] += x.v[OQ][ii / 4][e] * S[ii + e];
        }
      }
      const float acc = group_sum<R>((ap[0] + ap[1]) + (ap[2] + ap[3]));
      if (r == 0 && live) a.o[(long)(row0 + t0 + t) * a.os + (long)h * a.dv + j] = acc;
    };
    if constexpr (PREFETCH) {   // two register sets in turn: the next token's operands are read under this token's arithmetic
      TokenOps<DKT, NOPS> xa, xb;
      fetch(0, xa);
      for (int t = 0; t < nt; t += 2) {
        if (t + 1 < nt) fetch(t + 1, xb);
        step(xa, t);
        if (t + 1 < nt) {
          if (t + 2 < nt) fetch(t + 2, xa);
          step(xb, t + 1);
        }
      }
    } else {
      TokenOps<DKT, NOPS> x;
      for (int t = 0; t < nt; ++t) {
        fetch(t, x);
        step(x, t);
      }
    }
  }
  if (live) {
#pragma unroll
    for (int ii = 0; ii < DKT; ++ii) {
      const int i = r * DKT + ii;
      if (i < a.dk) Sg[(long)i * a.dv] = S[ii];
    }
  }
}

template <typename TQ, int DKT, int R>
int launch_scan(const ScanParams& a, int S, bool full, hipStream_t st) {
  constexpr int threads = 256, cols = threads / R;  // state columns per workgroup
  dim3 grid((unsigned)S, (unsigned)a.H, (unsigned)((a.dv + cols - 1) / cols));
  if (full) delta_scan_kernel<TQ, DKT, R, true><<<grid, threads, 0, st>>>(a);
  else delta_scan_kernel<TQ, DKT, R, false><<<grid, threads, 0, st>>>(a);
  LK_CHECK_LAUNCH();
  return 0;
}

// A state column is split over 4 lanes when (sequence, head) pairs alone fill the chip, over 16 when they
// do not: the recurrence is a chain over the tokens, so with few sequences the time of a step is the work
// of one lane per token, and more lanes per column shorten exactly that.
template <typename TQ>
int scan_t(const ScanParams& a, int S, bool full, int wide, hipStream_t st) {
  if (a.dk <= 16) return wide ? launch_scan<TQ, 4, 4>(a, S, full, st) : launch_scan<TQ, 16, 1>(a, S, full, st);
  if (a.dk <= 32) return wide ? launch_scan<TQ, 4, 8>(a, S, full, st) : launch_scan<TQ, 16, 2>(a, S, full, st);
  if (a.dk <= 64) return wide ? launch_scan<TQ, 4, 16>(a, S, full, st) : launch_scan<TQ, 16, 4>(a, S, full, st);
  if (a.dk <= 128) return wide ? launch_scan<TQ, 8, 16>(a, S, full, st) : launch_scan<TQ, 32, 4>(a, S, full, st);
  if (a.dk <= 256) return wide ? launch_scan<TQ, 16, 16>(a, S, full, st) : launch_scan<TQ, 64, 4>(a, S, full, st);
  return -1;
}

LK_DEVICE float sigmoid_f(float x) { return 1.f / (1.f + expf(-x)); }
LK_DEVICE float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// One workgroup per token, its waves take the jobs in turn: job < Hk: the unit query of q/k head job
// (times dk^-1/2); job < 2 Hk: the unit key; else value head h = job - 2 Hk: g, p = beta kn, z = g kn over
// its key channels (the key's norm recomputed: dk values) and vb = beta v.
template <typename T>
__global__ __launch_bounds__(256) void gated_delta_prep_kernel(const T* __restrict__ q, long qs, const T* __restrict__ k, long ks,
                                                               const T* __restrict__ v, long vs, const T* __restrict__ beta,
                                                               long bs, const T* __restrict__ dt, long dts,
                                                               const float* __restrict__ dt_bias, const float* __restrict__ A_log,
                                                               int H, int Hk, int dk, int dv, float* __restrict__ qn,
                                                               float* __restrict__ kn, float* __restrict__ vb,
                                                               float* __restrict__ g, float* __restrict__ p, float* __restrict__ z) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, rep = H / Hk;
  for (int job = wv; job < 2 * Hk + H; job += 4) {
    if (job < 2 * Hk) {
      const bool isq = job < Hk;
      const int kh = isq ? job : job - Hk;
      const T* x = (isq ? q + t * qs : k + t * ks) + (long)kh * dk;
      float ss = 0.f;
      for (int c = lane; c < dk; c += 64) {
        const float e = ldf<T>(x + c);
        ss += e * e;
      }
      const float inv = (1.f / sqrtf(wave_sum(ss) + 1e-6f)) * (isq ? 1.f / sqrtf((float)dk) : 1.f);
      float* dst = (isq ? qn : kn) + t * (long)Hk * dk + (long)kh * dk;
      for (int c = lane; c < dk; c += 64) dst[c] = ldf<T>(x + c) * inv;
    } else {
      const int h = job - 2 * Hk, kh = h / rep;
      const T* x = k + t * ks + (long)kh * dk;
      float ss = 0.f;
      for (int c = lane; c < dk; c += 64) {
        const float e = ldf<T>(x + c);
        ss += e * e;
      }
      const float inv = 1.f / sqrtf(wave_sum(ss) + 1e-6f);
      const float b = sigmoid_f(ldf<T>(beta + t * bs + h));
      const float rate = expf(A_log[h]);
      const long o = t * (long)H * dk + (long)h * dk;
      for (int c = lane; c < dk; c += 64) {
        const float kc = ldf<T>(x + c) * inv;
        const float gg = expf(-rate * softplus_f(ldf<T>(dt + t * dts + (long)h * dk + c) + dt_bias[(long)h * dk + c]));
        g[o + c] = gg;
        p[o + c] = b * kc;
        z[o + c] = gg * kc;
      }
      for (int c = lane; c < dv; c += 64) vb[t * (long)H * dv + (long)h * dv + c] = b * ldf<T>(v + t * vs + (long)h * dv + c);
    }
  }
}

// One workgroup per token, a wave per head in turn: u = unit key; w = exp(-e^(-1/2) sigmoid(wraw + w0)),
// p = sigmoid(araw + a_b) u, z = u.
template <typename T>
__global__ __launch_bounds__(256) void general_delta_prep_kernel(const T* __restrict__ k, long ks, const T* __restrict__ wraw,
                                                                 long wrs, const float* __restrict__ w0,
                                                                 const T* __restrict__ araw, long ars,
                                                                 const float* __restrict__ a_b, int H, int dk,
                                                                 float* __restrict__ w, float* __restrict__ p,
                                                                 float* __restrict__ z) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  for (int h = wv; h < H; h += 4) {
    const T* x = k + t * ks + (long)h * dk;
    float ss = 0.f;
    for (int c = lane; c < dk; c += 64) {
      const float e = ldf<T>(x + c);
      ss += e * e;
    }
    const float inv = 1.f / sqrtf(wave_sum(ss) + 1e-6f);
    const long o = t * (long)H * dk + (long)h * dk;
    for (int c = lane; c < dk; c += 64) {
      const long hc = (long)h * dk + c;
      const float u = ldf<T>(x + c) * inv;
      w[o + c] = expf(-0.6065306597126334f * sigmoid_f(ldf<T>(wraw + t * wrs + hc) + w0[hc]));
      p[o + c] = sigmoid_f(ldf<T>(araw + t * ars + hc) + a_b[hc]) * u;
      z[o + c] = u;
    }
  }
}

// One workgroup per token, a wave per head in turn: out = o / rms(o) * w * gate(g), gate = silu (0) or sigmoid (1)
template <typename TG, typename TO>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, long os, const TG* __restrict__ g, long gs,
                                                             const float* __restrict__ w, int H, int dv, float eps, int kind,
                                                             TO* __restrict__ out, long outs) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  for (int h = wv; h < H; h += 4) {
    const float* x = o + t * os + (long)h * dv;
    float ss = 0.f;
    for (int c = lane; c < dv; c += 64) ss += x[c] * x[c];
    const float inv = 1.f / sqrtf(wave_sum(ss) / (float)dv + eps);
    for (int c = lane; c < dv; c += 64) {
      const long hc = (long)h * dv + c;
      const float gv = ldf<TG>(g + t * gs + hc);
      const float s = sigmoid_f(gv);
      stf<TO>(out + t * outs + hc, x[c] * inv * (w ? w[hc] : 1.f) * (kind == 0 ? gv * s : s));
    }
  }
}

// The same for fewer heads than waves (one norm over a long row): the whole workgroup takes each head in turn
template <typename TG, typename TO>
__global__ __launch_bounds__(256) void row_norm_gate_kernel(const float* __restrict__ o, long os, const TG* __restrict__ g, long gs,
                                                            const float* __restrict__ w, int H, int dv, float eps, int kind,
                                                            TO* __restrict__ out, long outs) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  for (int h = 0; h < H; ++h) {
    const float* x = o + t * os + (long)h * dv;
    float ss = 0.f;
    for (int c = threadIdx.x; c < dv; c += 256) ss += x[c] * x[c];
    const float inv = 1.f / sqrtf(block_sum<4>(ss, red) / (float)dv + eps);
    for (int c = threadIdx.x; c < dv; c += 256) {
      const long hc = (long)h * dv + c;
      const float gv = ldf<TG>(g + t * gs + hc);
      const float s = sigmoid_f(gv);
      stf<TO>(out + t * outs + hc, x[c] * inv * (w ? w[hc] : 1.f) * (kind == 0 ? gv * s : s));
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void tanh_kernel(T* __restrict__ x, long xs, int n) {
  const long t = blockIdx.x;
  for (int c = threadIdx.x; c < n; c += 256) stf<T>(x + t * xs + c, tanhf(ldf<T>(x + t * xs + c)));
}

}  // namespace

int lk_delta_scan(const void* q, long qs, const void* k, long ks, const void* v, long vs, int qkv_esz, const float* w, long ws,
                  const float* p, long ps, const float* z, long zs, const float* w_head, float k_scale, float* state,
                  const int* cu, const int* slots, const int* positions, int S, int H, int Hk, int dk, int dv, float* o, long os,
                  int wide, int act, hipStream_t st) {
  if (S <= 0) return 0;
  if (H < 1 || Hk < 1 || H % Hk || dk < 1 || dk > 256 || dv < 1 || H > 65535) return -1;
  const bool full = w != nullptr;
  if (full ? (p == nullptr || z == nullptr) : (w_head == nullptr || p != nullptr || z != nullptr)) return -1;
  ScanParams a;
  a.q = q; a.k = k; a.v = v; a.qs = qs; a.ks = ks; a.vs = vs;
  a.w = w; a.p = p; a.z = z; a.ws = ws; a.ps = ps; a.zs = zs; a.w_head = w_head; a.k_scale = k_scale; a.act = act;
  a.state = state; a.cu = cu; a.slots = slots; a.positions = positions; a.o = o; a.os = os;
  a.H = H; a.Hk = Hk; a.dk = dk; a.dv = dv;
  return qkv_esz == 2 ? scan_t<bf16_t>(a, S, full, wide, st) : scan_t<float>(a, S, full, wide, st);
}

int lk_gated_delta_prep(const void* q, long qs, const void* k, long ks, const void* v, long vs, const void* beta, long bs,
                        const void* dt, long dts, const float* dt_bias, const float* A_log, long T, int H, int Hk, int dk, int dv,
                        float* qn, float* kn, float* vb, float* g, float* p, float* z, int esz, hipStream_t st) {
  if (T <= 0) return 0;
  if (H < 1 || Hk < 1 || H % Hk) return -1;
  if (esz == 2)
    gated_delta_prep_kernel<bf16_t><<<(unsigned)T, 256, 0, st>>>((const bf16_t*)q, qs, (const bf16_t*)k, ks, (const bf16_t*)v, vs,
                                                                 (const bf16_t*)beta, bs, (const bf16_t*)dt, dts, dt_bias, A_log, H, Hk,
                                                                 dk, dv, qn, kn, vb, g, p, z);
  else
    gated_delta_prep_kernel<float><<<(unsigned)T, 256, 0, st>>>((const float*)q, qs, (const float*)k, ks, (const float*)v, vs,
                                                                (const float*)beta, bs, (const float*)dt, dts, dt_bias, A_log, H, Hk, dk,
                                                                dv, qn, kn, vb, g, p, z);
  LK_CHECK_LAUNCH();
  return 0;
}

int lk_general_delta_prep(const void* k, long ks, const void* wraw, long wrs, const float* w0, const void* araw, long ars,
                          const float* a_b, long T, int H, int dk, float* w, float* p, float* z, int esz, hipStream_t st) {
  if (T <= 0) return 0;
  if (esz == 2)
    general_delta_prep_kernel<bf16_t><<<(unsigned)T, 256, 0, st>>>((const bf16_t*)k, ks, (const bf16_t*)wraw, wrs, w0,
                                                                   (const bf16_t*)araw, ars, a_b, H, dk, w, p, z);
  else
    general_delta_prep_kernel<float><<<(unsigned)T, 256, 0, st>>>((const float*)k, ks, (const float*)wraw, wrs, w0, (const float*)araw,
                                                                  ars, a_b, H, dk, w, p, z);
  LK_CHECK_LAUNCH();
  return 0;
}

int lk_head_norm_gate(const float* o, long os, const void* g, long gs, int g_esz, const float* w, long T, int H, int dv, float eps,
                      int kind, void* out, long outs, int out_esz, hipStream_t st) {
  if (T <= 0) return 0;
  if (kind != 0 && kind != 1) return -1;
#define LK_HNG(TG, TO)                                                                                                          \
  if (H < 4 && dv >= 256)                                                                                                       \
    row_norm_gate_kernel<TG, TO><<<(unsigned)T, 256, 0, st>>>(o, os, (const TG*)g, gs, w, H, dv, eps, kind, (TO*)out, outs);   \
  else                                                                                                                          \
    head_norm_gate_kernel<TG, TO><<<(unsigned)T, 256, 0, st>>>(o, os, (const TG*)g, gs, w, H, dv, eps, kind, (TO*)out, outs)
  if (g_esz == 2 && out_esz == 2) LK_HNG(bf16_t, bf16_t);
  else if (g_esz == 4 && out_esz == 4) LK_HNG(float, float);
  else if (g_esz == 2) LK_HNG(bf16_t, float);
  else LK_HNG(float, bf16_t);
#undef LK_HNG
  LK_CHECK_LAUNCH();
  return 0;
}

int lk_tanh_(void* x, long xs, long T, int n, int esz, hipStream_t st) {
  if (T <= 0 || n <= 0) return 0;
  if (esz == 2) tanh_kernel<bf16_t><<<(unsigned)T, 256, 0, st>>>((bf16_t*)x, xs, n);
  else tanh_kernel<float><<<(unsigned)T, 256, 0, st>>>((float*)x, xs, n);
  LK_CHECK_LAUNCH();
  return 0;
}

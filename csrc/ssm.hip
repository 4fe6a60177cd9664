// Mamba-2 style selective state-space mixer, token-parallel where it can be and sequential only
// along the recurrence:
//
//   u_t  = [z | x B C | dt]                       the input projection's row (bf16 or f32)
//   xBC  = silu(causal_conv(x B C) + b)           per channel, `taps` wide (act = 0: without the SiLU), the last column is the
//                                                 current token's; the taps - 1 inputs before a chunk
//                                                 come from the sequence's conv state
//   dt   = softplus(dt + dt_bias)                 f32, no clamp
//   S_t  = exp(-exp(A_log) dt) S_{t-1} + dt B_t x_t^T      S: [N, P] per head, f32, carried per sequence
//   y_t  = S_t^T C_t + D x_t                      f32
//   out  = groupRMS(y * silu(z)) * w              the gate comes before the norm
//
// A batch is a list of sequences (prefill chunks of any length, decode rows of length 1): rows
// [cu[s], cu[s+1]) belong to sequence s, whose state lives in slot slots[s] (< 0: a padding row,
// skipped) and starts from zero when its first row sits at position 0.
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

constexpr int kMaxTaps = 8;
constexpr int kConvRows = 16;  // tokens per workgroup of the convolution

template <bool EXACT>
LK_DEVICE float silu_f(float x) {
  if constexpr (EXACT) return x / (1.f + expf(-x));
  else return x * __builtin_amdgcn_rcpf(1.f + __expf(-x));
}

// grid (sequence, token tile, channel block): out[row][c] = silu(sum_k w[c][k] in(i - (taps-1) + k) + b[c])
template <typename T>
__global__ __launch_bounds__(256) void conv_silu_kernel(const T* __restrict__ u, long us, int C, int taps,
                                                        const float* __restrict__ w, const float* __restrict__ bias,
                                                        const T* __restrict__ state, const int* __restrict__ cu,
                                                        const int* __restrict__ slots,
                                                        const int* __restrict__ positions, T* __restrict__ out,
                                                        long os, int act) {
  const int s = blockIdx.x, c = blockIdx.z * 256 + threadIdx.x;
  const int row0 = cu[s], len = cu[s + 1] - row0, slot = slots[s];
  const int i0 = blockIdx.y * kConvRows;
  if (c >= C || i0 >= len) return;
  if (slot < 0) {
    for (int i = i0; i < min(len, i0 + kConvRows); ++i) stf<T>(out + (long)(row0 + i) * os + c, 0.f);
    return;
  }
  const bool past = positions[row0] > 0;
  const T* st = state + (long)slot * (taps - 1) * C + c;
  float wk[kMaxTaps];
#pragma unroll
  for (int k = 0; k < kMaxTaps; ++k) wk[k] = k < taps ? w[(long)c * taps + k] : 0.f;
  const float b = bias ? bias[c] : 0.f;
  for (int i = i0; i < min(len, i0 + kConvRows); ++i) {
    float acc = b;
#pragma unroll
    for (int k = 0; k < kMaxTaps; ++k) {
      if (k < taps) {
        const int idx = i - (taps - 1) + k;
        float v = 0.f;
        if (idx >= 0) v = ldf<T>(u + (long)(row0 + idx) * us + c);
        else if (past) v = ldf<T>(st + (long)(taps - 1 + idx) * C);
        acc += wk[k] * v;
      }
    }
    stf<T>(out + (long)(row0 + i) * os + c, act ? silu_f<sizeof(T) == 4>(acc) : acc);
  }
}

// The same for taps <= 4 with 16-byte accesses: a thread owns EV adjacent channels and walks its `rows`
// tokens with the three previous inputs in registers (weights right-aligned in a 4-tap window, the
// unused leading taps zero), so every input row is read once per tile instead of once per tap.
// Needs C % EV == 0 and 16-byte aligned rows of u, out and the state.
template <typename T>
__global__ __launch_bounds__(256) void conv_silu_vec_kernel(const T* __restrict__ u, long us, int C, int taps,
                                                            const float* __restrict__ w, const float* __restrict__ bias,
                                                            const T* __restrict__ state, const int* __restrict__ cu,
                                                            const int* __restrict__ slots,
                                                            const int* __restrict__ positions, T* __restrict__ out,
                                                            long os, int act, int rows) {
  constexpr int EV = 16 / sizeof(T);
  const int s = blockIdx.x, c0 = (blockIdx.z * 256 + threadIdx.x) * EV;
  const int row0 = cu[s], len = cu[s + 1] - row0, slot = slots[s];
  const int i0 = blockIdx.y * rows;
  if (c0 >= C || i0 >= len) return;
  const int i1 = min(len, i0 + rows);
  auto ldrow = [&](const T* p, float (&f)[EV]) {
    if constexpr (sizeof(T) == 2) {
      load8(p, f);
    } else {
      const floatx4 v = *reinterpret_cast<const floatx4*>(p);
#pragma unroll
      for (int e = 0; e < EV; ++e) f[e] = v[e];
    }
  };
  auto strow = [&](T* p, const float (&f)[EV]) {
    if constexpr (sizeof(T) == 2) {
      store8(p, f);
    } else {
      *reinterpret_cast<floatx4*>(p) = floatx4{f[0], f[1], f[2], f[3]};
    }
  };
  if (slot < 0) {
    float z[EV];
#pragma unroll
    for (int e = 0; e < EV; ++e) z[e] = 0.f;
    for (int i = i0; i < i1; ++i) strow(out + (long)(row0 + i) * os + c0, z);
    return;
  }
  const bool past = positions[row0] > 0;
  float wk[4][EV], b[EV], win[3][EV];
#pragma unroll
  for (int e = 0; e < EV; ++e) {
    b[e] = bias ? bias[c0 + e] : 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k) wk[k][e] = k >= 4 - taps ? w[(long)(c0 + e) * taps + (k - (4 - taps))] : 0.f;
  }
#pragma unroll
  for (int d = 3; d >= 1; --d) {  // win[3 - d] = the input d tokens before the tile's first
    const int idx = i0 - d, si = taps - 1 + idx;
#pragma unroll
    for (int e = 0; e < EV; ++e) win[3 - d][e] = 0.f;
    if (d <= taps - 1) {
      if (idx >= 0) ldrow(u + (long)(row0 + idx) * us + c0, win[3 - d]);
      else if (past && si >= 0) ldrow(state + ((long)slot * (taps - 1) + si) * C + c0, win[3 - d]);
    }
  }
  for (int i = i0; i < i1; ++i) {
    float cur[EV], r[EV];
    ldrow(u + (long)(row0 + i) * us + c0, cur);
#pragma unroll
    for (int e = 0; e < EV; ++e) {
      const float acc = b[e] + wk[0][e] * win[0][e] + wk[1][e] * win[1][e] + wk[2][e] * win[2][e] + wk[3][e] * cur[e];
      r[e] = act ? silu_f<sizeof(T) == 4>(acc) : acc;
      win[0][e] = win[1][e];
      win[1][e] = win[2][e];
      win[2][e] = cur[e];
    }
    strow(out + (long)(row0 + i) * os + c0, r);
  }
}

// grid (sequence, channel block): the sequence's last taps - 1 inputs become its conv state.
// Runs after conv_silu_kernel (which reads the old state).
template <typename T>
__global__ __launch_bounds__(256) void conv_state_kernel(const T* __restrict__ u, long us, int C, int taps,
                                                         T* __restrict__ state, const int* __restrict__ cu,
                                                         const int* __restrict__ slots,
                                                         const int* __restrict__ positions) {
  const int s = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  const int row0 = cu[s], len = cu[s + 1] - row0, slot = slots[s];
  if (c >= C || slot < 0 || len <= 0) return;
  const bool past = positions[row0] > 0;
  T* st = state + (long)slot * (taps - 1) * C + c;
  T keep[kMaxTaps];
#pragma unroll
  for (int i = 0; i < kMaxTaps; ++i) {
    if (i < taps - 1) {
      const int idx = len - (taps - 1) + i;
      T v;
      stf<T>(&v, 0.f);
      if (idx >= 0) v = u[(long)(row0 + idx) * us + c];
      else if (past) v = st[(long)(i + len) * C];
      keep[i] = v;
    }
  }
#pragma unroll
  for (int i = 0; i < kMaxTaps; ++i)
    if (i < taps - 1) st[(long)i * C] = keep[i];
}

// Sequential scan.  grid (sequence, head, P / 16): 256 threads = 16 state columns p x 16 slices of
// the N state rows (thread holds rows ns * NR .. ns * NR + NR - 1), so y_t[p] is a 16-lane butterfly.
// Tokens are taken in tiles of kScanTile: the tile's B, C (as f32), x, softplus(dt) and the decay are
// staged in LDS with coalesced loads (16-byte ones when the row layout allows), so the recurrence
// itself runs on LDS reads only -- per-token global loads of a few bytes per lane made the first
// version address-unit bound (18 tiny loads per lane and token).
constexpr int kScanTile = 16;

template <typename T, int NR>
__global__ __launch_bounds__(256) void ssm_scan_kernel(const T* __restrict__ xbc, long xs, const T* __restrict__ dtp,
                                                       long dts, int heads, int P, int N, int groups,
                                                       const float* __restrict__ dt_bias,
                                                       const float* __restrict__ A_log, const float* __restrict__ Dp,
                                                       float* __restrict__ state, const int* __restrict__ cu,
                                                       const int* __restrict__ slots,
                                                       const int* __restrict__ positions, float* __restrict__ y,
                                                       long ys) {
  constexpr int NP = NR * 16;  // padded state rows
  constexpr int EV = 16 / sizeof(T);
  __shared__ __attribute__((aligned(16))) float sB[kScanTile][NP];
  __shared__ __attribute__((aligned(16))) float sC[kScanTile][NP];
  __shared__ float sx[kScanTile][16], sy[kScanTile][16], sdt[kScanTile], sdA[kScanTile];
  const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int ns = tid & 15, pl = tid >> 4, p0 = blockIdx.z * 16, p = p0 + pl;
  const int row0 = cu[s], len = cu[s + 1] - row0, slot = slots[s];
  if (len <= 0) return;
  const bool pv = p < P;
  if (slot < 0) {
    for (int i = tid; i < len * 16; i += 256)
      if (p0 + (i & 15) < P) y[(long)(row0 + (i >> 4)) * ys + (long)h * P + p0 + (i & 15)] = 0.f;
    return;
  }
  const int inner = heads * P, grp = h / (heads / groups);
  const long xo = (long)h * P + p0, bo = inner + (long)grp * N, co = inner + (long)groups * N + (long)grp * N;
  float* sp = state + (((long)slot * heads + h) * P + (pv ? p : 0)) * N;
  float S[NR];
  const bool past = positions[row0] > 0;
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int n = ns * NR + i;
    S[i] = (past && pv && n < N) ? sp[n] : 0.f;
  }
  const float nA = -expf(A_log[h]), db = dt_bias[h], Dh = Dp[h];
  // 16-byte staging loads need every row's B / C run to start on a 16-byte boundary
  const bool vec = N % EV == 0 && xs % EV == 0 && bo % EV == 0 && co % EV == 0 &&
                   (reinterpret_cast<uintptr_t>(xbc) & 15) == 0;
  // vector path: the next tile's global loads are issued before the current tile is computed and
  // land in registers meanwhile (a tile's exposed load latency was ~2/3 of its time otherwise)
  constexpr int NPF = (2 * kScanTile * NP / EV + 255) / 256;
  uint4_t pre[NPF];
  float prex = 0.f, predt = 0.f;
  auto fetch = [&](int t0) {
    const int tl = min(kScanTile, len - t0), cpr = N / EV;
#pragma unroll
    for (int k = 0; k < NPF; ++k) {
      const int i = tid + 256 * k;
      if (i < tl * cpr * 2) {
        const int which = i / (tl * cpr), r = i % (tl * cpr), t = r / cpr, c = r % cpr;
        pre[k] = *reinterpret_cast<const uint4_t*>(xbc + (long)(row0 + t0 + t) * xs + (which ? co : bo) + c * EV);
      }
    }
    const int t = tid >> 4, c = tid & 15;
    prex = (t < tl && p0 + c < P) ? ldf<T>(xbc + (long)(row0 + t0 + t) * xs + xo + c) : 0.f;
    if (tid < tl) predt = ldf<T>(dtp + (long)(row0 + t0 + tid) * dts + h);
  };
  if (vec) fetch(0);
  for (int t0 = 0; t0 < len; t0 += kScanTile) {
    const int tl = min(kScanTile, len - t0);
    __syncthreads();  // the previous tile's sy / sB readers are done
    float dtraw = 0.f;
    if (vec) {
      const int cpr = N / EV;
#pragma unroll
      for (int k = 0; k < NPF; ++k) {
        const int i = tid + 256 * k;
        if (i < tl * cpr * 2) {
          const int which = i / (tl * cpr), r = i % (tl * cpr), t = r / cpr, c = r % cpr;
          float* dst = (which ? sC[t] : sB[t]) + c * EV;
          if constexpr (sizeof(T) == 2) {
            const short8 v = __builtin_bit_cast(short8, pre[k]);
#pragma unroll
            for (int e = 0; e < 8; ++e) dst[e] = bf2f((bf16_t)v[e]);
          } else {
            *reinterpret_cast<uint4_t*>(dst) = pre[k];
          }
        }
      }
      if ((tid >> 4) < tl) sx[tid >> 4][tid & 15] = prex;
      dtraw = predt;
    } else {
      for (int i = tid; i < tl * N * 2; i += 256) {
        const int which = i / (tl * N), r = i % (tl * N), t = r / N, n = r % N;
        (which ? sC[t] : sB[t])[n] = ldf<T>(xbc + (long)(row0 + t0 + t) * xs + (which ? co : bo) + n);
      }
      const int t = tid >> 4, c = tid & 15;  // 16 tokens x 16 columns: one x each
      if (t < tl) sx[t][c] = p0 + c < P ? ldf<T>(xbc + (long)(row0 + t0 + t) * xs + xo + c) : 0.f;
      if (tid < tl) dtraw = ldf<T>(dtp + (long)(row0 + t0 + tid) * dts + h);
    }
    if (N < NP)
      for (int i = tid; i < tl * (NP - N); i += 256) {
        const int t = i / (NP - N), n = N + i % (NP - N);
        sB[t][n] = 0.f;
        sC[t][n] = 0.f;
      }
    if (tid < tl) {
      const float a = dtraw + db;
      const float dt = a > 20.f ? a : log1pf(expf(a));
      sdt[tid] = dt;
      sdA[tid] = expf(nA * dt);
    }
    __syncthreads();
    if (vec && t0 + kScanTile < len) fetch(t0 + kScanTile);
    auto token = [&](int t) {
      const float x = sx[t][pl], dA = sdA[t], dx = sdt[t] * x;
      float acc = 0.f;
#pragma unroll
      for (int k = 0; k < NR; ++k) {
        S[k] = dA * S[k] + dx * sB[t][ns * NR + k];
        acc += S[k] * sC[t][ns * NR + k];
      }
      acc += __shfl_xor(acc, 1, 64);
      acc += __shfl_xor(acc, 2, 64);
      acc += __shfl_xor(acc, 4, 64);
      acc += __shfl_xor(acc, 8, 64);
      if (ns == 0) sy[t][pl] = acc + Dh * x;
    };
    if (tl == kScanTile) {  // whole tile: unrolled, so a token's LDS reads issue under its predecessor's reduction
#pragma unroll
      for (int t = 0; t < kScanTile; ++t) token(t);
    } else {
      for (int t = 0; t < tl; ++t) token(t);
    }
    __syncthreads();
    {
      const int t = tid >> 4, c = tid & 15;
      if (t < tl && p0 + c < P) y[(long)(row0 + t0 + t) * ys + (long)h * P + p0 + c] = sy[t][c];
    }
  }
  if (pv) {
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int n = ns * NR + i;
      if (n < N) sp[n] = S[i];
    }
  }
}

// Chunked (matrix-form) scan for prompt portions: the recurrence is unrolled over chunks of 16
// tokens and every product runs on true-f32 MFMAs (v_mfma_f32_16x16x4_f32), the state staying in
// the accumulators' layout from chunk to chunk.  With a_t = -exp(A_log) dt_t, c_t = a_1 + .. + a_t
// inside the chunk and S the state before it:
//   y_t  = exp(c_t) C_t^T S  +  sum_{s<=t} exp(c_t - c_s) dt_s (C_t . B_s) x_s  +  D x_t
//   S'   = exp(c_L) S  +  sum_s exp(c_L - c_s) dt_s B_s x_s^T
// grid (sequence, head, P / 64): wave w owns the 16 state columns p0 + 16 w .. +15 (all N rows:
// N / 16 accumulator tiles).  Per chunk a wave issues about 12 + 4 N / 16 ... MFMAs instead of
// 16 x 2 N / 16 scalar FMA rounds per lane; tokens past the end of the last chunk get dt = a = 0,
// so they neither decay nor feed the state.  Operand orders are permuted as in attn_sigmoid.hip so
// that accumulators feed the next MFMA without shuffles.
template <typename T, int NR>
__global__ __launch_bounds__(256) void ssm_chunk_kernel(const T* __restrict__ xbc, long xs, const T* __restrict__ dtp,
                                                        long dts, int heads, int P, int N, int groups,
                                                        const float* __restrict__ dt_bias,
                                                        const float* __restrict__ A_log, const float* __restrict__ Dp,
                                                        float* __restrict__ state, const int* __restrict__ cu,
                                                        const int* __restrict__ slots,
                                                        const int* __restrict__ positions, float* __restrict__ y,
                                                        long ys) {
  constexpr int NP = NR * 16, LD = NP + 4, L = 16;
  constexpr int EV = 16 / sizeof(T);
  __shared__ __attribute__((aligned(16))) float sB[L][LD];
  __shared__ __attribute__((aligned(16))) float sC[L][LD];
  __shared__ float sx[L][64], sdt[L], sa[L];
  const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, p0 = blockIdx.z * 64;
  const int lane = tid & 63, w = tid >> 6, n16 = lane & 15, g = lane >> 4;
  const int pcol = p0 + 16 * w + n16;
  const bool pv = pcol < P;
  const int row0 = cu[s], len = cu[s + 1] - row0, slot = slots[s];
  if (len <= 0) return;
  if (slot < 0) {
    for (int i = tid; i < len * 64; i += 256)
      if (p0 + (i & 63) < P) y[(long)(row0 + (i >> 6)) * ys + (long)h * P + p0 + (i & 63)] = 0.f;
    return;
  }
  const int inner = heads * P, grp = h / (heads / groups);
  const long xo = (long)h * P + p0, bo = inner + (long)grp * N, co = inner + (long)groups * N + (long)grp * N;
  float* sp = state + (((long)slot * heads + h) * P + (pv ? pcol : 0)) * N;
  const bool past = positions[row0] > 0;
  floatx4 S[NR];
#pragma unroll
  for (int nt = 0; nt < NR; ++nt)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = nt * 16 + 4 * g + j;
      S[nt][j] = (past && pv && n < N) ? sp[n] : 0.f;
    }
  const float nA = -expf(A_log[h]), db = dt_bias[h], Dh = Dp[h];
  const bool vec = N % EV == 0 && xs % EV == 0 && bo % EV == 0 && co % EV == 0 &&
                   (reinterpret_cast<uintptr_t>(xbc) & 15) == 0;
  // vector path: the next chunk's operands are requested before this chunk's products are issued
  constexpr int NPF = (2 * L * NP / EV + 255) / 256;
  uint4_t pre[NPF];
  float prex[4], predt = 0.f;
  auto fetch = [&](int t0) {
    const int tl = min(L, len - t0), cpr = NP / EV, ncpr = N / EV;
#pragma unroll
    for (int k = 0; k < NPF; ++k) {
      const int i = tid + 256 * k;
      pre[k] = uint4_t{0u, 0u, 0u, 0u};
      if (i < L * cpr * 2) {
        const int which = i / (L * cpr), r = i % (L * cpr), t = r / cpr, c = r % cpr;
        if (t < tl && c < ncpr)
          pre[k] = *reinterpret_cast<const uint4_t*>(xbc + (long)(row0 + t0 + t) * xs + (which ? co : bo) + c * EV);
      }
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int i = tid + 256 * k, t = i >> 6, c = i & 63;
      prex[k] = (t < tl && p0 + c < P) ? ldf<T>(xbc + (long)(row0 + t0 + t) * xs + xo + c) : 0.f;
    }
    predt = tid < tl ? ldf<T>(dtp + (long)(row0 + t0 + tid) * dts + h) : 0.f;
  };
  if (vec) fetch(0);
  for (int t0 = 0; t0 < len; t0 += L) {
    const int tl = min(L, len - t0);
    __syncthreads();
    float dtraw = 0.f;
    if (vec) {
      const int cpr = NP / EV;
#pragma unroll
      for (int k = 0; k < NPF; ++k) {
        const int i = tid + 256 * k;
        if (i < L * cpr * 2) {
          const int which = i / (L * cpr), r = i % (L * cpr), t = r / cpr, c = r % cpr;
          float* dst = (which ? sC[t] : sB[t]) + c * EV;
          if constexpr (sizeof(T) == 2) {
            const short8 v = __builtin_bit_cast(short8, pre[k]);
#pragma unroll
            for (int e = 0; e < 8; ++e) dst[e] = bf2f((bf16_t)v[e]);
          } else {
            *reinterpret_cast<uint4_t*>(dst) = pre[k];
          }
        }
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int i = tid + 256 * k;
        sx[i >> 6][i & 63] = prex[k];
      }
      dtraw = predt;
    } else {
      for (int i = tid; i < L * NP * 2; i += 256) {
        const int which = i / (L * NP), r = i % (L * NP), t = r / NP, n = r % NP;
        (which ? sC[t] : sB[t])[n] =
            (t < tl && n < N) ? ldf<T>(xbc + (long)(row0 + t0 + t) * xs + (which ? co : bo) + n) : 0.f;
      }
      for (int i = tid; i < L * 64; i += 256) {
        const int t = i >> 6, c = i & 63;
        sx[t][c] = (t < tl && p0 + c < P) ? ldf<T>(xbc + (long)(row0 + t0 + t) * xs + xo + c) : 0.f;
      }
      if (tid < tl) dtraw = ldf<T>(dtp + (long)(row0 + t0 + tid) * dts + h);
    }
    if (tid < L) {
      float dt = 0.f;
      if (tid < tl) {
        const float a = dtraw + db;
        dt = a > 20.f ? a : log1pf(expf(a));
      }
      sdt[tid] = dt;
      sa[tid] = nA * dt;
    }
    __syncthreads();
    if (vec && t0 + L < len) fetch(t0 + L);
    // inclusive prefix of the log-decays inside every 16-lane group: lane n16 ends up with c_(n16)
    float cum = sa[n16];
#pragma unroll
    for (int o = 1; o < 16; o <<= 1) {
      const float v = __shfl_up(cum, o, 16);
      if (n16 >= o) cum += v;
    }
    // G^T: lane (t = n16, g) gets G[t][s = 4g + j] = C_t . B_s
    floatx4 gt = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int nb = 0; nb < NR; ++nb) {
      const floatx4 a4 = *reinterpret_cast<const floatx4*>(&sB[n16][nb * 16 + 4 * g]);
      const floatx4 b4 = *reinterpret_cast<const floatx4*>(&sC[n16][nb * 16 + 4 * g]);
#pragma unroll
      for (int j = 0; j < 4; ++j) gt = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[j], b4[j], gt, 0, 0, 0);
    }
    const float ct = cum, cl = __shfl(cum, 15, 16);
    float M[4], xv[4], wv[4], ec[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int sj = 4 * g + j;
      const float cs = __shfl(cum, sj, 16), ds = sdt[sj];
      M[j] = sj <= n16 ? gt[j] * expf(ct - cs) * ds : 0.f;
      xv[j] = sx[sj][16 * w + n16];
      wv[j] = expf(cl - cs) * ds;
      ec[j] = expf(cs);
    }
    // y: rows t = 4g + j, column p = n16 of this wave's tile
    floatx4 ya = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int nt = 0; nt < NR; ++nt) {
      const floatx4 c4 = *reinterpret_cast<const floatx4*>(&sC[n16][nt * 16 + 4 * g]);
#pragma unroll
      for (int j = 0; j < 4; ++j) ya = __builtin_amdgcn_mfma_f32_16x16x4f32(c4[j], S[nt][j], ya, 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) ya[j] *= ec[j];
#pragma unroll
    for (int j = 0; j < 4; ++j) ya = __builtin_amdgcn_mfma_f32_16x16x4f32(M[j], xv[j], ya, 0, 0, 0);
    if (pv) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int t = 4 * g + j;
        if (t < tl) y[(long)(row0 + t0 + t) * ys + (long)h * P + pcol] = ya[j] + Dh * xv[j];
      }
    }
    // state: rows n = 16 nt + 4g + j, column p = n16
    const float dec = expf(cl);
#pragma unroll
    for (int nt = 0; nt < NR; ++nt) {
#pragma unroll
      for (int j = 0; j < 4; ++j) S[nt][j] *= dec;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        S[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(sB[4 * g + j][nt * 16 + n16] * wv[j], xv[j], S[nt], 0, 0, 0);
    }
  }
  if (pv) {
#pragma unroll
    for (int nt = 0; nt < NR; ++nt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = nt * 16 + 4 * g + j;
        if (n < N) sp[n] = S[nt][j];
      }
  }
}

// grid (row, norm group): out = (y * silu(z)) / sqrt(mean_group((y silu z)^2) + eps) * w
template <typename T>
__global__ __launch_bounds__(256) void gated_group_rmsnorm_kernel(const float* __restrict__ y, long ys,
                                                                  const T* __restrict__ z, long zs,
                                                                  const float* __restrict__ w, int gs, float eps,
                                                                  T* __restrict__ out, long os) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  const int c0 = blockIdx.y * gs;
  float ss = 0.f;
  for (int c = threadIdx.x; c < gs; c += 256) {
    const float v = y[row * ys + c0 + c] * silu_f<sizeof(T) == 4>(ldf<T>(z + row * zs + c0 + c));
    ss += v * v;
  }
  ss = block_sum<4>(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)gs + eps);
  for (int c = threadIdx.x; c < gs; c += 256) {
    const float v = y[row * ys + c0 + c] * silu_f<sizeof(T) == 4>(ldf<T>(z + row * zs + c0 + c));
    stf<T>(out + row * os + c0 + c, v * inv * w[c0 + c]);
  }
}

// prompt portions (some sequence of the step has >= kChunkMin rows): the chunked MFMA kernel
constexpr int kChunkMin = 8;

template <typename T>
int scan_t(const T* xbc, long xs, const T* dtp, long dts, int S, int heads, int P, int N, int groups,
           const float* dt_bias, const float* A_log, const float* D, float* state, const int* cu, const int* slots,
           const int* positions, float* y, long ys, int max_len, hipStream_t st) {
  if (max_len >= kChunkMin) {
    dim3 cgrid(S, heads, (P + 63) / 64);
#define LK_CHUNK(NR)                                                                                                   \
  ssm_chunk_kernel<T, NR><<<cgrid, 256, 0, st>>>(xbc, xs, dtp, dts, heads, P, N, groups, dt_bias, A_log, D, state, cu, \
                                                 slots, positions, y, ys)
    if (N <= 16) LK_CHUNK(1);
    else if (N <= 32) LK_CHUNK(2);
    else if (N <= 64) LK_CHUNK(4);
    else if (N <= 128) LK_CHUNK(8);
    else if (N <= 256) LK_CHUNK(16);
    else return -1;
#undef LK_CHUNK
    LK_CHECK_LAUNCH();
    return 0;
  }
  dim3 grid(S, heads, (P + 15) / 16);
#define LK_SCAN(NR)                                                                                                 \
  ssm_scan_kernel<T, NR><<<grid, 256, 0, st>>>(xbc, xs, dtp, dts, heads, P, N, groups, dt_bias, A_log, D, state, cu, \
                                               slots, positions, y, ys)
  if (N <= 16) LK_SCAN(1);
  else if (N <= 32) LK_SCAN(2);
  else if (N <= 64) LK_SCAN(4);
  else if (N <= 128) LK_SCAN(8);
  else if (N <= 256) LK_SCAN(16);
  else return -1;
#undef LK_SCAN
  LK_CHECK_LAUNCH();
  return 0;
}

}  // namespace

int lk_conv_silu(const void* u, long us, int C, int taps, const float* w, const float* bias, void* state, const int* cu,
                 const int* slots, const int* positions, int S, int max_len, void* out, long os, int act, int esz,
                 hipStream_t st) {
  if (S <= 0 || max_len <= 0) return 0;
  if (taps < 1 || taps > kMaxTaps || C <= 0) return -1;
  dim3 grid(S, (max_len + kConvRows - 1) / kConvRows, (C + 255) / 256), g2(S, (C + 255) / 256);
  const int ev = 16 / esz;
  const auto a16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (taps <= 4 && C % ev == 0 && us % ev == 0 && os % ev == 0 && a16(u) && a16(out) && a16(state)) {
    const int cblocks = (C / ev + 255) / 256;
    // tokens per workgroup (a kernel argument: tiles of 4 tokens were tried for steps of few, long sequences, where 16-token
    // tiles leave a chip of 256 CUs a handful of waves each, and measured slower: 79 us against 61 us at 4 x 1,024 x 2,048)
    const int rows = kConvRows;
    dim3 gv(S, (max_len + rows - 1) / rows, cblocks);
    if (esz == 2)
      conv_silu_vec_kernel<bf16_t><<<gv, 256, 0, st>>>((const bf16_t*)u, us, C, taps, w, bias, (const bf16_t*)state, cu,
                                                       slots, positions, (bf16_t*)out, os, act, rows);
    else
      conv_silu_vec_kernel<float><<<gv, 256, 0, st>>>((const float*)u, us, C, taps, w, bias, (const float*)state, cu, slots,
                                                      positions, (float*)out, os, act, rows);
    LK_CHECK_LAUNCH();
    if (taps > 1) {
      if (esz == 2) conv_state_kernel<bf16_t><<<g2, 256, 0, st>>>((const bf16_t*)u, us, C, taps, (bf16_t*)state, cu, slots, positions);
      else conv_state_kernel<float><<<g2, 256, 0, st>>>((const float*)u, us, C, taps, (float*)state, cu, slots, positions);
      LK_CHECK_LAUNCH();
    }
    return 0;
  }
  if (esz == 2) {
    conv_silu_kernel<bf16_t><<<grid, 256, 0, st>>>((const bf16_t*)u, us, C, taps, w, bias, (const bf16_t*)state, cu,
                                                   slots, positions, (bf16_t*)out, os, act);
    LK_CHECK_LAUNCH();
    if (taps > 1) conv_state_kernel<bf16_t><<<g2, 256, 0, st>>>((const bf16_t*)u, us, C, taps, (bf16_t*)state, cu, slots, positions);
  } else {
    conv_silu_kernel<float><<<grid, 256, 0, st>>>((const float*)u, us, C, taps, w, bias, (const float*)state, cu, slots,
                                                  positions, (float*)out, os, act);
    LK_CHECK_LAUNCH();
    if (taps > 1) conv_state_kernel<float><<<g2, 256, 0, st>>>((const float*)u, us, C, taps, (float*)state, cu, slots, positions);
  }
  LK_CHECK_LAUNCH();
  return 0;
}

int lk_ssm_scan(const void* xbc, long xs, const void* dt, long dts, int S, int heads, int P, int N, int groups,
                const float* dt_bias, const float* A_log, const float* D, float* state, const int* cu, const int* slots,
                const int* positions, float* y, long ys, int max_len, int esz, hipStream_t st) {
  if (S <= 0) return 0;
  if (heads <= 0 || groups <= 0 || heads % groups || P <= 0 || N <= 0) return -1;
  return esz == 2 ? scan_t<bf16_t>((const bf16_t*)xbc, xs, (const bf16_t*)dt, dts, S, heads, P, N, groups, dt_bias,
                                   A_log, D, state, cu, slots, positions, y, ys, max_len, st)
                  : scan_t<float>((const float*)xbc, xs, (const float*)dt, dts, S, heads, P, N, groups, dt_bias, A_log,
                                  D, state, cu, slots, positions, y, ys, max_len, st);
}

int lk_gated_group_rmsnorm(const float* y, long ys, const void* z, long zs, const float* w, long rows, int inner,
                           int ngroups, float eps, void* out, long os, int esz, hipStream_t st) {
  if (rows <= 0) return 0;
  if (ngroups <= 0 || inner % ngroups) return -1;
  dim3 grid((unsigned)rows, ngroups);
  if (esz == 2)
    gated_group_rmsnorm_kernel<bf16_t><<<grid, 256, 0, st>>>(y, ys, (const bf16_t*)z, zs, w, inner / ngroups, eps,
                                                             (bf16_t*)out, os);
  else
    gated_group_rmsnorm_kernel<float><<<grid, 256, 0, st>>>(y, ys, (const float*)z, zs, w, inner / ngroups, eps,
                                                            (float*)out, os);
  LK_CHECK_LAUNCH();
  return 0;
}

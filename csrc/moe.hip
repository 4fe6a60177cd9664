// Feed-forward of experts chosen per token by a table of token ids (no routing network, equal weights).
//
//   lk_moe_route  (token, choice) pairs p = t * top + k sorted by their expert table[ids[t]][k] (ids null: table[t][k], the
//                 choice a router made for each token of the step): seg[e] .. seg[e + 1] are
//                 expert e's places in `order`.  One workgroup: a histogram and a placement with LDS atomics (the order
//                 inside an expert's segment is arbitrary; every row of the products below is computed on its own).
//   lk_moe_gemm   grouped product over the sorted pairs on MFMA tiles of 16 pairs: a tile's rows belong to one expert,
//                 so its B operand is that expert's weight rows.  The tile list is not materialised: a workgroup finds
//                 its (expert, first pair) by walking seg[], so the launch needs nothing from the host and a step with
//                 experts can be captured in a graph.
//                   act = 1:  mid[place] = silu(W_gate x_t) * (W_up x_t)   (x row of the pair's token; rows of `mid` in
//                             sorted order; W = [gate rows | up rows], F columns each)
//                   act = 0:  out[p]     = W_down mid[place]               (rows of `out` in pair order, so a token's
//                             `top` results are adjacent for the consumer that averages them)
//
// Fragments go straight from global memory / L2 into the MFMA operands (16-byte loads where rows are 16-byte
// aligned, element loads otherwise), f32 accumulation, bf16 (v_mfma_f32_16x16x32_bf16) or f32 (16x16x4) activations.
#include "common.h"
#include "kernels.h"
#include "attn_frag.h"

namespace {

constexpr int kRouteThreads = 1024;
constexpr int kMaxExperts = 1024;

__global__ __launch_bounds__(kRouteThreads) void moe_route_kernel(const int* __restrict__ ids, const int* __restrict__ table, int vocab,
                                                                  int top, int E, int T, int* __restrict__ seg,
                                                                  int* __restrict__ order) {
  __shared__ int cnt[kMaxExperts];
  __shared__ int nxt[kMaxExperts];
  const int n = T * top;
  for (int e = threadIdx.x; e < E; e += kRouteThreads) cnt[e] = 0;
  __syncthreads();
  auto expert_of = [&](int p) {
    int id = ids ? ids[p / top] : p / top;      // no ids: the table has one row per token of the step
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const int e = table[(long)id * top + p % top];
    return e < 0 ? 0 : (e >= E ? E - 1 : e);
  };
  for (int p = threadIdx.x; p < n; p += kRouteThreads) atomicAdd(&cnt[expert_of(p)], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int acc = 0;
    for (int e = 0; e < E; ++e) {
      seg[e] = acc;
      nxt[e] = acc;
      acc += cnt[e];
    }
    seg[E] = acc;
  }
  __syncthreads();
  for (int p = threadIdx.x; p < n; p += kRouteThreads) order[atomicAdd(&nxt[expert_of(p)], 1)] = p;
}

// 16 bytes of row `r` at element k (EV elements; zeros past K): one vector load when the row allows it
template <typename T>
LK_DEVICE uint4_t frag(const T* r, int k, int K, bool vec) {
  constexpr int EV = El<T>::V;
  if (vec && k + EV <= K) return ld16(r + k);
  alignas(16) T tmp[EV];
#pragma unroll
  for (int e = 0; e < EV; ++e) tmp[e] = k + e < K ? r[k + e] : T(0);
  return *reinterpret_cast<const uint4_t*>(tmp);
}

// grid (row tiles of 16 RT pairs: at most pairs / (16 RT) + E, column blocks): 4 waves side by side along the columns, each
// RT row tiles x NB column tiles of 16 x 16 in registers, so a step of the contraction costs RT + NB fragment loads for
// RT x NB MFMAs (RT = 1, NB = 2: decode-sized steps, where the experts' weights are read once and little else
// matters; RT = 4, NB = 4: prompt portions).  The waves of a workgroup read the same x rows (L1 hits).
//   act: a wave's column tiles are NB / 2 gate tiles and the up tiles of the same columns;
//   else: NB neighbouring tiles of output columns.
template <typename T, bool ACT, int RT>
__global__ __launch_bounds__(256) void moe_gemm_kernel(const T* __restrict__ x, long xs, const int* __restrict__ order,
                                                       const int* __restrict__ seg, int E, int top, const T* __restrict__ w, int N,
                                                       int K, T* __restrict__ out, long os, int vec) {
  constexpr int EV = El<T>::V, NB = RT == 1 ? 2 : 4, CW = ACT ? NB / 2 : NB;   // CW: 16-column tiles of output per wave
  constexpr bool EXACT = sizeof(T) == 4;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, n16 = lane & 15, g = lane >> 4;
  // this workgroup's expert and first place: tiles are counted expert by expert
  int e = 0, place0 = 0, end = 0, acc = 0;
  {
    const int tile = blockIdx.x;
    bool found = false;
    for (int i = 0; i < E; ++i) {
      const int a = seg[i], b = seg[i + 1], nt = (b - a + 16 * RT - 1) / (16 * RT);
      if (!found && tile < acc + nt) {
        found = true;
        e = i;
        place0 = a + (tile - acc) * 16 * RT;
        end = b;
      }
      acc += nt;
    }
    if (!found) return;
  }
  const int F = ACT ? N / 2 : N;                       // output columns
  const int c0 = (blockIdx.y * 4 + wv) * CW * 16;
  if (c0 >= F) return;
  const T* xrow[RT];
  bool rvalid[RT];
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    const int place = place0 + 16 * r + n16;
    rvalid[r] = place < end;
    const int pair = rvalid[r] ? order[place] : 0;
    xrow[r] = x + (long)(ACT ? pair / top : (rvalid[r] ? place : 0)) * xs;
  }
  const T* wbase = w + (long)e * N * K;
  // B operand rows: rows of columns past the end read row 0 and are not stored
  const T* wrow[NB];
#pragma unroll
  for (int c = 0; c < NB; ++c) {
    const int oc = c0 + 16 * (c % CW) + n16;                       // output column of this tile
    const int row = ACT && c >= CW ? F + oc : oc;                   // up rows follow the F gate rows
    wrow[c] = wbase + (long)(oc < F ? row : 0) * K;
  }
  floatx4 accv[RT][NB];
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int c = 0; c < NB; ++c) accv[r][c] = floatx4{0.f, 0.f, 0.f, 0.f};
  // Every lane runs every step (the MFMAs need the whole wave).  With 16-byte aligned rows, groups of U whole steps are
  // plain vector loads issued together before their MFMAs (U x (RT + NB) requests in flight per lane: a decode-sized step
  // is a stream of expert weights, and what it needs is memory-level parallelism); rows behind the end of a tile read a
  // valid row whose results are never stored.  What is left, and unaligned rows, go through frag(), which pads with zeros.
  constexpr int U = RT == 1 ? 4 : 1;
  int kb = 0;
  if (vec) {
    for (; kb + U * 4 * EV <= K; kb += U * 4 * EV) {
      uint4_t a[U][RT], b[U][NB];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int k = kb + (4 * u + g) * EV;
#pragma unroll
        for (int r = 0; r < RT; ++r) a[u][r] = ld16(xrow[r] + k);
#pragma unroll
        for (int c = 0; c < NB; ++c) b[u][c] = ld16(wrow[c] + k);
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int r = 0; r < RT; ++r)
#pragma unroll
          for (int c = 0; c < NB; ++c) accv[r][c] = mma_qk<T>(a[u][r], b[u][c], accv[r][c]);
    }
  }
  for (; kb < K; kb += 4 * EV) {
    const int k = kb + g * EV;
    uint4_t a[RT], b[NB];
#pragma unroll
    for (int r = 0; r < RT; ++r) a[r] = frag<T>(xrow[r], k, K, vec);
#pragma unroll
    for (int c = 0; c < NB; ++c) b[c] = frag<T>(wrow[c], k, K, vec);
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
      for (int c = 0; c < NB; ++c) accv[r][c] = mma_qk<T>(a[r], b[c], accv[r][c]);
  }
  // accumulator j of this lane: pair row 4 g + j of the row tile, column n16 of the column tile
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int pl = place0 + 16 * r + 4 * g + j;
      if (pl >= end) continue;
      T* orow = out + (long)(ACT ? pl : order[pl]) * os;
#pragma unroll
      for (int c = 0; c < CW; ++c) {
        const int col = c0 + 16 * c + n16;
        if (col >= F) continue;
        if constexpr (ACT) {
          const float gt = accv[r][c][j];
          const float sg = EXACT ? gt / (1.f + expf(-gt)) : gt * __builtin_amdgcn_rcpf(1.f + __expf(-gt));
          El<T>::st(orow + col, sg * accv[r][CW + c][j]);
        } else {
          El<T>::st(orow + col, accv[r][c][j]);
        }
      }
    }
}

// The same product for prompt-sized steps with 16-byte aligned rows: a workgroup owns 32 RT pairs x 128 weight
// rows (act: 64 gate rows and the 64 up rows of the same columns), its 4 waves 16 RT x 64 quarters of it (RT = 4).  Both operands of a
// 64-byte step of the contraction are fetched once per workgroup with coalesced 16-byte loads (the next step's while this
// one is multiplied), staged in LDS (rows padded to 80 bytes against bank conflicts, two buffers, one barrier per step)
// and read from there as MFMA fragments, so global memory sees each operand byte once per workgroup instead of once per wave.
template <typename T, bool ACT, int RT>
__global__ __launch_bounds__(256) void moe_gemm_lds_kernel(const T* __restrict__ x, long xs, const int* __restrict__ order,
                                                           const int* __restrict__ seg, int E, int top, const T* __restrict__ w, int N,
                                                           int K, T* __restrict__ out, long os) {
  constexpr int EV = El<T>::V, KS = 4 * EV, TM = 32 * RT, TN = 128, PA = TM / 64;   // PA: 16-byte pieces of the A tile per thread
  constexpr bool EXACT = sizeof(T) == 4;
  __shared__ uint4_t sA[2][TM][5];
  __shared__ uint4_t sB[2][TN][5];
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, n16 = lane & 15, g = lane >> 4;
  const int F = ACT ? N / 2 : N;
  const int CB = (F + (ACT ? 64 : 128) - 1) / (ACT ? 64 : 128);   // column blocks
  // Work items in the order (expert, column block, row tile of the expert), dealt to the XCDs in contiguous runs: the
  // workgroups an XCD runs together share a few row tiles of x (they stay in its L2 over the column blocks) and each
  // block of weight rows among an expert's row tiles.
  int e = 0, place0 = 0, end = 0, cb = 0, acc = 0;
  {
    const int item = xcd_remap(blockIdx.x, gridDim.x);
    bool found = false;
    for (int i = 0; i < E; ++i) {
      const int a = seg[i], b = seg[i + 1], nt = (b - a + TM - 1) / TM;
      if (!found && item < acc + nt * CB) {
        found = true;
        e = i;
        cb = (item - acc) / nt;
        place0 = a + ((item - acc) % nt) * TM;
        end = b;
      }
      acc += nt * CB;
    }
    if (!found) return;   // the whole workgroup leaves: no barrier is skipped by a part of it
  }
  const int c0 = cb * (ACT ? 64 : 128);
  const T* wbase = w + (long)e * N * K;
  // this thread's two 16-byte pieces of the A tile and of the B tile: piece = tid + 256 i -> row piece / 4, segment piece % 4
  const T* ap[PA];
  const T* bp[2];
  const int pseg = tid & 3, prow = tid >> 2;   // piece tid + 256 i: row prow + 64 i, segment pseg
#pragma unroll
  for (int i = 0; i < PA; ++i) {
    const int place = place0 + prow + 64 * i;
    ap[i] = place < end ? x + (long)(ACT ? order[place] / top : place) * xs : nullptr;
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = prow + 64 * i;
    const int oc = ACT ? c0 + (r & 63) : c0 + r;
    const int row = ACT && r >= 64 ? F + oc : oc;
    bp[i] = oc < F ? wbase + (long)row * K : nullptr;
  }
  const int wy = wv >> 1, wx = wv & 1;
  int brow[4];   // first B-tile row of the wave's column tiles
#pragma unroll
  for (int c = 0; c < 4; ++c) brow[c] = ACT ? (c < 2 ? wx * 32 + 16 * c : 64 + wx * 32 + 16 * (c - 2)) : wx * 64 + 16 * c;
  floatx4 accv[RT][4];
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int c = 0; c < 4; ++c) accv[r][c] = floatx4{0.f, 0.f, 0.f, 0.f};
  uint4_t ra[PA], rb[2];
  auto fetch = [&](int kb) {
    const int k = kb + pseg * EV;
#pragma unroll
    for (int i = 0; i < PA; ++i) ra[i] = ap[i] && k < K ? ld16(ap[i] + k) : uint4_t{0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < 2; ++i) rb[i] = bp[i] && k < K ? ld16(bp[i] + k) : uint4_t{0u, 0u, 0u, 0u};
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int i = 0; i < PA; ++i) sA[buf][prow + 64 * i][pseg] = ra[i];
#pragma unroll
    for (int i = 0; i < 2; ++i) sB[buf][prow + 64 * i][pseg] = rb[i];
  };
  fetch(0);
  stage(0);
  __syncthreads();
  int cur = 0;
  for (int kb = 0; kb < K; kb += KS) {
    const bool more = kb + KS < K;
    if (more) fetch(kb + KS);
    uint4_t a[RT], b[4];
#pragma unroll
    for (int r = 0; r < RT; ++r) a[r] = sA[cur][wy * 16 * RT + 16 * r + n16][g];
#pragma unroll
    for (int c = 0; c < 4; ++c) b[c] = sB[cur][brow[c] + n16][g];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
      for (int c = 0; c < 4; ++c) accv[r][c] = mma_qk<T>(a[r], b[c], accv[r][c]);
    if (more) stage(cur ^ 1);
    __syncthreads();
    cur ^= 1;
  }
  constexpr int CW = ACT ? 2 : 4;
  const int wc0 = c0 + (ACT ? wx * 32 : wx * 64);
#pragma unroll
  for (int r = 0; r < RT; ++r)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int pl = place0 + wy * 16 * RT + 16 * r + 4 * g + j;
      if (pl >= end) continue;
      T* orow = out + (long)(ACT ? pl : order[pl]) * os;
#pragma unroll
      for (int c = 0; c < CW; ++c) {
        const int col = wc0 + 16 * c + n16;
        if (col >= F) continue;
        if constexpr (ACT) {
          const float gt = accv[r][c][j];
          const float sg = EXACT ? gt / (1.f + expf(-gt)) : gt * __builtin_amdgcn_rcpf(1.f + __expf(-gt));
          El<T>::st(orow + col, sg * accv[r][CW + c][j]);
        } else {
          El<T>::st(orow + col, accv[r][c][j]);
        }
      }
    }
}

template <typename T, bool ACT, int RT>
int launch_moe_lds(const void* x, long xs, const int* order, const int* seg, int E, int top, long pairs, const void* w, int N, int K,
                   void* out, long os, hipStream_t st) {
  const int F = ACT ? N / 2 : N, per_wg = ACT ? 64 : 128, TM = 32 * RT;
  const long items = ((pairs + TM - 1) / TM + E) * ((F + per_wg - 1) / per_wg);
  if (items > 2147483647L) return -1;
  const dim3 grid((unsigned)items);
  moe_gemm_lds_kernel<T, ACT, RT><<<grid, 256, 0, st>>>((const T*)x, xs, order, seg, E, top, (const T*)w, N, K, (T*)out, os);
  LK_CHECK_LAUNCH();
  return 0;
}

template <typename T, bool ACT, int RT>
int launch_moe(const void* x, long xs, const int* order, const int* seg, int E, int top, long pairs, const void* w, int N, int K,
               void* out, long os, int vec, hipStream_t st) {
  constexpr int NB = RT == 1 ? 2 : 4, per_wg = 4 * 16 * (ACT ? NB / 2 : NB);
  const int F = ACT ? N / 2 : N;
  const long tiles = (pairs + 16 * RT - 1) / (16 * RT) + E;
  if (tiles > 2147483647L || (F + per_wg - 1) / per_wg > 65535) return -1;
  const dim3 grid((unsigned)tiles, (unsigned)((F + per_wg - 1) / per_wg));
  moe_gemm_kernel<T, ACT, RT><<<grid, 256, 0, st>>>((const T*)x, xs, order, seg, E, top, (const T*)w, N, K, (T*)out, os, vec);
  LK_CHECK_LAUNCH();
  return 0;
}

template <typename T>
int moe_gemm_t(const void* x, long xs, const int* order, const int* seg, int E, int top, long pairs, const void* w, int N, int K,
               int act, void* out, long os, int vec, hipStream_t st) {
  // wide row tiles once an expert has 64 pairs on average (a choice by sizes the host knows: the same for every replay)
  const bool wide = pairs >= 64L * E;
  if (wide && vec) {   // 128-pair tiles staged in LDS (256-pair tiles, RT = 8, measured slower: 575 us against 365 us)
    return act ? launch_moe_lds<T, true, 4>(x, xs, order, seg, E, top, pairs, w, N, K, out, os, st)
               : launch_moe_lds<T, false, 4>(x, xs, order, seg, E, top, pairs, w, N, K, out, os, st);
  }
  if (act) return wide ? launch_moe<T, true, 4>(x, xs, order, seg, E, top, pairs, w, N, K, out, os, vec, st)
                       : launch_moe<T, true, 1>(x, xs, order, seg, E, top, pairs, w, N, K, out, os, vec, st);
  return wide ? launch_moe<T, false, 4>(x, xs, order, seg, E, top, pairs, w, N, K, out, os, vec, st)
              : launch_moe<T, false, 1>(x, xs, order, seg, E, top, pairs, w, N, K, out, os, vec, st);
}

}  // namespace

int lk_moe_route(const int* ids, const int* table, int vocab, int top, int E, int T, int* seg, int* order, hipStream_t st) {
  if (T <= 0) return 0;
  if (E < 1 || E > kMaxExperts || top < 1 || vocab < 1) return -1;
  moe_route_kernel<<<1, kRouteThreads, 0, st>>>(ids, table, vocab, top, E, T, seg, order);
  LK_CHECK_LAUNCH();
  return 0;
}

int lk_moe_gemm(const void* x, long xs, const int* order, const int* seg, int E, int top, long pairs, const void* w, int N, int K,
                int act, void* out, long os, int esz, hipStream_t st) {
  if (pairs <= 0) return 0;
  if (E < 1 || top < 1 || N < 1 || K < 1 || (act && N % 2)) return -1;
  const int ev = 16 / esz;
  const int vec = K % ev == 0 && xs % ev == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0;
  return esz == 2 ? moe_gemm_t<bf16_t>(x, xs, order, seg, E, top, pairs, w, N, K, act, out, os, vec, st)
                  : moe_gemm_t<float>(x, xs, order, seg, E, top, pairs, w, N, K, act, out, os, vec, st);
}

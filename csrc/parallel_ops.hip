// Kernels around parallel sublayers and routed experts (bf16 or f32 activations; everything between the loads and
// the stores is f32):
//
//   lk_stream_parallel_norm  x += a + b + sum_k yw[t, k] y[t top + k];  o1 = rms(x) w1,  o2 = rms(x) w2   (one root)
//   lk_router_topk           z = W_router h (f32), s = sigmoid(z) (evaluated in f64); experts in equal groups of neighbours, a group's
//                            score = the sum of its two largest s, only the `keep` best groups can be chosen; the
//                            `top` largest s among those; weights s / (sum of the chosen s + 1e-20) * scale
//   lk_clamped_glu           g = min(gate, limit), u = clamp(up, -limit, limit):  g sigmoid(alpha g) (u + 1)
//   lk_silu_, lk_sigmoid_mul_  element-wise, in place on a block of columns
//
// rms(v) = v / sqrt(mean(v^2) + eps).
#include "common.h"
#include "kernels.h"

namespace {

template <typename T>
LK_DEVICE float ldv(const T* p);
template <>
LK_DEVICE float ldv<bf16_t>(const bf16_t* p) { return bf2f(*p); }
template <>
LK_DEVICE float ldv<float>(const float* p) { return *p; }
template <typename T>
LK_DEVICE void stv(T* p, float v);
template <>
LK_DEVICE void stv<bf16_t>(bf16_t* p, float v) { *p = f2bf(v); }
template <>
LK_DEVICE void stv<float>(float* p, float v) { *p = v; }

template <typename T, int V>
LK_DEVICE void ldn(const T* p, float (&f)[V]) {
  if constexpr (V == 4 && sizeof(T) == 4) {
    const floatx4 t = *reinterpret_cast<const floatx4*>(p);
#pragma unroll
    for (int e = 0; e < 4; ++e) f[e] = t[e];
  } else if constexpr (V == 4) {
    const short4_t t = *reinterpret_cast<const short4_t*>(p);
#pragma unroll
    for (int e = 0; e < 4; ++e) f[e] = bf2f((bf16_t)t[e]);
  } else {
    f[0] = ldv<T>(p);
  }
}

template <typename T, int V>
LK_DEVICE void stn(T* p, const float (&f)[V]) {
  if constexpr (V == 4 && sizeof(T) == 4) {
    *reinterpret_cast<floatx4*>(p) = floatx4{f[0], f[1], f[2], f[3]};
  } else if constexpr (V == 4) {
    *reinterpret_cast<short4_t*>(p) = short4_t{(short)f2bf(f[0]), (short)f2bf(f[1]), (short)f2bf(f[2]), (short)f2bf(f[3])};
  } else {
    stv<T>(p, f[0]);
  }
}

struct ParNormParams {
  float* x;
  const void* a;   // [T, W] or null
  long as;
  const void* b;   // [T, W] or null
  long bs;
  const void* y;   // [T * top, W] or null
  long ys;
  const float* yw; // [T, top]
  int top;
  const float* w1; // null: no o1
  const float* w2;
  float eps;
  void* o1;
  long o1s;
  void* o2;
  long o2s;
  int W;
};

// One workgroup per token; thread i owns the column groups i, i + 256, ... of V adjacent columns (MAXI groups at most)
// in registers between the stream update and the two normed copies.  V = 4: 16-byte f32 / 8-byte bf16 accesses.
template <typename T, int MAXI, int V>
__global__ __launch_bounds__(256) void stream_parallel_norm_kernel(ParNormParams p) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  const int ng = p.W / V;
  const T* a = reinterpret_cast<const T*>(p.a);
  const T* b = reinterpret_cast<const T*>(p.b);
  const T* y = reinterpret_cast<const T*>(p.y);
  const bool upd = a || b || y;
  float v[MAXI][V];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < MAXI; ++i) {
    const int c = (threadIdx.x + 256 * i) * V;
    if (threadIdx.x + 256 * i < ng) {
      float d[V], t[V];
#pragma unroll
      for (int e = 0; e < V; ++e) d[e] = 0.f;
      if (a) {
        ldn<T, V>(a + row * p.as + c, t);
#pragma unroll
        for (int e = 0; e < V; ++e) d[e] += t[e];
      }
      if (b) {
        ldn<T, V>(b + row * p.bs + c, t);
#pragma unroll
        for (int e = 0; e < V; ++e) d[e] += t[e];
      }
      if (y) {
        for (int k = 0; k < p.top; ++k) {
          const float wk = p.yw[row * p.top + k];
          ldn<T, V>(y + (row * p.top + k) * p.ys + c, t);
#pragma unroll
          for (int e = 0; e < V; ++e) d[e] += wk * t[e];
        }
      }
      ldn<float, V>(p.x + row * p.W + c, v[i]);
#pragma unroll
      for (int e = 0; e < V; ++e) {
        v[i][e] += d[e];
        ss += v[i][e] * v[i][e];
      }
      if (upd) stn<float, V>(p.x + row * p.W + c, v[i]);
    }
  }
  if (!p.o1 && !p.o2) return;
  ss = block_sum<4>(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)p.W + p.eps);
#pragma unroll
  for (int i = 0; i < MAXI; ++i) {
    const int c = (threadIdx.x + 256 * i) * V;
    if (threadIdx.x + 256 * i < ng) {
      float wv[V], r[V];
      if (p.o1) {
        ldn<float, V>(p.w1 + c, wv);
#pragma unroll
        for (int e = 0; e < V; ++e) r[e] = v[i][e] * inv * wv[e];
        stn<T, V>(reinterpret_cast<T*>(p.o1) + row * p.o1s + c, r);
      }
      if (p.o2) {
        ldn<float, V>(p.w2 + c, wv);
#pragma unroll
        for (int e = 0; e < V; ++e) r[e] = v[i][e] * inv * wv[e];
        stn<T, V>(reinterpret_cast<T*>(p.o2) + row * p.o2s + c, r);
      }
    }
  }
}

template <typename T>
int par_norm_t(const ParNormParams& p, long rows, bool vec, hipStream_t st) {
  if (vec && p.W <= 4 * 256 * 8) stream_parallel_norm_kernel<T, 8, 4><<<(unsigned)rows, 256, 0, st>>>(p);
  else if (p.W <= 256 * 16) stream_parallel_norm_kernel<T, 16, 1><<<(unsigned)rows, 256, 0, st>>>(p);
  else return -1;
  LK_CHECK_LAUNCH();
  return 0;
}

// ---- router ------------------------------------------------------------------------------------------------
constexpr int kRouterTok = 4;        // tokens per workgroup: a weight row is read once for all of them
constexpr int kRouterMaxE = 1024;
constexpr int kRouterMaxTop = 64;

// (score, index) -> the lane pair with the larger score, the smaller index on equal scores
LK_DEVICE void wave_argmax(double& s, int& i) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const double so = __shfl_xor(s, o, 64);
    const int io = __shfl_xor(i, o, 64);
    if (so > s || (so == s && io < i)) {
      s = so;
      i = io;
    }
  }
}

// grid = ceil(T / kRouterTok); dynamic LDS: kRouterTok rows of W floats and of E scores.  The 4 waves take the experts in
// blocks of 4 (lanes stride the width), then wave w makes the choice of token w.
template <typename T>
__global__ __launch_bounds__(256) void router_topk_kernel(const T* __restrict__ h, long hs, const float* __restrict__ wr, int E, int W,
                                                          long rows, int top, int groups, int keep, float scale,
                                                          int* __restrict__ experts, float* __restrict__ weights) {
  // [kRouterTok][W] rows, then the f32 logits [kRouterTok][E], then the scores [kRouterTok][E].  The logits are f32 sums of f32
  // products; the sigmoid, the group sums and the weights are evaluated in f64: an f32 sigmoid near 1 keeps 6e-8 of absolute
  // resolution where neighbouring scores differ by less, so it would tie logits that are clearly apart
  extern __shared__ __attribute__((aligned(16))) float hrow[];
  float* zs = hrow + (long)kRouterTok * W;
  double* sc = reinterpret_cast<double*>(zs + (long)kRouterTok * E);
  const bool vec = W % 4 == 0 && reinterpret_cast<uintptr_t>(wr) % 16 == 0;
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const long t0 = (long)blockIdx.x * kRouterTok;
  for (int k = 0; k < kRouterTok; ++k) {
    const long t = t0 + k;
    for (int c = threadIdx.x; c < W; c += 256) hrow[k * W + c] = t < rows ? ldv<T>(h + t * hs + c) : 0.f;
  }
  __syncthreads();
  // a wave takes blocks of 4 experts; per pass over the width the 16 weight loads (4 experts x 4 x 16 bytes per lane) are
  // requested together and a row fragment read from LDS serves the 4 experts
  for (int eb = wv * 4; eb < E; eb += 16) {
    float acc[4][kRouterTok];
#pragma unroll
    for (int x = 0; x < 4; ++x)
#pragma unroll
      for (int k = 0; k < kRouterTok; ++k) acc[x][k] = 0.f;
    if (vec) {
      const int nv = W >> 2;
      for (int c0 = lane; c0 < nv; c0 += 256) {
        floatx4 w4[4][4];
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          const float* wrow = wr + (long)min(eb + x, E - 1) * W;
#pragma unroll
          for (int u = 0; u < 4; ++u)
            w4[x][u] = c0 + 64 * u < nv ? *reinterpret_cast<const floatx4*>(wrow + 4 * (c0 + 64 * u)) : floatx4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int c = min(c0 + 64 * u, nv - 1);   // columns past the end multiply zero weights
#pragma unroll
          for (int k = 0; k < kRouterTok; ++k) {
            const floatx4 hv = *reinterpret_cast<const floatx4*>(hrow + k * W + 4 * c);
#pragma unroll
            for (int x = 0; x < 4; ++x)
              acc[x][k] += (w4[x][u][0] * hv[0] + w4[x][u][1] * hv[1]) + (w4[x][u][2] * hv[2] + w4[x][u][3] * hv[3]);
          }
        }
      }
    } else {
      for (int c = lane; c < W; c += 64) {
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          const float w = wr[(long)min(eb + x, E - 1) * W + c];
#pragma unroll
          for (int k = 0; k < kRouterTok; ++k) acc[x][k] += w * hrow[k * W + c];
        }
      }
    }
#pragma unroll
    for (int x = 0; x < 4; ++x)
#pragma unroll
      for (int k = 0; k < kRouterTok; ++k) {
        const float z = wave_sum(acc[x][k]);
        if (lane == 0 && eb + x < E) zs[k * E + eb + x] = z;
      }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < kRouterTok * E; i += 256) sc[i] = 1.0 / (1.0 + exp(-(double)zs[i]));
  __syncthreads();
  const long t = t0 + wv;
  if (t >= rows) return;
  double* s = sc + (long)wv * E;
  const int per = E / groups;
  if (groups > 1) {
    // lane g: the sum of group g's two largest scores (at most 64 groups, checked on the host)
    double mine = -3.0;
    if (lane < groups) {
      double b1 = -1.0, b2 = -1.0;
      for (int j = 0; j < per; ++j) {
        const double v = s[lane * per + j];
        if (v > b1) { b2 = b1; b1 = v; } else if (v > b2) { b2 = v; }
      }
      mine = b1 + (per > 1 ? b2 : 0.0);
    }
    // pick the `keep` best groups; the others' scores are struck out (-1 < any sigmoid)
    bool kept = false;
    for (int r = 0; r < keep; ++r) {
      double bs = kept ? -3.0 : mine;
      int bi = lane;
      wave_argmax(bs, bi);
      if (bi == lane) kept = true;
    }
    for (int g = 0; g < groups; ++g) {
      const bool kg = __shfl((int)kept, g, 64) != 0;
      if (!kg)
        for (int j = lane; j < per; j += 64) s[g * per + j] = -1.0 - s[g * per + j];   // struck out: below every live score
    }
    __builtin_amdgcn_wave_barrier();
  }
  // top experts among the scores left: `top` rounds of a wave-wide argmax
  double chosen_s = 0.0;   // lane r holds the r-th choice
  int chosen_e = 0;
  double sum = 0.0;
  for (int r = 0; r < top; ++r) {
    double bs = -2.0;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const double v = s[e];
      if (v >= 0.0 && (v > bs || (v == bs && e < bi))) { bs = v; bi = e; }
    }
    wave_argmax(bs, bi);
    if (bi >= E) bi = 0;                       // nothing left to choose (NaN scores): keep the indices in range
    else if (lane == (bi & 63)) s[bi] = -1.0 - s[bi];
    if (lane == r) { chosen_s = bs; chosen_e = bi; }
    sum += bs;
  }
  if (lane < top) {
    experts[t * top + lane] = chosen_e;
    weights[t * top + lane] = (float)(chosen_s / (sum + 1e-20) * (double)scale);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void clamped_glu_kernel(const T* __restrict__ gu, long gs, T* __restrict__ out, long os, int F,
                                                          float limit, float alpha) {
  const long t = blockIdx.x;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < F; c += 256 * gridDim.y) {
    const float g = fminf(ldv<T>(gu + t * gs + c), limit);
    const float u = fminf(fmaxf(ldv<T>(gu + t * gs + F + c), -limit), limit);
    stv<T>(out + t * os + c, g / (1.f + expf(-alpha * g)) * (u + 1.f));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void silu_kernel(T* __restrict__ x, long xs, int n) {
  const long t = blockIdx.x;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < n; c += 256 * gridDim.y) {
    const float v = ldv<T>(x + t * xs + c);
    stv<T>(x + t * xs + c, v / (1.f + expf(-v)));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void sigmoid_mul_kernel(T* __restrict__ x, long xs, const T* __restrict__ g, long gs, int n) {
  const long t = blockIdx.x;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < n; c += 256 * gridDim.y)
    stv<T>(x + t * xs + c, ldv<T>(x + t * xs + c) / (1.f + expf(-ldv<T>(g + t * gs + c))));
}

dim3 row_grid(long rows, int n) { return dim3((unsigned)rows, (unsigned)((n + 2047) / 2048 > 0 ? (n + 2047) / 2048 : 1)); }

}  // namespace

int lk_stream_parallel_norm(float* x, const void* a, long as, const void* b, long bs, const void* y, long ys, const float* yw, int top,
                            const float* w1, const float* w2, float eps, void* o1, long o1s, void* o2, long o2s, long rows, int W,
                            int esz, hipStream_t st) {
  if (rows <= 0) return 0;
  if (W < 1 || (y && (!yw || top < 1)) || (o1 && !w1) || (o2 && !w2)) return -1;
  const auto al = [](const void* p, long stride_bytes, int vec_bytes) {
    return p == nullptr || (reinterpret_cast<uintptr_t>(p) % vec_bytes == 0 && stride_bytes % vec_bytes == 0);
  };
  const int tv = esz == 2 ? 8 : 16;
  const bool vec = W % 4 == 0 && al(x, (long)W * 4, 16) && al(w1, 0, 16) && al(w2, 0, 16) && al(a, as * (long)esz, tv) &&
                   al(b, bs * (long)esz, tv) && al(y, ys * (long)esz, tv) && al(o1, o1s * (long)esz, tv) && al(o2, o2s * (long)esz, tv);
  ParNormParams p;
  p.x = x; p.a = a; p.as = as; p.b = b; p.bs = bs; p.y = y; p.ys = ys; p.yw = yw; p.top = top; p.w1 = w1; p.w2 = w2; p.eps = eps;
  p.o1 = o1; p.o1s = o1s; p.o2 = o2; p.o2s = o2s; p.W = W;
  return esz == 2 ? par_norm_t<bf16_t>(p, rows, vec, st) : par_norm_t<float>(p, rows, vec, st);
}

int lk_router_topk(const void* h, long hs, const float* wr, int E, int W, long rows, int top, int groups, int keep, float scale,
                   int* experts, float* weights, int esz, hipStream_t st) {
  if (rows <= 0) return 0;
  if (E < 1 || E > kRouterMaxE || W < 1 || groups < 1 || groups > 64 || E % groups || keep < 1 || keep > groups || top < 1 ||
      top > kRouterMaxTop || top > (E / groups) * keep)
    return -1;
  const size_t lds = (size_t)kRouterTok * ((W + E) * sizeof(float) + E * sizeof(double));
  if (lds > 128 * 1024) return -1;
  const unsigned grid = (unsigned)((rows + kRouterTok - 1) / kRouterTok);
  if (esz == 2) {
    LK_SET_MAX_LDS(router_topk_kernel<bf16_t>, 128 * 1024);
    router_topk_kernel<bf16_t><<<grid, 256, lds, st>>>((const bf16_t*)h, hs, wr, E, W, rows, top, groups, keep, scale, experts, weights);
  } else {
    LK_SET_MAX_LDS(router_topk_kernel<float>, 128 * 1024);
    router_topk_kernel<float><<<grid, 256, lds, st>>>((const float*)h, hs, wr, E, W, rows, top, groups, keep, scale, experts, weights);
  }
  LK_CHECK_LAUNCH();
  return 0;
}

int lk_clamped_glu(const void* gu, long gs, void* out, long os, long rows, int F, float limit, float alpha, int esz, hipStream_t st) {
  if (rows <= 0 || F <= 0) return 0;
  if (esz == 2) clamped_glu_kernel<bf16_t><<<row_grid(rows, F), 256, 0, st>>>((const bf16_t*)gu, gs, (bf16_t*)out, os, F, limit, alpha);
  else clamped_glu_kernel<float><<<row_grid(rows, F), 256, 0, st>>>((const float*)gu, gs, (float*)out, os, F, limit, alpha);
  LK_CHECK_LAUNCH();
  return 0;
}

int lk_silu_(void* x, long xs, long rows, int n, int esz, hipStream_t st) {
  if (rows <= 0 || n <= 0) return 0;
  if (esz == 2) silu_kernel<bf16_t><<<row_grid(rows, n), 256, 0, st>>>((bf16_t*)x, xs, n);
  else silu_kernel<float><<<row_grid(rows, n), 256, 0, st>>>((float*)x, xs, n);
  LK_CHECK_LAUNCH();
  return 0;
}

int lk_sigmoid_mul_(void* x, long xs, const void* g, long gs, long rows, int n, int esz, hipStream_t st) {
  if (rows <= 0 || n <= 0) return 0;
  if (esz == 2) sigmoid_mul_kernel<bf16_t><<<row_grid(rows, n), 256, 0, st>>>((bf16_t*)x, xs, (const bf16_t*)g, gs, n);
  else sigmoid_mul_kernel<float><<<row_grid(rows, n), 256, 0, st>>>((float*)x, xs, (const float*)g, gs, n);
  LK_CHECK_LAUNCH();
  return 0;
}

// Post-norm f32 residual stream: the layer update
//
//   x <- LN(alpha * x + ls * y) * w + b        LN(v) = (v - mean) / sqrt(mean((v - mean)^2) + eps)
//
// in one pass over the row (the row lives in registers between the two reductions), together with the
// activation-dtype copy of the new x that the next projections read.  Beside it: the token gather that
// starts the stream, the gated tanh-GELU activation of a fused [gate | up] projection, and the mean of
// two RMS-normed branches.  Everything is f32 arithmetic; bf16 only where a value is read from or
// written for a GEMM.
#include <type_traits>

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

// one workgroup per token: x f32 [T, W] = row * scale and (copy != null) the same values in the table's dtype
template <typename T>
__global__ __launch_bounds__(256) void embed_stream_kernel(const int* __restrict__ ids, const T* __restrict__ tok, long V, int W,
                                                           float* __restrict__ x, T* __restrict__ copy, float scale) {
  const long t = blockIdx.x;
  long id = ids[t];
  id = id < 0 ? 0 : (id >= V ? V - 1 : id);
  const T* src = tok + id * W;
  for (int c = threadIdx.x; c < W; c += 256) {
    const float v = ldv<T>(src + c) * scale;
    x[t * W + c] = v;
    if (copy) stv<T>(copy + t * W + c, v);
  }
}

// One workgroup per output row; thread i owns the column groups i, i + 256, ... of V adjacent columns (MAXI
// groups at most) in registers; V = 4 (16-byte f32 accesses) when W % 4 == 0, else 1.
//   idx == null: rows of x are updated in place, `out` (may be null) receives the copy in TO;
//   idx != null: row idx[r] of x is read, nothing of x is written, out[r] receives the result.
template <typename TY, typename TO, int MAXI, int V>
__global__ __launch_bounds__(256) void stream_layernorm_kernel(float* __restrict__ x, const TY* __restrict__ y, long ys,
                                                               const float* __restrict__ ls, float alpha,
                                                               const float* __restrict__ w, const float* __restrict__ b,
                                                               float eps, const long* __restrict__ idx, TO* __restrict__ out,
                                                               long os, int W) {
  __shared__ float red[4];
  const long orow = blockIdx.x, row = idx ? idx[orow] : orow;
  float v[MAXI][V];
  float s = 0.f;
  auto ldn = [](const auto* p, float (&f)[V]) {   // V adjacent values as f32
    using E = std::remove_cv_t<std::remove_reference_t<decltype(*p)>>;
    if constexpr (V == 4 && sizeof(E) == 4) {
      const floatx4 t = *reinterpret_cast<const floatx4*>(p);
#pragma unroll
      for (int e = 0; e < 4; ++e) f[e] = t[e];
    } else if constexpr (V == 4) {
      const short4_t t = *reinterpret_cast<const short4_t*>(p);
#pragma unroll
      for (int e = 0; e < 4; ++e) f[e] = bf2f((bf16_t)t[e]);
    } else {
      f[0] = ldv<E>(p);
    }
  };
#pragma unroll
  for (int i = 0; i < MAXI; ++i) {
    const int c = (threadIdx.x + 256 * i) * V;
#pragma unroll
    for (int e = 0; e < V; ++e) v[i][e] = 0.f;
    if (c < W) {
      ldn(x + row * W + c, v[i]);
      if (y) {
        float yy[V], ll[V];
        ldn(y + row * ys + c, yy);
        if (ls) ldn(ls + c, ll);
#pragma unroll
        for (int e = 0; e < V; ++e) v[i][e] = alpha * v[i][e] + (ls ? ll[e] : 1.f) * yy[e];
      }
#pragma unroll
      for (int e = 0; e < V; ++e) s += v[i][e];
    }
  }
  const float mean = block_sum<4>(s, red) / (float)W;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < MAXI; ++i) {
    if ((threadIdx.x + 256 * i) * V < W) {
#pragma unroll
      for (int e = 0; e < V; ++e) {
        v[i][e] -= mean;
        q += v[i][e] * v[i][e];
      }
    }
  }
  const float inv = 1.f / sqrtf(block_sum<4>(q, red) / (float)W + eps);
#pragma unroll
  for (int i = 0; i < MAXI; ++i) {
    const int c = (threadIdx.x + 256 * i) * V;
    if (c < W) {
      float ww[V], bb[V], r[V];
      ldn(w + c, ww);
      ldn(b + c, bb);
#pragma unroll
      for (int e = 0; e < V; ++e) r[e] = v[i][e] * inv * ww[e] + bb[e];
      if constexpr (V == 4) {
        if (!idx) *reinterpret_cast<floatx4*>(x + row * W + c) = floatx4{r[0], r[1], r[2], r[3]};
        if (out) {
          if constexpr (sizeof(TO) == 4) {
            *reinterpret_cast<floatx4*>(out + orow * os + c) = floatx4{r[0], r[1], r[2], r[3]};
          } else {
            short4_t t;
#pragma unroll
            for (int e = 0; e < 4; ++e) t[e] = (short)f2bf(r[e]);
            *reinterpret_cast<short4_t*>(out + orow * os + c) = t;
          }
        }
      } else {
        if (!idx) x[row * W + c] = r[0];
        if (out) stv<TO>(out + orow * os + c, r[0]);
      }
    }
  }
}

template <typename T, bool EXACT>
__global__ __launch_bounds__(256) void gelu_tanh_mul_kernel(const T* __restrict__ gu, long gs, T* __restrict__ out, long os, int F) {
  const long t = blockIdx.x;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < F; c += 256 * gridDim.y) {
    const float g = ldv<T>(gu + t * gs + c), u = ldv<T>(gu + t * gs + F + c);
    const float z = 0.7978845608028654f * (g + 0.044715f * g * g * g);
    float th;
    if constexpr (EXACT) th = tanhf(z);
    else th = 1.f - 2.f * __builtin_amdgcn_rcpf(1.f + __expf(2.f * z));
    stv<T>(out + t * os + c, 0.5f * g * (1.f + th) * u);
  }
}

// out f32 = 0.5 (a / rms(a) * wa + b / rms(b) * wb), one workgroup per row
template <typename T>
__global__ __launch_bounds__(256) void dual_rmsnorm_mean_kernel(const T* __restrict__ a, long as, const float* __restrict__ wa,
                                                                const T* __restrict__ b, long bs, const float* __restrict__ wb,
                                                                float eps, float* __restrict__ out, int W) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  float sa = 0.f, sb = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    const float va = ldv<T>(a + t * as + c), vb = ldv<T>(b + t * bs + c);
    sa += va * va;
    sb += vb * vb;
  }
  sa = block_sum<4>(sa, red);
  sb = block_sum<4>(sb, red);
  const float ia = 1.f / sqrtf(sa / (float)W + eps), ib = 1.f / sqrtf(sb / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += 256)
    out[t * W + c] = 0.5f * (ldv<T>(a + t * as + c) * ia * wa[c] + ldv<T>(b + t * bs + c) * ib * wb[c]);
}

template <typename TY, typename TO>
int launch_ln(float* x, const void* y, long ys, const float* ls, float alpha, const float* w, const float* b, float eps,
              const long* idx, void* out, long os, long rows, int W, hipStream_t st) {
  // 16-byte accesses need whole groups of 4 columns and rows that start on 16-byte (f32) / 8-byte (bf16) borders
  const bool vec = W % 4 == 0 && (!y || (ys % 4 == 0 && (uintptr_t)y % 16 == 0)) && (!out || (os % 4 == 0 && (uintptr_t)out % 16 == 0)) &&
                   (uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0 && (uintptr_t)b % 16 == 0 && (!ls || (uintptr_t)ls % 16 == 0);
#define LK_LN(MAXI, V)                                                                                                            \
  stream_layernorm_kernel<TY, TO, MAXI, V><<<(unsigned)rows, 256, 0, st>>>(x, (const TY*)y, ys, ls, alpha, w, b, eps, idx, (TO*)out, \
                                                                           os, W)
  if (vec) {
    if (W <= 1024) LK_LN(1, 4);
    else if (W <= 4096) LK_LN(4, 4);
    else if (W <= 16384) LK_LN(16, 4);
    else return -1;
  } else {
    if (W <= 1024) LK_LN(4, 1);
    else if (W <= 4096) LK_LN(16, 1);
    else if (W <= 16384) LK_LN(64, 1);
    else return -1;
  }
#undef LK_LN
  LK_CHECK_LAUNCH();
  return 0;
}

}  // namespace

int lk_embed_stream(const int* ids, const void* tok, long V, long T, int W, float* x, void* copy, float scale, int esz,
                    hipStream_t st) {
  if (T <= 0) return 0;
  if (esz == 2) embed_stream_kernel<bf16_t><<<(unsigned)T, 256, 0, st>>>(ids, (const bf16_t*)tok, V, W, x, (bf16_t*)copy, scale);
  else embed_stream_kernel<float><<<(unsigned)T, 256, 0, st>>>(ids, (const float*)tok, V, W, x, (float*)copy, scale);
  LK_CHECK_LAUNCH();
  return 0;
}

// y_esz: element size of y (2 or 4; ignored when y is null); out_esz: of out (ignored when out is null)
int lk_stream_layernorm(float* x, const void* y, long ys, int y_esz, const float* ls, float alpha, const float* w, const float* b,
                        float eps, const long* idx, long rows, void* out, long os, int out_esz, int W, hipStream_t st) {
  if (rows <= 0) return 0;
  if (!w || !b || (idx && !out)) return -1;
  const bool yb = y && y_esz == 2, ob = out && out_esz == 2;
  if (yb && ob) return launch_ln<bf16_t, bf16_t>(x, y, ys, ls, alpha, w, b, eps, idx, out, os, rows, W, st);
  if (yb) return launch_ln<bf16_t, float>(x, y, ys, ls, alpha, w, b, eps, idx, out, os, rows, W, st);
  if (ob) return launch_ln<float, bf16_t>(x, y, ys, ls, alpha, w, b, eps, idx, out, os, rows, W, st);
  return launch_ln<float, float>(x, y, ys, ls, alpha, w, b, eps, idx, out, os, rows, W, st);
}

int lk_gelu_tanh_mul(const void* gu, long gs, void* out, long os, long rows, int F, int esz, hipStream_t st) {
  if (rows <= 0 || F <= 0) return 0;
  dim3 grid((unsigned)rows, (unsigned)((F + 2047) / 2048));
  if (esz == 2) gelu_tanh_mul_kernel<bf16_t, false><<<grid, 256, 0, st>>>((const bf16_t*)gu, gs, (bf16_t*)out, os, F);
  else gelu_tanh_mul_kernel<float, true><<<grid, 256, 0, st>>>((const float*)gu, gs, (float*)out, os, F);
  LK_CHECK_LAUNCH();
  return 0;
}

int lk_dual_rmsnorm_mean(const void* a, long as, const float* wa, const void* b, long bs, const float* wb, float eps, float* out,
                         long rows, int W, int esz, hipStream_t st) {
  if (rows <= 0) return 0;
  if (esz == 2)
    dual_rmsnorm_mean_kernel<bf16_t><<<(unsigned)rows, 256, 0, st>>>((const bf16_t*)a, as, wa, (const bf16_t*)b, bs, wb, eps, out, W);
  else
    dual_rmsnorm_mean_kernel<float><<<(unsigned)rows, 256, 0, st>>>((const float*)a, as, wa, (const float*)b, bs, wb, eps, out, W);
  LK_CHECK_LAUNCH();
  return 0;
}

// Kernels around windowed attention with pooled blocks and latent attention (bf16 or f32 activations;
// everything between the loads and the stores is f32):
//
//   lk_stream_gated_norm  x += rms(v) w_post,  v = mean_parts(y) * sigmoid(g + b);  out = rms(x) w_next
//   lk_rms_cols           out = rms(u[:, col0 : col0 + n]) w
//   lk_rot_kv_write       rotation of adjacent pairs by position * freq[i] (cos and sin times mag) on queries (in
//                         place) and keys; a key head = [per-head part | part shared by the heads | zeros];
//                         keys and values into the paged cache K [NB, G, BS, KD], V [NB, G, VD, BS]; the cached value may
//                         be a blend (1 - b) v + b v2 with a second set of value rows
//   lk_pool_kv_write      mean key / value of every block of P positions whose last position is new in this step,
//                         read from the cache (so it is the mean of what the cache holds) and filed at the block's
//                         index b, taken as a logical position of the sequence's block table, in a second pair
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

// One workgroup per token; thread i owns the column groups i, i + 256, ... of V adjacent columns (MAXI groups at
// most) in registers through the three passes: gated value and its mean square, stream update and its mean
// square, normed copy.  V = 4: 16-byte f32 / 8-byte bf16 accesses (W % 4 == 0, aligned rows); V = 1 otherwise.
template <typename T, int MAXI, int V>
__global__ __launch_bounds__(256) void stream_gated_norm_kernel(float* __restrict__ x, const T* __restrict__ y, long ys, int parts,
                                                                const T* __restrict__ g, long gs, const float* __restrict__ gb,
                                                                const float* __restrict__ wpost, const float* __restrict__ wnext,
                                                                float eps, T* __restrict__ out, long os, int W) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  const int ng = W / V;
  const float invp = 1.f / (float)parts;
  float v[MAXI][V];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < MAXI; ++i) {
    const int c = (threadIdx.x + 256 * i) * V;
    if (threadIdx.x + 256 * i < ng) {
      float a[V], t[V], gv[V], bv[V];
      ldn<T, V>(y + row * parts * ys + c, a);
      for (int p = 1; p < parts; ++p) {
        ldn<T, V>(y + (row * parts + p) * ys + c, t);
#pragma unroll
        for (int e = 0; e < V; ++e) a[e] += t[e];
      }
      ldn<T, V>(g + row * gs + c, gv);
      ldn<float, V>(gb + c, bv);
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const float val = parts > 1 ? a[e] * invp : a[e];
        v[i][e] = val / (1.f + expf(-(gv[e] + bv[e])));
        ss += v[i][e] * v[i][e];
      }
    }
  }
  ss = block_sum<4>(ss, red);
  const float inv1 = 1.f / sqrtf(ss / (float)W + eps);
  float s2 = 0.f;
#pragma unroll
  for (int i = 0; i < MAXI; ++i) {
    const int c = (threadIdx.x + 256 * i) * V;
    if (threadIdx.x + 256 * i < ng) {
      float xv[V], wv[V];
      ldn<float, V>(x + row * W + c, xv);
      ldn<float, V>(wpost + c, wv);
#pragma unroll
      for (int e = 0; e < V; ++e) {
        v[i][e] = xv[e] + v[i][e] * inv1 * wv[e];
        s2 += v[i][e] * v[i][e];
      }
      stn<float, V>(x + row * W + c, v[i]);
    }
  }
  if (!out) return;
  s2 = block_sum<4>(s2, red);
  const float inv2 = 1.f / sqrtf(s2 / (float)W + eps);
#pragma unroll
  for (int i = 0; i < MAXI; ++i) {
    const int c = (threadIdx.x + 256 * i) * V;
    if (threadIdx.x + 256 * i < ng) {
      float wv[V], r[V];
      ldn<float, V>(wnext + c, wv);
#pragma unroll
      for (int e = 0; e < V; ++e) r[e] = v[i][e] * inv2 * wv[e];
      stn<T, V>(out + row * os + c, r);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void rms_cols_kernel(const T* __restrict__ u, long us, int n, const float* __restrict__ w, float eps,
                                                       T* __restrict__ out, long os) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  const T* src = u + row * us;
  float ss = 0.f;
  for (int c = threadIdx.x; c < n; c += 256) {
    const float v = ldv<T>(src + c);
    ss += v * v;
  }
  ss = block_sum<4>(ss, red);
  const float inv = 1.f / sqrtf(ss / (float)n + eps);
  for (int c = threadIdx.x; c < n; c += 256) stv<T>(out + row * os + c, ldv<T>(src + c) * inv * w[c]);
}

constexpr int kRotMaxHead = 256;

struct RotParams {
  void* q;
  long qs;
  int H, qdim;
  const void* k;
  long ks;
  int G, kdim;
  const void* sh;   // key part shared by the heads (null: none)
  long shs;
  int sdim;
  const void* v;
  long vs;
  int vdim;
  const void* v2;   // rows of G heads of vdim columns blended into v (null: none): cached = (1 - blend) v + blend v2
  long v2s;
  float blend;
  int rot_off, rot;  // dimensions [rot_off, rot_off + rot) of a query / key head are rotated in adjacent pairs
  const float* freq;
  float mag;
  const int* positions;
  void* kc;
  void* vc;
  const int* slots;
  int BS, KD, VD;
};

// One workgroup per token; its 4 waves take the H + 2 G (head, kind) jobs in turn.  The token's cos and sin
// (accurate sincosf of the f32 angle, times mag) are computed once per pair into LDS and shared by all heads.
// A head's elements and their rotation partners are in registers (up to 4 of each per lane) before anything is
// written, so the in-place q is safe.
template <typename T>
__global__ __launch_bounds__(256) void rot_kv_write_kernel(RotParams p) {
  __shared__ float scs[kRotMaxHead / 2], ssn[kRotMaxHead / 2];
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int slot = p.slots[t];
  const float pos = (float)p.positions[t];
  for (int i = threadIdx.x; i < p.rot / 2; i += 256) {
    float sn, cs;
    sincosf(pos * p.freq[i], &sn, &cs);
    scs[i] = cs * p.mag;
    ssn[i] = sn * p.mag;
  }
  __syncthreads();
  const long blk = slot >= 0 ? slot / p.BS : 0;
  const int off = slot >= 0 ? slot % p.BS : 0;
  const T* krow = reinterpret_cast<const T*>(p.k) + t * p.ks;
  const T* shrow = p.sh ? reinterpret_cast<const T*>(p.sh) + t * p.shs : nullptr;
  for (int job = w; job < p.H + 2 * p.G; job += 4) {
    if (job < p.H + p.G) {
      const bool isq = job < p.H;
      if (!isq && slot < 0) continue;
      const int hd = isq ? p.qdim : p.KD;   // columns written
      const int kh = job - p.H;
      T* qrow = reinterpret_cast<T*>(p.q) + t * p.qs + (long)job * p.qdim;
      auto src = [&](int c) -> float {
        if (isq) return ldv<T>(qrow + c);
        if (c < p.kdim) return ldv<T>(krow + (long)kh * p.kdim + c);
        if (c < p.kdim + p.sdim) return ldv<T>(shrow + (c - p.kdim));
        return 0.f;
      };
      float own[4], par[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = lane + 64 * i;
        own[i] = par[i] = 0.f;
        if (c < hd) {
          own[i] = src(c);
          const int r = c - p.rot_off;
          if (r >= 0 && r < p.rot) par[i] = src((r & 1) ? c - 1 : c + 1);
        }
      }
      T* dst = isq ? qrow : reinterpret_cast<T*>(p.kc) + ((blk * p.G + kh) * p.BS + off) * p.KD;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = lane + 64 * i;
        if (c < hd) {
          float y = own[i];
          const int r = c - p.rot_off;
          if (r >= 0 && r < p.rot) {
            const float sn = ssn[r >> 1], cs = scs[r >> 1];
            y = (r & 1) ? own[i] * cs + par[i] * sn : own[i] * cs - par[i] * sn;
          }
          stv<T>(dst + c, y);
        }
      }
    } else if (slot >= 0) {
      const int gh = job - p.H - p.G;
      const T* x = reinterpret_cast<const T*>(p.v) + t * p.vs + (long)gh * p.vdim;
      const T* x2 = p.v2 ? reinterpret_cast<const T*>(p.v2) + t * p.v2s + (long)gh * p.vdim : nullptr;
      T* dst = reinterpret_cast<T*>(p.vc) + (blk * p.G + gh) * (long)p.VD * p.BS + off;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = lane + 64 * i;
        if (c < p.VD) {
          float val = c < p.vdim ? ldv<T>(x + c) : 0.f;
          if (x2 && c < p.vdim) val = (1.f - p.blend) * val + p.blend * ldv<T>(x2 + c);
          stv<T>(dst + (long)c * p.BS, val);
        }
      }
    }
  }
}

// grid (blocks a sequence may complete in this step, G, sequences).  Sequence s holds ctx cached tokens, the last
// qlen of them new: the blocks past / P .. ctx / P - 1 end on a new position.
template <typename T>
__global__ __launch_bounds__(256) void pool_kv_write_kernel(const T* __restrict__ kc, const T* __restrict__ vc, T* __restrict__ pkc,
                                                            T* __restrict__ pvc, int P, const int* __restrict__ bt, int bt_stride,
                                                            const int* __restrict__ ctx_lens, const int* __restrict__ cu_q,
                                                            const int* __restrict__ slots, int row0, int G, int BS, int dim,
                                                            int vdim) {
  const int s = blockIdx.z, g = blockIdx.y;
  const int first = cu_q ? cu_q[s] : s, qlen = cu_q ? cu_q[s + 1] - first : 1;
  if (qlen <= 0 || slots[row0 + first] < 0) return;
  const int ctx = ctx_lens[s], past = ctx - qlen;
  const int b = past / P + blockIdx.x;
  if (b >= ctx / P) return;
  const int* tb = bt + (long)s * bt_stride;
  const float invp = 1.f / (float)P;
  const long dblk = tb[b / BS];
  const int doff = b % BS;
  for (int d = threadIdx.x; d < dim + vdim; d += 256) {
    float acc = 0.f;
    if (d < dim) {
      for (int i = 0; i < P; ++i) {
        const int pos = b * P + i;
        acc += ldv<T>(kc + (((long)tb[pos / BS] * G + g) * BS + pos % BS) * dim + d);
      }
      stv<T>(pkc + ((dblk * G + g) * BS + doff) * dim + d, acc * invp);
    } else {
      const int dv = d - dim;
      for (int i = 0; i < P; ++i) {
        const int pos = b * P + i;
        acc += ldv<T>(vc + (((long)tb[pos / BS] * G + g) * vdim + dv) * BS + pos % BS);
      }
      stv<T>(pvc + ((dblk * G + g) * vdim + dv) * BS + doff, acc * invp);
    }
  }
}

template <typename T>
int gated_norm_t(float* x, const void* y, long ys, int parts, const void* g, long gs, const float* gb, const float* wpost,
                 const float* wnext, float eps, void* out, long os, long rows, int W, bool vec, hipStream_t st) {
  const T* yp = reinterpret_cast<const T*>(y);
  const T* gp = reinterpret_cast<const T*>(g);
  T* op = reinterpret_cast<T*>(out);
  if (vec && W <= 4 * 256 * 8)
    stream_gated_norm_kernel<T, 8, 4><<<(unsigned)rows, 256, 0, st>>>(x, yp, ys, parts, gp, gs, gb, wpost, wnext, eps, op, os, W);
  else if (W <= 256 * 16)
    stream_gated_norm_kernel<T, 16, 1><<<(unsigned)rows, 256, 0, st>>>(x, yp, ys, parts, gp, gs, gb, wpost, wnext, eps, op, os, W);
  else
    return -1;
  LK_CHECK_LAUNCH();
  return 0;
}

}  // namespace

int lk_stream_gated_norm(float* x, const void* y, long ys, int parts, const void* g, long gs, const float* gb, const float* wpost,
                         const float* wnext, float eps, void* out, long os, long rows, int W, int esz, hipStream_t st) {
  if (rows <= 0) return 0;
  if (parts < 1 || W < 1 || !y || !g || !gb || !wpost || (out && !wnext)) return -1;
  const auto al = [](const void* p, long stride_bytes, int vec_bytes) {
    return p == nullptr || (reinterpret_cast<uintptr_t>(p) % vec_bytes == 0 && stride_bytes % vec_bytes == 0);
  };
  const int tv = esz == 2 ? 8 : 16;
  const bool vec = W % 4 == 0 && al(x, (long)W * 4, 16) && al(gb, 0, 16) && al(wpost, 0, 16) && al(wnext, 0, 16) &&
                   al(y, ys * (long)esz, tv) && al(g, gs * (long)esz, tv) && al(out, os * (long)esz, tv);
  return esz == 2 ? gated_norm_t<bf16_t>(x, y, ys, parts, g, gs, gb, wpost, wnext, eps, out, os, rows, W, vec, st)
                  : gated_norm_t<float>(x, y, ys, parts, g, gs, gb, wpost, wnext, eps, out, os, rows, W, vec, st);
}

int lk_rms_cols(const void* u, long us, int n, const float* w, float eps, void* out, long os, long rows, int esz, hipStream_t st) {
  if (rows <= 0) return 0;
  if (n < 1 || !w) return -1;
  if (esz == 2) rms_cols_kernel<bf16_t><<<(unsigned)rows, 256, 0, st>>>((const bf16_t*)u, us, n, w, eps, (bf16_t*)out, os);
  else rms_cols_kernel<float><<<(unsigned)rows, 256, 0, st>>>((const float*)u, us, n, w, eps, (float*)out, os);
  LK_CHECK_LAUNCH();
  return 0;
}

int lk_rot_kv_write(void* q, long qs, int H, int qdim, const void* k, long ks, int G, int kdim, const void* sh, long shs, int sdim,
                    const void* v, long vs, int vdim, int rot_off, int rot, const float* freq, float mag, const int* positions,
                    void* kc, void* vc, const int* slots, int BS, int KD, int VD, long T, const void* v2, long v2s, float blend, int esz,
                    hipStream_t st) {
  if (T <= 0) return 0;
  if (H < 1 || G < 1 || qdim < 1 || kdim < 0 || sdim < 0 || (sdim > 0 && !sh) || vdim < 1 || qdim > kRotMaxHead || KD > kRotMaxHead ||
      VD > kRotMaxHead || kdim + sdim > KD || kdim + sdim < 1 || vdim > VD || rot < 0 || rot % 2 || rot_off < 0 ||
      rot_off + rot > qdim || rot_off + rot > kdim + sdim || (rot > 0 && !freq) || BS < 1)
    return -1;
  RotParams p;
  p.q = q; p.qs = qs; p.H = H; p.qdim = qdim; p.k = k; p.ks = ks; p.G = G; p.kdim = kdim; p.sh = sdim > 0 ? sh : nullptr; p.shs = shs;
  p.sdim = sdim; p.v = v; p.vs = vs; p.vdim = vdim; p.rot_off = rot_off; p.rot = rot; p.freq = freq; p.mag = mag;
  p.positions = positions; p.kc = kc; p.vc = vc; p.slots = slots; p.BS = BS; p.KD = KD; p.VD = VD;
  p.v2 = v2; p.v2s = v2s; p.blend = blend;
  if (esz == 2) rot_kv_write_kernel<bf16_t><<<(unsigned)T, 256, 0, st>>>(p);
  else rot_kv_write_kernel<float><<<(unsigned)T, 256, 0, st>>>(p);
  LK_CHECK_LAUNCH();
  return 0;
}

int lk_pool_kv_write(const void* kc, const void* vc, void* pkc, void* pvc, int P, const int* bt, int bt_stride, const int* ctx_lens,
                     const int* cu_q, const int* slots, int row0, int S, int max_len, int G, int BS, int dim, int vdim, int esz,
                     hipStream_t st) {
  if (S <= 0 || max_len <= 0) return 0;
  if (P < 1 || G < 1 || BS < 1 || dim < 1 || vdim < 1 || S > 65535 || G > 65535) return -1;
  // a run of max_len new positions ends at most (max_len + P - 1) / P blocks (+ 1 when it starts inside one)
  const dim3 grid((unsigned)((max_len + P - 1) / P + 1), (unsigned)G, (unsigned)S);
  if (esz == 2)
    pool_kv_write_kernel<bf16_t><<<grid, 256, 0, st>>>((const bf16_t*)kc, (const bf16_t*)vc, (bf16_t*)pkc, (bf16_t*)pvc, P, bt, bt_stride,
                                                       ctx_lens, cu_q, slots, row0, G, BS, dim, vdim);
  else
    pool_kv_write_kernel<float><<<grid, 256, 0, st>>>((const float*)kc, (const float*)vc, (float*)pkc, (float*)pvc, P, bt, bt_stride,
                                                      ctx_lens, cu_q, slots, row0, G, BS, dim, vdim);
  LK_CHECK_LAUNCH();
  return 0;
}

// PyTorch bindings for the gfx950 kernel library (module `_C`).
// Every op validates device / dtype / shape on the host BEFORE launching: a bad
// launch shape on the GPU box can fault the device for every tenant, so nothing
// reaches a kernel unchecked.  Kernels run on PyTorch's current HIP stream, so the
// ops compose with torch.cuda.graphs (hipGraph capture) and stream semantics.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include "kernels.h"

namespace {

hipStream_t cur_stream() { return c10::hip::getCurrentHIPStream().stream(); }

#define CHECK_CUDA(x) TORCH_CHECK((x).is_cuda(), #x " must be a GPU tensor")
#define CHECK_BF16(x) TORCH_CHECK((x).scalar_type() == at::kBFloat16, #x " must be bfloat16")
#define CHECK_I32(x) TORCH_CHECK((x).scalar_type() == at::kInt, #x " must be int32")
#define CHECK_F32(x) TORCH_CHECK((x).scalar_type() == at::kFloat, #x " must be float32")
#define CHECK_LASTDIM(x) TORCH_CHECK((x).stride(-1) == 1, #x " must be contiguous in its last dim")
#define CHECK_CONTIG(x) TORCH_CHECK((x).is_contiguous(), #x " must be contiguous")
// Every launcher's return code AND the HIP launch state are checked after each op: a rejected
// launch raises here instead of returning an uninitialised output (common.h LK_CHECK_LAUNCH).
void check_rc(int rc, const char* name) {
  const hipError_t e = hipGetLastError();  // launchers that do not check their own launches
  if (rc <= kLkAttrError && rc > kLkAttrError - 1000)
    TORCH_CHECK(false, name, ": kernel dynamic-LDS attribute refused: ", hipGetErrorString((hipError_t)(kLkAttrError - rc)));
  if (rc <= kLkLaunchError && rc > kLkLaunchError - 1000)
    TORCH_CHECK(false, name, ": kernel launch failed: ", hipGetErrorString((hipError_t)(kLkLaunchError - rc)));
  TORCH_CHECK(rc == 0, name, ": unsupported shape/config (code ", rc, ")");
  TORCH_CHECK(e == hipSuccess, name, ": kernel launch failed: ", hipGetErrorString(e));
}
#define CHECK_RC(rc, name) check_rc((rc), (name))

inline bf16_t* bp(const at::Tensor& t) { return reinterpret_cast<bf16_t*>(t.data_ptr()); }
inline bf16_t* bpo(const c10::optional<at::Tensor>& t) { return t ? bp(*t) : nullptr; }
inline const int* ip(const at::Tensor& t) { return t.data_ptr<int>(); }
inline const int* ipo(const c10::optional<at::Tensor>& t) { return t ? ip(*t) : nullptr; }

// shape support of the prefill GEMM for a schedule variant (3 / 4 / 5: gemm1w.hip, 256-wide column
// tiles, 256 / 192 / 128-row tiles)
bool gemm_shape_ok(int M, int N, int K, int epi, int bn, int splits, int variant) {
  if (lk_gemm1w_bm(variant)) return bn == 256 && lk_gemm1w_supported(M, N, K, epi, splits, lk_gemm1w_bm(variant)) != 0;
  return lk_gemm_supported(M, N, K, epi, bn, splits) != 0;
}

// 16-byte alignment of every row start (vector loads)
void check_rows16(const at::Tensor& t, const char* name) {
  TORCH_CHECK(reinterpret_cast<uintptr_t>(t.data_ptr()) % 16 == 0, name, " must be 16-byte aligned");
  if (t.dim() >= 2) TORCH_CHECK((t.stride(0) * t.element_size()) % 16 == 0, name, " row stride must be a multiple of 16 bytes");
}

at::Tensor rmsnorm(const at::Tensor& x, const at::Tensor& w, double eps,
                   const c10::optional<at::Tensor>& residual, const c10::optional<at::Tensor>& out_) {
  CHECK_CUDA(x); CHECK_BF16(x); CHECK_BF16(w); CHECK_LASTDIM(x);
  TORCH_CHECK(x.dim() == 2, "x must be [T, H]");
  const long T = x.size(0);
  const int H = x.size(1);
  TORCH_CHECK(w.numel() == H && w.is_contiguous(), "weight shape");
  check_rows16(x, "x");
  at::Tensor out = out_ ? *out_ : at::empty({T, H}, x.options());
  CHECK_LASTDIM(out); check_rows16(out, "out");
  TORCH_CHECK(out.size(0) == T && out.size(1) == H, "out shape");
  long rs = 0;
  if (residual) {
    CHECK_BF16(*residual); CHECK_LASTDIM(*residual); check_rows16(*residual, "residual");
    TORCH_CHECK(residual->size(0) == T && residual->size(1) == H, "residual shape");
    rs = residual->stride(0);
  }
  int rc = lk_rmsnorm(bp(out), bpo(residual), bp(x), bp(w), T, H, (float)eps, x.stride(0),
                      out.stride(0), rs, cur_stream());
  CHECK_RC(rc, "rmsnorm");
  return out;
}

at::Tensor layernorm(const at::Tensor& x, const at::Tensor& w, const c10::optional<at::Tensor>& b,
                     double eps, const c10::optional<at::Tensor>& residual, bool write_residual) {
  CHECK_CUDA(x); CHECK_BF16(x); CHECK_BF16(w); CHECK_LASTDIM(x);
  TORCH_CHECK(x.dim() == 2, "x must be [T, H]");
  const long T = x.size(0);
  const int H = x.size(1);
  TORCH_CHECK(w.numel() == H, "weight shape");
  if (b) { CHECK_BF16(*b); TORCH_CHECK(b->numel() == H, "bias shape"); }
  check_rows16(x, "x");
  at::Tensor out = at::empty({T, H}, x.options());
  long rs = 0;
  if (residual) {
    CHECK_BF16(*residual); CHECK_LASTDIM(*residual); check_rows16(*residual, "residual");
    TORCH_CHECK(residual->size(0) == T && residual->size(1) == H, "residual shape");
    rs = residual->stride(0);
  }
  int rc = lk_layernorm(bp(out), bp(x), bpo(residual), (residual && write_residual) ? bp(*residual) : nullptr,
                        bp(w), bpo(b), T, H, (float)eps, x.stride(0), out.stride(0), rs, cur_stream());
  CHECK_RC(rc, "layernorm");
  return out;
}

at::Tensor embed_layernorm(const at::Tensor& ids, const c10::optional<at::Tensor>& pos_ids,
                           const c10::optional<at::Tensor>& type_ids, const at::Tensor& tok,
                           const c10::optional<at::Tensor>& pos, const c10::optional<at::Tensor>& typ,
                           const at::Tensor& w, const at::Tensor& b, double eps) {
  CHECK_CUDA(ids); CHECK_I32(ids); CHECK_BF16(tok); CHECK_CONTIG(tok); CHECK_CONTIG(ids);
  const long T = ids.numel();
  const int H = tok.size(1);
  if (pos) { CHECK_BF16(*pos); CHECK_CONTIG(*pos); TORCH_CHECK(pos_ids.has_value(), "pos_ids required"); CHECK_I32(*pos_ids); TORCH_CHECK(pos_ids->numel() == T, "pos_ids"); TORCH_CHECK(pos->size(1) == H, "pos table"); }
  if (typ) { CHECK_BF16(*typ); CHECK_CONTIG(*typ); TORCH_CHECK(typ->size(1) == H, "type table"); }
  if (type_ids) { CHECK_I32(*type_ids); TORCH_CHECK(type_ids->numel() == T, "type_ids"); }
  at::Tensor out = at::empty({T, H}, tok.options());
  int rc = lk_embed_layernorm(bp(out), ip(ids), ipo(pos_ids), ipo(type_ids), bp(tok), bpo(pos), bpo(typ),
                              bp(w), bp(b), T, H, (float)eps, cur_stream());
  CHECK_RC(rc, "embed_layernorm");
  return out;
}

at::Tensor silu_mul(const at::Tensor& x, const c10::optional<at::Tensor>& out_) {
  CHECK_CUDA(x); CHECK_BF16(x); CHECK_LASTDIM(x);
  TORCH_CHECK(x.dim() == 2 && x.size(1) % 2 == 0, "x must be [T, 2I]");
  check_rows16(x, "x");
  const long T = x.size(0);
  const int I = x.size(1) / 2;
  at::Tensor out = out_ ? *out_ : at::empty({T, I}, x.options());
  TORCH_CHECK(out.size(0) == T && out.size(1) == I, "out shape"); CHECK_LASTDIM(out);
  check_rows16(out, "out");
  int rc = lk_silu_mul(bp(out), bp(x), T, I, x.stride(0), out.stride(0), cur_stream());
  CHECK_RC(rc, "silu_mul");
  return out;
}

// Decode-regime linear: x [M, K] (M <= 256, row-contiguous) . w[N, K]^T -> [M, N];
// swiglu=true: w = [Wg; Wu] (2I rows) -> silu(x Wg^T) * (x Wu^T) [M, I].  Rows beyond
// 128 are processed as a second launch (the weight stream is re-read; still far
// below the library GEMM at these shapes).
at::Tensor skinny_linear(const at::Tensor& x, const at::Tensor& w, bool swiglu, int64_t splits,
                         const c10::optional<at::Tensor>& out_) {
  CHECK_CUDA(x); CHECK_BF16(x); CHECK_BF16(w); CHECK_LASTDIM(x); CHECK_CONTIG(w);
  TORCH_CHECK(x.dim() == 2 && w.dim() == 2 && x.size(1) == w.size(1), "x [M,K], w [N,K]");
  check_rows16(x, "x"); check_rows16(w, "w");
  const int M = x.size(0), K = x.size(1), N = w.size(0);
  TORCH_CHECK(M >= 1 && M <= 256, "skinny_linear: M must be in [1, 256]");
  const int n_out = swiglu ? N / 2 : N;
  at::Tensor out = out_ ? *out_ : at::empty({M, n_out}, x.options());
  CHECK_BF16(out); CHECK_LASTDIM(out); check_rows16(out, "out");
  TORCH_CHECK(out.size(0) == M && out.size(1) == n_out, "out shape");
  const int S = splits > 0 ? (int)splits : lk_skinny_splits(std::min(M, 128), N, K, swiglu);
  at::Tensor part;
  if (S > 1) part = at::empty({(long)S * std::min(M, 128) * N}, x.options().dtype(at::kFloat));
  for (int m0 = 0; m0 < M; m0 += 128) {
    const int mc = std::min(128, M - m0);
    int rc = lk_skinny_gemm(bp(x) + (long)m0 * x.stride(0), x.stride(0), bp(w), mc, N, K, S, swiglu ? 1 : 0,
                            bp(out) + (long)m0 * out.stride(0), out.stride(0),
                            S > 1 ? part.data_ptr<float>() : nullptr, cur_stream());
    CHECK_RC(rc, "skinny_linear");
  }
  return out;
}

// Weight-streaming GEMM for 64 < M <= 256 (LDS-DMA staged, csrc/skinny_gemm.hip wsgemm)
at::Tensor ws_linear(const at::Tensor& x, const at::Tensor& w, bool swiglu, int64_t bn, int64_t splits,
                     const c10::optional<at::Tensor>& out_) {
  CHECK_CUDA(x); CHECK_BF16(x); CHECK_BF16(w); CHECK_LASTDIM(x); CHECK_CONTIG(w);
  TORCH_CHECK(x.dim() == 2 && w.dim() == 2 && x.size(1) == w.size(1), "x [M,K], w [N,K]");
  check_rows16(x, "x"); check_rows16(w, "w");
  const int M = x.size(0), K = x.size(1), N = w.size(0);
  TORCH_CHECK(M >= 1 && M <= 256, "ws_linear: M must be in [1, 256]");
  const int n_out = swiglu ? N / 2 : N;
  at::Tensor out = out_ ? *out_ : at::empty({M, n_out}, x.options());
  CHECK_BF16(out); CHECK_LASTDIM(out);
  TORCH_CHECK(out.size(0) == M && out.size(1) == n_out, "out shape");
  int BN = (int)bn, S = (int)splits;
  if (BN <= 0 || S <= 0) {
    int pb = 64, ps = 1;
    lk_wsgemm_plan(M, N, K, swiglu ? 1 : 0, &pb, &ps);
    if (BN <= 0) BN = pb;
    if (S <= 0) S = ps;
  }
  at::Tensor part;
  if (S > 1) part = at::empty({(long)S * M * N}, x.options().dtype(at::kFloat));
  int rc = lk_wsgemm(bp(x), x.stride(0), bp(w), M, N, K, BN, S, swiglu ? 1 : 0, bp(out), out.stride(0),
                     S > 1 ? part.data_ptr<float>() : nullptr, cur_stream());
  CHECK_RC(rc, "ws_linear");
  return out;
}

// Decode-step fusions (split-K weight-streaming GEMM whose reduction is done by the
// consumer kernel): the partial slabs never become a bf16 tensor, one launch fewer each.
namespace {
struct WsSplit {
  int M, N, K, BN, S;
};
WsSplit ws_split(const at::Tensor& x, const at::Tensor& w, int64_t bn, int64_t splits, const char* name) {
  CHECK_CUDA(x); CHECK_BF16(x); CHECK_BF16(w); CHECK_LASTDIM(x); CHECK_CONTIG(w);
  TORCH_CHECK(x.dim() == 2 && w.dim() == 2 && x.size(1) == w.size(1), name, ": x [M,K], w [N,K]");
  check_rows16(x, "x"); check_rows16(w, "w");
  WsSplit p{(int)x.size(0), (int)w.size(0), (int)x.size(1), (int)bn, (int)splits};
  TORCH_CHECK(p.M >= 1 && p.M <= 256, name, ": M must be in [1, 256]");
  if (p.BN <= 0 || p.S <= 0) {
    int pb = 64, ps = 1;
    lk_wsgemm_plan(p.M, p.N, p.K, 0, &pb, &ps);
    if (p.BN <= 0) p.BN = pb;
    if (p.S <= 0) p.S = ps;
  }
  TORCH_CHECK(p.S >= 2, name, ": needs a split-K plan (S >= 2)");
  return p;
}
}  // namespace

// out = RMSNorm(x W^T + residual) * norm_w, residual += x W^T (bf16, in place)
at::Tensor ws_linear_rmsnorm(const at::Tensor& x, const at::Tensor& w, at::Tensor& residual,
                             const at::Tensor& norm_w, double eps, int64_t bn, int64_t splits,
                             const c10::optional<at::Tensor>& tickets) {
  const WsSplit p = ws_split(x, w, bn, splits, "ws_linear_rmsnorm");
  CHECK_CUDA(residual); CHECK_BF16(residual); CHECK_LASTDIM(residual); check_rows16(residual, "residual");
  TORCH_CHECK(residual.dim() == 2 && residual.size(0) == p.M && residual.size(1) == p.N, "residual shape");
  CHECK_BF16(norm_w); TORCH_CHECK(norm_w.numel() == p.N && norm_w.is_contiguous(), "norm weight shape");
  at::Tensor part = at::empty({(long)p.S * p.M * p.N}, x.options().dtype(at::kFloat));
  at::Tensor out = at::empty({p.M, p.N}, x.options());
  if (tickets && p.M <= 4 && (p.S == 2 || p.S == 4 || p.S == 8)) {  // reduction fused into the GEMM
    CHECK_CUDA(*tickets); CHECK_I32(*tickets); CHECK_CONTIG(*tickets);
    TORCH_CHECK(tickets->numel() >= 1, "tickets");
    int rc = lk_ws_rmsnorm_fused(bp(x), x.stride(0), bp(w), p.M, p.N, p.K, p.BN, p.S, part.data_ptr<float>(),
                                 tickets->data_ptr<int>(), bp(out), out.stride(0), bp(residual), residual.stride(0),
                                 bp(norm_w), (float)eps, cur_stream());
    CHECK_RC(rc, "ws_linear_rmsnorm (fused)");
    return out;
  }
  int rc = lk_wsgemm_part(bp(x), x.stride(0), bp(w), p.M, p.N, p.K, p.BN, p.S, part.data_ptr<float>(), cur_stream());
  CHECK_RC(rc, "ws_linear_rmsnorm (gemm)");
  rc = lk_splitk_rmsnorm(bp(out), bp(residual), part.data_ptr<float>(), p.S, bp(norm_w), p.M, p.N, (float)eps,
                         out.stride(0), residual.stride(0), cur_stream());
  CHECK_RC(rc, "ws_linear_rmsnorm (norm)");
  return out;
}

// qkv = x W^T with RoPE applied and K/V scattered into the paged cache (as rope_kv_)
at::Tensor ws_linear_rope_kv(const at::Tensor& x, const at::Tensor& w, const at::Tensor& positions,
                             const at::Tensor& cos_sin, int64_t Hq, int64_t Hkv, int64_t D,
                             const c10::optional<at::Tensor>& k_cache, const c10::optional<at::Tensor>& v_cache,
                             const c10::optional<at::Tensor>& slots, bool neox, bool write_k_inplace, int64_t bn,
                             int64_t splits, const c10::optional<at::Tensor>& tickets) {
  const WsSplit p = ws_split(x, w, bn, splits, "ws_linear_rope_kv");
  TORCH_CHECK(p.N == (Hq + 2 * Hkv) * D, "w must be the fused [(Hq + 2 Hkv) * D, K] projection");
  CHECK_I32(positions); CHECK_F32(cos_sin); CHECK_CONTIG(cos_sin); CHECK_CONTIG(positions);
  TORCH_CHECK(positions.numel() == p.M, "positions");
  TORCH_CHECK(cos_sin.dim() == 2 && cos_sin.size(1) == D, "cos_sin must be [max_pos, D]");
  int BS = 1;
  if (k_cache || v_cache) {
    TORCH_CHECK(k_cache && v_cache && slots, "k_cache, v_cache and slots go together");
    CHECK_BF16(*k_cache); CHECK_BF16(*v_cache); CHECK_CONTIG(*k_cache); CHECK_CONTIG(*v_cache);
    CHECK_I32(*slots); TORCH_CHECK(slots->numel() == p.M, "slots");
    TORCH_CHECK(k_cache->dim() == 4 && k_cache->size(1) == Hkv && k_cache->size(3) == D, "k_cache must be [NB, Hkv, BS, D]");
    TORCH_CHECK(v_cache->sizes() == k_cache->sizes(), "v_cache shape");
    BS = k_cache->size(2);
  }
  at::Tensor part = at::empty({(long)p.S * p.M * p.N}, x.options().dtype(at::kFloat));
  at::Tensor qkv = at::empty({p.M, p.N}, x.options());
  if (tickets && p.BN == D && D == 128 && (p.S == 2 || p.S == 4 || p.S == 8)) {  // reduction fused into the GEMM
    CHECK_CUDA(*tickets); CHECK_I32(*tickets); CHECK_CONTIG(*tickets);
    TORCH_CHECK(tickets->numel() >= Hq + 2 * Hkv, "tickets: one per head");
    int rc = lk_ws_rope_kv_fused(bp(x), x.stride(0), bp(w), p.M, p.K, p.BN, p.S, part.data_ptr<float>(),
                                 tickets->data_ptr<int>(), bp(qkv), qkv.stride(0), ip(positions),
                                 cos_sin.data_ptr<float>(), (int)Hq, (int)Hkv, (int)D, bpo(k_cache), bpo(v_cache),
                                 ipo(slots), BS, neox ? 1 : 0, write_k_inplace ? 1 : 0, cur_stream());
    CHECK_RC(rc, "ws_linear_rope_kv (fused)");
    return qkv;
  }
  int rc = lk_wsgemm_part(bp(x), x.stride(0), bp(w), p.M, p.N, p.K, p.BN, p.S, part.data_ptr<float>(), cur_stream());
  CHECK_RC(rc, "ws_linear_rope_kv (gemm)");
  rc = lk_splitk_rope_kv(part.data_ptr<float>(), p.S, bp(qkv), qkv.stride(0), ip(positions), cos_sin.data_ptr<float>(),
                         p.M, (int)Hq, (int)Hkv, (int)D, bpo(k_cache), bpo(v_cache), ipo(slots), BS, neox ? 1 : 0,
                         write_k_inplace ? 1 : 0, cur_stream());
  CHECK_RC(rc, "ws_linear_rope_kv (rope)");
  return qkv;
}

// Weight-streaming GEMM whose workgroups compute their own X rows first (lk_wsgemm_pro):
//   kind 1: x (written) = RMSNorm(bf16(sum of pp's slabs) + res_in) * gamma; res_out = the summed
//           residual (a tensor other than res_in)
//   kind 2: x = the paged-decode output, rows with > 1 split merged from (po, pml) first
// Returns the f32 partial slabs [S, M, N] when S > 1 (reduce == false), else the bf16 (SwiGLU)
// output.
at::Tensor ws_pro(at::Tensor& x, const at::Tensor& w, bool swiglu, int64_t bn, int64_t splits, int64_t kind,
                  bool reduce, const c10::optional<at::Tensor>& pp, const c10::optional<at::Tensor>& res_in,
                  const c10::optional<at::Tensor>& res_out, const c10::optional<at::Tensor>& gamma, double eps,
                  const c10::optional<at::Tensor>& po, const c10::optional<at::Tensor>& pml,
                  const c10::optional<at::Tensor>& ctx, int64_t split, int64_t max_splits, int64_t Hq) {
  CHECK_CUDA(x); CHECK_BF16(x); CHECK_BF16(w); CHECK_CONTIG(x); CHECK_CONTIG(w);
  TORCH_CHECK(x.dim() == 2 && w.dim() == 2 && x.size(1) == w.size(1), "ws_pro: x [M,K], w [N,K]");
  check_rows16(x, "x"); check_rows16(w, "w");
  const int M = x.size(0), K = x.size(1), N = w.size(0), S = (int)splits;
  TORCH_CHECK(M >= 1 && M <= 64 && S >= 1, "ws_pro: 1 <= M <= 64, splits >= 1");
  const int n_out = swiglu ? N / 2 : N;
  at::Tensor part, out;
  if (S > 1) part = at::empty({(long)S, M, N}, x.options().dtype(at::kFloat));
  if (kind == 0) {  // plain X: the partial slabs only (the producer of a kind-1 consumer)
    TORCH_CHECK(S > 1 && !swiglu, "ws_pro kind 0: split-K partials (splits > 1, no SwiGLU)");
    CHECK_RC(lk_wsgemm_part(bp(x), x.stride(0), bp(w), M, N, K, (int)bn, S, part.data_ptr<float>(), cur_stream()),
             "ws_pro (part)");
    return part;
  }
  if (S == 1 || reduce) out = at::empty({M, n_out}, x.options());
  const float* ppp = nullptr;
  int pS = 0;
  const bf16_t* rin = nullptr;
  bf16_t* rout = nullptr;
  long rs = 0;
  const bf16_t* g = nullptr;
  if (kind == 1) {
    TORCH_CHECK(pp && res_in && res_out && gamma, "ws_pro kind 1: pp, res_in, res_out, gamma");
    CHECK_CUDA(*pp); CHECK_F32(*pp); CHECK_CONTIG(*pp);
    TORCH_CHECK(pp->dim() == 3 && pp->size(1) == M && pp->size(2) == K, "pp must be [S, M, K]");
    CHECK_BF16(*res_in); CHECK_BF16(*res_out); CHECK_CONTIG(*res_in); CHECK_CONTIG(*res_out);
    TORCH_CHECK(res_in->size(0) == M && res_in->size(1) == K && res_out->sizes() == res_in->sizes(), "residual shapes");
    TORCH_CHECK(res_in->data_ptr() != res_out->data_ptr(), "res_out must not alias res_in");
    CHECK_BF16(*gamma); TORCH_CHECK(gamma->numel() == K && gamma->is_contiguous(), "gamma [K]");
    ppp = pp->data_ptr<float>();
    pS = pp->size(0);
    rin = bp(*res_in);
    rout = bp(*res_out);
    rs = res_in->stride(0);
    g = bp(*gamma);
  }
  const float* pop = nullptr;
  const float* pmp = nullptr;
  const int* cp = nullptr;
  int D = 0;
  if (kind == 2) {
    TORCH_CHECK(po && pml && ctx, "ws_pro kind 2: po, pml, ctx");
    CHECK_F32(*po); CHECK_F32(*pml); CHECK_CONTIG(*po); CHECK_CONTIG(*pml); CHECK_I32(*ctx); CHECK_CONTIG(*ctx);
    TORCH_CHECK(Hq > 0 && K % Hq == 0, "Hq");
    D = K / Hq;
    TORCH_CHECK(po->numel() >= (long)M * Hq * max_splits * D && pml->numel() >= (long)M * Hq * max_splits * 2 &&
                ctx->numel() >= M, "decode partials / ctx too small");
    pop = po->data_ptr<float>();
    pmp = pml->data_ptr<float>();
    cp = ctx->data_ptr<int>();
  }
  int rc = lk_wsgemm_pro((int)kind, bp(x), bp(w), M, N, K, (int)bn, S, swiglu ? 1 : 0,
                         out.defined() ? bp(out) : nullptr, out.defined() ? out.stride(0) : 0,
                         S > 1 ? part.data_ptr<float>() : nullptr, ppp, pS, rin, rout, rs, g, (float)eps, pop, pmp, cp,
                         (int)Hq, D, (int)max_splits, (int)split, cur_stream());
  CHECK_RC(rc, "ws_pro");
  return out.defined() ? out : part;
}

// rope_kv_ over the reduce of split-K QKV slabs part [S, M, N] (as ws_linear_rope_kv's second half)
at::Tensor splitk_rope_kv(const at::Tensor& part, const at::Tensor& positions, const at::Tensor& cos_sin, int64_t Hq,
                          int64_t Hkv, int64_t D, const c10::optional<at::Tensor>& k_cache,
                          const c10::optional<at::Tensor>& v_cache, const c10::optional<at::Tensor>& slots, bool neox,
                          bool write_k_inplace) {
  CHECK_CUDA(part); CHECK_F32(part); CHECK_CONTIG(part);
  TORCH_CHECK(part.dim() == 3 && part.size(2) == (Hq + 2 * Hkv) * D, "part must be [S, M, (Hq + 2 Hkv) * D]");
  const int S = part.size(0), M = part.size(1), N = part.size(2);
  CHECK_I32(positions); CHECK_F32(cos_sin); CHECK_CONTIG(cos_sin); CHECK_CONTIG(positions);
  TORCH_CHECK(positions.numel() == M, "positions");
  TORCH_CHECK(cos_sin.dim() == 2 && cos_sin.size(1) == D, "cos_sin must be [max_pos, D]");
  int BS = 1;
  if (k_cache || v_cache) {
    TORCH_CHECK(k_cache && v_cache && slots, "k_cache, v_cache and slots go together");
    CHECK_BF16(*k_cache); CHECK_BF16(*v_cache); CHECK_CONTIG(*k_cache); CHECK_CONTIG(*v_cache);
    CHECK_I32(*slots); TORCH_CHECK(slots->numel() == M, "slots");
    TORCH_CHECK(k_cache->dim() == 4 && k_cache->size(1) == Hkv && k_cache->size(3) == D, "k_cache must be [NB, Hkv, BS, D]");
    TORCH_CHECK(v_cache->sizes() == k_cache->sizes(), "v_cache shape");
    BS = k_cache->size(2);
  }
  at::Tensor qkv = at::empty({M, N}, part.options().dtype(at::kBFloat16));
  int rc = lk_splitk_rope_kv(part.data_ptr<float>(), S, bp(qkv), qkv.stride(0), ip(positions), cos_sin.data_ptr<float>(),
                             M, (int)Hq, (int)Hkv, (int)D, bpo(k_cache), bpo(v_cache), ipo(slots), BS, neox ? 1 : 0,
                             write_k_inplace ? 1 : 0, cur_stream());
  CHECK_RC(rc, "splitk_rope_kv");
  return qkv;
}

// RMSNorm(bf16(sum of part's slabs) + residual) * w, residual updated in place (lk_splitk_rmsnorm)
at::Tensor splitk_rmsnorm(const at::Tensor& part, at::Tensor& residual, const at::Tensor& w, double eps) {
  CHECK_CUDA(part); CHECK_F32(part); CHECK_CONTIG(part);
  CHECK_BF16(residual); CHECK_LASTDIM(residual); CHECK_BF16(w); check_rows16(residual, "residual");
  TORCH_CHECK(part.dim() == 3 && part.size(1) == residual.size(0) && part.size(2) == residual.size(1), "part [S, M, H]");
  const long M = residual.size(0);
  const int H = residual.size(1);
  TORCH_CHECK(w.numel() == H && w.is_contiguous(), "w [H]");
  at::Tensor out = at::empty({M, H}, residual.options());
  CHECK_RC(lk_splitk_rmsnorm(bp(out), bp(residual), part.data_ptr<float>(), part.size(0), bp(w), M, H, (float)eps,
                             out.stride(0), residual.stride(0), cur_stream()), "splitk_rmsnorm");
  return out;
}

// Decode GEMV for M <= 2 rows (csrc/gemv_decode.hip).  mode 0: returns x.w^T; 1: res += x.w^T in
// place (returns res); 2: SwiGLU over w = [Wg; Wu] (returns [M, N/2]); 3: RoPE + paged-KV write of a
// packed QKV projection (returns the qkv rows).  gamma: RMSNorm(x) * gamma is the GEMV's input.
at::Tensor gemv_decode(int64_t mode, const at::Tensor& x, const at::Tensor& w, const c10::optional<at::Tensor>& gamma,
                       double eps, const c10::optional<at::Tensor>& res, const c10::optional<at::Tensor>& positions,
                       const c10::optional<at::Tensor>& cos_sin, int64_t Hq, int64_t Hkv, int64_t D,
                       const c10::optional<at::Tensor>& k_cache, const c10::optional<at::Tensor>& v_cache,
                       const c10::optional<at::Tensor>& slots, bool neox, const c10::optional<at::Tensor>& po,
                       const c10::optional<at::Tensor>& pml, const c10::optional<at::Tensor>& ctx,
                       int64_t max_splits, int64_t split) {
  CHECK_CUDA(x); CHECK_BF16(x); CHECK_BF16(w); CHECK_LASTDIM(x); CHECK_CONTIG(w);
  TORCH_CHECK(x.dim() == 2 && w.dim() == 2 && x.size(1) == w.size(1), "gemv_decode: x [M,K], w [N,K]");
  if (po) {  // the O projection merging the paged-decode split partials of x's rows
    TORCH_CHECK(mode == 1 && pml && ctx && !gamma, "gemv_decode merge prologue: mode 1 with pml, ctx, no gamma");
    CHECK_F32(*po); CHECK_F32(*pml); CHECK_I32(*ctx); CHECK_CONTIG(*po); CHECK_CONTIG(*pml);
    TORCH_CHECK(po->dim() == 4 && po->size(0) >= x.size(0) && po->size(1) == Hq && po->size(2) == max_splits &&
                    po->size(3) == D && Hq * D == x.size(1), "po [M, Hq, max_splits, D]");
    TORCH_CHECK(pml->dim() == 4 && pml->size(0) == po->size(0) && pml->size(1) == Hq && pml->size(2) == max_splits &&
                    pml->size(3) == 2, "pml [M, Hq, max_splits, 2]");
    TORCH_CHECK(ctx->numel() >= x.size(0) && split > 0, "ctx: one per row; split > 0");
  }
  check_rows16(x, "x"); check_rows16(w, "w");
  const int M = x.size(0), K = x.size(1), N = w.size(0);
  TORCH_CHECK(lk_gemv_supported(M, N, K, (int)mode), "gemv_decode: unsupported shape M", M, " N", N, " K", K);
  if (gamma) { CHECK_BF16(*gamma); TORCH_CHECK(gamma->numel() == K && gamma->is_contiguous(), "gamma [K]"); }
  at::Tensor out;
  bf16_t* rp = nullptr;
  long ldr = 0;
  const int *pos = nullptr, *sl = nullptr;
  const float* cs = nullptr;
  bf16_t *kc = nullptr, *vc = nullptr;
  int BS = 0;
  if (mode == 0) {
    out = at::empty({M, N}, x.options());
  } else if (mode == 1) {
    TORCH_CHECK(res.has_value(), "gemv_decode mode 1: res");
    CHECK_BF16(*res); CHECK_LASTDIM(*res);
    TORCH_CHECK(res->size(0) == M && res->size(1) == N && res->stride(0) % 2 == 0, "res [M, N]");
    out = *res;
    rp = bp(*res);
    ldr = res->stride(0);
  } else if (mode == 2) {
    out = at::empty({M, N / 2}, x.options());
  } else if (mode == 3) {
    TORCH_CHECK(positions && cos_sin && slots, "gemv_decode mode 3: positions, cos_sin, slots");
    CHECK_I32(*positions); CHECK_I32(*slots); CHECK_F32(*cos_sin); CHECK_CONTIG(*cos_sin);
    TORCH_CHECK(positions->numel() >= M && slots->numel() >= M, "positions / slots: one per row");
    TORCH_CHECK(cos_sin->dim() == 2 && cos_sin->size(1) == D, "cos_sin [P, D]");
    TORCH_CHECK(N == (Hq + 2 * Hkv) * D, "qkv rows = (Hq + 2 Hkv) D");
    out = at::empty({M, N}, x.options());
    pos = ip(*positions); sl = ip(*slots); cs = cos_sin->data_ptr<float>();
    if (k_cache) {
      TORCH_CHECK(v_cache.has_value(), "k_cache without v_cache");
      CHECK_BF16(*k_cache); CHECK_BF16(*v_cache); CHECK_CONTIG(*k_cache); CHECK_CONTIG(*v_cache);
      TORCH_CHECK(k_cache->dim() == 4 && k_cache->size(1) == Hkv && k_cache->size(3) == D &&
                  v_cache->sizes() == k_cache->sizes(), "cache [blocks, Hkv, BS, D]");
      kc = bp(*k_cache); vc = bp(*v_cache); BS = k_cache->size(2);
    }
  } else {
    TORCH_CHECK(false, "gemv_decode: mode 0..3");
  }
  CHECK_RC(lk_gemv_decode((int)mode, bp(x), x.stride(0), bpo(gamma), (float)eps, bp(w), M, N, K,
                          mode == 1 ? nullptr : bp(out), mode == 1 ? 0 : out.stride(0), rp, ldr, pos, cs, (int)Hq,
                          (int)Hkv, (int)D, kc, vc, sl, BS, neox ? 1 : 0, po ? po->data_ptr<float>() : nullptr,
                          pml ? pml->data_ptr<float>() : nullptr, ctx ? ip(*ctx) : nullptr, (int)max_splits,
                          (int)split, cur_stream()),
           "gemv_decode");
  return out;
}

// Prefill / encoder-regime linear (csrc/gemm.hip): epi(x [M, K] . w[N, K]^T (+ bias)).
// epi 0 none, 1 SwiGLU (w = [Wg; Wu], out [M, N/2]), 2 bias, 3 bias+GELU(erf), 4 bias+ReLU.
at::Tensor gemm(const at::Tensor& x, const at::Tensor& w, const c10::optional<at::Tensor>& bias, int64_t epi,
                int64_t bn, const c10::optional<at::Tensor>& out_, int64_t variant, int64_t splits) {
  CHECK_CUDA(x); CHECK_BF16(x); CHECK_BF16(w); CHECK_LASTDIM(x); CHECK_CONTIG(w);
  TORCH_CHECK(x.dim() == 2 && w.dim() == 2 && x.size(1) == w.size(1), "x [M,K], w [N,K]");
  check_rows16(x, "x"); check_rows16(w, "w");
  const int M = x.size(0), K = x.size(1), N = w.size(0);
  TORCH_CHECK(gemm_shape_ok(M, N, K, (int)epi, (int)bn, (int)splits, (int)variant), "gemm: unsupported shape M", M, " N", N,
              " K", K, " epi", epi, " bn", bn, " splits", splits);
  if (epi >= 2) {
    TORCH_CHECK(bias.has_value(), "gemm: this epilogue needs a bias");
    CHECK_CUDA(*bias); CHECK_BF16(*bias); CHECK_CONTIG(*bias);
    TORCH_CHECK(bias->numel() == N && reinterpret_cast<uintptr_t>(bias->data_ptr()) % 16 == 0, "gemm: bias [N], 16-B aligned");
  }
  const int n_out = epi == 1 ? N / 2 : N;
  at::Tensor out = out_ ? *out_ : at::empty({M, n_out}, x.options());
  CHECK_BF16(out); CHECK_LASTDIM(out);
  TORCH_CHECK(out.dim() == 2 && out.size(0) == M && out.size(1) == n_out, "out shape");
  TORCH_CHECK(reinterpret_cast<uintptr_t>(out.data_ptr()) % 16 == 0 && out.stride(0) % 8 == 0, "out alignment (16 B)");
  // split-K partials: fp32 [splits, M, N] from the caching allocator (stream-ordered reuse)
  at::Tensor ws;
  if (splits > 1) ws = at::empty({splits, M, N}, x.options().dtype(at::kFloat));
  int rc = lk_gemm(bp(x), x.stride(0), bp(w), epi >= 2 ? bp(*bias) : nullptr, M, N, K, (int)epi, (int)bn, (int)variant, bp(out),
                   out.stride(0), cur_stream(), (int)splits, splits > 1 ? ws.data_ptr<float>() : nullptr);
  CHECK_RC(rc, "gemm");
  return out;
}


// The fused prefill chain (csrc/gemm.hip LkEpi): epi 0 / 1 / 7 with an optional folded-RMSNorm
// row scale from ss_in [nt, ld] f32, epi 6 (RESID) updating `resid` in place and writing the
// per-256-column partial sums of squares into ss_out [N / 256, ld].  Returns `out` (RESID: resid).
at::Tensor gemm_fused(const at::Tensor& x, const at::Tensor& w, int64_t epi, int64_t bn, const c10::optional<at::Tensor>& out_,
                      int64_t variant, int64_t splits, const c10::optional<at::Tensor>& ss_in, double eps,
                      const c10::optional<at::Tensor>& resid, const c10::optional<at::Tensor>& ss_out,
                      const c10::optional<at::Tensor>& positions, const c10::optional<at::Tensor>& cos_sin,
                      const c10::optional<at::Tensor>& slots, const c10::optional<at::Tensor>& k_cache,
                      const c10::optional<at::Tensor>& v_cache, int64_t hq, int64_t hkv, int64_t hd) {
  CHECK_CUDA(x); CHECK_BF16(x); CHECK_BF16(w); CHECK_LASTDIM(x); CHECK_CONTIG(w);
  TORCH_CHECK(x.dim() == 2 && w.dim() == 2 && x.size(1) == w.size(1), "x [M,K], w [N,K]");
  check_rows16(x, "x"); check_rows16(w, "w");
  const int M = x.size(0), K = x.size(1), N = w.size(0);
  TORCH_CHECK(epi == 0 || epi == 1 || epi == 6 || epi == 7, "gemm_fused: epi must be NONE / SWIGLU / RESID / QKV");
  TORCH_CHECK(gemm_shape_ok(M, N, K, (int)epi, (int)bn, (int)splits, (int)variant), "gemm_fused: unsupported shape M", M, " N", N,
              " K", K, " epi", epi, " bn", bn, " splits", splits);
  LkEpi ea;
  const int H = K;
  if (ss_in) {
    CHECK_CUDA(*ss_in); CHECK_F32(*ss_in); CHECK_CONTIG(*ss_in);
    TORCH_CHECK(ss_in->dim() == 2 && ss_in->size(0) >= 1 && ss_in->size(0) <= 32 && ss_in->size(1) >= M,
                "ss_in must be [nt <= 32, >= M] f32");
    ea.ss_in = ss_in->data_ptr<float>();
    ea.ss_nt = ss_in->size(0);
    ea.ss_ld = ss_in->size(1);
    ea.inv_h = 1.f / (float)H;
    ea.eps = (float)eps;
  }
  at::Tensor out;
  if (epi == 6) {
    TORCH_CHECK(resid && ss_out, "RESID needs resid and ss_out");
    CHECK_CUDA(*resid); CHECK_BF16(*resid); CHECK_LASTDIM(*resid); check_rows16(*resid, "resid");
    TORCH_CHECK(resid->dim() == 2 && resid->size(0) == M && resid->size(1) == N, "resid must be [M, N]");
    CHECK_CUDA(*ss_out); CHECK_F32(*ss_out); CHECK_CONTIG(*ss_out);
    TORCH_CHECK(ss_out->dim() == 2 && ss_out->size(0) == N / 256 && ss_out->size(1) >= M, "ss_out must be [N/256, >= M]");
    ea.resid = bp(*resid);
    ea.ldr = resid->stride(0);
    ea.ss_out = ss_out->data_ptr<float>();
    ea.ss_out_ld = ss_out->size(1);
    out = *resid;
  } else {
    const int n_out = epi == 1 ? N / 2 : N;
    out = out_ ? *out_ : at::empty({M, n_out}, x.options());
    CHECK_BF16(out); CHECK_LASTDIM(out);
    TORCH_CHECK(out.dim() == 2 && out.size(0) == M && out.size(1) == n_out, "out shape");
    TORCH_CHECK(reinterpret_cast<uintptr_t>(out.data_ptr()) % 16 == 0 && out.stride(0) % 8 == 0, "out alignment (16 B)");
  }
  if (epi == 7) {
    TORCH_CHECK(positions && cos_sin, "QKV needs positions and cos_sin");
    CHECK_I32(*positions); CHECK_CONTIG(*positions); CHECK_F32(*cos_sin); CHECK_CONTIG(*cos_sin);
    TORCH_CHECK(positions->numel() >= M, "positions [>= M]");
    TORCH_CHECK(cos_sin->dim() == 2 && cos_sin->size(1) == hd, "cos_sin [max_pos, hd]");
    TORCH_CHECK(N == (hq + 2 * hkv) * hd && hd % 16 == 0, "QKV: N must be (hq + 2 hkv) * hd");
    ea.pos = ip(*positions);
    ea.cos_sin = cos_sin->data_ptr<float>();
    ea.hq = hq; ea.hkv = hkv; ea.hd = hd;
    if (k_cache || v_cache) {
      TORCH_CHECK(k_cache && v_cache && slots, "QKV: k_cache, v_cache and slots together");
      CHECK_BF16(*k_cache); CHECK_BF16(*v_cache); CHECK_CONTIG(*k_cache); CHECK_CONTIG(*v_cache);
      CHECK_I32(*slots); CHECK_CONTIG(*slots);
      TORCH_CHECK(slots->numel() >= M, "slots [>= M]");
      TORCH_CHECK(k_cache->dim() == 4 && k_cache->size(1) == hkv && k_cache->size(3) == hd && k_cache->sizes() == v_cache->sizes(),
                  "caches [num_blocks, hkv, bs, hd]");
      ea.kc = bp(*k_cache); ea.vc = bp(*v_cache); ea.slots = ip(*slots); ea.bs = k_cache->size(2);
    }
  }
  at::Tensor ws;
  if (splits > 1) ws = at::empty({splits, M, N}, x.options().dtype(at::kFloat));
  int rc = lk_gemm(bp(x), x.stride(0), bp(w), nullptr, M, N, K, (int)epi, (int)bn, (int)variant, bp(out), out.stride(0),
                   cur_stream(), (int)splits, splits > 1 ? ws.data_ptr<float>() : nullptr, &ea);
  CHECK_RC(rc, "gemm_fused");
  return out;
}

// embedding rows from int32 ids (vocab shard [lo, lo + n_local) of a vocab-parallel table: others 0)
at::Tensor embed_rows(const at::Tensor& table, const at::Tensor& ids, int64_t lo, int64_t n_local) {
  CHECK_CUDA(table); CHECK_BF16(table); CHECK_CONTIG(table); CHECK_CUDA(ids); CHECK_I32(ids); CHECK_CONTIG(ids);
  const int strict = (lo == 0 && n_local < 0) ? 1 : 0;  // the whole table: an id outside it is an error
  if (n_local < 0) n_local = table.size(0);
  TORCH_CHECK(table.dim() == 2 && table.size(1) % 8 == 0 && n_local <= table.size(0), "table [V, H], H % 8");
  check_rows16(table, "table");
  at::Tensor out = at::empty({ids.numel(), table.size(1)}, table.options());
  CHECK_RC(lk_embed_rows(bp(out), bp(table), ip(ids), ids.numel(), table.size(1), lo, n_local, cur_stream(), strict),
           "embed_rows");
  return out;
}

// ids[dst] = prev[src] (in-flight decode inputs of a pipelined step)
void scatter_ids(at::Tensor& ids, const at::Tensor& dst, const at::Tensor& prev, const at::Tensor& src) {
  CHECK_CUDA(ids); CHECK_I32(ids); CHECK_CONTIG(ids); CHECK_I32(prev); CHECK_CONTIG(prev);
  TORCH_CHECK(dst.scalar_type() == at::kLong && src.scalar_type() == at::kLong && dst.is_contiguous() && src.is_contiguous() &&
              dst.numel() == src.numel(), "dst / src int64 of equal length");
  CHECK_RC(lk_scatter_ids(ids.data_ptr<int>(), dst.data_ptr<int64_t>(), prev.data_ptr<int>(), src.data_ptr<int64_t>(),
                          (int)dst.numel(), cur_stream()), "scatter_ids");
}

// out[r] = x[idx[r]] (bf16 rows)
at::Tensor gather_rows(const at::Tensor& x, const at::Tensor& idx) {
  CHECK_CUDA(x); CHECK_BF16(x); CHECK_LASTDIM(x); check_rows16(x, "x");
  TORCH_CHECK(x.dim() == 2 && x.size(1) % 8 == 0, "x [T, H], H % 8");
  TORCH_CHECK(idx.scalar_type() == at::kLong && idx.is_contiguous(), "idx int64");
  at::Tensor out = at::empty({idx.numel(), x.size(1)}, x.options());
  CHECK_RC(lk_gather_rows(bp(out), bp(x), x.stride(0), idx.data_ptr<int64_t>(), idx.numel(), x.size(1), cur_stream()),
           "gather_rows");
  return out;
}

int64_t gemm_streamk(int64_t mode) { return lk_gemm_streamk((int)mode); }

bool gemm_supported(int64_t M, int64_t N, int64_t K, int64_t epi, int64_t bn, int64_t splits, int64_t variant) {
  return gemm_shape_ok((int)M, (int)N, (int)K, (int)epi, (int)bn, (int)splits, (int)variant);
}

std::vector<int64_t> ws_plan(int64_t M, int64_t N, int64_t K, bool swiglu) {
  int bn = 64, s = 1;
  lk_wsgemm_plan((int)M, (int)N, (int)K, swiglu ? 1 : 0, &bn, &s);
  return {bn, s};
}

int64_t skinny_splits(int64_t M, int64_t N, int64_t K, bool swiglu) {
  return lk_skinny_splits((int)M, (int)N, (int)K, swiglu ? 1 : 0);
}

void activation_(at::Tensor& x, const c10::optional<at::Tensor>& bias, int64_t kind) {
  CHECK_CUDA(x); CHECK_BF16(x); CHECK_LASTDIM(x);
  TORCH_CHECK(x.dim() == 2, "x must be 2-D");
  check_rows16(x, "x");
  if (bias) { CHECK_BF16(*bias); TORCH_CHECK(bias->numel() == x.size(1), "bias shape"); }
  int rc = lk_activation(bp(x), bpo(bias), x.size(0), x.size(1), x.stride(0), (int)kind, cur_stream());
  CHECK_RC(rc, "activation");
}

void rope_kv_(at::Tensor& qkv, const at::Tensor& positions, const at::Tensor& cos_sin, int64_t Hq,
              int64_t Hkv, int64_t D, const c10::optional<at::Tensor>& k_cache,
              const c10::optional<at::Tensor>& v_cache, const c10::optional<at::Tensor>& slots,
              bool neox, bool write_k_inplace) {
  CHECK_CUDA(qkv); CHECK_BF16(qkv); CHECK_LASTDIM(qkv); CHECK_I32(positions); CHECK_F32(cos_sin);
  CHECK_CONTIG(cos_sin); CHECK_CONTIG(positions);
  TORCH_CHECK(qkv.dim() == 2 && qkv.size(1) >= (Hq + 2 * Hkv) * D, "qkv must be [T, >=(Hq+2Hkv)*D]");
  TORCH_CHECK(cos_sin.size(1) == D, "cos_sin must be [max_pos, D]");
  check_rows16(qkv, "qkv");
  const long T = qkv.size(0);
  TORCH_CHECK(positions.numel() == T, "positions");
  int BS = 1;
  if (k_cache || v_cache) {
    TORCH_CHECK(k_cache && v_cache && slots, "k_cache, v_cache and slots go together");
    CHECK_BF16(*k_cache); CHECK_BF16(*v_cache); CHECK_CONTIG(*k_cache); CHECK_CONTIG(*v_cache);
    CHECK_I32(*slots); TORCH_CHECK(slots->numel() == T, "slots");
    TORCH_CHECK(k_cache->dim() == 4 && k_cache->size(1) == Hkv && k_cache->size(3) == D, "k_cache must be [NB, Hkv, BS, D]");
    TORCH_CHECK(v_cache->sizes() == k_cache->sizes(), "v_cache shape");
    BS = k_cache->size(2);
  }
  int rc = lk_rope_kv(bp(qkv), qkv.stride(0), ip(positions), cos_sin.data_ptr<float>(), T, Hq, Hkv, D,
                      bpo(k_cache), bpo(v_cache), ipo(slots), BS, neox ? 1 : 0, write_k_inplace ? 1 : 0,
                      cur_stream());
  CHECK_RC(rc, "rope_kv");
}

void kv_write(const at::Tensor& k, const at::Tensor& v, at::Tensor& k_cache, at::Tensor& v_cache,
              const at::Tensor& slots) {
  CHECK_CUDA(k); CHECK_BF16(k); CHECK_BF16(v); CHECK_I32(slots);
  TORCH_CHECK(k.dim() == 3 && v.sizes() == k.sizes(), "k/v must be [T, Hkv, D]");
  TORCH_CHECK(k.stride(2) == 1 && k.stride(1) == k.size(2) && v.stride(2) == 1 && v.stride(1) == v.size(2), "k/v inner layout");
  const int Hkv = k.size(1), D = k.size(2);
  TORCH_CHECK(k_cache.dim() == 4 && k_cache.size(1) == Hkv && k_cache.size(3) == D && k_cache.is_contiguous() && v_cache.is_contiguous(), "cache layout");
  int rc = lk_kv_write(bp(k), k.stride(0), bp(v), v.stride(0), bp(k_cache), bp(v_cache), ip(slots),
                       k.size(0), Hkv, D, k_cache.size(2), cur_stream());
  CHECK_RC(rc, "kv_write");
}

int64_t decode_splits(int64_t max_context, int64_t split) { return lk_decode_splits((int)max_context, (int)split); }
int64_t decode_split_size(int64_t B, int64_t Hkv) { return lk_decode_split_size((int)B, (int)Hkv); }

// k_start: optional device int32 [1] -- keys [0, k_start) are a prefix shared by every row,
// attended separately (flash_prefill partial mode) into pp_o [B, Hq, D] / pp_ml [B, Hq, 2]
// and merged by the reduce kernel (cascade decode).
at::Tensor paged_decode(const at::Tensor& q, const at::Tensor& k_cache, const at::Tensor& v_cache,
                        const at::Tensor& block_tables, const at::Tensor& ctx_lens, int64_t max_splits,
                        int64_t split, double scale, const c10::optional<at::Tensor>& part_o,
                        const c10::optional<at::Tensor>& part_ml, const c10::optional<at::Tensor>& out_,
                        const c10::optional<at::Tensor>& k_start, const c10::optional<at::Tensor>& pp_o,
                        const c10::optional<at::Tensor>& pp_ml, const c10::optional<at::Tensor>& tickets,
                        bool reduce) {
  CHECK_CUDA(q); CHECK_BF16(q); CHECK_BF16(k_cache); CHECK_BF16(v_cache);
  CHECK_I32(block_tables); CHECK_I32(ctx_lens); CHECK_CONTIG(ctx_lens);
  TORCH_CHECK(q.dim() == 3 && q.stride(2) == 1 && q.stride(1) == q.size(2), "q must be [B, Hq, D] (row-strided)");
  const int B = q.size(0), Hq = q.size(1), D = q.size(2);
  TORCH_CHECK(k_cache.dim() == 4 && k_cache.is_contiguous() && v_cache.is_contiguous() && v_cache.sizes() == k_cache.sizes(), "cache layout");
  const int Hkv = k_cache.size(1), BS = k_cache.size(2);
  TORCH_CHECK(k_cache.size(3) == D, "head dim mismatch");
  TORCH_CHECK(block_tables.dim() == 2 && block_tables.size(0) >= B && block_tables.stride(1) == 1, "block_tables");
  TORCH_CHECK(ctx_lens.numel() >= B, "ctx_lens");
  TORCH_CHECK(split >= 32 && split <= 2048 && split % 32 == 0 && split % BS == 0, "decode split must be a multiple of 32 and of the block size, <= 2048");
  TORCH_CHECK(max_splits >= 1 && (long)(max_splits - 1) * split < (long)block_tables.size(1) * BS, "max_splits exceeds block table capacity");
  check_rows16(q, "q");
  const bool cascade = pp_o.has_value();
  TORCH_CHECK(cascade == pp_ml.has_value() && cascade == k_start.has_value(), "cascade needs k_start, pp_o and pp_ml");
  if (cascade) {
    CHECK_CUDA(*k_start); CHECK_I32(*k_start); TORCH_CHECK(k_start->numel() >= 1, "k_start");
    CHECK_F32(*pp_o); CHECK_F32(*pp_ml); CHECK_CONTIG(*pp_o); CHECK_CONTIG(*pp_ml);
    TORCH_CHECK(pp_o->numel() >= (long)B * Hq * D && pp_ml->numel() >= (long)B * Hq * 2, "prefix partials too small");
  }
  at::Tensor out = out_ ? *out_ : at::empty({B, Hq, D}, q.options());
  TORCH_CHECK(out.size(0) == B && out.size(1) == Hq && out.size(2) == D && out.stride(2) == 1 && out.stride(1) == D, "out layout");
  at::Tensor po, pm;
  const bool parts = max_splits > 1 || cascade;
  if (parts) {
    po = part_o ? *part_o : at::empty({B, Hq, max_splits, D}, q.options().dtype(at::kFloat));
    pm = part_ml ? *part_ml : at::empty({B, Hq, max_splits, 2}, q.options().dtype(at::kFloat));
    TORCH_CHECK(po.numel() >= (long)B * Hq * max_splits * D && pm.numel() >= (long)B * Hq * max_splits * 2, "partials too small");
    CHECK_F32(po); CHECK_F32(pm);
  }
  if (tickets) {  // fused split merge: one zero-initialised int32 counter per (seq, kv head)
    CHECK_CUDA(*tickets); CHECK_I32(*tickets); CHECK_CONTIG(*tickets);
    TORCH_CHECK(tickets->numel() >= (long)B * Hkv, "tickets: one counter per (sequence, kv head)");
  }
  int rc = lk_paged_decode(bp(q), q.stride(0), bp(k_cache), bp(v_cache), ip(block_tables), block_tables.stride(0),
                           ip(ctx_lens), bp(out), out.stride(0), parts ? po.data_ptr<float>() : nullptr,
                           parts ? pm.data_ptr<float>() : nullptr, B, Hq, Hkv, D, BS, (int)max_splits,
                           (int)split, (float)scale, cascade ? ip(*k_start) : nullptr,
                           cascade ? pp_o->data_ptr<float>() : nullptr, cascade ? pp_ml->data_ptr<float>() : nullptr,
                           cur_stream(), tickets ? tickets->data_ptr<int>() : nullptr, reduce ? 1 : 0);
  CHECK_RC(rc, "paged_decode");
  return out;
}

int64_t prefill_rows_per_tile(int64_t G, int64_t D) { return lk_prefill_rows_per_tile((int)G, (int)D); }

at::Tensor flash_prefill(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v,
                         const c10::optional<at::Tensor>& block_tables, const at::Tensor& cu_q,
                         const c10::optional<at::Tensor>& ctx_lens, const at::Tensor& tile_seq,
                         const at::Tensor& tile_q0, int64_t Hq, int64_t Hkv, int64_t D, double scale,
                         bool causal, const c10::optional<at::Tensor>& out_,
                         const c10::optional<at::Tensor>& part_o, const c10::optional<at::Tensor>& part_ml,
                         const c10::optional<at::Tensor>& q_past) {
  CHECK_CUDA(q); CHECK_BF16(q); CHECK_BF16(k); CHECK_BF16(v); CHECK_LASTDIM(q);
  if (q_past) {
    CHECK_I32(*q_past);
    TORCH_CHECK(q_past->numel() >= cu_q.numel() - 1, "q_past: one entry per sequence");
  }
  CHECK_I32(cu_q); CHECK_I32(tile_seq); CHECK_I32(tile_q0);
  TORCH_CHECK(q.dim() == 2 && q.size(1) >= Hq * D, "q must be [T, >=Hq*D] (head-major rows)");
  check_rows16(q, "q");
  const long T = q.size(0);
  const bool paged = block_tables.has_value();
  int BS = 0, bt_stride = 0;
  long ks = 0, vs = 0;
  if (paged) {
    CHECK_I32(*block_tables);
    TORCH_CHECK(ctx_lens.has_value(), "ctx_lens required for paged prefill");
    TORCH_CHECK(k.dim() == 4 && k.size(1) == Hkv && k.size(3) == D && k.is_contiguous() && v.is_contiguous() && v.sizes() == k.sizes(), "cache layout");
    BS = k.size(2);
    bt_stride = block_tables->stride(0);
  } else {
    TORCH_CHECK(k.dim() == 2 && v.dim() == 2 && k.size(0) == T && v.size(0) == T && k.size(1) >= Hkv * D && v.size(1) >= Hkv * D, "dense k/v must be [T, >=Hkv*D]");
    CHECK_LASTDIM(k); CHECK_LASTDIM(v); check_rows16(k, "k"); check_rows16(v, "v");
    ks = k.stride(0);
    vs = v.stride(0);
  }
  if (ctx_lens) CHECK_I32(*ctx_lens);
  TORCH_CHECK(tile_seq.numel() == tile_q0.numel(), "tile arrays");
  const bool partial = part_o.has_value();
  TORCH_CHECK(partial == part_ml.has_value(), "partial mode needs part_o and part_ml");
  if (partial) {
    CHECK_F32(*part_o); CHECK_F32(*part_ml); CHECK_CONTIG(*part_o); CHECK_CONTIG(*part_ml);
    TORCH_CHECK(part_o->numel() >= T * Hq * D && part_ml->numel() >= T * Hq * 2, "partials too small");
    TORCH_CHECK(D % 4 == 0, "partial mode needs D % 4 == 0");
  }
  at::Tensor out = out_ ? *out_ : (partial ? *part_o : at::empty({T, Hq * D}, q.options()));
  if (!partial) {
    CHECK_LASTDIM(out); check_rows16(out, "out");
    TORCH_CHECK(out.size(0) == T && out.size(1) >= Hq * D, "out shape");
  }
  int rc = lk_flash_prefill(bp(q), q.stride(0), bp(k), bp(v), ks, vs, paged ? ip(*block_tables) : nullptr,
                            bt_stride, ip(cu_q), ipo(ctx_lens), ip(tile_seq), ip(tile_q0), tile_seq.numel(),
                            partial ? nullptr : bp(out), partial ? 0 : out.stride(0), Hq, Hkv, D, BS, (float)scale,
                            causal ? 1 : 0, paged ? 1 : 0, partial ? part_o->data_ptr<float>() : nullptr,
                            partial ? part_ml->data_ptr<float>() : nullptr, ipo(q_past), cur_stream());
  CHECK_RC(rc, "flash_prefill");
  return out;
}

std::vector<at::Tensor> knn_topk(const at::Tensor& corpus, const at::Tensor& cnorm, const at::Tensor& queries,
                                 const at::Tensor& qnorm, int64_t K, bool force_fused) {
  CHECK_CUDA(corpus); CHECK_BF16(corpus); CHECK_CONTIG(corpus); CHECK_F32(cnorm); CHECK_CONTIG(cnorm);
  CHECK_BF16(queries); CHECK_CONTIG(queries); CHECK_F32(qnorm); CHECK_CONTIG(qnorm);
  TORCH_CHECK(corpus.dim() == 2 && queries.dim() == 2 && corpus.size(1) == queries.size(1), "dimension mismatch");
  const long N = corpus.size(0);
  const int D = corpus.size(1), nq = queries.size(0);
  TORCH_CHECK(cnorm.numel() == N && qnorm.numel() == nq, "norm shapes");
  TORCH_CHECK(K >= 1 && K <= 64, "K in [1, 64]");
  auto fo = corpus.options().dtype(at::kFloat);
  auto io = corpus.options().dtype(at::kInt);
  const int kk = (int)std::min<long>(K, std::max<long>(N, 1));
  // the merge kernel writes every one of the K slots of every query (-inf / -1 pads)
  if (N == 0 || nq == 0) return {at::full({nq, (long)K}, -INFINITY, fo), at::full({nq, (long)K}, -1, io)};
  at::Tensor out_s = at::empty({nq, (long)K}, fo);
  at::Tensor out_i = at::empty({nq, (long)K}, io);
  if (D % 64 == 0 && nq <= 256 && !force_fused) {
    // corpus streamed once by the LDS-DMA weight-streaming GEMM (dots in f32), then a
    // normalise + chunked top-k pass and the shared merge
    at::Tensor scores = at::empty({nq, N}, fo);
    int rc = lk_ws_scores_f32(bp(queries), D, bp(corpus), nq, N, D, scores.data_ptr<float>(), N, cur_stream());
    CHECK_RC(rc, "knn scores");
    const int nc = lk_knn_score_chunks(N);
    at::Tensor ps = at::empty({nq, nc, kk}, fo);
    at::Tensor pi = at::empty({nq, nc, kk}, io);
    rc = lk_knn_score_topk(scores.data_ptr<float>(), N, cnorm.data_ptr<float>(), qnorm.data_ptr<float>(), N, nq, kk,
                           ps.data_ptr<float>(), pi.data_ptr<int>(), cur_stream());
    CHECK_RC(rc, "knn score_topk");
    rc = lk_knn_merge(ps.data_ptr<float>(), pi.data_ptr<int>(), nq, nc * kk, (int)K, out_s.data_ptr<float>(),
                      out_i.data_ptr<int>(), cur_stream());
    CHECK_RC(rc, "knn_merge");
    return {out_s, out_i};
  }
  const int nb = lk_knn_nblocks(N);
  at::Tensor ps = at::empty({nq, nb, kk}, fo);
  at::Tensor pi = at::empty({nq, nb, kk}, io);
  int rc = lk_knn_partial(bp(corpus), cnorm.data_ptr<float>(), N, D, bp(queries), qnorm.data_ptr<float>(), nq, kk,
                          ps.data_ptr<float>(), pi.data_ptr<int>(), cur_stream());
  CHECK_RC(rc, "knn_partial");
  rc = lk_knn_merge(ps.data_ptr<float>(), pi.data_ptr<int>(), nq, nb * kk, (int)K, out_s.data_ptr<float>(),
                    out_i.data_ptr<int>(), cur_stream());
  CHECK_RC(rc, "knn_merge");
  return {out_s, out_i};
}

std::vector<at::Tensor> knn_merge(const at::Tensor& cand_s, const at::Tensor& cand_i, int64_t K) {
  CHECK_CUDA(cand_s); CHECK_F32(cand_s); CHECK_I32(cand_i); CHECK_CONTIG(cand_s); CHECK_CONTIG(cand_i);
  TORCH_CHECK(cand_s.dim() == 2 && cand_s.sizes() == cand_i.sizes(), "candidates [nq, ncand]");
  const int nq = cand_s.size(0), nc = cand_s.size(1);
  at::Tensor out_s = at::empty({nq, K}, cand_s.options());
  at::Tensor out_i = at::empty({nq, K}, cand_i.options());
  int rc = lk_knn_merge(cand_s.data_ptr<float>(), cand_i.data_ptr<int>(), nq, nc, (int)K, out_s.data_ptr<float>(),
                        out_i.data_ptr<int>(), cur_stream());
  CHECK_RC(rc, "knn_merge");
  return {out_s, out_i};
}

// out: optional destination rows [B, H] (f32 or bf16, unit last stride, 16-byte rows), e.g. a
// slice of the caller's embedding matrix; default a new f32 [B, H]
at::Tensor pool_normalize(const at::Tensor& hidden, const at::Tensor& cu, int64_t mode, bool normalize,
                          const c10::optional<at::Tensor>& out_) {
  CHECK_CUDA(hidden); CHECK_BF16(hidden); CHECK_LASTDIM(hidden); CHECK_I32(cu); CHECK_CONTIG(cu);
  check_rows16(hidden, "hidden");
  const int B = cu.numel() - 1, H = hidden.size(1);
  at::Tensor out = out_ ? *out_ : at::empty({B, H}, hidden.options().dtype(at::kFloat));
  const bool obf = out.scalar_type() == at::kBFloat16;
  TORCH_CHECK(obf || out.scalar_type() == at::kFloat, "out must be f32 or bf16");
  CHECK_CUDA(out); CHECK_LASTDIM(out); check_rows16(out, "out");
  TORCH_CHECK(out.dim() == 2 && out.size(0) == B && out.size(1) == H, "out [B, H]");
  int rc = lk_pool_normalize(bp(hidden), hidden.stride(0), ip(cu), B, H, (int)mode, normalize ? 1 : 0,
                             out.data_ptr(), out.stride(0), obf ? 1 : 0, cur_stream());
  CHECK_RC(rc, "pool_normalize");
  return out;
}

at::Tensor row_norms(const at::Tensor& x) {
  CHECK_CUDA(x); CHECK_BF16(x); CHECK_CONTIG(x);
  at::Tensor out = at::empty({x.size(0)}, x.options().dtype(at::kFloat));
  int rc = lk_row_norms(bp(x), x.size(0), x.size(1), out.data_ptr<float>(), cur_stream());
  CHECK_RC(rc, "row_norms");
  return out;
}

at::Tensor select_tokens(const at::Tensor& logits, const c10::optional<at::Tensor>& temps, int64_t seed,
                         int64_t step, const c10::optional<at::Tensor>& out_) {
  CHECK_CUDA(logits); CHECK_LASTDIM(logits);
  TORCH_CHECK(logits.dim() == 2, "logits [B, V]");
  const bool is_bf16 = logits.scalar_type() == at::kBFloat16;
  TORCH_CHECK(is_bf16 || logits.scalar_type() == at::kFloat, "logits must be bf16 or f32");
  TORCH_CHECK(logits.stride(0) % 8 == 0 && reinterpret_cast<uintptr_t>(logits.data_ptr()) % 32 == 0, "logits rows must be 32-byte aligned");
  const int B = logits.size(0), V = logits.size(1);
  if (temps) { CHECK_F32(*temps); TORCH_CHECK(temps->numel() >= B, "temps"); }
  at::Tensor out = out_ ? *out_ : at::empty({B}, logits.options().dtype(at::kInt));
  CHECK_I32(out);
  int rc = lk_select_tokens(logits.data_ptr(), is_bf16 ? 1 : 0, logits.stride(0), B, V,
                            temps ? temps->data_ptr<float>() : nullptr, (unsigned long long)seed, (int)step,
                            out.data_ptr<int>(), cur_stream());
  CHECK_RC(rc, "select_tokens");
  return out;
}

// vocab-parallel greedy (parallel/tp.py TPGroup.greedy_ids): per-row packed (value, id) keys
at::Tensor argmax_key(const at::Tensor& logits, int64_t vocab_lo) {
  CHECK_CUDA(logits); CHECK_LASTDIM(logits);
  TORCH_CHECK(logits.dim() == 2, "logits [B, V]");
  const bool is_bf16 = logits.scalar_type() == at::kBFloat16;
  TORCH_CHECK(is_bf16 || logits.scalar_type() == at::kFloat, "logits must be bf16 or f32");
  TORCH_CHECK(logits.stride(0) % 8 == 0 && reinterpret_cast<uintptr_t>(logits.data_ptr()) % 32 == 0, "logits rows must be 32-byte aligned");
  TORCH_CHECK(vocab_lo >= 0 && vocab_lo + logits.size(1) < (1ll << 31), "vocab_lo");
  const int B = logits.size(0), V = logits.size(1);
  at::Tensor keys = at::empty({B}, logits.options().dtype(at::kLong));
  int rc = lk_argmax_key(logits.data_ptr(), is_bf16 ? 1 : 0, logits.stride(0), B, V, (int)vocab_lo,
                         reinterpret_cast<long long*>(keys.data_ptr<int64_t>()), cur_stream());
  CHECK_RC(rc, "argmax_key");
  return keys;
}

at::Tensor keys_to_ids(const at::Tensor& keys) {
  CHECK_CUDA(keys); CHECK_CONTIG(keys);
  TORCH_CHECK(keys.scalar_type() == at::kLong && keys.dim() == 2, "keys [W, R] int64");
  const int W = keys.size(0), R = keys.size(1);
  at::Tensor ids = at::empty({R}, keys.options().dtype(at::kInt));
  int rc = lk_keys_to_ids(reinterpret_cast<const long long*>(keys.data_ptr<int64_t>()), W, R, ids.data_ptr<int>(), cur_stream());
  CHECK_RC(rc, "keys_to_ids");
  return ids;
}

// token selection restricted per row to an allowed id list (grammar-constrained decoding)
at::Tensor select_allowed(const at::Tensor& logits, const at::Tensor& plan, const c10::optional<at::Tensor>& temps,
                          int64_t seed, int64_t step) {
  CHECK_CUDA(logits); CHECK_LASTDIM(logits); CHECK_CUDA(plan); CHECK_I32(plan); CHECK_CONTIG(plan);
  TORCH_CHECK(logits.dim() == 2, "logits [B, V]");
  const bool is_bf16 = logits.scalar_type() == at::kBFloat16;
  TORCH_CHECK(is_bf16 || logits.scalar_type() == at::kFloat, "logits must be bf16 or f32");
  TORCH_CHECK(logits.stride(0) % 8 == 0 && reinterpret_cast<uintptr_t>(logits.data_ptr()) % 32 == 0, "logits rows must be 32-byte aligned");
  const int B = logits.size(0), V = logits.size(1);
  TORCH_CHECK(plan.numel() >= 2 * B + 1, "plan must hold [B flags | B+1 offsets | ids]");
  if (temps) { CHECK_F32(*temps); TORCH_CHECK(temps->numel() >= B, "temps"); }
  at::Tensor out = at::empty({B}, logits.options().dtype(at::kInt));
  int rc = lk_select_allowed(logits.data_ptr(), is_bf16 ? 1 : 0, logits.stride(0), B, V,
                             temps ? temps->data_ptr<float>() : nullptr, (unsigned long long)seed, (int)step,
                             plan.data_ptr<int>(), out.data_ptr<int>(), cur_stream());
  CHECK_RC(rc, "select_allowed");
  return out;
}

// Fused Ollama-default sampler (csrc/sampling.hip lk_sample): see kernels.h
at::Tensor sample(at::Tensor& logits, const at::Tensor& prm, at::Tensor& hist, at::Tensor& hist_len, int64_t seed,
                  const c10::optional<at::Tensor>& out_) {
  CHECK_CUDA(logits); CHECK_F32(logits); CHECK_LASTDIM(logits);
  TORCH_CHECK(logits.dim() == 2, "logits [B, V]");
  const int B = logits.size(0), V = logits.size(1);
  CHECK_I32(prm); CHECK_CONTIG(prm); TORCH_CHECK(prm.dim() == 2 && prm.size(0) == B && prm.size(1) == 8, "prm [B, 8]");
  CHECK_I32(hist); CHECK_CONTIG(hist); TORCH_CHECK(hist.dim() == 2, "hist [slots, W]");
  CHECK_I32(hist_len); CHECK_CONTIG(hist_len); TORCH_CHECK(hist_len.numel() == hist.size(0), "hist_len [slots]");
  TORCH_CHECK(prm.is_cuda() && hist.is_cuda() && hist_len.is_cuda(), "sampler state must be on the GPU");
  // slot ids / top_k are read by the kernel: checked here (one small D2H of the parameter rows is
  // avoided by the caller, which validates the host copy it uploads: ops.sample)
  at::Tensor out = out_ ? *out_ : at::empty({B}, logits.options().dtype(at::kInt));
  CHECK_I32(out);
  int rc = lk_sample(logits.data_ptr<float>(), logits.stride(0), B, V, ip(prm), hist.data_ptr<int>(),
                     hist_len.data_ptr<int>(), hist.size(1), (unsigned long long)seed, out.data_ptr<int>(), cur_stream());
  CHECK_RC(rc, "sample");
  return out;
}

void repeat_penalty_(at::Tensor& logits, const at::Tensor& window, const at::Tensor& penalty) {
  CHECK_CUDA(logits); CHECK_I32(window); CHECK_F32(penalty); CHECK_CONTIG(window);
  const bool is_bf16 = logits.scalar_type() == at::kBFloat16;
  TORCH_CHECK(window.dim() == 2 && window.size(0) == logits.size(0), "window [B, W]");
  int rc = lk_repeat_penalty(logits.data_ptr(), is_bf16 ? 1 : 0, logits.stride(0), logits.size(0), ip(window),
                             window.size(1), penalty.data_ptr<float>(), cur_stream());
  CHECK_RC(rc, "repeat_penalty");
}

// One-shot xGMI all-reduce state of one rank (K14): its IPC-exported staging + signal buffers
// and the peers' buffers opened in this process.  Python exchanges handles() over the TP
// control group, then calls open(); all_reduce() is hipGraph-capturable.
struct XgmiAr {
  int rank = 0, world = 1;
  size_t bytes = 0;
  void* data = nullptr;
  void* sig = nullptr;
  int* err = nullptr;
  std::vector<void*> pdata, psig;  // per rank, as mapped here
  std::vector<void*> opened;       // IPC mappings to close

  XgmiAr(int rank_, int world_, int64_t bytes_) : rank(rank_), world(world_), bytes((size_t)bytes_) {
    TORCH_CHECK(world >= 1 && world <= lk_xgmi_ar_max_ranks() && rank >= 0 && rank < world, "xgmi_ar: rank/world");
    TORCH_CHECK(bytes_ > 0 && bytes_ % 16 == 0, "xgmi_ar: staging bytes must be a positive multiple of 16");
    const size_t sig_bytes = (size_t)lk_xgmi_ar_sig_words() * sizeof(unsigned);
    // two regions of `bytes`: the staged inputs and (two-shot) the reduced slices
    TORCH_CHECK(hipMalloc(&data, 2 * bytes) == hipSuccess, "xgmi_ar: hipMalloc staging");
    TORCH_CHECK(hipExtMallocWithFlags(&sig, sig_bytes, hipDeviceMallocUncached) == hipSuccess, "xgmi_ar: signal alloc");
    TORCH_CHECK(hipMalloc(reinterpret_cast<void**>(&err), sizeof(int)) == hipSuccess, "xgmi_ar: hipMalloc err");
    TORCH_CHECK(hipMemset(sig, 0, sig_bytes) == hipSuccess && hipMemset(err, 0, sizeof(int)) == hipSuccess &&
                hipDeviceSynchronize() == hipSuccess, "xgmi_ar: init");
    pdata.assign(world, nullptr);
    psig.assign(world, nullptr);
    pdata[rank] = data;
    psig[rank] = sig;
  }
  ~XgmiAr() {
    for (void* p : opened) (void)hipIpcCloseMemHandle(p);
    if (data) (void)hipFree(data);
    if (sig) (void)hipFree(sig);
    if (err) (void)hipFree(err);
  }
  py::bytes handles() const {
    hipIpcMemHandle_t h[2];
    TORCH_CHECK(hipIpcGetMemHandle(&h[0], data) == hipSuccess, "xgmi_ar: hipIpcGetMemHandle(staging)");
    TORCH_CHECK(hipIpcGetMemHandle(&h[1], sig) == hipSuccess, "xgmi_ar: hipIpcGetMemHandle(signal)");
    return py::bytes(reinterpret_cast<const char*>(h), sizeof(h));
  }
  void open(const std::vector<py::bytes>& all) {
    TORCH_CHECK((int)all.size() == world, "xgmi_ar: one handle blob per rank");
    for (int r = 0; r < world; ++r) {
      if (r == rank) continue;
      std::string s = all[r];
      TORCH_CHECK(s.size() == 2 * sizeof(hipIpcMemHandle_t), "xgmi_ar: bad handle blob");
      hipIpcMemHandle_t h[2];
      memcpy(h, s.data(), sizeof(h));
      void *d = nullptr, *g = nullptr;
      TORCH_CHECK(hipIpcOpenMemHandle(&d, h[0], hipIpcMemLazyEnablePeerAccess) == hipSuccess,
                  "xgmi_ar: hipIpcOpenMemHandle(staging) of rank ", r);
      TORCH_CHECK(hipIpcOpenMemHandle(&g, h[1], hipIpcMemLazyEnablePeerAccess) == hipSuccess,
                  "xgmi_ar: hipIpcOpenMemHandle(signal) of rank ", r);
      opened.push_back(d);
      opened.push_back(g);
      pdata[r] = d;
      psig[r] = g;
    }
  }
  void all_reduce(const at::Tensor& in, at::Tensor& out) {
    CHECK_CUDA(in); CHECK_BF16(in); CHECK_BF16(out); CHECK_CONTIG(in); CHECK_CONTIG(out);
    TORCH_CHECK(in.numel() == out.numel(), "xgmi_ar: in/out size");
    TORCH_CHECK(in.numel() % 8 == 0 && (size_t)in.numel() * 2 <= bytes, "xgmi_ar: numel must be a multiple of 8 and fit the staging buffer");
    for (int r = 0; r < world; ++r) TORCH_CHECK(pdata[r] && psig[r], "xgmi_ar: open() not called");
    TORCH_CHECK(reinterpret_cast<uintptr_t>(in.data_ptr()) % 16 == 0 && reinterpret_cast<uintptr_t>(out.data_ptr()) % 16 == 0, "xgmi_ar: 16-B alignment");
    int rc = lk_xgmi_allreduce(reinterpret_cast<bf16_t* const*>(pdata.data()), reinterpret_cast<unsigned* const*>(psig.data()),
                               rank, world, bp(in), bp(out), in.numel(), err, cur_stream());
    CHECK_RC(rc, "xgmi_allreduce");
  }
  // out = RMSNorm(allreduce(x) + residual) * w with residual updated in place (one kernel)
  void all_reduce_rmsnorm(const at::Tensor& x, at::Tensor& residual, const at::Tensor& w, double eps, at::Tensor& out) {
    CHECK_CUDA(x); CHECK_BF16(x); CHECK_BF16(residual); CHECK_BF16(w); CHECK_BF16(out);
    CHECK_CONTIG(x); CHECK_CONTIG(residual); CHECK_CONTIG(w); CHECK_CONTIG(out);
    TORCH_CHECK(x.dim() == 2 && residual.sizes() == x.sizes() && out.sizes() == x.sizes() && w.numel() == x.size(1),
                "xgmi_ar_rmsnorm: x / residual / out [T, H], w [H]");
    TORCH_CHECK(x.size(1) % 8 == 0 && (size_t)x.numel() * 2 <= bytes, "xgmi_ar_rmsnorm: H % 8 and the staging size");
    for (int r = 0; r < world; ++r) TORCH_CHECK(pdata[r] && psig[r], "xgmi_ar: open() not called");
    int rc = lk_xgmi_allreduce_rmsnorm(reinterpret_cast<bf16_t* const*>(pdata.data()),
                                       reinterpret_cast<unsigned* const*>(psig.data()), rank, world, bp(x), bp(residual),
                                       bp(w), bp(out), (int)x.size(0), (int)x.size(1), (float)eps, err, cur_stream());
    CHECK_RC(rc, "xgmi_allreduce_rmsnorm");
  }
  // two-shot (reduce-scatter + all-gather over the peer mappings) all-reduce of x [T, H] into
  // out, or with residual / w given: residual += sum, out = RMSNorm(residual) * w
  void all_reduce2(const at::Tensor& x, at::Tensor& out, const c10::optional<at::Tensor>& residual,
                   const c10::optional<at::Tensor>& w, double eps) {
    CHECK_CUDA(x); CHECK_BF16(x); CHECK_BF16(out); CHECK_CONTIG(x); CHECK_CONTIG(out);
    TORCH_CHECK(x.dim() == 2 && out.sizes() == x.sizes() && x.size(1) % 8 == 0, "xgmi_ar2: x / out [T, H], H % 8");
    TORCH_CHECK((size_t)x.numel() * 2 <= bytes, "xgmi_ar2: message larger than the staging region");
    TORCH_CHECK(residual.has_value() == w.has_value(), "xgmi_ar2: residual and w together");
    bf16_t* rp = nullptr;
    const bf16_t* wp = nullptr;
    if (residual.has_value()) {
      CHECK_BF16((*residual)); CHECK_CONTIG((*residual)); CHECK_BF16((*w)); CHECK_CONTIG((*w));
      TORCH_CHECK(residual->sizes() == x.sizes() && w->numel() == x.size(1), "xgmi_ar2: residual [T, H], w [H]");
      rp = bp(*residual);
      wp = bp(*w);
    }
    for (int r = 0; r < world; ++r) TORCH_CHECK(pdata[r] && psig[r], "xgmi_ar: open() not called");
    TORCH_CHECK(reinterpret_cast<uintptr_t>(x.data_ptr()) % 16 == 0 && reinterpret_cast<uintptr_t>(out.data_ptr()) % 16 == 0, "xgmi_ar2: 16-B alignment");
    int rc = lk_xgmi_allreduce2(reinterpret_cast<bf16_t* const*>(pdata.data()),
                                reinterpret_cast<unsigned* const*>(psig.data()), (long)(bytes / 2), rank, world, bp(x), rp,
                                wp, bp(out), (int)x.size(0), (int)x.size(1), (float)eps, rp != nullptr, err,
                                cur_stream());
    CHECK_RC(rc, "xgmi_allreduce2");
  }
  // raw-byte all-gather (root < 0: out = world x in) or broadcast from root (out = root's in)
  void gather(const at::Tensor& in, at::Tensor& out, int64_t root) {
    CHECK_CUDA(in); CHECK_CUDA(out); CHECK_CONTIG(in); CHECK_CONTIG(out);
    const long nb = in.numel() * in.element_size();
    TORCH_CHECK(nb % 16 == 0 && (size_t)nb <= bytes, "xgmi_gather: bytes must be a multiple of 16 and fit the staging buffer");
    TORCH_CHECK(out.numel() * out.element_size() == (root < 0 ? world * nb : nb), "xgmi_gather: out size");
    TORCH_CHECK(root < world, "xgmi_gather: root");
    TORCH_CHECK(reinterpret_cast<uintptr_t>(in.data_ptr()) % 16 == 0 && reinterpret_cast<uintptr_t>(out.data_ptr()) % 16 == 0,
                "xgmi_gather: 16-B alignment");
    for (int r = 0; r < world; ++r) TORCH_CHECK(pdata[r] && psig[r], "xgmi_ar: open() not called");
    int rc = lk_xgmi_gather(reinterpret_cast<bf16_t* const*>(pdata.data()), reinterpret_cast<unsigned* const*>(psig.data()),
                            rank, world, (int)root, in.data_ptr(), out.data_ptr(), nb, err, cur_stream());
    CHECK_RC(rc, "xgmi_gather");
  }
  int64_t max_bytes() const { return (int64_t)bytes; }
  int error() const {
    int h = 0;
    TORCH_CHECK(hipMemcpy(&h, err, sizeof(int), hipMemcpyDeviceToHost) == hipSuccess, "xgmi_ar: read error word");
    return h;
  }
};

// ---------------------------------------------------------------------------------------------
// f32 residual stream, sigmoid attention, state-space mixer (bf16 or f32 activations)
int esz_of(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.scalar_type() == at::kBFloat16 || t.scalar_type() == at::kFloat, name, " must be bfloat16 or float32");
  return (int)t.element_size();
}
void same_type(const at::Tensor& a, const at::Tensor& b, const char* name) {
  TORCH_CHECK(a.scalar_type() == b.scalar_type(), name, ": dtype differs from the activations'");
}
const float* fpo(const c10::optional<at::Tensor>& t, int64_t n, const char* name) {
  if (!t) return nullptr;
  TORCH_CHECK(t->is_cuda() && t->scalar_type() == at::kFloat && t->is_contiguous() && t->numel() == n, name, " must be f32 [", n, "]");
  return t->data_ptr<float>();
}
const float* fp(const at::Tensor& t, int64_t n, const char* name) { return fpo(c10::optional<at::Tensor>(t), n, name); }

std::vector<at::Tensor> embed_pos(const at::Tensor& ids, const at::Tensor& positions, const at::Tensor& tok,
                                  const at::Tensor& pos, bool keep_copy) {
  CHECK_CUDA(ids); CHECK_I32(ids); CHECK_I32(positions); CHECK_CONTIG(ids); CHECK_CONTIG(positions);
  const int esz = esz_of(tok, "tok");
  same_type(tok, pos, "pos");
  TORCH_CHECK(tok.dim() == 2 && pos.dim() == 2 && tok.is_contiguous() && pos.is_contiguous() && tok.size(1) == pos.size(1), "tables");
  const long T = ids.numel();
  TORCH_CHECK(positions.numel() == T, "positions");
  const int W = tok.size(1);
  at::Tensor x = at::empty({T, W}, tok.options().dtype(at::kFloat));
  at::Tensor copy = keep_copy ? at::empty({T, W}, x.options()) : at::Tensor();
  CHECK_RC(lk_embed_pos(ip(ids), ip(positions), tok.data_ptr(), tok.size(0), pos.data_ptr(), pos.size(0), T, W,
                        x.data_ptr<float>(), keep_copy ? copy.data_ptr<float>() : nullptr, esz, cur_stream()), "embed_pos");
  return keep_copy ? std::vector<at::Tensor>{x, copy} : std::vector<at::Tensor>{x};
}

at::Tensor stream_rmsnorm(at::Tensor& x, const c10::optional<at::Tensor>& a, const c10::optional<at::Tensor>& a_bias,
                          const c10::optional<at::Tensor>& b,
                          const c10::optional<at::Tensor>& e, double mult, const c10::optional<at::Tensor>& w,
                          double woff, double eps, const c10::optional<at::Tensor>& idx, at::ScalarType out_dtype) {
  CHECK_CUDA(x); CHECK_F32(x); CHECK_CONTIG(x);
  TORCH_CHECK(x.dim() == 2, "x must be [T, W]");
  const long T = x.size(0);
  const int W = x.size(1);
  at::Tensor out = at::empty({idx ? idx->numel() : T, W}, x.options().dtype(out_dtype));
  const int esz = esz_of(out, "out");
  long as = 0, bs = 0;
  if (a) { CHECK_CUDA(*a); same_type(*a, out, "a"); CHECK_LASTDIM(*a); TORCH_CHECK(a->dim() == 2 && a->size(0) == T && a->size(1) == W, "a shape"); as = a->stride(0); }
  if (b) { CHECK_CUDA(*b); same_type(*b, out, "b"); CHECK_LASTDIM(*b); TORCH_CHECK(b->dim() == 2 && b->size(0) == T && b->size(1) == W, "b shape"); bs = b->stride(0); }
  if (e) { CHECK_CUDA(*e); CHECK_F32(*e); CHECK_CONTIG(*e); TORCH_CHECK(e->sizes() == x.sizes(), "e shape"); }
  if (idx) { CHECK_CUDA(*idx); TORCH_CHECK(idx->scalar_type() == at::kLong && idx->is_contiguous(), "idx must be int64"); }
  CHECK_RC(lk_stream_rmsnorm(x.data_ptr<float>(), a ? a->data_ptr() : nullptr, as, fpo(a_bias, W, "a_bias"), b ? b->data_ptr() : nullptr, bs,
                             e ? e->data_ptr<float>() : nullptr, (float)mult, fpo(w, W, "w"), (float)woff, (float)eps,
                             idx ? idx->data_ptr<int64_t>() : nullptr, out.size(0), out.data_ptr(), out.stride(0), W, esz,
                             cur_stream()), "stream_rmsnorm");
  return out;
}

at::Tensor softcap(const at::Tensor& z, double cap) {
  CHECK_CUDA(z); CHECK_LASTDIM(z);
  TORCH_CHECK(z.dim() == 2, "logits must be [R, V]");
  const int esz = esz_of(z, "logits");
  at::Tensor out = at::empty({z.size(0), z.size(1)}, z.options().dtype(at::kFloat));
  CHECK_RC(lk_softcap(z.data_ptr(), z.stride(0), (float)cap, out.data_ptr<float>(), out.stride(0), z.size(0), z.size(1), esz,
                      cur_stream()), "softcap");
  return out;
}

at::Tensor silu_mul_f32(const at::Tensor& x) {
  CHECK_CUDA(x); CHECK_F32(x); CHECK_LASTDIM(x);
  TORCH_CHECK(x.dim() == 2 && x.size(1) % 2 == 0, "x must be [T, 2 I]");
  const int I = x.size(1) / 2;
  at::Tensor out = at::empty({x.size(0), I}, x.options());
  CHECK_RC(lk_silu_mul_f32(x.data_ptr<float>(), x.stride(0), out.data_ptr<float>(), out.stride(0), x.size(0), I, cur_stream()),
           "silu_mul_f32");
  return out;
}

void check_sig_caches(const at::Tensor& act, const at::Tensor& kc, const at::Tensor& vc, int G, int dim, int vdim) {
  CHECK_CUDA(kc); CHECK_CUDA(vc); same_type(kc, act, "k_cache"); same_type(vc, act, "v_cache");
  TORCH_CHECK(kc.dim() == 4 && vc.dim() == 4 && kc.is_contiguous() && vc.is_contiguous(), "caches must be contiguous 4-d");
  TORCH_CHECK(kc.size(1) == G && kc.size(3) == dim && vc.size(0) == kc.size(0) && vc.size(1) == G && vc.size(2) == vdim &&
              vc.size(3) == kc.size(2), "cache layout: K [NB, G, BS, dim], V [NB, G, vdim, BS]");
  TORCH_CHECK(reinterpret_cast<uintptr_t>(kc.data_ptr()) % 16 == 0 && reinterpret_cast<uintptr_t>(vc.data_ptr()) % 16 == 0, "cache alignment");
}

void unitnorm_kv_write(at::Tensor& qkv, int64_t H, int64_t G, int64_t dim, int64_t vdim, int64_t norm_dim, double eps, at::Tensor& kc,
                       at::Tensor& vc, const at::Tensor& slots, const c10::optional<at::Tensor>& bias) {
  CHECK_CUDA(qkv); CHECK_LASTDIM(qkv); CHECK_I32(slots); CHECK_CONTIG(slots);
  const int esz = esz_of(qkv, "qkv");
  TORCH_CHECK(qkv.dim() == 2 && qkv.size(1) == (H + G) * dim + G * vdim, "qkv must be [T, (H + G) dim + G vdim]");
  TORCH_CHECK(slots.numel() >= qkv.size(0), "slots");
  check_sig_caches(qkv, kc, vc, G, dim, vdim);
  const int BS = kc.size(2);
  if (bias) {
    CHECK_CUDA(*bias); same_type(*bias, qkv, "bias");
    TORCH_CHECK(bias->is_contiguous() && bias->numel() == qkv.size(1), "bias must be [(H + G) dim + G vdim]");
  }
  CHECK_RC(lk_unitnorm_kv_write(qkv.data_ptr(), qkv.stride(0), qkv.size(0), H, G, dim, vdim, norm_dim, (float)eps, kc.data_ptr(),
                                vc.data_ptr(), ip(slots), BS, bias ? bias->data_ptr() : nullptr, esz, cur_stream()),
           "unitnorm_kv_write");
}

at::Tensor sigattn_prefill(const at::Tensor& q, const at::Tensor& kc, const at::Tensor& vc, const at::Tensor& bt,
                           const at::Tensor& cu_q, const at::Tensor& ctx, const at::Tensor& tile_seq,
                           const at::Tensor& tile_q0, int64_t H, int64_t G, int64_t dim, int64_t vdim, double scale,
                           const at::Tensor& r1, const at::Tensor& r2, const at::Tensor& pb, at::Tensor& out) {
  CHECK_CUDA(q); CHECK_LASTDIM(q); CHECK_LASTDIM(out); same_type(out, q, "out");
  const int esz = esz_of(q, "q");
  check_sig_caches(q, kc, vc, G, dim, vdim);
  CHECK_I32(bt); CHECK_I32(cu_q); CHECK_I32(ctx); CHECK_I32(tile_seq); CHECK_I32(tile_q0);
  CHECK_CONTIG(cu_q); CHECK_CONTIG(ctx); CHECK_CONTIG(tile_seq); CHECK_CONTIG(tile_q0);
  TORCH_CHECK(bt.dim() == 2 && bt.stride(1) == 1 && bt.size(0) >= cu_q.numel() - 1 && ctx.numel() >= cu_q.numel() - 1, "block tables / ctx");
  TORCH_CHECK(q.dim() == 2 && q.size(1) >= H * dim && out.dim() == 2 && out.size(0) >= q.size(0) && out.size(1) >= H * vdim, "q / out shape");
  TORCH_CHECK(tile_seq.numel() == tile_q0.numel(), "tiles");
  check_rows16(q, "q");
  CHECK_RC(lk_sigattn_prefill(q.data_ptr(), q.stride(0), kc.data_ptr(), vc.data_ptr(), ip(bt), bt.stride(0), ip(cu_q), ip(ctx),
                              ip(tile_seq), ip(tile_q0), tile_seq.numel(), H, G, dim, vdim, kc.size(2), (float)scale,
                              fp(r1, H, "r1"), fp(r2, H, "r2"), fp(pb, H, "pb"), out.data_ptr(), out.stride(0), esz,
                              cur_stream()), "sigattn_prefill");
  return out;
}

at::Tensor sigattn_decode(const at::Tensor& q, const at::Tensor& kc, const at::Tensor& vc, const at::Tensor& bt,
                          const at::Tensor& ctx, int64_t Z, int64_t H, int64_t G, int64_t dim, int64_t vdim, double scale,
                          const at::Tensor& r1, const at::Tensor& r2, const at::Tensor& pb, at::Tensor& out,
                          const c10::optional<at::Tensor>& part) {
  CHECK_CUDA(q); CHECK_LASTDIM(q); CHECK_LASTDIM(out); same_type(out, q, "out");
  const int esz = esz_of(q, "q");
  check_sig_caches(q, kc, vc, G, dim, vdim);
  CHECK_I32(bt); CHECK_I32(ctx); CHECK_CONTIG(ctx);
  const long B = q.size(0);
  TORCH_CHECK(bt.dim() == 2 && bt.stride(1) == 1 && bt.size(0) >= B && ctx.numel() >= B, "block tables / ctx");
  TORCH_CHECK(q.dim() == 2 && q.size(1) >= H * dim && out.dim() == 2 && out.size(0) >= B && out.size(1) >= H * vdim, "q / out shape");
  TORCH_CHECK(Z >= 1 && Z <= 65535, "splits");
  float* pp = nullptr;
  if (Z > 1) {
    TORCH_CHECK(part && part->is_cuda() && part->scalar_type() == at::kFloat && part->is_contiguous() &&
                part->numel() >= B * H * Z * vdim, "part must be f32 [B, H, Z, vdim]");
    pp = part->data_ptr<float>();
  }
  check_rows16(q, "q");
  CHECK_RC(lk_sigattn_decode(q.data_ptr(), q.stride(0), kc.data_ptr(), vc.data_ptr(), ip(bt), bt.stride(0), ip(ctx), B, Z, H, G,
                             dim, vdim, kc.size(2), (float)scale, fp(r1, H, "r1"), fp(r2, H, "r2"), fp(pb, H, "pb"),
                             out.data_ptr(), out.stride(0), pp, esz, cur_stream()), "sigattn_decode");
  return out;
}

void check_seqs(const at::Tensor& cu, const at::Tensor& slots, const at::Tensor& positions, long rows) {
  CHECK_CUDA(cu); CHECK_I32(cu); CHECK_I32(slots); CHECK_I32(positions);
  CHECK_CONTIG(cu); CHECK_CONTIG(slots); CHECK_CONTIG(positions);
  TORCH_CHECK(cu.numel() >= 2 && slots.numel() >= cu.numel() - 1 && positions.numel() >= rows, "cu / slots / positions");
}

// u: [T, >= col0 + C] rows of the input projection; the convolved channels are columns [col0, col0 + C)
at::Tensor conv_silu(const at::Tensor& u, int64_t col0, int64_t C, const at::Tensor& w, const c10::optional<at::Tensor>& bias,
                     at::Tensor& state, const at::Tensor& cu, const at::Tensor& slots, const at::Tensor& positions,
                     int64_t max_len, bool act) {
  CHECK_CUDA(u); CHECK_LASTDIM(u);
  const int esz = esz_of(u, "u");
  TORCH_CHECK(u.dim() == 2 && col0 >= 0 && col0 + C <= u.size(1), "u columns");
  TORCH_CHECK(w.dim() == 2 && w.size(0) == C, "conv weight must be [C, taps]");
  const int taps = w.size(1);
  check_seqs(cu, slots, positions, u.size(0));
  CHECK_CUDA(state); same_type(state, u, "conv state"); CHECK_CONTIG(state);
  TORCH_CHECK(state.dim() == 3 && state.size(1) == std::max(taps - 1, 1) && state.size(2) == C, "conv state must be [slots, taps - 1, C]");
  TORCH_CHECK(max_len >= 1 && max_len <= u.size(0), "max_len");
  at::Tensor out = at::empty({u.size(0), C}, u.options());
  CHECK_RC(lk_conv_silu((const char*)u.data_ptr() + col0 * esz, u.stride(0), C, taps, fp(w, C * taps, "conv weight"),
                        fpo(bias, C, "conv bias"), state.data_ptr(), ip(cu), ip(slots), ip(positions), cu.numel() - 1, max_len,
                        out.data_ptr(), out.stride(0), act ? 1 : 0, esz, cur_stream()), "conv_silu");
  return out;
}

// xbc: [T, heads P + 2 groups N] = [x | B | C] after the convolution; dt: [T, heads] view (row-strided)
at::Tensor ssm_scan(const at::Tensor& xbc, const at::Tensor& dt, int64_t heads, int64_t P, int64_t N, int64_t groups,
                    const at::Tensor& dt_bias, const at::Tensor& A_log, const at::Tensor& D, at::Tensor& state,
                    const at::Tensor& cu, const at::Tensor& slots, const at::Tensor& positions, int64_t max_len) {
  CHECK_CUDA(xbc); CHECK_LASTDIM(xbc); CHECK_LASTDIM(dt);
  const int esz = esz_of(xbc, "xbc");
  same_type(dt, xbc, "dt");
  TORCH_CHECK(xbc.dim() == 2 && xbc.size(1) == heads * P + 2 * groups * N && dt.dim() == 2 && dt.size(0) == xbc.size(0) && dt.size(1) == heads, "xbc / dt shape");
  check_seqs(cu, slots, positions, xbc.size(0));
  CHECK_CUDA(state); CHECK_F32(state); CHECK_CONTIG(state);
  TORCH_CHECK(state.dim() == 4 && state.size(1) == heads && state.size(2) == P && state.size(3) == N, "state must be f32 [slots, heads, P, N]");
  at::Tensor y = at::empty({xbc.size(0), heads * P}, xbc.options().dtype(at::kFloat));
  CHECK_RC(lk_ssm_scan(xbc.data_ptr(), xbc.stride(0), dt.data_ptr(), dt.stride(0), cu.numel() - 1, heads, P, N, groups,
                       fp(dt_bias, heads, "dt_bias"), fp(A_log, heads, "A_log"), fp(D, heads, "D"), state.data_ptr<float>(),
                       ip(cu), ip(slots), ip(positions), y.data_ptr<float>(), y.stride(0), (int)max_len, esz, cur_stream()), "ssm_scan");
  return y;
}

at::Tensor gated_group_rmsnorm(const at::Tensor& y, const at::Tensor& z, const at::Tensor& w, int64_t ngroups, double eps) {
  CHECK_CUDA(y); CHECK_F32(y); CHECK_LASTDIM(y); CHECK_CUDA(z); CHECK_LASTDIM(z);
  const int esz = esz_of(z, "z");
  TORCH_CHECK(y.dim() == 2 && z.dim() == 2 && z.size(0) == y.size(0) && z.size(1) == y.size(1), "y / z shape");
  const int inner = y.size(1);
  at::Tensor out = at::empty({y.size(0), inner}, z.options());
  CHECK_RC(lk_gated_group_rmsnorm(y.data_ptr<float>(), y.stride(0), z.data_ptr(), z.stride(0), fp(w, inner, "w"), y.size(0),
                                  inner, ngroups, (float)eps, out.data_ptr(), out.stride(0), esz, cur_stream()),
           "gated_group_rmsnorm");
  return out;
}

// ---------------------------------------------------------------------------------------------
// post-norm f32 stream, linear-state scans, softmax attention with a sink (bf16 or f32 activations)
std::vector<at::Tensor> embed_stream(const at::Tensor& ids, const at::Tensor& tok, at::ScalarType out_dtype, double scale) {
  CHECK_CUDA(ids); CHECK_I32(ids); CHECK_CONTIG(ids); CHECK_CUDA(tok); CHECK_CONTIG(tok);
  const int esz = esz_of(tok, "tok");
  TORCH_CHECK(tok.dim() == 2 && tok.scalar_type() == out_dtype, "token table must be [V, W] in the activation dtype");
  const long T = ids.numel();
  const int W = tok.size(1);
  at::Tensor x = at::empty({T, W}, tok.options().dtype(at::kFloat));
  at::Tensor copy = esz == 2 ? at::empty({T, W}, tok.options()) : x;
  CHECK_RC(lk_embed_stream(ip(ids), tok.data_ptr(), tok.size(0), T, W, x.data_ptr<float>(), esz == 2 ? copy.data_ptr() : nullptr, (float)scale, esz,
                           cur_stream()), "embed_stream");
  return {x, copy};
}

at::Tensor stream_layernorm(at::Tensor& x, const c10::optional<at::Tensor>& y, const c10::optional<at::Tensor>& ls, double alpha,
                            const at::Tensor& w, const at::Tensor& b, double eps, const c10::optional<at::Tensor>& idx,
                            at::ScalarType out_dtype) {
  CHECK_CUDA(x); CHECK_F32(x); CHECK_CONTIG(x);
  TORCH_CHECK(x.dim() == 2, "x must be [T, W]");
  TORCH_CHECK(out_dtype == at::kBFloat16 || out_dtype == at::kFloat, "out dtype");
  const long T = x.size(0);
  const int W = x.size(1);
  long ys = 0;
  int yesz = 4;
  if (y) {
    CHECK_CUDA(*y); CHECK_LASTDIM(*y);
    yesz = esz_of(*y, "y");
    TORCH_CHECK(y->dim() == 2 && y->size(0) == T && y->size(1) == W, "y shape");
    ys = y->stride(0);
  }
  if (idx) { CHECK_CUDA(*idx); TORCH_CHECK(idx->scalar_type() == at::kLong && idx->is_contiguous(), "idx must be int64"); }
  // in place: f32 activations read x itself; rows chosen by idx always go to a new tensor
  const bool copy = idx || out_dtype == at::kBFloat16;
  at::Tensor out = copy ? at::empty({idx ? idx->numel() : T, W}, x.options().dtype(out_dtype)) : x;
  CHECK_RC(lk_stream_layernorm(x.data_ptr<float>(), y ? y->data_ptr() : nullptr, ys, yesz, fpo(ls, W, "ls"), (float)alpha,
                               fp(w, W, "w"), fp(b, W, "b"), (float)eps, idx ? idx->data_ptr<int64_t>() : nullptr, out.size(0),
                               copy ? out.data_ptr() : nullptr, out.stride(0), (int)out.element_size(), W, cur_stream()),
           "stream_layernorm");
  return out;
}

at::Tensor gelu_tanh_mul(const at::Tensor& gu) {
  CHECK_CUDA(gu); CHECK_LASTDIM(gu);
  const int esz = esz_of(gu, "gu");
  TORCH_CHECK(gu.dim() == 2 && gu.size(1) % 2 == 0, "gu must be [T, 2 F]");
  const int F = gu.size(1) / 2;
  at::Tensor out = at::empty({gu.size(0), F}, gu.options());
  CHECK_RC(lk_gelu_tanh_mul(gu.data_ptr(), gu.stride(0), out.data_ptr(), out.stride(0), gu.size(0), F, esz, cur_stream()),
           "gelu_tanh_mul");
  return out;
}

at::Tensor dual_rmsnorm_mean(const at::Tensor& a, const at::Tensor& wa, const at::Tensor& b, const at::Tensor& wb, double eps) {
  CHECK_CUDA(a); CHECK_CUDA(b); CHECK_LASTDIM(a); CHECK_LASTDIM(b);
  const int esz = esz_of(a, "a");
  same_type(b, a, "b");
  TORCH_CHECK(a.dim() == 2 && b.dim() == 2 && a.sizes() == b.sizes(), "a / b shape");
  const int W = a.size(1);
  at::Tensor out = at::empty({a.size(0), W}, a.options().dtype(at::kFloat));
  CHECK_RC(lk_dual_rmsnorm_mean(a.data_ptr(), a.stride(0), fp(wa, W, "wa"), b.data_ptr(), b.stride(0), fp(wb, W, "wb"), (float)eps,
                                out.data_ptr<float>(), a.size(0), W, esz, cur_stream()), "dual_rmsnorm_mean");
  return out;
}

// rows of a 2-d tensor with at least n columns, contiguous along the row
void check_rows(const at::Tensor& t, long T, long n, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.dim() == 2 && t.size(0) == T && t.size(1) >= n && t.stride(1) == 1, name, " must be GPU rows of >= ", n);
}
const float* f32_rows(const c10::optional<at::Tensor>& t, long T, long n, const char* name, long* stride) {
  if (!t) return nullptr;
  check_rows(*t, T, n, name);
  TORCH_CHECK(t->scalar_type() == at::kFloat, name, " must be float32");
  *stride = t->stride(0);
  return t->data_ptr<float>();
}

at::Tensor delta_scan(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, const c10::optional<at::Tensor>& w,
                      const c10::optional<at::Tensor>& p, const c10::optional<at::Tensor>& z, at::Tensor& state, const at::Tensor& cu,
                      const at::Tensor& slots, const at::Tensor& positions, int64_t H, int64_t Hk, int64_t dk, int64_t dv,
                      const c10::optional<at::Tensor>& w_head, double k_scale, int64_t max_len, int64_t lanes, bool act) {
  const long T = q.size(0);
  TORCH_CHECK(H >= 1 && Hk >= 1 && H % Hk == 0 && dk >= 1 && dk <= 256 && dv >= 1, "delta_scan sizes");
  check_rows(q, T, Hk * dk, "q"); check_rows(k, T, Hk * dk, "k"); check_rows(v, T, H * dv, "v");
  const int esz = esz_of(q, "q");
  same_type(k, q, "k"); same_type(v, q, "v");
  long ws = 0, ps = 0, zs = 0;
  const float* wp = f32_rows(w, T, H * dk, "w", &ws);
  const float* pp = f32_rows(p, T, H * dk, "p", &ps);
  const float* zp = f32_rows(z, T, H * dk, "z", &zs);
  TORCH_CHECK((wp != nullptr) == (pp != nullptr) && (pp != nullptr) == (zp != nullptr), "w, p, z come together (or none, with w_head)");
  TORCH_CHECK(wp != nullptr || w_head.has_value(), "w or w_head");
  check_seqs(cu, slots, positions, T);
  CHECK_CUDA(state); CHECK_F32(state); CHECK_CONTIG(state);
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == dk && state.size(3) == dv, "state must be f32 [slots, H, dk, dv]");
  at::Tensor o = at::empty({T, H * dv}, q.options().dtype(at::kFloat));
  // few (sequence, head) pairs: 16 lanes per state column instead of 4 (a static function of the step's shape)
  const long S = cu.numel() - 1;
  // (lanes: 4 or 16 forces one of the two forms -- tests; anything else: by the step's shape)
  const int wide = lanes == 16 ? 1 : lanes == 4 ? 0 : (S * H * ((dv * 4 + 255) / 256) < 2 * 256 ? 1 : 0);
  CHECK_RC(lk_delta_scan(q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0), esz, wp, ws, pp, ps, zp, zs,
                         wp ? nullptr : fpo(w_head, H, "w_head"), (float)k_scale, state.data_ptr<float>(), ip(cu), ip(slots),
                         ip(positions), cu.numel() - 1, (int)H, (int)Hk, (int)dk, (int)dv, o.data_ptr<float>(), o.stride(0),
                         wide, act ? 1 : 0, cur_stream()), "delta_scan");
  return o;
}

std::vector<at::Tensor> gated_delta_prep(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, const at::Tensor& beta,
                                         const at::Tensor& dt, const at::Tensor& dt_bias, const at::Tensor& A_log, int64_t H,
                                         int64_t Hk, int64_t dk, int64_t dv) {
  const long T = q.size(0);
  TORCH_CHECK(H >= 1 && Hk >= 1 && H % Hk == 0, "heads");
  check_rows(q, T, Hk * dk, "q"); check_rows(k, T, Hk * dk, "k"); check_rows(v, T, H * dv, "v");
  check_rows(beta, T, H, "beta"); check_rows(dt, T, H * dk, "dt");
  const int esz = esz_of(q, "q");
  same_type(k, q, "k"); same_type(v, q, "v"); same_type(beta, q, "beta"); same_type(dt, q, "dt");
  auto f = q.options().dtype(at::kFloat);
  at::Tensor qn = at::empty({T, Hk * dk}, f), kn = at::empty({T, Hk * dk}, f), vb = at::empty({T, H * dv}, f);
  at::Tensor g = at::empty({T, H * dk}, f), p = at::empty({T, H * dk}, f), z = at::empty({T, H * dk}, f);
  CHECK_RC(lk_gated_delta_prep(q.data_ptr(), q.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0), beta.data_ptr(),
                               beta.stride(0), dt.data_ptr(), dt.stride(0), fp(dt_bias, H * dk, "dt_bias"), fp(A_log, H, "A_log"), T,
                               (int)H, (int)Hk, (int)dk, (int)dv, qn.data_ptr<float>(), kn.data_ptr<float>(), vb.data_ptr<float>(),
                               g.data_ptr<float>(), p.data_ptr<float>(), z.data_ptr<float>(), esz, cur_stream()), "gated_delta_prep");
  return {qn, kn, vb, g, p, z};
}

std::vector<at::Tensor> general_delta_prep(const at::Tensor& k, const at::Tensor& wraw, const at::Tensor& w0, const at::Tensor& araw,
                                           const at::Tensor& a_b, int64_t H, int64_t dk) {
  const long T = k.size(0);
  check_rows(k, T, H * dk, "k"); check_rows(wraw, T, H * dk, "wraw"); check_rows(araw, T, H * dk, "araw");
  const int esz = esz_of(k, "k");
  same_type(wraw, k, "wraw"); same_type(araw, k, "araw");
  auto f = k.options().dtype(at::kFloat);
  at::Tensor w = at::empty({T, H * dk}, f), p = at::empty({T, H * dk}, f), z = at::empty({T, H * dk}, f);
  CHECK_RC(lk_general_delta_prep(k.data_ptr(), k.stride(0), wraw.data_ptr(), wraw.stride(0), fp(w0, H * dk, "w0"), araw.data_ptr(),
                                 araw.stride(0), fp(a_b, H * dk, "a_b"), T, (int)H, (int)dk, w.data_ptr<float>(), p.data_ptr<float>(),
                                 z.data_ptr<float>(), esz, cur_stream()), "general_delta_prep");
  return {w, p, z};
}

at::Tensor head_norm_gate(const at::Tensor& o, const at::Tensor& gate, const c10::optional<at::Tensor>& w, int64_t H, double eps,
                          int64_t kind, at::ScalarType out_dtype) {
  CHECK_CUDA(o); CHECK_F32(o); CHECK_LASTDIM(o);
  TORCH_CHECK(o.dim() == 2 && H >= 1 && o.size(1) % H == 0, "o must be [T, H dv]");
  TORCH_CHECK(out_dtype == at::kBFloat16 || out_dtype == at::kFloat, "out dtype");
  const long T = o.size(0), n = o.size(1);
  check_rows(gate, T, n, "gate");
  const int gesz = esz_of(gate, "gate");
  at::Tensor out = at::empty({T, n}, o.options().dtype(out_dtype));
  CHECK_RC(lk_head_norm_gate(o.data_ptr<float>(), o.stride(0), gate.data_ptr(), gate.stride(0), gesz, fpo(w, n, "w"), T, (int)H,
                             (int)(n / H), (float)eps, (int)kind, out.data_ptr(), out.stride(0), (int)out.element_size(), cur_stream()),
           "head_norm_gate");
  return out;
}

void tanh_(at::Tensor& x) {
  CHECK_CUDA(x); CHECK_LASTDIM(x);
  TORCH_CHECK(x.dim() == 2, "x must be 2-d");
  CHECK_RC(lk_tanh_(x.data_ptr(), x.stride(0), x.size(0), (int)x.size(1), esz_of(x, "x"), cur_stream()), "tanh_");
}

void normrope_kv_write(at::Tensor& qkv, int64_t H, int64_t G, int64_t dim, int64_t vdim, int64_t norm_dim, int64_t norm_vdim,
                       const at::Tensor& qw, const at::Tensor& kw, int64_t rot, const at::Tensor& inv_freq, const at::Tensor& positions,
                       double eps, at::Tensor& kc, at::Tensor& vc, const at::Tensor& slots, bool v_unit) {
  CHECK_CUDA(qkv); CHECK_LASTDIM(qkv); CHECK_I32(slots); CHECK_CONTIG(slots); CHECK_CUDA(positions); CHECK_I32(positions);
  CHECK_CONTIG(positions);
  const int esz = esz_of(qkv, "qkv");
  const long T = qkv.size(0);
  TORCH_CHECK(qkv.dim() == 2 && qkv.size(1) >= (H + G) * dim + G * vdim, "qkv must be [T, >= (H + G) dim + G vdim]");
  TORCH_CHECK(slots.numel() >= T && positions.numel() >= T, "slots / positions");
  TORCH_CHECK(rot >= 0 && rot % 2 == 0 && rot <= dim, "rot");
  check_sig_caches(qkv, kc, vc, G, dim, vdim);
  CHECK_RC(lk_normrope_kv_write(qkv.data_ptr(), qkv.stride(0), T, (int)H, (int)G, (int)dim, (int)vdim, (int)norm_dim, (int)norm_vdim,
                                fp(qw, dim, "q norm weight"), fp(kw, dim, "k norm weight"), (int)rot,
                                fp(inv_freq, std::max<int64_t>(rot / 2, 1), "inv_freq"), ip(positions), (float)eps, kc.data_ptr(),
                                vc.data_ptr(), ip(slots), (int)kc.size(2), v_unit ? 1 : 0, esz, cur_stream()), "normrope_kv_write");
}

const void* gate_rows(const c10::optional<at::Tensor>& gate, const at::Tensor& q, int64_t gate_col, int64_t H, long* gs) {
  if (!gate) return nullptr;   // H: the gate's columns (one per head, or one per output element)
  check_rows(*gate, q.size(0), gate_col + H, "gate");
  same_type(*gate, q, "gate");
  TORCH_CHECK(gate_col >= 0, "gate_col");
  *gs = gate->stride(0);
  return gate->data_ptr();
}

// the pooled cache pair of a window mask (pool > 0): the same shapes and type as the K / V caches
void pooled_caches(const at::Tensor& q, const at::Tensor& kc, const c10::optional<at::Tensor>& pkc, const c10::optional<at::Tensor>& pvc,
                   int64_t pool, int64_t G, int64_t dim, int64_t vdim, const void** pkp, const void** pvp) {
  TORCH_CHECK(pool >= 0, "pool");
  if (pool == 0) return;
  TORCH_CHECK(pkc.has_value() && pvc.has_value(), "pooled caches are missing");
  check_sig_caches(q, *pkc, *pvc, G, dim, vdim);
  TORCH_CHECK(pkc->size(0) == kc.size(0) && pkc->size(2) == kc.size(2), "pooled caches must have the K / V caches' blocks");
  *pkp = pkc->data_ptr();
  *pvp = pvc->data_ptr();
}

void sinkattn_prefill(const at::Tensor& q, const at::Tensor& kc, const at::Tensor& vc, const at::Tensor& bt, const at::Tensor& cu_q,
                      const at::Tensor& ctx, const at::Tensor& tile_seq, const at::Tensor& tile_q0, int64_t H, int64_t G, int64_t dim,
                      int64_t vdim, const at::Tensor& hscale, int64_t mkind, int64_t msize, bool sink,
                      const c10::optional<at::Tensor>& gate, int64_t gate_col, at::Tensor& out,
                      const c10::optional<at::Tensor>& pkc, const c10::optional<at::Tensor>& pvc, int64_t pool, int64_t keep_first,
                      double softcap, bool gate_elem) {
  CHECK_CUDA(q); CHECK_LASTDIM(q); CHECK_CUDA(out); CHECK_LASTDIM(out);
  const int esz = esz_of(q, "q");
  const void *pkp = nullptr, *pvp = nullptr;
  pooled_caches(q, kc, pkc, pvc, pool, G, dim, vdim, &pkp, &pvp);
  same_type(out, q, "out");
  TORCH_CHECK(q.dim() == 2 && q.size(1) >= H * dim && out.dim() == 2 && out.size(0) == q.size(0) && out.size(1) >= H * vdim, "q / out shape");
  check_rows16(q, "q");
  check_sig_caches(q, kc, vc, G, dim, vdim);
  CHECK_CUDA(bt); CHECK_I32(bt); CHECK_I32(cu_q); CHECK_I32(ctx); CHECK_I32(tile_seq); CHECK_I32(tile_q0);
  CHECK_CONTIG(cu_q); CHECK_CONTIG(ctx); CHECK_CONTIG(tile_seq); CHECK_CONTIG(tile_q0);
  TORCH_CHECK(bt.dim() == 2 && bt.stride(1) == 1 && bt.size(0) >= cu_q.numel() - 1 && ctx.numel() >= cu_q.numel() - 1 &&
              tile_q0.numel() == tile_seq.numel(), "block tables / lengths / tiles");
  long gs = 0;
  const void* gp = gate_rows(gate, q, gate_col, gate_elem ? H * vdim : H, &gs);
  TORCH_CHECK(keep_first >= 0 && softcap >= 0, "keep_first / softcap");
  CHECK_RC(lk_sinkattn_prefill(q.data_ptr(), q.stride(0), kc.data_ptr(), vc.data_ptr(), ip(bt), (int)bt.stride(0), ip(cu_q), ip(ctx),
                               ip(tile_seq), ip(tile_q0), (int)tile_seq.numel(), (int)H, (int)G, (int)dim, (int)vdim, (int)kc.size(2),
                               fp(hscale, H, "hscale"), (int)mkind, (int)msize, sink ? 1 : 0, gp, gs, (int)gate_col, out.data_ptr(),
                               out.stride(0), pkp, pvp, (int)pool, (int)keep_first, (float)softcap, gate_elem ? 1 : 0, esz, cur_stream()),
           "sinkattn_prefill");
}

void sinkattn_decode(const at::Tensor& q, const at::Tensor& kc, const at::Tensor& vc, const at::Tensor& bt, const at::Tensor& ctx,
                     int64_t Z, int64_t H, int64_t G, int64_t dim, int64_t vdim, const at::Tensor& hscale, int64_t mkind,
                     int64_t msize, bool sink, const c10::optional<at::Tensor>& gate, int64_t gate_col, at::Tensor& out,
                     const c10::optional<at::Tensor>& part, const c10::optional<at::Tensor>& pkc,
                     const c10::optional<at::Tensor>& pvc, int64_t pool, int64_t keep_first, double softcap, bool gate_elem) {
  CHECK_CUDA(q); CHECK_LASTDIM(q); CHECK_CUDA(out); CHECK_LASTDIM(out);
  const int esz = esz_of(q, "q");
  const void *pkp = nullptr, *pvp = nullptr;
  pooled_caches(q, kc, pkc, pvc, pool, G, dim, vdim, &pkp, &pvp);
  same_type(out, q, "out");
  const long B = q.size(0);
  TORCH_CHECK(q.dim() == 2 && q.size(1) >= H * dim && out.dim() == 2 && out.size(0) == B && out.size(1) >= H * vdim, "q / out shape");
  check_rows16(q, "q");
  check_sig_caches(q, kc, vc, G, dim, vdim);
  CHECK_CUDA(bt); CHECK_I32(bt); CHECK_I32(ctx); CHECK_CONTIG(ctx);
  TORCH_CHECK(bt.dim() == 2 && bt.stride(1) == 1 && bt.size(0) >= B && ctx.numel() >= B && Z >= 1 && Z <= 65535, "block tables / lengths / splits");
  float* pp = nullptr;
  if (Z > 1) {
    TORCH_CHECK(part.has_value() && part->is_cuda() && part->scalar_type() == at::kFloat && part->is_contiguous() &&
                part->numel() >= B * H * Z * (vdim + 2), "part must be f32 [B, H, Z, vdim + 2]");
    pp = part->data_ptr<float>();
  }
  long gs = 0;
  const void* gp = gate_rows(gate, q, gate_col, gate_elem ? H * vdim : H, &gs);
  TORCH_CHECK(keep_first >= 0 && softcap >= 0, "keep_first / softcap");
  CHECK_RC(lk_sinkattn_decode(q.data_ptr(), q.stride(0), kc.data_ptr(), vc.data_ptr(), ip(bt), (int)bt.stride(0), ip(ctx), (int)B, (int)Z,
                              (int)H, (int)G, (int)dim, (int)vdim, (int)kc.size(2), fp(hscale, H, "hscale"), (int)mkind, (int)msize,
                              sink ? 1 : 0, gp, gs, (int)gate_col, out.data_ptr(), out.stride(0), pp, pkp, pvp, (int)pool, (int)keep_first,
                              (float)softcap, gate_elem ? 1 : 0, esz, cur_stream()),
           "sinkattn_decode");
}

// ---------------------------------------------------------------------------------------------
// windowed attention with pooled blocks, latent attention, table-routed experts
c10::optional<at::Tensor> stream_gated_norm(at::Tensor& x, const at::Tensor& y, int64_t parts, const at::Tensor& g, const at::Tensor& gb,
                                            const at::Tensor& wpost, const c10::optional<at::Tensor>& wnext, double eps,
                                            at::ScalarType out_dtype) {
  CHECK_CUDA(x); CHECK_F32(x); CHECK_CONTIG(x); CHECK_CUDA(y); CHECK_LASTDIM(y); CHECK_CUDA(g); CHECK_LASTDIM(g);
  const int esz = esz_of(y, "y");
  same_type(g, y, "g");
  TORCH_CHECK(x.dim() == 2 && y.dim() == 2 && g.dim() == 2 && parts >= 1, "x, y, g must be 2-d");
  const long T = x.size(0);
  const int W = x.size(1);
  TORCH_CHECK(y.size(0) == T * parts && y.size(1) == W && g.size(0) == T && g.size(1) == W, "y must be [T * parts, W], g [T, W]");
  TORCH_CHECK(y.scalar_type() == out_dtype, "out dtype must be the activations'");
  at::Tensor out;
  if (wnext) out = at::empty({T, W}, y.options());
  CHECK_RC(lk_stream_gated_norm(x.data_ptr<float>(), y.data_ptr(), y.stride(0), (int)parts, g.data_ptr(), g.stride(0), fp(gb, W, "gate bias"),
                                fp(wpost, W, "post norm weight"), fpo(wnext, W, "next norm weight"), (float)eps,
                                wnext ? out.data_ptr() : nullptr, wnext ? out.stride(0) : 0, T, W, esz, cur_stream()),
           "stream_gated_norm");
  if (!wnext) return c10::nullopt;
  return out;
}

at::Tensor rms_cols(const at::Tensor& u, int64_t col0, int64_t n, const at::Tensor& w, double eps) {
  CHECK_CUDA(u); CHECK_LASTDIM(u);
  const int esz = esz_of(u, "u");
  TORCH_CHECK(u.dim() == 2 && col0 >= 0 && n >= 1 && col0 + n <= u.size(1), "u columns");
  at::Tensor out = at::empty({u.size(0), n}, u.options());
  CHECK_RC(lk_rms_cols((const char*)u.data_ptr() + col0 * esz, u.stride(0), (int)n, fp(w, n, "norm weight"), (float)eps, out.data_ptr(),
                       out.stride(0), u.size(0), esz, cur_stream()), "rms_cols");
  return out;
}

void rot_kv_write(at::Tensor& q, int64_t H, int64_t qdim, const at::Tensor& k, int64_t G, int64_t kdim,
                  const c10::optional<at::Tensor>& kshared, int64_t sdim, const at::Tensor& v, int64_t vdim, int64_t rot_off,
                  int64_t rot, const at::Tensor& freq, double mag, const at::Tensor& positions, at::Tensor& kc, at::Tensor& vc,
                  const at::Tensor& slots, const c10::optional<at::Tensor>& v_other, double v_blend) {
  CHECK_CUDA(q); CHECK_LASTDIM(q); CHECK_CUDA(k); CHECK_LASTDIM(k); CHECK_CUDA(v); CHECK_LASTDIM(v);
  CHECK_CUDA(slots); CHECK_I32(slots); CHECK_CONTIG(slots); CHECK_CUDA(positions); CHECK_I32(positions); CHECK_CONTIG(positions);
  const int esz = esz_of(q, "q");
  same_type(k, q, "k"); same_type(v, q, "v");
  const long T = q.size(0);
  TORCH_CHECK(q.dim() == 2 && k.dim() == 2 && v.dim() == 2 && k.size(0) == T && v.size(0) == T, "q, k, v rows");
  TORCH_CHECK(H >= 1 && G >= 1 && q.size(1) >= H * qdim && k.size(1) >= G * kdim && v.size(1) >= G * vdim, "q, k, v columns");
  TORCH_CHECK(slots.numel() >= T && positions.numel() >= T, "slots / positions");
  const void* shp = nullptr;
  long shs = 0;
  if (sdim > 0) {
    TORCH_CHECK(kshared.has_value(), "shared key part is missing");
    CHECK_CUDA(*kshared); CHECK_LASTDIM(*kshared); same_type(*kshared, q, "kshared");
    TORCH_CHECK(kshared->dim() == 2 && kshared->size(0) == T && kshared->size(1) >= sdim, "shared key part must be [T, >= sdim]");
    shp = kshared->data_ptr();
    shs = kshared->stride(0);
  }
  CHECK_CUDA(kc); CHECK_CUDA(vc); CHECK_CONTIG(kc); CHECK_CONTIG(vc); same_type(kc, q, "k cache"); same_type(vc, q, "v cache");
  TORCH_CHECK(kc.dim() == 4 && vc.dim() == 4 && kc.size(1) == G && vc.size(1) == G && kc.size(0) == vc.size(0) && vc.size(3) == kc.size(2),
              "caches must be K [NB, G, BS, KD], V [NB, G, VD, BS]");
  CHECK_CUDA(freq); CHECK_F32(freq); CHECK_CONTIG(freq);
  TORCH_CHECK(rot >= 0 && rot % 2 == 0 && freq.numel() >= rot / 2, "rot / freq");
  const void* v2p = nullptr;
  long v2s = 0;
  if (v_other) {
    CHECK_CUDA(*v_other); CHECK_LASTDIM(*v_other); same_type(*v_other, q, "v_other");
    TORCH_CHECK(v_other->dim() == 2 && v_other->size(0) == T && v_other->size(1) >= G * vdim, "v_other must be [T, >= G vdim]");
    v2p = v_other->data_ptr();
    v2s = v_other->stride(0);
  }
  CHECK_RC(lk_rot_kv_write(q.data_ptr(), q.stride(0), (int)H, (int)qdim, k.data_ptr(), k.stride(0), (int)G, (int)kdim, shp, shs, (int)sdim,
                           v.data_ptr(), v.stride(0), (int)vdim, (int)rot_off, (int)rot, freq.data_ptr<float>(), (float)mag,
                           ip(positions), kc.data_ptr(), vc.data_ptr(), ip(slots), (int)kc.size(2), (int)kc.size(3), (int)vc.size(2), T,
                           v2p, v2s, (float)v_blend, esz, cur_stream()), "rot_kv_write");
}

void pool_kv_write(const at::Tensor& kc, const at::Tensor& vc, at::Tensor& pkc, at::Tensor& pvc, int64_t P, const at::Tensor& bt,
                   const at::Tensor& ctx, const c10::optional<at::Tensor>& cu_q, const at::Tensor& slots, int64_t row0,
                   int64_t max_len) {
  CHECK_CUDA(kc); CHECK_CUDA(vc); CHECK_CUDA(pkc); CHECK_CUDA(pvc); CHECK_CONTIG(kc); CHECK_CONTIG(vc); CHECK_CONTIG(pkc); CHECK_CONTIG(pvc);
  const int esz = esz_of(kc, "k cache");
  same_type(vc, kc, "v cache"); same_type(pkc, kc, "pooled k cache"); same_type(pvc, kc, "pooled v cache");
  TORCH_CHECK(kc.dim() == 4 && vc.dim() == 4 && kc.sizes() == pkc.sizes() && vc.sizes() == pvc.sizes() && kc.size(0) == vc.size(0) &&
              kc.size(1) == vc.size(1) && vc.size(3) == kc.size(2), "caches must be K [NB, G, BS, dim], V [NB, G, vdim, BS], pooled pair alike");
  CHECK_CUDA(bt); CHECK_I32(bt); CHECK_CUDA(ctx); CHECK_I32(ctx); CHECK_CONTIG(ctx); CHECK_CUDA(slots); CHECK_I32(slots); CHECK_CONTIG(slots);
  const long S = cu_q ? cu_q->numel() - 1 : ctx.numel();
  if (cu_q) { CHECK_CUDA(*cu_q); CHECK_I32(*cu_q); CHECK_CONTIG(*cu_q); }
  TORCH_CHECK(bt.dim() == 2 && bt.stride(1) == 1 && bt.size(0) >= S && ctx.numel() >= S && P >= 1 && row0 >= 0 && max_len >= 1,
              "block tables / lengths");
  TORCH_CHECK(cu_q.has_value() || slots.numel() >= row0 + S, "slots");
  CHECK_RC(lk_pool_kv_write(kc.data_ptr(), vc.data_ptr(), pkc.data_ptr(), pvc.data_ptr(), (int)P, ip(bt), (int)bt.stride(0), ip(ctx),
                            ipo(cu_q), ip(slots), (int)row0, (int)S, (int)max_len, (int)kc.size(1), (int)kc.size(2), (int)kc.size(3),
                            (int)vc.size(2), esz, cur_stream()), "pool_kv_write");
}

// x [rows, K] sorted by expert -- or, with `gather` int32 [rows], any x whose row gather[r] is sorted row r's input; the
// result's rows are sorted, or with `scatter` int32 [rows] sorted row r lands in out row scatter[r] (a permutation)
at::Tensor gemm_grouped(const at::Tensor& x, const at::Tensor& seg, const at::Tensor& w, bool swiglu,
                        const c10::optional<at::Tensor>& gather, const c10::optional<at::Tensor>& scatter) {
  CHECK_CUDA(x); CHECK_BF16(x); CHECK_LASTDIM(x); CHECK_CUDA(w); CHECK_BF16(w); CHECK_CONTIG(w); CHECK_CUDA(seg); CHECK_I32(seg);
  CHECK_CONTIG(seg);
  TORCH_CHECK(x.dim() == 2 && w.dim() == 3 && w.size(2) == x.size(1) && seg.numel() == w.size(0) + 1, "x [rows, K], w [E, N, K], seg [E + 1]");
  const int N = w.size(1), K = w.size(2);
  TORCH_CHECK(lk_gemm_grouped_supported(N, K, swiglu ? 1 : 0), "shape not tiled by the grouped GEMM");
  long rows = x.size(0);
  if (gather) { CHECK_CUDA(*gather); CHECK_I32(*gather); CHECK_CONTIG(*gather); rows = gather->numel(); }
  if (scatter) { CHECK_CUDA(*scatter); CHECK_I32(*scatter); CHECK_CONTIG(*scatter); TORCH_CHECK(scatter->numel() == rows, "scatter rows"); }
  at::Tensor out = at::empty({rows, swiglu ? N / 2 : N}, x.options());
  CHECK_RC(lk_gemm_grouped(bp(x), x.stride(0), bp(w), ip(seg), (int)w.size(0), rows, N, K, swiglu ? 1 : 0, bp(out), out.stride(0),
                           cur_stream(), ipo(gather), x.size(0), ipo(scatter)), "gemm_grouped");
  return out;
}

// ids absent: the table has one row per token of the step (a router's choice)
std::vector<at::Tensor> moe_route(const c10::optional<at::Tensor>& ids, const at::Tensor& table, int64_t E) {
  CHECK_CUDA(table); CHECK_I32(table); CHECK_CONTIG(table);
  if (ids) { CHECK_CUDA(*ids); CHECK_I32(*ids); CHECK_CONTIG(*ids); }
  TORCH_CHECK(table.dim() == 2 && E >= 1, "table must be int32 [vocab, top]");
  const long T = ids ? ids->numel() : table.size(0);
  const int top = table.size(1);
  at::Tensor seg = at::empty({E + 1}, table.options());
  at::Tensor order = at::empty({T * top}, table.options());
  CHECK_RC(lk_moe_route(ipo(ids), ip(table), (int)table.size(0), top, (int)E, (int)T, seg.data_ptr<int>(), order.data_ptr<int>(),
                        cur_stream()), "moe_route");
  return {seg, order};
}

// ---------------------------------------------------------------------------------------------
// parallel sublayers and routed experts
std::vector<c10::optional<at::Tensor>> stream_parallel_norm(at::Tensor& x, const c10::optional<at::Tensor>& a, const c10::optional<at::Tensor>& b,
                                                            const c10::optional<at::Tensor>& y, const c10::optional<at::Tensor>& yw,
                                                            const c10::optional<at::Tensor>& w1, const c10::optional<at::Tensor>& w2,
                                                            double eps, at::ScalarType out_dtype) {
  CHECK_CUDA(x); CHECK_F32(x); CHECK_CONTIG(x);
  TORCH_CHECK(x.dim() == 2, "x must be [T, W]");
  TORCH_CHECK(out_dtype == at::kBFloat16 || out_dtype == at::kFloat, "out dtype");
  const long T = x.size(0);
  const int W = x.size(1);
  const int esz = out_dtype == at::kFloat ? 4 : 2;
  auto rows_of = [&](const c10::optional<at::Tensor>& t, long rows, const char* what, long* stride) -> const void* {
    if (!t) return nullptr;
    CHECK_CUDA(*t); CHECK_LASTDIM(*t);
    TORCH_CHECK(t->dim() == 2 && t->size(0) == rows && t->size(1) == W, what, " must be [", rows, ", ", W, "]");
    TORCH_CHECK(t->scalar_type() == out_dtype, what, ": dtype must be the activations'");
    *stride = t->stride(0);
    return t->data_ptr();
  };
  long as = 0, bs = 0, ys = 0;
  const void* ap = rows_of(a, T, "a", &as);
  const void* bp_ = rows_of(b, T, "b", &bs);
  int top = 0;
  const float* ywp = nullptr;
  if (y) {
    TORCH_CHECK(yw.has_value(), "expert rows need their weights");
    CHECK_CUDA(*yw); CHECK_F32(*yw); CHECK_CONTIG(*yw);
    TORCH_CHECK(yw->dim() == 2 && yw->size(0) == T && yw->size(1) >= 1, "weights must be f32 [T, top]");
    top = yw->size(1);
    ywp = yw->data_ptr<float>();
  }
  const void* yp = rows_of(y, T * std::max(top, 1), "y", &ys);
  c10::optional<at::Tensor> o1, o2;
  auto opt = x.options().dtype(out_dtype);
  if (w1) o1 = at::empty({T, W}, opt);
  if (w2) o2 = at::empty({T, W}, opt);
  CHECK_RC(lk_stream_parallel_norm(x.data_ptr<float>(), ap, as, bp_, bs, yp, ys, ywp, top, fpo(w1, W, "norm weight 1"),
                                   fpo(w2, W, "norm weight 2"), (float)eps, o1 ? o1->data_ptr() : nullptr, o1 ? o1->stride(0) : 0,
                                   o2 ? o2->data_ptr() : nullptr, o2 ? o2->stride(0) : 0, T, W, esz, cur_stream()),
           "stream_parallel_norm");
  return {o1, o2};
}

std::vector<at::Tensor> router_topk(const at::Tensor& h, const at::Tensor& wr, int64_t top, int64_t groups, int64_t keep, double scale) {
  CHECK_CUDA(h); CHECK_LASTDIM(h); CHECK_CUDA(wr); CHECK_F32(wr); CHECK_CONTIG(wr);
  const int esz = esz_of(h, "h");
  TORCH_CHECK(h.dim() == 2 && wr.dim() == 2 && wr.size(1) == h.size(1), "h [T, W], router [E, W]");
  const long T = h.size(0);
  at::Tensor experts = at::empty({T, top}, h.options().dtype(at::kInt));
  at::Tensor weights = at::empty({T, top}, h.options().dtype(at::kFloat));
  CHECK_RC(lk_router_topk(h.data_ptr(), h.stride(0), wr.data_ptr<float>(), (int)wr.size(0), (int)wr.size(1), T, (int)top, (int)groups,
                          (int)keep, (float)scale, experts.data_ptr<int>(), weights.data_ptr<float>(), esz, cur_stream()),
           "router_topk");
  return {experts, weights};
}

at::Tensor clamped_glu(const at::Tensor& gu, double limit, double alpha) {
  CHECK_CUDA(gu); CHECK_LASTDIM(gu);
  const int esz = esz_of(gu, "gu");
  TORCH_CHECK(gu.dim() == 2 && gu.size(1) % 2 == 0, "gu must be [T, 2F]");
  const int F = gu.size(1) / 2;
  at::Tensor out = at::empty({gu.size(0), F}, gu.options());
  CHECK_RC(lk_clamped_glu(gu.data_ptr(), gu.stride(0), out.data_ptr(), out.stride(0), gu.size(0), F, (float)limit, (float)alpha, esz,
                          cur_stream()), "clamped_glu");
  return out;
}

void silu_(at::Tensor& x) {
  CHECK_CUDA(x); CHECK_LASTDIM(x);
  TORCH_CHECK(x.dim() == 2, "x must be 2-d");
  CHECK_RC(lk_silu_(x.data_ptr(), x.stride(0), x.size(0), (int)x.size(1), esz_of(x, "x"), cur_stream()), "silu_");
}

void sigmoid_mul_(at::Tensor& x, const at::Tensor& g) {
  CHECK_CUDA(x); CHECK_LASTDIM(x); CHECK_CUDA(g); CHECK_LASTDIM(g);
  same_type(g, x, "gate");
  TORCH_CHECK(x.dim() == 2 && g.dim() == 2 && g.size(0) == x.size(0) && g.size(1) >= x.size(1), "x [T, n], gate [T, >= n]");
  CHECK_RC(lk_sigmoid_mul_(x.data_ptr(), x.stride(0), g.data_ptr(), g.stride(0), x.size(0), (int)x.size(1), esz_of(x, "x"), cur_stream()),
           "sigmoid_mul_");
}

at::Tensor moe_gemm(const at::Tensor& x, const at::Tensor& order, const at::Tensor& seg, const at::Tensor& w, int64_t top, bool act) {
  CHECK_CUDA(x); CHECK_LASTDIM(x); CHECK_CUDA(w); CHECK_CONTIG(w); CHECK_CUDA(order); CHECK_I32(order); CHECK_CONTIG(order);
  CHECK_CUDA(seg); CHECK_I32(seg); CHECK_CONTIG(seg);
  const int esz = esz_of(x, "x");
  same_type(w, x, "w");
  TORCH_CHECK(x.dim() == 2 && w.dim() == 3 && w.size(2) == x.size(1) && seg.numel() == w.size(0) + 1 && top >= 1, "x [rows, K], w [E, N, K]");
  const long pairs = order.numel();
  TORCH_CHECK(act ? x.size(0) * top == pairs : x.size(0) == pairs, "rows of x: tokens (act) or sorted pairs");
  const int N = w.size(1);
  at::Tensor out = at::empty({pairs, act ? N / 2 : N}, x.options());
  CHECK_RC(lk_moe_gemm(x.data_ptr(), x.stride(0), ip(order), ip(seg), (int)w.size(0), (int)top, pairs, w.data_ptr(), N, (int)w.size(2),
                       act ? 1 : 0, out.data_ptr(), out.stride(0), esz, cur_stream()), "moe_gemm");
  return out;
}

}  // namespace
// build provenance: "LKSTAMP:<hash of sources + flags>", generated by csrc/build.py at link time
extern "C" const char lk_source_stamp[];

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("embed_pos", &embed_pos);
  m.def("stream_embed_errors", []() { return lk_stream_embed_errors(); });
  m.def("stream_rmsnorm", &stream_rmsnorm);
  m.def("softcap", &softcap);
  m.def("silu_mul_f32", &silu_mul_f32);
  m.def("sigattn_supported", [](int64_t H, int64_t G, int64_t dim, int64_t vdim, int64_t BS, int64_t esz) {
    return lk_sigattn_supported((int)H, (int)G, (int)dim, (int)vdim, (int)BS, (int)esz) != 0;
  });
  m.def("unitnorm_kv_write", &unitnorm_kv_write);
  m.def("sigattn_prefill", &sigattn_prefill);
  m.def("sigattn_decode", &sigattn_decode);
  m.def("conv_silu", &conv_silu);
  m.def("ssm_scan", &ssm_scan);
  m.def("gated_group_rmsnorm", &gated_group_rmsnorm);
  m.def("embed_stream", &embed_stream);
  m.def("stream_layernorm", &stream_layernorm);
  m.def("gelu_tanh_mul", &gelu_tanh_mul);
  m.def("dual_rmsnorm_mean", &dual_rmsnorm_mean);
  m.def("delta_scan", &delta_scan);
  m.def("gated_delta_prep", &gated_delta_prep);
  m.def("general_delta_prep", &general_delta_prep);
  m.def("head_norm_gate", &head_norm_gate);
  m.def("tanh_", &tanh_);
  m.def("normrope_kv_write", &normrope_kv_write);
  m.def("sinkattn_prefill", &sinkattn_prefill);
  m.def("sinkattn_decode", &sinkattn_decode);
  m.def("stream_gated_norm", &stream_gated_norm);
  m.def("rms_cols", &rms_cols);
  m.def("rot_kv_write", &rot_kv_write);
  m.def("pool_kv_write", &pool_kv_write);
  m.def("moe_route", &moe_route);
  m.def("stream_parallel_norm", &stream_parallel_norm);
  m.def("router_topk", &router_topk);
  m.def("clamped_glu", &clamped_glu);
  m.def("silu_", &silu_);
  m.def("sigmoid_mul_", &sigmoid_mul_);
  m.def("gemm_grouped", &gemm_grouped);
  m.def("gemm_grouped_supported", [](int64_t N, int64_t K, bool swiglu) { return lk_gemm_grouped_supported((int)N, (int)K, swiglu ? 1 : 0) != 0; });
  m.def("moe_gemm", &moe_gemm);
  m.def("window_mark", [](int64_t id) { CHECK_RC(lk_window_mark((int)id, cur_stream()), "window_mark"); });
  m.def("debug_invalid_launch", []() { CHECK_RC(lk_debug_invalid_launch(cur_stream()), "debug_invalid_launch"); });
  // a HIP stream restricted to the CUs of a bit mask (32 CUs per word): two kernels that
  // would each fill the chip (a mixed step's flash prefill and paged decode) run side by side
  // on disjoint CU sets.  Returned as an integer handle for torch.cuda.ExternalStream; the
  // stream lives for the process.
  m.def("cu_mask_stream", [](std::vector<int64_t> words) {
    std::vector<uint32_t> w(words.size());
    for (size_t i = 0; i < words.size(); ++i) w[i] = (uint32_t)(words[i] & 0xffffffffLL);
    hipStream_t st = nullptr;
    TORCH_CHECK(hipExtStreamCreateWithCUMask(&st, (uint32_t)w.size(), w.data()) == hipSuccess,
                "hipExtStreamCreateWithCUMask failed");
    return (int64_t)reinterpret_cast<uintptr_t>(st);
  });
  m.def("stream_cu_mask", [](int64_t handle, int64_t nwords) {
    std::vector<uint32_t> w((size_t)nwords, 0u);
    TORCH_CHECK(hipExtStreamGetCUMask(reinterpret_cast<hipStream_t>((uintptr_t)handle), (uint32_t)nwords, w.data()) ==
                    hipSuccess, "hipExtStreamGetCUMask failed");
    return std::vector<int64_t>(w.begin(), w.end());
  });
  m.def("source_stamp", [] { return std::string(lk_source_stamp + 8); });
  py::class_<XgmiAr>(m, "XgmiAr")
      .def(py::init<int, int, int64_t>(), py::arg("rank"), py::arg("world"), py::arg("bytes"))
      .def("handles", &XgmiAr::handles)
      .def("open", &XgmiAr::open)
      .def("all_reduce", &XgmiAr::all_reduce)
      .def("all_reduce_rmsnorm", &XgmiAr::all_reduce_rmsnorm)
      .def("all_reduce2", &XgmiAr::all_reduce2, "", py::arg("x"), py::arg("out"), py::arg("residual") = py::none(),
           py::arg("w") = py::none(), py::arg("eps") = 1e-5)
      .def("gather", &XgmiAr::gather, "", py::arg("in"), py::arg("out"), py::arg("root") = -1)
      .def("max_bytes", &XgmiAr::max_bytes)
      .def("error", &XgmiAr::error)
      .def_readonly("bytes", &XgmiAr::bytes);
  m.doc() = "gfx950 (MI355X) HIP kernel library";
  m.def("rmsnorm", &rmsnorm, "", py::arg("x"), py::arg("w"), py::arg("eps"), py::arg("residual") = py::none(), py::arg("out") = py::none());
  m.def("layernorm", &layernorm, "", py::arg("x"), py::arg("w"), py::arg("b"), py::arg("eps"), py::arg("residual") = py::none(), py::arg("write_residual") = false);
  m.def("embed_layernorm", &embed_layernorm);
  m.def("skinny_linear", &skinny_linear, "", py::arg("x"), py::arg("w"), py::arg("swiglu") = false,
        py::arg("splits") = 0, py::arg("out") = py::none());
  m.def("skinny_splits", &skinny_splits);
  m.def("ws_linear", &ws_linear, "", py::arg("x"), py::arg("w"), py::arg("swiglu") = false, py::arg("bn") = 0,
        py::arg("splits") = 0, py::arg("out") = py::none());
  m.def("ws_plan", &ws_plan);
  m.def("gemm", &gemm, "", py::arg("x"), py::arg("w"), py::arg("bias") = py::none(), py::arg("epi") = 0,
        py::arg("bn") = 256, py::arg("out") = py::none(), py::arg("variant") = 1,
        py::arg("splits") = 1);
  m.def("gemm_fused", &gemm_fused, "", py::arg("x"), py::arg("w"), py::arg("epi"), py::arg("bn"), py::arg("out") = py::none(),
        py::arg("variant") = 2, py::arg("splits") = 1, py::arg("ss_in") = py::none(), py::arg("eps") = 1e-5,
        py::arg("resid") = py::none(), py::arg("ss_out") = py::none(), py::arg("positions") = py::none(),
        py::arg("cos_sin") = py::none(), py::arg("slots") = py::none(), py::arg("k_cache") = py::none(),
        py::arg("v_cache") = py::none(), py::arg("hq") = 0, py::arg("hkv") = 0, py::arg("hd") = 0);
  m.def("embed_rows", &embed_rows, "", py::arg("table"), py::arg("ids"), py::arg("lo") = 0, py::arg("n_local") = -1);
  m.def("embed_errors", []() { return (int64_t)lk_embed_errors(); },
        "token ids outside the (whole) embedding table seen since the last call (resets)");
  m.def("scatter_ids", &scatter_ids);
  m.def("gather_rows", &gather_rows);
  m.def("argmax_key", &argmax_key, "", py::arg("logits"), py::arg("vocab_lo") = 0);
  m.def("keys_to_ids", &keys_to_ids);
  m.def("gemm_streamk", &gemm_streamk,
        "stream-K policy of the prefill GEMM (mode 0 off / 1 on / -1 keep); returns the waits that gave up since the last call",
        py::arg("mode") = -1);
  m.def("gemm_supported", &gemm_supported, "", py::arg("M"), py::arg("N"), py::arg("K"), py::arg("epi"), py::arg("bn"),
        py::arg("splits") = 1, py::arg("variant") = -1);
  m.def("silu_mul", &silu_mul, "", py::arg("x"), py::arg("out") = py::none());
  m.def("activation_", &activation_);
  m.def("rope_kv_", &rope_kv_);
  m.def("ws_set_rot", [](int64_t r) { lk_wsgemm_set_rot((int)r); });
  m.def("ws_linear_rmsnorm", &ws_linear_rmsnorm, "", py::arg("x"), py::arg("w"), py::arg("residual"),
        py::arg("norm_w"), py::arg("eps"), py::arg("bn") = 0, py::arg("splits") = 0, py::arg("tickets") = py::none());
  m.def("ws_linear_rope_kv", &ws_linear_rope_kv, "", py::arg("x"), py::arg("w"), py::arg("positions"),
        py::arg("cos_sin"), py::arg("Hq"), py::arg("Hkv"), py::arg("D"), py::arg("k_cache"), py::arg("v_cache"),
        py::arg("slots"), py::arg("neox") = true, py::arg("write_k_inplace") = false, py::arg("bn") = 0,
        py::arg("splits") = 0, py::arg("tickets") = py::none());
  m.def("kv_write", &kv_write);
  m.def("decode_splits", &decode_splits);
  m.def("decode_split_size", &decode_split_size);
  m.def("paged_decode", &paged_decode, "", py::arg("q"), py::arg("k_cache"), py::arg("v_cache"), py::arg("block_tables"), py::arg("ctx_lens"), py::arg("max_splits"), py::arg("split"), py::arg("scale"), py::arg("part_o") = py::none(), py::arg("part_ml") = py::none(), py::arg("out") = py::none(), py::arg("k_start") = py::none(), py::arg("pp_o") = py::none(), py::arg("pp_ml") = py::none(), py::arg("tickets") = py::none(), py::arg("reduce") = true);
  m.def("prefill_rows_per_tile", &prefill_rows_per_tile);
  m.def("ws_pro", &ws_pro, "", py::arg("x"), py::arg("w"), py::arg("swiglu"), py::arg("bn"), py::arg("splits"),
        py::arg("kind"), py::arg("reduce") = false, py::arg("pp") = py::none(), py::arg("res_in") = py::none(),
        py::arg("res_out") = py::none(), py::arg("gamma") = py::none(), py::arg("eps") = 0.0,
        py::arg("po") = py::none(), py::arg("pml") = py::none(), py::arg("ctx") = py::none(), py::arg("split") = 0,
        py::arg("max_splits") = 0, py::arg("Hq") = 0);
  m.def("splitk_rope_kv", &splitk_rope_kv);
  m.def("splitk_rmsnorm", &splitk_rmsnorm);
  m.def("gemv_decode", &gemv_decode, "", py::arg("mode"), py::arg("x"), py::arg("w"), py::arg("gamma") = py::none(),
        py::arg("eps") = 1e-5, py::arg("res") = py::none(), py::arg("positions") = py::none(),
        py::arg("cos_sin") = py::none(), py::arg("Hq") = 0, py::arg("Hkv") = 0, py::arg("D") = 0,
        py::arg("k_cache") = py::none(), py::arg("v_cache") = py::none(), py::arg("slots") = py::none(),
        py::arg("neox") = true, py::arg("po") = py::none(), py::arg("pml") = py::none(), py::arg("ctx") = py::none(),
        py::arg("max_splits") = 0, py::arg("split") = 0);
  m.def("gemv_supported", [](int64_t M, int64_t N, int64_t K, int64_t mode) {
    return lk_gemv_supported((int)M, (int)N, (int)K, (int)mode) != 0;
  });
  m.def("gemv_set_wgs", [](int64_t n) { lk_gemv_set_wgs((int)n); });
  m.def("gemv_set_ksplit", [](bool on) { lk_gemv_set_ksplit(on ? 1 : 0); });
  // read rows [r0, r1) of a contiguous 2-D tensor through the Infinity Cache (lk_l3_prefetch)
  m.def("l3_prefetch", [](const at::Tensor& t, int64_t r0, int64_t r1, int64_t wgs, at::Tensor& sink) {
    CHECK_CUDA(t); CHECK_CONTIG(t); CHECK_CUDA(sink);
    TORCH_CHECK(sink.scalar_type() == at::kInt && sink.numel() >= 1, "sink: int32 [>= 1]");
    TORCH_CHECK(t.dim() == 2 && 0 <= r0 && r0 <= r1 && r1 <= t.size(0), "rows out of range");
    const long row = t.size(1) * t.element_size();
    const char* base = reinterpret_cast<const char*>(t.data_ptr()) + r0 * row;
    CHECK_RC(lk_l3_prefetch(base, (r1 - r0) * row, (int)wgs, reinterpret_cast<unsigned*>(sink.data_ptr<int>()),
                            cur_stream()), "l3_prefetch");
  });
  m.def("ws_set_variant", [](int64_t M, int64_t N, int64_t K, bool swiglu, int64_t v) {
    CHECK_RC(lk_wsgemm_set_variant((int)M, (int)N, (int)K, swiglu ? 1 : 0, (int)v), "ws_set_variant");
  }, "weight-streaming GEMM kernel for this (M bucket, N, K, swiglu): 0 ring, 1 loader waves, -1 default",
        py::arg("M"), py::arg("N"), py::arg("K"), py::arg("swiglu"), py::arg("variant"));
  m.def("flash_prefill", &flash_prefill, "", py::arg("q"), py::arg("k"), py::arg("v"), py::arg("block_tables"), py::arg("cu_q"), py::arg("ctx_lens"), py::arg("tile_seq"), py::arg("tile_q0"), py::arg("Hq"), py::arg("Hkv"), py::arg("D"), py::arg("scale"), py::arg("causal"), py::arg("out") = py::none(), py::arg("part_o") = py::none(), py::arg("part_ml") = py::none(), py::arg("q_past") = py::none());
  m.def("knn_topk", &knn_topk, "", py::arg("corpus"), py::arg("cnorm"), py::arg("queries"), py::arg("qnorm"),
        py::arg("K"), py::arg("force_fused") = false);
  m.def("knn_merge", &knn_merge);
  m.def("pool_normalize", &pool_normalize, "", py::arg("hidden"), py::arg("cu"), py::arg("mode"), py::arg("normalize"),
        py::arg("out") = py::none());
  m.def("row_norms", &row_norms);
  m.def("select_allowed", &select_allowed, "", py::arg("logits"), py::arg("plan"), py::arg("temps") = py::none(),
        py::arg("seed") = 0, py::arg("step") = 0);
  m.def("select_tokens", &select_tokens, "", py::arg("logits"), py::arg("temps") = py::none(), py::arg("seed") = 0, py::arg("step") = 0, py::arg("out") = py::none());
  m.def("repeat_penalty_", &repeat_penalty_);
  m.def("sample", &sample, "", py::arg("logits"), py::arg("prm"), py::arg("hist"), py::arg("hist_len"),
        py::arg("seed") = 0, py::arg("out") = py::none());
}

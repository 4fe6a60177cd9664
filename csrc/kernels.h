// Host-callable launchers of the gfx950 kernel library.  Raw pointers + an explicit
// stream keep the .hip translation units free of torch headers (fast rebuilds) and
// make every launcher capturable in a hipGraph (no allocation, no sync inside).
// Return 0 on success, <0 for an unsupported shape (checked before launch).
#pragma once
#include <hip/hip_runtime.h>

typedef unsigned short bf16_t;

// Launch-failure return codes (common.h LK_CHECK_LAUNCH / LK_SET_MAX_LDS): the bindings raise
// with the HIP error string instead of handing back an uninitialised output.
constexpr int kLkLaunchError = -1000;  // rc = kLkLaunchError - hipError_t
constexpr int kLkAttrError = -2000;    // rc = kLkAttrError - hipError_t (dynamic-LDS opt-in refused)

// norm.hip
int lk_rmsnorm(bf16_t* out, bf16_t* residual, const bf16_t* x, const bf16_t* w, long rows, int H,
               float eps, long xs, long os, long rs, hipStream_t st);
int lk_splitk_rmsnorm(bf16_t* out, bf16_t* residual, const float* part, int S, const bf16_t* w, long rows, int H,
                      float eps, long os, long rs, hipStream_t st);
int lk_layernorm(bf16_t* out, const bf16_t* x, const bf16_t* res, bf16_t* res_out, const bf16_t* w,
                 const bf16_t* b, long rows, int H, float eps, long xs, long os, long rs,
                 hipStream_t st);
int lk_embed_layernorm(bf16_t* out, const int* ids, const int* pos_ids, const int* type_ids,
                       const bf16_t* tok, const bf16_t* pos, const bf16_t* typ, const bf16_t* w,
                       const bf16_t* b, long rows, int H, float eps, hipStream_t st);

// activation.hip
int lk_silu_mul(bf16_t* out, const bf16_t* x, long rows, int I, long xs, long os, hipStream_t st);
int lk_activation(bf16_t* x, const bf16_t* bias, long rows, int N, long xs, int kind,
                  hipStream_t st);

// skinny_gemm.hip (decode-regime linear, optional fused SwiGLU)
int lk_skinny_splits(int M, int N, int K, int swiglu);
int lk_skinny_gemm(const bf16_t* x, long ldx, const bf16_t* w, int M, int N, int K, int S, int swiglu,
                   bf16_t* out, long ldo, float* part, hipStream_t st);

void lk_wsgemm_plan(int M, int N, int K, int swiglu, int* bn_out, int* s_out);
int lk_wsgemm_pro(int kind, bf16_t* x, const bf16_t* w, int M, int N, int K, int BN, int S, int swiglu,
                  bf16_t* out, long ldo, float* part, const float* pp, int pS, const bf16_t* res, bf16_t* res_out,
                  long rs, const bf16_t* gamma, float eps, const float* po, const float* pml, const int* ctx, int Hq,
                  int D, int max_splits, int split, hipStream_t st);
int lk_wsgemm(const bf16_t* x, long ldx, const bf16_t* w, int M, int N, int K, int BN, int S, int swiglu,
              bf16_t* out, long ldo, float* part, hipStream_t st);

// gemv_decode.hip (decode GEMV for M <= 2 rows; mode 0 out, 1 res += out, 2 SwiGLU, 3 RoPE + paged KV;
// gamma != nullptr: RMSNorm prologue over x; po != nullptr (mode 1): x = the paged-decode split merge)
int lk_gemv_supported(int M, int N, int K, int mode);
void lk_gemv_set_wgs(int wgs);
void lk_gemv_set_ksplit(int on);
int lk_l3_prefetch(const void* p, long bytes, int wgs, unsigned* sink, hipStream_t st);
int lk_gemv_decode(int mode, const bf16_t* x, long ldx, const bf16_t* gamma, float eps, const bf16_t* w, int M, int N,
                   int K, bf16_t* out, long ldo, bf16_t* res, long ldr, const int* positions, const float* cos_sin,
                   int Hq, int Hkv, int D, bf16_t* kc, bf16_t* vc, const int* slots, int BS, int neox,
                   const float* po, const float* pml, const int* ctx, int max_splits, int split, hipStream_t st);

// GEMM part only (S >= 2): f32 partial slabs part[S][M][N], for a consumer that fuses the
// split-K reduction (lk_splitk_rmsnorm, lk_splitk_rope_kv)
int lk_wsgemm_set_variant(int M, int N, int K, int swiglu, int variant);  // -1 = back to the default
int lk_wsgemm_part(const bf16_t* x, long ldx, const bf16_t* w, int M, int N, int K, int BN, int S, float* part,
                   hipStream_t st);
// the same split-K GEMM with the reduction fused into its last workgroup(s): RoPE + paged-KV
// write per head (BN == D == 128), or residual + RMSNorm for M <= 4 (skinny_gemm.hip WsTail)
int lk_ws_rope_kv_fused(const bf16_t* x, long ldx, const bf16_t* w, int M, int K, int BN, int S, float* part,
                        int* tickets, bf16_t* qkv, long qs, const int* positions, const float* cos_sin, int Hq,
                        int Hkv, int D, bf16_t* kc, bf16_t* vc, const int* slots, int BS, int neox,
                        int write_k_inplace, hipStream_t st);
int lk_ws_rmsnorm_fused(const bf16_t* x, long ldx, const bf16_t* w, int M, int N, int K, int BN, int S, float* part,
                        int* tickets, bf16_t* out, long os, bf16_t* residual, long rs, const bf16_t* norm_w, float eps,
                        hipStream_t st);

void lk_wsgemm_set_rot(int rot_mul);  // K-step rotation per column tile (0 = off, -1 = policy)

int lk_ws_scores_f32(const bf16_t* x, long ldx, const bf16_t* w, int M, long N, int K, float* out, long ldo,
                     hipStream_t st);

// xgmi_allreduce.hip (one-shot / two-shot all-reduce over IPC-mapped peer buffers, K14)
int lk_xgmi_ar_sig_words();
int lk_xgmi_gather(bf16_t* const* data, unsigned* const* sig, int rank, int world, int root, const void* in,
                   void* out, long nbytes, int* err, hipStream_t st);
int lk_xgmi_allreduce2(bf16_t* const* data, unsigned* const* sig, long red_off, int rank, int world,
                       const bf16_t* in, bf16_t* residual, const bf16_t* w, bf16_t* out, int T, int H, float eps,
                       int norm, int* err, hipStream_t st);
int lk_xgmi_ar_max_ranks();
int lk_xgmi_allreduce_rmsnorm(bf16_t* const* data, unsigned* const* sig, int rank, int world, const bf16_t* in,
                              bf16_t* residual, const bf16_t* w, bf16_t* out, int T, int H, float eps, int* err,
                              hipStream_t st);
int lk_xgmi_allreduce(bf16_t* const* data, unsigned* const* sig, int rank, int world, const bf16_t* in,
                      bf16_t* out, long n, int* err, hipStream_t st);

// gemm.hip (prefill / encoder-regime linear, 256 x {256,192} MFMA tiles, fused epilogues)
// epi: 0 none, 1 SwiGLU (W = [Wg; Wu]), 2 bias, 3 bias + GELU(erf), 4 bias + ReLU; bn: 256 | 192
// ks > 1: split-K over ks K-ranges, fp32 partials in ws [ks, M, N], then a reduce applies the
// epilogue (not SwiGLU) -- for shapes with fewer tiles than CUs
int lk_gemm_supported(int M, int N, int K, int epi, int bn, int ks = 1);
int lk_gemm_streamk(int mode);
// Fused prefill-chain epilogues of lk_gemm (the RMSNorm of the pre-norm decoder block folded
// into its neighbouring GEMMs, the norm weight g folded into the consumer's weight rows):
//   row scale (any of epi NONE / SWIGLU / QKV, when ss_in is set): acc *= rsqrt(sum_t
//     ss_in[t * ss_ld + row] / H + eps) before the epilogue -- the consumer side of the norm;
//   epi RESID (6): r = bf16(r + bf16(acc)) in place in resid [M, ldr], and the per-row partial
//     sums of squares of the new r over this column tile into ss_out[tn * ss_out_ld + row]
//     (tn = column tile of 256) -- the producer side; `out` is not written;
//   epi QKV (7): out = the qkv row, q / k heads rotated with interleaved-pair RoPE (weights
//     permuted at load: models/llama.py), K / V scattered into the paged cache at slots[row]
//     (slot < 0: not cached).
struct LkEpi {
  const float* ss_in = nullptr;  // [nt][ss_ld] fp32 partial sums of squares (row scale)
  int ss_nt = 0;                 // partials per row (<= 32)
  long ss_ld = 0;                // row stride of one partial plane (>= M)
  float inv_h = 0.f;             // 1 / hidden size
  float eps = 0.f;
  bf16_t* resid = nullptr;       // RESID: residual stream, updated in place
  long ldr = 0;
  float* ss_out = nullptr;       // RESID: [N / 256][ss_out_ld] partial sums of squares
  long ss_out_ld = 0;
  const int* pos = nullptr;      // QKV: positions [M]
  const float* cos_sin = nullptr;  // QKV: [max_pos, D] = [cos(D/2) | sin(D/2)]
  const int* slots = nullptr;    // QKV: cache slot per row (block * bs + offset), -1 = skip
  bf16_t* kc = nullptr;          // QKV: paged caches [num_blocks, hkv, bs, hd]
  bf16_t* vc = nullptr;
  int bs = 0, hq = 0, hkv = 0, hd = 0;
  // grouped form only (gemm_grouped_kernel): tile row j of the expert reads X row gather[j] (null: row j of the
  // expert's own rows) and writes out row scatter[j] (null: row j); x_rows = rows of X behind the gather
  const int* gather = nullptr;
  const int* scatter = nullptr;
  long x_rows = 0;
};
// variant: K-loop schedule of gemm.hip (0 / 1 / 2), or 3 = gemm1w.hip (bn 256)
int lk_gemm(const bf16_t* x, long ldx, const bf16_t* w, const bf16_t* bias, int M, int N, int K, int epi, int bn,
            int variant, bf16_t* out, long ldo, hipStream_t st, int ks = 1, float* ws = nullptr,
            const LkEpi* ea = nullptr);

// grouped form of lk_gemm for rows sorted by expert (segment offsets on the device; weights [E, N, K]); no bias, epilogue
// none or SwiGLU.  Needs K % 64 == 0, K >= 128, N % 256 or N % 192 == 0 (SwiGLU: N/2 % 128 == 0)
int lk_gemm_grouped_supported(int N, int K, int swiglu);
int lk_gemm_grouped(const bf16_t* x, long ldx, const bf16_t* w, const int* seg, int E, long rows, int N, int K, int swiglu,
                    bf16_t* out, long ldo, hipStream_t st, const int* gather = nullptr, long x_rows = 0, const int* scatter = nullptr);

// gemm1w.hip: the one-wave-per-SIMD bm x 256 prefill GEMM (hipBLASLt's gfx950 K-loop schedule,
// every lk_gemm epilogue); lk_gemm routes variants 3 / 4 / 5 here (row tile bm = 256 / 192 / 128).
// Needs K % 64 == 0 and >= 3 K-tiles per split, N % 256 == 0 (SwiGLU: N/2 % 128).
// group_m <= 0: LK_GEMM_GROUP_M (4).
// Variants 6 / 7: a column split -- the column tiles that fill whole waves of the CUs on 256-row
// tiles, the remaining (less than a wave) on 128 / 192-row tiles, as two launches.
constexpr int LK_GEMM1W_SPLIT128 = 1, LK_GEMM1W_SPLIT192 = 2;
inline int lk_gemm1w_bm(int variant) {
  return variant == 3 ? 256 : variant == 4 ? 192 : variant == 5 ? 128 : variant == 6 ? LK_GEMM1W_SPLIT128
       : variant == 7 ? LK_GEMM1W_SPLIT192 : 0;
}
// 256-wide column tiles of a variant 6 / 7 split that run on 256-row tiles (0 or all: no split)
int lk_gemm1w_split_cols(int M, int TN, int cus);
int lk_gemm1w_supported(int M, int N, int K, int epi, int ks, int bm = 256);
int lk_gemm1w(const bf16_t* x, long ldx, const bf16_t* w, const bf16_t* bias, int M, int N, int K, int epi,
              bf16_t* out, long ldo, hipStream_t st, int ks, float* ws, const LkEpi* ea, int group_m, int bm = 256);

// rope_kv.hip
int lk_rope_kv(bf16_t* qkv, long qs, const int* positions, const float* cos_sin, long T, int Hq,
               int Hkv, int D, bf16_t* kc, bf16_t* vc, const int* slots, int BS, int neox,
               int write_k_inplace, hipStream_t st);
// RoPE + paged-KV write fused with the split-K reduction of the QKV projection:
// part[S][T][N] f32 -> qkv [T, N] bf16 (q rotated, k as lk_rope_kv leaves it, v) + caches
int lk_splitk_rope_kv(const float* part, int S, bf16_t* qkv, long qs, const int* positions, const float* cos_sin,
                      long T, int Hq, int Hkv, int D, bf16_t* kc, bf16_t* vc, const int* slots, int BS, int neox,
                      int write_k_inplace, hipStream_t st);
int lk_kv_write(const bf16_t* k, long ks, const bf16_t* v, long vs, bf16_t* kc, bf16_t* vc,
                const int* slots, long T, int Hkv, int D, int BS, hipStream_t st);

// attn_decode.hip
int lk_decode_split_size(int B, int Hkv);
int lk_decode_splits(int max_context, int split);
int lk_paged_decode(const bf16_t* q, long qs, const bf16_t* kc, const bf16_t* vc,
                    const int* block_tables, int bt_stride, const int* ctx_lens, bf16_t* out,
                    long os, float* part_o, float* part_ml, int B, int Hq, int Hkv, int D, int BS,
                    int max_splits, int split, float scale, const int* k_start, const float* pp_o,
                    const float* pp_ml, hipStream_t st, int* tickets = nullptr, int reduce = 1);

// attn_prefill.hip
int lk_prefill_rows_per_tile(int G, int D);
int lk_flash_prefill(const bf16_t* q, long qs, const bf16_t* k, const bf16_t* v, long ks, long vs,
                     const int* block_tables, int bt_stride, const int* cu_q, const int* ctx_lens,
                     const int* tile_seq, const int* tile_q0, int ntiles, bf16_t* out, long os,
                     int Hq, int Hkv, int D, int BS, float scale, int causal, int paged,
                     float* part_o, float* part_ml, const int* q_past, hipStream_t st);

// knn.hip
int lk_knn_nblocks(long N);
int lk_knn_partial(const bf16_t* corpus, const float* cnorm, long N, int D, const bf16_t* queries,
                   const float* qnorm, int nq, int K, float* part_s, int* part_i, hipStream_t st);
int lk_knn_score_chunks(long N);
int lk_knn_score_topk(const float* scores, long ld, const float* cnorm, const float* qnorm, long N, int nq, int K,
                      float* part_s, int* part_i, hipStream_t st);
int lk_knn_merge(const float* cand_s, const int* cand_i, int nq, int ncand, int K, float* out_s,
                 int* out_i, hipStream_t st);

// pooling.hip
int lk_pool_normalize(const bf16_t* hidden, long hs, const int* cu, int B, int H, int mode,
                      int normalize, void* out, long os, int out_bf16, hipStream_t st);
int lk_row_norms(const bf16_t* x, long N, int D, float* out, hipStream_t st);

// sampling.hip
// plan: int32 [B flags | B+1 offsets | allowed ids] (ids in [0, V), checked by the caller)
int lk_select_allowed(const void* logits, int is_bf16, long ls, int B, int V, const float* temps,
                      unsigned long long seed, int step, const int* plan, int* out, hipStream_t st);
int lk_select_tokens(const void* logits, int is_bf16, long ls, int B, int V, const float* temps,
                     unsigned long long seed, int step, int* out, hipStream_t st);
// vocab-parallel greedy: per row an order-preserving int64 key of (max value, vocab_lo + argmax)
// (larger = larger value, then lower id); keys_to_ids: the max over W gathered key rows -> ids
int lk_argmax_key(const void* logits, int is_bf16, long ls, int B, int V, int vocab_lo, long long* keys, hipStream_t st);
int lk_keys_to_ids(const long long* keys, int W, int R, int* ids, hipStream_t st);
int lk_repeat_penalty(void* logits, int is_bf16, long ls, int B, const int* window, int W,
                      const float* penalty, hipStream_t st);
// Ollama-default sampling (repeat penalty from a device history ring, top-k, top-p,
// temperature; greedy rows = argmax).  prm: int32 [B, 8] = temperature, top_p, penalty (f32
// bits), top_k, last_n, slot, reset, seed.  hist: int32 [slots, W] ring, hist_len: [slots].
// logits (f32, modified in place by the penalty) -> out int32 [B]; the token is appended to the ring.
int lk_sample(float* logits, long ls, int B, int V, const int* prm, int* hist, int* hist_len, int W,
              unsigned long long seed, int* out, hipStream_t st);

// csrc/marker.hip: a one-wave marker kernel bounding a timed window in kernel traces
int lk_window_mark(int id, hipStream_t st);
// a launch the runtime rejects (2048 threads): returns the LK_CHECK_LAUNCH code, runs nothing
int lk_debug_invalid_launch(hipStream_t st);

// csrc/step_ops.hip: the forward's small per-step gathers (no framework kernels in a step)
int lk_embed_rows(bf16_t* out, const bf16_t* table, const int* ids, long T, int H, long lo, long n_local,
                  hipStream_t st, int strict = 0);
int lk_embed_errors();  // out-of-table ids seen by strict lk_embed_rows since the last call
int lk_scatter_ids(int* ids, const long* dst, const int* prev, const long* src, int n, hipStream_t st);
int lk_gather_rows(bf16_t* out, const bf16_t* x, long xs, const long* idx, long R, int H, hipStream_t st);

// csrc/stream_f32.hip: f32 residual stream (esz = element size of the bf16 / f32 activations)
int lk_embed_pos(const int* ids, const int* positions, const void* tok, int vocab, const void* pos, int max_pos, long rows,
                 int W, float* x, float* copy, int esz, hipStream_t st);
int lk_stream_embed_errors();  // ids / positions outside their tables seen by lk_embed_pos (their rows are zero)
int lk_stream_rmsnorm(float* x, const void* a, long as, const float* a_bias, const void* b, long bs, const float* e, float m, const float* w,
                      float woff, float eps, const long* idx, long out_rows, void* out, long os, int W, int esz,
                      hipStream_t st);
int lk_silu_mul_f32(const float* x, long xs, float* out, long os, long rows, int I, hipStream_t st);
int lk_softcap(const void* in, long is, float cap, float* out, long os, long rows, int V, int esz, hipStream_t st);

// csrc/attn_sigmoid.hip: sigmoid attention with a log-distance penalty (K cache [NB, G, BS, dim], V cache
// [NB, G, vdim, BS])
int lk_sigattn_supported(int H, int G, int dim, int vdim, int BS, int esz);
int lk_unitnorm_kv_write(void* qkv, long qs, long T, int H, int G, int dim, int vdim, int norm_dim, float eps, void* kc, void* vc,
                         const int* slots, int BS, const void* bias, int esz, hipStream_t st);
int lk_sigattn_prefill(const void* q, long qs, const void* kc, const void* vc, const int* bt, int bt_stride,
                       const int* cu_q, const int* ctx_lens, const int* tile_seq, const int* tile_q0, int ntiles, int H,
                       int G, int dim, int vdim, int BS, float scale, const float* r1, const float* r2, const float* pb,
                       void* out, long os, int esz, hipStream_t st);
int lk_sigattn_decode(const void* q, long qs, const void* kc, const void* vc, const int* bt, int bt_stride,
                      const int* ctx_lens, int B, int Z, int H, int G, int dim, int vdim, int BS, float scale,
                      const float* r1, const float* r2, const float* pb, void* out, long os, float* part, int esz,
                      hipStream_t st);

// csrc/ssm.hip: selective state-space mixer (sequences = rows [cu[s], cu[s+1]), state slot slots[s])
int lk_conv_silu(const void* u, long us, int C, int taps, const float* w, const float* bias, void* state, const int* cu,
                 const int* slots, const int* positions, int S, int max_len, void* out, long os, int act, int esz,
                 hipStream_t st);
int lk_ssm_scan(const void* xbc, long xs, const void* dt, long dts, int S, int heads, int P, int N, int groups,
                const float* dt_bias, const float* A_log, const float* D, float* state, const int* cu, const int* slots,
                const int* positions, float* y, long ys, int max_len, int esz, hipStream_t st);
int lk_gated_group_rmsnorm(const float* y, long ys, const void* z, long zs, const float* w, long rows, int inner,
                           int ngroups, float eps, void* out, long os, int esz, hipStream_t st);

// csrc/stream_ln.hip: post-norm f32 stream (x <- LN(alpha x + ls * y) * w + b with an activation-dtype copy), token gather,
// gated tanh-GELU of a fused [gate | up] projection, mean of two RMS-normed branches
int lk_embed_stream(const int* ids, const void* tok, long V, long T, int W, float* x, void* copy, float scale, int esz, hipStream_t st);
int lk_stream_layernorm(float* x, const void* y, long ys, int y_esz, const float* ls, float alpha, const float* w, const float* b,
                        float eps, const long* idx, long rows, void* out, long os, int out_esz, int W, hipStream_t st);
int lk_gelu_tanh_mul(const void* gu, long gs, void* out, long os, long rows, int F, int esz, hipStream_t st);
int lk_dual_rmsnorm_mean(const void* a, long as, const float* wa, const void* b, long bs, const float* wb, float eps, float* out,
                         long rows, int W, int esz, hipStream_t st);

// csrc/delta_scan.hip: S_t = diag(w_t) S_(t-1) - p_t (z_t^T S_(t-1)) + k_t v_t^T, o_t = S_t^T q_t over per-sequence state slots
// (state f32 [slots, H, dk, dv]); operand preparation of the gated and the generalized delta rule; per-head RMS norm with a gate
int lk_delta_scan(const void* q, long qs, const void* k, long ks, const void* v, long vs, int qkv_esz, const float* w, long ws,
                  const float* p, long ps, const float* z, long zs, const float* w_head, float k_scale, float* state,
                  const int* cu, const int* slots, const int* positions, int S, int H, int Hk, int dk, int dv, float* o, long os,
                  int wide, int act, hipStream_t st);
int lk_gated_delta_prep(const void* q, long qs, const void* k, long ks, const void* v, long vs, const void* beta, long bs,
                        const void* dt, long dts, const float* dt_bias, const float* A_log, long T, int H, int Hk, int dk, int dv,
                        float* qn, float* kn, float* vb, float* g, float* p, float* z, int esz, hipStream_t st);
int lk_general_delta_prep(const void* k, long ks, const void* wraw, long wrs, const float* w0, const void* araw, long ars,
                          const float* a_b, long T, int H, int dk, float* w, float* p, float* z, int esz, hipStream_t st);
int lk_head_norm_gate(const float* o, long os, const void* g, long gs, int g_esz, const float* w, long T, int H, int dv, float eps,
                      int kind, void* out, long outs, int out_esz, hipStream_t st);
int lk_tanh_(void* x, long xs, long T, int n, int esz, hipStream_t st);

// csrc/attn_sink.hip: softmax attention with a sink and a position mask (0 causal, 1 chunks, 2 window) over the paged caches
// K [NB, G, BS, dim], V [NB, G, vdim, BS], optionally beside pooled keys / values of whole blocks before a window (pkc, pvc,
// pool); q / k RMS norm + partial rotation, v norm and the cache write
int lk_normrope_kv_write(void* qkv, long qs, long T, int H, int G, int dim, int vdim, int norm_dim, int norm_vdim, const float* qw,
                         const float* kw, int rot, const float* inv_freq, const int* positions, float eps, void* kc, void* vc,
                         const int* slots, int BS, int v_unit, int esz, hipStream_t st);
int lk_sinkattn_prefill(const void* q, long qs, const void* kc, const void* vc, const int* bt, int bt_stride, const int* cu_q,
                        const int* ctx_lens, const int* tile_seq, const int* tile_q0, int ntiles, int H, int G, int dim, int vdim,
                        int BS, const float* hscale, int mkind, int msize, int sink, const void* gate, long gs, int gcol, void* out,
                        long os, const void* pkc, const void* pvc, int pool, int keep, float cap, int gelem, int esz, hipStream_t st);
int lk_sinkattn_decode(const void* q, long qs, const void* kc, const void* vc, const int* bt, int bt_stride, const int* ctx_lens,
                       int B, int Z, int H, int G, int dim, int vdim, int BS, const float* hscale, int mkind, int msize, int sink,
                       const void* gate, long gs, int gcol, void* out, long os, float* part, const void* pkc, const void* pvc,
                       int pool, int keep, float cap, int gelem, int esz, hipStream_t st);

// csrc/window_ops.hip: gated + normed sublayer result into the f32 stream (+ the next norm), RMS norm of a column block,
// pair rotation + key assembly + paged K / V write, pooled (mean) keys / values of finished blocks
int lk_stream_gated_norm(float* x, const void* y, long ys, int parts, const void* g, long gs, const float* gb, const float* wpost,
                         const float* wnext, float eps, void* out, long os, long rows, int W, int esz, hipStream_t st);
int lk_rms_cols(const void* u, long us, int n, const float* w, float eps, void* out, long os, long rows, int esz, hipStream_t st);
int lk_rot_kv_write(void* q, long qs, int H, int qdim, const void* k, long ks, int G, int kdim, const void* sh, long shs, int sdim,
                    const void* v, long vs, int vdim, int rot_off, int rot, const float* freq, float mag, const int* positions,
                    void* kc, void* vc, const int* slots, int BS, int KD, int VD, long T, const void* v2, long v2s, float blend, int esz,
                    hipStream_t st);
int lk_pool_kv_write(const void* kc, const void* vc, void* pkc, void* pvc, int P, const int* bt, int bt_stride, const int* ctx_lens,
                     const int* cu_q, const int* slots, int row0, int S, int max_len, int G, int BS, int dim, int vdim, int esz,
                     hipStream_t st);

// csrc/parallel_ops.hip: sum of a parallel block's results into the f32 stream + the next block's two norms, f32 router with
// group-limited top-k, clamped gated activation, element-wise silu / sigmoid gate in place
int lk_stream_parallel_norm(float* x, const void* a, long as, const void* b, long bs, const void* y, long ys, const float* yw, int top,
                            const float* w1, const float* w2, float eps, void* o1, long o1s, void* o2, long o2s, long rows, int W,
                            int esz, hipStream_t st);
int lk_router_topk(const void* h, long hs, const float* wr, int E, int W, long rows, int top, int groups, int keep, float scale,
                   int* experts, float* weights, int esz, hipStream_t st);
int lk_clamped_glu(const void* gu, long gs, void* out, long os, long rows, int F, float limit, float alpha, int esz, hipStream_t st);
int lk_silu_(void* x, long xs, long rows, int n, int esz, hipStream_t st);
int lk_sigmoid_mul_(void* x, long xs, const void* g, long gs, long rows, int n, int esz, hipStream_t st);

// csrc/moe.hip: experts chosen by a table of token ids: pairs sorted by expert on the device, grouped MFMA products
int lk_moe_route(const int* ids, const int* table, int vocab, int top, int E, int T, int* seg, int* order, hipStream_t st);
int lk_moe_gemm(const void* x, long xs, const int* order, const int* seg, int E, int top, long pairs, const void* w, int N, int K,
                int act, void* out, long os, int esz, hipStream_t st);

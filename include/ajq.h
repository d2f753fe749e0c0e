/*
 * ajq -- MI355X (gfx950) quantized linear: quantize/pack, decode GEMV, prefill GEMM.
 *
 * C ABI of libajq.so.  Every pointer is a DEVICE pointer owned by the caller
 * (in practice a PyTorch-ROCm tensor's data_ptr); the library never allocates,
 * frees or keeps a pointer past the call.  Every compute entry point is
 * asynchronous: it enqueues on `stream` (a hipStream_t, e.g.
 * torch.cuda.current_stream().cuda_stream; NULL = the default stream) and
 * returns without a host sync.  Return value: 0 on success, a negative
 * ajq_status otherwise; ajq_last_error() gives the thread-local message.
 *
 * The reference project (Huangsj1/ajLLM) has exactly one linear operator,
 *     Linear.forward:  inputs @ weight.transpose(-2, -1)
 *     (src/ajllm/modeling/layers.py:9-33)
 * and no quantized path, so there is no reference FFI to mirror; these entry
 * points are what a quantized twin of that operator binds.  Each declaration
 * names the reference call it stands behind.
 *
 * Canonical interchange tensors (what "bit-exact" compares):
 *   W8 : q       int8   [N, K]       row-major
 *        scales  fp16   [N]
 *   W4 : qweight int32  [N, K/8]     word c of row n = sum_j q[n, 8c+j] << 4j
 *        scales  fp16   [N, K/128]
 *        zeros   uint8  [N, K/128]   values 0..15
 * Kernel-private tensors (made by ajq_repack_*, restored bit-for-bit by
 * ajq_unrepack_*):
 *   W4 : wq   uint32 [N/16, K/128, 64, 4]   one 1 KiB tile = 16 rows x 128 k,
 *             element (lane = 16*kc + nl, dword j) holds the 8 weights
 *             n = 16*tile_n + nl, k = 128*g + 32*j + 8*kc + e (e = 0..7) with
 *             weight e in nibble (e>>1) + 4*(e&1)
 *        meta uint32 [N/16, K/128, 16]      fp16 scale bits | fp16(128+zero) << 16
 *   W8 : wq   uint32 [N/16, K/64, 64, 4]    tile = 16 rows x 64 k; lane (kc, nl)
 *             holds bytes k = 64*t + 32*j + 8*kc + e for j = 0,1 in k order
 *             (dword 2j+0: e=0..3, dword 2j+1: e=4..7), int8 unchanged
 */
#ifndef AJQ_H
#define AJQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum ajq_status {
  AJQ_OK = 0,
  AJQ_ERR_NULL = -1,        /* a required pointer is NULL */
  AJQ_ERR_SHAPE = -2,       /* N, K or M outside what the kernel supports */
  AJQ_ERR_ALIGN = -3,       /* a pointer is not 16-byte aligned */
  AJQ_ERR_UNSUPPORTED = -4, /* flag / dtype combination not implemented */
  AJQ_ERR_HIP = -5,         /* the HIP runtime reported an error at launch */
  AJQ_ERR_WORKSPACE = -6    /* workspace missing or too small */
} ajq_status;

/* output element type of the matmul entry points */
#define AJQ_OUT_BF16 0
#define AJQ_OUT_F32 1 /* same accumulation, final cast skipped (parity checks) */

/* element type of the key/value caches of the decode-step operators */
#define AJQ_KV_F32 0
#define AJQ_KV_BF16 1 /* rounded to nearest even on write; attention still computes in fp32 */

/* The w1 | w3 matmul of a SwiGLU feed-forward with the gate formed in its epilogue:
 * wq / meta / scales are the private tensors of the 2 F rows (w1's F rows, then w3's: the
 * concatenation of the two layers' tensors), y[M, F] = bf16( silu(x w1^T) * (x w3^T) )
 * (SwiGLU.forward, src/ajllm/modeling/activations.py:24-25, up to its down projection); equal bit
 * for bit to ajq_w*a16_gemm with fp32 output followed by ajq_swiglu, without the [M, 2 F] fp32
 * intermediate.  Tile kernels only: ajq_gemm_gate_supported(M, 2 F, K, w4) says whether the shape
 * qualifies (M >= 128, F a multiple of 64, large enough for the tile kernels); the W4 form needs
 * the workspace of ajq_w4a16_gemm_workspace_bytes(M, K). */
int ajq_gemm_gate_supported(int M, int N2, int K, int w4);
int ajq_w4a16_gemm_gate(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta, int N2,
                        uint16_t* y, void* workspace, size_t workspace_bytes, void* stream);
int ajq_w8a16_gemm_gate(const uint16_t* x, int M, int K, const uint32_t* wq, const uint16_t* scales, int N2,
                        uint16_t* y, void* stream);

int ajq_version(void);
const char* ajq_last_error(void);
const char* ajq_status_string(int status);

/* ---- quantize / pack (stands behind Linear.__init__'s fp32 weight[out, in],
 *      src/ajllm/modeling/layers.py:19-30) -------------------------------- */

/* W fp32 [N, K] -> q int8 [N, K], scales fp16 [N].  K % 4 == 0. */
int ajq_quantize_w8(const float* W, int N, int K, int8_t* q, uint16_t* scales, void* stream);

/* W fp32 [N, K] -> qweight int32 [N, K/8], scales fp16 [N, K/128],
 * zeros uint8 [N, K/128].  K % 128 == 0. */
int ajq_quantize_w4_g128(const float* W, int N, int K, int32_t* qweight, uint16_t* scales,
                         uint8_t* zeros, void* stream);

/* canonical -> kernel-private layout and back.  N % 16 == 0; K % 128 == 0 for W4,
 * K % 64 == 0 for W8 (the W8 matmuls below additionally need K % 128 == 0). */
int ajq_repack_w4(const int32_t* qweight, const uint16_t* scales, const uint8_t* zeros, int N, int K,
                  uint32_t* wq, uint32_t* meta, void* stream);
int ajq_unrepack_w4(const uint32_t* wq, const uint32_t* meta, int N, int K, int32_t* qweight,
                    uint16_t* scales, uint8_t* zeros, void* stream);
int ajq_repack_w8(const int8_t* q, int N, int K, uint32_t* wq, void* stream);
int ajq_unrepack_w8(const uint32_t* wq, int N, int K, int8_t* q, void* stream);

/* ---- fused dequantize-matmul (stands behind Linear.forward,
 *      src/ajllm/modeling/layers.py:32-33: y[M, N] = x[M, K] @ W_hat[N, K]^T) ---
 * x bf16 [M, K] row-major, y bf16 or fp32 [M, N] row-major (out_dtype).
 * fp32 accumulation; scales applied in fp32; the bf16 cast is round-to-nearest-even.
 */

/* decode shapes, 1 <= M <= 16; HBM-bound */
int ajq_w4a16_gemv(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta, int N,
                   void* y, int out_dtype, void* stream);
int ajq_w8a16_gemv(const uint16_t* x, int M, int K, const uint32_t* wq, const uint16_t* scales, int N,
                   void* y, int out_dtype, void* stream);

/* The same GEMV with its activations produced on the way in (one launch less per use):
 *   _norm: x = bf16(RMSNorm(h_in + delta) * gain) and h_out = h_in + delta (delta may be NULL;
 *          h_out must not be h_in) -- the residual add and RMSNorm of TransformerBlock.forward
 *          (src/ajllm/modeling/transformer.py:45-50, layers.py:70-74) in front of q|k|v or w1|w3;
 *   _gate: x = bf16(silu(a) * u) for ab[M, 2K] = (a | u) -- SwiGLU.forward's product
 *          (src/ajllm/modeling/activations.py:24-25) in front of w2.
 * Built for the (M, K) that ajq_gemv_fused_supported reports: K = 1024 and 2048 (M <= 16), 4096
 * and 5632 (M <= 8); AJQ_ERR_UNSUPPORTED otherwise (use the separate operators below). */
int ajq_gemv_fused_supported(int M, int K);
int ajq_w4a16_gemv_norm(const float* h_in, const float* delta, const float* gain, float eps, float* h_out,
                        int M, int K, const uint32_t* wq, const uint32_t* meta, int N, void* y,
                        int out_dtype, void* stream);
int ajq_w8a16_gemv_norm(const float* h_in, const float* delta, const float* gain, float eps, float* h_out,
                        int M, int K, const uint32_t* wq, const uint16_t* scales, int N, void* y,
                        int out_dtype, void* stream);
int ajq_w4a16_gemv_gate(const float* ab, int M, int K, const uint32_t* wq, const uint32_t* meta, int N,
                        void* y, int out_dtype, void* stream);
int ajq_w8a16_gemv_gate(const float* ab, int M, int K, const uint32_t* wq, const uint16_t* scales, int N,
                        void* y, int out_dtype, void* stream);
/* The same GEMV with work around the matmul, for decode steps, where a launch of its own
 * for the residual add, the RMSNorm or the SwiGLU gate costs more than the operation itself
 * (TransformerBlock.forward, src/ajllm/modeling/transformer.py:45-50; RMSNorm, layers.py:70-74; SwiGLU,
 * activations.py:24-25).  The row scale of an RMSNorm commutes with the matmul, so the pair below computes
 *     h_out = h_in + x W1^T ;   y = (RMSNorm(h_out) * gain) W2^T
 * in two launches, without a norm kernel between them:
 *   _residual: h_out[M, N] = h_in + x W^T (fp32; h_out must not be h_in), xt_out = bf16(h_out * gain)
 *              (gain[N]: of the norm that follows) and ssq_out[max(16, M)][N / 16]: per row, the sum of squares of
 *              h_out over each 16-column tile (rows >= M are not written);
 *   _rowscale: y = rstd[m] * (xt W^T) with rstd[m] = rsqrt(sum(ssq[m][0 .. parts)) / K + eps), ssq laid out
 *              [max(16, M)][parts] as _residual leaves it; parts must be K / 16 and at most 256 (K <= 4096), or 352
 *              for K = 5632 with M <= 8: ajq_gemv_rowscale_supported reports whether (M, K) is taken.  gate != 0: the rows of W are tiles of 8 gate-projection rows followed by the 8
 *              matching up-projection rows (w1 and w3 interleaved in blocks of 8) and
 *              y[M, N / 2] = bf16(silu(a) * u), out_dtype AJQ_OUT_BF16.
 * xt is rounded to bf16 BEFORE the row scale is applied (the reference order rounds the normalised value);
 * both are one bf16 rounding of the same quantity up to the fp32 factor rstd.  Sums run in a fixed order:
 * results are run-to-run identical.  Built for the (M, K) that ajq_gemv_epilogue_supported reports: 1 <= M <= 255,
 * K % 128 == 0 (the GEMV kernel for M <= 16 with K = 2048 or 4096 and M <= 8 with K = 5632, the weight-streaming
 * kernel otherwise; ssq has max(16, M) rows); AJQ_ERR_UNSUPPORTED otherwise.  _rowscale is built for the narrower
 * set that ajq_gemv_rowscale_supported reports (its K is the width whose K / 16 tile sums it adds up): the
 * _residual -> _rowscale pair needs both queries to say yes, the first for the producer's (M, K), the second
 * for the consumer's. */
int ajq_gemv_epilogue_supported(int M, int K);
int ajq_gemv_rowscale_supported(int M, int K);
int ajq_w4a16_gemv_residual(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta, int N,
                            const float* h_in, const float* gain, float* h_out, uint16_t* xt_out, float* ssq_out,
                            void* stream);
int ajq_w8a16_gemv_residual(const uint16_t* x, int M, int K, const uint32_t* wq, const uint16_t* scales, int N,
                            const float* h_in, const float* gain, float* h_out, uint16_t* xt_out, float* ssq_out,
                            void* stream);
int ajq_w4a16_gemv_rowscale(const uint16_t* xt, const float* ssq, int parts, float eps, int M, int K,
                            const uint32_t* wq, const uint32_t* meta, int N, void* y, int out_dtype, int gate,
                            void* stream);
int ajq_w8a16_gemv_rowscale(const uint16_t* xt, const float* ssq, int parts, float eps, int M, int K,
                            const uint32_t* wq, const uint16_t* scales, int N, void* y, int out_dtype, int gate,
                            void* stream);
/*   _gated:    y[M, N / 2] = bf16(silu(a) * u) for the plain bf16 activations x, the rows of W interleaved as for
 *              _rowscale's gate: w1|w3 with SwiGLU's product in its epilogue (activations.py:24-25), no row scale. */
int ajq_w4a16_gemv_gated(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta, int N, void* y,
                         void* stream);
int ajq_w8a16_gemv_gated(const uint16_t* x, int M, int K, const uint32_t* wq, const uint16_t* scales, int N, void* y,
                         void* stream);
/*   _norm_sums: y = (RMSNorm(h) * gain) W^T with the activations rounded exactly where the reference rounds them,
 *              bf16((h / rms) * gain) (layers.py:70-74 then the bf16 input of the quantized linear), rms taken from
 *              the sums of squares that _residual left in ssq ([rows][parts], parts = K / 16 <= 256): the GEMV with a
 *              norm prologue (ajq_w*a16_gemv_norm) without the add, without the reduction and without its
 *              workgroup barrier.  h is _residual's h_out (fp32 [M, K]); gate as in _rowscale.  Built for the (M, K)
 *              of ajq_gemv_fused_supported.  _residual's xt_out may be NULL when only this consumer follows. */
int ajq_w4a16_gemv_norm_sums(const float* h, const float* ssq, int parts, const float* gain, float eps, int M, int K,
                             const uint32_t* wq, const uint32_t* meta, int N, void* y, int out_dtype, int gate,
                             void* stream);
int ajq_w8a16_gemv_norm_sums(const float* h, const float* ssq, int parts, const float* gain, float eps, int M, int K,
                             const uint32_t* wq, const uint16_t* scales, int N, void* y, int out_dtype, int gate,
                             void* stream);
/*   _merge_residual: _residual whose x is the single-query attention output merged from the S partial results
 *              per (row, head) in ajq_attn_step_partial's workspace, as in _merge below (same limits:
 *              ajq_gemv_merge_max_splits): the output projection of a decode step at small batch, with the
 *              merge on its way in and the residual add and the next norm's preparation on its way out. */
int ajq_w4a16_gemv_merge_residual(const float* partial, int S, int M, int K, const uint32_t* wq, const uint32_t* meta,
                                  int N, const float* h_in, const float* gain, float* h_out, uint16_t* xt_out,
                                  float* ssq_out, void* stream);
int ajq_w8a16_gemv_merge_residual(const float* partial, int S, int M, int K, const uint32_t* wq, const uint16_t* scales,
                                  int N, const float* h_in, const float* gain, float* h_out, uint16_t* xt_out,
                                  float* ssq_out, void* stream);
/*   _merge: x = bf16 of the single-query attention output [M, K] (K = heads * 128), merged from the S
 *          partial results per (row, head) that ajq_attn_step_partial left in its workspace -- the
 *          softmax-weighted value sum of scaled_dot_product_attention (src/ajllm/modeling/attention.py:20-33)
 *          in front of output_proj (attention.py:120).  ajq_gemv_merge_max_splits(M, K) is the largest S
 *          built for the shape (0: not built; K = 2048 with M <= 4, K = 4096 with M <= 2). */
int ajq_gemv_merge_max_splits(int M, int K);
int ajq_w4a16_gemv_merge(const float* partial, int S, int M, int K, const uint32_t* wq, const uint32_t* meta, int N,
                         void* y, int out_dtype, void* stream);
int ajq_w8a16_gemv_merge(const float* partial, int S, int M, int K, const uint32_t* wq, const uint16_t* scales, int N,
                         void* y, int out_dtype, void* stream);

/* any M >= 1; bf16 MFMA.  M <= 16 runs the GEMV above, 17 <= M < 128 (several sequences decoded
 * together) a weight-streaming kernel with 32-row activation blocks, and from M = 128 on the
 * fastest by a measured cost model of that kernel, a 128 x 128 tile kernel (shapes with few
 * tiles) and a 256 x 128 tile kernel (M >= 256, prefill).
 * Of the W4 kernels only the 128 x 128 tile kernel needs a workspace (per-row, per-group activation sums): the
 * 256 x 128 tile kernel subtracts the zero-points when it unpacks the weights and runs as one launch.
 * ajq_w4a16_gemm_workspace_bytes_for(M, N, K) is what a call on that shape needs (0 unless the 128 x 128 kernel
 * is chosen; workspace may then be NULL); ajq_w4a16_gemm_workspace_bytes(M, K) is its upper bound over all N
 * (0 below M = 128). */
size_t ajq_w4a16_gemm_workspace_bytes(int M, int K);
size_t ajq_w4a16_gemm_workspace_bytes_for(int M, int N, int K);
int ajq_w4a16_gemm(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta, int N,
                   void* y, int out_dtype, void* workspace, size_t workspace_bytes, void* stream);
int ajq_w8a16_gemm(const uint16_t* x, int M, int K, const uint32_t* wq, const uint16_t* scales, int N,
                   void* y, int out_dtype, void* stream);

/* A device buffer lent to the matmul entry points called from THIS host thread (all of ajq_w*a16_gemm, _gemv, _gemv_residual,
 * _gemv_gated, _gemv_rowscale, _gemv_norm_sums), for the split-K forms of the weight-streaming kernels: at 17 <= M <= 32
 * with K >= 8192, and at 9 <= M <= 16 with K = 14336, both with N <= 4096 (the down projection of a SwiGLU feed-forward
 * in a batched decode step), four workgroups share four row tiles and a quarter of K each, exchange their partial sums
 * through this buffer and the last one to arrive adds them in a fixed order (results are run-to-run identical; they differ from the unsplit kernel's in the
 * last bits, the sum being associated differently).  No counterpart in the reference.
 *   - ajq_matmul_workspace_bytes() bytes, 16-byte aligned; its first 4096 bytes must be ZERO when it is lent (the
 *     kernels leave them zero) and the buffer must stay allocated while launches that were given it can still run
 *     (HIP graphs recorded while it was set included);
 *   - launches that share one buffer must not overlap in time (one stream, or streams that are ordered): a second
 *     stream or host thread takes a buffer of its own;
 *   - workspace == NULL ends the loan (the state is per host thread; nothing is set initially, and without a buffer
 *     every shape runs the kernels that need none). */
size_t ajq_matmul_workspace_bytes(void);
int ajq_matmul_workspace_set(void* workspace, size_t bytes);

/* ajq_w4a16_gemm for callers that cannot allocate device memory or pass a workspace (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the group sums live in
 * a 16 MiB array inside the library's code object, one copy per GPU, held until the process ends
 * (ajq_noalloc_scratch_bytes() returns its size).  No counterpart in the reference.  The call
 * allocates and frees nothing; shapes whose ajq_w4a16_gemm_workspace_bytes(M, K) exceeds the
 * array return AJQ_ERR_WORKSPACE.  All calls on one GPU share the array: two calls that overlap
 * in time on one GPU (different streams, or threads) race on it; calls on one stream do not.
 * The first call on a device resolves the array's address and should not run under capture.  The array used is
 * the CURRENT device's (hipGetDevice at the time of the call): that device must be the one `stream` and every
 * pointer belong to. */
size_t ajq_noalloc_scratch_bytes(void);
int ajq_w4a16_gemm_noalloc(const uint16_t* x, int M, int K, const uint32_t* wq, const uint32_t* meta, int N,
                           void* y, int out_dtype, void* stream);

/* ---- the small operators of one decode step around the linears -------------------
 * fp32 residual stream; fp32 or bf16 KV cache (cache_dtype); outputs that feed a linear are bf16.  `pos` is a
 * DEVICE pointer to the step's cache row, so a recorded HIP graph replays per token. */

/* hidden[B, D] += delta[B, D] (delta may be NULL), out = bf16(RMSNorm(hidden) * gain)
 * (RMSNorm.forward, src/ajllm/modeling/layers.py:70-74, with the residual add of
 * TransformerBlock.forward, src/ajllm/modeling/transformer.py:45-50, in front). */
int ajq_add_rmsnorm(float* hidden, const float* delta, const float* gain, float eps, uint16_t* out,
                    int B, int D, void* stream);

/* qkv[B, (H + 2 Hkv) * head_dim] -> rotated q[B, H, head_dim]; rotated k and v go to row
 * *pos of the caches [B, Hkv, max_len, head_dim].  Interleaved-pair rotation with the
 * cosine / sine tables [positions, head_dim / 2] (RotaryPositionalEmbedding.forward,
 * src/ajllm/modeling/attention.py:36-60).  The reference has no KV cache
 * (src/ajllm/generation/generator.py:20-27 recomputes the sequence): the cache is this build's. */
int ajq_rope_cache(const float* qkv, const float* cosine, const float* sine, const int64_t* pos,
                   float* q_out, void* kcache, void* vcache, int cache_dtype, int B, int H, int Hkv,
                   int head_dim, int max_len, void* stream);

/* The same rotation for T new positions per sequence (prefill): qkv[B * T, (H + 2 Hkv) * head_dim],
 * row b * T + t at absolute position start + t; rotated queries to q_out[B, H, T, head_dim] (what
 * ajq_attn_prefill reads), rotated keys and values to rows start + t of the caches. */
int ajq_rope_prefill(const float* qkv, const float* cosine, const float* sine, float* q_out, void* kcache,
                     void* vcache, int cache_dtype, int B, int T, int H, int Hkv, int head_dim, int start,
                     int max_len, void* stream);

/* single-query softmax attention over cache rows 0 .. *pos, out bf16 [B, H * head_dim]
 * (scaled_dot_product_attention, src/ajllm/modeling/attention.py:20-33, for one query row;
 * H / Hkv = 1, 2 or 4 query heads share a cache head, whose rows are read once for all of
 * them).  head_dim 128, 64 (the reference's configs/models/transformer_medium.yaml: 768 / 12 heads) or 32
 * (transformer_baseline.yaml: 512 / 16 heads).
 * The workspace holds the partial results of up to 16 row chunks. */
size_t ajq_attn_decode_workspace_bytes(int B, int H);
/* Row chunks per cache head that ajq_attn_decode and ajq_attn_step use for this shape (0: bad shape).  With 1
 * the attention is a single launch (no merge kernel; the workspace is not touched): any shape with at least 256
 * (sequence, cache head) pairs, where one workgroup reads a whole head. */
int ajq_attn_row_chunks(int B, int Hkv, int max_len);
int ajq_attn_decode(const float* q, const void* kcache, const void* vcache, int cache_dtype,
                    const int64_t* pos, int B, int H, int Hkv, int head_dim, int max_len, uint16_t* out,
                    void* workspace, size_t workspace_bytes, void* stream);

/* The two operators above in one kernel: qkv as for ajq_rope_cache; the step's key and value
 * rows are written to row *pos of the caches and attended to from registers.  head_dim 128, 64 or 32. */
size_t ajq_attn_step_workspace_bytes(int B, int H);
int ajq_attn_step(const float* qkv, const float* cosine, const float* sine, const int64_t* pos,
                  void* kcache, void* vcache, int cache_dtype, int B, int H, int Hkv, int head_dim,
                  int max_len, uint16_t* out, void* workspace, size_t workspace_bytes, void* stream);

/* ajq_attn_step without the merge of its row chunks: the S partial results per (sequence, query
 * head) stay in the workspace as records of 132 floats (maximum as a base-2 exponent, denominator,
 * two pad words, 128 weighted value sums) for ajq_w*a16_gemv_merge, the output projection that
 * merges them on its way in (one launch less per layer).  At most max_splits chunks are used (what
 * ajq_gemv_merge_max_splits allows for the batch); *splits (host memory) receives S.  head_dim 128 only
 * (the record layout ajq_w*a16_gemv_merge reads). */
int ajq_attn_step_partial(const float* qkv, const float* cosine, const float* sine, const int64_t* pos,
                          void* kcache, void* vcache, int cache_dtype, int B, int H, int Hkv, int head_dim,
                          int max_len, int max_splits, int* splits, void* workspace, size_t workspace_bytes,
                          void* stream);

/* ab[B, 2F] = (w1 x | w3 x) -> out[B, F] = bf16(silu(w1 x) * w3 x)
 * (SwiGLU.forward, src/ajllm/modeling/activations.py:24-25, between its linears). */
int ajq_swiglu(const float* ab, uint16_t* out, int B, int F, void* stream);

/* Causal attention of T new positions (absolute positions start .. start + T - 1) over cache
 * rows 0 .. start + T - 1, which the caller has already written; q fp32 [B, H, T, head_dim]
 * (rotated), out [B, T, H * head_dim] fp32 or bf16 (out_dtype: AJQ_OUT_F32 / AJQ_OUT_BF16, the
 * rounding of the fp32 result).  Flash-attention arithmetic: bf16 MFMA products,
 * fp32 online softmax, no T x T matrix (scaled_dot_product_attention under a causal mask,
 * src/ajllm/modeling/attention.py:20-33,106-117; the reference's own tiled and Triton variants,
 * src/ajllm/modeling/flash_attention.py:44-108,194-298, are CUDA-gated).  head_dim 128, 64 or 32 (the head sizes of
 * the benchmark models and of the reference's configs/models/transformer_medium.yaml and transformer_baseline.yaml). */
int ajq_attn_prefill(const float* q, const void* kcache, const void* vcache, int cache_dtype, int B, int H,
                     int Hkv, int T, int start, int max_len, int head_dim, void* out, int out_dtype, void* stream);

/* Greedy choice at the end of a decode step: token[b] = argmax(logits[b, 0..V)) (row stride ld;
 * the lowest index among equal maxima: next = argmax(logits[:, -1]) of generate,
 * src/ajllm/generation/generator.py:20-27, sampling.py:9-10), also stored at out[b, *step] (row
 * stride out_ld), and hidden[b, :] = embedding[token[b], :] (Embedding.forward,
 * src/ajllm/modeling/layers.py:52-53), the next step's input.  token, out, step: int64. */
int ajq_greedy_pick(const float* logits, int B, int V, int ld, const float* embedding, int D, float* hidden,
                    int64_t* token, int64_t* out, int out_ld, const int64_t* step, int64_t* advance, uint32_t* ticket,
                    void* stream);

/* Temperature / nucleus sampling at the end of a decode step (sample_next_token,
 * src/ajllm/generation/sampling.py:8-22: p = softmax(logits / temperature); with top_p < 1 the tokens whose
 * probability mass strictly above them, in descending order, is below top_p are kept; the choice is drawn from the
 * kept tokens in proportion to p) with ajq_greedy_pick's outputs.  temperature > 0 (the reference's
 * temperature <= 0 is ajq_greedy_pick); top_p in (0, 1], 1 = no filter.  The draw is the inverse CDF over the kept
 * tokens in INDEX order at u = uniforms[min(*step, uniform_rows - 1), b] (fp32 [uniform_rows, B], each in [0, 1):
 * the caller's random numbers, so a recorded HIP graph replays with fresh ones per step); the reference draws with
 * torch.multinomial, the same distribution from other random bits.  Probabilities are compared and added as
 * 40-bit fixed-point integers: equal inputs give equal tokens.  embedding / hidden may both be NULL (no embedding row
 * is fetched); kept (optional, int32 [B]) receives the number of tokens the filter kept.  V <= 1048576; ld % 4 == 0
 * and logits 16-byte aligned. */
int ajq_sample_pick(const float* logits, int B, int V, int ld, float temperature, float top_p, const float* uniforms,
                    int uniform_rows, const float* embedding, int D, float* hidden, int64_t* token, int64_t* out,
                    int out_ld, const int64_t* step, int64_t* advance, uint32_t* ticket, int32_t* kept, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* AJQ_H */

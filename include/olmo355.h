/*
 * olmo355 -- C-ABI of the MI355X (gfx950) kernels behind the OLMo inference forward pass.
 *
 * Conventions, every entry point:
 *   - plain pointers and sizes only; every pointer is a *device* pointer borrowed for the
 *     duration of the call (nothing is allocated, freed or kept by the library);
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); kernels are
 *     launched on it asynchronously and the call returns without synchronising;
 *   - returns 0 on success, else an O355_E* code; olmo355_status_string() names it.  No
 *     kernel is launched when an argument check fails;
 *   - no process-global state: safe from any host thread that has made its device current
 *     (one stated exception: olmo355_attn_decode_static, which owns a fixed device scratch array);
 *   - `dtype` is the activation dtype: O355_F32, O355_BF16 or O355_F16.  Every element-wise, attention,
 *     sampling and beam entry point takes all three; the fused decode forms (chained norms, relay,
 *     fused merge, key-split prefill attention) are bf16 only and say so where they are declared.
 *
 * Each declaration cites the reference interface it stands in for.  Paths are relative to
 * the reference tree; "AGQ/" = inference/compression/dependencies/AutoGPTQ/.
 */
#ifndef OLMO355_H
#define OLMO355_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define O355_OK 0
#define O355_EINVAL 1       /* null pointer, non-positive or misaligned size */
#define O355_EUNSUPPORTED 2 /* shape / dtype / group size outside what the kernel handles */
#define O355_ELAUNCH 3      /* hipGetLastError() != hipSuccess after the launch */
#define O355_ETOOBIG 4      /* sizes beyond the fixed scratch of an entry point that allocates nothing */

#define O355_F32 0
#define O355_BF16 1
#define O355_F16 2

int olmo355_version(void);
const char* olmo355_status_string(int status);

/* ---- int4 group-wise weights ------------------------------------------------------------
 * Checkpoint layout (AGQ/auto_gptq/nn_modules/qlinear/qlinear_cuda_old.py:48-67):
 *   qweight int32 [K/8, N]   nibble j of qweight[r][n] is q[8r+j][n]
 *   qzeros  int32 [K/g, N/8] nibble j of qzeros[G][c] is the stored zero of column 8c+j
 *   scales  fp16  [K/g, N]
 *   g_idx   int32 [K]        group of row k; NULL means k / group
 * Tiled layout ("w4t", built once by olmo355_w4_repack, K % 128 == 0, N % 16 == 0, group 128):
 *   wt  uint32 [N/16][K/128][64 lanes][4]  lane l, word j: column 16*nt + (l&15), rows
 *        128*g + 32*j + 8*(l>>4) + e, e = 0..7; nibble p of the word holds e = 2p (p<4) or
 *        2(p-4)+1 (p>=4), i.e. one MFMA 16x16x32 operand fragment per word
 *   st  fp16  [N/16][K/128][16]  scale of column 16*nt + c
 *   zt  uint8 [N/16][K/128][8]   stored-zero nibbles of the 16 columns, low nibble first
 */

/* Dense fp16 table W[K,N] = fp16(scale * (q - (zero_stored + 1))), bit-exact with the
 * reference's torch dequantize: AGQ qlinear_cuda_old.py:236-285 (g_idx == NULL) and
 * qlinear_cuda.py:211-265 (g_idx given).  Also what exllama's reconstruct kernel produces
 * (AGQ/autogptq_extension/exllama/cuda_func/q4_matrix.cu:171-225).  K % 8 == 0, N % 8 == 0,
 * group % 8 == 0 when g_idx is NULL. */
int olmo355_w4_dequant_fp16(const int32_t* qweight, const int32_t* qzeros, const uint16_t* scales,
                            const int32_t* g_idx, uint16_t* out_kn, int K, int N, int group, void* stream);

/* One-time re-tiling of a checkpoint-layout weight into the w4t layout; the counterpart of
 * the reference's post_init hook that rewrites qweight for its kernels
 * (AGQ qlinear_exllama.py:85-98, q4_matrix.cu:105-169). */
int olmo355_w4_repack(const int32_t* qweight, const int32_t* qzeros, const uint16_t* scales, uint32_t* wt,
                      uint16_t* st, uint8_t* zt, int K, int N, int group, void* stream);

/* Same table as olmo355_w4_dequant_fp16, read from the tiled layout (checks the repack). */
int olmo355_w4t_dequant_fp16(const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* out_kn, int K,
                             int N, void* stream);

/* y[M,N] = x[M,K] . W[K,N], bf16 in / bf16 out, fp32 accumulation, W = scale*(q-zero) exact.
 * Small-M path (M <= 64): stands in for vecquant4matmul_faster_old
 * (AGQ/autogptq_extension/cuda_256/autogptq_cuda_256.cpp:158-171, kernel
 * autogptq_cuda_kernel_256.cu:1365-1435) and exllama's q4_matmul GEMV
 * (exllama/cuda_func/q4_matmul.cu:32-143).  Deterministic: no atomics, fixed summation order. */
int olmo355_w4_gemv(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y,
                    int M, int N, int K, void* stream);

/* The same product with up to two neighbouring steps of a decode block folded in (M <= 16):
 *   resid != NULL: the activations are first formed as x' = resid + rmsnorm(x; norm_w, eps) -- the
 *     post-norm residual update that precedes att_proj / ff_proj (olmo/model.py:786-794,814-821),
 *     with RMSLayerNorm's rounding points (olmo/model.py:241-255) -- and also written to x_out [M,K];
 *   swiglu != 0: y [M, N/2] = silu(gate) * up of the two halves of the product (olmo/model.py:365-368).
 * Returns O355_EUNSUPPORTED for shapes the fused kernels do not cover (the caller then issues the
 * separate kernels). */
int olmo355_w4_gemv_fused(const uint16_t* x, const uint16_t* resid, const uint16_t* norm_w, float eps,
                          uint16_t* x_out, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y,
                          int M, int N, int K, int swiglu, void* stream);

/* olmo355_w4_gemv_fused for M <= 8 with the norms chained between launches: RMSNorm needs the sum
 * of squares of a whole row, and the launch that *produces* that row can leave it behind per 16-column
 * tile, so the consumer's prologue neither re-reads the row nor synchronises its workgroup.
 *   ssq_out != NULL (swiglu == 0): ssq_out[m][N/16] = sum of squares of the bf16 outputs of row m, per tile;
 *   resid != NULL: ssq_in[m][K/16] (left by the launch that wrote x) must be given; x' as above.
 * Used for the three norms of a decode block (olmo/model.py:786-794 attention/MLP post-norms and the
 * full-width QK-norm of :711-716 via olmo355_attn_decode_fused).  Up to 4 rows keep the activations in LDS; 5 to 8 rows
 * take them as matrix-core operand fragments straight from memory (no size limit from LDS; K up to 12288 without a
 * prologue, 8192 with one).  O355_EUNSUPPORTED: use the calls above. */
int olmo355_w4_gemv_chain(const uint16_t* x, const uint16_t* resid, const uint16_t* norm_w, float eps, uint16_t* x_out,
                          const float* ssq_in, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y,
                          float* ssq_out, int M, int N, int K, int swiglu, void* stream);

/* Large-M path: dequantise tiles into LDS as bf16 and multiply on the matrix cores.  Stands
 * in for the reference's dequantise-then-matmul branch (AGQ qlinear_cuda_old.py:236-287) and
 * exllama's reconstruct + cublasHgemm (exllama/cuda_func/q4_matmul.cu:222-260).
 * The matrix-core entries (this one, olmo355_b16_gemm, the split-K and SwiGLU forms) write 16 bytes at a time:
 * y (and the split-K workspace) must be 16-byte aligned, O355_EINVAL otherwise; N % 16 == 0 keeps every row so. */
int olmo355_w4_gemm(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y,
                    int M, int N, int K, void* stream);
/* Split-K forms of olmo355_w4_gemm / olmo355_b16_gemm for launches with fewer output tiles than CUs (prompts of
 * 65 to a few hundred tokens): `splits` workgroups per 128 x 64 tile, each over its own run of K, fp32 partial
 * sums in `workspace` (splits * M * N floats), added in split order and rounded once by a second kernel.  Same
 * product as the plain entry up to the order of the fp32 additions (QuantLinear.forward's matmul,
 * qlinear_cuda_old.py:287-290; F.linear of the dense layers, olmo/model.py:746-823).
 * olmo355_gemm_splitk_plan returns the number of splits worth using for a shape (1: call the plain entry).
 * Needs K % 256 == 0, N % 64 == 0, 2 <= splits <= K / 256. */
int olmo355_gemm_splitk_plan(int M, int N, int K);
int olmo355_w4_gemm_splitk(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y,
                           int M, int N, int K, int splits, float* workspace, void* stream);
int olmo355_b16_gemm_splitk(const uint16_t* x, const uint16_t* wt, uint16_t* y, int M, int N, int K, int splits,
                            float* workspace, void* stream);

/* Stream-K forms of the same products for row counts whose 256 x 256 tiles do not fill a whole number of rounds of
 * the CUs (one prompt of 2048 tokens: 384 tiles for att_proj, 128 for attn_out and ff_out): one workgroup per CU,
 * the tiles' K runs (units of 256) dealt out evenly, so a tile's K may be shared by two or three workgroups; the one
 * that ends it adds the others' fp32 partials (in a fixed order: results are reproducible, and differ from the
 * tiled entry only in the order of fp32 additions) and writes the output.  Same product as QuantLinear.forward's
 * matmul (qlinear_cuda_old.py:287-290) / F.linear (olmo/model.py:746-823).
 * `workspace`: ws_bytes >= olmo355_gemm_streamk_workspace_bytes() bytes (O355_EINVAL otherwise), 16-byte aligned,
 * zeroed once when allocated and never cleaned afterwards.  Its first 4096 bytes are int32 words: one hand-over flag
 * per workgroup, which holds the `epoch` of the launch whose partial the slot carries, and at index
 * O355_STREAMK_STATUS_WORD a status word.  `epoch`: any non-zero value that differs from the epoch of every earlier
 * launch on this workspace whose flags may still be set (a counter that skips 0 will do; O355_EINVAL for 0).  A stale
 * flag of an earlier launch therefore never passes for a partial of this one, whatever state that launch ended in
 * (for the same reason these launches must not be recorded into a HIP graph: a replay would repeat its epoch).
 * Launches that share a workspace must be ordered on one stream.  A finishing workgroup that does not see a partial
 * announced within about two seconds writes NaN into its tile instead of waiting on and stores the launch's epoch
 * into the status word: a caller that reads a non-zero status word knows that the output of that launch is not
 * valid; the next launch (with a new epoch) needs no clean-up of the workspace.
 * Needs K % 256 == 0, N % 16 == 0 (SwiGLU form: N % 256 == 0) and at least one unit of 256 per CU; otherwise
 * O355_EUNSUPPORTED.  olmo355_gemm_streamk_plan: 1 when this form is expected to beat the tiled launch. */
#define O355_STREAMK_STATUS_WORD 513
int64_t olmo355_gemm_streamk_workspace_bytes(void);
int olmo355_gemm_streamk_plan(int M, int N, int K);
int olmo355_w4_gemm_streamk(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y,
                            int M, int N, int K, void* workspace, int64_t ws_bytes, int epoch, void* stream);
int olmo355_w4_gemm_swiglu_streamk(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt,
                                   uint16_t* y, int M, int N, int K, void* workspace, int64_t ws_bytes, int epoch,
                                   void* stream);
int olmo355_b16_gemm_streamk(const uint16_t* x, const uint16_t* wt, uint16_t* y, int M, int N, int K, void* workspace,
                             int64_t ws_bytes, int epoch, void* stream);

/* The product for fp16 activations, the arithmetic of the reference's own QuantLinear (qlinear_cuda_old.py:253-265,
 * 287-290: weights fp16(scale * (q - zero)), fp16 activations, here with fp32 accumulation; its known-answer vectors,
 * AGQ tests/test_q4.py:1071-1104, are met to 2 fp16 ulp).  x [M,K] and y [M,N] are fp16.  olmo355_w4_gemv_f16: up to 16
 * rows whose K fits LDS (the decode kernel on the fp16 matrix instruction, nibbles as 1024 + q, scale and zero applied
 * in fp32); olmo355_w4_gemm_f16: any M (tiled launches).  O355_EUNSUPPORTED: use the other. */
int olmo355_w4_gemv_f16(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y, int M,
                        int N, int K, void* stream);
int olmo355_w4_gemm_f16(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y, int M,
                        int N, int K, void* stream);

/* The same product for an ff_proj weight ([up | gate] column halves) with SwiGLU (olmo/model.py:365-368,813-819)
 * in the epilogue: y [M, N/2] = silu(gate) * up, each factor rounded to bf16 first as the separate Linear and
 * activation would.  N a multiple of 256; O355_EUNSUPPORTED otherwise: olmo355_w4_gemm + olmo355_swiglu. */
int olmo355_w4_gemm_swiglu(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y,
                           int M, int N, int K, void* stream);

/* ---- dense Linear (nn.Linear without bias: olmo/model.py:452-462,695-701,1129-1139) -------
 * bf16: weight pre-tiled by olmo355_b16_repack into [N/16][K/32][64 lanes][8 bf16]
 * (lane l: row n = 16*nt + (l&15), columns 32*ks + 8*(l>>4) .. +7); K % 32 == 0, N % 16 == 0.
 * fp32: weight in torch layout [N,K]. */
int olmo355_b16_repack(const uint16_t* w_nk, uint16_t* wt, int N, int K, void* stream);
/* small-M (<= 64) path */
int olmo355_b16_gemv(const uint16_t* x, const uint16_t* wt, uint16_t* y, int M, int N, int K, void* stream);
int olmo355_b16_gemv_fused(const uint16_t* x, const uint16_t* resid, const uint16_t* norm_w, float eps,
                           uint16_t* x_out, const uint16_t* wt, uint16_t* y, int M, int N, int K, int swiglu,
                           void* stream);
int olmo355_b16_gemm(const uint16_t* x, const uint16_t* wt, uint16_t* y, int M, int N, int K, void* stream);
/* fp16 activations and fp16 weights (tiled by olmo355_b16_repack, which moves 16-bit elements of
 * either type), fp32 accumulate, fp16 out: the same nn.Linear under `model.half()`.  Any M. */
int olmo355_f16_gemm(const uint16_t* x, const uint16_t* wt, uint16_t* y, int M, int N, int K, void* stream);
int olmo355_f32_linear(const float* x, const float* w_nk, float* y, int M, int N, int K, void* stream);

/* ---- norms ------------------------------------------------------------------------------ */
/* RMSLayerNorm.forward (olmo/model.py:241-255): y = w * round(x * rsqrt(mean(x^2)+eps)),
 * both roundings to `dtype`; if `residual` != NULL, out = residual + y (the post-norm
 * residual add of olmo/model.py:786-794,814-821).  weight may be NULL.  rows x d. */
int olmo355_rmsnorm(const void* x, const void* weight, const void* residual, void* out, int rows, int d, float eps,
                    int dtype, void* stream);
/* The last block's post-norm update and the final norm of a decode step in one launch
 * (olmo/model.py:814-821 followed by olmo/model.py:1421-1423): x1 = residual + rmsnorm(x; w1),
 * out = rmsnorm(x1; w2), with every rounding of the two olmo355_rmsnorm calls it replaces (bit-identical to them).
 * O355_EUNSUPPORTED when d is not a multiple of 8 (4 for fp32) or above 8192 (4096): issue the two calls then. */
int olmo355_rmsnorm_pair(const void* x, const void* w1, const void* residual, const void* w2, void* out, int rows, int d,
                         float eps, int dtype, void* stream);
/* Non-parametric LayerNorm.forward (olmo/model.py:212-225): F.layer_norm without weight/bias. */
int olmo355_layernorm_np(const void* x, void* out, int rows, int d, float eps, int dtype, void* stream);

/* ---- attention input: QK-norm + rotary + cache write --------------------------------------
 * Per token row of the fused projection qkv [B*T, (H + 2*Hkv)*hd] (olmo/model.py:754-759):
 *   optional RMS norm of q over all H*hd channels and of k over all Hkv*hd channels with
 *   weights qw / kw (olmo/model.py:603-605; pass NULL for no QK-norm);
 *   rotary embedding in fp32 at absolute position past_len + t (olmo/model.py:298-324), with
 *   the caller's fp32 sin / cos tables [n_pos, hd] (olmo/model.py:285-296);
 *   q -> q_out [B*T, H*hd]; k (rotated) and v -> the contiguous per-layer cache
 *   kcache / vcache [B, Hkv, Lmax, hd] at row past_len + t.
 * Caching the rotated key equals the reference's re-rotation of the whole cache at every
 * step (olmo/model.py:615-625) because the rotation depends on (k, position) only.
 * past_len_dev (device int32, may be NULL) overrides past_len when given, so that one
 * captured launch can be replayed at successive positions. */
int olmo355_qknorm_rope_kvwrite(const void* qkv, const void* qw, const void* kw, const float* sin_tab,
                                const float* cos_tab, void* q_out, void* kcache, void* vcache, int B, int T, int H,
                                int Hkv, int hd, int Lmax, int n_pos, int past_len, const int32_t* past_len_dev,
                                float eps, int dtype, void* stream);

/* ---- attention (olmo/model.py:533-586,627-648): softmax(q k^T / sqrt(hd) + bias) v ---------
 * q [B*T, H*hd]; caches [B, Hkv, Lmax, hd] already holding rows 0 .. past_len+T-1;
 * out [B*T, H*hd].  Query t sits at absolute position past_len + t and sees keys 0..past_len+t.
 * key_bias (may be NULL): fp32 [B, bias_stride] added to the scores of key j (the padding part
 * of olmo/model.py:1337-1376); entries <= -1e30 mark the key as masked: its score is replaced
 * by the dtype's most negative finite value (olmo/torch_util.py:81-90), never -inf. */
int olmo355_attn_prefill(const void* q, const void* kcache, const void* vcache, const float* key_bias, void* out,
                         int B, int T, int H, int Hkv, int hd, int Lmax, int past_len, int bias_stride, int dtype,
                         void* stream);
/* The same with a workspace.  A launch of a single round of workgroups -- one prompt from scratch -- lasts as long as
 * its longest query block (causal work grows with the block's position); with a workspace the blocks whose keys run
 * past 1024 (1536 when the plain launch would fill the chip) are shared between workgroups along the keys, and
 * the one that finishes a block last combines all partial results and writes the rows (no workgroup waits for
 * another; same products, the partial sums of a row combined in the order of their keys whoever comes last).
 * olmo355_attn_prefill_workspace_bytes: the bytes that form needs for this call, 0 where the plain launch is the one
 * to use (ws may then be NULL).  ws: zeroed when allocated (its first 4096 bytes are int32 counters, one per (batch,
 * head, query block), which every launch leaves at zero again, so one workspace may serve calls of different shapes); O355_EINVAL when ws_bytes is smaller than needed. */
int64_t olmo355_attn_prefill_workspace_bytes(int B, int T, int H, int hd, int past_len, int dtype);
int olmo355_attn_prefill_ws(const void* q, const void* kcache, const void* vcache, const float* key_bias, void* out,
                            void* ws, int64_t ws_bytes, int B, int T, int H, int Hkv, int hd, int Lmax, int past_len,
                            int bias_stride, int dtype, void* stream);

/* T == 1 with the keys split over workgroups.  n_keys_max bounds the number of keys for the
 * launch grid; the true count is past_len + 1 (or *past_len_dev + 1 when given).
 * ws: ws_bytes >= olmo355_attn_decode_workspace_bytes(B,H,hd,n_keys_max) bytes (O355_EINVAL, nothing launched,
 * when smaller: the launch writes one partial per 128 keys of every (batch, head)), zeroed when allocated: it begins with
 * two int32 counters per (batch, head) that olmo355_attn_decode_fused uses to let one workgroup of a head
 * merge the partial results (B * H ticket counters, which every launch leaves at zero, then B * H launch counters
 * whose value marks the partials of the current launch; the regions are apart, so one workspace may serve
 * launches that merge either way, for the same B and H); the partials follow, (hd + 2) numbers per 128 keys with
 * room for a flag word each. */
int64_t olmo355_attn_decode_workspace_bytes(int B, int H, int hd, int n_keys_max);
int olmo355_attn_decode(const void* q, const void* kcache, const void* vcache, const float* key_bias, void* out,
                        void* ws, int64_t ws_bytes, int B, int H, int Hkv, int hd, int Lmax, int past_len,
                        const int32_t* past_len_dev, int n_keys_max, int bias_stride, int dtype, void* stream);

/* olmo355_attn_decode for callers that cannot allocate device memory or pass a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same
 * arguments without `ws`: the per-chunk partial results live in a device array of the library itself,
 * olmo355_attn_decode_static_max_bytes() = 16 MiB per GPU, held from the first call on that GPU until the
 * process ends.  Returns O355_ETOOBIG (nothing launched) when
 * olmo355_attn_decode_workspace_bytes(B, H, hd, n_keys_max) exceeds that.  Calls no hipMalloc / hipFree / allocating
 * library routine.  All calls on one GPU share the array and it keeps the last call's contents: calls that
 * overlap on one GPU (different streams or host threads) race; calls on one stream are ordered.
 * The first call on a GPU looks the array's device address up (hipGetSymbolAddress, a query that is not
 * permitted while a stream of the process is capturing): make one call on every GPU, e.g. a warm-up step, before
 * the first capture; later calls only launch kernels. */
int64_t olmo355_attn_decode_static_max_bytes(void);
int olmo355_attn_decode_static(const void* q, const void* kcache, const void* vcache, const float* key_bias, void* out,
                               int B, int H, int Hkv, int hd, int Lmax, int past_len, const int32_t* past_len_dev,
                               int n_keys_max, int bias_stride, int dtype, void* stream);

/* olmo355_attn_decode for beam search: the B rows are beam b % beam of sequence b / beam.  Where the
 * reference keeps the beams' caches consistent by gathering every cache tensor along the batch axis after each
 * step (olmo/beam_search.py:1062-1078, called at :1000), here no cache row moves: the keys and values of
 * positions < prompt_len are read from row (b / beam) * beam (the prefill of the sequence), and those of
 * position prompt_len + i from row beam_src[b * src_stride + i] (int32, the row whose beam wrote the i-th
 * generated token of b's history; entries past the current length must still be valid row numbers).  The
 * search updates beam_src with its backpointers.  Needs prompt_len + src_stride >= n_keys_max. */
int olmo355_attn_decode_beam(const void* q, const void* kcache, const void* vcache, const float* key_bias, void* out,
                             void* ws, int64_t ws_bytes, int B, int H, int Hkv, int hd, int Lmax, int past_len,
                             const int32_t* past_len_dev, int n_keys_max, int bias_stride, const int32_t* beam_src,
                             int src_stride, int prompt_len, int beam, int dtype, void* stream);

/* olmo355_qknorm_rope_kvwrite (T == 1) and olmo355_attn_decode in one pass over the new token's
 * fused projection qkv [B, (H+2*Hkv)*hd]: bf16, hd 64 or 128; O355_EUNSUPPORTED otherwise (the caller
 * then issues the two separate calls).  Same workspace as olmo355_attn_decode.
 * qk_ssq: NULL, or the per-tile sums of squares [B][(H+2*Hkv)*hd/16] that olmo355_w4_gemv_chain left for
 * qkv (the q and k norms then do not re-read the rows).
 * rope_now: NULL, or the rotary rows of the current position, float [2*hd] = sin row | cos row, as kept
 * by olmo355_rope_advance: with the position in device memory (past_len_dev) the table lookup would be a
 * dependent load behind the whole cache stream. */
int olmo355_attn_decode_fused(const void* qkv, const void* qw, const void* kw, const float* sin_tab,
                              const float* cos_tab, void* kcache, void* vcache, const float* key_bias, void* out,
                              void* ws, int64_t ws_bytes, int B, int H, int Hkv, int hd, int Lmax, int n_pos,
                              int past_len, const int32_t* past_len_dev, int n_keys_max, int bias_stride, float eps,
                              const float* qk_ssq, const float* rope_now, int dtype, void* stream);
/* Between captured decode steps: *pos += delta, then rope_now [2*hd] = sin_tab[*pos] | cos_tab[*pos]
 * (rows of get_rotary_embedding's tables, olmo/model.py:285-296).  delta 0 initialises rope_now. */
int olmo355_rope_advance(int32_t* pos, int delta, const float* sin_tab, const float* cos_tab, float* rope_now, int hd,
                         int n_pos, void* stream);

/* ---- MLP activation: SwiGLU.forward (olmo/model.py:365-368) --------------------------------
 * x [rows, 2h]: first half "up", second half "gate"; out [rows, h] = silu(gate) * up. */
int olmo355_swiglu(const void* x, void* out, int rows, int h, int dtype, void* stream);

/* ---- small helpers on the path ---------------------------------------------------------- */
/* wte lookup (olmo/model.py:1318): out[r,:] = table[ids[r],:]; ids int64. */
int olmo355_embedding(const int64_t* ids, const void* table, void* out, int rows, int d, int vocab, int dtype,
                      void* stream);
/* Act-order (desc_act) int4 weights: the rows of W are sorted by group once at load and the activation
 * columns follow at run time, out[m][k] = x[m][perm[k]], 16-bit elements, K even, M <= 65535 -- the column
 * remap of the reference's exllama back-end (AGQ/autogptq_extension/exllama/cuda_func/column_remap.cu:9-63,
 * q4_matrix.cu:105-169); perm int32 [K], a permutation of 0..K-1 (not checked). */
int olmo355_gather_columns(const uint16_t* x, const int32_t* perm, uint16_t* out, int M, int K, void* stream);
/* clip_qkv (olmo/model.py:756-757): x := clamp(x, -c, c) in place over n elements, c > 0. */
int olmo355_clamp(void* x, int64_t n, float c, int dtype, void* stream);
/* out = a + b (residual add of the pre-norm block, olmo/model.py:794,821). */
int olmo355_add(const void* a, const void* b, void* out, int64_t n, int dtype, void* stream);
/* out[m][n] = x[m][n] + bias[n]: the bias of a quantised Linear
 * (AGQ/auto_gptq/nn_modules/qlinear/qlinear_cuda_old.py:288-290); x, out bf16 [M, N], bias fp16 [N] as the
 * checkpoint stores it, sum in fp32, one rounding. */
int olmo355_add_bias_bf16(const uint16_t* x, const uint16_t* bias_f16, uint16_t* out, int M, int N, void* stream);
int olmo355_add_bias_f16(const uint16_t* x, const uint16_t* bias_f16, uint16_t* out, int M, int N, void* stream); /* fp16 rows */
/* Greedy step (olmo/beam_search.py:102-113 with beam 1): first index of the row maximum,
 * written as int64 to out[r], and the same value appended at ids_next when non-NULL. */
int olmo355_argmax(const void* logits, int64_t* out, int rows, int n, int dtype, void* stream);
/* The end of a greedy decode step in one launch: olmo355_argmax per row into ids_out, the chosen token's row of the
 * embedding table (olmo/model.py:1318) into x_next [rows, d] as the next step's input, and olmo355_rope_advance(pos, 1,
 * ...) for the step that follows.  Ids at or past `vocab` (rows of the table) read its last row, as
 * olmo355_embedding does. */
int olmo355_greedy_next(const void* logits, int64_t* ids_out, const void* table, void* x_next, int rows, int n, int d,
                        int vocab, int32_t* pos, const float* sin_tab, const float* cos_tab, float* rope_now, int hd,
                        int n_pos, int dtype, void* stream);
/* The two selections of a beam-search step (olmo/beam_search.py:813-1045 with the DeterministicSampler,
 * :102-113), one workgroup per row.
 * olmo355_log_softmax: F.log_softmax of the step function (olmo/model.py:1705) over rows of n logits in the
 *   activation dtype; fp32 log-probabilities out [rows, n].
 * olmo355_topk: torch.topk(x, k, dim=-1) of fp32 rows: out_vals / out_idx [rows, k], descending; equal values
 *   in ascending index order (torch leaves that order open).  k <= n, k <= 1024; NaNs are not supported. */
int olmo355_log_softmax(const void* logits, float* out, int rows, int n, int dtype, void* stream);
int olmo355_topk(const float* x, int rows, int n, int k, float* out_vals, int64_t* out_idx, void* stream);
/* Sampling inside a beam search (torch.multinomial of the MultinomialSampler / TopKSampler / TopPSampler,
 * olmo/beam_search.py:135-146, 171-203, 238-289): out = x * inv_temp + Gumbel(0, 1) noise from
 * (seed, counter, element), entries <= -1.7e38 -> -inf.  olmo355_topk(out, k) is then k draws without replacement
 * from softmax(x * inv_temp); the reference's random stream is not reproduced. */
int olmo355_gumbel_perturb(const float* x, float* out, int rows, int n, float inv_temp, uint64_t seed,
                           uint64_t counter, void* stream);
/* GumbelSampler.gumbel_with_max (olmo/beam_search.py:395-421): per row, Gumbel(phi) samples conditioned on their
 * maximum being row_max[row]; fp32 [rows, n] in and out, noise from (seed, counter, element). */
int olmo355_gumbel_with_max(const float* phi, const float* row_max, float* out, int rows, int n, uint64_t seed,
                            uint64_t counter, void* stream);

/* One sampled step (olmo/beam_search.py:117-277 with beam size 1): z = logits / temperature; top_k > 0 keeps the
 * k largest, then top_p < 1 keeps the most probable tokens up to and including the one at which the cumulative
 * probability reaches top_p (of what top-k kept); the draw is from what remains, renormalised.  top_k = 0 and
 * top_p = 1 is MultinomialSampler.  out[r] = token (int64), logprob[r] = log_softmax(logits)[token] at
 * temperature 1, as the reference's samplers return.  The uniform number comes from (seed, counter, row), with the
 * counter read from *counter_dev when that is non-NULL (e.g. the device-side position, so that a captured step
 * draws a fresh number on every replay).  Tokens tied with a filter's threshold are all kept.  The reference's
 * random stream (torch.multinomial) is not reproduced.  temperature > 0, 0 <= top_p <= 1. */
int olmo355_sample(const void* logits, int rows, int n, float temperature, int top_k, float top_p, uint64_t seed,
                   const int32_t* counter_dev, int counter, int64_t* out, float* logprob, int dtype, void* stream);
/* *p += 1 for a device int32 (advances the position between captured decode steps). */
int olmo355_incr_i32(int32_t* p, void* stream);



#ifdef __cplusplus
}
#endif
#endif /* OLMO355_H */

/* Entry points of libolmo355.so beside the drop-in interface of include/olmo355.h; none has a counterpart in the
 * reference.  Variants: a declared entry point with one more argument that names the kernel variant the dispatcher would
 * otherwise choose by shape, so that tests and tuning runs can reach every variant on any shape.  The decode relay: an
 * opt-in form of the one-row decode step on two streams (measured, not the default).  Measuring probes.  Like the
 * rest of the library they keep no state. */
#ifndef OLMO355_DEBUG_H
#define OLMO355_DEBUG_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* olmo355_w4_gemm / olmo355_b16_gemm with the tile shape given: 0 = choose; 256 / 192 / 128 = 256 rows by that
 * many columns; 128128 / 128064 = 128-row tiles. */
int olmo355_w4_gemm_tile(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y,
                         int M, int N, int K, int tile, void* stream);
int olmo355_b16_gemm_tile(const uint16_t* x, const uint16_t* wt, uint16_t* y, int M, int N, int K, int tile,
                          void* stream);

/* olmo355_w4_gemm_streamk with the finishing workgroups' patience (polls of a hand-over flag before the tile is
 * given up as NaN) and with publish = 0, which makes the partials' owners leave their flags down: the give-up path
 * forced from the host, every workgroup still exits. */
int olmo355_w4_gemm_streamk_patience(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y,
                                  int M, int N, int K, void* workspace, int64_t ws_bytes, int epoch, int spin_limit,
                                  int publish, void* stream);

/* olmo355_w4_gemv with the kernel family given: 0 = choose; 1 = the kernels that keep all rows of x in LDS per
 * workgroup (the lean M <= 16 kernel where it applies), never the staged-activation kernel; 2 = the
 * staged-activation kernel (w4_mid_kernel), 3 / 4 = the same with one / two column-tile pairs per workgroup;
 * 5 = the older kernels only (w4_gemv_rot_kernel / w4_gemv_kernel). */
int olmo355_w4_gemv_form(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y,
                         int M, int N, int K, int form, void* stream);

/* olmo355_w4_gemv_chain through the kernel for 5 to 8 rows (any M <= 8 is accepted here) with the column tiles per
 * workgroup (nt: 1, 2 or 3; with swiglu 2 or 4; 0 = choose) and the waves per workgroup (8, 16; 0 = choose) given. */
int olmo355_w4_gemv_r8_form(const uint16_t* x, const uint16_t* resid, const uint16_t* norm_w, float eps, uint16_t* x_out,
                            const float* ssq_in, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y,
                            float* ssq_out, int M, int N, int K, int swiglu, int nt, int waves, void* stream);

/* olmo355_attn_decode_fused with the merge of a head's key chunks given: -1 = choose, 0 = in the kernel (the last
 * workgroup of a (batch, head) to finish, found by a ticket drawn after its stores have landed), 1 = in the kernel by
 * the workgroup of the head's last chunk, which polls flag words stored together with the numbers (the writers
 * wait for nothing), 2 = the separate combine kernel. */
int olmo355_attn_decode_fused_merge(const void* qkv, const void* qw, const void* kw, const float* sin_tab,
                                    const float* cos_tab, void* kcache, void* vcache, const float* key_bias, void* out,
                                    void* ws, int64_t ws_bytes, int B, int H, int Hkv, int hd, int Lmax, int n_pos,
                                    int past_len, const int32_t* past_len_dev, int n_keys_max, int bias_stride, float eps,
                                    const float* qk_ssq, const float* rope_now, int dtype, int merge, void* stream);

#include "olmo355.h"

/* ---- the batch-1 decode step as a relay on two streams ---------------------------------------------------------
 * The launches of a decode step -- att_proj, attention, attn_out, ff_proj, ff_out of every block, i.e. the calls
 * OLMoSequentialBlock.forward makes one after the other (olmo/model.py:746-823), each linear a QuantLinear.forward
 * (AGQ/auto_gptq/nn_modules/qlinear/qlinear_cuda_old.py:192-290) -- form a chain in which every launch needs the whole
 * output of the one before but none of its weights depend on it.  In the relay form launch n+1 may run on a second
 * stream while launch n is still at work: it requests all of its weights (cache rows) first and then waits for its
 * input rows, which carry the hand-over themselves:
 *   tagged row   uint32 per element: bf16 bits << 16 | (epoch & 0xffff)
 *   tagged sums  uint32 per 16-column tile: the tile's sum of squares as a float rounded to 20 mantissa bits,
 *                the low 4 bits = epoch & 0xf
 * `epoch` is a device word that the caller changes before every step (olmo355_incr_i32); every tagged buffer is
 * written exactly once per step, by one launch, and must not be reused for anything else while the step runs.  A
 * consumer polls its inputs with device-coherent loads until every tag equals the epoch, at most `spin_limit` times;
 * then it sets status[0] = 1, uses what it has and ends (results undefined, nothing hangs; `status` is 8 words:
 * with status[4] set by the host, the int4 linears also leave the longest waits of a run in status[1..3]).  On one stream the same
 * calls simply never wait.  hint_out / hint_in (optional, O355_RELAY_HINT_COPIES words O355_RELAY_HINT_STRIDE bytes apart per launch,
 * handed from a launch to its consumer): the producer's last workgroup stores the epoch there when it is done, and a consumer that found its rows
 * unfinished watches that one word before it asks for the rows again -- polling whole rows from every workgroup
 * would cost more traffic than the weights.  A hint only: the tags decide.
 *
 * Two launches of the relay that are in flight together (consecutive ones on the two streams) must fit the chip side
 * by side: olmo355_relay_pair_ok(older, younger, n_cu, lds_per_cu) says whether the younger one, all of its
 * workgroups waiting, can never keep a workgroup of the older one from starting; footprints (workgroups, waves per
 * workgroup, vector registers per lane, LDS bytes per workgroup) come from the *_footprint calls.  Use the second
 * stream only when every consecutive pair passes; never more than two streams.
 *
 * olmo355_w4_relay: y = x' . W at ONE row.  x: tagged row (x_tagged) or bf16 [K].  resid != NULL: x' = resid +
 * rmsnorm(x; norm_w, eps) with the mean square from ssq_in (tagged sums [K/16]), x' also written to x_out (tagged; resid
 * and x_out tagged rows; needs x_tagged, K <= 8192); else x' = x and ssq_in, norm_w, x_out are NULL.  y: tagged (y_tagged)
 * or bf16, [N], or [N/2] = silu(gate) * up with swiglu (olmo/model.py:365-368; needs resid); ssq_out: NULL or tagged sums
 * [N/16] (not with swiglu).  cfg: 0 = choose the launch shape, else waves per workgroup (4, 8, 16) | column tiles
 * per workgroup (1, 2) << 8.  O355_EUNSUPPORTED when a wave's share of K exceeds its registers (K / 128 / waves > 12). */
#define O355_RELAY_HINT_COPIES 64
#define O355_RELAY_HINT_STRIDE 1024 /* bytes between the copies: a hint buffer is 64 KiB */
int olmo355_w4_relay(const void* x, int x_tagged, const uint32_t* ssq_in, const uint32_t* resid, const uint16_t* norm_w,
                     float eps, uint32_t* x_out, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, void* y,
                     int y_tagged, uint32_t* ssq_out, int N, int K, int swiglu, const int32_t* epoch, int32_t* status,
                     const int32_t* hint_in, int32_t* hint_out, int spin_limit, int cfg, void* stream);
int olmo355_w4_relay_footprint(int N, int K, int norm, int x_tagged, int swiglu, int cfg, int* out4);
int olmo355_relay_pair_ok(const int* older4, const int* younger4, int n_cu, int lds_per_cu);
int olmo355_relay_device(int* out2); /* CUs of the current device, bytes of LDS per CU */
/* olmo355_attn_decode_fused as a leg of the relay: qkv tagged [B, (H + 2 Hkv) hd], qk_ssq tagged sums (required with
 * QK-norm), out tagged [B, H hd]; the cache rows are requested before the wait.  Only launches whose chunks are
 * merged inside the kernel (B * H * chunks <= 1536), H hd <= 8192. */
int olmo355_attn_decode_relay(const uint32_t* qkv, const void* qw, const void* kw, const float* sin_tab,
                              const float* cos_tab, void* kcache, void* vcache, const float* key_bias, uint32_t* out,
                              void* ws, int64_t ws_bytes, int B, int H, int Hkv, int hd, int Lmax, int n_pos,
                              int past_len, const int32_t* past_len_dev, int n_keys_max, int bias_stride, float eps,
                              const uint32_t* qk_ssq, const float* rope_now, const int32_t* epoch, int32_t* status,
                              const int32_t* hint_in, int32_t* hint_out, int spin_limit, void* stream);
int olmo355_attn_decode_relay_footprint(int B, int H, int hd, int n_keys_max, int* out4);
/* out (bf16 [K]) = resid + rmsnorm(x; norm_w, eps) from tagged rows and tagged sums: the last block's pending update
 * (olmo/model.py:814-821) handed to the launches after the relay.  olmo355_relay_tag: bf16 -> tagged row (the
 * step's first residual row, the token's embedding). */
int olmo355_relay_final(const uint32_t* x, const uint32_t* ssq_in, const uint32_t* resid, const uint16_t* norm_w, float eps,
                        uint16_t* out, int K, const int32_t* epoch, int32_t* status, int spin_limit, void* stream);
int olmo355_relay_tag(const uint16_t* x, uint32_t* out, int n, const int32_t* epoch, void* stream);


/* ---- measuring probes (no counterpart in the reference; used by bench.py only) -------------------
 * What a kernel that only streams `bytes` from HBM takes (16-byte non-temporal loads per lane, launch shaped
 * like the small-M linears; nothing is written), and what the matrix cores sustain on random bf16 operands
 * (256 workgroups x 8 waves x iters x 16 v_mfma_f32_16x16x32_bf16, the prefill GEMM's instruction; *flops = total
 * floating-point operations).
 * `sink` is a device buffer of at least 2 KiB that stays unwritten. */
int olmo355_probe_stream_read(const void* src, int64_t bytes, void* sink, void* stream);
/* The same over n buffers (host arrays of device pointers and byte counts, n <= 160) in ONE launch of a persistent
 * grid of two workgroups per CU: no launch boundary and no ramp per buffer. */
int olmo355_probe_stream_read_many(const void* const* srcs, const int64_t* bytes, int n, void* sink, void* stream);
int olmo355_probe_mfma_bf16(int iters, void* sink, double* flops, void* stream);
/* For tests: leaves `pattern` in every 32-bit word of the LDS of every CU (LDS keeps what the last workgroup left
 * there, so a kernel that reads LDS it has not written gives results that depend on what ran before it; with a NaN
 * pattern in place such a read shows in the output). */
int olmo355_probe_fill_lds(uint32_t pattern, void* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* OLMO355_DEBUG_H */

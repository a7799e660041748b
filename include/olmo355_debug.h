/* Variant entry points of libolmo355.so: each is one of the declared entry points of include/olmo355.h with one
 * more argument that names the kernel variant the dispatcher would otherwise choose by shape, so that tests and
 * tuning runs can reach every variant on any shape.  Like the rest of the library they keep no state: the choice
 * is an argument of the call.  Not part of the drop-in interface; no counterpart in the reference. */
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
                                  int M, int N, int K, void* workspace, int spin_limit, int publish, void* stream);

/* olmo355_w4_gemv with the kernel family given: 0 = choose; 1 = the kernels that keep all rows of x in LDS per
 * workgroup (the lean M <= 16 kernel where it applies), never the staged-activation kernel; 2 = the
 * staged-activation kernel (w4_mid_kernel), 3 / 4 = the same with one / two column-tile pairs per workgroup;
 * 5 = the older kernels only (w4_gemv_rot_kernel / w4_gemv_kernel). */
int olmo355_w4_gemv_form(const uint16_t* x, const uint32_t* wt, const uint16_t* st, const uint8_t* zt, uint16_t* y,
                         int M, int N, int K, int form, void* stream);

/* olmo355_attn_decode_fused with the merge of a head's key chunks given: -1 = choose, 0 = in the kernel (the last
 * workgroup of a (batch, head) to finish, found by a ticket drawn after its stores have landed), 1 = in the kernel by
 * the workgroup of the head's last chunk, which polls flag words stored together with the numbers (the writers
 * wait for nothing), 2 = the separate combine kernel. */
int olmo355_attn_decode_fused_merge(const void* qkv, const void* qw, const void* kw, const float* sin_tab,
                                    const float* cos_tab, void* kcache, void* vcache, const float* key_bias, void* out,
                                    void* ws, int B, int H, int Hkv, int hd, int Lmax, int n_pos, int past_len,
                                    const int32_t* past_len_dev, int n_keys_max, int bias_stride, float eps,
                                    const float* qk_ssq, const float* rope_now, int dtype, int merge, void* stream);

/* olmo355_w4_chain that also records when each wave passed the stations of each phase: trace is
 * int64 [grid][8 waves][4 phases][8 stations], ticks of the 100 MHz constant clock (phase entered, activations staged,
 * staging barrier passed, first weights landed, items done, rows published, all workgroups arrived, phase left). */
#include "olmo355.h"
int olmo355_w4_chain_trace(const olmo355_chain_phase* phases, int n_phases, int M, int32_t* sync, int32_t* status,
                           int spin_limit, int64_t* trace, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* OLMO355_DEBUG_H */

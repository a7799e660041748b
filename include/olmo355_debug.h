/* Test hooks of libolmo355.so: force one of the kernel variants the dispatchers choose between, so that tests
 * and tuning runs can reach every variant on any shape.  They set process-wide state, are not thread-safe and are
 * not part of the drop-in interface (include/olmo355.h has no state); 0 / -1 restores the dispatcher's choice.
 * No counterpart in the reference. */
#ifndef OLMO355_DEBUG_H
#define OLMO355_DEBUG_H
#ifdef __cplusplus
extern "C" {
#endif

/* GEMM tile: 0 = choose; 256 / 192 / 128 = 256 rows by that many columns; 128128 / 128064 = 128-row tiles. */
void olmo355_debug_set_gemm_tile(int shape);
/* Older small-M int4 kernel (w4_gemv_kernel / w4_gemv_rot_kernel): waves per workgroup (-1 = choose) and
 * whether the activations are staged in LDS (-1 = choose). */
void olmo355_debug_set_gemv_plan(int waves, int xlds);
/* 1 = the dispatcher's choice (default); 0 = never the lean / staged-activation kernels; 2 = the
 * staged-activation kernel (w4_mid_kernel) for every plain call. */
void olmo355_debug_set_gemv_small(int mode);
/* w4_mid_kernel: column-tile pairs per workgroup, 0 = choose, 1 or 2. */
void olmo355_debug_set_mid_pairs(int pairs);
/* Fused decode attention, how the key chunks of a head are merged: -1 = choose (default), 0 = always in the
 * kernel (last workgroup of a head, ticket), 1 = one workgroup per (batch, head) and no chunks, 2 = always the
 * separate combine kernel. */
void olmo355_debug_set_attn_mode(int mode);

#ifdef __cplusplus
}
#endif
#endif /* OLMO355_DEBUG_H */

/*
 * tagi_hip_test_hooks.h - kernel-selection switches of libtagi_hip.so for its own
 * parity tests and tuning sweeps. NOT part of the drop-in boundary (tagi_hip.h): a
 * binding of the reference never includes this file, and nothing a caller of the
 * reference does maps to it. It has no counterpart in the reference.
 */
#ifndef TAGI_HIP_TEST_HOOKS_H
#define TAGI_HIP_TEST_HOOKS_H

#ifdef __cplusplus
extern "C" {
#endif

/* Every knob is process-wide (set it only while no other thread is inside the
 * library). The parity tests use them to force each code path, the tuning sweeps
 * to compare them; value < 0 restores the built-in heuristic, unknown keys return
 * TAGI_ERR_INVALID_ARG. Linear: "linear.tile", "linear.fwd.splits",
 * "linear.dz.splits", "linear.dw.splits", "linear.gemv_max_batch" (largest batch of
 * the streaming kernels, at most 16), "linear.gemv.swizzle",
 * "linear.gemv.fwd_variant", "linear.gemv.reverse", "linear.gemv16" (0: 9..16
 * samples on the kernels for up to 8), "linear.gemv32" (0: the forward of 17..32
 * samples on the tiled kernel instead of the 16-wide streaming one; 2: their state
 * backward on the streaming kernel too), "linear.gemv16.whole_lines" (load
 * pattern of the 16-wide streaming forward: 1 whole 128-byte lines with streaming loads, 2
 * whole lines with plain loads, 3 whole lines with plain loads for mu_w and streaming
 * loads for var_w, 4 the other way round, 0 sixteen rows x 64 bytes per instruction;
 * < 0 by size), "linear.gemv16.fwd_waves" (8 or 16 waves per workgroup of that forward, < 0 by
 * size), "linear.gemv16.min_batch" (smallest batch that takes the 16-wide forward,
 * 1 by default; the 4x4x1 forward serves the batches below it), "linear.dw_side" (0: bias innovations and
 * the state-backward fold as launches of their own instead of inside the
 * weight-backward launch), "linear.double_buffer", "linear.stream_min_weights" (the
 * smallest weight matrix, in elements, that goes to the streaming kernels; 0 sends every
 * layer whose batch fits there, < 0 restores the measured thresholds; any value >= 0 also
 * keeps small layers off their one-launch forward kernel), "linear.small" (0: no
 * one-launch forward for small layers). Conv2d: "conv2d.tile",
 * "conv2d.splits", "conv2d.dw.tile", "conv2d.dw.splits", "conv2d.group_loads",
 * "conv2d.stencil", "conv2d.phase_order", "conv2d.s2_all" (0 switches the named path
 * off; s2_all: the stencil kernels of the stride-2 layers - forward, state backward with
 * all four phases in one workgroup and its pair-wise fold, weight backward - which leaves
 * those layers on the table-driven kernels; "conv2d.bwd_pair": 0 gives the state and the
 * weight backward of tagi_conv2d_bwd launches of their own). "batchnorm.fused_train": 0
 * gives tagi_batchnorm2d_fwd_train a launch of its own for the merge of the statistics. */
int tagi_hip_tune(const char *key /* host */, int value);

#ifdef __cplusplus
}
#endif
#endif /* TAGI_HIP_TEST_HOOKS_H */

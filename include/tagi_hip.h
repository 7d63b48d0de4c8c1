/*
 * tagi_hip.h - C ABI of the MI355X (gfx950) backend for the TAGI Linear and
 * Conv2d hot path.
 *
 * The reference (cuTAGI) has no C ABI: its GPU layers link C++ classes against
 * CUDA kernels directly. Each entry point below replaces one kernel-dispatch
 * function of that code and is what a binding of the reference would call in
 * its place; the reference interface is cited per function (paths relative to
 * the reference tree).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer to fp32 (or int32 for index tables)
 *     unless it is marked "host";
 *   - layouts are the reference's: weights [N][K] row-major (conv: OIHW),
 *     activations [B][K] (conv: NCHW), outputs [B][N];
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     calls only enqueue work and never synchronise, except where noted;
 *   - every function returns TAGI_OK (0) or a negative TAGI_ERR_* code, or a
 *     positive hipError_t when the HIP runtime failed; nothing throws;
 *     tagi_hip_error_string() describes any of them;
 *   - the library owns no user buffer. It keeps one grow-only device workspace
 *     per (GPU, stream) for split-reduction partial sums (see
 *     tagi_hip_workspace_reserve), so calls on different streams never share
 *     scratch memory; calls issued to ONE stream from several host threads must be
 *     serialised by the caller, as with any stream-ordered API.
 */
#ifndef TAGI_HIP_H
#define TAGI_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TAGI_OK 0
#define TAGI_ERR_INVALID_ARG (-1) /* null pointer, non-positive size, ... */
#define TAGI_ERR_UNSUPPORTED (-2) /* shape outside what the kernels cover */
#define TAGI_ERR_NO_DEVICE (-3)

/* ---- runtime ------------------------------------------------------------ */

/* ABI version of this header (major * 100 + minor). */
int tagi_hip_version(void);
/* replaces get_cuda_device_count (src/cuda_utils.cpp) as used by
 * Sequential::to_device (src/sequential.cpp:32-73). */
int tagi_hip_device_count(int *count /* host, out */);
const char *tagi_hip_error_string(int code);
/* Grow the workspace of `stream` on the current device to at least `bytes` now
 * (synchronises the device if it has to reallocate). Optional: entry points grow it
 * on demand. */
int tagi_hip_workspace_reserve(size_t bytes, void *stream);
/* Free the workspaces of all devices. */
int tagi_hip_shutdown(void);
/* Compute units, peak engine clock (MHz) and name of the current device, as the
 * runtime reports them (hipGetDeviceProperties); any pointer may be NULL. The
 * reference's counterpart is get_cuda_device_properties (src/cuda_utils.cpp). */
int tagi_hip_device_info(int *compute_units /* host */, int *clock_mhz /* host */,
                         char *name /* host */, size_t name_capacity);

/* ---- Linear -------------------------------------------------------------- */

/* mu_z = mu_a * mu_w^T + mu_b ; var_z = (var_a + mu_a^2) * var_w^T
 *                                        + var_a * (mu_w^2)^T + var_b
 * replaces linear_forward_cuda (src/linear_layer_cuda.cu:12-73) and the kernels
 * it dispatches (include/linear_cuda_kernel.cuh:50-573).
 * mu_b/var_b may be NULL when bias == 0. */
int tagi_linear_fwd(const float *mu_w, const float *var_w, const float *mu_b,
                    const float *var_b, const float *mu_a, const float *var_a,
                    int K, int N, int B, int bias, float *mu_z, float *var_z,
                    void *stream);

/* tagi_linear_fwd with the activation that follows the layer applied to its sums
 * before anything is stored: mu_out / var_out / jcb_out [B][N] receive what
 * relu_mean_var_cuda or mixture_relu_mean_var_cuda (src/activation_cuda.cu:130-150,
 * 726-760) would write from this layer's output; the pre-activation moments are never
 * written. Replaces the LinearCuda::forward + ReLUCuda / MixtureReLUCuda::forward
 * pair of a Sequential (src/sequential.cpp:323-331 runs them back to back). */
#define TAGI_ACT_RELU 1
#define TAGI_ACT_MIXTURE_RELU 2
int tagi_linear_fwd_act(const float *mu_w, const float *var_w, const float *mu_b,
                        const float *var_b, const float *mu_a, const float *var_a,
                        int K, int N, int B, int bias, int activation,
                        float *mu_out, float *var_out, float *jcb_out, void *stream);

/* tagi_linear_fwd for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc). It has no
 * counterpart in the reference. Same arguments, same kernels and bit-identical
 * results; the partial sums of a sliced reduction go to a fixed array of
 * TAGI_LINEAR_FWD_STATIC_SCRATCH_BYTES that every GPU holds from the moment the
 * library is loaded until the process ends, so the call never reaches hipMalloc,
 * hipFree or the grow-only workspace. A shape whose partial sums need more than
 * that returns TAGI_ERR_UNSUPPORTED and launches nothing (2 * slices * B * N * 4
 * bytes; 32 MiB at K = N = 4096, B = 256). All calls on one GPU share the array:
 * calls that overlap on one GPU (two streams, two host threads) race. The first
 * call on a device looks the array's address up once; make that call outside a
 * graph capture. The array is part of the library's device image: every process
 * that loads the library holds these 64 MiB on every GPU it touches, whether or
 * not it ever calls this entry point. */
#define TAGI_LINEAR_FWD_STATIC_SCRATCH_BYTES ((size_t)64 << 20)
int tagi_linear_fwd_static(const float *mu_w, const float *var_w,
                           const float *mu_b, const float *var_b,
                           const float *mu_a, const float *var_a, int K, int N,
                           int B, int bias, float *mu_z, float *var_z,
                           void *stream);

/* delta_mu_z = (delta_mu * mu_w) .* jcb ; delta_var_z = (delta_var * mu_w^2) .* jcb^2
 * replaces linear_state_backward_cuda (src/linear_layer_cuda.cu:75-121). */
int tagi_linear_bwd_dz(const float *mu_w, const float *jcb,
                       const float *delta_mu, const float *delta_var, int K,
                       int N, int B, float *delta_mu_z, float *delta_var_z,
                       void *stream);

/* delta_mu_w = (delta_mu^T * mu_a) .* var_w ; delta_var_w = (delta_var^T * mu_a^2) .* var_w^2
 * replaces linear_weight_backward_cuda (src/linear_layer_cuda.cu:123-168). */
int tagi_linear_bwd_dw(const float *var_w, const float *mu_a,
                       const float *delta_mu, const float *delta_var, int K,
                       int N, int B, float *delta_mu_w, float *delta_var_w,
                       void *stream);

/* delta_mu_b = colsum(delta_mu) .* var_b ; delta_var_b = colsum(delta_var) .* var_b^2
 * replaces the linear_bwd_delta_b launch of LinearCuda::backward
 * (src/linear_layer_cuda.cu:311-321, kernel include/linear_cuda_kernel.cuh:1492-1519). */
int tagi_linear_bwd_db(const float *var_b, const float *delta_mu,
                       const float *delta_var, int N, int B, float *delta_mu_b,
                       float *delta_var_b, void *stream);

/* The whole of LinearCuda::backward (src/linear_layer_cuda.cu:273-323) in one
 * call: the state update when state_update != 0, the weight update when
 * param_update != 0 and the bias update when additionally bias != 0. */
int tagi_linear_bwd(const float *mu_w, const float *var_w, const float *var_b,
                    const float *mu_a, const float *jcb, const float *delta_mu,
                    const float *delta_var, int K, int N, int B, int bias,
                    int state_update, int param_update, float *delta_mu_z,
                    float *delta_var_z, float *delta_mu_w, float *delta_var_w,
                    float *delta_mu_b, float *delta_var_b, void *stream);

/* ---- Conv2d -------------------------------------------------------------- */

/* Output size of a convolution; replaces compute_downsample_img_size_v2
 * (src/conv2d_layer.cpp:581-628). Host only. TAGI_ERR_INVALID_ARG where the
 * reference throws (stride does not divide). */
int tagi_conv2d_out_size(int kernel, int stride, int wi, int hi, int pad,
                         int pad_type, int *wo /* host */, int *ho /* host */);

/* Index tables of a convolution, on the host, int32 and 1-based exactly as
 * get_conv2d_idx builds them (src/conv2d_layer.cpp:656-719 over
 * src/indices.cpp): Fmwa_2 [wo*ho][k*k] (padding = -1), FCzwa_1 [w][h]
 * (padding = param_pad_idx) and Szz_ud [h][w] (padding = -1).
 * Capacity needed: Fmwa_2 wo*ho*k*k ints, the other two wi*hi*k*k ints each.
 * All pointers host. Square images only, like the reference. */
int tagi_conv2d_build_idx(int kernel, int stride, int wi, int hi, int pad,
                          int pad_type, int param_pad_idx, int *Fmwa_2,
                          int *FCzwa_1, int *Szz_ud, int *w, int *h);

/* Forward through the Fmwa_2 table (device copy `aidx`); replaces
 * conv2d_forward_cuda (src/conv2d_layer_cuda.cu:22-88).
 * mu_a/var_a [B][fi][wihi], weights [fo][fi*ki*ki], out [B][fo][woho]. */
int tagi_conv2d_fwd(const float *mu_w, const float *var_w, const float *mu_b,
                    const float *var_b, const float *mu_a, const float *var_a,
                    const int *aidx, int woho, int fo, int wihi, int fi,
                    int ki, int B, int bias, float *mu_z, float *var_z,
                    void *stream);

/* tagi_conv2d_fwd with the activation that follows the layer (TAGI_ACT_*) applied
 * before anything is stored, as tagi_linear_fwd_act: outputs [B][fo][woho]. */
int tagi_conv2d_fwd_act(const float *mu_w, const float *var_w, const float *mu_b,
                        const float *var_b, const float *mu_a, const float *var_a,
                        const int *aidx, int woho, int fo, int wihi, int fi,
                        int ki, int B, int bias, int activation, float *mu_out,
                        float *var_out, float *jcb_out, void *stream);

/* State backward through FCzwa_1 (`zw_idx`, [wihi][nr]) and Szz_ud (`zud_idx`,
 * [nr][wihi]); replaces conv2d_state_backward_cuda
 * (src/conv2d_layer_cuda.cu:90-147) including the Jacobian permutation
 * Conv2dCuda::backward runs before it (src/conv2d_layer_cuda.cu:501-509):
 * `jcb` is the un-permuted [B][fi][wihi] Jacobian. Requires every input pixel
 * to be covered (w == wihi), as the reference's kernels assume. */
int tagi_conv2d_bwd_dz(const float *mu_w, const float *jcb,
                       const float *delta_mu_out, const float *delta_var_out,
                       const int *zw_idx, const int *zud_idx, int woho, int fo,
                       int wihi, int fi, int ki, int nr, int B,
                       float *delta_mu, float *delta_var, void *stream);

/* tagi_conv2d_bwd_dz for the first layer of a ResNetBlock's main block, with the
 * block's residual innovations added in the same pass (res_* laid out like the
 * output, [B][fi][wihi]). res_mode 1, identity shortcut: (sum + res) .* jcb, which is
 * the layer's result plus add_shortcut_delta_cuda (src/resnet_block_cuda.cu:20-33) on
 * the block's incoming innovations; res_mode 2, shortcut branch: the layer's result
 * plus add_shortcut_mean_var_cuda (7-18) on the branch's finished innovations, as
 * ResNetBlockCuda::backward runs them (301-347). */
int tagi_conv2d_bwd_dz_res(const float *mu_w, const float *jcb,
                           const float *delta_mu_out, const float *delta_var_out,
                           const int *zw_idx, const int *zud_idx, int woho, int fo,
                           int wihi, int fi, int ki, int nr, int B,
                           const float *res_mu, const float *res_var, int res_mode,
                           float *delta_mu, float *delta_var, void *stream);

/* Weight (and, with bias != 0, bias) backward through Fmwa_2; replaces
 * conv2d_param_backward_cuda (src/conv2d_layer_cuda.cu:149-227) including its
 * delta permutation, and the bias reduction of Conv2dCuda::backward (478-498): delta_*_out are the un-permuted [B][fo][woho] deltas. */
int tagi_conv2d_bwd_dw(const float *var_w, const float *var_b,
                       const float *mu_a, const float *delta_mu_out,
                       const float *delta_var_out, const int *aidx, int B,
                       int fo, int woho, int wihi, int fi, int ki, int bias,
                       float *delta_mu_w, float *delta_var_w,
                       float *delta_mu_b, float *delta_var_b, void *stream);

/* All of Conv2dCuda::backward (src/conv2d_layer_cuda.cu:349-476) in one call: the state
 * innovations (state_update; with res_mu / res_var != NULL also the residual add of
 * tagi_conv2d_bwd_dz_res) and the weight / bias innovations (param_update; bias ones
 * only when bias != 0). Where both contractions run on their regular-stencil kernels
 * (3x3, stride 1, "same" padding, whole groups of 64 channels) they share ONE launch:
 * the two tile grids are independent, and as one grid neither kernel's ramp-up nor its
 * tail leaves the chip idle. Otherwise the same as tagi_conv2d_bwd_dw followed by
 * tagi_conv2d_bwd_dz(_res). Uses the workspace. */
int tagi_conv2d_bwd(const float *mu_w, const float *var_w, const float *var_b,
                    const float *mu_a, const float *jcb,
                    const float *delta_mu_out, const float *delta_var_out,
                    const int *aidx, const int *zw_idx, const int *zud_idx, int B,
                    int fo, int woho, int wihi, int fi, int ki, int nr, int bias,
                    int state_update, int param_update,
                    const float *res_mu /* may be NULL */, const float *res_var,
                    int res_mode, float *delta_mu, float *delta_var,
                    float *delta_mu_w, float *delta_var_w, float *delta_mu_b,
                    float *delta_var_b, void *stream);

/* ---- layer glue ------------------------------------------------------------ */

/* Keep what the backward pass needs and reset the output Jacobian; replaces
 * BaseLayerCuda::store_states_for_training_cuda
 * (src/base_layer_cuda.cu:464-486): bwd_mu_a/bwd_jcb <- first n_in entries of
 * mu_a/jcb, out_jcb[0..n_out) <- 1. jcb and bwd_jcb may both be NULL (an input
 * Jacobian that is known to be one everywhere: only the mean is kept); out_jcb may
 * be NULL with n_out == 0. */
int tagi_store_states(const float *mu_a, const float *jcb, size_t n_in,
                      float *bwd_mu_a, float *bwd_jcb, float *out_jcb,
                      size_t n_out, void *stream);

/* Capped parameter step, p += sign(d) * min(|d|, sqrt(var)/cap), with
 * var <= 0 -> 1e-5; replaces device_weight_update / device_bias_update
 * (src/base_layer_cuda.cu:56-103). neg_var_count (device int, may be NULL) is
 * incremented once per clamped variance; the caller zeroes it. */
int tagi_param_update(const float *delta_mu, const float *delta_var,
                      float cap_factor, size_t n, float *mu, float *var,
                      int *neg_var_count, void *stream);

/* Uncapped step, mu += delta_mu, var += delta_var; replaces device_raw_weight_update
 * / device_raw_bias_update (src/base_layer_cuda.cu:28-54) as
 * BaseLayerCuda::raw_update_weights / raw_update_biases launch them (127-159). */
int tagi_param_raw_update(const float *delta_mu, const float *delta_var, size_t n,
                          float *mu, float *var, void *stream);

/* tagi_param_update for the weights and the biases of one layer in a single launch, as Sequential::step
 * issues them back to back (src/sequential.cpp:444-447: update_weights, then
 * update_biases of every layer): the capped step of the num_weights weights and
 * the num_biases biases (num_biases may be 0). neg_var_count (device int[2], may
 * be NULL): the clamped weight variances of this call are added to
 * neg_var_count[slot], and neg_var_count[1 - slot] is set to zero; a caller that
 * zeroes both once and alternates slot 0, 1, 0, ... reads each call's count from
 * its slot without ever resetting anything. */
int tagi_layer_update(const float *delta_mu_w, const float *delta_var_w,
                      size_t num_weights, float *mu_w, float *var_w,
                      const float *delta_mu_b, const float *delta_var_b,
                      size_t num_biases, float *mu_b, float *var_b,
                      float cap_factor, int *neg_var_count, int slot,
                      void *stream);

/* tagi_layer_update for every layer of a model in as few launches as the kernel
 * argument space allows (24 layers per launch), as Sequential::step walks its layers
 * (src/sequential.cpp:440-448): item i carries the arguments of one
 * tagi_layer_update call. `items` is a host array, read before the call returns. */
typedef struct tagi_update_item {
    const float *delta_mu_w, *delta_var_w;
    float *mu_w, *var_w;
    size_t num_weights;
    const float *delta_mu_b, *delta_var_b;
    float *mu_b, *var_b;
    size_t num_biases;
    float cap_factor;
    int *neg_var_count;
    int slot;
} tagi_update_item;
int tagi_model_update(const tagi_update_item *items /* host */, int n_items,
                      void *stream);

/* Cap factor for a batch size (src/base_layer.cpp:164-187); `prev` is returned
 * for batch sizes below 1. Host only. */
float tagi_cap_factor(int batch_size, float prev);

/* ---- output updater -------------------------------------------------------- */

/* delta_mu = jcb/(var_a+var_obs) * (obs-mu_a), delta_var = -jcb^2/(var_a+var_obs),
 * inf/nan -> 0; replaces update_delta_z_cuda (src/output_updater_cuda.cu:27-44).
 * The caller zeroes the delta buffers first, as reset_zeros does. */
int tagi_out_update_dense(const float *mu_a, const float *var_a,
                          const float *jcb, const float *obs,
                          const float *var_obs, int n, float *delta_mu,
                          float *delta_var, void *stream);

/* The same for the selected (1-based) output indices of hierarchical softmax;
 * replaces update_delta_z_using_indices_cuda (src/output_updater_cuda.cu:3-26). */
int tagi_out_update_indexed(const float *mu_a, const float *var_a,
                            const float *jcb, const float *obs,
                            const float *var_obs, const int *selected_idx,
                            int n_obs, int n_enc, int n, float *delta_mu,
                            float *delta_var, void *stream);

/* The same with the clearing of the innovation buffers included (one launch for
 * DeltaStateCuda::reset_zeros, src/data_struct_cuda.cu:262-275, and the update as
 * OutputUpdater::update_using_indices runs them, src/base_output_updater.cpp:178-205):
 * delta_mu / delta_var [0 .. delta_len) end up zero except at the selected entries.
 * obs, var_obs and selected_idx may point to pinned host memory (each value is read
 * once), which saves the transfer of the observations. n must be a multiple of n_enc
 * and (n / n_enc) * n_obs <= delta_len. */
int tagi_out_update_indexed_reset(const float *mu_a, const float *var_a,
                                  const float *jcb, const float *obs /* device or pinned host */,
                                  const float *var_obs /* device or pinned host */,
                                  const int *selected_idx /* device or pinned host */,
                                  int n_obs, int n_enc, int n, float *delta_mu,
                                  float *delta_var, size_t delta_len, void *stream);

/* Output layer with a learned (heteroscedastic) error variance: the 2n output
 * units are pairs, unit 2i the mean output and unit 2i+1 the expected squared error,
 * and obs holds n observations. Unit 2i is updated as in the dense form with the
 * expected squared error as observation noise; unit 2i+1 through the posterior
 * moments of the error and of its square. inf/nan observations give zeros. Replaces
 * update_delta_z_cuda_heteros (src/output_updater_cuda.cu:46-135, launched at
 * 225-269); CPU form src/base_output_updater.cpp:131-226. Arrays 8-byte aligned. */
int tagi_out_update_heteros(const float *mu_a, const float *var_a,
                            const float *jcb, const float *obs, int n,
                            float *delta_mu, float *delta_var, void *stream);

/* ---- ReLU -------------------------------------------------------------------- */

/* A batch of inputs from PINNED host memory (hipHostMalloc) into a state buffer: mu_a
 * <- host_mu, var_a <- host_var, or zeros when host_var is NULL; n values each. The
 * kernel reads the host arrays over the bus itself, so the transfer is one launch on
 * the compute queue; replaces the transfers of HiddenStateCuda::set_input_x +
 * chunks_to_device (src/data_struct_cuda.cu:58-80, 112-123). The host arrays must stay
 * untouched until the launch has run (record an event on `stream` after the call). */
int tagi_upload_input(const float *host_mu /* pinned host */,
                      const float *host_var /* pinned host, may be NULL */, size_t n,
                      float *mu_a, float *var_a, void *stream);
/* The way back: host_mu / host_var (PINNED host memory) <- the first n entries of mu_a /
 * var_a, written by the kernel itself; valid once `stream` has been synchronised.
 * With host_flag (pinned host memory too, may be NULL) the kernel stores flag_value there
 * after all of the data, with release order at system scope: a host thread that polls
 * *host_flag until it reads flag_value (then an acquire fence) may read the data without
 * synchronising the stream; use a value the flag does not hold yet. With a flag n is
 * limited to 2^20 (TAGI_ERR_UNSUPPORTED beyond).
 * Replaces the two transfers of HiddenStateCuda::to_host as Sequential::get_outputs /
 * output_to_host use it (src/data_struct_cuda.cu:82-110, src/sequential.cpp:470-497). */
int tagi_download_outputs(const float *mu_a, const float *var_a, size_t n,
                          float *host_mu /* pinned host */, float *host_var /* pinned host */,
                          unsigned *host_flag /* pinned host or NULL */, unsigned flag_value,
                          void *stream);

/* mu_a = max(mu_z, 0); jcb, var_a = (0, 0) where that is 0, else (1, var_z);
 * replaces relu_mean_var_cuda (src/activation_cuda.cu), CPU form
 * src/activation.cpp:7-29. In place allowed. */
int tagi_relu_fwd(const float *mu_z, const float *var_z, size_t n, float *mu_a,
                  float *jcb, float *var_a, void *stream);

/* ---- MixtureReLU ------------------------------------------------------------- */

/* Moments of max(z, 0) for z ~ N(mu_z, var_z), both floored at 1e-6; jcb = P(z > 0).
 * Replaces mixture_relu_mean_var_cuda as MixtureReLUCuda::forward launches it
 * (src/activation_cuda.cu:130-150, 726-760); CPU form src/activation.cpp:152-178.
 * In place allowed. */
int tagi_mixture_relu_fwd(const float *mu_z, const float *var_z, size_t n,
                          float *mu_a, float *jcb, float *var_a, void *stream);

/* ---- BatchNorm2d ------------------------------------------------------------- */
/* Tensors are [B][fi][wihi]; a fully-connected input is wihi = 1, fi = features.
 * Parameters, statistics and running averages are [fi]. */

/* Training-mode statistics: mu_s = mean over (B, wihi), var_s = (sum of squared
 * deviations + sum of var_a) / (B*wihi - 1), then mu_ra/var_ra <- ra*momentum +
 * s*(1 - momentum). Replaces the reduction sequence of BatchNorm2dCuda::forward
 * (src/batchnorm_layer_cuda.cu:915-948); CPU form src/batchnorm_layer.cpp:15-26,
 * 127-168. Uses the workspace. */
int tagi_batchnorm2d_stats(const float *mu_a, const float *var_a, int wihi,
                           int fi, int B, float momentum, float *mu_s,
                           float *var_s, float *mu_ra, float *var_ra,
                           void *stream);

/* mu_z = (mu_a - mu_norm)/sqrt(var_norm + eps) * mu_w (+ mu_b); var_z likewise
 * with Gaussian weights. mu_norm/var_norm: batch statistics when training, running
 * averages otherwise. Replaces batchnorm2d_fwd_mean_var_cuda
 * (src/batchnorm_layer_cuda.cu:507-543, launched at 950-959); CPU form
 * src/batchnorm_layer.cpp:170-206. */
int tagi_batchnorm2d_fwd(const float *mu_w, const float *var_w,
                         const float *mu_b, const float *var_b,
                         const float *mu_a, const float *var_a,
                         const float *mu_norm, const float *var_norm, int bias,
                         float epsilon, int wihi, int fi, int B, float *mu_z,
                         float *var_z, void *stream);

/* tagi_batchnorm2d_fwd followed by the residual add that ends on this layer, in one
 * pass: mu_z += mu_res, var_z += var_res ([B][fi][wihi] like the output). Replaces a
 * BatchNorm2dCuda::forward that closes the main block of a ResNetBlock together with
 * the add_shortcut_mean_var_cuda launch of ResNetBlockCuda::forward
 * (src/resnet_block_cuda.cu:7-18, 262-287). */
int tagi_batchnorm2d_fwd_res(const float *mu_w, const float *var_w,
                             const float *mu_b, const float *var_b,
                             const float *mu_a, const float *var_a,
                             const float *mu_norm, const float *var_norm,
                             const float *mu_res, const float *var_res, int bias,
                             float epsilon, int wihi, int fi, int B, float *mu_z,
                             float *var_z, void *stream);

/* A training-mode forward in one call: tagi_batchnorm2d_stats followed by
 * tagi_batchnorm2d_fwd (mu_res == NULL) or tagi_batchnorm2d_fwd_res with the batch
 * statistics, i.e. all of BatchNorm2dCuda::forward in training mode
 * (src/batchnorm_layer_cuda.cu:915-959). The results are the same bits; where the
 * 16-byte path applies the statistics are merged by the normalising kernel itself (two
 * launches instead of three). mu_s / var_s receive the batch statistics (the backward
 * pass needs them), mu_ra / var_ra are updated. Uses the workspace. */
int tagi_batchnorm2d_fwd_train(const float *mu_w, const float *var_w,
                               const float *mu_b, const float *var_b,
                               const float *mu_a, const float *var_a,
                               const float *mu_res /* may be NULL */,
                               const float *var_res, int bias, float momentum,
                               float epsilon, int wihi, int fi, int B, float *mu_s,
                               float *var_s, float *mu_ra, float *var_ra,
                               float *mu_z, float *var_z, void *stream);

/* All of BatchNorm2dCuda::backward (src/batchnorm_layer_cuda.cu:969-1102) in one
 * call: state innovations (state_update) and the per-channel weight / bias
 * innovations (param_update; bias ones only when bias != 0). mu_a and jcb are the
 * layer's stored input states. CPU form src/batchnorm_layer.cpp:233-255, 307-354
 * and delta_param_sum (src/common.cpp:360-378). Uses the workspace. */
int tagi_batchnorm2d_bwd(const float *mu_w, const float *var_w,
                         const float *var_b, const float *mu_a,
                         const float *jcb, const float *mu_norm,
                         const float *var_norm, const float *delta_mu_out,
                         const float *delta_var_out, float epsilon, int wihi,
                         int fi, int B, int bias, int state_update,
                         int param_update, float *delta_mu, float *delta_var,
                         float *delta_mu_w, float *delta_var_w,
                         float *delta_mu_b, float *delta_var_b, void *stream);

/* ---- AvgPool2d ---------------------------------------------------------------- */

/* Host tables of a pooling layer, as AvgPool2d::lazy_index_init builds them
 * (src/pooling_layer.cpp:186-210 over get_pool_index, 453-484): pool_idx
 * [kernel*kernel][wo*ho] (1-based input pixel, -1 = padding) and, only when the
 * windows overlap (*overlap = 1), z_ud_idx [h][w] (1-based output pixel, -1 =
 * none). Caller provides pool_idx[wo*ho*k*k] and z_ud_idx[wi*hi*k*k]. The output
 * size comes from tagi_conv2d_out_size; stride -1 (the pooling default) is valid
 * for a window that covers the whole image. */
int tagi_avgpool2d_build_idx(int kernel, int stride, int wi, int hi, int pad,
                             int pad_type, int *pool_idx, int *z_ud_idx, int *w,
                             int *h, int *overlap);

/* mu_z = window sum / k^2, var_z = window sum / k^4 (padding counts in the
 * divisor); n_out = woho*channels*B. Replaces avgpool2d_fwd_*_mean_var_cuda
 * (src/pooling_layer_cuda.cu:13-64, launched at 167-218); CPU form
 * src/pooling_layer.cpp:201-225, 259-280. */
int tagi_avgpool2d_fwd(const float *mu_a, const float *var_a,
                       const int *pool_idx, int woho, int wihi, int ki,
                       int n_out, float *mu_z, float *var_z, void *stream);

/* State innovations of the pooling layer; n_in = wihi*channels*B. overlap != 0
 * walks z_ud_idx (nr rows); otherwise the windows tile the image and wo (output
 * width) is enough. Replaces avgpool2d_bwd_*_delta_z_cuda
 * (src/pooling_layer_cuda.cu:66-120, launched at 220-270); CPU form
 * src/pooling_layer.cpp:316-340, 379-399. */
int tagi_avgpool2d_bwd_dz(const float *jcb, const float *delta_mu_out,
                          const float *delta_var_out, const int *z_ud_idx,
                          int woho, int wihi, int ki, int nr, int wo, int n_in,
                          int overlap, float *delta_mu, float *delta_var,
                          void *stream);

/* ---- residual connection -------------------------------------------------------- */

/* mu_a += mu_s, var_a += var_s; replaces add_shortcut_mean_var_cuda
 * (src/resnet_block_cuda.cu:7-18); CPU form src/resnet_block.cpp:8-18. */
int tagi_add_shortcut(const float *mu_s, const float *var_s, size_t n,
                      float *mu_a, float *var_a, void *stream);

/* mu_a += mu_s*jcb_s, var_a += var_s*jcb_s^2; replaces add_shortcut_delta_cuda
 * (src/resnet_block_cuda.cu:20-33); CPU form src/resnet_block.cpp:20-31. */
int tagi_add_shortcut_delta(const float *mu_s, const float *var_s,
                            const float *jcb_s, size_t n, float *mu_a,
                            float *var_a, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TAGI_HIP_H */

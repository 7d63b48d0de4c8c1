/*
 * CPU oracle for the TAGI Linear / Conv2d hot path and the layers around it
 * (MixtureReLU, BatchNorm2d, AvgPool2d, residual adds).
 *
 * TEST INFRASTRUCTURE ONLY. This is a plain C++ restatement of the reference
 * CPU algorithms (cuTAGI, src/*.cpp), used as the checker in tests, in the
 * smoke test and as the timed CPU baseline of the benchmark. Nothing in the
 * shipped library links, loads or calls it.
 *
 * Every function walks its outputs in the reference's order, accumulates in
 * fp32 in the reference's term order and fans out over `threads` std::threads
 * the way the reference's `_mp` wrappers do (contiguous chunks of the flat
 * output index, remainder spread over the first threads), so that a build with
 * the reference's flags (-O3, no -march=native, no fast-math) is bit-identical
 * to the compiled reference. `threads <= 1` runs the serial loop.
 *
 * Layouts: weights [N][K] row-major, activations [B][K], outputs [B][N];
 * conv weights OIHW, conv activations NCHW; index tables int32, 1-based.
 *
 * Pinning status of each function (what it was checked against):
 *   all functions below  - bit-for-bit against oracle/_ref (the reference's own
 *                          sources compiled here) on seeded inputs, and against
 *                          fp64 closed forms / brute force in tests/.
 */
#pragma once
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- Linear ------------------------------------------------------------ */
/* reference: src/linear_layer.cpp:10-61 (+ _mp 63-99) */
void oracle_linear_fwd(const float *mu_w, const float *var_w,
                       const float *mu_b, const float *var_b,
                       const float *mu_a, const float *var_a, int K, int N,
                       int B, int bias, int threads, float *mu_z,
                       float *var_z);
/* reference: src/linear_layer.cpp:245-273 (+ _mp 275-312) */
void oracle_linear_bwd_dz(const float *mu_w, const float *jcb,
                          const float *delta_mu, const float *delta_var, int K,
                          int N, int B, int threads, float *delta_mu_z,
                          float *delta_var_z);
/* reference: src/linear_layer.cpp:314-350 (+ _mp 352-389) */
void oracle_linear_bwd_dw(const float *var_w, const float *mu_a,
                          const float *delta_mu, const float *delta_var, int K,
                          int N, int B, int threads, float *delta_mu_w,
                          float *delta_var_w);
/* reference: src/linear_layer.cpp:391-424 (+ _mp 426-459) */
void oracle_linear_bwd_db(const float *var_b, const float *delta_mu,
                          const float *delta_var, int N, int B, int threads,
                          float *delta_mu_b, float *delta_var_b);

/* ---- Conv2d index tables ------------------------------------------------ */
/* reference: src/conv2d_layer.cpp:581-628. Returns 0, or -1 when the geometry
 * does not divide (the reference throws there). */
int oracle_conv2d_out_size(int kernel, int stride, int wi, int hi, int pad,
                           int pad_type, int *wo, int *ho);
/* reference: src/conv2d_layer.cpp:656-719 over src/indices.cpp (image
 * construction 10-137, receptive field 142-262, reference sort 267-464,
 * table fill 514-696) and src/common.cpp:36-55 (transpose).
 * Caller provides Fmwa_2[wo*ho*k*k], FCzwa_1[wi*hi*k*k], Szz_ud[wi*hi*k*k];
 * the used part is w*h ints. pad_idx_in/out = -1, as Conv2d::lazy_index_init
 * passes (conv2d_layer.cpp:96-115). Returns 0 on success. */
int oracle_conv2d_build_idx(int kernel, int stride, int wi, int hi, int wo,
                            int ho, int pad, int pad_type, int param_pad_idx,
                            int *Fmwa_2, int *FCzwa_1, int *Szz_ud, int *w,
                            int *h);

/* ---- Conv2d -------------------------------------------------------------- */
/* reference: src/conv2d_layer.cpp:274-323 (+ _mp 325-361) */
void oracle_conv2d_fwd(const float *mu_w, const float *var_w,
                       const float *mu_b, const float *var_b,
                       const float *mu_a, const float *var_a, const int *aidx,
                       int woho, int fo, int wihi, int fi, int ki, int B,
                       int bias, int threads, float *mu_z, float *var_z);
/* reference: permute_jacobian (conv2d_layer.cpp:444-457) followed by
 * conv2d_bwd_delta_z (363-404, _mp 406-442). jcb is the un-permuted
 * [B][fi][wihi] Jacobian; tmp is scratch of B*fi*wihi floats. */
void oracle_conv2d_bwd_dz(const float *mu_w, const float *jcb,
                          const float *delta_mu_out,
                          const float *delta_var_out, const int *zw_idx,
                          const int *zud_idx, int woho, int fo, int wihi,
                          int fi, int ki, int nr, int B, int threads,
                          float *tmp, float *delta_mu, float *delta_var);
/* reference: permute_delta (conv2d_layer.cpp:558-575) followed by
 * conv2d_bwd_delta_w (459-495, _mp 497-536) and, when bias != 0,
 * conv2d_bwd_delta_b (538-556). tmp_1/tmp_2 are scratch of B*fo*woho. */
void oracle_conv2d_bwd_dw(const float *var_w, const float *var_b,
                          const float *mu_a, const float *delta_mu_out,
                          const float *delta_var_out, const int *aidx, int B,
                          int fo, int woho, int wihi, int fi, int ki, int bias,
                          int threads, float *tmp_1, float *tmp_2,
                          float *delta_mu_w, float *delta_var_w,
                          float *delta_mu_b, float *delta_var_b);

/* ---- Parameter update ---------------------------------------------------- */
/* reference: src/base_layer.cpp:164-187. `prev` is the factor the layer held
 * before (the reference leaves it untouched for batch sizes <= 0). */
float oracle_cap_factor(int batch_size, float prev);
/* reference: src/base_layer.cpp:116-162 (weights and biases share the loop;
 * only the weight call counts clamped variances). Returns that count. */
int oracle_param_update(float *mu, float *var, const float *delta_mu,
                        const float *delta_var, size_t n, float cap_factor);

/* ---- Output updater ------------------------------------------------------ */
/* reference: src/base_output_updater.cpp:8-29 */
void oracle_out_update_dense(const float *mu_a, const float *var_a,
                             const float *jcb, const float *obs,
                             const float *var_obs, int n, float *delta_mu,
                             float *delta_var);
/* reference: src/base_output_updater.cpp:131-226; n observations, 2n output units
 * (mean at 2i, learned error variance at 2i+1) */
void oracle_out_update_heteros(const float *mu_a, const float *var_a,
                               const float *jcb, const float *obs, int n,
                               float *delta_mu, float *delta_var);
/* reference: src/base_output_updater.cpp:67-93; selected_idx is 1-based */
void oracle_out_update_indexed(const float *mu_a, const float *var_a,
                               const float *jcb, const float *obs,
                               const float *var_obs, const int *selected_idx,
                               int n_obs, int n_enc, int n, float *delta_mu,
                               float *delta_var);

/* ---- ReLU ----------------------------------------------------------------- */
/* reference: src/activation.cpp:7-29 */
void oracle_relu_fwd(const float *mu_z, const float *var_z, int n, float *mu_a,
                     float *jcb, float *var_a);

/* ---- MixtureReLU ---------------------------------------------------------- */
/* reference: src/activation.cpp:152-178 (+ _mp 180-212) */
void oracle_mixture_relu_fwd(const float *mu_z, const float *var_z, int n,
                             int threads, float *mu_a, float *jcb,
                             float *var_a);

/* ---- BatchNorm2d ----------------------------------------------------------- */
/* Batch statistics of a [B][fi][wihi] tensor, training mode. reference:
 * batchnorm2d_stat_mean_var (src/batchnorm_layer.cpp:127-147), then
 * batchnorm2d_sample_var (149-168), then running_mean_var (15-26) with the
 * given momentum. var_s_tmp holds fi floats (the sums of var_a).
 * A fully-connected input is the case wihi = 1, fi = features. */
void oracle_batchnorm2d_stats(const float *mu_a, const float *var_a, int wihi,
                              int fi, int B, float momentum, int threads,
                              float *var_s_tmp, float *mu_s, float *var_s,
                              float *mu_ra, float *var_ra);
/* reference: src/batchnorm_layer.cpp:170-206 (+ _mp 521-556). mu_norm/var_norm
 * are the batch statistics (training) or the running averages (inference). */
void oracle_batchnorm2d_fwd(const float *mu_w, const float *var_w,
                            const float *mu_b, const float *var_b,
                            const float *mu_a, const float *var_a,
                            const float *mu_norm, const float *var_norm,
                            int bias, float epsilon, int wihi, int fi, int B,
                            int threads, float *mu_z, float *var_z);
/* reference: src/batchnorm_layer.cpp:233-255 (+ _mp 593-626) */
void oracle_batchnorm2d_bwd_dz(const float *mu_w, const float *jcb,
                               const float *var_norm, const float *delta_mu_out,
                               const float *delta_var_out, float epsilon,
                               int wihi, int fi, int B, int threads,
                               float *delta_mu, float *delta_var);
/* reference: batchnorm2d_bwd_delta_w (src/batchnorm_layer.cpp:307-332) and,
 * when bias != 0, batchnorm2d_bwd_delta_b (334-354), each followed by
 * delta_param_sum (src/common.cpp:360-378). tmp_1/tmp_2: B*fi*wihi floats. */
void oracle_batchnorm2d_bwd_dw(const float *var_w, const float *var_b,
                               const float *mu_a, const float *mu_norm,
                               const float *var_norm, const float *delta_mu_out,
                               const float *delta_var_out, float epsilon,
                               int wihi, int fi, int B, int bias, int threads,
                               float *tmp_1, float *tmp_2, float *delta_mu_w,
                               float *delta_var_w, float *delta_mu_b,
                               float *delta_var_b);

/* ---- AvgPool2d -------------------------------------------------------------- */
/* reference: get_pool_index (src/pooling_layer.cpp:453-484) as
 * AvgPool2d::lazy_index_init calls it (pad indices -1). pool_idx is
 * [kernel*kernel][wo*ho] (1-based input pixel, -1 = padding); z_ud_idx is
 * [h][w] (1-based output pixel, -1 = none) and is only filled for overlapping
 * windows (*overlap = 1), as the reference leaves it empty otherwise.
 * Caller provides pool_idx[wo*ho*k*k] and z_ud_idx[wi*hi*k*k]. */
int oracle_avgpool2d_build_idx(int kernel, int stride, int wi, int hi, int wo,
                               int ho, int pad, int pad_type, int *pool_idx,
                               int *z_ud_idx, int *w, int *h, int *overlap);
/* reference: avgpool2d_fwd_overlapped_mean_var (src/pooling_layer.cpp:201-225)
 * when overlap != 0, else avgpool2d_fwd_mean_var (259-280); n_out = woho*fo*B,
 * n_in = wihi*fo*B */
void oracle_avgpool2d_fwd(const float *mu_a, const float *var_a,
                          const int *pool_idx, int woho, int wihi, int ki,
                          int n_out, int n_in, int overlap, int threads,
                          float *mu_z, float *var_z);
/* reference: avgpool2d_bwd_overlapped_delta_z (src/pooling_layer.cpp:316-340)
 * when overlap != 0 (nr = rows of z_ud_idx), else avgpool2d_bwd_delta_z
 * (379-399) with wo the output width; n_in = wihi*fi*B, n_out = woho*fi*B */
void oracle_avgpool2d_bwd_dz(const float *jcb, const float *delta_mu_out,
                             const float *delta_var_out, const int *z_ud_idx,
                             int woho, int wihi, int ki, int nr, int wo,
                             int n_in, int n_out, int overlap, int threads,
                             float *delta_mu, float *delta_var);

/* ---- Residual connection ------------------------------------------------------ */
/* reference: add_shortcut_mean_var (src/resnet_block.cpp:8-18) */
void oracle_add_shortcut(const float *mu_s, const float *var_s, int n,
                         float *mu_a, float *var_a);
/* reference: add_shortcut_delta (src/resnet_block.cpp:20-31) */
void oracle_add_shortcut_delta(const float *mu_s, const float *var_s,
                               const float *jcb_s, int n, float *mu_a,
                               float *var_a);

#ifdef __cplusplus
}
#endif

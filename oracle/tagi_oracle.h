/*
 * CPU oracle for the TAGI Linear / Conv2d hot path.
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

#ifdef __cplusplus
}
#endif

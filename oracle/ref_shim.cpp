// extern "C" wrappers around the reference's own CPU functions, compiled by
// oracle/Makefile together with the reference sources where they lie (the
// REF variable, by default /root/reference) into oracle/_ref/libtagi_ref.so.
// TEST INFRASTRUCTURE ONLY: used to validate tagi_oracle.cpp bit for bit and to
// write the golden vectors under tests/golden/. It carries the same signatures
// as tagi_oracle.h with a `ref_` prefix. No reference source is copied here:
// this file only includes the reference headers and calls into them.
#include <cstring>
#include <fstream>
#include <memory>
#include <stdexcept>
#include <tuple>
#include <vector>

#include "activation.h"
#include "base_layer.h"
#include "base_output_updater.h"
#include "conv2d_layer.h"
#include "cost.h"
#include "linear_layer.h"
#include "batchnorm_layer.h"
#include "layer_block.h"
#include "pooling_layer.h"
#include "resnet_block.h"

// Free functions the reference defines in its .cpp files without declaring them
// in a header (src/batchnorm_layer.cpp:15-354,457-775, src/resnet_block.cpp:8-31,
// src/common.cpp:360-378): declared here so that they can be called.
void running_mean_var(const std::vector<float> &mu_s, const std::vector<float> &var_s,
                      float momentum, int start_chunk, int end_chunk,
                      std::vector<float> &mu_ra, std::vector<float> &var_ra);
void running_mean_var_mp(const std::vector<float> &mu_s, const std::vector<float> &var_s,
                         float momentum, int num_states, const int num_threads,
                         std::vector<float> &mu_ra, std::vector<float> &var_ra);
void batchnorm2d_stat_mean_var(const std::vector<float> &mu_a, const std::vector<float> &var_a,
                               int wihi, int fi, int batch_size, int start_chunk, int end_chunk,
                               std::vector<float> &mu_s, std::vector<float> &var_s);
void batchnorm2d_stat_mean_var_mp(const std::vector<float> &mu_a,
                                  const std::vector<float> &var_a, int wihi, int fi,
                                  int batch_size, const int num_threads,
                                  std::vector<float> &mu_s, std::vector<float> &var_s);
void batchnorm2d_sample_var(const std::vector<float> &mu_a, const std::vector<float> &mu_s,
                            const std::vector<float> &var_s, int wihi, int fi, int batch_size,
                            int start_chunk, int end_chunk, std::vector<float> &var);
void batchnorm2d_sample_var_mp(const std::vector<float> &mu_a, const std::vector<float> &mu_s,
                               const std::vector<float> &var_s, int wihi, int fi,
                               int batch_size, const int num_threads, std::vector<float> &var);
void batchnorm2d_fwd_mean_var(const std::vector<float> &mu_w, const std::vector<float> &var_w,
                              const std::vector<float> &mu_b, const std::vector<float> &var_b,
                              const std::vector<float> &mu_a, const std::vector<float> &var_a,
                              const std::vector<float> &mu_ra, const std::vector<float> &var_ra,
                              bool bias, float epsilon, int wihi, int fi, int batch_size,
                              int start_chunk, int end_chunk, std::vector<float> &mu_z,
                              std::vector<float> &var_z);
void batchnorm2d_fwd_mean_var_mp(const std::vector<float> &mu_w, const std::vector<float> &var_w,
                                 const std::vector<float> &mu_b, const std::vector<float> &var_b,
                                 const std::vector<float> &mu_a, const std::vector<float> &var_a,
                                 const std::vector<float> &mu_ra,
                                 const std::vector<float> &var_ra, bool bias, float epsilon,
                                 int wihi, int fi, int batch_size, const int num_threads,
                                 std::vector<float> &mu_z, std::vector<float> &var_z);
void batchnorm2d_bwd_delta_z(const std::vector<float> &mu_w, const std::vector<float> &jcb,
                             const std::vector<float> &var_ra,
                             const std::vector<float> &delta_mu_out,
                             const std::vector<float> &delta_var_out, float epsilon, int wihi,
                             int fi, int batch_size, int start_chunk, int end_chunk,
                             std::vector<float> &delta_mu, std::vector<float> &delta_var);
void batchnorm2d_bwd_delta_z_mp(const std::vector<float> &mu_w, const std::vector<float> &jcb,
                                const std::vector<float> &var_ra,
                                const std::vector<float> &delta_mu_out,
                                const std::vector<float> &delta_var_out, float epsilon, int wihi,
                                int fi, int batch_size, const int num_threads,
                                std::vector<float> &delta_mu, std::vector<float> &delta_var);
void batchnorm2d_bwd_delta_w(const std::vector<float> &var_w, const std::vector<float> &mu_a,
                             const std::vector<float> &mu_ra, const std::vector<float> &var_ra,
                             const std::vector<float> &delta_mu_out,
                             const std::vector<float> &delta_var_out, float epsilon, int wihi,
                             int fi, int batch_size, int start_chunk, int end_chunk,
                             std::vector<float> &delta_mu_w, std::vector<float> &delta_var_w);
void batchnorm2d_bwd_delta_w_mp(const std::vector<float> &var_w, const std::vector<float> &mu_a,
                                const std::vector<float> &mu_ra,
                                const std::vector<float> &var_ra,
                                const std::vector<float> &delta_mu_out,
                                const std::vector<float> &delta_var_out, float epsilon, int wihi,
                                int fi, int batch_size, const int num_threads,
                                std::vector<float> &delta_mu_w, std::vector<float> &delta_var_w);
void batchnorm2d_bwd_delta_b(const std::vector<float> &var_b,
                             const std::vector<float> &delta_mu_out,
                             const std::vector<float> &delta_var_out, float epsilon, int wihi,
                             int fi, int start_chunk, int end_chunk,
                             std::vector<float> &delta_mu_b, std::vector<float> &delta_var_b);
void batchnorm2d_bwd_delta_b_mp(const std::vector<float> &var_b,
                                const std::vector<float> &delta_mu_out,
                                const std::vector<float> &delta_var_out, float epsilon, int wihi,
                                int fi, int batch_size, const int num_threads,
                                std::vector<float> &delta_mu_b, std::vector<float> &delta_var_b);
void delta_param_sum(const std::vector<float> &delta_mu_e, const std::vector<float> &delta_var_e,
                     int wihi, int fi, int batch_size, std::vector<float> &delta_mu,
                     std::vector<float> &delta_var);
void add_shortcut_mean_var(const std::vector<float> &mu_s, const std::vector<float> &var_s,
                           int num_states, std::vector<float> &mu_a, std::vector<float> &var_a);
void add_shortcut_delta(const std::vector<float> &mu_s, const std::vector<float> &var_s,
                        const std::vector<float> &jcb_s, int num_states,
                        std::vector<float> &mu_a, std::vector<float> &var_a);

namespace {
std::vector<float> vec(const float *p, size_t n) {
    return p ? std::vector<float>(p, p + n) : std::vector<float>();
}
std::vector<int> ivec(const int *p, size_t n) { return std::vector<int>(p, p + n); }
void put(const std::vector<float> &v, float *out) {
    std::memcpy(out, v.data(), v.size() * sizeof(float));
}
}  // namespace

extern "C" {

void ref_linear_fwd(const float *mu_w, const float *var_w, const float *mu_b,
                    const float *var_b, const float *mu_a, const float *var_a,
                    int K, int N, int B, int bias, int threads, float *mu_z,
                    float *var_z) {
    auto mw = vec(mu_w, (size_t)N * K), vw = vec(var_w, (size_t)N * K);
    auto mb = vec(bias ? mu_b : nullptr, N), vb = vec(bias ? var_b : nullptr, N);
    auto ma = vec(mu_a, (size_t)B * K), va = vec(var_a, (size_t)B * K);
    std::vector<float> mz((size_t)B * N), vz((size_t)B * N);
    if (threads > 1)
        linear_fwd_mean_var_mp(mw, vw, mb, vb, ma, va, K, N, B, bias != 0, threads, mz, vz);
    else
        linear_fwd_mean_var(mw, vw, mb, vb, ma, va, 0, N * B, K, N, B, bias != 0, mz, vz);
    put(mz, mu_z);
    put(vz, var_z);
}

void ref_linear_bwd_dz(const float *mu_w, const float *jcb, const float *delta_mu,
                       const float *delta_var, int K, int N, int B, int threads,
                       float *delta_mu_z, float *delta_var_z) {
    auto mw = vec(mu_w, (size_t)N * K), jc = vec(jcb, (size_t)B * K);
    auto dm = vec(delta_mu, (size_t)B * N), dv = vec(delta_var, (size_t)B * N);
    std::vector<float> om((size_t)B * K), ov((size_t)B * K);
    if (threads > 1)
        linear_bwd_fc_delta_z_mp(mw, jc, dm, dv, K, N, B, threads, om, ov);
    else
        linear_bwd_fc_delta_z(mw, jc, dm, dv, K, N, B, 0, B * K, om, ov);
    put(om, delta_mu_z);
    put(ov, delta_var_z);
}

void ref_linear_bwd_dw(const float *var_w, const float *mu_a, const float *delta_mu,
                       const float *delta_var, int K, int N, int B, int threads,
                       float *delta_mu_w, float *delta_var_w) {
    auto vw = vec(var_w, (size_t)N * K), ma = vec(mu_a, (size_t)B * K);
    auto dm = vec(delta_mu, (size_t)B * N), dv = vec(delta_var, (size_t)B * N);
    std::vector<float> om((size_t)N * K), ov((size_t)N * K);
    if (threads > 1)
        linear_bwd_fc_delta_w_mp(vw, ma, dm, dv, K, N, B, threads, om, ov);
    else
        linear_bwd_fc_delta_w(vw, ma, dm, dv, K, N, B, 0, K * N, om, ov);
    put(om, delta_mu_w);
    put(ov, delta_var_w);
}

void ref_linear_bwd_db(const float *var_b, const float *delta_mu, const float *delta_var,
                       int N, int B, int threads, float *delta_mu_b, float *delta_var_b) {
    auto vb = vec(var_b, N);
    auto dm = vec(delta_mu, (size_t)B * N), dv = vec(delta_var, (size_t)B * N);
    std::vector<float> om(N), ov(N);
    if (threads > 1)
        linear_bwd_fc_delta_b_mp(vb, dm, dv, N, B, threads, om, ov);
    else
        linear_bwd_fc_delta_b(vb, dm, dv, N, B, 0, N, om, ov);
    put(om, delta_mu_b);
    put(ov, delta_var_b);
}

int ref_conv2d_out_size(int kernel, int stride, int wi, int hi, int pad, int pad_type,
                        int *wo, int *ho) {
    try {
        std::tie(*wo, *ho) = compute_downsample_img_size_v2(kernel, stride, wi, hi, pad, pad_type);
    } catch (const std::exception &) {
        return -1;
    }
    return 0;
}

int ref_conv2d_build_idx(int kernel, int stride, int wi, int hi, int wo, int ho, int pad,
                         int pad_type, int param_pad_idx, int *Fmwa_2, int *FCzwa_1,
                         int *Szz_ud, int *w, int *h) {
    try {
        Conv2dIndex idx =
            get_conv2d_idx(kernel, stride, wi, hi, wo, ho, pad, pad_type, -1, -1, param_pad_idx);
        std::memcpy(Fmwa_2, idx.Fmwa_2_idx.data(), idx.Fmwa_2_idx.size() * sizeof(int));
        std::memcpy(FCzwa_1, idx.FCzwa_1_idx.data(), idx.FCzwa_1_idx.size() * sizeof(int));
        std::memcpy(Szz_ud, idx.Szz_ud_idx.data(), idx.Szz_ud_idx.size() * sizeof(int));
        *w = idx.w;
        *h = idx.h;
    } catch (const std::exception &) {
        return -1;
    }
    return 0;
}

void ref_conv2d_fwd(const float *mu_w, const float *var_w, const float *mu_b,
                    const float *var_b, const float *mu_a, const float *var_a,
                    const int *aidx, int woho, int fo, int wihi, int fi, int ki, int B,
                    int bias, int threads, float *mu_z, float *var_z) {
    const size_t nw = (size_t)ki * ki * fi * fo;
    auto mw = vec(mu_w, nw), vw = vec(var_w, nw);
    auto mb = vec(bias ? mu_b : nullptr, fo), vb = vec(bias ? var_b : nullptr, fo);
    auto ma = vec(mu_a, (size_t)B * fi * wihi), va = vec(var_a, (size_t)B * fi * wihi);
    auto ai = ivec(aidx, (size_t)woho * ki * ki);
    std::vector<float> mz((size_t)B * fo * woho), vz((size_t)B * fo * woho);
    const int pad_idx = wihi * fi * B + 1;
    if (threads > 1)
        conv2d_fwd_mean_var_mp(mw, vw, mb, vb, ma, va, ai, woho, fo, wihi, fi, ki, B, pad_idx,
                               bias != 0, threads, mz, vz);
    else
        conv2d_fwd_mean_var(mw, vw, mb, vb, ma, va, ai, woho, fo, wihi, fi, ki, B, pad_idx,
                            bias != 0, 0, woho * B * fo, mz, vz);
    put(mz, mu_z);
    put(vz, var_z);
}

void ref_conv2d_bwd_dz(const float *mu_w, const float *jcb, const float *delta_mu_out,
                       const float *delta_var_out, const int *zw_idx, const int *zud_idx,
                       int woho, int fo, int wihi, int fi, int ki, int nr, int B, int threads,
                       float *tmp, float *delta_mu, float *delta_var) {
    const size_t nw = (size_t)ki * ki * fi * fo;
    auto mw = vec(mu_w, nw);
    auto jc = vec(jcb, (size_t)B * fi * wihi);
    auto dm = vec(delta_mu_out, (size_t)B * fo * woho), dv = vec(delta_var_out, (size_t)B * fo * woho);
    auto zw = ivec(zw_idx, (size_t)wihi * nr), zud = ivec(zud_idx, (size_t)wihi * nr);
    std::vector<float> t1((size_t)B * fi * wihi), om((size_t)B * fi * wihi), ov((size_t)B * fi * wihi);
    permute_jacobian(jc, wihi, fi, B, t1);
    const int pad_idx = woho * fo * B + 1;
    if (threads > 1)
        conv2d_bwd_delta_z_mp(mw, t1, dm, dv, zw, zud, woho, fo, wihi, fi, ki, nr, nr * fo, B,
                              pad_idx, threads, om, ov);
    else
        conv2d_bwd_delta_z(mw, t1, dm, dv, zw, zud, woho, fo, wihi, fi, ki, nr, nr * fo, B,
                           pad_idx, 0, wihi * B * fi, om, ov);
    put(t1, tmp);
    put(om, delta_mu);
    put(ov, delta_var);
}

void ref_conv2d_bwd_dw(const float *var_w, const float *var_b, const float *mu_a,
                       const float *delta_mu_out, const float *delta_var_out, const int *aidx,
                       int B, int fo, int woho, int wihi, int fi, int ki, int bias, int threads,
                       float *tmp_1, float *tmp_2, float *delta_mu_w, float *delta_var_w,
                       float *delta_mu_b, float *delta_var_b) {
    const size_t nw = (size_t)ki * ki * fi * fo;
    auto vw = vec(var_w, nw);
    auto vb = vec(bias ? var_b : nullptr, fo);
    auto ma = vec(mu_a, (size_t)B * fi * wihi);
    auto dm = vec(delta_mu_out, (size_t)B * fo * woho), dv = vec(delta_var_out, (size_t)B * fo * woho);
    auto ai = ivec(aidx, (size_t)woho * ki * ki);
    std::vector<float> t1((size_t)B * fo * woho), t2((size_t)B * fo * woho), om(nw), ov(nw);
    permute_delta(dm, dv, woho, woho * fo, B, t1, t2);
    const int pad_idx = wihi * fi * B + 1;
    if (threads > 1)
        conv2d_bwd_delta_w_mp(vw, ma, t1, t2, ai, B, fo, woho, wihi, fi, ki, pad_idx, threads, om, ov);
    else
        conv2d_bwd_delta_w(vw, ma, t1, t2, ai, B, fo, woho, wihi, fi, ki, pad_idx, 0, (int)nw, om, ov);
    put(t1, tmp_1);
    put(t2, tmp_2);
    put(om, delta_mu_w);
    put(ov, delta_var_w);
    if (bias) {
        std::vector<float> bm(fo), bv(fo);
        conv2d_bwd_delta_b(vb, t1, t2, woho * B, fo, bm, bv);
        put(bm, delta_mu_b);
        put(bv, delta_var_b);
    }
}

float ref_cap_factor(int batch_size, float prev) {
    BaseLayer layer;
    layer.cap_factor_update = prev;
    layer.set_cap_factor_udapte(batch_size);
    return layer.cap_factor_update;
}

// weights != 0: BaseLayer::update_weights, else BaseLayer::update_biases
int ref_param_update(float *mu, float *var, const float *delta_mu, const float *delta_var,
                     size_t n, float cap_factor, int weights) {
    BaseLayer layer;
    layer.cap_factor_update = cap_factor;
    layer.bias = true;
    if (weights) {
        layer.mu_w = vec(mu, n); layer.var_w = vec(var, n);
        layer.delta_mu_w = vec(delta_mu, n); layer.delta_var_w = vec(delta_var, n);
        layer.update_weights();
        put(layer.mu_w, mu); put(layer.var_w, var);
        return layer.get_neg_var_w_counter();
    }
    layer.mu_b = vec(mu, n); layer.var_b = vec(var, n);
    layer.delta_mu_b = vec(delta_mu, n); layer.delta_var_b = vec(delta_var, n);
    layer.update_biases();
    put(layer.mu_b, mu); put(layer.var_b, var);
    return 0;
}

void ref_out_update_dense(const float *mu_a, const float *var_a, const float *jcb,
                          const float *obs, const float *var_obs, int n, float *delta_mu,
                          float *delta_var) {
    auto ma = vec(mu_a, n), va = vec(var_a, n), jc = vec(jcb, n), ob = vec(obs, n), vo = vec(var_obs, n);
    auto dm = vec(delta_mu, n), dv = vec(delta_var, n);
    compute_delta_z_output(ma, va, jc, ob, vo, 0, n, dm, dv);
    put(dm, delta_mu);
    put(dv, delta_var);
}

// n observations, 2n output units
void ref_out_update_heteros(const float *mu_a, const float *var_a, const float *jcb,
                            const float *obs, int n, float *delta_mu, float *delta_var) {
    auto ma = vec(mu_a, 2 * n), va = vec(var_a, 2 * n), jc = vec(jcb, 2 * n), ob = vec(obs, n);
    auto dm = vec(delta_mu, 2 * n), dv = vec(delta_var, 2 * n);
    compute_delta_z_heteros(ma, va, jc, ob, 0, 2 * n, dm, dv);
    put(dm, delta_mu);
    put(dv, delta_var);
}

// n_states = block_size * n_obs floats in the state / delta arrays
void ref_out_update_indexed(const float *mu_a, const float *var_a, const float *jcb,
                            const float *obs, const float *var_obs, const int *selected_idx,
                            int n_obs, int n_enc, int n, int n_states, float *delta_mu,
                            float *delta_var) {
    auto ma = vec(mu_a, n_states), va = vec(var_a, n_states), jc = vec(jcb, n_states);
    auto ob = vec(obs, n), vo = vec(var_obs, n);
    auto si = ivec(selected_idx, n);
    auto dm = vec(delta_mu, n_states), dv = vec(delta_var, n_states);
    compute_selected_delta_z_output(ma, va, jc, ob, vo, si, n_obs, n_enc, 0, n, dm, dv);
    put(dm, delta_mu);
    put(dv, delta_var);
}

void ref_relu_fwd(const float *mu_z, const float *var_z, int n, float *mu_a, float *jcb,
                  float *var_a) {
    auto mz = vec(mu_z, n), vz = vec(var_z, n);
    std::vector<float> ma(n), jc(n), va(n);
    relu_mean_var(mz, vz, 0, n, ma, jc, va);
    put(ma, mu_a);
    put(jc, jcb);
    put(va, var_a);
}

void ref_mixture_relu_fwd(const float *mu_z, const float *var_z, int n, int threads,
                          float *mu_a, float *jcb, float *var_a) {
    auto mz = vec(mu_z, n), vz = vec(var_z, n);
    std::vector<float> ma(n), jc(n), va(n);
    if (threads > 1)
        mixture_relu_mean_var_mp(mz, vz, n, threads, ma, jc, va);
    else
        mixture_relu_mean_var(mz, vz, 0, n, ma, jc, va);
    put(ma, mu_a);
    put(jc, jcb);
    put(va, var_a);
}

void ref_batchnorm2d_stats(const float *mu_a, const float *var_a, int wihi, int fi, int B,
                           float momentum, int threads, float *var_s_tmp, float *mu_s,
                           float *var_s, float *mu_ra, float *var_ra) {
    const size_t n = (size_t)B * fi * wihi;
    auto ma = vec(mu_a, n), va = vec(var_a, n);
    std::vector<float> ms(fi), tmp(fi), vs(fi);
    auto mra = vec(mu_ra, fi), vra = vec(var_ra, fi);
    if (threads > 1) {
        batchnorm2d_stat_mean_var_mp(ma, va, wihi, fi, B, threads, ms, tmp);
        batchnorm2d_sample_var_mp(ma, ms, tmp, wihi, fi, B, threads, vs);
        running_mean_var_mp(ms, vs, momentum, fi, threads, mra, vra);
    } else {
        batchnorm2d_stat_mean_var(ma, va, wihi, fi, B, 0, fi, ms, tmp);
        batchnorm2d_sample_var(ma, ms, tmp, wihi, fi, B, 0, fi, vs);
        running_mean_var(ms, vs, momentum, 0, fi, mra, vra);
    }
    put(tmp, var_s_tmp);
    put(ms, mu_s);
    put(vs, var_s);
    put(mra, mu_ra);
    put(vra, var_ra);
}

void ref_batchnorm2d_fwd(const float *mu_w, const float *var_w, const float *mu_b,
                         const float *var_b, const float *mu_a, const float *var_a,
                         const float *mu_norm, const float *var_norm, int bias, float epsilon,
                         int wihi, int fi, int B, int threads, float *mu_z, float *var_z) {
    const size_t n = (size_t)B * fi * wihi;
    auto mw = vec(mu_w, fi), vw = vec(var_w, fi);
    auto mb = vec(bias ? mu_b : nullptr, fi), vb = vec(bias ? var_b : nullptr, fi);
    auto ma = vec(mu_a, n), va = vec(var_a, n), mn = vec(mu_norm, fi), vn = vec(var_norm, fi);
    std::vector<float> mz(n), vz(n);
    if (threads > 1)
        batchnorm2d_fwd_mean_var_mp(mw, vw, mb, vb, ma, va, mn, vn, bias != 0, epsilon, wihi, fi,
                                    B, threads, mz, vz);
    else
        batchnorm2d_fwd_mean_var(mw, vw, mb, vb, ma, va, mn, vn, bias != 0, epsilon, wihi, fi, B,
                                 0, fi * B, mz, vz);
    put(mz, mu_z);
    put(vz, var_z);
}

void ref_batchnorm2d_bwd_dz(const float *mu_w, const float *jcb, const float *var_norm,
                            const float *delta_mu_out, const float *delta_var_out,
                            float epsilon, int wihi, int fi, int B, int threads,
                            float *delta_mu, float *delta_var) {
    const size_t n = (size_t)B * fi * wihi;
    auto mw = vec(mu_w, fi), jc = vec(jcb, n), vn = vec(var_norm, fi);
    auto dm = vec(delta_mu_out, n), dv = vec(delta_var_out, n);
    std::vector<float> om(n), ov(n);
    if (threads > 1)
        batchnorm2d_bwd_delta_z_mp(mw, jc, vn, dm, dv, epsilon, wihi, fi, B, threads, om, ov);
    else
        batchnorm2d_bwd_delta_z(mw, jc, vn, dm, dv, epsilon, wihi, fi, B, 0, fi * B, om, ov);
    put(om, delta_mu);
    put(ov, delta_var);
}

void ref_batchnorm2d_bwd_dw(const float *var_w, const float *var_b, const float *mu_a,
                            const float *mu_norm, const float *var_norm,
                            const float *delta_mu_out, const float *delta_var_out,
                            float epsilon, int wihi, int fi, int B, int bias, int threads,
                            float *tmp_1, float *tmp_2, float *delta_mu_w, float *delta_var_w,
                            float *delta_mu_b, float *delta_var_b) {
    const size_t n = (size_t)B * fi * wihi;
    auto vw = vec(var_w, fi), vb = vec(bias ? var_b : nullptr, fi), ma = vec(mu_a, n);
    auto mn = vec(mu_norm, fi), vn = vec(var_norm, fi);
    auto dm = vec(delta_mu_out, n), dv = vec(delta_var_out, n);
    std::vector<float> t1(n), t2(n), ow(fi), ovw(fi), ob(fi), ovb(fi);
    if (threads > 1)
        batchnorm2d_bwd_delta_w_mp(vw, ma, mn, vn, dm, dv, epsilon, wihi, fi, B, threads, t1, t2);
    else
        batchnorm2d_bwd_delta_w(vw, ma, mn, vn, dm, dv, epsilon, wihi, fi, B, 0, fi * B, t1, t2);
    delta_param_sum(t1, t2, wihi, fi, B, ow, ovw);
    put(ow, delta_mu_w);
    put(ovw, delta_var_w);
    if (!bias) return;
    if (threads > 1)
        batchnorm2d_bwd_delta_b_mp(vb, dm, dv, epsilon, wihi, fi, B, threads, t1, t2);
    else
        batchnorm2d_bwd_delta_b(vb, dm, dv, epsilon, wihi, fi, 0, fi * B, t1, t2);
    delta_param_sum(t1, t2, wihi, fi, B, ob, ovb);
    put(ob, delta_mu_b);
    put(ovb, delta_var_b);
}

int ref_avgpool2d_build_idx(int kernel, int stride, int wi, int hi, int wo, int ho, int pad,
                            int pad_type, int *pool_idx, int *z_ud_idx, int *w, int *h,
                            int *overlap) {
    try {
        Pool2dIndex idx = get_pool_index(kernel, stride, wi, hi, wo, ho, pad, pad_type, -1, -1);
        std::memcpy(pool_idx, idx.pool_idx.data(), idx.pool_idx.size() * sizeof(int));
        std::memcpy(z_ud_idx, idx.z_ud_idx.data(), idx.z_ud_idx.size() * sizeof(int));
        // AvgPool2d::lazy_index_init (src/pooling_layer.cpp:186-210)
        *overlap = !(kernel == stride || kernel == wi);
        *w = idx.z_ud_idx.empty() ? 0 : idx.w;
        *h = idx.z_ud_idx.empty() ? 0 : idx.h;
        return 0;
    } catch (const std::exception &) {
        return -1;
    }
}

void ref_avgpool2d_fwd(const float *mu_a, const float *var_a, const int *pool_idx, int woho,
                       int wihi, int ki, int n_out, int n_in, int overlap, int threads,
                       float *mu_z, float *var_z) {
    auto ma = vec(mu_a, n_in), va = vec(var_a, n_in);
    auto idx = ivec(pool_idx, (size_t)ki * ki * woho);
    std::vector<float> mz(n_out), vz(n_out);
    if (overlap) {
        if (threads > 1)
            avgpool2d_fwd_overlapped_mean_var_mp(ma, va, idx, woho, wihi, ki, n_out, n_in + 1,
                                                 threads, mz, vz);
        else
            avgpool2d_fwd_overlapped_mean_var(ma, va, idx, woho, wihi, ki, n_out, n_in + 1, 0,
                                              n_out, mz, vz);
    } else {
        if (threads > 1)
            avgpool2d_fwd_mean_var_mp(ma, va, idx, woho, wihi, ki, n_out, threads, mz, vz);
        else
            avgpool2d_fwd_mean_var(ma, va, idx, woho, wihi, ki, n_out, 0, n_out, mz, vz);
    }
    put(mz, mu_z);
    put(vz, var_z);
}

void ref_avgpool2d_bwd_dz(const float *jcb, const float *delta_mu_out,
                          const float *delta_var_out, const int *z_ud_idx, int woho, int wihi,
                          int ki, int nr, int wo, int n_in, int n_out, int overlap, int threads,
                          float *delta_mu, float *delta_var) {
    auto jc = vec(jcb, n_in), dm = vec(delta_mu_out, n_out), dv = vec(delta_var_out, n_out);
    std::vector<float> om(n_in), ov(n_in);
    if (overlap) {
        auto idx = ivec(z_ud_idx, (size_t)nr * wihi);
        if (threads > 1)
            avgpool2d_bwd_overlapped_delta_z_mp(jc, dm, dv, idx, woho, wihi, ki, nr, n_in,
                                                n_out + 1, threads, om, ov);
        else
            avgpool2d_bwd_overlapped_delta_z(jc, dm, dv, idx, woho, wihi, ki, nr, n_in,
                                             n_out + 1, 0, n_in, om, ov);
    } else {
        const int nums = n_in / (ki * wo);  // src/pooling_layer.cpp:162-164
        if (threads > 1)
            avgpool2d_bwd_delta_z_mp(jc, dm, dv, wo, ki, nums, threads, om, ov);
        else
            avgpool2d_bwd_delta_z(jc, dm, dv, wo, ki, nums, 0, ki * wo * nums, om, ov);
    }
    put(om, delta_mu);
    put(ov, delta_var);
}

void ref_add_shortcut(const float *mu_s, const float *var_s, int n, float *mu_a, float *var_a) {
    auto ms = vec(mu_s, n), vs = vec(var_s, n), ma = vec(mu_a, n), va = vec(var_a, n);
    add_shortcut_mean_var(ms, vs, n, ma, va);
    put(ma, mu_a);
    put(va, var_a);
}

void ref_add_shortcut_delta(const float *mu_s, const float *var_s, const float *jcb_s, int n,
                            float *mu_a, float *var_a) {
    auto ms = vec(mu_s, n), vs = vec(var_s, n), js = vec(jcb_s, n);
    auto ma = vec(mu_a, n), va = vec(var_a, n);
    add_shortcut_delta(ms, vs, js, n, ma, va);
    put(ma, mu_a);
    put(va, var_a);
}

// Hierarchical-softmax label encoding (src/cost.cpp:76-143). obs and idx hold
// n_classes * ceil(log2(n_classes)) entries.
void ref_class_to_obs(int n_classes, float *obs, int *idx, int *n_obs, int *len) {
    HRCSoftmax hs = class_to_obs(n_classes);
    std::memcpy(obs, hs.obs.data(), hs.obs.size() * sizeof(float));
    std::memcpy(idx, hs.idx.data(), hs.idx.size() * sizeof(int));
    *n_obs = (int)hs.n_obs;
    *len = (int)hs.len;
}

// ---- checkpoint files ---------------------------------------------------------
// Two small models built from the reference's own layer classes, sized the way
// Sequential::compute_input_output_size does it (src/sequential.cpp:144-164), to
// write and read the reference's binary checkpoint (BaseLayer::save/load,
// src/base_layer.cpp:230-297; BatchNorm2d adds its running averages,
// src/batchnorm_layer.cpp:1143-1230; blocks save their members in order,
// src/layer_block.cpp, src/resnet_block.cpp:299-317).
//   model 0: Linear(13,7) ReLU Linear(7,3)
//   model 1: Conv2d(3,4,k3,p1) BatchNorm2d(4) MixtureReLU
//            ResNetBlock(main: Conv2d(4,8,k3,s2,p1 type 2) ReLU BatchNorm2d(8);
//                        shortcut: Conv2d(4,8,k2,s2)) AvgPool2d(4) Linear(8,5)
}  // extern "C"

namespace {
struct Zoo {
    std::vector<std::shared_ptr<BaseLayer>> top;
    std::vector<BaseLayer *> leaves;  // in the order their parameters are saved
};

Zoo make_zoo(int model) {
    Zoo z;
    auto leaf = [&](std::shared_ptr<BaseLayer> l) {
        z.leaves.push_back(l.get());
        return l;
    };
    if (model == 0) {
        z.top.push_back(leaf(std::make_shared<Linear>(13, 7)));
        z.top.push_back(leaf(std::make_shared<ReLU>()));
        z.top.push_back(leaf(std::make_shared<Linear>(7, 3)));
    } else {
        z.top.push_back(leaf(std::make_shared<Conv2d>(3, 4, 3, false, 1, 1, 1, 8, 8)));
        z.top.push_back(leaf(std::make_shared<BatchNorm2d>(4)));
        z.top.push_back(leaf(std::make_shared<MixtureReLU>()));
        auto main = std::make_shared<LayerBlock>();
        main->add_layer(leaf(std::make_shared<Conv2d>(4, 8, 3, false, 2, 1, 2)));
        main->add_layer(leaf(std::make_shared<ReLU>()));
        main->add_layer(leaf(std::make_shared<BatchNorm2d>(8)));
        auto shortcut = std::make_shared<LayerBlock>();
        shortcut->add_layer(leaf(std::make_shared<Conv2d>(4, 8, 2, false, 2)));
        z.top.push_back(std::make_shared<ResNetBlock>(main, shortcut));
        z.top.push_back(leaf(std::make_shared<AvgPool2d>(4)));
        z.top.push_back(leaf(std::make_shared<Linear>(8, 5)));
    }
    int w = z.top.front()->in_width, h = z.top.front()->in_height,
        d = z.top.front()->in_channels;
    for (auto &l : z.top) {
        InitArgs args(w, h, d);
        l->compute_input_output_size(args);
        w = l->out_width;
        h = l->out_height;
        d = l->out_channels;
    }
    for (auto &l : z.top) l->preinit_layer();
    return z;
}

std::vector<std::vector<float> *> arrays_of(BaseLayer *l) {
    std::vector<std::vector<float> *> a = {&l->mu_w, &l->var_w, &l->mu_b, &l->var_b};
    if (auto *bn = dynamic_cast<BatchNorm2d *>(l)) {
        a.push_back(&bn->mu_ra);
        a.push_back(&bn->var_ra);
    }
    return a;
}
}  // namespace

extern "C" {

// Fills every parameter of the model with value(leaf, array, i) =
// (leaf + 1) + 0.1 * (array + 1) + 1e-4 * i and saves it. Returns the number of
// floats written, -1 on failure.
int ref_checkpoint_save(int model, const char *path) {
    try {
        Zoo z = make_zoo(model);
        int total = 0;
        for (size_t L = 0; L < z.leaves.size(); L++) {
            auto arrs = arrays_of(z.leaves[L]);
            for (size_t a = 0; a < arrs.size(); a++)
                for (size_t i = 0; i < arrs[a]->size(); i++, total++)
                    (*arrs[a])[i] = (float)(L + 1) + 0.1f * (float)(a + 1) + 1e-4f * (float)i;
        }
        std::ofstream file(path, std::ios::binary);
        if (!file.is_open()) return -1;
        for (auto &l : z.top) l->save(file);
        return total;
    } catch (const std::exception &) {
        return -1;
    }
}

// Loads a checkpoint into a freshly built model and writes its parameters, leaf
// by leaf in saving order, to out. Returns the number of floats, -1 on failure
// (a layer name that does not match throws in the reference).
int ref_checkpoint_load(int model, const char *path, float *out, int capacity) {
    try {
        Zoo z = make_zoo(model);
        std::ifstream file(path, std::ios::binary);
        if (!file.is_open()) return -1;
        for (auto &l : z.top) l->load(file);
        int n = 0;
        for (auto *l : z.leaves)
            for (auto *arr : arrays_of(l))
                for (float v : *arr) {
                    if (n >= capacity) return -1;
                    out[n++] = v;
                }
        return n;
    } catch (const std::exception &) {
        return -1;
    }
}

// Classification error and class probabilities from the output layer's moments
// (src/cost.cpp:195-246 over obs_to_class, 150-190). er: [B], prob: [B][n_classes].
void ref_get_error(const float *mz, const float *Sz, const int *labels, int n_classes, int B,
                   int len, int *er, float *prob) {
    std::vector<float> m(mz, mz + (size_t)B * len), S(Sz, Sz + (size_t)B * len);
    std::vector<int> l(labels, labels + B);
    std::vector<int> e;
    std::vector<float> P;
    std::tie(e, P) = get_error(m, S, l, n_classes, B);
    std::memcpy(er, e.data(), e.size() * sizeof(int));
    std::memcpy(prob, P.data(), P.size() * sizeof(float));
}

// The text format of Sequential::save_csv / load_csv (src/sequential.cpp:612-709):
// one value per line through write_csv / read_csv (include/common.h:135-207).
int ref_write_csv(const char *path, const float *data, int n) {
    try {
        std::vector<float> v(data, data + n);
        write_csv(std::string(path), v);
        return 0;
    } catch (const std::exception &) {
        return -1;
    }
}

int ref_read_csv(const char *path, float *out, int n) {
    try {
        std::vector<float> v(n);
        std::string name(path);
        read_csv(name, v, 1, false);
        std::memcpy(out, v.data(), n * sizeof(float));
        return 0;
    } catch (const std::exception &) {
        return -1;
    }
}

}  // extern "C"

// CPU oracle for the TAGI Linear / Conv2d hot path: see tagi_oracle.h.
// TEST INFRASTRUCTURE ONLY: the checker in tests, the smoke test and the
// benchmark's CPU baseline. The shipped library never links or loads it.
//
// Build with the reference's flags (-O3, x86-64 baseline, no fast-math) so the
// fp32 results equal the compiled reference bit for bit: no fused multiply-add
// exists on the baseline ISA and nothing here lets the compiler reassociate.
#include "tagi_oracle.h"

#include <algorithm>
#include <cmath>
#include <thread>
#include <utility>
#include <vector>

namespace {

// Thread fan-out of the reference's `_mp` wrappers (e.g.
// src/linear_layer.cpp:72-98): `total` flat output indices, contiguous chunks,
// the first `total % threads` chunks one longer; fresh threads per call.
template <typename Body>
void fan_out(int total, int threads, Body body) {
    if (threads <= 1) {
        body(0, total);
        return;
    }
    std::vector<std::thread> pool;
    pool.reserve(threads);
    const int per = total / threads;
    const int extra = total % threads;
    for (int t = 0; t < threads; t++) {
        const int lo = t * per + std::min(t, extra);
        const int hi = lo + per + (t < extra ? 1 : 0);
        pool.emplace_back([=] { body(lo, hi); });
    }
    for (auto &th : pool) th.join();
}

}  // namespace

extern "C" {

// ---------------------------------------------------------------------------
// Linear
// ---------------------------------------------------------------------------

// src/linear_layer.cpp:10-61: flat index i -> row = i / B (output unit),
// col = i % B (sample); serial dot of length K; bias added after the sum.
void oracle_linear_fwd(const float *mu_w, const float *var_w,
                       const float *mu_b, const float *var_b,
                       const float *mu_a, const float *var_a, int K, int N,
                       int B, int bias, int threads, float *mu_z,
                       float *var_z) {
    fan_out(N * B, threads, [=](int lo, int hi) {
        for (int i = lo; i < hi; i++) {
            const int row = i / B, col = i % B;
            float s_mu = 0.0f, s_var = 0.0f;
            for (int j = 0; j < K; j++) {
                const float ma = mu_a[K * col + j];
                const float va = var_a[K * col + j];
                const float mw = mu_w[row * K + j];
                const float vw = var_w[row * K + j];
                s_mu += mw * ma;
                s_var += (mw * mw + vw) * va + vw * ma * ma;
            }
            if (bias) {
                mu_z[col * N + row] = s_mu + mu_b[row];
                var_z[col * N + row] = s_var + var_b[row];
            } else {
                mu_z[col * N + row] = s_mu;
                var_z[col * N + row] = s_var;
            }
        }
    });
}

// src/linear_layer.cpp:245-273: flat j -> row = j / B (input unit), col = j % B;
// walks column `row` of mu_w; variance term ordered w * dvar * w.
void oracle_linear_bwd_dz(const float *mu_w, const float *jcb,
                          const float *delta_mu, const float *delta_var, int K,
                          int N, int B, int threads, float *delta_mu_z,
                          float *delta_var_z) {
    fan_out(K * B, threads, [=](int lo, int hi) {
        for (int j = lo; j < hi; j++) {
            const int row = j / B, col = j % B;
            float s_mu = 0.0f, s_var = 0.0f;
            for (int i = 0; i < N; i++) {
                const float w = mu_w[K * i + row];
                s_mu += w * delta_mu[col * N + i];
                s_var += w * delta_var[col * N + i] * w;
            }
            const float jc = jcb[col * K + row];
            delta_mu_z[col * K + row] = s_mu * jc;
            delta_var_z[col * K + row] = s_var * jc * jc;
        }
    });
}

// src/linear_layer.cpp:314-350: flat j -> row = j / N (input unit),
// col = j % N (output unit); reduction over the batch; scaled by var_w, var_w^2.
void oracle_linear_bwd_dw(const float *var_w, const float *mu_a,
                          const float *delta_mu, const float *delta_var, int K,
                          int N, int B, int threads, float *delta_mu_w,
                          float *delta_var_w) {
    fan_out(K * N, threads, [=](int lo, int hi) {
        for (int j = lo; j < hi; j++) {
            const int row = j / N, col = j % N;
            float s_mu = 0.0f, s_var = 0.0f;
            for (int i = 0; i < B; i++) {
                const float a = mu_a[K * i + row];
                s_mu += a * delta_mu[col + N * i];
                s_var += a * a * delta_var[col + N * i];
            }
            const float v = var_w[col * K + row];
            delta_mu_w[col * K + row] = s_mu * v;
            delta_var_w[col * K + row] = s_var * v * v;
        }
    });
}

// src/linear_layer.cpp:391-424; the _mp wrapper (426-459) chunks over N.
void oracle_linear_bwd_db(const float *var_b, const float *delta_mu,
                          const float *delta_var, int N, int B, int threads,
                          float *delta_mu_b, float *delta_var_b) {
    fan_out(N, threads, [=](int lo, int hi) {
        for (int row = lo; row < hi; row++) {
            float s_mu = 0.0f, s_var = 0.0f;
            for (int i = 0; i < B; i++) {
                s_mu += delta_mu[N * i + row];
                s_var += delta_var[N * i + row];
            }
            delta_mu_b[row] = s_mu * var_b[row];
            delta_var_b[row] = s_var * var_b[row] * var_b[row];
        }
    });
}

// ---------------------------------------------------------------------------
// Conv2d index tables
// ---------------------------------------------------------------------------

// src/conv2d_layer.cpp:581-628
int oracle_conv2d_out_size(int kernel, int stride, int wi, int hi, int pad,
                           int pad_type, int *wo, int *ho) {
    int nom_w, nom_h;
    if (pad_type == 1) {
        nom_w = wi - kernel + 2 * pad;
        nom_h = hi - kernel + 2 * pad;
    } else if (pad_type == 2) {
        nom_w = wi - kernel + pad;
        nom_h = hi - kernel + pad;
    } else {
        nom_w = wi - kernel;
        nom_h = hi - kernel;
    }
    if (nom_w % stride != 0 || nom_h % stride != 0) return -1;
    *wo = nom_w / stride + 1;
    *ho = nom_h / stride + 1;
    return 0;
}

namespace {

// src/indices.cpp:349-378: argsort through (value, position) pairs, so equal
// values keep their original order.
std::vector<int> argsort(const std::vector<int> &v) {
    std::vector<std::pair<int, int>> pv(v.size());
    for (size_t i = 0; i < v.size(); i++) pv[i] = {v[i], (int)i};
    std::sort(pv.begin(), pv.end());
    std::vector<int> out(v.size());
    for (size_t i = 0; i < v.size(); i++) out[i] = pv[i].second;
    return out;
}

// src/indices.cpp:514-542 fed by 544-590: drop the padded positions of `full`,
// reorder by `ref`, then pour row by row into the cells of `base` that are set.
std::vector<int> pour_into_base(const std::vector<int> &full,
                                const std::vector<int> &pad_pos, int pad,
                                const std::vector<int> &ref,
                                const std::vector<int> &base, int fill, int w,
                                int h, bool *ok) {
    std::vector<int> kept(full);
    if (pad > 0) {
        for (int p : pad_pos) kept[p] = -1;
        kept.erase(std::remove(kept.begin(), kept.end(), -1), kept.end());
    }
    if (kept.size() != ref.size()) {
        *ok = false;
        return {};
    }
    std::vector<int> out((size_t)w * h);
    size_t next = 0;
    for (int r = 0; r < h; r++)
        for (int c = 0; c < w; c++)
            out[(size_t)r * w + c] =
                base[(size_t)r * w + c] == 1 ? kept[ref[next++]] : fill;
    return out;
}

}  // namespace

int oracle_conv2d_build_idx(int kernel, int stride, int wi, int hi, int wo,
                            int ho, int pad, int pad_type, int param_pad_idx,
                            int *Fmwa_2_out, int *FCzwa_1_out, int *Szz_ud_out,
                            int *w_out, int *h_out) {
    // The reference pads rows and columns with the same bounds
    // (src/indices.cpp:55-59) and sizes the layer as in_width * in_width
    // (src/conv2d_layer.cpp:63): square images only.
    if (wi != hi) return -2;
    const int pad_idx = -1;  // src/conv2d_layer.cpp:104-107
    const int k2 = kernel * kernel;

    // src/indices.cpp:63-103: geometry of the padded image
    int w_p = wi, h_p = hi, start = 0, end = 0, offset = 0;
    if (pad > 0) {
        if (pad_type == 1) {
            start = pad; end = wi + pad; offset = pad;
            w_p = wi + 2 * pad; h_p = hi + 2 * pad;
        } else if (pad_type == 2) {
            start = 0; end = wi; offset = 0;
            w_p = wi + pad; h_p = hi + pad;
        } else {
            return -3;  // the reference leaves the sizes unset here
        }
    }
    // src/indices.cpp:10-61,105-137: 1-based pixel ids, padding = pad_idx
    std::vector<int> padded((size_t)w_p * h_p);
    if (pad > 0) {
        std::fill(padded.begin(), padded.end(), pad_idx);
        for (int r = start; r < end; r++)
            for (int c = start; c < end; c++)
                padded[(size_t)r * w_p + c] = (r - offset) * wi + (c - offset) + 1;
    } else {
        for (int i = 0; i < w_p * h_p; i++) padded[i] = i + 1;
    }

    // src/indices.cpp:224-262: receptive fields, first kernel window shifted by
    // the stride along the row, then whole rows shifted down.
    if ((h_p - kernel) / stride + 1 != wo && kernel != 1) return -4;
    std::vector<int> first(k2);
    for (int r = 0; r < kernel; r++)
        for (int c = 0; c < kernel; c++) first[r * kernel + c] = r * w_p + c + 1;
    std::vector<int> field((size_t)wo * ho * k2);
    for (int ox = 0; ox < wo; ox++)
        for (int t = 0; t < k2; t++) field[(size_t)ox * k2 + t] = first[t] + ox * stride;
    for (int oy = 1; oy < ho; oy++)
        for (int c = 0; c < k2 * wo; c++)
            field[(size_t)oy * k2 * wo + c] = field[c] + oy * stride * w_p;
    std::vector<int> M(field.size());
    for (size_t i = 0; i < field.size(); i++) M[i] = padded[field[i] - 1];

    // src/indices.cpp:267-315,443-464: distinct pixels, how often each occurs,
    // and the binary occupancy matrix [h][w]
    std::vector<int> uM(M);
    std::sort(uM.begin(), uM.end());
    uM.erase(std::unique(uM.begin(), uM.end()), uM.end());
    uM.erase(std::remove(uM.begin(), uM.end(), pad_idx), uM.end());
    if (uM.empty()) return -5;
    const int w = (int)uM.size();
    std::vector<int> freq(w);
    for (int i = 0; i < w; i++) freq[i] = (int)std::count(M.begin(), M.end(), uM[i]);
    const int h = *std::max_element(freq.begin(), freq.end());
    std::vector<int> base((size_t)w * h, 0);
    for (int r = 0; r < w; r++)
        for (int c = 0; c < freq[r]; c++) base[(size_t)c * w + r] = 1;

    // src/indices.cpp:320-347: pixel id of every set cell, row-major
    std::vector<int> ordered;
    for (int r = 0; r < h; r++)
        for (int c = 0; c < w; c++)
            if (base[(size_t)r * w + c] * uM[c] != 0) ordered.push_back(uM[c]);

    // src/indices.cpp:390-441: rank of every cell among the sorted cells,
    // mapped onto the sorted positions of the un-padded receptive field
    std::vector<int> rank = argsort(argsort(ordered));
    std::vector<int> pad_pos, sorted_field;
    if (pad > 0) {
        std::vector<int> no_pad(M);
        no_pad.erase(std::remove(no_pad.begin(), no_pad.end(), pad_idx), no_pad.end());
        sorted_field = argsort(no_pad);
        for (size_t i = 0; i < M.size(); i++)
            if (M[i] == pad_idx) pad_pos.push_back((int)i);
    } else {
        sorted_field = argsort(M);
    }
    if (sorted_field.size() != rank.size()) return -6;
    std::vector<int> ref(rank.size());
    for (size_t i = 0; i < rank.size(); i++) ref[i] = sorted_field[rank[i]];

    // src/indices.cpp:592-623: kernel-tap ids, one row of 1..k2 per output pixel
    std::vector<int> taps((size_t)wo * ho * k2);
    for (int o = 0; o < wo * ho; o++)
        for (int t = 0; t < k2; t++) taps[(size_t)o * k2 + t] = t + 1;
    // src/indices.cpp:669-696: output-pixel ids, each repeated k2 times
    std::vector<int> outs((size_t)wo * ho * k2);
    for (int o = 0; o < wo * ho; o++)
        for (int t = 0; t < k2; t++) outs[(size_t)o * k2 + t] = o + 1;

    bool ok = true;
    std::vector<int> zw = pour_into_base(taps, pad_pos, pad, ref, base, param_pad_idx, w, h, &ok);
    std::vector<int> zud = pour_into_base(outs, pad_pos, pad, ref, base, -1, w, h, &ok);
    if (!ok) return -7;

    for (size_t i = 0; i < M.size(); i++) Fmwa_2_out[i] = M[i];
    // src/common.cpp:36-55: FCzwa_1 is handed out transposed, [w][h]
    for (int r = 0; r < h; r++)
        for (int c = 0; c < w; c++) FCzwa_1_out[r + (size_t)c * h] = zw[c + (size_t)r * w];
    for (size_t i = 0; i < zud.size(); i++) Szz_ud_out[i] = zud[i];
    *w_out = w;
    *h_out = h;
    return 0;
}

// ---------------------------------------------------------------------------
// Conv2d
// ---------------------------------------------------------------------------

// src/conv2d_layer.cpp:274-323
void oracle_conv2d_fwd(const float *mu_w, const float *var_w,
                       const float *mu_b, const float *var_b,
                       const float *mu_a, const float *var_a, const int *aidx,
                       int woho, int fo, int wihi, int fi, int ki, int B,
                       int bias, int threads, float *mu_z, float *var_z) {
    const int ki2 = ki * ki;
    const int n = ki2 * fi;
    fan_out(woho * B * fo, threads, [=](int lo, int hi) {
        for (int j = lo; j < hi; j++) {
            const int row = j / (woho * B);
            const int col = j % (woho * B);
            float s_mu = 0, s_var = 0;
            for (int i = 0; i < n; i++) {
                int a = aidx[(col % woho) * ki2 + i % ki2];
                if (a > -1) {
                    a += (i / ki2) * wihi + (col / woho) * wihi * fi;
                    const float ma = mu_a[a - 1];
                    const float va = var_a[a - 1];
                    const float mw = mu_w[row * n + i];
                    const float vw = var_w[row * n + i];
                    s_mu += mw * ma;
                    s_var += (mw * mw + vw) * va + vw * ma * ma;
                }
            }
            const int out = woho * (col / woho) * fo + col % woho + row * woho;
            if (bias) {
                mu_z[out] = s_mu + mu_b[row];
                var_z[out] = s_var + var_b[row];
            } else {
                mu_z[out] = s_mu;
                var_z[out] = s_var;
            }
        }
    });
}

// src/conv2d_layer.cpp:444-457 then 363-404
void oracle_conv2d_bwd_dz(const float *mu_w, const float *jcb,
                          const float *delta_mu_out,
                          const float *delta_var_out, const int *zw_idx,
                          const int *zud_idx, int woho, int fo, int wihi,
                          int fi, int ki, int nr, int B, int threads,
                          float *tmp, float *delta_mu, float *delta_var) {
    // permute_jacobian: [B][fi][wihi] -> [fi][B][wihi]
    for (int col = 0; col < wihi * fi; col++)
        for (int row = 0; row < B; row++)
            tmp[wihi * (col / wihi) * B + col % wihi + row * wihi] =
                jcb[row * wihi * fi + col];

    const int k = wihi * B;
    const int ki2 = ki * ki;
    const int n = nr * fo;
    const float *jp = tmp;
    fan_out(wihi * B * fi, threads, [=](int lo, int hi) {
        for (int j = lo; j < hi; j++) {
            const int row = j / k, col = j % k;
            float s_mu = 0.0f, s_var = 0.0f;
            for (int i = 0; i < n; i++) {
                const int wid = zw_idx[(col % wihi) * nr + i % nr] +
                                (i / nr) * ki2 * fi + row * ki2 - 1;
                int a = zud_idx[col % wihi + wihi * (i % nr)];
                if (a > -1) {
                    a += (i / nr) * woho + (col / wihi) * woho * fo;
                    const float w = mu_w[wid];
                    s_mu += delta_mu_out[a - 1] * w;
                    s_var += w * delta_var_out[a - 1] * w;
                }
            }
            const int out = wihi * (col / wihi) * fi + col % wihi + row * wihi;
            delta_mu[out] = s_mu * jp[row * k + col];
            delta_var[out] = s_var * jp[row * k + col] * jp[row * k + col];
        }
    });
}

// src/conv2d_layer.cpp:558-575, 459-495, 538-556
void oracle_conv2d_bwd_dw(const float *var_w, const float *var_b,
                          const float *mu_a, const float *delta_mu_out,
                          const float *delta_var_out, const int *aidx, int B,
                          int fo, int woho, int wihi, int fi, int ki, int bias,
                          int threads, float *tmp_1, float *tmp_2,
                          float *delta_mu_w, float *delta_var_w,
                          float *delta_mu_b, float *delta_var_b) {
    // permute_delta: [B][fo][woho] -> [fo][B][woho]
    const int kp = woho * fo;
    for (int col = 0; col < kp; col++)
        for (int row = 0; row < B; row++) {
            const int dst = woho * (col / woho) * B + col % woho + row * woho;
            tmp_1[dst] = delta_mu_out[row * kp + col];
            tmp_2[dst] = delta_var_out[row * kp + col];
        }

    const int ki2 = ki * ki;
    const int m = ki2 * fi;
    const int n = woho * B;
    const float *dm = tmp_1, *dv = tmp_2;
    fan_out(ki2 * fi * fo, threads, [=](int lo, int hi) {
        for (int j = lo; j < hi; j++) {
            const int row = j / fo, col = j % fo;
            float s_mu = 0.0f, s_var = 0.0f;
            for (int i = 0; i < n; i++) {
                int a = aidx[ki2 * (i % woho) + row % ki2];
                if (a > -1) {
                    a += (row / ki2) * wihi + (i / woho) * wihi * fi;
                    const float ma = mu_a[a - 1];
                    s_mu += ma * dm[col * n + i];
                    s_var += ma * dv[col * n + i] * ma;
                }
            }
            const float v = var_w[col * m + row];
            delta_mu_w[col * m + row] = s_mu * v;
            delta_var_w[col * m + row] = s_var * v * v;
        }
    });

    if (bias) {
        for (int col = 0; col < fo; col++) {
            float s_mu = 0.0f, s_var = 0.0f;
            for (int i = 0; i < n; i++) {
                s_mu += dm[col * n + i];
                s_var += dv[col * n + i];
            }
            delta_mu_b[col] = s_mu * var_b[col];
            delta_var_b[col] = s_var * var_b[col] * var_b[col];
        }
    }
}

// ---------------------------------------------------------------------------
// Parameter update
// ---------------------------------------------------------------------------

// src/base_layer.cpp:164-187
float oracle_cap_factor(int batch_size, float prev) {
    float cap = prev;
    if (batch_size == 1) cap = 0.1f;
    if (batch_size > 1 && batch_size < 256) cap = 2.0f;
    if (batch_size >= 256) cap = 3.0f;
    return cap;
}

// src/base_layer.cpp:116-137 (139-162 for biases: same arithmetic)
int oracle_param_update(float *mu, float *var, const float *delta_mu,
                        const float *delta_var, size_t n, float cap_factor) {
    int clamped = 0;
    for (size_t i = 0; i < n; i++) {
        const float sign_mu = (delta_mu[i] > 0) - (delta_mu[i] < 0);
        const float sign_var = (delta_var[i] > 0) - (delta_var[i] < 0);
        const float bar = powf(var[i], 0.5) / cap_factor;
        mu[i] += sign_mu * std::min(std::abs(delta_mu[i]), bar);
        var[i] += sign_var * std::min(std::abs(delta_var[i]), bar);
        if (var[i] <= 0.0f) {
            var[i] = 1E-5f;
            clamped++;
        }
    }
    return clamped;
}

// ---------------------------------------------------------------------------
// Output updater
// ---------------------------------------------------------------------------

// src/base_output_updater.cpp:8-29
void oracle_out_update_dense(const float *mu_a, const float *var_a,
                             const float *jcb, const float *obs,
                             const float *var_obs, int n, float *delta_mu,
                             float *delta_var) {
    for (int col = 0; col < n; col++) {
        const float t = jcb[col] / (var_a[col] + var_obs[col]);
        if (std::isinf(t) || std::isnan(t) || std::isnan(obs[col])) {
            delta_mu[col] = 0.0f;
            delta_var[col] = 0.0f;
        } else {
            delta_mu[col] = t * (obs[col] - mu_a[col]);
            delta_var[col] = -t * jcb[col];
        }
    }
}

// src/base_output_updater.cpp:131-226. The output layer holds pairs: the mean
// output at 2i and the (positive) error variance V2_bar_tilde at 2i+1; n counts
// observations. The observation updates the mean output with the expected error
// variance as observation noise, and the error-variance unit through the Gaussian
// moments of V (posterior of the error) and V^2.
void oracle_out_update_heteros(const float *mu_a, const float *var_a, const float *jcb,
                               const float *obs, int n, float *delta_mu, float *delta_var) {
    for (int i = 0; i < n; i++) {
        const int col = 2 * i;
        const float var_y = var_a[col], mu_y = mu_a[col], jcb_y = jcb[col];
        const float mu_v2b = mu_a[col + 1], var_v2b = var_a[col + 1], cov_v2b = jcb[col + 1];
        const float mu_v2 = mu_v2b;
        const float var_v2 = 3.0f * var_v2b + 2.0f * mu_v2b * mu_v2b;
        const float cov_y_v = mu_v2;
        const float var_sum = var_y + mu_v2;
        const float t = jcb_y / var_sum;
        const float y = obs[i];
        const bool bad_obs = std::isinf(y) || std::isnan(y);
        if (std::isinf(t) || std::isnan(t) || bad_obs) {
            delta_mu[col] = 0.0f;
            delta_var[col] = 0.0f;
        } else {
            delta_mu[col] = t * (y - mu_y);
            delta_var[col] = -t * jcb_y;
        }
        if (bad_obs) {
            delta_mu[col + 1] = 0.0f;
            delta_var[col + 1] = 0.0f;
        } else {
            const float mu_v_pos = cov_y_v / var_sum * (y - mu_y);
            const float var_v_pos = mu_v2 - cov_y_v / var_sum * cov_y_v;
            const float mu_v2_pos = mu_v_pos * mu_v_pos + var_v_pos;
            const float var_v2_pos =
                2.0f * var_v_pos * var_v_pos + 4.0f * var_v_pos * mu_v_pos * mu_v_pos;
            const float k = var_v2b / var_v2;
            const float mu_v2b_pos = mu_v2b + k * (mu_v2_pos - mu_v2);
            const float var_v2b_pos = var_v2b + k * k * (var_v2_pos - var_v2);
            float jv = cov_v2b / var_v2b;
            if (std::isinf(jv) || std::isnan(jv)) jv = 0.0f;
            delta_mu[col + 1] = jv * (mu_v2b_pos - mu_v2b);
            delta_var[col + 1] = jv * jv * (var_v2b_pos - var_v2b);
        }
    }
}

// src/base_output_updater.cpp:67-93
void oracle_out_update_indexed(const float *mu_a, const float *var_a,
                               const float *jcb, const float *obs,
                               const float *var_obs, const int *selected_idx,
                               int n_obs, int n_enc, int n, float *delta_mu,
                               float *delta_var) {
    for (int col = 0; col < n; col++) {
        const int idx = selected_idx[col] + (col / n_enc) * n_obs - 1;
        const float t = jcb[idx] / (var_a[idx] + var_obs[col]);
        if (std::isinf(t) || std::isnan(t)) {
            delta_mu[idx] = 0.0f;
            delta_var[idx] = 0.0f;
        } else {
            delta_mu[idx] = t * (obs[col] - mu_a[idx]);
            delta_var[idx] = -t * jcb[idx];
        }
    }
}

// ---------------------------------------------------------------------------
// ReLU
// ---------------------------------------------------------------------------

// src/activation.cpp:7-29
void oracle_relu_fwd(const float *mu_z, const float *var_z, int n, float *mu_a,
                     float *jcb, float *var_a) {
    for (int col = 0; col < n; col++) {
        const float t = std::max(mu_z[col], 0.0f);
        mu_a[col] = t;
        if (t == 0) {
            jcb[col] = 0.0f;
            var_a[col] = 0.0f;
        } else {
            jcb[col] = 1.0f;
            var_a[col] = var_z[col];
        }
    }
}

// ---------------------------------------------------------------------------
// MixtureReLU
// ---------------------------------------------------------------------------

// src/activation.cpp:152-178; normcdf_cpu is src/common.cpp:315-319.
void oracle_mixture_relu_fwd(const float *mu_z, const float *var_z, int n,
                             int threads, float *mu_a, float *jcb,
                             float *var_a) {
    fan_out(n, threads, [=](int lo, int hi) {
        constexpr float SQRT_2PI = 2.5066282746310002f;
        for (int i = lo; i < hi; i++) {
            const float m = mu_z[i];
            const float sd = powf(var_z[i], 0.5);
            const float alpha = m / sd;
            const float pdf = (1.0f / SQRT_2PI) * expf(-0.5f * alpha * alpha);
            const float cdf = 0.5f * erfcf(-alpha * 0.7071067811865475f);
            const float t = m * cdf + sd * pdf;
            mu_a[i] = fmaxf(0.000001f, t);
            var_a[i] = fmaxf(0.000001f, -t * t + 2 * t * m - m * sd * pdf +
                                            (var_z[i] - m * m) * cdf);
            jcb[i] = cdf;
        }
    });
}

// ---------------------------------------------------------------------------
// BatchNorm2d
// ---------------------------------------------------------------------------

void oracle_batchnorm2d_stats(const float *mu_a, const float *var_a, int wihi,
                              int fi, int B, float momentum, int threads,
                              float *var_s_tmp, float *mu_s, float *var_s,
                              float *mu_ra, float *var_ra) {
    // src/batchnorm_layer.cpp:127-147
    fan_out(fi, threads, [=](int lo, int hi) {
        for (int col = lo; col < hi; col++) {
            float sum_mu = 0, sum_var = 0;
            for (int i = 0; i < wihi * B; i++) {
                const int at = (i / wihi) * wihi * fi + i % wihi + col * wihi;
                sum_mu += mu_a[at];
                sum_var += var_a[at];
            }
            mu_s[col] = sum_mu / (wihi * B);
            var_s_tmp[col] = sum_var;
        }
    });
    // src/batchnorm_layer.cpp:149-168
    fan_out(fi, threads, [=](int lo, int hi) {
        for (int col = lo; col < hi; col++) {
            float sum = 0;
            for (int i = 0; i < wihi * B; i++) {
                const int at = (i / wihi) * wihi * fi + i % wihi + col * wihi;
                sum += (mu_a[at] - mu_s[col]) * (mu_a[at] - mu_s[col]);
            }
            var_s[col] = (sum + var_s_tmp[col]) / (wihi * B - 1);
        }
    });
    // src/batchnorm_layer.cpp:15-26
    fan_out(fi, threads, [=](int lo, int hi) {
        for (int col = lo; col < hi; col++) {
            mu_ra[col] = mu_ra[col] * momentum + mu_s[col] * (1 - momentum);
            var_ra[col] = var_ra[col] * momentum + var_s[col] * (1 - momentum);
        }
    });
}

// src/batchnorm_layer.cpp:170-206: rows are (sample, channel) pairs
void oracle_batchnorm2d_fwd(const float *mu_w, const float *var_w,
                            const float *mu_b, const float *var_b,
                            const float *mu_a, const float *var_a,
                            const float *mu_norm, const float *var_norm,
                            int bias, float epsilon, int wihi, int fi, int B,
                            int threads, float *mu_z, float *var_z) {
    fan_out(fi * B, threads, [=](int lo, int hi) {
        for (int row = lo; row < hi; row++) {
            const float inv = 1.0f / std::sqrt(var_norm[row % fi] + epsilon);
            const float mra = mu_norm[row % fi];
            const float mw = mu_w[row % fi];
            for (int col = 0; col < wihi; col++) {
                const int at = col + row * wihi;
                const float d = mu_a[at] - mra;
                mu_z[at] = inv * d * mw;
                var_z[at] = inv * inv * (var_a[at] * (mw * mw + var_w[row % fi]) +
                                         var_w[row % fi] * d * d);
                if (bias) {
                    mu_z[at] += mu_b[row % fi];
                    var_z[at] += var_b[row % fi];
                }
            }
        }
    });
}

// src/batchnorm_layer.cpp:233-255
void oracle_batchnorm2d_bwd_dz(const float *mu_w, const float *jcb,
                               const float *var_norm, const float *delta_mu_out,
                               const float *delta_var_out, float epsilon,
                               int wihi, int fi, int B, int threads,
                               float *delta_mu, float *delta_var) {
    fan_out(fi * B, threads, [=](int lo, int hi) {
        for (int row = lo; row < hi; row++) {
            const float inv = 1.0f / std::sqrt(var_norm[row % fi] + epsilon);
            for (int col = 0; col < wihi; col++) {
                const int at = col + row * wihi;
                const float tmp = inv * mu_w[row % fi] * jcb[at];
                delta_mu[at] = tmp * delta_mu_out[at];
                delta_var[at] = tmp * delta_var_out[at] * tmp;
            }
        }
    });
}

namespace {
// src/common.cpp:360-378 (single-threaded in the reference)
void param_sum(const float *e_mu, const float *e_var, int wihi, int fi, int B,
               float *out_mu, float *out_var) {
    for (int col = 0; col < fi; col++) {
        float s_mu = 0.0f, s_var = 0.0f;
        for (int i = 0; i < wihi * B; i++) {
            const int at = (i / wihi) * wihi * fi + i % wihi + col * wihi;
            s_mu += e_mu[at];
            s_var += e_var[at];
        }
        out_mu[col] = s_mu;
        out_var[col] = s_var;
    }
}
}  // namespace

void oracle_batchnorm2d_bwd_dw(const float *var_w, const float *var_b,
                               const float *mu_a, const float *mu_norm,
                               const float *var_norm, const float *delta_mu_out,
                               const float *delta_var_out, float epsilon,
                               int wihi, int fi, int B, int bias, int threads,
                               float *tmp_1, float *tmp_2, float *delta_mu_w,
                               float *delta_var_w, float *delta_mu_b,
                               float *delta_var_b) {
    // src/batchnorm_layer.cpp:307-332
    fan_out(fi * B, threads, [=](int lo, int hi) {
        for (int row = lo; row < hi; row++) {
            const float inv = 1.0f / std::sqrt(var_norm[row % fi] + epsilon);
            const float mra = mu_norm[row % fi];
            for (int col = 0; col < wihi; col++) {
                const int at = col + row * wihi;
                const float tmp = inv * (mu_a[at] - mra) * var_w[row % fi];
                tmp_1[at] = tmp * delta_mu_out[at];
                tmp_2[at] = tmp * delta_var_out[at] * tmp;
            }
        }
    });
    param_sum(tmp_1, tmp_2, wihi, fi, B, delta_mu_w, delta_var_w);
    if (!bias) return;
    // src/batchnorm_layer.cpp:334-354
    fan_out(fi * B, threads, [=](int lo, int hi) {
        for (int row = lo; row < hi; row++) {
            for (int col = 0; col < wihi; col++) {
                const float tmp = var_b[row % fi];
                tmp_1[col + row * wihi] = tmp * delta_mu_out[col + row * wihi];
                tmp_2[col + row * wihi] = tmp * delta_var_out[col + row * wihi] * tmp;
            }
        }
    });
    param_sum(tmp_1, tmp_2, wihi, fi, B, delta_mu_b, delta_var_b);
}

// ---------------------------------------------------------------------------
// AvgPool2d
// ---------------------------------------------------------------------------

// src/pooling_layer.cpp:453-484: the receptive-field table of the conv layer,
// transposed to [tap][output pixel]; the per-input-pixel list of output pixels
// only when windows overlap.
int oracle_avgpool2d_build_idx(int kernel, int stride, int wi, int hi, int wo,
                               int ho, int pad, int pad_type, int *pool_idx,
                               int *z_ud_idx, int *w, int *h, int *overlap) {
    const int k2 = kernel * kernel;
    std::vector<int> fm((size_t)wo * ho * k2), zw((size_t)wi * hi * k2), zud((size_t)wi * hi * k2);
    int rc = oracle_conv2d_build_idx(kernel, stride, wi, hi, wo, ho, pad, pad_type, k2 + 1,
                                     fm.data(), zw.data(), zud.data(), w, h);
    if (rc != 0) return rc;
    for (int o = 0; o < wo * ho; o++)
        for (int t = 0; t < k2; t++) pool_idx[(size_t)t * wo * ho + o] = fm[(size_t)o * k2 + t];
    // AvgPool2d::lazy_index_init (src/pooling_layer.cpp:186-190)
    *overlap = !(kernel == stride || kernel == wi);
    if (*overlap) {
        for (int i = 0; i < *w * *h; i++) z_ud_idx[i] = zud[i];
    } else {
        *w = 0;
        *h = 0;
    }
    return 0;
}

void oracle_avgpool2d_fwd(const float *mu_a, const float *var_a,
                          const int *pool_idx, int woho, int wihi, int ki,
                          int n_out, int n_in, int overlap, int threads,
                          float *mu_z, float *var_z) {
    const int ki2 = ki * ki;
    fan_out(n_out, threads, [=](int lo, int hi) {
        for (int col = lo; col < hi; col++) {
            float s_mu = 0, s_var = 0;
            for (int i = 0; i < ki2; i++) {
                if (overlap) {  // src/pooling_layer.cpp:201-225
                    int a = pool_idx[col % woho + woho * i];
                    if (a > -1) {
                        a += (col / woho) * wihi;
                        s_mu += mu_a[a - 1];
                        s_var += var_a[a - 1];
                    }
                } else {  // src/pooling_layer.cpp:259-280
                    const int a = pool_idx[col % woho + woho * i] + (col / woho) * wihi - 1;
                    s_mu += mu_a[a];
                    s_var += var_a[a];
                }
            }
            mu_z[col] = s_mu / ki2;
            var_z[col] = s_var / (ki2 * ki2);
        }
    });
}

void oracle_avgpool2d_bwd_dz(const float *jcb, const float *delta_mu_out,
                             const float *delta_var_out, const int *z_ud_idx,
                             int woho, int wihi, int ki, int nr, int wo,
                             int n_in, int n_out, int overlap, int threads,
                             float *delta_mu, float *delta_var) {
    const int ki2 = ki * ki;
    if (overlap) {  // src/pooling_layer.cpp:316-340
        fan_out(n_in, threads, [=](int lo, int hi) {
            for (int col = lo; col < hi; col++) {
                float s_mu = 0, s_var = 0;
                for (int i = 0; i < nr; i++) {
                    int z = z_ud_idx[col % wihi + wihi * i];
                    if (z > -1) {
                        z += (col / wihi) * woho;
                        s_mu += delta_mu_out[z - 1];
                        s_var += delta_var_out[z - 1];
                    }
                }
                delta_mu[col] = s_mu * jcb[col] / ki2;
                delta_var[col] = s_var * jcb[col] * jcb[col] / (ki2 * ki2);
            }
        });
        return;
    }
    // src/pooling_layer.cpp:379-399 with k = n_in / (ki*wo) (line 163-164)
    const int m = ki * wo;
    const int k = n_in / m;
    fan_out(k * m, threads, [=](int lo, int hi) {
        for (int j = lo; j < hi; j++) {
            const int row = j / k, col = j % k;
            const int at = row + col * m, src = row / ki + (col / ki) * wo;
            delta_mu[at] = delta_mu_out[src] * jcb[at] / ki2;
            delta_var[at] = delta_var_out[src] * jcb[at] * jcb[at] / (ki2 * ki2);
        }
    });
}

// ---------------------------------------------------------------------------
// Residual connection
// ---------------------------------------------------------------------------

// src/resnet_block.cpp:8-18
void oracle_add_shortcut(const float *mu_s, const float *var_s, int n,
                         float *mu_a, float *var_a) {
    for (int i = 0; i < n; i++) {
        mu_a[i] += mu_s[i];
        var_a[i] += var_s[i];
    }
}

// src/resnet_block.cpp:20-31
void oracle_add_shortcut_delta(const float *mu_s, const float *var_s,
                               const float *jcb_s, int n, float *mu_a,
                               float *var_a) {
    for (int i = 0; i < n; i++) {
        mu_a[i] += mu_s[i] * jcb_s[i];
        var_a[i] += var_s[i] * jcb_s[i] * jcb_s[i];
    }
}

}  // extern "C"

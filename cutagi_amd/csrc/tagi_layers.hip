// The layers that sit between the Linear / Conv2d contractions of a TAGI
// network: MixtureReLU, BatchNorm2d (statistics, normalisation, backward),
// AvgPool2d and the residual adds. All of them are bandwidth-bound passes over
// [B][channels][pixels] tensors; gfx950.
#include <cstdint>

#include "tagi_internal.h"
#include "tagi_activation.h"

namespace tagi {
namespace {

constexpr int TPB = 256;

inline unsigned blocks_for(size_t n, int per_block) {
    return (unsigned)((n + per_block - 1) / per_block);
}
// (a null pointer counts as aligned: optional operands)
inline bool aligned16(const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; }

// ---------------------------------------------------------------------------
// MixtureReLU: moments of max(z, 0) for z ~ N(mu, var), floored at 1e-6; the
// Jacobian is the probability mass above zero.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(TPB) void mixture_relu_kernel(const float *__restrict__ mu_z,
                                                           const float *__restrict__ var_z,
                                                           size_t n, float *__restrict__ mu_a,
                                                           float *__restrict__ jcb,
                                                           float *__restrict__ var_a) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n) return;
    float m, v, j;
    mixture_relu_moments(mu_z[i], var_z[i], m, v, j);
    mu_a[i] = m;
    var_a[i] = v;
    jcb[i] = j;
}

// ---------------------------------------------------------------------------
// Block-wide sums of up to four values, folded in a fixed order.
// ---------------------------------------------------------------------------
template <int NV>
__device__ __forceinline__ void block_sum(float (&v)[NV], float (*s)[TPB / 64]) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int k = 0; k < NV; k++) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) v[k] += __shfl_down(v[k], off, 64);
        if (lane == 0) s[k][wave] = v[k];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < NV; k++) {
        float t = 0.f;
#pragma unroll
        for (int w = 0; w < TPB / 64; w++) t += s[k][w];
        v[k] = t;
    }
    __syncthreads();
}

// ---------------------------------------------------------------------------
// BatchNorm2d statistics. Workgroup (chunk, channel) owns the samples
// [b_lo, b_hi) of one channel: element count, mean, sum of squared deviations
// from that mean, and the sum of the activation variances. The chunks of a
// channel are merged pairwise in index order (Chan et al.), which keeps the
// two-pass accuracy of the reference's "mean first, then deviations".
// ---------------------------------------------------------------------------
// (VEC: wihi % 4 == 0 and 16-byte aligned arrays: four pixels of one channel map per
// load, two loads in flight per array)
template <bool VEC>
__global__ __launch_bounds__(TPB) void bn_stats_partial_kernel(
    const float *__restrict__ mu_a, const float *__restrict__ var_a, int wihi, int fi, int B,
    int b_per_chunk, float *__restrict__ part) {
    __shared__ float s[2][TPB / 64];
    const int c = blockIdx.y, chunk = blockIdx.x, chunks = gridDim.x;
    const int b_lo = chunk * b_per_chunk, b_hi = min(B, b_lo + b_per_chunk);
    const int count = max(0, b_hi - b_lo) * wihi;

    float v[2] = {0.f, 0.f};
    if (VEC) {
        const int w4 = wihi >> 2, n4 = count >> 2;
        for (int i = threadIdx.x; i < n4; i += TPB) {
            const int b = b_lo + i / w4, p = (i % w4) * 4;
            const size_t at = ((size_t)b * fi + c) * wihi + p;
            const float4 m = *reinterpret_cast<const float4 *>(mu_a + at);
            const float4 q = *reinterpret_cast<const float4 *>(var_a + at);
            v[0] += (m.x + m.y) + (m.z + m.w);
            v[1] += (q.x + q.y) + (q.z + q.w);
        }
    } else {
        for (int i = threadIdx.x; i < count; i += TPB) {
            const int b = b_lo + i / wihi, p = i % wihi;
            const size_t at = ((size_t)b * fi + c) * wihi + p;
            v[0] += mu_a[at];
            v[1] += var_a[at];
        }
    }
    block_sum<2>(v, s);
    const float mean = count > 0 ? v[0] / count : 0.f;
    const float sum_var = v[1];

    float d[1] = {0.f};
    if (VEC) {
        const int w4 = wihi >> 2, n4 = count >> 2;
        for (int i = threadIdx.x; i < n4; i += TPB) {
            const int b = b_lo + i / w4, p = (i % w4) * 4;
            const float4 m = *reinterpret_cast<const float4 *>(mu_a + ((size_t)b * fi + c) * wihi + p);
            const float x0 = m.x - mean, x1 = m.y - mean, x2 = m.z - mean, x3 = m.w - mean;
            d[0] += (x0 * x0 + x1 * x1) + (x2 * x2 + x3 * x3);
        }
    } else {
        for (int i = threadIdx.x; i < count; i += TPB) {
            const int b = b_lo + i / wihi, p = i % wihi;
            const float x = mu_a[((size_t)b * fi + c) * wihi + p] - mean;
            d[0] += x * x;
        }
    }
    block_sum<1>(d, s);
    if (threadIdx.x == 0) {
        float *o = part + ((size_t)c * chunks + chunk) * 4;
        o[0] = (float)count;
        o[1] = mean;
        o[2] = d[0];
        o[3] = sum_var;
    }
}

__global__ __launch_bounds__(64) void bn_stats_final_kernel(const float *__restrict__ part,
                                                            int fi, int chunks, float momentum,
                                                            float *__restrict__ mu_s,
                                                            float *__restrict__ var_s,
                                                            float *__restrict__ mu_ra,
                                                            float *__restrict__ var_ra) {
    const int c = blockIdx.x * 64 + threadIdx.x;
    if (c >= fi) return;
    float n = 0.f, mean = 0.f, m2 = 0.f, sum_var = 0.f;
    for (int q = 0; q < chunks; q++) {
        const float *o = part + ((size_t)c * chunks + q) * 4;
        const float nb = o[0];
        if (nb <= 0.f) continue;
        const float delta = o[1] - mean, tot = n + nb;
        mean += delta * (nb / tot);
        m2 += o[2] + delta * delta * (n * nb / tot);
        n = tot;
        sum_var += o[3];
    }
    const float var = (m2 + sum_var) / (n - 1.f);
    mu_s[c] = mean;
    var_s[c] = var;
    mu_ra[c] = mu_ra[c] * momentum + mean * (1.f - momentum);
    var_ra[c] = var_ra[c] * momentum + var * (1.f - momentum);
}

// z = (a - mean) / sqrt(var + eps) * w + b with Gaussian w, b and a.
__global__ __launch_bounds__(TPB) void bn_fwd_kernel(
    const float *__restrict__ mu_w, const float *__restrict__ var_w,
    const float *__restrict__ mu_b, const float *__restrict__ var_b,
    const float *__restrict__ mu_a, const float *__restrict__ var_a,
    const float *__restrict__ mu_norm, const float *__restrict__ var_norm, float epsilon,
    int wihi, int fi, size_t n, const float *__restrict__ mu_res,
    const float *__restrict__ var_res, float *__restrict__ mu_z, float *__restrict__ var_z) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n) return;
    const int c = (int)((i / wihi) % fi);
    const float inv = 1.0f / sqrtf(var_norm[c] + epsilon);
    const float mw = mu_w[c], vw = var_w[c];
    const float d = mu_a[i] - mu_norm[c];
    float mz = inv * d * mw;
    float vz = inv * inv * (var_a[i] * (mw * mw + vw) + vw * d * d);
    if (mu_b != nullptr) {
        mz += mu_b[c];
        vz += var_b[c];
    }
    if (mu_res != nullptr) {  // the residual connection that ends on this layer
        mz += mu_res[i];
        vz += var_res[i];
    }
    mu_z[i] = mz;
    var_z[i] = vz;
}

// The same for four consecutive pixels of one channel map per thread (wihi % 4 == 0,
// 16-byte aligned arrays).
__global__ __launch_bounds__(TPB) void bn_fwd_vec_kernel(
    const float *__restrict__ mu_w, const float *__restrict__ var_w,
    const float *__restrict__ mu_b, const float *__restrict__ var_b,
    const float *__restrict__ mu_a, const float *__restrict__ var_a,
    const float *__restrict__ mu_norm, const float *__restrict__ var_norm, float epsilon,
    int wihi, int fi, size_t n4, const float *__restrict__ mu_res,
    const float *__restrict__ var_res, float *__restrict__ mu_z, float *__restrict__ var_z) {
    const size_t i4 = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i4 >= n4) return;
    const size_t i = i4 * 4;
    const int c = (int)((i / wihi) % fi);
    const float4 ma = *reinterpret_cast<const float4 *>(mu_a + i);
    const float4 va = *reinterpret_cast<const float4 *>(var_a + i);
    float4 rm = make_float4(0.f, 0.f, 0.f, 0.f), rv = rm;
    if (mu_res != nullptr) {
        rm = *reinterpret_cast<const float4 *>(mu_res + i);
        rv = *reinterpret_cast<const float4 *>(var_res + i);
    }
    const float inv = 1.0f / sqrtf(var_norm[c] + epsilon);
    const float mw = mu_w[c], vw = var_w[c], mean = mu_norm[c];
    const float bm = mu_b != nullptr ? mu_b[c] : 0.f, bv = mu_b != nullptr ? var_b[c] : 0.f;
    const bool has_b = mu_b != nullptr, has_r = mu_res != nullptr;
    auto one = [&](float a, float v, float r0, float r1, float &mz, float &vz) {
        const float d = a - mean;
        mz = inv * d * mw;
        vz = inv * inv * (v * (mw * mw + vw) + vw * d * d);
        if (has_b) {
            mz += bm;
            vz += bv;
        }
        if (has_r) {
            mz += r0;
            vz += r1;
        }
    };
    float4 om, ov;
    one(ma.x, va.x, rm.x, rv.x, om.x, ov.x);
    one(ma.y, va.y, rm.y, rv.y, om.y, ov.y);
    one(ma.z, va.z, rm.z, rv.z, om.z, ov.z);
    one(ma.w, va.w, rm.w, rv.w, om.w, ov.w);
    *reinterpret_cast<float4 *>(mu_z + i) = om;
    *reinterpret_cast<float4 *>(var_z + i) = ov;
}

// Training-mode forward with the merge of the statistics inside: bn_stats_final_kernel's
// work is done per workgroup, for the channel maps the workgroup touches (the partial
// statistics are a few cache-resident floats per channel), which saves that kernel's
// launch. A workgroup owns FT_ITER * TPB consecutive groups of four pixels; thread t < maps
// merges the chunks of map t's channel in chunk order (the same arithmetic as
// bn_stats_final_kernel, so mean and variance are the same bits) and leaves them in LDS;
// the one workgroup that holds the start of map (image 0, channel c) also writes the batch
// statistics and moves the running averages. The normalisation is bn_fwd_vec_kernel's.
constexpr int FT_ITER = 4, FT_MAX_MAPS = FT_ITER * TPB / 4 + 1;   // wihi >= 16

__global__ __launch_bounds__(TPB) void bn_fwd_train_vec_kernel(
    const float *__restrict__ mu_w, const float *__restrict__ var_w,
    const float *__restrict__ mu_b, const float *__restrict__ var_b,
    const float *__restrict__ mu_a, const float *__restrict__ var_a,
    const float *__restrict__ part, int chunks, float momentum, float epsilon, int wihi, int fi,
    size_t n4, const float *__restrict__ mu_res, const float *__restrict__ var_res,
    float *__restrict__ mu_s, float *__restrict__ var_s, float *__restrict__ mu_ra,
    float *__restrict__ var_ra, float *__restrict__ mu_z, float *__restrict__ var_z) {
    __shared__ float s_mean[FT_MAX_MAPS], s_var[FT_MAX_MAPS];
    const int w4 = wihi >> 2;
    const size_t first = (size_t)blockIdx.x * (FT_ITER * TPB);
    const size_t end = min(n4, first + (size_t)FT_ITER * TPB);
    const size_t map_first = first / w4, map_last = (end - 1) / w4;
    const int maps = (int)(map_last - map_first + 1);
    for (int t = threadIdx.x; t < maps; t += TPB) {
        const size_t map = map_first + t;
        const int c = (int)(map % fi);
        float n = 0.f, mean = 0.f, m2 = 0.f, sum_var = 0.f;
        for (int q = 0; q < chunks; q++) {
            const float *o = part + ((size_t)c * chunks + q) * 4;
            const float nb = o[0];
            if (nb <= 0.f) continue;
            const float delta = o[1] - mean, tot = n + nb;
            mean += delta * (nb / tot);
            m2 += o[2] + delta * delta * (n * nb / tot);
            n = tot;
            sum_var += o[3];
        }
        const float var = (m2 + sum_var) / (n - 1.f);
        s_mean[t] = mean;
        s_var[t] = var;
        if (map < (size_t)fi && map * w4 >= first) {   // image 0: once per channel
            mu_s[c] = mean;
            var_s[c] = var;
            mu_ra[c] = mu_ra[c] * momentum + mean * (1.f - momentum);
            var_ra[c] = var_ra[c] * momentum + var * (1.f - momentum);
        }
    }
    __syncthreads();
    const bool has_b = mu_b != nullptr, has_r = mu_res != nullptr;
#pragma unroll
    for (int it = 0; it < FT_ITER; it++) {
        const size_t i4 = first + (size_t)it * TPB + threadIdx.x;
        if (i4 >= end) break;
        const size_t i = i4 * 4, map = i4 / w4;
        const int c = (int)(map % fi), li = (int)(map - map_first);
        const float4 ma = *reinterpret_cast<const float4 *>(mu_a + i);
        const float4 va = *reinterpret_cast<const float4 *>(var_a + i);
        float4 rm = make_float4(0.f, 0.f, 0.f, 0.f), rv = rm;
        if (has_r) {
            rm = *reinterpret_cast<const float4 *>(mu_res + i);
            rv = *reinterpret_cast<const float4 *>(var_res + i);
        }
        const float inv = 1.0f / sqrtf(s_var[li] + epsilon);
        const float mw = mu_w[c], vw = var_w[c], mean = s_mean[li];
        const float bm = has_b ? mu_b[c] : 0.f, bv = has_b ? var_b[c] : 0.f;
        auto one = [&](float a, float v, float r0, float r1, float &mz, float &vz) {
            const float d = a - mean;
            mz = inv * d * mw;
            vz = inv * inv * (v * (mw * mw + vw) + vw * d * d);
            if (has_b) {
                mz += bm;
                vz += bv;
            }
            if (has_r) {
                mz += r0;
                vz += r1;
            }
        };
        float4 om, ov;
        one(ma.x, va.x, rm.x, rv.x, om.x, ov.x);
        one(ma.y, va.y, rm.y, rv.y, om.y, ov.y);
        one(ma.z, va.z, rm.z, rv.z, om.z, ov.z);
        one(ma.w, va.w, rm.w, rv.w, om.w, ov.w);
        *reinterpret_cast<float4 *>(mu_z + i) = om;
        *reinterpret_cast<float4 *>(var_z + i) = ov;
    }
}

// Backward of one (chunk, channel): the state innovations element by element,
// and partial sums of the four parameter innovations of the channel.
template <bool VEC>
__global__ __launch_bounds__(TPB) void bn_bwd_partial_kernel(
    const float *__restrict__ mu_w, const float *__restrict__ var_w,
    const float *__restrict__ mu_a, const float *__restrict__ jcb,
    const float *__restrict__ mu_norm, const float *__restrict__ var_norm,
    const float *__restrict__ dmu_out, const float *__restrict__ dvar_out, float epsilon,
    int wihi, int fi, int B, int b_per_chunk, int state_update, int param_update,
    float *__restrict__ dmu, float *__restrict__ dvar, float *__restrict__ part) {
    __shared__ float s[4][TPB / 64];
    const int c = blockIdx.y, chunk = blockIdx.x, chunks = gridDim.x;
    const int b_lo = chunk * b_per_chunk, b_hi = min(B, b_lo + b_per_chunk);
    const int count = max(0, b_hi - b_lo) * wihi;
    const float inv = 1.0f / sqrtf(var_norm[c] + epsilon);
    const float mean = mu_norm[c], mw = mu_w[c], vw = var_w[c];

    float v[4] = {0.f, 0.f, 0.f, 0.f};
    if (VEC) {
        const int w4 = wihi >> 2, n4 = count >> 2;
        const float sj = inv * mw, sp = inv * vw;
        for (int i = threadIdx.x; i < n4; i += TPB) {
            const int b = b_lo + i / w4, p = (i % w4) * 4;
            const size_t at = ((size_t)b * fi + c) * wihi + p;
            const float4 dm = *reinterpret_cast<const float4 *>(dmu_out + at);
            const float4 dv = *reinterpret_cast<const float4 *>(dvar_out + at);
            if (state_update) {
                const float4 j = *reinterpret_cast<const float4 *>(jcb + at);
                const float t0 = sj * j.x, t1 = sj * j.y, t2 = sj * j.z, t3 = sj * j.w;
                *reinterpret_cast<float4 *>(dmu + at) =
                    make_float4(t0 * dm.x, t1 * dm.y, t2 * dm.z, t3 * dm.w);
                *reinterpret_cast<float4 *>(dvar + at) =
                    make_float4(t0 * dv.x * t0, t1 * dv.y * t1, t2 * dv.z * t2, t3 * dv.w * t3);
            }
            if (param_update) {
                const float4 a = *reinterpret_cast<const float4 *>(mu_a + at);
                const float t0 = sp * (a.x - mean), t1 = sp * (a.y - mean), t2 = sp * (a.z - mean),
                            t3 = sp * (a.w - mean);
                v[0] += (t0 * dm.x + t1 * dm.y) + (t2 * dm.z + t3 * dm.w);
                v[1] += (t0 * dv.x * t0 + t1 * dv.y * t1) + (t2 * dv.z * t2 + t3 * dv.w * t3);
                v[2] += (dm.x + dm.y) + (dm.z + dm.w);
                v[3] += (dv.x + dv.y) + (dv.z + dv.w);
            }
        }
    } else {
        for (int i = threadIdx.x; i < count; i += TPB) {
            const int b = b_lo + i / wihi, p = i % wihi;
            const size_t at = ((size_t)b * fi + c) * wihi + p;
            const float dm = dmu_out[at], dv = dvar_out[at];
            if (state_update) {
                const float t = inv * mw * jcb[at];
                dmu[at] = t * dm;
                dvar[at] = t * dv * t;
            }
            if (param_update) {
                const float t = inv * (mu_a[at] - mean) * vw;
                v[0] += t * dm;
                v[1] += t * dv * t;
                v[2] += dm;
                v[3] += dv;
            }
        }
    }
    if (!param_update) return;
    block_sum<4>(v, s);
    if (threadIdx.x < 4) part[((size_t)c * chunks + chunk) * 4 + threadIdx.x] = v[threadIdx.x];
}

__global__ __launch_bounds__(64) void bn_bwd_final_kernel(const float *__restrict__ part,
                                                          const float *__restrict__ var_b, int fi,
                                                          int chunks, float *__restrict__ dmu_w,
                                                          float *__restrict__ dvar_w,
                                                          float *__restrict__ dmu_b,
                                                          float *__restrict__ dvar_b) {
    const int c = blockIdx.x * 64 + threadIdx.x;
    if (c >= fi) return;
    float v[4] = {0.f, 0.f, 0.f, 0.f};
    for (int q = 0; q < chunks; q++) {
        const float *o = part + ((size_t)c * chunks + q) * 4;
#pragma unroll
        for (int k = 0; k < 4; k++) v[k] += o[k];
    }
    dmu_w[c] = v[0];
    dvar_w[c] = v[1];
    if (var_b != nullptr) {
        const float vb = var_b[c];
        dmu_b[c] = vb * v[2];
        dvar_b[c] = vb * v[3] * vb;
    }
}

// ---------------------------------------------------------------------------
// AvgPool2d. pool_idx [k*k][woho]: 1-based input pixel under tap t of output
// pixel o (-1: padding, which still counts in the divisor); z_ud_idx [nr][wihi]:
// the output pixels an input pixel contributes to (overlapping windows only).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(TPB) void avgpool_fwd_kernel(const float *__restrict__ mu_a,
                                                          const float *__restrict__ var_a,
                                                          const int *__restrict__ pool_idx,
                                                          int woho, int wihi, int ki2, int n_out,
                                                          float *__restrict__ mu_z,
                                                          float *__restrict__ var_z) {
    const int col = blockIdx.x * TPB + threadIdx.x;
    if (col >= n_out) return;
    const int o = col % woho;
    const size_t base = (size_t)(col / woho) * wihi;
    float sm = 0.f, sv = 0.f;
    for (int t = 0; t < ki2; t++) {
        const int a = pool_idx[o + woho * t];
        if (a > -1) {
            sm += mu_a[base + a - 1];
            sv += var_a[base + a - 1];
        }
    }
    mu_z[col] = sm / ki2;
    var_z[col] = sv / (ki2 * ki2);
}

__global__ __launch_bounds__(TPB) void avgpool_bwd_overlap_kernel(
    const float *__restrict__ jcb, const float *__restrict__ dmu_out,
    const float *__restrict__ dvar_out, const int *__restrict__ z_ud_idx, int woho, int wihi,
    int ki2, int nr, int n_in, float *__restrict__ dmu, float *__restrict__ dvar) {
    const int col = blockIdx.x * TPB + threadIdx.x;
    if (col >= n_in) return;
    const int p = col % wihi;
    const size_t base = (size_t)(col / wihi) * woho;
    float sm = 0.f, sv = 0.f;
    for (int i = 0; i < nr; i++) {
        const int z = z_ud_idx[p + wihi * i];
        if (z > -1) {
            sm += dmu_out[base + z - 1];
            sv += dvar_out[base + z - 1];
        }
    }
    const float j = jcb[col];
    dmu[col] = sm * j / ki2;
    dvar[col] = sv * j * j / (ki2 * ki2);
}

// Windows that tile the image: input element `at` lies in row at % (ki*wo) of
// image-row block at / (ki*wo); its window is (row / ki, block / ki).
__global__ __launch_bounds__(TPB) void avgpool_bwd_tiled_kernel(
    const float *__restrict__ jcb, const float *__restrict__ dmu_out,
    const float *__restrict__ dvar_out, int wo, int ki, int n_in, float *__restrict__ dmu,
    float *__restrict__ dvar) {
    const int at = blockIdx.x * TPB + threadIdx.x;
    if (at >= n_in) return;
    const int m = ki * wo, ki2 = ki * ki;
    const int row = at % m, blk = at / m;
    const int src = row / ki + (blk / ki) * wo;
    const float j = jcb[at];
    dmu[at] = dmu_out[src] * j / ki2;
    dvar[at] = dvar_out[src] * j * j / (ki2 * ki2);
}

// ---------------------------------------------------------------------------
// Residual connection
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(TPB) void add_shortcut_kernel(const float *__restrict__ mu_s,
                                                           const float *__restrict__ var_s,
                                                           const float *__restrict__ jcb_s,
                                                           size_t n, float *__restrict__ mu_a,
                                                           float *__restrict__ var_a) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n) return;
    if (jcb_s != nullptr) {
        const float j = jcb_s[i];
        mu_a[i] += mu_s[i] * j;
        var_a[i] += var_s[i] * j * j;
    } else {
        mu_a[i] += mu_s[i];
        var_a[i] += var_s[i];
    }
}

// Samples per chunk so that a channel-major grid has about 4 workgroups per CU.
int bn_chunks(int fi, int B, int *b_per_chunk) {
    int chunks = (4 * num_cu() + fi - 1) / fi;
    if (chunks > B) chunks = B;
    if (chunks < 1) chunks = 1;
    *b_per_chunk = (B + chunks - 1) / chunks;
    return (B + *b_per_chunk - 1) / *b_per_chunk;
}

}  // namespace

hipError_t launch_mixture_relu(const float *mu_z, const float *var_z, size_t n, float *mu_a,
                               float *jcb, float *var_a, hipStream_t stream) {
    hipLaunchKernelGGL(mixture_relu_kernel, dim3(blocks_for(n, TPB)), dim3(TPB), 0, stream, mu_z,
                       var_z, n, mu_a, jcb, var_a);
    return hipGetLastError();
}

size_t batchnorm2d_scratch_floats(int fi, int B) {
    int per = 0;
    return (size_t)bn_chunks(fi, B, &per) * fi * 4;
}

hipError_t launch_batchnorm2d_stats(const float *mu_a, const float *var_a, int wihi, int fi,
                                    int B, float momentum, float *scratch, float *mu_s,
                                    float *var_s, float *mu_ra, float *var_ra,
                                    hipStream_t stream) {
    int per = 0;
    const int chunks = bn_chunks(fi, B, &per);
    if (wihi % 4 == 0 && aligned16(mu_a) && aligned16(var_a))
        hipLaunchKernelGGL(bn_stats_partial_kernel<true>, dim3(chunks, fi), dim3(TPB), 0, stream,
                           mu_a, var_a, wihi, fi, B, per, scratch);
    else
        hipLaunchKernelGGL(bn_stats_partial_kernel<false>, dim3(chunks, fi), dim3(TPB), 0, stream,
                           mu_a, var_a, wihi, fi, B, per, scratch);
    hipLaunchKernelGGL(bn_stats_final_kernel, dim3((fi + 63) / 64), dim3(64), 0, stream, scratch,
                       fi, chunks, momentum, mu_s, var_s, mu_ra, var_ra);
    return hipGetLastError();
}

int g_bn_fused_train = 1;

// Statistics + normalisation of a training-mode forward: two launches where the 16-byte
// path applies (partial statistics, then the forward that merges them itself), otherwise
// the three of launch_batchnorm2d_stats + launch_batchnorm2d_fwd.
hipError_t launch_batchnorm2d_fwd_train(const float *mu_w, const float *var_w, const float *mu_b,
                                        const float *var_b, const float *mu_a, const float *var_a,
                                        const float *mu_res, const float *var_res, float momentum,
                                        float epsilon, int wihi, int fi, int B, float *scratch,
                                        float *mu_s, float *var_s, float *mu_ra, float *var_ra,
                                        float *mu_z, float *var_z, hipStream_t stream) {
    const bool vec = wihi % 4 == 0 && wihi >= 16 && aligned16(mu_a) && aligned16(var_a) &&
                     aligned16(mu_z) && aligned16(var_z) && aligned16(mu_res) && aligned16(var_res);
    if (!vec || !g_bn_fused_train) {
        hipError_t e = launch_batchnorm2d_stats(mu_a, var_a, wihi, fi, B, momentum, scratch, mu_s,
                                                var_s, mu_ra, var_ra, stream);
        if (e != hipSuccess) return e;
        return launch_batchnorm2d_fwd(mu_w, var_w, mu_b, var_b, mu_a, var_a, mu_s, var_s, epsilon,
                                      wihi, fi, B, mu_z, var_z, stream, mu_res, var_res);
    }
    int per = 0;
    const int chunks = bn_chunks(fi, B, &per);
    hipLaunchKernelGGL(bn_stats_partial_kernel<true>, dim3(chunks, fi), dim3(TPB), 0, stream, mu_a,
                       var_a, wihi, fi, B, per, scratch);
    const size_t n4 = (size_t)B * fi * wihi / 4;
    hipLaunchKernelGGL(bn_fwd_train_vec_kernel, dim3(blocks_for(n4, FT_ITER * TPB)), dim3(TPB), 0,
                       stream, mu_w, var_w, mu_b, var_b, mu_a, var_a, scratch, chunks, momentum,
                       epsilon, wihi, fi, n4, mu_res, var_res, mu_s, var_s, mu_ra, var_ra, mu_z,
                       var_z);
    return hipGetLastError();
}

hipError_t launch_batchnorm2d_fwd(const float *mu_w, const float *var_w, const float *mu_b,
                                  const float *var_b, const float *mu_a, const float *var_a,
                                  const float *mu_norm, const float *var_norm, float epsilon,
                                  int wihi, int fi, int B, float *mu_z, float *var_z,
                                  hipStream_t stream, const float *mu_res, const float *var_res) {
    const size_t n = (size_t)B * fi * wihi;
    if (wihi % 4 == 0 && aligned16(mu_a) && aligned16(var_a) && aligned16(mu_z) && aligned16(var_z) &&
        aligned16(mu_res) && aligned16(var_res)) {
        hipLaunchKernelGGL(bn_fwd_vec_kernel, dim3(blocks_for(n / 4, TPB)), dim3(TPB), 0, stream,
                           mu_w, var_w, mu_b, var_b, mu_a, var_a, mu_norm, var_norm, epsilon, wihi,
                           fi, n / 4, mu_res, var_res, mu_z, var_z);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(bn_fwd_kernel, dim3(blocks_for(n, TPB)), dim3(TPB), 0, stream, mu_w, var_w,
                       mu_b, var_b, mu_a, var_a, mu_norm, var_norm, epsilon, wihi, fi, n, mu_res,
                       var_res, mu_z, var_z);
    return hipGetLastError();
}

hipError_t launch_batchnorm2d_bwd(const float *mu_w, const float *var_w, const float *var_b,
                                  const float *mu_a, const float *jcb, const float *mu_norm,
                                  const float *var_norm, const float *dmu_out,
                                  const float *dvar_out, float epsilon, int wihi, int fi, int B,
                                  int state_update, int param_update, float *scratch, float *dmu,
                                  float *dvar, float *dmu_w, float *dvar_w, float *dmu_b,
                                  float *dvar_b, hipStream_t stream) {
    int per = 0;
    const int chunks = bn_chunks(fi, B, &per);
    const bool vec = wihi % 4 == 0 && aligned16(dmu_out) && aligned16(dvar_out) &&
                     (!state_update || (aligned16(jcb) && aligned16(dmu) && aligned16(dvar))) &&
                     (!param_update || aligned16(mu_a));
    if (vec)
        hipLaunchKernelGGL(bn_bwd_partial_kernel<true>, dim3(chunks, fi), dim3(TPB), 0, stream, mu_w,
                           var_w, mu_a, jcb, mu_norm, var_norm, dmu_out, dvar_out, epsilon, wihi,
                           fi, B, per, state_update, param_update, dmu, dvar, scratch);
    else
        hipLaunchKernelGGL(bn_bwd_partial_kernel<false>, dim3(chunks, fi), dim3(TPB), 0, stream,
                           mu_w, var_w, mu_a, jcb, mu_norm, var_norm, dmu_out, dvar_out, epsilon,
                           wihi, fi, B, per, state_update, param_update, dmu, dvar, scratch);
    if (param_update)
        hipLaunchKernelGGL(bn_bwd_final_kernel, dim3((fi + 63) / 64), dim3(64), 0, stream, scratch,
                           var_b, fi, chunks, dmu_w, dvar_w, dmu_b, dvar_b);
    return hipGetLastError();
}

hipError_t launch_avgpool2d_fwd(const float *mu_a, const float *var_a, const int *pool_idx,
                                int woho, int wihi, int ki, int n_out, float *mu_z, float *var_z,
                                hipStream_t stream) {
    hipLaunchKernelGGL(avgpool_fwd_kernel, dim3(blocks_for(n_out, TPB)), dim3(TPB), 0, stream,
                       mu_a, var_a, pool_idx, woho, wihi, ki * ki, n_out, mu_z, var_z);
    return hipGetLastError();
}

hipError_t launch_avgpool2d_bwd(const float *jcb, const float *dmu_out, const float *dvar_out,
                                const int *z_ud_idx, int woho, int wihi, int ki, int nr, int wo,
                                int n_in, int overlap, float *dmu, float *dvar,
                                hipStream_t stream) {
    if (overlap)
        hipLaunchKernelGGL(avgpool_bwd_overlap_kernel, dim3(blocks_for(n_in, TPB)), dim3(TPB), 0,
                           stream, jcb, dmu_out, dvar_out, z_ud_idx, woho, wihi, ki * ki, nr, n_in,
                           dmu, dvar);
    else
        hipLaunchKernelGGL(avgpool_bwd_tiled_kernel, dim3(blocks_for(n_in, TPB)), dim3(TPB), 0,
                           stream, jcb, dmu_out, dvar_out, wo, ki, n_in, dmu, dvar);
    return hipGetLastError();
}

hipError_t launch_add_shortcut(const float *mu_s, const float *var_s, const float *jcb_s,
                               size_t n, float *mu_a, float *var_a, hipStream_t stream) {
    hipLaunchKernelGGL(add_shortcut_kernel, dim3(blocks_for(n, TPB)), dim3(TPB), 0, stream, mu_s,
                       var_s, jcb_s, n, mu_a, var_a);
    return hipGetLastError();
}

}  // namespace tagi

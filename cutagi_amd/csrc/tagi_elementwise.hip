// Small bandwidth-bound kernels around the TAGI layers: bias innovation, state
// bookkeeping, capped parameter step, output innovation and ReLU. gfx950.
#include "tagi_internal.h"
#include "tagi_activation.h"

namespace tagi {
namespace {

constexpr int TPB = 256;

inline unsigned blocks_for(size_t n, int per_block) {
    return (unsigned)((n + per_block - 1) / per_block);
}

// delta_b[n] = var_b[n] * sum_b delta[b][n]. Block = 64 columns x 16 batch
// slices (one wave each): consecutive lanes read consecutive columns, the slices
// meet in LDS and are folded in a fixed order.
constexpr int BIAS_SLICES = 16;
__global__ __launch_bounds__(64 * BIAS_SLICES) void bias_delta_kernel(
    const float *__restrict__ var_b, const float *__restrict__ dmu,
    const float *__restrict__ dvar, int N, int B, float *__restrict__ dmu_b,
    float *__restrict__ dvar_b) {
    __shared__ float s0[BIAS_SLICES][64], s1[BIAS_SLICES][64];
    const int c = threadIdx.x & 63, slice = threadIdx.x >> 6;
    const int n = blockIdx.x * 64 + c;
    float a0 = 0.f, a1 = 0.f;
    if (n < N) {
        for (int b = slice; b < B; b += BIAS_SLICES) {
            a0 += dmu[(size_t)b * N + n];
            a1 += dvar[(size_t)b * N + n];
        }
    }
    s0[slice][c] = a0;
    s1[slice][c] = a1;
    __syncthreads();
    if (slice == 0 && n < N) {
        float m = 0.f, v = 0.f;
#pragma unroll
        for (int s = 0; s < BIAS_SLICES; s++) {
            m += s0[s][c];
            v += s1[s][c];
        }
        const float vb = var_b[n];
        dmu_b[n] = m * vb;
        dvar_b[n] = v * vb * vb;
    }
}

__global__ __launch_bounds__(TPB) void store_states_kernel(
    const float *__restrict__ mu_a, const float *__restrict__ jcb, size_t n_in,
    float *__restrict__ bwd_mu_a, float *__restrict__ bwd_jcb, float *__restrict__ out_jcb,
    size_t n_out) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i < n_in) {
        bwd_mu_a[i] = mu_a[i];
        if (jcb != nullptr) bwd_jcb[i] = jcb[i];  // (null: a Jacobian of one, only marked)
    }
    if (i < n_out) out_jcb[i] = 1.0f;
}

// Input of a network from pinned host memory straight into the state arrays: the mean
// is read over the bus by the kernel itself, the variance likewise or (host_var == null)
// set to zero. One launch on the compute queue instead of two copy-engine transfers and
// a fill, each of which costs a hand-over between engines on a short dependent chain.
__global__ __launch_bounds__(TPB) void upload_input_kernel(const float *__restrict__ host_mu,
                                                           const float *__restrict__ host_var,
                                                           size_t n, float *__restrict__ mu_a,
                                                           float *__restrict__ var_a) {
    const size_t stride = (size_t)gridDim.x * TPB;
    for (size_t i = (size_t)blockIdx.x * TPB + threadIdx.x; i < n; i += stride) {
        mu_a[i] = host_mu[i];
        var_a[i] = host_var != nullptr ? host_var[i] : 0.f;
    }
}

// The other direction: the first n means and variances of a state buffer written
// straight into pinned host memory by the kernel (one launch and one wait for the
// stream instead of two synchronous copies).
// With host_flag given the launch is one workgroup, which writes flag_value there after
// all of the data (release at system scope): a host thread that polls the flag sees the
// data complete without waiting for the stream through the runtime.
__global__ __launch_bounds__(TPB) void download_outputs_kernel(const float *__restrict__ mu_a,
                                                               const float *__restrict__ var_a,
                                                               size_t n, float *__restrict__ host_mu,
                                                               float *__restrict__ host_var,
                                                               unsigned *host_flag,
                                                               unsigned flag_value) {
    const size_t stride = (size_t)gridDim.x * TPB;
    for (size_t i = (size_t)blockIdx.x * TPB + threadIdx.x; i < n; i += stride) {
        host_mu[i] = mu_a[i];
        host_var[i] = var_a[i];
    }
    if (host_flag != nullptr) {
        __threadfence_system();
        __syncthreads();
        if (threadIdx.x == 0)
            __hip_atomic_store(host_flag, flag_value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
}

// p += sign(d) * min(|d|, sqrt(var)/cap); var <= 0 -> 1e-5 and counted. One
// atomic per wave: the clamped lanes are counted with a ballot.
__global__ __launch_bounds__(TPB) void param_update_kernel(
    const float *__restrict__ dmu, const float *__restrict__ dvar, float cap, size_t n,
    float *__restrict__ mu, float *__restrict__ var, int *__restrict__ neg_count) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    bool clamped = false;
    if (i < n) {
        const float dm = dmu[i], dv = dvar[i], v = var[i];
        const float sm = (float)((dm > 0.f) - (dm < 0.f));
        const float sv = (float)((dv > 0.f) - (dv < 0.f));
        const float bar = sqrtf(v) / cap;
        mu[i] += sm * fminf(fabsf(dm), bar);
        float nv = v + sv * fminf(fabsf(dv), bar);
        if (nv <= 0.0f) {
            nv = 1E-5f;
            clamped = true;
        }
        var[i] = nv;
    }
    if (neg_count != nullptr) {
        const unsigned long long mask = __ballot(clamped);
        if (mask != 0ull && (threadIdx.x & 63) == 0) atomicAdd(neg_count, __popcll(mask));
    }
}

// p += d without a cap or a floor.
__global__ __launch_bounds__(TPB) void param_raw_update_kernel(
    const float *__restrict__ dmu, const float *__restrict__ dvar, size_t n,
    float *__restrict__ mu, float *__restrict__ var) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n) return;
    mu[i] += dmu[i];
    var[i] += dvar[i];
}

// Both parameter sets of a layer in one launch: threads [0, nw) take the weights,
// [nw, nw + nb) the biases. Clamped weight variances are counted in count[slot];
// count[1 - slot], which this launch does not touch otherwise, is set to zero for
// the next step, so no launch is spent on resetting a counter.
__device__ __forceinline__ bool capped_step(float dm, float dv, float cap, float &m, float &v) {
    const float sm = (float)((dm > 0.f) - (dm < 0.f));
    const float sv = (float)((dv > 0.f) - (dv < 0.f));
    const float bar = sqrtf(v) / cap;
    m += sm * fminf(fabsf(dm), bar);
    float nv = v + sv * fminf(fabsf(dv), bar);
    const bool clamped = nv <= 0.0f;
    if (clamped) nv = 1E-5f;
    v = nv;
    return clamped;
}
__global__ __launch_bounds__(TPB) void layer_update_kernel(
    const float *__restrict__ dmu_w, const float *__restrict__ dvar_w, size_t nw,
    float *__restrict__ mu_w, float *__restrict__ var_w, const float *__restrict__ dmu_b,
    const float *__restrict__ dvar_b, size_t nb, float *__restrict__ mu_b,
    float *__restrict__ var_b, float cap, int *__restrict__ count, int slot) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i == 0 && count != nullptr) count[1 - slot] = 0;
    bool clamped = false;
    if (i < nw) {
        float m = mu_w[i], v = var_w[i];
        clamped = capped_step(dmu_w[i], dvar_w[i], cap, m, v);
        mu_w[i] = m;
        var_w[i] = v;
    } else if (i < nw + nb) {
        const size_t j = i - nw;
        float m = mu_b[j], v = var_b[j];
        capped_step(dmu_b[j], dvar_b[j], cap, m, v);
        mu_b[j] = m;
        var_b[j] = v;
    }
    if (count != nullptr) {
        const unsigned long long mask = __ballot(clamped);
        if (mask != 0ull && (threadIdx.x & 63) == 0) atomicAdd(count + slot, __popcll(mask));
    }
}

// layer_update_kernel for several layers at once: the block finds its layer in the
// table of first blocks (uniform over the block), then does that layer's step.
__global__ __launch_bounds__(TPB) void model_update_kernel(ModelUpdateArgs a) {
    int it = 0;
    while (it + 1 < a.n && blockIdx.x >= a.first_block[it + 1]) it++;
    const size_t i = (size_t)(blockIdx.x - a.first_block[it]) * TPB + threadIdx.x;
    const size_t nw = a.nw[it], nb = a.nb[it];
    int *count = a.count[it];
    const int slot = a.slot[it];
    const float cap = a.cap[it];
    if (i == 0 && count != nullptr) count[1 - slot] = 0;
    bool clamped = false;
    if (i < nw) {
        float m = a.mu_w[it][i], v = a.var_w[it][i];
        clamped = capped_step(a.dmu_w[it][i], a.dvar_w[it][i], cap, m, v);
        a.mu_w[it][i] = m;
        a.var_w[it][i] = v;
    } else if (i < nw + nb) {
        const size_t j = i - nw;
        float m = a.mu_b[it][j], v = a.var_b[it][j];
        capped_step(a.dmu_b[it][j], a.dvar_b[it][j], cap, m, v);
        a.mu_b[it][j] = m;
        a.var_b[it][j] = v;
    }
    if (count != nullptr) {
        const unsigned long long mask = __ballot(clamped);
        if (mask != 0ull && (threadIdx.x & 63) == 0) atomicAdd(count + slot, __popcll(mask));
    }
}

__global__ __launch_bounds__(TPB) void out_update_dense_kernel(
    const float *__restrict__ mu_a, const float *__restrict__ var_a,
    const float *__restrict__ jcb, const float *__restrict__ obs,
    const float *__restrict__ var_obs, int n, float *__restrict__ dmu,
    float *__restrict__ dvar) {
    const int col = blockIdx.x * TPB + threadIdx.x;
    if (col >= n) return;
    const float t = jcb[col] / (var_a[col] + var_obs[col]);
    if (isinf(t) || isnan(t) || isnan(obs[col])) {
        dmu[col] = 0.f;
        dvar[col] = 0.f;
    } else {
        dmu[col] = t * (obs[col] - mu_a[col]);
        dvar[col] = -t * jcb[col];
    }
}

// Output layer with a learned error variance: unit 2i is the mean output, unit
// 2i+1 the expected squared error (positive). One thread per observation.
__global__ __launch_bounds__(TPB) void out_update_heteros_kernel(
    const float2 *__restrict__ mu_a, const float2 *__restrict__ var_a,
    const float2 *__restrict__ jcb, const float *__restrict__ obs, int n,
    float2 *__restrict__ dmu, float2 *__restrict__ dvar) {
// differences of nearly equal moments: keep the reference's roundings (no fused
// multiply-adds), so that the cancellations lose the same digits on both sides
#pragma clang fp contract(off)
    const int i = blockIdx.x * TPB + threadIdx.x;
    if (i >= n) return;
    const float2 m = mu_a[i], v = var_a[i], j = jcb[i];
    const float y = obs[i];
    const float mu_v2 = m.y;                               // prior mean of V^2
    const float var_v2 = 3.0f * v.y + 2.0f * m.y * m.y;    // prior variance of V^2
    const float var_sum = v.x + mu_v2;                     // predictive variance of y
    const float t = j.x / var_sum;
    const bool bad_obs = isinf(y) || isnan(y);
    float2 om = make_float2(0.f, 0.f), ov = make_float2(0.f, 0.f);
    if (!(isinf(t) || isnan(t) || bad_obs)) {
        om.x = t * (y - m.x);
        ov.x = -t * j.x;
    }
    if (!bad_obs) {
        const float gain = mu_v2 / var_sum;                // cov(y, V) / var(y)
        const float mu_v_pos = gain * (y - m.x);
        const float var_v_pos = mu_v2 - gain * mu_v2;
        const float mu_v2_pos = mu_v_pos * mu_v_pos + var_v_pos;
        const float var_v2_pos =
            2.0f * var_v_pos * var_v_pos + 4.0f * var_v_pos * mu_v_pos * mu_v_pos;
        const float k = v.y / var_v2;
        const float mu_pos = m.y + k * (mu_v2_pos - mu_v2);
        const float var_pos = v.y + k * k * (var_v2_pos - var_v2);
        float jv = j.y / v.y;
        if (isinf(jv) || isnan(jv)) jv = 0.0f;
        om.y = jv * (mu_pos - m.y);
        ov.y = jv * jv * (var_pos - v.y);
    }
    dmu[i] = om;
    dvar[i] = ov;
}

__global__ __launch_bounds__(TPB) void out_update_indexed_kernel(
    const float *__restrict__ mu_a, const float *__restrict__ var_a,
    const float *__restrict__ jcb, const float *__restrict__ obs,
    const float *__restrict__ var_obs, const int *__restrict__ sel, int n_obs, int n_enc, int n,
    float *__restrict__ dmu, float *__restrict__ dvar) {
    const int col = blockIdx.x * TPB + threadIdx.x;
    if (col >= n) return;
    const int idx = sel[col] + (col / n_enc) * n_obs - 1;  // sel is 1-based
    const float t = jcb[idx] / (var_a[idx] + var_obs[col]);
    if (isinf(t) || isnan(t)) {
        dmu[idx] = 0.f;
        dvar[idx] = 0.f;
    } else {
        dmu[idx] = t * (obs[col] - mu_a[idx]);
        dvar[idx] = -t * jcb[idx];
    }
}

// The same with the clearing of the innovation buffers included: workgroup b < samples
// owns sample b's n_obs entries (zeroed, then the selected ones written, in that order
// behind a barrier); the workgroups after those zero the rest of the buffers. The
// observations may lie in pinned host memory (read once each).
__global__ __launch_bounds__(TPB) void out_update_indexed_reset_kernel(
    const float *__restrict__ mu_a, const float *__restrict__ var_a,
    const float *__restrict__ jcb, const float *__restrict__ obs,
    const float *__restrict__ var_obs, const int *__restrict__ sel, int n_obs, int n_enc,
    int samples, float *__restrict__ dmu, float *__restrict__ dvar, size_t delta_len) {
    if ((int)blockIdx.x < samples) {
        const int b = blockIdx.x;
        // ask for the observations first: they may come over the host link
        float y = 0.f, vy = 0.f;
        int s = 0;
        const bool has = (int)threadIdx.x < n_enc;
        if (has) {
            const int col = b * n_enc + threadIdx.x;
            y = obs[col];
            vy = var_obs[col];
            s = sel[col];
        }
        const size_t base = (size_t)b * n_obs;
        for (int i = threadIdx.x; i < n_obs; i += TPB)
            if (base + i < delta_len) {
                dmu[base + i] = 0.f;
                dvar[base + i] = 0.f;
            }
        __syncthreads();
        for (int e = threadIdx.x; e < n_enc; e += TPB) {
            if (e >= TPB) {      // more than one observation per thread: the later ones
                const int col = b * n_enc + e;
                y = obs[col];
                vy = var_obs[col];
                s = sel[col];
            }
            const size_t idx = base + s - 1;  // sel is 1-based
            const float j = jcb[idx];
            const float t = j / (var_a[idx] + vy);
            if (!(isinf(t) || isnan(t))) {
                dmu[idx] = t * (y - mu_a[idx]);
                dvar[idx] = -t * j;
            }
        }
        return;
    }
    const size_t first = (size_t)samples * n_obs;
    const size_t stride = (size_t)(gridDim.x - samples) * TPB;
    for (size_t i = first + (size_t)(blockIdx.x - samples) * TPB + threadIdx.x; i < delta_len;
         i += stride) {
        dmu[i] = 0.f;
        dvar[i] = 0.f;
    }
}

// No __restrict__: the call may run in place (mu_a == mu_z, var_a == var_z).
__global__ __launch_bounds__(TPB) void relu_kernel(const float *mu_z, const float *var_z,
                                                   size_t n, float *mu_a, float *jcb,
                                                   float *var_a) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x;
    if (i >= n) return;
    float m, v, j;
    relu_moments(mu_z[i], var_z[i], m, v, j);
    mu_a[i] = m;
    jcb[i] = j;
    var_a[i] = v;
}

}  // namespace

hipError_t launch_bias_delta(const float *var_b, const float *dmu, const float *dvar, int N,
                             int B, float *dmu_b, float *dvar_b, hipStream_t stream) {
    hipLaunchKernelGGL(bias_delta_kernel, dim3(blocks_for(N, 64)), dim3(64 * BIAS_SLICES), 0, stream, var_b,
                       dmu, dvar, N, B, dmu_b, dvar_b);
    return hipGetLastError();
}

hipError_t launch_store_states(const float *mu_a, const float *jcb, size_t n_in, float *bwd_mu_a,
                               float *bwd_jcb, float *out_jcb, size_t n_out, hipStream_t stream) {
    const size_t n = n_in > n_out ? n_in : n_out;
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(store_states_kernel, dim3(blocks_for(n, TPB)), dim3(TPB), 0, stream, mu_a,
                       jcb, n_in, bwd_mu_a, bwd_jcb, out_jcb, n_out);
    return hipGetLastError();
}

hipError_t launch_param_update(const float *dmu, const float *dvar, float cap, size_t n, float *mu,
                               float *var, int *neg_count, hipStream_t stream) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(param_update_kernel, dim3(blocks_for(n, TPB)), dim3(TPB), 0, stream, dmu,
                       dvar, cap, n, mu, var, neg_count);
    return hipGetLastError();
}

hipError_t launch_param_raw_update(const float *dmu, const float *dvar, size_t n, float *mu,
                                   float *var, hipStream_t stream) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(param_raw_update_kernel, dim3(blocks_for(n, TPB)), dim3(TPB), 0, stream,
                       dmu, dvar, n, mu, var);
    return hipGetLastError();
}

hipError_t launch_layer_update(const float *dmu_w, const float *dvar_w, size_t nw, float *mu_w,
                               float *var_w, const float *dmu_b, const float *dvar_b, size_t nb,
                               float *mu_b, float *var_b, float cap, int *count, int slot,
                               hipStream_t stream) {
    if (nw + nb == 0) return hipSuccess;
    hipLaunchKernelGGL(layer_update_kernel, dim3(blocks_for(nw + nb, TPB)), dim3(TPB), 0, stream,
                       dmu_w, dvar_w, nw, mu_w, var_w, dmu_b, dvar_b, nb, mu_b, var_b, cap, count,
                       slot);
    return hipGetLastError();
}

hipError_t launch_model_update(const ModelUpdateArgs &args, hipStream_t stream) {
    const unsigned blocks = args.first_block[args.n];
    if (args.n == 0 || blocks == 0) return hipSuccess;
    hipLaunchKernelGGL(model_update_kernel, dim3(blocks), dim3(TPB), 0, stream, args);
    return hipGetLastError();
}

hipError_t launch_out_update_dense(const float *mu_a, const float *var_a, const float *jcb,
                                   const float *obs, const float *var_obs, int n, float *dmu,
                                   float *dvar, hipStream_t stream) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(out_update_dense_kernel, dim3(blocks_for(n, TPB)), dim3(TPB), 0, stream,
                       mu_a, var_a, jcb, obs, var_obs, n, dmu, dvar);
    return hipGetLastError();
}

hipError_t launch_out_update_heteros(const float *mu_a, const float *var_a, const float *jcb,
                                     const float *obs, int n, float *dmu, float *dvar,
                                     hipStream_t stream) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(out_update_heteros_kernel, dim3(blocks_for(n, TPB)), dim3(TPB), 0, stream,
                       reinterpret_cast<const float2 *>(mu_a),
                       reinterpret_cast<const float2 *>(var_a),
                       reinterpret_cast<const float2 *>(jcb), obs, n,
                       reinterpret_cast<float2 *>(dmu), reinterpret_cast<float2 *>(dvar));
    return hipGetLastError();
}

hipError_t launch_out_update_indexed(const float *mu_a, const float *var_a, const float *jcb,
                                     const float *obs, const float *var_obs, const int *sel,
                                     int n_obs, int n_enc, int n, float *dmu, float *dvar,
                                     hipStream_t stream) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(out_update_indexed_kernel, dim3(blocks_for(n, TPB)), dim3(TPB), 0, stream,
                       mu_a, var_a, jcb, obs, var_obs, sel, n_obs, n_enc, n, dmu, dvar);
    return hipGetLastError();
}

hipError_t launch_out_update_indexed_reset(const float *mu_a, const float *var_a, const float *jcb,
                                           const float *obs, const float *var_obs, const int *sel,
                                           int n_obs, int n_enc, int samples, float *dmu,
                                           float *dvar, size_t delta_len, hipStream_t stream) {
    const size_t rest = delta_len > (size_t)samples * n_obs ? delta_len - (size_t)samples * n_obs : 0;
    unsigned zero_blocks = blocks_for(rest, 4 * TPB);
    if (zero_blocks > 1024u) zero_blocks = 1024u;
    if (samples + zero_blocks == 0) return hipSuccess;
    hipLaunchKernelGGL(out_update_indexed_reset_kernel, dim3(samples + zero_blocks), dim3(TPB), 0,
                       stream, mu_a, var_a, jcb, obs, var_obs, sel, n_obs, n_enc, samples, dmu,
                       dvar, delta_len);
    return hipGetLastError();
}

hipError_t launch_upload_input(const float *host_mu, const float *host_var, size_t n, float *mu_a,
                               float *var_a, hipStream_t stream) {
    if (n == 0) return hipSuccess;
    const unsigned blocks = blocks_for(n, TPB) < 1024u ? blocks_for(n, TPB) : 1024u;
    hipLaunchKernelGGL(upload_input_kernel, dim3(blocks), dim3(TPB), 0, stream, host_mu, host_var, n,
                       mu_a, var_a);
    return hipGetLastError();
}

hipError_t launch_download_outputs(const float *mu_a, const float *var_a, size_t n, float *host_mu,
                                   float *host_var, unsigned *host_flag, unsigned flag_value,
                                   hipStream_t stream) {
    if (n == 0 && host_flag == nullptr) return hipSuccess;
    unsigned blocks = blocks_for(n, TPB) < 1024u ? blocks_for(n, TPB) : 1024u;
    if (host_flag != nullptr || blocks == 0) blocks = 1;   // the flag follows one workgroup's data
    hipLaunchKernelGGL(download_outputs_kernel, dim3(blocks), dim3(TPB), 0, stream, mu_a, var_a, n,
                       host_mu, host_var, host_flag, flag_value);
    return hipGetLastError();
}

hipError_t launch_relu(const float *mu_z, const float *var_z, size_t n, float *mu_a, float *jcb,
                       float *var_a, hipStream_t stream) {
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(relu_kernel, dim3(blocks_for(n, TPB)), dim3(TPB), 0, stream, mu_z, var_z, n, mu_a,
                       jcb, var_a);
    return hipGetLastError();
}

}  // namespace tagi

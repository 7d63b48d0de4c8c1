// Forward of small Linear layers (reference: linear_fwd_mean_var,
// src/linear_layer.cpp:19-58; device form src/linear_layer_cuda.cu:27-125): the
// layers of the MNIST-sized multilayer perceptrons, whose weight matrices fit the L2
// cache many times over. Such a launch is bound by latency, not by throughput: the
// tiled kernel spends a memory round trip per k-tile in a handful of workgroups, or
// cuts the reduction into slices and pays a second launch to fold them. Here one
// wave owns RN output rows x RB samples and its 64 lanes span the reduction, 16
// bytes each per pass, so that a reduction of 256 elements is a single round of
// loads and the whole chip works on a 128 x 128 layer; the lanes' partial sums meet
// in a butterfly of cross-lane exchanges, and bias and activation are applied before
// the one store. For reductions longer than 256 the four waves of a workgroup share
// one tile and each takes a quarter of every 1024 elements (784 inputs: still one
// round of loads); their sums meet in 512 bytes of LDS. There is no second launch.
#include <hip/hip_runtime.h>

#include "tagi_activation.h"
#include "tagi_internal.h"

namespace tagi {
namespace {

constexpr int SMALL_WAVES = 4;   // waves per workgroup, one tile each

__device__ __forceinline__ float dot4(const float4 a, const float4 b) {
    return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w;
}

// Sums every entry of v[0..V) over the 64 lanes of the wave. Step s halves the
// entries a lane holds: a lane with bit s clear keeps the lower half and receives its
// partner's lower half, the partner keeps the upper halves. After log2(V) steps a
// lane holds one entry (index = the lane's low bits, reversed), summed over the
// lanes that differ in those bits; the remaining lane bits are folded by plain
// exchanges. Returns that entry's total in every lane.
// One v_cndmask per choice, spelled out: written as `upper ? a : b` on elements of the
// array the compiler turns the choice into an index and the access into a chain of
// sixteen selects.
__device__ __forceinline__ float pick(float if_clear, float if_set, unsigned long long set_lanes) {
    float r;
    asm("v_cndmask_b32_e64 %0, %1, %2, %3" : "=v"(r) : "v"(if_clear), "v"(if_set), "s"(set_lanes));
    return r;
}

template <int V>
__device__ __forceinline__ float butterfly_sum(float (&v)[V], int lane) {
    int step = 0;
#pragma unroll
    for (int n = V; n > 1; n >>= 1, step++) {
        const unsigned long long upper = __ballot((lane >> step) & 1);
#pragma unroll
        for (int i = 0; i < n / 2; i++) {
            const float send = pick(v[i + n / 2], v[i], upper);
            const float keep = pick(v[i], v[i + n / 2], upper);
            v[i] = keep + __shfl_xor(send, 1 << step);
        }
    }
    float total = v[0];
#pragma unroll
    for (int m = V; m < 64; m <<= 1) total += __shfl_xor(total, m);
    return total;
}

// KW: waves that share a tile's reduction (1 or SMALL_WAVES)
template <int RN, int RB, int KW>
__global__ __launch_bounds__(SMALL_WAVES * 64) void small_fwd_kernel(
    const float *__restrict__ mu_w, const float *__restrict__ var_w,
    const float *__restrict__ mu_b, const float *__restrict__ var_b,
    const float *__restrict__ mu_a, const float *__restrict__ var_a, int K, int N, int B, int act,
    float *__restrict__ out0, float *__restrict__ out1, float *__restrict__ out2) {
    constexpr int V = RN * RB;
    static_assert(V <= 64 && (V & (V - 1)) == 0, "one entry per lane after the butterfly");
    static_assert(KW == 1 || KW == SMALL_WAVES, "a tile belongs to one wave or to the workgroup");
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sample_tiles = (B + RB - 1) / RB;
    const int tile = KW == 1 ? blockIdx.x * SMALL_WAVES + wave : blockIdx.x;
    // uniform over the waves that meet at the barrier below (KW > 1: the whole workgroup)
    if (tile >= ((N + RN - 1) / RN) * sample_tiles) return;
    // consecutive tiles share their rows: the weights are fetched into the CU's cache once
    const int n0 = (tile / sample_tiles) * RN, b0 = (tile % sample_tiles) * RB;

    // the entry this lane holds after the butterfly: its low bits, reversed
    int idx = 0;
#pragma unroll
    for (int s = 0, n = V; n > 1; n >>= 1, s++) idx |= ((lane >> s) & 1) * (n >> 1);
    const int out_n = n0 + idx / RB, out_b = b0 + idx % RB;
    const bool writes = lane < V && out_n < N && out_b < B && (KW == 1 || wave == 0);

    const float *wm_row[RN], *wv_row[RN], *xm_row[RB], *xv_row[RB];
#pragma unroll
    for (int r = 0; r < RN; r++) {
        const size_t row = (size_t)min(n0 + r, N - 1) * K;    // rows past the end: recomputed,
        wm_row[r] = mu_w + row;                               // never stored
        wv_row[r] = var_w + row;
    }
#pragma unroll
    for (int b = 0; b < RB; b++) {
        const size_t row = (size_t)min(b0 + b, B - 1) * K;
        xm_row[b] = mu_a + row;
        xv_row[b] = var_a + row;
    }

    float sum_mu[V], sum_var[V];
#pragma unroll
    for (int i = 0; i < V; i++) sum_mu[i] = sum_var[i] = 0.f;
    // One lane adds the bias to its sums, in its first pass: the bias is then asked for
    // together with that pass's other loads instead of in a memory round trip of its own
    // before or after the reduction.
    bool bias_pending = mu_b != nullptr && lane == 0 && (KW == 1 || wave == 0);

    for (int k = 4 * (KW == 1 ? lane : wave * 64 + lane); k < K; k += 256 * KW) {
        float4 wm[RN], wv[RN], ws[RN];
#pragma unroll
        for (int r = 0; r < RN; r++) {
            wm[r] = *reinterpret_cast<const float4 *>(wm_row[r] + k);
            wv[r] = *reinterpret_cast<const float4 *>(wv_row[r] + k);
        }
        float4 xm[RB], xv[RB];
#pragma unroll
        for (int b = 0; b < RB; b++) {
            xm[b] = *reinterpret_cast<const float4 *>(xm_row[b] + k);
            xv[b] = *reinterpret_cast<const float4 *>(xv_row[b] + k);
        }
        float bias_mu[RN], bias_var[RN];
#pragma unroll
        for (int r = 0; r < RN; r++) {
            bias_mu[r] = bias_var[r] = 0.f;
            if (bias_pending) {
                bias_mu[r] = mu_b[min(n0 + r, N - 1)];
                bias_var[r] = var_b[min(n0 + r, N - 1)];
            }
        }
        bias_pending = false;
        // every load of the pass is in flight before the first use: one memory round
        // trip per pass (the scheduler would otherwise interleave loads and products
        // to save registers, and wait for each load in turn)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = 0; r < RN; r++)
            ws[r] = make_float4(wm[r].x * wm[r].x + wv[r].x, wm[r].y * wm[r].y + wv[r].y,
                                wm[r].z * wm[r].z + wv[r].z, wm[r].w * wm[r].w + wv[r].w);
#pragma unroll
        for (int b = 0; b < RB; b++) {
            const float4 sq = make_float4(xm[b].x * xm[b].x, xm[b].y * xm[b].y,
                                          xm[b].z * xm[b].z, xm[b].w * xm[b].w);
#pragma unroll
            for (int r = 0; r < RN; r++) {
                // var_z = sum (mu_w^2 + var_w) var_a + var_w mu_a^2
                sum_mu[r * RB + b] += dot4(wm[r], xm[b]) + bias_mu[r];
                sum_var[r * RB + b] += dot4(ws[r], xv[b]) + dot4(wv[r], sq) + bias_var[r];
            }
        }
    }

    float mu = butterfly_sum<V>(sum_mu, lane);
    float var = butterfly_sum<V>(sum_var, lane);
    if constexpr (KW > 1) {
        __shared__ float part[KW][2][V];
        if (lane < V) {
            part[wave][0][lane] = mu;
            part[wave][1][lane] = var;
        }
        __syncthreads();
        if (writes) {
            mu = var = 0.f;
#pragma unroll
            for (int w = 0; w < KW; w++) {       // in wave order: deterministic
                mu += part[w][0][lane];
                var += part[w][1][lane];
            }
        }
    }
    if (writes)
        store_activated(act, mu, var, (size_t)out_b * N + out_n, out0, out1, out2);
}

}  // namespace

// Layers this kernel is meant for: up to 64 samples and up to 2^18 weights (512^2),
// where a 2-row tile's repeated reads of the activations stay small.
bool small_fwd_supported(int K, int N, int B) {
    return B <= 64 && K % 4 == 0 && (long long)N * K <= (1ll << 18);
}

// All pointers 16-byte aligned and K % 4 == 0 (the caller checks); mu_b / var_b may be
// null; act / out2 as in GemmParams.
hipError_t launch_small_fwd(const float *mu_w, const float *var_w, const float *mu_b,
                            const float *var_b, const float *mu_a, const float *var_a, int K,
                            int N, int B, int act, float *out0, float *out1, float *out2,
                            hipStream_t stream) {
    if (K % 4 != 0 || K <= 0 || N <= 0 || B <= 0) return hipErrorInvalidValue;
    constexpr int RN = 2, RB = 8;
    const int tiles = ((N + RN - 1) / RN) * ((B + RB - 1) / RB);
    dim3 block(SMALL_WAVES * 64);
    if (K <= 256)
        hipLaunchKernelGGL((small_fwd_kernel<RN, RB, 1>), dim3((tiles + SMALL_WAVES - 1) / SMALL_WAVES),
                           block, 0, stream, mu_w, var_w, mu_b, var_b, mu_a, var_a, K, N, B, act,
                           out0, out1, out2);
    else
        hipLaunchKernelGGL((small_fwd_kernel<RN, RB, SMALL_WAVES>), dim3(tiles), block, 0, stream,
                           mu_w, var_w, mu_b, var_b, mu_a, var_a, K, N, B, act, out0, out1, out2);
    return hipGetLastError();
}

}  // namespace tagi

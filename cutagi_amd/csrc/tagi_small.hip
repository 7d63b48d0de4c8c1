// Small Linear layers in one launch per pass. Forward (reference: linear_fwd_mean_var,
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
// The code is kept short on purpose: a kernel this brief runs cold, and fetching its
// instructions is part of its latency (the first version of the butterfly, compiled to
// select chains, made the launch twice as long).
//
// The two backward kernels below follow the same rule - every load of a pass in flight
// before the first use, no second launch: the state backward (linear_bwd_fc_delta_z,
// src/linear_layer.cpp:180-219) splits the sum over the output units over eight slices
// of a workgroup, and the weight backward (linear_bwd_fc_delta_w / _b,
// src/linear_layer.cpp:221-327) needs no reduction across threads at all (the sum runs
// over the batch) and writes the bias innovations on the side.
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

// ---- state backward ---------------------------------------------------------------
// delta_mu_z[b][k] = jcb[b][k] sum_n mu_w[n][k] delta_mu[b][n], delta_var_z with mu_w^2
// and jcb^2. Workgroup = one sample x 128 input units (32 lanes of 16 bytes) x 8 slices
// of the output units; slice s takes the units s, s + 8, ...
constexpr int DZ_LANES = 32, DZ_SLICES = 8, DZ_BATCH = 16;

// (bx, b): column block and sample of the workgroup; red: 8 KB of LDS
__device__ __forceinline__ void small_dz_block(
    const float *__restrict__ mu_w, const float *__restrict__ jcb,
    const float *__restrict__ dmu, const float *__restrict__ dvar, int K, int N,
    float *__restrict__ out_mu, float *__restrict__ out_var, int bx, int b,
    float (*red)[DZ_LANES][8]) {
    const int kl = threadIdx.x & (DZ_LANES - 1), slice = threadIdx.x / DZ_LANES;
    const int k = (bx * DZ_LANES + kl) * 4;
    const bool valid = k < K;
    const float *w_col = mu_w + (valid ? k : 0);
    const float *dm_row = dmu + (size_t)b * N, *dv_row = dvar + (size_t)b * N;
    // after the sums: thread t folds entry t % 8 of lane t / 8 over the slices. Its
    // Jacobian is asked for now, not in a memory round trip of its own at the end.
    const int kl2 = threadIdx.x >> 3, c = threadIdx.x & 7;
    const int k2 = (bx * DZ_LANES + kl2) * 4 + (c & 3);
    const size_t at = (size_t)b * K + min(k2, K - 1);
    const float j = jcb[at];
    float4 m = make_float4(0.f, 0.f, 0.f, 0.f), v = m;
    for (int n0 = slice; n0 < N; n0 += DZ_SLICES * DZ_BATCH) {
        float4 w[DZ_BATCH];
        float d[DZ_BATCH], dv[DZ_BATCH];
#pragma unroll
        for (int u = 0; u < DZ_BATCH; u++) {
            const int n = n0 + u * DZ_SLICES;
            const int row = min(n, N - 1);          // rows past the end: read, weighted by zero
            w[u] = *reinterpret_cast<const float4 *>(w_col + (size_t)row * K);
            d[u] = dm_row[row];
            dv[u] = dv_row[row];
        }
        __builtin_amdgcn_sched_barrier(0);          // all loads of the batch before any use
#pragma unroll
        for (int u = 0; u < DZ_BATCH; u++) {
            if (n0 + u * DZ_SLICES >= N) d[u] = dv[u] = 0.f;
            m.x += w[u].x * d[u]; m.y += w[u].y * d[u]; m.z += w[u].z * d[u]; m.w += w[u].w * d[u];
            v.x += w[u].x * w[u].x * dv[u]; v.y += w[u].y * w[u].y * dv[u];
            v.z += w[u].z * w[u].z * dv[u]; v.w += w[u].w * w[u].w * dv[u];
        }
    }
    *reinterpret_cast<float4 *>(&red[slice][kl][0]) = m;
    *reinterpret_cast<float4 *>(&red[slice][kl][4]) = v;
    __syncthreads();
    if (k2 >= K) return;
    float sum = 0.f;
#pragma unroll
    for (int s2 = 0; s2 < DZ_SLICES; s2++) sum += red[s2][kl2][c];      // in slice order
    if (c < 4)
        out_mu[at] = sum * j;
    else
        out_var[at] = sum * j * j;
}

__global__ __launch_bounds__(DZ_LANES * DZ_SLICES) void small_dz_kernel(
    const float *__restrict__ mu_w, const float *__restrict__ jcb,
    const float *__restrict__ dmu, const float *__restrict__ dvar, int K, int N,
    float *__restrict__ out_mu, float *__restrict__ out_var) {
    __shared__ float red[DZ_SLICES][DZ_LANES][8];
    small_dz_block(mu_w, jcb, dmu, dvar, K, N, out_mu, out_var, blockIdx.x, blockIdx.y, red);
}

// ---- weight backward ----------------------------------------------------------------
// delta_mu_w[n][k] = var_w[n][k] sum_b mu_a[b][k] delta_mu[b][n], delta_var_w with
// var_w^2, mu_a^2 and delta_var; thread = DW_ROWS output units x 4 input units, DW_BATCH
// samples per round of loads (2 x 16 up to 16 samples, 1 x 32 beyond). The
// thread of a row's first input units also has that row's sum of delta over the batch:
// the bias innovations (x var_b, x var_b^2).
constexpr int DW_TPB = 256;

template <int DW_ROWS, int DW_BATCH>
__device__ __forceinline__ void small_dw_block(
    const float *__restrict__ var_w, const float *__restrict__ mu_a,
    const float *__restrict__ dmu, const float *__restrict__ dvar, int K, int N, int B,
    float *__restrict__ dmu_w, float *__restrict__ dvar_w, const float *__restrict__ var_b,
    float *__restrict__ dmu_b, float *__restrict__ dvar_b, int block) {
    const int K4 = K >> 2;
    const int item = block * DW_TPB + threadIdx.x;
    if (item >= ((N + DW_ROWS - 1) / DW_ROWS) * K4) return;
    const int n0 = (item / K4) * DW_ROWS, k = (item % K4) * 4;
    int row[DW_ROWS];
    float4 vw[DW_ROWS], am[DW_ROWS], av[DW_ROWS];
    float bm[DW_ROWS], bv[DW_ROWS];
#pragma unroll
    for (int r = 0; r < DW_ROWS; r++) {
        row[r] = min(n0 + r, N - 1);
        vw[r] = *reinterpret_cast<const float4 *>(var_w + (size_t)row[r] * K + k);
        am[r] = av[r] = make_float4(0.f, 0.f, 0.f, 0.f);
        bm[r] = bv[r] = 0.f;
    }
    for (int b0 = 0; b0 < B; b0 += DW_BATCH) {
        float4 a[DW_BATCH];
        float d[DW_BATCH][DW_ROWS], dv[DW_BATCH][DW_ROWS];
#pragma unroll
        for (int u = 0; u < DW_BATCH; u++) {
            const int b = min(b0 + u, B - 1);       // samples past the end: weighted by zero
            a[u] = *reinterpret_cast<const float4 *>(mu_a + (size_t)b * K + k);
#pragma unroll
            for (int r = 0; r < DW_ROWS; r++) {
                d[u][r] = dmu[(size_t)b * N + row[r]];
                dv[u][r] = dvar[(size_t)b * N + row[r]];
            }
        }
        __builtin_amdgcn_sched_barrier(0);          // all loads of the batch before any use
#pragma unroll
        for (int u = 0; u < DW_BATCH; u++) {
            if (b0 + u >= B) {
#pragma unroll
                for (int r = 0; r < DW_ROWS; r++) d[u][r] = dv[u][r] = 0.f;
            }
            const float4 sq = make_float4(a[u].x * a[u].x, a[u].y * a[u].y, a[u].z * a[u].z,
                                          a[u].w * a[u].w);
#pragma unroll
            for (int r = 0; r < DW_ROWS; r++) {
                am[r].x += a[u].x * d[u][r]; am[r].y += a[u].y * d[u][r];
                am[r].z += a[u].z * d[u][r]; am[r].w += a[u].w * d[u][r];
                av[r].x += sq.x * dv[u][r]; av[r].y += sq.y * dv[u][r];
                av[r].z += sq.z * dv[u][r]; av[r].w += sq.w * dv[u][r];
                bm[r] += d[u][r];
                bv[r] += dv[u][r];
            }
        }
    }
#pragma unroll
    for (int r = 0; r < DW_ROWS; r++) {
        if (n0 + r >= N) break;
        const size_t at = (size_t)row[r] * K + k;
        *reinterpret_cast<float4 *>(dmu_w + at) =
            make_float4(am[r].x * vw[r].x, am[r].y * vw[r].y, am[r].z * vw[r].z, am[r].w * vw[r].w);
        *reinterpret_cast<float4 *>(dvar_w + at) =
            make_float4(av[r].x * vw[r].x * vw[r].x, av[r].y * vw[r].y * vw[r].y,
                        av[r].z * vw[r].z * vw[r].z, av[r].w * vw[r].w * vw[r].w);
        if (k == 0 && var_b != nullptr) {
            const float vb = var_b[row[r]];
            dmu_b[row[r]] = bm[r] * vb;
            dvar_b[row[r]] = bv[r] * vb * vb;
        }
    }
}

template <int DW_ROWS, int DW_BATCH>
__global__ __launch_bounds__(DW_TPB) void small_dw_kernel(
    const float *__restrict__ var_w, const float *__restrict__ mu_a,
    const float *__restrict__ dmu, const float *__restrict__ dvar, int K, int N, int B,
    float *__restrict__ dmu_w, float *__restrict__ dvar_w, const float *__restrict__ var_b,
    float *__restrict__ dmu_b, float *__restrict__ dvar_b) {
    small_dw_block<DW_ROWS, DW_BATCH>(var_w, mu_a, dmu, dvar, K, N, B, dmu_w, dvar_w, var_b, dmu_b,
                                      dvar_b, blockIdx.x);
}

// Both backward kernels of a layer as one grid: the first blocks_z workgroups are the
// state backward's (column block, sample) pairs, the rest the weight backward's. The two
// read the same innovations and do not depend on each other; at these sizes a launch
// costs more than what it computes.
struct SmallBwdArgs {
    const float *mu_w, *var_w, *mu_a, *jcb, *dmu, *dvar, *var_b;
    float *out_mu, *out_var, *dmu_w, *dvar_w, *dmu_b, *dvar_b;
    int K, N, B, blocks_z, blocks_zx;
};
static_assert(DZ_LANES * DZ_SLICES == DW_TPB, "one workgroup size for both parts");

template <int DW_ROWS, int DW_BATCH>
__global__ __launch_bounds__(DW_TPB) void small_bwd_pair_kernel(SmallBwdArgs a) {
    __shared__ float red[DZ_SLICES][DZ_LANES][8];
    const int id = blockIdx.x;
    if (id < a.blocks_z)
        small_dz_block(a.mu_w, a.jcb, a.dmu, a.dvar, a.K, a.N, a.out_mu, a.out_var,
                       id % a.blocks_zx, id / a.blocks_zx, red);
    else
        small_dw_block<DW_ROWS, DW_BATCH>(a.var_w, a.mu_a, a.dmu, a.dvar, a.K, a.N, a.B, a.dmu_w,
                                          a.dvar_w, a.var_b, a.dmu_b, a.dvar_b, id - a.blocks_z);
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

// The backward kernels: the same layers (K % 4 == 0; mu_w / var_w / mu_a and the weight
// innovations 16-byte aligned, which the caller checks).
bool small_bwd_supported(int K, int N, int B) { return small_fwd_supported(K, N, B); }
// The weight backward: 9..32 samples (up to 8 the streaming kernel is quicker, beyond 32
// the tiled one).
bool small_dw_supported(int K, int N, int B) {
    return B > 8 && B <= 32 && small_bwd_supported(K, N, B);
}

hipError_t launch_small_dz(const float *mu_w, const float *jcb, const float *dmu, const float *dvar,
                           int K, int N, int B, float *out_mu, float *out_var,
                           hipStream_t stream) {
    if (K % 4 != 0 || K <= 0 || N <= 0 || B <= 0 || B > 65535) return hipErrorInvalidValue;
    dim3 grid(((K >> 2) + DZ_LANES - 1) / DZ_LANES, B), block(DZ_LANES * DZ_SLICES);
    hipLaunchKernelGGL(small_dz_kernel, grid, block, 0, stream, mu_w, jcb, dmu, dvar, K, N, out_mu,
                       out_var);
    return hipGetLastError();
}

// var_b null: no bias innovations (dmu_b / dvar_b unused).
hipError_t launch_small_dw(const float *var_w, const float *mu_a, const float *dmu,
                           const float *dvar, int K, int N, int B, float *dmu_w, float *dvar_w,
                           const float *var_b, float *dmu_b, float *dvar_b, hipStream_t stream) {
    if (K % 4 != 0 || K <= 0 || N <= 0 || B <= 0) return hipErrorInvalidValue;
    if (B <= 16) {
        const int items = ((N + 1) / 2) * (K >> 2);
        hipLaunchKernelGGL((small_dw_kernel<2, 16>), dim3((items + DW_TPB - 1) / DW_TPB), dim3(DW_TPB),
                           0, stream, var_w, mu_a, dmu, dvar, K, N, B, dmu_w, dvar_w, var_b, dmu_b,
                           dvar_b);
    } else {
        const int items = N * (K >> 2);
        hipLaunchKernelGGL((small_dw_kernel<1, 32>), dim3((items + DW_TPB - 1) / DW_TPB), dim3(DW_TPB),
                           0, stream, var_w, mu_a, dmu, dvar, K, N, B, dmu_w, dvar_w, var_b, dmu_b,
                           dvar_b);
    }
    return hipGetLastError();
}

// State and weight backward (+ bias innovations when var_b is given) of a layer for which
// small_bwd_supported and small_dw_supported hold, in one launch.
hipError_t launch_small_bwd_pair(const float *mu_w, const float *var_w, const float *mu_a,
                                 const float *jcb, const float *dmu, const float *dvar, int K, int N,
                                 int B, float *out_mu, float *out_var, float *dmu_w, float *dvar_w,
                                 const float *var_b, float *dmu_b, float *dvar_b,
                                 hipStream_t stream) {
    if (K % 4 != 0 || K <= 0 || N <= 0 || B <= 0) return hipErrorInvalidValue;
    SmallBwdArgs a;
    a.mu_w = mu_w; a.var_w = var_w; a.mu_a = mu_a; a.jcb = jcb; a.dmu = dmu; a.dvar = dvar;
    a.var_b = var_b; a.out_mu = out_mu; a.out_var = out_var; a.dmu_w = dmu_w; a.dvar_w = dvar_w;
    a.dmu_b = dmu_b; a.dvar_b = dvar_b; a.K = K; a.N = N; a.B = B;
    a.blocks_zx = ((K >> 2) + DZ_LANES - 1) / DZ_LANES;
    a.blocks_z = a.blocks_zx * B;
    if (B <= 16) {
        const int items = ((N + 1) / 2) * (K >> 2);
        hipLaunchKernelGGL((small_bwd_pair_kernel<2, 16>), dim3(a.blocks_z + (items + DW_TPB - 1) / DW_TPB),
                           dim3(DW_TPB), 0, stream, a);
    } else {
        const int items = N * (K >> 2);
        hipLaunchKernelGGL((small_bwd_pair_kernel<1, 32>), dim3(a.blocks_z + (items + DW_TPB - 1) / DW_TPB),
                           dim3(DW_TPB), 0, stream, a);
    }
    return hipGetLastError();
}

}  // namespace tagi

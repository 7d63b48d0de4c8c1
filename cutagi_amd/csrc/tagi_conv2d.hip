// TAGI Conv2d as implicit GEMMs on the fp32 MFMA tile core, gfx950. The im2col
// matrix is never materialised: the reference's index tables are applied while
// an operand tile is staged into LDS.
//
//   forward   D[fo][(b,o)]   = sum_{(c,t)}  w[fo][c][t] * a[b][c][Fmwa_2[o][t]]
//   weights   D[fo][(c,t)]   = sum_{(b,o)}  delta[b][fo][o] * a[b][c][Fmwa_2[o][t]]
//   states    D[c][(b,p)]    = sum_{(fo,t)} w[fo][c][t] * delta[b][fo][inv[t][p]]
//
// with o an output pixel, p an input pixel, t a kernel tap, and inv[t][p] the
// output pixel whose tap t lands on input pixel p (or none). `inv` is the same
// information as the reference's FCzwa_1 / Szz_ud pair (per input pixel, the
// list of (tap, output pixel) occurrences), re-keyed by tap so that the weight
// operand of the state backward does not depend on the pixel and the contraction
// is a plain GEMM. The permutations the reference runs as separate passes
// (Jacobian, deltas) are folded into the operand addressing.
#include "tagi_internal.h"
#include "tagi_mfma_tile.h"

namespace tagi {
namespace {

struct ConvParams {
    const float *w0, *w1;  // mu_w, var_w        [fo][fi*k2]
    const float *a0, *a1;  // mu_a, var_a        [B][fi][wihi]
    const float *d0, *d1;  // delta_mu, delta_var [B][fo][woho]
    const float *e0, *e1;  // forward: mu_b, var_b [fo] (or null); states: jcb; weights: var_w
    const int *idx;        // forward/weights: Fmwa_2 [woho][k2]; states: inv [k2][wihi]
    float *out0, *out1;
    int woho, fo, wihi, fi, k2, B;
    int M, N, R, splits, r_per_split;
    float *ws0, *ws1;
};

template <bool VEC>
__device__ __forceinline__ float4 load_rows_kc(const float *__restrict__ base, int ld, int row,
                                               int rows, int r, int r_end) {
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (row >= rows) return v;
    if (VEC) {
        if (r < r_end) v = *reinterpret_cast<const float4 *>(base + (size_t)row * ld + r);
    } else {
        float c[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (r + j < r_end) c[j] = base[(size_t)row * ld + r + j];
        v = make_float4(c[0], c[1], c[2], c[3]);
    }
    return v;
}

// ---- forward ---------------------------------------------------------------
// rows: weights [fo][R] (k-contiguous); columns: gathered activations, staged
// [k][pixel] so that consecutive lanes read consecutive pixels.
template <bool VEC>
struct ConvFwdProblem {
    using Params = ConvParams;
    static constexpr bool XK = true, YK = false;
    static constexpr int NX = 2, NY = 2, FLAVOR = FLAVOR_FWD_W_ROWS;

    __device__ static __forceinline__ float4 load_x(const Params &p, int arr, int m, int r,
                                                    int r_end) {
        return load_rows_kc<VEC>(arr ? p.w1 : p.w0, p.R, m, p.M, r, r_end);
    }
    __device__ static __forceinline__ float4 load_y(const Params &p, int arr, int n, int r,
                                                    int r_end) {
        float c[4] = {0.f, 0.f, 0.f, 0.f};
        if (r < r_end) {
            const float *__restrict__ act = arr ? p.a1 : p.a0;
            const int ch = r / p.k2, t = r - ch * p.k2;
            int b = n / p.woho, o = n - b * p.woho;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if (n + j < p.N) {
                    const int a = p.idx[o * p.k2 + t];
                    if (a > -1) c[j] = act[((size_t)b * p.fi + ch) * p.wihi + a - 1];
                }
                if (++o == p.woho) {
                    o = 0;
                    b++;
                }
            }
        }
        return make_float4(c[0], c[1], c[2], c[3]);
    }
    __device__ static __forceinline__ void store(const Params &p, int m, int n, float a0,
                                                 float a1) {
        const int b = n / p.woho, o = n - b * p.woho;
        const size_t at = ((size_t)b * p.fo + m) * p.woho + o;
        if (p.e0 != nullptr) {
            a0 += p.e0[m];
            a1 += p.e1[m];
        }
        p.out0[at] = a0;
        p.out1[at] = a1;
    }
};

// ---- weight backward ---------------------------------------------------------
// rows: deltas [fo][(b,o)]; columns: gathered activations [(c,t)][(b,o)]; both
// have the reduction (b,o) as their fast index.
template <bool VEC>
struct ConvDwProblem {
    using Params = ConvParams;
    static constexpr bool XK = true, YK = true;
    static constexpr int NX = 2, NY = 1, FLAVOR = FLAVOR_DELTA_ROWS;

    __device__ static __forceinline__ float4 load_x(const Params &p, int arr, int m, int r,
                                                    int r_end) {
        float c[4] = {0.f, 0.f, 0.f, 0.f};
        if (m < p.M && r < r_end) {
            const float *__restrict__ d = arr ? p.d1 : p.d0;
            int b = r / p.woho, o = r - b * p.woho;
            if (VEC) {  // woho % 4 == 0: the four positions share the image
                return *reinterpret_cast<const float4 *>(d + ((size_t)b * p.fo + m) * p.woho + o);
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if (r + j < r_end) c[j] = d[((size_t)b * p.fo + m) * p.woho + o];
                if (++o == p.woho) {
                    o = 0;
                    b++;
                }
            }
        }
        return make_float4(c[0], c[1], c[2], c[3]);
    }
    __device__ static __forceinline__ float4 load_y(const Params &p, int arr, int n, int r,
                                                    int r_end) {
        float c[4] = {0.f, 0.f, 0.f, 0.f};
        if (n < p.N && r < r_end) {
            const int ch = n / p.k2, t = n - ch * p.k2;
            int b = r / p.woho, o = r - b * p.woho;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if (r + j < r_end) {
                    const int a = p.idx[o * p.k2 + t];
                    if (a > -1) c[j] = p.a0[((size_t)b * p.fi + ch) * p.wihi + a - 1];
                }
                if (++o == p.woho) {
                    o = 0;
                    b++;
                }
            }
        }
        return make_float4(c[0], c[1], c[2], c[3]);
    }
    __device__ static __forceinline__ void store(const Params &p, int m, int n, float a0,
                                                 float a1) {
        const size_t at = (size_t)m * p.N + n;
        const float e = p.e0[at];
        p.out0[at] = a0 * e;
        p.out1[at] = a1 * e * e;
    }
};

// ---- state backward -----------------------------------------------------------
// rows: weights re-indexed [c][(fo,t)]; columns: gathered deltas [(fo,t)][(b,p)].
struct ConvDzProblem {
    using Params = ConvParams;
    static constexpr bool XK = true, YK = false;
    static constexpr int NX = 1, NY = 2, FLAVOR = FLAVOR_DELTA_COLS;

    __device__ static __forceinline__ float4 load_x(const Params &p, int, int m, int r,
                                                    int r_end) {
        float c[4] = {0.f, 0.f, 0.f, 0.f};
        if (m < p.M) {
            int f = r / p.k2, t = r - f * p.k2;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if (r + j < r_end) c[j] = p.w0[((size_t)f * p.fi + m) * p.k2 + t];
                if (++t == p.k2) {
                    t = 0;
                    f++;
                }
            }
        }
        return make_float4(c[0], c[1], c[2], c[3]);
    }
    __device__ static __forceinline__ float4 load_y(const Params &p, int arr, int n, int r,
                                                    int r_end) {
        float c[4] = {0.f, 0.f, 0.f, 0.f};
        if (r < r_end) {
            const float *__restrict__ d = arr ? p.d1 : p.d0;
            const int f = r / p.k2, t = r - f * p.k2;
            int b = n / p.wihi, px = n - b * p.wihi;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if (n + j < p.N) {
                    const int o = p.idx[t * p.wihi + px];
                    if (o > -1) c[j] = d[((size_t)b * p.fo + f) * p.woho + o];
                }
                if (++px == p.wihi) {
                    px = 0;
                    b++;
                }
            }
        }
        return make_float4(c[0], c[1], c[2], c[3]);
    }
    __device__ static __forceinline__ void store(const Params &p, int m, int n, float a0,
                                                 float a1) {
        const int b = n / p.wihi, px = n - b * p.wihi;
        const size_t at = ((size_t)b * p.fi + m) * p.wihi + px;
        const float e = p.e0[at];
        p.out0[at] = a0 * e;
        p.out1[at] = a1 * e * e;
    }
};

// inv[t][p] = 0-based output pixel whose tap t reads input pixel p, else -1,
// from FCzwa_1 (zw, [wihi][nr], 1-based taps) and Szz_ud (zud, [nr][wihi],
// 1-based output pixels, -1 = none).
__global__ __launch_bounds__(256) void conv_inv_fill_kernel(int *inv, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) inv[i] = -1;
}
__global__ __launch_bounds__(256) void conv_inv_build_kernel(const int *__restrict__ zw,
                                                             const int *__restrict__ zud, int wihi,
                                                             int nr, int k2, int *inv) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= wihi * nr) return;
    const int px = i / nr, j = i - px * nr;
    const int tap = zw[px * nr + j], o = zud[j * wihi + px];
    if (o > -1 && tap >= 1 && tap <= k2) inv[(tap - 1) * wihi + px] = o - 1;
}

// Bias innovation: per-channel sums over (b, o) in two stages.
__global__ __launch_bounds__(256) void conv_bias_partial_kernel(const float *__restrict__ dmu,
                                                                const float *__restrict__ dvar,
                                                                int B, int fo, int woho,
                                                                int chunks, float *part0,
                                                                float *part1) {
    __shared__ float s0[256], s1[256];
    const int f = blockIdx.x, chunk = blockIdx.y;
    const long total = (long)B * woho;
    const long per = (total + chunks - 1) / chunks;
    const long lo = chunk * per, hi = min(total, lo + per);
    float a0 = 0.f, a1 = 0.f;
    for (long q = lo + threadIdx.x; q < hi; q += 256) {
        const long b = q / woho, o = q - b * woho;
        const size_t at = ((size_t)b * fo + f) * woho + o;
        a0 += dmu[at];
        a1 += dvar[at];
    }
    s0[threadIdx.x] = a0;
    s1[threadIdx.x] = a1;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) {
            s0[threadIdx.x] += s0[threadIdx.x + s];
            s1[threadIdx.x] += s1[threadIdx.x + s];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        part0[chunk * fo + f] = s0[0];
        part1[chunk * fo + f] = s1[0];
    }
}
__global__ __launch_bounds__(64) void conv_bias_final_kernel(const float *__restrict__ part0,
                                                             const float *__restrict__ part1,
                                                             const float *__restrict__ var_b,
                                                             int fo, int chunks, float *dmu_b,
                                                             float *dvar_b) {
    const int f = blockIdx.x * 64 + threadIdx.x;
    if (f >= fo) return;
    float a0 = 0.f, a1 = 0.f;
    for (int c = 0; c < chunks; c++) {
        a0 += part0[c * fo + f];
        a1 += part1[c * fo + f];
    }
    const float v = var_b[f];
    dmu_b[f] = a0 * v;
    dvar_b[f] = a1 * v * v;
}

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline bool aligned16(const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; }

}  // namespace

hipError_t launch_conv2d_fwd(const float *mu_w, const float *var_w, const float *mu_b,
                             const float *var_b, const float *mu_a, const float *var_a,
                             const int *aidx, int woho, int fo, int wihi, int fi, int ki, int B,
                             int bias, float *mu_z, float *var_z, hipStream_t stream) {
    ConvParams p = {};
    p.w0 = mu_w; p.w1 = var_w; p.a0 = mu_a; p.a1 = var_a;
    p.e0 = bias ? mu_b : nullptr; p.e1 = bias ? var_b : nullptr;
    p.idx = aidx; p.out0 = mu_z; p.out1 = var_z;
    p.woho = woho; p.fo = fo; p.wihi = wihi; p.fi = fi; p.k2 = ki * ki; p.B = B;
    p.M = fo; p.N = B * woho; p.R = p.k2 * fi; p.splits = 1;
    p.r_per_split = ceil_div(p.R, KT) * KT;
    const int tile = fo > 64 ? TILE_128x128 : fo > 32 ? TILE_64x128 : TILE_32x128;
    const bool vec = (p.R % 4 == 0) && aligned16(mu_w) && aligned16(var_w);
    if (vec) return launch_tiles<ConvFwdProblem<true>>(tile, p, stream);
    return launch_tiles<ConvFwdProblem<false>>(tile, p, stream);
}

// `scratch` holds ki*ki*wihi ints for the re-keyed table.
hipError_t launch_conv2d_bwd_dz(const float *mu_w, const float *jcb, const float *dmu,
                                const float *dvar, const int *zw_idx, const int *zud_idx,
                                int woho, int fo, int wihi, int fi, int ki, int nr, int B,
                                int *scratch, float *out_dmu, float *out_dvar,
                                hipStream_t stream) {
    const int k2 = ki * ki;
    hipLaunchKernelGGL(conv_inv_fill_kernel, dim3(ceil_div(k2 * wihi, 256)), dim3(256), 0, stream,
                       scratch, k2 * wihi);
    hipLaunchKernelGGL(conv_inv_build_kernel, dim3(ceil_div(nr * wihi, 256)), dim3(256), 0, stream,
                       zw_idx, zud_idx, wihi, nr, k2, scratch);
    ConvParams p = {};
    p.w0 = mu_w; p.d0 = dmu; p.d1 = dvar; p.e0 = jcb; p.idx = scratch;
    p.out0 = out_dmu; p.out1 = out_dvar;
    p.woho = woho; p.fo = fo; p.wihi = wihi; p.fi = fi; p.k2 = k2; p.B = B;
    p.M = fi; p.N = B * wihi; p.R = k2 * fo; p.splits = 1;
    p.r_per_split = ceil_div(p.R, KT) * KT;
    const int tile = fi > 64 ? TILE_128x128 : fi > 32 ? TILE_64x128 : TILE_32x128;
    return launch_tiles<ConvDzProblem>(tile, p, stream);
}

hipError_t launch_conv2d_bwd_dw(const float *var_w, const float *mu_a, const float *dmu,
                                const float *dvar, const int *aidx, int B, int fo, int woho,
                                int wihi, int fi, int ki, int splits, float *ws0, float *ws1,
                                float *dmu_w, float *dvar_w, hipStream_t stream) {
    ConvParams p = {};
    p.a0 = mu_a; p.d0 = dmu; p.d1 = dvar; p.e0 = var_w; p.idx = aidx;
    p.out0 = dmu_w; p.out1 = dvar_w;
    p.woho = woho; p.fo = fo; p.wihi = wihi; p.fi = fi; p.k2 = ki * ki; p.B = B;
    p.M = fo; p.N = p.k2 * fi; p.R = B * woho;
    int per = ceil_div(ceil_div(p.R, splits), KT) * KT;
    p.splits = ceil_div(p.R, per);
    p.r_per_split = per;
    p.ws0 = ws0; p.ws1 = ws1;
    const bool vec = (woho % 4 == 0) && aligned16(dmu) && aligned16(dvar);
    hipError_t e = vec ? launch_tiles<ConvDwProblem<true>>(TILE_64x64, p, stream)
                       : launch_tiles<ConvDwProblem<false>>(TILE_64x64, p, stream);
    if (e != hipSuccess) return e;
    if (p.splits > 1)
        e = launch_reduce_splits(EPI_SCALE, ws0, ws1, p.splits, p.M, p.N, var_w, nullptr, dmu_w,
                                 dvar_w, p.N, stream);
    return e;
}

// `scratch` holds 2*chunks*fo floats.
hipError_t launch_conv2d_bwd_db(const float *var_b, const float *dmu, const float *dvar, int B,
                                int fo, int woho, int chunks, float *scratch, float *dmu_b,
                                float *dvar_b, hipStream_t stream) {
    float *p0 = scratch, *p1 = scratch + (size_t)chunks * fo;
    hipLaunchKernelGGL(conv_bias_partial_kernel, dim3(fo, chunks), dim3(256), 0, stream, dmu, dvar,
                       B, fo, woho, chunks, p0, p1);
    hipLaunchKernelGGL(conv_bias_final_kernel, dim3(ceil_div(fo, 64)), dim3(64), 0, stream, p0, p1,
                       var_b, fo, chunks, dmu_b, dvar_b);
    return hipGetLastError();
}

}  // namespace tagi

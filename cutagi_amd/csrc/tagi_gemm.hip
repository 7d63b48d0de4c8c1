// Tiled fp32-MFMA kernels for the three TAGI Linear contractions, gfx950: the
// problem definitions that plug the Linear operands into tagi_mfma_tile.h.
//
//   FWD: D[b][n]  = sum_k act[b][k] * w[n][k]; the variance is one GEMM over the
//        concatenated reduction [var_w | mu_w^2] x [var_a + mu_a^2 ; var_a] that
//        shares the LDS tiles of the mean GEMM (squares and sums are formed in
//        registers from the staged mu/var tiles). Both operands k-contiguous.
//   DZ : D[b][k'] = sum_n delta[b][n] * w[n][k'] (variance with w^2); delta is
//        k-contiguous, w is staged [n][k'] as it lies in memory.
//   DW : D[n][k'] = sum_b delta[b][n] * act[b][k'] (variance with act^2); both
//        operands are staged [b][...] as they lie in memory.
#include "tagi_internal.h"
#include "tagi_activation.h"
#include "tagi_mfma_tile.h"

namespace tagi {
extern int g_gemm_double_buffer;
namespace {

// Four elements of a row-major matrix `base` (leading dimension ld): along the
// reduction (KC) at (row, r..r+3), or along the rows at (row..row+3, r) where the
// reduction index is the slow one. Zero outside [0,rows) x [.., r_end).
template <bool KC, bool VEC>
__device__ __forceinline__ float4 load4(const float *__restrict__ base, int ld, int row, int rows,
                                        int r, int r_end) {
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (VEC) {
        if (row < rows && r < r_end) {
            const float *q = KC ? base + (size_t)row * ld + r : base + (size_t)r * ld + row;
            v = *reinterpret_cast<const float4 *>(q);
        }
    } else {
        float c[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (KC) {
                if (row < rows && r + j < r_end) c[j] = base[(size_t)row * ld + r + j];
            } else {
                if (r < r_end && row + j < rows) c[j] = base[(size_t)r * ld + row + j];
            }
        }
        v = make_float4(c[0], c[1], c[2], c[3]);
    }
    return v;
}

// The same for a problem whose every k-tile is complete (reduction length and
// slices are multiples of the k-tile, 16-byte rows): nothing to mask along the
// reduction, and a row beyond the matrix is read from its last row instead -- its
// sums land in accumulator rows that the epilogue never stores. No branch and no
// zero fill around the load.
template <bool KC>
__device__ __forceinline__ float4 load4_full(const float *__restrict__ base, int ld, int row,
                                             int rows, int r) {
    const int rr = min(row, rows - (KC ? 1 : 4));
    const float *q = KC ? base + (size_t)rr * ld + r : base + (size_t)r * ld + rr;
    return *reinterpret_cast<const float4 *>(q);
}

template <int MODE, bool VEC, bool FULL = false, bool DB = false>
struct LinearProblem {
    static_assert(VEC || !FULL, "complete k-tiles are a case of the 16-byte path");
    static_assert(FULL || !DB, "the double-buffered loop is built for complete k-tiles");
    using Params = GemmParams;
    static constexpr bool DOUBLE_BUFFER = DB;
    static constexpr bool XK = (MODE != GEMM_DW);
    static constexpr bool YK = (MODE == GEMM_FWD);
    static constexpr int NX = 2;
    static constexpr int NY = (MODE == GEMM_FWD) ? 2 : 1;
    static constexpr int FLAVOR = (MODE == GEMM_FWD) ? FLAVOR_FWD_ACT_ROWS : FLAVOR_DELTA_ROWS;

    using Ctx = TileNoCtx;
    static constexpr bool PROLOGUE_WRITES_LDS = false, SPLIT_PER_XCD = false;
    static constexpr int VARIANTS = 1;
    __device__ static __forceinline__ void adjust_range(const Params &, const Ctx &, int &, int &) {}
    __device__ static __forceinline__ int place_tile(const Params &, int tile, int, int) { return tile; }
    static constexpr int min_waves_per_simd(int, int, int) { return 0; }
    static size_t extra_lds_bytes(const Params &, int, int) { return 0; }
    __device__ static __forceinline__ void prologue(const Params &, Ctx &, int *, int, int, int,
                                                    int, int, int, int, int) {}
    __device__ static __forceinline__ void next_tile(const Params &, Ctx &) {}
    __device__ static __forceinline__ float4 fix_x(const Ctx &, int, const float4 &v) { return v; }
    __device__ static __forceinline__ float4 fix_y(const Ctx &, int, const float4 &v) { return v; }

    __device__ static __forceinline__ float4 load_x(const Params &p, Ctx &, int, int arr, int, int m0,
                                                    int row, int r, int r_end) {
        if (FULL) return load4_full<XK>(arr ? p.x1 : p.x0, p.ldx, m0 + row, p.M, r);
        return load4<XK, VEC>(arr ? p.x1 : p.x0, p.ldx, m0 + row, p.M, r, r_end);
    }
    __device__ static __forceinline__ float4 load_y(const Params &p, Ctx &, int, int arr, int, int n0,
                                                    int row, int r, int r_end) {
        if (FULL) return load4_full<YK>(arr ? p.y1 : p.y0, p.ldy, n0 + row, p.N, r);
        return load4<YK, VEC>(arr ? p.y1 : p.y0, p.ldy, n0 + row, p.N, r, r_end);
    }
    // delta_z / delta_w: the Jacobian / var_w element that scales an output
    static constexpr bool EPI_PREFETCH = (MODE != GEMM_FWD);
    __device__ static __forceinline__ float epi_load(const Params &p, int m, int n) {
        return p.e0[(size_t)m * p.ldo + n];
    }
    __device__ static __forceinline__ void store_with(const Params &p, int m, int n, float a0,
                                                      float a1, float e) {
        const size_t at = (size_t)m * p.ldo + n;
        p.out0[at] = a0 * e;
        p.out1[at] = a1 * (e * e);
    }
    __device__ static __forceinline__ void store(const Params &p, int m, int n, float a0,
                                                 float a1) {
        const size_t at = (size_t)m * p.ldo + n;
        if (MODE == GEMM_FWD) {
            if (p.e0 != nullptr) {
                a0 += p.e0[n];
                a1 += p.e1[n];
            }
            store_activated(p.act, a0, a1, at, p.out0, p.out1, p.out2);
            return;
        } else {
            const float e = p.e0[at];
            a0 *= e;
            a1 *= e * e;
        }
        p.out0[at] = a0;
        p.out1[at] = a1;
    }
};

template <int EPI, bool VEC>
__global__ __launch_bounds__(64) void reduce_splits_kernel(const float *__restrict__ ws0,
                                                            const float *__restrict__ ws1,
                                                            int splits, int M, int N,
                                                            const float *__restrict__ e0,
                                                            const float *__restrict__ e1,
                                                            float *__restrict__ out0,
                                                            float *__restrict__ out1, int ldo,
                                                            int act, float *__restrict__ out2) {
    const size_t total = (size_t)M * N;
    constexpr int W = VEC ? 4 : 1;
    const size_t idx = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * W;
    if (idx >= total) return;
    float s0[W], s1[W];
#pragma unroll
    for (int c = 0; c < W; c++) s0[c] = s1[c] = 0.f;
    // slices are folded in index order (deterministic); the unroll keeps several
    // slices' loads in flight
#pragma unroll 8
    for (int s = 0; s < splits; s++) {
        if constexpr (VEC) {
            const float4 a = *reinterpret_cast<const float4 *>(ws0 + s * total + idx);
            const float4 b = *reinterpret_cast<const float4 *>(ws1 + s * total + idx);
            s0[0] += a.x; s0[1] += a.y; s0[2] += a.z; s0[3] += a.w;
            s1[0] += b.x; s1[1] += b.y; s1[2] += b.z; s1[3] += b.w;
        } else {
            s0[0] += ws0[s * total + idx];
            s1[0] += ws1[s * total + idx];
        }
    }
    const int row = (int)(idx / N), col = (int)(idx % N);
    const size_t at = (size_t)row * ldo + col;
#pragma unroll
    for (int c = 0; c < W; c++) {
        if (EPI == EPI_BIAS) {
            if (e0 != nullptr) {
                s0[c] += e0[col + c];
                s1[c] += e1[col + c];
            }
        } else {
            const float e = e0[at + c];
            s0[c] *= e;
            s1[c] *= e * e;
        }
    }
    float s2[W];
    if (EPI == EPI_BIAS && act != ACT_NONE) {
#pragma unroll
        for (int c = 0; c < W; c++) {
            const float m = s0[c], v = s1[c];
            if (act == ACT_RELU)
                relu_moments(m, v, s0[c], s1[c], s2[c]);
            else
                mixture_relu_moments(m, v, s0[c], s1[c], s2[c]);
        }
        if constexpr (VEC)
            *reinterpret_cast<float4 *>(out2 + at) = make_float4(s2[0], s2[1], s2[2], s2[3]);
        else
            out2[at] = s2[0];
    }
    if constexpr (VEC) {
        *reinterpret_cast<float4 *>(out0 + at) = make_float4(s0[0], s0[1], s0[2], s0[3]);
        *reinterpret_cast<float4 *>(out1 + at) = make_float4(s1[0], s1[1], s1[2], s1[3]);
    } else {
        out0[at] = s0[0];
        out1[at] = s1[0];
    }
}

template <int MODE>
hipError_t launch_mode(int tile, bool vec, const GemmParams &p, hipStream_t stream) {
    const bool full = vec && p.R % KT == 0 && (p.splits == 1 || p.r_per_split % KT == 0) &&
                      p.M >= 4 && p.N >= 4;
    // The two-stage loop pays one memory round trip per 16 reduction elements when
    // nothing else runs on the CU to hide it: launches that leave most of the chip
    // empty (the layers of a small MLP) keep the single stage of 32.
    const int tiles = ((p.M + tile_rows(tile) - 1) / tile_rows(tile)) *
                      ((p.N + tile_cols(tile) - 1) / tile_cols(tile));
    if (full && g_gemm_double_buffer != 0 && tiles * p.splits >= num_cu())
        return launch_tiles<LinearProblem<MODE, true, true, true>>(tile, p, stream);
    if (full) return launch_tiles<LinearProblem<MODE, true, true>>(tile, p, stream);
    if (vec) return launch_tiles<LinearProblem<MODE, true>>(tile, p, stream);
    return launch_tiles<LinearProblem<MODE, false>>(tile, p, stream);
}


// ---------------------------------------------------------------------------
// Weight backward with the small jobs of the backward call riding along: the
// first workgroups of the launch (the first to be dispatched) fold the slices a
// sliced state backward left in the workspace, and sum the bias innovations over
// the batch, while the others already multiply tiles. That saves two dependent
// launches per layer (the weight backward needs neither result).
// ---------------------------------------------------------------------------
constexpr int SIDE_BIAS_COLS = 64;  // bias columns per side workgroup (8 batch slices each)

template <int NT>
__device__ __forceinline__ void side_workgroup(const LinearSideWork &w, int id) {
    if (id < w.bias_wgs) {
        // delta_b[n] = var_b[n] * sum_b delta[b][n]: NT/64 batch slices of 64 columns,
        // folded through LDS in slice order
        constexpr int SL = NT / 64;
        __shared__ float s0[SL][64], s1[SL][64];
        const int c = threadIdx.x & 63, slice = threadIdx.x >> 6;
        const int n = id * SIDE_BIAS_COLS + c;
        float a0 = 0.f, a1 = 0.f;
        if (n < w.bias_n) {
#pragma unroll 4
            for (int b = slice; b < w.bias_b; b += SL) {
                a0 += w.dmu[(size_t)b * w.bias_n + n];
                a1 += w.dvar[(size_t)b * w.bias_n + n];
            }
        }
        s0[slice][c] = a0;
        s1[slice][c] = a1;
        __syncthreads();
        if (slice == 0 && n < w.bias_n) {
            float m = 0.f, v = 0.f;
#pragma unroll
            for (int sl = 0; sl < SL; sl++) {
                m += s0[sl][c];
                v += s1[sl][c];
            }
            const float vb = w.var_b[n];
            w.dmu_b[n] = m * vb;
            w.dvar_b[n] = v * vb * vb;
        }
        return;
    }
    // fold: out = (sum over slices, in slice order) * jcb, * jcb^2; float4 items
    const int fid = id - w.bias_wgs, fold_wgs = w.side_wgs - w.bias_wgs;
    const size_t items = w.fold_total / 4;
    for (size_t it = (size_t)fid * NT + threadIdx.x; it < items; it += (size_t)fold_wgs * NT) {
        const size_t at = it * 4;
        float4 m = make_float4(0.f, 0.f, 0.f, 0.f), v = m;
        int sl = 0;
        for (; sl + 4 <= w.fold_splits; sl += 4) {
            float4 x[4], y[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                x[u] = *reinterpret_cast<const float4 *>(w.ws0 + (sl + u) * w.fold_total + at);
                y[u] = *reinterpret_cast<const float4 *>(w.ws1 + (sl + u) * w.fold_total + at);
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                m.x += x[u].x; m.y += x[u].y; m.z += x[u].z; m.w += x[u].w;
                v.x += y[u].x; v.y += y[u].y; v.z += y[u].z; v.w += y[u].w;
            }
        }
        for (; sl < w.fold_splits; sl++) {
            const float4 x = *reinterpret_cast<const float4 *>(w.ws0 + sl * w.fold_total + at);
            const float4 y = *reinterpret_cast<const float4 *>(w.ws1 + sl * w.fold_total + at);
            m.x += x.x; m.y += x.y; m.z += x.z; m.w += x.w;
            v.x += y.x; v.y += y.y; v.z += y.z; v.w += y.w;
        }
        const float4 j = *reinterpret_cast<const float4 *>(w.jcb + at);
        *reinterpret_cast<float4 *>(w.out0 + at) =
            make_float4(m.x * j.x, m.y * j.y, m.z * j.z, m.w * j.w);
        *reinterpret_cast<float4 *>(w.out1 + at) =
            make_float4(v.x * (j.x * j.x), v.y * (j.y * j.y), v.z * (j.z * j.z), v.w * (j.w * j.w));
    }
}

template <class P, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM *WN * 64) void linear_dw_side_kernel(GemmParams p,
                                                                      LinearSideWork w) {
    const int id = blockIdx.x;
    if (id < w.side_wgs) {
        side_workgroup<WM * WN * 64>(w, id);
        return;
    }
    // (side_wgs is a multiple of 8: a tile's workgroup keeps its XCD)
    tile_workgroup<P, BM, BN, WM, WN>(p, id - w.side_wgs, 0, (int)gridDim.x - w.side_wgs, 1);
}

template <bool FULL, bool DB = false>
hipError_t launch_dw_side(const GemmParams &p, const LinearSideWork &w, hipStream_t stream) {
    using P = LinearProblem<GEMM_DW, true, FULL, DB>;
    const int tiles = ((p.M + 63) / 64) * ((p.N + 127) / 128);
    hipLaunchKernelGGL((linear_dw_side_kernel<P, 64, 128, 2, 4>), dim3(tiles + w.side_wgs),
                       dim3(512), 0, stream, p, w);
    return hipGetLastError();
}
}  // namespace

int g_gemm_double_buffer = 1;

int gemm_tile_rows(int tile) { return tile_rows(tile); }
int gemm_tile_cols(int tile) { return tile_cols(tile); }
int gemm_tile_count() { return TILE_COUNT; }
int gemm_k_tile() { return KT; }

hipError_t launch_gemm(GemmMode mode, int tile, bool vec, const GemmParams &p,
                       hipStream_t stream) {
    switch (mode) {
        case GEMM_FWD: return launch_mode<GEMM_FWD>(tile, vec, p, stream);
        case GEMM_DZ: return launch_mode<GEMM_DZ>(tile, vec, p, stream);
        case GEMM_DW: return launch_mode<GEMM_DW>(tile, vec, p, stream);
    }
    return hipErrorInvalidValue;
}

bool gemm_dw_side_supported(int tile, bool vec, const GemmParams &p) {
    return tile == TILE_64x128 && vec && p.splits == 1;
}

hipError_t launch_gemm_dw_side(const GemmParams &p, LinearSideWork w, hipStream_t stream) {
    // side workgroups: one per 64 bias columns, then up to 64 for the fold (one
    // float4 of its result per thread and round); padded to a multiple of 8
    w.bias_wgs = w.var_b != nullptr ? (w.bias_n + SIDE_BIAS_COLS - 1) / SIDE_BIAS_COLS : 0;
    int fold_wgs = 0;
    if (w.ws0 != nullptr) {
        const size_t want = (w.fold_total / 4 + 511) / 512;
        fold_wgs = want < 64 ? (int)want : 64;
        if (fold_wgs < 1) fold_wgs = 1;
    }
    w.side_wgs = (w.bias_wgs + fold_wgs + 7) / 8 * 8;
    if (w.ws0 == nullptr) w.fold_total = 0;  // the padding workgroups find nothing to fold
    const bool full = p.R % KT == 0 && p.M >= 4 && p.N >= 4;
    const int tiles = ((p.M + 63) / 64) * ((p.N + 127) / 128);
    if (full && g_gemm_double_buffer != 0 && tiles >= num_cu())
        return launch_dw_side<true, true>(p, w, stream);
    return full ? launch_dw_side<true>(p, w, stream) : launch_dw_side<false>(p, w, stream);
}

hipError_t launch_reduce_splits(Epilogue epi, const float *ws0, const float *ws1, int splits,
                                int M, int N, const float *e0, const float *e1, float *out0,
                                float *out1, int ldo, hipStream_t stream, int act, float *out2) {
    const size_t total = (size_t)M * N;
    auto al = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    const bool vec = (N % 4 == 0) && (ldo % 4 == 0) && al(ws0) && al(ws1) && al(out0) &&
                     al(out1) && (epi == EPI_BIAS || al(e0)) && (act == ACT_NONE || al(out2));
    if (epi != EPI_BIAS) act = ACT_NONE;
    const size_t items = vec ? total / 4 : total;
    dim3 grid((unsigned)((items + 63) / 64)), block(64);
    if (epi == EPI_BIAS) {
        if (vec)
            hipLaunchKernelGGL((reduce_splits_kernel<EPI_BIAS, true>), grid, block, 0, stream, ws0,
                               ws1, splits, M, N, e0, e1, out0, out1, ldo, act, out2);
        else
            hipLaunchKernelGGL((reduce_splits_kernel<EPI_BIAS, false>), grid, block, 0, stream,
                               ws0, ws1, splits, M, N, e0, e1, out0, out1, ldo, act, out2);
    } else {
        if (vec)
            hipLaunchKernelGGL((reduce_splits_kernel<EPI_SCALE, true>), grid, block, 0, stream,
                               ws0, ws1, splits, M, N, e0, e1, out0, out1, ldo, act, out2);
        else
            hipLaunchKernelGGL((reduce_splits_kernel<EPI_SCALE, false>), grid, block, 0, stream,
                               ws0, ws1, splits, M, N, e0, e1, out0, out1, ldo, act, out2);
    }
    return hipGetLastError();
}

}  // namespace tagi

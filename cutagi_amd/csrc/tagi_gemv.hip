// Skinny-batch (B <= 16) kernels of the TAGI Linear layer, gfx950.
//
// With a handful of samples every weight is used only B times, so the layer is
// bound by streaming the weight matrices from HBM once. Nothing is staged in
// LDS: each lane loads 16 bytes of a weight row straight into the operand
// layout of v_mfma_f32_16x16x4_f32 (A[i][k]: lane = i + 16*k, B[k][j]: lane =
// j + 16*k, D[i][j]: register i%4 of lane j + 16*(i/4)), the batch sits in the
// 16 columns of the MFMA (columns >= B are fed zeros), and the reduction over
// the streamed dimension happens inside the matrix core. The weight backward
// has no reduction worth an MFMA (length B) and is a pure VALU streaming kernel.
//
// Reduction slices (gridDim.y) write partial sums [slice][B][cols]; the caller
// folds them, together with the bias or Jacobian epilogue, in reduce_splits.
#include "tagi_internal.h"

namespace tagi {

typedef float floatx4 __attribute__((ext_vector_type(4)));

namespace {

__device__ __forceinline__ float4 ld4(const float *p) {
    return *reinterpret_cast<const float4 *>(p);
}
__device__ __forceinline__ float4 zero4() { return make_float4(0.f, 0.f, 0.f, 0.f); }
__device__ __forceinline__ float comp(const float4 &v, int t) {
    return t == 0 ? v.x : t == 1 ? v.y : t == 2 ? v.z : v.w;
}
__device__ __forceinline__ floatx4 mfma16(float a, float b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// ---------------------------------------------------------------------------
// Forward. A wave owns 16 output rows (weight rows n0..n0+15) and one reduction
// slice; lane (i = l%16, g = l/16) reads U consecutive float4 of row n0+i
// starting at k = kb + 4*U*g, so one row is read in runs of 64*U bytes and the
// four lanes of a row cover 256*U bytes between them. MFMA (u, t) multiplies
// k = kb + 4*U*g + 4*u + t on both operands.
// ---------------------------------------------------------------------------
constexpr int FWD_U = 4;
constexpr int FWD_ROWS_PER_BLOCK = 64;  // 4 waves x 16 rows
constexpr int FWD_KSTEP = 16 * FWD_U;

struct FwdRegs {
    float4 wm[FWD_U], wv[FWD_U], am[FWD_U], av[FWD_U];
};

__device__ __forceinline__ void fwd_load(FwdRegs &r, const float *wm, const float *wv,
                                         const float *am, const float *av, bool row_ok,
                                         bool act_ok, int k, int k_end) {
#pragma unroll
    for (int u = 0; u < FWD_U; u++) {
        const int kk = k + 4 * u;
        const bool in = kk < k_end;
        r.wm[u] = (row_ok && in) ? ld4(wm + kk) : zero4();
        r.wv[u] = (row_ok && in) ? ld4(wv + kk) : zero4();
        r.am[u] = (act_ok && in) ? ld4(am + kk) : zero4();
        r.av[u] = (act_ok && in) ? ld4(av + kk) : zero4();
    }
}

__global__ __launch_bounds__(256) void gemv_fwd_kernel(
    const float *__restrict__ mu_w, const float *__restrict__ var_w,
    const float *__restrict__ mu_a, const float *__restrict__ var_a, int K, int N, int B,
    int k_per_split, float *__restrict__ ws0, float *__restrict__ ws1) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * FWD_ROWS_PER_BLOCK + wave * 16;
    const int split = blockIdx.y;
    const int k_begin = split * k_per_split;
    const int k_end = min(K, k_begin + k_per_split);
    const int row = n0 + i;
    const bool row_ok = row < N, act_ok = i < B;
    const float *wm = mu_w + (size_t)(row_ok ? row : 0) * K;
    const float *wv = var_w + (size_t)(row_ok ? row : 0) * K;
    const float *am = mu_a + (size_t)(act_ok ? i : 0) * K;
    const float *av = var_a + (size_t)(act_ok ? i : 0) * K;

    floatx4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
    FwdRegs cur, nxt;
    const int koff = 4 * FWD_U * g;
    fwd_load(cur, wm, wv, am, av, row_ok, act_ok, k_begin + koff, k_end);
    for (int kb = k_begin; kb < k_end; kb += FWD_KSTEP) {
        fwd_load(nxt, wm, wv, am, av, row_ok, act_ok, kb + FWD_KSTEP + koff, k_end);
#pragma unroll
        for (int u = 0; u < FWD_U; u++) {
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const float w = comp(cur.wm[u], t), v = comp(cur.wv[u], t);
                const float a = comp(cur.am[u], t), s = comp(cur.av[u], t);
                acc0 = mfma16(w, a, acc0);
                acc1 = mfma16(v, s + a * a, acc1);
                acc1 = mfma16(w * w, s, acc1);
            }
        }
        cur = nxt;
    }

    // D[i = row][j = sample]: lane (j = l%16, q = l/16) holds rows n0 + 4q + 0..3
    const int j = lane & 15, q = lane >> 4;
    if (j < B) {
        const size_t base = ((size_t)split * B + j) * N + n0 + 4 * q;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            if (n0 + 4 * q + v < N) {
                ws0[base + v] = acc0[v];
                ws1[base + v] = acc1[v];
            }
        }
    }
}

// ---------------------------------------------------------------------------
// State backward. A wave owns 64 consecutive input columns k' and one slice of
// the reduction over output rows n; lane (i = l%16, g = l/16) reads the float4
// W[n][c0 + 4i .. 4i+3] of rows n = nb + 4g + u (u = 0..3), i.e. every row is
// read in 256-byte runs. Component t of the float4 feeds accumulator t, whose
// row i is column c0 + 4i + t; the MFMA reduces over the four rows held by the
// four lane groups.
// ---------------------------------------------------------------------------
constexpr int DZ_COLS_PER_BLOCK = 256;  // 4 waves x 64 columns
constexpr int DZ_NSTEP = 16;

struct DzRegs {
    float4 w[4];
    float4 dm, dv;
};

__device__ __forceinline__ void dz_load(DzRegs &r, const float *w, size_t ldw, bool col_ok,
                                        const float *dm, const float *dv, bool act_ok, int n,
                                        int n_end) {
#pragma unroll
    for (int u = 0; u < 4; u++)
        r.w[u] = (col_ok && n + u < n_end) ? ld4(w + (size_t)(n + u) * ldw) : zero4();
    const bool in = act_ok && n < n_end;
    r.dm = in ? ld4(dm + n) : zero4();
    r.dv = in ? ld4(dv + n) : zero4();
}

__global__ __launch_bounds__(256) void gemv_dz_kernel(
    const float *__restrict__ mu_w, const float *__restrict__ dmu,
    const float *__restrict__ dvar, int K, int N, int B, int n_per_split,
    float *__restrict__ ws0, float *__restrict__ ws1) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = lane & 15, g = lane >> 4;
    const int c0 = blockIdx.x * DZ_COLS_PER_BLOCK + wave * 64;
    const int split = blockIdx.y;
    const int n_begin = split * n_per_split;
    const int n_end = min(N, n_begin + n_per_split);
    const int col = c0 + 4 * i;
    const bool col_ok = col < K, act_ok = i < B;
    const float *w = mu_w + (col_ok ? col : 0);
    const float *dm = dmu + (size_t)(act_ok ? i : 0) * N;
    const float *dv = dvar + (size_t)(act_ok ? i : 0) * N;

    floatx4 acc0[4], acc1[4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
        acc0[t] = (floatx4){0.f, 0.f, 0.f, 0.f};
        acc1[t] = (floatx4){0.f, 0.f, 0.f, 0.f};
    }
    DzRegs cur, nxt;
    dz_load(cur, w, K, col_ok, dm, dv, act_ok, n_begin + 4 * g, n_end);
    for (int nb = n_begin; nb < n_end; nb += DZ_NSTEP) {
        dz_load(nxt, w, K, col_ok, dm, dv, act_ok, nb + DZ_NSTEP + 4 * g, n_end);
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const float d0 = comp(cur.dm, u), d1 = comp(cur.dv, u);
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const float x = comp(cur.w[u], t);
                acc0[t] = mfma16(x, d0, acc0[t]);
                acc1[t] = mfma16(x * x, d1, acc1[t]);
            }
        }
        cur = nxt;
    }

    // D_t[i][j]: lane (j = l%16, q = l/16), register v -> i = 4q + v, i.e. column
    // c0 + 16q + 4v + t: 16 consecutive columns per lane.
    const int j = lane & 15, q = lane >> 4;
    if (j < B) {
        const size_t base = ((size_t)split * B + j) * K + c0 + 16 * q;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            if (c0 + 16 * q + 4 * v < K) {  // K % 4 == 0 on this path
                *reinterpret_cast<float4 *>(ws0 + base + 4 * v) =
                    make_float4(acc0[0][v], acc0[1][v], acc0[2][v], acc0[3][v]);
                *reinterpret_cast<float4 *>(ws1 + base + 4 * v) =
                    make_float4(acc1[0][v], acc1[1][v], acc1[2][v], acc1[3][v]);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Weight backward. delta_w[n][k'] = var_w[n][k'] * sum_b delta[b][n] * a[b][k'].
// A lane keeps a[b][k'..k'+3] and its squares for all b in registers and walks
// rows; the 2*B innovations of a row are wave-uniform and come from LDS as
// broadcast reads. Per row a wave reads 1 KB of var_w and writes 2 KB.
// ---------------------------------------------------------------------------
constexpr int DW_COLS_PER_BLOCK = 256;  // 64 lanes x 4 columns, shared by the 4 waves
constexpr int DW_ROWS_PER_BLOCK = 64;   // 16 rows per wave

template <int BMAX>
__global__ __launch_bounds__(256) void gemv_dw_kernel(
    const float *__restrict__ var_w, const float *__restrict__ mu_a,
    const float *__restrict__ dmu, const float *__restrict__ dvar, int K, int N, int B,
    float *__restrict__ dmu_w, float *__restrict__ dvar_w) {
    __shared__ __attribute__((aligned(16))) float s_dm[DW_ROWS_PER_BLOCK][BMAX];
    __shared__ __attribute__((aligned(16))) float s_dv[DW_ROWS_PER_BLOCK][BMAX];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = blockIdx.x * DW_COLS_PER_BLOCK + lane * 4;
    const int n0 = blockIdx.y * DW_ROWS_PER_BLOCK;

    for (int e = threadIdx.x; e < DW_ROWS_PER_BLOCK * BMAX; e += 256) {
        const int b = e / DW_ROWS_PER_BLOCK, r = e % DW_ROWS_PER_BLOCK;
        const bool ok = b < B && n0 + r < N;
        s_dm[r][b] = ok ? dmu[(size_t)b * N + n0 + r] : 0.f;
        s_dv[r][b] = ok ? dvar[(size_t)b * N + n0 + r] : 0.f;
    }

    const bool col_ok = col < K;  // K % 4 == 0 on this path
    float4 a[BMAX], a2[BMAX];
#pragma unroll
    for (int b = 0; b < BMAX; b++) {
        a[b] = (col_ok && b < B) ? ld4(mu_a + (size_t)b * K + col) : zero4();
        a2[b] = make_float4(a[b].x * a[b].x, a[b].y * a[b].y, a[b].z * a[b].z, a[b].w * a[b].w);
    }
    __syncthreads();
    if (!col_ok) return;

    constexpr int RPW = DW_ROWS_PER_BLOCK / 4;
#pragma unroll 4
    for (int rr = 0; rr < RPW; rr++) {
        const int r = wave * RPW + rr;
        const int n = n0 + r;
        if (n >= N) break;
        const float4 vw = ld4(var_w + (size_t)n * K + col);
        float4 sm = zero4(), sv = zero4();
#pragma unroll
        for (int b = 0; b < BMAX; b++) {
            const float d0 = s_dm[r][b], d1 = s_dv[r][b];
            sm.x += d0 * a[b].x; sm.y += d0 * a[b].y; sm.z += d0 * a[b].z; sm.w += d0 * a[b].w;
            sv.x += d1 * a2[b].x; sv.y += d1 * a2[b].y; sv.z += d1 * a2[b].z; sv.w += d1 * a2[b].w;
        }
        float4 om = make_float4(sm.x * vw.x, sm.y * vw.y, sm.z * vw.z, sm.w * vw.w);
        float4 ov = make_float4(sv.x * vw.x * vw.x, sv.y * vw.y * vw.y, sv.z * vw.z * vw.z,
                                sv.w * vw.w * vw.w);
        floatx4 *pm = reinterpret_cast<floatx4 *>(dmu_w + (size_t)n * K + col);
        floatx4 *pv = reinterpret_cast<floatx4 *>(dvar_w + (size_t)n * K + col);
        __builtin_nontemporal_store((floatx4){om.x, om.y, om.z, om.w}, pm);
        __builtin_nontemporal_store((floatx4){ov.x, ov.y, ov.z, ov.w}, pv);
    }
}

}  // namespace

int gemv_fwd_rows_per_block() { return FWD_ROWS_PER_BLOCK; }
int gemv_fwd_k_step() { return FWD_KSTEP; }
int gemv_dz_cols_per_block() { return DZ_COLS_PER_BLOCK; }
int gemv_dz_n_step() { return DZ_NSTEP; }

hipError_t launch_gemv_fwd(const float *mu_w, const float *var_w, const float *mu_a,
                           const float *var_a, int K, int N, int B, int splits, float *ws0,
                           float *ws1, hipStream_t stream) {
    int per = (K + splits - 1) / splits;
    per = (per + FWD_KSTEP - 1) / FWD_KSTEP * FWD_KSTEP;
    dim3 grid((N + FWD_ROWS_PER_BLOCK - 1) / FWD_ROWS_PER_BLOCK, splits), block(256);
    hipLaunchKernelGGL(gemv_fwd_kernel, grid, block, 0, stream, mu_w, var_w, mu_a, var_a, K, N, B,
                       per, ws0, ws1);
    return hipGetLastError();
}

hipError_t launch_gemv_dz(const float *mu_w, const float *dmu, const float *dvar, int K, int N,
                          int B, int splits, float *ws0, float *ws1, hipStream_t stream) {
    int per = (N + splits - 1) / splits;
    per = (per + DZ_NSTEP - 1) / DZ_NSTEP * DZ_NSTEP;
    dim3 grid((K + DZ_COLS_PER_BLOCK - 1) / DZ_COLS_PER_BLOCK, splits), block(256);
    hipLaunchKernelGGL(gemv_dz_kernel, grid, block, 0, stream, mu_w, dmu, dvar, K, N, B, per, ws0,
                       ws1);
    return hipGetLastError();
}

hipError_t launch_gemv_dw(const float *var_w, const float *mu_a, const float *dmu,
                          const float *dvar, int K, int N, int B, float *dmu_w, float *dvar_w,
                          hipStream_t stream) {
    dim3 grid((K + DW_COLS_PER_BLOCK - 1) / DW_COLS_PER_BLOCK,
              (N + DW_ROWS_PER_BLOCK - 1) / DW_ROWS_PER_BLOCK),
        block(256);
    if (B <= 4)
        hipLaunchKernelGGL(gemv_dw_kernel<4>, grid, block, 0, stream, var_w, mu_a, dmu, dvar, K, N,
                           B, dmu_w, dvar_w);
    else if (B <= 8)
        hipLaunchKernelGGL(gemv_dw_kernel<8>, grid, block, 0, stream, var_w, mu_a, dmu, dvar, K, N,
                           B, dmu_w, dvar_w);
    else
        hipLaunchKernelGGL(gemv_dw_kernel<16>, grid, block, 0, stream, var_w, mu_a, dmu, dvar, K,
                           N, B, dmu_w, dvar_w);
    return hipGetLastError();
}

}  // namespace tagi

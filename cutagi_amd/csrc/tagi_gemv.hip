// Skinny-batch (B <= 16) kernels of the TAGI Linear layer, gfx950.
//
// With a handful of samples every weight is used only B times, so the layer is
// bound by streaming the weight matrices from HBM once. Each lane loads 16 bytes
// of a weight row straight into the operand layout of v_mfma_f32_4x4x1_16b_f32,
// chosen because its 16 independent 4x4 blocks let a load instruction cover whole
// cache lines (4 rows x 256 B forward, 1 row x 1 KB backward) while the batch
// sits in the 4 columns of a block (groups of 4 samples, rows beyond B are fed
// zeros). The few activations / innovations a workgroup needs live in LDS. The
// weight backward has no reduction worth an MFMA (length B) and is a pure VALU
// streaming kernel.
//
// The forward and state-backward kernels here are instantiated for up to 16
// samples. As dispatched, the state backward serves B <= 8 (9..16 samples take the
// 16x16x4 kernel of tagi_gemv16.hip) and the forward none: the 16x16x4 forward
// measured faster for every batch, and this one stays behind a test switch
// ("linear.gemv16.min_batch"). The weight backward serves every B <= 16.
//
// Reduction slices (gridDim.y) write partial sums [slice][B][cols]; the caller
// folds them, together with the bias or Jacobian epilogue, in reduce_splits.
#include "tagi_internal.h"
#include "tagi_stage.h"

namespace tagi {

typedef float floatx4 __attribute__((ext_vector_type(4)));

namespace {

__device__ __forceinline__ float4 ld4(const float *p) {
    return *reinterpret_cast<const float4 *>(p);
}
// Streaming (non-temporal) load for weights that a kernel reads exactly once.
// Measured on the forward + backward sequence at 8192 x 8192, batch 8: with the
// forward and the state backward streaming their weights this way the whole step
// takes 288 us instead of 307 us; the weight backward is faster with plain loads.
__device__ __forceinline__ float4 ldnt4(const float *p) {
    const floatx4 v = __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(p));
    return make_float4(v[0], v[1], v[2], v[3]);
}
#ifndef TAGI_NT_MASK
#define TAGI_NT_MASK 3  // bit 0: forward, bit 1: state backward, bit 2: weight backward
#endif
__device__ __forceinline__ float4 ldw_fwd(const float *p) { return (TAGI_NT_MASK & 1) ? ldnt4(p) : ld4(p); }
__device__ __forceinline__ float4 ldw_dz(const float *p) { return (TAGI_NT_MASK & 2) ? ldnt4(p) : ld4(p); }
__device__ __forceinline__ float4 ldw_dw(const float *p) { return (TAGI_NT_MASK & 4) ? ldnt4(p) : ld4(p); }
__device__ __forceinline__ float4 zero4() { return make_float4(0.f, 0.f, 0.f, 0.f); }
__device__ __forceinline__ float comp(const float4 &v, int t) {
    return t == 0 ? v.x : t == 1 ? v.y : t == 2 ? v.z : v.w;
}

// ---------------------------------------------------------------------------
// Forward, v_mfma_f32_4x4x1_16b_f32: 16 independent 4x4 outer products per
// instruction, A_blk[i] taken from lane 4*blk+i, B_blk[j] from lane 4*blk+j,
// D_blk[i][j] in register i of lane 4*blk+j.
//
// Lane (blk = l/4, i = l%4) streams weight row n0+4*rg+i and holds the float4 at
// k = kb + 4*blk, so one load instruction covers 4 rows x 256 contiguous bytes
// (8 full cache lines). Block blk multiplies reduction elements kb+4*blk+t
// (t = 0..3, one MFMA each) against the activations of samples j+4*h, which the
// workgroup keeps in LDS for its whole reduction slice. The 16 blocks hold
// partial sums over different k; they meet in one cross-lane reduction when the
// slice is finished.
// ---------------------------------------------------------------------------
constexpr int FWD_WAVES = 8;
constexpr int FWD_KCHUNK = 64;    // reduction elements one load instruction covers per row
constexpr int FWD_KROUND = 512;   // slices are multiples of this (two stages of any variant)
constexpr int FWD_LDS_PAD = 8;    // row stride % 32 == 8: conflict-free 16-byte reads

__device__ __forceinline__ floatx4 mfma4(float a, float b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_4x4x1f32(a, b, c, 0, 0, 0);
}

// H: groups of 4 samples; RG: groups of 4 rows per wave; C: 64-element chunks per
// row and register stage (a stage holds RG*C float4 of each weight array).
template <int H, int RG, int C>
__global__ __launch_bounds__(FWD_WAVES * 64) void gemv_fwd_kernel(
    const float *__restrict__ mu_w, const float *__restrict__ var_w,
    const float *__restrict__ mu_a, const float *__restrict__ var_a, int K, int N, int B,
    int k_per_split, int splits, int swz, float *__restrict__ ws0, float *__restrict__ ws1) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int ROWS_PER_BLOCK = FWD_WAVES * RG * 4;
    constexpr int KSTEP = FWD_KCHUNK * C;  // reduction elements per register stage
    const int S = k_per_split + FWD_LDS_PAD;  // LDS row stride
    float *s_mu = lds, *s_var = lds + 4 * H * S;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int blk = lane >> 2, i = lane & 3;
    // Workgroup -> (row block, reduction slice). Workgroups are handed to the 8
    // XCDs round-robin; with the slice as the fast index inside an XCD, the
    // workgroups resident on one XCD cover all slices (all windows of a weight
    // row) instead of crowding into one.
    int row_block, split;
    const int id = blockIdx.x, row_blocks = gridDim.x / splits;
    if ((swz & 1) && row_blocks % 8 == 0) {
        const int xcd = id & 7, local = id >> 3;
        split = local % splits;
        row_block = (local / splits) * 8 + xcd;
    } else {
        row_block = id % row_blocks;
        split = id / row_blocks;
    }
    const int k_begin = split * k_per_split;
    const int kr = min(K, k_begin + k_per_split) - k_begin;  // this slice's length
    // each wave walks its slice from a different starting point (sums commute)
    const int rot = (swz & 2) ? ((row_block * FWD_WAVES + wave) * 2 * KSTEP) % k_per_split : 0;

    // stage the slice of the activations: [sample][k], zero beyond B and kr

    // Weight loads are never predicated (a predicated load costs a branch and
    // makes the compiler wait for every outstanding load): rows beyond N read row
    // N-1 and are dropped at the end, reduction elements beyond the slice read the
    // last float4 of the row and meet zero activations.
    const int n0 = row_block * ROWS_PER_BLOCK + wave * (RG * 4);
    const float *wm[RG], *wv[RG];
#pragma unroll
    for (int rg = 0; rg < RG; rg++) {
        const int row = min(n0 + 4 * rg + i, N - 1);
        wm[rg] = mu_w + (size_t)row * K;
        wv[rg] = var_w + (size_t)row * K;
    }
    const int k_lane = k_begin + 4 * blk, k_last = K - 4;

    floatx4 acc0[RG][H], acc1[RG][H];
#pragma unroll
    for (int rg = 0; rg < RG; rg++)
#pragma unroll
        for (int h = 0; h < H; h++) {
            acc0[rg][h] = (floatx4){0.f, 0.f, 0.f, 0.f};
            acc1[rg][h] = (floatx4){0.f, 0.f, 0.f, 0.f};
        }

    // Two register stages used in turn (no copies between them, so a stage's
    // loads stay in flight while the other stage is multiplied).
    float4 sm[2][RG][C], sv[2][RG][C];
    auto load = [&](float4(&m)[RG][C], float4(&v)[RG][C], int kb) {
#pragma unroll
        for (int c = 0; c < C; c++) {
            const int k = min(k_lane + kb + FWD_KCHUNK * c, k_last);
#pragma unroll
            for (int rg = 0; rg < RG; rg++) {
                m[rg][c] = ldw_fwd(wm[rg] + k);
                v[rg][c] = ldw_fwd(wv[rg] + k);
            }
        }
    };
    auto multiply = [&](const float4(&cm)[RG][C], const float4(&cv)[RG][C], int kb) {
#pragma unroll
        for (int c = 0; c < C; c++) {
            float4 am[H], as[H], av[H];
            const int at = kb + FWD_KCHUNK * c + 4 * blk;
#pragma unroll
            for (int h = 0; h < H; h++) {
                am[h] = *reinterpret_cast<const float4 *>(s_mu + (i + 4 * h) * S + at);
                av[h] = *reinterpret_cast<const float4 *>(s_var + (i + 4 * h) * S + at);
                as[h] = make_float4(av[h].x + am[h].x * am[h].x, av[h].y + am[h].y * am[h].y,
                                    av[h].z + am[h].z * am[h].z, av[h].w + am[h].w * am[h].w);
            }
#pragma unroll
            for (int rg = 0; rg < RG; rg++) {
                const float4 w = cm[rg][c], u = cv[rg][c];
                const float4 q = make_float4(w.x * w.x, w.y * w.y, w.z * w.z, w.w * w.w);
#pragma unroll
                for (int t = 0; t < 4; t++)
#pragma unroll
                    for (int h = 0; h < H; h++) {
                        acc0[rg][h] = mfma4(comp(w, t), comp(am[h], t), acc0[rg][h]);
                        acc1[rg][h] = mfma4(comp(u, t), comp(as[h], t), acc1[rg][h]);
                        acc1[rg][h] = mfma4(comp(q, t), comp(av[h], t), acc1[rg][h]);
                    }
            }
        }
    };

    // k_per_split is a multiple of two stages and the staged activations are zero
    // beyond the slice, so the loop needs no tail handling; positions are inside
    // the slice, rotated by `rot`.
    const int span = (swz & 2) ? k_per_split : (kr + 2 * KSTEP - 1) / (2 * KSTEP) * (2 * KSTEP);
    auto wrap = [&](int p) { return p >= k_per_split ? p - k_per_split : p; };
    load(sm[0], sv[0], rot);
    __builtin_amdgcn_sched_barrier(0);  // the first weights are on their way while the slice is staged
    stage_slice_pairs<FWD_WAVES * 64>(mu_a, var_a, 4 * H, B, K, k_begin, kr, k_per_split, tid,
                                      [&](int b, int k, float4 m, float4 v) {
                                          *reinterpret_cast<float4 *>(s_mu + b * S + k) = m;
                                          *reinterpret_cast<float4 *>(s_var + b * S + k) = v;
                                      });
    __syncthreads();
    for (int kb = 0; kb < span; kb += 2 * KSTEP) {
        // (the last pair has nothing left to prefetch: it re-reads the stage that
        // was just loaded, which is still in cache, instead of new memory)
        const int p0 = wrap(rot + kb), p1 = p0 + KSTEP;
        const int p2 = kb + 2 * KSTEP < span ? wrap(p0 + 2 * KSTEP) : p1;
        // the barriers keep the scheduler from sinking a stage's loads below the
        // MFMAs they are meant to overlap
        load(sm[1], sv[1], p1);
        __builtin_amdgcn_sched_barrier(0);
        multiply(sm[0], sv[0], p0);
        __builtin_amdgcn_sched_barrier(0);
        load(sm[0], sv[0], p2);
        __builtin_amdgcn_sched_barrier(0);
        multiply(sm[1], sv[1], p1);
        __builtin_amdgcn_sched_barrier(0);
    }

    // sum the 16 blocks (lanes with equal l%4), then lanes 0..3 (sample j = l%4)
    // hold D[row n0+4*rg+v][sample j+4*h] in register v
#pragma unroll
    for (int rg = 0; rg < RG; rg++)
#pragma unroll
        for (int h = 0; h < H; h++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
                float x0 = acc0[rg][h][v], x1 = acc1[rg][h][v];
#pragma unroll
                for (int m = 4; m < 64; m <<= 1) {
                    x0 += __shfl_xor(x0, m);
                    x1 += __shfl_xor(x1, m);
                }
                acc0[rg][h][v] = x0;
                acc1[rg][h][v] = x1;
            }
    if (blk == 0) {
#pragma unroll
        for (int h = 0; h < H; h++) {
            const int b = i + 4 * h;
            if (b >= B) continue;
#pragma unroll
            for (int rg = 0; rg < RG; rg++)
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const int n = n0 + 4 * rg + v;
                    if (n < N) {
                        const size_t at = ((size_t)split * B + b) * N + n;
                        ws0[at] = acc0[rg][h][v];
                        ws1[at] = acc1[rg][h][v];
                    }
                }
        }
    }
}

// ---------------------------------------------------------------------------
// State backward, same instruction. A wave owns 256 consecutive input columns
// (lane l: the float4 at c0 + 4*l, so one load instruction is one contiguous
// kilobyte of a weight row) and a range of output rows n; the MFMA for row n
// multiplies A_blk[i] = w[n][c0 + 16*blk + 4*i + t] by B_blk[j] = delta[j+4*h][n]
// and accumulates over the rows in place: register v of lane (blk, j) of
// accumulator (t, h) is column c0 + 16*blk + 4*v + t of sample j+4*h. The eight
// waves of a workgroup split its row slice and meet in an LDS tree reduction,
// so only gridDim.y partial sums per output reach memory.
// ---------------------------------------------------------------------------
constexpr int DZ_WAVES = 8;
constexpr int DZ_COLS_PER_BLOCK = 256;
constexpr int DZ_STAGE = 8;  // rows in flight per wave and pipeline stage
constexpr int DZ_NSTEP = DZ_WAVES * 2 * DZ_STAGE;  // slices: whole pairs of stages per wave

template <int H>
__global__ __launch_bounds__(DZ_WAVES * 64) void gemv_dz_kernel(
    const float *__restrict__ mu_w, const float *__restrict__ dmu,
    const float *__restrict__ dvar, int K, int N, int B, int n_per_split, int rev,
    float *__restrict__ ws0, float *__restrict__ ws1) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int S = n_per_split + 4;
    float *s_dm = lds, *s_dv = lds + 4 * H * S;

    // rows per pipeline stage: fewer for large batches, whose accumulators need
    // the registers
    constexpr int STAGE = H <= 2 ? DZ_STAGE : DZ_STAGE / 2;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int j = lane & 3;
    // (rev bit 0 walks the row slices from the end of the matrix; no gain measured)
    // Workgroup -> (column slab, row slice). Consecutive workgroup ids go to the 8
    // XCDs round-robin; mode 1 gives each XCD runs of 4 adjacent column slabs (4 KB
    // of every row, i.e. all of its L2 channels) instead of every 8th slab.
    int slab = blockIdx.x, split_raw = blockIdx.y;
    if ((rev & 2) && gridDim.x % 32 == 0) {
        const int id = blockIdx.y * gridDim.x + blockIdx.x;
        const int xcd = id & 7, local = id >> 3;        // local: 0 .. gridDim.x*gridDim.y/8
        const int groups = gridDim.x / 32;               // groups of 32 slabs (8 XCDs x 4)
        const int g = local % groups, rest = local / groups;
        slab = g * 32 + xcd * 4 + (rest & 3);
        split_raw = rest >> 2;
    }
    const int split = (rev & 1) ? gridDim.y - 1 - split_raw : split_raw;
    const int n_begin = split * n_per_split;
    const int nr = min(N, n_begin + n_per_split) - n_begin;

    // Weight loads are never predicated: columns beyond K read column K-4 and are
    // dropped at the end, rows beyond N read row N-1 and meet zero innovations.
    const int col = min(slab * DZ_COLS_PER_BLOCK + 4 * lane, K - 4);
    // rows of this wave: local [r_lo, r_hi)
    const int per_wave = n_per_split / DZ_WAVES;  // multiple of DZ_STAGE
    const int r_lo = wave * per_wave, r_hi = min(nr, r_lo + per_wave);
    const float *w = mu_w + col;
    const int n_last = N - 1;
    // Two register stages used in turn, as in the forward kernel.
    float4 st[2][STAGE];
    auto load = [&](float4(&x)[STAGE], int r) {
#pragma unroll
        for (int u = 0; u < STAGE; u++)
            x[u] = ldw_dz(w + (size_t)min(n_begin + r + u, n_last) * K);
    };
    // stage this slice of the innovations: [sample][n], zero beyond B and nr

    floatx4 acc0[4][H], acc1[4][H];
#pragma unroll
    for (int t = 0; t < 4; t++)
#pragma unroll
        for (int h = 0; h < H; h++) {
            acc0[t][h] = (floatx4){0.f, 0.f, 0.f, 0.f};
            acc1[t][h] = (floatx4){0.f, 0.f, 0.f, 0.f};
        }

    auto multiply = [&](const float4(&cur)[STAGE], int r) {
#pragma unroll
        for (int g = 0; g < STAGE / 4; g++) {
            float4 dm[H], dv[H];
#pragma unroll
            for (int h = 0; h < H; h++) {
                dm[h] = *reinterpret_cast<const float4 *>(s_dm + (j + 4 * h) * S + r + 4 * g);
                dv[h] = *reinterpret_cast<const float4 *>(s_dv + (j + 4 * h) * S + r + 4 * g);
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const float4 x = cur[4 * g + u];
                const float4 q = make_float4(x.x * x.x, x.y * x.y, x.z * x.z, x.w * x.w);
#pragma unroll
                for (int t = 0; t < 4; t++)
#pragma unroll
                    for (int h = 0; h < H; h++) {
                        acc0[t][h] = mfma4(comp(x, t), comp(dm[h], u), acc0[t][h]);
                        acc1[t][h] = mfma4(comp(q, t), comp(dv[h], u), acc1[t][h]);
                    }
            }
        }
    };

    load(st[0], r_lo);
    __builtin_amdgcn_sched_barrier(0);  // the first weights are on their way while the slice is staged
    stage_slice_pairs<DZ_WAVES * 64>(dmu, dvar, 4 * H, B, N, n_begin, nr, n_per_split, tid,
                                     [&](int b, int n, float4 m, float4 v) {
                                         *reinterpret_cast<float4 *>(s_dm + b * S + n) = m;
                                         *reinterpret_cast<float4 *>(s_dv + b * S + n) = v;
                                     });
    __syncthreads();
    for (int r = r_lo; r < r_hi; r += 2 * STAGE) {
        load(st[1], r + STAGE);
        __builtin_amdgcn_sched_barrier(0);
        multiply(st[0], r);
        __builtin_amdgcn_sched_barrier(0);
        // (nothing left to prefetch in the last pair: re-read the cached stage)
        load(st[0], r + 2 * STAGE < r_hi ? r + 2 * STAGE : r + STAGE);
        __builtin_amdgcn_sched_barrier(0);
        multiply(st[1], r + STAGE);
        __builtin_amdgcn_sched_barrier(0);
    }

    // tree reduction over the 8 waves through LDS (reusing the staging area):
    // slot layout [slot][value][lane]
    constexpr int NV = 4 * H * 4 * 2;  // values per lane
    __syncthreads();
    float *slot = lds;
#pragma unroll
    for (int half = DZ_WAVES / 2; half >= 1; half >>= 1) {
        if (wave >= half && wave < 2 * half) {
            float *dst = slot + (size_t)(wave - half) * NV * 64 + lane;
#pragma unroll
            for (int t = 0; t < 4; t++)
#pragma unroll
                for (int h = 0; h < H; h++)
#pragma unroll
                    for (int v = 0; v < 4; v++) {
                        dst[((t * H + h) * 4 + v) * 2 * 64] = acc0[t][h][v];
                        dst[(((t * H + h) * 4 + v) * 2 + 1) * 64] = acc1[t][h][v];
                    }
        }
        __syncthreads();
        if (wave < half) {
            const float *src = slot + (size_t)wave * NV * 64 + lane;
#pragma unroll
            for (int t = 0; t < 4; t++)
#pragma unroll
                for (int h = 0; h < H; h++)
#pragma unroll
                    for (int v = 0; v < 4; v++) {
                        acc0[t][h][v] += src[((t * H + h) * 4 + v) * 2 * 64];
                        acc1[t][h][v] += src[(((t * H + h) * 4 + v) * 2 + 1) * 64];
                    }
        }
        __syncthreads();
    }

    if (wave == 0) {
        const int blk = lane >> 2;
        const int c = slab * DZ_COLS_PER_BLOCK + 16 * blk;
#pragma unroll
        for (int h = 0; h < H; h++) {
            const int b = j + 4 * h;
            if (b >= B) continue;
            const size_t base = ((size_t)split * B + b) * K + c;
#pragma unroll
            for (int v = 0; v < 4; v++) {
                if (c + 4 * v < K) {  // K % 4 == 0 on this path
                    *reinterpret_cast<float4 *>(ws0 + base + 4 * v) = make_float4(
                        acc0[0][h][v], acc0[1][h][v], acc0[2][h][v], acc0[3][h][v]);
                    *reinterpret_cast<float4 *>(ws1 + base + 4 * v) = make_float4(
                        acc1[0][h][v], acc1[1][h][v], acc1[2][h][v], acc1[3][h][v]);
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Weight backward. delta_w[n][k'] = var_w[n][k'] * sum_b delta[b][n] * a[b][k'].
// A lane keeps a[b][k'..k'+3] and its squares for all b in registers and walks
// rows; the 2*B innovations of a row are wave-uniform and come from LDS as
// broadcast reads. Per row a wave reads 1 KB of var_w and writes 2 KB
// (non-temporal: the results are not read again by this kernel).
//
// Workgroups are small (16 rows x 256 columns, a wave loads its 4 rows at once,
// then multiplies and stores them) and are numbered along the rows of the matrix
// first: the workgroups resident at any time then sweep a narrow band of rows
// through var_w and the two results in address order. Measured at 8192 x 8192,
// batch 8, forward + backward step: 128 rows per workgroup 283 us, 32 rows 274 us,
// 16 rows 268 us, 8 rows 279 us.
//
// EXACT (K % 256 == 0 and N % 16 == 0): no predicate anywhere. The general
// variant guards every row and column.
// ---------------------------------------------------------------------------
constexpr int DW_COLS_PER_BLOCK = 256;  // 64 lanes x 4 columns, shared by the 4 waves
constexpr int DW_ROWS_PER_BLOCK = 16;   // 4 rows per wave
constexpr int DW_STAGE = 4;             // rows a wave has in flight per register stage

template <int BMAX>
__device__ __forceinline__ void dw_row(const float4 &vw, const float (*s_dm)[BMAX],
                                       const float (*s_dv)[BMAX], int r, const float4 (&a)[BMAX],
                                       const float4 (&a2)[BMAX], float *pm, float *pv) {
    float4 sm = zero4(), sv = zero4();
#pragma unroll
    for (int b = 0; b < BMAX; b++) {
        const float d0 = s_dm[r][b], d1 = s_dv[r][b];
        sm.x += d0 * a[b].x; sm.y += d0 * a[b].y; sm.z += d0 * a[b].z; sm.w += d0 * a[b].w;
        sv.x += d1 * a2[b].x; sv.y += d1 * a2[b].y; sv.z += d1 * a2[b].z; sv.w += d1 * a2[b].w;
    }
    const floatx4 om = {sm.x * vw.x, sm.y * vw.y, sm.z * vw.z, sm.w * vw.w};
    const floatx4 ov = {sv.x * vw.x * vw.x, sv.y * vw.y * vw.y, sv.z * vw.z * vw.z,
                        sv.w * vw.w * vw.w};
    __builtin_nontemporal_store(om, reinterpret_cast<floatx4 *>(pm));
    __builtin_nontemporal_store(ov, reinterpret_cast<floatx4 *>(pv));
}

template <int BMAX, bool EXACT>
__global__ __launch_bounds__(256) void gemv_dw_kernel(
    const float *__restrict__ var_w, const float *__restrict__ mu_a,
    const float *__restrict__ dmu, const float *__restrict__ dvar, int K, int N, int B, int rev,
    float *__restrict__ dmu_w, float *__restrict__ dvar_w, const float *__restrict__ var_b,
    float *__restrict__ dmu_b, float *__restrict__ dvar_b, DzFold fold, int col_blocks,
    int nfold) {
    constexpr int ROWS = DW_ROWS_PER_BLOCK;
    __shared__ __attribute__((aligned(16))) float s_dm[ROWS][BMAX];
    __shared__ __attribute__((aligned(16))) float s_dv[ROWS][BMAX];
    // The state backward that ran before this kernel may have left its slices
    // unfolded. The first nfold workgroups of the (one-dimensional) grid, the first
    // to be dispatched, do nothing but fold them, one float4 of the result per
    // thread and round, while the other workgroups already stream; that saves a
    // launch, and no streaming workgroup waits for the fold's dependent loads.
    int id = blockIdx.x;
    if (id < nfold) {
        const size_t items = fold.total / 4;
        for (size_t it = (size_t)id * 256 + threadIdx.x; it < items; it += (size_t)nfold * 256) {
            const size_t at = it * 4;
            float4 m = zero4(), v = zero4();
            int sl = 0;
            for (; sl + 4 <= fold.splits; sl += 4) {
                float4 x[4], y[4];
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    x[u] = ld4(fold.ws0 + (sl + u) * fold.total + at);
                    y[u] = ld4(fold.ws1 + (sl + u) * fold.total + at);
                }
#pragma unroll
                for (int u = 0; u < 4; u++) {  // slices are added in index order
                    m.x += x[u].x; m.y += x[u].y; m.z += x[u].z; m.w += x[u].w;
                    v.x += y[u].x; v.y += y[u].y; v.z += y[u].z; v.w += y[u].w;
                }
            }
            for (; sl < fold.splits; sl++) {
                const float4 a = ld4(fold.ws0 + sl * fold.total + at);
                const float4 b = ld4(fold.ws1 + sl * fold.total + at);
                m.x += a.x; m.y += a.y; m.z += a.z; m.w += a.w;
                v.x += b.x; v.y += b.y; v.z += b.z; v.w += b.w;
            }
            const float4 j = ld4(fold.jcb + at);
            *reinterpret_cast<float4 *>(fold.out0 + at) =
                make_float4(m.x * j.x, m.y * j.y, m.z * j.z, m.w * j.w);
            *reinterpret_cast<float4 *>(fold.out1 + at) = make_float4(
                v.x * (j.x * j.x), v.y * (j.y * j.y), v.z * (j.z * j.z), v.w * (j.w * j.w));
        }
        return;
    }
    id -= nfold;  // a multiple of 8 (launcher): the id's XCD (id % 8) stays
    const int grid_rows = ((int)gridDim.x - nfold) / col_blocks;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // same XCD-aware choice of the column block as in the state backward
    int cblock = id % col_blocks, rblock = id / col_blocks;
    if ((rev & 2) && col_blocks % 32 == 0) {
        const int xcd = id & 7, local = id >> 3;
        const int groups = col_blocks / 32;
        const int g = local % groups, rest = local / groups;
        cblock = g * 32 + xcd * 4 + (rest & 3);
        rblock = rest >> 2;
    }
    const int col = cblock * DW_COLS_PER_BLOCK + lane * 4;
    const int n0 = ((rev & 1) ? grid_rows - 1 - rblock : rblock) * ROWS;

    constexpr int RPW = ROWS / 4;  // rows per wave
    constexpr int STAGE = RPW < DW_STAGE ? RPW : DW_STAGE;
    const int r0 = wave * RPW;
    const float *src = var_w + (size_t)(n0 + r0) * K + col;
    float4 st[2][STAGE];
    auto load = [&](float4(&x)[STAGE], int rr) {
#pragma unroll
        for (int u = 0; u < STAGE; u++) x[u] = ldw_dw(src + (size_t)(rr + u) * K);
    };
    for (int e = threadIdx.x; e < ROWS * BMAX; e += 256) {
        const int b = e / ROWS, r = e % ROWS;
        const bool ok = b < B && n0 + r < N;
        s_dm[r][b] = ok ? dmu[(size_t)b * N + n0 + r] : 0.f;
        s_dv[r][b] = ok ? dvar[(size_t)b * N + n0 + r] : 0.f;
    }

    const bool col_ok = EXACT || col < K;  // K % 4 == 0 on this path
    float4 a[BMAX], a2[BMAX];
#pragma unroll
    for (int b = 0; b < BMAX; b++) {
        a[b] = (col_ok && b < B) ? ld4(mu_a + (size_t)b * K + col) : zero4();
        a2[b] = make_float4(a[b].x * a[b].x, a[b].y * a[b].y, a[b].z * a[b].z, a[b].w * a[b].w);
    }
    __syncthreads();

    // Bias innovations ride along: the staged innovations of this row block are
    // all that delta_b needs, so the first column block folds them over the batch.
    if (var_b != nullptr && cblock == 0) {
        for (int r = threadIdx.x; r < ROWS && n0 + r < N; r += 256) {
            float sm = 0.f, sv = 0.f;
#pragma unroll
            for (int b = 0; b < BMAX; b++) {
                sm += s_dm[r][b];
                sv += s_dv[r][b];
            }
            const float vb = var_b[n0 + r];
            dmu_b[n0 + r] = sm * vb;
            dvar_b[n0 + r] = sv * vb * vb;
        }
    }

    if (EXACT) {
        float *dm = dmu_w + (size_t)(n0 + r0) * K + col;
        float *dv = dvar_w + (size_t)(n0 + r0) * K + col;
        auto flush = [&](const float4(&x)[STAGE], int rr) {
#pragma unroll
            for (int u = 0; u < STAGE; u++)
                dw_row<BMAX>(x[u], s_dm, s_dv, r0 + rr + u, a, a2, dm + (size_t)(rr + u) * K,
                             dv + (size_t)(rr + u) * K);
        };
        static_assert(RPW % STAGE == 0, "whole stages per wave");
        load(st[0], 0);
#pragma unroll 1
        for (int rr = 0; rr < RPW; rr += 2 * STAGE) {
            const bool second = rr + STAGE < RPW;
            if (second) load(st[1], rr + STAGE);
            __builtin_amdgcn_sched_barrier(0);
            flush(st[0], rr);
            __builtin_amdgcn_sched_barrier(0);
            if (rr + 2 * STAGE < RPW) load(st[0], rr + 2 * STAGE);
            __builtin_amdgcn_sched_barrier(0);
            if (second) flush(st[1], rr + STAGE);
            __builtin_amdgcn_sched_barrier(0);
        }
    } else {
        if (!col_ok) return;
        // all rows of the wave are requested before the first store (a load that
        // follows a store would wait for it)
        float4 vw[RPW];
#pragma unroll
        for (int rr = 0; rr < RPW; rr++) {
            const int n = n0 + r0 + rr;
            vw[rr] = n < N ? ld4(var_w + (size_t)n * K + col) : zero4();
        }
#pragma unroll
        for (int rr = 0; rr < RPW; rr++) {
            const int n = n0 + r0 + rr;
            if (n < N)
                dw_row<BMAX>(vw[rr], s_dm, s_dv, r0 + rr, a, a2, dmu_w + (size_t)n * K + col,
                             dvar_w + (size_t)n * K + col);
        }
    }
}

}  // namespace

// Forward variants by index: row groups per wave (their chunks per stage are
// 1, 2, 2, 4: see the launcher's switch).
constexpr int FWD_VARIANTS = 5;
static const int kFwdRG[FWD_VARIANTS] = {2, 2, 1, 1, 1};

int gemv_fwd_variants() { return FWD_VARIANTS; }
int gemv_fwd_rows_per_block(int variant) { return FWD_WAVES * kFwdRG[variant] * 4; }
int gemv_fwd_k_step() { return FWD_KROUND; }
int gemv_dz_cols_per_block() { return DZ_COLS_PER_BLOCK; }
int gemv_dz_n_step() { return DZ_NSTEP; }

// Largest reduction slice whose staged activations / innovations fit in LDS.
int gemv_fwd_max_slice(int B) {
    const int H = (B + 3) / 4;
    return (72 * 1024 / (2 * 4 * H * 4) - FWD_LDS_PAD) / FWD_KROUND * FWD_KROUND;
}
int gemv_dz_max_slice(int B) {
    const int H = (B + 3) / 4;
    return (72 * 1024 / (2 * 4 * H * 4) - 4) / DZ_NSTEP * DZ_NSTEP;
}

template <int H, int RG, int C>
static hipError_t fwd_launch(const float *mu_w, const float *var_w, const float *mu_a,
                             const float *var_a, int K, int N, int B, int per, int splits,
                             int swz, float *ws0, float *ws1, hipStream_t stream) {
    const size_t lds = (size_t)2 * 4 * H * (per + FWD_LDS_PAD) * sizeof(float);
    static PerDeviceOnce once;
    hipError_t e = allow_dynamic_lds(once, reinterpret_cast<const void *>(gemv_fwd_kernel<H, RG, C>), 160 * 1024);
    if (e != hipSuccess) return e;
    constexpr int rows = FWD_WAVES * RG * 4;
    dim3 grid(((N + rows - 1) / rows) * splits), block(FWD_WAVES * 64);
    hipLaunchKernelGGL((gemv_fwd_kernel<H, RG, C>), grid, block, lds, stream, mu_w, var_w, mu_a,
                       var_a, K, N, B, per, splits, swz, ws0, ws1);
    return hipGetLastError();
}

template <int H>
static hipError_t fwd_variant(int variant, const float *mu_w, const float *var_w,
                              const float *mu_a, const float *var_a, int K, int N, int B, int per,
                              int splits, int swz, float *ws0, float *ws1, hipStream_t stream) {
    switch (variant) {
        case 0: return fwd_launch<H, 2, 1>(mu_w, var_w, mu_a, var_a, K, N, B, per, splits, swz, ws0, ws1, stream);
        case 1: return fwd_launch<H, 2, 2>(mu_w, var_w, mu_a, var_a, K, N, B, per, splits, swz, ws0, ws1, stream);
        case 2: return fwd_launch<H, 1, 2>(mu_w, var_w, mu_a, var_a, K, N, B, per, splits, swz, ws0, ws1, stream);
        case 3: return fwd_launch<H, 1, 4>(mu_w, var_w, mu_a, var_a, K, N, B, per, splits, swz, ws0, ws1, stream);
        case 4: return fwd_launch<H, 1, 1>(mu_w, var_w, mu_a, var_a, K, N, B, per, splits, swz, ws0, ws1, stream);
    }
    return hipErrorInvalidValue;
}

hipError_t launch_gemv_fwd(const float *mu_w, const float *var_w, const float *mu_a,
                           const float *var_a, int K, int N, int B, int splits, int swz,
                           int variant, float *ws0, float *ws1, hipStream_t stream) {
    int per = (K + splits - 1) / splits;
    per = (per + FWD_KROUND - 1) / FWD_KROUND * FWD_KROUND;
    if (per > gemv_fwd_max_slice(B) || variant < 0 || variant >= FWD_VARIANTS)
        return hipErrorInvalidValue;
    switch ((B + 3) / 4) {
        case 1: return fwd_variant<1>(variant, mu_w, var_w, mu_a, var_a, K, N, B, per, splits, swz, ws0, ws1, stream);
        case 2: return fwd_variant<2>(variant, mu_w, var_w, mu_a, var_a, K, N, B, per, splits, swz, ws0, ws1, stream);
        case 3: return fwd_variant<3>(variant, mu_w, var_w, mu_a, var_a, K, N, B, per, splits, swz, ws0, ws1, stream);
        case 4: return fwd_variant<4>(variant, mu_w, var_w, mu_a, var_a, K, N, B, per, splits, swz, ws0, ws1, stream);
    }
    return hipErrorInvalidValue;
}

template <int H>
static hipError_t dz_launch(const float *mu_w, const float *dmu, const float *dvar, int K, int N,
                            int B, int per, int splits, int rev, float *ws0, float *ws1,
                            hipStream_t stream) {
    size_t lds = (size_t)2 * 4 * H * (per + 4) * sizeof(float);
    const size_t red = (size_t)(DZ_WAVES / 2) * (4 * H * 4 * 2) * 64 * sizeof(float);
    if (red > lds) lds = red;
    static PerDeviceOnce once;
    hipError_t e = allow_dynamic_lds(once, reinterpret_cast<const void *>(gemv_dz_kernel<H>), 160 * 1024);
    if (e != hipSuccess) return e;
    dim3 grid((K + DZ_COLS_PER_BLOCK - 1) / DZ_COLS_PER_BLOCK, splits), block(DZ_WAVES * 64);
    hipLaunchKernelGGL(gemv_dz_kernel<H>, grid, block, lds, stream, mu_w, dmu, dvar, K, N, B, per,
                       rev, ws0, ws1);
    return hipGetLastError();
}

hipError_t launch_gemv_dz(const float *mu_w, const float *dmu, const float *dvar, int K, int N,
                          int B, int splits, int rev, float *ws0, float *ws1,
                          hipStream_t stream) {
    int per = (N + splits - 1) / splits;
    per = (per + DZ_NSTEP - 1) / DZ_NSTEP * DZ_NSTEP;
    if (per > gemv_dz_max_slice(B)) return hipErrorInvalidValue;
    switch ((B + 3) / 4) {
        case 1: return dz_launch<1>(mu_w, dmu, dvar, K, N, B, per, splits, rev, ws0, ws1, stream);
        case 2: return dz_launch<2>(mu_w, dmu, dvar, K, N, B, per, splits, rev, ws0, ws1, stream);
        case 3: return dz_launch<3>(mu_w, dmu, dvar, K, N, B, per, splits, rev, ws0, ws1, stream);
        case 4: return dz_launch<4>(mu_w, dmu, dvar, K, N, B, per, splits, rev, ws0, ws1, stream);
    }
    return hipErrorInvalidValue;
}

template <int BMAX>
static void dw_launch(const float *var_w, const float *mu_a, const float *dmu, const float *dvar,
                      int K, int N, int B, int rev, float *dmu_w, float *dvar_w,
                      const float *var_b, float *dmu_b, float *dvar_b, const DzFold &fold,
                      hipStream_t stream) {
    const int col_blocks = (K + DW_COLS_PER_BLOCK - 1) / DW_COLS_PER_BLOCK;
    const int row_blocks = (N + DW_ROWS_PER_BLOCK - 1) / DW_ROWS_PER_BLOCK;
    const bool exact = (K % DW_COLS_PER_BLOCK == 0) && (N % DW_ROWS_PER_BLOCK == 0);
    // workgroups that only fold the state backward's slices: 64, or as many as one
    // float4 of the result per thread asks for
    int nfold = 0;
    if (fold.ws0 != nullptr) {
        const size_t wgs = (fold.total / 4 + 255) / 256;
        nfold = wgs < 64 ? (int)((wgs + 7) / 8 * 8) : 64;
    }
    const dim3 grid((unsigned)((size_t)col_blocks * row_blocks + nfold));
    if (exact)
        hipLaunchKernelGGL((gemv_dw_kernel<BMAX, true>), grid, dim3(256), 0, stream, var_w, mu_a,
                           dmu, dvar, K, N, B, rev, dmu_w, dvar_w, var_b, dmu_b, dvar_b, fold,
                           col_blocks, nfold);
    else
        hipLaunchKernelGGL((gemv_dw_kernel<BMAX, false>), grid, dim3(256), 0, stream, var_w, mu_a,
                           dmu, dvar, K, N, B, rev, dmu_w, dvar_w, var_b, dmu_b, dvar_b, fold,
                           col_blocks, nfold);
}

hipError_t launch_gemv_dw(const float *var_w, const float *mu_a, const float *dmu,
                          const float *dvar, int K, int N, int B, int rev, float *dmu_w,
                          float *dvar_w, const float *var_b, float *dmu_b, float *dvar_b,
                          const DzFold *fold_in, hipStream_t stream) {
    const DzFold fold = fold_in ? *fold_in : DzFold();
    if (B > 16) return hipErrorInvalidValue;  // the kernels hold at most 16 samples
    if (B <= 4)
        dw_launch<4>(var_w, mu_a, dmu, dvar, K, N, B, rev, dmu_w, dvar_w, var_b, dmu_b, dvar_b,
                     fold, stream);
    else if (B <= 8)
        dw_launch<8>(var_w, mu_a, dmu, dvar, K, N, B, rev, dmu_w, dvar_w, var_b, dmu_b, dvar_b,
                     fold, stream);
    else
        dw_launch<16>(var_w, mu_a, dmu, dvar, K, N, B, rev, dmu_w, dvar_w, var_b, dmu_b, dvar_b,
                      fold, stream);
    return hipGetLastError();
}

}  // namespace tagi

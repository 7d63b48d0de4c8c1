// Skinny-batch kernels of the TAGI Linear layer on 16-wide MFMAs, gfx950: the forward
// for every batch up to 32 (two groups of sixteen samples beyond 16), the state
// backward for 9 <= B <= 16.
//
// Same plan as tagi_gemv.hip (the weight matrices stream from HBM once, straight
// into MFMA operand layout; the few activations / innovations sit in LDS), but on
// v_mfma_f32_16x16x4_f32: one instruction multiplies a 16 x 4 weight fragment by
// all (up to) 16 samples, so a wave needs a quarter of the instructions, LDS
// reads and accumulator registers that sixteen 4x4 blocks of four samples need.
// Operand layout of the instruction: A[i][k] from lane 16*k + i, B[k][j] from
// lane 16*k + j, D[4*(l/16) + v][l%16] in register v of lane l.
//
// The weight backward of tagi_gemv.hip serves every B <= 16 and is not repeated.
#include "tagi_internal.h"
#include "tagi_stage.h"

namespace tagi {

typedef float floatx4 __attribute__((ext_vector_type(4)));

namespace {

__device__ __forceinline__ float4 ld4(const float *p) {
    return *reinterpret_cast<const float4 *>(p);
}
__device__ __forceinline__ float4 ldnt4(const float *p) {
    const floatx4 v = __builtin_nontemporal_load(reinterpret_cast<const floatx4 *>(p));
    return make_float4(v[0], v[1], v[2], v[3]);
}
// Lanes of the banks in BANKS (a bank = four lanes of a row of sixteen) take `from` of
// the lane eight further round the row; the others keep `keep`.
template <int BANKS>
__device__ __forceinline__ float take_ror8(float keep, float from) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(keep), __float_as_int(from),
                                                      0x128 /* row_ror:8 */, 0xF, BANKS, false));
}
// a: loaded by lane (i, kk) from row i % 8 of the group, b: from row 8 + i % 8, both at
// chunk kk + 4 * (i / 8) of the 32-element window. Afterwards a is chunk kk and b chunk
// kk + 4 of row i: lanes i < 8 keep a and take b from the a of lane i + 8, lanes i >= 8
// keep b and take a from the b of lane i - 8.
__device__ __forceinline__ void swap_halves(float4 &a, float4 &b) {
    const float4 a0 = a;
    a.x = take_ror8<0xC>(a0.x, b.x);
    a.y = take_ror8<0xC>(a0.y, b.y);
    a.z = take_ror8<0xC>(a0.z, b.z);
    a.w = take_ror8<0xC>(a0.w, b.w);
    b.x = take_ror8<0x3>(b.x, a0.x);
    b.y = take_ror8<0x3>(b.y, a0.y);
    b.z = take_ror8<0x3>(b.z, a0.z);
    b.w = take_ror8<0x3>(b.w, a0.w);
}
__device__ __forceinline__ float4 zero4() { return make_float4(0.f, 0.f, 0.f, 0.f); }
__device__ __forceinline__ float comp(const float4 &v, int t) {
    return t == 0 ? v.x : t == 1 ? v.y : t == 2 ? v.z : v.w;
}
__device__ __forceinline__ float4 sq4(const float4 &v) {
    return make_float4(v.x * v.x, v.y * v.y, v.z * v.z, v.w * v.w);
}
__device__ __forceinline__ floatx4 mfma16(float a, float b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

constexpr int W16_SAMPLES = 16;

// ---------------------------------------------------------------------------
// Forward. Lane (i = l%16, kk = l/16) streams weight row n0 + 16*rg + i and
// holds the float4 at k = kb + 4*kk: one load instruction covers 16 rows x 64
// bytes, two of them a full 128-byte line of each row (plain loads: with
// streaming loads the second half of a line was fetched from memory again, 1.5x
// the traffic). Component t of that
// float4 is A[i][kk] of MFMA t, which multiplies reduction elements
// kb + 4*kk + t against B[kk][j] = the same elements of sample j = l%16, read
// from LDS as one float4 per lane. The sums over k are complete inside the
// accumulators: D[row][sample], no cross-lane reduction at the end.
// ---------------------------------------------------------------------------
// (measured at 8192 x 8192, batch 16, forward call: RG x C = 1x2 118 us, 2x2 120,
// 1x4 121, 2x4 124, 4x1 136, 1x8 138)
constexpr int F16_RG = 1;        // groups of 16 rows per wave
constexpr int F16_C = 2;         // 16-element chunks per row and register stage
constexpr int F16_KSTEP = 16 * F16_C;
constexpr int F16_PAD = 4;       // LDS row stride % 32 == 4

// NG: groups of 16 samples (1: up to 16 samples, 2: up to 32 - every weight fragment
// then feeds two MFMAs, one per group, from the same registers).
// WL: load instructions cover whole 128-byte lines (8 rows x 128 bytes each, two of them
// for the wave's sixteen rows) with streaming loads; lanes i and i ^ 8 then exchange one
// float4 each to arrive at the operand layout (see swap_halves).
// WAVES: 16 (one workgroup per CU, 256 rows share a staged slice) where that still gives
// every CU a workgroup, 8 on smaller matrices.
template <int NG, int WL, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void gemv16_fwd_kernel(
    const float *__restrict__ mu_w, const float *__restrict__ var_w,
    const float *__restrict__ mu_a, const float *__restrict__ var_a, int K, int N, int B,
    int k_per_split, int splits, float *__restrict__ ws0, float *__restrict__ ws1) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int RG = F16_RG, C = F16_C, KSTEP = F16_KSTEP;
    constexpr int ROWS_PER_BLOCK = WAVES * RG * 16;
    constexpr int NS = NG * W16_SAMPLES;
    const int S = k_per_split + F16_PAD;
    float *s_mu = lds, *s_var = lds + NS * S;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int i = lane & 15, kk = lane >> 4;
    // consecutive workgroup ids go to the 8 XCDs round-robin: the slice is the fast
    // index inside an XCD, so an XCD's workgroups cover all windows of a weight row
    int row_block, split;
    const int id = blockIdx.x, row_blocks = gridDim.x / splits;
    if (row_blocks % 8 == 0) {
        const int xcd = id & 7, local = id >> 3;
        split = local % splits;
        row_block = (local / splits) * 8 + xcd;
    } else {
        row_block = id % row_blocks;
        split = id / row_blocks;
    }
    const int k_begin = split * k_per_split;
    const int kr = min(K, k_begin + k_per_split) - k_begin;
    // each wave walks its slice from a different starting point (sums commute)
    const int rot = ((row_block * WAVES + wave) * 2 * KSTEP) % k_per_split;

    // stage the slice of the activations: [sample][k], zero beyond B and kr

    // Weight loads are never predicated: rows beyond N read row N-1 and are
    // dropped at the end, reduction elements beyond the slice read the last float4
    // of the row and meet zero activations.
    const int n0 = row_block * ROWS_PER_BLOCK + wave * (RG * 16);
    // WL: wm / wv point at row (i % 8) of the group's first eight rows, the second
    // eight lie `hi` floats further; the lane's chunk of the 32-element window is
    // kk + 4 * (i / 8)
    const float *wm[RG], *wv[RG];
    size_t hi[RG];
#pragma unroll
    for (int rg = 0; rg < RG; rg++) {
        const int row = min(n0 + 16 * rg + (WL ? (i & 7) : i), N - 1);
        wm[rg] = mu_w + (size_t)row * K;
        wv[rg] = var_w + (size_t)row * K;
        hi[rg] = (size_t)(min(n0 + 16 * rg + 8 + (i & 7), N - 1) - row) * K;
    }
    const int k_lane = k_begin + 4 * (WL ? kk + 4 * (i >> 3) : kk), k_last = K - 4;

    // the two variance terms have accumulators of their own, so that no MFMA waits
    // for the one issued just before it
    floatx4 acc0[NG][RG], acc1[NG][RG], acc2[NG][RG];
#pragma unroll
    for (int g = 0; g < NG; g++)
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            acc0[g][rg] = (floatx4){0.f, 0.f, 0.f, 0.f};
            acc1[g][rg] = acc0[g][rg];
            acc2[g][rg] = acc0[g][rg];
        }

    float4 sm[2][RG][C], sv[2][RG][C];
    auto load = [&](float4(&m)[RG][C], float4(&v)[RG][C], int kb) {
        if (WL) {
            static_assert(!WL || C % 2 == 0, "a 128-byte line is two chunks of 16 elements");
#pragma unroll
            for (int c = 0; c < C; c += 2) {
                const int k = min(k_lane + kb + 16 * c, k_last);
#pragma unroll
                for (int rg = 0; rg < RG; rg++) {
                    m[rg][c] = (WL == 1 || WL == 4) ? ldnt4(wm[rg] + k) : ld4(wm[rg] + k);
                    v[rg][c] = (WL == 1 || WL == 3) ? ldnt4(wv[rg] + k) : ld4(wv[rg] + k);
                    m[rg][c + 1] = (WL == 1 || WL == 4) ? ldnt4(wm[rg] + hi[rg] + k) : ld4(wm[rg] + hi[rg] + k);
                    v[rg][c + 1] = (WL == 1 || WL == 3) ? ldnt4(wv[rg] + hi[rg] + k) : ld4(wv[rg] + hi[rg] + k);
                }
            }
            return;
        }
#pragma unroll
        for (int c = 0; c < C; c++) {
            const int k = min(k_lane + kb + 16 * c, k_last);
#pragma unroll
            for (int rg = 0; rg < RG; rg++) {
                m[rg][c] = ld4(wm[rg] + k);
                v[rg][c] = ld4(wv[rg] + k);
            }
        }
    };
    auto multiply = [&](float4(&cm)[RG][C], float4(&cv)[RG][C], int kb) {
        if (WL) {
#pragma unroll
            for (int c = 0; c < C; c += 2)
#pragma unroll
                for (int rg = 0; rg < RG; rg++) {
                    swap_halves(cm[rg][c], cm[rg][c + 1]);
                    swap_halves(cv[rg][c], cv[rg][c + 1]);
                }
        }
#pragma unroll
        for (int c = 0; c < C; c++) {
            const int at = kb + 16 * c + 4 * kk;
            float4 am[NG], av[NG], as[NG];
#pragma unroll
            for (int g = 0; g < NG; g++) {
                am[g] = *reinterpret_cast<const float4 *>(s_mu + (16 * g + i) * S + at);
                av[g] = *reinterpret_cast<const float4 *>(s_var + (16 * g + i) * S + at);
                as[g] = make_float4(av[g].x + am[g].x * am[g].x, av[g].y + am[g].y * am[g].y,
                                    av[g].z + am[g].z * am[g].z, av[g].w + am[g].w * am[g].w);
            }
#pragma unroll
            for (int rg = 0; rg < RG; rg++) {
                const float4 w = cm[rg][c], u = cv[rg][c];
                const float4 q = sq4(w);
#pragma unroll
                for (int t = 0; t < 4; t++)
#pragma unroll
                    for (int g = 0; g < NG; g++) {
                        acc0[g][rg] = mfma16(comp(w, t), comp(am[g], t), acc0[g][rg]);
                        acc1[g][rg] = mfma16(comp(u, t), comp(as[g], t), acc1[g][rg]);
                        acc2[g][rg] = mfma16(comp(q, t), comp(av[g], t), acc2[g][rg]);
                    }
            }
        }
    };

    // k_per_split is a multiple of two stages; positions are inside the slice,
    // rotated by `rot`
    auto wrap = [&](int p) { return p >= k_per_split ? p - k_per_split : p; };
    load(sm[0], sv[0], rot);
    __builtin_amdgcn_sched_barrier(0);  // the first weights are on their way while the slice is staged
    stage_slice_pairs<WAVES * 64>(mu_a, var_a, NS, B, K, k_begin, kr, k_per_split, tid,
                                      [&](int b, int k, float4 m, float4 v) {
                                          *reinterpret_cast<float4 *>(s_mu + b * S + k) = m;
                                          *reinterpret_cast<float4 *>(s_var + b * S + k) = v;
                                      });
    __syncthreads();
    for (int kb = 0; kb < k_per_split; kb += 2 * KSTEP) {
        const int p0 = wrap(rot + kb), p1 = p0 + KSTEP;
        // (the last pair has nothing left to prefetch: it re-reads a cached stage)
        const int p2 = kb + 2 * KSTEP < k_per_split ? wrap(p0 + 2 * KSTEP) : p1;
        load(sm[1], sv[1], p1);
        __builtin_amdgcn_sched_barrier(0);
        multiply(sm[0], sv[0], p0);
        __builtin_amdgcn_sched_barrier(0);
        load(sm[0], sv[0], p2);
        __builtin_amdgcn_sched_barrier(0);
        multiply(sm[1], sv[1], p1);
        __builtin_amdgcn_sched_barrier(0);
    }

    // register v of lane l: row n0 + 16*rg + 4*(l/16) + v, sample 16*g + l%16
#pragma unroll
    for (int g = 0; g < NG; g++) {
        const int b = 16 * g + (lane & 15);
        if (b >= B) continue;
        const bool vec = (N & 3) == 0;
#pragma unroll
        for (int rg = 0; rg < RG; rg++) {
            const int n = n0 + 16 * rg + 4 * (lane >> 4);
            const size_t at = ((size_t)split * B + b) * N + n;
            const floatx4 m = acc0[g][rg], v = acc1[g][rg] + acc2[g][rg];
            if (vec && n + 3 < N) {
                *reinterpret_cast<float4 *>(ws0 + at) = make_float4(m[0], m[1], m[2], m[3]);
                *reinterpret_cast<float4 *>(ws1 + at) = make_float4(v[0], v[1], v[2], v[3]);
            } else {
#pragma unroll
                for (int c = 0; c < 4; c++)
                    if (n + c < N) {
                        ws0[at + c] = m[c];
                        ws1[at + c] = v[c];
                    }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// State backward. A wave owns 64 consecutive input columns; the eight waves of a
// workgroup sit side by side (512 columns) and walk the same slice of output
// rows, so the staged innovations of the slice serve all of them and no wave
// shares an output with another. Lane (i = l%16, kk = l/16) holds the float4 at
// row n + kk, columns c0 + 4*i ..: one load instruction covers 4 rows x 256
// bytes. MFMA t takes A[i][kk] = w[n+kk][c0 + 4*i + t] and B[kk][j] =
// delta[j][n+kk] and accumulates over the rows in place; register v of lane l of
// accumulator t is column c0 + 16*(l/16) + 4*v + t of sample l%16. The
// innovations are staged as [sample][kk][step] (step = row/4), so that a lane
// reads four steps' worth of its B operands as one float4.
// ---------------------------------------------------------------------------
constexpr int Z16_ST = 4;      // 4-row steps per register stage (= steps per LDS float4)
constexpr int Z16_PADQ = 1;    // plane stride per/4 + 4: spreads the kk planes over the banks
constexpr int Z16_WAVES = 8;   // side by side, 64 columns each (4 measured slower)
constexpr int Z16_COLS = Z16_WAVES * 64;

// (Measured and left out, 8192^2, batch 16, per call: streaming loads for the weights 60
// against 57 us; sixteen waves side by side 74 us; sixteen waves as two halves of the
// slice's rows that meet in LDS 58 against 56 us.)
template <int NG>
__global__ __launch_bounds__(Z16_WAVES * 64) void gemv16_dz_kernel(
    const float *__restrict__ mu_w, const float *__restrict__ dmu,
    const float *__restrict__ dvar, int K, int N, int B, int n_per_split,
    float *__restrict__ ws0, float *__restrict__ ws1) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int ST = Z16_ST;
    constexpr int NS = NG * W16_SAMPLES;
    // the float4 of B operands must start at a multiple of 4 steps: Q % 4 == 0
    const int Q = n_per_split / 4 + 4 * Z16_PADQ;  // steps per (sample, kk) plane
    const int S = 4 * Q;                           // floats per sample
    float *s_dm = lds, *s_dv = lds + NS * S;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int i = lane & 15, kk = lane >> 4;
    const int slab = blockIdx.x, split = blockIdx.y;
    const int n_begin = split * n_per_split;
    const int n_last = N - 1;

    // columns beyond K read column K-4 and are dropped at the end; rows beyond N
    // read row N-1 and meet zero innovations
    const int c0 = slab * Z16_COLS + wave * 64;
    const float *w = mu_w + min(c0 + 4 * i, K - 4);

    const int steps = n_per_split / 4;  // multiple of 2*ST
    float4 st[2][ST];
    auto load = [&](float4(&x)[ST], int s) {
#pragma unroll
        for (int u = 0; u < ST; u++)
            x[u] = ld4(w + (size_t)min(n_begin + 4 * (s + u) + kk, n_last) * K);
    };
    load(st[0], 0);
    // stage the innovations: global [sample][n] -> LDS [sample][n % 4][n / 4]
    // (N % 4 == 0 on this path)
    stage_slice_pairs<Z16_WAVES * 64>(dmu, dvar, NS, B, N, n_begin, N - n_begin, n_per_split, tid,
                                      [&](int b, int n, float4 m, float4 v) {
                                          float *pm = s_dm + b * S + n / 4, *pv = s_dv + b * S + n / 4;
                                          pm[0] = m.x; pm[Q] = m.y; pm[2 * Q] = m.z; pm[3 * Q] = m.w;
                                          pv[0] = v.x; pv[Q] = v.y; pv[2 * Q] = v.z; pv[3 * Q] = v.w;
                                      });

    floatx4 acc0[NG][4], acc1[NG][4];
#pragma unroll
    for (int g = 0; g < NG; g++)
#pragma unroll
        for (int t = 0; t < 4; t++) {
            acc0[g][t] = (floatx4){0.f, 0.f, 0.f, 0.f};
            acc1[g][t] = acc0[g][t];
        }

    auto multiply = [&](const float4(&cur)[ST], int s) {  // s: multiple of ST = 4
        float4 dm[NG], dv[NG];
#pragma unroll
        for (int g = 0; g < NG; g++) {
            dm[g] = *reinterpret_cast<const float4 *>(s_dm + (16 * g + i) * S + kk * Q + s);
            dv[g] = *reinterpret_cast<const float4 *>(s_dv + (16 * g + i) * S + kk * Q + s);
        }
#pragma unroll
        for (int u = 0; u < ST; u++) {
            const float4 x = cur[u];
            const float4 q = sq4(x);
#pragma unroll
            for (int t = 0; t < 4; t++)
#pragma unroll
                for (int g = 0; g < NG; g++) {
                    acc0[g][t] = mfma16(comp(x, t), comp(dm[g], u), acc0[g][t]);
                    acc1[g][t] = mfma16(comp(q, t), comp(dv[g], u), acc1[g][t]);
                }
        }
    };

    __syncthreads();
    for (int s = 0; s < steps; s += 2 * ST) {
        load(st[1], s + ST);
        __builtin_amdgcn_sched_barrier(0);
        multiply(st[0], s);
        __builtin_amdgcn_sched_barrier(0);
        // (nothing left to prefetch in the last pair: re-read the cached stage)
        load(st[0], s + 2 * ST < steps ? s + 2 * ST : s + ST);
        __builtin_amdgcn_sched_barrier(0);
        multiply(st[1], s + ST);
        __builtin_amdgcn_sched_barrier(0);
    }

    // register v of accumulator t of lane l: column c0 + 16*(l/16) + 4*v + t, sample
    // 16*g + l%16
#pragma unroll
    for (int g = 0; g < NG; g++) {
        const int b = 16 * g + i;
        if (b >= B) continue;
        const int c = c0 + 16 * (lane >> 4);
        const size_t base = ((size_t)split * B + b) * K + c;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            if (c + 4 * v < K) {  // K % 4 == 0 on this path
                *reinterpret_cast<float4 *>(ws0 + base + 4 * v) =
                    make_float4(acc0[g][0][v], acc0[g][1][v], acc0[g][2][v], acc0[g][3][v]);
                *reinterpret_cast<float4 *>(ws1 + base + 4 * v) =
                    make_float4(acc1[g][0][v], acc1[g][1][v], acc1[g][2][v], acc1[g][3][v]);
            }
        }
    }
}

constexpr int F16_KROUND = 2 * F16_KSTEP;                     // slices: whole pairs of stages
constexpr int Z16_NSTEP = 2 * Z16_ST * 4;                     // rows: whole pairs of stages
constexpr size_t W16_LDS_BUDGET = 72 * 1024;                  // slices of 512 elements for 16 samples

}  // namespace

// Waves per forward workgroup: -1 by size, else 8 or 16.
int g_gemv16_fwd_waves = -1;
static int fwd_waves(int N, int K, int B) {
    if (g_gemv16_fwd_waves == 8 || g_gemv16_fwd_waves == 16) return g_gemv16_fwd_waves;
    // Sixteen where 256-row blocks x 512-element slices still number two per CU, for up
    // to sixteen samples. Forward call, 16 against 8 waves: 8192^2 batch 16 99.7 / 103.9
    // us, batch 8 93.0 / 96.4; 8192 x 4096 batch 16 52.5 / 47.3; 8192^2 batch 32 150 / 144.
    return B <= W16_SAMPLES && (long long)N * K >= 2ll * num_cu() * 256 * 512 ? 16 : 8;
}
int gemv16_fwd_rows_per_block(int N, int K, int B) { return fwd_waves(N, K, B) * F16_RG * 16; }
int gemv16_fwd_k_step() { return F16_KROUND; }
// sample slots the kernels stage for a batch of B: 16 up to 16 samples, 32 beyond
static int sample_slots(int B) { return B <= W16_SAMPLES ? W16_SAMPLES : 2 * W16_SAMPLES; }
int gemv16_max_batch() { return 2 * W16_SAMPLES; }
int gemv16_fwd_max_slice(int B) {
    return (int)(W16_LDS_BUDGET / (2 * sample_slots(B) * sizeof(float)) - F16_PAD) / F16_KROUND *
           F16_KROUND;
}
int gemv16_dz_cols_per_block() { return Z16_COLS; }
int gemv16_dz_n_step() { return Z16_NSTEP; }
int gemv16_dz_max_slice(int B) {
    return (int)(W16_LDS_BUDGET / (2 * sample_slots(B) * sizeof(float)) - 16 * Z16_PADQ) /
           Z16_NSTEP * Z16_NSTEP;
}

// Forward load pattern. 0: sixteen rows x 64 bytes per instruction, plain loads; 1: whole
// 128-byte lines, streaming loads; 2: whole lines, plain loads; 3: whole lines, plain
// loads for mu_w and streaming loads for var_w; 4: the other way round; -1: by size
// against the 256 MB memory-side cache. Both matrices fit: 2 (they stay in it from one
// call to the next: 4096^2, batch 16, 27.9 us against 32.0 with streaming loads).
// Neither fits: 1. One fits: the forward streams one matrix and leaves the other in the
// cache for the backward of the same layer - var_w for the weight backward up to 8
// samples (4), mu_w for the 16-wide state backward beyond (3; that kernel's own plain
// loads would push var_w out again). Measured at 8192^2 per forward call, batch 16:
// 115 / 104 / 108 us for 0 / 1 / 2 with eight waves per workgroup, 100 us for 1 with
// sixteen, 3 and 4 the same as 1; forward + backward: batch 16 293 -> 283 us with 3
// (291 with 4), batch 8 265 -> 252 us with 4 (264 with 3). This helps where a layer's
// backward follows its forward closely; elsewhere it is neutral.
int g_gemv16_fwd_whole_lines = -1;

template <int NG, int WL, int WAVES>
static hipError_t run_gemv16_fwd(dim3 grid, size_t lds, hipStream_t stream,
                                 const float *mu_w, const float *var_w, const float *mu_a,
                                 const float *var_a, int K, int N, int B, int k_per_split,
                                 int splits, float *ws0, float *ws1) {
    static PerDeviceOnce once;
    hipError_t e = allow_dynamic_lds(
        once, reinterpret_cast<const void *>(gemv16_fwd_kernel<NG, WL, WAVES>), 160 * 1024);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((gemv16_fwd_kernel<NG, WL, WAVES>), grid, dim3(WAVES * 64), lds, stream, mu_w, var_w, mu_a,
                       var_a, K, N, B, k_per_split, splits, ws0, ws1);
    return hipGetLastError();
}

// k_per_split: a multiple of gemv16_fwd_k_step(), at most gemv16_fwd_max_slice(B);
// ws0/ws1: [splits][B][N] partial sums for the caller to fold.
hipError_t launch_gemv16_fwd(const float *mu_w, const float *var_w, const float *mu_a,
                             const float *var_a, int K, int N, int B, int k_per_split,
                             int splits, float *ws0, float *ws1, hipStream_t stream) {
    if (B < 1 || B > gemv16_max_batch() || K % 4 != 0 || k_per_split % gemv16_fwd_k_step() != 0 ||
        k_per_split > gemv16_fwd_max_slice(B) || (long long)k_per_split * splits < K)
        return hipErrorInvalidValue;
    size_t lds = (size_t)2 * sample_slots(B) * (k_per_split + F16_PAD) * sizeof(float);
    const int rows = gemv16_fwd_rows_per_block(N, K, B);
    dim3 grid(((N + rows - 1) / rows) * splits);
#define TAGI_RUN16(NG, WL)                                                                          \
    (rows == 256 ? run_gemv16_fwd<NG, WL, 16>(grid, lds, stream, mu_w, var_w, mu_a, var_a, K, N, B, \
                                              k_per_split, splits, ws0, ws1)                       \
                 : run_gemv16_fwd<NG, WL, 8>(grid, lds, stream, mu_w, var_w, mu_a, var_a, K, N, B,  \
                                             k_per_split, splits, ws0, ws1))
    int wl = g_gemv16_fwd_whole_lines;
    if (wl < 0 || wl > 4) {
        const size_t matrix = (size_t)N * K * sizeof(float), cache = (size_t)256 << 20;
        wl = 2 * matrix <= cache ? 2 : matrix > cache ? 1 : B <= 8 ? 4 : 3;
    }
    if (B <= W16_SAMPLES)
        return wl == 1 ? TAGI_RUN16(1, 1) : wl == 2 ? TAGI_RUN16(1, 2) : wl == 3 ? TAGI_RUN16(1, 3) : wl == 4 ? TAGI_RUN16(1, 4) : TAGI_RUN16(1, 0);
    return wl == 1 ? TAGI_RUN16(2, 1) : wl == 2 ? TAGI_RUN16(2, 2) : wl == 3 ? TAGI_RUN16(2, 3) : wl == 4 ? TAGI_RUN16(2, 4) : TAGI_RUN16(2, 0);
#undef TAGI_RUN16
}

template <int NG>
static hipError_t run_gemv16_dz(dim3 grid, dim3 block, size_t lds, hipStream_t stream,
                                const float *mu_w, const float *dmu, const float *dvar, int K, int N,
                                int B, int n_per_split, float *ws0, float *ws1) {
    static PerDeviceOnce once;
    hipError_t e = allow_dynamic_lds(
        once, reinterpret_cast<const void *>(gemv16_dz_kernel<NG>), 160 * 1024);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((gemv16_dz_kernel<NG>), grid, block, lds, stream, mu_w, dmu, dvar, K, N, B,
                       n_per_split, ws0, ws1);
    return hipGetLastError();
}

// n_per_split: a multiple of gemv16_dz_n_step(), at most gemv16_dz_max_slice(B);
// ws0/ws1: [splits][B][K] partial sums for the caller to fold.
hipError_t launch_gemv16_dz(const float *mu_w, const float *dmu, const float *dvar, int K, int N,
                            int B, int n_per_split, int splits, float *ws0, float *ws1,
                            hipStream_t stream) {
    if (B < 1 || B > gemv16_max_batch() || K % 4 != 0 || N % 4 != 0 ||
        n_per_split % Z16_NSTEP != 0 || n_per_split > gemv16_dz_max_slice(B) ||
        (long long)n_per_split * splits < N || splits > 65535)
        return hipErrorInvalidValue;
    const size_t lds = (size_t)2 * sample_slots(B) * (n_per_split + 16 * Z16_PADQ) * sizeof(float);
    const int cols = gemv16_dz_cols_per_block();
    dim3 grid((K + cols - 1) / cols, splits), block(Z16_WAVES * 64);
    if (B <= W16_SAMPLES)
        return run_gemv16_dz<1>(grid, block, lds, stream, mu_w, dmu, dvar, K, N, B, n_per_split, ws0, ws1);
    return run_gemv16_dz<2>(grid, block, lds, stream, mu_w, dmu, dvar, K, N, B, n_per_split, ws0, ws1);
}

}  // namespace tagi

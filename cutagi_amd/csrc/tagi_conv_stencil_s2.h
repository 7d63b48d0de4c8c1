// Regular-stencil kernel for the state backward of the stride-2 convolutions of a
// ResNet: the 3x3 kernel with one pixel of padding on the right and bottom only (the
// reference's padding type 2) and the 2x2 projection without padding - in both, tap
// (ky, kx) of output pixel (oy, ox) reads input pixel (2*oy + ky, 2*ox + kx)
// (src/indices.cpp:63-103) - on square input maps of width 8, 16 or 32. As in
// tagi_conv_stencil.h every workgroup first CHECKS the index tables it was given against
// that stencil, for its own pixels, and runs the table-driven loop if anything differs.
//
// An input pixel (y, x) is reached through the taps whose parity matches its own:
// ky = y (mod 2), kx likewise, i.e. through 4, 2, 2 or 1 of the 9 taps (one of the 4) by
// phase (y mod 2, x mod 2), from the output pixels ((y - ky) / 2, (x - kx) / 2). With the
// columns numbered phase by phase (ConvParams::perm_s = 2), the pixels (2*ly + py,
// 2*lx + px) of a phase form an (ly, lx) grid on which the contraction is a small stencil
// over the innovation maps: taps at offsets (-(ky / 2), -(kx / 2)), all in {-1, 0}.
//
// Included by tagi_conv2d.hip after tagi_conv_stencil.h.
#pragma once

namespace tagi {
namespace {

// ---- all four phases in one workgroup ----------------------------------------------------
// The four phases of a block of input pixels (2*ly + py, 2*lx + px) read the SAME
// innovation patch (output pixels (ly - a, lx - c), a, c in {0, 1}), each through its own
// taps. A workgroup that keeps four accumulator sets therefore stages the patch once
// and runs all KS*KS taps per staged channel pair - the reduction of a tile is KS*KS*fo
// long, as in the unit-stride stencil, instead of 1..4 taps * fo - and pays the table
// check, the first loads and the wind-down once per 4 x 64 x 128 outputs. Covers the
// 3x3 kernel and the 2x2 projection of a residual block (one tap per phase, no halo).
// (A workgroup per phase tile, the first form of this kernel, reduced over 1..4 taps * fo
// only and reached 36-55 % of the matrix peak on ResNet-18's three layers.) The weights of an output channel, w[f][(m0+row)*T + t] for the
// tile's 64 rows, are 64*T consecutive floats and are staged in that order.
// 128 accumulator registers per lane: one 8-wave workgroup per CU.

// Expected (tap, output pixel) occurrences of input pixel (y, x) on a 2*WO-wide map for a
// KS x KS kernel (KS = 2 or 3); returns the tap mask, out[t] = 1-based output pixel of tap t.
template <int WO, int KS>
__device__ __forceinline__ int s2k_occurrences(int y, int x, int (&out)[KS * KS]) {
    int mask = 0;
#pragma unroll
    for (int t = 0; t < KS * KS; t++) {
        const int ky = t / KS, kx = t - ky * KS;
        const int ny = y - ky, nx = x - kx;
        const bool hit = ny >= 0 && nx >= 0 && (ny & 1) == 0 && (nx & 1) == 0 &&
                         (ny >> 1) < WO && (nx >> 1) < WO;
        out[t] = hit ? (ny >> 1) * WO + (nx >> 1) + 1 : 0;
        mask |= hit ? 1 << t : 0;
    }
    return mask;
}

// Do the two tables list exactly those occurrences for the 4 x 128 pixels of the tile
// (phase-ordered columns ph * per_phase + q0 + c)? Thread (ph, c) owns one pixel and its
// whole list (at most NR entries), all requested before any is looked at. Uniform verdict;
// `scratch`: one int of LDS.
template <int WO, int KS>
__device__ __forceinline__ bool s2_all_tables_ok(const ConvParams &p, int q0, int per_phase,
                                                 int tid, int *scratch) {
    constexpr int T = KS * KS, NR = KS == 3 ? 4 : 1;
    if (tid == 0) *scratch = 1;
    __syncthreads();
    bool ok = p.nr == NR;
    if (ok) {
        const int ph = tid >> 7, c = tid & 127;
        const int px = dz_column(p, ph * per_phase + q0 + c).px;
        int o[NR], tap[NR];
#pragma unroll
        for (int j = 0; j < NR; j++) {
            o[j] = p.idx2[j * p.wihi + px];
            tap[j] = p.idx[px * NR + j];
        }
        int want[T];
        const int y = px / (2 * WO), x = px - y * (2 * WO);
        const int mask = s2k_occurrences<WO, KS>(y, x, want);
        int seen = 0;
#pragma unroll
        for (int j = 0; j < NR; j++) {
            if (o[j] <= -1) continue;
            if (tap[j] < 1 || tap[j] > T) {
                ok = false;
                continue;
            }
            const int t = tap[j] - 1;
            int w = 0;
#pragma unroll
            for (int q = 0; q < T; q++) w = q == t ? want[q] : w;
            ok = ok && o[j] == w && !(seen >> t & 1);
            seen |= 1 << t;
        }
        ok = ok && seen == mask;
    }
    if (!ok) *scratch = 0;
    __syncthreads();
    const bool verdict = __builtin_amdgcn_readfirstlane(*scratch) != 0;
    __syncthreads();
    return verdict;
}

// The epilogue of ConvDzProblem::store_with for two neighbouring input pixels at once.
__device__ __forceinline__ bool s2_pair_stores_ok(const ConvParams &p) {
    const uintptr_t all = reinterpret_cast<uintptr_t>(p.out0) | reinterpret_cast<uintptr_t>(p.out1) |
                          reinterpret_cast<uintptr_t>(p.e0) |
                          (p.res_mode ? reinterpret_cast<uintptr_t>(p.res0) |
                                            reinterpret_cast<uintptr_t>(p.res1)
                                      : 0);
    return (all & 7u) == 0;
}
__device__ __forceinline__ void s2_finish_pair(const ConvParams &p, size_t at, float2 mu, float2 var,
                                               float2 e, float2 r0, float2 r1) {
    if (p.res_mode == 1) {
        mu.x += r0.x; mu.y += r0.y;
        var.x += r1.x; var.y += r1.y;
    }
    mu.x *= e.x; mu.y *= e.y;
    var.x *= e.x * e.x; var.y *= e.y * e.y;
    if (p.res_mode == 2) {
        mu.x += r0.x; mu.y += r0.y;
        var.x += r1.x; var.y += r1.y;
    }
    *reinterpret_cast<float2 *>(p.out0 + at) = mu;
    *reinterpret_cast<float2 *>(p.out1 + at) = var;
}
// Accumulator register v of a lane is row row0 + 8*(v/4) + v%4 (tile_epilogue's layout);
// (ma, va) / (mb, vb): the sums of input pixels (y, 2*lx) / (y, 2*lx + 1) of image b.
template <int WO>
__device__ __forceinline__ void s2_store_row_pairs(const ConvParams &p, floatx16 (&ma)[1][1],
                                                   floatx16 (&va)[1][1], floatx16 (&mb)[1][1],
                                                   floatx16 (&vb)[1][1], int row0, int b, int y,
                                                   int lx) {
    constexpr int WI = 2 * WO;
    const size_t base = ((size_t)b * p.fi) * (WI * WI) + (size_t)y * WI + 2 * lx;
    const float2 zero = make_float2(0.f, 0.f);
    // the epilogue operands of eight rows are requested before their first store (a load
    // that follows a store waits for it)
#pragma unroll
    for (int h = 0; h < 16; h += 8) {
        float2 e[8], r0[8], r1[8];
#pragma unroll
        for (int v = h; v < h + 8; v++) {
            const size_t at = base + (size_t)(row0 + 8 * (v / 4) + (v % 4)) * (WI * WI);
            e[v - h] = *reinterpret_cast<const float2 *>(p.e0 + at);
            r0[v - h] = p.res_mode ? *reinterpret_cast<const float2 *>(p.res0 + at) : zero;
            r1[v - h] = p.res_mode ? *reinterpret_cast<const float2 *>(p.res1 + at) : zero;
        }
#pragma unroll
        for (int v = h; v < h + 8; v++) {
            const size_t at = base + (size_t)(row0 + 8 * (v / 4) + (v % 4)) * (WI * WI);
            s2_finish_pair(p, at, make_float2(ma[0][0][v], mb[0][0][v]),
                           make_float2(va[0][0][v], vb[0][0][v]), e[v - h], r0[v - h], r1[v - h]);
        }
    }
}

// Fold of a sliced reduction for phase-ordered columns (perm_s = 2) in the order of the
// OUTPUT: a thread owns two neighbouring input pixels (y, 2*lx), (y, 2*lx + 1) of one
// channel, whose partial sums lie in the two column phases of row phase y mod 2 at the
// same offset - consecutive threads read consecutive partial sums of either phase and
// write consecutive pairs. ws0/ws1 [split][M][N]; W = p.perm_w (even).
__global__ __launch_bounds__(256) void reduce_store_s2_pairs_kernel(ConvParams p) {
    const int W = p.perm_w, ws = W / 2;
    const size_t pairs = (size_t)p.M * p.N / 2;
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= pairs) return;
    // i = ((b * M + m) * W + y) * ws + lx : the order of the output tensor
    const int lx = (int)(i % ws);
    size_t rest = i / ws;
    const int y = (int)(rest % W);
    rest /= W;
    const int m = (int)(rest % p.M), b = (int)(rest / p.M);
    const int per_img = p.wihi / 4, per_phase = p.B * per_img;
    const size_t col = (size_t)((y & 1) * 2) * per_phase + (size_t)b * per_img + (y >> 1) * ws + lx;
    const size_t total = (size_t)p.M * p.N, src = (size_t)m * p.N + col;
    float2 mu = make_float2(0.f, 0.f), var = mu;
#pragma unroll 4
    for (int s = 0; s < p.splits; s++) {
        mu.x += p.ws0[s * total + src];
        mu.y += p.ws0[s * total + src + per_phase];
        var.x += p.ws1[s * total + src];
        var.y += p.ws1[s * total + src + per_phase];
    }
    const size_t at = ((size_t)b * p.M + m) * p.wihi + (size_t)y * W + 2 * lx;
    const float2 zero = make_float2(0.f, 0.f);
    s2_finish_pair(p, at, mu, var, *reinterpret_cast<const float2 *>(p.e0 + at),
                   p.res_mode ? *reinterpret_cast<const float2 *>(p.res0 + at) : zero,
                   p.res_mode ? *reinterpret_cast<const float2 *>(p.res1 + at) : zero);
}

inline hipError_t launch_reduce_store_s2_pairs(const ConvParams &p, hipStream_t stream) {
    const size_t pairs = (size_t)p.M * p.N / 2;
    hipLaunchKernelGGL(reduce_store_s2_pairs_kernel, dim3((unsigned)((pairs + 255) / 256)), dim3(256),
                       0, stream, p);
    return hipGetLastError();
}

template <int WO, int KS>
struct S2AllGeom {
    using G = StencilGeom<WO>;               // patch layout of one channel: rows -1 .. RPI, zero halo
    static constexpr int T = KS * KS;
    static constexpr int KC = WO == 4 ? 8 : 16;            // output channels per k-tile
    static constexpr int PATCH = KC * G::CS;
    static constexpr int UNITS = KC * G::SEGS * (G::RPI + 1) * (WO / 4);
    static constexpr int P_SLOTS = (UNITS + 511) / 512;
    static constexpr int WROW = 64 * T;                    // floats of one output channel
    static constexpr int W_VEC = KC * WROW / 4;            // 16-byte pieces per k-tile
    static constexpr int W_SLOTS = (W_VEC + 511) / 512;
    static constexpr int LDS_FLOATS = KC * WROW + 2 * PATCH;
};

template <int WO, int KS>
__device__ __forceinline__ void s2_all_body(const ConvParams &p, float *lds, int m0, int q0,
                                            int per_phase, int split, int c_begin, int c_end) {
    using S = S2AllGeom<WO, KS>;
    using G = StencilGeom<WO>;
    constexpr int W = WO, H = WO, NT = 512, KC = S::KC, T = S::T;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wrow = (wave / 4) * 32, wcol = (wave % 4) * 32, half = lane >> 5;
    float *lds_w = lds;                      // [KC][64 rows * T], memory order
    float *lds_p = lds + KC * S::WROW;       // [PATCH][2]: (delta_mu, delta_var) interleaved

    for (int i = tid; i < 2 * S::PATCH; i += NT) lds_p[i] = 0.f;

    // patch units of this thread (rows -1 .. RPI-1 of each segment; taps reach up and left)
    size_t punit[S::P_SLOTS];
    int pdst[S::P_SLOTS];
    bool p_ok[S::P_SLOTS];
#pragma unroll
    for (int i = 0; i < S::P_SLOTS; i++) {
        int u = tid + i * NT;
        const bool live = u < S::UNITS;
        u = live ? u : 0;
        const int x4 = u % (W / 4);
        u /= (W / 4);
        const int pr = u % (G::RPI + 1);
        u /= (G::RPI + 1);
        const int seg = u % G::SEGS, pc = u / G::SEGS;
        const int grow = q0 / W + seg * G::RPI;  // first (b, ly) row of the segment
        const int img = grow / H, y = grow % H + pr - 1;
        p_ok[i] = live && y >= 0 && y < H && img < p.B;
        punit[i] = p_ok[i] ? ((size_t)img * p.fo + c_begin + pc) * (W * H) + y * W + 4 * x4 : 0;
        pdst[i] = pc * G::CS + seg * G::SEG + pr * G::RS + G::XO + 4 * x4;
    }
    const size_t pstep = (size_t)KC * (W * H);

    // weight pieces of this thread: 16 bytes of w[c_begin + f][(m0 + row) * T + t]
    size_t wsrc[S::W_SLOTS];
    int wdst[S::W_SLOTS];
    bool w_ok[S::W_SLOTS];
#pragma unroll
    for (int i = 0; i < S::W_SLOTS; i++) {
        const int e = tid + i * NT;
        w_ok[i] = e < S::W_VEC;
        const int id = w_ok[i] ? e : 0;
        const int f = id / (S::WROW / 4), q = id - f * (S::WROW / 4);
        wsrc[i] = ((size_t)(c_begin + f) * p.fi + m0) * T + 4 * q;
        wdst[i] = f * S::WROW + 4 * q;
    }
    const size_t wstep = (size_t)KC * p.fi * T;

    // one accumulator pair per phase (py, px), named one by one: an array of them indexed
    // by the tap's phase is kept in scratch memory by the compiler
    floatx16 m00[1][1], m01[1][1], m10[1][1], m11[1][1], v00[1][1], v01[1][1], v10[1][1], v11[1][1];
#pragma unroll
    for (int v = 0; v < 16; v++) {
        m00[0][0][v] = m01[0][0][v] = m10[0][0][v] = m11[0][0][v] = 0.f;
        v00[0][0][v] = v01[0][0][v] = v10[0][0][v] = v11[0][0][v] = 0.f;
    }

    // staging registers, named one by one (arrays of them end up in scratch memory)
    static_assert(S::W_SLOTS <= 5 && S::P_SLOTS <= 2, "staging registers below");
    float4 rw0, rw1, rw2, rw3, rw4, rpa0, rpa1, rpb0, rpb1;
    rw0 = rw1 = rw2 = rw3 = rw4 = rpa0 = rpa1 = rpb0 = rpb1 = make_float4(0.f, 0.f, 0.f, 0.f);
#define TAGI_S2ALL_WLOAD(i)                                                           \
    if (i < S::W_SLOTS) {                                                             \
        rw##i = *reinterpret_cast<const float4 *>(p.w0 + wsrc[i < S::W_SLOTS ? i : 0]); \
        if (w_ok[i < S::W_SLOTS ? i : 0]) wsrc[i < S::W_SLOTS ? i : 0] += wstep;      \
    }
#define TAGI_S2ALL_WPUT(i)                                                            \
    if (i < S::W_SLOTS && w_ok[i < S::W_SLOTS ? i : 0])                               \
        *reinterpret_cast<float4 *>(lds_w + wdst[i < S::W_SLOTS ? i : 0]) = rw##i;
#define TAGI_S2ALL_PLOAD(i, A_, B_)                                                   \
    if (i < S::P_SLOTS) {                                                             \
        A_ = *reinterpret_cast<const float4 *>(p.d0 + punit[i < S::P_SLOTS ? i : 0]); \
        B_ = *reinterpret_cast<const float4 *>(p.d1 + punit[i < S::P_SLOTS ? i : 0]); \
        if (p_ok[i < S::P_SLOTS ? i : 0]) punit[i < S::P_SLOTS ? i : 0] += pstep;     \
    }
#define TAGI_S2ALL_PPUT(i, A_, B_)                                                    \
    if (i < S::P_SLOTS && p_ok[i < S::P_SLOTS ? i : 0]) {                             \
        float *dst_ = lds_p + 2 * pdst[i < S::P_SLOTS ? i : 0];                       \
        *reinterpret_cast<float4 *>(dst_) = make_float4(A_.x, B_.x, A_.y, B_.y);      \
        *reinterpret_cast<float4 *>(dst_ + 4) = make_float4(A_.z, B_.z, A_.w, B_.w);  \
    }
#define TAGI_S2ALL_FETCH()                                                            \
    do {                                                                              \
        TAGI_S2ALL_WLOAD(0) TAGI_S2ALL_WLOAD(1) TAGI_S2ALL_WLOAD(2)                   \
        TAGI_S2ALL_WLOAD(3) TAGI_S2ALL_WLOAD(4)                                       \
        TAGI_S2ALL_PLOAD(0, rpa0, rpb0) TAGI_S2ALL_PLOAD(1, rpa1, rpb1)               \
    } while (0)
#define TAGI_S2ALL_COMMIT()                                                           \
    do {                                                                              \
        TAGI_S2ALL_WPUT(0) TAGI_S2ALL_WPUT(1) TAGI_S2ALL_WPUT(2)                      \
        TAGI_S2ALL_WPUT(3) TAGI_S2ALL_WPUT(4)                                         \
        TAGI_S2ALL_PPUT(0, rpa0, rpb0) TAGI_S2ALL_PPUT(1, rpa1, rpb1)                 \
    } while (0)

    // operand addresses of this lane: patch cell (row ly - 1, column lx - 1) of its pixel
    // for output channel `half` of a pair; the T weights of its row
    const int pix = wcol + (lane & 31), prow = pix / W, px = pix - prow * W;
    const float *bp = lds_p + 2 * (half * G::CS + (prow / G::RPI) * G::SEG +
                                   (prow % G::RPI) * G::RS + G::XO - 1 + px);
    const float *wp = lds_w + half * S::WROW + (wrow + (lane & 31)) * T;

    __syncthreads();  // patch zeroed
    if (c_begin < c_end) {
        TAGI_S2ALL_FETCH();
        TAGI_S2ALL_COMMIT();
    }
    __syncthreads();

    for (int c0 = c_begin; c0 < c_end; c0 += KC) {
        const bool more = c0 + KC < c_end;
        if (more) TAGI_S2ALL_FETCH();
#pragma unroll
        for (int pair = 0; pair < KC / 2; pair++) {
            // the innovations of output pixels (ly - a, lx - c)
            float2 y[2][2];
#pragma unroll
            for (int a = 0; a < (KS + 1) / 2; a++)
#pragma unroll
                for (int c = 0; c < (KS + 1) / 2; c++)
                    y[a][c] = *reinterpret_cast<const float2 *>(
                        bp + 2 * (2 * pair * G::CS + (1 - a) * G::RS + (1 - c)));
            // tap (ky, kx): phase (ky & 1, kx & 1), innovation of output pixel (ly - ky/2, lx - kx/2)
#define TAGI_S2ALL_TAP(W_, M_, V_, Y_)                                                        \
    do {                                                                                      \
        const float w_ = (W_);                                                                \
        M_[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(w_, (Y_).x, M_[0][0], 0, 0, 0);       \
        V_[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(w_ * w_, (Y_).y, V_[0][0], 0, 0, 0);  \
    } while (0)
            if constexpr (KS == 2) {
                // 16 bytes per lane: rows at a stride of four floats would share banks
                const float4 w4 = *reinterpret_cast<const float4 *>(wp + 2 * pair * S::WROW);
                TAGI_S2ALL_TAP(w4.x, m00, v00, y[0][0]);
                TAGI_S2ALL_TAP(w4.y, m01, v01, y[0][0]);
                TAGI_S2ALL_TAP(w4.z, m10, v10, y[0][0]);
                TAGI_S2ALL_TAP(w4.w, m11, v11, y[0][0]);
            } else {
                const float *wq = wp + 2 * pair * S::WROW;   // stride 9 between rows: no conflicts
                TAGI_S2ALL_TAP(wq[0], m00, v00, y[0][0]);
                TAGI_S2ALL_TAP(wq[1], m01, v01, y[0][0]);
                TAGI_S2ALL_TAP(wq[2], m00, v00, y[0][1]);
                TAGI_S2ALL_TAP(wq[3], m10, v10, y[0][0]);
                TAGI_S2ALL_TAP(wq[4], m11, v11, y[0][0]);
                TAGI_S2ALL_TAP(wq[5], m10, v10, y[0][1]);
                TAGI_S2ALL_TAP(wq[6], m00, v00, y[1][0]);
                TAGI_S2ALL_TAP(wq[7], m01, v01, y[1][0]);
                TAGI_S2ALL_TAP(wq[8], m00, v00, y[1][1]);
            }
#undef TAGI_S2ALL_TAP
        }
        __syncthreads();
        if (more) {
            TAGI_S2ALL_COMMIT();
            __syncthreads();
        }
    }
#undef TAGI_S2ALL_FETCH
#undef TAGI_S2ALL_COMMIT
#undef TAGI_S2ALL_WLOAD
#undef TAGI_S2ALL_WPUT
#undef TAGI_S2ALL_PLOAD
#undef TAGI_S2ALL_PPUT
    if (p.splits > 1 || !s2_pair_stores_ok(p)) {
        // partial sums (contiguous in the phase-ordered workspace), or outputs that are
        // not 8-byte aligned: phase by phase
        tile_epilogue<ConvDzProblem, 64, 128, 2, 4>(p, m00, v00, m0, q0, split);
        tile_epilogue<ConvDzProblem, 64, 128, 2, 4>(p, m01, v01, m0, per_phase + q0, split);
        tile_epilogue<ConvDzProblem, 64, 128, 2, 4>(p, m10, v10, m0, 2 * per_phase + q0, split);
        tile_epilogue<ConvDzProblem, 64, 128, 2, 4>(p, m11, v11, m0, 3 * per_phase + q0, split);
        return;
    }
    // Complete sums: the two column phases of a lane's pixel are neighbours in memory
    // ((2*ly + py, 2*lx) and (2*ly + py, 2*lx + 1)), so they leave as one 8-byte store
    // and a wave writes whole rows. (Phase by phase the same outputs are 4-byte stores
    // two elements apart: 89 of 173 us at 64 -> 128 channels on 32 x 32 maps.)
    const int q = q0 + pix, b = q / (W * H), l = q - b * (W * H), ly = l / W, lx = l - ly * W;
    const int row0 = m0 + wrow + 4 * half;
    s2_store_row_pairs<W>(p, m00, v00, m01, v01, row0, b, 2 * ly, lx);
    s2_store_row_pairs<W>(p, m10, v10, m11, v11, row0, b, 2 * ly + 1, lx);
}

template <int WO, int KS>
struct S2AllLds {
    using P = ConvDzProblem;
    static constexpr int XF = TileGeom<P::XK, 64>::floats, YF = TileGeom<P::YK, 128>::floats;
    static constexpr int GENERIC = P::NX * XF + P::NY * YF;
    static constexpr int MINE = S2AllGeom<WO, KS>::LDS_FLOATS;
    static constexpr int FLOATS = MINE > GENERIC ? MINE : GENERIC;
};

// One workgroup of 8 waves per 64 input channels x 128 base pixels x 4 phases; grid.x =
// (fi / 64) * (B * WO * WO / 128), grid.y = reduction slices (whole groups of 32 output
// channels). Tables that are not the expected stencil: the four phase tiles run through
// the table-driven loop one after the other.
template <int WO, int KS>
__global__ __launch_bounds__(512) void conv_stencil_s2_all_dz_kernel(ConvParams p) {
    using P = ConvDzProblem;
    using L = S2AllLds<WO, KS>;
    __shared__ __attribute__((aligned(16))) float lds[L::FLOATS];
    extern __shared__ __attribute__((aligned(16))) int lds_extra[];

    const int per_phase = p.B * WO * WO;
    const int tiles_q = per_phase / 128;
    const int split = blockIdx.y;
    const int m0 = (blockIdx.x / tiles_q) * 64, q0 = (blockIdx.x % tiles_q) * 128;
    const int r_begin = split * p.r_per_split;
    const int r_end = min(p.R, r_begin + p.r_per_split);

    if (s2_all_tables_ok<WO, KS>(p, q0, per_phase, threadIdx.x, lds_extra)) {
        s2_all_body<WO, KS>(p, lds, m0, q0, per_phase, split, r_begin / (KS * KS), r_end / (KS * KS));
        return;
    }
    for (int ph = 0; ph < 4; ph++) {
        const int n0 = ph * per_phase + q0;
        __syncthreads();  // the previous phase's tables and tiles are done with
        typename P::Ctx ctx;
        P::prologue(p, ctx, lds_extra, threadIdx.x, 512, m0, n0, 64, 128, r_begin, r_end);
        __syncthreads();
        int r_lo = r_begin, r_hi = r_end;
        P::adjust_range(p, ctx, r_lo, r_hi);
        mfma_tile_body<P, 64, 128, 2, 4, 0>(p, ctx, reinterpret_cast<float (*)[L::XF]>(lds),
                                            reinterpret_cast<float (*)[L::YF]>(lds + P::NX * L::XF),
                                            m0, n0, split, r_lo, r_hi);
    }
}

template <int KS>
inline hipError_t launch_conv_stencil_s2_all_dz(int wo, const ConvParams &p, hipStream_t stream) {
    using P = ConvDzProblem;
    const dim3 grid((p.M / 64) * (p.B * wo * wo / 128), p.splits);
    const size_t extra = P::extra_lds_bytes(p, 64, 128);
    if (extra > kTileExtraLdsMax) return hipErrorInvalidValue;
#define TAGI_LAUNCH_S2ALL(WD)                                                                      \
    case WD: {                                                                                     \
        static PerDeviceOnce once;                                                                 \
        hipError_t e = allow_dynamic_lds(                                                          \
            once, reinterpret_cast<const void *>(conv_stencil_s2_all_dz_kernel<WD, KS>),           \
            (int)kTileExtraLdsMax);                                                                \
        if (e != hipSuccess) return e;                                                             \
        hipLaunchKernelGGL((conv_stencil_s2_all_dz_kernel<WD, KS>), grid, dim3(512), extra, stream, p); \
        return hipGetLastError();                                                                  \
    }
    switch (wo) {
        TAGI_LAUNCH_S2ALL(4)
        TAGI_LAUNCH_S2ALL(8)
        TAGI_LAUNCH_S2ALL(16)
    }
#undef TAGI_LAUNCH_S2ALL
    return hipErrorInvalidValue;
}

// ---- forward ---------------------------------------------------------------------------
// Output tile = 64 output channels x 128 output pixels = 128/WO whole output rows. The
// input rows those pixels read (2*oy + ky) are staged once per channel with 16-byte
// loads - 2*RPI + KS - 2 rows of 2*WO values per segment, plus one zero cell on the right
// and, where the last row leaves the image, a zero row: the padding of the 3x3 kernel -
// and tap (ky, kx) of a lane's pixel is the constant offset ky*RS + kx from the cell
// (2*oy, 2*ox) when the MFMA operand is read. A k-tile is 4 channels x 9 taps or
// 8 channels x 4 taps; lanes 0-31 / 32-63 of an MFMA step take the first / second half
// of its channels at the same (channel, tap) position, the weights stay in memory order.
template <int WO, int KS>
struct S2FwdGeom {
    static constexpr int W = WO, H = WO, WI = 2 * WO, T = KS * KS;
    static constexpr int KC = KS == 3 ? 4 : 8;             // channels per k-tile
    static constexpr int VPH = KC / 2 * T;                 // reduction steps per k-half
    static constexpr int NR = 128 / W;                     // output rows per tile
    static constexpr int RPI = NR < H ? NR : H;            // rows of one image among them
    static constexpr int SEGS = NR / RPI;                  // images (segments) per tile
    static constexpr int PR = 2 * RPI + KS - 2;            // staged input rows per segment
    static constexpr int RS = WI + 4;                      // values, one zero cell, 3 unused
    static constexpr int SEG = PR * RS;
    static constexpr int CS = SEGS * SEG + 4;
    static constexpr int PATCH = KC * CS;                  // floats per staged array
    static constexpr int UNITS = KC * SEGS * PR * (WI / 4);  // 16-byte loads per array
    static constexpr int P_SLOTS = (UNITS + 511) / 512;
    static constexpr int AS = KC * T + (KC * T == 36 ? 8 : 12);  // 44: rows on distinct bank groups
    static constexpr int A_VEC = 64 * KC * T / 4;          // 16-byte loads per weight array
    static constexpr int A_SLOTS = (A_VEC + 511) / 512;
    static constexpr int LDS_FLOATS = 2 * 64 * AS + 2 * PATCH;
    static_assert(P_SLOTS <= 2 && A_SLOTS <= 2 && VPH % 2 == 0 && (KC * T) % 4 == 0, "staging slots");
};

// Expected Fmwa_2 entry (1-based input pixel, -1 = padding) of tap t of output pixel o.
template <int WO, int KS>
__device__ __forceinline__ int s2_fmwa(int o, int t) {
    const int oy = o / WO, ox = o - oy * WO;
    const int iy = 2 * oy + t / KS, ix = 2 * ox + t % KS;
    return (iy < 2 * WO && ix < 2 * WO) ? iy * (2 * WO) + ix + 1 : -1;
}

// Does Fmwa_2 [woho][T] describe that stencil for the pixels n0 .. n0+127? Uniform verdict;
// entries are requested in batches before any is looked at. `scratch`: one int of LDS.
template <int WO, int KS>
__device__ __forceinline__ bool s2_fwd_tables_ok(const ConvParams &p, int n0, int tid, int *scratch) {
    constexpr int T = KS * KS, PAIRS = 128 * T, ITER = (PAIRS + 511) / 512;
    if (tid == 0) *scratch = 1;
    __syncthreads();
    int got[ITER], want[ITER];
#pragma unroll
    for (int i = 0; i < ITER; i++) {
        const int e = tid + i * 512, c = e / T, t = e - c * T, n = n0 + c;
        const bool live = e < PAIRS && n < p.N;
        const int o = live ? n % p.woho : 0;
        got[i] = p.idx[live ? o * T + t : 0];
        want[i] = live ? s2_fmwa<WO, KS>(o, t) : got[i];
    }
    bool ok = true;
#pragma unroll
    for (int i = 0; i < ITER; i++) ok = ok && got[i] == want[i];
    if (!ok) *scratch = 0;
    __syncthreads();
    const bool verdict = __builtin_amdgcn_readfirstlane(*scratch) != 0;
    __syncthreads();
    return verdict;
}

// One 64 x 128 tile on a verified stencil. c_begin / c_end: input channels of the
// reduction slice (multiples of KC).
template <int WO, int KS>
__device__ __forceinline__ void s2_fwd_body(const ConvParams &p, float *lds, int m0, int n0,
                                            int split, int c_begin, int c_end) {
    using G = S2FwdGeom<WO, KS>;
    constexpr int W = WO, H = WO, WI = G::WI, NT = 512, KC = G::KC, T = G::T;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wrow = (wave / 4) * 32, wcol = (wave % 4) * 32, half = lane >> 5;
    float *lds_a = lds;                      // [2 arrays][64 rows][AS]: KC*T values per row, memory order
    float *lds_p = lds + 2 * 64 * G::AS;     // [PATCH][2]: (mu_a, var_a) interleaved

    for (int i = tid; i < 2 * G::PATCH; i += NT) lds_p[i] = 0.f;

    // patch units of this thread: channel pc, segment, staged row pr, columns 4*x4 ..
    size_t punit[G::P_SLOTS];
    int pdst[G::P_SLOTS];
    bool p_ok[G::P_SLOTS];
#pragma unroll
    for (int i = 0; i < G::P_SLOTS; i++) {
        int u = tid + i * NT;
        const bool live = u < G::UNITS;
        u = live ? u : 0;
        const int x4 = u % (WI / 4);
        u /= (WI / 4);
        const int pr = u % G::PR;
        u /= G::PR;
        const int seg = u % G::SEGS, pc = u / G::SEGS;
        const int grow = n0 / W + seg * G::RPI;  // first output row of the segment, over the batch
        const int img = grow / H, y = 2 * (grow % H) + pr;
        p_ok[i] = live && y < 2 * H && img < p.B;
        punit[i] = p_ok[i] ? ((size_t)img * p.fi + c_begin + pc) * (WI * WI) + y * WI + 4 * x4 : 0;
        pdst[i] = pc * G::CS + seg * G::SEG + pr * G::RS + 4 * x4;
    }
    const size_t pstep = (size_t)KC * (WI * WI);

    // weight pieces of this thread: 16 bytes of w[m0 + row][c_begin*T + 4q ..]
    size_t asrc[G::A_SLOTS];
    int adst[G::A_SLOTS];
    bool a_ok[G::A_SLOTS];
#pragma unroll
    for (int i = 0; i < G::A_SLOTS; i++) {
        const int e = tid + i * NT;
        a_ok[i] = e < G::A_VEC;
        const int id = a_ok[i] ? e : 0;
        const int row = id / (KC * T / 4), q = id - row * (KC * T / 4);
        asrc[i] = (size_t)(m0 + row) * p.R + (size_t)c_begin * T + 4 * q;
        adst[i] = row * G::AS + 4 * q;
    }
    const size_t astep = (size_t)KC * T;

    floatx16 acc0[1][1], acc1[1][1];
#pragma unroll
    for (int v = 0; v < 16; v++) {
        acc0[0][0][v] = 0.f;
        acc1[0][0][v] = 0.f;
    }

    // staging registers, named one by one (arrays of them end up in scratch memory)
    float4 rm0, rm1, rv0, rv1, rpa0, rpa1, rpb0, rpb1;
    rm0 = rm1 = rv0 = rv1 = rpa0 = rpa1 = rpb0 = rpb1 = make_float4(0.f, 0.f, 0.f, 0.f);
#define TAGI_S2FWD_ALOAD(i)                                                           \
    if (i < G::A_SLOTS) {                                                             \
        rm##i = *reinterpret_cast<const float4 *>(p.w0 + asrc[i < G::A_SLOTS ? i : 0]); \
        rv##i = *reinterpret_cast<const float4 *>(p.w1 + asrc[i < G::A_SLOTS ? i : 0]); \
        if (a_ok[i < G::A_SLOTS ? i : 0]) asrc[i < G::A_SLOTS ? i : 0] += astep;      \
    }
#define TAGI_S2FWD_APUT(i)                                                            \
    if (i < G::A_SLOTS && a_ok[i < G::A_SLOTS ? i : 0]) {                             \
        *reinterpret_cast<float4 *>(lds_a + adst[i < G::A_SLOTS ? i : 0]) = rm##i;    \
        *reinterpret_cast<float4 *>(lds_a + 64 * G::AS + adst[i < G::A_SLOTS ? i : 0]) = rv##i; \
    }
#define TAGI_S2FWD_PLOAD(i, A_, B_)                                                   \
    if (i < G::P_SLOTS) {                                                             \
        A_ = *reinterpret_cast<const float4 *>(p.a0 + punit[i < G::P_SLOTS ? i : 0]); \
        B_ = *reinterpret_cast<const float4 *>(p.a1 + punit[i < G::P_SLOTS ? i : 0]); \
        if (p_ok[i < G::P_SLOTS ? i : 0]) punit[i < G::P_SLOTS ? i : 0] += pstep;     \
    }
#define TAGI_S2FWD_PPUT(i, A_, B_)                                                    \
    if (i < G::P_SLOTS && p_ok[i < G::P_SLOTS ? i : 0]) {                             \
        float *dst_ = lds_p + 2 * pdst[i < G::P_SLOTS ? i : 0];                       \
        *reinterpret_cast<float4 *>(dst_) = make_float4(A_.x, B_.x, A_.y, B_.y);      \
        *reinterpret_cast<float4 *>(dst_ + 4) = make_float4(A_.z, B_.z, A_.w, B_.w);  \
    }
#define TAGI_S2FWD_FETCH()                                                            \
    do {                                                                              \
        TAGI_S2FWD_ALOAD(0) TAGI_S2FWD_ALOAD(1)                                       \
        TAGI_S2FWD_PLOAD(0, rpa0, rpb0) TAGI_S2FWD_PLOAD(1, rpa1, rpb1)               \
    } while (0)
#define TAGI_S2FWD_COMMIT()                                                           \
    do {                                                                              \
        TAGI_S2FWD_APUT(0) TAGI_S2FWD_APUT(1)                                         \
        TAGI_S2FWD_PPUT(0, rpa0, rpb0) TAGI_S2FWD_PPUT(1, rpa1, rpb1)                 \
    } while (0)

    // operand addresses of this lane: patch cell (2*oy, 2*ox) of its pixel in the first
    // channel of its k-half; its row's values of that half
    const int pix = wcol + (lane & 31), prow = pix / W, px = pix - prow * W;
    const float *bp = lds_p + 2 * (half * (KC / 2) * G::CS + (prow / G::RPI) * G::SEG +
                                   2 * (prow % G::RPI) * G::RS + 2 * px);
    const float *a0 = lds_a + (wrow + (lane & 31)) * G::AS + half * G::VPH;
    const float *a1 = a0 + 64 * G::AS;

    __syncthreads();  // patch zeroed
    if (c_begin < c_end) {
        TAGI_S2FWD_FETCH();
        TAGI_S2FWD_COMMIT();
    }
    __syncthreads();

    for (int c0 = c_begin; c0 < c_end; c0 += KC) {
        const bool more = c0 + KC < c_end;
        if (more) TAGI_S2FWD_FETCH();
#pragma unroll
        for (int g = 0; g < G::VPH / 2; g++) {
            const float2 am = *reinterpret_cast<const float2 *>(a0 + 2 * g);
            const float2 av = *reinterpret_cast<const float2 *>(a1 + 2 * g);
#pragma unroll
            for (int e = 0; e < 2; e++) {
                const int s = 2 * g + e, ch = s / T, t = s - ch * T, ky = t / KS, kx = t - ky * KS;
                const float2 y = *reinterpret_cast<const float2 *>(bp + 2 * (ch * G::CS + ky * G::RS + kx));
                const float w = e ? am.y : am.x, wv = e ? av.y : av.x;
                // mean: mu_w mu_a; variance: var_w (var_a + mu_a^2) + mu_w^2 var_a
                acc0[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(w, y.x, acc0[0][0], 0, 0, 0);
                acc1[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(wv, y.x * y.x + y.y, acc1[0][0], 0, 0, 0);
                acc1[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(w * w, y.y, acc1[0][0], 0, 0, 0);
            }
        }
        __syncthreads();
        if (more) {
            TAGI_S2FWD_COMMIT();
            __syncthreads();
        }
    }
#undef TAGI_S2FWD_FETCH
#undef TAGI_S2FWD_COMMIT
#undef TAGI_S2FWD_ALOAD
#undef TAGI_S2FWD_APUT
#undef TAGI_S2FWD_PLOAD
#undef TAGI_S2FWD_PPUT
    tile_epilogue<ConvFwdProblem<true>, 64, 128, 2, 4>(p, acc0, acc1, m0, n0, split);
}

// One 64 x 128 tile per workgroup of 8 waves: verified stencil -> s2_fwd_body, anything
// else -> the table-driven loop of the generic tile kernel.
template <int WO, int KS>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4)))
void conv_stencil_s2_fwd_kernel(ConvParams p) {
    using G = S2FwdGeom<WO, KS>;
    using P = ConvFwdProblem<true>;
    constexpr int XF = TileGeom<P::XK, 64>::floats, YF = TileGeom<P::YK, 128>::floats;
    constexpr int GENERIC = P::NX * XF + P::NY * YF;
    __shared__ __attribute__((aligned(16))) float lds[GENERIC > G::LDS_FLOATS ? GENERIC : G::LDS_FLOATS];
    extern __shared__ __attribute__((aligned(16))) int lds_extra[];

    const int tiles_n = (p.N + 127) / 128;
    const int tile = blockIdx.x, split = blockIdx.y;
    const int m0 = (tile / tiles_n) * 64, n0 = (tile % tiles_n) * 128;
    const int r_begin = split * p.r_per_split;
    const int r_end = min(p.R, r_begin + p.r_per_split);

    if (s2_fwd_tables_ok<WO, KS>(p, n0, threadIdx.x, lds_extra)) {
        s2_fwd_body<WO, KS>(p, lds, m0, n0, split, r_begin / (KS * KS), r_end / (KS * KS));
        return;
    }
    typename P::Ctx ctx;
    P::prologue(p, ctx, lds_extra, threadIdx.x, 512, m0, n0, 64, 128, r_begin, r_end);
    __syncthreads();
    int r_lo = r_begin, r_hi = r_end;
    P::adjust_range(p, ctx, r_lo, r_hi);
    mfma_tile_body<P, 64, 128, 2, 4, 0>(p, ctx, reinterpret_cast<float (*)[XF]>(lds),
                                        reinterpret_cast<float (*)[YF]>(lds + P::NX * XF), m0, n0,
                                        split, r_lo, r_hi);
}

template <int KS>
inline hipError_t launch_conv_stencil_s2_fwd(int wo, const ConvParams &p, hipStream_t stream) {
    using P = ConvFwdProblem<true>;
    const dim3 grid(((p.M + 63) / 64) * ((p.N + 127) / 128), p.splits);
    const size_t extra = P::extra_lds_bytes(p, 64, 128);
    if (extra > kTileExtraLdsMax) return hipErrorInvalidValue;
#define TAGI_LAUNCH_S2FWD(WD)                                                                      \
    case WD: {                                                                                     \
        static PerDeviceOnce once;                                                                 \
        hipError_t e = allow_dynamic_lds(                                                          \
            once, reinterpret_cast<const void *>(conv_stencil_s2_fwd_kernel<WD, KS>),              \
            (int)kTileExtraLdsMax);                                                                \
        if (e != hipSuccess) return e;                                                             \
        hipLaunchKernelGGL((conv_stencil_s2_fwd_kernel<WD, KS>), grid, dim3(512), extra, stream, p); \
        return hipGetLastError();                                                                  \
    }
    switch (wo) {
        TAGI_LAUNCH_S2FWD(4)
        TAGI_LAUNCH_S2FWD(8)
        TAGI_LAUNCH_S2FWD(16)
    }
#undef TAGI_LAUNCH_S2FWD
    return hipErrorInvalidValue;
}

// ---- weight backward -----------------------------------------------------------------------
//   D[fo][(c,t)] = sum over (b, output pixel) of delta[b][fo][pixel] * a[b][c][2*pixel + tap t]
// As the unit-stride kernel of tagi_conv_stencil.h: rows are output channels, the 64
// columns of a tile are consecutive (channel, tap) pairs (8 channels of 9 taps or 16 of 4),
// the reduction runs over output pixels 64 at a time = 64/WO whole output rows, whose input
// rows are staged per k-tile (every cell rewritten, zero where a row leaves the image). A
// lane's column fixes its (channel, tap) = one LDS base address; the pixel of a reduction
// step is an immediate offset - here two cells per output pixel and two rows per output row.
template <int WO, int KS>
struct S2DwGeom {
    static constexpr int W = WO, H = WO, WI = 2 * WO, T = KS * KS;
    static constexpr int KP = 64;                          // output pixels per k-tile
    static constexpr int KC = KS == 3 ? 8 : 16;            // channels a column tile can touch
    static constexpr int NR = KP / W;                      // output rows per k-tile
    static constexpr int RPI = NR < H ? NR : H;
    static constexpr int SEGS = NR / RPI;
    static constexpr int PR = 2 * RPI + KS - 2;            // staged input rows per segment
    static constexpr int RS = WI + 4;                      // values, one zero cell, 3 unused
    static constexpr int SEG = PR * RS;
    static constexpr int CS = SEGS * SEG + 4;
    static constexpr int PATCH = KC * CS;
    static constexpr int UNITS = KC * SEGS * PR * (WI / 4);
    static constexpr int P_SLOTS = (UNITS + 511) / 512;
    static constexpr int AS = KP + 4;                      // innovation tile [64 rows][64 pixels + 4]
    static constexpr int LOG_PIX = WO == 4 ? 4 : WO == 8 ? 6 : 8;
    static_assert(P_SLOTS <= 2 && KP % W == 0 && NR % RPI == 0 && H % RPI == 0, "tile geometry");
    // LDS offset of the cell (2*oy, 2*ox) of output pixel k (0..63) of the k-tile
    static constexpr int pixel_offset(int k) {
        return ((k / W) / RPI) * SEG + 2 * ((k / W) % RPI) * RS + 2 * (k % W);
    }
};

template <int WO, int KS>
__device__ __forceinline__ void s2_dw_body(const ConvParams &p, float *lds, int m0, int n0,
                                           int split, int r_begin, int r_end) {
    using G = S2DwGeom<WO, KS>;
    constexpr int W = G::W, H = G::H, WI = G::WI, T = G::T, NT = 512, PIX = W * H, PIXI = WI * WI;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // eight waves: 2 x 2 sub-tiles of 32 x 32, each held by two waves that take the
    // first / second 32 pixels of every k-tile and add up at the end
    const int kgroup = wave >> 2;
    const int wrow = ((wave & 3) / 2) * 32, wcol = (wave & 1) * 32, half = lane >> 5;
    float *lds_a = lds;                        // [2][64][AS]
    float *lds_p = lds + 2 * 64 * G::AS;       // [PATCH]
    const int c_lo = n0 / T;                   // first channel of the column tile

    for (int i = tid; i < G::PATCH; i += NT) lds_p[i] = 0.f;

    // patch units: channel pc, segment, staged row pr, columns 4*x4 ... Output rows are
    // counted over the whole batch; `grow` is the first output row of the k-tile.
    int pseg[G::P_SLOTS], prw[G::P_SLOTS], pdst[G::P_SLOTS], pchan[G::P_SLOTS];
    bool has_unit[G::P_SLOTS];
#pragma unroll
    for (int i = 0; i < G::P_SLOTS; i++) {
        int u = tid + i * NT;
        has_unit[i] = u < G::UNITS;
        u = has_unit[i] ? u : 0;
        const int x4 = u % (WI / 4);
        u /= (WI / 4);
        prw[i] = u % G::PR;
        u /= G::PR;
        pseg[i] = u % G::SEGS;
        const int pc = u / G::SEGS;
        // channels past the layer's last one (a partial last column tile) are never read
        has_unit[i] = has_unit[i] && c_lo + pc < p.fi;
        pdst[i] = pc * G::CS + pseg[i] * G::SEG + prw[i] * G::RS + 4 * x4;
        pchan[i] = (c_lo + (has_unit[i] ? pc : 0)) * PIXI + 4 * x4;
    }
    int grow = r_begin / W;

    // innovation pieces: 16 bytes at pixel 4*q of rows tid/16 + 32*i
    const int q = tid % 16, arow = tid / 16;
    int gpix = r_begin + 4 * q;  // output pixel counted over the whole batch

    floatx16 acc0[1][1], acc1[1][1];
#pragma unroll
    for (int v = 0; v < 16; v++) {
        acc0[0][0][v] = 0.f;
        acc1[0][0][v] = 0.f;
    }

    float4 ra00, ra01, ra10, ra11, rp0, rp1;
    rp0 = rp1 = make_float4(0.f, 0.f, 0.f, 0.f);
    bool rp_ok0 = false, rp_ok1 = false;
#define TAGI_S2DW_PLOAD(i, R_, OK_)                                                        \
    if (i < G::P_SLOTS) {                                                                  \
        const int j_ = i < G::P_SLOTS ? i : 0;                                             \
        const int g_ = grow + pseg[j_] * G::RPI, img_ = g_ / H, y_ = 2 * (g_ - img_ * H) + prw[j_]; \
        OK_ = has_unit[j_] && y_ < 2 * H && img_ < p.B;                                    \
        R_ = *reinterpret_cast<const float4 *>(                                            \
            p.a0 + (OK_ ? (size_t)img_ * p.fi * PIXI + pchan[j_] + y_ * WI : 0));          \
    }
#define TAGI_S2DW_PPUT(i, R_, OK_)                                                         \
    if (i < G::P_SLOTS && has_unit[i < G::P_SLOTS ? i : 0])                                \
        *reinterpret_cast<float4 *>(lds_p + pdst[i < G::P_SLOTS ? i : 0]) =                \
            OK_ ? R_ : make_float4(0.f, 0.f, 0.f, 0.f);
#define TAGI_S2DW_FETCH()                                                                  \
    do {                                                                                   \
        const int b_ = gpix >> G::LOG_PIX, o_ = gpix & (PIX - 1);                          \
        const size_t at_ = ((size_t)b_ * p.fo + m0 + arow) * PIX + o_;                     \
        ra00 = *reinterpret_cast<const float4 *>(p.d0 + at_);                              \
        ra10 = *reinterpret_cast<const float4 *>(p.d1 + at_);                              \
        ra01 = *reinterpret_cast<const float4 *>(p.d0 + at_ + (size_t)32 * PIX);           \
        ra11 = *reinterpret_cast<const float4 *>(p.d1 + at_ + (size_t)32 * PIX);           \
        gpix += G::KP;                                                                     \
        TAGI_S2DW_PLOAD(0, rp0, rp_ok0) TAGI_S2DW_PLOAD(1, rp1, rp_ok1)                    \
        grow += G::NR;                                                                     \
    } while (0)
#define TAGI_S2DW_COMMIT()                                                                 \
    do {                                                                                   \
        float *d0_ = lds_a + arow * G::AS + 4 * q, *d1_ = d0_ + 64 * G::AS;                \
        *reinterpret_cast<float4 *>(d0_) = ra00;                                           \
        *reinterpret_cast<float4 *>(d0_ + 32 * G::AS) = ra01;                              \
        *reinterpret_cast<float4 *>(d1_) = ra10;                                           \
        *reinterpret_cast<float4 *>(d1_ + 32 * G::AS) = ra11;                              \
        TAGI_S2DW_PPUT(0, rp0, rp_ok0) TAGI_S2DW_PPUT(1, rp1, rp_ok1)                      \
    } while (0)

    // operand addresses of this lane: its column is (channel, tap)
    const int n = min(n0 + wcol + (lane & 31), p.N - 1);
    const int ch = n / T - c_lo, t = n - (n / T) * T, ky = t / KS, kx = t - ky * KS;
    const float *bp = lds_p + ch * G::CS + ky * G::RS + kx + (half ? G::pixel_offset(4) : 0) +
                      (kgroup ? G::pixel_offset(32) : 0);
    const float *a0 = lds_a + (wrow + (lane & 31)) * G::AS + 4 * half + 32 * kgroup;
    const float *a1 = a0 + 64 * G::AS;

    __syncthreads();  // patch zeroed
    if (r_begin < r_end) {
        TAGI_S2DW_FETCH();
        TAGI_S2DW_COMMIT();
    }
    __syncthreads();

    for (int r0 = r_begin; r0 < r_end; r0 += G::KP) {
        const bool more = r0 + G::KP < r_end;
        if (more) TAGI_S2DW_FETCH();
#pragma unroll
        for (int kk = 0; kk < G::KP / 2; kk += 8) {
            const float4 dm = *reinterpret_cast<const float4 *>(a0 + kk);
            const float4 dv = *reinterpret_cast<const float4 *>(a1 + kk);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float y = bp[G::pixel_offset(kk + e)];
                acc0[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(comp4(dm, e), y, acc0[0][0], 0, 0, 0);
                acc1[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(comp4(dv, e), y * y, acc1[0][0], 0, 0, 0);
            }
        }
        __syncthreads();
        if (more) {
            TAGI_S2DW_COMMIT();
            __syncthreads();
        }
    }
#undef TAGI_S2DW_FETCH
#undef TAGI_S2DW_COMMIT
#undef TAGI_S2DW_PLOAD
#undef TAGI_S2DW_PPUT

    // the second pixel group hands its sums over through LDS ([value][lane] layout)
    float *xch = lds;
    if (kgroup == 1) {
#pragma unroll
        for (int v = 0; v < 16; v++) {
            xch[v * 256 + (tid - 256)] = acc0[0][0][v];
            xch[(16 + v) * 256 + (tid - 256)] = acc1[0][0][v];
        }
    }
    __syncthreads();
    if (kgroup == 1) return;
#pragma unroll
    for (int v = 0; v < 16; v++) {
        acc0[0][0][v] += xch[v * 256 + tid];
        acc1[0][0][v] += xch[(16 + v) * 256 + tid];
    }
    tile_epilogue<ConvDwVecProblem, 64, 64, 2, 2>(p, acc0, acc1, m0, n0, split);
}

template <int WO, int KS>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4)))
void conv_stencil_s2_dw_kernel(ConvParams p) {
    using G = S2DwGeom<WO, KS>;
    using P = ConvDwVecProblem;
    constexpr int T = KS * KS;
    constexpr int XF = TileGeom<P::XK, 64>::floats, YF = TileGeom<P::YK, 64>::floats;
    constexpr int GENERIC = P::NX * XF + P::NY * YF;
    constexpr int STENCIL = 2 * 64 * G::AS + G::PATCH;
    static_assert(2 * 64 * G::AS >= 32 * 256, "the innovation tiles hold the final exchange");
    __shared__ __attribute__((aligned(16))) float lds[GENERIC > STENCIL ? GENERIC : STENCIL];
    __shared__ int regular_flag;

    const int tiles_n = (p.N + 63) / 64;
    int tile = blockIdx.x, split = blockIdx.y;
    if (gridDim.y % 8 == 0) {
        // all column tiles of one reduction slice on one XCD (see mfma_tile_kernel)
        const int id = blockIdx.y * gridDim.x + blockIdx.x;
        const int qq = id >> 3;
        tile = qq % gridDim.x;
        split = (qq / gridDim.x) * 8 + (id & 7);
    }
    const int m0 = (tile / tiles_n) * 64, n0 = (tile % tiles_n) * 64;
    const int r_begin = split * p.r_per_split;
    const int r_end = min(p.R, r_begin + p.r_per_split);

    // the output pixels of this slice, per image position: all of Fmwa_2 once the slice is
    // as long as a map; entries are requested six at a time before any is looked at
    if (threadIdx.x == 0) regular_flag = 1;
    __syncthreads();
    {
        const int total = min(max(r_end - r_begin, 0), p.woho) * T;
        bool ok = true;
        for (int base = threadIdx.x; base < total; base += 6 * 512) {
            int got[6], want[6];
#pragma unroll
            for (int i = 0; i < 6; i++) {
                const int e = base + i * 512, c = e / T, t = e - c * T;
                const bool live = e < total;
                const int o = live ? (r_begin + c) & (WO * WO - 1) : 0;
                got[i] = p.idx[live ? o * T + t : 0];
                want[i] = live ? s2_fmwa<WO, KS>(o, t) : got[i];
            }
#pragma unroll
            for (int i = 0; i < 6; i++) ok = ok && got[i] == want[i];
        }
        if (!ok) regular_flag = 0;
    }
    __syncthreads();
    if (__builtin_amdgcn_readfirstlane(regular_flag)) {
        s2_dw_body<WO, KS>(p, lds, m0, n0, split, r_begin, r_end);
        return;
    }
    // table-driven loop: written for four waves; the other four leave
    if (threadIdx.x >= 256) return;
    typename P::Ctx ctx;
    P::prologue(p, ctx, nullptr, threadIdx.x, 256, m0, n0, 64, 64, r_begin, r_end);
    mfma_tile_body<P, 64, 64, 2, 2, 0>(p, ctx, reinterpret_cast<float (*)[XF]>(lds),
                                       reinterpret_cast<float (*)[YF]>(lds + P::NX * XF), m0, n0,
                                       split, r_begin, r_end);
}

template <int KS>
inline hipError_t launch_conv_stencil_s2_dw(int wo, const ConvParams &p, hipStream_t stream) {
    const dim3 grid(((p.M + 63) / 64) * ((p.N + 63) / 64), p.splits);
    switch (wo) {
        case 4: hipLaunchKernelGGL((conv_stencil_s2_dw_kernel<4, KS>), grid, dim3(512), 0, stream, p); break;
        case 8: hipLaunchKernelGGL((conv_stencil_s2_dw_kernel<8, KS>), grid, dim3(512), 0, stream, p); break;
        case 16: hipLaunchKernelGGL((conv_stencil_s2_dw_kernel<16, KS>), grid, dim3(512), 0, stream, p); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// Output map width for which the strided kernels exist, 0 otherwise.
inline int s2_out_width(int out_pixels) {
    for (int w : {4, 8, 16})
        if (w * w == out_pixels) return w;
    return 0;
}

}  // namespace
}  // namespace tagi

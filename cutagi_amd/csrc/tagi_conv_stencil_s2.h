// Regular-stencil kernels for the strided convolutions of a ResNet: 3x3 kernel,
// stride 2, one pixel of padding on the right and bottom only (the reference's
// padding type 2: tap (ky, kx) of output pixel (oy, ox) reads input pixel
// (2*oy + ky, 2*ox + kx), src/indices.cpp:63-103), on square input maps of width
// 8, 16 or 32. As in tagi_conv_stencil.h every workgroup first CHECKS the index
// tables it was given against that stencil, for its own pixels, and runs the
// table-driven loop if anything differs.
//
// State backward. An input pixel (y, x) is reached through the taps whose parity
// matches its own: ky = y mod 2 (mod 2), kx likewise, i.e. through 4, 2, 2 or 1 of
// the 9 taps by phase (y mod 2, x mod 2), from the output pixels
// ((y - ky) / 2, (x - kx) / 2). With the columns numbered phase by phase
// (ConvParams::perm_s = 2) a 128-column tile holds pixels (2*ly + py, 2*lx + px) of
// ONE phase, and on the (ly, lx) grid of that phase the contraction is a small
// stencil over the innovation maps: taps at offsets (-(ky / 2), -(kx / 2)), all in
// {-1, 0}. So the workgroup stages the innovation rows of its channels once, with a
// zero halo on top and left, and every tap is a constant offset into that patch. A
// k-tile holds 32 / T output channels for a phase with T taps, which makes every
// k-tile 16 MFMA steps per k-half whatever the phase; only the weights of the
// phase's taps are staged.
//
// Included by tagi_conv2d.hip after tagi_conv_stencil.h.
#pragma once

namespace tagi {
namespace {

// ---- state backward ------------------------------------------------------------------

// Taps of the phase class: PY / PX = parity of the input row / column.
template <int PY, int PX>
struct PhaseTaps {
    static constexpr int TY = PY == 0 ? 2 : 1, TX = PX == 0 ? 2 : 1, T = TY * TX;
    // the i-th tap of the phase (row-major over its rows and columns)
    static constexpr int ky(int i) { return PY == 0 ? 2 * (i / TX) : 1; }
    static constexpr int kx(int i) { return PX == 0 ? 2 * (i % TX) : 1; }
};

// Expected (tap, output pixel) occurrences of input pixel (y, x) on a 2*WO-wide map;
// returns the tap mask, out[t] = 1-based output pixel of tap t.
template <int WO>
__device__ __forceinline__ int s2_occurrences(int y, int x, int (&out)[9]) {
    int mask = 0;
#pragma unroll
    for (int t = 0; t < 9; t++) {
        const int ky = t / 3, kx = t - ky * 3;
        const int ny = y - ky, nx = x - kx;
        const bool hit = ny >= 0 && nx >= 0 && (ny & 1) == 0 && (nx & 1) == 0 &&
                         (ny >> 1) < WO && (nx >> 1) < WO;
        out[t] = hit ? (ny >> 1) * WO + (nx >> 1) + 1 : 0;
        mask |= hit ? 1 << t : 0;
    }
    return mask;
}

// Do FCzwa_1 [wihi][nr] / Szz_ud [nr][wihi] list exactly those occurrences for the
// pixels of columns n0 .. n0+127 (any order within a pixel's list)? Uniform verdict.
// `scratch` holds 130 ints of LDS.
template <int WO>
__device__ __forceinline__ bool s2_dz_tables_ok(const ConvParams &p, int n0, int tid, int nthreads,
                                                int *scratch) {
    int *flag = scratch, *seen = scratch + 2;
    if (tid == 0) *flag = 1;
    if (tid < 128) seen[tid] = 0;
    __syncthreads();
    bool ok = p.nr >= 1 && p.nr <= 9;
    const int entries = 128 * min(max(p.nr, 1), 9);
    for (int e = tid; e < entries; e += nthreads) {
        const int j = e >> 7, c = e & 127, n = n0 + c;
        if (n >= p.N) continue;
        const int px = dz_column(p, n).px;
        const int o = p.idx2[j * p.wihi + px], tap = p.idx[px * p.nr + j];
        if (o <= -1) continue;
        if (tap < 1 || tap > 9) {
            ok = false;
            continue;
        }
        int want[9];
        const int y = px / (2 * WO), x = px - y * (2 * WO);
        const int mask = s2_occurrences<WO>(y, x, want);
        const int t = tap - 1;
        int w = 0;
#pragma unroll
        for (int q = 0; q < 9; q++) w = q == t ? want[q] : w;
        ok = ok && (mask >> t & 1) && o == w;
        if (atomicOr(&seen[c], 1 << t) >> t & 1) ok = false;  // listed twice
    }
    __syncthreads();
    if (tid < 128 && n0 + tid < p.N) {
        const int px = dz_column(p, n0 + tid).px;
        int want[9];
        const int y = px / (2 * WO), x = px - y * (2 * WO);
        ok = ok && seen[tid] == s2_occurrences<WO>(y, x, want);
    }
    if (!ok) *flag = 0;
    __syncthreads();
    const bool verdict = __builtin_amdgcn_readfirstlane(*flag) != 0;
    __syncthreads();
    return verdict;
}

template <int WO, int T>
struct S2DzGeom {
    using G = StencilGeom<WO>;               // patch layout of one channel: rows -1 .. RPI, zero halo
    // output channels per k-tile (the narrowest maps hold eight images per tile: their
    // patch is kept to 16 channels so that two workgroups still share a CU)
    static constexpr int KC = (WO == 4 && T == 1) ? 16 : 32 / T;
    static constexpr int PATCH = KC * G::CS;
    // rows -1 .. RPI-1 are read (taps reach up and left only); the bottom halo row is
    // never loaded and stays zero
    static constexpr int UNITS = KC * G::SEGS * (G::RPI + 1) * (WO / 4);
    static constexpr int P_SLOTS = (UNITS + 511) / 512;
    static constexpr int WS = 64 + 4;        // weight tile [T][KC][64 rows + 4]
    static constexpr int W_FLOATS = T * KC * WS;
    static constexpr int W_SLOTS = T * KC * 64 / 512;  // 4
    static constexpr int LDS_FLOATS = W_FLOATS + 2 * PATCH;
};

// One 64 x 128 tile of one phase on a verified stencil. c_begin / c_end: output
// channels of the reduction slice (multiples of 32).
template <int WO, int PY, int PX>
__device__ __forceinline__ void s2_dz_body(const ConvParams &p, float *lds, int m0, int n0,
                                           int split, int c_begin, int c_end) {
    using PT = PhaseTaps<PY, PX>;
    constexpr int T = PT::T;
    using S = S2DzGeom<WO, T>;
    using G = StencilGeom<WO>;
    constexpr int W = WO, H = WO, NT = 512, KC = S::KC;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wrow = (wave / 4) * 32, wcol = (wave % 4) * 32, half = lane >> 5;
    float *lds_w = lds;                 // [T][KC][WS]
    float *lds_p = lds + S::W_FLOATS;   // [PATCH][2]: (delta_mu, delta_var) interleaved

    for (int i = tid; i < 2 * S::PATCH; i += NT) lds_p[i] = 0.f;

    // position of the tile inside its phase: pixels (b, ly, lx) in the order of the
    // innovation maps
    const int per_phase = p.B * W * H;
    const int q0 = n0 % per_phase;

    // patch units of this thread
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

    // weight elements of this thread: w[f][m0 + row][tap ti], row fastest
    size_t wsrc[S::W_SLOTS];
    int wdst[S::W_SLOTS];
#pragma unroll
    for (int i = 0; i < S::W_SLOTS; i++) {
        const int e = tid + i * NT, row = e & 63, rest = e >> 6, f = rest % KC, ti = rest / KC;
        int tap = 0;
#pragma unroll
        for (int q = 0; q < T; q++) tap = q == ti ? PT::ky(q) * 3 + PT::kx(q) : tap;
        wsrc[i] = ((size_t)(c_begin + f) * p.fi + m0 + row) * 9 + tap;
        wdst[i] = (ti * KC + f) * S::WS + row;
    }
    const size_t wstep = (size_t)KC * p.fi * 9;

    floatx16 acc0[1][1], acc1[1][1];
#pragma unroll
    for (int v = 0; v < 16; v++) {
        acc0[0][0][v] = 0.f;
        acc1[0][0][v] = 0.f;
    }

    float4 rp0[S::P_SLOTS], rp1[S::P_SLOTS];
    float rw[S::W_SLOTS];

#define TAGI_S2DZ_FETCH()                                                             \
    do {                                                                              \
        _Pragma("unroll") for (int i = 0; i < S::W_SLOTS; i++) {                      \
            rw[i] = p.w0[wsrc[i]];                                                    \
            wsrc[i] += wstep;                                                         \
        }                                                                             \
        _Pragma("unroll") for (int i = 0; i < S::P_SLOTS; i++) {                      \
            rp0[i] = *reinterpret_cast<const float4 *>(p.d0 + punit[i]);              \
            rp1[i] = *reinterpret_cast<const float4 *>(p.d1 + punit[i]);              \
            if (p_ok[i]) punit[i] += pstep;                                           \
        }                                                                             \
    } while (0)
#define TAGI_S2DZ_COMMIT()                                                            \
    do {                                                                              \
        _Pragma("unroll") for (int i = 0; i < S::W_SLOTS; i++) lds_w[wdst[i]] = rw[i]; \
        _Pragma("unroll") for (int i = 0; i < S::P_SLOTS; i++) if (p_ok[i]) {         \
            *reinterpret_cast<float4 *>(lds_p + 2 * pdst[i]) =                        \
                make_float4(rp0[i].x, rp1[i].x, rp0[i].y, rp1[i].y);                  \
            *reinterpret_cast<float4 *>(lds_p + 2 * pdst[i] + 4) =                    \
                make_float4(rp0[i].z, rp1[i].z, rp0[i].w, rp1[i].w);                  \
        }                                                                             \
    } while (0)

    // operand addresses of this lane: patch cell (row ly - 1, column lx - 1) of its pixel
    // for output channel `half` of a pair; weights of its row
    const int pix = wcol + (lane & 31), prow = pix / W, px = pix - prow * W;
    const float *bp = lds_p + 2 * (half * G::CS + (prow / G::RPI) * G::SEG +
                                   (prow % G::RPI) * G::RS + G::XO - 1 + px);
    const float *wp = lds_w + half * S::WS + wrow + (lane & 31);

    __syncthreads();  // patch zeroed
    if (c_begin < c_end) {
        TAGI_S2DZ_FETCH();
        TAGI_S2DZ_COMMIT();
    }
    __syncthreads();

    for (int c0 = c_begin; c0 < c_end; c0 += KC) {
        const bool more = c0 + KC < c_end;
        if (more) TAGI_S2DZ_FETCH();
#pragma unroll
        for (int pair = 0; pair < KC / 2; pair++) {
#pragma unroll
            for (int ti = 0; ti < T; ti++) {
                // tap (ky, kx) brings the innovation of output pixel (ly - ky/2, lx - kx/2)
                const int off = (1 - PT::ky(ti) / 2) * G::RS + (1 - PT::kx(ti) / 2);
                const float2 y = *reinterpret_cast<const float2 *>(bp + 2 * (2 * pair * G::CS + off));
                const float w = wp[(ti * KC + 2 * pair) * S::WS];
                acc0[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(w, y.x, acc0[0][0], 0, 0, 0);
                acc1[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(w * w, y.y, acc1[0][0], 0, 0, 0);
            }
        }
        __syncthreads();
        if (more) {
            TAGI_S2DZ_COMMIT();
            __syncthreads();
        }
    }
#undef TAGI_S2DZ_FETCH
#undef TAGI_S2DZ_COMMIT
    tile_epilogue<ConvDzProblem, 64, 128, 2, 4>(p, acc0, acc1, m0, n0, split);
}

template <int WO>
struct S2DzLds {
    using P = ConvDzProblem;
    static constexpr int XF = TileGeom<P::XK, 64>::floats, YF = TileGeom<P::YK, 128>::floats;
    static constexpr int GENERIC = P::NX * XF + P::NY * YF;
    static constexpr int a = S2DzGeom<WO, 4>::LDS_FLOATS, b = S2DzGeom<WO, 2>::LDS_FLOATS,
                         c = S2DzGeom<WO, 1>::LDS_FLOATS;
    static constexpr int m1 = a > b ? a : b, m2 = m1 > c ? m1 : c;
    static constexpr int FLOATS = m2 > GENERIC ? m2 : GENERIC;
};

// One 64 x 128 tile per workgroup of 8 waves; columns are numbered phase by phase
// (perm_s = 2) and a tile lies inside one phase (batch * WO * WO is a multiple of 128).
template <int WO>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4)))
void conv_stencil_s2_dz_kernel(ConvParams p) {
    using P = ConvDzProblem;
    using L = S2DzLds<WO>;
    __shared__ __attribute__((aligned(16))) float lds[L::FLOATS];
    extern __shared__ __attribute__((aligned(16))) int lds_extra[];

    const int tiles_n = (p.N + 127) / 128;
    const int split = blockIdx.y;
    const int tile = P::place_tile(p, blockIdx.x, split, gridDim.x);
    const int m0 = (tile / tiles_n) * 64, n0 = (tile % tiles_n) * 128;
    const int r_begin = split * p.r_per_split;
    const int r_end = min(p.R, r_begin + p.r_per_split);

    if (s2_dz_tables_ok<WO>(p, n0, threadIdx.x, 512, lds_extra)) {
        const int phase = n0 / (p.B * WO * WO);
        const int c_begin = r_begin / 9, c_end = r_end / 9;
        switch (phase) {
            case 0: s2_dz_body<WO, 0, 0>(p, lds, m0, n0, split, c_begin, c_end); break;
            case 1: s2_dz_body<WO, 0, 1>(p, lds, m0, n0, split, c_begin, c_end); break;
            case 2: s2_dz_body<WO, 1, 0>(p, lds, m0, n0, split, c_begin, c_end); break;
            default: s2_dz_body<WO, 1, 1>(p, lds, m0, n0, split, c_begin, c_end); break;
        }
        return;
    }
    typename P::Ctx ctx;
    P::prologue(p, ctx, lds_extra, threadIdx.x, 512, m0, n0, 64, 128, r_begin, r_end);
    __syncthreads();
    int r_lo = r_begin, r_hi = r_end;
    P::adjust_range(p, ctx, r_lo, r_hi);
    mfma_tile_body<P, 64, 128, 2, 4, 0>(p, ctx, reinterpret_cast<float (*)[L::XF]>(lds),
                                        reinterpret_cast<float (*)[L::YF]>(lds + P::NX * L::XF), m0,
                                        n0, split, r_lo, r_hi);
}

// Output map width for which the strided kernels exist, 0 otherwise.
inline int s2_out_width(int out_pixels) {
    for (int w : {4, 8, 16})
        if (w * w == out_pixels) return w;
    return 0;
}

inline hipError_t launch_conv_stencil_s2_dz(int wo, const ConvParams &p, hipStream_t stream) {
    using P = ConvDzProblem;
    const dim3 grid(((p.M + 63) / 64) * ((p.N + 127) / 128), p.splits);
    const size_t extra = P::extra_lds_bytes(p, 64, 128);
    if (extra > kTileExtraLdsMax) return hipErrorInvalidValue;
#define TAGI_LAUNCH_S2DZ(WD)                                                                    \
    case WD: {                                                                                  \
        static PerDeviceOnce once;                                                              \
        hipError_t e = allow_dynamic_lds(                                                       \
            once, reinterpret_cast<const void *>(conv_stencil_s2_dz_kernel<WD>),                \
            (int)kTileExtraLdsMax);                                                             \
        if (e != hipSuccess) return e;                                                          \
        hipLaunchKernelGGL((conv_stencil_s2_dz_kernel<WD>), grid, dim3(512), extra, stream, p); \
        return hipGetLastError();                                                               \
    }
    switch (wo) {
        TAGI_LAUNCH_S2DZ(4)
        TAGI_LAUNCH_S2DZ(8)
        TAGI_LAUNCH_S2DZ(16)
    }
#undef TAGI_LAUNCH_S2DZ
    return hipErrorInvalidValue;
}

}  // namespace
}  // namespace tagi

// Conv2d forward and state backward for the geometry that carries almost all of
// a ResNet's work: 3x3 kernel, stride 1, one pixel of padding on every side, on
// square maps of width 4, 8, 16 or 32. For it the reference's index tables
// (src/conv2d_layer.cpp:274-323, 363-404 read them per tap) describe a regular
// stencil: tap (ky, kx) of output pixel (y, x) reads input pixel (y+ky-1, x+kx-1),
// and nothing outside the map. Each workgroup first CHECKS that against the
// tables it was given, for its own pixels; only then does it take the path below,
// otherwise the table-driven kernel body runs (included from tagi_conv2d.hip, so
// any table still gives the table's result).
//
// What the regular stencil buys: a 128-pixel tile is 128/W whole image rows, so
// instead of gathering nine shifted copies of every channel map (nine loads and
// nine table lookups per element) the workgroup stages each channel's rows ONCE,
// with a zero halo, and the nine taps are nine constant offsets into that patch
// when the MFMA operand is read from LDS. The k-tile is 8 channels x 9 taps = 72
// reduction steps; the two MFMA k-halves (lanes 0-31 / 32-63) take two channels a
// fixed distance apart at the same tap, so one LDS address per lane plus an
// immediate per step reaches every operand. Weights are staged in the order they
// have in memory (16-byte commits). What sits between the two barriers of a
// k-tile is exposed, LDS reads during the MFMAs are not, so layouts favour cheap
// commits over wide reads.
//
// Included by tagi_conv2d.hip after ConvParams, ConvFwdProblem and ConvDzProblem.
#pragma once

namespace tagi {
namespace {

template <int WIDTH>
struct StencilGeom {
    static constexpr int W = WIDTH, H = WIDTH;     // square maps
    static constexpr int BM = 64, BN = 128;        // output tile: rows x pixels
    static constexpr int KC = 8;                   // channels per k-tile
    static constexpr int NR = BN / W;              // image rows per tile
    static constexpr int RPI = NR < H ? NR : H;    // rows of one image among them
    static constexpr int SEGS = NR / RPI;          // images (segments) per tile
    // One patch row: [3 unused][left halo][W values][right halo = cell 0 of the
    // next row]; values start 16-byte aligned. Unused and halo cells stay zero.
    static constexpr int XO = 4;
    static constexpr int RS = W + 4;
    // Rows r = -1 .. RPI of a segment; the pad of the narrowest map moves the
    // second image of a 32-pixel column block onto other LDS banks.
    static constexpr int SEG = (RPI + 2) * RS + (W == 4 ? 4 : 0);
    static constexpr int CS = SEGS * SEG + 4;      // one channel (+ the last row's halo cell)
    static constexpr int PATCH = KC * CS;          // floats per staged array
    static constexpr int UNITS = KC * SEGS * (RPI + 2) * (W / 4);  // 16-byte loads per array
    // Weight tile [64 rows][2 k-halves][36 steps], row stride 76: eight consecutive
    // rows start on eight different groups of four banks. Forward: a half is four
    // channels in memory order; state backward: the even / odd channels.
    static constexpr int AS = 76;
    static constexpr int A_VEC = BM * KC * 9 / 4;  // 16-byte loads per weight array
    static_assert(UNITS <= 512 && BN % W == 0 && NR % RPI == 0 && H % RPI == 0, "tile geometry");
};

// Expected Fmwa_2 entry (1-based input pixel, -1 = padding) of tap t of output
// pixel o on a W x W map.
template <int W>
__device__ __forceinline__ int stencil_fmwa(int o, int t) {
    const int y = o / W, x = o - y * W;
    const int iy = y + t / 3 - 1, ix = x + t % 3 - 1;
    return (iy >= 0 && iy < W && ix >= 0 && ix < W) ? iy * W + ix + 1 : -1;
}

// Does the table describe the regular stencil for the pixels n0 .. n0+127? All
// threads of the workgroup call this; the verdict is uniform. `scratch` holds
// 130 ints of LDS. Table entries are requested in batches before any is looked
// at, so that the check costs one memory latency, not one per entry.
template <bool DZ, int WIDTH>
__device__ __forceinline__ bool stencil_tables_ok(const ConvParams &p, int n0, int tid,
                                                  int nthreads, int *scratch) {
    constexpr int W = WIDTH, H = WIDTH, PAIRS = 128 * 9;
    int *flag = scratch, *seen = scratch + 2;
    if (tid == 0) *flag = 1;
    if (DZ && tid < 128) seen[tid] = 0;
    __syncthreads();
    bool ok = true;
    if (!DZ) {
        // Fmwa_2 [woho][9]
        int got[3], want[3];
#pragma unroll
        for (int i = 0; i < 3; i++) {
            const int e = tid + i * nthreads, c = e / 9, t = e - c * 9, n = n0 + c;
            const bool live = e < PAIRS && n < p.N;
            const int o = live ? n % p.woho : 0;
            got[i] = p.idx[live ? o * 9 + t : 0];
            want[i] = live ? stencil_fmwa<W>(o, t) : got[i];
        }
#pragma unroll
        for (int i = 0; i < 3; i++) ok = ok && got[i] == want[i];
    } else {
        // FCzwa_1 [wihi][nr] / Szz_ud [nr][wihi]: per input pixel the (tap, output
        // pixel) pairs that touch it, in any order (nr = 9). Regular stencil: tap t
        // touches pixel (y, x) from output pixel (y-ky+1, x-kx+1) when that lies in
        // the map; every such tap must be listed exactly once.
        int out[3], tap[3], col[3];
#pragma unroll
        for (int i = 0; i < 3; i++) {
            const int e = tid + i * nthreads, j = e / 128, c = e - j * 128, n = n0 + c;
            const bool live = e < PAIRS && n < p.N;
            const int px = live ? n % p.wihi : 0;
            out[i] = p.idx2[live ? j * p.wihi + px : 0];
            tap[i] = p.idx[live ? px * 9 + j : 0];
            col[i] = live ? c : -1;
        }
#pragma unroll
        for (int i = 0; i < 3; i++) {
            if (col[i] < 0 || out[i] <= -1) continue;
            const int px = (n0 + col[i]) % p.wihi, y = px / W, x = px - y * W;
            if (tap[i] < 1 || tap[i] > 9) {
                ok = false;
                continue;
            }
            const int t = tap[i] - 1, qy = y - t / 3 + 1, qx = x - t % 3 + 1;
            ok = ok && qy >= 0 && qy < H && qx >= 0 && qx < W && out[i] == qy * W + qx + 1;
            if (atomicOr(&seen[col[i]], 1 << t) >> t & 1) ok = false;  // listed twice
        }
        __syncthreads();
        if (tid < 128 && n0 + tid < p.N) {
            const int px = (n0 + tid) % p.wihi, y = px / W, x = px - y * W;
            int want = 0;
#pragma unroll
            for (int t = 0; t < 9; t++) {
                const int qy = y - t / 3 + 1, qx = x - t % 3 + 1;
                if (qy >= 0 && qy < H && qx >= 0 && qx < W) want |= 1 << t;
            }
            ok = ok && seen[tid] == want;
        }
    }
    if (!ok) *flag = 0;
    __syncthreads();
    const bool verdict = __builtin_amdgcn_readfirstlane(*flag) != 0;
    __syncthreads();  // scratch may be reused
    return verdict;
}

// The tile loop on a verified stencil. `lds` holds the weight tile(s) followed by
// the two patches. r_begin / r_end are multiples of 72 (whole channels of 9 taps,
// 8 at a time).
template <bool DZ, int WIDTH>
__device__ __forceinline__ void stencil_body(const ConvParams &p, float *lds, int m0, int n0,
                                             int split, int r_begin, int r_end) {
    using G = StencilGeom<WIDTH>;
    using P = typename std::conditional<DZ, ConvDzProblem, ConvFwdProblem<true>>::type;
    constexpr int W = G::W, H = G::H, NA = DZ ? 1 : 2, NT = 512;
    constexpr int SLOTS = (G::A_VEC + NT - 1) / NT;  // 3
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wrow = (wave / 4) * 32, wcol = (wave % 4) * 32, half = lane >> 5;
    float *lds_a = lds;                       // [NA][64][AS]
    float *lds_p = lds + NA * 64 * G::AS;     // [PATCH][2]: the two gathered arrays interleaved,
                                              // so that one 8-byte read fetches a lane's pair
    // gathered tensor: activations [B][fi][W*H] (forward), innovations [B][fo][W*H]
    const float *src0 = DZ ? p.d0 : p.a0, *src1 = DZ ? p.d1 : p.a1;
    const int CH = DZ ? p.fo : p.fi;
    const int c_begin = r_begin / 9, c_end = r_end / 9;

    for (int i = tid; i < 2 * G::PATCH; i += NT) lds_p[i] = 0.f;

    // this thread's 16 bytes of the patch: channel c, segment, patch row pr, column 4*x4
    int u = tid < G::UNITS ? tid : 0;
    const int x4 = u % (W / 4);
    u /= (W / 4);
    const int pr = u % (G::RPI + 2);
    u /= (G::RPI + 2);
    const int seg = u % G::SEGS, pc = u / G::SEGS;
    const int grow = n0 / W + seg * G::RPI;  // first image row of the segment, counted over the batch
    const int img = grow / H, y = grow % H + pr - 1;
    const bool unit_ok = tid < G::UNITS && y >= 0 && y < H && img < p.B;
    // a unit outside the map loads element 0 instead and is never written
    size_t punit = unit_ok ? ((size_t)img * CH + c_begin + pc) * (W * H) + y * W + 4 * x4 : 0;
    const size_t pstep = unit_ok ? (size_t)G::KC * (W * H) : 0;
    const int pdst = pc * G::CS + seg * G::SEG + pr * G::RS + G::XO + 4 * x4;

    // this thread's 16-byte pieces of the weight tile and where they go in LDS
    size_t aunit[SLOTS];
    int adst[SLOTS];
    bool a_ok[SLOTS];
    const size_t astep = DZ ? (size_t)G::KC * p.fi * 9 : (size_t)G::KC * 9;
#pragma unroll
    for (int i = 0; i < SLOTS; i++) {
        const int idx = tid + i * NT;
        a_ok[i] = idx < G::A_VEC;
        const int id = a_ok[i] ? idx : 0;
        if (!DZ) {
            // rows = output channels, 72 consecutive values of w[row][c*9 + t]
            const int row = id / 18, q = id - row * 18;
            aunit[i] = (size_t)(m0 + row) * p.R + (size_t)c_begin * 9 + 4 * q;
            // kept in memory order (the 16 bytes stay together): lanes 0-31 of an MFMA
            // step take channels 0-3 of the k-tile = values 0-35 of the row, lanes
            // 32-63 channels 4-7
            adst[i] = row * G::AS + 4 * q;
        } else {
            // rows = input channels; for one output channel f the values
            // w[f][(m0+row)*9 + t] of the 64 rows are 576 consecutive floats
            const int f = id / 144, q = id - f * 144;
            aunit[i] = (size_t)(c_begin + f) * p.fi * 9 + (size_t)m0 * 9 + 4 * q;
            // kept in memory order too: [f][row * 9 + t] (576 values per output channel)
            adst[i] = f * 576 + 4 * q;
        }
        if (!a_ok[i]) aunit[i] = 0;
    }

    floatx16 acc0[1][1], acc1[1][1];
#pragma unroll
    for (int v = 0; v < 16; v++) {
        acc0[0][0][v] = 0.f;
        acc1[0][0][v] = 0.f;
    }

    // staging registers, named one by one (an array written in one lambda and read
    // in another is kept in scratch memory by the compiler)
    static_assert(SLOTS == 3, "three 16-byte pieces of the weight tile per thread");
    float4 rm0, rm1, rm2, rv0, rv1, rv2, rp0, rp1;
    rv0 = rv1 = rv2 = make_float4(0.f, 0.f, 0.f, 0.f);
    auto fetch = [&]() {
        rm0 = *reinterpret_cast<const float4 *>(p.w0 + aunit[0]);
        rm1 = *reinterpret_cast<const float4 *>(p.w0 + aunit[1]);
        rm2 = *reinterpret_cast<const float4 *>(p.w0 + aunit[2]);
        if (NA == 2) {
            rv0 = *reinterpret_cast<const float4 *>(p.w1 + aunit[0]);
            rv1 = *reinterpret_cast<const float4 *>(p.w1 + aunit[1]);
            rv2 = *reinterpret_cast<const float4 *>(p.w1 + aunit[2]);
        }
#pragma unroll
        for (int i = 0; i < SLOTS; i++)
            if (a_ok[i]) aunit[i] += astep;
        rp0 = *reinterpret_cast<const float4 *>(src0 + punit);
        rp1 = *reinterpret_cast<const float4 *>(src1 + punit);
        punit += pstep;
    };
    auto put = [&](float *dst, int i, const float4 &v) {
        if (a_ok[i]) *reinterpret_cast<float4 *>(dst + adst[i]) = v;
    };
    auto commit = [&]() {
        put(lds_a, 0, rm0);
        put(lds_a, 1, rm1);
        put(lds_a, 2, rm2);
        if (NA == 2) {
            put(lds_a + 64 * G::AS, 0, rv0);
            put(lds_a + 64 * G::AS, 1, rv1);
            put(lds_a + 64 * G::AS, 2, rv2);
        }
        if (unit_ok) {
            *reinterpret_cast<float4 *>(lds_p + 2 * pdst) = make_float4(rp0.x, rp1.x, rp0.y, rp1.y);
            *reinterpret_cast<float4 *>(lds_p + 2 * pdst + 4) =
                make_float4(rp0.z, rp1.z, rp0.w, rp1.w);
        }
    };

    // operand addresses of this lane
    const int pix = wcol + (lane & 31), prow = pix / W, px = pix - prow * W;
    // k-halves of an MFMA step: forward, channels c and c + 4 (weights stay in memory
    // order); state backward, channels 2c and 2c + 1
    constexpr int HALF_CH = DZ ? 1 : 4, STEP_CH = DZ ? 2 : 1;
    const float *bp = lds_p + 2 * (half * HALF_CH * G::CS + (prow / G::RPI) * G::SEG +
                                   (prow % G::RPI) * G::RS + G::XO - 1 + px);
    // weights: forward [row][72] (a lane reads four steps with 16 bytes); state
    // backward [f][row*9 + t] (one value per step; 32 rows at stride 9 floats fall on
    // 32 different banks)
    const float *a0 = DZ ? lds_a + (wrow + (lane & 31)) * 9 + half * 576
                         : lds_a + (wrow + (lane & 31)) * G::AS + half * 36;
    const float *a1 = a0 + 64 * G::AS;

    __syncthreads();  // patch zeroed
    if (c_begin < c_end) {
        fetch();
        commit();
    }
    __syncthreads();

    for (int c0 = c_begin; c0 < c_end; c0 += G::KC) {
        const bool more = c0 + G::KC < c_end;
        if (more) fetch();
#pragma unroll
        for (int g = 0; g < 9; g++) {
            float4 am = make_float4(0.f, 0.f, 0.f, 0.f), av = am;
            if (!DZ) {
                am = *reinterpret_cast<const float4 *>(a0 + 4 * g);
                av = *reinterpret_cast<const float4 *>(a1 + 4 * g);
            }
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int s = 4 * g + e, pair = s / 9, t = s - pair * 9, ky = t / 3, kx = t - ky * 3;
                const int off = pair * STEP_CH * G::CS +
                                (DZ ? (2 - ky) * G::RS + (2 - kx) : ky * G::RS + kx);
                const float2 y = *reinterpret_cast<const float2 *>(bp + 2 * off);
                const float w = DZ ? a0[pair * 1152 + t] : comp4(am, e), y0 = y.x, y1 = y.y;
                if (!DZ) {
                    // mean: mu_w mu_a; variance: var_w (var_a + mu_a^2) + mu_w^2 var_a
                    acc0[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(w, y0, acc0[0][0], 0, 0, 0);
                    acc1[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(comp4(av, e), y0 * y0 + y1,
                                                                      acc1[0][0], 0, 0, 0);
                    acc1[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(w * w, y1, acc1[0][0], 0, 0, 0);
                } else {
                    // mean: mu_w delta_mu; variance: mu_w^2 delta_var
                    acc0[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(w, y0, acc0[0][0], 0, 0, 0);
                    acc1[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(w * w, y1, acc1[0][0], 0, 0, 0);
                }
            }
        }
        __syncthreads();
        if (more) {
            commit();
            __syncthreads();
        }
    }
    tile_epilogue<P, 64, 128, 2, 4>(p, acc0, acc1, m0, n0, split);
}

// LDS floats a workgroup of conv_stencil_kernel<DZ, WIDTH> needs (stencil or table-driven loop).
template <bool DZ, int WIDTH>
constexpr int stencil_lds_floats() {
    using G = StencilGeom<WIDTH>;
    using P = typename std::conditional<DZ, ConvDzProblem, ConvFwdProblem<true>>::type;
    constexpr int XF = TileGeom<P::XK, 64>::floats, YF = TileGeom<P::YK, 128>::floats;
    constexpr int GENERIC = P::NX * XF + P::NY * YF;
    constexpr int STENCIL = (DZ ? 1 : 2) * 64 * G::AS + 2 * G::PATCH;
    return GENERIC > STENCIL ? GENERIC : STENCIL;
}

// One 64 x 128 tile by a workgroup of 8 waves: verified stencil -> stencil_body,
// anything else -> the table-driven loop of the generic tile kernel.
template <bool DZ, int WIDTH>
__device__ __forceinline__ void conv_stencil_block(const ConvParams &p, float *lds, int *lds_extra,
                                                   int tile, int split) {
    using P = typename std::conditional<DZ, ConvDzProblem, ConvFwdProblem<true>>::type;
    constexpr int XF = TileGeom<P::XK, 64>::floats, YF = TileGeom<P::YK, 128>::floats;
    const int tiles_n = (p.N + 127) / 128;
    const int m0 = (tile / tiles_n) * 64, n0 = (tile % tiles_n) * 128;
    const int r_begin = split * p.r_per_split;
    const int r_end = min(p.R, r_begin + p.r_per_split);

    if (stencil_tables_ok<DZ, WIDTH>(p, n0, threadIdx.x, 512, lds_extra)) {
        stencil_body<DZ, WIDTH>(p, lds, m0, n0, split, r_begin, r_end);
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

template <bool DZ, int WIDTH>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4)))
void conv_stencil_kernel(ConvParams p) {
    __shared__ __attribute__((aligned(16))) float lds[stencil_lds_floats<DZ, WIDTH>()];
    extern __shared__ __attribute__((aligned(16))) int lds_extra[];
    conv_stencil_block<DZ, WIDTH>(p, lds, lds_extra, blockIdx.x, blockIdx.y);
}

// Map width for which the stencil kernel exists, 0 otherwise (pixels = width^2).
inline int stencil_width(int pixels) {
    for (int w : {4, 8, 16, 32})
        if (w * w == pixels) return w;
    return 0;
}

template <bool DZ>
hipError_t launch_conv_stencil(int width, const ConvParams &p, hipStream_t stream) {
    using P = typename std::conditional<DZ, ConvDzProblem, ConvFwdProblem<true>>::type;
    const dim3 grid(((p.M + 63) / 64) * ((p.N + 127) / 128), p.splits);
    const size_t extra = P::extra_lds_bytes(p, 64, 128);
    if (extra > kTileExtraLdsMax) return hipErrorInvalidValue;
#define TAGI_LAUNCH_STENCIL(WD)                                                                  \
    case WD: {                                                                                   \
        static PerDeviceOnce once;                                                               \
        hipError_t e = allow_dynamic_lds(                                                        \
            once, reinterpret_cast<const void *>(conv_stencil_kernel<DZ, WD>),                   \
            (int)kTileExtraLdsMax);                                                              \
        if (e != hipSuccess) return e;                                                           \
        hipLaunchKernelGGL((conv_stencil_kernel<DZ, WD>), grid, dim3(512), extra, stream, p);    \
        return hipGetLastError();                                                                \
    }
    switch (width) {
        TAGI_LAUNCH_STENCIL(4)
        TAGI_LAUNCH_STENCIL(8)
        TAGI_LAUNCH_STENCIL(16)
        TAGI_LAUNCH_STENCIL(32)
    }
#undef TAGI_LAUNCH_STENCIL
    return hipErrorInvalidValue;
}

// ---- weight backward on the same stencil -------------------------------------------
//   D[fo][(c,t)] = sum over (b, pixel) of delta[b][fo][pixel] * a[b][c][pixel + tap t]
// Rows are output channels, the 64 columns of a tile are (channel, tap) pairs of
// exactly eight channels (fi is a multiple of 64), the reduction runs over pixels,
// 64 at a time = 64/W whole image rows. Per k-tile the workgroup stages the rows
// of its eight channels once (zero halo as above; halo ROWS now change from tile
// to tile, so every cell is rewritten, with zero where the row leaves the image);
// a lane's column fixes its (channel, tap) and with it one LDS base address, and
// the pixel of each reduction step is an immediate offset.
template <int WIDTH>
struct StencilDwGeom {
    static constexpr int W = WIDTH, H = WIDTH;
    static constexpr int KP = 64;                   // pixels per k-tile
    static constexpr int KC = 8;                    // channels per column tile
    static constexpr int NR = KP / W;               // image rows per k-tile
    static constexpr int RPI = NR < H ? NR : H;
    static constexpr int SEGS = NR / RPI;
    static constexpr int XO = 4, RS = W + 4;
    static constexpr int SEG = (RPI + 2) * RS + (W == 4 ? 4 : 0);
    static constexpr int CS = SEGS * SEG + 4;
    static constexpr int PATCH = KC * CS;
    static constexpr int UNITS = KC * SEGS * (RPI + 2) * (W / 4);
    static constexpr int AS = KP + 4;               // innovation tile [64 rows][64 pixels + 4]
    static constexpr int LOG_PIX = WIDTH == 4 ? 4 : WIDTH == 8 ? 6 : WIDTH == 16 ? 8 : 10;
    static_assert(UNITS <= 512 && KP % W == 0 && NR % RPI == 0 && H % RPI == 0, "tile geometry");
    // LDS offset of pixel k (0..63) of the k-tile relative to its first pixel
    static constexpr int pixel_offset(int k) {
        return ((k / W) / RPI) * SEG + ((k / W) % RPI) * RS + k % W;
    }
};

template <int WIDTH>
__device__ __forceinline__ void stencil_dw_body(const ConvParams &p, float *lds, int m0, int n0,
                                                int split, int r_begin, int r_end) {
    using G = StencilDwGeom<WIDTH>;
    constexpr int W = G::W, H = G::H, NT = 512, PIX = W * H, SLOTS = 64 * G::KP / 4 / NT;  // 2
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // eight waves: 2 x 2 sub-tiles of 32 x 32, each held by two waves that take
    // the first / second 32 pixels of every k-tile and add up at the end
    const int kgroup = wave >> 2;
    const int wrow = ((wave & 3) / 2) * 32, wcol = (wave & 1) * 32, half = lane >> 5;
    float *lds_a = lds;                        // [2][64][AS]
    float *lds_p = lds + 2 * 64 * G::AS;       // [PATCH]
    const int c_lo = n0 / 9;                   // first channel of the column tile

    for (int i = tid; i < G::PATCH; i += NT) lds_p[i] = 0.f;

    // patch unit: channel pc, segment, patch row pr, column 4*x4. Rows are counted
    // over the whole batch (image b, row y <-> b*H + y); `grow` is the first row of
    // the unit's segment in the current k-tile.
    int u = tid < G::UNITS ? tid : 0;
    const int x4 = u % (W / 4);
    u /= (W / 4);
    const int pr = u % (G::RPI + 2);
    u /= (G::RPI + 2);
    const int seg = u % G::SEGS, pc = u / G::SEGS;
    const bool has_unit = tid < G::UNITS;
    int grow = r_begin / W + seg * G::RPI;
    const int pdst = pc * G::CS + seg * G::SEG + pr * G::RS + G::XO + 4 * x4;
    const int pchan = (c_lo + pc) * PIX + 4 * x4;

    // innovation pieces: 16 bytes at pixel 4*q of rows tid/16 + 32*i
    const int q = tid % 16, arow = tid / 16;
    int gpix = r_begin + 4 * q;  // pixel counted over the whole batch

    floatx16 acc0[1][1], acc1[1][1];
#pragma unroll
    for (int v = 0; v < 16; v++) {
        acc0[0][0][v] = 0.f;
        acc1[0][0][v] = 0.f;
    }

    static_assert(SLOTS == 2, "two innovation pieces per thread and array");
    float4 ra00, ra01, ra10, ra11, rp;
    bool rp_ok;
    auto fetch = [&]() {
        const int b = gpix >> G::LOG_PIX, o = gpix & (PIX - 1);
        const size_t at = ((size_t)b * p.fo + m0 + arow) * PIX + o;
        ra00 = *reinterpret_cast<const float4 *>(p.d0 + at);
        ra10 = *reinterpret_cast<const float4 *>(p.d1 + at);
        ra01 = *reinterpret_cast<const float4 *>(p.d0 + at + (size_t)32 * PIX);
        ra11 = *reinterpret_cast<const float4 *>(p.d1 + at + (size_t)32 * PIX);
        gpix += G::KP;
        const int img = grow / H, y = grow - img * H + pr - 1;
        rp_ok = has_unit && y >= 0 && y < H;
        rp = *reinterpret_cast<const float4 *>(
            p.a0 + (rp_ok ? (size_t)img * p.fi * PIX + pchan + y * W : 0));
        grow += G::NR;
    };
    auto commit = [&]() {
        float *d0 = lds_a + arow * G::AS + 4 * q, *d1 = d0 + 64 * G::AS;
        *reinterpret_cast<float4 *>(d0) = ra00;
        *reinterpret_cast<float4 *>(d0 + 32 * G::AS) = ra01;
        *reinterpret_cast<float4 *>(d1) = ra10;
        *reinterpret_cast<float4 *>(d1 + 32 * G::AS) = ra11;
        if (has_unit)
            *reinterpret_cast<float4 *>(lds_p + pdst) =
                rp_ok ? rp : make_float4(0.f, 0.f, 0.f, 0.f);
    };

    // operand addresses of this lane: its column is (channel, tap)
    const int n = n0 + wcol + (lane & 31);
    const int ch = n / 9 - c_lo, t = n - (n / 9) * 9, ky = t / 3, kx = t - ky * 3;
    const float *bp = lds_p + ch * G::CS + ky * G::RS + kx + G::XO - 1 +
                      (half ? G::pixel_offset(4) : 0) + (kgroup ? G::pixel_offset(32) : 0);
    const float *a0 = lds_a + (wrow + (lane & 31)) * G::AS + 4 * half + 32 * kgroup;
    const float *a1 = a0 + 64 * G::AS;

    __syncthreads();  // patch zeroed
    if (r_begin < r_end) {
        fetch();
        commit();
    }
    __syncthreads();

    for (int r0 = r_begin; r0 < r_end; r0 += G::KP) {
        const bool more = r0 + G::KP < r_end;
        if (more) fetch();
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
            commit();
            __syncthreads();
        }
    }

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

template <int WIDTH>
constexpr int stencil_dw_lds_floats() {
    using G = StencilDwGeom<WIDTH>;
    using P = ConvDwVecProblem;
    constexpr int XF = TileGeom<P::XK, 64>::floats, YF = TileGeom<P::YK, 64>::floats;
    constexpr int GENERIC = P::NX * XF + P::NY * YF;
    constexpr int STENCIL = 2 * 64 * G::AS + G::PATCH;
    static_assert(2 * 64 * G::AS >= 32 * 256, "the innovation tiles hold the final exchange");
    return GENERIC > STENCIL ? GENERIC : STENCIL;
}

// One 64 x 64 tile of one reduction slice by a workgroup of 8 waves; (bx, by) of a
// (gx, gy) = (tiles, slices) grid. `regular_flag`: one int of LDS.
template <int WIDTH>
__device__ __forceinline__ void conv_stencil_dw_block(const ConvParams &p, float *lds,
                                                      int *regular_flag, int bx, int by, int gx,
                                                      int gy) {
    using P = ConvDwVecProblem;
    constexpr int XF = TileGeom<P::XK, 64>::floats, YF = TileGeom<P::YK, 64>::floats;
    const int tiles_n = (p.N + 63) / 64;
    int tile = bx, split = by;
    if (gy % 8 == 0) {
        // all column tiles of one reduction slice on one XCD (see mfma_tile_kernel)
        const int id = by * gx + bx;
        const int qq = id >> 3;
        tile = qq % gx;
        split = (qq / gx) * 8 + (id & 7);
    }
    const int m0 = (tile / tiles_n) * 64, n0 = (tile % tiles_n) * 64;
    const int r_begin = split * p.r_per_split;
    const int r_end = min(p.R, r_begin + p.r_per_split);

    // the pixels of this slice, per image position: all of Fmwa_2 once the slice
    // is as long as a map. Entries are requested six at a time before any is
    // looked at (one memory latency per batch, not per entry).
    if (threadIdx.x == 0) *regular_flag = 1;
    __syncthreads();
    {
        const int total = min(max(r_end - r_begin, 0), p.woho) * 9;
        bool ok = true;
        for (int base = threadIdx.x; base < total; base += 6 * 512) {
            int got[6], want[6];
#pragma unroll
            for (int i = 0; i < 6; i++) {
                const int e = base + i * 512, c = e / 9, t = e - c * 9;
                const bool live = e < total;
                const int o = live ? (r_begin + c) & (WIDTH * WIDTH - 1) : 0;
                got[i] = p.idx[live ? o * 9 + t : 0];
                want[i] = live ? stencil_fmwa<WIDTH>(o, t) : got[i];
            }
#pragma unroll
            for (int i = 0; i < 6; i++) ok = ok && got[i] == want[i];
        }
        if (!ok) *regular_flag = 0;
    }
    __syncthreads();
    if (__builtin_amdgcn_readfirstlane(*regular_flag)) {
        stencil_dw_body<WIDTH>(p, lds, m0, n0, split, r_begin, r_end);
        return;
    }
    // table-driven loop: written for four waves; the other four leave (a barrier
    // counts the waves that are still running)
    if (threadIdx.x >= 256) return;
    typename P::Ctx ctx;
    P::prologue(p, ctx, nullptr, threadIdx.x, 256, m0, n0, 64, 64, r_begin, r_end);
    mfma_tile_body<P, 64, 64, 2, 2, 0>(p, ctx, reinterpret_cast<float (*)[XF]>(lds),
                                       reinterpret_cast<float (*)[YF]>(lds + P::NX * XF), m0, n0,
                                       split, r_begin, r_end);
}

template <int WIDTH>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4)))
void conv_stencil_dw_kernel(ConvParams p) {
    __shared__ __attribute__((aligned(16))) float lds[stencil_dw_lds_floats<WIDTH>()];
    __shared__ int regular_flag;
    conv_stencil_dw_block<WIDTH>(p, lds, &regular_flag, blockIdx.x, blockIdx.y, gridDim.x, gridDim.y);
}

// State backward and weight backward of one layer in ONE launch: the first `blocks_z`
// workgroups are the state backward's (tile, slice) grid, the rest the weight backward's.
// The two contractions read the same innovations and are independent; as one grid the
// workgroups of the second start where those of the first leave CUs free, so neither
// kernel's ramp-up (table check, first loads) nor its tail runs on an otherwise idle chip.
template <int WIDTH>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4)))
void conv_stencil_bwd_pair_kernel(ConvParams pz, ConvParams pw, int blocks_z, int tiles_z,
                                  int tiles_w, int splits_w) {
    constexpr int FZ = stencil_lds_floats<true, WIDTH>(), FW = stencil_dw_lds_floats<WIDTH>();
    __shared__ __attribute__((aligned(16))) float lds[FZ > FW ? FZ : FW];
    __shared__ int regular_flag;
    extern __shared__ __attribute__((aligned(16))) int lds_extra[];
    const int id = blockIdx.x;
    if (id < blocks_z) {
        conv_stencil_block<true, WIDTH>(pz, lds, lds_extra, id % tiles_z, id / tiles_z);
    } else {
        const int j = id - blocks_z;
        conv_stencil_dw_block<WIDTH>(pw, lds, &regular_flag, j % tiles_w, j / tiles_w, tiles_w, splits_w);
    }
}

inline hipError_t launch_conv_stencil_bwd_pair(int width, const ConvParams &pz, const ConvParams &pw,
                                               hipStream_t stream) {
    using P = ConvDzProblem;
    const int tiles_z = ((pz.M + 63) / 64) * ((pz.N + 127) / 128);
    const int tiles_w = ((pw.M + 63) / 64) * ((pw.N + 63) / 64);
    const int blocks_z = tiles_z * pz.splits;
    const dim3 grid(blocks_z + tiles_w * pw.splits);
    const size_t extra = P::extra_lds_bytes(pz, 64, 128);
    if (extra > kTileExtraLdsMax) return hipErrorInvalidValue;
#define TAGI_LAUNCH_PAIR(WD)                                                                       \
    case WD: {                                                                                     \
        static PerDeviceOnce once;                                                                 \
        hipError_t e = allow_dynamic_lds(                                                          \
            once, reinterpret_cast<const void *>(conv_stencil_bwd_pair_kernel<WD>),                \
            (int)kTileExtraLdsMax);                                                                \
        if (e != hipSuccess) return e;                                                             \
        hipLaunchKernelGGL((conv_stencil_bwd_pair_kernel<WD>), grid, dim3(512), extra, stream, pz, \
                           pw, blocks_z, tiles_z, tiles_w, pw.splits);                             \
        return hipGetLastError();                                                                  \
    }
    switch (width) {
        TAGI_LAUNCH_PAIR(4)
        TAGI_LAUNCH_PAIR(8)
        TAGI_LAUNCH_PAIR(16)
        TAGI_LAUNCH_PAIR(32)
    }
#undef TAGI_LAUNCH_PAIR
    return hipErrorInvalidValue;
}

inline hipError_t launch_conv_stencil_dw(int width, const ConvParams &p, hipStream_t stream) {
    const dim3 grid(((p.M + 63) / 64) * ((p.N + 63) / 64), p.splits);
    switch (width) {
        case 4: hipLaunchKernelGGL(conv_stencil_dw_kernel<4>, grid, dim3(512), 0, stream, p); break;
        case 8: hipLaunchKernelGGL(conv_stencil_dw_kernel<8>, grid, dim3(512), 0, stream, p); break;
        case 16: hipLaunchKernelGGL(conv_stencil_dw_kernel<16>, grid, dim3(512), 0, stream, p); break;
        case 32: hipLaunchKernelGGL(conv_stencil_dw_kernel<32>, grid, dim3(512), 0, stream, p); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace
}  // namespace tagi

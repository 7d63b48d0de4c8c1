// Workgroup-tiled fp32 MFMA core shared by the Linear and Conv2d contractions,
// gfx950 (v_mfma_f32_32x32x2_f32, 64-lane waves).
//
// A workgroup owns a BM x BN tile of an output PAIR (accumulator 0: the
// mean-like sum, accumulator 1: the variance-like sum), walks its slice of the
// reduction in k-tiles of KT elements staged through LDS (global -> registers ->
// LDS, the next k-tile's global loads in flight while the current one is
// multiplied), and each of its WM x WN waves multiplies (BM/WM) x (BN/WN)
// sub-tiles.
//
// A `Problem` type supplies the operands and the epilogue:
//   Params                      kernel argument (must hold M, N, R, splits,
//                               r_per_split, ws0, ws1)
//   XK / YK                     is the row-side / column-side operand staged with
//                               its reduction index contiguous ([row][KT+4], read
//                               back with one 16-byte LDS load), or with the row
//                               index contiguous ([k][rows+4], read back with four
//                               4-byte loads)?  Either way lane l of a 32-row
//                               fragment holds reduction elements kk+4*(l/32)+t,
//                               t = 0..3, and the t-th of four MFMAs consumes
//                               component t, so both sides agree on k.
//   NX / NY                     number of arrays on each side (1 or 2)
//   FLAVOR                      how the MFMA operands are formed, see Flavor
//   SPLIT_PER_XCD               map all tiles of a reduction slice to one XCD
//   Ctx                         per-thread state that lives across the k-tiles
//                               (TileNoCtx when a problem needs none)
//   extra_lds_bytes(p, BM, BN)  host: dynamic LDS the prologue wants (index tables)
//   prologue(p, ctx, extra, tid, nthreads, m0, n0, BM, BN, r_begin, r_end)
//                               runs once before the first load; a barrier follows
//   min_waves_per_simd(BM, BN, waves)
//                               occupancy the register allocation must allow (0: none)
//   EPI_PREFETCH, epi_load(p, row, col), store_with(p, row, col, a0, a1, e)
//                               optional: the epilogue's per-element operand, loaded
//                               for a whole fragment before its stores
//   place_tile(p, tile, split, tiles)
//                               which tile the workgroup (tile, split) of the grid takes
//                               (a permutation of the tiles for every split)
//   adjust_range(p, ctx, r_begin, r_end)
//                               after the prologue: a problem whose reduction is shorter
//                               for this tile than for others re-states its slice
//   VARIANTS, variant(ctx)      number of loader variants (1 or 2) and, after the
//                               prologue, which one this workgroup uses (uniform)
//   load_x(p, ctx, V, arr, i, m0, row, r, r_end)
//                               four elements of row-side array `arr` for the
//                               thread's i-th slot: row m0+row, reduction r..r+3
//                               when XK; rows m0+row..+3 at reduction r otherwise;
//                               zero outside the problem. Slots are visited for
//                               consecutive k-tiles in increasing order, so Ctx may
//                               carry what the next tile's loads need.
//   load_y(p, ctx, V, arr, i, n0, row, r, r_end)   the same for the column side
//   next_tile(p, ctx)           runs after all loads of a k-tile were issued
//   fix_x(ctx, i, v) / fix_y    applied to slot i's loaded values when they are
//                               written to LDS, i.e. after the MFMAs of the previous
//                               k-tile: masking done here instead of right after the
//                               load keeps the loads in flight during the MFMAs
//   store(p, m, n, acc0, acc1)  final epilogue of one output element
#pragma once
#include <hip/hip_runtime.h>

namespace tagi {

typedef float floatx16 __attribute__((ext_vector_type(16)));

// Which products feed the two accumulators (x = row side, y = column side):
enum Flavor {
    // acc0 += x0*y0 ; acc1 += (x1 + x0^2)*y1 + x1*y0^2   rows: (mu_a,var_a), cols: (mu_w,var_w)
    FLAVOR_FWD_ACT_ROWS = 0,
    // acc0 += x0*y0 ; acc1 += x1*(y1 + y0^2) + x0^2*y1   rows: (mu_w,var_w), cols: (mu_a,var_a)
    FLAVOR_FWD_W_ROWS = 1,
    // acc0 += x0*y0 ; acc1 += x1*y0^2                    rows: (delta_mu,delta_var), cols: (v)
    FLAVOR_DELTA_ROWS = 2,
    // acc0 += x0*y0 ; acc1 += x0^2*y1                    rows: (w), cols: (delta_mu,delta_var)
    FLAVOR_DELTA_COLS = 3,
};

constexpr int KT = 32;  // reduction elements per LDS stage

struct TileNoCtx {};

// A [row][k] stage of sixteen reduction elements is four 16-byte chunks per row. Without
// padding, chunk c of row r sits at position c ^ ((r / 4) % 4): sixteen lanes that read
// one chunk of sixteen consecutive rows, and sixteen lanes that write the four chunks of
// four rows, then both touch each of the 64 banks once.
template <bool KC, int KTILE>
constexpr bool tile_swizzled() { return KC && KTILE == 16; }
template <bool KC, int ROWS, int KTILE = KT>
struct TileGeom {
    static constexpr int stride = KC ? (tile_swizzled<KC, KTILE>() ? KTILE : KTILE + 4) : ROWS + 4;
    static constexpr int floats = KC ? ROWS * stride : KTILE * stride;
};
// column of reduction element k (a multiple of 4) of `row` in a [row][k] stage
template <bool KC, int KTILE>
__device__ __forceinline__ int kc_col(int row, int k) {
    return tile_swizzled<KC, KTILE>() ? (((k >> 2) ^ ((row >> 2) & 3)) << 2) : k;
}

__device__ __forceinline__ float comp4(const float4 &v, int t) {
    return t == 0 ? v.x : t == 1 ? v.y : t == 2 ? v.z : v.w;
}
__device__ __forceinline__ float4 sq4(const float4 &a) {
    return make_float4(a.x * a.x, a.y * a.y, a.z * a.z, a.w * a.w);
}
__device__ __forceinline__ float4 add_sq4(const float4 &v, const float4 &m) {
    return make_float4(v.x + m.x * m.x, v.y + m.y * m.y, v.z + m.z * m.z, v.w + m.w * m.w);
}

// Position of the f-th float4 of a staged tile: (row, k) of its first element.
template <bool KC, int ROWS, int KTILE = KT>
__device__ __forceinline__ void tile_pos(int f, int &row, int &k) {
    if (KC) {
        row = f / (KTILE / 4);
        k = (f % (KTILE / 4)) * 4;
    } else {
        k = f / (ROWS / 4);
        row = (f % (ROWS / 4)) * 4;
    }
}

template <bool KC, int ROWS, int KTILE = KT>
__device__ __forceinline__ float4 read_frag(const float *lds, int row, int kk, int lane) {
    constexpr int S = TileGeom<KC, ROWS, KTILE>::stride;
    const int k = kk + 4 * (lane >> 5);
    if (KC) {
        return *reinterpret_cast<const float4 *>(lds + (row + (lane & 31)) * S +
                                                 kc_col<KC, KTILE>(row + (lane & 31), k));
    } else {
        const float *q = lds + k * S + row + (lane & 31);
        return make_float4(q[0], q[S], q[2 * S], q[3 * S]);
    }
}

// Waves per SIMD the register allocation has to leave room for: what the
// workgroup size implies, or more where the problem asks for it (two 8-wave
// workgroups on a CU need four, i.e. at most 128 registers per lane; a kernel that
// would land just above such a step loses a whole workgroup per CU).
template <class P>
constexpr int tile_min_waves(int bm, int bn, int waves) {
    return P::min_waves_per_simd(bm, bn, waves) > (waves + 3) / 4
               ? P::min_waves_per_simd(bm, bn, waves)
               : (waves + 3) / 4;
}

// Writes a workgroup's accumulators: partial sums of a reduction slice go to the
// workspace, a complete sum to the problem's epilogue. Accumulator register v of
// lane l is D[8*(v/4) + 4*(l/32) + v%4][l%32]: lanes run along the output columns.
template <class P, int BM, int BN, int WM, int WN>
__device__ __forceinline__ void tile_epilogue(const typename P::Params &p,
                                              floatx16 (&acc0)[BM / WM / 32][BN / WN / 32],
                                              floatx16 (&acc1)[BM / WM / 32][BN / WN / 32],
                                              int m0, int n0, int split) {
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wrow = (wave / WN) * (TM * 32), wcol = (wave % WN) * (TN * 32);
    const bool partial = p.splits > 1;
    // a tile inside the matrix needs no per-element bounds checks
    const bool inside = m0 + BM <= p.M && n0 + BN <= p.N;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int col = n0 + wcol + j * 32 + (lane & 31);
            const int row0 = m0 + wrow + i * 32 + 4 * (lane >> 5);  // + 8*(v/4) + v%4
            if (inside) {
                if (partial) {
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        const int row = row0 + 8 * (v / 4) + (v % 4);
                        const size_t at = ((size_t)split * p.M + row) * p.N + col;
                        p.ws0[at] = acc0[i][j][v];
                        p.ws1[at] = acc1[i][j][v];
                    }
                    continue;
                }
                if constexpr (P::EPI_PREFETCH) {
                    // the epilogue operands of the fragment are all requested before the
                    // stores that use them: a load that follows a store waits for it
                    constexpr int EPI_BATCH = 16;
#pragma unroll
                    for (int h = 0; h < 16; h += EPI_BATCH) {
                        float e[EPI_BATCH];
#pragma unroll
                        for (int v = h; v < h + EPI_BATCH; v++)
                            e[v - h] = P::epi_load(p, row0 + 8 * (v / 4) + (v % 4), col);
#pragma unroll
                        for (int v = h; v < h + EPI_BATCH; v++)
                            P::store_with(p, row0 + 8 * (v / 4) + (v % 4), col, acc0[i][j][v],
                                          acc1[i][j][v], e[v - h]);
                    }
                    continue;
                }
            }
            if (col >= p.N) continue;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int row = row0 + 8 * (v / 4) + (v % 4);
                if (row >= p.M) continue;
                if (partial) {
                    const size_t at = ((size_t)split * p.M + row) * p.N + col;
                    p.ws0[at] = acc0[i][j][v];
                    p.ws1[at] = acc1[i][j][v];
                } else {
                    P::store(p, row, col, acc0[i][j][v], acc1[i][j][v]);
                }
            }
        }
}

// Everything a workgroup does after its prologue, instantiated once per loader
// variant V (a problem whose prologue chooses between two ways of loading gets two
// copies of the loop instead of a branch at every load).
template <class P, int BM, int BN, int WM, int WN, int V>
__device__ __forceinline__ void mfma_tile_body(const typename P::Params &p, typename P::Ctx &ctx,
                                               float (*lds_x)[TileGeom<P::XK, BM>::floats],
                                               float (*lds_y)[TileGeom<P::YK, BN>::floats],
                                               int m0, int n0, int split, int r_begin,
                                               int r_end) {
    constexpr bool XK = P::XK, YK = P::YK;
    constexpr int NX = P::NX, NY = P::NY, FL = P::FLAVOR;
    constexpr int NT = WM * WN * 64;
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int XS = TileGeom<XK, BM>::stride, YS = TileGeom<YK, BN>::stride;
    constexpr int LX = BM * KT / 4 / NT, LY = BN * KT / 4 / NT;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wrow = (wave / WN) * (TM * 32), wcol = (wave % WN) * (TN * 32);

    floatx16 acc0[TM][TN], acc1[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                acc0[i][j][v] = 0.f;
                acc1[i][j][v] = 0.f;
            }

    float4 rx[NX][LX], ry[NY][LY];

    auto fetch = [&](int r0) {
#pragma unroll
        for (int a = 0; a < NX; a++)
#pragma unroll
            for (int i = 0; i < LX; i++) {
                int row, k;
                tile_pos<XK, BM>(tid + i * NT, row, k);
                rx[a][i] = P::load_x(p, ctx, V, a, i, m0, row, r0 + k, r_end);
            }
#pragma unroll
        for (int a = 0; a < NY; a++)
#pragma unroll
            for (int i = 0; i < LY; i++) {
                int row, k;
                tile_pos<YK, BN>(tid + i * NT, row, k);
                ry[a][i] = P::load_y(p, ctx, V, a, i, n0, row, r0 + k, r_end);
            }
        P::next_tile(p, ctx);
    };
    auto commit = [&]() {
#pragma unroll
        for (int a = 0; a < NX; a++)
#pragma unroll
            for (int i = 0; i < LX; i++) {
                int row, k;
                tile_pos<XK, BM>(tid + i * NT, row, k);
                *reinterpret_cast<float4 *>(&lds_x[a][XK ? row * XS + k : k * XS + row]) =
                    P::fix_x(ctx, i, rx[a][i]);
            }
#pragma unroll
        for (int a = 0; a < NY; a++)
#pragma unroll
            for (int i = 0; i < LY; i++) {
                int row, k;
                tile_pos<YK, BN>(tid + i * NT, row, k);
                *reinterpret_cast<float4 *>(&lds_y[a][YK ? row * YS + k : k * YS + row]) =
                    P::fix_y(ctx, i, ry[a][i]);
            }
    };

    if (r_begin < r_end) {
        fetch(r_begin);
        commit();
    }
    __syncthreads();

    for (int r0 = r_begin; r0 < r_end; r0 += KT) {
        const bool more = r0 + KT < r_end;
        if (more) fetch(r0 + KT);

#pragma unroll
        for (int kk = 0; kk < KT; kk += 8) {
            // MFMA operand fragments: mean (A0,B0), variance (A1,B1) [+ (A2,B2)]
            float4 A0[TM], A1[TM], A2[TM], B0[TN], B1[TN], B2[TN];
#pragma unroll
            for (int i = 0; i < TM; i++) {
                const float4 x0 = read_frag<XK, BM>(lds_x[0], wrow + i * 32, kk, lane);
                float4 x1 = x0;
                if (NX == 2) x1 = read_frag<XK, BM>(lds_x[NX - 1], wrow + i * 32, kk, lane);
                A0[i] = x0;
                if (FL == FLAVOR_FWD_ACT_ROWS) {
                    A1[i] = add_sq4(x1, x0);
                    A2[i] = x1;
                } else if (FL == FLAVOR_FWD_W_ROWS) {
                    A1[i] = x1;
                    A2[i] = sq4(x0);
                } else if (FL == FLAVOR_DELTA_ROWS) {
                    A1[i] = x1;
                } else {
                    A1[i] = sq4(x0);
                }
            }
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const float4 y0 = read_frag<YK, BN>(lds_y[0], wcol + j * 32, kk, lane);
                float4 y1 = y0;
                if (NY == 2) y1 = read_frag<YK, BN>(lds_y[NY - 1], wcol + j * 32, kk, lane);
                B0[j] = y0;
                if (FL == FLAVOR_FWD_ACT_ROWS) {
                    B1[j] = y1;
                    B2[j] = sq4(y0);
                } else if (FL == FLAVOR_FWD_W_ROWS) {
                    B1[j] = add_sq4(y1, y0);
                    B2[j] = y1;
                } else if (FL == FLAVOR_DELTA_ROWS) {
                    B1[j] = sq4(y0);
                } else {
                    B1[j] = y1;
                }
            }
#pragma unroll
            for (int t = 0; t < 4; t++)
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++) {
                        acc0[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                            comp4(A0[i], t), comp4(B0[j], t), acc0[i][j], 0, 0, 0);
                        acc1[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                            comp4(A1[i], t), comp4(B1[j], t), acc1[i][j], 0, 0, 0);
                        if (FL == FLAVOR_FWD_ACT_ROWS || FL == FLAVOR_FWD_W_ROWS)
                            acc1[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                                comp4(A2[i], t), comp4(B2[j], t), acc1[i][j], 0, 0, 0);
                    }
        }
        __syncthreads();
        if (more) {
            commit();
            __syncthreads();
        }
    }

    tile_epilogue<P, BM, BN, WM, WN>(p, acc0, acc1, m0, n0, split);
}


// Does the problem ask for the double-buffered loop below? (A problem opts in with
// `static constexpr bool DOUBLE_BUFFER = true`; it must not depend on the slot index
// of its loaders, because slots are dealt to the threads differently there.)
template <class P, class = void>
struct tile_double_buffer { static constexpr bool value = false; };
template <class P>
struct tile_double_buffer<P, decltype((void)P::DOUBLE_BUFFER)> {
    static constexpr bool value = P::DOUBLE_BUFFER;
};

constexpr int KT_DB = 16;  // reduction elements per stage of the double-buffered loop

// The fragments of one 8-element step of a stage, as read from LDS, and the MFMAs on them.
template <class P, int BM, int BN, int WM, int WN>
struct TileFrags {
    float4 x0[BM / WM / 32], x1[BM / WM / 32], y0[BN / WN / 32], y1[BN / WN / 32];
};
template <class P, int BM, int BN, int WM, int WN, int KTILE>
__device__ __forceinline__ void tile_read_frags(
    const float (*lx)[TileGeom<P::XK, BM, KTILE>::floats],
    const float (*ly)[TileGeom<P::YK, BN, KTILE>::floats], int kk, int wrow, int wcol, int lane,
    TileFrags<P, BM, BN, WM, WN> &f) {
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
#pragma unroll
    for (int i = 0; i < TM; i++) {
        f.x0[i] = read_frag<P::XK, BM, KTILE>(lx[0], wrow + i * 32, kk, lane);
        f.x1[i] = f.x0[i];
        if (P::NX == 2) f.x1[i] = read_frag<P::XK, BM, KTILE>(lx[P::NX - 1], wrow + i * 32, kk, lane);
    }
#pragma unroll
    for (int j = 0; j < TN; j++) {
        f.y0[j] = read_frag<P::YK, BN, KTILE>(ly[0], wcol + j * 32, kk, lane);
        f.y1[j] = f.y0[j];
        if (P::NY == 2) f.y1[j] = read_frag<P::YK, BN, KTILE>(ly[P::NY - 1], wcol + j * 32, kk, lane);
    }
}
template <class P, int BM, int BN, int WM, int WN>
__device__ __forceinline__ void tile_mfma_frags(const TileFrags<P, BM, BN, WM, WN> &f,
                                                floatx16 (&acc0)[BM / WM / 32][BN / WN / 32],
                                                floatx16 (&acc1)[BM / WM / 32][BN / WN / 32]) {
    constexpr int FL = P::FLAVOR;
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    float4 A0[TM], A1[TM], A2[TM], B0[TN], B1[TN], B2[TN];
#pragma unroll
    for (int i = 0; i < TM; i++) {
        A0[i] = f.x0[i];
        if (FL == FLAVOR_FWD_ACT_ROWS) {
            A1[i] = add_sq4(f.x1[i], f.x0[i]);
            A2[i] = f.x1[i];
        } else if (FL == FLAVOR_FWD_W_ROWS) {
            A1[i] = f.x1[i];
            A2[i] = sq4(f.x0[i]);
        } else if (FL == FLAVOR_DELTA_ROWS) {
            A1[i] = f.x1[i];
        } else {
            A1[i] = sq4(f.x0[i]);
        }
    }
#pragma unroll
    for (int j = 0; j < TN; j++) {
        B0[j] = f.y0[j];
        if (FL == FLAVOR_FWD_ACT_ROWS) {
            B1[j] = f.y1[j];
            B2[j] = sq4(f.y0[j]);
        } else if (FL == FLAVOR_FWD_W_ROWS) {
            B1[j] = add_sq4(f.y1[j], f.y0[j]);
            B2[j] = f.y1[j];
        } else if (FL == FLAVOR_DELTA_ROWS) {
            B1[j] = sq4(f.y0[j]);
        } else {
            B1[j] = f.y1[j];
        }
    }
#pragma unroll
    for (int t = 0; t < 4; t++)
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) {
                acc0[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(comp4(A0[i], t), comp4(B0[j], t),
                                                                  acc0[i][j], 0, 0, 0);
                acc1[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(comp4(A1[i], t), comp4(B1[j], t),
                                                                  acc1[i][j], 0, 0, 0);
                if (FL == FLAVOR_FWD_ACT_ROWS || FL == FLAVOR_FWD_W_ROWS)
                    acc1[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                        comp4(A2[i], t), comp4(B2[j], t), acc1[i][j], 0, 0, 0);
            }
}

// The k-loop with two LDS stages of KT_DB reduction elements each (the same LDS
// footprint as one stage of KT): while a stage is multiplied, the registers that hold
// the next k-tile are written to the other stage, so a k-tile costs one barrier and no
// wave waits between its multiplies and its LDS writes for the others to finish
// reading. The float4 slots of a stage are dealt to the threads across the arrays of a
// side (slot g of NX*BM*KT_DB/4: array g / (BM*KT_DB/4)).
// Measured on Linear 4096^2, batch 256, forward (210 us, of which 24 us do not depend
// on the reduction length: launch, first tile, partial sums and their fold): the loop
// with its MFMAs alone runs at the matrix peak; LDS reads cost it 2 %, the barrier 5 %,
// staging the next tile 5 %.
template <class P, int BM, int BN, int WM, int WN>
__device__ __forceinline__ void mfma_tile_body_db(
    const typename P::Params &p, typename P::Ctx &ctx,
    float (*lds_x)[P::NX][TileGeom<P::XK, BM, KT_DB>::floats],
    float (*lds_y)[P::NY][TileGeom<P::YK, BN, KT_DB>::floats], int m0, int n0, int split,
    int r_begin, int r_end) {
    constexpr bool XK = P::XK, YK = P::YK;
    constexpr int NX = P::NX, NY = P::NY;
    constexpr int NT = WM * WN * 64;
    constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
    constexpr int XS = TileGeom<XK, BM, KT_DB>::stride, YS = TileGeom<YK, BN, KT_DB>::stride;
    constexpr int FX = BM * KT_DB / 4, FY = BN * KT_DB / 4;  // float4 per array and stage
    static_assert((NX * FX) % NT == 0 && (NY * FY) % NT == 0, "slots must divide evenly");
    constexpr int SX = NX * FX / NT, SY = NY * FY / NT;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wrow = (wave / WN) * (TM * 32), wcol = (wave % WN) * (TN * 32);

    floatx16 acc0[TM][TN], acc1[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                acc0[i][j][v] = 0.f;
                acc1[i][j][v] = 0.f;
            }

    float4 rx[SX], ry[SY];
    auto fetch = [&](int r0) {
#pragma unroll
        for (int s = 0; s < SX; s++) {
            const int g = tid + s * NT;
            int row, k;
            tile_pos<XK, BM, KT_DB>(g % FX, row, k);
            rx[s] = P::load_x(p, ctx, 0, g / FX, s, m0, row, r0 + k, r_end);
        }
#pragma unroll
        for (int s = 0; s < SY; s++) {
            const int g = tid + s * NT;
            int row, k;
            tile_pos<YK, BN, KT_DB>(g % FY, row, k);
            ry[s] = P::load_y(p, ctx, 0, g / FY, s, n0, row, r0 + k, r_end);
        }
    };
    auto commit = [&](int stage) {
#pragma unroll
        for (int s = 0; s < SX; s++) {
            const int g = tid + s * NT;
            int row, k;
            tile_pos<XK, BM, KT_DB>(g % FX, row, k);
            *reinterpret_cast<float4 *>(
                &lds_x[stage][g / FX][XK ? row * XS + kc_col<XK, KT_DB>(row, k) : k * XS + row]) = rx[s];
        }
#pragma unroll
        for (int s = 0; s < SY; s++) {
            const int g = tid + s * NT;
            int row, k;
            tile_pos<YK, BN, KT_DB>(g % FY, row, k);
            *reinterpret_cast<float4 *>(
                &lds_y[stage][g / FY][YK ? row * YS + kc_col<YK, KT_DB>(row, k) : k * YS + row]) = ry[s];
        }
    };

    // A stage is two steps of eight reduction elements. The fragments of a step are read
    // from LDS while the MFMAs of the step before run, across the barrier too: tile t+1 is
    // committed at the start of stage t (its buffer was released by the last barrier), so
    // after this stage's barrier its first fragments can be read under the MFMAs of the
    // second step. No wave waits for LDS with nothing to multiply, and a k-tile still
    // costs one barrier.
    static_assert(KT_DB == 16, "two steps per stage");
    TileFrags<P, BM, BN, WM, WN> f0, f1;
    if (r_begin < r_end) {
        fetch(r_begin);
        commit(0);
    }
    __syncthreads();
    if (r_begin + KT_DB < r_end) fetch(r_begin + KT_DB);
    if (r_begin < r_end)
        tile_read_frags<P, BM, BN, WM, WN, KT_DB>(lds_x[0], lds_y[0], 0, wrow, wcol, lane, f0);
    int r0 = r_begin;
    // steady state: both stages of a trip have a next tile to commit and one to fetch, so
    // the body is straight-line code (and its waits count only what they must)
    for (; r0 + 3 * KT_DB < r_end; r0 += 2 * KT_DB) {
#pragma unroll
        for (int stage = 0; stage < 2; stage++) {
            commit(stage ^ 1);
            fetch(r0 + (stage + 2) * KT_DB);
            tile_read_frags<P, BM, BN, WM, WN, KT_DB>(lds_x[stage], lds_y[stage], 8, wrow, wcol, lane,
                                                      f1);
            // (the scheduler would otherwise sink the reads below the MFMAs they are meant
            // to run under)
            __builtin_amdgcn_sched_barrier(0);
            tile_mfma_frags<P, BM, BN, WM, WN>(f0, acc0, acc1);
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();
            tile_read_frags<P, BM, BN, WM, WN, KT_DB>(lds_x[stage ^ 1], lds_y[stage ^ 1], 0, wrow,
                                                      wcol, lane, f0);
            __builtin_amdgcn_sched_barrier(0);
            tile_mfma_frags<P, BM, BN, WM, WN>(f1, acc0, acc1);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // the last tiles
    for (; r0 < r_end; r0 += 2 * KT_DB) {
#pragma unroll
        for (int stage = 0; stage < 2; stage++) {
            const int r = r0 + stage * KT_DB;
            if (r < r_end) {
                const bool more = r + KT_DB < r_end;
                if (more) commit(stage ^ 1);
                if (r + 2 * KT_DB < r_end) fetch(r + 2 * KT_DB);
                tile_read_frags<P, BM, BN, WM, WN, KT_DB>(lds_x[stage], lds_y[stage], 8, wrow, wcol,
                                                          lane, f1);
                __builtin_amdgcn_sched_barrier(0);
                tile_mfma_frags<P, BM, BN, WM, WN>(f0, acc0, acc1);
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();
                if (more)
                    tile_read_frags<P, BM, BN, WM, WN, KT_DB>(lds_x[stage ^ 1], lds_y[stage ^ 1], 0,
                                                              wrow, wcol, lane, f0);
                __builtin_amdgcn_sched_barrier(0);
                tile_mfma_frags<P, BM, BN, WM, WN>(f1, acc0, acc1);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    tile_epilogue<P, BM, BN, WM, WN>(p, acc0, acc1, m0, n0, split);
}


// What the workgroup (bx, by) of a gx x gy grid of (tiles, reduction slices) does.
template <class P, int BM, int BN, int WM, int WN>
__device__ __forceinline__ void tile_workgroup(const typename P::Params &p, int bx, int by, int gx,
                                               int gy) {
    constexpr bool XK = P::XK, YK = P::YK;
    constexpr int NX = P::NX, NY = P::NY;
    constexpr int NT = WM * WN * 64;
    constexpr int XF = TileGeom<XK, BM>::floats, YF = TileGeom<YK, BN>::floats;
    constexpr int LX = BM * KT / 4 / NT, LY = BN * KT / 4 / NT;
    static_assert(LX >= 1 && LY >= 1, "tile too small for the thread count");

    extern __shared__ __attribute__((aligned(16))) int lds_extra[];

    const int tiles_n = (p.N + BN - 1) / BN;
    int tile = bx, split = by;
    if (P::SPLIT_PER_XCD && gy % 8 == 0) {
        // Workgroups are handed to the 8 XCDs round-robin in launch order. Give all
        // tiles of one reduction slice to one XCD, so that the operands they share
        // are fetched into one L2 instead of eight.
        const int id = by * gx + bx;
        const int q = id >> 3;
        tile = q % gx;
        split = (q / gx) * 8 + (id & 7);
    }
    tile = P::place_tile(p, tile, split, gx);
    const int m0 = (tile / tiles_n) * BM, n0 = (tile % tiles_n) * BN;
    const int r_begin = split * p.r_per_split;
    const int r_end = min(p.R, r_begin + p.r_per_split);

    typename P::Ctx ctx;
    P::prologue(p, ctx, lds_extra, threadIdx.x, NT, m0, n0, BM, BN, r_begin, r_end);
    if (P::PROLOGUE_WRITES_LDS) __syncthreads();
    int r_lo = r_begin, r_hi = r_end;
    P::adjust_range(p, ctx, r_lo, r_hi);
    if constexpr (tile_double_buffer<P>::value) {
        __shared__ __attribute__((aligned(16))) float
            dbx[2][NX][TileGeom<XK, BM, KT_DB>::floats], dby[2][NY][TileGeom<YK, BN, KT_DB>::floats];
        mfma_tile_body_db<P, BM, BN, WM, WN>(p, ctx, dbx, dby, m0, n0, split, r_lo, r_hi);
        return;
    }
    __shared__ __attribute__((aligned(16))) float lds_x[NX][XF];
    __shared__ __attribute__((aligned(16))) float lds_y[NY][YF];
    if constexpr (P::VARIANTS > 1) {
        if (P::variant(ctx)) {
            mfma_tile_body<P, BM, BN, WM, WN, 1>(p, ctx, lds_x, lds_y, m0, n0, split, r_lo, r_hi);
            return;
        }
    }
    mfma_tile_body<P, BM, BN, WM, WN, 0>(p, ctx, lds_x, lds_y, m0, n0, split, r_lo, r_hi);
}

template <class P, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM *WN * 64)
__attribute__((amdgpu_waves_per_eu(tile_min_waves<P>(BM, BN, WM * WN))))
void mfma_tile_kernel(typename P::Params p) {
    tile_workgroup<P, BM, BN, WM, WN>(p, blockIdx.x, blockIdx.y, gridDim.x, gridDim.y);
}

// Folds the partial sums of a sliced reduction (ws0/ws1 [split][M][N]) in slice
// order and hands every output element to the problem's epilogue.
template <class P>
__global__ __launch_bounds__(256) void reduce_store_kernel(typename P::Params p) {
    const size_t total = (size_t)p.M * p.N;
    const size_t at = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (at >= total) return;
    float s0 = 0.f, s1 = 0.f;
#pragma unroll 4
    for (int s = 0; s < p.splits; s++) {
        s0 += p.ws0[s * total + at];
        s1 += p.ws1[s * total + at];
    }
    P::store(p, (int)(at / p.N), (int)(at % p.N), s0, s1);
}

template <class P>
hipError_t launch_reduce_store(const typename P::Params &p, hipStream_t stream) {
    const size_t total = (size_t)p.M * p.N;
    hipLaunchKernelGGL((reduce_store_kernel<P>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       stream, p);
    return hipGetLastError();
}

// Launch over a (tiles, splits) grid for one of the instantiated tile shapes.
// (A 64x128 tile held by four waves of 32 x 64 instead of eight of 32 x 32 needs
// 250 VGPRs and measured slower on every shape; so did a 128x128 tile held by four
// waves of 64 x 64 with the double-buffered loop, which halves the LDS reads and
// operand arithmetic per MFMA: 4096^2 at batch 1024, weight backward 528 -> 537 us.)
enum TileShape { TILE_128x128 = 0, TILE_64x128 = 1, TILE_32x128 = 2, TILE_64x64 = 3, TILE_COUNT = 4 };

inline int tile_rows(int t) { return t == TILE_128x128 ? 128 : t == TILE_32x128 ? 32 : 64; }
inline int tile_cols(int t) { return t == TILE_64x64 ? 64 : 128; }

// Dynamic LDS a problem may ask for on top of the staged tiles.
constexpr size_t kTileExtraLdsMax = 64 * 1024;

template <class P, int BM, int BN, int WM, int WN>
hipError_t launch_tile(dim3 grid, size_t extra, const typename P::Params &p, hipStream_t stream) {
    if (extra > 0) {
        // static + dynamic LDS beyond 64 KB has to be allowed once per kernel and device
        static PerDeviceOnce once;
        hipError_t e = allow_dynamic_lds(
            once, reinterpret_cast<const void *>(mfma_tile_kernel<P, BM, BN, WM, WN>),
            (int)kTileExtraLdsMax);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((mfma_tile_kernel<P, BM, BN, WM, WN>), grid, dim3(WM * WN * 64), extra,
                       stream, p);
    return hipGetLastError();
}

template <class P>
hipError_t launch_tiles(int tile, const typename P::Params &p, hipStream_t stream) {
    const int tiles = ((p.M + tile_rows(tile) - 1) / tile_rows(tile)) *
                      ((p.N + tile_cols(tile) - 1) / tile_cols(tile));
    dim3 grid(tiles, p.splits);
    const size_t extra = P::extra_lds_bytes(p, tile_rows(tile), tile_cols(tile));
    if (extra > kTileExtraLdsMax) return hipErrorInvalidValue;
    switch (tile) {
        case TILE_128x128: return launch_tile<P, 128, 128, 2, 4>(grid, extra, p, stream);
        case TILE_64x128: return launch_tile<P, 64, 128, 2, 4>(grid, extra, p, stream);
        case TILE_32x128: return launch_tile<P, 32, 128, 1, 4>(grid, extra, p, stream);
        case TILE_64x64: return launch_tile<P, 64, 64, 2, 2>(grid, extra, p, stream);
    }
    return hipErrorInvalidValue;
}

}  // namespace tagi

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
// is a plain GEMM; each workgroup re-keys the lists of its own pixels in LDS.
// The permutations the reference runs as separate passes (Jacobian, deltas) are
// folded into the operand addressing. Offsets inside one tensor are 32-bit: the
// entry points refuse tensors of 2^31 elements or more.
#include <type_traits>

#include "tagi_internal.h"
#include "tagi_activation.h"
#include "tagi_mfma_tile.h"

namespace tagi {
namespace {

struct ConvParams {
    const float *w0, *w1;  // mu_w, var_w        [fo][fi*k2]
    const float *a0, *a1;  // mu_a, var_a        [B][fi][wihi]
    const float *d0, *d1;  // delta_mu, delta_var [B][fo][woho]
    const float *e0, *e1;  // forward: mu_b, var_b [fo] (or null); states: jcb; weights: var_w
    const int *idx;        // forward/weights: Fmwa_2 [woho][k2]; states: FCzwa_1 [wihi][nr]
    const int *idx2;       // states: Szz_ud [nr][wihi]
    float *out0, *out1;
    int woho, fo, wihi, fi, k2, B, nr;
    int M, N, R, splits, r_per_split;
    float *ws0, *ws1;
    int group_loads;  // 0: never use the sixteen-byte group loads
    // states: column order. perm_s > 1 numbers the input pixels phase by phase
    // ((y mod s, x mod s) major, then image, then pixel) on maps of width perm_w.
    int perm_s, perm_w;
    // forward only: activation applied to the sums before they are stored
    // (tagi_activation.h); out2 then receives its Jacobian
    int act;
    float *out2;
    // states only: innovations of a residual connection added to the result, laid out
    // like the output. res_mode 1: added before the Jacobian scaling (identity
    // shortcut: (sum + res) * jcb), 2: added after it (a shortcut branch's finished
    // innovations), 0: none.
    const float *res0, *res1;
    int res_mode;
};

// All operand loads below are unconditional: an element outside the problem (or
// a padding tap) reads element 0 of its array and is replaced by zero afterwards.
// Loads under a branch would each wait for their index to arrive before the next
// one is issued; this way a thread's loads of one k-tile are all in flight at once.

// ---- gathered column operand staged [k][column] -------------------------------
// The four columns of a thread are fixed for the whole kernel, only the reduction
// index (channel, tap) moves. The prologue leaves in LDS, for every tap t and
// local column c, the 0-based offset inside one channel map that tap t of column c
// reads (tab[t*BN + c], -1 = nothing); Ctx keeps the image base of the columns.
// Where the four columns of a thread read four CONSECUTIVE elements for every tap
// (stride-1 geometry, groups that do not straddle an image), one unaligned 16-byte
// load replaces the four gathers: the prologue also leaves, per tap and group of
// four columns, (first offset, validity mask) in LDS (qtab), and a flag telling
// whether every group of the tile has that form. Otherwise the tile gathers
// element by element.
struct GatherCtx {
    int img[4];
    int bn;
    const int *tab;
    const int *qtab;
    int fast;      // wave-uniform: all groups of this tile are consecutive
    int ymask[4];  // per column slot: which of the four loaded values are real
    int xok[2];    // per row slot: the loaded values are real
    int taps;      // states: taps that reach any column of this tile (rows of tab)
    const int *act;  // states: their tap numbers
};

__device__ __forceinline__ float4 keep_masked(const float4 &v, int mask) {
    return make_float4((mask & 1) ? v.x : 0.f, (mask & 2) ? v.y : 0.f, (mask & 4) ? v.z : 0.f,
                       (mask & 8) ? v.w : 0.f);
}

typedef float float4u __attribute__((ext_vector_type(4), aligned(4)));

// Second half of the prologue: tab[t*bn + c] is complete (a barrier was passed).
// image_of(n) = image of column n, `src_pix` = elements per channel
// map of the gathered tensor, B = images. A group whose 16-byte window could leave
// the tensor (it starts before the first element of image 0 or ends after the
// last element of image B-1) makes the whole tile gather element by element.
template <class ImageOf>
__device__ __forceinline__ void build_group_table(GatherCtx &ctx, int *tab, int k2, int bn, int n0,
                                                  int N, ImageOf image_of, int src_pix, int B,
                                                  int tid, int nthreads, int allow) {
    int *qtab = tab + k2 * bn, *flag = qtab + k2 * (bn / 4);
    if (tid == 0) *flag = (allow && src_pix >= 4) ? 0 : 1;
    __syncthreads();
    for (int e = tid; e < k2 * (bn / 4); e += nthreads) {
        const int t = e / (bn / 4), c = (e - t * (bn / 4)) * 4, n = n0 + c;
        const int4 off = *reinterpret_cast<const int4 *>(tab + t * bn + c);
        const int o[4] = {off.x, off.y, off.z, off.w};
        int mask = 0, base = 0;
        bool ok = true;
#pragma unroll
        for (int j = 3; j >= 0; j--)
            if (o[j] >= 0) {
                mask |= 1 << j;
                base = o[j] - j;
            }
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (o[j] >= 0 && o[j] != base + j) ok = false;
        if (mask != 0) {
            const int b = image_of(n);
            if (n + 3 >= N || b != image_of(n + 3)) ok = false;
            if (b == 0 && base < 0) ok = false;
            if (b == B - 1 && base + 3 > src_pix - 1) ok = false;
        }
        qtab[e] = ok ? (((base + 4) << 4) | mask) : 0;
        if (!ok) *flag = 1;
    }
    __syncthreads();
    ctx.qtab = qtab;
    ctx.fast = __builtin_amdgcn_readfirstlane(*flag == 0 ? 1 : 0);
}

// Loads the slot's four values and records in ctx.ymask[slot] which of them are
// real; nothing here depends on the loaded data (see fix_y).
__device__ __forceinline__ float4 gather_cols(const float *__restrict__ src, GatherCtx &ctx,
                                              int fast, int slot, int row, int r, int r_end,
                                              int R, int k2, int cstride) {
    const int rr = min(r, R - 1);
    const int ch = rr / k2, t = rr - ch * k2;
    const bool live = r < r_end;
    if (fast) {
        const int e = ctx.qtab[t * (ctx.bn >> 2) + (row >> 2)];
        ctx.ymask[slot] = live ? (e & 15) : 0;
        // an empty group has first offset 0; either way the window lies inside the
        // tensor (the prologue has checked the groups at its two ends)
        const float4u v =
            *reinterpret_cast<const float4u *>(src + (ctx.img[0] + ch * cstride + (e >> 4) - 4));
        return make_float4(v.x, v.y, v.z, v.w);
    }
    const int4 off = *reinterpret_cast<const int4 *>(ctx.tab + t * ctx.bn + row);
    const int o[4] = {off.x, off.y, off.z, off.w};
    float c[4];
    int mask = 0;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const bool ok = live && o[j] >= 0;
        mask |= ok ? (1 << j) : 0;
        c[j] = src[ok ? ctx.img[j] + ch * cstride + o[j] : 0];
    }
    ctx.ymask[slot] = mask;
    return make_float4(c[0], c[1], c[2], c[3]);
}

// Four consecutive reduction elements of row `m` of a [rows][R] matrix; *mask says
// which of them are real (the others were read from a clamped address).
template <bool VEC>
__device__ __forceinline__ float4 load_rows_kc(const float *__restrict__ base, int R, int m,
                                               int rows, int r, int r_end, int *mask) {
    const bool row_ok = m < rows;
    const size_t at = (size_t)(row_ok ? m : 0) * R;
    if (VEC) {  // R % 4 == 0, 16-byte aligned base
        const bool ok = row_ok && r < r_end;
        *mask = ok ? 15 : 0;
        return *reinterpret_cast<const float4 *>(base + at + (ok ? r : 0));
    }
    float c[4];
    int bits = 0;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const bool ok = row_ok && r + j < r_end;
        bits |= ok ? (1 << j) : 0;
        c[j] = base[at + (ok ? r + j : 0)];
    }
    *mask = bits;
    return make_float4(c[0], c[1], c[2], c[3]);
}

// ---- forward ---------------------------------------------------------------
// rows: weights [fo][R] (k-contiguous); columns: gathered activations, staged
// [k][pixel] so that consecutive lanes read consecutive pixels.
template <bool VEC>
struct ConvFwdProblem {
    using Params = ConvParams;
    using Ctx = GatherCtx;
    static constexpr bool XK = true, YK = false, PROLOGUE_WRITES_LDS = true, SPLIT_PER_XCD = false;
    static constexpr bool EPI_PREFETCH = false;
    static constexpr int VARIANTS = 2;  // 1: sixteen-byte loads of consecutive groups
    __device__ static __forceinline__ void adjust_range(const Params &, const Ctx &, int &, int &) {}
    __device__ static __forceinline__ int place_tile(const Params &, int tile, int, int) { return tile; }
    // 130 registers without the request: one 64x128 workgroup per CU instead of two
    static constexpr int min_waves_per_simd(int bm, int bn, int waves) {
        return waves == 8 && bm * bn <= 64 * 128 ? 4 : 0;
    }
    __device__ static __forceinline__ bool variant(const Ctx &ctx) { return ctx.fast != 0; }
    static constexpr int NX = 2, NY = 2, FLAVOR = FLAVOR_FWD_W_ROWS;

    static size_t extra_lds_bytes(const Params &p, int, int bn) {
        return ((size_t)p.k2 * bn + (size_t)p.k2 * (bn / 4) + 4) * sizeof(int);
    }
    __device__ static __forceinline__ void prologue(const Params &p, Ctx &ctx, int *tab, int tid,
                                                    int nthreads, int, int n0, int, int bn, int,
                                                    int) {
        for (int e = tid; e < p.k2 * bn; e += nthreads) {
            const int t = e / bn, c = e - t * bn, n = n0 + c;
            int off = -1;
            if (n < p.N) {
                const int a = p.idx[(n % p.woho) * p.k2 + t];
                if (a > -1) off = a - 1;
            }
            tab[e] = off;
        }
        const int row = (tid % (bn / 4)) * 4;
#pragma unroll
        for (int j = 0; j < 4; j++)
            ctx.img[j] = n0 + row + j < p.N ? ((n0 + row + j) / p.woho) * p.fi * p.wihi : 0;
        ctx.bn = bn;
        ctx.tab = tab;
        build_group_table(
            ctx, tab, p.k2, bn, n0, p.N, [&](int n) { return n / p.woho; }, p.wihi, p.B, tid,
            nthreads, p.group_loads);
    }
    __device__ static __forceinline__ void next_tile(const Params &, Ctx &) {}
    __device__ static __forceinline__ float4 fix_x(const Ctx &ctx, int i, const float4 &v) {
        return keep_masked(v, ctx.xok[i]);
    }
    __device__ static __forceinline__ float4 fix_y(const Ctx &ctx, int i, const float4 &v) {
        return keep_masked(v, ctx.ymask[i]);
    }
    __device__ static __forceinline__ float4 load_x(const Params &p, Ctx &ctx, int, int arr, int i,
                                                    int m0, int row, int r, int r_end) {
        return load_rows_kc<VEC>(arr ? p.w1 : p.w0, p.R, m0 + row, p.M, r, r_end, &ctx.xok[i]);
    }
    __device__ static __forceinline__ float4 load_y(const Params &p, Ctx &ctx, int V, int arr, int i,
                                                    int, int row, int r, int r_end) {
        return gather_cols(arr ? p.a1 : p.a0, ctx, V, i, row, r, r_end, p.R, p.k2, p.wihi);
    }
    __device__ static __forceinline__ void store(const Params &p, int m, int n, float a0,
                                                 float a1) {
        const int b = n / p.woho, o = n - b * p.woho;
        const size_t at = ((size_t)b * p.fo + m) * p.woho + o;
        if (p.e0 != nullptr) {
            a0 += p.e0[m];
            a1 += p.e1[m];
        }
        store_activated(p.act, a0, a1, at, p.out0, p.out1, p.out2);
    }
};

// ---- weight backward ---------------------------------------------------------
// rows: deltas [fo][(b,o)]; columns: gathered activations [(c,t)][(b,o)]; both
// have the reduction (b,o) as their fast index. A thread's column (channel, tap)
// is fixed per slot; the four reduction positions of a slot move by one k-tile
// per visit, and the table entries for the NEXT visit are requested right after
// the current visit's gathers, so that the table lookup is never waited for.
constexpr int DW_SLOTS = 4;  // most column slots a thread can have (32x128 tile)

template <bool VEC>
struct ConvDwProblem {
    using Params = ConvParams;
    struct Ctx {
        int cb[DW_SLOTS];       // channel offset ch*wihi of the slot's column, -1: no column
        int tap[DW_SLOTS];
        int nidx[DW_SLOTS][4];  // table entries of the next visit
        int nimg[DW_SLOTS][4];  // image offsets b*fi*wihi of the next visit
    };
    static constexpr bool XK = true, YK = true, PROLOGUE_WRITES_LDS = false, SPLIT_PER_XCD = true;
    static constexpr bool EPI_PREFETCH = true;
    static constexpr int VARIANTS = 1;
    __device__ static __forceinline__ void adjust_range(const Params &, const Ctx &, int &, int &) {}
    __device__ static __forceinline__ int place_tile(const Params &, int tile, int, int) { return tile; }
    static constexpr int min_waves_per_simd(int, int, int) { return 0; }
    static constexpr int NX = 2, NY = 1, FLAVOR = FLAVOR_DELTA_ROWS;

    static size_t extra_lds_bytes(const Params &, int, int) { return 0; }

    __device__ static __forceinline__ void lookup(const Params &p, Ctx &ctx, int i, int r) {
        const int rr = min(r, p.R - 1);  // positions past the end repeat the last one
        int b = rr / p.woho, o = rr - b * p.woho;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            ctx.nidx[i][j] = p.idx[o * p.k2 + ctx.tap[i]];
            ctx.nimg[i][j] = b * p.fi * p.wihi;
            if (rr + j + 1 < p.R && ++o == p.woho) {
                o = 0;
                b++;
            }
        }
    }
    __device__ static __forceinline__ void prologue(const Params &p, Ctx &ctx, int *, int tid,
                                                    int nthreads, int, int n0, int, int bn,
                                                    int r_begin, int) {
        const int slots = bn * KT / 4 / nthreads;
#pragma unroll
        for (int i = 0; i < DW_SLOTS; i++) {
            if (i >= slots) break;
            const int f = tid + i * nthreads;
            const int n = n0 + f / (KT / 4);
            const int nn = min(n, p.N - 1);
            const int ch = nn / p.k2;
            ctx.tap[i] = nn - ch * p.k2;
            ctx.cb[i] = n < p.N ? ch * p.wihi : -1;
            lookup(p, ctx, i, r_begin + (f % (KT / 4)) * 4);
        }
    }
    __device__ static __forceinline__ void next_tile(const Params &, Ctx &) {}
    __device__ static __forceinline__ float4 fix_x(const Ctx &, int, const float4 &v) { return v; }
    __device__ static __forceinline__ float4 fix_y(const Ctx &, int, const float4 &v) { return v; }
    __device__ static __forceinline__ float4 load_x(const Params &p, Ctx &, int, int arr, int, int m0,
                                                    int row, int r, int r_end) {
        const float *__restrict__ d = arr ? p.d1 : p.d0;
        const int m = m0 + row;
        const bool row_ok = m < p.M;
        const int mm = row_ok ? m : 0;
        const int rr = min(r, p.R - 1);
        int b = rr / p.woho, o = rr - b * p.woho;
        if (VEC) {  // woho % 4 == 0: the four positions share the image
            const bool ok = row_ok && r < r_end;
            const float4 v = *reinterpret_cast<const float4 *>(
                d + (ok ? ((size_t)b * p.fo + mm) * p.woho + o : 0));
            return ok ? v : make_float4(0.f, 0.f, 0.f, 0.f);
        }
        float c[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const bool ok = row_ok && r + j < r_end;
            const float v = d[ok ? ((size_t)b * p.fo + mm) * p.woho + o : 0];
            c[j] = ok ? v : 0.f;
            if (++o == p.woho) {
                o = 0;
                b++;
            }
        }
        return make_float4(c[0], c[1], c[2], c[3]);
    }
    __device__ static __forceinline__ float4 load_y(const Params &p, Ctx &ctx, int, int, int i, int,
                                                    int, int r, int r_end) {
        float c[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int a = ctx.nidx[i][j];
            const bool ok = ctx.cb[i] >= 0 && r + j < r_end && a > -1;
            const float v = p.a0[ok ? ctx.nimg[i][j] + ctx.cb[i] + a - 1 : 0];
            c[j] = ok ? v : 0.f;
        }
        lookup(p, ctx, i, r + KT);
        return make_float4(c[0], c[1], c[2], c[3]);
    }
    __device__ static __forceinline__ float epi_load(const Params &p, int m, int n) {
        return p.e0[(size_t)m * p.N + n];
    }
    __device__ static __forceinline__ void store_with(const Params &p, int m, int n, float a0,
                                                      float a1, float e) {
        const size_t at = (size_t)m * p.N + n;
        p.out0[at] = a0 * e;
        p.out1[at] = a1 * e * e;
    }
    __device__ static __forceinline__ void store(const Params &p, int m, int n, float a0,
                                                 float a1) {
        store_with(p, m, n, a0, a1, epi_load(p, m, n));
    }
};

// The same contraction when every group of four reduction positions lies in one
// image (woho % 4 == 0, 16-byte aligned innovations): all positions of a thread
// move together, so the thread keeps (pixel, image offsets) of its group in
// registers and advances them by one k-tile per visit instead of dividing; the
// innovations are one 16-byte load.
struct ConvDwVecProblem {
    using Params = ConvParams;
    struct Ctx {
        int o;      // pixel of the group in the tile being fetched
        int xoff;   // b*fo*woho + o of that group
        int img;    // b*fi*wihi
        int xrow[2];            // m*woho of the row slots, -1: no row
        int cb[DW_SLOTS];       // ch*wihi of the column slots, -1: no column
        int tap[DW_SLOTS];
        int nidx[DW_SLOTS][4];  // table entries of the tile being fetched
        int xok[2];             // masks of the values in flight, applied by fix_x / fix_y
        int ymask[DW_SLOTS];
    };
    static constexpr bool XK = true, YK = true, PROLOGUE_WRITES_LDS = false, SPLIT_PER_XCD = true;
    static constexpr bool EPI_PREFETCH = true;
    static constexpr int VARIANTS = 1;
    __device__ static __forceinline__ void adjust_range(const Params &, const Ctx &, int &, int &) {}
    __device__ static __forceinline__ int place_tile(const Params &, int tile, int, int) { return tile; }
    // (asking for four or five 64x64 workgroups per CU instead of three measured
    // no gain)
    static constexpr int min_waves_per_simd(int, int, int) { return 0; }
    static constexpr int NX = 2, NY = 1, FLAVOR = FLAVOR_DELTA_ROWS;

    static size_t extra_lds_bytes(const Params &, int, int) { return 0; }

    __device__ static __forceinline__ void lookup(const Params &p, Ctx &ctx, int i, int o) {
        const int *q = p.idx + (size_t)(o * p.k2 + ctx.tap[i]);
#pragma unroll
        for (int j = 0; j < 4; j++) ctx.nidx[i][j] = q[j * p.k2];
    }
    __device__ static __forceinline__ void prologue(const Params &p, Ctx &ctx, int *, int tid,
                                                    int nthreads, int m0, int n0, int bm, int bn,
                                                    int r_begin, int) {
        const int r = min(r_begin + (tid % (KT / 4)) * 4, p.R - 4);
        const int b = r / p.woho;
        ctx.o = r - b * p.woho;
        ctx.xoff = b * p.fo * p.woho + ctx.o;
        ctx.img = b * p.fi * p.wihi;
        const int xslots = bm * KT / 4 / nthreads, yslots = bn * KT / 4 / nthreads;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            if (i >= xslots) break;
            const int m = m0 + (tid + i * nthreads) / (KT / 4);
            ctx.xrow[i] = m < p.M ? m * p.woho : -1;
        }
#pragma unroll
        for (int i = 0; i < DW_SLOTS; i++) {
            if (i >= yslots) break;
            const int n = n0 + (tid + i * nthreads) / (KT / 4);
            const int nn = min(n, p.N - 1);
            const int ch = nn / p.k2;
            ctx.tap[i] = nn - ch * p.k2;
            ctx.cb[i] = n < p.N ? ch * p.wihi : -1;
            lookup(p, ctx, i, ctx.o);
        }
    }
    __device__ static __forceinline__ void next_tile(const Params &p, Ctx &ctx) {
        ctx.o += KT;
        ctx.xoff += KT;
        while (ctx.o >= p.woho) {
            ctx.o -= p.woho;
            ctx.img += p.fi * p.wihi;
            ctx.xoff += (p.fo - 1) * p.woho;
        }
    }
    __device__ static __forceinline__ float4 load_x(const Params &p, Ctx &ctx, int, int arr, int i, int,
                                                    int, int r, int r_end) {
        const bool ok = r < r_end && ctx.xrow[i] >= 0;
        const float *__restrict__ d = arr ? p.d1 : p.d0;
        ctx.xok[i] = ok ? 15 : 0;
        return *reinterpret_cast<const float4 *>(d + (ok ? ctx.xrow[i] + ctx.xoff : 0));
    }
    __device__ static __forceinline__ float4 fix_x(const Ctx &ctx, int i, const float4 &v) {
        return keep_masked(v, ctx.xok[i]);
    }
    __device__ static __forceinline__ float4 fix_y(const Ctx &ctx, int i, const float4 &v) {
        return keep_masked(v, ctx.ymask[i]);
    }
    __device__ static __forceinline__ float4 load_y(const Params &p, Ctx &ctx, int, int, int i, int,
                                                    int, int r, int r_end) {
        const bool live = r < r_end && ctx.cb[i] >= 0;
        const int base = ctx.img + ctx.cb[i] - 1;
        float c[4];
        int mask = 0;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int a = ctx.nidx[i][j];
            const bool ok = live && a > -1;
            mask |= ok ? (1 << j) : 0;
            c[j] = p.a0[ok ? base + a : 0];
        }
        ctx.ymask[i] = mask;
        // table entries of the next k-tile (always inside the table: the pixel
        // index wraps, and a group of four never straddles its end)
        int o = ctx.o + KT;
        while (o >= p.woho) o -= p.woho;
        lookup(p, ctx, i, o);
        return make_float4(c[0], c[1], c[2], c[3]);
    }
    __device__ static __forceinline__ float epi_load(const Params &p, int m, int n) {
        return p.e0[(size_t)m * p.N + n];
    }
    __device__ static __forceinline__ void store_with(const Params &p, int m, int n, float a0,
                                                      float a1, float e) {
        const size_t at = (size_t)m * p.N + n;
        p.out0[at] = a0 * e;
        p.out1[at] = a1 * e * e;
    }
    __device__ static __forceinline__ void store(const Params &p, int m, int n, float a0,
                                                 float a1) {
        store_with(p, m, n, a0, a1, epi_load(p, m, n));
    }
};

// ---- state backward -----------------------------------------------------------
// rows: weights re-indexed [c][(fo,t)]; columns: gathered deltas [(fo,t)][(b,p)].
// The reference's FCzwa_1 / Szz_ud pair lists, per input pixel, the (tap, output
// pixel) occurrences; the prologue re-keys the lists of the tile's pixels by tap
// (each tap meets a pixel at most once), which is the table gather_cols wants.
//
// A strided convolution reaches an input pixel through few of its taps, and which
// ones depends on the pixel's phase (y mod s, x mod s): a 3x3 stride-2 kernel
// touches a pixel through 4, 2, 2 or 1 of its 9 taps. Summing over all taps would
// multiply three zeros for every product. So the columns can be numbered phase
// by phase (ConvParams::perm_s), which makes the pixels of a tile share their
// taps, and every tile reduces over the taps that reach any of ITS columns only:
// the prologue finds them in the table, whatever the table holds, and keeps one
// table row per such tap. The numbering only decides which pixels sit together;
// results do not depend on it.
struct DzColumn {
    int b, px;
};
__device__ __forceinline__ DzColumn dz_column(const ConvParams &p, int n) {
    DzColumn c;
    if (p.perm_s <= 1) {
        c.b = n / p.wihi;
        c.px = n - c.b * p.wihi;
        return c;
    }
    const int s = p.perm_s, W = p.perm_w, ws = W / s;
    const int per_img = p.wihi / (s * s), per_phase = p.B * per_img;
    const int phase = n / per_phase, rem = n - phase * per_phase;
    c.b = rem / per_img;
    const int l = rem - c.b * per_img, ly = l / ws, lx = l - ly * ws;
    c.px = (ly * s + phase / s) * W + lx * s + phase % s;
    return c;
}

struct ConvDzProblem {
    using Params = ConvParams;
    using Ctx = GatherCtx;
    static constexpr bool XK = true, YK = false, PROLOGUE_WRITES_LDS = true, SPLIT_PER_XCD = false;
    static constexpr bool EPI_PREFETCH = true;
    static constexpr int VARIANTS = 2;  // 1: sixteen-byte loads of consecutive groups
    static constexpr int min_waves_per_simd(int, int, int) { return 0; }
    __device__ static __forceinline__ bool variant(const Ctx &ctx) { return ctx.fast != 0; }
    static constexpr int NX = 1, NY = 2, FLAVOR = FLAVOR_DELTA_COLS;

    // [k2][bn] offsets, [k2][bn/4] groups + flag, tap mask, [k2] active taps
    static size_t extra_lds_bytes(const Params &p, int, int bn) {
        return ((size_t)p.k2 * bn + (size_t)p.k2 * (bn / 4) + 4 + 4 + p.k2) * sizeof(int);
    }
    __device__ static __forceinline__ void prologue(const Params &p, Ctx &ctx, int *tab, int tid,
                                                    int nthreads, int, int n0, int, int bn, int,
                                                    int) {
        int *mask = tab + p.k2 * bn + p.k2 * (bn / 4) + 4, *act = mask + 4;
        // pass 1: which taps reach a column of this tile (more than 32 taps: all)
        if (tid == 0) *mask = p.k2 > 32 ? -1 : 0;
        __syncthreads();
        if (p.k2 <= 32) {
            int seen = 0;
            for (int e = tid; e < p.nr * bn; e += nthreads) {
                const int j = e / bn, c = e - j * bn, n = n0 + c;
                if (n >= p.N) continue;
                const int px = dz_column(p, n).px;
                const int tap = p.idx[px * p.nr + j], o = p.idx2[j * p.wihi + px];
                if (o > -1 && tap >= 1 && tap <= p.k2) seen |= 1 << (tap - 1);
            }
            if (seen) atomicOr(mask, seen);
        }
        __syncthreads();
        const int m = *mask;
        const int taps = p.k2 > 32 ? p.k2 : __popc(m);
        for (int t = tid; t < p.k2; t += nthreads) {
            if (p.k2 > 32)
                act[t] = t;
            else if (m >> t & 1)
                act[__popc(m & ((1 << t) - 1))] = t;
        }
        for (int e = tid; e < taps * bn; e += nthreads) tab[e] = -1;
        __syncthreads();
        // pass 2: one table row per such tap
        for (int e = tid; e < p.nr * bn; e += nthreads) {
            const int j = e / bn, c = e - j * bn, n = n0 + c;
            if (n >= p.N) continue;
            const int px = dz_column(p, n).px;
            const int tap = p.idx[px * p.nr + j], o = p.idx2[j * p.wihi + px];
            if (o > -1 && tap >= 1 && tap <= p.k2) {
                const int row = p.k2 > 32 ? tap - 1 : __popc(m & ((1 << (tap - 1)) - 1));
                tab[row * bn + c] = o - 1;
            }
        }
        const int row = (tid % (bn / 4)) * 4;
#pragma unroll
        for (int j = 0; j < 4; j++)
            ctx.img[j] = n0 + row + j < p.N ? dz_column(p, n0 + row + j).b * p.fo * p.woho : 0;
        ctx.bn = bn;
        ctx.tab = tab;
        ctx.taps = taps;
        ctx.act = act;
        build_group_table(
            ctx, tab, taps, bn, n0, p.N, [&](int n) { return dz_column(p, n).b; }, p.woho, p.B, tid,
            nthreads, p.group_loads);
    }
    // Tiles of different phases differ in length (4, 2, 2, 1 taps for 3x3 stride 2)
    // and lie phase by phase. The two slices of a tile tend to land on the same CU;
    // odd slices walk the tiles backwards, so a CU gets a long and a short one.
    __device__ static __forceinline__ int place_tile(const Params &p, int tile, int split,
                                                     int tiles) {
        return (p.perm_s > 1 && (split & 1)) ? tiles - 1 - tile : tile;
    }
    // The slice [r_begin, r_end) was cut in units of k2 (whole output channels);
    // with `taps` rows per channel it becomes this.
    __device__ static __forceinline__ void adjust_range(const Params &p, const Ctx &ctx,
                                                        int &r_begin, int &r_end) {
        r_begin = (r_begin / p.k2) * ctx.taps;
        r_end = (r_end / p.k2) * ctx.taps;
    }
    __device__ static __forceinline__ void next_tile(const Params &, Ctx &) {}
    __device__ static __forceinline__ float4 fix_x(const Ctx &ctx, int i, const float4 &v) {
        return keep_masked(v, ctx.xok[i]);
    }
    __device__ static __forceinline__ float4 fix_y(const Ctx &ctx, int i, const float4 &v) {
        return keep_masked(v, ctx.ymask[i]);
    }
    __device__ static __forceinline__ float4 load_x(const Params &p, Ctx &ctx, int, int, int i, int m0,
                                                    int row, int r, int r_end) {
        const int m = m0 + row;
        const bool row_ok = m < p.M;
        const int rr = min(r, max(p.fo * ctx.taps - 1, 0));
        int f = ctx.taps ? rr / ctx.taps : 0, ti = rr - f * ctx.taps;
        float c[4];
        int mask = 0;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const bool ok = row_ok && r + j < r_end;
            mask |= ok ? (1 << j) : 0;
            c[j] = p.w0[ok ? ((size_t)f * p.fi + m) * p.k2 + ctx.act[ti] : 0];
            if (++ti >= ctx.taps) {
                ti = 0;
                f++;
            }
        }
        ctx.xok[i] = mask;
        return make_float4(c[0], c[1], c[2], c[3]);
    }
    __device__ static __forceinline__ float4 load_y(const Params &p, Ctx &ctx, int V, int arr, int i,
                                                    int, int row, int r, int r_end) {
        return gather_cols(arr ? p.d1 : p.d0, ctx, V, i, row, r, r_end,
                           max(p.fo * ctx.taps, 1), max(ctx.taps, 1), p.woho);
    }
    __device__ static __forceinline__ size_t out_index(const Params &p, int m, int n) {
        const DzColumn c = dz_column(p, n);
        return ((size_t)c.b * p.fi + m) * p.wihi + c.px;
    }
    __device__ static __forceinline__ float epi_load(const Params &p, int m, int n) {
        return p.e0[out_index(p, m, n)];
    }
    __device__ static __forceinline__ void store_with(const Params &p, int m, int n, float a0,
                                                      float a1, float e) {
        const size_t at = out_index(p, m, n);
        if (p.res_mode == 1) {
            a0 += p.res0[at];
            a1 += p.res1[at];
        }
        a0 *= e;
        a1 *= e * e;
        if (p.res_mode == 2) {
            a0 += p.res0[at];
            a1 += p.res1[at];
        }
        p.out0[at] = a0;
        p.out1[at] = a1;
    }
    __device__ static __forceinline__ void store(const Params &p, int m, int n, float a0,
                                                 float a1) {
        store_with(p, m, n, a0, a1, epi_load(p, m, n));
    }
};

}  // namespace
}  // namespace tagi

#include "tagi_conv_stencil.h"
#include "tagi_conv_stencil_s2.h"

namespace tagi {
namespace {

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

// Tile shape and number of reduction slices of the forward / state-backward
// GEMMs: M rows (output or input channels), N columns (batch x pixels), R
// reduction (taps x channels). Late ResNet stages have few columns and a long
// reduction; slicing it keeps every CU busy.
void conv2d_plan(int M, int N, int R, int *tile, int *splits) {
    *tile = M > 32 ? TILE_64x128 : TILE_32x128;
    const int tiles = ceil_div(M, tile_rows(*tile)) * ceil_div(N, tile_cols(*tile));
    const int k_tiles = ceil_div(R, KT);
    int s = ceil_div(2 * num_cu(), tiles);
    const int cap = k_tiles / 8 > 0 ? k_tiles / 8 : 1;  // at least 8 k-tiles per slice
    if (s > cap) s = cap;
    if (s < 1) s = 1;
    const int per = ceil_div(ceil_div(R, s), KT) * KT;
    *splits = ceil_div(R, per);
}

namespace {
// `stencil`: map width when the regular-stencil kernel applies (slices are then
// whole groups of 32 channels: a multiple of its 72-step and of the table-driven
// loop's 32-step k-tile), 0 otherwise.
inline int lcm_int(int a, int b) {
    int x = a, y = b;
    while (y) {
        const int t = x % y;
        x = y;
        y = t;
    }
    return a / x * b;
}

// `s2_all`: output map width when the stride-2 state-backward stencil kernel applies.
template <class P, bool DZ>
hipError_t run_sliced(int tile, int splits, int stencil, float *ws0, float *ws1, ConvParams &p,
                      hipStream_t stream, int s2_all = 0, int s2_fwd = 0) {
    // the state backward re-states its slices per tile in whole output channels
    // (the stencil kernels: in whole groups of 32 channels)
    const int unit = (stencil || s2_all || s2_fwd) ? 32 * p.k2 : DZ ? lcm_int(KT, p.k2) : KT;
    const int per = ceil_div(ceil_div(p.R, splits), unit) * unit;
    p.splits = ceil_div(p.R, per);
    p.r_per_split = per;
    p.ws0 = ws0;
    p.ws1 = ws1;
    hipError_t e = hipSuccess;
    if constexpr (!DZ) {
        if (s2_fwd) {
            e = p.k2 == 9 ? launch_conv_stencil_s2_fwd<3>(s2_fwd, p, stream)
                          : launch_conv_stencil_s2_fwd<2>(s2_fwd, p, stream);
            if (e != hipSuccess || p.splits == 1) return e;
            return launch_reduce_store<P>(p, stream);
        }
    }
    e = s2_all     ? (p.k2 == 9 ? launch_conv_stencil_s2_all_dz<3>(s2_all, p, stream)
                                           : launch_conv_stencil_s2_all_dz<2>(s2_all, p, stream))
                   : stencil  ? launch_conv_stencil<DZ>(stencil, p, stream)
                              : launch_tiles<P>(tile, p, stream);
    if (e != hipSuccess || p.splits == 1) return e;
    if constexpr (DZ) {
        // phase-ordered columns of a stride-2 layer: fold in the order of the output
        const uintptr_t ptrs = reinterpret_cast<uintptr_t>(p.out0) | reinterpret_cast<uintptr_t>(p.out1) |
                               reinterpret_cast<uintptr_t>(p.e0) | reinterpret_cast<uintptr_t>(p.res0) |
                               reinterpret_cast<uintptr_t>(p.res1);
        if (p.perm_s == 2 && p.perm_w % 2 == 0 && (ptrs & 7u) == 0 && g_conv2d_s2_all)
            return launch_reduce_store_s2_pairs(p, stream);
    }
    return launch_reduce_store<P>(p, stream);
}
}  // namespace

int g_conv2d_group_loads = 1;
int g_conv2d_stencil = 1;
int g_conv2d_phase_order = 1;
int g_conv2d_s2_all = 1;

// Output map width when the state backward of a stride-2 layer runs on the kernel that
// keeps all four phases in one workgroup (3x3 with padding on the right and bottom, or
// 2x2 without padding; the kernel verifies the tables), 0 otherwise.
int conv2d_bwd_dz_s2_all(const float *mu_w, const float *dmu, const float *dvar, int B, int fo,
                         int woho, int wihi, int fi, int ki, int nr) {
    if (!g_conv2d_stencil || !g_conv2d_s2_all || !g_conv2d_phase_order) return 0;
    if (!((ki == 3 && nr == 4) || (ki == 2 && nr == 1))) return 0;
    if (wihi != 4 * woho || fo % 32 != 0 || fi % 64 != 0 || ((long long)B * woho) % 128 != 0 ||
        !aligned16(mu_w) || !aligned16(dmu) || !aligned16(dvar))
        return 0;
    return s2_out_width(woho);
}

// Its reduction slices: one workgroup per CU is resident; whole groups of 32 channels.
int conv2d_bwd_dz_s2_all_splits(int B, int fo, int woho, int fi) {
    const int tiles = (fi / 64) * (int)((long long)B * woho / 128);
    int s = tiles > 0 ? num_cu() / tiles : 1;
    if (s > fo / 32) s = fo / 32;
    return s < 1 ? 1 : s;
}

hipError_t launch_conv2d_fwd(const float *mu_w, const float *var_w, const float *mu_b,
                             const float *var_b, const float *mu_a, const float *var_a,
                             const int *aidx, int woho, int fo, int wihi, int fi, int ki, int B,
                             int bias, int tile, int splits, float *ws0, float *ws1, float *mu_z,
                             float *var_z, hipStream_t stream, int act, float *jcb) {
    ConvParams p = {};
    p.act = act; p.out2 = jcb;
    p.w0 = mu_w; p.w1 = var_w; p.a0 = mu_a; p.a1 = var_a;
    p.e0 = bias ? mu_b : nullptr; p.e1 = bias ? var_b : nullptr;
    p.idx = aidx; p.out0 = mu_z; p.out1 = var_z;
    p.woho = woho; p.fo = fo; p.wihi = wihi; p.fi = fi; p.k2 = ki * ki; p.B = B;
    p.M = fo; p.N = B * woho; p.R = p.k2 * fi;
    p.group_loads = g_conv2d_group_loads;
    const bool vec = (p.R % 4 == 0) && aligned16(mu_w) && aligned16(var_w);
    // 3x3, stride 1, "same" padding on a square map (the kernel verifies the table)
    int stencil = 0;
    if (g_conv2d_stencil && vec && ki == 3 && woho == wihi && fi % 8 == 0 && fo % 64 == 0 &&
        tile == TILE_64x128 && aligned16(mu_a) && aligned16(var_a))
        stencil = stencil_width(wihi);
    // stride 2 on a square map, 3x3 with padding on the right and bottom or 2x2 (the
    // kernel verifies the table)
    int s2_fwd = 0;
    if (g_conv2d_stencil && g_conv2d_s2_all && vec && (ki == 3 || ki == 2) && wihi == 4 * woho &&
        fi % 8 == 0 && fo % 64 == 0 && tile == TILE_64x128 && aligned16(mu_a) && aligned16(var_a))
        s2_fwd = s2_out_width(woho);
    if (vec)
        return run_sliced<ConvFwdProblem<true>, false>(tile, splits, stencil, ws0, ws1, p, stream, 0,
                                                       s2_fwd);
    return run_sliced<ConvFwdProblem<false>, false>(tile, splits, 0, ws0, ws1, p, stream);
}

namespace {
// Problem description of the state backward; *stencil / *s2_all: map width when the
// unit-stride / stride-2 stencil kernel applies, 0 otherwise.
ConvParams dz_params(const float *mu_w, const float *jcb, const float *dmu, const float *dvar,
                     const int *zw_idx, const int *zud_idx, int woho, int fo, int wihi, int fi,
                     int ki, int nr, int B, int tile, float *out_dmu, float *out_dvar,
                     const float *res_mu, const float *res_var, int res_mode, int *stencil,
                     int *s2_all) {
    const int k2 = ki * ki;
    ConvParams p = {};
    p.res0 = res_mu; p.res1 = res_var; p.res_mode = res_mu != nullptr ? res_mode : 0;
    p.w0 = mu_w; p.d0 = dmu; p.d1 = dvar; p.e0 = jcb; p.idx = zw_idx; p.idx2 = zud_idx;
    p.out0 = out_dmu; p.out1 = out_dvar;
    p.woho = woho; p.fo = fo; p.wihi = wihi; p.fi = fi; p.k2 = k2; p.B = B; p.nr = nr;
    p.M = fi; p.N = B * wihi; p.R = k2 * fo;
    p.group_loads = g_conv2d_group_loads;
    // strided convolution on a square map: number the columns phase by phase
    p.perm_s = 1;
    p.perm_w = 0;
    if (g_conv2d_phase_order && wihi > woho && wihi % woho == 0) {
        int s = 1, w = 1;
        while (s * s < wihi / woho) s++;
        while (w * w < wihi) w++;
        if (s * s == wihi / woho && w * w == wihi && w % s == 0) {
            p.perm_s = s;
            p.perm_w = w;
        }
    }
    *stencil = 0;
    if (g_conv2d_stencil && ki == 3 && nr == 9 && woho == wihi && fo % 8 == 0 && fi % 64 == 0 &&
        tile == TILE_64x128 && aligned16(mu_w) && aligned16(dmu) && aligned16(dvar))
        *stencil = stencil_width(wihi);
    // stride 2, 3x3 with padding on the right and bottom or 2x2 (the kernel verifies the tables)
    *s2_all = (p.perm_s == 2 && tile == TILE_64x128)
                  ? conv2d_bwd_dz_s2_all(mu_w, dmu, dvar, B, fo, woho, wihi, fi, ki, nr)
                  : 0;
    return p;
}

// Reduction slices of a launch: whole `unit`s per slice.
void plan_slices(ConvParams &p, int splits, int unit, float *ws0, float *ws1) {
    const int per = ceil_div(ceil_div(p.R, splits), unit) * unit;
    p.splits = ceil_div(p.R, per);
    p.r_per_split = per;
    p.ws0 = ws0;
    p.ws1 = ws1;
}
}  // namespace

hipError_t launch_conv2d_bwd_dz(const float *mu_w, const float *jcb, const float *dmu,
                                const float *dvar, const int *zw_idx, const int *zud_idx,
                                int woho, int fo, int wihi, int fi, int ki, int nr, int B,
                                int tile, int splits, float *ws0, float *ws1, float *out_dmu,
                                float *out_dvar, hipStream_t stream, const float *res_mu,
                                const float *res_var, int res_mode) {
    int stencil = 0, s2_all = 0;
    ConvParams p = dz_params(mu_w, jcb, dmu, dvar, zw_idx, zud_idx, woho, fo, wihi, fi, ki, nr, B,
                             tile, out_dmu, out_dvar, res_mu, res_var, res_mode, &stencil, &s2_all);
    return run_sliced<ConvDzProblem, true>(tile, splits, stencil, ws0, ws1, p, stream, s2_all);
}

// Workgroups of the weight-backward kernel that one CU holds at a time.
int conv2d_bwd_dw_blocks_per_cu(int tile) {
    static int cached[TILE_COUNT] = {};
    if (tile < 0 || tile >= TILE_COUNT) return 1;
    if (cached[tile] == 0) {
        int n = 0;
        hipError_t e = hipErrorInvalidValue;
        using P = ConvDwVecProblem;
        switch (tile) {
            case TILE_128x128:
                e = hipOccupancyMaxActiveBlocksPerMultiprocessor(
                    &n, reinterpret_cast<const void *>(mfma_tile_kernel<P, 128, 128, 2, 4>), 512, 0);
                break;
            case TILE_64x128:
                e = hipOccupancyMaxActiveBlocksPerMultiprocessor(
                    &n, reinterpret_cast<const void *>(mfma_tile_kernel<P, 64, 128, 2, 4>), 512, 0);
                break;
            case TILE_32x128:
                e = hipOccupancyMaxActiveBlocksPerMultiprocessor(
                    &n, reinterpret_cast<const void *>(mfma_tile_kernel<P, 32, 128, 1, 4>), 256, 0);
                break;
            case TILE_64x64:
                e = hipOccupancyMaxActiveBlocksPerMultiprocessor(
                    &n, reinterpret_cast<const void *>(mfma_tile_kernel<P, 64, 64, 2, 2>), 256, 0);
                break;
        }
        cached[tile] = (e == hipSuccess && n >= 1) ? n : 1;
    }
    return cached[tile];
}

// Map width when the weight backward runs on the regular-stencil kernel (3x3,
// stride 1, "same" padding on a square map -- the kernel verifies the table; 64 x 64
// tiles of whole channels, slices of whole 64-pixel k-tiles), 0 otherwise.
int conv2d_bwd_dw_stencil(const float *mu_a, const float *dmu, const float *dvar, int B, int fo,
                          int woho, int wihi, int fi, int ki, int tile) {
    if (!g_conv2d_stencil || ki != 3 || woho != wihi || woho % 4 != 0 || fi % 64 != 0 ||
        fo % 64 != 0 || ((long long)B * woho) % 64 != 0 || tile != TILE_64x64 ||
        !aligned16(mu_a) || !aligned16(dmu) || !aligned16(dvar))
        return 0;
    return stencil_width(wihi);
}

// The same for the stride-2 layers (3x3 with padding on the right and bottom, 2x2 without):
// output map width when the weight backward runs on their stencil kernel, 0 otherwise.
int conv2d_bwd_dw_s2(const float *mu_a, const float *dmu, const float *dvar, int B, int fo,
                     int woho, int wihi, int fi, int ki, int tile) {
    if (!g_conv2d_stencil || !g_conv2d_s2_all || (ki != 3 && ki != 2) || wihi != 4 * woho ||
        fi % 64 != 0 || fo % 64 != 0 || ((long long)B * woho) % 64 != 0 || tile != TILE_64x64 ||
        !aligned16(mu_a) || !aligned16(dmu) || !aligned16(dvar))
        return 0;
    return s2_out_width(woho);
}

// Reduction slices for the stencil kernel (two 8-wave workgroups per CU): the
// fewest rounds of resident workgroups that are at least 95 % full, else the
// fullest of up to four rounds. A partly filled round costs as much as a full one.
int conv2d_bwd_dw_stencil_splits(int out_tiles) {
    const int resident = 2 * num_cu();
    int best = 1;
    double best_fill = 0.0;
    for (int rounds = 1; rounds <= 4; rounds++) {
        const int s = rounds * resident / out_tiles;
        if (s < 1) continue;
        const double fill = (double)out_tiles * s / (rounds * resident);
        if (fill >= 0.95) return s;
        if (fill > best_fill) {
            best_fill = fill;
            best = s;
        }
    }
    return best;
}

namespace {
ConvParams dw_params(const float *var_w, const float *mu_a, const float *dmu, const float *dvar,
                     const int *aidx, int B, int fo, int woho, int wihi, int fi, int ki,
                     float *dmu_w, float *dvar_w) {
    ConvParams p = {};
    p.a0 = mu_a; p.d0 = dmu; p.d1 = dvar; p.e0 = var_w; p.idx = aidx;
    p.out0 = dmu_w; p.out1 = dvar_w;
    p.woho = woho; p.fo = fo; p.wihi = wihi; p.fi = fi; p.k2 = ki * ki; p.B = B;
    p.M = fo; p.N = p.k2 * fi; p.R = B * woho;
    return p;
}
}  // namespace

hipError_t launch_conv2d_bwd_dw(const float *var_w, const float *mu_a, const float *dmu,
                                const float *dvar, const int *aidx, int B, int fo, int woho,
                                int wihi, int fi, int ki, int tile, int splits, float *ws0, float *ws1,
                                float *dmu_w, float *dvar_w, hipStream_t stream) {
    ConvParams p = dw_params(var_w, mu_a, dmu, dvar, aidx, B, fo, woho, wihi, fi, ki, dmu_w, dvar_w);
    const bool vec = (woho % 4 == 0) && aligned16(dmu) && aligned16(dvar);
    const int stencil = conv2d_bwd_dw_stencil(mu_a, dmu, dvar, B, fo, woho, wihi, fi, ki, tile);
    const int s2 = conv2d_bwd_dw_s2(mu_a, dmu, dvar, B, fo, woho, wihi, fi, ki, tile);
    plan_slices(p, splits, (stencil || s2) ? 64 : KT, ws0, ws1);
    hipError_t e = stencil ? launch_conv_stencil_dw(stencil, p, stream)
                   : s2    ? (ki == 3 ? launch_conv_stencil_s2_dw<3>(s2, p, stream)
                                      : launch_conv_stencil_s2_dw<2>(s2, p, stream))
                   : vec   ? launch_tiles<ConvDwVecProblem>(tile, p, stream)
                           : launch_tiles<ConvDwProblem<false>>(tile, p, stream);
    if (e != hipSuccess) return e;
    if (p.splits > 1)
        e = launch_reduce_splits(EPI_SCALE, ws0, ws1, p.splits, p.M, p.N, var_w, nullptr, dmu_w,
                                 dvar_w, p.N, stream);
    return e;
}

int g_conv2d_bwd_pair = 1;

// Map width when the state backward and the weight backward of a layer can share one
// launch (both on their unit-stride stencil kernels), 0 otherwise.
int conv2d_bwd_pair(const float *mu_w, const float *mu_a, const float *dmu, const float *dvar, int B,
                    int fo, int woho, int wihi, int fi, int ki, int nr) {
    if (!g_conv2d_bwd_pair || !g_conv2d_stencil || ki != 3 || nr != 9 || woho != wihi ||
        fo % 64 != 0 || fi % 64 != 0 || !aligned16(mu_w))
        return 0;
    return conv2d_bwd_dw_stencil(mu_a, dmu, dvar, B, fo, woho, wihi, fi, ki, TILE_64x64);
}

// Both backward contractions of a layer for which conv2d_bwd_pair() holds: one launch for
// the two tile grids, then the folds of whichever is sliced. (z: state backward, 64 x 128
// tiles; w: weight backward, 64 x 64 tiles; workspaces of their own.)
hipError_t launch_conv2d_bwd_pair(const float *mu_w, const float *var_w, const float *mu_a,
                                  const float *jcb, const float *dmu, const float *dvar,
                                  const int *aidx, const int *zw_idx, const int *zud_idx, int B,
                                  int fo, int woho, int wihi, int fi, int ki, int nr, int splits_z,
                                  float *wz0, float *wz1, int splits_w, float *ww0, float *ww1,
                                  const float *res_mu, const float *res_var, int res_mode,
                                  float *out_dmu, float *out_dvar, float *dmu_w, float *dvar_w,
                                  hipStream_t stream) {
    int stencil = 0, s2_all = 0;
    ConvParams pz = dz_params(mu_w, jcb, dmu, dvar, zw_idx, zud_idx, woho, fo, wihi, fi, ki, nr, B,
                              TILE_64x128, out_dmu, out_dvar, res_mu, res_var, res_mode, &stencil,
                              &s2_all);
    ConvParams pw = dw_params(var_w, mu_a, dmu, dvar, aidx, B, fo, woho, wihi, fi, ki, dmu_w, dvar_w);
    const int width = conv2d_bwd_pair(mu_w, mu_a, dmu, dvar, B, fo, woho, wihi, fi, ki, nr);
    if (width == 0 || stencil != width) return hipErrorInvalidValue;
    plan_slices(pz, splits_z, 32 * pz.k2, wz0, wz1);
    plan_slices(pw, splits_w, 64, ww0, ww1);
    hipError_t e = launch_conv_stencil_bwd_pair(width, pz, pw, stream);
    if (e != hipSuccess) return e;
    if (pz.splits > 1) {
        e = launch_reduce_store<ConvDzProblem>(pz, stream);
        if (e != hipSuccess) return e;
    }
    if (pw.splits > 1)
        e = launch_reduce_splits(EPI_SCALE, ww0, ww1, pw.splits, pw.M, pw.N, var_w, nullptr, dmu_w,
                                 dvar_w, pw.N, stream);
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

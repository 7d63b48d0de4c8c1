// C ABI of the backend (include/tagi_hip.h): argument checks, kernel selection
// by shape, and the per-device workspace for split-reduction partial sums.
#include <cstdint>
#include <cstring>
#include <mutex>
#include <utility>
#include <vector>

#include "../../include/tagi_hip.h"
#include "../../include/tagi_hip_test_hooks.h"
#include "tagi_internal.h"

using namespace tagi;

// Device memory that exists from module load on, for tagi_linear_fwd_static. In
// host code the name is only a handle: the address that kernels, copies and
// memsets can use comes from hipGetSymbolAddress, once per device (every GPU
// holds its own copy of the array at its own address).
constexpr size_t STATIC_SCRATCH_BYTES = TAGI_LINEAR_FWD_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) float scratch[STATIC_SCRATCH_BYTES / sizeof(float)];

namespace {

constexpr int ABI_VERSION = 106;

#define TAGI_TRY(expr)                          \
    do {                                        \
        hipError_t _e = (expr);                 \
        if (_e != hipSuccess) return (int)_e;   \
    } while (0)

struct Workspace {
    float *ptr = nullptr;
    size_t bytes = 0;
};
// One grow-only workspace per (device, stream): partial sums stay in it between the
// launches of a call, so calls on different streams of a device must not share one.
// Calls on one stream are ordered by the stream and share theirs.
struct DeviceWorkspaces {
    std::vector<std::pair<hipStream_t, Workspace>> by_stream;
};
DeviceWorkspaces g_ws[MAX_DEVICES];
std::mutex g_ws_mutex;
int g_num_cu[MAX_DEVICES];

// Grow-only. Reallocation waits for the device, so buffers still in use by
// queued kernels are never freed under them.
int workspace_get(size_t bytes, hipStream_t stream, float **out) {
    int dev = 0;
    TAGI_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES) return TAGI_ERR_NO_DEVICE;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    Workspace *w = nullptr;
    for (auto &entry : g_ws[dev].by_stream)
        if (entry.first == stream) w = &entry.second;
    if (w == nullptr) {
        g_ws[dev].by_stream.emplace_back(stream, Workspace());
        w = &g_ws[dev].by_stream.back().second;
    }
    if (w->bytes < bytes) {
        TAGI_TRY(hipDeviceSynchronize());
        if (w->ptr != nullptr) TAGI_TRY(hipFree(w->ptr));
        w->ptr = nullptr;
        w->bytes = 0;
        const size_t want = (bytes + ((size_t)1 << 20) - 1) & ~(((size_t)1 << 20) - 1);
        TAGI_TRY(hipMalloc(reinterpret_cast<void **>(&w->ptr), want));
        w->bytes = want;
    }
    *out = w->ptr;
    return TAGI_OK;
}

// Where a call's partial sums go: the grow-only workspace above, or the static
// array of the entry point that allocates nothing.
typedef int (*ScratchSource)(size_t bytes, hipStream_t stream, float **out);

float *g_scratch_ptr[MAX_DEVICES];
std::mutex g_scratch_mutex;

int static_scratch_get(size_t bytes, hipStream_t, float **out) {
    if (bytes > STATIC_SCRATCH_BYTES) return TAGI_ERR_UNSUPPORTED;
    int dev = 0;
    TAGI_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= MAX_DEVICES) return TAGI_ERR_NO_DEVICE;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        float *p = nullptr;
        TAGI_TRY(hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(scratch)));
        if (p == nullptr) return TAGI_ERR_NO_DEVICE;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return TAGI_OK;
}

struct Tuning {
    int fwd_splits = -1;
    int dz_splits = -1;
    int dw_splits = -1;
    int gemv_max_batch = -1;
    int conv_dw_tile = -1;
    int conv_splits = -1;
    int conv_tile = -1;
    int tile = -1;
    int conv_dw_splits = -1;
    int gemv_swz = -1;
    int gemv_fwd_variant = -1;
    // bits 0-1: state backward, bits 2-3: weight backward; low bit of each pair:
    // walk rows from the end, high bit: XCD-aware column mapping
    int gemv_rev = -1;
    int gemv16 = -1;    // 0: 9..16 samples on the 4x4x1 kernels too
    int gemv16_min = -1;  // smallest batch the 16-wide forward takes (default 1)
    int wide32 = -1;    // 0: 17..32 samples on the tiled kernels; 2: state backward streams too
    int dw_side = -1;   // 0: bias innovations and the state-backward fold as launches of their own
    // >= 0: the smallest weight matrix (elements) the streaming kernels take, whatever the
    // batch; -1: the measured thresholds of streams_weights()
    long long stream_min_weights = -1;
    int small = -1;     // 0: small layers on the tiled / streaming kernels too
};
Tuning g_tune;

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

int pick_tile(int rows) {
    // tile ids: 0 = 128x128, 1 = 64x128, 2 = 32x128 (rows x columns)
    if (g_tune.tile >= 0 && g_tune.tile < gemm_tile_count()) return g_tune.tile;
    // 64x128 keeps the accumulators small enough for two workgroups per CU,
    // which measures faster than one 128x128 workgroup on every shape tried
    if (rows > 32) return 1;
    return 2;
}

// Reduction slices so that a launch reaches about two workgroups per CU (one where that
// takes more than eight slices), while every slice keeps at least `min_tiles` k-tiles of
// work.
int pick_splits(int tiles, int reduction, int forced, int min_tiles = 8) {
    const int kt = gemm_k_tile();
    const int k_tiles = ceil_div(reduction, kt);
    int s = forced > 0 ? forced : ceil_div(2 * num_cu(), tiles);
    // Beyond eight slices the partial sums cost more than the second workgroup per CU
    // gives: one per CU then (4096^2, forward + backward: batch 64 163 -> 156 us with 8
    // instead of 16 slices, batch 128 272 -> 270 us with 4 instead of 8; batch 256 and
    // 512 are faster with two per CU, 496 against 500 us and 947 against 958 us).
    if (forced <= 0 && s > 8) s = std::max(8, ceil_div(num_cu(), tiles));
    int cap = k_tiles / min_tiles > 0 ? k_tiles / min_tiles : 1;
    // A launch that leaves most of the chip empty is bound by the latency of its
    // k-tile loop (one memory round trip per k-tile, nothing else on the CU to hide
    // it), not by throughput: such a launch is cut into single k-tiles when its
    // reduction is long enough to pay for the fold (784 -> 128, batch 32: forward
    // 31 -> 12 us).
    if (tiles * 8 <= num_cu() && k_tiles >= 8) cap = k_tiles < 32 ? k_tiles : 32;
    if (forced <= 0 && s > cap) s = cap;
    if (s > k_tiles) s = k_tiles;
    if (s < 1) s = 1;
    return s;
}

// the streaming kernels hold at most 16 samples
int gemv_max_batch() {
    return g_tune.gemv_max_batch >= 0 && g_tune.gemv_max_batch < 16 ? g_tune.gemv_max_batch : 16;
}
// ... except the 16x16x4 forward, which also takes two groups of 16 (17..32 samples:
// twice the MFMA work per weight byte, still one pass over the weights). Measured against
// the tiled kernel at 4096^2: forward 35-37 us instead of 40-41 us for 17..32 samples. The
// state backward has the same two-group form but measured slower than the tiled kernel
// there (39 against 30 us at batch 32) and keeps to 16 samples. The knob that limits the
// streaming kernels limits these too.
int wide_max_batch() {
    if (g_tune.gemv_max_batch >= 0 && g_tune.gemv_max_batch < 16) return g_tune.gemv_max_batch;
    return g_tune.wide32 == 0 ? 16 : gemv16_max_batch();
}

// Whether a layer of n x k weights goes to the streaming kernels (one pass over the
// weights, activations resident in LDS) or to the tiled kernel. The streaming kernels win
// where reading the weights is what takes the time; on smaller layers a launch is bound by
// latency and the tiled kernel's many short slices finish sooner. Thresholds from kernel
// times at 128^2 .. 4096^2 (weights in elements):
//   forward        <= 16 samples: 4M (2048^2: 15.0 against 17-19 us; 2048 x 1024: 14.7-15.4
//                  against 13.7-15.1 us)
//                  17..32: 8M (4096 x 2048: 23.4 against 28 us; 2048^2: 21.6 against 21.0 us)
//   state backward <= 8 samples: 4M (4096^2: 19-22 against 28 us; 1024^2: 13-16 against 11 us)
//                  9..16: 2M (2048x1024: 13.5 against 14.4 us; 1024^2: 12.7 against 12.2 us)
enum StreamOp { STREAM_FWD, STREAM_DZ };
bool streams_weights(StreamOp op, int n, int k, int batch) {
    const long long weights = (long long)n * k;
    if (g_tune.stream_min_weights >= 0) return weights >= g_tune.stream_min_weights;
    const long long M = 1ll << 20;
    if (op == STREAM_FWD) return weights >= (batch <= 16 ? 4 * M : 8 * M);
    return weights >= (batch <= 8 ? 4 * M : 2 * M);
}

// the one-launch kernels for small layers, unless a test forces another path
bool use_small_kernels() { return g_tune.small != 0 && g_tune.stream_min_weights < 0; }

// Tile shape and reduction slices of a tiled launch.
void plan_gemm(GemmMode mode, GemmParams &p, int forced_splits, int *tile_out) {
    const int tile = pick_tile(p.M);
    const int tiles = ceil_div(p.M, gemm_tile_rows(tile)) * ceil_div(p.N, gemm_tile_cols(tile));
    const int kt = gemm_k_tile();
    int splits = (mode == GEMM_DW && forced_splits <= 0) ? 1
                                                          : pick_splits(tiles, p.R, forced_splits);
    const int per = ceil_div(ceil_div(p.R, splits), kt) * kt;
    p.splits = ceil_div(p.R, per);
    p.r_per_split = per;
    *tile_out = tile;
}

// Tiled MFMA launch + (when sliced) the fold of the partial sums. With `defer`
// given (state backward), a fold that the 16-byte path can do is left to a later
// kernel and described in *defer instead.
int run_gemm(GemmMode mode, GemmParams p, bool vec, int forced_splits, hipStream_t stream,
             DzFold *defer = nullptr, ScratchSource scratch_get = workspace_get) {
    int tile = 0;
    plan_gemm(mode, p, forced_splits, &tile);
    const int splits = p.splits;
    if (splits > 1) {
        float *ws = nullptr;
        const size_t part = (size_t)splits * p.M * p.N;
        int rc = scratch_get(2 * part * sizeof(float), stream, &ws);
        if (rc != TAGI_OK) return rc;
        p.ws0 = ws;
        p.ws1 = ws + part;
    }
    TAGI_TRY(launch_gemm(mode, tile, vec, p, stream));
    if (splits > 1) {
        const size_t total = (size_t)p.M * p.N;
        if (defer != nullptr && mode == GEMM_DZ && p.ldo == p.N && total % 4 == 0 &&
            aligned16(p.e0) && aligned16(p.out0) && aligned16(p.out1)) {
            defer->ws0 = p.ws0; defer->ws1 = p.ws1; defer->jcb = p.e0;
            defer->out0 = p.out0; defer->out1 = p.out1;
            defer->splits = splits; defer->total = total;
            return TAGI_OK;
        }
        TAGI_TRY(launch_reduce_splits(mode == GEMM_FWD ? EPI_BIAS : EPI_SCALE, p.ws0, p.ws1,
                                      splits, p.M, p.N, p.e0, p.e1, p.out0, p.out1, p.ldo,
                                      stream, p.act, p.out2));
    }
    return TAGI_OK;
}

}  // namespace

namespace tagi {
int num_cu() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return 256;
    if (g_num_cu[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
            n <= 0) {
            (void)hipGetLastError();
            n = 256;
        }
        g_num_cu[dev] = n;
    }
    return g_num_cu[dev];
}
}  // namespace tagi

extern "C" {

int tagi_hip_version(void) { return ABI_VERSION; }

int tagi_hip_device_count(int *count) {
    if (count == nullptr) return TAGI_ERR_INVALID_ARG;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        *count = 0;
        (void)hipGetLastError();
        return e == hipErrorNoDevice ? TAGI_OK : (int)e;
    }
    *count = n;
    return TAGI_OK;
}

const char *tagi_hip_error_string(int code) {
    switch (code) {
        case TAGI_OK: return "ok";
        case TAGI_ERR_INVALID_ARG: return "tagi: invalid argument";
        case TAGI_ERR_UNSUPPORTED: return "tagi: unsupported shape";
        case TAGI_ERR_NO_DEVICE: return "tagi: no usable device";
        default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "tagi: unknown error";
}

int tagi_hip_workspace_reserve(size_t bytes, void *stream) {
    float *p = nullptr;
    return workspace_get(bytes, static_cast<hipStream_t>(stream), &p);
}

int tagi_hip_device_info(int *compute_units, int *clock_mhz, char *name, size_t name_capacity) {
    int dev = 0;
    TAGI_TRY(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    TAGI_TRY(hipGetDeviceProperties(&prop, dev));
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (clock_mhz) *clock_mhz = prop.clockRate / 1000;
    if (name && name_capacity > 0) {
        strncpy(name, prop.name, name_capacity - 1);
        name[name_capacity - 1] = '\0';
    }
    return TAGI_OK;
}

int tagi_hip_shutdown(void) {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    int cur = 0;
    if (hipGetDevice(&cur) != hipSuccess) return TAGI_OK;
    for (int d = 0; d < MAX_DEVICES; d++) {
        if (g_ws[d].by_stream.empty()) continue;
        TAGI_TRY(hipSetDevice(d));
        TAGI_TRY(hipDeviceSynchronize());
        for (auto &entry : g_ws[d].by_stream)
            if (entry.second.ptr != nullptr) TAGI_TRY(hipFree(entry.second.ptr));
        g_ws[d].by_stream.clear();
    }
    TAGI_TRY(hipSetDevice(cur));
    return TAGI_OK;
}

int tagi_hip_tune(const char *key, int value) {
    if (key == nullptr) return TAGI_ERR_INVALID_ARG;
    if (!strcmp(key, "linear.fwd.splits")) g_tune.fwd_splits = value;
    else if (!strcmp(key, "linear.dz.splits")) g_tune.dz_splits = value;
    else if (!strcmp(key, "linear.dw.splits")) g_tune.dw_splits = value;
    else if (!strcmp(key, "linear.gemv_max_batch")) g_tune.gemv_max_batch = value;
    else if (!strcmp(key, "conv2d.dw.tile")) g_tune.conv_dw_tile = value;
    else if (!strcmp(key, "conv2d.splits")) g_tune.conv_splits = value;
    else if (!strcmp(key, "conv2d.tile")) g_tune.conv_tile = value;
    else if (!strcmp(key, "conv2d.group_loads")) g_conv2d_group_loads = value;
    else if (!strcmp(key, "conv2d.stencil")) g_conv2d_stencil = value;
    else if (!strcmp(key, "conv2d.phase_order")) g_conv2d_phase_order = value;
    else if (!strcmp(key, "conv2d.s2_all")) g_conv2d_s2_all = value < 0 ? 1 : value;
    else if (!strcmp(key, "conv2d.bwd_pair")) g_conv2d_bwd_pair = value < 0 ? 1 : value;
    else if (!strcmp(key, "batchnorm.fused_train")) g_bn_fused_train = value < 0 ? 1 : value;
    else if (!strcmp(key, "linear.tile")) g_tune.tile = value;
    else if (!strcmp(key, "linear.double_buffer")) g_gemm_double_buffer = value < 0 ? 1 : value;
    else if (!strcmp(key, "conv2d.dw.splits")) g_tune.conv_dw_splits = value;
    else if (!strcmp(key, "linear.gemv.swizzle")) g_tune.gemv_swz = value;
    else if (!strcmp(key, "linear.gemv.fwd_variant")) g_tune.gemv_fwd_variant = value;
    else if (!strcmp(key, "linear.gemv.reverse")) g_tune.gemv_rev = value;
    else if (!strcmp(key, "linear.dw_side")) g_tune.dw_side = value;
    else if (!strcmp(key, "linear.gemv16")) g_tune.gemv16 = value;
    else if (!strcmp(key, "linear.gemv16.min_batch")) g_tune.gemv16_min = value;
    else if (!strcmp(key, "linear.gemv32")) g_tune.wide32 = value;
    else if (!strcmp(key, "linear.gemv16.fwd_waves")) g_gemv16_fwd_waves = value;
    else if (!strcmp(key, "linear.gemv16.whole_lines")) g_gemv16_fwd_whole_lines = value;
    else if (!strcmp(key, "linear.stream_min_weights")) g_tune.stream_min_weights = value;
    else if (!strcmp(key, "linear.small")) g_tune.small = value;
    else return TAGI_ERR_INVALID_ARG;
    return TAGI_OK;
}

// ---------------------------------------------------------------------------
// Linear
// ---------------------------------------------------------------------------

static int linear_fwd_impl(const float *mu_w, const float *var_w, const float *mu_b,
                           const float *var_b, const float *mu_a, const float *var_a, int K, int N,
                           int B, int bias, float *mu_z, float *var_z, void *stream_,
                           ScratchSource scratch_get, int act = 0, float *jcb = nullptr) {
    if (act < 0 || act > 2 || (act != 0 && jcb == nullptr)) return TAGI_ERR_INVALID_ARG;
    if (!mu_w || !var_w || !mu_a || !var_a || !mu_z || !var_z) return TAGI_ERR_INVALID_ARG;
    if (K <= 0 || N <= 0 || B <= 0) return TAGI_ERR_INVALID_ARG;
    if (bias && (!mu_b || !var_b)) return TAGI_ERR_INVALID_ARG;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const float *e0 = bias ? mu_b : nullptr, *e1 = bias ? var_b : nullptr;
    const bool vec = (K % 4 == 0) && aligned16(mu_w) && aligned16(var_w) && aligned16(mu_a) &&
                     aligned16(var_a);

    if (vec && use_small_kernels() && small_fwd_supported(K, N, B)) {
        // small layers: one launch, bias and activation included
        TAGI_TRY(launch_small_fwd(mu_w, var_w, e0, e1, mu_a, var_a, K, N, B, act, mu_z, var_z, jcb,
                                  stream));
        return TAGI_OK;
    }
    const bool streams = streams_weights(STREAM_FWD, N, K, B);
    if (B >= (g_tune.gemv16_min > 0 ? g_tune.gemv16_min : 1) && B <= wide_max_batch() && vec &&
        g_tune.gemv16 != 0 && streams) {
        // 9..32 samples: the 16-wide streaming kernel (two sample groups beyond 16)
        const int blocks = ceil_div(N, gemv16_fwd_rows_per_block(N, K, B));
        const int step = gemv16_fwd_k_step();
        int splits = g_tune.fwd_splits > 0 ? g_tune.fwd_splits : ceil_div(2 * num_cu(), blocks);
        const int max_splits = ceil_div(K, 4 * step);
        if (splits > max_splits) splits = max_splits;
        const int min_splits = ceil_div(K, gemv16_fwd_max_slice(B));
        if (splits < min_splits) splits = min_splits;
        const int per = ceil_div(ceil_div(K, splits), step) * step;
        splits = ceil_div(K, per);
        float *ws = nullptr;
        const size_t part = (size_t)splits * B * N;
        int rc = scratch_get(2 * part * sizeof(float), stream, &ws);
        if (rc != TAGI_OK) return rc;
        TAGI_TRY(launch_gemv16_fwd(mu_w, var_w, mu_a, var_a, K, N, B, per, splits, ws, ws + part,
                                   stream));
        TAGI_TRY(launch_reduce_splits(EPI_BIAS, ws, ws + part, splits, B, N, e0, e1, mu_z, var_z, N,
                                      stream, act, jcb));
        return TAGI_OK;
    }

    if (B <= gemv_max_batch() && vec && streams) {
        // slices: short enough for the LDS-resident activations, and enough of
        // them for about two workgroups per CU
        const int variant = (g_tune.gemv_fwd_variant >= 0 &&
                             g_tune.gemv_fwd_variant < gemv_fwd_variants())
                                ? g_tune.gemv_fwd_variant
                                : 0;
        const int blocks = ceil_div(N, gemv_fwd_rows_per_block(variant));
        const int step = gemv_fwd_k_step();
        int splits = g_tune.fwd_splits > 0 ? g_tune.fwd_splits : ceil_div(2 * num_cu(), blocks);
        const int max_splits = ceil_div(K, 4 * step);
        if (splits > max_splits) splits = max_splits;
        const int min_splits = ceil_div(K, gemv_fwd_max_slice(B));
        if (splits < min_splits) splits = min_splits;
        int per = ceil_div(ceil_div(K, splits), step) * step;
        splits = ceil_div(K, per);
        float *ws = nullptr;
        const size_t part = (size_t)splits * B * N;
        int rc = scratch_get(2 * part * sizeof(float), stream, &ws);
        if (rc != TAGI_OK) return rc;
        TAGI_TRY(launch_gemv_fwd(mu_w, var_w, mu_a, var_a, K, N, B, splits,
                                 g_tune.gemv_swz >= 0 ? g_tune.gemv_swz : 3, variant, ws,
                                 ws + part, stream));
        TAGI_TRY(launch_reduce_splits(EPI_BIAS, ws, ws + part, splits, B, N, e0, e1, mu_z, var_z, N,
                                      stream, act, jcb));
        return TAGI_OK;
    }

    GemmParams p = {};
    p.x0 = mu_a; p.x1 = var_a; p.y0 = mu_w; p.y1 = var_w;
    p.M = B; p.N = N; p.R = K; p.ldx = K; p.ldy = K;
    p.out0 = mu_z; p.out1 = var_z; p.ldo = N;
    p.e0 = e0; p.e1 = e1;
    p.act = act; p.out2 = jcb;
    return run_gemm(GEMM_FWD, p, vec, g_tune.fwd_splits, stream, nullptr, scratch_get);
}

int tagi_linear_fwd(const float *mu_w, const float *var_w, const float *mu_b, const float *var_b,
                    const float *mu_a, const float *var_a, int K, int N, int B, int bias,
                    float *mu_z, float *var_z, void *stream) {
    return linear_fwd_impl(mu_w, var_w, mu_b, var_b, mu_a, var_a, K, N, B, bias, mu_z, var_z,
                           stream, workspace_get);
}

int tagi_linear_fwd_act(const float *mu_w, const float *var_w, const float *mu_b,
                        const float *var_b, const float *mu_a, const float *var_a, int K, int N,
                        int B, int bias, int activation, float *mu_out, float *var_out,
                        float *jcb_out, void *stream) {
    if (activation != TAGI_ACT_RELU && activation != TAGI_ACT_MIXTURE_RELU)
        return TAGI_ERR_INVALID_ARG;
    return linear_fwd_impl(mu_w, var_w, mu_b, var_b, mu_a, var_a, K, N, B, bias, mu_out, var_out,
                           stream, workspace_get, activation, jcb_out);
}

int tagi_linear_fwd_static(const float *mu_w, const float *var_w, const float *mu_b,
                           const float *var_b, const float *mu_a, const float *var_a, int K,
                           int N, int B, int bias, float *mu_z, float *var_z, void *stream) {
    return linear_fwd_impl(mu_w, var_w, mu_b, var_b, mu_a, var_a, K, N, B, bias, mu_z, var_z,
                           stream, static_scratch_get);
}

// State backward; with `defer` given and the skinny-batch kernel running, the
// slices are left unfolded and described in *defer for a later kernel to fold.
static int linear_bwd_dz_impl(const float *mu_w, const float *jcb, const float *delta_mu,
                              const float *delta_var, int K, int N, int B, float *delta_mu_z,
                              float *delta_var_z, DzFold *defer, void *stream_) {
    if (!mu_w || !jcb || !delta_mu || !delta_var || !delta_mu_z || !delta_var_z)
        return TAGI_ERR_INVALID_ARG;
    if (K <= 0 || N <= 0 || B <= 0) return TAGI_ERR_INVALID_ARG;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const bool vec = (K % 4 == 0) && (N % 4 == 0) && aligned16(mu_w) && aligned16(delta_mu) &&
                     aligned16(delta_var);

    const bool wide16 = B > 8 && B <= (g_tune.wide32 == 2 ? wide_max_batch() : gemv_max_batch()) &&
                        g_tune.gemv16 != 0;
    if (use_small_kernels() && K % 4 == 0 && aligned16(mu_w) && small_bwd_supported(K, N, B)) {
        TAGI_TRY(launch_small_dz(mu_w, jcb, delta_mu, delta_var, K, N, B, delta_mu_z, delta_var_z,
                                 stream));
        return TAGI_OK;
    }
    if ((B <= gemv_max_batch() || wide16) && vec && streams_weights(STREAM_DZ, N, K, B)) {
        const int blocks = ceil_div(K, wide16 ? gemv16_dz_cols_per_block() : gemv_dz_cols_per_block());
        const int step = wide16 ? gemv16_dz_n_step() : gemv_dz_n_step();
        int splits = g_tune.dz_splits > 0 ? g_tune.dz_splits : ceil_div(num_cu(), blocks);
        const int max_splits = ceil_div(N, 2 * step);
        if (splits > max_splits) splits = max_splits;
        const int min_splits = ceil_div(N, wide16 ? gemv16_dz_max_slice(B) : gemv_dz_max_slice(B));
        if (splits < min_splits) splits = min_splits;
        int per = ceil_div(ceil_div(N, splits), step) * step;
        splits = ceil_div(N, per);
        float *ws = nullptr;
        const size_t part = (size_t)splits * B * K;
        int rc = workspace_get(2 * part * sizeof(float), stream, &ws);
        if (rc != TAGI_OK) return rc;
        if (wide16)
            TAGI_TRY(launch_gemv16_dz(mu_w, delta_mu, delta_var, K, N, B, per, splits, ws,
                                      ws + part, stream));
        else
            TAGI_TRY(launch_gemv_dz(mu_w, delta_mu, delta_var, K, N, B, splits,
                                    (g_tune.gemv_rev >= 0 ? g_tune.gemv_rev : 0) & 3, ws,
                                    ws + part, stream));
        if (defer != nullptr && aligned16(jcb) && aligned16(delta_mu_z) && aligned16(delta_var_z)) {
            defer->ws0 = ws; defer->ws1 = ws + part; defer->jcb = jcb;
            defer->out0 = delta_mu_z; defer->out1 = delta_var_z;
            defer->splits = splits; defer->total = (size_t)B * K;
            return TAGI_OK;
        }
        TAGI_TRY(launch_reduce_splits(EPI_SCALE, ws, ws + part, splits, B, K, jcb, nullptr,
                                      delta_mu_z, delta_var_z, K, stream));
        return TAGI_OK;
    }

    GemmParams p = {};
    p.x0 = delta_mu; p.x1 = delta_var; p.y0 = mu_w; p.y1 = nullptr;
    p.M = B; p.N = K; p.R = N; p.ldx = N; p.ldy = K;
    p.out0 = delta_mu_z; p.out1 = delta_var_z; p.ldo = K;
    p.e0 = jcb; p.e1 = nullptr;
    return run_gemm(GEMM_DZ, p, vec, g_tune.dz_splits, stream, defer);
}

int tagi_linear_bwd_dz(const float *mu_w, const float *jcb, const float *delta_mu,
                       const float *delta_var, int K, int N, int B, float *delta_mu_z,
                       float *delta_var_z, void *stream) {
    return linear_bwd_dz_impl(mu_w, jcb, delta_mu, delta_var, K, N, B, delta_mu_z, delta_var_z,
                              nullptr, stream);
}

// Weight backward; when the bias pointers are given and the skinny-batch kernel
// runs, that kernel also writes the bias innovations and *bias_done is set.
static int linear_bwd_dw_impl(const float *var_w, const float *mu_a, const float *delta_mu,
                              const float *delta_var, int K, int N, int B, float *delta_mu_w,
                              float *delta_var_w, const float *var_b, float *delta_mu_b,
                              float *delta_var_b, bool *bias_done, const DzFold *fold,
                              bool *fold_done, void *stream_) {
    if (!var_w || !mu_a || !delta_mu || !delta_var || !delta_mu_w || !delta_var_w)
        return TAGI_ERR_INVALID_ARG;
    if (K <= 0 || N <= 0 || B <= 0) return TAGI_ERR_INVALID_ARG;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const bool k_vec = (K % 4 == 0) && aligned16(mu_a) && aligned16(var_w) &&
                       aligned16(delta_mu_w) && aligned16(delta_var_w);

    if (use_small_kernels() && k_vec && fold == nullptr && small_dw_supported(K, N, B)) {
        TAGI_TRY(launch_small_dw(var_w, mu_a, delta_mu, delta_var, K, N, B, delta_mu_w, delta_var_w,
                                 var_b, delta_mu_b, delta_var_b, stream));
        if (bias_done) *bias_done = var_b != nullptr;
        return TAGI_OK;
    }
    if (B <= gemv_max_batch() && k_vec) {
        TAGI_TRY(launch_gemv_dw(var_w, mu_a, delta_mu, delta_var, K, N, B,
                                ((g_tune.gemv_rev >= 0 ? g_tune.gemv_rev : 0) >> 2) & 3,
                                delta_mu_w, delta_var_w, var_b, delta_mu_b, delta_var_b, fold,
                                stream));
        if (bias_done) *bias_done = var_b != nullptr;
        if (fold_done) *fold_done = fold != nullptr;
        return TAGI_OK;
    }

    const bool vec = k_vec && (N % 4 == 0) && aligned16(delta_mu) && aligned16(delta_var);
    GemmParams p = {};
    p.x0 = delta_mu; p.x1 = delta_var; p.y0 = mu_a; p.y1 = nullptr;
    p.M = N; p.N = K; p.R = B; p.ldx = N; p.ldy = K;
    p.out0 = delta_mu_w; p.out1 = delta_var_w; p.ldo = K;
    p.e0 = var_w; p.e1 = nullptr;
    // The bias innovations and a pending fold of the state backward ride along
    // with an unsliced tile launch (its first workgroups do them).
    GemmParams q = p;
    int tile = 0;
    plan_gemm(GEMM_DW, q, g_tune.dw_splits, &tile);
    const bool want_bias = var_b != nullptr && bias_done != nullptr;
    const bool want_fold = fold != nullptr && fold_done != nullptr;
    if (want_fold && q.splits > 1) {
        // a sliced weight backward takes the workspace the pending slices lie in
        TAGI_TRY(launch_reduce_splits(EPI_SCALE, fold->ws0, fold->ws1, fold->splits,
                                      (int)(fold->total / K), K, fold->jcb, nullptr, fold->out0,
                                      fold->out1, K, stream));
        *fold_done = true;
    } else if ((want_bias || want_fold) && g_tune.dw_side != 0 &&
               gemm_dw_side_supported(tile, vec, q)) {
        LinearSideWork w;
        if (want_fold) {
            w.ws0 = fold->ws0; w.ws1 = fold->ws1; w.jcb = fold->jcb;
            w.out0 = fold->out0; w.out1 = fold->out1;
            w.fold_splits = fold->splits; w.fold_total = fold->total;
        }
        if (want_bias) {
            w.var_b = var_b; w.dmu = delta_mu; w.dvar = delta_var;
            w.dmu_b = delta_mu_b; w.dvar_b = delta_var_b;
            w.bias_n = N; w.bias_b = B;
        }
        TAGI_TRY(launch_gemm_dw_side(q, w, stream));
        if (want_bias) *bias_done = true;
        if (want_fold) *fold_done = true;
        return TAGI_OK;
    }
    return run_gemm(GEMM_DW, p, vec, g_tune.dw_splits, stream);
}

int tagi_linear_bwd_dw(const float *var_w, const float *mu_a, const float *delta_mu,
                       const float *delta_var, int K, int N, int B, float *delta_mu_w,
                       float *delta_var_w, void *stream) {
    return linear_bwd_dw_impl(var_w, mu_a, delta_mu, delta_var, K, N, B, delta_mu_w, delta_var_w,
                              nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, stream);
}

int tagi_linear_bwd_db(const float *var_b, const float *delta_mu, const float *delta_var, int N,
                       int B, float *delta_mu_b, float *delta_var_b, void *stream_) {
    if (!var_b || !delta_mu || !delta_var || !delta_mu_b || !delta_var_b)
        return TAGI_ERR_INVALID_ARG;
    if (N <= 0 || B <= 0) return TAGI_ERR_INVALID_ARG;
    TAGI_TRY(launch_bias_delta(var_b, delta_mu, delta_var, N, B, delta_mu_b, delta_var_b,
                               static_cast<hipStream_t>(stream_)));
    return TAGI_OK;
}

int tagi_linear_bwd(const float *mu_w, const float *var_w, const float *var_b, const float *mu_a,
                    const float *jcb, const float *delta_mu, const float *delta_var, int K, int N,
                    int B, int bias, int state_update, int param_update, float *delta_mu_z,
                    float *delta_var_z, float *delta_mu_w, float *delta_var_w, float *delta_mu_b,
                    float *delta_var_b, void *stream) {
    int rc = TAGI_OK;
    if (param_update && bias && (!var_b || !delta_mu_b || !delta_var_b))
        return TAGI_ERR_INVALID_ARG;
    if (state_update && param_update && use_small_kernels() && g_tune.dw_side != 0 && mu_w && var_w &&
        mu_a && jcb && delta_mu && delta_var && delta_mu_z && delta_var_z && delta_mu_w &&
        delta_var_w && K > 0 && N > 0 && B > 0 && K % 4 == 0 && aligned16(mu_w) && aligned16(mu_a) &&
        aligned16(var_w) && aligned16(delta_mu_w) && aligned16(delta_var_w) &&
        small_bwd_supported(K, N, B) && small_dw_supported(K, N, B)) {
        // a small layer: both contractions (and the bias innovations) in one launch
        TAGI_TRY(launch_small_bwd_pair(mu_w, var_w, mu_a, jcb, delta_mu, delta_var, K, N, B,
                                       delta_mu_z, delta_var_z, delta_mu_w, delta_var_w,
                                       bias ? var_b : nullptr, delta_mu_b, delta_var_b,
                                       static_cast<hipStream_t>(stream)));
        return TAGI_OK;
    }
    DzFold fold;
    if (state_update) {
        rc = linear_bwd_dz_impl(mu_w, jcb, delta_mu, delta_var, K, N, B, delta_mu_z, delta_var_z,
                                param_update ? &fold : nullptr, stream);
        if (rc != TAGI_OK) return rc;
    }
    const bool pending = fold.ws0 != nullptr;
    bool fold_done = false;
    if (param_update) {
        bool bias_done = false;
        rc = linear_bwd_dw_impl(var_w, mu_a, delta_mu, delta_var, K, N, B, delta_mu_w, delta_var_w,
                                bias ? var_b : nullptr, delta_mu_b, delta_var_b, &bias_done,
                                pending ? &fold : nullptr, &fold_done, stream);
        if (rc != TAGI_OK) return rc;
        if (bias && !bias_done) {
            rc = tagi_linear_bwd_db(var_b, delta_mu, delta_var, N, B, delta_mu_b, delta_var_b,
                                    stream);
            if (rc != TAGI_OK) return rc;
        }
    }
    if (pending && !fold_done) {  // the weight backward took the tiled path: fold here
        TAGI_TRY(launch_reduce_splits(EPI_SCALE, fold.ws0, fold.ws1, fold.splits, B, K, fold.jcb,
                                      nullptr, fold.out0, fold.out1, K,
                                      static_cast<hipStream_t>(stream)));
    }
    return rc;
}

// ---------------------------------------------------------------------------
// Conv2d
// ---------------------------------------------------------------------------

// The conv kernels keep element offsets inside one tensor in 32 bits and stage a
// per-tap table of 128 columns in LDS.
static bool conv_sizes_ok(int B, int fo, int woho, int fi, int wihi, int ki) {
    const long long lim = 0x7fffffffLL;
    return (long long)B * fo * woho < lim && (long long)B * fi * wihi < lim &&
           (long long)ki * ki * fi * fo < lim && (long long)ki * ki * (128 + 32 + 1) * 4 + 48 <= 64 * 1024;
}

int tagi_conv2d_out_size(int kernel, int stride, int wi, int hi, int pad, int pad_type, int *wo,
                         int *ho) {
    if (!wo || !ho) return TAGI_ERR_INVALID_ARG;
    return conv2d_out_size(kernel, stride, wi, hi, pad, pad_type, wo, ho) == 0
               ? TAGI_OK
               : TAGI_ERR_INVALID_ARG;
}

int tagi_conv2d_build_idx(int kernel, int stride, int wi, int hi, int pad, int pad_type,
                          int param_pad_idx, int *Fmwa_2, int *FCzwa_1, int *Szz_ud, int *w,
                          int *h) {
    if (!Fmwa_2 || !FCzwa_1 || !Szz_ud || !w || !h) return TAGI_ERR_INVALID_ARG;
    return conv2d_build_idx(kernel, stride, wi, hi, pad, pad_type, param_pad_idx, Fmwa_2, FCzwa_1,
                            Szz_ud, w, h) == 0
               ? TAGI_OK
               : TAGI_ERR_INVALID_ARG;
}

static int conv2d_fwd_impl(const float *mu_w, const float *var_w, const float *mu_b,
                           const float *var_b, const float *mu_a, const float *var_a,
                           const int *aidx, int woho, int fo, int wihi, int fi, int ki, int B,
                           int bias, float *mu_z, float *var_z, void *stream_, int act,
                           float *jcb) {
    if (act < 0 || act > 2 || (act != 0 && jcb == nullptr)) return TAGI_ERR_INVALID_ARG;
    if (!mu_w || !var_w || !mu_a || !var_a || !aidx || !mu_z || !var_z)
        return TAGI_ERR_INVALID_ARG;
    if (woho <= 0 || fo <= 0 || wihi <= 0 || fi <= 0 || ki <= 0 || B <= 0)
        return TAGI_ERR_INVALID_ARG;
    if (bias && (!mu_b || !var_b)) return TAGI_ERR_INVALID_ARG;
    if (!conv_sizes_ok(B, fo, woho, fi, wihi, ki)) return TAGI_ERR_UNSUPPORTED;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    int tile = 0, splits = 1;
    conv2d_plan(fo, B * woho, ki * ki * fi, &tile, &splits);
    if (g_tune.conv_splits > 0) splits = g_tune.conv_splits;
    if (g_tune.conv_tile >= 0 && g_tune.conv_tile < gemm_tile_count()) tile = g_tune.conv_tile;
    float *ws = nullptr;
    const size_t part = splits > 1 ? (size_t)splits * fo * B * woho : 0;
    if (part) {
        int rc = workspace_get(2 * part * sizeof(float), stream, &ws);
        if (rc != TAGI_OK) return rc;
    }
    TAGI_TRY(launch_conv2d_fwd(mu_w, var_w, mu_b, var_b, mu_a, var_a, aidx, woho, fo, wihi, fi, ki,
                               B, bias, tile, splits, ws, ws + part, mu_z, var_z, stream, act,
                               jcb));
    return TAGI_OK;
}

int tagi_conv2d_fwd(const float *mu_w, const float *var_w, const float *mu_b, const float *var_b,
                    const float *mu_a, const float *var_a, const int *aidx, int woho, int fo,
                    int wihi, int fi, int ki, int B, int bias, float *mu_z, float *var_z,
                    void *stream) {
    return conv2d_fwd_impl(mu_w, var_w, mu_b, var_b, mu_a, var_a, aidx, woho, fo, wihi, fi, ki, B,
                           bias, mu_z, var_z, stream, 0, nullptr);
}

int tagi_conv2d_fwd_act(const float *mu_w, const float *var_w, const float *mu_b,
                        const float *var_b, const float *mu_a, const float *var_a,
                        const int *aidx, int woho, int fo, int wihi, int fi, int ki, int B,
                        int bias, int activation, float *mu_out, float *var_out, float *jcb_out,
                        void *stream) {
    if (activation != TAGI_ACT_RELU && activation != TAGI_ACT_MIXTURE_RELU)
        return TAGI_ERR_INVALID_ARG;
    return conv2d_fwd_impl(mu_w, var_w, mu_b, var_b, mu_a, var_a, aidx, woho, fo, wihi, fi, ki, B,
                           bias, mu_out, var_out, stream, activation, jcb_out);
}

static int conv2d_bwd_dz_impl(const float *mu_w, const float *jcb, const float *delta_mu_out,
                       const float *delta_var_out, const int *zw_idx, const int *zud_idx, int woho,
                       int fo, int wihi, int fi, int ki, int nr, int B, float *delta_mu,
                       float *delta_var, void *stream_, const float *res_mu,
                              const float *res_var, int res_mode) {
    if (!mu_w || !jcb || !delta_mu_out || !delta_var_out || !zw_idx || !zud_idx || !delta_mu ||
        !delta_var)
        return TAGI_ERR_INVALID_ARG;
    if (woho <= 0 || fo <= 0 || wihi <= 0 || fi <= 0 || ki <= 0 || nr <= 0 || B <= 0)
        return TAGI_ERR_INVALID_ARG;
    if (!conv_sizes_ok(B, fo, woho, fi, wihi, ki)) return TAGI_ERR_UNSUPPORTED;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    int tile = 0, splits = 1;
    conv2d_plan(fi, B * wihi, ki * ki * fo, &tile, &splits);
    // A strided layer's tiles differ in length by the phase of their pixels (a 3x3
    // stride-2 kernel: 4, 2, 2 or 1 taps). When they fill the chip exactly once, the
    // launch lasts as long as its longest tiles while most CUs idle; three slices make
    // enough shorter units to even that out (128 -> 256 channels at 16x16, batch 128:
    // 238 -> 174 us including the fold).
    if (splits == 1 && ki > 2 && wihi > woho && wihi % woho == 0 && g_conv2d_phase_order != 0) {
        const int tiles = ceil_div(fi, gemm_tile_rows(tile)) * ceil_div(B * wihi, gemm_tile_cols(tile));
        if (tiles >= 2 * num_cu() && tiles < 4 * num_cu() && ki * ki * fo >= 3 * 8 * gemm_k_tile())
            splits = 3;
    }
    if (conv2d_bwd_dz_s2_all(mu_w, delta_mu_out, delta_var_out, B, fo, woho, wihi, fi, ki, nr)) {
        // all four phases of a pixel block in one workgroup, one workgroup per CU
        tile = 1;  // 64 x 128 (tile ids as in pick_tile)
        splits = conv2d_bwd_dz_s2_all_splits(B, fo, woho, fi);
    }
    if (g_tune.conv_splits > 0) splits = g_tune.conv_splits;
    if (g_tune.conv_tile >= 0 && g_tune.conv_tile < gemm_tile_count()) tile = g_tune.conv_tile;
    float *ws = nullptr;
    const size_t part = splits > 1 ? (size_t)splits * fi * B * wihi : 0;
    if (part) {
        int rc = workspace_get(2 * part * sizeof(float), stream, &ws);
        if (rc != TAGI_OK) return rc;
    }
    TAGI_TRY(launch_conv2d_bwd_dz(mu_w, jcb, delta_mu_out, delta_var_out, zw_idx, zud_idx, woho,
                                  fo, wihi, fi, ki, nr, B, tile, splits, ws, ws + part, delta_mu,
                                  delta_var, stream, res_mu, res_var, res_mode));
    return TAGI_OK;
}

int tagi_conv2d_bwd_dz(const float *mu_w, const float *jcb, const float *delta_mu_out,
                       const float *delta_var_out, const int *zw_idx, const int *zud_idx, int woho,
                       int fo, int wihi, int fi, int ki, int nr, int B, float *delta_mu,
                       float *delta_var, void *stream) {
    return conv2d_bwd_dz_impl(mu_w, jcb, delta_mu_out, delta_var_out, zw_idx, zud_idx, woho, fo,
                              wihi, fi, ki, nr, B, delta_mu, delta_var, stream, nullptr, nullptr, 0);
}

int tagi_conv2d_bwd_dz_res(const float *mu_w, const float *jcb, const float *delta_mu_out,
                           const float *delta_var_out, const int *zw_idx, const int *zud_idx,
                           int woho, int fo, int wihi, int fi, int ki, int nr, int B,
                           const float *res_mu, const float *res_var, int res_mode,
                           float *delta_mu, float *delta_var, void *stream) {
    if (!res_mu || !res_var || (res_mode != 1 && res_mode != 2)) return TAGI_ERR_INVALID_ARG;
    return conv2d_bwd_dz_impl(mu_w, jcb, delta_mu_out, delta_var_out, zw_idx, zud_idx, woho, fo,
                              wihi, fi, ki, nr, B, delta_mu, delta_var, stream, res_mu, res_var,
                              res_mode);
}

int tagi_conv2d_bwd_dw(const float *var_w, const float *var_b, const float *mu_a,
                       const float *delta_mu_out, const float *delta_var_out, const int *aidx,
                       int B, int fo, int woho, int wihi, int fi, int ki, int bias,
                       float *delta_mu_w, float *delta_var_w, float *delta_mu_b,
                       float *delta_var_b, void *stream_) {
    if (!var_w || !mu_a || !delta_mu_out || !delta_var_out || !aidx || !delta_mu_w ||
        !delta_var_w)
        return TAGI_ERR_INVALID_ARG;
    if (woho <= 0 || fo <= 0 || wihi <= 0 || fi <= 0 || ki <= 0 || B <= 0)
        return TAGI_ERR_INVALID_ARG;
    if (bias && (!var_b || !delta_mu_b || !delta_var_b)) return TAGI_ERR_INVALID_ARG;
    if (!conv_sizes_ok(B, fo, woho, fi, wihi, ki)) return TAGI_ERR_UNSUPPORTED;
    hipStream_t stream = static_cast<hipStream_t>(stream_);

    // The reduction runs over all B*woho output positions while the result is
    // only fo x (ki*ki*fi): slice the reduction to fill the GPU.
    const int red = B * woho;
    const int tile = (g_tune.conv_dw_tile >= 0 && g_tune.conv_dw_tile < gemm_tile_count())
                         ? g_tune.conv_dw_tile
                         : 3;  // 64 x 64
    const int out_tiles =
        ceil_div(fo, gemm_tile_rows(tile)) * ceil_div(ki * ki * fi, gemm_tile_cols(tile));
    // (three full rounds of resident workgroups: a partly filled last round
    // costs as much time as a full one)
    const bool stencil = conv2d_bwd_dw_stencil(mu_a, delta_mu_out, delta_var_out, B, fo, woho, wihi,
                                               fi, ki, tile) != 0 ||
                         conv2d_bwd_dw_s2(mu_a, delta_mu_out, delta_var_out, B, fo, woho, wihi, fi,
                                          ki, tile) != 0;
    int splits = g_tune.conv_dw_splits > 0 ? g_tune.conv_dw_splits
                 : stencil                 ? conv2d_bwd_dw_stencil_splits(out_tiles)
                                           : 3 * conv2d_bwd_dw_blocks_per_cu(tile) * num_cu() / out_tiles;
    const int max_splits = ceil_div(red, 256);
    if (splits > max_splits) splits = max_splits;
    if (splits < 1) splits = 1;
    float *ws = nullptr;
    const size_t part = (size_t)splits * fo * ki * ki * fi;
    const int chunks = 64;  // slices of the (b, o) range in the bias reduction
    int rc = workspace_get((2 * part + 2 * (size_t)chunks * fo) * sizeof(float), stream, &ws);
    if (rc != TAGI_OK) return rc;
    TAGI_TRY(launch_conv2d_bwd_dw(var_w, mu_a, delta_mu_out, delta_var_out, aidx, B, fo, woho, wihi,
                                  fi, ki, tile, splits, ws, ws + part, delta_mu_w, delta_var_w, stream));
    if (bias) {
        TAGI_TRY(launch_conv2d_bwd_db(var_b, delta_mu_out, delta_var_out, B, fo, woho, chunks,
                                      ws + 2 * part, delta_mu_b, delta_var_b, stream));
    }
    return TAGI_OK;
}

int tagi_conv2d_bwd(const float *mu_w, const float *var_w, const float *var_b, const float *mu_a,
                    const float *jcb, const float *delta_mu_out, const float *delta_var_out,
                    const int *aidx, const int *zw_idx, const int *zud_idx, int B, int fo, int woho,
                    int wihi, int fi, int ki, int nr, int bias, int state_update, int param_update,
                    const float *res_mu, const float *res_var, int res_mode, float *delta_mu,
                    float *delta_var, float *delta_mu_w, float *delta_var_w, float *delta_mu_b,
                    float *delta_var_b, void *stream_) {
    if (res_mu != nullptr && (!res_var || (res_mode != 1 && res_mode != 2) || !state_update))
        return TAGI_ERR_INVALID_ARG;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const bool both = state_update && param_update && mu_w && var_w && mu_a && jcb && delta_mu_out &&
                      delta_var_out && aidx && zw_idx && zud_idx && delta_mu && delta_var &&
                      delta_mu_w && delta_var_w && B > 0 && fo > 0 && woho > 0 && wihi > 0 && fi > 0 &&
                      ki > 0 && nr > 0 && (!bias || (var_b && delta_mu_b && delta_var_b)) &&
                      conv_sizes_ok(B, fo, woho, fi, wihi, ki) && g_tune.conv_tile < 0 &&
                      g_tune.conv_dw_tile < 0;
    if (both && conv2d_bwd_pair(mu_w, mu_a, delta_mu_out, delta_var_out, B, fo, woho, wihi, fi, ki, nr)) {
        // both contractions on their stencil kernels: one launch for the two tile grids
        int tile_z = 0, splits_z = 1;
        conv2d_plan(fi, B * wihi, ki * ki * fo, &tile_z, &splits_z);
        if (g_tune.conv_splits > 0) splits_z = g_tune.conv_splits;
        const int out_tiles = ceil_div(fo, 64) * ceil_div(ki * ki * fi, 64);
        int splits_w = g_tune.conv_dw_splits > 0 ? g_tune.conv_dw_splits
                                                 : conv2d_bwd_dw_stencil_splits(out_tiles);
        const int max_splits = ceil_div(B * woho, 256);
        if (splits_w > max_splits) splits_w = max_splits;
        if (splits_w < 1) splits_w = 1;
        if (tile_z == 1) {  // 64 x 128, the tile of the state-backward stencil
            const size_t part_z = splits_z > 1 ? (size_t)splits_z * fi * B * wihi : 0;
            const size_t part_w = (size_t)splits_w * fo * ki * ki * fi;
            const int chunks = 64;  // slices of the (b, o) range in the bias reduction
            float *ws = nullptr;
            int rc = workspace_get((2 * part_z + 2 * part_w + 2 * (size_t)chunks * fo) * sizeof(float),
                                   stream, &ws);
            if (rc != TAGI_OK) return rc;
            float *wz = ws, *ww = ws + 2 * part_z;
            TAGI_TRY(launch_conv2d_bwd_pair(mu_w, var_w, mu_a, jcb, delta_mu_out, delta_var_out, aidx,
                                            zw_idx, zud_idx, B, fo, woho, wihi, fi, ki, nr, splits_z,
                                            wz, wz + part_z, splits_w, ww, ww + part_w, res_mu,
                                            res_var, res_mode, delta_mu, delta_var, delta_mu_w,
                                            delta_var_w, stream));
            if (bias)
                TAGI_TRY(launch_conv2d_bwd_db(var_b, delta_mu_out, delta_var_out, B, fo, woho, chunks,
                                              ww + 2 * part_w, delta_mu_b, delta_var_b, stream));
            return TAGI_OK;
        }
    }
    if (param_update) {
        int rc = tagi_conv2d_bwd_dw(var_w, var_b, mu_a, delta_mu_out, delta_var_out, aidx, B, fo, woho,
                                    wihi, fi, ki, bias, delta_mu_w, delta_var_w, delta_mu_b,
                                    delta_var_b, stream_);
        if (rc != TAGI_OK) return rc;
    }
    if (state_update)
        return conv2d_bwd_dz_impl(mu_w, jcb, delta_mu_out, delta_var_out, zw_idx, zud_idx, woho, fo,
                                  wihi, fi, ki, nr, B, delta_mu, delta_var, stream_, res_mu, res_var,
                                  res_mode);
    return TAGI_OK;
}

// ---------------------------------------------------------------------------
// Layer glue, update, output updater, ReLU
// ---------------------------------------------------------------------------

int tagi_store_states(const float *mu_a, const float *jcb, size_t n_in, float *bwd_mu_a,
                      float *bwd_jcb, float *out_jcb, size_t n_out, void *stream_) {
    if (n_in > 0 && (!mu_a || !bwd_mu_a || (jcb != nullptr) != (bwd_jcb != nullptr)))
        return TAGI_ERR_INVALID_ARG;
    if (n_out > 0 && !out_jcb) return TAGI_ERR_INVALID_ARG;
    TAGI_TRY(launch_store_states(mu_a, jcb, n_in, bwd_mu_a, bwd_jcb, out_jcb, n_out,
                                 static_cast<hipStream_t>(stream_)));
    return TAGI_OK;
}

int tagi_param_update(const float *delta_mu, const float *delta_var, float cap_factor, size_t n,
                      float *mu, float *var, int *neg_var_count, void *stream_) {
    if (n > 0 && (!delta_mu || !delta_var || !mu || !var)) return TAGI_ERR_INVALID_ARG;
    if (!(cap_factor > 0.0f)) return TAGI_ERR_INVALID_ARG;
    TAGI_TRY(launch_param_update(delta_mu, delta_var, cap_factor, n, mu, var, neg_var_count,
                                 static_cast<hipStream_t>(stream_)));
    return TAGI_OK;
}

int tagi_param_raw_update(const float *delta_mu, const float *delta_var, size_t n, float *mu,
                          float *var, void *stream_) {
    if (n > 0 && (!delta_mu || !delta_var || !mu || !var)) return TAGI_ERR_INVALID_ARG;
    TAGI_TRY(launch_param_raw_update(delta_mu, delta_var, n, mu, var,
                                     static_cast<hipStream_t>(stream_)));
    return TAGI_OK;
}

int tagi_layer_update(const float *delta_mu_w, const float *delta_var_w, size_t num_weights,
                      float *mu_w, float *var_w, const float *delta_mu_b,
                      const float *delta_var_b, size_t num_biases, float *mu_b, float *var_b,
                      float cap_factor, int *neg_var_count, int slot, void *stream_) {
    if (num_weights > 0 && (!delta_mu_w || !delta_var_w || !mu_w || !var_w))
        return TAGI_ERR_INVALID_ARG;
    if (num_biases > 0 && (!delta_mu_b || !delta_var_b || !mu_b || !var_b))
        return TAGI_ERR_INVALID_ARG;
    if (!(cap_factor > 0.0f) || (slot != 0 && slot != 1)) return TAGI_ERR_INVALID_ARG;
    TAGI_TRY(launch_layer_update(delta_mu_w, delta_var_w, num_weights, mu_w, var_w, delta_mu_b,
                                 delta_var_b, num_biases, mu_b, var_b, cap_factor, neg_var_count,
                                 slot, static_cast<hipStream_t>(stream_)));
    return TAGI_OK;
}

int tagi_model_update(const tagi_update_item *items, int n_items, void *stream_) {
    if (n_items < 0 || (n_items > 0 && items == nullptr)) return TAGI_ERR_INVALID_ARG;
    for (int i = 0; i < n_items; i++) {
        const tagi_update_item &t = items[i];
        if (t.num_weights > 0 && (!t.delta_mu_w || !t.delta_var_w || !t.mu_w || !t.var_w))
            return TAGI_ERR_INVALID_ARG;
        if (t.num_biases > 0 && (!t.delta_mu_b || !t.delta_var_b || !t.mu_b || !t.var_b))
            return TAGI_ERR_INVALID_ARG;
        if (!(t.cap_factor > 0.0f) || (t.slot != 0 && t.slot != 1)) return TAGI_ERR_INVALID_ARG;
        if ((t.num_weights + t.num_biases + 255) / 256 > 0x3fffffffu) return TAGI_ERR_UNSUPPORTED;
    }
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    int i = 0;
    while (i < n_items) {
        ModelUpdateArgs a = {};
        unsigned long long blocks = 0;
        for (; i < n_items && a.n < MODEL_UPDATE_MAX; i++) {
            const tagi_update_item &t = items[i];
            const unsigned long long b = (t.num_weights + t.num_biases + 255) / 256;
            if (b == 0) continue;
            if (a.n > 0 && blocks + b > 0x7fffffffULL) break;  // the rest: next launch
            const int k = a.n++;
            a.dmu_w[k] = t.delta_mu_w; a.dvar_w[k] = t.delta_var_w;
            a.mu_w[k] = t.mu_w; a.var_w[k] = t.var_w; a.nw[k] = t.num_weights;
            a.dmu_b[k] = t.delta_mu_b; a.dvar_b[k] = t.delta_var_b;
            a.mu_b[k] = t.mu_b; a.var_b[k] = t.var_b; a.nb[k] = t.num_biases;
            a.cap[k] = t.cap_factor; a.count[k] = t.neg_var_count; a.slot[k] = t.slot;
            a.first_block[k] = (unsigned)blocks;
            blocks += b;
        }
        a.first_block[a.n] = (unsigned)blocks;
        TAGI_TRY(launch_model_update(a, stream));
    }
    return TAGI_OK;
}

float tagi_cap_factor(int batch_size, float prev) {
    if (batch_size == 1) return 0.1f;
    if (batch_size > 1 && batch_size < 256) return 2.0f;
    if (batch_size >= 256) return 3.0f;
    return prev;
}

int tagi_out_update_dense(const float *mu_a, const float *var_a, const float *jcb,
                          const float *obs, const float *var_obs, int n, float *delta_mu,
                          float *delta_var, void *stream_) {
    if (n < 0) return TAGI_ERR_INVALID_ARG;
    if (n > 0 && (!mu_a || !var_a || !jcb || !obs || !var_obs || !delta_mu || !delta_var))
        return TAGI_ERR_INVALID_ARG;
    TAGI_TRY(launch_out_update_dense(mu_a, var_a, jcb, obs, var_obs, n, delta_mu, delta_var,
                                     static_cast<hipStream_t>(stream_)));
    return TAGI_OK;
}

int tagi_out_update_heteros(const float *mu_a, const float *var_a, const float *jcb,
                            const float *obs, int n, float *delta_mu, float *delta_var,
                            void *stream_) {
    if (n < 0) return TAGI_ERR_INVALID_ARG;
    if (n > 0 && (!mu_a || !var_a || !jcb || !obs || !delta_mu || !delta_var))
        return TAGI_ERR_INVALID_ARG;
    // pairs are read and written as 8-byte elements
    if (n > 0 && (((uintptr_t)mu_a | (uintptr_t)var_a | (uintptr_t)jcb | (uintptr_t)delta_mu |
                   (uintptr_t)delta_var) & 7u))
        return TAGI_ERR_INVALID_ARG;
    TAGI_TRY(launch_out_update_heteros(mu_a, var_a, jcb, obs, n, delta_mu, delta_var,
                                       static_cast<hipStream_t>(stream_)));
    return TAGI_OK;
}

int tagi_out_update_indexed(const float *mu_a, const float *var_a, const float *jcb,
                            const float *obs, const float *var_obs, const int *selected_idx,
                            int n_obs, int n_enc, int n, float *delta_mu, float *delta_var,
                            void *stream_) {
    if (n < 0 || n_obs <= 0 || n_enc <= 0) return TAGI_ERR_INVALID_ARG;
    if (n > 0 && (!mu_a || !var_a || !jcb || !obs || !var_obs || !selected_idx || !delta_mu ||
                  !delta_var))
        return TAGI_ERR_INVALID_ARG;
    TAGI_TRY(launch_out_update_indexed(mu_a, var_a, jcb, obs, var_obs, selected_idx, n_obs, n_enc,
                                       n, delta_mu, delta_var, static_cast<hipStream_t>(stream_)));
    return TAGI_OK;
}

int tagi_out_update_indexed_reset(const float *mu_a, const float *var_a, const float *jcb,
                                  const float *obs, const float *var_obs, const int *selected_idx,
                                  int n_obs, int n_enc, int n, float *delta_mu, float *delta_var,
                                  size_t delta_len, void *stream_) {
    if (n < 0 || n_obs <= 0 || n_enc <= 0 || n % n_enc != 0) return TAGI_ERR_INVALID_ARG;
    if ((n > 0 || delta_len > 0) && (!delta_mu || !delta_var)) return TAGI_ERR_INVALID_ARG;
    if (n > 0 && (!mu_a || !var_a || !jcb || !obs || !var_obs || !selected_idx))
        return TAGI_ERR_INVALID_ARG;
    if ((size_t)(n / n_enc) * n_obs > delta_len) return TAGI_ERR_INVALID_ARG;
    TAGI_TRY(launch_out_update_indexed_reset(mu_a, var_a, jcb, obs, var_obs, selected_idx, n_obs,
                                             n_enc, n / n_enc, delta_mu, delta_var, delta_len,
                                             static_cast<hipStream_t>(stream_)));
    return TAGI_OK;
}

int tagi_upload_input(const float *host_mu, const float *host_var, size_t n, float *mu_a,
                      float *var_a, void *stream_) {
    if (n > 0 && (!host_mu || !mu_a || !var_a)) return TAGI_ERR_INVALID_ARG;
    TAGI_TRY(launch_upload_input(host_mu, host_var, n, mu_a, var_a,
                                 static_cast<hipStream_t>(stream_)));
    return TAGI_OK;
}

int tagi_download_outputs(const float *mu_a, const float *var_a, size_t n, float *host_mu,
                          float *host_var, unsigned *host_flag, unsigned flag_value,
                          void *stream_) {
    if (n > 0 && (!mu_a || !var_a || !host_mu || !host_var)) return TAGI_ERR_INVALID_ARG;
    // with a flag the copy is one workgroup's loop: meant for outputs, not for whole buffers
    if (host_flag != nullptr && n > ((size_t)1 << 20)) return TAGI_ERR_UNSUPPORTED;
    TAGI_TRY(launch_download_outputs(mu_a, var_a, n, host_mu, host_var, host_flag, flag_value,
                                     static_cast<hipStream_t>(stream_)));
    return TAGI_OK;
}

int tagi_relu_fwd(const float *mu_z, const float *var_z, size_t n, float *mu_a, float *jcb,
                  float *var_a, void *stream_) {
    if (n > 0 && (!mu_z || !var_z || !mu_a || !jcb || !var_a)) return TAGI_ERR_INVALID_ARG;
    TAGI_TRY(launch_relu(mu_z, var_z, n, mu_a, jcb, var_a, static_cast<hipStream_t>(stream_)));
    return TAGI_OK;
}

// ---------------------------------------------------------------------------
// MixtureReLU, BatchNorm2d, AvgPool2d, residual adds
// ---------------------------------------------------------------------------

int tagi_mixture_relu_fwd(const float *mu_z, const float *var_z, size_t n, float *mu_a,
                          float *jcb, float *var_a, void *stream) {
    if (!mu_z || !var_z || !mu_a || !jcb || !var_a) return TAGI_ERR_INVALID_ARG;
    if (n == 0) return TAGI_OK;
    TAGI_TRY(launch_mixture_relu(mu_z, var_z, n, mu_a, jcb, var_a,
                                 static_cast<hipStream_t>(stream)));
    return TAGI_OK;
}

static bool bn_sizes_ok(int wihi, int fi, int B) {
    return wihi > 0 && fi > 0 && B > 0 && fi <= 65535 &&
           (long long)wihi * fi * B < 0x7fffffffLL;
}

int tagi_batchnorm2d_stats(const float *mu_a, const float *var_a, int wihi, int fi, int B,
                           float momentum, float *mu_s, float *var_s, float *mu_ra,
                           float *var_ra, void *stream) {
    if (!mu_a || !var_a || !mu_s || !var_s || !mu_ra || !var_ra) return TAGI_ERR_INVALID_ARG;
    if (!bn_sizes_ok(wihi, fi, B)) return TAGI_ERR_INVALID_ARG;
    float *ws = nullptr;
    int rc = workspace_get(batchnorm2d_scratch_floats(fi, B) * sizeof(float),
                           static_cast<hipStream_t>(stream), &ws);
    if (rc != TAGI_OK) return rc;
    TAGI_TRY(launch_batchnorm2d_stats(mu_a, var_a, wihi, fi, B, momentum, ws, mu_s, var_s, mu_ra,
                                      var_ra, static_cast<hipStream_t>(stream)));
    return TAGI_OK;
}

static int batchnorm2d_fwd_impl(const float *mu_w, const float *var_w, const float *mu_b,
                         const float *var_b, const float *mu_a, const float *var_a,
                         const float *mu_norm, const float *var_norm, int bias, float epsilon,
                         int wihi, int fi, int B, float *mu_z, float *var_z, void *stream,
                               const float *mu_res, const float *var_res) {
    if (!mu_w || !var_w || !mu_a || !var_a || !mu_norm || !var_norm || !mu_z || !var_z)
        return TAGI_ERR_INVALID_ARG;
    if (bias && (!mu_b || !var_b)) return TAGI_ERR_INVALID_ARG;
    if (!bn_sizes_ok(wihi, fi, B)) return TAGI_ERR_INVALID_ARG;
    TAGI_TRY(launch_batchnorm2d_fwd(mu_w, var_w, bias ? mu_b : nullptr, bias ? var_b : nullptr,
                                    mu_a, var_a, mu_norm, var_norm, epsilon, wihi, fi, B, mu_z,
                                    var_z, static_cast<hipStream_t>(stream), mu_res, var_res));
    return TAGI_OK;
}

int tagi_batchnorm2d_fwd_train(const float *mu_w, const float *var_w, const float *mu_b,
                               const float *var_b, const float *mu_a, const float *var_a,
                               const float *mu_res, const float *var_res, int bias, float momentum,
                               float epsilon, int wihi, int fi, int B, float *mu_s, float *var_s,
                               float *mu_ra, float *var_ra, float *mu_z, float *var_z,
                               void *stream) {
    if (!mu_w || !var_w || !mu_a || !var_a || !mu_s || !var_s || !mu_ra || !var_ra || !mu_z || !var_z)
        return TAGI_ERR_INVALID_ARG;
    if (bias && (!mu_b || !var_b)) return TAGI_ERR_INVALID_ARG;
    if ((mu_res == nullptr) != (var_res == nullptr)) return TAGI_ERR_INVALID_ARG;
    if (!bn_sizes_ok(wihi, fi, B)) return TAGI_ERR_INVALID_ARG;
    float *ws = nullptr;
    int rc = workspace_get(batchnorm2d_scratch_floats(fi, B) * sizeof(float),
                           static_cast<hipStream_t>(stream), &ws);
    if (rc != TAGI_OK) return rc;
    TAGI_TRY(launch_batchnorm2d_fwd_train(mu_w, var_w, bias ? mu_b : nullptr, bias ? var_b : nullptr,
                                          mu_a, var_a, mu_res, var_res, momentum, epsilon, wihi, fi,
                                          B, ws, mu_s, var_s, mu_ra, var_ra, mu_z, var_z,
                                          static_cast<hipStream_t>(stream)));
    return TAGI_OK;
}

int tagi_batchnorm2d_fwd(const float *mu_w, const float *var_w, const float *mu_b,
                         const float *var_b, const float *mu_a, const float *var_a,
                         const float *mu_norm, const float *var_norm, int bias, float epsilon,
                         int wihi, int fi, int B, float *mu_z, float *var_z, void *stream) {
    return batchnorm2d_fwd_impl(mu_w, var_w, mu_b, var_b, mu_a, var_a, mu_norm, var_norm, bias,
                                epsilon, wihi, fi, B, mu_z, var_z, stream, nullptr, nullptr);
}

int tagi_batchnorm2d_fwd_res(const float *mu_w, const float *var_w, const float *mu_b,
                             const float *var_b, const float *mu_a, const float *var_a,
                             const float *mu_norm, const float *var_norm, const float *mu_res,
                             const float *var_res, int bias, float epsilon, int wihi, int fi,
                             int B, float *mu_z, float *var_z, void *stream) {
    if (!mu_res || !var_res) return TAGI_ERR_INVALID_ARG;
    return batchnorm2d_fwd_impl(mu_w, var_w, mu_b, var_b, mu_a, var_a, mu_norm, var_norm, bias,
                                epsilon, wihi, fi, B, mu_z, var_z, stream, mu_res, var_res);
}

int tagi_batchnorm2d_bwd(const float *mu_w, const float *var_w, const float *var_b,
                         const float *mu_a, const float *jcb, const float *mu_norm,
                         const float *var_norm, const float *delta_mu_out,
                         const float *delta_var_out, float epsilon, int wihi, int fi, int B,
                         int bias, int state_update, int param_update, float *delta_mu,
                         float *delta_var, float *delta_mu_w, float *delta_var_w,
                         float *delta_mu_b, float *delta_var_b, void *stream) {
    if (!mu_w || !var_w || !mu_norm || !var_norm || !delta_mu_out || !delta_var_out)
        return TAGI_ERR_INVALID_ARG;
    if (state_update && (!jcb || !delta_mu || !delta_var)) return TAGI_ERR_INVALID_ARG;
    if (param_update && (!mu_a || !delta_mu_w || !delta_var_w)) return TAGI_ERR_INVALID_ARG;
    if (param_update && bias && (!var_b || !delta_mu_b || !delta_var_b))
        return TAGI_ERR_INVALID_ARG;
    if (!bn_sizes_ok(wihi, fi, B)) return TAGI_ERR_INVALID_ARG;
    if (!state_update && !param_update) return TAGI_OK;
    float *ws = nullptr;
    int rc = workspace_get(batchnorm2d_scratch_floats(fi, B) * sizeof(float),
                           static_cast<hipStream_t>(stream), &ws);
    if (rc != TAGI_OK) return rc;
    TAGI_TRY(launch_batchnorm2d_bwd(mu_w, var_w, bias ? var_b : nullptr, mu_a, jcb, mu_norm,
                                    var_norm, delta_mu_out, delta_var_out, epsilon, wihi, fi, B,
                                    state_update, param_update, ws, delta_mu, delta_var,
                                    delta_mu_w, delta_var_w, delta_mu_b, delta_var_b,
                                    static_cast<hipStream_t>(stream)));
    return TAGI_OK;
}

int tagi_avgpool2d_build_idx(int kernel, int stride, int wi, int hi, int pad, int pad_type,
                             int *pool_idx, int *z_ud_idx, int *w, int *h, int *overlap) {
    if (!pool_idx || !z_ud_idx || !w || !h || !overlap) return TAGI_ERR_INVALID_ARG;
    return avgpool2d_build_idx(kernel, stride, wi, hi, pad, pad_type, pool_idx, z_ud_idx, w, h,
                               overlap) == 0
               ? TAGI_OK
               : TAGI_ERR_INVALID_ARG;
}

int tagi_avgpool2d_fwd(const float *mu_a, const float *var_a, const int *pool_idx, int woho,
                       int wihi, int ki, int n_out, float *mu_z, float *var_z, void *stream) {
    if (!mu_a || !var_a || !pool_idx || !mu_z || !var_z) return TAGI_ERR_INVALID_ARG;
    if (woho <= 0 || wihi <= 0 || ki <= 0 || n_out <= 0 || n_out % woho != 0)
        return TAGI_ERR_INVALID_ARG;
    TAGI_TRY(launch_avgpool2d_fwd(mu_a, var_a, pool_idx, woho, wihi, ki, n_out, mu_z, var_z,
                                  static_cast<hipStream_t>(stream)));
    return TAGI_OK;
}

int tagi_avgpool2d_bwd_dz(const float *jcb, const float *delta_mu_out, const float *delta_var_out,
                          const int *z_ud_idx, int woho, int wihi, int ki, int nr, int wo,
                          int n_in, int overlap, float *delta_mu, float *delta_var,
                          void *stream) {
    if (!jcb || !delta_mu_out || !delta_var_out || !delta_mu || !delta_var)
        return TAGI_ERR_INVALID_ARG;
    if (woho <= 0 || wihi <= 0 || ki <= 0 || n_in <= 0 || n_in % wihi != 0)
        return TAGI_ERR_INVALID_ARG;
    if (overlap && (!z_ud_idx || nr <= 0)) return TAGI_ERR_INVALID_ARG;
    if (!overlap && (wo <= 0 || n_in % (ki * wo) != 0)) return TAGI_ERR_INVALID_ARG;
    TAGI_TRY(launch_avgpool2d_bwd(jcb, delta_mu_out, delta_var_out, z_ud_idx, woho, wihi, ki, nr,
                                  wo, n_in, overlap, delta_mu, delta_var,
                                  static_cast<hipStream_t>(stream)));
    return TAGI_OK;
}

int tagi_add_shortcut(const float *mu_s, const float *var_s, size_t n, float *mu_a, float *var_a,
                      void *stream) {
    if (!mu_s || !var_s || !mu_a || !var_a) return TAGI_ERR_INVALID_ARG;
    if (n == 0) return TAGI_OK;
    TAGI_TRY(launch_add_shortcut(mu_s, var_s, nullptr, n, mu_a, var_a,
                                 static_cast<hipStream_t>(stream)));
    return TAGI_OK;
}

int tagi_add_shortcut_delta(const float *mu_s, const float *var_s, const float *jcb_s, size_t n,
                            float *mu_a, float *var_a, void *stream) {
    if (!mu_s || !var_s || !jcb_s || !mu_a || !var_a) return TAGI_ERR_INVALID_ARG;
    if (n == 0) return TAGI_OK;
    TAGI_TRY(launch_add_shortcut(mu_s, var_s, jcb_s, n, mu_a, var_a,
                                 static_cast<hipStream_t>(stream)));
    return TAGI_OK;
}

}  // extern "C"

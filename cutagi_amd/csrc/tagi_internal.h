// Internal launcher interface between the C ABI (tagi_capi.hip) and the kernel
// translation units. Not installed; the public surface is include/tagi_hip.h.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

namespace tagi {

// Compute units of the current device (256 on an MI355X), asked of the runtime once
// per device; launch shapes that aim at "workgroups per CU" are derived from it.
int num_cu();
constexpr int MAX_DEVICES = 16;

// Raises a kernel's dynamic-LDS limit, once per device: the attribute belongs to the
// kernel's code object on the device that is current when it is set.
struct PerDeviceOnce {
    bool done[MAX_DEVICES] = {};
};
inline hipError_t allow_dynamic_lds(PerDeviceOnce &once, const void *kernel, int bytes) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= MAX_DEVICES) return hipErrorInvalidDevice;
    if (once.done[dev]) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess) once.done[dev] = true;
    return e;
}

// Which contraction of the layer a tiled GEMM launch computes.
//   FWD: D[b][n]  = sum_k  act[b][k] * w[n][k]      (mean; variance with 2 terms)
//   DZ : D[b][k'] = sum_n  delta[b][n] * w[n][k']   (variance with w^2)
//   DW : D[n][k'] = sum_b  delta[b][n] * act[b][k'] (variance with act^2)
enum GemmMode { GEMM_FWD = 0, GEMM_DZ = 1, GEMM_DW = 2 };

// Epilogue applied to the two accumulators (mean-like `0`, variance-like `1`).
//   EPI_BIAS : out0 = acc0 + e0[col], out1 = acc1 + e1[col]   (e0 == nullptr: none)
//   EPI_SCALE: out0 = acc0 * e0[row][col], out1 = acc1 * e0[row][col]^2
enum Epilogue { EPI_BIAS = 0, EPI_SCALE = 1 };

struct GemmParams {
    const float *x0, *x1;  // row-side operands (FWD: mu_a,var_a; DZ/DW: delta_mu,delta_var)
    const float *y0, *y1;  // column-side operands (FWD: mu_w,var_w; DZ: mu_w; DW: mu_a)
    int M, N, R;           // D is M x N, reduction length R
    int ldx, ldy;          // leading dimensions of the operands as stored
    float *out0, *out1;    // M x N, leading dimension ldo
    int ldo;
    const float *e0, *e1;  // epilogue operands, see Epilogue
    int splits;            // number of reduction slices (gridDim.y)
    int r_per_split;       // reduction elements per slice, multiple of the k-tile
    float *ws0, *ws1;      // [splits][M][N] partial sums when splits > 1
    // FWD only: activation applied to the sums before they are stored (tagi_activation.h);
    // then out0/out1 receive its mean / variance and out2 its Jacobian
    int act;
    float *out2;
};

// Tile shapes the tiled kernels are instantiated for (indices 0..count-1).
int gemm_tile_count();
int gemm_tile_rows(int tile);
int gemm_tile_cols(int tile);
int gemm_k_tile();

// 0 keeps the Linear tile kernels on the single-stage k-loop (tuning knob).
extern int g_gemm_double_buffer;

// Launches the tiled MFMA kernel. `vec` selects 16-byte global loads (the caller
// guarantees the alignment rules); partial sums go to ws0/ws1 when splits > 1
// and the caller then runs reduce_splits.
hipError_t launch_gemm(GemmMode mode, int tile, bool vec, const GemmParams &p,
                       hipStream_t stream);

// Small jobs of a Linear backward call that ride along with the tiled weight
// backward (first workgroups of its launch): the fold of a sliced state backward
// (out = sum over slices of ws, times jcb / jcb^2; total a multiple of 4, all
// pointers 16-byte aligned) and the bias innovations. A null ws0 / var_b leaves
// the job out.
struct LinearSideWork {
    const float *ws0 = nullptr, *ws1 = nullptr, *jcb = nullptr;
    float *out0 = nullptr, *out1 = nullptr;
    int fold_splits = 0;
    size_t fold_total = 0;
    const float *var_b = nullptr, *dmu = nullptr, *dvar = nullptr;
    float *dmu_b = nullptr, *dvar_b = nullptr;
    int bias_n = 0, bias_b = 0;
    int bias_wgs = 0, side_wgs = 0;  // set by the launcher
};
bool gemm_dw_side_supported(int tile, bool vec, const GemmParams &p);
hipError_t launch_gemm_dw_side(const GemmParams &p, LinearSideWork w, hipStream_t stream);

// out = epilogue(sum over splits of ws[s]) for the two accumulators.
// (EPI_BIAS only: `act` / `out2` as in GemmParams.)
hipError_t launch_reduce_splits(Epilogue epi, const float *ws0, const float *ws1,
                                int splits, int M, int N, const float *e0,
                                const float *e1, float *out0, float *out1, int ldo,
                                hipStream_t stream, int act = 0, float *out2 = nullptr);

// Forward of small layers in one launch (no slices, no LDS): one wave per 2 rows x 8
// samples, lanes across the reduction. Needs K % 4 == 0 and 16-byte aligned pointers.
bool small_fwd_supported(int K, int N, int B);
hipError_t launch_small_fwd(const float *mu_w, const float *var_w, const float *mu_b,
                            const float *var_b, const float *mu_a, const float *var_a, int K,
                            int N, int B, int act, float *out0, float *out1, float *out2,
                            hipStream_t stream);

// State and weight backward of the same layers, one launch each; the weight backward
// also writes the bias innovations when var_b is given.
bool small_bwd_supported(int K, int N, int B);
bool small_dw_supported(int K, int N, int B);
hipError_t launch_small_dz(const float *mu_w, const float *jcb, const float *dmu, const float *dvar,
                           int K, int N, int B, float *out_mu, float *out_var, hipStream_t stream);
hipError_t launch_small_dw(const float *var_w, const float *mu_a, const float *dmu,
                           const float *dvar, int K, int N, int B, float *dmu_w, float *dvar_w,
                           const float *var_b, float *dmu_b, float *dvar_b, hipStream_t stream);

hipError_t launch_small_bwd_pair(const float *mu_w, const float *var_w, const float *mu_a,
                                 const float *jcb, const float *dmu, const float *dvar, int K, int N,
                                 int B, float *out_mu, float *out_var, float *dmu_w, float *dvar_w,
                                 const float *var_b, float *dmu_b, float *dvar_b,
                                 hipStream_t stream);

// Skinny-batch (B <= 16) streaming kernels: weights are read once from HBM
// straight into MFMA operand layout, nothing is staged in LDS.
hipError_t launch_gemv_fwd(const float *mu_w, const float *var_w, const float *mu_a,
                           const float *var_a, int K, int N, int B, int splits, int swz,
                           int variant, float *ws0, float *ws1, hipStream_t stream);
hipError_t launch_gemv_dz(const float *mu_w, const float *dmu, const float *dvar, int K,
                          int N, int B, int splits, int rev, float *ws0, float *ws1,
                          hipStream_t stream);
// Partial sums of a sliced state backward that a later kernel folds:
// out = (sum over slices of ws) * jcb (mean) and * jcb^2 (variance).
struct DzFold {
    const float *ws0 = nullptr, *ws1 = nullptr;  // [splits][total]
    const float *jcb = nullptr;
    float *out0 = nullptr, *out1 = nullptr;
    int splits = 0;
    size_t total = 0;  // B * K, a multiple of 4
};
hipError_t launch_gemv_dw(const float *var_w, const float *mu_a, const float *dmu,
                          const float *dvar, int K, int N, int B, int rev, float *dmu_w,
                          float *dvar_w, const float *var_b, float *dmu_b, float *dvar_b,
                          const DzFold *fold, hipStream_t stream);
// The same for 9 <= B <= 32 on the 16x16x4 MFMA (tagi_gemv16.hip; beyond 16 samples every
// weight fragment feeds two MFMAs); slices are
// multiples of the *_step() and at most the *_max_slice().
hipError_t launch_gemv16_fwd(const float *mu_w, const float *var_w, const float *mu_a,
                             const float *var_a, int K, int N, int B, int k_per_split,
                             int splits, float *ws0, float *ws1, hipStream_t stream);
hipError_t launch_gemv16_dz(const float *mu_w, const float *dmu, const float *dvar, int K, int N,
                            int B, int n_per_split, int splits, float *ws0, float *ws1,
                            hipStream_t stream);
// 1: the 9..16-sample forward kernel that loads whole cache lines (default 0)
extern int g_gemv16_fwd_whole_lines;
int gemv16_fwd_rows_per_block(int N, int K, int B);
extern int g_gemv16_fwd_waves;
int gemv16_fwd_k_step();
int gemv16_fwd_max_slice(int B);
int gemv16_max_batch();  // 32: two groups of sixteen samples
int gemv16_dz_cols_per_block();
int gemv16_dz_n_step();
int gemv16_dz_max_slice(int B);
int gemv_fwd_variants();
int gemv_fwd_rows_per_block(int variant);
int gemv_fwd_k_step();
int gemv_dz_cols_per_block();
int gemv_dz_n_step();
int gemv_fwd_max_slice(int B);  // longest reduction slice whose activations fit in LDS
int gemv_dz_max_slice(int B);

// Elementwise / small kernels
hipError_t launch_bias_delta(const float *var_b, const float *dmu, const float *dvar, int N,
                             int B, float *dmu_b, float *dvar_b, hipStream_t stream);
hipError_t launch_store_states(const float *mu_a, const float *jcb, size_t n_in,
                               float *bwd_mu_a, float *bwd_jcb, float *out_jcb, size_t n_out,
                               hipStream_t stream);
hipError_t launch_param_update(const float *dmu, const float *dvar, float cap, size_t n,
                               float *mu, float *var, int *neg_count, hipStream_t stream);
hipError_t launch_param_raw_update(const float *dmu, const float *dvar, size_t n, float *mu,
                                   float *var, hipStream_t stream);
hipError_t launch_layer_update(const float *dmu_w, const float *dvar_w, size_t nw, float *mu_w,
                               float *var_w, const float *dmu_b, const float *dvar_b, size_t nb,
                               float *mu_b, float *var_b, float cap, int *count, int slot,
                               hipStream_t stream);
// Up to MODEL_UPDATE_MAX layers per launch; block b belongs to the item whose
// [first_block, first_block of the next) range holds it.
constexpr int MODEL_UPDATE_MAX = 24;
struct ModelUpdateArgs {
    const float *dmu_w[MODEL_UPDATE_MAX], *dvar_w[MODEL_UPDATE_MAX];
    float *mu_w[MODEL_UPDATE_MAX], *var_w[MODEL_UPDATE_MAX];
    const float *dmu_b[MODEL_UPDATE_MAX], *dvar_b[MODEL_UPDATE_MAX];
    float *mu_b[MODEL_UPDATE_MAX], *var_b[MODEL_UPDATE_MAX];
    int *count[MODEL_UPDATE_MAX];
    unsigned long long nw[MODEL_UPDATE_MAX], nb[MODEL_UPDATE_MAX];
    float cap[MODEL_UPDATE_MAX];
    int slot[MODEL_UPDATE_MAX];
    unsigned first_block[MODEL_UPDATE_MAX + 1];
    int n;
};
hipError_t launch_model_update(const ModelUpdateArgs &args, hipStream_t stream);
hipError_t launch_out_update_dense(const float *mu_a, const float *var_a, const float *jcb,
                                   const float *obs, const float *var_obs, int n, float *dmu,
                                   float *dvar, hipStream_t stream);
hipError_t launch_out_update_heteros(const float *mu_a, const float *var_a, const float *jcb,
                                     const float *obs, int n, float *dmu, float *dvar,
                                     hipStream_t stream);
hipError_t launch_out_update_indexed(const float *mu_a, const float *var_a, const float *jcb,
                                     const float *obs, const float *var_obs, const int *sel,
                                     int n_obs, int n_enc, int n, float *dmu, float *dvar,
                                     hipStream_t stream);
hipError_t launch_relu(const float *mu_z, const float *var_z, size_t n, float *mu_a, float *jcb,
                       float *var_a, hipStream_t stream);
hipError_t launch_out_update_indexed_reset(const float *mu_a, const float *var_a, const float *jcb,
                                           const float *obs, const float *var_obs, const int *sel,
                                           int n_obs, int n_enc, int samples, float *dmu,
                                           float *dvar, size_t delta_len, hipStream_t stream);
hipError_t launch_download_outputs(const float *mu_a, const float *var_a, size_t n, float *host_mu,
                                   float *host_var, unsigned *host_flag, unsigned flag_value,
                                   hipStream_t stream);
hipError_t launch_upload_input(const float *host_mu, const float *host_var, size_t n, float *mu_a,
                               float *var_a, hipStream_t stream);

// Layers between the contractions (tagi_layers.hip)
hipError_t launch_mixture_relu(const float *mu_z, const float *var_z, size_t n, float *mu_a,
                               float *jcb, float *var_a, hipStream_t stream);
size_t batchnorm2d_scratch_floats(int fi, int B);
hipError_t launch_batchnorm2d_stats(const float *mu_a, const float *var_a, int wihi, int fi,
                                    int B, float momentum, float *scratch, float *mu_s,
                                    float *var_s, float *mu_ra, float *var_ra,
                                    hipStream_t stream);
extern int g_bn_fused_train;  // 0: statistics merged by a launch of their own
hipError_t launch_batchnorm2d_fwd_train(const float *mu_w, const float *var_w, const float *mu_b,
                                        const float *var_b, const float *mu_a, const float *var_a,
                                        const float *mu_res, const float *var_res, float momentum,
                                        float epsilon, int wihi, int fi, int B, float *scratch,
                                        float *mu_s, float *var_s, float *mu_ra, float *var_ra,
                                        float *mu_z, float *var_z, hipStream_t stream);
hipError_t launch_batchnorm2d_fwd(const float *mu_w, const float *var_w, const float *mu_b,
                                  const float *var_b, const float *mu_a, const float *var_a,
                                  const float *mu_norm, const float *var_norm, float epsilon,
                                  int wihi, int fi, int B, float *mu_z, float *var_z,
                                  hipStream_t stream, const float *mu_res = nullptr,
                                  const float *var_res = nullptr);
hipError_t launch_batchnorm2d_bwd(const float *mu_w, const float *var_w, const float *var_b,
                                  const float *mu_a, const float *jcb, const float *mu_norm,
                                  const float *var_norm, const float *dmu_out,
                                  const float *dvar_out, float epsilon, int wihi, int fi, int B,
                                  int state_update, int param_update, float *scratch, float *dmu,
                                  float *dvar, float *dmu_w, float *dvar_w, float *dmu_b,
                                  float *dvar_b, hipStream_t stream);
hipError_t launch_avgpool2d_fwd(const float *mu_a, const float *var_a, const int *pool_idx,
                                int woho, int wihi, int ki, int n_out, float *mu_z, float *var_z,
                                hipStream_t stream);
hipError_t launch_avgpool2d_bwd(const float *jcb, const float *dmu_out, const float *dvar_out,
                                const int *z_ud_idx, int woho, int wihi, int ki, int nr, int wo,
                                int n_in, int overlap, float *dmu, float *dvar,
                                hipStream_t stream);
hipError_t launch_add_shortcut(const float *mu_s, const float *var_s, const float *jcb_s,
                               size_t n, float *mu_a, float *var_a, hipStream_t stream);

// Conv2d (implicit GEMM through the index tables)
void conv2d_plan(int M, int N, int R, int *tile, int *splits);
// 0 switches the sixteen-byte group loads of the conv2d gathers off (tuning knob).
extern int g_conv2d_group_loads;
// 0 switches the regular-stencil kernels of the conv2d forward / state backward off.
extern int g_conv2d_stencil;
// 0 keeps the natural column order in the conv2d state backward of strided layers.
extern int g_conv2d_phase_order;
extern int g_conv2d_s2_all;   // 0: no stencil kernels for the stride-2 layers
int conv2d_bwd_dz_s2_all(const float *mu_w, const float *dmu, const float *dvar, int B, int fo,
                         int woho, int wihi, int fi, int ki, int nr);
int conv2d_bwd_dz_s2_all_splits(int B, int fo, int woho, int fi);

hipError_t launch_conv2d_fwd(const float *mu_w, const float *var_w, const float *mu_b,
                             const float *var_b, const float *mu_a, const float *var_a,
                             const int *aidx, int woho, int fo, int wihi, int fi, int ki, int B,
                             int bias, int tile, int splits, float *ws0, float *ws1, float *mu_z,
                             float *var_z, hipStream_t stream, int act = 0, float *jcb = nullptr);
hipError_t launch_conv2d_bwd_dz(const float *mu_w, const float *jcb, const float *dmu,
                                const float *dvar, const int *zw_idx, const int *zud_idx,
                                int woho, int fo, int wihi, int fi, int ki, int nr, int B,
                                int tile, int splits, float *ws0, float *ws1, float *out_dmu,
                                float *out_dvar, hipStream_t stream, const float *res_mu = nullptr,
                                const float *res_var = nullptr, int res_mode = 0);
int conv2d_bwd_dw_blocks_per_cu(int tile);
int conv2d_bwd_dw_stencil(const float *mu_a, const float *dmu, const float *dvar, int B, int fo,
                          int woho, int wihi, int fi, int ki, int tile);
int conv2d_bwd_dw_stencil_splits(int out_tiles);
int conv2d_bwd_dw_s2(const float *mu_a, const float *dmu, const float *dvar, int B, int fo,
                     int woho, int wihi, int fi, int ki, int tile);
hipError_t launch_conv2d_bwd_dw(const float *var_w, const float *mu_a, const float *dmu,
                                const float *dvar, const int *aidx, int B, int fo, int woho,
                                int wihi, int fi, int ki, int tile, int splits, float *ws0, float *ws1,
                                float *dmu_w, float *dvar_w, hipStream_t stream);
// 0: state and weight backward of a layer always as launches of their own
extern int g_conv2d_bwd_pair;
int conv2d_bwd_pair(const float *mu_w, const float *mu_a, const float *dmu, const float *dvar, int B,
                    int fo, int woho, int wihi, int fi, int ki, int nr);
hipError_t launch_conv2d_bwd_pair(const float *mu_w, const float *var_w, const float *mu_a,
                                  const float *jcb, const float *dmu, const float *dvar,
                                  const int *aidx, const int *zw_idx, const int *zud_idx, int B,
                                  int fo, int woho, int wihi, int fi, int ki, int nr, int splits_z,
                                  float *wz0, float *wz1, int splits_w, float *ww0, float *ww1,
                                  const float *res_mu, const float *res_var, int res_mode,
                                  float *out_dmu, float *out_dvar, float *dmu_w, float *dvar_w,
                                  hipStream_t stream);
hipError_t launch_conv2d_bwd_db(const float *var_b, const float *dmu, const float *dvar, int B,
                                int fo, int woho, int chunks, float *scratch, float *dmu_b,
                                float *dvar_b, hipStream_t stream);

// Host-side index tables (tagi_conv_idx.cpp)
int conv2d_out_size(int kernel, int stride, int wi, int hi, int pad, int pad_type, int *wo,
                    int *ho);
int conv2d_build_idx(int kernel, int stride, int wi, int hi, int pad, int pad_type,
                     int param_pad_idx, int *Fmwa_2, int *FCzwa_1, int *Szz_ud, int *w, int *h);
int avgpool2d_build_idx(int kernel, int stride, int wi, int hi, int pad, int pad_type,
                        int *pool_idx, int *z_ud_idx, int *w, int *h, int *overlap);

}  // namespace tagi

// Layer classes of the hot path, mirroring the reference's interface so that a
// model description written for it runs unchanged: BaseLayer
// (include/base_layer.h:38-160), its device side (include/base_layer_cuda.cuh:16-78),
// Linear / Conv2d / ReLU and their device forms. The host forms only hold
// parameters and geometry: every computation happens on the GPU behind the C ABI,
// and calling forward/backward/update on a layer that was not moved to the device
// raises (there is no CPU compute path in this library).
#pragma once
#include <fstream>
#include <memory>
#include <random>
#include <string>
#include <tuple>
#include <vector>

#include "../../include/tagi_hip.h"
#include "states.h"

namespace tagi_host {

enum class LayerType { Base, Linear, Conv2d, Activation, Pool2d, Norm, LayerBlock, ResNetBlock };

class InitArgs {
   public:
    size_t width = 0, height = 0, depth = 0;
    int batch_size = 1;
    InitArgs(size_t width = 0, size_t height = 0, size_t depth = 0, int batch_size = 1)
        : width(width), height(height), depth(depth), batch_size(batch_size) {}
};

// Seeded generator shared by every parameter initialisation
// (reference: include/param_init.h:12-31).
class SeedManager {
   public:
    static SeedManager &get_instance() {
        static SeedManager inst;
        return inst;
    }
    void set_seed(int seed) { engine.seed(seed); }
    std::mt19937 &get_engine() { return engine; }

   private:
    SeedManager() : engine(std::random_device{}()) {}
    std::mt19937 engine;
};
void manual_seed(int seed);

// mean ~ N(0, scale^2), variance = (gain*scale)^2 with scale from "He" (1/fan_in)
// or "Xavier" (2/(fan_in+fan_out)); reference: src/param_init.cpp:5-77,158-223.
ParameterTuple init_gaussian_params(const std::string &method, float gain_w, float gain_b,
                                    float fan_in, float fan_out, size_t num_weights,
                                    size_t num_biases);

class BaseLayer {
   public:
    size_t input_size = 0, output_size = 0;
    size_t num_weights = 0, num_biases = 0;
    size_t in_width = 0, in_height = 0, in_channels = 0;
    size_t out_width = 0, out_height = 0, out_channels = 0;
    bool bias = true;
    bool param_update = true;
    float cap_factor_update = 1.0f;
    int neg_var_w_counter = 0;
    int device_idx = 0;

    std::vector<float> mu_w, var_w, mu_b, var_b;
    std::vector<float> delta_mu_w, delta_var_w, delta_mu_b, delta_var_b;
    std::unique_ptr<BaseBackwardStates> bwd_states;
    // One-shot request to the next forward() of a layer that can_fuse_activation():
    // apply this activation (TAGI_ACT_*) in the kernel's epilogue and write its
    // moments and Jacobian instead of the layer's own output. Set by the owner of the
    // layer list when the next layer is that activation; forward() clears it.
    int fused_activation = 0;
    virtual bool can_fuse_activation() const { return false; }

    unsigned int num_threads = 4;
    bool training = true;
    std::string device = "cpu";

    BaseLayer();
    virtual ~BaseLayer() = default;
    BaseLayer(const BaseLayer &) = delete;
    BaseLayer &operator=(const BaseLayer &) = delete;

    virtual std::string get_layer_info() const { return "Base()"; }
    virtual std::string get_layer_name() const { return "Base"; }
    virtual LayerType get_layer_type() const { return LayerType::Base; }
    virtual int get_input_size() { return (int)input_size; }
    virtual int get_output_size() { return (int)output_size; }
    virtual int get_max_num_states() { return (int)std::max(input_size, output_size); }
    virtual std::string get_device() { return device + ":" + std::to_string(device_idx); }

    virtual void init_weight_bias() {}
    virtual void forward(BaseHiddenStates &input_states, BaseHiddenStates &output_states,
                         BaseTempStates &temp_states);
    virtual void backward(BaseDeltaStates &input_delta_states, BaseDeltaStates &output_delta_states,
                          BaseTempStates &temp_states, bool state_udapte = true);
    virtual void allocate_param_delta();
    virtual void update_weights();
    virtual void update_biases();
    // the same steps without the cap and the variance floor
    // (reference: BaseLayer::raw_update_weights / raw_update_biases)
    virtual void raw_update_weights();
    virtual void raw_update_biases();
    // Both of them, as Sequential::step issues them (one launch on the device).
    virtual void update_params() {
        this->update_weights();
        this->update_biases();
    }
    // For Sequential::step: a device layer appends what one tagi_layer_update call
    // would take, so that the whole model is updated in one launch; a layer that
    // cannot describe its update that way performs it on the spot.
    virtual void collect_update_items(std::vector<tagi_update_item> &) { this->update_params(); }
    virtual void set_cap_factor_udapte(int batch_size);
    virtual void set_threads(int num) { num_threads = num; }
    virtual void compute_input_output_size(const InitArgs &args);
    virtual void train() { training = true; }
    virtual void eval() { training = false; }
    virtual void save(std::ofstream &file);
    virtual void load(std::ifstream &file);
    virtual std::unique_ptr<BaseLayer> to_cuda(int device_idx = 0);
    virtual void to(int idx) { device_idx = idx; }
    virtual ParameterMap get_parameters_as_map(std::string suffix = "");
    virtual void load_parameters_from_map(const ParameterMap &param_map,
                                          const std::string &suffix = "");
    virtual std::vector<ParameterTuple> parameters();
    virtual void preinit_layer() {}
    virtual int get_neg_var_w_counter() { return neg_var_w_counter; }
    // Running averages and last batch statistics of the normalisation layers inside
    // this layer, one entry per such layer: (mu_ra, var_ra, mu_norm_batch,
    // var_norm_batch). Empty for everything else (reference: include/base_layer.h,
    // BaseLayer::get_norm_mean_var).
    using NormStats = std::tuple<std::vector<std::vector<float>>, std::vector<std::vector<float>>,
                                 std::vector<std::vector<float>>, std::vector<std::vector<float>>>;
    virtual NormStats get_norm_mean_var() { return NormStats(); }
    // host <-> device copies of the parameters; layers without device storage
    // have nothing to move, blocks pass the call on to their members
    virtual void params_to_device() {}
    virtual void params_to_host() {}
    virtual void delta_params_to_host() {}
    virtual void delta_params_to_device() {}

   protected:
    [[noreturn]] void no_cpu_path(const char *what) const;
};

// Device side shared by every parametrised layer
// (reference: src/base_layer_cuda.cu:105-500).
class BaseLayerHip : public BaseLayer {
   public:
    float *d_mu_w = nullptr, *d_var_w = nullptr, *d_mu_b = nullptr, *d_var_b = nullptr;
    float *d_delta_mu_w = nullptr, *d_delta_var_w = nullptr;
    float *d_delta_mu_b = nullptr, *d_delta_var_b = nullptr;
    int *d_neg_var_count = nullptr;
    // Threads per block of the reference's elementwise launches. Kept so that code
    // written for the reference runs; the kernels here choose their own launch shape.
    unsigned int num_cuda_threads = 16;

    BaseLayerHip();
    ~BaseLayerHip() override;

    void allocate_param_delta() override;
    void update_weights() override;
    void update_biases() override;
    void update_params() override;
    void collect_update_items(std::vector<tagi_update_item> &items) override;
    void raw_update_weights() override;
    void raw_update_biases() override;
    void set_cuda_threads(int num) { num_cuda_threads = (unsigned int)num; }
    void save(std::ofstream &file) override;
    void load(std::ifstream &file) override;
    ParameterMap get_parameters_as_map(std::string suffix = "") override;
    void load_parameters_from_map(const ParameterMap &param_map,
                                  const std::string &suffix = "") override;
    std::vector<ParameterTuple> parameters() override;
    int get_neg_var_w_counter() override;

    void params_to_device() override;
    void params_to_host() override;
    void delta_params_to_host() override;
    void delta_params_to_device() override;
    void copy_params_from(const BaseLayer &source);
    // The host vectors were replaced from outside (state dict, another model): take
    // the layer's sizes from them, make the device storage fit - also on a layer that
    // has not allocated anything yet - and upload.
    void adopt_host_params();

   protected:
    void allocate_param_memory();
    void release_param_memory();
    void store_states_for_training_hip(HiddenStateHip &input_states, HiddenStateHip &output_states);
    size_t alloc_w = 0, alloc_b = 0;  // sizes the device parameter arrays were allocated for
    bool neg_var_dirty = false;
    int neg_var_slot = 0;  // which of the two device counters holds the last update's count
};

// ---- Linear -----------------------------------------------------------------------
class Linear : public BaseLayer {
   public:
    float gain_w, gain_b;
    std::string init_method;

    Linear(size_t ip_size, size_t op_size, bool bias = true, float gain_weight = 1.0f,
           float gain_bias = 1.0f, std::string method = "He", int device_idx = 0);
    std::string get_layer_info() const override;
    std::string get_layer_name() const override { return "Linear"; }
    LayerType get_layer_type() const override { return LayerType::Linear; }
    void init_weight_bias() override;
    std::unique_ptr<BaseLayer> to_cuda(int device_idx = 0) override;
};

class LinearHip : public BaseLayerHip {
   public:
    float gain_w, gain_b;
    std::string init_method;

    LinearHip(size_t ip_size, size_t op_size, bool bias = true, float gain_weight = 1.0f,
              float gain_bias = 1.0f, std::string method = "He", int device_idx = 0);
    std::string get_layer_info() const override;
    // the reference names its device layers *Cuda; state_dict keys derive from this
    std::string get_layer_name() const override { return "LinearCuda"; }
    LayerType get_layer_type() const override { return LayerType::Linear; }
    bool can_fuse_activation() const override { return true; }
    void init_weight_bias() override;
    void forward(BaseHiddenStates &input_states, BaseHiddenStates &output_states,
                 BaseTempStates &temp_states) override;
    void backward(BaseDeltaStates &input_delta_states, BaseDeltaStates &output_delta_states,
                  BaseTempStates &temp_states, bool state_udapte = true) override;
};

// ---- Conv2d -----------------------------------------------------------------------
class Conv2d : public BaseLayer {
   public:
    size_t kernel_size;
    int stride, padding, padding_type;
    float gain_w, gain_b;
    std::string init_method;

    Conv2d(size_t in_channels, size_t out_channels, size_t kernel_size, bool bias = true,
           int stride = 1, int padding = 0, int padding_type = 1, size_t in_width = 0,
           size_t in_height = 0, float gain_w = 1.0f, float gain_b = 1.0f,
           std::string init_method = "He", int device_idx = 0);
    std::string get_layer_info() const override;
    std::string get_layer_name() const override { return "Conv2d"; }
    LayerType get_layer_type() const override { return LayerType::Conv2d; }
    void compute_input_output_size(const InitArgs &args) override;
    void init_weight_bias() override;
    void preinit_layer() override;
    std::unique_ptr<BaseLayer> to_cuda(int device_idx = 0) override;
};

class Conv2dHip : public BaseLayerHip {
   public:
    size_t kernel_size;
    int stride, padding, padding_type;
    float gain_w, gain_b;
    std::string init_method;
    std::vector<int> idx_mwa_2, idx_cov_zwa_1, idx_var_z_ud;
    // One-shot, set by a ResNetBlock whose main block starts with this layer: the next
    // backward() adds the block's residual innovations to its state innovations in the
    // same pass (mode 1: identity shortcut, scaled by this layer's Jacobian like its own
    // sum; mode 2: a shortcut branch's finished innovations). Cleared by backward().
    const float *bwd_residual_mu = nullptr, *bwd_residual_var = nullptr;
    int bwd_residual_mode = 0;
    int row_zw = 0, col_z_ud = 0;
    int *d_idx_mwa_2 = nullptr, *d_idx_cov_zwa_1 = nullptr, *d_idx_var_z_ud = nullptr;

    Conv2dHip(size_t in_channels, size_t out_channels, size_t kernel_size, bool bias = true,
              int stride = 1, int padding = 0, int padding_type = 1, size_t in_width = 0,
              size_t in_height = 0, float gain_w = 1.0f, float gain_b = 1.0f,
              std::string init_method = "He", int device_idx = 0);
    ~Conv2dHip() override;
    std::string get_layer_info() const override;
    std::string get_layer_name() const override { return "Conv2dCuda"; }
    LayerType get_layer_type() const override { return LayerType::Conv2d; }
    bool can_fuse_activation() const override { return true; }
    void compute_input_output_size(const InitArgs &args) override;
    void get_number_param();
    void init_weight_bias() override;
    void lazy_index_init();
    void preinit_layer() override;
    void forward(BaseHiddenStates &input_states, BaseHiddenStates &output_states,
                 BaseTempStates &temp_states) override;
    void backward(BaseDeltaStates &input_delta_states, BaseDeltaStates &output_delta_states,
                  BaseTempStates &temp_states, bool state_udapte = true) override;
};

// ---- ReLU -------------------------------------------------------------------------
class ReLU : public BaseLayer {
   public:
    ReLU() = default;
    std::string get_layer_info() const override { return "ReLU()"; }
    std::string get_layer_name() const override { return "ReLU"; }
    LayerType get_layer_type() const override { return LayerType::Activation; }
    // Activations own no section of a checkpoint file (reference:
    // include/activation.h:142-144).
    void save(std::ofstream &) override {}
    void load(std::ifstream &) override {}
    std::unique_ptr<BaseLayer> to_cuda(int device_idx = 0) override;
};

class ReLUHip : public BaseLayer {
   public:
    ReLUHip() { this->device = "cuda"; }
    std::string get_layer_info() const override { return "Relu()"; }
    std::string get_layer_name() const override { return "ReLUCuda"; }
    LayerType get_layer_type() const override { return LayerType::Activation; }
    // Activations own no section of a checkpoint file (reference:
    // include/activation.h:142-144).
    void save(std::ofstream &) override {}
    void load(std::ifstream &) override {}
    void forward(BaseHiddenStates &input_states, BaseHiddenStates &output_states,
                 BaseTempStates &temp_states) override;
    // Nothing to propagate: the Jacobian rides in the hidden state and is applied
    // by the state backward of the layer below.
    void backward(BaseDeltaStates &, BaseDeltaStates &, BaseTempStates &, bool = true) override {}
    void update_weights() override {}
    void update_biases() override {}
    void update_params() override {}
    std::unique_ptr<BaseLayer> to_cuda(int = 0) override;
};

// Fusion of an activation layer into the forward of the layer before it (the
// reference runs them as two launches with a round trip through memory between
// them). fusable_activation: TAGI_ACT_* when `next` is a device ReLU / MixtureReLU
// that `layer` can absorb and fusion is switched on, else 0. After the fused forward
// the owner calls activation_absorbed so that the skipped layer's sizes read as if it
// had run. set_fused_activations(false) switches the fusion off (tests, comparisons).
int fusable_activation(const BaseLayer *layer, const BaseLayer *next);
void activation_absorbed(BaseLayer *activation, const BaseHiddenStates &output_states);
void set_fused_activations(bool on);

std::tuple<int, int> compute_downsample_img_size_v2(int kernel, int stride, int wi, int hi, int pad,
                                                    int pad_type);

}  // namespace tagi_host

// The layers a TAGI ResNet needs around Conv2d / Linear, mirroring the
// reference's interface: MixtureReLU (include/activation.h), BatchNorm2d
// (include/batchnorm_layer.h), AvgPool2d (include/pooling_layer.h), LayerBlock
// (include/layer_block.h) and ResNetBlock (include/resnet_block.h), each with the
// device form that to_cuda() returns. As for every layer here, the host forms
// only hold configuration and parameters; all arithmetic runs on the GPU behind
// the C ABI.
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "layers.h"

namespace tagi_host {

// ---- MixtureReLU ---------------------------------------------------------------------
class MixtureReLU : public BaseLayer {
   public:
    MixtureReLU() = default;
    std::string get_layer_info() const override { return "MixtureReLU()"; }
    std::string get_layer_name() const override { return "MixtureReLU"; }
    LayerType get_layer_type() const override { return LayerType::Activation; }
    // Activations own no section of a checkpoint file (reference:
    // include/activation.h:142-144).
    void save(std::ofstream &) override {}
    void load(std::ifstream &) override {}
    std::unique_ptr<BaseLayer> to_cuda(int device_idx = 0) override;
};

class MixtureReLUHip : public BaseLayer {
   public:
    MixtureReLUHip() { this->device = "cuda"; }
    std::string get_layer_info() const override { return "MixtureReLU()"; }
    std::string get_layer_name() const override { return "MixtureReLUCuda"; }
    LayerType get_layer_type() const override { return LayerType::Activation; }
    // Activations own no section of a checkpoint file (reference:
    // include/activation.h:142-144).
    void save(std::ofstream &) override {}
    void load(std::ifstream &) override {}
    void forward(BaseHiddenStates &input_states, BaseHiddenStates &output_states,
                 BaseTempStates &temp_states) override;
    void backward(BaseDeltaStates &, BaseDeltaStates &, BaseTempStates &, bool = true) override {}
    void update_weights() override {}
    void update_biases() override {}
    void update_params() override {}
    std::unique_ptr<BaseLayer> to_cuda(int device_idx = 0) override;
};

// ---- BatchNorm2d -----------------------------------------------------------------------
class BatchNorm2d : public BaseLayer {
   public:
    int num_features;
    std::vector<float> mu_ra, var_ra, mu_norm_batch, var_norm_batch;
    NormStats get_norm_mean_var() override {
        return NormStats({mu_ra}, {var_ra}, {mu_norm_batch}, {var_norm_batch});
    }
    float epsilon, momentum, gain_w, gain_b;

    BatchNorm2d(int num_features, float eps = 1e-5f, float momentum = 0.9f, bool bias = true,
                float gain_weight = 1.0f, float gain_bias = 1.0f, int device_idx = 0);
    std::string get_layer_info() const override { return "BatchNorm2d()"; }
    std::string get_layer_name() const override { return "BatchNorm2d"; }
    LayerType get_layer_type() const override { return LayerType::Norm; }
    void init_weight_bias() override;
    void save(std::ofstream &file) override;
    void load(std::ifstream &file) override;
    std::unique_ptr<BaseLayer> to_cuda(int device_idx = 0) override;
};

class BatchNorm2dHip : public BaseLayerHip {
   public:
    int num_features;
    std::vector<float> mu_ra, var_ra, mu_norm_batch, var_norm_batch;
    float *d_mu_ra = nullptr, *d_var_ra = nullptr;
    float *d_mu_norm_batch = nullptr, *d_var_norm_batch = nullptr;
    float epsilon, momentum, gain_w, gain_b;
    // One-shot, set by a ResNetBlock whose main block ends on this layer: the next
    // forward() adds these arrays (the shortcut's output) to its own output.
    const float *residual_mu = nullptr, *residual_var = nullptr;

    BatchNorm2dHip(int num_features, float eps = 1e-5f, float momentum = 0.9f, bool bias = true,
                   float gain_weight = 1.0f, float gain_bias = 1.0f, int device_idx = 0);
    ~BatchNorm2dHip() override;
    std::string get_layer_info() const override { return "BatchNorm2d()"; }
    std::string get_layer_name() const override { return "BatchNorm2dCuda"; }
    LayerType get_layer_type() const override { return LayerType::Norm; }
    void init_weight_bias() override;
    void forward(BaseHiddenStates &input_states, BaseHiddenStates &output_states,
                 BaseTempStates &temp_states) override;
    void backward(BaseDeltaStates &input_delta_states, BaseDeltaStates &output_delta_states,
                  BaseTempStates &temp_states, bool state_udapte = true) override;
    void save(std::ofstream &file) override;
    void load(std::ifstream &file) override;
    void running_mean_var_to_host();
    void running_mean_var_to_device();
    // refreshed from the device
    NormStats get_norm_mean_var() override;

   private:
    void allocate_running_mean_var();
};

// ---- AvgPool2d -------------------------------------------------------------------------
class AvgPool2d : public BaseLayer {
   public:
    size_t kernel_size;
    int stride, padding_type, padding;

    AvgPool2d(size_t kernel_size, int stride = -1, int padding = 0, int padding_type = 0,
              int device_idx = 0);
    std::string get_layer_info() const override;
    std::string get_layer_name() const override { return "AvgPool2d"; }
    LayerType get_layer_type() const override { return LayerType::Pool2d; }
    void compute_input_output_size(const InitArgs &args) override;
    void allocate_param_delta() override {}
    std::unique_ptr<BaseLayer> to_cuda(int device_idx = 0) override;
};

class AvgPool2dHip : public BaseLayerHip {
   public:
    size_t kernel_size;
    int stride, padding_type, padding;
    std::vector<int> pool_idx, z_ud_idx;
    int *d_pool_idx = nullptr, *d_z_ud_idx = nullptr;
    size_t row_zw = 0, col_z_ud = 0;
    bool overlap = true;

    AvgPool2dHip(size_t kernel_size, int stride = -1, int padding = 0, int padding_type = 0,
                 int device_idx = 0);
    ~AvgPool2dHip() override;
    std::string get_layer_info() const override;
    std::string get_layer_name() const override { return "AvgPool2dCuda"; }
    LayerType get_layer_type() const override { return LayerType::Pool2d; }
    void compute_input_output_size(const InitArgs &args) override;
    void forward(BaseHiddenStates &input_states, BaseHiddenStates &output_states,
                 BaseTempStates &temp_states) override;
    void backward(BaseDeltaStates &input_delta_states, BaseDeltaStates &output_delta_states,
                  BaseTempStates &temp_states, bool state_udapte = true) override;
    void allocate_param_delta() override {}
    void update_weights() override {}
    void update_biases() override {}
    void update_params() override {}
    void preinit_layer() override;
    void params_to_device() override {}
    void params_to_host() override {}

   private:
    void lazy_index_init();
};

// ---- LayerBlock --------------------------------------------------------------------------
// A run of layers used as one layer. It has no device form of its own: to_cuda()
// moves its members and returns the same kind of object.
class LayerBlock : public BaseLayer {
   public:
    std::vector<std::shared_ptr<BaseLayer>> layers;
    // One-shot requests of an enclosing ResNetBlock: the next forward() lets its first
    // layer read this state, the next backward() lets its last layer read these
    // innovations, instead of the first argument - which then only serves as the second
    // ping-pong buffer. The enclosing block keeps the named object unchanged, so nothing
    // has to be copied to protect it from the block's own passes.
    BaseHiddenStates *first_input = nullptr;
    BaseDeltaStates *first_delta_input = nullptr;

    LayerBlock() = default;
    explicit LayerBlock(const std::vector<std::shared_ptr<BaseLayer>> &layers);
    void add_layer(std::shared_ptr<BaseLayer> layer);
    void add_layers();
    void switch_to_cuda();

    std::string get_layer_info() const override;
    std::string get_layer_name() const override { return "LayerBlock"; }
    LayerType get_layer_type() const override { return LayerType::LayerBlock; }
    int get_max_num_states() override;
    std::string get_device() override;
    void init_weight_bias() override;
    void set_threads(int num) override;
    void train() override;
    void eval() override;
    void forward(BaseHiddenStates &input_states, BaseHiddenStates &output_states,
                 BaseTempStates &temp_states) override;
    void backward(BaseDeltaStates &input_delta_states, BaseDeltaStates &output_delta_states,
                  BaseTempStates &temp_states, bool state_update = true) override;
    void update_weights() override;
    void update_biases() override;
    void update_params() override;
    void collect_update_items(std::vector<tagi_update_item> &items) override;
    void compute_input_output_size(const InitArgs &args) override;
    void save(std::ofstream &file) override;
    void load(std::ifstream &file) override;
    ParameterMap get_parameters_as_map(std::string suffix = "") override;
    void load_parameters_from_map(const ParameterMap &param_map,
                                  const std::string &suffix = "") override;
    std::vector<ParameterTuple> parameters() override;
    std::unique_ptr<BaseLayer> to_cuda(int device_idx = 0) override;
    void preinit_layer() override;
    int get_neg_var_w_counter() override;
    NormStats get_norm_mean_var() override;
    void params_to_device() override;
    void params_to_host() override;
    void delta_params_to_host() override;
};

// ---- ResNetBlock -------------------------------------------------------------------------
// output = main_block(input) + shortcut(input), the shortcut being the identity
// when none is given.
class ResNetBlock : public BaseLayer {
   public:
    std::shared_ptr<BaseLayer> main_block;
    std::shared_ptr<BaseLayer> shortcut;
    std::shared_ptr<BaseHiddenStates> input_z, shortcut_output_z;
    std::shared_ptr<BaseDeltaStates> input_delta_z, shortcut_output_delta_z;

    ResNetBlock(std::shared_ptr<BaseLayer> main_block, std::shared_ptr<BaseLayer> shortcut = nullptr);
    std::string get_layer_info() const override;
    std::string get_layer_name() const override { return "ResNetBlock"; }
    LayerType get_layer_type() const override { return LayerType::ResNetBlock; }
    int get_max_num_states() override;
    std::string get_device() override;
    void compute_input_output_size(const InitArgs &args) override;
    void init_weight_bias() override;
    void set_threads(int num) override;
    void train() override;
    void eval() override;
    void forward(BaseHiddenStates &input_states, BaseHiddenStates &output_states,
                 BaseTempStates &temp_states) override;
    void backward(BaseDeltaStates &input_delta_states, BaseDeltaStates &output_delta_states,
                  BaseTempStates &temp_states, bool state_update = true) override;
    void update_weights() override;
    void update_biases() override;
    void update_params() override;
    void collect_update_items(std::vector<tagi_update_item> &items) override;
    void save(std::ofstream &file) override;
    void load(std::ifstream &file) override;
    ParameterMap get_parameters_as_map(std::string suffix = "") override;
    void load_parameters_from_map(const ParameterMap &param_map,
                                  const std::string &suffix = "") override;
    std::vector<ParameterTuple> parameters() override;
    std::unique_ptr<BaseLayer> to_cuda(int device_idx = 0) override;
    void preinit_layer() override;
    int get_neg_var_w_counter() override;
    NormStats get_norm_mean_var() override;
    void params_to_device() override;
    void params_to_host() override;
    void delta_params_to_host() override;

   protected:
    bool on_device = false;
    int batch_size_ = 0;
    size_t buffer_size_ = 0;
    // buffers of `size` floats per array (0: what the block's own layers need)
    void init_buffers(size_t size = 0);
    // both branches are LayerBlocks (or the shortcut is the identity): they can be told to
    // read the block's own copy of its input, so that copy can be a trade of arrays
    bool can_trade() const;
};

// Device form: same object layout, device state buffers, residual adds on the GPU.
class ResNetBlockHip : public ResNetBlock {
   public:
    ResNetBlockHip(std::shared_ptr<BaseLayer> main_block, std::shared_ptr<BaseLayer> shortcut,
                   int device_idx);
    std::string get_layer_info() const override;
    std::string get_layer_name() const override { return "ResNetBlockCuda"; }
    std::unique_ptr<BaseLayer> to_cuda(int device_idx = 0) override;
};

}  // namespace tagi_host

// MixtureReLU, BatchNorm2d, AvgPool2d, LayerBlock and ResNetBlock: see blocks.h.
#include "blocks.h"

#include <algorithm>

#include "../../include/tagi_hip.h"
#include "host_util.h"
#include "logger.h"

namespace tagi_host {

namespace {
void set_output_dims(BaseHiddenStates &out, const BaseLayer &layer, size_t batch_size) {
    out.width = layer.out_width;
    out.height = layer.out_height;
    out.depth = layer.out_channels;
    out.block_size = batch_size;
    out.actual_size = layer.output_size;
}
}  // namespace

// ---- MixtureReLU ---------------------------------------------------------------------
std::unique_ptr<BaseLayer> MixtureReLU::to_cuda(int device_idx) {
    this->device = "cuda";
    auto layer = std::make_unique<MixtureReLUHip>();
    layer->device_idx = device_idx;
    return layer;
}

std::unique_ptr<BaseLayer> MixtureReLUHip::to_cuda(int device_idx) {
    auto layer = std::make_unique<MixtureReLUHip>();
    layer->device_idx = device_idx;
    return layer;
}

// ---- activation fusion --------------------------------------------------------------------
static bool g_fused_activations = true;
void set_fused_activations(bool on) { g_fused_activations = on; }

int fusable_activation(const BaseLayer *layer, const BaseLayer *next) {
    if (!g_fused_activations || layer == nullptr || next == nullptr) return 0;
    if (!layer->can_fuse_activation()) return 0;
    if (dynamic_cast<const ReLUHip *>(next) != nullptr) return TAGI_ACT_RELU;
    if (dynamic_cast<const MixtureReLUHip *>(next) != nullptr) return TAGI_ACT_MIXTURE_RELU;
    return 0;
}

void activation_absorbed(BaseLayer *activation, const BaseHiddenStates &output_states) {
    activation->input_size = output_states.actual_size;
    activation->output_size = output_states.actual_size;
}

// reference: MixtureReLUCuda::forward, src/activation_cuda.cu:726-760
void MixtureReLUHip::forward(BaseHiddenStates &input_states, BaseHiddenStates &output_states,
                             BaseTempStates &) {
    auto *in = as<HiddenStateHip>(input_states);
    auto *out = as<HiddenStateHip>(output_states);
    const size_t n = input_states.actual_size * input_states.block_size;
    if (n > out->size) LOG(LogLevel::ERROR, "Output state buffer too small for MixtureReLU");
    TAGI_OK_OR_THROW(tagi_mixture_relu_fwd(in->d_mu_a, in->d_var_a, n, out->d_mu_a, out->d_jcb,
                                           out->d_var_a, host_stream()));
    out->jcb_ones = false;
    this->input_size = input_states.actual_size;
    this->output_size = input_states.actual_size;
    output_states.block_size = input_states.block_size;
    output_states.actual_size = input_states.actual_size;
    output_states.width = input_states.width;
    output_states.height = input_states.height;
    output_states.depth = input_states.depth;
}

// ---- BatchNorm2d -----------------------------------------------------------------------
namespace {
// weights start at one with variance 2/(in+out) * gain^2, biases at zero
// (reference: init_weight_bias_norm, src/param_init.cpp:225-242)
void init_norm_params(int nf, bool bias, float gain_w, float gain_b, std::vector<float> &mu_w,
                      std::vector<float> &var_w, std::vector<float> &mu_b,
                      std::vector<float> &var_b) {
    const float scale = 2.0f / (nf + nf);
    mu_w.assign(nf, 1.0f);
    var_w.assign(nf, scale * gain_w * gain_w);
    mu_b.clear();
    var_b.clear();
    if (bias) {
        mu_b.assign(nf, 0.0f);
        var_b.assign(nf, scale * gain_b * gain_b);
    }
}
}  // namespace

BatchNorm2d::BatchNorm2d(int num_features, float eps, float momentum, bool bias, float gain_weight,
                         float gain_bias, int device_idx)
    : num_features(num_features), epsilon(eps), momentum(momentum), gain_w(gain_weight),
      gain_b(gain_bias) {
    this->bias = bias;
    this->device_idx = device_idx;
    this->init_weight_bias();
    mu_ra.assign(num_features, 0.0f);
    var_ra.assign(num_features, 1.0f);
    mu_norm_batch.assign(num_features, 0.0f);
    var_norm_batch.assign(num_features, 0.0f);
    if (this->training) this->allocate_param_delta();
}

void BatchNorm2d::init_weight_bias() {
    this->num_weights = num_features;
    this->num_biases = bias ? num_features : 0;
    init_norm_params(num_features, bias, gain_w, gain_b, mu_w, var_w, mu_b, var_b);
}

// The running averages follow the parameters in the file
// (reference: src/batchnorm_layer.cpp:1140-1229).
void BatchNorm2d::save(std::ofstream &file) {
    BaseLayer::save(file);
    write_floats(file, mu_ra);
    write_floats(file, var_ra);
}

void BatchNorm2d::load(std::ifstream &file) {
    BaseLayer::load(file);
    read_floats(file, mu_ra);
    read_floats(file, var_ra);
}

std::unique_ptr<BaseLayer> BatchNorm2d::to_cuda(int device_idx) {
    this->device = "cuda";
    this->device_idx = device_idx;
    auto layer = std::make_unique<BatchNorm2dHip>(num_features, epsilon, momentum, bias, gain_w,
                                                  gain_b, device_idx);
    layer->copy_params_from(*this);
    layer->mu_ra = mu_ra;
    layer->var_ra = var_ra;
    layer->running_mean_var_to_device();
    return layer;
}

BatchNorm2dHip::BatchNorm2dHip(int num_features, float eps, float momentum, bool bias,
                               float gain_weight, float gain_bias, int device_idx)
    : num_features(num_features), epsilon(eps), momentum(momentum), gain_w(gain_weight),
      gain_b(gain_bias) {
    this->bias = bias;
    this->device_idx = device_idx;
    this->num_weights = num_features;
    this->num_biases = bias ? num_features : 0;
    this->init_weight_bias();
    this->allocate_running_mean_var();
    if (this->training) this->allocate_param_delta();
}

BatchNorm2dHip::~BatchNorm2dHip() {
    dev_free_t(d_mu_ra);
    dev_free_t(d_var_ra);
    dev_free_t(d_mu_norm_batch);
    dev_free_t(d_var_norm_batch);
}

void BatchNorm2dHip::init_weight_bias() {
    init_norm_params(num_features, bias, gain_w, gain_b, mu_w, var_w, mu_b, var_b);
    this->allocate_param_memory();
    this->params_to_device();
}

void BatchNorm2dHip::allocate_running_mean_var() {
    mu_ra.assign(num_features, 0.0f);
    var_ra.assign(num_features, 1.0f);
    mu_norm_batch.assign(num_features, 0.0f);
    var_norm_batch.assign(num_features, 0.0f);
    d_mu_ra = dev_alloc_t<float>(num_features, device_idx);
    d_var_ra = dev_alloc_t<float>(num_features, device_idx);
    d_mu_norm_batch = dev_alloc_t<float>(num_features, device_idx);
    d_var_norm_batch = dev_alloc_t<float>(num_features, device_idx);
    this->running_mean_var_to_device();
}

void BatchNorm2dHip::running_mean_var_to_device() {
    h2d(d_mu_ra, mu_ra);
    h2d(d_var_ra, var_ra);
    h2d(d_mu_norm_batch, mu_norm_batch);
    h2d(d_var_norm_batch, var_norm_batch);
}

void BatchNorm2dHip::running_mean_var_to_host() {
    d2h(mu_ra, d_mu_ra, num_features);
    d2h(var_ra, d_var_ra, num_features);
    d2h(mu_norm_batch, d_mu_norm_batch, num_features);
    d2h(var_norm_batch, d_var_norm_batch, num_features);
}

BaseLayer::NormStats BatchNorm2dHip::get_norm_mean_var() {
    this->running_mean_var_to_host();
    return NormStats({mu_ra}, {var_ra}, {mu_norm_batch}, {var_norm_batch});
}

// appends the entries of `from` to `to`
static void append_norm_stats(BaseLayer::NormStats &to, const BaseLayer::NormStats &from) {
    auto add = [](std::vector<std::vector<float>> &a, const std::vector<std::vector<float>> &b) {
        a.insert(a.end(), b.begin(), b.end());
    };
    add(std::get<0>(to), std::get<0>(from));
    add(std::get<1>(to), std::get<1>(from));
    add(std::get<2>(to), std::get<2>(from));
    add(std::get<3>(to), std::get<3>(from));
}

// reference: BatchNorm2dCuda::forward, src/batchnorm_layer_cuda.cu:832-967. After a
// convolution the statistics are per channel over (batch, pixels); after a
// fully-connected layer the same kernels run with one "pixel" per feature. The
// running averages always move with the layer's momentum, as in the reference's
// device path and its default (multi-threaded) host path.
void BatchNorm2dHip::forward(BaseHiddenStates &input_states, BaseHiddenStates &output_states,
                             BaseTempStates &) {
    // (the one-shot residual request is taken before anything can throw)
    const float *res_mu = this->residual_mu, *res_var = this->residual_var;
    this->residual_mu = this->residual_var = nullptr;
    auto *in = as<HiddenStateHip>(input_states);
    auto *out = as<HiddenStateHip>(output_states);
    const int batch_size = (int)input_states.block_size;
    this->set_cap_factor_udapte(batch_size);
    if (this->input_size == 0 || this->output_size == 0) {
        this->input_size = input_states.actual_size;
        this->output_size = input_states.actual_size;
    }
    const bool per_channel = (size_t)num_features == in_channels;
    const int fi = per_channel ? (int)in_channels : (int)this->input_size;
    const int wihi = per_channel ? (int)(in_width * in_height) : 1;
    if (fi != num_features)
        LOG(LogLevel::ERROR, "BatchNorm2d(" + std::to_string(num_features) + ") received " +
                                 std::to_string(fi) + " features");
    if ((size_t)wihi * fi != input_states.actual_size)
        LOG(LogLevel::ERROR, "Input size mismatch: " + std::to_string((size_t)wihi * fi) + " vs " +
                                 std::to_string(input_states.actual_size));
    if (input_states.actual_size * batch_size > out->size)
        LOG(LogLevel::ERROR, "Output state buffer too small for " + this->get_layer_info());

    output_states.width = this->out_width;
    output_states.height = this->out_height;
    output_states.depth = this->out_channels;
    output_states.block_size = batch_size;
    output_states.actual_size = this->output_size;

    if (this->training) {
        if (batch_size * wihi < 2)
            LOG(LogLevel::ERROR, "BatchNorm2d needs more than one value per feature in training");
        // statistics, running averages and the normalisation (+ the residual add) in one call
        TAGI_OK_OR_THROW(tagi_batchnorm2d_fwd_train(
            d_mu_w, d_var_w, d_mu_b, d_var_b, in->d_mu_a, in->d_var_a, res_mu, res_var,
            bias ? 1 : 0, momentum, epsilon, wihi, fi, batch_size, d_mu_norm_batch, d_var_norm_batch,
            d_mu_ra, d_var_ra, out->d_mu_a, out->d_var_a, host_stream()));
    } else if (res_mu != nullptr) {
        TAGI_OK_OR_THROW(tagi_batchnorm2d_fwd_res(d_mu_w, d_var_w, d_mu_b, d_var_b, in->d_mu_a,
                                                  in->d_var_a, d_mu_ra, d_var_ra, res_mu, res_var,
                                                  bias ? 1 : 0, epsilon, wihi, fi, batch_size,
                                                  out->d_mu_a, out->d_var_a, host_stream()));
    } else {
        TAGI_OK_OR_THROW(tagi_batchnorm2d_fwd(d_mu_w, d_var_w, d_mu_b, d_var_b, in->d_mu_a,
                                              in->d_var_a, d_mu_ra, d_var_ra, bias ? 1 : 0, epsilon,
                                              wihi, fi, batch_size, out->d_mu_a, out->d_var_a,
                                              host_stream()));
    }
    out->jcb_ones = true;
    if (this->training) this->store_states_for_training_hip(*in, *out);
}

// reference: BatchNorm2dCuda::backward, src/batchnorm_layer_cuda.cu:969-1102
void BatchNorm2dHip::backward(BaseDeltaStates &input_delta_states,
                              BaseDeltaStates &output_delta_states, BaseTempStates &,
                              bool state_udapte) {
    auto *din = as<DeltaStateHip>(input_delta_states);
    auto *dout = as<DeltaStateHip>(output_delta_states);
    auto *bwd = dynamic_cast<BackwardStateHip *>(this->bwd_states.get());
    const int batch_size = (int)input_delta_states.block_size;
    const bool per_channel = (size_t)num_features == in_channels;
    const int fi = per_channel ? (int)in_channels : (int)this->input_size;
    const int wihi = per_channel ? (int)(in_width * in_height) : 1;
    if (state_udapte && (size_t)wihi * fi * batch_size > dout->size)
        LOG(LogLevel::ERROR, "Delta state buffer too small for " + this->get_layer_info());
    TAGI_OK_OR_THROW(tagi_batchnorm2d_bwd(
        d_mu_w, d_var_w, d_var_b, bwd->d_mu_a, bwd->jcb_ptr(), d_mu_norm_batch, d_var_norm_batch,
        din->d_delta_mu, din->d_delta_var, epsilon, wihi, fi, batch_size, bias ? 1 : 0,
        state_udapte ? 1 : 0, param_update ? 1 : 0, dout->d_delta_mu, dout->d_delta_var,
        d_delta_mu_w, d_delta_var_w, d_delta_mu_b, d_delta_var_b, host_stream()));
}

void BatchNorm2dHip::save(std::ofstream &file) {
    BaseLayerHip::save(file);
    this->running_mean_var_to_host();
    write_floats(file, mu_ra);
    write_floats(file, var_ra);
}

void BatchNorm2dHip::load(std::ifstream &file) {
    BaseLayerHip::load(file);
    read_floats(file, mu_ra);
    read_floats(file, var_ra);
    this->running_mean_var_to_device();
}

// ---- AvgPool2d -------------------------------------------------------------------------
AvgPool2d::AvgPool2d(size_t kernel_size, int stride, int padding, int padding_type, int device_idx)
    : kernel_size(kernel_size), stride(stride), padding_type(padding_type), padding(padding) {
    this->device_idx = device_idx;
}

std::string AvgPool2d::get_layer_info() const {
    return "AvgPool2d(" + std::to_string(in_channels) + "," + std::to_string(out_channels) + "," +
           std::to_string(out_width) + "," + std::to_string(out_height) + "," +
           std::to_string(kernel_size) + ")";
}

// reference: src/pooling_layer.cpp:42-59
void AvgPool2d::compute_input_output_size(const InitArgs &args) {
    in_width = args.width;
    in_height = args.height;
    in_channels = out_channels = args.depth;
    std::tie(out_width, out_height) = compute_downsample_img_size_v2(
        (int)kernel_size, stride, (int)in_width, (int)in_height, padding, padding_type);
    input_size = in_width * in_width * in_channels;
    output_size = out_width * out_height * out_channels;
}

std::unique_ptr<BaseLayer> AvgPool2d::to_cuda(int device_idx) {
    this->device = "cuda";
    this->device_idx = device_idx;
    return std::make_unique<AvgPool2dHip>(kernel_size, stride, padding, padding_type, device_idx);
}

AvgPool2dHip::AvgPool2dHip(size_t kernel_size, int stride, int padding, int padding_type,
                           int device_idx)
    : kernel_size(kernel_size), stride(stride), padding_type(padding_type), padding(padding) {
    this->device_idx = device_idx;
    this->bias = false;
}

AvgPool2dHip::~AvgPool2dHip() {
    dev_free_t(d_pool_idx);
    dev_free_t(d_z_ud_idx);
}

std::string AvgPool2dHip::get_layer_info() const {
    return "AvgPool2d(" + std::to_string(in_channels) + "," + std::to_string(out_channels) + "," +
           std::to_string(out_width) + "," + std::to_string(out_height) + "," +
           std::to_string(kernel_size) + ")";
}

void AvgPool2dHip::compute_input_output_size(const InitArgs &args) {
    in_width = args.width;
    in_height = args.height;
    in_channels = out_channels = args.depth;
    std::tie(out_width, out_height) = compute_downsample_img_size_v2(
        (int)kernel_size, stride, (int)in_width, (int)in_height, padding, padding_type);
    input_size = in_width * in_width * in_channels;
    output_size = out_width * out_height * out_channels;
}

// reference: AvgPool2dCuda::lazy_index_init, src/pooling_layer_cuda.cu:272-327
void AvgPool2dHip::lazy_index_init() {
    const int k2 = (int)(kernel_size * kernel_size);
    pool_idx.assign(out_width * out_height * k2, 0);
    z_ud_idx.assign(in_width * in_height * k2, 0);
    int w = 0, h = 0, ov = 0;
    if (tagi_avgpool2d_build_idx((int)kernel_size, stride, (int)in_width, (int)in_height, padding,
                                 padding_type, pool_idx.data(), z_ud_idx.data(), &w, &h,
                                 &ov) != TAGI_OK)
        LOG(LogLevel::ERROR, "Cannot build the index tables of " + this->get_layer_info());
    overlap = ov != 0;
    z_ud_idx.resize((size_t)w * h);
    row_zw = w;
    col_z_ud = h;
    if (overlap && (size_t)w != in_width * in_height)
        LOG(LogLevel::ERROR, "AvgPool2d geometry leaves input pixels unused; not supported");
    auto upload = [&](int *&d, const std::vector<int> &v) {
        dev_free_t(d);
        if (v.empty()) return;
        d = dev_alloc_t<int>(v.size(), device_idx);
        HIP_OK(hipMemcpy(d, v.data(), v.size() * sizeof(int), hipMemcpyHostToDevice));
    };
    upload(d_pool_idx, pool_idx);
    upload(d_z_ud_idx, z_ud_idx);
}

void AvgPool2dHip::preinit_layer() {
    if (pool_idx.empty()) this->lazy_index_init();
}

// reference: AvgPool2dCuda::forward, src/pooling_layer_cuda.cu:167-218
void AvgPool2dHip::forward(BaseHiddenStates &input_states, BaseHiddenStates &output_states,
                           BaseTempStates &) {
    auto *in = as<HiddenStateHip>(input_states);
    auto *out = as<HiddenStateHip>(output_states);
    const int batch_size = (int)input_states.block_size;
    if (pool_idx.empty()) this->lazy_index_init();
    if (this->input_size != input_states.actual_size)
        LOG(LogLevel::ERROR, "Input size mismatch: " + std::to_string(this->input_size) + " vs " +
                                 std::to_string(input_states.actual_size));
    if (this->output_size * batch_size > out->size)
        LOG(LogLevel::ERROR, "Output state buffer too small for " + this->get_layer_info());
    set_output_dims(output_states, *this, batch_size);
    const int woho = (int)(out_width * out_height), wihi = (int)(in_width * in_height);
    TAGI_OK_OR_THROW(tagi_avgpool2d_fwd(in->d_mu_a, in->d_var_a, d_pool_idx, woho, wihi,
                                        (int)kernel_size, woho * (int)out_channels * batch_size,
                                        out->d_mu_a, out->d_var_a, host_stream()));
    out->jcb_ones = true;
    if (this->training) this->store_states_for_training_hip(*in, *out);
}

// reference: AvgPool2dCuda::backward, src/pooling_layer_cuda.cu:220-270
void AvgPool2dHip::backward(BaseDeltaStates &input_delta_states,
                            BaseDeltaStates &output_delta_states, BaseTempStates &,
                            bool state_udapte) {
    if (!state_udapte) return;
    auto *din = as<DeltaStateHip>(input_delta_states);
    auto *dout = as<DeltaStateHip>(output_delta_states);
    auto *bwd = dynamic_cast<BackwardStateHip *>(this->bwd_states.get());
    const int batch_size = (int)input_delta_states.block_size;
    const int woho = (int)(out_width * out_height), wihi = (int)(in_width * in_height);
    const int n_in = wihi * (int)in_channels * batch_size;
    if ((size_t)n_in > dout->size)
        LOG(LogLevel::ERROR, "Delta state buffer too small for " + this->get_layer_info());
    TAGI_OK_OR_THROW(tagi_avgpool2d_bwd_dz(bwd->jcb_ptr(), din->d_delta_mu, din->d_delta_var,
                                           d_z_ud_idx, woho, wihi, (int)kernel_size,
                                           (int)col_z_ud, (int)out_width, n_in, overlap ? 1 : 0,
                                           dout->d_delta_mu, dout->d_delta_var, host_stream()));
}

// ---- LayerBlock --------------------------------------------------------------------------
LayerBlock::LayerBlock(const std::vector<std::shared_ptr<BaseLayer>> &list) {
    for (const auto &layer : list) this->add_layer(layer);
    this->add_layers();
}

void LayerBlock::add_layer(std::shared_ptr<BaseLayer> layer) {
    if (this->device == "cpu")
        this->layers.push_back(std::move(layer));
    else if (this->device == "cuda")
        this->layers.push_back(layer->to_cuda(this->device_idx));
    else
        LOG(LogLevel::ERROR, "Invalid device: [" + this->device + "]");
}

// reference: src/layer_block.cpp:13-27
void LayerBlock::add_layers() {
    if (layers.empty()) return;
    this->input_size = layers.front()->input_size;
    this->output_size = layers.back()->output_size;
    LayerType type = layers.back()->get_layer_type();
    int i = (int)layers.size() - 2;
    while (type == LayerType::Activation && i >= 0) {
        this->output_size = layers[i]->output_size;
        type = layers[i]->get_layer_type();
        i--;
    }
}

void LayerBlock::switch_to_cuda() {
    for (auto &layer : layers) layer = layer->to_cuda(this->device_idx);
}

std::string LayerBlock::get_layer_info() const {
    return "LayerBlock(" + std::to_string(input_size) + "," + std::to_string(output_size) + ")";
}

int LayerBlock::get_max_num_states() {
    int max_size = 0;
    for (const auto &layer : layers) max_size = std::max(max_size, layer->get_max_num_states());
    return max_size;
}

std::string LayerBlock::get_device() {
    const std::string block_device = this->device + ":" + std::to_string(this->device_idx);
    for (auto &layer : layers) {
        const std::string d = layer->get_device();
        if (d != block_device)
            LOG(LogLevel::ERROR, "Layer device [" + d + "] does not match block device [" +
                                     block_device + "]");
    }
    return block_device;
}

void LayerBlock::init_weight_bias() {
    for (auto &layer : layers) layer->init_weight_bias();
}
void LayerBlock::set_threads(int num) {
    for (auto &layer : layers) layer->set_threads(num);
}
void LayerBlock::train() {
    this->training = true;
    for (auto &layer : layers) layer->train();
}
void LayerBlock::eval() {
    this->training = false;
    for (auto &layer : layers) layer->eval();
}

// reference: src/layer_block.cpp:151-183. The two buffers are used in turn; after
// an even number of layers the result sits in the caller's input object, so the
// two objects trade contents.
void LayerBlock::forward(BaseHiddenStates &input_states, BaseHiddenStates &output_states,
                         BaseTempStates &temp_states) {
    BaseHiddenStates *first = this->first_input;  // one-shot: taken before anything can throw
    this->first_input = nullptr;
    BaseHiddenStates *in = &input_states, *out = &output_states;
    const size_t batch_size = first != nullptr ? first->block_size : input_states.block_size;
    size_t passes = 0;
    for (size_t i = 0; i < layers.size(); i++, passes++) {
        // an activation that follows a Linear / Conv2d layer runs in that layer's epilogue
        const int act = i + 1 < layers.size()
                            ? fusable_activation(layers[i].get(), layers[i + 1].get())
                            : 0;
        layers[i]->fused_activation = act;
        layers[i]->forward(i == 0 && first != nullptr ? *first : *in, *out, temp_states);
        if (act != 0) activation_absorbed(layers[++i].get(), *out);
        std::swap(in, out);
    }
    if (passes % 2 == 0) output_states.swap(input_states);
    set_output_dims(output_states, *this, batch_size);
}

// reference: src/layer_block.cpp:185-220
void LayerBlock::backward(BaseDeltaStates &input_delta_states,
                          BaseDeltaStates &output_delta_states, BaseTempStates &temp_states,
                          bool state_update) {
    // (one-shot request: the innovations arrive in another object than the first buffer)
    BaseDeltaStates *src = this->first_delta_input != nullptr ? this->first_delta_input
                                                              : &input_delta_states;
    this->first_delta_input = nullptr;
    for (auto it = layers.rbegin(); it != layers.rend() - 1; ++it) {
        BaseLayer *layer = it->get();
        layer->backward(*src, output_delta_states, temp_states);
        if (layer->get_layer_type() != LayerType::Activation) {
            input_delta_states.swap(output_delta_states);
            src = &input_delta_states;
        }
    }
    if (state_update && layers.size() > 1)
        layers[0]->backward(*src, output_delta_states, temp_states, state_update);
    if (layers[0]->get_layer_type() == LayerType::Activation || !state_update ||
        layers.size() == 1)
        output_delta_states.swap(input_delta_states);
}

void LayerBlock::update_weights() {
    for (auto &layer : layers)
        if (layer->get_layer_type() != LayerType::Activation) layer->update_weights();
}
void LayerBlock::update_biases() {
    for (auto &layer : layers)
        if (layer->get_layer_type() != LayerType::Activation) layer->update_biases();
}

void LayerBlock::update_params() {
    for (auto &layer : layers)
        if (layer->get_layer_type() != LayerType::Activation) layer->update_params();
}

void LayerBlock::compute_input_output_size(const InitArgs &args) {
    in_channels = args.depth;
    in_height = args.height;
    in_width = args.width;
    InitArgs tmp(args.width, args.height, args.depth);
    for (auto &layer : layers) {
        layer->compute_input_output_size(tmp);
        tmp.width = layer->out_width;
        tmp.height = layer->out_height;
        tmp.depth = layer->out_channels;
    }
    out_channels = layers.back()->out_channels;
    out_height = layers.back()->out_height;
    out_width = layers.back()->out_width;
    input_size = in_width * in_width * in_channels;
    output_size = out_width * out_height * out_channels;
}

void LayerBlock::save(std::ofstream &file) {
    for (auto &layer : layers) layer->save(file);
}
void LayerBlock::load(std::ifstream &file) {
    for (auto &layer : layers) layer->load(file);
}

ParameterMap LayerBlock::get_parameters_as_map(std::string suffix) {
    ParameterMap params;
    for (size_t i = 0; i < layers.size(); i++) {
        const LayerType t = layers[i]->get_layer_type();
        if (t == LayerType::Activation || t == LayerType::Pool2d) continue;
        auto p = layers[i]->get_parameters_as_map(suffix + "." + std::to_string(i));
        params.insert(p.begin(), p.end());
    }
    return params;
}

void LayerBlock::load_parameters_from_map(const ParameterMap &param_map,
                                          const std::string &suffix) {
    for (size_t i = 0; i < layers.size(); i++) {
        const LayerType t = layers[i]->get_layer_type();
        if (t == LayerType::Activation || t == LayerType::Pool2d) continue;
        layers[i]->load_parameters_from_map(param_map, suffix + "." + std::to_string(i));
    }
}

std::vector<ParameterTuple> LayerBlock::parameters() {
    std::vector<ParameterTuple> params;
    for (auto &layer : layers) {
        const LayerType t = layer->get_layer_type();
        if (t == LayerType::Activation || t == LayerType::Pool2d) continue;
        auto p = layer->parameters();
        params.insert(params.end(), p.begin(), p.end());
    }
    return params;
}

// Input / output image sizes a caller may have set on a block before it is moved to
// the device (a network that starts with a block has nothing else to take them from).
static void copy_geometry(const BaseLayer &from, BaseLayer &to) {
    to.in_width = from.in_width; to.in_height = from.in_height; to.in_channels = from.in_channels;
    to.out_width = from.out_width; to.out_height = from.out_height;
    to.out_channels = from.out_channels;
}

std::unique_ptr<BaseLayer> LayerBlock::to_cuda(int device_idx) {
    auto block = std::make_unique<LayerBlock>();
    block->device = "cuda";
    block->device_idx = device_idx;
    for (auto &layer : layers) block->layers.push_back(layer->to_cuda(device_idx));
    block->input_size = input_size;
    block->output_size = output_size;
    block->training = training;
    copy_geometry(*this, *block);
    this->device = "cuda";
    this->device_idx = device_idx;
    return block;
}

void LayerBlock::preinit_layer() {
    for (auto &layer : layers) layer->preinit_layer();
}

int LayerBlock::get_neg_var_w_counter() {
    int total = 0;
    for (auto &layer : layers) total += layer->get_neg_var_w_counter();
    return total;
}
BaseLayer::NormStats LayerBlock::get_norm_mean_var() {
    NormStats all;
    for (auto &layer : layers) append_norm_stats(all, layer->get_norm_mean_var());
    return all;
}
void LayerBlock::params_to_device() {
    for (auto &layer : layers) layer->params_to_device();
}
void LayerBlock::params_to_host() {
    for (auto &layer : layers) layer->params_to_host();
}
void LayerBlock::delta_params_to_host() {
    for (auto &layer : layers) layer->delta_params_to_host();
}

// ---- ResNetBlock -------------------------------------------------------------------------
ResNetBlock::ResNetBlock(std::shared_ptr<BaseLayer> main, std::shared_ptr<BaseLayer> sc)
    : main_block(std::move(main)), shortcut(std::move(sc)) {
    if (!main_block) LOG(LogLevel::ERROR, "ResNetBlock needs a main block");
    this->input_size = main_block->input_size;
    this->output_size = main_block->output_size;
}

std::string ResNetBlock::get_layer_info() const {
    return "ResNetBlock(" + std::to_string(input_size) + "," + std::to_string(output_size) + ")";
}

int ResNetBlock::get_max_num_states() {
    int m = main_block->get_max_num_states();
    if (shortcut) m = std::max(m, shortcut->get_max_num_states());
    return m;
}

std::string ResNetBlock::get_device() {
    const std::string own = this->device + ":" + std::to_string(this->device_idx);
    const std::string m = main_block->get_device();
    if (m != own) return m;
    if (shortcut) {
        const std::string s = shortcut->get_device();
        if (s != own) return s;
    }
    return own;
}

void ResNetBlock::compute_input_output_size(const InitArgs &args) {
    in_channels = args.depth;
    in_height = args.height;
    in_width = args.width;
    main_block->compute_input_output_size(args);
    if (shortcut) shortcut->compute_input_output_size(args);
    out_channels = main_block->out_channels;
    out_height = main_block->out_height;
    out_width = main_block->out_width;
    input_size = in_width * in_width * in_channels;
    output_size = out_width * out_height * out_channels;
    if (shortcut && shortcut->output_size != output_size)
        LOG(LogLevel::ERROR, "ResNetBlock: shortcut output " +
                                 std::to_string(shortcut->output_size) + " vs main block output " +
                                 std::to_string(output_size));
    if (!shortcut && input_size != output_size)
        LOG(LogLevel::ERROR, "ResNetBlock without a shortcut needs equal input and output sizes");
}

void ResNetBlock::init_weight_bias() {
    main_block->init_weight_bias();
    if (shortcut) shortcut->init_weight_bias();
}
void ResNetBlock::set_threads(int num) {
    main_block->set_threads(num);
    if (shortcut) shortcut->set_threads(num);
}
void ResNetBlock::train() {
    this->training = true;
    main_block->train();
    if (shortcut) shortcut->train();
}
void ResNetBlock::eval() {
    this->training = false;
    main_block->eval();
    if (shortcut) shortcut->eval();
}

// reference: init_input_buffer / init_shortcut_state / init_shortcut_delta_state,
// src/resnet_block_cuda.cu:106-139
void ResNetBlock::init_buffers(size_t size) {
    if (size == 0) {
        int states = (int)this->input_size;
        if (shortcut) states = std::max(states, shortcut->get_max_num_states());
        states = std::max(states, (int)this->output_size);
        size = (size_t)states * batch_size_;
    }
    buffer_size_ = size;
    input_z = std::make_shared<HiddenStateHip>(size, batch_size_, device_idx);
    input_delta_z = std::make_shared<DeltaStateHip>(size, batch_size_, device_idx);
    if (shortcut) {
        shortcut_output_z = std::make_shared<HiddenStateHip>(size, batch_size_, device_idx);
        // the shortcut's layers ping-pong between this buffer and another one that nothing
        // else reads once the shortcut has run, so its layers may keep their arrays
        as<HiddenStateHip>(*shortcut_output_z)->transient = true;
        if (training)
            shortcut_output_delta_z = std::make_shared<DeltaStateHip>(size, batch_size_, device_idx);
    }
}

bool ResNetBlock::can_trade() const {
    auto *m = dynamic_cast<LayerBlock *>(main_block.get());
    if (m == nullptr || m->layers.size() < 2) return false;
    if (!shortcut) return true;
    auto *sc = dynamic_cast<LayerBlock *>(shortcut.get());
    return sc != nullptr && sc->layers.size() >= 2;
}

// reference: ResNetBlockCuda::forward, src/resnet_block_cuda.cu:211-299
void ResNetBlock::forward(BaseHiddenStates &input_states, BaseHiddenStates &output_states,
                          BaseTempStates &temp_states) {
    if (!on_device) no_cpu_path("forward");
    auto *in = as<HiddenStateHip>(input_states);
    const int batch_size = (int)input_states.block_size;
    // The block keeps its input for the shortcut (the reference copies it: mu_a, var_a,
    // jcb, and once more into the block's bwd_states). Where the input arrives in a
    // ping-pong buffer of the enclosing network, and both branches can be told where to
    // read (LayerBlocks), the block TRADES arrays with that buffer instead: its own
    // state object (as large as the buffer) takes the input, the buffer takes the
    // block's arrays of the previous step and serves on as scratch. Nothing is copied,
    // and the first layers of both branches borrow the kept arrays for their backward.
    const bool trade = in->transient && this->can_trade();
    const size_t want = trade ? in->size : 0;
    if (batch_size != batch_size_ || !input_z || (trade && buffer_size_ != want) ||
        (training && shortcut && !shortcut_output_delta_z)) {
        batch_size_ = batch_size;
        this->init_buffers(want);
    }
    auto *kept = as<HiddenStateHip>(*input_z);
    auto *main_lb = dynamic_cast<LayerBlock *>(main_block.get());
    if (trade) {
        kept->swap(input_states);
        kept->stable = true;
        kept->transient = false;
    } else {
        kept->stable = false;
        kept->transient = shortcut != nullptr;  // read by the shortcut only, then dead
        input_z->copy_from(input_states, (int)(this->input_size * batch_size));
    }
    // The shortcut runs first, so that a main block that ends on a BatchNorm2d layer can
    // add the shortcut's output in that layer's pass instead of in a pass of its own.
    HiddenStateHip *sc = nullptr;
    if (shortcut) {
        if (trade) {
            // first layer reads the kept input; the traded-away buffer is its scratch
            dynamic_cast<LayerBlock *>(shortcut.get())->first_input = input_z.get();
            shortcut->forward(input_states, *shortcut_output_z, temp_states);
        } else {
            shortcut->forward(*input_z, *shortcut_output_z, temp_states);
        }
        sc = as<HiddenStateHip>(*shortcut_output_z);
    } else {
        sc = kept;
    }
    BatchNorm2dHip *closing = nullptr;
    if (main_lb != nullptr && !main_lb->layers.empty())
        closing = dynamic_cast<BatchNorm2dHip *>(main_lb->layers.back().get());
    if (closing != nullptr) {
        closing->residual_mu = sc->d_mu_a;
        closing->residual_var = sc->d_var_a;
    }
    if (trade) main_lb->first_input = input_z.get();
    main_block->forward(input_states, output_states, temp_states);

    auto *out = as<HiddenStateHip>(output_states);
    const size_t num_states = output_states.block_size * this->output_size;
    if (closing == nullptr)
        TAGI_OK_OR_THROW(tagi_add_shortcut(sc->d_mu_a, sc->d_var_a, num_states, out->d_mu_a,
                                           out->d_var_a, host_stream()));
    set_output_dims(output_states, *this, batch_size);
    out->jcb_ones = true;  // the block's output Jacobian is one: marked, not written
}

// reference: ResNetBlockCuda::backward, src/resnet_block_cuda.cu:301-347
void ResNetBlock::backward(BaseDeltaStates &input_delta_states,
                           BaseDeltaStates &output_delta_states, BaseTempStates &temp_states,
                           bool state_update) {
    if (!on_device) no_cpu_path("backward");
    const int batch_size = (int)input_delta_states.block_size;
    // As in forward(): the incoming innovations are needed by both branches; trade arrays
    // with the buffer they arrive in where both branches can be told where to read.
    auto *din = as<DeltaStateHip>(input_delta_states);
    auto *main_lb = dynamic_cast<LayerBlock *>(main_block.get());
    const bool trade = this->can_trade() && din->size == as<DeltaStateHip>(*input_delta_z)->size &&
                       (!shortcut || as<DeltaStateHip>(*shortcut_output_delta_z)->size == din->size);
    if (trade)
        input_delta_z->swap(input_delta_states);
    else
        input_delta_z->copy_from(input_delta_states, (int)(this->output_size * batch_size));
    // The residual's innovations are added by the state backward of the main block's
    // first layer where that is a convolution (one pass less per block); the shortcut
    // branch then runs first, so that its result is there to be added.
    Conv2dHip *opening = nullptr;
    if (state_update && main_lb != nullptr && main_lb->layers.size() > 1)
        opening = dynamic_cast<Conv2dHip *>(main_lb->layers.front().get());
    auto *dout = as<DeltaStateHip>(output_delta_states);
    const size_t num_states = (size_t)batch_size * this->input_size;
    if (shortcut) {
        if (trade) {
            dynamic_cast<LayerBlock *>(shortcut.get())->first_delta_input = input_delta_z.get();
            shortcut->backward(input_delta_states, *shortcut_output_delta_z, temp_states, state_update);
        } else {
            shortcut->backward(*input_delta_z, *shortcut_output_delta_z, temp_states, state_update);
        }
        auto *sc = as<DeltaStateHip>(*shortcut_output_delta_z);
        if (opening != nullptr) {
            opening->bwd_residual_mu = sc->d_delta_mu;
            opening->bwd_residual_var = sc->d_delta_var;
            opening->bwd_residual_mode = 2;
        }
        if (trade) {
            main_lb->first_delta_input = input_delta_z.get();
            input_delta_states.block_size = batch_size;
        }
        main_block->backward(input_delta_states, output_delta_states, temp_states, state_update);
        if (!state_update || opening != nullptr) return;
        TAGI_OK_OR_THROW(tagi_add_shortcut(sc->d_delta_mu, sc->d_delta_var, num_states,
                                           dout->d_delta_mu, dout->d_delta_var, host_stream()));
    } else {
        auto *sc = as<DeltaStateHip>(*input_delta_z);
        if (opening != nullptr) {
            // (the opening layer's stored Jacobian is the block input's)
            opening->bwd_residual_mu = sc->d_delta_mu;
            opening->bwd_residual_var = sc->d_delta_var;
            opening->bwd_residual_mode = 1;
        }
        if (trade) {
            main_lb->first_delta_input = input_delta_z.get();
            input_delta_states.block_size = batch_size;
        }
        main_block->backward(input_delta_states, output_delta_states, temp_states, state_update);
        if (!state_update || opening != nullptr) return;
        auto *kept = as<HiddenStateHip>(*input_z);
        TAGI_OK_OR_THROW(tagi_add_shortcut_delta(sc->d_delta_mu, sc->d_delta_var, kept->jcb_ptr(),
                                                 num_states, dout->d_delta_mu, dout->d_delta_var,
                                                 host_stream()));
    }
}

void ResNetBlock::update_weights() {
    main_block->update_weights();
    if (shortcut) shortcut->update_weights();
}
void ResNetBlock::update_biases() {
    main_block->update_biases();
    if (shortcut) shortcut->update_biases();
}
void LayerBlock::collect_update_items(std::vector<tagi_update_item> &items) {
    for (auto &layer : layers)
        if (layer->get_layer_type() != LayerType::Activation) layer->collect_update_items(items);
}
void ResNetBlock::collect_update_items(std::vector<tagi_update_item> &items) {
    main_block->collect_update_items(items);
    if (shortcut) shortcut->collect_update_items(items);
}
void ResNetBlock::update_params() {
    main_block->update_params();
    if (shortcut) shortcut->update_params();
}
void ResNetBlock::save(std::ofstream &file) {
    main_block->save(file);
    if (shortcut) shortcut->save(file);
}
void ResNetBlock::load(std::ifstream &file) {
    main_block->load(file);
    if (shortcut) shortcut->load(file);
}

ParameterMap ResNetBlock::get_parameters_as_map(std::string suffix) {
    ParameterMap params = main_block->get_parameters_as_map("main." + suffix);
    if (shortcut) {
        auto p = shortcut->get_parameters_as_map("shortcut." + suffix);
        params.insert(p.begin(), p.end());
    }
    return params;
}

void ResNetBlock::load_parameters_from_map(const ParameterMap &param_map,
                                           const std::string &suffix) {
    main_block->load_parameters_from_map(param_map, "main." + suffix);
    if (shortcut) shortcut->load_parameters_from_map(param_map, "shortcut." + suffix);
}

std::vector<ParameterTuple> ResNetBlock::parameters() {
    std::vector<ParameterTuple> params = main_block->parameters();
    if (shortcut) {
        auto p = shortcut->parameters();
        params.insert(params.end(), p.begin(), p.end());
    }
    return params;
}

std::unique_ptr<BaseLayer> ResNetBlock::to_cuda(int device_idx) {
    this->device = "cuda";
    this->device_idx = device_idx;
    std::shared_ptr<BaseLayer> m = main_block->to_cuda(device_idx);
    std::shared_ptr<BaseLayer> s = shortcut ? shortcut->to_cuda(device_idx) : nullptr;
    auto block = std::make_unique<ResNetBlockHip>(std::move(m), std::move(s), device_idx);
    copy_geometry(*this, *block);
    return block;
}

void ResNetBlock::preinit_layer() {
    main_block->preinit_layer();
    if (shortcut) shortcut->preinit_layer();
}

int ResNetBlock::get_neg_var_w_counter() {
    return main_block->get_neg_var_w_counter() + (shortcut ? shortcut->get_neg_var_w_counter() : 0);
}

BaseLayer::NormStats ResNetBlock::get_norm_mean_var() {
    NormStats all = main_block->get_norm_mean_var();
    if (shortcut) append_norm_stats(all, shortcut->get_norm_mean_var());
    return all;
}

void ResNetBlock::params_to_device() {
    main_block->params_to_device();
    if (shortcut) shortcut->params_to_device();
}
void ResNetBlock::params_to_host() {
    main_block->params_to_host();
    if (shortcut) shortcut->params_to_host();
}
void ResNetBlock::delta_params_to_host() {
    main_block->delta_params_to_host();
    if (shortcut) shortcut->delta_params_to_host();
}

ResNetBlockHip::ResNetBlockHip(std::shared_ptr<BaseLayer> main, std::shared_ptr<BaseLayer> sc,
                               int device_idx)
    : ResNetBlock(std::move(main), std::move(sc)) {
    this->device = "cuda";
    this->device_idx = device_idx;
    this->on_device = true;
    this->bwd_states = std::make_unique<BackwardStateHip>();
}

std::string ResNetBlockHip::get_layer_info() const {
    return "ResNetBlockCuda(" + std::to_string(input_size) + "," + std::to_string(output_size) + ")";
}

std::unique_ptr<BaseLayer> ResNetBlockHip::to_cuda(int device_idx) {
    // already on the device: hand the members over to a fresh block
    return std::make_unique<ResNetBlockHip>(main_block, shortcut, device_idx);
}

}  // namespace tagi_host

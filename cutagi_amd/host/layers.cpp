// Layer classes: see layers.h. All arithmetic is delegated to libtagi_hip.so
// through the C ABI (include/tagi_hip.h) on the null stream.
#include "layers.h"

#include <algorithm>
#include <cmath>
#include <cstring>

#include "../../include/tagi_hip.h"
#include "host_util.h"
#include "logger.h"

namespace tagi_host {


void manual_seed(int seed) { SeedManager::get_instance().set_seed(seed); }

ParameterTuple init_gaussian_params(const std::string &method, float gain_w, float gain_b,
                                    float fan_in, float fan_out, size_t num_weights,
                                    size_t num_biases) {
    float scale = 0.0f;
    if (method == "He" || method == "he")
        scale = std::pow(1.0f / fan_in, 0.5f);
    else if (method == "Xavier" || method == "xavier")
        scale = std::pow(2.0f / (fan_in + fan_out), 0.5f);
    else
        LOG(LogLevel::ERROR, "Initial parameter method [" + method + "] is not supported.");
    std::mt19937 &gen = SeedManager::get_instance().get_engine();
    auto draw = [&](size_t n, float gain, std::vector<float> &mu, std::vector<float> &var) {
        std::normal_distribution<float> dist(0.0f, scale);
        mu.resize(n);
        var.assign(n, (gain * scale) * (gain * scale));
        for (auto &m : mu) m = dist(gen);
    };
    std::vector<float> mu_w, var_w, mu_b, var_b;
    draw(num_weights, gain_w, mu_w, var_w);
    if (num_biases > 0) draw(num_biases, gain_b, mu_b, var_b);
    return {mu_w, var_w, mu_b, var_b};
}

// reference: src/conv2d_layer.cpp:581-628 (throws where the stride does not divide)
std::tuple<int, int> compute_downsample_img_size_v2(int kernel, int stride, int wi, int hi, int pad,
                                                    int pad_type) {
    int wo = 0, ho = 0;
    if (tagi_conv2d_out_size(kernel, stride, wi, hi, pad, pad_type, &wo, &ho) != TAGI_OK)
        LOG(LogLevel::ERROR, "Invalid hyperparameters for conv2d layer: wi=" + std::to_string(wi) +
                                 ", hi=" + std::to_string(hi) + ", kernel=" +
                                 std::to_string(kernel) + ", stride=" + std::to_string(stride));
    return {wo, ho};
}

// ---- BaseLayer ----------------------------------------------------------------------
BaseLayer::BaseLayer() { this->bwd_states = std::make_unique<BaseBackwardStates>(); }

void BaseLayer::no_cpu_path(const char *what) const {
    LOG(LogLevel::ERROR, std::string(what) + " of " + this->get_layer_info() +
                             ": this library computes on the GPU only; move the model with "
                             "to_device(\"cuda\") first");
    throw std::runtime_error("unreachable");
}

void BaseLayer::forward(BaseHiddenStates &, BaseHiddenStates &, BaseTempStates &) {
    no_cpu_path("forward");
}
void BaseLayer::backward(BaseDeltaStates &, BaseDeltaStates &, BaseTempStates &, bool) {
    no_cpu_path("backward");
}
void BaseLayer::update_weights() { no_cpu_path("update_weights"); }
void BaseLayer::update_biases() { no_cpu_path("update_biases"); }
void BaseLayer::raw_update_weights() { no_cpu_path("raw_update_weights"); }
void BaseLayer::raw_update_biases() { no_cpu_path("raw_update_biases"); }

void BaseLayer::allocate_param_delta() {
    delta_mu_w.assign(num_weights, 0.0f);
    delta_var_w.assign(num_weights, 0.0f);
    delta_mu_b.assign(num_biases, 0.0f);
    delta_var_b.assign(num_biases, 0.0f);
}

void BaseLayer::set_cap_factor_udapte(int batch_size) {
    this->cap_factor_update = tagi_cap_factor(batch_size, this->cap_factor_update);
}

void BaseLayer::compute_input_output_size(const InitArgs &args) {
    in_width = out_width = args.width;
    in_height = out_height = args.height;
    in_channels = out_channels = args.depth;
}

// File layout of the reference (src/base_layer.cpp:230-297): size_t name length,
// get_layer_info() text, then mu_w, var_w, mu_b, var_b as raw floats.
void BaseLayer::save(std::ofstream &file) {
    if (!file.is_open()) LOG(LogLevel::ERROR, "Failed to open file for saving");
    const std::string name = this->get_layer_info();
    const size_t len = name.length();
    file.write(reinterpret_cast<const char *>(&len), sizeof(len));
    file.write(name.c_str(), len);
    write_floats(file, mu_w);
    write_floats(file, var_w);
    write_floats(file, mu_b);
    write_floats(file, var_b);
}

void BaseLayer::load(std::ifstream &file) {
    if (!file.is_open()) LOG(LogLevel::ERROR, "Failed to open file for loading");
    size_t len = 0;
    file.read(reinterpret_cast<char *>(&len), sizeof(len));
    std::string found(len, '\0');
    file.read(&found[0], len);
    const std::string expected = this->get_layer_info();
    if (found != expected)
        LOG(LogLevel::ERROR, "Layer name are not match. Expected: " + expected + ", Found: " + found);
    read_floats(file, mu_w);
    read_floats(file, var_w);
    read_floats(file, mu_b);
    read_floats(file, var_b);
    num_weights = mu_w.size();
    num_biases = mu_b.size();
    if (training) this->allocate_param_delta();
}

std::unique_ptr<BaseLayer> BaseLayer::to_cuda(int) {
    LOG(LogLevel::ERROR, "This layer has no device form");
    return nullptr;
}

ParameterMap BaseLayer::get_parameters_as_map(std::string suffix) {
    std::string key = this->get_layer_name();
    if (!suffix.empty()) key += "." + suffix;
    return {{key, std::make_tuple(mu_w, var_w, mu_b, var_b)}};
}

void BaseLayer::load_parameters_from_map(const ParameterMap &param_map, const std::string &suffix) {
    std::string key = this->get_layer_name();
    if (!suffix.empty()) key += "." + suffix;
    auto it = param_map.find(key);
    if (it == param_map.end()) LOG(LogLevel::ERROR, "Key " + key + " not found in parameter map.");
    std::tie(mu_w, var_w, mu_b, var_b) = it->second;
}

std::vector<ParameterTuple> BaseLayer::parameters() {
    return {std::make_tuple(mu_w, var_w, mu_b, var_b)};
}

// ---- BaseLayerHip ---------------------------------------------------------------------
BaseLayerHip::BaseLayerHip() {
    this->device = "cuda";
    this->bwd_states = std::make_unique<BackwardStateHip>();
}

BaseLayerHip::~BaseLayerHip() { this->release_param_memory(); }

void BaseLayerHip::release_param_memory() {
    dev_free_t(d_mu_w); dev_free_t(d_var_w); dev_free_t(d_mu_b); dev_free_t(d_var_b);
    dev_free_t(d_delta_mu_w); dev_free_t(d_delta_var_w);
    dev_free_t(d_delta_mu_b); dev_free_t(d_delta_var_b);
    dev_free_t(d_neg_var_count);
}

void BaseLayerHip::allocate_param_memory() {
    dev_free_t(d_mu_w); dev_free_t(d_var_w); dev_free_t(d_mu_b); dev_free_t(d_var_b);
    d_mu_w = dev_alloc_t<float>(num_weights, device_idx);
    d_var_w = dev_alloc_t<float>(num_weights, device_idx);
    d_mu_b = dev_alloc_t<float>(num_biases, device_idx);
    d_var_b = dev_alloc_t<float>(num_biases, device_idx);
    alloc_w = num_weights;
    alloc_b = num_biases;
    if (d_neg_var_count == nullptr) {
        d_neg_var_count = dev_alloc_t<int>(2, device_idx);
        HIP_OK(hipMemset(d_neg_var_count, 0, 2 * sizeof(int)));
    }
}

void BaseLayerHip::allocate_param_delta() {
    BaseLayer::allocate_param_delta();
    dev_free_t(d_delta_mu_w); dev_free_t(d_delta_var_w);
    dev_free_t(d_delta_mu_b); dev_free_t(d_delta_var_b);
    d_delta_mu_w = dev_alloc_t<float>(num_weights, device_idx);
    d_delta_var_w = dev_alloc_t<float>(num_weights, device_idx);
    d_delta_mu_b = dev_alloc_t<float>(num_biases, device_idx);
    d_delta_var_b = dev_alloc_t<float>(num_biases, device_idx);
    if (num_weights) {
        HIP_OK(hipMemset(d_delta_mu_w, 0, num_weights * sizeof(float)));
        HIP_OK(hipMemset(d_delta_var_w, 0, num_weights * sizeof(float)));
    }
    if (num_biases) {
        HIP_OK(hipMemset(d_delta_mu_b, 0, num_biases * sizeof(float)));
        HIP_OK(hipMemset(d_delta_var_b, 0, num_biases * sizeof(float)));
    }
}

void BaseLayerHip::params_to_device() {
    if (mu_w.size() != num_weights || mu_b.size() != num_biases)
        LOG(LogLevel::ERROR, "Parameter vectors do not match the layer's parameter count");
    h2d(d_mu_w, mu_w); h2d(d_var_w, var_w); h2d(d_mu_b, mu_b); h2d(d_var_b, var_b);
}

void BaseLayerHip::params_to_host() {
    d2h(mu_w, d_mu_w, num_weights); d2h(var_w, d_var_w, num_weights);
    d2h(mu_b, d_mu_b, num_biases); d2h(var_b, d_var_b, num_biases);
}

void BaseLayerHip::delta_params_to_host() {
    d2h(delta_mu_w, d_delta_mu_w, num_weights); d2h(delta_var_w, d_delta_var_w, num_weights);
    d2h(delta_mu_b, d_delta_mu_b, num_biases); d2h(delta_var_b, d_delta_var_b, num_biases);
}

// reference: BaseLayerCuda::delta_params_to_device, src/base_layer_cuda.cu:313-332
void BaseLayerHip::delta_params_to_device() {
    if (delta_mu_w.size() != num_weights || delta_var_w.size() != num_weights ||
        (bias && (delta_mu_b.size() != num_biases || delta_var_b.size() != num_biases)))
        LOG(LogLevel::ERROR, "Host parameter innovations do not have the layer's sizes");
    if (d_delta_mu_w == nullptr) {  // allocation zeroes the host vectors: keep them
        auto keep = std::make_tuple(delta_mu_w, delta_var_w, delta_mu_b, delta_var_b);
        this->allocate_param_delta();
        std::tie(delta_mu_w, delta_var_w, delta_mu_b, delta_var_b) = keep;
    }
    h2d(d_delta_mu_w, delta_mu_w); h2d(d_delta_var_w, delta_var_w);
    if (bias) {
        h2d(d_delta_mu_b, delta_mu_b); h2d(d_delta_var_b, delta_var_b);
    }
}

// reference: BaseLayerCuda::raw_update_weights / raw_update_biases,
// src/base_layer_cuda.cu:127-159
void BaseLayerHip::raw_update_weights() {
    TAGI_OK_OR_THROW(tagi_param_raw_update(d_delta_mu_w, d_delta_var_w, num_weights, d_mu_w,
                                           d_var_w, host_stream()));
}
void BaseLayerHip::raw_update_biases() {
    if (!bias) return;
    TAGI_OK_OR_THROW(tagi_param_raw_update(d_delta_mu_b, d_delta_var_b, num_biases, d_mu_b,
                                           d_var_b, host_stream()));
}

void BaseLayerHip::copy_params_from(const BaseLayer &source) {
    this->num_weights = source.mu_w.size();
    this->num_biases = source.mu_b.size();
    this->allocate_param_memory();
    mu_w = source.mu_w; var_w = source.var_w; mu_b = source.mu_b; var_b = source.var_b;
    this->params_to_device();
}

// The clamped-variance counter stays on the device; it is read back only when
// somebody asks for it (the reference copies it in both directions every step,
// src/base_layer_cuda.cu:170-185). There are two counters used in turn: the
// update that counts into one zeroes the other for the next update.
void BaseLayerHip::update_weights() {
    HIP_OK(hipMemsetAsync(d_neg_var_count, 0, 2 * sizeof(int), host_stream()));
    neg_var_slot = 0;
    TAGI_OK_OR_THROW(tagi_param_update(d_delta_mu_w, d_delta_var_w, cap_factor_update, num_weights,
                                       d_mu_w, d_var_w, d_neg_var_count, host_stream()));
    neg_var_dirty = true;
}

void BaseLayerHip::update_biases() {
    if (!bias) return;
    TAGI_OK_OR_THROW(tagi_param_update(d_delta_mu_b, d_delta_var_b, cap_factor_update, num_biases,
                                       d_mu_b, d_var_b, nullptr, host_stream()));
}

// Weights and biases in one launch, no launch for the counter.
void BaseLayerHip::update_params() {
    neg_var_slot = 1 - neg_var_slot;
    TAGI_OK_OR_THROW(tagi_layer_update(d_delta_mu_w, d_delta_var_w, num_weights, d_mu_w, d_var_w,
                                       d_delta_mu_b, d_delta_var_b, bias ? num_biases : 0, d_mu_b,
                                       d_var_b, cap_factor_update, d_neg_var_count, neg_var_slot,
                                       host_stream()));
    neg_var_dirty = true;
}

void BaseLayerHip::collect_update_items(std::vector<tagi_update_item> &items) {
    if (num_weights == 0 || d_mu_w == nullptr || d_delta_mu_w == nullptr) return;  // nothing to update
    neg_var_slot = 1 - neg_var_slot;
    tagi_update_item t = {};
    t.delta_mu_w = d_delta_mu_w; t.delta_var_w = d_delta_var_w;
    t.mu_w = d_mu_w; t.var_w = d_var_w; t.num_weights = num_weights;
    t.delta_mu_b = d_delta_mu_b; t.delta_var_b = d_delta_var_b;
    t.mu_b = d_mu_b; t.var_b = d_var_b; t.num_biases = bias ? num_biases : 0;
    t.cap_factor = cap_factor_update;
    t.neg_var_count = d_neg_var_count;
    t.slot = neg_var_slot;
    items.push_back(t);
    neg_var_dirty = true;
}

int BaseLayerHip::get_neg_var_w_counter() {
    if (neg_var_dirty) {
        HIP_OK(hipMemcpy(&neg_var_w_counter, d_neg_var_count + neg_var_slot, sizeof(int),
                         hipMemcpyDeviceToHost));
        neg_var_dirty = false;
    }
    return neg_var_w_counter;
}

void BaseLayerHip::save(std::ofstream &file) {
    this->params_to_host();
    BaseLayer::save(file);
}

void BaseLayerHip::load(std::ifstream &file) {
    BaseLayer::load(file);
    this->params_to_device();
}

ParameterMap BaseLayerHip::get_parameters_as_map(std::string suffix) {
    this->params_to_host();
    return BaseLayer::get_parameters_as_map(suffix);
}

void BaseLayerHip::adopt_host_params() {
    if (var_w.size() != mu_w.size() || var_b.size() != mu_b.size())
        LOG(LogLevel::ERROR, "Parameter means and variances differ in size");
    num_weights = mu_w.size();
    num_biases = mu_b.size();
    if (d_mu_w == nullptr || alloc_w != num_weights || alloc_b != num_biases)
        this->allocate_param_memory();
    if (training && (d_delta_mu_w == nullptr || delta_mu_w.size() != num_weights ||
                     delta_mu_b.size() != num_biases))
        this->allocate_param_delta();
    this->params_to_device();
}

void BaseLayerHip::load_parameters_from_map(const ParameterMap &param_map, const std::string &suffix) {
    BaseLayer::load_parameters_from_map(param_map, suffix);
    this->adopt_host_params();
}

std::vector<ParameterTuple> BaseLayerHip::parameters() {
    this->params_to_host();
    return BaseLayer::parameters();
}

// What the backward pass needs from the input (its mean and its Jacobian), and the
// output's Jacobian of one; reference: store_states_for_training_cuda,
// src/base_layer_cuda.cu:464-486 (two device copies and a fill kernel per layer).
// Here the output is only marked (HiddenStateHip::jcb_ones); an input Jacobian that is
// marked is not copied either; and where the input is one of its owner's ping-pong
// buffers, whose contents are dead once this layer has read them, the layer keeps the
// input's arrays and leaves its own arrays of the previous step in their place: no
// copy and no launch at all. Called after the layer's own kernels were queued (they
// hold the old addresses).
void BaseLayerHip::store_states_for_training_hip(HiddenStateHip &in, HiddenStateHip &out) {
    auto *bwd = dynamic_cast<BackwardStateHip *>(this->bwd_states.get());
    const size_t n_in = in.actual_size * in.block_size;
    bwd->device_idx = in.device_idx;
    out.jcb_ones = true;
    if (in.stable) {
        // the owner keeps these arrays as they are until the backward pass is over
        bwd->borrow(in.d_mu_a, in.d_jcb, in.jcb_ones, in.size);
        return;
    }
    if (in.transient) {
        bwd->resize_exact(in.size, !in.jcb_ones);
        std::swap(bwd->d_mu_a, in.d_mu_a);
        bwd->jcb_ones = in.jcb_ones;
        if (!in.jcb_ones) std::swap(bwd->d_jcb, in.d_jcb);
        return;
    }
    if (bwd->size < n_in) bwd->set_size(n_in);
    bwd->jcb_ones = in.jcb_ones;
    if (in.jcb_ones) {
        // (a kernel rather than a copy command where the work may be recorded into a
        // graph: copy nodes make a graph launch far more expensive than its kernels)
        if (host_stream() != nullptr)
            TAGI_OK_OR_THROW(tagi_store_states(in.d_mu_a, nullptr, n_in, bwd->d_mu_a, nullptr,
                                               nullptr, 0, host_stream()));
        else
            HIP_OK(hipMemcpyAsync(bwd->d_mu_a, in.d_mu_a, n_in * sizeof(float),
                                  hipMemcpyDeviceToDevice, host_stream()));
        return;
    }
    TAGI_OK_OR_THROW(tagi_store_states(in.d_mu_a, in.d_jcb, n_in, bwd->d_mu_a, bwd->d_jcb, nullptr,
                                       0, host_stream()));
}

// ---- Linear -----------------------------------------------------------------------------
Linear::Linear(size_t ip_size, size_t op_size, bool bias, float gain_weight, float gain_bias,
               std::string method, int device_idx)
    : gain_w(gain_weight), gain_b(gain_bias), init_method(std::move(method)) {
    this->input_size = ip_size;
    this->output_size = op_size;
    this->bias = bias;
    this->device_idx = device_idx;
    this->num_weights = ip_size * op_size;
    this->num_biases = bias ? op_size : 0;
    this->init_weight_bias();
    if (this->training) this->allocate_param_delta();
}

std::string Linear::get_layer_info() const {
    return "Linear(" + std::to_string(input_size) + "," + std::to_string(output_size) + ")";
}

void Linear::init_weight_bias() {
    std::tie(mu_w, var_w, mu_b, var_b) = init_gaussian_params(
        init_method, gain_w, gain_b, (float)input_size, (float)output_size, num_weights, num_biases);
}

std::unique_ptr<BaseLayer> Linear::to_cuda(int device_idx) {
    this->device = "cuda";
    this->device_idx = device_idx;
    auto layer = std::make_unique<LinearHip>(input_size, output_size, bias, gain_w, gain_b,
                                             init_method, device_idx);
    layer->copy_params_from(*this);
    return layer;
}

LinearHip::LinearHip(size_t ip_size, size_t op_size, bool bias, float gain_weight, float gain_bias,
                     std::string method, int device_idx)
    : gain_w(gain_weight), gain_b(gain_bias), init_method(std::move(method)) {
    this->input_size = ip_size;
    this->output_size = op_size;
    this->bias = bias;
    this->device_idx = device_idx;
    this->num_weights = ip_size * op_size;
    this->num_biases = bias ? op_size : 0;
    if (this->training) this->allocate_param_delta();
}

std::string LinearHip::get_layer_info() const {
    return "Linear(" + std::to_string(input_size) + "," + std::to_string(output_size) + ")";
}

void LinearHip::init_weight_bias() {
    std::tie(mu_w, var_w, mu_b, var_b) = init_gaussian_params(
        init_method, gain_w, gain_b, (float)input_size, (float)output_size, num_weights, num_biases);
    this->allocate_param_memory();
    this->params_to_device();
}

// reference: LinearCuda::forward, src/linear_layer_cuda.cu:231-271
void LinearHip::forward(BaseHiddenStates &input_states, BaseHiddenStates &output_states,
                        BaseTempStates &) {
    // (the one-shot request is taken before anything can throw)
    const int act = this->fused_activation;
    this->fused_activation = 0;
    auto *in = as<HiddenStateHip>(input_states);
    auto *out = as<HiddenStateHip>(output_states);
    const int batch_size = (int)input_states.block_size;
    this->set_cap_factor_udapte(batch_size);
    if (this->input_size != input_states.actual_size)
        LOG(LogLevel::ERROR, "Input size mismatch: " + std::to_string(this->input_size) + " vs " +
                                 std::to_string(input_states.actual_size));
    if (this->output_size * batch_size > out->size)
        LOG(LogLevel::ERROR, "Output state buffer too small for " + this->get_layer_info());
    if (d_mu_w == nullptr) LOG(LogLevel::ERROR, "Parameters of " + get_layer_info() + " are not on the device");

    if (act != 0)
        TAGI_OK_OR_THROW(tagi_linear_fwd_act(d_mu_w, d_var_w, d_mu_b, d_var_b, in->d_mu_a,
                                             in->d_var_a, (int)input_size, (int)output_size,
                                             batch_size, bias ? 1 : 0, act, out->d_mu_a,
                                             out->d_var_a, out->d_jcb, host_stream()));
    else
        TAGI_OK_OR_THROW(tagi_linear_fwd(d_mu_w, d_var_w, d_mu_b, d_var_b, in->d_mu_a,
                                         in->d_var_a, (int)input_size, (int)output_size,
                                         batch_size, bias ? 1 : 0, out->d_mu_a, out->d_var_a,
                                         host_stream()));
    output_states.width = this->out_width;
    output_states.height = this->out_height;
    output_states.depth = this->out_channels;
    output_states.block_size = batch_size;
    output_states.actual_size = this->output_size;
    out->jcb_ones = true;
    if (this->training) this->store_states_for_training_hip(*in, *out);
    if (act != 0) out->jcb_ones = false;  // the activation's Jacobian was written
}

// reference: LinearCuda::backward, src/linear_layer_cuda.cu:273-323
void LinearHip::backward(BaseDeltaStates &input_delta_states, BaseDeltaStates &output_delta_states,
                         BaseTempStates &, bool state_udapte) {
    auto *din = as<DeltaStateHip>(input_delta_states);
    auto *dout = as<DeltaStateHip>(output_delta_states);
    auto *bwd = dynamic_cast<BackwardStateHip *>(this->bwd_states.get());
    const int batch_size = (int)input_delta_states.block_size;
    if (state_udapte && input_size * batch_size > dout->size)
        LOG(LogLevel::ERROR, "Delta state buffer too small for " + this->get_layer_info());
    TAGI_OK_OR_THROW(tagi_linear_bwd(d_mu_w, d_var_w, d_var_b, bwd->d_mu_a, bwd->jcb_ptr(),
                                     din->d_delta_mu, din->d_delta_var, (int)input_size,
                                     (int)output_size, batch_size, bias ? 1 : 0, state_udapte ? 1 : 0,
                                     param_update ? 1 : 0, dout->d_delta_mu, dout->d_delta_var,
                                     d_delta_mu_w, d_delta_var_w, d_delta_mu_b, d_delta_var_b,
                                     host_stream()));
}

// ---- Conv2d -----------------------------------------------------------------------------
Conv2d::Conv2d(size_t in_channels, size_t out_channels, size_t kernel_size, bool bias, int stride,
               int padding, int padding_type, size_t in_width, size_t in_height, float gain_w,
               float gain_b, std::string init_method, int device_idx)
    : kernel_size(kernel_size), stride(stride), padding(padding), padding_type(padding_type),
      gain_w(gain_w), gain_b(gain_b), init_method(std::move(init_method)) {
    this->in_width = in_width;
    this->in_height = in_height;
    this->in_channels = in_channels;
    this->out_channels = out_channels;
    this->bias = bias;
    this->device_idx = device_idx;
}

std::string Conv2d::get_layer_info() const {
    return "Conv2d(" + std::to_string(in_channels) + "," + std::to_string(out_channels) + "," +
           std::to_string(out_width) + "," + std::to_string(out_height) + "," +
           std::to_string(kernel_size) + ")";
}

// Square images: the reference sizes the layer as in_width * in_width
// (src/conv2d_layer.cpp:63) and builds its index tables for square inputs only.
void Conv2d::compute_input_output_size(const InitArgs &args) {
    if (in_width == 0 || in_height == 0) {
        in_width = args.width;
        in_height = args.height;
    }
    std::tie(out_width, out_height) = compute_downsample_img_size_v2(
        (int)kernel_size, stride, (int)in_width, (int)in_height, padding, padding_type);
    input_size = in_width * in_width * in_channels;
    output_size = out_width * out_height * out_channels;
}

void Conv2d::init_weight_bias() {
    const float k2 = (float)(kernel_size * kernel_size);
    std::tie(mu_w, var_w, mu_b, var_b) = init_gaussian_params(
        init_method, gain_w, gain_b, k2 * in_channels, k2 * out_channels, num_weights, num_biases);
}

void Conv2d::preinit_layer() {
    if (num_weights == 0) {
        num_weights = kernel_size * kernel_size * in_channels * out_channels;
        num_biases = bias ? out_channels : 0;
        this->init_weight_bias();
    }
}

std::unique_ptr<BaseLayer> Conv2d::to_cuda(int device_idx) {
    this->device = "cuda";
    this->device_idx = device_idx;
    auto layer = std::make_unique<Conv2dHip>(in_channels, out_channels, kernel_size, bias, stride,
                                             padding, padding_type, in_width, in_height, gain_w,
                                             gain_b, init_method, device_idx);
    // Parameters that already exist on the host (preinit_layer, load_state_dict)
    // move with the layer; otherwise the device layer initialises lazily.
    if (!mu_w.empty()) layer->copy_params_from(*this);
    return layer;
}

Conv2dHip::Conv2dHip(size_t in_channels, size_t out_channels, size_t kernel_size, bool bias,
                     int stride, int padding, int padding_type, size_t in_width, size_t in_height,
                     float gain_w, float gain_b, std::string init_method, int device_idx)
    : kernel_size(kernel_size), stride(stride), padding(padding), padding_type(padding_type),
      gain_w(gain_w), gain_b(gain_b), init_method(std::move(init_method)) {
    this->in_width = in_width;
    this->in_height = in_height;
    this->in_channels = in_channels;
    this->out_channels = out_channels;
    this->bias = bias;
    this->device_idx = device_idx;
}

Conv2dHip::~Conv2dHip() {
    dev_free_t(d_idx_mwa_2);
    dev_free_t(d_idx_cov_zwa_1);
    dev_free_t(d_idx_var_z_ud);
}

std::string Conv2dHip::get_layer_info() const {
    return "Conv2d(" + std::to_string(in_channels) + "," + std::to_string(out_channels) + "," +
           std::to_string(out_width) + "," + std::to_string(out_height) + "," +
           std::to_string(kernel_size) + ")";
}

void Conv2dHip::compute_input_output_size(const InitArgs &args) {
    if (in_width == 0 || in_height == 0) {
        in_width = args.width;
        in_height = args.height;
    }
    std::tie(out_width, out_height) = compute_downsample_img_size_v2(
        (int)kernel_size, stride, (int)in_width, (int)in_height, padding, padding_type);
    input_size = in_width * in_width * in_channels;
    output_size = out_width * out_height * out_channels;
}

void Conv2dHip::get_number_param() {
    num_weights = kernel_size * kernel_size * in_channels * out_channels;
    num_biases = bias ? out_channels : 0;
}

void Conv2dHip::init_weight_bias() {
    const float k2 = (float)(kernel_size * kernel_size);
    std::tie(mu_w, var_w, mu_b, var_b) = init_gaussian_params(
        init_method, gain_w, gain_b, k2 * in_channels, k2 * out_channels, num_weights, num_biases);
    this->allocate_param_memory();
    this->params_to_device();
}

// reference: Conv2dCuda::lazy_index_init, src/conv2d_layer_cuda.cu:363-385
void Conv2dHip::lazy_index_init() {
    const int k2 = (int)(kernel_size * kernel_size);
    const int wihi = (int)(in_width * in_height), woho = (int)(out_width * out_height);
    idx_mwa_2.assign((size_t)woho * k2, 0);
    idx_cov_zwa_1.assign((size_t)wihi * k2, 0);
    idx_var_z_ud.assign((size_t)wihi * k2, 0);
    int w = 0, h = 0;
    const int param_pad_idx = k2 * (int)in_channels * (int)out_channels + 1;
    if (tagi_conv2d_build_idx((int)kernel_size, stride, (int)in_width, (int)in_height, padding,
                              padding_type, param_pad_idx, idx_mwa_2.data(), idx_cov_zwa_1.data(),
                              idx_var_z_ud.data(), &w, &h) != TAGI_OK)
        LOG(LogLevel::ERROR, "Cannot build the index tables of " + this->get_layer_info());
    if (w != wihi)
        LOG(LogLevel::ERROR, "Conv2d geometry leaves input pixels unused; not supported");
    idx_cov_zwa_1.resize((size_t)w * h);
    idx_var_z_ud.resize((size_t)w * h);
    row_zw = col_z_ud = h;
    auto upload = [&](int *&d, const std::vector<int> &v) {
        dev_free_t(d);
        d = dev_alloc_t<int>(v.size(), device_idx);
        HIP_OK(hipMemcpy(d, v.data(), v.size() * sizeof(int), hipMemcpyHostToDevice));
    };
    upload(d_idx_mwa_2, idx_mwa_2);
    upload(d_idx_cov_zwa_1, idx_cov_zwa_1);
    upload(d_idx_var_z_ud, idx_var_z_ud);
}

void Conv2dHip::preinit_layer() {
    if (num_weights == 0) {
        this->get_number_param();
        this->init_weight_bias();
        if (training) this->allocate_param_delta();
    }
    if (idx_mwa_2.empty()) this->lazy_index_init();
}

// reference: Conv2dCuda::forward, src/conv2d_layer_cuda.cu:387-451
void Conv2dHip::forward(BaseHiddenStates &input_states, BaseHiddenStates &output_states,
                        BaseTempStates &) {
    const int act = this->fused_activation;  // one-shot: taken before anything can throw
    this->fused_activation = 0;
    auto *in = as<HiddenStateHip>(input_states);
    auto *out = as<HiddenStateHip>(output_states);
    if (this->input_size != input_states.actual_size)
        LOG(LogLevel::ERROR, "Input size mismatch: " + std::to_string(this->input_size) + " vs " +
                                 std::to_string(input_states.actual_size));
    const int batch_size = (int)input_states.block_size;
    this->set_cap_factor_udapte(batch_size);
    if (num_weights == 0) {
        this->get_number_param();
        this->init_weight_bias();
    }
    if (training && d_delta_mu_w == nullptr) this->allocate_param_delta();
    if (idx_mwa_2.empty()) this->lazy_index_init();
    if (this->output_size * batch_size > out->size)
        LOG(LogLevel::ERROR, "Output state buffer too small for " + this->get_layer_info());

    output_states.width = out_width;
    output_states.height = out_height;
    output_states.depth = out_channels;
    output_states.block_size = batch_size;
    output_states.actual_size = output_size;

    const int woho = (int)(out_width * out_height), wihi = (int)(in_width * in_height);
    if (act != 0)
        TAGI_OK_OR_THROW(tagi_conv2d_fwd_act(d_mu_w, d_var_w, d_mu_b, d_var_b, in->d_mu_a,
                                             in->d_var_a, d_idx_mwa_2, woho, (int)out_channels,
                                             wihi, (int)in_channels, (int)kernel_size, batch_size,
                                             bias ? 1 : 0, act, out->d_mu_a, out->d_var_a,
                                             out->d_jcb, host_stream()));
    else
        TAGI_OK_OR_THROW(tagi_conv2d_fwd(d_mu_w, d_var_w, d_mu_b, d_var_b, in->d_mu_a,
                                         in->d_var_a, d_idx_mwa_2, woho, (int)out_channels, wihi,
                                         (int)in_channels, (int)kernel_size, batch_size,
                                         bias ? 1 : 0, out->d_mu_a, out->d_var_a, host_stream()));
    out->jcb_ones = true;
    if (training) this->store_states_for_training_hip(*in, *out);
    if (act != 0) out->jcb_ones = false;  // the activation's Jacobian was written
}

// reference: Conv2dCuda::backward, src/conv2d_layer_cuda.cu:453-519. No temporary
// buffers are needed: the permutations are folded into the kernels' addressing.
void Conv2dHip::backward(BaseDeltaStates &input_delta_states, BaseDeltaStates &output_delta_states,
                         BaseTempStates &, bool state_udapte) {
    const float *res_mu = bwd_residual_mu, *res_var = bwd_residual_var;
    const int res_mode = bwd_residual_mode;
    bwd_residual_mu = bwd_residual_var = nullptr;
    bwd_residual_mode = 0;
    auto *din = as<DeltaStateHip>(input_delta_states);
    auto *dout = as<DeltaStateHip>(output_delta_states);
    auto *bwd = dynamic_cast<BackwardStateHip *>(this->bwd_states.get());
    const int batch_size = (int)input_delta_states.block_size;
    const int woho = (int)(out_width * out_height), wihi = (int)(in_width * in_height);
    if (state_udapte && input_size * batch_size > dout->size)
        LOG(LogLevel::ERROR, "Delta state buffer too small for " + this->get_layer_info());
    if (!state_udapte && res_mu != nullptr)
        LOG(LogLevel::ERROR, "Residual innovations handed to a layer that skips its state update");
    // one call for both contractions: where they run on the stencil kernels they share a launch
    TAGI_OK_OR_THROW(tagi_conv2d_bwd(
        d_mu_w, d_var_w, d_var_b, bwd->d_mu_a, bwd->jcb_ptr(), din->d_delta_mu, din->d_delta_var,
        d_idx_mwa_2, d_idx_cov_zwa_1, d_idx_var_z_ud, batch_size, (int)out_channels, woho, wihi,
        (int)in_channels, (int)kernel_size, row_zw, bias ? 1 : 0, state_udapte ? 1 : 0,
        param_update ? 1 : 0, res_mu, res_var, res_mode, dout->d_delta_mu, dout->d_delta_var,
        d_delta_mu_w, d_delta_var_w, d_delta_mu_b, d_delta_var_b, host_stream()));
}

// ---- ReLU ---------------------------------------------------------------------------------
std::unique_ptr<BaseLayer> ReLU::to_cuda(int device_idx) {
    this->device = "cuda";
    auto layer = std::make_unique<ReLUHip>();
    layer->device_idx = device_idx;
    return layer;
}

std::unique_ptr<BaseLayer> ReLUHip::to_cuda(int device_idx) {
    auto layer = std::make_unique<ReLUHip>();
    layer->device_idx = device_idx;
    return layer;
}

// reference: ReLUCuda::forward (src/activation_cuda.cu), CPU form src/activation.cpp:552-577
void ReLUHip::forward(BaseHiddenStates &input_states, BaseHiddenStates &output_states,
                      BaseTempStates &) {
    auto *in = as<HiddenStateHip>(input_states);
    auto *out = as<HiddenStateHip>(output_states);
    const size_t n = input_states.actual_size * input_states.block_size;
    if (n > out->size) LOG(LogLevel::ERROR, "Output state buffer too small for ReLU");
    TAGI_OK_OR_THROW(tagi_relu_fwd(in->d_mu_a, in->d_var_a, n, out->d_mu_a, out->d_jcb, out->d_var_a,
                                   host_stream()));
    out->jcb_ones = false;
    this->input_size = input_states.actual_size;
    this->output_size = input_states.actual_size;
    output_states.block_size = input_states.block_size;
    output_states.actual_size = input_states.actual_size;
    output_states.width = input_states.width;
    output_states.height = input_states.height;
    output_states.depth = input_states.depth;
}

}  // namespace tagi_host

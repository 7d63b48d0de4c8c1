// Sequential and OutputUpdater: see sequential.h.
#include "sequential.h"

#include "host_util.h"

#include <hip/hip_runtime_api.h>
#include <sys/stat.h>

#include <fstream>
#include <sstream>

#include "../../include/tagi_hip.h"
#include "logger.h"

namespace tagi_host {

constexpr int PACK_SIZE = 4;  // state buffers are sized in multiples of 4 floats

int get_cuda_device_count() {
    int n = 0;
    if (tagi_hip_device_count(&n) != TAGI_OK) return 0;
    return n;
}
bool is_cuda_available() { return get_cuda_device_count() > 0; }

int get_current_cuda_device() {
    if (!is_cuda_available()) return -1;
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess) {
        LOG(LogLevel::ERROR, "Failed to get current CUDA device");
        return -1;
    }
    return device;
}

bool set_cuda_device(int device_index) {
    if (!is_cuda_available()) {
        LOG(LogLevel::ERROR, "CUDA is not available");
        return false;
    }
    if (device_index < 0 || device_index >= get_cuda_device_count()) {
        LOG(LogLevel::ERROR, "Invalid CUDA device index: " + std::to_string(device_index));
        return false;
    }
    if (hipSetDevice(device_index) != hipSuccess) {
        LOG(LogLevel::ERROR, "Failed to set CUDA device");
        return false;
    }
    return true;
}

bool is_cuda_device_available(int device_index) {
    if (!is_cuda_available()) return false;
    if (device_index < 0 || device_index >= get_cuda_device_count()) return false;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device_index) != hipSuccess) {
        LOG(LogLevel::ERROR, "Failed to get CUDA device properties");
        return false;
    }
    return prop.computeMode != hipComputeModeProhibited;
}

bool is_nccl_available() { return false; }

std::string get_cuda_device_properties(int device_index) {
    if (!is_cuda_available()) return "CUDA is not available";
    if (device_index < 0 || device_index >= get_cuda_device_count())
        return "Invalid CUDA device index: " + std::to_string(device_index);
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device_index) != hipSuccess)
        return "Failed to get CUDA device properties";
    std::stringstream ss;
    ss << "Device " << device_index << ": " << prop.name << " (" << prop.gcnArchName << ")\n";
    ss << "  Total global memory: " << prop.totalGlobalMem / (1024 * 1024) << " MB\n";
    ss << "  Compute units: " << prop.multiProcessorCount << "\n";
    ss << "  Max threads per block: " << prop.maxThreadsPerBlock << "\n";
    ss << "  Shared memory (LDS) per block: " << prop.sharedMemPerBlock / 1024 << " KB\n";
    ss << "  Wavefront size: " << prop.warpSize << "\n";
    ss << "  Clock rate: " << prop.clockRate / 1000 << " MHz\n";
    ss << "  Memory clock rate: " << prop.memoryClockRate / 1000 << " MHz\n";
    ss << "  Memory bus width: " << prop.memoryBusWidth << " bits\n";
    ss << "  L2 cache size: " << prop.l2CacheSize / 1024 << " KB\n";
    return ss.str();
}

bool get_cuda_device_memory(int device_index, size_t &free_memory, size_t &total_memory) {
    if (!is_cuda_available()) {
        LOG(LogLevel::ERROR, "CUDA is not available");
        return false;
    }
    if (device_index < 0 || device_index >= get_cuda_device_count()) {
        LOG(LogLevel::ERROR, "Invalid CUDA device index: " + std::to_string(device_index));
        return false;
    }
    int current = 0;
    if (hipGetDevice(&current) != hipSuccess || hipSetDevice(device_index) != hipSuccess) {
        LOG(LogLevel::ERROR, "Failed to set CUDA device");
        return false;
    }
    const hipError_t e = hipMemGetInfo(&free_memory, &total_memory);
    (void)hipSetDevice(current);
    if (e != hipSuccess) {
        LOG(LogLevel::ERROR, "Failed to get CUDA memory info");
        return false;
    }
    return true;
}

// ---- OutputUpdater ------------------------------------------------------------------
OutputUpdater::OutputUpdater(const std::string model_device) : device(model_device) {
    const size_t colon = model_device.find(':');
    if (colon != std::string::npos) {
        this->device_idx = std::stoi(model_device.substr(colon + 1));
        this->device = model_device.substr(0, colon);
    }
    if (this->device == "hip") this->device = "cuda";
    if (this->device == "cuda")
        this->obs = std::make_shared<ObservationHip>(this->device_idx);
    else
        this->obs = std::make_shared<BaseObservation>();
}

ObservationHip *OutputUpdater::device_obs() {
    auto *o = dynamic_cast<ObservationHip *>(this->obs.get());
    if (o == nullptr)
        LOG(LogLevel::ERROR,
            "OutputUpdater(\"" + device + "\"): this library computes on the GPU only; "
            "construct it with the model's device (\"cuda\")");
    return o;
}

void OutputUpdater::update(BaseHiddenStates &output_states, std::vector<float> &mu_obs,
                           std::vector<float> &var_obs, BaseDeltaStates &delta_states) {
    if (mu_obs.size() != var_obs.size())
        LOG(LogLevel::ERROR, "Observation size does not fit the output buffers");
    this->update_raw(output_states, mu_obs.data(), var_obs.data(), mu_obs.size(), delta_states);
}

void OutputUpdater::update_raw(BaseHiddenStates &output_states, const float *mu_obs,
                               const float *var_obs, size_t n, BaseDeltaStates &delta_states) {
    ObservationHip *o = this->device_obs();
    auto *out = dynamic_cast<HiddenStateHip *>(&output_states);
    auto *delta = dynamic_cast<DeltaStateHip *>(&delta_states);
    if (out == nullptr || delta == nullptr)
        LOG(LogLevel::ERROR, "OutputUpdater needs device state buffers");
    if (n > out->size || n > delta->size)
        LOG(LogLevel::ERROR, "Observation size does not fit the output buffers");
    o->block_size = output_states.block_size;
    o->size = n;
    o->actual_size = output_states.block_size ? n / output_states.block_size : 0;
    o->upload(mu_obs, var_obs, n, nullptr, 0);
    delta->reset_zeros();
    TAGI_OK_OR_THROW(tagi_out_update_dense(out->d_mu_a, out->d_var_a, out->jcb_ptr(), o->d_mu_obs,
                                           o->d_var_obs, (int)o->size, delta->d_delta_mu,
                                           delta->d_delta_var, host_stream()));
}

void OutputUpdater::update_using_indices(BaseHiddenStates &output_states,
                                         std::vector<float> &mu_obs, std::vector<float> &var_obs,
                                         std::vector<int> &selected_idx,
                                         BaseDeltaStates &delta_states) {
    if (mu_obs.size() != var_obs.size() || selected_idx.size() != mu_obs.size())
        LOG(LogLevel::ERROR, "Observations, variances and indices must have one size, a multiple "
                             "of the batch size");
    this->update_using_indices_raw(output_states, mu_obs.data(), var_obs.data(),
                                   selected_idx.data(), mu_obs.size(), delta_states);
}

void OutputUpdater::update_using_indices_raw(BaseHiddenStates &output_states,
                                             const float *mu_obs, const float *var_obs,
                                             const int *selected_idx, size_t n,
                                             BaseDeltaStates &delta_states) {
    ObservationHip *o = this->device_obs();
    auto *out = dynamic_cast<HiddenStateHip *>(&output_states);
    auto *delta = dynamic_cast<DeltaStateHip *>(&delta_states);
    if (out == nullptr || delta == nullptr)
        LOG(LogLevel::ERROR, "OutputUpdater needs device state buffers");
    if (output_states.block_size == 0 || n % output_states.block_size != 0)
        LOG(LogLevel::ERROR, "Observations, variances and indices must have one size, a multiple "
                             "of the batch size");
    const int n_obs = (int)output_states.actual_size;
    for (size_t i = 0; i < n; i++)
        if (selected_idx[i] < 1 || selected_idx[i] > n_obs)
            LOG(LogLevel::ERROR, "Selected index " + std::to_string(selected_idx[i]) +
                                     " outside 1.." + std::to_string(n_obs));
    o->block_size = output_states.block_size;
    o->size = n;
    o->actual_size = n / output_states.block_size;
    o->idx_size = n;
    const int n_enc = (int)(o->idx_size / output_states.block_size);
    if ((size_t)output_states.block_size * n_obs > delta->size)
        LOG(LogLevel::ERROR, "Output size does not fit the innovation buffers");
    // one launch: the kernel reads the observations where they are staged in pinned
    // memory and clears the rest of the innovation buffers itself
    const float *mu_at = nullptr, *var_at = nullptr;
    const int *idx_at = nullptr;
    o->stage(mu_obs, var_obs, n, selected_idx, &mu_at, &var_at, &idx_at);
    TAGI_OK_OR_THROW(tagi_out_update_indexed_reset(out->d_mu_a, out->d_var_a, out->jcb_ptr(), mu_at,
                                                   var_at, idx_at, n_obs, n_enc, (int)n,
                                                   delta->d_delta_mu, delta->d_delta_var,
                                                   delta->size, host_stream()));
    o->staged_work_queued();
}

void OutputUpdater::update_heteros(BaseHiddenStates &output_states, std::vector<float> &mu_obs,
                                   BaseDeltaStates &delta_states) {
    this->update_heteros_raw(output_states, mu_obs.data(), mu_obs.size(), delta_states);
}

void OutputUpdater::update_heteros_raw(BaseHiddenStates &output_states, const float *mu_obs,
                                       size_t n, BaseDeltaStates &delta_states) {
    ObservationHip *o = this->device_obs();
    auto *out = dynamic_cast<HiddenStateHip *>(&output_states);
    auto *delta = dynamic_cast<DeltaStateHip *>(&delta_states);
    if (out == nullptr || delta == nullptr)
        LOG(LogLevel::ERROR, "OutputUpdater needs device state buffers");
    if (2 * n > out->size || 2 * n > delta->size)
        LOG(LogLevel::ERROR, "Observation size does not fit the output buffers");
    o->block_size = output_states.block_size;
    o->size = n;
    o->actual_size = output_states.block_size ? n / output_states.block_size : 0;
    o->upload(mu_obs, nullptr, n, nullptr, 0);
    delta->reset_zeros();
    TAGI_OK_OR_THROW(tagi_out_update_heteros(out->d_mu_a, out->d_var_a, out->jcb_ptr(), o->d_mu_obs,
                                             (int)o->size, delta->d_delta_mu, delta->d_delta_var,
                                             host_stream()));
}

// ---- Sequential -----------------------------------------------------------------------
void Sequential::add_layer(std::shared_ptr<BaseLayer> layer) {
    if (this->device == "cpu")
        this->layers.push_back(layer);
    else if (this->device == "cuda")
        this->layers.push_back(layer->to_cuda(this->device_idx));
    else
        LOG(LogLevel::ERROR, "Invalid device: [" + this->device + "]");
}

void Sequential::add_layers() {
    if (this->layers.empty()) return;
    this->compute_input_output_size();
    this->set_buffer_size();
}

void Sequential::switch_to_cuda() {
    for (auto &layer : this->layers) layer = layer->to_cuda(this->device_idx);
}

// reference: src/sequential.cpp:32-73. "hip" is accepted as a synonym of "cuda".
void Sequential::to_device(const std::string &new_device) {
    this->clear_graphs();  // what a recorded graph refers to may change here
    if (new_device == "cpu") {
        this->device = "cpu";
        return;
    }
    std::string name = new_device;
    int idx = 0;
    const size_t colon = new_device.find(':');
    if (colon != std::string::npos) {
        name = new_device.substr(0, colon);
        try {
            idx = std::stoi(new_device.substr(colon + 1));
        } catch (const std::exception &) {
            LOG(LogLevel::ERROR, "Invalid device index format in: [" + new_device + "]");
        }
    }
    if (name == "hip") name = "cuda";
    if (name != "cuda") LOG(LogLevel::ERROR, "Invalid device: [" + new_device + "]");
    const int count = get_cuda_device_count();
    if (count == 0) LOG(LogLevel::ERROR, "CUDA is not available");
    if (idx < 0 || idx >= count)
        LOG(LogLevel::ERROR, "Invalid CUDA device index: " + std::to_string(idx) +
                                 ". Available devices: " + std::to_string(count));
    const bool already = this->device == "cuda";
    this->device = name;
    this->device_idx = idx;
    if (!already) this->switch_to_cuda();
    this->compute_input_output_size();
    this->set_buffer_size();
}

void Sequential::params_to_host() {
    for (auto &layer : layers) layer->params_to_host();
}
void Sequential::params_to_device() {
    for (auto &layer : layers) layer->params_to_device();
}

void Sequential::set_buffer_size() {
    int per_sample = this->z_buffer_block_size > 0 ? this->z_buffer_size / this->z_buffer_block_size
                                                   : this->z_buffer_size;
    for (auto &layer : layers) per_sample = std::max(per_sample, layer->get_max_num_states());
    per_sample = (per_sample + PACK_SIZE - 1) / PACK_SIZE * PACK_SIZE;
    this->z_buffer_size =
        this->z_buffer_block_size > 0 ? per_sample * this->z_buffer_block_size : per_sample;
}

void Sequential::compute_input_output_size() {
    int w = (int)layers.front()->in_width, h = (int)layers.front()->in_height;
    int d = (int)layers.front()->in_channels;
    for (auto &layer : layers) {
        layer->compute_input_output_size(InitArgs(w, h, d));
        w = (int)layer->out_width;
        h = (int)layer->out_height;
        d = (int)layer->out_channels;
    }
}

void Sequential::require_device(const char *what) const {
    if (this->device != "cuda")
        LOG(LogLevel::ERROR, std::string(what) + ": this library computes on the GPU only; call "
                                                 "to_device(\"cuda\") first");
}

void Sequential::init_output_state_buffer() {
    output_z_buffer = std::make_shared<HiddenStateHip>(z_buffer_size, z_buffer_block_size, device_idx);
    input_z_buffer = std::make_shared<HiddenStateHip>(z_buffer_size, z_buffer_block_size, device_idx);
    // ping-pong buffers: what a layer has read is dead, so it may keep the arrays
    for (auto *b : {output_z_buffer.get(), input_z_buffer.get()})
        dynamic_cast<HiddenStateHip *>(b)->transient = !graphs_on_;
    temp_states = std::make_shared<TempStateHip>(0, z_buffer_block_size, device_idx);
}

void Sequential::init_delta_state_buffer() {
    output_delta_z_buffer =
        std::make_shared<DeltaStateHip>(z_buffer_size, z_buffer_block_size, device_idx);
    input_delta_z_buffer =
        std::make_shared<DeltaStateHip>(z_buffer_size, z_buffer_block_size, device_idx);
}

// Lazy allocation at the first batch, regrowth when the batch size changes
// (reference: src/sequential.cpp:290-318).
void Sequential::prepare_buffers(int batch_size) {
    if (this->z_buffer_block_size == 0) {
        this->z_buffer_block_size = batch_size;
        this->z_buffer_size = batch_size * this->z_buffer_size;
        this->init_output_state_buffer();
        if (this->training) this->init_delta_state_buffer();
    }
    if (batch_size != this->z_buffer_block_size) {
        this->z_buffer_size = batch_size * (this->z_buffer_size / this->z_buffer_block_size);
        this->z_buffer_block_size = batch_size;
        this->input_z_buffer->set_size(this->z_buffer_size, batch_size);
        this->output_z_buffer->set_size(this->z_buffer_size, batch_size);
        // a model first run in eval mode has no delta buffers yet: they are created
        // below at the new size
        if (this->training && this->input_delta_z_buffer) {
            this->input_delta_z_buffer->set_size(this->z_buffer_size, batch_size);
            this->output_delta_z_buffer->set_size(this->z_buffer_size, batch_size);
        }
    }
    if (this->training && !this->input_delta_z_buffer) this->init_delta_state_buffer();
}

void Sequential::set_threads(unsigned n) {
    this->num_threads = n;
    for (auto &layer : layers) layer->set_threads(n);
}
void Sequential::train() {
    this->clear_graphs();  // what a recorded graph refers to may change here
    this->training = true;
    for (auto &layer : layers) layer->train();
}
void Sequential::eval() {
    this->clear_graphs();  // what a recorded graph refers to may change here
    this->training = false;
    for (auto &layer : layers) layer->eval();
}
std::string Sequential::get_device() { return this->device; }

void Sequential::forward(const std::vector<float> &mu_x, const std::vector<float> &var_x) {
    if (!var_x.empty() && var_x.size() != mu_x.size())
        LOG(LogLevel::ERROR, "Input mean and variance differ in size");
    this->forward(mu_x.data(), var_x.empty() ? nullptr : var_x.data(), mu_x.size());
}

void Sequential::forward(const float *mu_x, const float *var_x, size_t n) {
    this->require_device("forward");
    const int in_size = this->layers.front()->get_input_size();
    if (in_size <= 0 || n == 0 || n % in_size != 0)
        LOG(LogLevel::ERROR, "Input size mismatch: " + std::to_string(in_size) + " vs " +
                                 std::to_string(n));
    const int batch_size = (int)(n / in_size);
    this->prepare_buffers(batch_size);
    auto *in = dynamic_cast<HiddenStateHip *>(this->input_z_buffer.get());
    in->set_input_raw(mu_x, var_x, n, batch_size);
    auto *out = dynamic_cast<HiddenStateHip *>(this->output_z_buffer.get());
    this->run_or_replay(GraphKey(0, in->d_mu_a, out->d_mu_a, batch_size, training ? 1 : 0),
                        [this] { this->forward_layers(0); });
}

// Layers from `first` on, reading input_z_buffer; the network's output ends up in
// output_z_buffer. An activation that follows a Linear / Conv2d layer runs in that
// layer's epilogue (one launch and one pass over the tensor instead of two).
void Sequential::forward_layers(size_t first) {
    for (size_t i = first; i < layers.size(); i++) {
        const int act = i + 1 < layers.size()
                            ? fusable_activation(layers[i].get(), layers[i + 1].get())
                            : 0;
        layers[i]->fused_activation = act;
        layers[i]->forward(*input_z_buffer, *output_z_buffer, *temp_states);
        if (act != 0) activation_absorbed(layers[++i].get(), *output_z_buffer);
        std::swap(input_z_buffer, output_z_buffer);
    }
    std::swap(output_z_buffer, input_z_buffer);
}

void Sequential::forward(BaseHiddenStates &input_states) {
    this->require_device("forward");
    this->prepare_buffers((int)input_states.block_size);
    layers.front()->forward(input_states, *input_z_buffer, *temp_states);
    this->forward_layers(1);
}

// reference: src/sequential.cpp:387-411. Activations do not consume a delta
// buffer; the first layer propagates to its input only on request.
void Sequential::backward() {
    this->require_device("backward");
    auto *din = dynamic_cast<DeltaStateHip *>(this->input_delta_z_buffer.get());
    auto *dout = dynamic_cast<DeltaStateHip *>(this->output_delta_z_buffer.get());
    if (din == nullptr || dout == nullptr)
        LOG(LogLevel::ERROR, "backward needs a forward pass in training mode first");
    this->run_or_replay(GraphKey(1, din->d_delta_mu, dout->d_delta_mu, (int)din->block_size,
                                 (input_state_update ? 1 : 0) | (param_update ? 2 : 0)),
                        [this] { this->backward_layers(); });
}

void Sequential::backward_layers() {
    for (size_t i = layers.size() - 1; i >= 1; i--) {
        BaseLayer *layer = layers[i].get();
        layer->backward(*input_delta_z_buffer, *output_delta_z_buffer, *temp_states);
        if (layer->get_layer_type() != LayerType::Activation)
            std::swap(input_delta_z_buffer, output_delta_z_buffer);
    }
    layers.front()->backward(*input_delta_z_buffer, *output_delta_z_buffer, *temp_states,
                             this->input_state_update);
}

// ---- HIP graph replay -------------------------------------------------------------------
static hipStream_t graph_stream() {
    static hipStream_t stream = nullptr;
    // an ordinary (blocking) stream at the default priority: synchronous copies on the
    // null stream still order with it
    if (stream == nullptr) HIP_OK(hipStreamCreateWithFlags(&stream, hipStreamDefault));
    return stream;
}

void Sequential::enable_graphs(bool on) {
    this->require_device("enable_graphs");
    if (on == graphs_on_) return;
    HIP_OK(hipDeviceSynchronize());
    this->clear_graphs();
    graphs_on_ = on;
    // the host classes share one stream: it is the recording stream while any model has
    // graphs on, the null stream otherwise
    static int models_with_graphs = 0;
    models_with_graphs += on ? 1 : -1;
    set_host_stream(models_with_graphs > 0 ? graph_stream() : nullptr);
    // replayed work must meet the same arrays every step: no trading with the buffers
    for (auto *b : {output_z_buffer.get(), input_z_buffer.get()})
        if (auto *h = dynamic_cast<HiddenStateHip *>(b)) h->transient = !on;
}

Sequential::~Sequential() {
    // (a model destroyed with graphs on hands the stream back like one that switches off)
    if (graphs_on_ && this->device == "cuda") {
        try {
            this->enable_graphs(false);
        } catch (...) {
        }
    }
    this->clear_graphs();
}

int Sequential::graphs_captured() const {
    int n = 0;
    for (const auto &kv : graphs_) n += kv.second.exec != nullptr ? 1 : 0;
    return n;
}

void Sequential::clear_graphs() {
    for (auto &kv : graphs_)
        if (kv.second.exec != nullptr)
            (void)hipGraphExecDestroy(static_cast<hipGraphExec_t>(kv.second.exec));
    graphs_.clear();
}

bool Sequential::only_plain_layers() const {
    for (const auto &layer : layers) {
        const LayerType t = layer->get_layer_type();
        if (t == LayerType::LayerBlock || t == LayerType::ResNetBlock) return false;
    }
    return true;
}

// `body` queues device work on host_stream() and moves the buffer pointers around; it
// is run as it is, or recorded into a graph, or skipped in favour of the recorded graph
// (whose effect on the buffer pointers is then repeated by hand).
void Sequential::run_or_replay(const GraphKey &key, const std::function<void()> &body) {
    if (!graphs_on_ || host_stream() == nullptr || !this->only_plain_layers()) {
        body();
        return;
    }
    GraphEntry &e = graphs_[key];
    hipStream_t stream = host_stream();
    if (e.exec != nullptr) {
        HIP_OK(hipGraphLaunch(static_cast<hipGraphExec_t>(e.exec), stream));
        if (e.swaps_state) std::swap(input_z_buffer, output_z_buffer);
        if (e.swaps_delta) std::swap(input_delta_z_buffer, output_delta_z_buffer);
        return;
    }
    // the first runs allocate (workspaces, what layers keep for the backward pass):
    // they stay eager
    if (e.unusable || e.warm_runs < 2) {
        e.warm_runs++;
        body();
        return;
    }
    const auto state_before = input_z_buffer, out_before = output_z_buffer;
    const auto delta_before = input_delta_z_buffer, dout_before = output_delta_z_buffer;
    auto restore = [&] {
        input_z_buffer = state_before;
        output_z_buffer = out_before;
        input_delta_z_buffer = delta_before;
        output_delta_z_buffer = dout_before;
    };
    if (hipStreamBeginCapture(stream, hipStreamCaptureModeRelaxed) != hipSuccess) {
        (void)hipGetLastError();
        e.unusable = true;
        body();
        return;
    }
    hipGraph_t graph = nullptr;
    try {
        body();
    } catch (...) {
        (void)hipStreamEndCapture(stream, &graph);
        if (graph != nullptr) (void)hipGraphDestroy(graph);
        (void)hipGetLastError();
        e.unusable = true;
        throw;
    }
    hipGraphExec_t exec = nullptr;
    hipError_t rc = hipStreamEndCapture(stream, &graph);
    if (rc == hipSuccess && graph != nullptr) rc = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    if (graph != nullptr) (void)hipGraphDestroy(graph);
    if (rc != hipSuccess || exec == nullptr) {
        // something in the body cannot be recorded: nothing has run yet, so run it now
        (void)hipGetLastError();
        e.unusable = true;
        restore();
        body();
        return;
    }
    e.exec = exec;
    e.swaps_state = input_z_buffer != state_before;
    e.swaps_delta = input_delta_z_buffer != delta_before;
    HIP_OK(hipGraphLaunch(exec, stream));
}

void Sequential::step() {
    this->require_device("step");
    // update_weights + update_biases of every layer (reference: src/sequential.cpp:
    // 440-448), gathered into one launch per 24 layers
    std::vector<tagi_update_item> items;
    for (auto &layer : layers) {
        if (layer->get_layer_type() == LayerType::Activation) continue;
        layer->collect_update_items(items);
    }
    if (!items.empty())
        TAGI_OK_OR_THROW(tagi_model_update(items.data(), (int)items.size(), host_stream()));
}

std::string Sequential::get_layer_stack_info() const {
    std::stringstream ss;
    for (const auto &layer : layers)
        if (layer) ss << layer->get_layer_info() << "\n";
    return ss.str();
}

void Sequential::preinit_layer() {
    for (auto &layer : layers)
        if (layer) layer->preinit_layer();
}

// Creates the directory part of `filename` when it does not exist yet (one level,
// as the reference's create_directory does, src/common.cpp:57-73).
static void make_parent_directory(const std::string &filename) {
    const size_t cut = filename.find_last_of("\\/");
    if (cut == std::string::npos || cut == 0) return;
    const std::string dir = filename.substr(0, cut);
    struct stat st;
    if (stat(dir.c_str(), &st) == -1) mkdir(dir.c_str(), 0777);
}

void Sequential::save(const std::string &filename) {
    make_parent_directory(filename);
    std::ofstream file(filename, std::ios::binary);
    if (!file.is_open()) LOG(LogLevel::ERROR, "Failed to open file for saving");
    for (auto &layer : layers) layer->save(file);
}

void Sequential::load(const std::string &filename) {
    this->clear_graphs();  // what a recorded graph refers to may change here
    this->preinit_layer();
    std::ifstream file(filename, std::ios::binary);
    if (!file.is_open()) LOG(LogLevel::ERROR, "Failed to open file for loading");
    for (auto &layer : layers) layer->load(file);
}

// Text checkpoint (reference: Sequential::save_csv / load_csv,
// src/sequential.cpp:612-709 over write_csv / read_csv, include/common.h:135-207):
// four files `<filename>_1_mw.csv`, `_2_Sw.csv`, `_3_mb.csv`, `_4_Sb.csv`, each the
// concatenation over the top-level layers of that parameter vector, one value
// per line in the stream's default float format (six significant digits). As in
// the reference only the vectors the top-level layers hold themselves are
// written: the members of a LayerBlock / ResNetBlock keep theirs and are skipped.
static void write_csv_column(const std::string &path, const std::vector<float> &v) {
    std::ofstream file(path);
    if (!file.is_open()) LOG(LogLevel::ERROR, "Failed to open file for saving: " + path);
    for (float x : v) file << x << "\n";
}

static void read_csv_column(const std::string &path, std::vector<float> &v) {
    std::ifstream file(path);
    if (!file.is_open()) LOG(LogLevel::ERROR, "Could not open the file: " + path);
    size_t count = 0;
    std::string line, cell;
    while (count < v.size() && std::getline(file, line)) {
        std::stringstream row(line);
        while (count < v.size() && std::getline(row, cell, ',')) {
            std::stringstream value(cell);
            float d = 0.0f;
            value >> d;
            v[count++] = d;
        }
    }
    if (count != v.size())
        LOG(LogLevel::ERROR, "There is missing data in " + path + ": expected " +
                                 std::to_string(v.size()) + " values, found " +
                                 std::to_string(count));
}

void Sequential::save_csv(const std::string &filename) {
    make_parent_directory(filename);
    std::vector<float> mu_w, var_w, mu_b, var_b;
    for (auto &layer : layers) {
        layer->params_to_host();
        mu_w.insert(mu_w.end(), layer->mu_w.begin(), layer->mu_w.end());
        var_w.insert(var_w.end(), layer->var_w.begin(), layer->var_w.end());
        mu_b.insert(mu_b.end(), layer->mu_b.begin(), layer->mu_b.end());
        var_b.insert(var_b.end(), layer->var_b.begin(), layer->var_b.end());
    }
    write_csv_column(filename + "_1_mw.csv", mu_w);
    write_csv_column(filename + "_2_Sw.csv", var_w);
    write_csv_column(filename + "_3_mb.csv", mu_b);
    write_csv_column(filename + "_4_Sb.csv", var_b);
}

void Sequential::load_csv(const std::string &filename) {
    this->clear_graphs();  // what a recorded graph refers to may change here
    size_t num_weights = 0, num_biases = 0;
    for (auto &layer : layers) {
        num_weights += layer->mu_w.size();
        num_biases += layer->mu_b.size();
    }
    std::vector<float> mu_w(num_weights), var_w(num_weights), mu_b(num_biases), var_b(num_biases);
    read_csv_column(filename + "_1_mw.csv", mu_w);
    read_csv_column(filename + "_2_Sw.csv", var_w);
    read_csv_column(filename + "_3_mb.csv", mu_b);
    read_csv_column(filename + "_4_Sb.csv", var_b);
    size_t w0 = 0, b0 = 0;
    for (auto &layer : layers) {
        const size_t nw = layer->mu_w.size(), nb = layer->mu_b.size();
        std::copy(mu_w.begin() + w0, mu_w.begin() + w0 + nw, layer->mu_w.begin());
        std::copy(var_w.begin() + w0, var_w.begin() + w0 + nw, layer->var_w.begin());
        std::copy(mu_b.begin() + b0, mu_b.begin() + b0 + nb, layer->mu_b.begin());
        std::copy(var_b.begin() + b0, var_b.begin() + b0 + nb, layer->var_b.begin());
        w0 += nw;
        b0 += nb;
        if (auto *d = dynamic_cast<BaseLayerHip *>(layer.get()))
            if (d->d_mu_w != nullptr) d->params_to_device();
    }
}

// reference: Sequential::get_norm_mean_var, src/sequential.cpp:521-553
std::unordered_map<std::string, BaseLayer::NormStats> Sequential::get_norm_mean_var() {
    std::unordered_map<std::string, BaseLayer::NormStats> all;
    for (size_t i = 0; i < layers.size(); i++) {
        auto stats = layers[i]->get_norm_mean_var();
        if (std::get<0>(stats).empty()) continue;
        all[layers[i]->get_layer_info() + "_" + std::to_string(i)] = stats;
    }
    return all;
}

std::vector<ParameterTuple> Sequential::parameters() {
    std::vector<ParameterTuple> params;
    for (auto &layer : layers) {
        if (layer->get_layer_type() == LayerType::Activation ||
            layer->get_layer_type() == LayerType::Pool2d)
            continue;
        auto p = layer->parameters();
        params.insert(params.end(), p.begin(), p.end());
    }
    return params;
}

ParameterMap Sequential::state_dict() {
    ParameterMap sd;
    for (size_t i = 0; i < layers.size(); i++) {
        if (layers[i]->get_layer_type() == LayerType::Activation ||
            layers[i]->get_layer_type() == LayerType::Pool2d)
            continue;
        auto p = layers[i]->get_parameters_as_map(std::to_string(i));
        sd.insert(p.begin(), p.end());
    }
    return sd;
}

void Sequential::load_state_dict(const ParameterMap &sd) {
    this->clear_graphs();  // what a recorded graph refers to may change here
    for (size_t i = 0; i < layers.size(); i++) {
        if (layers[i]->get_layer_type() == LayerType::Activation ||
            layers[i]->get_layer_type() == LayerType::Pool2d)
            continue;
        layers[i]->load_parameters_from_map(sd, std::to_string(i));
    }
}

void Sequential::params_from(const Sequential &ref) {
    this->clear_graphs();  // what a recorded graph refers to may change here
    if (layers.size() != ref.layers.size()) LOG(LogLevel::ERROR, "Model architecture is different.");
    for (size_t i = 0; i < layers.size(); i++) {
        BaseLayer *src = ref.layers[i].get();
        if (auto *s = dynamic_cast<BaseLayerHip *>(src)) s->params_to_host();
        layers[i]->num_weights = src->num_weights;
        layers[i]->num_biases = src->num_biases;
        layers[i]->mu_w = src->mu_w;
        layers[i]->var_w = src->var_w;
        layers[i]->mu_b = src->mu_b;
        layers[i]->var_b = src->var_b;
        if (auto *d = dynamic_cast<BaseLayerHip *>(layers[i].get())) d->adopt_host_params();
    }
}

std::unordered_map<std::string, int> Sequential::get_neg_var_w_counter() {
    std::unordered_map<std::string, int> counter;
    for (size_t i = 0; i < layers.size(); i++) {
        if (layers[i]->get_layer_type() == LayerType::Activation) continue;
        counter[layers[i]->get_layer_name() + "." + std::to_string(i)] =
            layers[i]->get_neg_var_w_counter();
    }
    return counter;
}

void Sequential::output_to_host() {
    if (auto *o = dynamic_cast<HiddenStateHip *>(output_z_buffer.get())) o->to_host();
}

void Sequential::delta_z_to_host() {
    if (auto *d = dynamic_cast<DeltaStateHip *>(input_delta_z_buffer.get())) d->to_host();
    if (auto *d = dynamic_cast<DeltaStateHip *>(output_delta_z_buffer.get())) d->to_host();
}

// reference: src/sequential.cpp:499-515 (the vectors replace the host copy of the
// input delta buffer and must have its capacity)
void Sequential::set_delta_z(std::vector<float> &delta_mu, std::vector<float> &delta_var) {
    auto *d = dynamic_cast<DeltaStateHip *>(input_delta_z_buffer.get());
    if (d == nullptr) LOG(LogLevel::ERROR, "set_delta_z needs a forward pass in training mode first");
    if (delta_mu.size() != d->size || delta_var.size() != d->size)
        LOG(LogLevel::ERROR, "set_delta_z: vectors must have the buffer size " +
                                 std::to_string(d->size));
    d->delta_mu = delta_mu;
    d->delta_var = delta_var;
    d->to_device();
}

std::tuple<std::vector<float>, std::vector<float>> Sequential::get_outputs_vec() {
    auto *o = dynamic_cast<HiddenStateHip *>(output_z_buffer.get());
    if (o == nullptr) LOG(LogLevel::ERROR, "get_outputs needs a forward pass first");
    const size_t n = o->block_size * layers.back()->output_size;
    o->to_host(n);  // only the part that holds outputs, not the whole capacity
    return {std::vector<float>(o->mu_a.begin(), o->mu_a.begin() + n),
            std::vector<float>(o->var_a.begin(), o->var_a.begin() + n)};
}

// innovations that reached the model's input (needs input_state_update)
std::tuple<std::vector<float>, std::vector<float>> Sequential::get_input_states_vec() {
    if (!this->input_state_update) LOG(LogLevel::ERROR, "input_state_update is set to False.");
    auto *d = dynamic_cast<DeltaStateHip *>(output_delta_z_buffer.get());
    if (d == nullptr) LOG(LogLevel::ERROR, "get_input_states needs a backward pass first");
    d->to_host();
    const size_t n = this->z_buffer_block_size * layers.front()->input_size;
    return {std::vector<float>(d->delta_mu.begin(), d->delta_mu.begin() + n),
            std::vector<float>(d->delta_var.begin(), d->delta_var.begin() + n)};
}

}  // namespace tagi_host

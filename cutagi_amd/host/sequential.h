// Model driver and output updater, mirroring the reference's Sequential
// (include/sequential.h, src/sequential.cpp:25-73,102-448,574-768) and
// OutputUpdater (include/base_output_updater.h, src/base_output_updater.cpp:269-386,
// src/output_updater_cuda.cu:146-223).
#pragma once
#include <functional>
#include <map>
#include <memory>
#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

#include "layers.h"

namespace tagi_host {

// Device queries under the reference's names (src/cuda_utils.cpp:11-230); "cuda"
// means the HIP device here, as everywhere in this API.
bool is_cuda_available();
int get_cuda_device_count();
int get_current_cuda_device();                 // -1 without a device
bool set_cuda_device(int device_index);        // logs and throws on an invalid index
bool is_cuda_device_available(int device_index);
bool is_nccl_available();                      // always false: one GPU, no collectives
std::string get_cuda_device_properties(int device_index);
bool get_cuda_device_memory(int device_index, size_t &free_memory, size_t &total_memory);

class OutputUpdater {
   public:
    std::string device = "cpu";
    int device_idx = 0;
    std::shared_ptr<BaseObservation> obs;

    explicit OutputUpdater(const std::string model_device);
    void update(BaseHiddenStates &output_states, std::vector<float> &mu_obs,
                std::vector<float> &var_obs, BaseDeltaStates &delta_states);
    void update_using_indices(BaseHiddenStates &output_states, std::vector<float> &mu_obs,
                              std::vector<float> &var_obs, std::vector<int> &selected_idx,
                              BaseDeltaStates &delta_states);
    // The same two updates with the observations read straight from caller memory
    // (what the Python binding passes for float32 / int32 numpy arrays).
    void update_raw(BaseHiddenStates &output_states, const float *mu_obs, const float *var_obs,
                    size_t n, BaseDeltaStates &delta_states);
    void update_using_indices_raw(BaseHiddenStates &output_states, const float *mu_obs,
                                  const float *var_obs, const int *selected_idx, size_t n,
                                  BaseDeltaStates &delta_states);
    // Output layer with a learned error variance (twice as many output units as
    // observations); reference: OutputUpdater::update_heteros,
    // src/base_output_updater.cpp:391-408.
    void update_heteros(BaseHiddenStates &output_states, std::vector<float> &mu_obs,
                        BaseDeltaStates &delta_states);
    void update_heteros_raw(BaseHiddenStates &output_states, const float *mu_obs, size_t n,
                            BaseDeltaStates &delta_states);

   private:
    ObservationHip *device_obs();
};

class Sequential {
   public:
    std::shared_ptr<BaseHiddenStates> output_z_buffer, input_z_buffer;
    std::shared_ptr<BaseDeltaStates> output_delta_z_buffer, input_delta_z_buffer;
    std::shared_ptr<BaseTempStates> temp_states;

    int z_buffer_size = 0;        // per-sample capacity until the first forward, then x batch
    int z_buffer_block_size = 0;  // batch size the buffers were made for
    int num_samples = 0;
    int input_size = 0;
    bool training = true;
    bool param_update = true;
    bool input_state_update = false;
    unsigned num_threads = 1;
    std::string device = "cpu";
    int device_idx = 0;
    std::vector<std::shared_ptr<BaseLayer>> layers;

    Sequential() = default;
    ~Sequential();
    Sequential(const Sequential &) = delete;
    Sequential &operator=(const Sequential &) = delete;
    void add_layer(std::shared_ptr<BaseLayer> layer);
    void add_layers();  // call once after the last add_layer

    void to_device(const std::string &new_device);
    void params_to_host();
    void params_to_device();
    void set_threads(unsigned num_threads);
    void train();
    void eval();
    std::string get_device();

    void forward(const std::vector<float> &mu_x,
                 const std::vector<float> &var_x = std::vector<float>());
    // n values per array; var_x may be null (zero input variance)
    void forward(const float *mu_x, const float *var_x, size_t n);
    void forward(BaseHiddenStates &input_states);
    void backward();
    void step();

    // Not in the reference. A small network's training step is a chain of a dozen short
    // launches, and the host needs longer to queue them than the GPU to run them. With
    // graphs on, the launches of a forward pass (and of a backward pass) are recorded into
    // a HIP graph the third time they run with the same buffers and batch size, and
    // replayed as one submission from then on. What is replayed must not change between
    // steps, so in this mode layers copy what they keep for the backward pass instead of
    // trading arrays with the buffers, all device work of the host classes moves to one
    // ordinary stream (the null stream cannot be captured), and only networks of plain
    // layers (no LayerBlock / ResNetBlock, whose buffers trade contents) are replayed;
    // others run as before. Input transfers, the output update and step() are not part
    // of a graph. Results are the same kernels' results either way.
    void enable_graphs(bool on);
    bool graphs_enabled() const { return graphs_on_; }
    int graphs_captured() const;  // graphs held at the moment (for tests)

    std::string get_layer_stack_info() const;
    void preinit_layer();
    void save(const std::string &filename);
    void load(const std::string &filename);
    void save_csv(const std::string &filename);
    // per normalisation-carrying layer, keyed `<layer info>_<index>`
    std::unordered_map<std::string, BaseLayer::NormStats> get_norm_mean_var();
    void load_csv(const std::string &filename);
    std::vector<ParameterTuple> parameters();
    ParameterMap state_dict();
    void load_state_dict(const ParameterMap &state_dict);
    void params_from(const Sequential &ref_model);
    std::unordered_map<std::string, int> get_neg_var_w_counter();

    void output_to_host();
    void delta_z_to_host();
    void set_delta_z(std::vector<float> &delta_mu, std::vector<float> &delta_var);
    // first batch*outputs entries of the output buffer, copied to the host
    std::tuple<std::vector<float>, std::vector<float>> get_outputs_vec();
    std::tuple<std::vector<float>, std::vector<float>> get_input_states_vec();

   private:
    void switch_to_cuda();
    void compute_input_output_size();
    void set_buffer_size();
    void init_output_state_buffer();
    void init_delta_state_buffer();
    void prepare_buffers(int batch_size);
    void forward_layers(size_t first);
    void backward_layers();
    void require_device(const char *what) const;

    struct GraphEntry {
        void *exec = nullptr;    // hipGraphExec_t
        int warm_runs = 0;       // eager runs seen with this key (allocations happen in them)
        bool unusable = false;   // capture failed: stay eager
        bool swaps_state = false, swaps_delta = false;  // net effect on the buffer pointers
    };
    // (kind, first buffer's arrays, second buffer's arrays, batch size, flags)
    using GraphKey = std::tuple<int, const void *, const void *, int, int>;
    std::map<GraphKey, GraphEntry> graphs_;
    bool graphs_on_ = false;
    void clear_graphs();
    bool only_plain_layers() const;
    void run_or_replay(const GraphKey &key, const std::function<void()> &body);
};

}  // namespace tagi_host

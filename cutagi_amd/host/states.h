// State containers the layers exchange, mirroring the reference's
// include/data_struct.h:14-202 (host side) and include/data_struct_cuda.cuh:9-139
// (device side): same member names, same grow-only sizing, pointer-swapping
// ping-pong. The *Hip classes add raw device pointers next to the host vectors;
// the host vectors are refreshed only by an explicit to_host().
#pragma once
#include <hip/hip_runtime_api.h>

#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

namespace tagi_host {

using ParameterTuple =
    std::tuple<std::vector<float>, std::vector<float>, std::vector<float>, std::vector<float>>;
using ParameterMap = std::unordered_map<std::string, ParameterTuple>;

class BaseHiddenStates {
   public:
    std::vector<float> mu_a, var_a, jcb;
    size_t size = 0;         // capacity in floats
    size_t block_size = 0;   // batch size
    size_t actual_size = 0;  // features per sample currently held
    size_t width = 0, height = 0, depth = 0;
    int device_idx = 0;

    BaseHiddenStates(size_t n, size_t m, int device_idx = 0);
    BaseHiddenStates() = default;
    virtual ~BaseHiddenStates() = default;
    virtual std::string get_name() const { return "BaseHiddenStates"; }
    virtual void set_input_x(const std::vector<float> &mu_x, const std::vector<float> &var_x,
                             size_t block_size);
    virtual void set_size(size_t size, size_t block_size);
    virtual void swap(BaseHiddenStates &other);
    virtual void copy_from(const BaseHiddenStates &source, int num_data = -1);
};

class BaseDeltaStates {
   public:
    std::vector<float> delta_mu, delta_var;
    size_t size = 0, block_size = 0, actual_size = 0;
    int device_idx = 0;

    BaseDeltaStates(size_t n, size_t m, int device_idx = 0);
    BaseDeltaStates() = default;
    virtual ~BaseDeltaStates() = default;
    virtual std::string get_name() const { return "BaseDeltaStates"; }
    virtual void reset_zeros();
    virtual void copy_from(const BaseDeltaStates &source, int num_data = -1);
    virtual void set_size(size_t size, size_t block_size);
    virtual void swap(BaseDeltaStates &other);
};

class BaseTempStates {
   public:
    std::vector<float> tmp_1, tmp_2;
    size_t size = 0, block_size = 0, actual_size = 0;
    int device_idx = 0;

    BaseTempStates(size_t n, size_t m, int device_idx = 0);
    BaseTempStates() = default;
    virtual ~BaseTempStates() = default;
    virtual std::string get_name() const { return "BaseTempStates"; }
    virtual void set_size(size_t size, size_t block_size);
};

class BaseBackwardStates {
   public:
    std::vector<float> mu_a, jcb;
    size_t size = 0;
    int device_idx = 0;

    explicit BaseBackwardStates(int num);
    BaseBackwardStates() = default;
    virtual ~BaseBackwardStates() = default;
    virtual std::string get_name() const { return "BaseBackwardStates"; }
    virtual void set_size(size_t size);
};

class BaseObservation {
   public:
    std::vector<float> mu_obs, var_obs;
    std::vector<int> selected_idx;
    size_t size = 0, block_size = 0, actual_size = 0, idx_size = 0;
    int device_idx = 0;

    BaseObservation() = default;
    virtual ~BaseObservation() = default;
    virtual std::string get_name() const { return "BaseObservation"; }
    void set_obs(std::vector<float> &mu_obs, std::vector<float> &var_obs);
    void set_selected_idx(std::vector<int> &selected_idx);
};

// ---- device side ---------------------------------------------------------------

// A device array of ones, at least n long, on the given device (grow-only, shared):
// what a consumer reads for a Jacobian that is known to be one everywhere.
const float *device_ones(size_t n, int device_idx);

class HiddenStateHip : public BaseHiddenStates {
   public:
    float *d_mu_a = nullptr, *d_var_a = nullptr, *d_jcb = nullptr;
    // The Jacobian is one everywhere and d_jcb was NOT written: Linear, Conv2d,
    // BatchNorm2d, AvgPool2d and the residual add produce such outputs, and marking
    // them costs nothing where the reference runs a fill kernel per layer
    // (src/base_layer_cuda.cu:464-486). Readers go through jcb_ptr().
    bool jcb_ones = false;
    // Set by the owner of a ping-pong buffer (Sequential, ResNetBlock): after a layer
    // has read it, its contents are dead, so the layer may keep its arrays for the
    // backward pass and leave its own old ones in their place instead of copying.
    bool transient = false;
    // Set by an owner that keeps the contents unchanged until its backward pass has run
    // (a ResNetBlock's copy of its input): a layer that reads it may borrow the arrays for
    // its own backward pass instead of copying them.
    bool stable = false;
    const float *jcb_ptr() const { return jcb_ones ? device_ones(size, device_idx) : d_jcb; }

    HiddenStateHip(size_t n, size_t m, int device_idx = 0);
    HiddenStateHip() = default;
    ~HiddenStateHip() override;
    std::string get_name() const override { return "HiddenStateCuda"; }
    void set_input_x(const std::vector<float> &mu_x, const std::vector<float> &var_x,
                     size_t block_size) override;
    void allocate_memory();
    void deallocate_memory();
    void to_device();
    void chunks_to_device(size_t chunk_size);
    // Inputs straight from caller memory to the device: mean copied, variance
    // copied or (var_x == nullptr) cleared on the device, Jacobian set to one by a
    // kernel. The host mirrors are not touched.
    void set_input_raw(const float *mu_x, const float *var_x, size_t n, size_t block_size);
    void to_host();
    void to_host(size_t n);  // first n entries only
    void set_size(size_t size, size_t block_size) override;
    void swap(BaseHiddenStates &other) override;
    void copy_from(const BaseHiddenStates &source, int num_data = -1) override;
};

class DeltaStateHip : public BaseDeltaStates {
   public:
    float *d_delta_mu = nullptr, *d_delta_var = nullptr;

    DeltaStateHip(size_t n, size_t m, int device_idx = 0);
    DeltaStateHip() = default;
    ~DeltaStateHip() override;
    std::string get_name() const override { return "DeltaStateCuda"; }
    void allocate_memory();
    void deallocate_memory();
    void to_device();
    void to_host();
    void reset_zeros() override;
    void copy_from(const BaseDeltaStates &source, int num_data = -1) override;
    void set_size(size_t size, size_t block_size) override;
    void swap(BaseDeltaStates &other) override;
};

class TempStateHip : public BaseTempStates {
   public:
    float *d_tmp_1 = nullptr, *d_tmp_2 = nullptr;

    TempStateHip(size_t n, size_t m, int device_idx = 0);
    TempStateHip() = default;
    ~TempStateHip() override;
    std::string get_name() const override { return "TempStateCuda"; }
    void allocate_memory();
    void deallocate_memory();
    void set_size(size_t size, size_t block_size) override;
};

class BackwardStateHip : public BaseBackwardStates {
   public:
    float *d_mu_a = nullptr, *d_jcb = nullptr;
    bool jcb_ones = false;  // as HiddenStateHip::jcb_ones
    // The arrays belong to a HiddenStateHip marked `stable` (nothing is freed here).
    bool borrowed = false;
    const float *jcb_ptr() const { return jcb_ones ? device_ones(size, device_idx) : d_jcb; }
    // exactly new_size floats per array (reallocates when the size differs)
    void resize_exact(size_t new_size, bool need_jcb);
    // points at the arrays of a stable state instead of owning any
    void borrow(float *mu_a, float *jcb, bool ones, size_t n);

    BackwardStateHip() = default;
    ~BackwardStateHip() override;
    std::string get_name() const override { return "BackwardStateCuda"; }
    void allocate_memory();
    void deallocate_memory();
    void to_host();
    void set_size(size_t size) override;
};

class ObservationHip : public BaseObservation {
   public:
    float *d_mu_obs = nullptr, *d_var_obs = nullptr;
    int *d_selected_idx = nullptr;
    size_t cap_obs = 0, cap_idx = 0;

    explicit ObservationHip(int device_idx = 0) { this->device_idx = device_idx; }
    ~ObservationHip() override;
    std::string get_name() const override { return "ObservationCuda"; }
    void to_device();  // grows the device arrays as needed, then copies
    // Same, straight from caller memory (no host mirror is kept): n observations and
    // variances, n_idx selected indices (idx may be null with n_idx = 0).
    void upload(const float *mu, const float *var, size_t n, const int *idx, size_t n_idx);
    // Copies the three arrays into pinned host memory that kernels can read and returns
    // where they lie; the caller queues the kernel that reads them on host_stream() and
    // then calls staged_work_queued(). The device arrays above are not touched.
    void stage(const float *mu, const float *var, size_t n, const int *idx, const float **mu_at,
               const float **var_at, const int **idx_at);
    void staged_work_queued();
   private:
    void reserve(size_t n, size_t n_idx);
};

}  // namespace tagi_host

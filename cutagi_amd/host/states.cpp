// Host and device state containers: see states.h. Device buffers are plain
// hipMalloc allocations owned by the object that made them. Everything runs on
// the null stream, which orders copies and kernels. The per-batch transfers
// (inputs, observations) go through a small ring of pinned staging buffers and do
// not block the host, so the host can queue a step's launches while the GPU still
// works on the previous ones, and device-to-device copies are asynchronous too;
// whole-buffer transfers (to_device / to_host) are plain synchronous copies.
#include "states.h"

#include "../../include/tagi_hip.h"

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstring>

#include "logger.h"

namespace tagi_host {

// inputs up to this size are fetched from pinned memory by a kernel (tagi_upload_input)
static constexpr size_t kKernelUploadMaxBytes = (size_t)1 << 20;

// (declared in host_util.h) the stream the host classes queue their device work on
static hipStream_t g_host_stream = nullptr;
hipStream_t host_stream() { return g_host_stream; }
void set_host_stream(hipStream_t stream) { g_host_stream = stream; }

namespace {
float *dev_alloc(size_t n, int device_idx) {
    float *p = nullptr;
    if (n == 0) return p;
    HIP_OK(hipSetDevice(device_idx));
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&p), n * sizeof(float)));
    return p;
}
void dev_free(float *&p) {
    if (p != nullptr) (void)hipFree(p);
    p = nullptr;
}
void h2d(float *dst, const float *src, size_t n) {
    if (n) HIP_OK(hipMemcpy(dst, src, n * sizeof(float), hipMemcpyHostToDevice));
}
void d2h(float *dst, const float *src, size_t n) {
    if (n) HIP_OK(hipMemcpy(dst, src, n * sizeof(float), hipMemcpyDeviceToHost));
}
void d2d(float *dst, const float *src, size_t n) {
    if (n)
        HIP_OK(hipMemcpyAsync(dst, src, n * sizeof(float), hipMemcpyDeviceToDevice, host_stream()));
}

// Pinned staging for the small host-to-device transfers of every batch. A copy
// from pageable memory blocks the host until the stream has drained; a copy from
// pinned memory does not. The caller's data is copied into the next slot of a
// ring, the transfer is queued from there, and an event marks when the slot may
// be written again (waited for only when the ring comes round to it).
class StagingRing {
   public:
    static constexpr int SLOTS = 8;
    // queues dst[0..bytes) = src[0..bytes) on the null stream of the current device
    void upload(void *dst, const void *src, size_t bytes) {
        const void *parts[1] = {src};
        const size_t sizes[1] = {bytes};
        this->upload_parts(dst, parts, sizes, 1);
    }
    // the same for several host pieces that lie back to back on the device: one transfer
    void upload_parts(void *dst, const void *const *parts, const size_t *sizes, int n) {
        size_t bytes = 0;
        for (int i = 0; i < n; i++) bytes += sizes[i];
        if (bytes == 0) return;
        void *host = this->stage(parts, sizes, n);
        HIP_OK(hipMemcpyAsync(dst, host, bytes, hipMemcpyHostToDevice, host_stream()));
        this->staged_work_queued();
    }
    // Copies the pieces back to back into the next pinned slot and returns it; the caller
    // queues the device work that reads the slot and then calls staged_work_queued().
    void *stage(const void *const *parts, const size_t *sizes, int n) {
        size_t bytes = 0;
        for (int i = 0; i < n; i++) bytes += sizes[i];
        Slot &s = slots_[next_];
        current_ = next_;
        next_ = (next_ + 1) % SLOTS;
        if (s.event == nullptr) HIP_OK(hipEventCreateWithFlags(&s.event, hipEventDisableTiming));
        if (s.used) HIP_OK(hipEventSynchronize(s.event));
        if (s.cap < bytes) {
            if (s.host != nullptr) HIP_OK(hipHostFree(s.host));
            s.cap = std::max(bytes, (size_t)1 << 16);
            HIP_OK(hipHostMalloc(&s.host, s.cap, hipHostMallocDefault));
        }
        size_t at = 0;
        for (int i = 0; i < n; i++) {
            if (sizes[i]) std::memcpy(static_cast<char *>(s.host) + at, parts[i], sizes[i]);
            at += sizes[i];
        }
        return s.host;
    }
    void staged_work_queued() {
        Slot &s = slots_[current_];
        HIP_OK(hipEventRecord(s.event, host_stream()));
        s.used = true;
    }

   private:
    struct Slot {
        void *host = nullptr;
        size_t cap = 0;
        hipEvent_t event = nullptr;
        bool used = false;
    };
    Slot slots_[SLOTS];
    int next_ = 0, current_ = 0;
};
// one ring per device, created on first use and kept until the process ends
StagingRing &staging_ring(int device_idx) {
    static StagingRing rings[16];
    return rings[device_idx >= 0 && device_idx < 16 ? device_idx : 0];
}
}  // namespace

const float *device_ones(size_t n, int device_idx) {
    static float *ones[16] = {};
    static size_t cap[16] = {};
    if (device_idx < 0 || device_idx >= 16) LOG(LogLevel::ERROR, "Invalid device index");
    if (n > cap[device_idx]) {
        HIP_OK(hipSetDevice(device_idx));
        HIP_OK(hipDeviceSynchronize());  // kernels in flight may still read the old array
        dev_free(ones[device_idx]);
        ones[device_idx] = dev_alloc(n, device_idx);
        cap[device_idx] = n;
        if (tagi_store_states(nullptr, nullptr, 0, nullptr, nullptr, ones[device_idx], n,
                              nullptr) != TAGI_OK)
            LOG(LogLevel::ERROR, "Cannot fill the array of ones");
    }
    return ones[device_idx];
}

// ---- BaseHiddenStates (reference: src/data_struct.cpp:6-95) ---------------------
BaseHiddenStates::BaseHiddenStates(size_t n, size_t m, int device_idx)
    : mu_a(n, 0.0f), var_a(n, 0.0f), jcb(n, 1.0f), size(n), block_size(m), device_idx(device_idx) {
    this->actual_size = m ? n / m : 0;
}

void BaseHiddenStates::set_input_x(const std::vector<float> &mu_x, const std::vector<float> &var_x,
                                   size_t block_size) {
    const size_t n = mu_x.size();
    this->actual_size = n / block_size;
    this->block_size = block_size;
    std::copy(mu_x.begin(), mu_x.end(), this->mu_a.begin());
    std::fill(this->jcb.begin(), this->jcb.begin() + n, 1.0f);
    if (var_x.size() == n)
        std::copy(var_x.begin(), var_x.end(), this->var_a.begin());
    else
        std::fill(this->var_a.begin(), this->var_a.begin() + n, 0.0f);
}

void BaseHiddenStates::set_size(size_t new_size, size_t new_block_size) {
    if (new_size > this->size) {
        this->size = new_size;
        this->mu_a.resize(new_size, 0.0f);
        this->var_a.resize(new_size, 0.0f);
        this->jcb.resize(new_size, 1.0f);
    }
    this->block_size = new_block_size;
    this->actual_size = new_size / new_block_size;
}

void BaseHiddenStates::swap(BaseHiddenStates &other) {
    std::swap(mu_a, other.mu_a);
    std::swap(var_a, other.var_a);
    std::swap(jcb, other.jcb);
    std::swap(size, other.size);
    std::swap(block_size, other.block_size);
    std::swap(actual_size, other.actual_size);
    std::swap(width, other.width);
    std::swap(height, other.height);
    std::swap(depth, other.depth);
}

void BaseHiddenStates::copy_from(const BaseHiddenStates &source, int num_data) {
    if (num_data == -1) num_data = (int)std::min(source.size, this->size);
    std::copy_n(source.mu_a.begin(), num_data, this->mu_a.begin());
    std::copy_n(source.var_a.begin(), num_data, this->var_a.begin());
    std::copy_n(source.jcb.begin(), num_data, this->jcb.begin());
    this->block_size = source.block_size;
    this->actual_size = source.actual_size;
    this->width = source.width;
    this->height = source.height;
    this->depth = source.depth;
}

// ---- BaseDeltaStates (src/data_struct.cpp:100-160) ------------------------------
BaseDeltaStates::BaseDeltaStates(size_t n, size_t m, int device_idx)
    : delta_mu(n, 0.0f), delta_var(n, 0.0f), size(n), block_size(m), device_idx(device_idx) {
    this->actual_size = m ? n / m : 0;
}

void BaseDeltaStates::reset_zeros() {
    std::fill(delta_mu.begin(), delta_mu.end(), 0.0f);
    std::fill(delta_var.begin(), delta_var.end(), 0.0f);
}

void BaseDeltaStates::copy_from(const BaseDeltaStates &source, int num_data) {
    if (num_data == -1) num_data = (int)std::min(source.size, this->size);
    std::copy_n(source.delta_mu.begin(), num_data, this->delta_mu.begin());
    std::copy_n(source.delta_var.begin(), num_data, this->delta_var.begin());
    this->block_size = source.block_size;
}

void BaseDeltaStates::set_size(size_t new_size, size_t new_block_size) {
    if (new_size > this->size) {
        this->size = new_size;
        this->reset_zeros();
        this->delta_mu.resize(new_size, 0.0f);
        this->delta_var.resize(new_size, 0.0f);
    }
    this->block_size = new_block_size;
    this->actual_size = new_size / new_block_size;
}

void BaseDeltaStates::swap(BaseDeltaStates &other) {
    std::swap(delta_mu, other.delta_mu);
    std::swap(delta_var, other.delta_var);
    std::swap(size, other.size);
    std::swap(block_size, other.block_size);
    std::swap(actual_size, other.actual_size);
}

// ---- BaseTempStates / BaseBackwardStates / BaseObservation ----------------------
BaseTempStates::BaseTempStates(size_t n, size_t m, int device_idx)
    : tmp_1(n, 0.0f), tmp_2(n, 0.0f), size(n), block_size(m), device_idx(device_idx) {
    this->actual_size = m ? n / m : 0;
}

void BaseTempStates::set_size(size_t new_size, size_t new_block_size) {
    if (new_size > this->size) {
        this->size = new_size;
        this->tmp_1.resize(new_size, 0.0f);
        this->tmp_2.resize(new_size, 0.0f);
    }
    this->block_size = new_block_size;
    this->actual_size = new_size / new_block_size;
}

BaseBackwardStates::BaseBackwardStates(int num) : mu_a(num, 0.0f), jcb(num, 1.0f), size(num) {}

void BaseBackwardStates::set_size(size_t new_size) {
    if (new_size > this->size) {
        this->size = new_size;
        this->mu_a.resize(new_size, 0.0f);
        this->jcb.resize(new_size, 1.0f);
    }
}

void BaseObservation::set_obs(std::vector<float> &mu, std::vector<float> &var) {
    this->mu_obs = mu;
    this->var_obs = var;
}
void BaseObservation::set_selected_idx(std::vector<int> &idx) { this->selected_idx = idx; }

// ---- HiddenStateHip (reference: src/data_struct_cuda.cu:9-200) ------------------
HiddenStateHip::HiddenStateHip(size_t n, size_t m, int device_idx)
    : BaseHiddenStates(n, m, device_idx) {
    this->allocate_memory();
}
HiddenStateHip::~HiddenStateHip() { this->deallocate_memory(); }

void HiddenStateHip::allocate_memory() {
    this->deallocate_memory();
    d_mu_a = dev_alloc(size, device_idx);
    d_var_a = dev_alloc(size, device_idx);
    d_jcb = dev_alloc(size, device_idx);
    this->to_device();
}
void HiddenStateHip::deallocate_memory() {
    dev_free(d_mu_a);
    dev_free(d_var_a);
    dev_free(d_jcb);
}
void HiddenStateHip::to_device() { this->chunks_to_device(this->size); }
void HiddenStateHip::chunks_to_device(size_t n) {
    h2d(d_mu_a, mu_a.data(), n);
    h2d(d_var_a, var_a.data(), n);
    h2d(d_jcb, jcb.data(), n);
    jcb_ones = false;
}
void HiddenStateHip::to_host() { this->to_host(this->size); }
// grow-only pinned buffer per device that tagi_download_outputs writes into
static float *download_buffer(size_t floats, int device_idx) {
    static float *buf[16] = {};
    static size_t cap[16] = {};
    if (device_idx < 0 || device_idx >= 16) LOG(LogLevel::ERROR, "Invalid device index");
    if (cap[device_idx] < floats) {
        if (buf[device_idx] != nullptr) HIP_OK(hipHostFree(buf[device_idx]));
        cap[device_idx] = std::max(floats, (size_t)1 << 14);
        HIP_OK(hipHostMalloc(reinterpret_cast<void **>(&buf[device_idx]),
                             cap[device_idx] * sizeof(float), hipHostMallocDefault));
        std::memset(buf[device_idx], 0, 64);      // the completion flag starts cleared
    }
    return buf[device_idx];
}

void HiddenStateHip::to_host(size_t n) {
    n = std::min(n, this->size);
    if (n > 0 && n * sizeof(float) <= kKernelUploadMaxBytes) {
        // small results: one kernel writes both arrays into pinned memory, one wait
        HIP_OK(hipSetDevice(device_idx));
        // [0]: the flag the kernel sets after the data (64 bytes to itself), then the data
        float *buf = download_buffer(2 * n + 16, device_idx);
        unsigned *flag = reinterpret_cast<unsigned *>(buf);
        float *host = buf + 16;
        static unsigned sequence = 0;
        const unsigned expect = ++sequence == 0 ? ++sequence : sequence;   // never the initial 0
        // (one workgroup copies when a flag is asked for: only for the sizes of outputs)
        const bool poll = n <= 16384;
        TAGI_OK_OR_THROW(tagi_download_outputs(d_mu_a, d_var_a, n, host, host + n,
                                               poll ? flag : nullptr, expect, host_stream()));
        if (!poll) HIP_OK(hipStreamSynchronize(host_stream()));
        // Poll the flag: the data is a few hundred bytes behind kernels that take
        // microseconds, and waking up through the runtime's stream wait costs more than
        // the wait itself. Bounded: after 2 ms the ordinary wait takes over (which also
        // reports a failed launch).
        const auto t0 = std::chrono::steady_clock::now();
        unsigned spins = 0;
        while (poll && *static_cast<volatile unsigned *>(flag) != expect) {
            if ((++spins & 1023u) == 0 &&
                std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(2)) {
                HIP_OK(hipStreamSynchronize(host_stream()));
                break;
            }
        }
        std::atomic_thread_fence(std::memory_order_acquire);
        std::memcpy(mu_a.data(), host, n * sizeof(float));
        std::memcpy(var_a.data(), host + n, n * sizeof(float));
    } else {
        d2h(mu_a.data(), d_mu_a, n);
        d2h(var_a.data(), d_var_a, n);
    }
    if (jcb_ones)
        std::fill(jcb.begin(), jcb.begin() + n, 1.0f);
    else
        d2h(jcb.data(), d_jcb, n);
}
void HiddenStateHip::set_input_x(const std::vector<float> &mu_x, const std::vector<float> &var_x,
                                 size_t block_size) {
    if (mu_x.size() > this->size)
        LOG(LogLevel::ERROR, "Input of " + std::to_string(mu_x.size()) +
                                 " values exceeds the state buffer of " + std::to_string(size));
    this->set_input_raw(mu_x.data(), var_x.size() == mu_x.size() ? var_x.data() : nullptr,
                        mu_x.size(), block_size);
}
// The reference fills host vectors first and then copies all three of them
// (src/data_struct_cuda.cu:58-80): three host passes and three transfers per
// batch. Here only what the caller supplied crosses the bus.
void HiddenStateHip::set_input_raw(const float *mu_x, const float *var_x, size_t n,
                                   size_t new_block_size) {
    if (n > this->size)
        LOG(LogLevel::ERROR, "Input of " + std::to_string(n) +
                                 " values exceeds the state buffer of " + std::to_string(size));
    if (n == 0 || new_block_size == 0) LOG(LogLevel::ERROR, "Empty input");
    this->actual_size = n / new_block_size;
    this->block_size = new_block_size;
    HIP_OK(hipSetDevice(device_idx));
    StagingRing &ring = staging_ring(device_idx);
    if (n * sizeof(float) <= kKernelUploadMaxBytes) {
        // small batches: one kernel reads the pinned copy over the bus and fills both arrays
        // (a copy-engine transfer costs a short dependent chain more than it carries)
        const void *parts[2] = {mu_x, var_x};
        const size_t sizes[2] = {n * sizeof(float), var_x != nullptr ? n * sizeof(float) : 0};
        const float *host = static_cast<const float *>(ring.stage(parts, sizes, 2));
        TAGI_OK_OR_THROW(tagi_upload_input(host, var_x != nullptr ? host + n : nullptr, n, d_mu_a,
                                           d_var_a, host_stream()));
        ring.staged_work_queued();
    } else {
        ring.upload(d_mu_a, mu_x, n * sizeof(float));
        if (var_x != nullptr)
            ring.upload(d_var_a, var_x, n * sizeof(float));
        else
            HIP_OK(hipMemsetAsync(d_var_a, 0, n * sizeof(float), host_stream()));
    }
    jcb_ones = true;  // the input's Jacobian is one: marked, not written
}
void HiddenStateHip::set_size(size_t new_size, size_t new_block_size) {
    if (new_size > this->size) {
        BaseHiddenStates::set_size(new_size, new_block_size);
        HIP_OK(hipDeviceSynchronize());
        this->allocate_memory();
    } else {
        this->block_size = new_block_size;
        this->actual_size = new_size / new_block_size;
    }
}
void HiddenStateHip::swap(BaseHiddenStates &other) {
    auto *o = dynamic_cast<HiddenStateHip *>(&other);
    if (o == nullptr) LOG(LogLevel::ERROR, "Swap needs two device hidden states");
    BaseHiddenStates::swap(other);
    std::swap(d_mu_a, o->d_mu_a);
    std::swap(d_var_a, o->d_var_a);
    std::swap(d_jcb, o->d_jcb);
    std::swap(jcb_ones, o->jcb_ones);
    // `transient` stays: it says what role the OBJECT plays for its owner (a ping-pong
    // buffer whose contents are dead once read), not what the arrays hold. A caller's
    // input state that trades arrays with such a buffer remains the caller's.
}
void HiddenStateHip::copy_from(const BaseHiddenStates &source, int num_data) {
    auto *s = dynamic_cast<const HiddenStateHip *>(&source);
    if (s == nullptr) LOG(LogLevel::ERROR, "Copy needs a device hidden state as source");
    if (num_data == -1) num_data = (int)std::min(source.size, this->size);
    d2d(d_mu_a, s->d_mu_a, num_data);
    d2d(d_var_a, s->d_var_a, num_data);
    if (!s->jcb_ones) d2d(d_jcb, s->d_jcb, num_data);
    this->jcb_ones = s->jcb_ones;
    this->block_size = source.block_size;
    this->actual_size = source.actual_size;
    this->width = source.width;
    this->height = source.height;
    this->depth = source.depth;
}

// ---- DeltaStateHip (src/data_struct_cuda.cu:205-330) -----------------------------
DeltaStateHip::DeltaStateHip(size_t n, size_t m, int device_idx) : BaseDeltaStates(n, m, device_idx) {
    this->allocate_memory();
}
DeltaStateHip::~DeltaStateHip() { this->deallocate_memory(); }
// The two arrays are one allocation, so that reset_zeros is one launch; swap() exchanges
// both pointers, which keeps pairs together. The variance starts at the next multiple of
// 64 floats after the mean, so that both arrays are 256-byte aligned for any size (the
// kernels choose their 16-byte paths by pointer alignment).
static size_t delta_var_offset(size_t size) { return (size + 63) / 64 * 64; }
void DeltaStateHip::allocate_memory() {
    this->deallocate_memory();
    d_delta_mu = dev_alloc(delta_var_offset(size) + size, device_idx);
    d_delta_var = d_delta_mu != nullptr ? d_delta_mu + delta_var_offset(size) : nullptr;
    this->to_device();
}
void DeltaStateHip::deallocate_memory() {
    dev_free(d_delta_mu);
    d_delta_var = nullptr;
}
void DeltaStateHip::to_device() {
    h2d(d_delta_mu, delta_mu.data(), size);
    h2d(d_delta_var, delta_var.data(), size);
}
void DeltaStateHip::to_host() {
    d2h(delta_mu.data(), d_delta_mu, size);
    d2h(delta_var.data(), d_delta_var, size);
}
void DeltaStateHip::reset_zeros() {
    if (size == 0) return;
    HIP_OK(hipMemsetAsync(d_delta_mu, 0, (delta_var_offset(size) + size) * sizeof(float), host_stream()));
}
void DeltaStateHip::copy_from(const BaseDeltaStates &source, int num_data) {
    auto *s = dynamic_cast<const DeltaStateHip *>(&source);
    if (s == nullptr) LOG(LogLevel::ERROR, "Copy needs a device delta state as source");
    if (num_data == -1) num_data = (int)std::min(source.size, this->size);
    d2d(d_delta_mu, s->d_delta_mu, num_data);
    d2d(d_delta_var, s->d_delta_var, num_data);
    this->block_size = source.block_size;
}
void DeltaStateHip::set_size(size_t new_size, size_t new_block_size) {
    if (new_size > this->size) {
        this->size = new_size;
        this->delta_mu.assign(new_size, 0.0f);
        this->delta_var.assign(new_size, 0.0f);
        HIP_OK(hipDeviceSynchronize());
        this->allocate_memory();
    }
    this->block_size = new_block_size;
    this->actual_size = new_size / new_block_size;
}
void DeltaStateHip::swap(BaseDeltaStates &other) {
    auto *o = dynamic_cast<DeltaStateHip *>(&other);
    if (o == nullptr) LOG(LogLevel::ERROR, "Swap needs two device delta states");
    BaseDeltaStates::swap(other);
    std::swap(d_delta_mu, o->d_delta_mu);
    std::swap(d_delta_var, o->d_delta_var);
}

// ---- TempStateHip / BackwardStateHip / ObservationHip ----------------------------
TempStateHip::TempStateHip(size_t n, size_t m, int device_idx) : BaseTempStates(n, m, device_idx) {
    this->allocate_memory();
}
TempStateHip::~TempStateHip() { this->deallocate_memory(); }
void TempStateHip::allocate_memory() {
    this->deallocate_memory();
    d_tmp_1 = dev_alloc(size, device_idx);
    d_tmp_2 = dev_alloc(size, device_idx);
}
void TempStateHip::deallocate_memory() {
    dev_free(d_tmp_1);
    dev_free(d_tmp_2);
}
void TempStateHip::set_size(size_t new_size, size_t new_block_size) {
    if (new_size > this->size) {
        BaseTempStates::set_size(new_size, new_block_size);
        HIP_OK(hipDeviceSynchronize());
        this->allocate_memory();
    } else {
        this->block_size = new_block_size;
        this->actual_size = new_size / new_block_size;
    }
}

BackwardStateHip::~BackwardStateHip() { this->deallocate_memory(); }
void BackwardStateHip::allocate_memory() {
    this->deallocate_memory();
    d_mu_a = dev_alloc(size, device_idx);
    d_jcb = dev_alloc(size, device_idx);
}
void BackwardStateHip::deallocate_memory() {
    if (borrowed) {
        d_mu_a = d_jcb = nullptr;
        borrowed = false;
        size = 0;
        return;
    }
    dev_free(d_mu_a);
    dev_free(d_jcb);
}
void BackwardStateHip::borrow(float *mu, float *jac, bool ones, size_t n) {
    if (!borrowed) {
        HIP_OK(hipDeviceSynchronize());
        this->deallocate_memory();
    }
    borrowed = true;
    d_mu_a = mu;
    d_jcb = ones ? nullptr : jac;
    jcb_ones = ones;
    size = n;
}
void BackwardStateHip::to_host() {
    mu_a.resize(size);
    jcb.resize(size);
    d2h(mu_a.data(), d_mu_a, size);
    if (jcb_ones)
        std::fill(jcb.begin(), jcb.end(), 1.0f);
    else
        d2h(jcb.data(), d_jcb, size);
}
// Exactly `new_size` elements (the arrays are traded with a buffer of that size). The
// Jacobian array is only allocated once a Jacobian that is not all ones has to be kept.
void BackwardStateHip::resize_exact(size_t new_size, bool need_jcb) {
    if (borrowed) this->deallocate_memory();
    if (new_size != this->size || d_mu_a == nullptr) {
        this->size = new_size;
        HIP_OK(hipDeviceSynchronize());
        this->deallocate_memory();
        d_mu_a = dev_alloc(size, device_idx);
    }
    if (need_jcb && d_jcb == nullptr) d_jcb = dev_alloc(size, device_idx);
}
void BackwardStateHip::set_size(size_t new_size) {
    if (borrowed) this->deallocate_memory();
    if (new_size > this->size) {
        this->size = new_size;
        HIP_OK(hipDeviceSynchronize());
        this->allocate_memory();
    }
}

// Observations, their variances and the selected indices live in one device block,
// back to back in that order, so that a batch's observations are one transfer.
ObservationHip::~ObservationHip() { dev_free(d_mu_obs); }
void ObservationHip::reserve(size_t n, size_t ni) {
    const size_t words = 2 * n + ni;  // floats and ints are both four bytes
    if (words > cap_obs) {
        HIP_OK(hipDeviceSynchronize());
        dev_free(d_mu_obs);
        d_mu_obs = dev_alloc(words, device_idx);
        cap_obs = words;
    }
    cap_idx = ni;
    d_var_obs = d_mu_obs + n;
    d_selected_idx = reinterpret_cast<int *>(d_mu_obs + 2 * n);
}
void ObservationHip::upload(const float *mu, const float *var, size_t n, const int *idx,
                            size_t ni) {
    HIP_OK(hipSetDevice(device_idx));
    this->reserve(n, ni);
    StagingRing &ring = staging_ring(device_idx);
    if (var != nullptr) {
        const void *parts[3] = {mu, var, idx};
        const size_t sizes[3] = {n * sizeof(float), n * sizeof(float), ni * sizeof(int)};
        ring.upload_parts(d_mu_obs, parts, sizes, 3);
    } else {
        ring.upload(d_mu_obs, mu, n * sizeof(float));
        if (ni) ring.upload(d_selected_idx, idx, ni * sizeof(int));
    }
}
void ObservationHip::stage(const float *mu, const float *var, size_t n, const int *idx,
                           const float **mu_at, const float **var_at, const int **idx_at) {
    HIP_OK(hipSetDevice(device_idx));
    const void *parts[3] = {mu, var, idx};
    const size_t sizes[3] = {n * sizeof(float), n * sizeof(float), n * sizeof(int)};
    char *host = static_cast<char *>(staging_ring(device_idx).stage(parts, sizes, 3));
    *mu_at = reinterpret_cast<const float *>(host);
    *var_at = reinterpret_cast<const float *>(host + sizes[0]);
    *idx_at = reinterpret_cast<const int *>(host + sizes[0] + sizes[1]);
}
void ObservationHip::staged_work_queued() { staging_ring(device_idx).staged_work_queued(); }
void ObservationHip::to_device() {
    this->upload(mu_obs.data(), var_obs.data(), mu_obs.size(), selected_idx.data(),
                 selected_idx.size());
}

}  // namespace tagi_host

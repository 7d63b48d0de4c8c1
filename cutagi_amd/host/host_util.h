// Small helpers shared by the host classes: device allocation, host <-> device
// copies of float vectors, raw float I/O, and checked casts of the state
// containers to their device forms.
#pragma once
#include <hip/hip_runtime_api.h>

#include <fstream>
#include <vector>

#include "logger.h"
#include "states.h"

namespace tagi_host {

// The stream every host class queues its device work on: the null stream, or - once a
// model has switched graph replay on - one ordinary (blocking) stream of its own,
// because work on the null stream cannot be captured into a HIP graph. A blocking
// stream still orders with the synchronous copies that go through the null stream.
hipStream_t host_stream();
void set_host_stream(hipStream_t stream);

template <typename T>
T *dev_alloc_t(size_t n, int device_idx) {
    T *p = nullptr;
    if (n == 0) return p;
    HIP_OK(hipSetDevice(device_idx));
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&p), n * sizeof(T)));
    return p;
}
template <typename T>
void dev_free_t(T *&p) {
    if (p != nullptr) (void)hipFree(p);
    p = nullptr;
}
inline void h2d(float *dst, const std::vector<float> &src) {
    if (!src.empty())
        HIP_OK(hipMemcpy(dst, src.data(), src.size() * sizeof(float), hipMemcpyHostToDevice));
}
inline void d2h(std::vector<float> &dst, const float *src, size_t n) {
    dst.resize(n);
    if (n) HIP_OK(hipMemcpy(dst.data(), src, n * sizeof(float), hipMemcpyDeviceToHost));
}
inline void write_floats(std::ofstream &f, const std::vector<float> &v) {
    f.write(reinterpret_cast<const char *>(v.data()), v.size() * sizeof(float));
}
inline void read_floats(std::ifstream &f, std::vector<float> &v) {
    f.read(reinterpret_cast<char *>(v.data()), v.size() * sizeof(float));
}
template <typename T>
T *as(BaseHiddenStates &s) {
    auto *p = dynamic_cast<T *>(&s);
    if (p == nullptr) LOG(LogLevel::ERROR, "Device layer received host state buffers");
    return p;
}
template <typename T>
T *as(BaseDeltaStates &s) {
    auto *p = dynamic_cast<T *>(&s);
    if (p == nullptr) LOG(LogLevel::ERROR, "Device layer received host delta buffers");
    return p;
}

}  // namespace tagi_host

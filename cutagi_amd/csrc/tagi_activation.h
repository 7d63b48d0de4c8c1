// Activations as device functions, shared by the stand-alone activation kernels and
// by the forward epilogues of the Linear / Conv2d kernels that apply them to their
// sums before anything is stored (reference: src/activation.cpp:7-29 ReLU,
// 152-178 MixtureReLU; device forms src/activation_cuda.cu:130-150, 726-760).
#pragma once
#include <hip/hip_runtime.h>

namespace tagi {

enum Activation { ACT_NONE = 0, ACT_RELU = 1, ACT_MIXTURE_RELU = 2 };

// mu_a = max(mu_z, 0); where that is zero, var_a = jcb = 0, else var_a = var_z, jcb = 1
__device__ __forceinline__ void relu_moments(float m, float v, float &mu_a, float &var_a,
                                             float &jcb) {
    mu_a = fmaxf(m, 0.f);
    jcb = (mu_a == 0.f) ? 0.f : 1.f;
    var_a = (mu_a == 0.f) ? 0.f : v;
}

// Moments of max(z, 0) for z ~ N(m, v), both floored at 1e-6; jcb = P(z > 0).
__device__ __forceinline__ void mixture_relu_moments(float m, float v, float &mu_a, float &var_a,
                                                     float &jcb) {
    constexpr float INV_SQRT_2PI = 1.0f / 2.5066282746310002f;
    const float sd = sqrtf(v);
    const float alpha = m / sd;
    const float pdf = INV_SQRT_2PI * expf(-0.5f * alpha * alpha);
    const float cdf = 0.5f * erfcf(-alpha * 0.7071067811865475f);
    const float t = m * cdf + sd * pdf;
    mu_a = fmaxf(0.000001f, t);
    var_a = fmaxf(0.000001f, -t * t + 2.f * t * m - m * sd * pdf + (v - m * m) * cdf);
    jcb = cdf;
}

// Stores the layer output (act == ACT_NONE: the two sums; otherwise the activation's
// three moments, out2 = Jacobian) at element `at`.
__device__ __forceinline__ void store_activated(int act, float a0, float a1, size_t at,
                                                float *__restrict__ out0,
                                                float *__restrict__ out1,
                                                float *__restrict__ out2) {
    if (act == ACT_NONE) {
        out0[at] = a0;
        out1[at] = a1;
        return;
    }
    float mu, var, jcb;
    if (act == ACT_RELU)
        relu_moments(a0, a1, mu, var, jcb);
    else
        mixture_relu_moments(a0, a1, mu, var, jcb);
    out0[at] = mu;
    out1[at] = var;
    out2[at] = jcb;
}

}  // namespace tagi

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

// Density and distribution function of the standard normal at alpha, from ONE exponential:
// Phi(-t) = phi(t) M(t) for t >= 0 with the Mills ratio M(t) = u Q(u), u = 1 / (1 + 0.35 t),
// Q a polynomial of degree 10 fitted to relative error 1.4e-8 over t in [0, inf) (1.6e-7
// evaluated in fp32). exp(x) = 2^(x log2 e) with the rounding error of the product carried
// as a first-order correction. About 35 instructions instead of the ~100 of expf + erfcf:
// the activation runs in the epilogue of the conv kernels, where it is pure VALU time
// (8.4 M outputs of a 32 x 32 layer: 19 us).
__device__ __forceinline__ void normal_pdf_cdf(float alpha, float &pdf, float &cdf) {
    constexpr float INV_SQRT_2PI = 1.0f / 2.5066282746310002f;
    constexpr float LOG2E_HI = 1.44269504f, LOG2E_LO = 1.925963033500e-8f, LN2 = 0.69314718f;
    const float t = fabsf(alpha);
    const float x = fmaxf(-0.5f * t * t, -120.f);   // e^-120 is zero in fp32; keeps inf out of the fma
    const float hi = x * LOG2E_HI;
    const float lo = fmaf(x, LOG2E_HI, -hi) + x * LOG2E_LO;
    float e = __builtin_amdgcn_exp2f(hi);
    e = fmaf(e, lo * LN2, e);
    pdf = e * INV_SQRT_2PI;
    const float u = __builtin_amdgcn_rcpf(fmaf(0.35f, t, 1.f));
    float q = 4.850552919e-02f;
    q = fmaf(q, u, -2.722857298e-01f);
    q = fmaf(q, u, 5.921097785e-01f);
    q = fmaf(q, u, -5.671834525e-01f);
    q = fmaf(q, u, 1.749514740e-01f);
    q = fmaf(q, u, -7.139860880e-02f);
    q = fmaf(q, u, 1.213802339e-01f);
    q = fmaf(q, u, 2.200412660e-01f);
    q = fmaf(q, u, 3.071950457e-01f);
    q = fmaf(q, u, 3.499985812e-01f);
    q = fmaf(q, u, 3.500000047e-01f);
    const float tail = pdf * (u * q);                // Phi(-t)
    cdf = alpha < 0.f ? tail : 1.f - tail;
}

// Moments of max(z, 0) for z ~ N(m, v), both floored at 1e-6; jcb = P(z > 0).
__device__ __forceinline__ void mixture_relu_moments(float m, float v, float &mu_a, float &var_a,
                                                     float &jcb) {
    const float sd = sqrtf(v);
    const float alpha = m / sd;
    float pdf, cdf;
    normal_pdf_cdf(alpha, pdf, cdf);
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

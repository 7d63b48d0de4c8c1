// Staging of a workgroup's slice of the per-sample vectors (activations or
// innovations) into LDS for the skinny-batch Linear kernels.
//
// The slice is [slots][per] float4-wise out of two global arrays laid out
// [B][ld]; slots beyond B and elements beyond `valid` are staged as zeros. A
// thread's loads of four rounds are issued before the first of them is used: a
// loop that loads, waits and writes per round pays one memory latency per round
// (the slice is mostly not in the L2, which the weight stream keeps flushing), and
// a workgroup cannot start on its weights before the slice is there.
#pragma once
#include <hip/hip_runtime.h>

namespace tagi {

// store(b, x, m, v): writes the float4 pair of slot b, element x (a multiple of 4)
template <int THREADS, typename Store>
__device__ __forceinline__ void stage_slice_pairs(const float *__restrict__ a0,
                                                  const float *__restrict__ a1, int slots, int B,
                                                  int ld, int begin, int valid, int per, int tid,
                                                  Store store) {
    constexpr int ROUNDS = 4;
    const int q = per / 4, total = slots * q;
    const int last = ld - 4;  // ld % 4 == 0 on every path that stages 16 bytes at a time
    for (int e0 = tid; e0 < total; e0 += ROUNDS * THREADS) {
        float4 m[ROUNDS], v[ROUNDS];
        int sb[ROUNDS], sx[ROUNDS];
#pragma unroll
        for (int u = 0; u < ROUNDS; u++) {
            const int e = min(e0 + u * THREADS, total - 1);
            sb[u] = e / q;
            sx[u] = (e - sb[u] * q) * 4;
            // never predicated: out-of-range slots read the last sample, out-of-range
            // elements the last float4 of the row; both are replaced by zeros below
            const size_t at = (size_t)min(sb[u], B - 1) * ld + min(begin + sx[u], last);
            m[u] = *reinterpret_cast<const float4 *>(a0 + at);
            v[u] = *reinterpret_cast<const float4 *>(a1 + at);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < ROUNDS; u++) {
            const bool live = sb[u] < B && sx[u] < valid;
            float4 pm, pv;
            pm.x = live ? m[u].x : 0.f; pm.y = live ? m[u].y : 0.f;
            pm.z = live ? m[u].z : 0.f; pm.w = live ? m[u].w : 0.f;
            pv.x = live ? v[u].x : 0.f; pv.y = live ? v[u].y : 0.f;
            pv.z = live ? v[u].z : 0.f; pv.w = live ? v[u].w : 0.f;
            // (a round beyond the slice re-writes the last element with the same values)
            store(sb[u], sx[u], pm, pv);
        }
    }
}

}  // namespace tagi

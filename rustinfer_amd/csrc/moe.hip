// A feed-forward of many small experts of which every token uses a few.
//
//   moe_route           32-bit router logits [T][E] -> weights [T][E]: the softmax probability for the
//                       `top` experts with the largest probabilities (ties: the lower index), 0 for
//                       the others; optionally divided by the chosen ones' sum.
//   moe_swiglu_weighted act[t][e F + i] = weight[t][e] * silu(gu[t][e 2F + i]) * gu[t][e 2F + F + i]:
//                       the experts' activations side by side, each scaled by its token's weight, so
//                       that ONE product with the experts' down matrices side by side is the weighted
//                       sum of the chosen experts' outputs (an expert that was not chosen adds zeros).
#include "common.h"
#include <math.h>

namespace {

constexpr int MOE_EPL = 8;       // experts a lane: up to 512 experts

__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits, int l_stride, float* __restrict__ weights,
                                                       int T, int E, int top, int renorm) {
    const int lane = threadIdx.x & 63, t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= T) return;
    const float* z = logits + (size_t)t * l_stride;
    float s[MOE_EPL];
    float m = -INFINITY;
#pragma unroll
    for (int j = 0; j < MOE_EPL; ++j) {
        const int e = lane + 64 * j;
        s[j] = e < E ? z[e] : -INFINITY;
        m = fmaxf(m, s[j]);
    }
    m = wave_max(m);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < MOE_EPL; ++j) {
        s[j] = (lane + 64 * j) < E ? expf(s[j] - m) : -1.f;     // probabilities are >= 0: -1 marks "not there"
        if (s[j] > 0.f) sum += s[j];
    }
    sum = wave_sum(sum);
    const float inv = 1.f / sum;
    unsigned chosen = 0;             // bit j: this lane's expert lane + 64 j is chosen
    float kept = 0.f;
    for (int n = 0; n < top; ++n) {
        float best = -1.f;
        int best_e = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < MOE_EPL; ++j) {
            const int e = lane + 64 * j;
            if (!(chosen >> j & 1u) && e < E && (s[j] > best || (s[j] == best && e < best_e))) { best = s[j]; best_e = e; }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, 64);
            const int oe = __shfl_xor(best_e, o, 64);
            if (ob > best || (ob == best && oe < best_e)) { best = ob; best_e = oe; }
        }
        if (best_e < E && (best_e & 63) == lane) chosen |= 1u << (best_e >> 6);
        kept += best * inv;
    }
    const float f = renorm ? inv / kept : inv;
    float* wr = weights + (size_t)t * E;
#pragma unroll
    for (int j = 0; j < MOE_EPL; ++j) {
        const int e = lane + 64 * j;
        if (e < E) wr[e] = (chosen >> j & 1u) ? s[j] * f : 0.f;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_swiglu_weighted_kernel(const T* __restrict__ gu, int gu_stride, const float* __restrict__ weights,
                                                                 T* __restrict__ act, int act_stride, int E, int F) {
    const int t = blockIdx.y;
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= E * F) return;
    const int e = idx / F, i = idx - e * F;
    const float wgt = weights[(size_t)t * E + e];
    float y = 0.f;
    if (wgt != 0.f) {
        const T* row = gu + (size_t)t * gu_stride + (size_t)e * 2 * F;
        const float g = ld_f32(row + i), u = ld_f32(row + F + i);
        y = wgt * (g / (1.f + expf(-g))) * u;
    }
    st_f32(act + (size_t)t * act_stride + idx, y);
}

}  // namespace

extern "C" int ri_moe_route(const float* logits, int l_stride, float* weights, int T, int E, int top, int renorm, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && E > 0 && top > 0 && top <= E && l_stride >= E, "ri_moe_route: bad sizes T=%d E=%d top=%d", T, E, top);
    RI_REQUIRE(E <= 64 * MOE_EPL, "ri_moe_route: %d experts, the kernel takes up to %d", E, 64 * MOE_EPL);
    if (T == 0) return 0;
    RI_REQUIRE(logits && weights, "ri_moe_route: null pointer");
    moe_route_kernel<<<(T + 3) / 4, 256, 0, stream>>>(logits, l_stride, weights, T, E, top, renorm);
    RI_LAUNCHED("ri_moe_route");
    return 0;
}

extern "C" int ri_moe_swiglu_weighted(const void* gu, int gu_stride, const float* weights, void* act, int act_stride, int dtype,
                                      int T, int E, int F, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && E > 0 && F > 0 && gu_stride >= 2 * E * F && act_stride >= E * F, "ri_moe_swiglu_weighted: bad sizes");
    if (T == 0) return 0;
    RI_REQUIRE(gu && weights && act, "ri_moe_swiglu_weighted: null pointer");
    RI_REQUIRE(T <= 65535, "ri_moe_swiglu_weighted: too many rows for the grid");
    const dim3 grid((E * F + 255) / 256, T);
    if (dtype == RI_F32) moe_swiglu_weighted_kernel<float><<<grid, 256, 0, stream>>>((const float*)gu, gu_stride, weights, (float*)act, act_stride, E, F);
    else if (dtype == RI_BF16) moe_swiglu_weighted_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)gu, gu_stride, weights, (bf16_t*)act, act_stride, E, F);
    else return ri_fail("ri_moe_swiglu_weighted: unknown dtype %d", dtype);
    RI_LAUNCHED("ri_moe_swiglu_weighted");
    return 0;
}

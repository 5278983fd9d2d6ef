// A feed-forward of many small experts of which every token uses a few.
//
//   moe_route           32-bit router logits [T][E] -> weights [T][E]: the softmax probability for the
//                       `top` experts with the largest probabilities (ties: the lower index), 0 for
//                       the others; optionally divided by the chosen ones' sum.
//   moe_swiglu_weighted act[t][e F + i] = weight[t][e] * silu(gu[t][e 2F + i]) * gu[t][e 2F + F + i]:
//                       the experts' activations side by side, each scaled by its token's weight, so
//                       that ONE product with the experts' down matrices side by side is the weighted
//                       sum of the chosen experts' outputs (an expert that was not chosen adds zeros).
//                       A router may also score with a sigmoid of each logit instead of the softmax over all
//                       (the chosen scores divided by their sum + eps if renormalised), and multiply the
//                       weights by a constant.  Fs more columns after the experts' are a shared expert that
//                       every token uses with weight 1: act[t][E F + i] = silu(gu[t][2 E F + i]) * gu[t][2 E F + Fs + i];
//                       columns beyond E F + Fs up to the width given are zeros.
//   moe_swiglu_routed   the two in one launch: every block makes its token's weights from the logits
//                       itself (what the engine runs; the two above are its halves, kept for callers
//                       that want the weights).
#include "common.h"
#include <math.h>

namespace {

constexpr int MOE_EPL = 8;       // experts a lane: up to 512 experts

// One wave: the weights of a token's experts from its logits z [E] into wr [E] (global or LDS).
struct RouteHow {
    int sigmoid;       // scores are sigmoid(z) of each logit, else softmax(z) over all experts
    int renorm;        // the chosen scores are divided by their sum + eps
    float eps, scale;  // scale: a factor on every weight
};

__device__ __forceinline__ void route_token(const float* __restrict__ z, float* wr, int E, int top, RouteHow how, int lane) {
    const int renorm = how.renorm;
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
        if (how.sigmoid) s[j] = (lane + 64 * j) < E ? 1.f / (1.f + expf(-s[j])) : -1.f;
        else s[j] = (lane + 64 * j) < E ? expf(s[j] - m) : -1.f;     // scores are >= 0: -1 marks "not there"
        if (s[j] > 0.f) sum += s[j];
    }
    sum = wave_sum(sum);
    const float inv = how.sigmoid ? 1.f : 1.f / sum;
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
    const float f = (renorm ? inv / (kept + how.eps) : inv) * how.scale;
#pragma unroll
    for (int j = 0; j < MOE_EPL; ++j) {
        const int e = lane + 64 * j;
        if (e < E) wr[e] = (chosen >> j & 1u) ? s[j] * f : 0.f;
    }
}

__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ logits, int l_stride, float* __restrict__ weights,
                                                       int T, int E, int top, RouteHow how) {
    const int lane = threadIdx.x & 63, t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= T) return;
    route_token(logits + (size_t)t * l_stride, weights + (size_t)t * E, E, top, how, lane);
}

// column i of the shared expert's activation from its gate and up columns [gate Fs | up Fs]; 0 beyond Fs
template <typename T>
__device__ __forceinline__ float shared_column(const T* __restrict__ row, int i, int Fs) {
    if (i >= Fs) return 0.f;
    const float g = ld_f32(row + i), u = ld_f32(row + Fs + i);
    return (g / (1.f + expf(-g))) * u;
}

// moe_swiglu_weighted with the routing done on the way: the block's first wave makes the token's weights
// from its logits into LDS (every block of a token the same ones), then all threads use them.
template <typename T>
__global__ __launch_bounds__(256) void moe_swiglu_routed_kernel(const T* __restrict__ gu, int gu_stride, const float* __restrict__ logits,
                                                               int l_stride, T* __restrict__ act, int act_stride, int E, int F,
                                                               int top, RouteHow how, int Fs, int width) {
    __shared__ float wts[64 * MOE_EPL];
    const int t = blockIdx.y;
    if (threadIdx.x < 64) route_token(logits + (size_t)t * l_stride, wts, E, top, how, threadIdx.x);
    __syncthreads();
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= width) return;
    if (idx >= E * F) { st_f32(act + (size_t)t * act_stride + idx, shared_column(gu + (size_t)t * gu_stride + (size_t)E * 2 * F, idx - E * F, Fs)); return; }
    const int e = idx / F, i = idx - e * F;
    const float wgt = wts[e];
    float y = 0.f;
    if (wgt != 0.f) {
        const T* row = gu + (size_t)t * gu_stride + (size_t)e * 2 * F;
        const float g = ld_f32(row + i), u = ld_f32(row + F + i);
        y = wgt * (g / (1.f + expf(-g))) * u;
    }
    st_f32(act + (size_t)t * act_stride + idx, y);
}

template <typename T>
__global__ __launch_bounds__(256) void moe_swiglu_weighted_kernel(const T* __restrict__ gu, int gu_stride, const float* __restrict__ weights,
                                                                 T* __restrict__ act, int act_stride, int E, int F, int Fs, int width) {
    const int t = blockIdx.y;
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= width) return;
    if (idx >= E * F) { st_f32(act + (size_t)t * act_stride + idx, shared_column(gu + (size_t)t * gu_stride + (size_t)E * 2 * F, idx - E * F, Fs)); return; }
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

extern "C" int ri_moe_route_as(const float* logits, int l_stride, float* weights, int T, int E, int top, int renorm,
                               int sigmoid, float eps, float scale, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && E > 0 && top > 0 && top <= E && l_stride >= E, "ri_moe_route: bad sizes T=%d E=%d top=%d", T, E, top);
    RI_REQUIRE(E <= 64 * MOE_EPL, "ri_moe_route: %d experts, the kernel takes up to %d", E, 64 * MOE_EPL);
    if (T == 0) return 0;
    RI_REQUIRE(logits && weights, "ri_moe_route: null pointer");
    const RouteHow how{sigmoid, renorm, eps, scale};
    moe_route_kernel<<<(T + 3) / 4, 256, 0, stream>>>(logits, l_stride, weights, T, E, top, how);
    RI_LAUNCHED("ri_moe_route");
    return 0;
}

extern "C" int ri_moe_route(const float* logits, int l_stride, float* weights, int T, int E, int top, int renorm, hipStream_t stream) {
    return ri_moe_route_as(logits, l_stride, weights, T, E, top, renorm, 0, 0.f, 1.f, stream);
}

// Fs: columns of a shared expert behind the experts' (0: none); width: columns of act that are written
// (E F + Fs of activations, zeros beyond).
extern "C" int ri_moe_swiglu_weighted_shared(const void* gu, int gu_stride, const float* weights, void* act, int act_stride, int dtype,
                                             int T, int E, int F, int Fs, int width, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && E > 0 && F > 0 && Fs >= 0 && width >= E * F + Fs && gu_stride >= 2 * E * F + 2 * Fs && act_stride >= width,
               "ri_moe_swiglu_weighted: bad sizes");
    if (T == 0) return 0;
    RI_REQUIRE(gu && weights && act, "ri_moe_swiglu_weighted: null pointer");
    RI_REQUIRE(T <= 65535, "ri_moe_swiglu_weighted: too many rows for the grid");
    const dim3 grid((width + 255) / 256, T);
    if (dtype == RI_F32) moe_swiglu_weighted_kernel<float><<<grid, 256, 0, stream>>>((const float*)gu, gu_stride, weights, (float*)act, act_stride, E, F, Fs, width);
    else if (dtype == RI_BF16) moe_swiglu_weighted_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)gu, gu_stride, weights, (bf16_t*)act, act_stride, E, F, Fs, width);
    else return ri_fail("ri_moe_swiglu_weighted: unknown dtype %d", dtype);
    RI_LAUNCHED("ri_moe_swiglu_weighted");
    return 0;
}

extern "C" int ri_moe_swiglu_weighted(const void* gu, int gu_stride, const float* weights, void* act, int act_stride, int dtype,
                                      int T, int E, int F, hipStream_t stream) {
    return ri_moe_swiglu_weighted_shared(gu, gu_stride, weights, act, act_stride, dtype, T, E, F, 0, E * F, stream);
}

// The two in one launch: act from gate_up and the router's 32-bit logits [T][>= E].
extern "C" int ri_moe_swiglu_routed_as(const void* gu, int gu_stride, const float* logits, int l_stride, void* act, int act_stride,
                                       int dtype, int T, int E, int F, int top, int renorm, int sigmoid, float eps, float scale,
                                       int Fs, int width, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && E > 0 && F > 0 && Fs >= 0 && width >= E * F + Fs && gu_stride >= 2 * E * F + 2 * Fs && act_stride >= width && l_stride >= E,
               "ri_moe_swiglu_routed: bad sizes");
    RI_REQUIRE(top > 0 && top <= E && E <= 64 * MOE_EPL, "ri_moe_swiglu_routed: top %d of %d experts (up to %d)", top, E, 64 * MOE_EPL);
    if (T == 0) return 0;
    RI_REQUIRE(gu && logits && act, "ri_moe_swiglu_routed: null pointer");
    RI_REQUIRE(T <= 65535, "ri_moe_swiglu_routed: too many rows for the grid");
    const dim3 grid((width + 255) / 256, T);
    const RouteHow how{sigmoid, renorm, eps, scale};
    if (dtype == RI_F32) moe_swiglu_routed_kernel<float><<<grid, 256, 0, stream>>>((const float*)gu, gu_stride, logits, l_stride, (float*)act, act_stride, E, F, top, how, Fs, width);
    else if (dtype == RI_BF16) moe_swiglu_routed_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)gu, gu_stride, logits, l_stride, (bf16_t*)act, act_stride, E, F, top, how, Fs, width);
    else return ri_fail("ri_moe_swiglu_routed: unknown dtype %d", dtype);
    RI_LAUNCHED("ri_moe_swiglu_routed");
    return 0;
}

extern "C" int ri_moe_swiglu_routed(const void* gu, int gu_stride, const float* logits, int l_stride, void* act, int act_stride,
                                    int dtype, int T, int E, int F, int top, int renorm, hipStream_t stream) {
    return ri_moe_swiglu_routed_as(gu, gu_stride, logits, l_stride, act, act_stride, dtype, T, E, F, top, renorm, 0, 0.f, 1.f, 0, E * F, stream);
}

// Layer norm (mean taken off, weight and bias) around sub-layers whose result is gated and normed
// before it joins the residual stream, and the activation of a feed-forward that norms powers.
// All arithmetic 32-bit; the stream x is 32-bit [T][d].
//
//   layer_norm            out[t] = (x[r] - mean) / sqrt(var + eps) * w + b, r = rows[t] or t
//   gated_norm_residual   y = (sum of delta parts + delta_bias) * sigmoid(gate + gate_bias);
//                         x[t] += (y - mean) / sqrt(var + eps) * w + b; optionally, in the same pass,
//                         next_out[t] = layer norm of the new x[t] with a second weight and bias (the
//                         norm in front of the next sub-layer)
//   stream_add            x[t] += other[t] (optional) + vec
//   poly_norm             act[t] = a N(z) + b N(z^2) + c N(z^3) + e with z = up[t] + up_bias and
//                         N(v) = v / sqrt(mean(v^2) + eps) over the row
//
// One block a row; a row of the gated norm passes through LDS (d floats).
#include "common.h"
#include <math.h>

namespace {

template <typename TO>
__global__ __launch_bounds__(256) void layer_norm_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                                                        const float* __restrict__ w, const float* __restrict__ b, float eps,
                                                        TO* __restrict__ out, int d) {
    __shared__ float red[16];
    const int t = blockIdx.x;
    const float* xr = x + (size_t)(rows ? rows[t] : t) * d;
    float s = 0.f;
    for (int i = threadIdx.x; i < d; i += 256) s += xr[i];
    const float mean = block_sum(s, red) / (float)d;
    float v = 0.f;
    for (int i = threadIdx.x; i < d; i += 256) { const float c = xr[i] - mean; v = fmaf(c, c, v); }
    const float rstd = 1.f / sqrtf(block_sum(v, red) / (float)d + eps);
    TO* o = out + (size_t)t * d;
    for (int i = threadIdx.x; i < d; i += 256) st_f32(o + i, (xr[i] - mean) * rstd * w[i] + b[i]);
}

template <typename TD, typename TG, typename TO>
__global__ __launch_bounds__(256) void gated_norm_residual_kernel(
        float* __restrict__ x, const TD* __restrict__ delta, int parts, size_t part_stride, const float* __restrict__ delta_bias,
        const TG* __restrict__ gate, int gate_stride, const float* __restrict__ gate_bias,
        const float* __restrict__ w, const float* __restrict__ b, float eps,
        const float* __restrict__ nw, const float* __restrict__ nb, TO* __restrict__ next_out, int d) {
    extern __shared__ float row[];                   // [d]
    __shared__ float red[16];
    const int t = blockIdx.x;
    float s = 0.f;
    for (int i = threadIdx.x; i < d; i += 256) {
        float y = ld_f32(delta + (size_t)t * d + i);
        for (int p = 1; p < parts; ++p) y += ld_f32(delta + p * part_stride + (size_t)t * d + i);
        if (delta_bias) y += delta_bias[i];
        if (gate) {
            const float z = ld_f32(gate + (size_t)t * gate_stride + i) + (gate_bias ? gate_bias[i] : 0.f);
            y *= 1.f / (1.f + expf(-z));
        }
        row[i] = y;
        s += y;
    }
    const float mean = block_sum(s, red) / (float)d;
    float v = 0.f;
    for (int i = threadIdx.x; i < d; i += 256) { const float c = row[i] - mean; v = fmaf(c, c, v); }
    const float rstd = 1.f / sqrtf(block_sum(v, red) / (float)d + eps);
    float* xr = x + (size_t)t * d;
    s = 0.f;
    for (int i = threadIdx.x; i < d; i += 256) {
        const float xn = xr[i] + ((row[i] - mean) * rstd * w[i] + b[i]);
        xr[i] = xn;
        row[i] = xn;
        s += xn;
    }
    if (next_out == nullptr) return;                 // (uniform over the block)
    const float mean2 = block_sum(s, red) / (float)d;
    v = 0.f;
    for (int i = threadIdx.x; i < d; i += 256) { const float c = row[i] - mean2; v = fmaf(c, c, v); }
    const float rstd2 = 1.f / sqrtf(block_sum(v, red) / (float)d + eps);
    TO* o = next_out + (size_t)t * d;
    for (int i = threadIdx.x; i < d; i += 256) st_f32(o + i, (row[i] - mean2) * rstd2 * nw[i] + nb[i]);
}

template <typename TA>
__global__ __launch_bounds__(256) void stream_add_kernel(float* __restrict__ x, const TA* __restrict__ other,
                                                        const float* __restrict__ vec, size_t n, int d) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float y = x[i];
    if (other) y += ld_f32(other + i);
    if (vec) y += vec[i % d];
    x[i] = y;
}

template <typename T>
__global__ __launch_bounds__(256) void poly_norm_kernel(const T* __restrict__ up, int up_stride, const float* __restrict__ bias,
                                                       float ca, float cb, float cc, float ce, float eps,
                                                       T* __restrict__ act, int act_stride, int n) {
    __shared__ float red[16];
    const int t = blockIdx.x;
    const T* zr = up + (size_t)t * up_stride;
    float s1 = 0.f, s2 = 0.f, s3 = 0.f;
    for (int i = threadIdx.x; i < n; i += 256) {
        const float z = ld_f32(zr + i) + (bias ? bias[i] : 0.f);
        const float z2 = z * z, z3 = z2 * z;
        s1 = fmaf(z, z, s1); s2 = fmaf(z2, z2, s2); s3 = fmaf(z3, z3, s3);
    }
    const float r1 = ca / sqrtf(block_sum(s1, red) / (float)n + eps);
    const float r2 = cb / sqrtf(block_sum(s2, red) / (float)n + eps);
    const float r3 = cc / sqrtf(block_sum(s3, red) / (float)n + eps);
    T* o = act + (size_t)t * act_stride;
    for (int i = threadIdx.x; i < n; i += 256) {
        const float z = ld_f32(zr + i) + (bias ? bias[i] : 0.f);
        const float z2 = z * z;
        st_f32(o + i, fmaf(z, r1, fmaf(z2, r2, fmaf(z2 * z, r3, ce))));
    }
}

}  // namespace

extern "C" int ri_layer_norm(const float* x, const int* rows, const float* w, const float* b, float eps,
                             void* out, int out_dtype, int n_out, int d, hipStream_t stream) {
    RI_REQUIRE(n_out >= 0 && d > 0 && eps > 0.f, "ri_layer_norm: bad sizes rows=%d d=%d", n_out, d);
    if (n_out == 0) return 0;
    RI_REQUIRE(x && w && b && out, "ri_layer_norm: null pointer");
    if (out_dtype == RI_F32) layer_norm_kernel<float><<<n_out, 256, 0, stream>>>(x, rows, w, b, eps, (float*)out, d);
    else if (out_dtype == RI_BF16) layer_norm_kernel<bf16_t><<<n_out, 256, 0, stream>>>(x, rows, w, b, eps, (bf16_t*)out, d);
    else return ri_fail("ri_layer_norm: unknown dtype %d", out_dtype);
    RI_LAUNCHED("ri_layer_norm");
    return 0;
}

// delta [parts][T][d] of delta_dtype (a stack of partial sums is 32-bit); gate [T][>= d] of act_dtype with
// a row stride, or null; next_out [T][d] of act_dtype, or null.
extern "C" int ri_gated_norm_residual(float* x, const void* delta, int delta_dtype, int parts, long long part_stride,
                                      const float* delta_bias, const void* gate, int gate_stride, const float* gate_bias,
                                      const float* w, const float* b, float eps, const float* next_w, const float* next_b,
                                      void* next_out, int act_dtype, int T, int d, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && d > 0 && eps > 0.f && parts >= 1 && part_stride >= 0, "ri_gated_norm_residual: bad sizes T=%d d=%d parts=%d", T, d, parts);
    RI_REQUIRE(d <= 16384, "ri_gated_norm_residual: rows of %d values, the kernel takes up to 16384", d);
    if (T == 0) return 0;
    RI_REQUIRE(x && delta && w && b, "ri_gated_norm_residual: null pointer");
    RI_REQUIRE(parts == 1 || delta_dtype == RI_F32, "ri_gated_norm_residual: partial sums must be 32-bit");
    RI_REQUIRE(!gate || gate_stride >= d, "ri_gated_norm_residual: the gate's row stride is too small");
    RI_REQUIRE(!next_out || (next_w && next_b), "ri_gated_norm_residual: the next norm needs its weight and bias");
    const size_t lds = sizeof(float) * (size_t)d, ps = (size_t)part_stride;
#define RI_GNR(DD, TD, AD, TA) if (delta_dtype == DD && act_dtype == AD) { \
        gated_norm_residual_kernel<TD, TA, TA><<<T, 256, lds, stream>>>(x, (const TD*)delta, parts, ps, delta_bias, (const TA*)gate, \
            gate_stride, gate_bias, w, b, eps, next_w, next_b, (TA*)next_out, d); \
        RI_LAUNCHED("ri_gated_norm_residual"); return 0; }
    RI_GNR(RI_F32, float, RI_F32, float)
    RI_GNR(RI_F32, float, RI_BF16, bf16_t)
    RI_GNR(RI_BF16, bf16_t, RI_BF16, bf16_t)
#undef RI_GNR
    return ri_fail("ri_gated_norm_residual: dtypes delta=%d activations=%d not taken", delta_dtype, act_dtype);
}

// x [T][d] += other [T][d] (of other_dtype, or null) + vec [d] (32-bit, or null)
extern "C" int ri_stream_add(float* x, const void* other, int other_dtype, const float* vec, int T, int d, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && d > 0, "ri_stream_add: bad sizes");
    if (T == 0 || (!other && !vec)) return 0;
    RI_REQUIRE(x, "ri_stream_add: null pointer");
    const size_t n = (size_t)T * d;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (!other || other_dtype == RI_F32) stream_add_kernel<float><<<blocks, 256, 0, stream>>>(x, (const float*)other, vec, n, d);
    else if (other_dtype == RI_BF16) stream_add_kernel<bf16_t><<<blocks, 256, 0, stream>>>(x, (const bf16_t*)other, vec, n, d);
    else return ri_fail("ri_stream_add: unknown dtype %d", other_dtype);
    RI_LAUNCHED("ri_stream_add");
    return 0;
}

extern "C" int ri_poly_norm(const void* up, int up_stride, const float* bias, float ca, float cb, float cc, float ce, float eps,
                            void* act, int act_stride, int dtype, int T, int n, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && n > 0 && eps > 0.f && up_stride >= n && act_stride >= n, "ri_poly_norm: bad sizes T=%d n=%d", T, n);
    if (T == 0) return 0;
    RI_REQUIRE(up && act, "ri_poly_norm: null pointer");
    if (dtype == RI_F32) poly_norm_kernel<float><<<T, 256, 0, stream>>>((const float*)up, up_stride, bias, ca, cb, cc, ce, eps, (float*)act, act_stride, n);
    else if (dtype == RI_BF16) poly_norm_kernel<bf16_t><<<T, 256, 0, stream>>>((const bf16_t*)up, up_stride, bias, ca, cb, cc, ce, eps, (bf16_t*)act, act_stride, n);
    else return ri_fail("ri_poly_norm: unknown dtype %d", dtype);
    RI_LAUNCHED("ri_poly_norm");
    return 0;
}

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

// The kernels below take BLOCK threads a row and VEC values a thread and load (4 where the row length,
// every row stride and every pointer allow 16-byte loads of 32-bit values, else 1).  Steps of few rows
// run with 1,024 threads a row, so that a row's loads are all in flight at once: with eight rows the
// time is that of the longest chain of dependent loads, not of the bytes.

template <typename TO, int BLOCK, int VEC>
__global__ __launch_bounds__(BLOCK) void layer_norm_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                                                          const float* __restrict__ w, const float* __restrict__ b, float eps,
                                                          TO* __restrict__ out, int d) {
    __shared__ float red[16];
    using L = VecLoad<VEC>;
    constexpr int CACHE = 4;                         // a row up to CACHE * VEC * BLOCK values stays in registers
    const int t = blockIdx.x;
    const float* xr = x + (size_t)(rows ? rows[t] : t) * d;
    float y[CACHE][VEC];
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < CACHE; ++k) {
        const int i = (threadIdx.x + k * BLOCK) * VEC;
        if (i < d) {
            L::ld(xr + i, y[k]);
#pragma unroll
            for (int e = 0; e < VEC; ++e) s += y[k][e];
        }
    }
    for (int i = (threadIdx.x + CACHE * BLOCK) * VEC; i < d; i += BLOCK * VEC) {
        float v[VEC];
        L::ld(xr + i, v);
#pragma unroll
        for (int e = 0; e < VEC; ++e) s += v[e];
    }
    const float mean = block_sum(s, red) / (float)d;
    float q = 0.f;
#pragma unroll
    for (int k = 0; k < CACHE; ++k) {
        const int i = (threadIdx.x + k * BLOCK) * VEC;
        if (i < d) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) { const float c = y[k][e] - mean; q = fmaf(c, c, q); }
        }
    }
    for (int i = (threadIdx.x + CACHE * BLOCK) * VEC; i < d; i += BLOCK * VEC) {
        float v[VEC];
        L::ld(xr + i, v);
#pragma unroll
        for (int e = 0; e < VEC; ++e) { const float c = v[e] - mean; q = fmaf(c, c, q); }
    }
    const float rstd = 1.f / sqrtf(block_sum(q, red) / (float)d + eps);
    TO* o = out + (size_t)t * d;
    auto finish = [&](int i, const float* v) {
        float wv[VEC], bv[VEC], r[VEC];
        L::ld(w + i, wv);
        L::ld(b + i, bv);
#pragma unroll
        for (int e = 0; e < VEC; ++e) r[e] = (v[e] - mean) * rstd * wv[e] + bv[e];
        L::st(o + i, r);
    };
#pragma unroll
    for (int k = 0; k < CACHE; ++k) {
        const int i = (threadIdx.x + k * BLOCK) * VEC;
        if (i < d) finish(i, y[k]);
    }
    for (int i = (threadIdx.x + CACHE * BLOCK) * VEC; i < d; i += BLOCK * VEC) {
        float v[VEC];
        L::ld(xr + i, v);
        finish(i, v);
    }
}

// PARTS > 0: that many partial sums, all asked for before any is added; 0: a runtime count.
// A thread reads back from LDS only what it wrote there itself.
template <typename TD, typename TG, typename TO, int BLOCK, int VEC, int PARTS>
__global__ __launch_bounds__(BLOCK) void gated_norm_residual_kernel(
        float* __restrict__ x, const TD* __restrict__ delta, int parts, size_t part_stride, const float* __restrict__ delta_bias,
        const TG* __restrict__ gate, int gate_stride, const float* __restrict__ gate_bias,
        const float* __restrict__ w, const float* __restrict__ b, float eps,
        const float* __restrict__ nw, const float* __restrict__ nb, TO* __restrict__ next_out, int d) {
    extern __shared__ float row[];                   // [d]
    __shared__ float red[16];
    using L = VecLoad<VEC>;
    const int t = blockIdx.x;
    const TD* dr = delta + (size_t)t * d;
    const TG* gr = gate ? gate + (size_t)t * gate_stride : nullptr;
    float s = 0.f;
    for (int i = threadIdx.x * VEC; i < d; i += BLOCK * VEC) {
        float y[VEC];
        if (PARTS > 0) {
            float p[PARTS > 0 ? PARTS : 1][VEC];
#pragma unroll
            for (int k = 0; k < PARTS; ++k) L::ld(dr + k * part_stride + i, p[k]);
#pragma unroll
            for (int e = 0; e < VEC; ++e) y[e] = p[0][e];
#pragma unroll
            for (int k = 1; k < PARTS; ++k)
#pragma unroll
                for (int e = 0; e < VEC; ++e) y[e] += p[k][e];
        } else {
            L::ld(dr + i, y);
            for (int k = 1; k < parts; ++k) {
                float p[VEC];
                L::ld(dr + k * part_stride + i, p);
#pragma unroll
                for (int e = 0; e < VEC; ++e) y[e] += p[e];
            }
        }
        if (delta_bias) {
            float c[VEC];
            L::ld(delta_bias + i, c);
#pragma unroll
            for (int e = 0; e < VEC; ++e) y[e] += c[e];
        }
        if (gr) {
            float z[VEC];
            L::ld(gr + i, z);
            if (gate_bias) {
                float c[VEC];
                L::ld(gate_bias + i, c);
#pragma unroll
                for (int e = 0; e < VEC; ++e) z[e] += c[e];
            }
#pragma unroll
            for (int e = 0; e < VEC; ++e) y[e] *= 1.f / (1.f + expf(-z[e]));
        }
        L::st(row + i, y);
#pragma unroll
        for (int e = 0; e < VEC; ++e) s += y[e];
    }
    const float mean = block_sum(s, red) / (float)d;
    float q = 0.f;
    for (int i = threadIdx.x * VEC; i < d; i += BLOCK * VEC) {
        float y[VEC];
        L::ld(row + i, y);
#pragma unroll
        for (int e = 0; e < VEC; ++e) { const float c = y[e] - mean; q = fmaf(c, c, q); }
    }
    const float rstd = 1.f / sqrtf(block_sum(q, red) / (float)d + eps);
    float* xr = x + (size_t)t * d;
    s = 0.f;
    for (int i = threadIdx.x * VEC; i < d; i += BLOCK * VEC) {
        float y[VEC], xv[VEC], wv[VEC], bv[VEC];
        L::ld(xr + i, xv);
        L::ld(w + i, wv);
        L::ld(b + i, bv);
        L::ld(row + i, y);
#pragma unroll
        for (int e = 0; e < VEC; ++e) { xv[e] += (y[e] - mean) * rstd * wv[e] + bv[e]; s += xv[e]; }
        L::st(xr + i, xv);
        L::st(row + i, xv);
    }
    if (next_out == nullptr) return;                 // (uniform over the block)
    const float mean2 = block_sum(s, red) / (float)d;
    q = 0.f;
    for (int i = threadIdx.x * VEC; i < d; i += BLOCK * VEC) {
        float y[VEC];
        L::ld(row + i, y);
#pragma unroll
        for (int e = 0; e < VEC; ++e) { const float c = y[e] - mean2; q = fmaf(c, c, q); }
    }
    const float rstd2 = 1.f / sqrtf(block_sum(q, red) / (float)d + eps);
    TO* o = next_out + (size_t)t * d;
    for (int i = threadIdx.x * VEC; i < d; i += BLOCK * VEC) {
        float y[VEC], wv[VEC], bv[VEC];
        L::ld(nw + i, wv);
        L::ld(nb + i, bv);
        L::ld(row + i, y);
#pragma unroll
        for (int e = 0; e < VEC; ++e) y[e] = (y[e] - mean2) * rstd2 * wv[e] + bv[e];
        L::st(o + i, y);
    }
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

template <typename T, int BLOCK, int VEC>
__global__ __launch_bounds__(BLOCK) void poly_norm_kernel(const T* __restrict__ up, int up_stride, const float* __restrict__ bias,
                                                         float ca, float cb, float cc, float ce, float eps,
                                                         T* __restrict__ act, int act_stride, int n) {
    __shared__ float red[48];
    using L = VecLoad<VEC>;
    constexpr int CACHE = 4;                         // a row up to CACHE * VEC * BLOCK values stays in registers
    const int t = blockIdx.x;
    const T* zr = up + (size_t)t * up_stride;
    auto value_at = [&](int i, float* z) {
        L::ld(zr + i, z);
        if (bias) {
            float c[VEC];
            L::ld(bias + i, c);
#pragma unroll
            for (int e = 0; e < VEC; ++e) z[e] += c[e];
        }
    };
    float z[CACHE][VEC];
    float s1 = 0.f, s2 = 0.f, s3 = 0.f;
    auto sums = [&](const float* v) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float z2 = v[e] * v[e], z3 = z2 * v[e];
            s1 += z2; s2 = fmaf(z2, z2, s2); s3 = fmaf(z3, z3, s3);
        }
    };
#pragma unroll
    for (int k = 0; k < CACHE; ++k) {
        const int i = (threadIdx.x + k * BLOCK) * VEC;
        if (i < n) { value_at(i, z[k]); sums(z[k]); }
    }
    for (int i = (threadIdx.x + CACHE * BLOCK) * VEC; i < n; i += BLOCK * VEC) {
        float v[VEC];
        value_at(i, v);
        sums(v);
    }
    block_sum3(s1, s2, s3, red);
    const float r1 = ca / sqrtf(s1 / (float)n + eps);
    const float r2 = cb / sqrtf(s2 / (float)n + eps);
    const float r3 = cc / sqrtf(s3 / (float)n + eps);
    T* o = act + (size_t)t * act_stride;
    auto finish = [&](int i, const float* v) {
        float r[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float z2 = v[e] * v[e];
            r[e] = fmaf(v[e], r1, fmaf(z2, r2, fmaf(z2 * v[e], r3, ce)));
        }
        L::st(o + i, r);
    };
#pragma unroll
    for (int k = 0; k < CACHE; ++k) {
        const int i = (threadIdx.x + k * BLOCK) * VEC;
        if (i < n) finish(i, z[k]);
    }
    for (int i = (threadIdx.x + CACHE * BLOCK) * VEC; i < n; i += BLOCK * VEC) {
        float v[VEC];
        value_at(i, v);
        finish(i, v);
    }
}

constexpr int FEW_ROWS = 256;                      // up to this many rows, 1,024 threads a row
static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }
static bool aligned8(const void* p) { return ((uintptr_t)p & 7) == 0; }
// whether 4 values of this dtype can be read at once from p (16 bytes of 32-bit floats, 8 of bfloat16)
static bool vec4_ok(const void* p, int dtype) { return !p || (dtype == RI_F32 ? aligned16(p) : aligned8(p)); }

}  // namespace

extern "C" int ri_layer_norm(const float* x, const int* rows, const float* w, const float* b, float eps,
                             void* out, int out_dtype, int n_out, int d, hipStream_t stream) {
    RI_REQUIRE(n_out >= 0 && d > 0 && eps > 0.f, "ri_layer_norm: bad sizes rows=%d d=%d", n_out, d);
    if (n_out == 0) return 0;
    RI_REQUIRE(x && w && b && out, "ri_layer_norm: null pointer");
    const bool v4 = d % 4 == 0 && aligned16(x) && aligned16(w) && aligned16(b) && vec4_ok(out, out_dtype);
    const bool wide = n_out <= FEW_ROWS && d >= 1024;
#define RI_LN(TO, BLOCK, VEC) layer_norm_kernel<TO, BLOCK, VEC><<<n_out, BLOCK, 0, stream>>>(x, rows, w, b, eps, (TO*)out, d)
#define RI_LN_T(TO) do { if (!v4) RI_LN(TO, 256, 1); else if (wide) RI_LN(TO, 1024, 4); else RI_LN(TO, 256, 4); } while (0)
    if (out_dtype == RI_F32) RI_LN_T(float);
    else if (out_dtype == RI_BF16) RI_LN_T(bf16_t);
    else return ri_fail("ri_layer_norm: unknown dtype %d", out_dtype);
#undef RI_LN_T
#undef RI_LN
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
    const bool v4 = d % 4 == 0 && gate_stride % 4 == 0 && (parts == 1 || ps % 4 == 0) && aligned16(x) && vec4_ok(delta, delta_dtype) &&
                    aligned16(delta_bias) && vec4_ok(gate, act_dtype) && aligned16(gate_bias) && aligned16(w) && aligned16(b) &&
                    aligned16(next_w) && aligned16(next_b) && vec4_ok(next_out, act_dtype);
    const bool wide = T <= FEW_ROWS && d >= 1024;
#define RI_GNR_L(TD, TA, BLOCK, VEC, PARTS) gated_norm_residual_kernel<TD, TA, TA, BLOCK, VEC, PARTS><<<T, BLOCK, lds, stream>>>( \
        x, (const TD*)delta, parts, ps, delta_bias, (const TA*)gate, gate_stride, gate_bias, w, b, eps, next_w, next_b, (TA*)next_out, d)
#define RI_GNR_P(TD, TA, BLOCK, VEC) do { \
        if (parts == 1) RI_GNR_L(TD, TA, BLOCK, VEC, 1); else if (parts == 2) RI_GNR_L(TD, TA, BLOCK, VEC, 2); \
        else if (parts == 4) RI_GNR_L(TD, TA, BLOCK, VEC, 4); else if (parts == 8) RI_GNR_L(TD, TA, BLOCK, VEC, 8); \
        else RI_GNR_L(TD, TA, BLOCK, VEC, 0); } while (0)
#define RI_GNR(DD, TD, AD, TA) if (delta_dtype == DD && act_dtype == AD) { \
        if (!v4) RI_GNR_L(TD, TA, 256, 1, 0); else if (wide) RI_GNR_P(TD, TA, 1024, 4); else RI_GNR_P(TD, TA, 256, 4); \
        RI_LAUNCHED("ri_gated_norm_residual"); return 0; }
    RI_GNR(RI_F32, float, RI_F32, float)
    RI_GNR(RI_F32, float, RI_BF16, bf16_t)
    RI_GNR(RI_BF16, bf16_t, RI_BF16, bf16_t)
#undef RI_GNR
#undef RI_GNR_P
#undef RI_GNR_L
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
    const bool v4 = n % 4 == 0 && up_stride % 4 == 0 && act_stride % 4 == 0 && vec4_ok(up, dtype) && vec4_ok(act, dtype) && aligned16(bias);
    const bool wide = T <= FEW_ROWS && n >= 1024;
#define RI_PN(TT, BLOCK, VEC) poly_norm_kernel<TT, BLOCK, VEC><<<T, BLOCK, 0, stream>>>((const TT*)up, up_stride, bias, ca, cb, cc, ce, eps, (TT*)act, act_stride, n)
#define RI_PN_T(TT) do { if (!v4) RI_PN(TT, 256, 1); else if (wide) RI_PN(TT, 1024, 4); else RI_PN(TT, 256, 4); } while (0)
    if (dtype == RI_F32) RI_PN_T(float);
    else if (dtype == RI_BF16) RI_PN_T(bf16_t);
    else return ri_fail("ri_poly_norm: unknown dtype %d", dtype);
#undef RI_PN_T
#undef RI_PN
    RI_LAUNCHED("ri_poly_norm");
    return 0;
}

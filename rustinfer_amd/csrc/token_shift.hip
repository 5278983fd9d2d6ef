// Two small operations on rows of the model's width.
//
//   token_shift   out[t] = h[t] + (h[t - 1] - h[t]) * mix   per channel, h[t - 1] the same request's previous
//                 token (zeros before position 0).  The last h of a request is kept in its state slot
//                 [slots][d] (32-bit) from step to step.  h is 32-bit (what a norm leaves before it is
//                 rounded); out is in the activations' dtype.  The block of a row's first token reads the
//                 old state and is also the one that writes the new one (the row's last h), thread by thread
//                 over the same channels, so no other block reads what it overwrites: prompt portions and
//                 single tokens are one kernel, and a position's result does not depend on the cut.
//   stream_pair   out[t] = [ round(x[t] + sum of the delta's parts) | round(y[t]) ] side by side, [T][2 d]:
//                 the input of a product that reads two streams at once.
#include "common.h"

namespace {

template <typename TO>
__global__ __launch_bounds__(256) void token_shift_kernel(
        const float* __restrict__ h, const float* __restrict__ mix, float* __restrict__ state, TO* __restrict__ out,
        int d, const int* __restrict__ positions, const int* __restrict__ row_of_token, const int* __restrict__ cu_q,
        const int* __restrict__ slots) {
    const int t = blockIdx.x;
    const int b = row_of_token[t];
    if (b < 0) return;                                 // padding token
    const int t_lo = cu_q[b], t_hi = cu_q[b + 1];
    const bool first = t == t_lo;
    const int pos = positions[t];
    const float* cur = h + (size_t)t * d;
    const float* last = h + (size_t)(t_hi - 1) * d;
    float* st = state + (size_t)slots[b] * d;
    TO* o = out + (size_t)t * d;
    for (int c = threadIdx.x; c < d; c += 256) {
        const float x = cur[c];
        const float prev = first ? (pos > 0 ? st[c] : 0.f) : cur[c - d];
        st_f32(o + c, fmaf(prev - x, mix[c], x));
        if (first) st[c] = last[c];
    }
}

// VEC values a thread (4 where the row length, the parts' stride and every pointer allow 16-byte loads of 32-bit
// values); a row is dealt to several blocks, and up to eight partial sums are asked for before any is added.
template <typename TD, typename TY, typename TO, int VEC>
__global__ __launch_bounds__(256) void stream_pair_kernel(
        const float* __restrict__ x, const TD* __restrict__ delta, int parts, size_t part_stride,
        const TY* __restrict__ y, TO* __restrict__ out, int d) {
    using L = VecLoad<VEC>;
    const int t = blockIdx.x;
    const int c = ((int)blockIdx.y * 256 + threadIdx.x) * VEC;
    if (c >= d) return;
    const size_t at = (size_t)t * d + c;
    float v[VEC], yv[VEC];
    L::ld(x + at, v);
    L::ld(y + at, yv);
    if (delta) {
        for (int p0 = 0; p0 < parts; p0 += 8) {
            float part[8][VEC];
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (p0 + i < parts) L::ld(delta + (size_t)(p0 + i) * part_stride + at, part[i]);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (p0 + i < parts) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) v[e] += part[i][e];
                }
        }
    }
    TO* o = out + (size_t)t * 2 * d;
    L::st(o + c, v);
    L::st(o + d + c, yv);
}

}  // namespace

// h [T][d] 32-bit, mix [d] 32-bit, state [slots][d] 32-bit, out [T][d] of out_dtype.
extern "C" int ri_token_shift(const float* h, const float* mix, float* state, int num_slots, void* out, int out_dtype,
                              int T, int d, const int* positions, const int* row_of_token, const int* cu_q,
                              const int* slots, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && d > 0 && num_slots > 0, "ri_token_shift: bad sizes");
    if (T == 0) return 0;
    RI_REQUIRE(h && mix && state && out && positions && row_of_token && cu_q && slots, "ri_token_shift: null pointer");
    if (out_dtype == RI_F32) token_shift_kernel<float><<<T, 256, 0, stream>>>(h, mix, state, (float*)out, d, positions, row_of_token, cu_q, slots);
    else if (out_dtype == RI_BF16) token_shift_kernel<bf16_t><<<T, 256, 0, stream>>>(h, mix, state, (bf16_t*)out, d, positions, row_of_token, cu_q, slots);
    else return ri_fail("ri_token_shift: unknown dtype %d", out_dtype);
    RI_LAUNCHED("ri_token_shift");
    return 0;
}

// x [T][d] 32-bit; delta null, or [parts][T][d] of delta_dtype with part_stride elements between parts;
// y [T][d] of y_dtype; out [T][2 d] of out_dtype.
extern "C" int ri_stream_pair(const float* x, const void* delta, int delta_dtype, int parts, long long part_stride,
                              const void* y, int y_dtype, void* out, int out_dtype, int T, int d, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && d > 0, "ri_stream_pair: bad sizes");
    RI_REQUIRE(!delta || (parts >= 1 && part_stride >= 0), "ri_stream_pair: bad parts");
    if (T == 0) return 0;
    RI_REQUIRE(x && y && out, "ri_stream_pair: null pointer");
    const size_t ps = (size_t)part_stride;
    const bool vec = d % 4 == 0 && part_stride % 4 == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)y % 16 == 0 && (uintptr_t)delta % 16 == 0
                     && (uintptr_t)out % 16 == 0;
    const dim3 grid(T, vec ? (d / 4 + 255) / 256 : (d + 255) / 256);
#define RI_PAIR(TD, TY, TO) do { if (vec) stream_pair_kernel<TD, TY, TO, 4><<<grid, 256, 0, stream>>>(x, (const TD*)delta, parts, ps, (const TY*)y, (TO*)out, d); \
        else stream_pair_kernel<TD, TY, TO, 1><<<grid, 256, 0, stream>>>(x, (const TD*)delta, parts, ps, (const TY*)y, (TO*)out, d); } while (0)
    if (!delta) delta_dtype = RI_F32;
    if (delta_dtype == RI_F32 && y_dtype == RI_F32 && out_dtype == RI_F32) RI_PAIR(float, float, float);
    else if (delta_dtype == RI_F32 && y_dtype == RI_F32 && out_dtype == RI_BF16) RI_PAIR(float, float, bf16_t);
    else if (delta_dtype == RI_BF16 && y_dtype == RI_F32 && out_dtype == RI_BF16) RI_PAIR(bf16_t, float, bf16_t);
    else return ri_fail("ri_stream_pair: dtypes %d / %d / %d not taken", delta_dtype, y_dtype, out_dtype);
#undef RI_PAIR
    RI_LAUNCHED("ri_stream_pair");
    return 0;
}

// A short causal convolution over time, channel by channel, with the inputs of the last taps - 1
// positions carried from step to step:
//
//   y[p][c] = f( sum_j w[c][j] * x[p - (taps - 1) + j][c] + bias[c] ),   j = 0 .. taps - 1,   x = 0 before position 0
//
// (the last column of w multiplies the current token's input), f = silu or nothing.  Up to four
// segments of channels (the columns of several projections) go through one launch; each has its input
// columns, its weights and its place in the output and in the state.  state [slots][taps - 1][C] keeps
// every request's last taps - 1 inputs (32-bit, oldest first); a row whose first position is 0 starts
// from zeros whatever its slot holds.
//
// A thread owns a channel for a chunk of a row's tokens; a row's first chunk reads the old state and
// is also the one that writes the new state (from the old one and the row's last inputs), so no other
// block reads what it overwrites: prompt portions and single tokens are one kernel, and what a
// position adds up does not depend on how the request was cut into steps.
#include "common.h"
#include <math.h>

namespace {

constexpr int SC_SEGS = 4;
constexpr int SC_CHUNK = 32;      // tokens a block walks; at least taps - 1
constexpr int SC_MAX_TAPS = 8;

struct ConvSeg {
    const void* x;       // [T][x_stride], the segment's first column
    const void* w;       // [n][taps]
    const float* bias;   // [n] or null
    int x_stride, n, out_col, first_block;
};

struct ConvArgs {
    ConvSeg seg[SC_SEGS];
    int nseg, taps, C, silu;
    float* state;        // [slots][taps - 1][C]
    float* out;          // [T][out_stride]
    int out_stride;
    const int *cu_q, *q_start, *slots;
};

template <typename T>
__global__ __launch_bounds__(256) void short_conv_kernel(const ConvArgs a) {
    int si = 0;
    while (si + 1 < a.nseg && (int)blockIdx.x >= a.seg[si + 1].first_block) ++si;
    const ConvSeg sg = a.seg[si];
    const int c = ((int)blockIdx.x - sg.first_block) * 256 + threadIdx.x;
    const int b = blockIdx.z;
    const int t_lo = a.cu_q[b], n = a.cu_q[b + 1] - t_lo;
    const int i0 = blockIdx.y * SC_CHUNK;
    if (c >= sg.n || i0 >= n) return;                 // (a row without tokens leaves everything as it is)
    const int taps = a.taps, hist = taps - 1, C = a.C;
    const int start = a.q_start[b];
    const int oc = sg.out_col + c;                    // the channel's place among all channels
    const T* xs = reinterpret_cast<const T*>(sg.x) + c;
    float* st = a.state + (size_t)a.slots[b] * hist * C + oc;
    float w[SC_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < SC_MAX_TAPS; ++j) w[j] = j < taps ? ld_f32(reinterpret_cast<const T*>(sg.w) + (size_t)c * taps + j) : 0.f;
    const float bias = sg.bias ? sg.bias[c] : 0.f;
    // the input at the row's local index i (negative: before this step)
    auto input = [&](int i) -> float {
        if (i >= 0) return ld_f32(xs + (size_t)(t_lo + i) * sg.x_stride);
        return start + i >= 0 ? st[(size_t)(hist + i) * C] : 0.f;
    };
    float old[SC_MAX_TAPS - 1];
    if (i0 == 0) {
#pragma unroll
        for (int j = 0; j < SC_MAX_TAPS - 1; ++j) old[j] = j < hist ? input(j - hist) : 0.f;
    }
    // a window of the last taps inputs slides over the chunk
    float win[SC_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < SC_MAX_TAPS - 1; ++j) {
        const int i = i0 - hist + j;
        win[j] = j < hist ? (i0 == 0 ? old[j] : input(i)) : 0.f;
    }
    const int i1 = min(n, i0 + SC_CHUNK);
    // eight inputs are asked for before the first is used: the loads of a chunk wait together, not in turn
    for (int i8 = i0; i8 < i1; i8 += 8) {
        float ahead[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) ahead[u] = i8 + u < i1 ? input(i8 + u) : 0.f;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = i8 + u;
            if (i >= i1) break;
            const float cur = ahead[u];
            float y = bias;
#pragma unroll
            for (int j = 0; j < SC_MAX_TAPS - 1; ++j) if (j < hist) y = fmaf(w[j], win[j], y);
            y = fmaf(w[hist], cur, y);
#pragma unroll
            for (int j = 0; j < SC_MAX_TAPS - 2; ++j) if (j + 1 < hist) win[j] = win[j + 1];
            if (hist > 0) win[hist - 1] = cur;
            if (a.silu) y = y / (1.f + expf(-y));
            a.out[(size_t)(t_lo + i) * a.out_stride + oc] = y;
        }
    }
    if (i0 != 0) return;
    // the new state: the last taps - 1 inputs up to the row's last token, older ones from the old state
#pragma unroll
    for (int j = 0; j < SC_MAX_TAPS - 1; ++j) {
        if (j >= hist) break;
        const int i = n - hist + j;                   // local index of the input that goes to place j
        float v = 0.f;
        if (i >= 0) v = ld_f32(xs + (size_t)(t_lo + i) * sg.x_stride);
        else {
            // place n + j of the old state (zeros there already stand for positions before 0)
#pragma unroll
            for (int jj = 0; jj < SC_MAX_TAPS - 1; ++jj) if (jj == n + j) v = old[jj];
        }
        st[(size_t)j * C] = v;
    }
}

}  // namespace

// nseg segments: x[s] (columns of `dtype`, row stride x_stride[s]), w[s] [n[s]][taps] of `dtype`; the
// segments' outputs lie side by side in out [T][out_stride] (32-bit) and in state, in the order given.
// bias: null, or nseg pointers to 32-bit [n[s]] (each may be null).
extern "C" int ri_short_conv(int nseg, const void* const* x, const int* x_stride, const void* const* w, const float* const* bias, const int* n,
                             int dtype, int taps, int silu, float* state, int num_slots, float* out, int out_stride,
                             const int* cu_q, const int* q_start, const int* slots, int num_rows, int T, int max_q_len,
                             hipStream_t stream) {
    RI_REQUIRE(nseg > 0 && nseg <= SC_SEGS, "ri_short_conv: %d segments, up to %d are taken", nseg, SC_SEGS);
    RI_REQUIRE(taps >= 1 && taps <= SC_MAX_TAPS, "ri_short_conv: %d taps, 1 to %d are taken", taps, SC_MAX_TAPS);
    RI_REQUIRE(num_rows >= 0 && T >= 0 && num_slots > 0 && max_q_len >= 0, "ri_short_conv: bad counts");
    ConvArgs a;
    int C = 0, blocks = 0;
    for (int s = 0; s < nseg; ++s) {
        RI_REQUIRE(n[s] > 0 && x_stride[s] >= n[s], "ri_short_conv: segment %d: bad sizes", s);
        a.seg[s].x = x[s]; a.seg[s].w = w[s]; a.seg[s].x_stride = x_stride[s]; a.seg[s].n = n[s];
        a.seg[s].bias = bias ? bias[s] : nullptr;
        a.seg[s].out_col = C; a.seg[s].first_block = blocks;
        C += n[s];
        blocks += (n[s] + 255) / 256;
    }
    RI_REQUIRE(out_stride >= C, "ri_short_conv: the output's row stride is too small");
    if (num_rows == 0 || T == 0) return 0;
    for (int s = 0; s < nseg; ++s) RI_REQUIRE(x[s] && w[s], "ri_short_conv: null pointer");
    RI_REQUIRE((state || taps == 1) && out && cu_q && q_start && slots, "ri_short_conv: null pointer");
    RI_REQUIRE(num_rows <= 65535, "ri_short_conv: too many rows for the grid");
    a.nseg = nseg; a.taps = taps; a.C = C; a.silu = silu; a.state = state; a.out = out; a.out_stride = out_stride;
    a.cu_q = cu_q; a.q_start = q_start; a.slots = slots;
    const int chunks = max(1, (max_q_len + SC_CHUNK - 1) / SC_CHUNK);
    RI_REQUIRE(chunks <= 65535, "ri_short_conv: rows of %d tokens are too long for the grid", max_q_len);
    const dim3 grid(blocks, chunks, num_rows);
    if (dtype == RI_F32) short_conv_kernel<float><<<grid, 256, 0, stream>>>(a);
    else if (dtype == RI_BF16) short_conv_kernel<bf16_t><<<grid, 256, 0, stream>>>(a);
    else return ri_fail("ri_short_conv: unknown dtype %d", dtype);
    RI_LAUNCHED("ri_short_conv");
    return 0;
}

// Mixers that carry a matrix of state from token to token instead of a cache of keys:
//
//   S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T,      o_t = S_t^T r_t
//
// per head, S of [dk][dv] 32-bit floats in the request's state slot.  Two forms:
//   decay form:  w_t = one constant per head, no second term (a = 0); r, k, v may pass through silu
//                (linear attention with a fixed decay);
//   delta form:  u_t = k_t / sqrt(|k_t|^2 + unit_eps),  w_t = exp(-c * sigmoid(wl_t + w0)),
//                a_t = sigmoid(al_t + ab), all per key channel (a generalized delta rule: the
//                state forgets by w and gives up what it held along u at the rate a).
//   gated form:  the delta form's walk with one decay and one write strength a head and token
//                (a gated delta rule: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q, which
//                is w = g, a u = beta g k, and beta k in place of k in the last term): q and k are made
//                unit vectors (q also times q_scale), beta = sigmoid(bl_t), g = exp(-A softplus(gl_t +
//                dt_bias)); several heads may share one head of q and k.
//   channel-gated form: the gated form with a decay for every key channel, g = exp(-A_h softplus(gl + dt_bias))
//                over heads x dk: S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T is the walk with
//                u-vector g * k, a u = beta k, w = g and beta k in the last term.
//   channel-decay forms (no second term, a decay vector a token): S <- diag(w) S + k v^T, o = S^T r (+ skip_h v):
//                w = sigmoid(gl + bias)^(1/tau) for every key channel and r times q_scale (gated linear
//                attention); or w = exp(-A_h dt) for the whole head with dt = softplus(gl_h + dt_bias_h),
//                k = dt B, r = C, several heads sharing one head of B and C, and the output also gets
//                skip_h v (a state-space layer in its recurrent form).
// Both terms of the delta form read the old state.  Everything after the projections is 32-bit.
//
// One kernel walks a request's tokens of the step in order; a step of single tokens is the same
// walk of one token.  A thread keeps R = 8 key rows (16 beyond 128 of them) of one value column in
// registers; the P threads that share a column (P = the power of two with R P >= dk, at most 16)
// are neighbouring lanes and add their partial dot products with lane exchanges that stay in the
// vector unit.  The walk is a chain from token to token and a request has only heads x columns x P
// threads, so what counts is how few instructions a thread spends on a token: hence few rows a
// thread.  The vectors of a stretch of eight tokens are asked for a stretch ahead, brought into one
// of two LDS buffers already activated, and read by the walk as broadcasts.  What a token adds up, and in which order, does not depend on how the request was
// cut into steps, so the state and the outputs have the same bits for every cut.
// A block holds four waves (256 / P columns) that share the staging, or one wave for a head of
// no more than 64 threads.
#include "common.h"
#include <math.h>

namespace {

constexpr int SC_CH = 8;         // tokens a stretch

struct ScanArgs {
    const void *r, *k, *v, *wl, *al;
    int r_stride, k_stride, v_stride, wl_stride, al_stride;
    const float *w0, *ab, *decay;
    float* state;
    float* out;
    int out_stride;
    const int *cu_q, *q_start, *slots;
    int H, dk, dv, P, silu_in;
    float unit_eps, decay_c;
    // the decay form's rotation of r and k by the token's position over their first `rot` features
    // (feature i with i + rot/2; tables [positions][rot/2], null: none), and a factor on k after it
    const float *rot_cos, *rot_sin;
    int rot;
    float k_scale;
    // the gated form: wl, al hold one value a head ([T][>= H], 32-bit or bfloat16 by gate_bf16);
    // w0 = A [H], ab = dt_bias [H]; kv_group heads share a head of r and k; r is multiplied by q_scale
    int gate_bf16, kv_group;
    float q_scale;
    int decay_bf16;      // the dtype of al where it differs from wl's (the decays' inputs may stay 32-bit)
    // the channel forms: al holds the decays' inputs ([T][>= H dk], or [T][>= H] for a decay a head) in the gates'
    // dtype; ab their bias; w0 = A [H] where the form has one; decay_c = 1 / tau; skip [H] or null
    const float* skip;
};

__device__ __forceinline__ float ld_gate(const void* p, size_t at, int is_bf16) {
    return is_bf16 ? bf16_to_f32(reinterpret_cast<const bf16_t*>(p)[at]) : reinterpret_cast<const float*>(p)[at];
}
__device__ __forceinline__ float softplusf_(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// exp on the hardware's 2^x (an error of a unit or two in the last place of 32 bits) and a division
// without the library's special cases: the staging of a stretch is a third of the walk's time
__device__ __forceinline__ float expf_(float z) { return __expf(z); }
__device__ __forceinline__ float sigmoidf_(float z) { return __fdividef(1.f, 1.f + __expf(-z)); }
__device__ __forceinline__ float siluf_(float z) { return __fdividef(z, 1.f + __expf(-z)); }
// softplus on the hardware's 2^x and log2 (an absolute error of a few 1e-8 where the result is small): for the
// decays of every key channel, which the staging makes dk at a time
__device__ __forceinline__ float softplus_fast(float z) { return z > 20.f ? z : __logf(1.f + __expf(z)); }

// Sum over the P adjacent lanes that share a column (P a power of two up to 16), every lane
// getting the same bits: exchanges inside a quad, between the quads of half a row, between the
// halves of a row of 16 lanes.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float group_sum(float x, int P) {
    if (P >= 2) x += dpp_f<0xB1>(x);                   // quad_perm [1, 0, 3, 2]
    if (P >= 4) x += dpp_f<0x4E>(x);                   // quad_perm [2, 3, 0, 1]
    if (P >= 8) x += dpp_f<0x141>(x);                  // row_half_mirror
    if (P >= 16) x += dpp_f<0x140>(x);                 // row_mirror
    return x;
}

// The block's barrier for data that passes through LDS only: the wave's LDS writes are done, then
// the barrier.  __syncthreads() would also wait for the global loads just asked for and for the
// outputs just stored, a trip to memory for every stretch of eight tokens (it was two thirds of
// the walk's time).
__device__ __forceinline__ void lds_barrier() {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// EPL: key rows a lane stages for one token (64 EPL >= dk)
// Sum over the 64 lanes with exchanges that stay in the vector unit, then one read of each row
// of 16 lanes; the same bits in every lane.
__device__ __forceinline__ float wave_sum_rows(float x) {
    x = group_sum(x, 16);
    return ((__builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 0))
           + __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 16)))
          + (__builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 32))
           + __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 48))));
}

// VAR: 0 the forms above; GATED and 1: the channel-gated form; not DELTA and 1: a decay a key channel
// (sigmoid^(1/tau)); not DELTA and 2: a decay a head and token with k = dt B (the state-space form)
template <typename T, bool DELTA, int R, int NW, int EPL, bool ROT, bool GATED = false, int VAR = 0>
__global__ __launch_bounds__(NW * 64) void linear_scan_kernel(const ScanArgs a) {
    static_assert(!GATED || (DELTA && !ROT), "the gated form is a delta form without a rotation");
    static_assert(VAR == 0 || (!ROT && (GATED || !DELTA)), "the channel forms take no rotation");
    constexpr bool VDEC = !DELTA && VAR > 0;            // a decay vector a token, no second term
    constexpr bool CHAN_IN = (GATED && VAR == 1) || (VDEC && VAR == 1);    // decay inputs for every key channel, in the gates' dtype
    constexpr int SC_EPL = EPL;
    extern __shared__ __align__(16) float lds[];
    constexpr int TPW = SC_CH / NW;                    // tokens of a stretch a wave stages
    constexpr int NA = DELTA ? 5 : (VDEC ? 3 : 2);
    const int P = a.P, DKP = P * R, dk = a.dk, dv = a.dv, H = a.H;
    const int CW = 64 / P, CPB = NW * CW;
    const int BUF = NA * SC_CH * DKP + SC_CH * CPB;    // floats of one of the two stretch buffers
    const int b = blockIdx.z, h = blockIdx.y;
    const int t_lo = a.cu_q[b], n = a.cu_q[b + 1] - t_lo;
    if (n <= 0) return;                                // a row without tokens (padding of a captured shape)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int pl = lane % P, cl = lane / P;            // the P lanes of a column are neighbours
    const int jc = wave * CW + cl, j = blockIdx.x * CPB + jc;
    const bool col_ok = j < dv;
    float* Sg = a.state + ((size_t)a.slots[b] * H + h) * (size_t)dk * dv;
    const bool fresh = a.q_start[b] == 0;              // a request's first tokens start from nothing
    float S[R];
#pragma unroll
    for (int ii = 0; ii < R; ++ii) {
        const int i = pl * R + ii;
        S[ii] = (!fresh && col_ok && i < dk) ? Sg[(size_t)i * dv + j] : 0.f;
    }
    const float dec = (DELTA || VDEC) ? 0.f : a.decay[h];
    const float skip = (VDEC && a.skip) ? a.skip[h] : 0.f;
    const T* rp = (const T*)a.r; const T* kp = (const T*)a.k; const T* vp = (const T*)a.v;
    const T* wlp = (const T*)a.wl; const T* alp = (const T*)a.al;

    // what this thread stages of a stretch: asked for a stretch ahead, so that the walk hides the wait
    float raw_r[TPW][SC_EPL], raw_k[TPW][SC_EPL], raw_w[(DELTA && !GATED) || CHAN_IN ? TPW : 1][SC_EPL], raw_a[DELTA && !GATED ? TPW : 1][SC_EPL];
    float raw_v[SC_CH];
    float raw_gb[GATED ? TPW : 1], raw_ga[GATED || VAR == 2 ? TPW : 1];       // the gated forms' numbers a token and head
    const int hk = (GATED || VAR == 2) ? h / a.kv_group : h;       // the head of r and k this head reads
    // ROT: the rotation partners of r and k (feature idx +- rot/2), asked for with them
    float part_r[ROT ? TPW : 1][SC_EPL], part_k[ROT ? TPW : 1][SC_EPL];
    const int rot_half = ROT ? a.rot >> 1 : 0;
    const int pos0 = ROT ? a.q_start[b] : 0;
    auto ask = [&](int c0) {
        const int nc = min(SC_CH, n - c0);
#pragma unroll
        for (int i = 0; i < TPW; ++i) {
            const int tt = wave + i * NW;
#pragma unroll
            for (int e = 0; e < SC_EPL; ++e) {
                const int idx = e * 64 + lane;
                const bool on = tt < nc && idx < dk;
                const size_t t = (size_t)(t_lo + c0 + (on ? tt : 0));
                const int c = hk * dk + (on ? idx : 0);
                raw_r[i][e] = on ? ld_f32(rp + t * a.r_stride + c) : 0.f;
                raw_k[i][e] = on ? ld_f32(kp + t * a.k_stride + c) : 0.f;
                if (ROT) {
                    const bool turn = on && idx < a.rot;
                    const int cp = turn ? (idx < rot_half ? c + rot_half : c - rot_half) : c;
                    part_r[i][e] = turn ? ld_f32(rp + t * a.r_stride + cp) : 0.f;
                    part_k[i][e] = turn ? ld_f32(kp + t * a.k_stride + cp) : 0.f;
                }
                if (DELTA && !GATED) {
                    raw_w[i][e] = on ? ld_f32(wlp + t * a.wl_stride + c) : 0.f;
                    raw_a[i][e] = on ? ld_f32(alp + t * a.al_stride + c) : 0.f;
                }
                if (CHAN_IN) raw_w[i][e] = on ? ld_gate(a.al, t * a.al_stride + h * dk + idx, a.decay_bf16) : 0.f;
            }
            if (GATED || VAR == 2) {
                const size_t t = (size_t)(t_lo + c0 + (tt < nc ? tt : 0));
                if (GATED) raw_gb[i] = ld_gate(a.wl, t * a.wl_stride + h, a.gate_bf16);
                if (!CHAN_IN) raw_ga[i] = ld_gate(a.al, t * a.al_stride + h, a.decay_bf16);
            }
        }
#pragma unroll
        for (int e = 0; e < SC_CH; ++e) {
            if (e * (NW * 64) >= SC_CH * CPB) break;    // a stretch has SC_CH * CPB values: SC_CH / P a thread
            const int x = e * (NW * 64) + tid;
            const int tt = x / CPB, c = x - tt * CPB, jj = blockIdx.x * CPB + c;
            raw_v[e] = (x < nc * CPB && jj < dv) ? ld_f32(vp + (size_t)(t_lo + c0 + tt) * a.v_stride + h * dv + jj) : 0.f;
        }
    };
    auto stage = [&](float* buf, int nc, int c0) {
        float* rs = buf;                               // [SC_CH][DKP] each
        float* ks = rs + SC_CH * DKP;
        float* us = ks + SC_CH * DKP;                  // the delta form's three
        float* aus = us + SC_CH * DKP;
        float* ws = VDEC ? us : aus + SC_CH * DKP;     // (the channel-decay forms keep r, k and w only)
        float* vs = buf + NA * SC_CH * DKP;            // [SC_CH][CPB]
#pragma unroll
        for (int i = 0; i < TPW; ++i) {
            const int tt = wave + i * NW;
            if (tt >= nc) continue;
            if (VDEC) {
                float dt = 0.f, dec = 0.f;
                if (VAR == 2) {
                    dt = softplus_fast(raw_ga[i] + a.ab[h]);
                    dec = expf_(-a.w0[h] * dt);
                }
#pragma unroll
                for (int e = 0; e < SC_EPL; ++e) {
                    const int idx = e * 64 + lane;
                    if (idx >= DKP) continue;
                    float r = 0.f, k = 0.f, w = 0.f;
                    if (idx < dk) {
                        if (VAR == 1) {
                            // sigmoid(z)^(1/tau) = exp(-softplus(-z) / tau)
                            r = raw_r[i][e] * a.q_scale; k = raw_k[i][e];
                            w = expf_(-softplus_fast(-(raw_w[i][e] + a.ab[h * dk + idx])) * a.decay_c);
                        } else {
                            r = raw_r[i][e]; k = dt * raw_k[i][e]; w = dec;
                        }
                    }
                    rs[tt * DKP + idx] = r; ks[tt * DKP + idx] = k; ws[tt * DKP + idx] = w;
                }
            } else if (GATED && VAR == 1) {
                float sk = 0.f, sq = 0.f;
#pragma unroll
                for (int e = 0; e < SC_EPL; ++e) { sk = fmaf(raw_k[i][e], raw_k[i][e], sk); sq = fmaf(raw_r[i][e], raw_r[i][e], sq); }
                sk = wave_sum_rows(sk);
                sq = wave_sum_rows(sq);
                const float inv_k = 1.f / sqrtf(sk + a.unit_eps), inv_q = a.q_scale / sqrtf(sq + a.unit_eps);
                const float beta = sigmoidf_(raw_gb[i]);
                const float rate = a.w0[h];
#pragma unroll
                for (int e = 0; e < SC_EPL; ++e) {
                    const int idx = e * 64 + lane;
                    if (idx >= DKP) continue;
                    const bool in = idx < dk;
                    const float u = in ? raw_k[i][e] * inv_k : 0.f;
                    const float g = in ? expf_(-rate * softplus_fast(raw_w[i][e] + a.ab[h * dk + idx])) : 0.f;
                    rs[tt * DKP + idx] = in ? raw_r[i][e] * inv_q : 0.f;
                    us[tt * DKP + idx] = g * u; ks[tt * DKP + idx] = beta * u;
                    aus[tt * DKP + idx] = beta * u; ws[tt * DKP + idx] = g;
                }
            } else if (GATED) {
                float sk = 0.f, sq = 0.f;
#pragma unroll
                for (int e = 0; e < SC_EPL; ++e) { sk = fmaf(raw_k[i][e], raw_k[i][e], sk); sq = fmaf(raw_r[i][e], raw_r[i][e], sq); }
                sk = wave_sum_rows(sk);
                sq = wave_sum_rows(sq);
                const float inv_k = 1.f / sqrtf(sk + a.unit_eps), inv_q = a.q_scale / sqrtf(sq + a.unit_eps);
                const float beta = 1.f / (1.f + expf(-raw_gb[i]));
                const float g = expf(-a.w0[h] * softplusf_(raw_ga[i] + a.ab[h]));
#pragma unroll
                for (int e = 0; e < SC_EPL; ++e) {
                    const int idx = e * 64 + lane;
                    if (idx >= DKP) continue;
                    const float u = idx < dk ? raw_k[i][e] * inv_k : 0.f;
                    rs[tt * DKP + idx] = idx < dk ? raw_r[i][e] * inv_q : 0.f;
                    us[tt * DKP + idx] = u; ks[tt * DKP + idx] = beta * u;
                    aus[tt * DKP + idx] = beta * g * u; ws[tt * DKP + idx] = g;
                }
            } else if (DELTA) {
                float ssq = 0.f;
#pragma unroll
                for (int e = 0; e < SC_EPL; ++e) ssq = fmaf(raw_k[i][e], raw_k[i][e], ssq);
                ssq = wave_sum_rows(ssq);
                const float inv = 1.f / sqrtf(ssq + a.unit_eps);
#pragma unroll
                for (int e = 0; e < SC_EPL; ++e) {
                    const int idx = e * 64 + lane;
                    if (idx >= DKP) continue;
                    float u = 0.f, au = 0.f, w = 0.f;
                    if (idx < dk) {
                        const int c = h * dk + idx;
                        u = raw_k[i][e] * inv;
                        au = sigmoidf_(raw_a[i][e] + a.ab[c]) * u;
                        w = expf_(-a.decay_c * sigmoidf_(raw_w[i][e] + a.w0[c]));
                    }
                    rs[tt * DKP + idx] = raw_r[i][e]; ks[tt * DKP + idx] = raw_k[i][e];
                    us[tt * DKP + idx] = u; aus[tt * DKP + idx] = au; ws[tt * DKP + idx] = w;
                }
            } else {
#pragma unroll
                for (int e = 0; e < SC_EPL; ++e) {
                    const int idx = e * 64 + lane;
                    if (idx >= DKP) continue;
                    float r = raw_r[i][e], k = raw_k[i][e];
                    if (a.silu_in && idx < dk) { r = siluf_(r); k = siluf_(k); }
                    if (ROT) {
                        if (idx < a.rot) {
                            const size_t at = (size_t)(pos0 + c0 + tt) * rot_half + (idx < rot_half ? idx : idx - rot_half);
                            const float cs = a.rot_cos[at], sn = idx < rot_half ? -a.rot_sin[at] : a.rot_sin[at];
                            r = fmaf(part_r[i][e], sn, r * cs);
                            k = fmaf(part_k[i][e], sn, k * cs);
                        }
                        k *= a.k_scale;
                    }
                    rs[tt * DKP + idx] = r; ks[tt * DKP + idx] = k;
                }
            }
        }
#pragma unroll
        for (int e = 0; e < SC_CH; ++e) {
            if (e * (NW * 64) >= SC_CH * CPB) break;
            const int x = e * (NW * 64) + tid;
            if (x < nc * CPB) vs[x] = (!DELTA && a.silu_in) ? siluf_(raw_v[e]) : raw_v[e];
        }
    };

    ask(0);
    for (int c0 = 0, turn = 0; c0 < n; c0 += SC_CH, turn ^= 1) {
        const int nc = min(SC_CH, n - c0);
        float* buf = lds + turn * BUF;
        // the other buffer may still be walked by a slower wave; this one was last walked two
        // stretches ago, before the barrier of the last stretch
        stage(buf, nc, c0);
        if (c0 + SC_CH < n) ask(c0 + SC_CH);
        lds_barrier();
        const float* rs = buf;
        const float* ks = rs + SC_CH * DKP;
        const float* us = ks + SC_CH * DKP;
        const float* aus = us + SC_CH * DKP;
        const float* ws = VDEC ? us : aus + SC_CH * DKP;
        const float* vs = buf + NA * SC_CH * DKP;
        // a token of the stretch; a whole stretch is unrolled, so that its reads from LDS are all asked for before
        // the first is used (a wave alone on its SIMD waits out every read it asks for late)
        auto walk = [&](int tt) {
            const float vv = vs[tt * CPB + jc];
            const int base = tt * DKP + pl * R;
            if (DELTA) {
                float dot = 0.f;
#pragma unroll
                for (int ii = 0; ii < R; ii += 4) {
                    const float4 u4 = *reinterpret_cast<const float4*>(us + base + ii);
                    dot = fmaf(u4.x, S[ii], dot); dot = fmaf(u4.y, S[ii + 1], dot);
                    dot = fmaf(u4.z, S[ii + 2], dot); dot = fmaf(u4.w, S[ii + 3], dot);
                }
                dot = group_sum(dot, P);
#pragma unroll
                for (int ii = 0; ii < R; ii += 4) {
                    const float4 w4 = *reinterpret_cast<const float4*>(ws + base + ii);
                    const float4 a4 = *reinterpret_cast<const float4*>(aus + base + ii);
                    const float4 k4 = *reinterpret_cast<const float4*>(ks + base + ii);
                    S[ii] = fmaf(w4.x, S[ii], fmaf(-a4.x, dot, k4.x * vv));
                    S[ii + 1] = fmaf(w4.y, S[ii + 1], fmaf(-a4.y, dot, k4.y * vv));
                    S[ii + 2] = fmaf(w4.z, S[ii + 2], fmaf(-a4.z, dot, k4.z * vv));
                    S[ii + 3] = fmaf(w4.w, S[ii + 3], fmaf(-a4.w, dot, k4.w * vv));
                }
            } else if (VDEC) {
#pragma unroll
                for (int ii = 0; ii < R; ii += 4) {
                    const float4 w4 = *reinterpret_cast<const float4*>(ws + base + ii);
                    const float4 k4 = *reinterpret_cast<const float4*>(ks + base + ii);
                    S[ii] = fmaf(w4.x, S[ii], k4.x * vv); S[ii + 1] = fmaf(w4.y, S[ii + 1], k4.y * vv);
                    S[ii + 2] = fmaf(w4.z, S[ii + 2], k4.z * vv); S[ii + 3] = fmaf(w4.w, S[ii + 3], k4.w * vv);
                }
            } else {
#pragma unroll
                for (int ii = 0; ii < R; ii += 4) {
                    const float4 k4 = *reinterpret_cast<const float4*>(ks + base + ii);
                    S[ii] = fmaf(dec, S[ii], k4.x * vv); S[ii + 1] = fmaf(dec, S[ii + 1], k4.y * vv);
                    S[ii + 2] = fmaf(dec, S[ii + 2], k4.z * vv); S[ii + 3] = fmaf(dec, S[ii + 3], k4.w * vv);
                }
            }
            float o = 0.f;
#pragma unroll
            for (int ii = 0; ii < R; ii += 4) {
                const float4 r4 = *reinterpret_cast<const float4*>(rs + base + ii);
                o = fmaf(r4.x, S[ii], o); o = fmaf(r4.y, S[ii + 1], o);
                o = fmaf(r4.z, S[ii + 2], o); o = fmaf(r4.w, S[ii + 3], o);
            }
            o = group_sum(o, P);
            if (VDEC) o = fmaf(skip, vv, o);
            if (pl == 0 && col_ok) a.out[(size_t)(t_lo + c0 + tt) * a.out_stride + h * dv + j] = o;
        };
        if (nc == SC_CH) {
#pragma unroll
            for (int tt = 0; tt < SC_CH; ++tt) walk(tt);
        } else {
#pragma unroll 1
            for (int tt = 0; tt < nc; ++tt) walk(tt);
        }
    }
#pragma unroll
    for (int ii = 0; ii < R; ++ii) {
        const int i = pl * R + ii;
        if (col_ok && i < dk) Sg[(size_t)i * dv + j] = S[ii];
    }
}

template <typename T, bool DELTA, int R, int NW, int EPL, bool ROT, bool GATED = false, int VAR = 0>
int launch_scan_rot(const ScanArgs& a, int num_rows, hipStream_t stream) {
    const int P = a.P, DKP = P * R, CPB = NW * (64 / P);
    const size_t lds = sizeof(float) * 2 * ((DELTA ? 5 : (VAR > 0 ? 3 : 2)) * SC_CH * DKP + SC_CH * CPB);
    dim3 grid((a.dv + CPB - 1) / CPB, a.H, num_rows);
    auto kernel = linear_scan_kernel<T, DELTA, R, NW, EPL, ROT, GATED, VAR>;
    if (lds > 64 * 1024) {
        // more LDS than a kernel gets unasked (the delta form with more than 128 key rows)
        static bool asked = false;
        if (!asked) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);
            RI_REQUIRE(e == hipSuccess, "ri_linear_scan: %zu bytes of LDS refused: %s", lds, hipGetErrorString(e));
            asked = true;
        }
    }
    kernel<<<grid, NW * 64, lds, stream>>>(a);
    return 0;
}

template <typename T, bool DELTA, int R, int NW, int EPL, bool GATED = false, int VAR = 0>
int launch_scan_as(const ScanArgs& a, int num_rows, hipStream_t stream) {
    if constexpr (GATED) return launch_scan_rot<T, true, R, NW, EPL, false, true, VAR>(a, num_rows, stream);
    if constexpr (VAR > 0) return launch_scan_rot<T, false, R, NW, EPL, false, false, VAR>(a, num_rows, stream);
    if constexpr (!DELTA) {
        if (a.rot_cos != nullptr || a.k_scale != 1.f) return launch_scan_rot<T, DELTA, R, NW, EPL, true>(a, num_rows, stream);
    }
    return launch_scan_rot<T, DELTA, R, NW, EPL, false>(a, num_rows, stream);
}

template <typename T, bool DELTA, int R, bool GATED = false, int VAR = 0>
int launch_scan(const ScanArgs& a, int num_rows, hipStream_t stream) {
    // Four waves a block share the staging of a stretch (a wave alone spends more instructions on
    // staging than on the walk); one wave where a head has no more than 64 threads.
    const bool four = (long)a.dv * a.P > 64;
    const int epl = (a.dk + 63) / 64;
    if (four) {
        if (epl == 1) return launch_scan_as<T, DELTA, R, 4, 1, GATED, VAR>(a, num_rows, stream);
        if (epl == 2) return launch_scan_as<T, DELTA, R, 4, 2, GATED, VAR>(a, num_rows, stream);
        return launch_scan_as<T, DELTA, R, 4, 4, GATED, VAR>(a, num_rows, stream);
    }
    if (epl == 1) return launch_scan_as<T, DELTA, R, 1, 1, GATED, VAR>(a, num_rows, stream);
    if (epl == 2) return launch_scan_as<T, DELTA, R, 1, 2, GATED, VAR>(a, num_rows, stream);
    return launch_scan_as<T, DELTA, R, 1, 4, GATED, VAR>(a, num_rows, stream);
}

}  // namespace

// The walk for the tokens of a step.  r, k [T, >= H dk], v [T, >= H dv] are columns of the
// projections (any row stride), in `dtype`; wl, al, w0, ab go with the delta form (delta != 0),
// decay [H] with the decay form.  state [slots][H][dk][dv] and out [T][out_stride >= H dv] are
// 32-bit.  A row whose q_start is 0 starts from a state of zeros (its slot is overwritten).
extern "C" int ri_linear_scan(
        const void* r, int r_stride, const void* k, int k_stride, const void* v, int v_stride,
        const void* wl, int wl_stride, const void* al, int al_stride, int dtype,
        const float* w0, const float* ab, const float* decay, int delta, int silu_in,
        float unit_eps, float decay_c, float* state, int num_slots, float* out, int out_stride,
        const int* cu_q, const int* q_start, const int* slots, int num_rows, int T,
        int H, int dk, int dv, const float* rot_cos, const float* rot_sin, int rot, int rot_rows, int max_position,
        float k_scale, hipStream_t stream) {
    RI_REQUIRE(H > 0 && dk > 0 && dv > 0 && dk <= 256, "ri_linear_scan: bad sizes H=%d dk=%d dv=%d (dk <= 256)", H, dk, dv);
    RI_REQUIRE(num_rows >= 0 && T >= 0 && num_slots > 0, "ri_linear_scan: bad counts");
    RI_REQUIRE(r_stride >= H * dk && k_stride >= H * dk && v_stride >= H * dv && out_stride >= H * dv,
               "ri_linear_scan: row strides too small");
    if (num_rows == 0 || T == 0) return 0;
    RI_REQUIRE(r && k && v && state && out && cu_q && q_start && slots, "ri_linear_scan: null pointer");
    RI_REQUIRE(H <= 65535 && num_rows <= 65535, "ri_linear_scan: too many heads or rows for the grid");
    if (delta) RI_REQUIRE(wl && al && w0 && ab && wl_stride >= H * dk && al_stride >= H * dk, "ri_linear_scan: the delta form needs wl, al, w0, ab");
    else RI_REQUIRE(decay, "ri_linear_scan: the decay form needs a decay for each head");
    if (rot_cos) RI_REQUIRE(!delta && !silu_in && rot_sin && rot > 0 && rot % 2 == 0 && rot <= dk && rot_rows > 0 && max_position < rot_rows,
                            "ri_linear_scan: a rotation goes with the decay form without silu, an even rot <= dk and tables of %d positions (got %d rows)", max_position + 1, rot_rows);
    if (delta) RI_REQUIRE(!rot_cos && k_scale == 1.f, "ri_linear_scan: the delta form takes no rotation and no key factor");
    // key rows a thread: 8, or 16 where 8 would need more than the 16 lanes a column may have
    const int R = dk <= 128 ? 8 : 16;
    int P = 1;
    while (P * R < dk) P *= 2;
    ScanArgs a;
    a.r = r; a.k = k; a.v = v; a.wl = wl; a.al = al;
    a.r_stride = r_stride; a.k_stride = k_stride; a.v_stride = v_stride; a.wl_stride = wl_stride; a.al_stride = al_stride;
    a.w0 = w0; a.ab = ab; a.decay = decay; a.state = state; a.out = out; a.out_stride = out_stride;
    a.cu_q = cu_q; a.q_start = q_start; a.slots = slots;
    a.H = H; a.dk = dk; a.dv = dv; a.P = P; a.silu_in = silu_in; a.unit_eps = unit_eps; a.decay_c = decay_c;
    a.rot_cos = rot_cos; a.rot_sin = rot_sin; a.rot = rot_cos ? rot : 0; a.k_scale = k_scale;
    a.gate_bf16 = 0; a.kv_group = 1; a.q_scale = 1.f; a.skip = nullptr; a.decay_bf16 = 0;
    int rc;
#define RI_SCAN(TT, DD) (R == 8 ? launch_scan<TT, DD, 8>(a, num_rows, stream) : launch_scan<TT, DD, 16>(a, num_rows, stream))
    if (dtype == RI_F32) rc = delta ? RI_SCAN(float, true) : RI_SCAN(float, false);
    else if (dtype == RI_BF16) rc = delta ? RI_SCAN(bf16_t, true) : RI_SCAN(bf16_t, false);
    else return ri_fail("ri_linear_scan: unknown dtype %d", dtype);
#undef RI_SCAN
    if (rc) return rc;
    RI_LAUNCHED("ri_linear_scan");
    return 0;
}

// The gated form of the walk.  q, k [T, >= Hk dk] and v [T, >= H dv] are 32-bit (what the short
// convolutions leave); bl, gl [T, >= H] hold the write strength's and the decay's inputs, one a head, in
// gate_dtype; A, dt_bias [H] 32-bit: g = exp(-A softplus(gl + dt_bias)), beta = sigmoid(bl).  Head h reads
// q/k head h / (H / Hk).  q and k are divided by sqrt(|.|^2 + unit_eps), q also times q_scale.
extern "C" int ri_gated_delta_scan(
        const float* q, int q_stride, const float* k, int k_stride, const float* v, int v_stride,
        const void* bl, int bl_stride, const void* gl, int gl_stride, int gate_dtype,
        const float* A, const float* dt_bias, float unit_eps, float q_scale,
        float* state, int num_slots, float* out, int out_stride,
        const int* cu_q, const int* q_start, const int* slots, int num_rows, int T,
        int H, int Hk, int dk, int dv, hipStream_t stream) {
    RI_REQUIRE(H > 0 && Hk > 0 && H % Hk == 0 && dk > 0 && dv > 0 && dk <= 256, "ri_gated_delta_scan: bad sizes H=%d Hk=%d dk=%d dv=%d (dk <= 256)", H, Hk, dk, dv);
    RI_REQUIRE(num_rows >= 0 && T >= 0 && num_slots > 0, "ri_gated_delta_scan: bad counts");
    RI_REQUIRE(q_stride >= Hk * dk && k_stride >= Hk * dk && v_stride >= H * dv && out_stride >= H * dv && bl_stride >= H && gl_stride >= H,
               "ri_gated_delta_scan: row strides too small");
    RI_REQUIRE(gate_dtype == RI_F32 || gate_dtype == RI_BF16, "ri_gated_delta_scan: unknown dtype %d", gate_dtype);
    if (num_rows == 0 || T == 0) return 0;
    RI_REQUIRE(q && k && v && bl && gl && A && dt_bias && state && out && cu_q && q_start && slots, "ri_gated_delta_scan: null pointer");
    RI_REQUIRE(H <= 65535 && num_rows <= 65535, "ri_gated_delta_scan: too many heads or rows for the grid");
    const int R = dk <= 128 ? 8 : 16;
    int P = 1;
    while (P * R < dk) P *= 2;
    ScanArgs a;
    a.r = q; a.k = k; a.v = v; a.wl = bl; a.al = gl;
    a.r_stride = q_stride; a.k_stride = k_stride; a.v_stride = v_stride; a.wl_stride = bl_stride; a.al_stride = gl_stride;
    a.w0 = A; a.ab = dt_bias; a.decay = nullptr; a.state = state; a.out = out; a.out_stride = out_stride;
    a.cu_q = cu_q; a.q_start = q_start; a.slots = slots;
    a.H = H; a.dk = dk; a.dv = dv; a.P = P; a.silu_in = 0; a.unit_eps = unit_eps; a.decay_c = 0.f;
    a.rot_cos = nullptr; a.rot_sin = nullptr; a.rot = 0; a.k_scale = 1.f;
    a.gate_bf16 = gate_dtype == RI_BF16; a.kv_group = H / Hk; a.q_scale = q_scale; a.skip = nullptr; a.decay_bf16 = a.gate_bf16;
    const int rc = R == 8 ? launch_scan<float, true, 8, true>(a, num_rows, stream) : launch_scan<float, true, 16, true>(a, num_rows, stream);
    if (rc) return rc;
    RI_LAUNCHED("ri_gated_delta_scan");
    return 0;
}

// The channel-gated form of the walk: ri_gated_delta_scan with a decay for every key channel.  gl [T, >= H dk]
// holds the decays' inputs in decay_dtype (bl [T, >= H] in gate_dtype), dt_bias [H dk] and A [H] are 32-bit:
// g = exp(-A_h softplus(gl + dt_bias)) over heads x dk.
extern "C" int ri_channel_delta_scan(
        const float* q, int q_stride, const float* k, int k_stride, const float* v, int v_stride,
        const void* bl, int bl_stride, const void* gl, int gl_stride, int gate_dtype, int decay_dtype,
        const float* A, const float* dt_bias, float unit_eps, float q_scale,
        float* state, int num_slots, float* out, int out_stride,
        const int* cu_q, const int* q_start, const int* slots, int num_rows, int T,
        int H, int Hk, int dk, int dv, hipStream_t stream) {
    RI_REQUIRE(decay_dtype == RI_F32 || decay_dtype == RI_BF16, "ri_channel_delta_scan: unknown dtype %d", decay_dtype);
    RI_REQUIRE(H > 0 && Hk > 0 && H % Hk == 0 && dk > 0 && dv > 0 && dk <= 256, "ri_channel_delta_scan: bad sizes H=%d Hk=%d dk=%d dv=%d (dk <= 256)", H, Hk, dk, dv);
    RI_REQUIRE(num_rows >= 0 && T >= 0 && num_slots > 0, "ri_channel_delta_scan: bad counts");
    RI_REQUIRE(q_stride >= Hk * dk && k_stride >= Hk * dk && v_stride >= H * dv && out_stride >= H * dv && bl_stride >= H && gl_stride >= H * dk,
               "ri_channel_delta_scan: row strides too small");
    RI_REQUIRE(gate_dtype == RI_F32 || gate_dtype == RI_BF16, "ri_channel_delta_scan: unknown dtype %d", gate_dtype);
    if (num_rows == 0 || T == 0) return 0;
    RI_REQUIRE(q && k && v && bl && gl && A && dt_bias && state && out && cu_q && q_start && slots, "ri_channel_delta_scan: null pointer");
    RI_REQUIRE(H <= 65535 && num_rows <= 65535, "ri_channel_delta_scan: too many heads or rows for the grid");
    const int R = dk <= 128 ? 8 : 16;
    int P = 1;
    while (P * R < dk) P *= 2;
    ScanArgs a;
    a.r = q; a.k = k; a.v = v; a.wl = bl; a.al = gl;
    a.r_stride = q_stride; a.k_stride = k_stride; a.v_stride = v_stride; a.wl_stride = bl_stride; a.al_stride = gl_stride;
    a.w0 = A; a.ab = dt_bias; a.decay = nullptr; a.state = state; a.out = out; a.out_stride = out_stride;
    a.cu_q = cu_q; a.q_start = q_start; a.slots = slots;
    a.H = H; a.dk = dk; a.dv = dv; a.P = P; a.silu_in = 0; a.unit_eps = unit_eps; a.decay_c = 0.f;
    a.rot_cos = nullptr; a.rot_sin = nullptr; a.rot = 0; a.k_scale = 1.f;
    a.gate_bf16 = gate_dtype == RI_BF16; a.kv_group = H / Hk; a.q_scale = q_scale; a.skip = nullptr; a.decay_bf16 = decay_dtype == RI_BF16;
    const int rc = R == 8 ? launch_scan<float, true, 8, true, 1>(a, num_rows, stream) : launch_scan<float, true, 16, true, 1>(a, num_rows, stream);
    if (rc) return rc;
    RI_LAUNCHED("ri_channel_delta_scan");
    return 0;
}

// The channel-decay forms of the walk: S <- diag(w) S + k v^T, out = S^T r (+ skip_h v).
//   mode 1: r, k [T, >= H dk], v [T, >= H dv] in `dtype`; gl [T, >= H dk] in gate_dtype, bias [H dk]:
//           w = sigmoid(gl + bias)^(1 / tau) for every key channel, r times q_scale.
//   mode 2: r, k [T, >= Hk dk] (head h reads head h / (H / Hk)), v [T, >= H dv] in `dtype`; gl [T, >= H] in
//           gate_dtype, bias [H], A [H]: dt = softplus(gl + bias), w = exp(-A dt) for the whole head, k times dt.
// skip [H] or null.  state [slots][H][dk][dv] and out are 32-bit; a row whose q_start is 0 starts from zeros.
extern "C" int ri_decay_scan(
        int mode, const void* r, int r_stride, const void* k, int k_stride, const void* v, int v_stride, int dtype,
        const void* gl, int gl_stride, int gate_dtype, const float* bias, const float* A, float inv_tau, float q_scale,
        const float* skip, float* state, int num_slots, float* out, int out_stride,
        const int* cu_q, const int* q_start, const int* slots, int num_rows, int T,
        int H, int Hk, int dk, int dv, hipStream_t stream) {
    RI_REQUIRE(mode == 1 || mode == 2, "ri_decay_scan: mode %d", mode);
    RI_REQUIRE(H > 0 && Hk > 0 && H % Hk == 0 && dk > 0 && dv > 0 && dk <= 256, "ri_decay_scan: bad sizes H=%d Hk=%d dk=%d dv=%d (dk <= 256)", H, Hk, dk, dv);
    RI_REQUIRE(mode == 2 || Hk == H, "ri_decay_scan: a decay a key channel goes with a head of r and k for every head");
    RI_REQUIRE(num_rows >= 0 && T >= 0 && num_slots > 0, "ri_decay_scan: bad counts");
    RI_REQUIRE(r_stride >= Hk * dk && k_stride >= Hk * dk && v_stride >= H * dv && out_stride >= H * dv && gl_stride >= (mode == 1 ? H * dk : H),
               "ri_decay_scan: row strides too small");
    RI_REQUIRE((dtype == RI_F32 || dtype == RI_BF16) && (gate_dtype == RI_F32 || gate_dtype == RI_BF16), "ri_decay_scan: unknown dtype");
    if (num_rows == 0 || T == 0) return 0;
    RI_REQUIRE(r && k && v && gl && bias && (mode == 1 || A) && state && out && cu_q && q_start && slots, "ri_decay_scan: null pointer");
    RI_REQUIRE(H <= 65535 && num_rows <= 65535, "ri_decay_scan: too many heads or rows for the grid");
    const int R = dk <= 128 ? 8 : 16;
    int P = 1;
    while (P * R < dk) P *= 2;
    ScanArgs a;
    a.r = r; a.k = k; a.v = v; a.wl = nullptr; a.al = gl;
    a.r_stride = r_stride; a.k_stride = k_stride; a.v_stride = v_stride; a.wl_stride = 0; a.al_stride = gl_stride;
    a.w0 = A; a.ab = bias; a.decay = nullptr; a.state = state; a.out = out; a.out_stride = out_stride;
    a.cu_q = cu_q; a.q_start = q_start; a.slots = slots;
    a.H = H; a.dk = dk; a.dv = dv; a.P = P; a.silu_in = 0; a.unit_eps = 0.f; a.decay_c = inv_tau;
    a.rot_cos = nullptr; a.rot_sin = nullptr; a.rot = 0; a.k_scale = 1.f;
    a.gate_bf16 = gate_dtype == RI_BF16; a.kv_group = H / Hk; a.q_scale = q_scale; a.skip = skip; a.decay_bf16 = a.gate_bf16;
    int rc;
#define RI_DSCAN(TT, VV) (R == 8 ? launch_scan<TT, false, 8, false, VV>(a, num_rows, stream) : launch_scan<TT, false, 16, false, VV>(a, num_rows, stream))
    if (dtype == RI_F32) rc = mode == 1 ? RI_DSCAN(float, 1) : RI_DSCAN(float, 2);
    else rc = mode == 1 ? RI_DSCAN(bf16_t, 1) : RI_DSCAN(bf16_t, 2);
#undef RI_DSCAN
    if (rc) return rc;
    RI_LAUNCHED("ri_decay_scan");
    return 0;
}

// ---------------------------------------------------------------------------
// y = o / sqrt(mean_group(o^2) + eps) * w * sigmoid(gate) (w null: no weight; gate_silu: silu(gate)
// in place of the sigmoid): the norm over groups of `group`
// consecutive features (all of a row, or a head) that follows the walk, with the output gate.
// gate_first: the gate multiplies o before the norm (the norm is over o * silu(gate)).
// o is 32-bit; gate and out are activations of `dtype` with row strides; w has n entries.
// A wave a group, or the whole block for a group of more than 512 features.
// ---------------------------------------------------------------------------
namespace {
// BLOCK_GROUP: the block's 256 threads share one group (large groups); else a wave a group,
// group blockIdx.y * waves + wave.
template <typename T, typename TW, bool BLOCK_GROUP>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(
        const float* __restrict__ o, int o_stride, int n, int group, const TW* __restrict__ w,
        const T* __restrict__ gate, int gate_stride, T* __restrict__ out, int out_stride, float eps, int gate_silu, int gate_first) {
    __shared__ float red[16];
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const float* orow = o + (size_t)t * o_stride;
    const int gidx = BLOCK_GROUP ? blockIdx.y : blockIdx.y * nw + wave;
    const int g0 = gidx * group;
    if (g0 >= n) return;
    const int first = BLOCK_GROUP ? threadIdx.x : lane, step = BLOCK_GROUP ? blockDim.x : 64;
    float ss = 0.f;
    const bool pre = gate_first && gate;
    auto gated = [&](int c) -> float {
        const float z = ld_f32(gate + (size_t)t * gate_stride + c);
        return orow[c] * (gate_silu ? siluf_(z) : sigmoidf_(z));
    };
    for (int i = first; i < group; i += step) { const float x = pre ? gated(g0 + i) : orow[g0 + i]; ss = fmaf(x, x, ss); }
    ss = BLOCK_GROUP ? block_sum(ss, red) : wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float)group + eps);
    for (int i = first; i < group; i += step) {
        const int c = g0 + i;
        float y = (pre ? gated(c) : orow[c]) * inv;
        if (w) y *= ld_f32(w + c);
        if (gate && !pre) {
            const float z = ld_f32(gate + (size_t)t * gate_stride + c);
            y *= gate_silu ? siluf_(z) : sigmoidf_(z);
        }
        st_f32(out + (size_t)t * out_stride + c, y);
    }
}
}  // namespace

extern "C" int ri_gated_group_norm(const float* o, int o_stride, int T, int n, int group, const void* w, int w_dtype,
                                   const void* gate, int gate_stride, void* out, int out_stride, int dtype,
                                   float eps, int gate_silu, int gate_first, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && n > 0 && group > 0 && n % group == 0, "ri_gated_group_norm: %d features do not split into groups of %d", n, group);
    RI_REQUIRE(o_stride >= n && out_stride >= n && (!gate || gate_stride >= n), "ri_gated_group_norm: row strides too small");
    if (T == 0) return 0;
    RI_REQUIRE(o && out, "ri_gated_group_norm: null pointer");
    if (!w) w_dtype = RI_F32;
    RI_REQUIRE(T <= 2147483647 && n / group <= 65535 * 4, "ri_gated_group_norm: too many groups for the grid");
    const int groups = n / group;
    const bool big = group > 512;
    const int block = big ? 256 : 64 * min(4, groups);
    const dim3 grid(T, big ? groups : (groups + block / 64 - 1) / (block / 64));
#define RI_GGN(TT, TW) do { if (big) gated_group_norm_kernel<TT, TW, true><<<grid, block, 0, stream>>>(o, o_stride, n, group, (const TW*)w, (const TT*)gate, gate_stride, (TT*)out, out_stride, eps, gate_silu, gate_first); \
        else gated_group_norm_kernel<TT, TW, false><<<grid, block, 0, stream>>>(o, o_stride, n, group, (const TW*)w, (const TT*)gate, gate_stride, (TT*)out, out_stride, eps, gate_silu, gate_first); } while (0)
    if (dtype == RI_F32 && w_dtype == RI_F32) RI_GGN(float, float);
    else if (dtype == RI_BF16 && w_dtype == RI_F32) RI_GGN(bf16_t, float);
    else if (dtype == RI_BF16 && w_dtype == RI_BF16) RI_GGN(bf16_t, bf16_t);
    else return ri_fail("ri_gated_group_norm: dtypes %d / %d not taken", dtype, w_dtype);
#undef RI_GGN
    RI_LAUNCHED("ri_gated_group_norm");
    return 0;
}

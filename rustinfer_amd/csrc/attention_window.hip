// Softmax attention over the paged cache for key heads of size dk and value heads of another
// size dv, inside a sliding window, with values that carry their position:
//
//   the value of position j is cached turned by j (pair m by the angle j * f_m), and the weighted
//   sum a query at position i collects is turned back by i, so that a value enters the output
//   turned by (j - i): a position code on the values that needs no second look at them.
//
// Query token t of request row b at position p, head h (key/value head g = h / (H / Hkv)):
//   keys j in [max(0, p + 1 - window), min(kv_len_b, p + 1)),  s_j = (q . K_j) * scale,
//   out = turn(-p) sum_j softmax(s)_j V_j.
// Storage is 32-bit or bfloat16; scores, weights, sums and the turns are 32-bit.
// Cache layout: keys [pages][Hkv][page][dk], values [pages][Hkv][dv][page] (positions of a
// feature contiguous).
//
// rotate_kv_write: one block a token; rotates q in place over its first `rot` features (feature
// i with i + rot/2), writes the rotated key and the turned value into the token's page.
//
// Three attention kernels: attn_window (FMA, any mix of rows; below), attn_window_mfma (steps with
// prompt portions, on the 32-bit matrix instructions; further down) and attn_window_decode with
// attn_window_combine (steps of single tokens, a row's keys divided between waves).
// attn_window: a block of four waves owns up to 32 query rows: TQ = 32 / G consecutive tokens of
// one request (G = H / Hkv query heads each) on one key/value head; a row of one token is a tile
// of its own.  Keys go by in blocks of NK (64 where LDS allows) aligned to absolute positions, so
// that what a query row adds up, and in which order, depends on its position alone and not on how
// the request was cut into steps or what else the step holds.  A block of keys and values is
// brought into LDS as 32-bit by all threads; a wave then works on four of its rows at a time
// with one key a lane for the scores and one value feature a lane (up to four) for the sums;
// each block of keys leaves a partial result that is merged into the row's running one.
#include "common.h"
#include <math.h>

namespace {

constexpr int AW_ROWS = 32;
constexpr int AW_NORM_HEADS = 1024;   // query and key heads whose unit factors rotate_kv_write holds

template <typename T>
__global__ __launch_bounds__(256) void rotate_kv_write_kernel(
        T* __restrict__ q, int q_stride, const T* __restrict__ k, int k_stride, const T* __restrict__ v, int v_stride,
        int H, int Hkv, int dk, int dv, int rot, const float* __restrict__ cos_t, const float* __restrict__ sin_t,
        const float* __restrict__ vcos, const float* __restrict__ vsin, int v_interleaved,
        const int* __restrict__ positions, const int* __restrict__ row_of_token,
        T* __restrict__ kc, T* __restrict__ vc, const int* __restrict__ table, int max_blocks, int page, int write_kv,
        float unit_eps) {
    __shared__ float inv[AW_NORM_HEADS];     // unit_eps > 0: 1 / root mean square of every query head, then of every key head
    const int t = blockIdx.x;
    const int b = row_of_token[t];
    if (b < 0) return;                       // padding token
    const int pos = positions[t];
    const int half = rot >> 1;
    const bool rotate = cos_t != nullptr;
    const bool unit = unit_eps > 0.f;
    const float* cs = rotate ? cos_t + (size_t)pos * half : nullptr;
    const float* sn = rotate ? sin_t + (size_t)pos * half : nullptr;
    T* qrow = q + (size_t)t * q_stride;
    const T* krow = k + (size_t)t * k_stride;
    if (unit) {
        // a rotation leaves a head's sum of squares as it is: the factors are made from the rows as projected
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        const int nk = write_kv ? Hkv : 0;
        for (int h = wave; h < H + nk; h += 4) {
            const T* row = h < H ? qrow + h * dk : krow + (h - H) * dk;
            float ss = 0.f;
            for (int d = lane; d < dk; d += 64) { const float x = ld_f32(row + d); ss = fmaf(x, x, ss); }
            ss = wave_sum(ss);
            if (lane == 0) inv[h] = 1.f / sqrtf(ss / (float)dk + unit_eps);
        }
        __syncthreads();
    }
    const int q_pairs = rotate ? H * half : 0;
    for (int idx = threadIdx.x; idx < q_pairs; idx += 256) {
        const int h = idx / half, i = idx - h * half;
        T* qh = qrow + h * dk;
        const float a = ld_f32(qh + i), bb = ld_f32(qh + i + half);
        const float c = cs[i], s = sn[i], f = unit ? inv[h] : 1.f;
        st_f32(qh + i, (a * c - bb * s) * f);
        st_f32(qh + i + half, (bb * c + a * s) * f);
    }
    if (unit) {
        const int first = rotate ? rot : 0, rest = dk - first;        // the features that are not turned
        for (int idx = threadIdx.x; idx < H * rest; idx += 256) {
            const int h = idx / rest, d = first + idx - h * rest;
            st_f32(qrow + h * dk + d, ld_f32(qrow + h * dk + d) * inv[h]);
        }
    }
    if (!write_kv) return;
    const int blk = table[(size_t)b * max_blocks + pos / page];
    if (blk < 0) return;
    const int slot = pos % page;
    for (int idx = threadIdx.x; idx < Hkv * dk; idx += 256) {
        const int g = idx / dk, dd = idx - g * dk;
        const T* kh = krow + g * dk;
        float val;
        if (rotate && dd < half) val = ld_f32(kh + dd) * cs[dd] - ld_f32(kh + dd + half) * sn[dd];
        else if (rotate && dd < rot) val = ld_f32(kh + dd) * cs[dd - half] + ld_f32(kh + dd - half) * sn[dd - half];
        else val = ld_f32(kh + dd);
        if (unit) val *= inv[H + g];
        st_f32(kc + (((size_t)blk * Hkv + g) * page + slot) * dk + dd, val);
    }
    const T* vrow = v + (size_t)t * v_stride;
    if (vcos != nullptr) {
        const int vh = dv >> 1;
        const float* vcs = vcos + (size_t)pos * vh;
        const float* vsn = vsin + (size_t)pos * vh;
        for (int idx = threadIdx.x; idx < Hkv * vh; idx += 256) {
            const int g = idx / vh, m = idx - g * vh;
            const int i0 = v_interleaved ? 2 * m : m, i1 = v_interleaved ? 2 * m + 1 : m + vh;
            const float a = ld_f32(vrow + g * dv + i0), bb = ld_f32(vrow + g * dv + i1);
            const float c = vcs[m], s = vsn[m];
            T* base = vc + ((size_t)blk * Hkv + g) * dv * page + slot;
            st_f32(base + (size_t)i0 * page, a * c - bb * s);
            st_f32(base + (size_t)i1 * page, bb * c + a * s);
        }
    } else {
        for (int idx = threadIdx.x; idx < Hkv * dv; idx += 256) {
            const int g = idx / dv, dd = idx - g * dv;
            vc[(((size_t)blk * Hkv + g) * dv + dd) * page + slot] = vrow[idx];
        }
    }
}

// One row's scores against the keys of a block, one key a lane: the block's maximum, the weights
// relative to it and their sum.  m_b = -inf (l_b = 0) if the row sees no key of the block.
__device__ __forceinline__ float aw_block_scores(float dot, bool mine, float scale, float& m_b, float& l_b) {
    const float sc = mine ? dot * scale : -INFINITY;
    m_b = wave_max(sc);
    float pj = 0.f;
    if (m_b > -INFINITY) pj = mine ? expf(sc - m_b) : 0.f;
    l_b = wave_sum(pj);
    return pj;
}

// The same for weights that are sigmoids of the scores plus a number a head, with no normalisation over
// the keys: the block's "maximum" is 0 where the row sees a key of it, so that merging adds the blocks' sums
// as they are (exp(0 - 0) = 1), and the result is the sum itself (aw_final_factor gives 1).
__device__ __forceinline__ float aw_block_sigmoids(float dot, bool mine, float scale, float bias, float& m_b, float& l_b) {
    const float pj = mine ? 1.f / (1.f + expf(-(dot * scale + bias))) : 0.f;
    m_b = __any(mine) ? 0.f : -INFINITY;
    l_b = wave_sum(pj);
    return pj;
}

template <int NC>
__device__ __forceinline__ void aw_merge(float& m, float& l, float (&acc)[NC], float m_b, float l_b, const float (&acc_b)[NC]) {
    if (!(m_b > -INFINITY)) return;
    const float M = fmaxf(m, m_b);
    const float alpha = expf(m - M);                   // 0 while nothing has been seen (m = -inf)
    const float beta = expf(m_b - M);
    l = l * alpha + l_b * beta;
#pragma unroll
    for (int c = 0; c < NC; ++c) acc[c] = acc[c] * alpha + acc_b[c] * beta;
    m = M;
}

// What a row's sums are multiplied by at the end: 1 / l, or, with a sink (a learned score that has no
// key and no value and counts once in the denominator), exp(m - M) / (l exp(m - M) + exp(sink - M)) with
// M = max(m, sink).  0 where nothing was seen.
__device__ __forceinline__ float aw_final_factor(float m, float l, const float* __restrict__ sink, int head) {
    if (!(l > 0.f)) return 0.f;
    if (sink == nullptr) return 1.f / l;
    const float s = sink[head], M = fmaxf(m, s), a = expf(m - M);
    return a / (l * a + expf(s - M));
}

// 16 bytes of the cache as 32-bit values: 4 floats or 8 bfloat16
__device__ __forceinline__ void ld_vec16(const float* p, float* f) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
}
__device__ __forceinline__ void ld_vec16(const bf16_t* p, float* f) {
    const uint4 v = *reinterpret_cast<const uint4*>(p);
    f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
    f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
    f[4] = __uint_as_float(v.z << 16); f[5] = __uint_as_float(v.z & 0xffff0000u);
    f[6] = __uint_as_float(v.w << 16); f[7] = __uint_as_float(v.w & 0xffff0000u);
}

template <typename T, int NC>    // NC: 64-wide slices of the value head a lane holds
__global__ __launch_bounds__(256) void attn_window_kernel(
        const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride,
        const T* __restrict__ kc, const T* __restrict__ vc, const int* __restrict__ table, int max_blocks,
        const int* __restrict__ cu_q, const int* __restrict__ q_start, const int* __restrict__ kv_lens,
        int num_rows, int H, int Hkv, int dk, int dv, int page, float scale, int window, int TQ, int NK,
        const float* __restrict__ vcos, const float* __restrict__ vsin, int v_interleaved, const float* __restrict__ sink,
        int keep, const float* __restrict__ sig_bias) {
    extern __shared__ __align__(16) float lds[];
    const int dkp = (dk + 3) & ~3, ks_stride = dkp + 4, vs_stride = dv + 1;
    float* Qs = lds;                                   // [AW_ROWS][dkp]
    float* Ps = Qs + AW_ROWS * dkp;                    // [AW_ROWS][NK]
    int* koff = reinterpret_cast<int*>(Ps + AW_ROWS * NK);      // [64] key slot in the cache, -1: none
    float* Ks = reinterpret_cast<float*>(koff + 64);   // [NK][dkp + 4]
    float* Vs = Ks + NK * ks_stride;                   // [NK][dv + 1]
    float* Os = Ks;                                    // [AW_ROWS][dv], after the last block of keys

    const int tile = blockIdx.x, g = blockIdx.y, G = H / Hkv;
    int b = -1, t0 = 0, nt = 0, before = 0;
    for (int r = 0; r < num_rows; ++r) {
        const int lo = cu_q[r], ql = cu_q[r + 1] - lo, tiles = (ql + TQ - 1) / TQ;
        if (tile < before + tiles) {
            b = r;
            t0 = lo + (tile - before) * TQ;
            nt = min(TQ, lo + ql - t0);
            break;
        }
        before += tiles;
    }
    if (b < 0) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int R = nt * G;                              // rows in use: row r = token r / G, head g G + r % G
    const int p0 = q_start[b] + (t0 - cu_q[b]);        // position of the tile's first token
    const int kv_len = kv_lens[b];
    const int last_visible = min(kv_len, p0 + nt);
    const int first_key = window > 0 ? max(0, p0 + 1 - window) : 0;

    for (int e = tid; e < AW_ROWS * dkp; e += 256) {
        const int r = e / dkp, dd = e - r * dkp;
        Qs[e] = (r < R && dd < dk) ? ld_f32(q + (size_t)(t0 + r / G) * q_stride + (g * G + r % G) * dk + dd) : 0.f;
    }
    const int batches = (R + 15) / 16;                 // the same for all waves: they share the barriers
    float m[8], l[8], acc[8][NC];
    int row_lo[8], row_hi[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        m[i] = -INFINITY;
        l[i] = 0.f;
#pragma unroll
        for (int c = 0; c < NC; ++c) acc[i][c] = 0.f;
        const int r = wave + 4 * i, p = p0 + r / G;
        row_hi[i] = r < R ? min(kv_len, p + 1) : 0;
        row_lo[i] = window > 0 ? max(0, p + 1 - window) : 0;
    }

    // keep > 0: the first `keep` positions stay in sight behind the window: their blocks of keys first
    for (int kb = keep > 0 ? 0 : first_key / NK; kb * NK < last_visible; ++kb) {
        if (kb * NK >= keep && kb < first_key / NK) kb = first_key / NK;      // from the kept positions on to the window
        const int j_base = kb * NK;
        __syncthreads();                               // the last block of keys has been used (first pass: Qs is written)
        if (tid < NK) {
            const int j = j_base + tid;
            int off = -1;
            if (j < last_visible && (j >= first_key || j < keep)) {
                const int pid = table[(size_t)b * max_blocks + j / page];
                if (pid >= 0) off = (pid * Hkv + g) * page + j % page;      // -1: a page the window has given back
            }
            koff[tid] = off;
        }
        __syncthreads();
        constexpr int VL = 16 / sizeof(T);              // elements of a 16-byte load
        if (dk % VL == 0) {                            // keys: 16 bytes a thread and load
            const int pieces = dk / VL;
            for (int e = tid; e < NK * pieces; e += 256) {
                const int jj = e / pieces, pc = e - jj * pieces, off = koff[jj];
                float f[VL];
#pragma unroll
                for (int u = 0; u < VL; ++u) f[u] = 0.f;
                if (off >= 0) ld_vec16(kc + (size_t)off * dk + pc * VL, f);
#pragma unroll
                for (int u = 0; u < VL; u += 4)
                    *reinterpret_cast<float4*>(Ks + jj * ks_stride + pc * VL + u) = make_float4(f[u], f[u + 1], f[u + 2], f[u + 3]);
            }
        } else {
            for (int e = tid; e < NK * dkp; e += 256) {
                const int jj = e / dkp, dd = e - jj * dkp, off = koff[jj];
                Ks[jj * ks_stride + dd] = (off >= 0 && dd < dk) ? ld_f32(kc + (size_t)off * dk + dd) : 0.f;
            }
        }
        if (page % VL == 0) {
            // values: the positions of a feature are contiguous; VL of them (inside one page,
            // since blocks of keys and pages both start at multiples of VL) a thread and load
            const int runs = NK / VL;
            for (int e = tid; e < runs * dv; e += 256) {
                const int d = e / runs, jj0 = (e - d * runs) * VL;
                float f[VL];
#pragma unroll
                for (int u = 0; u < VL; ++u) f[u] = 0.f;
                int first = -1;
#pragma unroll
                for (int u = 0; u < VL; ++u) if (first < 0 && koff[jj0 + u] >= 0) first = u;
                if (first >= 0) {
                    const int off = koff[jj0 + first] - first;           // slot of the run's first position
                    ld_vec16(vc + (size_t)(off / page) * page * dv + (size_t)d * page + off % page, f);
                }
#pragma unroll
                for (int u = 0; u < VL; ++u) Vs[(jj0 + u) * vs_stride + d] = koff[jj0 + u] >= 0 ? f[u] : 0.f;
            }
        } else {
            const int jj = tid % NK, off = koff[jj];
            const size_t vbase = off >= 0 ? (size_t)(off / page) * page * dv + off % page : 0;
            for (int d = tid / NK; d < dv; d += 256 / NK)
                Vs[jj * vs_stride + d] = off >= 0 ? ld_f32(vc + vbase + (size_t)d * page) : 0.f;
        }
        __syncthreads();
        float m_b[8], l_b[8], acc_b[8][NC];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            m_b[i] = -INFINITY;
            l_b[i] = 0.f;
#pragma unroll
            for (int c = 0; c < NC; ++c) acc_b[i][c] = 0.f;
        }
#pragma unroll
        for (int bi = 0; bi < 2; ++bi) {
            if (bi >= batches) break;
            // rows of this batch that exist for this wave (a step of single tokens has G rows a tile)
            const int nrb = min(4, (R - wave + 3) / 4 - 4 * bi);
            float s[4] = {0.f, 0.f, 0.f, 0.f};
            const float* kr = Ks + (lane < NK ? lane : 0) * ks_stride;
#pragma unroll 2
            for (int dd = 0; dd < dkp; dd += 4) {
                const float4 k4 = *reinterpret_cast<const float4*>(kr + dd);
#pragma unroll
                for (int rb = 0; rb < 4; ++rb) {
                    if (rb >= nrb) break;
                    const float4 q4 = *reinterpret_cast<const float4*>(Qs + (wave + 4 * (4 * bi + rb)) * dkp + dd);
                    s[rb] = fmaf(q4.x, k4.x, s[rb]);
                    s[rb] = fmaf(q4.y, k4.y, s[rb]);
                    s[rb] = fmaf(q4.z, k4.z, s[rb]);
                    s[rb] = fmaf(q4.w, k4.w, s[rb]);
                }
            }
            const int j = j_base + lane;
#pragma unroll
            for (int rb = 0; rb < 4; ++rb) {
                const int i = 4 * bi + rb;
                const bool mine = lane < NK && (j >= row_lo[i] || j < keep) && j < row_hi[i];
                const float pj = sig_bias ? aw_block_sigmoids(s[rb], mine, scale, sig_bias[g * G + (wave + 4 * i) % G], m_b[i], l_b[i])
                                          : aw_block_scores(s[rb], mine, scale, m_b[i], l_b[i]);
                if (lane < NK) Ps[(wave + 4 * i) * NK + lane] = pj;
            }
        }
        __syncthreads();
#pragma unroll
        for (int bi = 0; bi < 2; ++bi) {
            if (bi >= batches) break;
            const int nrb = min(4, (R - wave + 3) / 4 - 4 * bi);
            if (nrb <= 0) break;
#pragma unroll 1
            for (int jj = 0; jj < NK; jj += 4) {
                float4 p4[4];
#pragma unroll
                for (int rb = 0; rb < 4; ++rb)
                    p4[rb] = *reinterpret_cast<const float4*>(Ps + (wave + 4 * (4 * bi + rb)) * NK + jj);
#pragma unroll
                for (int u = 0; u < 4; ++u) {
#pragma unroll
                    for (int c = 0; c < NC; ++c) {
                        const int d = lane + 64 * c;
                        const float v = d < dv ? Vs[(jj + u) * vs_stride + d] : 0.f;
#pragma unroll
                        for (int rb = 0; rb < 4; ++rb) {
                            if (rb >= nrb) break;
                            const float pv = u == 0 ? p4[rb].x : u == 1 ? p4[rb].y : u == 2 ? p4[rb].z : p4[rb].w;
                            acc_b[4 * bi + rb][c] = fmaf(pv, v, acc_b[4 * bi + rb][c]);
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) aw_merge<NC>(m[i], l[i], acc[i], m_b[i], l_b[i], acc_b[i]);
    }
    if (vcos == nullptr) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int r = wave + 4 * i;
            if (r >= R) continue;
            T* o = out + (size_t)(t0 + r / G) * out_stride + (g * G + r % G) * dv;
            const float fin = sig_bias ? 1.f : sink ? aw_final_factor(m[i], l[i], sink, g * G + r % G) : 0.f;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const int d = lane + 64 * c;
                if (d < dv) st_f32(o + d, (sink || sig_bias) ? acc[i][c] * fin : (l[i] > 0.f ? acc[i][c] / l[i] : 0.f));
            }
        }
        return;
    }
    // the sums are turned back by the query's position: through LDS, since a pair's two
    // features lie in different lanes
    __syncthreads();                                   // the last keys and values have been used
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int r = wave + 4 * i;
        if (r >= R) continue;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const int d = lane + 64 * c;
            if (d < dv) Os[r * dv + d] = sig_bias ? acc[i][c] : sink ? acc[i][c] * aw_final_factor(m[i], l[i], sink, g * G + r % G) : (l[i] > 0.f ? acc[i][c] / l[i] : 0.f);
        }
    }
    __syncthreads();
    const int vh = dv >> 1;
    for (int r = wave; r < R; r += 4) {
        const int p = p0 + r / G;
        T* o = out + (size_t)(t0 + r / G) * out_stride + (g * G + r % G) * dv;
        for (int mm = lane; mm < vh; mm += 64) {
            const int i0 = v_interleaved ? 2 * mm : mm, i1 = v_interleaved ? 2 * mm + 1 : mm + vh;
            const float a = Os[r * dv + i0], bb = Os[r * dv + i1];
            const float c = vcos[(size_t)p * vh + mm], s = vsin[(size_t)p * vh + mm];
            st_f32(o + i0, a * c + bb * s);
            st_f32(o + i1, bb * c - a * s);
        }
    }
}

// Single tokens with kept first positions: how many of the blocks of NK keys that hold kept positions lie
// wholly before the window's first block and hold a key the row sees (the others are the window's, or empty).
__device__ __forceinline__ int aw_keep_used(int keep, int NK, int first_key, int visible) {
    const int seen = min(keep, visible);
    return min((seen + NK - 1) / NK, first_key / NK);
}

// Steps of single tokens: merge the partial results of a row's blocks of keys in ascending order
// (the order and the arithmetic of the loop in attn_window_kernel), divide, turn back, write.
// One wave a (token, head).
template <typename T, int NC>
__global__ __launch_bounds__(64) void attn_window_combine_kernel(
        const float* __restrict__ part_ml, const float* __restrict__ part_o, T* __restrict__ out, int out_stride,
        const int* __restrict__ cu_q, const int* __restrict__ q_start, const int* __restrict__ kv_lens,
        int H, int dv, int window, int NK, int slots,
        const float* __restrict__ vcos, const float* __restrict__ vsin, int v_interleaved, const float* __restrict__ sink,
        int keep, int sigmoid_weights) {
    __shared__ float Os[256];
    const int b = blockIdx.y, h = blockIdx.x, lane = threadIdx.x;
    const int t = cu_q[b];
    if (cu_q[b + 1] - t <= 0) return;                  // a row without a token
    const int p = q_start[b];
    const int visible = min(kv_lens[b], p + 1);
    const int first_key = window > 0 ? max(0, p + 1 - window) : 0;
    // the first slots belong to the blocks of the kept positions (those that lie before the window's first block)
    const int keep_slots = (keep + NK - 1) / NK, keep_used = aw_keep_used(keep, NK, first_key, visible);
    const int n = keep_slots + (visible + NK - 1) / NK - first_key / NK;
    float m = -INFINITY, l = 0.f, acc[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) acc[c] = 0.f;
    // eight blocks' partial results are asked for at once, then merged one after the other in the
    // order of the blocks: the loads of a block do not wait for the merge of the one before
    constexpr int AHEAD = 8;
    const int count = min(n, slots);
    for (int s0 = 0; s0 < count; s0 += AHEAD) {
        float acc_b[AHEAD][NC], m_b[AHEAD], l_b[AHEAD];
#pragma unroll
        for (int i = 0; i < AHEAD; ++i) {
            const bool on = s0 + i < count && (s0 + i >= keep_slots || s0 + i < keep_used);
            const size_t at = ((size_t)t * H + h) * slots + (on ? s0 + i : 0);
            m_b[i] = on ? part_ml[at * 2] : -INFINITY;
            l_b[i] = on ? part_ml[at * 2 + 1] : 0.f;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const int d = lane + 64 * c;
                acc_b[i][c] = (on && d < dv) ? part_o[at * dv + d] : 0.f;
            }
        }
#pragma unroll
        for (int i = 0; i < AHEAD; ++i)
            if (s0 + i < count) aw_merge<NC>(m, l, acc, m_b[i], l_b[i], acc_b[i]);        // (a slot that is off has m_b = -inf)
    }
    T* o = out + (size_t)t * out_stride + h * dv;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        const int d = lane + 64 * c;
        if (d < dv) {
            const float y = sigmoid_weights ? acc[c] : sink ? acc[c] * aw_final_factor(m, l, sink, h) : (l > 0.f ? acc[c] / l : 0.f);
            if (vcos == nullptr) st_f32(o + d, y);
            else Os[d] = y;
        }
    }
    if (vcos == nullptr) return;
    __syncthreads();
    const int vh = dv >> 1;
    for (int mm = lane; mm < vh; mm += 64) {
        const int i0 = v_interleaved ? 2 * mm : mm, i1 = v_interleaved ? 2 * mm + 1 : mm + vh;
        const float a = Os[i0], bb = Os[i1];
        const float c = vcos[(size_t)p * vh + mm], s = vsin[(size_t)p * vh + mm];
        st_f32(o + i0, a * c + bb * s);
        st_f32(o + i1, bb * c - a * s);
    }
}

// Steps of single tokens, the partial results: one wave a block of 64 keys of a row's window
// and all G query heads of a key/value head, nothing staged.  Scores with a key a lane (the
// key's row read straight from the cache, 16 bytes at a time; the query rows are the same address
// for all lanes), the weights through the wave's own LDS rows, sums with a value feature a lane
// (up to four) over the positions of a feature, 16 bytes at a time.  Same partial results and the
// same arithmetic, term for term, as a block of keys in attn_window_kernel.
constexpr int AD_KEYS = 64;

template <typename T, int NC>
__global__ __launch_bounds__(256) void attn_window_decode_kernel(
        const T* __restrict__ q, int q_stride, const T* __restrict__ kc, const T* __restrict__ vc,
        const int* __restrict__ table, int max_blocks, const int* __restrict__ cu_q, const int* __restrict__ q_start,
        const int* __restrict__ kv_lens, int H, int Hkv, int dk, int dv, int page, float scale, int window, int slots,
        float* __restrict__ part_ml, float* __restrict__ part_o, int heads_a_wave, int keep, const float* __restrict__ sig_bias) {
    extern __shared__ __align__(16) float lds[];       // [4 waves][G][64] weights
    // many query heads a key/value head (one shared latent, say): the heads are dealt to several
    // blocks in stretches of heads_a_wave, each reading the block of keys for its own heads
    const int G = H / Hkv, stretches = (G + heads_a_wave - 1) / heads_a_wave;
    const int b = blockIdx.z, g = blockIdx.y / stretches;
    const int h_lo = (blockIdx.y % stretches) * heads_a_wave, h_hi = min(G, h_lo + heads_a_wave);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t = cu_q[b];
    if (cu_q[b + 1] - t <= 0) return;                  // a row without a token
    const int p = q_start[b];
    const int visible = min(kv_lens[b], p + 1);
    const int j0 = window > 0 ? max(0, p + 1 - window) : 0;
    const int slot = (int)blockIdx.x * 4 + wave;
    const int keep_slots = (keep + AD_KEYS - 1) / AD_KEYS;
    if (slot < keep_slots && slot >= aw_keep_used(keep, AD_KEYS, j0, visible)) return;
    const int kb = slot < keep_slots ? slot : j0 / AD_KEYS + slot - keep_slots;
    if (slot >= slots || kb * AD_KEYS >= visible) return;
    float* Ps = lds + (size_t)wave * G * AD_KEYS;
    constexpr int VL = 16 / sizeof(T);

    const int j = kb * AD_KEYS + lane;
    const bool mine = (j >= j0 || j < keep) && j < visible;
    long long off = -1;
    int own_pid = -1;                                  // the page of the lane's own key
    if (mine) {
        const int pid = table[(size_t)b * max_blocks + j / page];
        own_pid = pid;
        if (pid >= 0) off = ((long long)pid * Hkv + g) * page + j % page;
    }
    const T* kr = off >= 0 ? kc + (size_t)off * dk : nullptr;
    const T* qrow = q + (size_t)t * q_stride + (size_t)g * G * dk;
    const size_t at0 = ((size_t)t * H + (size_t)g * G) * slots + slot;      // + head * slots
    const bool kvec = dk % VL == 0;
    for (int h0 = h_lo; h0 < h_hi; h0 += 4) {
        float s[4] = {0.f, 0.f, 0.f, 0.f};
        if (kvec) {
            for (int dd = 0; dd < dk; dd += VL) {
                float kf[VL];
#pragma unroll
                for (int u = 0; u < VL; ++u) kf[u] = 0.f;
                if (kr) ld_vec16(kr + dd, kf);
#pragma unroll
                for (int rb = 0; rb < 4; ++rb) {
                    if (h0 + rb >= h_hi) break;
                    float qf[VL];
                    ld_vec16(qrow + (size_t)(h0 + rb) * dk + dd, qf);
#pragma unroll
                    for (int u = 0; u < VL; ++u) s[rb] = fmaf(qf[u], kf[u], s[rb]);
                }
            }
        } else {
            for (int dd = 0; dd < dk; ++dd) {
                const float kf = kr ? ld_f32(kr + dd) : 0.f;
#pragma unroll
                for (int rb = 0; rb < 4; ++rb)
                    if (h0 + rb < h_hi) s[rb] = fmaf(ld_f32(qrow + (size_t)(h0 + rb) * dk + dd), kf, s[rb]);
            }
        }
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) {
            if (h0 + rb >= h_hi) break;
            float m_b, l_b;
            Ps[(h0 + rb) * AD_KEYS + lane] = sig_bias ? aw_block_sigmoids(s[rb], mine, scale, sig_bias[g * G + h0 + rb], m_b, l_b)
                                                      : aw_block_scores(s[rb], mine, scale, m_b, l_b);
            if (lane == 0) {
                float* dst = part_ml + (at0 + (size_t)(h0 + rb) * slots) * 2;
                dst[0] = m_b;
                dst[1] = l_b;
            }
        }
    }
    __builtin_amdgcn_wave_barrier();                   // the wave's own weights are in LDS (LDS keeps a wave's order)
    const bool vvec = page % VL == 0;
    for (int h0 = h_lo; h0 < h_hi; h0 += 4) {
        float acc[4][NC];
#pragma unroll
        for (int rb = 0; rb < 4; ++rb)
#pragma unroll
            for (int c = 0; c < NC; ++c) acc[rb][c] = 0.f;
        for (int jj = 0; jj < AD_KEYS; jj += VL) {
            const int key = kb * AD_KEYS + jj;         // VL keys of one page where pages allow
            if (key >= visible) break;
            float v[VL][NC];
#pragma unroll
            for (int u = 0; u < VL; ++u)
#pragma unroll
                for (int c = 0; c < NC; ++c) v[u][c] = 0.f;
            if (vvec) {
                // the group's page from the lane of its first key that the row sees (the same page: VL keys
                // do not cross one), not from the table again: a trip to memory less for every group
                const int pid = key < keep ? __shfl(own_pid, jj, 64) : key + VL > j0 ? __shfl(own_pid, max(jj, j0 - kb * AD_KEYS), 64) : -1;
                if (pid >= 0) {
#pragma unroll
                    for (int c = 0; c < NC; ++c) {
                        const int d = lane + 64 * c;
                        if (d < dv) {
                            float f[VL];
                            ld_vec16(vc + (((size_t)pid * Hkv + g) * dv + d) * page + key % page, f);
                            if ((key >= j0 || key + VL <= keep) && key + VL <= visible) {      // (the same for the whole wave)
#pragma unroll
                                for (int u = 0; u < VL; ++u) v[u][c] = f[u];
                            } else {                                     // a group at the window's, the kept positions' or the request's end
#pragma unroll
                                for (int u = 0; u < VL; ++u) v[u][c] = ((key + u >= j0 || key + u < keep) && key + u < visible) ? f[u] : 0.f;
                            }
                        }
                    }
                }
            } else {
#pragma unroll
                for (int u = 0; u < VL; ++u) {
                    const int ku = key + u;
                    if ((ku < j0 && ku >= keep) || ku >= visible) continue;
                    const int pid = table[(size_t)b * max_blocks + ku / page];
                    if (pid < 0) continue;
#pragma unroll
                    for (int c = 0; c < NC; ++c) {
                        const int d = lane + 64 * c;
                        if (d < dv) v[u][c] = ld_f32(vc + (((size_t)pid * Hkv + g) * dv + d) * page + ku % page);
                    }
                }
            }
#pragma unroll
            for (int rb = 0; rb < 4; ++rb) {
                if (h0 + rb >= h_hi) break;
#pragma unroll
                for (int u = 0; u < VL; ++u) {
                    const float pv = Ps[(h0 + rb) * AD_KEYS + jj + u];
#pragma unroll
                    for (int c = 0; c < NC; ++c) acc[rb][c] = fmaf(pv, v[u][c], acc[rb][c]);
                }
            }
        }
#pragma unroll
        for (int rb = 0; rb < 4; ++rb) {
            if (h0 + rb >= h_hi) break;
            float* dst = part_o + (at0 + (size_t)(h0 + rb) * slots) * dv;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const int d = lane + 64 * c;
                if (d < dv) dst[d] = acc[rb][c];
            }
        }
    }
}

int aw_keys_a_block(int dk, int dv);

size_t aw_lds_bytes(int dk, int dv, int NK) {
    const int dkp = (dk + 3) & ~3;
    const size_t kv = (size_t)NK * (dkp + 4) + (size_t)NK * (dv + 1);
    const size_t os = (size_t)AW_ROWS * dv;
    return sizeof(float) * ((size_t)AW_ROWS * dkp + (size_t)AW_ROWS * NK + 64 + (kv > os ? kv : os));
}

constexpr size_t AW_LDS_MOST = 150 * 1024;

int aw_keys_a_block(int dk, int dv) {
    int NK = 64;
    while (NK > 16 && aw_lds_bytes(dk, dv, NK) > AW_LDS_MOST) NK >>= 1;
    return NK;
}

// blocks of keys the window of a single token can touch when no request is longer than max_kv_len
int aw_slots(int dk, int dv, int window, int max_kv_len, int keep) {
    const int NK = AD_KEYS;
    const int span = window > 0 ? min(window, max_kv_len) : max_kv_len;
    // a window may begin inside a block: one more; the blocks of the kept positions come first
    return (span + NK - 1) / NK + (window > 0 ? 1 : 0) + (window > 0 ? (keep + NK - 1) / NK : 0);
}

}  // namespace

extern "C" int ri_attention_window_supported(int H, int Hkv, int dk, int dv) {
    return H > 0 && Hkv > 0 && H % Hkv == 0 && H / Hkv <= AW_ROWS && dk > 0 && dk <= 256 && dv > 0 && dv <= 256
        && aw_lds_bytes(dk, dv, 16) <= AW_LDS_MOST;
}

extern "C" int ri_rotate_kv_write(
        void* q, int q_stride, const void* k, int k_stride, const void* v, int v_stride, int dtype, int T,
        int H, int Hkv, int dk, int dv, int rot, const float* cos_t, const float* sin_t, int table_rows,
        const float* vcos, const float* vsin, int v_table_rows, int v_interleaved,
        const int* positions, const int* row_of_token, void* kc, void* vc, int num_pages,
        const int* table, int max_blocks, int page, int write_kv, float unit_eps, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && H > 0 && Hkv > 0 && dk > 0 && dv > 0 && page > 0, "ri_rotate_kv_write: bad sizes");
    RI_REQUIRE(unit_eps >= 0.f && (unit_eps == 0.f || H + Hkv <= AW_NORM_HEADS), "ri_rotate_kv_write: unit queries and keys for up to %d heads", AW_NORM_HEADS);
    RI_REQUIRE(q_stride >= H * dk, "ri_rotate_kv_write: query row stride %d too small", q_stride);
    if (cos_t) RI_REQUIRE(rot > 0 && rot % 2 == 0 && rot <= dk && sin_t && table_rows > 0, "ri_rotate_kv_write: rot %d must be even and within the key size %d", rot, dk);
    if (vcos) RI_REQUIRE(dv % 2 == 0 && vsin && v_table_rows > 0, "ri_rotate_kv_write: a turned value needs an even size, got %d", dv);
    if (write_kv) RI_REQUIRE(k && v && kc && vc && table && max_blocks > 0 && num_pages > 0 && k_stride >= Hkv * dk && v_stride >= Hkv * dv,
                             "ri_rotate_kv_write: no keys, values or cache given, or their row strides too small");
    if (T == 0) return 0;
    RI_REQUIRE(q && positions && row_of_token, "ri_rotate_kv_write: null pointer");
    if (dtype == RI_F32)
        rotate_kv_write_kernel<float><<<T, 256, 0, stream>>>((float*)q, q_stride, (const float*)k, k_stride, (const float*)v, v_stride, H, Hkv, dk, dv, rot, cos_t, sin_t, vcos, vsin, v_interleaved, positions, row_of_token, (float*)kc, (float*)vc, table, max_blocks, page, write_kv, unit_eps);
    else if (dtype == RI_BF16)
        rotate_kv_write_kernel<bf16_t><<<T, 256, 0, stream>>>((bf16_t*)q, q_stride, (const bf16_t*)k, k_stride, (const bf16_t*)v, v_stride, H, Hkv, dk, dv, rot, cos_t, sin_t, vcos, vsin, v_interleaved, positions, row_of_token, (bf16_t*)kc, (bf16_t*)vc, table, max_blocks, page, write_kv, unit_eps);
    else
        return ri_fail("ri_rotate_kv_write: unknown dtype %d", dtype);
    RI_LAUNCHED("ri_rotate_kv_write");
    return 0;
}

namespace {
template <typename T>
int aw_launch(const T* q, int q_stride, T* out, int out_stride, const T* kc, const T* vc, const int* table, int max_blocks,
              const int* cu_q, const int* q_start, const int* kv_lens, int num_rows, int Tn, int H, int Hkv, int dk, int dv,
              int page, float scale, int window, const float* vcos, const float* vsin, int v_interleaved,
              int slots, float* workspace, const float* sink, int keep, const float* sig_bias, hipStream_t stream) {
    const int G = H / Hkv, TQ = AW_ROWS / G;
    const int NK = aw_keys_a_block(dk, dv);
    const size_t lds = aw_lds_bytes(dk, dv, NK);
    const int NC = (dv + 63) / 64;
    auto kernel = NC == 1 ? attn_window_kernel<T, 1> : NC == 2 ? attn_window_kernel<T, 2> : NC == 3 ? attn_window_kernel<T, 3> : attn_window_kernel<T, 4>;
    if (lds > 64 * 1024) {
        // more LDS than a kernel gets unasked: requested once for each form of the kernel
        static bool asked[5] = {};
        if (!asked[NC]) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)AW_LDS_MOST);
            RI_REQUIRE(e == hipSuccess, "ri_attention_window: %zu bytes of LDS refused: %s", lds, hipGetErrorString(e));
            asked[NC] = true;
        }
    }
    if (slots > 0) {
        // every row has at most one token: a tile a row, a block a block of keys, then the merge
        float* part_ml = workspace;
        float* part_o = workspace + (size_t)Tn * H * slots * 2;
        auto part = NC == 1 ? attn_window_decode_kernel<T, 1> : NC == 2 ? attn_window_decode_kernel<T, 2>
                  : NC == 3 ? attn_window_decode_kernel<T, 3> : attn_window_decode_kernel<T, 4>;
        // beyond eight heads a key/value head, four heads a wave (one pass over the block of keys): a step
        // of few rows then has waves enough to hide the loads of one another (32 heads on one latent, 8 rows
        // of 2,048 keys: 258 us with all heads in one wave, 78 with eight, 47 with four, 74 with two)
        // (a window of 1,024 keys leaves half as many waves as 2,048 keys and a wave takes as long: when the
        // waves are fewer than one and a half for each of the chip's 1,024 SIMDs, two heads a wave: 46 -> 42 us.
        // Asking for four pieces of a key row, or two groups of values, before the first is used: 112 us.)
        int heads_a_wave = G <= 8 ? G : 4;
        if (G > 8 && (long)slots * Hkv * ((G + 3) / 4) * num_rows < 1536) heads_a_wave = 2;
        const int stretches = (G + heads_a_wave - 1) / heads_a_wave;
        RI_REQUIRE((long)Hkv * stretches <= 65535, "ri_attention_window: too many heads for the grid");
        part<<<dim3((slots + 3) / 4, Hkv * stretches, num_rows), 256, sizeof(float) * 4 * G * AD_KEYS, stream>>>(
            q, q_stride, kc, vc, table, max_blocks, cu_q, q_start, kv_lens, H, Hkv, dk, dv, page, scale, window, slots, part_ml, part_o,
            heads_a_wave, keep, sig_bias);
        auto combine = NC == 1 ? attn_window_combine_kernel<T, 1> : NC == 2 ? attn_window_combine_kernel<T, 2>
                     : NC == 3 ? attn_window_combine_kernel<T, 3> : attn_window_combine_kernel<T, 4>;
        combine<<<dim3(H, num_rows), 64, 0, stream>>>(part_ml, part_o, out, out_stride, cu_q, q_start, kv_lens, H, dv, window, AD_KEYS, slots,
                                                      vcos, vsin, v_interleaved, sink, keep, sig_bias != nullptr);
        return 0;
    }
    const int tiles = (Tn + TQ - 1) / TQ + num_rows;   // at most: every request may end in a short tile
    kernel<<<dim3(tiles, Hkv), 256, lds, stream>>>(q, q_stride, out, out_stride, kc, vc, table, max_blocks, cu_q, q_start, kv_lens,
                                                   num_rows, H, Hkv, dk, dv, page, scale, window, TQ, NK, vcos, vsin, v_interleaved, sink,
                                                   keep, sig_bias);
    return 0;
}
}  // namespace

// Floats of workspace for a step of T single tokens whose longest request has max_kv_len keys
// (0: such a step has one block of keys a row at most and needs none).
extern "C" size_t ri_attention_window_workspace(int T, int H, int dk, int dv, int window, int max_kv_len, int keep) {
    const int slots = aw_slots(dk, dv, window, max_kv_len, window > 0 ? keep : 0);
    return slots <= 1 ? 0 : (size_t)T * H * slots * (dv + 2);
}

// Attention of the step's tokens (rotated queries in q) over the cache; out [T][>= H dv].
// vcos / vsin [positions][dv / 2]: the sums are turned back by the query's position (null: not).
// sink [H] (null: none): a score a query head that counts once in the softmax's denominator.
// single_tokens != 0: every row of the step has at most one token and row b's token is token
// cu_q[b]; with a workspace of ri_attention_window_workspace floats the keys of a row are then
// divided between blocks (the same bits as without).
// keep: with a window, the first `keep` positions of a request stay in sight of every later query.
// sig_bias [H] (null: softmax): the weight of a visible key is sigmoid(score + sig_bias[head]) and the
// weights are not normalised over the keys (no sink then).
extern "C" int ri_attention_window(
        const void* q, int q_stride, void* out, int out_stride, int dtype, const void* kc, const void* vc,
        int num_pages, int page, int H, int Hkv, int dk, int dv, const int* table, int max_blocks,
        const int* cu_q, const int* q_start, const int* kv_lens, int num_rows, int T,
        float scale, int window, const float* vcos, const float* vsin, int v_table_rows, int v_interleaved,
        int single_tokens, int max_kv_len, float* workspace, size_t workspace_floats, const float* sink,
        int keep, const float* sig_bias, hipStream_t stream) {
    RI_REQUIRE(ri_attention_window_supported(H, Hkv, dk, dv), "ri_attention_window: sizes not taken (H=%d Hkv=%d dk=%d dv=%d)", H, Hkv, dk, dv);
    RI_REQUIRE(keep >= 0 && !(sink && sig_bias), "ri_attention_window: keep must be >= 0, and sigmoid weights take no sink");
    if (window == 0) keep = 0;
    RI_REQUIRE(T >= 0 && num_rows >= 0 && max_blocks > 0 && num_pages > 0 && window >= 0 && page > 0, "ri_attention_window: bad sizes");
    RI_REQUIRE(q_stride >= H * dk && out_stride >= H * dv, "ri_attention_window: row strides too small");
    if (vcos) RI_REQUIRE(vsin && dv % 2 == 0 && v_table_rows > 0, "ri_attention_window: a turned value needs an even size and both tables");
    if (T == 0 || num_rows == 0) return 0;
    RI_REQUIRE(q && out && kc && vc && table && cu_q && q_start && kv_lens, "ri_attention_window: null pointer");
    RI_REQUIRE(Hkv <= 65535, "ri_attention_window: too many key/value heads for the grid");
    int slots = 0;
    if (single_tokens && workspace && max_kv_len > 0) {
        slots = aw_slots(dk, dv, window, max_kv_len, keep);
        if (slots <= 1) slots = 0;
        else RI_REQUIRE(workspace_floats >= (size_t)T * H * slots * (dv + 2) && slots <= 65535 && num_rows <= 65535 && H <= 65535,
                        "ri_attention_window: workspace of %zu floats for %d slots, or too many rows for the grid", workspace_floats, slots);
    }
    int rc;
    if (dtype == RI_F32)
        rc = aw_launch<float>((const float*)q, q_stride, (float*)out, out_stride, (const float*)kc, (const float*)vc, table, max_blocks, cu_q, q_start, kv_lens, num_rows, T, H, Hkv, dk, dv, page, scale, window, vcos, vsin, v_interleaved, slots, workspace, sink, keep, sig_bias, stream);
    else if (dtype == RI_BF16)
        rc = aw_launch<bf16_t>((const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)kc, (const bf16_t*)vc, table, max_blocks, cu_q, q_start, kv_lens, num_rows, T, H, Hkv, dk, dv, page, scale, window, vcos, vsin, v_interleaved, slots, workspace, sink, keep, sig_bias, stream);
    else
        return ri_fail("ri_attention_window: unknown dtype %d", dtype);
    if (rc) return rc;
    RI_LAUNCHED("ri_attention_window");
    return 0;
}

// ---------------------------------------------------------------------------
// Prompt portions on the matrix cores, in 32-bit: v_mfma_f32_32x32x2_f32 for both products, so
// that scores, softmax weights and weighted sums keep 32 bits (the bfloat16 matrix instructions
// would round the weights).  A wave owns 32 query tokens of one head and computes, for a tile of
// 32 keys, S^T = K Q^T (keys down the registers, ONE query a lane: the softmax of a query is a
// reduction over the lane's own 16 registers and one exchange with the lane 32 further on), then
// O^T += V^T P^T with the weights used where they lie: step i of the second product takes key
// 8 (i / 4) + i % 4 of the tile from the lower 32 lanes and key 8 (i / 4) + 4 + i % 4 from the
// upper, which is what accumulator register i of the first product holds.  The query's features
// stay in registers for the whole tile; keys and values of 64 positions at a time go through LDS
// as 32-bit for the four waves of a block: the heads of one key/value head (four at a time), or,
// for fewer than four heads a key/value head, consecutive tiles of 32 tokens.  Key tiles are
// aligned to absolute positions and a query's arithmetic does not depend on its place in the tile:
// a token's output has the same bits however its request was cut.
// QU: 8-feature units of the (zero-padded) key head; FT: 32-feature tiles of the value head.
// ---------------------------------------------------------------------------
namespace {

typedef float aw_f16 __attribute__((ext_vector_type(16)));
constexpr int AM_KEYS = 64;      // keys a stage

size_t am_lds_bytes(int QU, int dv) {
    const size_t stage = (size_t)AM_KEYS * (8 * QU + 4) + (size_t)AM_KEYS * (dv + 8);
    const size_t outs = (size_t)128 * dv;
    return sizeof(float) * (64 + (stage > outs ? stage : outs));
}

template <typename T, int QU, int FT>
__global__ __launch_bounds__(256) void attn_window_mfma_kernel(
        const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride,
        const T* __restrict__ kc, const T* __restrict__ vc, const int* __restrict__ table, int max_blocks,
        const int* __restrict__ cu_q, const int* __restrict__ q_start, const int* __restrict__ kv_lens,
        int num_rows, int H, int Hkv, int dk, int dv, int page, float scale, int window,
        const float* __restrict__ vcos, const float* __restrict__ vsin, int v_interleaved, const float* __restrict__ sink,
        int keep, const float* __restrict__ sig_bias) {
    extern __shared__ __align__(16) float lds[];
    constexpr int DKP = 8 * QU, KS = DKP + 4;
    const int vs_stride = dv + 8;
    int* koff = reinterpret_cast<int*>(lds);           // [64]
    float* Ks = lds + 64;                              // [64][DKP + 4]
    float* Vs = Ks + AM_KEYS * KS;                     // [64][dv + 8]
    float* Os = Ks;                                    // [4 waves][32][dv], after the last stage

    const int G = H / Hkv, HB = G < 4 ? G : 4, SB = 4 / HB, TQB = 32 * SB;
    const int g = blockIdx.y, hgroup = blockIdx.z;
    int b = -1, t0 = 0, nt = 0, before = 0;
    for (int r = 0; r < num_rows; ++r) {
        const int lo = cu_q[r], ql = cu_q[r + 1] - lo, tiles = (ql + TQB - 1) / TQB;
        if ((int)blockIdx.x < before + tiles) {
            b = r;
            t0 = lo + ((int)blockIdx.x - before) * TQB;
            nt = min(TQB, lo + ql - t0);
            break;
        }
        before += tiles;
    }
    if (b < 0) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lq = lane & 31, lh = lane >> 5;          // the lane's query, and which half of the key pairs
    const int p0 = q_start[b] + (t0 - cu_q[b]);
    const int kv_len = kv_lens[b];
    const int blk_last = min(kv_len, p0 + nt);
    const int blk_first = window > 0 ? max(0, p0 + 1 - window) : 0;
    // this wave's 32 tokens and head
    const int sub = wave / HB, hh = hgroup * 4 + wave % HB;
    const bool wave_on = sub < SB && hh < G && nt - 32 * sub > 0;
    const int t0w = t0 + 32 * sub, ntw = wave_on ? min(32, nt - 32 * sub) : 0, p0w = p0 + 32 * sub;
    const int head = g * G + (hh < G ? hh : 0);
    const int w_last = wave_on ? min(kv_len, p0w + ntw) : 0;
    const int w_first = window > 0 ? max(0, p0w + 1 - window) : 0;
    const bool row_on = lq < ntw;
    const int pq = p0w + lq;                           // the lane's query position

    // the query's features, in the order the products take them: unit u, step c -> feature 8 u + 4 lh + c
    float qr[QU * 4];
#pragma unroll
    for (int u = 0; u < QU; ++u)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int d = 8 * u + 4 * lh + c;
            qr[u * 4 + c] = (row_on && d < dk) ? ld_f32(q + (size_t)(t0w + lq) * q_stride + head * dk + d) * scale : 0.f;
        }
    // the padding of the key rows beyond dk stays zero: the staging writes features below dk only
    for (int e = tid; e < AM_KEYS * KS; e += 256) Ks[e] = 0.f;

    aw_f16 o[FT];
#pragma unroll
    for (int ft = 0; ft < FT; ++ft)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[ft][i] = 0.f;
    float m = -INFINITY, l = 0.f;

    const float bias = sig_bias ? sig_bias[head] : 0.f;
    for (int st = keep > 0 ? 0 : blk_first / AM_KEYS; st * AM_KEYS < blk_last; ++st) {
        if (st * AM_KEYS >= keep && st < blk_first / AM_KEYS) st = blk_first / AM_KEYS;      // from the kept positions on to the window
        const int j_base = st * AM_KEYS;
        __syncthreads();                               // the last stage has been used (first pass: the zeros are written)
        if (tid < AM_KEYS) {
            const int j = j_base + tid;
            int off = -1;
            if (j < blk_last && (j >= blk_first || j < keep)) {
                const int pid = table[(size_t)b * max_blocks + j / page];
                if (pid >= 0) off = (pid * Hkv + g) * page + j % page;
            }
            koff[tid] = off;
        }
        __syncthreads();
        constexpr int VL = 16 / sizeof(T);
        if (dk % VL == 0) {
            const int pieces = dk / VL;
            for (int e = tid; e < AM_KEYS * pieces; e += 256) {
                const int jj = e / pieces, pc = e - jj * pieces, off = koff[jj];
                float f[VL];
#pragma unroll
                for (int u = 0; u < VL; ++u) f[u] = 0.f;
                if (off >= 0) ld_vec16(kc + (size_t)off * dk + pc * VL, f);
#pragma unroll
                for (int u = 0; u < VL; u += 4)
                    *reinterpret_cast<float4*>(Ks + jj * KS + pc * VL + u) = make_float4(f[u], f[u + 1], f[u + 2], f[u + 3]);
            }
        } else {
            for (int e = tid; e < AM_KEYS * dk; e += 256) {
                const int jj = e / dk, dd = e - jj * dk, off = koff[jj];
                Ks[jj * KS + dd] = off >= 0 ? ld_f32(kc + (size_t)off * dk + dd) : 0.f;
            }
        }
        if (page % VL == 0) {
            const int runs = AM_KEYS / VL;
            for (int e = tid; e < runs * dv; e += 256) {
                const int d = e / runs, jj0 = (e - d * runs) * VL;
                float f[VL];
#pragma unroll
                for (int u = 0; u < VL; ++u) f[u] = 0.f;
                int first = -1;
#pragma unroll
                for (int u = 0; u < VL; ++u) if (first < 0 && koff[jj0 + u] >= 0) first = u;
                if (first >= 0) {
                    const int off = koff[jj0 + first] - first;
                    ld_vec16(vc + (size_t)(off / page) * page * dv + (size_t)d * page + off % page, f);
                }
#pragma unroll
                for (int u = 0; u < VL; ++u) Vs[(jj0 + u) * vs_stride + d] = koff[jj0 + u] >= 0 ? f[u] : 0.f;
            }
        } else {
            const int jj = tid & 63, off = koff[jj];
            const size_t vbase = off >= 0 ? (size_t)(off / page) * page * dv + off % page : 0;
            for (int d = tid >> 6; d < dv; d += 4)
                Vs[jj * vs_stride + d] = off >= 0 ? ld_f32(vc + vbase + (size_t)d * page) : 0.f;
        }
        __syncthreads();
#pragma unroll 1
        for (int half = 0; half < 2; ++half) {
            const int kt0 = j_base + 32 * half;        // first key of the tile
            if (kt0 >= w_last || (kt0 + 32 <= w_first && kt0 >= keep)) continue;     // none of the wave's queries sees it (the same for all lanes)
            // S^T = K Q^T (the scale is in the query)
            aw_f16 s;
#pragma unroll
            for (int i = 0; i < 16; ++i) s[i] = 0.f;
            const float* krow = Ks + (32 * half + lq) * KS + 4 * lh;
#pragma unroll
            for (int u = 0; u < QU; ++u) {
                const float4 k4 = *reinterpret_cast<const float4*>(krow + 8 * u);
                s = __builtin_amdgcn_mfma_f32_32x32x2f32(k4.x, qr[u * 4 + 0], s, 0, 0, 0);
                s = __builtin_amdgcn_mfma_f32_32x32x2f32(k4.y, qr[u * 4 + 1], s, 0, 0, 0);
                s = __builtin_amdgcn_mfma_f32_32x32x2f32(k4.z, qr[u * 4 + 2], s, 0, 0, 0);
                s = __builtin_amdgcn_mfma_f32_32x32x2f32(k4.w, qr[u * 4 + 3], s, 0, 0, 0);
            }
            // register i: key kt0 + 8 (i / 4) + 4 lh + i % 4, for the lane's query
            const int j_lo = window > 0 ? pq + 1 - window : 0, j_hi = min(pq + 1, kv_len);
            float mt = -INFINITY;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int j = kt0 + 8 * (i >> 2) + 4 * lh + (i & 3);
                const bool vis = row_on && (j >= j_lo || j < keep) && j < j_hi;
                s[i] = vis ? s[i] : -INFINITY;
                mt = fmaxf(mt, s[i]);
            }
            if (sig_bias) {
                // sigmoids of the scores, added up as they are: nothing to rescale
#pragma unroll
                for (int i = 0; i < 16; ++i) s[i] = s[i] > -INFINITY ? 1.f / (1.f + expf(-(s[i] + bias))) : 0.f;
            } else {
                mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
                const float m_new = fmaxf(m, mt);
                const bool any = m_new > -INFINITY;        // else the query has seen no key yet: nothing to add
                const float alpha = any ? expf(m - m_new) : 1.f;
                float psum = 0.f;
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    s[i] = (any && s[i] > -INFINITY) ? expf(s[i] - m_new) : 0.f;
                    psum += s[i];
                }
                l = l * alpha + psum;
                m = m_new;
#pragma unroll
                for (int ft = 0; ft < FT; ++ft)
#pragma unroll
                    for (int i = 0; i < 16; ++i) o[ft][i] *= alpha;
            }
            // O^T += V^T P^T
#pragma unroll
            for (int ft = 0; ft < FT; ++ft) {
                const int f = 32 * ft + lq;
                if (32 * ft >= dv) continue;
                const float* vcol = Vs + (32 * half + 4 * lh) * vs_stride + (f < dv ? f : 0);
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const float a = f < dv ? vcol[(8 * (i >> 2) + (i & 3)) * vs_stride] : 0.f;
                    o[ft] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, s[i], o[ft], 0, 0, 0);
                }
            }
        }
    }
    // the sums of a query lie in the lane of its lower and of its upper half: add the two l
    l += __shfl_xor(l, 32, 64);
    const float inv = sig_bias ? 1.f : aw_final_factor(m, l, sink, head);
    __syncthreads();                                   // the last keys and values have been used
    float* ow = Os + (size_t)wave * 32 * dv;
    if (wave_on) {
#pragma unroll
        for (int ft = 0; ft < FT; ++ft)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int f = 32 * ft + 8 * (i >> 2) + 4 * lh + (i & 3);
                if (f < dv) ow[lq * dv + f] = o[ft][i] * inv;
            }
    }
    __syncthreads();
    if (!wave_on) return;
    const int vh = dv >> 1;
    for (int r = 0; r < ntw; ++r) {
        T* orow = out + (size_t)(t0w + r) * out_stride + head * dv;
        if (vcos == nullptr) {
            for (int f = lane; f < dv; f += 64) st_f32(orow + f, ow[r * dv + f]);
        } else {
            const int p = p0w + r;
            for (int mm = lane; mm < vh; mm += 64) {
                const int i0 = v_interleaved ? 2 * mm : mm, i1 = v_interleaved ? 2 * mm + 1 : mm + vh;
                const float a = ow[r * dv + i0], bb = ow[r * dv + i1];
                const float c = vcos[(size_t)p * vh + mm], s_ = vsin[(size_t)p * vh + mm];
                st_f32(orow + i0, a * c + bb * s_);
                st_f32(orow + i1, bb * c - a * s_);
            }
        }
    }
}

template <typename T, int QU, int FT>
int am_launch_as(const T* q, int q_stride, T* out, int out_stride, const T* kc, const T* vc, const int* table, int max_blocks,
                 const int* cu_q, const int* q_start, const int* kv_lens, int num_rows, int Tn, int H, int Hkv, int dk, int dv,
                 int page, float scale, int window, const float* vcos, const float* vsin, int v_interleaved, const float* sink,
                 int keep, const float* sig_bias, hipStream_t stream) {
    const int G = H / Hkv, HB = G < 4 ? G : 4, SB = 4 / HB, TQB = 32 * SB;
    const size_t lds = am_lds_bytes(QU, dv);
    auto kernel = attn_window_mfma_kernel<T, QU, FT>;
    if (lds > 64 * 1024) {
        static bool asked = false;
        if (!asked) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            RI_REQUIRE(e == hipSuccess, "ri_attention_window: %zu bytes of LDS refused: %s", lds, hipGetErrorString(e));
            asked = true;
        }
    }
    const int tiles = (Tn + TQB - 1) / TQB + num_rows;
    kernel<<<dim3(tiles, Hkv, (G + 3) / 4), 256, lds, stream>>>(q, q_stride, out, out_stride, kc, vc, table, max_blocks, cu_q, q_start,
                                                               kv_lens, num_rows, H, Hkv, dk, dv, page, scale, window, vcos, vsin, v_interleaved, sink, keep, sig_bias);
    return 0;
}

template <typename T>
int am_launch(const T* q, int q_stride, T* out, int out_stride, const T* kc, const T* vc, const int* table, int max_blocks,
              const int* cu_q, const int* q_start, const int* kv_lens, int num_rows, int Tn, int H, int Hkv, int dk, int dv,
              int page, float scale, int window, const float* vcos, const float* vsin, int v_interleaved, const float* sink,
              int keep, const float* sig_bias, hipStream_t stream) {
#define RI_AM(QU, FT) return am_launch_as<T, QU, FT>(q, q_stride, out, out_stride, kc, vc, table, max_blocks, cu_q, q_start, kv_lens, \
        num_rows, Tn, H, Hkv, dk, dv, page, scale, window, vcos, vsin, v_interleaved, sink, keep, sig_bias, stream)
    if (dk <= 64) { if (dv <= 64) RI_AM(8, 2); if (dv <= 128) RI_AM(8, 4); RI_AM(8, 8); }
    if (dk <= 128) { if (dv <= 64) RI_AM(16, 2); if (dv <= 128) RI_AM(16, 4); RI_AM(16, 8); }
    if (dv <= 64) RI_AM(32, 2);
    if (dv <= 128) RI_AM(32, 4);
    RI_AM(32, 8);
#undef RI_AM
}

}  // namespace

extern "C" int ri_attention_window_mfma_supported(int H, int Hkv, int dk, int dv) {
    if (!ri_attention_window_supported(H, Hkv, dk, dv)) return 0;
    const int QU = dk <= 64 ? 8 : dk <= 128 ? 16 : 32;
    return am_lds_bytes(QU, dv) <= 160 * 1024;
}

// The same attention as ri_attention_window for steps with prompt portions, on the 32-bit matrix
// instructions.
extern "C" int ri_attention_window_mfma(
        const void* q, int q_stride, void* out, int out_stride, int dtype, const void* kc, const void* vc,
        int num_pages, int page, int H, int Hkv, int dk, int dv, const int* table, int max_blocks,
        const int* cu_q, const int* q_start, const int* kv_lens, int num_rows, int T,
        float scale, int window, const float* vcos, const float* vsin, int v_table_rows, int v_interleaved,
        const float* sink, int keep, const float* sig_bias, hipStream_t stream) {
    RI_REQUIRE(ri_attention_window_mfma_supported(H, Hkv, dk, dv), "ri_attention_window_mfma: sizes not taken (H=%d Hkv=%d dk=%d dv=%d)", H, Hkv, dk, dv);
    RI_REQUIRE(keep >= 0 && !(sink && sig_bias), "ri_attention_window_mfma: keep must be >= 0, and sigmoid weights take no sink");
    if (window == 0) keep = 0;
    RI_REQUIRE(T >= 0 && num_rows >= 0 && max_blocks > 0 && num_pages > 0 && window >= 0 && page > 0, "ri_attention_window_mfma: bad sizes");
    RI_REQUIRE(q_stride >= H * dk && out_stride >= H * dv, "ri_attention_window_mfma: row strides too small");
    if (vcos) RI_REQUIRE(vsin && dv % 2 == 0 && v_table_rows > 0, "ri_attention_window_mfma: a turned value needs an even size and both tables");
    if (T == 0 || num_rows == 0) return 0;
    RI_REQUIRE(q && out && kc && vc && table && cu_q && q_start && kv_lens, "ri_attention_window_mfma: null pointer");
    RI_REQUIRE(Hkv <= 65535, "ri_attention_window_mfma: too many key/value heads for the grid");
    int rc;
    if (dtype == RI_F32)
        rc = am_launch<float>((const float*)q, q_stride, (float*)out, out_stride, (const float*)kc, (const float*)vc, table, max_blocks, cu_q, q_start, kv_lens, num_rows, T, H, Hkv, dk, dv, page, scale, window, vcos, vsin, v_interleaved, sink, keep, sig_bias, stream);
    else if (dtype == RI_BF16)
        rc = am_launch<bf16_t>((const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)kc, (const bf16_t*)vc, table, max_blocks, cu_q, q_start, kv_lens, num_rows, T, H, Hkv, dk, dv, page, scale, window, vcos, vsin, v_interleaved, sink, keep, sig_bias, stream);
    else
        return ri_fail("ri_attention_window_mfma: unknown dtype %d", dtype);
    if (rc) return rc;
    RI_LAUNCHED("ri_attention_window_mfma");
    return 0;
}

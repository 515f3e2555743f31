// q/k bias + RoPE + KV-cache append, and decode attention over the step-indexed KV cache.
//
// Cache layout (HuginnStaticCache of the reference, recpre/raven_modeling_minimal.py:344-349):
// K, V = [n_slots, batch, n_heads, t_max, head_dim]; one head's positions are contiguous, so a
// workgroup streams [positions x head_dim] with 16-byte lane-contiguous loads.
//
// Attention kernel: a position occupies one row of 16 lanes (head_dim * sizeof(T) / 16 of them active,
// 12 for head_dim 96 in bf16); a wave covers 4 positions per load instruction and the 4 waves of a
// workgroup interleave, so each load step of a workgroup reads 16 consecutive positions of K and of V.
// Scores are reduced with DPP row operations; every 16-lane row runs its own online softmax (one max
// update per 4 positions) and the rows are merged through LDS.  Small batches split the positions over
// several workgroups and merge the partials in a second, tiny launch: a merge inside the kernel needs a
// device-scope fence per workgroup, which measured 10x slower on this part than the extra launch.

#include <math.h>

#include <atomic>

#include "raven_common.h"

namespace raven {

struct CacheView {
    void* k;
    void* v;
    int64_t slot_off;  // element offset of the slot: slot * batch * nh * t_max * hd
    int batch, nh, t_max, hd;
    // partial fill (tokens computed with different numbers of recurrences): see raven_kv_cache in the header
    const int* steps_present;  // null: every position below the new rows is cached at this slot
    int lookup_mode;           // RAVEN_LOOKUP_*
    int core_step;             // slot's step index - 2 (>= 0 when steps_present is set)
    int64_t slot_stride;       // elements between two slots
};

// Where position p (older than the new rows) is read from when the slot holds core step `cs`: the element offset
// to add (a multiple of the slot stride), or `false` when the position takes no part.  sp = number of core steps
// cached for p.  The reference's loops over its dict cache (recpre/raven_modeling_minimal.py:206-253), for a
// cache whose positions each hold a prefix 2, 3, ... of the core steps:
//   latest-m4 / available-m4: the deepest cached step <= cs of the same block (same step index mod 4);
//   always-last-m4: the deepest cached step of the same block, also beyond cs;
//   skip, and `full` with gaps: positions that are not cached at this step are left out.
__device__ __forceinline__ bool lookup_source(const CacheView& cv, int p, int64_t* delta) {
    const int sp = cv.steps_present[p], cs = cv.core_step;
    *delta = 0;
    if (cv.lookup_mode != RAVEN_LOOKUP_ALWAYS_LAST && cs < sp) return true;
    if (cv.lookup_mode == RAVEN_LOOKUP_SKIP) return false;
    const int j = cs & 3;
    if (sp - 1 - j < 0) return false;  // the block never ran for this position (the host rejects such caches)
    const int src = j + ((sp - 1 - j) >> 2) * 4;
    *delta = (int64_t)(src - cs) * cv.slot_stride;
    return true;
}

// ------------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void qkv_rope_append_kernel(
    const T* __restrict__ qkv, const T* __restrict__ qk_bias, const float* __restrict__ freqs, T* __restrict__ q_out,
    CacheView cv, int S, int pos0, const int* __restrict__ pos_dev) {
    constexpr int E = Chunk<T>::N;
    const int h = cv.nh * cv.hd;
    const int chunks_per_sec = h / E;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= 3 * chunks_per_sec) return;
    const int m = blockIdx.y;
    const int b = m / S, s = m - b * S;
    const int pos = (pos_dev ? *pos_dev : pos0) + s;
    const int sec = c / chunks_per_sec;  // 0 q, 1 k, 2 v
    const int col = (c - sec * chunks_per_sec) * E;  // column inside the section
    const int head = col / cv.hd, d = col - head * cv.hd;

    Chunk<T> x = load_chunk(qkv + (int64_t)m * 3 * h + sec * h + col);
    if (sec < 2) {
        if (qk_bias) {
            const Chunk<T> bch = load_chunk(qk_bias + sec * h + col);
#pragma unroll
            for (int e = 0; e < E; ++e) x.v[e] = from_f32<T>(to_f32(x.v[e]) + to_f32(bch.v[e]));
        }
        const float* f = freqs + ((int64_t)pos * (cv.hd / 2) + d / 2) * 2;
#pragma unroll
        for (int e = 0; e < E; e += 2) rope_pair<T>(x.v[e], x.v[e + 1], f[e], f[e + 1]);
    }
    if (sec == 0) {
        store_chunk(q_out + (int64_t)m * h + col, x);
    } else if (pos < cv.t_max) {
        T* base = static_cast<T*>(sec == 1 ? cv.k : cv.v);
        const int64_t off = cv.slot_off + (((int64_t)b * cv.nh + head) * cv.t_max + pos) * cv.hd + d;
        store_chunk(base + off, x);
    }
}

// ------------------------------------------------------------------------------------------------
constexpr int kAttnMaxHd = 128;
}  // namespace raven
extern "C" size_t raven_decode_attention_workspace_bytes(int32_t M, int32_t n_heads, int32_t head_dim);
namespace raven {

// bias + RoPE of one 16-byte chunk of a q or k head row (sec 0 = q, 1 = k); d = first column of the chunk
template <typename T>
__device__ __forceinline__ Chunk<T> bias_rope_chunk(Chunk<T> x, const T* __restrict__ qk_bias, int sec, int h, int col,
                                                    const float* __restrict__ freqs, int pos, int hd, int d) {
    constexpr int E = Chunk<T>::N;
    if (qk_bias) {
        const Chunk<T> bch = load_chunk(qk_bias + sec * h + col);
#pragma unroll
        for (int e = 0; e < E; ++e) x.v[e] = from_f32<T>(to_f32(x.v[e]) + to_f32(bch.v[e]));
    }
    const float* f = freqs + ((int64_t)pos * (hd / 2) + d / 2) * 2;
#pragma unroll
    for (int e = 0; e < E; e += 2) rope_pair<T>(x.v[e], x.v[e + 1], f[e], f[e + 1]);
    return x;
}

// What one lane holds of a position's head row: CPL neighbouring 16-byte chunks (1, or 2 for fp32 heads wider than
// 64 elements, whose rows are more than 16 chunks long).
template <typename T, int CPL>
struct Piece {
    Chunk<T> c[CPL];
};
template <typename T, int CPL, bool STREAM = false>
__device__ __forceinline__ Piece<T, CPL> load_piece(const T* p) {
    Piece<T, CPL> r;
#pragma unroll
    for (int i = 0; i < CPL; ++i) r.c[i] = STREAM ? load_chunk_stream(p + i * Chunk<T>::N) : load_chunk(p + i * Chunk<T>::N);
    return r;
}
template <typename T, int CPL>
__device__ __forceinline__ void store_piece(T* p, const Piece<T, CPL>& v) {
#pragma unroll
    for (int i = 0; i < CPL; ++i) store_chunk(p + i * Chunk<T>::N, v.c[i]);
}
template <typename T, int CPL>
__device__ __forceinline__ Piece<T, CPL> zero_piece() {
    Piece<T, CPL> r;
#pragma unroll
    for (int i = 0; i < CPL; ++i) r.c[i] = zero_chunk<T>();
    return r;
}
template <typename T, int CPL>
__device__ __forceinline__ float dot_piece(const Piece<T, CPL>& a, const Piece<T, CPL>& b) {
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < CPL; ++i) acc = dot_chunk(a.c[i], b.c[i], acc);
    return acc;
}

// 2^x as the hardware instruction computes it (results below the smallest normal number come out as 0, which is what
// a softmax weight that small amounts to); exp2f() wraps the same instruction in a range reduction for denormal results
__device__ __forceinline__ float exp2_raw(float x) { return __builtin_amdgcn_exp2f(x); }

// Online-softmax state (running maximum, sum, unnormalised output) of a wave's four 16-lane rows merged into one, in
// registers; afterwards every row of the wave holds the merged state.
template <int E>
__device__ __forceinline__ void merge_wave_rows(float& m_run, float& l_run, float (&o)[E]) {
    float m4 = fmaxf(m_run, __shfl_xor(m_run, 16, 64));
    m4 = fmaxf(m4, __shfl_xor(m4, 32, 64));
    const float w = (m_run == -INFINITY) ? 0.f : exp2f(m_run - m4);
    float l4 = l_run * w;
    l4 += __shfl_xor(l4, 16, 64);
    l4 += __shfl_xor(l4, 32, 64);
#pragma unroll
    for (int e = 0; e < E; ++e) {
        float v = o[e] * w;
        v += __shfl_xor(v, 16, 64);
        v += __shfl_xor(v, 32, 64);
        o[e] = v;
    }
    m_run = m4;
    l_run = l4;
}

// Grid (heads, token rows, splits).  With one split a workgroup owns a whole (head, row) and writes y.
// With several (few heads x rows, i.e. small batches: one CU cannot pull a head's K/V fast enough) each
// workgroup covers a contiguous range of positions with all of its loads in flight at once and writes
// an fp32 partial (max, sum, unnormalised output); combine_kernel, the next launch on the stream, merges
// them -- the kernel boundary is the only synchronisation.  FUSED (decode, S == 1): q, and the new
// position's k and v, come straight from the fused qkv GEMM output -- bias and RoPE are applied here,
// the new k/v row is written to the cache by the workgroup whose range holds it and used from registers.
// LOOKUP: some older positions are not cached at this slot (cv.steps_present says which).
// G = 16-lane rows per workgroup (16 x G threads): 16, or 64 for the variant that gives a whole (head, row) to one
// workgroup of 1024 threads whose every load is in flight at once -- what the split launch achieves with several
// workgroups and a second launch, without that launch.
// Waves per SIMD the register budget is held to: with a second tile in flight the 2-position variant must still hold the
// 1760 workgroups of 32 rows x 55 heads at once (7 waves = 72 registers).
template <typename T, bool FUSED, int kAttnU, bool LOOKUP = false, int CPL = 1, int G = 16, bool PF = false>
__global__ __launch_bounds__(16 * G, (G == 16 && kAttnU == 2 && CPL == 1 && PF) ? 7 : 4) void decode_attention_kernel(
    const T* __restrict__ q_or_qkv, const T* __restrict__ qk_bias, const float* __restrict__ freqs, T* __restrict__ y,
    CacheView cv, int S, int pos0, const int* __restrict__ pos_dev, float scale_log2, int n_splits,
    float* __restrict__ ws_ml, float* __restrict__ ws_o) {
    constexpr int EC = Chunk<T>::N;   // elements per 16-byte chunk
    constexpr int E = EC * CPL;       // elements per lane and position
    // kAttnU = positions per 16-lane row and loop iteration: 4 when a few workgroups must each keep many loads
    // in flight, 2 when the grid is large and register pressure decides how many workgroups a CU holds
    __shared__ float sm_m[G / 4], sm_l[G / 4];  // one entry per wave
    __shared__ float sm_o[G / 4][kAttnMaxHd];

    const int head = blockIdx.x, m = blockIdx.y, split = blockIdx.z;
    const int hd = cv.hd, h = cv.nh * hd;
    const int b = m / S, s = m - b * S;
    const int first_new = pos_dev ? *pos_dev : pos0;
    const int pos = first_new + s;  // position of this row's own token
    const int len = min(pos + 1, cv.t_max);
    const int per = (len + n_splits - 1) / n_splits;
    const int start = split * per, end = min(len, start + per);

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane >> 4, ci = lane & 15;
    const int cp = hd / E;  // chunks per position
    const bool active = ci < cp;
    const int group = wave * 4 + r;

    const int64_t head_off = cv.slot_off + ((int64_t)b * cv.nh + head) * cv.t_max * hd;
    const T* Kb = static_cast<const T*>(cv.k) + head_off + ci * E;
    const T* Vb = static_cast<const T*>(cv.v) + head_off + ci * E;

    // q (and the new k, v) first: these loads are the oldest, so their data is back before the K/V tiles
    typedef Piece<T, CPL> P;
    P qraw = zero_piece<T, CPL>(), kraw = zero_piece<T, CPL>(), vnew = zero_piece<T, CPL>();
    // FUSED: the bias chunks and the (cos, sin) pairs of the row's position as well -- requested behind the tiles they would
    // return behind them, and the rotation of q would wait for every tile load in flight
    P bias_q = zero_piece<T, CPL>(), bias_k = zero_piece<T, CPL>();
    alignas(16) float cs[FUSED ? E : 1];
    const int col = head * hd + ci * E;
    if (active) {
        if (FUSED) {
            const T* row = q_or_qkv + (int64_t)m * 3 * h;
            qraw = load_piece<T, CPL>(row + col);
            kraw = load_piece<T, CPL>(row + h + col);
            vnew = load_piece<T, CPL>(row + 2 * h + col);
            if (qk_bias) {
                bias_q = load_piece<T, CPL>(qk_bias + col);
                bias_k = load_piece<T, CPL>(qk_bias + h + col);
            }
            const float* f = freqs + ((int64_t)pos * (hd / 2) + ci * E / 2) * 2;
#pragma unroll
            for (int e = 0; e < E; e += 4) *reinterpret_cast<f32x4*>(&cs[FUSED ? e : 0]) = *reinterpret_cast<const f32x4*>(f + e);
        } else {
            qraw = load_piece<T, CPL>(q_or_qkv + (int64_t)m * h + col);
        }
    }
    // K/V tiles: kAttnU positions per 16-lane row.  Without lookups every load of a tile is unconditional, so that all
    // of them are in flight before the first is waited for (a load under a per-lane condition makes the compiler wait for
    // it inside the conditional block, one position after the other): positions past the range read the last position
    // that is certainly cached instead, lanes past the head row's chunks repeat its last chunk (their q is zero), and the
    // scores of such positions are masked below.  FUSED: the row's own position, the last one, is not read at all; it is
    // added from registers behind the loop.
    struct Tile {
        P k[kAttnU], v[kAttnU];
        bool left_out[kAttnU];  // LOOKUP: the position takes no part
    };
    const int end_c = FUSED ? min(end, pos) : end;       // end of the cached positions of this range
    const int last_ok = max((FUSED ? pos : len) - 1, 0);  // initialised whenever a tile is consumed at all (then end_c >= 1)
    const T* Kh = static_cast<const T*>(cv.k) + head_off;
    const T* Vh = static_cast<const T*>(cv.v) + head_off;
    const unsigned lane_off = (unsigned)(min(ci, cp - 1) * E);
    auto load_tile = [&](int base, Tile& t) {
#pragma unroll
        for (int j = 0; j < kAttnU; ++j) {
            const int p = base + j * G + group;
            if constexpr (LOOKUP) {
                int64_t delta = 0;
                t.left_out[j] = false;
                if (cv.steps_present != nullptr && p < end_c && p < first_new) t.left_out[j] = !lookup_source(cv, p, &delta);
                if (active && p < end_c && !t.left_out[j]) {
                    t.k[j] = load_piece<T, CPL, kAttnU == 2>(Kb + delta + (int64_t)p * hd);
                    t.v[j] = load_piece<T, CPL, kAttnU == 2>(Vb + delta + (int64_t)p * hd);
                } else {
                    t.k[j] = zero_piece<T, CPL>();
                    t.v[j] = zero_piece<T, CPL>();
                }
            } else {
                // large grids (the 2-position variant) stream K/V past the caches: +8 % at batch 32; small ones do not gain
                // a 32-bit byte offset from the workgroup's (uniform) head row: scalar base + vector offset addressing
                const unsigned off = ((unsigned)min(p, last_ok) * (unsigned)hd + lane_off) * (unsigned)sizeof(T);
                t.k[j] = load_piece<T, CPL, kAttnU == 2>(reinterpret_cast<const T*>(reinterpret_cast<const char*>(Kh) + off));
                t.v[j] = load_piece<T, CPL, kAttnU == 2>(reinterpret_cast<const T*>(reinterpret_cast<const char*>(Vh) + off));
                t.left_out[j] = false;
            }
        }
    };
    Tile ta, tb;
    load_tile(start, ta);  // requested before q is touched
    if constexpr (PF && !LOOKUP) load_tile(start + G * kAttnU, tb);  // and so is the second tile: bias and RoPE of q take a few memory latencies

    P qc = qraw, knew = kraw;
    if (FUSED && active) {
#pragma unroll
        for (int i = 0; i < CPL; ++i) {  // the arithmetic of bias_rope_chunk, on operands loaded above
            if (qk_bias) {
#pragma unroll
                for (int e = 0; e < EC; ++e) {
                    qc.c[i].v[e] = from_f32<T>(to_f32(qraw.c[i].v[e]) + to_f32(bias_q.c[i].v[e]));
                    knew.c[i].v[e] = from_f32<T>(to_f32(kraw.c[i].v[e]) + to_f32(bias_k.c[i].v[e]));
                }
            }
#pragma unroll
            for (int e = 0; e < EC; e += 2) {
                rope_pair<T>(qc.c[i].v[e], qc.c[i].v[e + 1], cs[FUSED ? i * EC + e : 0], cs[FUSED ? i * EC + e + 1 : 0]);
                rope_pair<T>(knew.c[i].v[e], knew.c[i].v[e + 1], cs[FUSED ? i * EC + e : 0], cs[FUSED ? i * EC + e + 1 : 0]);
            }
        }
        if (group == 0 && pos >= start && pos < end) {
            store_piece<T, CPL>(static_cast<T*>(cv.k) + head_off + (int64_t)pos * hd + ci * E, knew);
            store_piece<T, CPL>(static_cast<T*>(cv.v) + head_off + (int64_t)pos * hd + ci * E, vnew);
        }
    }

    float m_run = -INFINITY, l_run = 0.f, o[E];
#pragma unroll
    for (int e = 0; e < E; ++e) o[e] = 0.f;

    auto consume = [&](int base, const Tile& t) {
        float sc[kAttnU], m_new = m_run;
#pragma unroll
        for (int j = 0; j < kAttnU; ++j) {
            const int p = base + j * G + group;
            sc[j] = row16_sum(dot_piece<T, CPL>(qc, t.k[j])) * scale_log2;
            if (p >= end_c || (LOOKUP && t.left_out[j])) sc[j] = -INFINITY;
            m_new = fmaxf(m_new, sc[j]);
        }
        if (m_new == -INFINITY) return;  // this row has not seen a valid position yet
        const float corr = exp2_raw(m_run - m_new);
        float pe[kAttnU], psum = 0.f;
#pragma unroll
        for (int j = 0; j < kAttnU; ++j) {
            pe[j] = exp2_raw(sc[j] - m_new);
            psum += pe[j];
        }
        l_run = l_run * corr + psum;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            float acc = o[e] * corr;
#pragma unroll
            for (int j = 0; j < kAttnU; ++j) acc = __builtin_fmaf(pe[j], to_f32(t.v[j].c[e / EC].v[e % EC]), acc);
            o[e] = acc;
        }
        m_run = m_new;
    };
    constexpr int STEP = G * kAttnU;
    if constexpr (PF && !LOOKUP) {
        // two tiles in turn, each requested again as soon as it is used, the first two in front of everything else; always
        // whole pairs (a tile past the range re-reads cached lines and adds nothing), so that the number of loads in flight
        // is the same on every path and the waits can leave the younger tile's loads outstanding
        for (int base = start; base < end_c; base += 2 * STEP) {  // trip count is uniform over the workgroup
            consume(base, ta);
            load_tile(base + 2 * STEP, ta);
            consume(base + STEP, tb);
            load_tile(base + 3 * STEP, tb);
        }
    } else {
        for (int base = start; base < end_c;) {
            consume(base, ta);
            base += STEP;
            if (base < end_c) load_tile(base, ta);
        }
    }
    if (FUSED && group == 0 && pos >= start && pos < end) {  // the row's own position, from registers
        const float sc = row16_sum(dot_piece<T, CPL>(qc, knew)) * scale_log2;
        const float m_new = fmaxf(m_run, sc);
        const float corr = exp2_raw(m_run - m_new), pe = exp2_raw(sc - m_new);
        l_run = l_run * corr + pe;
#pragma unroll
        for (int e = 0; e < E; ++e) o[e] = __builtin_fmaf(pe, to_f32(vnew.c[e / EC].v[e % EC]), o[e] * corr);
        m_run = m_new;
    }

    // merge: first the wave's four 16-lane rows in registers, then the waves through LDS
    merge_wave_rows<E>(m_run, l_run, o);
    if (r == 0) {
        if (ci == 0) {
            sm_m[wave] = m_run;
            sm_l[wave] = l_run;
        }
        if (active) {
#pragma unroll
            for (int e = 0; e < E; ++e) sm_o[wave][ci * E + e] = o[e];
        }
    }
    __syncthreads();
    const int t = threadIdx.x;
    if (t < hd) {
        float M = -INFINITY, L = 0.f, O = 0.f;
#pragma unroll
        for (int g = 0; g < G / 4; ++g) M = fmaxf(M, sm_m[g]);
#pragma unroll
        for (int g = 0; g < G / 4; ++g) {
            const float wgt = (sm_m[g] == -INFINITY) ? 0.f : exp2f(sm_m[g] - M);
            L += sm_l[g] * wgt;
            O += sm_o[g][t] * wgt;
        }
        if (n_splits == 1) {
            y[(int64_t)m * h + head * hd + t] = from_f32<T>(O / L);
        } else {
            const int64_t idx = ((int64_t)m * cv.nh + head) * n_splits + split;
            ws_o[idx * hd + t] = O;
            if (t == 0) {
                ws_ml[idx * 2] = M;
                ws_ml[idx * 2 + 1] = L;
            }
        }
    }
}

// y[m, head] = sum_s w_s O_s / sum_s w_s L_s with w_s = 2^(M_s - max M); grid (heads, rows), 128 threads (hd <= 128).
// The launch is all latency, so every load is requested at once: thread t < n_splits fetches split t's (M, L) pair while
// every thread fetches its column of all partial outputs (32 loads in flight; splits past n_splits repeat the last one and
// get weight 0).  The sums then run over the splits in order, out of LDS and registers.
constexpr int kCombineSplits = 32;  // = kAttnMaxSplits, the most a launch is split into
// NS: the splits a thread holds in registers, 8 / 16 / 32 >= n_splits
template <typename T, int NS>
__global__ __launch_bounds__(128) void attention_combine_kernel(const float* __restrict__ ws_ml, const float* __restrict__ ws_o,
                                                                T* __restrict__ y, int nh, int hd, int n_splits) {
    __shared__ float sm_m[kCombineSplits], sm_l[kCombineSplits];
    const int head = blockIdx.x, m = blockIdx.y, t = threadIdx.x;
    const int64_t mh = (int64_t)m * nh + head;
    if (t < n_splits) {
        const float2 ml = *reinterpret_cast<const float2*>(ws_ml + (mh * n_splits + t) * 2);
        sm_m[t] = ml.x;
        sm_l[t] = ml.y;
    }
    float o[NS];
    const int col = t < hd ? t : hd - 1;
#pragma unroll
    for (int sp = 0; sp < NS; ++sp) o[sp] = ws_o[(mh * n_splits + min(sp, n_splits - 1)) * hd + col];
    __syncthreads();
    if (t >= hd) return;
    float Mg = -INFINITY;
    for (int sp = 0; sp < n_splits; ++sp) Mg = fmaxf(Mg, sm_m[sp]);
    float Lg = 0.f, Og = 0.f;
#pragma unroll
    for (int sp = 0; sp < NS; ++sp) {
        if (sp < n_splits) {
            const float ms = sm_m[sp];
            const float wgt = (ms == -INFINITY) ? 0.f : exp2f(ms - Mg);
            Lg += sm_l[sp] * wgt;
            Og += o[sp] * wgt;
        }
    }
    y[(int64_t)m * nh * hd + head * hd + t] = from_f32<T>(Lg > 0.f ? Og / Lg : 0.f);  // no position at all (an empty paged sequence): zeros
}

template <typename T>
static void launch_combine(const float* ws_ml, const float* ws_o, T* y, int nh, int hd, int rows, int n_splits, hipStream_t s) {
    const dim3 grid(nh, rows), block(128);
    if (n_splits <= 8) attention_combine_kernel<T, 8><<<grid, block, 0, s>>>(ws_ml, ws_o, y, nh, hd, n_splits);
    else if (n_splits <= 16) attention_combine_kernel<T, 16><<<grid, block, 0, s>>>(ws_ml, ws_o, y, nh, hd, n_splits);
    else attention_combine_kernel<T, kCombineSplits><<<grid, block, 0, s>>>(ws_ml, ws_o, y, nh, hd, n_splits);
}

// ------------------------------------------------------------------------------------------------
// Paged KV cache (the layout vLLM's attention layer owns): K and V are [num_blocks, block_size, n_heads, head_dim];
// a sequence's position p lives in block block_table[seq][p / block_size] at offset p % block_size, and every
// sequence has its own length.  One new query row per sequence (decode).  Same arithmetic as decode_attention_kernel:
// 16 lanes per position, online softmax per 16-lane row, rows merged through LDS, splits merged by
// attention_combine_kernel.
// ------------------------------------------------------------------------------------------------
struct PagedView {
    const void* k;
    const void* v;
    const int* block_table;  // [B, max_blocks]
    const int* seq_lens;     // [B]: positions to attend to, the new token's own included
    int max_blocks, block_size, nh, hd;
    int block_shift;         // log2(block_size), or -1 when it is not a power of two
    int64_t pos_stride;      // elements between two positions of a block: nh * hd (RAVEN_PAGED_NHD) or hd (RAVEN_PAGED_HND)
    int64_t head_stride;     // elements between two heads: hd (NHD) or block_size * hd (HND)
};

// FUSED: q_or_qkv is the fused projection's output [B, 3 * h]; bias and RoPE (row seq_lens[b] - 1 of the table) are
// applied here, the new position's k / v row is written to its page by the workgroup whose range holds it and used
// from registers (the paged counterpart of decode_attention_kernel<FUSED>).
template <typename T, int CPL, bool FUSED = false>
__global__ __launch_bounds__(256) void paged_decode_attention_kernel(const T* __restrict__ q_or_qkv, const T* __restrict__ qk_bias,
                                                                     const float* __restrict__ freqs, T* __restrict__ y, PagedView pv,
                                                                     float scale_log2, int n_splits, float* __restrict__ ws_ml,
                                                                     float* __restrict__ ws_o) {
    constexpr int EC = Chunk<T>::N, E = EC * CPL, G = 16, U = 2;
    __shared__ float sm_m[G / 4], sm_l[G / 4];
    __shared__ float sm_o[G / 4][kAttnMaxHd];
    typedef Piece<T, CPL> P;
    const int head = blockIdx.x, b = blockIdx.y, split = blockIdx.z;
    const int hd = pv.hd, h = pv.nh * hd;
    const int len = pv.seq_lens[b];
    const int per = (len + n_splits - 1) / n_splits;
    const int start = split * per, end = min(len, start + per);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane >> 4, ci = lane & 15;
    const bool active = ci < hd / E;
    const int group = wave * 4 + r;
    const int* table = pv.block_table + (int64_t)b * pv.max_blocks;
    const T* K = static_cast<const T*>(pv.k);
    const T* V = static_cast<const T*>(pv.v);
    const int col = head * hd + ci * E;
    const int pos = len - 1;  // FUSED: the new token's position
    // this workgroup's part of the block table, read once: the loop's addresses then depend on LDS only
    constexpr int kTbl = 1024;
    __shared__ int tbl[kTbl];
    auto block_of = [&](int p) { return pv.block_shift >= 0 ? p >> pv.block_shift : p / pv.block_size; };
    auto offset_of = [&](int p) { return pv.block_shift >= 0 ? p & (pv.block_size - 1) : p % pv.block_size; };
    const int blk0 = block_of(start);
    if (start < end) {
        const int n_blk = block_of(end - 1) - blk0 + 1;
        for (int i = threadIdx.x; i < min(n_blk, kTbl); i += 256) tbl[i] = table[blk0 + i];
    }
    __syncthreads();
    const int64_t blk_stride = (int64_t)pv.block_size * pv.nh * hd;
    const int64_t lane_off = head * pv.head_stride + min(ci, hd / E - 1) * E;  // lanes past the head row repeat its last chunk (their q is zero)
    auto elem_of = [&](int p) {  // this lane's first element of position p
        const int i = block_of(p) - blk0;
        const int blk = i < kTbl ? tbl[i] : table[blk0 + i];
        return (int64_t)blk * blk_stride + offset_of(p) * pv.pos_stride + lane_off;
    };
    P qc = zero_piece<T, CPL>(), knew = zero_piece<T, CPL>(), vnew = zero_piece<T, CPL>();
    if (active && !FUSED) qc = load_piece<T, CPL>(q_or_qkv + (int64_t)b * h + col);
    if (FUSED && active && len > 0) {
        const T* row = q_or_qkv + (int64_t)b * 3 * h;
        qc = load_piece<T, CPL>(row + col);
        knew = load_piece<T, CPL>(row + h + col);
        vnew = load_piece<T, CPL>(row + 2 * h + col);
#pragma unroll
        for (int i = 0; i < CPL; ++i) {
            qc.c[i] = bias_rope_chunk<T>(qc.c[i], qk_bias, 0, h, col + i * EC, freqs, pos, hd, ci * E + i * EC);
            knew.c[i] = bias_rope_chunk<T>(knew.c[i], qk_bias, 1, h, col + i * EC, freqs, pos, hd, ci * E + i * EC);
        }
        if (group == 0 && pos >= start && pos < end) {
            const int64_t off = elem_of(pos);
            store_piece<T, CPL>(const_cast<T*>(K) + off, knew);
            store_piece<T, CPL>(const_cast<T*>(V) + off, vnew);
        }
    }

    float m_run = -INFINITY, l_run = 0.f, o[E];
#pragma unroll
    for (int e = 0; e < E; ++e) o[e] = 0.f;
    // As in decode_attention_kernel: every load of a tile is unconditional (positions past the cached ones of this range
    // re-read the range's last cached position, and their scores are masked), so that all of a tile's loads are in
    // flight before the first is waited for; FUSED: the new token's own position is added from registers behind the loop.
    const int end_c = FUSED ? min(end, pos) : end;
    const int last_ok = end_c - 1;  // inside this workgroup's range, so that its page is among the staged table entries
    for (int base = start; base < end_c; base += G * U) {  // trip count is uniform over the workgroup
        P kc[U], vc[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int64_t off = elem_of(min(base + j * G + group, last_ok));
            kc[j] = load_piece<T, CPL, true>(K + off);
            vc[j] = load_piece<T, CPL, true>(V + off);
        }
        float sc[U], m_new = m_run;
#pragma unroll
        for (int j = 0; j < U; ++j) {
            sc[j] = row16_sum(dot_piece<T, CPL>(qc, kc[j])) * scale_log2;
            if (base + j * G + group >= end_c) sc[j] = -INFINITY;
            m_new = fmaxf(m_new, sc[j]);
        }
        if (m_new == -INFINITY) continue;
        const float corr = exp2_raw(m_run - m_new);
        float pe[U], psum = 0.f;
#pragma unroll
        for (int j = 0; j < U; ++j) {
            pe[j] = exp2_raw(sc[j] - m_new);
            psum += pe[j];
        }
        l_run = l_run * corr + psum;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            float acc = o[e] * corr;
#pragma unroll
            for (int j = 0; j < U; ++j) acc = __builtin_fmaf(pe[j], to_f32(vc[j].c[e / EC].v[e % EC]), acc);
            o[e] = acc;
        }
        m_run = m_new;
    }
    if (FUSED && group == 0 && len > 0 && pos >= start && pos < end) {  // the new token's own position, from registers
        const float sc = row16_sum(dot_piece<T, CPL>(qc, knew)) * scale_log2;
        const float m_new = fmaxf(m_run, sc);
        const float corr = exp2_raw(m_run - m_new), pe = exp2_raw(sc - m_new);
        l_run = l_run * corr + pe;
#pragma unroll
        for (int e = 0; e < E; ++e) o[e] = __builtin_fmaf(pe, to_f32(vnew.c[e / EC].v[e % EC]), o[e] * corr);
        m_run = m_new;
    }
    merge_wave_rows<E>(m_run, l_run, o);
    if (r == 0) {
        if (ci == 0) {
            sm_m[wave] = m_run;
            sm_l[wave] = l_run;
        }
        if (active) {
#pragma unroll
            for (int e = 0; e < E; ++e) sm_o[wave][ci * E + e] = o[e];
        }
    }
    __syncthreads();
    const int t = threadIdx.x;
    if (t < hd) {
        float M = -INFINITY, L = 0.f, O = 0.f;
#pragma unroll
        for (int g = 0; g < G / 4; ++g) M = fmaxf(M, sm_m[g]);
#pragma unroll
        for (int g = 0; g < G / 4; ++g) {
            const float wgt = (sm_m[g] == -INFINITY) ? 0.f : exp2f(sm_m[g] - M);
            L += sm_l[g] * wgt;
            O += sm_o[g][t] * wgt;
        }
        if (n_splits == 1) {
            y[(int64_t)b * h + head * hd + t] = from_f32<T>(L > 0.f ? O / L : 0.f);  // an empty sequence gives zeros
        } else {
            const int64_t idx = ((int64_t)b * pv.nh + head) * n_splits + split;
            ws_o[idx * hd + t] = O;
            if (t == 0) {
                ws_ml[idx * 2] = M;
                ws_ml[idx * 2 + 1] = L;
            }
        }
    }
}

// cache[slot_mapping[t]] = row t, for K and V: rows of [n_heads * head_dim] elements; negative slots are skipped.
// slot = block * block_size + offset; pos_stride / head_stride as in PagedView.
template <typename T>
__global__ __launch_bounds__(256) void paged_kv_append_kernel(const T* __restrict__ k, const T* __restrict__ v, T* __restrict__ kc,
                                                              T* __restrict__ vc, const int64_t* __restrict__ slots, int h, int hd,
                                                              int block_size, int64_t pos_stride, int64_t head_stride) {
    constexpr int E = Chunk<T>::N;
    const int t = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
    const int64_t slot = slots[t];
    if (c >= h / E || slot < 0) return;
    const int64_t blk = slot / block_size, off = slot - blk * block_size;
    const int head = c * E / hd, d = c * E - head * hd;
    const int64_t dst = blk * block_size * h + off * pos_stride + head * head_stride + d;
    store_chunk(kc + dst, load_chunk(k + (int64_t)t * h + c * E));
    store_chunk(vc + dst, load_chunk(v + (int64_t)t * h + c * E));
}

// Rows of a fused projection [T, 3 * h] on their way into block-paged caches: q and k get the bias and the rotation of
// their own position (positions[t], any order -- rows of several sequences in one launch), q goes to q_out [T, h], k and
// v to slot slots[t] of the pages (negative slot: not stored).  blockIdx.z = 0 / 1 / 2 for q / k / v.
template <typename T>
__global__ __launch_bounds__(256) void paged_qkv_rope_append_kernel(const T* __restrict__ qkv, const T* __restrict__ qk_bias,
                                                                    const float* __restrict__ freqs, const int64_t* __restrict__ positions,
                                                                    const int64_t* __restrict__ slots, T* __restrict__ q_out,
                                                                    T* __restrict__ kc, T* __restrict__ vc, int h, int hd, int block_size,
                                                                    int64_t pos_stride, int64_t head_stride) {
    constexpr int E = Chunk<T>::N;
    const int t = blockIdx.y, sec = blockIdx.z, c = blockIdx.x * 256 + threadIdx.x;
    if (c >= h / E) return;
    const int col = c * E, head = col / hd, d = col - head * hd;
    Chunk<T> x = load_chunk(qkv + (int64_t)t * 3 * h + (int64_t)sec * h + col);
    if (sec < 2) x = bias_rope_chunk<T>(x, qk_bias, sec, h, col, freqs, (int)positions[t], hd, d);
    if (sec == 0) {
        store_chunk(q_out + (int64_t)t * h + col, x);
        return;
    }
    const int64_t slot = slots[t];
    if (slot < 0) return;
    const int64_t blk = slot / block_size, off = slot - blk * block_size;
    store_chunk((sec == 1 ? kc : vc) + blk * block_size * h + off * pos_stride + head * head_stride + d, x);
}

constexpr int kAttnMaxSplits = 32;
static_assert(kAttnMaxSplits == kCombineSplits, "the merge kernel holds one partial output per split in registers");
int g_rope_tiled_rows = 16;       // chunk length from which the append kernel works on (head, 16 positions) tiles ("rope_tiled_rows")
int g_attn_nosplit_pairs = 165;   // (head, row) pairs from which a launch over the contiguous cache is never split ("attn_nosplit_pairs", at most 1024)
int g_attn_nosplit_len = 1536;    // cache positions up to which two rows and more are not split either ("attn_nosplit_len", 0 = off)
int g_attn_split_target = 1536;  // workgroups a split launch aims for (raven_set_tuning "attn_split_target"); 1536 beats 2048 by 2-6 us at 3..9 sequences
int g_attn_big_grid = 1280;      // workgroups from which the 2-positions-per-row variant is used ("attn_big_grid")
// Few (head, row) pairs and a short cache: one 1024-thread workgroup per pair instead of a split launch and its merge
// launch.  Alone the step is faster (bs=1, 513 positions: 11.5 us against 13.8; bs=4: 13.9 against 19.1; it loses beyond
// about 2000 positions and from 8 sequences on), inside a decoded token the gain does not show (bs=1: 18.9-19.1 ms per
// token either way; bs=4: -0.4 %), so it is off unless asked for.  "attn_wide" = longest cache it is used for, 0 = never.
int g_attn_wide = 0;
int g_attn_prefetch = 1;  // raven_set_tuning("attn_prefetch"): 0 = a decode-attention workgroup requests a tile only when it needs it

// Splits are worth their extra launch only while heads x rows cannot fill the chip.
// The contiguous cache's kernel (contiguous = true) has variants that keep two tiles of four positions per 16-lane row in
// flight, with which one workgroup per (head, row) beats a split launch and its merge launch (4.8 us) for two rows and
// more over caches of up to about 1500 positions.  Core iteration at 1024 positions, split / unsplit, ms: 2 sequences
// 0.682 / 0.679, 4: 0.710 / 0.699, 8: 0.770 / 0.768, 12: 0.824 / 0.810, 16: 0.900 / 0.881.  One sequence stays split:
// measured alone (cache partly held by the memory-side cache) the unsplit launch is 3 us faster, inside the iteration,
// whose slots stream from HBM, it is not (0.568 / 0.570 ms), and beyond 2000 positions the split wins clearly
// (2048: 17.2 / 19.7 us, 4090: 23.5 / 35.8 us per step; 2 sequences: 23.1 / 22.5 and 37.9 / 40.2).
static int splits_for(int M, int nh, int len_hint, bool contiguous = false) {
    if ((int64_t)M * nh >= (contiguous ? g_attn_nosplit_pairs : 1024)) return 1;
    if (contiguous && M >= 2 && len_hint <= g_attn_nosplit_len) return 1;
    int ns = (len_hint + 63) / 64;  // 64 positions per workgroup keeps every load in one round trip
    const int cap = (g_attn_split_target + M * nh - 1) / (M * nh);
    if (ns > cap) ns = cap;
    if (ns > kAttnMaxSplits) ns = kAttnMaxSplits;
    return ns < 1 ? 1 : ns;
}

static int make_view(const char* who, const raven_kv_cache* cache, int slot, int B, int nh, int hd, CacheView* cv) {
    RAVEN_REQUIRE(cache && cache->k && cache->v, "%s: null cache", who);
    RAVEN_REQUIRE(cache->n_slots > 0 && cache->t_max > 0 && cache->batch > 0, "%s: empty cache", who);
    RAVEN_REQUIRE(B <= cache->batch, "%s: batch %d exceeds the cache's %d", who, B, cache->batch);
    const int sl = slot >= 0 ? slot : cache->n_slots + slot;
    RAVEN_REQUIRE(sl >= 0 && sl < cache->n_slots, "%s: slot %d outside [0, %d)", who, slot, cache->n_slots);
    cv->k = cache->k;
    cv->v = cache->v;
    cv->batch = cache->batch;
    cv->nh = nh;
    cv->t_max = cache->t_max;
    cv->hd = hd;
    cv->slot_stride = (int64_t)cache->batch * nh * cache->t_max * hd;
    cv->slot_off = (int64_t)sl * cv->slot_stride;
    cv->steps_present = nullptr;
    cv->lookup_mode = RAVEN_LOOKUP_NONE;
    cv->core_step = sl - cache->core_slot0;
    if (cache->steps_present != nullptr && cache->lookup_mode != RAVEN_LOOKUP_NONE && cv->core_step >= 0) {
        RAVEN_REQUIRE(cache->lookup_mode >= RAVEN_LOOKUP_SKIP && cache->lookup_mode <= RAVEN_LOOKUP_ALWAYS_LAST,
                      "%s: unknown lookup mode %d", who, cache->lookup_mode);
        RAVEN_REQUIRE(cache->core_slot0 >= 0, "%s: core_slot0 %d", who, cache->core_slot0);
        cv->steps_present = cache->steps_present;
        cv->lookup_mode = cache->lookup_mode;
    }
    return 0;
}

static int check_heads(const char* who, int nh, int hd, int dtype) {
    RAVEN_REQUIRE(dtype == RAVEN_F32 || dtype == RAVEN_BF16, "%s: unknown dtype %d", who, dtype);
    const int elts = 16 / (int)raven_host::elt_size(dtype);
    RAVEN_REQUIRE(nh > 0 && hd > 0 && hd % elts == 0 && hd % 2 == 0, "%s: head_dim %d must be an even multiple of %d", who, hd, elts);
    RAVEN_REQUIRE(hd / elts <= 32 && hd <= kAttnMaxHd, "%s: head_dim %d too large for one 16-lane row", who, hd);
    RAVEN_REQUIRE(hd / elts <= 16 || hd % (2 * elts) == 0, "%s: head_dim %d must be a multiple of %d", who, hd, 2 * elts);
    return 0;
}

// The same for chunks of many positions: a workgroup takes one (section, head) and 64 consecutive positions, 16 lanes
// per position and four positions per lane (all four loads issued before the first is used), so that what it writes to
// the cache is one contiguous run of 64 head rows (the kernel above writes a token's heads to 55 places, one 192-byte
// piece each).  Grid (position tiles, 3 * heads, sequences).
template <typename T>
__global__ __launch_bounds__(256) void qkv_rope_append_tiled_kernel(
    const T* __restrict__ qkv, const T* __restrict__ qk_bias, const float* __restrict__ freqs, T* __restrict__ q_out,
    CacheView cv, int S, int pos0, const int* __restrict__ pos_dev) {
    constexpr int E = Chunk<T>::N, PPL = 4;
    const int h = cv.nh * cv.hd;
    const int s0 = blockIdx.x * 16 * PPL + (threadIdx.x >> 4), ci = threadIdx.x & 15;
    const int sec = blockIdx.y / cv.nh, head = blockIdx.y - sec * cv.nh;  // 0 q, 1 k, 2 v
    const int b = blockIdx.z;
    const int d = ci * E;
    if (d >= cv.hd) return;
    const int first = pos_dev ? *pos_dev : pos0;
    const int col = head * cv.hd + d;
    Chunk<T> x[PPL];
#pragma unroll
    for (int j = 0; j < PPL; ++j) {
        const int s = s0 + 16 * j;
        x[j] = s < S ? load_chunk(qkv + ((int64_t)b * S + s) * 3 * h + sec * h + col) : zero_chunk<T>();
    }
    if (sec < 2) {
        Chunk<T> bch = zero_chunk<T>();
        if (qk_bias) bch = load_chunk(qk_bias + sec * h + col);
#pragma unroll
        for (int j = 0; j < PPL; ++j) {
            const int s = min(s0 + 16 * j, S - 1);
            if (qk_bias) {
#pragma unroll
                for (int e = 0; e < E; ++e) x[j].v[e] = from_f32<T>(to_f32(x[j].v[e]) + to_f32(bch.v[e]));
            }
            const float* f = freqs + ((int64_t)(first + s) * (cv.hd / 2) + d / 2) * 2;
#pragma unroll
            for (int e = 0; e < E; e += 2) rope_pair<T>(x[j].v[e], x[j].v[e + 1], f[e], f[e + 1]);
        }
    }
#pragma unroll
    for (int j = 0; j < PPL; ++j) {
        const int s = s0 + 16 * j, pos = first + s;
        if (s >= S) continue;
        if (sec == 0) {
            store_chunk(q_out + ((int64_t)b * S + s) * h + col, x[j]);
        } else if (pos < cv.t_max) {
            T* base = static_cast<T*>(sec == 1 ? cv.k : cv.v);
            store_chunk(base + cv.slot_off + (((int64_t)b * cv.nh + head) * cv.t_max + pos) * cv.hd + d, x[j]);
        }
    }
}

}  // namespace raven

extern "C" int raven_qkv_bias_rope_cache_append(const void* qkv, const void* qk_bias, const float* freqs, void* q_out,
                                                const raven_kv_cache* cache, int32_t slot, int32_t B, int32_t S,
                                                int32_t pos0, const int32_t* pos_dev, int32_t n_heads, int32_t head_dim,
                                                int32_t dtype, void* stream) {
    using namespace raven;
    if (int rc = check_heads("qkv_append", n_heads, head_dim, dtype)) return rc;
    RAVEN_REQUIRE(qkv && freqs && q_out, "qkv_append: null pointer");
    RAVEN_REQUIRE(B > 0 && S > 0 && pos0 >= 0, "qkv_append: bad B=%d S=%d pos0=%d", B, S, pos0);
    CacheView cv;
    if (int rc = make_view("qkv_append", cache, slot, B, n_heads, head_dim, &cv)) return rc;
    RAVEN_REQUIRE(pos0 + S <= cv.t_max, "qkv_append: positions %d..%d exceed the cache length %d", pos0, pos0 + S - 1, cv.t_max);
    const int elts = 16 / (int)raven_host::elt_size(dtype);
    const int chunks = 3 * n_heads * head_dim / elts;
    dim3 grid((chunks + 255) / 256, B * S);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (S >= g_rope_tiled_rows && head_dim / elts <= 16 && B <= 65535 && 3 * n_heads <= 65535) {
        const dim3 tiles((S + 63) / 64, 3 * n_heads, B);
        if (dtype == RAVEN_BF16)
            qkv_rope_append_tiled_kernel<bf16><<<tiles, dim3(256), 0, s>>>((const bf16*)qkv, (const bf16*)qk_bias, freqs, (bf16*)q_out, cv, S, pos0, pos_dev);
        else
            qkv_rope_append_tiled_kernel<float><<<tiles, dim3(256), 0, s>>>((const float*)qkv, (const float*)qk_bias, freqs, (float*)q_out, cv, S, pos0, pos_dev);
        return raven_host::check_launch("qkv_append");
    }
    if (dtype == RAVEN_BF16)
        qkv_rope_append_kernel<bf16><<<grid, dim3(256), 0, s>>>((const bf16*)qkv, (const bf16*)qk_bias, freqs, (bf16*)q_out, cv, S, pos0, pos_dev);
    else
        qkv_rope_append_kernel<float><<<grid, dim3(256), 0, s>>>((const float*)qkv, (const float*)qk_bias, freqs, (float*)q_out, cv, S, pos0, pos_dev);
    return raven_host::check_launch("qkv_append");
}

namespace raven {
extern int g_tiled_min_rows;
bool tiled_gemm_fits(int M, int N, int K0, int K1, int dtype);
int tiled_gemm_qkv_rope(const void* x, const void* wqkv, const void* qk_bias, const float* freqs, void* q_out, void* k_cache,
                        void* v_cache, int64_t slot_off, int nh, int hd, int t_max, int M, int S, int K, int ldx, int pos0,
                        const int* pos_dev, hipStream_t s);
int g_fuse_qkv_rope = 1;  // raven_set_tuning("fuse_qkv_rope"): 0 = a chunk's q | k | v product is stored and rotated by a launch of its own

// A chunk's Wqkv product with raven_qkv_bias_rope_cache_append as its epilogue (bf16 shapes that take the tiled GEMM):
// *done = 0 and nothing launched when the shape does not take that path.  ldx: elements between two rows of x (0 = n_embd).
int qkv_linear_rope_append(const void* x, int ldx, const void* wqkv, const void* qk_bias, const float* freqs, void* q_out,
                           const raven_kv_cache* cache, int slot, int B, int S, int pos0, const int32_t* pos_dev, int n_heads,
                           int head_dim, int dtype, hipStream_t s, int* done) {
    *done = 0;
    const int M = B * S, h = n_heads * head_dim;
    if (!g_fuse_qkv_rope || dtype != RAVEN_BF16 || M < g_tiled_min_rows || head_dim % 8 != 0 || !tiled_gemm_fits(M, 3 * h, h, 0, dtype)) return 0;
    if (int rc = check_heads("qkv_append", n_heads, head_dim, dtype)) return rc;
    RAVEN_REQUIRE(x && wqkv && freqs && q_out, "qkv_append: null pointer");
    RAVEN_REQUIRE(B > 0 && S > 0 && pos0 >= 0, "qkv_append: bad B=%d S=%d pos0=%d", B, S, pos0);
    CacheView cv;
    if (int rc = make_view("qkv_append", cache, slot, B, n_heads, head_dim, &cv)) return rc;
    RAVEN_REQUIRE(pos0 + S <= cv.t_max, "qkv_append: positions %d..%d exceed the cache length %d", pos0, pos0 + S - 1, cv.t_max);
    *done = 1;
    return tiled_gemm_qkv_rope(x, wqkv, qk_bias, freqs, q_out, cv.k, cv.v, cv.slot_off, cv.nh, cv.hd, cv.t_max, M, S, h, ldx, pos0, pos_dev, s);
}
}  // namespace raven

template <typename T>
static void launch_attention(bool fused, const void* q, const void* bias, const float* freqs, void* y, const raven::CacheView& cv,
                             int S, int M, int pos0, const int32_t* pos_dev, float scale_log2, int ns, float* ws_ml, float* ws_o,
                             bool wide, hipStream_t s) {
    using namespace raven;
    if (wide) {  // one 1024-thread workgroup per (head, row), 384 positions per round trip, no second launch
        constexpr int WIDE_G = 64, WIDE_U = 6;  // 6 positions per 16-lane row: what 128 registers per lane hold without spilling
        const dim3 g1(cv.nh, M, 1);
        decode_attention_kernel<T, true, WIDE_U, false, 1, WIDE_G><<<g1, dim3(16 * WIDE_G), 0, s>>>((const T*)q, (const T*)bias, freqs, (T*)y, cv, S, pos0,
                                                                                   pos_dev, scale_log2, 1, nullptr, nullptr);
        return;
    }
    const dim3 grid(cv.nh, M, ns);
    // the 2-positions-per-row variant streams K/V past the caches and keeps more workgroups per CU: it wins whenever
    // the launch is not split (512 or more (head, row) pairs), and for split launches from g_attn_big_grid workgroups on
    const bool big = ns == 1 ? (int64_t)cv.nh * M >= 512 : (int64_t)cv.nh * M * ns >= g_attn_big_grid;
    const T* bias_t = (const T*)bias;
#define RAVEN_ATTN_LAUNCH(FUSED_, U_, LOOKUP_, PF_)                                                                       \
    decode_attention_kernel<T, FUSED_, U_, LOOKUP_, 1, 16, PF_><<<grid, dim3(256), 0, s>>>((const T*)q, FUSED_ ? bias_t : nullptr, \
        FUSED_ ? freqs : nullptr, (T*)y, cv, S, pos0, pos_dev, scale_log2, ns, ws_ml, ws_o)
    // a workgroup that walks many tiles requests the next tile before it uses the current one (unsplit launches of 512
    // or more (head, row) pairs: 117.5 -> 114 us at 32 rows and 1024 positions; split launches, whose workgroups
    // walk a few tiles each, lose 8 % to the tile of the last pair that lies past the range)
    const int per = (pos0 + S + ns - 1) / ns;
    // ... and of fewer than 256 pairs; in between (256 .. 1023 pairs unsplit) requesting a tile only when it is needed is as
    // fast or faster (10 sequences x 1024 positions: 37.1 us against 42.0; 5: 24.7 against 27.9; 8, 14, 16, 18: equal)
    const int64_t pairs = (int64_t)cv.nh * M;
    const bool pf = g_attn_prefetch && (ns == 1 || g_attn_prefetch == 2) && per >= 8 * 16 * (big ? 2 : 4) &&
                    (g_attn_prefetch == 2 || ns > 1 || pairs < 256 || pairs >= 1024);
    if (cv.hd / Chunk<T>::N > 16) {  // fp32 heads wider than 64 elements: two chunks per lane, one variant per entry point
        if constexpr (sizeof(T) == 4) {
            if (fused) decode_attention_kernel<T, true, 2, true, 2><<<grid, dim3(256), 0, s>>>((const T*)q, bias_t, freqs, (T*)y, cv, S, pos0, pos_dev, scale_log2, ns, ws_ml, ws_o);
            else decode_attention_kernel<T, false, 2, true, 2><<<grid, dim3(256), 0, s>>>((const T*)q, nullptr, nullptr, (T*)y, cv, S, pos0, pos_dev, scale_log2, ns, ws_ml, ws_o);
        }
    } else if (cv.steps_present) {  // partial fill: rare, one variant per entry point
        if (fused) RAVEN_ATTN_LAUNCH(true, 2, true, false);
        else RAVEN_ATTN_LAUNCH(false, 2, true, false);
    } else if (fused) {
        if (big && pf) RAVEN_ATTN_LAUNCH(true, 2, false, true);
        else if (big) RAVEN_ATTN_LAUNCH(true, 2, false, false);
        else if (pf) RAVEN_ATTN_LAUNCH(true, 4, false, true);
        else RAVEN_ATTN_LAUNCH(true, 4, false, false);
    } else {
        if (big && pf) RAVEN_ATTN_LAUNCH(false, 2, false, true);
        else if (big) RAVEN_ATTN_LAUNCH(false, 2, false, false);
        else if (pf) RAVEN_ATTN_LAUNCH(false, 4, false, true);
        else RAVEN_ATTN_LAUNCH(false, 4, false, false);
    }
#undef RAVEN_ATTN_LAUNCH
    if (ns > 1) launch_combine<T>(ws_ml, ws_o, (T*)y, cv.nh, cv.hd, M, ns, s);
}

static int attention_common(const char* who, bool fused, const void* q, const void* bias, const float* freqs, void* y,
                            const raven_kv_cache* cache, int slot, int B, int S, int pos0, const int32_t* pos_dev, int n_heads,
                            int head_dim, int dtype, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace raven;
    if (int rc = check_heads(who, n_heads, head_dim, dtype)) return rc;
    RAVEN_REQUIRE(q && y, "%s: null pointer", who);
    RAVEN_REQUIRE(!fused || freqs, "%s: null RoPE table", who);
    RAVEN_REQUIRE(B > 0 && S > 0 && pos0 >= 0, "%s: bad B=%d S=%d pos0=%d", who, B, S, pos0);
    CacheView cv;
    if (int rc = make_view(who, cache, slot, B, n_heads, head_dim, &cv)) return rc;
    RAVEN_REQUIRE(pos0 + S <= cv.t_max, "%s: positions up to %d exceed the cache length %d", who, pos0 + S - 1, cv.t_max);
    const int M = B * S;
    RAVEN_REQUIRE(M <= 65535, "%s: too many token rows (%d)", who, M);
    const int elts = 16 / (int)raven_host::elt_size(dtype);
    // the variants for partially filled caches and for two chunks per lane keep one tile in flight: they split as before
    int ns = splits_for(M, n_heads, pos0 + S, !cv.steps_present && head_dim / elts <= 16);
    const bool wide = fused && ns > 1 && pos0 + S <= g_attn_wide && M * n_heads <= 256 && !cv.steps_present && head_dim / elts <= 16;
    if (wide) ns = 1;
    float *ws_ml = nullptr, *ws_o = nullptr;
    if (ns > 1) {
        const size_t need = raven_decode_attention_workspace_bytes(M, n_heads, head_dim);
        if (workspace == nullptr || workspace_bytes < need) {
            ns = 1;  // no room for partials: one workgroup per (head, row) still gives the same result
        } else {
            RAVEN_REQUIRE(((uintptr_t)workspace & 255) == 0, "%s: workspace must be 256-byte aligned", who);
            ws_ml = static_cast<float*>(workspace);
            ws_o = reinterpret_cast<float*>(static_cast<char*>(workspace) + raven_host::align_up((size_t)M * n_heads * kAttnMaxSplits * 2 * 4));
        }
    }
    const float scale_log2 = (float)(1.0 / sqrt((double)head_dim) * 1.4426950408889634);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == RAVEN_BF16) launch_attention<bf16>(fused, q, bias, freqs, y, cv, S, M, pos0, pos_dev, scale_log2, ns, ws_ml, ws_o, wide, s);
    else launch_attention<float>(fused, q, bias, freqs, y, cv, S, M, pos0, pos_dev, scale_log2, ns, ws_ml, ws_o, wide, s);
    return raven_host::check_launch(who);
}

extern "C" size_t raven_decode_attention_workspace_bytes(int32_t M, int32_t n_heads, int32_t head_dim) {
    using namespace raven;
    if (M <= 0 || n_heads <= 0 || head_dim <= 0) return 0;
    if ((int64_t)M * n_heads >= 1024) return 0;  // enough (head, row) pairs: never split
    const size_t mh = (size_t)M * n_heads;
    return raven_host::align_up(mh * kAttnMaxSplits * 2 * 4) + raven_host::align_up(mh * kAttnMaxSplits * head_dim * 4);
}

extern "C" int raven_decode_attention(const void* q, void* y, const raven_kv_cache* cache, int32_t slot, int32_t B,
                                      int32_t S, int32_t pos0, const int32_t* pos_dev, int32_t n_heads, int32_t head_dim,
                                      int32_t dtype, void* workspace, size_t workspace_bytes, void* stream) {
    return attention_common("decode_attention", false, q, nullptr, nullptr, y, cache, slot, B, S, pos0, pos_dev, n_heads, head_dim,
                            dtype, workspace, workspace_bytes, stream);
}

extern "C" int raven_qkv_attention_decode(const void* qkv, const void* qk_bias, const float* freqs, void* y,
                                          const raven_kv_cache* cache, int32_t slot, int32_t B, int32_t pos0,
                                          const int32_t* pos_dev, int32_t n_heads, int32_t head_dim, int32_t dtype,
                                          void* workspace, size_t workspace_bytes, void* stream) {
    return attention_common("qkv_attention_decode", true, qkv, qk_bias, freqs, y, cache, slot, B, 1, pos0, pos_dev, n_heads,
                            head_dim, dtype, workspace, workspace_bytes, stream);
}

// ---- the decode step without a caller's workspace --------------------------------------------------------------
// Partial results of a split launch (per (head, row) pair and split: running maximum, sum, unnormalised output) go to a
// buffer that is part of the loaded code object instead of an allocation: sized for the largest launch that is ever
// split (fewer than 1024 (head, row) pairs, kAttnMaxSplits splits, head_dim up to 128).  In host code the array's name
// is only a handle; its device address is looked up once per device.
constexpr size_t kScratchMaxPairs = 1023, kScratchMaxHeadDim = 128;
constexpr size_t kScratchBytes = ((kScratchMaxPairs * raven::kAttnMaxSplits * 2 * 4 + 255) / 256 * 256) +
                                 ((kScratchMaxPairs * raven::kAttnMaxSplits * kScratchMaxHeadDim * 4 + 255) / 256 * 256);
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kScratchMaxDevices = 64;
// per device: each GPU holds its own copy of the array at its own address.  Published atomically: two threads that race on
// a device's first call both look the address up and store the same value
static std::atomic<void*> g_scratch_ptr[kScratchMaxDevices];

extern "C" size_t raven_qkv_attention_decode_static_scratch_bytes(void) { return kScratchBytes; }

extern "C" int raven_qkv_attention_decode_static(const void* qkv, const void* qk_bias, const float* freqs, void* y,
                                                 const raven_kv_cache* cache, int32_t slot, int32_t B, int32_t pos0,
                                                 const int32_t* pos_dev, int32_t n_heads, int32_t head_dim, int32_t dtype,
                                                 void* stream) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kScratchMaxDevices) {
        raven_host::set_error("qkv_attention_decode_static: cannot tell the current device (%s, device %d of at most %d)",
                              hipGetErrorString(e), dev, kScratchMaxDevices);
        return e != hipSuccess ? (int)e : -1;
    }
    void* scratch_dev = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (scratch_dev == nullptr) {  // the first call on this device (make it outside a stream capture)
        e = hipGetSymbolAddress(&scratch_dev, HIP_SYMBOL(scratch));
        if (e != hipSuccess || scratch_dev == nullptr) {
            raven_host::set_error("qkv_attention_decode_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
            return e != hipSuccess ? (int)e : -1;
        }
        g_scratch_ptr[dev].store(scratch_dev, std::memory_order_release);
    }
    // the same size rule as raven_decode_attention_workspace_bytes; what would not fit the array is refused
    const size_t need = raven_decode_attention_workspace_bytes(B, n_heads, head_dim);
    RAVEN_REQUIRE(need <= kScratchBytes,
                  "qkv_attention_decode_static: %d sequences x %d heads of %d need %zu bytes of partial results, the built-in buffer holds %zu "
                  "(at most %zu (head, row) pairs in a split launch, head_dim up to %zu)",
                  B, n_heads, head_dim, need, kScratchBytes, kScratchMaxPairs, kScratchMaxHeadDim);
    return attention_common("qkv_attention_decode_static", true, qkv, qk_bias, freqs, y, cache, slot, B, 1, pos0, pos_dev, n_heads,
                            head_dim, dtype, scratch_dev, kScratchBytes, stream);
}


static int paged_strides(const char* who, int kv_layout, int block_size, int n_heads, int head_dim, int64_t* pos_stride, int64_t* head_stride) {
    RAVEN_REQUIRE(kv_layout == RAVEN_PAGED_NHD || kv_layout == RAVEN_PAGED_HND, "%s: unknown kv_layout %d", who, kv_layout);
    RAVEN_REQUIRE(block_size > 0, "%s: bad block_size %d", who, block_size);
    *pos_stride = kv_layout == RAVEN_PAGED_NHD ? (int64_t)n_heads * head_dim : head_dim;
    *head_stride = kv_layout == RAVEN_PAGED_NHD ? head_dim : (int64_t)block_size * head_dim;
    return 0;
}

extern "C" int raven_paged_kv_append(const void* k, const void* v, void* k_cache, void* v_cache, const int64_t* slot_mapping,
                                     int32_t T, int32_t n_heads, int32_t head_dim, int32_t block_size, int32_t kv_layout,
                                     int32_t dtype, void* stream) {
    using namespace raven;
    if (int rc = check_heads("paged_kv_append", n_heads, head_dim, dtype)) return rc;
    int64_t ps, hs;
    if (int rc = paged_strides("paged_kv_append", kv_layout, block_size, n_heads, head_dim, &ps, &hs)) return rc;
    RAVEN_REQUIRE(T >= 0 && T <= 65535, "paged_kv_append: bad row count %d", T);
    if (T == 0) return 0;
    RAVEN_REQUIRE(k && v && k_cache && v_cache && slot_mapping, "paged_kv_append: null pointer");
    const int h = n_heads * head_dim, elts = 16 / (int)raven_host::elt_size(dtype);
    const dim3 grid((h / elts + 255) / 256, T);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == RAVEN_BF16) paged_kv_append_kernel<bf16><<<grid, dim3(256), 0, s>>>((const bf16*)k, (const bf16*)v, (bf16*)k_cache, (bf16*)v_cache, slot_mapping, h, head_dim, block_size, ps, hs);
    else paged_kv_append_kernel<float><<<grid, dim3(256), 0, s>>>((const float*)k, (const float*)v, (float*)k_cache, (float*)v_cache, slot_mapping, h, head_dim, block_size, ps, hs);
    return raven_host::check_launch("paged_kv_append");
}

extern "C" int raven_paged_qkv_rope_append(const void* qkv, const void* qk_bias, const float* freqs, const int64_t* positions,
                                           const int64_t* slot_mapping, void* q_out, void* k_cache, void* v_cache, int32_t T,
                                           int32_t n_heads, int32_t head_dim, int32_t block_size, int32_t kv_layout, int32_t dtype,
                                           void* stream) {
    using namespace raven;
    if (int rc = check_heads("paged_qkv_rope_append", n_heads, head_dim, dtype)) return rc;
    int64_t ps, hs;
    if (int rc = paged_strides("paged_qkv_rope_append", kv_layout, block_size, n_heads, head_dim, &ps, &hs)) return rc;
    RAVEN_REQUIRE(T >= 0 && T <= 65535, "paged_qkv_rope_append: bad row count %d", T);
    if (T == 0) return 0;
    RAVEN_REQUIRE(qkv && freqs && positions && slot_mapping && q_out && k_cache && v_cache, "paged_qkv_rope_append: null pointer");
    const int h = n_heads * head_dim, elts = 16 / (int)raven_host::elt_size(dtype);
    const dim3 grid((h / elts + 255) / 256, T, 3);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == RAVEN_BF16)
        paged_qkv_rope_append_kernel<bf16><<<grid, dim3(256), 0, s>>>((const bf16*)qkv, (const bf16*)qk_bias, freqs, positions, slot_mapping,
                                                                      (bf16*)q_out, (bf16*)k_cache, (bf16*)v_cache, h, head_dim, block_size, ps, hs);
    else
        paged_qkv_rope_append_kernel<float><<<grid, dim3(256), 0, s>>>((const float*)qkv, (const float*)qk_bias, freqs, positions, slot_mapping,
                                                                       (float*)q_out, (float*)k_cache, (float*)v_cache, h, head_dim, block_size, ps, hs);
    return raven_host::check_launch("paged_qkv_rope_append");
}

static int paged_attention_common(const char* who, bool fused, const void* q, const void* bias, const float* freqs, void* y,
                                  const void* k_cache, const void* v_cache, const int32_t* block_table, const int32_t* seq_lens,
                                  int32_t B, int32_t max_blocks, int32_t block_size, int32_t kv_layout, int32_t max_seq_len,
                                  int32_t n_heads, int32_t head_dim, int32_t dtype, void* workspace, size_t workspace_bytes,
                                  void* stream) {
    using namespace raven;
    if (int rc = check_heads(who, n_heads, head_dim, dtype)) return rc;
    int64_t ps, hs;
    if (int rc = paged_strides(who, kv_layout, block_size, n_heads, head_dim, &ps, &hs)) return rc;
    RAVEN_REQUIRE(B >= 0 && B <= 65535 && max_blocks > 0 && block_size > 0 && max_seq_len > 0, "%s: bad B=%d max_blocks=%d block_size=%d max_seq_len=%d", who, B, max_blocks, block_size, max_seq_len);
    if (B == 0) return 0;
    RAVEN_REQUIRE(q && y && k_cache && v_cache && block_table && seq_lens, "%s: null pointer", who);
    RAVEN_REQUIRE(!fused || freqs, "%s: null RoPE table", who);
    RAVEN_REQUIRE((int64_t)max_blocks * block_size >= max_seq_len, "%s: %d blocks of %d cannot hold %d positions", who, max_blocks, block_size, max_seq_len);
    int ns = splits_for(B, n_heads, max_seq_len);
    float *ws_ml = nullptr, *ws_o = nullptr;
    if (ns > 1) {
        const size_t need = raven_decode_attention_workspace_bytes(B, n_heads, head_dim);
        if (workspace == nullptr || workspace_bytes < need) {
            ns = 1;
        } else {
            RAVEN_REQUIRE(((uintptr_t)workspace & 255) == 0, "%s: workspace must be 256-byte aligned", who);
            ws_ml = static_cast<float*>(workspace);
            ws_o = reinterpret_cast<float*>(static_cast<char*>(workspace) + raven_host::align_up((size_t)B * n_heads * kAttnMaxSplits * 2 * 4));
        }
    }
    int shift = -1;
    for (int b = 0; b < 31; ++b)
        if (block_size == (1 << b)) shift = b;
    PagedView pv{k_cache, v_cache, block_table, seq_lens, max_blocks, block_size, n_heads, head_dim, shift, ps, hs};
    const float scale_log2 = (float)(1.0 / sqrt((double)head_dim) * 1.4426950408889634);
    const dim3 grid(n_heads, B, ns);
    hipStream_t s = static_cast<hipStream_t>(stream);
#define RAVEN_PAGED_LAUNCH(T_, CPL_)                                                                                            \
    do {                                                                                                                        \
        if (fused) paged_decode_attention_kernel<T_, CPL_, true><<<grid, dim3(256), 0, s>>>((const T_*)q, (const T_*)bias, freqs, (T_*)y, pv, scale_log2, ns, ws_ml, ws_o); \
        else paged_decode_attention_kernel<T_, CPL_, false><<<grid, dim3(256), 0, s>>>((const T_*)q, nullptr, nullptr, (T_*)y, pv, scale_log2, ns, ws_ml, ws_o); \
    } while (0)
    if (dtype == RAVEN_BF16) {
        RAVEN_PAGED_LAUNCH(bf16, 1);
        if (ns > 1) launch_combine<bf16>(ws_ml, ws_o, (bf16*)y, n_heads, head_dim, B, ns, s);
    } else {
        if (head_dim / 4 > 16) RAVEN_PAGED_LAUNCH(float, 2);
        else RAVEN_PAGED_LAUNCH(float, 1);
        if (ns > 1) launch_combine<float>(ws_ml, ws_o, (float*)y, n_heads, head_dim, B, ns, s);
    }
#undef RAVEN_PAGED_LAUNCH
    return raven_host::check_launch(who);
}

extern "C" int raven_paged_decode_attention(const void* q, void* y, const void* k_cache, const void* v_cache,
                                            const int32_t* block_table, const int32_t* seq_lens, int32_t B, int32_t max_blocks,
                                            int32_t block_size, int32_t kv_layout, int32_t max_seq_len, int32_t n_heads,
                                            int32_t head_dim, int32_t dtype, void* workspace, size_t workspace_bytes, void* stream) {
    return paged_attention_common("paged_decode_attention", false, q, nullptr, nullptr, y, k_cache, v_cache, block_table, seq_lens, B,
                                  max_blocks, block_size, kv_layout, max_seq_len, n_heads, head_dim, dtype, workspace, workspace_bytes,
                                  stream);
}

extern "C" int raven_paged_qkv_attention_decode(const void* qkv, const void* qk_bias, const float* freqs, void* y, void* k_cache,
                                                void* v_cache, const int32_t* block_table, const int32_t* seq_lens, int32_t B,
                                                int32_t max_blocks, int32_t block_size, int32_t kv_layout, int32_t max_seq_len,
                                                int32_t n_heads, int32_t head_dim, int32_t dtype, void* workspace,
                                                size_t workspace_bytes, void* stream) {
    return paged_attention_common("paged_qkv_attention_decode", true, qkv, qk_bias, freqs, y, k_cache, v_cache, block_table, seq_lens,
                                  B, max_blocks, block_size, kv_layout, max_seq_len, n_heads, head_dim, dtype, workspace, workspace_bytes,
                                  stream);
}

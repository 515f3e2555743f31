// q/k bias + RoPE + KV-cache append, and decode attention over the step-indexed KV cache.
//
// Cache layout (HuginnStaticCache of the reference, recpre/raven_modeling_minimal.py:344-349):
// K, V = [n_slots, batch, n_heads, t_max, head_dim]; one head's positions are contiguous, so a
// workgroup streams [positions x head_dim] with 16-byte lane-contiguous loads.
//
// Attention kernel: grid (splits, heads, token rows).  A position occupies one row of 16 lanes
// (head_dim * sizeof(T) / 16 of them active, 12 for head_dim 96 in bf16); a wave covers 4 positions
// per load instruction and the 4 waves of a workgroup interleave, so each iteration of a
// workgroup reads 16 consecutive positions of K and of V.  Scores are reduced with DPP row
// operations; every 16-lane row runs its own online softmax and the rows are merged through LDS.
// With more than one split the partial (max, sum, unnormalised output) triples go to a workspace and
// the last workgroup to arrive for a (row, head) merges them (arrival counter + __threadfence).

#include <math.h>

#include "raven_common.h"

namespace raven {

struct CacheView {
    void* k;
    void* v;
    int64_t slot_off;  // element offset of the slot: slot * batch * nh * t_max * hd
    int batch, nh, t_max, hd;
};

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
        for (int e = 0; e < E; e += 2) {
            const float cs = f[e], sn = f[e + 1];
            const float x0 = to_f32(x.v[e]), x1 = to_f32(x.v[e + 1]);
            x.v[e] = from_f32<T>(x0 * cs - x1 * sn);
            x.v[e + 1] = from_f32<T>(x1 * cs + x0 * sn);
        }
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
constexpr int kAttnMaxSplits = 32;
constexpr int kAttnMaxHd = 128;

template <typename T>
__global__ __launch_bounds__(256) void decode_attention_kernel(
    const T* __restrict__ q, T* __restrict__ y, CacheView cv, int S, int pos0, const int* __restrict__ pos_dev,
    int n_splits, float scale_log2, int* __restrict__ counters, float* __restrict__ ws_ml, float* __restrict__ ws_o) {
    constexpr int E = Chunk<T>::N;
    __shared__ float sm_m[16], sm_l[16];
    __shared__ float sm_o[16][kAttnMaxHd];
    __shared__ int sm_ticket;

    const int split = blockIdx.x, head = blockIdx.y, m = blockIdx.z;
    const int hd = cv.hd, h = cv.nh * hd;
    const int b = m / S, s = m - b * S;
    int len = (pos_dev ? *pos_dev : pos0) + s + 1;
    len = min(len, cv.t_max);
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

    Chunk<T> qc = zero_chunk<T>();
    if (active) qc = load_chunk(q + (int64_t)m * h + head * hd + ci * E);

    float m_run = -INFINITY, l_run = 0.f, o[E];
#pragma unroll
    for (int e = 0; e < E; ++e) o[e] = 0.f;

    constexpr int U = 2;
    for (int base = start; base < end; base += 16 * U) {  // trip count is uniform over the workgroup
        const int p0 = base + group;
        Chunk<T> kc[U], vc[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int p = p0 + 16 * j;
            if (active && p < end) {
                kc[j] = load_chunk(Kb + (int64_t)p * hd);
                vc[j] = load_chunk(Vb + (int64_t)p * hd);
            } else {
                kc[j] = zero_chunk<T>();
                vc[j] = zero_chunk<T>();
            }
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const int p = p0 + 16 * j;
            float sc = row16_sum(dot_chunk(qc, kc[j], 0.f)) * scale_log2;
            if (p < end) {
                const float m_new = fmaxf(m_run, sc);
                const float corr = exp2f(m_run - m_new);
                const float pe = exp2f(sc - m_new);
                l_run = l_run * corr + pe;
#pragma unroll
                for (int e = 0; e < E; ++e) o[e] = o[e] * corr + pe * to_f32(vc[j].v[e]);
                m_run = m_new;
            }
        }
    }

    // merge the 16 row groups of the workgroup
    if (ci == 0) {
        sm_m[group] = m_run;
        sm_l[group] = l_run;
    }
    if (active) {
#pragma unroll
        for (int e = 0; e < E; ++e) sm_o[group][ci * E + e] = o[e];
    }
    __syncthreads();
    const int t = threadIdx.x;
    float M = -INFINITY, L = 0.f, O = 0.f;
    if (t < hd) {
#pragma unroll
        for (int g = 0; g < 16; ++g) M = fmaxf(M, sm_m[g]);
#pragma unroll
        for (int g = 0; g < 16; ++g) {
            const float wgt = (sm_m[g] == -INFINITY) ? 0.f : exp2f(sm_m[g] - M);
            L += sm_l[g] * wgt;
            O += sm_o[g][t] * wgt;
        }
    }
    if (n_splits == 1) {
        if (t < hd) y[(int64_t)m * h + head * hd + t] = from_f32<T>(O / L);
        return;
    }

    const int64_t mh = (int64_t)m * cv.nh + head;
    if (t < hd) {
        ws_o[(mh * n_splits + split) * hd + t] = O;
        if (t == 0) {
            ws_ml[(mh * n_splits + split) * 2] = M;
            ws_ml[(mh * n_splits + split) * 2 + 1] = L;
        }
    }
    __threadfence();
    __syncthreads();
    if (t == 0) sm_ticket = atomicAdd(&counters[mh], 1);
    __syncthreads();
    if (sm_ticket != n_splits - 1) return;
    __threadfence();
    if (t == 0) counters[mh] = 0;  // leave the counter ready for the next call
    if (t < hd) {
        float Mg = -INFINITY;
        for (int sp = 0; sp < n_splits; ++sp) Mg = fmaxf(Mg, ws_ml[(mh * n_splits + sp) * 2]);
        float Lg = 0.f, Og = 0.f;
        for (int sp = 0; sp < n_splits; ++sp) {
            const float ms = ws_ml[(mh * n_splits + sp) * 2];
            const float wgt = (ms == -INFINITY) ? 0.f : exp2f(ms - Mg);
            Lg += ws_ml[(mh * n_splits + sp) * 2 + 1] * wgt;
            Og += ws_o[(mh * n_splits + sp) * hd + t] * wgt;
        }
        y[(int64_t)m * h + head * hd + t] = from_f32<T>(Og / Lg);
    }
}

static int max_splits_for(int M, int nh) {
    int ns = (1024 + nh * M - 1) / (nh * M);
    if (ns < 1) ns = 1;
    if (ns > kAttnMaxSplits) ns = kAttnMaxSplits;
    return ns;
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
    cv->slot_off = (int64_t)sl * cache->batch * nh * cache->t_max * hd;
    return 0;
}

static int check_heads(const char* who, int nh, int hd, int dtype) {
    RAVEN_REQUIRE(dtype == RAVEN_F32 || dtype == RAVEN_BF16, "%s: unknown dtype %d", who, dtype);
    const int elts = 16 / (int)raven_host::elt_size(dtype);
    RAVEN_REQUIRE(nh > 0 && hd > 0 && hd % elts == 0 && hd % 2 == 0, "%s: head_dim %d must be an even multiple of %d", who, hd, elts);
    RAVEN_REQUIRE(hd / elts <= 16 && hd <= kAttnMaxHd, "%s: head_dim %d too large for one 16-lane row", who, hd);
    return 0;
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
    if (dtype == RAVEN_BF16)
        qkv_rope_append_kernel<bf16><<<grid, dim3(256), 0, s>>>((const bf16*)qkv, (const bf16*)qk_bias, freqs, (bf16*)q_out, cv, S, pos0, pos_dev);
    else
        qkv_rope_append_kernel<float><<<grid, dim3(256), 0, s>>>((const float*)qkv, (const float*)qk_bias, freqs, (float*)q_out, cv, S, pos0, pos_dev);
    return raven_host::check_launch("qkv_append");
}

extern "C" size_t raven_decode_attention_workspace_bytes(int32_t M, int32_t n_heads, int32_t head_dim) {
    using namespace raven;
    if (M <= 0 || n_heads <= 0 || head_dim <= 0) return 0;
    const size_t ns = (size_t)max_splits_for(M, n_heads);
    const size_t mh = (size_t)M * n_heads;
    return raven_host::align_up(mh * 4) + raven_host::align_up(mh * ns * 2 * 4) + raven_host::align_up(mh * ns * head_dim * 4);
}

extern "C" int raven_decode_attention(const void* q, void* y, const raven_kv_cache* cache, int32_t slot, int32_t B,
                                      int32_t S, int32_t pos0, const int32_t* pos_dev, int32_t n_heads, int32_t head_dim,
                                      int32_t dtype, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace raven;
    if (int rc = check_heads("decode_attention", n_heads, head_dim, dtype)) return rc;
    RAVEN_REQUIRE(q && y, "decode_attention: null pointer");
    RAVEN_REQUIRE(B > 0 && S > 0 && pos0 >= 0, "decode_attention: bad B=%d S=%d pos0=%d", B, S, pos0);
    CacheView cv;
    if (int rc = make_view("decode_attention", cache, slot, B, n_heads, head_dim, &cv)) return rc;
    RAVEN_REQUIRE(pos0 + S <= cv.t_max, "decode_attention: positions up to %d exceed the cache length %d", pos0 + S - 1, cv.t_max);
    const int M = B * S;
    RAVEN_REQUIRE(M <= 65535, "decode_attention: too many token rows (%d)", M);
    int ns = max_splits_for(M, n_heads);
    const int by_len = (pos0 + S + 63) / 64;  // at least 64 positions per split
    if (ns > by_len) ns = by_len;
    if (ns < 1) ns = 1;
    const size_t mh = (size_t)M * n_heads;
    int* counters = nullptr;
    float *ws_ml = nullptr, *ws_o = nullptr;
    if (ns > 1) {
        const size_t need = raven_decode_attention_workspace_bytes(M, n_heads, head_dim);
        RAVEN_REQUIRE(workspace && workspace_bytes >= need, "decode_attention: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
        RAVEN_REQUIRE(((uintptr_t)workspace & 255) == 0, "decode_attention: workspace must be 256-byte aligned");
        char* p = static_cast<char*>(workspace);
        counters = reinterpret_cast<int*>(p);
        p += raven_host::align_up(mh * 4);
        ws_ml = reinterpret_cast<float*>(p);
        p += raven_host::align_up(mh * (size_t)max_splits_for(M, n_heads) * 2 * 4);
        ws_o = reinterpret_cast<float*>(p);
    }
    const float scale_log2 = (float)(1.0 / sqrt((double)head_dim) * 1.4426950408889634);
    dim3 grid(ns, n_heads, M);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == RAVEN_BF16)
        decode_attention_kernel<bf16><<<grid, dim3(256), 0, s>>>((const bf16*)q, (bf16*)y, cv, S, pos0, pos_dev, ns, scale_log2, counters, ws_ml, ws_o);
    else
        decode_attention_kernel<float><<<grid, dim3(256), 0, s>>>((const float*)q, (float*)y, cv, S, pos0, pos_dev, ns, scale_log2, counters, ws_ml, ws_o);
    return raven_host::check_launch("decode_attention");
}

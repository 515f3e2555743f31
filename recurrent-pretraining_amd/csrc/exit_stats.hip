// Per-row statistics behind the per-iteration exit criteria of adaptive compute
// (recpre/raven_modeling_minimal.py:2128-2260): entropy of the next-token distribution, KL divergence
// between successive distributions (plain and min-p filtered), and relative change / cosine of successive
// latent states.  One workgroup per row; a row of 65536 logits is 256 KB and stays in L2 across the passes.

#include <math.h>

#include "raven_common.h"

namespace raven {

constexpr int kStatThreads = 1024;

__device__ __forceinline__ float block_reduce(float v, bool is_max, float* sm) {
    v = is_max ? wave_max(v) : wave_sum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();  // sm may still be read from the previous reduction
    if (lane == 0) sm[wave] = v;
    __syncthreads();
    float r = is_max ? -INFINITY : 0.f;
    for (int w = 0; w < kStatThreads / 64; ++w) r = is_max ? fmaxf(r, sm[w]) : r + sm[w];
    return r;
}

// kind 0: out = -sum p log(p + 1e-10)                                      (RMM:2142-2144)
// kind 1: lp = log_softmax(x); out = sum exp(prev) (prev - lp); prev <- lp  (RMM:2182-2186)
// kind 2: p = softmax(x); p[p < 0.1 max p] = 1/V; p /= sum p; lp = log p; then as kind 1 (RMM:2200-2216)
__global__ __launch_bounds__(kStatThreads) void logit_stats_kernel(const float* __restrict__ logits, float* __restrict__ prev,
                                                                   float* __restrict__ out, int V, int kind) {
    __shared__ float sm[kStatThreads / 64];
    const float* x = logits + (int64_t)blockIdx.x * V;
    float* pv = prev ? prev + (int64_t)blockIdx.x * V : nullptr;
    float mx = -INFINITY;
    for (int i = threadIdx.x; i < V; i += kStatThreads) mx = fmaxf(mx, x[i]);
    mx = block_reduce(mx, true, sm);
    float se = 0.f;
    for (int i = threadIdx.x; i < V; i += kStatThreads) se += expf(x[i] - mx);
    se = block_reduce(se, false, sm);
    float acc = 0.f;
    if (kind == 0) {
        for (int i = threadIdx.x; i < V; i += kStatThreads) {
            const float p = expf(x[i] - mx) / se;
            acc += p * logf(p + 1e-10f);
        }
        acc = -block_reduce(acc, false, sm);
    } else if (kind == 1) {
        const float lse = mx + logf(se);
        for (int i = threadIdx.x; i < V; i += kStatThreads) {
            const float lp = x[i] - lse, t = pv[i];
            acc += expf(t) * (t - lp);
            pv[i] = lp;
        }
        acc = block_reduce(acc, false, sm);
    } else {
        const float pmax = 1.f / se, floor_p = 1.f / (float)V;  // the largest probability is exp(0) / se
        float s2 = 0.f;
        for (int i = threadIdx.x; i < V; i += kStatThreads) {
            const float p = expf(x[i] - mx) / se;
            s2 += p < 0.1f * pmax ? floor_p : p;
        }
        s2 = block_reduce(s2, false, sm);
        for (int i = threadIdx.x; i < V; i += kStatThreads) {
            float p = expf(x[i] - mx) / se;
            p = p < 0.1f * pmax ? floor_p : p;
            const float lp = logf(p / s2), t = pv[i];
            acc += expf(t) * (t - lp);
            pv[i] = lp;
        }
        acc = block_reduce(acc, false, sm);
    }
    if (threadIdx.x == 0) out[blockIdx.x] = acc;
}

// rel[m] = |a - b| / |a| and cosv[m] = <a, b> / |a| / |b| with the roundings of the reference's tensor
// expressions in dtype T (RMM:2162, 2256-2259): the difference a - b and the product a * b are tensors of T
// (rounded) before they are reduced, reductions accumulate in fp32 and round their result to T, each division
// rounds to T.
template <typename T>
__global__ __launch_bounds__(256) void latent_stats_kernel(const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ rel,
                                                           T* __restrict__ cosv, int h) {
    __shared__ float sm[4][4];
    const T* pa = a + (int64_t)blockIdx.x * h;
    const T* pb = b + (int64_t)blockIdx.x * h;
    float dd = 0.f, aa = 0.f, bb = 0.f, ab = 0.f;
    for (int i = threadIdx.x; i < h; i += 256) {
        const float x = to_f32(pa[i]), y = to_f32(pb[i]);
        const float d = round_to<T>(x - y);
        dd += d * d;
        aa += x * x;
        bb += y * y;
        ab += round_to<T>(x * y);
    }
    dd = wave_sum(dd); aa = wave_sum(aa); bb = wave_sum(bb); ab = wave_sum(ab);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) { sm[wave][0] = dd; sm[wave][1] = aa; sm[wave][2] = bb; sm[wave][3] = ab; }
    __syncthreads();
    if (threadIdx.x == 0) {
        dd = sm[0][0] + sm[1][0] + sm[2][0] + sm[3][0];
        aa = sm[0][1] + sm[1][1] + sm[2][1] + sm[3][1];
        bb = sm[0][2] + sm[1][2] + sm[2][2] + sm[3][2];
        ab = sm[0][3] + sm[1][3] + sm[2][3] + sm[3][3];
        const float nd = round_to<T>(sqrtf(dd)), na = round_to<T>(sqrtf(aa)), nb = round_to<T>(sqrtf(bb));
        if (rel) rel[blockIdx.x] = from_f32<T>(nd / na);
        if (cosv) cosv[blockIdx.x] = from_f32<T>(round_to<T>(round_to<T>(ab) / na) / nb);
    }
}

}  // namespace raven

extern "C" int raven_exit_logit_stats(const float* logits, float* prev_log_probs, float* out, int32_t rows, int32_t V, int32_t kind,
                                      void* stream) {
    using namespace raven;
    RAVEN_REQUIRE(rows >= 0 && V > 0, "exit_logit_stats: bad shape rows=%d V=%d", rows, V);
    RAVEN_REQUIRE(kind >= RAVEN_EXIT_ENTROPY && kind <= RAVEN_EXIT_MINP_KL, "exit_logit_stats: unknown kind %d", kind);
    if (rows == 0) return 0;
    RAVEN_REQUIRE(logits && out, "exit_logit_stats: null pointer");
    RAVEN_REQUIRE(kind == RAVEN_EXIT_ENTROPY || prev_log_probs, "exit_logit_stats: the KL kinds need prev_log_probs");
    logit_stats_kernel<<<dim3(rows), dim3(kStatThreads), 0, static_cast<hipStream_t>(stream)>>>(logits, prev_log_probs, out, V, kind);
    return raven_host::check_launch("exit_logit_stats");
}

extern "C" int raven_exit_latent_stats(const void* latents, const void* prev, void* rel_change, void* cosine, int32_t rows,
                                       int32_t h, int32_t dtype, void* stream) {
    using namespace raven;
    RAVEN_REQUIRE(dtype == RAVEN_F32 || dtype == RAVEN_BF16, "exit_latent_stats: unknown dtype %d", dtype);
    RAVEN_REQUIRE(rows >= 0 && h > 0, "exit_latent_stats: bad shape rows=%d h=%d", rows, h);
    if (rows == 0) return 0;
    RAVEN_REQUIRE(latents && prev && (rel_change || cosine), "exit_latent_stats: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == RAVEN_BF16)
        latent_stats_kernel<bf16><<<dim3(rows), dim3(256), 0, s>>>((const bf16*)latents, (const bf16*)prev, (bf16*)rel_change,
                                                                   (bf16*)cosine, h);
    else
        latent_stats_kernel<float><<<dim3(rows), dim3(256), 0, s>>>((const float*)latents, (const float*)prev, (float*)rel_change,
                                                                    (float*)cosine, h);
    return raven_host::check_launch("exit_latent_stats");
}

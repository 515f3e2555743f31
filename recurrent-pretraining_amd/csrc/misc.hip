// Small kernels around the recurrence (embedding gather, greedy argmax, device-side position) and
// the library's error/identity plumbing.

#include <stdarg.h>
#include <stdio.h>

#include "raven_common.h"

namespace raven_host {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: launch failed: %s", what, hipGetErrorString(e));
        return (int)e;
    }
    return 0;
}

}  // namespace raven_host

namespace raven {

// out[m] = T(wte[ids[m]] * scale)   (recpre/raven_modeling_minimal.py:667-671)
template <typename T>
__global__ __launch_bounds__(256) void embed_kernel(const T* __restrict__ wte, const int64_t* __restrict__ ids,
                                                    T* __restrict__ out, int dim, int64_t vocab, float scale) {
    constexpr int E = Chunk<T>::N;
    const int m = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= dim / E) return;
    int64_t id = ids[m];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);  // never read outside the table
    Chunk<T> v = load_chunk(wte + id * dim + c * E);
#pragma unroll
    for (int e = 0; e < E; ++e) v.v[e] = from_f32<T>(to_f32(v.v[e]) * scale);
    store_chunk(out + (int64_t)m * dim + c * E, v);
}

// first index of the row maximum; one 1024-thread workgroup per row
__global__ __launch_bounds__(1024) void argmax_kernel(const float* __restrict__ logits, int64_t* __restrict__ out, int64_t vocab) {
    __shared__ float sv[16];
    __shared__ long long si[16];
    const float* row = logits + (int64_t)blockIdx.x * vocab;
    float best = -INFINITY;
    long long bi = 0x7fffffffffffffffll;
    for (int64_t i = threadIdx.x; i < vocab; i += 1024) {
        const float v = row[i];
        if (v > best) {  // indices grow, so the first maximum of this thread's stripe wins
            best = v;
            bi = i;
        }
    }
    // wave reduce, then across the 16 waves
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(best, off, 64);
        const long long oi = __shfl_xor(bi, off, 64);
        if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = best; si[threadIdx.x >> 6] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; ++w)
            if (sv[w] > best || (sv[w] == best && si[w] < bi)) { best = sv[w]; bi = si[w]; }
        out[blockIdx.x] = bi == 0x7fffffffffffffffll ? 0 : bi;
    }
}

// out[m, j] = T(T(silu(z[m, j])) * z[m, I + j])   (recpre/raven_modeling_minimal.py:507-508, after a library GEMM)
template <typename T>
__global__ __launch_bounds__(256) void swiglu_kernel(const T* __restrict__ z, T* __restrict__ out, int inter) {
    constexpr int E = Chunk<T>::N;
    const int64_t m = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= inter / E) return;
    const Chunk<T> g = load_chunk(z + m * 2 * inter + c * E);
    const Chunk<T> u = load_chunk(z + m * 2 * inter + inter + c * E);
    Chunk<T> o;
#pragma unroll
    for (int e = 0; e < E; ++e) o.v[e] = from_f32<T>(round_to<T>(silu_f32(to_f32(g.v[e]))) * to_f32(u.v[e]));
    store_chunk(out + m * inter + c * E, o);
}

// Test-time noise (recpre/raven_modeling_minimal.py:815-833): y = T(T(x * keep) + n) with n = T(noise * a), divided once
// more by d and rounded again when d != 0 -- the reference's elementwise torch expression, one rounding per operation.
template <typename T>
__global__ __launch_bounds__(256) void noise_mix_kernel(const T* __restrict__ x, const T* __restrict__ noise, T* __restrict__ y,
                                                        int64_t chunks, float keep, float a, float d) {
#pragma clang fp contract(off)  // float32 states: the product and the sum are two roundings, never one fused multiply-add
    constexpr int E = Chunk<T>::N;
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= chunks) return;
    const Chunk<T> xv = load_chunk(x + c * E), nv = load_chunk(noise + c * E);
    Chunk<T> o;
#pragma unroll
    for (int e = 0; e < E; ++e) {
        float n = round_to<T>(to_f32(nv.v[e]) * a);
        if (d != 0.f) n = round_to<T>(n / d);
        o.v[e] = from_f32<T>(round_to<T>(to_f32(xv.v[e]) * keep) + n);
    }
    store_chunk(y + c * E, o);
}

__global__ void advance_pos_kernel(int* pos, int delta) {
    if (threadIdx.x == 0 && blockIdx.x == 0) *pos += delta;
}

}  // namespace raven

extern "C" int raven_version(void) { return 1; }
extern "C" const char* raven_arch(void) { return "gfx950"; }
extern "C" const char* raven_last_error(void) { return raven_host::g_err; }

extern "C" int raven_embed(const void* wte, const int64_t* ids, void* out, int32_t M, int32_t dim, int64_t vocab,
                           float scale, int32_t dtype, void* stream) {
    using namespace raven;
    RAVEN_REQUIRE(dtype == RAVEN_F32 || dtype == RAVEN_BF16, "embed: unknown dtype %d", dtype);
    RAVEN_REQUIRE(wte && ids && out, "embed: null pointer");
    const int elts = 16 / (int)raven_host::elt_size(dtype);
    RAVEN_REQUIRE(M >= 0 && M <= 65535 && dim > 0 && dim % elts == 0 && vocab > 0, "embed: bad shape M=%d dim=%d", M, dim);
    if (M == 0) return 0;
    dim3 grid((dim / elts + 255) / 256, M);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == RAVEN_BF16)
        embed_kernel<bf16><<<grid, dim3(256), 0, s>>>((const bf16*)wte, ids, (bf16*)out, dim, vocab, scale);
    else
        embed_kernel<float><<<grid, dim3(256), 0, s>>>((const float*)wte, ids, (float*)out, dim, vocab, scale);
    return raven_host::check_launch("embed");
}

extern "C" int raven_argmax(const float* logits, int64_t* out, int32_t M, int64_t vocab, void* stream) {
    using namespace raven;
    RAVEN_REQUIRE(logits && out, "argmax: null pointer");
    RAVEN_REQUIRE(M >= 0 && vocab > 0, "argmax: bad shape M=%d vocab=%lld", M, (long long)vocab);
    if (M == 0) return 0;
    argmax_kernel<<<dim3(M), dim3(1024), 0, static_cast<hipStream_t>(stream)>>>(logits, out, vocab);
    return raven_host::check_launch("argmax");
}

extern "C" int raven_swiglu(const void* z, void* out, int32_t M, int32_t I, int32_t dtype, void* stream) {
    using namespace raven;
    RAVEN_REQUIRE(dtype == RAVEN_F32 || dtype == RAVEN_BF16, "swiglu: unknown dtype %d", dtype);
    if (M == 0) return 0;
    RAVEN_REQUIRE(z && out, "swiglu: null pointer");
    const int elts = 16 / (int)raven_host::elt_size(dtype);
    RAVEN_REQUIRE(M > 0 && M <= 65535 && I > 0 && I % elts == 0, "swiglu: bad shape M=%d I=%d", M, I);
    dim3 grid((I / elts + 255) / 256, M);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == RAVEN_BF16) swiglu_kernel<bf16><<<grid, dim3(256), 0, s>>>((const bf16*)z, (bf16*)out, I);
    else swiglu_kernel<float><<<grid, dim3(256), 0, s>>>((const float*)z, (float*)out, I);
    return raven_host::check_launch("swiglu");
}

extern "C" int raven_noise_mix(const void* x, const void* noise, void* y, int64_t n, float keep, float a, float d, int32_t dtype,
                               void* stream) {
    using namespace raven;
    RAVEN_REQUIRE(dtype == RAVEN_F32 || dtype == RAVEN_BF16, "noise_mix: unknown dtype %d", dtype);
    RAVEN_REQUIRE(x && noise && y, "noise_mix: null pointer");
    const int elts = 16 / (int)raven_host::elt_size(dtype);
    RAVEN_REQUIRE(n >= 0 && n % elts == 0, "noise_mix: %lld elements are not a multiple of %d", (long long)n, elts);
    if (n == 0) return 0;
    const int64_t chunks = n / elts;
    RAVEN_REQUIRE((chunks + 255) / 256 <= 0x7fffffff, "noise_mix: too many elements");
    const dim3 grid((unsigned)((chunks + 255) / 256));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == RAVEN_BF16) noise_mix_kernel<bf16><<<grid, dim3(256), 0, s>>>((const bf16*)x, (const bf16*)noise, (bf16*)y, chunks, keep, a, d);
    else noise_mix_kernel<float><<<grid, dim3(256), 0, s>>>((const float*)x, (const float*)noise, (float*)y, chunks, keep, a, d);
    return raven_host::check_launch("noise_mix");
}

extern "C" int raven_advance_pos(int32_t* pos_dev, int32_t delta, void* stream) {
    using namespace raven;
    RAVEN_REQUIRE(pos_dev, "advance_pos: null pointer");
    advance_pos_kernel<<<dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream)>>>(pos_dev, delta);
    return raven_host::check_launch("advance_pos");
}

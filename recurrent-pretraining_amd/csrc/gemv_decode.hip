// Decode fast path for ONE token row: y = epilogue( prologue(x) W^T ), one launch per weight matrix.
//
// One 256-thread workgroup per pair of weight rows; its four waves split K.  Every lane first issues
// its x loads (served by L1/L2: x is a few KB shared by all workgroups), then ALL of its weight loads
// (16-byte, lane-contiguous, non-temporal: each weight byte is read once per token), so the complete
// share of both rows is in flight before any arithmetic starts.  While the weights stream in, the
// workgroup computes the RMSNorm prologue on the x registers:
//     x <- norm_a(x) [stored by workgroup 0 when the caller needs it], x <- norm_b(x)
// which folds norm_4 -> norm_1 (before Wqkv), norm_2 -> norm_3 (before mlp.fc) and norm_4 (before the
// adapter) of the reference's SandwichBlock (recpre/raven_modeling_minimal.py:525-536, 776) into the
// GEMV that consumes them.  Dot products use v_dot2_f32_bf16 / fp32 FMA, a DPP wave reduction and a
// 4-way LDS reduction finish the pair, and the epilogue is the same as in gemm_skinny.hip:
// plain (+ residual, + float store) or SwiGLU (rows j and j + N).
//
// C = weight chunks per lane, per row: ceil(ceil(K / E / 4) / 64) rounded up to 3, 6 or 9.

#include "raven_common.h"

namespace raven {

struct Gemv1Args {
    const void* w;         // [N or 2N, K]
    const void* x0;        // [k0]
    const void* x1;        // [K - k0] or null
    const void* norm_a;    // [k0] or null: first RMSNorm weight applied to x0
    const void* norm_b;    // [k0] or null: second RMSNorm weight
    void* xa_out;          // [k0] or null: receives norm_a(x0)
    const void* residual;  // [N] or null
    void* y;               // [N]
    int N, K, k0;
    int out_f32;
    float eps;
};

template <bool NT, typename T>
__device__ __forceinline__ Chunk<T> ld_weight(const T* p) {
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    Chunk<T> c;
    if (NT) *reinterpret_cast<u32x4*>(&c) = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    else c = load_chunk(p);
    return c;
}

// sum over the 256 threads through LDS; `red` has 4 floats
__device__ __forceinline__ float wg_sum(float v, float* red) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return red[0] + red[1] + red[2] + red[3];
}

template <typename T, int C, bool SWIGLU, bool NORM>
__global__ __launch_bounds__(256) void gemv1_kernel(Gemv1Args a) {
    constexpr int E = Chunk<T>::N;
    __shared__ float red[4];
    __shared__ float part[4][2];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n_chunks = a.K / E, c0 = a.k0 / E;
    const int cb = (int)((int64_t)n_chunks * wave / 4), ce = (int)((int64_t)n_chunks * (wave + 1) / 4);
    const int unit = blockIdx.x;
    int r0, r1;
    bool r1_ok = true;
    if (SWIGLU) {
        r0 = unit;
        r1 = unit + a.N;
    } else {
        r0 = 2 * unit;
        r1 = r0 + 1;
        if (r1 >= a.N) { r1 = r0; r1_ok = false; }
    }
    const T* w0 = static_cast<const T*>(a.w) + (int64_t)r0 * a.K;
    const T* w1 = static_cast<const T*>(a.w) + (int64_t)r1 * a.K;
    const T* x0 = static_cast<const T*>(a.x0);
    const T* x1 = static_cast<const T*>(a.x1);

    // x first (older loads return first), then every weight chunk of this lane
    Chunk<T> xc[C], na[NORM ? C : 1], nb[NORM ? C : 1], wa[C], wb[C];
    bool ok[C], in0[C];
#pragma unroll
    for (int j = 0; j < C; ++j) {
        const int c = cb + lane + 64 * j;
        ok[j] = c < ce;
        in0[j] = ok[j] && c < c0;
        xc[j] = zero_chunk<T>();
        if (ok[j]) xc[j] = (c < c0) ? load_chunk(x0 + c * E) : load_chunk(x1 + (c - c0) * E);
    }
    if (NORM && a.norm_a) {
#pragma unroll
        for (int j = 0; j < C; ++j)
            if (in0[j]) na[NORM ? j : 0] = load_chunk(static_cast<const T*>(a.norm_a) + (cb + lane + 64 * j) * E);
    }
    if (NORM && a.norm_b) {
#pragma unroll
        for (int j = 0; j < C; ++j)
            if (in0[j]) nb[NORM ? j : 0] = load_chunk(static_cast<const T*>(a.norm_b) + (cb + lane + 64 * j) * E);
    }
#pragma unroll
    for (int j = 0; j < C; ++j) {
        const int c = cb + lane + 64 * j;
        if (ok[j]) {
            wa[j] = ld_weight<true>(w0 + c * E);
            wb[j] = ld_weight<true>(w1 + c * E);
        } else {
            wa[j] = zero_chunk<T>();
            wb[j] = zero_chunk<T>();
        }
    }

    // RMSNorm prologue(s) over x0 (recpre/raven_modeling_minimal.py:137-142): fp32 statistics,
    // round to T, multiply by the weight in T
    if (NORM && a.norm_a) {
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < C; ++j)
            if (in0[j]) {
#pragma unroll
                for (int e = 0; e < E; ++e) ss = __builtin_fmaf(to_f32(xc[j].v[e]), to_f32(xc[j].v[e]), ss);
            }
        const float inv = rsqrtf(wg_sum(ss, red) / (float)a.k0 + a.eps);
#pragma unroll
        for (int j = 0; j < C; ++j)
            if (in0[j]) {
#pragma unroll
                for (int e = 0; e < E; ++e) xc[j].v[e] = from_f32<T>(round_to<T>(to_f32(xc[j].v[e]) * inv) * to_f32(na[NORM ? j : 0].v[e]));
                if (a.xa_out && blockIdx.x == 0) store_chunk(static_cast<T*>(a.xa_out) + (cb + lane + 64 * j) * E, xc[j]);
            }
    }
    if (NORM && a.norm_b) {
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < C; ++j)
            if (in0[j]) {
#pragma unroll
                for (int e = 0; e < E; ++e) ss = __builtin_fmaf(to_f32(xc[j].v[e]), to_f32(xc[j].v[e]), ss);
            }
        const float inv = rsqrtf(wg_sum(ss, red) / (float)a.k0 + a.eps);
#pragma unroll
        for (int j = 0; j < C; ++j)
            if (in0[j]) {
#pragma unroll
                for (int e = 0; e < E; ++e) xc[j].v[e] = from_f32<T>(round_to<T>(to_f32(xc[j].v[e]) * inv) * to_f32(nb[NORM ? j : 0].v[e]));
            }
    }

    float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
    for (int j = 0; j < C; ++j) {
        acc0 = dot_chunk(wa[j], xc[j], acc0);
        acc1 = dot_chunk(wb[j], xc[j], acc1);
    }
    acc0 = wave_sum(acc0);
    acc1 = wave_sum(acc1);
    if (lane == 0) {
        part[wave][0] = acc0;
        part[wave][1] = acc1;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const float s0 = part[0][0] + part[1][0] + part[2][0] + part[3][0];
        const float s1 = part[0][1] + part[1][1] + part[2][1] + part[3][1];
        if (SWIGLU) {
            const float g = round_to<T>(s0), u = round_to<T>(s1);
            static_cast<T*>(a.y)[unit] = from_f32<T>(round_to<T>(silu_f32(g)) * u);
        } else {
            const T* res = static_cast<const T*>(a.residual);
            float v0 = round_to<T>(s0), v1 = round_to<T>(s1);
            if (res) {
                v0 = round_to<T>(v0 + to_f32(res[r0]));
                if (r1_ok) v1 = round_to<T>(v1 + to_f32(res[r1]));
            }
            if (a.out_f32) {
                static_cast<float*>(a.y)[r0] = v0;
                if (r1_ok) static_cast<float*>(a.y)[r1] = v1;
            } else {
                static_cast<T*>(a.y)[r0] = from_f32<T>(v0);
                if (r1_ok) static_cast<T*>(a.y)[r1] = from_f32<T>(v1);
            }
        }
    }
}

template <typename T, bool SWIGLU>
static int launch_gemv1(const Gemv1Args& a, hipStream_t s) {
    constexpr int E = Chunk<T>::N;
    const int n_chunks = a.K / E;
    const int per_wave = (n_chunks + 3) / 4 + 1;  // a quarter, rounded up
    const int c = (per_wave + 63) / 64;
    const int units = SWIGLU ? a.N : (a.N + 1) / 2;
    const bool norm = a.norm_a != nullptr;
#define RAVEN_GEMV1(CC)                                                                       \
    do {                                                                                      \
        if (norm) gemv1_kernel<T, CC, SWIGLU, true><<<dim3(units), dim3(256), 0, s>>>(a);     \
        else gemv1_kernel<T, CC, SWIGLU, false><<<dim3(units), dim3(256), 0, s>>>(a);         \
    } while (0)
    if (c <= 3) RAVEN_GEMV1(3);
    else if (c <= 6) RAVEN_GEMV1(6);
    else if (c <= 9) RAVEN_GEMV1(9);
    else {
        raven_host::set_error("gemv_fused: K=%d is too long for the one-row kernel (max %d)", a.K, 9 * 64 * 4 * E - 4 * E);
        return -1;
    }
#undef RAVEN_GEMV1
    return raven_host::check_launch("gemv_fused");
}

}  // namespace raven

extern "C" int raven_gemv_fused(const void* x0, const void* x1, const void* norm_a, const void* norm_b, void* xa_out,
                                const void* w, const void* residual, void* y, int32_t N, int32_t K0, int32_t K1, float eps,
                                int32_t swiglu, int32_t out_f32, int32_t dtype, void* stream) {
    using namespace raven;
    RAVEN_REQUIRE(dtype == RAVEN_F32 || dtype == RAVEN_BF16, "gemv_fused: unknown dtype %d", dtype);
    RAVEN_REQUIRE(x0 && w && y, "gemv_fused: null pointer");
    const int elts = 16 / (int)raven_host::elt_size(dtype);
    RAVEN_REQUIRE(N > 0 && K0 > 0 && K1 >= 0 && K0 % elts == 0 && K1 % elts == 0, "gemv_fused: bad shape N=%d K0=%d K1=%d", N, K0, K1);
    RAVEN_REQUIRE((K1 == 0) == (x1 == nullptr), "gemv_fused: x1 and K1 must be given together");
    RAVEN_REQUIRE(norm_a || !norm_b, "gemv_fused: norm_b without norm_a");
    RAVEN_REQUIRE(norm_a || !xa_out, "gemv_fused: xa_out needs norm_a");
    RAVEN_REQUIRE(!(swiglu && (residual || out_f32)), "gemv_fused: the SwiGLU epilogue takes no residual and stores T");
    Gemv1Args a{};
    a.w = w; a.x0 = x0; a.x1 = x1; a.norm_a = norm_a; a.norm_b = norm_b; a.xa_out = xa_out;
    a.residual = residual; a.y = y; a.N = N; a.K = K0 + K1; a.k0 = K0; a.out_f32 = out_f32; a.eps = eps;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == RAVEN_BF16) return swiglu ? launch_gemv1<bf16, true>(a, s) : launch_gemv1<bf16, false>(a, s);
    return swiglu ? launch_gemv1<float, true>(a, s) : launch_gemv1<float, false>(a, s);
}

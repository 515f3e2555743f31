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

#include <string>

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
    int pairs_per_wg;      // weight-row pairs each workgroup walks through
    int ldw;               // elements between two weight rows (K, or more for a column block of a wider matrix)
    const float* acc_in;   // [N] or null: fp32 sums of the remaining columns, added before the result is rounded
    int raw_out;           // y receives the unrounded fp32 sums (the other half of acc_in)
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

constexpr int kMaxPairsPerWg = 16;

// MULTI: the workgroup walks several row pairs and double-buffers their weights in registers
template <typename T, int C, bool SWIGLU, bool NORM, bool MULTI>
__global__ __launch_bounds__(256) void gemv1_kernel(Gemv1Args a) {
    constexpr int E = Chunk<T>::N;
    __shared__ float red[4];
    __shared__ float part[kMaxPairsPerWg][4][2];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n_chunks = a.K / E, c0 = a.k0 / E;
    const int cb = (int)((int64_t)n_chunks * wave / 4), ce = (int)((int64_t)n_chunks * (wave + 1) / 4);
    const int n_units = SWIGLU ? a.N : (a.N + 1) / 2;
    const int ppw = MULTI ? a.pairs_per_wg : 1;
    const T* W = static_cast<const T*>(a.w);
    const T* x0 = static_cast<const T*>(a.x0);
    const T* x1 = static_cast<const T*>(a.x1);

    // pair p of this workgroup; consecutive workgroups take consecutive pairs, so the grid as a whole
    // walks the matrix front to back
    auto unit_of = [&](int p) { return p * (int)gridDim.x + (int)blockIdx.x; };
    auto load_pair = [&](int unit, Chunk<T>* wa, Chunk<T>* wb) {
        const int r0 = SWIGLU ? unit : 2 * unit;
        const int r1 = SWIGLU ? unit + a.N : min(r0 + 1, a.N - 1);
        const T* w0 = W + (int64_t)r0 * a.ldw;
        const T* w1 = W + (int64_t)r1 * a.ldw;
#pragma unroll
        for (int j = 0; j < C; ++j) {
            const int c = cb + lane + 64 * j;
            if (c < ce && unit < n_units) {
                wa[j] = ld_weight<true>(w0 + c * E);
                wb[j] = ld_weight<true>(w1 + c * E);
            } else {
                wa[j] = zero_chunk<T>();
                wb[j] = zero_chunk<T>();
            }
        }
    };

    // x first (older loads return first), then the first pair's weights
    Chunk<T> xc[C], na[NORM ? C : 1], nb[NORM ? C : 1];
    bool in0[C];
#pragma unroll
    for (int j = 0; j < C; ++j) {
        const int c = cb + lane + 64 * j;
        in0[j] = c < ce && c < c0;
        xc[j] = zero_chunk<T>();
        if (c < ce) xc[j] = (c < c0) ? load_chunk(x0 + c * E) : load_chunk(x1 + (c - c0) * E);
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
    Chunk<T> wa0[C], wb0[C], wa1[MULTI ? C : 1], wb1[MULTI ? C : 1];
    load_pair(unit_of(0), wa0, wb0);

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

    auto finish_pair = [&](int p, const Chunk<T>* wa, const Chunk<T>* wb) {
        float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
        for (int j = 0; j < C; ++j) {
            acc0 = dot_chunk(wa[j], xc[j], acc0);
            acc1 = dot_chunk(wb[j], xc[j], acc1);
        }
        acc0 = wave_sum(acc0);
        acc1 = wave_sum(acc1);
        if (lane == 0) {
            part[p][wave][0] = acc0;
            part[p][wave][1] = acc1;
        }
    };
    // the next pair's weights are requested before the current pair is reduced
    if (MULTI) {
        for (int p = 0; p < ppw; p += 2) {
            if (p + 1 < ppw) load_pair(unit_of(p + 1), wa1, wb1);
            finish_pair(p, wa0, wb0);
            if (p + 1 < ppw) {
                if (p + 2 < ppw) load_pair(unit_of(p + 2), wa0, wb0);
                finish_pair(p + 1, wa1, wb1);
            }
        }
    } else {
        finish_pair(0, wa0, wb0);
    }
    __syncthreads();

    const int p = threadIdx.x;
    if (p < ppw && unit_of(p) < n_units) {
        const int unit = unit_of(p);
        float s0 = part[p][0][0] + part[p][1][0] + part[p][2][0] + part[p][3][0];
        float s1 = part[p][0][1] + part[p][1][1] + part[p][2][1] + part[p][3][1];
        if (!SWIGLU && (a.acc_in || a.raw_out)) {
            const int r0 = 2 * unit, r1 = r0 + 1;
            if (a.acc_in) {
                s0 += a.acc_in[r0];
                if (r1 < a.N) s1 += a.acc_in[r1];
            }
            if (a.raw_out) {
                static_cast<float*>(a.y)[r0] = s0;
                if (r1 < a.N) static_cast<float*>(a.y)[r1] = s1;
                return;
            }
        }
        if (SWIGLU) {
            const float g = round_to<T>(s0), u = round_to<T>(s1);
            static_cast<T*>(a.y)[unit] = from_f32<T>(round_to<T>(silu_f32(g)) * u);
        } else {
            const int r0 = 2 * unit, r1 = r0 + 1;
            const bool r1_ok = r1 < a.N;
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

struct Gemv1Tuning {
    int pairs_norm = 0;    // pairs per workgroup when a norm prologue has to be amortised; 0 = by shape (about ten workgroups per CU)
    int pairs_plain = 1;   // ... and when there is none
};
static Gemv1Tuning g_gemv1_tuning;

static int gemv1_cus() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0;
        hipDeviceProp_t p;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) cus = p.multiProcessorCount;
        if (cus <= 0) cus = 256;
    }
    return cus;
}

template <typename T, bool SWIGLU>
static int launch_gemv1(Gemv1Args a, hipStream_t s) {
    constexpr int E = Chunk<T>::N;
    const int n_chunks = a.K / E;
    const int per_wave = (n_chunks + 3) / 4 + 1;  // a quarter, rounded up
    const int c = (per_wave + 63) / 64;
    const int units = SWIGLU ? a.N : (a.N + 1) / 2;
    const bool norm = a.norm_a != nullptr;
    int ppw = norm ? g_gemv1_tuning.pairs_norm : g_gemv1_tuning.pairs_plain;
    // with a norm prologue: as many pairs as leave about ten workgroups per CU -- 4 for Wqkv (7920 pairs, 1980 workgroups),
    // 7 for mlp.fc (17920 gate / up pairs, 2560 workgroups: 57.6 us against 58.4 with 4, while Wqkv loses with more than 4)
    if (norm && ppw <= 0) ppw = (units + 10 * gemv1_cus() - 1) / (10 * gemv1_cus());
    if (ppw < 1) ppw = 1;
    if (ppw > kMaxPairsPerWg) ppw = kMaxPairsPerWg;
    while (ppw > 1 && (units + ppw - 1) / ppw < 1024) --ppw;  // keep at least ~4 workgroups per CU
    if (c > 3) ppw = 1;  // the double-buffered variant exists for short rows only (registers)
    a.pairs_per_wg = ppw;
    const int wgs = (units + ppw - 1) / ppw;
#define RAVEN_GEMV1(CC)                                                                            \
    do {                                                                                           \
        if (norm) gemv1_kernel<T, CC, SWIGLU, true, false><<<dim3(wgs), dim3(256), 0, s>>>(a);     \
        else gemv1_kernel<T, CC, SWIGLU, false, false><<<dim3(wgs), dim3(256), 0, s>>>(a);         \
    } while (0)
    if (c <= 3 && ppw > 1) {
        if (norm) gemv1_kernel<T, 3, SWIGLU, true, true><<<dim3(wgs), dim3(256), 0, s>>>(a);
        else gemv1_kernel<T, 3, SWIGLU, false, true><<<dim3(wgs), dim3(256), 0, s>>>(a);
    } else if (c <= 3) RAVEN_GEMV1(3);
    else if (c <= 6) RAVEN_GEMV1(6);
    else if (c <= 9) RAVEN_GEMV1(9);
    else {
        raven_host::set_error("gemv_fused: K=%d is too long for the one-row kernel (max %d)", a.K, 9 * 64 * 4 * E - 4 * E);
        return -1;
    }
#undef RAVEN_GEMV1
    return raven_host::check_launch("gemv_fused");
}

int set_gemv1_tuning(const char* key, int value) {
    const std::string k(key);
    if (k == "gemv1_pairs_norm") g_gemv1_tuning.pairs_norm = value;
    else if (k == "gemv1_pairs_plain") g_gemv1_tuning.pairs_plain = value;
    else return -1;
    return 0;
}

// One column block of a wider weight matrix: y = round(norm_a(x) W[:, c0 : c0 + K]^T + acc_in), or the unrounded
// fp32 sums when raw_out is set.  A product over concatenated inputs (the adapter's [state, embedding],
// recpre/raven_modeling_minimal.py:776) whose second input does not change between calls is split with it: the sums of
// the unchanged half are kept in fp32 and enter the other half's accumulator before the one rounding the product has.
int gemv1_column_block(const void* x, const void* norm_a, const void* w_block, int ldw, const float* acc_in, void* y, int raw_out,
                       int N, int K, float eps, int dtype, hipStream_t s) {
    Gemv1Args a{};
    a.w = w_block; a.x0 = x; a.norm_a = norm_a; a.y = y; a.N = N; a.K = K; a.k0 = K; a.eps = eps;
    a.ldw = ldw; a.acc_in = acc_in; a.raw_out = raw_out;
    return dtype == RAVEN_BF16 ? launch_gemv1<bf16, false>(a, s) : launch_gemv1<float, false>(a, s);
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
    a.ldw = a.K;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == RAVEN_BF16) return swiglu ? launch_gemv1<bf16, true>(a, s) : launch_gemv1<bf16, false>(a, s);
    return swiglu ? launch_gemv1<float, true>(a, s) : launch_gemv1<float, false>(a, s);
}

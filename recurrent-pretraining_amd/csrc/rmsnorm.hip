// Fused (residual add +) RMSNorm (+ second RMSNorm) for [rows, dim] activations.
// One 256-thread workgroup per row; the row stays in registers between the add, the two
// reductions and the stores, so HBM sees each element once on the way in and once per output.
// Arithmetic follows RMSNorm.forward of the reference (recpre/raven_modeling_minimal.py:137-142):
// normalise in fp32, round to T, then multiply by the weight in T (a second rounding).

#include "raven_common.h"

namespace raven {

constexpr int kNormThreads = 256;
constexpr int kNormMaxChunks = 16;  // per thread, in the largest variant: dim <= 256 * 16 * (16 / sizeof(T)) elements

__device__ __forceinline__ float block_sum_256(float v, float* red) {
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6;
    __syncthreads();  // protects `red` against the previous use
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    return red[0] + red[1] + red[2] + red[3];
}

// ldy, ldy2: elements between two rows of y and of y2 (dim, or more where the rows are padded to whole cache lines for
// the tiled GEMM that reads them); x, residual and sum_out are dim apart.
// MC = 16-byte chunks a thread keeps of its row (4 covers 5280 bf16 elements; fp32 rows of that length need 8)
// EARLY: the weights are requested before the row, so that no load waits behind a reduction (taken for up to 64 rows;
// measured at 5280 columns it is worth 0.1 us of a 3.6 us launch at best, the weights being cache hits).  Otherwise
// each weight chunk is fetched where it is used, which keeps 32 registers free and more rows in flight per CU: from
// 1024 rows on the early form is 3-20 % slower (4096 rows: 25.7 against 23.7 us, two norms 31.9 against 26.7).
//
// KS > 0: the row is not read from x but formed from the fp32 partial sums of KS slices that a K-split product left behind
// (gemm_splitk.hip): extra + slice 0 + slice 1 + ... in this order, rounded to T, plus the residual, rounded again -- the
// arithmetic of that file's second launch, which this launch then replaces.  The slice count is a template argument so
// that every load of the row (slices, extra, residual) is requested before the first sum: with a run-time loop over the
// slices each one was a memory round trip of its own, KS + 2 in a row per chunk.
struct SplitSums {
    const float* partial;  // [ks][rows][dim]
    const float* extra;    // [rows][dim] or null
    int ks;
    int64_t slice_stride;  // rows * dim
};

template <typename T, int MC, bool EARLY, int KS>
__global__ __launch_bounds__(kNormThreads) void rmsnorm_kernel(
    const T* __restrict__ x, const T* __restrict__ residual, const T* __restrict__ weight, T* __restrict__ y,
    T* __restrict__ sum_out, const T* __restrict__ weight2, T* __restrict__ y2, int dim, float eps, SplitSums sp, int ldy, int ldy2) {
    constexpr int E = Chunk<T>::N;
    __shared__ float red[4];
    const int64_t row = blockIdx.x;
    const int n_chunks = dim / E;
    const T* xr = x + row * dim;
    const T* rr = residual ? residual + row * dim : nullptr;

    Chunk<T> cw[EARLY ? MC : 1], cw2[EARLY ? MC : 1];
    if constexpr (EARLY) {
#pragma unroll
        for (int i = 0; i < MC; ++i) {
            const int c = threadIdx.x + i * kNormThreads;
            if (c < n_chunks) {
                cw[i] = load_chunk(weight + c * E);
                if (weight2) cw2[i] = load_chunk(weight2 + c * E);
            }
        }
    }

    float v[MC][E];
    float ss = 0.f;
    constexpr bool SPLIT = KS > 0;
    constexpr int Q = E / 4;
    Chunk<T> cxs[MC], crs[MC];
    f32x4 pv[SPLIT ? MC : 1][SPLIT ? KS + 1 : 1][Q];  // [.][0]: extra, [.][1 + sl]: slice sl
#pragma unroll
    for (int i = 0; i < MC; ++i) {
        const int c = threadIdx.x + i * kNormThreads;
        if (c < n_chunks) {
            if constexpr (SPLIT) {
                const int64_t at = row * dim + c * E;
#pragma unroll
                for (int q = 0; q < Q; ++q) {
                    pv[i][0][q] = sp.extra ? *reinterpret_cast<const f32x4*>(sp.extra + at + 4 * q) : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int sl = 0; sl < KS; ++sl) pv[i][1 + sl][q] = *reinterpret_cast<const f32x4*>(sp.partial + sl * sp.slice_stride + at + 4 * q);
                }
            } else {
                cxs[i] = load_chunk(xr + c * E);
            }
            if (rr) crs[i] = load_chunk(rr + c * E);
        }
    }
#pragma unroll
    for (int i = 0; i < MC; ++i) {
        const int c = threadIdx.x + i * kNormThreads;
        if (c < n_chunks) {
            Chunk<T> cx;
            if constexpr (SPLIT) {
#pragma unroll
                for (int q = 0; q < Q; ++q) {
                    f32x4 acc = pv[i][0][q];
#pragma unroll
                    for (int sl = 0; sl < KS; ++sl) acc += pv[i][1 + sl][q];
#pragma unroll
                    for (int e = 0; e < 4; ++e) cx.v[4 * q + e] = from_f32<T>(acc[e]);
                }
            } else {
                cx = cxs[i];
            }
            if (rr) {
#pragma unroll
                for (int e = 0; e < E; ++e) cx.v[e] = from_f32<T>(to_f32(cx.v[e]) + to_f32(crs[i].v[e]));
            }
            if (sum_out && (rr || SPLIT)) store_chunk(sum_out + row * dim + c * E, cx);
#pragma unroll
            for (int e = 0; e < E; ++e) {
                v[i][e] = to_f32(cx.v[e]);
                ss = __builtin_fmaf(v[i][e], v[i][e], ss);
            }
        }
    }
    float inv = rsqrtf(block_sum_256(ss, red) / (float)dim + eps);

    float ss2 = 0.f;
#pragma unroll
    for (int i = 0; i < MC; ++i) {
        const int c = threadIdx.x + i * kNormThreads;
        if (c < n_chunks) {
            const Chunk<T> w1 = EARLY ? cw[EARLY ? i : 0] : load_chunk(weight + c * E);
            Chunk<T> co;
#pragma unroll
            for (int e = 0; e < E; ++e) {
                co.v[e] = from_f32<T>(round_to<T>(v[i][e] * inv) * to_f32(w1.v[e]));
                v[i][e] = to_f32(co.v[e]);
                ss2 = __builtin_fmaf(v[i][e], v[i][e], ss2);
            }
            if (y) store_chunk(y + row * ldy + c * E, co);
        }
    }
    // padded rows: the pad is written as zeros, so that a product may also run over the padded length
    if (y && ldy > dim && (int)threadIdx.x < (ldy - dim) / E) store_chunk(y + row * ldy + dim + threadIdx.x * E, zero_chunk<T>());
    if (weight2 == nullptr) return;

    inv = rsqrtf(block_sum_256(ss2, red) / (float)dim + eps);
#pragma unroll
    for (int i = 0; i < MC; ++i) {
        const int c = threadIdx.x + i * kNormThreads;
        if (c < n_chunks) {
            const Chunk<T> w2 = EARLY ? cw2[EARLY ? i : 0] : load_chunk(weight2 + c * E);
            Chunk<T> co;
#pragma unroll
            for (int e = 0; e < E; ++e) co.v[e] = from_f32<T>(round_to<T>(v[i][e] * inv) * to_f32(w2.v[e]));
            store_chunk(y2 + row * ldy2 + c * E, co);
        }
    }
    if (ldy2 > dim && (int)threadIdx.x < (ldy2 - dim) / E) store_chunk(y2 + row * ldy2 + dim + threadIdx.x * E, zero_chunk<T>());
}

int g_norm_early = -1;  // raven_set_tuning("norm_early"): -1 = by row count, 0 / 1 = weights fetched late / early

// The second launch of a K-split product (its slices added in order, rounded, plus the residual) and the RMSNorm(s) that
// consume the result, as one launch: bf16, up to 32 rows of at most 8192 columns.  sum_out (may be null) receives the
// product's value, y (may be null) the first norm's, y2 the second's when weight2 is given.
int splitk_sums_then_norm(const float* partial, int ks, const float* extra, const void* residual, void* sum_out, const void* weight,
                          void* y, const void* weight2, void* y2, int rows, int dim, float eps, hipStream_t s, int ldy, int ldy2) {
    RAVEN_REQUIRE(partial && ks >= 1 && weight && (y || y2) && (weight2 == nullptr) == (y2 == nullptr), "splitk_sums_then_norm: bad arguments");
    if (ldy <= 0) ldy = dim;
    if (ldy2 <= 0) ldy2 = dim;
    RAVEN_REQUIRE(ldy >= dim && ldy2 >= dim && ldy % 8 == 0 && ldy2 % 8 == 0 && ldy - dim <= 8 * kNormThreads && ldy2 - dim <= 8 * kNormThreads,
                  "splitk_sums_then_norm: bad output row pitch %d / %d", ldy, ldy2);
    RAVEN_REQUIRE(rows >= 1 && dim % 8 == 0 && dim / 8 <= kNormThreads * 4, "splitk_sums_then_norm: unsupported shape %d x %d", rows, dim);
    SplitSums sp{partial, extra, ks, (int64_t)rows * dim};
#define RAVEN_SPLIT_NORM(KS_)                                                                                            \
    case KS_:                                                                                                           \
        rmsnorm_kernel<bf16, 4, true, KS_><<<dim3((unsigned)rows), dim3(kNormThreads), 0, s>>>(                          \
            nullptr, (const bf16*)residual, (const bf16*)weight, (bf16*)y, (bf16*)sum_out, (const bf16*)weight2, (bf16*)y2, dim, eps, sp, ldy, ldy2); \
        break;
    switch (ks) {
        RAVEN_SPLIT_NORM(1) RAVEN_SPLIT_NORM(2) RAVEN_SPLIT_NORM(3) RAVEN_SPLIT_NORM(4)
        RAVEN_SPLIT_NORM(5) RAVEN_SPLIT_NORM(6) RAVEN_SPLIT_NORM(7) RAVEN_SPLIT_NORM(8)
        default: RAVEN_REQUIRE(false, "splitk_sums_then_norm: %d slices (at most 8)", ks);
    }
#undef RAVEN_SPLIT_NORM
    return raven_host::check_launch("split-K sums + rmsnorm");
}

}  // namespace raven

namespace raven {
// raven_rmsnorm_residual with the rows of y and of y2 ldy and ldy2 elements apart (>= dim)
int rmsnorm_pitched(const void* x, const void* residual, const void* weight, void* y, int ldy, void* sum_out, const void* weight2,
                    void* y2, int ldy2, int64_t rows, int32_t dim, float eps, int32_t dtype, void* stream) {
    RAVEN_REQUIRE(dtype == RAVEN_F32 || dtype == RAVEN_BF16, "rmsnorm: unknown dtype %d", dtype);
    if (rows == 0) return 0;  // an empty tensor has no storage to point at
    RAVEN_REQUIRE(x && weight && (y || y2), "rmsnorm: null x / weight / output");
    RAVEN_REQUIRE((weight2 == nullptr) == (y2 == nullptr), "rmsnorm: weight2 and y2 must be given together");
    RAVEN_REQUIRE(sum_out == nullptr || residual != nullptr, "rmsnorm: sum_out needs a residual");
    const int elts = 16 / (int)raven_host::elt_size(dtype);
    RAVEN_REQUIRE(dim > 0 && dim % elts == 0, "rmsnorm: dim %d is not a multiple of %d", dim, elts);
    RAVEN_REQUIRE(dim / elts <= kNormThreads * kNormMaxChunks, "rmsnorm: dim %d too large (max %d)", dim,
                  kNormThreads * kNormMaxChunks * elts);
    RAVEN_REQUIRE(rows > 0 && rows < (1ll << 31), "rmsnorm: bad row count %lld", (long long)rows);
    RAVEN_REQUIRE(ldy >= dim && ldy2 >= dim && ldy % elts == 0 && ldy2 % elts == 0 && ldy - dim <= elts * kNormThreads &&
                      ldy2 - dim <= elts * kNormThreads, "rmsnorm: bad output row pitch %d / %d", ldy, ldy2);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int per_thread = (dim / elts + kNormThreads - 1) / kNormThreads;
    const bool early = g_norm_early >= 0 ? g_norm_early != 0 : rows <= 64;
    const SplitSums none{};
#define RAVEN_NORM_LAUNCH(T_, MC_)                                                                                           \
    do {                                                                                                                     \
        if (early)                                                                                                           \
            rmsnorm_kernel<T_, MC_, true, 0><<<dim3((unsigned)rows), dim3(kNormThreads), 0, s>>>(                        \
                (const T_*)x, (const T_*)residual, (const T_*)weight, (T_*)y, (T_*)sum_out, (const T_*)weight2, (T_*)y2, dim, eps, none, ldy, ldy2); \
        else                                                                                                                 \
            rmsnorm_kernel<T_, MC_, false, 0><<<dim3((unsigned)rows), dim3(kNormThreads), 0, s>>>(                       \
                (const T_*)x, (const T_*)residual, (const T_*)weight, (T_*)y, (T_*)sum_out, (const T_*)weight2, (T_*)y2, dim, eps, none, ldy, ldy2); \
    } while (0)
    if (dtype == RAVEN_BF16) {
        if (per_thread <= 4) RAVEN_NORM_LAUNCH(bf16, 4);
        else if (per_thread <= 8) RAVEN_NORM_LAUNCH(bf16, 8);
        else RAVEN_NORM_LAUNCH(bf16, 16);
    } else {
        if (per_thread <= 4) RAVEN_NORM_LAUNCH(float, 4);
        else if (per_thread <= 8) RAVEN_NORM_LAUNCH(float, 8);
        else RAVEN_NORM_LAUNCH(float, 16);
    }
#undef RAVEN_NORM_LAUNCH
    return raven_host::check_launch("rmsnorm");
}
}  // namespace raven

extern "C" int raven_rmsnorm_residual(const void* x, const void* residual, const void* weight, void* y,
                                      void* sum_out, const void* weight2, void* y2, int64_t rows, int32_t dim,
                                      float eps, int32_t dtype, void* stream) {
    return raven::rmsnorm_pitched(x, residual, weight, y, dim, sum_out, weight2, y2, dim, rows, dim, eps, dtype, stream);
}

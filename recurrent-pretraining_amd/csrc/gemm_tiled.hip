// Tiled MFMA GEMM for many token rows (prefill chunks, wide decode batches): Y[M,N] = concat(X0, X1)[M,K] W[N,K]^T in
// bf16 with fp32 accumulation -- the nn.Linear products of the reference at M = B*S rows
// (recpre/raven_modeling_minimal.py:463 Wqkv, 493 attn.proj, 507-509 mlp.fc / SwiGLU / mlp.proj, 776 adapter over
// cat([x, input_embeds]), 711 lm_head), with the epilogues of the skinny kernels: plain, + residual (RMM:534-535),
// float store (RMM:711), SwiGLU (RMM:507-508).  The concat of RMM:776 is two K segments of the X operand.
//
// Shape of the kernel (gfx950):
//   * a workgroup of 8 waves owns a BN x BM tile of Y^T (BN weight rows x BM token rows, 256 x 256 in the main
//     variant); wave (wm, wn) owns TN x TM MFMA tiles of 32 x 32 (v_mfma_f32_32x32x16_bf16, W rows as the A operand, X
//     rows as B, so that a lane ends up with 4 neighbouring output columns of one token row);
//   * K advances in steps of 32 through a ring of LDS stages.  A stage holds BN + BM rows of 64 bytes; it is filled by
//     global -> LDS loads that never touch registers (16 bytes per lane, a wave instruction fills 1 KB = 16 rows).
//     The 16-byte pieces of a row are stored in an order permuted by the row number ((row >> 2) & 3), chosen on the
//     global side of the load, so that the 16 lanes of a quarter wave, which read the same piece of 16 neighbouring
//     rows, hit all 64 banks;
//   * the waves work in two groups of four (one wave of each group per SIMD) half a step apart: while one group
//     multiplies the fragments it holds, the other issues its loads for three steps ahead and reads its fragments of
//     the next step out of LDS; two workgroup barriers per step keep the groups in that rhythm.  The matrix pipe of a
//     SIMD then always has one wave that does nothing but MFMAs;
//   * workgroups are numbered so that the 32 that run together on one XCD (ids congruent modulo 8) cover 8 x 4
//     neighbouring tiles and find each other's panels in that XCD's L2.
//   * SwiGLU: a 32-row A tile holds 16 gate rows and the 16 matching up rows, so gate and up of one output element
//     sit in the same lane, 8 accumulator registers apart.
// M, N and the last tile: rows past the end are clamped on the load side and not stored.  K0 and K1 are multiples of 32.

#include <type_traits>
#include <utility>

#include "raven_common.h"

namespace raven {

struct TiledArgs {
    const bf16* w;         // [N or 2N, K0 + K1]
    const bf16* x0;        // [M, K0]
    const bf16* x1;        // [M, K1] or null
    const bf16* residual;  // [M, N] or null
    void* y;               // [M, N] bf16, or float when out_f32
    int M, N, K0, K1;      // N = output columns (I for SwiGLU)
    int out_f32;
    int tiles_m, tiles_n;
};

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) unsigned char lds_byte;

template <int... I, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F&&>(f));
}

// LDS read that the compiler does not see as one: it would otherwise order every such read behind all outstanding
// global -> LDS loads.  The result is valid after wait_lds().
template <int OFF>
__device__ __forceinline__ void lds_read16(u32x4& dst, unsigned addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}

template <bool SWIGLU, int TM, int TN, int STAGES>
__global__ __launch_bounds__(512) void gemm_tiled_kernel(TiledArgs a) {
    constexpr int BM = 2 * TM * 32, BN = 4 * TN * 32;
    constexpr int ROWS = BN + BM;              // LDS rows of a stage: the W tile, then the X tile
    constexpr int STAGE_BYTES = ROWS * 64;
    constexpr int LPW = ROWS / 16 / 8;         // global -> LDS instructions per wave and stage
    static_assert(ROWS % 128 == 0 && (BN / 16) % LPW == 0, "a wave loads rows of one operand only");
    constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;  // output columns per tile
    extern __shared__ __align__(1024) unsigned char smem[];

    // ---- which tile -----------------------------------------------------------------------------------------------
    const int n_tiles = a.tiles_m * a.tiles_n;
    const int per_xcd = (n_tiles + 7) >> 3;
    const int logical = ((int)blockIdx.x & 7) * per_xcd + ((int)blockIdx.x >> 3);
    if (logical >= n_tiles) return;
    constexpr int GROUP = 8;
    const int band = logical / (GROUP * a.tiles_n);
    const int first_m = band * GROUP;
    const int gsz = min(a.tiles_m - first_m, GROUP);
    const int in_band = logical - band * GROUP * a.tiles_n;
    const int tile_n = in_band / gsz;
    const int tile_m = first_m + (in_band - tile_n * gsz);

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wn = wave & 3, wm = wave >> 2;
    const int K = a.K0 + a.K1;
    const int nk0 = a.K0 >> 5, nk = K >> 5;

    // ---- global -> LDS: this wave fills rows (wave * LPW + jj) * 16 ..+15 of every stage ---------------------------
    const bool loads_w = wave * LPW < BN / 16;
    const int piece = (lane & 3) ^ (lane >> 4);   // the piece this lane fetches so that slot (lane & 3) of its row holds it
    int rowidx[LPW];
#pragma unroll
    for (int jj = 0; jj < LPW; ++jj) {
        const int r = (wave * LPW + jj) * 16 + (lane >> 2);
        if (loads_w) {
            if (SWIGLU) {
                const int col = min(tile_n * BN_OUT + (r >> 5) * 16 + (r & 15), a.N - 1);
                rowidx[jj] = col + ((r & 16) ? a.N : 0);
            } else {
                rowidx[jj] = min(tile_n * BN + r, a.N - 1);
            }
        } else {
            rowidx[jj] = min(tile_m * BM + (r - BN), a.M - 1);
        }
    }
    lds_byte* const lds0 = (lds_byte*)smem;
    auto issue = [&](int kk, int buf) {
        const bf16* base;
        int ld, kcol;
        if (loads_w) { base = a.w; ld = K; kcol = kk << 5; }
        else if (kk < nk0) { base = a.x0; ld = a.K0; kcol = kk << 5; }
        else { base = a.x1; ld = a.K1; kcol = (kk - nk0) << 5; }
        lds_byte* dst = lds0 + buf * STAGE_BYTES + wave * (LPW * 1024);
#pragma unroll
        for (int jj = 0; jj < LPW; ++jj) {
            const bf16* src = base + ((int64_t)rowidx[jj] * ld + kcol + piece * 8);
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src, dst + jj * 1024, 16, 0, 0);
        }
    };

    // ---- LDS -> registers: fragment addresses ------------------------------------------------------------------------
    const int l32 = lane & 31, hi = lane >> 5;
    const int swz = (l32 >> 2) & 3;
    const unsigned lds_base = (unsigned)(uintptr_t)lds0;
    unsigned a_addr[2], b_addr[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        const int pos = ((2 * ks + hi) ^ swz) * 16;
        a_addr[ks] = lds_base + (wn * TN * 32 + l32) * 64 + pos;
        b_addr[ks] = lds_base + (BN + wm * TM * 32 + l32) * 64 + pos;
    }

    f32x16 acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[tn][tm][e] = 0.f;

    u32x4 fa[2][TN], fb[2][TM];
    auto read_frags = [&](int buf) {
        const unsigned off = buf * STAGE_BYTES;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            static_for<TN>([&](auto t) { lds_read16<decltype(t)::value * 2048>(fa[ks][decltype(t)::value], a_addr[ks] + off); });
            static_for<TM>([&](auto t) { lds_read16<decltype(t)::value * 2048>(fb[ks][decltype(t)::value], b_addr[ks] + off); });
        }
    };
    auto wait_lds = [&]() {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
            for (int t = 0; t < TN; ++t) asm volatile("" : "+v"(fa[ks][t]));
#pragma unroll
            for (int t = 0; t < TM; ++t) asm volatile("" : "+v"(fb[ks][t]));
        }
    };
    auto multiply = [&]() {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int tn = 0; tn < TN; ++tn)
#pragma unroll
                for (int tm = 0; tm < TM; ++tm)
                    acc[tn][tm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa[ks][tn]),
                                                                          __builtin_bit_cast(bf16x8, fb[ks][tm]), acc[tn][tm], 0, 0, 0);
    };

    // ---- the K loop -------------------------------------------------------------------------------------------------
    // Loads of step kk land in stage kk % STAGES.  A wave waits for its own loads of step k + 1 at the end of its
    // memory phase of step k, in front of a barrier; every reader of that stage starts behind that barrier.  A stage is
    // overwritten (loads of step k + STAGES - 1, issued in the memory phase of step k) one barrier after the other
    // group has finished reading step k - 1 from it.
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s)
        if (s < nk) issue(s, s);
    if (nk > STAGES - 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((STAGES - 2) * LPW) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    if (wm == 1) __builtin_amdgcn_s_barrier();  // the second group runs half a step behind

    int buf = 0, buf_load = STAGES - 1;
    for (int k = 0; k < nk; ++k) {
        // memory phase
        const bool more = k + STAGES - 1 < nk;
        if (more) issue(k + STAGES - 1, buf_load);
        read_frags(buf);
        wait_lds();
        if (more) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((STAGES - 2) * LPW) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        // compute phase
        __builtin_amdgcn_s_setprio(1);
        multiply();
        __builtin_amdgcn_s_setprio(0);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        buf = buf + 1 == STAGES ? 0 : buf + 1;
        buf_load = buf_load + 1 == STAGES ? 0 : buf_load + 1;
    }
    if (wm == 0) __builtin_amdgcn_s_barrier();

    // ---- epilogue: lane holds, for token row m = .. + l32, output columns 8 j + 4 hi + (0..3) of each 32-row A tile ----
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
        const int m = tile_m * BM + (wm * TM + tm) * 32 + l32;
        if (m >= a.M) continue;
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
            const int t32 = wn * TN + tn;
            if (SWIGLU) {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int n = tile_n * BN_OUT + t32 * 16 + 8 * j + 4 * hi;
                    if (n >= a.N) continue;
                    bf16 o[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float g = round_to<bf16>(acc[tn][tm][4 * j + i]), u = round_to<bf16>(acc[tn][tm][8 + 4 * j + i]);
                        o[i] = from_f32<bf16>(round_to<bf16>(silu_f32(g)) * u);
                    }
                    *reinterpret_cast<u32x2*>(static_cast<bf16*>(a.y) + (int64_t)m * a.N + n) = *reinterpret_cast<const u32x2*>(o);
                }
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int n = tile_n * BN + t32 * 32 + 8 * j + 4 * hi;
                    if (n >= a.N) continue;
                    float r[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) r[i] = round_to<bf16>(acc[tn][tm][4 * j + i]);
                    if (a.residual) {
                        bf16 res[4];
                        *reinterpret_cast<u32x2*>(res) = *reinterpret_cast<const u32x2*>(a.residual + (int64_t)m * a.N + n);
#pragma unroll
                        for (int i = 0; i < 4; ++i) r[i] = round_to<bf16>(r[i] + to_f32(res[i]));
                    }
                    if (a.out_f32) {
                        *reinterpret_cast<f32x4*>(static_cast<float*>(a.y) + (int64_t)m * a.N + n) = f32x4{r[0], r[1], r[2], r[3]};
                    } else {
                        bf16 o[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) o[i] = from_f32<bf16>(r[i]);
                        *reinterpret_cast<u32x2*>(static_cast<bf16*>(a.y) + (int64_t)m * a.N + n) = *reinterpret_cast<const u32x2*>(o);
                    }
                }
            }
        }
    }
}

int g_tiled_min_rows = 33;  // raven_set_tuning("gemm_tiled_min_rows"): fewest rows that take this kernel
int g_tiled_variant = 0;  // raven_set_tuning("gemm_tiled_variant"): 0 = by shape, 1 = 256 x 256 tiles, 2 = 128 x 128 tiles

template <bool SWIGLU, int TM, int TN>
static int launch_tiled(TiledArgs a, hipStream_t s) {
    constexpr int STAGES = 4;
    constexpr int BM = 2 * TM * 32, BN = 4 * TN * 32, BN_OUT = SWIGLU ? BN / 2 : BN;
    constexpr size_t lds = (size_t)STAGES * (BM + BN) * 64;
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_tiled_kernel<SWIGLU, TM, TN, STAGES>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) {
            raven_host::set_error("gemm (tiled): hipFuncSetAttribute failed: %s", hipGetErrorString(e));
            return (int)e;
        }
        attr_set = true;
    }
    a.tiles_m = (a.M + BM - 1) / BM;
    a.tiles_n = (a.N + BN_OUT - 1) / BN_OUT;
    const int64_t n_tiles = (int64_t)a.tiles_m * a.tiles_n;
    RAVEN_REQUIRE(n_tiles < (1 << 28), "gemm (tiled): too many tiles (M=%d N=%d)", a.M, a.N);
    const unsigned grid = (unsigned)((n_tiles + 7) / 8 * 8);
    gemm_tiled_kernel<SWIGLU, TM, TN, STAGES><<<dim3(grid), dim3(512), lds, s>>>(a);
    return raven_host::check_launch("gemm (tiled MFMA)");
}

// Host entry for the other translation units: true when the shape is one the tiled kernel takes.
bool tiled_gemm_fits(int M, int N, int K0, int K1, int dtype) {
    return dtype == RAVEN_BF16 && M >= 1 && N % 8 == 0 && K0 % 32 == 0 && K1 % 32 == 0 && K0 + K1 >= 32;
}

int tiled_gemm(const void* x0, const void* x1, const void* w, const void* residual, void* y, int M, int N, int K0, int K1, int swiglu,
               int out_f32, hipStream_t s) {
    RAVEN_REQUIRE(tiled_gemm_fits(M, N, K0, K1, RAVEN_BF16), "gemm (tiled): unsupported shape M=%d N=%d K0=%d K1=%d", M, N, K0, K1);
    RAVEN_REQUIRE(!(swiglu && (residual || out_f32)), "gemm (tiled): the SwiGLU epilogue has no residual and stores bf16");
    RAVEN_REQUIRE(((uintptr_t)x0 & 15) == 0 && ((uintptr_t)x1 & 15) == 0 && ((uintptr_t)w & 15) == 0 && ((uintptr_t)y & 15) == 0 &&
                      ((uintptr_t)residual & 7) == 0, "gemm (tiled): operands must be 16-byte aligned");
    TiledArgs a{};
    a.w = static_cast<const bf16*>(w);
    a.x0 = static_cast<const bf16*>(x0);
    a.x1 = static_cast<const bf16*>(x1);
    a.residual = static_cast<const bf16*>(residual);
    a.y = y;
    a.M = M; a.N = N; a.K0 = K0; a.K1 = x1 ? K1 : 0; a.out_f32 = out_f32;
    // 256 x 256 tiles when they fill the chip at least once; 128 x 128 tiles otherwise
    const int64_t big_tiles = (int64_t)((M + 255) / 256) * ((N + (swiglu ? 127 : 255)) / (swiglu ? 128 : 256));
    const bool big = g_tiled_variant == 1 || (g_tiled_variant == 0 && big_tiles >= 256);
    if (swiglu) return big ? launch_tiled<true, 4, 2>(a, s) : launch_tiled<true, 2, 1>(a, s);
    return big ? launch_tiled<false, 4, 2>(a, s) : launch_tiled<false, 2, 1>(a, s);
}

}  // namespace raven

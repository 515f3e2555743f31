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
    unsigned long long* dbg;  // experiments only
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

// Epilogue of both kernels.  A lane holds, for token row m = .. + l32, output columns 8 j + 4 hi + (0 .. 3) of each
// 32-row A tile (SwiGLU: gate columns in registers 0 .. 7, the matching up columns in 8 .. 15).
template <bool SWIGLU, int TM, int TN>
__device__ __forceinline__ void store_tiles(const TiledArgs& a, const f32x16 (&acc)[TN][TM], int tile_m, int tile_n, int wm, int wn,
                                            int l32, int hi) {
    constexpr int BM = 2 * TM * 32, BN = 4 * TN * 32, BN_OUT = SWIGLU ? BN / 2 : BN;
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

__device__ __align__(16) unsigned int g_zero_piece[4];  // what a 16-byte piece past the end of K is loaded from

template <bool SWIGLU, int TM, int TN, int EXP = 0, int PFD = 0>
__global__ __launch_bounds__(512) void gemm_tiled_kernel(TiledArgs a) {
    constexpr int BM = 2 * TM * 32, BN = 4 * TN * 32;
    constexpr int ROWS = BN + BM;              // LDS rows of a stage: the W tile, then the X tile
    constexpr int STAGE_BYTES = ROWS * 128;
    constexpr int LPW = ROWS / 8 / 8;          // global -> LDS instructions (8 rows each) per wave and stage
    static_assert(ROWS % 64 == 0 && (BN / 8) % LPW == 0 && LPW % 2 == 0, "a wave loads rows of one operand only");
    constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;
    constexpr int NM = TN * TM;                // MFMAs per k-slice
    // the loads of a step are issued in three portions, under the products of three k-slices
    constexpr int P0 = (LPW * 3 + 7) / 8, P1 = (LPW * 6 + 7) / 8;
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
    const int nk = (K + 63) >> 6;

    // ---- global -> LDS: this wave fills rows (wave * LPW + jj) * 8 ..+7 of every stage -------------------------------
    const bool loads_w = wave * LPW < BN / 8;
    int rowidx[LPW];
#pragma unroll
    for (int jj = 0; jj < LPW; ++jj) {
        const int r = (wave * LPW + jj) * 8 + (lane >> 3);
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
    // column (in elements) of the piece this lane fetches, for instructions of even / odd index: slot (lane & 7) of row
    // r holds piece (lane & 7) ^ ((r >> 1) & 7)
    int pcol[2];
#pragma unroll
    for (int par = 0; par < 2; ++par) pcol[par] = ((lane & 7) ^ ((4 * par) | (lane >> 4))) * 8;
    lds_byte* const lds0 = (lds_byte*)smem;
    const bf16* const zero = reinterpret_cast<const bf16*>(g_zero_piece);
    // where a step's pieces come from: when the whole step lies inside one segment, one base pointer for all lanes
    // and a 32-bit offset per lane
    struct StepSrc {
        const char* base;
        unsigned ld2;  // row pitch in bytes
        int kk;
        bool uniform, live;
    };
    auto step_src = [&](int kk) {
        StepSrc s;
        const int k0 = kk << 6;
        s.kk = kk;
        s.live = kk < nk;
        s.uniform = loads_w ? (k0 + 64 <= K) : (k0 + 64 <= a.K0 || (k0 >= a.K0 && k0 + 64 <= K));
        if (loads_w) { s.base = reinterpret_cast<const char*>(a.w + k0); s.ld2 = 2u * K; }
        else if (k0 < a.K0) { s.base = reinterpret_cast<const char*>(a.x0 + k0); s.ld2 = 2u * a.K0; }
        else { s.base = reinterpret_cast<const char*>(a.x1 + (k0 - a.K0)); s.ld2 = 2u * a.K1; }
        return s;
    };
    // one instruction: piece jj of a step into stage kk & 1
    auto issue = [&](const StepSrc& s, auto jj_tag) {
        constexpr int jj = decltype(jj_tag)::value;
        if ((EXP & 2) || !s.live) return;
        lds_byte* dst = lds0 + (s.kk & 1) * STAGE_BYTES + wave * (LPW * 1024) + jj * 1024;
        if (s.uniform) {
            const unsigned off = __umul24((unsigned)rowidx[jj], s.ld2) + 2u * pcol[jj & 1];
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(s.base + off), dst, 16, 0, 0);
        } else {
            const int col = (s.kk << 6) + pcol[jj & 1];
            const bool second = !loads_w && col >= a.K0;
            const bf16* b = loads_w ? a.w : (second ? a.x1 : a.x0);
            const int ld = loads_w ? K : (second ? a.K1 : a.K0);
            const bf16* src = b + ((int64_t)rowidx[jj] * ld + (second ? col - a.K0 : col));
            if (col >= K) src = zero;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src, dst, 16, 0, 0);
        }
    };

    // ---- L2 prefetch (PFD > 0): PFD steps beyond the loads, one lane touches one 128-byte line.  The workgroups that run
    // together on an XCD share panels (8 token-row tiles per weight panel, 4 weight tiles per token-row panel): each of
    // them touches its share of the lines, wave 0 of the weight panel, wave 4 of the token-row panel.
    const bool does_pf = PFD > 0 && (wave == 0 || wave == 4);
    const char* pf_ptr = nullptr;
    bool pf_lane = false;
    if (PFD > 0) {
        if (wave == 0) {
            const int r = (tile_m & 7) * (BN / 8) + lane;
            pf_lane = lane < BN / 8;
            int g;
            if (SWIGLU) g = min(tile_n * BN_OUT + (r >> 5) * 16 + (r & 15), a.N - 1) + ((r & 16) ? a.N : 0);
            else g = min(tile_n * BN + r, a.N - 1);
            pf_ptr = reinterpret_cast<const char*>(a.w + (int64_t)g * K);
        } else if (wave == 4) {
            const int r = (tile_n & 3) * (BM / 4) + lane;
            pf_lane = lane < BM / 4;
            pf_ptr = reinterpret_cast<const char*>(a.x0 + (int64_t)min(tile_m * BM + r, a.M - 1) * a.K0);
        }
    }
    lds_byte* const pf_dst = lds0 + 2 * STAGE_BYTES;
    const int pf_limit = wave == 0 ? K : a.K0;  // the token-row operand is prefetched inside its first segment only
    auto prefetch = [&](int kk) {  // always one instruction, so that the count of outstanding loads stays uniform
        int k0 = kk << 6;
        if (kk >= nk || k0 + 64 > pf_limit) k0 = 0;
        if (pf_lane) __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(pf_ptr + 2 * k0), pf_dst, 4, 0, 0);
    };

    // ---- LDS -> registers -------------------------------------------------------------------------------------------
    const int l32 = lane & 31, hi = lane >> 5;
    const int swz = (l32 >> 1) & 7;
    const unsigned lds_base = (unsigned)(uintptr_t)lds0;
    const unsigned a_row = lds_base + (wn * TN * 32 + l32) * 128;
    const unsigned b_row = lds_base + (BN + wm * TM * 32 + l32) * 128;
    unsigned pos[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) pos[ks] = ((2 * ks + hi) ^ swz) * 16;

    f32x16 acc[TN][TM];
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[tn][tm][e] = 0.f;

    u32x4 fa[2][TN], fb[2][TM];
    auto read_frags = [&](auto ks_tag, int buf) {  // k-slice ks of stage buf into fragment set ks & 1
        constexpr int ks = decltype(ks_tag)::value;
        if (EXP & 4) return;
        const unsigned off = buf * STAGE_BYTES + pos[ks];
        static_for<TN>([&](auto t) { lds_read16<decltype(t)::value * 4096>(fa[ks & 1][decltype(t)::value], a_row + off); });
        static_for<TM>([&](auto t) { lds_read16<decltype(t)::value * 4096>(fb[ks & 1][decltype(t)::value], b_row + off); });
    };
    auto settle = [&](int set) {  // the fragments of this set are valid from here on (behind a wait for the LDS counter)
#pragma unroll
        for (int t = 0; t < TN; ++t) asm volatile("" : "+v"(fa[set][t]));
#pragma unroll
        for (int t = 0; t < TM; ++t) asm volatile("" : "+v"(fb[set][t]));
    };
    // the NM products of one k-slice; after(i) is called behind product i
    auto products = [&](int set, auto&& after) {
        static_for<NM>([&](auto it) {
            constexpr int i = decltype(it)::value, tn = i / TM, tm = i % TM;
            if (!(EXP & 8))
                acc[tn][tm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa[set][tn]),
                                                                      __builtin_bit_cast(bf16x8, fb[set][tm]), acc[tn][tm], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            after(it);
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    // portion [LO, HI) of the loads of step kk, spread behind the products 1, 3, 5, ... of a slice
    auto spread = [&](auto it, const StepSrc& src, auto lo_tag, auto hi_tag) {
        constexpr int i = decltype(it)::value, LO = decltype(lo_tag)::value, HI = decltype(hi_tag)::value;
        static_for<HI - LO>([&](auto p) {
            constexpr int slot = 1 + 2 * decltype(p)::value < NM - 1 ? 1 + 2 * decltype(p)::value : NM - 1;
            if (slot == i) issue(src, std::integral_constant<int, LO + decltype(p)::value>{});
        });
    };
    using ic0 = std::integral_constant<int, 0>;

    // ---- the K loop: two stages, one barrier per step -----------------------------------------------------------------
    // Step k is multiplied out of stage k & 1 in four k-slices of 16.  The barrier of step k sits between the products
    // of slices 2 and 3: in front of it every wave has all fragments of the step in registers and its loads of step k + 1
    // have landed, so behind it stage k & 1 may be overwritten (loads of step k + 2: a first portion under the products
    // of slice 3, the rest under slices 0 and 1 of the next step) and stage (k + 1) & 1 may be read.
    StepSrc src1 = step_src(0), src2 = step_src(1);  // inside the loop: the sources of steps k + 1 and k + 2
    static_for<LPW>([&](auto jj) { issue(src1, jj); });
    if (1 < nk) {
        static_for<P0>([&](auto jj) { issue(src2, jj); });
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(P0) : "memory");
    } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __builtin_amdgcn_s_barrier();
    if (does_pf) prefetch(2);  // from here on a prefetch is this wave's youngest load at every wait
    unsigned long long dbg_vm = 0, dbg_bar = 0, dbg_t0 = 0;
    unsigned long long dbg_r0 = 0;
    if (EXP & 64) { dbg_t0 = __builtin_readcyclecounter(); dbg_r0 = __builtin_amdgcn_s_memrealtime(); }
    read_frags(ic0{}, 0);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    settle(0);
    for (int k = 0; k < nk; ++k) {
        const int cur = k & 1;
        src1 = src2;
        src2 = step_src(k + 2);
        static_for<3>([&](auto ks_tag) {
            constexpr int ks = decltype(ks_tag)::value;
            products(ks & 1, [&](auto it) {
                if (decltype(it)::value == 0) read_frags(std::integral_constant<int, ks + 1>{}, cur);
                if (ks == 0) spread(it, src1, std::integral_constant<int, P0>{}, std::integral_constant<int, P1>{});
                if (ks == 1) {
                    spread(it, src1, std::integral_constant<int, P1>{}, std::integral_constant<int, LPW>{});
                    if (decltype(it)::value == NM - 1 && does_pf) prefetch(k + 2 + PFD);
                }
            });
            if (ks < 2) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                settle((ks + 1) & 1);
            }
        });
        unsigned long long t0 = 0, t1 = 0, t2 = 0;
        if (EXP & 64) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            t0 = __builtin_readcyclecounter();
        }
        if (does_pf) asm volatile("s_waitcnt vmcnt(1) lgkmcnt(0)" ::: "memory");  // the prefetch issued last may still be out
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        settle(1);
        if (EXP & 64) t1 = __builtin_readcyclecounter();
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        if (EXP & 64) {
            t2 = __builtin_readcyclecounter();
            dbg_vm += t1 - t0;
            dbg_bar += t2 - t1;
        }
        products(1, [&](auto it) {
            if (decltype(it)::value == 0 && k + 1 < nk) read_frags(ic0{}, cur ^ 1);
            spread(it, src2, ic0{}, std::integral_constant<int, P0>{});
        });
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        settle(0);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if ((EXP & 64) && a.dbg && lane == 0 && blockIdx.x < 64) {
        unsigned long long* d = a.dbg + ((size_t)blockIdx.x * 8 + wave) * 4;
        d[0] = __builtin_readcyclecounter() - dbg_t0;
        d[1] = dbg_vm;
        d[2] = dbg_bar;
        d[3] = ((unsigned long long)nk << 32) | (unsigned)(__builtin_amdgcn_s_memrealtime() - dbg_r0);
    }
    store_tiles<SWIGLU, TM, TN>(a, acc, tile_m, tile_n, wm, wn, l32, hi);
}

int g_tiled_min_rows = 33;  // raven_set_tuning("gemm_tiled_min_rows"): fewest rows that take this kernel
int g_tiled_variant = 0;    // raven_set_tuning("gemm_tiled_variant"): 0 = by shape, 1 = 256 x 256 tiles, 2 = 128 x 128 tiles
int g_tiled_exp = 0;

template <bool SWIGLU, int TM, int TN, int EXP = 0, int PFD = 0>
static int launch_tiled(TiledArgs a, hipStream_t s) {
    constexpr int BM = 2 * TM * 32, BN = 4 * TN * 32, BN_OUT = SWIGLU ? BN / 2 : BN;
    constexpr size_t lds = (size_t)2 * (BM + BN) * 128 + 256;
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_tiled_kernel<SWIGLU, TM, TN, EXP, PFD>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
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
    gemm_tiled_kernel<SWIGLU, TM, TN, EXP, PFD><<<dim3(grid), dim3(512), lds, s>>>(a);
    return raven_host::check_launch("gemm (tiled MFMA)");
}

// Host entry for the other translation units: true when the shape is one the tiled kernel takes.
bool tiled_gemm_fits(int M, int N, int K0, int K1, int dtype) {
    return dtype == RAVEN_BF16 && M >= 1 && N % 8 == 0 && K0 % 8 == 0 && K1 % 8 == 0 && K0 > 0 && (int64_t)M * (K0 > K1 ? K0 : K1) < (1ll << 31) &&
           (int64_t)N * 2 * (K0 + K1) < (1ll << 31);
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
    a.dbg = (g_tiled_exp & 64) ? static_cast<unsigned long long*>(const_cast<void*>(residual)) : nullptr;
    if (a.dbg) a.residual = nullptr;
    // 256 x 256 tiles when they fill the chip at least once; 128 x 128 tiles otherwise
    const int64_t big_tiles = (int64_t)((M + 255) / 256) * ((N + (swiglu ? 127 : 255)) / (swiglu ? 128 : 256));
    const bool big = g_tiled_variant == 1 || (g_tiled_variant == 0 && big_tiles >= 256);
    if (!swiglu && big && g_tiled_exp) {
        switch (g_tiled_exp) {
            case 2: return launch_tiled<false, 4, 2, 2>(a, s);
            case 4: return launch_tiled<false, 4, 2, 4>(a, s);
            case 6: return launch_tiled<false, 4, 2, 6>(a, s);
            case 8: return launch_tiled<false, 4, 2, 8>(a, s);
            case 12: return launch_tiled<false, 4, 2, 12>(a, s);
            case 64: return launch_tiled<false, 4, 2, 64>(a, s);
            case 66: return launch_tiled<false, 4, 2, 66>(a, s);
            case 70: return launch_tiled<false, 4, 2, 70>(a, s);
            case 76: return launch_tiled<false, 4, 2, 76>(a, s);
            case 103: return launch_tiled<false, 4, 2, 0, 3>(a, s);
            case 167: return launch_tiled<false, 4, 2, 64, 3>(a, s);
        }
    }
    if (swiglu) return big ? launch_tiled<true, 4, 2>(a, s) : launch_tiled<true, 2, 1>(a, s);
    return big ? launch_tiled<false, 4, 2>(a, s) : launch_tiled<false, 2, 1>(a, s);
}

}  // namespace raven

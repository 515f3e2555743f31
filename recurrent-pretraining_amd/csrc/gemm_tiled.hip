// Tiled MFMA GEMM for many token rows (prefill chunks, wide decode batches): Y[M,N] = concat(X0, X1)[M,K] W[N,K]^T in
// bf16 with fp32 accumulation -- the nn.Linear products of the reference at M = B*S rows
// (recpre/raven_modeling_minimal.py:463 Wqkv, 493 attn.proj, 507-509 mlp.fc / SwiGLU / mlp.proj, 776 adapter over
// cat([x, input_embeds]), 711 lm_head), with the epilogues of the skinny kernels: plain, + residual (RMM:534-535),
// float store (RMM:711), SwiGLU (RMM:507-508).  The concat of RMM:776 is two K segments of the X operand.
//
// Shape of the kernel (gfx950):
//   * a workgroup of 8 waves (2 along the token rows x 4 along the weight rows, two waves per SIMD) owns a BN x BM tile
//     of Y^T (256 weight rows x 256 token rows in the main variant); a wave owns TN x TM MFMA tiles of 32 x 32
//     (v_mfma_f32_32x32x16_bf16, W rows as the A operand, X rows as B, so that a lane ends up with 4 neighbouring output
//     columns of one token row);
//   * K advances in steps of 64 through two LDS stages of BN + BM rows of 128 bytes.  The 16-byte pieces of a row are
//     kept at position piece ^ ((row >> 1) & 7), so that the 16 lanes of a quarter wave, which read the same piece of 16
//     neighbouring rows, hit all 64 banks;
//   * operands travel global -> registers -> LDS: 8 lanes fetch one whole 128-byte row step (the L1 address path
//     serves full lines at twice the rate of half lines), a wave instruction 8 rows.  Every lane keeps one step of its
//     pieces in registers; a piece is written to LDS one step after it was requested and its registers are reloaded at
//     once, two pieces under the products of each k-slice, so that loads flow evenly and each has a whole step to land;
//   * a step is four k-slices of 16; fragments of the next slice are read from LDS under the products of this one.  One
//     workgroup barrier per step, between the products of slices 2 and 3;
//   * the K loop is one basic block of plain loads, stores and MFMAs with the scheduler pinned between them: the
//     compiler then counts the outstanding loads exactly and waits for one piece at a time;
//   * workgroups are numbered so that the 32 that run together on one XCD (ids congruent modulo 8) cover 8 x 4
//     neighbouring tiles and find each other's panels in that XCD's L2;
//   * SwiGLU: a 32-row A tile holds 16 gate rows and the 16 matching up rows, so gate and up of one output element sit
//     in the same lane, 8 accumulator registers apart.
// M, N and the last tile: rows past the end are clamped on the load side and not stored.  K0 and K1 are multiples of 8
// (pieces past K come from a zero page); two segments share one row pitch (K1 == K0).

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
typedef __attribute__((address_space(3))) u32x4 lds_u32x4;

template <int... I, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F&&>(f));
}

// Epilogue of both kernels.  A lane holds, for token row m = .. + l32, output columns 8 j + 4 hi + (0 .. 3) of each
// 32-row A tile (SwiGLU: gate columns in registers 0 .. 7, the matching up columns in 8 .. 15).
template <bool SWIGLU, int TM, int TN, int WM = 2, int WN = 4>
__device__ __forceinline__ void store_tiles(const TiledArgs& a, const f32x16 (&acc)[TN][TM], int tile_m, int tile_n, int wm, int wn,
                                            int l32, int hi) {
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32, BN_OUT = SWIGLU ? BN / 2 : BN;
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

// Epilogue through LDS for the bf16 outputs: the accumulators (a lane: 4 columns of 32 different token rows per store)
// are laid down as the output tile, rows of BN_OUT columns, and read back so that a wave instruction stores two whole
// tile rows, 16 bytes per lane: full 128-byte lines instead of 32 pieces of 16 bytes.  The residual is fetched the same
// way, before the tile is laid down, so that its latency hides behind the transposition.  16-byte unit u of tile row r
// sits at position u ^ (r mod units per row): the 32 rows a store instruction spreads over then fall on different banks.
template <bool SWIGLU, int TM, int TN, int WM = 2, int WN = 4>
__device__ __forceinline__ void store_tiles_lds(const TiledArgs& a, const f32x16 (&acc)[TN][TM], int tile_m, int tile_n, int wave, int lane,
                                                unsigned lds_base) {
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32, BN_OUT = SWIGLU ? BN / 2 : BN;
    constexpr int RB = BN_OUT * 2, U = RB / 16;      // bytes and 16-byte units per tile row
    constexpr int ITERS = BM * U / (64 * WM * WN);    // 16-byte units per lane
    const int wn = wave % WN, wm = wave / WN, l32 = lane & 31, hi = lane >> 5;
    bf16* const y = static_cast<bf16*>(a.y);
    int64_t goff[ITERS];                             // element offset of this lane's unit in y / residual, -1: outside
    u32x4 res[ITERS];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int idx = (wave * ITERS + it) * 64 + lane;
        const int m = tile_m * BM + idx / U, n = tile_n * BN_OUT + (idx % U) * 8;
        goff[it] = (m < a.M && n < a.N) ? (int64_t)m * a.N + n : -1;
        res[it] = u32x4{0, 0, 0, 0};
        if (!SWIGLU && a.residual && goff[it] >= 0) res[it] = *reinterpret_cast<const u32x4*>(a.residual + goff[it]);
    }
    // every wave has its last fragments; the stages are free
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
        const int row = (wm * TM + tm) * 32 + l32;
        const unsigned row_addr = lds_base + row * RB + hi * 8;
        const int sw = row & (U - 1);
#pragma unroll
        for (int tn = 0; tn < TN; ++tn) {
            const int t32 = wn * TN + tn;
#pragma unroll
            for (int j = 0; j < (SWIGLU ? 2 : 4); ++j) {
                bf16 o[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (SWIGLU) {
                        const float g = round_to<bf16>(acc[tn][tm][4 * j + i]), u = round_to<bf16>(acc[tn][tm][8 + 4 * j + i]);
                        o[i] = from_f32<bf16>(round_to<bf16>(silu_f32(g)) * u);
                    } else {
                        o[i] = from_f32<bf16>(acc[tn][tm][4 * j + i]);
                    }
                }
                const int unit = t32 * (SWIGLU ? 2 : 4) + j;
                *reinterpret_cast<__attribute__((address_space(3))) u32x2*>(row_addr + ((unit ^ sw) * 16)) = *reinterpret_cast<const u32x2*>(o);
            }
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int idx = (wave * ITERS + it) * 64 + lane;
        const int row = idx / U, unit = idx % U;
        u32x4 v = *reinterpret_cast<const lds_u32x4*>(lds_base + row * RB + ((unit ^ (row & (U - 1))) * 16));
        if (!SWIGLU && a.residual) {
            bf16 o[8], r[8];
            *reinterpret_cast<u32x4*>(o) = v;
            *reinterpret_cast<u32x4*>(r) = res[it];
#pragma unroll
            for (int i = 0; i < 8; ++i) o[i] = from_f32<bf16>(to_f32(o[i]) + to_f32(r[i]));
            v = *reinterpret_cast<const u32x4*>(o);
        }
        if (goff[it] >= 0) *reinterpret_cast<u32x4*>(y + goff[it]) = v;
    }
}

__device__ __align__(16) unsigned int g_zero_piece[4];  // what a 16-byte piece past the end of K is loaded from

template <bool SWIGLU, int TM, int TN, int WM = 2, int WN = 4>
__global__ __launch_bounds__(64 * WM * WN) void gemm_tiled_kernel(TiledArgs a) {
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    constexpr int NWAVES = WM * WN;
    constexpr int ROWS = BN + BM;              // LDS rows of a stage: the W tile, then the X tile
    constexpr int STAGE_BYTES = ROWS * 128;
    constexpr int LPW = ROWS / 8 / NWAVES;     // 16-byte pieces per lane and step: piece p of a wave = 8 rows x 128 bytes
    static_assert(ROWS % (32 * NWAVES) == 0 && (BN / 8) % LPW == 0, "a wave loads rows of one operand only, the same number under every k-slice");
    constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;
    constexpr int NM = TN * TM;                // MFMAs per k-slice
    constexpr int PPS = LPW / 4;               // pieces handled under the products of one k-slice
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
    const int wn = wave % WN, wm = wave / WN;
    const int K = a.K0 + a.K1;
    const int nk = (K + 63) >> 6;

    // ---- global -> registers -> LDS: this wave moves rows (wave * LPW + p) * 8 ..+7 of every stage, piece p = one
    // instruction; lane l brings bytes 16 (l & 7) ..+15 of the 128-byte row step of row l >> 3 --------------------------
    const bool loads_w = wave * LPW < BN / 8;
    const int col8 = (lane & 7) * 8;           // this lane's column inside a step, in elements
    unsigned goff[LPW];                        // byte offset of this lane's row + column inside its operand (both segments
                                               // of the token rows have one row pitch)
    const unsigned ld2 = 2u * (loads_w ? K : a.K0);
#pragma unroll
    for (int p = 0; p < LPW; ++p) {
        const int r = (wave * LPW + p) * 8 + (lane >> 3);
        int row;
        if (loads_w) {
            if (SWIGLU) row = min(tile_n * BN_OUT + (r >> 5) * 16 + (r & 15), a.N - 1) + ((r & 16) ? a.N : 0);
            else row = min(tile_n * BN + r, a.N - 1);
        } else {
            row = min(tile_m * BM + (r - BN), a.M - 1);
        }
        goff[p] = (unsigned)row * ld2 + 2u * col8;
    }
    // LDS slot of the piece: row r keeps piece c at position c ^ ((r >> 1) & 7); (r >> 1) & 7 = (lane >> 4) | 4 (p & 1)
    const unsigned lds_base = (unsigned)(uintptr_t)(lds_byte*)smem;
    unsigned wr_addr[2];
#pragma unroll
    for (int par = 0; par < 2; ++par)
        wr_addr[par] = lds_base + (wave * LPW * 8 + (lane >> 3)) * 128 + (((lane & 7) ^ ((lane >> 4) | (4 * par))) * 16);
    const char* const zero = reinterpret_cast<const char*>(g_zero_piece);
    const char* const seg0 = reinterpret_cast<const char*>(loads_w ? a.w : a.x0);
    const char* const seg1 = reinterpret_cast<const char*>(a.x1) - 2 * (int64_t)a.K0;  // column c >= K0 of the token rows
    const int k_split = loads_w ? K : a.K0;    // columns from here on come from the second segment

    // Plain loads and stores, and no branch inside the K loop: the compiler then knows the order of all outstanding loads
    // and waits, in front of the LDS write of a piece, for exactly that piece's load (issued one step earlier).
    // Where this lane's 16 bytes of step kk come from: its segment's pointer (rebased so that the piece's offset is
    // goff[p] + 2 * 64 kk), or the zero page for columns past K -- which is every column of a step past the last one.
    struct StepSrc {
        const char* base;
        bool past;  // this lane's column lies past K
    };
    auto step_src = [&](int kk) {
        const int col = (kk << 6) + col8;
        StepSrc s;
        s.past = col >= K;
        s.base = s.past ? zero : (col < k_split ? seg0 : seg1) + 2 * (kk << 6);
        return s;
    };
    u32x4 stg[LPW];
    auto load_piece = [&](const StepSrc& src, auto p_tag) {
        constexpr int p = decltype(p_tag)::value;
        stg[p] = *reinterpret_cast<const u32x4*>(src.base + (src.past ? 0u : goff[p]));
    };
    auto store_piece = [&](int kk, auto p_tag) {
        constexpr int p = decltype(p_tag)::value;
        *reinterpret_cast<lds_u32x4*>(wr_addr[p & 1] + (kk & 1) * STAGE_BYTES + p * 1024) = stg[p];
    };
    // Piece p of step j moves on: into stage j & 1; the registers take the piece of step j + 1 (source: next).
    auto move_piece = [&](int j, const StepSrc& next, auto p_tag) {
        store_piece(j, p_tag);
        load_piece(next, p_tag);
    };

    // ---- LDS -> registers -------------------------------------------------------------------------------------------
    const int l32 = lane & 31, hi = lane >> 5;
    const int swz = (l32 >> 1) & 7;
    const unsigned a_row = lds_base + (wn * TN * 32 + l32) * 128;
    const unsigned b_row = lds_base + (BN + wm * TM * 32 + l32) * 128;
    const unsigned pos0 = (hi ^ swz) * 16;     // position of k-slice ks: pos0 ^ (32 ks)

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
        const unsigned off = buf * STAGE_BYTES + (pos0 ^ (32 * ks));
#pragma unroll
        for (int t = 0; t < TN; ++t) fa[ks & 1][t] = *reinterpret_cast<const lds_u32x4*>(a_row + off + t * 4096);
#pragma unroll
        for (int t = 0; t < TM; ++t) fb[ks & 1][t] = *reinterpret_cast<const lds_u32x4*>(b_row + off + t * 4096);
    };
    // the NM products of one k-slice; after(i) is called behind product i
    auto products = [&](int set, auto&& after) {
        static_for<NM>([&](auto it) {
            constexpr int i = decltype(it)::value, tn = i / TM, tm = i % TM;
            acc[tn][tm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa[set][tn]),
                                                                      __builtin_bit_cast(bf16x8, fb[set][tm]), acc[tn][tm], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            after(it);
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    // pieces FIRST .. FIRST + PPS - 1 of step j, behind products 1, 1 + NM / PPS, ... of a slice
    auto move_under = [&](auto it, int j, const StepSrc& next, auto first_tag) {
        constexpr int i = decltype(it)::value, FIRST = decltype(first_tag)::value;
        static_for<PPS>([&](auto q) {
            constexpr int slot = 1 + decltype(q)::value * (NM / PPS) < NM - 1 ? 1 + decltype(q)::value * (NM / PPS) : NM - 1;
            if (slot == i) move_piece(j, next, std::integral_constant<int, FIRST + decltype(q)::value>{});
        });
    };
    using ic0 = std::integral_constant<int, 0>;

    // ---- the K loop: two LDS stages and one set of staging registers, one barrier per step --------------------------
    // Step k is multiplied out of stage k & 1 in four k-slices of 16.  The barrier of step k sits between the products of
    // slices 2 and 3: in front of it every wave has all fragments of step k in registers and has written its pieces of
    // step k + 1; behind it stage k & 1 is free for step k + 2 and stage (k + 1) & 1 may be read.  Every piece goes round
    // once per step: under slice 3 of step k the pieces 0 .. PPS - 1 of step k + 2 are written and reloaded for step
    // k + 3, under slices 0 .. 2 of the next step the others -- each load has a whole step to land and the loads flow
    // evenly.
    {
        const StepSrc s0 = step_src(0), s1 = step_src(1), s2 = step_src(2);
        static_for<LPW>([&](auto p) { load_piece(s0, p); });
        static_for<LPW>([&](auto p) { move_piece(0, s1, p); });
        static_for<PPS>([&](auto p) { move_piece(1, s2, p); });  // as under slice 3 of a step in front of the first
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    read_frags(ic0{}, 0);
    for (int k = 0; k < nk; ++k) {
        const int cur = k & 1;
        const StepSrc src2 = step_src(k + 2), src3 = step_src(k + 3);
        static_for<3>([&](auto ks_tag) {
            constexpr int ks = decltype(ks_tag)::value;
            products(ks & 1, [&](auto it) {
                if (decltype(it)::value == 0) read_frags(std::integral_constant<int, ks + 1>{}, cur);
                move_under(it, k + 1, src2, std::integral_constant<int, PPS * (ks + 1)>{});
            });
        });
        // every LDS write of step k + 1 and every read of step k has completed in front of the barrier
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("" ::: "memory");
        products(1, [&](auto it) {
            if (decltype(it)::value == 0) read_frags(ic0{}, cur ^ 1);  // behind the last step: zeros, not used
            move_under(it, k + 2, src3, ic0{});
        });
    }
    if (a.out_f32) store_tiles<SWIGLU, TM, TN, WM, WN>(a, acc, tile_m, tile_n, wm, wn, l32, hi);
    else store_tiles_lds<SWIGLU, TM, TN, WM, WN>(a, acc, tile_m, tile_n, wave, lane, lds_base);
}

int g_tiled_min_rows = 33;  // raven_set_tuning("gemm_tiled_min_rows"): fewest rows that take this kernel
int g_tiled_variant = 0;    // raven_set_tuning("gemm_tiled_variant"): 0 = by shape, 1 = 256 x 256 tiles, 2 = 128 x 128 tiles

template <bool SWIGLU, int TM, int TN, int WM = 2, int WN = 4>
static int launch_tiled(TiledArgs a, hipStream_t s) {
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32, BN_OUT = SWIGLU ? BN / 2 : BN;
    constexpr size_t lds = (size_t)2 * (BM + BN) * 128;
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_tiled_kernel<SWIGLU, TM, TN, WM, WN>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
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
    gemm_tiled_kernel<SWIGLU, TM, TN, WM, WN><<<dim3(grid), dim3(64 * WM * WN), lds, s>>>(a);
    return raven_host::check_launch("gemm (tiled MFMA)");
}

// Host entry for the other translation units: true when the shape is one the tiled kernel takes and is the better choice
// for.  Few token rows against a matrix with few rows give too few tiles to fill the chip (there is no K split here):
// up to 160 rows those go to the skinny kernels, 32 rows per pass over the weights.
bool tiled_gemm_fits(int M, int N, int K0, int K1, int dtype) {
    const int64_t small_tiles = (int64_t)((M + 127) / 128) * ((N + 127) / 128);
    if (g_tiled_variant == 0 && M <= 160 && small_tiles < 128) return false;
    return dtype == RAVEN_BF16 && M >= 1 && N % 8 == 0 && K0 % 8 == 0 && K0 > 0 && (K1 == 0 || K1 == K0) && (int64_t)M * (K0 > K1 ? K0 : K1) < (1ll << 31) &&
           (int64_t)N * 2 * (K0 + K1) < (1ll << 31);
}

int tiled_gemm(const void* x0, const void* x1, const void* w, const void* residual, void* y, int M, int N, int K0, int K1, int swiglu,
               int out_f32, hipStream_t s) {
    RAVEN_REQUIRE(tiled_gemm_fits(M, N, K0, K1, RAVEN_BF16), "gemm (tiled): unsupported shape M=%d N=%d K0=%d K1=%d", M, N, K0, K1);
    RAVEN_REQUIRE(!(swiglu && (residual || out_f32)), "gemm (tiled): the SwiGLU epilogue has no residual and stores bf16");
    RAVEN_REQUIRE(((uintptr_t)x0 & 15) == 0 && ((uintptr_t)x1 & 15) == 0 && ((uintptr_t)w & 15) == 0 && ((uintptr_t)y & 15) == 0 &&
                      ((uintptr_t)residual & 15) == 0, "gemm (tiled): operands must be 16-byte aligned");
    TiledArgs a{};
    a.w = static_cast<const bf16*>(w);
    a.x0 = static_cast<const bf16*>(x0);
    a.x1 = static_cast<const bf16*>(x1);
    a.residual = static_cast<const bf16*>(residual);
    a.y = y;
    a.M = M; a.N = N; a.K0 = K0; a.K1 = x1 ? K1 : 0; a.out_f32 = out_f32;
    // 256 x 256 tiles when they fill the chip at least once; 128 x 128 tiles otherwise
    const int bn_out = swiglu ? 128 : 256;
    const int64_t tiles_n = (N + bn_out - 1) / bn_out, tiles_m = (M + 255) / 256;
    const int64_t big_tiles = tiles_m * tiles_n;
    const bool big = g_tiled_variant == 1 || (g_tiled_variant == 0 && big_tiles >= 256);
    auto launch = [&](const TiledArgs& t, bool as_big) {
        if (swiglu) return as_big ? launch_tiled<true, 4, 2>(t, s) : launch_tiled<true, 2, 1>(t, s);
        return as_big ? launch_tiled<false, 4, 2>(t, s) : launch_tiled<false, 2, 1>(t, s);
    };
    return launch(a, big);
}

}  // namespace raven

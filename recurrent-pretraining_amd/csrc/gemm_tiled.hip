// Tiled MFMA GEMM for many token rows (prefill chunks, wide decode batches): Y[M,N] = concat(X0, X1)[M,K] W[N,K]^T in
// bf16 with fp32 accumulation -- the nn.Linear products of the reference at M = B*S rows
// (recpre/raven_modeling_minimal.py:463 Wqkv, 493 attn.proj, 507-509 mlp.fc / SwiGLU / mlp.proj, 776 adapter over
// cat([x, input_embeds]), 711 lm_head), with the epilogues of the skinny kernels: plain, + residual (RMM:534-535),
// float store (RMM:711), SwiGLU (RMM:507-508).  The concat of RMM:776 is two K segments of the X operand.
//
// Two kernels: gemm_ring_kernel (further down) multiplies the 256 x 256 tiles; gemm_tiled_kernel, described here, the
// 128 x 128 tiles (few tiles, and the last tile columns of a launch whose last round would be nearly empty), and the
// 256 x 256 tiles too when asked to (tuning key gemm_tiled_variant = 3).  Both issue the same products in the same order
// per accumulator: a result does not depend on which of them computed it.
//
// Shape of gemm_tiled_kernel (gfx950):
//   * a workgroup of 8 waves (2 along the token rows x 4 along the weight rows, two waves per SIMD) owns a BN x BM tile
//     of Y^T (256 weight rows x 256 token rows in the main variant); a wave owns 2 TN x 2 TM MFMA tiles of 16 x 16
//     (v_mfma_f32_16x16x32_bf16, W rows as the A operand, X rows as B, so that a lane ends up with 4 neighbouring output
//     columns of one token row).  The 16 x 16 x 32 instruction has the same rate per product as 32 x 32 x 16 and needs
//     the same LDS traffic here; measured, it runs the main variant 1 % to 5 % faster at the model's shapes;
//   * K advances in steps of 64 through two LDS stages of BN + BM rows of 128 bytes.  The 16-byte pieces of a row are
//     kept at position piece ^ ((row >> 1) & 7), so that the 16 lanes of a quarter wave, which read the same piece of 16
//     neighbouring rows, hit all 64 banks;
//   * operands travel global -> registers -> LDS: 8 lanes fetch one whole 128-byte row step (the L1 address path
//     serves full lines at twice the rate of half lines), a wave instruction 8 rows.  Every lane keeps one step of its
//     pieces in registers; a piece is written to LDS one step after it was requested and its registers are reloaded at
//     once, two pieces under the products of each quarter step, so that loads flow evenly and each has a whole step to land;
//   * a step is two k-slices of 32 and a slice two quarter steps, each all weight tiles of the wave against half of its
//     token tiles.  A token fragment is replaced in place, as soon as its products are issued, by the one the next
//     quarter needs; the weight fragments of the next slice go into a second register set.  One workgroup barrier per
//     step, in front of the last quarter;
//   * a loop over K steps is one basic block of plain loads, stores and MFMAs with the scheduler pinned between them:
//     the compiler then counts the outstanding loads exactly and waits for one piece at a time.  Besides the MFMAs it
//     holds little vector arithmetic (one 64-bit add per piece, six address updates per step): steps whose 64 columns
//     lie in one segment and below K take their pieces from a scalar base, and the LDS addresses that alternate
//     between the stages live in registers.  Steps near a segment boundary or the end of K run in loops of their own
//     with a per-lane source; every lambda of the loops is forced inline, or the compiler keeps one shared copy with
//     the accumulators in memory;
//   * workgroups are numbered so that the 32 that run together on one XCD (ids congruent modulo 8) cover 8 x 4
//     neighbouring tiles and find each other's panels in that XCD's L2;
//   * SwiGLU: 32 weight rows of the tile are 16 gate rows and the 16 matching up rows, so gate and up of one output
//     element sit in the same lane, in neighbouring accumulator tiles.
// M, N and the last tile: rows past the end are clamped on the load side and not stored.  K0 and K1 are multiples of 8
// (pieces past K come from a zero page); two segments share one row pitch (K1 == K0).

#include <type_traits>
#include <utility>

#include <mutex>
#include <unordered_map>

#include "raven_common.h"

namespace raven {

struct TiledArgs {
    const bf16* w;         // [N or 2N, K0 + K1]
    const bf16* x0;        // [M, K0]
    const bf16* x1;        // [M, K1] or null
    const bf16* residual;  // [M, N] or null
    void* y;               // [M, N] bf16, or float when out_f32
    int M, N, K0, K1;      // N = output columns of this launch (I for SwiGLU)
    int ldy;               // row pitch of y and residual in elements (>= N: a launch may cover a range of columns)
    int ldw, ldx;          // row pitch of w and of x0 / x1 in elements: K0 + K1 and K0, or more where rows are padded to whole 128-byte lines
    int up_off;            // SwiGLU: weight rows between a gate row and its up row (the whole matrix's I)
    int out_f32;
    int tiles_m, tiles_n;
    int rope_on;           // the epilogue below instead of y
    // The product is a chunk's fused q | k | v rows (3 * nh * hd columns): instead of y, the epilogue adds the q / k bias,
    // rotates q and k (RoPE on adjacent pairs) and writes q to q_out and k, v to their cache rows -- what
    // qkv_rope_append_tiled_kernel (attention.hip) does to a stored product, with the same functions in the same order.
    struct RopeAppend {
        const float* freqs;
        const bf16* qk_bias;   // [2, nh * hd] or null
        bf16* q_out;           // [M, nh * hd]
        bf16 *k, *v;           // cache tensors, [.., batch, nh, t_max, hd] from slot_off on
        int64_t slot_off;
        const int* pos_dev;    // position of a sequence's first row, on the device (or null: pos0)
        int nh, hd, t_max, S, pos0;
        int col0;              // column of the whole product that this launch's column 0 is
    } rope;
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

// Epilogue of both kernels.  Accumulator tile [ta][tb] (16 weight rows x 16 token rows) leaves a lane with token row
// 16 tb + l16 and output columns 16 ta + 4 q4 + (0 .. 3); under SwiGLU tile 2 t holds gate columns and 2 t + 1 the
// matching up columns.
template <bool SWIGLU, int TM, int TN, int WM = 2, int WN = 4>
__device__ __forceinline__ void store_tiles(const TiledArgs& a, const f32x4 (&acc)[2 * TN][2 * TM], int tile_m, int tile_n, int wm, int wn,
                                            int l16, int q4) {
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32, BN_OUT = SWIGLU ? BN / 2 : BN;
    constexpr int NA = 2 * TN, NB = 2 * TM, NT = SWIGLU ? TN : NA;
#pragma unroll
    for (int tb = 0; tb < NB; ++tb) {
        const int m = tile_m * BM + (wm * NB + tb) * 16 + l16;
        if (m >= a.M) continue;
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const int n = tile_n * BN_OUT + (wn * NT + t) * 16 + 4 * q4;
            if (n >= a.N) continue;
            if (SWIGLU) {
                bf16 o[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float g = round_to<bf16>(acc[2 * t][tb][i]), u = round_to<bf16>(acc[2 * t + 1][tb][i]);
                    o[i] = from_f32<bf16>(round_to<bf16>(silu_f32(g)) * u);
                }
                *reinterpret_cast<u32x2*>(static_cast<bf16*>(a.y) + (int64_t)m * a.ldy + n) = *reinterpret_cast<const u32x2*>(o);
            } else {
                float r[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) r[i] = round_to<bf16>(acc[t][tb][i]);
                if (a.residual) {
                    bf16 res[4];
                    *reinterpret_cast<u32x2*>(res) = *reinterpret_cast<const u32x2*>(a.residual + (int64_t)m * a.ldy + n);
#pragma unroll
                    for (int i = 0; i < 4; ++i) r[i] = round_to<bf16>(r[i] + to_f32(res[i]));
                }
                if (a.out_f32) {
                    *reinterpret_cast<f32x4*>(static_cast<float*>(a.y) + (int64_t)m * a.ldy + n) = f32x4{r[0], r[1], r[2], r[3]};
                } else {
                    bf16 o[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) o[i] = from_f32<bf16>(r[i]);
                    *reinterpret_cast<u32x2*>(static_cast<bf16*>(a.y) + (int64_t)m * a.ldy + n) = *reinterpret_cast<const u32x2*>(o);
                }
            }
        }
    }
}

// The accumulators of a workgroup laid down in LDS as the output tile (rows of BN_OUT columns, 16-byte unit u of row r at
// position u ^ (r mod units per row)), between two workgroup barriers: the first because the K loop's stages are reused.
template <bool SWIGLU, int TM, int TN, int WM, int WN>
__device__ __forceinline__ void lay_tiles_lds(const f32x4 (&acc)[2 * TN][2 * TM], int wave, int lane, unsigned lds_base) {
    constexpr int BN = WN * TN * 32, BN_OUT = SWIGLU ? BN / 2 : BN;
    constexpr int NA = 2 * TN, NB = 2 * TM, NT = SWIGLU ? TN : NA;
    constexpr int RB = BN_OUT * 2, U = RB / 16;
    const int wn = wave % WN, wm = wave / WN, l16 = lane & 15, q4 = lane >> 4;
    // every wave has its last fragments; the stages are free
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int tb = 0; tb < NB; ++tb) {
        const int row = (wm * NB + tb) * 16 + l16;
        const unsigned row_addr = lds_base + row * RB + (q4 & 1) * 8;
        const int sw = row & (U - 1);
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            bf16 o[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (SWIGLU) {
                    const float g = round_to<bf16>(acc[2 * t][tb][i]), u = round_to<bf16>(acc[2 * t + 1][tb][i]);
                    o[i] = from_f32<bf16>(round_to<bf16>(silu_f32(g)) * u);
                } else {
                    o[i] = from_f32<bf16>(acc[t][tb][i]);
                }
            }
            const int unit = (wn * NT + t) * 2 + (q4 >> 1);
            *reinterpret_cast<__attribute__((address_space(3))) u32x2*>(row_addr + ((unit ^ sw) * 16)) = *reinterpret_cast<const u32x2*>(o);
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// Epilogue through LDS for the bf16 outputs: the accumulators (a lane: 4 columns of one token row per store, a wave
// instruction 16 token rows) are laid down as the output tile, rows of BN_OUT columns, and read back so that a wave
// instruction stores two whole tile rows, 16 bytes per lane: full 128-byte lines instead of pieces of 8 bytes.  The
// residual is fetched the same way, before the tile is laid down, so that its latency hides behind the transposition.
// 16-byte unit u of tile row r sits at position u ^ (r mod units per row): the 16 rows a store instruction spreads over
// then fall on different banks.
template <bool SWIGLU, int TM, int TN, int WM = 2, int WN = 4>
__device__ __forceinline__ void store_tiles_lds(const TiledArgs& a, const f32x4 (&acc)[2 * TN][2 * TM], int tile_m, int tile_n, int wave,
                                                int lane, unsigned lds_base) {
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32, BN_OUT = SWIGLU ? BN / 2 : BN;
    constexpr int NA = 2 * TN, NB = 2 * TM, NT = SWIGLU ? TN : NA;
    constexpr int RB = BN_OUT * 2, U = RB / 16;      // bytes and 16-byte units per tile row
    constexpr int ITERS = BM * U / (64 * WM * WN);    // 16-byte units per lane
    const int wn = wave % WN, wm = wave / WN, l16 = lane & 15, q4 = lane >> 4;
    bf16* const y = static_cast<bf16*>(a.y);
    int64_t goff[ITERS];                             // element offset of this lane's unit in y / residual, -1: outside
    u32x4 res[ITERS];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int idx = (wave * ITERS + it) * 64 + lane;
        const int m = tile_m * BM + idx / U, n = tile_n * BN_OUT + (idx % U) * 8;
        goff[it] = (m < a.M && n < a.N) ? (int64_t)m * a.ldy + n : -1;
        res[it] = u32x4{0, 0, 0, 0};
        if (!SWIGLU && a.residual && goff[it] >= 0) res[it] = *reinterpret_cast<const u32x4*>(a.residual + goff[it]);
    }
    lay_tiles_lds<SWIGLU, TM, TN, WM, WN>(acc, wave, lane, lds_base);
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

// Epilogue of a chunk's q | k | v product (TiledArgs::rope): the tile goes through LDS as above; each 16-byte unit (8
// columns of one head, of one token row) then gets the q / k bias and the rotation and goes to q_out or to its cache row.
// A lane's units all lie in the same 8 columns, so section, head and bias are fixed per lane; the (cos, sin) pairs of a
// unit's position are requested eight units ahead (the first eight before the tile is laid down).
template <int TM, int TN, int WM, int WN>
__device__ __forceinline__ void store_tiles_rope(const TiledArgs& a, const f32x4 (&acc)[2 * TN][2 * TM], int tile_m, int tile_n, int wave,
                                                 int lane, unsigned lds_base) {
    constexpr int BM = WM * TM * 32, BN_OUT = WN * TN * 32;
    constexpr int RB = BN_OUT * 2, U = RB / 16, RS = 64 / U;  // rows a wave instruction covers
    constexpr int ITERS = BM * U / (64 * WM * WN);
    constexpr int PD = ITERS < 8 ? ITERS : 8;
    // read from the kernel's argument block here, through a pointer the compiler cannot trace: as ordinary kernel
    // arguments the fields are fetched at the top and held in scalar registers through the K loop
    const char __attribute__((address_space(4)))* ka = (const char __attribute__((address_space(4)))*)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(ka));
    TiledArgs::RopeAppend r;
#define RAVEN_ROPE_FIELD(F_) r.F_ = *reinterpret_cast<const decltype(r.F_) __attribute__((address_space(4)))*>(ka + offsetof(TiledArgs, rope) + offsetof(TiledArgs::RopeAppend, F_))
    RAVEN_ROPE_FIELD(freqs); RAVEN_ROPE_FIELD(qk_bias); RAVEN_ROPE_FIELD(q_out); RAVEN_ROPE_FIELD(k); RAVEN_ROPE_FIELD(v);
    RAVEN_ROPE_FIELD(slot_off); RAVEN_ROPE_FIELD(pos_dev); RAVEN_ROPE_FIELD(nh); RAVEN_ROPE_FIELD(hd); RAVEN_ROPE_FIELD(t_max);
    RAVEN_ROPE_FIELD(S); RAVEN_ROPE_FIELD(pos0); RAVEN_ROPE_FIELD(col0);
#undef RAVEN_ROPE_FIELD
    const int unit = lane % U, row0 = wave * ITERS * RS + lane / U;
    const int n_local = tile_n * BN_OUT + unit * 8;
    const bool col_ok = n_local < a.N;
    const int h = r.nh * r.hd;
    const int n = col_ok ? r.col0 + n_local : 0;
    const int sec = n >= 2 * h ? 2 : (n >= h ? 1 : 0);   // q, k or v columns
    const int col = n - sec * h, head = col / r.hd, d = col - head * r.hd;
    const int first = r.pos_dev ? *r.pos_dev : r.pos0;
    Chunk<bf16> bch = zero_chunk<bf16>();
    if (sec < 2 && r.qk_bias) bch = load_chunk(r.qk_bias + sec * h + col);
    // sequence and position inside it of this lane's row: one division for the first row, then RS rows further per unit
    // (two walkers: the requests run PD units ahead of the units that are stored)
    struct RowWalk {
        int b, sq;
    };
    const int m_first = tile_m * BM + row0;
    RowWalk ahead{m_first / r.S, 0}, here;
    ahead.sq = m_first - ahead.b * r.S;
    here = ahead;
    auto advance = [&](RowWalk& w) {
        w.sq += RS;
        while (w.sq >= r.S) {
            w.sq -= r.S;
            ++w.b;
        }
    };
    // the table rows of positions pos0 + sq: sq < S whatever the row, so a row past M still names a valid table row
    const float* const f_base = r.freqs + ((int64_t)first * (r.hd / 2) + d / 2) * 2;
    const int f_step = (r.hd / 2) * 2;
    f32x4 fq[PD][2];
    auto request = [&](f32x4 (&f)[2]) {
        const float* fp = f_base + (int64_t)ahead.sq * f_step;
        f[0] = *reinterpret_cast<const f32x4*>(fp);
        f[1] = *reinterpret_cast<const f32x4*>(fp + 4);
        advance(ahead);
    };
#pragma unroll
    for (int it = 0; it < PD; ++it) request(fq[it]);
    lay_tiles_lds<false, TM, TN, WM, WN>(acc, wave, lane, lds_base);
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
        const int row = row0 + it * RS;
        const u32x4 v = *reinterpret_cast<const lds_u32x4*>(lds_base + row * RB + ((unit ^ (row & (U - 1))) * 16));
        const int m = m_first + it * RS, b = here.b, pos = first + here.sq;
        advance(here);
        Chunk<bf16> x;
        *reinterpret_cast<u32x4*>(x.v) = v;
        const f32x4 f0 = fq[it % PD][0], f1 = fq[it % PD][1];
        if (it + PD < ITERS) request(fq[it % PD]);
        if (sec < 2) {
            if (r.qk_bias) {
#pragma unroll
                for (int e = 0; e < 8; ++e) x.v[e] = from_f32<bf16>(to_f32(x.v[e]) + to_f32(bch.v[e]));
            }
            rope_pair<bf16>(x.v[0], x.v[1], f0[0], f0[1]);
            rope_pair<bf16>(x.v[2], x.v[3], f0[2], f0[3]);
            rope_pair<bf16>(x.v[4], x.v[5], f1[0], f1[1]);
            rope_pair<bf16>(x.v[6], x.v[7], f1[2], f1[3]);
        }
        if (!col_ok || tile_m * BM + row >= a.M) continue;
        if (sec == 0) store_chunk(r.q_out + (int64_t)m * h + col, x);
        else if (pos < r.t_max) store_chunk((sec == 1 ? r.k : r.v) + r.slot_off + (((int64_t)b * r.nh + head) * r.t_max + pos) * r.hd + d, x);
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
    constexpr int NA = 2 * TN, NB = 2 * TM;   // 16-row MFMA tiles of a wave along the weight rows / the token rows
    constexpr int HB = NB / 2;                 // token tiles of a quarter step
    static_assert(NA == HB, "one weight fragment is fetched behind each group of a quarter step");
    constexpr int NM = NA * HB;                // MFMAs per quarter step
    constexpr int PPS = LPW / 4;               // pieces handled under the products of one quarter step
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
    const unsigned ld2 = 2u * (loads_w ? a.ldw : a.ldx);
#pragma unroll
    for (int p = 0; p < LPW; ++p) {
        const int r = (wave * LPW + p) * 8 + (lane >> 3);
        int row;
        if (loads_w) {
            if (SWIGLU) row = min(tile_n * BN_OUT + (r >> 5) * 16 + (r & 15), a.N - 1) + ((r & 16) ? a.up_off : 0);
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

    // Plain loads and stores inside a step: the compiler then knows the order of all outstanding loads and waits, in
    // front of the LDS write of a piece, for exactly that piece's load (issued one step earlier).
    // Where this lane's 16 bytes of step kk come from: its segment's pointer (rebased so that the piece's offset is
    // goff[p] + 2 * 64 kk), or the zero page for columns past K -- which is every column of a step past the last one.
    // A step whose 64 columns lie in one segment and below K has one source for the whole wave (WHOLE): a scalar base
    // plus the lane's 32-bit offset, no vector arithmetic per piece.
    struct StepSrc {
        const char* base;
        bool past;  // this lane's column lies past K
    };
    auto step_src = [&](int kk) __attribute__((always_inline)) {
        const int col = (kk << 6) + col8;
        StepSrc s;
        s.past = col >= K;
        s.base = s.past ? zero : (col < k_split ? seg0 : seg1) + 2 * (kk << 6);
        return s;
    };
    auto whole_step = [&](int kk) __attribute__((always_inline)) {  // wave-uniform
        const int c0 = kk << 6;
        return c0 + 64 <= k_split || (c0 >= k_split && c0 + 64 <= K);
    };
    auto whole_src = [&](int kk) __attribute__((always_inline)) {   // wave-uniform
        const int c0 = kk << 6;
        StepSrc s;
        s.past = false;
        s.base = (c0 < k_split ? seg0 : seg1) + 2 * c0;
        return s;
    };
    u32x4 stg[LPW];
    auto load_piece = [&](const StepSrc& src, auto p_tag, auto whole_tag) __attribute__((always_inline)) {
        constexpr int p = decltype(p_tag)::value;
        if constexpr (decltype(whole_tag)::value) stg[p] = *reinterpret_cast<const u32x4*>(src.base + goff[p]);
        else stg[p] = *reinterpret_cast<const u32x4*>(src.base + (src.past ? 0u : goff[p]));
    };
    // LDS addresses that alternate between the two stages are kept in registers and advanced once per step
    unsigned wr_cur[2] = {wr_addr[0] + STAGE_BYTES, wr_addr[1] + STAGE_BYTES};  // the first step of the loop writes stage 1
    auto store_piece_at = [&](int kk, auto p_tag) __attribute__((always_inline)) {  // in front of the loops
        constexpr int p = decltype(p_tag)::value;
        *reinterpret_cast<lds_u32x4*>(wr_addr[p & 1] + (kk & 1) * STAGE_BYTES + p * 1024) = stg[p];
    };
    // Piece p moves on into the stage wr_cur points at; the registers take the piece of the step after (source: next).
    auto move_piece = [&](const StepSrc& next, auto p_tag, auto whole_tag) __attribute__((always_inline)) {
        constexpr int p = decltype(p_tag)::value;
        *reinterpret_cast<lds_u32x4*>(wr_cur[p & 1] + p * 1024) = stg[p];
        load_piece(next, p_tag, whole_tag);
    };

    // ---- LDS -> registers -------------------------------------------------------------------------------------------
    // v_mfma_f32_16x16x32_bf16: lane l supplies row l & 15 of its tile, columns 8 (l >> 4) ..+7 of a 32-column k-slice.
    const int l16 = lane & 15, q4 = lane >> 4;
    const int swz = (l16 >> 1) & 7;
    const unsigned a_row = lds_base + (wn * TN * 32 + l16) * 128;
    const unsigned b_row = lds_base + (BN + wm * TM * 32 + l16) * 128;
    const unsigned pos0 = (q4 ^ swz) * 16;     // position of k-slice s: pos0 ^ (64 s)

    f32x4 acc[NA][NB];
#pragma unroll
    for (int ta = 0; ta < NA; ++ta)
#pragma unroll
        for (int tb = 0; tb < NB; ++tb) acc[ta][tb] = f32x4{0.f, 0.f, 0.f, 0.f};

    // A step is two k-slices of 32, a slice two quarter steps: the NA weight tiles against one half of the token tiles
    // (HB of them), token tile by token tile.  The weight fragments of a slice live through both its quarters and
    // have a second register set, filled under the slice before; a token fragment is replaced by the one the next
    // quarter needs in the same place as soon as its NA products are issued -- 3/4 of a quarter ahead of its use.
    u32x4 fa[2][NA], fb[HB];
    unsigned ra[2] = {a_row + pos0, a_row + (pos0 ^ 64)}, rb[2] = {b_row + pos0, b_row + (pos0 ^ 64)};  // slice 0 / 1, stage 0
    auto read_a = [&](auto set_tag, auto t_tag) __attribute__((always_inline)) {  // weight tile t of slice `set` into fragment set `set`
        constexpr int set = decltype(set_tag)::value, t = decltype(t_tag)::value;
        fa[set][t] = *reinterpret_cast<const lds_u32x4*>(ra[set] + t * 2048);
    };
    auto read_b = [&](auto slice_tag, auto half_tag, auto j_tag) __attribute__((always_inline)) {
        constexpr int slice = decltype(slice_tag)::value, half = decltype(half_tag)::value, j = decltype(j_tag)::value;
        fb[j] = *reinterpret_cast<const lds_u32x4*>(rb[slice] + (half * HB + j) * 2048);
    };
    // Quarter q of a step: slice q >> 1, token half q & 1.  Behind the first NA products of a second half the weight
    // fragments of the next slice are requested (for q = 3: of the next step; ra[0] and rb[0] point there by then).
    auto quarter = [&](auto q_tag, auto&& extra) __attribute__((always_inline)) {
        constexpr int q = decltype(q_tag)::value, s = q >> 1, h = q & 1;
        constexpr int sn = ((q + 1) & 3) >> 1, hn = (q + 1) & 1;
        static_for<NM>([&](auto it) {
            constexpr int i = decltype(it)::value, j = i / NA, ta = i % NA;
            acc[ta][h * HB + j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, fa[s][ta]),
                                                                           __builtin_bit_cast(bf16x8, fb[j]), acc[ta][h * HB + j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (h == 1 && i < NA) read_a(std::integral_constant<int, s ^ 1>{}, std::integral_constant<int, (i < NA ? i : 0)>{});
            if (ta == NA - 1) read_b(std::integral_constant<int, sn>{}, std::integral_constant<int, hn>{}, std::integral_constant<int, j>{});
            extra(it);
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    // pieces FIRST .. FIRST + PPS - 1, spread over the products of a quarter
    auto move_under = [&](auto it, const StepSrc& next, auto first_tag, auto whole_tag) __attribute__((always_inline)) {
        constexpr int i = decltype(it)::value, FIRST = decltype(first_tag)::value;
        static_for<PPS>([&](auto qq) {
            constexpr int want = NA + 1 + decltype(qq)::value * (NM / PPS);
            constexpr int slot = want < NM - 1 ? want : NM - 1;
            if (slot == i) move_piece(next, std::integral_constant<int, FIRST + decltype(qq)::value>{}, whole_tag);
        });
    };
    using ic0 = std::integral_constant<int, 0>;

    // ---- the K loop: two LDS stages and one set of staging registers, one barrier per step --------------------------
    // Step k is multiplied out of stage k & 1 in four quarters.  The barrier of step k sits between quarters 2 and 3:
    // in front of it every wave has requested all it needs of stage k & 1 and has written its pieces of step k + 1;
    // behind it stage k & 1 is free for step k + 2 and stage (k + 1) & 1 may be read.  Every piece goes round once per
    // step: under quarter 3 of step k the pieces 0 .. PPS - 1 of step k + 2 are written and reloaded for step k + 3,
    // under quarters 0 .. 2 of the next step the others -- each load has a whole step to land and the loads flow evenly.
    {
        const StepSrc s0 = step_src(0), s1 = step_src(1), s2 = step_src(2);
        static_for<LPW>([&](auto p) { load_piece(s0, p, std::false_type{}); });
        static_for<LPW>([&](auto p) { store_piece_at(0, p); load_piece(s1, p, std::false_type{}); });
        static_for<PPS>([&](auto p) { store_piece_at(1, p); load_piece(s2, p, std::false_type{}); });  // as under quarter 3 of a step before
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    static_for<NA>([&](auto t) { read_a(ic0{}, t); });
    static_for<HB>([&](auto j) { read_b(ic0{}, ic0{}, j); });
    // One step; src2 / src3: where steps k + 2 / k + 3 come from.  flip = +-STAGE_BYTES: from this step's stage to the other.
    auto step = [&](const StepSrc& src2, const StepSrc& src3, int flip, auto whole_tag) __attribute__((always_inline)) {
        static_for<3>([&](auto q_tag) {
            constexpr int q = decltype(q_tag)::value;
            quarter(q_tag, [&](auto it) { move_under(it, src2, std::integral_constant<int, PPS * (q + 1)>{}, whole_tag); });
        });
        // every LDS write of step k + 1 and every read of stage k & 1 has completed in front of the barrier
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("" ::: "memory");
        // from here on: fragments of the next step out of the other stage, pieces of step k + 2 into this one
        ra[0] += flip; ra[1] += flip; rb[0] += flip; rb[1] += flip;
        wr_cur[0] -= flip; wr_cur[1] -= flip;
        // behind the last step the fragments requested here are zeros and not used
        quarter(std::integral_constant<int, 3>{}, [&](auto it) { move_under(it, src3, ic0{}, whole_tag); });
    };
    // Runs of steps that take their pieces from whole steps alternate with runs that do not (around the boundary
    // between two segments when it is not a multiple of 64, and at the end of K); each run is a loop of its own, so
    // that a loop body stays one basic block.
    auto whole_ok = [&](int k) __attribute__((always_inline)) { return whole_step(k + 2) && whole_step(k + 3); };
    auto run = [&](int k, int k_end, auto whole_tag) __attribute__((always_inline)) {
        for (; k < k_end; ++k) {
            const int flip = (k & 1) ? -STAGE_BYTES : STAGE_BYTES;
            if constexpr (decltype(whole_tag)::value) step(whole_src(k + 2), whole_src(k + 3), flip, whole_tag);
            else step(step_src(k + 2), step_src(k + 3), flip, whole_tag);
        }
    };
    int e1 = 0, e2, e3;
    while (e1 < nk && whole_ok(e1)) ++e1;
    e2 = e1;
    while (e2 < nk && !whole_ok(e2)) ++e2;
    e3 = e2;
    while (e3 < nk && whole_ok(e3)) ++e3;
    run(0, e1, std::true_type{});
    run(e1, e2, std::false_type{});
    run(e2, e3, std::true_type{});
    run(e3, nk, std::false_type{});
    if constexpr (!SWIGLU) {
        if (a.rope_on) {  // uniform over the launch
            store_tiles_rope<TM, TN, WM, WN>(a, acc, tile_m, tile_n, wave, lane, lds_base);
            return;
        }
    }
    if (a.out_f32) store_tiles<SWIGLU, TM, TN, WM, WN>(a, acc, tile_m, tile_n, wm, wn, l16, q4);
    else store_tiles_lds<SWIGLU, TM, TN, WM, WN>(a, acc, tile_m, tile_n, wave, lane, lds_base);
}

// ------------------------------------------------------------------------------------------------
// The 256 x 256 tile with FOUR waves (2 x 2, one per SIMD, 128 x 128 each: 64 accumulator tiles in the 256 accumulation
// registers) and operands that go global -> LDS directly.  Per K step of 64 a wave then issues 128 products, 32 fragment
// reads (a third fewer than eight waves need), 16 requests and no LDS write or staging register at all.
//   * LDS is a ring of five half stages of 32 KB (256 rows x 128 bytes, swizzled as above): the weight rows of step k
//     sit in half stage 2k mod 5, the token rows in 2k + 1 mod 5.  Two and a half steps fit, so the token rows of step
//     k + 2 and the weight rows of step k + 3 move into the two halves that step k vacates;
//   * the fragments of a whole step live in registers (2 k-slices x (8 + 8) fragments = 128 registers): slice 1 is read
//     under the products of slice 0, so that the step's halves are read out -- FIRST barrier -- well before its products
//     end; from there on the 16 requests of the next window are issued one behind every eighth product (the address path
//     takes a kilobyte per 16 cycles; four waves that request in bursts stall on it, and with one wave per SIMD a stalled
//     wave idles the matrix core), M0 set two products ahead of its request;
//   * under slice 1 the SECOND barrier, in front of it a wait that leaves the 14 youngest requests outstanding: both halves
//     of step k + 1 have landed, and its slice 0 is read under the last products.  A request has between 1.4 and 2.4
//     steps to land.
// Same products in the same order per accumulator as the eight-wave kernel: bit-identical results.
template <bool SWIGLU>
__global__ __launch_bounds__(256) void gemm_ring_kernel(TiledArgs a) {
    constexpr int TM = 4, TN = 4, WM = 2, WN = 2;
    constexpr int BM = 256, BN = 256, BN_OUT = SWIGLU ? BN / 2 : BN;
    constexpr int NA = 8, NB = 8, NP = NA * NB;   // 16-row tiles of a wave along the weight / token rows; products of a k-slice
    constexpr int HALF = 32768, RING = 5 * HALF;
    constexpr int PPW = 8;                        // pieces (8 rows x 128 bytes) a wave requests per operand and step
    extern __shared__ __align__(1024) unsigned char smem[];

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
    const unsigned lds_base = (unsigned)(uintptr_t)(lds_byte*)smem;

    // ---- global side: wave w requests rows 64 w ..+63 of both operands' tiles, piece p = rows 8 p ..+7 of those; the lane
    // that fills position s of LDS row r fetches piece s ^ ((r >> 1) & 7) of the row's 128-byte step
    const int colp[2] = {((lane & 7) ^ (lane >> 4)) * 8, ((lane & 7) ^ ((lane >> 4) | 4)) * 8};
    unsigned goff_w[PPW], goff_x[PPW];
#pragma unroll
    for (int p = 0; p < PPW; ++p) {
        const int r = (wave * PPW + p) * 8 + (lane >> 3);
        int row_w;
        if (SWIGLU) row_w = min(tile_n * BN_OUT + (r >> 5) * 16 + (r & 15), a.N - 1) + ((r & 16) ? a.up_off : 0);
        else row_w = min(tile_n * BN + r, a.N - 1);
        goff_w[p] = (unsigned)row_w * (2u * a.ldw) + 2u * colp[p & 1];
        goff_x[p] = (unsigned)min(tile_m * BM + r, a.M - 1) * (2u * a.ldx) + 2u * colp[p & 1];
    }
    const char* const zero = reinterpret_cast<const char*>(g_zero_piece);
    const char* const w0 = reinterpret_cast<const char*>(a.w);
    const char* const x0 = reinterpret_cast<const char*>(a.x0);
    const char* const x1 = reinterpret_cast<const char*>(a.x1) - 2 * (int64_t)a.K0;  // column c >= K0 of the token rows
    auto whole_step = [&](int kk) __attribute__((always_inline)) {  // the step's 64 columns lie in one segment and below K
        const int c0 = kk << 6;
        return c0 + 64 <= a.K0 || (c0 >= a.K0 && c0 + 64 <= K);
    };
    // M0 = where the wave's next kilobyte goes: half stage offset `o`, the wave's eight pieces, piece p
    auto aim = [&](int o, auto p_tag) __attribute__((always_inline)) {
        constexpr int p = decltype(p_tag)::value;
        const unsigned sbase = lds_base + o + wave * (PPW * 1024);
        asm volatile("s_add_u32 m0, %0, %1" ::"s"(sbase), "n"(p * 1024) : "scc", "memory");
    };
    auto request = [&](auto is_w_tag, int kk, auto p_tag, auto whole_tag) __attribute__((always_inline)) {
        constexpr bool is_w = decltype(is_w_tag)::value;
        constexpr int p = decltype(p_tag)::value;
        const int c0 = kk << 6;
        if constexpr (decltype(whole_tag)::value) {
            const char* base = (is_w ? w0 : (c0 < a.K0 ? x0 : x1)) + 2 * c0;
            asm volatile("global_load_lds_dwordx4 %0, %1" ::"v"(is_w ? goff_w[p] : goff_x[p]), "s"(base) : "memory");
        } else {
            const int col = c0 + colp[p & 1];
            const char* gp = col >= K ? zero : (is_w ? w0 : (col < a.K0 ? x0 : x1)) + 2 * c0 + (is_w ? goff_w[p] : goff_x[p]);
            asm volatile("global_load_lds_dwordx4 %0, off" ::"v"(gp) : "memory");
        }
    };
    auto next_half = [](int o) __attribute__((always_inline)) { return o + 2 * HALF >= RING ? o + 2 * HALF - RING : o + 2 * HALF; };

    // ---- LDS -> registers
    const int l16 = lane & 15, q4 = lane >> 4;
    const unsigned pos0 = (q4 ^ ((l16 >> 1) & 7)) * 16;
    const unsigned a_lane[2] = {lds_base + (wn * 128 + l16) * 128 + pos0, lds_base + (wn * 128 + l16) * 128 + (pos0 ^ 64)};
    const unsigned b_lane[2] = {lds_base + (wm * 128 + l16) * 128 + pos0, lds_base + (wm * 128 + l16) * 128 + (pos0 ^ 64)};
    unsigned ra[2], rb[2];
    u32x4 ga[2][NA], gb[2][NB];
    auto rd = [&](auto sl_tag, auto n_tag) __attribute__((always_inline)) {  // fragment n of a slice: the weight tiles, then the token tiles
        constexpr int sl = decltype(sl_tag)::value, n = decltype(n_tag)::value;
        if constexpr (n < NA) ga[sl][n] = *reinterpret_cast<const lds_u32x4*>(ra[sl] + n * 2048);
        else gb[sl][n - NA] = *reinterpret_cast<const lds_u32x4*>(rb[sl] + (n - NA) * 2048);
    };
    f32x4 acc[NA][NB];
#pragma unroll
    for (int ta = 0; ta < NA; ++ta)
#pragma unroll
        for (int tb = 0; tb < NB; ++tb) {
            acc[ta][tb] = f32x4{0.f, 0.f, 0.f, 0.f};
            asm volatile("" : "+a"(acc[ta][tb]));  // 64 separate values, each born in its accumulation registers
        }
    using ic0 = std::integral_constant<int, 0>;
    using ic1 = std::integral_constant<int, 1>;

    // ---- in front of the loop: both halves of steps 0 and 1 and the first piece of the weight rows of step 2
    {
        int o = 0;  // half stages in ring order: W(0), X(0), W(1), X(1), W(2)
        static_for<PPW>([&](auto p) { aim(0, p); request(std::true_type{}, 0, p, std::false_type{}); });
        static_for<PPW>([&](auto p) { aim(HALF, p); request(std::false_type{}, 0, p, std::false_type{}); });
        static_for<PPW>([&](auto p) { aim(2 * HALF, p); request(std::true_type{}, 1, p, std::false_type{}); });
        static_for<PPW>([&](auto p) { aim(3 * HALF, p); request(std::false_type{}, 1, p, std::false_type{}); });
        aim(4 * HALF, ic0{});
        request(std::true_type{}, 2, ic0{}, std::false_type{});
        aim(4 * HALF, ic1{});  // for the request behind product 0 of step 0
        (void)o;
    }
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * PPW + 1) : "memory");  // step 0 has landed
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    ra[0] = a_lane[0]; ra[1] = a_lane[1]; rb[0] = b_lane[0] + HALF; rb[1] = b_lane[1] + HALF;
    static_for<NA + 1>([&](auto n) { rd(ic0{}, n); });  // the weight fragments and the first token fragment of slice 0; the others inside the step

    // ring offsets as step k sees them: the halves of step k + 1 (read behind the second barrier), the weight rows of step
    // k + 2 (the rest of the window opened in step k - 1), the token rows of step k + 2 and the weight rows of step k + 3
    int o_w1 = 2 * HALF, o_x1 = 3 * HALF, o_w2 = 4 * HALF, o_x2 = 0, o_w3 = HALF;
    auto step = [&](int k, auto whole_tag) __attribute__((always_inline)) {
        static_for<2 * NP>([&](auto it) {
            constexpr int i = decltype(it)::value, sl = i / NP, r = i % NP, j = r / NA, ta = r % NA;
            asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[ta][j]) : "v"(ga[sl][ta]), "v"(gb[sl][j]));
            __builtin_amdgcn_sched_barrier(0);
            // requests: behind every eighth product, M0 two products earlier.  Products 0 .. 48: pieces 1 .. 7 of the weight
            // rows of step k + 2; 56 .. 112: the token rows of step k + 2; 120: piece 0 of the weight rows of step k + 3
            if constexpr (i % 8 == 6 && i < 48) aim(o_w2, std::integral_constant<int, (i < 48 ? i / 8 + 2 : 0) % PPW>{});
            if constexpr (i % 8 == 0 && i > 0 && i <= 48) request(std::true_type{}, k + 2, std::integral_constant<int, (i <= 48 ? i / 8 + 1 : 0) % PPW>{}, whole_tag);
            if constexpr (i == 0) request(std::true_type{}, k + 2, ic1{}, whole_tag);  // its M0 was set behind product 126 of the step before
            if constexpr (i % 8 == 6 && i >= 54 && i < 118) aim(o_x2, std::integral_constant<int, (i >= 54 && i < 118 ? (i - 54) / 8 : 0)>{});
            if constexpr (i % 8 == 0 && i >= 56 && i <= 112) request(std::false_type{}, k + 2, std::integral_constant<int, (i >= 56 && i <= 112 ? (i - 56) / 8 : 0)>{}, whole_tag);
            if constexpr (i == 118) aim(o_w3, ic0{});
            if constexpr (i == 120) request(std::true_type{}, k + 3, ic0{}, whole_tag);
            if constexpr (i == 126) aim(o_w3, ic1{});  // for the request behind product 0 of the next step
            // fragments of slice 1: under products 1 .. 49, not where a request or its M0 sits
            constexpr int R1[16] = {2, 4, 7, 10, 13, 15, 18, 20, 23, 26, 29, 31, 34, 36, 39, 42};
            static_for<16>([&](auto n_tag) {
                constexpr int n = decltype(n_tag)::value;
                if constexpr (i == R1[n]) rd(ic1{}, n_tag);
            });
            // token fragments 1 .. 7 of slice 0, seven products ahead of their use (their half stays untouched until the
            // second barrier: the weight rows of step k + 3 move into it from product 120 on)
            if constexpr (i % 8 == 1 && i < 56) rd(ic0{}, std::integral_constant<int, NA + (i < 56 ? i / 8 + 1 : 1)>{});
            if constexpr (i == 52) {  // FIRST barrier: the weight half of this step is read out (the token fragment requested behind product 49 may still be on its way)
                asm volatile("s_waitcnt lgkmcnt(1)" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_sched_barrier(0);
                asm volatile("" ::: "memory");
            }
            if constexpr (i == 103) {  // SECOND barrier: step k + 1 has landed (younger: the weight rows of step k + 2 and six token pieces)
                asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PPW + 6) : "memory");
                __builtin_amdgcn_sched_barrier(0);
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_sched_barrier(0);
                asm volatile("" ::: "memory");
                ra[0] = a_lane[0] + o_w1; ra[1] = a_lane[1] + o_w1; rb[0] = b_lane[0] + o_x1; rb[1] = b_lane[1] + o_x1;
            }
            // fragments of slice 0 of step k + 1: under products 105 .. 124
            constexpr int R0[9] = {105, 106, 107, 108, 109, 111, 113, 114, 115};  // token tile 0, then the weight tiles
            if constexpr (i == R0[0]) rd(ic0{}, std::integral_constant<int, NA>{});
            static_for<8>([&](auto n_tag) {
                constexpr int n = decltype(n_tag)::value;
                if constexpr (i == R0[n + 1]) rd(ic0{}, n_tag);
            });
            __builtin_amdgcn_sched_barrier(0);
        });
        o_w1 = next_half(o_w1); o_x1 = next_half(o_x1); o_w2 = o_w3; o_x2 = next_half(o_x2); o_w3 = next_half(o_w3);
    };
    auto whole_ok = [&](int k) __attribute__((always_inline)) { return whole_step(k + 2) && whole_step(k + 3); };
    auto run = [&](int k, int k_end, auto whole_tag) __attribute__((always_inline)) {
        for (; k < k_end; ++k) step(k, whole_tag);
    };
    int e1 = 0, e2, e3;
    while (e1 < nk && whole_ok(e1)) ++e1;
    e2 = e1;
    while (e2 < nk && !whole_ok(e2)) ++e2;
    e3 = e2;
    while (e3 < nk && whole_ok(e3)) ++e3;
    run(0, e1, std::true_type{});
    run(e1, e2, std::false_type{});
    run(e2, e3, std::true_type{});
    run(e3, nk, std::false_type{});
    // requests past the last step still write into the ring, and the last products must land before their tiles are read
    asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
    if constexpr (!SWIGLU) {
        if (a.rope_on) {  // uniform over the launch
            store_tiles_rope<TM, TN, WM, WN>(a, acc, tile_m, tile_n, wave, lane, lds_base);
            return;
        }
    }
    if (a.out_f32) store_tiles<SWIGLU, TM, TN, WM, WN>(a, acc, tile_m, tile_n, wm, wn, l16, q4);
    else store_tiles_lds<SWIGLU, TM, TN, WM, WN>(a, acc, tile_m, tile_n, wave, lane, lds_base);
}

template <bool SWIGLU>
static int launch_ring(TiledArgs a, hipStream_t s) {
    constexpr int BM = 256, BN_OUT = SWIGLU ? 128 : 256;
    constexpr size_t lds = 5 * 32768;
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)gemm_ring_kernel<SWIGLU>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) {
            raven_host::set_error("gemm (ring): hipFuncSetAttribute failed: %s", hipGetErrorString(e));
            return (int)e;
        }
        attr_set = true;
    }
    a.tiles_m = (a.M + BM - 1) / BM;
    a.tiles_n = (a.N + BN_OUT - 1) / BN_OUT;
    const int64_t n_tiles = (int64_t)a.tiles_m * a.tiles_n;
    RAVEN_REQUIRE(n_tiles < (1 << 28), "gemm (ring): too many tiles (M=%d N=%d)", a.M, a.N);
    const unsigned grid = (unsigned)((n_tiles + 7) / 8 * 8);
    gemm_ring_kernel<SWIGLU><<<dim3(grid), dim3(256), lds, s>>>(a);
    return raven_host::check_launch("gemm (ring MFMA)");
}

int g_tiled_min_rows = 33;  // raven_set_tuning("gemm_tiled_min_rows"): fewest rows that take this kernel
int g_tiled_variant = 0;    // raven_set_tuning("gemm_tiled_variant"): 0 = by shape, 1 = 256 x 256 tiles, 2 = 128 x 128 tiles, 3 = 256 x 256 tiles by the eight-wave kernel
int g_tiled_split_tail = 1; // raven_set_tuning("gemm_tiled_split_tail"): 0 = never hand the last round's tile columns to 128 x 128 tiles

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
// those go to the skinny kernels, 32 rows per pass over the weights -- up to two passes at K = 5280, four at 10560 and
// five (160 rows) at 17920, where the passes' split over K still beats one round of 128 x 128 tiles walking the whole of K
// (measured at 33 .. 160 rows: Wqkv 98 / 130 us in three / four passes against 75 / 81 tiled, mlp.proj 172 against 199).
bool tiled_gemm_fits(int M, int N, int K0, int K1, int dtype) {
    const int64_t small_tiles = (int64_t)((M + 127) / 128) * ((N + 127) / 128);
    const int passes = (K0 + K1 + 3499) / 3500;
    if (g_tiled_variant == 0 && small_tiles < 128 && M <= 160 && M <= 32 * passes) return false;
    return dtype == RAVEN_BF16 && M >= 1 && N % 8 == 0 && K0 % 8 == 0 && K0 > 0 && (K1 == 0 || K1 == K0) && (int64_t)M * (K0 > K1 ? K0 : K1) < (1ll << 31) &&
           (int64_t)N * 2 * (K0 + K1) < (1ll << 31);
}

// Copies of weight matrices with their rows padded to whole 128-byte lines (raven_register_packed_weight): at K = 5280 every
// second row of [N, K] starts 64 bytes into a line, each 128-byte row piece of a K step is then two half lines, and the
// tiled kernels lose 5 to 7 % to the extra requests.  Keyed by the address of the matrix as the caller passes it.
struct PackedWeight {
    const bf16* packed;
    int rows, K, ld;
};
static std::mutex g_packed_mutex;
static std::unordered_map<const void*, PackedWeight> g_packed;

// The registered copy of w ([rows, K]) and its row pitch, or null
const void* packed_weight_of(const void* w, int rows, int K, int* ld) {
    std::lock_guard<std::mutex> lock(g_packed_mutex);
    const auto it = g_packed.find(w);
    if (it == g_packed.end() || it->second.K != K || it->second.rows != rows) return nullptr;
    *ld = it->second.ld;
    return it->second.packed;
}

__global__ __launch_bounds__(256) void pack_rows_kernel(const bf16* __restrict__ w, bf16* __restrict__ out, int K, int ld) {
    const int64_t row = blockIdx.x;
    for (int c = threadIdx.x * 8; c < ld; c += 256 * 8) {
        Chunk<bf16> v = zero_chunk<bf16>();
        if (c < K) v = load_chunk(w + row * K + c);
        store_chunk(out + row * ld + c, v);
    }
}

static int tiled_gemm_impl(const void* x0, int ldx, const void* x1, const void* w, const void* residual, void* y, int M, int N, int K0,
                           int K1, int swiglu, int out_f32, const TiledArgs::RopeAppend* rope, hipStream_t s) {
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
    a.ldy = N;
    a.up_off = N;
    a.ldw = K0 + a.K1;
    a.ldx = ldx > 0 ? ldx : K0;
    RAVEN_REQUIRE(a.ldx >= K0 && a.ldx % 8 == 0 && (a.ldx == K0 || a.K1 == 0) && (int64_t)M * a.ldx < (1ll << 31), "gemm (tiled): bad row pitch %d of x", ldx);
    {
        std::lock_guard<std::mutex> lock(g_packed_mutex);
        const auto it = g_packed.find(w);
        if (it != g_packed.end() && it->second.K == a.ldw && it->second.rows == (swiglu ? 2 * N : N) && (int64_t)it->second.rows * it->second.ld < (1ll << 31)) {
            a.w = it->second.packed;
            a.ldw = it->second.ld;
        }
    }
    if (rope) {
        a.rope = *rope;
        a.rope_on = 1;
    }
    // 256 x 256 tiles when they fill the chip at least once; 128 x 128 tiles otherwise
    const int bn_out = swiglu ? 128 : 256;
    const int64_t tiles_n = (N + bn_out - 1) / bn_out, tiles_m = (M + 255) / 256;
    const int64_t big_tiles = tiles_m * tiles_n;
    const bool big = g_tiled_variant == 1 || g_tiled_variant == 3 || (g_tiled_variant == 0 && big_tiles >= 256);
    auto launch = [&](const TiledArgs& t, bool as_big) {
        // 256 x 256 tiles: four waves, operands straight into an LDS ring (5 to 8 % faster than eight waves with staging
        // registers at the model's shapes, same bits); the eight-wave kernel stays selectable and serves the small tiles
        if (as_big && g_tiled_variant != 3) return swiglu ? launch_ring<true>(t, s) : launch_ring<false>(t, s);
        if (swiglu) return as_big ? launch_tiled<true, 4, 2>(t, s) : launch_tiled<true, 2, 1>(t, s);
        return as_big ? launch_tiled<false, 4, 2>(t, s) : launch_tiled<false, 2, 1>(t, s);
    };
    // The last round of 256 x 256 tiles: when it would fill at most half of the 256 CUs and is whole tile columns, those
    // columns are multiplied as 128 x 128 tiles instead -- four times as many workgroups, a quarter of the time each
    // (5.25 rounds of work then take about 5.4 rounds instead of 6: the N = 5280 products of the model at 16384 rows;
    // mlp.fc of a 512-token prompt: 280 tiles, 1.3 rounds instead of 2).
    const int64_t rest = big_tiles % 256;
    if (big && g_tiled_variant == 0 && g_tiled_split_tail && big_tiles > 256 && rest > 0 && rest <= 128 && rest % tiles_m == 0) {
        const int cols = (int)(rest / tiles_m);              // trailing tile columns
        const int n_big = (int)(tiles_n - cols) * bn_out;    // output columns of the first launch
        TiledArgs head = a, tail = a;
        head.N = n_big;
        tail.N = N - n_big;
        tail.w = a.w + (int64_t)n_big * a.ldw;
        tail.residual = a.residual ? a.residual + n_big : nullptr;
        tail.y = out_f32 ? static_cast<void*>(static_cast<float*>(y) + n_big) : static_cast<void*>(static_cast<bf16*>(y) + n_big);
        tail.rope.col0 = n_big;
        const int rc = launch(head, true);
        return rc ? rc : launch(tail, false);
    }
    return launch(a, big);
}

int tiled_gemm(const void* x0, const void* x1, const void* w, const void* residual, void* y, int M, int N, int K0, int K1, int swiglu,
               int out_f32, hipStream_t s) {
    return tiled_gemm_impl(x0, 0, x1, w, residual, y, M, N, K0, K1, swiglu, out_f32, nullptr, s);
}

// The same with the rows of x `ldx` elements apart (>= K, one segment): activations whose rows are padded to whole cache lines
int tiled_gemm_pitched(const void* x, int ldx, const void* w, const void* residual, void* y, int M, int N, int K, int swiglu, hipStream_t s) {
    return tiled_gemm_impl(x, ldx, nullptr, w, residual, y, M, N, K, 0, swiglu, 0, nullptr, s);
}

// A chunk's q | k | v product (wqkv: [3 * nh * hd, K]) whose epilogue adds the q / k bias, applies RoPE and writes q to
// q_out [M, nh * hd] and k, v to the cache rows of positions pos0 (or *pos_dev) + 0 .. S - 1 of each of the M / S sequences:
// the product itself is never stored.  k_cache / v_cache: the cache tensors, slot_off the slot's element offset.
int tiled_gemm_qkv_rope(const void* x, const void* wqkv, const void* qk_bias, const float* freqs, void* q_out, void* k_cache,
                        void* v_cache, int64_t slot_off, int nh, int hd, int t_max, int M, int S, int K, int ldx, int pos0,
                        const int* pos_dev, hipStream_t s) {
    RAVEN_REQUIRE(freqs && q_out && k_cache && v_cache && hd % 8 == 0 && S > 0 && M % S == 0, "gemm (tiled, q/k/v epilogue): bad arguments");
    TiledArgs::RopeAppend r{};
    r.freqs = freqs;
    r.qk_bias = static_cast<const bf16*>(qk_bias);
    r.q_out = static_cast<bf16*>(q_out);
    r.k = static_cast<bf16*>(k_cache);
    r.v = static_cast<bf16*>(v_cache);
    r.slot_off = slot_off;
    r.pos_dev = pos_dev;
    r.nh = nh; r.hd = hd; r.t_max = t_max; r.S = S; r.pos0 = pos0; r.col0 = 0;
    return tiled_gemm_impl(x, ldx, nullptr, wqkv, nullptr, nullptr, M, 3 * nh * hd, K, 0, 0, 0, &r, s);
}

}  // namespace raven

extern "C" int64_t raven_packed_weight_bytes(int32_t rows, int32_t K) {
    if (rows <= 0 || K <= 0) return 0;
    return (int64_t)rows * ((K + 63) / 64 * 64) * (int64_t)sizeof(raven::bf16);
}

extern "C" int raven_register_packed_weight(const void* w, int32_t rows, int32_t K, void* packed, void* stream) {
    using namespace raven;
    RAVEN_REQUIRE(w && packed && rows > 0 && K > 0 && K % 8 == 0, "register_packed_weight: bad arguments (rows=%d K=%d)", rows, K);
    RAVEN_REQUIRE(((uintptr_t)w & 15) == 0 && ((uintptr_t)packed & 127) == 0, "register_packed_weight: w must be 16-byte and packed 128-byte aligned");
    const int ld = (K + 63) / 64 * 64;
    pack_rows_kernel<<<dim3((unsigned)rows), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(static_cast<const bf16*>(w), static_cast<bf16*>(packed), K, ld);
    if (int rc = raven_host::check_launch("register_packed_weight")) return rc;
    std::lock_guard<std::mutex> lock(g_packed_mutex);
    g_packed[w] = PackedWeight{static_cast<const bf16*>(packed), rows, K, ld};
    return 0;
}

extern "C" int raven_unregister_packed_weight(const void* w) {
    using namespace raven;
    std::lock_guard<std::mutex> lock(g_packed_mutex);
    g_packed.erase(w);
    return 0;
}

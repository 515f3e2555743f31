// Causal attention for prefill chunks (many query rows per sequence) on the matrix cores, bf16.
//
// softmax(q K^T / sqrt(hd)) V for the S new rows of each sequence against positions 0 .. pos0 + s of
// the step-indexed KV cache (the three mask cases of recpre/raven_modeling_minimal.py:484-491 with
// S > 1: plain causal when the cache was empty, lower-right-aligned causal otherwise).  The new
// keys/values are already in the cache (raven_qkv_bias_rope_cache_append ran before).
//
// Grid (query blocks of 64 or 128 rows, heads, sequences), the blocks with the most keys first; 4 waves, each owns
// RG groups of 16 query rows (RG = 1 or 2) and walks all key tiles of 64 positions on its own (no cross-wave softmax
// state).  Per key tile:
//   * the workgroup stages K [64 x hd] and V [64 x hd] in one of two LDS buffers, through registers that
//     were loaded one tile earlier (so the tile two ahead is in flight during the products; one barrier per tile);
//   * S^T = K Q^T with v_mfma_f32_16x16x32_bf16, every K fragment multiplied into all row groups: a lane then holds,
//     for ONE query (l % 16) of each group, the scores of keys 4*(l/16) + v of each 16-key sub-tile -- exactly the
//     lane-row / k-slice shape the A operand of the next MFMA wants, so P never leaves registers: the 32 "k" slots
//     of a P V MFMA are mapped to keys (sub-tile pair, 4*(l/16) + v), and V is read from LDS with ds_read_b64_tr_b16 in that order (no transposed copy);
//   * online softmax per query against a reference maximum that moves only when a tile exceeds it by 2^8 (O is then
//     rescaled, with factors fetched by one shuffle per row); exp2 with the scale folded in; the row sums come from
//     one more MFMA against a tile of ones, in O's own layout;
//   * O += P V with three V fragments in flight and the exponentials of the second k-step between the products of
//     the first; the wave raises its priority for the product phases so that the other wave of the SIMD fills the
//     gaps with its softmax.
// The output goes through LDS once, to be written as 16-byte pieces of whole rows.

#include <math.h>

#include <type_traits>

#include "raven_common.h"

namespace raven {

constexpr int kPfKeys = 64;     // keys per tile

struct PrefillArgs {
    const bf16* q;   // [B*S, h]
    bf16* y;         // [B*S, h], rows ldy elements apart
    int ldy;
    const bf16* k;   // cache tensors
    const bf16* v;
    int64_t slot_off;
    int nh, hd, t_max, S, pos0;
    const int* pos_dev;
    float scale_log2;
    // block-paged caches (the PAGED kernels): sequence b's query rows are q_start[b] .. q_start[b + 1] - 1 of q, they are
    // the LAST positions of its seq_lens[b] cached positions, and position p lives in page block_table[b][p / block_size]
    const int* block_table;  // [B, max_blocks]
    const int* seq_lens;     // [B]
    const int* q_start;      // [B + 1]
    int max_blocks, block_size, block_shift;  // block_shift = log2(block_size), or -1 when that is not a power of two
    int64_t page_stride, pos_stride, head_stride;  // elements between two pages / positions of a page / heads
};

constexpr int kPfTable = 1024;  // block-table entries of a sequence held in LDS (beyond that they are read from memory)

// Maximum over the four lanes l, l^16, l^32, l^48 (the lanes that share a query), in every lane, with the two row-swap
// instructions of gfx950 instead of two round trips through the LDS crossbar: after v_permlane16_swap of a register
// with a copy of itself the pair holds rows (0,0,2,2) and (1,1,3,3) of 16 lanes, after v_permlane32_swap the two halves.
__device__ __forceinline__ float max_over_quarters(float x) {
    typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
    unsigned u = __builtin_bit_cast(unsigned, x);
    const u32x2 r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    u = __builtin_bit_cast(unsigned, fmaxf(__builtin_bit_cast(float, r[0]), __builtin_bit_cast(float, r[1])));
    const u32x2 q = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__builtin_bit_cast(float, q[0]), __builtin_bit_cast(float, q[1]));
}

template <int HD, int RG, bool PAGED = false, int NW = 4>
__global__ __launch_bounds__(NW * 64, NW == 6 ? 3 : 2) void attention_prefill_kernel(PrefillArgs a) {
    constexpr int NTH = NW * 64;     // threads; NW waves, each with its own query rows
    constexpr int KS = HD / 32;      // k-steps of the score MFMA
    constexpr int NT = HD / 16;      // 16-wide output tiles of O; tile NT holds the row sums
    constexpr int KP = HD + 8;       // K tile row pitch (elements): (HD*2+16) bytes, 16-byte aligned rows
    constexpr int WR = 16 * RG;      // query rows per wave
    constexpr int ROWS = NW * WR;    // query rows per workgroup
    constexpr int kVPitch = HD + 16;
    // one block of LDS: the two K buffers, then the two V buffers; the output pass at the end reuses all of it
    constexpr int SK_ELEMS = 2 * kPfKeys * KP, SV_ELEMS = 2 * kPfKeys * kVPitch;
    static_assert(SK_ELEMS + SV_ELEMS >= NW * (RG == 1 ? 16 : 32) * KP, "the output pass fits the staging buffers");
    __shared__ __align__(16) bf16 smem_kv[SK_ELEMS + SV_ELEMS];
    bf16(*sk)[kPfKeys][KP] = reinterpret_cast<bf16(*)[kPfKeys][KP]>(smem_kv);
    // bf16 elements per V row in LDS: HD + 16, i.e. 40 / 56 / 72 banks -- an odd multiple of 8, so that the 8 key rows that
    // 32 lanes read transposed (8 banks each) hit 64 different banks
    bf16(*sv)[kPfKeys][kVPitch] = reinterpret_cast<bf16(*)[kPfKeys][kVPitch]>(smem_kv + SK_ELEMS);

    const int qb = gridDim.x - 1 - blockIdx.x;  // the blocks with the most keys start first
    const int head = blockIdx.y, b = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int qc = lane & 15, s4 = lane >> 4;
    const int h = a.nh * HD;
    __shared__ int tbl[PAGED ? kPfTable : 1];
    // rows of this sequence in q / y, their number, the number of cached positions that may be read, and the position
    // of the first row
    int64_t q_row0;
    int n_rows, t_lim, pos0;
    const int* table_row = nullptr;
    if constexpr (PAGED) {
        q_row0 = a.q_start[b];
        n_rows = a.q_start[b + 1] - (int)q_row0;
        t_lim = a.seq_lens[b];
        pos0 = t_lim - n_rows;
        table_row = a.block_table + (int64_t)b * a.max_blocks;
        if (n_rows <= 0 || pos0 < 0 || qb * ROWS >= n_rows) return;  // the grid is sized for the longest sequence
    } else {
        q_row0 = (int64_t)b * a.S;
        n_rows = a.S;
        t_lim = a.t_max;
        pos0 = a.pos_dev ? *a.pos_dev : a.pos0;
    }

    const int row0 = qb * ROWS + wave * WR;            // first query row (within the sequence) of this wave
    const int64_t head_off = PAGED ? (int64_t)head * a.head_stride : a.slot_off + ((int64_t)b * a.nh + head) * a.t_max * HD;
    const bf16* Kb = a.k + head_off;
    const bf16* Vb = a.v + head_off;

    // Q fragments (B operand of S^T = K Q^T): lane supplies Q[q = l%16][d = 32*ks + 8*(l/16) ..+8] of each row group
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
    bf16x8 qf[RG][KS];
    int my_limit[RG];  // the query of group g whose scores this lane holds sees keys <= my_limit[g]
#pragma unroll
    for (int g = 0; g < RG; ++g) {
        const int my_row = row0 + 16 * g + qc;
        my_limit[g] = pos0 + my_row;
        const bf16* qp = a.q + (q_row0 + min(my_row, n_rows - 1)) * h + head * HD + 8 * s4;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qf[g][ks] = *reinterpret_cast<const bf16x8*>(qp + 32 * ks);
    }

    f32x4 o[RG][NT + 1];
    float ms_run[RG];  // reference maximum of each query's scores, in scaled log2 units
#pragma unroll
    for (int g = 0; g < RG; ++g) {
        ms_run[g] = -INFINITY;
#pragma unroll
        for (int nt = 0; nt <= NT; ++nt) o[g][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    bf16x8 ones;
#pragma unroll
    for (int e = 0; e < 8; ++e) ones[e] = static_cast<bf16>(1.0f);

    // keys this workgroup needs: everything up to the last row's own position
    const int last_row = min(qb * ROWS + ROWS, n_rows) - 1;
    const int n_keys = min(pos0 + last_row + 1, t_lim);
    const int wave_last = pos0 + row0 + WR - 1;  // the last key that any row of this wave sees

    // Global -> registers -> LDS, two tiles ahead of the multiply and two LDS buffers: the loads of tile i + 2 are in
    // flight while tile i is multiplied and tile i + 1 sits in the other buffer; one barrier per tile.
    // K and V tiles are contiguous pieces of the cache (or gathered page rows), moved as 16-byte chunks of key rows; V
    // stays row-major in LDS and is read through ds_read_b64_tr_b16, which hands a lane four keys of one column.
    constexpr int CPR = HD / 8;                     // chunks per key row
    constexpr int KCH = kPfKeys * CPR / NTH;        // chunks per thread, of K and of V
    static_assert(kPfKeys * CPR % NTH == 0, "staging shape");
    u32x4 kreg[KCH];
    u32x4 vreg[KCH];
    const bf16* k_src = Kb + threadIdx.x * 8;
    const bf16* v_src = Vb + threadIdx.x * 8;
    int k_dst[KCH], v_dst[KCH];  // element offsets inside one buffer
#pragma unroll
    for (int i = 0; i < KCH; ++i) {
        const int c = threadIdx.x + NTH * i;
        k_dst[i] = (c / CPR) * KP + (c % CPR) * 8;
        v_dst[i] = (c / CPR) * kVPitch + (c % CPR) * 8;
    }
    // paged: element offset of position p's head row.  Positions past the last key this workgroup needs repeat that key
    // (they are masked): only the pages up to it are in `tbl`, and only those are known to exist.
    auto paged_off = [&](int p) {
        p = min(p, n_keys - 1);
        const int pg = a.block_shift >= 0 ? p >> a.block_shift : p / a.block_size;
        const int page = pg < kPfTable ? tbl[pg] : table_row[pg];
        return (int64_t)page * a.page_stride + (int64_t)(p - pg * a.block_size) * a.pos_stride;
    };
    auto fetch = [&](int kt) {
        if constexpr (PAGED) {
            if (a.block_shift >= 0 && kt + kPfKeys <= n_keys) {
                // a whole tile of needed keys, pages of 2^n positions: shifts instead of divisions, no clamping
                const int mask = a.block_size - 1;
                auto off = [&](int p) {
                    const int pg = p >> a.block_shift;
                    const int page = pg < kPfTable ? tbl[pg] : table_row[pg];
                    return (int64_t)page * a.page_stride + (int64_t)((p & mask) * (int)a.pos_stride);
                };
#pragma unroll
                for (int i = 0; i < KCH; ++i) {
                    const int c = threadIdx.x + NTH * i;
                    const int key = c / CPR, dc = c - key * CPR;
                    const int64_t o = off(kt + key);
                    kreg[i] = *reinterpret_cast<const u32x4*>(Kb + o + dc * 8);
                    vreg[i] = *reinterpret_cast<const u32x4*>(Vb + o + dc * 8);
                }
            } else {
#pragma unroll
                for (int i = 0; i < KCH; ++i) {
                    const int c = threadIdx.x + NTH * i;
                    const int key = c / CPR, dc = c - key * CPR;
                    const int64_t o = paged_off(kt + key);
                    kreg[i] = *reinterpret_cast<const u32x4*>(Kb + o + dc * 8);
                    vreg[i] = *reinterpret_cast<const u32x4*>(Vb + o + dc * 8);
                }
            }
        } else if (kt + kPfKeys <= a.t_max) {
#pragma unroll
            for (int i = 0; i < KCH; ++i) kreg[i] = *reinterpret_cast<const u32x4*>(k_src + (int64_t)kt * HD + NTH * 8 * i);
#pragma unroll
            for (int i = 0; i < KCH; ++i) vreg[i] = *reinterpret_cast<const u32x4*>(v_src + (int64_t)kt * HD + NTH * 8 * i);
        } else {  // the cache ends inside this tile: rows past it are masked below, their loads stay in bounds
#pragma unroll
            for (int i = 0; i < KCH; ++i) {
                const int c = threadIdx.x + NTH * i;
                const int key = c / CPR, dc = c - key * CPR;
                const int64_t o = (int64_t)min(kt + key, a.t_max - 1) * HD + dc * 8;
                kreg[i] = *reinterpret_cast<const u32x4*>(Kb + o);
                vreg[i] = *reinterpret_cast<const u32x4*>(Vb + o);
            }
        }
    };
    auto park = [&](int buf) {
        bf16* kb = &sk[buf][0][0];
#pragma unroll
        for (int i = 0; i < KCH; ++i) *reinterpret_cast<u32x4*>(kb + k_dst[i]) = kreg[i];
        bf16* vb = &sv[buf][0][0];
#pragma unroll
        for (int i = 0; i < KCH; ++i) *reinterpret_cast<u32x4*>(vb + v_dst[i]) = vreg[i];
    };

    // One key tile against the wave's rows.  MASKED: some key of the tile is hidden from some row (the tiles on the
    // diagonal); all other tiles run the same code without the comparisons.
    auto tile = [&](int kt, int buf, auto masked_tag) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        // S^T sub-tiles: sc[g][t][v] = score of key kt + 16 t + 4 s4 + v against query qc of group g
        f32x4 sc[RG][4];
#pragma unroll
        for (int g = 0; g < RG; ++g)
#pragma unroll
            for (int t = 0; t < 4; ++t) sc[g][t] = f32x4{0.f, 0.f, 0.f, 0.f};
        __builtin_amdgcn_s_setprio(3);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const bf16x8 kf = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&sk[buf][16 * t + qc][32 * ks + 8 * s4]));
#pragma unroll
                for (int g = 0; g < RG; ++g) sc[g][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[g][ks], sc[g][t], 0, 0, 0);
            }
        __builtin_amdgcn_s_setprio(0);
        float ms_new[RG];
        bool moved = false;
#pragma unroll
        for (int g = 0; g < RG; ++g) {
            if (MASKED) {
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        if (kt + 16 * t + 4 * s4 + v > my_limit[g]) sc[g][t][v] = -INFINITY;
            }
            float mx = -INFINITY;
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int v = 0; v < 4; ++v) mx = fmaxf(mx, sc[g][t][v]);
            mx = max_over_quarters(mx);
            // The reference maximum follows the scores lazily: it moves only when a tile exceeds it by more than 2^8
            // (weights stay below 256, far inside the range of float and bf16), so O is rescaled a few times per query
            // instead of whenever any of its 16 queries sees a new maximum.
            const float mxs = mx * a.scale_log2;
            const bool up = mxs > ms_run[g] + 8.f;
            ms_new[g] = up ? mxs : ms_run[g];
            moved |= up;
        }
        if (__builtin_amdgcn_ballot_w64(moved) != 0) {
#pragma unroll
            for (int g = 0; g < RG; ++g) {
                // 0 for the first tile, 1 where nothing moved (also for a query that has not seen a key yet)
                const float corr = (ms_new[g] == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(ms_run[g] - ms_new[g]);
                // O rows are queries 4*s4 + v: fetch their factor from the lane that tracks that query
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float cv = __shfl(corr, 4 * s4 + v, 64);
#pragma unroll
                    for (int nt = 0; nt <= NT; ++nt) o[g][nt][v] *= cv;
                }
                ms_run[g] = ms_new[g];
            }
        }
        // O += P V in 2*NT steps: step i multiplies V fragment i = (k-step c = i / NT, columns 16*(i % NT) ..+15) into both
        // row groups.  Three fragments are in flight (the first ones are requested before the exponentials), and the
        // exponentials of the second k-step sit between the products of the first; scheduling fences keep that order.
        constexpr int NF = 2 * NT;
        // V fragment i, the B operand [32 key slots x 16 columns]: two transposing reads.  In each, lane l of a group of 16
        // points at four columns (4 * (l % 4) ..+3 of the tile's 16) of key row l / 4 of four, and receives the four keys
        // of column l % 16; the four keys are 4 * s4 ..+3 of sub-tile 2c (first read) and 2c + 1 (second), P's order.
        typedef short s16x4 __attribute__((ext_vector_type(4)));
        const bf16* vtr = &sv[buf][4 * s4 + (qc >> 2)][4 * (qc & 3)];
        auto vfrag = [&](int i) {
            const bf16* p0 = vtr + (32 * (i / NT)) * kVPitch + 16 * (i % NT);
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(p0));
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(p0 + 16 * kVPitch));
            return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        };
        bf16x8 vf[3];
#pragma unroll
        for (int i = 0; i < 3; ++i) vf[i] = vfrag(i);
        float ms[RG];
        bf16x8 pf[RG][2];
#pragma unroll
        for (int g = 0; g < RG; ++g) {
            // a query with no visible key yet (rows past S only) still has -inf: subtract 0 instead, every weight is then 0
            ms[g] = (ms_run[g] == -INFINITY) ? 0.f : ms_run[g];
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    pf[g][0][t * 4 + v] = static_cast<bf16>(__builtin_amdgcn_exp2f(__builtin_fmaf(sc[g][t][v], a.scale_log2, -ms[g])));
        }
        constexpr int LATE = RG * 8;                 // weights of the second k-step
        constexpr int PER = (LATE + NT - 1) / NT;    // of them per step of the first k-step
        __builtin_amdgcn_s_setprio(3);
#pragma unroll
        for (int i = 0; i < NF; ++i) {
            __builtin_amdgcn_sched_barrier(0);
            const int c = i / NT, nt = i % NT;
#pragma unroll
            for (int g = 0; g < RG; ++g) o[g][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf[g][c], vf[i % 3], o[g][nt], 0, 0, 0);
            // the row sums, in O's layout, from the weights as rounded for the product: a tile of ones as V
            if (nt == NT - 1) {
#pragma unroll
                for (int g = 0; g < RG; ++g) o[g][NT] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf[g][c], ones, o[g][NT], 0, 0, 0);
            }
            if (i + 3 < NF) vf[i % 3] = vfrag(i + 3);
            if (c == 0) {
#pragma unroll
                for (int j = nt * PER; j < (nt + 1) * PER && j < LATE; ++j) {
                    const int g = j / 8, e = j % 8;
                    pf[g][1][e] = static_cast<bf16>(__builtin_amdgcn_exp2f(__builtin_fmaf(sc[g][2 + e / 4][e % 4], a.scale_log2, -ms[g])));
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_setprio(0);
    };

    if constexpr (PAGED) {
        const int n_pages = min((n_keys + a.block_size - 1) / a.block_size, kPfTable);
        for (int i = threadIdx.x; i < n_pages; i += NTH) tbl[i] = table_row[i];
        __syncthreads();
    }
    if (n_keys > 0) {
        fetch(0);
        park(0);
    }
    // The Q fragments pass through an empty asm statement: the compiler waits for their loads here, once, and inside
    // the loop they are no longer load results -- otherwise its wait for them (counted from the newest load) sits in the
    // loop and drains the tile fetched ahead on every trip.
#pragma unroll
    for (int g = 0; g < RG; ++g)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            u32x4 t = __builtin_bit_cast(u32x4, qf[g][ks]);
            asm volatile("" : "+v"(t));
            qf[g][ks] = __builtin_bit_cast(bf16x8, t);
        }
    if (kPfKeys < n_keys) fetch(kPfKeys);
    __syncthreads();
    int buf = 0;
    for (int kt = 0; kt < n_keys; kt += kPfKeys, buf ^= 1) {
        if (kt + kPfKeys - 1 <= pos0 + row0) tile(kt, buf, std::false_type{});
        else if (kt <= wave_last) tile(kt, buf, std::true_type{});
        if (kt + kPfKeys < n_keys) {
            park(buf ^ 1);  // last read two tiles ago; every wave has passed the barrier since
            if (kt + 2 * kPfKeys < n_keys) fetch(kt + 2 * kPfKeys);
        }
        __syncthreads();
    }

    // Normalise and store.  O row v of this lane is query 4*s4 + v of its group, column 16*nt + qc: the wave turns its
    // rows round through LDS (the K buffers are free after the last barrier; each wave has its own WR x KP piece) and
    // writes 16-byte pieces of whole rows.
    constexpr int ER = RG == 1 ? 16 : 32;  // rows per pass
    bf16* ot = smem_kv + wave * (ER * KP);
#pragma unroll
    for (int g0 = 0; g0 < RG; g0 += ER / 16) {
#pragma unroll
        for (int gg = 0; gg < ER / 16; ++gg)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float inv = __builtin_amdgcn_rcpf(o[g0 + gg][NT][v]);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
                    ot[(16 * gg + 4 * s4 + v) * KP + 16 * nt + qc] = from_f32<bf16>(o[g0 + gg][nt][v] * inv);
            }
        // the wave reads only what it wrote itself: no barrier, the LDS operations of a wave complete in order
        constexpr int OCH = ER * CPR / 64;  // 16-byte pieces per lane
#pragma unroll
        for (int i = 0; i < OCH; ++i) {
            const int c = lane + 64 * i;
            const int r = c / CPR, dc = c - r * CPR;
            const int row = row0 + 16 * g0 + r;
            if (row < n_rows)
                *reinterpret_cast<u32x4*>(a.y + (q_row0 + row) * a.ldy + head * HD + dc * 8) = *reinterpret_cast<const u32x4*>(ot + r * KP + dc * 8);
        }
    }
}

}  // namespace raven

namespace raven {
int g_prefill_waves = 0;  // raven_set_tuning("prefill_waves"): 0 = by shape, 4 or 6 = waves per workgroup where the shape allows both
}

namespace raven {
// raven_prefill_attention with the rows of y ldy elements apart (>= n_heads * head_dim)
int prefill_attention_pitched(const void* q, void* y, int ldy, const raven_kv_cache* cache, int32_t slot, int32_t B, int32_t S,
                              int32_t pos0, const int32_t* pos_dev, int32_t n_heads, int32_t head_dim, int32_t dtype, void* stream) {
    RAVEN_REQUIRE(ldy >= n_heads * head_dim && ldy % 8 == 0, "prefill_attention: bad output row pitch %d", ldy);
    RAVEN_REQUIRE(dtype == RAVEN_BF16, "prefill_attention: bf16 only (dtype %d)", dtype);
    RAVEN_REQUIRE(head_dim == 64 || head_dim == 96 || head_dim == 128, "prefill_attention: head_dim %d not in {64, 96, 128}", head_dim);
    RAVEN_REQUIRE(q && y && cache && cache->k && cache->v, "prefill_attention: null pointer");
    RAVEN_REQUIRE(B > 0 && S > 0 && pos0 >= 0 && n_heads > 0, "prefill_attention: bad B=%d S=%d pos0=%d", B, S, pos0);
    RAVEN_REQUIRE(B <= cache->batch, "prefill_attention: batch %d exceeds the cache's %d", B, cache->batch);
    RAVEN_REQUIRE(cache->steps_present == nullptr || cache->lookup_mode == RAVEN_LOOKUP_NONE,
                  "prefill_attention: partially filled caches (steps_present) are served by raven_decode_attention only");
    const int sl = slot >= 0 ? slot : cache->n_slots + slot;
    RAVEN_REQUIRE(sl >= 0 && sl < cache->n_slots, "prefill_attention: slot %d outside [0, %d)", slot, cache->n_slots);
    RAVEN_REQUIRE(pos0 + S <= cache->t_max, "prefill_attention: positions up to %d exceed the cache length %d", pos0 + S - 1, cache->t_max);
    RAVEN_REQUIRE(B <= 65535 && n_heads <= 65535, "prefill_attention: grid too large");
    PrefillArgs a{};
    a.q = static_cast<const bf16*>(q);
    a.y = static_cast<bf16*>(y);
    a.ldy = ldy;
    a.k = static_cast<const bf16*>(cache->k);
    a.v = static_cast<const bf16*>(cache->v);
    a.slot_off = (int64_t)sl * cache->batch * n_heads * cache->t_max * head_dim;
    a.nh = n_heads; a.hd = head_dim; a.t_max = cache->t_max; a.S = S; a.pos0 = pos0; a.pos_dev = pos_dev;
    a.scale_log2 = (float)(1.0 / sqrt((double)head_dim) * 1.4426950408889634);
    hipStream_t s = static_cast<hipStream_t>(stream);
    // Two row groups of 16 per wave (128 query rows per workgroup) share every K and V fragment read from LDS; short
    // launches keep 64 rows per workgroup so that there are more workgroups than compute units.
    const int64_t wgs128 = (int64_t)((S + 127) / 128) * n_heads * B;
    const int rg = wgs128 >= 512 ? 2 : 1;
    // head_dim 96, long launches: six waves (192 query rows) per workgroup.  Two such workgroups fit a CU's LDS, which
    // puts three waves on every SIMD instead of two, and each staged K / V tile serves half as many rows again.
    const bool six = head_dim == 96 && rg == 2 && g_prefill_waves != 4 &&
                     (g_prefill_waves == 6 || (int64_t)((S + 191) / 192) * n_heads * B >= 512);
    const int rows = six ? 192 : 64 * rg;
    const dim3 grid((S + rows - 1) / rows, n_heads, B);
#define RAVEN_PREFILL(HD)                                                                  \
    if (rg == 2) attention_prefill_kernel<HD, 2><<<grid, dim3(256), 0, s>>>(a);            \
    else attention_prefill_kernel<HD, 1><<<grid, dim3(256), 0, s>>>(a)
    if (six) attention_prefill_kernel<96, 2, false, 6><<<grid, dim3(384), 0, s>>>(a);
    else if (head_dim == 64) { RAVEN_PREFILL(64); }
    else if (head_dim == 96) { RAVEN_PREFILL(96); }
    else { RAVEN_PREFILL(128); }
#undef RAVEN_PREFILL
    return raven_host::check_launch("prefill_attention");
}
}  // namespace raven

extern "C" int raven_prefill_attention(const void* q, void* y, const raven_kv_cache* cache, int32_t slot, int32_t B, int32_t S,
                                       int32_t pos0, const int32_t* pos_dev, int32_t n_heads, int32_t head_dim, int32_t dtype,
                                       void* stream) {
    return raven::prefill_attention_pitched(q, y, n_heads * head_dim, cache, slot, B, S, pos0, pos_dev, n_heads, head_dim, dtype, stream);
}

extern "C" int raven_paged_prefill_attention(const void* q, void* y, const void* k_cache, const void* v_cache,
                                             const int32_t* block_table, const int32_t* seq_lens, const int32_t* q_start, int32_t B,
                                             int32_t max_q_len, int32_t max_blocks, int32_t block_size, int32_t kv_layout,
                                             int32_t n_heads, int32_t head_dim, int32_t dtype, void* stream) {
    using namespace raven;
    RAVEN_REQUIRE(dtype == RAVEN_BF16, "paged_prefill_attention: bf16 only (dtype %d)", dtype);
    RAVEN_REQUIRE(head_dim == 64 || head_dim == 96 || head_dim == 128, "paged_prefill_attention: head_dim %d not in {64, 96, 128}", head_dim);
    RAVEN_REQUIRE(kv_layout == RAVEN_PAGED_NHD || kv_layout == RAVEN_PAGED_HND, "paged_prefill_attention: unknown kv_layout %d", kv_layout);
    RAVEN_REQUIRE(B >= 0 && B <= 65535 && n_heads > 0 && n_heads <= 65535 && max_q_len >= 0 && max_blocks > 0 && block_size > 0,
                  "paged_prefill_attention: bad B=%d max_q_len=%d max_blocks=%d block_size=%d", B, max_q_len, max_blocks, block_size);
    if (B == 0 || max_q_len == 0) return 0;
    RAVEN_REQUIRE(q && y && k_cache && v_cache && block_table && seq_lens && q_start, "paged_prefill_attention: null pointer");
    PrefillArgs a{};
    a.q = static_cast<const bf16*>(q);
    a.y = static_cast<bf16*>(y);
    a.ldy = n_heads * head_dim;
    a.k = static_cast<const bf16*>(k_cache);
    a.v = static_cast<const bf16*>(v_cache);
    a.nh = n_heads; a.hd = head_dim;
    a.scale_log2 = (float)(1.0 / sqrt((double)head_dim) * 1.4426950408889634);
    a.block_table = block_table; a.seq_lens = seq_lens; a.q_start = q_start;
    a.max_blocks = max_blocks; a.block_size = block_size; a.block_shift = -1;
    for (int sh = 0; sh < 31; ++sh)
        if (block_size == (1 << sh)) a.block_shift = sh;
    RAVEN_REQUIRE((int64_t)block_size * n_heads * head_dim < (1ll << 31), "paged_prefill_attention: a page of %d positions is too large", block_size);
    a.page_stride = (int64_t)block_size * n_heads * head_dim;
    a.pos_stride = kv_layout == RAVEN_PAGED_NHD ? (int64_t)n_heads * head_dim : head_dim;
    a.head_stride = kv_layout == RAVEN_PAGED_NHD ? head_dim : (int64_t)block_size * head_dim;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t wgs128 = (int64_t)((max_q_len + 127) / 128) * n_heads * B;
    const int rg = wgs128 >= 512 ? 2 : 1;
    const int rows = 64 * rg;
    const dim3 grid((max_q_len + rows - 1) / rows, n_heads, B);
#define RAVEN_PREFILL(HD)                                                                        \
    if (rg == 2) attention_prefill_kernel<HD, 2, true><<<grid, dim3(256), 0, s>>>(a);            \
    else attention_prefill_kernel<HD, 1, true><<<grid, dim3(256), 0, s>>>(a)
    if (head_dim == 64) { RAVEN_PREFILL(64); }
    else if (head_dim == 96) { RAVEN_PREFILL(96); }
    else { RAVEN_PREFILL(128); }
#undef RAVEN_PREFILL
    return raven_host::check_launch("paged_prefill_attention");
}

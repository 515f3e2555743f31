// Causal attention for prefill chunks (many query rows per sequence) on the matrix cores, bf16.
//
// softmax(q K^T / sqrt(hd)) V for the S new rows of each sequence against positions 0 .. pos0 + s of
// the step-indexed KV cache (the three mask cases of recpre/raven_modeling_minimal.py:484-491 with
// S > 1: plain causal when the cache was empty, lower-right-aligned causal otherwise).  The new
// keys/values are already in the cache (raven_qkv_bias_rope_cache_append ran before).
//
// Grid (query blocks of 64, heads, sequences); 4 waves, each owns 16 query rows and walks all key
// tiles of 64 positions on its own (no cross-wave softmax state).  Per key tile:
//   * the workgroup stages K [64 x hd] and V transposed [hd x 64] in LDS;
//   * S^T = K Q^T with v_mfma_f32_16x16x32_bf16: a lane then holds, for ONE query (l % 16), the scores
//     of keys 4*(l/16) + v of each 16-key sub-tile -- exactly the lane-row / k-slice shape the A operand
//     of the next MFMA wants, so P never leaves registers: the 32 "k" slots of a P V MFMA are mapped to
//     keys (sub-tile pair, 4*(l/16) + v), and V^T is read from LDS with the same mapping;
//   * online softmax per query: max/sum across the 4 lanes that share a query (two shuffles each),
//     exp2 with the scale folded in; the output tile O [16 q x hd] lives in the MFMA accumulator layout
//     (q = 4*(l/16) + v), so the per-query rescale factors are fetched with one shuffle per v.

#include <math.h>

#include "raven_common.h"

namespace raven {

constexpr int kPfKeys = 64;     // keys per tile
constexpr int kPfRows = 64;     // query rows per workgroup
constexpr int kVtPitch = 72;    // bf16 elements per V^T row: 64 + 8 (144 bytes: the 8-byte reads of a half-wave hit 32 different bank pairs)

struct PrefillArgs {
    const bf16* q;   // [B*S, h]
    bf16* y;         // [B*S, h]
    const bf16* k;   // cache tensors
    const bf16* v;
    int64_t slot_off;
    int nh, hd, t_max, S, pos0;
    const int* pos_dev;
    float scale_log2;
};

template <int HD>
__global__ __launch_bounds__(256) void attention_prefill_kernel(PrefillArgs a) {
    constexpr int KS = HD / 32;      // k-steps of the score MFMA
    constexpr int NT = HD / 16;      // 16-wide output tiles of O
    constexpr int KP = HD + 8;       // K tile row pitch (elements): (HD*2+16) bytes, 16-byte aligned rows
    __shared__ __align__(16) bf16 sk[kPfKeys][KP];
    __shared__ __align__(16) bf16 svt[HD][kVtPitch];

    const int qb = blockIdx.x, head = blockIdx.y, b = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int qc = lane & 15, s4 = lane >> 4;
    const int h = a.nh * HD;
    const int pos0 = a.pos_dev ? *a.pos_dev : a.pos0;

    const int row0 = qb * kPfRows + wave * 16;         // first query row (within the sequence) of this wave
    const int my_row = row0 + qc;                      // the query whose scores this lane holds
    const int64_t head_off = a.slot_off + ((int64_t)b * a.nh + head) * a.t_max * HD;
    const bf16* Kb = a.k + head_off;
    const bf16* Vb = a.v + head_off;

    // Q fragments (B operand of S^T = K Q^T): lane supplies Q[q = l%16][d = 32*ks + 8*(l/16) ..+8]
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    bf16x8 qf[KS];
    {
        const int r = min(my_row, a.S - 1);
        const bf16* qp = a.q + ((int64_t)b * a.S + r) * h + head * HD + 8 * s4;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qf[ks] = *reinterpret_cast<const bf16x8*>(qp + 32 * ks);
    }

    f32x4 o[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) o[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;

    // keys this workgroup needs: everything up to the last row's own position
    const int last_row = min(qb * kPfRows + kPfRows, a.S) - 1;
    const int n_keys = min(pos0 + last_row + 1, a.t_max);
    const int my_limit = pos0 + my_row;  // this lane's query sees keys <= my_limit

    // Global -> registers -> LDS, one tile ahead: the loads of tile kt + 64 are in flight while tile kt is multiplied.
    // K: 16-byte chunks, row-major.  V: a thread takes the same 8 columns of 4 consecutive keys and writes, per
    // column, the 4 keys as one 8-byte piece of the transposed tile.
    constexpr int CPR = HD / 8;                          // chunks per key row
    constexpr int KCH = (kPfKeys * CPR + 255) / 256;     // K chunks per thread
    constexpr int VTASKS = (kPfKeys / 4) * CPR;          // V tasks per tile (at most 256)
    static_assert(VTASKS <= 256, "one V task per thread");
    u32x4 kreg[KCH];
    Chunk<bf16> vreg[4];
    const int v_kg = threadIdx.x % (kPfKeys / 4), v_dc = threadIdx.x / (kPfKeys / 4);
    auto fetch = [&](int kt) {
#pragma unroll
        for (int i = 0; i < KCH; ++i) {
            const int c = threadIdx.x + 256 * i;
            if (c < kPfKeys * CPR) {
                const int key = c / CPR, dc = c - key * CPR;
                const int kpos = min(kt + key, a.t_max - 1);  // rows past n_keys are masked below; stay in bounds
                kreg[i] = *reinterpret_cast<const u32x4*>(Kb + (int64_t)kpos * HD + dc * 8);
            }
        }
        if (threadIdx.x < VTASKS) {
#pragma unroll
            for (int i = 0; i < 4; ++i) vreg[i] = load_chunk(Vb + (int64_t)min(kt + 4 * v_kg + i, a.t_max - 1) * HD + v_dc * 8);
        }
    };
    auto park = [&]() {
#pragma unroll
        for (int i = 0; i < KCH; ++i) {
            const int c = threadIdx.x + 256 * i;
            if (c < kPfKeys * CPR) {
                const int key = c / CPR, dc = c - key * CPR;
                *reinterpret_cast<u32x4*>(&sk[key][dc * 8]) = kreg[i];
            }
        }
        if (threadIdx.x < VTASKS) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                bf16 four[4] = {vreg[0].v[e], vreg[1].v[e], vreg[2].v[e], vreg[3].v[e]};
                typedef unsigned int u32x2s __attribute__((ext_vector_type(2)));
                *reinterpret_cast<u32x2s*>(&svt[v_dc * 8 + e][4 * v_kg]) = *reinterpret_cast<const u32x2s*>(four);
            }
        }
    };
    if (n_keys > 0) fetch(0);
    for (int kt = 0; kt < n_keys; kt += kPfKeys) {
        __syncthreads();  // the previous tile has been consumed
        park();
        if (kt + kPfKeys < n_keys) fetch(kt + kPfKeys);
        __syncthreads();

        // S^T sub-tiles: sc[t][v] = score of key kt + 16 t + 4 s4 + v against query qc
        f32x4 sc[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            sc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const bf16x8 kf = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&sk[16 * t + qc][32 * ks + 8 * s4]));
                sc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[ks], sc[t], 0, 0, 0);
            }
        }
        // scale, causal mask (only tiles that reach past the wave's first query need it), tile maximum for this query
        float mx = -INFINITY;
        if (kt + kPfKeys - 1 <= pos0 + row0) {
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    sc[t][v] *= a.scale_log2;
                    mx = fmaxf(mx, sc[t][v]);
                }
        } else {
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int key = kt + 16 * t + 4 * s4 + v;
                    float x = sc[t][v] * a.scale_log2;
                    if (key > my_limit) x = -INFINITY;
                    sc[t][v] = x;
                    mx = fmaxf(mx, x);
                }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        // a query with no visible key yet (rows past S only) has m_new = -inf: subtract 0 instead, every weight is then 0
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        float psum = 0.f;  // over this lane's 16 keys; the four lanes of a query are added up once, after the last tile
        bf16x8 pf[2];
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float p = __builtin_amdgcn_exp2f(sc[t][v] - m_use);
                psum += p;
                pf[t >> 1][(t & 1) * 4 + v] = static_cast<bf16>(p);
            }
        // the running maximum of most queries stops moving after a few tiles: rescale only when some lane's did
        if (__builtin_amdgcn_ballot_w64(m_new != m_run) != 0) {
            const float corr = __builtin_amdgcn_exp2f(m_run - m_use);  // 0 for the first visible tile (m_run = -inf)
            l_run = l_run * corr + psum;
            // O rows are queries 4*s4 + v: fetch their rescale factor from the lane that tracks that query
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float cv = __shfl(corr, 4 * s4 + v, 64);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) o[nt][v] *= cv;
            }
        } else {
            l_run += psum;
        }
        m_run = m_new;

        // O += P V: k-step c covers sub-tiles (2c, 2c+1); slot (s4, e) is key 16*(2c + e/4) + 4*s4 + e%4
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const bf16* vrow = &svt[16 * nt + qc][0];
                typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
                const u32x2 lo = *reinterpret_cast<const u32x2*>(vrow + 32 * c + 4 * s4);
                const u32x2 hi = *reinterpret_cast<const u32x2*>(vrow + 32 * c + 16 + 4 * s4);
                const u32x4 both = {lo.x, lo.y, hi.x, hi.y};
                o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf[c], __builtin_bit_cast(bf16x8, both), o[nt], 0, 0, 0);
            }
    }

    // normalise and store: O row v of this lane is query 4*s4 + v, column 16*nt + qc
    l_run += __shfl_xor(l_run, 16, 64);
    l_run += __shfl_xor(l_run, 32, 64);
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const float lv = __shfl(l_run, 4 * s4 + v, 64);
        const int row = row0 + 4 * s4 + v;
        if (row < a.S) {
            bf16* yp = a.y + ((int64_t)b * a.S + row) * h + head * HD + qc;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) yp[16 * nt] = from_f32<bf16>(o[nt][v] / lv);
        }
    }
}

}  // namespace raven

extern "C" int raven_prefill_attention(const void* q, void* y, const raven_kv_cache* cache, int32_t slot, int32_t B, int32_t S,
                                       int32_t pos0, const int32_t* pos_dev, int32_t n_heads, int32_t head_dim, int32_t dtype,
                                       void* stream) {
    using namespace raven;
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
    PrefillArgs a;
    a.q = static_cast<const bf16*>(q);
    a.y = static_cast<bf16*>(y);
    a.k = static_cast<const bf16*>(cache->k);
    a.v = static_cast<const bf16*>(cache->v);
    a.slot_off = (int64_t)sl * cache->batch * n_heads * cache->t_max * head_dim;
    a.nh = n_heads; a.hd = head_dim; a.t_max = cache->t_max; a.S = S; a.pos0 = pos0; a.pos_dev = pos_dev;
    a.scale_log2 = (float)(1.0 / sqrt((double)head_dim) * 1.4426950408889634);
    const dim3 grid((S + kPfRows - 1) / kPfRows, n_heads, B);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (head_dim == 64) attention_prefill_kernel<64><<<grid, dim3(256), 0, s>>>(a);
    else if (head_dim == 96) attention_prefill_kernel<96><<<grid, dim3(256), 0, s>>>(a);
    else attention_prefill_kernel<128><<<grid, dim3(256), 0, s>>>(a);
    return raven_host::check_launch("prefill_attention");
}

// Composed entry points: one SandwichBlock and one recurrence iteration, as sequences of the
// kernels in this library on one stream.  Follows SandwichBlock.forward and core_block_forward of
// the reference (recpre/raven_modeling_minimal.py:525-536, 764-781):
//   a  = proj(attention(norm_1(x)));  x2 = norm_2(a + x);  out = norm_4(mlp(norm_3(x2)) + x2)
//
// Two schedules:
//   one token row (decode, bs = 1): 5 launches per block -- every RMSNorm rides in the prologue of the
//     GEMV that consumes it (norm_4 of the previous block + norm_1 before Wqkv, norm_2 + norm_3 before
//     mlp.fc), the residual adds ride in the proj / mlp.proj epilogues, bias + RoPE + cache append ride in
//     the attention kernel; one closing norm_4 (+ ln_f) launch per call.
//   several rows: the residual adds still ride in the GEMM epilogues, norm_2 + norm_3 are one launch, and
//     inside an iteration norm_4 of one block and norm_1 of the next are one launch.  From 33 rows on the five
//     products are tiles on the matrix cores (SwiGLU and the residual adds in their epilogues, the adapter's two
//     operands as two K segments), and chunks of 16 or more rows per sequence attend through the MFMA kernel.

#include "raven_common.h"

extern "C" int raven_gemv_fused(const void* x0, const void* x1, const void* norm_a, const void* norm_b, void* xa_out,
                                const void* w, const void* residual, void* y, int32_t N, int32_t K0, int32_t K1, float eps,
                                int32_t swiglu, int32_t out_f32, int32_t dtype, void* stream);

namespace raven {

int gemv1_column_block(const void* x, const void* norm_a, const void* w_block, int ldw, const float* acc_in, void* y, int raw_out,
                       int N, int K, float eps, int dtype, hipStream_t s);

int linear_column_block(const void* x, const void* w_block, int ldw, const float* extra, void* y, int raw_out, int M, int N, int K,
                        void* workspace, size_t workspace_bytes, hipStream_t s);

int linear_leave_sums(const void* x0, const void* x1, const void* w, int ldw, const float* extra, const void* residual, void* y, int M,
                      int N, int K0, int K1, int dtype, void* workspace, size_t workspace_bytes, hipStream_t s, int* ks_left);

int splitk_sums_then_norm(const float* partial, int ks, const float* extra, const void* residual, void* sum_out, const void* weight,
                          void* y, const void* weight2, void* y2, int rows, int dim, float eps, hipStream_t s, int ldy = 0, int ldy2 = 0);
const void* packed_weight_of(const void* w, int rows, int K, int* ld);

int qkv_linear_rope_append(const void* x, int ldx, const void* wqkv, const void* qk_bias, const float* freqs, void* q_out,
                           const raven_kv_cache* cache, int slot, int B, int S, int pos0, const int32_t* pos_dev, int n_heads,
                           int head_dim, int dtype, hipStream_t s, int* done);

extern int g_tiled_min_rows;
bool tiled_gemm_fits(int M, int N, int K0, int K1, int dtype);
int tiled_gemm_pitched(const void* x, int ldx, const void* w, const void* residual, void* y, int M, int N, int K, int swiglu, hipStream_t s);
int rmsnorm_pitched(const void* x, const void* residual, const void* weight, void* y, int ldy, void* sum_out, const void* weight2,
                    void* y2, int ldy2, int64_t rows, int32_t dim, float eps, int32_t dtype, void* stream);
int prefill_attention_pitched(const void* q, void* y, int ldy, const raven_kv_cache* cache, int32_t slot, int32_t B, int32_t S,
                              int32_t pos0, const int32_t* pos_dev, int32_t n_heads, int32_t head_dim, int32_t dtype, void* stream);

// y = round(round(x W^T) + residual), then RMSNorm(weight) -> out1 and RMSNorm(weight2) of that -> out2 (either may be
// null): two launches where the product is K-split (the norm launch adds the slices), three otherwise
static int linear_then_norm(const void* x, const void* w, const void* residual, void* y, const void* weight, void* out1,
                            const void* weight2, void* out2, int M, int N, int K, float eps, int dtype, void* ws, size_t ws_bytes,
                            hipStream_t s, int ld_out2 = 0) {
    int ks = 0;
    if (int rc = linear_leave_sums(x, nullptr, w, 0, nullptr, residual, y, M, N, K, 0, dtype, ws, ws_bytes, s, &ks)) return rc;
    // ld_out2: the row pitch of the LAST output (out2, or out1 when there is no second norm)
    const int ld1 = (weight2 == nullptr && ld_out2) ? ld_out2 : N, ld2 = ld_out2 ? ld_out2 : N;
    if (ks) return splitk_sums_then_norm(static_cast<const float*>(ws), ks, nullptr, residual, nullptr, weight, out1, weight2, out2, M, N, eps, s, ld1, ld2);
    return rmsnorm_pitched(y, nullptr, weight, out1, ld1, nullptr, weight2, out2, ld2, M, N, eps, dtype, s);
}

int g_pad_chunk_rows = 1;  // raven_set_tuning("pad_chunk_rows"): 0 = the activations of a chunk keep rows n_embd elements apart
int g_pad_decode_rows = 1; // raven_set_tuning("pad_decode_rows"): 0 = decode steps of 17..32 rows read Wqkv / mlp.fc and their inputs with rows n_embd elements apart

struct BlockScratch {
    char *n1, *qkv, *q, *ya, *x1, *x2, *n3, *g, *x3, *xa, *xr;
    int ld_pad;     // n1, ya and n3 have room for rows this many elements apart (n_embd, or the next multiple of 64 for chunks)
    float* e_sums;  // up to 32 rows: fp32 sums of the adapter's embedding half, computed once for all recurrences
    void* attn_ws;
    size_t attn_ws_bytes;
    void* lin_ws;
    size_t lin_ws_bytes;
};

static size_t carve(const raven_dims* d, int M, char* base, BlockScratch* out) {
    const size_t es = raven_host::elt_size(d->dtype);
    const size_t row = raven_host::align_up((size_t)M * d->n_embd * es);
    // bf16 rows that are not whole cache lines (n_embd = 5280: 82.5 lines), 17 rows and more: the activations that the
    // products with K = n_embd read (norm_1's and norm_3's output, for chunks the attention output too) may be laid out
    // with padded rows
    const int ld_pad = (d->dtype == RAVEN_BF16 && M >= 17 && d->n_embd % 64 != 0) ? (d->n_embd + 63) / 64 * 64 : d->n_embd;
    const size_t row_pad = raven_host::align_up((size_t)M * ld_pad * es);
    size_t off = 0;
    auto take = [&](size_t bytes) {
        char* p = base ? base + off : nullptr;
        off += raven_host::align_up(bytes);
        return p;
    };
    BlockScratch s;
    s.ld_pad = ld_pad;
    s.n1 = take(row_pad);
    s.qkv = take(3 * row);
    s.q = take(row);
    s.ya = take(row_pad);
    s.x1 = take(row);
    s.x2 = take(row);
    s.n3 = take(row_pad);
    s.g = take((size_t)M * d->intermediate * es);
    s.x3 = take(row);
    s.xa = take(row);
    s.xr = take(row);
    s.e_sums = reinterpret_cast<float*>(take(M <= 32 ? (size_t)M * d->n_embd * sizeof(float) : 0));
    s.attn_ws_bytes = raven_decode_attention_workspace_bytes(M, d->n_heads, d->head_dim);
    s.attn_ws = s.attn_ws_bytes ? take(s.attn_ws_bytes) : nullptr;
    const int widest = 3 * d->n_embd > 2 * d->intermediate ? 3 * d->n_embd : 2 * d->intermediate;
    s.lin_ws_bytes = M > 1 ? raven_linear_workspace_bytes(M, widest) : 0;
    s.lin_ws = s.lin_ws_bytes ? take(s.lin_ws_bytes) : nullptr;
    if (out) *out = s;
    return off;
}

static int check_dims(const char* who, const raven_dims* d) {
    RAVEN_REQUIRE(d != nullptr, "%s: null dims", who);
    RAVEN_REQUIRE(d->dtype == RAVEN_F32 || d->dtype == RAVEN_BF16, "%s: unknown dtype %d", who, d->dtype);
    RAVEN_REQUIRE(d->n_embd > 0 && d->n_heads > 0 && d->head_dim > 0 && d->intermediate > 0, "%s: non-positive dimension", who);
    RAVEN_REQUIRE(d->n_embd == d->n_heads * d->head_dim, "%s: n_embd %d != n_heads %d * head_dim %d", who, d->n_embd, d->n_heads, d->head_dim);
    return 0;
}

static int check_block_weights(const char* who, const raven_block_weights* w) {
    RAVEN_REQUIRE(w && w->norm_1 && w->norm_2 && w->norm_3 && w->norm_4 && w->wqkv && w->proj && w->fc && w->mlp_proj,
                  "%s: null block weight", who);
    return 0;
}

// the one-row kernel keeps a quarter of K per wave in registers: 9 chunks of 16 bytes per lane at most
static bool one_row_fits(const raven_dims* d) {
    const int elts = 16 / (int)raven_host::elt_size(d->dtype);
    const int longest = d->intermediate > 2 * d->n_embd ? d->intermediate : 2 * d->n_embd;
    return ((longest / elts + 3) / 4 + 1 + 63) / 64 <= 9;
}

// The padded row length that the decode steps of a call use for norm_1's / norm_3's output and for Wqkv / mlp.fc (see
// run_block), or 0: 17..32 bf16 rows, an n_embd that is not a multiple of 64, and line-aligned copies registered for both
// matrices of every block.
static int decode_row_pitch(const raven_dims* d, const BlockScratch& s, const raven_block_weights* blocks, int n_blocks, int M, int S,
                            bool paged) {
    const int h = d->n_embd;
    if (!g_pad_decode_rows || (S != 1 && !paged) || d->dtype != RAVEN_BF16 || M < 17 || M > 32 || s.ld_pad == h) return 0;
    for (int j = 0; j < n_blocks; ++j) {
        int l1 = 0, l2 = 0;
        if (!packed_weight_of(blocks[j].wqkv, 3 * h, h, &l1) || !packed_weight_of(blocks[j].fc, 2 * d->intermediate, h, &l2) ||
            l1 != s.ld_pad || l2 != s.ld_pad) return 0;
    }
    return s.ld_pad;
}

// Several rows.  n1_ready: scratch.n1 already holds norm_1(x_in).  tail_w / tail_out: a second norm
// applied to the block output (next block's norm_1, or ln_f); y_out may be null when only the tail
// result is wanted.
static int run_block(const raven_dims* d, const raven_block_weights* w, const BlockScratch& s, bool n1_ready,
                     const void* x_in, void* y_out, const void* tail_w, void* tail_out, const float* freqs,
                     const raven_kv_cache* cache, int slot, int B, int S, int pos0, const int32_t* pos_dev, void* stream,
                     const raven_paged_kv* paged = nullptr, int layer = 0, int ld_decode = 0) {
    const int M = B * S, h = d->n_embd, I = d->intermediate, dt = d->dtype;
    hipStream_t hs = static_cast<hipStream_t>(stream);
    int rc;
    // chunks of 16 or more rows per sequence: 64 or 128 query rows of a head per workgroup on the matrix cores; a few
    // rows per sequence (or a partially filled cache, which only that kernel looks up): one row at a time
    const bool chunk = !paged && S > 1;
    const bool mfma = chunk && dt == RAVEN_BF16 && S >= 16 && (d->head_dim == 64 || d->head_dim == 96 || d->head_dim == 128) &&
                      (cache->steps_present == nullptr || cache->lookup_mode == RAVEN_LOOKUP_NONE);
    // Rows of n_embd bf16 values that are not whole cache lines (5280: 82.5 lines): norm_1's and norm_3's output and the
    // attention output, which the tiled GEMM reads as its token rows, are laid out with rows padded to whole lines (the pad
    // is never read: the products' K stays n_embd).  Every block of a call decides this the same way.
    const bool pad = g_pad_chunk_rows && mfma && s.ld_pad != h && M >= g_tiled_min_rows && tiled_gemm_fits(M, 3 * h, h, 0, dt) &&
                     tiled_gemm_fits(M, h, h, 0, dt) && tiled_gemm_fits(M, I, h, 0, dt);
    // Decode steps of 17..32 rows: the MFMA kernels of Wqkv and mlp.fc stream 5 % faster over operands with rows of whole
    // lines (fc 67.9 -> 64.5 us, Wqkv 33.1 -> 31.6 at 32 rows; no gain at 8).  Where the caller has registered line-aligned
    // copies of both matrices, the two products run over the padded length: the copies' pad columns are zeros, and so are
    // the pad columns the norm launches write behind norm_1's and norm_3's output.
    // ld_decode: that padded length, decided once for all blocks of a call (decode_row_pitch), or 0.
    int ldw_qkv = 0, ldw_fc = 0;
    const void *wqkv_p = nullptr, *fc_p = nullptr;
    const bool padk = ld_decode != 0 && !chunk;
    if (padk) {
        wqkv_p = packed_weight_of(w->wqkv, 3 * h, h, &ldw_qkv);
        fc_p = packed_weight_of(w->fc, 2 * I, h, &ldw_fc);
        RAVEN_REQUIRE(wqkv_p && fc_p && ldw_qkv == ld_decode && ldw_fc == ld_decode && ld_decode == s.ld_pad, "block: the line-aligned weight copies changed during the call");
    }
    const int ld = (pad || padk) ? s.ld_pad : h;
    if (!n1_ready)
        if ((rc = rmsnorm_pitched(x_in, nullptr, w->norm_1, s.n1, ld, nullptr, nullptr, nullptr, ld, M, h, d->eps, dt, stream))) return rc;
    // a chunk of tokens on the tiled GEMM: bias, RoPE and the cache append are that product's epilogue
    int qkv_done = 0;
    if (chunk)
        if ((rc = qkv_linear_rope_append(s.n1, ld, w->wqkv, w->qk_bias, freqs, s.q, cache, slot, B, S, pos0, pos_dev, d->n_heads, d->head_dim,
                                         dt, hs, &qkv_done))) return rc;
    if (!qkv_done) {
        if (pad) rc = tiled_gemm_pitched(s.n1, ld, w->wqkv, nullptr, s.qkv, M, 3 * h, h, 0, hs);
        else if (padk) rc = raven_linear(s.n1, nullptr, wqkv_p, nullptr, s.qkv, M, 3 * h, ld, 0, 0, 0, dt, s.lin_ws, s.lin_ws_bytes, stream);
        else rc = raven_linear(s.n1, nullptr, w->wqkv, nullptr, s.qkv, M, 3 * h, h, 0, 0, 0, dt, s.lin_ws, s.lin_ws_bytes, stream);
        if (rc) return rc;
    }
    if (paged) {   // decode over block-paged caches, every sequence at its own position
        if ((rc = raven_paged_qkv_attention_decode(s.qkv, w->qk_bias, freqs, s.ya, paged->k_caches[layer], paged->v_caches[layer],
                                                   paged->block_table, paged->seq_lens, B, paged->max_blocks, paged->block_size,
                                                   paged->kv_layout, paged->max_seq_len, d->n_heads, d->head_dim, dt, s.attn_ws, s.attn_ws_bytes, stream))) return rc;
    } else if (S == 1) {  // decode: bias, RoPE, cache append and attention in one launch
        if ((rc = raven_qkv_attention_decode(s.qkv, w->qk_bias, freqs, s.ya, cache, slot, B, pos0, pos_dev, d->n_heads,
                                             d->head_dim, dt, s.attn_ws, s.attn_ws_bytes, stream))) return rc;
    } else {       // a chunk of S tokens: every row's keys must be in the cache before any row attends
        if (!qkv_done)
            if ((rc = raven_qkv_bias_rope_cache_append(s.qkv, w->qk_bias, freqs, s.q, cache, slot, B, S, pos0, pos_dev, d->n_heads,
                                                       d->head_dim, dt, stream))) return rc;
        if (mfma) rc = prefill_attention_pitched(s.q, s.ya, ld, cache, slot, B, S, pos0, pos_dev, d->n_heads, d->head_dim, dt, stream);
        else rc = raven_decode_attention(s.q, s.ya, cache, slot, B, S, pos0, pos_dev, d->n_heads, d->head_dim, dt, s.attn_ws, s.attn_ws_bytes, stream);
        if (rc) return rc;
    }
    if (pad) {
        if ((rc = tiled_gemm_pitched(s.ya, ld, w->proj, x_in, s.x1, M, h, h, 0, hs))) return rc;
        if ((rc = rmsnorm_pitched(s.x1, nullptr, w->norm_2, s.x2, h, nullptr, w->norm_3, s.n3, ld, M, h, d->eps, dt, stream))) return rc;
        if ((rc = tiled_gemm_pitched(s.n3, ld, w->fc, nullptr, s.g, M, I, h, 1, hs))) return rc;
    } else {
        if ((rc = linear_then_norm(s.ya, w->proj, x_in, s.x1, w->norm_2, s.x2, w->norm_3, s.n3, M, h, h, d->eps, dt, s.lin_ws, s.lin_ws_bytes, hs, ld))) return rc;
        if (padk) rc = raven_linear(s.n3, nullptr, fc_p, nullptr, s.g, M, I, ld, 0, 1, 0, dt, s.lin_ws, s.lin_ws_bytes, stream);
        else rc = raven_linear(s.n3, nullptr, w->fc, nullptr, s.g, M, I, h, 0, 1, 0, dt, s.lin_ws, s.lin_ws_bytes, stream);
        if (rc) return rc;
    }
    // the tail norm's output is the next block's norm_1 input when it goes to scratch.n1: rows as that block will read them
    const int tail_ld = tail_out == static_cast<void*>(s.n1) ? ld : h;
    return linear_then_norm(s.g, w->mlp_proj, s.x2, s.x3, w->norm_4, y_out, tail_w, tail_out, M, h, I, d->eps, dt, s.lin_ws, s.lin_ws_bytes, hs, tail_ld);
}

// One row.  x_raw is the block input before `pre_norm` (the previous block's norm_4, or null when x_raw is
// the input itself).  Leaves the block output BEFORE its norm_4 in scratch.x3.
static int run_block_one_row(const raven_dims* d, const raven_block_weights* w, const BlockScratch& s, const void* x_raw,
                             const void* pre_norm, const float* freqs, const raven_kv_cache* cache, int slot, int pos0,
                             const int32_t* pos_dev, void* stream, const raven_paged_kv* paged = nullptr, int layer = 0) {
    const int h = d->n_embd, I = d->intermediate, dt = d->dtype;
    const float eps = d->eps;
    int rc;
    const void* x_res = x_raw;  // the residual the attention output is added to (RMM:534)
    if (pre_norm) {
        if ((rc = raven_gemv_fused(x_raw, nullptr, pre_norm, w->norm_1, s.xr, w->wqkv, nullptr, s.qkv, 3 * h, h, 0, eps, 0, 0, dt, stream))) return rc;
        x_res = s.xr;
    } else {
        if ((rc = raven_gemv_fused(x_raw, nullptr, w->norm_1, nullptr, nullptr, w->wqkv, nullptr, s.qkv, 3 * h, h, 0, eps, 0, 0, dt, stream))) return rc;
    }
    if (paged)
        rc = raven_paged_qkv_attention_decode(s.qkv, w->qk_bias, freqs, s.ya, paged->k_caches[layer], paged->v_caches[layer],
                                              paged->block_table, paged->seq_lens, 1, paged->max_blocks, paged->block_size,
                                              paged->kv_layout, paged->max_seq_len, d->n_heads, d->head_dim, dt, s.attn_ws, s.attn_ws_bytes, stream);
    else
        rc = raven_qkv_attention_decode(s.qkv, w->qk_bias, freqs, s.ya, cache, slot, 1, pos0, pos_dev, d->n_heads, d->head_dim, dt,
                                        s.attn_ws, s.attn_ws_bytes, stream);
    if (rc) return rc;
    if ((rc = raven_gemv_fused(s.ya, nullptr, nullptr, nullptr, nullptr, w->proj, x_res, s.x1, h, h, 0, eps, 0, 0, dt, stream))) return rc;
    if ((rc = raven_gemv_fused(s.x1, nullptr, w->norm_2, w->norm_3, s.x2, w->fc, nullptr, s.g, I, h, 0, eps, 1, 0, dt, stream))) return rc;
    return raven_gemv_fused(s.g, nullptr, nullptr, nullptr, nullptr, w->mlp_proj, s.x2, s.x3, h, I, 0, eps, 0, 0, dt, stream);
}

// closing norm_4 (+ ln_f) of the one-row schedule
static int close_one_row(const raven_dims* d, const BlockScratch& s, const void* norm_4, const void* ln_f, void* out, void* stream) {
    if (ln_f) return raven_rmsnorm_residual(s.x3, nullptr, norm_4, nullptr, nullptr, ln_f, out, 1, d->n_embd, d->eps, d->dtype, stream);
    return raven_rmsnorm_residual(s.x3, nullptr, norm_4, out, nullptr, nullptr, nullptr, 1, d->n_embd, d->eps, d->dtype, stream);
}

}  // namespace raven

extern "C" size_t raven_block_workspace_bytes(const raven_dims* dims, int32_t M) {
    if (!dims || M <= 0) return 0;
    return raven::carve(dims, M, nullptr, nullptr);
}

extern "C" int raven_sandwich_block(const raven_dims* dims, const raven_block_weights* w, const void* ln_f, const void* x_in,
                                    void* x_out, const float* freqs, const raven_kv_cache* cache, int32_t slot, int32_t B,
                                    int32_t S, int32_t pos0, const int32_t* pos_dev, void* workspace, size_t workspace_bytes,
                                    void* stream) {
    using namespace raven;
    if (int rc = check_dims("sandwich_block", dims)) return rc;
    if (int rc = check_block_weights("sandwich_block", w)) return rc;
    RAVEN_REQUIRE(x_in && x_out && freqs, "sandwich_block: null pointer");
    RAVEN_REQUIRE(B > 0 && S > 0, "sandwich_block: bad B=%d S=%d", B, S);
    const size_t need = carve(dims, B * S, nullptr, nullptr);
    RAVEN_REQUIRE(workspace && workspace_bytes >= need, "sandwich_block: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    RAVEN_REQUIRE(((uintptr_t)workspace & 255) == 0, "sandwich_block: workspace must be 256-byte aligned");
    BlockScratch s;
    carve(dims, B * S, static_cast<char*>(workspace), &s);
    if (B * S == 1 && one_row_fits(dims)) {
        if (int rc = run_block_one_row(dims, w, s, x_in, nullptr, freqs, cache, slot, pos0, pos_dev, stream)) return rc;
        return close_one_row(dims, s, w->norm_4, ln_f, x_out, stream);
    }
    const int ld_decode = decode_row_pitch(dims, s, w, 1, B * S, S, false);
    if (ln_f) return run_block(dims, w, s, false, x_in, nullptr, ln_f, x_out, freqs, cache, slot, B, S, pos0, pos_dev, stream, nullptr, 0, ld_decode);
    return run_block(dims, w, s, false, x_in, x_out, nullptr, nullptr, freqs, cache, slot, B, S, pos0, pos_dev, stream, nullptr, 0, ld_decode);
}

namespace raven {

// n_iterations x ([adapter product] + n_blocks blocks), the closing norm(s) at the end.  The K/V of block j live either
// in slot slots[it * n_blocks + j] of a contiguous cache (all sequences at position pos0 / *pos_dev) or, with `paged`,
// in the j-th block-paged cache (every sequence at its own position, the same cache in every iteration).
static int iterations_impl(const char* who, const raven_dims* dims, const void* adapter_w, const raven_block_weights* blocks,
                           int32_t n_blocks, const void* ln_f, const void* state_in, const void* embeds, void* state_out,
                           const float* freqs, const raven_kv_cache* cache, const int32_t* slots, const raven_paged_kv* paged,
                           int32_t n_iterations, int32_t B, int32_t S, int32_t pos0, const int32_t* pos_dev, void* workspace,
                           size_t workspace_bytes, void* stream) {
    if (int rc = check_dims(who, dims)) return rc;
    RAVEN_REQUIRE(state_in && state_out && freqs && (slots || paged), "%s: null pointer", who);
    RAVEN_REQUIRE((adapter_w == nullptr) == (embeds == nullptr), "%s: the adapter weight and its second input come together", who);
    RAVEN_REQUIRE(n_blocks >= 1 && blocks, "%s: needs at least one block", who);
    RAVEN_REQUIRE(n_iterations >= 1, "%s: needs at least one iteration (got %d)", who, n_iterations);
    RAVEN_REQUIRE(adapter_w || n_iterations == 1, "%s: several iterations need the adapter", who);
    RAVEN_REQUIRE(B > 0 && S > 0, "%s: bad B=%d S=%d", who, B, S);
    for (int j = 0; j < n_blocks; ++j)
        if (int rc = check_block_weights(who, &blocks[j])) return rc;
    const int M = B * S, h = dims->n_embd;
    const size_t need = carve(dims, M, nullptr, nullptr);
    RAVEN_REQUIRE(workspace && workspace_bytes >= need, "%s: workspace of %zu bytes needed, %zu given", who, need, workspace_bytes);
    RAVEN_REQUIRE(((uintptr_t)workspace & 255) == 0, "%s: workspace must be 256-byte aligned", who);
    BlockScratch s;
    carve(dims, M, static_cast<char*>(workspace), &s);
    const raven_block_weights& last_blk = blocks[n_blocks - 1];
    hipStream_t hs = static_cast<hipStream_t>(stream);

    int rc;
    if (M == 1 && one_row_fits(dims)) {
        // One row: between two iterations the last block's closing norm_4 is the prologue of the next adapter product
        // (no launch of its own); only the last iteration closes with a norm launch (norm_4, then ln_f if asked for).
        // The embedding half of the adapter product is the same in every recurrence: with two or more of them its fp32
        // sums are formed once, and each recurrence streams the state half of the weight only.
        const bool split = n_iterations >= 2;
        const size_t es = raven_host::elt_size(dims->dtype);
        if (split)
            if ((rc = gemv1_column_block(embeds, nullptr, static_cast<const char*>(adapter_w) + (size_t)h * es, 2 * h, nullptr, s.e_sums,
                                         1, h, h, dims->eps, dims->dtype, hs))) return rc;
        for (int it = 0; it < n_iterations; ++it) {
            const int32_t* sl = slots ? slots + (size_t)it * n_blocks : nullptr;
            const void* x_in = it == 0 ? state_in : (const void*)s.x3;
            const void* pre_norm = it == 0 ? nullptr : last_blk.norm_4;
            if (adapter_w) {
                if (split)
                    rc = gemv1_column_block(x_in, pre_norm, adapter_w, 2 * h, s.e_sums, s.xa, 0, h, h, dims->eps, dims->dtype, hs);
                else
                    rc = raven_gemv_fused(x_in, embeds, pre_norm, nullptr, nullptr, adapter_w, nullptr, s.xa, h, h, h, dims->eps, 0, 0,
                                          dims->dtype, stream);
                if (rc) return rc;
            }
            for (int j = 0; j < n_blocks; ++j) {
                const void* x_raw = j == 0 ? (adapter_w ? (const void*)s.xa : state_in) : (const void*)s.x3;
                const void* pre = j == 0 ? nullptr : blocks[j - 1].norm_4;
                if ((rc = run_block_one_row(dims, &blocks[j], s, x_raw, pre, freqs, cache, sl ? sl[j] : 0, pos0, pos_dev, stream, paged, j)))
                    return rc;
            }
        }
        return close_one_row(dims, s, last_blk.norm_4, ln_f, state_out, stream);
    }
    // 2..32 rows in bf16: the adapter is split by columns as for one row (embedding half summed once, in fp32)
    const bool split = adapter_w && n_iterations >= 2 && dims->dtype == RAVEN_BF16 && M >= 2 && M <= 32 && h % 32 == 0 && h >= 256 &&
                       s.lin_ws;
    if (split)
        if ((rc = linear_column_block(embeds, static_cast<const char*>(adapter_w) + (size_t)h * 2, 2 * h, nullptr, s.e_sums, 1, M, h, h,
                                      s.lin_ws, s.lin_ws_bytes, hs))) return rc;
    const int ld_decode = decode_row_pitch(dims, s, blocks, n_blocks, M, S, paged != nullptr);
    for (int it = 0; it < n_iterations; ++it) {
        const int32_t* sl = slots ? slots + (size_t)it * n_blocks : nullptr;
        const bool last_it = it == n_iterations - 1;
        // the adapter product consumes the state before the last block of this iteration overwrites state_out
        const void* st = it == 0 ? state_in : state_out;
        bool n1_ready = false;  // scratch.n1 holds norm_1 of the first block's input
        if (adapter_w) {
            // where the product is K-split, the launch that adds its slices also applies the first block's norm_1
            int ks = 0;
            if (split) rc = linear_leave_sums(st, nullptr, adapter_w, 2 * h, s.e_sums, nullptr, s.xa, M, h, h, 0, dims->dtype, s.lin_ws, s.lin_ws_bytes, hs, &ks);
            else rc = linear_leave_sums(st, embeds, adapter_w, 0, nullptr, nullptr, s.xa, M, h, h, h, dims->dtype, s.lin_ws, s.lin_ws_bytes, hs, &ks);
            if (rc) return rc;
            if (ks) {
                if ((rc = splitk_sums_then_norm(static_cast<const float*>(s.lin_ws), ks, split ? s.e_sums : nullptr, nullptr, s.xa, blocks[0].norm_1,
                                                s.n1, nullptr, nullptr, M, h, dims->eps, hs, ld_decode, 0))) return rc;
                n1_ready = true;
            }
        }
        const void* lnw = last_it ? ln_f : nullptr;
        for (int j = 0; j < n_blocks; ++j) {
            const bool last = j == n_blocks - 1;
            const void* x_in = (j == 0 && !adapter_w) ? state_in : (const void*)s.xa;
            void* y_out = last ? (lnw ? nullptr : state_out) : s.xa;
            const void* tail_w = last ? lnw : blocks[j + 1].norm_1;
            void* tail_out = last ? (lnw ? state_out : nullptr) : s.n1;
            if ((rc = run_block(dims, &blocks[j], s, j > 0 || n1_ready, x_in, y_out, tail_w, tail_out, freqs, cache, sl ? sl[j] : 0, B, S, pos0,
                                pos_dev, stream, paged, j, ld_decode))) return rc;
        }
    }
    return 0;
}

}  // namespace raven

extern "C" int raven_core_iterations(const raven_dims* dims, const void* adapter_w, const raven_block_weights* blocks,
                                     int32_t n_blocks, const void* ln_f, const void* state_in, const void* embeds,
                                     void* state_out, const float* freqs, const raven_kv_cache* cache, const int32_t* slots,
                                     int32_t n_iterations, int32_t B, int32_t S, int32_t pos0, const int32_t* pos_dev,
                                     void* workspace, size_t workspace_bytes, void* stream) {
    RAVEN_REQUIRE(adapter_w && embeds && slots, "core_iterations: null pointer");
    return raven::iterations_impl("core_iterations", dims, adapter_w, blocks, n_blocks, ln_f, state_in, embeds, state_out, freqs, cache,
                                  slots, nullptr, n_iterations, B, S, pos0, pos_dev, workspace, workspace_bytes, stream);
}

extern "C" int raven_paged_decode_blocks(const raven_dims* dims, const void* adapter_w, const raven_block_weights* blocks,
                                         int32_t n_blocks, const void* ln_f, const void* x_in, const void* embeds, void* x_out,
                                         const float* freqs, const raven_paged_kv* kv, int32_t n_iterations, int32_t B,
                                         void* workspace, size_t workspace_bytes, void* stream) {
    RAVEN_REQUIRE(kv && kv->k_caches && kv->v_caches && kv->block_table && kv->seq_lens, "paged_decode_blocks: null cache description");
    RAVEN_REQUIRE(n_blocks >= 1 && n_blocks <= 64, "paged_decode_blocks: needs 1..64 blocks (got %d)", n_blocks);
    for (int j = 0; j < n_blocks; ++j)
        RAVEN_REQUIRE(kv->k_caches[j] && kv->v_caches[j], "paged_decode_blocks: null cache for block %d", j);
    return raven::iterations_impl("paged_decode_blocks", dims, adapter_w, blocks, n_blocks, ln_f, x_in, embeds, x_out, freqs, nullptr,
                                  nullptr, kv, n_iterations, B, 1, 0, nullptr, workspace, workspace_bytes, stream);
}

extern "C" int raven_core_iteration(const raven_dims* dims, const void* adapter_w, const raven_block_weights* blocks,
                                    int32_t n_blocks, const void* ln_f, const void* state_in, const void* embeds,
                                    void* state_out, const float* freqs, const raven_kv_cache* cache, int32_t first_slot,
                                    int32_t B, int32_t S, int32_t pos0, const int32_t* pos_dev, void* workspace,
                                    size_t workspace_bytes, void* stream) {
    RAVEN_REQUIRE(n_blocks >= 1 && n_blocks <= 64, "core_iteration: needs 1..64 blocks (got %d)", n_blocks);
    int32_t slots[64];
    for (int j = 0; j < n_blocks; ++j) slots[j] = first_slot + j;
    return raven_core_iterations(dims, adapter_w, blocks, n_blocks, ln_f, state_in, embeds, state_out, freqs, cache, slots, 1, B, S,
                                 pos0, pos_dev, workspace, workspace_bytes, stream);
}

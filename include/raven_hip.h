/*
 * raven_hip.h -- C ABI of libraven_hip.so: hand-written gfx950 (MI355X) kernels for the
 * recurrent-core decode path of the Huginn/Raven model.
 *
 * The reference (seal-rg/recurrent-pretraining) is pure Python and has no FFI; each entry point
 * below names the lines of recpre/raven_modeling_minimal.py ("RMM") whose arithmetic it replaces.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless the name ends in _host; buffers are caller-owned;
 *     nothing here allocates, frees or synchronises; work is enqueued on `stream` (a hipStream_t).
 *   - tensors are dense row-major. "T" is the model dtype: RAVEN_F32 or RAVEN_BF16.
 *   - token rows: activations are [M, h] with M = B*S rows; row m belongs to sequence b = m / S and
 *     has position pos0 + (m % S).  Decode is S = 1; a prefill chunk is S > 1.
 *   - `pos_dev` (nullable): when given, kernels read pos0 from this device int32 instead of the
 *     by-value argument, so a captured HIP graph can be replayed as the sequence grows; the by-value
 *     `pos0` then only sizes grids and must be >= the largest value *pos_dev will take.
 *   - return value: 0 ok; < 0 invalid argument (see raven_last_error()); > 0 a hipError_t.
 *   - workspaces must be 256-byte aligned; calls that share a workspace must be ordered on one stream.
 */
#ifndef RAVEN_HIP_H
#define RAVEN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { RAVEN_F32 = 0, RAVEN_BF16 = 1 };

/* Shape of one SandwichBlock (recpre/raven_config_minimal.py:12-91). */
typedef struct raven_dims {
    int32_t n_embd;       /* h                                   */
    int32_t n_heads;      /* nh, with h == nh * head_dim          */
    int32_t head_dim;     /* hd, even, hd * sizeof(T) <= 256      */
    int32_t intermediate; /* I: fc is [2I, h], mlp.proj is [h, I] */
    float   eps;          /* RMSNorm epsilon                      */
    int32_t dtype;        /* RAVEN_F32 | RAVEN_BF16               */
} raven_dims;

/* Weights of one SandwichBlock, state-dict names in comments (RMM:515-523). */
typedef struct raven_block_weights {
    const void* norm_1;   /* [h]      norm_1.weight          */
    const void* norm_2;   /* [h]      norm_2.weight          */
    const void* norm_3;   /* [h]      norm_3.weight          */
    const void* norm_4;   /* [h]      norm_4.weight          */
    const void* wqkv;     /* [3h, h]  attn.Wqkv.weight       */
    const void* qk_bias;  /* [2,nh,hd] attn.qk_bias or NULL  */
    const void* proj;     /* [h, h]   attn.proj.weight       */
    const void* fc;       /* [2I, h]  mlp.fc.weight          */
    const void* mlp_proj; /* [h, I]   mlp.proj.weight        */
} raven_block_weights;

/* Step-indexed KV cache, the HuginnStaticCache layout (RMM:344-349): K and V are
 * [n_slots, batch, nh, t_max, hd] of T.  The `slot` argument of the calls below is an index into the
 * first dimension (negative values count from the end); which step index lives in which slot is the
 * caller's business, except for the partial-fill lookups:
 *
 * Tokens computed with different numbers of recurrences leave positions that are not cached at the
 * deeper steps.  HuginnDynamicCache.update then builds K/V per position according to its lookup strategy
 * (RMM:199-253).  The attention kernels do the same in place when steps_present is given: steps_present[p]
 * = how many core steps (step index 2, 3, 4, ... in this order, slots core_slot0, core_slot0 + 1, ...) are
 * cached for position p, shared by the batch.  It is consulted for positions older than the rows of the
 * call and for slots >= core_slot0 only; NULL or RAVEN_LOOKUP_NONE = everything is cached (no lookups). */
enum { RAVEN_LOOKUP_NONE = 0,
       RAVEN_LOOKUP_SKIP = 1,         /* "skip", and "full" with gaps: leave uncached positions out (RMM:199-204, 247-254) */
       RAVEN_LOOKUP_LATEST = 2,       /* "latest-m4", "available-m4": deepest cached step <= this one of the same block (RMM:206-232) */
       RAVEN_LOOKUP_ALWAYS_LAST = 3   /* "always-last-m4": deepest cached step of the same block (RMM:233-246) */ };
typedef struct raven_kv_cache {
    void*   k;
    void*   v;
    int32_t n_slots;
    int32_t batch;
    int32_t t_max;
    int32_t lookup_mode;           /* RAVEN_LOOKUP_* */
    const int32_t* steps_present;  /* device, [t_max], or NULL */
    int32_t core_slot0;            /* slot of step index 2 */
} raven_kv_cache;

/* Library identity: version, the gfx arch the kernels were compiled for, last error text. */
int         raven_version(void);
const char* raven_arch(void);
const char* raven_last_error(void);

/* Launch-shape overrides for experiments (grid sizing and load hints of the skinny-GEMM kernels);
 * results never depend on them.  Keys: gemv_units_per_wave, gemv_interleave, gemv_nontemporal,
 * gemv_wgs_per_cu, gemv1_pairs_norm (weight-row pairs per workgroup of the one-row kernel with a norm prologue; 0 = by shape,
 * about ten workgroups per compute unit), gemv1_pairs_plain, gemm_four_tiles (0 / 1 / 2 = never / by rule / always use
 * the four-tile MFMA variant), attn_split_target / attn_big_grid (workgroups a split decode-attention launch aims
 * for / from which its 2-positions-per-row variant is used), attn_nosplit_pairs ((head, row) pairs from which a launch over the contiguous cache is
 * never split, at most 1024; the paged entry point stops splitting at 1024), attn_nosplit_len (cache positions up to
 * which two rows and more over the contiguous cache are not split either; 0 = off), rope_tiled_rows (chunk length from which raven_qkv_bias_rope_cache_append works on tiles
 * of one head and 64 positions), attn_wide (longest cache for which few (head, row) pairs get
 * one 1024-thread workgroup each instead of a split launch; 0 = never), gemm_mfma_min_rows (fewest rows the MFMA
 * kernels take; fewer go to the vector kernels), linear_min_rows (most rows raven_linear still hands to the kernels
 * without a workspace), linear_ks (K slices of the split-K kernel behind raven_linear;
 * non-zero also makes raven_linear use that kernel for every shape it accepts), gemm_tiled_min_rows (fewest rows, 33 or
 * more, that the tiled MFMA kernel takes), gemm_tiled_variant (0 = tile size by shape, 1 = 256 x 256, 2 = 128 x 128 and
 * no tile-count rule, 3 = 256 x 256 by the eight-wave kernel instead of the four-wave ring kernel), gemm_tiled_split_tail
 * (1 = the tile columns of a last round that fills at most half the chip go to
 * 128 x 128 tiles, 0 = never), prefill_waves (waves per workgroup of the chunk attention at head_dim 96: 0 = by shape, 4 or 6),
 * attn_prefetch (1 = an unsplit decode-attention launch of fewer than 256 or of 1024 and more (head, row) pairs requests a
 * tile before it uses the one before, 2 = every launch does, 0 = never),
 * gemm_ragged (1 = a 5..32-row product whose output columns divide into about two workgroups per compute unit runs as one
 * round of workgroups with a partly empty last tile, 0 = whole tiles only), norm_early (1 / 0 = the RMSNorm kernel requests
 * its weights before / after the row reduction, -1 = by row count), fuse_sums_norm (1 = a K-split product that feeds a
 * norm leaves its slices to that norm's launch, which adds them in the same order; 0 = a launch of its own adds them),
 * fuse_qkv_rope (1 = inside raven_sandwich_block / raven_core_iteration(s) a chunk's q | k | v product on the tiled GEMM
 * applies bias, RoPE and the cache append in its epilogue; 0 = the product is stored and raven_qkv_bias_rope_cache_append's
 * kernel follows; same bits either way), pad_chunk_rows (1 = inside the composed entry points the activations that the tiled
 * GEMMs of a bf16 chunk read -- norm_1's and norm_3's output, the attention output -- are laid out in the workspace with rows
 * padded to a multiple of 64 elements when n_embd is not one; 0 = rows n_embd elements apart; same bits either way),
 * pad_decode_rows (1 = decode steps of 17..32 bf16 rows inside the composed entry points run Wqkv and mlp.fc over the padded
 * length when line-aligned copies of both matrices of every block are registered -- zeros in the pads of the copies and of
 * norm_1's / norm_3's output, another summation order than over the matrices themselves; 0 = never).
 * Not needed in normal use: the defaults are the tuned values.  The knobs are process-global
 * state read at every launch: changing them while another thread or stream is inside a call of this library is a race. */
int raven_set_tuning(const char* key, int32_t value);

/* RMSNorm with the reference's two roundings, optionally preceded by a residual add and followed by
 * a second norm.  RMM:137-142 (norm), RMM:534-535 (the adds feeding norm_2 / norm_4).
 *   s  = residual ? T(x + residual) : x          -> stored to sum_out when non-NULL
 *   y  = T(s32 * rsqrt(mean(s32^2) + eps)) * weight          (y may be NULL when only y2 is wanted)
 *   y2 = T(y32 * rsqrt(mean(y32^2) + eps)) * weight2         (only when weight2 and y2 are given)
 * x, residual, y, sum_out, y2: [rows, dim] of T; weights [dim] of T. dim * sizeof(T) % 16 == 0. */
int raven_rmsnorm_residual(const void* x, const void* residual, const void* weight, void* y,
                           void* sum_out, const void* weight2, void* y2,
                           int64_t rows, int32_t dim, float eps, int32_t dtype, void* stream);

/* Y[M,N] = X[M,K] W[N,K]^T for skinny M (any M >= 1; the weight matrix is streamed once per 32
 * (bf16) or 8 (f32) rows).  Replaces the nn.Linear calls of attn.proj (RMM:493), mlp.proj (RMM:509)
 * and lm_head (RMM:711).  fp32 accumulate, result rounded to T; then, if residual != NULL,
 * Y = T(Y + residual) (RMM:534-535); if out_f32 != 0 the rounded result is stored as float
 * (the `.float()` of RMM:711).  K * sizeof(T) % 16 == 0. */
int raven_gemm(const void* x, const void* w, const void* residual, void* y,
               int32_t M, int32_t N, int32_t K, int32_t dtype, int32_t out_f32, void* stream);

/* Adapter Linear(2h -> h) over concat(state, embeds) without materialising the concat
 * (RMM:776: torch.cat([x, input_embeds], -1) then nn.Linear).  w is [N, K0 + K1]; x0 [M, K0] pairs
 * with w[:, :K0] and x1 [M, K1] with w[:, K0:]. */
int raven_adapter_gemm_concat(const void* x0, const void* x1, const void* w, void* y,
                              int32_t M, int32_t N, int32_t K0, int32_t K1, int32_t dtype, void* stream);

/* GatedMLP first half with the activation in the epilogue (RMM:507-508):
 *   z = X fc^T, gate = T(z[:, :I]), up = T(z[:, I:]), out[M, I] = T(T(silu(gate)) * up). */
int raven_gemm_swiglu(const void* x, const void* fc, void* out,
                      int32_t M, int32_t I, int32_t K, int32_t dtype, void* stream);

/* The general form of the three calls above with an optional workspace:
 *     z = concat(x0, x1) W^T,  y = swiglu ? T(T(silu(T(z[:, :N]))) * T(z[:, N:])) : T(z) [+ residual] [as float]
 * With a workspace (raven_linear_workspace_bytes(M, widest output: 2N for SwiGLU)) and 5 or more bf16 rows,
 * K is split across workgroups and the X tile of a K step is shared by the workgroup's waves, which is
 * what batches of 8..32 rows need to approach HBM bandwidth; partial sums are added in a fixed order.
 * Without one (or for 1..4 rows, fp32) the call is forwarded to raven_gemm / _adapter_gemm_concat / _gemm_swiglu. */
size_t raven_linear_workspace_bytes(int32_t M, int32_t n_out_max);
int    raven_linear(const void* x0, const void* x1, const void* w, const void* residual, void* y,
                    int32_t M, int32_t N, int32_t K0, int32_t K1, int32_t swiglu, int32_t out_f32,
                    int32_t dtype, void* workspace, size_t workspace_bytes, void* stream);

/* Line-aligned copies of bf16 weight matrices for products over 33 and more token rows.  No counterpart in the reference
 * (its nn.Linear weights are [out, in] with rows K elements apart, RMM:463, 493, 507-509, and stay the layout every entry point
 * takes).  Where K * 2 bytes is not a multiple of 128 (K = 5280: every second row starts 64 bytes into a cache line) the
 * tiled MFMA kernels lose 5 to 7 % to half-line requests.  raven_register_packed_weight copies w [rows, K] (rows = out
 * features; 2 * I for a GatedMLP fc matrix) into `packed` -- caller-allocated, raven_packed_weight_bytes(rows, K) bytes,
 * 128-byte aligned, rows padded with zeros to a multiple of 64 elements -- on `stream`, and from then on every product
 * whose weight pointer is `w`, with this K and these rows, that runs on the tiled kernels reads the copy: same values in
 * the same order, same bits.  The caller registers again after changing w, and calls raven_unregister_packed_weight(w)
 * before it frees either buffer.  Products of fewer rows read w itself, with one exception: decode steps of 17..32 rows
 * inside raven_sandwich_block / raven_core_iteration(s) / raven_paged_decode_blocks take Wqkv and mlp.fc from the copies
 * when both are registered for every block of the call (5 % faster there; see pad_decode_rows under raven_set_tuning). */
int64_t raven_packed_weight_bytes(int32_t rows, int32_t K);
int     raven_register_packed_weight(const void* w, int32_t rows, int32_t K, void* packed, void* stream);
int     raven_unregister_packed_weight(const void* w);

/* Statistics behind the per-iteration exit criteria of adaptive compute (RMM:2128-2260), one value per row.
 * raven_exit_logit_stats on logits [rows, V] float:
 *   RAVEN_EXIT_ENTROPY  out = -sum p log(p + 1e-10), p = softmax(logits)                       (RMM:2142-2144)
 *   RAVEN_EXIT_KL       lp = log_softmax(logits); out = sum exp(prev) (prev - lp); prev <- lp  (RMM:2182-2186)
 *   RAVEN_EXIT_MINP_KL  the same with p[p < 0.1 max p] = 1/V, renormalised, before the log     (RMM:2200-2216)
 * prev_log_probs [rows, V] float is read and overwritten by the KL kinds (NULL for the entropy).
 * raven_exit_latent_stats on latents, prev [rows, h] of T: rel_change = |latents - prev| / |latents| (RMM:2162),
 * cosine = <latents, prev> / |latents| / |prev| (RMM:2256), each [rows] of T, either may be NULL. */
enum { RAVEN_EXIT_ENTROPY = 0, RAVEN_EXIT_KL = 1, RAVEN_EXIT_MINP_KL = 2 };
int raven_exit_logit_stats(const float* logits, float* prev_log_probs, float* out, int32_t rows, int32_t V,
                           int32_t kind, void* stream);
int raven_exit_latent_stats(const void* latents, const void* prev, void* rel_change, void* cosine,
                            int32_t rows, int32_t h, int32_t dtype, void* stream);

/* Paged KV cache, the layout the attention layer of the reference's vLLM plugin is given (vllm/raven_vllm.py:174-201
 * hands rotated q, k and v to vLLM's Attention, which owns a block-paged cache): k_cache and v_cache are
 * [num_blocks, block_size, n_heads, head_dim] of T (kv_layout RAVEN_PAGED_NHD) or [num_blocks, n_heads, block_size,
 * head_dim] (RAVEN_PAGED_HND: a head's positions of a block are contiguous, which the attention kernel reads faster);
 * position p of sequence b lives in block block_table[b * max_blocks + p / block_size] at offset p % block_size.
 * raven_paged_kv_append: rows k, v [T, n_heads * head_dim] (k already biased and rotated) go to the flat slots
 *   slot_mapping[t] = block * block_size + offset (negative: skipped).
 * raven_paged_decode_attention: one query row per sequence, q / y [B, n_heads * head_dim]; sequence b attends to its
 *   first seq_lens[b] positions (its own new token included; 0 gives zeros).  max_seq_len >= every seq_lens[b] sizes the
 *   launch.  workspace as for raven_decode_attention (raven_decode_attention_workspace_bytes(B, ...)).
 * raven_paged_qkv_attention_decode: the whole decode step of the plugin's attention layer in one launch
 *   (vllm/raven_vllm.py:186-201: split, q/k bias, RoPE, cache write, attention): qkv [B, 3 * n_heads * head_dim] is the
 *   fused projection's output, qk_bias [2, n_heads, head_dim] or NULL, freqs the (cos, sin) table; sequence b's new
 *   token sits at position seq_lens[b] - 1: its rotated k and its v are written to that position's page and the row
 *   attends to positions 0..seq_lens[b] - 1 (seq_lens[b] = 0: nothing written, zeros returned).
 * raven_paged_qkv_rope_append: the same layer up to the cache write for ANY rows (prompt chunks and decode rows of
 *   several sequences in one launch, vllm/raven_vllm.py:186-199): row t of qkv [T, 3 * n_heads * head_dim] gets the q/k
 *   bias and the rotation of positions[t] (a row of freqs; the caller keeps it inside the table), q goes to
 *   q_out [T, n_heads * head_dim], k and v to slot slot_mapping[t] of the pages (negative: not stored).
 * raven_paged_prefill_attention: causal attention of such rows on the matrix cores (bf16, head_dim 64 / 96 / 128), the
 *   variable-length form vLLM's backends call: sequence b owns rows q_start[b] .. q_start[b + 1] - 1 of q / y
 *   [T, n_heads * head_dim]; they are the LAST positions of its seq_lens[b] cached positions (already appended), so row
 *   r of the sequence attends to positions 0 .. seq_lens[b] - (rows of b) + r.  max_q_len >= every sequence's row count
 *   sizes the launch; a sequence with no rows, or more rows than positions, is left alone.  Same kernel as
 *   raven_prefill_attention with the key tiles gathered through the block table. */
enum { RAVEN_PAGED_NHD = 0, RAVEN_PAGED_HND = 1 };
int raven_paged_kv_append(const void* k, const void* v, void* k_cache, void* v_cache, const int64_t* slot_mapping,
                          int32_t T, int32_t n_heads, int32_t head_dim, int32_t block_size, int32_t kv_layout,
                          int32_t dtype, void* stream);
int raven_paged_decode_attention(const void* q, void* y, const void* k_cache, const void* v_cache,
                                 const int32_t* block_table, const int32_t* seq_lens, int32_t B, int32_t max_blocks,
                                 int32_t block_size, int32_t kv_layout, int32_t max_seq_len, int32_t n_heads,
                                 int32_t head_dim, int32_t dtype, void* workspace, size_t workspace_bytes, void* stream);
int raven_paged_qkv_attention_decode(const void* qkv, const void* qk_bias, const float* freqs, void* y, void* k_cache,
                                     void* v_cache, const int32_t* block_table, const int32_t* seq_lens, int32_t B,
                                     int32_t max_blocks, int32_t block_size, int32_t kv_layout, int32_t max_seq_len,
                                     int32_t n_heads, int32_t head_dim, int32_t dtype, void* workspace,
                                     size_t workspace_bytes, void* stream);

int raven_paged_qkv_rope_append(const void* qkv, const void* qk_bias, const float* freqs, const int64_t* positions,
                                const int64_t* slot_mapping, void* q_out, void* k_cache, void* v_cache, int32_t T,
                                int32_t n_heads, int32_t head_dim, int32_t block_size, int32_t kv_layout,
                                int32_t dtype, void* stream);
int raven_paged_prefill_attention(const void* q, void* y, const void* k_cache, const void* v_cache,
                                  const int32_t* block_table, const int32_t* seq_lens, const int32_t* q_start,
                                  int32_t B, int32_t max_q_len, int32_t max_blocks, int32_t block_size,
                                  int32_t kv_layout, int32_t n_heads, int32_t head_dim, int32_t dtype, void* stream);

/* A stack of SandwichBlocks over block-paged caches, one decode row per sequence (the flat layer list the plugin's
 * model runs, vllm/raven_vllm.py:365-432: every flat layer owns ONE paged cache, which the recurrences of a token
 * overwrite in turn, so older positions hold their last recurrence).  k_caches / v_caches: HOST arrays of n_blocks
 * device pointers, block j's cache in the layout kv_layout names; block_table [B, max_blocks] and
 * seq_lens [B] (new token included) in device memory, shared by all blocks.
 * adapter_w / embeds non-NULL: n_iterations x (adapter([x, embeds]) then the blocks), i.e. the recurrent core;
 * both NULL: the blocks once (prelude, coda).  ln_f non-NULL: applied to the result.  x_in, embeds, x_out [B, h].
 * workspace: raven_block_workspace_bytes(dims, B). */
typedef struct raven_paged_kv {
    void* const* k_caches;
    void* const* v_caches;
    const int32_t* block_table;
    const int32_t* seq_lens;
    int32_t max_blocks, block_size, max_seq_len;
    int32_t kv_layout; /* RAVEN_PAGED_NHD or RAVEN_PAGED_HND */
} raven_paged_kv;
int raven_paged_decode_blocks(const raven_dims* dims, const void* adapter_w, const raven_block_weights* blocks,
                              int32_t n_blocks, const void* ln_f, const void* x_in, const void* embeds, void* x_out,
                              const float* freqs, const raven_paged_kv* kv, int32_t n_iterations, int32_t B,
                              void* workspace, size_t workspace_bytes, void* stream);

/* Decode fast path for ONE token row, one launch:
 *     x  = norm_a ? T(rmsnorm(x0) * norm_a) : x0      -> stored to xa_out when non-NULL
 *     x  = norm_b ? T(rmsnorm(x)  * norm_b) : x
 *     z  = concat(x, x1) W^T                          (x1 / K1 optional: the adapter's second operand)
 *     y  = swiglu ? T(T(silu(T(z[:N]))) * T(z[N:]))   : T(z) [+ residual, in T] [stored as float]
 * i.e. the RMSNorms of RMM:525-536 folded into the nn.Linear that consumes them (norm_4 of the
 * previous block and norm_1 before Wqkv, norm_2 and norm_3 before mlp.fc), with the epilogues of
 * raven_gemm / raven_gemm_swiglu.  x0 [K0], x1 [K1], norm_a / norm_b / xa_out [K0], w [N or 2N, K0+K1],
 * residual / y [N].  xa_out must not alias x0.  (K0 + K1) * sizeof(T) <= 36 KiB. */
int raven_gemv_fused(const void* x0, const void* x1, const void* norm_a, const void* norm_b, void* xa_out,
                     const void* w, const void* residual, void* y, int32_t N, int32_t K0, int32_t K1,
                     float eps, int32_t swiglu, int32_t out_f32, int32_t dtype, void* stream);

/* Split fused qkv rows, add q/k bias, rotate q and k, append k and v to the cache slot
 * (RMM:463-479 and HuginnStaticCache.update's index_copy_, RMM:375-380).
 *   qkv [M, 3h] of T; freqs [n_pos, hd/2, 2] float (cos, sin) -- rows picked by position;
 *   q_out [M, h] of T receives the rotated queries. */
int raven_qkv_bias_rope_cache_append(const void* qkv, const void* qk_bias, const float* freqs,
                                     void* q_out, const raven_kv_cache* cache, int32_t slot,
                                     int32_t B, int32_t S, int32_t pos0, const int32_t* pos_dev,
                                     int32_t n_heads, int32_t head_dim, int32_t dtype, void* stream);

/* softmax(q K^T / sqrt(hd)) V over the cached positions of one slot, for each of the M = B*S rows
 * (RMM:481-491).  Row m attends to positions 0 .. pos0 + (m % S) inclusive: for S == 1 this is the
 * unmasked decode case, for S > 1 the lower-right-aligned causal case.  The new keys/values must
 * already be in the cache.  q [M, h]; y [M, h] in the layout y.transpose(1,2).reshape(B,S,h) has.
 * workspace (nullable, raven_decode_attention_workspace_bytes): room for partial results when few
 * (head, row) pairs make a split over positions worthwhile; without it the result is the same, slower. */
size_t raven_decode_attention_workspace_bytes(int32_t M, int32_t n_heads, int32_t head_dim);
int    raven_decode_attention(const void* q, void* y, const raven_kv_cache* cache, int32_t slot,
                              int32_t B, int32_t S, int32_t pos0, const int32_t* pos_dev,
                              int32_t n_heads, int32_t head_dim, int32_t dtype,
                              void* workspace, size_t workspace_bytes, void* stream);

/* Decode step (S == 1) of RMM:463-491: takes the fused qkv GEMM output [B, 3h], adds the q/k bias,
 * rotates q and k for position pos0, writes the new k and v rows into the cache slot and returns
 * softmax(q K^T / sqrt(hd)) V over positions 0 .. pos0 in y [B, h].  workspace as above. */
int raven_qkv_attention_decode(const void* qkv, const void* qk_bias, const float* freqs, void* y,
                               const raven_kv_cache* cache, int32_t slot, int32_t B, int32_t pos0,
                               const int32_t* pos_dev, int32_t n_heads, int32_t head_dim,
                               int32_t dtype, void* workspace, size_t workspace_bytes, void* stream);

/* raven_qkv_attention_decode for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): the same decode step with no workspace argument.  It has no counterpart in the
 * reference.  The partial results of a split launch go to an array that is part of this library's code object
 * (raven_qkv_attention_decode_static_scratch_bytes() bytes, about 17 MB, held by every GPU the library runs on until the
 * process ends); its device address is looked up on the first call on each device (make that call outside a graph
 * capture).  Same results, bit for bit, as raven_qkv_attention_decode with a workspace of
 * raven_decode_attention_workspace_bytes(B, n_heads, head_dim).  A launch whose partial results would not fit the array
 * (more than 1023 (head, row) pairs in a split launch, head_dim above 128: neither is reachable with the present
 * splitting rule) is refused with a negative status.  All calls on one GPU share the array: calls that overlap on one
 * GPU (two streams) race; every launch writes each partial result before it reads it, nothing needs clearing. */
size_t raven_qkv_attention_decode_static_scratch_bytes(void);
int    raven_qkv_attention_decode_static(const void* qkv, const void* qk_bias, const float* freqs, void* y,
                                         const raven_kv_cache* cache, int32_t slot, int32_t B, int32_t pos0,
                                         const int32_t* pos_dev, int32_t n_heads, int32_t head_dim,
                                         int32_t dtype, void* stream);

/* Causal attention for a prefill chunk on the matrix cores (bf16; head_dim 64, 96 or 128): the S > 1
 * cases of RMM:484-491.  Same contract as raven_decode_attention -- row m of sequence b attends to cached
 * positions 0 .. pos0 + (m % S), the chunk's keys/values are already in the cache -- but one workgroup
 * serves 64 or 128 query rows of a head and streams the keys once for all of them. */
int raven_prefill_attention(const void* q, void* y, const raven_kv_cache* cache, int32_t slot,
                            int32_t B, int32_t S, int32_t pos0, const int32_t* pos_dev,
                            int32_t n_heads, int32_t head_dim, int32_t dtype, void* stream);

/* SiLU-gate of a materialised fc output (RMM:507-508): out[m, j] = T(T(silu(z[m, j])) * z[m, I + j]);
 * z [M, 2I], out [M, I].  For callers that run mlp.fc as a library GEMM (large M). */
int raven_swiglu(const void* z, void* out, int32_t M, int32_t I, int32_t dtype, void* stream);

/* The state perturbation in front of a recurrence when the config's test_time_noise is set (RMM:815-833, before the
 * renormalisation, which is raven_rmsnorm_residual with the last core block's norm_4): y = T(T(x * keep) + m) with
 * m = T(noise * a), and m = T(m / d) when d != 0 -- one rounding per torch operation of the reference's expression
 * `x * (1 - c) + randn_like(x) * n [/ step]`; the caller draws `noise` and computes keep, a, d for the noise type. */
int raven_noise_mix(const void* x, const void* noise, void* y, int64_t n, float keep, float a, float d,
                    int32_t dtype, void* stream);

/* Token embedding times sqrt(h) (RMM:667-671): out[m] = T(wte[ids[m]] * scale); ids are int64. */
int raven_embed(const void* wte, const int64_t* ids, void* out, int32_t M, int32_t dim,
                int64_t vocab, float scale, int32_t dtype, void* stream);

/* Greedy selection (RMM:1988-1989): out[m] = index of the first maximum of logits[m, :]. */
int raven_argmax(const float* logits, int64_t* out, int32_t M, int64_t vocab, void* stream);

/* *pos += delta, on the stream: advances the device-side position a replayed graph reads. */
int raven_advance_pos(int32_t* pos_dev, int32_t delta, void* stream);

/* One SandwichBlock (RMM:525-536) on M = B*S token rows: x_in -> x_out, both [M, h] (may alias).
 * `slot` is the cache slot this block appends to and reads.  ln_f (nullable) applies one more
 * RMSNorm to the block output (the ln_f after the last recurrence, RMM:762, and after the coda,
 * RMM:701); in that case x_out receives the normed values. */
size_t raven_block_workspace_bytes(const raven_dims* dims, int32_t M);
int    raven_sandwich_block(const raven_dims* dims, const raven_block_weights* w, const void* ln_f,
                            const void* x_in, void* x_out, const float* freqs,
                            const raven_kv_cache* cache, int32_t slot,
                            int32_t B, int32_t S, int32_t pos0, const int32_t* pos_dev,
                            void* workspace, size_t workspace_bytes, void* stream);

/* One recurrence iteration (core_block_forward, RMM:764-781): adapter over (state, embeds), then
 * n_blocks SandwichBlocks using cache slots first_slot .. first_slot + n_blocks - 1.
 * state_in / embeds / state_out: [M, h]; state_out may alias state_in.  ln_f as above. */
int raven_core_iteration(const raven_dims* dims, const void* adapter_w,
                         const raven_block_weights* blocks, int32_t n_blocks, const void* ln_f,
                         const void* state_in, const void* embeds, void* state_out,
                         const float* freqs, const raven_kv_cache* cache, int32_t first_slot,
                         int32_t B, int32_t S, int32_t pos0, const int32_t* pos_dev,
                         void* workspace, size_t workspace_bytes, void* stream);

/* n_iterations recurrences in a row (the loop of iterate_forward, RMM:751-761): iteration i reads and appends to the
 * cache slots slots[i * n_blocks + j], j = 0 .. n_blocks - 1 (a host array, read before the call returns).  The same
 * results as n_iterations calls of raven_core_iteration with ln_f on the last one; for one token row the closing
 * norm_4 of an iteration runs as the prologue of the next adapter product instead of a launch of its own.
 * state_out may not alias state_in or embeds. */
int raven_core_iterations(const raven_dims* dims, const void* adapter_w, const raven_block_weights* blocks,
                          int32_t n_blocks, const void* ln_f, const void* state_in, const void* embeds,
                          void* state_out, const float* freqs, const raven_kv_cache* cache, const int32_t* slots,
                          int32_t n_iterations, int32_t B, int32_t S, int32_t pos0, const int32_t* pos_dev,
                          void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* RAVEN_HIP_H */

// Skinny bf16 GEMM for 5..32 token rows with a caller-provided workspace: Y[M,N] = X[M,K] W[N,K]^T.
//
// The four waves of a workgroup own four different 16-row weight tiles (a gate tile and an up tile each
// for the SwiGLU epilogue) and walk the SAME K range, so the X tile of a macro-step (128 k-values) is
// fetched once per workgroup and shared through LDS instead of once per wave: the L2 -> L1 path, which
// bounds the K-split kernel in gemm_skinny.hip, carries a quarter of the X traffic.  What the K split
// inside the workgroup used to provide -- enough workgroups for matrices with few rows -- now comes from
// splitting K across workgroups (grid.y): each writes an fp32 partial tile to the workspace and a second,
// small launch adds the partials in a fixed order (deterministic, no atomics) and applies the epilogue.
// Weight rows are read with row-contiguous 16-byte lanes, parked in a wave-private LDS tile and picked up
// in MFMA operand layout, exactly as in gemm_skinny.hip; X goes through a double-buffered shared tile, one
// workgroup barrier per macro-step.
// As in gemm_skinny.hip, tiles are built from rows of one parity when the row pitch is an odd multiple of
// 64 bytes, and the macro-steps start at the rows' first 128-byte line boundary, so that a quarter-wave's
// 256 bytes are two whole lines; the elements in front of that boundary and behind the last full macro-step
// are single 32-wide steps done by the last K slice.

#include "raven_common.h"

extern "C" int raven_gemm(const void* x, const void* w, const void* residual, void* y, int32_t M, int32_t N, int32_t K,
                          int32_t dtype, int32_t out_f32, void* stream);
extern "C" int raven_adapter_gemm_concat(const void* x0, const void* x1, const void* w, void* y, int32_t M, int32_t N,
                                         int32_t K0, int32_t K1, int32_t dtype, void* stream);
extern "C" int raven_gemm_swiglu(const void* x, const void* fc, void* out, int32_t M, int32_t I, int32_t K, int32_t dtype,
                                 void* stream);

namespace raven {

extern int g_tiled_min_rows;
bool tiled_gemm_fits(int M, int N, int K0, int K1, int dtype);
int tiled_gemm(const void* x0, const void* x1, const void* w, const void* residual, void* y, int M, int N, int K0, int K1, int swiglu,
               int out_f32, hipStream_t s);

constexpr int kNsPitch = 136;  // bf16 elements per LDS row: 128 + 8 (272 bytes)
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

struct NsArgs {
    const bf16* w;         // [N or 2N, K]
    const bf16* x0;        // [M, k0]
    const bf16* x1;        // [M, k1] or null
    const bf16* residual;  // [M, N] or null
    void* y;               // [M, N] bf16 or float
    float* partial;        // [ks, M, n_total] when ks > 1
    int M, N, K, k0, k1;   // N = output columns (I for SwiGLU)
    int out_f32, ks;
    int row_stride;        // 1 = a tile is 16 neighbouring weight rows, 2 = every second row (rows of one parity)
    int line_aligned;      // the rows of a tile all start at the same offset inside a 128-byte line
    int ldw;               // elements between two weight rows: K, or more for a column block of a wider matrix
    const float* extra;    // [M, N] or null: fp32 sums of the remaining columns, added with the K-slice partials
    int raw_out;           // y receives the unrounded fp32 sums (what `extra` of a later call holds)
};

template <bool SWIGLU>
__device__ __forceinline__ void ns_epilogue(const NsArgs& a, int m, int n, float v0, float v1) {
    if (SWIGLU) {
        const float g = round_to<bf16>(v0), u = round_to<bf16>(v1);
        static_cast<bf16*>(a.y)[(int64_t)m * a.N + n] = from_f32<bf16>(round_to<bf16>(silu_f32(g)) * u);
    } else {
        float r = round_to<bf16>(v0);
        if (a.residual) r = round_to<bf16>(r + to_f32(a.residual[(int64_t)m * a.N + n]));
        if (a.out_f32) static_cast<float*>(a.y)[(int64_t)m * a.N + n] = r;
        else static_cast<bf16*>(a.y)[(int64_t)m * a.N + n] = from_f32<bf16>(r);
    }
}

template <int MT, bool SWIGLU>
__global__ __launch_bounds__(256) void mfma_ns_kernel(NsArgs a) {
    constexpr int NT = SWIGLU ? 2 : 1;
    __shared__ __align__(16) bf16 xs[2][16 * MT][kNsPitch];
    __shared__ __align__(16) bf16 wsm[4][16 * NT][kNsPitch];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int ln = lane & 15, kq = lane >> 4;
    const int lr = lane >> 4, lc = (lane & 15) * 8;  // loader role inside a wave: row of a group of 4, first element of the chunk
    const int K = a.ldw;  // row pitch of W

    // this wave's weight tile(s): row i of the tile is tile_row0 + i * rs, its output column out0 + i * rs
    const int rs = a.row_stride;
    const int group = rs == 2 ? blockIdx.x >> 1 : blockIdx.x, parity = rs == 2 ? blockIdx.x & 1 : 0;
    const int first = (group * 4 + wave) * 16 * rs;
    const bool tile_ok = first < a.N;
    const int out0 = (tile_ok ? first : group * 4 * 16 * rs) + parity;
    int tile_row0[NT];
    tile_row0[0] = out0;
    if (SWIGLU) tile_row0[NT - 1] = a.N + out0;

    // elements in front of the first 128-byte line boundary of the weight rows, per X segment (0 or 32, else
    // not used); the same for the four waves, whose rows are whole lines apart
    auto line_shift = [&](int wk0, int seg_len) {
        if (!a.line_aligned) return 0;
        const int mis = (int)(reinterpret_cast<uintptr_t>(a.w + (int64_t)tile_row0[0] * K + wk0) & 127);
        int sh = mis == 64 ? 32 : 0;
        if (SWIGLU && (int)(reinterpret_cast<uintptr_t>(a.w + (int64_t)tile_row0[NT - 1] * K + wk0) & 127) != mis) sh = 0;
        return sh <= seg_len ? sh : 0;
    };
    const int shift0 = line_shift(0, a.k0), shift1 = line_shift(a.k0, a.k1);

    // macro-steps of 128 k-values over the (up to two) X segments; this workgroup's share of them
    const int mac0 = (a.k0 - shift0) / 128, mac1 = (a.k1 - shift1) / 128;
    const int n_mac = mac0 + mac1;
    // (the division runs on the vector unit: readfirstlane tells the compiler that the result is the same in every lane)
    const int mb = __builtin_amdgcn_readfirstlane((int)((int64_t)n_mac * blockIdx.y / a.ks));
    const int me = __builtin_amdgcn_readfirstlane((int)((int64_t)n_mac * (blockIdx.y + 1) / a.ks));

    f32x4 acc[NT][MT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    int64_t wrow[NT][4];  // element offset of this lane's chunk column in each of the rows it loads
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) wrow[t][i] = (int64_t)(tile_row0[t] + (4 * i + lr) * rs) * K + lc;
    // D register sets: the loads of D macro-steps are in flight per wave.  A K slice is short (5 macro-steps for attn.proj of
    // the 3.5b shape with 8 slices), so with one set in flight a workgroup's life was one memory latency per step.
    constexpr int D = SWIGLU ? 2 : 4;
    struct Set {
        u32x4 x[MT], w[NT][4];
    };
    Set st[D];
    const int n_steps = me - mb;
    const int xrow = threadIdx.x >> 4, xc = (threadIdx.x & 15) * 8;
    // global -> registers.  Steps past the end of the slice load the first elements of X and W instead, which every
    // workgroup keeps hitting in the cache: the offsets are selected, not the loads, so that the loop body has no branch
    // around a load and the waits the compiler inserts count only the loads of the set being parked
    auto fetch = [&](int step, Set& set) {
        const bool live = step < n_steps;
        const int mac = mb + (live ? step : 0);
        const bool s1 = mac >= mac0;
        const bf16* X = s1 ? a.x1 : a.x0;
        const int ldx = s1 ? a.k1 : a.k0;
        const int kx = s1 ? shift1 + (mac - mac0) * 128 : shift0 + mac * 128;  // column inside the segment
        const int kw = (s1 ? a.k0 : 0) + kx;            // column of W
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = min(mt * 16 + xrow, a.M - 1);  // rows past M repeat the last one; never stored
            const int64_t off = live ? (int64_t)m * ldx + kx + xc : (int64_t)(xc + 128 * mt);  // distinct, or the compiler merges the idle loads and branches
            set.x[mt] = *reinterpret_cast<const u32x4*>(X + off);
        }
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int64_t off = live ? wrow[t][i] + kw : (int64_t)(lc + 128 * (4 * t + i));
                set.w[t][i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(a.w + off));
            }
    };
    auto park = [&](const Set& set, int buf) {  // registers -> LDS
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) *reinterpret_cast<u32x4*>(&xs[buf][mt * 16 + xrow][xc]) = set.x[mt];
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(&wsm[wave][t * 16 + 4 * i + lr][lc]) = set.w[t][i];
    };
    auto multiply = [&](int buf) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            bf16x8 bv[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                bv[mt] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&xs[buf][mt * 16 + ln][32 * j + 8 * kq]));
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                const bf16x8 av = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&wsm[wave][t * 16 + ln][32 * j + 8 * kq]));
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, bv[mt], acc[t][mt], 0, 0, 0);
            }
        }
    };

    // lanes of a wave exchange data through wsm[wave] without a workgroup barrier: pin the order of the LDS
    // accesses for the compiler (the LDS itself executes one wave's accesses in order)
    auto wave_sync = []() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    if (n_steps > 0) {
#pragma unroll
        for (int d = 0; d < D; ++d) fetch(d, st[d]);
    }
    // step s parks into xs[s & 1] before its barrier and multiplies out of it behind the barrier; the buffer it overwrites
    // was last read in step s - 2, which every wave has left when it passed the barrier of step s - 1.  The loop runs in
    // rounds of D steps; the steps of the last round that lie past the slice park their idle loads and skip the products,
    // so that every round issues the same loads in the same order (and the compiler's wait counts stay exact)
    for (int s0 = 0; s0 < n_steps; s0 += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            park(st[d], d & 1);         // D is even: step s0 + d has the parity of d
            fetch(s0 + d + D, st[d]);
            __syncthreads();
            if (s0 + d < n_steps) multiply(d & 1);
            wave_sync();                // this wave is done with its own weight tile
        }
    }

    // k-values in front of the first and behind the last full macro-step of each segment (32 for K = 5280):
    // the last K slice takes them, straight from global memory
    if ((int)blockIdx.y == a.ks - 1) {
#pragma unroll 1
        for (int part = 0; part < 4; ++part) {
            const int seg = part >> 1;
            const int seg_len = seg == 0 ? a.k0 : a.k1;
            const bf16* X = seg == 0 ? a.x0 : a.x1;
            const int wk0 = seg == 0 ? 0 : a.k0;
            const int sh = seg == 0 ? shift0 : shift1;
            const int kb = (part & 1) ? sh + (seg == 0 ? mac0 : mac1) * 128 : 0;
            const int ke = (part & 1) ? seg_len : sh;
            for (int k = kb; k < ke; k += 32) {
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const bf16x8 wv = *reinterpret_cast<const bf16x8*>(a.w + (int64_t)(tile_row0[t] + ln * rs) * K + wk0 + k + kq * 8);
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) {
                        const int m = min(mt * 16 + ln, a.M - 1);
                        const bf16x8 xv = *reinterpret_cast<const bf16x8*>(X + (int64_t)m * seg_len + k + kq * 8);
                        acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv, xv, acc[t][mt], 0, 0, 0);
                    }
                }
            }
        }
    }

    if (!tile_ok) return;
    // D layout: lane holds rows n = 4*kq + v of the tile for batch row m = mt*16 + ln
    const int n_total = SWIGLU ? 2 * a.N : a.N;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + ln;
        if (m >= a.M) continue;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int n = out0 + (kq * 4 + v) * rs;
            if (a.ks == 1) {
                ns_epilogue<SWIGLU>(a, m, n, acc[0][mt][v], acc[NT - 1][mt][v]);
            } else {
                float* p = a.partial + ((int64_t)blockIdx.y * a.M + m) * n_total;
                p[n] = acc[0][mt][v];
                if (SWIGLU) p[a.N + n] = acc[NT - 1][mt][v];
            }
        }
    }
}

// adds the K-slice partials in slice order and applies the epilogue; one thread per output element
template <bool SWIGLU>
__global__ __launch_bounds__(256) void splitk_finalize_kernel(NsArgs a) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)a.M * a.N) return;
    const int m = (int)(idx / a.N), n = (int)(idx - (int64_t)m * a.N);
    const int n_total = SWIGLU ? 2 * a.N : a.N;
    float v0 = a.extra ? a.extra[idx] : 0.f, v1 = 0.f;
    for (int s = 0; s < a.ks; ++s) {
        const float* p = a.partial + ((int64_t)s * a.M + m) * n_total;
        v0 += p[n];
        if (SWIGLU) v1 += p[a.N + n];
    }
    if (a.raw_out) static_cast<float*>(a.y)[idx] = v0;
    else ns_epilogue<SWIGLU>(a, m, n, v0, v1);
}

static int ns_cus() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0;
        hipDeviceProp_t p;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) cus = p.multiProcessorCount;
        if (cus <= 0) cus = 256;
    }
    return cus;
}

int g_linear_min_rows = 1;  // raven_set_tuning("linear_min_rows"): up to this many rows go to the kernels without a workspace
int g_linear_ks = 0;  // raven_set_tuning("linear_ks"): K slices per weight tile, 0 = choose from the grid size

// ks_left (may be null): the caller adds the K slices itself (rmsnorm.hip, splitk_sums_then_norm); receives their number,
// 0 when the product was finished here
template <bool SWIGLU>
static int launch_ns(NsArgs a, void* workspace, size_t workspace_bytes, hipStream_t s, int* ks_left = nullptr) {
    // tiles of one row parity when the row pitch is an odd multiple of 64 bytes (needs whole pairs of tiles)
    if (a.ldw == 0) a.ldw = a.K;
    a.row_stride = ((a.ldw * 2) % 128 == 64 && a.N % 32 == 0) ? 2 : 1;
    a.line_aligned = (a.ldw * 2 * a.row_stride) % 128 == 0;
    const int rs = a.row_stride;
    const int blocks = (a.N / 16 + 4 * rs - 1) / (4 * rs) * rs;
    const int n_mac = a.k0 / 128 + a.k1 / 128;
    const int n_total = SWIGLU ? 2 * a.N : a.N;
    // As few K slices as give every CU a workgroup (84 tile groups x 3 slices = 252 for the 5280-row products of the 3.5b
    // shape), at least four macro-steps per slice.  With four macro-steps of loads in flight per wave one workgroup keeps
    // a CU's memory pipe busy, and the launch then ends in one round: us per product (both launches) at 32 rows with
    // 2 / 3 / 5 / 6 / 8 slices: attn.proj 20.6 / 18.6 / 22.6 / 21.7 / 25.8, mlp.proj 45.2 / 37.4 / 43.2 / 41.7 / 45.9
    int ks = g_linear_ks > 0 ? g_linear_ks : (ns_cus() * 9 / 10 + blocks - 1) / blocks;
    if (ks > n_mac / 4) ks = n_mac / 4;
    if (ks > 8) ks = 8;
    if (ks < 1) ks = 1;
    while (ks > 1 && (size_t)ks * a.M * n_total * sizeof(float) > workspace_bytes) --ks;
    if ((a.extra || a.raw_out) && ks < 2) {  // those go through the second launch
        ks = 2;
        if (n_mac < 2 || (size_t)ks * a.M * n_total * sizeof(float) > workspace_bytes) {
            raven_host::set_error("linear: a column block needs two K slices (K=%d) and their workspace", a.K);
            return -1;
        }
    }
    a.ks = ks;
    a.partial = ks > 1 ? static_cast<float*>(workspace) : nullptr;
    const dim3 grid(blocks, ks);
    if (a.M <= 16) mfma_ns_kernel<1, SWIGLU><<<grid, dim3(256), 0, s>>>(a);
    else mfma_ns_kernel<2, SWIGLU><<<grid, dim3(256), 0, s>>>(a);
    if (ks_left) *ks_left = ks > 1 ? ks : 0;
    if (ks > 1 && !ks_left) {
        const int64_t n_out = (int64_t)a.M * a.N;
        splitk_finalize_kernel<SWIGLU><<<dim3((unsigned)((n_out + 255) / 256)), dim3(256), 0, s>>>(a);
    }
    return raven_host::check_launch("linear (split-K MFMA)");
}

// Column block [c0, c0 + K) of a wider bf16 weight matrix with row pitch ldw, for 2..32 rows:
// y = round(x W[:, c0 : c0 + K]^T + extra), or the unrounded fp32 sums (raw_out) that a later call takes as `extra`.
// The adapter product over [state, embedding] (recpre/raven_modeling_minimal.py:776) is split with it when the
// embedding half stays the same over many calls; the product keeps its single rounding.
int linear_column_block(const void* x, const void* w_block, int ldw, const float* extra, void* y, int raw_out, int M, int N, int K,
                        void* workspace, size_t workspace_bytes, hipStream_t s) {
    if (M < 2 || M > 32 || N % 16 || K % 32 || K < 256 || !workspace || ((uintptr_t)workspace & 255)) {
        raven_host::set_error("linear_column_block: unsupported shape M=%d N=%d K=%d", M, N, K);
        return -1;
    }
    NsArgs a{};
    a.w = static_cast<const bf16*>(w_block);
    a.x0 = static_cast<const bf16*>(x);
    a.y = y;
    a.M = M; a.N = N; a.K = K; a.k0 = K; a.k1 = 0; a.ldw = ldw; a.extra = extra; a.raw_out = raw_out;
    return launch_ns<false>(a, workspace, workspace_bytes, s);
}

int g_fuse_sums_norm = 1;  // raven_set_tuning("fuse_sums_norm"): 0 = a K-split product always adds its slices in a launch of its own

// A product whose result goes straight into an RMSNorm launch: y = round(round(x W^T [+ extra]) + residual) for at most 32
// bf16 rows, W either a whole [N, K0 + K1] matrix (ldw = 0) or a column block with row pitch ldw (K1 = 0).  When the product
// takes the K-split kernel, its slices are left in the workspace un-added (*ks_left slices, to be handed to
// splitk_sums_then_norm before anything else uses the workspace) and y is not written; otherwise the product is finished
// into y and *ks_left is 0.
int linear_leave_sums(const void* x0, const void* x1, const void* w, int ldw, const float* extra, const void* residual, void* y, int M,
                      int N, int K0, int K1, int dtype, void* workspace, size_t workspace_bytes, hipStream_t s, int* ks_left) {
    *ks_left = 0;
    bool split = g_fuse_sums_norm && dtype == RAVEN_BF16 && M >= 2 && M <= 32 && N % 16 == 0 && N <= 8192 && K0 % 32 == 0 && K1 % 32 == 0 &&
                 workspace != nullptr && ((uintptr_t)workspace & 255) == 0 && K0 / 128 + K1 / 128 >= 8 && M > g_linear_min_rows;
    if (split && !ldw && g_linear_ks == 0) split = N / 16 < 2 * ns_cus() && (M >= 5 || K0 + K1 >= 8192);  // from 5 rows on, from 2 for long K: the product's second launch is saved, and the norm launch requests all slices of a row at once (5 / 8 / 12 rows: 228.7 / 350.7 / 501.5 tokens/s against 228.3 / 348.5 / 495.0 with the K split only from 13 rows or K >= 8192)
    if (!split) {
        if (ldw) return linear_column_block(x0, w, ldw, extra, y, 0, M, N, K0, workspace, workspace_bytes, s);
        return raven_linear(x0, x1, w, residual, y, M, N, K0, K1, 0, 0, dtype, workspace, workspace_bytes, s);
    }
    NsArgs a{};
    a.w = static_cast<const bf16*>(w);
    a.x0 = static_cast<const bf16*>(x0);
    a.x1 = static_cast<const bf16*>(x1);
    a.residual = static_cast<const bf16*>(residual);
    a.y = y;
    a.M = M; a.N = N; a.K = K0 + K1; a.k0 = K0; a.k1 = K1; a.ldw = ldw; a.extra = extra;
    return launch_ns<false>(a, workspace, workspace_bytes, s, ks_left);
}

}  // namespace raven

extern "C" size_t raven_linear_workspace_bytes(int32_t M, int32_t n_out_max) {
    if (M <= 0 || n_out_max <= 0) return 0;
    const int rows = M < 32 ? M : 32;
    return raven_host::align_up((size_t)8 * rows * n_out_max * sizeof(float));
}

extern "C" int raven_linear(const void* x0, const void* x1, const void* w, const void* residual, void* y, int32_t M, int32_t N,
                            int32_t K0, int32_t K1, int32_t swiglu, int32_t out_f32, int32_t dtype, void* workspace,
                            size_t workspace_bytes, void* stream) {
    using namespace raven;
    RAVEN_REQUIRE(dtype == RAVEN_F32 || dtype == RAVEN_BF16, "linear: unknown dtype %d", dtype);
    RAVEN_REQUIRE(M >= 0 && N > 0 && K0 > 0 && K1 >= 0, "linear: bad shape M=%d N=%d K0=%d K1=%d", M, N, K0, K1);
    if (M == 0) return 0;
    RAVEN_REQUIRE(x0 && w && y, "linear: null pointer");
    RAVEN_REQUIRE((K1 == 0) == (x1 == nullptr), "linear: x1 and K1 must be given together");
    RAVEN_REQUIRE(!(swiglu && (residual || out_f32 || K1)), "linear: the SwiGLU epilogue takes one operand, no residual, and stores T");
    RAVEN_REQUIRE(!(K1 && (residual || out_f32)), "linear: the two-operand form has a plain epilogue");
    if (M >= g_tiled_min_rows && tiled_gemm_fits(M, N, K0, K1, dtype))  // many rows: tiles of the whole product on the matrix cores
        return tiled_gemm(x0, x1, w, residual, y, M, N, K0, K1, swiglu, out_f32, static_cast<hipStream_t>(stream));
    bool fits = dtype == RAVEN_BF16 && M > g_linear_min_rows && N % 16 == 0 && K0 % 32 == 0 && K1 % 32 == 0 && workspace != nullptr &&
                ((uintptr_t)workspace & 255) == 0 && K0 / 128 + K1 / 128 >= 1;
    // Matrices with many rows give the kernel without a workspace enough workgroups and it is then the faster one
    // (its waves never wait for each other); the K split pays for few rows, once X re-reads (more than 16 token
    // rows) or the length of a wave's K range (K >= 8192) hold that kernel back.
    if (fits && g_linear_ks == 0) fits = (swiglu ? 2 * N : N) / 16 < 2 * ns_cus() && (M > 16 || K0 + K1 >= 8192);
    if (!fits) {  // one to four rows, fp32, odd shapes, large N: the kernels without a workspace
        if (swiglu) return raven_gemm_swiglu(x0, w, y, M, N, K0, dtype, stream);
        if (K1) return raven_adapter_gemm_concat(x0, x1, w, y, M, N, K0, K1, dtype, stream);
        return raven_gemm(x0, w, residual, y, M, N, K0, dtype, out_f32, stream);
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t out_es = out_f32 ? 4 : 2;
    for (int m0 = 0; m0 < M; m0 += 32) {  // the weight matrix is streamed once per 32 rows
        NsArgs a{};
        a.M = (M - m0) < 32 ? (M - m0) : 32;
        if (a.M <= g_linear_min_rows) {  // a short last pass
            const char* r = residual ? static_cast<const char*>(residual) + (size_t)m0 * N * 2 : nullptr;
            char* yy = static_cast<char*>(y) + (size_t)m0 * N * out_es;
            const char* xa = static_cast<const char*>(x0) + (size_t)m0 * K0 * 2;
            const char* xb = x1 ? static_cast<const char*>(x1) + (size_t)m0 * K1 * 2 : nullptr;
            int rc;
            if (swiglu) rc = raven_gemm_swiglu(xa, w, yy, a.M, N, K0, dtype, stream);
            else if (K1) rc = raven_adapter_gemm_concat(xa, xb, w, yy, a.M, N, K0, K1, dtype, stream);
            else rc = raven_gemm(xa, w, r, yy, a.M, N, K0, dtype, out_f32, stream);
            if (rc) return rc;
            continue;
        }
        a.w = static_cast<const bf16*>(w);
        a.x0 = static_cast<const bf16*>(x0) + (size_t)m0 * K0;
        a.x1 = x1 ? static_cast<const bf16*>(x1) + (size_t)m0 * K1 : nullptr;
        a.residual = residual ? static_cast<const bf16*>(residual) + (size_t)m0 * N : nullptr;
        a.y = static_cast<char*>(y) + (size_t)m0 * N * out_es;
        a.N = N; a.K = K0 + K1; a.k0 = K0; a.k1 = K1; a.out_f32 = out_f32;
        const int rc = swiglu ? launch_ns<true>(a, workspace, workspace_bytes, s) : launch_ns<false>(a, workspace, workspace_bytes, s);
        if (rc) return rc;
    }
    return 0;
}

// Skinny GEMMs of the decode path: Y[M,N] = X[M,K] W[N,K]^T with M = a handful of token rows and
// W a weight matrix that is streamed from HBM exactly once per call (per 32 rows of X).
//
// Two kernels:
//   gemv_kernel  (any T, up to 8 rows of X per pass)  -- X lives in LDS, every wave owns whole rows
//                of W, reads them with 16-byte lane-contiguous loads and accumulates with
//                v_dot2_f32_bf16 / fp32 FMA; a DPP wave reduction finishes each row.
//   mfma_kernel  (bf16, up to 32 rows of X per pass)   -- 16-row tiles of W are the A operand of
//                v_mfma_f32_16x16x32_bf16, X is the B operand; the four waves of a workgroup split
//                K and reduce through LDS.
// Epilogues (all round the fp32 accumulator to T first, as an nn.Linear output would be stored):
//   plain (+ residual add in T, + optional float store)   RMM:493, 509, 711, 534-535
//   SwiGLU: T(T(silu(gate)) * up), gate row j, up row j+I  RMM:507-508
// The adapter's concat (RMM:776) is folded in by giving X as two pointers that cover K0 and K1.

#include <string>

#include "raven_common.h"

extern "C" int raven_gemv_fused(const void* x0, const void* x1, const void* norm_a, const void* norm_b, void* xa_out,
                                const void* w, const void* residual, void* y, int32_t N, int32_t K0, int32_t K1, float eps,
                                int32_t swiglu, int32_t out_f32, int32_t dtype, void* stream);

namespace raven {

int set_gemv1_tuning(const char* key, int value);
extern int g_linear_ks;
extern int g_tiled_min_rows, g_tiled_variant, g_tiled_split_tail;
bool tiled_gemm_fits(int M, int N, int K0, int K1, int dtype);
int tiled_gemm(const void* x0, const void* x1, const void* w, const void* residual, void* y, int M, int N, int K0, int K1, int swiglu,
               int out_f32, hipStream_t s);
extern int g_attn_split_target, g_attn_big_grid, g_attn_wide, g_linear_min_rows, g_attn_nosplit_pairs, g_attn_nosplit_len, g_rope_tiled_rows, g_prefill_waves, g_norm_early, g_fuse_sums_norm, g_attn_prefetch, g_fuse_qkv_rope, g_pad_chunk_rows, g_pad_decode_rows;

enum { EPI_PLAIN = 0, EPI_SWIGLU = 1 };

struct GemmArgs {
    const void* w;         // [N_total, K]
    const void* x0;        // [M, k0]
    const void* x1;        // [M, k1] or null
    const void* residual;  // [M, N] or null
    void* y;               // [M, N] (T, or float when out_f32)
    int M, N, K, k0, k1;   // N = number of output columns (I for SwiGLU)
    int out_f32;
    int units_per_wave;    // gemv: row pairs per wave
    int interleave;        // gemv: unit = u * total_waves + wave (1) or wave * units_per_wave + u (0)
    int row_stride;        // mfma: 1 = a tile is 16 neighbouring weight rows, 2 = every second row (see mfma_kernel)
    int line_aligned;      // mfma: the rows of a tile all start at the same offset inside a 128-byte line
    int rows_per_unit;     // mfma, ragged variants: weight rows (per side for SwiGLU) a workgroup owns; its last tile is partly empty
};

// Launch-shape knobs (raven_set_tuning); 0 = automatic.
struct Tuning {
    int gemv_units_per_wave = 0;
    int gemv_interleave = 1;
    int gemv_nontemporal = 1;
    int gemv_wgs_per_cu = 4;
    int gemm_four_tiles = 1;
    int gemm_mfma_min_rows = 2;  // fewer rows go to the vector kernels (one row: the K-split GEMV)
    int gemm_ragged = 1;         // 0 never, 1 = one workgroup per resident slot with partly empty last tiles where the shape divides so
};
static Tuning g_tuning;

// weight rows are read exactly once: stream them past the caches
template <bool NT, typename T>
__device__ __forceinline__ Chunk<T> load_weight(const T* p) {
    if (!NT) return load_chunk(p);
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    Chunk<T> c;
    *reinterpret_cast<u32x4*>(&c) = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return c;
}

template <typename T>
__device__ __forceinline__ void store_out(const GemmArgs& a, int m, int n, float acc) {
    float r = round_to<T>(acc);
    if (a.residual) r = round_to<T>(r + to_f32(static_cast<const T*>(a.residual)[(int64_t)m * a.N + n]));
    if (a.out_f32)
        static_cast<float*>(a.y)[(int64_t)m * a.N + n] = r;
    else
        static_cast<T*>(a.y)[(int64_t)m * a.N + n] = from_f32<T>(r);
}

template <typename T>
__device__ __forceinline__ float swiglu(float gate_acc, float up_acc) {
    const float g = round_to<T>(gate_acc), u = round_to<T>(up_acc);
    return round_to<T>(round_to<T>(silu_f32(g)) * u);
}

// ------------------------------------------------------------------------------------------------
// gemv_kernel: 256 threads; dynamic LDS holds X as [MB][K] of T.
// ------------------------------------------------------------------------------------------------
template <typename T, int MB, int EPI, bool NT>
__global__ __launch_bounds__(256) void gemv_kernel(GemmArgs a) {
    constexpr int E = Chunk<T>::N;
    constexpr int U = 4;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* xs = reinterpret_cast<T*>(smem_raw);

    const int K = a.K, n_chunks = K / E, c0 = a.k0 / E;
    // stage X: row m of LDS = concat(x0[m], x1[m]); rows >= M are zero
    for (int i = threadIdx.x; i < MB * n_chunks; i += 256) {
        const int m = i / n_chunks, c = i - m * n_chunks;
        Chunk<T> v = zero_chunk<T>();
        if (m < a.M) {
            v = (c < c0) ? load_chunk(static_cast<const T*>(a.x0) + (int64_t)m * a.k0 + c * E)
                         : load_chunk(static_cast<const T*>(a.x1) + (int64_t)m * a.k1 + (c - c0) * E);
        }
        store_chunk(xs + (int64_t)m * K + c * E, v);
    }
    __syncthreads();

    const int lane = threadIdx.x & 63;
    const int gwave = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int total_waves = gridDim.x * 4;
    const int n_units = (EPI == EPI_SWIGLU) ? a.N : (a.N + 1) / 2;
    const T* W = static_cast<const T*>(a.w);

    for (int u = 0; u < a.units_per_wave; ++u) {
        // interleaved: at any moment the waves of the whole grid read neighbouring rows
        const int unit = a.interleave ? u * total_waves + gwave : gwave * a.units_per_wave + u;
        if (unit >= n_units) break;
        int r0, r1;
        bool r1_ok = true;
        if (EPI == EPI_SWIGLU) {
            r0 = unit;
            r1 = unit + a.N;
        } else {
            r0 = 2 * unit;
            r1 = r0 + 1;
            if (r1 >= a.N) { r1 = r0; r1_ok = false; }
        }
        const T* w0 = W + (int64_t)r0 * K;
        const T* w1 = W + (int64_t)r1 * K;
        float acc0[MB], acc1[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) acc0[m] = acc1[m] = 0.f;

        for (int c = lane; c < n_chunks; c += 64 * U) {
            Chunk<T> a0[U], a1[U];
#pragma unroll
            for (int j = 0; j < U; ++j) {
                const int cc = c + 64 * j;
                if (cc < n_chunks) {
                    a0[j] = load_weight<NT>(w0 + cc * E);
                    a1[j] = load_weight<NT>(w1 + cc * E);
                } else {
                    a0[j] = zero_chunk<T>();
                    a1[j] = zero_chunk<T>();
                }
            }
#pragma unroll
            for (int j = 0; j < U; ++j) {
                const int cc = min(c + 64 * j, n_chunks - 1);
#pragma unroll
                for (int m = 0; m < MB; ++m) {
                    const Chunk<T> xv = load_chunk(xs + (int64_t)m * K + cc * E);
                    acc0[m] = dot_chunk(a0[j], xv, acc0[m]);
                    acc1[m] = dot_chunk(a1[j], xv, acc1[m]);
                }
            }
        }
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            acc0[m] = wave_sum(acc0[m]);
            acc1[m] = wave_sum(acc1[m]);
        }
        if (lane == 0) {
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                if (m < a.M) {
                    if (EPI == EPI_SWIGLU) {
                        static_cast<T*>(a.y)[(int64_t)m * a.N + unit] = from_f32<T>(swiglu<T>(acc0[m], acc1[m]));
                    } else {
                        store_out<T>(a, m, r0, acc0[m]);
                        if (r1_ok) store_out<T>(a, m, r1, acc1[m]);
                    }
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// mfma_kernel: bf16, 256 threads = 4 waves that split K; MT = ceil(M/16) batch tiles; NT weight
// tiles of 16 rows per workgroup.  D = A * B with A = W tile [16 n x 32 k], B = X^T [32 k x 16 m]:
// lane l supplies A[n = l%16][k = 8*(l/16) ..+8] and B[k = 8*(l/16) ..+8][m = l%16] and receives
// D[n = 4*(l/16) + v][m = l%16], v = 0..3.
//
// The MFMA operand layout puts 16 different matrix rows into 16 neighbouring lanes; loading it straight
// from global memory makes every quarter-wave touch 16 cache lines for 256 bytes, and the L1 address path
// (not HBM) then caps the kernel near 3 TB/s.  So K is walked in macro-steps of 128 elements: each wave
// loads its rows with row-contiguous 16-byte lanes (a quarter-wave reads 256 consecutive bytes of one
// row), parks them in a wave-private LDS tile with 272-byte row pitch, and reads the MFMA fragments from
// there (conflict-free: 16 rows x 16 bytes cover the 64 banks once).  The next macro-step's global loads
// are issued into registers as soon as the current one is parked, before it is multiplied.  No barrier inside the K loop: every
// wave only touches its own LDS tile.
//
// A quarter-wave's 256 bytes should also be two whole 128-byte lines: a row that starts 64 bytes into a line
// makes them three, and that alone costs 20 % of the bandwidth.  K = 5280 (10560 bytes per row) puts every
// second row there.  So with row_stride = 2 a tile is made of 16 rows of the SAME parity, all its rows are
// misaligned by the same amount, and the macro-steps of such a tile start `shift` elements into the row
// (at the next line boundary); the `shift` elements before them and whatever is left behind the last full
// macro-step are single 32-wide MFMA steps straight from global memory (first and last wave).
// ------------------------------------------------------------------------------------------------
// KM = k-values per macro-step: 128, or 64 for the variants with four weight tiles per workgroup (the same
// bytes per macro-step; a quarter-wave then reads two rows of 128 bytes).  LDS rows are KM + 8 elements long
// (272 or 144 bytes: both spread 16 rows over the 64 banks without conflicts for 16-byte reads).
//
// RAG: a workgroup owns a.rows_per_unit rows (per side for SwiGLU) instead of 16 per tile slot: its tile slots cover them
// 16 at a time and the last slot is partly empty (its missing rows are neither loaded nor stored).  This lets the host cut
// a matrix into exactly as many workgroups as the chip holds at once (17920 gate rows = 512 x 35), where whole tiles
// would leave a partly filled last round.
template <int MT, int NT, int EPI, int KM = 128, bool RAG = false>
__global__ __launch_bounds__(256) void mfma_kernel(GemmArgs a) {
    constexpr int ROWS = 16 * (NT + MT);
    constexpr int kPitch = KM + 8;
    constexpr int LPR = KM / 8;        // lanes per row of a macro-step
    constexpr int RPI = 64 / LPR;      // rows per load instruction
    constexpr int IPT = 16 / RPI;      // load instructions per 16-row tile
    constexpr int NG = EPI == EPI_SWIGLU ? NT / 2 : NT;  // tiles side by side along N (SwiGLU: NG gate tiles + their NG up tiles)
    __shared__ __align__(16) bf16 stage[4][ROWS][kPitch];
    static_assert(sizeof(bf16) * 4 * ROWS * kPitch >= sizeof(float) * 3 * NT * MT * 64 * 4, "stage doubles as the reduction buffer");
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int ln = lane & 15, kq = lane >> 4;
    const int K = a.K;
    const int rs = a.row_stride;
    // a group is rs units: with rs = 2 the even unit takes the even rows of the group's tiles, the odd unit the odd rows
    const int group = rs == 2 ? blockIdx.x >> 1 : blockIdx.x;
    const int parity = rs == 2 ? blockIdx.x & 1 : 0;

    const bf16* W = static_cast<const bf16*>(a.w);
    int tile_row0[NT];  // first weight row of each tile; row i of the tile is tile_row0 + i * rs
    int tile_out0[NT];  // output column of that row
    bool tile_ok[NT];
    int tile_rows[NT];  // RAG: rows of the tile that exist (1..16 where tile_ok); 16 otherwise
    const int rpu = RAG ? a.rows_per_unit : 16 * NG;  // rows a unit owns per side
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const int first = (group * rpu + (t % NG) * 16) * rs;   // SwiGLU: the first NG tiles are gate tiles, the others their up tiles
        tile_ok[t] = first < a.N && (!RAG || (t % NG) * 16 < rpu);
        tile_rows[t] = RAG ? min(16, rpu - (t % NG) * 16) : 16;
        tile_out0[t] = (tile_ok[t] ? first : group * rpu * rs) + parity;
        tile_row0[t] = tile_out0[t] + (EPI == EPI_SWIGLU ? (t / NG) * a.N : 0);
        if (RAG && !tile_ok[t]) tile_rows[t] = 1;  // reads row 0 of the unit's first tile, stores nothing
    }

    f32x4 acc[NT][MT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    struct Staged {
        u32x4 w[NT][IPT];
        u32x4 x[MT][IPT];
    };
    bf16(*my)[kPitch] = stage[wave];
    const int lr = lane / LPR, lc = (lane % LPR) * 8;  // loader role: row within a group of RPI, first element of the chunk

    // X is given as up to two K segments (the adapter's concat); each is walked on its own
#pragma unroll 1
    for (int seg = 0; seg < 2; ++seg) {
        const int seg_len = seg == 0 ? a.k0 : a.k1;
        if (seg_len == 0) continue;
        const int wk0 = seg == 0 ? 0 : a.k0;  // column of W where this segment starts
        const bf16* X = static_cast<const bf16*>(seg == 0 ? a.x0 : a.x1);
        const int ldx = seg == 0 ? a.k0 : a.k1;
        // elements in front of the first 128-byte line boundary of this segment's weight rows (0 or 32, else not used)
        int shift = 0;
        if (a.line_aligned) {
            const int mis = (int)(reinterpret_cast<uintptr_t>(W + (int64_t)tile_row0[0] * K + wk0) & 127);
            shift = mis == 64 ? 32 : 0;
#pragma unroll
            for (int t = 1; t < NT; ++t)
                if ((int)(reinterpret_cast<uintptr_t>(W + (int64_t)tile_row0[t] * K + wk0) & 127) != mis) shift = 0;
            if (shift > seg_len) shift = 0;
        }
        const int n_macro = (seg_len - shift) / KM;
        // the four waves take the macro-steps in turn, so that the workgroup as a whole walks its rows in pieces of
        // 4 * KM contiguous elements (DRAM pages are then read in longer runs than one wave's 256 bytes)
        const int mb = wave, me = n_macro;

        auto fetch = [&](int mac, Staged& st) {  // global -> registers, row-contiguous lanes
            const int k = shift + mac * KM + lc;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int i = 0; i < IPT; ++i) {
                    const int m = min(mt * 16 + RPI * i + lr, a.M - 1);  // rows past M repeat the last one; never stored
                    st.x[mt][i] = *reinterpret_cast<const u32x4*>(X + (int64_t)m * ldx + k);
                }
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int i = 0; i < IPT; ++i) {
                    if (RAG && RPI * i + lr >= tile_rows[t]) continue;  // rows the tile does not have: their products are never stored
                    st.w[t][i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(W + (int64_t)(tile_row0[t] + (RPI * i + lr) * rs) * K + wk0 + k));
                }
        };
        auto park = [&](const Staged& st) {  // registers -> this wave's LDS tile
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int i = 0; i < IPT; ++i) *reinterpret_cast<u32x4*>(&my[t * 16 + RPI * i + lr][lc]) = st.w[t][i];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int i = 0; i < IPT; ++i) *reinterpret_cast<u32x4*>(&my[(NT + mt) * 16 + RPI * i + lr][lc]) = st.x[mt][i];
        };
        auto multiply = [&]() {  // LDS -> MFMA fragments
#pragma unroll
            for (int j = 0; j < KM / 32; ++j) {
                bf16x8 bv[MT];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)  // same access type as the stores in park(): the two must stay ordered
                    bv[mt] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&my[(NT + mt) * 16 + ln][32 * j + 8 * kq]));
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const bf16x8 av = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&my[t * 16 + ln][32 * j + 8 * kq]));
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, bv[mt], acc[t][mt], 0, 0, 0);
                }
            }
        };

        // lanes exchange data through the tile without a workgroup barrier: pin the order of the LDS
        // accesses for the compiler (the LDS itself executes one wave's accesses in order)
        auto wave_sync = []() {
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        };
        // one register set: its loads for macro-step s+1 are in flight while step s is multiplied out of LDS
        Staged st{};
        if (mb < me) fetch(mb, st);
        for (int mac = mb; mac < me; mac += 4) {
            park(st);
            wave_sync();
            if (mac + 4 < me) fetch(mac + 4, st);
            multiply();
            wave_sync();
        }
        // 32-element steps in front of the first and behind the last macro-step: first and last wave, straight from global memory
        if (wave == 0 || wave == 3) {
            const int kb = wave == 0 ? 0 : shift + n_macro * KM, ke = wave == 0 ? shift : seg_len;
            for (int k = kb; k < ke; k += 32) {
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const int wr = RAG ? min(ln, tile_rows[t] - 1) : ln;  // a partly empty tile repeats its last row
                    const bf16x8 wv = *reinterpret_cast<const bf16x8*>(W + (int64_t)(tile_row0[t] + wr * rs) * K + wk0 + k + kq * 8);
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) {
                        const int m = min(mt * 16 + ln, a.M - 1);
                        const bf16x8 xv = *reinterpret_cast<const bf16x8*>(X + (int64_t)m * ldx + k + kq * 8);
                        acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv, xv, acc[t][mt], 0, 0, 0);
                    }
                }
            }
        }
    }

    // cross-wave reduction over the K split (the staging tiles are free now)
    __syncthreads();
    float(*red)[NT * MT][64][4] = reinterpret_cast<float(*)[NT * MT][64][4]>(&stage[0][0][0]);
    if (wave > 0) {
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int v = 0; v < 4; ++v) red[wave - 1][t * MT + mt][lane][v] = acc[t][mt][v];
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int v = 0; v < 4; ++v)
                acc[t][mt][v] += red[0][t * MT + mt][lane][v] + red[1][t * MT + mt][lane][v] + red[2][t * MT + mt][lane][v];

#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + ln;
        if (m >= a.M) continue;
        if (EPI == EPI_SWIGLU) {
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                if (!tile_ok[g]) continue;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    if (RAG && kq * 4 + v >= tile_rows[g]) continue;
                    const int n = tile_out0[g] + (kq * 4 + v) * rs;
                    static_cast<bf16*>(a.y)[(int64_t)m * a.N + n] = from_f32<bf16>(swiglu<bf16>(acc[g][mt][v], acc[NG + g][mt][v]));
                }
            }
        } else {
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                if (!tile_ok[t]) continue;
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (!RAG || kq * 4 + v < tile_rows[t]) store_out<bf16>(a, m, tile_out0[t] + (kq * 4 + v) * rs, acc[t][mt][v]);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// host dispatch
// ------------------------------------------------------------------------------------------------
static int n_cus() {
    static int cus = 0;
    if (cus == 0) {
        int dev = 0;
        hipDeviceProp_t p;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) cus = p.multiProcessorCount;
        if (cus <= 0) cus = 256;
    }
    return cus;
}

template <typename T, int MB, int EPI, bool NT>
static int launch_gemv_nt(GemmArgs a, hipStream_t s) {
    const size_t lds = (size_t)MB * a.K * sizeof(T);
    RAVEN_REQUIRE(lds <= 160 * 1024, "gemm: %d rows x K=%d does not fit the 160 KB LDS", MB, a.K);
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)gemv_kernel<T, MB, EPI, NT>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) {
            raven_host::set_error("gemm: hipFuncSetAttribute failed: %s", hipGetErrorString(e));
            return (int)e;
        }
        attr_set = true;
    }
    const int n_units = (EPI == EPI_SWIGLU) ? a.N : (a.N + 1) / 2;
    // as few units per wave as keeps every workgroup resident at once
    const int max_wgs = n_cus() * (g_tuning.gemv_wgs_per_cu > 0 ? g_tuning.gemv_wgs_per_cu : 4);
    int upw = g_tuning.gemv_units_per_wave;
    if (upw <= 0) {
        upw = 1;
        while ((n_units + 4 * upw - 1) / (4 * upw) > max_wgs) ++upw;
    }
    a.units_per_wave = upw;
    a.interleave = g_tuning.gemv_interleave;
    const int wgs = (n_units + 4 * upw - 1) / (4 * upw);
    gemv_kernel<T, MB, EPI, NT><<<dim3(wgs), dim3(256), lds, s>>>(a);
    return raven_host::check_launch("gemv");
}

template <typename T, int MB, int EPI>
static int launch_gemv(GemmArgs a, hipStream_t s) {
    return g_tuning.gemv_nontemporal ? launch_gemv_nt<T, MB, EPI, true>(a, s) : launch_gemv_nt<T, MB, EPI, false>(a, s);
}

template <typename T, int EPI>
static int dispatch_gemv(GemmArgs a, hipStream_t s) {
    if (a.M <= 1) return launch_gemv<T, 1, EPI>(a, s);
    if (a.M <= 2) return launch_gemv<T, 2, EPI>(a, s);
    if (a.M <= 4) return launch_gemv<T, 4, EPI>(a, s);
    return launch_gemv<T, 8, EPI>(a, s);
}

template <int EPI>
static int dispatch_mfma(GemmArgs a, hipStream_t s) {
    const int n_tiles16 = a.N / 16;
    // rows alternate between line-aligned and 64 bytes off when the row pitch is an odd multiple of 64 bytes:
    // tiles of equal parity then (needs whole pairs of tiles); any multiple of 128 bytes needs nothing special
    const int pitch = a.K * 2;
    a.row_stride = (pitch % 128 == 64 && a.N % 32 == 0) ? 2 : 1;
    a.line_aligned = (pitch * a.row_stride) % 128 == 0;
    const int rs = a.row_stride;
    // Four tiles per workgroup (64-wide K steps) halve the X re-reads per weight byte: 5.0 -> 5.7 TB/s in steady state
    // at 32 rows.  Their workgroups are twice as long, so the gain only survives where the grid is balanced: at most
    // one workgroup per CU (Wqkv: 248), or so many that the last round does not matter.  Tuning key gemm_four_tiles:
    // 0 never, 1 by this rule, 2 whenever the shape allows.
    const int groups4 = (n_tiles16 + 4 * rs - 1) / (4 * rs) * rs;       // plain epilogue: 4 tiles side by side
    const int groups2 = (n_tiles16 + 2 * rs - 1) / (2 * rs) * rs;       // SwiGLU with 4 tiles: 2 gate + 2 up
    const int g4 = EPI == EPI_SWIGLU ? groups2 : groups4;
    const bool four = g_tuning.gemm_four_tiles == 2 ||
                      (g_tuning.gemm_four_tiles == 1 && a.M > 16 && g4 >= n_cus() / 2 && (g4 <= n_cus() || g4 >= 8 * n_cus()));
    if constexpr (EPI == EPI_SWIGLU) {
        // A matrix that divides into one workgroup per resident slot (two per CU) of 33..48 gate rows: three tile slots
        // per side, the last one partly empty -- one full round instead of a partly filled last one, and the X tile is
        // fetched once per 70 weight rows instead of once per 32.  mlp.fc of the 3.5b shape (17920 = 512 x 35), us per
        // launch against the whole-tile variants: 32 rows 67.7 / 79.1, 16 rows 60.2 / 66.2, 8 rows 58.9 / 61.7
        int rpu = 0;
        if (g_tuning.gemm_ragged)
            for (int r = 33; r <= 48 && !rpu; ++r)
                if (a.N % (r * rs) == 0 && a.N / r <= 2 * n_cus() && a.N / r >= 2 * n_cus() - n_cus() / 4) rpu = r;
        if (rpu) {
            a.rows_per_unit = rpu;
            if (a.M <= 16) mfma_kernel<1, 6, EPI, 64, true><<<dim3(a.N / rpu), dim3(256), 0, s>>>(a);
            else           mfma_kernel<2, 6, EPI, 64, true><<<dim3(a.N / rpu), dim3(256), 0, s>>>(a);
        } else if (four) {
            if (a.M <= 16) mfma_kernel<1, 4, EPI, 64><<<dim3(groups2), dim3(256), 0, s>>>(a);
            else           mfma_kernel<2, 4, EPI, 64><<<dim3(groups2), dim3(256), 0, s>>>(a);
        } else if (a.M <= 16)
            mfma_kernel<1, 2, EPI><<<dim3(n_tiles16), dim3(256), 0, s>>>(a);
        else
            mfma_kernel<2, 2, EPI><<<dim3(n_tiles16), dim3(256), 0, s>>>(a);
    } else if (four) {
        if (a.M <= 16) mfma_kernel<1, 4, EPI, 64><<<dim3(groups4), dim3(256), 0, s>>>(a);
        else           mfma_kernel<2, 4, EPI, 64><<<dim3(groups4), dim3(256), 0, s>>>(a);
    } else {
        // two tiles per workgroup (X is then re-read from L2 once per two tiles) while that still leaves every
        // CU more than one workgroup; L2 -> L1 traffic, not HBM, is what limits this kernel
        const bool two = n_tiles16 / 2 >= n_cus() + n_cus() / 2;
        const int units = two ? groups2 : n_tiles16;
        if (a.M <= 16) {
            if (two) mfma_kernel<1, 2, EPI><<<dim3(units), dim3(256), 0, s>>>(a);
            else     mfma_kernel<1, 1, EPI><<<dim3(units), dim3(256), 0, s>>>(a);
        } else {
            if (two) mfma_kernel<2, 2, EPI><<<dim3(units), dim3(256), 0, s>>>(a);
            else     mfma_kernel<2, 1, EPI><<<dim3(units), dim3(256), 0, s>>>(a);
        }
    }
    return raven_host::check_launch("mfma gemm");
}

// Runs one GEMM over all M rows, in passes of at most 32 (MFMA) or 8 / 4 (vector) rows.
template <int EPI>
static int run_gemm(GemmArgs a, int dtype, hipStream_t s) {
    const size_t es = raven_host::elt_size(dtype);
    const bool mfma_ok = dtype == RAVEN_BF16 && a.K % 32 == 0 && a.k0 % 32 == 0 && a.N % 16 == 0;
    const int M = a.M;
    const size_t out_es = a.out_f32 ? 4 : es;
    for (int m0 = 0; m0 < M;) {
        const int left = M - m0;
        int pass;
        const int elts = 16 / (int)es;
        if (left == 1 && ((a.K / elts + 3) / 4 + 1 + 63) / 64 <= 9) {  // a single row: the K-split one-row kernel
            const char* x0 = static_cast<const char*>(a.x0) + (size_t)m0 * a.k0 * es;
            const char* x1 = a.x1 ? static_cast<const char*>(a.x1) + (size_t)m0 * a.k1 * es : nullptr;
            const char* res = a.residual ? static_cast<const char*>(a.residual) + (size_t)m0 * a.N * es : nullptr;
            char* y = static_cast<char*>(a.y) + (size_t)m0 * a.N * out_es;
            return raven_gemv_fused(x0, x1, nullptr, nullptr, nullptr, a.w, res, y, a.N, a.k0, a.k1, 0.f, EPI == EPI_SWIGLU, a.out_f32,
                                    dtype, s);
        }
        const bool use_mfma = mfma_ok && left >= g_tuning.gemm_mfma_min_rows;
        if (use_mfma) pass = left < 32 ? left : 32;
        else {
            pass = dtype == RAVEN_BF16 ? (left < 4 ? left : 4) : (left < 8 ? left : 8);
            // the vector kernel keeps its X rows in LDS: as many rows per pass (1, 2, 4 or 8) as fit
            const size_t row_bytes = (size_t)a.K * es;
            RAVEN_REQUIRE(row_bytes <= 160 * 1024, "gemm: one row of K=%d elements does not fit the 160 KB LDS", a.K);
            while (pass > 1 && (size_t)(pass <= 2 ? 2 : pass <= 4 ? 4 : 8) * row_bytes > 160 * 1024) pass = pass > 4 ? 4 : pass > 2 ? 2 : 1;
        }
        GemmArgs p = a;
        p.M = pass;
        p.x0 = static_cast<const char*>(a.x0) + (size_t)m0 * a.k0 * es;
        if (a.x1) p.x1 = static_cast<const char*>(a.x1) + (size_t)m0 * a.k1 * es;
        if (a.residual) p.residual = static_cast<const char*>(a.residual) + (size_t)m0 * a.N * es;
        p.y = static_cast<char*>(a.y) + (size_t)m0 * a.N * out_es;
        int rc;
        if (use_mfma) rc = dispatch_mfma<EPI>(p, s);
        else if (dtype == RAVEN_BF16) rc = dispatch_gemv<bf16, EPI>(p, s);
        else rc = dispatch_gemv<float, EPI>(p, s);
        if (rc != 0) return rc;
        m0 += pass;
    }
    return 0;
}

static int check_common(const char* who, int M, int N, int K, int dtype) {
    RAVEN_REQUIRE(dtype == RAVEN_F32 || dtype == RAVEN_BF16, "%s: unknown dtype %d", who, dtype);
    RAVEN_REQUIRE(M >= 0 && N > 0 && K > 0, "%s: bad shape M=%d N=%d K=%d", who, M, N, K);
    const int elts = 16 / (int)raven_host::elt_size(dtype);
    RAVEN_REQUIRE(K % elts == 0, "%s: K=%d must be a multiple of %d", who, K, elts);
    return 0;
}

}  // namespace raven

extern "C" int raven_set_tuning(const char* key, int32_t value) {
    using namespace raven;
    RAVEN_REQUIRE(key != nullptr, "set_tuning: null key");
    const std::string k(key);
    if (k == "gemv_units_per_wave") g_tuning.gemv_units_per_wave = value;
    else if (k == "gemv_interleave") g_tuning.gemv_interleave = value;
    else if (k == "gemv_nontemporal") g_tuning.gemv_nontemporal = value;
    else if (k == "gemv_wgs_per_cu") g_tuning.gemv_wgs_per_cu = value;
    else if (k == "linear_ks") g_linear_ks = value;
    else if (k == "gemm_four_tiles") g_tuning.gemm_four_tiles = value;
    else if (k == "gemm_ragged") g_tuning.gemm_ragged = value;
    else if (k == "gemm_mfma_min_rows" && value >= 2) g_tuning.gemm_mfma_min_rows = value;
    else if (k == "attn_split_target" && value > 0) g_attn_split_target = value;
    else if (k == "attn_big_grid" && value > 0) g_attn_big_grid = value;
    else if (k == "attn_wide") g_attn_wide = value;
    else if (k == "attn_prefetch" && value >= 0 && value <= 2) g_attn_prefetch = value;
    else if (k == "prefill_waves" && (value == 0 || value == 4 || value == 6)) g_prefill_waves = value;
    else if (k == "rope_tiled_rows" && value > 0) g_rope_tiled_rows = value;
    else if (k == "fuse_qkv_rope" && (value == 0 || value == 1)) g_fuse_qkv_rope = value;
    else if (k == "pad_chunk_rows" && (value == 0 || value == 1)) g_pad_chunk_rows = value;
    else if (k == "pad_decode_rows" && (value == 0 || value == 1)) g_pad_decode_rows = value;
    else if (k == "attn_nosplit_pairs" && value > 0 && value <= 1024) g_attn_nosplit_pairs = value;
    else if (k == "attn_nosplit_len" && value >= 0) g_attn_nosplit_len = value;
    else if (k == "linear_min_rows" && value >= 1) g_linear_min_rows = value;
    else if (k == "norm_early" && value >= -1 && value <= 1) g_norm_early = value;
    else if (k == "fuse_sums_norm" && (value == 0 || value == 1)) g_fuse_sums_norm = value;
    else if (k == "gemm_tiled_min_rows" && value >= 33) g_tiled_min_rows = value;
    else if (k == "gemm_tiled_variant" && value >= 0 && value <= 3) g_tiled_variant = value;
    else if (k == "gemm_tiled_split_tail" && (value == 0 || value == 1)) g_tiled_split_tail = value;
    else RAVEN_REQUIRE(set_gemv1_tuning(key, value) == 0, "set_tuning: unknown key %s", key);
    return 0;
}

extern "C" int raven_gemm(const void* x, const void* w, const void* residual, void* y, int32_t M, int32_t N, int32_t K,
                          int32_t dtype, int32_t out_f32, void* stream) {
    using namespace raven;
    if (int rc = check_common("gemm", M, N, K, dtype)) return rc;
    if (M == 0) return 0;
    RAVEN_REQUIRE(x && w && y, "gemm: null pointer");
    if (M >= g_tiled_min_rows && tiled_gemm_fits(M, N, K, 0, dtype))
        return tiled_gemm(x, nullptr, w, residual, y, M, N, K, 0, 0, out_f32, static_cast<hipStream_t>(stream));
    GemmArgs a{};
    a.w = w; a.x0 = x; a.x1 = nullptr; a.residual = residual; a.y = y;
    a.M = M; a.N = N; a.K = K; a.k0 = K; a.k1 = 0; a.out_f32 = out_f32;
    return run_gemm<EPI_PLAIN>(a, dtype, static_cast<hipStream_t>(stream));
}

extern "C" int raven_adapter_gemm_concat(const void* x0, const void* x1, const void* w, void* y, int32_t M, int32_t N,
                                         int32_t K0, int32_t K1, int32_t dtype, void* stream) {
    using namespace raven;
    if (int rc = check_common("adapter", M, N, K0 + K1, dtype)) return rc;
    if (M == 0) return 0;
    RAVEN_REQUIRE(x0 && x1 && w && y, "adapter: null pointer");
    const int elts = 16 / (int)raven_host::elt_size(dtype);
    RAVEN_REQUIRE(K0 > 0 && K1 > 0 && K0 % elts == 0 && K1 % elts == 0, "adapter: K0=%d, K1=%d must be positive multiples of %d", K0, K1, elts);
    if (M >= g_tiled_min_rows && tiled_gemm_fits(M, N, K0, K1, dtype))
        return tiled_gemm(x0, x1, w, nullptr, y, M, N, K0, K1, 0, 0, static_cast<hipStream_t>(stream));
    GemmArgs a{};
    a.w = w; a.x0 = x0; a.x1 = x1; a.residual = nullptr; a.y = y;
    a.M = M; a.N = N; a.K = K0 + K1; a.k0 = K0; a.k1 = K1; a.out_f32 = 0;
    return run_gemm<EPI_PLAIN>(a, dtype, static_cast<hipStream_t>(stream));
}

extern "C" int raven_gemm_swiglu(const void* x, const void* fc, void* out, int32_t M, int32_t I, int32_t K, int32_t dtype,
                                 void* stream) {
    using namespace raven;
    if (int rc = check_common("gemm_swiglu", M, I, K, dtype)) return rc;
    if (M == 0) return 0;
    RAVEN_REQUIRE(x && fc && out, "gemm_swiglu: null pointer");
    if (M >= g_tiled_min_rows && tiled_gemm_fits(M, I, K, 0, dtype))
        return tiled_gemm(x, nullptr, fc, nullptr, out, M, I, K, 0, 1, 0, static_cast<hipStream_t>(stream));
    GemmArgs a{};
    a.w = fc; a.x0 = x; a.x1 = nullptr; a.residual = nullptr; a.y = out;
    a.M = M; a.N = I; a.K = K; a.k0 = K; a.k1 = 0; a.out_f32 = 0;
    return run_gemm<EPI_SWIGLU>(a, dtype, static_cast<hipStream_t>(stream));
}

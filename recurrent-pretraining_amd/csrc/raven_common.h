// Device helpers shared by the gfx950 kernels: dtype traits, 16-byte vector access,
// wave64 reductions built on DPP row operations.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "raven_hip.h"

namespace raven {

typedef __bf16 bf16;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int kWave = 64;

// One 16-byte chunk of T: 8 bf16 or 4 floats.
template <typename T> struct Chunk;
template <> struct Chunk<float> {
    static constexpr int N = 4;
    float v[4];
};
template <> struct Chunk<bf16> {
    static constexpr int N = 8;
    bf16 v[8];
};

template <typename T>
__device__ __forceinline__ Chunk<T> load_chunk(const T* p) {
    Chunk<T> c;
    *reinterpret_cast<uint4*>(&c) = *reinterpret_cast<const uint4*>(p);
    return c;
}
// for data that is read once per launch: a load hinted to stream past the caches
template <typename T>
__device__ __forceinline__ Chunk<T> load_chunk_stream(const T* p) {
    typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
    Chunk<T> c;
    *reinterpret_cast<u32x4_t*>(&c) = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
    return c;
}
template <typename T>
__device__ __forceinline__ void store_chunk(T* p, const Chunk<T>& c) {
    *reinterpret_cast<uint4*>(p) = *reinterpret_cast<const uint4*>(&c);
}
template <typename T>
__device__ __forceinline__ Chunk<T> zero_chunk() {
    Chunk<T> c;
    *reinterpret_cast<uint4*>(&c) = make_uint4(0, 0, 0, 0);
    return c;
}

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(bf16 x) { return static_cast<float>(x); }
template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float x) { return static_cast<bf16>(x); }  // RNE

// round-trip through T: what storing an fp32 value in a T tensor and reading it back gives
template <typename T> __device__ __forceinline__ float round_to(float x) { return to_f32(from_f32<T>(x)); }

// dot of two 16-byte chunks, accumulated in fp32
__device__ __forceinline__ float dot_chunk(const Chunk<float>& a, const Chunk<float>& b, float acc) {
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_fmaf(a.v[i], b.v[i], acc);
    return acc;
}
__device__ __forceinline__ float dot_chunk(const Chunk<bf16>& a, const Chunk<bf16>& b, float acc) {
    const bf16x2* pa = reinterpret_cast<const bf16x2*>(&a);
    const bf16x2* pb = reinterpret_cast<const bf16x2*>(&b);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_fdot2_f32_bf16(pa[i], pb[i], acc, false);
    return acc;
}

// ---- DPP based reductions -------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// sum over each row of 16 lanes, result in all 16 lanes
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_f<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_f<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_f<0x141>(v);  // row_half_mirror
    v += dpp_f<0x140>(v);  // row_mirror
    return v;
}
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_f<0xB1>(v));
    v = fmaxf(v, dpp_f<0x4E>(v));
    v = fmaxf(v, dpp_f<0x141>(v));
    v = fmaxf(v, dpp_f<0x140>(v));
    return v;
}
// sum over the 64 lanes of a wave, result in all lanes
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
    v = row16_max(v);
    v = fmaxf(v, __shfl_xor(v, 16, 64));
    v = fmaxf(v, __shfl_xor(v, 32, 64));
    return v;
}

// x * sigmoid(x).  The reciprocal is the hardware's (1 ulp): its error vanishes in the bf16 rounding that follows and stays
// inside the fp32 bar, and a true division costs five times the instructions in the SwiGLU epilogue of a 256 x 256 tile.
__device__ __forceinline__ float silu_f32(float x) { return x * __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }

// One RoPE pair, adjacent elements (recpre/raven_modeling_minimal.py:118-131): products and sums rounded one by one in
// fp32, as the reference's separate elementwise kernels do; every kernel that rotates uses this one function, so that
// the fused and the two-launch paths write the same bits.
template <typename T>
__device__ __forceinline__ void rope_pair(T& a, T& b, float cs, float sn) {
#pragma clang fp contract(off)
    const float x0 = to_f32(a), x1 = to_f32(b);
    const float r0 = x0 * cs - x1 * sn;
    const float r1 = x1 * cs + x0 * sn;
    a = from_f32<T>(r0);
    b = from_f32<T>(r1);
}

}  // namespace raven

// ---- host side ------------------------------------------------------------------------------
namespace raven_host {
void set_error(const char* fmt, ...);
int  check_launch(const char* what);
inline size_t elt_size(int dtype) { return dtype == RAVEN_BF16 ? 2 : 4; }
inline size_t align_up(size_t x, size_t a = 256) { return (x + a - 1) / a * a; }
}  // namespace raven_host

#define RAVEN_REQUIRE(cond, ...)                 \
    do {                                         \
        if (!(cond)) {                           \
            raven_host::set_error(__VA_ARGS__);  \
            return -1;                           \
        }                                        \
    } while (0)

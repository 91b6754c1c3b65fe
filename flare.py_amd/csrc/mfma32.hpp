// Helpers shared by the kernels on v_mfma_f32_32x32x16_bf16 (forward: mixer_mfma32.hip, backward: mixer_bwd_mfma32.hip).
// Operand conventions of the 32x32x16 product (c32 = lane % 32, g2 = lane / 32):
//   A (32 x 16): lane holds row c32,    k-slots 8 g2 .. 8 g2 + 7
//   B (16 x 32): lane holds column c32, k-slots 8 g2 .. 8 g2 + 7
//   D (32 x 32): lane holds column c32, register r = 4 j + i holds row 8 j + 4 g2 + i
#pragma once

#include <type_traits>

#include "common.hpp"

namespace flare {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// range of an unshifted softmax denominator that proves no exponential overflowed or lost the terms that
// matter to underflow (2^-60 .. 2^120)
constexpr float kLMin = 8.6736174e-19f, kLMax = 1.329228e36f;

__device__ __forceinline__ f32x16 mma32(u32x4 a, u32x4 b, f32x16 c)
{
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

// c + (sum of the four bf16 values the lane holds in p), in every register of the result
__device__ __forceinline__ f32x4 lane_sum4(u32x2 p, f32x4 c)
{
    const s16x4 ones = {0x3f80, 0x3f80, 0x3f80, 0x3f80};
    return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(ones, __builtin_bit_cast(s16x4, p), c, 0, 0, 0);
}

__device__ __forceinline__ uint32_t pack2(float lo, float hi)
{
    bf16x2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
}

__device__ __forceinline__ float dot2_ones(uint32_t pk, float acc)
{
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, pk), __builtin_bit_cast(bf16x2, 0x3f803f80u), acc, false);
}

__device__ __forceinline__ u32x4 zero4() { return u32x4{0u, 0u, 0u, 0u}; }
__device__ __forceinline__ f32x16 zero16()
{
    return f32x16{0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
}

__device__ __forceinline__ u32x4 load16(const void* p) { return *reinterpret_cast<const u32x4*>(p); }
__device__ __forceinline__ u32x4 load16_stream(const void* p)
{
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}

// multiply 8 packed bf16 by f (fp32) and repack
__device__ __forceinline__ u32x4 scale8(u32x4 v, float f)
{
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float lo = __uint_as_float(v[i] << 16) * f;
        const float hi = __uint_as_float(v[i] & 0xffff0000u) * f;
        o[i] = uint32_t(f32_to_bf16_bits(lo)) | (uint32_t(f32_to_bf16_bits(hi)) << 16);
    }
    return o;
}

// exponentials of the four scores of quarter Q of a tile ...
template <int Q> __device__ __forceinline__ f32x4 exp_quarter(const f32x16& s)
{
    return f32x4{fast_exp2(s[4 * Q]), fast_exp2(s[4 * Q + 1]), fast_exp2(s[4 * Q + 2]), fast_exp2(s[4 * Q + 3])};
}
// ... and their pack into the two registers they occupy in the B operands of the value product
template <int Q> __device__ __forceinline__ void pack_quarter(f32x4 e, u32x4 (&p)[2])
{
    p[Q >> 1][2 * (Q & 1)] = pack2(e[0], e[1]);
    p[Q >> 1][2 * (Q & 1) + 1] = pack2(e[2], e[3]);
}
// The order of a pipeline quarter is fixed by hand: matrix product, four exponentials (which cover its 32 cycles
// in the matrix pipe), the 4x4x4 denominator product, two packs.  The fences keep the compiler's scheduler from
// putting two matrix instructions next to each other, where the second one would stall its wave.
#define FLARE_FENCE() __builtin_amdgcn_sched_barrier(0)

// f(integral_constant<int, I>) for I = I0 .. N - 1, unrolled at compile time
template <int I, int N, typename F> __device__ __forceinline__ void static_for(F& f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// LDS transpose read: the 16 lanes of a group each name 8 bytes (4 elements) of a row-major tile; lane i of
// the group receives element i of the four 16-element rows named by lane quads 0..3.
__device__ __forceinline__ u32x2 lds_read_tr16(const void* lds_addr)
{
    typedef s16x4 __attribute__((address_space(3))) * lds_ptr_t;
    asm volatile("" ::: "memory");
    const s16x4 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr_t)(uintptr_t)lds_addr);
    asm volatile("" ::: "memory");
    return __builtin_bit_cast(u32x2, r);
}

__device__ __forceinline__ float max16(const f32x16& s)
{
    float m = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])), fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
    return fmaxf(m, fmaxf(fmaxf(fmaxf(s[8], s[9]), fmaxf(s[10], s[11])), fmaxf(fmaxf(s[12], s[13]), fmaxf(s[14], s[15]))));
}

}  // namespace

}  // namespace flare

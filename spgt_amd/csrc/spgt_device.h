// Device-side helpers shared by the gfx950 kernels of this library.
//
// Everything here assumes wave64 (CDNA) and is only ever compiled for gfx950.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace spgt {

typedef float v2f __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
// 4-byte aligned vector types for rows of [d, S] tensors with odd S (see f2u / f4u below)
typedef v2f v2f_a4 __attribute__((aligned(4)));
typedef v4f v4f_a4 __attribute__((aligned(4)));

// 4-byte aligned vector views: rows of a [d, S] tensor with odd S start at
// arbitrary 4-byte offsets, and the hardware handles unaligned dwordx2/x4
// global accesses, so the compiler is told only what is true.
struct __attribute__((packed, aligned(4))) f2u { float x, y; };
struct __attribute__((packed, aligned(4))) f4u { float x, y, z, w; };

// DPP controls (a DPP row = 16 consecutive lanes).
#define SPGT_DPP_QUAD_XOR1 0xB1         // quad_perm:[1,0,3,2]
#define SPGT_DPP_QUAD_XOR2 0x4E         // quad_perm:[2,3,0,1]
#define SPGT_DPP_ROW_HALF_MIRROR 0x141  // lane i <-> 7-i inside each 8 lanes
#define SPGT_DPP_ROW_MIRROR 0x140       // lane i <-> 15-i inside each 16 lanes
#define SPGT_DPP_ROW_ROR8 0x128         // rotate by 8 inside each 16 lanes: lane i <-> i^8

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// Sum over the 16 lanes of a DPP row; every lane of the row receives the same
// bit pattern (each step adds a value to its mirror image, and fp add commutes).
__device__ __forceinline__ float row16_allsum(float v) {
    v += dpp_move<SPGT_DPP_QUAD_XOR1>(v);
    v += dpp_move<SPGT_DPP_QUAD_XOR2>(v);
    v += dpp_move<SPGT_DPP_ROW_HALF_MIRROR>(v);
    v += dpp_move<SPGT_DPP_ROW_MIRROR>(v);
    return v;
}

// The same sum for N independent values, one DPP step at a time across all of
// them: a DPP result needs two wait states before its consumer, and stepping the
// values in lock-step fills those slots with the neighbours' steps.
template <int N>
__device__ __forceinline__ void row16_allsum_n(float (&v)[N]) {
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] += dpp_move<SPGT_DPP_QUAD_XOR1>(v[i]);
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] += dpp_move<SPGT_DPP_QUAD_XOR2>(v[i]);
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] += dpp_move<SPGT_DPP_ROW_HALF_MIRROR>(v[i]);
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] += dpp_move<SPGT_DPP_ROW_MIRROR>(v[i]);
}

// Sum over groups of 8 consecutive lanes (same guarantee as above).
__device__ __forceinline__ float row8_allsum(float v) {
    v += dpp_move<SPGT_DPP_QUAD_XOR1>(v);
    v += dpp_move<SPGT_DPP_QUAD_XOR2>(v);
    v += dpp_move<SPGT_DPP_ROW_HALF_MIRROR>(v);
    return v;
}

// Sum of one value over the four 16-lane rows of a wave (lanes l, l^16, l^32, l^48).
__device__ __forceinline__ float rows4_allsum(float v) {
    v += __shfl_xor(v, 16, 64);
    v += __shfl_xor(v, 32, 64);
    return v;
}

// D(16x16) += A(16x4) * B(4x16), fp32.
//   lane l supplies A[l%16][l/16] and B[l/16][l%16];
//   lane l, element r of the result holds D[4*(l/16)+r][l%16].
__device__ __forceinline__ v4f mfma16(float a, float b, v4f c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
}

// D(32x32) += A(32x2) * B(2x32), fp32.
//   lane l supplies A[l%32][l/32] and B[l/32][l%32];
//   lane l, element r holds D[8*(r/4) + 4*(l/32) + r%4][l%32].
__device__ __forceinline__ v16f mfma32(float a, float b, v16f c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

// Streaming (touch-once) global accesses: NT selects the non-temporal form.
template <bool NT>
__device__ __forceinline__ float2 ld_stream(const float2* p) {
    if (NT) {
        const v2f v = __builtin_nontemporal_load(reinterpret_cast<const v2f*>(p));
        return make_float2(v.x, v.y);
    }
    return *p;
}
template <bool NT>
__device__ __forceinline__ float4 ld_stream(const float4* p) {
    if (NT) {
        const v4f v = __builtin_nontemporal_load(reinterpret_cast<const v4f*>(p));
        return make_float4(v.x, v.y, v.z, v.w);
    }
    return *p;
}
template <bool NT>
__device__ __forceinline__ void st_stream(float2* p, float2 v) {
    if (NT)
        __builtin_nontemporal_store(v2f{v.x, v.y}, reinterpret_cast<v2f*>(p));
    else
        *p = v;
}
template <bool NT>
__device__ __forceinline__ void st_stream(float4* p, float4 v) {
    if (NT)
        __builtin_nontemporal_store(v4f{v.x, v.y, v.z, v.w}, reinterpret_cast<v4f*>(p));
    else
        *p = v;
}

__host__ __device__ __forceinline__ int ceil_div(int a, int b) { return (a + b - 1) / b; }
__host__ __device__ __forceinline__ int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace spgt

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

// Rows [lo, hi) of an [H_all, W_all] plane that lie outside two row windows (at most three spans).
struct SpecSpans {
    int lo[3], hi[3];
    int n;
};

inline SpecSpans rows_outside_windows(int H_all, int H_low, int H_base_1, int H_base_2) {
    SpecSpans spans{};
    const int lo1 = H_base_1 < H_base_2 ? H_base_1 : H_base_2;
    const int lo2 = H_base_1 < H_base_2 ? H_base_2 : H_base_1;
    const int edges[4] = {lo1, lo1 + H_low, lo2, lo2 + H_low};
    int cursor = 0;
    for (int e = 0; e < 4; e += 2) {
        if (edges[e] > cursor) {
            spans.lo[spans.n] = cursor;
            spans.hi[spans.n] = edges[e];
            ++spans.n;
        }
        cursor = cursor > edges[e + 1] ? cursor : edges[e + 1];
    }
    if (cursor < H_all) {
        spans.lo[spans.n] = cursor;
        spans.hi[spans.n] = H_all;
        ++spans.n;
    }
    return spans;
}

// Stores zeros to out[lo, hi) (complex elements) with all 256 threads of a workgroup: 16-byte stores between an
// 8-byte head and tail.
__device__ __forceinline__ void zero_complex_range(float2* __restrict__ out, int64_t lo, int64_t hi) {
    if (lo >= hi) return;
    if ((reinterpret_cast<uintptr_t>(out + lo) & 15u) != 0) {
        if (threadIdx.x == 0) out[lo] = make_float2(0.f, 0.f);
        ++lo;
    }
    const int64_t pairs = (hi - lo) >> 1;
    float4* o4 = reinterpret_cast<float4*>(out + lo);
    for (int64_t t = threadIdx.x; t < pairs; t += 256) o4[t] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (((hi - lo) & 1) && threadIdx.x == 0) out[hi - 1] = make_float2(0.f, 0.f);
}

// Zero fill of chunk c (of `chunks`) of the rows in `spans` of plane p: out [planes, H_all, W_all] complex.
__device__ __forceinline__ void zero_span_chunk(float2* __restrict__ out, const SpecSpans& spans, int64_t p, int c,
                                                int chunks, int64_t plane, int W_all) {
    int64_t total = 0;
    for (int s = 0; s < spans.n; ++s) total += (int64_t)(spans.hi[s] - spans.lo[s]) * W_all;
    const int64_t per = ((total + chunks - 1) / chunks + 1) & ~(int64_t)1;
    const int64_t a = c * per, b = total < a + per ? total : a + per;
    int64_t off = 0;
    for (int s = 0; s < spans.n; ++s) {  // the chunk's share of each span
        const int64_t len = (int64_t)(spans.hi[s] - spans.lo[s]) * W_all;
        const int64_t lo = a > off ? a : off, hi = b < off + len ? b : off + len;
        if (lo < hi) {
            const int64_t base = p * plane + (int64_t)spans.lo[s] * W_all - off;
            zero_complex_range(out, base + lo, base + hi);
        }
        off += len;
    }
}

// Zeroes, in plane p of out [planes, H_all, W_all] (complex), the elements of the window rows that lie in
// neither window: [h_base_k, h_base_k + m_h) x [w_base_k, w_base_k + m_w), k = 0, 1.  Wave v of the
// workgroup takes the row slots v, v + 4, ...; lanes run along w.
__device__ __forceinline__ void zero_window_row_remainders(float2* __restrict__ out, int64_t p, int64_t plane,
                                                           int W_all, int m_h, int m_w, int hb0, int wb0, int hb1,
                                                           int wb1) {
    const int lane = threadIdx.x & 63;
    float2* pl = out + p * plane;
    for (int slot = threadIdx.x >> 6; slot < 2 * m_h; slot += 4) {
        const int k0 = slot >= m_h;
        const int h = (k0 ? hb1 : hb0) + slot - k0 * m_h;
        const bool in0 = h >= hb0 && h < hb0 + m_h;
        const bool in1 = h >= hb1 && h < hb1 + m_h;
        if (k0 && in0) continue;  // counted with the first window's rows
        float2* orow = pl + (int64_t)h * W_all;
        for (int w = lane; w < W_all; w += 64) {
            const bool c0 = in0 && w >= wb0 && w < wb0 + m_w;
            const bool c1 = in1 && w >= wb1 && w < wb1 + m_w;
            if (!c0 && !c1) orow[w] = make_float2(0.f, 0.f);
        }
    }
}

// Dropout inside a kernel (the reference's F.dropout calls, on by default also in inference): the keep decision of
// element (row, column) of a site is an integer hash of (seed, site, row, column) compared with p * 2^32; kept values
// are scaled by 1 / (1 - p).  A row is a token of a [T, C] tensor or a plane (n, c) of an NCHW one, the column the
// position inside it; the row's base value is mixed once, an element costs one more mix.  The two seed words are read
// from device memory, so that a captured graph whose seed tensor is refilled by a generator kernel draws new masks
// on every replay.
__device__ __forceinline__ uint32_t dropout_mix(uint32_t h) {
    h ^= h >> 16;
    h *= 0x21f0aaadu;
    h ^= h >> 15;
    h *= 0x735a2d97u;
    h ^= h >> 15;
    return h;
}
struct DropoutSite {
    uint32_t base, threshold;
    float scale;
};
__device__ __forceinline__ uint32_t dropout_threshold(float p) {
    return p <= 0.f ? 0u : (uint32_t)fminf(p * 4294967296.0f, 4294967040.0f);
}
__device__ __forceinline__ DropoutSite dropout_site(const uint32_t* seed, uint32_t site, int64_t row, float p) {
    DropoutSite d;
    const uint32_t lo = (uint32_t)row, hi = (uint32_t)((uint64_t)row >> 32);
    d.base = dropout_mix(dropout_mix(seed[0] ^ (lo * 0x9e3779b1u)) ^ seed[1] ^ (hi * 0x85ebca77u) ^ (site * 0xc2b2ae3du));
    d.threshold = dropout_threshold(p);
    d.scale = p <= 0.f ? 1.f : 1.f / (1.f - p);
    return d;
}
__device__ __forceinline__ bool dropout_keep(const DropoutSite& d, uint32_t column) {
    return dropout_mix(d.base + column * 0x27d4eb2fu) >= d.threshold;
}
__device__ __forceinline__ float dropout_apply(const DropoutSite& d, uint32_t column, float v) {
    return dropout_keep(d, column) ? v * d.scale : 0.f;
}
// Site numbers of the kernels that drop (distinct, so that one seed may serve a whole forward).
enum { kDropSiteFc = 0, kDropSiteFfn = 1, kDropSiteBiasAct = 2, kDropSiteConvResample = 3, kDropSiteConcat = 4 };

__host__ __device__ __forceinline__ int ceil_div(int a, int b) { return (a + b - 1) / b; }
__host__ __device__ __forceinline__ int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace spgt

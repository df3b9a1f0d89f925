// Truncated DFT along the last grid axis of the FNO spectral layer, as MFMA products
// against a small table of twiddle factors.
//
// Sp_SpectralConv2D (network/sp_layer.py:136-152) keeps only modes kw < m of rfft2 and
// feeds irfft2 a spectrum that is zero elsewhere.  Along w that is, per grid row (n, h),
//   forward   Y[c, j] = sum_w x[w, c] * F[w, j]          j = (kw, re|im), 2m columns
//   inverse   y[w, o] = sum_j Fi[w, j] * U[o, j]
// with F[w, (kw, re|im)] = (cos, -sin)(2 pi kw w / r) / sqrt(r) and Fi the same scaled by
// c_kw (1 for kw = 0 and the Nyquist column, else 2): two skinny real products per row,
// both bound by the one pass over the [N, r, r, C] tensor.  The tables come from the
// caller (built once in fp64).
//
// One wave owns one (row, 32-channel block).  Forward: the table is the MFMA A operand
// (mode x w, from LDS), x rows are the B operand read straight from global memory (lanes
// along channels, 128-byte runs), the accumulator holds modes along registers and
// channels along lanes.  Inverse: the table is A (w x mode, from LDS), the row's 2m x 32
// coefficients stay in registers as B, and each accumulator row is a 128-byte run of the
// channels-last output.
#include "spgt_device.h"
#include "spgt_host.h"

namespace spgt {

// grid (workgroups), block 256; waves stride over the rows * C/32 (row, channel block) items.
// tab [2*ceil(r/2)][32 MB]: row w holds the m2 table entries of grid point w, zero elsewhere.
// Y [rows][C][m2], or planar [rows/r][m2][r][C].  CT = C when known at compile time (row offsets
// become immediates), 0 = any C.  MB = blocks of 32 table columns (m2 <= 32 MB): one accumulator per block,
// all fed by the same x operand (the host launches MB = 1; more than 32 columns go to dft_rows_forward_fold_k).
template <int CT, int MB>
__global__ __launch_bounds__(256) void dft_rows_forward_k(const float* __restrict__ x, const float* __restrict__ tab,
                                                          float* __restrict__ Y, int64_t rows, int r, int C_, int m2,
                                                          int planar) {
    extern __shared__ float ts[];  // a copy of `tab`
    const int C = CT ? CT : C_;
    const int KH = (r + 1) / 2;
    {
        // straight 16-byte copy, eight loads in flight per thread: one memory round trip for r <= 256
        const int total4 = 2 * KH * 8 * MB;
        const float4* src = reinterpret_cast<const float4*>(tab);
        float4* dst = reinterpret_cast<float4*>(ts);
        for (int e0 = threadIdx.x; e0 < total4; e0 += 256 * 8) {
            float4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                v[u] = (e0 + 256 * u < total4) ? src[e0 + 256 * u] : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (e0 + 256 * u < total4) dst[e0 + 256 * u] = v[u];
        }
    }
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const int tk = lane & 31;
    const int kh = lane >> 5;
    const int CB = C / 32;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    constexpr int TP = 64 * MB;                // table words per MFMA step (two grid points)
    const float* tl = ts + kh * 32 * MB + tk;  // step kk, column block mb reads tl[TP * kk + 32 * mb]
    constexpr int BK = 16;
    const int nfull = (KH - 1) / BK;  // batches whose steps all lie before the final one
    const int nb = nfull + 1;
    for (int64_t gw = (int64_t)blockIdx.x * 4 + wave; gw < rows * CB; gw += (int64_t)gridDim.x * 4) {
        const int64_t row = gw / CB;
        const int cb = (int)(gw % CB);
        // wave-uniform row base + 32-bit lane offset: step kk reads grid points 2kk (lanes 0-31) and 2kk+1
        const float* base = x + row * (int64_t)r * C;
        const uint32_t voff = (uint32_t)(kh * C + cb * 32 + tk);
        // the last step of an odd r would read point r: those lanes re-read point r-1 against a zero table row
        const uint32_t voff_tail = (uint32_t)(min(2 * (KH - 1) + kh, r - 1) * C + cb * 32 + tk);
        float xa[BK], ta[MB][BK], xb[BK], tb[MB][BK];
        v16f acc[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[mb][i] = 0.f;
        // Full batches read 2*BK grid points at compile-time offsets; the last batch holds the
        // remaining steps and the (possibly clamped) final one.
#define SPGT_DFT_FETCH_FULL(XV, TV, B)                                                   \
        {                                                                                \
            const float* xb_ = base + (int64_t)(B) * (2 * BK) * C;                       \
            const float* tb_ = tl + (B) * (TP * BK);                                     \
            _Pragma("unroll") for (int u = 0; u < BK; ++u) {                             \
                XV[u] = xb_[voff + (uint32_t)(2 * u * C)];                               \
                _Pragma("unroll") for (int mb = 0; mb < MB; ++mb) TV[mb][u] = tb_[TP * u + 32 * mb]; \
            }                                                                            \
        }
#define SPGT_DFT_FETCH_TAIL(XV, TV)                                                      \
        _Pragma("unroll") for (int u = 0; u < BK; ++u) {                                 \
            const int kk = nfull * BK + u;                                               \
            XV[u] = (kk < KH - 1) ? base[voff + (uint32_t)(2 * kk * C)] : base[voff_tail]; \
            _Pragma("unroll") for (int mb = 0; mb < MB; ++mb)                            \
                TV[mb][u] = tl[TP * min(kk, KH - 1) + 32 * mb];                          \
        }
#define SPGT_DFT_FETCH(XV, TV, B)                                                        \
        if ((B) < nfull) SPGT_DFT_FETCH_FULL(XV, TV, B) else { SPGT_DFT_FETCH_TAIL(XV, TV) }
#define SPGT_DFT_MUL(XV, TV, B)                                                          \
        if ((B) < nfull) {                                                               \
            _Pragma("unroll") for (int u = 0; u < BK; ++u)                               \
                _Pragma("unroll") for (int mb = 0; mb < MB; ++mb)                        \
                    acc[mb] = mfma32(TV[mb][u], XV[u], acc[mb]);                         \
        } else {                                                                         \
            _Pragma("unroll") for (int u = 0; u < BK; ++u)                               \
                if (nfull * BK + u < KH) {                                               \
                    _Pragma("unroll") for (int mb = 0; mb < MB; ++mb)                    \
                        acc[mb] = mfma32(TV[mb][u], XV[u], acc[mb]);                     \
                }                                                                        \
        }
        SPGT_DFT_FETCH(xa, ta, 0)
        for (int b = 0; b < nb; b += 2) {
            if (b + 1 < nb) { SPGT_DFT_FETCH(xb, tb, b + 1) }
            __builtin_amdgcn_sched_barrier(0);
            SPGT_DFT_MUL(xa, ta, b)
            __builtin_amdgcn_sched_barrier(0);
            if (b + 2 < nb) { SPGT_DFT_FETCH(xa, ta, b + 2) }
            __builtin_amdgcn_sched_barrier(0);
            if (b + 1 < nb) { SPGT_DFT_MUL(xb, tb, b + 1) }
            __builtin_amdgcn_sched_barrier(0);
        }
#undef SPGT_DFT_FETCH_FULL
#undef SPGT_DFT_FETCH_TAIL
#undef SPGT_DFT_FETCH
#undef SPGT_DFT_MUL
        // acc[mb][r] = Y[c = cb*32 + tk][j = 32*mb + 8*(r/4) + 4*kh + r%4]
        if (planar) {
            // Y[n][j][h][c] with row = n*r + h: every store is a 128-byte run along c
            const int64_t n = row / r;
            const int64_t h = row - n * r;
            float* yp = Y + (n * m2 * r + h) * (int64_t)C + cb * 32 + tk;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int j = 32 * mb + 8 * q + 4 * kh + e;
                        if (j < m2) yp[(int64_t)j * r * C] = acc[mb][4 * q + e];
                    }
        } else {
            float* yr = Y + (row * C + cb * 32 + tk) * (int64_t)m2;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int j = 32 * mb + 8 * q + 4 * kh + e;
                        if (j < m2) yr[j] = acc[mb][4 * q + e];
                    }
        }
    }
}

// The forward transform for 32 < 2m <= 64 table columns, with the grid row folded onto itself first:
// cos(2 pi kw (r - w) / r) = cos(2 pi kw w / r) and sin(..(r - w)..) = -sin(..w..), so with
//   xe[f] = x[f] + x[r - f],  xo[f] = x[f] - x[r - f]      f = 1 .. ceil(r/2) - 1
// (f = 0 and, for even r, f = r/2 stand alone) the real columns are sums of xe against the cosines and the
// imaginary columns sums of xo against the sines over F = floor(r/2) + 1 folded points: half the contraction
// length, one 32-column block each, i.e. half the MFMAs of the unfolded form with two column blocks.
// The LDS copy of the table holds row f as [32 real entries | 32 imaginary entries]; the real entries of the
// points that stand alone are halved (their xe is formed as x[f] + x[f]).  Sums run in a fixed order.
// V channels per lane (C % (32 V) == 0): a lane loads V consecutive channels of its grid point at once (a wave
// issues a quarter of the load instructions at V = 4, which is what bounds the V = 1 form at 128 channels) and
// component e of the piece feeds accumulator e, whose lane tk stands for channel V tk + e; one table entry from
// LDS serves the V MFMAs of a step.  V = 4 keeps 128 accumulator registers: one wave per SIMD.
// grid (workgroups), block 256, dynamic LDS 2 * ceil(F/2) * 64 floats; tab as for dft_rows_forward_k<CT, 2>.
template <int V>
struct FoldPiece;
template <>
struct FoldPiece<1> { typedef float type; };
template <>
struct FoldPiece<2> { typedef float2 type; };
template <>
struct FoldPiece<4> { typedef float4 type; };
__device__ __forceinline__ float fold_get(float v, int) { return v; }
__device__ __forceinline__ float fold_get(const float2& v, int e) { return e == 0 ? v.x : v.y; }
__device__ __forceinline__ float fold_get(const float4& v, int e) { return e == 0 ? v.x : e == 1 ? v.y : e == 2 ? v.z : v.w; }

template <int CT, int V>
__global__ __launch_bounds__(256) void dft_rows_forward_fold_k(const float* __restrict__ x,
                                                               const float* __restrict__ tab, float* __restrict__ Y,
                                                               int64_t rows, int r, int C_, int m2, int planar) {
    typedef typename FoldPiece<V>::type piece_t;
    extern __shared__ float ts[];
    const int C = CT ? CT : C_;
    const int F = r / 2 + 1;
    const int KHf = (F + 1) / 2;  // MFMA steps: two folded points each
    for (int e = threadIdx.x; e < 2 * KHf * 64; e += 256) {
        const int f = e >> 6, col = e & 63, kw = col & 31, part = col >> 5;
        float v = (f < F && 2 * kw + part < m2) ? tab[(int64_t)f * 64 + 2 * kw + part] : 0.f;
        if (part == 0 && (f == 0 || 2 * f == r)) v *= 0.5f;
        ts[e] = v;
    }
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const int tk = lane & 31;
    const int kh = lane >> 5;
    const int CB = C / (32 * V);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    constexpr int BK = V == 1 ? 16 : 8;
    const int nb = (KHf + BK - 1) / BK;
    for (int64_t gw = (int64_t)blockIdx.x * 4 + wave; gw < rows * CB; gw += (int64_t)gridDim.x * 4) {
        const int64_t row = gw / CB;
        const int cb = (int)(gw % CB);
        const float* base = x + row * (int64_t)r * C + cb * (32 * V) + tk * V;
        piece_t a0[BK], b0[BK], a1[BK], b1[BK];
        v16f acc_re[V], acc_im[V];
#pragma unroll
        for (int e = 0; e < V; ++e)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc_re[e][i] = acc_im[e][i] = 0.f;
        // steps past the last folded point read that point again (against zero table rows); the partner of
        // point 0 is point 0 itself
#define SPGT_FOLD_FETCH(AV, BV, B)                                                                   \
        _Pragma("unroll") for (int u = 0; u < BK; ++u) {                                              \
            const int f = min(2 * ((B) * BK + u) + kh, F - 1);                                        \
            AV[u] = *reinterpret_cast<const piece_t*>(base + (uint32_t)(f * C));                      \
            BV[u] = *reinterpret_cast<const piece_t*>(base + (uint32_t)((f == 0 ? 0 : r - f) * C));   \
        }
#define SPGT_FOLD_MUL(AV, BV, B)                                                                      \
        _Pragma("unroll") for (int u = 0; u < BK; ++u) {                                              \
            const int kk = (B) * BK + u;                                                              \
            if (kk < KHf) {                                                                           \
                const float* tr = ts + (2 * kk + kh) * 64 + tk;                                       \
                const float tre = tr[0], tim = tr[32];                                                \
                _Pragma("unroll") for (int e = 0; e < V; ++e) {                                       \
                    const float av = fold_get(AV[u], e), bv = fold_get(BV[u], e);                     \
                    acc_re[e] = mfma32(tre, av + bv, acc_re[e]);                                      \
                    acc_im[e] = mfma32(tim, av - bv, acc_im[e]);                                      \
                }                                                                                     \
            }                                                                                         \
        }
        SPGT_FOLD_FETCH(a0, b0, 0)
        for (int b = 0; b < nb; b += 2) {
            if (b + 1 < nb) { SPGT_FOLD_FETCH(a1, b1, b + 1) }
            __builtin_amdgcn_sched_barrier(0);
            SPGT_FOLD_MUL(a0, b0, b)
            __builtin_amdgcn_sched_barrier(0);
            if (b + 2 < nb) { SPGT_FOLD_FETCH(a0, b0, b + 2) }
            __builtin_amdgcn_sched_barrier(0);
            if (b + 1 < nb) { SPGT_FOLD_MUL(a1, b1, b + 1) }
            __builtin_amdgcn_sched_barrier(0);
        }
#undef SPGT_FOLD_FETCH
#undef SPGT_FOLD_MUL
        // acc_re[e][4q + i] = Re Y[c = cb*32V + V tk + e][kw = 8q + 4kh + i], acc_im the imaginary part:
        // columns 2kw, 2kw + 1
        if (planar) {
            const int64_t n = row / r;
            const int64_t h = row - n * r;
            float* yp = Y + (n * m2 * r + h) * (int64_t)C + cb * (32 * V) + tk * V;
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int j = 2 * (8 * q + 4 * kh + i);
                    if (j < m2) {
                        float* pre = yp + (int64_t)j * r * C;
                        float* pim = yp + (int64_t)(j + 1) * r * C;
                        if (V == 4) {
                            *reinterpret_cast<float4*>(pre) = make_float4(acc_re[0][4 * q + i], acc_re[1 % V][4 * q + i],
                                                                          acc_re[2 % V][4 * q + i], acc_re[3 % V][4 * q + i]);
                            *reinterpret_cast<float4*>(pim) = make_float4(acc_im[0][4 * q + i], acc_im[1 % V][4 * q + i],
                                                                          acc_im[2 % V][4 * q + i], acc_im[3 % V][4 * q + i]);
                        } else if (V == 2) {
                            *reinterpret_cast<float2*>(pre) = make_float2(acc_re[0][4 * q + i], acc_re[1 % V][4 * q + i]);
                            *reinterpret_cast<float2*>(pim) = make_float2(acc_im[0][4 * q + i], acc_im[1 % V][4 * q + i]);
                        } else {
                            pre[0] = acc_re[0][4 * q + i];
                            pim[0] = acc_im[0][4 * q + i];
                        }
                    }
                }
        } else {
#pragma unroll
            for (int e = 0; e < V; ++e) {
                float* yr = Y + (row * C + cb * (32 * V) + tk * V + e) * (int64_t)m2;
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int j = 2 * (8 * q + 4 * kh + i);
                        if (j < m2) {
                            yr[j] = acc_re[e][4 * q + i];
                            yr[j + 1] = acc_im[e][4 * q + i];
                        }
                    }
            }
        }
    }
}

// grid (workgroups), block 256; waves stride over the (row, channel block) items.
// tab [32*ceil(r/32)][m2 + 1]: row w holds the m2 table entries of grid point w, zero elsewhere.
// U [rows][C][m2] (or planar [rows/r][m2][r][C]) -> y [rows][r][C].  KMAX >= m2 / 2: MFMA steps held in registers.
template <int KMAX>
__global__ __launch_bounds__(256) void dft_rows_inverse_k(const float* __restrict__ U, const float* __restrict__ tab,
                                                          float* __restrict__ y, int64_t rows, int r, int C, int m2,
                                                          int planar) {
    extern __shared__ float ts[];  // [32 * ceil(r/32)][m2 + 1], zero beyond r rows: a copy of `tab`
    const int pitch = m2 + 1;
    const int WT = (r + 31) / 32;
    {
        const int total4 = WT * 32 * pitch / 4;  // 32 * pitch is a multiple of 4
        const float4* src = reinterpret_cast<const float4*>(tab);
        float4* dst = reinterpret_cast<float4*>(ts);
        for (int e0 = threadIdx.x; e0 < total4; e0 += 256 * 8) {
            float4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                v[u] = (e0 + 256 * u < total4) ? src[e0 + 256 * u] : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (e0 + 256 * u < total4) dst[e0 + 256 * u] = v[u];
        }
    }
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const int tk = lane & 31;
    const int kh = lane >> 5;
    const int CB = C / 32;
    for (int64_t gw = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); gw < rows * CB; gw += (int64_t)gridDim.x * 4) {
    const int64_t row = gw / CB;
    const int cb = (int)(gw % CB);
    // B operand: U[o = cb*32 + tk][j = 2kk + kh]
    float ureg[KMAX];
    if (planar) {
        const int64_t n = row / r;
        const int64_t h = row - n * r;
        const float* up = U + (n * m2 * r + h) * (int64_t)C + cb * 32 + tk;  // U[n][j][h][o]
#pragma unroll
        for (int kk = 0; kk < KMAX; ++kk) ureg[kk] = (2 * kk + kh < m2) ? up[(int64_t)(2 * kk + kh) * r * C] : 0.f;
    } else {
        const float* ur = U + (row * C + cb * 32 + tk) * (int64_t)m2;
#pragma unroll
        for (int kk = 0; kk < KMAX; ++kk) ureg[kk] = (2 * kk + kh < m2) ? ur[2 * kk + kh] : 0.f;
    }
    float* yr = y + row * (int64_t)r * C + cb * 32 + tk;
    const int KH = m2 / 2;
    for (int wt = 0; wt < WT; ++wt) {
        const float* ta = ts + (wt * 32 + tk) * pitch + kh;
        v16f acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
        for (int kk = 0; kk < KMAX; ++kk)
            if (kk < KH) acc = mfma32(ta[2 * kk], ureg[kk], acc);
        // acc[q] = y[w = wt*32 + 8*(q/4) + 4*kh + q%4][o = cb*32 + tk]
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            const int w = wt * 32 + 8 * (q >> 2) + 4 * kh + (q & 3);
            if (w < r) yr[(int64_t)w * C] = acc[q];
        }
    }
    }
}

// Everything between the two w-direction products of the spectral layer
// (network/sp_layer.py:136-151 restricted to the kept modes), in two launches:
//   Z[kh, c] = sum_h G[kh, h] Y[h, c]          forward DFT along h, 2m kept rows kh      } spectral_rows_contract_k
//   O[kh, o] = sum_c Z[kh, c] W[kh, kw, c, o]  complex contraction (network/layer.py:249-261) }
//   U[h, o]  = sum_kh Gi[h, kh] O[kh, o]       inverse DFT along h                        } spectral_rows_expand_k
// on planar operands Y [N][2m][r][Cin] and U [N][2m][r][Cout] (plane 2kw = real, 2kw+1 = imaginary).
// Lanes run along channels, so every global access is a 256-byte run; twiddle factors sit in LDS and
// are wave-uniform.  All loads of a phase are in flight together (the data is a few MB: the kernels
// are bound by memory round trips, not bandwidth), and every sum runs in a fixed order.
constexpr int kMidC = 64;     // output channels (lanes of the contraction's result)
constexpr int kMidRows = 3;   // kept rows kh per workgroup of the first kernel
constexpr int kMidHB = 32;    // grid rows h fetched per batch (per channel of a lane)

// grid (m, N, ceil(2m / kMidRows)), block 256.  O [N][m][2m][Cout] complex.
// CPL: input channels per lane (Cin <= 64 CPL): a lane forms Z for channels lane, lane + 64, ...
template <int CPL>
__global__ __launch_bounds__(256) void spectral_rows_contract_k(
    const float* __restrict__ Y, const float2* __restrict__ G, const float2* __restrict__ W1,
    const float2* __restrict__ W2, float2* __restrict__ O, int r, int Cin, int Cout, int m) {
    constexpr int MC = 64 * CPL;
    constexpr int HB = kMidHB / CPL;
    extern __shared__ float2 lds[];
    // [tab: kMidRows x r][part: 4 x kMidRows x MC]; part doubles as the per-c-quarter partial O
    float2* tab = lds;
    float2 (*part)[kMidRows][MC] = reinterpret_cast<float2 (*)[kMidRows][MC]>(lds + kMidRows * r);
    __shared__ float2 Zs[kMidRows][MC];
    const int m2 = 2 * m;
    const int kw = blockIdx.x;
    const int64_t n = blockIdx.y;
    const int kh0 = blockIdx.z * kMidRows;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    for (int e = threadIdx.x; e < kMidRows * r; e += 256) {
        const int q = e / r, h = e - q * r;
        tab[e] = (kh0 + q < m2) ? G[(int64_t)(kh0 + q) * r + h] : make_float2(0.f, 0.f);
    }
    __syncthreads();

    // Z = G Y: wave hq sums its quarter of h for the workgroup's rows; lane = input channel (+ 64 j)
    {
        const int hlen = (r + 3) / 4;
        const int h0 = wave * hlen;
        const int h1 = min(r, h0 + hlen);
        const float* yre = Y + ((n * m2 + 2 * kw) * r) * (int64_t)Cin;
        const float* yim = yre + (int64_t)r * Cin;
        int cj[CPL];
        bool cok[CPL];
#pragma unroll
        for (int j = 0; j < CPL; ++j) {
            cok[j] = lane + 64 * j < Cin;
            cj[j] = min(lane + 64 * j, Cin - 1);
        }
        float2 acc[kMidRows][CPL];
#pragma unroll
        for (int q = 0; q < kMidRows; ++q)
#pragma unroll
            for (int j = 0; j < CPL; ++j) acc[q][j] = make_float2(0.f, 0.f);
        for (int hb = h0; hb < h1; hb += HB) {
            float a[CPL][HB], b[CPL][HB];
#pragma unroll
            for (int u = 0; u < HB; ++u) {
                const int h = min(hb + u, h1 - 1);
#pragma unroll
                for (int j = 0; j < CPL; ++j) {
                    const float av = yre[(int64_t)h * Cin + cj[j]], bv = yim[(int64_t)h * Cin + cj[j]];
                    a[j][u] = cok[j] ? av : 0.f;
                    b[j][u] = cok[j] ? bv : 0.f;
                }
            }
#pragma unroll
            for (int u = 0; u < HB; ++u) {
                if (hb + u < h1) {
#pragma unroll
                    for (int q = 0; q < kMidRows; ++q) {
                        const float2 g = tab[q * r + hb + u];
#pragma unroll
                        for (int j = 0; j < CPL; ++j) {
                            acc[q][j].x = fmaf(g.x, a[j][u], acc[q][j].x);
                            acc[q][j].x = fmaf(-g.y, b[j][u], acc[q][j].x);
                            acc[q][j].y = fmaf(g.x, b[j][u], acc[q][j].y);
                            acc[q][j].y = fmaf(g.y, a[j][u], acc[q][j].y);
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int q = 0; q < kMidRows; ++q)
#pragma unroll
            for (int j = 0; j < CPL; ++j) part[wave][q][lane + 64 * j] = acc[q][j];
    }
    __syncthreads();
    for (int e = threadIdx.x; e < kMidRows * MC; e += 256) {
        const int q = e / MC, c = e % MC;
        const float2 p0 = part[0][q][c], p1 = part[1][q][c], p2 = part[2][q][c], p3 = part[3][q][c];
        Zs[q][c] = make_float2((p0.x + p1.x) + (p2.x + p3.x), (p0.y + p1.y) + (p2.y + p3.y));
    }
    __syncthreads();

    // O = Z . W: wave w takes input channels [w MC/4, (w + 1) MC/4) of every row, sixteen at a time; lane = output
    // channel
    {
        constexpr int CQ = MC / 4;
        const bool ook = lane < Cout;
        float2 o[kMidRows];
#pragma unroll
        for (int q = 0; q < kMidRows; ++q) o[q] = make_float2(0.f, 0.f);
#pragma unroll
        for (int c0 = 0; c0 < CQ; c0 += 16) {
            float2 wv[kMidRows][16];
#pragma unroll
            for (int q = 0; q < kMidRows; ++q) {
                const int kh = min(kh0 + q, m2 - 1);
                const float2* Wm = (kh < m ? W1 + ((int64_t)kh * m + kw) * Cin * Cout
                                           : W2 + ((int64_t)(kh - m) * m + kw) * Cin * Cout) + min(lane, Cout - 1);
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    const int c = wave * CQ + c0 + u;
                    const float2 wval = Wm[(int64_t)min(c, Cin - 1) * Cout];
                    wv[q][u] = (ook && c < Cin) ? wval : make_float2(0.f, 0.f);
                }
            }
#pragma unroll
            for (int q = 0; q < kMidRows; ++q) {
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    const float2 z = Zs[q][wave * CQ + c0 + u];
                    o[q].x = fmaf(z.x, wv[q][u].x, o[q].x);
                    o[q].x = fmaf(-z.y, wv[q][u].y, o[q].x);
                    o[q].y = fmaf(z.y, wv[q][u].x, o[q].y);
                    o[q].y = fmaf(z.x, wv[q][u].y, o[q].y);
                }
            }
        }
#pragma unroll
        for (int q = 0; q < kMidRows; ++q) part[wave][q][lane] = o[q];
    }
    __syncthreads();
    for (int e = threadIdx.x; e < kMidRows * kMidC; e += 256) {
        const int q = e / kMidC, o = e % kMidC;
        if (kh0 + q < m2 && o < Cout) {
            const float2 p0 = part[0][q][o], p1 = part[1][q][o], p2 = part[2][q][o], p3 = part[3][q][o];
            O[((n * m + kw) * m2 + kh0 + q) * (int64_t)Cout + o] =
                make_float2((p0.x + p1.x) + (p2.x + p3.x), (p0.y + p1.y) + (p2.y + p3.y));
        }
    }
}

// grid (m, N, chunks of h), block 256.  LPR = 64: wave w of a workgroup takes rows h = h0 + w, h0 + w + 4, ...
// with a lane per output channel; LPR = 32 (Cout <= 32): each half of a wave takes a row of its own.
// KHMAX >= 2m: kept rows held in registers.
template <int KHMAX, int LPR>
__global__ __launch_bounds__(256) void spectral_rows_expand_k(
    const float2* __restrict__ O, const float2* __restrict__ Gi, float* __restrict__ U, int r, int Cout, int m,
    int rows_per_wg) {
    extern __shared__ float2 lds[];  // Gi rows of the chunk: [rows_per_wg][2m]
    constexpr int RPW = 64 / LPR;    // rows a wave works on at a time
    const int m2 = 2 * m;
    const int kw = blockIdx.x;
    const int64_t n = blockIdx.y;
    const int h0 = blockIdx.z * rows_per_wg;
    const int h1 = min(r, h0 + rows_per_wg);
    const int lane = threadIdx.x & 63;
    const int o = lane % LPR;
    const int sub = lane / LPR;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    for (int e = threadIdx.x; e < (h1 - h0) * m2; e += 256) lds[e] = Gi[(int64_t)h0 * m2 + e];
    // the mode's O[kh][o] for all kept rows stays in registers
    float2 ov[KHMAX];
    const float2* Om = O + ((n * m + kw) * m2) * (int64_t)Cout + o;
#pragma unroll
    for (int kh = 0; kh < KHMAX; ++kh) ov[kh] = (kh < m2 && o < Cout) ? Om[(int64_t)kh * Cout] : make_float2(0.f, 0.f);
    __syncthreads();
    float* ure = U + ((n * m2 + 2 * kw) * r) * (int64_t)Cout + o;
    float* uim = ure + (int64_t)r * Cout;
    for (int hb = h0 + wave * RPW; hb < h1; hb += 4 * RPW) {
        const int h = hb + sub;
        const float2* g = lds + (min(h, h1 - 1) - h0) * m2;
        float2 acc = make_float2(0.f, 0.f);
#pragma unroll
        for (int kh = 0; kh < KHMAX; ++kh) {
            if (kh < m2) {
                acc.x = fmaf(g[kh].x, ov[kh].x, acc.x);
                acc.x = fmaf(-g[kh].y, ov[kh].y, acc.x);
                acc.y = fmaf(g[kh].x, ov[kh].y, acc.y);
                acc.y = fmaf(g[kh].y, ov[kh].x, acc.y);
            }
        }
        if (o < Cout && h < h1) {
            ure[(int64_t)h * Cout] = acc.x;
            uim[(int64_t)h * Cout] = acc.y;
        }
    }
}

// The end of Sp_SpectralConv2D.forward (network/sp_layer.py:132, 149-155) in one pass over the grid:
//   out[row, w, o] = act( sum_c x[row, w, c] W[c, o] + bias[o] + sum_j table[w, j] U[row, o, j] )
// i.e. the residual Linear, the inverse DFT along w of the retained modes, their sum and the activation;
// the inverse transform's result never goes to memory.  CIN = 32, 64 or 128 channels in, COUT = 32 or 64 out,
// planar U [N][2m][r][COUT].
// Both terms are MFMA products with output channels along the accumulator's registers and grid points along
// its lanes (so a lane stores 16-byte pieces of its grid point's row): A = W resp. U in registers,
// B = x tile (from a wave-private LDS tile, 16-byte reads, lane (w, kh) takes channels kh*C/2 + kk) resp.
// table entries (handed over in operand order, tabA[tile][kk][lane] = table[32 tile + lane%32][2kk +
// lane/32], zero outside).  No barriers.
// One wave per SIMD (waves that share a SIMD's matrix pipe run their MFMAs at about half the rate of a lone
// wave; with four waves per SIMD and a wave per half of the channels this pass took 44 us at [4, 211, 211, 64],
// with two fatter waves 43-51 us, with one 34 us): a wave makes all channels of a 32-point tile (for C = 64 two
// independent accumulator chains off the same x and table operands), and takes a run of consecutive (grid row,
// tile) pairs (the runs of the 4 * gridDim.x waves differ by at most one pair), so that a row's U is fetched once
// per run and row.  Per pair: the parked x rows go to the wave's LDS tile; U when the row changes, this pair's
// table entries and the next pair's x rows are requested (wave-uniform base + 32-bit lane offsets, computed once
// for U); then the 64 MFMAs of the Linear, the MFMAs of the inverse transform, activation and stores.  Stores
// are unconditional: points
// past the end of a grid row are computed from the row's last point and that point's table entries, and write
// its own values to its address.
// KSU: MFMA steps of the inverse transform, modes rounded up (the table entries of the steps past the modes are
// zero); a template parameter so that neither the loads nor the MFMAs sit behind branches.  TS: steps per tile in
// the operand table.  CIN: input channels of the Linear (32, 64 or 128; a lane's contraction channels are
// kh * CIN/2 + kk), COUT: channels of U and of the result (32 or 64).
// grid (min(ceil(pairs / 4), CUs)), block 256, dynamic LDS 4 * 32 * (CIN + 4) floats.
template <int ACT, int KSU, int CIN, int COUT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void spectral_inverse_linear_k(
    const float* __restrict__ U, const float* __restrict__ tabA, const float* __restrict__ x,
    const float* __restrict__ Wkn, const float* __restrict__ bias, float* __restrict__ out, int r, int m2,
    unsigned pairs) {
    constexpr int PX = CIN + 4;
    constexpr int NCB = COUT / 32;   // blocks of 32 output channels, one accumulator chain each
    constexpr int KL = CIN / 2;      // contraction channels of the Linear per lane (MFMA steps)
    constexpr int LPR = CIN / 4;     // lanes per grid point when a tile is fetched in 16-byte pieces
    constexpr int NP = CIN / 8;      // such pieces per lane and tile
    constexpr int TS = KSU <= 16 ? 16 : 32;
    static_assert(CIN == 32 || CIN == 64 || CIN == 128, "32, 64 or 128 input channels");
    static_assert(COUT == 32 || COUT == 64, "32 or 64 output channels");
    static_assert(KSU % 4 == 0 && KSU >= 4 && KSU <= 32, "4 .. 32 steps in fours");
    extern __shared__ __attribute__((aligned(16))) float xs_all[];  // [4 waves][32 * PX]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tk = lane & 31;
    const int kh = lane >> 5;
    const unsigned WT = (unsigned)(r + 31) / 32;

    float wreg0[KL], wreg1[KL];  // W[c = kh*KL + kk][o = cb*32 + tk], cb = 0, 1
#pragma unroll
    for (int kk = 0; kk < KL; ++kk) {
        wreg0[kk] = Wkn[(kh * KL + kk) * COUT + tk];
        wreg1[kk] = NCB == 2 ? Wkn[(kh * KL + kk) * COUT + (NCB - 1) * 32 + tk] : 0.f;
    }
    // bias in accumulator layout (element 4q + e of half cb belongs to channel cb*32 + 8q + 4kh + e): the C operand
    // of a pair's first MFMAs
    v16f bo0, bo1;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
        const float4 b0 = bias ? *reinterpret_cast<const float4*>(bias + 8 * q + 4 * kh) : z;
        const float4 b1 = (bias && NCB == 2) ? *reinterpret_cast<const float4*>(bias + (NCB - 1) * 32 + 8 * q + 4 * kh) : z;
        bo0[4 * q + 0] = b0.x; bo0[4 * q + 1] = b0.y; bo0[4 * q + 2] = b0.z; bo0[4 * q + 3] = b0.w;
        bo1[4 * q + 0] = b1.x; bo1[4 * q + 1] = b1.y; bo1[4 * q + 2] = b1.z; bo1[4 * q + 3] = b1.w;
    }
    // lane offsets of U[n][j = 2kk + kh][h][o = tk] from U[n][0][h][0]; steps past the modes read the last mode
    // (finite values that meet zero table entries)
    uint32_t uoff[KSU];
#pragma unroll
    for (int kk = 0; kk < KSU; ++kk) uoff[kk] = (uint32_t)min(2 * kk + kh, m2 - 1) * (uint32_t)(r * COUT) + (uint32_t)tk;
    float* const xw = xs_all + wave * (32 * PX);

    // (named registers and macros: a register array that lives across the loop ends up in scratch memory)
    // piece I of a tile is grid point (lane + 64 I) / LPR, channels 4 (lane % LPR) ..; points past the end of the
    // grid row read its last point
    float4 s0, s1, s2, s3, s4, s5, s6, s7, s8, s9, s10, s11, s12, s13, s14, s15;
#define SPGT_X_PIECE(BASE_, W0_, I_) \
    (*reinterpret_cast<const float4*>((BASE_) + (uint32_t)(min((W0_) + ((lane + 64 * (I_)) / LPR), r - 1) * CIN + 4 * (lane % LPR))))
#define SPGT_LOAD_X_TILE(T_)                                                                        \
    {                                                                                               \
        const unsigned row_ = (T_) / WT;                                                            \
        const int w0_ = (int)((T_) - row_ * WT) * 32;                                               \
        const float* xb_ = x + (int64_t)row_ * r * CIN;                                             \
        s0 = SPGT_X_PIECE(xb_, w0_, 0); s1 = SPGT_X_PIECE(xb_, w0_, 1); s2 = SPGT_X_PIECE(xb_, w0_, 2); \
        s3 = SPGT_X_PIECE(xb_, w0_, 3);                                                             \
        if (NP >= 8) {                                                                              \
            s4 = SPGT_X_PIECE(xb_, w0_, 4); s5 = SPGT_X_PIECE(xb_, w0_, 5);                         \
            s6 = SPGT_X_PIECE(xb_, w0_, 6); s7 = SPGT_X_PIECE(xb_, w0_, 7);                         \
        }                                                                                           \
        if (NP >= 16) {                                                                             \
            s8 = SPGT_X_PIECE(xb_, w0_, 8); s9 = SPGT_X_PIECE(xb_, w0_, 9);                         \
            s10 = SPGT_X_PIECE(xb_, w0_, 10); s11 = SPGT_X_PIECE(xb_, w0_, 11);                     \
            s12 = SPGT_X_PIECE(xb_, w0_, 12); s13 = SPGT_X_PIECE(xb_, w0_, 13);                     \
            s14 = SPGT_X_PIECE(xb_, w0_, 14); s15 = SPGT_X_PIECE(xb_, w0_, 15);                     \
        }                                                                                           \
    }
#define SPGT_STORE_X_PIECE(I_, V_) \
    *reinterpret_cast<float4*>(xw + ((lane + 64 * (I_)) / LPR) * PX + 4 * (lane % LPR)) = V_;
    s4 = s5 = s6 = s7 = s8 = s9 = s10 = s11 = s12 = s13 = s14 = s15 = make_float4(0.f, 0.f, 0.f, 0.f);
    // a wave takes a run of consecutive pairs (runs differ by at most one pair): the tiles of a grid row follow
    // each other, and the row's U stays in registers until the row changes
    const unsigned waves = gridDim.x * 4, wi = blockIdx.x * 4 + wave;
    const unsigned per = pairs / waves, extra = pairs % waves;
    unsigned t = wi * per + min(wi, extra);
    const unsigned t_end = t + per + (wi < extra ? 1u : 0u);
    typedef float vKf __attribute__((ext_vector_type(KSU)));
    vKf ureg0, ureg1;
    unsigned u_row = ~0u;
    if (t < t_end) SPGT_LOAD_X_TILE(t)
    for (; t < t_end; ++t) {
        const unsigned row = t / WT;
        const int wt = (int)(t - row * WT);
        SPGT_STORE_X_PIECE(0, s0) SPGT_STORE_X_PIECE(1, s1) SPGT_STORE_X_PIECE(2, s2) SPGT_STORE_X_PIECE(3, s3)
        if (NP >= 8) {
            SPGT_STORE_X_PIECE(4, s4) SPGT_STORE_X_PIECE(5, s5) SPGT_STORE_X_PIECE(6, s6) SPGT_STORE_X_PIECE(7, s7)
        }
        if (NP >= 16) {
            SPGT_STORE_X_PIECE(8, s8) SPGT_STORE_X_PIECE(9, s9) SPGT_STORE_X_PIECE(10, s10) SPGT_STORE_X_PIECE(11, s11)
            SPGT_STORE_X_PIECE(12, s12) SPGT_STORE_X_PIECE(13, s13) SPGT_STORE_X_PIECE(14, s14) SPGT_STORE_X_PIECE(15, s15)
        }
        // (the widest shape has no registers to spare for that and fetches U for every pair)
        constexpr bool KEEP_U = !(KSU == 32 && CIN == 128 && COUT == 64);
        if (!KEEP_U || row != u_row) {
            u_row = row;
            const unsigned n = row / (unsigned)r;
            const unsigned h = row - n * (unsigned)r;
            const float* ub = U + ((int64_t)n * m2 * r + h) * COUT;  // U[n][0][h][0]
#pragma unroll
            for (int kk = 0; kk < KSU; ++kk) {
                ureg0[kk] = ub[uoff[kk]];
                ureg1[kk] = NCB == 2 ? ub[uoff[kk] + (uint32_t)((NCB - 1) * 32)] : 0.f;
            }
        }
        // the operand table holds TS steps per tile; points past the row's end take the last point's entries
        const float* tb = tabA + (int64_t)wt * (TS * 64);
        const uint32_t tl = (uint32_t)(kh * 32 + min(tk, r - 1 - wt * 32));
        float ta[KSU];
#pragma unroll
        for (int kk = 0; kk < KSU; ++kk) ta[kk] = tb[tl + (uint32_t)(kk * 64)];
        SPGT_LOAD_X_TILE(min(t + 1, t_end - 1))  // after the last pair: loaded again, not used
        const float* xr = xw + tk * PX + kh * KL;
        float4 xv[NP];
#pragma unroll
        for (int g = 0; g < NP; ++g) xv[g] = *reinterpret_cast<const float4*>(xr + 4 * g);
        __builtin_amdgcn_sched_barrier(0);
        v16f acc0 = bo0, acc1 = bo1;
#pragma unroll
        for (int g = 0; g < NP; ++g) {
            acc0 = mfma32(wreg0[4 * g + 0], xv[g].x, acc0);
            if (NCB == 2) acc1 = mfma32(wreg1[4 * g + 0], xv[g].x, acc1);
            acc0 = mfma32(wreg0[4 * g + 1], xv[g].y, acc0);
            if (NCB == 2) acc1 = mfma32(wreg1[4 * g + 1], xv[g].y, acc1);
            acc0 = mfma32(wreg0[4 * g + 2], xv[g].z, acc0);
            if (NCB == 2) acc1 = mfma32(wreg1[4 * g + 2], xv[g].z, acc1);
            acc0 = mfma32(wreg0[4 * g + 3], xv[g].w, acc0);
            if (NCB == 2) acc1 = mfma32(wreg1[4 * g + 3], xv[g].w, acc1);
        }
#pragma unroll
        for (int kk = 0; kk < KSU; ++kk) {
            acc0 = mfma32(ureg0[kk], ta[kk], acc0);
            if (NCB == 2) acc1 = mfma32(ureg1[kk], ta[kk], acc1);
        }
        // acc{cb}[4q + e] = out[w][o = cb*32 + 8q + 4kh + e] before the activation
        float y[32];
#pragma unroll
        for (int q = 0; q < 16; ++q) y[q] = acc0[q], y[16 + q] = acc1[q];
#pragma unroll
        for (int q = 0; q < 16 * NCB; ++q) {
            if (ACT == SPGT_ACT_RELU) y[q] = fmaxf(y[q], 0.f);
            if (ACT == SPGT_ACT_SILU) y[q] = y[q] * __builtin_amdgcn_rcpf(1.f + __expf(-y[q]));
        }
        // Through the wave's LDS tile (its x rows are in registers since before the MFMAs) the results leave as
        // whole rows: a lane's accumulator holds 16-byte pieces 32 bytes apart in its grid point's row, and stores
        // of those touch 32 cache lines per instruction; as rows, a store instruction writes 1 KB in one run
        // (33-34 -> 32 us at [8, 141, 141, 64] and [4, 211, 211, 64], non-temporal form; as plain stores the row
        // form was slower than the pieces).  Grid points past the row's end hold the last point's values and go to
        // its address.
        constexpr int PO = COUT + 4;
        constexpr int LPO = COUT / 4;  // lanes per output row
#pragma unroll
        for (int q = 0; q < 4 * NCB; ++q)
            *reinterpret_cast<float4*>(xw + tk * PO + 4 * kh + 8 * q) =
                make_float4(y[4 * q], y[4 * q + 1], y[4 * q + 2], y[4 * q + 3]);
        float4 rows[4 * NCB];
#pragma unroll
        for (int i = 0; i < 4 * NCB; ++i)
            rows[i] = *reinterpret_cast<const float4*>(xw + ((lane + 64 * i) / LPO) * PO + 4 * (lane % LPO));
        float* const orow = out + (int64_t)row * r * COUT + 4 * (lane % LPO);
#pragma unroll
        for (int i = 0; i < 4 * NCB; ++i) {
            const int pnt = min(wt * 32 + (lane + 64 * i) / LPO, r - 1);
            st_stream<true>(reinterpret_cast<float4*>(orow + (uint32_t)(pnt * COUT)), rows[i]);
        }
    }
#undef SPGT_LOAD_X_TILE
#undef SPGT_X_PIECE
#undef SPGT_STORE_X_PIECE
}

}  // namespace spgt

using namespace spgt;

namespace {

int dft_rows_check(const char* who, const void* a, const void* tab, const void* b, int64_t rows, int r, int C,
                   int m2) {
    if (!a || !tab || !b) return fail(SPGT_ERR_INVALID_ARGUMENT, "truncated_dft_rows: null pointer argument");
    if (rows <= 0 || r <= 0) return fail(SPGT_ERR_INVALID_ARGUMENT, "truncated_dft_rows: rows and r must be positive");
    if (C <= 0 || C % 32 != 0) return fail(SPGT_ERR_INVALID_ARGUMENT, "truncated_dft_rows: channels must be a multiple of 32");
    if (m2 <= 0 || m2 > 64 || (m2 & 1))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "truncated_dft_rows: 2*modes must be even and at most 64");
    if (r > (m2 > 32 ? 512 : 1024))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "truncated_dft_rows: r exceeds 1024 (512 when 2*modes > 32)");
    if (ceil_div(rows * (C / 32), (int64_t)4) > INT32_MAX)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "truncated_dft_rows: too many rows");
    if (!aligned4(a) || !aligned16(tab) || !aligned4(b))
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "truncated_dft_rows: operands must be 4-byte aligned, the table 16-byte aligned");
    (void)who;
    return SPGT_OK;
}

template <typename K>
void allow_lds(K kernel, size_t lds) {
    (void)allow_dynamic_lds(kernel, lds);
}

}  // namespace

extern "C" int spgt_truncated_dft_rows_supported(int r, int channels, int modes) {
    return (r > 0 && channels > 0 && channels % 32 == 0 && modes > 0 && 2 * modes <= 64 &&
            r <= (2 * modes > 32 ? 512 : 1024)) ? 1 : 0;
}

extern "C" int spgt_truncated_dft_rows_forward(const float* x, const float* table, float* Y, int64_t rows, int r,
                                               int channels, int modes, int planar, hipStream_t stream) {
    const int m2 = 2 * modes;
    if (int rc = dft_rows_check("truncated_dft_rows_forward", x, table, Y, rows, r, channels, m2)) return rc;
    if (planar && rows % r != 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "truncated_dft_rows_forward: planar output needs rows = N * r");
    const int mb = m2 > 32 ? 2 : 1;
    const size_t lds = (size_t)2 * ((r + 1) / 2) * 32 * mb * sizeof(float);
    // workgroups loop over (row, channel block) items: about two per CU, so the table is staged few times
    const unsigned grid = (unsigned)std::min<int64_t>(ceil_div(rows * (channels / 32), (int64_t)4), 2 * device_cu_count());
#define SPGT_DFT_FWD(CT, MB)                                                                                    \
    {                                                                                                           \
        allow_lds(dft_rows_forward_k<CT, MB>, lds);                                                             \
        hipLaunchKernelGGL((dft_rows_forward_k<CT, MB>), dim3(grid), dim3(256), lds, stream, x, table, Y, rows, r, \
                           channels, m2, planar);                                                               \
    }
    if (mb == 1) {
        if (channels == 64) SPGT_DFT_FWD(64, 1) else if (channels == 32) SPGT_DFT_FWD(32, 1)
        else if (channels == 128) SPGT_DFT_FWD(128, 1) else SPGT_DFT_FWD(0, 1)
    } else {
        const size_t lds_fold = (size_t)2 * ((r / 2 + 2) / 2) * 64 * sizeof(float);
        // the widest pieces the alignment of x and the channel count allow
        const bool planar_ok16 = !planar || aligned16(Y), planar_ok8 = !planar || aligned8(Y);
        const int v = (channels % 128 == 0 && aligned16(x) && planar_ok16) ? 4
                      : (channels % 64 == 0 && aligned8(x) && planar_ok8) ? 2 : 1;
        const unsigned grid_fold = (unsigned)std::min<int64_t>(ceil_div(rows * (channels / (32 * v)), (int64_t)4),
                                                               (v == 4 ? 1 : 2) * device_cu_count());
#define SPGT_DFT_FOLD(CT, V)                                                                                    \
    {                                                                                                           \
        allow_lds(dft_rows_forward_fold_k<CT, V>, lds_fold);                                                    \
        hipLaunchKernelGGL((dft_rows_forward_fold_k<CT, V>), dim3(grid_fold), dim3(256), lds_fold, stream, x,   \
                           table, Y, rows, r, channels, m2, planar);                                            \
    }
        if (v == 4) {
            if (channels == 128) SPGT_DFT_FOLD(128, 4) else SPGT_DFT_FOLD(0, 4)
        } else if (v == 2) {
            if (channels == 64) SPGT_DFT_FOLD(64, 2) else SPGT_DFT_FOLD(0, 2)
        } else {
            if (channels == 32) SPGT_DFT_FOLD(32, 1) else SPGT_DFT_FOLD(0, 1)
        }
#undef SPGT_DFT_FOLD
    }
#undef SPGT_DFT_FWD
    return check_launch("truncated_dft_rows_forward");
}

extern "C" int spgt_truncated_dft_rows_inverse(const float* U, const float* table, float* y, int64_t rows, int r,
                                               int channels, int modes, int planar, hipStream_t stream) {
    const int m2 = 2 * modes;
    if (int rc = dft_rows_check("truncated_dft_rows_inverse", U, table, y, rows, r, channels, m2)) return rc;
    if (planar && rows % r != 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "truncated_dft_rows_inverse: planar input needs rows = N * r");
    const size_t lds = (size_t)((r + 31) / 32) * 32 * (m2 + 1) * sizeof(float);
    const unsigned grid = (unsigned)std::min<int64_t>(ceil_div(rows * (channels / 32), (int64_t)4), 2 * device_cu_count());
    if (m2 <= 32) {
        allow_lds(dft_rows_inverse_k<16>, lds);
        hipLaunchKernelGGL(dft_rows_inverse_k<16>, dim3(grid), dim3(256), lds, stream, U, table, y, rows, r, channels, m2,
                           planar);
    } else {
        allow_lds(dft_rows_inverse_k<32>, lds);
        hipLaunchKernelGGL(dft_rows_inverse_k<32>, dim3(grid), dim3(256), lds, stream, U, table, y, rows, r, channels, m2,
                           planar);
    }
    return check_launch("truncated_dft_rows_inverse");
}

extern "C" int spgt_spectral_modes_middle_supported(int r, int Cin, int Cout, int modes) {
    return (r > 0 && r <= 4096 && Cin > 0 && Cin <= 2 * kMidC && Cout > 0 && Cout <= kMidC && modes > 0 &&
            2 * modes <= 64 && 2 * modes <= r) ? 1 : 0;
}

extern "C" size_t spgt_spectral_modes_middle_workspace_bytes(int N, int Cout, int modes) {
    if (N <= 0 || Cout <= 0 || modes <= 0) return 0;
    return (size_t)N * modes * 2 * modes * Cout * sizeof(float2);
}

extern "C" int spgt_spectral_modes_middle(const float* Y, const float* table_h, const float* table_h_inverse,
                                          const float* weight_1, const float* weight_2, float* U, void* workspace,
                                          size_t workspace_bytes, int N, int r, int Cin, int Cout, int modes,
                                          hipStream_t stream) {
    if (!Y || !table_h || !table_h_inverse || !weight_1 || !weight_2 || !U || !workspace)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_modes_middle: null pointer argument");
    if (N <= 0 || N > 65535) return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_modes_middle: N must be 1..65535");
    if (!spgt_spectral_modes_middle_supported(r, Cin, Cout, modes))
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "spectral_modes_middle: needs Cin <= 128, Cout <= 64, 2*modes <= min(64, r), r <= 4096");
    if (workspace_bytes < spgt_spectral_modes_middle_workspace_bytes(N, Cout, modes))
        return fail(SPGT_ERR_WORKSPACE, "spectral_modes_middle: workspace too small");
    if (!aligned4(Y) || !aligned4(U) || !aligned8(table_h) || !aligned8(table_h_inverse) || !aligned8(weight_1) ||
        !aligned8(weight_2) || !aligned8(workspace))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_modes_middle: complex operands must be 8-byte aligned");
    const int m2 = 2 * modes;
    float2* O = reinterpret_cast<float2*>(workspace);
    const int cpl = Cin > kMidC ? 2 : 1;
    const size_t lds1 = ((size_t)kMidRows * r + 4 * kMidRows * kMidC * cpl) * sizeof(float2);
    const dim3 grid1(modes, N, ceil_div(m2, kMidRows));
#define SPGT_MID_CONTRACT(CPL)                                                                                       \
    {                                                                                                                \
        allow_lds(spectral_rows_contract_k<CPL>, lds1);                                                              \
        hipLaunchKernelGGL(spectral_rows_contract_k<CPL>, grid1, dim3(256), lds1, stream, Y,                         \
                           reinterpret_cast<const float2*>(table_h), reinterpret_cast<const float2*>(weight_1),      \
                           reinterpret_cast<const float2*>(weight_2), O, r, Cin, Cout, modes);                       \
    }
    if (cpl == 1) SPGT_MID_CONTRACT(1) else SPGT_MID_CONTRACT(2)
#undef SPGT_MID_CONTRACT
    // about three workgroups per CU for the expansion; a chunk's table rows must fit 64 KiB of LDS
    int chunks = std::max(1, std::min(ceil_div(r, 4), ceil_div(3 * device_cu_count(), modes * N)));
    chunks = std::max(chunks, ceil_div(r * m2 * (int)sizeof(float2), 64 * 1024));
    const int rows_per_wg = ceil_div(r, chunks);
    const size_t lds2 = (size_t)rows_per_wg * m2 * sizeof(float2);
    const dim3 grid2(modes, N, ceil_div(r, rows_per_wg));
#define SPGT_MID_EXPAND(KHMAX, LPR)                                                                                  \
    hipLaunchKernelGGL((spectral_rows_expand_k<KHMAX, LPR>), grid2, dim3(256), lds2, stream, O,                      \
                       reinterpret_cast<const float2*>(table_h_inverse), U, r, Cout, modes, rows_per_wg)
    if (m2 <= 32) {
        if (Cout <= 32) SPGT_MID_EXPAND(32, 32); else SPGT_MID_EXPAND(32, 64);
    } else {
        if (Cout <= 32) SPGT_MID_EXPAND(64, 32); else SPGT_MID_EXPAND(64, 64);
    }
#undef SPGT_MID_EXPAND
    return check_launch("spectral_modes_middle");
}

extern "C" int spgt_spectral_inverse_linear_supported(int r, int in_features, int out_features, int modes) {
    const bool pair = (in_features == out_features && (in_features == 32 || in_features == 64)) ||
                      (in_features == 64 && out_features == 32) ||
                      (in_features == 128 && (out_features == 32 || out_features == 64));
    return (r > 0 && r <= 1024 && pair && modes > 0 && 2 * modes <= 64 && 2 * modes <= r) ? 1 : 0;
}

namespace {

template <int ACT, int CIN, int COUT>
int launch_inverse_linear(const float* U, const float* table_operand, const float* x, const float* weight_kn,
                          const float* bias, float* out, int r, int modes, int64_t pairs, hipStream_t stream) {
    const dim3 grid((unsigned)std::min<int64_t>(ceil_div(pairs, (int64_t)4), (int64_t)device_cu_count()));
    const size_t lds = (size_t)4 * 32 * (CIN + 4) * sizeof(float);
#define SPGT_SIL_LAUNCH(KSU)                                                                                        \
    {                                                                                                               \
        if (!allow_dynamic_lds(spectral_inverse_linear_k<ACT, KSU, CIN, COUT>, lds))                                \
            return fail(SPGT_ERR_LAUNCH, "spectral_inverse_linear: the kernel was refused its dynamic LDS size");    \
        hipLaunchKernelGGL((spectral_inverse_linear_k<ACT, KSU, CIN, COUT>), grid, dim3(256), lds, stream, U,       \
                           table_operand, x, weight_kn, bias, out, r, 2 * modes, (unsigned)pairs);                  \
    }
    if (modes <= 4) SPGT_SIL_LAUNCH(4)
    else if (modes <= 8) SPGT_SIL_LAUNCH(8)
    else if (modes <= 12) SPGT_SIL_LAUNCH(12)
    else if (modes <= 16) SPGT_SIL_LAUNCH(16)
    else if (modes <= 24) SPGT_SIL_LAUNCH(24)
    else SPGT_SIL_LAUNCH(32)
#undef SPGT_SIL_LAUNCH
    return SPGT_OK;
}

template <int CIN, int COUT>
int launch_inverse_linear_act(int activation, const float* U, const float* table_operand, const float* x,
                              const float* weight_kn, const float* bias, float* out, int r, int modes, int64_t pairs,
                              hipStream_t stream) {
    if (activation == SPGT_ACT_RELU)
        return launch_inverse_linear<SPGT_ACT_RELU, CIN, COUT>(U, table_operand, x, weight_kn, bias, out, r, modes, pairs, stream);
    if (activation == SPGT_ACT_SILU)
        return launch_inverse_linear<SPGT_ACT_SILU, CIN, COUT>(U, table_operand, x, weight_kn, bias, out, r, modes, pairs, stream);
    return launch_inverse_linear<SPGT_ACT_NONE, CIN, COUT>(U, table_operand, x, weight_kn, bias, out, r, modes, pairs, stream);
}

}  // namespace

extern "C" int spgt_spectral_inverse_linear(const float* U, const float* table_operand, const float* x,
                                            const float* weight_kn, const float* bias, int activation, float* out,
                                            int64_t rows, int r, int in_features, int out_features, int modes,
                                            hipStream_t stream) {
    if (!U || !table_operand || !x || !weight_kn || !out)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_inverse_linear: null pointer argument");
    if (!spgt_spectral_inverse_linear_supported(r, in_features, out_features, modes))
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "spectral_inverse_linear: needs (in, out) features in {32->32, 64->64, 64->32, 128->32, 128->64}, "
                    "2*modes <= min(64, r), r <= 1024");
    if (rows <= 0 || rows % r != 0 || rows > INT32_MAX)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_inverse_linear: rows must be a positive multiple of r");
    if (activation != SPGT_ACT_NONE && activation != SPGT_ACT_RELU && activation != SPGT_ACT_SILU)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_inverse_linear: unknown activation");
    if (!aligned4(U) || !aligned4(table_operand) || !aligned16(x) || !aligned4(weight_kn) || !aligned16(out) ||
        (bias && !aligned16(bias)))
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "spectral_inverse_linear: x, out and bias must be 16-byte aligned, the rest 4-byte aligned");
    if (out == x) return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_inverse_linear: out must not alias x");
    const int64_t pairs = (int64_t)rows * ((r + 31) / 32);
    if (pairs > (int64_t)INT32_MAX - 4096)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_inverse_linear: more than 2^31 tiles of 32 grid points");
    int rc;
#define SPGT_SIL_SHAPE(CIN, COUT)                                                                                 \
    rc = launch_inverse_linear_act<CIN, COUT>(activation, U, table_operand, x, weight_kn, bias, out, r, modes, pairs, \
                                              stream)
    if (in_features == 32) SPGT_SIL_SHAPE(32, 32);
    else if (in_features == 64 && out_features == 64) SPGT_SIL_SHAPE(64, 64);
    else if (in_features == 64) SPGT_SIL_SHAPE(64, 32);
    else if (out_features == 32) SPGT_SIL_SHAPE(128, 32);
    else SPGT_SIL_SHAPE(128, 64);
#undef SPGT_SIL_SHAPE
    if (rc != SPGT_OK) return rc;
    return check_launch("spectral_inverse_linear");
}

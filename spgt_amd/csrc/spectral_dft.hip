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
// tab [r][m2] row-major, m2 <= 32.
// Y [rows][C][m2].
__global__ __launch_bounds__(256) void dft_rows_forward_k(const float* __restrict__ x, const float* __restrict__ tab,
                                                          float* __restrict__ Y, int64_t rows, int r, int C, int m2) {
    extern __shared__ float ts[];  // [2*KH][32], zero beyond r rows and m2 columns
    const int KH = (r + 1) / 2;
    {
        // table fill with eight loads in flight per thread
        const int total = 2 * KH * 32;
        for (int e0 = threadIdx.x; e0 < total; e0 += 256 * 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int e = e0 + 256 * u;
                const int w = e >> 5, j = e & 31;
                v[u] = (e < total && w < r && j < m2) ? tab[w * m2 + j] : 0.f;
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (e0 + 256 * u < total) ts[e0 + 256 * u] = v[u];
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
    const float* xr = x + row * (int64_t)r * C + cb * 32 + tk;

    constexpr int BK = 32;
    float xv[2][BK];
    auto load_batch = [&](int b) {
#pragma unroll
        for (int u = 0; u < BK; ++u) {
            const int w = min(2 * (b * BK + u) + kh, r - 1);  // rows past r meet zero table entries
            xv[b & 1][u] = xr[(int64_t)w * C];
        }
    };
    v16f acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    const int nb = (KH + BK - 1) / BK;
    load_batch(0);
    for (int b = 0; b < nb; b += 2) {
        // two batches per trip so that the buffer index is a compile-time constant
        if (b + 1 < nb) {
#pragma unroll
            for (int u = 0; u < BK; ++u) {
                const int w = min(2 * ((b + 1) * BK + u) + kh, r - 1);
                xv[1][u] = xr[(int64_t)w * C];
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < BK; ++u) {
            const int kk = b * BK + u;
            if (kk < KH) acc = mfma32(ts[(2 * kk + kh) * 32 + tk], xv[0][u], acc);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (b + 2 < nb) {
#pragma unroll
            for (int u = 0; u < BK; ++u) {
                const int w = min(2 * ((b + 2) * BK + u) + kh, r - 1);
                xv[0][u] = xr[(int64_t)w * C];
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        if (b + 1 < nb) {
#pragma unroll
            for (int u = 0; u < BK; ++u) {
                const int kk = (b + 1) * BK + u;
                if (kk < KH) acc = mfma32(ts[(2 * kk + kh) * 32 + tk], xv[1][u], acc);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    // acc[r] = Y[c = cb*32 + tk][j = 8*(r/4) + 4*kh + r%4]
    float* yr = Y + (row * C + cb * 32 + tk) * (int64_t)m2;
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int j = 8 * q + 4 * kh + e;
            if (j < m2) yr[j] = acc[4 * q + e];
        }
    }
}

// grid (workgroups), block 256; waves stride over the (row, channel block) items.
// tab [r][m2] row-major, m2 <= 32 and even.
// U [rows][C][m2] -> y [rows][r][C].
__global__ __launch_bounds__(256) void dft_rows_inverse_k(const float* __restrict__ U, const float* __restrict__ tab,
                                                          float* __restrict__ y, int64_t rows, int r, int C, int m2) {
    extern __shared__ float ts[];  // [32 * ceil(r/32)][m2 + 1], zero beyond r rows
    const int pitch = m2 + 1;
    const int WT = (r + 31) / 32;
    {
        const int total = WT * 32 * m2;
        for (int e0 = threadIdx.x; e0 < total; e0 += 256 * 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int e = e0 + 256 * u;
                v[u] = (e < r * m2) ? tab[e] : 0.f;
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int e = e0 + 256 * u;
                if (e < total) ts[(e / m2) * pitch + e % m2] = v[u];
            }
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
    const float* ur = U + (row * C + cb * 32 + tk) * (int64_t)m2;
    float ureg[16];
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) ureg[kk] = (2 * kk + kh < m2) ? ur[2 * kk + kh] : 0.f;
    float* yr = y + row * (int64_t)r * C + cb * 32 + tk;
    const int KH = m2 / 2;
    for (int wt = 0; wt < WT; ++wt) {
        const float* ta = ts + (wt * 32 + tk) * pitch + kh;
        v16f acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
        for (int kk = 0; kk < 16; ++kk)
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

}  // namespace spgt

using namespace spgt;

namespace {

int dft_rows_check(const char* who, const void* a, const void* tab, const void* b, int64_t rows, int r, int C,
                   int m2) {
    if (!a || !tab || !b) return fail(SPGT_ERR_INVALID_ARGUMENT, "truncated_dft_rows: null pointer argument");
    if (rows <= 0 || r <= 0) return fail(SPGT_ERR_INVALID_ARGUMENT, "truncated_dft_rows: rows and r must be positive");
    if (C <= 0 || C % 32 != 0) return fail(SPGT_ERR_INVALID_ARGUMENT, "truncated_dft_rows: channels must be a multiple of 32");
    if (m2 <= 0 || m2 > 32 || (m2 & 1))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "truncated_dft_rows: 2*modes must be even and at most 32");
    if (r > 1024) return fail(SPGT_ERR_INVALID_ARGUMENT, "truncated_dft_rows: r exceeds 1024");
    if (ceil_div(rows * (C / 32), (int64_t)4) > INT32_MAX)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "truncated_dft_rows: too many rows");
    if (!aligned4(a) || !aligned4(tab) || !aligned4(b))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "truncated_dft_rows: operands must be 4-byte aligned");
    (void)who;
    return SPGT_OK;
}

}  // namespace

extern "C" int spgt_truncated_dft_rows_supported(int r, int channels, int modes) {
    return (r > 0 && r <= 1024 && channels > 0 && channels % 32 == 0 && modes > 0 && 2 * modes <= 32) ? 1 : 0;
}

extern "C" int spgt_truncated_dft_rows_forward(const float* x, const float* table, float* Y, int64_t rows, int r,
                                               int channels, int modes, hipStream_t stream) {
    const int m2 = 2 * modes;
    if (int rc = dft_rows_check("truncated_dft_rows_forward", x, table, Y, rows, r, channels, m2)) return rc;
    const size_t lds = (size_t)2 * ((r + 1) / 2) * 32 * sizeof(float);
    auto kernel = dft_rows_forward_k;
    if (lds > 64 * 1024)
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)lds);
    // workgroups loop over (row, channel block) items: about two per CU, so the table is staged few times
    const unsigned grid = (unsigned)std::min<int64_t>(ceil_div(rows * (channels / 32), (int64_t)4), 2 * device_cu_count());
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), lds, stream, x, table, Y, rows, r, channels, m2);
    return check_launch("truncated_dft_rows_forward");
}

extern "C" int spgt_truncated_dft_rows_inverse(const float* U, const float* table, float* y, int64_t rows, int r,
                                               int channels, int modes, hipStream_t stream) {
    const int m2 = 2 * modes;
    if (int rc = dft_rows_check("truncated_dft_rows_inverse", U, table, y, rows, r, channels, m2)) return rc;
    const size_t lds = (size_t)((r + 31) / 32) * 32 * (m2 + 1) * sizeof(float);
    auto kernel = dft_rows_inverse_k;
    if (lds > 64 * 1024)
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  (int)lds);
    const unsigned grid = (unsigned)std::min<int64_t>(ceil_div(rows * (channels / 32), (int64_t)4), 2 * device_cu_count());
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), lds, stream, U, table, y, rows, r, channels, m2);
    return check_launch("truncated_dft_rows_inverse");
}

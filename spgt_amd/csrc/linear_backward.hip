// Weight and bias gradients of a token-major Linear y = x W + b:
//   dW[k][n] = sum_t x[t][k] g[t][n]        db[n] = sum_t g[t][n]
// (reference: extension/bind/galerkin_attention.cu:41-46, where the two are a library GEMM on the
// transposed input and a library reduction).  The contraction runs over the tokens, tens of thousands
// to millions of them, against 128 x 128 results: a split over token chunks, each chunk's [K, N] tile
// accumulated in MFMA registers straight from global memory (both operands are read with lanes along
// the feature axis, 128-byte runs; no transpose of x is ever formed), then one deterministic
// second-stage sum over the chunks (tile_reduce), bias gradient included.
#include "spgt_device.h"
#include "spgt_host.h"
#include "spgt_kernels.h"

namespace spgt {

// partial[batch][chunk][k * N + n] = sum over the chunk's tokens of x[t][k] * g[t][n]
// partial[batch][chunk][K * N + n] = sum over the chunk's tokens of g[t][n]
// grid (nchunk, batch * nstrip, ceil(K / 128)), block 256: wave w takes rows k in [32 (4 z + w), +32) of the strip
// of NT * 32 columns.  MFMA 32x32x2 step kk contracts tokens 2 kk and 2 kk + 1 of the chunk (lane half = token),
// A = x[t][k0 + lane % 32], B = g[t][n0 + 32 nt + lane % 32].  Operand batches of BK steps are requested one
// batch ahead of the MFMAs that consume them.
// TSPLIT (for K <= 32, where three of the four waves would have no rows): the four waves take the same 32 rows and
// a quarter of the chunk's tokens each, and their tiles are added through LDS in a fixed order.
template <int NT, bool TSPLIT>
__global__ __launch_bounds__(256, 2) void xtg_partial_k(const float* __restrict__ X, int64_t ldx, int64_t x_batch,
                                                     const float* __restrict__ G, int64_t ldg, int64_t g_batch,
                                                     float* __restrict__ partial, int64_t T, int K, int N,
                                                     int tokens_per_chunk, int nstrip) {
    constexpr int BK = 8;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tk = lane & 31;
    const int kh = lane >> 5;
    const int chunk = blockIdx.x;
    const int nchunk = gridDim.x;
    const int b = blockIdx.y / nstrip;
    const int strip = blockIdx.y - b * nstrip;
    const int k0 = TSPLIT ? 0 : (blockIdx.z * 4 + wave) * 32;
    const int n0 = strip * NT * 32;
    const int E = K * N + N;
    if (!TSPLIT && k0 >= K) return;  // whole wave: no barrier follows
    const int64_t c0 = (int64_t)chunk * tokens_per_chunk;
    const int64_t c1 = min(T, c0 + tokens_per_chunk);
    const int64_t quarter = TSPLIT ? (tokens_per_chunk / 4) : 0;  // tokens_per_chunk is a multiple of 16
    const int64_t t0 = TSPLIT ? min(c1, c0 + wave * quarter) : c0;
    const int64_t t1 = TSPLIT ? min(c1, t0 + quarter) : c1;
    const int steps = (int)((t1 - t0 + 1) / 2);
    // clamped feature indices: rows past K and columns past N read valid memory and are masked to zero
    const bool kok = k0 + tk < K;
    const float* xp = X + b * x_batch + t0 * ldx + min(k0 + tk, K - 1);
    const float* gp = G + b * g_batch + t0 * ldg;
    uint32_t goff[NT];
    bool nok[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        nok[nt] = n0 + 32 * nt + tk < N;
        goff[nt] = (uint32_t)min(n0 + 32 * nt + tk, N - 1);
    }
    v16f acc[NT];
    float colsum[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        colsum[nt] = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[nt][r] = 0.f;
    }
    const int last = (int)(t1 - t0) - 1;  // last valid token of the chunk, relative
    float xa[BK], ga[NT][BK], xb[BK], gb[NT][BK];
    // fetch only requests (clamped addresses); the masks are applied when the values are used, so that a batch's
    // loads stay in flight under the previous batch's MFMAs
    auto fetch = [&](float (&xv)[BK], float (&gv)[NT][BK], int batch) {
#pragma unroll
        for (int u = 0; u < BK; ++u) {
            const int64_t tr = min(2 * (batch * BK + u) + kh, last);
            xv[u] = xp[tr * ldx];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) gv[nt][u] = gp[tr * ldg + goff[nt]];
        }
    };
    auto multiply = [&](const float (&xv)[BK], const float (&gv)[NT][BK], int batch) {
#pragma unroll
        for (int u = 0; u < BK; ++u) {
            const bool ok = 2 * (batch * BK + u) + kh <= last;
            const float xm = (ok && kok) ? xv[u] : 0.f;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const float gm = (ok && nok[nt]) ? gv[nt][u] : 0.f;
                acc[nt] = mfma32(xm, gm, acc[nt]);
                colsum[nt] += gm;
            }
        }
    };
    const int nbatch = (steps + BK - 1) / BK;  // steps past the chunk's end contribute zeros
    if (nbatch > 0) fetch(xa, ga, 0);
    for (int bt = 0; bt < nbatch; bt += 2) {
        if (bt + 1 < nbatch) fetch(xb, gb, bt + 1);
        __builtin_amdgcn_sched_barrier(0);
        multiply(xa, ga, bt);
        __builtin_amdgcn_sched_barrier(0);
        if (bt + 2 < nbatch) fetch(xa, ga, bt + 2);
        __builtin_amdgcn_sched_barrier(0);
        if (bt + 1 < nbatch) multiply(xb, gb, bt + 1);
        __builtin_amdgcn_sched_barrier(0);
    }
    float* out = partial + ((int64_t)b * nchunk + chunk) * E;
    if constexpr (TSPLIT) {
        // the four waves' tiles and column sums: waves 1..3 to LDS, wave 0 adds them in order
        __shared__ float red[3][NT * 17 * 64];
        if (wave > 0) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
                for (int r = 0; r < 16; ++r) red[wave - 1][(nt * 17 + r) * 64 + lane] = acc[nt][r];
                red[wave - 1][(nt * 17 + 16) * 64 + lane] = colsum[nt];
            }
        }
        __syncthreads();
        if (wave > 0) return;
#pragma unroll
        for (int w = 0; w < 3; ++w)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[nt][r] += red[w][(nt * 17 + r) * 64 + lane];
                colsum[nt] += red[w][(nt * 17 + 16) * 64 + lane];
            }
    }
    // acc[nt][r] = dW[k0 + 8 (r / 4) + 4 kh + r % 4][n0 + 32 nt + tk]
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        if (nok[nt]) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int k = k0 + 8 * (r >> 2) + 4 * kh + (r & 3);
                if (k < K) out[(int64_t)k * N + n0 + 32 * nt + tk] = acc[nt][r];
            }
        }
        // bias gradient: the two token halves of a column meet; written once per strip, by the wave of rows 0..31
        const float cs = colsum[nt] + __shfl_xor(colsum[nt], 32, 64);
        if (k0 == 0 && kh == 0 && nok[nt]) out[(int64_t)K * N + n0 + 32 * nt + tk] = cs;
    }
}

// The same partial sums for 128 x 128 blocks of dW with 16-byte loads: a wave takes every fourth pair of the
// chunk's tokens and holds the whole block, 16 accumulators of 32 x 32.  Lane (i = lane % 32, h = lane / 32) loads
// x[t + h][k0 + 4 i .. 4 i + 3] and g[t + h][n0 + 4 i .. 4 i + 3]; register a of the x piece against register b of
// the g piece is one MFMA 32x32x2 whose row index i stands for feature k0 + 4 i + a and whose column index j for
// n0 + 4 j + b, so the features never have to be rearranged: two load instructions feed 16 MFMAs (the kernel
// above issues five loads for four).  The four waves' blocks are summed through LDS in a fixed order.
// grid (nchunk, batch * nstrip, ceil(K / 128)), block 256, one workgroup per compute unit (512 registers per lane).
// Requires N a multiple of 128, K a multiple of 4 and at least 128 (the rows of the last block past K are read from
// the row's last piece, used as zeros and not stored), ldx and ldg multiples of 4, 16-byte aligned x and g.
__global__ __launch_bounds__(256, 1) void xtg_partial_wide_k(const float* __restrict__ X, int64_t ldx, int64_t x_batch,
                                                             const float* __restrict__ G, int64_t ldg,
                                                             int64_t g_batch, float* __restrict__ partial, int64_t T,
                                                             int K, int N, int tokens_per_chunk, int nstrip) {
    constexpr int D = 4;  // steps of operands in flight ahead of the MFMAs
    __shared__ float4 tile[16 * 4 * 64];  // [a][b][r / 4][lane]: one wave's block, 64 KB
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tk = lane & 31;
    const int kh = lane >> 5;
    const int chunk = blockIdx.x;
    const int nchunk = gridDim.x;
    const int b = blockIdx.y / nstrip;
    const int strip = blockIdx.y - b * nstrip;
    const int k0 = blockIdx.z * 128;
    const int n0 = strip * 128;
    const int E = K * N + N;
    const int64_t t0 = (int64_t)chunk * tokens_per_chunk;
    const int64_t t1 = min(T, t0 + tokens_per_chunk);
    const int last = (int)(t1 - t0) - 1;
    const int pairs = (last + 2) / 2;            // token pairs of the chunk
    const int steps = (pairs - wave + 3) / 4;    // pairs wave, wave + 4, ... of them
    const bool kok = k0 + 4 * tk < K;  // K is a multiple of 4: a piece lies inside the row or past it
    const float* xp = X + b * x_batch + t0 * ldx + min(k0 + 4 * tk, K - 4);
    const float* gp = G + b * g_batch + t0 * ldg + n0 + 4 * tk;
    v16f acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][c][r] = 0.f;
    float colsum[4] = {0.f, 0.f, 0.f, 0.f};
    float4 xq[D], gq[D];
    auto issue = [&](int slot, int s) {
        const int64_t tr = min(2 * (4 * s + wave) + kh, last);  // past the end: a valid row, masked when used
        xq[slot] = *reinterpret_cast<const float4*>(xp + tr * ldx);
        gq[slot] = *reinterpret_cast<const float4*>(gp + tr * ldg);
    };
    auto use = [&](int slot, int s) {
        const bool ok = 2 * (4 * s + wave) + kh <= last;
        const bool xok = ok && kok;
        const float xr[4] = {xok ? xq[slot].x : 0.f, xok ? xq[slot].y : 0.f, xok ? xq[slot].z : 0.f,
                             xok ? xq[slot].w : 0.f};
        const float gr[4] = {ok ? gq[slot].x : 0.f, ok ? gq[slot].y : 0.f, ok ? gq[slot].z : 0.f, ok ? gq[slot].w : 0.f};
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int c = 0; c < 4; ++c) acc[a][c] = mfma32(xr[a], gr[c], acc[a][c]);
#pragma unroll
        for (int c = 0; c < 4; ++c) colsum[c] += gr[c];
    };
    if (last >= 0) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            issue(d, d);  // in the loop's own order, so that the loop waits for the oldest step only
            __builtin_amdgcn_sched_barrier(0);
        }
        for (int s = 0; s < steps; s += D) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
                use(d, s + d);  // a step past the wave's last contributes zeros
                __builtin_amdgcn_sched_barrier(0);
                issue(d, s + d + D);  // stays D - 1 steps of MFMAs ahead of its use
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    float* out = partial + ((int64_t)b * nchunk + chunk) * E;
    // bias gradient: the two token halves of a column meet, then the four waves in a fixed order
    float* colsm = reinterpret_cast<float*>(tile);  // [4][128], before the blocks need the space
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const float cs = colsum[c] + __shfl_xor(colsum[c], 32, 64);
        if (kh == 0) colsm[wave * 128 + 4 * tk + c] = cs;
    }
    __syncthreads();
    if (wave == 1 && k0 == 0) {
        for (int n = lane; n < 128; n += 64)
            out[(int64_t)K * N + n0 + n] = (colsm[n] + colsm[128 + n]) + (colsm[256 + n] + colsm[384 + n]);
    }
    __syncthreads();
    // the waves' blocks: wave 3 -> LDS, wave 2 adds and writes, wave 1 adds and writes, wave 0 adds and stores
#pragma unroll 1
    for (int turn = 3; turn >= 0; --turn) {
        if (wave == turn) {
            if (turn < 3) {
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    float4 v[16];  // a row group's sixteen pieces are requested before the first is used
#pragma unroll
                    for (int i = 0; i < 16; ++i) v[i] = tile[(a * 16 + i) * 64 + lane];
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int c = 0; c < 4; ++c)
#pragma unroll
                        for (int r4 = 0; r4 < 4; ++r4) {
                            const float4 w = v[c * 4 + r4];
                            acc[a][c][4 * r4] += w.x, acc[a][c][4 * r4 + 1] += w.y;
                            acc[a][c][4 * r4 + 2] += w.z, acc[a][c][4 * r4 + 3] += w.w;
                        }
                }
            }
            if (turn > 0) {
#pragma unroll
                for (int a = 0; a < 4; ++a)
#pragma unroll
                    for (int c = 0; c < 4; ++c)
#pragma unroll
                        for (int r4 = 0; r4 < 4; ++r4)
                            tile[((a * 4 + c) * 4 + r4) * 64 + lane] = make_float4(
                                acc[a][c][4 * r4], acc[a][c][4 * r4 + 1], acc[a][c][4 * r4 + 2], acc[a][c][4 * r4 + 3]);
            }
        }
        if (turn > 0) __syncthreads();
    }
    if (wave == 0) {
        // acc[a][c][r] = dW[k0 + 4 (8 (r / 4) + 4 kh + r % 4) + a][n0 + 4 tk + c]
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int k = k0 + 4 * (8 * (r >> 2) + 4 * kh + (r & 3)) + a;
                if (k < K)
                    *reinterpret_cast<float4*>(out + (int64_t)k * N + n0 + 4 * tk) =
                        make_float4(acc[a][0][r], acc[a][1][r], acc[a][2][r], acc[a][3][r]);
            }
    }
}

// out = residual + dropout(y) on [rows, cols] (cols a multiple of 4; residual may be null): the reference's
// F.dropout followed by the residual add (network/sp_layer.py:76, 100-103; network/layer.py:173) in one pass, with
// the keep decisions of dropout_site / dropout_apply (spgt_device.h).  The same call on a gradient with the
// forward's seed is the backward of the dropout.  A thread takes 16-byte pieces, grid-stride.
__global__ __launch_bounds__(256) void dropout_add_k(const float* __restrict__ y, const float* __restrict__ residual,
                                                     float* __restrict__ out, int64_t pieces, int cols4,
                                                     const uint32_t* __restrict__ seed, float p, uint32_t site) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < pieces; e += stride) {
        const int64_t row = e / cols4;
        const uint32_t col = 4u * (uint32_t)(e - row * cols4);
        const DropoutSite ds = dropout_site(seed, site, row, p);
        const float4 v = reinterpret_cast<const float4*>(y)[e];
        float4 o = make_float4(dropout_apply(ds, col, v.x), dropout_apply(ds, col + 1, v.y),
                               dropout_apply(ds, col + 2, v.z), dropout_apply(ds, col + 3, v.w));
        if (residual) {
            const float4 r = reinterpret_cast<const float4*>(residual)[e];
            o.x += r.x, o.y += r.y, o.z += r.z, o.w += r.w;
        }
        reinterpret_cast<float4*>(out)[e] = o;
    }
}

}  // namespace spgt

using namespace spgt;

namespace {

struct WgradPlan {
    int nt, nstrip, kz, tpc, nchunk;
    bool wide;
};

// The plan depends on the sizes only (the workspace query has nothing else): the wide kernel serves N a multiple
// of 128 with K a multiple of 4 from 128 up and is chosen then; a call whose strides or alignment do not fit it
// runs the kernel above on the same chunks.
WgradPlan wgrad_plan(int64_t T, int K, int N, int batch) {
    WgradPlan p;
    p.wide = K % 4 == 0 && K >= 128 && N % 128 == 0;
    p.nt = N >= 128 ? 4 : (N > 32 ? 2 : 1);
    p.nstrip = ceil_div(N, p.nt * 32);
    p.kz = ceil_div(K, 128);
    // about two workgroups per compute unit (one for the wide kernel, whose waves hold 512 registers), at most
    // as many chunks as tile_reduce sums, at least 64 tokens each
    const int per = std::max(1, (p.wide ? 1 : 2) * device_cu_count() / std::max(1, batch * p.nstrip * p.kz));
    int64_t nchunk = std::min<int64_t>(std::min(per, kReduceChains * kReduceMaxPerChain), std::max<int64_t>(1, T / 64));
    int64_t tpc = ceil_div(ceil_div(T, nchunk), (int64_t)16) * 16;
    p.tpc = (int)tpc;
    p.nchunk = (int)ceil_div(T, tpc);
    return p;
}

}  // namespace

extern "C" size_t spgt_linear_weight_grad_workspace_bytes(int64_t tokens, int in_features, int out_features,
                                                          int batch) {
    if (tokens <= 0 || in_features <= 0 || out_features <= 0 || batch <= 0 || out_features % 4 != 0) return 0;
    if (tokens > ((int64_t)1 << 31) - 1024 || (int64_t)in_features * out_features + out_features > INT32_MAX) return 0;
    const WgradPlan p = wgrad_plan(tokens, in_features, out_features, batch);
    return (size_t)batch * p.nchunk * ((size_t)in_features * out_features + out_features) * sizeof(float);
}

extern "C" int spgt_linear_weight_grad(const float* x, int64_t ldx, int64_t x_batch_stride, const float* grad,
                                       int64_t ldg, int64_t grad_batch_stride, float* out, void* workspace,
                                       size_t workspace_bytes, int64_t tokens, int in_features, int out_features,
                                       int batch, hipStream_t stream) {
    if (!x || !grad || !out || !workspace)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "linear_weight_grad: null pointer argument");
    const size_t need = spgt_linear_weight_grad_workspace_bytes(tokens, in_features, out_features, batch);
    if (need == 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "linear_weight_grad: sizes must be positive, out_features a multiple of 4, tokens below 2^31");
    if (ldx < in_features || ldg < out_features)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "linear_weight_grad: row strides shorter than the rows");
    const int64_t E = (int64_t)in_features * out_features + out_features;
    if (workspace_bytes < need || !aligned16(workspace))
        return fail(SPGT_ERR_WORKSPACE, "linear_weight_grad: workspace missing, misaligned or too small");
    if (!aligned4(x) || !aligned4(grad) || !aligned16(out))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "linear_weight_grad: out must be 16-byte aligned");
    const WgradPlan p = wgrad_plan(tokens, in_features, out_features, batch);
    if ((int64_t)batch * p.nstrip > 65535 || p.kz > 65535)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "linear_weight_grad: too many column strips or row blocks");
    float* partial = static_cast<float*>(workspace);
    const dim3 grid(p.nchunk, batch * p.nstrip, p.kz);
#define SPGT_XTG(NT)                                                                                               \
    if (in_features <= 32)                                                                                         \
        hipLaunchKernelGGL((xtg_partial_k<NT, true>), grid, dim3(256), 0, stream, x, ldx, x_batch_stride, grad, ldg, \
                           grad_batch_stride, partial, tokens, in_features, out_features, p.tpc, p.nstrip);        \
    else                                                                                                           \
        hipLaunchKernelGGL((xtg_partial_k<NT, false>), grid, dim3(256), 0, stream, x, ldx, x_batch_stride, grad, ldg, \
                           grad_batch_stride, partial, tokens, in_features, out_features, p.tpc, p.nstrip)
    const bool wide_ok = p.wide && ldx % 4 == 0 && ldg % 4 == 0 && x_batch_stride % 4 == 0 &&
                         grad_batch_stride % 4 == 0 && aligned16(x) && aligned16(grad);
    if (wide_ok)
        hipLaunchKernelGGL(xtg_partial_wide_k, grid, dim3(256), 0, stream, x, ldx, x_batch_stride, grad, ldg,
                           grad_batch_stride, partial, tokens, in_features, out_features, p.tpc, p.nstrip);
    else if (p.nt == 4) { SPGT_XTG(4); }
    else if (p.nt == 2) { SPGT_XTG(2); }
    else { SPGT_XTG(1); }
#undef SPGT_XTG
    hipLaunchKernelGGL(tile_reduce, dim3(ceil_div((int)E, 256), batch), dim3(1024), 0, stream, partial, out, (int)E,
                       p.nchunk, 1.0f);
    return check_launch("linear_weight_grad");
}

extern "C" int spgt_dropout_add(const float* y, const float* residual, float* out, int64_t rows, int cols,
                                const uint32_t* seed, float droprate, int site, hipStream_t stream) {
    if (!y || !out || !seed) return fail(SPGT_ERR_INVALID_ARGUMENT, "dropout_add: null pointer argument");
    if (rows < 0 || cols <= 0 || cols % 4 != 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "dropout_add: cols must be a positive multiple of 4");
    if (!(droprate >= 0.f && droprate < 1.f)) return fail(SPGT_ERR_INVALID_ARGUMENT, "dropout_add: the rate must lie in [0, 1)");
    if (!aligned16(y) || !aligned16(out) || (residual && !aligned16(residual)) || !aligned8(seed))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "dropout_add: tensors must be 16-byte aligned, the seed 8-byte aligned");
    if (rows == 0) return SPGT_OK;
    const int64_t pieces = rows * (cols / 4);
    const unsigned grid = (unsigned)std::min<int64_t>(ceil_div(pieces, (int64_t)256), (int64_t)16 * device_cu_count());
    hipLaunchKernelGGL(dropout_add_k, dim3(grid), dim3(256), 0, stream, y, residual, out, pieces, cols / 4, seed, droprate,
                       (uint32_t)site);
    return check_launch("dropout_add");
}

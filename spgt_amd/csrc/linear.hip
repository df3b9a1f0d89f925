// Token-major fused linear layer for the modules either side of the attention:
//   y[t, n]  = sum_k x[t, k] * W[k, n] + bias[n]
//   out[t,n] = act(y + res)          (residual_mode 1)
//            = act(y) + res          (residual_mode 2)
//            = act(y)                (residual_mode 0)
// with act in {identity, ReLU, SiLU}.  It stands in for the nn.Linear calls and
// the elementwise kernels that follow them in the reference's modules:
//   FeedForward.forward                      network/layer.py:155-174
//   Sp_GalerkinAttention fc_layer, residuals network/sp_layer.py:75, 97-103
//   Sp_SpectralConv2D residual_layer + act   network/sp_layer.py:132, 155
//   Sp_DecoderRegressor                      network/sp_model.py:60, 63
//
// One wave owns 32 output columns: its W[:, n0 .. n0+31] stays in registers for
// the whole kernel as the MFMA A operand (column x k).  Token tiles of x go
// through LDS once (coalesced rows in, one k-strided word per lane out as the
// B operand).  The 32x32 accumulator then has output columns along registers
// and tokens along lanes, so a lane stores four 16-byte pieces of its token's
// row.  LDS reads for the next batch of MFMAs are issued before the current
// batch so that their latency hides behind the matrix pipe.
//
// Kernels in this file, all on that scheme:
//   linear_tm_k        any supported shape; several workgroups per CU share the matrix pipes
//   linear_ws_k        long inputs, whole 128-column groups: one MFMA wave per SIMD fed by load and store waves
//   linear_resident_k  the packed 128 -> 384 projection on long inputs: one wave per SIMD, all weights resident
//   ffn_scalar_k       two-layer net with one output feature (regression head)
//   encoder_tail_k     output projection + residuals + feed-forward net of an encoder layer, all weights resident
#include <type_traits>

#include "spgt_device.h"
#include "spgt_host.h"

namespace spgt {

namespace {

// Activation of N values with the choice made once, outside the loop: per-element calls with a run-time
// `act` compile to a branch tree per element, which is most of an epilogue's time.
template <int N>
__device__ __forceinline__ void activate_all(float (&v)[N], int act) {
    if (act == SPGT_ACT_RELU) {
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = fmaxf(v[i], 0.f);
    } else if (act == SPGT_ACT_SILU) {
#pragma unroll
        for (int i = 0; i < N; ++i) v[i] = v[i] * __builtin_amdgcn_rcpf(1.f + __expf(-v[i]));
    }
}

// Epilogue shared by the linear kernels: y = acc + bias (+ extra columns) (+ residual before or after
// the activation), written as four 16-byte pieces of the lane's token row.  Uniform choices (activation,
// residual placement, extra columns) are made once per call, not per element.
template <bool RES>
__device__ __forceinline__ void linear_epilogue(const v16f& acc, const float4 (&bq)[4], const float4* rq, int res_mode,
                                                int act, const float (&x2v)[4], const float* W2row, int ldw, int r2,
                                                float* orow) {
    float y[16];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        y[4 * q + 0] = acc[4 * q + 0] + bq[q].x;
        y[4 * q + 1] = acc[4 * q + 1] + bq[q].y;
        y[4 * q + 2] = acc[4 * q + 2] + bq[q].z;
        y[4 * q + 3] = acc[4 * q + 3] + bq[q].w;
    }
    if (r2 > 0) {
        for (int p = 0; p < r2; ++p) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float4 w4 = *reinterpret_cast<const float4*>(W2row + (int64_t)p * ldw + 8 * q);
                y[4 * q + 0] = fmaf(x2v[p], w4.x, y[4 * q + 0]);
                y[4 * q + 1] = fmaf(x2v[p], w4.y, y[4 * q + 1]);
                y[4 * q + 2] = fmaf(x2v[p], w4.z, y[4 * q + 2]);
                y[4 * q + 3] = fmaf(x2v[p], w4.w, y[4 * q + 3]);
            }
        }
    }
    const float before = (RES && res_mode == SPGT_RES_BEFORE_ACT) ? 1.f : 0.f;
    if (RES) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            y[4 * q + 0] = fmaf(rq[q].x, before, y[4 * q + 0]);
            y[4 * q + 1] = fmaf(rq[q].y, before, y[4 * q + 1]);
            y[4 * q + 2] = fmaf(rq[q].z, before, y[4 * q + 2]);
            y[4 * q + 3] = fmaf(rq[q].w, before, y[4 * q + 3]);
        }
    }
    activate_all(y, act);
    if (RES) {
        const float after = 1.f - before;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            y[4 * q + 0] = fmaf(rq[q].x, after, y[4 * q + 0]);
            y[4 * q + 1] = fmaf(rq[q].y, after, y[4 * q + 1]);
            y[4 * q + 2] = fmaf(rq[q].z, after, y[4 * q + 2]);
            y[4 * q + 3] = fmaf(rq[q].w, after, y[4 * q + 3]);
        }
    }
#pragma unroll
    for (int q = 0; q < 4; ++q)
        *reinterpret_cast<float4*>(orow + 8 * q) = make_float4(y[4 * q], y[4 * q + 1], y[4 * q + 2], y[4 * q + 3]);
}

}  // namespace

// grid (token groups * column groups, rounded up to a multiple of 8), block 256, the column group
// varying fastest so that the workgroups that share an x tile run together, on one XCD.  NCB column blocks of 32 per
// workgroup; the 4/NCB waves that share a column block take different 32-token
// sub-tiles of the workgroup's TT = 32*(4/NCB)-token tile.
template <int K, int NCB, bool RES>
__global__ __launch_bounds__(256) void linear_tm_k(
    const float* __restrict__ x, int64_t ldx, const float* __restrict__ W, int ldw,
    const float* __restrict__ bias, const float* res, int64_t ldr, int res_mode, int act,
    const float* __restrict__ x2, int64_t ldx2, const float* __restrict__ W2, int r2,
    float* out, int64_t ldo, int plane_cols, int64_t plane_stride, int64_t T, int tiles_per_wg, int gy,
    int total_wgs) {
    constexpr int KH = K / 2;
    constexpr int PITCH = K + 1;
    constexpr int TT = 32 * (4 / NCB);
    constexpr int BK = 16;  // MFMAs per LDS read batch
    constexpr int NB = (KH + BK - 1) / BK;
    constexpr int NVEC = TT * K / 4;  // float4 pieces of an x tile
    constexpr int NLD = (NVEC + 255) / 256;
    extern __shared__ float xs[];  // [TT][PITCH]
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int tk = lane & 31;
    const int kh = lane >> 5;
    // Workgroups go round-robin to the 8 XCDs, each with its own L2: consecutive logical ids are mapped
    // onto one XCD so that the column groups of a token tile share the x rows in that L2.
    const int per_xcd = gridDim.x >> 3;
    const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (logical >= total_wgs) return;
    const int cg = logical % gy;
    const int tg = logical / gy;
    const int n0 = (cg * NCB + wave % NCB) * 32;
    const int sub = wave / NCB;

    // A operand: W[2kk + kh][n0 + tk]
    float wreg[KH];
#pragma unroll
    for (int kk = 0; kk < KH; ++kk) wreg[kk] = (W + (int64_t)(2 * kk) * ldw)[(uint32_t)(kh * ldw + n0 + tk)];
    // accumulator element r holds column n0 + 8*(r/4) + 4*kh + r%4; the workgroup's 32*NCB bias values
    // wait in LDS for the epilogue (16 registers less per lane: a third wave per SIMD fits)
    __shared__ __align__(16) float bias_s[32 * NCB];
    if (threadIdx.x < 32 * NCB) bias_s[threadIdx.x] = bias ? bias[cg * NCB * 32 + threadIdx.x] : 0.f;
    const float* bias_l = bias_s + (wave % NCB) * 32 + 4 * kh;
    // output column n lives in plane n / plane_cols at column n % plane_cols
    const int64_t out_col = (n0 / plane_cols) * plane_stride + n0 % plane_cols + 4 * kh;

    const int64_t t_begin = (int64_t)tg * tiles_per_wg * TT;
    const int64_t t_end = min(T, t_begin + (int64_t)tiles_per_wg * TT);
    float4 stage[NLD];
    auto load_tile = [&](int64_t t0) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int e = threadIdx.x + 256 * i;
            const int row = e / (K / 4);
            const int c4 = e % (K / 4);
            const int64_t t = t0 + row;
            stage[i] = (e < NVEC && t < t_end) ? *reinterpret_cast<const float4*>(x + t * ldx + 4 * c4)
                                               : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int e = threadIdx.x + 256 * i;
            if (e < NVEC) {
                const int row = e / (K / 4);
                const int c4 = e % (K / 4);
                float* d = xs + row * PITCH + 4 * c4;
                d[0] = stage[i].x; d[1] = stage[i].y; d[2] = stage[i].z; d[3] = stage[i].w;
            }
        }
    };

    if (t_begin < t_end) load_tile(t_begin);
    for (int64_t t0 = t_begin; t0 < t_end; t0 += TT) {
        __syncthreads();  // previous tile fully consumed
        store_tile();
        __syncthreads();
        if (t0 + TT < t_end) load_tile(t0 + TT);

        const float* xr = xs + (sub * 32 + tk) * PITCH + kh;
        float xv[2][BK];
        auto lds_batch = [&](int bt) {
#pragma unroll
            for (int j = 0; j < BK; ++j)
                if (bt * BK + j < KH) xv[bt & 1][j] = xr[2 * (bt * BK + j)];
        };
        lds_batch(0);
        // the residual is fetched ahead of the MFMAs so that its latency hides behind them
        const int64_t t = t0 + sub * 32 + tk;
        float4 rq[RES ? 4 : 1];
        if (RES) {
#pragma unroll
            for (int q = 0; q < 4; ++q)
                rq[q] = (t < t_end) ? *reinterpret_cast<const float4*>(res + t * ldr + n0 + 4 * kh + 8 * q)
                                    : make_float4(0.f, 0.f, 0.f, 0.f);
        }
        // the few extra input columns (r2 <= 4) are a rank-r2 update of the tile, done on the vector ALU
        float x2v[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int p = 0; p < 4; ++p)
            if (p < r2 && t < t_end) x2v[p] = x2[t * ldx2 + p];
        v16f acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
        for (int bt = 0; bt < NB; ++bt) {
            if (bt + 1 < NB) lds_batch(bt + 1);
            __builtin_amdgcn_sched_barrier(0);  // keep the next batch's reads ahead of this batch's MFMAs
#pragma unroll
            for (int j = 0; j < BK; ++j)
                if (bt * BK + j < KH) acc = mfma32(wreg[bt * BK + j], xv[bt & 1][j], acc);
            __builtin_amdgcn_sched_barrier(0);
        }

        if (t < t_end) {
            float4 bq[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) bq[q] = *reinterpret_cast<const float4*>(bias_l + 8 * q);
            linear_epilogue<RES>(acc, bq, rq, res_mode, act, x2v, W2 + n0 + 4 * kh, ldw, r2, out + out_col + t * ldo);
        }
    }
}

// The same product with the waves of a workgroup split by role.  On this part two waves that both issue
// long chains of fp32 MFMAs with many distinct operand registers share a SIMD badly (a register-only loop
// drops from 136 to 77 TFLOP/s), so there is one MFMA wave per SIMD, and with a single MFMA wave per SIMD
// nothing else fills the matrix pipe while that wave does anything but MFMAs.  So:
//  - the wave's own epilogue is software-pipelined: the residual / activation arithmetic of tile i-1 is
//    spread, a quarter of a 32-token half at a time, between the MFMAs of tile i (two sets of accumulators;
//    the bias is the first MFMA's addend), and its result goes to an LDS output tile rather than to memory;
//  - with 64-token tiles the two 32-token halves are two independent MFMA chains issued alternately, so
//    that no MFMA waits for the one before it;
//  - lane (token, kh) takes k = kh*K/2 + j for MFMA j, so that four consecutive MFMAs' operands are one
//    16-byte LDS read, and rows are K+4 words apart, which makes those reads and the movers' 16-byte
//    writes both free of bank conflicts.
// Alone, the compute waves then take 8400 cycles for the 128 MFMAs of a 64-token tile at 128 input features
// (8192 is the matrix pipe's own time).  What bounds the kernel is the data movement beside them: next to a
// busy MFMA wave, another wave's LDS write or global store of 16 bytes per lane takes about 500 cycles,
// whatever its priority or its target (a global load -> LDS without registers is no quicker once stores
// run beside it), so the 32 + 32 such instructions of a tile are spread over all four SIMDs: 2 load waves
// (global -> registers -> LDS, one tile ahead) and 2 store waves (LDS -> global as whole 512-byte rows, two
// tiles behind) each need about one tile time for their share.
// 512 threads = 4 compute + 2 load + 2 store waves, two LDS buffers each way, one workgroup per CU, one
// barrier per tile.  Used for out_features % 128 == 0 on long inputs without extra input columns.
// grid (slots * column groups), block 512; workgroup (slot, cg) takes tiles slot, slot + slots, ...
template <int K>
struct LinearWs {
    static constexpr int SUBT = (K <= 136) ? 2 : 1;  // 32-token halves per tile = MFMA chains
    static constexpr int TT = 32 * SUBT;
    static constexpr int PITCH = K + 4;   // input tile rows
    static constexpr int OPITCH = 132;    // output tile rows
    static constexpr size_t lds_bytes = (size_t)2 * TT * (PITCH + OPITCH) * sizeof(float);
};

template <int K, bool RES, int ACT>
__global__ __launch_bounds__(512) void linear_ws_k(
    const float* __restrict__ x, int64_t ldx, const float* __restrict__ W, int ldw,
    const float* __restrict__ bias, const float* res, int64_t ldr, int res_mode,
    float* out, int64_t ldo, int plane_cols, int64_t plane_stride, int64_t T, int gy) {
    constexpr int KH = K / 2;
    constexpr int PITCH = LinearWs<K>::PITCH;
    constexpr int OPITCH = LinearWs<K>::OPITCH;
    constexpr int SUBT = LinearWs<K>::SUBT;
    constexpr int TT = LinearWs<K>::TT;
    constexpr int BK = 8;
    constexpr int NB = (KH + BK - 1) / BK;
    constexpr int NVEC = TT * K / 4;
    constexpr int NLD = (NVEC + 127) / 128;
    static_assert(KH % 4 == 0, "16-byte operand reads");
    extern __shared__ float xs[];                 // [2][TT][PITCH]
    float* const os = xs + 2 * TT * PITCH;        // [2][TT][OPITCH]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int cg = blockIdx.x % gy;
    const int slot = blockIdx.x / gy;
    const int slots = gridDim.x / gy;
    const int64_t ntiles = (T + TT - 1) / TT;
    const int64_t mine = slot < ntiles ? (ntiles - slot + slots - 1) / slots : 0;  // tiles of this workgroup
    // Step s (s = 0 .. mine): the compute waves run the MFMAs of tile s (s < mine) and, under them, the epilogue
    // of tile s-1 into output buffer s&1; the store waves write out buffer (s-1)&1 = tile s-2; the load waves
    // put tile s+1's input in place and start the loads of tile s+2.

    if (wave >= 6) {
        // ---- store waves (2): LDS output tile -> global, whole 512-byte rows.  Their stores may wait for
        // room in the memory pipeline; nothing else depends on these waves within a step.
        __builtin_amdgcn_s_setprio(3);  // their few vector ALU instructions otherwise queue behind the MFMA wave's
        const int lt = threadIdx.x - 384;
        // this thread's output pieces: column 4*(lt%32) of the group, rows lt/32 + 4*r
        const int oc = cg * 128 + 4 * (lt & 31);
        float* const ocol = out + (oc / plane_cols) * plane_stride + oc % plane_cols;
        auto flush_tile = [&](int64_t ti) {
            if (ti < 0 || ti >= mine) return;
#pragma unroll
            for (int h = 0; h < TT / 16; ++h) {
                const float* buf = os + (((ti + 1) & 1) * TT + h * 16 + (lt >> 5)) * OPITCH + 4 * (lt & 31);
                const int64_t t0 = (slot + ti * slots) * TT + h * 16;
                float4 v0 = *reinterpret_cast<const float4*>(buf);
                float4 v1 = *reinterpret_cast<const float4*>(buf + 4 * OPITCH);
                float4 v2 = *reinterpret_cast<const float4*>(buf + 8 * OPITCH);
                float4 v3 = *reinterpret_cast<const float4*>(buf + 12 * OPITCH);
                float* const o = ocol + (t0 + (lt >> 5)) * ldo;
                if (t0 + 16 <= T) {
                    // whole block in range: straight-line code, so the reads go out together
                    *reinterpret_cast<float4*>(o) = v0;
                    *reinterpret_cast<float4*>(o + 4 * ldo) = v1;
                    *reinterpret_cast<float4*>(o + 8 * ldo) = v2;
                    *reinterpret_cast<float4*>(o + 12 * ldo) = v3;
                } else {
                    const int64_t left = T - t0 - (lt >> 5);  // rows of this thread's column that exist
                    if (left > 0) *reinterpret_cast<float4*>(o) = v0;
                    if (left > 4) *reinterpret_cast<float4*>(o + 4 * ldo) = v1;
                    if (left > 8) *reinterpret_cast<float4*>(o + 8 * ldo) = v2;
                    if (left > 12) *reinterpret_cast<float4*>(o + 12 * ldo) = v3;
                }
            }
        };
        __syncthreads();  // input buffer 0 ready
        for (int64_t s = 0; s <= mine; ++s) {
            flush_tile(s - 2);
            __syncthreads();  // step s done
        }
        flush_tile(mine - 1);
        return;
    }
    if (wave >= 4) {
        // ---- load waves (2): global -> registers -> LDS input tile, one tile ahead
        __builtin_amdgcn_s_setprio(3);
        const int lt = threadIdx.x - 256;
        float4 stage[NLD];
        auto load_tile = [&](int64_t tile) {
            const int64_t t0 = tile * TT;
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const int e = lt + 128 * i;
                const int row = e / (K / 4);
                const int c4 = e % (K / 4);
                const int64_t t = t0 + row;
                stage[i] = (e < NVEC && t < T) ? *reinterpret_cast<const float4*>(x + t * ldx + 4 * c4)
                                               : make_float4(0.f, 0.f, 0.f, 0.f);
            }
        };
        auto store_tile = [&](float* buf) {
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const int e = lt + 128 * i;
                if (e < NVEC) *reinterpret_cast<float4*>(buf + (e / (K / 4)) * PITCH + 4 * (e % (K / 4))) = stage[i];
            }
        };
        if (mine > 0) {
            load_tile(slot);
            store_tile(xs);
        }
        if (mine > 1) load_tile(slot + slots);
        __syncthreads();  // input buffer 0 ready
        for (int64_t s = 0; s <= mine; ++s) {
            if (s + 1 < mine) store_tile(xs + ((s + 1) & 1) * TT * PITCH);
            if (s + 2 < mine) load_tile(slot + (s + 2) * slots);
            __syncthreads();  // step s done
        }
        return;
    }

    // ---- compute waves: wave w owns columns cg*128 + 32w .. +31
    const int tk = lane & 31;
    const int kh = lane >> 5;
    const int n0 = (cg * 4 + wave) * 32;
    float wreg[KH];  // W[kh*KH + j][n0 + tk]
#pragma unroll
    for (int j = 0; j < KH; ++j) wreg[j] = (W + (int64_t)j * ldw)[(uint32_t)(kh * KH * ldw + n0 + tk)];
    // the bias in accumulator layout: every chain's first MFMA adds to it
    v16f biasv;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const float4 b4 = bias ? *reinterpret_cast<const float4*>(bias + n0 + 4 * kh + 8 * q) : make_float4(0.f, 0.f, 0.f, 0.f);
        biasv[4 * q + 0] = b4.x; biasv[4 * q + 1] = b4.y; biasv[4 * q + 2] = b4.z; biasv[4 * q + 3] = b4.w;
    }
    const float before = (RES && res_mode == SPGT_RES_BEFORE_ACT) ? 1.f : 0.f;
    const float after = 1.f - before;
    v16f acc[2][SUBT];  // [tile parity][chain]
#pragma unroll
    for (int c = 0; c < SUBT; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[0][c][r] = acc[1][c][r] = 0.f;
    __builtin_amdgcn_s_waitcnt(0);  // weights are in: no wait for them is left inside the loop

    // A quarter of an epilogue: residual + activation of values 4q .. 4q+3 of chain c of accumulator set P,
    // as one 16-byte LDS write into this lane's token row.  Straight-line code that the scheduler can spread
    // between MFMAs; a step has 4*SUBT of these.
    auto quarter = [&](auto Pc, int c, int q, const float4& rq, float* orow) {
        constexpr int P = decltype(Pc)::value;
        float y[4] = {acc[P][c][4 * q + 0], acc[P][c][4 * q + 1], acc[P][c][4 * q + 2], acc[P][c][4 * q + 3]};
        if (RES) {
            y[0] = fmaf(rq.x, before, y[0]); y[1] = fmaf(rq.y, before, y[1]);
            y[2] = fmaf(rq.z, before, y[2]); y[3] = fmaf(rq.w, before, y[3]);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            if (ACT == SPGT_ACT_RELU) y[r] = fmaxf(y[r], 0.f);
            if (ACT == SPGT_ACT_SILU) y[r] = y[r] * __builtin_amdgcn_rcpf(1.f + __expf(-y[r]));
        }
        if (RES) {
            y[0] = fmaf(rq.x, after, y[0]); y[1] = fmaf(rq.y, after, y[1]);
            y[2] = fmaf(rq.z, after, y[2]); y[3] = fmaf(rq.w, after, y[3]);
        }
        *reinterpret_cast<float4*>(orow + 8 * q) = make_float4(y[0], y[1], y[2], y[3]);
    };
    // this lane's row of chain c in the output buffer of step s
    auto out_row = [&](int64_t s, int c) { return os + ((s & 1) * TT + c * 32 + tk) * OPITCH + wave * 32 + 4 * kh; };
    // residual rows of tile s-1 (rows outside the input read a valid row: their results are never written out)
    auto load_residual = [&](int64_t s, float4 (&rq)[SUBT][RES ? 4 : 1]) {
        if (!RES) return;
#pragma unroll
        for (int c = 0; c < SUBT; ++c) {
            const int64_t t = min(max((slot + (s - 1) * slots) * TT + c * 32 + tk, (int64_t)0), T - 1);
#pragma unroll
            for (int q = 0; q < 4; ++q) rq[c][q] = *reinterpret_cast<const float4*>(res + t * ldr + n0 + 4 * kh + 8 * q);
        }
    };
    constexpr int NQ = 4 * SUBT;                  // epilogue quarters per step
    constexpr int QPB = (NQ + NB - 1) / NB;       // quarters per batch, from batch 0 on

    // step s < mine: MFMAs of tile s into accumulator set P, epilogue of set P^1 (tile s-1) under the first batches
    auto step = [&](auto Pc, int64_t s) {
        constexpr int P = decltype(Pc)::value;
        const float* xr = xs + ((s & 1) * TT + tk) * PITCH + kh * KH;
        float4 xv[2][SUBT][BK / 4];
#pragma unroll
        for (int c = 0; c < SUBT; ++c)
#pragma unroll
            for (int g = 0; g < BK / 4; ++g) xv[0][c][g] = *reinterpret_cast<const float4*>(xr + c * 32 * PITCH + 4 * g);
        float4 rq[SUBT][RES ? 4 : 1];
        load_residual(s, rq);
#pragma unroll
        for (int bt = 0; bt < NB; ++bt) {
            if (bt + 1 < NB) {
#pragma unroll
                for (int c = 0; c < SUBT; ++c)
#pragma unroll
                    for (int g = 0; g < BK / 4; ++g)
                        if ((bt + 1) * BK + 4 * g < KH)
                            xv[(bt + 1) & 1][c][g] =
                                *reinterpret_cast<const float4*>(xr + c * 32 * PITCH + (bt + 1) * BK + 4 * g);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = bt * QPB; u < (bt + 1) * QPB && u < NQ; ++u)
                quarter(std::integral_constant<int, P ^ 1>{}, u / 4, u % 4, rq[u / 4][RES ? u % 4 : 0], out_row(s, u / 4));
#pragma unroll
            for (int j = 0; j < BK; ++j) {
                if (bt * BK + j < KH) {
                    const int g = j / 4, e = j % 4;
#pragma unroll
                    for (int c = 0; c < SUBT; ++c) {
                        const float4 v4 = xv[bt & 1][c][g];
                        const float b = e == 0 ? v4.x : e == 1 ? v4.y : e == 2 ? v4.z : v4.w;
                        acc[P][c] = mfma32(wreg[bt * BK + j], b, (bt == 0 && j == 0) ? biasv : acc[P][c]);
                    }
                }
            }
            if (bt * QPB < NQ) {
                // one MFMA, then a slice of the epilogue in its shadow
#pragma unroll
                for (int j = 0; j < BK * SUBT; ++j) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, (QPB * 44 + BK * SUBT - 1) / (BK * SUBT), 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // step mine: only the epilogue of the last tile
    auto last_step = [&](auto Pc) {
        constexpr int P = decltype(Pc)::value;
        float4 rq[SUBT][RES ? 4 : 1];
        load_residual(mine, rq);
#pragma unroll
        for (int u = 0; u < NQ; ++u)
            quarter(std::integral_constant<int, P>{}, u / 4, u % 4, rq[u / 4][RES ? u % 4 : 0], out_row(mine, u / 4));
    };

    __syncthreads();  // input buffer 0 ready
    for (int64_t s = 0; s < mine; s += 2) {
        step(std::integral_constant<int, 0>{}, s);
        __syncthreads();  // step s done
        if (s + 1 < mine) {
            step(std::integral_constant<int, 1>{}, s + 1);
            __syncthreads();
        }
    }
    // accumulator set (mine-1)&1 holds the last tile
    if (mine & 1) last_step(std::integral_constant<int, 0>{});
    else if (mine > 0) last_step(std::integral_constant<int, 1>{});
    __syncthreads();  // step mine done
}

// Two-layer feed-forward net with a single output feature:
//   out[t] = sum_n act(x[t, :] . W1[:, n] + b1[n]) * w2[n] + b2
// (FeedForward with out_dim 1, the regression head of network/sp_model.py:51, 63).
// The hidden activations never leave registers.  grid (workgroups), block 256;
// wave w owns hidden columns 32*(w + 4c) .. +31 for c < CBW; HID = 128*CBW.
template <int K, int CBW>
__global__ __launch_bounds__(256) void ffn_scalar_k(
    const float* __restrict__ x, int64_t ldx, const float* __restrict__ W1, const float* __restrict__ b1,
    const float* __restrict__ w2, const float* __restrict__ b2, int act, float* __restrict__ out, int64_t T,
    int tiles_per_wg) {
    constexpr int KH = K / 2;
    constexpr int PITCH = K + 1;
    constexpr int TT = 32;
    constexpr int HID = 128 * CBW;
    constexpr int BK = 16;
    constexpr int NB = (KH + BK - 1) / BK;
    constexpr int NVEC = TT * K / 4;
    constexpr int NLD = (NVEC + 255) / 256;
    __shared__ float xs[TT * PITCH];
    __shared__ float red[4][32];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int tk = lane & 31;
    const int kh = lane >> 5;

    float wreg[CBW][KH], breg[CBW][16], vreg[CBW][16];
#pragma unroll
    for (int c = 0; c < CBW; ++c) {
        const int n0 = 32 * (wave + 4 * c);
#pragma unroll
        for (int kk = 0; kk < KH; ++kk) wreg[c][kk] = (W1 + (int64_t)(2 * kk) * HID)[(uint32_t)(kh * HID + n0 + tk)];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int n = n0 + 8 * (r >> 2) + 4 * kh + (r & 3);
            breg[c][r] = b1 ? b1[n] : 0.f;
            vreg[c][r] = w2[n];
        }
    }
    const float bias2 = b2 ? b2[0] : 0.f;

    const int64_t t_begin = (int64_t)blockIdx.x * tiles_per_wg * TT;
    const int64_t t_end = min(T, t_begin + (int64_t)tiles_per_wg * TT);
    float4 stage[NLD];
    auto load_tile = [&](int64_t t0) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int e = threadIdx.x + 256 * i;
            const int row = e / (K / 4);
            const int c4 = e % (K / 4);
            const int64_t t = t0 + row;
            stage[i] = (e < NVEC && t < t_end) ? *reinterpret_cast<const float4*>(x + t * ldx + 4 * c4)
                                               : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int e = threadIdx.x + 256 * i;
            if (e < NVEC) {
                const int row = e / (K / 4);
                const int c4 = e % (K / 4);
                float* d = xs + row * PITCH + 4 * c4;
                d[0] = stage[i].x; d[1] = stage[i].y; d[2] = stage[i].z; d[3] = stage[i].w;
            }
        }
    };

    if (t_begin < t_end) load_tile(t_begin);
    for (int64_t t0 = t_begin; t0 < t_end; t0 += TT) {
        __syncthreads();  // previous tile and its partial sums fully consumed
        store_tile();
        __syncthreads();
        if (t0 + TT < t_end) load_tile(t0 + TT);

        const float* xr = xs + tk * PITCH + kh;
        float xv[2][BK];
        auto lds_batch = [&](int bt) {
#pragma unroll
            for (int j = 0; j < BK; ++j)
                if (bt * BK + j < KH) xv[bt & 1][j] = xr[2 * (bt * BK + j)];
        };
        lds_batch(0);
        v16f acc[CBW];
#pragma unroll
        for (int c = 0; c < CBW; ++c)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[c][r] = 0.f;
#pragma unroll
        for (int bt = 0; bt < NB; ++bt) {
            if (bt + 1 < NB) lds_batch(bt + 1);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < BK; ++j)
                if (bt * BK + j < KH) {
#pragma unroll
                    for (int c = 0; c < CBW; ++c) acc[c] = mfma32(wreg[c][bt * BK + j], xv[bt & 1][j], acc[c]);
                }
            __builtin_amdgcn_sched_barrier(0);
        }
        // this lane's share of token t0 + tk: 16*CBW hidden columns
        float part = 0.f;
#pragma unroll
        for (int c = 0; c < CBW; ++c) {
                float hv[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) hv[r] = acc[c][r] + breg[c][r];
                activate_all(hv, act);
#pragma unroll
                for (int r = 0; r < 16; ++r) part = fmaf(hv[r], vreg[c][r], part);
            }
        part += __shfl_xor(part, 32, 64);
        if (kh == 0) red[wave][tk] = part;
        __syncthreads();
        if (wave == 0 && kh == 0) {
            const int64_t t = t0 + tk;
            if (t < t_end) out[t] = ((red[0][tk] + red[1][tk]) + (red[2][tk] + red[3][tk])) + bias2;
        }
    }
}

// MFMA with the weight operand and the accumulator in accumulation registers.  A kernel that keeps more than
// 256 registers of weights has most of them there, and the compiler's own form copies each one into a vector
// register first (v_accvgpr_read), which next to a running MFMA costs about 20 cycles per MFMA (85 against 64
// cycles per instruction measured).  The compiler does not see an MFMA in these statements, so the wait states
// it would insert are written out: two before (operand just written by a vector instruction), and
// mfma_acc_done() before the accumulator is read (an MFMA of 16 passes needs 18 after it).
// With SPGT_MFMA_BUILTIN the same helpers are the compiler's intrinsic (which it schedules and protects itself):
// the build makes a second library from that form, and a test compares the two bit for bit, so that a compiler
// change that breaks the hand-counted wait states shows up as a failing test.
#ifdef SPGT_MFMA_BUILTIN
__device__ __forceinline__ void mfma32_acc_first(v16f& acc, float w, float x) {
    v16f zero;
#pragma unroll
    for (int i = 0; i < 16; ++i) zero[i] = 0.f;
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(w, x, zero, 0, 0, 0);
}
__device__ __forceinline__ void mfma32_acc(v16f& acc, float w, float x) {
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(w, x, acc, 0, 0, 0);
}
__device__ __forceinline__ void mfma_acc_done(v16f&) {}
#else
__device__ __forceinline__ void mfma32_acc_first(v16f& acc, float w, float x) {
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x2_f32 %0, %1, %2, 0" : "=a"(acc) : "a"(w), "v"(x));
}
__device__ __forceinline__ void mfma32_acc(v16f& acc, float w, float x) {
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x2_f32 %0, %1, %2, %0" : "+a"(acc) : "a"(w), "v"(x));
}
__device__ __forceinline__ void mfma_acc_done(v16f& acc) { asm volatile("s_nop 15\n\ts_nop 7" : "+a"(acc)); }
#endif

// The tail of an encoder layer after the attention core, one launch per layer
// (Sp_EncoderLayer.forward, network/sp_layer.py:97-103, with the attention's fc_layer, :75, and
// FeedForward, network/layer.py:155-174):
//   y1  = x + a @ Wfc + bfc                       a = attention output [T, K1], x = residual stream [T, 128]
//   out = y1 + act(y1 @ W1 + b1) @ W2 + b2        hidden width 256
// y1 and the hidden activations live in LDS, never in HBM, and every weight is resident: one workgroup of
// four waves per CU, one wave per SIMD, and each wave keeps its 32-column slices of all three weight matrices
// in registers for the whole kernel (68 + 128 + 128 of the 512 a lone wave may use), so the 82k weights are
// read once per CU instead of once per 32 tokens, and a single MFMA wave per SIMD runs at the matrix pipe's
// rate instead of sharing it badly with others.
// Workgroups loop over 32-token tiles (tile = blockIdx.x + i*gridDim.x); the next tile's attention rows and
// residual rows are requested a tile ahead.  Operand layout as in linear_ws_k: lane (token, kh) takes
// k = kh*KK/2 + j for MFMA j, rows KK+4 words apart, 16-byte conflict-free LDS reads; each product runs as two
// independent MFMA chains (the two hidden column blocks of the first feed-forward product, alternate groups
// of four k-steps otherwise).  In-kernel cycle counts per tile (MFMA pipe time 4352 + 8192 + 8192): 4650 +
// 900 epilogue, 10 700 (2500 of it the SiLU epilogue), 9000, 2000 for loads, LDS staging and barriers.
// grid (min(tiles, CUs)), block 256.
// FOLD: the attention's Q.(K^T V / S) product is folded into the output projection.  (Q~ M_h) Wfc_h = Q~ (M_h Wfc_h),
// so `a` is the projected Q [T, 128] itself, Wfc a per-batch matrix [B][128][128] (M folded in, the head's
// feature rows), and the rows of M Wfc that belong to the position columns, summed over the heads, Wpos
// [B][2][128], meet the token's position pos [T][2] as a rank-2 update of y1 (no Wpos: no position columns).
// Tiles then never straddle two of the B sequences of S tokens, a workgroup takes consecutive tiles (so that
// the sequence, and with it the resident fc weights, changes at most a few times), and T = B * S.
// DROP: the reference's two dropouts of an encoder layer (always on, also in inference: F.dropout's default,
// network/sp_layer.py:76 and network/layer.py:173) applied where their operands are formed,
//   y1 = x + dropout(a @ Wfc + bfc, p_fc)        out = y1 + dropout(act(..) @ W2 + b2, p_ffn)
// with the keep decision of element (token t, column n) a hash of (seed, site, t, n) (dropout_site, dropout_apply).
template <int K1, bool FOLD, bool DROP>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void encoder_tail_k(
    const float* __restrict__ a, int64_t lda, const float* __restrict__ x, const float* __restrict__ Wfc,
    const float* __restrict__ bfc, const float* __restrict__ W1, const float* __restrict__ b1,
    const float* __restrict__ W2, const float* __restrict__ b2, int act, float* __restrict__ out, int64_t T,
    const float* __restrict__ Wpos, const float* __restrict__ pos, int64_t S, const uint32_t* __restrict__ seed,
    float p_fc, float p_ffn) {
    static_assert(!FOLD || K1 == 128, "the folded form reads the projected Q");
    constexpr int D = 128, F = 256, TT = 32;
    constexpr int PA = K1 + 4, PY = D + 4, PH = F + 4;
    constexpr int NVEC = TT * K1 / 4;          // 16-byte pieces of an attention tile
    constexpr int NLD = (NVEC + 255) / 256;
    extern __shared__ float lds[];
    float* const bufA = lds;                   // [TT][PA]
    float* const bufY = bufA + TT * PA;        // [TT][PY]
    float* const bufH = bufY + TT * PY;        // [TT][PH]
    float* const bias_s = bufH + TT * PH;      // bfc[128] | b1[256] | b2[128]
    float* const posw_s = bias_s + 512;        // FOLD: Wpos of the current sequence [2][128]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tk = lane & 31;
    const int kh = lane >> 5;
    const int n0 = wave * 32;
    // tile -> first token, end of its sequence; the workgroup's tiles are first, first + step, ... below limit
    const int64_t tpb = FOLD ? (S + TT - 1) / TT : 0;  // tiles per sequence
    const int64_t ntiles = FOLD ? (T / S) * tpb : (T + TT - 1) / TT;
    const int64_t per_wg = (ntiles + gridDim.x - 1) / gridDim.x;
    const int64_t first = FOLD ? blockIdx.x * per_wg : blockIdx.x;
    const int64_t limit = FOLD ? min(ntiles, first + per_wg) : ntiles;
    const int64_t step = FOLD ? 1 : gridDim.x;
    // (tile counts fit 32 bits: the divisions are cheap ones)
    auto tile_seq = [&](int64_t tile) { return FOLD ? (int64_t)((uint32_t)tile / (uint32_t)max(tpb, (int64_t)1)) : (int64_t)0; };
    auto tile_t0 = [&](int64_t tile) {
        if (!FOLD) return tile * TT;
        const int64_t b = tile_seq(tile);
        return b * S + (tile - b * tpb) * TT;
    };
    auto tile_end = [&](int64_t tile) { return FOLD ? (tile_seq(tile) + 1) * S : T; };

    // ---- resident weights: W?[kh*KK/2 + j][column block + tk]
    float wA[K1 / 2], wB[2][D / 2], wC[F / 2];
    auto load_fc = [&](const float* W) {
#pragma unroll
        for (int j = 0; j < K1 / 2; ++j) wA[j] = (W + (int64_t)j * D)[(uint32_t)(kh * (K1 / 2) * D + n0 + tk)];
    };
    if (!FOLD) load_fc(Wfc);
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int j = 0; j < D / 2; ++j) wB[c][j] = (W1 + (int64_t)j * F)[(uint32_t)(kh * (D / 2) * F + n0 + 128 * c + tk)];
#pragma unroll
    for (int j = 0; j < F / 2; ++j) wC[j] = (W2 + (int64_t)j * D)[(uint32_t)(kh * (F / 2) * D + n0 + tk)];
    for (int i = threadIdx.x; i < 512; i += 256)
        bias_s[i] = i < 128 ? bfc[i] : i < 384 ? b1[i - 128] : b2[i - 384];

    // attention rows of a tile: coalesced 16-byte loads into registers, 16-byte LDS writes a tile later.
    // Piece e = threadIdx + 256 i of a tile is row e / (K1/4), columns 4 (e % (K1/4)) ..; its offset from the
    // tile's first row is the same for every tile but for the row clamp (rows past the end read the last row:
    // their results are never written out).
    // (named registers: an array reached through these lambdas ends up in scratch memory)
    static_assert(NLD == 4 || NLD == 5, "attention tile pieces per thread");
    float4 sg0, sg1, sg2, sg3, sg4;
    auto piece_row = [&](int i) { return min((int)threadIdx.x + 256 * i, NVEC - 1) / (K1 / 4); };
    auto piece_col = [&](int i) { return 4 * (min((int)threadIdx.x + 256 * i, NVEC - 1) % (K1 / 4)); };
    const uint32_t ulda = (uint32_t)lda;
    auto load_a = [&](int64_t tile) {
        const int64_t t0 = tile_t0(tile);
        const float* const base = a + t0 * lda;
        const int lastrow = (int)min((int64_t)TT - 1, tile_end(tile) - 1 - t0);  // wave-uniform
        auto ld = [&](int i) {
            return *reinterpret_cast<const float4*>(base + (uint32_t)min(piece_row(i), lastrow) * ulda + (uint32_t)piece_col(i));
        };
        sg0 = ld(0); sg1 = ld(1); sg2 = ld(2); sg3 = ld(3);
        if (NLD > 4) sg4 = ld(4);
    };
    auto store_a = [&]() {
        auto st = [&](int i, const float4& v) {
            if ((int)threadIdx.x + 256 * i < NVEC) *reinterpret_cast<float4*>(bufA + piece_row(i) * PA + piece_col(i)) = v;
        };
        st(0, sg0); st(1, sg1); st(2, sg2); st(3, sg3);
        if (NLD > 4) st(4, sg4);
    };
    // acc0/acc1 += src[tk][k] * w over k-step groups [0, NG) of four; group g goes to chain chain_of(g).
    // Operands are read from LDS 16 k-steps ahead of their MFMAs.
    constexpr int GB = 4;  // groups per operand batch
    auto read_batch = [&](float4 (&xv)[GB], const float* xr, int g0, int NG) {
#pragma unroll
        for (int g = 0; g < GB; ++g)
            if (g0 + g < NG) xv[g] = *reinterpret_cast<const float4*>(xr + 4 * (g0 + g));
    };
    auto comp = [](const float4& v, int e) { return e == 0 ? v.x : e == 1 ? v.y : e == 2 ? v.z : v.w; };

    // residual rows of a tile, requested a tile ahead too (rows past the end read the last row: never written out)
    float4 xq[4];
    float2 pq = make_float2(0.f, 0.f);  // FOLD: the token's position
    auto load_x = [&](int64_t tile) {
        const int64_t row = min(tile_t0(tile) + tk, tile_end(tile) - 1);
#pragma unroll
        for (int q = 0; q < 4; ++q) xq[q] = *reinterpret_cast<const float4*>(x + row * D + n0 + 4 * kh + 8 * q);
        if (FOLD && Wpos) pq = *reinterpret_cast<const float2*>(pos + row * 2);
    };
    int64_t cur_b = -1;  // FOLD: the sequence whose fc weights are resident
    if (first < limit) {
        load_a(first);
        store_a();
        load_x(first);
    }
    __builtin_amdgcn_s_waitcnt(0);  // weights are in: no wait for them is left inside the loop
    __syncthreads();
    for (int64_t tile = first; tile < limit; tile += step) {
        const int64_t t = tile_t0(tile) + tk;
        const bool tok = t < tile_end(tile);
        const bool more = tile + step < limit;
        DropoutSite site_fc, site_ffn;
        if (DROP) {
            site_fc = dropout_site(seed, kDropSiteFc, t, p_fc);
            site_ffn = dropout_site(seed, kDropSiteFfn, t, p_ffn);
        }
        if (FOLD && tile_seq(tile) != cur_b) {
            // another sequence: its fc weights into the registers, its position rows into LDS (last read before
            // the barrier that ended the previous tile)
            cur_b = tile_seq(tile);
            load_fc(Wfc + cur_b * (int64_t)(K1 * D));
            if (Wpos) posw_s[threadIdx.x] = Wpos[cur_b * 2 * D + threadIdx.x];
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
        }
        if (more) load_a(tile + step);

        // ---- y1 = x + a @ Wfc + bfc: wave w owns columns 32w .. 32w+31
        {
            constexpr int NG = K1 / 8;
            const float* xr = bufA + tk * PA + kh * (K1 / 2);
            v16f acc[2];
            float4 xv[2][GB];
            read_batch(xv[0], xr, 0, NG);
#pragma unroll
            for (int g0 = 0; g0 < NG; g0 += GB) {
                if (g0 + GB < NG) read_batch(xv[((g0 / GB) + 1) & 1], xr, g0 + GB, NG);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int g = 0; g < GB; ++g)
                        if (g0 + g < NG) {
                            if (g0 == 0 && e == 0 && g < 2) mfma32_acc_first(acc[g & 1], wA[4 * g + e], comp(xv[0][g], e));
                            else mfma32_acc(acc[g & 1], wA[4 * (g0 + g) + e], comp(xv[(g0 / GB) & 1][g], e));
                        }
                __builtin_amdgcn_sched_barrier(0);
            }
            mfma_acc_done(acc[0]);
            mfma_acc_done(acc[1]);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const float4 bq = *reinterpret_cast<const float4*>(bias_s + n0 + 4 * kh + 8 * q);
                float4 y;
                if (!DROP) {
                    y.x = (acc[0][4 * q + 0] + acc[1][4 * q + 0]) + bq.x + xq[q].x;
                    y.y = (acc[0][4 * q + 1] + acc[1][4 * q + 1]) + bq.y + xq[q].y;
                    y.z = (acc[0][4 * q + 2] + acc[1][4 * q + 2]) + bq.z + xq[q].z;
                    y.w = (acc[0][4 * q + 3] + acc[1][4 * q + 3]) + bq.w + xq[q].w;
                } else {
                    y.x = (acc[0][4 * q + 0] + acc[1][4 * q + 0]) + bq.x;
                    y.y = (acc[0][4 * q + 1] + acc[1][4 * q + 1]) + bq.y;
                    y.z = (acc[0][4 * q + 2] + acc[1][4 * q + 2]) + bq.z;
                    y.w = (acc[0][4 * q + 3] + acc[1][4 * q + 3]) + bq.w;
                }
                if (FOLD && Wpos) {
                    const float4 w0 = *reinterpret_cast<const float4*>(posw_s + n0 + 4 * kh + 8 * q);
                    const float4 w1 = *reinterpret_cast<const float4*>(posw_s + D + n0 + 4 * kh + 8 * q);
                    y.x += pq.x * w0.x + pq.y * w1.x; y.y += pq.x * w0.y + pq.y * w1.y;
                    y.z += pq.x * w0.z + pq.y * w1.z; y.w += pq.x * w0.w + pq.y * w1.w;
                }
                if (DROP) {
                    // the whole output of fc_layer (bias and position rows included) is what the reference drops
                    const int n = n0 + 4 * kh + 8 * q;
                    y.x = dropout_apply(site_fc, n + 0, y.x) + xq[q].x;
                    y.y = dropout_apply(site_fc, n + 1, y.y) + xq[q].y;
                    y.z = dropout_apply(site_fc, n + 2, y.z) + xq[q].z;
                    y.w = dropout_apply(site_fc, n + 3, y.w) + xq[q].w;
                }
                *reinterpret_cast<float4*>(bufY + tk * PY + n0 + 8 * q + 4 * kh) = y;
            }
        }
        if (more) load_x(tile + step);
        __syncthreads();  // bufY complete

        // ---- h = act(y1 @ W1 + b1): wave w owns hidden column blocks w and w + 4, one MFMA chain each
        {
            constexpr int NG = D / 8;
            const float* xr = bufY + tk * PY + kh * (D / 2);
            v16f acc[2];
            float4 xv[2][GB];
            read_batch(xv[0], xr, 0, NG);
#pragma unroll
            for (int g0 = 0; g0 < NG; g0 += GB) {
                if (g0 + GB < NG) read_batch(xv[((g0 / GB) + 1) & 1], xr, g0 + GB, NG);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int g = 0; g < GB; ++g)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float b = comp(xv[(g0 / GB) & 1][g], e);
                        if (g0 == 0 && g == 0 && e == 0) {
                            mfma32_acc_first(acc[0], wB[0][0], b);
                            mfma32_acc_first(acc[1], wB[1][0], b);
                        } else {
                            mfma32_acc(acc[0], wB[0][4 * (g0 + g) + e], b);
                            mfma32_acc(acc[1], wB[1][4 * (g0 + g) + e], b);
                        }
                    }
                __builtin_amdgcn_sched_barrier(0);
            }
            mfma_acc_done(acc[0]);
            mfma_acc_done(acc[1]);
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                float hv[16];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float4 bq = *reinterpret_cast<const float4*>(bias_s + 128 + n0 + 128 * c + 4 * kh + 8 * q);
                    hv[4 * q + 0] = acc[c][4 * q + 0] + bq.x;
                    hv[4 * q + 1] = acc[c][4 * q + 1] + bq.y;
                    hv[4 * q + 2] = acc[c][4 * q + 2] + bq.z;
                    hv[4 * q + 3] = acc[c][4 * q + 3] + bq.w;
                }
                activate_all(hv, act);
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    *reinterpret_cast<float4*>(bufH + tk * PH + n0 + 128 * c + 8 * q + 4 * kh) =
                        make_float4(hv[4 * q + 0], hv[4 * q + 1], hv[4 * q + 2], hv[4 * q + 3]);
            }
        }
        __syncthreads();  // bufH complete

        // ---- out = y1 + h @ W2 + b2
        {
            constexpr int NG = F / 8;
            const float* xr = bufH + tk * PH + kh * (F / 2);
            v16f acc[2];
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[0][r] = acc[1][r] = 0.f;
            float4 xv[2][GB];
            read_batch(xv[0], xr, 0, NG);
#pragma unroll
            for (int g0 = 0; g0 < NG; g0 += GB) {
                if (g0 + GB < NG) read_batch(xv[((g0 / GB) + 1) & 1], xr, g0 + GB, NG);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int e = 0; e < 4; ++e)
#pragma unroll
                    for (int g = 0; g < GB; ++g)
                        acc[g & 1] = mfma32(wC[4 * (g0 + g) + e], comp(xv[(g0 / GB) & 1][g], e), acc[g & 1]);
                __builtin_amdgcn_sched_barrier(0);
            }
            // the next tile's attention rows go to LDS before this tile's stores are issued: the wait for
            // their loads would otherwise also wait for those stores (bufA was last read two barriers ago)
            if (more) store_a();
            if (tok) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float4 bq = *reinterpret_cast<const float4*>(bias_s + 384 + n0 + 4 * kh + 8 * q);
                    const float4 y1 = *reinterpret_cast<const float4*>(bufY + tk * PY + n0 + 8 * q + 4 * kh);
                    float4 o;
                    if (!DROP) {
                        o.x = (acc[0][4 * q + 0] + acc[1][4 * q + 0]) + bq.x + y1.x;
                        o.y = (acc[0][4 * q + 1] + acc[1][4 * q + 1]) + bq.y + y1.y;
                        o.z = (acc[0][4 * q + 2] + acc[1][4 * q + 2]) + bq.z + y1.z;
                        o.w = (acc[0][4 * q + 3] + acc[1][4 * q + 3]) + bq.w + y1.w;
                    } else {
                        const int n = n0 + 4 * kh + 8 * q;
                        o.x = dropout_apply(site_ffn, n + 0, (acc[0][4 * q + 0] + acc[1][4 * q + 0]) + bq.x) + y1.x;
                        o.y = dropout_apply(site_ffn, n + 1, (acc[0][4 * q + 1] + acc[1][4 * q + 1]) + bq.y) + y1.y;
                        o.z = dropout_apply(site_ffn, n + 2, (acc[0][4 * q + 2] + acc[1][4 * q + 2]) + bq.z) + y1.z;
                        o.w = dropout_apply(site_ffn, n + 3, (acc[0][4 * q + 3] + acc[1][4 * q + 3]) + bq.w) + y1.w;
                    }
                    *reinterpret_cast<float4*>(out + t * D + n0 + 4 * kh + 8 * q) = o;
                }
            }
        }
        __syncthreads();  // next tile's bufA in place; bufH free
    }
}

// The weight operand in a vector register, the accumulator in accumulation registers.
#ifdef SPGT_MFMA_BUILTIN
__device__ __forceinline__ void mfma32_accv_first(v16f& acc, float w, float x) { mfma32_acc_first(acc, w, x); }
__device__ __forceinline__ void mfma32_accv(v16f& acc, float w, float x) { mfma32_acc(acc, w, x); }
#else
__device__ __forceinline__ void mfma32_accv_first(v16f& acc, float w, float x) {
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x2_f32 %0, %1, %2, 0" : "=a"(acc) : "v"(w), "v"(x));
}
__device__ __forceinline__ void mfma32_accv(v16f& acc, float w, float x) {
    asm volatile("s_nop 1\n\tv_mfma_f32_32x32x2_f32 %0, %1, %2, %0" : "+a"(acc) : "v"(w), "v"(x));
}
#endif

// Wide linear layers on long inputs with every weight resident (the structure of encoder_tail_k):
//   out[t, n] = act(x[t, :] . W[:, n] + bias[n]),  in_features 128, out_features 128*NCB,
// no residual and no extra columns; used for the packed Q|K|V projection (NCB 3, output planes).  One workgroup of four waves per CU; wave w owns the 32-column blocks w, w+4,
// (w+8) and keeps their weights in registers for the whole kernel (64 per block: two blocks in accumulation
// registers, a third in vector registers).  Workgroups loop over 32-token tiles.  Per tile a wave runs NCB
// independent MFMA chains off one 16-byte LDS operand read per four k-steps; the bias / activation / store of
// the previous tile (second set of accumulators) is placed by hand between the MFMAs, a quarter block at a
// time, because the MFMAs are assembly statements that the scheduler neither moves nor counts.  The next
// tile's rows are requested at the start of a tile and written to the other LDS buffer at its end; one
// barrier per tile.  grid (min(tiles, CUs)), block 256.
template <int NCB, int ACT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void linear_resident_k(
    const float* __restrict__ x, int64_t ldx, const float* __restrict__ W, const float* __restrict__ bias,
    float* __restrict__ out, int64_t ldo, int plane_cols, int64_t plane_stride, int64_t T) {
    constexpr int K = 128, KH = 64, TT = 32, PX = K + 4, N = 128 * NCB;
    constexpr int NCA = NCB < 2 ? NCB : 2;  // column blocks with weights in accumulation registers
    constexpr int NCV = NCB - NCA;          // ... in vector registers
    constexpr int GB = 4;                   // 16-byte operand pieces per batch
    extern __shared__ float lds[];
    float* const xs = lds;                      // [2][TT][PX]
    float* const bias_s = xs + 2 * TT * PX;     // [N]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tk = lane & 31;
    const int kh = lane >> 5;
    const int64_t ntiles = (T + TT - 1) / TT;

    // ---- resident weights: W[kh*KH + j][32*(wave + 4c) + tk]
    float wa[NCA][KH], wv[NCV > 0 ? NCV : 1][KH];
#pragma unroll
    for (int c = 0; c < NCB; ++c)
#pragma unroll
        for (int j = 0; j < KH; ++j) {
            const float w = (W + (int64_t)j * N)[(uint32_t)(kh * KH * N + 32 * (wave + 4 * c) + tk)];
            if (c < NCA) wa[c][j] = w;
            else wv[c - NCA][j] = w;
        }
    for (int i = threadIdx.x; i < N; i += 256) bias_s[i] = bias ? bias[i] : 0.f;
    // where this lane's 16-byte pieces of column block c start in a row of the output
    int64_t ocol[NCB];
#pragma unroll
    for (int c = 0; c < NCB; ++c) {
        const int n0 = 32 * (wave + 4 * c);
        ocol[c] = (n0 / plane_cols) * plane_stride + n0 % plane_cols + 4 * kh;
    }

    // input rows of a tile: coalesced 16-byte loads into registers, 16-byte LDS writes a tile later
    // (thread -> row threadIdx/32 + 8i, piece threadIdx%32; rows past the end read the last row)
    float4 st0, st1, st2, st3;
    const float* const xcol = x + 4 * (threadIdx.x & 31);
    const int srow = threadIdx.x >> 5;
    auto load_x = [&](int64_t tile) {
        const int64_t r0 = tile * TT + srow;
        st0 = *reinterpret_cast<const float4*>(xcol + min(r0, T - 1) * ldx);
        st1 = *reinterpret_cast<const float4*>(xcol + min(r0 + 8, T - 1) * ldx);
        st2 = *reinterpret_cast<const float4*>(xcol + min(r0 + 16, T - 1) * ldx);
        st3 = *reinterpret_cast<const float4*>(xcol + min(r0 + 24, T - 1) * ldx);
    };
    auto store_x = [&](int b) {
        float* const d = xs + (b * TT + srow) * PX + 4 * (threadIdx.x & 31);
        *reinterpret_cast<float4*>(d) = st0;
        *reinterpret_cast<float4*>(d + 8 * PX) = st1;
        *reinterpret_cast<float4*>(d + 16 * PX) = st2;
        *reinterpret_cast<float4*>(d + 24 * PX) = st3;
    };
    auto comp = [](const float4& v, int e) { return e == 0 ? v.x : e == 1 ? v.y : e == 2 ? v.z : v.w; };

    v16f acc[2][NCB];  // [tile parity][column block]
    // bias, activation and store of values 4q .. 4q+3 of column block c of accumulator set P, for row t
    auto quarter = [&](auto Pc, int c, int q, int64_t t) {
        constexpr int P = decltype(Pc)::value;
        const float4 b4 = *reinterpret_cast<const float4*>(bias_s + 32 * (wave + 4 * c) + 4 * kh + 8 * q);
        float y[4] = {acc[P][c][4 * q + 0] + b4.x, acc[P][c][4 * q + 1] + b4.y, acc[P][c][4 * q + 2] + b4.z,
                      acc[P][c][4 * q + 3] + b4.w};
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            if (ACT == SPGT_ACT_RELU) y[r] = fmaxf(y[r], 0.f);
            if (ACT == SPGT_ACT_SILU) y[r] = y[r] * __builtin_amdgcn_rcpf(1.f + __expf(-y[r]));
        }
        if (t < T) *reinterpret_cast<float4*>(out + ocol[c] + t * ldo + 8 * q) = make_float4(y[0], y[1], y[2], y[3]);
    };
    auto mma = [&](auto Pc, int c, int j, float b, bool first) {
        constexpr int P = decltype(Pc)::value;
        if (c < NCA) {
            if (first) mfma32_acc_first(acc[P][c], wa[c][j], b);
            else mfma32_acc(acc[P][c], wa[c][j], b);
        } else {
            if (first) mfma32_accv_first(acc[P][c], wv[c - NCA][j], b);
            else mfma32_accv(acc[P][c], wv[c - NCA][j], b);
        }
    };
    // tile number i of this workgroup (LDS buffer i&1) into accumulator set P; between its MFMAs the
    // epilogue of set P^1 = the tile before, whose first row is tprev0 (none if negative)
    auto step = [&](auto Pc, int64_t i, int64_t tile, int64_t tprev0) {
        constexpr int P = decltype(Pc)::value;
        const bool more = tile + gridDim.x < ntiles;
        if (more) load_x(tile + gridDim.x);
        const float* xr = xs + ((int)(i & 1) * TT + tk) * PX + kh * KH;
        float4 xv[2][GB];
#pragma unroll
        for (int g = 0; g < GB; ++g) xv[0][g] = *reinterpret_cast<const float4*>(xr + 4 * g);
#pragma unroll
        for (int g0 = 0; g0 < KH / 4; g0 += GB) {
            if (g0 + GB < KH / 4) {
#pragma unroll
                for (int g = 0; g < GB; ++g)
                    xv[((g0 / GB) + 1) & 1][g] = *reinterpret_cast<const float4*>(xr + 4 * (g0 + GB + g));
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int g = 0; g < GB; ++g) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float b = comp(xv[(g0 / GB) & 1][g], e);
#pragma unroll
                    for (int c = 0; c < NCB; ++c) mma(Pc, c, 4 * (g0 + g) + e, b, g0 + g == 0 && e == 0);
                }
                // one quarter of the previous tile's epilogue after each group of four k-steps
                const int u = g0 + g;
                if (u < 4 * NCB && tprev0 >= 0) quarter(std::integral_constant<int, P ^ 1>{}, u / 4, u % 4, tprev0 + tk);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // the compiler does not know that set P was written by MFMAs: keep any read of it the needed distance away
#pragma unroll
        for (int c = 0; c < NCB; ++c) mfma_acc_done(acc[P][c]);
        if (more) store_x((int)((i + 1) & 1));
        __syncthreads();  // next tile in place; this tile's buffer free for the tile after
    };

    const int64_t first = blockIdx.x;
    if (first < ntiles) {
        load_x(first);
        store_x(0);
    }
    __builtin_amdgcn_s_waitcnt(0);  // weights are in: no wait for them is left inside the loop
    __syncthreads();
    int64_t i = 0, tprev0 = -1;
    for (int64_t tile = first; tile < ntiles; tile += 2 * (int64_t)gridDim.x, i += 2) {
        step(std::integral_constant<int, 0>{}, i, tile, tprev0);
        tprev0 = tile * TT;
        const int64_t tile1 = tile + gridDim.x;
        if (tile1 < ntiles) {
            step(std::integral_constant<int, 1>{}, i + 1, tile1, tprev0);
            tprev0 = tile1 * TT;
        } else {
            // the last tile went into set 0
#pragma unroll
            for (int u = 0; u < 4 * NCB; ++u) quarter(std::integral_constant<int, 0>{}, u / 4, u % 4, tprev0 + tk);
            return;
        }
    }
    if (tprev0 >= 0) {
        // the last tile went into set 1
#pragma unroll
        for (int u = 0; u < 4 * NCB; ++u) quarter(std::integral_constant<int, 1>{}, u / 4, u % 4, tprev0 + tk);
    }
}

namespace {

// Tiles per workgroup.  Measured on MI355X at 356k tokens: grids of 2 or 4 workgroups per CU run the
// 128 -> 384 product in 355-370 us, a grid of 3 per CU in 450-520 us, whether two or three workgroups
// fit on a CU at once.  The plan therefore counts workgroups per CU in pairs (an odd one costs as much
// as two), takes the cheapest tiles_per_wg, and among equals the one closest to two per CU (fewer
// re-reads of W than with more, something to overlap with unlike one).
inline int pick_tiles_per_wg(int64_t tiles, int gy, int cus) {
    int best = 1;
    int64_t best_cost = INT64_MAX;
    double best_dist = 0;
    for (int tpw = 1; tpw <= 64; ++tpw) {
        const int64_t wgs = ceil_div(tiles, (int64_t)tpw) * gy;
        const int64_t per_cu = ceil_div(wgs, (int64_t)cus);
        const int64_t cost = tpw * 2 * ceil_div(per_cu, (int64_t)2);
        const double dist = per_cu >= 2 ? (double)per_cu / 2 : 2.5;
        if (cost < best_cost || (cost == best_cost && dist < best_dist)) {
            best = tpw;
            best_cost = cost;
            best_dist = dist;
        }
        if (wgs <= gy) break;
    }
    return best;
}

template <int K, int NCB, bool RES>
void launch_linear(const float* x, int64_t ldx, const float* W, const float* bias, const float* res, int64_t ldr,
                   int res_mode, int act, const float* x2, int64_t ldx2, const float* W2, int r2, float* out,
                   int64_t ldo, int plane_cols, int64_t plane_stride, int64_t T, int N, hipStream_t stream) {
    constexpr int TT = 32 * (4 / NCB);
    const size_t lds = (size_t)TT * (K + 1) * sizeof(float);
    const int gy = N / (32 * NCB);
    const int64_t tiles = ceil_div(T, (int64_t)TT);
    auto kernel = linear_tm_k<K, NCB, RES>;
    const int tpw = pick_tiles_per_wg(tiles, gy, device_cu_count());
    const int total_wgs = (int)(ceil_div(tiles, (int64_t)tpw) * gy);
    // More than two workgroups per CU run in rounds of two (see pick_tiles_per_wg): asking for more
    // than a third of the CU's 160 KB of LDS keeps a third workgroup from joining a round.
    size_t lds_request = lds;
    if (total_wgs > 2 * device_cu_count()) lds_request = std::max<size_t>(lds, 72 * 1024);
    const dim3 grid((unsigned)(ceil_div(total_wgs, 8) * 8));  // whole rounds over the 8 XCDs
    (void)allow_dynamic_lds(kernel, lds_request);
    hipLaunchKernelGGL(kernel, grid, dim3(256), lds_request, stream, x, ldx, W, N, bias, res, ldr, res_mode, act, x2, ldx2, W2,
                       r2, out, ldo, plane_cols, plane_stride, T, tpw, gy, total_wgs);
}

template <int K, bool RES, int ACT>
void launch_linear_ws(const float* x, int64_t ldx, const float* W, const float* bias, const float* res, int64_t ldr,
                      int res_mode, float* out, int64_t ldo, int plane_cols, int64_t plane_stride, int64_t T, int N,
                      hipStream_t stream) {
    const int gy = N / 128;
    const int slots = std::max(1, device_cu_count() / gy);  // one workgroup per CU
    // at least half of the CU's LDS so that no second workgroup joins
    const size_t lds = std::max<size_t>(LinearWs<K>::lds_bytes, 84 * 1024);
    auto kernel = linear_ws_k<K, RES, ACT>;
    (void)allow_dynamic_lds(kernel, lds);
    hipLaunchKernelGGL(kernel, dim3(slots * gy), dim3(512), lds, stream, x, ldx, W, N, bias, res, ldr, res_mode, out,
                       ldo, plane_cols, plane_stride, T, gy);
}

template <int K, bool RES>
void launch_linear_ws_act(const float* x, int64_t ldx, const float* W, const float* bias, const float* res, int64_t ldr,
                          int res_mode, int act, float* out, int64_t ldo, int plane_cols, int64_t plane_stride,
                          int64_t T, int N, hipStream_t stream) {
#define SPGT_WS_ARGS x, ldx, W, bias, res, ldr, res_mode, out, ldo, plane_cols, plane_stride, T, N, stream
    if (act == SPGT_ACT_RELU) launch_linear_ws<K, RES, SPGT_ACT_RELU>(SPGT_WS_ARGS);
    else if (act == SPGT_ACT_SILU) launch_linear_ws<K, RES, SPGT_ACT_SILU>(SPGT_WS_ARGS);
    else launch_linear_ws<K, RES, SPGT_ACT_NONE>(SPGT_WS_ARGS);
#undef SPGT_WS_ARGS
}

template <int NCB>
void launch_linear_resident(const float* x, int64_t ldx, const float* W, const float* bias, int act, float* out,
                            int64_t ldo, int plane_cols, int64_t plane_stride, int64_t T, hipStream_t stream) {
    const unsigned grid = (unsigned)std::min<int64_t>(ceil_div(T, (int64_t)32), device_cu_count());
    const size_t lds = std::max<size_t>(((size_t)2 * 32 * 132 + 128 * NCB) * sizeof(float), 84 * 1024);
#define SPGT_RES_LAUNCH(ACT)                                                                                  \
    {                                                                                                         \
        auto kernel = linear_resident_k<NCB, ACT>;                                                            \
        (void)allow_dynamic_lds(kernel, lds);                                                                 \
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), lds, stream, x, ldx, W, bias, out, ldo, plane_cols, \
                           plane_stride, T);                                                                  \
    }
    if (act == SPGT_ACT_RELU) SPGT_RES_LAUNCH(SPGT_ACT_RELU)
    else if (act == SPGT_ACT_SILU) SPGT_RES_LAUNCH(SPGT_ACT_SILU)
    else SPGT_RES_LAUNCH(SPGT_ACT_NONE)
#undef SPGT_RES_LAUNCH
}

template <int K>
void launch_linear_k(int ncb, const float* x, int64_t ldx, const float* W, const float* bias, const float* res,
                     int64_t ldr, int res_mode, int act, const float* x2, int64_t ldx2, const float* W2, int r2,
                     float* out, int64_t ldo, int plane_cols, int64_t plane_stride, int64_t T, int N,
                     hipStream_t stream) {
#define SPGT_ARGS x, ldx, W, bias, res, ldr, res_mode, act, x2, ldx2, W2, r2, out, ldo, plane_cols, plane_stride, T, N, stream
    // 128 -> 384 without residual or extra columns on long inputs (the packed Q|K|V projection): every weight
    // resident in registers, 6 % faster than the role-split kernel at 356k and 159k tokens (128 -> 256 is not)
    if constexpr (K == 128) {
        if (N == 384 && r2 == 0 && res_mode == SPGT_RES_NONE && T >= (int64_t)256 * device_cu_count()) {
            launch_linear_resident<3>(x, ldx, W, bias, act, out, ldo, plane_cols, plane_stride, T, stream);
            return;
        }
    }
    // Long inputs with whole 128-column groups and no extra columns: role-split workgroups, one per CU.
    // With 256 input features they win from one 64-token tile per CU on; with fewer, from four on (below
    // that the plain kernel's finer split balances the CUs better).
    const int64_t ws_tokens = (int64_t)(K >= 256 ? 64 : 256) * device_cu_count();
    if (ncb == 4 && r2 == 0 && T >= ws_tokens && N / 128 <= device_cu_count()) {
        if (res_mode != SPGT_RES_NONE)
            launch_linear_ws_act<K, true>(x, ldx, W, bias, res, ldr, res_mode, act, out, ldo, plane_cols, plane_stride, T, N, stream);
        else
            launch_linear_ws_act<K, false>(x, ldx, W, bias, res, ldr, res_mode, act, out, ldo, plane_cols, plane_stride, T, N, stream);
        return;
    }
    if (res_mode != SPGT_RES_NONE) {
        if (ncb == 4) launch_linear<K, 4, true>(SPGT_ARGS);
        else if (ncb == 2) launch_linear<K, 2, true>(SPGT_ARGS);
        else launch_linear<K, 1, true>(SPGT_ARGS);
    } else {
        if (ncb == 4) launch_linear<K, 4, false>(SPGT_ARGS);
        else if (ncb == 2) launch_linear<K, 2, false>(SPGT_ARGS);
        else launch_linear<K, 1, false>(SPGT_ARGS);
    }
#undef SPGT_ARGS
}

template <int K, int CBW>
void launch_ffn_scalar(const float* x, int64_t ldx, const float* W1, const float* b1, const float* w2, const float* b2,
                       int act, float* out, int64_t T, hipStream_t stream) {
    const int64_t tiles = ceil_div(T, (int64_t)32);
    const int tpw = pick_tiles_per_wg(tiles, 1, device_cu_count());
    hipLaunchKernelGGL((ffn_scalar_k<K, CBW>), dim3((unsigned)ceil_div(tiles, (int64_t)tpw)), dim3(256), 0, stream, x,
                       ldx, W1, b1, w2, b2, act, out, T, tpw);
}

}  // namespace

}  // namespace spgt

using namespace spgt;

extern "C" int spgt_linear_supported(int in_features, int out_features) {
    const bool k_ok = in_features == 64 || in_features == 128 || in_features == 136 || in_features == 256;
    return (k_ok && out_features > 0 && out_features % 32 == 0 && out_features <= 65535 * 32) ? 1 : 0;
}

extern "C" int spgt_linear_forward(const float* x, int64_t ldx, const float* weight_kn, const float* bias,
                                   const float* residual, int64_t ldr, int residual_mode, int activation,
                                   const float* x_extra, int64_t ldx_extra, const float* weight_extra_kn,
                                   int extra_features, float* out, int64_t ldo, int out_plane_cols,
                                   int64_t out_plane_stride, int64_t tokens, int in_features, int out_features,
                                   hipStream_t stream) {
    if (!x || !weight_kn || !out) return fail(SPGT_ERR_INVALID_ARGUMENT, "linear_forward: null pointer argument");
    if (tokens < 0) return fail(SPGT_ERR_INVALID_ARGUMENT, "linear_forward: negative token count");
    if (!spgt_linear_supported(in_features, out_features))
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "linear_forward: in_features must be 64, 128, 136 or 256 and out_features a multiple of 32");
    if (activation != SPGT_ACT_NONE && activation != SPGT_ACT_RELU && activation != SPGT_ACT_SILU)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "linear_forward: unknown activation");
    if (residual_mode != SPGT_RES_NONE && residual_mode != SPGT_RES_BEFORE_ACT && residual_mode != SPGT_RES_AFTER_ACT)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "linear_forward: unknown residual_mode");
    if (residual_mode != SPGT_RES_NONE && !residual)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "linear_forward: residual is null with a residual_mode");
    if (extra_features < 0 || extra_features > 4)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "linear_forward: extra_features must be 0..4");
    if (extra_features > 0 && (!x_extra || !weight_extra_kn || ldx_extra < extra_features || !aligned4(x_extra) ||
                               !aligned16(weight_extra_kn)))
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "linear_forward: x_extra / weight_extra_kn missing, misaligned or with too small a row stride");
    if (out_plane_cols <= 0 || out_plane_cols > out_features) out_plane_cols = out_features;
    if (out_plane_cols % 32 != 0 || out_features % out_plane_cols != 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "linear_forward: out_plane_cols must be a multiple of 32 that divides out_features");
    if (out_plane_cols < out_features && (out_plane_stride & 3))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "linear_forward: out_plane_stride must be a multiple of 4");
    if (ldx < in_features || ldo < out_plane_cols || (residual_mode && ldr < out_features))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "linear_forward: a row stride is smaller than its row");
    if ((ldx & 3) || (ldo & 3) || (residual_mode && (ldr & 3)) || !aligned16(x) || !aligned16(out) ||
        (residual_mode && !aligned16(residual)) || !aligned4(weight_kn) || (bias && !aligned4(bias)))
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "linear_forward: x, residual and out must be 16-byte aligned with row strides that are multiples of 4");
    if (tokens == 0) return SPGT_OK;
    const int ncb = out_features % 128 == 0 ? 4 : (out_features % 64 == 0 ? 2 : 1);
    const float* res = residual_mode ? residual : nullptr;
#define SPGT_LIN(KV) \
    launch_linear_k<KV>(ncb, x, ldx, weight_kn, bias, res, ldr, residual_mode, activation, x_extra, ldx_extra,      \
                        weight_extra_kn, extra_features, out, ldo, out_plane_cols, out_plane_stride, tokens,        \
                        out_features, stream)
    switch (in_features) {
        case 64: SPGT_LIN(64); break;
        case 128: SPGT_LIN(128); break;
        case 136: SPGT_LIN(136); break;
        default: SPGT_LIN(256); break;
    }
#undef SPGT_LIN
    return check_launch("linear_forward");
}

extern "C" int spgt_ffn_scalar_supported(int in_features, int hidden_features) {
    return ((in_features == 32 || in_features == 64 || in_features == 128) &&
            (hidden_features == 128 || hidden_features == 256)) ? 1 : 0;
}

extern "C" int spgt_ffn_scalar_forward(const float* x, int64_t ldx, const float* weight1_kn, const float* bias1,
                                       const float* weight2, const float* bias2, int activation, float* out,
                                       int64_t tokens, int in_features, int hidden_features, hipStream_t stream) {
    if (!x || !weight1_kn || !weight2 || !out)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "ffn_scalar_forward: null pointer argument");
    if (tokens < 0) return fail(SPGT_ERR_INVALID_ARGUMENT, "ffn_scalar_forward: negative token count");
    if (!spgt_ffn_scalar_supported(in_features, hidden_features))
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "ffn_scalar_forward: in_features must be 32, 64 or 128 and hidden_features 128 or 256");
    if (activation != SPGT_ACT_NONE && activation != SPGT_ACT_RELU && activation != SPGT_ACT_SILU)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "ffn_scalar_forward: unknown activation");
    if (ldx < in_features || (ldx & 3) || !aligned16(x) || !aligned4(out) || !aligned4(weight1_kn) ||
        !aligned4(weight2))
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "ffn_scalar_forward: x must be 16-byte aligned with a row stride that is a multiple of 4");
    if (tokens == 0) return SPGT_OK;
#define SPGT_FFN(KV, CB) \
    launch_ffn_scalar<KV, CB>(x, ldx, weight1_kn, bias1, weight2, bias2, activation, out, tokens, stream)
    if (in_features == 32)      { if (hidden_features == 128) SPGT_FFN(32, 1); else SPGT_FFN(32, 2); }
    else if (in_features == 64) { if (hidden_features == 128) SPGT_FFN(64, 1); else SPGT_FFN(64, 2); }
    else                        { if (hidden_features == 128) SPGT_FFN(128, 1); else SPGT_FFN(128, 2); }
#undef SPGT_FFN
    return check_launch("ffn_scalar_forward");
}

namespace {

int dropout_args_ok(const uint32_t* seed, float p_fc, float p_ffn) {
    if (!(p_fc >= 0.f && p_fc < 1.f) || !(p_ffn >= 0.f && p_ffn < 1.f))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "encoder_tail dropout: drop rates must lie in [0, 1)");
    if ((p_fc > 0.f || p_ffn > 0.f) && (!seed || !aligned8(seed)))
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "encoder_tail dropout: drop rates above 0 need an 8-byte aligned seed (two 32-bit words) in device memory");
    return SPGT_OK;
}

int encoder_tail_folded_common(const float* q, int64_t ld_q, const float* position, const float* x,
                               const float* folded_fc, const float* folded_pos, const float* fc_bias,
                               const float* ffn1_weight_kn, const float* ffn1_bias, const float* ffn2_weight_kn,
                               const float* ffn2_bias, int activation, float* out, int B, int64_t S, int dp,
                               int dim_hidden, int ffn_hidden, const uint32_t* seed, float p_fc, float p_ffn,
                               hipStream_t stream) {
    if (!q || !x || !folded_fc || !fc_bias || !ffn1_weight_kn || !ffn1_bias || !ffn2_weight_kn || !ffn2_bias || !out)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "encoder_tail_folded_forward: null pointer argument");
    if ((dp != 0 && dp != 2) || (dp == 2 && (!position || !folded_pos)))
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "encoder_tail_folded_forward: dp must be 0 or 2, with positions and their folded rows for 2");
    if (B <= 0 || S <= 0) return fail(SPGT_ERR_INVALID_ARGUMENT, "encoder_tail_folded_forward: B and S must be positive");
    if (dim_hidden != 128 || ffn_hidden != 256)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "encoder_tail_folded_forward: needs dim_hidden 128, ffn_hidden 256");
    if (activation != SPGT_ACT_NONE && activation != SPGT_ACT_RELU && activation != SPGT_ACT_SILU)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "encoder_tail_folded_forward: unknown activation");
    if (ld_q < 128 || (ld_q & 3) || !aligned16(q) || !aligned16(x) || !aligned16(out) || !aligned16(fc_bias) ||
        !aligned16(ffn1_bias) || !aligned16(ffn2_bias) || !aligned4(folded_fc) || !aligned4(ffn1_weight_kn) ||
        !aligned4(ffn2_weight_kn) || (dp == 2 && (!aligned8(position) || !aligned4(folded_pos))))
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "encoder_tail_folded_forward: activations and biases must be 16-byte aligned, ld_q a multiple of 4");
    if (out == x || out == q) return fail(SPGT_ERR_INVALID_ARGUMENT, "encoder_tail_folded_forward: out must not alias an input");
    const int64_t tiles = (int64_t)B * ceil_div(S, (int64_t)32);
    if (tiles > INT32_MAX) return fail(SPGT_ERR_INVALID_ARGUMENT, "encoder_tail_folded_forward: too many tokens");
    // as many workgroups as CUs at most, each with the same number of consecutive tiles
    const int64_t per_wg = ceil_div(tiles, (int64_t)device_cu_count());
    const unsigned grid = (unsigned)ceil_div(tiles, per_wg);
    const size_t lds = std::max<size_t>(((size_t)32 * (128 + 4 + 132 + 260) + 512 + 256) * sizeof(float), 84 * 1024);
    if (p_fc > 0.f || p_ffn > 0.f) (void)allow_dynamic_lds(encoder_tail_k<128, true, true>, lds);
    else (void)allow_dynamic_lds(encoder_tail_k<128, true, false>, lds);
    if (p_fc > 0.f || p_ffn > 0.f)
        hipLaunchKernelGGL((encoder_tail_k<128, true, true>), dim3(grid), dim3(256), lds, stream, q, ld_q, x, folded_fc,
                           fc_bias, ffn1_weight_kn, ffn1_bias, ffn2_weight_kn, ffn2_bias, activation, out, (int64_t)B * S,
                           dp == 2 ? folded_pos : nullptr, position, S, seed, p_fc, p_ffn);
    else
        hipLaunchKernelGGL((encoder_tail_k<128, true, false>), dim3(grid), dim3(256), lds, stream, q, ld_q, x, folded_fc,
                           fc_bias, ffn1_weight_kn, ffn1_bias, ffn2_weight_kn, ffn2_bias, activation, out, (int64_t)B * S,
                           dp == 2 ? folded_pos : nullptr, position, S, nullptr, 0.f, 0.f);
    return check_launch("encoder_tail_folded_forward");
}

}  // namespace

extern "C" int spgt_encoder_tail_folded_forward(const float* q, int64_t ld_q, const float* position, const float* x,
                                                const float* folded_fc, const float* folded_pos,
                                                const float* fc_bias, const float* ffn1_weight_kn,
                                                const float* ffn1_bias, const float* ffn2_weight_kn,
                                                const float* ffn2_bias, int activation, float* out, int B,
                                                int64_t S, int dp, int dim_hidden, int ffn_hidden,
                                                hipStream_t stream) {
    return encoder_tail_folded_common(q, ld_q, position, x, folded_fc, folded_pos, fc_bias, ffn1_weight_kn, ffn1_bias,
                                      ffn2_weight_kn, ffn2_bias, activation, out, B, S, dp, dim_hidden, ffn_hidden,
                                      nullptr, 0.f, 0.f, stream);
}

extern "C" int spgt_encoder_tail_folded_forward_dropout(const float* q, int64_t ld_q, const float* position,
                                                        const float* x, const float* folded_fc, const float* folded_pos,
                                                        const float* fc_bias, const float* ffn1_weight_kn,
                                                        const float* ffn1_bias, const float* ffn2_weight_kn,
                                                        const float* ffn2_bias, int activation, float* out, int B,
                                                        int64_t S, int dp, int dim_hidden, int ffn_hidden,
                                                        const uint32_t* seed, float fc_droprate, float ffn_droprate,
                                                        hipStream_t stream) {
    if (int rc = dropout_args_ok(seed, fc_droprate, ffn_droprate)) return rc;
    return encoder_tail_folded_common(q, ld_q, position, x, folded_fc, folded_pos, fc_bias, ffn1_weight_kn, ffn1_bias,
                                      ffn2_weight_kn, ffn2_bias, activation, out, B, S, dp, dim_hidden, ffn_hidden, seed,
                                      fc_droprate, ffn_droprate, stream);
}

extern "C" int spgt_encoder_tail_supported(int attn_features, int dim_hidden, int ffn_hidden) {
    return ((attn_features == 128 || attn_features == 136) && dim_hidden == 128 && ffn_hidden == 256) ? 1 : 0;
}

namespace {

int encoder_tail_common(const float* attn_out, int64_t ld_attn, const float* x, const float* fc_weight_kn,
                        const float* fc_bias, const float* ffn1_weight_kn, const float* ffn1_bias,
                        const float* ffn2_weight_kn, const float* ffn2_bias, int activation, float* out, int64_t tokens,
                        int attn_features, int dim_hidden, int ffn_hidden, const uint32_t* seed, float p_fc,
                        float p_ffn, hipStream_t stream) {
    if (!attn_out || !x || !fc_weight_kn || !fc_bias || !ffn1_weight_kn || !ffn1_bias || !ffn2_weight_kn ||
        !ffn2_bias || !out)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "encoder_tail_forward: null pointer argument");
    if (tokens < 0) return fail(SPGT_ERR_INVALID_ARGUMENT, "encoder_tail_forward: negative token count");
    if (!spgt_encoder_tail_supported(attn_features, dim_hidden, ffn_hidden))
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "encoder_tail_forward: needs attn_features 128 or 136, dim_hidden 128, ffn_hidden 256");
    if (activation != SPGT_ACT_NONE && activation != SPGT_ACT_RELU && activation != SPGT_ACT_SILU)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "encoder_tail_forward: unknown activation");
    if (ld_attn < attn_features || (ld_attn & 3) || !aligned16(attn_out) || !aligned16(x) || !aligned16(out) ||
        !aligned16(fc_bias) || !aligned16(ffn1_bias) || !aligned16(ffn2_bias) || !aligned4(fc_weight_kn) ||
        !aligned4(ffn1_weight_kn) || !aligned4(ffn2_weight_kn))
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "encoder_tail_forward: activations and biases must be 16-byte aligned, ld_attn a multiple of 4");
    if (out == x || out == attn_out)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "encoder_tail_forward: out must not alias an input");
    if (tokens == 0) return SPGT_OK;
    if (ceil_div(tokens, (int64_t)32) > INT32_MAX)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "encoder_tail_forward: too many tokens");
    const unsigned grid = (unsigned)std::min<int64_t>(ceil_div(tokens, (int64_t)32), device_cu_count());
    // attention tile + y1 + hidden tile + biases; at least half of the CU's LDS (one workgroup per CU anyway:
    // a wave uses most of its SIMD's registers)
    const size_t lds = std::max<size_t>(((size_t)32 * ((size_t)attn_features + 4 + 132 + 260) + 512 + 256) * sizeof(float), 84 * 1024);
    const bool drop = p_fc > 0.f || p_ffn > 0.f;
#define SPGT_TAIL(K1, DROPF)                                                                                          \
    (void)allow_dynamic_lds(encoder_tail_k<K1, false, DROPF>, lds);                                                    \
    hipLaunchKernelGGL((encoder_tail_k<K1, false, DROPF>), dim3(grid), dim3(256), lds, stream, attn_out, ld_attn, x,   \
                       fc_weight_kn, fc_bias, ffn1_weight_kn, ffn1_bias, ffn2_weight_kn, ffn2_bias, activation, out,   \
                       tokens, nullptr, nullptr, (int64_t)0, drop ? seed : nullptr, p_fc, p_ffn)
    if (attn_features == 136) {
        if (drop) { SPGT_TAIL(136, true); } else { SPGT_TAIL(136, false); }
    } else {
        if (drop) { SPGT_TAIL(128, true); } else { SPGT_TAIL(128, false); }
    }
#undef SPGT_TAIL
    return check_launch("encoder_tail_forward");
}

}  // namespace

extern "C" int spgt_encoder_tail_forward(const float* attn_out, int64_t ld_attn, const float* x,
                                         const float* fc_weight_kn, const float* fc_bias,
                                         const float* ffn1_weight_kn, const float* ffn1_bias,
                                         const float* ffn2_weight_kn, const float* ffn2_bias, int activation,
                                         float* out, int64_t tokens, int attn_features, int dim_hidden,
                                         int ffn_hidden, hipStream_t stream) {
    return encoder_tail_common(attn_out, ld_attn, x, fc_weight_kn, fc_bias, ffn1_weight_kn, ffn1_bias, ffn2_weight_kn,
                               ffn2_bias, activation, out, tokens, attn_features, dim_hidden, ffn_hidden, nullptr, 0.f,
                               0.f, stream);
}

extern "C" int spgt_encoder_tail_forward_dropout(const float* attn_out, int64_t ld_attn, const float* x,
                                                 const float* fc_weight_kn, const float* fc_bias,
                                                 const float* ffn1_weight_kn, const float* ffn1_bias,
                                                 const float* ffn2_weight_kn, const float* ffn2_bias, int activation,
                                                 float* out, int64_t tokens, int attn_features, int dim_hidden,
                                                 int ffn_hidden, const uint32_t* seed, float fc_droprate,
                                                 float ffn_droprate, hipStream_t stream) {
    if (int rc = dropout_args_ok(seed, fc_droprate, ffn_droprate)) return rc;
    return encoder_tail_common(attn_out, ld_attn, x, fc_weight_kn, fc_bias, ffn1_weight_kn, ffn1_bias, ffn2_weight_kn,
                               ffn2_bias, activation, out, tokens, attn_features, dim_hidden, ffn_hidden, seed,
                               fc_droprate, ffn_droprate, stream);
}

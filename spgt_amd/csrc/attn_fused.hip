// Fused softmax-free Galerkin attention core on token-major operands.
//
//   Q, K, V : [B, S, H*32] fp32 (rows may be strided: one x@[Wq|Wk|Wv] GEMM
//             output serves all three), optional position [B, S, 2]
//   out     : [B, S, H*(dp+32)]
//
// Semantics follow the reference's plain PyTorch path
// (network/layer.py:114-152): K and V are LayerNorm'ed per token and per head
// over the 32 head features (biased variance, eps inside the square root,
// per-head affine), the position channels are prepended to every head, then
// M = K'^T V' / S and out = Q' M.
//
// Three launches:
//   1. ktv_ln_partial_tm  - one pass over K and V: LayerNorm in registers
//      (16 lanes share a token, DPP row reductions), partial d x d tiles
//      accumulated on the fp32 matrix cores, one tile per (chunk, head).
//   2. tile_reduce        - deterministic fixed-order sum of the partial tiles,
//      scaled by 1/S.
//   3. qm_apply_tm        - streams Q once, keeps the head's d x d matrix in
//      registers as the MFMA A operand, writes out once.
#include "spgt_device.h"
#include "spgt_host.h"
#include "spgt_kernels.h"

#include <atomic>
#include <vector>

// Size of the device array behind spgt_galerkin_attention_fused_forward_static (16 MiB: the headline shape
// B=8, S=44521, H=4 needs 4.2 MB of partial tiles, one per 1024-thread workgroup and head).
#ifndef SPGT_STATIC_SCRATCH_BYTES
#define SPGT_STATIC_SCRATCH_BYTES (16u << 20)
#endif

// Cache policy of the three touch-once streams (K/V reads, Q reads, out
// writes).  Measured on MI355X at B=8, S=44521 over all eight combinations,
// with consecutive calls on different inputs and outputs (so that no call
// finds its Q, or the lines it writes, in the 256 MB last-level cache):
// non-temporal K/V loads and out stores with plain Q loads is the fastest
// (154 us per call; plain stores 155-159 us; plain K/V loads 157-176 us,
// because the K/V pass then runs at 71-101 us instead of 69 us).
#ifndef SPGT_NT_P1LD
#define SPGT_NT_P1LD true
#endif
#ifndef SPGT_NT_P2LD
#define SPGT_NT_P2LD false
#endif
#ifndef SPGT_NT_TILE
#define SPGT_NT_TILE true
#endif
#ifndef SPGT_NT_P2ST
#define SPGT_NT_P2ST true
#endif

namespace spgt {

namespace {

template <int DP>
struct KtvUnit {
    float2 k, v, p;
};

// LayerNorm of the two features this lane holds; the other 30 features of the
// token live in the other 15 lanes of the DPP row.
__device__ __forceinline__ float2 ln_pair(float2 x, float g0, float g1, float b0, float b1, float eps) {
    const float mean = row16_allsum(x.x + x.y) * (1.0f / 32.0f);
    const float d0 = x.x - mean;
    const float d1 = x.y - mean;
    const float ss = row16_allsum(fmaf(d1, d1, d0 * d0));
    const float rstd = __builtin_amdgcn_rsqf(fmaf(ss, 1.0f / 32.0f, eps));  // v_rsq_f32, 1 ulp
    float2 y;
    y.x = fmaf(d0 * rstd, g0, b0);
    y.y = fmaf(d1 * rstd, g1, b1);
    return y;
}

}  // namespace

// grid (nchunk, H/4, B), block 256 * NSUB: wave w handles head 4*blockIdx.y + w % 4 on the sub-range w / 4 of the
// workgroup's chunk (tokens_per_chunk / NSUB tokens each).  With NSUB > 1 the waves' tiles meet in LDS and the
// workgroup writes their sum, sub-ranges in increasing order: a third or a quarter of the partial tiles reach
// memory (at B=8, S=44521 the 12.6 MB of one-tile-per-wave cost the pass 5 us of its 67, most of it the
// write-back at the end of the kernel).
// Lane l of a wave: token slot t = l/16, feature pair p = l%16 (features 2p, 2p+1).
template <int DP, int U, int NSUB>
__global__ __launch_bounds__(256 * NSUB) void ktv_ln_partial_tm(
    const float* __restrict__ K, const float* __restrict__ V, const float* __restrict__ pos,
    const float* __restrict__ lnwK, const float* __restrict__ lnbK,
    const float* __restrict__ lnwV, const float* __restrict__ lnbV, float eps,
    float* __restrict__ partial, int S, int H, int64_t ld, int tokens_per_chunk) {
    constexpr int D = DP + 32;
    extern __shared__ __attribute__((aligned(16))) float sub_tiles[];  // NSUB > 1: [NSUB][4 heads][D * D]
    // DP == 2: the positions of a group of 4*U tokens are 8*U consecutive floats, fetched by one load instruction
    // per group (a float per lane) and handed to the lanes that need them through this wave-private stage, one
    // token slot's U positions side by side: a load of its own per unit would be a third more vector memory
    // instructions than the K and V loads, for 1.5 % more bytes.
    __shared__ __attribute__((aligned(16))) float pos_stage[DP == 2 ? 4 * NSUB * 8 * U : 4];
    const int lane = threadIdx.x & 63;
    const int wave = (threadIdx.x >> 6) & 3;
    const int sub = threadIdx.x >> 8;
    const int h = blockIdx.y * 4 + wave;
    const int b = blockIdx.z;
    const int chunk = blockIdx.x;
    const int nchunk = gridDim.x;
    const int t = lane >> 4;
    const int p = lane & 15;

    const int sub_len = tokens_per_chunk / NSUB;
    const int s0 = min(S, chunk * tokens_per_chunk + sub * sub_len);
    const int s1 = min(S, s0 + sub_len);

    const int f = h * 32 + 2 * p;
    const float gK0 = lnwK[f], gK1 = lnwK[f + 1], bK0 = lnbK[f], bK1 = lnbK[f + 1];
    const float gV0 = lnwV[f], gV1 = lnwV[f + 1], bV0 = lnbV[f], bV1 = lnbV[f + 1];

    // Wave-uniform chunk bases; per-lane offsets stay 32-bit so that loads
    // use the scalar-base + vector-offset addressing form.
    const float* kchunk = K + ((int64_t)b * S + s0) * ld;
    const float* vchunk = V + ((int64_t)b * S + s0) * ld;
    const float* pchunk = pos + ((int64_t)b * S + s0) * 2;
    const uint32_t uld = (uint32_t)ld;

    v4f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
    float kp[2][2] = {{0.f, 0.f}, {0.f, 0.f}};  // sum yK[ta] * pos[a]
    float pv[2][2] = {{0.f, 0.f}, {0.f, 0.f}};  // sum pos[a] * yV[tb]
    float pp[3] = {0.f, 0.f, 0.f};              // sum p0p0, p0p1, p1p1
    // The position block is the same for every head: where the heads' tiles meet in LDS (NSUB > 1) only the first
    // head's waves form it, and the other heads' tiles take it from there when the workgroup writes them out.
    const bool pp_here = NSUB == 1 || wave == 0;

    // `rel` is the token index relative to the chunk start.
    auto load_unit = [&](const float* kg, const float* vg, const float* pg, uint32_t rel, bool with_pos) {
        KtvUnit<DP> u;
        const uint32_t off = rel * uld + (uint32_t)f;
        u.k = ld_stream<SPGT_NT_P1LD>(reinterpret_cast<const float2*>(kg + off));
        u.v = ld_stream<SPGT_NT_P1LD>(reinterpret_cast<const float2*>(vg + off));
        if (DP == 2 && with_pos) u.p = *reinterpret_cast<const float2*>(pg + rel * 2u);
        else u.p = make_float2(0.f, 0.f);
        return u;
    };
    auto compute_unit = [&](const KtvUnit<DP>& u, bool valid) {
        float2 yk = ln_pair(u.k, gK0, gK1, bK0, bK1, eps);
        const float2 yv = ln_pair(u.v, gV0, gV1, bV0, bV1, eps);
        float2 pz = u.p;
        if (!valid) {
            yk.x = 0.f;
            yk.y = 0.f;
            if (DP == 2) { pz.x = 0.f; pz.y = 0.f; }
        }
        acc[0][0] = mfma16(yk.x, yv.x, acc[0][0]);
        acc[0][1] = mfma16(yk.x, yv.y, acc[0][1]);
        acc[1][0] = mfma16(yk.y, yv.x, acc[1][0]);
        acc[1][1] = mfma16(yk.y, yv.y, acc[1][1]);
        if (DP == 2) {
            kp[0][0] = fmaf(yk.x, u.p.x, kp[0][0]);
            kp[0][1] = fmaf(yk.x, u.p.y, kp[0][1]);
            kp[1][0] = fmaf(yk.y, u.p.x, kp[1][0]);
            kp[1][1] = fmaf(yk.y, u.p.y, kp[1][1]);
            pv[0][0] = fmaf(pz.x, yv.x, pv[0][0]);
            pv[0][1] = fmaf(pz.x, yv.y, pv[0][1]);
            pv[1][0] = fmaf(pz.y, yv.x, pv[1][0]);
            pv[1][1] = fmaf(pz.y, yv.y, pv[1][1]);
            if (pp_here) {
                pp[0] = fmaf(pz.x, pz.x, pp[0]);
                pp[1] = fmaf(pz.x, pz.y, pp[1]);
                pp[2] = fmaf(pz.y, pz.y, pp[2]);
            }
        }
    };

    // Software pipeline over full groups of G = 4*U tokens with two register
    // buffers (no buffer-to-buffer copies inside the loop: a copy of a value
    // still in flight would force a wait for every outstanding load).  The
    // ragged remainder of the chunk is one extra clamped and masked group.
    constexpr int G = 4 * U;
    const int len = s1 - s0;
    const int nfull = len / G;
    KtvUnit<DP> bufA[U], bufB[U];
    float prawA = 0.f, prawB = 0.f;  // DP == 2: float (lane % (8 U)) of the group's positions
    static_assert(DP == 0 || 8 * U <= 64, "a group's positions are one float per lane");
    // where that float goes in the stage: token 4u + ts, component c -> [ts][u][c]
    const int pl = lane % (8 * U);
    const int pdst = ((pl >> 1) & 3) * (2 * U) + (pl >> 3) * 2 + (pl & 1);
    float* const pstage = pos_stage + (sub * 4 + wave) * (8 * U);
    auto load_group = [&](KtvUnit<DP>(&buf)[U], float& praw, int g) {  // g is clamped to the full groups
        const int64_t go = (int64_t)min(g, nfull - 1) * G;
        const float* kg = kchunk + go * ld;
        const float* vg = vchunk + go * ld;
        const float* pg = pchunk + go * 2;
#pragma unroll
        for (int u = 0; u < U; ++u) buf[u] = load_unit(kg, vg, pg, (uint32_t)(4 * u + t), false);
        if (DP == 2) praw = pg[pl];
    };
    // A full group normalises its 2*U (token, tensor) pairs in lock-step; each
    // value sees the same operations in the same order as in ln_pair.
    auto compute_full = [&](const KtvUnit<DP>(&buf)[U], float praw) {
        constexpr int N = 2 * U;
        float x0[N], x1[N], red[N];
        float pzs[2 * U];  // this lane's token slot: positions of units 0 .. U-1
        if (DP == 2) {
            // (the stage is the wave's own: LDS operations of one wave complete in order, no barrier)
            pstage[pdst] = praw;
#pragma unroll
            for (int i = 0; i < 2 * U; i += 4) {
                const float4 q = *reinterpret_cast<const float4*>(pstage + t * (2 * U) + i);
                pzs[i] = q.x; pzs[i + 1] = q.y; pzs[i + 2] = q.z; pzs[i + 3] = q.w;
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            x0[2 * u] = buf[u].k.x;
            x1[2 * u] = buf[u].k.y;
            x0[2 * u + 1] = buf[u].v.x;
            x1[2 * u + 1] = buf[u].v.y;
        }
#pragma unroll
        for (int i = 0; i < N; ++i) red[i] = x0[i] + x1[i];
        row16_allsum_n(red);
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const float mean = red[i] * (1.0f / 32.0f);
            x0[i] -= mean;
            x1[i] -= mean;
            red[i] = fmaf(x1[i], x1[i], x0[i] * x0[i]);
        }
        row16_allsum_n(red);
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const float rstd = __builtin_amdgcn_rsqf(fmaf(red[i], 1.0f / 32.0f, eps));
            const bool isv = i & 1;
            x0[i] = fmaf(x0[i] * rstd, isv ? gV0 : gK0, isv ? bV0 : bK0);
            x1[i] = fmaf(x1[i] * rstd, isv ? gV1 : gK1, isv ? bV1 : bK1);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const float yk0 = x0[2 * u], yk1 = x1[2 * u], yv0 = x0[2 * u + 1], yv1 = x1[2 * u + 1];
            acc[0][0] = mfma16(yk0, yv0, acc[0][0]);
            acc[0][1] = mfma16(yk0, yv1, acc[0][1]);
            acc[1][0] = mfma16(yk1, yv0, acc[1][0]);
            acc[1][1] = mfma16(yk1, yv1, acc[1][1]);
            if (DP == 2) {
                const float2 pz = make_float2(pzs[2 * u], pzs[2 * u + 1]);
                kp[0][0] = fmaf(yk0, pz.x, kp[0][0]);
                kp[0][1] = fmaf(yk0, pz.y, kp[0][1]);
                kp[1][0] = fmaf(yk1, pz.x, kp[1][0]);
                kp[1][1] = fmaf(yk1, pz.y, kp[1][1]);
                pv[0][0] = fmaf(pz.x, yv0, pv[0][0]);
                pv[0][1] = fmaf(pz.x, yv1, pv[0][1]);
                pv[1][0] = fmaf(pz.y, yv0, pv[1][0]);
                pv[1][1] = fmaf(pz.y, yv1, pv[1][1]);
            }
        }
        if (DP == 2 && pp_here) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                pp[0] = fmaf(pzs[2 * u], pzs[2 * u], pp[0]);
                pp[1] = fmaf(pzs[2 * u], pzs[2 * u + 1], pp[1]);
                pp[2] = fmaf(pzs[2 * u + 1], pzs[2 * u + 1], pp[2]);
            }
        }
    };
    if (nfull > 0) {
        load_group(bufA, prawA, 0);
        int g = 0;
        for (; g + 2 <= nfull; g += 2) {
            load_group(bufB, prawB, g + 1);
            __builtin_amdgcn_sched_barrier(0);  // keep the prefetch ahead of the arithmetic
            compute_full(bufA, prawA);
            __builtin_amdgcn_sched_barrier(0);
            load_group(bufA, prawA, g + 2);
            __builtin_amdgcn_sched_barrier(0);
            compute_full(bufB, prawB);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (g < nfull) compute_full(bufA, prawA);
    }
    if (nfull * G < len) {
        const int rel0 = nfull * G + t;
#pragma unroll
        for (int u = 0; u < U; ++u)
            bufA[u] = load_unit(kchunk, vchunk, pchunk, (uint32_t)min(rel0 + 4 * u, len - 1), true);
#pragma unroll
        for (int u = 0; u < U; ++u) compute_unit(bufA[u], (rel0 + 4 * u) < len);
    }

    // acc[ta][tb][r] = M[2*(4t+r)+ta][2p+tb]
    float* tile = NSUB > 1 ? sub_tiles + (sub * 4 + wave) * (D * D)
                           : partial + (((int64_t)b * H + h) * nchunk + chunk) * (D * D);
#pragma unroll
    for (int ta = 0; ta < 2; ++ta)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int i = DP + 8 * t + 2 * r + ta;
            float2 o;
            o.x = acc[ta][0][r];
            o.y = acc[ta][1][r];
            if (NSUB == 1) st_stream<SPGT_NT_TILE>(reinterpret_cast<float2*>(tile + i * D + DP + 2 * p), o);
            else *reinterpret_cast<float2*>(tile + i * D + DP + 2 * p) = o;
        }
    if (DP == 2) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                kp[i][j] = rows4_allsum(kp[i][j]);
                pv[i][j] = rows4_allsum(pv[i][j]);
            }
#pragma unroll
        for (int i = 0; i < 3; ++i) pp[i] = rows4_allsum(pp[i]);
        if (t == 0) {
#pragma unroll
            for (int ta = 0; ta < 2; ++ta) {
                float2 o;
                o.x = kp[ta][0];
                o.y = kp[ta][1];
                *reinterpret_cast<float2*>(tile + (DP + 2 * p + ta) * D) = o;
            }
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                float2 o;
                o.x = pv[a][0];
                o.y = pv[a][1];
                *reinterpret_cast<float2*>(tile + a * D + DP + 2 * p) = o;
            }
            if (p == 0) {
                tile[0] = pp[0];
                tile[1] = pp[1];
                tile[D] = pp[1];
                tile[D + 1] = pp[2];
            }
        }
    }
    if constexpr (NSUB > 1) {
        __syncthreads();
        // the four heads' tiles are contiguous in LDS per sub-range and in memory per chunk only within a head
        constexpr int E4 = D * D / 4;  // float4 per tile
        for (int e = threadIdx.x; e < 4 * E4; e += 256 * NSUB) {
            const int hh = e / E4;
            const int r4 = e - hh * E4;
            float4 sum = *reinterpret_cast<const float4*>(sub_tiles + hh * (D * D) + 4 * r4);
#pragma unroll
            for (int q = 1; q < NSUB; ++q) {
                const float4 v = *reinterpret_cast<const float4*>(sub_tiles + (q * 4 + hh) * (D * D) + 4 * r4);
                sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
            }
            if (DP == 2 && hh != 0 && (r4 == 0 || r4 == D / 4)) {
                // the position block M[0..1][0..1] (floats 0, 1, D, D + 1 of the tile) as the first head has it
                float4 z = *reinterpret_cast<const float4*>(sub_tiles + 4 * r4);
#pragma unroll
                for (int q = 1; q < NSUB; ++q) {
                    const float4 v = *reinterpret_cast<const float4*>(sub_tiles + (q * 4) * (D * D) + 4 * r4);
                    z.x += v.x; z.y += v.y; z.z += v.z; z.w += v.w;
                }
                if (r4 == 0) { sum.x = z.x; sum.y = z.y; }
                else { sum.z = z.z; sum.w = z.w; }
            }
            float* dst = partial + (((int64_t)b * H + blockIdx.y * 4 + hh) * nchunk + chunk) * (D * D) + 4 * r4;
            st_stream<SPGT_NT_TILE>(reinterpret_cast<float4*>(dst), sum);
        }
    }
}

// out[bh][e] = scale * sum_c partial[bh][c][e], summed in a fixed order:
// sixteen interleaved chains (c = q, q+16, ...), each summed in increasing c,
// then combined by a fixed binary tree.  All loads of a chain are issued before
// the first add, so the kernel costs about one memory round trip.
// grid (ceil(E/256), BH), block 1024 = 64 element-quads x 16 chains.
__global__ __launch_bounds__(1024) void tile_reduce(
    const float* __restrict__ partial, float* __restrict__ out, int E, int nchunk, float scale) {
    __shared__ float4 sm[kReduceChains][64];
    const int q = threadIdx.x >> 6;
    const int e4 = threadIdx.x & 63;
    const int e = (blockIdx.x * 64 + e4) * 4;
    const int64_t bh = blockIdx.y;
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    if (e < E) {
        const float* src = partial + bh * nchunk * (int64_t)E + e;
        float4 v[kReduceMaxPerChain];
#pragma unroll
        for (int i = 0; i < kReduceMaxPerChain; ++i) {
            const int c = q + kReduceChains * i;
            v[i] = (c < nchunk) ? *reinterpret_cast<const float4*>(src + (int64_t)c * E)
                                : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int i = 0; i < kReduceMaxPerChain; ++i) {
            s.x += v[i].x; s.y += v[i].y; s.z += v[i].z; s.w += v[i].w;
        }
    }
    sm[q][e4] = s;
    __syncthreads();
    if (q == 0 && e < E) {
        float4 t[kReduceChains];
#pragma unroll
        for (int i = 0; i < kReduceChains; ++i) t[i] = sm[i][e4];
#pragma unroll
        for (int w = kReduceChains / 2; w >= 1; w /= 2)
#pragma unroll
            for (int i = 0; i < w; ++i) {
                t[i].x += t[i + w].x; t[i].y += t[i + w].y; t[i].z += t[i + w].z; t[i].w += t[i + w].w;
            }
        *reinterpret_cast<float4*>(out + bh * E + e) =
            make_float4(t[0].x * scale, t[0].y * scale, t[0].z * scale, t[0].w * scale);
    }
}

// grid (nchunk, H/4, B), block 256: wave w handles head 4*blockIdx.y + w.
// Lane l: token slot tk = l%16, feature group g = l/16; the lane loads
// Q[s][4g..4g+3] and Q[s][16+4g..16+4g+3] of its token.  MFMA step kk contracts
// the four features {i(kk, g) : g = 0..3}, i(kk,g) = 4g+kk (kk<4) or 16+4g+kk-4.
template <int DP, int U>
__global__ __launch_bounds__(256) void qm_apply_tm(
    const float* __restrict__ Q, const float* __restrict__ pos, const float* __restrict__ M,
    float* __restrict__ out, int S, int H, int64_t ld, int tokens_per_chunk) {
    constexpr int D = DP + 32;
    // DP == 2: output rows of 4 heads x 34 floats are staged in LDS per group of U units and
    // written out by the whole workgroup as one contiguous run (two buffers, one barrier per group).
    constexpr int kStagePitch = 4 * D + 4;  // floats per token row in LDS (padding spreads the banks)
    __shared__ __attribute__((aligned(16))) float stage[DP == 2 ? 2 * U * 16 * kStagePitch : 4];
    int stage_parity = 0;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int h = blockIdx.y * 4 + wave;
    const int b = blockIdx.z;
    const int tk = lane & 15;
    const int g = lane >> 4;
    const int s0 = blockIdx.x * tokens_per_chunk;
    const int s1 = min(S, s0 + tokens_per_chunk);
    const int64_t ldo = (int64_t)H * D;

    const float* m = M + ((int64_t)b * H + h) * (D * D);
    float mreg[8][2];
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
        const int i = (kk < 4) ? (4 * g + kk) : (16 + 4 * g + kk - 4);
#pragma unroll
        for (int jb = 0; jb < 2; ++jb) mreg[kk][jb] = m[(DP + i) * D + DP + jb * 16 + tk];
    }
    // DP == 2 only: rows 0,1 of M for this lane's output features, and
    // columns 0,1 of M for this lane's input features.
    float mrow[2][2][4];
    float mcol[8][2];
    float mpp[2][2];
    if (DP == 2) {
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int jb = 0; jb < 2; ++jb)
#pragma unroll
                for (int r = 0; r < 4; ++r) mrow[a][jb][r] = m[a * D + DP + jb * 16 + 4 * g + r];
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
            const int i = (kk < 4) ? (4 * g + kk) : (16 + 4 * g + kk - 4);
            mcol[kk][0] = m[(DP + i) * D + 0];
            mcol[kk][1] = m[(DP + i) * D + 1];
        }
        mpp[0][0] = m[0]; mpp[0][1] = m[1]; mpp[1][0] = m[D]; mpp[1][1] = m[D + 1];
    }

    const float* qbase = Q + (int64_t)b * S * ld + h * 32 + 4 * g;
    const float* pbase = pos + (int64_t)b * S * 2;
    float* obase = out + (int64_t)b * S * ldo + h * D;

    struct Unit { float4 q0, q1; float2 p; };
    auto load_unit = [&](int s) {
        Unit u;
        const float* qp = qbase + (int64_t)s * ld;
        u.q0 = ld_stream<SPGT_NT_P2LD>(reinterpret_cast<const float4*>(qp));
        u.q1 = ld_stream<SPGT_NT_P2LD>(reinterpret_cast<const float4*>(qp + 16));
        if (DP == 2) u.p = *reinterpret_cast<const float2*>(pbase + (int64_t)s * 2);
        return u;
    };
    // `sb` is the first token of the unit (this lane's token is sb + tk, clamped loads aside).
    auto compute_unit = [&](const Unit& u, int sb, int slot) {
        const int s = sb + tk;
        const bool valid = s < s1;
        const float q[8] = {u.q0.x, u.q0.y, u.q0.z, u.q0.w, u.q1.x, u.q1.y, u.q1.z, u.q1.w};
        v4f acc[2];
#pragma unroll
        for (int jb = 0; jb < 2; ++jb) {
            if (DP == 2) {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    acc[jb][r] = fmaf(u.p.y, mrow[1][jb][r], u.p.x * mrow[0][jb][r]);
            } else {
                acc[jb] = v4f{0.f, 0.f, 0.f, 0.f};
            }
        }
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
            acc[0] = mfma16(mreg[kk][0], q[kk], acc[0]);
            acc[1] = mfma16(mreg[kk][1], q[kk], acc[1]);
        }
        if (DP == 2) {
            float c0 = 0.f, c1 = 0.f;
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) {
                c0 = fmaf(q[kk], mcol[kk][0], c0);
                c1 = fmaf(q[kk], mcol[kk][1], c1);
            }
            c0 = rows4_allsum(c0);
            c1 = rows4_allsum(c1);
            float* row = stage + ((stage_parity * U + slot) * 16 + tk) * kStagePitch + (h & 3) * D;
            if (g == 0) {
                float2 o;
                o.x = fmaf(u.p.y, mpp[1][0], fmaf(u.p.x, mpp[0][0], c0));
                o.y = fmaf(u.p.y, mpp[1][1], fmaf(u.p.x, mpp[0][1], c1));
                *reinterpret_cast<float2*>(row) = o;
            }
#pragma unroll
            for (int jb = 0; jb < 2; ++jb) {
                float* o = row + DP + jb * 16 + 4 * g;
                *reinterpret_cast<float2*>(o) = make_float2(acc[jb][0], acc[jb][1]);
                *reinterpret_cast<float2*>(o + 2) = make_float2(acc[jb][2], acc[jb][3]);
            }
            (void)valid;
        } else {
            // Lanes tk and tk^8 swap halves so that one store instruction writes
            // whole 128-byte head rows of 8 tokens (non-temporal stores of partial
            // lines cost extra HBM write traffic).
            const bool lo = tk < 8;
            // cross-lane moves first, with every lane active; selects afterwards
            float o0[4], o1[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                o0[r] = dpp_move<SPGT_DPP_ROW_ROR8>(acc[0][r]);
                o1[r] = dpp_move<SPGT_DPP_ROW_ROR8>(acc[1][r]);
            }
            float4 x, y;
            x.x = lo ? acc[0][0] : o1[0];
            x.y = lo ? acc[0][1] : o1[1];
            x.z = lo ? acc[0][2] : o1[2];
            x.w = lo ? acc[0][3] : o1[3];
            y.x = lo ? o0[0] : acc[1][0];
            y.y = lo ? o0[1] : acc[1][1];
            y.z = lo ? o0[2] : acc[1][2];
            y.w = lo ? o0[3] : acc[1][3];
            const int fo = (lo ? 0 : 16) + 4 * g;
            const int sx = sb + (tk & 7);
            const int sy = sx + 8;
            if (sx < s1) st_stream<SPGT_NT_P2ST>(reinterpret_cast<float4*>(obase + (int64_t)sx * ldo + fo), x);
            if (sy < s1) st_stream<SPGT_NT_P2ST>(reinterpret_cast<float4*>(obase + (int64_t)sy * ldo + fo), y);
        }
    };

    // Same two-buffer software pipeline as in ktv_ln_partial_tm.
    constexpr int G = 16 * U;
    const int len = s1 - s0;
    const int nfull = len / G;
    const int ntot = (len + G - 1) / G;
    Unit bufA[U], bufB[U];
    auto load_group = [&](Unit(&buf)[U], int gi) {
        const int sg = s0 + min(gi, ntot - 1) * G + tk;
#pragma unroll
        for (int u = 0; u < U; ++u) buf[u] = load_unit(min(sg + 16 * u, s1 - 1));
    };
    // DP == 2: after the group's units are staged, the workgroup copies min(G, s1 - sg) token rows
    // of 4*D floats (one contiguous run in `out`) with 16-byte stores.
    auto flush_group = [&](int sg) {
        if (DP != 2) return;
        __syncthreads();
        const int ntok = min(G, s1 - sg);
        const float* src = stage + stage_parity * U * 16 * kStagePitch;
        float* dst = out + ((int64_t)b * S + sg) * ldo + (int64_t)(blockIdx.y * 4) * D;
        constexpr int R4 = D;  // float4 per token row (4 heads x D floats)
        for (int e = threadIdx.x; e < ntok * R4; e += 256) {
            const int tok = e / R4;
            const int c4 = e - tok * R4;
            const float4 v = *reinterpret_cast<const float4*>(src + tok * kStagePitch + 4 * c4);
            st_stream<SPGT_NT_P2ST>(reinterpret_cast<float4*>(dst + (int64_t)tok * ldo + 4 * c4), v);
        }
        stage_parity ^= 1;
    };
    auto compute_group = [&](const Unit(&buf)[U], int gi) {
        const int sg = s0 + gi * G;
#pragma unroll
        for (int u = 0; u < U; ++u) compute_unit(buf[u], sg + 16 * u, u);
        flush_group(sg);
    };
    load_group(bufA, 0);
    int gi = 0;
    for (; gi + 2 <= nfull; gi += 2) {
        load_group(bufB, gi + 1);
        __builtin_amdgcn_sched_barrier(0);  // keep the prefetch ahead of the arithmetic
        compute_group(bufA, gi);
        __builtin_amdgcn_sched_barrier(0);
        load_group(bufA, gi + 2);
        __builtin_amdgcn_sched_barrier(0);
        compute_group(bufB, gi + 1);
        __builtin_amdgcn_sched_barrier(0);
    }
    if (gi < nfull) {
        load_group(bufB, gi + 1);
        compute_group(bufA, gi);
#pragma unroll
        for (int u = 0; u < U; ++u) bufA[u] = bufB[u];
        ++gi;
    }
    if (gi < ntot) compute_group(bufA, gi);
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------

namespace {

struct FusedPlan {
    int nsub;           // K^T V pass: waves per head in a workgroup
    int tpc1, nchunk1;  // K^T V pass
    int tpc2, nchunk2;  // Q M pass
};

constexpr int kU1 = 4;  // 16 tokens per unrolled group in pass 1
constexpr int kU2 = 2;  // 32 tokens per unrolled group in pass 2

// Workgroups of the 256-thread plans: three per compute unit in the K/V pass, four in the Q pass.  Measured on
// MI355X (256 CUs) at B=8, S=44521 with inputs and outputs that change from call to call: counts that are whole
// multiples of the CU count beat those in between by 3-10 %; the Q pass takes 77 / 74.6 us with 768 / 1024
// workgroups without position channels and 90 / 83 us with them (512: 94 us, 1280: 97 us, 1536: 89 us).
constexpr int g_target_wg1 = 0;

// Long sequences give every wave of a 1024-thread workgroup (4 heads x 4 sub-ranges) enough tokens: one
// workgroup per CU then, whose four tiles per head are summed in LDS before they go to memory.
#ifndef SPGT_KSUB
#define SPGT_KSUB 4
#endif
#ifndef SPGT_SUB_WG_PER_CU
#define SPGT_SUB_WG_PER_CU 1
#endif
constexpr int kSub = SPGT_KSUB;
constexpr int kSubMinTokens = 256;  // per wave

FusedPlan make_plan(int B, int S, int H) {
    // Chunks are whole unrolled groups so that only the last chunk of a batch has a ragged tail.
    // The K/V pass never uses more chunks than tile_reduce can sum.
    const int bg = std::max(1, B * (H / 4));
    const int cus = device_cu_count();
    const int dflt = 3 * cus;
    FusedPlan p;
    const int g1 = 4 * kU1, g2 = 16 * kU2;
    const int t2 = 4 * cus;
    const int per_bh2 = std::max(1, t2 / bg);
    p.tpc2 = std::max(g2, ceil_div(ceil_div(S, per_bh2), g2) * g2);
    p.nchunk2 = ceil_div(S, p.tpc2);
    // K/V pass: one 1024-thread workgroup per CU when the sequence is long enough ...
    const int per_bh_sub = std::max(1, SPGT_SUB_WG_PER_CU * cus / bg);
    const int gs = g1 * kSub;
    const int tpc_sub = std::max(gs, ceil_div(ceil_div(S, per_bh_sub), gs) * gs);
    if (g_target_wg1 == 0 && tpc_sub / kSub >= kSubMinTokens && ceil_div(S, tpc_sub) <= kReduceChains * kReduceMaxPerChain) {
        p.nsub = kSub;
        p.tpc1 = tpc_sub;
        p.nchunk1 = ceil_div(S, tpc_sub);
        return p;
    }
    // ... else 256-thread workgroups, three per CU; for short sequences, where a chunk of that plan would hold
    // fewer than 128 tokens and the partial tiles it writes (D*D floats per head) weigh as much as the K and V
    // rows it reads, one per CU (B=4, S=5041: K/V pass 14.5 -> 10 us, reduction 4.4 -> 3.7 us; fewer still is
    // slower again).
    const int short_t1 = S / std::max(1, dflt / bg) < 128 ? cus : dflt;
    const int t1 = g_target_wg1 > 0 ? g_target_wg1 : short_t1;
    const int per_bh1 = std::min(kReduceChains * kReduceMaxPerChain, std::max(1, t1 / bg));
    p.nsub = 1;
    p.tpc1 = std::max(g1, ceil_div(ceil_div(S, per_bh1), g1) * g1);
    p.nchunk1 = ceil_div(S, p.tpc1);
    return p;
}

}  // namespace

}  // namespace spgt

using namespace spgt;

extern "C" size_t spgt_galerkin_attention_fused_workspace_bytes(int B, int S, int H, int dp) {
    if (B <= 0 || S <= 0 || H <= 0 || (dp != 0 && dp != 2)) return 0;
    const FusedPlan p = make_plan(B, S, H);
    const size_t D = dp + 32;
    return (size_t)B * H * p.nchunk1 * D * D * sizeof(float);
}

namespace {

constexpr int kMaxDevices = 64;
std::atomic<int> g_sub_lds_allowed[kMaxDevices];

// The long-sequence K/V pass asks for 64 KiB (72 KiB with position channels) of dynamic LDS, which a kernel
// must be allowed once per device.  Done on a device's first call (not a stream operation: callers that
// capture graphs make one call outside the capture first); a failure is reported, not ignored.
int allow_sub_range_lds() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return fail(SPGT_ERR_LAUNCH, "galerkin_attention_fused: no current device");
    if (g_sub_lds_allowed[dev].load(std::memory_order_acquire)) return SPGT_OK;
    const hipError_t e0 = hipFuncSetAttribute(reinterpret_cast<const void*>(&ktv_ln_partial_tm<0, kU1, kSub>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize,
                                              (int)(kSub * 4 * 32 * 32 * sizeof(float)));
    const hipError_t e2 = hipFuncSetAttribute(reinterpret_cast<const void*>(&ktv_ln_partial_tm<2, kU1, kSub>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize,
                                              (int)(kSub * 4 * 34 * 34 * sizeof(float)));
    if (e0 != hipSuccess || e2 != hipSuccess)
        return fail(SPGT_ERR_LAUNCH, "galerkin_attention_fused: the K/V pass was refused its dynamic LDS size");
    g_sub_lds_allowed[dev].store(1, std::memory_order_release);
    return SPGT_OK;
}

// Validates, then enqueues the three launches.  With `ev` (4 events) an event
// is recorded before the first launch (unless record_first is false: the caller
// has recorded it already) and after each launch.
int fused_forward_impl(
    const float* Q, const float* K, const float* V, int64_t ld_in, const float* position,
    const float* ln_weight_K, const float* ln_bias_K, const float* ln_weight_V,
    const float* ln_bias_V, float norm_eps, float* out, float* ktv, void* workspace,
    size_t workspace_bytes, int B, int S, int H, int dp, hipStream_t stream, hipEvent_t* ev,
    bool record_first = true) {
    const bool apply = Q != nullptr || out != nullptr;  // neither: K/V pass and reduction only
    if ((apply && (!Q || !out)) || !K || !V || !ktv || !ln_weight_K || !ln_bias_K || !ln_weight_V || !ln_bias_V)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_fused: null pointer argument");
    if (B <= 0 || S <= 0 || H <= 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_fused: B, S, H must be positive");
    if (H % 4 != 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_fused: num_head must be a multiple of 4");
    if (dp != 0 && dp != 2)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_fused: dim_position must be 0 or 2");
    if (dp == 2 && !position)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_fused: position is null with dim_position 2");
    if (ld_in < (int64_t)H * 32 || (ld_in % 4) != 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "galerkin_attention_fused: row stride must be >= H*32 and a multiple of 4 floats");
    if ((apply && (!aligned16(Q) || !aligned16(out))) || !aligned16(K) || !aligned16(V) || !aligned16(ktv) ||
        (position && !aligned8(position)))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_fused: operands must be 16-byte aligned");
    if (B > 65535 || H / 4 > 65535)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_fused: batch or head count exceeds the grid limit");
    const size_t need = spgt_galerkin_attention_fused_workspace_bytes(B, S, H, dp);
    if (!workspace || workspace_bytes < need || !aligned16(workspace))
        return fail(SPGT_ERR_WORKSPACE, "galerkin_attention_fused: workspace missing, misaligned or too small");

    const FusedPlan p = make_plan(B, S, H);
    const int D = dp + 32;
    float* partial = static_cast<float*>(workspace);
    const dim3 block(256);
    const dim3 grid1(p.nchunk1, H / 4, B);
    const dim3 grid2(p.nchunk2, H / 4, B);
    const dim3 gridr(ceil_div(D * D, 256), B * H);
    const dim3 blockr(1024);
    const float* pos = position ? position : K;  // never dereferenced when dp == 0
    if (ev && record_first) (void)hipEventRecord(ev[0], stream);
    if (p.nsub > 1) {
        const dim3 block_sub(256 * kSub);
        const size_t lds = (size_t)kSub * 4 * D * D * sizeof(float);
        if (int rc = allow_sub_range_lds()) return rc;
        if (dp == 0) {
            hipLaunchKernelGGL((ktv_ln_partial_tm<0, kU1, kSub>), grid1, block_sub, lds, stream, K, V, pos, ln_weight_K,
                               ln_bias_K, ln_weight_V, ln_bias_V, norm_eps, partial, S, H, ld_in, p.tpc1);
        } else {
            hipLaunchKernelGGL((ktv_ln_partial_tm<2, kU1, kSub>), grid1, block_sub, lds, stream, K, V, pos, ln_weight_K,
                               ln_bias_K, ln_weight_V, ln_bias_V, norm_eps, partial, S, H, ld_in, p.tpc1);
        }
    } else if (dp == 0) {
        hipLaunchKernelGGL((ktv_ln_partial_tm<0, kU1, 1>), grid1, block, 0, stream, K, V, pos, ln_weight_K,
                           ln_bias_K, ln_weight_V, ln_bias_V, norm_eps, partial, S, H, ld_in, p.tpc1);
    } else {
        hipLaunchKernelGGL((ktv_ln_partial_tm<2, kU1, 1>), grid1, block, 0, stream, K, V, pos, ln_weight_K,
                           ln_bias_K, ln_weight_V, ln_bias_V, norm_eps, partial, S, H, ld_in, p.tpc1);
    }
    if (ev) (void)hipEventRecord(ev[1], stream);
    hipLaunchKernelGGL(tile_reduce, gridr, blockr, 0, stream, partial, ktv, D * D, p.nchunk1, 1.0f / (float)S);
    if (ev) (void)hipEventRecord(ev[2], stream);
    if (!apply) return check_launch("galerkin_attention_ktv");
    if (dp == 0) {
        hipLaunchKernelGGL((qm_apply_tm<0, kU2>), grid2, block, 0, stream, Q, pos, ktv, out, S, H, ld_in, p.tpc2);
    } else {
        hipLaunchKernelGGL((qm_apply_tm<2, kU2>), grid2, block, 0, stream, Q, pos, ktv, out, S, H, ld_in, p.tpc2);
    }
    if (ev) (void)hipEventRecord(ev[3], stream);
    return check_launch("galerkin_attention_fused");
}

}  // namespace

extern "C" int spgt_galerkin_attention_fused_forward(
    const float* Q, const float* K, const float* V, int64_t ld_in, const float* position,
    const float* ln_weight_K, const float* ln_bias_K, const float* ln_weight_V,
    const float* ln_bias_V, float norm_eps, float* out, float* ktv, void* workspace,
    size_t workspace_bytes, int B, int S, int H, int dp, hipStream_t stream) {
    return fused_forward_impl(Q, K, V, ld_in, position, ln_weight_K, ln_bias_K, ln_weight_V, ln_bias_V, norm_eps,
                              out, ktv, workspace, workspace_bytes, B, S, H, dp, stream, nullptr);
}

// ---------------------------------------------------------------------------
// allocation-free variant: the partial tiles live in a device array of the library
// ---------------------------------------------------------------------------

namespace spgt {
namespace {

constexpr size_t kStaticScratchBytes = SPGT_STATIC_SCRATCH_BYTES;

// One copy per GPU the library's code object is loaded on, held until the process ends.
static __device__ __align__(256) float scratch[kStaticScratchBytes / sizeof(float)];

std::atomic<float*> g_scratch_ptr[64];

// Device address of `scratch` on the current device (looked up once per device), or null with the
// error recorded.  The array's name is only a host-side handle for this lookup; every launch and
// copy uses the pointer returned here.
float* static_scratch_ptr() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        (void)fail(SPGT_ERR_LAUNCH, "galerkin_attention_fused_static: no current device");
        return nullptr;
    }
    float* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (ptr) return ptr;
    void* sym = nullptr;
    const hipError_t e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !sym) {
        (void)fail(SPGT_ERR_LAUNCH, "galerkin_attention_fused_static: hipGetSymbolAddress(scratch) failed");
        return nullptr;
    }
    ptr = static_cast<float*>(sym);
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
    return ptr;
}

}  // namespace
}  // namespace spgt

extern "C" size_t spgt_galerkin_attention_fused_static_max_bytes(void) { return kStaticScratchBytes; }

extern "C" int spgt_galerkin_attention_fused_forward_static(
    const float* Q, const float* K, const float* V, int64_t ld_in, const float* position,
    const float* ln_weight_K, const float* ln_bias_K, const float* ln_weight_V,
    const float* ln_bias_V, float norm_eps, float* out, float* ktv, int B, int S, int H, int dp,
    hipStream_t stream) {
    if (!Q || !out)  // the K/V-only form of the shared implementation is not offered here
        return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_fused_static: null pointer argument");
    const size_t need = spgt_galerkin_attention_fused_workspace_bytes(B, S, H, dp);
    if (need == 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "galerkin_attention_fused_static: B, S, H must be positive and dim_position 0 or 2");
    if (need > kStaticScratchBytes)
        return fail(SPGT_ERR_WORKSPACE,
                    "galerkin_attention_fused_static: shape needs more partial-tile scratch than the library's "
                    "static array holds (spgt_galerkin_attention_fused_static_max_bytes); use "
                    "spgt_galerkin_attention_fused_forward with a caller workspace");
    float* ws = static_scratch_ptr();
    if (!ws) return SPGT_ERR_LAUNCH;
    if (int rc = allow_sub_range_lds()) return rc;  // with the lookup above: all one-time set-up of a device
    // Every partial tile the reduction reads is written by the K/V pass of the same call, so nothing
    // in the array has to start at zero.
    return fused_forward_impl(Q, K, V, ld_in, position, ln_weight_K, ln_bias_K, ln_weight_V, ln_bias_V, norm_eps,
                              out, ktv, ws, kStaticScratchBytes, B, S, H, dp, stream, nullptr);
}

extern "C" int spgt_galerkin_attention_ktv_forward(
    const float* K, const float* V, int64_t ld_in, const float* position, const float* ln_weight_K,
    const float* ln_bias_K, const float* ln_weight_V, const float* ln_bias_V, float norm_eps, float* ktv,
    void* workspace, size_t workspace_bytes, int B, int S, int H, int dp, hipStream_t stream) {
    return fused_forward_impl(nullptr, K, V, ld_in, position, ln_weight_K, ln_bias_K, ln_weight_V, ln_bias_V,
                              norm_eps, nullptr, ktv, workspace, workspace_bytes, B, S, H, dp, stream, nullptr);
}

namespace spgt {
namespace {

// folded[b][h*32 + i][n] = sum_j ktv[b][h][dp + i][j] * fc[h*D + j][n]          (feature rows, i < 32)
// wpos[b][p][n]          = sum_h sum_j ktv[b][h][p][j] * fc[h*D + j][n]         (position rows, p < dp)
// i.e. M_h Wfc_h for every head, with the rows split the way the folded encoder tail reads them: the head's 32
// feature rows meet the projected Q, the position rows of all heads meet the same token position and are summed.
// grid (4 H + 1, B), block 256.  Workgroup x < 4 H makes 8 feature rows of head x / 4: thread = (output column n,
// n + 128, ...; half of the rows), with the D values fc[h*D + j][n] of its column in registers (requested before
// anything else) and the head's M in LDS.  Workgroup 4 H makes the position rows, all heads' columns requested
// together.  D is a compile-time value so that these loads go out together, behind no branch.
template <int DP>
__global__ __launch_bounds__(256) void fold_ktv_into_fc_k(const float* __restrict__ ktv, const float* __restrict__ fc,
                                                          float* __restrict__ folded, float* __restrict__ wpos,
                                                          int H, int N) {
    constexpr int D = DP + 32;
    extern __shared__ float ms[];  // feature workgroups: the head's M [D][D]; position workgroup: [H][DP][D]
    const int64_t b = blockIdx.y;
    const int half = threadIdx.x >> 7;
    const int n0 = threadIdx.x & 127;
    if ((int)blockIdx.x < 4 * H) {
        const int h = blockIdx.x >> 2;
        const int i0 = 8 * (blockIdx.x & 3) + 4 * half;  // this thread's 4 feature rows
        float w[D];
        const int nc = min(n0, N - 1);
#pragma unroll
        for (int j = 0; j < D; ++j) w[j] = fc[(int64_t)(h * D + j) * N + nc];
        for (int e = threadIdx.x; e < D * D; e += 256) ms[e] = ktv[(b * H + h) * D * D + e];
        __syncthreads();
        for (int n = n0; n < N; n += 128) {
            if (n != n0) {
#pragma unroll
                for (int j = 0; j < D; ++j) w[j] = fc[(int64_t)(h * D + j) * N + n];
            }
#pragma unroll
            for (int i = i0; i < i0 + 4; ++i) {
                const float* m = ms + (DP + i) * D;
                float acc = 0.f;
#pragma unroll
                for (int j = 0; j < D; ++j) acc = fmaf(m[j], w[j], acc);
                folded[(b * H * 32 + h * 32 + i) * (int64_t)N + n] = acc;
            }
        }
    } else if constexpr (DP > 0) {
        for (int e = threadIdx.x; e < H * DP * D; e += 256) {
            const int hh = e / (DP * D), rest = e - hh * (DP * D);
            ms[e] = ktv[(b * H + hh) * D * D + rest];  // rows 0 .. DP-1 of head hh
        }
        __syncthreads();
        if (half < DP) {
            for (int n = n0; n < N; n += 128) {
                float acc = 0.f;
                for (int hh = 0; hh < H; hh += 4) {  // four heads' columns in flight
                    float w[4][D];
#pragma unroll
                    for (int u = 0; u < 4; ++u)
#pragma unroll
                        for (int j = 0; j < D; ++j) w[u][j] = fc[(int64_t)(min(hh + u, H - 1) * D + j) * N + n];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        if (hh + u < H) {
                            const float* m = ms + ((hh + u) * DP + half) * D;
#pragma unroll
                            for (int j = 0; j < D; ++j) acc = fmaf(m[j], w[u][j], acc);
                        }
                    }
                }
                wpos[(b * DP + half) * (int64_t)N + n] = acc;
            }
        }
    }
}

}  // namespace
}  // namespace spgt

extern "C" int spgt_fold_ktv_into_fc(const float* ktv, const float* fc_weight_kn, float* folded, float* folded_pos,
                                     int B, int H, int dp, int out_features, hipStream_t stream) {
    if (!ktv || !fc_weight_kn || !folded || (dp > 0 && !folded_pos))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "fold_ktv_into_fc: null pointer argument");
    if (B <= 0 || H <= 0 || out_features <= 0 || (dp != 0 && dp != 2) || B > 65535 || H > 16000)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "fold_ktv_into_fc: B, H, out_features must be positive, dp 0 or 2");
    const int D = dp + 32;
    const size_t lds = (size_t)std::max(D * D, H * dp * D) * sizeof(float);
    if (lds > 64 * 1024) return fail(SPGT_ERR_INVALID_ARGUMENT, "fold_ktv_into_fc: too many heads for one workgroup");
    if (dp == 2)
        hipLaunchKernelGGL(spgt::fold_ktv_into_fc_k<2>, dim3(4 * H + 1, B), dim3(256), lds, stream, ktv, fc_weight_kn,
                           folded, folded_pos, H, out_features);
    else
        hipLaunchKernelGGL(spgt::fold_ktv_into_fc_k<0>, dim3(4 * H, B), dim3(256), lds, stream, ktv, fc_weight_kn,
                           folded, folded_pos, H, out_features);
    return check_launch("fold_ktv_into_fc");
}

extern "C" int spgt_galerkin_attention_fused_profile(
    const float* const* Q_sets, const float* const* K_sets, const float* const* V_sets, float* const* out_sets,
    int n_sets, int64_t ld_in, const float* position, const float* ln_weight_K, const float* ln_bias_K,
    const float* ln_weight_V, const float* ln_bias_V, float norm_eps, float* ktv, void* workspace,
    size_t workspace_bytes, int B, int S, int H, int dp, hipStream_t stream, int iterations, float* stage_ms) {
    if (iterations <= 0 || iterations > 4096 || !stage_ms || n_sets <= 0 || !Q_sets || !K_sets || !V_sets || !out_sets)
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "galerkin_attention_fused_profile: 1..4096 iterations, stage_ms and at least one input set required");
    // event 3 i + k: before launch k of iteration i; the last event closes the last launch
    const int nev = 3 * iterations + 1;
    std::vector<hipEvent_t> ev(nev);
    for (int i = 0; i < nev; ++i)
        if (hipEventCreate(&ev[i]) != hipSuccess) {
            for (int j = 0; j < i; ++j) (void)hipEventDestroy(ev[j]);
            return fail(SPGT_ERR_LAUNCH, "galerkin_attention_fused_profile: hipEventCreate failed");
        }
    int rc = SPGT_OK;
    for (int it = 0; it < iterations && rc == SPGT_OK; ++it) {
        const int s = it % n_sets;
        hipEvent_t four[4] = {ev[3 * it], ev[3 * it + 1], ev[3 * it + 2], ev[3 * it + 3]};
        // the closing event of one iteration is the opening event of the next: it is recorded once, by the
        // iteration it closes, and iteration 0 records its own opening event
        rc = fused_forward_impl(Q_sets[s], K_sets[s], V_sets[s], ld_in, position, ln_weight_K, ln_bias_K, ln_weight_V,
                                ln_bias_V, norm_eps, out_sets[s], ktv, workspace, workspace_bytes, B, S, H, dp, stream,
                                four, it == 0);
    }
    if (rc == SPGT_OK && hipEventSynchronize(ev[nev - 1]) != hipSuccess)
        rc = fail(SPGT_ERR_LAUNCH, "galerkin_attention_fused_profile: hipEventSynchronize failed");
    if (rc == SPGT_OK)
        for (int i = 0; i < 3 * iterations; ++i) {
            float ms = 0.f;
            (void)hipEventElapsedTime(&ms, ev[i], ev[i + 1]);
            stage_ms[i] = ms;
        }
    for (int i = 0; i < nev; ++i) (void)hipEventDestroy(ev[i]);
    return rc;
}

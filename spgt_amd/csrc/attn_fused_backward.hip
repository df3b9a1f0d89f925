// Backward of the fused Galerkin attention core on token-major operands, so that training runs on the same
// layout as the fused forward (attn_fused.hip): no feature-major copies, no separate LayerNorm backward pass.
//
// Reference behaviour restated here:
//   multihead_galerkin_attention_cccr_backward      extension/bind/galerkin_attention.cu:126-173
//   mh32::lnorm_grad_ccc_cuda (LayerNorm backward)  extension/native/multihead_dim32.cu:148-271
// Forward, per batch entry and head (D = dp + 32, rows of Q~, K~, V~ are [position | features]):
//   K~ = [pos | LN_K(k)],  V~ = [pos | LN_V(v)],  Q~ = [pos | q],  M = K~^T V~ / S,  out = Q~ M
// Backward from G = dL/dout [S, D]:
//   N    = Q~^T G / S                                        (D x D; pass 1 + tile_reduce)
//   dq   = (G M^T)[:, dp:]                                    }
//   dK~  = V~ N^T,  dV~ = K~ N                                } pass 2, one stream over k, v, G
//   dk   = LN_K'(k; dK~[:, dp:]),  dv = LN_V'(v; dV~[:, dp:]) }
//   dgamma, dbeta of both LayerNorms: per-workgroup sums, then a fixed-order sum over the workgroups.
// The LayerNorm statistics are recomputed from k and v (cheaper than storing and re-reading them); the position
// columns receive no gradient (the position tensor is an input of the model, not a parameter).
#include "spgt_device.h"
#include "spgt_host.h"
#include "spgt_kernels.h"

// Cache policy of the touch-once streams: q (pass 1) and k, v (pass 2) are read once, grad_out is read by both
// passes (182 MB at B=8, S=44521: it can stay in the 256 MB last-level cache between them if the other streams
// do not displace it).
#ifndef SPGT_BWD_NT_Q
#define SPGT_BWD_NT_Q true
#endif
#ifndef SPGT_BWD_NT_KV
#define SPGT_BWD_NT_KV true
#endif

namespace spgt {

// Pass 1: partial[b][h][chunk] = sum over the chunk's tokens of Q~[s]^T G[s]  (D x D, row-major; the dp x dp
// corner is not needed by pass 2 and is written as zero).
// grid (nchunk, H/4, B), block 256 * NSUB: wave w handles head 4 blockIdx.y + w % 4 on the sub-range w / 4 of the
// workgroup's chunk; with NSUB > 1 the sub-ranges' tiles meet in LDS and the workgroup writes their sum (sub-ranges
// in increasing order), as in the forward's K/V pass: one 1024-thread workgroup per CU on long sequences.
// Lane l: token slot t = l/16, feature pair p = l%16; a 16x16x4 MFMA contracts the four token slots:
// A = q[2p + ta], B = G[2p + tb].
template <int DP, int U, int NSUB>
__global__ __launch_bounds__(256 * NSUB) void qtg_partial_tm(const float* __restrict__ Q, int64_t ld,
                                                             const float* __restrict__ pos,
                                                             const float* __restrict__ G,
                                                             float* __restrict__ partial, int S, int H,
                                                             int tokens_per_chunk) {
    constexpr int D = DP + 32;
    extern __shared__ __attribute__((aligned(16))) float sub_tiles[];  // NSUB > 1: [NSUB][4 heads][D * D]
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
    const int64_t ldg = (int64_t)H * D;
    const float* qb = Q + ((int64_t)b * S + s0) * ld + h * 32 + 2 * p;
    const float* gb = G + ((int64_t)b * S + s0) * ldg + h * D;
    const float* pb = pos + ((int64_t)b * S + s0) * 2;

    struct Unit { float2 q, g; };
    v4f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};
    float qgp[2][2] = {{0.f, 0.f}, {0.f, 0.f}};  // sum q[ta] * G[position column a]
    float pg[2][2] = {{0.f, 0.f}, {0.f, 0.f}};   // sum pos[a] * G[feature tb]

    // DP == 2: a group of 4*U tokens needs 8*U position floats and 8*U floats of G's position columns.  One load
    // instruction per group fetches both (lanes 0-31 a position float, lanes 32-63 a float of G) and a
    // wave-private LDS stage hands each token slot its U pairs of either kind, side by side; loads of their own
    // per unit would double the vector memory instructions of the pass for 3 % more bytes.
    static_assert(DP == 0 || 8 * U == 32, "a group's position floats fill half a wave");
    __shared__ __attribute__((aligned(16))) float pair_stage[DP == 2 ? 4 * NSUB * 16 * U : 4];
    float* const pstage = pair_stage + (sub * 4 + wave) * (16 * U);
    const int pkind = lane >> 5;                 // 0: position, 1: G's position columns
    const int ptok = (lane & 31) >> 1;           // token of the group
    const int pc = lane & 1;
    const int pdst = (ptok & 3) * (4 * U) + pkind * (2 * U) + (ptok >> 2) * 2 + pc;  // [slot][kind][unit][c]

    auto load_unit = [&](int rel) {
        Unit u;
        u.q = ld_stream<SPGT_BWD_NT_Q>(reinterpret_cast<const float2*>(qb + (int64_t)rel * ld));
        u.g = *reinterpret_cast<const float2*>(gb + (int64_t)rel * ldg + DP + 2 * p);
        return u;
    };
    auto compute_unit = [&](const Unit& u, float2 ps, float2 gp, bool valid) {
        const float q0 = valid ? u.q.x : 0.f, q1 = valid ? u.q.y : 0.f;
        acc[0][0] = mfma16(q0, u.g.x, acc[0][0]);
        acc[0][1] = mfma16(q0, u.g.y, acc[0][1]);
        acc[1][0] = mfma16(q1, u.g.x, acc[1][0]);
        acc[1][1] = mfma16(q1, u.g.y, acc[1][1]);
        if (DP == 2) {
            const float p0 = valid ? ps.x : 0.f, p1 = valid ? ps.y : 0.f;
            qgp[0][0] = fmaf(q0, gp.x, qgp[0][0]);
            qgp[0][1] = fmaf(q0, gp.y, qgp[0][1]);
            qgp[1][0] = fmaf(q1, gp.x, qgp[1][0]);
            qgp[1][1] = fmaf(q1, gp.y, qgp[1][1]);
            pg[0][0] = fmaf(p0, u.g.x, pg[0][0]);
            pg[0][1] = fmaf(p0, u.g.y, pg[0][1]);
            pg[1][0] = fmaf(p1, u.g.x, pg[1][0]);
            pg[1][1] = fmaf(p1, u.g.y, pg[1][1]);
        }
    };
    // two register buffers of U units (4 tokens each), the next group requested before the current one is used
    constexpr int GT = 4 * U;
    const int len = s1 - s0;
    const int ngroup = (len + GT - 1) / GT;
    Unit bufA[U], bufB[U];
    float prawA = 0.f, prawB = 0.f;
    auto load_group = [&](Unit(&buf)[U], float& praw, int g) {
        const int gbase = min(g, ngroup - 1) * GT;
        const int base = gbase + t;
#pragma unroll
        for (int u = 0; u < U; ++u) buf[u] = load_unit(min(base + 4 * u, len - 1));
        if (DP == 2) {
            const int64_t rel = min(gbase + ptok, len - 1);
            praw = pkind == 0 ? pb[rel * 2 + pc] : gb[rel * ldg + pc];
        }
    };
    auto compute_group = [&](const Unit(&buf)[U], float praw, int g) {
        const int base = g * GT + t;
        float pairs[4 * U];  // this lane's token slot: positions of units 0 .. U-1, then G's position columns
        if (DP == 2) {
            // (the stage is the wave's own: LDS operations of one wave complete in order, no barrier)
            pstage[pdst] = praw;
#pragma unroll
            for (int i = 0; i < 4 * U; i += 4) {
                const float4 v = *reinterpret_cast<const float4*>(pstage + t * (4 * U) + i);
                pairs[i] = v.x; pairs[i + 1] = v.y; pairs[i + 2] = v.z; pairs[i + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4 * U; ++i) pairs[i] = 0.f;
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            compute_unit(buf[u], make_float2(pairs[2 * u], pairs[2 * u + 1]),
                         make_float2(pairs[2 * U + 2 * u], pairs[2 * U + 2 * u + 1]), base + 4 * u < len);
    };
    if (ngroup > 0) {
        load_group(bufA, prawA, 0);
        for (int g = 0; g < ngroup; g += 2) {
            load_group(bufB, prawB, g + 1);
            __builtin_amdgcn_sched_barrier(0);
            compute_group(bufA, prawA, g);
            __builtin_amdgcn_sched_barrier(0);
            load_group(bufA, prawA, g + 2);
            __builtin_amdgcn_sched_barrier(0);
            if (g + 1 < ngroup) compute_group(bufB, prawB, g + 1);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // acc[ta][tb][r] = N[DP + 2 (4 t + r) + ta][DP + 2 p + tb]
    float* tile = NSUB > 1 ? sub_tiles + (sub * 4 + wave) * (D * D)
                           : partial + (((int64_t)b * H + h) * nchunk + chunk) * (D * D);
#pragma unroll
    for (int ta = 0; ta < 2; ++ta)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int i = DP + 8 * t + 2 * r + ta;
            *reinterpret_cast<float2*>(tile + i * D + DP + 2 * p) = make_float2(acc[ta][0][r], acc[ta][1][r]);
        }
    if (DP == 2) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                qgp[i][j] = rows4_allsum(qgp[i][j]);
                pg[i][j] = rows4_allsum(pg[i][j]);
            }
        if (t == 0) {
#pragma unroll
            for (int ta = 0; ta < 2; ++ta)
                *reinterpret_cast<float2*>(tile + (DP + 2 * p + ta) * D) = make_float2(qgp[ta][0], qgp[ta][1]);
#pragma unroll
            for (int a = 0; a < 2; ++a)
                *reinterpret_cast<float2*>(tile + a * D + DP + 2 * p) = make_float2(pg[a][0], pg[a][1]);
            if (p == 0) {
                tile[0] = 0.f; tile[1] = 0.f; tile[D] = 0.f; tile[D + 1] = 0.f;
            }
        }
    }
    if constexpr (NSUB > 1) {
        __syncthreads();
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
            float* dst = partial + (((int64_t)b * H + blockIdx.y * 4 + hh) * nchunk + chunk) * (D * D) + 4 * r4;
            *reinterpret_cast<float4*>(dst) = sum;
        }
    }
}

// Pass 2.  grid (nchunk, H/4, B), block 256: wave = head.  Lane l: token slot tk = l%16, feature group g = l/16;
// the lane holds features f(e) = 4g + e (e < 4) and 16 + 4g + e - 4 (e >= 4) of its token, for inputs and results
// alike: a 16x16x4 MFMA step kk contracts the features {f(kk) of g = 0..3}, and element r of accumulator jb is
// result feature 16 jb + 4g + r = f(4 jb + r).
//   gpart [gridDim.x * B][H/4][4][128]: per workgroup the sums over its tokens of dy*x_hat (K), dy (K), dy*x_hat (V),
//   dy (V) for the 128 features of its four heads.
template <int DP>
__global__ __launch_bounds__(256) void attn_bwd_apply_tm(
    const float* __restrict__ K, const float* __restrict__ V, int64_t ld, const float* __restrict__ pos,
    const float* __restrict__ G, const float* __restrict__ M, const float* __restrict__ Nm,
    const float* __restrict__ lnwK, const float* __restrict__ lnbK, const float* __restrict__ lnwV,
    const float* __restrict__ lnbV, float eps, float* __restrict__ dQ, float* __restrict__ dK,
    float* __restrict__ dV, int64_t ldo, float* __restrict__ gpart, int S, int H, int tokens_per_chunk) {
    constexpr int D = DP + 32;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int h = blockIdx.y * 4 + wave;
    const int b = blockIdx.z;
    const int tk = lane & 15;
    const int g = lane >> 4;
    const int s0 = blockIdx.x * tokens_per_chunk;
    const int s1 = min(S, s0 + tokens_per_chunk);
    const int64_t ldg = (int64_t)H * D;
    auto feat = [&](int e) { return e < 4 ? 4 * g + e : 16 + 4 * g + e - 4; };

    const float* m = M + ((int64_t)b * H + h) * (D * D);
    const float* n = Nm + ((int64_t)b * H + h) * (D * D);
    // MFMA A operands: W[kk][jb] = W_op[result feature 16 jb + tk][contraction feature f(kk)]
    float wq[8][2], wk[8][2], wv[8][2];
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
        const int c = feat(kk);
#pragma unroll
        for (int jb = 0; jb < 2; ++jb) {
            const int o = 16 * jb + tk;
            wq[kk][jb] = m[(DP + o) * D + DP + c];  // dq[o]  = sum_c G[c]   M[o][c]
            wk[kk][jb] = n[(DP + o) * D + DP + c];  // dK~[o] = sum_c V~[c]  N[o][c]
            wv[kk][jb] = n[(DP + c) * D + DP + o];  // dV~[o] = sum_c K~[c]  N[c][o]
        }
    }
    // position columns / rows of the two matrices for this lane's result features
    float mq_p[8][2], nk_p[8][2], nv_p[8][2];
    if (DP == 2) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int o = feat(e);
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                mq_p[e][a] = m[(DP + o) * D + a];
                nk_p[e][a] = n[(DP + o) * D + a];
                nv_p[e][a] = n[a * D + DP + o];
            }
        }
    }
    float gK[8], bK[8], gV[8], bV[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int f = h * 32 + feat(e);
        gK[e] = lnwK[f]; bK[e] = lnbK[f]; gV[e] = lnwV[f]; bV[e] = lnbV[f];
    }
    float sgK[8], sbK[8], sgV[8], sbV[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) sgK[e] = sbK[e] = sgV[e] = sbV[e] = 0.f;

    const float* kbase = K + (int64_t)b * S * ld + h * 32 + 4 * g;
    const float* vbase = V + (int64_t)b * S * ld + h * 32 + 4 * g;
    const float* gbase = G + (int64_t)b * S * ldg + h * D;
    const float* pbase = pos + (int64_t)b * S * 2;
    float* qo = dQ + (int64_t)b * S * ldo + h * 32;
    float* ko = dK + (int64_t)b * S * ldo + h * 32;
    float* vo = dV + (int64_t)b * S * ldo + h * 32;

    struct Unit { float4 k0, k1, v0, v1; float2 g0, g1, g2, g3, gp, ps; };
    auto load_unit = [&](int s) {
        Unit u;
        const float* kp = kbase + (int64_t)s * ld;
        const float* vp = vbase + (int64_t)s * ld;
        const float* gp = gbase + (int64_t)s * ldg + DP + 4 * g;
        u.k0 = ld_stream<SPGT_BWD_NT_KV>(reinterpret_cast<const float4*>(kp));
        u.k1 = ld_stream<SPGT_BWD_NT_KV>(reinterpret_cast<const float4*>(kp + 16));
        u.v0 = ld_stream<SPGT_BWD_NT_KV>(reinterpret_cast<const float4*>(vp));
        u.v1 = ld_stream<SPGT_BWD_NT_KV>(reinterpret_cast<const float4*>(vp + 16));
        u.g0 = *reinterpret_cast<const float2*>(gp);       // rows of 34 floats: 8-byte pieces
        u.g1 = *reinterpret_cast<const float2*>(gp + 2);
        u.g2 = *reinterpret_cast<const float2*>(gp + 16);
        u.g3 = *reinterpret_cast<const float2*>(gp + 18);
        if (DP == 2) {
            u.gp = *reinterpret_cast<const float2*>(gbase + (int64_t)s * ldg);
            u.ps = *reinterpret_cast<const float2*>(pbase + (int64_t)s * 2);
        } else {
            u.gp = make_float2(0.f, 0.f);
            u.ps = make_float2(0.f, 0.f);
        }
        return u;
    };
    // rows of 8 tokens x 128 bytes per store instruction: lanes tk and tk^8 swap halves (see qm_apply_tm)
    auto store_rows = [&](float* base, const v4f (&acc)[2], int sb) {
        const bool lo = tk < 8;
        float o0[4], o1[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            o0[r] = dpp_move<SPGT_DPP_ROW_ROR8>(acc[0][r]);
            o1[r] = dpp_move<SPGT_DPP_ROW_ROR8>(acc[1][r]);
        }
        float4 x, y;
        x.x = lo ? acc[0][0] : o1[0]; x.y = lo ? acc[0][1] : o1[1]; x.z = lo ? acc[0][2] : o1[2]; x.w = lo ? acc[0][3] : o1[3];
        y.x = lo ? o0[0] : acc[1][0]; y.y = lo ? o0[1] : acc[1][1]; y.z = lo ? o0[2] : acc[1][2]; y.w = lo ? o0[3] : acc[1][3];
        const int fo = (lo ? 0 : 16) + 4 * g;
        const int sx = sb + (tk & 7);
        const int sy = sx + 8;
        if (sx < s1) st_stream<true>(reinterpret_cast<float4*>(base + (int64_t)sx * ldo + fo), x);
        if (sy < s1) st_stream<true>(reinterpret_cast<float4*>(base + (int64_t)sy * ldo + fo), y);
    };
    auto compute_unit = [&](const Unit& u, int sb) {
        const bool valid = sb + tk < s1;
        const float vm = valid ? 1.f : 0.f;
        float kx[8] = {u.k0.x, u.k0.y, u.k0.z, u.k0.w, u.k1.x, u.k1.y, u.k1.z, u.k1.w};
        float vx[8] = {u.v0.x, u.v0.y, u.v0.z, u.v0.w, u.v1.x, u.v1.y, u.v1.z, u.v1.w};
        const float gx[8] = {u.g0.x, u.g0.y, u.g1.x, u.g1.y, u.g2.x, u.g2.y, u.g3.x, u.g3.y};
        // LayerNorm statistics of the token's 32 features of this head (8 here, 24 in lanes l^16, l^32, l^48)
        float sk = 0.f, sv = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) { sk += kx[e]; sv += vx[e]; }
        const float mk = rows4_allsum(sk) * (1.0f / 32.0f), mv = rows4_allsum(sv) * (1.0f / 32.0f);
        float qk = 0.f, qv = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            kx[e] -= mk; vx[e] -= mv;
            qk = fmaf(kx[e], kx[e], qk); qv = fmaf(vx[e], vx[e], qv);
        }
        const float rk = __builtin_amdgcn_rsqf(fmaf(rows4_allsum(qk), 1.0f / 32.0f, eps));
        const float rv = __builtin_amdgcn_rsqf(fmaf(rows4_allsum(qv), 1.0f / 32.0f, eps));
        float yk[8], yv[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            kx[e] *= rk; vx[e] *= rv;  // x_hat
            yk[e] = fmaf(kx[e], gK[e], bK[e]);
            yv[e] = fmaf(vx[e], gV[e], bV[e]);
        }
        v4f aq[2], ak[2], av[2];
#pragma unroll
        for (int jb = 0; jb < 2; ++jb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int e = 4 * jb + r;
                if (DP == 2) {
                    aq[jb][r] = fmaf(u.gp.y, mq_p[e][1], u.gp.x * mq_p[e][0]);
                    ak[jb][r] = fmaf(u.ps.y, nk_p[e][1], u.ps.x * nk_p[e][0]);
                    av[jb][r] = fmaf(u.ps.y, nv_p[e][1], u.ps.x * nv_p[e][0]);
                } else {
                    aq[jb][r] = 0.f; ak[jb][r] = 0.f; av[jb][r] = 0.f;
                }
            }
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
            aq[0] = mfma16(wq[kk][0], gx[kk], aq[0]);
            aq[1] = mfma16(wq[kk][1], gx[kk], aq[1]);
            ak[0] = mfma16(wk[kk][0], yv[kk], ak[0]);
            ak[1] = mfma16(wk[kk][1], yv[kk], ak[1]);
            av[0] = mfma16(wv[kk][0], yk[kk], av[0]);
            av[1] = mfma16(wv[kk][1], yk[kk], av[1]);
        }
        // LayerNorm backward: a = dy * gamma; dx = rstd * (a - mean(a) - x_hat * mean(a * x_hat))
        float a1k = 0.f, a2k = 0.f, a1v = 0.f, a2v = 0.f;
        float ka[8], va[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float dyk = ak[e >> 2][e & 3], dyv = av[e >> 2][e & 3];
            ka[e] = dyk * gK[e]; va[e] = dyv * gV[e];
            a1k += ka[e]; a1v += va[e];
            a2k = fmaf(ka[e], kx[e], a2k); a2v = fmaf(va[e], vx[e], a2v);
            sgK[e] = fmaf(dyk * vm, kx[e], sgK[e]); sbK[e] = fmaf(dyk, vm, sbK[e]);
            sgV[e] = fmaf(dyv * vm, vx[e], sgV[e]); sbV[e] = fmaf(dyv, vm, sbV[e]);
        }
        a1k = rows4_allsum(a1k) * (1.0f / 32.0f); a2k = rows4_allsum(a2k) * (1.0f / 32.0f);
        a1v = rows4_allsum(a1v) * (1.0f / 32.0f); a2v = rows4_allsum(a2v) * (1.0f / 32.0f);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            ak[e >> 2][e & 3] = rk * (ka[e] - a1k - kx[e] * a2k);
            av[e >> 2][e & 3] = rv * (va[e] - a1v - vx[e] * a2v);
        }
        store_rows(qo, aq, sb);
        store_rows(ko, ak, sb);
        store_rows(vo, av, sb);
    };

    const int len = s1 - s0;
    const int nunit = (len + 15) / 16;
    if (nunit > 0) {
        Unit ua = load_unit(min(s0 + tk, s1 - 1)), ub;
        for (int i = 0; i < nunit; i += 2) {
            ub = load_unit(min(s0 + 16 * min(i + 1, nunit - 1) + tk, s1 - 1));
            __builtin_amdgcn_sched_barrier(0);
            compute_unit(ua, s0 + 16 * i);
            __builtin_amdgcn_sched_barrier(0);
            ua = load_unit(min(s0 + 16 * min(i + 2, nunit - 1) + tk, s1 - 1));
            __builtin_amdgcn_sched_barrier(0);
            if (i + 1 < nunit) compute_unit(ub, s0 + 16 * (i + 1));
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // sums over the wave's token slots (the 16 lanes of a DPP row), one row of 4 x 128 values per workgroup
    float* gp = gpart + (((int64_t)blockIdx.x * gridDim.z + b) * gridDim.y + blockIdx.y) * (4 * 128) + wave * 32;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float v0 = row16_allsum(sgK[e]), v1 = row16_allsum(sbK[e]);
        const float v2 = row16_allsum(sgV[e]), v3 = row16_allsum(sbV[e]);
        if (tk == 0) {
            const int f = feat(e);
            gp[f] = v0; gp[128 + f] = v1; gp[256 + f] = v2; gp[384 + f] = v3;
        }
    }
}

// out[which][h * 32 + f] = sum over blocks of gpart[block][h / 4][which][32 (h % 4) + f]: the per-workgroup rows
// have the four heads of a head group side by side; this gathers them into [4][H * 32] sums, blocks in a fixed
// order (eight interleaved chains, then a fixed tree).  grid (H / 4, 4), block 1024 = 8 chains x 128 features.
__global__ __launch_bounds__(1024) void ln_param_sum_k(const float* __restrict__ gpart, float* __restrict__ out,
                                                       int nblock, int HG, int H) {
    __shared__ float sm[8][128];
    const int q = threadIdx.x >> 7;   // chain 0..7
    const int c = threadIdx.x & 127;  // feature of the head group
    const int hg = blockIdx.x, which = blockIdx.y;
    const float* src = gpart + ((int64_t)hg * 4 + which) * 128 + c;
    const int64_t stride = (int64_t)HG * 4 * 128;
    float s = 0.f;
    for (int b0 = q; b0 < nblock; b0 += 8 * 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int blk = b0 + 8 * u;
            v[u] = blk < nblock ? src[(int64_t)blk * stride] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) s += v[u];
    }
    sm[q][c] = s;
    __syncthreads();
    if (q == 0) {
        float t[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) t[i] = sm[i][c];
#pragma unroll
        for (int w = 4; w >= 1; w /= 2)
#pragma unroll
            for (int i = 0; i < w; ++i) t[i] += t[i + w];
        out[(int64_t)which * H * 32 + hg * 128 + c] = t[0];
    }
}

}  // namespace spgt

using namespace spgt;

namespace {

size_t round256(size_t x) { return (x + 255) & ~(size_t)255; }

constexpr int kBwdSub = 4;           // token sub-ranges per 1024-thread workgroup of pass 1 on long sequences
constexpr int kBwdSubMinTokens = 256;  // per wave

struct FusedBwdPlan {
    int nsub, tpc1, nchunk1, tpc2, nchunk2;
    size_t off_n, off_gpart, bytes;
};

FusedBwdPlan fused_bwd_plan(int B, int S, int H, int dp) {
    const int D = dp + 32;
    const int bg = std::max(1, B * (H / 4));
    const int cus = device_cu_count();
    FusedBwdPlan p;
    // pass 1: three workgroups per CU (one per CU when that leaves chunks of under 128 tokens), at most as many
    // chunks as tile_reduce sums
    const int t1 = S / std::max(1, 3 * cus / bg) < 128 ? cus : 3 * cus;
    const int per1 = std::min(kReduceChains * kReduceMaxPerChain, std::max(1, t1 / bg));
    p.nsub = 1;
    p.tpc1 = std::max(16, ceil_div(ceil_div(S, per1), 16) * 16);
    // long sequences: one workgroup of kBwdSub x 4 waves per CU, whose sub-range tiles are summed in LDS
    const int gs = 16 * kBwdSub;
    const int tpc_sub = std::max(gs, ceil_div(ceil_div(S, std::max(1, cus / bg)), gs) * gs);
    if (tpc_sub / kBwdSub >= kBwdSubMinTokens && ceil_div(S, tpc_sub) <= kReduceChains * kReduceMaxPerChain) {
        p.nsub = kBwdSub;
        p.tpc1 = tpc_sub;
    }
    p.nchunk1 = ceil_div(S, p.tpc1);
    // pass 2: two workgroups per CU
    const int per2 = std::max(1, 2 * cus / bg);
    p.tpc2 = std::max(32, ceil_div(ceil_div(S, per2), 32) * 32);
    p.nchunk2 = ceil_div(S, p.tpc2);
    const size_t tiles = (size_t)B * H * p.nchunk1 * D * D * sizeof(float);
    p.off_n = round256(tiles);
    p.off_gpart = p.off_n + round256((size_t)B * H * D * D * sizeof(float));
    p.bytes = p.off_gpart + round256((size_t)p.nchunk2 * B * (H / 4) * 4 * 128 * sizeof(float));
    return p;
}

}  // namespace

extern "C" size_t spgt_galerkin_attention_fused_backward_workspace_bytes(int B, int S, int H, int dp) {
    if (B <= 0 || S <= 0 || H <= 0 || H % 4 != 0 || (dp != 0 && dp != 2)) return 0;
    return fused_bwd_plan(B, S, H, dp).bytes;
}

extern "C" int spgt_galerkin_attention_fused_backward(
    const float* grad_out, const float* Q, const float* K, const float* V, int64_t ld_in, const float* position,
    const float* ln_weight_K, const float* ln_bias_K, const float* ln_weight_V, const float* ln_bias_V,
    float norm_eps, const float* ktv, float* grad_Q, float* grad_K, float* grad_V, int64_t ld_out, float* grad_ln,
    void* workspace, size_t workspace_bytes, int B, int S, int H, int dp, hipStream_t stream) {
    if (!grad_out || !Q || !K || !V || !ln_weight_K || !ln_bias_K || !ln_weight_V || !ln_bias_V || !ktv || !grad_Q ||
        !grad_K || !grad_V || !grad_ln)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_fused_backward: null pointer argument");
    if (B <= 0 || S <= 0 || H <= 0 || H % 4 != 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "galerkin_attention_fused_backward: B, S, H must be positive, H a multiple of 4");
    if (dp != 0 && dp != 2)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_fused_backward: dim_position must be 0 or 2");
    if (dp == 2 && !position)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_fused_backward: position is null with dim_position 2");
    if (ld_in < (int64_t)H * 32 || ld_in % 4 != 0 || ld_out < (int64_t)H * 32 || ld_out % 4 != 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "galerkin_attention_fused_backward: row strides must be >= H*32 and multiples of 4 floats");
    if (!aligned16(Q) || !aligned16(K) || !aligned16(V) || !aligned16(grad_Q) || !aligned16(grad_K) ||
        !aligned16(grad_V) || !aligned8(grad_out) || !aligned16(ktv) || !aligned16(grad_ln) ||
        (position && !aligned8(position)))
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "galerkin_attention_fused_backward: operands must be 16-byte aligned (grad_out, position: 8)");
    if (B > 65535 || H / 4 > 65535)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_fused_backward: batch or head count exceeds the grid limit");
    const FusedBwdPlan p = fused_bwd_plan(B, S, H, dp);
    if (!workspace || workspace_bytes < p.bytes || !aligned16(workspace))
        return fail(SPGT_ERR_WORKSPACE, "galerkin_attention_fused_backward: workspace missing, misaligned or too small");
    const int D = dp + 32;
    char* ws = static_cast<char*>(workspace);
    float* partial = reinterpret_cast<float*>(ws);
    float* nmat = reinterpret_cast<float*>(ws + p.off_n);
    float* gpart = reinterpret_cast<float*>(ws + p.off_gpart);
    const float* pos = position ? position : K;  // never dereferenced when dp == 0
    const dim3 grid1(p.nchunk1, H / 4, B), grid2(p.nchunk2, H / 4, B);
    if (p.nsub > 1) {
        const size_t lds = (size_t)kBwdSub * 4 * D * D * sizeof(float);
        const void* fn = dp == 0 ? reinterpret_cast<const void*>(&qtg_partial_tm<0, 4, kBwdSub>)
                                 : reinterpret_cast<const void*>(&qtg_partial_tm<2, 4, kBwdSub>);
        if (!allow_dynamic_lds(fn, lds))
            return fail(SPGT_ERR_LAUNCH, "galerkin_attention_fused_backward: pass 1 was refused its dynamic LDS size");
        if (dp == 0)
            hipLaunchKernelGGL((qtg_partial_tm<0, 4, kBwdSub>), grid1, dim3(256 * kBwdSub), lds, stream, Q, ld_in, pos,
                               grad_out, partial, S, H, p.tpc1);
        else
            hipLaunchKernelGGL((qtg_partial_tm<2, 4, kBwdSub>), grid1, dim3(256 * kBwdSub), lds, stream, Q, ld_in, pos,
                               grad_out, partial, S, H, p.tpc1);
    } else if (dp == 0) {
        hipLaunchKernelGGL((qtg_partial_tm<0, 4, 1>), grid1, dim3(256), 0, stream, Q, ld_in, pos, grad_out, partial, S, H, p.tpc1);
    } else {
        hipLaunchKernelGGL((qtg_partial_tm<2, 4, 1>), grid1, dim3(256), 0, stream, Q, ld_in, pos, grad_out, partial, S, H, p.tpc1);
    }
    hipLaunchKernelGGL(tile_reduce, dim3(ceil_div(D * D, 256), B * H), dim3(1024), 0, stream, partial, nmat, D * D,
                       p.nchunk1, 1.0f / (float)S);
    if (dp == 0)
        hipLaunchKernelGGL((attn_bwd_apply_tm<0>), grid2, dim3(256), 0, stream, K, V, ld_in, pos, grad_out, ktv, nmat,
                           ln_weight_K, ln_bias_K, ln_weight_V, ln_bias_V, norm_eps, grad_Q, grad_K, grad_V, ld_out,
                           gpart, S, H, p.tpc2);
    else
        hipLaunchKernelGGL((attn_bwd_apply_tm<2>), grid2, dim3(256), 0, stream, K, V, ld_in, pos, grad_out, ktv, nmat,
                           ln_weight_K, ln_bias_K, ln_weight_V, ln_bias_V, norm_eps, grad_Q, grad_K, grad_V, ld_out,
                           gpart, S, H, p.tpc2);
    hipLaunchKernelGGL(ln_param_sum_k, dim3(H / 4, 4), dim3(1024), 0, stream, gpart, grad_ln, p.nchunk2 * B, H / 4, H);
    return check_launch("galerkin_attention_fused_backward");
}

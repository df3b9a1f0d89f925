// Galerkin attention on feature-major operands (the reference operator's layout):
//   Q, K, V : [B*H, D, S] (S contiguous, rows only 4-byte aligned when S is odd)
//   out     : [B*H, S, D],  out[s][j] = sum_i Q[i][s] * ( sum_t K[i][t] V[j][t] / S )
// D = 32, or 34 with two position rows in front of the 32 feature rows.
//
// Reference behaviour restated here:
//   multihead_galerkin_attention_cccr_forward   extension/bind/galerkin_attention.cu:104-124
//   (split-K SGEMM order RCC, then the small-K SGEMM order CCR;
//    extension/native/sgemm_32x32_splitk.cu:662-705, extension/native/sgemm_32x32.cu:683-710)
//
// Three launches:
//   1. ktv_partial_fm - K and V rows of one (batch, head) and one token range are
//      staged through LDS with 512-byte row reads; each wave contracts a quarter of
//      every 128-token step on v_mfma_f32_32x32x2_f32 (feature rows), the two
//      position rows/columns (D = 34) go through the VALU from broadcast LDS reads;
//      the four wave accumulators are added in wave order.
//   2. tile_reduce    - fixed-order sum of the partial D x D tiles, x 1/S.
//   3. qm_apply_fm    - streams Q with 16-byte row reads (4 tokens per lane), keeps
//      M^T in registers as the v_mfma_f32_16x16x4_f32 A operand, writes whole
//      128-byte output rows.
#include "spgt_device.h"
#include "spgt_host.h"
#include "spgt_kernels.h"

namespace spgt {

namespace {
constexpr int kFmKT = 128;     // tokens per LDS stage
constexpr int kFmPitch = 129;  // odd pitch: conflict-free column reads
}  // namespace

// grid (nchunk, BH), block 256.  partial[(bh * nchunk + chunk) * D*D + i*D + j]
template <int D>
__global__ __launch_bounds__(256) void ktv_partial_fm(const float* __restrict__ K, const float* __restrict__ V,
                                                      float* __restrict__ partial, int S, int tokens_per_chunk) {
    constexpr int DP = D - 32;
    constexpr int RPW = (D + 3) / 4;  // rows per wave in the loader
    __shared__ float sk[D * kFmPitch];
    __shared__ float sv[D * kFmPitch];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t bh = blockIdx.y;
    const int chunk = blockIdx.x;
    const int s0 = chunk * tokens_per_chunk;
    const int s1 = min(S, s0 + tokens_per_chunk);
    const float* Kb = K + bh * D * (int64_t)S;
    const float* Vb = V + bh * D * (int64_t)S;

    v16f acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    float ck[2] = {0.f, 0.f};   // sum_k K[DP + lane%32][k] * V[a][k]   -> M[DP+i][a]
    float rv[2] = {0.f, 0.f};   // sum_k K[a][k] * V[DP + lane%32][k]   -> M[a][DP+j]
    float pp[4] = {0.f, 0.f, 0.f, 0.f};  // sum_k K[a][k] * V[a'][k]

    float2 rk[RPW], rvv[RPW];
    auto load_step = [&](int sb) {
        const int s = sb + 2 * lane;
#pragma unroll
        for (int i = 0; i < RPW; ++i) {
            const int row = wave + 4 * i;
            float2 a = make_float2(0.f, 0.f), b = make_float2(0.f, 0.f);
            if (row < D) {
                const float* kp = Kb + (int64_t)row * S + s;
                const float* vp = Vb + (int64_t)row * S + s;
                if (s + 1 < s1) {
                    const v2f ka = __builtin_nontemporal_load(reinterpret_cast<const v2f_a4*>(kp));
                    const v2f va = __builtin_nontemporal_load(reinterpret_cast<const v2f_a4*>(vp));
                    a = make_float2(ka.x, ka.y);
                    b = make_float2(va.x, va.y);
                } else if (s < s1) {
                    a.x = kp[0];
                    b.x = vp[0];
                }
            }
            rk[i] = a;
            rvv[i] = b;
        }
    };
    auto store_step = [&]() {
#pragma unroll
        for (int i = 0; i < RPW; ++i) {
            const int row = wave + 4 * i;
            if (row < D) {
                float* dk = sk + row * kFmPitch + 2 * lane;
                float* dv = sv + row * kFmPitch + 2 * lane;
                dk[0] = rk[i].x; dk[1] = rk[i].y;
                dv[0] = rvv[i].x; dv[1] = rvv[i].y;
            }
        }
    };

    if (s0 < s1) load_step(s0);
    for (int sb = s0; sb < s1; sb += kFmKT) {
        __syncthreads();  // previous stage fully consumed
        store_step();
        __syncthreads();
        if (sb + kFmKT < s1) load_step(sb + kFmKT);
        const float* ak = sk + (DP + (lane & 31)) * kFmPitch;
        const float* bv = sv + (DP + (lane & 31)) * kFmPitch;
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            const int k = 32 * wave + 2 * kk + (lane >> 5);
            const float a = ak[k];
            const float b = bv[k];
            acc = mfma32(a, b, acc);
            if (DP == 2) {
                const float k0 = sk[k], k1 = sk[kFmPitch + k];
                const float v0 = sv[k], v1 = sv[kFmPitch + k];
                ck[0] = fmaf(a, v0, ck[0]);
                ck[1] = fmaf(a, v1, ck[1]);
                rv[0] = fmaf(k0, b, rv[0]);
                rv[1] = fmaf(k1, b, rv[1]);
                pp[0] = fmaf(k0, v0, pp[0]);
                pp[1] = fmaf(k0, v1, pp[1]);
                pp[2] = fmaf(k1, v0, pp[2]);
                pp[3] = fmaf(k1, v1, pp[3]);
            }
        }
    }
    __syncthreads();
    // Cross-wave sum in wave order through LDS: the K stage holds the tiles of waves 0 and 1,
    // the V stage those of waves 2 and 3 (2 * D*D <= D * 129 floats).
    float* red01 = sk;
    float* red23 = sv;
    float* mine = (wave < 2 ? red01 : red23) + (wave & 1) * (D * D);
    if (DP == 2) {
        // the two half-waves hold different k parities
#pragma unroll
        for (int a = 0; a < 2; ++a) {
            ck[a] += __shfl_xor(ck[a], 32, 64);
            rv[a] += __shfl_xor(rv[a], 32, 64);
        }
#pragma unroll
        for (int a = 0; a < 4; ++a) pp[a] += __shfl_xor(pp[a], 32, 64);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int i = 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        mine[(DP + i) * D + DP + (lane & 31)] = acc[r];
    }
    if (DP == 2 && lane < 32) {
        mine[(DP + lane) * D + 0] = ck[0];
        mine[(DP + lane) * D + 1] = ck[1];
        mine[0 * D + DP + lane] = rv[0];
        mine[1 * D + DP + lane] = rv[1];
        if (lane == 0) {
            mine[0] = pp[0]; mine[1] = pp[1]; mine[D] = pp[2]; mine[D + 1] = pp[3];
        }
    }
    __syncthreads();
    float* dst = partial + (bh * gridDim.x + chunk) * (int64_t)(D * D);
    for (int e = threadIdx.x; e < D * D; e += 256)
        dst[e] = ((red01[e] + red01[D * D + e]) + red23[e]) + red23[D * D + e];
}

// The backward's second reduction, N[i][j] = sum_t Q[i][t] G[t][j] with Q feature-major [D, S] and G = grad_out
// token-major [S, D]: the structure of ktv_partial_fm, with the Q rows staged through LDS as K is there and the
// G operand read straight from memory (a token's feature row is 128 contiguous bytes: two rows per load
// instruction), one 128-token stage ahead.  grid (nchunk, BH), block 256.
template <int D>
__global__ __launch_bounds__(256) void qg_partial_fm(const float* __restrict__ Q, const float* __restrict__ G,
                                                     float* __restrict__ partial, int S, int tokens_per_chunk) {
    constexpr int DP = D - 32;
    constexpr int RPW = (D + 3) / 4;  // rows per wave in the loader
    // the Q stage [D][kFmPitch]; at the end the four waves' D x D tiles
    __shared__ float sq[D * kFmPitch > 4 * D * D ? D * kFmPitch : 4 * D * D];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t bh = blockIdx.y;
    const int chunk = blockIdx.x;
    const int s0 = chunk * tokens_per_chunk;
    const int s1 = min(S, s0 + tokens_per_chunk);
    const float* Qb = Q + bh * D * (int64_t)S;
    const float* Gb = G + bh * D * (int64_t)S;

    v16f acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    float ck[2] = {0.f, 0.f};   // sum_t Q[DP + lane%32][t] * G[t][a]   -> N[DP+i][a]
    float rv[2] = {0.f, 0.f};   // sum_t Q[a][t] * G[t][DP + lane%32]   -> N[a][DP+j]
    float pp[4] = {0.f, 0.f, 0.f, 0.f};  // sum_t Q[a][t] * G[t][a']

    float2 rq[RPW];
    float gb[16];       // G[t][DP + lane%32] for this lane's 16 tokens of the stage
    float2 gp[16];      // G[t][0], G[t][1] (D == 34)
    auto load_step = [&](int sb) {
        const int s = sb + 2 * lane;
#pragma unroll
        for (int i = 0; i < RPW; ++i) {
            const int row = wave + 4 * i;
            float2 a = make_float2(0.f, 0.f);
            if (row < D) {
                const float* qp = Qb + (int64_t)row * S + s;
                if (s + 1 < s1) {
                    const v2f qa = __builtin_nontemporal_load(reinterpret_cast<const v2f_a4*>(qp));
                    a = make_float2(qa.x, qa.y);
                } else if (s < s1) {
                    a.x = qp[0];
                }
            }
            rq[i] = a;
        }
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            const int t = sb + 32 * wave + 2 * kk + (lane >> 5);
            const float* gr = Gb + (int64_t)min(t, s1 - 1) * D;
            const float v = gr[DP + (lane & 31)];
            gb[kk] = t < s1 ? v : 0.f;
            if (DP == 2) {
                const float2 pz = *reinterpret_cast<const float2*>(gr);
                gp[kk] = t < s1 ? pz : make_float2(0.f, 0.f);
            }
        }
    };
    auto store_step = [&]() {
#pragma unroll
        for (int i = 0; i < RPW; ++i) {
            const int row = wave + 4 * i;
            if (row < D) {
                float* dq = sq + row * kFmPitch + 2 * lane;
                dq[0] = rq[i].x; dq[1] = rq[i].y;
            }
        }
    };

    if (s0 < s1) load_step(s0);
    for (int sb = s0; sb < s1; sb += kFmKT) {
        __syncthreads();  // previous stage fully consumed
        store_step();
        float gcur[16];
        float2 pcur[16];
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            gcur[kk] = gb[kk];
            if (DP == 2) pcur[kk] = gp[kk];
        }
        __syncthreads();
        if (sb + kFmKT < s1) load_step(sb + kFmKT);
        const float* aq = sq + (DP + (lane & 31)) * kFmPitch;
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            const int k = 32 * wave + 2 * kk + (lane >> 5);
            const float a = aq[k];
            const float b = gcur[kk];
            acc = mfma32(a, b, acc);
            if (DP == 2) {
                const float q0 = sq[k], q1 = sq[kFmPitch + k];
                const float g0 = pcur[kk].x, g1 = pcur[kk].y;
                ck[0] = fmaf(a, g0, ck[0]);
                ck[1] = fmaf(a, g1, ck[1]);
                rv[0] = fmaf(q0, b, rv[0]);
                rv[1] = fmaf(q1, b, rv[1]);
                pp[0] = fmaf(q0, g0, pp[0]);
                pp[1] = fmaf(q0, g1, pp[1]);
                pp[2] = fmaf(q1, g0, pp[2]);
                pp[3] = fmaf(q1, g1, pp[3]);
            }
        }
    }
    __syncthreads();
    // Cross-wave sum in wave order through LDS.
    float* tiles = sq;
    float* mine = tiles + wave * (D * D);
    if (DP == 2) {
#pragma unroll
        for (int a = 0; a < 2; ++a) {
            ck[a] += __shfl_xor(ck[a], 32, 64);
            rv[a] += __shfl_xor(rv[a], 32, 64);
        }
#pragma unroll
        for (int a = 0; a < 4; ++a) pp[a] += __shfl_xor(pp[a], 32, 64);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int i = 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        mine[(DP + i) * D + DP + (lane & 31)] = acc[r];
    }
    if (DP == 2 && lane < 32) {
        mine[(DP + lane) * D + 0] = ck[0];
        mine[(DP + lane) * D + 1] = ck[1];
        mine[0 * D + DP + lane] = rv[0];
        mine[1 * D + DP + lane] = rv[1];
        if (lane == 0) {
            mine[0] = pp[0]; mine[1] = pp[1]; mine[D] = pp[2]; mine[D + 1] = pp[3];
        }
    }
    __syncthreads();
    float* dst = partial + (bh * gridDim.x + chunk) * (int64_t)(D * D);
    for (int e = threadIdx.x; e < D * D; e += 256)
        dst[e] = ((tiles[e] + tiles[D * D + e]) + tiles[2 * D * D + e]) + tiles[3 * D * D + e];
}

// grid (nchunk, BH), block 256; every wave owns a contiguous quarter of the chunk.
// Lane l: token slot tk = l%16 (tokens 4*tk .. 4*tk+3 of a 64-token unit), feature
// group g = l/16.  M is row-major [D][D] (already scaled by 1/S).
template <int D>
__global__ __launch_bounds__(256) void qm_apply_fm(const float* __restrict__ Q, const float* __restrict__ M,
                                                   float* __restrict__ out, int S, int tokens_per_chunk) {
    constexpr int DP = D - 32;
    // D == 34: a wave stages the 64 x 34 output rows of a unit in its own LDS slice, laid out as they are in
    // memory, and copies the contiguous 8704-byte run with 16-byte accesses (rows of 136 bytes would otherwise
    // go out in 8-byte pieces); the run starts at a multiple of 8 bytes only (S * 136 bytes per (batch, head)).
    constexpr int kStagePitch = 34;
    __shared__ __attribute__((aligned(16))) float stage_all[DP == 2 ? 4 * 64 * kStagePitch : 4];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    float* stage = stage_all + (DP == 2 ? wave * 64 * kStagePitch : 0);
    const int tk = lane & 15;
    const int g = lane >> 4;
    const int64_t bh = blockIdx.y;
    const int tpw = tokens_per_chunk / 4;
    const int s0 = blockIdx.x * tokens_per_chunk + wave * tpw;
    const int s1 = min(S, s0 + tpw);
    if (s0 >= s1) return;

    const float* m = M + bh * (D * D);
    float mreg[8][2];
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
        const int i = (kk < 4) ? (4 * g + kk) : (16 + 4 * g + kk - 4);
#pragma unroll
        for (int jb = 0; jb < 2; ++jb) mreg[kk][jb] = m[(DP + i) * D + DP + jb * 16 + tk];
    }
    float mrow[2][2][4], mcol[8][2], mpp[2][2];
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

    const float* Qb = Q + bh * D * (int64_t)S;
    float* ob = out + bh * (int64_t)S * D;

    struct Unit { float4 q[8]; float4 p[2]; };
    // Full unit: all 64 tokens inside [s0, s1).
    auto load_full = [&](Unit& u, int sb) {
        const int s = sb + 4 * tk;
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
            const int i = (kk < 4) ? (4 * g + kk) : (16 + 4 * g + kk - 4);
            const f4u v = *reinterpret_cast<const f4u*>(Qb + (int64_t)(DP + i) * S + s);
            u.q[kk] = make_float4(v.x, v.y, v.z, v.w);
        }
        if (DP == 2) {
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                const f4u v = *reinterpret_cast<const f4u*>(Qb + (int64_t)a * S + s);
                u.p[a] = make_float4(v.x, v.y, v.z, v.w);
            }
        }
    };
    auto load_tail = [&](Unit& u, int sb) {
        const int s = sb + 4 * tk;
        auto ld4 = [&](const float* row) {
            float4 v;
            v.x = (s + 0 < s1) ? row[s + 0] : 0.f;
            v.y = (s + 1 < s1) ? row[s + 1] : 0.f;
            v.z = (s + 2 < s1) ? row[s + 2] : 0.f;
            v.w = (s + 3 < s1) ? row[s + 3] : 0.f;
            return v;
        };
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
            const int i = (kk < 4) ? (4 * g + kk) : (16 + 4 * g + kk - 4);
            u.q[kk] = ld4(Qb + (int64_t)(DP + i) * S);
        }
        if (DP == 2) {
            u.p[0] = ld4(Qb);
            u.p[1] = ld4(Qb + S);
        }
    };
    auto compute_unit = [&](const Unit& u, int sb) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            auto comp = [&](const float4& v) { return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w; };
            float q[8];
#pragma unroll
            for (int kk = 0; kk < 8; ++kk) q[kk] = comp(u.q[kk]);
            const float p0 = DP == 2 ? comp(u.p[0]) : 0.f;
            const float p1 = DP == 2 ? comp(u.p[1]) : 0.f;
            v4f acc[2];
#pragma unroll
            for (int jb = 0; jb < 2; ++jb) {
                if (DP == 2) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[jb][r] = fmaf(p1, mrow[1][jb][r], p0 * mrow[0][jb][r]);
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
                float* row = stage + (4 * tk + j) * kStagePitch;
                if (g == 0)
                    *reinterpret_cast<float2*>(row) = make_float2(fmaf(p1, mpp[1][0], fmaf(p0, mpp[0][0], c0)),
                                                                  fmaf(p1, mpp[1][1], fmaf(p0, mpp[0][1], c1)));
#pragma unroll
                for (int jb = 0; jb < 2; ++jb) {
                    float* o = row + DP + jb * 16 + 4 * g;
                    *reinterpret_cast<float2*>(o) = make_float2(acc[jb][0], acc[jb][1]);
                    *reinterpret_cast<float2*>(o + 2) = make_float2(acc[jb][2], acc[jb][3]);
                }
            } else {
                // lanes tk and tk^8 swap halves: each store writes whole 128-byte rows of 8 tokens
                const bool lo = tk < 8;
                float o0[4], o1[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    o0[r] = dpp_move<SPGT_DPP_ROW_ROR8>(acc[0][r]);
                    o1[r] = dpp_move<SPGT_DPP_ROW_ROR8>(acc[1][r]);
                }
                const float4 x = make_float4(lo ? acc[0][0] : o1[0], lo ? acc[0][1] : o1[1], lo ? acc[0][2] : o1[2],
                                             lo ? acc[0][3] : o1[3]);
                const float4 y = make_float4(lo ? o0[0] : acc[1][0], lo ? o0[1] : acc[1][1], lo ? o0[2] : acc[1][2],
                                             lo ? o0[3] : acc[1][3]);
                const int fo = (lo ? 0 : 16) + 4 * g;
                const int sx = sb + 4 * (tk & 7) + j;
                const int sy = sx + 32;
                if (sx < s1) st_stream<true>(reinterpret_cast<float4*>(ob + (int64_t)sx * D + fo), x);
                if (sy < s1) st_stream<true>(reinterpret_cast<float4*>(ob + (int64_t)sy * D + fo), y);
            }
        }
        if (DP == 2) {
            // the wave's own LDS slice: program order is enough, no barrier
            const int ntok = min(64, s1 - sb);
            float* dst = ob + (int64_t)sb * D;
            typedef v4f v4f_a8 __attribute__((aligned(8)));
            const int n4 = ntok * D / 4;  // whole 16-byte pieces of the run
            for (int e = lane; e < n4; e += 64) {
                const v4f v = *reinterpret_cast<const v4f_a8*>(stage + 4 * e);
                __builtin_nontemporal_store(v, reinterpret_cast<v4f_a8*>(dst + 4 * e));
            }
            if ((ntok * D) & 2) {  // an odd number of tokens leaves one 8-byte piece
                if (lane == 0)
                    st_stream<true>(reinterpret_cast<float2*>(dst + 4 * n4),
                                    *reinterpret_cast<const float2*>(stage + 4 * n4));
            }
        }
    };

    // two-buffer software pipeline over the wave's full 64-token units
    const int len = s1 - s0;
    const int nfull = len / 64;
    Unit bufA, bufB;
    if (nfull > 0) {
        load_full(bufA, s0);
        int u = 0;
        for (; u + 2 <= nfull; u += 2) {
            load_full(bufB, s0 + 64 * (u + 1));
            __builtin_amdgcn_sched_barrier(0);
            compute_unit(bufA, s0 + 64 * u);
            __builtin_amdgcn_sched_barrier(0);
            load_full(bufA, s0 + 64 * min(u + 2, nfull - 1));
            __builtin_amdgcn_sched_barrier(0);
            compute_unit(bufB, s0 + 64 * (u + 1));
            __builtin_amdgcn_sched_barrier(0);
        }
        if (u < nfull) compute_unit(bufA, s0 + 64 * u);
    }
    if (nfull * 64 < len) {
        load_tail(bufA, s0 + nfull * 64);
        compute_unit(bufA, s0 + nfull * 64);
    }
}

}  // namespace spgt

namespace spgt {

// K V^T / S of every (batch, head) into m [bh, D, D] row-major: the K/V pass followed by the tile
// reduction, with `partial` holding bh * nchunk * D*D floats.  Shared with the backward operator.
size_t ktv_fm_partial_bytes(int bh, int D, int nchunk) { return (size_t)bh * nchunk * D * D * sizeof(float); }

int launch_ktv_fm(const float* K, const float* V, float* m, float* partial, int bh, int D, int S, int tpc,
                  int nchunk, hipStream_t stream) {
    const dim3 grid1(nchunk, bh), gridr(ceil_div(D * D, 256), bh);
    if (D == 32)
        hipLaunchKernelGGL((ktv_partial_fm<32>), grid1, dim3(256), 0, stream, K, V, partial, S, tpc);
    else
        hipLaunchKernelGGL((ktv_partial_fm<34>), grid1, dim3(256), 0, stream, K, V, partial, S, tpc);
    hipLaunchKernelGGL(tile_reduce, gridr, dim3(1024), 0, stream, partial, m, D * D, nchunk, 1.0f / (float)S);
    return SPGT_OK;
}

// n [bh, D, D] = Q G / S by qg_partial_fm and the fixed-order reduction (the backward's second D x D matrix).
int launch_qg_fm(const float* Q, const float* G, float* n, float* partial, int bh, int D, int S, int tpc, int nchunk,
                 hipStream_t stream) {
    const dim3 grid1(nchunk, bh), gridr(ceil_div(D * D, 256), bh);
    if (D == 32)
        hipLaunchKernelGGL((qg_partial_fm<32>), grid1, dim3(256), 0, stream, Q, G, partial, S, tpc);
    else
        hipLaunchKernelGGL((qg_partial_fm<34>), grid1, dim3(256), 0, stream, Q, G, partial, S, tpc);
    hipLaunchKernelGGL(tile_reduce, gridr, dim3(1024), 0, stream, partial, n, D * D, nchunk, 1.0f / (float)S);
    return SPGT_OK;
}

}  // namespace spgt

using namespace spgt;

namespace {

struct FmPlan {
    int tpc1, nchunk1, tpc2, nchunk2;
};

FmPlan make_fm_plan(int bh, int S) {
    const int target = 3 * device_cu_count();
    FmPlan p;
    const int per1 = std::min(kReduceChains * kReduceMaxPerChain, std::max(1, target / bh));
    p.tpc1 = std::max(kFmKT, ceil_div(ceil_div(S, per1), kFmKT) * kFmKT);
    p.nchunk1 = ceil_div(S, p.tpc1);
    const int per2 = std::max(1, target / bh);
    p.tpc2 = std::max(256, ceil_div(ceil_div(S, per2), 256) * 256);
    p.nchunk2 = ceil_div(S, p.tpc2);
    return p;
}

size_t round256(size_t x) { return (x + 255) & ~(size_t)255; }

}  // namespace

extern "C" size_t spgt_galerkin_attention_cccr_workspace_bytes(int batch, int num_head, int d_posk, int seqlen) {
    if (batch <= 0 || num_head <= 0 || seqlen <= 0 || (d_posk != 32 && d_posk != 34)) return 0;
    const int bh = batch * num_head;
    const FmPlan p = make_fm_plan(bh, seqlen);
    const size_t dd = (size_t)d_posk * d_posk * sizeof(float);
    // [K^T V / S per (batch, head)] followed by the partial tiles
    return round256((size_t)bh * dd) + (size_t)bh * p.nchunk1 * dd;
}

extern "C" int spgt_galerkin_attention_cccr_forward(const float* Q, const float* K, const float* V, float* out,
                                                    void* workspace, size_t workspace_bytes, int batch,
                                                    int num_head, int d_posk, int seqlen, hipStream_t stream) {
    if (!Q || !K || !V || !out) return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_cccr: null pointer argument");
    if (batch <= 0 || num_head <= 0 || seqlen <= 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_cccr: batch, num_head, seqlen must be positive");
    if (d_posk != 32 && d_posk != 34)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_cccr: d_posk must be 32 or 34");
    const int64_t bh64 = (int64_t)batch * num_head;
    if (bh64 > 65535) return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_cccr: batch*num_head exceeds 65535");
    if (!aligned4(Q) || !aligned4(K) || !aligned4(V) || !aligned16(out))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_cccr: inputs must be 4-byte, out 16-byte aligned");
    const size_t need = spgt_galerkin_attention_cccr_workspace_bytes(batch, num_head, d_posk, seqlen);
    if (!workspace || workspace_bytes < need || !aligned16(workspace))
        return fail(SPGT_ERR_WORKSPACE, "galerkin_attention_cccr: workspace missing, misaligned or too small");
    const int bh = (int)bh64;
    const int D = d_posk;
    const FmPlan p = make_fm_plan(bh, seqlen);
    float* mt = static_cast<float*>(workspace);
    float* partial = reinterpret_cast<float*>(static_cast<char*>(workspace) +
                                              round256((size_t)bh * D * D * sizeof(float)));
    const dim3 grid2(p.nchunk2, bh);
    launch_ktv_fm(K, V, mt, partial, bh, D, seqlen, p.tpc1, p.nchunk1, stream);
    if (D == 32)
        hipLaunchKernelGGL((qm_apply_fm<32>), grid2, dim3(256), 0, stream, Q, mt, out, seqlen, p.tpc2);
    else
        hipLaunchKernelGGL((qm_apply_fm<34>), grid2, dim3(256), 0, stream, Q, mt, out, seqlen, p.tpc2);
    return check_launch("galerkin_attention_cccr");
}

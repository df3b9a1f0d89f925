// Backward kernels of the attention operators.
//
// Reference behaviour restated here:
//   multihead_galerkin_attention_cccr_backward      extension/bind/galerkin_attention.cu:126-173
//   datamove::batched_transpose_gather              extension/native/datamove.cu:121-163
//   mh32::lnorm_grad_ccc_cuda (LayerNorm backward)  extension/native/multihead_dim32.cu:148-271, 601-618
//
// With M = K V^T / S and N = Q G / S (both D x D; G = grad_out, token-major [S, D]):
//   dQ[i][s] = sum_j M[i][j] G[s][j]      dK[i][s] = sum_j N[i][j] V[j][s]      dV[j][s] = sum_i N[i][j] K[i][s]
// The two D x D matrices come from the split-K kernels of the forward pass; the
// three products above are `apply_to_fm_v4`: out[n][s] = sum_k W[n][k] X(k, s) with a
// feature-major [D, S] result (stores run along the contiguous sequence axis).
//
// LayerNorm backward differs from the reference in one point on purpose: it
// takes the pre-LayerNorm projection (recomputed by the caller) instead of
// recovering x_hat as (y - beta) / gamma, which breaks when a gamma is zero.
#include "spgt_device.h"
#include "spgt_host.h"
#include "spgt_kernels.h"

namespace spgt {

// out[bh][n][s] = sum_k W[bh][n*wn + k*wk] * X(k, s)
//   X_TM == false: X is feature-major [D, S];  X_TM == true: X is token-major [S, D].
// Lane l of a wave: contraction half kh = l/32; MFMA step kk contracts the two contraction indices kidx(kk, 0) and
// kidx(kk, 1).  Four consecutive tokens per lane: 16-byte accesses along the sequence axis on the
// feature-major side(s), 512-byte runs per row and wave instruction.  A wave takes blocks of 128 tokens; lane
// (tk, kh) holds tokens 4 tk .. 4 tk + 3, four accumulators (one per token of the lane) share the weight operand.
// The chunk's last, partial block goes 32 tokens per wave with word accesses.
// grid (nchunk, BH), block 256.
template <int D, bool X_TM>
__global__ __launch_bounds__(256) void apply_to_fm_v4(const float* __restrict__ W, int wn, int wk,
                                                      const float* __restrict__ X, float* __restrict__ out, int S,
                                                      int tokens_per_chunk) {
    constexpr int NK = D / 2;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int tk = lane & 31;
    const int kh = lane >> 5;
    const int64_t bh = blockIdx.y;
    const int s0 = blockIdx.x * tokens_per_chunk;
    const int s1 = min(S, s0 + tokens_per_chunk);
    const int nblk = (s1 - s0) / 128;  // whole blocks of this chunk
    auto kidx = [&](int kk) { return X_TM ? (NK * kh + kk) : (2 * kk + kh); };

    const float* w = W + bh * (D * D);
    float wreg[NK];
    float wext[NK][2];
#pragma unroll
    for (int kk = 0; kk < NK; ++kk) {
        wreg[kk] = w[tk * wn + kidx(kk) * wk];
        if (D == 34) {
            wext[kk][0] = w[32 * wn + kidx(kk) * wk];
            wext[kk][1] = w[33 * wn + kidx(kk) * wk];
        }
    }
    const float* Xb = X + bh * D * (int64_t)S;
    float* ob = out + bh * D * (int64_t)S;

    // x[kk][e]: contraction index kidx(kk), token 4 tk + e of the block
    auto load_block = [&](float (&x)[NK][4], int blk) {
        const int sb = s0 + 128 * min(blk, nblk - 1) + 4 * tk;
        if (X_TM) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float* row = Xb + (int64_t)(sb + e) * D + NK * kh;
#pragma unroll
                for (int kk = 0; kk < NK; ++kk) x[kk][e] = row[kk];
            }
        } else {
#pragma unroll
            for (int kk = 0; kk < NK; ++kk) {
                const v4f v = *reinterpret_cast<const v4f_a4*>(Xb + (int64_t)(2 * kk + kh) * S + sb);
                x[kk][0] = v.x; x[kk][1] = v.y; x[kk][2] = v.z; x[kk][3] = v.w;
            }
        }
    };
    auto compute_block = [&](const float (&x)[NK][4], int blk) {
        const int sb = s0 + 128 * blk + 4 * tk;
        v16f acc[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[e][r] = 0.f;
#pragma unroll
        for (int kk = 0; kk < NK; ++kk)
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] = mfma32(wreg[kk], x[kk][e], acc[e]);
        float e0[4] = {0.f, 0.f, 0.f, 0.f}, e1[4] = {0.f, 0.f, 0.f, 0.f};
        if (D == 34) {
#pragma unroll
            for (int kk = 0; kk < NK; ++kk)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    e0[e] = fmaf(wext[kk][0], x[kk][e], e0[e]);
                    e1[e] = fmaf(wext[kk][1], x[kk][e], e1[e]);
                }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                e0[e] += __shfl_xor(e0[e], 32, 64);
                e1[e] += __shfl_xor(e1[e], 32, 64);
            }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int n = 8 * (r >> 2) + 4 * kh + (r & 3);
            *reinterpret_cast<v4f_a4*>(ob + (int64_t)n * S + sb) = v4f{acc[0][r], acc[1][r], acc[2][r], acc[3][r]};
        }
        if (D == 34)
            *reinterpret_cast<v4f_a4*>(ob + (int64_t)(32 + kh) * S + sb) =
                kh == 0 ? v4f{e0[0], e0[1], e0[2], e0[3]} : v4f{e1[0], e1[1], e1[2], e1[3]};
    };
    float xa[NK][4], xb[NK][4];
    int blk = wave;
    if (blk < nblk) load_block(xa, blk);
    for (; blk < nblk; blk += 8) {
        load_block(xb, blk + 4);
        __builtin_amdgcn_sched_barrier(0);
        compute_block(xa, blk);
        __builtin_amdgcn_sched_barrier(0);
        load_block(xa, blk + 8);
        __builtin_amdgcn_sched_barrier(0);
        if (blk + 4 < nblk) compute_block(xb, blk + 4);
        __builtin_amdgcn_sched_barrier(0);
    }
    // the chunk's last, partial block (only the last chunk of a sequence has one): 32 tokens per wave, word accesses
    const int st = s0 + 128 * nblk + 32 * wave + tk;
    if (s0 + 128 * nblk + 32 * wave < s1) {
        const int sl = min(st, s1 - 1);
        float x[NK];
        if (X_TM) {
            const float* row = Xb + (int64_t)sl * D + NK * kh;
#pragma unroll
            for (int kk = 0; kk < NK; ++kk) x[kk] = row[kk];
        } else {
#pragma unroll
            for (int kk = 0; kk < NK; ++kk) x[kk] = Xb[(int64_t)(2 * kk + kh) * S + sl];
        }
        v16f acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) acc = mfma32(wreg[kk], x[kk], acc);
        float t0 = 0.f, t1 = 0.f;
        if (D == 34) {
#pragma unroll
            for (int kk = 0; kk < NK; ++kk) {
                t0 = fmaf(wext[kk][0], x[kk], t0);
                t1 = fmaf(wext[kk][1], x[kk], t1);
            }
            t0 += __shfl_xor(t0, 32, 64);
            t1 += __shfl_xor(t1, 32, 64);
        }
        if (st < s1) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int n = 8 * (r >> 2) + 4 * kh + (r & 3);
                ob[(int64_t)n * S + st] = acc[r];
            }
            if (D == 34) ob[(int64_t)(32 + kh) * S + st] = kh == 0 ? t0 : t1;
        }
    }
}

// src [B, H, D, S] rows dp..dp+31 of every head  ->  dst [B, S, H*32]
// grid (ceil(S/64), H, B), block 256.
__global__ __launch_bounds__(256) void heads_fm_to_tm_k(const float* __restrict__ src, float* __restrict__ dst,
                                                        int S, int H, int D, int dp) {
    __shared__ float tile[32 * 65];
    const int tx = threadIdx.x & 63;
    const int ty = threadIdx.x >> 6;
    const int s0 = blockIdx.x * 64;
    const int h = blockIdx.y;
    const int64_t b = blockIdx.z;
    const float* s = src + ((b * H + h) * D + dp) * (int64_t)S;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int j = 4 * i + ty;
        if (s0 + tx < S) tile[j * 65 + tx] = s[(int64_t)j * S + s0 + tx];
    }
    __syncthreads();
    float* d = dst + b * S * (int64_t)(H * 32) + h * 32;
    const int j = threadIdx.x & 31;
    const int t0 = threadIdx.x >> 5;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int t = 8 * i + t0;
        if (s0 + t < S) d[(int64_t)(s0 + t) * (H * 32) + j] = tile[j * 65 + t];
    }
}

// LayerNorm backward per token and head on token-major data.
//   p  : pre-LayerNorm values [B*S, H*32]        dy : gradient of the LayerNorm output, same layout
//   dp : gradient w.r.t. p                        gpart/bpart [nblock, H*32]: per-workgroup sums of
//        dy * x_hat and dy over the workgroup's tokens (reduced afterwards in a fixed order)
// grid (nblock, H/4), block 256: wave = head, lane = (token slot l/16, feature pair l%16).
__global__ __launch_bounds__(256) void layernorm_heads_backward_k(
    const float* __restrict__ p, const float* __restrict__ dy, const float* __restrict__ gamma, float eps,
    float* __restrict__ dp_out, float* __restrict__ gpart, float* __restrict__ bpart, int64_t tokens, int H,
    int tokens_per_block) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int h = blockIdx.y * 4 + wave;
    const int t = lane >> 4;
    const int pr = lane & 15;
    const int f = h * 32 + 2 * pr;
    const int C = H * 32;
    const float g0 = gamma[f], g1 = gamma[f + 1];
    const int64_t t0 = (int64_t)blockIdx.x * tokens_per_block;
    const int64_t t1 = min(tokens, t0 + tokens_per_block);
    float sg0 = 0.f, sg1 = 0.f, sb0 = 0.f, sb1 = 0.f;
    for (int64_t tb = t0; tb < t1; tb += 4) {
        const int64_t tok = tb + t;
        const bool valid = tok < t1;
        const int64_t tl = valid ? tok : t1 - 1;
        const float2 x = *reinterpret_cast<const float2*>(p + tl * C + f);
        float2 d = *reinterpret_cast<const float2*>(dy + tl * C + f);
        if (!valid) d = make_float2(0.f, 0.f);
        const float mean = row16_allsum(x.x + x.y) * (1.0f / 32.0f);
        const float c0 = x.x - mean, c1 = x.y - mean;
        const float rstd = __builtin_amdgcn_rsqf(fmaf(row16_allsum(fmaf(c1, c1, c0 * c0)), 1.0f / 32.0f, eps));
        const float h0 = c0 * rstd, h1 = c1 * rstd;        // x_hat
        const float a0 = d.x * g0, a1 = d.y * g1;          // d x_hat
        const float m1 = row16_allsum(a0 + a1) * (1.0f / 32.0f);
        const float m2 = row16_allsum(fmaf(a1, h1, a0 * h0)) * (1.0f / 32.0f);
        if (valid) {
            float2 o;
            o.x = rstd * (a0 - m1 - h0 * m2);
            o.y = rstd * (a1 - m1 - h1 * m2);
            *reinterpret_cast<float2*>(dp_out + tok * C + f) = o;
        }
        sg0 = fmaf(d.x, h0, sg0);
        sg1 = fmaf(d.y, h1, sg1);
        sb0 += d.x;
        sb1 += d.y;
    }
    // sum the four token slots (lanes l, l^16, l^32, l^48), then one row per workgroup and head
    sg0 = rows4_allsum(sg0); sg1 = rows4_allsum(sg1); sb0 = rows4_allsum(sb0); sb1 = rows4_allsum(sb1);
    if (t == 0) {
        float* gp = gpart + (int64_t)blockIdx.x * C + f;
        float* bp = bpart + (int64_t)blockIdx.x * C + f;
        gp[0] = sg0; gp[1] = sg1; bp[0] = sb0; bp[1] = sb1;
    }
}

// out[c] = sum_blocks part[block][c] in a fixed order: sixteen interleaved chains (block = q, q + 16, ...), each
// summed in increasing block order with eight loads in flight, then combined by a fixed binary tree.  (One thread
// per column walking all blocks took 235 us for the 4096 blocks of 65 536 tokens: one dependent load at a time.)
// grid ceil(C/64), block 1024 = 64 columns x 16 chains.
__global__ __launch_bounds__(1024) void column_sum_k(const float* __restrict__ part, float* __restrict__ out, int C,
                                                     int nblock) {
    __shared__ float sm[16][64];
    const int q = threadIdx.x >> 6;
    const int c = blockIdx.x * 64 + (threadIdx.x & 63);
    float s = 0.f;
    if (c < C) {
        const float* src = part + c;
        for (int b0 = q; b0 < nblock; b0 += 16 * 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int b = b0 + 16 * u;
                v[u] = b < nblock ? src[(int64_t)b * C] : 0.f;
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) s += v[u];
        }
    }
    sm[q][threadIdx.x & 63] = s;
    __syncthreads();
    if (q == 0 && c < C) {
        float t[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) t[i] = sm[i][threadIdx.x & 63];
#pragma unroll
        for (int w = 8; w >= 1; w /= 2)
#pragma unroll
            for (int i = 0; i < w; ++i) t[i] += t[i + w];
        out[c] = t[0];
    }
}

}  // namespace spgt

using namespace spgt;

namespace {

size_t round256(size_t x) { return (x + 255) & ~(size_t)255; }

struct BwdPlan {
    int tpc1, nchunk1, tpc2, nchunk2;
    size_t off_m, off_n, off_partial, bytes;
};

BwdPlan make_bwd_plan(int bh, int D, int S) {
    const int target = 3 * device_cu_count();
    BwdPlan p;
    const int per1 = std::min(kReduceChains * kReduceMaxPerChain, std::max(1, target / bh));
    p.tpc1 = std::max(128, ceil_div(ceil_div(S, per1), 128) * 128);
    p.nchunk1 = ceil_div(S, p.tpc1);
    const int per2 = std::max(1, target / bh);
    p.tpc2 = std::max(128, ceil_div(ceil_div(S, per2), 128) * 128);
    p.nchunk2 = ceil_div(S, p.tpc2);
    const size_t dd = (size_t)D * D * sizeof(float);
    p.off_m = 0;
    p.off_n = round256((size_t)bh * dd);
    p.off_partial = p.off_n + round256((size_t)bh * dd);
    p.bytes = p.off_partial;
    return p;
}

}  // namespace

// defined in attn_fm.hip / splitk_gemm.hip
namespace spgt {
int launch_ktv_fm(const float* K, const float* V, float* m, float* partial, int bh, int D, int S, int tpc, int nchunk,
                  hipStream_t stream);
int launch_qg_fm(const float* Q, const float* G, float* n, float* partial, int bh, int D, int S, int tpc, int nchunk,
                 hipStream_t stream);
size_t ktv_fm_partial_bytes(int bh, int D, int nchunk);
}  // namespace spgt

extern "C" size_t spgt_galerkin_attention_cccr_backward_workspace_bytes(int batch, int num_head, int d_posk,
                                                                        int seqlen) {
    if (batch <= 0 || num_head <= 0 || seqlen <= 0 || (d_posk != 32 && d_posk != 34)) return 0;
    const int bh = batch * num_head;
    const BwdPlan p = make_bwd_plan(bh, d_posk, seqlen);
    const size_t part_m = ktv_fm_partial_bytes(bh, d_posk, p.nchunk1);
    return p.bytes + round256(part_m);  // the two reductions use the partial-tile space one after the other
}

extern "C" int spgt_galerkin_attention_cccr_backward(const float* grad_out, const float* Q, const float* K,
                                                     const float* V, float* grad_Q, float* grad_K, float* grad_V,
                                                     void* workspace, size_t workspace_bytes, int batch,
                                                     int num_head, int d_posk, int seqlen, hipStream_t stream) {
    if (!grad_out || !Q || !K || !V || !grad_Q || !grad_K || !grad_V)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_cccr_backward: null pointer argument");
    if (batch <= 0 || num_head <= 0 || seqlen <= 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_cccr_backward: sizes must be positive");
    if (d_posk != 32 && d_posk != 34)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_cccr_backward: d_posk must be 32 or 34");
    const int64_t bh64 = (int64_t)batch * num_head;
    if (bh64 > 65535)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "galerkin_attention_cccr_backward: batch*num_head exceeds 65535");
    const size_t need = spgt_galerkin_attention_cccr_backward_workspace_bytes(batch, num_head, d_posk, seqlen);
    if (!workspace || workspace_bytes < need || !aligned16(workspace))
        return fail(SPGT_ERR_WORKSPACE, "galerkin_attention_cccr_backward: workspace missing, misaligned or too small");
    const int bh = (int)bh64;
    const int D = d_posk;
    const int S = seqlen;
    const BwdPlan p = make_bwd_plan(bh, D, S);
    char* ws = static_cast<char*>(workspace);
    float* m = reinterpret_cast<float*>(ws + p.off_m);      // M[i][j] = sum_t K[i,t] V[j,t] / S, row-major
    float* n = reinterpret_cast<float*>(ws + p.off_n);      // N[i][j] = sum_t Q[i,t] G[t,j] / S, row-major
    float* partial = reinterpret_cast<float*>(ws + p.off_partial);
    const dim3 grid2(p.nchunk2, bh);

    int rc = launch_ktv_fm(K, V, m, partial, bh, D, S, p.tpc1, p.nchunk1, stream);
    if (rc != SPGT_OK) return rc;
    // dQ = M G^T
    if (D == 32)
        hipLaunchKernelGGL((apply_to_fm_v4<32, true>), grid2, dim3(256), 0, stream, m, D, 1, grad_out, grad_Q, S, p.tpc2);
    else
        hipLaunchKernelGGL((apply_to_fm_v4<34, true>), grid2, dim3(256), 0, stream, m, D, 1, grad_out, grad_Q, S, p.tpc2);
    // N = Q G / S   (A = Q [D, S] row-major, B = G [S, D] row-major, C row-major)
    rc = launch_qg_fm(Q, grad_out, n, partial, bh, D, S, p.tpc1, p.nchunk1, stream);
    if (rc != SPGT_OK) return rc;
    // dK = N V ;  dV = N^T K
    if (D == 32) {
        hipLaunchKernelGGL((apply_to_fm_v4<32, false>), grid2, dim3(256), 0, stream, n, D, 1, V, grad_K, S, p.tpc2);
        hipLaunchKernelGGL((apply_to_fm_v4<32, false>), grid2, dim3(256), 0, stream, n, 1, D, K, grad_V, S, p.tpc2);
    } else {
        hipLaunchKernelGGL((apply_to_fm_v4<34, false>), grid2, dim3(256), 0, stream, n, D, 1, V, grad_K, S, p.tpc2);
        hipLaunchKernelGGL((apply_to_fm_v4<34, false>), grid2, dim3(256), 0, stream, n, 1, D, K, grad_V, S, p.tpc2);
    }
    return check_launch("galerkin_attention_cccr_backward");
}

extern "C" int spgt_heads_feature_to_token_major(const float* src, float* dst, int batch, int num_head,
                                                 int dim_position, int dim_head, int seqlen, hipStream_t stream) {
    if (!src || !dst) return fail(SPGT_ERR_INVALID_ARGUMENT, "heads_feature_to_token_major: null pointer argument");
    if (batch <= 0 || num_head <= 0 || seqlen <= 0 || dim_position < 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "heads_feature_to_token_major: sizes must be positive");
    if (dim_head != 32) return fail(SPGT_ERR_INVALID_ARGUMENT, "heads_feature_to_token_major: dim_head must be 32");
    if (batch > 65535 || num_head > 65535)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "heads_feature_to_token_major: batch or num_head exceeds 65535");
    const dim3 grid(ceil_div(seqlen, 64), num_head, batch);
    hipLaunchKernelGGL(heads_fm_to_tm_k, grid, dim3(256), 0, stream, src, dst, seqlen, num_head,
                       dim_position + dim_head, dim_position);
    return check_launch("heads_feature_to_token_major");
}

extern "C" size_t spgt_layernorm_heads_backward_workspace_bytes(int64_t tokens, int num_head) {
    if (tokens <= 0 || num_head <= 0 || num_head % 4 != 0) return 0;
    const int nblock = (int)std::min<int64_t>(1024, (tokens + 63) / 64);
    return (size_t)2 * nblock * num_head * 32 * sizeof(float);
}

extern "C" int spgt_layernorm_heads_backward(const float* pre_ln, const float* grad_ln, const float* ln_weight,
                                             float norm_eps, float* grad_pre_ln, float* grad_ln_weight,
                                             float* grad_ln_bias, void* workspace, size_t workspace_bytes,
                                             int64_t tokens, int num_head, hipStream_t stream) {
    if (!pre_ln || !grad_ln || !ln_weight || !grad_pre_ln || !grad_ln_weight || !grad_ln_bias)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "layernorm_heads_backward: null pointer argument");
    if (tokens <= 0 || num_head <= 0 || num_head % 4 != 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "layernorm_heads_backward: tokens > 0 and num_head a multiple of 4 required");
    if (!aligned8(pre_ln) || !aligned8(grad_ln) || !aligned8(grad_pre_ln))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "layernorm_heads_backward: operands must be 8-byte aligned");
    const size_t need = spgt_layernorm_heads_backward_workspace_bytes(tokens, num_head);
    if (!workspace || workspace_bytes < need || !aligned16(workspace))
        return fail(SPGT_ERR_WORKSPACE, "layernorm_heads_backward: workspace missing, misaligned or too small");
    const int C = num_head * 32;
    const int nblock = (int)std::min<int64_t>(1024, (tokens + 63) / 64);
    const int tpb = (int)(((tokens + nblock - 1) / nblock + 3) / 4 * 4);
    const int nb = (int)((tokens + tpb - 1) / tpb);
    float* gpart = static_cast<float*>(workspace);
    float* bpart = gpart + (size_t)nblock * C;
    hipLaunchKernelGGL(layernorm_heads_backward_k, dim3(nb, num_head / 4), dim3(256), 0, stream, pre_ln, grad_ln,
                       ln_weight, norm_eps, grad_pre_ln, gpart, bpart, tokens, num_head, tpb);
    hipLaunchKernelGGL(column_sum_k, dim3(ceil_div(C, 64)), dim3(1024), 0, stream, gpart, grad_ln_weight, C, nb);
    hipLaunchKernelGGL(column_sum_k, dim3(ceil_div(C, 64)), dim3(1024), 0, stream, bpart, grad_ln_bias, C, nb);
    return check_launch("layernorm_heads_backward");
}

// Multi-head projection with bias, optional per-head LayerNorm and position
// rows, written feature-major:
//   out[b, h, dp + j, s] = sum_k x[b, s, k] * W[k, h*32 + j] + bias[h*32 + j]
//   out[b, h, 0:dp, s]   = position[b, s, 0:dp]
// and, for the LayerNorm variant, each (b, h, s) column of 32 features is
// normalised (biased variance, eps under the root) and scaled by the head's
// affine before it is stored; invsigma[b, h, s] = 1 / sqrt(var + eps).
//
// Reference behaviour restated here:
//   multihead_projection_with_position_rrc_forward            extension/bind/galerkin_attention.cu:9-24
//   multihead_projection_layernorm_with_position_rrc_forward  extension/bind/galerkin_attention.cu:50-68
//   mh32::sgemm_rrc_cuda and its kernels                      extension/native/multihead_dim32.cu:6-146, 490-599
// The weight is used as stored, x @ W (multihead_dim32.cu:343-344).
//
// One wave owns one head.  Its 32 weight columns W[:, h*32 .. h*32+31] stay in
// registers for the whole kernel as the MFMA A operand (feature x k), token
// tiles of x go through LDS once (coalesced 512-byte rows in, k-strided reads
// out as the B operand), so the 32x32 accumulator holds features along rows
// and 32 consecutive tokens along lanes: stores run along the contiguous
// sequence axis, and a token's 32 features sit in two lanes x 16 registers,
// which makes the LayerNorm statistics an in-register sum plus one lane swap.
#include "spgt_device.h"
#include "spgt_host.h"

namespace spgt {

// Results are collected per wave in LDS for kProjStage tiles (96 tokens of each of the wave's 32 feature rows) and
// leave as 384-byte runs per row, two rows per store instruction: rows of [D, S] start at arbitrary 4-byte offsets
// when S is odd, so every piece of a row touches a partial cache line at either end, and with 128-byte pieces (one
// tile at a time, straight from the accumulators) the kernel wrote 1.43 times its output.  0 = store every tile
// straight from the accumulators.
#ifndef SPGT_PROJ_STAGE
#define SPGT_PROJ_STAGE 3
#endif
constexpr int kProjStage = SPGT_PROJ_STAGE;
constexpr int kProjStagePitch = 32 * (kProjStage > 0 ? kProjStage : 1) + 4;  // floats per staged row (16-byte rows)

// grid (nchunk, H/4, B), block 256; at 128 input features two workgroups share a CU, and one fills its LDS tile
// and drains its staged rows while the other multiplies (one workgroup per CU with two alternating LDS tiles:
// 160-176 us against 130-145 us at B=8, S=44521).  KC = dim_hidden / 128.
// Lane (token tk, half kh) takes k = kh K/2 + j for MFMA j: four consecutive MFMAs' x operands are one 16-byte LDS
// read, and with rows K + 4 words apart those reads and the 16-byte writes of the incoming tile are free of bank
// conflicts.  Two accumulator chains alternate over groups of four k-steps, so that no MFMA waits for the one
// before it.
template <int KC, int DP, bool LN>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(KC == 1 ? 2 : 1))) void projection_rrc_k(
    const float* __restrict__ x, const float* __restrict__ W, const float* __restrict__ bias,
    const float* __restrict__ lnw, const float* __restrict__ lnb, const float* __restrict__ pos,
    float* __restrict__ out, float* __restrict__ invsigma, int S, int H, float eps, int tokens_per_chunk) {
    constexpr int K = 128 * KC;
    constexpr int D = DP + 32;
    constexpr int PITCH = K + 4;
    constexpr int TT = 32;  // tokens per tile
    constexpr int TB = 1;
    extern __shared__ __attribute__((aligned(16))) float xs[];  // [TT][PITCH], then [4 waves][32][kProjStagePitch]
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    constexpr int XS_WORDS = TT * PITCH;
    float* const os = xs + XS_WORDS + wave * (32 * kProjStagePitch);  // this wave's staged rows
    const int h = blockIdx.y * 4 + wave;
    const int b = blockIdx.z;
    const int tk = lane & 31;
    const int kh = lane >> 5;
    const int s_begin = blockIdx.x * tokens_per_chunk;
    const int s_end = min(S, s_begin + tokens_per_chunk);

    // A operand: W[kh K/2 + kk][h*32 + tk]
    float wreg[K / 2];
#pragma unroll
    for (int kk = 0; kk < K / 2; ++kk) wreg[kk] = W[(int64_t)(kh * (K / 2) + kk) * K + h * 32 + tk];
    // accumulator element r holds feature i(r) = 8*(r/4) + 4*kh + r%4
    float breg[16], greg[16], oreg[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int i = 8 * (r >> 2) + 4 * kh + (r & 3);
        breg[r] = bias[h * 32 + i];
        if (LN) {
            greg[r] = lnw[h * 32 + i];
            oreg[r] = lnb[h * 32 + i];
        }
    }

    const float* xb = x + (int64_t)b * S * K;
    float* ob = out + ((int64_t)b * H + h) * D * S;
    constexpr int NLD = TT * K / 4 / 256;  // float4 loads per thread per tile
    float4 stage[NLD];
    auto load_tile = [&](int s0) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int e = threadIdx.x + 256 * i;
            const int row = e / (K / 4);
            const int c4 = e % (K / 4);
            const int s = s0 + row;
            stage[i] = (s < s_end) ? *reinterpret_cast<const float4*>(xb + (int64_t)s * K + 4 * c4)
                                   : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int e = threadIdx.x + 256 * i;
            const int row = e / (K / 4);
            const int c4 = e % (K / 4);
            *reinterpret_cast<float4*>(xs + row * PITCH + 4 * c4) = stage[i];
        }
    };

    if (s_begin < s_end) {
        load_tile(s_begin);
        store_tile();
        if (s_begin + TT < s_end) load_tile(s_begin + TT);
    }
    __syncthreads();
    for (int s0 = s_begin; s0 < s_end; s0 += TT) {
        v16f accs[TB];
        {
            const float* xr = xs + tk * PITCH + kh * (K / 2);
            // operands are read from LDS a batch of four groups (sixteen k-steps) ahead of their MFMAs
            constexpr int NG = K / 8, GB = 4;
            v16f acc0, acc1;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc0[r] = acc1[r] = 0.f;
            float4 xv[2][GB];
#pragma unroll
            for (int g = 0; g < GB; ++g) xv[0][g] = *reinterpret_cast<const float4*>(xr + 4 * g);
#pragma unroll
            for (int g0 = 0; g0 < NG; g0 += GB) {
                if (g0 + GB < NG) {
#pragma unroll
                    for (int g = 0; g < GB; ++g)
                        xv[((g0 / GB) + 1) & 1][g] = *reinterpret_cast<const float4*>(xr + 4 * (g0 + GB + g));
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int g = 0; g < GB; ++g) {
                    const float4 v = xv[(g0 / GB) & 1][g];
                    if (g & 1) {
                        acc1 = mfma32(wreg[4 * (g0 + g) + 0], v.x, acc1);
                        acc1 = mfma32(wreg[4 * (g0 + g) + 1], v.y, acc1);
                        acc1 = mfma32(wreg[4 * (g0 + g) + 2], v.z, acc1);
                        acc1 = mfma32(wreg[4 * (g0 + g) + 3], v.w, acc1);
                    } else {
                        acc0 = mfma32(wreg[4 * (g0 + g) + 0], v.x, acc0);
                        acc0 = mfma32(wreg[4 * (g0 + g) + 1], v.y, acc0);
                        acc0 = mfma32(wreg[4 * (g0 + g) + 2], v.z, acc0);
                        acc0 = mfma32(wreg[4 * (g0 + g) + 3], v.w, acc0);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) accs[0][r] = acc0[r] + acc1[r];
        }
#pragma unroll
        for (int tb = 0; tb < TB; ++tb) {
            const v16f acc = accs[tb];
            const int s = s0 + tb * 32 + tk;
            float y[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) y[r] = acc[r] + breg[r];
            if (LN) {
                float sum = 0.f;
#pragma unroll
                for (int r = 0; r < 16; ++r) sum += y[r];
                sum += __shfl_xor(sum, 32, 64);
                const float mean = sum * (1.0f / 32.0f);
                float ss = 0.f;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    y[r] -= mean;
                    ss = fmaf(y[r], y[r], ss);
                }
                ss += __shfl_xor(ss, 32, 64);
                const float rstd = __builtin_amdgcn_rsqf(fmaf(ss, 1.0f / 32.0f, eps));
#pragma unroll
                for (int r = 0; r < 16; ++r) y[r] = fmaf(y[r] * rstd, greg[r], oreg[r]);
                if (kh == 0 && s < s_end) invsigma[((int64_t)b * H + h) * S + s] = rstd;
            }
            if (kProjStage == 0) {
                if (s < s_end) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int i = 8 * (r >> 2) + 4 * kh + (r & 3);
                        ob[(int64_t)(DP + i) * S + s] = y[r];
                    }
                }
            } else {
                // into the wave's LDS rows; they leave when kProjStage tiles are there or the chunk ends
                const int slot = ((s0 - s_begin) / 32 + tb) % kProjStage;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int i = 8 * (r >> 2) + 4 * kh + (r & 3);
                    os[i * kProjStagePitch + slot * 32 + tk] = y[r];
                }
                const bool last_tile = s0 + (tb + 1) * 32 >= s_end;
                if (slot == kProjStage - 1 || last_tile) {
                    const int w0 = s0 + tb * 32 - slot * 32;      // first token of the staged window
                    const int nvalid = min(s_end - w0, (slot + 1) * 32);
                    // lane (tk, kh): tokens 4 tk .. 4 tk + 3 of row 2 q + kh; 4-byte aligned 16-byte stores
                    const int t4 = 4 * tk;  // lanes past the window (tk >= 8 kProjStage) read its last piece and store nothing
                    const int t4r = min(t4, 32 * kProjStage - 4);
#pragma unroll
                    for (int q = 0; q < 16; ++q) {
                        const int i = 2 * q + kh;
                        const float4 v = *reinterpret_cast<const float4*>(os + i * kProjStagePitch + t4r);
                        float* dst = ob + (int64_t)(DP + i) * S + w0 + t4;
                        if (t4 + 3 < nvalid) {
                            *reinterpret_cast<v4f_a4*>(dst) = v4f{v.x, v.y, v.z, v.w};
                        } else if (t4 < nvalid) {
                            dst[0] = v.x;
                            if (t4 + 1 < nvalid) dst[1] = v.y;
                            if (t4 + 2 < nvalid) dst[2] = v.z;
                        }
                    }
                }
            }
            if (s < s_end) {
                if (DP == 2) ob[(int64_t)kh * S + s] = pos[((int64_t)b * S + s) * 2 + kh];
            }
        }
        __syncthreads();  // the tile has been read by every wave
        if (s0 + TT < s_end) {
            store_tile();
            if (s0 + 2 * TT < s_end) load_tile(s0 + 2 * TT);
        }
        __syncthreads();
    }
}

namespace {

template <int KC, int DP, bool LN>
void launch_projection(const float* x, const float* W, const float* bias, const float* lnw, const float* lnb,
                       const float* pos, float* out, float* invsigma, int B, int S, int H, float eps,
                       hipStream_t stream) {
    constexpr int K = 128 * KC;
    constexpr int TT = 32;
    const size_t lds = ((size_t)TT * (K + 4) + (kProjStage > 0 ? 4 * 32 * kProjStagePitch : 0)) * sizeof(float);
    // about two workgroups per CU; chunks are whole tiles
    const int per_b = std::max(1, 2 * device_cu_count() / std::max(1, B * (H / 4)));
    const int tpc = std::max(TT, ceil_div(ceil_div(S, per_b), TT) * TT);
    const dim3 grid(ceil_div(S, tpc), H / 4, B);
    auto kernel = projection_rrc_k<KC, DP, LN>;
    (void)allow_dynamic_lds(kernel, lds);
    hipLaunchKernelGGL(kernel, grid, dim3(256), lds, stream, x, W, bias, lnw, lnb, pos, out, invsigma, S, H, eps, tpc);
}

int projection_common(const char* who, const float* input, const float* weight, const float* bias,
                      const float* ln_weight, const float* ln_bias, float norm_eps, const float* position, float* out,
                      float* invsigma, int batch, int seqlen, int dim_hidden, int num_head, int dim_head,
                      int dim_position, bool ln, hipStream_t stream) {
    if (!input || !weight || !bias || !out || (ln && (!ln_weight || !ln_bias || !invsigma)))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "multihead_projection: null pointer argument");
    if (batch <= 0 || seqlen <= 0) return fail(SPGT_ERR_INVALID_ARGUMENT, "multihead_projection: batch and seqlen must be positive");
    if (dim_head != 32 || num_head * dim_head != dim_hidden)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "multihead_projection: dim_head must be 32 and num_head*32 == dim_hidden");
    if (dim_hidden != 128 && dim_hidden != 256 && dim_hidden != 384 && dim_hidden != 512)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "multihead_projection: dim_hidden must be 128, 256, 384 or 512");
    if (dim_position != 0 && dim_position != 2)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "multihead_projection: dim_position must be 0 or 2");
    if (dim_position == 2 && !position)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "multihead_projection: position is null with dim_position 2");
    if (batch > 65535) return fail(SPGT_ERR_INVALID_ARGUMENT, "multihead_projection: batch exceeds 65535");
    if (!aligned16(input) || !aligned4(weight) || !aligned4(bias) || !aligned4(out))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "multihead_projection: input must be 16-byte aligned");
    const float* pos = position ? position : input;
    const int kc = dim_hidden / 128;
#define SPGT_PROJ(KC, DP, LNF)                                                                                   \
    launch_projection<KC, DP, LNF>(input, weight, bias, ln_weight, ln_bias, pos, out, invsigma, batch, seqlen, \
                                   num_head, norm_eps, stream)
    if (kc == 1) {
        if (ln) { if (dim_position) SPGT_PROJ(1, 2, true); else SPGT_PROJ(1, 0, true); }
        else    { if (dim_position) SPGT_PROJ(1, 2, false); else SPGT_PROJ(1, 0, false); }
    } else if (kc == 2) {
        if (ln) { if (dim_position) SPGT_PROJ(2, 2, true); else SPGT_PROJ(2, 0, true); }
        else    { if (dim_position) SPGT_PROJ(2, 2, false); else SPGT_PROJ(2, 0, false); }
    } else if (kc == 3) {
        if (ln) { if (dim_position) SPGT_PROJ(3, 2, true); else SPGT_PROJ(3, 0, true); }
        else    { if (dim_position) SPGT_PROJ(3, 2, false); else SPGT_PROJ(3, 0, false); }
    } else {
        if (ln) { if (dim_position) SPGT_PROJ(4, 2, true); else SPGT_PROJ(4, 0, true); }
        else    { if (dim_position) SPGT_PROJ(4, 2, false); else SPGT_PROJ(4, 0, false); }
    }
#undef SPGT_PROJ
    return check_launch(who);
}

}  // namespace

}  // namespace spgt

using namespace spgt;

extern "C" int spgt_multihead_projection_with_position_rrc_forward(
    const float* input, const float* weight, const float* bias, const float* position, float* out, int seqlen,
    int dim_hidden, int num_head, int dim_head, int dim_position, int batch, hipStream_t stream) {
    return projection_common("multihead_projection_with_position_rrc_forward", input, weight, bias, nullptr, nullptr,
                             0.f, position, out, nullptr, batch, seqlen, dim_hidden, num_head, dim_head, dim_position,
                             false, stream);
}

extern "C" int spgt_multihead_projection_layernorm_with_position_rrc_forward(
    const float* input, const float* weight, const float* bias, const float* ln_weight, const float* ln_bias,
    float norm_eps, const float* position, float* out, float* invsigma, int seqlen, int dim_hidden, int num_head,
    int dim_head, int dim_position, int batch, hipStream_t stream) {
    return projection_common("multihead_projection_layernorm_with_position_rrc_forward", input, weight, bias,
                             ln_weight, ln_bias, norm_eps, position, out, invsigma, batch, seqlen, dim_hidden, num_head,
                             dim_head, dim_position, true, stream);
}

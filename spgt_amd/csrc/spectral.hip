// FNO2d spectral-mode complex channel contraction, fused with the gather of the
// two retained corner windows and the scatter into a zero-filled output
// spectrum, and bilinear (align_corners) resampling.
//
// Reference behaviour restated here:
//   Sp_SpectralConv2D.forward, the part between rfft2 and irfft2
//       network/sp_layer.py:139-148 (gather_dual, two complex matmuls, scatter_dual)
//   SpectralConv2D.complex_matmul_2D      network/layer.py:249-261
//   F.interpolate(mode='bilinear', align_corners=True) in DownScaler2D / UpScaler2D
//       network/model.py:30, 36, 59, 63
#include "spgt_device.h"
#include "spgt_host.h"
#include "spgt_kernels.h"

// complex elements a zero-fill block writes, roughly (tuned on MI355X)
#ifndef SPGT_ROWS_NB
#define SPGT_ROWS_NB 4
#endif
#ifndef SPGT_ROWS_WU
#define SPGT_ROWS_WU 8
#endif
#ifndef SPGT_ZERO_CHUNK
#define SPGT_ZERO_CHUNK 2048
#endif

namespace spgt {

struct SpecWindows {
    int h_base[2];
    int w_base[2];
};

// Element strides (in complex elements) of the spectrum operands: element (n, c, h, w) of X sits at
// n*x_n + c*x_c + h*x_h + w*x_w, likewise for the output.  `compact` operands hold only the two
// windows, stacked along h: row index k*m_h + hh instead of h_base[k] + hh, column ww.
struct SpecLayout {
    int64_t x_n, x_c, x_h, x_w;
    int64_t o_n, o_c, o_h, o_w;
    int compact;
};

// out[n, o, hb_k + hh, wb_k + ww] = sum_i X[n, i, hb_k + hh, wb_k + ww] * W_k[hh, ww, i, o]   (complex)
// grid (m_h * m_w, 2, ceil(Cout/64)), block 256 = 64 output channels x 4 batch groups.
// One workgroup per mode: the mode's input column X[:, :, h, w] is staged in LDS
// (NB batch entries at a time), the mode's weight block [Cin, 64] is streamed
// once per batch group with 512-byte coalesced rows.
constexpr int kSpecNB = 16;
constexpr int kSpecWB = 32;  // weight rows per load batch

__global__ __launch_bounds__(256) void spectral_mode_contract_k(
    const float2* __restrict__ X, const float2* __restrict__ W0, const float2* __restrict__ W1,
    float2* __restrict__ out, int N, int Cin, int Cout, int m_h, int m_w, SpecWindows win, SpecLayout lay) {
    extern __shared__ float2 xs[];  // [kSpecNB][Cin]
    const int mode = blockIdx.x;
    const int k = blockIdx.y;
    const int hh = mode / m_w;
    const int ww = mode % m_w;
    const int h = win.h_base[k] + hh;
    const int w = win.w_base[k] + ww;
    // Where the windows overlap the second one wins (the reference assigns it last).
    if (!lay.compact && k == 0 && h >= win.h_base[1] && h < win.h_base[1] + m_h && w >= win.w_base[1] &&
        w < win.w_base[1] + m_w)
        return;
    const int o = blockIdx.z * 64 + (threadIdx.x & 63);
    const int ng = threadIdx.x >> 6;
    const float2* Wm = (k == 0 ? W0 : W1) + (int64_t)mode * Cin * Cout;
    const int he = lay.compact ? k * m_h + hh : h;
    const int we = lay.compact ? ww : w;
    const int64_t xpix = he * lay.x_h + we * lay.x_w;
    const int64_t opix = he * lay.o_h + we * lay.o_w;

    for (int n0 = 0; n0 < N; n0 += kSpecNB) {
        const int nb = min(kSpecNB, N - n0);
        __syncthreads();
        for (int e = threadIdx.x; e < nb * Cin; e += 256) {
            const int n = e / Cin;
            const int i = e - n * Cin;
            xs[e] = X[(n0 + n) * lay.x_n + i * lay.x_c + xpix];
        }
        __syncthreads();
        float2 acc[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = make_float2(0.f, 0.f);
        if (o < Cout) {
            // the weight rows are fetched kSpecWB at a time, all loads of a batch in flight together:
            // the kernel's time is a few memory round trips, not one per input channel
            for (int i0 = 0; i0 < Cin; i0 += kSpecWB) {
                float2 wv[kSpecWB];
#pragma unroll
                for (int u = 0; u < kSpecWB; ++u)
                    wv[u] = (i0 + u < Cin) ? Wm[(int64_t)(i0 + u) * Cout + o] : make_float2(0.f, 0.f);
#pragma unroll
                for (int u = 0; u < kSpecWB; ++u) {
                    const int i = min(i0 + u, Cin - 1);  // rows past Cin carry zero weights
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int n = ng + 4 * j;
                        if (n < nb) {
                            const float2 xv = xs[n * Cin + i];
                            acc[j].x = fmaf(xv.x, wv[u].x, acc[j].x);
                            acc[j].x = fmaf(-xv.y, wv[u].y, acc[j].x);
                            acc[j].y = fmaf(xv.y, wv[u].x, acc[j].y);
                            acc[j].y = fmaf(xv.x, wv[u].y, acc[j].y);
                        }
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n = ng + 4 * j;
                if (n < nb) out[(n0 + n) * lay.o_n + o * lay.o_c + opix] = acc[j];
            }
        }
    }
}

// Zeros every element of out [planes, H_all, W_all] (complex) outside the two windows.
__global__ __launch_bounds__(256) void spectrum_zero_outside_k(float2* __restrict__ out, int64_t total, int H_all,
                                                               int W_all, int m_h, int m_w, SpecWindows win) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += stride) {
        const int w = (int)(e % W_all);
        const int h = (int)((e / W_all) % H_all);
        const bool in0 = h >= win.h_base[0] && h < win.h_base[0] + m_h && w >= win.w_base[0] && w < win.w_base[0] + m_w;
        const bool in1 = h >= win.h_base[1] && h < win.h_base[1] + m_h && w >= win.w_base[1] && w < win.w_base[1] + m_w;
        if (!in0 && !in1) out[e] = make_float2(0.f, 0.f);
    }
}

// The full-spectrum form in ONE launch: contraction, scatter into the output spectrum and zero fill.
// Blocks [0, nA) each own JW window columns of one output row h that lies in a window, for NB batch entries and
// 64 output planes.  Thread (o, q) multiplies the input channels i = q, q+4, ...: its weights for a step of 32
// channels are loaded once (JW * 8 loads in flight, 512-byte coalesced rows) and meet the rows of all NB batch
// entries, which wait in LDS; the four partial sums per output are added in LDS in a fixed order.  Blocks
// [nA, ...) zero everything else: the rows that lie in no window as contiguous spans of a plane with 16-byte
// stores, and the window rows' columns outside the windows.  Where the windows overlap the second one wins
// (the reference scatters it last).
constexpr int kRowsNB = SPGT_ROWS_NB;
constexpr int kRowsWU = SPGT_ROWS_WU;  // input channels per thread and step (all blocks of the launch share its register budget)

template <int JW>
__global__ __launch_bounds__(256) void spectral_contract_rows_k(
    const float2* __restrict__ X, const float2* __restrict__ W0, const float2* __restrict__ W1,
    float2* __restrict__ out, int N, int Cin, int Cout, int H_all, int W_all, int m_h, int m_w, SpecWindows win,
    SpecSpans spans, int nA, int chunks_per_plane) {
    extern __shared__ float2 xrow[];  // [kRowsNB][Cin][JW] inputs, then [4 entries][4][JW][64] partial sums
    const int64_t plane = (int64_t)H_all * W_all;
    if ((int)blockIdx.x >= nA) {
        // chunks_per_plane blocks per plane for the rows outside the windows, one more for the window rows' rest
        const int bz = blockIdx.x - nA;
        const int64_t p = bz / (chunks_per_plane + 1);
        const int c = bz - (int)p * (chunks_per_plane + 1);
        if (c < chunks_per_plane)
            zero_span_chunk(out, spans, p, c, chunks_per_plane, plane, W_all);
        else
            zero_window_row_remainders(out, p, plane, W_all, m_h, m_w, win.h_base[0], win.w_base[0], win.h_base[1],
                                       win.w_base[1]);
        return;
    }
    const int og_count = ceil_div(Cout, 64);
    const int wq_count = ceil_div(m_w, JW);
    int a = blockIdx.x;
    const int wq = a % wq_count;
    a /= wq_count;
    const int og = a % og_count;
    a /= og_count;
    const int slot = a % (2 * m_h);
    const int n0 = (a / (2 * m_h)) * kRowsNB;
    const int nb = min(kRowsNB, N - n0);
    const int k0 = slot / m_h;
    const int h = win.h_base[k0] + (slot - k0 * m_h);
    const bool in0 = h >= win.h_base[0] && h < win.h_base[0] + m_h;
    const bool in1 = h >= win.h_base[1] && h < win.h_base[1] + m_h;
    if (k0 == 1 && in0) return;  // the first window's block owns a row that lies in both
    const bool ink[2] = {in0, in1};
    const int ww0 = wq * JW;
    const int ol = threadIdx.x & 63;
    const int o = og * 64 + ol;
    const int q = threadIdx.x >> 6;
    const int oc = min(o, Cout - 1);
    float2* red = xrow + kRowsNB * Cin * JW;  // [4][4][JW][64]
    for (int k = 0; k < 2; ++k) {
        if (!ink[k]) continue;
        const int hh = h - win.h_base[k];
        const float2* Wk = (k == 0 ? W0 : W1) + ((int64_t)hh * m_w) * Cin * Cout + oc;
        float2 wv[JW][kRowsWU];
        auto load_weights = [&](int i0) {  // channels i0, i0+4, ..., clamped (their products are skipped)
#pragma unroll
            for (int j = 0; j < JW; ++j) {
                const int ww = min(ww0 + j, m_w - 1);
#pragma unroll
                for (int u = 0; u < kRowsWU; ++u)
                    wv[j][u] = Wk[((int64_t)ww * Cin + min(i0 + 4 * u, Cin - 1)) * Cout];
            }
        };
        load_weights(q);  // in flight while the rows travel to LDS
        __syncthreads();
        {
            // eight loads per thread in flight at a time (a plain loop would wait for each before the next)
            const int total = nb * Cin * JW;
            const float2* xbase = X + (int64_t)n0 * Cin * plane + (int64_t)h * W_all + win.w_base[k];
            for (int base = 0; base < total; base += 256 * 8) {
                float2 tmp[8];
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const int e = min(base + (int)threadIdx.x + 256 * t, total - 1);
                    const int ni = e / JW;  // (entry, channel): planes of X are in this order
                    tmp[t] = xbase[ni * plane + min(ww0 + (e - ni * JW), m_w - 1)];
                }
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const int e = base + (int)threadIdx.x + 256 * t;
                    if (e < total) xrow[e] = tmp[t];
                }
            }
        }
        __syncthreads();
        float2 acc[kRowsNB][JW];
#pragma unroll
        for (int nn = 0; nn < kRowsNB; ++nn)
#pragma unroll
            for (int j = 0; j < JW; ++j) acc[nn][j] = make_float2(0.f, 0.f);
        for (int i0 = q; i0 < Cin; i0 += 4 * kRowsWU) {  // this thread's channels i0, i0+4, ..., kRowsWU per step
            if (i0 != q) load_weights(i0);
#pragma unroll
            for (int u = 0; u < kRowsWU; ++u) {
                if (i0 + 4 * u < Cin) {
#pragma unroll
                    for (int nn = 0; nn < kRowsNB; ++nn) {
                        if (nn < nb) {
#pragma unroll
                            for (int j = 0; j < JW; ++j) {
                                const float2 xv = xrow[(nn * Cin + i0 + 4 * u) * JW + j];
                                acc[nn][j].x = fmaf(xv.x, wv[j][u].x, acc[nn][j].x);
                                acc[nn][j].x = fmaf(-xv.y, wv[j][u].y, acc[nn][j].x);
                                acc[nn][j].y = fmaf(xv.y, wv[j][u].x, acc[nn][j].y);
                                acc[nn][j].y = fmaf(xv.x, wv[j][u].y, acc[nn][j].y);
                            }
                        }
                    }
                }
            }
        }
        // four batch entries at a time: partial sums to LDS, thread (o, q) finishes entry q
#pragma unroll
        for (int g = 0; g < kRowsNB; g += 4) {
            if (g >= nb) break;
            __syncthreads();
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4)
#pragma unroll
                for (int j = 0; j < JW; ++j) red[((e4 * 4 + q) * JW + j) * 64 + ol] = acc[g + e4][j];
            __syncthreads();
            const int nn = g + q;
            if (nn < nb && o < Cout) {
                float2* orow = out + ((int64_t)(n0 + nn) * Cout + o) * plane + (int64_t)h * W_all;
#pragma unroll
                for (int j = 0; j < JW; ++j) {
                    const int ww = ww0 + j;
                    const int w = win.w_base[k] + ww;
                    const bool hidden = k == 0 && in1 && w >= win.w_base[1] && w < win.w_base[1] + m_w;
                    if (ww >= m_w || hidden) continue;
                    float2 sum = red[((q * 4 + 0) * JW + j) * 64 + ol];
#pragma unroll
                    for (int qq = 1; qq < 4; ++qq) {
                        const float2 t = red[((q * 4 + qq) * JW + j) * 64 + ol];
                        sum.x += t.x;
                        sum.y += t.y;
                    }
                    orow[w] = sum;
                }
            }
        }
    }
}

// Activations that the resampling kernels can apply to the source samples (`pre_n` times) and to
// the result, standing in for the separate elementwise kernels of ConvResBlock2D and the scalers.
struct ResampleAct {
    int pre, pre_n, post;
};

// Dropout of the source samples (ConvResBlock2D's conv -> dropout -> activation, network/layer.py:7-24, always on
// in the reference): seed = two words in device memory, null for none; see dropout_site in spgt_device.h.
struct DropArgs {
    const uint32_t* seed;
    float p;
};

// act applied `count` times to every element of v, with the choice of activation made once for all of them: the
// element-wise form puts a branch tree between the loads of successive samples, which then go out a few at a time.
template <int N>
__device__ __forceinline__ void act_many(float (&v)[N], int act, int count) {
    if (act == SPGT_ACT_SILU) {
        for (int r = 0; r < count; ++r) {
#pragma unroll
            for (int j = 0; j < N; ++j) v[j] = v[j] * __builtin_amdgcn_rcpf(1.f + __expf(-v[j]));
        }
    } else if (act == SPGT_ACT_RELU && count > 0) {
#pragma unroll
        for (int j = 0; j < N; ++j) v[j] = fmaxf(v[j], 0.f);
    }
}

// NV output values from their 4 * NV source samples: t[4j .. 4j+3] = (top left, top right, bottom left, bottom
// right) of value j, bias[j] its channel's bias.  Same arithmetic as torch's upsample_bilinear2d: columns are
// blended first, rows last.
template <bool PRE, int NV>
__device__ __forceinline__ void blend_many(float (&t)[4 * NV], const float (&bias)[NV], float w0l, float w1l,
                                           float h0l, float h1l, ResampleAct act, float (&v)[NV]) {
    if (PRE) {
#pragma unroll
        for (int j = 0; j < 4 * NV; ++j) t[j] += bias[j >> 2];
        act_many<4 * NV>(t, act.pre, act.pre_n);
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const float top = w0l * t[4 * j] + w1l * t[4 * j + 1];
        const float bot = w0l * t[4 * j + 2] + w1l * t[4 * j + 3];
        v[j] = h0l * top + h1l * bot;
    }
    act_many<NV>(v, act.post, 1);
}

// Source row, its lower neighbour and the two row weights of output row oy (align_corners=True:
// scale = (in-1)/(out-1) in fp32, 0 when out == 1; source coordinate scale*dst, weights (1-l, l)).
struct ResampleTap {
    int i1, ip;  // first source index and the step (0 or 1) to the second
    float l0, l1;
};
__device__ __forceinline__ ResampleTap resample_tap(float scale, int o, int in_size) {
    const float r = scale * (float)o;
    ResampleTap t;
    t.i1 = (int)r;
    t.ip = (t.i1 < in_size - 1) ? 1 : 0;
    t.l1 = r - (float)t.i1;
    t.l0 = 1.0f - t.l1;
    return t;
}

// Logical tile of a one-dimensional launch whose size is a multiple of 8.  Workgroups go round-robin to the 8
// XCDs, each with its own L2; consecutive logical tiles are mapped onto one XCD, so that tiles which share
// source rows, or halves of an output cache line, meet in one L2.
__device__ __forceinline__ int xcd_contiguous_tile() {
    const int per_xcd = gridDim.x >> 3;
    return (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
}

// Bilinear resampling with align_corners=True of [planes, Hin, Win] -> [planes, Hout, Wout].
// Tiles of 64 x 4 output positions x (4 planes at a time, every zb-th group of 4); a thread makes one output
// position of 4 consecutive planes at a time, 16 source samples in flight.  One-dimensional launch of xt * yt * zb
// tiles rounded up to a multiple of 8, block (64, 4); the tiles of a plane group are consecutive logical tiles, so
// the source rows that neighbouring tiles share are fetched into one XCD's L2 (a three-dimensional grid spread
// them over the XCDs: 1.3 to 3 times the source bytes came from memory).
template <bool PRE>
__global__ __launch_bounds__(256) void bilinear_align_corners_k(const float* __restrict__ src,
                                                                const float* __restrict__ pre_bias, int C,
                                                                float* __restrict__ dst, int planes, int Hin,
                                                                int Win, int Hout, int Wout, float hscale,
                                                                float wscale, ResampleAct act, int xt, int yt,
                                                                int zb) {
    const int logical = xcd_contiguous_tile();
    if (logical >= xt * yt * zb) return;
    const int ox = (logical % xt) * 64 + threadIdx.x;
    const int oy = ((logical / xt) % yt) * 4 + threadIdx.y;
    const int bz = logical / (xt * yt);
    if (ox >= Wout || oy >= Hout) return;
    const ResampleTap th = resample_tap(hscale, oy, Hin), tw = resample_tap(wscale, ox, Win);
    const float* base = src + (int64_t)th.i1 * Win + tw.i1;
    for (int64_t p0 = (int64_t)bz * 4; p0 < planes; p0 += (int64_t)zb * 4) {
        float t[16], pb[4], v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t pl = min(p0 + j, (int64_t)planes - 1);  // planes past the end repeat the last, unwritten
            const float* r0 = base + pl * Hin * Win;
            const float* r1 = r0 + (int64_t)th.ip * Win;
            t[4 * j] = r0[0], t[4 * j + 1] = r0[tw.ip], t[4 * j + 2] = r1[0], t[4 * j + 3] = r1[tw.ip];
            pb[j] = (PRE && pre_bias) ? pre_bias[pl % C] : 0.f;
        }
        blend_many<PRE, 4>(t, pb, tw.l0, tw.l1, th.l0, th.l1, act, v);
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (p0 + j < planes) dst[((p0 + j) * Hout + oy) * Wout + ox] = v[j];
    }
}

// The same resampling with a channels-last result: src [N, C, Hin, Win] -> dst [N, Hout, Wout, C].
// grid (ceil(Wout/32), Hout, N), block 256 = 32 output columns x 8 channel lanes.  Reads run along the
// source rows of one channel, a 32 x 32 (channel x column) tile is turned in LDS, writes run along C.
template <bool PRE>
__global__ __launch_bounds__(256) void bilinear_align_corners_nhwc_k(const float* __restrict__ src,
                                                                     const float* __restrict__ pre_bias,
                                                                     float* __restrict__ dst, int C, int Hin,
                                                                     int Win, int Hout, int Wout, float hscale,
                                                                     float wscale, ResampleAct act) {
    __shared__ float tile[32 * 33];
    const int tx = threadIdx.x & 31;
    const int ty = threadIdx.x >> 5;
    const int oy = blockIdx.y;
    const int64_t n = blockIdx.z;
    const ResampleTap th = resample_tap(hscale, oy, Hin);
    const ResampleTap tw = resample_tap(wscale, min((int)blockIdx.x * 32 + tx, Wout - 1), Win);
    const int64_t plane = (int64_t)Hin * Win;
    const float* base = src + n * C * plane + (int64_t)th.i1 * Win + tw.i1;
    float* drow = dst + ((n * Hout + oy) * (int64_t)Wout) * C;
    for (int c0 = 0; c0 < C; c0 += 32) {
        float t[16], pb[4], v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = min(c0 + 8 * i + ty, C - 1);  // channels past the end repeat the last one and are not written
            const float* r0 = base + (int64_t)c * plane;
            const float* r1 = r0 + (int64_t)th.ip * Win;
            t[4 * i] = r0[0], t[4 * i + 1] = r0[tw.ip], t[4 * i + 2] = r1[0], t[4 * i + 3] = r1[tw.ip];
            pb[i] = (PRE && pre_bias) ? pre_bias[c] : 0.f;
        }
        blend_many<PRE, 4>(t, pb, tw.l0, tw.l1, th.l0, th.l1, act, v);
#pragma unroll
        for (int i = 0; i < 4; ++i) tile[(8 * i + ty) * 33 + tx] = v[i];
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int xl = 8 * i + ty;
            const int x = blockIdx.x * 32 + xl;
            if (x < Wout && c0 + tx < C) drow[(int64_t)x * C + c0 + tx] = tile[tx * 33 + xl];
        }
        __syncthreads();
    }
}

// The same resampling from a channels-last source: src [N, Hin, Win, C] -> dst [N, C, Hout, Wout].
// grid (ceil(Wout/32), Hout, N), block 256 = 32 channels x 8 column lanes.  Reads run along C (the
// four source pixels of an output column are 128-byte runs), a 32 x 32 (column x channel) tile is
// turned in LDS, writes run along the output row of one channel.
template <bool PRE>
__global__ __launch_bounds__(256) void bilinear_align_corners_from_nhwc_k(const float* __restrict__ src,
                                                                          const float* __restrict__ pre_bias,
                                                                          float* __restrict__ dst, int C, int Hin,
                                                                          int Win, int Hout, int Wout, float hscale,
                                                                          float wscale, ResampleAct act) {
    __shared__ float tile[32 * 33];
    const int tx = threadIdx.x & 31;
    const int ty = threadIdx.x >> 5;
    const int oy = blockIdx.y;
    const int64_t n = blockIdx.z;
    const ResampleTap th = resample_tap(hscale, oy, Hin);
    const float* rows = src + (n * Hin + th.i1) * (int64_t)Win * C;
    const int64_t rstep = (int64_t)th.ip * Win * C;
    for (int c0 = 0; c0 < C; c0 += 32) {
        const int c = min(c0 + tx, C - 1);  // channels past the end repeat the last one and are not written
        const float pb1 = (PRE && pre_bias) ? pre_bias[c] : 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int xl = 8 * i + ty;
            const ResampleTap tw = resample_tap(wscale, min((int)blockIdx.x * 32 + xl, Wout - 1), Win);
            const float* p0 = rows + (int64_t)tw.i1 * C + c;
            const float* p1 = p0 + rstep;
            float t[4] = {p0[0], p0[tw.ip * C], p1[0], p1[tw.ip * C]};
            const float pb[1] = {pb1};
            float v[1];
            blend_many<PRE, 1>(t, pb, tw.l0, tw.l1, th.l0, th.l1, act, v);
            tile[xl * 33 + tx] = v[0];
        }
        __syncthreads();
        const int ox = blockIdx.x * 32 + tx;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int cl = 8 * i + ty;
            if (ox < Wout && c0 + cl < C)
                dst[((n * C + c0 + cl) * Hout + oy) * (int64_t)Wout + ox] = tile[tx * 33 + cl];
        }
        __syncthreads();
    }
}

// NCHW -> channels-last for C a multiple of 4 with a 16-byte aligned result: one workgroup makes 32 output
// columns x 128 channels of one output row.  A thread blends 4 consecutive channels of one column and puts them
// into LDS as one 16-byte piece; the workgroup then writes the tile as whole pixels, 1 KB contiguous per wave.
// grid: tiles = N * Hout * ceil(Wout/32), rounded up to a multiple of 8; block 256.
// SAME: input and output sizes are equal, every output is its own source sample (weights 1 and 0), and the kernel
// is bias + activation + permute with one load per value.
template <bool PRE, bool SAME>
__global__ __launch_bounds__(256) void bilinear_to_nhwc_wide_k(const float* __restrict__ src,
                                                               const float* __restrict__ pre_bias,
                                                               float* __restrict__ dst, int C, int Hin, int Win,
                                                               int Hout, int Wout, float hscale, float wscale,
                                                               ResampleAct act, int xtiles, int tiles) {
    __shared__ float4 tile[32 * 33];  // [column][channel quad], 33 quads apart: 8 lanes' pieces fall in 8 bank groups
    const int logical = xcd_contiguous_tile();
    if (logical >= tiles) return;
    const int x0 = (logical % xtiles) * 32;
    const int oy = (logical / xtiles) % Hout;
    const int64_t n = logical / (xtiles * Hout);
    const int tx = threadIdx.x & 31;
    const int ty = threadIdx.x >> 5;
    const ResampleTap th = resample_tap(hscale, oy, Hin);
    const ResampleTap tw = resample_tap(wscale, min(x0 + tx, Wout - 1), Win);
    const int64_t plane = (int64_t)Hin * Win;
    const float* base = src + n * C * plane + (int64_t)th.i1 * Win + tw.i1;
    float* drow = dst + ((n * Hout + oy) * (int64_t)Wout) * C;
    for (int c0 = 0; c0 < C; c0 += 128) {
#pragma unroll 2
        for (int i = 0; i < 4; ++i) {
            const int q = 8 * i + ty;
            const int c = min(c0 + 4 * q, C - 4);  // quads past the end repeat the last one and are not written
            float pb[4], v[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) pb[k] = (PRE && pre_bias) ? pre_bias[c + k] : 0.f;
            if (SAME) {
#pragma unroll
                for (int k = 0; k < 4; ++k) v[k] = base[(int64_t)(c + k) * plane] + pb[k];
                if (PRE) act_many<4>(v, act.pre, act.pre_n);
                act_many<4>(v, act.post, 1);
            } else {
                float t[16];
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const float* r0 = base + (int64_t)(c + k) * plane;
                    const float* r1 = r0 + (int64_t)th.ip * Win;
                    t[4 * k] = r0[0], t[4 * k + 1] = r0[tw.ip], t[4 * k + 2] = r1[0], t[4 * k + 3] = r1[tw.ip];
                }
                blend_many<PRE, 4>(t, pb, tw.l0, tw.l1, th.l0, th.l1, act, v);
            }
            tile[tx * 33 + q] = make_float4(v[0], v[1], v[2], v[3]);
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int xl = 8 * j + ty;
            const int x = x0 + xl;
            const int c = c0 + 4 * tx;
            if (x < Wout && c < C) *reinterpret_cast<float4*>(drow + (int64_t)x * C + c) = tile[xl * 33 + tx];
        }
        __syncthreads();
    }
}

// Up to four NCHW tensors that stand for their concatenation along C (DownScaler2D's cat([X1, X2, X3]) before its
// second interpolate, network/model.py:35-36).  Source s holds channels first[s] .. first[s+1]-1 of the result;
// bit s of pre_mask says that its samples still lack their bias and activation(s).
struct ResampleSources {
    const float *src0, *src1, *src2, *src3;
    const float *bias0, *bias1, *bias2, *bias3;  // null: no bias
    int first1, first2, first3;                  // the total channel count for absent sources
    int pre_mask;
};

// bilinear_to_nhwc_wide_k over such a concatenation, which is never materialised: every channel finds its tensor.
// The source activations are computed for all samples and kept where the mask asks for them.
// grid: tiles = N * Hout * ceil(Wout/32), rounded up to a multiple of 8; block 256.
__global__ __launch_bounds__(256) void bilinear_concat_to_nhwc_k(ResampleSources S, float* __restrict__ dst, int C,
                                                                 int Hin, int Win, int Hout, int Wout, float hscale,
                                                                 float wscale, ResampleAct act, int xtiles, int tiles,
                                                                 DropArgs drop) {
    __shared__ float4 tile[32 * 33];
    const int logical = xcd_contiguous_tile();
    if (logical >= tiles) return;
    const int x0 = (logical % xtiles) * 32;
    const int oy = (logical / xtiles) % Hout;
    const int64_t n = logical / (xtiles * Hout);
    const int tx = threadIdx.x & 31;
    const int ty = threadIdx.x >> 5;
    const ResampleTap th = resample_tap(hscale, oy, Hin);
    const ResampleTap tw = resample_tap(wscale, min(x0 + tx, Wout - 1), Win);
    const int64_t plane = (int64_t)Hin * Win;
    const int64_t off = (int64_t)th.i1 * Win + tw.i1;
    float* drow = dst + ((n * Hout + oy) * (int64_t)Wout) * C;
    for (int c0 = 0; c0 < C; c0 += 128) {
#pragma unroll 2
        for (int i = 0; i < 4; ++i) {
            const int q = 8 * i + ty;
            const int c = min(c0 + 4 * q, C - 4);  // quads past the end repeat the last one and are not written
            float t[16], u[16], v[4];
            bool pre[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int ch = c + k;
                const int s = (ch >= S.first1) + (ch >= S.first2) + (ch >= S.first3);
                const float* p = s == 0 ? S.src0 : s == 1 ? S.src1 : s == 2 ? S.src2 : S.src3;
                const float* b = s == 0 ? S.bias0 : s == 1 ? S.bias1 : s == 2 ? S.bias2 : S.bias3;
                const int lo = s == 0 ? 0 : s == 1 ? S.first1 : s == 2 ? S.first2 : S.first3;
                const int hi = s == 0 ? S.first1 : s == 1 ? S.first2 : s == 2 ? S.first3 : C;
                pre[k] = (S.pre_mask >> s) & 1;
                const float* r0 = p + (n * (hi - lo) + (ch - lo)) * plane + off;
                const float* r1 = r0 + (int64_t)th.ip * Win;
                t[4 * k] = r0[0], t[4 * k + 1] = r0[tw.ip], t[4 * k + 2] = r1[0], t[4 * k + 3] = r1[tw.ip];
                const float pb = (pre[k] && b) ? b[ch - lo] : 0.f;
#pragma unroll
                for (int j = 0; j < 4; ++j) u[4 * k + j] = t[4 * k + j] + pb;
                if (drop.seed && pre[k]) {
                    // a flagged source is a convolution output before its dropout: one decision per source sample,
                    // the same for every output that reads it
                    const DropoutSite ds = dropout_site(drop.seed, kDropSiteConcat, n * (hi - lo) + (ch - lo), drop.p);
                    const uint32_t e = (uint32_t)off;
                    u[4 * k] = dropout_apply(ds, e, u[4 * k]);
                    u[4 * k + 1] = dropout_apply(ds, e + (uint32_t)tw.ip, u[4 * k + 1]);
                    u[4 * k + 2] = dropout_apply(ds, e + (uint32_t)(th.ip * Win), u[4 * k + 2]);
                    u[4 * k + 3] = dropout_apply(ds, e + (uint32_t)(th.ip * Win + tw.ip), u[4 * k + 3]);
                }
            }
            if (S.pre_mask) {
                act_many<16>(u, act.pre, act.pre_n);
#pragma unroll
                for (int j = 0; j < 16; ++j) t[j] = pre[j >> 2] ? u[j] : t[j];
            }
            const float no_bias[4] = {0.f, 0.f, 0.f, 0.f};
            blend_many<false, 4>(t, no_bias, tw.l0, tw.l1, th.l0, th.l1, act, v);
            tile[tx * 33 + q] = make_float4(v[0], v[1], v[2], v[3]);
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int xl = 8 * j + ty;
            const int x = x0 + xl;
            const int c = c0 + 4 * tx;
            if (x < Wout && c < C) *reinterpret_cast<float4*>(drow + (int64_t)x * C + c) = tile[xl * 33 + tx];
        }
        __syncthreads();
    }
}

// Channels-last -> NCHW for C a multiple of 4 with a 16-byte aligned source: one workgroup makes 32 output columns
// x 128 channels of one output row.  A thread reads the four source pixels of a column 16 bytes (4 channels) at a
// time, 512-byte runs per 32 lanes, and blends them; the tile is turned in LDS and written along the output rows.
// Row c of the LDS tile holds column x at position x ^ (c / 32 % 4): the 32 lanes that write one column for 128
// channels then hit 32 banks, and a row read is a permutation of one row.
// grid: tiles = N * Hout * ceil(Wout/32), rounded up to a multiple of 8; block 256.
template <bool PRE>
__global__ __launch_bounds__(256) void bilinear_from_nhwc_wide_k(const float* __restrict__ src,
                                                                 const float* __restrict__ pre_bias,
                                                                 float* __restrict__ dst, int C, int Hin, int Win,
                                                                 int Hout, int Wout, float hscale, float wscale,
                                                                 ResampleAct act, int xtiles, int tiles) {
    __shared__ float tile[128 * 33];
    const int logical = xcd_contiguous_tile();
    if (logical >= tiles) return;
    const int x0 = (logical % xtiles) * 32;
    const int oy = (logical / xtiles) % Hout;
    const int64_t n = logical / (xtiles * Hout);
    const int tx = threadIdx.x & 31;
    const int ty = threadIdx.x >> 5;
    const ResampleTap th = resample_tap(hscale, oy, Hin);
    const float* rows = src + (n * Hin + th.i1) * (int64_t)Win * C;
    const int64_t rstep = (int64_t)th.ip * Win * C;
    for (int c0 = 0; c0 < C; c0 += 128) {
        const int c = min(c0 + 4 * tx, C - 4);  // quads past the end repeat the last one and are not written
        float pb[4] = {0.f, 0.f, 0.f, 0.f};
        if (PRE && pre_bias) {
            const float4 b4 = *reinterpret_cast<const float4*>(pre_bias + c);
            pb[0] = b4.x, pb[1] = b4.y, pb[2] = b4.z, pb[3] = b4.w;
        }
#pragma unroll 2
        for (int i = 0; i < 4; ++i) {
            const int xl = 8 * i + ty;
            const ResampleTap tw = resample_tap(wscale, min(x0 + xl, Wout - 1), Win);
            const float* p0 = rows + (int64_t)tw.i1 * C + c;
            const float* p1 = p0 + rstep;
            const float4 a00 = *reinterpret_cast<const float4*>(p0);
            const float4 a01 = *reinterpret_cast<const float4*>(p0 + tw.ip * C);
            const float4 a10 = *reinterpret_cast<const float4*>(p1);
            const float4 a11 = *reinterpret_cast<const float4*>(p1 + tw.ip * C);
            float t[16] = {a00.x, a01.x, a10.x, a11.x, a00.y, a01.y, a10.y, a11.y,
                           a00.z, a01.z, a10.z, a11.z, a00.w, a01.w, a10.w, a11.w};
            float v[4];
            blend_many<PRE, 4>(t, pb, tw.l0, tw.l1, th.l0, th.l1, act, v);
            const int pos = xl ^ (tx >> 3);
#pragma unroll
            for (int k = 0; k < 4; ++k) tile[(4 * tx + k) * 33 + pos] = v[k];
        }
        __syncthreads();
        const int ox = x0 + tx;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int cl = 8 * i + ty;
            if (ox < Wout && c0 + cl < C)
                dst[((n * C + c0 + cl) * Hout + oy) * (int64_t)Wout + ox] = tile[cl * 33 + (tx ^ (cl >> 5))];
        }
        __syncthreads();
    }
}

// Channels-last on both sides for C a multiple of 4, with the few extra input columns of a following Linear
// folded in: dst[n, y, x, c] = bilinear(src)[n, y, x, c] + sum_e extra[n, y, x, e] * w_extra[e, c].  A Linear over
// the channels commutes with the resampling (the blend weights of an output sum to 1), so the decoder's input
// layer Linear(cat([X, grid])) (network/sp_model.py:60) can run on the low-resolution X before UpScaler2D's last
// interpolate (network/model.py:63) instead of after it; what remains for the full resolution is the grid
// columns' rank-E update, applied here.  A thread makes 4 channels of 4 neighbouring pixels of an output row: the
// source pixels are 16-byte loads, contiguous across the lanes of a pixel and all 16 in flight together, and the
// results are 16-byte stores.
// grid: ceil(N*Hout*ceil(Wout/4)*C/4 / 256) rounded up to a multiple of 8, block 256.
__global__ __launch_bounds__(256) void bilinear_nhwc_affine_k(const float* __restrict__ src, float* __restrict__ dst,
                                                              int C4, int Hin, int Win, int Hout, int Wout,
                                                              float hscale, float wscale,
                                                              const float* __restrict__ extra,
                                                              const float* __restrict__ w_extra, int E,
                                                              unsigned items) {
    const unsigned f = (unsigned)xcd_contiguous_tile() * 256u + threadIdx.x;  // items < 2^31: 32-bit divisions
    if (f >= items) return;
    const unsigned xgroups = (unsigned)(Wout + 3) >> 2;
    const int q = (int)(f % (unsigned)C4);
    const unsigned group = f / (unsigned)C4;
    const int ox0 = (int)(group % xgroups) * 4;
    const unsigned line = group / xgroups;
    const int oy = (int)(line % (unsigned)Hout);
    const int64_t n = line / (unsigned)Hout;
    const ResampleTap th = resample_tap(hscale, oy, Hin);
    const int64_t C = 4 * (int64_t)C4;
    const float* row0 = src + (n * Hin + th.i1) * (int64_t)Win * C + 4 * q;
    const float* row1 = row0 + (int64_t)th.ip * Win * C;
    ResampleTap tw[4];
    float4 a00[4], a01[4], a10[4], a11[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        tw[j] = resample_tap(wscale, min(ox0 + j, Wout - 1), Win);  // pixels past the row's end: computed, not stored
        const int64_t o0 = (int64_t)tw[j].i1 * C, o1 = o0 + tw[j].ip * C;
        a00[j] = *reinterpret_cast<const float4*>(row0 + o0);
        a01[j] = *reinterpret_cast<const float4*>(row0 + o1);
        a10[j] = *reinterpret_cast<const float4*>(row1 + o0);
        a11[j] = *reinterpret_cast<const float4*>(row1 + o1);
    }
    const int64_t pix0 = ((n * Hout + oy) * (int64_t)Wout) + ox0;
    float4 wx[4];
    float gx[4][4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        wx[e] = e < E ? *reinterpret_cast<const float4*>(w_extra + e * C + 4 * q) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int j = 0; j < 4; ++j) gx[j][e] = (e < E && ox0 + j < Wout) ? extra[(pix0 + j) * E + e] : 0.f;
    }
    const float no_bias[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        float t[16] = {a00[j].x, a01[j].x, a10[j].x, a11[j].x, a00[j].y, a01[j].y, a10[j].y, a11[j].y,
                       a00[j].z, a01[j].z, a10[j].z, a11[j].z, a00[j].w, a01[j].w, a10[j].w, a11[j].w};
        float v[4];
        blend_many<false, 4>(t, no_bias, tw[j].l0, tw[j].l1, th.l0, th.l1, ResampleAct{SPGT_ACT_NONE, 0, SPGT_ACT_NONE},
                             v);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            v[0] = fmaf(gx[j][e], wx[e].x, v[0]), v[1] = fmaf(gx[j][e], wx[e].y, v[1]);
            v[2] = fmaf(gx[j][e], wx[e].z, v[2]), v[3] = fmaf(gx[j][e], wx[e].w, v[3]);
        }
        if (ox0 + j < Wout)
            *reinterpret_cast<float4*>(dst + (pix0 + j) * C + 4 * q) = make_float4(v[0], v[1], v[2], v[3]);
    }
}

// ---- adjoint of the resampling (its backward) -------------------------------------------------------------------
// The resampling is linear in its source, out[o] = sum over i of A[o][i] in[i] per axis with at most two non-zero
// weights per output, so the gradient of the source is grad_in[i] = sum over o of A[o][i] grad_out[o].  The reference
// leaves this to autograd of F.interpolate (network/model.py:30-38, 59-64), whose backward scatters with atomic
// additions; here every source position gathers from the few outputs that touch it, in a fixed order.

// Weight with which output index o reads source index i: both taps count (at the last source index they coincide).
__device__ __forceinline__ float adjoint_weight(float scale, int o, int i, int in_size) {
    const ResampleTap t = resample_tap(scale, o, in_size);
    return (t.i1 == i ? t.l0 : 0.f) + (t.i1 + t.ip == i ? t.l1 : 0.f);
}

__device__ __forceinline__ bool adjoint_touches(float scale, int o, int i, int in_size) {
    const ResampleTap t = resample_tap(scale, o, in_size);
    return t.i1 == i || t.i1 + t.ip == i;
}

// The outputs that touch source index i: first source index scale * o in (i - 1, i + 1).  The bounds are estimated
// in floating point and then widened while the neighbouring output still touches i, with the forward's own
// arithmetic, so that no contribution is lost to rounding; an output inside the range that does not touch i has
// weight zero.  lo > hi when no output reads i (down-sampling by more than two).
struct AdjointRange {
    int lo, hi;
};
__device__ __forceinline__ AdjointRange adjoint_range(float scale, int i, int in_size, int out_size) {
    AdjointRange r;
    if (!(scale > 0.f)) {
        r.lo = 0, r.hi = out_size - 1;
        return r;
    }
    const float inv = 1.0f / scale;
    r.lo = min(max((int)ceilf(((float)i - 1.f) * inv), 0), out_size - 1);
    r.hi = max(min((int)floorf(((float)i + 1.f) * inv), out_size - 1), 0);
    while (r.lo > 0 && adjoint_touches(scale, r.lo - 1, i, in_size)) --r.lo;
    while (r.hi < out_size - 1 && adjoint_touches(scale, r.hi + 1, i, in_size)) ++r.hi;
    return r;
}

// Channels-last on both sides: grad_out [N, Hout, Wout, C] -> grad_in [N, Hin, Win, C], C a multiple of 4.  A thread
// makes 4 channels of one source pixel; the lanes of a pixel read 16-byte pieces of one 4*C-byte run.  G outputs
// of a row are requested together (indices past the range repeat its last one with weight zero).
// grid: ceil(N*Hin*Win*C/4 / 256) rounded up to a multiple of 8, block 256.
template <int G>
__global__ __launch_bounds__(256) void bilinear_adjoint_nhwc_k(const float* __restrict__ gout,
                                                               float* __restrict__ gin, int C4, int Hin, int Win,
                                                               int Hout, int Wout, float hscale, float wscale,
                                                               unsigned items) {
    const unsigned f = (unsigned)xcd_contiguous_tile() * 256u + threadIdx.x;
    if (f >= items) return;
    const int q = (int)(f % (unsigned)C4);
    const unsigned pix = f / (unsigned)C4;
    const int x = (int)(pix % (unsigned)Win);
    const unsigned line = pix / (unsigned)Win;
    const int y = (int)(line % (unsigned)Hin);
    const int64_t n = line / (unsigned)Hin;
    const int64_t C = 4 * (int64_t)C4;
    const AdjointRange ry = adjoint_range(hscale, y, Hin, Hout), rx = adjoint_range(wscale, x, Win, Wout);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int oy = ry.lo; oy <= ry.hi; ++oy) {
        const float hw = adjoint_weight(hscale, oy, y, Hin);
        const float* row = gout + ((n * Hout + oy) * (int64_t)Wout) * C + 4 * q;
        for (int ox0 = rx.lo; ox0 <= rx.hi; ox0 += G) {
            float4 v[G];
            float w[G];
#pragma unroll
            for (int j = 0; j < G; ++j) {
                v[j] = *reinterpret_cast<const float4*>(row + (int64_t)min(ox0 + j, rx.hi) * C);
                w[j] = ox0 + j <= rx.hi ? hw * adjoint_weight(wscale, ox0 + j, x, Win) : 0.f;
            }
#pragma unroll
            for (int j = 0; j < G; ++j) {
                acc.x = fmaf(w[j], v[j].x, acc.x), acc.y = fmaf(w[j], v[j].y, acc.y);
                acc.z = fmaf(w[j], v[j].z, acc.z), acc.w = fmaf(w[j], v[j].w, acc.w);
            }
        }
    }
    *reinterpret_cast<float4*>(gin + (int64_t)pix * C + 4 * q) = acc;
}

// Planes on both sides: grad_out [planes, Hout, Wout] -> grad_in [planes, Hin, Win].  A thread makes one source
// position of 4 consecutive planes at a time; lanes run along the source row.
// One-dimensional launch of xt * yt * zb tiles (64 x 4 source positions, every zb-th group of 4 planes) rounded up to
// a multiple of 8, block (64, 4), the tiles of a plane group consecutive on one XCD as in bilinear_align_corners_k.
__global__ __launch_bounds__(256) void bilinear_adjoint_planes_k(const float* __restrict__ gout,
                                                                 float* __restrict__ gin, int planes, int Hin,
                                                                 int Win, int Hout, int Wout, float hscale,
                                                                 float wscale, int xt, int yt, int zb) {
    const int logical = xcd_contiguous_tile();
    if (logical >= xt * yt * zb) return;
    const int x = (logical % xt) * 64 + threadIdx.x;
    const int y = ((logical / xt) % yt) * 4 + threadIdx.y;
    const int bz = logical / (xt * yt);
    if (x >= Win || y >= Hin) return;
    const AdjointRange ry = adjoint_range(hscale, y, Hin, Hout), rx = adjoint_range(wscale, x, Win, Wout);
    const int64_t oplane = (int64_t)Hout * Wout;
    for (int64_t p0 = (int64_t)bz * 4; p0 < planes; p0 += (int64_t)zb * 4) {
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        const float* base[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) base[j] = gout + min(p0 + j, (int64_t)planes - 1) * oplane;  // repeats, unwritten
        for (int oy = ry.lo; oy <= ry.hi; ++oy) {
            const float hw = adjoint_weight(hscale, oy, y, Hin);
            for (int ox = rx.lo; ox <= rx.hi; ++ox) {
                const float w = hw * adjoint_weight(wscale, ox, x, Win);
                const int64_t o = (int64_t)oy * Wout + ox;
                float v[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) v[j] = base[j][o];
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[j] = fmaf(w, v[j], acc[j]);
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (p0 + j < planes) gin[((p0 + j) * Hin + y) * Win + x] = acc[j];
    }
}

// UpScaler2D's interpolate -> conv3x3(padding 1) -> bias -> activation(s) (network/model.py:59-62) with the channel
// mixing done before the interpolation.  Both steps are linear, so
//   conv(interp(X))[y, x, co] = sum over the 9 taps (ky, kx) of interp(Z_t)[y + ky - 1, x + kx - 1, co],
//   Z_t = X . W_t  (the 1x1 product with the tap's [Cin, Cout] weight slice), t = 3 ky + kx,
// where a tap that falls outside the interpolated image contributes nothing (the convolution's zero padding).
// The products Z [N, Hin, Win, 9, C] come from one GEMM on the low-resolution tokens, (Hout/Hin)^2 times fewer
// than the convolution would see; this kernel gathers: per output pixel and tap the four source pixels of
// Z_t, blended as in the resampling kernels, summed over the taps in a fixed order, then bias and the
// activation `act` applied `count` times.  Channels-last result [N, Hout, Wout, C], C a multiple of 4.
// A thread makes 4 channels of one pixel; the lanes of a pixel read 16-byte pieces of one 4*C-byte run, and the
// 8 (or more) neighbouring pixels of a workgroup share most of their source pixels through the L1.
// grid: ceil(N*Hout*Wout*C/4 / 256) rounded up to a multiple of 8, block 256.
__global__ __launch_bounds__(256) void upsample_conv3x3_gather_k(const float* __restrict__ Z,
                                                                 const float* __restrict__ bias,
                                                                 float* __restrict__ dst, int C4, int Hin, int Win,
                                                                 int Hout, int Wout, float hscale, float wscale, int act,
                                                                 int count, unsigned items) {
    const unsigned f = (unsigned)xcd_contiguous_tile() * 256u + threadIdx.x;  // items < 2^31: 32-bit divisions
    if (f >= items) return;
    const int q = (int)(f % (unsigned)C4);
    const unsigned pixel = f / (unsigned)C4;
    const int ox = (int)(pixel % (unsigned)Wout);
    const unsigned line = pixel / (unsigned)Wout;
    const int oy = (int)(line % (unsigned)Hout);
    const int64_t n = line / (unsigned)Hout;
    const int64_t C = 4 * (int64_t)C4;
    const int64_t pitch = 9 * C;  // floats per source pixel
    const float* Zn = Z + n * Hin * (int64_t)Win * pitch + 4 * q;
    ResampleTap tw[3];
    bool xin[3];
#pragma unroll
    for (int kx = 0; kx < 3; ++kx) {
        const int qx = ox + kx - 1;
        xin[kx] = qx >= 0 && qx < Wout;
        tw[kx] = resample_tap(wscale, min(max(qx, 0), Wout - 1), Win);
    }
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ky = 0; ky < 3; ++ky) {
        const int qy = oy + ky - 1;
        if (qy < 0 || qy >= Hout) continue;  // the same for all lanes of a pixel and for most of a workgroup
        const ResampleTap th = resample_tap(hscale, qy, Hin);
        const float* row0 = Zn + (int64_t)th.i1 * Win * pitch + (3 * ky) * C;
        const float* row1 = row0 + (int64_t)th.ip * Win * pitch;
        float4 a00[3], a01[3], a10[3], a11[3];
#pragma unroll
        for (int kx = 0; kx < 3; ++kx) {
            const int64_t o0 = (int64_t)tw[kx].i1 * pitch + kx * C, o1 = o0 + tw[kx].ip * pitch;
            a00[kx] = *reinterpret_cast<const float4*>(row0 + o0);
            a01[kx] = *reinterpret_cast<const float4*>(row0 + o1);
            a10[kx] = *reinterpret_cast<const float4*>(row1 + o0);
            a11[kx] = *reinterpret_cast<const float4*>(row1 + o1);
        }
#pragma unroll
        for (int kx = 0; kx < 3; ++kx) {
            float t[16] = {a00[kx].x, a01[kx].x, a10[kx].x, a11[kx].x, a00[kx].y, a01[kx].y, a10[kx].y, a11[kx].y,
                           a00[kx].z, a01[kx].z, a10[kx].z, a11[kx].z, a00[kx].w, a01[kx].w, a10[kx].w, a11[kx].w};
            const float no_bias[4] = {0.f, 0.f, 0.f, 0.f};
            float v[4];
            blend_many<false, 4>(t, no_bias, tw[kx].l0, tw[kx].l1, th.l0, th.l1,
                                 ResampleAct{SPGT_ACT_NONE, 0, SPGT_ACT_NONE}, v);
#pragma unroll
            for (int k = 0; k < 4; ++k) acc[k] += xin[kx] ? v[k] : 0.f;
        }
    }
    if (bias) {
        const float4 b = *reinterpret_cast<const float4*>(bias + 4 * q);
        acc[0] += b.x, acc[1] += b.y, acc[2] += b.z, acc[3] += b.w;
    }
    act_many<4>(acc, act, count);
    *reinterpret_cast<float4*>(dst + (int64_t)pixel * C + 4 * q) = make_float4(acc[0], acc[1], acc[2], acc[3]);
}

// The adjoint of upsample_conv3x3_gather_k without bias and activation (its backward): the gradient of the per-tap
// products, dZ[n, yl, xl, t, c] = sum over the output pixels (oy, ox) whose tap t = (ky, kx) reads the interpolated
// image at (qy, qx) = (oy + ky - 1, ox + kx - 1) inside the image, of weight(qy -> yl) weight(qx -> xl) g[n, oy, ox, c],
// with the weights of the resampling's adjoint (adjoint_weight).  A thread makes 4 channels of all nine taps of one
// low-resolution pixel: it walks the window of output pixels one wider than the range of interpolated positions
// that touch the pixel and adds each value into the taps that reach a touching position from it; fixed order.
// g [N, Hout, Wout, C], dZ [N, Hin, Win, 9, C].  grid: ceil(N*Hin*Win*C/4 / 256) rounded up to a multiple of 8.
__global__ __launch_bounds__(256) void upsample_conv3x3_gather_adjoint_k(const float* __restrict__ g,
                                                                         float* __restrict__ dZ, int C4, int Hin,
                                                                         int Win, int Hout, int Wout, float hscale,
                                                                         float wscale, unsigned items) {
    const unsigned f = (unsigned)xcd_contiguous_tile() * 256u + threadIdx.x;
    if (f >= items) return;
    const int q = (int)(f % (unsigned)C4);
    const unsigned pix = f / (unsigned)C4;
    const int xl = (int)(pix % (unsigned)Win);
    const unsigned line = pix / (unsigned)Win;
    const int yl = (int)(line % (unsigned)Hin);
    const int64_t n = line / (unsigned)Hin;
    const int64_t C = 4 * (int64_t)C4;
    const AdjointRange ry = adjoint_range(hscale, yl, Hin, Hout), rx = adjoint_range(wscale, xl, Win, Wout);
    float4 acc[9];
#pragma unroll
    for (int t = 0; t < 9; ++t) acc[t] = make_float4(0.f, 0.f, 0.f, 0.f);
    const int y0 = max(ry.lo - 1, 0), y1 = min(ry.hi + 1, Hout - 1);
    const int x0 = max(rx.lo - 1, 0), x1 = min(rx.hi + 1, Wout - 1);
    for (int oy = y0; oy <= y1; ++oy) {
        float hwk[3];
#pragma unroll
        for (int ky = 0; ky < 3; ++ky) {
            const int qy = oy + ky - 1;
            hwk[ky] = (qy >= 0 && qy < Hout) ? adjoint_weight(hscale, qy, yl, Hin) : 0.f;
        }
        const float* row = g + ((n * Hout + oy) * (int64_t)Wout) * C + 4 * q;
        for (int ox = x0; ox <= x1; ++ox) {
            float wwk[3];
#pragma unroll
            for (int kx = 0; kx < 3; ++kx) {
                const int qx = ox + kx - 1;
                wwk[kx] = (qx >= 0 && qx < Wout) ? adjoint_weight(wscale, qx, xl, Win) : 0.f;
            }
            const float4 v = *reinterpret_cast<const float4*>(row + (int64_t)ox * C);
#pragma unroll
            for (int ky = 0; ky < 3; ++ky)
#pragma unroll
                for (int kx = 0; kx < 3; ++kx) {
                    const float w = hwk[ky] * wwk[kx];
                    float4& a = acc[3 * ky + kx];
                    a.x = fmaf(w, v.x, a.x), a.y = fmaf(w, v.y, a.y), a.z = fmaf(w, v.z, a.z), a.w = fmaf(w, v.w, a.w);
                }
        }
    }
    float* dst = dZ + (int64_t)pix * 9 * C + 4 * q;
#pragma unroll
    for (int t = 0; t < 9; ++t) *reinterpret_cast<float4*>(dst + t * C) = acc[t];
}

// DownScaler2D's first stage in one pass for a few input channels (network/model.py:30-33:
// conv0 = ConvResBlock2D(in_dim, out_dim, 3x3, padding 1), interpolate to resolution_size[1],
// activation): out[n, c, oy, ox] = post(bilinear(pre(conv3x3(x)[n, c] + bias[c]))).  The four
// convolution outputs an output pixel blends need a 4x4 input patch per input channel, which the
// thread keeps in registers while it walks the output channels (weights are wave-uniform), so the
// full-resolution convolution output (91 MB at the Darcy shape) never exists.
// x [N, H, W, CIN] channels-last, weight [Cout, CIN, 3, 3], out [N, Cout, Hout, Wout].
// grid (ceil(Wout/64), Hout, N), block (64, 4): threadIdx.y walks the output channels 4 apart.
template <int CIN>
__global__ __launch_bounds__(256) void conv3x3_resample_k(const float* __restrict__ x,
                                                          const float* __restrict__ weight,
                                                          const float* __restrict__ bias, float* __restrict__ out,
                                                          int Cout, int H, int W, int Hout, int Wout, float hscale,
                                                          float wscale, ResampleAct act, DropArgs drop) {
    const int ox = blockIdx.x * 64 + threadIdx.x;
    const int oy = blockIdx.y;
    const int64_t n = blockIdx.z;
    const int oxc = min(ox, Wout - 1);
    const float hr = hscale * (float)oy;
    const int h1 = (int)hr;
    const int hp = (h1 < H - 1) ? 1 : 0;
    const float h1l = hr - (float)h1;
    const float h0l = 1.0f - h1l;
    const float wr = wscale * (float)oxc;
    const int w1 = (int)wr;
    const int wp = (w1 < W - 1) ? 1 : 0;
    const float w1l = wr - (float)w1;
    const float w0l = 1.0f - w1l;
    // patch[ci][dy][dx] = x[n, h1 - 1 + dy, w1 - 1 + dx, ci], zero outside the image
    float patch[CIN][4][4];
#pragma unroll
    for (int dy = 0; dy < 4; ++dy)
#pragma unroll
        for (int dx = 0; dx < 4; ++dx) {
            const int yy = h1 - 1 + dy, xx = w1 - 1 + dx;
            const bool in = yy >= 0 && yy < H && xx >= 0 && xx < W;
            const float* px = x + ((n * H + min(max(yy, 0), H - 1)) * (int64_t)W + min(max(xx, 0), W - 1)) * CIN;
#pragma unroll
            for (int ci = 0; ci < CIN; ++ci) patch[ci][dy][dx] = in ? px[ci] : 0.f;
        }
    // weights and biases of all output channels go through LDS once per workgroup (broadcast reads)
    extern __shared__ float wlds[];  // [Cout][CIN*9] then [Cout]
    float* blds = wlds + Cout * CIN * 9;
    const int tid = threadIdx.y * 64 + threadIdx.x;
    for (int e = tid; e < Cout * CIN * 9; e += 256) wlds[e] = weight[e];
    for (int e = tid; e < Cout; e += 256) blds[e] = bias ? bias[e] : 0.f;
    __syncthreads();
    const int wave_c = __builtin_amdgcn_readfirstlane(threadIdx.y);
    for (int c = wave_c; c < Cout; c += 4) {
        const float* wc = wlds + c * CIN * 9;
        const float b = blds[c];
        float v00 = b, v01 = b, v10 = b, v11 = b;  // conv at (h1, w1), (h1, w1+wp), (h1+hp, w1), (h1+hp, w1+wp)
#pragma unroll
        for (int ci = 0; ci < CIN; ++ci)
#pragma unroll
            for (int ky = 0; ky < 3; ++ky)
#pragma unroll
                for (int kx = 0; kx < 3; ++kx) {
                    const float wv = wc[ci * 9 + ky * 3 + kx];
                    v00 = fmaf(wv, patch[ci][ky][kx], v00);
                    v01 = fmaf(wv, patch[ci][ky][kx + 1], v01);
                    v10 = fmaf(wv, patch[ci][ky + 1][kx], v10);
                    v11 = fmaf(wv, patch[ci][ky + 1][kx + 1], v11);
                }
        // at the last row / column (hp or wp = 0) the second sample is the first one again
        float t[4] = {v00, wp ? v01 : v00, hp ? v10 : v00, hp ? (wp ? v11 : v10) : (wp ? v01 : v00)};
        if (drop.seed) {
            // the block's dropout sits between its convolution and its activation: one decision per convolution
            // output (n, c, y, x), the same for every resampled pixel that reads it
            const DropoutSite ds = dropout_site(drop.seed, kDropSiteConvResample, n * Cout + c, drop.p);
            const uint32_t e = (uint32_t)(h1 * W + w1);
            t[0] = dropout_apply(ds, e, t[0]);
            t[1] = dropout_apply(ds, e + (uint32_t)wp, t[1]);
            t[2] = dropout_apply(ds, e + (uint32_t)(hp * W), t[2]);
            t[3] = dropout_apply(ds, e + (uint32_t)(hp * W + wp), t[3]);
        }
        const float no_bias[1] = {0.f};  // the bias is in the convolution sums already
        float v[1];
        blend_many<true, 1>(t, no_bias, w0l, w1l, h0l, h1l, act, v);
        if (ox < Wout) out[((n * Cout + c) * Hout + oy) * (int64_t)Wout + ox] = v[0];
    }
}

// Backward of conv3x3_resample_k for an input that needs no gradient (the model's input field): the gradients of
// the convolution's weight and bias from the gradient of P = bilinear(pre(dropout(conv3x3(x) + bias))) (no post
// activation).  Nothing of the full-resolution chain was stored by the forward, so every source position (y, x)
// of a plane (n, c) is formed again: z = conv + bias, the dropout decision of the forward's seed, the derivative
// of the pre activation at the dropped value, and the resampling's adjoint gathered from the gradient plane
// (adjoint_range / adjoint_weight); gz = adjoint * act' * keep-scale then meets the 3x3 patch:
//   db[c] += gz,   dW[c][ci][ky][kx] += gz * x[n, y + ky - 1, x + kx - 1, ci].
// A workgroup takes one output channel and a run of image rows (rows of all images counted through), a wave a
// row at a time, lanes along x; per-thread sums are reduced over the workgroup in a fixed order and written as one
// record of R = 4 ceil((1 + 9 CIN) / 4) floats, [db, dW...]; tile_reduce adds the records of the runs.
// x [N, H, W, CIN] channels-last, grad [N, Cout, Hout, Wout], partial [runs][Cout][R].
// grid (runs, Cout), block (64, 4).
template <int CIN>
__global__ __launch_bounds__(256) void conv3x3_resample_backward_k(const float* __restrict__ x,
                                                                   const float* __restrict__ weight,
                                                                   const float* __restrict__ bias,
                                                                   const float* __restrict__ grad,
                                                                   float* __restrict__ partial, int N, int Cout, int H,
                                                                   int W, int Hout, int Wout, float hscale, float wscale,
                                                                   int pre_act, DropArgs drop, int rows_per_run) {
    constexpr int NV = 1 + 9 * CIN;
    constexpr int R = (NV + 3) / 4 * 4;
    const int c = blockIdx.y;
    const int run = blockIdx.x;
    const int lane = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.y);
    float wreg[9 * CIN];
#pragma unroll
    for (int k = 0; k < 9 * CIN; ++k) wreg[k] = weight[(int64_t)c * 9 * CIN + k];
    const float b = bias ? bias[c] : 0.f;
    float acc[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) acc[k] = 0.f;
    const int64_t total_rows = (int64_t)N * H;
    const int64_t g0 = (int64_t)run * rows_per_run, g1 = min(total_rows, g0 + rows_per_run);
    for (int64_t gr = g0 + wave; gr < g1; gr += 4) {
        const int64_t n = gr / H;
        const int y = (int)(gr - n * H);
        const AdjointRange ry = adjoint_range(hscale, y, H, Hout);
        DropoutSite ds;
        if (drop.seed) ds = dropout_site(drop.seed, kDropSiteConvResample, n * Cout + c, drop.p);
        const float* gplane = grad + (n * Cout + c) * (int64_t)Hout * Wout;
        for (int xx = lane; xx < W; xx += 64) {
            const AdjointRange rx = adjoint_range(wscale, xx, W, Wout);
            float gsum = 0.f;
            for (int oy = ry.lo; oy <= ry.hi; ++oy) {
                const float hw = adjoint_weight(hscale, oy, y, H);
                for (int ox = rx.lo; ox <= rx.hi; ++ox)
                    gsum = fmaf(hw * adjoint_weight(wscale, ox, xx, W), gplane[(int64_t)oy * Wout + ox], gsum);
            }
            float patch[9 * CIN];
#pragma unroll
            for (int ky = 0; ky < 3; ++ky)
#pragma unroll
                for (int kx = 0; kx < 3; ++kx) {
                    const int yy = y + ky - 1, xq = xx + kx - 1;
                    const bool in = yy >= 0 && yy < H && xq >= 0 && xq < W;
                    const float* px = x + ((n * H + min(max(yy, 0), H - 1)) * (int64_t)W + min(max(xq, 0), W - 1)) * CIN;
#pragma unroll
                    for (int ci = 0; ci < CIN; ++ci) patch[ci * 9 + ky * 3 + kx] = in ? px[ci] : 0.f;
                }
            float z = b;
#pragma unroll
            for (int k = 0; k < 9 * CIN; ++k) z = fmaf(wreg[k], patch[k], z);
            const bool keep = !drop.seed || dropout_keep(ds, (uint32_t)(y * W + xx));
            const float keep_scale = !keep ? 0.f : (drop.seed ? ds.scale : 1.f);
            const float zd = z * keep_scale;
            float d = 1.f;
            if (pre_act == SPGT_ACT_RELU) {
                d = zd > 0.f ? 1.f : 0.f;
            } else if (pre_act == SPGT_ACT_SILU) {
                const float sg = __builtin_amdgcn_rcpf(1.f + __expf(-zd));
                d = sg * (1.f + zd * (1.f - sg));
            }
            const float gz = gsum * d * keep_scale;
            acc[0] += gz;
#pragma unroll
            for (int k = 0; k < 9 * CIN; ++k) acc[1 + k] = fmaf(gz, patch[k], acc[1 + k]);
        }
    }
    // lanes of a wave, then the four waves, in a fixed order
    __shared__ float red[4][R];
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        float v = acc[k];
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
        if (lane == 0) red[wave][k] = v;
    }
    __syncthreads();
    const int tid = threadIdx.y * 64 + threadIdx.x;
    if (tid < R)
        partial[((int64_t)run * Cout + c) * R + tid] =
            tid < NV ? (red[0][tid] + red[1][tid]) + (red[2][tid] + red[3][tid]) : 0.f;
}

// The adjoint's geometry along one axis as a table, for resamplings that do not enlarge (scale >= 1: a source
// index is read by at most three outputs): entry i = (first output lo, weights of outputs lo, lo + 1, lo + 2; zero
// where the output does not read i).  grid (ceil(in_size / 256)), block 256.
__global__ __launch_bounds__(256) void adjoint_table_k(float scale, int in_size, int out_size, float4* __restrict__ table) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= in_size) return;
    AdjointRange r = adjoint_range(scale, i, in_size, out_size);
    // outputs at the range's start that touch i with weight zero are skipped: with scale >= 1 the source positions
    // of the outputs are at least one apart, so at most three of them lie within one of i
    while (r.lo < r.hi && adjoint_weight(scale, r.lo, i, in_size) == 0.f) ++r.lo;
    float w[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) w[k] = (r.lo + k <= r.hi) ? adjoint_weight(scale, r.lo + k, i, in_size) : 0.f;
    table[i] = make_float4(__int_as_float(max(r.lo, 0)), w[0], w[1], w[2]);
}

// conv3x3_resample_backward_k with the adjoint's geometry read from adjoint_table_k's tables (rows: ytab, columns:
// xtab) instead of being formed per position and channel, and CG output channels per workgroup, which share a
// position's input patch, its nine gather weights and offsets.  Records as in conv3x3_resample_backward_k.
// grid (runs, ceil(Cout / CG)), block (64, 4).
template <int CIN, int CG>
__global__ __launch_bounds__(256) void conv3x3_resample_backward_tab_k(
    const float* __restrict__ x, const float* __restrict__ weight, const float* __restrict__ bias,
    const float* __restrict__ grad, float* __restrict__ partial, int N, int Cout, int H, int W, int Hout, int Wout,
    const float4* __restrict__ ytab, const float4* __restrict__ xtab, int pre_act, DropArgs drop, int rows_per_run) {
    constexpr int NV = 1 + 9 * CIN;
    constexpr int R = (NV + 3) / 4 * 4;
    const int c0 = blockIdx.y * CG;
    const int run = blockIdx.x;
    const int lane = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.y);
    float wreg[CG][9 * CIN], breg[CG], acc[CG][NV];
#pragma unroll
    for (int j = 0; j < CG; ++j) {
        const int c = min(c0 + j, Cout - 1);  // channels past the end repeat the last and are not written
#pragma unroll
        for (int k = 0; k < 9 * CIN; ++k) wreg[j][k] = weight[(int64_t)c * 9 * CIN + k];
        breg[j] = bias ? bias[c] : 0.f;
#pragma unroll
        for (int k = 0; k < NV; ++k) acc[j][k] = 0.f;
    }
    const int64_t total_rows = (int64_t)N * H;
    const int64_t g0 = (int64_t)run * rows_per_run, g1 = min(total_rows, g0 + rows_per_run);
    const int64_t oplane = (int64_t)Hout * Wout;
    for (int64_t gr = g0 + wave; gr < g1; gr += 4) {
        const int64_t n = gr / H;
        const int y = (int)(gr - n * H);
        const float4 ty = ytab[y];
        const int ylo = __float_as_int(ty.x);
        const float hw[3] = {ty.y, ty.z, ty.w};
        int yoff[3];
#pragma unroll
        for (int a = 0; a < 3; ++a) yoff[a] = min(ylo + a, Hout - 1) * Wout;
        DropoutSite ds[CG];
        if (drop.seed) {
#pragma unroll
            for (int j = 0; j < CG; ++j)
                ds[j] = dropout_site(drop.seed, kDropSiteConvResample, n * Cout + min(c0 + j, Cout - 1), drop.p);
        }
        const float* gimg = grad + (n * Cout + c0) * oplane;
        for (int xx = lane; xx < W; xx += 64) {
            const float4 tx = xtab[xx];
            const int xlo = __float_as_int(tx.x);
            const float ww[3] = {tx.y, tx.z, tx.w};
            float wgt[9];
            int off[9];
#pragma unroll
            for (int a = 0; a < 3; ++a)
#pragma unroll
                for (int e = 0; e < 3; ++e) {
                    wgt[3 * a + e] = hw[a] * ww[e];
                    off[3 * a + e] = yoff[a] + min(xlo + e, Wout - 1);
                }
            float patch[9 * CIN];
#pragma unroll
            for (int ky = 0; ky < 3; ++ky)
#pragma unroll
                for (int kx = 0; kx < 3; ++kx) {
                    const int yy = y + ky - 1, xq = xx + kx - 1;
                    const bool in = yy >= 0 && yy < H && xq >= 0 && xq < W;
                    const float* px = x + ((n * H + min(max(yy, 0), H - 1)) * (int64_t)W + min(max(xq, 0), W - 1)) * CIN;
#pragma unroll
                    for (int ci = 0; ci < CIN; ++ci) patch[ci * 9 + ky * 3 + kx] = in ? px[ci] : 0.f;
                }
            const uint32_t e = (uint32_t)(y * W + xx);
#pragma unroll
            for (int j = 0; j < CG; ++j) {
                const float* gp = gimg + min(j, Cout - 1 - c0) * oplane;
                float gsum = 0.f;
#pragma unroll
                for (int t = 0; t < 9; ++t) gsum = fmaf(wgt[t], gp[off[t]], gsum);
                float z = breg[j];
#pragma unroll
                for (int k = 0; k < 9 * CIN; ++k) z = fmaf(wreg[j][k], patch[k], z);
                const bool keep = !drop.seed || dropout_keep(ds[j], e);
                const float keep_scale = !keep ? 0.f : (drop.seed ? ds[j].scale : 1.f);
                const float zd = z * keep_scale;
                float d = 1.f;
                if (pre_act == SPGT_ACT_RELU) {
                    d = zd > 0.f ? 1.f : 0.f;
                } else if (pre_act == SPGT_ACT_SILU) {
                    const float sg = __builtin_amdgcn_rcpf(1.f + __expf(-zd));
                    d = sg * (1.f + zd * (1.f - sg));
                }
                const float gz = gsum * d * keep_scale;
                acc[j][0] += gz;
#pragma unroll
                for (int k = 0; k < 9 * CIN; ++k) acc[j][1 + k] = fmaf(gz, patch[k], acc[j][1 + k]);
            }
        }
    }
    __shared__ float red[4][CG * R];
#pragma unroll
    for (int j = 0; j < CG; ++j)
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            float v = acc[j][k];
#pragma unroll
            for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
            if (lane == 0) red[wave][j * R + k] = v;
        }
    __syncthreads();
    const int tid = threadIdx.y * 64 + threadIdx.x;
    for (int i = tid; i < CG * R; i += 256) {
        const int j = i / R, k = i - j * R;
        if (c0 + j < Cout)
            partial[((int64_t)run * Cout + c0 + j) * R + k] =
                k < NV ? (red[0][i] + red[1][i]) + (red[2][i] + red[3][i]) : 0.f;
    }
}

// x[n, c, :] = act^count(x[n, c, :] + bias[c]) in place on [planes = N*C, HW]: the bias add and the
// activation(s) that follow a bias-free convolution.  grid (chunks, planes), block 256.
__global__ __launch_bounds__(256) void bias_activation_nchw_k(float* __restrict__ x, const float* __restrict__ bias,
                                                              int C, int64_t HW, int act, int count, DropArgs drop) {
    const int64_t pl = blockIdx.y;
    const float b = bias ? bias[pl % C] : 0.f;
    float* row = x + pl * HW;
    const int64_t stride = (int64_t)gridDim.x * 256;
    DropoutSite ds;
    if (drop.seed) ds = dropout_site(drop.seed, kDropSiteBiasAct, pl, drop.p);
    for (int64_t e0 = (int64_t)blockIdx.x * 256 + threadIdx.x; e0 < HW; e0 += 4 * stride) {
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = row[min(e0 + j * stride, HW - 1)] + b;  // past the end: read, not written
        if (drop.seed) {
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = dropout_apply(ds, (uint32_t)min(e0 + j * stride, HW - 1), v[j]);
        }
        act_many<4>(v, act, count);
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (e0 + j * stride < HW) row[e0 + j * stride] = v[j];
    }
}

}  // namespace spgt

using namespace spgt;

extern "C" int spgt_spectral_mode_contract(const float* X_ft, const float* weight_1, const float* weight_2,
                                           float* Out_ft, int N, int Cin, int Cout, int H_all, int W_all,
                                           int H_low, int W_low, int H_base_1, int W_base_1, int H_base_2,
                                           int W_base_2, hipStream_t stream) {
    if (!X_ft || !weight_1 || !weight_2 || !Out_ft)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_mode_contract: null pointer argument");
    if (N <= 0 || Cin <= 0 || Cout <= 0 || H_all <= 0 || W_all <= 0 || H_low <= 0 || W_low <= 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_mode_contract: sizes must be positive");
    if (H_base_1 < 0 || H_base_2 < 0 || W_base_1 < 0 || W_base_2 < 0 || H_base_1 + H_low > H_all ||
        H_base_2 + H_low > H_all || W_base_1 + W_low > W_all || W_base_2 + W_low > W_all)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_mode_contract: a window leaves the [H_all, W_all] plane");
    if ((size_t)kSpecNB * Cin * sizeof(float2) > 64 * 1024)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_mode_contract: Cin above 512 is not supported");
    if (ceil_div(Cout, 64) > 65535)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_mode_contract: Cout too large");
    if (X_ft == Out_ft) return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_mode_contract: in-place call is not supported");
    if (!aligned8(X_ft) || !aligned8(weight_1) || !aligned8(weight_2) || !aligned8(Out_ft))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_mode_contract: complex operands must be 8-byte aligned");
    SpecWindows win{{H_base_1, H_base_2}, {W_base_1, W_base_2}};
    const int64_t plane = (int64_t)H_all * W_all;
    const int jw = W_low % 3 == 0 ? 3 : (W_low < 4 ? W_low : 4);  // window columns per contraction block
    const size_t row_lds = ((size_t)kRowsNB * Cin * jw + (size_t)4 * 4 * jw * 64) * sizeof(float2);
    const int64_t nA64 = (int64_t)ceil_div(N, kRowsNB) * 2 * H_low * ceil_div(Cout, 64) * ceil_div(W_low, jw);
    if (row_lds <= 64 * 1024 && nA64 + (int64_t)N * Cout * 8 < ((int64_t)1 << 31)) {
        // one launch: window rows by contraction blocks, all other rows by zero-fill blocks
        const SpecSpans spans = rows_outside_windows(H_all, H_low, H_base_1, H_base_2);
        int64_t zero_rows = 0;
        for (int sidx = 0; sidx < spans.n; ++sidx) zero_rows += spans.hi[sidx] - spans.lo[sidx];
        // 16 KB of zeros per block or thereabouts
        const int chunks = zero_rows == 0 ? 0 : (int)std::max<int64_t>(1, std::min<int64_t>(8, zero_rows * W_all / SPGT_ZERO_CHUNK));
        const int nA = (int)nA64;
        const int64_t nB = (int64_t)N * Cout * (std::max(1, chunks) + 1);
        const dim3 grid((unsigned)(nA + nB));
#define SPGT_ROWS_LAUNCH(JW)                                                                                         \
    hipLaunchKernelGGL((spectral_contract_rows_k<JW>), grid, dim3(256), row_lds, stream,                              \
                       reinterpret_cast<const float2*>(X_ft), reinterpret_cast<const float2*>(weight_1),             \
                       reinterpret_cast<const float2*>(weight_2), reinterpret_cast<float2*>(Out_ft), N, Cin, Cout,   \
                       H_all, W_all, H_low, W_low, win, spans, nA, std::max(1, chunks))
        if (jw == 1) SPGT_ROWS_LAUNCH(1);
        else if (jw == 2) SPGT_ROWS_LAUNCH(2);
        else if (jw == 3) SPGT_ROWS_LAUNCH(3);
        else SPGT_ROWS_LAUNCH(4);
#undef SPGT_ROWS_LAUNCH
        return check_launch("spectral_mode_contract");
    }
    // very wide inputs: zero fill, then one workgroup per mode
    const int64_t total = (int64_t)N * Cout * H_all * W_all;
    const int fill_blocks = (int)std::min<int64_t>((total + 255) / 256, 256 * 32);
    hipLaunchKernelGGL(spectrum_zero_outside_k, dim3(fill_blocks), dim3(256), 0, stream,
                       reinterpret_cast<float2*>(Out_ft), total, H_all, W_all, H_low, W_low, win);
    const dim3 grid(H_low * W_low, 2, ceil_div(Cout, 64));
    const SpecLayout lay{Cin * plane, plane, W_all, 1, Cout * plane, plane, W_all, 1, 0};
    hipLaunchKernelGGL(spectral_mode_contract_k, grid, dim3(256), (size_t)kSpecNB * Cin * sizeof(float2), stream,
                       reinterpret_cast<const float2*>(X_ft), reinterpret_cast<const float2*>(weight_1),
                       reinterpret_cast<const float2*>(weight_2), reinterpret_cast<float2*>(Out_ft), N, Cin, Cout,
                       H_low, W_low, win, lay);
    return check_launch("spectral_mode_contract");
}

extern "C" int spgt_spectral_modes_compact(const float* Z, const float* weight_1, const float* weight_2, float* O,
                                           int N, int Cin, int Cout, int H_low, int W_low, hipStream_t stream) {
    if (!Z || !weight_1 || !weight_2 || !O)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_modes_compact: null pointer argument");
    if (N <= 0 || Cin <= 0 || Cout <= 0 || H_low <= 0 || W_low <= 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_modes_compact: sizes must be positive");
    if ((size_t)kSpecNB * Cin * sizeof(float2) > 64 * 1024)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_modes_compact: Cin above 512 is not supported");
    if (Z == O) return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_modes_compact: in-place call is not supported");
    if (!aligned8(Z) || !aligned8(weight_1) || !aligned8(weight_2) || !aligned8(O))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "spectral_modes_compact: complex operands must be 8-byte aligned");
    // Z [N, 2*H_low, Cin, W_low], O [N, 2*H_low, Cout, W_low]
    const SpecWindows win{{0, 0}, {0, 0}};
    const SpecLayout lay{(int64_t)2 * H_low * Cin * W_low, W_low, (int64_t)Cin * W_low, 1,
                         (int64_t)2 * H_low * Cout * W_low, W_low, (int64_t)Cout * W_low, 1, 1};
    const dim3 grid(H_low * W_low, 2, ceil_div(Cout, 64));
    hipLaunchKernelGGL(spectral_mode_contract_k, grid, dim3(256), (size_t)kSpecNB * Cin * sizeof(float2), stream,
                       reinterpret_cast<const float2*>(Z), reinterpret_cast<const float2*>(weight_1),
                       reinterpret_cast<const float2*>(weight_2), reinterpret_cast<float2*>(O), N, Cin, Cout, H_low,
                       W_low, win, lay);
    return check_launch("spectral_modes_compact");
}

namespace {

bool act_known(int a) { return a == SPGT_ACT_NONE || a == SPGT_ACT_RELU || a == SPGT_ACT_SILU; }

int resample_common(const char* who, const float* src, const float* pre_bias, float* dst, int N, int C, int H_in, int W_in, int H_out,
                    int W_out, int src_layout, int dst_layout, ResampleAct act, hipStream_t stream) {
    if (!src || !dst) return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear resampling: null pointer argument");
    if (N <= 0 || C <= 0 || H_in <= 0 || W_in <= 0 || H_out <= 0 || W_out <= 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear resampling: sizes must be positive");
    if (!aligned4(src) || !aligned4(dst))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear resampling: operands must be 4-byte aligned");
    if (!act_known(act.pre) || !act_known(act.post) || act.pre_n < 0 || act.pre_n > 2)
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "bilinear resampling: unknown activation, or more than two source activations");
    const float hscale = H_out > 1 ? (float)(H_in - 1) / (float)(H_out - 1) : 0.f;
    const float wscale = W_out > 1 ? (float)(W_in - 1) / (float)(W_out - 1) : 0.f;
    if (act.pre == SPGT_ACT_NONE) act.pre_n = 0;
    const bool pre = pre_bias != nullptr || act.pre_n > 0;
    if (src_layout == SPGT_LAYOUT_NCHW && dst_layout == SPGT_LAYOUT_NCHW) {
        const int64_t planes = (int64_t)N * C;
        if (planes > INT32_MAX)
            return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear resampling: more than 2^31 planes");
        const int xt = ceil_div(W_out, 64), yt = ceil_div(H_out, 4);
        // about 16 tiles per compute unit: a thread then walks several plane groups with one set of taps
        const int zb = (int)std::max<int64_t>(1, std::min<int64_t>(ceil_div(planes, (int64_t)4),
                                                                   16 * (int64_t)device_cu_count() / ((int64_t)xt * yt)));
        if ((int64_t)xt * yt > (1 << 30))
            return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear resampling: more than 2^38 output positions per plane");
        const unsigned blocks = (unsigned)(ceil_div((int64_t)xt * yt * zb, (int64_t)8) * 8);
        hipLaunchKernelGGL(pre ? bilinear_align_corners_k<true> : bilinear_align_corners_k<false>, dim3(blocks),
                           dim3(64, 4), 0, stream, src, pre_bias, C, dst, (int)planes, H_in, W_in, H_out, W_out, hscale,
                           wscale, act, xt, yt, zb);
    } else if (src_layout != dst_layout && (src_layout == SPGT_LAYOUT_NCHW || src_layout == SPGT_LAYOUT_NHWC) &&
               (dst_layout == SPGT_LAYOUT_NCHW || dst_layout == SPGT_LAYOUT_NHWC)) {
        if (H_out > 65535 || N > 65535)
            return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear resampling: N or H_out exceeds 65535");
        const dim3 grid(ceil_div(W_out, 32), H_out, N);
        // whole pixels of 4-channel pieces: the wide kernels, with a one-dimensional XCD-aware launch
        const int xtiles = ceil_div(W_out, 32);
        const int64_t tiles = (int64_t)N * H_out * xtiles;
        const bool wide = C % 4 == 0 && tiles <= (1 << 30) && (!pre_bias || aligned16(pre_bias)) &&
                          aligned16(dst_layout == SPGT_LAYOUT_NHWC ? (const void*)dst : (const void*)src);
        const dim3 wide_grid((unsigned)(ceil_div(tiles, (int64_t)8) * 8));
        const bool same = H_in == H_out && W_in == W_out;
        if (wide && dst_layout == SPGT_LAYOUT_NHWC)
            hipLaunchKernelGGL(same ? (pre ? bilinear_to_nhwc_wide_k<true, true> : bilinear_to_nhwc_wide_k<false, true>)
                                    : (pre ? bilinear_to_nhwc_wide_k<true, false> : bilinear_to_nhwc_wide_k<false, false>),
                               wide_grid, dim3(256), 0, stream, src, pre_bias, dst, C, H_in, W_in, H_out, W_out, hscale,
                               wscale, act, xtiles, (int)tiles);
        else if (wide)
            hipLaunchKernelGGL(pre ? bilinear_from_nhwc_wide_k<true> : bilinear_from_nhwc_wide_k<false>, wide_grid,
                               dim3(256), 0, stream, src, pre_bias, dst, C, H_in, W_in, H_out, W_out, hscale, wscale,
                               act, xtiles, (int)tiles);
        else if (dst_layout == SPGT_LAYOUT_NHWC)
            hipLaunchKernelGGL(pre ? bilinear_align_corners_nhwc_k<true> : bilinear_align_corners_nhwc_k<false>, grid,
                               dim3(256), 0, stream, src, pre_bias, dst, C, H_in, W_in, H_out, W_out, hscale, wscale,
                               act);
        else
            hipLaunchKernelGGL(pre ? bilinear_align_corners_from_nhwc_k<true> : bilinear_align_corners_from_nhwc_k<false>,
                               grid, dim3(256), 0, stream, src, pre_bias, dst, C, H_in, W_in, H_out, W_out, hscale,
                               wscale, act);
    } else {
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "bilinear resampling: layouts must be NCHW->NCHW, NCHW->NHWC or NHWC->NCHW");
    }
    return check_launch(who);
}

}  // namespace

extern "C" int spgt_bilinear_align_corners(const float* src, float* dst, int planes, int H_in, int W_in, int H_out,
                                           int W_out, hipStream_t stream) {
    return resample_common("bilinear_align_corners", src, nullptr, dst, 1, planes, H_in, W_in, H_out, W_out, SPGT_LAYOUT_NCHW,
                           SPGT_LAYOUT_NCHW, ResampleAct{SPGT_ACT_NONE, 0, SPGT_ACT_NONE}, stream);
}

extern "C" int spgt_bilinear_align_corners_nhwc(const float* src, float* dst, int N, int C, int H_in, int W_in,
                                                int H_out, int W_out, hipStream_t stream) {
    return resample_common("bilinear_align_corners_nhwc", src, nullptr, dst, N, C, H_in, W_in, H_out, W_out, SPGT_LAYOUT_NCHW,
                           SPGT_LAYOUT_NHWC, ResampleAct{SPGT_ACT_NONE, 0, SPGT_ACT_NONE}, stream);
}

namespace {

// seed / rate of the entry points that drop: rate 0 means none (seed may then be null)
int drop_args(const uint32_t* seed, float droprate, spgt::DropArgs* out) {
    if (!(droprate >= 0.f && droprate < 1.f)) return fail(SPGT_ERR_INVALID_ARGUMENT, "dropout: the rate must lie in [0, 1)");
    if (droprate > 0.f && (!seed || !aligned8(seed)))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "dropout: a rate above 0 needs an 8-byte aligned seed (two 32-bit words) in device memory");
    out->seed = droprate > 0.f ? seed : nullptr;
    out->p = droprate;
    return SPGT_OK;
}

int resample_concat_common(const float* const* srcs, const float* const* pre_biases, const int* channels,
                           const int* pre_flags, int n_src, float* dst, int N, int H_in, int W_in, int H_out, int W_out,
                           int pre_activation, int pre_activation_count, int post_activation, spgt::DropArgs drop,
                           hipStream_t stream) {
    if (!srcs || !channels || !dst) return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear_resample_concat: null pointer argument");
    if (n_src < 1 || n_src > 4) return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear_resample_concat: 1 to 4 sources");
    if (N <= 0 || H_in <= 0 || W_in <= 0 || H_out <= 0 || W_out <= 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear_resample_concat: sizes must be positive");
    ResampleAct act{pre_activation, pre_activation_count, post_activation};
    if (!act_known(act.pre) || !act_known(act.post) || act.pre_n < 0 || act.pre_n > 2)
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "bilinear_resample_concat: unknown activation, or more than two source activations");
    if (act.pre == SPGT_ACT_NONE) act.pre_n = 0;
    const float* src[4] = {nullptr, nullptr, nullptr, nullptr};
    const float* bias[4] = {nullptr, nullptr, nullptr, nullptr};
    int first[5] = {0, 0, 0, 0, 0}, mask = 0;
    int64_t C = 0;
    for (int s = 0; s < n_src; ++s) {
        if (!srcs[s] || channels[s] <= 0 || !aligned4(srcs[s]))
            return fail(SPGT_ERR_INVALID_ARGUMENT,
                        "bilinear_resample_concat: every source needs a 4-byte aligned pointer and a positive channel count");
        src[s] = srcs[s];
        first[s] = (int)C;
        C += channels[s];
        if (pre_flags && pre_flags[s]) {
            mask |= 1 << s;
            bias[s] = pre_biases ? pre_biases[s] : nullptr;
            if (bias[s] && !aligned4(bias[s]))
                return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear_resample_concat: biases must be 4-byte aligned");
        }
    }
    if (C % 4 != 0 || C > (1 << 24) || !aligned16(dst))
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "bilinear_resample_concat: the channels must add up to a multiple of 4 and dst be 16-byte aligned");
    for (int s = n_src; s < 5; ++s) first[s] = (int)C;
    const int xtiles = ceil_div(W_out, 32);
    const int64_t tiles = (int64_t)N * H_out * xtiles;
    if (tiles > (1 << 30)) return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear_resample_concat: too many output tiles");
    const float hscale = H_out > 1 ? (float)(H_in - 1) / (float)(H_out - 1) : 0.f;
    const float wscale = W_out > 1 ? (float)(W_in - 1) / (float)(W_out - 1) : 0.f;
    const ResampleSources S{src[0], src[1], src[2], src[3], bias[0], bias[1], bias[2], bias[3],
                            first[1], first[2], first[3], mask};
    if ((int64_t)H_in * W_in > UINT32_MAX) return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear_resample_concat: source planes above 2^32 samples");
    hipLaunchKernelGGL(spgt::bilinear_concat_to_nhwc_k, dim3((unsigned)(ceil_div(tiles, (int64_t)8) * 8)), dim3(256), 0,
                       stream, S, dst, (int)C, H_in, W_in, H_out, W_out, hscale, wscale, act, xtiles, (int)tiles, drop);
    return check_launch("bilinear_resample_concat");
}

}  // namespace

extern "C" int spgt_bilinear_resample_concat(const float* const* srcs, const float* const* pre_biases,
                                             const int* channels, const int* pre_flags, int n_src, float* dst, int N,
                                             int H_in, int W_in, int H_out, int W_out, int pre_activation,
                                             int pre_activation_count, int post_activation, hipStream_t stream) {
    return resample_concat_common(srcs, pre_biases, channels, pre_flags, n_src, dst, N, H_in, W_in, H_out, W_out,
                                  pre_activation, pre_activation_count, post_activation, spgt::DropArgs{nullptr, 0.f},
                                  stream);
}

extern "C" int spgt_bilinear_resample_concat_dropout(const float* const* srcs, const float* const* pre_biases,
                                                     const int* channels, const int* pre_flags, int n_src, float* dst,
                                                     int N, int H_in, int W_in, int H_out, int W_out,
                                                     int pre_activation, int pre_activation_count, int post_activation,
                                                     const uint32_t* seed, float droprate, hipStream_t stream) {
    spgt::DropArgs drop;
    if (int rc = drop_args(seed, droprate, &drop)) return rc;
    return resample_concat_common(srcs, pre_biases, channels, pre_flags, n_src, dst, N, H_in, W_in, H_out, W_out,
                                  pre_activation, pre_activation_count, post_activation, drop, stream);
}

extern "C" int spgt_upsample_conv3x3_gather(const float* Z, const float* bias, float* dst, int N, int C, int H_in,
                                            int W_in, int H_out, int W_out, int activation, int activation_count,
                                            hipStream_t stream) {
    if (!Z || !dst) return fail(SPGT_ERR_INVALID_ARGUMENT, "upsample_conv3x3_gather: null pointer argument");
    if (N <= 0 || C <= 0 || H_in <= 0 || W_in <= 0 || H_out <= 0 || W_out <= 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "upsample_conv3x3_gather: sizes must be positive");
    if (C % 4 != 0) return fail(SPGT_ERR_INVALID_ARGUMENT, "upsample_conv3x3_gather: C must be a multiple of 4");
    if (!act_known(activation) || activation_count < 0 || activation_count > 2)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "upsample_conv3x3_gather: unknown activation or count outside 0..2");
    if (!aligned16(Z) || !aligned16(dst) || (bias && !aligned16(bias)))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "upsample_conv3x3_gather: operands must be 16-byte aligned");
    const int64_t items = (int64_t)N * H_out * W_out * (C / 4);
    if (items > (int64_t)INT32_MAX - 2048)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "upsample_conv3x3_gather: more than 2^33 output elements");
    const int64_t blocks = ceil_div(ceil_div(items, (int64_t)256), (int64_t)8) * 8;
    const float hscale = H_out > 1 ? (float)(H_in - 1) / (float)(H_out - 1) : 0.f;
    const float wscale = W_out > 1 ? (float)(W_in - 1) / (float)(W_out - 1) : 0.f;
    hipLaunchKernelGGL(spgt::upsample_conv3x3_gather_k, dim3((unsigned)blocks), dim3(256), 0, stream, Z, bias, dst,
                       C / 4, H_in, W_in, H_out, W_out, hscale, wscale, activation,
                       activation == SPGT_ACT_NONE ? 0 : activation_count, (unsigned)items);
    return check_launch("upsample_conv3x3_gather");
}

extern "C" int spgt_upsample_conv3x3_gather_adjoint(const float* grad, float* dZ, int N, int C, int H_in, int W_in,
                                                    int H_out, int W_out, hipStream_t stream) {
    if (!grad || !dZ) return fail(SPGT_ERR_INVALID_ARGUMENT, "upsample_conv3x3_gather_adjoint: null pointer argument");
    if (N <= 0 || C <= 0 || H_in <= 0 || W_in <= 0 || H_out <= 0 || W_out <= 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "upsample_conv3x3_gather_adjoint: sizes must be positive");
    if (C % 4 != 0) return fail(SPGT_ERR_INVALID_ARGUMENT, "upsample_conv3x3_gather_adjoint: C must be a multiple of 4");
    if (!aligned16(grad) || !aligned16(dZ))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "upsample_conv3x3_gather_adjoint: operands must be 16-byte aligned");
    if (H_in > (1 << 23) || W_in > (1 << 23) || H_out > (1 << 23) || W_out > (1 << 23))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "upsample_conv3x3_gather_adjoint: image sides above 2^23");
    const int64_t items = (int64_t)N * H_in * W_in * (C / 4);
    if (items > (int64_t)INT32_MAX - 2048 || (int64_t)N * H_out * W_out * (C / 4) > (int64_t)INT32_MAX)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "upsample_conv3x3_gather_adjoint: more than 2^33 elements on one side");
    const int64_t blocks = ceil_div(ceil_div(items, (int64_t)256), (int64_t)8) * 8;
    const float hscale = H_out > 1 ? (float)(H_in - 1) / (float)(H_out - 1) : 0.f;
    const float wscale = W_out > 1 ? (float)(W_in - 1) / (float)(W_out - 1) : 0.f;
    hipLaunchKernelGGL(spgt::upsample_conv3x3_gather_adjoint_k, dim3((unsigned)blocks), dim3(256), 0, stream, grad, dZ,
                       C / 4, H_in, W_in, H_out, W_out, hscale, wscale, (unsigned)items);
    return check_launch("upsample_conv3x3_gather_adjoint");
}

extern "C" int spgt_bilinear_nhwc_affine(const float* src, float* dst, int N, int C, int H_in, int W_in, int H_out,
                                         int W_out, const float* extra, const float* w_extra, int n_extra,
                                         hipStream_t stream) {
    if (!src || !dst) return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear_nhwc_affine: null pointer argument");
    if (N <= 0 || C <= 0 || H_in <= 0 || W_in <= 0 || H_out <= 0 || W_out <= 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear_nhwc_affine: sizes must be positive");
    if (C % 4 != 0) return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear_nhwc_affine: C must be a multiple of 4");
    if (n_extra < 0 || n_extra > 4 || (n_extra > 0 && (!extra || !w_extra)))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear_nhwc_affine: 0..4 extra columns, with both of their operands");
    if (!aligned16(src) || !aligned16(dst) || (n_extra > 0 && (!aligned4(extra) || !aligned16(w_extra))))
        return fail(SPGT_ERR_INVALID_ARGUMENT,
                    "bilinear_nhwc_affine: src, dst and w_extra must be 16-byte aligned, extra 4-byte aligned");
    const int64_t items = (int64_t)N * H_out * ceil_div(W_out, 4) * (C / 4);  // 4 pixels x 4 channels each
    if (items > (int64_t)INT32_MAX - 2048)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear_nhwc_affine: more than 2^35 output elements");
    const int64_t blocks = ceil_div(ceil_div(items, (int64_t)256), (int64_t)8) * 8;
    const float hscale = H_out > 1 ? (float)(H_in - 1) / (float)(H_out - 1) : 0.f;
    const float wscale = W_out > 1 ? (float)(W_in - 1) / (float)(W_out - 1) : 0.f;
    hipLaunchKernelGGL(spgt::bilinear_nhwc_affine_k, dim3((unsigned)blocks), dim3(256), 0, stream, src, dst, C / 4,
                       H_in, W_in, H_out, W_out, hscale, wscale, extra, w_extra, n_extra, (unsigned)items);
    return check_launch("bilinear_nhwc_affine");
}

extern "C" int spgt_bilinear_adjoint(const float* grad_out, float* grad_in, int N, int C, int H_in, int W_in,
                                     int H_out, int W_out, int layout, hipStream_t stream) {
    if (!grad_out || !grad_in) return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear_adjoint: null pointer argument");
    if (N <= 0 || C <= 0 || H_in <= 0 || W_in <= 0 || H_out <= 0 || W_out <= 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear_adjoint: sizes must be positive");
    if (H_in > (1 << 23) || W_in > (1 << 23) || H_out > (1 << 23) || W_out > (1 << 23))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear_adjoint: image sides above 2^23");
    const float hscale = H_out > 1 ? (float)(H_in - 1) / (float)(H_out - 1) : 0.f;
    const float wscale = W_out > 1 ? (float)(W_in - 1) / (float)(W_out - 1) : 0.f;
    if (layout == SPGT_LAYOUT_NHWC) {
        if (C % 4 != 0 || !aligned16(grad_out) || !aligned16(grad_in))
            return fail(SPGT_ERR_INVALID_ARGUMENT,
                        "bilinear_adjoint: channels-last needs C a multiple of 4 and 16-byte aligned tensors");
        const int64_t items = (int64_t)N * H_in * W_in * (C / 4);
        if (items > (int64_t)INT32_MAX - 2048 || (int64_t)N * H_out * W_out * (C / 4) > (int64_t)INT32_MAX)
            return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear_adjoint: more than 2^33 elements on one side");
        const int64_t blocks = ceil_div(ceil_div(items, (int64_t)256), (int64_t)8) * 8;
        // an up-sampling's sources are each read by three or four outputs of a row, a down-sampling's by one or two
        if (wscale < 1.f)
            hipLaunchKernelGGL(spgt::bilinear_adjoint_nhwc_k<4>, dim3((unsigned)blocks), dim3(256), 0, stream, grad_out,
                               grad_in, C / 4, H_in, W_in, H_out, W_out, hscale, wscale, (unsigned)items);
        else
            hipLaunchKernelGGL(spgt::bilinear_adjoint_nhwc_k<2>, dim3((unsigned)blocks), dim3(256), 0, stream, grad_out,
                               grad_in, C / 4, H_in, W_in, H_out, W_out, hscale, wscale, (unsigned)items);
    } else if (layout == SPGT_LAYOUT_NCHW) {
        const int64_t planes = (int64_t)N * C;
        if (planes > INT32_MAX || !aligned4(grad_out) || !aligned4(grad_in))
            return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear_adjoint: more than 2^31 planes, or misaligned tensors");
        const int xt = ceil_div(W_in, 64), yt = ceil_div(H_in, 4);
        if ((int64_t)xt * yt > (1 << 30))
            return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear_adjoint: more than 2^38 source positions per plane");
        // about 16 tiles per compute unit: a thread then walks several plane groups with one set of output ranges
        const int zb = (int)std::max<int64_t>(1, std::min<int64_t>(ceil_div(planes, (int64_t)4),
                                                                   16 * (int64_t)device_cu_count() / ((int64_t)xt * yt)));
        const unsigned blocks = (unsigned)(ceil_div((int64_t)xt * yt * zb, (int64_t)8) * 8);
        hipLaunchKernelGGL(spgt::bilinear_adjoint_planes_k, dim3(blocks), dim3(64, 4), 0, stream, grad_out, grad_in,
                           (int)planes, H_in, W_in, H_out, W_out, hscale, wscale, xt, yt, zb);
    } else {
        return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear_adjoint: layout must be NCHW or NHWC (both tensors alike)");
    }
    return check_launch("bilinear_adjoint");
}

extern "C" int spgt_bilinear_resample(const float* src, const float* pre_bias, float* dst, int N, int C, int H_in,
                                      int W_in, int H_out, int W_out, int src_layout, int dst_layout,
                                      int pre_activation, int pre_activation_count, int post_activation,
                                      hipStream_t stream) {
    if (pre_bias && !aligned4(pre_bias))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "bilinear_resample: pre_bias must be 4-byte aligned");
    return resample_common("bilinear_resample", src, pre_bias, dst, N, C, H_in, W_in, H_out, W_out, src_layout, dst_layout,
                           ResampleAct{pre_activation, pre_activation_count, post_activation}, stream);
}

namespace spgt {
namespace {

// The last two steps of the model's forward (Sp_GalerkinTransformer2D.forward, network/sp_model.py:109-111):
// out = x * scale + shift (the target normalizer's inverse, rounded after the multiply and after the add like
// the two tensor operations it stands for), then zero on the boundary of the [H, W] grid (Dirichlet condition:
// the reference pads the interior with zeros).  x, out [N, H, W, C]; scale and shift hold one value, or one per
// (h, w, c) when per_point is set.  grid (ceil(H*W*C / 256), N), block 256.
__global__ __launch_bounds__(256) void denormalize_boundary_k(const float* __restrict__ x, const float* __restrict__ scale,
                                                              const float* __restrict__ shift, int per_point,
                                                              float* __restrict__ out, int H, int W, int C,
                                                              int zero_boundary) {
    const int64_t plane = (int64_t)H * W * C;
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= plane) return;
    const int64_t i = (int64_t)blockIdx.y * plane + e;
    const int w = (int)((e / C) % W);
    const int h = (int)(e / ((int64_t)C * W));
    float v = 0.f;
    if (!zero_boundary || (h > 0 && h < H - 1 && w > 0 && w < W - 1)) {
#pragma clang fp contract(off)  // two roundings, as two tensor operations give; the default would fuse them
        const float sc = scale[per_point ? e : 0], sh = shift[per_point ? e : 0];
        const float prod = x[i] * sc;
        v = prod + sh;
    }
    out[i] = v;
}

}  // namespace
}  // namespace spgt

extern "C" int spgt_denormalize_boundary(const float* x, const float* scale, const float* shift, int per_point,
                                         float* out, int N, int H, int W, int C, int zero_boundary,
                                         hipStream_t stream) {
    if (!x || !scale || !shift || !out)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "denormalize_boundary: null pointer argument");
    if (N <= 0 || H <= 0 || W <= 0 || C <= 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "denormalize_boundary: sizes must be positive");
    if (N > 65535) return fail(SPGT_ERR_INVALID_ARGUMENT, "denormalize_boundary: N exceeds 65535");
    if (!aligned4(x) || !aligned4(scale) || !aligned4(shift) || !aligned4(out))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "denormalize_boundary: operands must be 4-byte aligned");
    const int64_t plane = (int64_t)H * W * C;
    if (ceil_div(plane, (int64_t)256) > INT32_MAX)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "denormalize_boundary: grid too large");
    hipLaunchKernelGGL(denormalize_boundary_k, dim3((unsigned)ceil_div(plane, (int64_t)256), N), dim3(256), 0, stream, x,
                       scale, shift, per_point ? 1 : 0, out, H, W, C, zero_boundary ? 1 : 0);
    return check_launch("denormalize_boundary");
}

namespace {

int bias_activation_common(float* x, const float* bias, int N, int C, int64_t HW, int activation, int activation_count,
                           spgt::DropArgs drop, hipStream_t stream) {
    if (!x) return fail(SPGT_ERR_INVALID_ARGUMENT, "bias_activation_nchw: null pointer argument");
    if (N <= 0 || C <= 0 || HW <= 0) return fail(SPGT_ERR_INVALID_ARGUMENT, "bias_activation_nchw: sizes must be positive");
    if ((int64_t)N * C > 65535) return fail(SPGT_ERR_INVALID_ARGUMENT, "bias_activation_nchw: N*C exceeds 65535");
    if (!act_known(activation) || activation_count < 0 || activation_count > 2)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "bias_activation_nchw: unknown activation or count outside 0..2");
    if (!aligned4(x) || (bias && !aligned4(bias)))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "bias_activation_nchw: operands must be 4-byte aligned");
    const int chunks = (int)std::min<int64_t>(ceil_div(HW, (int64_t)1024), 64);
    if (HW > UINT32_MAX) return fail(SPGT_ERR_INVALID_ARGUMENT, "bias_activation_nchw: planes above 2^32 elements");
    hipLaunchKernelGGL(bias_activation_nchw_k, dim3(chunks, N * C), dim3(256), 0, stream, x, bias, C, HW, activation,
                       activation == SPGT_ACT_NONE ? 0 : activation_count, drop);
    return check_launch("bias_activation_nchw");
}

}  // namespace

extern "C" int spgt_bias_activation_nchw(float* x, const float* bias, int N, int C, int64_t HW, int activation,
                                         int activation_count, hipStream_t stream) {
    return bias_activation_common(x, bias, N, C, HW, activation, activation_count, spgt::DropArgs{nullptr, 0.f}, stream);
}

extern "C" int spgt_bias_activation_nchw_dropout(float* x, const float* bias, int N, int C, int64_t HW, int activation,
                                                 int activation_count, const uint32_t* seed, float droprate,
                                                 hipStream_t stream) {
    spgt::DropArgs drop;
    if (int rc = drop_args(seed, droprate, &drop)) return rc;
    return bias_activation_common(x, bias, N, C, HW, activation, activation_count, drop, stream);
}

extern "C" int spgt_conv3x3_resample_supported(int Cin) { return (Cin >= 1 && Cin <= 4) ? 1 : 0; }

namespace {

int conv3x3_resample_common(const float* x, const float* weight, const float* bias, float* out, int N, int Cin, int Cout,
                            int H_in, int W_in, int H_out, int W_out, int pre_activation, int post_activation,
                            spgt::DropArgs drop, hipStream_t stream) {
    if (!x || !weight || !out) return fail(SPGT_ERR_INVALID_ARGUMENT, "conv3x3_resample: null pointer argument");
    if (N <= 0 || Cout <= 0 || H_in <= 0 || W_in <= 0 || H_out <= 0 || W_out <= 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "conv3x3_resample: sizes must be positive");
    if (!spgt_conv3x3_resample_supported(Cin))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "conv3x3_resample: 1 to 4 input channels");
    if (H_out > 65535 || N > 65535) return fail(SPGT_ERR_INVALID_ARGUMENT, "conv3x3_resample: N or H_out exceeds 65535");
    if (!act_known(pre_activation) || !act_known(post_activation))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "conv3x3_resample: unknown activation");
    if (!aligned4(x) || !aligned4(weight) || !aligned4(out) || (bias && !aligned4(bias)))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "conv3x3_resample: operands must be 4-byte aligned");
    const float hscale = H_out > 1 ? (float)(H_in - 1) / (float)(H_out - 1) : 0.f;
    const float wscale = W_out > 1 ? (float)(W_in - 1) / (float)(W_out - 1) : 0.f;
    const ResampleAct act{pre_activation, pre_activation == SPGT_ACT_NONE ? 0 : 1, post_activation};
    const dim3 grid(ceil_div(W_out, 64), H_out, N), block(64, 4);
    const size_t lds = (size_t)Cout * (Cin * 9 + 1) * sizeof(float);
    if (lds > 64 * 1024) return fail(SPGT_ERR_INVALID_ARGUMENT, "conv3x3_resample: too many output channels");
#define SPGT_CONV(CI)                                                                                                \
    hipLaunchKernelGGL(conv3x3_resample_k<CI>, grid, block, lds, stream, x, weight, bias, out, Cout, H_in, W_in,      \
                       H_out, W_out, hscale, wscale, act, drop)
    if ((int64_t)H_in * W_in > UINT32_MAX) return fail(SPGT_ERR_INVALID_ARGUMENT, "conv3x3_resample: planes above 2^32 samples");
    switch (Cin) {
        case 1: SPGT_CONV(1); break;
        case 2: SPGT_CONV(2); break;
        case 3: SPGT_CONV(3); break;
        default: SPGT_CONV(4); break;
    }
#undef SPGT_CONV
    return check_launch("conv3x3_resample");
}

}  // namespace

extern "C" int spgt_conv3x3_resample(const float* x, const float* weight, const float* bias, float* out, int N,
                                     int Cin, int Cout, int H_in, int W_in, int H_out, int W_out, int pre_activation,
                                     int post_activation, hipStream_t stream) {
    return conv3x3_resample_common(x, weight, bias, out, N, Cin, Cout, H_in, W_in, H_out, W_out, pre_activation,
                                   post_activation, spgt::DropArgs{nullptr, 0.f}, stream);
}

extern "C" int spgt_conv3x3_resample_dropout(const float* x, const float* weight, const float* bias, float* out, int N,
                                             int Cin, int Cout, int H_in, int W_in, int H_out, int W_out,
                                             int pre_activation, int post_activation, const uint32_t* seed,
                                             float droprate, hipStream_t stream) {
    spgt::DropArgs drop;
    if (int rc = drop_args(seed, droprate, &drop)) return rc;
    return conv3x3_resample_common(x, weight, bias, out, N, Cin, Cout, H_in, W_in, H_out, W_out, pre_activation,
                                   post_activation, drop, stream);
}

namespace {

struct ConvBackwardPlan {
    int record, rows_per_run, runs;
};

ConvBackwardPlan conv_backward_plan(int N, int Cin, int H_in) {
    ConvBackwardPlan p;
    p.record = (1 + 9 * Cin + 3) / 4 * 4;
    const int64_t rows = (int64_t)N * H_in;
    // as many runs of rows as tile_reduce sums, at least four rows (one per wave) each
    const int64_t runs = std::max<int64_t>(1, std::min<int64_t>(kReduceChains * kReduceMaxPerChain, rows / 4));
    p.rows_per_run = (int)ceil_div(rows, runs);
    p.runs = (int)ceil_div(rows, (int64_t)p.rows_per_run);
    return p;
}

}  // namespace

extern "C" size_t spgt_conv3x3_resample_backward_workspace_bytes(int N, int Cin, int Cout, int H_in, int W_in) {
    if (N <= 0 || Cout <= 0 || H_in <= 0 || W_in <= 0 || !spgt_conv3x3_resample_supported(Cin)) return 0;
    const ConvBackwardPlan p = conv_backward_plan(N, Cin, H_in);
    // the records of the runs, then the two geometry tables (16 bytes per row and per column)
    return (size_t)p.runs * Cout * p.record * sizeof(float) + ((size_t)H_in + W_in) * sizeof(float4);
}

extern "C" int spgt_conv3x3_resample_backward(const float* x, const float* weight, const float* bias, const float* grad,
                                              float* out, void* workspace, size_t workspace_bytes, int N, int Cin,
                                              int Cout, int H_in, int W_in, int H_out, int W_out, int pre_activation,
                                              const uint32_t* seed, float droprate, hipStream_t stream) {
    if (!x || !weight || !grad || !out || !workspace)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "conv3x3_resample_backward: null pointer argument");
    if (N <= 0 || Cout <= 0 || H_in <= 0 || W_in <= 0 || H_out <= 0 || W_out <= 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "conv3x3_resample_backward: sizes must be positive");
    if (!spgt_conv3x3_resample_supported(Cin))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "conv3x3_resample_backward: 1 to 4 input channels");
    if (!act_known(pre_activation)) return fail(SPGT_ERR_INVALID_ARGUMENT, "conv3x3_resample_backward: unknown activation");
    if (Cout > 65535 || (int64_t)H_in * W_in > UINT32_MAX || H_in > (1 << 23) || W_in > (1 << 23) ||
        H_out > (1 << 23) || W_out > (1 << 23))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "conv3x3_resample_backward: more than 65535 output channels or too large an image");
    spgt::DropArgs drop;
    if (int rc = drop_args(seed, droprate, &drop)) return rc;
    const size_t need = spgt_conv3x3_resample_backward_workspace_bytes(N, Cin, Cout, H_in, W_in);
    if (workspace_bytes < need || !aligned16(workspace))
        return fail(SPGT_ERR_WORKSPACE, "conv3x3_resample_backward: workspace missing, misaligned or too small");
    if (!aligned4(x) || !aligned4(weight) || !aligned4(grad) || !aligned16(out) || (bias && !aligned4(bias)))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "conv3x3_resample_backward: out must be 16-byte aligned");
    const ConvBackwardPlan p = conv_backward_plan(N, Cin, H_in);
    const int64_t E = (int64_t)Cout * p.record;
    if (E > INT32_MAX) return fail(SPGT_ERR_INVALID_ARGUMENT, "conv3x3_resample_backward: too many output channels");
    const float hscale = H_out > 1 ? (float)(H_in - 1) / (float)(H_out - 1) : 0.f;
    const float wscale = W_out > 1 ? (float)(W_in - 1) / (float)(W_out - 1) : 0.f;
    float* partial = static_cast<float*>(workspace);
    const dim3 grid(p.runs, Cout), block(64, 4);
    if (hscale >= 1.f && wscale >= 1.f) {
        // not an enlargement: at most three outputs read a source index along an axis, and their weights come from
        // two small tables made first
        float4* ytab = reinterpret_cast<float4*>(partial + (size_t)p.runs * Cout * p.record);
        float4* xtab = ytab + H_in;
        hipLaunchKernelGGL(adjoint_table_k, dim3(ceil_div(H_in, 256)), dim3(256), 0, stream, hscale, H_in, H_out, ytab);
        hipLaunchKernelGGL(adjoint_table_k, dim3(ceil_div(W_in, 256)), dim3(256), 0, stream, wscale, W_in, W_out, xtab);
#define SPGT_CONVT(CI, CGR)                                                                                          \
    hipLaunchKernelGGL((conv3x3_resample_backward_tab_k<CI, CGR>), dim3(p.runs, ceil_div(Cout, CGR)), block, 0, stream, \
                       x, weight, bias, grad, partial, N, Cout, H_in, W_in, H_out, W_out, ytab, xtab, pre_activation,   \
                       drop, p.rows_per_run)
        switch (Cin) {
            case 1: SPGT_CONVT(1, 4); break;
            case 2: SPGT_CONVT(2, 2); break;
            case 3: SPGT_CONVT(3, 2); break;
            default: SPGT_CONVT(4, 1); break;
        }
#undef SPGT_CONVT
    } else {
#define SPGT_CONVB(CI)                                                                                             \
    hipLaunchKernelGGL(conv3x3_resample_backward_k<CI>, grid, block, 0, stream, x, weight, bias, grad, partial, N, \
                       Cout, H_in, W_in, H_out, W_out, hscale, wscale, pre_activation, drop, p.rows_per_run)
        switch (Cin) {
            case 1: SPGT_CONVB(1); break;
            case 2: SPGT_CONVB(2); break;
            case 3: SPGT_CONVB(3); break;
            default: SPGT_CONVB(4); break;
        }
#undef SPGT_CONVB
    }
    hipLaunchKernelGGL(tile_reduce, dim3(ceil_div((int)E, 256), 1), dim3(1024), 0, stream, partial, out, (int)E, p.runs, 1.0f);
    return check_launch("conv3x3_resample_backward");
}

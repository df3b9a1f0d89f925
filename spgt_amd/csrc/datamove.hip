// Pure data-movement kernels of the FNO path: batched 2-D transpose, and the
// corner-window gather / scatter (with transposition) of a half spectrum.
// Every kernel copies 32-bit or 64-bit words unchanged, so results are
// bit-exact whatever the payload (NaN payloads, -0.0, ...).
//
// Reference behaviour restated here:
//   batched_transpose       extension/bind/datamove.cu:8-23,  native/datamove.cu:8-32, 92-99
//   transpose_gather_dual   extension/bind/datamove.cu:25-44, native/datamove.cu:34-61, 102-109
//   transpose_scatter_dual  extension/bind/datamove.cu:46-64, native/datamove.cu:63-89, 112-119
#include "spgt_device.h"
#include "spgt_host.h"

// complex elements a zero-fill block writes, roughly (tuned on MI355X)
#ifndef SPGT_ZERO_CHUNK
#define SPGT_ZERO_CHUNK 2048
#endif

namespace spgt {

typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef u4 u4_a4 __attribute__((aligned(4)));  // rows of odd length start at any 4-byte offset

// [batch, M, N] -> [batch, N, M], 32-bit words.  grid (8 * ceil(tiles / 8)), block 256; tiles = tiles_n * tiles_m *
// batch, the tile index running along n first.
// A 64x64 tile goes through LDS (pitch 65: conflict-free both ways).  Both global sides move 16 bytes per
// lane: a wave reads four 256-byte row pieces per instruction and writes four; tile edges fall back to words.
// Workgroups go round the eight XCDs by their index, each XCD with its own L2: workgroup 8j + x takes tile
// x * ceil(tiles / 8) + j, so the tiles that are neighbours along n run on the same XCD at about the same time.
// When N or M is odd the rows start at any 4-byte offset and a tile's 256-byte row pieces share their first and
// last cache line with the neighbouring tiles: with the neighbours on other XCDs every shared line is fetched
// twice (measured at [8, 64, 19881]: 60.5 MB read for 40.7 MB) and written in two masked parts.
__global__ __launch_bounds__(256) void batched_transpose_64(const uint32_t* __restrict__ src,
                                                            uint32_t* __restrict__ dst, int M, int N, int tiles_n,
                                                            int tiles_m, int tiles) {
    __shared__ uint32_t tile[64 * 65];
    const int per_xcd = (tiles + 7) >> 3;
    const int t = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if (t >= tiles) return;
    const int tn = t % tiles_n;
    const int tm = (t / tiles_n) % tiles_m;
    const int q = threadIdx.x & 15;  // group of four columns
    const int r = threadIdx.x >> 4;  // row within a pass of 16 rows
    const int n0 = tn * 64;
    const int m0 = tm * 64;
    const int64_t base = (int64_t)(t / (tiles_n * tiles_m)) * M * N;
    const uint32_t* s = src + base;
    uint32_t* d = dst + base;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int mr = r + 16 * i;
        const int m = m0 + mr;
        const int n = n0 + 4 * q;
        if (m < M) {
            uint32_t* t = tile + mr * 65 + 4 * q;
            const uint32_t* g = s + (int64_t)m * N + n;
            if (n + 3 < N) {
                const u4 v = *reinterpret_cast<const u4_a4*>(g);
                t[0] = v.x; t[1] = v.y; t[2] = v.z; t[3] = v.w;
            } else {
                for (int j = 0; j < 4 && n + j < N; ++j) t[j] = g[j];
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int nr = r + 16 * i;
        const int n = n0 + nr;
        const int m = m0 + 4 * q;
        if (n < N) {
            const uint32_t* t = tile + (4 * q) * 65 + nr;
            uint32_t* g = d + (int64_t)n * M + m;
            if (m + 3 < M) {
                u4 v;
                v.x = t[0]; v.y = t[65]; v.z = t[130]; v.w = t[195];
                *reinterpret_cast<u4_a4*>(g) = v;
            } else {
                for (int j = 0; j < 4 && m + j < M; ++j) g[j] = t[65 * j];
            }
        }
    }
}

struct Windows {
    int h_base[2];
    int w_base[2];
};

// src [dim, H_all, W_all] (64-bit words) -> out_k [H_low, W_low, dim] for the two windows.
// grid (ceil(dim/64), H_low, 2), block 256: a block moves 64 values of `dim` for one window row.
__global__ __launch_bounds__(256) void transpose_gather_dual_k(const uint64_t* __restrict__ src,
                                                               uint64_t* __restrict__ out1,
                                                               uint64_t* __restrict__ out2, int dim, int H_all,
                                                               int W_all, int H_low, int W_low, Windows win) {
    extern __shared__ uint64_t gtile[];  // [W_low][65]
    const int d0 = blockIdx.x * 64;
    const int h = blockIdx.y;
    const int k = blockIdx.z;
    uint64_t* out = k == 0 ? out1 : out2;
    const int64_t plane = (int64_t)H_all * W_all;
    const uint64_t* row = src + (int64_t)(win.h_base[k] + h) * W_all + win.w_base[k];
    // read: consecutive threads walk along w (contiguous in src), then along dim
    for (int e = threadIdx.x; e < 64 * W_low; e += 256) {
        const int w = e % W_low;
        const int dd = e / W_low;
        if (d0 + dd < dim) gtile[w * 65 + dd] = row[(int64_t)(d0 + dd) * plane + w];
    }
    __syncthreads();
    // write: consecutive threads walk along dim (contiguous in out)
    for (int e = threadIdx.x; e < 64 * W_low; e += 256) {
        const int dd = e & 63;
        const int w = e >> 6;
        if (d0 + dd < dim) out[((int64_t)h * W_low + w) * dim + d0 + dd] = gtile[w * 65 + dd];
    }
}

// out [dim, H_all, W_all] (64-bit words): zero everywhere except the two windows,
// which receive src_k [H_low, W_low, dim] transposed.  Where the windows overlap the
// second one wins (the reference scatters window 1, then window 2).
// Blocks [0, nA): (group of 64 planes, window row slot): the block that owns an output row h inside a window
// writes that row of its planes: window elements through an LDS transposition, zeros elsewhere.  Blocks
// [nA, ...): zero fill of the rows outside both windows, contiguous spans of a plane with 16-byte stores.
__global__ __launch_bounds__(256) void transpose_scatter_dual_k(const uint64_t* __restrict__ src1,
                                                                const uint64_t* __restrict__ src2,
                                                                uint64_t* __restrict__ out, int dim, int H_all,
                                                                int W_all, int H_low, int W_low, Windows win,
                                                                SpecSpans spans, int nA, int chunks_per_plane) {
    extern __shared__ uint64_t stile[];  // [2][W_low][65]
    const int64_t plane = (int64_t)H_all * W_all;
    if ((int)blockIdx.x >= nA) {
        const int bz = blockIdx.x - nA;
        const int64_t p = bz / chunks_per_plane;
        zero_span_chunk(reinterpret_cast<float2*>(out), spans, p, bz - (int)p * chunks_per_plane, chunks_per_plane,
                        plane, W_all);
        return;
    }
    const int groups = ceil_div(dim, 64);
    const int d0 = ((int)blockIdx.x % groups) * 64;
    const int slot = (int)blockIdx.x / groups;
    const int k0 = slot / H_low;
    const int h = win.h_base[k0] + (slot - k0 * H_low);
    bool in_win[2];
    in_win[0] = h >= win.h_base[0] && h < win.h_base[0] + H_low;
    in_win[1] = h >= win.h_base[1] && h < win.h_base[1] + H_low;
    if (k0 == 1 && in_win[0]) return;  // the first window's block owns a row that lies in both
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        if (in_win[k]) {
            const uint64_t* s = (k == 0 ? src1 : src2) + (int64_t)(h - win.h_base[k]) * W_low * dim;
            uint64_t* t = stile + k * W_low * 65;
            // four loads per thread in flight at a time (a plain loop would wait for each before the next)
            const int dd = threadIdx.x & 63;
            const int ddc = min(d0 + dd, dim - 1);
            for (int w0 = threadIdx.x >> 6; w0 < W_low; w0 += 16) {
                uint64_t v[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) v[u] = s[(int64_t)min(w0 + 4 * u, W_low - 1) * dim + ddc];
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    if (w0 + 4 * u < W_low) t[(w0 + 4 * u) * 65 + dd] = v[u];
            }
        }
    }
    __syncthreads();
    // wave v writes row h of planes d0 + 16 v .. d0 + 16 v + 15, lanes along w
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    for (int qq = 0; qq < 16; ++qq) {
        const int dd = wave * 16 + qq;
        if (d0 + dd >= dim) break;
        uint64_t* orow = out + (int64_t)(d0 + dd) * plane + (int64_t)h * W_all;
        for (int w = lane; w < W_all; w += 64) {
            uint64_t v = 0;
            if (in_win[1] && w >= win.w_base[1] && w < win.w_base[1] + W_low)
                v = stile[(W_low + w - win.w_base[1]) * 65 + dd];
            else if (in_win[0] && w >= win.w_base[0] && w < win.w_base[0] + W_low)
                v = stile[(w - win.w_base[0]) * 65 + dd];
            orow[w] = v;
        }
    }
}

// One launch that refreshes many small derived tensors: block (x, y) copies elements of descriptor y.
// Elements are walked in dst order (axis 2 fastest), so writes coalesce; reads follow the source strides
// (a transposed weight is read column-wise out of the caches: these are kilobytes).
struct CopyBatch {
    spgt_copy_desc d[64];
};

__global__ __launch_bounds__(256) void strided_copy_batch_k(const CopyBatch batch) {
    const spgt_copy_desc& d = batch.d[blockIdx.y];
    const int n1 = d.size[1], n2 = d.size[2];
    const int total = d.size[0] * n1 * n2;
    const uint32_t* __restrict__ src = reinterpret_cast<const uint32_t*>(d.src);
    uint32_t* __restrict__ dst = reinterpret_cast<uint32_t*>(d.dst);
    for (int e = blockIdx.x * 256 + threadIdx.x; e < total; e += gridDim.x * 256) {
        const int i2 = e % n2;
        const int r = e / n2;
        const int i1 = r % n1;
        const int i0 = r / n1;
        dst[(int64_t)i0 * d.dst_stride[0] + (int64_t)i1 * d.dst_stride[1] + (int64_t)i2 * d.dst_stride[2]] =
            src[(int64_t)i0 * d.src_stride[0] + (int64_t)i1 * d.src_stride[1] + (int64_t)i2 * d.src_stride[2]];
    }
}

namespace {

int check_windows(const char* who, int dim, int H_all, int W_all, int H_low, int W_low, int hb1, int wb1, int hb2,
                  int wb2) {
    if (dim <= 0 || H_all <= 0 || W_all <= 0 || H_low <= 0 || W_low <= 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "transpose_gather/scatter_dual: sizes must be positive");
    if (hb1 < 0 || hb2 < 0 || wb1 < 0 || wb2 < 0 || hb1 + H_low > H_all || hb2 + H_low > H_all ||
        wb1 + W_low > W_all || wb2 + W_low > W_all)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "transpose_gather/scatter_dual: a window leaves the [H_all, W_all] plane");
    // the scatter kernel keeps two windows' rows of 64 planes in LDS (W_low * 65 * 8 bytes each) out of 160 KiB
    if ((size_t)W_low * 65 * 8 * 2 > 160 * 1024)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "transpose_gather/scatter_dual: W_low above 157 is not supported");
    if (H_all > 65535 || H_low > 65535)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "transpose_gather/scatter_dual: H_all exceeds 65535");
    (void)who;
    return SPGT_OK;
}

}  // namespace

}  // namespace spgt

using namespace spgt;

extern "C" int spgt_batched_transpose(const float* src, float* dst, int batch_count, int M, int N,
                                      hipStream_t stream) {
    if (!src || !dst) return fail(SPGT_ERR_INVALID_ARGUMENT, "batched_transpose: null pointer argument");
    if (batch_count <= 0 || M <= 0 || N <= 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "batched_transpose: batch_count, M, N must be positive");
    if (src == dst) return fail(SPGT_ERR_INVALID_ARGUMENT, "batched_transpose: in-place transposition is not supported");
    const int tiles_n = ceil_div(N, 64), tiles_m = ceil_div(M, 64);
    const int64_t tiles = (int64_t)tiles_n * tiles_m * batch_count;
    if (tiles > INT32_MAX - 8)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "batched_transpose: more than 2^31 tiles of 64 x 64");
    if (!aligned4(src) || !aligned4(dst))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "batched_transpose: operands must be 4-byte aligned");
    const dim3 grid((unsigned)(8 * ceil_div(tiles, (int64_t)8)));
    hipLaunchKernelGGL(batched_transpose_64, grid, dim3(256), 0, stream, reinterpret_cast<const uint32_t*>(src),
                       reinterpret_cast<uint32_t*>(dst), M, N, tiles_n, tiles_m, (int)tiles);
    return check_launch("batched_transpose");
}

extern "C" int spgt_transpose_gather_dual(const float* src, float* out1, float* out2, int dim, int H_all, int W_all,
                                          int H_low, int W_low, int H_base_1, int W_base_1, int H_base_2,
                                          int W_base_2, hipStream_t stream) {
    if (!src || !out1 || !out2) return fail(SPGT_ERR_INVALID_ARGUMENT, "transpose_gather_dual: null pointer argument");
    const int rc = check_windows("gather", dim, H_all, W_all, H_low, W_low, H_base_1, W_base_1, H_base_2, W_base_2);
    if (rc != SPGT_OK) return rc;
    if (!aligned8(src) || !aligned8(out1) || !aligned8(out2))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "transpose_gather_dual: complex operands must be 8-byte aligned");
    Windows win{{H_base_1, H_base_2}, {W_base_1, W_base_2}};
    const dim3 grid(ceil_div(dim, 64), H_low, 2);
    const size_t lds = (size_t)W_low * 65 * 8;
    if (lds > 64 * 1024 && !allow_dynamic_lds(reinterpret_cast<const void*>(transpose_gather_dual_k), lds))
        return fail(SPGT_ERR_LAUNCH, "transpose_gather_dual: the kernel was refused its dynamic LDS size");
    hipLaunchKernelGGL(transpose_gather_dual_k, grid, dim3(256), lds, stream,
                       reinterpret_cast<const uint64_t*>(src), reinterpret_cast<uint64_t*>(out1),
                       reinterpret_cast<uint64_t*>(out2), dim, H_all, W_all, H_low, W_low, win);
    return check_launch("transpose_gather_dual");
}

extern "C" int spgt_transpose_scatter_dual(const float* src1, const float* src2, float* out, int dim, int H_all,
                                           int W_all, int H_low, int W_low, int H_base_1, int W_base_1,
                                           int H_base_2, int W_base_2, hipStream_t stream) {
    if (!src1 || !src2 || !out) return fail(SPGT_ERR_INVALID_ARGUMENT, "transpose_scatter_dual: null pointer argument");
    const int rc = check_windows("scatter", dim, H_all, W_all, H_low, W_low, H_base_1, W_base_1, H_base_2, W_base_2);
    if (rc != SPGT_OK) return rc;
    if (!aligned8(src1) || !aligned8(src2) || !aligned8(out))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "transpose_scatter_dual: complex operands must be 8-byte aligned");
    Windows win{{H_base_1, H_base_2}, {W_base_1, W_base_2}};
    const SpecSpans spans = rows_outside_windows(H_all, H_low, H_base_1, H_base_2);
    int64_t zero_rows = 0;
    for (int i = 0; i < spans.n; ++i) zero_rows += spans.hi[i] - spans.lo[i];
    const int chunks = zero_rows == 0 ? 0 : (int)std::max<int64_t>(1, std::min<int64_t>(8, zero_rows * W_all / SPGT_ZERO_CHUNK));
    const int64_t nA = (int64_t)ceil_div(dim, 64) * 2 * H_low;
    const int64_t nB = (int64_t)dim * chunks;
    if (nA + nB >= ((int64_t)1 << 31))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "transpose_scatter_dual: too many planes for one launch");
    const size_t lds = (size_t)W_low * 65 * 8 * 2;
    if (lds > 64 * 1024 && !allow_dynamic_lds(reinterpret_cast<const void*>(transpose_scatter_dual_k), lds))
        return fail(SPGT_ERR_LAUNCH, "transpose_scatter_dual: the kernel was refused its dynamic LDS size");
    hipLaunchKernelGGL(transpose_scatter_dual_k, dim3((unsigned)(nA + nB)), dim3(256), lds, stream,
                       reinterpret_cast<const uint64_t*>(src1), reinterpret_cast<const uint64_t*>(src2),
                       reinterpret_cast<uint64_t*>(out), dim, H_all, W_all, H_low, W_low, win, spans, (int)nA,
                       std::max(1, chunks));
    return check_launch("transpose_scatter_dual");
}

extern "C" int spgt_strided_copy_batch(const spgt_copy_desc* descs, int count, hipStream_t stream) {
    if (count < 0 || (count > 0 && !descs))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "strided_copy_batch: descriptor array missing");
    for (int i = 0; i < count; ++i) {
        const spgt_copy_desc& d = descs[i];
        if (!d.src || !d.dst || !aligned4(d.src) || !aligned4(d.dst))
            return fail(SPGT_ERR_INVALID_ARGUMENT, "strided_copy_batch: null or misaligned pointer in a descriptor");
        int64_t total = 1;
        for (int a = 0; a < 3; ++a) {
            if (d.size[a] <= 0 || d.src_stride[a] < 0 || d.dst_stride[a] < 0)
                return fail(SPGT_ERR_INVALID_ARGUMENT, "strided_copy_batch: sizes must be positive, strides non-negative");
            total *= d.size[a];
        }
        if (total > (int64_t)1 << 30)
            return fail(SPGT_ERR_INVALID_ARGUMENT, "strided_copy_batch: a descriptor exceeds 2^30 elements");
    }
    for (int first = 0; first < count; first += 64) {
        const int n = std::min(64, count - first);
        CopyBatch batch;
        int64_t largest = 0;
        for (int i = 0; i < n; ++i) {
            batch.d[i] = descs[first + i];
            largest = std::max<int64_t>(largest, (int64_t)batch.d[i].size[0] * batch.d[i].size[1] * batch.d[i].size[2]);
        }
        for (int i = n; i < 64; ++i) batch.d[i] = batch.d[0];
        const int bx = (int)std::min<int64_t>(64, ceil_div(largest, (int64_t)1024));
        hipLaunchKernelGGL(strided_copy_batch_k, dim3(bx, n), dim3(256), 0, stream, batch);
    }
    return check_launch("strided_copy_batch");
}

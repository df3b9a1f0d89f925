// Batched skinny GEMM (small M, N; long K) with a deterministic two-stage
// split-K reduction, for all eight operand storage orders.
//
// Reference behaviour restated here:
//   sgemm_32x32_4x8_SplitK::sgemm_cuda   extension/native/sgemm_32x32_splitk.cu:662-705
//   batched_skinny_gemm                  extension/bind/galerkin_attention.cu:175-198
//
// Stage 1 (splitk_partial): a workgroup owns one 32x32 output tile and one
// contiguous K range.  Operand tiles are staged through LDS so that global
// reads are always along the operand's contiguous axis whatever its storage
// order; each of the 4 waves contracts a quarter of every 64-wide K step on
// the fp32 matrix cores (v_mfma_f32_32x32x2_f32) and the four wave
// accumulators are added in wave order through LDS.
// Stage 2 (splitk_reduce_store): fixed-order sum over the K ranges, alpha,
// bounds and the output storage order.
#include "spgt_device.h"
#include "spgt_host.h"

namespace spgt {

namespace {

constexpr int kKT = 64;       // K step per LDS stage
constexpr int kPitchK = 65;   // [row][k] layout, odd pitch: conflict-free column reads
constexpr int kPitchR = 32;   // [k][row] layout
constexpr int kTileFloats = 32 * kPitchK;  // 2080 >= 64*32

// Loads this thread's 8 elements of a 32(row) x 64(k) operand tile.
//   KC == true : X[row][k], k contiguous (row stride ldx); wave w takes rows 8w..8w+7, lane = k.
//   KC == false: X[k][row], row contiguous (k stride ldx); wave w takes k 16w..16w+15, lane%32 = row.
template <bool KC>
__device__ __forceinline__ void load_tile(const float* __restrict__ X, int64_t ldx, int row0, int rows,
                                          int k0, int k1, int wave, int lane, float (&reg)[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        int row, k;
        if (KC) {
            row = row0 + 8 * wave + i;
            k = k0 + lane;
        } else {
            row = row0 + (lane & 31);
            k = k0 + 16 * wave + 2 * i + (lane >> 5);
        }
        float v = 0.f;
        if (row < rows && k < k1) v = KC ? X[(int64_t)row * ldx + k] : X[(int64_t)k * ldx + row];
        reg[i] = v;
    }
}

template <bool KC>
__device__ __forceinline__ void store_tile(float* __restrict__ Xs, int wave, int lane, const float (&reg)[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        if (KC)
            Xs[(8 * wave + i) * kPitchK + lane] = reg[i];
        else
            Xs[(16 * wave + 2 * i + (lane >> 5)) * kPitchR + (lane & 31)] = reg[i];
    }
}

// Element (row = lane%32, k) of a staged tile.
template <bool KC>
__device__ __forceinline__ float read_tile(const float* __restrict__ Xs, int lane, int k) {
    return KC ? Xs[(lane & 31) * kPitchK + k] : Xs[k * kPitchR + (lane & 31)];
}

}  // namespace

// grid (tiles_m * tiles_n, nsplit, batch), block 256.
// partial[((batch * ntile + tile) * nsplit + split) * 1024 + i * 32 + j]
// DIRECT (one K range per tile, the small-K case): the tile goes straight to C (`partial` is C then), scaled by
// alpha, row-major or column-major, and no workspace is involved.
template <bool AKC, bool BKC, bool DIRECT = false>
__global__ __launch_bounds__(256) void splitk_partial(
    const float* __restrict__ A, const float* __restrict__ B, float* __restrict__ partial, int M, int N,
    int K, int64_t a_stride, int64_t b_stride, int split_len, int64_t c_stride = 0, float alpha = 1.f,
    int c_col = 0) {
    __shared__ float smem[2][2][kTileFloats];  // [buffer][A|B]
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int tiles_n = ceil_div(N, 32);
    const int tile = blockIdx.x;
    const int m0 = (tile / tiles_n) * 32;
    const int n0 = (tile % tiles_n) * 32;
    const int split = blockIdx.y;
    const int nsplit = gridDim.y;
    const int batch = blockIdx.z;
    const int kbeg = split * split_len;
    const int kend = min(K, kbeg + split_len);

    const float* Ab = A + (int64_t)batch * a_stride;
    const float* Bb = B + (int64_t)batch * b_stride;
    const int64_t lda = AKC ? K : M;
    const int64_t ldb = BKC ? K : N;

    v16f acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;

    float ra[8], rb[8];
    const int nsteps = ceil_div(kend - kbeg, kKT);
    if (nsteps > 0) {
        load_tile<AKC>(Ab, lda, m0, M, kbeg, kend, wave, lane, ra);
        load_tile<BKC>(Bb, ldb, n0, N, kbeg, kend, wave, lane, rb);
    }
    for (int step = 0; step < nsteps; ++step) {
        float* As = smem[step & 1][0];
        float* Bs = smem[step & 1][1];
        store_tile<AKC>(As, wave, lane, ra);
        store_tile<BKC>(Bs, wave, lane, rb);
        __syncthreads();
        if (step + 1 < nsteps) {
            const int kn = kbeg + (step + 1) * kKT;
            load_tile<AKC>(Ab, lda, m0, M, kn, kend, wave, lane, ra);
            load_tile<BKC>(Bb, ldb, n0, N, kn, kend, wave, lane, rb);
        }
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) {
            const int k = 16 * wave + 2 * kk + (lane >> 5);
            acc = mfma32(read_tile<AKC>(As, lane, k), read_tile<BKC>(Bs, lane, k), acc);
        }
    }
    __syncthreads();
    // Cross-wave sum in wave order.  acc[r] = C[8*(r/4) + 4*(lane/32) + r%4][lane%32].
    float* red = &smem[0][0][0];  // 4 * 1024 floats <= 2 * 2 * 2080
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int i = 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        red[wave * 1024 + i * 32 + (lane & 31)] = acc[r];
    }
    __syncthreads();
    if constexpr (DIRECT) {
        float* Cb = partial + (int64_t)batch * c_stride;
        // thread = four consecutive elements along C's contiguous axis
        const int major = threadIdx.x >> 3;       // row i (row-major C) or column j (column-major C)
        const int minor = (threadIdx.x & 7) * 4;  // first of the four columns j or rows i
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            const int i = c_col ? minor + x : major;
            const int j = c_col ? major : minor + x;
            const int e1 = i * 32 + j;
            const float v = (((red[e1] + red[1024 + e1]) + red[2048 + e1]) + red[3072 + e1]) * alpha;
            if (m0 + i < M && n0 + j < N) {
                if (c_col) Cb[(int64_t)(n0 + j) * M + m0 + i] = v;
                else Cb[(int64_t)(m0 + i) * N + n0 + j] = v;
            }
        }
        return;
    }
    float* dst = partial + (((int64_t)batch * gridDim.x + tile) * nsplit + split) * 1024;
    const int e = threadIdx.x * 4;
    const float4 w0 = *reinterpret_cast<const float4*>(red + e);
    const float4 w1 = *reinterpret_cast<const float4*>(red + 1024 + e);
    const float4 w2 = *reinterpret_cast<const float4*>(red + 2048 + e);
    const float4 w3 = *reinterpret_cast<const float4*>(red + 3072 + e);
    float4 o;
    o.x = ((w0.x + w1.x) + w2.x) + w3.x;
    o.y = ((w0.y + w1.y) + w2.y) + w3.y;
    o.z = ((w0.z + w1.z) + w2.z) + w3.z;
    o.w = ((w0.w + w1.w) + w2.w) + w3.w;
    *reinterpret_cast<float4*>(dst + e) = o;
}

// grid (ntile, batch), block 256: thread = 4 consecutive tile elements.
// Splits are summed as four interleaved chains combined in a fixed order.
template <bool CCOL>
__global__ __launch_bounds__(256) void splitk_reduce_store(
    const float* __restrict__ partial, float* __restrict__ C, int M, int N, int64_t c_stride, int nsplit,
    float alpha) {
    const int tile = blockIdx.x;
    const int batch = blockIdx.y;
    const int tiles_n = ceil_div(N, 32);
    const int m0 = (tile / tiles_n) * 32;
    const int n0 = (tile % tiles_n) * 32;
    const int e = threadIdx.x * 4;
    const float* src = partial + ((int64_t)batch * gridDim.x + tile) * nsplit * 1024 + e;
    float4 s[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) s[q] = make_float4(0.f, 0.f, 0.f, 0.f);
    int c = 0;
    for (; c + 4 <= nsplit; c += 4) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float4 v = *reinterpret_cast<const float4*>(src + (int64_t)(c + q) * 1024);
            s[q].x += v.x; s[q].y += v.y; s[q].z += v.z; s[q].w += v.w;
        }
    }
    for (int q = 0; c < nsplit; ++c, ++q) {
        const float4 v = *reinterpret_cast<const float4*>(src + (int64_t)c * 1024);
        s[q].x += v.x; s[q].y += v.y; s[q].z += v.z; s[q].w += v.w;
    }
    float r[4];
    r[0] = ((s[0].x + s[1].x) + (s[2].x + s[3].x)) * alpha;
    r[1] = ((s[0].y + s[1].y) + (s[2].y + s[3].y)) * alpha;
    r[2] = ((s[0].z + s[1].z) + (s[2].z + s[3].z)) * alpha;
    r[3] = ((s[0].w + s[1].w) + (s[2].w + s[3].w)) * alpha;
    const int i = m0 + (e >> 5);
    float* Cb = C + (int64_t)batch * c_stride;
    if (i < M) {
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            const int j = n0 + (e & 31) + x;
            if (j < N) {
                if (CCOL)
                    Cb[(int64_t)j * M + i] = r[x];
                else
                    Cb[(int64_t)i * N + j] = r[x];
            }
        }
    }
}

namespace {

struct SplitPlan {
    int split_len, nsplit, ntile;
};

// K ranges are whole 64-wide steps; their number is chosen so that the grid
// has roughly four workgroups per CU, and never leaves a range empty.
SplitPlan make_split_plan(int M, int N, int K, int batch_count) {
    SplitPlan p;
    p.ntile = ceil_div(M, 32) * ceil_div(N, 32);
    const int64_t wgs = (int64_t)p.ntile * batch_count;
    const int target = 1024;
    int want = (int)std::max<int64_t>(1, target / std::max<int64_t>(1, wgs));
    const int steps = ceil_div(K, kKT);
    want = std::min(want, steps);
    const int steps_per_split = ceil_div(steps, want);
    p.split_len = steps_per_split * kKT;
    p.nsplit = ceil_div(K, p.split_len);
    return p;
}

int launch_splitk(const float* A, const float* B, float* C, float alpha, int M, int N, int K,
                  int64_t a_stride, int64_t b_stride, int64_t c_stride, int order, int batch_count,
                  float* partial, hipStream_t stream) {
    const SplitPlan p = make_split_plan(M, N, K, batch_count);
    const bool a_kc = (order & 4) == 0;  // A row-major  -> K contiguous
    const bool b_kc = (order & 2) != 0;  // B col-major  -> K contiguous
    const bool c_col = (order & 1) != 0;
    const dim3 block(256);
    const dim3 grid(p.ntile, p.nsplit, batch_count);
#define SPGT_LAUNCH_PARTIAL(AK, BK)                                                                  \
    hipLaunchKernelGGL((splitk_partial<AK, BK>), grid, block, 0, stream, A, B, partial, M, N, K,    \
                       a_stride, b_stride, p.split_len)
    if (a_kc && b_kc) SPGT_LAUNCH_PARTIAL(true, true);
    else if (a_kc && !b_kc) SPGT_LAUNCH_PARTIAL(true, false);
    else if (!a_kc && b_kc) SPGT_LAUNCH_PARTIAL(false, true);
    else SPGT_LAUNCH_PARTIAL(false, false);
#undef SPGT_LAUNCH_PARTIAL
    const dim3 gridr(p.ntile, batch_count);
    if (c_col)
        hipLaunchKernelGGL((splitk_reduce_store<true>), gridr, block, 0, stream, partial, C, M, N, c_stride,
                           p.nsplit, alpha);
    else
        hipLaunchKernelGGL((splitk_reduce_store<false>), gridr, block, 0, stream, partial, C, M, N, c_stride,
                           p.nsplit, alpha);
    return SPGT_OK;
}

size_t splitk_partial_bytes(int M, int N, int K, int batch_count) {
    const SplitPlan p = make_split_plan(M, N, K, batch_count);
    return (size_t)batch_count * p.ntile * p.nsplit * 1024 * sizeof(float);
}

}  // namespace

}  // namespace spgt

using namespace spgt;

extern "C" size_t spgt_batched_skinny_gemm_workspace_bytes(int M, int N, int K, int batch_count) {
    if (M <= 0 || N <= 0 || K <= 0 || batch_count <= 0) return 0;
    return splitk_partial_bytes(M, N, K, batch_count);
}

extern "C" int spgt_batched_skinny_gemm(const float* A, const float* B, float* C, float alpha, int M, int N,
                                        int K, int64_t a_stride, int64_t b_stride, int64_t c_stride,
                                        int order, int batch_count, void* workspace, size_t workspace_bytes,
                                        hipStream_t stream) {
    if (!A || !B || !C) return fail(SPGT_ERR_INVALID_ARGUMENT, "batched_skinny_gemm: null pointer argument");
    if (M <= 0 || N <= 0 || K <= 0 || batch_count <= 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "batched_skinny_gemm: M, N, K, batch_count must be positive");
    if (order < 0 || order > 7) return fail(SPGT_ERR_INVALID_ARGUMENT, "batched_skinny_gemm: unknown operand order");
    if (batch_count > 65535) return fail(SPGT_ERR_INVALID_ARGUMENT, "batched_skinny_gemm: batch_count exceeds 65535");
    if (!aligned4(A) || !aligned4(B) || !aligned4(C))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "batched_skinny_gemm: operands must be 4-byte aligned");
    const size_t need = spgt_batched_skinny_gemm_workspace_bytes(M, N, K, batch_count);
    if (!workspace || workspace_bytes < need || !aligned16(workspace))
        return fail(SPGT_ERR_WORKSPACE, "batched_skinny_gemm: workspace missing, misaligned or too small");
    launch_splitk(A, B, C, alpha, M, N, K, a_stride, b_stride, c_stride, order, batch_count,
                  static_cast<float*>(workspace), stream);
    return check_launch("batched_skinny_gemm");
}

extern "C" int spgt_batched_small_k_gemm(const float* A, const float* B, float* C, float alpha, int M, int N, int K,
                                         int64_t a_stride, int64_t b_stride, int64_t c_stride, int order,
                                         int batch_count, hipStream_t stream) {
    if (!A || !B || !C) return fail(SPGT_ERR_INVALID_ARGUMENT, "batched_small_k_gemm: null pointer argument");
    if (M <= 0 || N <= 0 || K <= 0 || batch_count <= 0)
        return fail(SPGT_ERR_INVALID_ARGUMENT, "batched_small_k_gemm: M, N, K, batch_count must be positive");
    if (order < 0 || order > 7) return fail(SPGT_ERR_INVALID_ARGUMENT, "batched_small_k_gemm: unknown operand order");
    if (batch_count > 65535) return fail(SPGT_ERR_INVALID_ARGUMENT, "batched_small_k_gemm: batch_count exceeds 65535");
    if (!aligned4(A) || !aligned4(B) || !aligned4(C))
        return fail(SPGT_ERR_INVALID_ARGUMENT, "batched_small_k_gemm: operands must be 4-byte aligned");
    const int64_t ntile = (int64_t)ceil_div(M, 32) * ceil_div(N, 32);
    if (ntile >= ((int64_t)1 << 31)) return fail(SPGT_ERR_INVALID_ARGUMENT, "batched_small_k_gemm: too many tiles");
    const bool a_kc = (order & 4) == 0;
    const bool b_kc = (order & 2) != 0;
    const int c_col = order & 1;
    const dim3 grid((unsigned)ntile, 1, batch_count);
    const int split_len = ceil_div(K, kKT) * kKT;  // one K range
#define SPGT_LAUNCH_DIRECT(AK, BK)                                                                              \
    hipLaunchKernelGGL((splitk_partial<AK, BK, true>), grid, dim3(256), 0, stream, A, B, C, M, N, K, a_stride, \
                       b_stride, split_len, c_stride, alpha, c_col)
    if (a_kc && b_kc) SPGT_LAUNCH_DIRECT(true, true);
    else if (a_kc && !b_kc) SPGT_LAUNCH_DIRECT(true, false);
    else if (!a_kc && b_kc) SPGT_LAUNCH_DIRECT(false, true);
    else SPGT_LAUNCH_DIRECT(false, false);
#undef SPGT_LAUNCH_DIRECT
    return check_launch("batched_small_k_gemm");
}

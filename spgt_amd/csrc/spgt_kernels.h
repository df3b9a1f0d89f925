// Kernels shared between translation units of the library.
#pragma once
#include <hip/hip_runtime.h>

namespace spgt {

// tile_reduce sums at most kReduceChains * kReduceMaxPerChain partial tiles per output tile.
constexpr int kReduceChains = 16;
constexpr int kReduceMaxPerChain = 16;

// out[bh][e] = scale * sum_c partial[bh][c][e] in a fixed order (defined in attn_fused.hip).
// grid (ceil(E/256), BH), block 1024; E must be a multiple of 4.
__global__ void tile_reduce(const float* __restrict__ partial, float* __restrict__ out, int E, int nchunk,
                            float scale);

}  // namespace spgt

// What the grouped GEMM kernels share: the tile's slot lists in LDS and the order workgroups take tiles in.
#ifndef BM_GEMM_HPP
#define BM_GEMM_HPP

#include "bm_stream.hpp"

namespace bmk {

struct GemmLds {
    u32 col[kGemmBN];  // the tile's activation columns
    u32 slot[kGemmBN]; // and slots
};

// Workgroup b of a GEMM grid: tile and row slab. Workgroups go to the chip's eight dies in turn (b to die b % 8,
// each with its own L2), so a tile's row slabs are consecutive workgroups of one die: the tile's activation columns
// come from memory once and serve all the slabs from that L2. The grid is 8 * ceil(tiles / 8) * n_slabs workgroups.
__device__ __forceinline__ u32 tile_of_block(u32 b, u32 n_slabs) { return ((b >> 3) / n_slabs) * 8 + (b & 7); }
__device__ __forceinline__ u32 slab_of_block(u32 b, u32 n_slabs) { return (b >> 3) % n_slabs; }

} // namespace bmk

#endif // BM_GEMM_HPP

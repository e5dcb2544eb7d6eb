// 64-key bf16 tiles of the paged K / V caches, staged through registers into LDS, for the matrix-core attention
// kernels of seqmix.hip and gatedmix.hip.
#pragma once
#include "common.h"

namespace grag {

// ---- 64-key tiles of the paged K / V caches for the matrix-core attention kernels.  Thread t of the 256 owns row
// t / 4 of a tile (one key) and the 16-byte vectors (t % 4) + 4u of that row, for K and for V alike: one block-table
// lookup per thread and tile, no integer division in the tile loop (the row's position in the paged cache is kept
// as (block-table index, offset in block) and stepped by 64 keys).  Tiles are loaded into registers one tile AHEAD
// of the tile being computed, then stored row-major into LDS (row stride `stride`, a multiple of 8 elements).
struct RowCursor {
  int bi, off;  // block-table index and offset within the block of this thread's row
  int q64, r64;
  __device__ __forceinline__ void init(int key, int BS) {
    bi = key / BS;
    off = key - bi * BS;
    q64 = 64 / BS;
    r64 = 64 - q64 * BS;
  }
  __device__ __forceinline__ void advance(int BS) {
    bi += q64;
    off += r64;
    if (off >= BS) {
      off -= BS;
      ++bi;
    }
  }
};
// the cache block of the cursor's row (-1: the row lies at or past `kend`, or the table entry is out of range)
__device__ __forceinline__ int tile_block(const RowCursor& rc, const int* __restrict__ bt, int key, int kend,
                                          int nblocks, unsigned code) {
  if (key >= kend) return -1;
  const int blk = bt[rc.bi];
  return index_ok(blk, nblocks, code) ? blk : -1;
}
template <int NL>
__device__ __forceinline__ void tile_load(bf16x8_t (&reg)[NL], const bf16* __restrict__ cache, int blk, int off,
                                          int rowlen, int G, int g, int BS, int stride = -1) {
  // (stride: elements from one cached row to the next, when the rows read are the head of wider ones)
  const int r8 = rowlen >> 3;
  const bf16* row = cache + (((size_t)(blk < 0 ? 0 : blk) * G + g) * BS + off) * (stride < 0 ? rowlen : stride);
#pragma unroll
  for (int u = 0; u < NL; ++u) {
    const int c = (threadIdx.x & 3) + 4 * u;
    reg[u] = bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
    if (blk >= 0 && c < r8) reg[u] = *reinterpret_cast<const bf16x8_t*>(row + c * 8);
  }
}
template <int NL>
__device__ __forceinline__ void tile_store(const bf16x8_t (&reg)[NL], short* __restrict__ dst, int rowlen,
                                           int stride) {
  const int r8 = rowlen >> 3;
  short* row = dst + (threadIdx.x >> 2) * stride;
#pragma unroll
  for (int u = 0; u < NL; ++u) {
    const int c = (threadIdx.x & 3) + 4 * u;
    if (c < r8) *reinterpret_cast<bf16x8_t*>(row + c * 8) = reg[u];
  }
}

// V tiles are stored for the B fragment of P V: [16 groups of 4 keys][vd][4 keys] (group stride vd * 4 + 8), so a lane's
// four keys at one value dim are 8 contiguous bytes.
template <int NL>
__device__ __forceinline__ void tile_store_v4(const bf16x8_t (&reg)[NL], short* __restrict__ dst, int vd, int gstride) {
  const int r8 = vd >> 3;
  const int kk = threadIdx.x >> 2;
  short* grp = dst + (kk >> 2) * gstride + (kk & 3);
#pragma unroll
  for (int u = 0; u < NL; ++u) {
    const int c = (threadIdx.x & 3) + 4 * u;
    if (c < r8) {
#pragma unroll
      for (int e = 0; e < 8; ++e) grp[(c * 8 + e) * 4] = reg[u][e];
    }
  }
}

}  // namespace grag

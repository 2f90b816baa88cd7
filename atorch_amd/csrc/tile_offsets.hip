// Prefix of per-group tile counts, computed on the device from the group offsets: the first kernel of every
// grouped launch (quantisers and GEMMs), so that no launch needs the routing on the host.
#include "common.hpp"

namespace aamd {

// tile_off[e] = sum_{j<e} ceil(rows_j / tile); one block, any E.
__global__ __launch_bounds__(256) void group_tile_offsets_kernel(const int64_t* __restrict__ goff, int E, int tile,
                                                                 int32_t* __restrict__ tile_off) {
  __shared__ int buf[256];
  __shared__ int carry;
  if (threadIdx.x == 0) {
    carry = 0;
    tile_off[0] = 0;
  }
  __syncthreads();
  for (int base = 0; base < E; base += 256) {
    const int e = base + threadIdx.x;
    int n = 0;
    if (e < E) n = (int)((goff[e + 1] - goff[e] + tile - 1) / tile);
    buf[threadIdx.x] = n;
    __syncthreads();
    for (int d = 1; d < 256; d <<= 1) {
      int t = (int)threadIdx.x >= d ? buf[threadIdx.x - d] : 0;
      __syncthreads();
      buf[threadIdx.x] += t;
      __syncthreads();
    }
    if (e < E) tile_off[e + 1] = carry + buf[threadIdx.x];
    __syncthreads();
    if (threadIdx.x == 255) carry += buf[255];
    __syncthreads();
  }
}

int launch_group_tile_offsets(const int64_t* goff, int E, int tile, int32_t* tile_off, hipStream_t st) {
  group_tile_offsets_kernel<<<1, 256, 0, st>>>(goff, E, tile, tile_off);
  AAMD_LAUNCH_CHECK("group_tile_offsets");
  return AAMD_OK;
}

}  // namespace aamd

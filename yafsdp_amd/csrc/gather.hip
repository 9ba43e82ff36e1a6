// Instantiations and dtype dispatch of the gather-in (reduce copy-in) kernel.
#include "launch.h"
#include "tuning.h"

namespace yafsdp {
namespace {

template <class META, class S, class D, int SCALE, int BLOCK>
hipError_t go(const META& meta, void* flat, int64_t padded, int n_tiles, float k, int pad_zero, int wt_from, int grid,
              hipStream_t stream) {
  return launch_kernel(gather_in_kernel<META, S, D, SCALE, BLOCK, kGatherUnroll, kTableNtLoad, kGatherStorePolicy>, grid,
                       BLOCK, stream, meta, flat, padded, n_tiles, k, pad_zero, wt_from);
}

template <class META, class S, class D, int SCALE>
hipError_t by_block(int block, const META& meta, void* flat, int64_t padded, int n_tiles, float k, int pad_zero,
                    int wt_from, int grid, hipStream_t stream) {
  if (block == kTableBlockSmall) return go<META, S, D, SCALE, kTableBlockSmall>(meta, flat, padded, n_tiles, k, pad_zero, wt_from, grid, stream);
  if (block == kTableBlockLarge) return go<META, S, D, SCALE, kTableBlockLarge>(meta, flat, padded, n_tiles, k, pad_zero, wt_from, grid, stream);
  return hipErrorInvalidValue;
}

template <class META, class S, class D>
hipError_t by_scale(int block, int scale, const META& meta, void* flat, int64_t padded, int n_tiles, float k,
                    int pad_zero, int wt_from, int grid, hipStream_t stream) {
  switch (scale) {
    case SCALE_NONE: return by_block<META, S, D, SCALE_NONE>(block, meta, flat, padded, n_tiles, k, pad_zero, wt_from, grid, stream);
    case SCALE_MUL: return by_block<META, S, D, SCALE_MUL>(block, meta, flat, padded, n_tiles, k, pad_zero, wt_from, grid, stream);
    case SCALE_DIV: return by_block<META, S, D, SCALE_DIV>(block, meta, flat, padded, n_tiles, k, pad_zero, wt_from, grid, stream);
  }
  return hipErrorInvalidValue;
}

template <class META, class S>
hipError_t by_flat(int block, int flat_dt, int scale, const META& meta, void* flat, int64_t padded, int n_tiles,
                   float k, int pad_zero, int wt_from, int grid, hipStream_t stream) {
  switch (flat_dt) {
    case DT_F32: return by_scale<META, S, F32>(block, scale, meta, flat, padded, n_tiles, k, pad_zero, wt_from, grid, stream);
    case DT_BF16: return by_scale<META, S, BF16>(block, scale, meta, flat, padded, n_tiles, k, pad_zero, wt_from, grid, stream);
    case DT_F16: return by_scale<META, S, F16>(block, scale, meta, flat, padded, n_tiles, k, pad_zero, wt_from, grid, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace

template <class META>
hipError_t launch_gather(int block, int tensor_dt, int flat_dt, int scale, const META& meta, void* flat,
                         int64_t padded, int n_tiles, float k, int pad_zero, int wt_from, int grid, hipStream_t stream) {
  // the kernel looks its first tile up before it tests the tile count: every workgroup must own a tile
  if (n_tiles < 1 || grid < 1 || grid > n_tiles) return hipErrorInvalidValue;
  switch (tensor_dt) {
    case DT_F32: return by_flat<META, F32>(block, flat_dt, scale, meta, flat, padded, n_tiles, k, pad_zero, wt_from, grid, stream);
    case DT_BF16: return by_flat<META, BF16>(block, flat_dt, scale, meta, flat, padded, n_tiles, k, pad_zero, wt_from, grid, stream);
    case DT_F16: return by_flat<META, F16>(block, flat_dt, scale, meta, flat, padded, n_tiles, k, pad_zero, wt_from, grid, stream);
  }
  return hipErrorInvalidValue;
}

template hipError_t launch_gather<SmallMeta>(int, int, int, int, const SmallMeta&, void*, int64_t, int, float, int,
                                             int, int, hipStream_t);
template hipError_t launch_gather<LargeMeta>(int, int, int, int, const LargeMeta&, void*, int64_t, int, float, int,
                                             int, int, hipStream_t);

}  // namespace yafsdp

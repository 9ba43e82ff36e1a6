// Instantiations and dtype dispatch of the scatter-out (copy-out) kernel.
#include "launch.h"
#include "tuning.h"

namespace yafsdp {
namespace {

template <class META, class S, class D, int BLOCK, int U>
hipError_t go(const META& meta, const void* flat, int64_t total, int n_tiles, int wt_from, int grid, hipStream_t stream) {
  return launch_kernel(scatter_out_kernel<META, S, D, BLOCK, U, kTableNtLoad, kScatterStorePolicy>, grid, BLOCK,
                       stream, meta, flat, total, n_tiles, wt_from);
}

// `block` packs the shape the table was built for: workgroup size * 16 + units per lane
template <class META, class S, class D>
hipError_t by_block(int block, const META& meta, const void* flat, int64_t total, int n_tiles, int wt_from, int grid,
                    hipStream_t stream) {
  const int wg = block >> 4, unroll = block & 15;
  if (wg == kTableBlockSmall && unroll == kScatterShortUnroll)
    return go<META, S, D, kTableBlockSmall, kScatterShortUnroll>(meta, flat, total, n_tiles, wt_from, grid, stream);
  if (wg == kTableBlockSmall && unroll == kGatherUnroll)
    return go<META, S, D, kTableBlockSmall, kGatherUnroll>(meta, flat, total, n_tiles, wt_from, grid, stream);
  if (wg == kTableBlockLarge && unroll == kGatherUnroll)
    return go<META, S, D, kTableBlockLarge, kGatherUnroll>(meta, flat, total, n_tiles, wt_from, grid, stream);
  return hipErrorInvalidValue;
}

template <class META, class S>
hipError_t by_tensor(int block, int tensor_dt, const META& meta, const void* flat, int64_t total, int n_tiles,
                     int wt_from, int grid, hipStream_t stream) {
  switch (tensor_dt) {
    case DT_F32: return by_block<META, S, F32>(block, meta, flat, total, n_tiles, wt_from, grid, stream);
    case DT_BF16: return by_block<META, S, BF16>(block, meta, flat, total, n_tiles, wt_from, grid, stream);
    case DT_F16: return by_block<META, S, F16>(block, meta, flat, total, n_tiles, wt_from, grid, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace

template <class META>
hipError_t launch_scatter(int block, int flat_dt, int tensor_dt, const META& meta, const void* flat, int64_t total,
                          int n_tiles, int wt_from, int grid, hipStream_t stream) {
  switch (flat_dt) {
    case DT_F32: return by_tensor<META, F32>(block, tensor_dt, meta, flat, total, n_tiles, wt_from, grid, stream);
    case DT_BF16: return by_tensor<META, BF16>(block, tensor_dt, meta, flat, total, n_tiles, wt_from, grid, stream);
    case DT_F16: return by_tensor<META, F16>(block, tensor_dt, meta, flat, total, n_tiles, wt_from, grid, stream);
  }
  return hipErrorInvalidValue;
}

template hipError_t launch_scatter<SmallMeta>(int, int, int, const SmallMeta&, const void*, int64_t, int, int, int,
                                              hipStream_t);
template hipError_t launch_scatter<LargeMeta>(int, int, int, const LargeMeta&, const void*, int64_t, int, int, int,
                                              hipStream_t);

}  // namespace yafsdp

// Instantiations and dtype dispatch of the gather-in (reduce copy-in) kernel.
#include "launch.h"
#include "tuning.h"

namespace yafsdp {
namespace {

template <class S, class D, int SCALE>
hipError_t go(const TableView& tv, const DynArgs& dyn, void* flat, float k, int pad_zero, int grid,
              hipStream_t stream) {
  gather_in_kernel<S, D, SCALE, kTableBlock, kTableUnroll, kTableNtLoad, kTableNtStore>
      <<<dim3(grid), dim3(kTableBlock), 0, stream>>>(tv, dyn, flat, k, pad_zero);
  return hipGetLastError();
}

template <class S, class D>
hipError_t by_scale(int scale, const TableView& tv, const DynArgs& dyn, void* flat, float k, int pad_zero, int grid,
                    hipStream_t stream) {
  switch (scale) {
    case SCALE_NONE: return go<S, D, SCALE_NONE>(tv, dyn, flat, k, pad_zero, grid, stream);
    case SCALE_MUL: return go<S, D, SCALE_MUL>(tv, dyn, flat, k, pad_zero, grid, stream);
    case SCALE_DIV: return go<S, D, SCALE_DIV>(tv, dyn, flat, k, pad_zero, grid, stream);
  }
  return hipErrorInvalidValue;
}

template <class S>
hipError_t by_flat(int flat_dt, int scale, const TableView& tv, const DynArgs& dyn, void* flat, float k, int pad_zero,
                   int grid, hipStream_t stream) {
  switch (flat_dt) {
    case DT_F32: return by_scale<S, F32>(scale, tv, dyn, flat, k, pad_zero, grid, stream);
    case DT_BF16: return by_scale<S, BF16>(scale, tv, dyn, flat, k, pad_zero, grid, stream);
    case DT_F16: return by_scale<S, F16>(scale, tv, dyn, flat, k, pad_zero, grid, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace

hipError_t launch_gather(int tensor_dt, int flat_dt, int scale, const TableView& tv, const DynArgs& dyn, void* flat,
                         float k, int pad_zero, int grid, hipStream_t stream) {
  switch (tensor_dt) {
    case DT_F32: return by_flat<F32>(flat_dt, scale, tv, dyn, flat, k, pad_zero, grid, stream);
    case DT_BF16: return by_flat<BF16>(flat_dt, scale, tv, dyn, flat, k, pad_zero, grid, stream);
    case DT_F16: return by_flat<F16>(flat_dt, scale, tv, dyn, flat, k, pad_zero, grid, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace yafsdp

// Instantiations and dtype dispatch of the scatter-out (copy-out) kernel.
#include "launch.h"
#include "tuning.h"

namespace yafsdp {
namespace {

template <class S, class D>
hipError_t go(const TableView& tv, const DynArgs& dyn, const void* flat, int grid, hipStream_t stream) {
  scatter_out_kernel<S, D, kTableBlock, kTableUnroll, kTableNtLoad, kTableNtStore>
      <<<dim3(grid), dim3(kTableBlock), 0, stream>>>(tv, dyn, flat);
  return hipGetLastError();
}

template <class S>
hipError_t by_tensor(int tensor_dt, const TableView& tv, const DynArgs& dyn, const void* flat, int grid,
                     hipStream_t stream) {
  switch (tensor_dt) {
    case DT_F32: return go<S, F32>(tv, dyn, flat, grid, stream);
    case DT_BF16: return go<S, BF16>(tv, dyn, flat, grid, stream);
    case DT_F16: return go<S, F16>(tv, dyn, flat, grid, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace

hipError_t launch_scatter(int flat_dt, int tensor_dt, const TableView& tv, const DynArgs& dyn, const void* flat,
                          int grid, hipStream_t stream) {
  switch (flat_dt) {
    case DT_F32: return by_tensor<F32>(tensor_dt, tv, dyn, flat, grid, stream);
    case DT_BF16: return by_tensor<BF16>(tensor_dt, tv, dyn, flat, grid, stream);
    case DT_F16: return by_tensor<F16>(tensor_dt, tv, dyn, flat, grid, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace yafsdp

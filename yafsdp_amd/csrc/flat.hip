// Instantiations and dtype dispatch of the flat kernels.
#include "launch.h"
#include "tuning.h"

namespace yafsdp {
namespace {

template <class S, class D, int SCALE, bool ACC>
hipError_t go(void* dst, const void* src, int64_t n, int head, float k, int wt_from, int grid, hipStream_t stream) {
  // an armed timeline buffer is consumed by this launch if it is large enough for the grid
  TimedLaunch& t = tl_timed_launch;
  unsigned long long* trace = nullptr;
  if (t.trace != nullptr) {
    if (int64_t(grid) <= t.trace_capacity) {
      trace = t.trace;
      if (t.trace_workgroups != nullptr) *t.trace_workgroups = grid;
    } else if (t.trace_workgroups != nullptr) {
      *t.trace_workgroups = -int64_t(grid);  // not traced: the buffer is too small for this many workgroups
    }
    t.trace = nullptr;
    t.trace_capacity = 0;
    t.trace_workgroups = nullptr;
  }
  return launch_kernel(flat_kernel<S, D, SCALE, ACC, kFlatBlock, kFlatUnroll, kFlatNtLoad, kFlatStorePolicy>, grid,
                       kFlatBlock, stream, dst, src, n, head, k, trace, wt_from);
}

template <class S, class D>
hipError_t by_op(int scale, bool acc, void* dst, const void* src, int64_t n, int head, float k, int wt_from,
                 int grid, hipStream_t stream) {
  switch (scale * 2 + (acc ? 1 : 0)) {
    case 0: return go<S, D, SCALE_NONE, false>(dst, src, n, head, k, wt_from, grid, stream);
    case 1: return go<S, D, SCALE_NONE, true>(dst, src, n, head, k, wt_from, grid, stream);
    case 2: return go<S, D, SCALE_MUL, false>(dst, src, n, head, k, wt_from, grid, stream);
    case 3: return go<S, D, SCALE_MUL, true>(dst, src, n, head, k, wt_from, grid, stream);
    case 4: return go<S, D, SCALE_DIV, false>(dst, src, n, head, k, wt_from, grid, stream);
    case 5: return go<S, D, SCALE_DIV, true>(dst, src, n, head, k, wt_from, grid, stream);
  }
  return hipErrorInvalidValue;
}

template <class S>
hipError_t by_dst(int dst_dt, int scale, bool acc, void* dst, const void* src, int64_t n, int head, float k,
                  int wt_from, int grid, hipStream_t stream) {
  switch (dst_dt) {
    case DT_F32: return by_op<S, F32>(scale, acc, dst, src, n, head, k, wt_from, grid, stream);
    case DT_BF16: return by_op<S, BF16>(scale, acc, dst, src, n, head, k, wt_from, grid, stream);
    case DT_F16: return by_op<S, F16>(scale, acc, dst, src, n, head, k, wt_from, grid, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace

hipError_t launch_flat(int src_dt, int dst_dt, int scale, bool acc, void* dst, const void* src, int64_t n, int head,
                       float k, int wt_from, int grid, hipStream_t stream) {
  switch (src_dt) {
    case DT_F32: return by_dst<F32>(dst_dt, scale, acc, dst, src, n, head, k, wt_from, grid, stream);
    case DT_BF16: return by_dst<BF16>(dst_dt, scale, acc, dst, src, n, head, k, wt_from, grid, stream);
    case DT_F16: return by_dst<F16>(dst_dt, scale, acc, dst, src, n, head, k, wt_from, grid, stream);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_bytes(void* dst, const void* src, int64_t n, int head, int wt_from, int grid, hipStream_t stream) {
  return launch_kernel(bytes_kernel<kFlatBlock, kFlatNtLoad, kFlatStorePolicy>, grid, kFlatBlock, stream, dst, src, n,
                       head, wt_from);
}

}  // namespace yafsdp

// Instantiations and dtype dispatch of the fan-out / fan-in kernels.
#include "fan_kernels.hip.h"
#include "launch.h"
#include "tuning.h"

namespace yafsdp {
namespace {

template <class S, class D>
hipError_t fanout_go(const FanPtrs& dsts, const void* src, int64_t n, int grid, hipStream_t stream) {
  return launch_kernel(fanout_kernel<S, D, kFanOutBlock, kFanOutUnroll, kOptNtLoad, kFanOutStorePolicy>, grid, kFanOutBlock, stream,
                       dsts, src, n);
}

template <class S>
hipError_t fanout_by_dst(int dst_dt, const FanPtrs& dsts, const void* src, int64_t n, int grid, hipStream_t stream) {
  switch (dst_dt) {
    case DT_F32: return fanout_go<S, F32>(dsts, src, n, grid, stream);
    case DT_BF16: return fanout_go<S, BF16>(dsts, src, n, grid, stream);
    case DT_F16: return fanout_go<S, F16>(dsts, src, n, grid, stream);
  }
  return hipErrorInvalidValue;
}

template <class S, class D, int SCALE, bool ACC>
hipError_t fanin_go(void* shard, const FanPtrs& chunks, int64_t n, float k, int grid, hipStream_t stream) {
  return launch_kernel(fanin_kernel<S, D, SCALE, ACC, kFanInBlock, kFanInUnroll, kOptNtLoad, kOptNtStore>, grid, kFanInBlock,
                       stream, shard, chunks, n, k);
}

template <class S, class D>
hipError_t fanin_by_op(int scale, bool acc, void* shard, const FanPtrs& chunks, int64_t n, float k, int grid,
                       hipStream_t stream) {
  switch (scale * 2 + (acc ? 1 : 0)) {
    case 0: return fanin_go<S, D, SCALE_NONE, false>(shard, chunks, n, k, grid, stream);
    case 1: return fanin_go<S, D, SCALE_NONE, true>(shard, chunks, n, k, grid, stream);
    case 2: return fanin_go<S, D, SCALE_MUL, false>(shard, chunks, n, k, grid, stream);
    case 3: return fanin_go<S, D, SCALE_MUL, true>(shard, chunks, n, k, grid, stream);
    case 4: return fanin_go<S, D, SCALE_DIV, false>(shard, chunks, n, k, grid, stream);
    case 5: return fanin_go<S, D, SCALE_DIV, true>(shard, chunks, n, k, grid, stream);
    case 6: return fanin_go<S, D, SCALE_PREMUL, false>(shard, chunks, n, k, grid, stream);
    case 7: return fanin_go<S, D, SCALE_PREMUL, true>(shard, chunks, n, k, grid, stream);
  }
  return hipErrorInvalidValue;
}

template <class S>
hipError_t fanin_by_dst(int dst_dt, int scale, bool acc, void* shard, const FanPtrs& chunks, int64_t n, float k,
                        int grid, hipStream_t stream) {
  switch (dst_dt) {
    case DT_F32: return fanin_by_op<S, F32>(scale, acc, shard, chunks, n, k, grid, stream);
    case DT_BF16: return fanin_by_op<S, BF16>(scale, acc, shard, chunks, n, k, grid, stream);
    case DT_F16: return fanin_by_op<S, F16>(scale, acc, shard, chunks, n, k, grid, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace

hipError_t launch_fanout(int src_dt, int dst_dt, const FanPtrs& dsts, const void* src, int64_t n, int grid,
                         hipStream_t stream) {
  switch (src_dt) {
    case DT_F32: return fanout_by_dst<F32>(dst_dt, dsts, src, n, grid, stream);
    case DT_BF16: return fanout_by_dst<BF16>(dst_dt, dsts, src, n, grid, stream);
    case DT_F16: return fanout_by_dst<F16>(dst_dt, dsts, src, n, grid, stream);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_fanin(int chunk_dt, int shard_dt, int scale, bool acc, void* shard, const FanPtrs& chunks, int64_t n,
                        float k, int grid, hipStream_t stream) {
  switch (chunk_dt) {
    case DT_F32: return fanin_by_dst<F32>(shard_dt, scale, acc, shard, chunks, n, k, grid, stream);
    case DT_BF16: return fanin_by_dst<BF16>(shard_dt, scale, acc, shard, chunks, n, k, grid, stream);
    case DT_F16: return fanin_by_dst<F16>(shard_dt, scale, acc, shard, chunks, n, k, grid, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace yafsdp

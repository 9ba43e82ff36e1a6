// Instantiations and dtype dispatch of the two fused launches (fused_kernels.hip.h).
#include "fused_kernels.hip.h"
#include "launch.h"
#include "tuning.h"

namespace yafsdp {
namespace {

// ---- copy-in + copy-out -----------------------------------------------------------------------------------------
template <class M, class P, int US>
hipError_t unshard_go(const SmallMeta& meta, const void* gathered, int n_slots, void* ag_in, const void* master,
                      int64_t n, int head, int n_flat_blocks, int grid, hipStream_t stream) {
  return launch_kernel(unshard_kernel<M, P, kTableBlockSmall, kFusedFlatUnroll, US, kTableNtLoad, kFlatStorePolicy,
                                      kScatterStorePolicy>,
                       grid, kTableBlockSmall, stream, meta, gathered, n_slots, ag_in, master, n, head, n_flat_blocks);
}

template <class M, class P>
hipError_t unshard_by_shape(int scatter_unroll, const SmallMeta& meta, const void* gathered, int n_slots, void* ag_in,
                            const void* master, int64_t n, int head, int n_flat_blocks, int grid, hipStream_t stream) {
  if (scatter_unroll == kScatterShortUnroll)
    return unshard_go<M, P, kScatterShortUnroll>(meta, gathered, n_slots, ag_in, master, n, head, n_flat_blocks, grid, stream);
  if (scatter_unroll == kGatherUnroll)
    return unshard_go<M, P, kGatherUnroll>(meta, gathered, n_slots, ag_in, master, n, head, n_flat_blocks, grid, stream);
  return hipErrorInvalidValue;
}

template <class M>
hipError_t unshard_by_param(int p_dt, int scatter_unroll, const SmallMeta& meta, const void* gathered, int n_slots,
                            void* ag_in, const void* master, int64_t n, int head, int n_flat_blocks, int grid,
                            hipStream_t stream) {
  switch (p_dt) {
    case DT_F32: return unshard_by_shape<M, F32>(scatter_unroll, meta, gathered, n_slots, ag_in, master, n, head, n_flat_blocks, grid, stream);
    case DT_BF16: return unshard_by_shape<M, BF16>(scatter_unroll, meta, gathered, n_slots, ag_in, master, n, head, n_flat_blocks, grid, stream);
    case DT_F16: return unshard_by_shape<M, F16>(scatter_unroll, meta, gathered, n_slots, ag_in, master, n, head, n_flat_blocks, grid, stream);
  }
  return hipErrorInvalidValue;
}

// ---- reduce copy-in + post-reduce -------------------------------------------------------------------------------
template <class S, class D, class O>
hipError_t gp_go(int block, const SmallMeta& meta, void* flat, void* shard, int64_t padded, int n_tiles, int pad_zero,
                 int acc, int grid, hipStream_t stream) {
  if (block == kTableBlockSmall)
    return launch_kernel(gather_post_kernel<S, D, O, kTableBlockSmall, kGatherUnroll, kTableNtLoad>, grid,
                         kTableBlockSmall, stream, meta, flat, shard, padded, n_tiles, pad_zero, acc);
  if (block == kTableBlockLarge)
    return launch_kernel(gather_post_kernel<S, D, O, kTableBlockLarge, kGatherUnroll, kTableNtLoad>, grid,
                         kTableBlockLarge, stream, meta, flat, shard, padded, n_tiles, pad_zero, acc);
  return hipErrorInvalidValue;
}

template <class S, class D>
hipError_t gp_by_shard(int o_dt, int block, const SmallMeta& meta, void* flat, void* shard, int64_t padded,
                       int n_tiles, int pad_zero, int acc, int grid, hipStream_t stream) {
  switch (o_dt) {
    case DT_F32: return gp_go<S, D, F32>(block, meta, flat, shard, padded, n_tiles, pad_zero, acc, grid, stream);
    case DT_BF16: return gp_go<S, D, BF16>(block, meta, flat, shard, padded, n_tiles, pad_zero, acc, grid, stream);
    case DT_F16: return gp_go<S, D, F16>(block, meta, flat, shard, padded, n_tiles, pad_zero, acc, grid, stream);
  }
  return hipErrorInvalidValue;
}

template <class S>
hipError_t gp_by_flat(int d_dt, int o_dt, int block, const SmallMeta& meta, void* flat, void* shard, int64_t padded,
                      int n_tiles, int pad_zero, int acc, int grid, hipStream_t stream) {
  // the reduce buffer has the gradients' dtype or binary32 (reduce_dtype=float32)
  if (d_dt == S::kId) return gp_by_shard<S, S>(o_dt, block, meta, flat, shard, padded, n_tiles, pad_zero, acc, grid, stream);
  if (d_dt == DT_F32) return gp_by_shard<S, F32>(o_dt, block, meta, flat, shard, padded, n_tiles, pad_zero, acc, grid, stream);
  return hipErrorInvalidValue;
}

}  // namespace

bool fused_reduce_supports(int tensor_dt, int flat_dt) { return flat_dt == tensor_dt || flat_dt == DT_F32; }

hipError_t launch_unshard(int scatter_unroll, int master_dt, int param_dt, const SmallMeta& meta, const void* gathered,
                          int n_slots, void* ag_in, const void* master, int64_t n, int head, int n_flat_blocks,
                          int grid, hipStream_t stream) {
  switch (master_dt) {
    case DT_F32: return unshard_by_param<F32>(param_dt, scatter_unroll, meta, gathered, n_slots, ag_in, master, n, head, n_flat_blocks, grid, stream);
    case DT_BF16: return unshard_by_param<BF16>(param_dt, scatter_unroll, meta, gathered, n_slots, ag_in, master, n, head, n_flat_blocks, grid, stream);
    case DT_F16: return unshard_by_param<F16>(param_dt, scatter_unroll, meta, gathered, n_slots, ag_in, master, n, head, n_flat_blocks, grid, stream);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_gather_post(int block, int tensor_dt, int flat_dt, int shard_dt, const SmallMeta& meta, void* flat,
                              void* shard, int64_t padded, int n_tiles, int pad_zero, int acc, int grid,
                              hipStream_t stream) {
  switch (tensor_dt) {
    case DT_F32: return gp_by_flat<F32>(flat_dt, shard_dt, block, meta, flat, shard, padded, n_tiles, pad_zero, acc, grid, stream);
    case DT_BF16: return gp_by_flat<BF16>(flat_dt, shard_dt, block, meta, flat, shard, padded, n_tiles, pad_zero, acc, grid, stream);
    case DT_F16: return gp_by_flat<F16>(flat_dt, shard_dt, block, meta, flat, shard, padded, n_tiles, pad_zero, acc, grid, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace yafsdp

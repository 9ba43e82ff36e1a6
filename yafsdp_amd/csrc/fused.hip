// Instantiations and dtype dispatch of the two fused launches (fused_kernels.hip.h).
#include "fused_kernels.hip.h"
#include "launch.h"
#include "tuning.h"

namespace yafsdp {
namespace {

// ---- copy-in + copy-out -----------------------------------------------------------------------------------------
template <class META, class M, class P, int BLOCK, int US>
hipError_t unshard_go(const META& meta, const void* gathered, int n_slots, int wt_from, void* ag_in, const void* master, int64_t n,
                      int head, int n_flat_blocks, int flat_wt_from, int grid, hipStream_t stream) {
  return launch_kernel(unshard_kernel<META, M, P, BLOCK, kFusedFlatUnroll, US, kTableNtLoad, kFlatStorePolicy,
                                      kScatterStorePolicy>,
                       grid, BLOCK, stream, meta, gathered, n_slots, wt_from, ag_in, master, n, head, n_flat_blocks, flat_wt_from);
}

// the three scatter-out shapes a table can have (scatter_shape_for)
template <class META, class M, class P>
hipError_t unshard_by_shape(int shape, const META& meta, const void* gathered, int n_slots, int wt_from, void* ag_in,
                            const void* master, int64_t n, int head, int n_flat_blocks, int flat_wt_from, int grid, hipStream_t stream) {
  if (shape == kTableBlockSmall * 16 + kScatterShortUnroll)
    return unshard_go<META, M, P, kTableBlockSmall, kScatterShortUnroll>(meta, gathered, n_slots, wt_from, ag_in, master, n, head, n_flat_blocks, flat_wt_from, grid, stream);
  if (shape == kTableBlockSmall * 16 + kGatherUnroll)
    return unshard_go<META, M, P, kTableBlockSmall, kGatherUnroll>(meta, gathered, n_slots, wt_from, ag_in, master, n, head, n_flat_blocks, flat_wt_from, grid, stream);
  if (shape == kTableBlockLarge * 16 + kGatherUnroll)
    return unshard_go<META, M, P, kTableBlockLarge, kGatherUnroll>(meta, gathered, n_slots, wt_from, ag_in, master, n, head, n_flat_blocks, flat_wt_from, grid, stream);
  return hipErrorInvalidValue;
}

template <class META, class M>
hipError_t unshard_by_param(int p_dt, int shape, const META& meta, const void* gathered, int n_slots, int wt_from, void* ag_in,
                            const void* master, int64_t n, int head, int n_flat_blocks, int flat_wt_from, int grid, hipStream_t stream) {
  switch (p_dt) {
    case DT_F32: return unshard_by_shape<META, M, F32>(shape, meta, gathered, n_slots, wt_from, ag_in, master, n, head, n_flat_blocks, flat_wt_from, grid, stream);
    case DT_BF16: return unshard_by_shape<META, M, BF16>(shape, meta, gathered, n_slots, wt_from, ag_in, master, n, head, n_flat_blocks, flat_wt_from, grid, stream);
    case DT_F16: return unshard_by_shape<META, M, F16>(shape, meta, gathered, n_slots, wt_from, ag_in, master, n, head, n_flat_blocks, flat_wt_from, grid, stream);
  }
  return hipErrorInvalidValue;
}

// ---- reduce copy-in + post-reduce -------------------------------------------------------------------------------
template <class META, class S, class D, class O, bool DIV>
hipError_t gp_launch(int block, const META& meta, void* flat, void* shard, int64_t padded, int n_tiles, int pad_zero,
                     int acc, const ReduceDivides& dv, int grid, hipStream_t stream) {
  if (block == kTableBlockSmall)
    return launch_kernel(gather_post_kernel<META, S, D, O, DIV, kTableBlockSmall, kGatherUnroll, kTableNtLoad>, grid,
                         kTableBlockSmall, stream, meta, flat, shard, padded, n_tiles, pad_zero, acc, dv);
  if (block == kTableBlockLarge)
    return launch_kernel(gather_post_kernel<META, S, D, O, DIV, kTableBlockLarge, kGatherUnroll, kTableNtLoad>, grid,
                         kTableBlockLarge, stream, meta, flat, shard, padded, n_tiles, pad_zero, acc, dv);
  return hipErrorInvalidValue;
}

template <class META, class S, class D, class O>
hipError_t gp_go(int block, const META& meta, void* flat, void* shard, int64_t padded, int n_tiles, int pad_zero,
                 int acc, const ReduceDivides& dv, int grid, hipStream_t stream) {
  if (dv.a_mode == SCALE_NONE && dv.b_mode == SCALE_NONE)
    return gp_launch<META, S, D, O, false>(block, meta, flat, shard, padded, n_tiles, pad_zero, acc, dv, grid, stream);
  return gp_launch<META, S, D, O, true>(block, meta, flat, shard, padded, n_tiles, pad_zero, acc, dv, grid, stream);
}

template <class META, class S, class D>
hipError_t gp_by_shard(int o_dt, int block, const META& meta, void* flat, void* shard, int64_t padded, int n_tiles,
                       int pad_zero, int acc, const ReduceDivides& dv, int grid, hipStream_t stream) {
  switch (o_dt) {
    case DT_F32: return gp_go<META, S, D, F32>(block, meta, flat, shard, padded, n_tiles, pad_zero, acc, dv, grid, stream);
    case DT_BF16: return gp_go<META, S, D, BF16>(block, meta, flat, shard, padded, n_tiles, pad_zero, acc, dv, grid, stream);
    case DT_F16: return gp_go<META, S, D, F16>(block, meta, flat, shard, padded, n_tiles, pad_zero, acc, dv, grid, stream);
  }
  return hipErrorInvalidValue;
}

template <class META, class S>
hipError_t gp_by_flat(int d_dt, int o_dt, int block, const META& meta, void* flat, void* shard, int64_t padded,
                      int n_tiles, int pad_zero, int acc, const ReduceDivides& dv, int grid, hipStream_t stream) {
  // the reduce buffer has the gradients' dtype or binary32 (reduce_dtype=float32)
  if (d_dt == S::kId) return gp_by_shard<META, S, S>(o_dt, block, meta, flat, shard, padded, n_tiles, pad_zero, acc, dv, grid, stream);
  if (d_dt == DT_F32) return gp_by_shard<META, S, F32>(o_dt, block, meta, flat, shard, padded, n_tiles, pad_zero, acc, dv, grid, stream);
  return hipErrorInvalidValue;
}

}  // namespace

bool fused_reduce_supports(int tensor_dt, int flat_dt) { return flat_dt == tensor_dt || flat_dt == DT_F32; }

template <class META>
hipError_t launch_unshard(int scatter_shape, int master_dt, int param_dt, const META& meta, const void* gathered,
                          int n_slots, int wt_from, void* ag_in, const void* master, int64_t n, int head, int n_flat_blocks,
                          int flat_wt_from, int grid, hipStream_t stream) {
  switch (master_dt) {
    case DT_F32: return unshard_by_param<META, F32>(param_dt, scatter_shape, meta, gathered, n_slots, wt_from, ag_in, master, n, head, n_flat_blocks, flat_wt_from, grid, stream);
    case DT_BF16: return unshard_by_param<META, BF16>(param_dt, scatter_shape, meta, gathered, n_slots, wt_from, ag_in, master, n, head, n_flat_blocks, flat_wt_from, grid, stream);
    case DT_F16: return unshard_by_param<META, F16>(param_dt, scatter_shape, meta, gathered, n_slots, wt_from, ag_in, master, n, head, n_flat_blocks, flat_wt_from, grid, stream);
  }
  return hipErrorInvalidValue;
}

template <class META>
hipError_t launch_gather_post(int block, int tensor_dt, int flat_dt, int shard_dt, const META& meta, void* flat,
                              void* shard, int64_t padded, int n_tiles, int pad_zero, int acc, const ReduceDivides& dv,
                              int grid, hipStream_t stream) {
  switch (tensor_dt) {
    case DT_F32: return gp_by_flat<META, F32>(flat_dt, shard_dt, block, meta, flat, shard, padded, n_tiles, pad_zero, acc, dv, grid, stream);
    case DT_BF16: return gp_by_flat<META, BF16>(flat_dt, shard_dt, block, meta, flat, shard, padded, n_tiles, pad_zero, acc, dv, grid, stream);
    case DT_F16: return gp_by_flat<META, F16>(flat_dt, shard_dt, block, meta, flat, shard, padded, n_tiles, pad_zero, acc, dv, grid, stream);
  }
  return hipErrorInvalidValue;
}

template hipError_t launch_unshard<SmallMeta>(int, int, int, const SmallMeta&, const void*, int, int, void*, const void*,
                                              int64_t, int, int, int, int, hipStream_t);
template hipError_t launch_unshard<LargeMeta>(int, int, int, const LargeMeta&, const void*, int, int, void*, const void*,
                                              int64_t, int, int, int, int, hipStream_t);
template hipError_t launch_gather_post<SmallMeta>(int, int, int, int, const SmallMeta&, void*, void*, int64_t, int, int,
                                                  int, const ReduceDivides&, int, hipStream_t);
template hipError_t launch_gather_post<LargeMeta>(int, int, int, int, const LargeMeta&, void*, void*, int64_t, int, int,
                                                  int, const ReduceDivides&, int, hipStream_t);

}  // namespace yafsdp

// Internal launcher interface between the C ABI (api.hip) and the translation
// units that instantiate the kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "table_kernels.cuh"

namespace yafsdp {

// dst[i] = post_elem(src[i], dst[i]); scale is SCALE_NONE / SCALE_MUL / SCALE_DIV
hipError_t launch_flat(int src_dt, int dst_dt, int scale, bool acc, void* dst, const void* src, int64_t n, int head,
                       float k, int grid, hipStream_t stream);

// META is SmallMeta or LargeMeta (explicitly instantiated in gather.hip / scatter.hip);
// `block` is the workgroup size the table was built for (kTableBlockSmall or kTableBlockLarge)
template <class META>
hipError_t launch_gather(int block, int tensor_dt, int flat_dt, int scale, const META& meta, void* flat,
                         int64_t padded, int n_tiles, float k, int pad_zero, int grid, hipStream_t stream);
template <class META>
hipError_t launch_scatter(int block, int flat_dt, int tensor_dt, const META& meta, const void* flat, int64_t total,
                          int n_tiles, int grid, hipStream_t stream);

}  // namespace yafsdp

// Internal launcher interface between the C ABI (api.hip) and the translation
// units that instantiate the kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include "table_kernels.hip.h"

namespace yafsdp {

// When a start/stop event pair has been armed on this thread (yafsdp_time_next_launch), or a completion event
// alone (yafsdp_complete_next_launch), the next kernel launched through the library is dispatched with the events
// attached to that dispatch: they carry the kernel's own begin and end (no launch gap in between, and no packet
// of their own in the queue, which an event recorded after the kernel costs).
struct TimedLaunch {
  hipEvent_t start = nullptr, stop = nullptr;
  // per-workgroup timeline of the next flat kernel (yafsdp_trace_next_flat_launch): device buffer of 2 * capacity
  // counts, and where to report the number of workgroups that wrote into it
  unsigned long long* trace = nullptr;
  int64_t trace_capacity = 0;
  int64_t* trace_workgroups = nullptr;
};
extern thread_local TimedLaunch tl_timed_launch;

template <class... Params, class... Args>
inline hipError_t launch_kernel(void (*kernel)(Params...), int grid, int block, hipStream_t stream, Args... args) {
  TimedLaunch& t = tl_timed_launch;
  if (t.start != nullptr || t.stop != nullptr) {
    const hipEvent_t a = t.start, b = t.stop;
    t.start = t.stop = nullptr;
    hipExtLaunchKernelGGL(kernel, dim3(grid), dim3(block), 0, stream, a, b, 0, static_cast<Params>(args)...);
  } else {
    kernel<<<dim3(grid), dim3(block), 0, stream>>>(static_cast<Params>(args)...);
  }
  return hipGetLastError();
}

// dst[i] = post_elem(src[i], dst[i]); scale is SCALE_NONE / SCALE_MUL / SCALE_DIV
// (full tiles before tile `wt_from` store non-temporal, the others write through)
hipError_t launch_flat(int src_dt, int dst_dt, int scale, bool acc, void* dst, const void* src, int64_t n, int head,
                       float k, int wt_from, int grid, hipStream_t stream);
// dst[0:n] = src[0:n], opaque bytes at any byte address; head: bytes up to dst's first 128-byte line (< workgroup size)
hipError_t launch_bytes(void* dst, const void* src, int64_t n, int head, int wt_from, int grid, hipStream_t stream);
// the same pass, also writing partials[0:grid] = per-workgroup sums of squares of the stored values (postsumsq.hip);
// grid must equal the number of tiles
hipError_t launch_post_reduce_sumsq(int src_dt, int dst_dt, int scale, bool acc, void* dst, const void* src, int64_t n,
                                    int head, float k, double* partials, int wt_from, int grid, hipStream_t stream);

// META is SmallMeta or LargeMeta (explicitly instantiated in gather.hip / scatter.hip);
// `block` is the workgroup size the table was built for (kTableBlockSmall or kTableBlockLarge); for launch_scatter
// it is the table's scatter shape packed as workgroup size * 16 + units per lane.  Full tiles from tile (gather-in)
// or tile slot (scatter-out, launch_unshard) `wt_from` on write through (n_tiles: none do)
template <class META>
hipError_t launch_gather(int block, int tensor_dt, int flat_dt, int scale, const META& meta, void* flat,
                         int64_t padded, int n_tiles, float k, int pad_zero, int wt_from, int grid,
                         hipStream_t stream);
template <class META>
hipError_t launch_scatter(int block, int flat_dt, int tensor_dt, const META& meta, const void* flat, int64_t total,
                          int n_tiles, int wt_from, int grid, hipStream_t stream);

// the two fused launches (fused.hip).  launch_unshard: the first n_flat_blocks workgroups of the grid cast
// master[0:n] into ag_in (tiles of workgroup size * kFusedFlatUnroll units), the others run the scatter-out tile
// slots; `scatter_shape` is the table's (workgroup size * 16 + units per lane), and the whole grid has its
// workgroup size.
constexpr int kFusedFlatUnroll = 2;
template <class META>
hipError_t launch_unshard(int scatter_shape, int master_dt, int param_dt, const META& meta, const void* gathered,
                          int n_slots, int wt_from, void* ag_in, const void* master, int64_t n, int head,
                          int n_flat_blocks, int flat_wt_from, int grid, hipStream_t stream);
// reduce copy-in + post-reduce of a size-1 shard group; `block`: the table's gather-in workgroup size
// The divides of the reduce step, applied by that kernel at run time (wave-uniform branches; a shard group of size
// one has none unless the caller set a custom factor or reduces in fp16 with one):
//   a: on the whole reduce buffer, in place (the pre-divide, ya_fsdp/_collectives.py:139, or the custom division
//      of :146-148), rounded to the buffer's dtype; the buffer keeps this value
//   b: the post-divide (:165), rounded to the buffer's dtype; only the gradient shard sees it
struct ReduceDivides {
  int a_mode, b_mode;  // SCALE_NONE / SCALE_MUL (k = exact reciprocal) / SCALE_DIV (k = factor)
  float a_k, b_k;
};
bool fused_reduce_supports(int tensor_dt, int flat_dt);
template <class META>
hipError_t launch_gather_post(int block, int tensor_dt, int flat_dt, int shard_dt, const META& meta, void* flat,
                              void* shard, int64_t padded, int n_tiles, int pad_zero, int acc, const ReduceDivides& dv,
                              int grid, hipStream_t stream);

// fan-out / fan-in over several buffers (fan.hip); all buffers 16-byte aligned
constexpr int kFanMax = 16;
struct FanPtrs {
  void* p[kFanMax];
  int n;
};
hipError_t launch_fanout(int src_dt, int dst_dt, const FanPtrs& dsts, const void* src, int64_t n, int grid,
                         hipStream_t stream);
hipError_t launch_fanin(int chunk_dt, int shard_dt, int scale, bool acc, void* shard, const FanPtrs& chunks, int64_t n,
                        float k, int grid, hipStream_t stream);

// optimizer-side passes (optim.hip); `head` leading elements bring the range to a 16-byte boundary
// scalars of one Adam step, binary32 as they enter the tensor ops (see adamw_kernel)
struct AdamScalars {
  float decay;     // 1 - lr*wd (AdamW), unused otherwise
  float l2;        // wd for the L2 form, unused otherwise
  float w;         // 1 - beta1
  float w_m1;      // w - 1, rounded to binary32
  float beta2;
  float one_m_beta2;
  float bc2_sqrt;  // sqrt(1 - beta2^t)
  float eps;
  float neg_step;  // -(lr / (1 - beta1^t))
  int flags;       // bit 0: decoupled decay, bit 1: L2 decay, bit 2: w < 0.5, bit 3: zero the gradient
};
enum : int { ADAM_DECOUPLED = 1, ADAM_L2 = 2, ADAM_W_SMALL = 4, ADAM_ZERO_GRAD = 8 };
hipError_t launch_fill(int dt, void* dst, int64_t n, int head, uint32_t pattern, int grid, hipStream_t stream);
hipError_t launch_scale(int dt, void* buf, int64_t n, int head, const float* coef, int grid, hipStream_t stream);
// partials[0:grid] = per-workgroup sums of squares
hipError_t launch_sumsq_partials(int dt, const void* src, int64_t n, int head, double* partials, int grid,
                                 hipStream_t stream);
// sumsq[0] (+)= sum(partials[0:count]) (if given); norm_and_coef = {norm, clip coefficient} (if given)
hipError_t launch_sumsq_finish(const double* partials, int64_t count, double* sumsq, int accumulate, float max_norm,
                               float* norm_and_coef, hipStream_t stream);
// out[b] = sum(in[b * 4096 : (b + 1) * 4096]) for b < grid = ceil(count / 4096)
hipError_t launch_sumsq_reduce(const double* in, int64_t count, double* out, int grid, hipStream_t stream);
hipError_t launch_clip_coef(const double* sumsq, float max_norm, float* norm_and_coef, hipStream_t stream);
hipError_t launch_adamw(int out_dt, float* p, float* g, float* m, float* v, void* out16, int64_t n, int head,
                        const AdamScalars& s, const float* grad_scale, int grid, hipStream_t stream);

}  // namespace yafsdp

/* C ABI of libyafsdp_hip.so: MI355X (gfx950) kernels for the per-rank buffer
 * path of YaFSDP-style sharded data parallelism.
 *
 * The reference (yandex/YaFSDP) has no FFI layer: this path is a handful of
 * torch ops inside ya_fsdp/_collectives.py and ya_fsdp/_param_group.py.  Each
 * entry point below names the reference call sites it replaces.
 *
 * Conventions
 *  - All pointers except the `*_ptrs`, `*_numels`, `*_mode` arrays and out
 *    parameters are DEVICE pointers owned by the caller.  Nothing here
 *    allocates or frees caller memory; the only library-owned objects are
 *    metadata tables (yafsdp_table_create / yafsdp_table_destroy).
 *  - `stream` is a hipStream_t passed as void* (NULL = the null stream).  All
 *    work is enqueued on it; no entry point waits for the device, except
 *    yafsdp_table_create / yafsdp_binding_create (one-time set-up: blocking
 *    copies) and yafsdp_table_destroy (waits for the table's queued calls).
 *  - dtype arguments take the yafsdp_dtype values.
 *  - Return value: 0 on success, a positive hipError_t value if a HIP call
 *    failed, a negative yafsdp_status otherwise.  yafsdp_error_string() turns
 *    either into text.
 *  - Divide factors follow ya_fsdp/_collectives.py:270-272: a factor is applied
 *    only if it is > 1 (pass 0 for "None").  The factor is rounded to binary32
 *    and the division is a correctly rounded binary32 division (what torch does
 *    on the host CPU); results are rounded to nearest even into the dtype of the
 *    tensor the reference would have materialised at that step.
 *  - Entry points are re-entrant.  Calls that use the same table from several
 *    host threads are serialised internally.
 */
#ifndef YAFSDP_HIP_H_
#define YAFSDP_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum yafsdp_dtype { YAFSDP_F32 = 0, YAFSDP_BF16 = 1, YAFSDP_F16 = 2 } yafsdp_dtype;

typedef enum yafsdp_status {
  YAFSDP_OK = 0,
  YAFSDP_ERR_INVALID_ARGUMENT = -1,
  YAFSDP_ERR_UNSUPPORTED_DTYPE = -2,
  YAFSDP_ERR_MISALIGNED = -3,
  YAFSDP_ERR_WRONG_DEVICE = -4,
  YAFSDP_ERR_OUT_OF_MEMORY = -5,
  YAFSDP_ERR_TOO_LARGE = -6,
  YAFSDP_ERR_BUSY = -7,
  YAFSDP_ERR_UNSUPPORTED = -8
} yafsdp_status;

/* per-tensor mode of yafsdp_gather_in / yafsdp_scatter_out / fragments */
typedef enum yafsdp_mode { YAFSDP_MODE_SKIP = 0, YAFSDP_MODE_COPY = 1, YAFSDP_MODE_ADD = 2 } yafsdp_mode;

typedef struct yafsdp_table yafsdp_table;

/* ABI version of this header (major * 1000 + minor). */
int yafsdp_version(void);

/* Text for a return code of any entry point. The pointer stays valid. */
const char* yafsdp_error_string(int code);

/* dst[i] = cast(src[i]), i < n: `Tensor.copy_` between flat buffers.
 * Replaces: copy-in  all_gather_input.copy_(padded_sharded_param_data)
 *           (ya_fsdp/_collectives.py:53-54); the size-1-group all-gather
 *           all_gather_output.copy_(all_gather_input) (:56-58); the size-1-group
 *           reduce-scatter output_tensor.copy_(rs_input) (:140-150); and
 *           padded_sharded_param_grad.copy_(output_tensor) (:185).
 * Same dtype: a byte copy.  dst == src with equal element sizes is in place;
 * any other overlap of the two byte ranges is refused (this holds for every
 * flat entry point below). */
int yafsdp_flat_copy(void* dst, int dst_dtype, const void* src, int src_dtype, int64_t n, void* stream);

/* dst[0:n_bytes] = src[0:n_bytes]: `Tensor.copy_` between contiguous ranges of
 * one element type that the arithmetic of this path never touches (1-byte
 * types: float8, int8, uint8; any other type copies the same way).  The two
 * ranges may start at any byte address.
 * Replaces: the per-parameter copy of a tensor-subclass all-gather input into
 *           its fragment of the flat all-gather input,
 *           self._all_gather_input.copy_(all_gather_input)
 *           (ya_fsdp/_param.py:281-291, input from fsdp_pre_all_gather), and the
 *           size-1-group all-gather all_gather_output.copy_(all_gather_input)
 *           (ya_fsdp/_collectives.py:56-58) of such an all-gather dtype
 *           (MixedPrecisionPolicy.all_gather_dtype_to_param_cls,
 *           ya_fsdp/_api.py:13, ya_fsdp/_param_group.py:194-227).
 * dst == src is a no-op; any other overlap is refused. */
int yafsdp_flat_copy_bytes(void* dst, const void* src, int64_t n_bytes, void* stream);

/* buf[i] = round(buf[i] / factor) in place, only if factor > 1.
 * Replaces: _div_if_needed / tensor.div_ (ya_fsdp/_collectives.py:139, 165,
 * 270-272). */
int yafsdp_flat_div(void* buf, int dtype, int64_t n, double factor, void* stream);

/* dst[i] = cast_dst(round_src(src[i] / divisor)), for ANY finite non-zero
 * divisor (no "> 1" rule): the out-of-place divide of the size-1-group branch
 * with a custom factor,
 *   output_tensor.copy_(padded_unsharded_param_grad / gradient_divide_factor)
 * (ya_fsdp/_collectives.py:141-148).  dst == src with equal dtypes is allowed. */
int yafsdp_flat_div_copy(void* dst, int dst_dtype, const void* src, int src_dtype, int64_t n, double divisor,
                         void* stream);

/* Fused post-reduce on the rank's chunk of the reduce buffer:
 *   t = chunk[i];  if (post_factor > 1) t = round_chunk_dtype(t / post_factor);
 *   shard[i] = round_shard_dtype(accumulate ? shard[i] + t : t)
 * Replaces: _div_if_needed(output_tensor, postdivide_factor)
 * (ya_fsdp/_collectives.py:165) followed by padded_sharded_param_grad.copy_ (:185)
 * or .add_ (:189).  The chunk is not written (it is scratch after this point
 * in the reference). */
int yafsdp_post_reduce(void* shard, int shard_dtype, const void* chunk, int chunk_dtype, int64_t n,
                       double post_factor, int accumulate, void* stream);

/* This rank's share of a reduce-scatter whose reduction scales inside the collective
 * (ya_fsdp/_collectives.py:243-249: ReduceOp.AVG, or _make_nccl_premul_sum(1 / factor), handed to
 * dist.reduce_scatter_tensor at :152-162).  The collective library defines both as a PRE-MULTIPLIED sum
 * (ncclRedOpCreatePreMulSum; ncclAvg on floating-point data uses the scalar 1 / nRanks): the scalar is converted to
 * the data type, and every rank's element is multiplied by it and rounded to the data type before the sum.  It
 * is not a division: x * round(1 / f) and x / f differ when f is no power of two.
 *   k = round_dtype(float(scalar))
 *   yafsdp_flat_premul:         buf[i] = round_dtype(buf[i] * k)                       (in place)
 *   yafsdp_post_reduce_premul:  t = round_chunk_dtype(chunk[i] * k);
 *                               shard[i] = round_shard_dtype(accumulate ? shard[i] + t : t)
 * i.e. the collective's share fused with padded_sharded_param_grad.copy_ (:185) / .add_ (:189); the chunk is not
 * written.  Any finite scalar is applied (there is no "> 1" rule inside the collective). */
int yafsdp_flat_premul(void* buf, int dtype, int64_t n, double scalar, void* stream);
int yafsdp_post_reduce_premul(void* shard, int shard_dtype, const void* chunk, int chunk_dtype, int64_t n,
                              double scalar, int accumulate, void* stream);

/* yafsdp_post_reduce that also returns the sum of squares of the shard it
 * writes, as per-workgroup partial sums in binary64 (squares of binary32
 * numbers are exact there): the gradient norm of clip_grad_norm_
 * (ya_fsdp/_tensor.py:220-242, ya_fsdp/ya_fsdp.py:543-562) then needs no
 * pass of its own over the gradient shard.  partials[0 : *n_written] are
 * written (`capacity` doubles available; at least
 * yafsdp_post_reduce_sumsq_count(n) are needed); hand them to
 * yafsdp_clip_coef_from_partials, alone or next to the partial sums of other
 * shards.  The values squared are the stored ones (after rounding to the
 * shard's dtype).  shard and chunk must not overlap.  For a shard that does
 * not start on a 16-byte boundary *n_written can be one less than
 * yafsdp_post_reduce_sumsq_count(n); entries of a larger slot beyond
 * *n_written are not touched, so a caller that adds up the whole slot zeroes
 * them first. */
int64_t yafsdp_post_reduce_sumsq_count(int64_t n);
int yafsdp_post_reduce_sumsq(void* shard, int shard_dtype, const void* chunk, int chunk_dtype, int64_t n,
                             double post_factor, int accumulate, double* partials, int64_t capacity,
                             int64_t* n_written, void* stream);

/* Same as yafsdp_post_reduce but per ragged fragment: fragment f covers
 * elements [sum(numels[:f]), sum(numels[:f+1])) of both shard and chunk and is
 * copied (YAFSDP_MODE_COPY), accumulated (YAFSDP_MODE_ADD) or left untouched
 * (YAFSDP_MODE_SKIP).  `frag_numels` and `frag_mode` are host arrays.
 * Replaces: the _foreach_copy_ / _foreach_add_ pair over per-parameter
 * fragments (ya_fsdp/_collectives.py:191-214). */
int yafsdp_post_reduce_fragments(void* shard, int shard_dtype, const void* chunk, int chunk_dtype,
                                 int n_fragments, const int64_t* frag_numels, const uint8_t* frag_mode,
                                 double post_factor, void* stream);

/* Build the device-resident metadata table of one flat buffer: `n_tensors`
 * tensors laid out back to back, tensor p at elements
 * [sum(numels[:p]), sum(numels[:p+1])), followed by pad lanes up to
 * `padded_numel`.  `numels` is a host array.  The table is bound to the current
 * HIP device and is static for the life of a parameter group (the layout of
 * ya_fsdp/_param_group.py:245-265, 441-457 never changes after construction). */
int yafsdp_table_create(int n_tensors, const int64_t* numels, int64_t padded_numel, yafsdp_table** out);
int yafsdp_table_destroy(yafsdp_table* table);
/* Number of tensors / total elements (without pad) / padded elements. */
int yafsdp_table_info(const yafsdp_table* table, int* n_tensors, int64_t* total_numel, int64_t* padded_numel);

/* Reduce copy-in: gather the tensors of a table into the flat reduce buffer.
 * Per tensor p, with `mode` a host array of n_tensors yafsdp_mode bytes (NULL =
 * all COPY) and `tensor_ptrs` a host array of n_tensors device pointers
 * (ignored for SKIP tensors and empty tensors):
 *   COPY  view_p = cast(tensor_p)                 torch._foreach_copy_
 *         (ya_fsdp/_param_group.py:693-700)
 *   ADD   view_p = round(view_p + tensor_p)       torch._foreach_add_
 *         (ya_fsdp/_param_group.py:701-708)
 *   SKIP  view_p untouched
 * then, if pre_factor > 1, every element of the padded buffer (SKIP tensors
 * and pad lanes included) is divided in the same pass:
 *   flat = round(flat / pre_factor)               _div_if_needed(rs_input, pre)
 *         (ya_fsdp/_collectives.py:139)
 * zero_pad != 0 writes 0 to the pad lanes [total, padded) (the reference leaves
 * them uninitialised).  `flat` must be 16-byte aligned.
 * Tables with more than 16 tensors hand `tensor_ptrs` and `mode` to the kernel
 * through one of 8 staging slots inside the table (a pinned-host to device
 * copy on `stream`).  A call whose arrays equal those of an earlier call still
 * held by a slot reuses that slot's device copy: no copy is enqueued.  The host
 * never waits: if all 8 slots belong to calls whose kernels have not finished
 * yet, the call returns YAFSDP_ERR_BUSY and enqueues nothing (the same holds
 * for yafsdp_scatter_out, which shares the slots). */
int yafsdp_gather_in(yafsdp_table* table, const void* const* tensor_ptrs, const uint8_t* mode, int tensor_dtype,
                     void* flat, int flat_dtype, double pre_factor, int zero_pad, void* stream);

/* Materialising copy-out: tensor_p = cast(flat[offset_p : offset_p + numel_p])
 * for every tensor whose mode is not SKIP (`mode` NULL = all).  The reference's
 * own copy-out is zero-copy views (ya_fsdp/_param_group.py:441-457,
 * ya_fsdp/_param.py:209); this is the `split` + `copy_` form of the same split,
 * for consumers that need separately allocated parameters.  `flat` must be
 * 16-byte aligned; pad lanes are never read. */
int yafsdp_scatter_out(yafsdp_table* table, const void* flat, int flat_dtype, void* const* tensor_ptrs,
                       const uint8_t* mode, int tensor_dtype, void* stream);

/* ---- two launches that do the work of two each --------------------------------
 * For groups whose per-launch cost matters (a small layer takes 4-7 us per
 * launch whatever it moves) and, for the second, for the bytes it saves.  Tables
 * of any size are served, with the staging rules of yafsdp_gather_in for tables
 * of more than 16 tensors (YAFSDP_ERR_BUSY included). */

/* Copy-in and materialising copy-out as one grid:
 *   ag_in[0:n] = cast(master[0:n])                       yafsdp_flat_copy
 *     (all_gather_input.copy_(padded_sharded_param_data), ya_fsdp/_collectives.py:53-54)
 *   tensor_p   = flat[offset_p : offset_p + numel_p]     yafsdp_scatter_out
 *     (the split of the gathered buffer, ya_fsdp/_param_group.py:441-457)
 * The two jobs are independent: `flat` is a gathered buffer that is already
 * complete (in the reference both sit back to back on the all-gather stream:
 * the cast of the next group's shard and the views of the group just
 * gathered).  ag_in and the tensors have the dtype of `flat`. */
int yafsdp_copy_in_scatter_out(yafsdp_table* table, const void* flat, int flat_dtype, void* const* tensor_ptrs,
                               const uint8_t* mode, void* ag_in, const void* master, int master_dtype, int64_t n,
                               void* stream);

/* Reduce copy-in and post-reduce of a shard group of size ONE as one pass.
 * There the rank's chunk of the reduce buffer is the whole buffer and the
 * "reduce-scatter" copies the buffer onto itself (ya_fsdp/_collectives.py:
 * 140-150), so per element
 *   flat  = COPY: cast(tensor) | ADD: round(flat + tensor) | SKIP: flat
 *           (ya_fsdp/_param_group.py:693-708; pad lanes: 0 if zero_pad)
 *   flat  = round(flat / pre_factor)      if pre_factor > 1        (:139)
 *   flat  = round(flat / custom_divisor)  if custom_divisor != 0   (:146-148;
 *           any divisor, as yafsdp_flat_div_copy; excludes the other two)
 *   chunk = round(flat / post_factor)     if post_factor > 1       (:165)
 *   shard = accumulate ? round(shard + chunk) : cast(chunk)        (:185 / :189)
 * with the roundings and the contents of `flat` afterwards (everything up to
 * the post-divide, which only the shard sees) that yafsdp_gather_in,
 * yafsdp_flat_div_copy and yafsdp_post_reduce give in a row.  Pass 0 for an
 * absent factor.  `shard` has the table's padded element count.  Both buffers
 * 16-byte aligned.  `flat` has the tensors' dtype or binary32;
 * YAFSDP_ERR_UNSUPPORTED otherwise, with nothing launched (the separate entry
 * points serve every combination).  The reduce buffer is not read back: 12
 * instead of 14 bytes per element for bf16 gradients, a bf16 buffer and a
 * binary32 shard that accumulates. */
int yafsdp_gather_in_post_reduce(yafsdp_table* table, const void* const* tensor_ptrs, const uint8_t* mode,
                                 int tensor_dtype, void* flat, int flat_dtype, double pre_factor, double custom_divisor,
                                 double post_factor, int zero_pad, void* shard, int shard_dtype, int accumulate,
                                 void* stream);

/* ---- the two exchange points, over several buffers ------------------------------
 * One GPU: all buffers are local.  With peer-mapped pointers the same two calls
 * are the direct (non-ring) forms of the all-gather and the reduce-scatter; no
 * inter-GPU code is part of this library.  All buffers 16-byte aligned; at most
 * 16 destinations / sources. */

/* dst_k[0:n] = cast(src[0:n]) for every k < n_dst: the copy-in cast
 * (ya_fsdp/_collectives.py:53-54) written straight to this rank's slot of several
 * gathered buffers, i.e. the cast plus the placement that
 * all_gather_into_tensor performs (:60-65), reading the master shard once. */
int yafsdp_flat_copy_fanout(void* const* dsts, int n_dst, int dst_dtype, const void* src, int src_dtype, int64_t n,
                            void* stream);

/* The reduce-scatter result and what follows it, from the ranks' reduce buffers:
 *   sum   = chunk_0 + chunk_1 + ... in binary32, in index order (the binary32
 *           accumulation the reference asks of its collective with
 *           bit32_acc_for_bit16_reduce_scatter, ya_fsdp/_collectives.py:157-161)
 *   out   = round(sum) to the chunk dtype        (the collective's output tensor)
 *   out   = _div_if_needed(out, post_factor)     (:165)
 *   shard = out or shard + out                   (:185 / :189)
 * chunk_k is this rank's chunk of rank k's reduce buffer. */
int yafsdp_post_reduce_fanin(void* shard, int shard_dtype, const void* const* chunks, int n_src, int chunk_dtype,
                             int64_t n, double post_factor, int accumulate, void* stream);

/* The same for a collective that scales inside the reduction: ReduceOp.AVG, or
 * the pre-multiplied sum the reference builds for a custom divide factor
 * (ya_fsdp/_collectives.py:243-249).  The collective library multiplies every
 * rank's element by the scalar converted to the chunk dtype, which rounds each
 * product to that dtype, and adds the products:
 *   term_k = round(chunk_k * round(scalar))       both roundings to the chunk dtype
 *   sum    = term_0 + term_1 + ... in binary32, in index order
 *   out    = round(sum) to the chunk dtype;   shard = out or shard + out
 * With one chunk this is yafsdp_post_reduce_premul. */
int yafsdp_post_reduce_fanin_premul(void* shard, int shard_dtype, const void* const* chunks, int n_src,
                                    int chunk_dtype, int64_t n, double scalar, int accumulate, void* stream);

/* The tensor side of a table fixed for many calls.  The reference's unsharded
 * parameters and gradient accumulators are views of pre-allocated buffers that
 * live as long as the group (ya_fsdp/_param_group.py:409-457), and consumers of
 * the materialising copy-out keep their tensors as well: for such tensor sets
 * the pointers, modes and dtype are validated (and, for tables with more than
 * 16 tensors, copied to device memory) once, here; the bound calls then pass
 * only the flat buffer.  No per-call host work beyond the launch and no
 * per-call staging copy, so bound calls can be captured into a HIP graph
 * whatever the table size.  The tensors must stay allocated, and the table
 * alive, while the binding is used.  Semantics are those of yafsdp_gather_in /
 * yafsdp_scatter_out. */
typedef struct yafsdp_binding yafsdp_binding;
int yafsdp_binding_create(yafsdp_table* table, const void* const* tensor_ptrs, const uint8_t* mode,
                          int tensor_dtype, yafsdp_binding** out);
int yafsdp_binding_destroy(yafsdp_binding* binding);
int yafsdp_gather_in_bound(yafsdp_binding* binding, void* flat, int flat_dtype, double pre_factor, int zero_pad,
                           void* stream);
int yafsdp_scatter_out_bound(yafsdp_binding* binding, const void* flat, int flat_dtype, void* stream);

/* ---- optimizer-side passes over the flat shard buffers ------------------------
 * The reference runs the optimizer and gradient clipping as torch foreach ops
 * over the per-parameter fragments of the flat shard (dispatch table of its
 * tensor subclass, ya_fsdp/_tensor.py:122-316).  The fragments of one group are
 * consecutive ranges of one flat buffer, so each op is one pass over that
 * buffer here.  Every pointer below is device memory; ranges may start at any
 * element-aligned address (16-byte aligned starts skip the peeled head). */

/* dst[0:n] = cast(value).  `_foreach_zero_` of optimizer.zero_grad(set_to_none=False)
 * (ya_fsdp/_tensor.py:243-245; the legacy wrapper allows no other form,
 * ya_fsdp/ya_fsdp.py:591-601) and the zero-initialised grad shard
 * (ya_fsdp/_param_group.py:276). */
int yafsdp_flat_fill(void* dst, int dtype, int64_t n, double value, void* stream);

/* Bytes of device workspace yafsdp_flat_sumsq needs (a constant). */
size_t yafsdp_sumsq_workspace_bytes(void);

/* *sumsq = (accumulate ? *sumsq : 0) + sum_i float(src[i])^2, in binary64.
 * The squared 2-norm behind `_foreach_norm(grads, 2)` (ya_fsdp/_tensor.py:220-242)
 * and the legacy clip_grad_norm_ (ya_fsdp/ya_fsdp.py:545-556), whose per-buffer
 * norms are squared and summed again.  The reference adds in binary32 in an
 * order its backend chooses; this sum is exact to binary64 rounding and its
 * order depends only on n, so it is reproducible.  `workspace` is scratch for
 * the duration of the call on `stream` (calls sharing one workspace must not
 * overlap).  Two launches: per-workgroup partial sums, then their sum. */
int yafsdp_flat_sumsq(const void* src, int dtype, int64_t n, double* sumsq, int accumulate, void* workspace,
                      size_t workspace_bytes, void* stream);

/* yafsdp_flat_sumsq for callers that cannot allocate and have no workspace to hand over (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same
 * kernels, same order of additions and so the same bits as yafsdp_flat_sumsq; the per-workgroup partial sums go to a
 * fixed 128 KiB array in the library's own device image (one copy per GPU, held until the process ends) instead of
 * a workspace argument.  The call allocates and frees nothing.  n is limited to
 * yafsdp_flat_sumsq_static_max_numel() = 2^31 elements; more returns YAFSDP_ERR_TOO_LARGE.  The first call on a
 * device looks the array's address up; a call with n == 0 does only that (make one before capturing a graph).
 * All calls on one GPU share the array: calls that overlap in time (different streams, or threads) race on it, and
 * the caller has to order them.  Nothing in it needs clearing between calls. */
int64_t yafsdp_flat_sumsq_static_max_numel(void);
int yafsdp_flat_sumsq_static(const void* src, int dtype, int64_t n, double* sumsq, int accumulate, void* stream);

/* The same split in two for several buffers (the groups of a model): each call
 * of yafsdp_sumsq_partials writes at most `capacity` per-workgroup sums of
 * squares of one buffer to `partials` and reports how many (*n_written, at most
 * yafsdp_sumsq_workspace_bytes() / 8 per call); the caller lays the calls out
 * one after the other in one array, and yafsdp_clip_coef_from_partials adds
 * the whole array in a fixed order and derives the norm and the coefficient
 * (and stores the sum to *sumsq if not NULL): one launch per buffer plus one. */
int yafsdp_sumsq_partials(const void* src, int dtype, int64_t n, double* partials, int64_t capacity,
                          int64_t* n_written, void* stream);
int yafsdp_clip_coef_from_partials(const double* partials, int64_t n_partials, double max_norm, double* sumsq,
                                   float* norm_and_coef, void* stream);

/* First stage for long arrays of partial sums (many shards, or shards of
 * hundreds of millions of elements through yafsdp_post_reduce_sumsq):
 * out[b] = sum(partials[4096 b : 4096 (b + 1)]), b < ceil(n_partials / 4096),
 * one workgroup each, in a fixed order; *n_written receives that count
 * (`capacity` doubles available in `out`).  yafsdp_clip_coef_from_partials adds
 * with a single workgroup, which is the faster way below about 16 K sums. */
int yafsdp_sumsq_reduce_partials(const double* partials, int64_t n_partials, double* out, int64_t capacity,
                                 int64_t* n_written, void* stream);

/* norm_and_coef[0] = float(sqrt(*sumsq)); norm_and_coef[1] = min(max_norm /
 * (norm + 1e-6), 1.0), binary32 like the reference's tensors
 * (ya_fsdp/ya_fsdp.py:557-559; torch.nn.utils.clip_grads_with_norm_). */
int yafsdp_clip_coef(const double* sumsq, double max_norm, float* norm_and_coef, void* stream);

/* buf[i] = round(float(buf[i]) * *coef), the coefficient read on the device
 * (`grad.mul_(total_norm_coef)`, ya_fsdp/ya_fsdp.py:560-561; `_foreach_mul_.Tensor`,
 * ya_fsdp/_tensor.py:256-262).  Returns without touching memory when *coef == 1. */
int yafsdp_flat_scale(void* buf, int dtype, int64_t n, const float* coef, void* stream);

/* One Adam / AdamW step on a flat binary32 shard (param, grad, exp_avg,
 * exp_avg_sq of n elements), in the operation order of torch.optim.Adam(W)
 * (`_fused_adam_` / `_fused_adamw_` and the foreach lerp / addcmul / addcdiv
 * ops the reference forwards to the local tensors, ya_fsdp/_tensor.py:269-312),
 * fused with the copy-in cast of the next iteration
 * (`all_gather_input.copy_(shard)`, ya_fsdp/_collectives.py:53-54): when `out16` is
 * not NULL it receives the updated parameters rounded to `out16_dtype` (bf16 or
 * f16).  `step` is the 1-based step count.  `grad_scale` (device, may be NULL)
 * multiplies the gradient first, as a preceding `grad.mul_(coef)` would, without
 * writing it back.  flags: YAFSDP_ADAM_DECOUPLED_DECAY = AdamW, otherwise the
 * L2 form of Adam; YAFSDP_ADAM_ZERO_GRAD also zero-fills `grad`.  The four
 * binary32 arrays must share one address residue modulo 16 bytes and `out16`
 * half of it modulo 8 (true for one fragment range of identically laid out
 * shards). */
enum { YAFSDP_ADAM_DECOUPLED_DECAY = 1, YAFSDP_ADAM_ZERO_GRAD = 2 };
int yafsdp_adamw_step(float* param, float* grad, float* exp_avg, float* exp_avg_sq, void* out16, int out16_dtype,
                      int64_t n, double lr, double beta1, double beta2, double eps, double weight_decay,
                      int64_t step, const float* grad_scale, int flags, void* stream);

/* Measurement hook: arms a pair of HIP events (hipEvent_t, created with timing
 * enabled) for the calling thread.  The next kernel this thread launches
 * through the library is dispatched with the pair attached to that dispatch
 * (hipExtLaunchKernel), so hipEventElapsedTime(start, stop) is the kernel's own
 * duration without the launch gap an event record around the call would add.
 * The pair is consumed by that one launch (the first one, for entry points that
 * launch several kernels); NULL, NULL disarms. */
int yafsdp_time_next_launch(void* start_event, void* stop_event);

/* The next kernel this thread launches through the library records `event` (a hipEvent_t; timing may be disabled)
 * when it completes, as hipEventRecord(event, stream) right after the call would, but on the kernel's own
 * dispatch (hipExtLaunchKernel): no marker packet follows the kernel in its queue.  A marker between two kernels
 * of one stream was measured at 6.5 us of idle GPU, a kernel -> event -> wait -> kernel hop between two streams at
 * 11.4 us; the reference records one event per all-gather and two per reduce (ya_fsdp/_collectives.py:73-76,
 * 215; ya_fsdp/_param_group.py:595-606, 757-769).  Consumed by ONE launch (the first, for an entry point that
 * launches several kernels: use it with single-launch calls).  A call that launches nothing (an empty range)
 * leaves the event armed: yafsdp_complete_next_launch_pending() then returns 1 and the caller records the event
 * itself after disarming with NULL.  No counterpart in the reference (torch records events as queue markers). */
int yafsdp_complete_next_launch(void* event);
int yafsdp_complete_next_launch_pending(void);

/* Measurement hook: per-workgroup timeline of the next kernel that this thread launches through
 * yafsdp_flat_copy / yafsdp_flat_div / yafsdp_flat_div_copy / yafsdp_post_reduce.  Workgroup b of that launch
 * stores the GPU's 100 MHz wall-clock count at its start into trace[2 b] and, once its loads have arrived and its
 * stores are acknowledged, at its end into trace[2 b + 1] (`trace`: device memory for 2 * capacity 64-bit
 * counts).  *n_workgroups (host memory, may be NULL) receives the grid size when the launch is made, or minus the
 * grid size if it exceeded `capacity` (then nothing is traced).  Consumed by one launch; NULL disarms. */
int yafsdp_trace_next_flat_launch(uint64_t* trace, int64_t capacity, int64_t* n_workgroups);

/* Launch-shape and store-policy options (process-wide): */
typedef enum yafsdp_option {
  YAFSDP_OPT_FLAT_BLOCKS_PER_CU = 0,  /* workgroups per compute unit of the flat kernels' grid */
  YAFSDP_OPT_TABLE_BLOCKS_PER_CU = 1, /* same for gather-in / scatter-out */
  YAFSDP_OPT_TABLE_LARGE_LOG2 = 2,    /* 0..62: tables created from now on whose padded size exceeds
                                         2^value elements run two waves per workgroup instead of one */
  YAFSDP_OPT_SCATTER_TILE = 3,        /* tile of yafsdp_scatter_out for tables created from now on: 0 = from the
                                         layout (short 512-element tiles when every tensor starts on a 128-byte
                                         line of the flat buffer, the gather-in tile otherwise), 1 = always
                                         short, 2 = never short */
  YAFSDP_OPT_GATHER_TAIL_MB = 4,      /* 0..2^20, default 64: yafsdp_gather_in / yafsdp_gather_in_bound write the last
                                         `value` megabytes of the flat buffer through the L2s instead of leaving
                                         them there as dirty lines (a store-policy choice; the bytes written are
                                         the same).  The memory-side cache absorbs them and writes them back
                                         later: the kernel ends with clean L2s, and the lines are still in that
                                         256-MB cache when the buffer is read again soon.  0 = off */
  YAFSDP_OPT_SCATTER_TAIL_MB = 5,     /* 0..2^20, default 0: the same for the tile slots of the last `value`
                                         megabytes of tensors in yafsdp_scatter_out / yafsdp_scatter_out_bound /
                                         yafsdp_copy_in_scatter_out */
  YAFSDP_OPT_FLAT_TAIL_MB = 6,        /* 0..2^20, default 0: the same for yafsdp_flat_copy, yafsdp_flat_copy_bytes,
                                         yafsdp_flat_div, yafsdp_flat_div_copy and the cast part of
                                         yafsdp_copy_in_scatter_out; 2^20 = they write through everywhere */
  YAFSDP_OPT_POST_REDUCE_TAIL_MB = 7  /* the same for yafsdp_post_reduce / yafsdp_post_reduce_sumsq /
                                         yafsdp_post_reduce_fragments.
                                         Written-through lines pay if they are still in the 256-MB memory-side
                                         cache when their buffer is read or written again, and cost if they are
                                         evicted in the middle of other kernels.  The defaults of options 4-7
                                         (64 / 0 / 0 / 0) are cache-neutral: they suit parameter groups that take
                                         turns on shared buffers (up to four reduce buffers in rotation; with ONE
                                         gradient buffer for all groups, as in the reference, 128 for option 4 is
                                         better still).  A caller that rewrites ONE set of buffers in a loop gains
                                         2-4 % from 96 / 0 / 2^20 / 2^20 (the loop then finds its own output in
                                         that cache, which a training run does not) */
} yafsdp_option;
int yafsdp_set_option(int option, int value);
int yafsdp_get_option(int option, int* value);
/* The same two store-policy options for ONE table (YAFSDP_OPT_GATHER_TAIL_MB, YAFSDP_OPT_SCATTER_TAIL_MB; every
 * other option is refused): the table's own value, 0..2^20, takes precedence over the process-wide one in every
 * call on this table; -1 (the state a table is created in) follows the process-wide option again.  How soon a
 * flat buffer comes round again is a property of the parameter group that owns it (how many gradient buffers its
 * model rotates through), not of the process: two models in one process keep their own settings this way.
 * No counterpart in the reference (its ops take no cache policy). */
int yafsdp_table_set_option(yafsdp_table* table, int option, int value);
int yafsdp_table_get_option(const yafsdp_table* table, int option, int* value);

#ifdef __cplusplus
}
#endif
#endif /* YAFSDP_HIP_H_ */

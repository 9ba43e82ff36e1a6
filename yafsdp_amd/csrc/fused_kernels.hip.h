// Two launches that each do the work of two, for groups whose per-launch cost
// matters (small layers, a shard group of size one):
//
//  * unshard_kernel: copy-in (cast of the master shard into the all-gather
//    input) and the materialising copy-out of a gathered buffer as ONE grid.
//    The two jobs do not depend on each other (the copy-out reads a gathered
//    buffer that is already complete); the first `n_flat_blocks` workgroups
//    run the flat pass, the others the scatter-out tile slots (full tiles
//    of the slots from `wt_from` on store write-through, see tuning.h).
//
//  * gather_post_kernel: reduce copy-in and post-reduce as one pass, for a
//    shard group of size ONE.  There the rank's chunk of the reduce buffer IS
//    the whole buffer and no collective sits between the two steps
//    (ya_fsdp/_collectives.py:140-150), so every element can go
//        gradient -> (copy | add) into the reduce buffer, rounded to its dtype
//                 -> copy | accumulate into the gradient shard, rounded to its dtype
//    in one go, with the same rounding points as the separate kernels and the
//    reduce buffer written as they would leave it.  The divides of the reduce
//    step (absent at size one unless the caller asks for them,
//    ya_fsdp/_collectives.py:221-267) are applied at run time, each with its
//    own rounding.
//
// META is SmallMeta (at most kSmallMax tensors: metadata in the kernel arguments)
// or LargeMeta (records and per-call pointers in device memory), as in the
// kernels they stand for.  Lanes of gather_post_kernel always take the quad
// arrangement (elem.hip.h): the gradient shard is binary32 in the usual case.
#pragma once
#include "launch.h"
#include "table_kernels.hip.h"

namespace yafsdp {

// M: master dtype, P: dtype of the all-gather input, of the gathered buffer and of the tensors.
template <class META, class M, class P, int BLOCK, int UF, int US, bool NTL, int STP_FLAT, int STP_SCATTER>
__global__ void __launch_bounds__(BLOCK)
unshard_kernel(META meta, const void* gathered, int n_slots, int wt_from, void* ag_in, const void* master, int64_t n,
               int head, int n_flat_blocks, int flat_wt_from) {
  const int b = blockIdx.x;
  if (b < n_flat_blocks) {
    flat_body<M, P, SCALE_NONE, false, BLOCK, UF, kFlatNtLoad, STP_FLAT>(ag_in, master, n, head, 1.0f, b, n_flat_blocks,
                                                                       flat_wt_from);
  } else {
    scatter_body<META, P, P, BLOCK, US, NTL, STP_SCATTER>(meta, gathered, n_slots, wt_from, b - n_flat_blocks,
                                                              int(gridDim.x) - n_flat_blocks);
  }
}

template <class D>
__device__ __forceinline__ float divide_stage(float y, int mode, float k) {
  if (mode == SCALE_MUL) return round_to<D>(apply_scale<SCALE_MUL>(y, k));
  if (mode == SCALE_DIV) return round_to<D>(apply_scale<SCALE_DIV>(y, k));
  return y;
}

// One element of the fused reduce path.  MODE: how the gradient enters the reduce buffer.
// DIV: whether any divide is applied (the kernel without them is a separate instantiation: the division's code
// doubles the register count, which the common case should not pay for).
template <class S, class D, int MODE, bool DIV>
__device__ __forceinline__ void gather_post_elem(float s, float d_old, float o_old, bool acc, const ReduceDivides& dv,
                                                 float& d_new, float& o_new) {
  float y;
  if constexpr (MODE == MODE_ZERO) y = 0.f;
  else y = round_to<D>(gather_elem<S, D, SCALE_NONE, MODE>(s, d_old, 1.0f));
  float c;
  if constexpr (DIV) {
    d_new = divide_stage<D>(y, dv.a_mode, dv.a_k);  // what the reduce buffer holds afterwards
    c = divide_stage<D>(d_new, dv.b_mode, dv.b_k);  // what the "reduce-scatter" hands on
  } else {
    d_new = c = y;
  }
  o_new = acc ? __fadd_rn(o_old, c) : c;  // caller rounds to O on store
}

template <class S, class D, class O, int MODE, bool DIV>
__device__ __forceinline__ void gather_post_scalar(char* flat, const char* src, char* shard, int64_t i, bool acc,
                                                   const ReduceDivides& dv) {
  typedef typename S::storage s_t;
  typedef typename D::storage d_t;
  typedef typename O::storage o_t;
  d_t* d = reinterpret_cast<d_t*>(flat) + i;
  o_t* o = reinterpret_cast<o_t*>(shard) + i;
  float s = 0.f, d_old = 0.f, o_old = 0.f;
  if constexpr (MODE == MODE_COPY || MODE == MODE_ADD) s = to_f32<S>(reinterpret_cast<const s_t*>(src)[i]);
  if constexpr (MODE == MODE_ADD || MODE == MODE_SKIP) d_old = to_f32<D>(*d);
  if (acc) o_old = to_f32<O>(*o);
  float d_new, o_new;
  gather_post_elem<S, D, MODE, DIV>(s, d_old, o_old, acc, dv, d_new, o_new);
  const bool divided = DIV && dv.a_mode != SCALE_NONE;
  if (MODE == MODE_COPY && same_t<S, D>::value && !divided) *d = reinterpret_cast<const s_t*>(src)[i];
  else if (MODE != MODE_SKIP || divided) *d = from_f32<D>(d_new);
  *o = from_f32<O>(o_new);
}

// One full tile (BLOCK*U units) inside one tensor; flat and shard 16-byte aligned at the tile, src at any
// element-aligned address.
template <class S, class D, class O, int MODE, bool DIV, int BLOCK, int U, bool NTL>
__device__ __forceinline__ void gather_post_full_tile(char* flat, const char* src, char* shard, bool acc,
                                                      const ReduceDivides& dv) {
  constexpr bool kReadSrc = (MODE == MODE_COPY || MODE == MODE_ADD);
  constexpr bool kReadFlat = (MODE == MODE_ADD || MODE == MODE_SKIP);
  const bool divided = DIV && dv.a_mode != SCALE_NONE;
  Quad<S> s[2 * U];
  Quad<D> d[2 * U];
  Quad<O> o[2 * U];
  if constexpr (kReadSrc) {
#pragma unroll
    for (int q = 0; q < 2 * U; q++) s[q] = load_quad<S, NTL>(src + quad_elem<BLOCK, U>(q) * S::kSize);
  }
  if constexpr (kReadFlat) {
#pragma unroll
    for (int q = 0; q < 2 * U; q++) d[q] = load_quad<D, NTL>(flat + quad_elem<BLOCK, U>(q) * D::kSize);
  }
  if (acc) {
#pragma unroll
    for (int q = 0; q < 2 * U; q++) o[q] = load_quad<O, NTL>(shard + quad_elem<BLOCK, U>(q) * O::kSize);
  }
#pragma unroll
  for (int q = 0; q < 2 * U; q++) {
    float fs[4] = {0.f, 0.f, 0.f, 0.f}, fd[4] = {0.f, 0.f, 0.f, 0.f}, fo[4] = {0.f, 0.f, 0.f, 0.f}, nd[4], no[4];
    if constexpr (kReadSrc) unpack_quad<S>(s[q], fs);
    if constexpr (kReadFlat) unpack_quad<D>(d[q], fd);
    if (acc) unpack_quad<O>(o[q], fo);
#pragma unroll
    for (int e = 0; e < 4; e++) gather_post_elem<S, D, MODE, DIV>(fs[e], fd[e], fo[e], acc, dv, nd[e], no[e]);
    char* f = flat + quad_elem<BLOCK, U>(q) * D::kSize;
    if (MODE == MODE_COPY && same_t<S, D>::value && !divided) {
      // same dtype, nothing divided: the reduce buffer receives the gradient's bytes (NaN payloads included), as
      // the copy kernel does
      Quad<D> raw;
      if constexpr (same_t<S, D>::value) raw.v = s[q].v;
      store_quad<D, true>(f, raw);
    } else if (MODE != MODE_SKIP || divided) {
      store_quad<D, true>(f, pack_quad<D>(nd));
    }
    store_quad<O, true>(shard + quad_elem<BLOCK, U>(q) * O::kSize, pack_quad<O>(no));
  }
}

// n elements of one segment (part of a tile that crosses a tensor boundary or the end of the buffer), one element
// per lane and step: such tiles are rare (at most one per tensor boundary).
template <class S, class D, class O, int MODE, bool DIV, int BLOCK>
__device__ __forceinline__ void gather_post_segment(char* flat, const char* src, char* shard, int64_t n, bool acc,
                                                    const ReduceDivides& dv) {
  for (int64_t i = threadIdx.x; i < n; i += BLOCK) gather_post_scalar<S, D, O, MODE, DIV>(flat, src, shard, i, acc, dv);
}

// S: gradient dtype, D: reduce buffer dtype, O: gradient shard dtype.  `shard` has `padded` elements like `flat`.
// pad_zero != 0 writes zeros (divided like everything else) to the pad lanes of the reduce buffer, otherwise they
// only see the divide; in both cases the pad lanes of the shard receive what the separate post-reduce would give them.
template <class META, class S, class D, class O, bool DIV, int BLOCK, int U, bool NTL>
__global__ void __launch_bounds__(BLOCK)
gather_post_kernel(META meta, void* flat, void* shard, int64_t padded, int n_tiles, int pad_zero, int accumulate,
                   ReduceDivides dv) {
  constexpr int64_t kTile = int64_t(BLOCK) * U * 8;
  char* fbase = reinterpret_cast<char*>(flat);
  char* obase = reinterpret_cast<char*>(shard);
  const bool acc = accumulate != 0;
  for (int tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const int64_t t0 = int64_t(tile) * kTile;
    const int64_t t1 = (t0 + kTile < padded) ? t0 + kTile : padded;
    const TileLookup rec = meta.lookup(tile, t0, kTile);
    int p = rec.first;
    if (rec.full) {
      const int mode = meta.mode(p);
      const char* src = reinterpret_cast<const char*>(meta.tensor(p)) + rec.delta * S::kSize;
      char* f = fbase + t0 * D::kSize;
      char* o = obase + t0 * O::kSize;
      if (mode == MODE_COPY) gather_post_full_tile<S, D, O, MODE_COPY, DIV, BLOCK, U, NTL>(f, src, o, acc, dv);
      else if (mode == MODE_ADD) gather_post_full_tile<S, D, O, MODE_ADD, DIV, BLOCK, U, NTL>(f, src, o, acc, dv);
      else gather_post_full_tile<S, D, O, MODE_SKIP, DIV, BLOCK, U, NTL>(f, src, o, acc, dv);
      continue;
    }
    int64_t pos = t0;
    while (pos < t1) {
      char* f = fbase + pos * D::kSize;
      char* o = obase + pos * O::kSize;
      if (p >= meta.n_tensors) {  // pad lanes
        if (pad_zero) gather_post_segment<S, D, O, MODE_ZERO, DIV, BLOCK>(f, nullptr, o, t1 - pos, acc, dv);
        else gather_post_segment<S, D, O, MODE_SKIP, DIV, BLOCK>(f, nullptr, o, t1 - pos, acc, dv);
        break;
      }
      const int64_t o1 = meta.offset(p + 1);
      if (o1 <= pos) { ++p; continue; }  // empty tensor
      const int64_t o0 = meta.offset(p);
      const int64_t e = o1 < t1 ? o1 : t1;
      const int mode = meta.mode(p);
      const char* src = reinterpret_cast<const char*>(meta.tensor(p)) + (pos - o0) * S::kSize;
      if (mode == MODE_COPY) gather_post_segment<S, D, O, MODE_COPY, DIV, BLOCK>(f, src, o, e - pos, acc, dv);
      else if (mode == MODE_ADD) gather_post_segment<S, D, O, MODE_ADD, DIV, BLOCK>(f, src, o, e - pos, acc, dv);
      else gather_post_segment<S, D, O, MODE_SKIP, DIV, BLOCK>(f, src, o, e - pos, acc, dv);
      pos = e;
      if (e == o1) ++p;
    }
  }
}

}  // namespace yafsdp

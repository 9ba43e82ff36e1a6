// Two launches that each do the work of two, for groups whose per-launch cost
// matters (small layers, a shard group of size one):
//
//  * unshard_kernel: copy-in (cast of the master shard into the all-gather
//    input) and the materialising copy-out of a gathered buffer as ONE grid.
//    The two jobs do not depend on each other (the copy-out reads a gathered
//    buffer that is already complete); the first `n_flat_blocks` workgroups
//    run the flat pass, the others the scatter-out tile slots.
//
//  * gather_post_kernel: reduce copy-in and post-reduce as one pass, for a
//    shard group of size ONE.  There the rank's chunk of the reduce buffer IS
//    the whole buffer and no collective sits between the two steps
//    (ya_fsdp/_collectives.py:140-150), so every element can go
//        gradient -> (copy | add) into the reduce buffer, rounded to its dtype
//                 -> copy | accumulate into the gradient shard, rounded to its dtype
//    in one go, with the same two rounding points as the separate kernels and
//    the reduce buffer written as they would leave it.  No divide: at size one
//    the reference's factors are absent or 1 (ya_fsdp/_collectives.py:221-267).
//
// META is SmallMeta (at most kSmallMax tensors: metadata in the kernel arguments)
// or LargeMeta (records and per-call pointers in device memory), as in the
// kernels they stand for.  Lanes of gather_post_kernel always take the quad
// arrangement (elem.hip.h): the gradient shard is binary32 in the usual case.
#pragma once
#include "table_kernels.hip.h"

namespace yafsdp {

// M: master dtype, P: dtype of the all-gather input, of the gathered buffer and of the tensors.
template <class META, class M, class P, int BLOCK, int UF, int US, bool NTL, int STP_FLAT, int STP_SCATTER>
__global__ void __launch_bounds__(BLOCK)
unshard_kernel(META meta, const void* gathered, int n_slots, void* ag_in, const void* master, int64_t n, int head,
               int n_flat_blocks) {
  const int b = blockIdx.x;
  if (b < n_flat_blocks) {
    flat_body<M, P, SCALE_NONE, false, BLOCK, UF, NTL, STP_FLAT>(ag_in, master, n, head, 1.0f, b, n_flat_blocks);
  } else {
    scatter_body<META, P, P, BLOCK, US, NTL, STP_SCATTER>(meta, gathered, n_slots, b - n_flat_blocks,
                                                              int(gridDim.x) - n_flat_blocks);
  }
}

// One element of the fused reduce path.  MODE: how the gradient enters the reduce buffer.
template <class S, class D, class O, int MODE>
__device__ __forceinline__ void gather_post_elem(float s, float d_old, float o_old, bool acc, float& d_new, float& o_new) {
  const float y = gather_elem<S, D, SCALE_NONE, MODE>(s, d_old, 1.0f);
  d_new = round_to<D>(y);                     // what the reduce buffer holds afterwards
  o_new = acc ? __fadd_rn(o_old, d_new) : d_new;  // caller rounds to O on store
}

template <class S, class D, class O, int MODE>
__device__ __forceinline__ void gather_post_scalar(char* flat, const char* src, char* shard, int64_t i, bool acc,
                                                   bool write_flat) {
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
  if constexpr (MODE == MODE_ZERO) {
    d_new = 0.f;
    o_new = acc ? __fadd_rn(o_old, 0.f) : 0.f;
  } else {
    gather_post_elem<S, D, O, MODE>(s, d_old, o_old, acc, d_new, o_new);
  }
  if constexpr (MODE == MODE_COPY && same_t<S, D>::value) *d = reinterpret_cast<const s_t*>(src)[i];
  else if (write_flat) *d = from_f32<D>(d_new);
  *o = from_f32<O>(o_new);
}

// One full tile (BLOCK*U units) inside one tensor; flat and shard 16-byte aligned at the tile, src at any
// element-aligned address.
template <class S, class D, class O, int MODE, int BLOCK, int U, bool NTL>
__device__ __forceinline__ void gather_post_full_tile(char* flat, const char* src, char* shard, bool acc) {
  constexpr bool kReadSrc = (MODE == MODE_COPY || MODE == MODE_ADD);
  constexpr bool kReadFlat = (MODE == MODE_ADD || MODE == MODE_SKIP);
  constexpr bool kWriteFlat = (MODE != MODE_SKIP);
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
    for (int e = 0; e < 4; e++) {
      if constexpr (MODE == MODE_ZERO) {
        nd[e] = 0.f;
        no[e] = acc ? __fadd_rn(fo[e], 0.f) : 0.f;
      } else {
        gather_post_elem<S, D, O, MODE>(fs[e], fd[e], fo[e], acc, nd[e], no[e]);
      }
    }
    if constexpr (MODE == MODE_COPY && same_t<S, D>::value) {
      // same dtype: the reduce buffer receives the gradient's bytes (NaN payloads included), as the copy kernel does
      Quad<D> raw;
      raw.v = s[q].v;
      store_quad<D, true>(flat + quad_elem<BLOCK, U>(q) * D::kSize, raw);
    } else if constexpr (kWriteFlat) {
      store_quad<D, true>(flat + quad_elem<BLOCK, U>(q) * D::kSize, pack_quad<D>(nd));
    }
    store_quad<O, true>(shard + quad_elem<BLOCK, U>(q) * O::kSize, pack_quad<O>(no));
  }
}

// n elements of one segment (part of a tile that crosses a tensor boundary or the end of the buffer), one element
// per lane and step: such tiles are rare (at most one per tensor boundary).
template <class S, class D, class O, int MODE, int BLOCK>
__device__ __forceinline__ void gather_post_segment(char* flat, const char* src, char* shard, int64_t n, bool acc,
                                                    bool write_flat) {
  for (int64_t i = threadIdx.x; i < n; i += BLOCK) gather_post_scalar<S, D, O, MODE>(flat, src, shard, i, acc, write_flat);
}

// S: gradient dtype, D: reduce buffer dtype, O: gradient shard dtype.  `shard` has `padded` elements like `flat`.
// pad_zero != 0 writes zeros to the pad lanes of the reduce buffer (otherwise they stay as they are); in both cases
// the pad lanes of the shard receive what the separate post-reduce would give them.
template <class META, class S, class D, class O, int BLOCK, int U, bool NTL>
__global__ void __launch_bounds__(BLOCK)
gather_post_kernel(META meta, void* flat, void* shard, int64_t padded, int n_tiles, int pad_zero, int accumulate) {
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
      if (mode == MODE_COPY) gather_post_full_tile<S, D, O, MODE_COPY, BLOCK, U, NTL>(f, src, o, acc);
      else if (mode == MODE_ADD) gather_post_full_tile<S, D, O, MODE_ADD, BLOCK, U, NTL>(f, src, o, acc);
      else gather_post_full_tile<S, D, O, MODE_SKIP, BLOCK, U, NTL>(f, src, o, acc);
      continue;
    }
    int64_t pos = t0;
    while (pos < t1) {
      char* f = fbase + pos * D::kSize;
      char* o = obase + pos * O::kSize;
      if (p >= meta.n_tensors) {  // pad lanes
        if (pad_zero) gather_post_segment<S, D, O, MODE_ZERO, BLOCK>(f, nullptr, o, t1 - pos, acc, true);
        else gather_post_segment<S, D, O, MODE_SKIP, BLOCK>(f, nullptr, o, t1 - pos, acc, false);
        break;
      }
      const int64_t o1 = meta.offset(p + 1);
      if (o1 <= pos) { ++p; continue; }  // empty tensor
      const int64_t o0 = meta.offset(p);
      const int64_t e = o1 < t1 ? o1 : t1;
      const int mode = meta.mode(p);
      const char* src = reinterpret_cast<const char*>(meta.tensor(p)) + (pos - o0) * S::kSize;
      if (mode == MODE_COPY) gather_post_segment<S, D, O, MODE_COPY, BLOCK>(f, src, o, e - pos, acc, true);
      else if (mode == MODE_ADD) gather_post_segment<S, D, O, MODE_ADD, BLOCK>(f, src, o, e - pos, acc, true);
      else gather_post_segment<S, D, O, MODE_SKIP, BLOCK>(f, src, o, e - pos, acc, false);
      pos = e;
      if (e == o1) ++p;
    }
  }
}

}  // namespace yafsdp

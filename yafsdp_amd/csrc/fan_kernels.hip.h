// The two places where ranks exchange data, as one-GPU kernels over several
// buffers: the copy-in cast written to several destinations (this rank's slot
// of every rank's gathered buffer), and the reduce step that reads one chunk
// from several reduce buffers, adds them in binary32, and accumulates into the
// gradient shard.  On one GPU all buffers are local; with peer-mapped pointers
// the same kernels are the direct (non-ring) all-gather and reduce-scatter.
//
// Lanes own quads (4 consecutive elements); quad j of lane t inside a tile of
// BLOCK*U quads is t + j*BLOCK, so every wave64 access is one contiguous span.
// All buffers are 16-byte aligned.
#pragma once
#include "flat_kernels.hip.h"
#include "launch.h"

namespace yafsdp {


// dst_k[i] = cast(src[i]) for every k < dsts.n   (ya_fsdp/_collectives.py:53-54
// followed by the placement the all-gather performs, :60-65).  The kernel is
// dominated by its stores (n_dst of them per load), so lanes own units (8
// consecutive elements): every store is a full 16 bytes of a 2-byte dtype.
template <class S, class D, int BLOCK, int U, bool NTL, int STP>
__global__ void __launch_bounds__(BLOCK)
fanout_kernel(FanPtrs dsts, const void* src, int64_t n) {
  typedef typename S::storage s_t;
  typedef typename D::storage d_t;
  constexpr bool NTS = (STP == ST_NT);  // the ragged last tile keeps ordinary global stores
  const int64_t n_units = n >> 3;
  constexpr int64_t kTile = int64_t(BLOCK) * U;
  constexpr int kTileBytes = int(kTile) * 8 * D::kSize;
  const int64_t n_tiles = (n_units + kTile - 1) / kTile;
  const char* sbase = reinterpret_cast<const char*>(src);
  for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const int64_t u0 = tile * kTile + threadIdx.x;
    if (tile * kTile + kTile <= n_units) {
      Unit<D> y[U];
#pragma unroll
      for (int j = 0; j < U; j++) {
        const Unit<S> x = load_unit<S, NTL>(sbase + (u0 + j * BLOCK) * (8 * S::kSize));
        Unit<D> unused;
        y[j] = flat_unit<S, D, SCALE_NONE, false>(x, unused, 0.f);
      }
      for (int k = 0; k < dsts.n; k++) {
        const TileStore<D, STP> out(reinterpret_cast<char*>(dsts.p[k]) + tile * kTileBytes, kTileBytes);
#pragma unroll
        for (int j = 0; j < U; j++) store_unit_at<D, STP>(out, (int(threadIdx.x) + j * BLOCK) * (8 * D::kSize), y[j]);
      }
    } else {
      for (int64_t u = u0; u < n_units; u += BLOCK) {
        const Unit<S> x = load_unit<S, NTL>(sbase + u * (8 * S::kSize));
        Unit<D> unused;
        const Unit<D> y = flat_unit<S, D, SCALE_NONE, false>(x, unused, 0.f);
        for (int k = 0; k < dsts.n; k++) store_unit<D, NTS>(reinterpret_cast<char*>(dsts.p[k]) + u * (8 * D::kSize), y);
      }
    }
  }
  if (blockIdx.x == 0) {
    const int64_t i = (n_units << 3) + threadIdx.x;
    if (i < n) {
      d_t v;
      if constexpr (same_t<S, D>::value) v = reinterpret_cast<const s_t*>(src)[i];
      else v = from_f32<D>(to_f32<S>(reinterpret_cast<const s_t*>(src)[i]));
      for (int k = 0; k < dsts.n; k++) reinterpret_cast<d_t*>(dsts.p[k])[i] = v;
    }
  }
}

// One element of the fan-in: the chunks are added in binary32 in index order
// (what a reduce-scatter with binary32 accumulation does, bit32_acc in the
// reference, ya_fsdp/_collectives.py:157-161), the sum is rounded to the chunk
// dtype as the collective's output tensor is, then post-divide (:165) and
// copy_ / add_ into the gradient shard (:185 / :189).
//
// SCALE_PREMUL is the collective that scales inside the reduction (ReduceOp.AVG, or the pre-multiplied sum of
// _make_nccl_premul_sum, :243-249): the collective library multiplies every rank's element by the scalar, both in
// the chunk dtype, i.e. rounds each product to that dtype, and adds the products; there is no post-divide then.
template <class S, class D, int SCALE, bool ACC>
__device__ __forceinline__ float fanin_finish(float sum, float d_old, float k) {
  constexpr int kAfterSum = SCALE == SCALE_PREMUL ? SCALE_NONE : SCALE;
  return post_elem<S, D, kAfterSum, ACC>(round_to<S>(sum), d_old, k);
}

// one rank's element as it enters the sum
template <class S, int SCALE>
__device__ __forceinline__ float fanin_term(float x, float k) {
  if constexpr (SCALE == SCALE_PREMUL) return round_to<S>(apply_scale<SCALE_MUL>(x, k));
  else return x;
}

template <class S, class D, int SCALE, bool ACC, int BLOCK, int U, bool NTL, bool NTS>
__global__ void __launch_bounds__(BLOCK)
fanin_kernel(void* shard, FanPtrs chunks, int64_t n, float k) {
  typedef typename S::storage s_t;
  typedef typename D::storage d_t;
  const int64_t n_quads = n >> 2;
  constexpr int64_t kTile = int64_t(BLOCK) * U;
  const int64_t n_tiles = (n_quads + kTile - 1) / kTile;
  char* dbase = reinterpret_cast<char*>(shard);
  for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const int64_t q0 = tile * kTile + threadIdx.x;
    const bool full = tile * kTile + kTile <= n_quads;
#pragma unroll
    for (int j = 0; j < U; j++) {
      const int64_t q = q0 + j * BLOCK;
      if (!full && q >= n_quads) break;
      Quad<S> x[kFanMax];
#pragma unroll
      for (int c = 0; c < kFanMax; c++)
        if (c < chunks.n) x[c] = load_quad<S, NTL>(reinterpret_cast<const char*>(chunks.p[c]) + q * (4 * S::kSize));
      Quad<D> old;
      if constexpr (ACC) old = load_quad<D, NTL>(dbase + q * (4 * D::kSize));
      float sum[4], fo[4] = {0.f, 0.f, 0.f, 0.f}, fy[4];
      unpack_quad<S>(x[0], sum);
#pragma unroll
      for (int e = 0; e < 4; e++) sum[e] = fanin_term<S, SCALE>(sum[e], k);
#pragma unroll
      for (int c = 1; c < kFanMax; c++) {
        if (c < chunks.n) {
          float f[4];
          unpack_quad<S>(x[c], f);
#pragma unroll
          for (int e = 0; e < 4; e++) sum[e] = __fadd_rn(sum[e], fanin_term<S, SCALE>(f[e], k));
        }
      }
      if constexpr (ACC) unpack_quad<D>(old, fo);
#pragma unroll
      for (int e = 0; e < 4; e++) fy[e] = fanin_finish<S, D, SCALE, ACC>(sum[e], fo[e], k);
      store_quad<D, NTS>(dbase + q * (4 * D::kSize), pack_quad<D>(fy));
    }
  }
  if (blockIdx.x == 0) {
    const int64_t i = (n_quads << 2) + threadIdx.x;
    if (i < n) {
      float sum = fanin_term<S, SCALE>(to_f32<S>(reinterpret_cast<const s_t*>(chunks.p[0])[i]), k);
      for (int c = 1; c < chunks.n; c++)
        sum = __fadd_rn(sum, fanin_term<S, SCALE>(to_f32<S>(reinterpret_cast<const s_t*>(chunks.p[c])[i]), k));
      d_t* d = reinterpret_cast<d_t*>(shard) + i;
      float d_old = 0.f;
      if constexpr (ACC) d_old = to_f32<D>(*d);
      *d = from_f32<D>(fanin_finish<S, D, SCALE, ACC>(sum, d_old, k));
    }
  }
}

}  // namespace yafsdp

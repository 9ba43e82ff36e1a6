// Post-reduce (divide + copy / accumulate into the gradient shard, as
// flat_kernel does it) that also returns the sum of squares of what it stored:
// the gradient norm then needs no pass of its own over the shard.
//
// Same tiling, same arithmetic and same stores as flat_kernel.  Every lane
// adds the squares of the values it stores (after rounding to the shard's
// dtype, i.e. exactly what a later read would see) in binary64, where the
// square of a binary32 number is exact; the workgroup's sum goes to
// partials[blockIdx.x].  One workgroup per tile, so the number of partial sums
// and the order of all additions depend only on (n, head).
#pragma once
#include "flat_kernels.hip.h"

namespace yafsdp {

template <class D>
__device__ __forceinline__ double unit_sumsq(const Unit<D>& r, double acc) {
  float f[8];
  unpack<D>(r, f);
#pragma unroll
  for (int e = 0; e < 8; e++) acc = __fma_rn(double(f[e]), double(f[e]), acc);
  return acc;
}

template <class D>
__device__ __forceinline__ double quad_sumsq(const Quad<D>& r, double acc) {
  float f[4];
  unpack_quad<D>(r, f);
#pragma unroll
  for (int e = 0; e < 4; e++) acc = __fma_rn(double(f[e]), double(f[e]), acc);
  return acc;
}

template <class S, class D, int SCALE, bool ACC>
__device__ __forceinline__ double post_scalar_sumsq(void* dst, const void* src, int64_t i, float k) {
  typedef typename S::storage s_t;
  typedef typename D::storage d_t;
  d_t y;
  if constexpr (same_t<S, D>::value && SCALE == SCALE_NONE && !ACC) {
    y = reinterpret_cast<const s_t*>(src)[i];  // byte copy, as flat_scalar
  } else {
    const float s = to_f32<S>(reinterpret_cast<const s_t*>(src)[i]);
    float d_old = 0.f;
    if constexpr (ACC) d_old = to_f32<D>(reinterpret_cast<const d_t*>(dst)[i]);
    y = from_f32<D>(post_elem<S, D, SCALE, ACC>(s, d_old, k));
  }
  reinterpret_cast<d_t*>(dst)[i] = y;
  const float stored = to_f32<D>(y);
  return double(stored) * double(stored);
}

// One full tile of the pass: stores with policy STP, adds the squares of what it stored to acc0 / acc1.
template <class S, class D, int SCALE, bool ACC, int BLOCK, int U, bool NTL, int STP>
__device__ __forceinline__ void post_sumsq_full_tile(char* dt, const char* st, float k, double& acc0, double& acc1) {
  const TileStore<D, STP> out(dt, BLOCK * U * 8 * D::kSize);
  if constexpr (wide_pair<S, D>::value) {
    Quad<S> s[2 * U];
    Quad<D> d[2 * U];
#pragma unroll
    for (int q = 0; q < 2 * U; q++) s[q] = load_quad<S, NTL>(st + quad_elem<BLOCK, U>(q) * S::kSize);
    if constexpr (ACC) {
#pragma unroll
      for (int q = 0; q < 2 * U; q++) d[q] = load_quad<D, NTL>(dt + quad_elem<BLOCK, U>(q) * D::kSize);
    }
#pragma unroll
    for (int q = 0; q < 2 * U; q++) {
      const Quad<D> r = flat_quad<S, D, SCALE, ACC>(s[q], d[q], k);
      store_quad_at<D, STP>(out, quad_elem<BLOCK, U>(q) * D::kSize, r);
      if (q & 1) acc1 = quad_sumsq<D>(r, acc1);
      else acc0 = quad_sumsq<D>(r, acc0);
    }
  } else {
    Unit<S> s[U];
    Unit<D> d[U];
#pragma unroll
    for (int j = 0; j < U; j++) s[j] = load_unit<S, NTL>(st + unit_index<BLOCK, U>(j) * (8 * S::kSize));
    if constexpr (ACC) {
#pragma unroll
      for (int j = 0; j < U; j++) d[j] = load_unit<D, NTL>(dt + unit_index<BLOCK, U>(j) * (8 * D::kSize));
    }
#pragma unroll
    for (int j = 0; j < U; j++) {
      const Unit<D> r = flat_unit<S, D, SCALE, ACC>(s[j], d[j], k);
      store_unit_at<D, STP>(out, unit_index<BLOCK, U>(j) * (8 * D::kSize), r);
      if (j & 1) acc1 = unit_sumsq<D>(r, acc1);
      else acc0 = unit_sumsq<D>(r, acc0);
    }
  }
}

// With STP = ST_WT the full tiles before tile `wt_from` store non-temporal instead (0: every tile writes through),
// as in flat_kernel.
template <class S, class D, int SCALE, bool ACC, int BLOCK, int U, bool NTL, int STP>
__global__ void __launch_bounds__(BLOCK)
post_reduce_sumsq_kernel(void* dst, const void* src, int64_t n, int head, float k, double* partials, int wt_from) {
  __shared__ double lds[BLOCK / 64];
  constexpr bool NTS = (STP == ST_NT);  // the partial last tile keeps ordinary global stores
  const int tid = threadIdx.x;
  const int64_t n_units = (n - head) >> 3;
  const int64_t body_end = head + (n_units << 3);
  double acc0 = 0.0, acc1 = 0.0;
  if (blockIdx.x == 0) {
    if (tid < head) acc0 += post_scalar_sumsq<S, D, SCALE, ACC>(dst, src, tid, k);
    const int tail = int(n - body_end);
    const int t = BLOCK - 1 - tid;
    if (t < tail) acc1 += post_scalar_sumsq<S, D, SCALE, ACC>(dst, src, body_end + t, k);
  }
  char* dbase = reinterpret_cast<char*>(dst) + int64_t(head) * D::kSize;
  const char* sbase = reinterpret_cast<const char*>(src) + int64_t(head) * S::kSize;
  constexpr int64_t kTile = int64_t(BLOCK) * U;
  const int64_t n_tiles = (n_units + kTile - 1) / kTile;
  for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    char* dt = dbase + tile * kTile * (8 * D::kSize);
    const char* st = sbase + tile * kTile * (8 * S::kSize);
    if (tile * kTile + kTile <= n_units) {
      if (STP == ST_WT && tile < wt_from)
        post_sumsq_full_tile<S, D, SCALE, ACC, BLOCK, U, NTL, ST_NT>(dt, st, k, acc0, acc1);
      else
        post_sumsq_full_tile<S, D, SCALE, ACC, BLOCK, U, NTL, STP>(dt, st, k, acc0, acc1);
    } else {  // last, partial tile
      for (int64_t u = tile * kTile + tid; u < n_units; u += BLOCK) {
        Unit<S> s = load_unit<S, NTL>(sbase + u * (8 * S::kSize));
        Unit<D> d;
        if constexpr (ACC) d = load_unit<D, NTL>(dbase + u * (8 * D::kSize));
        const Unit<D> r = flat_unit<S, D, SCALE, ACC>(s, d, k);
        store_unit<D, NTS>(dbase + u * (8 * D::kSize), r);
        acc0 = unit_sumsq<D>(r, acc0);
      }
    }
  }
  const double total = block_sum<BLOCK>(acc0 + acc1, lds);
  if (tid == 0) partials[blockIdx.x] = total;
}

}  // namespace yafsdp

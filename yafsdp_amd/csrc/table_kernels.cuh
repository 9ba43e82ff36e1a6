// Multi-tensor kernels of the buffer path, driven by a device-resident table:
//   gather-in   P tensors  -> flat reduce buffer   (reduce copy-in: copy / add /
//               absent per tensor, fused pre-divide, pad zero-fill)
//   scatter-out flat gathered buffer -> P tensors   (materialising copy-out)
//
// The flat buffer is cut into tiles of BLOCK*U units (a unit is 8 elements).
// `tile_first[t]` names the tensor that holds the tile's first element (the
// first tensor whose end lies beyond it; n_tensors when the tile starts in the
// pad), so a workgroup finds its work with one table read instead of a search.
// A tile that lies wholly inside one tensor takes the unrolled path: U
// dwordx4-wide loads per lane in flight, flat side 16-byte aligned, tensor side
// at whatever element-aligned address the ragged offset gives.  A tile that
// crosses tensor boundaries (or the end of the buffer) walks its segments; each
// segment peels up to 7 elements on either end so that its unit loop is again
// aligned on the flat side.
//
// Tensor base pointers and per-tensor modes change every call (autograd
// allocates gradients afresh), so they travel outside the static table: in the
// kernel arguments for up to kKargMax tensors, else through a small device
// array the host refreshes on the same stream before the launch.
#pragma once
#include "flat_kernels.cuh"

namespace yafsdp {

constexpr int kKargMax = 32;
enum : int { MODE_ZERO = 3 };  // internal: fill with zeros (pad lanes)

struct DynArgs {
  const void* ptr[kKargMax];
  uint8_t mode[kKargMax];
  const void* const* dev_ptr;  // non-null when the table has more than kKargMax tensors
  const uint8_t* dev_mode;
};

struct TableView {
  const int64_t* offsets;     // n_tensors + 1 prefix offsets (elements), offsets[n_tensors] == total
  const int32_t* tile_first;  // n_tiles entries
  int64_t total;              // T
  int64_t padded;             // T_pad
  int32_t n_tensors;
  int32_t n_tiles;
};

__device__ __forceinline__ const void* dyn_ptr(const DynArgs& a, int p) {
  return a.dev_ptr != nullptr ? a.dev_ptr[p] : a.ptr[p];
}
__device__ __forceinline__ int dyn_mode(const DynArgs& a, int p) {
  return a.dev_ptr != nullptr ? a.dev_mode[p] : a.mode[p];
}

// ------------------------------------------------------------------ gather-in --
template <class S, class D, int SCALE, int MODE>
__device__ __forceinline__ void gather_scalar(void* dst, const void* src, int64_t i, float k) {
  typedef typename S::storage s_t;
  typedef typename D::storage d_t;
  d_t* d = reinterpret_cast<d_t*>(dst) + i;
  if constexpr (MODE == MODE_ZERO) {
    *d = d_t(0);
  } else if constexpr (MODE == MODE_COPY && same_t<S, D>::value && SCALE == SCALE_NONE) {
    *d = reinterpret_cast<const s_t*>(src)[i];
  } else {
    float s = 0.f, d_old = 0.f;
    if constexpr (MODE != MODE_SKIP) s = to_f32<S>(reinterpret_cast<const s_t*>(src)[i]);
    if constexpr (MODE != MODE_COPY) d_old = to_f32<D>(*d);
    *d = from_f32<D>(gather_elem<S, D, SCALE, MODE>(s, d_old, k));
  }
}

template <class S, class D, int SCALE, int MODE>
__device__ __forceinline__ Unit<D> gather_unit(const Unit<S>& s, const Unit<D>& d_old, float k) {
  if constexpr (MODE == MODE_ZERO) {
    Unit<D> z;
#pragma unroll
    for (int i = 0; i < D::kVecs; i++) z.v[i] = u32x4{0u, 0u, 0u, 0u};
    return z;
  } else if constexpr (MODE == MODE_COPY && same_t<S, D>::value && SCALE == SCALE_NONE) {
    return s;
  } else {
    float fs[8], fd[8], fy[8];
    if constexpr (MODE != MODE_SKIP) unpack<S>(s, fs);
    if constexpr (MODE != MODE_COPY) unpack<D>(d_old, fd);
#pragma unroll
    for (int e = 0; e < 8; e++)
      fy[e] = gather_elem<S, D, SCALE, MODE>(MODE != MODE_SKIP ? fs[e] : 0.f, MODE != MODE_COPY ? fd[e] : 0.f, k);
    return pack<D>(fy);
  }
}

template <class S, class D, int SCALE, int MODE, int BLOCK, int U, bool NTL, bool NTS>
__device__ __forceinline__ void gather_full_tile(char* dst, const char* src, float k) {
  constexpr bool kReadSrc = (MODE == MODE_COPY || MODE == MODE_ADD);
  constexpr bool kReadDst = (MODE == MODE_ADD || MODE == MODE_SKIP);
  const int tid = threadIdx.x;
  Unit<S> s[U];
  Unit<D> d[U];
  if constexpr (kReadSrc) {
#pragma unroll
    for (int j = 0; j < U; j++) s[j] = load_unit<S, NTL>(src + (tid + j * BLOCK) * (8 * S::kSize));
  }
  if constexpr (kReadDst) {
#pragma unroll
    for (int j = 0; j < U; j++) d[j] = load_unit<D, NTL>(dst + (tid + j * BLOCK) * (8 * D::kSize));
  }
#pragma unroll
  for (int j = 0; j < U; j++)
    store_unit<D, NTS>(dst + (tid + j * BLOCK) * (8 * D::kSize), gather_unit<S, D, SCALE, MODE>(s[j], d[j], k));
}

// n elements; dst points at flat element `flat_index`, src at the matching
// tensor element.
template <class S, class D, int SCALE, int MODE, int BLOCK, bool NTL, bool NTS>
__device__ __forceinline__ void gather_segment(char* dst, const char* src, int64_t n, int64_t flat_index, float k) {
  constexpr bool kReadSrc = (MODE == MODE_COPY || MODE == MODE_ADD);
  constexpr bool kReadDst = (MODE == MODE_ADD || MODE == MODE_SKIP);
  const int tid = threadIdx.x;
  int64_t head = (8 - (flat_index & 7)) & 7;
  if (head > n) head = n;
  const int64_t units = (n - head) >> 3;
  const int64_t body_end = head + (units << 3);
  const int tail = int(n - body_end);
  if (tid < head) gather_scalar<S, D, SCALE, MODE>(dst, src, tid, k);
  const int t = BLOCK - 1 - tid;
  if (t < tail) gather_scalar<S, D, SCALE, MODE>(dst, src, body_end + t, k);
  char* db = dst + head * D::kSize;
  const char* sb = src + head * S::kSize;
  for (int64_t u = tid; u < units; u += BLOCK) {
    Unit<S> s;
    Unit<D> d;
    if constexpr (kReadSrc) s = load_unit<S, NTL>(sb + u * (8 * S::kSize));
    if constexpr (kReadDst) d = load_unit<D, NTL>(db + u * (8 * D::kSize));
    store_unit<D, NTS>(db + u * (8 * D::kSize), gather_unit<S, D, SCALE, MODE>(s, d, k));
  }
}

// S: tensor dtype, D: flat buffer dtype.  pad_zero != 0 writes zeros to
// [total, padded); otherwise pad lanes only see the divide (as in the
// reference, whose pad content is whatever the buffer held).
template <class S, class D, int SCALE, int BLOCK, int U, bool NTL, bool NTS>
__global__ void __launch_bounds__(BLOCK)
gather_in_kernel(TableView tv, DynArgs dyn, void* flat, float k, int pad_zero) {
  constexpr int64_t kTile = int64_t(BLOCK) * U * 8;
  char* fbase = reinterpret_cast<char*>(flat);
  for (int tile = blockIdx.x; tile < tv.n_tiles; tile += gridDim.x) {
    const int64_t t0 = int64_t(tile) * kTile;
    const int64_t t1 = (t0 + kTile < tv.padded) ? t0 + kTile : tv.padded;
    int p = tv.tile_first[tile];
    if (p < tv.n_tensors) {
      const int64_t o0 = tv.offsets[p];
      const int64_t o1 = tv.offsets[p + 1];
      if (o1 - t0 >= kTile) {  // the whole tile lies inside tensor p
        const int mode = dyn_mode(dyn, p);
        const char* src = reinterpret_cast<const char*>(dyn_ptr(dyn, p)) + (t0 - o0) * S::kSize;
        char* dst = fbase + t0 * D::kSize;
        if (mode == MODE_COPY) gather_full_tile<S, D, SCALE, MODE_COPY, BLOCK, U, NTL, NTS>(dst, src, k);
        else if (mode == MODE_ADD) gather_full_tile<S, D, SCALE, MODE_ADD, BLOCK, U, NTL, NTS>(dst, src, k);
        else if (SCALE != SCALE_NONE) gather_full_tile<S, D, SCALE, MODE_SKIP, BLOCK, U, NTL, NTS>(dst, src, k);
        continue;
      }
    }
    int64_t pos = t0;
    while (pos < t1) {
      if (p >= tv.n_tensors) {  // pad lanes
        char* dst = fbase + pos * D::kSize;
        if (pad_zero) gather_segment<S, D, SCALE, MODE_ZERO, BLOCK, NTL, NTS>(dst, nullptr, t1 - pos, pos, k);
        else if (SCALE != SCALE_NONE) gather_segment<S, D, SCALE, MODE_SKIP, BLOCK, NTL, NTS>(dst, nullptr, t1 - pos, pos, k);
        break;
      }
      const int64_t o1 = tv.offsets[p + 1];
      if (o1 <= pos) { ++p; continue; }  // empty tensor
      const int64_t o0 = tv.offsets[p];
      const int64_t e = o1 < t1 ? o1 : t1;
      const int mode = dyn_mode(dyn, p);
      const char* src = reinterpret_cast<const char*>(dyn_ptr(dyn, p)) + (pos - o0) * S::kSize;
      char* dst = fbase + pos * D::kSize;
      if (mode == MODE_COPY) gather_segment<S, D, SCALE, MODE_COPY, BLOCK, NTL, NTS>(dst, src, e - pos, pos, k);
      else if (mode == MODE_ADD) gather_segment<S, D, SCALE, MODE_ADD, BLOCK, NTL, NTS>(dst, src, e - pos, pos, k);
      else if (SCALE != SCALE_NONE) gather_segment<S, D, SCALE, MODE_SKIP, BLOCK, NTL, NTS>(dst, src, e - pos, pos, k);
      pos = e;
      if (e == o1) ++p;
    }
  }
}

// ---------------------------------------------------------------- scatter-out --
template <class S, class D, int BLOCK, int U, bool NTL, bool NTS>
__device__ __forceinline__ void scatter_full_tile(char* dst, const char* src) {
  const int tid = threadIdx.x;
  Unit<S> s[U];
  Unit<D> unused;
#pragma unroll
  for (int j = 0; j < U; j++) s[j] = load_unit<S, NTL>(src + (tid + j * BLOCK) * (8 * S::kSize));
#pragma unroll
  for (int j = 0; j < U; j++)
    store_unit<D, NTS>(dst + (tid + j * BLOCK) * (8 * D::kSize), flat_unit<S, D, SCALE_NONE, false>(s[j], unused, 0.f));
}

template <class S, class D, int BLOCK, bool NTL, bool NTS>
__device__ __forceinline__ void scatter_segment(char* dst, const char* src, int64_t n, int64_t flat_index) {
  const int tid = threadIdx.x;
  int64_t head = (8 - (flat_index & 7)) & 7;
  if (head > n) head = n;
  const int64_t units = (n - head) >> 3;
  const int64_t body_end = head + (units << 3);
  const int tail = int(n - body_end);
  if (tid < head) flat_scalar<S, D, SCALE_NONE, false>(dst, src, tid, 0.f);
  const int t = BLOCK - 1 - tid;
  if (t < tail) flat_scalar<S, D, SCALE_NONE, false>(dst, src, body_end + t, 0.f);
  char* db = dst + head * D::kSize;
  const char* sb = src + head * S::kSize;
  Unit<D> unused;
  for (int64_t u = tid; u < units; u += BLOCK) {
    Unit<S> s = load_unit<S, NTL>(sb + u * (8 * S::kSize));
    store_unit<D, NTS>(db + u * (8 * D::kSize), flat_unit<S, D, SCALE_NONE, false>(s, unused, 0.f));
  }
}

// S: flat buffer dtype, D: tensor dtype.  Tensors with mode 0 are not written.
template <class S, class D, int BLOCK, int U, bool NTL, bool NTS>
__global__ void __launch_bounds__(BLOCK)
scatter_out_kernel(TableView tv, DynArgs dyn, const void* flat) {
  constexpr int64_t kTile = int64_t(BLOCK) * U * 8;
  const char* fbase = reinterpret_cast<const char*>(flat);
  for (int tile = blockIdx.x; tile < tv.n_tiles; tile += gridDim.x) {
    const int64_t t0 = int64_t(tile) * kTile;
    const int64_t t1 = (t0 + kTile < tv.total) ? t0 + kTile : tv.total;  // pad lanes are never read
    int p = tv.tile_first[tile];
    if (p >= tv.n_tensors) continue;
    {
      const int64_t o0 = tv.offsets[p];
      const int64_t o1 = tv.offsets[p + 1];
      if (o1 - t0 >= kTile) {
        if (dyn_mode(dyn, p) != MODE_SKIP) {
          char* dst = reinterpret_cast<char*>(const_cast<void*>(dyn_ptr(dyn, p))) + (t0 - o0) * D::kSize;
          scatter_full_tile<S, D, BLOCK, U, NTL, NTS>(dst, fbase + t0 * S::kSize);
        }
        continue;
      }
    }
    int64_t pos = t0;
    while (pos < t1 && p < tv.n_tensors) {
      const int64_t o1 = tv.offsets[p + 1];
      if (o1 <= pos) { ++p; continue; }
      const int64_t o0 = tv.offsets[p];
      const int64_t e = o1 < t1 ? o1 : t1;
      if (dyn_mode(dyn, p) != MODE_SKIP) {
        char* dst = reinterpret_cast<char*>(const_cast<void*>(dyn_ptr(dyn, p))) + (pos - o0) * D::kSize;
        scatter_segment<S, D, BLOCK, NTL, NTS>(dst, fbase + pos * S::kSize, e - pos, pos);
      }
      pos = e;
      if (e == o1) ++p;
    }
  }
}

}  // namespace yafsdp

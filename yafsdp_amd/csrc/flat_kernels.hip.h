// Flat (one contiguous range -> one contiguous range) kernels of the buffer
// path: copy-in cast, single-rank all-gather/reduce-scatter copies, in-place
// pre/post divide, and the fused post-reduce (divide + copy/accumulate into the
// gradient shard).
//
// Work partitioning: the range is cut into tiles of BLOCK*U units (a unit is 8
// elements), one workgroup per tile (grid-stride if the grid is capped).
//  * pairs of 2-byte dtypes: lane l touches units l, l+BLOCK, ...: every wave64
//    access is one contiguous 1 KiB span;
//  * pairs with an fp32 side: quad arrangement (see elem.hip.h): every wave64
//    access is a contiguous 1 KiB (fp32) or 512 B (2-byte) span.
// All loads of a lane are issued before its first store.  The destination is
// aligned for the tile loop: the host peels the leading elements up to its next
// 128-byte line (fewer than 64; 16-byte alignment is what the kernel needs, the
// line keeps two workgroups from writing into one cache line), handled by
// workgroup 0 together with the tail; the source may sit at any element-aligned
// address.
#pragma once
#include "elem.hip.h"
#include "tuning.h"

namespace yafsdp {

template <class S, class D, int SCALE, bool ACC>
__device__ __forceinline__ void flat_scalar(void* dst, const void* src, int64_t i, float k) {
  typedef typename S::storage s_t;
  typedef typename D::storage d_t;
  if constexpr (same_t<S, D>::value && SCALE == SCALE_NONE && !ACC) {
    reinterpret_cast<d_t*>(dst)[i] = reinterpret_cast<const s_t*>(src)[i];
  } else {
    float s = to_f32<S>(reinterpret_cast<const s_t*>(src)[i]);
    float d_old = 0.f;
    if constexpr (ACC) d_old = to_f32<D>(reinterpret_cast<const d_t*>(dst)[i]);
    reinterpret_cast<d_t*>(dst)[i] = from_f32<D>(post_elem<S, D, SCALE, ACC>(s, d_old, k));
  }
}

template <class S, class D, int SCALE, bool ACC>
__device__ __forceinline__ Unit<D> flat_unit(const Unit<S>& s, const Unit<D>& d_old, float k) {
  if constexpr (same_t<S, D>::value && SCALE == SCALE_NONE && !ACC) {
    return s;  // byte copy: NaN payloads and all bit patterns pass through
  } else {
    float fs[8], fd[8], fy[8];
    unpack<S>(s, fs);
    if constexpr (ACC) unpack<D>(d_old, fd);
#pragma unroll
    for (int e = 0; e < 8; e++) fy[e] = post_elem<S, D, SCALE, ACC>(fs[e], ACC ? fd[e] : 0.f, k);
    return pack<D>(fy);
  }
}

template <class S, class D, int SCALE, bool ACC>
__device__ __forceinline__ Quad<D> flat_quad(const Quad<S>& s, const Quad<D>& d_old, float k) {
  if constexpr (same_t<S, D>::value && SCALE == SCALE_NONE && !ACC) {
    return s;
  } else {
    float fs[4], fd[4], fy[4];
    unpack_quad<S>(s, fs);
    if constexpr (ACC) unpack_quad<D>(d_old, fd);
#pragma unroll
    for (int e = 0; e < 4; e++) fy[e] = post_elem<S, D, SCALE, ACC>(fs[e], ACC ? fd[e] : 0.f, k);
    return pack_quad<D>(fy);
  }
}

// One full tile (BLOCK*U units) at dst/src; dst 16-byte aligned.  STP: store policy (ST_PLAIN / ST_NT / ST_WT).
template <class S, class D, int SCALE, bool ACC, int BLOCK, int U, bool NTL, int STP>
__device__ __forceinline__ void flat_full_tile(char* dst, const char* src, float k) {
  const TileStore<D, STP> out(dst, BLOCK * U * 8 * D::kSize);
  if constexpr (wide_pair<S, D>::value) {
    Quad<S> s[2 * U];
    Quad<D> d[2 * U];
#pragma unroll
    for (int q = 0; q < 2 * U; q++) s[q] = load_quad<S, NTL>(src + quad_elem<BLOCK, U>(q) * S::kSize);
    if constexpr (ACC) {
#pragma unroll
      for (int q = 0; q < 2 * U; q++) d[q] = load_quad<D, NTL>(dst + quad_elem<BLOCK, U>(q) * D::kSize);
    }
#pragma unroll
    for (int q = 0; q < 2 * U; q++)
      store_quad_at<D, STP>(out, quad_elem<BLOCK, U>(q) * D::kSize, flat_quad<S, D, SCALE, ACC>(s[q], d[q], k));
  } else {
    Unit<S> s[U];
    Unit<D> d[U];
#pragma unroll
    for (int j = 0; j < U; j++) s[j] = load_unit<S, NTL>(src + unit_index<BLOCK, U>(j) * (8 * S::kSize));
    if constexpr (ACC) {
#pragma unroll
      for (int j = 0; j < U; j++) d[j] = load_unit<D, NTL>(dst + unit_index<BLOCK, U>(j) * (8 * D::kSize));
    }
#pragma unroll
    for (int j = 0; j < U; j++)
      store_unit_at<D, STP>(out, unit_index<BLOCK, U>(j) * (8 * D::kSize), flat_unit<S, D, SCALE, ACC>(s[j], d[j], k));
  }
}

// dst[i] = op(src[i], dst[i]) for i in [0, n).  `head` leading elements bring
// dst to a 16-byte boundary.  dst == src is allowed (in-place divide).
// `trace` (normally null) is a measurement hook: workgroup b stores the 100 MHz
// wall-clock count at its start and, after its stores have been acknowledged,
// at its end into trace[2 b], trace[2 b + 1].
// The flat pass as seen by workgroup `block` of `n_blocks` (the whole grid of flat_kernel, or the part of a
// larger grid that serves this job).  With STP = ST_WT the full tiles before tile `wt_from` store non-temporal
// instead (0: every tile writes through).
template <class S, class D, int SCALE, bool ACC, int BLOCK, int U, bool NTL, int STP>
__device__ __forceinline__ void flat_body(void* dst, const void* src, int64_t n, int head, float k, int block,
                                          int n_blocks, int wt_from) {
  const int tid = threadIdx.x;
  const int64_t n_units = (n - head) >> 3;
  const int64_t body_end = head + (n_units << 3);
  if (block == 0) {
    if (tid < head) flat_scalar<S, D, SCALE, ACC>(dst, src, tid, k);
    const int tail = int(n - body_end);
    const int t = BLOCK - 1 - tid;
    if (t < tail) flat_scalar<S, D, SCALE, ACC>(dst, src, body_end + t, k);
  }
  char* dbase = reinterpret_cast<char*>(dst) + int64_t(head) * D::kSize;
  const char* sbase = reinterpret_cast<const char*>(src) + int64_t(head) * S::kSize;
  constexpr int64_t kTile = int64_t(BLOCK) * U;
  const int64_t n_tiles = (n_units + kTile - 1) / kTile;
  for (int64_t tile = block; tile < n_tiles; tile += n_blocks) {
    if (tile * kTile + kTile <= n_units) {
      if (STP == ST_WT && tile < wt_from)  // before the write-through part of the output (see tuning.h)
        flat_full_tile<S, D, SCALE, ACC, BLOCK, U, NTL, ST_NT>(dbase + tile * kTile * (8 * D::kSize),
                                                               sbase + tile * kTile * (8 * S::kSize), k);
      else
        flat_full_tile<S, D, SCALE, ACC, BLOCK, U, NTL, STP>(dbase + tile * kTile * (8 * D::kSize),
                                                             sbase + tile * kTile * (8 * S::kSize), k);
    } else {  // last, partial tile
      for (int64_t u = tile * kTile + tid; u < n_units; u += BLOCK) {
        Unit<S> s = load_unit<S, NTL>(sbase + u * (8 * S::kSize));
        Unit<D> d;
        if constexpr (ACC) d = load_unit<D, NTL>(dbase + u * (8 * D::kSize));
        store_unit<D, STP == ST_NT>(dbase + u * (8 * D::kSize), flat_unit<S, D, SCALE, ACC>(s, d, k));
      }
    }
  }
}

template <class S, class D, int SCALE, bool ACC, int BLOCK, int U, bool NTL, int STP>
__global__ void __launch_bounds__(BLOCK)
flat_kernel(void* dst, const void* src, int64_t n, int head, float k, unsigned long long* trace, int wt_from) {
  unsigned long long t_start = 0;
  if (trace != nullptr) t_start = wall_clock64();
  flat_body<S, D, SCALE, ACC, BLOCK, U, NTL, STP>(dst, src, n, head, k, int(blockIdx.x), int(gridDim.x), wt_from);
  if (trace != nullptr) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // every load has arrived, every store is acknowledged
    if (threadIdx.x == 0) {
      trace[2 * blockIdx.x] = t_start;
      trace[2 * blockIdx.x + 1] = wall_clock64();
    }
  }
}

// ---- opaque bytes ------------------------------------------------------------
// dst[0:n] = src[0:n] for byte ranges at ANY byte address: the same-dtype copy of
// 1-byte element types (fp8, int8, uint8), whose ragged per-parameter fragments
// start and end at odd addresses.  `head` (0..127, at most BLOCK) leading bytes bring dst
// to a 128-byte line; the body is 16-byte vectors, one per lane and tile (aligned
// stores; the loads sit at whatever byte alignment the two addresses leave, which
// the hardware serves natively like the element-aligned loads of the other
// kernels); workgroup 0 also copies the head and the up to 15 trailing bytes.
typedef u32x4 u32x4_a1 __attribute__((aligned(1)));

template <int BLOCK, bool NTL, int STP>
__global__ void __launch_bounds__(BLOCK)
bytes_kernel(void* dst, const void* src, int64_t n, int head, int wt_from) {
  static_assert(BLOCK >= 128, "workgroup 0 copies up to 127 leading bytes, one per lane");
  const int tid = threadIdx.x;
  const int64_t n_vecs = (n - head) >> 4;
  const int64_t body_end = head + (n_vecs << 4);
  uint8_t* d8 = reinterpret_cast<uint8_t*>(dst);
  const uint8_t* s8 = reinterpret_cast<const uint8_t*>(src);
  if (blockIdx.x == 0) {
    if (tid < head) d8[tid] = s8[tid];
    const int tail = int(n - body_end);
    const int t = BLOCK - 1 - tid;
    if (t < tail) d8[body_end + t] = s8[body_end + t];
  }
  char* dbase = reinterpret_cast<char*>(dst) + head;
  const char* sbase = reinterpret_cast<const char*>(src) + head;
  const int64_t n_tiles = (n_vecs + BLOCK - 1) / BLOCK;
  for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const int64_t v = tile * BLOCK + tid;
    if (tile * BLOCK + BLOCK <= n_vecs) {
      const u32x4_a1* q = reinterpret_cast<const u32x4_a1*>(sbase + v * 16);
      u32x4 x;
      if constexpr (NTL) x = __builtin_nontemporal_load(q);
      else x = *q;
      if (STP == ST_WT && tile < wt_from) {  // before the write-through part of the output, as in flat_body
        const TileStore<BF16, ST_NT> out(dbase + tile * BLOCK * 16, BLOCK * 16);
        out.vec(tid * 16, x);
      } else {
        const TileStore<BF16, STP> out(dbase + tile * BLOCK * 16, BLOCK * 16);
        out.vec(tid * 16, x);
      }
    } else if (v < n_vecs) {  // last, partial tile
      const u32x4 x = *reinterpret_cast<const u32x4_a1*>(sbase + v * 16);
      *reinterpret_cast<u32x4*>(dbase + v * 16) = x;
    }
  }
}

}  // namespace yafsdp

// Multi-tensor kernels of the buffer path, driven by a device-resident table:
//   gather-in   P tensors  -> flat reduce buffer   (reduce copy-in: copy / add /
//               absent per tensor, fused pre-divide, pad zero-fill)
//   scatter-out flat gathered buffer -> P tensors   (materialising copy-out)
//
// The flat buffer is cut into tiles of BLOCK*U units (a unit is 8 elements),
// one workgroup per tile.  A workgroup first learns which tensor holds the
// tile's first element (the first tensor whose end lies beyond it; n_tensors
// when the tile starts in the pad), whether the whole tile lies inside that
// tensor, and the tile's element offset inside it.
// A tile that lies wholly inside one tensor takes the unrolled path: all loads
// of a lane in flight before its first store, flat side 16-byte aligned, tensor
// side at whatever element-aligned address the ragged offset gives.  A tile
// that crosses tensor boundaries (or the end of the buffer) walks its segments;
// each segment peels up to 7 elements on either end so that its unit loop is
// again aligned on the flat side.
//
// Scatter-out tiles the DESTINATION instead: tile j of tensor p covers the
// elements of p between two consecutive multiples of the tile size counted from
// the 128-byte line that holds the tensor's first element, so no two workgroups
// ever write the same cache line and every 16-byte store is aligned; the flat
// side is then read at whatever alignment results (unaligned loads are nearly
// free, unaligned stores and shared lines are not).  Every non-empty tensor owns
// ceil(numel / tile) + 1 tile slots, whatever its address (the last slot is
// empty when the tensor starts on a line boundary), so the slot table does not
// depend on the per-call pointers.
//
// Metadata reaches a workgroup through scalar loads only (one tile is one
// wave-uniform lookup), by one of two routes:
//  * SmallMeta (up to kSmallMax tensors, e.g. one decoder layer): tensor
//    pointers, modes, prefix offsets and each tensor's first tile travel in the
//    kernel arguments; the tile -> tensor search is a handful of scalar compares
//    and nothing is read from global memory before the data itself.
//  * LargeMeta: the static part (prefix offsets, one 16-byte record per tile:
//    first tensor, whole-tile flag, offset inside that tensor) is device
//    resident and built once per table; the per-call part (tensor pointers and
//    modes, which change every call because autograd allocates gradients
//    afresh) is refreshed by the host on the same stream before the launch.
//    All of it is read through the constant address space, i.e. as scalar loads.
#pragma once
#include "flat_kernels.hip.h"
#include "tuning.h"

namespace yafsdp {

constexpr int kSmallMax = 16;
// tables with at most this many tensors take the SmallMeta route (at most kSmallMax: the arrays' size).  Sending
// a 9-tensor layer through per-tile records instead measured 1 us slower per table kernel and 13 us slower per
// step (the staging of pointers).
constexpr int kSmallRoute = 16;
static_assert(kSmallRoute >= 0 && kSmallRoute <= kSmallMax, "SmallMeta holds at most kSmallMax tensors");
enum : int { MODE_ZERO = 3 };  // internal: fill with zeros (pad lanes)

struct TileRec {
  int32_t first;  // tensor holding the tile's first element, n_tensors if in the pad
  int32_t full;   // 1 when the whole tile lies inside tensor `first`
  int64_t delta;  // tile start minus start of tensor `first` (elements)
};

struct TileLookup {
  int first;
  bool full;
  int64_t delta;
  const void* base;  // tensor `first` (unspecified for a tile that starts in the pad)
  int mode;          // its mode
};

struct ScatterLookup {
  int tensor;   // n_tensors or more: nothing to do
  int index;    // tile slot inside the tensor
};

#define YAFSDP_CONST_AS __attribute__((address_space(4)))

struct SmallMeta {
  const void* ptr[kSmallMax];
  int64_t off[kSmallMax + 1];         // prefix offsets; entries past n_tensors repeat the total
  int32_t tile_start[kSmallMax + 1];  // ceil(off[i] / tile elements); INT32_MAX past n_tensors
  int32_t slot_start[kSmallMax + 1];  // scatter-out: first tile slot of tensor i; INT32_MAX past n_tensors
  uint32_t modes;                     // 2 bits per tensor
  int32_t n_tensors;

  __device__ __forceinline__ ScatterLookup lookup_scatter(int tile) const {
    int p = 0;
#pragma unroll
    for (int i = 1; i <= kSmallMax; i++) p += (slot_start[i] <= tile) ? 1 : 0;
    ScatterLookup r;
    r.tensor = p;
    r.index = tile - slot_start[p < kSmallMax ? p : kSmallMax - 1];
    return r;
  }

  __device__ __forceinline__ TileLookup lookup(int tile, int64_t t0, int64_t tile_elems) const {
    // tile_start is ascending: the last i with tile_start[i] <= tile is the tensor (a chain of scalar selects)
    int p = 0;
#pragma unroll
    for (int i = 1; i <= kSmallMax; i++) p = (tile_start[i] <= tile) ? i : p;
    TileLookup r;
    r.first = p;
    // the three loads that depend on p leave together, before anything branches on their results
    const int pc = p < kSmallMax ? p : kSmallMax - 1;
    const int64_t o0 = off[p];
    const int64_t o1 = off[pc + 1];
    r.base = ptr[pc];
    // (the empty statement reads the three values here, so that the compiler cannot sink each load to the branch
    // that first uses it, where it would wait for them one after the other; they are inputs only, which keeps
    // the pointer's address space known: global loads, not flat ones)
    asm volatile("" ::"s"(o0), "s"(o1), "s"(r.base));
    r.mode = int((modes >> (2 * pc)) & 3u);
    r.full = p < n_tensors && (o1 - t0 >= tile_elems);
    r.delta = t0 - o0;
    return r;
  }
  __device__ __forceinline__ const void* tensor(int p) const { return ptr[p]; }
  __device__ __forceinline__ int mode(int p) const { return int((modes >> (2 * p)) & 3u); }
  __device__ __forceinline__ int64_t offset(int p) const { return off[p]; }
};

struct LargeMeta {
  const int64_t* offsets;    // n_tensors + 1 prefix offsets (elements)
  const TileRec* tiles;      // n_tiles records (gather-in: tiles of the flat buffer)
  const TileRec* slots;      // scatter-out tile slots: first = tensor, delta = slot index inside it
  const void* const* ptrs;   // n_tensors device pointers (per call)
  const uint32_t* modes_;    // n_tensors modes (per call)
  int32_t n_tensors;

  __device__ __forceinline__ TileLookup lookup(int tile, int64_t, int64_t) const {
    typedef const TileRec YAFSDP_CONST_AS* cptr;
    const cptr t = (cptr)(uintptr_t)tiles;
    TileLookup r;
    r.first = t[tile].first;
    r.full = t[tile].full != 0;
    r.delta = t[tile].delta;
    const int pc = r.first < n_tensors ? r.first : (n_tensors > 0 ? n_tensors - 1 : 0);
    r.base = n_tensors > 0 ? tensor(pc) : nullptr;
    r.mode = n_tensors > 0 ? mode(pc) : 0;
    return r;
  }
  __device__ __forceinline__ ScatterLookup lookup_scatter(int tile) const {
    typedef const TileRec YAFSDP_CONST_AS* cptr;
    const cptr t = (cptr)(uintptr_t)slots;
    ScatterLookup r;
    r.tensor = t[tile].first;
    r.index = int(t[tile].delta);
    return r;
  }
  __device__ __forceinline__ const void* tensor(int p) const {
    typedef const void* const YAFSDP_CONST_AS* cptr;
    return ((cptr)(uintptr_t)ptrs)[p];
  }
  __device__ __forceinline__ int mode(int p) const {
    typedef const uint32_t YAFSDP_CONST_AS* cptr;
    return int(((cptr)(uintptr_t)modes_)[p]);
  }
  __device__ __forceinline__ int64_t offset(int p) const {
    typedef const int64_t YAFSDP_CONST_AS* cptr;
    return ((cptr)(uintptr_t)offsets)[p];
  }
};

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

template <class S, class D, int SCALE, int MODE>
__device__ __forceinline__ Quad<D> gather_quad(const Quad<S>& s, const Quad<D>& d_old, float k) {
  if constexpr (MODE == MODE_COPY && same_t<S, D>::value && SCALE == SCALE_NONE) {
    return s;
  } else {
    float fs[4], fd[4], fy[4];
    if constexpr (MODE != MODE_SKIP) unpack_quad<S>(s, fs);
    if constexpr (MODE != MODE_COPY) unpack_quad<D>(d_old, fd);
#pragma unroll
    for (int e = 0; e < 4; e++)
      fy[e] = gather_elem<S, D, SCALE, MODE>(MODE != MODE_SKIP ? fs[e] : 0.f, MODE != MODE_COPY ? fd[e] : 0.f, k);
    return pack_quad<D>(fy);
  }
}

template <class S, class D, int SCALE, int MODE, int BLOCK, int U, bool NTL, int STP>
__device__ __forceinline__ void gather_full_tile(char* dst, const char* src, float k) {
  constexpr bool kReadSrc = (MODE == MODE_COPY || MODE == MODE_ADD);
  constexpr bool kReadDst = (MODE == MODE_ADD || MODE == MODE_SKIP);
  const TileStore<D, STP> out(dst, BLOCK * U * 8 * D::kSize);
  if constexpr (wide_pair<S, D>::value) {
    Quad<S> s[2 * U];
    Quad<D> d[2 * U];
    if constexpr (kReadSrc) {
#pragma unroll
      for (int q = 0; q < 2 * U; q++) s[q] = load_quad<S, NTL>(src + quad_elem<BLOCK, U>(q) * S::kSize);
    }
    if constexpr (kReadDst) {
#pragma unroll
      for (int q = 0; q < 2 * U; q++) d[q] = load_quad<D, NTL>(dst + quad_elem<BLOCK, U>(q) * D::kSize);
    }
#pragma unroll
    for (int q = 0; q < 2 * U; q++)
      store_quad_at<D, STP>(out, quad_elem<BLOCK, U>(q) * D::kSize, gather_quad<S, D, SCALE, MODE>(s[q], d[q], k));
    return;
  }
  Unit<S> s[U];
  Unit<D> d[U];
  if constexpr (kReadSrc) {
#pragma unroll
    for (int j = 0; j < U; j++) s[j] = load_unit<S, NTL>(src + unit_index<BLOCK, U>(j) * (8 * S::kSize));
  }
  if constexpr (kReadDst) {
#pragma unroll
    for (int j = 0; j < U; j++) d[j] = load_unit<D, NTL>(dst + unit_index<BLOCK, U>(j) * (8 * D::kSize));
  }
#pragma unroll
  for (int j = 0; j < U; j++)
    store_unit_at<D, STP>(out, unit_index<BLOCK, U>(j) * (8 * D::kSize), gather_unit<S, D, SCALE, MODE>(s[j], d[j], k));
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

// a full tile of gather-in under the (wave-uniform) mode of its tensor; a skipped tensor's lanes still see the divide
template <class S, class D, int SCALE, int BLOCK, int U, bool NTL, int STP>
__device__ __forceinline__ void gather_full_tile_by_mode(int mode, char* dst, const char* src, float k) {
  if (mode == MODE_COPY) gather_full_tile<S, D, SCALE, MODE_COPY, BLOCK, U, NTL, STP>(dst, src, k);
  else if (mode == MODE_ADD) gather_full_tile<S, D, SCALE, MODE_ADD, BLOCK, U, NTL, STP>(dst, src, k);
  else if (SCALE != SCALE_NONE) gather_full_tile<S, D, SCALE, MODE_SKIP, BLOCK, U, NTL, STP>(dst, src, k);
}

// S: tensor dtype, D: flat buffer dtype.  pad_zero != 0 writes zeros to
// [total, padded); otherwise pad lanes only see the divide (as in the
// reference, whose pad content is whatever the buffer held).  Full tiles
// from tile wt_from on store write-through when STP is ST_NT.
template <class META, class S, class D, int SCALE, int BLOCK, int U, bool NTL, int STP>
__global__ void __launch_bounds__(BLOCK)
gather_in_kernel(META meta, void* flat, int64_t padded, int n_tiles, float k, int pad_zero, int wt_from) {
  constexpr int64_t kTile = int64_t(BLOCK) * U * 8;
  constexpr bool NTS = (STP == ST_NT);  // ragged segments keep ordinary global stores
  char* fbase = reinterpret_cast<char*>(flat);
  // Workgroup b handles tile b (the host launches at most n_tiles workgroups and at least one when n_tiles > 0).
  // A loop that tests at its end: the first tile's lookup then does not wait for n_tiles to arrive before its own
  // loads leave.
  int tile = blockIdx.x;
  do {
    const int64_t t0 = int64_t(tile) * kTile;
    const int64_t t1 = (t0 + kTile < padded) ? t0 + kTile : padded;
    const TileLookup rec = meta.lookup(tile, t0, kTile);
    int p = rec.first;
    if (rec.full) {  // the whole tile lies inside tensor p
      const int mode = rec.mode;
      const char* src = reinterpret_cast<const char*>(rec.base) + rec.delta * S::kSize;
      char* dst = fbase + t0 * D::kSize;
      if (STP == ST_NT && tile >= wt_from)  // the end of the buffer writes through (see tuning.h)
        gather_full_tile_by_mode<S, D, SCALE, BLOCK, U, NTL, ST_WT>(mode, dst, src, k);
      else
        gather_full_tile_by_mode<S, D, SCALE, BLOCK, U, NTL, STP>(mode, dst, src, k);
      continue;
    }
    int64_t pos = t0;
    while (pos < t1) {
      if (p >= meta.n_tensors) {  // pad lanes
        char* dst = fbase + pos * D::kSize;
        if (pad_zero) gather_segment<S, D, SCALE, MODE_ZERO, BLOCK, NTL, NTS>(dst, nullptr, t1 - pos, pos, k);
        else if (SCALE != SCALE_NONE) gather_segment<S, D, SCALE, MODE_SKIP, BLOCK, NTL, NTS>(dst, nullptr, t1 - pos, pos, k);
        break;
      }
      const int64_t o1 = meta.offset(p + 1);
      if (o1 <= pos) { ++p; continue; }  // empty tensor
      const int64_t o0 = meta.offset(p);
      const int64_t e = o1 < t1 ? o1 : t1;
      const int mode = meta.mode(p);
      const char* src = reinterpret_cast<const char*>(meta.tensor(p)) + (pos - o0) * S::kSize;
      char* dst = fbase + pos * D::kSize;
      if (mode == MODE_COPY) gather_segment<S, D, SCALE, MODE_COPY, BLOCK, NTL, NTS>(dst, src, e - pos, pos, k);
      else if (mode == MODE_ADD) gather_segment<S, D, SCALE, MODE_ADD, BLOCK, NTL, NTS>(dst, src, e - pos, pos, k);
      else if (SCALE != SCALE_NONE) gather_segment<S, D, SCALE, MODE_SKIP, BLOCK, NTL, NTS>(dst, src, e - pos, pos, k);
      pos = e;
      if (e == o1) ++p;
    }
  } while ((tile += gridDim.x) < n_tiles);
}

// ---------------------------------------------------------------- scatter-out --
// One full tile: dst (tensor side) starts on a 128-byte line, src (flat side)
// sits at whatever element-aligned address results.  (Tiling the flat side
// instead and storing at odd tensor offsets measured 13 % slower on a
// 1427-tensor table: two workgroups then share the cache line at every tile
// boundary.  Loads at odd offsets cost about 1 %.)
template <class S, class D, int BLOCK, int U, bool NTL, int STP>
__device__ __forceinline__ void scatter_full_tile(char* dst, const char* src) {
  const TileStore<D, STP> out(dst, BLOCK * U * 8 * D::kSize);
  if constexpr (wide_pair<S, D>::value) {
    Quad<S> s[2 * U];
    Quad<D> unused_q;
#pragma unroll
    for (int q = 0; q < 2 * U; q++) s[q] = load_quad<S, NTL>(src + quad_elem<BLOCK, U>(q) * S::kSize);
#pragma unroll
    for (int q = 0; q < 2 * U; q++)
      store_quad_at<D, STP>(out, quad_elem<BLOCK, U>(q) * D::kSize, flat_quad<S, D, SCALE_NONE, false>(s[q], unused_q, 0.f));
    return;
  }
  Unit<S> s[U];
  Unit<D> unused;
#pragma unroll
  for (int j = 0; j < U; j++) s[j] = load_unit<S, NTL>(src + unit_index<BLOCK, U>(j) * (8 * S::kSize));
#pragma unroll
  for (int j = 0; j < U; j++)
    store_unit_at<D, STP>(out, unit_index<BLOCK, U>(j) * (8 * D::kSize), flat_unit<S, D, SCALE_NONE, false>(s[j], unused, 0.f));
}

// n elements (fewer than a tile): up to 7 leading elements bring dst to a
// 16-byte boundary, then whole units, then the tail.
template <class S, class D, int BLOCK, bool NTL, bool NTS>
__device__ __forceinline__ void scatter_segment(char* dst, const char* src, int64_t n) {
  const int tid = threadIdx.x;
  int64_t head = ((16 - (reinterpret_cast<uintptr_t>(dst) & 15)) & 15) / D::kSize;
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

// S: flat buffer dtype, D: tensor dtype.  Tensors with mode 0 are not written;
// pad lanes of the flat buffer are never read.  n_tiles counts tile slots; full tiles of the slots from wt_from on
// store write-through when STP is ST_NT.  `block` of `n_blocks`: the workgroup's place in the grid of
// scatter_out_kernel, or in the part of a larger grid that serves this job.
template <class META, class S, class D, int BLOCK, int U, bool NTL, int STP>
__device__ __forceinline__ void scatter_body(const META& meta, const void* flat, int n_tiles, int wt_from, int block,
                                             int n_blocks) {
  constexpr int64_t kTile = int64_t(BLOCK) * U * 8;
  constexpr bool NTS = (STP == ST_NT);  // ragged segments keep ordinary global stores
  constexpr int64_t kLineElems = 128 / D::kSize;
  const char* fbase = reinterpret_cast<const char*>(flat);
  for (int tile = block; tile < n_tiles; tile += n_blocks) {
    const ScatterLookup rec = meta.lookup_scatter(tile);
    const int p = rec.tensor;
    if (p >= meta.n_tensors) continue;
    if (meta.mode(p) == MODE_SKIP) continue;
    const int64_t o0 = meta.offset(p);
    const int64_t n = meta.offset(p + 1) - o0;
    char* tbase = reinterpret_cast<char*>(const_cast<void*>(meta.tensor(p)));
    // elements between the start of the tensor's first cache line and the tensor
    const int64_t lead = int64_t((reinterpret_cast<uintptr_t>(tbase) / D::kSize) & uintptr_t(kLineElems - 1));
    const int64_t start = int64_t(rec.index) * kTile - lead;
    const int64_t lo = start > 0 ? start : 0;
    const int64_t hi = start + kTile < n ? start + kTile : n;
    if (lo >= hi) continue;
    char* dst = tbase + lo * D::kSize;
    const char* src = fbase + (o0 + lo) * S::kSize;
    if (hi - lo == kTile) {
      if (STP == ST_NT && tile >= wt_from) scatter_full_tile<S, D, BLOCK, U, NTL, ST_WT>(dst, src);
      else scatter_full_tile<S, D, BLOCK, U, NTL, STP>(dst, src);
    } else {
      scatter_segment<S, D, BLOCK, NTL, NTS>(dst, src, hi - lo);
    }
  }
}

template <class META, class S, class D, int BLOCK, int U, bool NTL, int STP>
__global__ void __launch_bounds__(BLOCK)
scatter_out_kernel(META meta, const void* flat, int64_t total, int n_tiles, int wt_from) {
  (void)total;
  scatter_body<META, S, D, BLOCK, U, NTL, STP>(meta, flat, n_tiles, wt_from, int(blockIdx.x), int(gridDim.x));
}

}  // namespace yafsdp

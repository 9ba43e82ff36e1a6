// Element types, 8-element vector units and the per-element arithmetic of the
// buffer path, for gfx950 (wave64).
//
// A "unit" is 8 consecutive elements: 16 bytes of a 2-byte dtype (one
// global_load/store_dwordx4 per lane) or 32 bytes of fp32 (two).  All
// arithmetic is done in binary32, every materialisation point of the reference
// rounds once (RNE) to the dtype of the tensor it materialises, and no
// multiply-add is ever contracted (the translation units are built with
// -ffp-contract=off as well).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace yafsdp {

enum : int { DT_F32 = 0, DT_BF16 = 1, DT_F16 = 2 };
// how a divide factor is applied: not at all, as an exact multiply by the
// reciprocal (power-of-two factors only: same bits as a division), or as a
// correctly rounded binary32 division.
// SCALE_PREMUL exists for the fan-in only: every contribution is multiplied by k and rounded BEFORE the sum
enum : int { SCALE_NONE = 0, SCALE_MUL = 1, SCALE_DIV = 2, SCALE_PREMUL = 3 };

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
// 16-byte vectors that may sit at any element-aligned address; gfx950 under
// the HSA runtime executes dwordx4 accesses at such addresses natively
typedef u32x4 u32x4_a4 __attribute__((aligned(4)));
typedef u32x4 u32x4_a2 __attribute__((aligned(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef u32x2 u32x2_a2 __attribute__((aligned(2)));

struct F32 {
  typedef float storage;
  typedef u32x4_a4 vec_unaligned;
  typedef u32x4 quad;               // 4 elements
  typedef u32x4_a4 quad_unaligned;
  static constexpr int kId = DT_F32;
  static constexpr int kSize = 4;
  static constexpr int kVecs = 2;  // dwordx4 accesses per unit
};
struct BF16 {
  typedef uint16_t storage;
  typedef u32x4_a2 vec_unaligned;
  typedef u32x2 quad;
  typedef u32x2_a2 quad_unaligned;
  static constexpr int kId = DT_BF16;
  static constexpr int kSize = 2;
  static constexpr int kVecs = 1;
};
struct F16 {
  typedef uint16_t storage;
  typedef u32x4_a2 vec_unaligned;
  typedef u32x2 quad;
  typedef u32x2_a2 quad_unaligned;
  static constexpr int kId = DT_F16;
  static constexpr int kSize = 2;
  static constexpr int kVecs = 1;
};

template <class A, class B>
struct same_t { static constexpr bool value = false; };
template <class A>
struct same_t<A, A> { static constexpr bool value = true; };

template <class T>
struct Unit { u32x4 v[T::kVecs]; };

// ---- memory -----------------------------------------------------------------
// `p` only needs element alignment.  NT selects the non-temporal (streaming)
// cache policy.
template <class T, bool NT>
__device__ __forceinline__ Unit<T> load_unit(const void* p) {
  Unit<T> r;
  const typename T::vec_unaligned* q = reinterpret_cast<const typename T::vec_unaligned*>(p);
#pragma unroll
  for (int i = 0; i < T::kVecs; i++) {
    if constexpr (NT) r.v[i] = __builtin_nontemporal_load(q + i);
    else r.v[i] = q[i];
  }
  return r;
}

template <class T, bool NT>
__device__ __forceinline__ void store_unit(void* p, const Unit<T>& u) {
  typename T::vec_unaligned* q = reinterpret_cast<typename T::vec_unaligned*>(p);
#pragma unroll
  for (int i = 0; i < T::kVecs; i++) {
    if constexpr (NT) __builtin_nontemporal_store(u.v[i], q + i);
    else q[i] = u.v[i];
  }
}

// ---- stores of one tile with a cache policy --------------------------------------
// ST_PLAIN and ST_NT are ordinary global stores (non-temporal for ST_NT: the line
// is kept in the L2 with streaming priority and written back when it is evicted
// or when the kernel ends).  ST_WT writes through: buffer stores carrying sc0 sc1
// hand every line to the memory side at once, in the order the tile loop produces
// them, so the L2 does not fill up with dirty lines whose write-back the kernel's
// end (and the loads of the kernel after it) would have to wait for.  Measured on
// the 27 M-element shard kernels of a Llama-3-8B layer: bf16 -> fp32 copy 29.3 ->
// 24.3 us, accumulate 43.3 -> 40.0 us, fp32 -> bf16 cast 26.5 -> 25.1 us; on
// 400 MB tables the two policies are level.
// Buffer stores address `base + byte offset` with a wave-uniform base (the tile's
// first byte; readfirstlane is free when the compiler already knows that) and a
// per-lane 32-bit offset; stores beyond `bytes` would be dropped by the hardware.
enum : int { ST_PLAIN = 0, ST_NT = 1, ST_WT = 2 };

template <class T, int POLICY>
struct TileStore {
  char* base;
  __amdgpu_buffer_rsrc_t rsrc;
  static constexpr int kAux = 1 | 16;  // sc0 | sc1

  __device__ __forceinline__ TileStore(char* tile_base, int bytes) : base(tile_base) {
    if constexpr (POLICY == ST_WT) {
      const uint64_t a = reinterpret_cast<uint64_t>(tile_base);
      const uint32_t lo = __builtin_amdgcn_readfirstlane(uint32_t(a));
      const uint32_t hi = __builtin_amdgcn_readfirstlane(uint32_t(a >> 32));
      rsrc = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>((uint64_t(hi) << 32) | lo), 0, bytes, 0x00020000);
    }
  }
  // 16 bytes (4 fp32 or 8 two-byte elements) at byte offset `off`, 16-byte aligned
  __device__ __forceinline__ void vec(int off, u32x4 v) const {
    if constexpr (POLICY == ST_WT) __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, off, 0, kAux);
    else if constexpr (POLICY == ST_NT) __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(base + off));
    else *reinterpret_cast<u32x4*>(base + off) = v;
  }
  // 8 bytes (4 two-byte elements) at byte offset `off`, 8-byte aligned
  __device__ __forceinline__ void half(int off, u32x2 v) const {
    if constexpr (POLICY == ST_WT) __builtin_amdgcn_raw_buffer_store_b64(v, rsrc, off, 0, kAux);
    else if constexpr (POLICY == ST_NT) __builtin_nontemporal_store(v, reinterpret_cast<u32x2*>(base + off));
    else *reinterpret_cast<u32x2*>(base + off) = v;
  }
};

// ---- scalar conversions -------------------------------------------------------
__device__ __forceinline__ float bits_to_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f32_to_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

template <class T> __device__ __forceinline__ float to_f32(typename T::storage s);
template <> __device__ __forceinline__ float to_f32<F32>(float s) { return s; }
template <> __device__ __forceinline__ float to_f32<BF16>(uint16_t s) { return bits_to_f32(uint32_t(s) << 16); }
template <> __device__ __forceinline__ float to_f32<F16>(uint16_t s) {
  return (float)__builtin_bit_cast(_Float16, s);
}

// round to nearest even (hardware v_cvt_pk_bf16_f32 / v_cvt_f16_f32)
template <class T> __device__ __forceinline__ typename T::storage from_f32(float f);
template <> __device__ __forceinline__ float from_f32<F32>(float f) { return f; }
template <> __device__ __forceinline__ uint16_t from_f32<BF16>(float f) {
  return __builtin_bit_cast(uint16_t, (__bf16)f);
}
template <> __device__ __forceinline__ uint16_t from_f32<F16>(float f) {
  return __builtin_bit_cast(uint16_t, (_Float16)f);
}

// the value a binary32 number has after being stored as T and read back
template <class T>
__device__ __forceinline__ float round_to(float f) {
  if constexpr (same_t<T, F32>::value) return f;
  else return to_f32<T>(from_f32<T>(f));
}

// ---- unit <-> 8 floats --------------------------------------------------------
template <class T>
__device__ __forceinline__ void unpack(const Unit<T>& u, float (&f)[8]) {
  if constexpr (same_t<T, F32>::value) {
#pragma unroll
    for (int i = 0; i < 4; i++) { f[i] = bits_to_f32(u.v[0][i]); f[4 + i] = bits_to_f32(u.v[1][i]); }
  } else if constexpr (same_t<T, BF16>::value) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      uint32_t w = u.v[0][i];
      f[2 * i] = bits_to_f32(w << 16);
      f[2 * i + 1] = bits_to_f32(w & 0xFFFF0000u);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const uint32_t w = u.v[0][i];
      f[2 * i] = (float)__builtin_bit_cast(_Float16, uint16_t(w & 0xFFFFu));
      f[2 * i + 1] = (float)__builtin_bit_cast(_Float16, uint16_t(w >> 16));
    }
  }
}

template <class T>
__device__ __forceinline__ Unit<T> pack(const float (&f)[8]) {
  Unit<T> u;
  if constexpr (same_t<T, F32>::value) {
#pragma unroll
    for (int i = 0; i < 4; i++) { u.v[0][i] = f32_to_bits(f[i]); u.v[1][i] = f32_to_bits(f[4 + i]); }
  } else if constexpr (same_t<T, BF16>::value) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      f32x2 x = {f[2 * i], f[2 * i + 1]};
      u.v[0][i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2));
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      f32x2 x = {f[2 * i], f[2 * i + 1]};
      u.v[0][i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(x, f16x2));
    }
  }
  return u;
}

// ---- quads: 4 consecutive elements --------------------------------------------
// Used when one side of a pair is fp32: lane l of a wave then owns elements
// 4l..4l+3 and 256+4l..256+4l+3 of a 512-element wave tile, so that every
// access instruction of the wave covers one contiguous span (64 x 16 bytes of
// fp32, 64 x 8 bytes of a 2-byte dtype) made of whole cache lines.  With 8
// consecutive fp32 elements per lane instead, each dwordx4 instruction would
// touch only every other 16 bytes of the span.
template <class T>
struct Quad { typename T::quad v; };

template <class T, bool NT>
__device__ __forceinline__ Quad<T> load_quad(const void* p) {
  Quad<T> r;
  const typename T::quad_unaligned* q = reinterpret_cast<const typename T::quad_unaligned*>(p);
  if constexpr (NT) r.v = __builtin_nontemporal_load(q);
  else r.v = *q;
  return r;
}

template <class T, bool NT>
__device__ __forceinline__ void store_quad(void* p, const Quad<T>& u) {
  typename T::quad_unaligned* q = reinterpret_cast<typename T::quad_unaligned*>(p);
  if constexpr (NT) __builtin_nontemporal_store(u.v, q);
  else *q = u.v;
}

template <class T>
__device__ __forceinline__ void unpack_quad(const Quad<T>& u, float (&f)[4]) {
  if constexpr (same_t<T, F32>::value) {
#pragma unroll
    for (int i = 0; i < 4; i++) f[i] = bits_to_f32(u.v[i]);
  } else if constexpr (same_t<T, BF16>::value) {
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const uint32_t w = u.v[i];
      f[2 * i] = bits_to_f32(w << 16);
      f[2 * i + 1] = bits_to_f32(w & 0xFFFF0000u);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const uint32_t w = u.v[i];
      f[2 * i] = (float)__builtin_bit_cast(_Float16, uint16_t(w & 0xFFFFu));
      f[2 * i + 1] = (float)__builtin_bit_cast(_Float16, uint16_t(w >> 16));
    }
  }
}

template <class T>
__device__ __forceinline__ Quad<T> pack_quad(const float (&f)[4]) {
  Quad<T> u;
  if constexpr (same_t<T, F32>::value) {
#pragma unroll
    for (int i = 0; i < 4; i++) u.v[i] = f32_to_bits(f[i]);
  } else if constexpr (same_t<T, BF16>::value) {
#pragma unroll
    for (int i = 0; i < 2; i++) {
      f32x2 x = {f[2 * i], f[2 * i + 1]};
      u.v[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2));
    }
  } else {
#pragma unroll
    for (int i = 0; i < 2; i++) {
      f32x2 x = {f[2 * i], f[2 * i + 1]};
      u.v[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(x, f16x2));
    }
  }
  return u;
}

// one unit / one quad of a tile through its TileStore (byte offset inside the tile)
template <class T, int POLICY>
__device__ __forceinline__ void store_unit_at(const TileStore<T, POLICY>& ts, int off, const Unit<T>& u) {
#pragma unroll
  for (int i = 0; i < T::kVecs; i++) ts.vec(off + 16 * i, u.v[i]);
}

template <class T, int POLICY>
__device__ __forceinline__ void store_quad_at(const TileStore<T, POLICY>& ts, int off, const Quad<T>& u) {
  if constexpr (T::kSize == 4) ts.vec(off, u.v);
  else ts.half(off, u.v);
}

// a pair of dtypes takes the quad arrangement when either side is fp32
template <class S, class D>
struct wide_pair { static constexpr bool value = (S::kSize == 4 || D::kSize == 4); };

// unit index of the j-th unit (0 .. U-1) of this lane inside a tile of BLOCK*U
// units: lane-strided by BLOCK, so consecutive waves own consecutive 1 KiB
// spans.  (Giving each wave U consecutive spans instead measured 0-2 % slower.)
template <int BLOCK, int U>
__device__ __forceinline__ int unit_index(int j) {
  return int(threadIdx.x) + j * BLOCK;
}

// byte-free element index of quad q (0 .. 2U-1) of this lane inside a tile of
// BLOCK*U units: wave tiles of 512 elements, two quads per lane per wave tile
template <int BLOCK, int U = 1>
__device__ __forceinline__ int quad_elem(int q) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  return ((q >> 1) * (BLOCK / 64) + wave) * 512 + (q & 1) * 256 + lane * 4;
}

// ---- the arithmetic -----------------------------------------------------------
// Keeps a value opaque to the instruction selector (emits nothing).  Without it
// a multiply next to an fp16 conversion is selected as v_fma_mix*(a, b, +0),
// whose +0 addend turns a -0 product into +0.
__device__ __forceinline__ float opaque(float y) {
  asm("" : "+v"(y));
  return y;
}

template <int SCALE>
__device__ __forceinline__ float apply_scale(float y, float k) {
  if constexpr (SCALE == SCALE_MUL) return opaque(__fmul_rn(opaque(y), k));  // k = 1/factor, exact
  else if constexpr (SCALE == SCALE_DIV) return __fdiv_rn(y, k);             // k = factor
  else return y;
}

// Reduce copy-in element (tensor dtype S -> flat reduce buffer dtype D):
//   view.copy_(grad) or view.add_(grad)   -> rounds to D
//   buffer.div_(pre)                      -> rounds to D again
// MODE: 1 copy, 2 add, 0 tensor absent (only the divide touches the element).
enum : int { MODE_SKIP = 0, MODE_COPY = 1, MODE_ADD = 2 };

template <class S, class D, int SCALE, int MODE>
__device__ __forceinline__ float gather_elem(float s, float d_old, float k) {
  float y;
  if constexpr (MODE == MODE_COPY) y = s;
  else if constexpr (MODE == MODE_ADD) y = __fadd_rn(d_old, s);
  else y = d_old;
  if constexpr (SCALE != SCALE_NONE) {
    // the copy / add materialises in D before the divide reads it.  A copied value that D represents exactly
    // (same dtype, or binary32 as the destination) needs no rounding instruction.
    constexpr bool kExactCopy = MODE == MODE_COPY && (same_t<S, D>::value || same_t<D, F32>::value);
    if constexpr (MODE != MODE_SKIP && !kExactCopy) y = round_to<D>(y);
    y = apply_scale<SCALE>(y, k);
  }
  return y;  // caller rounds to D on store
}

// Post-reduce element (chunk dtype S -> grad shard dtype D):
//   chunk.div_(post)                      -> rounds to S
//   shard.copy_(chunk) or shard.add_(chunk) -> rounds to D
template <class S, class D, int SCALE, bool ACC>
__device__ __forceinline__ float post_elem(float s, float d_old, float k) {
  float y = s;
  if constexpr (SCALE != SCALE_NONE) {
    y = apply_scale<SCALE>(y, k);
    if constexpr (ACC || !same_t<S, D>::value) y = round_to<S>(y);
  }
  if constexpr (ACC) y = __fadd_rn(d_old, y);
  return y;  // caller rounds to D on store
}

// Sum of one binary64 value per lane over a workgroup of BLOCK lanes, in a fixed
// order (wave shuffles, then the waves' sums through `lds[BLOCK / 64]`).  Valid
// in thread 0.
template <int BLOCK>
__device__ __forceinline__ double block_sum(double v, double* lds) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) lds[wave] = v;
  __syncthreads();
  double t = 0.0;
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 0; w < BLOCK / 64; w++) t += lds[w];
  }
  return t;
}

}  // namespace yafsdp

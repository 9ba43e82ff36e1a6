// Optimizer-side passes over the flat shard buffers of a parameter group: fill
// (zero_grad), sum of squares (gradient norm), scale by a device-resident
// coefficient (gradient clipping) and the fused AdamW step that also emits the
// 16-bit all-gather input of the next iteration.
//
// All four are single passes over contiguous ranges (up to 3 or 7 leading
// elements are peeled to reach a 16-byte boundary).  A lane
// owns quads (4 consecutive elements); quad j of lane t inside a tile of
// BLOCK*U quads is t + j*BLOCK, so every wave64 access is one contiguous span
// (1 KiB of fp32, 512 B of a 2-byte dtype).  All loads of a lane are issued
// before its first store.
#pragma once
#include "elem.hip.h"
#include "launch.h"

namespace yafsdp {

// ------------------------------------------------------------------- fill ----
// dst[i] = pattern for i in [0, n); `pattern` holds the element replicated to 32
// bits.  `head` leading elements bring dst to a 16-byte boundary; workgroup 0
// writes them and the tail one by one.
template <class D>
__device__ __forceinline__ void fill_scalar(void* dst, int64_t i, uint32_t pattern) {
  if constexpr (D::kSize == 4) reinterpret_cast<uint32_t*>(dst)[i] = pattern;
  else reinterpret_cast<uint16_t*>(dst)[i] = uint16_t(pattern & 0xFFFFu);
}

template <class D, int BLOCK, int U, bool NTS>
__global__ void __launch_bounds__(BLOCK)
fill_kernel(void* dst0, int64_t n0, int head, uint32_t pattern) {
  constexpr int kPer = 16 / D::kSize;  // elements per 16-byte store
  if (blockIdx.x == 0 && int(threadIdx.x) < head) fill_scalar<D>(dst0, threadIdx.x, pattern);
  void* dst = reinterpret_cast<char*>(dst0) + int64_t(head) * D::kSize;
  const int64_t n = n0 - head;
  const int64_t n_vec = n / kPer;
  constexpr int64_t kTile = int64_t(BLOCK) * U;
  const int64_t n_tiles = (n_vec + kTile - 1) / kTile;
  const u32x4 v = {pattern, pattern, pattern, pattern};
  u32x4* out = reinterpret_cast<u32x4*>(dst);
  for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const int64_t base = tile * kTile + threadIdx.x;
    if (tile * kTile + kTile <= n_vec) {
#pragma unroll
      for (int j = 0; j < U; j++) {
        if constexpr (NTS) __builtin_nontemporal_store(v, out + base + j * BLOCK);
        else out[base + j * BLOCK] = v;
      }
    } else {
      for (int64_t i = base; i < n_vec; i += BLOCK) out[i] = v;
    }
  }
  if (blockIdx.x == 0) {
    const int64_t i = n_vec * kPer + threadIdx.x;
    if (i < n) fill_scalar<D>(dst, i, pattern);
  }
}

// ------------------------------------------------------------------ scale ----
// buf[i] = round(buf[i] * *coef) in place (grad.mul_(clip_coef)); nothing is
// touched when the coefficient is exactly 1 (x * 1 == x for every x).
template <class D, int BLOCK, int U, bool NTL, bool NTS>
__global__ void __launch_bounds__(BLOCK)
scale_kernel(void* buf0, int64_t n0, int head, const float* coef) {
  typedef typename D::storage d_t;
  const float c = *reinterpret_cast<const __attribute__((address_space(4))) float*>(
      reinterpret_cast<uintptr_t>(coef));
  if (c == 1.0f) return;
  if (blockIdx.x == 0 && int(threadIdx.x) < head) {
    d_t* p = reinterpret_cast<d_t*>(buf0);
    p[threadIdx.x] = from_f32<D>(opaque(__fmul_rn(opaque(to_f32<D>(p[threadIdx.x])), c)));
  }
  void* buf = reinterpret_cast<char*>(buf0) + int64_t(head) * D::kSize;
  const int64_t n = n0 - head;
  const int64_t n_quads = n >> 2;
  constexpr int64_t kTile = int64_t(BLOCK) * U;
  const int64_t n_tiles = (n_quads + kTile - 1) / kTile;
  char* base = reinterpret_cast<char*>(buf);
  constexpr int kQuadBytes = 4 * D::kSize;
  for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const int64_t q0 = tile * kTile + threadIdx.x;
    if (tile * kTile + kTile <= n_quads) {
      Quad<D> x[U];
#pragma unroll
      for (int j = 0; j < U; j++) x[j] = load_quad<D, NTL>(base + (q0 + j * BLOCK) * kQuadBytes);
#pragma unroll
      for (int j = 0; j < U; j++) {
        float f[4];
        unpack_quad<D>(x[j], f);
#pragma unroll
        for (int e = 0; e < 4; e++) f[e] = opaque(__fmul_rn(opaque(f[e]), c));
        store_quad<D, NTS>(base + (q0 + j * BLOCK) * kQuadBytes, pack_quad<D>(f));
      }
    } else {
      for (int64_t q = q0; q < n_quads; q += BLOCK) {
        Quad<D> x = load_quad<D, NTL>(base + q * kQuadBytes);
        float f[4];
        unpack_quad<D>(x, f);
#pragma unroll
        for (int e = 0; e < 4; e++) f[e] = opaque(__fmul_rn(opaque(f[e]), c));
        store_quad<D, NTS>(base + q * kQuadBytes, pack_quad<D>(f));
      }
    }
  }
  if (blockIdx.x == 0) {
    const int64_t i = (n_quads << 2) + threadIdx.x;
    if (i < n) {
      d_t* p = reinterpret_cast<d_t*>(buf);
      p[i] = from_f32<D>(opaque(__fmul_rn(opaque(to_f32<D>(p[i])), c)));
    }
  }
}

// ---------------------------------------------------------- sum of squares ----
// partials[blockIdx.x] = sum over this workgroup's tiles of x^2, accumulated in
// binary64 (the square of a binary32 number is exact there).  The order of the
// additions depends only on (n, gridDim, BLOCK, U): results are reproducible
// from run to run.  (Folding the final sum into this kernel with a last-
// workgroup ticket was measured: the agent-scope release/acquire that it needs
// per workgroup makes the pass ten times slower.)
template <class S, int BLOCK, int U, bool NTL>
__global__ void __launch_bounds__(BLOCK)
sumsq_kernel(const void* src0, int64_t n0, int head, double* partials) {
  typedef typename S::storage s_t;
  __shared__ double lds[BLOCK / 64];
  const void* src = reinterpret_cast<const char*>(src0) + int64_t(head) * S::kSize;
  const int64_t n = n0 - head;
  const int64_t n_quads = n >> 2;
  constexpr int64_t kTile = int64_t(BLOCK) * U;
  const int64_t n_tiles = (n_quads + kTile - 1) / kTile;
  const char* base = reinterpret_cast<const char*>(src);
  constexpr int kQuadBytes = 4 * S::kSize;
  double acc[4] = {0.0, 0.0, 0.0, 0.0};
  for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const int64_t q0 = tile * kTile + threadIdx.x;
    if (tile * kTile + kTile <= n_quads) {
      Quad<S> x[U];
#pragma unroll
      for (int j = 0; j < U; j++) x[j] = load_quad<S, NTL>(base + (q0 + j * BLOCK) * kQuadBytes);
#pragma unroll
      for (int j = 0; j < U; j++) {
        float f[4];
        unpack_quad<S>(x[j], f);
#pragma unroll
        for (int e = 0; e < 4; e++) acc[e] = __fma_rn(double(f[e]), double(f[e]), acc[e]);
      }
    } else {
      for (int64_t q = q0; q < n_quads; q += BLOCK) {
        Quad<S> x = load_quad<S, NTL>(base + q * kQuadBytes);
        float f[4];
        unpack_quad<S>(x, f);
#pragma unroll
        for (int e = 0; e < 4; e++) acc[e] = __fma_rn(double(f[e]), double(f[e]), acc[e]);
      }
    }
  }
  if (blockIdx.x == 0) {
    const int64_t i = (n_quads << 2) + threadIdx.x;
    if (i < n) {
      const double x = double(to_f32<S>(reinterpret_cast<const s_t*>(src)[i]));
      acc[0] = __fma_rn(x, x, acc[0]);
    }
    if (int(threadIdx.x) < head) {
      const double x = double(to_f32<S>(reinterpret_cast<const s_t*>(src0)[threadIdx.x]));
      acc[1] = __fma_rn(x, x, acc[1]);
    }
  }
  const double t = block_sum<BLOCK>((acc[0] + acc[1]) + (acc[2] + acc[3]), lds);
  if (threadIdx.x == 0) partials[blockIdx.x] = t;
}

// First stage for long arrays of partial sums: workgroup b adds in[b * kChunk : (b + 1) * kChunk] (bounded by count)
// in a fixed order and writes out[b].
constexpr int kSumsqReduceChunk = 4096;
template <int BLOCK>
__global__ void __launch_bounds__(BLOCK)
sumsq_reduce_kernel(const double* in, int64_t count, double* out) {
  __shared__ double lds[BLOCK / 64];
  const int64_t base = int64_t(blockIdx.x) * kSumsqReduceChunk;
  double acc[kSumsqReduceChunk / BLOCK];
#pragma unroll
  for (int j = 0; j < kSumsqReduceChunk / BLOCK; j++) {
    const int64_t i = base + threadIdx.x + int64_t(j) * BLOCK;
    acc[j] = i < count ? in[i] : 0.0;
  }
  double v = acc[0];
#pragma unroll
  for (int j = 1; j < kSumsqReduceChunk / BLOCK; j++) v += acc[j];
  const double t = block_sum<BLOCK>(v, lds);
  if (threadIdx.x == 0) out[blockIdx.x] = t;
}

// One workgroup adds `count` partial sums in a fixed order:
//   sumsq[0] = (accumulate ? sumsq[0] : 0) + sum          (when sumsq is given)
//   norm_and_coef = {float(sqrt(total)), min(max_norm / (norm + 1e-6), 1)}   (when given; NaN kept, as
//   torch.clamp(max=1.0) keeps it)
template <int BLOCK>
__global__ void __launch_bounds__(BLOCK)
sumsq_finish_kernel(const double* partials, int64_t count, double* sumsq, int accumulate, float max_norm,
                    float* norm_and_coef) {
  __shared__ double lds[BLOCK / 64];
  double acc[4] = {0.0, 0.0, 0.0, 0.0};
  int64_t i = threadIdx.x;
  for (; i + 3 * BLOCK < count; i += 4 * BLOCK) {  // four independent loads in flight per lane
    const double a = partials[i], b = partials[i + BLOCK], c = partials[i + 2 * BLOCK], d = partials[i + 3 * BLOCK];
    acc[0] += a; acc[1] += b; acc[2] += c; acc[3] += d;
  }
  for (; i < count; i += BLOCK) acc[0] += partials[i];
  double total = block_sum<BLOCK>((acc[0] + acc[1]) + (acc[2] + acc[3]), lds);
  if (threadIdx.x != 0) return;
  if (sumsq != nullptr) {
    if (accumulate) total += sumsq[0];
    sumsq[0] = total;
  }
  if (norm_and_coef != nullptr) {
    const float norm = float(__builtin_sqrt(total));
    float c = __fdiv_rn(max_norm, __fadd_rn(norm, 1e-6f));
    if (c > 1.0f) c = 1.0f;
    norm_and_coef[0] = norm;
    norm_and_coef[1] = c;
  }
}

// norm_and_coef[0] = sqrt(sumsq) as binary32; norm_and_coef[1] = min(max_norm /
// (norm + 1e-6), 1) in binary32, NaN kept (torch.clamp(max=1.0) keeps it too)
__global__ void clip_coef_kernel(const double* sumsq, float max_norm, float* norm_and_coef) {
  if (threadIdx.x != 0 || blockIdx.x != 0) return;
  const float norm = float(__builtin_sqrt(sumsq[0]));
  float c = __fdiv_rn(max_norm, __fadd_rn(norm, 1e-6f));
  if (c > 1.0f) c = 1.0f;
  norm_and_coef[0] = norm;
  norm_and_coef[1] = c;
}

// ------------------------------------------------------------------ AdamW ----
// Per element, the operation order of torch.optim.AdamW / Adam (single-tensor
// and foreach forms alike) with every intermediate tensor rounded to binary32:
//   g   = grad * grad_scale                        (when a scale pointer is given)
//   g   = fma(p, wd, g)                            (Adam, L2 form: grad.add(param, alpha=wd))
//   p   = p * (1 - lr*wd)                          (AdamW: param.mul_)
//   m   = fma(w, g - m, m)          w = 1 - beta1 < 0.5      (exp_avg.lerp_(grad, w))
//       = fma(w - 1, g - m, g)      otherwise
//   v   = fma((1 - beta2) * g, g, v * beta2)       (mul_ then addcmul_)
//   den = sqrt(v) / sqrt(1 - beta2^t) + eps
//   p   = p + (-(lr / (1 - beta1^t)) * m) / den    (addcdiv_)
//   out16 = round16(p)                             (next iteration's all-gather input)
// The multiply-adds are fused exactly where torch's CPU kernels fuse them;
// division and square root are correctly rounded (the compiler's default for
// binary32 `/` and sqrtf in HIP code; the *_rn sqrt intrinsic is the 1-ulp one).

__device__ __forceinline__ void adam_elem(float& p, float g, float& m, float& v, const AdamScalars& s, bool scaled,
                                          float gs) {
  if (scaled) g = __fmul_rn(g, gs);
  if (s.flags & ADAM_L2) g = __fmaf_rn(p, s.l2, g);
  if (s.flags & ADAM_DECOUPLED) p = __fmul_rn(p, s.decay);
  const float d = __fsub_rn(g, m);
  m = (s.flags & ADAM_W_SMALL) ? __fmaf_rn(s.w, d, m) : __fmaf_rn(s.w_m1, d, g);
  v = __fmaf_rn(__fmul_rn(s.one_m_beta2, g), g, __fmul_rn(v, s.beta2));
  const float den = __fadd_rn(__fdiv_rn(__builtin_sqrtf(v), s.bc2_sqrt), s.eps);
  p = __fadd_rn(p, __fdiv_rn(__fmul_rn(s.neg_step, m), den));
}

// O is the 16-bit output dtype, or F32 for "no 16-bit output"; ZERO_GRAD also zero-fills the gradient.
template <class O, bool ZERO_GRAD, int BLOCK, int U, bool NTL, int STP>
__global__ void __launch_bounds__(BLOCK)
adamw_kernel(float* p0, float* g0, float* m0, float* v0, void* out0, int64_t n0, int head, AdamScalars s,
             const float* grad_scale) {
  static_assert(BLOCK >= 8, "workgroup 0 peels the tail with lanes 0-3 and the head with lanes 4-7");
  constexpr bool kOut = !same_t<O, F32>::value;
  constexpr bool NTS = (STP == ST_NT);  // the partial last tile keeps ordinary global stores
  const bool scaled = grad_scale != nullptr;
  float gs = 1.0f;
  if (scaled)
    gs = *reinterpret_cast<const __attribute__((address_space(4))) float*>(reinterpret_cast<uintptr_t>(grad_scale));
  // `head` leading elements bring the four binary32 arrays (which share one
  // residue modulo 16 bytes) to a 16-byte boundary
  float *p = p0 + head, *g = g0 + head, *m = m0 + head, *v = v0 + head;
  void* out16 = kOut ? reinterpret_cast<char*>(out0) + int64_t(head) * O::kSize : nullptr;
  const int64_t n = n0 - head;
  const int64_t n_quads = n >> 2;
  constexpr int64_t kTile = int64_t(BLOCK) * U;
  const int64_t n_tiles = (n_quads + kTile - 1) / kTile;
  for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const int64_t q0 = tile * kTile + threadIdx.x;
    if (tile * kTile + kTile <= n_quads) {
      Quad<F32> qp[U], qg[U], qm[U], qv[U];
#pragma unroll
      for (int j = 0; j < U; j++) {
        const int64_t e = (q0 + j * BLOCK) << 2;
        qp[j] = load_quad<F32, NTL>(p + e);
        qg[j] = load_quad<F32, NTL>(g + e);
        qm[j] = load_quad<F32, NTL>(m + e);
        qv[j] = load_quad<F32, NTL>(v + e);
      }
      // the tile's first byte in every array it writes (wave-uniform), lane offsets inside the tile
      const int64_t t0 = tile * kTile * 4;
      constexpr int kTileBytes = int(kTile) * 16;
      const TileStore<F32, STP> sp(reinterpret_cast<char*>(p + t0), kTileBytes);
      const TileStore<F32, STP> sm(reinterpret_cast<char*>(m + t0), kTileBytes);
      const TileStore<F32, STP> sv(reinterpret_cast<char*>(v + t0), kTileBytes);
      const TileStore<F32, STP> sg(reinterpret_cast<char*>(g + t0), kTileBytes);
      const TileStore<O, STP> so(reinterpret_cast<char*>(out16) + t0 * O::kSize, int(kTile) * 4 * O::kSize);
#pragma unroll
      for (int j = 0; j < U; j++) {
        const int off = (int(threadIdx.x) + j * BLOCK) * 16;  // bytes inside the tile, binary32 arrays
        float fp[4], fg[4], fm[4], fv[4];
        unpack_quad<F32>(qp[j], fp);
        unpack_quad<F32>(qg[j], fg);
        unpack_quad<F32>(qm[j], fm);
        unpack_quad<F32>(qv[j], fv);
#pragma unroll
        for (int i = 0; i < 4; i++) adam_elem(fp[i], fg[i], fm[i], fv[i], s, scaled, gs);
        store_quad_at<F32, STP>(sp, off, pack_quad<F32>(fp));
        store_quad_at<F32, STP>(sm, off, pack_quad<F32>(fm));
        store_quad_at<F32, STP>(sv, off, pack_quad<F32>(fv));
        if constexpr (kOut) store_quad_at<O, STP>(so, off / 4 * O::kSize, pack_quad<O>(fp));
        if constexpr (ZERO_GRAD) {
          Quad<F32> z;
          z.v = u32x4{0u, 0u, 0u, 0u};
          store_quad_at<F32, STP>(sg, off, z);
        }
      }
    } else {
      for (int64_t q = q0; q < n_quads; q += BLOCK) {
        const int64_t e = q << 2;
        float fp[4], fg[4], fm[4], fv[4];
        unpack_quad<F32>(load_quad<F32, NTL>(p + e), fp);
        unpack_quad<F32>(load_quad<F32, NTL>(g + e), fg);
        unpack_quad<F32>(load_quad<F32, NTL>(m + e), fm);
        unpack_quad<F32>(load_quad<F32, NTL>(v + e), fv);
#pragma unroll
        for (int i = 0; i < 4; i++) adam_elem(fp[i], fg[i], fm[i], fv[i], s, scaled, gs);
        store_quad<F32, NTS>(p + e, pack_quad<F32>(fp));
        store_quad<F32, NTS>(m + e, pack_quad<F32>(fm));
        store_quad<F32, NTS>(v + e, pack_quad<F32>(fv));
        if constexpr (kOut) store_quad<O, NTS>(reinterpret_cast<char*>(out16) + e * O::kSize, pack_quad<O>(fp));
        if constexpr (ZERO_GRAD) {
          Quad<F32> z;
          z.v = u32x4{0u, 0u, 0u, 0u};
          store_quad<F32, NTS>(g + e, z);
        }
      }
    }
  }
  if (blockIdx.x == 0) {
    // lanes 0-3: tail elements; lanes 4-7: head elements (negative indices from the aligned base)
    int64_t i = n;
    if (threadIdx.x < 4) i = (n_quads << 2) + threadIdx.x;
    else if (int(threadIdx.x) - 4 < head) i = int64_t(threadIdx.x) - 4 - head;
    if (i < n) {
      float fp = p[i], fm = m[i], fv = v[i];
      adam_elem(fp, g[i], fm, fv, s, scaled, gs);
      p[i] = fp;
      m[i] = fm;
      v[i] = fv;
      if constexpr (kOut) reinterpret_cast<typename O::storage*>(out16)[i] = from_f32<O>(fp);
      if constexpr (ZERO_GRAD) g[i] = 0.0f;
    }
  }
}

}  // namespace yafsdp

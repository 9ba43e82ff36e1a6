/* Plain-C restatement of the element arithmetic of YaFSDP's per-rank buffer
 * path.  TEST INFRASTRUCTURE ONLY: nothing in the shipped package links or
 * loads this file; tests use it as a second, torch-free checker.
 *
 * The reference performs every step with a torch op whose result is a
 * materialised tensor, so each step rounds once, to the dtype of that tensor:
 *
 *   copy-in            dst.copy_(src)                 ya_fsdp/_collectives.py:54
 *   reduce copy-in     _foreach_copy_(views, grads)   ya_fsdp/_param_group.py:693-700
 *                      _foreach_add_(views, grads)    ya_fsdp/_param_group.py:701-708
 *   pre / post divide  tensor.div_(factor)            ya_fsdp/_collectives.py:139,165,270-272
 *   reduce copy-out    shard.copy_(chunk)             ya_fsdp/_collectives.py:185
 *                      shard.add_(chunk)              ya_fsdp/_collectives.py:189
 *   copy-out           flat[:T].split(numels)         ya_fsdp/_param_group.py:441-457
 *
 * Written from the IEEE-754 definitions, not from torch's sources: casts are
 * round-to-nearest-even on the integer representation, arithmetic is done in
 * binary32 (the op-math type torch uses for bf16/fp16), division is a true
 * binary32 division by the factor rounded to binary32.
 *
 * Build: see oracle/build.py (gcc -O2 -ffp-contract=off, no fast-math).
 */
#include <stdint.h>
#include <string.h>

enum { DT_F32 = 0, DT_BF16 = 1, DT_F16 = 2 };

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* binary32 -> bfloat16, round to nearest even; NaN -> 0x7FC0 (quiet). */
uint16_t ref_f32_to_bf16(uint32_t x) {
  if ((x & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0;
  uint32_t lsb = (x >> 16) & 1u;
  return (uint16_t)((x + 0x7FFFu + lsb) >> 16);
}

uint32_t ref_bf16_to_f32(uint16_t h) { return ((uint32_t)h) << 16; }

/* binary32 -> binary16, round to nearest even, gradual underflow. */
uint16_t ref_f32_to_f16(uint32_t x) {
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t a = x & 0x7FFFFFFFu;
  if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);  /* NaN */
  if (a >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u); /* >= 65520 -> inf */
  if (a >= 0x38800000u) {                                  /* normal half */
    uint32_t mant = a & 0x7FFFFFu;
    uint32_t e = (a >> 23) - 112u;
    uint32_t h = (e << 10) | (mant >> 13);
    uint32_t rem = mant & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (uint16_t)(sign | h);
  }
  if (a <= 0x33000000u) return (uint16_t)sign;             /* <= 2^-25 -> 0 */
  uint32_t mant = (a & 0x7FFFFFu) | 0x800000u;
  uint32_t shift = 126u - (a >> 23);                       /* 14..24 */
  uint32_t h = mant >> shift;
  uint32_t rem = mant & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1u);
  if (rem > half || (rem == half && (h & 1u))) h++;
  return (uint16_t)(sign | h);
}

uint32_t ref_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1Fu;
  uint32_t m = h & 0x3FFu;
  if (e == 0x1Fu) return sign | 0x7F800000u | (m << 13);
  if (e != 0) return sign | ((e + 112u) << 23) | (m << 13);
  if (m == 0) return sign;
  /* subnormal: normalise */
  uint32_t k = 0;
  while (!(m & 0x400u)) { m <<= 1; k++; }
  m &= 0x3FFu;
  return sign | ((113u - k) << 23) | (m << 13);
}

static inline float load_f(const void* p, int dt, int64_t i) {
  switch (dt) {
    case DT_F32: return ((const float*)p)[i];
    case DT_BF16: return u2f(ref_bf16_to_f32(((const uint16_t*)p)[i]));
    default: return u2f(ref_f16_to_f32(((const uint16_t*)p)[i]));
  }
}

static inline void store_f(void* p, int dt, int64_t i, float v) {
  switch (dt) {
    case DT_F32: ((float*)p)[i] = v; break;
    case DT_BF16: ((uint16_t*)p)[i] = ref_f32_to_bf16(f2u(v)); break;
    default: ((uint16_t*)p)[i] = ref_f32_to_f16(f2u(v)); break;
  }
}

/* value after it has been stored in dtype dt and read back */
static inline float round_to(int dt, float v) {
  switch (dt) {
    case DT_F32: return v;
    case DT_BF16: return u2f(ref_bf16_to_f32(ref_f32_to_bf16(f2u(v))));
    default: return u2f(ref_f16_to_f32(ref_f32_to_f16(f2u(v))));
  }
}

static inline int itemsize(int dt) { return dt == DT_F32 ? 4 : 2; }

/* dst.copy_(src) with a dtype change; same dtype is a byte copy. */
void ref_flat_copy(void* dst, int dd, const void* src, int sd, int64_t n) {
  if (dd == sd) { memmove(dst, src, (size_t)n * itemsize(dd)); return; }
  for (int64_t i = 0; i < n; i++) store_f(dst, dd, i, load_f(src, sd, i));
}

/* buf.div_(factor), applied only when factor > 1 (_div_if_needed). */
void ref_flat_div(void* buf, int dt, int64_t n, double factor) {
  if (!(factor > 1.0)) return;
  float f = (float)factor;
  for (int64_t i = 0; i < n; i++) store_f(buf, dt, i, load_f(buf, dt, i) / f);
}

/* One rank's contribution to a reduce-scatter whose reduction is a pre-multiplied
 * sum (ya_fsdp/_collectives.py:243-249, 152-162: ReduceOp.AVG or
 * _make_nccl_premul_sum(1 / factor) handed to dist.reduce_scatter_tensor).  The
 * collective library (NCCL / RCCL, not part of the reference's tree) defines the
 * op as: the scalar is converted to the data type, every rank's input element is
 * multiplied by it and the product rounded to the data type BEFORE the sum
 * (ncclRedOpCreatePreMulSum); ncclAvg on floating-point data is that op with the
 * scalar 1/nRanks.  Not a division: for a factor that is no power of two
 * x * round(1/f) and x / f differ. */
void ref_flat_premul(void* buf, int dt, int64_t n, double scalar) {
  const float k = round_to(dt, (float)scalar);
  for (int64_t i = 0; i < n; i++) store_f(buf, dt, i, load_f(buf, dt, i) * k);
}

/* chunk.div_(post) [rounds to the chunk dtype]; then shard.copy_(chunk) or
 * shard.add_(chunk) [binary32 add, rounds to the shard dtype]. The chunk itself
 * is left unmodified here (it is scratch in the reference after this point). */
void ref_post_reduce(void* shard, int sdt, const void* chunk, int cdt, int64_t n,
                     double post, int accumulate) {
  int scale = post > 1.0;
  float f = (float)post;
  for (int64_t i = 0; i < n; i++) {
    float y = load_f(chunk, cdt, i);
    if (scale) y = round_to(cdt, y / f);
    if (accumulate) y = load_f(shard, sdt, i) + y;
    store_f(shard, sdt, i, y);
  }
}

/* Reduce copy-in over a table of tensors laid out back to back in the flat
 * buffer: mode[p] 0 = tensor absent (its range keeps its old content),
 * 1 = view.copy_(grad), 2 = view.add_(grad).  Then flat.div_(pre) over the whole
 * padded buffer when pre > 1.  Pad lanes [T, T_pad) are set to zero first when
 * zero_pad is non-zero (the reference leaves them uninitialised). */
void ref_gather_in(int n_tensors, const void* const* tensors, const int64_t* offsets,
                   const uint8_t* mode, int tdt, void* flat, int fdt, int64_t t_pad,
                   double pre, int zero_pad) {
  for (int p = 0; p < n_tensors; p++) {
    int64_t o = offsets[p], n = offsets[p + 1] - o;
    if (mode[p] == 1) {
      if (tdt == fdt) memcpy((char*)flat + o * itemsize(fdt), tensors[p], (size_t)n * itemsize(fdt));
      else for (int64_t i = 0; i < n; i++) store_f(flat, fdt, o + i, load_f(tensors[p], tdt, i));
    } else if (mode[p] == 2) {
      for (int64_t i = 0; i < n; i++)
        store_f(flat, fdt, o + i, load_f(flat, fdt, o + i) + load_f(tensors[p], tdt, i));
    }
  }
  if (zero_pad) {
    int64_t t = offsets[n_tensors];
    memset((char*)flat + t * itemsize(fdt), 0, (size_t)(t_pad - t) * itemsize(fdt));
  }
  ref_flat_div(flat, fdt, t_pad, pre);
}

/* Materialising copy-out: flat[:T].split(numels)[p] -> tensors[p]. */
void ref_scatter_out(int n_tensors, void* const* tensors, const int64_t* offsets, int tdt,
                     const void* flat, int fdt) {
  for (int p = 0; p < n_tensors; p++) {
    int64_t o = offsets[p], n = offsets[p + 1] - o;
    if (tdt == fdt) memcpy(tensors[p], (const char*)flat + o * itemsize(fdt), (size_t)n * itemsize(fdt));
    else for (int64_t i = 0; i < n; i++) store_f(tensors[p], tdt, i, load_f(flat, fdt, o + i));
  }
}

/* ---- optimizer-side passes over the flat shard --------------------------------
 * The reference forwards torch.optim's foreach / fused Adam ops to the local
 * fragments of the flat shard (ya_fsdp/_tensor.py:269-312).  Per element, with
 * every intermediate tensor rounded to binary32, torch.optim.Adam(W) computes
 * (torch/optim/adam.py, `_single_tensor_adam`, the non-capturable branch):
 *
 *   grad = grad.add(param, alpha=wd)               Adam (L2 form) only
 *   param.mul_(1 - lr*wd)                          AdamW only
 *   exp_avg.lerp_(grad, 1 - beta1)
 *   exp_avg_sq.mul_(beta2).addcmul_(grad, grad, value=1 - beta2)
 *   denom = (exp_avg_sq.sqrt() / sqrt(1 - beta2^t)).add_(eps)
 *   param.addcdiv_(exp_avg, denom, value=-(lr / (1 - beta1^t)))
 *
 * torch's CPU kernels evaluate `add(alpha)`, `lerp_` and `addcmul_` with one
 * fused multiply-add each: fma(param, wd, grad); fma(w, grad - exp_avg, exp_avg)
 * for |w| < 0.5 and fma(w - 1, grad - exp_avg, grad) otherwise; fma((1-beta2)*grad,
 * grad, exp_avg_sq).  `addcdiv_` is not fused: param + (value*exp_avg)/denom.
 * (Established by comparing each torch op with both candidates on a million
 * random elements; tests/test_optim_oracle.py repeats the comparison.)  Square
 * root and division are correctly rounded here; torch's CPU sqrt is off by one
 * ulp for about 0.6 % of inputs, so whole steps agree with torch to 1 ulp, not
 * bit for bit. */
#include <math.h>

void ref_adamw_step(float* p, float* g, float* m, float* v, void* out16, int out_dt, int64_t n,
                    double lr, double beta1, double beta2, double eps, double wd, int64_t step,
                    int decoupled, int has_scale, float grad_scale, int zero_grad) {
  const float decay = (float)(1.0 - lr * wd);
  const float l2 = (float)wd;
  const float w = (float)(1.0 - beta1);
  const float w_m1 = w - 1.0f;
  const float b2 = (float)beta2;
  const float a = (float)(1.0 - beta2);
  const double bc1 = 1.0 - pow(beta1, (double)step);
  const double bc2 = 1.0 - pow(beta2, (double)step);
  const float bc2_sqrt = (float)pow(bc2, 0.5);
  const float epsf = (float)eps;
  const float neg_step = (float)(-(lr / bc1));
  for (int64_t i = 0; i < n; i++) {
    float gi = g[i], pi = p[i], mi = m[i], vi = v[i];
    if (has_scale) gi = gi * grad_scale;
    if (wd != 0.0) {
      if (decoupled) pi = pi * decay;
      else gi = fmaf(pi, l2, gi);
    }
    const float d = gi - mi;
    mi = (fabsf(w) < 0.5f) ? fmaf(w, d, mi) : fmaf(w_m1, d, gi);
    vi = vi * b2;
    vi = fmaf(a * gi, gi, vi);
    const float den = sqrtf(vi) / bc2_sqrt + epsf;
    pi = pi + (neg_step * mi) / den;
    p[i] = pi;
    m[i] = mi;
    v[i] = vi;
    if (out16) store_f(out16, out_dt, i, pi);
    if (zero_grad) g[i] = 0.0f;
  }
}

/* sum of squares in binary64 (each square is exact there), added in index order
 * with Neumaier's compensation, so the result is the exact sum rounded to
 * binary64 to within an ulp or two whatever the length */
double ref_sumsq(const void* src, int dt, int64_t n) {
  double sum = 0.0, comp = 0.0;
  for (int64_t i = 0; i < n; i++) {
    const double x = (double)load_f(src, dt, i);
    const double y = x * x;
    const double t = sum + y;
    if (fabs(sum) >= fabs(y)) comp += (sum - t) + y;
    else comp += (y - t) + sum;
    sum = t;
  }
  if (!isfinite(sum)) return sum; /* overflow or NaN input: the compensation term is meaningless */
  return sum + comp;
}

/* out[0] = float(sqrt(sumsq)); out[1] = min(max_norm / (out[0] + 1e-6), 1)
 * (ya_fsdp/ya_fsdp.py:557-559), NaN kept */
void ref_clip_coef(double sumsq, double max_norm, float* out) {
  const float norm = (float)sqrt(sumsq);
  float c = (float)max_norm / (norm + 1e-6f);
  if (c > 1.0f) c = 1.0f;
  out[0] = norm;
  out[1] = c;
}

/* buf[i] = round(float(buf[i]) * coef)   (grad.mul_(coef), ya_fsdp/ya_fsdp.py:560-561) */
void ref_flat_scale(void* buf, int dt, int64_t n, float coef) {
  for (int64_t i = 0; i < n; i++) store_f(buf, dt, i, load_f(buf, dt, i) * coef);
}

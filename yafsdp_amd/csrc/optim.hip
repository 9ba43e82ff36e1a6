// Instantiations and dtype dispatch of the optimizer-side kernels.
#include "launch.h"
#include "optim_kernels.hip.h"
#include "tuning.h"

namespace yafsdp {

hipError_t launch_fill(int dt, void* dst, int64_t n, int head, uint32_t pattern, int grid, hipStream_t stream) {
  switch (dt) {
    case DT_F32:
      return launch_kernel(fill_kernel<F32, kFillBlock, kFillUnroll, kOptNtStore>, grid, kFillBlock, stream, dst, n, head,
                           pattern);
    case DT_BF16:
      return launch_kernel(fill_kernel<BF16, kFillBlock, kFillUnroll, kOptNtStore>, grid, kFillBlock, stream, dst, n, head,
                           pattern);
    case DT_F16:
      return launch_kernel(fill_kernel<F16, kFillBlock, kFillUnroll, kOptNtStore>, grid, kFillBlock, stream, dst, n, head,
                           pattern);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_scale(int dt, void* buf, int64_t n, int head, const float* coef, int grid, hipStream_t stream) {
  switch (dt) {
    case DT_F32:
      return launch_kernel(scale_kernel<F32, kScaleBlock, kScaleUnroll, kOptNtLoad, kOptNtStore>, grid, kScaleBlock,
                           stream, buf, n, head, coef);
    case DT_BF16:
      return launch_kernel(scale_kernel<BF16, kScaleBlock, kScaleUnroll, kOptNtLoad, kOptNtStore>, grid, kScaleBlock,
                           stream, buf, n, head, coef);
    case DT_F16:
      return launch_kernel(scale_kernel<F16, kScaleBlock, kScaleUnroll, kOptNtLoad, kOptNtStore>, grid, kScaleBlock,
                           stream, buf, n, head, coef);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_sumsq_partials(int dt, const void* src, int64_t n, int head, double* partials, int grid,
                                 hipStream_t stream) {
  switch (dt) {
    case DT_F32:
      return launch_kernel(sumsq_kernel<F32, kSumsqBlock, kSumsqUnroll, kOptNtLoad>, grid, kSumsqBlock, stream, src, n,
                           head, partials);
    case DT_BF16:
      return launch_kernel(sumsq_kernel<BF16, kSumsqBlock, kSumsqUnroll, kOptNtLoad>, grid, kSumsqBlock, stream, src, n,
                           head, partials);
    case DT_F16:
      return launch_kernel(sumsq_kernel<F16, kSumsqBlock, kSumsqUnroll, kOptNtLoad>, grid, kSumsqBlock, stream, src, n,
                           head, partials);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_sumsq_finish(const double* partials, int64_t count, double* sumsq, int accumulate, float max_norm,
                               float* norm_and_coef, hipStream_t stream) {
  return launch_kernel(sumsq_finish_kernel<1024>, 1, 1024, stream, partials, count, sumsq, accumulate, max_norm,
                       norm_and_coef);
}

hipError_t launch_sumsq_reduce(const double* in, int64_t count, double* out, int grid, hipStream_t stream) {
  return launch_kernel(sumsq_reduce_kernel<1024>, grid, 1024, stream, in, count, out);
}

hipError_t launch_clip_coef(const double* sumsq, float max_norm, float* norm_and_coef, hipStream_t stream) {
  return launch_kernel(clip_coef_kernel, 1, 64, stream, sumsq, max_norm, norm_and_coef);
}

namespace {
template <class O, bool ZERO_GRAD>
hipError_t adamw_go(float* p, float* g, float* m, float* v, void* out16, int64_t n, int head, const AdamScalars& s,
                    const float* grad_scale, int grid, hipStream_t stream) {
  return launch_kernel(adamw_kernel<O, ZERO_GRAD, kAdamBlock, kAdamUnroll, kOptNtLoad, kAdamStorePolicy>, grid, kAdamBlock,
                       stream, p, g, m, v, out16, n, head, s, grad_scale);
}
template <class O>
hipError_t adamw_by_zero(float* p, float* g, float* m, float* v, void* out16, int64_t n, int head,
                         const AdamScalars& s, const float* grad_scale, int grid, hipStream_t stream) {
  if (s.flags & ADAM_ZERO_GRAD) return adamw_go<O, true>(p, g, m, v, out16, n, head, s, grad_scale, grid, stream);
  return adamw_go<O, false>(p, g, m, v, out16, n, head, s, grad_scale, grid, stream);
}
}  // namespace

hipError_t launch_adamw(int out_dt, float* p, float* g, float* m, float* v, void* out16, int64_t n, int head,
                        const AdamScalars& s, const float* grad_scale, int grid, hipStream_t stream) {
  if (out16 == nullptr) return adamw_by_zero<F32>(p, g, m, v, nullptr, n, head, s, grad_scale, grid, stream);
  if (out_dt == DT_BF16) return adamw_by_zero<BF16>(p, g, m, v, out16, n, head, s, grad_scale, grid, stream);
  if (out_dt == DT_F16) return adamw_by_zero<F16>(p, g, m, v, out16, n, head, s, grad_scale, grid, stream);
  return hipErrorInvalidValue;
}

}  // namespace yafsdp

// Instantiations and dtype dispatch of the optimizer-side kernels.
#include "launch.h"
#include "optim_kernels.cuh"
#include "tuning.h"

namespace yafsdp {

hipError_t launch_fill(int dt, void* dst, int64_t n, int head, uint32_t pattern, int grid, hipStream_t stream) {
  switch (dt) {
    case DT_F32:
      fill_kernel<F32, kFillBlock, kFillUnroll, kOptNtStore><<<dim3(grid), dim3(kFillBlock), 0, stream>>>(dst, n, head, pattern);
      break;
    case DT_BF16:
      fill_kernel<BF16, kFillBlock, kFillUnroll, kOptNtStore><<<dim3(grid), dim3(kFillBlock), 0, stream>>>(dst, n, head, pattern);
      break;
    case DT_F16:
      fill_kernel<F16, kFillBlock, kFillUnroll, kOptNtStore><<<dim3(grid), dim3(kFillBlock), 0, stream>>>(dst, n, head, pattern);
      break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t launch_scale(int dt, void* buf, int64_t n, int head, const float* coef, int grid, hipStream_t stream) {
  switch (dt) {
    case DT_F32:
      scale_kernel<F32, kScaleBlock, kScaleUnroll, kOptNtLoad, kOptNtStore>
          <<<dim3(grid), dim3(kScaleBlock), 0, stream>>>(buf, n, head, coef);
      break;
    case DT_BF16:
      scale_kernel<BF16, kScaleBlock, kScaleUnroll, kOptNtLoad, kOptNtStore>
          <<<dim3(grid), dim3(kScaleBlock), 0, stream>>>(buf, n, head, coef);
      break;
    case DT_F16:
      scale_kernel<F16, kScaleBlock, kScaleUnroll, kOptNtLoad, kOptNtStore>
          <<<dim3(grid), dim3(kScaleBlock), 0, stream>>>(buf, n, head, coef);
      break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t launch_sumsq_partials(int dt, const void* src, int64_t n, int head, double* partials, int grid,
                                 hipStream_t stream) {
  switch (dt) {
    case DT_F32:
      sumsq_kernel<F32, kSumsqBlock, kSumsqUnroll, kOptNtLoad><<<dim3(grid), dim3(kSumsqBlock), 0, stream>>>(src, n, head, partials);
      break;
    case DT_BF16:
      sumsq_kernel<BF16, kSumsqBlock, kSumsqUnroll, kOptNtLoad><<<dim3(grid), dim3(kSumsqBlock), 0, stream>>>(src, n, head, partials);
      break;
    case DT_F16:
      sumsq_kernel<F16, kSumsqBlock, kSumsqUnroll, kOptNtLoad><<<dim3(grid), dim3(kSumsqBlock), 0, stream>>>(src, n, head, partials);
      break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t launch_sumsq_finish(const double* partials, int64_t count, double* sumsq, int accumulate, float max_norm,
                               float* norm_and_coef, hipStream_t stream) {
  sumsq_finish_kernel<1024><<<dim3(1), dim3(1024), 0, stream>>>(partials, count, sumsq, accumulate, max_norm,
                                                              norm_and_coef);
  return hipGetLastError();
}

hipError_t launch_clip_coef(const double* sumsq, float max_norm, float* norm_and_coef, hipStream_t stream) {
  clip_coef_kernel<<<dim3(1), dim3(64), 0, stream>>>(sumsq, max_norm, norm_and_coef);
  return hipGetLastError();
}

namespace {
template <class O, bool ZERO_GRAD>
hipError_t adamw_go(float* p, float* g, float* m, float* v, void* out16, int64_t n, int head, const AdamScalars& s,
                    const float* grad_scale, int grid, hipStream_t stream) {
  adamw_kernel<O, ZERO_GRAD, kAdamBlock, kAdamUnroll, kOptNtLoad, kOptNtStore>
      <<<dim3(grid), dim3(kAdamBlock), 0, stream>>>(p, g, m, v, out16, n, head, s, grad_scale);
  return hipGetLastError();
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

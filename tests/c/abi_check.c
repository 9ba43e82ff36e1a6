/* A plain C program on the C ABI of libyafsdp_hip.so: no Python, no torch.
 * Device buffers come from the HIP runtime, inputs from a fixed generator, and
 * every result is compared bit for bit (sum of squares: to binary64 rounding)
 * with the plain-C restatement in oracle/bufpath_ref.c, linked as
 * libbufpath_ref.so.  Prints one line per check and exits non-zero on the first
 * mismatch.  Built by tests/c/build.py; run by tests/test_gpu_c_program.py. */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../../include/yafsdp_hip.h"

/* oracle/bufpath_ref.c */
void ref_flat_copy(void* dst, int dd, const void* src, int sd, int64_t n);
void ref_post_reduce(void* shard, int sdt, const void* chunk, int cdt, int64_t n, double post, int accumulate);
void ref_flat_premul(void* buf, int dt, int64_t n, double scalar);
void ref_gather_in(int n_tensors, const void* const* tensors, const int64_t* offsets, const uint8_t* mode, int tdt,
                   void* flat, int fdt, int64_t t_pad, double pre, int zero_pad);
void ref_scatter_out(int n_tensors, void* const* tensors, const int64_t* offsets, int tdt, const void* flat, int fdt);
void ref_adamw_step(float* p, float* g, float* m, float* v, void* out16, int out_dt, int64_t n, double lr, double beta1,
                    double beta2, double eps, double wd, int64_t step, int decoupled, int has_scale, float grad_scale,
                    int zero_grad);
double ref_sumsq(const void* src, int dt, int64_t n);
void ref_clip_coef(double sumsq, double max_norm, float* out);

#define HIP(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); return 2; } } while (0)
#define YA(x) do { int r_ = (x); if (r_ != 0) { printf("%s -> %s (line %d)\n", #x, yafsdp_error_string(r_), __LINE__); return 3; } } while (0)

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static float next_float(float scale) { /* roughly uniform in (-scale, scale), plus a few exact zeros */
  rng_state = rng_state * 6364136223846793005ull + 1442695040888963407ull;
  const uint32_t r = (uint32_t)(rng_state >> 33);
  if ((r & 1023u) == 0) return 0.0f;
  return scale * ((float)(r & 0xFFFFFFu) / 8388608.0f - 1.0f);
}
static uint16_t to_bf16(float f) { uint16_t out; ref_flat_copy(&out, YAFSDP_BF16, &f, YAFSDP_F32, 1); return out; }

static int same(const char* what, const void* a, const void* b, size_t bytes) {
  if (memcmp(a, b, bytes) != 0) {
    const unsigned char *x = a, *y = b;
    size_t i = 0;
    while (x[i] == y[i]) i++;
    printf("MISMATCH %s at byte %zu of %zu\n", what, i, bytes);
    return 0;
  }
  printf("ok %s (%zu bytes)\n", what, bytes);
  return 1;
}

int main(void) {
  printf("library version %d\n", yafsdp_version());
  HIP(hipSetDevice(0));
  hipStream_t stream;
  HIP(hipStreamCreate(&stream));
  enum { P = 4 };
  const int64_t numels[P] = {1000003, 77, 0, 333331};
  int64_t offsets[P + 1] = {0};
  for (int p = 0; p < P; p++) offsets[p + 1] = offsets[p] + numels[p];
  const int64_t total = offsets[P], padded = total + 29;

  /* ---- reduce copy-in: bf16 gradients -> fp32 flat buffer, copy / add / absent, /8, pad zero-fill */
  uint16_t* h_grads[P];
  void* d_grads[P];
  for (int p = 0; p < P; p++) {
    h_grads[p] = malloc((size_t)(numels[p] ? numels[p] : 1) * 2);
    for (int64_t i = 0; i < numels[p]; i++) h_grads[p][i] = to_bf16(next_float(1e-2f));
    HIP(hipMalloc(&d_grads[p], (size_t)(numels[p] ? numels[p] : 1) * 2));
    HIP(hipMemcpy(d_grads[p], h_grads[p], (size_t)numels[p] * 2, hipMemcpyHostToDevice));
  }
  float* h_flat = malloc((size_t)padded * 4);
  float* h_want = malloc((size_t)padded * 4);
  for (int64_t i = 0; i < padded; i++) h_flat[i] = next_float(1e-3f);
  memcpy(h_want, h_flat, (size_t)padded * 4);
  const uint8_t modes[P] = {YAFSDP_MODE_ADD, YAFSDP_MODE_COPY, YAFSDP_MODE_COPY, YAFSDP_MODE_SKIP};
  ref_gather_in(P, (const void* const*)h_grads, offsets, modes, YAFSDP_BF16, h_want, YAFSDP_F32, padded, 8.0, 1);
  float* d_flat;
  HIP(hipMalloc((void**)&d_flat, (size_t)padded * 4));
  HIP(hipMemcpy(d_flat, h_flat, (size_t)padded * 4, hipMemcpyHostToDevice));
  yafsdp_table* table = NULL;
  YA(yafsdp_table_create(P, numels, padded, &table));
  YA(yafsdp_gather_in(table, (const void* const*)d_grads, modes, YAFSDP_BF16, d_flat, YAFSDP_F32, 8.0, 1, stream));
  HIP(hipStreamSynchronize(stream));
  HIP(hipMemcpy(h_flat, d_flat, (size_t)padded * 4, hipMemcpyDeviceToHost));
  if (!same("gather_in bf16 -> f32, /8", h_flat, h_want, (size_t)padded * 4)) return 1;

  /* ---- copy-out through a binding: fp32 flat -> bf16 tensors */
  uint16_t* h_out[P];
  uint16_t* h_out_want[P];
  void* d_out[P];
  for (int p = 0; p < P; p++) {
    const size_t bytes = (size_t)(numels[p] ? numels[p] : 1) * 2;
    h_out[p] = malloc(bytes);
    h_out_want[p] = malloc(bytes);
    HIP(hipMalloc(&d_out[p], bytes));
  }
  ref_scatter_out(P, (void* const*)h_out_want, offsets, YAFSDP_BF16, h_want, YAFSDP_F32);
  yafsdp_binding* binding = NULL;
  YA(yafsdp_binding_create(table, (const void* const*)d_out, NULL, YAFSDP_BF16, &binding));
  YA(yafsdp_scatter_out_bound(binding, d_flat, YAFSDP_F32, stream));
  HIP(hipStreamSynchronize(stream));
  for (int p = 0; p < P; p++) {
    HIP(hipMemcpy(h_out[p], d_out[p], (size_t)numels[p] * 2, hipMemcpyDeviceToHost));
    char what[64];
    snprintf(what, sizeof what, "scatter_out (bound) tensor %d", p);
    if (!same(what, h_out[p], h_out_want[p], (size_t)numels[p] * 2)) return 1;
  }

  /* ---- copy-in + copy-out as ONE launch: fp32 master shard -> bf16 all-gather input, next to the split of a bf16
   * gathered buffer into bf16 tensors */
  {
    const int64_t ns = 123457;
    float* h_master = malloc((size_t)ns * 4);
    uint16_t *h_ag = malloc((size_t)ns * 2), *h_ag_want = malloc((size_t)ns * 2);
    uint16_t* h_gathered = malloc((size_t)padded * 2);
    for (int64_t i = 0; i < ns; i++) h_master[i] = next_float(2e-2f);
    for (int64_t i = 0; i < padded; i++) h_gathered[i] = to_bf16(next_float(2e-2f));
    ref_flat_copy(h_ag_want, YAFSDP_BF16, h_master, YAFSDP_F32, ns);
    ref_scatter_out(P, (void* const*)h_out_want, offsets, YAFSDP_BF16, h_gathered, YAFSDP_BF16);
    float* d_master;
    void *d_ag, *d_gathered;
    HIP(hipMalloc((void**)&d_master, (size_t)ns * 4));
    HIP(hipMalloc(&d_ag, (size_t)ns * 2));
    HIP(hipMalloc(&d_gathered, (size_t)padded * 2));
    HIP(hipMemcpy(d_master, h_master, (size_t)ns * 4, hipMemcpyHostToDevice));
    HIP(hipMemcpy(d_gathered, h_gathered, (size_t)padded * 2, hipMemcpyHostToDevice));
    YA(yafsdp_copy_in_scatter_out(table, d_gathered, YAFSDP_BF16, d_out, NULL, d_ag, d_master, YAFSDP_F32, ns, stream));
    HIP(hipStreamSynchronize(stream));
    HIP(hipMemcpy(h_ag, d_ag, (size_t)ns * 2, hipMemcpyDeviceToHost));
    if (!same("copy_in_scatter_out: all-gather input", h_ag, h_ag_want, (size_t)ns * 2)) return 1;
    for (int p = 0; p < P; p++) {
      HIP(hipMemcpy(h_out[p], d_out[p], (size_t)numels[p] * 2, hipMemcpyDeviceToHost));
      char what[64];
      snprintf(what, sizeof what, "copy_in_scatter_out: tensor %d", p);
      if (!same(what, h_out[p], h_out_want[p], (size_t)numels[p] * 2)) return 1;
    }
    free(h_master); free(h_ag); free(h_ag_want); free(h_gathered);
    HIP(hipFree(d_master)); HIP(hipFree(d_ag)); HIP(hipFree(d_gathered));
  }

  /* ---- reduce copy-in + post-reduce of a shard group of size one as ONE launch: bf16 gradients -> fp32 reduce
   * buffer (copy / add / absent), /4 before and /3 after the "reduce-scatter", accumulated into a bf16 shard */
  {
    float *h_rs = malloc((size_t)padded * 4), *h_rs_want = malloc((size_t)padded * 4);
    uint16_t *h_gs = malloc((size_t)padded * 2), *h_gs_want = malloc((size_t)padded * 2);
    for (int64_t i = 0; i < padded; i++) { h_rs[i] = next_float(1e-3f); h_gs[i] = to_bf16(next_float(1e-3f)); }
    memcpy(h_rs_want, h_rs, (size_t)padded * 4);
    memcpy(h_gs_want, h_gs, (size_t)padded * 2);
    ref_gather_in(P, (const void* const*)h_grads, offsets, modes, YAFSDP_BF16, h_rs_want, YAFSDP_F32, padded, 4.0, 1);
    ref_post_reduce(h_gs_want, YAFSDP_BF16, h_rs_want, YAFSDP_F32, padded, 3.0, 1);
    float* d_rs;
    void* d_gs;
    HIP(hipMalloc((void**)&d_rs, (size_t)padded * 4));
    HIP(hipMalloc(&d_gs, (size_t)padded * 2));
    HIP(hipMemcpy(d_rs, h_rs, (size_t)padded * 4, hipMemcpyHostToDevice));
    HIP(hipMemcpy(d_gs, h_gs, (size_t)padded * 2, hipMemcpyHostToDevice));
    YA(yafsdp_gather_in_post_reduce(table, (const void* const*)d_grads, modes, YAFSDP_BF16, d_rs, YAFSDP_F32, 4.0, 0.0,
                                    3.0, 1, d_gs, YAFSDP_BF16, 1, stream));
    HIP(hipStreamSynchronize(stream));
    HIP(hipMemcpy(h_rs, d_rs, (size_t)padded * 4, hipMemcpyDeviceToHost));
    HIP(hipMemcpy(h_gs, d_gs, (size_t)padded * 2, hipMemcpyDeviceToHost));
    if (!same("gather_in_post_reduce: reduce buffer", h_rs, h_rs_want, (size_t)padded * 4)) return 1;
    if (!same("gather_in_post_reduce: gradient shard", h_gs, h_gs_want, (size_t)padded * 2)) return 1;
    free(h_rs); free(h_rs_want); free(h_gs); free(h_gs_want);
    HIP(hipFree(d_rs)); HIP(hipFree(d_gs));
  }

  /* ---- post-reduce: bf16 chunk /3 accumulated into an fp32 shard */
  const int64_t s = 500009;
  float* h_shard = malloc((size_t)s * 4);
  float* h_shard_want = malloc((size_t)s * 4);
  for (int64_t i = 0; i < s; i++) h_shard[i] = next_float(1e-4f);
  memcpy(h_shard_want, h_shard, (size_t)s * 4);
  ref_post_reduce(h_shard_want, YAFSDP_F32, h_grads[0], YAFSDP_BF16, s, 3.0, 1);
  float* d_shard;
  HIP(hipMalloc((void**)&d_shard, (size_t)s * 4));
  HIP(hipMemcpy(d_shard, h_shard, (size_t)s * 4, hipMemcpyHostToDevice));
  YA(yafsdp_post_reduce(d_shard, YAFSDP_F32, d_grads[0], YAFSDP_BF16, s, 3.0, 1, stream));
  HIP(hipStreamSynchronize(stream));
  HIP(hipMemcpy(h_shard, d_shard, (size_t)s * 4, hipMemcpyDeviceToHost));
  if (!same("post_reduce bf16 /3 += f32", h_shard, h_shard_want, (size_t)s * 4)) return 1;

  /* ---- the same post-reduce through the entry point that also leaves the squared norm of the shard */
  {
    float* d_shard2;
    double* d_part;
    const int64_t cap = yafsdp_post_reduce_sumsq_count(s);
    int64_t n_part = 0;
    HIP(hipMalloc((void**)&d_shard2, (size_t)s * 4));
    HIP(hipMalloc((void**)&d_part, (size_t)cap * 8));
    for (int64_t i = 0; i < s; i++) h_shard[i] = h_shard_want[i];  /* start from the first result: accumulate again */
    float* h_twice = malloc((size_t)s * 4);
    memcpy(h_twice, h_shard_want, (size_t)s * 4);
    ref_post_reduce(h_twice, YAFSDP_F32, h_grads[0], YAFSDP_BF16, s, 3.0, 1);
    HIP(hipMemcpy(d_shard2, h_shard, (size_t)s * 4, hipMemcpyHostToDevice));
    YA(yafsdp_post_reduce_sumsq(d_shard2, YAFSDP_F32, d_grads[0], YAFSDP_BF16, s, 3.0, 1, d_part, cap, &n_part, stream));
    HIP(hipStreamSynchronize(stream));
    HIP(hipMemcpy(h_shard, d_shard2, (size_t)s * 4, hipMemcpyDeviceToHost));
    if (!same("post_reduce_sumsq shard", h_shard, h_twice, (size_t)s * 4)) return 1;
    double* h_part = malloc((size_t)cap * 8);
    HIP(hipMemcpy(h_part, d_part, (size_t)n_part * 8, hipMemcpyDeviceToHost));
    double got = 0.0;
    for (int64_t i = 0; i < n_part; i++) got += h_part[i];
    const double want = ref_sumsq(h_twice, YAFSDP_F32, s);
    if (n_part < 1 || n_part > cap || fabs(got - want) > 1e-12 * want) {
      printf("MISMATCH post_reduce_sumsq: %lld sums, %.17g vs %.17g\n", (long long)n_part, got, want);
      return 1;
    }
    printf("ok post_reduce_sumsq %.17g in %lld partial sums\n", got, (long long)n_part);
    free(h_twice); free(h_part);
    HIP(hipFree(d_shard2)); HIP(hipFree(d_part));
    memcpy(h_shard, h_shard_want, (size_t)s * 4);
  }

  /* ---- this rank's share of a reduce-scatter that scales inside the reduction (ReduceOp.AVG over 3 ranks): the
   * bf16 chunk times bf16(1 / 3), rounded to bf16, accumulated into the fp32 shard - not a division by 3.  The
   * completion event is recorded by the kernel's own dispatch instead of by a marker behind it. */
  {
    uint16_t* h_chunk = malloc((size_t)s * 2);
    float* h_share_want = malloc((size_t)s * 4);
    float* h_by_division = malloc((size_t)s * 4);
    memcpy(h_chunk, h_grads[0], (size_t)s * 2);
    memcpy(h_share_want, h_shard_want, (size_t)s * 4);
    memcpy(h_by_division, h_shard_want, (size_t)s * 4);
    ref_post_reduce(h_by_division, YAFSDP_F32, h_chunk, YAFSDP_BF16, s, 3.0, 1);
    ref_flat_premul(h_chunk, YAFSDP_BF16, s, 1.0 / 3.0);
    ref_post_reduce(h_share_want, YAFSDP_F32, h_chunk, YAFSDP_BF16, s, 0.0, 1);
    float* d_share;
    hipEvent_t done;
    HIP(hipMalloc((void**)&d_share, (size_t)s * 4));
    HIP(hipMemcpy(d_share, h_shard_want, (size_t)s * 4, hipMemcpyHostToDevice));
    HIP(hipEventCreateWithFlags(&done, hipEventDisableTiming));
    YA(yafsdp_complete_next_launch(done));
    YA(yafsdp_post_reduce_premul(d_share, YAFSDP_F32, d_grads[0], YAFSDP_BF16, s, 1.0 / 3.0, 1, stream));
    if (yafsdp_complete_next_launch_pending()) { printf("MISMATCH the launch left the completion event armed\n"); return 1; }
    HIP(hipEventSynchronize(done));  /* the kernel has completed: no stream synchronisation needed */
    HIP(hipMemcpy(h_shard, d_share, (size_t)s * 4, hipMemcpyDeviceToHost));
    if (!same("post_reduce_premul bf16 * bf16(1/3) += f32, event from the dispatch", h_shard, h_share_want, (size_t)s * 4))
      return 1;
    int64_t differ = 0;
    for (int64_t i = 0; i < s; i++) differ += memcmp(&h_share_want[i], &h_by_division[i], 4) != 0;
    if (differ == 0) { printf("MISMATCH the scaled share equals a division by 3 everywhere\n"); return 1; }
    printf("ok the share differs from a division by 3 on %lld of %lld elements\n", (long long)differ, (long long)s);
    HIP(hipEventDestroy(done));
    HIP(hipFree(d_share));
    free(h_chunk); free(h_share_want); free(h_by_division);
    memcpy(h_shard, h_shard_want, (size_t)s * 4);
  }

  /* ---- store policy of one table: the write-through tail is an option per table that follows the process-wide
   * default until it is set; it
   * changes no result */
  {
    int v = -2;
    YA(yafsdp_table_get_option(table, YAFSDP_OPT_GATHER_TAIL_MB, &v));
    if (v != -1) { printf("MISMATCH a new table's option reads %d, not -1 (follow the process)\n", v); return 1; }
    YA(yafsdp_table_set_option(table, YAFSDP_OPT_GATHER_TAIL_MB, 1));
    YA(yafsdp_table_get_option(table, YAFSDP_OPT_GATHER_TAIL_MB, &v));
    if (v != 1) { printf("MISMATCH table option reads %d after setting 1\n", v); return 1; }
    float* h_again = malloc((size_t)padded * 4);
    for (int64_t i = 0; i < padded; i++) h_again[i] = next_float(1e-3f);
    memcpy(h_want, h_again, (size_t)padded * 4);
    ref_gather_in(P, (const void* const*)h_grads, offsets, modes, YAFSDP_BF16, h_want, YAFSDP_F32, padded, 8.0, 1);
    HIP(hipMemcpy(d_flat, h_again, (size_t)padded * 4, hipMemcpyHostToDevice));
    YA(yafsdp_gather_in(table, (const void* const*)d_grads, modes, YAFSDP_BF16, d_flat, YAFSDP_F32, 8.0, 1, stream));
    HIP(hipStreamSynchronize(stream));
    HIP(hipMemcpy(h_again, d_flat, (size_t)padded * 4, hipMemcpyDeviceToHost));
    if (!same("gather_in with a 1-MB write-through tail on this table", h_again, h_want, (size_t)padded * 4)) return 1;
    YA(yafsdp_table_set_option(table, YAFSDP_OPT_GATHER_TAIL_MB, -1));
    printf("ok table option\n");
    free(h_again);
  }

  /* ---- gradient norm, clip coefficient, fused AdamW with bf16 copy-in */
  double want_sumsq = ref_sumsq(h_shard_want, YAFSDP_F32, s);
  float want_nc[2];
  ref_clip_coef(want_sumsq, 1e-3, want_nc);
  double* d_sumsq;
  float* d_nc;
  void* d_ws;
  HIP(hipMalloc((void**)&d_sumsq, 8));
  HIP(hipMalloc((void**)&d_nc, 8));
  HIP(hipMalloc(&d_ws, yafsdp_sumsq_workspace_bytes()));
  YA(yafsdp_flat_sumsq(d_shard, YAFSDP_F32, s, d_sumsq, 0, d_ws, yafsdp_sumsq_workspace_bytes(), stream));
  YA(yafsdp_clip_coef(d_sumsq, 1e-3, d_nc, stream));
  HIP(hipStreamSynchronize(stream));
  double got_sumsq;
  float got_nc[2];
  HIP(hipMemcpy(&got_sumsq, d_sumsq, 8, hipMemcpyDeviceToHost));
  HIP(hipMemcpy(got_nc, d_nc, 8, hipMemcpyDeviceToHost));
  if (fabs(got_sumsq - want_sumsq) > 1e-12 * want_sumsq) { printf("MISMATCH sumsq %.17g vs %.17g\n", got_sumsq, want_sumsq); return 1; }
  printf("ok sumsq %.17g\n", got_sumsq);
  if (!same("norm and clip coefficient", got_nc, want_nc, 8)) return 1;

  float *h_p = malloc((size_t)s * 4), *h_m = calloc((size_t)s, 4), *h_v = calloc((size_t)s, 4);
  uint16_t *h_o16 = malloc((size_t)s * 2), *h_o16_want = malloc((size_t)s * 2);
  for (int64_t i = 0; i < s; i++) h_p[i] = next_float(2e-2f);
  float *d_p, *d_m, *d_v;
  void* d_o16;
  HIP(hipMalloc((void**)&d_p, (size_t)s * 4));
  HIP(hipMalloc((void**)&d_m, (size_t)s * 4));
  HIP(hipMalloc((void**)&d_v, (size_t)s * 4));
  HIP(hipMalloc(&d_o16, (size_t)s * 2));
  HIP(hipMemcpy(d_p, h_p, (size_t)s * 4, hipMemcpyHostToDevice));
  HIP(hipMemset(d_m, 0, (size_t)s * 4));
  HIP(hipMemset(d_v, 0, (size_t)s * 4));
  YA(yafsdp_adamw_step(d_p, d_shard, d_m, d_v, d_o16, YAFSDP_BF16, s, 3e-4, 0.9, 0.95, 1e-8, 0.1, 1, d_nc + 1,
                       YAFSDP_ADAM_DECOUPLED_DECAY | YAFSDP_ADAM_ZERO_GRAD, stream));
  HIP(hipStreamSynchronize(stream));
  ref_adamw_step(h_p, h_shard_want, h_m, h_v, h_o16_want, YAFSDP_BF16, s, 3e-4, 0.9, 0.95, 1e-8, 0.1, 1, 1, 1, want_nc[1], 1);
  float* h_tmp = malloc((size_t)s * 4);
  HIP(hipMemcpy(h_tmp, d_p, (size_t)s * 4, hipMemcpyDeviceToHost));
  if (!same("adamw parameters", h_tmp, h_p, (size_t)s * 4)) return 1;
  HIP(hipMemcpy(h_tmp, d_m, (size_t)s * 4, hipMemcpyDeviceToHost));
  if (!same("adamw exp_avg", h_tmp, h_m, (size_t)s * 4)) return 1;
  HIP(hipMemcpy(h_tmp, d_v, (size_t)s * 4, hipMemcpyDeviceToHost));
  if (!same("adamw exp_avg_sq", h_tmp, h_v, (size_t)s * 4)) return 1;
  HIP(hipMemcpy(h_tmp, d_shard, (size_t)s * 4, hipMemcpyDeviceToHost));
  if (!same("adamw zero-filled gradient", h_tmp, h_shard_want, (size_t)s * 4)) return 1;
  HIP(hipMemcpy(h_o16, d_o16, (size_t)s * 2, hipMemcpyDeviceToHost));
  if (!same("adamw bf16 copy-in", h_o16, h_o16_want, (size_t)s * 2)) return 1;

  /* opaque bytes at odd addresses on both sides (1-byte all-gather dtypes): d_p's bytes, shifted by 3, into
   * d_m's, shifted by 5; the bytes around the destination range stay as they are */
  {
    const size_t n_bytes = (size_t)s * 4 - 64 - 7;
    unsigned char* h_dst = malloc((size_t)s * 4);
    HIP(hipMemcpy(h_dst, d_m, (size_t)s * 4, hipMemcpyDeviceToHost));
    memcpy(h_dst + 5, (const unsigned char*)h_p + 3, n_bytes);
    YA(yafsdp_flat_copy_bytes((char*)d_m + 5, (const char*)d_p + 3, (int64_t)n_bytes, stream));
    HIP(hipStreamSynchronize(stream));
    HIP(hipMemcpy(h_tmp, d_m, (size_t)s * 4, hipMemcpyDeviceToHost));
    if (!same("byte copy at odd addresses", h_tmp, h_dst, (size_t)s * 4)) return 1;
    free(h_dst);
  }

  YA(yafsdp_binding_destroy(binding));
  YA(yafsdp_table_destroy(table));
  printf("PASS\n");
  return 0;
}

// C ABI of libyafsdp_hip.so: argument validation, metadata tables, launch
// shapes.  Declarations and the reference call sites each entry point replaces
// are in include/yafsdp_hip.h.
#include <atomic>
#include <cmath>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "../../include/yafsdp_hip.h"
#include "launch.h"
#include "stage_ring.h"
#include "tuning.h"

using namespace yafsdp;

thread_local yafsdp::TimedLaunch yafsdp::tl_timed_launch;

// Scratch of yafsdp_flat_sumsq_static: the per-workgroup partial sums that yafsdp_flat_sumsq keeps in the caller's
// workspace.  One copy per GPU the library runs on (128 KiB each), held until the process ends.  In host code this
// name is only a handle for hipGetSymbolAddress; device memory is reached through the per-device pointer below.
static __device__ __align__(256) double g_sumsq_static_scratch[yafsdp::kSumsqMaxPartials];

namespace {

std::atomic<int> g_flat_blocks_per_cu{kFlatBlocksPerCu};
std::atomic<int> g_table_blocks_per_cu{kTableBlocksPerCu};
std::atomic<int> g_table_large_log2{kTableLargeThresholdLog2};
std::atomic<int> g_gather_tail_mb{kGatherTailWriteThroughMb};
std::atomic<int> g_scatter_tail_mb{kScatterTailWriteThroughMb};
std::atomic<int> g_flat_tail_mb{kFlatTailWriteThroughMb};
std::atomic<int> g_post_reduce_tail_mb{kPostReduceTailWriteThroughMb};
std::atomic<int> g_scatter_tile_mode{0};

constexpr int kMaxDevices = 64;
std::atomic<int> g_cu_count[kMaxDevices];
// device address of g_sumsq_static_scratch on each device (every GPU holds its own copy at its own address)
std::atomic<double*> g_sumsq_static_ptr[kMaxDevices];

// Address of the static scratch on the current device, looked up once per device.
int sumsq_static_scratch(double** out) {
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return int(e);
  if (device < 0 || device >= kMaxDevices) return YAFSDP_ERR_WRONG_DEVICE;
  double* p = g_sumsq_static_ptr[device].load(std::memory_order_acquire);
  if (p == nullptr) {
    void* sym = nullptr;
    e = hipGetSymbolAddress(&sym, HIP_SYMBOL(g_sumsq_static_scratch));
    if (e != hipSuccess) return int(e);
    if (sym == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
    p = static_cast<double*>(sym);
    g_sumsq_static_ptr[device].store(p, std::memory_order_release);  // the same value from whichever thread wins
  }
  *out = p;
  return YAFSDP_OK;
}

int cu_count(int device) {
  if (device < 0 || device >= kMaxDevices) return 256;
  int c = g_cu_count[device].load(std::memory_order_relaxed);
  if (c > 0) return c;
  int v = 0;
  if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || v <= 0) v = 256;
  g_cu_count[device].store(v, std::memory_order_relaxed);
  return v;
}

inline bool valid_dtype(int dt) { return dt == DT_F32 || dt == DT_BF16 || dt == DT_F16; }
inline int item_size(int dt) { return dt == DT_F32 ? 4 : 2; }
inline bool aligned_to(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// How a divide factor is applied (ya_fsdp/_collectives.py:270-272: only > 1).
// A power-of-two factor whose reciprocal is a normal binary32 number becomes an
// exact multiply: x * 2^-k and x / 2^k are the same real number rounded once.
void scale_plan(double factor, int* scale, float* k) {
  *scale = SCALE_NONE;
  *k = 1.0f;
  if (!(factor > 1.0)) return;
  const float f = static_cast<float>(factor);
  if (!(f > 1.0f)) return;  // rounded down to 1: dividing by 1.0f changes nothing
  int e = 0;
  const float m = std::frexp(f, &e);
  if (m == 0.5f && e <= 126 && std::isfinite(f)) {
    *scale = SCALE_MUL;
    *k = 1.0f / f;
  } else {
    *scale = SCALE_DIV;
    *k = f;
  }
}

// Same for a division that is applied whatever the factor (not the "> 1" rule).
bool scale_plan_any(double divisor, int* scale, float* k) {
  const float f = static_cast<float>(divisor);
  if (!std::isfinite(f) || f == 0.0f) return false;
  int e = 0;
  const float m = std::frexp(std::fabs(f), &e);
  if (m == 0.5f && e <= 126 && e >= -124) {  // +-2^(e-1), reciprocal is a normal number
    *scale = SCALE_MUL;
    *k = 1.0f / f;
  } else {
    *scale = SCALE_DIV;
    *k = f;
  }
  return true;
}

// The scalar of a pre-multiplied sum as the collective applies it: converted to the data type (through binary32,
// round to nearest even), here as the binary32 number of that value.  A product with it is one exact binary32
// multiply for the 16-bit types (8 x 8 or 11 x 11 significand bits) and one rounded multiply for binary32.
bool premul_plan(double scalar, int dtype, int* scale, float* k) {
  float f = static_cast<float>(scalar);
  if (dtype == DT_BF16) {
    uint32_t bits;
    std::memcpy(&bits, &f, 4);
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return false;
    bits = ((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16) << 16;
    std::memcpy(&f, &bits, 4);
  } else if (dtype == DT_F16) {
    f = static_cast<float>(static_cast<_Float16>(f));
  }
  if (!std::isfinite(f)) return false;
  *scale = f == 1.0f ? SCALE_NONE : SCALE_MUL;
  *k = f;
  return true;
}

int grid_for(int64_t n_tiles, int blocks_per_cu, int device) {
  int64_t cap = int64_t(cu_count(device)) * (blocks_per_cu > 0 ? blocks_per_cu : 1);
  int64_t g = n_tiles < cap ? n_tiles : cap;
  return g < 1 ? 1 : int(g);
}

// first tile of a flat pass that writes through: the last tail_mb megabytes of its output (tile_units: 8-element
// units per tile; tail_mb: YAFSDP_OPT_FLAT_TAIL_MB, or YAFSDP_OPT_POST_REDUCE_TAIL_MB for the post-reduce)
int flat_wt_from(int64_t n_tiles, int64_t tile_units, int dst_dt, const std::atomic<int>& tail_mb) {
  const int64_t tile_bytes = tile_units * 8 * item_size(dst_dt);
  const int64_t tail = (int64_t(tail_mb.load(std::memory_order_relaxed)) << 20) / tile_bytes;
  const int64_t from = tail >= n_tiles ? 0 : n_tiles - tail;
  return from > INT32_MAX ? INT32_MAX : int(from);
}

int flat_launch(int src_dt, int dst_dt, int scale, bool acc, void* dst, const void* src, int64_t n, float k,
                hipStream_t stream, const std::atomic<int>& tail_mb = g_flat_tail_mb) {
  if (n == 0) return YAFSDP_OK;
  if (!aligned_to(dst, item_size(dst_dt)) || !aligned_to(src, item_size(src_dt))) return YAFSDP_ERR_MISALIGNED;
  if (src_dt == dst_dt && scale == SCALE_NONE && !acc && src_dt != DT_BF16) {
    // a same-dtype copy moves bytes, whatever they encode: it runs as the copy of 2-byte units, whose lanes each own
    // 16 consecutive bytes (872 MB of binary32: 82 % of peak as 2-byte units against 77 % in the arrangement that
    // the casts between binary32 and a 2-byte dtype use)
    n = n * item_size(src_dt) / 2;
    src_dt = dst_dt = DT_BF16;
  }
  {
    // in place (same address, same element size) is fine: every element is read before it is written by the
    // same lane; any other overlap of the two byte ranges has no defined result (torch's copy_ refuses it too)
    const uintptr_t d0 = reinterpret_cast<uintptr_t>(dst), s0 = reinterpret_cast<uintptr_t>(src);
    const uintptr_t d1 = d0 + uintptr_t(n) * item_size(dst_dt), s1 = s0 + uintptr_t(n) * item_size(src_dt);
    const bool in_place = d0 == s0 && item_size(dst_dt) == item_size(src_dt);
    if (!in_place && d0 < s1 && s0 < d1) return YAFSDP_ERR_INVALID_ARGUMENT;
  }
  // leading elements up to the destination's next 128-byte line (at most 63, fewer than a workgroup has lanes):
  // tiles are whole lines from there on, so no two workgroups write into one cache line
  static_assert(kFlatBlock >= 64, "workgroup 0 peels up to 63 leading elements, one per lane");
  int64_t head = ((128 - (reinterpret_cast<uintptr_t>(dst) & 127)) & 127) / item_size(dst_dt);
  if (head > n) head = n;
  const int64_t units = (n - head) >> 3;
  const int64_t tile = int64_t(kFlatBlock) * kFlatUnroll;
  const int64_t n_tiles = (units + tile - 1) / tile;
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return int(e);
  const int grid = grid_for(n_tiles, g_flat_blocks_per_cu.load(std::memory_order_relaxed), device);
  e = launch_flat(src_dt, dst_dt, scale, acc, dst, src, n, int(head), k, flat_wt_from(n_tiles, tile, dst_dt, tail_mb),
                  grid,
                  stream);
  return int(e);
}

}  // namespace

// The HIP side of the staging slots' state machine.
struct HipRuntime {
  typedef hipStream_t Stream;
  typedef hipEvent_t Event;
  static constexpr int kNotReady = int(hipErrorNotReady);
  int stream_wait_event(Stream s, Event e) { return int(hipStreamWaitEvent(s, e, 0)); }
  int event_query(Event e) { return int(hipEventQuery(e)); }
  int memcpy_h2d_async(void* dst, const void* src, size_t n, Stream s) {
    return int(hipMemcpyAsync(dst, src, n, hipMemcpyHostToDevice, s));
  }
  int event_record(Event e, Stream s) { return int(hipEventRecord(e, s)); }
};

struct yafsdp_table {
  int device = 0;
  int32_t n_tensors = 0;
  int64_t total = 0;
  int64_t padded = 0;
  std::vector<int64_t> offsets;  // host copy, n_tensors + 1
  int64_t* d_offsets = nullptr;
  int block = kTableBlockSmall;  // workgroup size of the table kernels, chosen from the padded size
  int64_t tile_elems = 0;        // gather-in tile: block * kGatherUnroll * 8 elements of the flat buffer
  int scatter_shape = 0;         // scatter-out: workgroup size * 16 + units per lane (see scatter_shape_for)
  int64_t slot_elems = 0;        // scatter-out tile (elements of one tensor)
  int32_t n_tiles = 0;           // gather-in: tiles of the flat buffer
  TileRec* d_tiles = nullptr;    // only for tables with more than kSmallMax tensors
  // scatter-out: tile slots per tensor (ceil(numel / tile) + 1 for a non-empty tensor)
  std::vector<int64_t> slot_start;  // host, n_tensors + 1
  int32_t n_slots = 0;
  TileRec* d_slots = nullptr;    // only for tables with more than kSmallMax tensors
  // staging slots for the per-call pointer / mode arrays of tables with more than kSmallMax tensors (stage_ring.h)
  StageRing<HipRuntime> ring;
  std::vector<char> scratch;        // host: the arrays of the current call in staging format
  std::mutex mu;
  // yafsdp_table_set_option: this table's own write-through tails, -1 = the process-wide option
  std::atomic<int> gather_tail_mb{-1};
  std::atomic<int> scatter_tail_mb{-1};
};

// The tensor side of a table fixed for many calls: validated once, and for
// tables with more than kSmallMax tensors staged to device memory once.
struct yafsdp_binding {
  yafsdp_table* table = nullptr;
  int tensor_dtype = 0;
  SmallMeta small;             // tables with at most kSmallMax tensors
  char* d_arrays = nullptr;    // others: pointers (8 bytes each) then modes (4 bytes each)
  LargeMeta large;
};

namespace {

// first gather-in tile that writes through: the last YAFSDP_OPT_GATHER_TAIL_MB megabytes of the flat buffer
int gather_wt_from(const yafsdp_table* t, int flat_dtype) {
  const int64_t tile_bytes = t->tile_elems * item_size(flat_dtype);
  if (tile_bytes <= 0) return 0;
  int mb = t->gather_tail_mb.load(std::memory_order_relaxed);
  if (mb < 0) mb = g_gather_tail_mb.load(std::memory_order_relaxed);
  const int64_t tail = (int64_t(mb) << 20) / tile_bytes;
  return tail >= t->n_tiles ? 0 : int(t->n_tiles - tail);
}

// first scatter-out tile slot that writes through: the slots of the last YAFSDP_OPT_SCATTER_TAIL_MB megabytes of tensors
int scatter_wt_from(const yafsdp_table* t, int tensor_dtype) {
  const int64_t slot_bytes = t->slot_elems * item_size(tensor_dtype);
  if (slot_bytes <= 0) return 0;  // a table without elements launches nothing
  int mb = t->scatter_tail_mb.load(std::memory_order_relaxed);
  if (mb < 0) mb = g_scatter_tail_mb.load(std::memory_order_relaxed);
  const int64_t tail = (int64_t(mb) << 20) / slot_bytes;
  return tail >= t->n_slots ? 0 : int(t->n_slots - tail);
}

void table_free(yafsdp_table* t) {
  if (t == nullptr) return;
  if (t->d_offsets) (void)hipFree(t->d_offsets);
  if (t->d_tiles) (void)hipFree(t->d_tiles);
  if (t->d_slots) (void)hipFree(t->d_slots);
  for (int i = 0; i < t->ring.kRing; i++) {
    if (t->ring.ev[i]) (void)hipEventDestroy(t->ring.ev[i]);
    if (t->ring.h_stage[i]) (void)hipHostFree(t->ring.h_stage[i]);
    if (t->ring.d_stage[i]) (void)hipFree(t->ring.d_stage[i]);
  }
  delete t;
}

// Validate the per-call host arrays.
int check_dyn(const yafsdp_table* t, const void* const* ptrs, const uint8_t* mode, int elem_size) {
  for (int p = 0; p < t->n_tensors; p++) {
    const uint8_t m = mode ? mode[p] : uint8_t(MODE_COPY);
    if (m > MODE_ADD) return YAFSDP_ERR_INVALID_ARGUMENT;
    const bool live = m != MODE_SKIP && t->offsets[p + 1] > t->offsets[p];
    if (live) {
      if (ptrs[p] == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
      if (!aligned_to(ptrs[p], elem_size)) return YAFSDP_ERR_MISALIGNED;
    }
  }
  return YAFSDP_OK;
}

// Small tables: everything travels in the kernel arguments.
void fill_small(const yafsdp_table* t, const void* const* ptrs, const uint8_t* mode, SmallMeta* m) {
  const int64_t tile_elems = t->tile_elems;
  std::memset(m, 0, sizeof(*m));
  const int n = t->n_tensors;
  m->n_tensors = n;
  m->modes = 0;
  for (int i = 0; i <= kSmallMax; i++) {
    const int64_t o = t->offsets[i <= n ? i : n];
    m->off[i] = o;
    m->tile_start[i] = i <= n ? int32_t((o + tile_elems - 1) / tile_elems) : INT32_MAX;
    m->slot_start[i] = i <= n ? int32_t(t->slot_start[i]) : INT32_MAX;
  }
  for (int p = 0; p < n; p++) {
    m->ptr[p] = ptrs[p];
    m->modes |= uint32_t(mode ? mode[p] : uint8_t(MODE_COPY)) << (2 * p);
  }
}

// Large tables: pointers (8 bytes each) and modes (4 bytes each) reach the kernel through a staging slot.
// Returns 0 or an error code; *slot is the slot used.  Never blocks the host: a slot whose last kernel has not
// finished is not overwritten, and when every slot is in that state the call fails with YAFSDP_ERR_BUSY.
int stage_large(yafsdp_table* t, const void* const* ptrs, const uint8_t* mode, LargeMeta* m, int* slot,
                hipStream_t stream) {
  const int n = t->n_tensors;
  char* cur = t->scratch.data();
  std::memcpy(cur, ptrs, size_t(n) * sizeof(void*));
  uint32_t* cm = reinterpret_cast<uint32_t*>(cur + size_t(n) * sizeof(void*));
  for (int p = 0; p < n; p++) cm[p] = mode ? mode[p] : uint32_t(MODE_COPY);
  const size_t used = size_t(n) * (sizeof(void*) + sizeof(uint32_t));
  HipRuntime rt;
  int s = -1;
  const int rc = t->ring.acquire(rt, cur, used, stream, YAFSDP_ERR_BUSY, &s);
  if (rc != 0) return rc;
  m->offsets = t->d_offsets;
  m->tiles = t->d_tiles;
  m->slots = t->d_slots;
  m->ptrs = reinterpret_cast<const void* const*>(t->ring.d_stage[s]);
  m->modes_ = reinterpret_cast<const uint32_t*>(t->ring.d_stage[s] + size_t(n) * sizeof(void*));
  m->n_tensors = n;
  *slot = s;
  return YAFSDP_OK;
}

int finish_large(yafsdp_table* t, int slot, hipStream_t stream) {
  HipRuntime rt;
  return t->ring.finish(rt, slot, stream);
}

// The launch after stage_large failed: the slot's content is no longer offered for reuse, and the slot stays
// ordered behind whatever stage_large enqueued (the event is recorded all the same).  Returns `launch_error`.
int abandon_large(yafsdp_table* t, int slot, hipStream_t stream, hipError_t launch_error) {
  HipRuntime rt;
  return t->ring.abandon(rt, slot, stream, int(launch_error));
}

}  // namespace

extern "C" {

int yafsdp_version(void) { return 1007; }

const char* yafsdp_error_string(int code) {
  switch (code) {
    case YAFSDP_OK: return "success";
    case YAFSDP_ERR_INVALID_ARGUMENT: return "yafsdp: invalid argument";
    case YAFSDP_ERR_UNSUPPORTED_DTYPE: return "yafsdp: unsupported dtype (expected 0=f32, 1=bf16, 2=f16)";
    case YAFSDP_ERR_MISALIGNED: return "yafsdp: pointer not aligned (element size; 16 bytes for flat table buffers)";
    case YAFSDP_ERR_WRONG_DEVICE: return "yafsdp: table belongs to another device than the current one";
    case YAFSDP_ERR_OUT_OF_MEMORY: return "yafsdp: host allocation failed";
    case YAFSDP_ERR_UNSUPPORTED:
      return "yafsdp: this fused entry point does not serve the dtype combination (a reduce buffer that has neither "
             "the gradients' dtype nor binary32): use the two separate entry points";
    case YAFSDP_ERR_BUSY:
      return "yafsdp: every staging slot of this table is still in use by a queued call (more than 8 different "
             "tensor sets in flight): synchronise the stream, or bind tensor sets that persist";
    case YAFSDP_ERR_TOO_LARGE:
      return "yafsdp: more elements than the entry point's fixed scratch is specified for (yafsdp_flat_sumsq_static: 2^31)";
    default: break;
  }
  if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
  return "yafsdp: unknown error code";
}

int yafsdp_binding_create(yafsdp_table* table, const void* const* tensor_ptrs, const uint8_t* mode,
                          int tensor_dtype, yafsdp_binding** out) {
  if (out == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  *out = nullptr;
  if (table == nullptr || (table->n_tensors > 0 && tensor_ptrs == nullptr)) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (!valid_dtype(tensor_dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return int(e);
  if (device != table->device) return YAFSDP_ERR_WRONG_DEVICE;
  const int rc = check_dyn(table, tensor_ptrs, mode, item_size(tensor_dtype));
  if (rc != YAFSDP_OK) return rc;
  yafsdp_binding* b = new (std::nothrow) yafsdp_binding();
  if (b == nullptr) return YAFSDP_ERR_OUT_OF_MEMORY;
  b->table = table;
  b->tensor_dtype = tensor_dtype;
  const int n = table->n_tensors;
  if (n <= kSmallRoute) {
    fill_small(table, tensor_ptrs, mode, &b->small);
  } else {
    const size_t bytes = size_t(n) * (sizeof(void*) + sizeof(uint32_t));
    std::vector<char> host;
    try {
      host.resize(bytes);
    } catch (const std::bad_alloc&) {
      delete b;
      return YAFSDP_ERR_OUT_OF_MEMORY;
    }
    std::memcpy(host.data(), tensor_ptrs, size_t(n) * sizeof(void*));
    uint32_t* hm = reinterpret_cast<uint32_t*>(host.data() + size_t(n) * sizeof(void*));
    for (int p = 0; p < n; p++) hm[p] = mode ? mode[p] : uint32_t(MODE_COPY);
    if ((e = hipMalloc(reinterpret_cast<void**>(&b->d_arrays), bytes)) != hipSuccess ||
        (e = hipMemcpy(b->d_arrays, host.data(), bytes, hipMemcpyHostToDevice)) != hipSuccess) {
      if (b->d_arrays) (void)hipFree(b->d_arrays);
      delete b;
      return int(e);
    }
    b->large.offsets = table->d_offsets;
    b->large.tiles = table->d_tiles;
    b->large.slots = table->d_slots;
    b->large.ptrs = reinterpret_cast<const void* const*>(b->d_arrays);
    b->large.modes_ = reinterpret_cast<const uint32_t*>(b->d_arrays + size_t(n) * sizeof(void*));
    b->large.n_tensors = n;
  }
  *out = b;
  return YAFSDP_OK;
}

int yafsdp_binding_destroy(yafsdp_binding* binding) {
  if (binding == nullptr) return YAFSDP_OK;
  if (binding->d_arrays) (void)hipFree(binding->d_arrays);
  delete binding;
  return YAFSDP_OK;
}

int yafsdp_gather_in_bound(yafsdp_binding* binding, void* flat, int flat_dtype, double pre_factor, int zero_pad,
                           void* stream) {
  if (binding == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  const yafsdp_table* table = binding->table;
  if (!valid_dtype(flat_dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (table->padded == 0) return YAFSDP_OK;
  if (flat == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (!aligned_to(flat, 16)) return YAFSDP_ERR_MISALIGNED;
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return int(e);
  if (device != table->device) return YAFSDP_ERR_WRONG_DEVICE;
  int scale;
  float k;
  scale_plan(pre_factor, &scale, &k);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int grid = grid_for(table->n_tiles, g_table_blocks_per_cu.load(std::memory_order_relaxed), device);
  if (table->n_tensors <= kSmallRoute)
    return int(launch_gather<SmallMeta>(table->block, binding->tensor_dtype, flat_dtype, scale, binding->small, flat,
                                        table->padded, table->n_tiles, k, zero_pad ? 1 : 0, gather_wt_from(table, flat_dtype),
                                        grid, s));
  return int(launch_gather<LargeMeta>(table->block, binding->tensor_dtype, flat_dtype, scale, binding->large, flat,
                                      table->padded, table->n_tiles, k, zero_pad ? 1 : 0,
                                      gather_wt_from(table, flat_dtype), grid, s));
}

int yafsdp_scatter_out_bound(yafsdp_binding* binding, const void* flat, int flat_dtype, void* stream) {
  if (binding == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  const yafsdp_table* table = binding->table;
  if (!valid_dtype(flat_dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (table->total == 0) return YAFSDP_OK;
  if (flat == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (!aligned_to(flat, 16)) return YAFSDP_ERR_MISALIGNED;
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return int(e);
  if (device != table->device) return YAFSDP_ERR_WRONG_DEVICE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int grid = grid_for(table->n_slots, g_table_blocks_per_cu.load(std::memory_order_relaxed), device);
  if (table->n_tensors <= kSmallRoute)
    return int(launch_scatter<SmallMeta>(table->scatter_shape, flat_dtype, binding->tensor_dtype, binding->small, flat,
                                         table->total, table->n_slots, scatter_wt_from(table, binding->tensor_dtype),
                                         grid, s));
  return int(launch_scatter<LargeMeta>(table->scatter_shape, flat_dtype, binding->tensor_dtype, binding->large, flat,
                                       table->total, table->n_slots, scatter_wt_from(table, binding->tensor_dtype),
                                       grid, s));
}

int yafsdp_time_next_launch(void* start_event, void* stop_event) {
  if ((start_event == nullptr) != (stop_event == nullptr)) return YAFSDP_ERR_INVALID_ARGUMENT;
  tl_timed_launch.start = static_cast<hipEvent_t>(start_event);
  tl_timed_launch.stop = static_cast<hipEvent_t>(stop_event);
  return YAFSDP_OK;
}

int yafsdp_complete_next_launch(void* event) {
  tl_timed_launch.start = nullptr;
  tl_timed_launch.stop = static_cast<hipEvent_t>(event);
  return YAFSDP_OK;
}

int yafsdp_complete_next_launch_pending(void) { return tl_timed_launch.stop != nullptr ? 1 : 0; }

int yafsdp_trace_next_flat_launch(uint64_t* trace, int64_t capacity, int64_t* n_workgroups) {
  if (trace == nullptr) {  // disarm
    tl_timed_launch.trace = nullptr;
    tl_timed_launch.trace_capacity = 0;
    tl_timed_launch.trace_workgroups = nullptr;
    return YAFSDP_OK;
  }
  if (capacity < 1 || !aligned_to(trace, 8)) return YAFSDP_ERR_INVALID_ARGUMENT;
  tl_timed_launch.trace = reinterpret_cast<unsigned long long*>(trace);
  tl_timed_launch.trace_capacity = capacity;
  tl_timed_launch.trace_workgroups = n_workgroups;
  if (n_workgroups != nullptr) *n_workgroups = 0;
  return YAFSDP_OK;
}

int yafsdp_set_option(int option, int value) {
  if (option == YAFSDP_OPT_TABLE_LARGE_LOG2) {
    if (value < 0 || value > 62) return YAFSDP_ERR_INVALID_ARGUMENT;
    g_table_large_log2.store(value);
    return YAFSDP_OK;
  }
  if (option == YAFSDP_OPT_GATHER_TAIL_MB || option == YAFSDP_OPT_SCATTER_TAIL_MB ||
      option == YAFSDP_OPT_FLAT_TAIL_MB || option == YAFSDP_OPT_POST_REDUCE_TAIL_MB) {
    if (value < 0 || value > (1 << 20)) return YAFSDP_ERR_INVALID_ARGUMENT;
    (option == YAFSDP_OPT_GATHER_TAIL_MB ? g_gather_tail_mb
     : option == YAFSDP_OPT_SCATTER_TAIL_MB ? g_scatter_tail_mb
     : option == YAFSDP_OPT_FLAT_TAIL_MB ? g_flat_tail_mb : g_post_reduce_tail_mb).store(value);
    return YAFSDP_OK;
  }
  if (option == YAFSDP_OPT_SCATTER_TILE) {
    if (value < 0 || value > 2) return YAFSDP_ERR_INVALID_ARGUMENT;
    g_scatter_tile_mode.store(value);
    return YAFSDP_OK;
  }
  if (value < 1 || value > 4096) return YAFSDP_ERR_INVALID_ARGUMENT;
  switch (option) {
    case YAFSDP_OPT_FLAT_BLOCKS_PER_CU: g_flat_blocks_per_cu.store(value); return YAFSDP_OK;
    case YAFSDP_OPT_TABLE_BLOCKS_PER_CU: g_table_blocks_per_cu.store(value); return YAFSDP_OK;
  }
  return YAFSDP_ERR_INVALID_ARGUMENT;
}

int yafsdp_table_set_option(yafsdp_table* table, int option, int value) {
  if (table == nullptr || value < -1 || value > (1 << 20)) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (option == YAFSDP_OPT_GATHER_TAIL_MB) table->gather_tail_mb.store(value);
  else if (option == YAFSDP_OPT_SCATTER_TAIL_MB) table->scatter_tail_mb.store(value);
  else return YAFSDP_ERR_INVALID_ARGUMENT;
  return YAFSDP_OK;
}

int yafsdp_table_get_option(const yafsdp_table* table, int option, int* value) {
  if (table == nullptr || value == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (option == YAFSDP_OPT_GATHER_TAIL_MB) *value = table->gather_tail_mb.load();
  else if (option == YAFSDP_OPT_SCATTER_TAIL_MB) *value = table->scatter_tail_mb.load();
  else return YAFSDP_ERR_INVALID_ARGUMENT;
  return YAFSDP_OK;
}

int yafsdp_get_option(int option, int* value) {
  if (value == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  switch (option) {
    case YAFSDP_OPT_FLAT_BLOCKS_PER_CU: *value = g_flat_blocks_per_cu.load(); return YAFSDP_OK;
    case YAFSDP_OPT_TABLE_BLOCKS_PER_CU: *value = g_table_blocks_per_cu.load(); return YAFSDP_OK;
    case YAFSDP_OPT_TABLE_LARGE_LOG2: *value = g_table_large_log2.load(); return YAFSDP_OK;
    case YAFSDP_OPT_SCATTER_TILE: *value = g_scatter_tile_mode.load(); return YAFSDP_OK;
    case YAFSDP_OPT_GATHER_TAIL_MB: *value = g_gather_tail_mb.load(); return YAFSDP_OK;
    case YAFSDP_OPT_SCATTER_TAIL_MB: *value = g_scatter_tail_mb.load(); return YAFSDP_OK;
    case YAFSDP_OPT_FLAT_TAIL_MB: *value = g_flat_tail_mb.load(); return YAFSDP_OK;
    case YAFSDP_OPT_POST_REDUCE_TAIL_MB: *value = g_post_reduce_tail_mb.load(); return YAFSDP_OK;
  }
  return YAFSDP_ERR_INVALID_ARGUMENT;
}

namespace {
// grid of an optimizer-side pass over `units` 16-byte (fill) or quad units
int opt_grid(int64_t units, int block, int unroll, int* device_out) {
  const int64_t tile = int64_t(block) * unroll;
  const int64_t n_tiles = (units + tile - 1) / tile;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) device = 0;
  if (device_out) *device_out = device;
  return grid_for(n_tiles, g_flat_blocks_per_cu.load(std::memory_order_relaxed), device);
}

// leading elements up to the next 16-byte boundary (at most n)
int head_elems(const void* p, int elem_size, int64_t n) {
  int64_t head = ((16 - (reinterpret_cast<uintptr_t>(p) & 15)) & 15) / elem_size;
  return int(head > n ? n : head);
}

uint32_t fill_pattern(int dtype, double value) {
  const float f = static_cast<float>(value);
  uint32_t bits;
  std::memcpy(&bits, &f, 4);
  if (dtype == DT_F32) return bits;
  uint16_t h;
  if (dtype == DT_BF16) {
    if (std::isnan(f)) h = 0x7FC0;
    else h = uint16_t((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);  // round to nearest even
  } else {
    const _Float16 x = static_cast<_Float16>(f);
    std::memcpy(&h, &x, 2);
  }
  return uint32_t(h) | (uint32_t(h) << 16);
}
}  // namespace

int yafsdp_flat_copy_fanout(void* const* dsts, int n_dst, int dst_dtype, const void* src, int src_dtype, int64_t n,
                            void* stream) {
  if (!valid_dtype(dst_dtype) || !valid_dtype(src_dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (n < 0 || n_dst < 1 || n_dst > kFanMax || dsts == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (n == 0) return YAFSDP_OK;
  if (src == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (!aligned_to(src, 16)) return YAFSDP_ERR_MISALIGNED;
  FanPtrs ptrs;
  std::memset(&ptrs, 0, sizeof(ptrs));
  ptrs.n = n_dst;
  for (int k = 0; k < n_dst; k++) {
    if (dsts[k] == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
    if (!aligned_to(dsts[k], 16)) return YAFSDP_ERR_MISALIGNED;
    ptrs.p[k] = dsts[k];
  }
  const int grid = opt_grid(n >> 3, kFanOutBlock, kFanOutUnroll, nullptr);
  return int(launch_fanout(src_dtype, dst_dtype, ptrs, src, n, grid, static_cast<hipStream_t>(stream)));
}

namespace {
int fanin_launch(void* shard, int shard_dtype, const void* const* chunks, int n_src, int chunk_dtype, int64_t n,
                 int scale, float k, int accumulate, void* stream) {
  if (n < 0 || n_src < 1 || n_src > kFanMax || chunks == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (n == 0) return YAFSDP_OK;
  if (shard == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (!aligned_to(shard, 16)) return YAFSDP_ERR_MISALIGNED;
  FanPtrs ptrs;
  std::memset(&ptrs, 0, sizeof(ptrs));
  ptrs.n = n_src;
  for (int c = 0; c < n_src; c++) {
    if (chunks[c] == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
    if (!aligned_to(chunks[c], 16)) return YAFSDP_ERR_MISALIGNED;
    ptrs.p[c] = const_cast<void*>(chunks[c]);
  }
  const int grid = opt_grid(n >> 2, kFanInBlock, kFanInUnroll, nullptr);
  return int(launch_fanin(chunk_dtype, shard_dtype, scale, accumulate != 0, shard, ptrs, n, k, grid,
                          static_cast<hipStream_t>(stream)));
}
}  // namespace

int yafsdp_post_reduce_fanin(void* shard, int shard_dtype, const void* const* chunks, int n_src, int chunk_dtype,
                             int64_t n, double post_factor, int accumulate, void* stream) {
  if (!valid_dtype(shard_dtype) || !valid_dtype(chunk_dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  int scale;
  float k;
  scale_plan(post_factor, &scale, &k);
  return fanin_launch(shard, shard_dtype, chunks, n_src, chunk_dtype, n, scale, k, accumulate, stream);
}

int yafsdp_post_reduce_fanin_premul(void* shard, int shard_dtype, const void* const* chunks, int n_src,
                                    int chunk_dtype, int64_t n, double scalar, int accumulate, void* stream) {
  if (!valid_dtype(shard_dtype) || !valid_dtype(chunk_dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  int scale;
  float k;
  if (!premul_plan(scalar, chunk_dtype, &scale, &k)) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (scale == SCALE_MUL) scale = SCALE_PREMUL;  // a scalar that rounds to 1 leaves the plain sum
  return fanin_launch(shard, shard_dtype, chunks, n_src, chunk_dtype, n, scale, k, accumulate, stream);
}

int yafsdp_flat_fill(void* dst, int dtype, int64_t n, double value, void* stream) {
  if (!valid_dtype(dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (n < 0 || (n > 0 && dst == nullptr)) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (n == 0) return YAFSDP_OK;
  if (!aligned_to(dst, item_size(dtype))) return YAFSDP_ERR_MISALIGNED;
  const int head = head_elems(dst, item_size(dtype), n);
  const int grid = opt_grid((n - head) / (16 / item_size(dtype)), kFillBlock, kFillUnroll, nullptr);
  return int(launch_fill(dtype, dst, n, head, fill_pattern(dtype, value), grid, static_cast<hipStream_t>(stream)));
}

size_t yafsdp_sumsq_workspace_bytes(void) { return size_t(kSumsqMaxPartials) * sizeof(double); }

int yafsdp_sumsq_partials(const void* src, int dtype, int64_t n, double* partials, int64_t capacity,
                          int64_t* n_written, void* stream) {
  if (!valid_dtype(dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (n < 0 || partials == nullptr || n_written == nullptr || capacity < 1 || (n > 0 && src == nullptr))
    return YAFSDP_ERR_INVALID_ARGUMENT;
  if (!aligned_to(src, item_size(dtype)) || !aligned_to(partials, 8)) return YAFSDP_ERR_MISALIGNED;
  const int head = head_elems(src, item_size(dtype), n);
  int64_t grid = opt_grid((n - head) >> 2, kSumsqBlock, kSumsqUnroll, nullptr);
  if (grid > kSumsqMaxPartials) grid = kSumsqMaxPartials;
  if (grid > capacity) grid = capacity;  // fewer workgroups, each striding over more tiles
  *n_written = grid;
  return int(launch_sumsq_partials(dtype, src, n, head, partials, int(grid), static_cast<hipStream_t>(stream)));
}

int yafsdp_flat_sumsq(const void* src, int dtype, int64_t n, double* sumsq, int accumulate, void* workspace,
                      size_t workspace_bytes, void* stream) {
  if (sumsq == nullptr || workspace == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (workspace_bytes < yafsdp_sumsq_workspace_bytes()) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (!aligned_to(sumsq, 8)) return YAFSDP_ERR_MISALIGNED;
  int64_t count = 0;
  const int rc = yafsdp_sumsq_partials(src, dtype, n, static_cast<double*>(workspace), kSumsqMaxPartials, &count,
                                       stream);
  if (rc != YAFSDP_OK) return rc;
  return int(launch_sumsq_finish(static_cast<double*>(workspace), count, sumsq, accumulate ? 1 : 0, 0.0f, nullptr,
                                 static_cast<hipStream_t>(stream)));
}

int64_t yafsdp_flat_sumsq_static_max_numel(void) { return int64_t(1) << 31; }

int yafsdp_flat_sumsq_static(const void* src, int dtype, int64_t n, double* sumsq, int accumulate, void* stream) {
  if (!valid_dtype(dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (n < 0 || (n > 0 && (src == nullptr || sumsq == nullptr))) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (n > yafsdp_flat_sumsq_static_max_numel()) return YAFSDP_ERR_TOO_LARGE;
  if (n > 0 && (!aligned_to(src, item_size(dtype)) || !aligned_to(sumsq, 8))) return YAFSDP_ERR_MISALIGNED;
  double* scratch = nullptr;
  const int rc0 = sumsq_static_scratch(&scratch);  // set-up on the first call on this device
  if (rc0 != YAFSDP_OK) return rc0;
  if (n == 0) {
    // nothing to add: like yafsdp_flat_sumsq, *sumsq becomes 0 unless it accumulates (a call with a null `sumsq`
    // only performs the set-up)
    if (sumsq == nullptr) return YAFSDP_OK;
    if (!aligned_to(sumsq, 8)) return YAFSDP_ERR_MISALIGNED;
    return int(launch_sumsq_finish(scratch, 0, sumsq, accumulate ? 1 : 0, 0.0f, nullptr, static_cast<hipStream_t>(stream)));
  }
  // every partial sum the finishing launch reads is written by the launch before it: nothing has to start at zero
  int64_t count = 0;
  const int rc = yafsdp_sumsq_partials(src, dtype, n, scratch, kSumsqMaxPartials, &count, stream);
  if (rc != YAFSDP_OK) return rc;
  return int(launch_sumsq_finish(scratch, count, sumsq, accumulate ? 1 : 0, 0.0f, nullptr,
                                 static_cast<hipStream_t>(stream)));
}

int yafsdp_clip_coef_from_partials(const double* partials, int64_t n_partials, double max_norm, double* sumsq,
                                   float* norm_and_coef, void* stream) {
  if (n_partials < 0 || norm_and_coef == nullptr || (n_partials > 0 && partials == nullptr))
    return YAFSDP_ERR_INVALID_ARGUMENT;
  if (!aligned_to(partials, 8) || !aligned_to(norm_and_coef, 4) || (sumsq != nullptr && !aligned_to(sumsq, 8)))
    return YAFSDP_ERR_MISALIGNED;
  return int(launch_sumsq_finish(partials, n_partials, sumsq, 0, static_cast<float>(max_norm), norm_and_coef,
                                 static_cast<hipStream_t>(stream)));
}

int yafsdp_sumsq_reduce_partials(const double* partials, int64_t n_partials, double* out, int64_t capacity,
                                 int64_t* n_written, void* stream) {
  if (n_partials < 0 || n_written == nullptr || (n_partials > 0 && (partials == nullptr || out == nullptr)))
    return YAFSDP_ERR_INVALID_ARGUMENT;
  *n_written = 0;
  if (n_partials == 0) return YAFSDP_OK;
  if (!aligned_to(partials, 8) || !aligned_to(out, 8)) return YAFSDP_ERR_MISALIGNED;
  const int64_t grid = (n_partials + 4095) / 4096;
  if (grid > capacity || grid > int64_t(INT32_MAX)) return YAFSDP_ERR_INVALID_ARGUMENT;
  const hipError_t e = launch_sumsq_reduce(partials, n_partials, out, int(grid), static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return int(e);
  *n_written = grid;
  return YAFSDP_OK;
}

int yafsdp_clip_coef(const double* sumsq, double max_norm, float* norm_and_coef, void* stream) {
  if (sumsq == nullptr || norm_and_coef == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (!aligned_to(sumsq, 8) || !aligned_to(norm_and_coef, 4)) return YAFSDP_ERR_MISALIGNED;
  return int(launch_clip_coef(sumsq, static_cast<float>(max_norm), norm_and_coef, static_cast<hipStream_t>(stream)));
}

int yafsdp_flat_scale(void* buf, int dtype, int64_t n, const float* coef, void* stream) {
  if (!valid_dtype(dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (n < 0 || coef == nullptr || (n > 0 && buf == nullptr)) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (n == 0) return YAFSDP_OK;
  if (!aligned_to(buf, item_size(dtype)) || !aligned_to(coef, 4)) return YAFSDP_ERR_MISALIGNED;
  const int head = head_elems(buf, item_size(dtype), n);
  const int grid = opt_grid((n - head) >> 2, kScaleBlock, kScaleUnroll, nullptr);
  return int(launch_scale(dtype, buf, n, head, coef, grid, static_cast<hipStream_t>(stream)));
}

int yafsdp_adamw_step(float* param, float* grad, float* exp_avg, float* exp_avg_sq, void* out16, int out16_dtype,
                      int64_t n, double lr, double beta1, double beta2, double eps, double weight_decay,
                      int64_t step, const float* grad_scale, int flags, void* stream) {
  if (n < 0 || step < 1) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (out16 != nullptr && out16_dtype != DT_BF16 && out16_dtype != DT_F16) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (n == 0) return YAFSDP_OK;
  if (param == nullptr || grad == nullptr || exp_avg == nullptr || exp_avg_sq == nullptr)
    return YAFSDP_ERR_INVALID_ARGUMENT;
  // the four binary32 arrays must share one residue modulo 16 bytes (fragments at
  // one offset of identically laid out shards do), and out16 the matching one
  // modulo 8, so that peeling `head` elements aligns all of them at once
  const uintptr_t res = reinterpret_cast<uintptr_t>(param) & 15;
  if ((res & 3) != 0 || (reinterpret_cast<uintptr_t>(grad) & 15) != res ||
      (reinterpret_cast<uintptr_t>(exp_avg) & 15) != res || (reinterpret_cast<uintptr_t>(exp_avg_sq) & 15) != res ||
      (out16 != nullptr && (reinterpret_cast<uintptr_t>(out16) & 7) != (res >> 1)) ||
      (grad_scale != nullptr && !aligned_to(grad_scale, 4)))
    return YAFSDP_ERR_MISALIGNED;
  const int head = head_elems(param, 4, n);
  // scalars exactly as torch.optim computes them: Python floats (binary64),
  // rounded to binary32 where they enter a tensor op
  AdamScalars s;
  std::memset(&s, 0, sizeof(s));
  s.flags = 0;
  if (weight_decay != 0.0) {
    if (flags & YAFSDP_ADAM_DECOUPLED_DECAY) {
      s.flags |= ADAM_DECOUPLED;
      s.decay = static_cast<float>(1.0 - lr * weight_decay);
    } else {
      s.flags |= ADAM_L2;
      s.l2 = static_cast<float>(weight_decay);
    }
  }
  s.w = static_cast<float>(1.0 - beta1);
  s.w_m1 = s.w - 1.0f;
  if (std::fabs(s.w) < 0.5f) s.flags |= ADAM_W_SMALL;
  s.beta2 = static_cast<float>(beta2);
  s.one_m_beta2 = static_cast<float>(1.0 - beta2);
  const double bc1 = 1.0 - std::pow(beta1, double(step));
  const double bc2 = 1.0 - std::pow(beta2, double(step));
  s.bc2_sqrt = static_cast<float>(std::pow(bc2, 0.5));
  s.eps = static_cast<float>(eps);
  s.neg_step = static_cast<float>(-(lr / bc1));
  if (flags & YAFSDP_ADAM_ZERO_GRAD) s.flags |= ADAM_ZERO_GRAD;
  const int grid = opt_grid((n - head) >> 2, kAdamBlock, kAdamUnroll, nullptr);
  return int(launch_adamw(out16_dtype, param, grad, exp_avg, exp_avg_sq, out16, n, head, s, grad_scale, grid,
                          static_cast<hipStream_t>(stream)));
}

int yafsdp_flat_copy(void* dst, int dst_dtype, const void* src, int src_dtype, int64_t n, void* stream) {
  if (!valid_dtype(dst_dtype) || !valid_dtype(src_dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (n < 0 || (n > 0 && (dst == nullptr || src == nullptr))) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (n > 0 && dst == src && dst_dtype == src_dtype) return YAFSDP_OK;  // aliasing self-copy
  return flat_launch(src_dtype, dst_dtype, SCALE_NONE, false, dst, src, n, 1.0f, static_cast<hipStream_t>(stream));
}

int yafsdp_flat_copy_bytes(void* dst, const void* src, int64_t n_bytes, void* stream) {
  if (n_bytes < 0 || (n_bytes > 0 && (dst == nullptr || src == nullptr))) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (n_bytes == 0 || dst == src) return YAFSDP_OK;
  const uintptr_t d0 = reinterpret_cast<uintptr_t>(dst), s0 = reinterpret_cast<uintptr_t>(src);
  if (((d0 | s0 | uintptr_t(n_bytes)) & 1) == 0)  // pairs of bytes at even addresses: the tuned 2-byte copy
    return flat_launch(DT_BF16, DT_BF16, SCALE_NONE, false, dst, src, n_bytes >> 1, 1.0f,
                       static_cast<hipStream_t>(stream));
  if (d0 < s0 + uintptr_t(n_bytes) && s0 < d0 + uintptr_t(n_bytes)) return YAFSDP_ERR_INVALID_ARGUMENT;  // overlap
  // up to the destination's next 128-byte line, so that no two workgroups write into one cache line (tiles are a
  // whole number of lines from there on): with 16-byte alignment only, every tile boundary split a line, and the
  // counters showed 3 % more bytes written than the copy holds
  int64_t head = int64_t((128 - (d0 & 127)) & 127);
  if (head > n_bytes) head = n_bytes;
  const int64_t n_tiles = (((n_bytes - head) >> 4) + kFlatBlock - 1) / kFlatBlock;
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return int(e);
  const int grid = grid_for(n_tiles, g_flat_blocks_per_cu.load(std::memory_order_relaxed), device);
  // (a tile is one 16-byte vector per lane)
  const int64_t tail_tiles = (int64_t(g_flat_tail_mb.load(std::memory_order_relaxed)) << 20) / (int64_t(kFlatBlock) * 16);
  const int64_t wt_from = tail_tiles >= n_tiles ? 0 : n_tiles - tail_tiles;
  return int(launch_bytes(dst, src, n_bytes, int(head), wt_from > INT32_MAX ? INT32_MAX : int(wt_from), grid,
                          static_cast<hipStream_t>(stream)));
}

int yafsdp_flat_div(void* buf, int dtype, int64_t n, double factor, void* stream) {
  if (!valid_dtype(dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (n < 0 || (n > 0 && buf == nullptr)) return YAFSDP_ERR_INVALID_ARGUMENT;
  int scale;
  float k;
  scale_plan(factor, &scale, &k);
  if (scale == SCALE_NONE) return YAFSDP_OK;
  return flat_launch(dtype, dtype, scale, false, buf, buf, n, k, static_cast<hipStream_t>(stream));
}

int yafsdp_flat_premul(void* buf, int dtype, int64_t n, double scalar, void* stream) {
  if (!valid_dtype(dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (n < 0 || (n > 0 && buf == nullptr)) return YAFSDP_ERR_INVALID_ARGUMENT;
  int scale;
  float k;
  if (!premul_plan(scalar, dtype, &scale, &k)) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (scale == SCALE_NONE || n == 0) return YAFSDP_OK;
  return flat_launch(dtype, dtype, scale, false, buf, buf, n, k, static_cast<hipStream_t>(stream));
}

int yafsdp_post_reduce_premul(void* shard, int shard_dtype, const void* chunk, int chunk_dtype, int64_t n,
                              double scalar, int accumulate, void* stream) {
  if (!valid_dtype(shard_dtype) || !valid_dtype(chunk_dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (n < 0 || (n > 0 && (shard == nullptr || chunk == nullptr))) return YAFSDP_ERR_INVALID_ARGUMENT;
  int scale;
  float k;
  if (!premul_plan(scalar, chunk_dtype, &scale, &k)) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (n == 0) return YAFSDP_OK;
  if (shard == chunk) {  // the collective wrote into the shard itself: only its scaling is left
    if (shard_dtype != chunk_dtype || accumulate) return YAFSDP_ERR_INVALID_ARGUMENT;
    if (scale == SCALE_NONE) return YAFSDP_OK;
  }
  return flat_launch(chunk_dtype, shard_dtype, scale, accumulate != 0, shard, chunk, n, k,
                     static_cast<hipStream_t>(stream), g_post_reduce_tail_mb);
}

int yafsdp_flat_div_copy(void* dst, int dst_dtype, const void* src, int src_dtype, int64_t n, double divisor,
                         void* stream) {
  if (!valid_dtype(dst_dtype) || !valid_dtype(src_dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (n < 0 || (n > 0 && (dst == nullptr || src == nullptr))) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (n == 0) return YAFSDP_OK;  // empty ranges may come with null or equal pointers
  if (dst == src && dst_dtype != src_dtype) return YAFSDP_ERR_INVALID_ARGUMENT;
  int scale;
  float k;
  if (!scale_plan_any(divisor, &scale, &k)) return YAFSDP_ERR_INVALID_ARGUMENT;
  return flat_launch(src_dtype, dst_dtype, scale, false, dst, src, n, k, static_cast<hipStream_t>(stream));
}

int yafsdp_post_reduce(void* shard, int shard_dtype, const void* chunk, int chunk_dtype, int64_t n, double post_factor,
                       int accumulate, void* stream) {
  if (!valid_dtype(shard_dtype) || !valid_dtype(chunk_dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (n < 0 || (n > 0 && (shard == nullptr || chunk == nullptr))) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (n == 0) return YAFSDP_OK;  // empty ranges may come with null or equal pointers
  int scale;
  float k;
  scale_plan(post_factor, &scale, &k);
  if (shard == chunk) {
    // the reduction already wrote into the shard: only the divide is left, and
    // accumulating a buffer into itself is not an operation of this path
    if (shard_dtype != chunk_dtype || accumulate) return YAFSDP_ERR_INVALID_ARGUMENT;
    if (scale == SCALE_NONE) return YAFSDP_OK;
  }
  return flat_launch(chunk_dtype, shard_dtype, scale, accumulate != 0, shard, chunk, n, k,
                     static_cast<hipStream_t>(stream), g_post_reduce_tail_mb);
}

int64_t yafsdp_post_reduce_sumsq_count(int64_t n) {
  if (n <= 0) return 0;
  const int64_t tile = int64_t(kPostSumsqBlock) * kPostSumsqUnroll;
  const int64_t n_tiles = ((n >> 3) + tile - 1) / tile;  // the peeled head can only lower the unit count
  return n_tiles < 1 ? 1 : n_tiles;
}

int yafsdp_post_reduce_sumsq(void* shard, int shard_dtype, const void* chunk, int chunk_dtype, int64_t n,
                             double post_factor, int accumulate, double* partials, int64_t capacity,
                             int64_t* n_written, void* stream) {
  if (!valid_dtype(shard_dtype) || !valid_dtype(chunk_dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (n < 0 || n_written == nullptr || (n > 0 && (shard == nullptr || chunk == nullptr || partials == nullptr)))
    return YAFSDP_ERR_INVALID_ARGUMENT;
  *n_written = 0;
  if (n == 0) return YAFSDP_OK;
  if (!aligned_to(shard, item_size(shard_dtype)) || !aligned_to(chunk, item_size(chunk_dtype)) ||
      !aligned_to(partials, 8))
    return YAFSDP_ERR_MISALIGNED;
  {
    const uintptr_t d0 = reinterpret_cast<uintptr_t>(shard), s0 = reinterpret_cast<uintptr_t>(chunk);
    const uintptr_t d1 = d0 + uintptr_t(n) * item_size(shard_dtype), s1 = s0 + uintptr_t(n) * item_size(chunk_dtype);
    if (d0 < s1 && s0 < d1) return YAFSDP_ERR_INVALID_ARGUMENT;
  }
  const int head = head_elems(shard, item_size(shard_dtype), n);
  const int64_t tile = int64_t(kPostSumsqBlock) * kPostSumsqUnroll;
  int64_t n_tiles = (((n - head) >> 3) + tile - 1) / tile;
  if (n_tiles < 1) n_tiles = 1;  // workgroup 0 handles head and tail
  if (n_tiles > capacity || n_tiles > int64_t(INT32_MAX)) return YAFSDP_ERR_INVALID_ARGUMENT;
  int scale;
  float k;
  scale_plan(post_factor, &scale, &k);
  const hipError_t e = launch_post_reduce_sumsq(chunk_dtype, shard_dtype, scale, accumulate != 0, shard, chunk, n, head,
                                                k, partials,
                                                flat_wt_from(n_tiles, tile, shard_dtype, g_post_reduce_tail_mb),
                                                int(n_tiles), static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return int(e);
  *n_written = n_tiles;
  return YAFSDP_OK;
}

int yafsdp_post_reduce_fragments(void* shard, int shard_dtype, const void* chunk, int chunk_dtype, int n_fragments,
                                 const int64_t* frag_numels, const uint8_t* frag_mode, double post_factor,
                                 void* stream) {
  if (!valid_dtype(shard_dtype) || !valid_dtype(chunk_dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (n_fragments < 0 || (n_fragments > 0 && (frag_numels == nullptr || frag_mode == nullptr)))
    return YAFSDP_ERR_INVALID_ARGUMENT;
  int64_t total = 0;
  for (int f = 0; f < n_fragments; f++) {
    if (frag_numels[f] < 0 || frag_mode[f] > MODE_ADD) return YAFSDP_ERR_INVALID_ARGUMENT;
    total += frag_numels[f];
  }
  if (total > 0 && (shard == nullptr || chunk == nullptr || shard == chunk)) return YAFSDP_ERR_INVALID_ARGUMENT;
  int scale;
  float k;
  scale_plan(post_factor, &scale, &k);
  // merge neighbouring fragments of equal mode into runs: one launch per run
  int64_t pos = 0;
  int f = 0;
  while (f < n_fragments) {
    const uint8_t m = frag_mode[f];
    int64_t run = 0;
    while (f < n_fragments && (frag_mode[f] == m || frag_numels[f] == 0)) run += frag_numels[f++];
    if (m != MODE_SKIP && run > 0) {
      char* d = static_cast<char*>(shard) + pos * item_size(shard_dtype);
      const char* s = static_cast<const char*>(chunk) + pos * item_size(chunk_dtype);
      int rc = flat_launch(chunk_dtype, shard_dtype, scale, m == MODE_ADD, d, s, run, k,
                           static_cast<hipStream_t>(stream), g_post_reduce_tail_mb);
      if (rc != YAFSDP_OK) return rc;
    }
    pos += run;
  }
  return YAFSDP_OK;
}

int yafsdp_table_create(int n_tensors, const int64_t* numels, int64_t padded_numel, yafsdp_table** out) {
  if (out == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  *out = nullptr;
  if (n_tensors < 0 || (n_tensors > 0 && numels == nullptr)) return YAFSDP_ERR_INVALID_ARGUMENT;
  yafsdp_table* t = new (std::nothrow) yafsdp_table();
  if (t == nullptr) return YAFSDP_ERR_OUT_OF_MEMORY;
  int rc = YAFSDP_OK;
  hipError_t e = hipSuccess;
  std::vector<TileRec> tiles;
  try {
  do {
    t->n_tensors = n_tensors;
    t->offsets.assign(size_t(n_tensors) + 1, 0);
    for (int p = 0; p < n_tensors; p++) {
      if (numels[p] < 0 || numels[p] > (int64_t(1) << 60) - t->offsets[p]) { rc = YAFSDP_ERR_INVALID_ARGUMENT; break; }
      t->offsets[p + 1] = t->offsets[p] + numels[p];
    }
    if (rc != YAFSDP_OK) break;
    t->total = t->offsets[n_tensors];
    t->padded = padded_numel;
    if (padded_numel < t->total || padded_numel > (int64_t(1) << 60)) { rc = YAFSDP_ERR_INVALID_ARGUMENT; break; }
    t->block = table_block_for(padded_numel, g_table_large_log2.load(std::memory_order_relaxed));
    t->tile_elems = gather_tile_elems(t->block);
    {
      bool line_aligned = true;  // every non-empty tensor starts on a multiple of 64 elements (128 bytes of a 2-byte dtype)
      for (int p = 0; p < n_tensors; p++)
        if (numels[p] > 0 && (t->offsets[p] & 63) != 0) line_aligned = false;
      const ScatterShape sh = scatter_shape_for(padded_numel, line_aligned, g_table_large_log2.load(std::memory_order_relaxed),
                                                g_scatter_tile_mode.load(std::memory_order_relaxed));
      t->scatter_shape = sh.block * 16 + sh.unroll;
      t->slot_elems = scatter_tile_elems(sh);
    }
    const int64_t n_tiles = (padded_numel + t->tile_elems - 1) / t->tile_elems;
    if (n_tiles > int64_t(INT32_MAX) - 4096) { rc = YAFSDP_ERR_INVALID_ARGUMENT; break; }
    t->n_tiles = int32_t(n_tiles);
    if ((e = hipGetDevice(&t->device)) != hipSuccess) break;
    if ((e = hipMalloc(reinterpret_cast<void**>(&t->d_offsets), t->offsets.size() * sizeof(int64_t))) != hipSuccess) break;
    if ((e = hipMemcpy(t->d_offsets, t->offsets.data(), t->offsets.size() * sizeof(int64_t), hipMemcpyHostToDevice)) != hipSuccess) break;
    if (n_tensors > kSmallRoute && n_tiles > 0) {
      // per tile: first tensor whose end lies beyond the tile's first element
      tiles.resize(size_t(n_tiles));
      int p = 0;
      for (int64_t tile = 0; tile < n_tiles; tile++) {
        const int64_t t0 = tile * t->tile_elems;
        while (p < n_tensors && t->offsets[p + 1] <= t0) p++;
        TileRec& r = tiles[size_t(tile)];
        r.first = p;
        r.full = (p < n_tensors && t->offsets[p + 1] - t0 >= t->tile_elems) ? 1 : 0;
        r.delta = p < n_tensors ? t0 - t->offsets[p] : 0;
      }
      if ((e = hipMalloc(reinterpret_cast<void**>(&t->d_tiles), tiles.size() * sizeof(TileRec))) != hipSuccess) break;
      if ((e = hipMemcpy(t->d_tiles, tiles.data(), tiles.size() * sizeof(TileRec), hipMemcpyHostToDevice)) != hipSuccess) break;
    }
    // scatter-out tile slots
    t->slot_start.assign(size_t(n_tensors) + 1, 0);
    for (int p = 0; p < n_tensors; p++) {
      const int64_t n = t->offsets[p + 1] - t->offsets[p];
      t->slot_start[p + 1] = t->slot_start[p] + (n > 0 ? (n + t->slot_elems - 1) / t->slot_elems + 1 : 0);
    }
    if (t->slot_start[n_tensors] > int64_t(INT32_MAX) - 4096) { rc = YAFSDP_ERR_INVALID_ARGUMENT; break; }
    t->n_slots = int32_t(t->slot_start[n_tensors]);
    if (n_tensors > kSmallRoute && t->n_slots > 0) {
      tiles.resize(size_t(t->n_slots));
      for (int p = 0; p < n_tensors; p++) {
        for (int64_t k = t->slot_start[p]; k < t->slot_start[p + 1]; k++) {
          TileRec& r = tiles[size_t(k)];
          r.first = p;
          r.full = 0;
          r.delta = k - t->slot_start[p];
        }
      }
      if ((e = hipMalloc(reinterpret_cast<void**>(&t->d_slots), tiles.size() * sizeof(TileRec))) != hipSuccess) break;
      if ((e = hipMemcpy(t->d_slots, tiles.data(), tiles.size() * sizeof(TileRec), hipMemcpyHostToDevice)) != hipSuccess) break;
    }
    if (n_tensors > kSmallRoute) {
      const size_t stage_bytes = (size_t(n_tensors) * (sizeof(void*) + sizeof(uint32_t)) + 15) & ~size_t(15);
      t->ring.stage_bytes = stage_bytes;
      t->scratch.assign(stage_bytes, 0);
      for (int i = 0; i < t->ring.kRing && e == hipSuccess; i++) {
        if ((e = hipHostMalloc(reinterpret_cast<void**>(&t->ring.h_stage[i]), stage_bytes, hipHostMallocDefault)) != hipSuccess) break;
        if ((e = hipMalloc(reinterpret_cast<void**>(&t->ring.d_stage[i]), stage_bytes)) != hipSuccess) break;
        if ((e = hipEventCreateWithFlags(&t->ring.ev[i], hipEventDisableTiming)) != hipSuccess) break;
      }
    }
  } while (false);
  } catch (const std::bad_alloc&) {  // host-side vectors: no exception may cross the C ABI
    rc = YAFSDP_ERR_OUT_OF_MEMORY;
  }
  if (rc == YAFSDP_OK && e != hipSuccess) rc = int(e);
  if (rc != YAFSDP_OK) {
    table_free(t);
    return rc;
  }
  *out = t;
  return YAFSDP_OK;
}

int yafsdp_table_destroy(yafsdp_table* table) {
  if (table == nullptr) return YAFSDP_OK;
  int rc = YAFSDP_OK;
  for (int i = 0; i < table->ring.kRing; i++) {
    if (table->ring.ev_pending[i]) {
      hipError_t e = hipEventSynchronize(table->ring.ev[i]);
      if (e != hipSuccess) rc = int(e);
    }
  }
  table_free(table);
  return rc;
}

int yafsdp_table_info(const yafsdp_table* table, int* n_tensors, int64_t* total_numel, int64_t* padded_numel) {
  if (table == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (n_tensors) *n_tensors = table->n_tensors;
  if (total_numel) *total_numel = table->total;
  if (padded_numel) *padded_numel = table->padded;
  return YAFSDP_OK;
}

int yafsdp_gather_in(yafsdp_table* table, const void* const* tensor_ptrs, const uint8_t* mode, int tensor_dtype,
                     void* flat, int flat_dtype, double pre_factor, int zero_pad, void* stream) {
  if (table == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (!valid_dtype(tensor_dtype) || !valid_dtype(flat_dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (table->padded == 0) return YAFSDP_OK;
  if (flat == nullptr || (table->n_tensors > 0 && tensor_ptrs == nullptr)) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (!aligned_to(flat, 16)) return YAFSDP_ERR_MISALIGNED;
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return int(e);
  if (device != table->device) return YAFSDP_ERR_WRONG_DEVICE;
  int scale;
  float k;
  scale_plan(pre_factor, &scale, &k);
  hipStream_t s = static_cast<hipStream_t>(stream);
  int rc = check_dyn(table, tensor_ptrs, mode, item_size(tensor_dtype));
  if (rc != YAFSDP_OK) return rc;
  const int n_tiles = table->n_tiles;
  const int grid = grid_for(n_tiles, g_table_blocks_per_cu.load(std::memory_order_relaxed), device);
  if (table->n_tensors <= kSmallRoute) {
    SmallMeta meta;
    fill_small(table, tensor_ptrs, mode, &meta);
    return int(launch_gather<SmallMeta>(table->block, tensor_dtype, flat_dtype, scale, meta, flat, table->padded,
                                        n_tiles, k, zero_pad ? 1 : 0, gather_wt_from(table, flat_dtype), grid, s));
  }
  std::lock_guard<std::mutex> lock(table->mu);
  LargeMeta meta;
  int slot = -1;
  rc = stage_large(table, tensor_ptrs, mode, &meta, &slot, s);
  if (rc != YAFSDP_OK) return rc;
  e = launch_gather<LargeMeta>(table->block, tensor_dtype, flat_dtype, scale, meta, flat, table->padded, n_tiles, k,
                               zero_pad ? 1 : 0, gather_wt_from(table, flat_dtype), grid, s);
  if (e != hipSuccess) return abandon_large(table, slot, s, e);
  return finish_large(table, slot, s);
}

int yafsdp_copy_in_scatter_out(yafsdp_table* table, const void* flat, int flat_dtype, void* const* tensor_ptrs,
                               const uint8_t* mode, void* ag_in, const void* master, int master_dtype, int64_t n,
                               void* stream) {
  if (table == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (!valid_dtype(flat_dtype) || !valid_dtype(master_dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (n < 0 || (n > 0 && (ag_in == nullptr || master == nullptr))) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (table->total > 0 && (flat == nullptr || tensor_ptrs == nullptr)) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (table->total > 0 && !aligned_to(flat, 16)) return YAFSDP_ERR_MISALIGNED;
  if (n > 0 && (!aligned_to(ag_in, item_size(flat_dtype)) || !aligned_to(master, item_size(master_dtype))))
    return YAFSDP_ERR_MISALIGNED;
  if (n > 0) {  // the cast must not be in place unless the dtypes agree (then there is nothing to do)
    const uintptr_t d0 = reinterpret_cast<uintptr_t>(ag_in), s0 = reinterpret_cast<uintptr_t>(master);
    const uintptr_t d1 = d0 + uintptr_t(n) * item_size(flat_dtype), s1 = s0 + uintptr_t(n) * item_size(master_dtype);
    if (d0 < s1 && s0 < d1) return YAFSDP_ERR_INVALID_ARGUMENT;
  }
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return int(e);
  if (device != table->device) return YAFSDP_ERR_WRONG_DEVICE;
  const void* const* ptrs = const_cast<const void* const*>(tensor_ptrs);
  if (table->total > 0) {
    const int rc = check_dyn(table, ptrs, mode, item_size(flat_dtype));
    if (rc != YAFSDP_OK) return rc;
  }
  const int block = table->scatter_shape >> 4;  // the whole grid has the scatter-out workgroup size
  int64_t head = n > 0 ? ((16 - (reinterpret_cast<uintptr_t>(ag_in) & 15)) & 15) / item_size(flat_dtype) : 0;
  if (head > n) head = n;
  const int64_t flat_tile = int64_t(block) * kFusedFlatUnroll;  // units per workgroup of the flat job
  int64_t n_flat_blocks = n > 0 ? (((n - head) >> 3) + flat_tile - 1) / flat_tile : 0;
  if (n > 0 && n_flat_blocks < 1) n_flat_blocks = 1;  // workgroup 0 of the flat job peels head and tail
  const int64_t n_slots = table->total > 0 ? table->n_slots : 0;
  const int64_t grid = n_flat_blocks + n_slots;
  if (grid == 0) return YAFSDP_OK;
  if (grid > int64_t(INT32_MAX) - 4096) return YAFSDP_ERR_INVALID_ARGUMENT;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int wt_from = scatter_wt_from(table, flat_dtype);  // the tensors have the gathered buffer's dtype here
  const int cast_wt_from = flat_wt_from(n_flat_blocks, flat_tile, flat_dtype, g_flat_tail_mb);  // one tile per workgroup of the cast
  if (table->n_tensors <= kSmallRoute) {
    SmallMeta meta;
    static const void* const kNoPtrs[kSmallMax] = {};
    fill_small(table, table->total > 0 ? ptrs : kNoPtrs, mode, &meta);
    return int(launch_unshard<SmallMeta>(table->scatter_shape, master_dtype, flat_dtype, meta, flat, int(n_slots),
                                         wt_from, ag_in, master, n, int(head), int(n_flat_blocks), cast_wt_from,
                                         int(grid), s));
  }
  if (table->total == 0)  // nothing to split: the cast alone
    return flat_launch(master_dtype, flat_dtype, SCALE_NONE, false, ag_in, master, n, 1.0f, s);
  std::lock_guard<std::mutex> lock(table->mu);
  LargeMeta meta;
  int slot = -1;
  const int rc = stage_large(table, ptrs, mode, &meta, &slot, s);
  if (rc != YAFSDP_OK) return rc;
  e = launch_unshard<LargeMeta>(table->scatter_shape, master_dtype, flat_dtype, meta, flat, int(n_slots), wt_from, ag_in,
                                master, n, int(head), int(n_flat_blocks), cast_wt_from, int(grid), s);
  if (e != hipSuccess) return abandon_large(table, slot, s, e);
  return finish_large(table, slot, s);
}

int yafsdp_gather_in_post_reduce(yafsdp_table* table, const void* const* tensor_ptrs, const uint8_t* mode,
                                 int tensor_dtype, void* flat, int flat_dtype, double pre_factor, double custom_divisor,
                                 double post_factor, int zero_pad, void* shard, int shard_dtype, int accumulate,
                                 void* stream) {
  if (table == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (!valid_dtype(tensor_dtype) || !valid_dtype(flat_dtype) || !valid_dtype(shard_dtype))
    return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (!fused_reduce_supports(tensor_dtype, flat_dtype)) return YAFSDP_ERR_UNSUPPORTED;
  ReduceDivides dv = {SCALE_NONE, SCALE_NONE, 1.0f, 1.0f};
  if (custom_divisor != 0.0) {
    // the reference takes this branch only when neither of the other two factors exists (:141-145)
    if (pre_factor != 0.0 || post_factor != 0.0) return YAFSDP_ERR_INVALID_ARGUMENT;
    if (!scale_plan_any(custom_divisor, &dv.a_mode, &dv.a_k)) return YAFSDP_ERR_INVALID_ARGUMENT;
  } else {
    scale_plan(pre_factor, &dv.a_mode, &dv.a_k);
    scale_plan(post_factor, &dv.b_mode, &dv.b_k);
  }
  if (table->padded == 0) return YAFSDP_OK;
  if (flat == nullptr || shard == nullptr || (table->n_tensors > 0 && tensor_ptrs == nullptr))
    return YAFSDP_ERR_INVALID_ARGUMENT;
  if (!aligned_to(flat, 16) || !aligned_to(shard, 16)) return YAFSDP_ERR_MISALIGNED;
  {
    const uintptr_t d0 = reinterpret_cast<uintptr_t>(shard), s0 = reinterpret_cast<uintptr_t>(flat);
    const uintptr_t d1 = d0 + uintptr_t(table->padded) * item_size(shard_dtype);
    const uintptr_t s1 = s0 + uintptr_t(table->padded) * item_size(flat_dtype);
    if (d0 < s1 && s0 < d1) return YAFSDP_ERR_INVALID_ARGUMENT;
  }
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return int(e);
  if (device != table->device) return YAFSDP_ERR_WRONG_DEVICE;
  int rc = check_dyn(table, tensor_ptrs, mode, item_size(tensor_dtype));
  if (rc != YAFSDP_OK) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int grid = grid_for(table->n_tiles, g_table_blocks_per_cu.load(std::memory_order_relaxed), device);
  if (table->n_tensors <= kSmallRoute) {
    SmallMeta meta;
    fill_small(table, tensor_ptrs, mode, &meta);
    return int(launch_gather_post<SmallMeta>(table->block, tensor_dtype, flat_dtype, shard_dtype, meta, flat, shard,
                                             table->padded, table->n_tiles, zero_pad ? 1 : 0, accumulate ? 1 : 0, dv,
                                             grid, s));
  }
  std::lock_guard<std::mutex> lock(table->mu);
  LargeMeta meta;
  int slot = -1;
  rc = stage_large(table, tensor_ptrs, mode, &meta, &slot, s);
  if (rc != YAFSDP_OK) return rc;
  e = launch_gather_post<LargeMeta>(table->block, tensor_dtype, flat_dtype, shard_dtype, meta, flat, shard,
                                    table->padded, table->n_tiles, zero_pad ? 1 : 0, accumulate ? 1 : 0, dv, grid, s);
  if (e != hipSuccess) return abandon_large(table, slot, s, e);
  return finish_large(table, slot, s);
}

int yafsdp_scatter_out(yafsdp_table* table, const void* flat, int flat_dtype, void* const* tensor_ptrs,
                       const uint8_t* mode, int tensor_dtype, void* stream) {
  if (table == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (!valid_dtype(tensor_dtype) || !valid_dtype(flat_dtype)) return YAFSDP_ERR_UNSUPPORTED_DTYPE;
  if (table->total == 0) return YAFSDP_OK;
  if (flat == nullptr || tensor_ptrs == nullptr) return YAFSDP_ERR_INVALID_ARGUMENT;
  if (!aligned_to(flat, 16)) return YAFSDP_ERR_MISALIGNED;
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return int(e);
  if (device != table->device) return YAFSDP_ERR_WRONG_DEVICE;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const void* const* ptrs = const_cast<const void* const*>(tensor_ptrs);
  int rc = check_dyn(table, ptrs, mode, item_size(tensor_dtype));
  if (rc != YAFSDP_OK) return rc;
  const int n_tiles = table->n_slots;
  const int grid = grid_for(n_tiles, g_table_blocks_per_cu.load(std::memory_order_relaxed), device);
  if (table->n_tensors <= kSmallRoute) {
    SmallMeta meta;
    fill_small(table, ptrs, mode, &meta);
    return int(launch_scatter<SmallMeta>(table->scatter_shape, flat_dtype, tensor_dtype, meta, flat, table->total, n_tiles,
                                         scatter_wt_from(table, tensor_dtype), grid, s));
  }
  std::lock_guard<std::mutex> lock(table->mu);
  LargeMeta meta;
  int slot = -1;
  rc = stage_large(table, ptrs, mode, &meta, &slot, s);
  if (rc != YAFSDP_OK) return rc;
  e = launch_scatter<LargeMeta>(table->scatter_shape, flat_dtype, tensor_dtype, meta, flat, table->total, n_tiles,
                                scatter_wt_from(table, tensor_dtype), grid, s);
  if (e != hipSuccess) return abandon_large(table, slot, s, e);
  return finish_large(table, slot, s);
}

}  // extern "C"

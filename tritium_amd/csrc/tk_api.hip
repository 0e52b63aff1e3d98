// Host side of the C ABI: validation in the reference's order, device buffers, dispatch between the
// decode GEMV and the prefill GEMM, and the trait-shaped host-slice entry points.
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "tk_host.h"
#include "tk_internal.h"

// ------------------------------------------------------------------------------------------
// errors: thread-local last message (crates/tritium-ffi/src/lib.rs:9-28)
// ------------------------------------------------------------------------------------------

static thread_local char g_err[512];
static thread_local size_t g_expected, g_got;

int tk_fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof g_err, fmt, ap);
  va_end(ap);
  return code;
}
int tk_fail_mismatch(size_t expected, size_t got) {
  g_expected = expected;
  g_got = got;
  return tk_fail(TK_ERR_SHAPE_MISMATCH, "shape mismatch: expected %zu, got %zu", expected, got);
}
int tk_fail_oom(size_t requested) {
  g_expected = requested;
  g_got = 0;
  return tk_fail(TK_ERR_OUT_OF_MEMORY, "out of device memory: requested %zu bytes", requested);
}
extern "C" const char *tk_last_error(void) { return g_err; }
extern "C" void tk_last_mismatch(size_t *expected, size_t *got) {
  if (expected) *expected = g_expected;
  if (got) *got = g_got;
}

#define HIPCHK(call)                                                                      \
  do {                                                                                    \
    hipError_t e_ = (call);                                                               \
    if (e_ != hipSuccess) return tk_fail(TK_ERR_BACKEND, "%s: %s", #call, hipGetErrorString(e_)); \
  } while (0)
#define TKCHK(call)            \
  do {                         \
    int rc_ = (call);          \
    if (rc_ != TK_OK) return rc_; \
  } while (0)

// ------------------------------------------------------------------------------------------
// objects
// ------------------------------------------------------------------------------------------

struct DevBuf {
  void *p = nullptr;
  size_t cap = 0;
};

struct tk_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  // A second stream and two events: the two kernels of a grouped launch that has both a flow part and a
  // prefill-kernel part run side by side (lazily created; default priority like the first)
  hipStream_t stream2 = nullptr;
  hipEvent_t ev_fork = nullptr, ev_join = nullptr;
  int group_overlap = 1;   // 1 = run those two kernels side by side, 0 = one after the other
  std::mutex mu;
  tk_device_info info{};
  std::string device_id;
  int gemm_min_m = 65;
  size_t exact_max_macs = (size_t)1 << 20;
  int stream_min_groups = 0;  // set at init to the CU count
  int decode_force = 0;  // DECODE_AUTO
  int flow_run_tiles = 0;  // 0 = automatic
  int flow_ring = 0;       // 0 = automatic
  int flow_mfma = 0;       // 0 = automatic, 16 / 32 = force the 16x16x64 / 32x32x32 form of the flow kernel
  int gemm_tiles = 0;      // 0 = automatic, 2 / 4 = tiles per wave of the one-plane prefill kernel
  int gemm_two_by_two = 0;  // one-plane prefill kernel, 64 x 128 form: 0 = four waves side by side, 1 = two by two
  int gemm_ksplit = 0;     // prefill kernel, single launches: 0 = K slices chosen per launch, 1 = never split, n = n slices
  unsigned long long fused_calls = 0;  // calls that ran as one launch (tk_get_fused_calls)
  const char *last_kernel = "";        // contraction kernel of the last single call (tk_last_kernel)
  // Host-slice calls (tk_mpgemm, tk_mpgemm_with_act_quant) of up to host_direct_bytes of operands go through this
  // pinned host block: a copy kernel reads the activation and the scales from it, the kernels write the output into
  // it -- no copy-engine transfers (see host_call; grow-only; freed with the context)
  void *pin = nullptr;
  size_t pin_cap = 0;
  size_t host_direct_bytes = (size_t)1 << 20;
  int fuse_tokens = -1;    // single decode calls of up to this many tokens build their operand rows inside the decode kernel (-1 = chosen per call, 0 = never)
  int gemm_rows = 0;       // one-plane int8-contract prefill, single launches: 0 = tile rows chosen per launch, 64 / 128 / 256 = force
  bool gemm256_form_forced = false;  // tk_set_gemm256_form was called: automatic launches keep that form
  int gemm256_form = 0;    // the 256-row kernel: 0 = 4 waves x 224 outputs, 1 = 8 waves x 224, 2 = 4 waves x (128 | 96), two workgroups per CU
  int zero_skip = 0;       // uploads: 0 = keep a zero-chunk map when at least 0.5% of the chunks are zero, 1 = never, 2 = always
  int flow_wg16 = -1;      // flow kernel, sixteen-wave workgroups where a CU holds one workgroup's rows only: -1 = automatic, 0 = never, 1 = wherever a form exists
  int flow_swap = 1;       // flow kernel, int8 contract: 1 = weights as the first operand of the matrix instruction (one wide store per lane), 0 = activations first
  int base3 = 0;           // uploads: 0 = no base-3 stream, 1 = TQ1_0 uploads keep one beside the 2-bit codes, 2 = every upload
  unsigned *d_count = nullptr;  // a device counter for the uploads

  uint8_t *static_scratch = nullptr;  // this device's copy of `scratch` (below), resolved at tk_init
  DevBuf ap, rowsum, fscale, aux, exps, flags, h_act, h_out, h_scales, tmp, ynorm, blocksum, kpart, kcount;
  int *d_invalid = nullptr;
  bool kcount_stale = false;  // a K-split launch failed: its arrival counters are cleared before the next one
  // The context itself plus every weight buffer and group created on it: tk_destroy gives up the
  // context's own reference, the stream and this record live until the last of them is released, so
  // buffers and groups may be freed after tk_destroy.
  std::atomic<int> refs{1};
};

static void ctx_release(tk_ctx *ctx) {
  if (ctx->refs.fetch_sub(1) != 1) return;
  (void)hipSetDevice(ctx->device);
  if (ctx->ev_fork) (void)hipEventDestroy(ctx->ev_fork);
  if (ctx->ev_join) (void)hipEventDestroy(ctx->ev_join);
  if (ctx->stream2) (void)hipStreamDestroy(ctx->stream2);
  (void)hipStreamDestroy(ctx->stream);
  delete ctx;
}

struct tk_weights {
  tk_ctx *ctx;
  uint8_t *codes;           // n_tiles * nb chunks of 1 KiB, then one chunk of all-zero trits (0x55)
  uint8_t *codes3;          // the same chunks as a base-3 stream of 832 bytes each (tk_internal.h), or null
  uint32_t *zero_map;       // one bit per chunk, set = all-zero trits; null when too few chunks are zero
  size_t zero_chunks;       // how many chunks are zero (counted at upload whether or not the map is kept)
  float *block_scales;  // [(tile, K block), 16 rows] f32, only for uploads that keep the block scales
  size_t n, k, nb, n_tiles, len_bytes;
  int format;
  long invalid_row;
};

struct tk_event {
  hipEvent_t ev;
};

static int dev_malloc(size_t bytes, void **out) {
  *out = nullptr;
  if (!bytes) bytes = 16;
  hipError_t e = hipMalloc(out, bytes);
  if (e == hipErrorOutOfMemory || e == hipErrorMemoryAllocation) {
    (void)hipGetLastError();
    return tk_fail_oom(bytes);
  }
  if (e != hipSuccess) return tk_fail(TK_ERR_BACKEND, "hipMalloc(%zu): %s", bytes, hipGetErrorString(e));
  return TK_OK;
}

// Grow-only workspace. Growth waits for the stream first: an earlier launch may still read it.
static int ensure(tk_ctx *ctx, DevBuf &b, size_t bytes) {
  if (bytes <= b.cap) return TK_OK;
  if (b.p) {
    HIPCHK(hipStreamSynchronize(ctx->stream));
    HIPCHK(hipFree(b.p));
    b.p = nullptr;
    b.cap = 0;
  }
  size_t want = bytes + bytes / 4 + 256;
  TKCHK(dev_malloc(want, &b.p));
  b.cap = want;
  return TK_OK;
}

static inline size_t num_blocks(size_t k) { return (k + 255) / 256; }
static inline size_t fmt_block_bytes(int format) {
  return format == TK_FORMAT_TQ2_0 ? 66 : (format == TK_FORMAT_TQ1_0 ? 54 : 0);
}
static inline size_t dtype_size(int dt) { return dt == TK_BF16 ? 2 : (dt == TK_I8 ? 1 : 4); }

static bool prefer_stream(const tk_ctx *ctx, unsigned groups) { return groups >= (unsigned)ctx->stream_min_groups; }

// Which decode kernel a launch takes. All three give identical bits.
static int choose_decode(const tk_ctx *ctx, bool flow_ok, unsigned flow_groups, unsigned stream_groups) {
  switch (ctx->decode_force) {
    case 1: return 1;
    case 2: return 2;
    case 3: return flow_ok ? 3 : 2;
    default: break;
  }
  if (flow_ok && prefer_stream(ctx, flow_groups)) return 3;
  if (!flow_ok && prefer_stream(ctx, stream_groups)) return 2;
  return 1;
}

// ------------------------------------------------------------------------------------------
// static device scratch: the workspace of the entry point that allocates nothing
// (tk_linear_a8_noalloc). Every GPU the library runs on holds its own copy of this array until the
// process ends. In host code the array's name is only a stand-in for the symbol: the device address
// is resolved once per context by tk_init (hipGetSymbolAddress with the context's device current)
// and kept in tk_ctx::static_scratch, which is what kernels, and nothing else, receive.
// ------------------------------------------------------------------------------------------
#define TK_STATIC_SCRATCH_BYTES TK_NOALLOC_SCRATCH_BYTES  // the stated maximum (include/tritium_mi355x.h)
static __device__ __align__(256) unsigned char scratch[TK_STATIC_SCRATCH_BYTES];

// ------------------------------------------------------------------------------------------
// lifetime
// ------------------------------------------------------------------------------------------

extern "C" int tk_device_count(int *count) {
  if (!count) return tk_fail(TK_ERR_INVALID_INPUT, "tk_device_count: null pointer");
  int c = 0;
  hipError_t e = hipGetDeviceCount(&c);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    *count = 0;
    return tk_fail(TK_ERR_BACKEND, "hipGetDeviceCount: %s", hipGetErrorString(e));
  }
  *count = c;
  return TK_OK;
}

extern "C" int tk_init(int device, tk_ctx **out) {
  if (!out) return tk_fail(TK_ERR_INVALID_INPUT, "tk_init: null out pointer");
  *out = nullptr;
  int count = 0;
  TKCHK(tk_device_count(&count));
  if (device < 0 || device >= count)
    return tk_fail(TK_ERR_BACKEND, "tk_init: no HIP device %d (%d visible)", device, count);
  int min_m = 65;
  if (const char *env = getenv("TRITIUM_MI355X_GEMM_MIN_M")) {
    char *end = nullptr;
    long v = strtol(env, &end, 10);
    if (!*env || *end || v < 2 || v > 65)
      return tk_fail(TK_ERR_INVALID_INPUT, "TRITIUM_MI355X_GEMM_MIN_M=\"%s\" - use an integer in 2..65", env);
    min_m = (int)v;
  }
  HIPCHK(hipSetDevice(device));
  hipDeviceProp_t prop;
  HIPCHK(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return tk_fail(TK_ERR_BACKEND, "tk_init: device %d is %s; this library holds gfx950 code only", device,
                   prop.gcnArchName);
  tk_ctx *ctx = new (std::nothrow) tk_ctx();
  if (!ctx) return tk_fail(TK_ERR_BACKEND, "tk_init: host allocation failed");
  ctx->device = device;
  ctx->gemm_min_m = min_m;
  ctx->device_id = "mi355x:" + std::to_string(device);
  snprintf(ctx->info.name, sizeof ctx->info.name, "%s", prop.name[0] ? prop.name : "AMD Instinct MI355X");
  snprintf(ctx->info.arch, sizeof ctx->info.arch, "%s", prop.gcnArchName);
  ctx->info.total_memory_bytes = prop.totalGlobalMem;
  ctx->info.compute_units = prop.multiProcessorCount;
  ctx->stream_min_groups = prop.multiProcessorCount;
  ctx->info.clock_khz = prop.clockRate;
  ctx->info.memory_clock_khz = prop.memoryClockRate;
  ctx->info.memory_bus_bits = prop.memoryBusWidth;
  ctx->info.wavefront_size = prop.warpSize;
  ctx->info.lds_bytes_per_cu = (int)prop.maxSharedMemoryPerMultiProcessor;
  hipError_t e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
  if (e != hipSuccess) {
    delete ctx;
    return tk_fail(TK_ERR_BACKEND, "hipStreamCreate: %s", hipGetErrorString(e));
  }
  void *p = nullptr;
  int rc = dev_malloc(2 * sizeof(int), &p);
  if (rc) {
    (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return rc;
  }
  ctx->d_invalid = (int *)p;
  ctx->d_count = (unsigned *)p + 1;
  void *sp = nullptr;
  e = hipGetSymbolAddress(&sp, HIP_SYMBOL(scratch));  // device `device` is current: its copy of the array
  if (e != hipSuccess || !sp) {
    (void)hipFree(ctx->d_invalid);
    (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return tk_fail(TK_ERR_BACKEND, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
  }
  ctx->static_scratch = (uint8_t *)sp;
  *out = ctx;
  return TK_OK;
}

extern "C" void tk_destroy(tk_ctx *ctx) {
  if (!ctx) return;
  {
    std::lock_guard<std::mutex> lk(ctx->mu);
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    if (ctx->stream2) (void)hipStreamSynchronize(ctx->stream2);
    DevBuf *bufs[] = {&ctx->ap, &ctx->rowsum, &ctx->fscale, &ctx->aux, &ctx->exps,
                      &ctx->flags, &ctx->h_act, &ctx->h_out, &ctx->h_scales, &ctx->tmp,
                      &ctx->ynorm, &ctx->blocksum, &ctx->kpart, &ctx->kcount};
    for (DevBuf *b : bufs) {
      if (b->p) (void)hipFree(b->p);
      b->p = nullptr;
      b->cap = 0;
    }
    if (ctx->d_invalid) (void)hipFree(ctx->d_invalid);
    ctx->d_invalid = nullptr;
    if (ctx->pin) (void)hipHostFree(ctx->pin);
    ctx->pin = nullptr;
    ctx->pin_cap = 0;
  }
  ctx_release(ctx);
}

extern "C" const char *tk_device_id(const tk_ctx *ctx) { return ctx ? ctx->device_id.c_str() : ""; }

extern "C" int tk_device_info_get(const tk_ctx *ctx, tk_device_info *out) {
  if (!ctx || !out) return tk_fail(TK_ERR_INVALID_INPUT, "tk_device_info_get: null pointer");
  *out = ctx->info;
  return TK_OK;
}

extern "C" int tk_set_gemm_min_m(tk_ctx *ctx, int min_m) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_gemm_min_m: null context");
  if (min_m < 2 || min_m > 65) return tk_fail(TK_ERR_INVALID_INPUT, "gemm_min_m=%d - use an integer in 2..65", min_m);
  std::lock_guard<std::mutex> lk(ctx->mu);
  ctx->gemm_min_m = min_m;
  return TK_OK;
}
extern "C" int tk_get_gemm_min_m(const tk_ctx *ctx) { return ctx ? ctx->gemm_min_m : 0; }

extern "C" int tk_set_stream_min_groups(tk_ctx *ctx, int groups) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_stream_min_groups: null context");
  if (groups < 1) return tk_fail(TK_ERR_INVALID_INPUT, "stream_min_groups=%d - use a positive integer", groups);
  std::lock_guard<std::mutex> lk(ctx->mu);
  ctx->stream_min_groups = groups;
  return TK_OK;
}
extern "C" int tk_get_stream_min_groups(const tk_ctx *ctx) { return ctx ? ctx->stream_min_groups : 0; }

extern "C" int tk_set_flow_run_tiles(tk_ctx *ctx, int tiles) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_flow_run_tiles: null context");
  if (tiles < 0 || tiles > 1024) return tk_fail(TK_ERR_INVALID_INPUT, "flow_run_tiles=%d - use 0 (automatic) .. 1024", tiles);
  std::lock_guard<std::mutex> lk(ctx->mu);
  ctx->flow_run_tiles = tiles;
  return TK_OK;
}

extern "C" int tk_set_flow_mfma(tk_ctx *ctx, int rows) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_flow_mfma: null context");
  if (rows != 0 && rows != 16 && rows != 32)
    return tk_fail(TK_ERR_INVALID_INPUT, "flow_mfma=%d - use 0 (automatic), 16 or 32", rows);
  std::lock_guard<std::mutex> lk(ctx->mu);
  ctx->flow_mfma = rows;
  return TK_OK;
}

extern "C" int tk_set_gemm_tiles(tk_ctx *ctx, int tiles) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_gemm_tiles: null context");
  if (tiles != 0 && tiles != 2 && tiles != 4)
    return tk_fail(TK_ERR_INVALID_INPUT, "gemm_tiles=%d - use 0 (automatic), 2 or 4", tiles);
  std::lock_guard<std::mutex> lk(ctx->mu);
  ctx->gemm_tiles = tiles;
  return TK_OK;
}

extern "C" int tk_set_gemm_two_by_two(tk_ctx *ctx, int on) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_gemm_two_by_two: null context");
  std::lock_guard<std::mutex> lk(ctx->mu);
  ctx->gemm_two_by_two = on ? 1 : 0;
  return TK_OK;
}

extern "C" int tk_set_prep_team_rows(tk_ctx *ctx, int rows) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_prep_team_rows: null context");
  if (rows < 0) return tk_fail(TK_ERR_INVALID_INPUT, "prep_team_rows=%d - use 0 or more", rows);
  std::lock_guard<std::mutex> lk(ctx->mu);
  tk_prep_set_team_rows(rows);
  return TK_OK;
}

extern "C" int tk_set_group_overlap(tk_ctx *ctx, int on) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_group_overlap: null context");
  std::lock_guard<std::mutex> lk(ctx->mu);
  ctx->group_overlap = on ? 1 : 0;
  return TK_OK;
}

extern "C" int tk_set_host_direct_bytes(tk_ctx *ctx, size_t bytes) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_host_direct_bytes: null context");
  if (bytes > ((size_t)64 << 20)) return tk_fail(TK_ERR_INVALID_INPUT, "host_direct_bytes=%zu - use at most 64 MiB (0 = never)", bytes);
  std::lock_guard<std::mutex> lk(ctx->mu);
  ctx->host_direct_bytes = bytes;
  return TK_OK;
}

extern "C" int tk_set_fuse_tokens(tk_ctx *ctx, int tokens) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_fuse_tokens: null context");
  if (tokens < -1 || tokens > 4) return tk_fail(TK_ERR_INVALID_INPUT, "fuse_tokens=%d - use -1 (automatic), 0 (never) or 1..4", tokens);
  std::lock_guard<std::mutex> lk(ctx->mu);
  ctx->fuse_tokens = tokens;
  return TK_OK;
}

extern "C" int tk_get_fused_calls(tk_ctx *ctx, unsigned long long *count) {
  if (!ctx || !count) return tk_fail(TK_ERR_INVALID_INPUT, "tk_get_fused_calls: null argument");
  std::lock_guard<std::mutex> lk(ctx->mu);
  *count = ctx->fused_calls;
  return TK_OK;
}

extern "C" const char *tk_last_kernel(tk_ctx *ctx) {
  if (!ctx) return "";
  std::lock_guard<std::mutex> lk(ctx->mu);
  return ctx->last_kernel;
}

extern "C" int tk_set_gemm_rows(tk_ctx *ctx, int rows) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_gemm_rows: null context");
  if (rows != 0 && rows != 64 && rows != 128 && rows != 256)
    return tk_fail(TK_ERR_INVALID_INPUT, "gemm_rows=%d - use 0 (automatic), 64, 128 or 256", rows);
  std::lock_guard<std::mutex> lk(ctx->mu);
  ctx->gemm_rows = rows;
  return TK_OK;
}

extern "C" int tk_set_gemm256_form(tk_ctx *ctx, int form) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_gemm256_form: null context");
  if (form < -1 || form > 2) return tk_fail(TK_ERR_INVALID_INPUT, "gemm256_form=%d - use -1 (chosen per launch), 0, 1 or 2", form);
  std::lock_guard<std::mutex> lk(ctx->mu);
  ctx->gemm256_form = form < 0 ? 0 : form;
  ctx->gemm256_form_forced = form >= 0;
  return TK_OK;
}

extern "C" int tk_set_gemm_ksplit(tk_ctx *ctx, int slices) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_gemm_ksplit: null context");
  if (slices < 0 || slices > 64) return tk_fail(TK_ERR_INVALID_INPUT, "gemm_ksplit=%d - use 0 (automatic), 1 (off) or 2..64", slices);
  std::lock_guard<std::mutex> lk(ctx->mu);
  ctx->gemm_ksplit = slices;
  return TK_OK;
}

extern "C" int tk_set_zero_skip(tk_ctx *ctx, int mode) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_zero_skip: null context");
  if (mode < 0 || mode > 2) return tk_fail(TK_ERR_INVALID_INPUT, "zero_skip=%d - use 0 (by threshold), 1 (never) or 2 (always)", mode);
  std::lock_guard<std::mutex> lk(ctx->mu);
  ctx->zero_skip = mode;
  return TK_OK;
}

extern "C" int tk_set_flow_operand_order(tk_ctx *ctx, int weights_first) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_flow_operand_order: null context");
  if (weights_first < 0 || weights_first > 1) return tk_fail(TK_ERR_INVALID_INPUT, "flow_operand_order=%d - use 0 (activations first) or 1 (weights first)", weights_first);
  std::lock_guard<std::mutex> lk(ctx->mu);
  ctx->flow_swap = weights_first;
  return TK_OK;
}

extern "C" int tk_set_flow_workgroup_waves(tk_ctx *ctx, int waves) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_flow_workgroup_waves: null context");
  if (waves != 0 && waves != 8 && waves != 16) return tk_fail(TK_ERR_INVALID_INPUT, "flow_workgroup_waves=%d - use 0 (automatic), 8 or 16", waves);
  std::lock_guard<std::mutex> lk(ctx->mu);
  ctx->flow_wg16 = waves == 16 ? 1 : (waves == 8 ? 0 : -1);
  return TK_OK;
}

extern "C" int tk_set_base3_stream(tk_ctx *ctx, int mode) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_base3_stream: null context");
  if (mode < 0 || mode > 2) return tk_fail(TK_ERR_INVALID_INPUT, "base3_stream=%d - use 0 (off), 1 (TQ1_0 uploads) or 2 (every upload)", mode);
  std::lock_guard<std::mutex> lk(ctx->mu);
  ctx->base3 = mode;
  return TK_OK;
}

extern "C" int tk_set_flow_ring(tk_ctx *ctx, int positions) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_flow_ring: null context");
  if (positions != 0 && (positions < 2 || positions > 5))
    return tk_fail(TK_ERR_INVALID_INPUT, "flow_ring=%d - use 0 (automatic) or 2..5", positions);
  std::lock_guard<std::mutex> lock(ctx->mu);
  ctx->flow_ring = positions;
  return TK_OK;
}

extern "C" int tk_set_decode_kernel(tk_ctx *ctx, int variant) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_decode_kernel: null context");
  if (variant < 0 || variant > 3) return tk_fail(TK_ERR_INVALID_INPUT, "decode kernel %d - use 0..3", variant);
  std::lock_guard<std::mutex> lk(ctx->mu);
  ctx->decode_force = variant;
  return TK_OK;
}

extern "C" int tk_set_exact_max_macs(tk_ctx *ctx, size_t macs) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_set_exact_max_macs: null context");
  std::lock_guard<std::mutex> lk(ctx->mu);
  ctx->exact_max_macs = macs;
  return TK_OK;
}
extern "C" size_t tk_get_exact_max_macs(const tk_ctx *ctx) { return ctx ? ctx->exact_max_macs : 0; }

// ------------------------------------------------------------------------------------------
// weights
// ------------------------------------------------------------------------------------------

static int upload_weights(tk_ctx *ctx, const uint8_t *packed, size_t packed_len, size_t n, size_t k, int format,
                          bool keep_block_scales, tk_weights **out);

extern "C" int tk_upload_weights(tk_ctx *ctx, const uint8_t *packed, size_t packed_len, size_t n, size_t k,
                                 int format, tk_weights **out) {
  return upload_weights(ctx, packed, packed_len, n, k, format, false, out);
}

extern "C" int tk_upload_weights_scaled(tk_ctx *ctx, const uint8_t *packed, size_t packed_len, size_t n, size_t k,
                                        tk_weights **out) {
  return upload_weights(ctx, packed, packed_len, n, k, TK_FORMAT_TQ2_0, true, out);
}

static int upload_weights(tk_ctx *ctx, const uint8_t *packed, size_t packed_len, size_t n, size_t k, int format,
                          bool keep_block_scales, tk_weights **out) {
  if (!ctx || !out) return tk_fail(TK_ERR_INVALID_INPUT, "tk_upload_weights: null pointer");
  *out = nullptr;
  const size_t bb = fmt_block_bytes(format);
  if (!bb) return tk_fail(TK_ERR_UNSUPPORTED_FORMAT, "unsupported ternary format: %d", format);
  const size_t nb = num_blocks(k);
  size_t row_bytes, expected;
  if (__builtin_mul_overflow(nb, bb, &row_bytes))
    return tk_fail(TK_ERR_INVALID_INPUT, "packed row byte count overflows");
  if (__builtin_mul_overflow(n, row_bytes, &expected))
    return tk_fail(TK_ERR_INVALID_INPUT, "packed weight byte count overflows");
  if (packed_len != expected)
    return tk_fail(TK_ERR_INVALID_INPUT, "packed len %zu != expected %zu for shape n=%zu k=%zu format %d",
                   packed_len, expected, n, k, format);
  if (!packed && packed_len) return tk_fail(TK_ERR_INVALID_INPUT, "tk_upload_weights: null packed pointer");
  if (n > (size_t)INT32_MAX - 16 || k > (size_t)INT32_MAX - 256)
    return tk_fail(TK_ERR_INVALID_INPUT, "shape n=%zu k=%zu exceeds the kernels' int index range", n, k);

  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  const size_t n_tiles = (n + 15) / 16;
  const size_t n_chunks = n_tiles * nb, code_bytes = n_chunks * TK_CHUNK_BYTES;
  const size_t map_words = (n_chunks + 31) / 32;
  void *codes = nullptr, *raw = nullptr, *bscales = nullptr, *zmap = nullptr, *codes3 = nullptr;
  const bool want3 = n_chunks && !keep_block_scales && (ctx->base3 == 2 || (ctx->base3 == 1 && format == TK_FORMAT_TQ1_0));
  TKCHK(dev_malloc(code_bytes + TK_ZERO_CHUNKS * TK_CHUNK_BYTES, &codes));  // + the resident all-zero chunks
  int rc = dev_malloc(packed_len, &raw);
  if (!rc && want3) rc = dev_malloc(n_chunks * TK_B3_CHUNK_BYTES, &codes3);
  if (!rc && keep_block_scales) rc = dev_malloc(n_tiles * nb * 16 * sizeof(float), &bscales);
  if (!rc && ctx->zero_skip != 1 && n_chunks) rc = dev_malloc(map_words * 4, &zmap);
  if (rc) {
    (void)hipFree(codes);
    if (raw) (void)hipFree(raw);
    if (bscales) (void)hipFree(bscales);
    if (codes3) (void)hipFree(codes3);
    return rc;
  }
  int invalid = INT32_MAX;
  unsigned zero_chunks = 0;
  hipError_t e = hipMemsetAsync((uint8_t *)codes + code_bytes, 0x55, TK_ZERO_CHUNKS * TK_CHUNK_BYTES, ctx->stream);
  if (e == hipSuccess && zmap) e = hipMemsetAsync(zmap, 0, map_words * 4, ctx->stream);
  if (e == hipSuccess && zmap) e = hipMemsetAsync(ctx->d_count, 0, sizeof(unsigned), ctx->stream);
  if (e == hipSuccess && packed_len) e = hipMemcpyAsync(raw, packed, packed_len, hipMemcpyHostToDevice, ctx->stream);
  if (e == hipSuccess) e = hipMemcpyAsync(ctx->d_invalid, &invalid, sizeof invalid, hipMemcpyHostToDevice, ctx->stream);
  if (e == hipSuccess) {
    if (format == TK_FORMAT_TQ2_0)
      e = tk_launch_relayout_tq2(ctx->stream, (const uint8_t *)raw, (uint8_t *)codes, n, nb, ctx->d_invalid,
                                 (float *)bscales);
    else
      e = tk_launch_relayout_tq1(ctx->stream, (const uint8_t *)raw, (uint8_t *)codes, n, nb);
  }
  if (e == hipSuccess && codes3) e = tk_launch_encode_base3(ctx->stream, (const uint8_t *)codes, (uint8_t *)codes3, n_chunks);
  if (e == hipSuccess && zmap)
    e = tk_launch_zero_chunk_map(ctx->stream, (const uint8_t *)codes, n_chunks, (uint32_t *)zmap, ctx->d_count);
  if (e == hipSuccess && zmap)
    e = hipMemcpyAsync(&zero_chunks, ctx->d_count, sizeof zero_chunks, hipMemcpyDeviceToHost, ctx->stream);
  if (e == hipSuccess) e = hipMemcpyAsync(&invalid, ctx->d_invalid, sizeof invalid, hipMemcpyDeviceToHost, ctx->stream);
  if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
  (void)hipFree(raw);
  // The map is worth carrying when enough chunks are zero: the reference's threshold for its per-row
  // bitmaps, BITMAP_MIN_ZERO_BLOCK_FRAC = 0.005 (crates/tritium-cuda/src/cuda/mod.rs:384-405), applied
  // to the 16-row chunks this layout streams.
  if (zmap && !(ctx->zero_skip == 2 || (double)zero_chunks >= 0.005 * (double)n_chunks)) {
    (void)hipFree(zmap);
    zmap = nullptr;
  }
  if (e != hipSuccess) {
    (void)hipFree(codes);
    if (bscales) (void)hipFree(bscales);
    if (zmap) (void)hipFree(zmap);
    if (codes3) (void)hipFree(codes3);
    return tk_fail(TK_ERR_BACKEND, "upload_weights: %s", hipGetErrorString(e));
  }
  tk_weights *w = new (std::nothrow) tk_weights();
  if (!w) {
    (void)hipFree(codes);
    if (bscales) (void)hipFree(bscales);
    if (zmap) (void)hipFree(zmap);
    if (codes3) (void)hipFree(codes3);
    return tk_fail(TK_ERR_BACKEND, "tk_upload_weights: host allocation failed");
  }
  w->zero_map = (uint32_t *)zmap;
  w->zero_chunks = zero_chunks;
  w->ctx = ctx;
  w->codes = (uint8_t *)codes;
  w->codes3 = (uint8_t *)codes3;
  w->block_scales = (float *)bscales;
  w->n = n;
  w->k = k;
  w->nb = nb;
  w->n_tiles = n_tiles;
  w->len_bytes = packed_len;
  w->format = format;
  w->invalid_row = invalid == INT32_MAX ? -1 : invalid;
  ctx->refs.fetch_add(1);
  *out = w;
  return TK_OK;
}

extern "C" int tk_upload_weights_i2s(tk_ctx *ctx, const uint8_t *payload, size_t payload_len, size_t n, size_t k,
                                     tk_weights **out, float *scale) {
  if (!ctx || !out || !scale) return tk_fail(TK_ERR_INVALID_INPUT, "tk_upload_weights_i2s: null pointer");
  *out = nullptr;
  // the payload must hold the tensor before anything is sized from the caller's n and k
  // (the converter's own checks, in its order and with its errors: crates/tritium-format/src/i2s.rs:122-135)
  size_t elems;
  if (__builtin_mul_overflow(n, k, &elems)) return tk_fail(TK_ERR_INVALID_INPUT, "I2_S element count overflows");
  if (elems % 128 != 0) return tk_fail(TK_ERR_INVALID_INPUT, "I2_S tensor of %zu elements is not a multiple of 128", elems);
  if (payload_len < elems / 4 + 4) return tk_fail_mismatch(elems / 4 + 4, payload_len);
  const size_t len = tk_packed_len(n, k, TK_FORMAT_TQ2_0);
  if (!len && n && k) return tk_fail(TK_ERR_INVALID_INPUT, "packed weight byte count overflows");
  std::vector<uint8_t> packed;
  try {
    packed.resize(len);
  } catch (const std::exception &) {
    return tk_fail(TK_ERR_BACKEND, "tk_upload_weights_i2s: host allocation of %zu bytes failed", len);
  }
  TKCHK(tk_convert_i2s_to_tq2_0(payload, payload_len, n, k, packed.data(), len, scale));
  return tk_upload_weights(ctx, packed.data(), len, n, k, TK_FORMAT_TQ2_0, out);
}

extern "C" int tk_upload_weights_gguf(tk_ctx *ctx, const tk_gguf *g, const uint8_t *file, size_t file_len,
                                      const char *name, tk_weights **out, float *row_scales, size_t row_scales_len) {
  if (!ctx || !out) return tk_fail(TK_ERR_INVALID_INPUT, "tk_upload_weights_gguf: null pointer");
  *out = nullptr;
  size_t n, k;
  int format;
  TKCHK(tk_gguf_ternary_shape(g, name, &n, &k, &format));
  // the dims of a tensor are the file's word: check them against the bytes the file really holds
  // before sizing anything from them (a crafted header may claim 2^62 rows)
  {
    tk_gguf_tensor info;
    uint64_t off = 0, plen = 0;
    if (!tk_gguf_tensor_find(g, name, &info)) return tk_fail(TK_ERR_INVALID_INPUT, "tensor `%s` not found", name);
    TKCHK(tk_gguf_tensor_payload(g, file_len, &info, &off, &plen));
    size_t nk;
    if (__builtin_mul_overflow(n, k, &nk) || nk / 5 > plen)  // the densest packing holds 5 trits per byte
      return tk_fail(TK_ERR_INVALID_INPUT, "tensor `%s` claims %zu x %zu elements but its payload holds %llu bytes", name, n, k,
                     (unsigned long long)plen);
  }
  const size_t len = tk_packed_len(n, k, format);
  if (!len && n && k) return tk_fail(TK_ERR_INVALID_INPUT, "packed weight byte count overflows");
  if (row_scales_len != n) return tk_fail_mismatch(n, row_scales_len);
  std::vector<uint8_t> packed;
  try {
    packed.resize(len);
  } catch (const std::exception &) {
    return tk_fail(TK_ERR_BACKEND, "tk_upload_weights_gguf: host allocation of %zu bytes failed", len);
  }
  TKCHK(tk_gguf_load_ternary(g, file, file_len, name, packed.data(), len, row_scales, row_scales_len));
  return tk_upload_weights(ctx, packed.data(), len, n, k, format, out);
}

extern "C" void tk_free_weights(tk_weights *w) {
  if (!w) return;
  tk_ctx *ctx = w->ctx;
  {
    std::lock_guard<std::mutex> lk(ctx->mu);
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipFree(w->codes);
    if (w->block_scales) (void)hipFree(w->block_scales);
    if (w->zero_map) (void)hipFree(w->zero_map);
    if (w->codes3) (void)hipFree(w->codes3);
    delete w;
  }
  ctx_release(ctx);
}
extern "C" size_t tk_weights_len_bytes(const tk_weights *w) { return w ? w->len_bytes : 0; }
extern "C" int tk_weights_zero_chunks(const tk_weights *w, size_t *zero, size_t *total, int *map_kept) {
  if (!w) return tk_fail(TK_ERR_INVALID_INPUT, "tk_weights_zero_chunks: null buffer");
  if (zero) *zero = w->zero_chunks;
  if (total) *total = w->n_tiles * w->nb;
  if (map_kept) *map_kept = w->zero_map ? 1 : 0;
  return TK_OK;
}
extern "C" size_t tk_weights_base3_bytes(const tk_weights *w) {
  return w && w->codes3 ? w->n_tiles * w->nb * (size_t)TK_B3_CHUNK_BYTES : 0;
}
extern "C" size_t tk_weights_n(const tk_weights *w) { return w ? w->n : 0; }
extern "C" size_t tk_weights_k(const tk_weights *w) { return w ? w->k : 0; }
extern "C" int tk_weights_format(const tk_weights *w) { return w ? w->format : 0; }

extern "C" int tk_weights_download_trits(tk_ctx *ctx, const tk_weights *w, int8_t *trits, size_t trits_len) {
  if (!ctx || !w || (!trits && trits_len)) return tk_fail(TK_ERR_INVALID_INPUT, "tk_weights_download_trits: null pointer");
  if (w->ctx != ctx) return tk_fail(TK_ERR_INVALID_INPUT, "buffer belongs to another context");
  if (trits_len != w->n * w->k) return tk_fail_mismatch(w->n * w->k, trits_len);
  if (!trits_len) return TK_OK;
  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  TKCHK(ensure(ctx, ctx->tmp, trits_len));
  HIPCHK(tk_launch_decode_trits(ctx->stream, w->codes, w->n, w->k, w->nb, (int8_t *)ctx->tmp.p));
  HIPCHK(hipMemcpyAsync(trits, ctx->tmp.p, trits_len, hipMemcpyDeviceToHost, ctx->stream));
  HIPCHK(hipStreamSynchronize(ctx->stream));
  return TK_OK;
}

// ------------------------------------------------------------------------------------------
// dispatch
// ------------------------------------------------------------------------------------------

static const size_t kLdsABudget = 48 * 1024;
static const int kSkinnyMaxRows = 64;

static int validate_layer(tk_ctx *ctx, const tk_linear_desc *layer, size_t *n, size_t *k) {
  if (!layer) return tk_fail(TK_ERR_INVALID_INPUT, "null layer descriptor");
  if (layer->n_planes < 1 || layer->n_planes > TK_MAX_PLANES)
    return tk_fail(TK_ERR_INVALID_INPUT, "n_planes=%d - use 1..%d", layer->n_planes, TK_MAX_PLANES);
  for (int p = 0; p < layer->n_planes; ++p) {
    const tk_weights *w = layer->planes[p];
    if (!w) return tk_fail(TK_ERR_INVALID_INPUT, "plane %d: null weights handle", p);
    if (w->ctx != ctx) return tk_fail(TK_ERR_INVALID_INPUT, "plane %d: buffer belongs to another context", p);
    if (!layer->scales[p] && w->n) return tk_fail(TK_ERR_INVALID_INPUT, "plane %d: null scales pointer", p);
    if (p && (w->n != layer->planes[0]->n || w->k != layer->planes[0]->k))
      return tk_fail(TK_ERR_INVALID_INPUT, "plane %d is [%zu,%zu] but plane 0 is [%zu,%zu]", p, w->n, w->k,
                     layer->planes[0]->n, layer->planes[0]->k);
    if (w->invalid_row >= 0)  // what the CPU backend's unpack reports (crates/tritium-cpu/src/lib.rs:213)
      return tk_fail(TK_ERR_BACKEND, "unpack row %ld: decoded value 2 outside ternary range", w->invalid_row);
  }
  *n = layer->planes[0]->n;
  *k = layer->planes[0]->k;
  return TK_OK;
}

struct Plan {
  TkProblem pr;
  TkPrep prep;
  int prep_kind;
  bool skinny;            // a decode kernel (<= 64 operand rows), else the GEMM
  TkLaunchCfg cfg;        // K-split decode kernel or GEMM
  unsigned grid_m, grid_n;
  // streaming decode kernel (same rt / planes as cfg)
  unsigned stream_groups; // workgroups this problem needs
  size_t stream_lds;
  int stream_kc;
  // flow decode kernel: needs every K block of the operand rows in LDS
  bool flow_ok;
  size_t flow_lds;
};

enum { DECODE_AUTO = 0, DECODE_KSPLIT = 1, DECODE_STREAM = 2, DECODE_FLOW = 3, DECODE_GEMM = 4 };

static const size_t kLdsFlowMax = 160 * 1024;
// Waves per workgroup of the flow kernels: four up to 64 KiB of operand rows, eight beyond; with two row tiles and
// more, eight as soon as a CU has room for at most two workgroups' rows (more than a third of the 160 KiB; one row
// tile keeps the 64 KiB limit: not measured there, and its single-launch form that builds the rows itself is a
// four-wave kernel). What counts is waves per CU: two four-wave workgroups are eight
// waves, two eight-wave workgroups sixteen where the registers allow it (the one-plane forms of two row tiles on a
// ring of two: 126), and where they do not a single eight-wave workgroup stages the rows once instead of twice.
// Measured, 96-128 layer copies per launch, four -> eight waves between 53 and 64 KiB of rows: one plane K=2560,
// 22 / 24 int8 rows x 6912 outputs 3.35 -> 4.36 / 3.30 -> 4.32 TB/s, 2560 outputs 3.39 -> 4.20, six float tokens
// 3.74 -> 4.83; the 32x32x32 form at 64 KiB (two planes K=2048, eight float tokens) 5.32 -> 5.70 with runs of four
// pairs on a ring of two.
static int flow_waves(size_t lds, int rt, bool sixteen = false) {
  if (sixteen && rt == 2 && lds > kLdsFlowMax / 2) return 16;
  return lds > (rt >= 2 ? kLdsFlowMax / 3 : 64 * 1024) ? 8 : 4;
}
// Sixteen-wave workgroups for 17..32 operand rows that take more than half of the LDS, so that a CU runs one workgroup:
// four waves per SIMD instead of two. The forms that exist with 1024 threads are those that stay within 128 registers by
// themselves: two row tiles of one or two planes on a ring of two, with weights first (int8 contract) or, activations
// first, from a problem table (float contract 5 / 6 / 8 tokens in groups: one plane K=5120 N=5120 102 -> 94.5 / 104 -> 96 /
// 109 -> 100 us, K=4096 N=11008 129 -> 129 / 135 -> 129.5 / 138.5 -> 133.5). Measured under the int8 contract, 64 layer copies
// per launch, eight -> sixteen waves (the eight on the ring they would pick): one plane K=5120 N=5120 17 / 24 / 32 rows
// 113 -> 102 / 118 -> 107 / 124 -> 112 us; K=4096 N=11008 24 / 32 rows 157 -> 149 / 167 -> 155; K=3584 N=8192 105 -> 102 /
// 108 -> 107; K=3072 N=8192 32 rows 94 -> 92. With the run length of each chosen by flow_run_tiles' model of such launches
// (32 layer copies, 24 / 32 rows, eight -> sixteen waves): three planes K=5120 N=17408 397 -> 387 / 407 -> 395, N=5120
// 133 -> 123 / 138 -> 125; two planes K=5120 N=17408 286 -> 268 / 295 -> 278, K=4096 N=4096 61 -> 56 / 64 -> 57; one plane
// K=5120 N=17408 164 -> 153 / 174 -> 156, K=4096 N=11008 88 -> 80 / 93 -> 84. A ring of three under sixteen waves is 2-6%
// slower than the ring of two. Launches too small to give every CU a workgroup of sixteen waves with runs of two
// tiles keep eight.
static bool flow_sixteen(const tk_ctx *ctx, bool int8_mode, bool table, bool wide, bool b3, int planes, size_t tiles, int tw) {
  if (!ctx->flow_wg16 || wide || b3 || planes > (int8_mode && ctx->flow_swap ? 3 : 2)) return false;
  if (!(int8_mode && ctx->flow_swap) && !table) return false;  // (activations first: only the forms that read a problem table)
  if (ctx->flow_ring != 0 && ctx->flow_ring != 2) return false;
  if (ctx->flow_wg16 > 0) return true;
  return tiles >= (size_t)ctx->info.compute_units * 16u * (size_t)tw * 2u;
}
// widest row stride any kernel asks of the staged operand rows of an R-row problem
static size_t kPrepRowsMax(size_t R) { return R + 16 > 64 ? R + 16 : 64; }

// The 32x32x32 form of the flow kernel: 17..64 operand rows, one or two planes (more would not fit the
// register file with a prefetch ring). Its operand rows have a fixed stride of 32 or 64 rows, in the
// workspace and in LDS, and 1 KiB of LDS behind them holds the row constants.
static const size_t kFlowWideExtraLds = 1024;
static size_t flow_wide_rows(int rt) { return rt <= 2 ? 32 : 64; }
static size_t flow_wide_lds(int rt, size_t nb) { return nb * 256 * flow_wide_rows(rt); }
// Measured over 128-192 layer copies of N=8192 with K=1024/2048/2560 and one or two planes, float and
// int8 contract: at 25..32 rows the wide form is 3-16% faster as long as its rows leave room for two
// workgroups per CU (<= 64 KiB); with one workgroup per CU, or at 20-24 rows (which both forms pad
// to 32), the 16x16x64 form is as fast or up to 4% faster. At 33..64 rows the picture is mixed (two
// planes K=2048 int8: 9% faster; one plane: 4-18% slower), so those keep the 16x16x64 form unless
// the wide one is asked for.
// weights_first (int8 contract, both forms with weights as the first operand, 96 copies, bf16 out, 25..32 rows): with
// one plane the 16x16x64 form is as fast or up to 19% faster (N=8192 K=2048 28 rows 94 vs 113 us; K=1024 32 rows 68 vs
// 72); with two planes and K=1024 it is 14% faster (103..116 vs 119..122), with two planes and K=1536..2048 the wide form
// wins by 0..8% at most sizes (N=8192 K=1536 28 rows 149 vs 139; K=2048 32 rows 178 vs 169; N=11008 K=2048 5% slower).
static bool flow_wide(const tk_ctx *ctx, int planes, int rt, size_t nb, size_t rows, bool weights_first) {
  if (rt < 2 || planes > 2 || flow_wide_lds(rt, nb) + kFlowWideExtraLds > kLdsFlowMax) return false;
  if (ctx->flow_mfma == 16) return false;
  if (ctx->flow_mfma == 32) return true;
  if (weights_first && (planes < 2 || flow_wide_lds(rt, nb) <= 32 * 1024)) return false;
  return rt == 2 && rows > 24 && flow_wide_lds(rt, nb) <= 64 * 1024;
}
static int flow_runs_per_wave(bool wide, bool b3, int planes, int rt, size_t rows) {
  if (b3) return tk_flow3_runs_per_wave(planes);
  return wide ? tk_flow32_runs_per_wave() : tk_flow_runs_per_wave(planes, rt, (int)rows);
}
// The base-3 form of the flow kernel: every plane of the problem carries a base-3 stream, at most three
// planes and 32 operand rows, and the rows fit in LDS behind the decode table.
static bool flow_base3(const TkProblem &pr, int planes, int rt, size_t rows_lds) {
  if (planes > 3 || rt > 2 || TK_B3_TABLE_BYTES + rows_lds > kLdsFlowMax) return false;
  for (int p = 0; p < planes; ++p)
    if (!pr.codes3[p]) return false;
  return true;
}
// Room for the zero-chunk maps of a flow launch: the tiles per workgroup whose map words are staged behind the operand
// rows (behind the row constants in the 32x32x32 form), or 0 when they do not fit or the form ignores the maps
// (base-3 stream; the fused single-launch form keeps its row constants there) -- plain loads then.
static size_t flow_zero_plan(bool wide, bool b3, bool fused, int planes, size_t flow_lds, size_t tiles_per_wg, size_t nb) {
  if (b3 || fused || !tiles_per_wg) return 0;
  const size_t words = (size_t)planes * tk_flow_zmap_words(tiles_per_wg, nb) * 4;
  return flow_lds + (wide ? kFlowWideExtraLds : 0) + words <= kLdsFlowMax ? tiles_per_wg : 0;
}
// zmap_tiles > 0: some plane of the launch carries a zero-chunk map (flow_zero_plan)
// (b3: flow_lds includes the decode table; ring and runs per wave are the base-3 kernel's own)
// swap: the launch runs under the int8 contract and the context asks for the second operand order where a form exists
// (both matrix-instruction forms of the kernel that reads a prepared set of operand rows)
static void flow_cfg_form(TkLaunchCfg *cfg, bool wide, bool b3, size_t flow_lds, size_t rows, size_t zmap_tiles = 0,
                          size_t zmap_nb = 0, bool swap = false) {
  cfg->wide_mfma = wide ? 1 : 0;
  cfg->base3 = b3 ? 1 : 0;
  if (b3) cfg->ring = 4;
  cfg->tw = flow_runs_per_wave(wide, b3, cfg->planes, cfg->rt, rows);
  cfg->lds_bytes = flow_lds + (wide ? kFlowWideExtraLds : 0);
  if (zmap_tiles) cfg->lds_bytes += (size_t)cfg->planes * tk_flow_zmap_words(zmap_tiles, zmap_nb) * 4;
  if (wide && cfg->ring > 4) cfg->ring = 4;
  cfg->zmap32 = wide && zmap_tiles ? 1 : 0;
  cfg->swap = swap && !b3 ? 1 : 0;
}

// Ring size of a flow launch: the kernels' own rule (tk_flow_ring), except that the 32x32x32 form in eight-wave
// workgroups of up to 64 KiB of rows takes two positions (two planes K=2048, eight float tokens: 5.54 -> 5.70 TB/s; one
// plane, 28 int8 rows: 3.65 -> 4.24: on two positions its one-plane forms stay within 128 registers, four waves per SIMD).
// One row tile of two or more planes over at most eight K blocks also takes two positions, at 4 rows (one float token)
// and from 9 rows on: K=2048 N=8192, 128 layer copies, four -> two positions, two planes, float contract 1 / 3 / 4 tokens
// 6.43 -> 6.61 / 5.96 -> 6.09 / 5.90 -> 5.99 TB/s, int8 contract 9 / 12 / 16 tokens 5.77 -> 5.85 / 5.73 -> 5.83 / 5.74 -> 5.81
// (3 int8 tokens 6.21 -> 6.14: left on four); three planes, one float token 6.33 -> 6.56. Sixteen K blocks (K=4096) show
// no difference either way.
static int pick_flow_ring(const tk_ctx *ctx, const int *nbs, const double *wts, int count, int rt, int rows, int tw,
                          bool wide, int waves, size_t lds, int planes) {
  if (waves >= 16) return 2;  // (the only forms with 1024 threads)
  if (ctx->flow_ring) return ctx->flow_ring;
  if (wide && waves >= 8 && lds <= 64 * 1024) return 2;
  int nb_max = 0;
  for (int i = 0; i < count; ++i) nb_max = nbs[i] > nb_max ? nbs[i] : nb_max;
  if (!wide && rt == 1 && planes >= 2 && nb_max <= 8 && (rows == 4 || rows >= 9)) return 2;
  return tk_flow_ring(nbs, wts, count, rt, rows, tw);
}

// Consecutive tiles per run of the flow kernel. A workgroup pays for staging its operand rows
// (lds_bytes) once, so it should stream several times that in weights; beyond that, shorter runs
// win (more, shorter-lived workgroups keep more loads in flight and balance the tail). Measured on
// K=2048 N=8192 x 2 planes over 128 layer copies: 4-16 operand rows peak at 2 tiles per run
// (128 KiB of weights per workgroup), 32 rows at 4 (4x the staged bytes, four-wave workgroups), 64
// rows at 8 (16x, eight-wave workgroups, one per CU). Re-measured with the ring at 4 positions: 4-8
// operand rows (8-16 KiB staged) are 5-8% faster with runs of ONE tile (64 KiB per workgroup), 16
// rows stay at 2.
// Re-measured with the weight stream read through non-temporal loads (same shape; sweep of run length x ring size): one
// row tile of two or more TOKENS now peaks at 2 tiles per run -- float contract 2 / 4 tokens 5.85 -> 6.33 / 5.58 -> 5.95
// TB/s, int8 contract 4 / 8 / 16 tokens 5.44 -> 6.16 / 4.99 -> 5.92 / 5.35 -> 5.76 -- and a single token stays at one
// (6.45 / 6.66 TB/s; 6.52 / 6.55 with two): what separates the two is the output a run writes when it ends. Tiles of
// less than 16 KiB of codes (one plane, K = 2560) take two per run at every token count (one int8 token 6.03 -> 6.47).
static int flow_run_tiles(const tk_ctx *ctx, unsigned total_tiles, int planes, int rt, int waves, size_t lds_bytes,
                          size_t nb, bool wide, bool b3, size_t rows, size_t tokens) {
  if (ctx->flow_run_tiles > 0) return ctx->flow_run_tiles;
  const size_t per_s = (size_t)waves * (size_t)flow_runs_per_wave(wide, b3, planes, rt, rows);
  const size_t tile_bytes = (size_t)planes * (nb ? nb : 1) * (b3 ? TK_B3_CHUNK_BYTES : TK_CHUNK_BYTES);
  const size_t w8 = waves > 8 ? 8 : (size_t)waves;  // (a sixteen-wave workgroup: twice the target of eight waves)
  size_t target = lds_bytes * w8 * w8 / (waves >= 8 && lds_bytes > 64 * 1024 ? 2 : 4) * ((size_t)waves / w8);
  if (target < 64 * 1024) target = 64 * 1024;
  size_t s = 1;
  while (s < 16 && per_s * (2 * s) * tile_bytes <= target) s *= 2;
  if (!wide && !b3 && rt == 1 && s < 2 && (tokens >= 2 || tile_bytes < 16 * 1024)) s = 2;
  // keep every CU supplied: two four-wave workgroups each, or one eight-wave workgroup (those fill
  // the LDS of a CU alone, and a single round of them has no change-over in the middle of the launch)
  const unsigned per_cu = waves >= 8 ? 1u : 2u;
  while (s > 1 && total_tiles / (per_s * s) < per_cu * (unsigned)ctx->info.compute_units) --s;
  while (s & (s - 1)) s &= s - 1;  // a power of two: runs of 3 tiles measured 5% slower than runs of 2 or 4
  // Two or four row tiles whose rows leave a CU room for ONE workgroup (more than 80 KiB): the launch
  // is a few rounds of one workgroup per CU, and what decides is how the workgroup count falls on the CUs. Cost of a
  // run length = (rounds + 1/4) x (bytes a workgroup streams + twice the bytes it stages), a last partial round counting for at
  // least three quarters (its workgroups share the memory system among fewer: 160 of 256 CUs busy measured as fast as
  // all) and the quarter standing for the start and the end of the launch, where every CU stages or drains at once
  // (one round of exactly 256 workgroups measured 13% slower than two rounds of half their length).
  // Measured against this model over N in {5120, 11008, 17408}, K in {4096, 5120}, one to three planes, 24 / 32 int8
  // rows, 32 layer copies, runs of 1 / 2 / 4 / 8 tiles, eight- and sixteen-wave workgroups: the model's choice is the
  // measured best or within 4% of it, where the rule above (fitted to K = 2048) was 15-29% behind (three planes N=17408
  // K=5120 24 rows, eight waves: 423 / 400 / 420 / 472 us, rule: 8 tiles; one plane, sixteen waves: 153 / 165 / 196 / 177).
  // Four row tiles likewise (40 / 64 int8 rows, 32 copies, runs of 1 / 2 / 4 / 8): one plane K=2560 N=6912 68 / 55 / 49 / 80
  // and 79 / 67 / 54 / 89 us, N=2560 32 / 24 / 41 / 77; K=2048 N=11008 64 rows 102 / 84 / 88 / 81; three planes K=2048 N=5120
  // 64 rows 95 / 90 / 102 / 86 -- the model picks the best of each. Four row tiles keep the rule's run length where it
  // fills its rounds to nine tenths: 128 copies of two planes K=2048 N=8192 at 64 rows (the benchmark's launches of this
  // kind) are ONE round of 256 workgroups with runs of 16, which measured 3% faster than the two rounds of 8 that the
  // model would take.
  // One row tile in eight-wave workgroups (more than 64 KiB of rows: 13..16 rows of K > 4096) is priced the same way, also
  // where two workgroups share a CU: a CU's time follows the number of workgroups it is handed (two planes K=5120 N=5120
  // 16 rows, 32 copies, runs of 1 / 2 / 4 / 8: 86 / 94 / 77 / 123 us, rule: 2; three planes N=17408 370 / 364 / 387 / 425,
  // rule: 4).
  bool use_model = !b3 && waves >= 8 && (rt == 1 || (rt >= 2 && lds_bytes > kLdsFlowMax / 2));
  if (use_model && rt > 2) {
    const double wgs = (double)((total_tiles + per_s * s - 1) / (per_s * s)), cus = (double)ctx->info.compute_units;
    const double rounds = (double)(size_t)((wgs + cus - 1.0) / cus);
    use_model = wgs < 0.9 * rounds * cus;
  }
  if (use_model) {
    const double cus = (double)ctx->info.compute_units;
    double best = 0.0;
    int best_s = 1;
    for (int c = 1; c <= 16; c *= 2) {
      const double wgs = (double)((total_tiles + per_s * (size_t)c - 1) / (per_s * (size_t)c));
      const double full = (double)(size_t)(wgs / cus), rem = wgs - full * cus;
      const double rounds = 0.25 + full + (rem > 0.0 ? (rem > 0.75 * cus ? rem : 0.75 * cus) / cus : 0.0);
      const double cost = rounds * ((double)c * (double)per_s * (double)tile_bytes + 2.0 * (double)lds_bytes);
      // (equal costs are common, the terms being powers of two: one row tile then measured better with the longer run
      // -- K=5120 N=5120 16 rows 48 vs 42 us, K=8192 N=8192 105 vs 97 --, two row tiles with the shorter)
      if (c == 1 || cost < best || (rt == 1 && cost <= best)) {
        best = cost;
        best_s = c;
      }
    }
    return best_s;
  }
  return (int)s;
}

// Members of a grouped launch get whole workgroups: a member of n tiles occupies ceil(n / per) * per
// tile slots, per = tiles per workgroup. With members of very different sizes (q/k/v/o/gate/up: 160,
// 40, 40, 160, 432, 432 tiles) long runs leave most slots of the small members empty: shorten the
// runs until at most a tenth of the slots is padding (30 layers x 6 projections at 32 tokens:
// 199 -> 174 us per step).
static int trim_run_tiles(const tk_ctx *ctx, int s, size_t per_s, const std::vector<unsigned> &member_tiles) {
  if (ctx->flow_run_tiles > 0) return s;
  unsigned total = 0;
  for (unsigned n : member_tiles) total += n;
  while (s > 1) {
    const unsigned per = (unsigned)per_s * (unsigned)s;
    unsigned slots = 0;
    for (unsigned n : member_tiles) slots += (n + per - 1) / per * per;
    if ((double)(slots - total) <= 0.10 * (double)slots) break;
    s >>= 1;
  }
  return s;
}

static const size_t kLdsStreamBudget = 64 * 1024;

// The streaming kernel wants every CU busy; below that the K-split kernel's finer grain wins.
static bool prefer_stream(const tk_ctx *ctx, unsigned groups);

// Fills everything of a plan that does not depend on workspace addresses.
// GEMM form of a planned problem: padded operand row stride, tile grid and its split over the XCDs.
// fill > 0 (single launches): one plane normally gives a wave 4 tiles; when that leaves fewer
// workgroups than `fill` (four per CU), 2 tiles per wave double them. A/B on one box, call incl.
// quantization, K=2560 N=6912: 64..256 tokens 25 -> 18-19 us, 512: 26.5 -> 23.6, 768: 33.2 -> 28.8,
// 2048 (864 workgroups): 59.8 -> 58.5; from 1088 workgroups on the 4-tile form wins (1024 x 5120 ->
// 17408: 100 vs 104 us; 4096 x 5120 -> 17408: 314 vs 362 us).
static void plan_gemm(Plan *pl, unsigned fill = 0, int force_nt = 0) {
  TkProblem &pr = pl->pr;
  const size_t R = (size_t)pr.R;
  // The GEMM reads, per K block, 16 segments of the operand rows that are exactly rs*16 bytes apart,
  // and all workgroups do so in step: with a power-of-two stride they would all land on the same
  // few memory channels. 16 rows (256 bytes) of padding walk the segments across the channels.
  pr.rs = (int)(R + 16);
  pl->cfg.rt = 4;
  pl->cfg.lds_bytes = (size_t)tk_gemm_lds_bytes();  // three 64-row blocks of 256 k + the row constants
  pl->grid_m = (unsigned)((R + 63) / 64);
  unsigned per_wg = (unsigned)tk_gemm_tiles_per_wg(pr.planes);
  pl->cfg.gemm_nt = 0;
  const bool few = fill && pl->grid_m * (((unsigned)pr.n_tiles + per_wg - 1) / per_wg) < fill;
  if (pr.planes == 1 && (force_nt == 2 || (force_nt == 0 && few))) {
    per_wg /= 2;
    pl->cfg.gemm_nt = 2;
  }
  pl->grid_n = ((unsigned)pr.n_tiles + per_wg - 1) / per_wg;
  // split the tile grid over the 8 XCDs so that each L2 holds few A row blocks and few weight
  // column blocks: minimise bytes touched per XCD = K*(64*sub_m + 4*tiles_per_wg*planes*sub_n)
  pr.grid_m = (int)pl->grid_m;
  pr.grid_n = (int)pl->grid_n;
  size_t best = (size_t)-1;
  for (int xr = 1; xr <= 8; xr *= 2) {
    const int xc = 8 / xr;
    const int sm = ((int)pl->grid_m + xr - 1) / xr, sn = ((int)pl->grid_n + xc - 1) / xc;
    const size_t cost = (size_t)64 * sm + (size_t)4 * per_wg * pr.planes * sn;
    const size_t waste = (size_t)8 * sm * sn;  // launched workgroups, some of them empty
    const size_t score = cost * 1024 + waste;
    if (score < best) {
      best = score;
      pr.xr = xr;
      pr.sub_m = sm;
      pr.sub_n = sn;
    }
  }
}

// The 128 x 256 kernel's grid: row blocks of 128 operand rows, column blocks of 16 tiles, split over the
// XCDs like plan_gemm's (the operand-row stride plan_gemm chose stays).
static void plan_gemm128(Plan *pl) {
  TkProblem &pr = pl->pr;
  pl->grid_m = (unsigned)(((size_t)pr.R + 127) / 128);
  pl->grid_n = ((unsigned)pr.n_tiles + 15u) / 16u;
  pr.grid_m = (int)pl->grid_m;
  pr.grid_n = (int)pl->grid_n;
  pr.ksplit = 0;
  size_t best = (size_t)-1;
  for (int xr = 1; xr <= 8; xr *= 2) {
    const int xc = 8 / xr;
    const int sm = ((int)pl->grid_m + xr - 1) / xr, sn = ((int)pl->grid_n + xc - 1) / xc;
    const size_t cost = (size_t)128 * sm + (size_t)64 * sn;  // bytes touched per XCD and unit of K
    const size_t waste = (size_t)8 * sm * sn;
    const size_t score = cost * 1024 + waste;
    if (score < best) {
      best = score;
      pr.xr = xr;
      pr.sub_m = sm;
      pr.sub_n = sn;
    }
  }
}

// The 256 x 224 kernel's grid: row blocks of 256 operand rows, column blocks of 14 tiles, split over the XCDs
// (the operand-row stride plan_gemm chose stays). An XCD reads, per unit of K, 256 bytes of operand rows per row
// block it owns and 56 bytes of codes per column block.
static void plan_gemm256(Plan *pl) {
  TkProblem &pr = pl->pr;
  pl->grid_m = (unsigned)(((size_t)pr.R + 255) / 256);
  pl->grid_n = ((unsigned)pr.n_tiles + 13u) / 14u;
  pr.grid_m = (int)pl->grid_m;
  pr.grid_n = (int)pl->grid_n;
  pr.ksplit = 0;
  size_t best = (size_t)-1;
  for (int xr = 1; xr <= 8; xr *= 2) {
    const int xc = 8 / xr;
    const int sm = ((int)pl->grid_m + xr - 1) / xr, sn = ((int)pl->grid_n + xc - 1) / xc;
    const size_t cost = (size_t)256 * sm + (size_t)56 * sn;
    const size_t waste = (size_t)8 * sm * sn;
    const size_t score = cost * 1024 + waste;
    if (score < best) {
      best = score;
      pr.xr = xr;
      pr.sub_m = sm;
      pr.sub_n = sn;
    }
  }
}

// Where the 128 x 256 kernel is chosen over the 64-row forms: launches it finishes in one round of its 512
// resident workgroups (two per CU) and that still give most CUs one. A/B on one box, int8 rows in, bf16 out,
// call incl. the operand re-ordering launch, 64-row kernels -> 128 x 256: 2048 x 2560 -> 6912 (432 blocks)
// 47.9 -> 44.7 us; 1024 tokens (216) 30.0 -> 28.2; 512 tokens (108) 17.6 -> 24.8; 256 tokens 13.8 -> 23.6;
// 2048 x 6912 -> 2560 (160) 52.0 -> 56.8; 2048 x 2560 -> 2560 (160) 27.7 -> 30.0; and with several rounds:
// 8192 x 2560 -> 6912 (1728) 135 -> 140; 4096 x 5120 -> 17408 (2176) 288 -> 302; 4096 x 17408 -> 5120 (640)
// 294 -> 330.
static bool gemm128_pays(const tk_ctx *ctx, size_t rows, size_t blocks128) {
  const size_t cus = (size_t)ctx->info.compute_units;
  return rows >= 1024 && blocks128 * 4 >= cus * 3 && blocks128 <= 2 * cus;
}

// Where the 256-row kernel (weight tile expanded once per workgroup) is chosen: launches of 1024 rows or more that give
// 0.7 .. 1 workgroups per CU, as eight waves of 32 rows over whole 224-output column blocks. A/B on one box, bf16 rows
// in and out, call incl. quantization, best of the 64-row / 128-row kernels -> this form: 2048 x 2560 -> 6912 (248
// blocks) 45.6 -> 41.6 us; 1536 x 2560 -> 6912 (186) 40.4 -> 38.9; 2048 x 5120 -> 5120 (184) 62.6 -> 59.8; 4096 x 2560 ->
// 2560 (192) 42.2 -> 40.8. Outside that window it loses -- one workgroup per CU leaves every round's prologue and
// epilogue in the open: 1024 x 2048 -> 8192 (148 blocks) 26.7 -> 31.2; 3072 x 2560 -> 6912 (372) 61.8 -> 64.5; 4096 x 17408
// -> 5120 320 -> 360 -- and the form with two workgroups per CU over 128 | 96 outputs is within 1-2% of the 64-row
// kernels either way (e.g. 4096 x 5120 -> 17408 282 -> 276, 1024 x 2048 -> 8192 26.7 -> 30.9): not chosen by itself.
static bool gemm256_pays(const tk_ctx *ctx, size_t rows, size_t n_tiles, int *form) {
  const size_t cus = (size_t)ctx->info.compute_units;
  const size_t blocks = ((rows + 255) / 256) * ((n_tiles + 13) / 14);
  *form = ctx->gemm256_form_forced ? ctx->gemm256_form : 1;
  return rows >= 1024 && blocks <= cus && blocks * 10 >= cus * 7;
}

static void plan_shape(tk_ctx *ctx, const tk_linear_desc *layer, size_t n, size_t k, size_t m, int mode,
                       int out_dtype, Plan *pl) {
  memset(pl, 0, sizeof *pl);
  TkProblem &pr = pl->pr;
  const size_t nb = num_blocks(k);
  const size_t R = mode == TK_MODE_DIGITS ? 4 * m : m;
  for (int p = 0; p < layer->n_planes; ++p) {
    pr.codes[p] = layer->planes[p]->codes;
    pr.codes3[p] = layer->planes[p]->codes3;
    pr.scales[p] = layer->scales[p];
    pr.zmap[p] = layer->planes[p]->zero_map;
    if (pr.zmap[p]) pr.zskip = 1;
  }
  pr.n = (int)n;
  pr.k = (int)k;
  pr.nb = (int)nb;
  pr.R = (int)R;
  pr.rs = (int)R;
  pr.M = (int)m;
  pr.mode = mode;
  pr.out_dtype = out_dtype;
  pr.planes = layer->n_planes;
  pr.n_tiles = (int)((n + 15) / 16);
  const bool small = R <= (size_t)kSkinnyMaxRows && (mode == TK_MODE_DIGITS || m < (size_t)ctx->gemm_min_m);
  pl->skinny = small;
  pl->cfg.planes = layer->n_planes;
  if (small) {
    const int rt = R <= 16 ? 1 : (R <= 32 ? 2 : 4);
    size_t kc = kLdsABudget / (256 * (R ? R : 1));
    if (kc < 1) kc = 1;
    if (kc > nb) kc = nb ? nb : 1;
    pr.kc = (int)kc;
    size_t lds_a = kc * 256 * R, lds_r = (size_t)4 * layer->n_planes * rt * 1024;
    pl->cfg.rt = rt;
    pl->cfg.lds_bytes = lds_a > lds_r ? lds_a : lds_r;
    pl->cfg.grid = (unsigned)pr.n_tiles;
    const unsigned tpw = (unsigned)tk_stream_tiles_per_wg(layer->n_planes, rt);
    pl->stream_groups = ((unsigned)pr.n_tiles + tpw - 1) / tpw;
    size_t skc = kLdsStreamBudget / (256 * (R ? R : 1));
    if (skc < 1) skc = 1;
    if (skc > nb) skc = nb ? nb : 1;
    pl->stream_kc = (int)skc;
    pl->stream_lds = skc * 256 * R;
    pl->flow_lds = nb * 256 * R;
    pl->flow_ok = pl->flow_lds <= kLdsFlowMax;
  } else {
    plan_gemm(pl, 4u * (unsigned)ctx->info.compute_units, ctx->gemm_tiles);
  }
}

static int check_norm(const tk_rmsnorm *norm) {
  if (!norm || !norm->weight) return tk_fail(TK_ERR_INVALID_INPUT, "null RMSNorm weight");
  if (!(norm->eps >= 0.0f) || !(norm->eps <= 3.402823466e38f))
    return tk_fail(TK_ERR_INVALID_INPUT, "RMSNorm eps %g - use a finite value >= 0", (double)norm->eps);
  return TK_OK;
}

// The per-call workspace of run_linear: operand rows and the per-row / per-token side arrays.
struct Workspace {
  int8_t *ap;
  int32_t *rowsum;
  float *fscale, *aux;
  int32_t *exps;
  uint32_t *flags;
  float *ynorm;
};

// From the context's grow-only buffers (may allocate), or -- static_ws -- carved out of the static
// device scratch, which allocates nothing and refuses what does not fit.
static int take_workspace(tk_ctx *ctx, bool static_ws, size_t ap_bytes, size_t R, size_t m, size_t ynorm_bytes,
                          Workspace *ws) {
  if (!static_ws) {
    TKCHK(ensure(ctx, ctx->ap, ap_bytes));
    TKCHK(ensure(ctx, ctx->rowsum, R * 4));
    TKCHK(ensure(ctx, ctx->fscale, m * 4));
    TKCHK(ensure(ctx, ctx->aux, m * 4));
    TKCHK(ensure(ctx, ctx->exps, m * 4));
    TKCHK(ensure(ctx, ctx->flags, m * 4));
    if (ynorm_bytes) TKCHK(ensure(ctx, ctx->ynorm, ynorm_bytes));
    *ws = Workspace{(int8_t *)ctx->ap.p,   (int32_t *)ctx->rowsum.p, (float *)ctx->fscale.p, (float *)ctx->aux.p,
                    (int32_t *)ctx->exps.p, (uint32_t *)ctx->flags.p, (float *)ctx->ynorm.p};
    return TK_OK;
  }
  size_t used = 0;
  auto carve = [&](size_t bytes) {
    uint8_t *p = ctx->static_scratch + used;
    used += (bytes + 255) & ~(size_t)255;
    return p;
  };
  ws->ap = (int8_t *)carve(ap_bytes);
  ws->rowsum = (int32_t *)carve(R * 4);
  ws->fscale = (float *)carve(m * 4);
  ws->aux = (float *)carve(m * 4);
  ws->exps = (int32_t *)carve(m * 4);
  ws->flags = (uint32_t *)carve(m * 4);
  ws->ynorm = ynorm_bytes ? (float *)carve(ynorm_bytes) : nullptr;
  if (used > TK_STATIC_SCRATCH_BYTES || ap_bytes > TK_STATIC_SCRATCH_BYTES)
    return tk_fail(TK_ERR_INVALID_INPUT,
                   "this call needs %zu bytes of workspace; the static scratch of the allocation-free entry point "
                   "holds %zu (operand rows take about tokens * ceil(k/256) * 256 bytes)",
                   used, (size_t)TK_STATIC_SCRATCH_BYTES);
  return TK_OK;
}

static int run_linear(tk_ctx *ctx, const tk_linear_desc *layer, int mode, int prep_kind, const void *act,
                      int act_dtype, const float *act_scale_in, size_t m, void *out, int out_dtype,
                      const tk_rmsnorm *norm = nullptr, bool static_ws = false, const void *residual = nullptr) {
  size_t n, k;
  TKCHK(validate_layer(ctx, layer, &n, &k));
  if (m == 0 || n == 0) return TK_OK;  // crates/tritium-rocm/src/rocm.rs:521-523
  if (!act || !out) return tk_fail(TK_ERR_INVALID_INPUT, "null activation or output pointer");
  if (out_dtype == TK_I32 && (layer->n_planes != 1 || mode != TK_MODE_INT8))
    return tk_fail(TK_ERR_INVALID_INPUT, "raw int32 accumulators need one plane and int8 activations");
  size_t total;
  if (__builtin_mul_overflow(m, n, &total) || total > (size_t)INT32_MAX || m * 4 > (size_t)INT32_MAX)
    return tk_fail(TK_ERR_INVALID_INPUT, "shape m=%zu n=%zu k=%zu exceeds the kernels' int index range", m, n, k);

  Plan pl;
  plan_shape(ctx, layer, n, k, m, mode, out_dtype, &pl);
  const size_t nb = pl.pr.nb, R = pl.pr.R;
  int variant = DECODE_KSPLIT, run_tiles = 1;
  unsigned flow_groups = 0;
  bool wide = false, b3 = false;
  size_t flow_lds = pl.flow_lds;
  if (pl.skinny) {
    b3 = pl.flow_ok && flow_base3(pl.pr, pl.cfg.planes, pl.cfg.rt, flow_lds);
    wide = !b3 && pl.flow_ok && flow_wide(ctx, pl.cfg.planes, pl.cfg.rt, nb, R, mode == TK_MODE_INT8 && ctx->flow_swap);
    if (wide) flow_lds = flow_wide_lds(pl.cfg.rt, nb);
    if (b3) flow_lds += TK_B3_TABLE_BYTES;
    const int fw = b3 ? tk_flow3_waves(pl.cfg.rt) : flow_waves(flow_lds, pl.cfg.rt, flow_sixteen(ctx, mode == TK_MODE_INT8, false, wide, b3, pl.cfg.planes, (size_t)pl.pr.n_tiles, flow_runs_per_wave(wide, b3, pl.cfg.planes, pl.cfg.rt, R)));
    run_tiles = flow_run_tiles(ctx, (unsigned)pl.pr.n_tiles, pl.cfg.planes, pl.cfg.rt, fw, flow_lds, nb, wide, b3, R, m);
    const unsigned per_wg = (unsigned)fw * (unsigned)flow_runs_per_wave(wide, b3, pl.cfg.planes, pl.cfg.rt, R) * (unsigned)run_tiles;
    flow_groups = ((unsigned)pl.pr.n_tiles + per_wg - 1) / per_wg;
    // (an eight-wave workgroup of the flow kernel fills a CU alone: it counts as two. 17408 x 5120 x 3 planes, 16 / 24 /
    // 32 int8 rows, 136 such workgroups: 36.8 / 32.0 / 32.1 us through the K-split or prefill kernel, 21.2 / 26.3 / 27.5
    // through the flow kernel)
    variant = choose_decode(ctx, pl.flow_ok, flow_groups * (unsigned)(fw >= 8 ? 2 : 1), pl.stream_groups);
    // One token of a layer of more than two tiles per CU: the K-split kernel's single-launch form has a workgroup per
    // tile and, beyond two workgroups per CU, hands each several tiles one after the other; the flow kernel's
    // single-launch form (below) walks them in waves side by side. bf16 token, int8 contract, rotating layer copies,
    // K-split -> flow at 640 / 768 tiles (512 tiles are a tie; from 1024 on the flow kernel is chosen anyway): one plane
    // K=2048 7.7 -> 5.9 / 8.8 -> 6.0 us, K=4096 10.3 -> 7.2 / 10.3 -> 7.3, K=8192 13.6 -> 10.1 / 13.9 -> 10.3; two planes
    // K=4096 11.4 -> 8.6 / 11.6 -> 8.6; three planes K=4096 13.4 -> 10.2 / 15.1 -> 10.7. More tokens are mixed (4 tokens:
    // two and three planes of K <= 4096 gain 10-20%, one plane of K=8192 loses 20%) and stay.
    if (ctx->decode_force == DECODE_AUTO && variant == DECODE_KSPLIT && pl.flow_ok && !wide && !b3 && m == 1 &&
        ctx->fuse_tokens != 0 && (unsigned)pl.pr.n_tiles > 2u * (unsigned)ctx->info.compute_units && pl.cfg.rt == 1 &&
        (prep_kind == TK_PREP_A8 || prep_kind == TK_PREP_DIGITS) && nb * 16 <= 512 && k % 256 == 0 &&
        ((uintptr_t)act & 15) == 0 && (act_dtype == TK_F32 || act_dtype == TK_BF16) &&
        (!norm || ((uintptr_t)norm->weight & 15) == 0) &&
        flow_lds + 1024 + (norm ? k * 4 + 1024 : 0) + 1024 <= 64 * 1024)
      variant = DECODE_FLOW;
    // Up to eight operand rows of two or more planes on such a layer likewise (both as prep + kernel, or against the
    // K-split kernel's single launch of two tokens): 640 / 768 tiles, two planes, 2 / 4 / 8 int8 tokens, K=2048 11.4 -> 9.9 /
    // 12.5 -> 10.4 / 13.0 -> 10.6 us, K=4096 13.6 -> 12.3 / 14.5 -> 12.7 / 15.6 -> 13.8, K=8192 21.2 -> 17.9 / 19.1 -> 18.6 /
    // 21.9 -> 20.7; three planes K=4096 15.2 -> 14.2 / 16.9 -> 14.7 / 18.5 -> 15.7. One plane is within 5% either way for
    // K <= 4096 and 15-24% slower through the flow kernel at K=8192: left.
    if (ctx->decode_force == DECODE_AUTO && variant == DECODE_KSPLIT && pl.flow_ok && !wide && !b3 && pl.cfg.rt == 1 &&
        R >= 2 && R <= 8 && pl.cfg.planes >= 2 && (unsigned)pl.pr.n_tiles > 2u * (unsigned)ctx->info.compute_units)
      variant = DECODE_FLOW;
    // Narrower layers of two or more planes with short rows (K <= 2560), 3..8 operand rows that the K-split kernel would
    // not build itself (three int8 tokens or more, two float tokens): the flow kernel again, both as prep + kernel.
    // 3 / 4 / 8 int8 tokens, K-split -> flow: two planes K=2048 N=2560 10.0 -> 9.2 / 10.6 -> 9.9 / 11.3 -> 10.2 us, N=8192
    // 4 / 8 tokens 11.8 -> 10.5 / 12.4 -> 10.5; three planes K=2048 N=6144 12.2 -> 10.3 / 12.7 -> 10.6 / 13.6 -> 11.3; K=2560
    // from 256 tiles on: two planes N=5120 11.2 -> 10.9 / 11.9 -> 11.1 / 12.5 -> 11.9, three planes 12.5 -> 11.4 / 13.4 -> 11.6 /
    // 14.0 -> 12.4 (160 tiles: two planes 10.4 -> 11.0: left). K=4096 is within 3-7% either way, K=5120 up to 14% slower
    // through the flow kernel: left.
    if (ctx->decode_force == DECODE_AUTO && variant == DECODE_KSPLIT && pl.flow_ok && !wide && !b3 && pl.cfg.rt == 1 &&
        pl.cfg.planes >= 2 && R >= 3 && R <= 8 && m >= (prep_kind == TK_PREP_A8 ? 3u : 2u) &&
        (nb <= 8 || (nb <= 10 && pl.pr.n_tiles >= 256)))
      variant = DECODE_FLOW;
    if (variant == DECODE_FLOW && wide) pl.pr.rs = (int)flow_wide_rows(pl.cfg.rt);
    // Operand rows that do not fit in LDS: the prefill kernel (rows streamed from L2 block by block)
    // beats the decode kernels that re-stage slices of K behind barriers, beyond 32 rows always and
    // from 17 rows on layers of at least 16384 outputs. A/B on one box, int8 rows,
    // call incl. quantization, decode kernel -> prefill kernel: 64 x 5120 -> 17408 with 1/2/3 planes
    // 63/71/70 -> 28/35/41 us; 64 x 17408 -> 5120 113 -> 68 us; 48 x 6912 -> 2560 38 -> 31 us;
    // 40 x 5120 -> 17408 46 -> 28 us; 32 x 6912 -> 16384 53 -> 32 us; 32 x 5632 -> 17408 x 3 planes
    // 60 -> 43 us. Narrower launches of up to 32 rows stay on the K-split kernel (32 x 6912 -> 2560: 31
    // vs 31 us; 24 rows 26 vs 31; 32 x 8192 -> 8192 x 2 planes: 40 vs 45; 17 x 17408 -> 5120: 55 vs 65).
    if (ctx->decode_force == DECODE_AUTO && !pl.flow_ok && (R > 32 || (R > 16 && pl.pr.n_tiles >= 1024))) {
      pl.skinny = false;
      plan_gemm(&pl, 4u * (unsigned)ctx->info.compute_units, ctx->gemm_tiles);
    }
    // Narrow launches that would take the K-split kernel (one workgroup per 16 outputs, each staging every operand
    // row): with its K split the prefill kernel is the faster one beyond 32 rows (the K-split kernel's four-row-tile
    // form), beyond 16 rows of one plane under the int8 contract (16384 x 2048, 24 rows: 18.4 -> 12.6 us; a tie on
    // layers of 2560 outputs), and from 16 rows when the rows need more than one pass through LDS (5120 x 17408 x 3
    // planes, 16 rows: 42.6 -> 38.8). Measured, call incl. prep, K-split -> prefill kernel, bf16 tokens: 2560 x 2560 one plane,
    // 32 / 48 / 64 int8 rows 15.4 -> 13.9 / 18.9 -> 14.0 / 22.1 -> 13.9 us, float contract 12 / 16 tokens 18.1 -> 15.1 /
    // 21.4 -> 15.1 (8 tokens 14.6 -> 15.1: left alone); 6912 x 2560 two planes 48 / 64 rows 21.1 -> 16.2 / 24.5 -> 16.1
    // (32 rows 17.1 -> 16.0, float 8 tokens 16.1 -> 17.1: left alone); K = 6912 (two passes) one plane 16 / 32 / 64
    // rows 18.5 -> 16.3 / 27.3 -> 16.6 / 43.8 -> 16.8, two planes 20 rows 23.6 -> 20.5 (16 rows 19.9 -> 20.4).
    const size_t n_passes = (nb + (size_t)pl.pr.kc - 1) / (size_t)(pl.pr.kc ? pl.pr.kc : 1);
    const bool one_a8 = pl.cfg.planes == 1 && mode == TK_MODE_INT8;
    // (two passes stay: 5120 x 5120 x 3 planes, 16 rows 18.8 vs 22.7 us; float contract 5 tokens of K = 2560, one plane
    // 13.2 vs 15.1. Three passes at 16 rows only for one plane of int8 rows: 2560 x 6912 18.6 -> 16.8, two planes
    // 19.8 -> 20.4, float contract 4 tokens x two planes 19.5 -> 21.9)
    const bool passes = (n_passes >= 3 && (R >= 20 || one_a8)) || n_passes >= 4;
    if (ctx->decode_force == DECODE_AUTO && pl.skinny && variant == DECODE_KSPLIT &&
        (R > 32 || (R > 16 && one_a8) || (passes && R >= 16))) {
      pl.skinny = false;
      plan_gemm(&pl, 4u * (unsigned)ctx->info.compute_units, ctx->gemm_tiles);
    }
  }
  // A single decode call of few tokens is two short dependent launches, and the gap between them costs more than
  // either: the flow kernel then builds the operand rows itself, every workgroup for itself (256 threads, at most
  // two 16-byte pieces of a token per thread, straight-line loads: whole K blocks, aligned f32 or bf16 rows).
  // Every workgroup repeats the tokens' arithmetic (about 25 instructions per element under the float contract),
  // which the prep launch does once, so the form pays for very few tokens. Measured, back-to-back calls, two
  // launches -> one: K=2560 N=6912 one plane f32, int8 contract 1 / 2 / 4 tokens 8.4 -> 5.3 / 9.0 -> 7.1 /
  // 10.0 -> 10.8 us, float contract 9.5 -> 6.4 / 10.0 -> 10.0 / 11.4 -> 16.3 us; K=2048 N=8192 two planes bf16
  // 9.0 -> 5.6 and 9.7 -> 6.7 us for one token; K=6912 N=2560 10.3 -> 6.8 and 12.7 -> 8.2; the flow kernel on
  // K=5120 N=17408 three planes 20.4 -> 17.7 and 22.1 -> 19.1 for one token, nothing for two. Left to itself: one
  // token, or two under the int8 contract in the K-split kernel.
  const int fuse_limit = ctx->fuse_tokens >= 0 ? ctx->fuse_tokens : ((prep_kind == TK_PREP_A8 && variant == DECODE_KSPLIT) ? 2 : 1);
  // Both decode kernels of single launches have the form: the K-split kernel (its rows fit LDS in one pass) and the
  // flow kernel in its 16x16x64 form.
  // An RMSNorm in front (one token): the row crosses LDS once more for the canonical sum of squares (k floats and
  // 1 KiB behind the row constants).
  const size_t fuse_lds = 1024 + (norm ? k * 4 + 1024 : 0);
  const bool fuse_rows = pl.skinny && pl.cfg.rt == 1 && (prep_kind == TK_PREP_A8 || prep_kind == TK_PREP_DIGITS) &&
                         m <= (size_t)fuse_limit && nb * 16 <= 512 && k % 256 == 0 && ((uintptr_t)act & 15) == 0 &&
                         (act_dtype == TK_F32 || act_dtype == TK_BF16) &&
                         (!norm || (m == 1 && fuse_limit >= 1 && ((uintptr_t)norm->weight & 15) == 0));
  const bool fused_flow = fuse_rows && variant == DECODE_FLOW && !wide && !b3 && flow_lds + fuse_lds + 1024 <= 64 * 1024;
  // (the K-split kernel has one workgroup per output tile; in this form each repeats the tokens' prep, and beyond two
  // workgroups per CU they queue up behind each other and the repeats cost more than the launch saved -- gate,up of
  // hidden 2560, 864 tiles: 8.4 -> 10.4 us, 10.1 -> 13.1 us behind a norm; q,k,v, 240 tiles: 8.0 -> 5.6 and 9.6 -> 7.0
  // us. Larger launches therefore give a workgroup up to four consecutive tiles behind one prep.)
  const size_t fused_ksplit_lds = nb * 256 * R + fuse_lds + (size_t)4096 * pl.cfg.planes;  // rows, constants (+ norm scratch), reduction
  const unsigned fuse_tpw = (pl.cfg.grid + 2u * (unsigned)ctx->info.compute_units - 1) / (2u * (unsigned)ctx->info.compute_units);
  const bool fused_ksplit = fuse_rows && variant == DECODE_KSPLIT && (size_t)pl.pr.kc >= nb && fused_ksplit_lds + 1024 <= 64 * 1024 &&
                            fuse_tpw <= 4;
  const bool fused = fused_flow || fused_ksplit;
  // One plane under the int8 contract with whole 16-byte output pieces: the wide-tile prefill kernels.
  const size_t out_esz = out_dtype == TK_BF16 ? 2 : 4;
  const bool can_wide = !pl.skinny && pl.pr.planes == 1 && mode == TK_MODE_INT8 && (out_dtype == TK_F32 || out_dtype == TK_BF16) &&
                        !residual && (n * out_esz) % 16 == 0 && ((uintptr_t)out & 15) == 0;
  int form256 = 0;
  const bool pays256 = gemm256_pays(ctx, R, (size_t)pl.pr.n_tiles, &form256);
  const bool use256 = can_wide && (ctx->gemm_rows == 256 || (ctx->gemm_rows == 0 && pays256));
  if (use256) plan_gemm256(&pl);
  Workspace ws;
  TKCHK(take_workspace(ctx, static_ws, (size_t)pl.pr.rs * nb * 256, R, m, norm ? m * k * 4 : 0, &ws));

  TkPrep &pp = pl.prep;
  if (norm) {
    pp.norm_kind = norm->zero_centered ? 2 : 1;
    pp.norm_eps = norm->eps;
    pp.norm_w = norm->weight;
    pp.ynorm = ws.ynorm;
  }
  pp.act = act;
  pp.ap = ws.ap;
  pp.rowsum = ws.rowsum;
  pp.act_scale = ws.fscale;
  pp.aux = ws.aux;
  pp.exps = ws.exps;
  pp.flags = ws.flags;
  pp.k = k;
  pp.nb = nb;
  pp.R = R;
  pp.rs = (size_t)pl.pr.rs;
  pp.act_dtype = act_dtype;
  pp.m = (int)m;
  if (!fused) HIPCHK(tk_launch_prep(ctx->stream, prep_kind, &pp, nullptr, 0, 0, (unsigned)m));

  TkProblem &pr = pl.pr;
  pr.ap = pp.ap;
  pr.rowsum = pp.rowsum;
  pr.out = out;
  pr.residual = residual;
  if (prep_kind == TK_PREP_A8) {
    pr.act_scale = pp.act_scale;
    pr.aux = pp.aux;
    pr.flags = pp.flags;
    pr.raw_act = norm ? (const void *)pp.ynorm : act;  // the exact fallback re-quantizes the normalized row
    pr.raw_dtype = norm ? TK_F32 : act_dtype;
    if (fused && norm) {  // the kernel normalizes the raw row itself
      pr.raw_act = act;
      pr.raw_dtype = act_dtype;
      pr.norm_kind = pp.norm_kind;
      pr.norm_eps = pp.norm_eps;
      pr.norm_w = pp.norm_w;
    }
  } else if (prep_kind == TK_PREP_DIGITS) {
    pr.exps = pp.exps;
    pr.flags = pp.flags;
    pr.raw_act = act;
    pr.raw_dtype = act_dtype;
  } else {
    pr.act_scale = act_scale_in;
  }
  if (pl.skinny && variant == DECODE_FLOW) {
    TkLaunchCfg cfg = pl.cfg;
    cfg.grid = flow_groups;
    cfg.lds_bytes = flow_lds;
    cfg.waves = b3 ? tk_flow3_waves(pl.cfg.rt) : flow_waves(flow_lds, pl.cfg.rt, flow_sixteen(ctx, mode == TK_MODE_INT8, false, wide, b3, pl.cfg.planes, (size_t)pl.pr.n_tiles, flow_runs_per_wave(wide, b3, pl.cfg.planes, pl.cfg.rt, R)));
    cfg.ring = pick_flow_ring(ctx, &pr.nb, nullptr, 1, pl.cfg.rt, pr.R, flow_runs_per_wave(wide, b3, pl.cfg.planes, pl.cfg.rt, R), wide, cfg.waves, flow_lds, pl.cfg.planes);
    const size_t ztiles = flow_zero_plan(wide, b3, fused, cfg.planes, flow_lds,
                                         pr.zskip ? (size_t)cfg.waves * (size_t)flow_runs_per_wave(wide, b3, pl.cfg.planes, pl.cfg.rt, R) * (size_t)run_tiles : 0, nb);
    if (!ztiles) pr.zskip = 0;  // no room for the maps behind the rows (or another form of the kernel): plain loads
    flow_cfg_form(&cfg, wide, b3, flow_lds, R, ztiles, nb, mode == TK_MODE_INT8 && ctx->flow_swap && !fused);
    if (fused) {
      cfg.fused = 1;
      cfg.lds_bytes += fuse_lds;
      ctx->fused_calls++;
    }
    pr.run_tiles = run_tiles;
    pr.group_begin = 0;
    ctx->last_kernel = b3 ? "flow3" : (wide ? "flow32" : "flow");
    if (b3) HIPCHK(tk_launch_flow3(ctx->stream, &pr, nullptr, nullptr, cfg));
    else HIPCHK(tk_launch_flow(ctx->stream, &pr, nullptr, nullptr, cfg));
  } else if (pl.skinny && variant == DECODE_STREAM) {
    TkLaunchCfg cfg = pl.cfg;
    cfg.grid = pl.stream_groups;
    cfg.lds_bytes = pl.stream_lds;
    pr.kc = pl.stream_kc;
    pr.group_begin = 0;
    ctx->last_kernel = "stream";
    HIPCHK(tk_launch_stream(ctx->stream, &pr, nullptr, nullptr, cfg));
  } else if (pl.skinny) {
    if (fused) {
      pl.cfg.fused = 1;
      pl.cfg.lds_bytes = fused_ksplit_lds;
      pr.run_tiles = (int)(fuse_tpw ? fuse_tpw : 1);
      pl.cfg.grid = (pl.cfg.grid + (unsigned)pr.run_tiles - 1) / (unsigned)pr.run_tiles;
      ctx->fused_calls++;
    }
    ctx->last_kernel = "ksplit_decode";
    HIPCHK(tk_launch_skinny(ctx->stream, &pr, nullptr, 0, pl.cfg));
  } else {
    // One plane under the int8 contract with whole 16-byte output pieces: the 128 x 256 kernel moves a third
    // of the bytes per op through the CU's memory path (both operands shared through LDS).
    const bool can128 = can_wide;
    if (use256) {
      ctx->last_kernel = "gemm256";
      const hipError_t le = tk_launch_gemm256(ctx->stream, &pr, form256);
      if (le != hipSuccess) {
        return tk_fail(TK_ERR_BACKEND, "prefill kernel launch: %s", hipGetErrorString(le));
      }
      return TK_OK;
    }
    const size_t blocks128 = ((R + 127) / 128) * (((size_t)pr.n_tiles + 15) / 16);
    const bool want128 = ctx->gemm_rows == 128 || (ctx->gemm_rows == 0 && gemm128_pays(ctx, R, blocks128));
    if (can128 && want128) {
      plan_gemm128(&pl);
      ctx->last_kernel = "gemm128";
      HIPCHK(tk_launch_gemm128(ctx->stream, &pr));
      return TK_OK;
    }
    // A single launch with few workgroups is a latency chain over K per workgroup: cut K into slices.
    // The partial sums cost 4 bytes per accumulator and slice, so few slices: measured, call incl.
    // quantization, 64 tokens x 3 planes: 17408 -> 5120 (40 workgroups) 108 us unsplit, 72 / 56 / 54 / 72
    // with 2 / 4 / 6 / 8 slices; 5120 -> 5120 39 -> 30 us at 4; 5120 -> 1024 (8 workgroups) 39 -> 28 at 4;
    // 5120 -> 17408 (136 workgroups) is best left alone (42 us; 53 with 2 slices). Rule: split when the
    // launch has at most a third of the CUs in workgroups, into about three quarters of the CUs, 2..6
    // slices of at least two K blocks.
    const unsigned wgs = 8u * (unsigned)pr.sub_m * (unsigned)pr.sub_n;
    int ksn = 1;
    if (!static_ws && pr.planes <= 3 && nb >= 4) {
      if (ctx->gemm_ksplit >= 2) ksn = ctx->gemm_ksplit;
      else if (ctx->gemm_ksplit == 0 && wgs * 3 <= (unsigned)ctx->info.compute_units) {
        ksn = (int)((3u * (unsigned)ctx->info.compute_units / 4u) / wgs);
        ksn = ksn < 2 ? 2 : (ksn > 6 ? 6 : ksn);
      }
      if ((size_t)ksn > nb / 2) ksn = (int)(nb / 2);  // every slice holds at least two K blocks (the kernel relies on it)
    }
    if (ksn > 1) {
      const size_t tiles = (size_t)pr.grid_m * (size_t)pr.grid_n;
      const size_t regs = (size_t)32 * (size_t)pr.planes * (pr.planes == 1 ? (pl.cfg.gemm_nt == 2 ? 1 : 2) : 1);  // 2 * NP * 16
      const bool fresh = tiles * 4 > ctx->kcount.cap;
      TKCHK(ensure(ctx, ctx->kpart, tiles * (size_t)ksn * regs * 256 * 4));
      TKCHK(ensure(ctx, ctx->kcount, tiles * 4));
      if (fresh || ctx->kcount_stale) HIPCHK(hipMemsetAsync(ctx->kcount.p, 0, ctx->kcount.cap, ctx->stream));  // the kernel leaves it zero
      ctx->kcount_stale = false;
      pr.ksplit = ksn;
      pr.kpart = (int32_t *)ctx->kpart.p;
      pr.kcount = (int *)ctx->kcount.p;
    }
    pl.cfg.gemm_two_by_two = ctx->gemm_two_by_two;
    ctx->last_kernel = ksn > 1 ? "gemm64_ksplit" : "gemm64";
    const hipError_t le = tk_launch_gemm(ctx->stream, &pr, nullptr, nullptr, pl.cfg);
    if (le != hipSuccess) {
      if (ksn > 1) ctx->kcount_stale = true;  // counters of a launch that did not complete may be non-zero
      return tk_fail(TK_ERR_BACKEND, "prefill kernel launch: %s", hipGetErrorString(le));
    }
  }
  return TK_OK;
}

static int check_act_dtype(int dt) {
  if (dt != TK_F32 && dt != TK_BF16) return tk_fail(TK_ERR_INVALID_INPUT, "activation dtype %d - use f32 or bf16", dt);
  return TK_OK;
}
static int check_out_dtype(int dt, bool allow_i32) {
  if (dt == TK_F32 || dt == TK_BF16 || (allow_i32 && dt == TK_I32)) return TK_OK;
  return tk_fail(TK_ERR_INVALID_INPUT, "output dtype %d not supported here", dt);
}

extern "C" int tk_linear_float(tk_ctx *ctx, const tk_linear_desc *layer, const void *act, int act_dtype, size_t m,
                               void *out, int out_dtype) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "null context");
  TKCHK(check_act_dtype(act_dtype));
  TKCHK(check_out_dtype(out_dtype, false));
  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  return run_linear(ctx, layer, TK_MODE_DIGITS, TK_PREP_DIGITS, act, act_dtype, nullptr, m, out, out_dtype);
}

extern "C" int tk_linear_a8(tk_ctx *ctx, const tk_linear_desc *layer, const void *act, int act_dtype, size_t m,
                            void *out, int out_dtype) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "null context");
  TKCHK(check_act_dtype(act_dtype));
  TKCHK(check_out_dtype(out_dtype, false));
  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  return run_linear(ctx, layer, TK_MODE_INT8, TK_PREP_A8, act, act_dtype, nullptr, m, out, out_dtype);
}

// tk_linear_a8 without any allocation: the workspace is the static device scratch. Calls that
// overlap on one GPU (other streams, other contexts of the same device, other threads) share that
// array and race; every element a kernel reads is written by the prep launch of the same call first,
// so nothing of an earlier call's contents needs clearing.
extern "C" int tk_linear_a8_noalloc(tk_ctx *ctx, const tk_linear_desc *layer, const void *act, int act_dtype, size_t m,
                                    void *out, int out_dtype) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "null context");
  TKCHK(check_act_dtype(act_dtype));
  TKCHK(check_out_dtype(out_dtype, false));
  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  return run_linear(ctx, layer, TK_MODE_INT8, TK_PREP_A8, act, act_dtype, nullptr, m, out, out_dtype, nullptr, true);
}

extern "C" int tk_linear_rmsnorm_a8(tk_ctx *ctx, const tk_linear_desc *layer, const void *x, int x_dtype,
                                    const tk_rmsnorm *norm, size_t m, void *out, int out_dtype) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "null context");
  TKCHK(check_act_dtype(x_dtype));
  TKCHK(check_out_dtype(out_dtype, false));
  TKCHK(check_norm(norm));
  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  return run_linear(ctx, layer, TK_MODE_INT8, TK_PREP_A8, x, x_dtype, nullptr, m, out, out_dtype, norm);
}

// Block-scale additive planes on float activations. seq != 0 forces the reference-order kernel.
static int run_salt(tk_ctx *ctx, const tk_salt_desc *layer, const void *act, int act_dtype, size_t m, void *out,
                    int out_dtype, bool seq) {
  if (!layer) return tk_fail(TK_ERR_INVALID_INPUT, "null layer descriptor");
  if (layer->n_planes < 1 || layer->n_planes > TK_MAX_PLANES)
    return tk_fail(TK_ERR_INVALID_INPUT, "n_planes=%d - use 1..%d", layer->n_planes, TK_MAX_PLANES);
  for (int p = 0; p < layer->n_planes; ++p) {
    const tk_weights *w = layer->planes[p];
    if (!w) return tk_fail(TK_ERR_INVALID_INPUT, "plane %d: null weights handle", p);
    if (w->ctx != ctx) return tk_fail(TK_ERR_INVALID_INPUT, "plane %d: buffer belongs to another context", p);
    if (!w->block_scales)
      return tk_fail(TK_ERR_INVALID_INPUT, "plane %d was uploaded without its block scales (tk_upload_weights_scaled)", p);
    if (p && (w->n != layer->planes[0]->n || w->k != layer->planes[0]->k))
      return tk_fail(TK_ERR_INVALID_INPUT, "plane %d is [%zu,%zu] but plane 0 is [%zu,%zu]", p, w->n, w->k,
                     layer->planes[0]->n, layer->planes[0]->k);
    if (w->invalid_row >= 0)
      return tk_fail(TK_ERR_BACKEND, "unpack row %ld: decoded value 2 outside ternary range", w->invalid_row);
  }
  const size_t n = layer->planes[0]->n, k = layer->planes[0]->k, nb = num_blocks(k);
  if (m == 0 || n == 0) return TK_OK;
  if (!act || !out) return tk_fail(TK_ERR_INVALID_INPUT, "null activation or output pointer");
  size_t total;
  if (__builtin_mul_overflow(m, n, &total) || total > (size_t)INT32_MAX || m * 4 > (size_t)INT32_MAX)
    return tk_fail(TK_ERR_INVALID_INPUT, "shape m=%zu n=%zu k=%zu exceeds the kernels' int index range", m, n, k);

  TkProblem pr;
  memset(&pr, 0, sizeof pr);
  for (int p = 0; p < layer->n_planes; ++p) {
    pr.codes[p] = layer->planes[p]->codes;
    pr.bscale[p] = layer->planes[p]->block_scales;
  }
  const size_t R = 4 * m;
  pr.n = (int)n;
  pr.k = (int)k;
  pr.nb = (int)nb;
  pr.R = (int)R;
  pr.rs = (int)R;
  pr.M = (int)m;
  pr.mode = TK_MODE_DIGITS;
  pr.out_dtype = out_dtype;
  pr.planes = layer->n_planes;
  pr.n_tiles = (int)((n + 15) / 16);
  pr.raw_act = act;
  pr.raw_dtype = act_dtype;
  pr.out = out;
  // More than 16 tokens: slices of 16 go through the matrix-core form one after the other (each
  // streams the planes again; a block-scale form of the prefill kernel does not exist yet).
  if (!seq && m > 16 && nb * 256 * 64 + nb * 64 * 4 <= kLdsFlowMax) {
    const size_t asz = act_dtype == TK_BF16 ? 2 : 4, osz = out_dtype == TK_BF16 ? 2 : 4;
    for (size_t m0 = 0; m0 < m; m0 += 16) {
      const size_t mc = m - m0 < 16 ? m - m0 : 16;
      TKCHK(run_salt(ctx, layer, (const uint8_t *)act + m0 * k * asz, act_dtype, mc, (uint8_t *)out + m0 * n * osz,
                     out_dtype, false));
    }
    return TK_OK;
  }
  const size_t lds = nb * 256 * R + nb * R * 4;  // operand rows + their per-block sums
  if (seq || R > 64 || lds > kLdsFlowMax) {
    HIPCHK(tk_launch_salt_seq(ctx->stream, &pr));
    return TK_OK;
  }
  TKCHK(ensure(ctx, ctx->ap, R * nb * 256));
  TKCHK(ensure(ctx, ctx->rowsum, R * 4));
  TKCHK(ensure(ctx, ctx->exps, m * 4));
  TKCHK(ensure(ctx, ctx->flags, m * 4));
  TKCHK(ensure(ctx, ctx->blocksum, nb * R * 4));
  TkPrep pp = {};
  pp.act = act;
  pp.ap = (int8_t *)ctx->ap.p;
  pp.rowsum = (int32_t *)ctx->rowsum.p;
  pp.exps = (int32_t *)ctx->exps.p;
  pp.flags = (uint32_t *)ctx->flags.p;
  pp.blocksum = (int32_t *)ctx->blocksum.p;
  pp.k = k;
  pp.nb = nb;
  pp.R = R;
  pp.rs = R;
  pp.act_dtype = act_dtype;
  pp.m = (int)m;
  HIPCHK(tk_launch_prep(ctx->stream, TK_PREP_DIGITS, &pp, nullptr, 0, 0, (unsigned)m));
  pr.ap = pp.ap;
  pr.rowsum = pp.rowsum;
  pr.exps = pp.exps;
  pr.flags = pp.flags;
  pr.blocksum = pp.blocksum;
  TkLaunchCfg cfg = {};
  cfg.planes = layer->n_planes;
  cfg.rt = R <= 16 ? 1 : (R <= 32 ? 2 : 4);
  cfg.lds_bytes = lds;
  cfg.waves = flow_waves(lds, 1);  // (the 64 KiB limit at every row count: this kernel was tuned with it)
  // tiles per run: as the plain flow kernel (2 / 4 / 8 for one / two / four row tiles), fewer when
  // the launch would not give every CU its workgroups
  int s_tiles = cfg.rt == 1 ? 2 : (cfg.rt == 2 ? 4 : 8);
  if (ctx->flow_run_tiles > 0) s_tiles = ctx->flow_run_tiles;
  const unsigned per_cu = cfg.waves >= 8 ? 1u : 2u;
  while (s_tiles > 1 && (unsigned)pr.n_tiles / ((unsigned)cfg.waves * (unsigned)s_tiles) < per_cu * (unsigned)ctx->info.compute_units)
    --s_tiles;
  pr.run_tiles = s_tiles;
  const unsigned per_wg = (unsigned)cfg.waves * (unsigned)s_tiles;
  cfg.grid = ((unsigned)pr.n_tiles + per_wg - 1) / per_wg;
  HIPCHK(tk_launch_salt_flow(ctx->stream, &pr, cfg));
  return TK_OK;
}

extern "C" int tk_linear_salt(tk_ctx *ctx, const tk_salt_desc *layer, const void *act, int act_dtype, size_t m,
                              void *out, int out_dtype) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "null context");
  TKCHK(check_act_dtype(act_dtype));
  TKCHK(check_out_dtype(out_dtype, false));
  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  return run_salt(ctx, layer, act, act_dtype, m, out, out_dtype, false);
}

extern "C" int tk_linear_salt_seq(tk_ctx *ctx, const tk_salt_desc *layer, const void *act, int act_dtype, size_t m,
                                  void *out, int out_dtype) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "null context");
  TKCHK(check_act_dtype(act_dtype));
  TKCHK(check_out_dtype(out_dtype, false));
  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  return run_salt(ctx, layer, act, act_dtype, m, out, out_dtype, true);
}

// A SALT tensor (n encoded rows back to back) -> block-scale planes. The rows are walked with the reader's own
// length function, unpacked (sparse residuals expanded) into one row-major TQ2_0 tensor per plane, and
// each plane uploaded with its block scales kept.
extern "C" int tk_upload_salt_rows(tk_ctx *ctx, const uint8_t *bytes, size_t len, size_t n, size_t k, size_t max_planes,
                                   tk_weights **planes_out, int *n_planes) {
  if (!ctx || !planes_out || !n_planes || (!bytes && len)) return tk_fail(TK_ERR_INVALID_INPUT, "tk_upload_salt_rows: null pointer");
  *n_planes = 0;
  const size_t row_bytes = num_blocks(k) * 66;
  size_t plane_len;
  if (__builtin_mul_overflow(n, row_bytes, &plane_len)) return tk_fail(TK_ERR_INVALID_INPUT, "packed weight byte count overflows");
  // the rows must fit the bytes given before anything is sized from n: a row is at least its header
  if (n > len / 10 + 1 && n) return tk_fail_mismatch(n * 10, len);
  std::vector<std::vector<uint8_t>> planes;
  std::vector<uint8_t> row_planes;
  size_t off = 0;
  try {
    for (size_t r = 0; r < n; ++r) {
      size_t rl = 0, rk = 0, rp = 0;
      TKCHK(tk_salt_row_len(bytes + off, len - off, &rl));
      TKCHK(tk_salt_row_info(bytes + off, rl, &rk, &rp, nullptr));
      if (rk != k) return tk_fail_mismatch(k, rk);
      const size_t keep = rp < max_planes ? rp : max_planes;
      if (keep > (size_t)TK_MAX_PLANES)
        return tk_fail(TK_ERR_UNSUPPORTED_FORMAT, "SALT row %zu keeps %zu planes; the kernels take at most %d", r, keep, TK_MAX_PLANES);
      row_planes.resize(keep * row_bytes);
      size_t got_k = 0, got_p = 0;
      TKCHK(tk_salt_row_unpack(bytes + off, rl, max_planes, row_planes.data(), row_planes.size(), &got_k, &got_p));
      while (planes.size() < got_p) {
        // a plane no earlier row had: all-zero trits with scale 0 for those rows
        std::vector<uint8_t> fresh(plane_len);
        for (size_t b = 0; b < plane_len; b += 66) {
          memset(fresh.data() + b, 0x55, 64);
          fresh[b + 64] = fresh[b + 65] = 0;
        }
        planes.push_back(std::move(fresh));
      }
      for (size_t p = 0; p < got_p; ++p) memcpy(planes[p].data() + r * row_bytes, row_planes.data() + p * row_bytes, row_bytes);
      off += rl;
    }
  } catch (const std::exception &) {
    return tk_fail(TK_ERR_BACKEND, "tk_upload_salt_rows: host allocation failed");
  }
  if (off != len) return tk_fail(TK_ERR_INVALID_INPUT, "%zu bytes follow the last of the %zu SALT rows", len - off, n);
  for (size_t p = 0; p < planes.size(); ++p) {
    int rc = tk_upload_weights_scaled(ctx, planes[p].data(), plane_len, n, k, &planes_out[p]);
    if (rc) {
      for (size_t q = 0; q < p; ++q) {
        tk_free_weights(planes_out[q]);
        planes_out[q] = nullptr;
      }
      return rc;
    }
  }
  *n_planes = (int)planes.size();
  return TK_OK;
}

// ------------------------------------------------------------------------------------------
// SALT V2
// ------------------------------------------------------------------------------------------
struct tk_salt_v2 {
  tk_ctx *ctx;
  void *payload, *scales, *tile_begin;
  TkSaltV2 dev;
};

extern "C" int tk_salt_v2_upload(tk_ctx *ctx, int codec, size_t scale_group, const uint8_t *payload, size_t payload_len,
                                 const uint16_t *scales_f16, size_t scale_count, const uint8_t *plane_counts, size_t tiles,
                                 size_t n, size_t k, tk_salt_v2 **out) {
  if (!ctx || !out) return tk_fail(TK_ERR_INVALID_INPUT, "tk_salt_v2_upload: null pointer");
  *out = nullptr;
  if (codec != TK_SALT_V2_D2 && codec != TK_SALT_V2_B3 && codec != TK_SALT_V2_S34)
    return tk_fail(TK_ERR_UNSUPPORTED_FORMAT, "SALT V2 codec %d", codec);
  if (scale_group != 128 && scale_group != 64)
    return tk_fail(TK_ERR_UNSUPPORTED_FORMAT, "SALT V2 scale group of %zu coefficients - the format defines 128 and 64", scale_group);
  size_t total;
  if (__builtin_mul_overflow(n, k, &total) || n > (size_t)UINT32_MAX || k > (size_t)UINT32_MAX)
    return tk_fail(TK_ERR_INVALID_INPUT, "SALT V2 shape n=%zu k=%zu exceeds the kernels' index range", n, k);
  if (tiles != (total + 255) / 256) return tk_fail_mismatch((total + 255) / 256, tiles);
  if ((!payload && payload_len) || (!scales_f16 && scale_count) || (!plane_counts && tiles))
    return tk_fail(TK_ERR_INVALID_INPUT, "tk_salt_v2_upload: null pointer");
  if (tk_salt_v2_lds_bytes(k, scale_group) > kLdsFlowMax)
    return tk_fail(TK_ERR_INVALID_INPUT, "SALT V2 rows of %zu columns exceed what the forward kernel stages", k);
  // running plane index per tile; every plane decoded once (a non-canonical payload is rejected here), and
  // the payload and the scales must be exactly as long as the tiles say
  std::vector<uint32_t> begin;
  std::vector<int8_t> scratch(256);
  try {
    begin.resize(tiles + 1);
  } catch (const std::exception &) {
    return tk_fail(TK_ERR_BACKEND, "tk_salt_v2_upload: host allocation failed");
  }
  size_t full_bytes = 0, planes = 0, pay = 0, sc = 0;
  TKCHK(tk_salt_v2_payload_bytes(codec, 256, &full_bytes));
  const size_t full_groups = 256 / scale_group;
  for (size_t t = 0; t < tiles; ++t) {
    const size_t ln = total - t * 256 < 256 ? total - t * 256 : 256;
    if (plane_counts[t] < 1 || plane_counts[t] > 3)
      return tk_fail(TK_ERR_INVALID_INPUT, "SALT V2 tile %zu has %u planes - one to three", t, (unsigned)plane_counts[t]);
    if (planes > (size_t)UINT32_MAX - 3) return tk_fail(TK_ERR_INVALID_INPUT, "SALT V2 plane count exceeds the index range");
    begin[t] = (uint32_t)planes;
    size_t cur_bytes = 0;
    TKCHK(tk_salt_v2_payload_bytes(codec, ln, &cur_bytes));
    const size_t cur_groups = (ln + scale_group - 1) / scale_group;
    for (unsigned j = 0; j < plane_counts[t]; ++j) {
      const size_t base = planes * full_bytes + (size_t)j * cur_bytes;
      if (base + cur_bytes > payload_len) return tk_fail_mismatch(base + cur_bytes, payload_len);
      TKCHK(tk_salt_v2_unpack(codec, payload + base, cur_bytes, ln, scratch.data()));
      pay = base + cur_bytes;
      sc = planes * full_groups + (size_t)j * cur_groups + cur_groups;
    }
    planes += plane_counts[t];
  }
  begin[tiles] = (uint32_t)planes;
  if (pay != payload_len) return tk_fail_mismatch(pay, payload_len);
  if (sc != scale_count) return tk_fail_mismatch(sc, scale_count);

  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  tk_salt_v2 *w = new (std::nothrow) tk_salt_v2();
  if (!w) return tk_fail(TK_ERR_BACKEND, "tk_salt_v2_upload: host allocation failed");
  w->ctx = ctx;
  w->payload = w->scales = w->tile_begin = nullptr;
  int rc = dev_malloc(payload_len, &w->payload);
  if (!rc) rc = dev_malloc(scale_count * 2, &w->scales);
  if (!rc) rc = dev_malloc((tiles + 1) * 4, &w->tile_begin);
  hipError_t e = hipSuccess;
  if (!rc && payload_len) e = hipMemcpyAsync(w->payload, payload, payload_len, hipMemcpyHostToDevice, ctx->stream);
  if (!rc && e == hipSuccess && scale_count) e = hipMemcpyAsync(w->scales, scales_f16, scale_count * 2, hipMemcpyHostToDevice, ctx->stream);
  if (!rc && e == hipSuccess) e = hipMemcpyAsync(w->tile_begin, begin.data(), (tiles + 1) * 4, hipMemcpyHostToDevice, ctx->stream);
  if (!rc && e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
  if (rc || e != hipSuccess) {
    if (w->payload) (void)hipFree(w->payload);
    if (w->scales) (void)hipFree(w->scales);
    if (w->tile_begin) (void)hipFree(w->tile_begin);
    delete w;
    return rc ? rc : tk_fail(TK_ERR_BACKEND, "tk_salt_v2_upload: %s", hipGetErrorString(e));
  }
  w->dev.payload = (const uint8_t *)w->payload;
  w->dev.scales = (const uint16_t *)w->scales;
  w->dev.tile_begin = (const uint32_t *)w->tile_begin;
  w->dev.n = (unsigned)n;
  w->dev.k = (unsigned)k;
  w->dev.codec = (unsigned)codec;
  w->dev.group = (unsigned)scale_group;
  w->dev.tiles = (unsigned)tiles;
  w->dev.total = total;
  ctx->refs.fetch_add(1);
  *out = w;
  return TK_OK;
}

extern "C" void tk_salt_v2_free(tk_salt_v2 *t) {
  if (!t) return;
  tk_ctx *ctx = t->ctx;
  {
    std::lock_guard<std::mutex> lk(ctx->mu);
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipFree(t->payload);
    (void)hipFree(t->scales);
    (void)hipFree(t->tile_begin);
    delete t;
  }
  ctx_release(ctx);
}

extern "C" int tk_salt_v2_forward(tk_ctx *ctx, const tk_salt_v2 *t, const float *act, size_t m, float *out) {
  if (!ctx || !t) return tk_fail(TK_ERR_INVALID_INPUT, "tk_salt_v2_forward: null pointer");
  if (t->ctx != ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tensor belongs to another context");
  if (m == 0 || t->dev.n == 0) return TK_OK;
  if (!act || !out) return tk_fail(TK_ERR_INVALID_INPUT, "null activation or output pointer");
  if (m > (size_t)65535 * TK_SALT_V2_TOKENS) return tk_fail(TK_ERR_INVALID_INPUT, "m=%zu - at most %d tokens per call", m, 65535 * TK_SALT_V2_TOKENS);
  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  const size_t bytes = m * (size_t)t->dev.n * sizeof(float);
  // the lane-per-row form keeps the terms of up to `chunk` tokens at a time (at most 256 MiB of them)
  const size_t per_token = tk_salt_v2_term_floats(t->dev) * sizeof(float);
  size_t chunk = 0;
  if (per_token && per_token <= ((size_t)256 << 20)) {
    chunk = ((size_t)256 << 20) / per_token;
    if (chunk > m) chunk = m;
  }
  const size_t out_bytes = (bytes + 255) & ~(size_t)255;
  TKCHK(ensure(ctx, ctx->tmp, out_bytes + chunk * per_token));
  unsigned flag = 0;
  HIPCHK(hipMemsetAsync(ctx->d_count, 0, sizeof(unsigned), ctx->stream));
  HIPCHK(tk_launch_salt_v2_forward(ctx->stream, t->dev, act, m, (float *)ctx->tmp.p, ctx->d_count,
                                   chunk ? (float *)((uint8_t *)ctx->tmp.p + out_bytes) : nullptr, chunk));
  // the device commits the results only when the flag stayed clear: one synchronization per call
  HIPCHK(tk_launch_salt_v2_commit(ctx->stream, (const float *)ctx->tmp.p, out, m * (size_t)t->dev.n, ctx->d_count));
  HIPCHK(hipMemcpyAsync(&flag, ctx->d_count, sizeof flag, hipMemcpyDeviceToHost, ctx->stream));
  HIPCHK(hipStreamSynchronize(ctx->stream));
  if (flag) return tk_fail(TK_ERR_INVALID_INPUT, "SALT V2 forward: a non-finite activation or result; the output was not written");
  return TK_OK;
}

extern "C" int tk_salt_v2_gather_rows(tk_ctx *ctx, const tk_salt_v2 *t, const uint32_t *rows, size_t count, float *out) {
  if (!ctx || !t) return tk_fail(TK_ERR_INVALID_INPUT, "tk_salt_v2_gather_rows: null pointer");
  if (t->ctx != ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tensor belongs to another context");
  if (count == 0 || t->dev.k == 0) return TK_OK;
  if (!rows || !out) return tk_fail(TK_ERR_INVALID_INPUT, "null row list or output pointer");
  for (size_t i = 0; i < count; ++i)
    if (rows[i] >= t->dev.n) return tk_fail(TK_ERR_INVALID_INPUT, "row %u of a matrix of %u rows", rows[i], t->dev.n);
  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  TKCHK(ensure(ctx, ctx->tmp, count * 4));
  HIPCHK(hipMemcpyAsync(ctx->tmp.p, rows, count * 4, hipMemcpyHostToDevice, ctx->stream));
  HIPCHK(tk_launch_salt_v2_gather(ctx->stream, t->dev, (const uint32_t *)ctx->tmp.p, count, out));
  HIPCHK(hipStreamSynchronize(ctx->stream));
  return TK_OK;
}

extern "C" int tk_linear_i8(tk_ctx *ctx, const tk_linear_desc *layer, const int8_t *q, const float *act_scale,
                            size_t m, void *out, int out_dtype) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "null context");
  TKCHK(check_out_dtype(out_dtype, true));
  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  return run_linear(ctx, layer, TK_MODE_INT8, TK_PREP_I8, q, TK_I8, act_scale, m, out, out_dtype);
}

// out = residual + linear(act): the fused residual-add epilogue of the reference's decode kernels
// (crates/tritium-cuda/kernels/tq2_0_add.cu:577-637,856-913)
extern "C" int tk_linear_a8_residual(tk_ctx *ctx, const tk_linear_desc *layer, const void *act, int act_dtype, size_t m,
                                     const void *residual, void *out, int out_dtype) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "null context");
  TKCHK(check_act_dtype(act_dtype));
  TKCHK(check_out_dtype(out_dtype, false));
  if (!residual && m && layer && layer->n_planes > 0 && layer->planes[0] && layer->planes[0]->n)
    return tk_fail(TK_ERR_INVALID_INPUT, "null residual pointer");
  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  return run_linear(ctx, layer, TK_MODE_INT8, TK_PREP_A8, act, act_dtype, nullptr, m, out, out_dtype, nullptr, false, residual);
}

extern "C" int tk_linear_i8_residual(tk_ctx *ctx, const tk_linear_desc *layer, const int8_t *q, const float *act_scale,
                                     size_t m, const void *residual, void *out, int out_dtype) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "null context");
  TKCHK(check_out_dtype(out_dtype, false));
  if (!residual && m && layer && layer->n_planes > 0 && layer->planes[0] && layer->planes[0]->n)
    return tk_fail(TK_ERR_INVALID_INPUT, "null residual pointer");
  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  return run_linear(ctx, layer, TK_MODE_INT8, TK_PREP_I8, q, TK_I8, act_scale, m, out, out_dtype, nullptr, false, residual);
}

extern "C" int tk_linear_float_seq(tk_ctx *ctx, const tk_linear_desc *layer, const void *act, int act_dtype, size_t m,
                                   void *out, int out_dtype) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "null context");
  TKCHK(check_act_dtype(act_dtype));
  TKCHK(check_out_dtype(out_dtype, false));
  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  size_t n, k;
  TKCHK(validate_layer(ctx, layer, &n, &k));
  if (m == 0 || n == 0) return TK_OK;
  if (!act || !out) return tk_fail(TK_ERR_INVALID_INPUT, "null activation or output pointer");
  size_t total;
  if (__builtin_mul_overflow(m, n, &total) || total > (size_t)INT32_MAX)
    return tk_fail(TK_ERR_INVALID_INPUT, "shape m=%zu n=%zu exceeds the kernels' int index range", m, n);
  Plan pl;
  plan_shape(ctx, layer, n, k, m, TK_MODE_DIGITS, out_dtype, &pl);
  pl.pr.raw_act = act;
  pl.pr.raw_dtype = act_dtype;
  pl.pr.out = out;
  HIPCHK(tk_launch_seq(ctx->stream, &pl.pr));
  return TK_OK;
}

static int act_quant(tk_ctx *ctx, const void *act, int act_dtype, const tk_rmsnorm *norm, size_t m, size_t k,
                     int8_t *q, float *act_scale, uint32_t *nonfinite_rows) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "null context");
  TKCHK(check_act_dtype(act_dtype));
  if (norm) TKCHK(check_norm(norm));
  if (m == 0) return TK_OK;
  if ((!act && k) || (!q && k) || !act_scale) return tk_fail(TK_ERR_INVALID_INPUT, "activation quantization: null pointer");
  if (m > (size_t)INT32_MAX || k > (size_t)INT32_MAX - 256)
    return tk_fail(TK_ERR_INVALID_INPUT, "shape m=%zu k=%zu exceeds the kernels' int index range", m, k);
  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  TkPrep pp = {};
  pp.act = act;
  pp.act_scale = act_scale;
  pp.flags = nonfinite_rows;
  pp.q_rowmajor = q;
  pp.k = k;
  pp.nb = num_blocks(k);
  pp.R = m;
  pp.rs = m;
  pp.act_dtype = act_dtype;
  pp.m = (int)m;
  if (norm) {
    pp.norm_kind = norm->zero_centered ? 2 : 1;
    pp.norm_eps = norm->eps;
    pp.norm_w = norm->weight;
  }
  HIPCHK(tk_launch_prep(ctx->stream, TK_PREP_A8, &pp, nullptr, 0, 0, (unsigned)m));
  return TK_OK;
}

extern "C" int tk_act_quant_i8(tk_ctx *ctx, const void *act, int act_dtype, size_t m, size_t k, int8_t *q,
                               float *act_scale, uint32_t *nonfinite_rows) {
  return act_quant(ctx, act, act_dtype, nullptr, m, k, q, act_scale, nonfinite_rows);
}

extern "C" int tk_rmsnorm_quant_i8(tk_ctx *ctx, const void *x, int x_dtype, const tk_rmsnorm *norm, size_t m, size_t k,
                                   int8_t *q, float *act_scale, uint32_t *nonfinite_rows) {
  if (!norm) return tk_fail(TK_ERR_INVALID_INPUT, "null RMSNorm weight");
  return act_quant(ctx, x, x_dtype, norm, m, k, q, act_scale, nonfinite_rows);
}

// ------------------------------------------------------------------------------------------
// trait-shaped host-slice entry points
// ------------------------------------------------------------------------------------------

static int host_call(tk_ctx *ctx, bool a8, const float *act, size_t act_len, const tk_weights *weights,
                     const float *scales, size_t scales_len, size_t m, size_t n, size_t k, int format, float *out,
                     size_t out_len) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "null context");
  if (!weights) return tk_fail(TK_ERR_INVALID_INPUT, "buffer is not a tritium-mi355x buffer");
  if (weights->ctx != ctx) return tk_fail(TK_ERR_INVALID_INPUT, "buffer belongs to another context");
  const bool identity_ok = weights->n == n && weights->k == k && weights->format == format;
  if (a8) {
    // the default fused path validates operand lengths first (crates/tritium-spec/src/lib.rs:275-292)
    if (act_len != m * k) return tk_fail_mismatch(m * k, act_len);
    if (out_len != m * n) return tk_fail_mismatch(m * n, out_len);
    if (scales_len != n) return tk_fail_mismatch(n, scales_len);
  }
  if (!fmt_block_bytes(format)) return tk_fail(TK_ERR_UNSUPPORTED_FORMAT, "unsupported ternary format: %d", format);
  if (!identity_ok)  // crates/tritium-cpu/src/lib.rs:123-135
    return tk_fail(TK_ERR_INVALID_INPUT, "buffer identity N=%zu K=%zu format=%d does not match N=%zu K=%zu format=%d",
                   weights->n, weights->k, weights->format, n, k, format);
  if (act_len != m * k) return tk_fail_mismatch(m * k, act_len);      // crates/tritium-cpu/src/lib.rs:319-324
  if (scales_len != n) return tk_fail_mismatch(n, scales_len);        // :325-330
  if (out_len != m * n) return tk_fail_mismatch(m * n, out_len);      // :331-336
  if (weights->invalid_row >= 0)
    return tk_fail(TK_ERR_BACKEND, "unpack row %ld: decoded value 2 outside ternary range", weights->invalid_row);
  if (m == 0 || n == 0) return TK_OK;
  if ((!act && act_len) || !scales || !out) return tk_fail(TK_ERR_INVALID_INPUT, "null operand pointer");

  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  size_t macs;
  const bool tiny = !__builtin_mul_overflow(m * n, k, &macs) && macs <= ctx->exact_max_macs;
  // Small calls (decode): the operands go through one pinned host block. A copy kernel brings the activation and the
  // scales to the device in one launch (so whatever reads them more than once reads device memory) and the kernels
  // write the output into the block themselves: two memcpy on the host, the launches and one synchronization in place
  // of four copy-engine transfers from and to pageable memory, which cost ~10 us each whatever their size.
  auto al = [](size_t b) { return (b + 255) & ~(size_t)255; };
  const size_t a_b = al(act_len * 4), s_b = al(n * 4), o_b = al(out_len * 4);
  if (a_b + s_b + o_b <= ctx->host_direct_bytes && (a8 || !tiny)) {
    if (a_b + s_b + o_b > ctx->pin_cap) {
      if (ctx->pin) {
        HIPCHK(hipStreamSynchronize(ctx->stream));
        (void)hipHostFree(ctx->pin);
        ctx->pin = nullptr;
        ctx->pin_cap = 0;
      }
      const size_t want = a_b + s_b + o_b + (a_b + s_b + o_b) / 4 + 4096;
      if (hipHostMalloc(&ctx->pin, want, hipHostMallocDefault) == hipSuccess) ctx->pin_cap = want;
      else { (void)hipGetLastError(); ctx->pin = nullptr; }  // no pinned memory to be had: the copies below
    }
    if (ctx->pin) {
      uint8_t *pa = (uint8_t *)ctx->pin, *ps = pa + a_b, *po = ps + s_b;
      memcpy(pa, act, act_len * 4);
      memcpy(ps, scales, n * 4);
      TKCHK(ensure(ctx, ctx->h_act, a_b + s_b));
      HIPCHK(tk_launch_copy(ctx->stream, ctx->h_act.p, pa, a_b + s_b));
      tk_linear_desc layer = {};
      layer.planes[0] = weights;
      layer.scales[0] = (const float *)((const uint8_t *)ctx->h_act.p + a_b);
      layer.n_planes = 1;
      TKCHK(run_linear(ctx, &layer, a8 ? TK_MODE_INT8 : TK_MODE_DIGITS, a8 ? TK_PREP_A8 : TK_PREP_DIGITS, ctx->h_act.p, TK_F32,
                       nullptr, m, po, TK_F32));
      HIPCHK(hipStreamSynchronize(ctx->stream));
      memcpy(out, po, out_len * 4);
      return TK_OK;
    }
  }
  TKCHK(ensure(ctx, ctx->h_act, act_len * 4));
  TKCHK(ensure(ctx, ctx->h_scales, n * 4));
  TKCHK(ensure(ctx, ctx->h_out, out_len * 4));
  if (act_len) HIPCHK(hipMemcpyAsync(ctx->h_act.p, act, act_len * 4, hipMemcpyHostToDevice, ctx->stream));
  HIPCHK(hipMemcpyAsync(ctx->h_scales.p, scales, n * 4, hipMemcpyHostToDevice, ctx->stream));
  tk_linear_desc layer = {};
  layer.planes[0] = weights;
  layer.scales[0] = (const float *)ctx->h_scales.p;
  layer.n_planes = 1;
  if (a8) {
    TKCHK(run_linear(ctx, &layer, TK_MODE_INT8, TK_PREP_A8, ctx->h_act.p, TK_F32, nullptr, m, ctx->h_out.p, TK_F32));
  } else if (tiny) {
    // Small float problems are latency-bound either way: run them in the reference's own summation
    // order, so the result is bit-identical to the CPU backend (crates/tritium-core/src/reference.rs:42-51).
    Plan pl;
    plan_shape(ctx, &layer, n, k, m, TK_MODE_DIGITS, TK_F32, &pl);
    pl.pr.raw_act = ctx->h_act.p;
    pl.pr.raw_dtype = TK_F32;
    pl.pr.out = ctx->h_out.p;
    HIPCHK(tk_launch_seq(ctx->stream, &pl.pr));
  } else {
    TKCHK(run_linear(ctx, &layer, TK_MODE_DIGITS, TK_PREP_DIGITS, ctx->h_act.p, TK_F32, nullptr, m, ctx->h_out.p, TK_F32));
  }
  HIPCHK(hipMemcpyAsync(out, ctx->h_out.p, out_len * 4, hipMemcpyDeviceToHost, ctx->stream));
  HIPCHK(hipStreamSynchronize(ctx->stream));
  return TK_OK;
}

extern "C" int tk_mpgemm(tk_ctx *ctx, const float *act, size_t act_len, const tk_weights *weights,
                         const float *scales, size_t scales_len, size_t m, size_t n, size_t k, int format,
                         float *out, size_t out_len) {
  return host_call(ctx, false, act, act_len, weights, scales, scales_len, m, n, k, format, out, out_len);
}

extern "C" int tk_mpgemm_with_act_quant(tk_ctx *ctx, const float *act, size_t act_len, const tk_weights *weights,
                                        const float *scales, size_t scales_len, size_t m, size_t n, size_t k,
                                        int format, float *out, size_t out_len) {
  return host_call(ctx, true, act, act_len, weights, scales, scales_len, m, n, k, format, out, out_len);
}

// ------------------------------------------------------------------------------------------
// mpgemm_projected_vjp (crates/tritium-spec/src/lib.rs:217-232)
// ------------------------------------------------------------------------------------------

static int vjp_weights_ok(tk_ctx *ctx, const tk_weights *weights) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "null context");
  if (!weights) return tk_fail(TK_ERR_INVALID_INPUT, "buffer is not a tritium-mi355x buffer");
  if (weights->ctx != ctx) return tk_fail(TK_ERR_INVALID_INPUT, "buffer belongs to another context");
  return TK_OK;
}

// Zero fill and launches shared by both forms; device pointers, ctx->mu held, device current.
static int vjp_enqueue(tk_ctx *ctx, const tk_weights *w, const float *scales, const float *act, const float *grad_output,
                       size_t m, float *grad_act, float *grad_w, float *grad_bias) {
  const size_t n = w->n, k = w->k;
  if (m > 0x7fffffffu || n > 0x7fffffffu || k > 0x7fffffffu || (m + 15) / 16 > 65535 || (n + 63) / 64 > 65535)
    return tk_fail(TK_ERR_INVALID_INPUT, "projected VJP launch bounds exceeded: M=%zu N=%zu K=%zu", m, n, k);
  // grad_act.fill(0.0); grad_projected_weight.fill(0.0) (crates/tritium-cpu/src/kernel.rs:122-123):
  // the kernels overwrite every element when m, n and k are all positive
  if (!(m && n && k)) {
    if (grad_act && m * k) HIPCHK(hipMemsetAsync(grad_act, 0, m * k * 4, ctx->stream));
    if (grad_w && n * k) HIPCHK(hipMemsetAsync(grad_w, 0, n * k * 4, ctx->stream));
  }
  HIPCHK(tk_launch_projected_vjp(ctx->stream, w->codes, w->nb, n, k, m, scales, act, grad_output, grad_act, grad_w,
                                 grad_bias));
  return TK_OK;
}

extern "C" int tk_projected_vjp(tk_ctx *ctx, const tk_weights *weights, const float *scales, const float *act,
                                const float *grad_output, size_t m, float *grad_act, float *grad_w,
                                float *grad_bias) {
  TKCHK(vjp_weights_ok(ctx, weights));
  if (weights->invalid_row >= 0)
    return tk_fail(TK_ERR_BACKEND, "unpack row %ld: decoded value 2 outside ternary range", weights->invalid_row);
  const size_t n = weights->n, k = weights->k;
  if ((m * n && (!grad_output || !scales)) || (m * k && grad_w && !act))
    return tk_fail(TK_ERR_INVALID_INPUT, "null operand pointer");
  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  return vjp_enqueue(ctx, weights, scales, act, grad_output, m, grad_act, grad_w, grad_bias);
}

extern "C" int tk_mpgemm_projected_vjp(tk_ctx *ctx, const float *act, size_t act_len, const tk_weights *weights,
                                       const float *scales, size_t scales_len, const float *grad_output,
                                       size_t grad_output_len, size_t m, size_t n, size_t k, int format,
                                       float *grad_act, size_t grad_act_len, float *grad_w, size_t grad_w_len,
                                       float *grad_bias, size_t grad_bias_len) {
  TKCHK(vjp_weights_ok(ctx, weights));
  // CpuBuffer::validate_identity, then the reserved-code refusal, before any length is looked at
  // (crates/tritium-cpu/src/lib.rs:359-370)
  if (!fmt_block_bytes(format)) return tk_fail(TK_ERR_UNSUPPORTED_FORMAT, "unsupported ternary format: %d", format);
  if (weights->n != n || weights->k != k || weights->format != format)
    return tk_fail(TK_ERR_INVALID_INPUT, "buffer identity N=%zu K=%zu format=%d does not match N=%zu K=%zu format=%d",
                   weights->n, weights->k, weights->format, n, k, format);
  if (weights->invalid_row >= 0)
    return tk_fail(TK_ERR_BACKEND, "unpack row %ld: decoded value 2 outside ternary range", weights->invalid_row);
  size_t mk, nk, mn;  // crates/tritium-cpu/src/kernel.rs:93-101
  if (__builtin_mul_overflow(m, k, &mk)) return tk_fail(TK_ERR_INVALID_INPUT, "M*K element count overflows");
  if (__builtin_mul_overflow(n, k, &nk)) return tk_fail(TK_ERR_INVALID_INPUT, "N*K element count overflows");
  if (__builtin_mul_overflow(m, n, &mn)) return tk_fail(TK_ERR_INVALID_INPUT, "M*N element count overflows");
  if (act_len != mk) return tk_fail_mismatch(mk, act_len);  // the reference's order (kernel.rs:102-120)
  if (scales_len != n) return tk_fail_mismatch(n, scales_len);
  if (grad_output_len != mn) return tk_fail_mismatch(mn, grad_output_len);
  if (grad_act_len != mk) return tk_fail_mismatch(mk, grad_act_len);
  if (grad_w_len != nk) return tk_fail_mismatch(nk, grad_w_len);
  if (grad_bias && grad_bias_len != n) return tk_fail_mismatch(n, grad_bias_len);
  if ((mk && (!act || !grad_act)) || (nk && !grad_w) || (n && !scales) || (mn && !grad_output))
    return tk_fail(TK_ERR_INVALID_INPUT, "null operand pointer");

  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  auto al = [](size_t x) { return (x + 63) & ~(size_t)63; };  // in floats
  const size_t in_floats = al(mk) + al(mn) + al(n), out_floats = al(mk) + al(nk) + al(n);
  TKCHK(ensure(ctx, ctx->h_act, in_floats * 4));
  TKCHK(ensure(ctx, ctx->h_out, out_floats * 4));
  float *d_act = (float *)ctx->h_act.p, *d_up = d_act + al(mk), *d_sc = d_up + al(mn);
  float *d_ga = (float *)ctx->h_out.p, *d_gw = d_ga + al(mk), *d_gb = d_gw + al(nk);
  if (mk) HIPCHK(hipMemcpyAsync(d_act, act, mk * 4, hipMemcpyHostToDevice, ctx->stream));
  if (mn) HIPCHK(hipMemcpyAsync(d_up, grad_output, mn * 4, hipMemcpyHostToDevice, ctx->stream));
  if (n) HIPCHK(hipMemcpyAsync(d_sc, scales, n * 4, hipMemcpyHostToDevice, ctx->stream));
  TKCHK(vjp_enqueue(ctx, weights, d_sc, d_act, d_up, m, d_ga, d_gw, grad_bias ? d_gb : nullptr));
  if (mk) HIPCHK(hipMemcpyAsync(grad_act, d_ga, mk * 4, hipMemcpyDeviceToHost, ctx->stream));
  if (nk) HIPCHK(hipMemcpyAsync(grad_w, d_gw, nk * 4, hipMemcpyDeviceToHost, ctx->stream));
  if (grad_bias && n) HIPCHK(hipMemcpyAsync(grad_bias, d_gb, n * 4, hipMemcpyDeviceToHost, ctx->stream));
  HIPCHK(hipStreamSynchronize(ctx->stream));
  return TK_OK;
}

// ------------------------------------------------------------------------------------------
// grouped launches
// ------------------------------------------------------------------------------------------

struct tk_group {
  tk_ctx *ctx;
  void *ws = nullptr;        // one allocation holding every member's operand rows and side arrays
  void *tables = nullptr;    // TkProblem[count], TkPrep[nprep], then int wg_prob[] (streaming form)
  int nprobs = 0, nprep = 0, prep_kind = 0;
  int prep_uniform_m = 0;    // > 0: prep entry j starts at token j * prep_uniform_m
  int prep_wave_pieces = 0;  // > 0: every entry fits the one-wave-per-token prep kernels; the largest piece count
  int prep_fast = 0;         // tk_prep_fast of every entry when they agree
  bool fused = false;        // the K-split kernel builds the operand rows itself: no prep launch (decided at creation)
  int prep_norm_fast = 0;    // some entry has an RMSNorm and tk_prep_norm_fast agrees for every entry: that value
  int prep_norm_pieces = 0;  // ... and the largest piece count
  unsigned prep_rows = 0;
  int variant = 1;
  size_t wg_prob_off = 0;
  TkLaunchCfg cfg{};
  // a second launch: the members of a prefill-form group whose operand rows do fit in LDS go
  // through the flow kernel
  bool has_flow_part = false;
  size_t flow_wg_prob_off = 0;
  TkLaunchCfg flow_cfg{};
};

static int group_create(tk_ctx *ctx, const tk_group_member *members, const tk_rmsnorm *norms, size_t count, int mode,
                        int act_dtype, int out_dtype, tk_group **out);

extern "C" int tk_group_create(tk_ctx *ctx, const tk_group_member *members, size_t count, int mode, int act_dtype,
                               int out_dtype, tk_group **out) {
  return group_create(ctx, members, nullptr, count, mode, act_dtype, out_dtype, out);
}

extern "C" int tk_group_create_normed(tk_ctx *ctx, const tk_group_member *members, const tk_rmsnorm *norms,
                                      size_t count, int act_dtype, int out_dtype, tk_group **out) {
  if (!norms && count) return tk_fail(TK_ERR_INVALID_INPUT, "tk_group_create_normed: null norms");
  return group_create(ctx, members, norms, count, TK_GROUP_A8, act_dtype, out_dtype, out);
}

static int group_create(tk_ctx *ctx, const tk_group_member *members, const tk_rmsnorm *norms, size_t count, int mode,
                        int act_dtype, int out_dtype, tk_group **out) {
  if (!ctx || !out || (!members && count)) return tk_fail(TK_ERR_INVALID_INPUT, "tk_group_create: null pointer");
  *out = nullptr;
  if (mode != TK_GROUP_FLOAT && mode != TK_GROUP_A8) return tk_fail(TK_ERR_INVALID_INPUT, "group mode %d", mode);
  if (norms)
    for (size_t i = 0; i < count; ++i)
      if (norms[i].weight) TKCHK(check_norm(&norms[i]));
  TKCHK(check_act_dtype(act_dtype));
  TKCHK(check_out_dtype(out_dtype, false));
  if (count == 0 || count > 65536) return tk_fail(TK_ERR_INVALID_INPUT, "group size %zu - use 1..65536", count);
  const int kmode = mode == TK_GROUP_FLOAT ? TK_MODE_DIGITS : TK_MODE_INT8;
  const int prep_kind = mode == TK_GROUP_FLOAT ? TK_PREP_DIGITS : TK_PREP_A8;

  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  std::vector<Plan> plans(count);
  std::vector<int> prep_of(count, -1);
  std::vector<TkPrep> preps;
  std::vector<size_t> prep_off;  // workspace offset of each distinct activation tensor
  size_t ws_bytes = 0;
  auto take = [&](size_t bytes) { size_t o = ws_bytes; ws_bytes += (bytes + 255) & ~(size_t)255; return o; };
  unsigned tiles = 0, rows = 0, sgroups = 0;
  int planes = 0, rt = 1;
  size_t lds = 0, slds = 0;
  for (size_t i = 0; i < count; ++i) {
    size_t n, k;
    TKCHK(validate_layer(ctx, &members[i].layer, &n, &k));
    const size_t m = members[i].m;
    if (!m || !n) return tk_fail(TK_ERR_INVALID_INPUT, "group member %zu is empty", i);
    if (!members[i].act || !members[i].out) return tk_fail(TK_ERR_INVALID_INPUT, "group member %zu: null pointer", i);
    plan_shape(ctx, &members[i].layer, n, k, m, kmode, out_dtype, &plans[i]);
    if (!plans[i].skinny)
      return tk_fail(TK_ERR_INVALID_INPUT, "group member %zu has %d operand rows; grouped launches take at most %d", i,
                     plans[i].pr.R, kSkinnyMaxRows);
    if (i == 0) planes = plans[i].cfg.planes;
    if (plans[i].cfg.planes != planes) return tk_fail(TK_ERR_INVALID_INPUT, "group members differ in plane count");
    if (plans[i].cfg.rt > rt) rt = plans[i].cfg.rt;
    if (plans[i].cfg.lds_bytes > lds) lds = plans[i].cfg.lds_bytes;
    // members reading the same activation tensor share one prep (q/k/v, gate/up)
    const tk_rmsnorm *nm_i = norms && norms[i].weight ? &norms[i] : nullptr;
    for (size_t j = 0; j < i; ++j) {
      const tk_rmsnorm *nm_j = norms && norms[j].weight ? &norms[j] : nullptr;
      const bool same_norm = (!nm_i && !nm_j) || (nm_i && nm_j && nm_i->weight == nm_j->weight && nm_i->eps == nm_j->eps &&
                                                  !nm_i->zero_centered == !nm_j->zero_centered);
      if (members[j].act == members[i].act && members[j].m == m && plans[j].pr.k == plans[i].pr.k && same_norm) {
        prep_of[i] = prep_of[j];
        break;
      }
    }
    if (prep_of[i] < 0) {
      TkPrep pp = {};
      const size_t R = plans[i].pr.R, nb = plans[i].pr.nb;
      pp.act = members[i].act;
      pp.k = k;
      pp.nb = nb;
      pp.R = R;
      pp.rs = R;
      pp.act_dtype = act_dtype;
      pp.m = (int)m;
      pp.row_begin = (int)rows;
      rows += (unsigned)m;
      if (nm_i) {
        pp.norm_kind = nm_i->zero_centered ? 2 : 1;
        pp.norm_eps = nm_i->eps;
        pp.norm_w = nm_i->weight;
      }
      prep_of[i] = (int)preps.size();
      preps.push_back(pp);
      prep_off.push_back(take(kPrepRowsMax(R) * nb * 256));  // room for the padded row strides (prefill kernel, 32x32x32 flow)
      take(R * 4); take(m * 4); take(m * 4); take(m * 4); take(m * 4);
      if (nm_i) take(m * k * 4);
    }
    plans[i].pr.tile_begin = (int)tiles;
    tiles += plans[i].cfg.grid;
  }
  size_t lds_r = (size_t)4 * planes * rt * 1024;
  if (lds_r > lds) lds = lds_r;
  // streaming / flow forms: every member is re-planned with the group's common rt
  const unsigned tpw = (unsigned)tk_stream_tiles_per_wg(planes, rt);
  size_t flds = 0;
  bool flow_ok = true;
  for (size_t i = 0; i < count; ++i) {
    if (plans[i].flow_lds > flds) flds = plans[i].flow_lds;
    flow_ok = flow_ok && plans[i].flow_ok;
  }
  size_t nb_max = 1, rows_max = 1, tokens_max = 1;
  for (size_t i = 0; i < count; ++i) {
    if ((size_t)plans[i].pr.nb > nb_max) nb_max = plans[i].pr.nb;
    if ((size_t)plans[i].pr.R > rows_max) rows_max = plans[i].pr.R;
    if ((size_t)plans[i].pr.M > tokens_max) tokens_max = plans[i].pr.M;
  }
  bool b3 = flow_ok;
  for (size_t i = 0; i < count && b3; ++i) b3 = flow_base3(plans[i].pr, planes, rt, flds);
  const bool wide = !b3 && flow_ok && flow_wide(ctx, planes, rt, nb_max, rows_max, kmode == TK_MODE_INT8 && ctx->flow_swap);
  if (wide) flds = flow_wide_lds(rt, nb_max);
  if (b3) flds += TK_B3_TABLE_BYTES;
  const int fw = b3 ? tk_flow3_waves(rt) : flow_waves(flds, rt, flow_sixteen(ctx, kmode == TK_MODE_INT8, true, wide, b3, planes, tiles, flow_runs_per_wave(wide, b3, planes, rt, rows_max)));
  int run_tiles = flow_run_tiles(ctx, tiles, planes, rt, fw, flds, nb_max, wide, b3, rows_max, tokens_max);
  {
    std::vector<unsigned> member_tiles(count);
    for (size_t i = 0; i < count; ++i) member_tiles[i] = (unsigned)plans[i].pr.n_tiles;
    run_tiles = trim_run_tiles(ctx, run_tiles, (size_t)fw * (size_t)flow_runs_per_wave(wide, b3, planes, rt, rows_max), member_tiles);
  }
  const unsigned fper = (unsigned)fw * (unsigned)flow_runs_per_wave(wide, b3, planes, rt, rows_max) * (unsigned)run_tiles;
  unsigned fgroups = 0;
  for (size_t i = 0; i < count; ++i) {
    sgroups += ((unsigned)plans[i].pr.n_tiles + tpw - 1) / tpw;
    fgroups += ((unsigned)plans[i].pr.n_tiles + fper - 1) / fper;
    if (plans[i].stream_lds > slds) slds = plans[i].stream_lds;
  }
  int variant = choose_decode(ctx, flow_ok, fgroups, sgroups);
  // One token for a group of more than two tiles per CU (gate,up): the flow kernel behind the prep launch, as for single
  // calls (run_linear) -- the K-split kernel would hand its workgroups several tiles each. gate,up of hidden 2560 behind
  // an RMSNorm, rotating over 30 layers: 13.4 -> 11.6 us (2 / 4 / 8 tokens 12.9 -> 12.9 / 13.9 -> 13.2 / 14.7 -> 13.8: left);
  // up to eight rows of two or more planes as well, as single calls.
  if (ctx->decode_force == DECODE_AUTO && variant == DECODE_KSPLIT && flow_ok && !wide && !b3 && rt == 1 &&
      (tokens_max == 1 || (rows_max <= 8 && planes >= 2)) && tiles > 2u * (unsigned)ctx->info.compute_units)
    variant = DECODE_FLOW;
  // Operand rows that do not fit in LDS, and more than one row tile of them: the prefill kernel
  // (operand rows streamed block by block, int8 MFMA over 64-row tiles) beats a decode kernel that
  // re-stages slices of K behind barriers.
  if (ctx->decode_force == DECODE_AUTO && !flow_ok && rt >= 2) variant = DECODE_GEMM;
  // A narrow group that would take the K-split kernel with more than one row tile (q,k,v or gate,up of a step of 17+
  // tokens): the prefill kernel, as for single launches (run_linear). Measured on hidden 2560, one plane, int8 contract
  // behind an RMSNorm, K-split -> prefill kernel: gate,up (864 tiles) 17 / 24 / 32 / 64 tokens 19.2 -> 14.9 / 21.6 ->
  // 14.9 / 23.7 -> 15.0 / 35.2 -> 15.3 us; q,k,v (240 tiles) 20 / 32 / 64 tokens 15.1 -> 14.8 / 16.6 -> 14.8 / 23.6 ->
  // 15.1 (17 tokens 13.7 -> 14.8: left alone). More planes and the float contract from 33 rows on, as single launches;
  // groups of more than two tiles per CU whatever their planes and contract.
  // (gate,up, float contract 5 / 8 tokens, one plane 18.2 / 20.3 us through the K-split kernel, 14.7 through the prefill
  // kernel; two planes of int8 rows, 17 / 32 tokens 20.0 / 24.3 against 16.8)
  const bool many_tiles = tiles > 2u * (unsigned)ctx->info.compute_units;
  const bool narrow_to_gemm = many_tiles || ((planes == 1 && kmode == TK_MODE_INT8) ? rows_max >= 20 : rows_max > 32);
  if (ctx->decode_force == DECODE_AUTO && variant == DECODE_KSPLIT && rt >= 2 && narrow_to_gemm) {
    variant = DECODE_GEMM;
    flow_ok = false;
    for (size_t i = 0; i < count; ++i) plans[i].flow_ok = false;
  }
  std::vector<int> wg_prob;
  int group_gemm_nt = 0;
  unsigned groups_total = 0;
  std::vector<int> flow_wg_prob;
  TkLaunchCfg flow_cfg{};
  if (variant == DECODE_GEMM) {
    // members whose rows fit go through the flow kernel in a launch of their own
    size_t pflds = 0, pnb_max = 1, prows_max = 1;
    unsigned ptiles = 0;
    std::vector<int> nbs;
    std::vector<double> wts;
    for (size_t i = 0; i < count; ++i) {
      if (!plans[i].flow_ok) continue;
      if (plans[i].flow_lds > pflds) pflds = plans[i].flow_lds;
      if ((size_t)plans[i].pr.nb > pnb_max) pnb_max = plans[i].pr.nb;
      if ((size_t)plans[i].pr.R > prows_max) prows_max = plans[i].pr.R;
      ptiles += (unsigned)plans[i].pr.n_tiles;
      nbs.push_back(plans[i].pr.nb);
      wts.push_back((double)plans[i].pr.n_tiles * (double)plans[i].pr.nb);
    }
    // one plane: two tiles per wave when four would leave fewer than four workgroups per CU (as for
    // single launches)
    bool gemm_nt2 = false;
    if (planes == 1) {
      unsigned total = 0;
      for (size_t i = 0; i < count; ++i) {
        if (plans[i].flow_ok) continue;
        Plan tmp = plans[i];
        plan_gemm(&tmp);
        total += 8u * (unsigned)tmp.pr.sub_m * (unsigned)tmp.pr.sub_n;
      }
      gemm_nt2 = ctx->gemm_tiles == 2 || (ctx->gemm_tiles == 0 && total < 4u * (unsigned)ctx->info.compute_units);
    }
    group_gemm_nt = gemm_nt2 ? 2 : 0;
    const bool pwide = ptiles && flow_wide(ctx, planes, rt, pnb_max, prows_max, kmode == TK_MODE_INT8 && ctx->flow_swap);
    if (pwide) pflds = flow_wide_lds(rt, pnb_max);
    const int pfw = flow_waves(pflds, rt, flow_sixteen(ctx, kmode == TK_MODE_INT8, true, pwide, false, planes, ptiles, flow_runs_per_wave(pwide, false, planes, rt, prows_max)));
    int prun = ptiles ? flow_run_tiles(ctx, ptiles, planes, rt, pfw, pflds, pnb_max, pwide, false, prows_max, tokens_max) : 1;
    {
      std::vector<unsigned> member_tiles;
      for (size_t i = 0; i < count; ++i)
        if (plans[i].flow_ok) member_tiles.push_back((unsigned)plans[i].pr.n_tiles);
      prun = trim_run_tiles(ctx, prun, (size_t)pfw * (size_t)flow_runs_per_wave(pwide, false, planes, rt, prows_max), member_tiles);
    }
    const unsigned pper = (unsigned)pfw * (unsigned)flow_runs_per_wave(pwide, false, planes, rt, prows_max) * (unsigned)prun;
    unsigned flow_total = 0;
    for (size_t i = 0; i < count; ++i) {
      if (plans[i].flow_ok) {
        const unsigned gi = ((unsigned)plans[i].pr.n_tiles + pper - 1) / pper;
        plans[i].pr.group_begin = (int)flow_total;
        plans[i].pr.run_tiles = prun;
        for (unsigned j = 0; j < gi; ++j) flow_wg_prob.push_back((int)i);
        flow_total += gi;
        if (pwide) {
          plans[i].pr.rs = (int)flow_wide_rows(rt);
          preps[prep_of[i]].rs = flow_wide_rows(rt);
        }
        continue;
      }
      plan_gemm(&plans[i], 0u, gemm_nt2 ? 2 : 4);
      const unsigned gi = 8u * (unsigned)plans[i].pr.sub_m * (unsigned)plans[i].pr.sub_n;
      plans[i].pr.group_begin = (int)groups_total;
      for (unsigned j = 0; j < gi; ++j) wg_prob.push_back((int)i);
      groups_total += gi;
      preps[prep_of[i]].rs = (size_t)plans[i].pr.rs;
    }
    if (flow_total) {
      flow_cfg.planes = planes;
      flow_cfg.rt = rt;
      flow_cfg.lds_bytes = pflds;
      flow_cfg.grid = flow_total;
      flow_cfg.waves = pfw;
      flow_cfg.ring = pick_flow_ring(ctx, nbs.data(), wts.data(), (int)nbs.size(), rt, (int)prows_max, flow_runs_per_wave(pwide, false, planes, rt, prows_max), pwide, pfw, pflds, planes);
      size_t ztiles = 0;
      for (size_t i = 0; i < count; ++i)
        if (plans[i].flow_ok && plans[i].pr.zskip) ztiles = pper;
      ztiles = flow_zero_plan(pwide, false, false, planes, pflds, ztiles, pnb_max);
      if (!ztiles)
        for (size_t i = 0; i < count; ++i)
          if (plans[i].flow_ok) plans[i].pr.zskip = 0;
      flow_cfg_form(&flow_cfg, pwide, false, pflds, prows_max, ztiles, pnb_max, kmode == TK_MODE_INT8 && ctx->flow_swap);
    }
  } else if (variant != DECODE_KSPLIT) {
    const unsigned per = variant == DECODE_FLOW ? fper : tpw;
    for (size_t i = 0; i < count; ++i) {
      const unsigned gi = ((unsigned)plans[i].pr.n_tiles + per - 1) / per;
      plans[i].pr.group_begin = (int)groups_total;
      plans[i].pr.run_tiles = run_tiles;
      if (variant == DECODE_STREAM) plans[i].pr.kc = plans[i].stream_kc;
      if (variant == DECODE_FLOW && wide) {
        plans[i].pr.rs = (int)flow_wide_rows(rt);
        preps[prep_of[i]].rs = flow_wide_rows(rt);
      }
      for (unsigned j = 0; j < gi; ++j) wg_prob.push_back((int)i);
      groups_total += gi;
    }
  }
  // zero-chunk maps in a flow-form group: room for the words of one workgroup's chunks behind the rows
  size_t group_ztiles = 0;
  if (variant == DECODE_FLOW) {
    for (size_t i = 0; i < count; ++i)
      if (plans[i].pr.zskip) group_ztiles = fper;
    group_ztiles = flow_zero_plan(wide, b3, false, planes, flds, group_ztiles, nb_max);
    if (!group_ztiles)
      for (size_t i = 0; i < count; ++i) plans[i].pr.zskip = 0;
  }
  // One launch for a group of single tokens (q,k,v or gate,up of a decode step, with their RMSNorm): the K-split
  // kernel builds every member's operand rows itself, as for single calls (run_linear). Measured on q,k,v of
  // hidden 2560 behind a norm, one token: prep 4.8 us + kernel 4.2 us as two dependent launches.
  bool gfused = variant == DECODE_KSPLIT && rt == 1 && (prep_kind == TK_PREP_A8 || prep_kind == TK_PREP_DIGITS) &&
                (act_dtype == TK_F32 || act_dtype == TK_BF16);
  size_t fuse_lds = 0;  // LDS of the fused form: the largest member's rows + constants (+ norm scratch) + reduction
  unsigned fuse_tpw = 1;
  {
    // (q,k,v of hidden 2560 without a norm, two tokens: int8 contract 8.6 -> 7.3 us, float contract 9.7 -> 9.2; three
    // tokens 9.0 -> 9.0 and 10.5 -> 11.2)
    const size_t glimit = ctx->fuse_tokens >= 0 ? (size_t)ctx->fuse_tokens : (prep_kind == TK_PREP_A8 ? 2 : 1);
    for (size_t i = 0; i < count && gfused; ++i) {
      const TkPrep &pp = preps[prep_of[i]];
      const size_t k = (size_t)plans[i].pr.k, nb = (size_t)plans[i].pr.nb;
      gfused = (size_t)members[i].m <= glimit && nb * 16 <= 512 && k % 256 == 0 && ((uintptr_t)members[i].act & 15) == 0 &&
               (size_t)plans[i].pr.kc >= nb &&
               (!pp.norm_kind || (members[i].m == 1 && ((uintptr_t)pp.norm_w & 15) == 0));
      const size_t need = nb * 256 * (size_t)plans[i].pr.R + 1024 + (pp.norm_kind ? k * 4 + 1024 : 0) + (size_t)4096 * planes;
      if (need > fuse_lds) fuse_lds = need;
    }
    fuse_tpw = (tiles + 2u * (unsigned)ctx->info.compute_units - 1) / (2u * (unsigned)ctx->info.compute_units);
    if (!fuse_tpw) fuse_tpw = 1;
    gfused = gfused && fuse_lds + 1024 <= 64 * 1024 && fuse_tpw <= 4;  // (as for single calls)
    if (gfused) {  // workgroups take fuse_tpw consecutive tiles of one member: tile_begin counts workgroups
      unsigned wgs = 0;
      for (size_t i = 0; i < count; ++i) {
        plans[i].pr.tile_begin = (int)wgs;
        plans[i].pr.run_tiles = (int)fuse_tpw;
        wgs += ((unsigned)plans[i].pr.n_tiles + fuse_tpw - 1) / fuse_tpw;
      }
      tiles = wgs;
    }
  }
  // The flow kernel has the form too (one token per member, four-wave workgroups of the 16x16x64 kernel with
  // activations first): every workgroup builds the row of the member it works for. gate,up of hidden 2560 behind an
  // RMSNorm, one bf16 token: 11.6 us as prep + kernel.
  // Every workgroup repeats its member's prep, so the form is for groups of a few workgroups per CU at most (as the K-split
  // kernel's): the 210 projections of a 30-layer step as ONE group took 173 us this way against 91 us behind one prep launch.
  bool gfused_flow = variant == DECODE_FLOW && !wide && !b3 && rt == 1 && planes <= 2 && fw == 4 && ctx->fuse_tokens != 0 &&
                     tiles <= 8u * (unsigned)ctx->info.compute_units &&
                     (prep_kind == TK_PREP_A8 || prep_kind == TK_PREP_DIGITS) && (act_dtype == TK_F32 || act_dtype == TK_BF16);
  size_t fuse_flow_extra = 1024;  // row constants (+ the norm's scratch) behind the rows
  for (size_t i = 0; i < count && gfused_flow; ++i) {
    const TkPrep &pp = preps[prep_of[i]];
    const size_t k = (size_t)plans[i].pr.k, nb = (size_t)plans[i].pr.nb;
    gfused_flow = members[i].m == 1 && nb * 16 <= 512 && k % 256 == 0 && ((uintptr_t)members[i].act & 15) == 0 &&
                  (!pp.norm_kind || ((uintptr_t)pp.norm_w & 15) == 0);
    if (pp.norm_kind && 1024 + k * 4 + 1024 > fuse_flow_extra) fuse_flow_extra = 1024 + k * 4 + 1024;
  }
  gfused_flow = gfused_flow && flds + fuse_flow_extra + 1024 <= 64 * 1024;
  if (gfused_flow) {  // (the form keeps its row constants where the zero-chunk maps would go)
    group_ztiles = 0;
    for (size_t i = 0; i < count; ++i) plans[i].pr.zskip = 0;
  }
  tk_group *g = new (std::nothrow) tk_group();
  if (!g) return tk_fail(TK_ERR_BACKEND, "tk_group_create: host allocation failed");
  g->ctx = ctx;
  g->fused = gfused || gfused_flow;
  int rc = dev_malloc(ws_bytes, &g->ws);
  const size_t wg_prob_off = count * sizeof(TkProblem) + preps.size() * sizeof(TkPrep);
  const size_t flow_wg_prob_off = wg_prob_off + wg_prob.size() * sizeof(int);
  if (!rc) rc = dev_malloc(flow_wg_prob_off + flow_wg_prob.size() * sizeof(int), &g->tables);
  if (rc) {
    if (g->ws) (void)hipFree(g->ws);
    delete g;
    return rc;
  }
  // hand out the side arrays in the same order `take` reserved them
  for (size_t j = 0; j < preps.size(); ++j) {
    const size_t R = preps[j].R, nb = preps[j].nb, m = (size_t)preps[j].m;
    auto al = [](size_t b) { return (b + 255) & ~(size_t)255; };
    uint8_t *base = (uint8_t *)g->ws + prep_off[j];
    preps[j].ap = (int8_t *)base; base += al(kPrepRowsMax(R) * nb * 256);
    preps[j].rowsum = (int32_t *)base; base += al(R * 4);
    preps[j].act_scale = (float *)base; base += al(m * 4);
    preps[j].aux = (float *)base; base += al(m * 4);
    preps[j].exps = (int32_t *)base; base += al(m * 4);
    preps[j].flags = (uint32_t *)base; base += al(m * 4);
    if (preps[j].norm_kind) preps[j].ynorm = (float *)base;
  }
  std::vector<TkProblem> probs(count);
  for (size_t i = 0; i < count; ++i) {
    TkProblem pr = plans[i].pr;
    const TkPrep &pp = preps[prep_of[i]];
    pr.ap = pp.ap;
    pr.rowsum = pp.rowsum;
    pr.flags = pp.flags;
    pr.raw_act = pp.norm_kind ? (const void *)pp.ynorm : members[i].act;  // the exact fallback reads the normalized row
    pr.raw_dtype = pp.norm_kind ? TK_F32 : act_dtype;
    pr.out = members[i].out;
    if (prep_kind == TK_PREP_A8) {
      pr.act_scale = pp.act_scale;
      pr.aux = pp.aux;
    } else {
      pr.exps = pp.exps;
    }
    if (gfused || gfused_flow) {  // the kernel reads (and normalizes) the raw rows itself
      pr.raw_act = members[i].act;
      pr.raw_dtype = act_dtype;
      pr.norm_kind = pp.norm_kind;
      pr.norm_eps = pp.norm_eps;
      pr.norm_w = pp.norm_w;
    }
    probs[i] = pr;
  }
  hipError_t e = hipMemcpy(g->tables, probs.data(), count * sizeof(TkProblem), hipMemcpyHostToDevice);
  if (e == hipSuccess)
    e = hipMemcpy((uint8_t *)g->tables + count * sizeof(TkProblem), preps.data(), preps.size() * sizeof(TkPrep),
                  hipMemcpyHostToDevice);
  if (e == hipSuccess && !wg_prob.empty())
    e = hipMemcpy((uint8_t *)g->tables + wg_prob_off, wg_prob.data(), wg_prob.size() * sizeof(int),
                  hipMemcpyHostToDevice);
  if (e == hipSuccess && !flow_wg_prob.empty())
    e = hipMemcpy((uint8_t *)g->tables + flow_wg_prob_off, flow_wg_prob.data(), flow_wg_prob.size() * sizeof(int),
                  hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    (void)hipFree(g->ws);
    (void)hipFree(g->tables);
    delete g;
    return tk_fail(TK_ERR_BACKEND, "tk_group_create: %s", hipGetErrorString(e));
  }
  g->has_flow_part = !flow_wg_prob.empty();
  g->flow_wg_prob_off = flow_wg_prob_off;
  g->flow_cfg = flow_cfg;
  g->variant = variant;
  g->wg_prob_off = wg_prob_off;
  g->nprobs = (int)count;
  g->nprep = (int)preps.size();
  g->prep_uniform_m = preps.empty() ? 0 : preps[0].m;
  for (size_t j = 0; j < preps.size(); ++j)
    if (preps[j].m != preps[0].m || preps[j].row_begin != (int)j * preps[0].m) g->prep_uniform_m = 0;
  g->prep_kind = prep_kind;
  g->prep_rows = rows;
  g->prep_wave_pieces = 0;
  {
    size_t pieces = 0;
    bool ok = true;
    for (const TkPrep &pp : preps) {
      ok = ok && !pp.norm_kind && !pp.blocksum;  // (which form, if any, takes that many pieces: the launcher's rule)
      if (pp.nb * 16 > pieces) pieces = pp.nb * 16;
    }
    if (ok) g->prep_wave_pieces = (int)pieces;
    g->prep_fast = preps.empty() ? 0 : tk_prep_fast(preps[0]);
    for (const TkPrep &pp : preps)
      if (tk_prep_fast(pp) != g->prep_fast) g->prep_fast = 0;
    bool any_norm = false;
    g->prep_norm_fast = preps.empty() ? 0 : tk_prep_norm_fast(preps[0]);
    for (const TkPrep &pp : preps) {
      any_norm = any_norm || pp.norm_kind != 0;
      if (tk_prep_norm_fast(pp) != g->prep_norm_fast) g->prep_norm_fast = 0;
    }
    if (!any_norm || prep_kind != TK_PREP_A8) g->prep_norm_fast = 0;
    g->prep_norm_pieces = (int)pieces;
  }
  g->cfg.planes = planes;
  g->cfg.rt = rt;
  g->cfg.lds_bytes = variant == DECODE_FLOW ? flds : (variant == DECODE_STREAM ? slds : lds);
  if (variant == DECODE_GEMM) g->cfg.lds_bytes = (size_t)tk_gemm_lds_bytes();
  g->cfg.gemm_nt = variant == DECODE_GEMM ? group_gemm_nt : 0;
  g->cfg.gemm_two_by_two = ctx->gemm_two_by_two;
  g->cfg.grid = variant == DECODE_KSPLIT ? tiles : groups_total;
  g->cfg.waves = fw;
  {
    std::vector<int> nbs(count);
    std::vector<double> wts(count);
    for (size_t i = 0; i < count; ++i) {
      nbs[i] = plans[i].pr.nb;
      wts[i] = (double)plans[i].pr.n_tiles * (double)plans[i].pr.nb;  // chunks of the member
    }
    g->cfg.ring = pick_flow_ring(ctx, nbs.data(), wts.data(), (int)count, rt, (int)rows_max, flow_runs_per_wave(wide, b3, planes, rt, rows_max), wide, fw, flds, planes);
  }
  if (variant == DECODE_FLOW) flow_cfg_form(&g->cfg, wide, b3, flds, rows_max, group_ztiles, nb_max, kmode == TK_MODE_INT8 && ctx->flow_swap && !gfused && !gfused_flow);
  if (gfused) {
    g->cfg.fused = 1;
    g->cfg.lds_bytes = fuse_lds;
  }
  if (gfused_flow) {
    g->cfg.fused = 1;
    g->cfg.lds_bytes += fuse_flow_extra;
  }
  ctx->refs.fetch_add(1);
  *out = g;
  return TK_OK;
}

extern "C" int tk_group_launch_parts(tk_ctx *ctx, tk_group *g, int do_prep, int do_main) {
  if (!ctx || !g || g->ctx != ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_group_launch: bad group");
  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  const TkProblem *probs = (const TkProblem *)g->tables;
  const TkPrep *preps = (const TkPrep *)((const uint8_t *)g->tables + (size_t)g->nprobs * sizeof(TkProblem));
  if (do_main && g->fused) ctx->fused_calls++;
  if (do_prep && !g->fused)  // (a group that runs as one launch has no prep part)
    HIPCHK(tk_launch_prep(ctx->stream, g->prep_kind, nullptr, preps, g->nprep, g->prep_uniform_m, g->prep_rows,
                          g->prep_wave_pieces, g->prep_fast, g->prep_norm_fast, g->prep_norm_pieces));
  const int *wg_prob = (const int *)((const uint8_t *)g->tables + g->wg_prob_off);
  // Members whose rows fit LDS take the flow kernel, the others one grouped launch of the prefill kernel. The
  // two read and write disjoint members and fit a CU together (one eight-wave workgroup with its rows in LDS
  // beside 49-KiB workgroups of the prefill kernel), so they run side by side on two streams: the second
  // starts behind everything enqueued so far and the first waits for it at the end.
  const bool both = do_main && g->has_flow_part && g->variant == DECODE_GEMM && g->cfg.grid > 0;
  bool forked = false;
  if (both && ctx->group_overlap) {
    if (!ctx->stream2 || !ctx->ev_fork || !ctx->ev_join) {  // all three or none
      hipStream_t s2 = nullptr;
      hipEvent_t ef = nullptr, ej = nullptr;
      hipError_t ce = hipStreamCreateWithFlags(&s2, hipStreamNonBlocking);
      if (ce == hipSuccess) ce = hipEventCreateWithFlags(&ef, hipEventDisableTiming);
      if (ce == hipSuccess) ce = hipEventCreateWithFlags(&ej, hipEventDisableTiming);
      if (ce != hipSuccess) {
        if (ej) (void)hipEventDestroy(ej);
        if (ef) (void)hipEventDestroy(ef);
        if (s2) (void)hipStreamDestroy(s2);
        return tk_fail(TK_ERR_BACKEND, "second stream of the context: %s", hipGetErrorString(ce));
      }
      ctx->stream2 = s2;
      ctx->ev_fork = ef;
      ctx->ev_join = ej;
    }
    HIPCHK(hipEventRecord(ctx->ev_fork, ctx->stream));
    HIPCHK(hipStreamWaitEvent(ctx->stream2, ctx->ev_fork, 0));
    // From here on the second stream may hold work: whatever fails below, the first stream is ordered behind it
    // before the call returns (join_error), so that nothing enqueued later, and no tk_sync, overtakes it.
    hipError_t fe = tk_launch_gemm(ctx->stream2, nullptr, probs, wg_prob, g->cfg);
    if (fe == hipSuccess) fe = hipEventRecord(ctx->ev_join, ctx->stream2);
    if (fe != hipSuccess) {
      (void)hipStreamSynchronize(ctx->stream2);
      return tk_fail(TK_ERR_BACKEND, "grouped prefill launch on the second stream: %s", hipGetErrorString(fe));
    }
    forked = true;
  }
  if (do_main && g->has_flow_part) {
    const hipError_t fe = tk_launch_flow(ctx->stream, nullptr, probs, (const int *)((const uint8_t *)g->tables + g->flow_wg_prob_off),
                                         g->flow_cfg);
    if (fe != hipSuccess) {
      if (forked && hipStreamWaitEvent(ctx->stream, ctx->ev_join, 0) != hipSuccess) (void)hipStreamSynchronize(ctx->stream2);
      return tk_fail(TK_ERR_BACKEND, "grouped flow launch: %s", hipGetErrorString(fe));
    }
  }
  if (forked) {
    if (hipStreamWaitEvent(ctx->stream, ctx->ev_join, 0) != hipSuccess) {
      (void)hipStreamSynchronize(ctx->stream2);
      return tk_fail(TK_ERR_BACKEND, "joining the second stream failed");
    }
  }
  else if (do_main && g->variant == DECODE_GEMM)
    HIPCHK(tk_launch_gemm(ctx->stream, nullptr, probs, wg_prob, g->cfg));
  else if (do_main && g->variant == DECODE_FLOW && g->cfg.base3)
    HIPCHK(tk_launch_flow3(ctx->stream, nullptr, probs, wg_prob, g->cfg));
  else if (do_main && g->variant == DECODE_FLOW)
    HIPCHK(tk_launch_flow(ctx->stream, nullptr, probs, wg_prob, g->cfg));
  else if (do_main && g->variant == DECODE_STREAM)
    HIPCHK(tk_launch_stream(ctx->stream, nullptr, probs, wg_prob, g->cfg));
  else if (do_main)
    HIPCHK(tk_launch_skinny(ctx->stream, nullptr, probs, g->nprobs, g->cfg));
  return TK_OK;
}

extern "C" int tk_group_launch(tk_ctx *ctx, tk_group *g) { return tk_group_launch_parts(ctx, g, 1, 1); }

extern "C" void tk_group_destroy(tk_group *g) {
  if (!g) return;
  tk_ctx *ctx = g->ctx;
  {
    std::lock_guard<std::mutex> lk(ctx->mu);
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    if (ctx->stream2) (void)hipStreamSynchronize(ctx->stream2);
    if (g->ws) (void)hipFree(g->ws);
    if (g->tables) (void)hipFree(g->tables);
  }
  delete g;
  ctx_release(ctx);
}

// ------------------------------------------------------------------------------------------
// plumbing
// ------------------------------------------------------------------------------------------

extern "C" int tk_malloc(tk_ctx *ctx, size_t bytes, void **dptr) {
  if (!ctx || !dptr) return tk_fail(TK_ERR_INVALID_INPUT, "tk_malloc: null pointer");
  HIPCHK(hipSetDevice(ctx->device));
  return dev_malloc(bytes, dptr);
}
extern "C" int tk_free(tk_ctx *ctx, void *dptr) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_free: null context");
  if (!dptr) return TK_OK;
  HIPCHK(hipSetDevice(ctx->device));
  HIPCHK(hipStreamSynchronize(ctx->stream));
  HIPCHK(hipFree(dptr));
  return TK_OK;
}
extern "C" int tk_memcpy_h2d(tk_ctx *ctx, void *dst, const void *src, size_t bytes) {
  if (!ctx || ((!dst || !src) && bytes)) return tk_fail(TK_ERR_INVALID_INPUT, "tk_memcpy_h2d: null pointer");
  if (!bytes) return TK_OK;
  HIPCHK(hipSetDevice(ctx->device));
  HIPCHK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
  HIPCHK(hipStreamSynchronize(ctx->stream));
  return TK_OK;
}
extern "C" int tk_memcpy_d2h(tk_ctx *ctx, void *dst, const void *src, size_t bytes) {
  if (!ctx || ((!dst || !src) && bytes)) return tk_fail(TK_ERR_INVALID_INPUT, "tk_memcpy_d2h: null pointer");
  if (!bytes) return TK_OK;
  HIPCHK(hipSetDevice(ctx->device));
  HIPCHK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
  HIPCHK(hipStreamSynchronize(ctx->stream));
  return TK_OK;
}
extern "C" int tk_memset(tk_ctx *ctx, void *dst, int value, size_t bytes) {
  if (!ctx || (!dst && bytes)) return tk_fail(TK_ERR_INVALID_INPUT, "tk_memset: null pointer");
  if (!bytes) return TK_OK;
  HIPCHK(hipSetDevice(ctx->device));
  HIPCHK(hipMemsetAsync(dst, value, bytes, ctx->stream));
  return TK_OK;
}
extern "C" int tk_sync(tk_ctx *ctx) {
  if (!ctx) return tk_fail(TK_ERR_INVALID_INPUT, "tk_sync: null context");
  HIPCHK(hipSetDevice(ctx->device));
  HIPCHK(hipStreamSynchronize(ctx->stream));
  return TK_OK;
}
extern "C" void *tk_stream(tk_ctx *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

extern "C" int tk_event_create(tk_ctx *ctx, tk_event **out) {
  if (!ctx || !out) return tk_fail(TK_ERR_INVALID_INPUT, "tk_event_create: null pointer");
  HIPCHK(hipSetDevice(ctx->device));
  tk_event *ev = new (std::nothrow) tk_event();
  if (!ev) return tk_fail(TK_ERR_BACKEND, "tk_event_create: host allocation failed");
  hipError_t e = hipEventCreate(&ev->ev);
  if (e != hipSuccess) {
    delete ev;
    return tk_fail(TK_ERR_BACKEND, "hipEventCreate: %s", hipGetErrorString(e));
  }
  *out = ev;
  return TK_OK;
}
extern "C" int tk_event_record(tk_ctx *ctx, tk_event *ev) {
  if (!ctx || !ev) return tk_fail(TK_ERR_INVALID_INPUT, "tk_event_record: null pointer");
  HIPCHK(hipEventRecord(ev->ev, ctx->stream));
  return TK_OK;
}
extern "C" int tk_event_elapsed_ms(tk_event *start, tk_event *stop, float *ms) {
  if (!start || !stop || !ms) return tk_fail(TK_ERR_INVALID_INPUT, "tk_event_elapsed_ms: null pointer");
  HIPCHK(hipEventSynchronize(stop->ev));
  HIPCHK(hipEventElapsedTime(ms, start->ev, stop->ev));
  return TK_OK;
}
extern "C" void tk_event_destroy(tk_event *ev) {
  if (!ev) return;
  (void)hipEventDestroy(ev->ev);
  delete ev;
}

extern "C" int tk_copy_kernel(tk_ctx *ctx, void *dst, const void *src, size_t bytes) {
  if (!ctx || !dst || !src) return tk_fail(TK_ERR_INVALID_INPUT, "tk_copy_kernel: null pointer");
  if (bytes % 16) return tk_fail(TK_ERR_INVALID_INPUT, "tk_copy_kernel: %zu bytes is not a multiple of 16", bytes);
  std::lock_guard<std::mutex> lk(ctx->mu);
  HIPCHK(hipSetDevice(ctx->device));
  HIPCHK(tk_launch_copy(ctx->stream, dst, src, bytes));
  return TK_OK;
}

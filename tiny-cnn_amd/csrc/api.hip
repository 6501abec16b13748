// api.hip — library state, device memory, events and the thin extern "C" layer that
// validates arguments before anything is launched.
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "common.h"

namespace tdh {

Context &ctx() {
  static Context c;
  return c;
}

static thread_local char g_error[512] = "";

int set_error(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

StreamSwap::StreamSwap(hipStream_t s) : saved(ctx().stream) { ctx().stream = s; }
StreamSwap::~StreamSwap() { ctx().stream = saved; }

int ws_begin(size_t total) {
  Context &c = ctx();
  if (c.ws_keep) {
    if (c.workspace_off + total <= c.workspace_size) return TDH_OK;
    return set_error(TDH_ERR_INVALID, "scratch reservation of %zu more bytes exceeds the locked %zu",
                     total, c.workspace_size);
  }
  c.workspace_off = 0;
  if (total <= c.workspace_size) return TDH_OK;
  if (c.ws_locked)
    return set_error(TDH_ERR_INVALID, "scratch reservation of %zu bytes exceeds the locked %zu",
                     total, c.workspace_size);
  if (c.workspace) TDH_HIP(hipFree(c.workspace));
  c.workspace      = nullptr;
  c.workspace_size = 0;
  const size_t want = ws_align(total + (total >> 2));
  void *p           = nullptr;
  if (hipMalloc(&p, want) != hipSuccess) {
    (void)hipGetLastError();
    return set_error(TDH_ERR_OOM, "cannot allocate %zu bytes of scratch", want);
  }
  c.workspace      = static_cast<char *>(p);
  c.workspace_size = want;
  return TDH_OK;
}

int ws_take(size_t bytes, void **out) {
  Context &c = ctx();
  const size_t need = ws_align(bytes);
  if (c.workspace_off + need > c.workspace_size)
    return set_error(TDH_ERR_INVALID, "scratch overrun: %zu + %zu > %zu (reservation too small)",
                     c.workspace_off, need, c.workspace_size);
  *out = c.workspace + c.workspace_off;
  c.workspace_off += need;
  return TDH_OK;
}

// ----------------------------------------------------- scratch that is never allocated
// tdh_conv2d_bwd_static runs the kernels of tdh_conv2d_bwd with their scratch (split partial
// sums, repacked filters, staged bias sums) in this file-scope device array instead of the
// grow-only buffer that ws_begin allocates, for callers that cannot allocate. Every device the
// library is initialised on holds its own copy of the array, at its own address, until the
// process ends. In host code the array's NAME is only a handle for hipGetSymbolAddress: the
// device address is looked up once per device in tdh_init and only that pointer is ever passed
// to kernels.
constexpr size_t kStaticScratchBytes = 64u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
static char *g_static_scratch[kMaxDevices] = {};

static int lookup_static_scratch(int device) {
  if (device < 0 || device >= kMaxDevices)
    return set_error(TDH_ERR_INVALID, "tdh_init: device %d beyond the %d this library keeps state for",
                     device, kMaxDevices);
  if (g_static_scratch[device]) return TDH_OK;
  void *p = nullptr;
  TDH_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));  // the current device's copy
  if (!p) return set_error(TDH_ERR_HIP, "tdh_init: the static scratch array has no device address");
  g_static_scratch[device] = static_cast<char *>(p);
  return TDH_OK;
}

// Points the context's scratch at the static array for one call; nothing can allocate meanwhile.
struct StaticScratchScope {
  Context &c;
  char *saved_ws;
  size_t saved_size, saved_off;
  bool saved_locked;
  StaticScratchScope(Context &cc, char *ptr)
      : c(cc), saved_ws(cc.workspace), saved_size(cc.workspace_size), saved_off(cc.workspace_off),
        saved_locked(cc.ws_locked) {
    c.workspace      = ptr;
    c.workspace_size = kStaticScratchBytes;
    c.workspace_off  = 0;
    c.ws_locked      = true;
  }
  ~StaticScratchScope() {
    c.workspace      = saved_ws;
    c.workspace_size = saved_size;
    c.workspace_off  = saved_off;
    c.ws_locked      = saved_locked;
  }
};

// Tuning sweeps only: the environment variable TDH_GEMM_PLAN="cfg,splits", read once by
// tdh_init, forces one tile configuration (0..9, see gemm_mfma.h) and split count for every
// GEMM of the process; unset, the plan is a function of the shape alone. Not part of the ABI.
static int g_force_cfg = -1, g_force_splits = 1, g_force_only_m = -1;

static void read_gemm_plan_override() {
  g_force_cfg    = -1;
  g_force_splits = 1;
  const char *e = std::getenv("TDH_GEMM_PLAN");
  int cfg = -1, splits = 1, only_m = -1;
  g_force_only_m = -1;
  if (e && std::sscanf(e, "%d,%d,%d", &cfg, &splits, &only_m) >= 2 && cfg >= 0 && cfg < 10 && splits >= 1) {
    g_force_cfg    = cfg;
    g_force_splits = splits;
    g_force_only_m = only_m;  // "cfg,splits,M": only products with M rows
  }
}

bool gemm_plan_override(int *cfg, int *splits, int M) {
  *cfg    = g_force_cfg;
  *splits = g_force_splits;
  return g_force_cfg >= 0 && (g_force_only_m < 0 || g_force_only_m == M);
}

// ----------------------------------------------------------------- profiler
namespace {
struct ProfRecord {
  std::string tag;
  double work;
  WorkUnit unit;
  std::vector<std::pair<hipEvent_t, hipEvent_t>> launches;  // (begin, end) of every kernel
};
struct ProfEntry {
  std::string tag;
  int64_t launches = 0;
  double total_ms = 0.0, work = 0.0;
  int unit = 0;
};
bool g_profiling = false;
int g_open_scope = -1;  // index into g_records of the innermost open ProfScope
std::vector<ProfRecord> g_records;
// Events go back to the pool of the role they had: the runtime remembers on an event handed to
// hipExtLaunchKernelGGL whether it stands for the begin or the end of the dispatch.
std::vector<hipEvent_t> g_event_pool[2];  // [0] start events, [1] stop events
std::vector<ProfEntry> g_entries;
// the kernel launches of the profiled region in dispatch order, as indices into g_records
// (-1: outside any scope), and after tdh_profile_end their tags
std::vector<int> g_launch_order;
std::vector<std::string> g_launch_tags;

hipEvent_t take_event(int role) {
  if (!g_event_pool[role].empty()) {
    hipEvent_t e = g_event_pool[role].back();
    g_event_pool[role].pop_back();
    return e;
  }
  hipEvent_t e = nullptr;
  (void)hipEventCreate(&e);
  return e;
}
}  // namespace

static int open_record(const std::string &tag, double work, WorkUnit unit) {
  g_records.push_back(ProfRecord{tag, work, unit, {}});
  return static_cast<int>(g_records.size()) - 1;
}

bool profiling_active() { return g_profiling; }

ProfScope::ProfScope(const char *tag, double work, WorkUnit unit) : slot(-1), outer(g_open_scope) {
  if (!g_profiling) return;
  slot = open_record(tag, work, unit);
  g_open_scope = slot;
}

ProfScope::ProfScope(const char *tag, int m, int n, int k) : slot(-1), outer(g_open_scope) {
  if (!g_profiling) return;
  char buf[160];
  std::snprintf(buf, sizeof(buf), "%s m=%d,n=%d,k=%d", tag, m, n, k);
  slot = open_record(buf, 2.0 * m * n * k, WORK_FLOP);
  g_open_scope = slot;
}

ProfScope::~ProfScope() {
  if (g_profiling) g_open_scope = outer;
}

void prof_launch_events(hipEvent_t *start, hipEvent_t *stop) {
  *start = *stop = nullptr;
  if (g_profiling) g_launch_order.push_back(g_open_scope);
  if (!g_profiling || g_open_scope < 0) return;
  hipEvent_t b = take_event(0), e = take_event(1);
  if (!b || !e) return;
  g_records[g_open_scope].launches.emplace_back(b, e);
  *start = b;
  *stop  = e;
}

// tiny_dnn/util/util.h:329-344
int conv_out_length(int in_length, int window, int stride, int dilation, int pad_same) {
  const int output_length = pad_same ? in_length : in_length - dilation * window + dilation;
  return (output_length + stride - 1) / stride;
}

// tiny_dnn/util/util.h:346-363: the quotient is formed in float, then floor/ceil
int pool_out_length(int in_length, int window, int stride, int ceil_mode, int pad_same) {
  const int output_length = pad_same ? in_length : in_length - window + 1;
  const float tmp = static_cast<float>(output_length + stride - 1) / static_cast<float>(stride);
  return static_cast<int>(ceil_mode ? std::ceil(tmp) : std::floor(tmp));
}

int check_conv_desc(const tdh_conv_desc *d, int batch, bool backward) {
  TDH_CHECK_ARG(d != nullptr, "conv: null descriptor");
  TDH_CHECK_ARG(batch >= 0, "conv: negative batch %d", batch);
  TDH_CHECK_ARG(d->in_w > 0 && d->in_h > 0 && d->in_c > 0 && d->out_c > 0 && d->k_w > 0 &&
                  d->k_h > 0,
                "conv: non-positive dimension");
  TDH_CHECK_ARG(d->w_stride > 0 && d->h_stride > 0 && d->w_dilation > 0 && d->h_dilation > 0,
                "conv: stride and dilation must be positive");
  if (backward && (d->w_dilation != 1 || d->h_dilation != 1))
    return set_error(TDH_ERR_UNSUPPORTED,
                     "conv backward with dilation %dx%d: the reference's backward kernel ignores "
                     "dilation, so no defined result exists to match",
                     d->w_dilation, d->h_dilation);
  if (d->pad_same && (d->w_dilation != 1 || d->h_dilation != 1))
    return set_error(TDH_ERR_UNSUPPORTED,
                     "conv with padding::same and dilation %dx%d: the reference pads by the undilated "
                     "window (convolutional_layer.h:470-474) and its kernel then reads past the padded "
                     "rows, so no defined result exists to match",
                     d->w_dilation, d->h_dilation);
  if (!d->pad_same)
    TDH_CHECK_ARG(d->in_w >= d->w_dilation * (d->k_w - 1) + 1 &&
                    d->in_h >= d->h_dilation * (d->k_h - 1) + 1,
                  "conv: window larger than the input");
  const long ow = conv_out_length(d->in_w, d->k_w, d->w_stride, d->w_dilation, d->pad_same);
  const long oh = conv_out_length(d->in_h, d->k_h, d->h_stride, d->h_dilation, d->pad_same);
  const long lim = 1L << 31;
  TDH_CHECK_ARG(static_cast<long>(batch) * d->in_c * d->in_h * d->in_w < lim &&
                  static_cast<long>(batch) * d->out_c * oh * ow < lim &&
                  static_cast<long>(d->out_c) * d->in_c * d->k_h * d->k_w < lim,
                "conv: tensor exceeds 2^31 elements");
  return TDH_OK;
}

static int check_pool_desc(const tdh_pool_desc *d, int batch) {
  TDH_CHECK_ARG(d != nullptr, "pool: null descriptor");
  TDH_CHECK_ARG(batch >= 0, "pool: negative batch %d", batch);
  TDH_CHECK_ARG(d->in_w > 0 && d->in_h > 0 && d->in_c > 0 && d->pool_w > 0 && d->pool_h > 0 &&
                  d->stride_w > 0 && d->stride_h > 0,
                "pool: non-positive dimension");
  if (!d->pad_same)
    TDH_CHECK_ARG(d->in_w >= d->pool_w && d->in_h >= d->pool_h, "pool: window larger than input");
  TDH_CHECK_ARG(static_cast<long>(batch) * d->in_c * d->in_h * d->in_w < (1L << 31),
                "pool: tensor exceeds 2^31 elements");
  return TDH_OK;
}

}  // namespace tdh

using namespace tdh;

extern "C" {

const char *tdh_version(void) { return "tdh 0.1 (gfx950)"; }

const char *tdh_last_error(void) { return g_error; }

int tdh_init(int device) {
  Context &c = ctx();
  if (c.ready && c.device == device) return TDH_OK;
  if (c.ready) TDH_TRY(tdh_shutdown());
  int count = 0;
  TDH_HIP(hipGetDeviceCount(&count));
  TDH_CHECK_ARG(device >= 0 && device < count, "tdh_init: device %d of %d", device, count);
  TDH_HIP(hipSetDevice(device));
  TDH_TRY(lookup_static_scratch(device));
  hipDeviceProp_t prop;
  TDH_HIP(hipGetDeviceProperties(&prop, device));
  std::snprintf(c.name, sizeof(c.name), "%s (%s)", prop.name, prop.gcnArchName);
  c.compute_units = prop.multiProcessorCount;
  c.global_mem    = prop.totalGlobalMem;
  TDH_HIP(hipStreamCreateWithFlags(&c.stream, hipStreamNonBlocking));
  c.device = device;
  c.ready  = true;
  read_gemm_plan_override();
  return TDH_OK;
}

int tdh_shutdown(void) {
  Context &c = ctx();
  if (!c.ready) return TDH_OK;
  TDH_HIP(hipStreamSynchronize(c.stream));
  if (c.workspace) TDH_HIP(hipFree(c.workspace));
  for (hipStream_t s : c.side)
    if (s) TDH_HIP(hipStreamDestroy(s));
  TDH_HIP(hipStreamDestroy(c.stream));
  c = Context();
  return TDH_OK;
}

int tdh_device_info(char *name, size_t name_len, int32_t *compute_units, size_t *global_mem_bytes) {
  TDH_REQUIRE_INIT();
  if (name && name_len) std::snprintf(name, name_len, "%s", ctx().name);
  if (compute_units) *compute_units = ctx().compute_units;
  if (global_mem_bytes) *global_mem_bytes = ctx().global_mem;
  return TDH_OK;
}

int tdh_malloc(void **dptr, size_t bytes) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(dptr != nullptr, "tdh_malloc: null result pointer");
  *dptr = nullptr;
  if (bytes == 0) bytes = 4;
  if (hipMalloc(dptr, bytes) != hipSuccess) {
    (void)hipGetLastError();
    return set_error(TDH_ERR_OOM, "tdh_malloc: cannot allocate %zu bytes", bytes);
  }
  return TDH_OK;
}

int tdh_free(void *dptr) {
  TDH_REQUIRE_INIT();
  if (dptr) TDH_HIP(hipFree(dptr));
  return TDH_OK;
}

int tdh_memcpy_h2d(void *dst, const void *src, size_t bytes) {
  TDH_REQUIRE_INIT();
  if (bytes == 0) return TDH_OK;
  TDH_CHECK_ARG(dst && src, "tdh_memcpy_h2d: null pointer");
  TDH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx().stream));
  TDH_HIP(hipStreamSynchronize(ctx().stream));  // the host buffer may be reused on return
  return TDH_OK;
}

int tdh_memcpy_d2h(void *dst, const void *src, size_t bytes) {
  TDH_REQUIRE_INIT();
  if (bytes == 0) return TDH_OK;
  TDH_CHECK_ARG(dst && src, "tdh_memcpy_d2h: null pointer");
  TDH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx().stream));
  TDH_HIP(hipStreamSynchronize(ctx().stream));
  return TDH_OK;
}

int tdh_memcpy_d2d(void *dst, const void *src, size_t bytes) {
  TDH_REQUIRE_INIT();
  if (bytes == 0) return TDH_OK;
  TDH_CHECK_ARG(dst && src, "tdh_memcpy_d2d: null pointer");
  // a kernel, not a DMA transfer, whenever it can be: safe under graph capture and visible in
  // kernel traces as a bandwidth yardstick
  if (bytes % 4 == 0 && reinterpret_cast<uintptr_t>(dst) % 4 == 0 && reinterpret_cast<uintptr_t>(src) % 4 == 0)
    return launch_copy(dst, src, bytes);
  TDH_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx().stream));
  return TDH_OK;
}

int tdh_fill_zero(void *dptr, size_t bytes) {
  TDH_REQUIRE_INIT();
  if (bytes == 0) return TDH_OK;
  TDH_CHECK_ARG(dptr != nullptr, "tdh_fill_zero: null pointer");
  TDH_CHECK_ARG(bytes % 4 == 0, "tdh_fill_zero: size %zu is not a multiple of 4", bytes);
  return launch_fill_zero(dptr, bytes);
}

int tdh_sync(void) {
  TDH_REQUIRE_INIT();
  TDH_HIP(hipStreamSynchronize(ctx().stream));
  return TDH_OK;
}

int tdh_event_create(void **event) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(event != nullptr, "tdh_event_create: null result pointer");
  hipEvent_t e;
  TDH_HIP(hipEventCreate(&e));
  *event = e;
  return TDH_OK;
}

int tdh_event_destroy(void *event) {
  TDH_REQUIRE_INIT();
  if (event) TDH_HIP(hipEventDestroy(static_cast<hipEvent_t>(event)));
  return TDH_OK;
}

int tdh_event_record(void *event) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(event != nullptr, "tdh_event_record: null event");
  TDH_HIP(hipEventRecord(static_cast<hipEvent_t>(event), ctx().stream));
  return TDH_OK;
}

int tdh_event_elapsed_ms(void *start, void *stop, float *ms) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(start && stop && ms, "tdh_event_elapsed_ms: null argument");
  TDH_HIP(hipEventSynchronize(static_cast<hipEvent_t>(stop)));
  TDH_HIP(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
  return TDH_OK;
}

int tdh_profile_begin(void) {
  TDH_REQUIRE_INIT();
  TDH_HIP(hipStreamSynchronize(ctx().stream));
  for (auto &r : g_records)
    for (auto &l : r.launches) {
      g_event_pool[0].push_back(l.first);
      g_event_pool[1].push_back(l.second);
    }
  g_records.clear();
  g_entries.clear();
  g_launch_order.clear();
  g_launch_tags.clear();
  g_open_scope = -1;
  g_profiling  = true;
  return TDH_OK;
}

int tdh_profile_end(int32_t *n_entries) {
  TDH_REQUIRE_INIT();
  g_profiling = false;
  TDH_HIP(hipStreamSynchronize(ctx().stream));
  std::map<std::string, ProfEntry> by_tag;
  g_open_scope = -1;
  g_launch_tags.clear();
  for (const int slot : g_launch_order)
    g_launch_tags.push_back(slot >= 0 && slot < static_cast<int>(g_records.size()) ? g_records[slot].tag : "-");
  g_launch_order.clear();
  for (auto &r : g_records) {
    if (r.launches.empty()) continue;  // a scope that launched nothing (its work was deferred)
    double ms_sum = 0.0;
    for (auto &l : r.launches) {
      float ms = 0.0f;
      TDH_HIP(hipEventElapsedTime(&ms, l.first, l.second));
      ms_sum += ms;
      g_event_pool[0].push_back(l.first);
      g_event_pool[1].push_back(l.second);
    }
    ProfEntry &e = by_tag[r.tag];
    e.tag        = r.tag;
    e.launches += 1;
    e.total_ms += ms_sum;
    e.work += r.work;
    e.unit = r.unit;
  }
  g_records.clear();
  g_entries.clear();
  for (auto &kv : by_tag) g_entries.push_back(kv.second);
  std::sort(g_entries.begin(), g_entries.end(),
            [](const ProfEntry &a, const ProfEntry &b) { return a.total_ms > b.total_ms; });
  if (n_entries) *n_entries = static_cast<int32_t>(g_entries.size());
  return TDH_OK;
}

int tdh_profile_entry(int32_t index, char *tag, size_t tag_len, int64_t *launches,
                      double *total_ms, double *work_per_launch, int32_t *work_unit) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(index >= 0 && index < static_cast<int32_t>(g_entries.size()),
                "tdh_profile_entry: index %d of %zu", index, g_entries.size());
  const ProfEntry &e = g_entries[index];
  if (tag && tag_len) std::snprintf(tag, tag_len, "%s", e.tag.c_str());
  if (launches) *launches = e.launches;
  if (total_ms) *total_ms = e.total_ms;
  if (work_per_launch) *work_per_launch = e.launches ? e.work / e.launches : 0.0;
  if (work_unit) *work_unit = e.unit;
  return TDH_OK;
}

int tdh_profile_mark(void *dptr, size_t bytes) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(dptr != nullptr && bytes >= 4 && bytes % 4 == 0,
                "tdh_profile_mark: needs a buffer of a positive multiple of 4 bytes");
  for (int i = 0; i < 3; ++i) TDH_TRY(launch_fill_zero(dptr, bytes, "profile_mark"));
  return TDH_OK;
}

int tdh_profile_launch(int32_t index, char *tag, size_t tag_len) {
  TDH_REQUIRE_INIT();
  if (index < 0 || index >= static_cast<int32_t>(g_launch_tags.size())) return TDH_ERR_INVALID;
  if (tag && tag_len) std::snprintf(tag, tag_len, "%s", g_launch_tags[index].c_str());
  return TDH_OK;
}

int tdh_conv_out_w(const tdh_conv_desc *d) {
  return conv_out_length(d->in_w, d->k_w, d->w_stride, d->w_dilation, d->pad_same);
}
int tdh_conv_out_h(const tdh_conv_desc *d) {
  return conv_out_length(d->in_h, d->k_h, d->h_stride, d->h_dilation, d->pad_same);
}
int tdh_pool_out_w(const tdh_pool_desc *d) {
  return pool_out_length(d->in_w, d->pool_w, d->stride_w, d->ceil_mode, d->pad_same);
}
int tdh_pool_out_h(const tdh_pool_desc *d) {
  return pool_out_length(d->in_h, d->pool_h, d->stride_h, d->ceil_mode, d->pad_same);
}

// ------------------------------------------------------------------ operators

int tdh_conv2d_fwd(const tdh_conv_desc *d, int batch, const float *x, const float *w,
                   const float *b, float *y) {
  TDH_REQUIRE_INIT();
  TDH_TRY(check_conv_desc(d, batch, false));
  if (batch == 0) return TDH_OK;
  TDH_CHECK_ARG(x && w && y, "tdh_conv2d_fwd: null tensor");
  TDH_CHECK_ARG(!d->has_bias || b, "tdh_conv2d_fwd: has_bias set but b is null");
  TDH_TRY(ws_begin(conv2d_workspace_bytes(d, batch)));
  return conv2d_fwd(d, batch, x, w, b, y);
}

int tdh_conv2d_bwd(const tdh_conv_desc *d, int batch, const float *x, const float *w,
                   const float *dy, float *dx, float *dw, float *db, int accumulate) {
  TDH_REQUIRE_INIT();
  TDH_TRY(check_conv_desc(d, batch, true));
  if (batch == 0) return TDH_OK;
  TDH_CHECK_ARG(x && w && dy, "tdh_conv2d_bwd: null tensor");
  TDH_TRY(ws_begin(conv2d_workspace_bytes(d, batch)));
  return conv2d_bwd(d, batch, x, w, dy, dx, dw, d->has_bias ? db : nullptr, accumulate, ActGrad());
}

int tdh_conv2d_bwd_static(const tdh_conv_desc *d, int batch, const float *x, const float *w,
                          const float *dy, float *dx, float *dw, float *db, int accumulate) {
  TDH_REQUIRE_INIT();
  TDH_TRY(check_conv_desc(d, batch, true));
  if (batch == 0) return TDH_OK;
  TDH_CHECK_ARG(x && w && dy, "tdh_conv2d_bwd_static: null tensor");
  // a connection table is uploaded from host memory through a staging copy that the call would
  // have to wait for: neither fits a caller that may not allocate or synchronize
  if (d->tbl)
    return set_error(TDH_ERR_UNSUPPORTED,
                     "tdh_conv2d_bwd_static: descriptors with a connection table are not served "
                     "(the table is staged through a host copy); use tdh_conv2d_bwd");
  Context &c = ctx();
  TDH_CHECK_ARG(!c.ws_keep && !c.ws_locked, "tdh_conv2d_bwd_static: called inside a network step");
  const size_t need = conv2d_workspace_bytes(d, batch);
  if (need > kStaticScratchBytes)
    return set_error(TDH_ERR_INVALID,
                     "tdh_conv2d_bwd_static: this shape needs %zu bytes of scratch, the static buffer "
                     "holds %zu; use tdh_conv2d_bwd",
                     need, kStaticScratchBytes);
  char *ptr = c.device >= 0 && c.device < kMaxDevices ? g_static_scratch[c.device] : nullptr;
  if (!ptr) return set_error(TDH_ERR_NOT_INIT, "tdh_conv2d_bwd_static: no static scratch on device %d", c.device);
  // Nothing in the array has to start at zero: every partial-sum slice, packed filter and
  // staged sum that a reduction reads is written in full by the launch in front of it, so the
  // previous call's contents are simply overwritten.
  StaticScratchScope scope(c, ptr);
  TDH_TRY(ws_begin(need));  // within the array by the test above; a locked scratch never allocates
  return conv2d_bwd(d, batch, x, w, dy, dx, dw, d->has_bias ? db : nullptr, accumulate, ActGrad());
}

int tdh_fc_fwd(int in, int out, int has_bias, int batch, const float *x, const float *w,
               const float *b, float *y) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(in > 0 && out > 0 && batch >= 0, "tdh_fc_fwd: bad shape %d->%d batch %d", in, out,
                batch);
  if (batch == 0) return TDH_OK;
  TDH_CHECK_ARG(x && w && y, "tdh_fc_fwd: null tensor");
  TDH_CHECK_ARG(!has_bias || b, "tdh_fc_fwd: has_bias set but b is null");
  TDH_CHECK_ARG(static_cast<long>(in) * out < (1L << 31) &&
                  static_cast<long>(batch) * in < (1L << 31) &&
                  static_cast<long>(batch) * out < (1L << 31),
                "tdh_fc_fwd: tensor exceeds 2^31 elements");
  TDH_TRY(ws_begin(fc_workspace_bytes(in, out, batch)));
  return fc_fwd(in, out, has_bias, batch, x, w, b, y);
}

int tdh_fc_bwd(int in, int out, int has_bias, int batch, const float *x, const float *w,
               const float *dy, float *dx, float *dw, float *db, int accumulate) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(in > 0 && out > 0 && batch >= 0, "tdh_fc_bwd: bad shape %d->%d batch %d", in, out,
                batch);
  if (batch == 0) return TDH_OK;
  TDH_CHECK_ARG(x && w && dy, "tdh_fc_bwd: null tensor");
  TDH_CHECK_ARG(static_cast<long>(in) * out < (1L << 31) &&
                  static_cast<long>(batch) * in < (1L << 31) &&
                  static_cast<long>(batch) * out < (1L << 31),
                "tdh_fc_bwd: tensor exceeds 2^31 elements");
  TDH_TRY(ws_begin(fc_workspace_bytes(in, out, batch)));
  return fc_bwd(in, out, has_bias, batch, x, w, dy, dx, dw, has_bias ? db : nullptr, accumulate,
                ActGrad());
}

int tdh_maxpool_fwd(const tdh_pool_desc *d, int batch, const float *x, float *y, int32_t *argmax) {
  TDH_REQUIRE_INIT();
  TDH_TRY(check_pool_desc(d, batch));
  if (batch == 0) return TDH_OK;
  TDH_CHECK_ARG(x && y, "tdh_maxpool_fwd: null tensor");
  return maxpool_fwd(d, batch, x, y, argmax);
}

int tdh_maxpool_bwd(const tdh_pool_desc *d, int batch, const float *dy, const int32_t *argmax,
                    float *dx) {
  TDH_REQUIRE_INIT();
  TDH_TRY(check_pool_desc(d, batch));
  if (batch == 0) return TDH_OK;
  TDH_CHECK_ARG(dy && argmax && dx, "tdh_maxpool_bwd: null tensor");
  return maxpool_bwd(d, batch, dy, argmax, dx);
}

int tdh_avepool_fwd(const tdh_pool_desc *d, int batch, const float *x, const float *w,
                    const float *b, float *y) {
  TDH_REQUIRE_INIT();
  TDH_TRY(check_pool_desc(d, batch));
  if (batch == 0) return TDH_OK;
  TDH_CHECK_ARG(x && w && b && y, "tdh_avepool_fwd: null tensor");
  return avepool_fwd(d, batch, x, w, b, y);
}

int tdh_avepool_bwd(const tdh_pool_desc *d, int batch, const float *x, const float *w,
                    const float *dy, float *dx, float *dw, float *db, int accumulate) {
  TDH_REQUIRE_INIT();
  TDH_TRY(check_pool_desc(d, batch));
  if (batch == 0) return TDH_OK;
  TDH_CHECK_ARG(x && w && dy, "tdh_avepool_bwd: null tensor");
  TDH_TRY(ws_begin(avepool_workspace_bytes(d, batch)));
  return avepool_bwd(d, batch, x, w, dy, dx, dw, db, accumulate);
}

void tdh_act_default_params(int kind, float *p) {
  if (!p) return;
  p[0] = p[1] = 0.0f;
  switch (kind) {
    case TDH_ACT_LEAKY_RELU: p[0] = 0.01f; break;                // leaky_relu_layer.h:25
    case TDH_ACT_ELU: p[0] = 1.0f; break;                        // elu_layer.h:18
    case TDH_ACT_SELU: p[0] = 1.05070f; p[1] = 1.67326f; break;  // selu_layer.h:26-27
    case TDH_ACT_SOFTPLUS: p[0] = 1.0f; p[1] = 20.0f; break;     // softplus_layer.h:26-27
  }
}

int tdh_act_fwd_p(int kind, const float *p, int batch, int len, const float *x, float *y) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(batch >= 0 && len >= 0, "tdh_act_fwd: negative size");
  if (batch == 0 || len == 0) return TDH_OK;
  TDH_CHECK_ARG(x && y, "tdh_act_fwd: null tensor");
  TDH_CHECK_ARG(static_cast<long>(batch) * len < (1L << 31), "tdh_act_fwd: tensor too large");
  float def[2];
  tdh_act_default_params(kind, def);
  return launch_act_fwd(kind, p ? p : def, batch, len, x, y);
}

int tdh_act_bwd_p(int kind, const float *p, int batch, int len, const float *x, const float *y,
                  const float *dy, float *dx) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(batch >= 0 && len >= 0, "tdh_act_bwd: negative size");
  if (batch == 0 || len == 0) return TDH_OK;
  TDH_CHECK_ARG(y && dy && dx, "tdh_act_bwd: null tensor");
  TDH_CHECK_ARG(static_cast<long>(batch) * len < (1L << 31), "tdh_act_bwd: tensor too large");
  float def[2];
  tdh_act_default_params(kind, def);
  return launch_act_bwd(kind, p ? p : def, batch, len, x, y, dy, dx);
}

int tdh_batchnorm_fwd(int channels, int spatial, int batch, float eps, int train, const float *x,
                      float *mean, float *variance, float *stddev, float *y) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(channels >= 0 && spatial >= 0 && batch >= 0, "tdh_batchnorm_fwd: negative size");
  if (channels == 0 || spatial == 0 || batch == 0) return TDH_OK;
  TDH_CHECK_ARG(x && y && mean && variance && stddev, "tdh_batchnorm_fwd: null tensor");
  TDH_CHECK_ARG(static_cast<long>(batch) * channels * spatial < (1L << 31), "tdh_batchnorm_fwd: tensor too large");
  TDH_TRY(ws_begin(batchnorm_workspace_bytes(channels, batch)));
  return batchnorm_fwd(channels, spatial, batch, eps, train, x, mean, variance, stddev, y);
}

int tdh_batchnorm_bwd(int channels, int spatial, int batch, const float *y, const float *dy,
                      const float *stddev, float *dx) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(channels >= 0 && spatial >= 0 && batch >= 0, "tdh_batchnorm_bwd: negative size");
  if (channels == 0 || spatial == 0 || batch == 0) return TDH_OK;
  TDH_CHECK_ARG(y && dy && stddev && dx, "tdh_batchnorm_bwd: null tensor");
  TDH_CHECK_ARG(static_cast<long>(batch) * channels * spatial < (1L << 31), "tdh_batchnorm_bwd: tensor too large");
  TDH_TRY(ws_begin(batchnorm_workspace_bytes(channels, batch)));
  return batchnorm_bwd(channels, spatial, batch, y, dy, stddev, dx);
}

int tdh_batchnorm_update_moving(int channels, float momentum, const float *mean_cur,
                                const float *var_cur, float *mean, float *variance) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(channels >= 0, "tdh_batchnorm_update_moving: negative size");
  if (channels == 0) return TDH_OK;
  TDH_CHECK_ARG(mean_cur && var_cur && mean && variance, "tdh_batchnorm_update_moving: null tensor");
  return batchnorm_update_moving(channels, momentum, mean_cur, var_cur, mean, variance);
}

int tdh_dropout_fwd(int batch, int len, int train, float scale, const uint8_t *mask, const float *x,
                    float *y) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(batch >= 0 && len >= 0, "tdh_dropout_fwd: negative size");
  if (batch == 0 || len == 0) return TDH_OK;
  TDH_CHECK_ARG(x && y && (mask || !train), "tdh_dropout_fwd: null tensor");
  return dropout_fwd(static_cast<size_t>(batch) * len, train, scale, mask, x, y);
}

int tdh_dropout_bwd(int batch, int len, const uint8_t *mask, const float *dy, float *dx) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(batch >= 0 && len >= 0, "tdh_dropout_bwd: negative size");
  if (batch == 0 || len == 0) return TDH_OK;
  TDH_CHECK_ARG(mask && dy && dx, "tdh_dropout_bwd: null tensor");
  return dropout_bwd(static_cast<size_t>(batch) * len, mask, dy, dx);
}

int tdh_act_fwd(int kind, int batch, int len, const float *x, float *y) {
  return tdh_act_fwd_p(kind, nullptr, batch, len, x, y);
}

int tdh_act_bwd(int kind, int batch, int len, const float *y, const float *dy, float *dx) {
  return tdh_act_bwd_p(kind, nullptr, batch, len, nullptr, y, dy, dx);
}

int tdh_loss_grad(int kind, int batch, int len, const float *y, const float *t, float *dy) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(batch >= 0 && len >= 0, "tdh_loss_grad: negative size");
  if (batch == 0 || len == 0) return TDH_OK;
  TDH_CHECK_ARG(y && t && dy, "tdh_loss_grad: null tensor");
  return launch_loss_grad(kind, batch, len, y, t, dy);
}

int tdh_softmax_xent_grad(int batch, int len, const float *y, const float *t, float *dz) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(batch >= 0 && len >= 0, "tdh_softmax_xent_grad: negative size");
  if (batch == 0 || len == 0) return TDH_OK;
  TDH_CHECK_ARG(y && t && dz, "tdh_softmax_xent_grad: null tensor");
  return launch_softmax_xent_grad(batch, len, y, t, dz);
}

// constructor defaults of tiny_dnn/optimizers/optimizer.h
void tdh_opt_default(tdh_opt *o, int kind) {
  std::memset(o, 0, sizeof(*o));
  o->kind = kind;
  switch (kind) {
    case TDH_OPT_SGD: o->alpha = 0.01f; break;
    case TDH_OPT_MOMENTUM:
    case TDH_OPT_NESTEROV: o->alpha = 0.01f; o->mu = 0.9f; break;
    case TDH_OPT_ADAM:
      o->alpha = 0.001f; o->b1 = 0.9f; o->b2 = 0.999f; o->b1_t = 0.9f; o->b2_t = 0.999f;
      o->eps = 1e-8f;
      break;
    case TDH_OPT_ADAGRAD: o->alpha = 0.01f; o->eps = 1e-8f; break;
    case TDH_OPT_RMSPROP: o->alpha = 0.0001f; o->mu = 0.99f; o->eps = 1e-8f; break;
    case TDH_OPT_ADAMAX:
      o->alpha = 0.002f; o->b1 = 0.9f; o->b2 = 0.999f; o->b1_t = 0.9f; o->eps = 1e-8f;
      break;
  }
}

int tdh_opt_update(tdh_opt *o, size_t n, const float *merged_grad, float grad_scale, float *w,
                   float *s0, float *s1) {
  TDH_REQUIRE_INIT();
  TDH_CHECK_ARG(o != nullptr, "tdh_opt_update: null optimizer");
  if (n == 0) return launch_opt_update(o, 0, nullptr, grad_scale, nullptr, nullptr, nullptr);
  TDH_CHECK_ARG(merged_grad && w, "tdh_opt_update: null tensor");
  return launch_opt_update(o, n, merged_grad, grad_scale, w, s0, s1);
}

}  // extern "C"

// C ABI of the backend: device, memory, kernels (hiprtc), events.  See include/ughip.h.
#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "internal.h"
#include "lower_hip.h"
#include "ughip.h"

namespace ughip {

static thread_local std::string g_last_error;

int set_error(int code, const char* fmt, ...) {
  char buf[4096];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_last_error = buf;
  // A failed HIP call also stays behind as the thread's "last error", and the next hipGetLastError() -- the
  // check after a <<<>>> launch -- would report it against a launch that went fine.  The failure is on record
  // here, so the runtime's copy is dropped.
  (void)hipGetLastError();
  return code;
}

static thread_local std::string g_last_kernel;

void note_kernel(const char* fmt, ...) {
  char buf[256];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_last_kernel = buf;
}

}  // namespace ughip

using namespace ughip;

// ---- handles -----------------------------------------------------------------------------
struct ughip_func {
  ughip_device* dev = nullptr;
  Lowered low;
  hipFunction_t function = nullptr, function2 = nullptr;
  void* scratch_part = nullptr;
};

struct ughip_event {
  ughip_device* dev = nullptr;
  hipEvent_t ev = nullptr;
};

namespace ughip {
int device_activate(ughip_device* d) {
  hipError_t e = hipSetDevice(d->ordinal);
  if (e != hipSuccess) return set_error(UGHIP_ERR_HIP, "hipSetDevice(%d): %s", d->ordinal, hipGetErrorString(e));
  return UGHIP_OK;
}
const char* dtype_name(int dt) {
  static const char* names[] = {"BF16", "F16", "F32", "I32", "I64"};
  return dt >= 0 && dt <= UGHIP_I64 ? names[dt] : "?";
}
}  // namespace ughip

#define HIPCHK UGHIP_HIPCHK

static size_t size_class(size_t bytes) {
  if (bytes <= 512) return 512;
  // 2^k * {1, 1.25, 1.5, 1.75}: at most 25% slack, few distinct sizes for growing tensors.
  size_t p = 512;
  while (p * 2 <= bytes) p *= 2;
  for (int q = 4; q <= 8; ++q) {
    size_t c = p / 4 * q;
    if (c >= bytes) return c;
  }
  return p * 2;
}

namespace ughip {
namespace {
const char* const kTuneNames[TUNE_COUNT] = {"GEMM_SHAPE", "GEMM_SPLIT", "GEMM_4WAVES", "GEMV_KS",        "GEMV_ROWS",   "GEMV_BF16_ROWS",
                                            "X3_DMA",     "X3_SPLIT", "X3_ROWS",   "ATT_SPLIT",   "NO_PARAMETRIC",  "NO_NT_LOADS", "GRID_REDUCE_BLOCKS", "GRID_REDUCE_THREADS", "NO_NT_STORES", "SOFTMAX_STREAM", "ATT_X6", "MATMUL_X6"};
constexpr long long kTuneUnset = INT64_MIN;
std::atomic<long long> g_tune[TUNE_COUNT];
std::once_flag g_tune_once;
void tune_init() {
  std::call_once(g_tune_once, [] {
    for (int k = 0; k < TUNE_COUNT; ++k) {
      const std::string name = std::string("UGHIP_") + kTuneNames[k];
      const char* e = getenv(name.c_str());
      g_tune[k].store(e ? strtoll(e, nullptr, 10) : kTuneUnset, std::memory_order_relaxed);
    }
  });
}
}  // namespace
bool tune_get(TuneKey k, long long* value) {
  tune_init();
  const long long v = g_tune[k].load(std::memory_order_relaxed);
  if (v == kTuneUnset) return false;
  *value = v;
  return true;
}
}  // namespace ughip

extern "C" {

const char* ughip_last_error(void) { return g_last_error.c_str(); }
const char* ughip_last_kernel(void) { return g_last_kernel.c_str(); }

int ughip_use_grid(void) { return 0; }

int ughip_set_tuning(const char* name, int set, int64_t value) {
  if (!name) return ughip::set_error(UGHIP_ERR_INVALID, "set_tuning: null name");
  ughip::tune_init();
  if (!strncmp(name, "UGHIP_", 6)) name += 6;
  for (int k = 0; k < ughip::TUNE_COUNT; ++k)
    if (!strcmp(name, ughip::kTuneNames[k])) {
      if (set && value == ughip::kTuneUnset) return ughip::set_error(UGHIP_ERR_INVALID, "set_tuning: value out of range");
      ughip::g_tune[k].store(set ? value : ughip::kTuneUnset, std::memory_order_relaxed);
      return UGHIP_OK;
    }
  return ughip::set_error(UGHIP_ERR_INVALID, "set_tuning: no switch named '%s'", name);
}

int ughip_device_create(int ordinal, ughip_device** out) {
  ughip::tune_init();
  if (!out) return set_error(UGHIP_ERR_INVALID, "null out pointer");
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count <= 0)
    return set_error(UGHIP_ERR_HIP, "no HIP device available (%s)", e == hipSuccess ? "count is 0" : hipGetErrorString(e));
  if (ordinal < 0 || ordinal >= count) return set_error(UGHIP_ERR_INVALID, "device ordinal %d out of range (%d devices)", ordinal, count);
  HIPCHK(hipSetDevice(ordinal));
  std::unique_ptr<ughip_device> d(new ughip_device);
  d->ordinal = ordinal;
  hipDeviceProp_t prop;
  HIPCHK(hipGetDeviceProperties(&prop, ordinal));
  d->arch = prop.gcnArchName;
  d->num_cus = prop.multiProcessorCount;
  size_t colon = d->arch.find(':');
  if (colon != std::string::npos) d->arch.resize(colon);
  HIPCHK(hipStreamCreateWithFlags(&d->stream, hipStreamNonBlocking));
  if (int rc = matmul_scratch_setup(d.get())) {
    hipStreamDestroy(d->stream);
    return rc;
  }
  *out = d.release();
  return UGHIP_OK;
}

int ughip_device_retain(ughip_device* dev) {
  if (!dev) return set_error(UGHIP_ERR_INVALID, "null device");
  dev->refs.fetch_add(1);
  return UGHIP_OK;
}

int ughip_device_release(ughip_device* dev) {
  if (!dev) return set_error(UGHIP_ERR_INVALID, "null device");
  if (dev->refs.fetch_sub(1) != 1) return UGHIP_OK;
  hipSetDevice(dev->ordinal);
  hipStreamSynchronize(dev->stream);
  if (dev->gemm_ws) hipFree(dev->gemm_ws);
  if (dev->att_ws) hipFree(dev->att_ws);
  if (dev->rows_ws) hipFree(dev->rows_ws);
  for (auto& kv : dev->pool)
    for (void* p : kv.second) hipFree(p);
  for (auto& kv : dev->modules) hipModuleUnload(kv.second.module);
  hipStreamDestroy(dev->stream);
  delete dev;
  return UGHIP_OK;
}

int ughip_synchronize(ughip_device* dev) {
  if (!dev) return set_error(UGHIP_ERR_INVALID, "null device");
  if (int rc = device_activate(dev)) return rc;
  HIPCHK(hipStreamSynchronize(dev->stream));
  return UGHIP_OK;
}

int ughip_device_set_zero_fill(ughip_device* dev, int on) {
  if (!dev) return set_error(UGHIP_ERR_INVALID, "null device");
  dev->zero_fill = on != 0;
  return UGHIP_OK;
}

int ughip_device_stats(ughip_device* dev, size_t* n_code_objects, size_t* pool_bytes, size_t* live_bytes) {
  if (!dev) return set_error(UGHIP_ERR_INVALID, "null device");
  std::lock_guard<std::mutex> g(dev->mu);
  if (n_code_objects) *n_code_objects = dev->modules.size();
  if (pool_bytes) *pool_bytes = dev->pool_bytes;
  if (live_bytes) *live_bytes = dev->live_bytes;
  return UGHIP_OK;
}

int ughip_device_arch(ughip_device* dev, char* buf, size_t buf_len) {
  if (!dev || !buf || !buf_len) return set_error(UGHIP_ERR_INVALID, "bad arguments");
  snprintf(buf, buf_len, "%s", dev->arch.c_str());
  return UGHIP_OK;
}

// ---- memory --------------------------------------------------------------------------------
int ughip_alloc(ughip_device* dev, int dtype, size_t len, ughip_slice** out) {
  if (!dev || !out) return set_error(UGHIP_ERR_INVALID, "null device/out");
  if (dtype < UGHIP_BF16 || dtype > UGHIP_I64) return set_error(UGHIP_ERR_INVALID, "unknown dtype %d", dtype);
  if (int rc = device_activate(dev)) return rc;
  std::unique_ptr<ughip_slice> s(new ughip_slice);
  s->dev = dev;
  s->dtype = dtype;
  s->len = len;
  if (len > SIZE_MAX / dtype_size(dtype)) return set_error(UGHIP_ERR_INVALID, "alloc: %zu elements of %s overflow size_t", len, dtype_name(dtype));
  size_t bytes = len * dtype_size(dtype);
  if (bytes) {
    size_t cls = size_class(bytes);
    {
      std::lock_guard<std::mutex> g(dev->mu);
      auto it = dev->pool.find(cls);
      if (it != dev->pool.end() && !it->second.empty()) {
        s->ptr = it->second.back();
        it->second.pop_back();
        dev->pool_bytes -= cls;
      }
    }
    if (!s->ptr) {
      hipError_t e = hipMalloc(&s->ptr, cls);
      if (e != hipSuccess) {
        // Give cached blocks back to the driver and retry once.
        (void)hipGetLastError();  // the retry may succeed: the failed attempt must not surface at a later launch check
        std::lock_guard<std::mutex> g(dev->mu);
        hipStreamSynchronize(dev->stream);
        for (auto& kv : dev->pool)
          for (void* p : kv.second) hipFree(p);
        dev->pool.clear();
        dev->pool_bytes = 0;
        e = hipMalloc(&s->ptr, cls);
        if (e != hipSuccess) return set_error(UGHIP_ERR_HIP, "hipMalloc(%zu): %s", cls, hipGetErrorString(e));
      }
    }
    s->cap_bytes = cls;
    {
      std::lock_guard<std::mutex> g(dev->mu);
      dev->live_bytes += cls;
    }
    if (dev->zero_fill) {
      hipError_t e = hipMemsetAsync(s->ptr, 0, bytes, dev->stream);
      if (e != hipSuccess) {
        // the block goes back to the pool and out of the live count, as ughip_free would do
        std::lock_guard<std::mutex> g(dev->mu);
        dev->pool[cls].push_back(s->ptr);
        dev->pool_bytes += cls;
        dev->live_bytes -= cls;
        return set_error(UGHIP_ERR_HIP, "hipMemsetAsync(%zu): %s", bytes, hipGetErrorString(e));
      }
    }
  }
  ughip_device_retain(dev);
  *out = s.release();
  return UGHIP_OK;
}

int ughip_free(ughip_slice* s) {
  if (!s) return UGHIP_OK;
  ughip_device* dev = s->dev;
  if (s->ptr) {
    std::lock_guard<std::mutex> g(dev->mu);
    dev->pool[s->cap_bytes].push_back(s->ptr);
    dev->pool_bytes += s->cap_bytes;
    dev->live_bytes -= s->cap_bytes;
  }
  delete s;
  ughip_device_release(dev);
  return UGHIP_OK;
}

size_t ughip_slice_len(const ughip_slice* s) { return s ? s->len : 0; }
int ughip_slice_dtype(const ughip_slice* s) { return s ? s->dtype : -1; }
void* ughip_slice_ptr(const ughip_slice* s) { return s ? s->ptr : nullptr; }

int ughip_h2d(ughip_slice* dst, const void* src, int dtype, size_t len) {
  if (!dst) return set_error(UGHIP_ERR_INVALID, "null slice");
  if (len != dst->len) return set_error(UGHIP_ERR_INVALID, "htod len mismatch, dst %zu, len %zu", dst->len, len);
  if (dtype != dst->dtype) return set_error(UGHIP_ERR_INVALID, "htod dtype mismatch, dst %s, src %s", dtype_name(dst->dtype), dtype_name(dtype));
  if (!len) return UGHIP_OK;
  if (!src) return set_error(UGHIP_ERR_INVALID, "null host pointer");
  if (int rc = device_activate(dst->dev)) return rc;
  HIPCHK(hipMemcpyAsync(dst->ptr, src, len * dtype_size(dtype), hipMemcpyHostToDevice, dst->dev->stream));
  HIPCHK(hipStreamSynchronize(dst->dev->stream));
  return UGHIP_OK;
}

int ughip_d2h(const ughip_slice* src, void* dst, int dtype, size_t len) {
  if (!src) return set_error(UGHIP_ERR_INVALID, "null slice");
  if (len != src->len) return set_error(UGHIP_ERR_INVALID, "dtoh len mismatch, dst %zu, len %zu", len, src->len);
  if (dtype != src->dtype) return set_error(UGHIP_ERR_INVALID, "dtoh dtype mismatch, dst %s, src %s", dtype_name(dtype), dtype_name(src->dtype));
  if (!len) return UGHIP_OK;
  if (!dst) return set_error(UGHIP_ERR_INVALID, "null host pointer");
  if (int rc = device_activate(src->dev)) return rc;
  HIPCHK(hipMemcpyAsync(dst, src->ptr, len * dtype_size(dtype), hipMemcpyDeviceToHost, src->dev->stream));
  HIPCHK(hipStreamSynchronize(src->dev->stream));
  return UGHIP_OK;
}

// ---- kernels -----------------------------------------------------------------------------------
static std::string sanitize_name(const char* name) {
  std::string s = "ug_";
  if (name)
    for (const char* p = name; *p && s.size() < 60; ++p) s += (isalnum((unsigned char)*p) || *p == '_') ? *p : '_';
  else
    s += "kernel";
  return s;
}

static int lower_checked(const ughip_ssa* ssa, const char* name, Lowered* out, bool as_written = false) {
  if (!ssa) return set_error(UGHIP_ERR_INVALID, "null ssa");
  try {
    *out = lower_ssa(*ssa, as_written && name && *name ? std::string(name) : sanitize_name(name), as_written);
  } catch (const std::exception& e) {
    return set_error(UGHIP_ERR_COMPILE, "%s", e.what());
  }
  return UGHIP_OK;
}

int ughip_codegen(const ughip_ssa* ssa, const char* name, char* buf, size_t buf_len, size_t* out_len, ughip_func_info* info) {
  Lowered low;
  if (int rc = lower_checked(ssa, name, &low)) return rc;
  if (out_len) *out_len = low.source.size();
  if (buf && buf_len) {
    size_t n = std::min(buf_len - 1, low.source.size());
    memcpy(buf, low.source.data(), n);
    buf[n] = 0;
  }
  if (info) {
    info->strategy = low.strategy;
    info->grid_dim = low.grid;
    info->block_dim = low.block;
    info->lds_bytes = low.lds_bytes;
    info->scratch_bytes = low.scratch_part_bytes;
  }
  return UGHIP_OK;
}

int ughip_codegen_min_len(const ughip_ssa* ssa, int64_t* min_len, size_t n_args) {
  Lowered low;
  if (int rc = lower_checked(ssa, nullptr, &low)) return rc;
  if (!min_len || n_args != low.min_len.size()) return set_error(UGHIP_ERR_INVALID, "codegen_min_len: the kernel has %zu arguments, room for %zu given", low.min_len.size(), n_args);
  for (size_t a = 0; a < n_args; ++a) min_len[a] = low.min_len[a];
  return UGHIP_OK;
}

int ughip_codegen_as_written(const ughip_ssa* ssa, const char* name, char* buf, size_t buf_len, size_t* out_len) {
  Lowered low;
  if (name) {
    if (!*name) return set_error(UGHIP_ERR_INVALID, "codegen: empty kernel name");
    for (const char* c = name; *c; ++c)
      if (!(*c == '_' || (*c >= 'a' && *c <= 'z') || (*c >= 'A' && *c <= 'Z') || (c != name && *c >= '0' && *c <= '9')))
        return set_error(UGHIP_ERR_INVALID, "codegen: '%s' is not a valid kernel name", name);
  }
  if (int rc = lower_checked(ssa, name, &low, true)) return rc;
  if (out_len) *out_len = low.source.size();
  if (buf && buf_len) {
    size_t n = std::min(buf_len - 1, low.source.size());
    memcpy(buf, low.source.data(), n);
    buf[n] = 0;
  }
  return UGHIP_OK;
}

// hiprtc: source -> gfx950 code object.
static int rtc_compile(const std::string& source, const std::string& arch, std::vector<char>* code) {
  hiprtcProgram prog;
  hiprtcResult r = hiprtcCreateProgram(&prog, source.c_str(), "ug_kernel.hip", 0, nullptr, nullptr);
  if (r != HIPRTC_SUCCESS) return set_error(UGHIP_ERR_COMPILE, "hiprtcCreateProgram: %s", hiprtcGetErrorString(r));
  std::string arch_opt = "--offload-arch=" + arch;
  const char* opts[] = {arch_opt.c_str(), "-O3", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
  r = hiprtcCompileProgram(prog, (int)(sizeof opts / sizeof opts[0]), opts);
  if (r != HIPRTC_SUCCESS) {
    size_t ls = 0;
    hiprtcGetProgramLogSize(prog, &ls);
    std::string log(ls, 0);
    if (ls) hiprtcGetProgramLog(prog, &log[0]);
    hiprtcDestroyProgram(&prog);
    return set_error(UGHIP_ERR_COMPILE, "compilation failed: %s\n%s", hiprtcGetErrorString(r), log.c_str());
  }
  size_t cs = 0;
  hiprtcGetCodeSize(prog, &cs);
  code->resize(cs);
  hiprtcGetCode(prog, code->data());
  hiprtcDestroyProgram(&prog);
  return UGHIP_OK;
}

// Exposed for CPU-side tests: compile a generated source for `arch` without a device.
int ughip_rtc_check(const char* source, const char* arch, size_t* code_size) {
  std::vector<char> code;
  if (int rc = rtc_compile(source ? source : "", arch ? arch : "gfx950", &code)) return rc;
  if (code_size) *code_size = code.size();
  return UGHIP_OK;
}

int ughip_compile(ughip_device* dev, const ughip_ssa* ssa, const char* name, ughip_func** out) {
  if (!dev || !out) return set_error(UGHIP_ERR_INVALID, "null device/out");
  if (int rc = device_activate(dev)) return rc;
  std::unique_ptr<ughip_func> f(new ughip_func);
  f->dev = dev;
  if (int rc = lower_checked(ssa, name, &f->low)) return rc;
  if (f->low.grid == 0) f->low.empty_launch = true;
  if (!f->low.empty_launch) {
    std::lock_guard<std::mutex> g(dev->mu);
    auto it = dev->modules.find(f->low.source);
    if (it == dev->modules.end()) {
      std::vector<char> code;
      if (int rc = rtc_compile(f->low.source, dev->arch, &code)) return rc;
      CachedModule cm;
      HIPCHK(hipModuleLoadData(&cm.module, code.data()));
      hipError_t e = hipModuleGetFunction(&cm.function, cm.module, f->low.entry.c_str());
      if (e == hipSuccess && !f->low.entry2.empty()) e = hipModuleGetFunction(&cm.function2, cm.module, f->low.entry2.c_str());
      if (e != hipSuccess) {
        hipModuleUnload(cm.module);
        return set_error(UGHIP_ERR_HIP, "hipModuleGetFunction(%s): %s", f->low.entry.c_str(), hipGetErrorString(e));
      }
      it = dev->modules.emplace(f->low.source, cm).first;
    }
    f->function = it->second.function;
    f->function2 = it->second.function2;
  }
  if (f->low.scratch_part_bytes) HIPCHK(hipMalloc(&f->scratch_part, f->low.scratch_part_bytes));
  ughip_device_retain(dev);
  *out = f.release();
  return UGHIP_OK;
}

int ughip_compile_source(ughip_device* dev, const char* source, const char* entry, size_t n_args, const int* arg_dtypes, unsigned grid_dim,
                         unsigned block_dim, unsigned shared_mem_bytes, ughip_func** out) {
  if (!dev || !out || !source || !entry || (n_args && !arg_dtypes)) return set_error(UGHIP_ERR_INVALID, "compile_source: null argument");
  if (n_args > 64) return set_error(UGHIP_ERR_INVALID, "compile_source: %zu arguments, at most 64 are supported", n_args);
  if (block_dim == 0 || block_dim > 1024) return set_error(UGHIP_ERR_INVALID, "compile_source: block_dim %u is not in 1..1024", block_dim);
  if (shared_mem_bytes > 160 * 1024) return set_error(UGHIP_ERR_INVALID, "compile_source: %u bytes of LDS, a workgroup has 160 KiB", shared_mem_bytes);
  for (size_t a = 0; a < n_args; ++a)
    if (arg_dtypes[a] < 0 || arg_dtypes[a] > UGHIP_I64) return set_error(UGHIP_ERR_INVALID, "compile_source: unknown dtype %d for argument %zu", arg_dtypes[a], a);
  if (int rc = device_activate(dev)) return rc;
  std::unique_ptr<ughip_func> f(new ughip_func);
  f->dev = dev;
  Lowered& low = f->low;
  low.source = source;
  low.entry = entry;
  low.strategy = UGHIP_STRAT_LITERAL;
  low.grid = grid_dim;
  low.block = block_dim;
  low.lds_bytes = shared_mem_bytes;
  low.arg_dtype.assign(arg_dtypes, arg_dtypes + n_args);
  low.min_len.assign(n_args, -1);     // what the source indexes is not known here
  low.arg_written.assign(n_args, 1);  // nor what it writes: no slice may be passed twice
  low.empty_launch = grid_dim == 0;
  {
    std::lock_guard<std::mutex> g(dev->mu);
    const std::string key = low.source + "\n// entry " + low.entry;
    auto it = dev->modules.find(key);
    if (it == dev->modules.end()) {
      std::vector<char> code;
      if (int rc = rtc_compile(low.source, dev->arch, &code)) return rc;
      CachedModule cm;
      HIPCHK(hipModuleLoadData(&cm.module, code.data()));
      hipError_t e = hipModuleGetFunction(&cm.function, cm.module, low.entry.c_str());
      if (e != hipSuccess) {
        hipModuleUnload(cm.module);
        return set_error(UGHIP_ERR_COMPILE, "compile_source: no kernel '%s' in the source (declare it extern \"C\" __global__): %s", low.entry.c_str(),
                         hipGetErrorString(e));
      }
      it = dev->modules.emplace(key, cm).first;
    }
    f->function = it->second.function;
  }
  ughip_device_retain(dev);
  *out = f.release();
  return UGHIP_OK;
}

int ughip_func_release(ughip_func* f) {
  if (!f) return UGHIP_OK;
  ughip_device* dev = f->dev;
  if (f->scratch_part) {
    hipSetDevice(dev->ordinal);
    hipStreamSynchronize(dev->stream);
    hipFree(f->scratch_part);
  }
  delete f;
  ughip_device_release(dev);
  return UGHIP_OK;
}

size_t ughip_func_source(const ughip_func* f, char* buf, size_t buf_len) {
  if (!f) return 0;
  if (buf && buf_len) {
    size_t n = std::min(buf_len - 1, f->low.source.size());
    memcpy(buf, f->low.source.data(), n);
    buf[n] = 0;
  }
  return f->low.source.size();
}

int ughip_func_get_info(const ughip_func* f, ughip_func_info* out) {
  if (!f || !out) return set_error(UGHIP_ERR_INVALID, "null func/out");
  out->strategy = f->low.strategy;
  out->grid_dim = f->low.grid;
  out->block_dim = f->low.block;
  out->lds_bytes = f->low.lds_bytes;
  out->scratch_bytes = f->low.scratch_part_bytes;
  return UGHIP_OK;
}

// which: 0 = every launch of the func, 1 / 2 = only its first / second kernel (timing aid).
static int run_impl(ughip_device* dev, ughip_func* f, ughip_slice* const* args, size_t n_args, int which) {
  if (!dev || !f) return set_error(UGHIP_ERR_INVALID, "null device/func");
  if (f->dev != dev) return set_error(UGHIP_ERR_INVALID, "func was compiled for another device");
  const Lowered& low = f->low;
  if (n_args != low.arg_dtype.size()) return set_error(UGHIP_ERR_INVALID, "kernel %s expects %zu args, got %zu", low.entry.c_str(), low.arg_dtype.size(), n_args);
  if (low.empty_launch) return UGHIP_OK;
  void* ptrs[64];
  void* params[66];
  if (n_args > 64) return set_error(UGHIP_ERR_INVALID, "unsupported number of args for kernel %zu", n_args);
  for (size_t a = 0; a < n_args; ++a) {
    const ughip_slice* s = args[a];
    if (!s) return set_error(UGHIP_ERR_INVALID, "null slice for arg %zu", a);
    if (s->dev != dev) return set_error(UGHIP_ERR_INVALID, "arg %zu lives on another device", a);
    if (s->dtype != low.arg_dtype[a])
      return set_error(UGHIP_ERR_INVALID, "arg %zu of %s: dtype %s, kernel expects %s", a, low.entry.c_str(), dtype_name(s->dtype), dtype_name(low.arg_dtype[a]));
    if (low.min_len[a] > 0 && (long long)s->len < low.min_len[a])
      return set_error(UGHIP_ERR_BOUNDS, "arg %zu of %s: slice has %zu elements, kernel indexes up to %lld", a, low.entry.c_str(), s->len, low.min_len[a] - 1);
    for (size_t b = 0; b < a; ++b)
      if (args[b] == s && (low.arg_written[a] || low.arg_written[b]))
        return set_error(UGHIP_ERR_INVALID, "arg %zu and %zu of %s alias the same slice (already borrowed)", b, a, low.entry.c_str());
    ptrs[a] = s->ptr;
    params[a] = &ptrs[a];
  }
  size_t np = n_args;
  if (low.scratch_part_bytes) params[np++] = &f->scratch_part;
  if (!low.kparams.empty()) params[np++] = const_cast<int*>(low.kparams.data());
  if (int rc = device_activate(dev)) return rc;
  if (which != 2) HIPCHK(hipModuleLaunchKernel(f->function, low.grid, 1, 1, low.block, 1, 1, low.lds_bytes, dev->stream, params, nullptr));
  if (f->function2 && which != 1) HIPCHK(hipModuleLaunchKernel(f->function2, low.grid2, 1, 1, low.block2, 1, 1, 0, dev->stream, params, nullptr));
  return UGHIP_OK;
}

int ughip_run(ughip_device* dev, ughip_func* f, ughip_slice* const* args, size_t n_args) { return run_impl(dev, f, args, n_args, 0); }

int ughip_run_part(ughip_device* dev, ughip_func* f, ughip_slice* const* args, size_t n_args, int part) {
  if (part != 1 && part != 2) return set_error(UGHIP_ERR_INVALID, "run_part: part is 1 or 2, got %d", part);
  if (f && part == 2 && !f->function2) return set_error(UGHIP_ERR_INVALID, "run_part: %s is a single kernel", f->low.entry.c_str());
  return run_impl(dev, f, args, n_args, part);
}

// ---- events --------------------------------------------------------------------------------------
int ughip_event_create(ughip_device* dev, ughip_event** out) {
  if (!dev || !out) return set_error(UGHIP_ERR_INVALID, "null device/out");
  if (int rc = device_activate(dev)) return rc;
  std::unique_ptr<ughip_event> e(new ughip_event);
  e->dev = dev;
  HIPCHK(hipEventCreate(&e->ev));
  *out = e.release();
  return UGHIP_OK;
}

int ughip_event_record(ughip_event* ev) {
  if (!ev) return set_error(UGHIP_ERR_INVALID, "null event");
  if (int rc = device_activate(ev->dev)) return rc;
  HIPCHK(hipEventRecord(ev->ev, ev->dev->stream));
  return UGHIP_OK;
}

int ughip_event_elapsed_ms(ughip_event* start, ughip_event* stop, float* ms) {
  if (!start || !stop || !ms) return set_error(UGHIP_ERR_INVALID, "null event/out");
  if (int rc = device_activate(stop->dev)) return rc;
  HIPCHK(hipEventSynchronize(stop->ev));
  HIPCHK(hipEventElapsedTime(ms, start->ev, stop->ev));
  return UGHIP_OK;
}

int ughip_event_destroy(ughip_event* ev) {
  if (!ev) return UGHIP_OK;
  hipSetDevice(ev->dev->ordinal);
  hipEventDestroy(ev->ev);
  delete ev;
  return UGHIP_OK;
}

}  // extern "C"

// Handle, stream and memory entry points of the runtime
// (reference: src/Tools/dnn-wrapper/cuda/wrapDNN*.cpp and the
// cudnnCreate/cudaStreamCreate rows of DNNAPISpecs.inc:92-95).
#include "common.h"

#include <stdarg.h>
#include <string.h>

#include <mutex>
#include <unordered_map>

namespace dnnrt {
static thread_local char g_err[512] = "";
void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof g_err, fmt, ap);
  va_end(ap);
}
}  // namespace dnnrt

using dnnrt::set_error;

namespace dnnrt {
// 16 bytes per thread, byte stores at the ragged ends (a slot's address is 32-byte aligned, its size is not)
__global__ __launch_bounds__(256) void fill_bytes_kernel(unsigned char *p, unsigned char byte, int64_t n) {
  const int64_t at = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 16;
  if (at >= n) return;
  if (at + 16 <= n && (reinterpret_cast<uintptr_t>(p + at) & 15u) == 0) {
    const unsigned w = byte * 0x01010101u;
    *reinterpret_cast<uint4 *>(p + at) = make_uint4(w, w, w, w);
  } else {
    for (int64_t i = at; i < n && i < at + 16; i++) p[i] = byte;
  }
}
}  // namespace dnnrt

namespace dnnrt {
// Every byte this library takes from the device allocator, counted: the pool, dnnrtMalloc, and a handle's
// reduction scratch when it cannot have the static one.
static std::mutex g_mem_mutex;
static std::unordered_map<void *, int64_t> g_mem_sizes;
static int64_t g_mem_now = 0, g_mem_peak = 0;

static hipError_t counted_malloc(void **ptr, int64_t bytes) {
  const int64_t n = bytes > 0 ? bytes : 1;
  hipError_t e = hipMalloc(ptr, (size_t)n);
  if (e != hipSuccess) return e;
  std::lock_guard<std::mutex> lock(g_mem_mutex);
  g_mem_sizes[*ptr] = n;
  g_mem_now += n;
  if (g_mem_now > g_mem_peak) g_mem_peak = g_mem_now;
  return e;
}
static hipError_t counted_free(void *ptr) {
  if (ptr) {
    std::lock_guard<std::mutex> lock(g_mem_mutex);
    auto it = g_mem_sizes.find(ptr);
    if (it != g_mem_sizes.end()) { g_mem_now -= it->second; g_mem_sizes.erase(it); }
  }
  return hipFree(ptr);
}

// The reduction scratch of a handle (partial tiles, then arrival counters) is a static array of the library: part
// of the loaded code object, so creating a handle takes nothing from the device allocator and a program's device
// memory is its pool.  One handle per device holds it at a time; a handle created while another one has it gets
// buffers of its own from the allocator (and those are counted).
constexpr int64_t HANDLE_SCRATCH_BYTES = SPLITK_PARTIAL_BYTES + (int64_t)SPLITK_MAX_TILES * sizeof(unsigned);
static __device__ __align__(256) unsigned char handle_scratch[HANDLE_SCRATCH_BYTES];
constexpr int MAX_DEVICES = 64;
static unsigned char *g_scratch_at[MAX_DEVICES];      // this device's copy of handle_scratch
static const dnnrtContext *g_scratch_holder[MAX_DEVICES];
static std::mutex g_scratch_mutex;
}  // namespace dnnrt

#define HIP_RET(call, what)                                                    \
  do {                                                                         \
    hipError_t e_ = (call);                                                    \
    if (e_ != hipSuccess) {                                                    \
      set_error("%s: %s", what, hipGetErrorString(e_));                        \
      return (int32_t)e_;                                                      \
    }                                                                          \
  } while (0)

extern "C" {

const char *dnnrtLastError(void) { return dnnrt::g_err; }
int32_t dnnrtIsHostBackend(void) { return 0; }

int32_t dnnrtCreate(dnnrtHandle_t *handle) {
  if (!handle) { set_error("dnnrtCreate: null handle pointer"); return 1; }
  int dev = 0;
  HIP_RET(hipGetDevice(&dev), "dnnrtCreate: hipGetDevice");
  hipDeviceProp_t prop;
  HIP_RET(hipGetDeviceProperties(&prop, dev), "dnnrtCreate: hipGetDeviceProperties");
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    set_error("dnnrtCreate: this library holds gfx950 code only, device is %s", prop.gcnArchName);
    return 1;
  }
  dnnrtContext *c = new dnnrtContext();
  c->stream = nullptr;
  c->format = DNNRT_NCHW;
  c->filter_layout = DNNRT_FILTER_KCRS;
  c->act_coef = 0.f;
  c->device = dev;
  c->num_cu = prop.multiProcessorCount;
  c->splitk_partials = nullptr;
  c->splitk_counters = nullptr;
  c->scratch_is_static = false;
  if (dev >= 0 && dev < dnnrt::MAX_DEVICES) {
    std::lock_guard<std::mutex> lock(dnnrt::g_scratch_mutex);
    if (!dnnrt::g_scratch_holder[dev]) {
      if (!dnnrt::g_scratch_at[dev]) {
        void *at = nullptr;
        hipError_t e = hipGetSymbolAddress(&at, HIP_SYMBOL(dnnrt::handle_scratch));
        if (e != hipSuccess || !at) {
          set_error("dnnrtCreate: hipGetSymbolAddress: %s", hipGetErrorString(e));
          delete c;
          return 1;
        }
        dnnrt::g_scratch_at[dev] = static_cast<unsigned char *>(at);
      }
      c->splitk_partials = reinterpret_cast<float *>(dnnrt::g_scratch_at[dev]);
      c->splitk_counters = reinterpret_cast<unsigned *>(dnnrt::g_scratch_at[dev] + dnnrt::SPLITK_PARTIAL_BYTES);
      c->scratch_is_static = true;
      dnnrt::g_scratch_holder[dev] = c;
    }
  }
  if ((!c->scratch_is_static &&
       (dnnrt::counted_malloc((void **)&c->splitk_partials, dnnrt::SPLITK_PARTIAL_BYTES) != hipSuccess ||
        dnnrt::counted_malloc((void **)&c->splitk_counters, dnnrt::SPLITK_MAX_TILES * sizeof(unsigned)) != hipSuccess)) ||
      hipMemset(c->splitk_counters, 0, dnnrt::SPLITK_MAX_TILES * sizeof(unsigned)) != hipSuccess) {
    set_error("dnnrtCreate: cannot set up the handle's reduction scratch");
    dnnrtDestroy(c);
    return 1;
  }
  c->splitk_partial_bytes = dnnrt::SPLITK_PARTIAL_BYTES;
  c->splitk_max_tiles = dnnrt::SPLITK_MAX_TILES;
  c->splitk_shared = false;
  c->f16_tile = 0;
  *handle = c;
  return 0;
}

int32_t dnnrtDestroy(dnnrtHandle_t handle) {
  if (handle) {
    if (handle->scratch_is_static) {
      (void)hipDeviceSynchronize();  // the next holder must not meet this handle's kernels (hipFree waits likewise)
      std::lock_guard<std::mutex> lock(dnnrt::g_scratch_mutex);
      if (handle->device >= 0 && handle->device < dnnrt::MAX_DEVICES && dnnrt::g_scratch_holder[handle->device] == handle)
        dnnrt::g_scratch_holder[handle->device] = nullptr;
    } else {
      (void)dnnrt::counted_free(handle->splitk_partials);
      (void)dnnrt::counted_free(handle->splitk_counters);
    }
  }
  delete handle;
  return 0;
}

int32_t dnnrtDeviceMemoryStats(int64_t *allocated_now, int64_t *allocated_peak, int64_t *static_bytes, int32_t reset_peak) {
  std::lock_guard<std::mutex> lock(dnnrt::g_mem_mutex);
  if (allocated_now) *allocated_now = dnnrt::g_mem_now;
  if (allocated_peak) *allocated_peak = dnnrt::g_mem_peak;
  if (static_bytes) *static_bytes = dnnrt::HANDLE_SCRATCH_BYTES + dnnrt::NOALLOC_PARTIAL_BYTES + (int64_t)dnnrt::NOALLOC_MAX_TILES * (int64_t)sizeof(unsigned);
  if (reset_peak) dnnrt::g_mem_peak = dnnrt::g_mem_now;
  return 0;
}

int32_t dnnrtStreamCreate(dnnrtStream_t *stream) {
  hipStream_t s;
  HIP_RET(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "dnnrtStreamCreate");
  *stream = s;
  return 0;
}

int32_t dnnrtStreamDestroy(dnnrtStream_t stream) {
  HIP_RET(hipStreamDestroy((hipStream_t)stream), "dnnrtStreamDestroy");
  return 0;
}

int32_t dnnrtSetStream(dnnrtHandle_t handle, dnnrtStream_t stream) {
  if (!handle) { set_error("dnnrtSetStream: null handle"); return 1; }
  handle->stream = (hipStream_t)stream;
  return 0;
}

int32_t dnnrtSetTensorFormat(dnnrtHandle_t handle, int32_t format) {
  if (!handle) { set_error("dnnrtSetTensorFormat: null handle"); return 1; }
  if (format != DNNRT_NCHW && format != DNNRT_NHWC && format != DNNRT_NCHW_TO_NHWC) {
    set_error("dnnrtSetTensorFormat: unknown format %d", format);
    return 1;
  }
  handle->format = format;
  return 0;
}

int32_t dnnrtSetActivationCoef(dnnrtHandle_t handle, float coef) {
  if (!handle) { dnnrt::set_error("dnnrtSetActivationCoef: null handle"); return 1; }
  if (coef != coef) { dnnrt::set_error("dnnrtSetActivationCoef: NaN"); return 1; }
  handle->act_coef = coef;
  return 0;
}

int32_t dnnrtListConvTiles(int32_t *ids, int32_t capacity) {
  int n = 0;
  for (const int *t = dnnrt::F16_TILE_IDS; *t; t++, n++)
    if (ids && n < capacity) ids[n] = *t;
  return n;
}

int32_t dnnrtSetConvTile(dnnrtHandle_t handle, int32_t tile) {
  if (!handle) { set_error("dnnrtSetConvTile: null handle"); return 1; }
  bool known = tile == 0;
  for (const int *t = dnnrt::F16_TILE_IDS; *t; t++) known = known || *t == tile || *t == -tile;
  if (!known) { set_error("dnnrtSetConvTile: no fp16 convolution variant %d in this build", tile); return 1; }
  handle->f16_tile = tile;
  return 0;
}

int32_t dnnrtSetFilterLayout(dnnrtHandle_t handle, int32_t layout) {
  if (!handle) { set_error("dnnrtSetFilterLayout: null handle"); return 1; }
  if (layout != DNNRT_FILTER_KCRS && layout != DNNRT_FILTER_CRSK) {
    set_error("dnnrtSetFilterLayout: unknown layout %d", layout);
    return 1;
  }
  handle->filter_layout = layout;
  return 0;
}

int32_t dnnrtSync(dnnrtHandle_t handle) {
  if (!handle) { set_error("dnnrtSync: null handle"); return 1; }
  HIP_RET(hipStreamSynchronize(handle->stream), "dnnrtSync");
  return 0;
}

int32_t dnnrtGraphBegin(dnnrtHandle_t handle) {
  if (!handle || !handle->stream) { set_error("dnnrtGraphBegin: the handle needs a stream of its own"); return 1; }
  HIP_RET(hipStreamBeginCapture(handle->stream, hipStreamCaptureModeThreadLocal), "dnnrtGraphBegin");
  return 0;
}

int32_t dnnrtGraphEnd(dnnrtHandle_t handle, void **graph) {
  if (!handle || !graph) { set_error("dnnrtGraphEnd: bad arguments"); return 1; }
  hipGraph_t g = nullptr;
  HIP_RET(hipStreamEndCapture(handle->stream, &g), "dnnrtGraphEnd: hipStreamEndCapture");
  hipGraphExec_t exec = nullptr;
  hipError_t e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
  (void)hipGraphDestroy(g);
  if (e != hipSuccess) { set_error("dnnrtGraphEnd: hipGraphInstantiate: %s", hipGetErrorString(e)); return (int32_t)e; }
  *graph = exec;
  return 0;
}

int32_t dnnrtGraphLaunch(dnnrtHandle_t handle, void *graph) {
  if (!handle || !graph) { set_error("dnnrtGraphLaunch: bad arguments"); return 1; }
  HIP_RET(hipGraphLaunch((hipGraphExec_t)graph, handle->stream), "dnnrtGraphLaunch");
  return 0;
}

int32_t dnnrtGraphDestroy(void *graph) {
  if (graph) HIP_RET(hipGraphExecDestroy((hipGraphExec_t)graph), "dnnrtGraphDestroy");
  return 0;
}

int32_t dnnrtEventCreate(void **event) {
  if (!event) { set_error("dnnrtEventCreate: null pointer"); return 1; }
  hipEvent_t e;
  HIP_RET(hipEventCreate(&e), "dnnrtEventCreate");
  *event = e;
  return 0;
}

int32_t dnnrtEventRecord(void *event, dnnrtStream_t stream) {
  HIP_RET(hipEventRecord((hipEvent_t)event, (hipStream_t)stream), "dnnrtEventRecord");
  return 0;
}

int32_t dnnrtEventElapsedMs(void *start, void *stop, float *ms) {
  if (!ms) { set_error("dnnrtEventElapsedMs: null pointer"); return 1; }
  HIP_RET(hipEventSynchronize((hipEvent_t)stop), "dnnrtEventElapsedMs: hipEventSynchronize");
  HIP_RET(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop), "dnnrtEventElapsedMs");
  return 0;
}

int32_t dnnrtEventDestroy(void *event) {
  if (event) HIP_RET(hipEventDestroy((hipEvent_t)event), "dnnrtEventDestroy");
  return 0;
}

int32_t dnnrtMemPoolInit(void **pool, int64_t bytes) {
  if (!pool || bytes < 0) { set_error("dnnrtMemPoolInit: bad arguments"); return 1; }
  HIP_RET(dnnrt::counted_malloc(pool, bytes), "dnnrtMemPoolInit: hipMalloc");
  return 0;
}

int32_t dnnrtMemOffset(void **ptr, void *base, int64_t offset, int64_t bytes) {
  (void)bytes;
  if (!ptr || !base || offset < 0) { set_error("dnnrtMemOffset: bad arguments"); return 1; }
  *ptr = static_cast<char *>(base) + offset;
  return 0;
}

int32_t dnnrtMemFill(void *ptr, int32_t byte, int64_t bytes, dnnrtStream_t stream) {
  if (bytes <= 0) return 0;
  if (!ptr || byte < 0 || byte > 255) { set_error("dnnrtMemFill: bad arguments"); return 1; }
  const int64_t blocks = (bytes + 256 * 16 - 1) / (256 * 16);
  if (blocks > INT32_MAX) { set_error("dnnrtMemFill: too large"); return 1; }
  hipLaunchKernelGGL(dnnrt::fill_bytes_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     static_cast<unsigned char *>(ptr), (unsigned char)byte, bytes);
  HIP_RET(hipGetLastError(), "dnnrtMemFill");
  return 0;
}

int32_t dnnrtMemcpy(void *dst, void *src, int64_t bytes, int32_t kind, dnnrtStream_t stream) {
  hipMemcpyKind k;
  switch (kind) {
    case DNNRT_H2D: k = hipMemcpyHostToDevice; break;
    case DNNRT_D2H: k = hipMemcpyDeviceToHost; break;
    case DNNRT_D2D: k = hipMemcpyDeviceToDevice; break;
    default: set_error("dnnrtMemcpy: kind %d", kind); return 1;
  }
  if (bytes <= 0) return 0;
  HIP_RET(hipMemcpyAsync(dst, src, (size_t)bytes, k, (hipStream_t)stream), "dnnrtMemcpy");
  return 0;
}

int32_t dnnrtMalloc(void **ptr, int64_t bytes) {
  if (!ptr || bytes < 0) { set_error("dnnrtMalloc: bad arguments"); return 1; }
  HIP_RET(dnnrt::counted_malloc(ptr, bytes), "dnnrtMalloc: hipMalloc");
  return 0;
}

int32_t dnnrtDealloc(void *ptr) {
  HIP_RET(dnnrt::counted_free(ptr), "dnnrtDealloc");
  return 0;
}

int32_t dnnrtHostAlloc(void **ptr, int64_t bytes) {
  if (!ptr || bytes < 0) { set_error("dnnrtHostAlloc: bad arguments"); return 1; }
  HIP_RET(hipHostMalloc(ptr, (size_t)(bytes > 0 ? bytes : 1), hipHostMallocDefault), "dnnrtHostAlloc");
  return 0;
}

int32_t dnnrtHostFree(void *ptr) {
  HIP_RET(hipHostFree(ptr), "dnnrtHostFree");
  return 0;
}

}  // extern "C"

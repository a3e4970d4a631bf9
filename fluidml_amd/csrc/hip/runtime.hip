// Device plumbing behind the C ABI: arena, constants, copies, streams, events
// and launch-plan capture.  It replaces what the reference gets from
// mlir::ExecutionEngine and a per-call host vector (src/worker/runner.cpp:56-120,
// src/structure/context/context.cpp:152-166).
#include <mutex>
#include <unordered_map>

#include <algorithm>
#include <vector>

#include "fl_common.h"

using namespace fl;

namespace {

// hipMemsetAsync nodes inside captured graphs have replayed wrongly on some
// ROCm stacks; zeroing is therefore a plain fill kernel, safe to capture.
__global__ __launch_bounds__(256) void FillZero(uint32_t *p, size_t n_words, uint8_t *tail, size_t n_tail) {
  const size_t stride = static_cast<size_t>(gridDim.x) * 256;
  for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < n_words; i += stride) p[i] = 0u;
  if (blockIdx.x == 0 && threadIdx.x < n_tail) tail[threadIdx.x] = 0;
}

}  // namespace

namespace fl {
namespace {
std::mutex g_workspace_mutex;
std::unordered_map<hipStream_t, StreamWorkspace> g_workspaces;
}  // namespace

StreamWorkspace *GetStreamWorkspace(hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_workspace_mutex);
  auto it = g_workspaces.find(stream);
  if (it != g_workspaces.end()) return &it->second;
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
    (void)hipGetLastError();
    return nullptr;
  }
  if (status != hipStreamCaptureStatusNone) return nullptr;  // no allocation while a graph is recorded
  StreamWorkspace ws;
  if (hipMalloc(reinterpret_cast<void **>(&ws.partials), kWorkspaceTiles * kWorkspaceTileFloats * sizeof(float)) != hipSuccess ||
      hipMalloc(reinterpret_cast<void **>(&ws.counters), kWorkspaceTiles * sizeof(uint32_t)) != hipSuccess ||
      hipMemset(ws.counters, 0, kWorkspaceTiles * sizeof(uint32_t)) != hipSuccess) {
    (void)hipGetLastError();
    if (ws.partials) (void)hipFree(ws.partials);
    if (ws.counters) (void)hipFree(ws.counters);
    return nullptr;
  }
  return &g_workspaces.emplace(stream, ws).first->second;
}

void DropStreamWorkspace(hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_workspace_mutex);
  auto it = g_workspaces.find(stream);
  if (it == g_workspaces.end()) return;
  (void)hipFree(it->second.partials);
  (void)hipFree(it->second.counters);
  g_workspaces.erase(it);
}

KernelTimer &ThreadKernelTimer() {
  static thread_local KernelTimer timer;
  return timer;
}

// What the matrix pipes deliver when nothing else is asked of them: every wave issues `count` dependent
// v_mfma_f32_32x32x2_f32 (4096 flops each) and stamps the 100 MHz wall clock and the shader clock around them.
typedef float RateAcc __attribute__((ext_vector_type(16)));
__global__ __launch_bounds__(256) void MfmaRateKernel(int count, uint64_t *out) {
  RateAcc acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
  const float a = static_cast<float>(threadIdx.x) * 0.001f, b = 1.0f;
  const uint64_t w0 = wall_clock64(), c0 = clock64();
  for (int i = 0; i < count; ++i) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
  asm volatile("" ::"v"(acc[0]));
  const uint64_t w1 = wall_clock64(), c1 = clock64();
  if (threadIdx.x % 64 == 0) {
    const uint32_t w = blockIdx.x * 4 + threadIdx.x / 64;
    out[2 * w] = w1 - w0;
    out[2 * w + 1] = c1 - c0;
  }
}
}  // namespace fl

extern "C" {

int fluidml_hip_abi_version(void) { return 3; }

const char *fluidml_hip_error_string(int code) {
  switch (code) {
    case FL_OK: return "ok";
    case FL_ERR_NULL: return "null pointer argument";
    case FL_ERR_RANK: return "rank out of range or ranks inconsistent";
    case FL_ERR_SHAPE: return "shapes do not satisfy the kernel's contract";
    case FL_ERR_DTYPE: return "unsupported element type combination";
    case FL_ERR_ATTR: return "attribute out of range";
    case FL_ERR_TOO_LARGE: return "view larger than 2^31-1 elements";
    case FL_ERR_SCRATCH: return "scratch buffer too small";
    case FL_ERR_UNSUPPORTED: return "not supported by this backend";
    case FL_ERR_STATIC_SCRATCH:
      return "split-K workspace of this problem exceeds the fixed scratch of fluidml_hip_matmul_no_alloc "
             "(FL_NO_ALLOC_SCRATCH_BYTES); use fluidml_hip_matmul";
    default: break;
  }
  if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
  return "unknown error";
}

int fluidml_hip_device_count(void) {
  int n = 0;
  hipError_t err = hipGetDeviceCount(&n);
  if (err != hipSuccess) return -static_cast<int>(err) - 1000;
  return n;
}

int fluidml_hip_device_info(int dev, char *name, size_t name_len, char *arch, size_t arch_len, int *compute_units,
                            size_t *total_mem) {
  hipDeviceProp_t prop;
  FL_HIP_CHECK(hipGetDeviceProperties(&prop, dev));
  if (name && name_len) {
    std::strncpy(name, prop.name, name_len - 1);
    name[name_len - 1] = '\0';
  }
  if (arch && arch_len) {
    std::strncpy(arch, prop.gcnArchName, arch_len - 1);
    arch[arch_len - 1] = '\0';
  }
  if (compute_units) *compute_units = prop.multiProcessorCount;
  if (total_mem) *total_mem = prop.totalGlobalMem;
  return FL_OK;
}

int fluidml_hip_arena_create(size_t bytes, void **arena) {
  if (arena == nullptr) return FL_ERR_NULL;
  *arena = nullptr;
  // keep a valid pointer for an empty plan; round up so 128-bit accesses near
  // the end of the last tensor stay inside the allocation
  const size_t alloc = ((bytes + 255) / 256 + 1) * 256;
  void *p = nullptr;
  FL_HIP_CHECK(hipMalloc(&p, alloc));
  hipError_t err = hipMemset(p, 0, alloc);
  if (err != hipSuccess) {
    (void)hipFree(p);
    return static_cast<int>(err);
  }
  *arena = p;
  return FL_OK;
}

int fluidml_hip_arena_destroy(void *arena) {
  if (arena == nullptr) return FL_OK;
  FL_HIP_CHECK(hipFree(arena));
  return FL_OK;
}

int fluidml_hip_arena_zero(void *arena, size_t bytes, void *stream) {
  if (arena == nullptr) return FL_ERR_NULL;
  if (bytes == 0) return FL_OK;
  const size_t n_words = bytes / 4, n_tail = bytes % 4;
  const size_t blocks = std::min<size_t>((n_words + 255) / 256 + 1, 4096);
  FL_LAUNCH(FillZero, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, AsStream(stream),
                     static_cast<uint32_t *>(arena), n_words, static_cast<uint8_t *>(arena) + n_words * 4, n_tail);
  return LaunchStatus();
}

int fluidml_hip_upload_constant(const void *host, size_t bytes, void **device) {
  if (device == nullptr || (host == nullptr && bytes > 0)) return FL_ERR_NULL;
  *device = nullptr;
  const size_t alloc = ((bytes + 255) / 256 + 1) * 256;
  void *p = nullptr;
  FL_HIP_CHECK(hipMalloc(&p, alloc));
  if (bytes > 0) {
    hipError_t err = hipMemcpy(p, host, bytes, hipMemcpyHostToDevice);
    if (err != hipSuccess) {
      (void)hipFree(p);
      return static_cast<int>(err);
    }
  }
  *device = p;
  return FL_OK;
}

int fluidml_hip_free(void *device) {
  if (device == nullptr) return FL_OK;
  FL_HIP_CHECK(hipFree(device));
  return FL_OK;
}

int fluidml_hip_memcpy_h2d(void *device, const void *host, size_t bytes, void *stream) {
  if (bytes == 0) return FL_OK;
  if (device == nullptr || host == nullptr) return FL_ERR_NULL;
  FL_HIP_CHECK(hipMemcpyAsync(device, host, bytes, hipMemcpyHostToDevice, AsStream(stream)));
  return FL_OK;
}

int fluidml_hip_memcpy_d2h(void *host, const void *device, size_t bytes, void *stream) {
  if (bytes == 0) return FL_OK;
  if (device == nullptr || host == nullptr) return FL_ERR_NULL;
  FL_HIP_CHECK(hipMemcpyAsync(host, device, bytes, hipMemcpyDeviceToHost, AsStream(stream)));
  return FL_OK;
}

int fluidml_hip_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream) {
  if (bytes == 0) return FL_OK;
  if (dst == nullptr || src == nullptr) return FL_ERR_NULL;
  FL_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, AsStream(stream)));
  return FL_OK;
}

int fluidml_hip_stream_create(void **stream) {
  if (stream == nullptr) return FL_ERR_NULL;
  hipStream_t s = nullptr;
  FL_HIP_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *stream = s;
  (void)GetStreamWorkspace(s);  // now, so that a later capture on this stream finds it
  (void)StaticScratch(nullptr);  // likewise the address of this device's fixed scratch
  return FL_OK;
}

int fluidml_hip_stream_destroy(void *stream) {
  if (stream == nullptr) return FL_OK;
  FL_HIP_CHECK(hipStreamSynchronize(AsStream(stream)));
  DropStreamWorkspace(AsStream(stream));
  FL_HIP_CHECK(hipStreamDestroy(AsStream(stream)));
  return FL_OK;
}

int fluidml_hip_stream_synchronize(void *stream) {
  FL_HIP_CHECK(hipStreamSynchronize(AsStream(stream)));
  return FL_OK;
}

int fluidml_hip_event_create(void **event) {
  if (event == nullptr) return FL_ERR_NULL;
  hipEvent_t e = nullptr;
  FL_HIP_CHECK(hipEventCreate(&e));
  *event = e;
  return FL_OK;
}

int fluidml_hip_event_destroy(void *event) {
  if (event == nullptr) return FL_OK;
  FL_HIP_CHECK(hipEventDestroy(static_cast<hipEvent_t>(event)));
  return FL_OK;
}

int fluidml_hip_event_record(void *event, void *stream) {
  if (event == nullptr) return FL_ERR_NULL;
  FL_HIP_CHECK(hipEventRecord(static_cast<hipEvent_t>(event), AsStream(stream)));
  return FL_OK;
}

int fluidml_hip_stream_wait_event(void *stream, void *event) {
  if (event == nullptr) return FL_ERR_NULL;
  FL_HIP_CHECK(hipStreamWaitEvent(AsStream(stream), static_cast<hipEvent_t>(event), 0));
  return FL_OK;
}

int fluidml_hip_event_elapsed_ns(void *start, void *stop, double *ns) {
  if (start == nullptr || stop == nullptr || ns == nullptr) return FL_ERR_NULL;
  FL_HIP_CHECK(hipEventSynchronize(static_cast<hipEvent_t>(stop)));
  float ms = 0.0f;
  FL_HIP_CHECK(hipEventElapsedTime(&ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
  *ns = static_cast<double>(ms) * 1.0e6;
  return FL_OK;
}

int fluidml_hip_time_kernels(void *start, void *stop) {
  if ((start == nullptr) != (stop == nullptr)) return FL_ERR_NULL;
  fl::KernelTimer &t = fl::ThreadKernelTimer();
  t.start = static_cast<hipEvent_t>(start);
  t.stop = static_cast<hipEvent_t>(stop);
  return FL_OK;
}

int fluidml_hip_mfma_rate(int32_t waves_per_simd, int32_t count, double *ns, double *shader_ticks) {
  if (ns == nullptr || shader_ticks == nullptr) return FL_ERR_NULL;
  if (waves_per_simd < 1 || waves_per_simd > 2 || count < 1 || count > (1 << 20)) return FL_ERR_ATTR;
  int dev = 0;
  FL_HIP_CHECK(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  FL_HIP_CHECK(hipGetDeviceProperties(&prop, dev));
  const int groups = prop.multiProcessorCount * waves_per_simd;  // four waves each: one per SIMD of a compute unit
  uint64_t *out = nullptr;
  FL_HIP_CHECK(hipMalloc(&out, static_cast<size_t>(groups) * 4 * 2 * sizeof(uint64_t)));
  std::vector<uint64_t> host(static_cast<size_t>(groups) * 8);
  hipError_t err = hipSuccess;
  for (int round = 0; round < 3 && err == hipSuccess; ++round) {  // (the last of three: clocks and caches settled)
    hipLaunchKernelGGL(fl::MfmaRateKernel, dim3(groups), dim3(256), 0, nullptr, count, out);
    err = hipDeviceSynchronize();
  }
  if (err == hipSuccess) err = hipMemcpy(host.data(), out, host.size() * sizeof(uint64_t), hipMemcpyDeviceToHost);
  (void)hipFree(out);
  if (err != hipSuccess) return static_cast<int>(err);
  std::vector<uint64_t> wall, ticks;
  for (size_t w = 0; w < host.size() / 2; ++w) {
    wall.push_back(host[2 * w]);
    ticks.push_back(host[2 * w + 1]);
  }
  std::nth_element(wall.begin(), wall.begin() + wall.size() / 2, wall.end());
  std::nth_element(ticks.begin(), ticks.begin() + ticks.size() / 2, ticks.end());
  *ns = static_cast<double>(wall[wall.size() / 2]) * 10.0;
  *shader_ticks = static_cast<double>(ticks[ticks.size() / 2]);
  return FL_OK;
}

int fluidml_hip_graph_begin_capture(void *stream) {
  if (stream == nullptr) return FL_ERR_NULL;  // the null stream cannot be captured
  FL_HIP_CHECK(hipStreamBeginCapture(AsStream(stream), hipStreamCaptureModeThreadLocal));
  return FL_OK;
}

int fluidml_hip_graph_end_capture(void *stream, void **graph_exec) {
  if (stream == nullptr || graph_exec == nullptr) return FL_ERR_NULL;
  *graph_exec = nullptr;
  hipGraph_t graph = nullptr;
  FL_HIP_CHECK(hipStreamEndCapture(AsStream(stream), &graph));
  hipGraphExec_t exec = nullptr;
  hipError_t err = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (err != hipSuccess) return static_cast<int>(err);
  *graph_exec = exec;
  return FL_OK;
}

int fluidml_hip_graph_launch(void *graph_exec, void *stream) {
  if (graph_exec == nullptr) return FL_ERR_NULL;
  FL_HIP_CHECK(hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec), AsStream(stream)));
  return FL_OK;
}

int fluidml_hip_graph_destroy(void *graph_exec) {
  if (graph_exec == nullptr) return FL_OK;
  FL_HIP_CHECK(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec)));
  return FL_OK;
}

}  // extern "C"

// C-ABI runtime shim: device, memory, streams, events, graph replay.  Mirrors what the reference's HIP device does through
// libamdhip64 (tinygrad/runtime/ops_hip.py:12-70): every HIP status != 0 becomes an error string the Python wrapper raises
// as RuntimeError("HIP Error n, <string>") (ops_hip.py:9-10).
#include "host.h"
#include <string.h>
#include <vector>

static thread_local char g_err[512] = "";

int tga_set_error(const char* fmt, ...) {
  va_list ap; va_start(ap, fmt); vsnprintf(g_err, sizeof(g_err), fmt, ap); va_end(ap);
  return 1;
}

extern "C" {

const char* tga_last_error(void) { return g_err; }

int tga_init(int device) {
  int n = 0;
  TGA_HIP(hipGetDeviceCount(&n));
  TGA_REQUIRE(device >= 0 && device < n, "tga_init: device %d out of range (have %d)", device, n);
  TGA_HIP(hipSetDevice(device));
  hipDeviceProp_t p;
  TGA_HIP(hipGetDeviceProperties(&p, device));
  TGA_REQUIRE(strncmp(p.gcnArchName, "gfx950", 6) == 0, "tga_init: kernels are built for gfx950 only, device is %s", p.gcnArchName);
  if (const int rc = tga_route_scratch_setup(device)) return rc;   // device address of the static workspace of tga_moe_route_static on this GPU
  return tga_qgemm64_setup(device);                          // workspace of the 17 .. 128 row GEMM (staged activations, split-K partial tiles)
}

int tga_device_name(char* buf, size_t len) {
  int dev = 0; hipDeviceProp_t p;
  TGA_HIP(hipGetDevice(&dev));
  TGA_HIP(hipGetDeviceProperties(&p, dev));
  // (the marketing name is empty on some driver / container combinations: the architecture string then stands for it)
  snprintf(buf, len, "%s (%s, %d CUs, %.0f MHz)", p.name[0] ? p.name : "AMD GPU", p.gcnArchName, p.multiProcessorCount, p.clockRate / 1000.0);
  return 0;
}

int tga_malloc(void** ptr, size_t nbytes) { TGA_REQUIRE(ptr, "tga_malloc: null out pointer"); TGA_HIP(hipMalloc(ptr, nbytes ? nbytes : 1)); return 0; }
int tga_free(void* ptr) { TGA_HIP(hipFree(ptr)); return 0; }
int tga_memcpy_h2d(void* dst, const void* src, size_t n) { TGA_HIP(hipMemcpy(dst, src, n, hipMemcpyHostToDevice)); return 0; }
int tga_memcpy_d2h(void* dst, const void* src, size_t n) { TGA_HIP(hipMemcpy(dst, src, n, hipMemcpyDeviceToHost)); return 0; }
int tga_memcpy_d2d(void* dst, const void* src, size_t n, void* stream) {
  TGA_HIP(hipMemcpyAsync(dst, src, n, hipMemcpyDeviceToDevice, (hipStream_t)stream)); return 0;
}
// Plain 16-byte-per-thread copy kernel of a known size: the yardstick the HBM traffic counters (FETCH_SIZE / WRITE_SIZE) of other
// kernels are scaled by.
__global__ __launch_bounds__(256) void copy_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, size_t n16) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256) dst[i] = src[i];
}
int tga_copy_kernel(void* dst, const void* src, size_t n, void* stream) {
  TGA_REQUIRE(dst && src && n % 16 == 0 && (((uintptr_t)dst | (uintptr_t)src) & 15) == 0, "tga_copy_kernel: pointers and size must be multiples of 16");
  if (n == 0) return 0;
  copy_kernel<<<2048, 256, 0, (hipStream_t)stream>>>((uint4*)dst, (const uint4*)src, n / 16);
  TGA_LAUNCH_CHECK();
  return 0;
}
// (refused while the stream is capturing: a memset node in a replayed graph has given wrong results on this platform; captured code clears with a fill kernel)
int tga_memset(void* dst, int value, size_t n, void* stream) {
  if (stream) {
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    TGA_HIP(hipStreamIsCapturing((hipStream_t)stream, &cs));
    TGA_REQUIRE(cs == hipStreamCaptureStatusNone, "tga_memset: the stream is capturing; use a fill kernel inside a capture");
  }
  TGA_HIP(hipMemsetAsync(dst, value, n, (hipStream_t)stream)); return 0;
}
int tga_sync(void) { TGA_HIP(hipDeviceSynchronize()); return 0; }

int tga_stream_create(void** stream) { TGA_HIP(hipStreamCreate((hipStream_t*)stream)); return 0; }   // default priority only
int tga_stream_destroy(void* stream) {
  // waits for the stream's work first: the workspace slot of the 17 .. 128 row GEMM that the stream holds may then pass to another stream at once
  TGA_HIP(hipStreamSynchronize((hipStream_t)stream));
  tga_qgemm64_release((hipStream_t)stream);
  TGA_HIP(hipStreamDestroy((hipStream_t)stream));
  return 0;
}
int tga_stream_sync(void* stream) { TGA_HIP(hipStreamSynchronize((hipStream_t)stream)); return 0; }

int tga_event_create(void** ev) { TGA_HIP(hipEventCreate((hipEvent_t*)ev)); return 0; }
int tga_event_destroy(void* ev) { TGA_HIP(hipEventDestroy((hipEvent_t)ev)); return 0; }
int tga_event_record(void* ev, void* stream) { TGA_HIP(hipEventRecord((hipEvent_t)ev, (hipStream_t)stream)); return 0; }
int tga_event_sync(void* ev) { TGA_HIP(hipEventSynchronize((hipEvent_t)ev)); return 0; }
int tga_event_elapsed_ms(void* start, void* stop, float* ms) { TGA_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop)); return 0; }

// HIPProgram.__call__ (tinygrad/runtime/ops_hip.py:36-57): launch a kernel of this library by its host-side handle with an array of
// pointers to the argument values (hipLaunchKernel's convention), grid counted in workgroups, no dynamic LDS.
int tga_launch_kernel(const void* host_function, const uint32_t* grid, const uint32_t* block, void** args, void* stream) {
  TGA_REQUIRE(host_function && grid && block && args, "tga_launch_kernel: null pointer");
  TGA_REQUIRE(grid[0] && grid[1] && grid[2] && block[0] && block[1] && block[2] && (uint64_t)block[0] * block[1] * block[2] <= 1024, "tga_launch_kernel: empty grid or block, or more than 1024 threads");
  TGA_HIP(hipLaunchKernel(host_function, dim3(grid[0], grid[1], grid[2]), dim3(block[0], block[1], block[2]), args, 0, (hipStream_t)stream));
  return 0;
}

// A captured launch sequence replayed as plain launches.  hipGraphLaunch costs 0.3-0.5 us more per kernel node than the same kernels enqueued
// one after the other on a stream (measured on a chain of dependent kernels of 2..32 MB each), and a decode step is about 200 small kernels.
// The sequence is still captured with the stream-capture API (so every entry point records itself without knowing about it); the kernel nodes of
// the captured graph - function, grid, block, dynamic LDS and the argument values, which the graph keeps alive - are then launched in capture
// order with hipLaunchKernel.  Only kernel nodes are accepted: anything else in the capture (memset, copy, host node) is refused.
struct TgaCmdList { hipGraph_t graph; std::vector<hipKernelNodeParams> kernels; };

int tga_cmdlist_end(void* stream, void** cmdlist) {
  TGA_REQUIRE(stream && cmdlist, "tga_cmdlist_end: null pointer");
  hipGraph_t g = nullptr;
  TGA_HIP(hipStreamEndCapture((hipStream_t)stream, &g));
  size_t n = 0;
  hipError_t e = hipGraphGetNodes(g, nullptr, &n);
  std::vector<hipGraphNode_t> nodes(n);
  if (e == hipSuccess && n) e = hipGraphGetNodes(g, nodes.data(), &n);
  if (e != hipSuccess) { (void)hipGraphDestroy(g); TGA_HIP(e); }
  // capture order = dependency order for a single-stream capture: every node depends on the one before it; verified below
  TgaCmdList* cl = new TgaCmdList{g, {}};
  for (size_t i = 0; i < n; i++) {
    hipGraphNodeType t;
    e = hipGraphNodeGetType(nodes[i], &t);
    if (e == hipSuccess && t != hipGraphNodeTypeKernel) { (void)hipGraphDestroy(g); delete cl; return tga_set_error("tga_cmdlist_end: node %zu of the capture is not a kernel launch (type %d)", i, (int)t); }
    size_t ndep = 0;
    if (e == hipSuccess) e = hipGraphNodeGetDependencies(nodes[i], nullptr, &ndep);
    if (e == hipSuccess && ndep > 1) { (void)hipGraphDestroy(g); delete cl; return tga_set_error("tga_cmdlist_end: node %zu has %zu dependencies (a linear single-stream capture is required)", i, ndep); }
    if (e == hipSuccess && ndep == 1) {
      hipGraphNode_t dep; size_t one = 1;
      e = hipGraphNodeGetDependencies(nodes[i], &dep, &one);
      if (e == hipSuccess && (i == 0 || dep != nodes[i - 1])) { (void)hipGraphDestroy(g); delete cl; return tga_set_error("tga_cmdlist_end: node %zu does not follow node %zu (nodes are not in capture order)", i, i - 1); }
    }
    hipKernelNodeParams p;
    if (e == hipSuccess) e = hipGraphKernelNodeGetParams(nodes[i], &p);
    if (e != hipSuccess) { (void)hipGraphDestroy(g); delete cl; TGA_HIP(e); }
    cl->kernels.push_back(p);
  }
  *cmdlist = cl;
  return 0;
}
int tga_cmdlist_launch(void* cmdlist, void* stream) {
  TGA_REQUIRE(cmdlist, "tga_cmdlist_launch: null list");
  const TgaCmdList* cl = (const TgaCmdList*)cmdlist;
  for (const hipKernelNodeParams& p : cl->kernels) {
    if (p.kernelParams) TGA_HIP(hipLaunchKernel(p.func, p.gridDim, p.blockDim, p.kernelParams, p.sharedMemBytes, (hipStream_t)stream));
    else return tga_set_error("tga_cmdlist_launch: a kernel node without an argument list");
  }
  return 0;
}
int tga_cmdlist_size(void* cmdlist) { return cmdlist ? (int)((const TgaCmdList*)cmdlist)->kernels.size() : 0; }
int tga_cmdlist_destroy(void* cmdlist) {
  if (!cmdlist) return 0;
  TgaCmdList* cl = (TgaCmdList*)cmdlist;
  (void)hipGraphDestroy(cl->graph);
  delete cl;
  return 0;
}

int tga_graph_begin(void* stream) {
  TGA_REQUIRE(stream, "tga_graph_begin: capture needs a non-null stream");
  TGA_HIP(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
  return 0;
}
int tga_graph_end(void* stream, void** graph_exec) {
  hipGraph_t g = nullptr;
  TGA_HIP(hipStreamEndCapture((hipStream_t)stream, &g));
  hipGraphExec_t ge = nullptr;
  hipError_t e = hipGraphInstantiate(&ge, g, nullptr, nullptr, 0);
  (void)hipGraphDestroy(g);
  TGA_HIP(e);
  *graph_exec = ge;
  return 0;
}
int tga_graph_launch(void* graph_exec, void* stream) { TGA_HIP(hipGraphLaunch((hipGraphExec_t)graph_exec, (hipStream_t)stream)); return 0; }
int tga_graph_destroy(void* graph_exec) { TGA_HIP(hipGraphExecDestroy((hipGraphExec_t)graph_exec)); return 0; }

}  // extern "C"

/* Device, stream, event and memory glue plus error reporting.
 * Counterpart of src/core/gpu/device_gpu.c:155-420, storage_gpu.c:61-302,
 * cuda.c:67-120 and solid/src/base/gpu/solid_gpu.c:28-236 in the reference,
 * written against the HIP runtime: one hipStream_t per stream handle,
 * stream-ordered allocation from the device's default memory pool. */
#include "och_common.h"
#include <string.h>
#include <atomic>
#include <map>
#include <mutex>
#include <utility>

namespace och {
static thread_local char g_errmsg[512] = "";
int set_error(const char *fmt, ...)
{
   va_list ap; va_start(ap, fmt); vsnprintf(g_errmsg, sizeof(g_errmsg), fmt, ap); va_end(ap);
   return -1;
}
void clear_error() { g_errmsg[0] = 0; }
static std::atomic<int> g_status(0);              /* hipSuccess, or the first error since the last check */
void note_status(int hip_error)
{  int none = 0;
   if (hip_error != 0) g_status.compare_exchange_strong(none, hip_error);
}
__global__ void warmup_kernel(int *p) { if (p) *p = 1; }
}

namespace och {
static std::map<std::pair<int, hipStream_t>, StreamContext> g_stream_ctx;
static std::mutex g_stream_ctx_mutex;

int stream_context(hipStream_t stream, StreamContext **out)
{
   int dev;
   OCH_CHECK_HIP(hipGetDevice(&dev));
   std::lock_guard<std::mutex> lock(g_stream_ctx_mutex);
   auto key = std::make_pair(dev, stream);
   auto it = g_stream_ctx.find(key);
   if (it == g_stream_ctx.end())
   {  StreamContext c = { nullptr, nullptr, nullptr };
      void *scratch = nullptr, *host = nullptr;
      /* the scratch cannot be created while the stream records a graph: allocation is not a graph node, and the
         zeroing below would become one and run again at every replay, in the middle of the recorded reductions */
      hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
      if (stream != nullptr) OCH_CHECK_HIP(hipStreamIsCapturing(stream, &capturing));
      if (capturing != hipStreamCaptureStatusNone)
         return set_error("a stream must be used once, or recording must start with och_stream_begin_capture, before library calls are recorded on it");
      OCH_CHECK_HIP(hipMalloc(&scratch, OCH_RED_SCRATCH));
      /* zeroed by a kernel on the owning stream itself: ordered before the stream's first reduction by the stream,
         whatever its blocking mode with respect to the null stream */
      hipError_t e = (fill_bytes(scratch, 0, OCH_RED_SCRATCH, stream) == 0) ? hipSuccess : hipErrorLaunchFailure;
      if (e == hipSuccess) e = hipHostMalloc(&host, 64, hipHostMallocDefault);
      if (e != hipSuccess) { (void)hipFree(scratch); return set_error("stream scratch: %s", hipGetErrorString(e)); }
      c.red_scratch = (char *)scratch; c.host_result = host;
      it = g_stream_ctx.insert(std::make_pair(key, c)).first;
   }
   *out = &it->second;                 /* std::map nodes stay where they are when other streams are added */
   return 0;
}
int stream_gemm_workspace(hipStream_t stream, char **workspace)
{
   StreamContext *c;
   if (stream_context(stream, &c) != 0) return -1;
   std::lock_guard<std::mutex> lock(g_stream_ctx_mutex);
   if (c->gemm_workspace == nullptr)
   {  /* from the stream-ordered pool: no device-wide synchronisation, and what och_stream_release_workspace gives back
         serves the next stream that needs one */
      void *w = nullptr;
      OCH_CHECK_HIP(hipMallocAsync(&w, OCH_GEMM_WORKSPACE, stream));
      c->gemm_workspace = (char *)w;
   }
   *workspace = c->gemm_workspace;
   return 0;
}
/* gives the stream's workspace back to the pool, behind the work already queued on the stream */
int stream_release_workspace(hipStream_t stream)
{
   int dev;
   OCH_CHECK_HIP(hipGetDevice(&dev));
   std::lock_guard<std::mutex> lock(g_stream_ctx_mutex);
   auto it = g_stream_ctx.find(std::make_pair(dev, stream));
   if (it == g_stream_ctx.end() || it->second.gemm_workspace == nullptr) return 0;
   char *w = it->second.gemm_workspace;
   it->second.gemm_workspace = nullptr;
   OCH_CHECK_HIP(hipFreeAsync(w, stream));
   return 0;
}
void stream_context_release(hipStream_t stream)
{
   int dev;
   if (hipGetDevice(&dev) != hipSuccess) return;
   std::lock_guard<std::mutex> lock(g_stream_ctx_mutex);
   auto it = g_stream_ctx.find(std::make_pair(dev, stream));
   if (it == g_stream_ctx.end()) return;
   (void)hipFree(it->second.red_scratch); (void)hipHostFree(it->second.host_result);
   if (it->second.gemm_workspace) (void)hipFreeAsync(it->second.gemm_workspace, stream);
   g_stream_ctx.erase(it);
}

typedef unsigned int fill_u32x4 __attribute__((ext_vector_type(4)));
/* 16-byte stores over the aligned body (grid-stride), single bytes for the unaligned head and tail (first block) */
__global__ __launch_bounds__(256) void fill_bytes_kernel(unsigned char *dst, unsigned int pattern, size_t head, size_t body, size_t tail)
{
   const fill_u32x4 v = { pattern, pattern, pattern, pattern };
   fill_u32x4 *b = reinterpret_cast<fill_u32x4 *>(dst + head);
   for (size_t g = (size_t)blockIdx.x * 256 + threadIdx.x; g < body; g += (size_t)gridDim.x * 256) b[g] = v;
   if (blockIdx.x == 0)
   {  if (threadIdx.x < head) dst[threadIdx.x] = (unsigned char)pattern;
      if (threadIdx.x < tail) dst[head + body * 16 + threadIdx.x] = (unsigned char)pattern;
   }
}
int fill_bytes(void *dst, int value, size_t nbytes, hipStream_t stream)
{
   if (nbytes == 0) return 0;
   if (dst == nullptr) return set_error("memset: null pointer");
   size_t head = (16 - ((uintptr_t)dst & 15)) & 15; if (head > nbytes) head = nbytes;
   const size_t body = (nbytes - head) / 16, tail = nbytes - head - body * 16;
   const unsigned int byte = (unsigned int)value & 0xFFu, pattern = byte * 0x01010101u;
   size_t blocks = (body + 255) / 256; if (blocks < 1) blocks = 1; if (blocks > 65536) blocks = 65536;
   hipLaunchKernelGGL(fill_bytes_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (unsigned char *)dst, pattern, head, body, tail);
   OCH_CHECK_LAUNCH();
   return 0;
}
}

extern "C" {

const int och_type_size[OCH_DTYPE_COUNT] = { 1, 1, 2, 4, 8, 1, 2, 4, 8, 2, 4, 8, 4, 8, 16 };

const char *och_last_error(void) { return och::g_errmsg; }

int och_status_check(void)
{  int e = och::g_status.exchange(0);
   if (e == 0) return 0;
   (void)hipGetLastError();
   return och::set_error("HIP error: %s", hipGetErrorString((hipError_t)e));
}
void och_status_clear(void) { och::g_status.store(0); }

int och_device_count(int *count)
{
   hipError_t e = hipGetDeviceCount(count);
   if (e == hipErrorNoDevice) { *count = 0; (void)hipGetLastError(); return 0; }
   OCH_CHECK_HIP(e);
   return 0;
}
int och_device_set(int device) { OCH_CHECK_HIP(hipSetDevice(device)); return 0; }
int och_device_get(int *device) { OCH_CHECK_HIP(hipGetDevice(device)); return 0; }

int och_device_properties(int device, och_device_prop *p)
{
   hipDeviceProp_t d;
   OCH_CHECK_HIP(hipGetDeviceProperties(&d, device));
   memset(p, 0, sizeof(*p));
   strncpy(p->name, d.name, sizeof(p->name) - 1);
   strncpy(p->arch, d.gcnArchName, sizeof(p->arch) - 1);
   p->total_global_mem = d.totalGlobalMem;
   p->shared_mem_per_block = d.sharedMemPerBlock;
   p->multiprocessor_count = d.multiProcessorCount;
   p->wavefront_size = d.warpSize;
   p->max_threads_per_block = d.maxThreadsPerBlock;
   p->max_threads_per_multiprocessor = d.maxThreadsPerMultiProcessor;
   p->clock_rate_khz = d.clockRate;
   p->memory_clock_rate_khz = d.memoryClockRate;
   p->memory_bus_width = d.memoryBusWidth;
   p->l2_cache_size = d.l2CacheSize;
   p->pci_bus_id = d.pciBusID; p->pci_device_id = d.pciDeviceID; p->pci_domain_id = d.pciDomainID;
   p->concurrent_kernels = d.concurrentKernels;
   p->ecc_enabled = d.ECCEnabled;
   p->total_const_mem = d.totalConstMem; p->mem_pitch = d.memPitch; p->regs_per_block = d.regsPerBlock;
   for (int i = 0; i < 3; i++) { p->max_threads_dim[i] = d.maxThreadsDim[i]; p->max_grid_size[i] = d.maxGridSize[i]; }
   p->major = d.major; p->minor = d.minor;
   p->async_engine_count = d.asyncEngineCount;
   p->kernel_exec_timeout_enabled = d.kernelExecTimeoutEnabled;
   p->integrated = d.integrated; p->can_map_host_memory = d.canMapHostMemory; p->compute_mode = d.computeMode;
   p->tcc_driver = 0;
   size_t total = 0;
   return och_device_mem_info(device, &p->free_global_mem, &total);
}

int och_device_mem_info(int device, size_t *free_bytes, size_t *total_bytes)
{
   int prev;
   if (!free_bytes || !total_bytes) return och::set_error("och_device_mem_info: null argument");
   OCH_CHECK_HIP(hipGetDevice(&prev));
   OCH_CHECK_HIP(hipSetDevice(device));
   const hipError_t e = hipMemGetInfo(free_bytes, total_bytes);
   OCH_CHECK_HIP(hipSetDevice(prev));
   OCH_CHECK_HIP(e);
   return 0;
}

int och_device_can_access_peer(int device, int peer, int *result)
{
   OCH_CHECK_HIP(hipDeviceCanAccessPeer(result, device, peer));
   return 0;
}

int och_device_warmup(int device)
{  /* pay the runtime's first-use cost (context, code object load) up front */
   int prev;
   OCH_CHECK_HIP(hipGetDevice(&prev));
   OCH_CHECK_HIP(hipSetDevice(device));
   hipLaunchKernelGGL(och::warmup_kernel, dim3(1), dim3(1), 0, 0, (int *)nullptr);
   OCH_CHECK_LAUNCH();
   OCH_CHECK_HIP(hipDeviceSynchronize());
   och::StreamContext *ctx;
   int status = och::stream_context(nullptr, &ctx);              /* scratch of the default stream */
   char *fixed;
   if (status == 0) status = och::reduce_static_scratch(&fixed); /* this device's address of the scratch that needs no allocation */
   OCH_CHECK_HIP(hipSetDevice(prev));
   return status;
}
int och_device_synchronize(void) { OCH_CHECK_HIP(hipDeviceSynchronize()); OCH_CHECK_AFTER_WAIT("the device"); return 0; }

int och_stream_create(och_stream *stream)
{
   hipStream_t s;
   OCH_CHECK_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
   *stream = (och_stream)s; return 0;
}
int och_stream_destroy(och_stream stream)
{  OCH_CHECK_HIP(hipStreamSynchronize((hipStream_t)stream));      /* its scratch may still be in use */
   och::stream_context_release((hipStream_t)stream);
   OCH_CHECK_HIP(hipStreamDestroy((hipStream_t)stream));
   return 0;
}
int och_stream_release_workspace(och_stream stream) { return och::stream_release_workspace((hipStream_t)stream); }
int och_stream_synchronize(och_stream stream) { OCH_CHECK_HIP(hipStreamSynchronize((hipStream_t)stream)); OCH_CHECK_AFTER_WAIT("a stream"); return 0; }
int och_stream_wait_event(och_stream stream, och_event event)
{  OCH_CHECK_HIP(hipStreamWaitEvent((hipStream_t)stream, (hipEvent_t)event, 0)); return 0; }

int och_event_create(och_event *event, int timing)
{
   hipEvent_t e;
   OCH_CHECK_HIP(hipEventCreateWithFlags(&e, timing ? hipEventDefault : hipEventDisableTiming));
   *event = (och_event)e; return 0;
}
int och_event_destroy(och_event event) { OCH_CHECK_HIP(hipEventDestroy((hipEvent_t)event)); return 0; }
int och_event_record(och_event event, och_stream stream)
{  OCH_CHECK_HIP(hipEventRecord((hipEvent_t)event, (hipStream_t)stream)); return 0; }
int och_event_synchronize(och_event event) { OCH_CHECK_HIP(hipEventSynchronize((hipEvent_t)event)); OCH_CHECK_AFTER_WAIT("an event"); return 0; }
int och_event_elapsed_ms(och_event start, och_event stop, float *ms)
{  OCH_CHECK_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop)); return 0; }

int och_stream_begin_capture(och_stream stream)
{  if (stream == nullptr) return och::set_error("the default stream cannot record a graph");
   char *workspace;                                    /* allocate the stream's scratch now: nothing may be allocated while it records */
   if (och::stream_gemm_workspace((hipStream_t)stream, &workspace) != 0) return -1;
   OCH_CHECK_HIP(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal));
   return 0;
}
/* A recorded graph keeps the stream it was recorded on: its reductions and split products address that stream's
   scratch (partial results, ticket counter, workspace), so a replay on another stream would share them with whatever
   runs on the recording stream at the same time. */
struct och_graph_record { hipGraphExec_t exec; hipStream_t stream; int device; };

int och_stream_end_capture(och_stream stream, och_graph *graph)
{  hipGraph_t g = nullptr; hipGraphExec_t exec = nullptr; int device = 0;
   if (graph == nullptr) return och::set_error("null graph pointer");
   *graph = nullptr;
   OCH_CHECK_HIP(hipStreamEndCapture((hipStream_t)stream, &g));
   if (g == nullptr) return och::set_error("the stream recorded no graph");
   hipError_t e = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
   (void)hipGraphDestroy(g);
   if (e != hipSuccess) return och::set_error("hipGraphInstantiate failed: %s", hipGetErrorString(e));
   if ((e = hipGetDevice(&device)) != hipSuccess) { (void)hipGraphExecDestroy(exec); return och::set_error("hipGetDevice failed: %s", hipGetErrorString(e)); }
   och_graph_record *r = new och_graph_record{ exec, (hipStream_t)stream, device };
   *graph = (och_graph)r;
   return 0;
}
int och_graph_launch(och_graph graph, och_stream stream)
{  if (graph == nullptr) return och::set_error("null graph");
   och_graph_record *r = (och_graph_record *)graph;
   if ((hipStream_t)stream != r->stream)
      return och::set_error("a graph replays on the stream that recorded it: its kernels use that stream's scratch memory");
   OCH_CHECK_HIP(hipGraphLaunch(r->exec, r->stream));
   return 0;
}
int och_graph_destroy(och_graph graph)
{  if (graph == nullptr) return 0;
   och_graph_record *r = (och_graph_record *)graph;
   hipError_t e = hipGraphExecDestroy(r->exec);
   delete r;
   OCH_CHECK_HIP(e);
   return 0;
}

int och_malloc_async(void **ptr, size_t nbytes, och_stream stream)
{
   *ptr = nullptr;
   if (nbytes == 0) return 0;
   OCH_CHECK_HIP(hipMallocAsync(ptr, nbytes, (hipStream_t)stream));
   return 0;
}
int och_free_async(void *ptr, och_stream stream)
{
   if (ptr == nullptr) return 0;
   OCH_CHECK_HIP(hipFreeAsync(ptr, (hipStream_t)stream));
   return 0;
}
int och_malloc_host(void **ptr, size_t nbytes) { OCH_CHECK_HIP(hipHostMalloc(ptr, nbytes ? nbytes : 1, hipHostMallocDefault)); return 0; }
int och_free_host(void *ptr) { if (ptr) OCH_CHECK_HIP(hipHostFree(ptr)); return 0; }

int och_memcpy_dtod_async(void *dst, const void *src, size_t nbytes, och_stream stream)
{  if (nbytes) OCH_CHECK_HIP(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToDevice, (hipStream_t)stream)); return 0; }
int och_memcpy_peer_async(void *dst, int dst_device, const void *src, int src_device, size_t nbytes, och_stream stream)
{  if (nbytes) OCH_CHECK_HIP(hipMemcpyPeerAsync(dst, dst_device, src, src_device, nbytes, (hipStream_t)stream)); return 0; }
int och_memcpy_htod_async(void *dst, const void *src, size_t nbytes, och_stream stream)
{  if (nbytes) OCH_CHECK_HIP(hipMemcpyAsync(dst, src, nbytes, hipMemcpyHostToDevice, (hipStream_t)stream)); return 0; }
int och_memcpy_dtoh_async(void *dst, const void *src, size_t nbytes, och_stream stream)
{  if (nbytes) OCH_CHECK_HIP(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToHost, (hipStream_t)stream)); return 0; }
int och_memcpy_htod(void *dst, const void *src, size_t nbytes, och_stream stream)
{
   if (nbytes == 0) return 0;
   OCH_CHECK_HIP(hipMemcpyAsync(dst, src, nbytes, hipMemcpyHostToDevice, (hipStream_t)stream));
   OCH_CHECK_HIP(hipStreamSynchronize((hipStream_t)stream));
   return 0;
}
int och_memcpy_dtoh(void *dst, const void *src, size_t nbytes, och_stream stream)
{
   if (nbytes == 0) return 0;
   OCH_CHECK_HIP(hipMemcpyAsync(dst, src, nbytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
   OCH_CHECK_HIP(hipStreamSynchronize((hipStream_t)stream));
   return 0;
}
int och_memset_async(void *dst, int value, size_t nbytes, och_stream stream)
{  return och::fill_bytes(dst, value, nbytes, (hipStream_t)stream); }

} /* extern "C" */

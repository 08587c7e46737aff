// nslm_rt.hip - the thin C-ABI layer over the HIP runtime (include/nslm_rt.h): what the reference's C99 host code calls
// the CUDA runtime for (engine/mova_cuda.c:183-222, 590, 892-896; tests/kernel_backend_cuda.c:17-41), one-to-one.
#include <hip/hip_runtime.h>
#include <string.h>

#include "nslm_rt.h"

namespace {
// nh_memset_async's fill: a kernel, so that the call can be captured into a graph (memset nodes gave wrong results on replays
// after the first on these GPUs).  Whole 16-byte pieces by 16-byte stores, the ragged ends by bytes.
__global__ void __launch_bounds__(256) k_fill_bytes(unsigned char* p, unsigned char v, size_t n) {
    const size_t i0 = (size_t) blockIdx.x * 256 + threadIdx.x, step = (size_t) gridDim.x * 256;
    const size_t head = (16 - ((uintptr_t) p & 15u)) & 15u, h = head < n ? head : n, mid = (n - h) / 16;
    const unsigned w = v * 0x01010101u;
    uint4* q = (uint4*) (p + h);
    for (size_t i = i0; i < mid; i += step) q[i] = make_uint4(w, w, w, w);
    for (size_t i = i0; i < h; i += step) p[i] = v;
    for (size_t i = h + mid * 16 + i0; i < n; i += step) p[i] = v;
}
}   // namespace

extern "C" {

int nh_device_count(int* n) { return (int) hipGetDeviceCount(n); }
int nh_set_device(int dev) { return (int) hipSetDevice(dev); }
int nh_malloc(void** p, size_t n) { return (int) hipMalloc(p, n ? n : 16); }
int nh_free(void* p) { return (int) hipFree(p); }
int nh_host_alloc(void** p, size_t n) { return (int) hipHostMalloc(p, n ? n : 16, hipHostMallocMapped); }
int nh_host_free(void* p) { return (int) hipHostFree(p); }
int nh_memcpy_h2d(void* dst, const void* src, size_t n) { return n ? (int) hipMemcpy(dst, src, n, hipMemcpyHostToDevice) : 0; }
int nh_memcpy_d2h(void* dst, const void* src, size_t n) { return n ? (int) hipMemcpy(dst, src, n, hipMemcpyDeviceToHost) : 0; }
int nh_memcpy_d2d(void* dst, const void* src, size_t n) { return n ? (int) hipMemcpy(dst, src, n, hipMemcpyDeviceToDevice) : 0; }
int nh_memcpy_h2d_async(void* dst, const void* src, size_t n, nh_stream_t s) {
    return n ? (int) hipMemcpyAsync(dst, src, n, hipMemcpyHostToDevice, (hipStream_t) s) : 0;
}
int nh_memcpy_d2h_async(void* dst, const void* src, size_t n, nh_stream_t s) {
    return n ? (int) hipMemcpyAsync(dst, src, n, hipMemcpyDeviceToHost, (hipStream_t) s) : 0;
}
int nh_memcpy_d2d_async(void* dst, const void* src, size_t n, nh_stream_t s) {
    return n ? (int) hipMemcpyAsync(dst, src, n, hipMemcpyDeviceToDevice, (hipStream_t) s) : 0;
}
int nh_memcpy_async(void* dst, const void* src, size_t n, nh_stream_t s) {
    return n ? (int) hipMemcpyAsync(dst, src, n, hipMemcpyDefault, (hipStream_t) s) : 0;
}
int nh_memset(void* p, int v, size_t n) { return n ? (int) hipMemset(p, v, n) : 0; }
int nh_memset_async(void* p, int v, size_t n, nh_stream_t s) {
    if (!n) return 0;
    size_t wg = (n / 16 + 255) / 256;
    if (wg < 1) wg = 1;
    if (wg > 4096) wg = 4096;
    hipLaunchKernelGGL(k_fill_bytes, dim3((unsigned) wg), dim3(256), 0, (hipStream_t) s, (unsigned char*) p, (unsigned char) v, n);
    return (int) hipGetLastError();
}
int nh_host_alloc_mapped(void** host, void** dev, size_t n) {
    const hipError_t e = hipHostMalloc(host, n ? n : 16, hipHostMallocMapped);
    if (e != hipSuccess) return (int) e;
    return dev ? (int) hipHostGetDevicePointer(dev, *host, 0) : 0;
}
int nh_host_device_ptr(void** dev, void* host) { return (int) hipHostGetDevicePointer(dev, host, 0); }
int nh_get_device(int* dev) { return (int) hipGetDevice(dev); }
int nh_stream_create(nh_stream_t* s) { return (int) hipStreamCreateWithFlags((hipStream_t*) s, hipStreamNonBlocking); }
int nh_stream_priority_range(int* least, int* greatest) {   // one priority: every stream of this library is a default-priority stream
    if (least) *least = 0;
    if (greatest) *greatest = 0;
    return 0;
}
int nh_stream_create_prio(nh_stream_t* s, int priority) {
    (void) priority;
    return nh_stream_create(s);
}
int nh_event_create_untimed(nh_event_t* e) { return (int) hipEventCreateWithFlags((hipEvent_t*) e, hipEventDisableTiming); }
int nh_stream_destroy(nh_stream_t s) { return (int) hipStreamDestroy((hipStream_t) s); }
int nh_stream_sync(nh_stream_t s) { return (int) hipStreamSynchronize((hipStream_t) s); }
int nh_device_sync(void) { return (int) hipDeviceSynchronize(); }
int nh_event_create(nh_event_t* e) { return (int) hipEventCreate((hipEvent_t*) e); }
int nh_event_destroy(nh_event_t e) { return (int) hipEventDestroy((hipEvent_t) e); }
int nh_event_record(nh_event_t e, nh_stream_t s) { return (int) hipEventRecord((hipEvent_t) e, (hipStream_t) s); }
int nh_event_sync(nh_event_t e) { return (int) hipEventSynchronize((hipEvent_t) e); }
int nh_event_elapsed_ms(float* ms, nh_event_t a, nh_event_t b) { return (int) hipEventElapsedTime(ms, (hipEvent_t) a, (hipEvent_t) b); }
int nh_stream_wait_event(nh_stream_t s, nh_event_t e) { return (int) hipStreamWaitEvent((hipStream_t) s, (hipEvent_t) e, 0); }
int nh_last_error(void) { return (int) hipGetLastError(); }
const char* nh_error_string(int err) { return hipGetErrorString((hipError_t) err); }
int nh_device_info(int dev, char* name, int namelen, int* cus, uint64_t* mem_bytes, int* clock_khz) {
    hipDeviceProp_t p;
    const hipError_t e = hipGetDeviceProperties(&p, dev);
    if (e != hipSuccess) return (int) e;
    if (name && namelen > 0) {
        strncpy(name, p.name, (size_t) namelen - 1);
        name[namelen - 1] = 0;
    }
    if (cus) *cus = p.multiProcessorCount;
    if (mem_bytes) *mem_bytes = (uint64_t) p.totalGlobalMem;
    if (clock_khz) *clock_khz = p.clockRate;
    return 0;
}
int nh_mem_info(uint64_t* free_bytes, uint64_t* total_bytes) {
    size_t f = 0, t = 0;
    const hipError_t e = hipMemGetInfo(&f, &t);
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = t;
    return (int) e;
}

// ---- capture / replay of a launch sequence (declared in moe_layer.h) ----
struct NslmGraph {
    hipGraph_t graph;
    hipGraphExec_t exec;
};
int nslm_graph_begin(void* s) { return (int) hipStreamBeginCapture((hipStream_t) s, hipStreamCaptureModeThreadLocal); }
NslmGraph* nslm_graph_end(void* s) {
    hipGraph_t g = nullptr;
    if (hipStreamEndCapture((hipStream_t) s, &g) != hipSuccess || !g) return nullptr;
    hipGraphExec_t ex = nullptr;
    if (hipGraphInstantiate(&ex, g, nullptr, nullptr, 0) != hipSuccess) {
        (void) hipGraphDestroy(g);
        return nullptr;
    }
    return new NslmGraph{g, ex};
}
int nslm_graph_launch(NslmGraph* g, void* s) { return (int) hipGraphLaunch(g->exec, (hipStream_t) s); }
int nslm_stream_capturing(void* s) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    return hipStreamIsCapturing((hipStream_t) s, &st) == hipSuccess && st == hipStreamCaptureStatusActive;
}
void nslm_graph_free(NslmGraph* g) {
    if (!g) return;
    (void) hipGraphExecDestroy(g->exec);
    (void) hipGraphDestroy(g->graph);
    delete g;
}

}   // extern "C"

/* include/nslm_rt.h - the thin C-ABI layer over the HIP runtime that a C99 host (the reference's engine/mova_cuda.c,
 * tests/kernel_backend_cuda.c) needs in place of its cuda* calls: device memory, copies, streams, events.  No HIP header
 * is needed to include this file.  Every function returns 0 on success or a non-zero hipError_t value; nh_error_string
 * names it.  The reference call each one stands in for is named beside it.
 */
#pragma once
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* nh_stream_t; /* = kc_stream_t */
typedef void* nh_event_t;

int nh_device_count(int* n);                                  /* cudaGetDeviceCount (tests/kernel_backend_cuda.c:45) */
int nh_set_device(int dev);                                   /* cudaSetDevice (engine/mova_cuda.c:590) */
int nh_malloc(void** p, size_t n);                            /* cudaMalloc */
int nh_free(void* p);                                         /* cudaFree */
int nh_host_alloc(void** p, size_t n);                        /* cudaHostAlloc, pinned and device-visible (engine/mova_cuda.c:193-202) */
int nh_host_free(void* p);                                    /* cudaFreeHost */
int nh_memcpy_h2d(void* dst, const void* src, size_t n);      /* cudaMemcpy(HostToDevice) */
int nh_memcpy_d2h(void* dst, const void* src, size_t n);      /* cudaMemcpy(DeviceToHost) */
int nh_memcpy_d2d(void* dst, const void* src, size_t n);      /* cudaMemcpy(DeviceToDevice) */
int nh_memcpy_h2d_async(void* dst, const void* src, size_t n, nh_stream_t s);   /* cudaMemcpyAsync */
int nh_memcpy_d2h_async(void* dst, const void* src, size_t n, nh_stream_t s);
int nh_memcpy_d2d_async(void* dst, const void* src, size_t n, nh_stream_t s);   /* cudaMemcpyAsync(DeviceToDevice) */
int nh_memcpy_async(void* dst, const void* src, size_t n, nh_stream_t s);       /* cudaMemcpyAsync(cudaMemcpyDefault): direction from the pointers */
int nh_memset(void* p, int v, size_t n);                      /* cudaMemset */
/* cudaMemsetAsync (engine/mova_cuda.c:1160): a fill kernel on s, not a memset node, so the call may be captured into a graph */
int nh_memset_async(void* p, int v, size_t n, nh_stream_t s);
/* cudaHostAlloc(cudaHostAllocMapped) + cudaHostGetDevicePointer (engine/mova_cuda.c:352, engine/qwen4_cuda.c:186,397): pinned host memory and the
 * address kernels use for it (results a kernel leaves where the host polls them; pass dev = NULL to skip the second call) */
int nh_host_alloc_mapped(void** host, void** dev, size_t n);
int nh_host_device_ptr(void** dev, void* host);               /* cudaHostGetDevicePointer, for memory from nh_host_alloc */
int nh_get_device(int* dev);                                  /* cudaGetDevice */
int nh_stream_create(nh_stream_t* s);                         /* cudaStreamCreateWithFlags(NonBlocking), default priority */
/* cudaDeviceGetStreamPriorityRange / cudaStreamCreateWithPriority (engine/mova_cuda.c:892, the copy stream): this layer
 * has one priority - the range is [0, 0] and the priority asked for is ignored - because streams of different priorities
 * are not used on these GPUs; a host that orders work by priority still runs, its streams then share the GPU evenly */
int nh_stream_priority_range(int* least, int* greatest);
int nh_stream_create_prio(nh_stream_t* s, int priority);
int nh_event_create_untimed(nh_event_t* e);                   /* cudaEventCreateWithFlags(cudaEventDisableTiming) */
int nh_stream_destroy(nh_stream_t s);
int nh_stream_sync(nh_stream_t s);                            /* cudaStreamSynchronize */
int nh_device_sync(void);                                     /* cudaDeviceSynchronize */
int nh_event_create(nh_event_t* e);                           /* cudaEventCreate */
int nh_event_destroy(nh_event_t e);
int nh_event_record(nh_event_t e, nh_stream_t s);             /* cudaEventRecord */
int nh_event_sync(nh_event_t e);                              /* cudaEventSynchronize */
int nh_event_elapsed_ms(float* ms, nh_event_t a, nh_event_t b); /* cudaEventElapsedTime */
int nh_stream_wait_event(nh_stream_t s, nh_event_t e);        /* cudaStreamWaitEvent */
int nh_last_error(void);                                      /* cudaGetLastError */
const char* nh_error_string(int err);                         /* cudaGetErrorString */
/* name (<= 255 chars), compute units, HBM bytes, shader clock kHz of a device */
int nh_device_info(int dev, char* name, int namelen, int* cus, uint64_t* mem_bytes, int* clock_khz);
/* free and total device memory: the reference's VRAM reserve helper reads these (engine/vram.h:9-15) */
int nh_mem_info(uint64_t* free_bytes, uint64_t* total_bytes);

#ifdef __cplusplus
}
#endif

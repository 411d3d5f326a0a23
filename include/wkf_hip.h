/*
 * wkf_hip.h -- level 0 of the C ABI: the thin HIP layer the tensor host calls
 * instead of wgpu.  Plain C, opaque handles, status-code returns; nothing here
 * throws or aborts across the boundary.
 *
 * Each entry point replaces one group of wgpu calls of the reference crate
 * (paths relative to the reference checkout).  One stream per device; every
 * call on a device is serialised by a per-device mutex, so handles may be used
 * from any thread.
 */
#ifndef WKF_HIP_H
#define WKF_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct wkf_device wkf_device;
typedef struct wkf_buffer wkf_buffer;
typedef struct wkf_kernel wkf_kernel;
typedef struct wkf_timer wkf_timer;

enum {
  WKF_OK = 0,
  WKF_ERR_HIP = 1,         /* a HIP runtime call failed */
  WKF_ERR_HIPRTC = 2,      /* JIT compilation failed; wkf_last_error() holds the log */
  WKF_ERR_INVALID_ARG = 3, /* shape / dtype / handle misuse (the reference panics here) */
  WKF_ERR_OOM = 4,
  WKF_ERR_NO_DEVICE = 5,   /* the call needs a GPU but the device is plan-only */
  WKF_ERR_UNSUPPORTED = 6
};

typedef struct wkf_props {
  int ordinal;               /* -1 for a plan-only device */
  int compute_units;
  int wave_size;             /* 64 on gfx950 */
  int max_threads_per_block; /* replaces limits().max_compute_workgroup_size_x, src/reduce.rs:340 */
  int clock_khz;
  size_t lds_bytes_per_block;
  size_t total_mem_bytes;
  char arch[32];
} wkf_props;

/* Replaces Instance::new / request_adapter / request_device, src/device.rs:14-32.
 * hipSetDevice(ordinal) + one hipStream_t at default priority. */
int wkf_device_create(int ordinal, wkf_device** out);
/* A device with no GPU behind it: buffers live in host memory, kernels are
 * generated and JIT-compiled for gfx950 but never launched, and downloading a
 * computed buffer fails with WKF_ERR_NO_DEVICE.  It exists so that layout,
 * fusion and code generation can be tested on a machine without a GPU; it
 * computes nothing.  No counterpart in the reference. */
int wkf_device_create_planner(wkf_device** out);
/* Drops the caller's handle.  While buffers of the device (or tensors that own some) are still alive the device
 * itself lives on and is torn down by the release of the last one, so a late wkf_buffer_release /
 * wkf_tensor_free is always safe; no new work may be started through the handle after this call.  Timers
 * are not counted: destroy them first. */
void wkf_device_destroy(wkf_device* dev);
int wkf_device_is_planner(const wkf_device* dev);
/* Replaces wgpu_device().limits(), src/reduce.rs:340. */
int wkf_device_props(wkf_device* dev, wkf_props* out);
/* Replaces device.poll(Wait) spun by every reference test (e.g.
 * src/element_wise.rs:216-221) and the implicit wait in queue.submit /
 * DownloadBuffer (src/compute_graph/mod.rs:241-248).  hipStreamSynchronize. */
int wkf_device_sync(wkf_device* dev);
/* Return cached free device memory of the buffer pool to the driver. */
int wkf_device_trim(wkf_device* dev);
/* Since the device was created: calls of wkf_buffer_alloc, the hipMalloc calls among them (the others were served
 * by the pool), timers created, and the buffers alive now.  No reference counterpart (wgpu keeps no such count);
 * lets a caller prove that a call allocated nothing.  Any pointer may be null. */
int wkf_device_alloc_stats(wkf_device* dev, uint64_t* buffer_allocs, uint64_t* device_mallocs, uint64_t* timers, uint64_t* live_buffers);

/* Replaces create_buffer (zero-initialised by wgpu): src/tensor.rs:334,369,
 * src/element_wise.rs:143, src/reduce.rs:300, src/matmul.rs:167.
 * zero_fill != 0 clears the buffer on the device stream (hipMalloc does not). */
int wkf_buffer_alloc(wkf_device* dev, size_t bytes, int zero_fill, wkf_buffer** out);
void wkf_buffer_retain(wkf_buffer* buf);
void wkf_buffer_release(wkf_buffer* buf);
/* Arc::strong_count(&buffer), i.e. TensorData::owned() at src/tensor.rs:413-415. */
int wkf_buffer_refcount(const wkf_buffer* buf);
size_t wkf_buffer_size(const wkf_buffer* buf);
void* wkf_buffer_ptr(const wkf_buffer* buf);
/* Replaces the mapped-at-creation write + unmap, src/tensor.rs:374-378. hipMemcpyAsync H2D. */
int wkf_buffer_upload(wkf_buffer* buf, size_t offset, const void* src, size_t bytes);
/* Replaces DownloadBuffer::read_buffer, src/tensor.rs:538-546. hipMemcpyAsync D2H + stream sync. */
int wkf_buffer_download(wkf_buffer* buf, size_t offset, void* dst, size_t bytes);
/* Device-to-device copy on the stream (no reference counterpart; used by benches to rotate inputs). */
int wkf_buffer_copy(wkf_buffer* dst, wkf_buffer* src, size_t bytes);

/* Replaces create_shader_module + pipeline / bind-group layout creation,
 * src/device.rs:34-44 and src/kernel.rs:179-272.  Looks the signature up in the
 * device's memory cache, then in the on-disk code-object cache, else compiles
 * `hip_source` with hiprtc for gfx950 and loads it (hipModuleLoadData +
 * hipModuleGetFunction).  The returned kernel is owned by the device. */
int wkf_module_get(wkf_device* dev, const char* signature, const char* hip_source,
                   const char* entry, wkf_kernel** out);
/* Memory-cache lookup only: *out is the kernel, or NULL when this device has not seen the
 * signature yet (the caller then generates the source and calls wkf_module_get).  Lets the
 * generator skip building source text on the hot path; no reference counterpart (the reference
 * regenerates and recompiles its WGSL on every launch, src/kernel.rs:262-271,371-373). */
int wkf_module_find(wkf_device* dev, const char* signature, wkf_kernel** out);
/* Cache statistics since device creation: kernels compiled by hiprtc, loaded
 * from disk, and served from memory. */
int wkf_module_stats(wkf_device* dev, uint64_t* compiled, uint64_t* disk_hits, uint64_t* mem_hits);

/* Replaces begin_compute_pass / set_pipeline / set_bind_group /
 * dispatch_workgroups, src/kernel.rs:375-384.  `args` is the packed kernel
 * argument block (it also replaces the per-tensor uniform buffers of
 * src/kernel.rs:274-361), laid out as the kernel's argument struct including
 * its tail padding: `arg_bytes` is a multiple of 8 (anything else is refused).
 * hipModuleLaunchKernel on the device stream; when
 * `timer` is non-NULL the launch carries the timer's two events in the dispatch
 * itself (hipExtModuleLaunchKernel): they take the kernel's own begin and end
 * timestamps, as the reference's timestamp queries around a compute pass do
 * (src/query.rs:50-126), and put nothing else on the stream.  With
 * WKF_TIMER_EVENTS=1 in the environment, or a grid of more than 2^32 - 1
 * work-items in one dimension, two events are recorded around the launch
 * instead (about 2.5 us more per launch, and the gap to the kernel before). */
int wkf_launch(wkf_device* dev, wkf_kernel* kernel, const uint32_t grid[3],
               const uint32_t block[3], uint32_t dyn_lds_bytes, const void* args,
               size_t arg_bytes, wkf_timer* timer);

/* Replace QuerySet / resolve_query_set / map_async, src/query.rs:51-114. */
int wkf_timer_create(wkf_device* dev, wkf_timer** out);
void wkf_timer_destroy(wkf_timer* t);
/* Record the timer's begin / end events on the device stream by hand. */
int wkf_timer_begin(wkf_timer* t);
int wkf_timer_end(wkf_timer* t);
/* QueryResults::elapsed(), src/query.rs:36-42.  Synchronises on the end event. */
int wkf_timer_elapsed_ns(wkf_timer* t, uint64_t* out);

/* The reference panics; this ABI returns a status code and keeps the message
 * (including the hiprtc log) in a thread-local string. */
const char* wkf_last_error(void);

#ifdef __cplusplus
}
#endif
#endif

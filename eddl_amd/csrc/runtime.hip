// Device runtime of libeddlhip.so: initialisation, memory, copies, events, error text.
// Stands where the reference's gpu_init / gpu_create_tensor / gpu_copy_* do
// (src/hardware/gpu/gpu_tensor.cu:121-240, src/hardware/gpu/gpu_core.cu:49-67).
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "common.h"

namespace eddlhip {

static DeviceState g_state[EDDLHIP_MAX_DEVICES];
static thread_local char g_error[512] = "";

DeviceState &state(int dev) { return g_state[dev]; }

int set_error(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

void clear_error() { g_error[0] = 0; }

int use_device(int dev) {
    if (dev < 0 || dev >= EDDLHIP_MAX_DEVICES) return set_error(EDDLHIP_ENODEV, "device index %d out of range", dev);
    DeviceState &s = g_state[dev];
    if (!s.inited) {
        int count = 0;
        EH_TRY_HIP(hipGetDeviceCount(&count));
        if (dev >= count) return set_error(EDDLHIP_ENODEV, "device %d requested, %d present", dev, count);
        EH_TRY_HIP(hipSetDevice(dev));
        hipDeviceProp_t prop;
        EH_TRY_HIP(hipGetDeviceProperties(&prop, dev));
        if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
            return set_error(EDDLHIP_ENODEV, "device %d is %s; this library holds gfx950 code only", dev, prop.gcnArchName);
        s.num_cu = prop.multiProcessorCount;
        EH_TRY_HIP(hipMalloc(&s.flag, 256));
        EH_TRY_HIP(hipMemset(s.flag, 0, 256));
        EH_TRY(conv_setup_device(dev));
        s.inited = true;
        return 0;
    }
    EH_TRY_HIP(hipSetDevice(dev));
    return 0;
}

int get_workspace(int dev, size_t bytes, void **ptr) {
    DeviceState &s = g_state[dev];
    if (bytes > s.workspace_bytes) {
        if (s.capturing)
            return set_error(EDDLHIP_EINVAL, "the workspace would have to grow to %zu bytes while a graph is being recorded: "
                             "run the same calls once before recording them", bytes);
        if (s.workspace) {
            EH_TRY_HIP(hipStreamSynchronize(s.stream));
            EH_TRY_HIP(hipFree(s.workspace));
            s.workspace = nullptr;
            s.workspace_bytes = 0;
        }
        size_t want = (bytes + (size_t(1) << 20) - 1) & ~((size_t(1) << 20) - 1);
        hipError_t e = hipMalloc(&s.workspace, want);
        if (e != hipSuccess) {
            s.workspace = nullptr;
            return set_error(EDDLHIP_ENOMEM, "workspace of %zu bytes: %s", want, hipGetErrorString(e));
        }
        s.workspace_bytes = want;
        s.workspace_generation++;
    }
    if (s.capturing && bytes > 0) s.capture_used_workspace = true;
    *ptr = s.workspace;
    return 0;
}

int release_workspace(int dev) {
    DeviceState &s = g_state[dev];
    if (s.workspace == nullptr) return 0;
    EH_TRY_HIP(hipStreamSynchronize(s.stream));
    EH_TRY_HIP(hipFree(s.workspace));
    s.workspace = nullptr;
    s.workspace_bytes = 0;
    s.workspace_generation++;  // graphs recorded before name memory that is gone
    return 0;
}

}  // namespace eddlhip

using namespace eddlhip;

extern "C" {

const char *eddlhip_version(void) { return "eddlhip 0.1 (gfx950)"; }

const char *eddlhip_last_error(void) { return g_error; }

int eddlhip_device_count(int *count) {
    EH_REQUIRE(count != nullptr, "count is NULL");
    EH_TRY_HIP(hipGetDeviceCount(count));
    return 0;
}

int eddlhip_init(int dev) { return use_device(dev); }

int eddlhip_shutdown(int dev) {
    if (dev < 0 || dev >= EDDLHIP_MAX_DEVICES) return set_error(EDDLHIP_ENODEV, "device index %d out of range", dev);
    DeviceState &s = g_state[dev];
    if (!s.inited) return 0;
    EH_NOT_CAPTURING(dev, "eddlhip_shutdown");
    EH_TRY_HIP(hipSetDevice(dev));
    EH_TRY_HIP(hipDeviceSynchronize());
    EH_TRY(eddlhip_conv2d_uncache_filters(dev, nullptr));
    if (s.workspace) EH_TRY_HIP(hipFree(s.workspace));
    if (s.flag) EH_TRY_HIP(hipFree(s.flag));
    for (hipStream_t cs : s.copy_stream)
        if (cs) EH_TRY_HIP(hipStreamDestroy(cs));
    if (s.capture_stream) EH_TRY_HIP(hipStreamDestroy(s.capture_stream));
    const unsigned long generation = s.workspace_generation;
    s = DeviceState();
    s.workspace_generation = generation + 1;  // graphs recorded before the shutdown name a workspace that is gone
    return 0;
}

int eddlhip_workspace_bytes(int dev, size_t *bytes) {
    EH_REQUIRE(bytes != nullptr, "bytes is NULL");
    EH_TRY(use_device(dev));
    *bytes = state(dev).workspace_bytes;
    return 0;
}

int eddlhip_workspace_trim(int dev) {
    EH_TRY(use_device(dev));
    EH_NOT_CAPTURING(dev, "eddlhip_workspace_trim");
    return release_workspace(dev);
}

int eddlhip_device_name(int dev, char *buf, size_t buflen) {
    EH_REQUIRE(buf != nullptr && buflen > 0, "buf is NULL");
    EH_TRY(use_device(dev));
    hipDeviceProp_t prop;
    EH_TRY_HIP(hipGetDeviceProperties(&prop, dev));
    snprintf(buf, buflen, "%s (%s, %d CUs)", prop.name, prop.gcnArchName, prop.multiProcessorCount);
    return 0;
}

int eddlhip_set_stream(int dev, void *hip_stream) {
    EH_TRY(use_device(dev));
    EH_NOT_CAPTURING(dev, "eddlhip_set_stream");
    state(dev).stream = (hipStream_t)hip_stream;
    return 0;
}

int eddlhip_synchronize(int dev) {
    EH_TRY(use_device(dev));
    EH_NOT_CAPTURING(dev, "eddlhip_synchronize");
    EH_TRY_HIP(hipStreamSynchronize(state(dev).stream));
    return 0;
}

int eddlhip_malloc(int dev, size_t bytes, void **dev_ptr) {
    EH_REQUIRE(dev_ptr != nullptr, "dev_ptr is NULL");
    EH_TRY(use_device(dev));
    EH_NOT_CAPTURING(dev, "eddlhip_malloc");
    *dev_ptr = nullptr;
    if (bytes == 0) return 0;
    hipError_t e = hipMalloc(dev_ptr, bytes);
    if (e != hipSuccess) {
        *dev_ptr = nullptr;
        (void)hipGetLastError();
        return set_error(EDDLHIP_ENOMEM, "hipMalloc(%zu): %s", bytes, hipGetErrorString(e));
    }
    return 0;
}

int eddlhip_free(int dev, void *dev_ptr) {
    if (!dev_ptr) return 0;
    EH_TRY(use_device(dev));
    EH_NOT_CAPTURING(dev, "eddlhip_free");
    void *base = nullptr;
    size_t size = 0;
    if (hipMemGetAddressRange(&base, &size, dev_ptr) == hipSuccess) conv_filters_released(dev, base, size);
    else (void)hipGetLastError();
    EH_TRY_HIP(hipFree(dev_ptr));
    return 0;
}

// The three copies wait for earlier kernels on the device's stream and return when the data
// has landed, like the reference's plain cudaMemcpy calls.
int eddlhip_memcpy_h2d(int dev, void *dev_dst, const void *host_src, size_t bytes) {
    if (bytes == 0) return 0;
    EH_REQUIRE(dev_dst && host_src, "NULL pointer in h2d copy");
    EH_TRY(use_device(dev));
    EH_NOT_CAPTURING(dev, "eddlhip_memcpy_h2d");
    conv_filters_written(dev, dev_dst, bytes);
    EH_TRY_HIP(hipMemcpyAsync(dev_dst, host_src, bytes, hipMemcpyHostToDevice, state(dev).stream));
    EH_TRY_HIP(hipStreamSynchronize(state(dev).stream));
    return 0;
}

int eddlhip_memcpy_d2h(int dev, void *host_dst, const void *dev_src, size_t bytes) {
    if (bytes == 0) return 0;
    EH_REQUIRE(host_dst && dev_src, "NULL pointer in d2h copy");
    EH_TRY(use_device(dev));
    EH_NOT_CAPTURING(dev, "eddlhip_memcpy_d2h");
    EH_TRY_HIP(hipMemcpyAsync(host_dst, dev_src, bytes, hipMemcpyDeviceToHost, state(dev).stream));
    EH_TRY_HIP(hipStreamSynchronize(state(dev).stream));
    return 0;
}

int eddlhip_memcpy_d2d(int dev, void *dev_dst, const void *dev_src, size_t bytes) {
    if (bytes == 0) return 0;
    EH_REQUIRE(dev_dst && dev_src, "NULL pointer in d2d copy");
    EH_TRY(use_device(dev));
    conv_filters_written(dev, dev_dst, bytes);
    EH_TRY_HIP(hipMemcpyAsync(dev_dst, dev_src, bytes, hipMemcpyDeviceToDevice, state(dev).stream));
    return 0;
}

// ---- batch staging: pinned host buffers and copies on a second stream, so that the transfer of
// batch i+1 and of the results of batch i-1 overlap the kernels of batch i
int eddlhip_host_malloc(int dev, void **host_ptr, size_t bytes) {
    EH_REQUIRE(host_ptr != nullptr, "host_ptr is NULL");
    EH_TRY(use_device(dev));
    *host_ptr = nullptr;
    if (bytes == 0) return 0;
    hipError_t e = hipHostMalloc(host_ptr, bytes, hipHostMallocDefault);
    if (e != hipSuccess) {
        *host_ptr = nullptr;
        (void)hipGetLastError();
        return set_error(EDDLHIP_ENOMEM, "hipHostMalloc(%zu): %s", bytes, hipGetErrorString(e));
    }
    return 0;
}

int eddlhip_host_free(int dev, void *host_ptr) {
    if (!host_ptr) return 0;
    EH_TRY(use_device(dev));
    EH_TRY_HIP(hipHostFree(host_ptr));
    return 0;
}

// which: 0 = upload stream, 1 = download stream (separate, so that an upload queued after a
// download that is still waiting for kernels does not wait with it)
static int copy_stream_of(int dev, int which, hipStream_t *out) {
    DeviceState &s = state(dev);
    if (!s.copy_stream[which]) EH_TRY_HIP(hipStreamCreateWithFlags(&s.copy_stream[which], hipStreamNonBlocking));
    *out = s.copy_stream[which];
    return 0;
}

int eddlhip_memcpy_h2d_async(int dev, void *dev_dst, const void *host_src, size_t bytes, void *done_event) {
    EH_REQUIRE(bytes == 0 || (dev_dst && host_src), "NULL pointer in asynchronous h2d copy");
    EH_TRY(use_device(dev));
    hipStream_t cs;
    EH_TRY(copy_stream_of(dev, 0, &cs));
    if (bytes) {
        conv_filters_written(dev, dev_dst, bytes);
        EH_TRY_HIP(hipMemcpyAsync(dev_dst, host_src, bytes, hipMemcpyHostToDevice, cs));
    }
    if (done_event) EH_TRY_HIP(hipEventRecord((hipEvent_t)done_event, cs));
    return 0;
}

int eddlhip_memcpy_d2h_async(int dev, void *host_dst, const void *dev_src, size_t bytes, void *done_event) {
    EH_REQUIRE(bytes == 0 || (host_dst && dev_src), "NULL pointer in asynchronous d2h copy");
    EH_TRY(use_device(dev));
    hipStream_t cs;
    EH_TRY(copy_stream_of(dev, 1, &cs));
    if (bytes) EH_TRY_HIP(hipMemcpyAsync(host_dst, dev_src, bytes, hipMemcpyDeviceToHost, cs));
    if (done_event) EH_TRY_HIP(hipEventRecord((hipEvent_t)done_event, cs));
    return 0;
}

int eddlhip_stream_wait_event(int dev, void *event) {
    EH_REQUIRE(event != nullptr, "event is NULL");
    EH_TRY(use_device(dev));
    EH_TRY_HIP(hipStreamWaitEvent(state(dev).stream, (hipEvent_t)event, 0));
    return 0;
}

int eddlhip_upload_wait_event(int dev, void *event) {
    EH_REQUIRE(event != nullptr, "event is NULL");
    EH_TRY(use_device(dev));
    hipStream_t cs;
    EH_TRY(copy_stream_of(dev, 0, &cs));
    EH_TRY_HIP(hipStreamWaitEvent(cs, (hipEvent_t)event, 0));
    return 0;
}

int eddlhip_download_wait_event(int dev, void *event) {
    EH_REQUIRE(event != nullptr, "event is NULL");
    EH_TRY(use_device(dev));
    hipStream_t cs;
    EH_TRY(copy_stream_of(dev, 1, &cs));
    EH_TRY_HIP(hipStreamWaitEvent(cs, (hipEvent_t)event, 0));
    return 0;
}

// ---- graphs: a fixed sequence of launches recorded once and replayed with one call, for plans whose
// kernels are so short that queueing them one by one takes longer than running them
//
// A recorded kernel that took the library's workspace has that address frozen into its arguments, and the
// workspace is replaced (freed) when a later call needs a larger one.  The handle therefore remembers which
// workspace the recording saw, and a replay after a replacement is refused instead of writing into freed memory.
namespace {
struct RecordedGraph {
    hipGraphExec_t exec;
    int dev;
    bool uses_workspace;
    unsigned long workspace_generation;
};
}  // namespace

int eddlhip_graph_begin(int dev) {
    EH_TRY(use_device(dev));
    DeviceState &s = state(dev);
    EH_REQUIRE(!s.capturing, "graph_begin: a graph is already being recorded on device %d", dev);
    if (!s.capture_stream) EH_TRY_HIP(hipStreamCreateWithFlags(&s.capture_stream, hipStreamNonBlocking));
    EH_TRY_HIP(hipStreamBeginCapture(s.capture_stream, hipStreamCaptureModeThreadLocal));
    s.stream_before_capture = s.stream;
    s.stream = s.capture_stream;
    s.capturing = true;
    s.capture_used_workspace = false;
    return 0;
}

int eddlhip_graph_end(int dev, void **graph) {
    EH_REQUIRE(graph != nullptr, "graph_end: graph is NULL");
    EH_TRY(use_device(dev));
    DeviceState &s = state(dev);
    EH_REQUIRE(s.capturing, "graph_end: no graph is being recorded on device %d", dev);
    *graph = nullptr;
    hipGraph_t g = nullptr;
    const hipError_t e = hipStreamEndCapture(s.capture_stream, &g);
    s.stream = s.stream_before_capture;
    s.capturing = false;
    if (e != hipSuccess || g == nullptr) {
        (void)hipGetLastError();
        if (g) (void)hipGraphDestroy(g);
        return set_error(EDDLHIP_EHIP, "graph_end: the recording is not valid (%s); a call that waits, copies to or from the host, "
                         "allocates or fails ends it", hipGetErrorString(e));
    }
    hipGraphExec_t exec = nullptr;
    const hipError_t ei = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (ei != hipSuccess) {
        (void)hipGetLastError();
        return set_error(EDDLHIP_EHIP, "graph_end: hipGraphInstantiate: %s", hipGetErrorString(ei));
    }
    *graph = (void *)new RecordedGraph{exec, dev, s.capture_used_workspace, s.workspace_generation};
    return 0;
}

int eddlhip_graph_launch(int dev, void *graph) {
    EH_REQUIRE(graph != nullptr, "graph_launch: graph is NULL");
    EH_TRY(use_device(dev));
    EH_NOT_CAPTURING(dev, "eddlhip_graph_launch");
    const RecordedGraph *g = (const RecordedGraph *)graph;
    EH_REQUIRE(g->dev == dev, "graph_launch: the graph was recorded on device %d, not %d", g->dev, dev);
    EH_REQUIRE(!g->uses_workspace || g->workspace_generation == state(dev).workspace_generation,
               "graph_launch: the library's workspace was reallocated since recording (a later call needed a larger one) and the "
               "graph's kernels still name the old one: record again");
    EH_TRY_HIP(hipGraphLaunch(g->exec, state(dev).stream));
    return 0;
}

int eddlhip_graph_destroy(int dev, void *graph) {
    if (!graph) return 0;
    EH_TRY(use_device(dev));
    RecordedGraph *g = (RecordedGraph *)graph;
    const hipError_t e = hipGraphExecDestroy(g->exec);
    delete g;
    EH_TRY_HIP(e);
    return 0;
}

int eddlhip_event_synchronize(int dev, void *event) {
    EH_REQUIRE(event != nullptr, "event is NULL");
    EH_TRY(use_device(dev));
    EH_TRY_HIP(hipEventSynchronize((hipEvent_t)event));
    return 0;
}

int eddlhip_event_create(int dev, void **event) {
    EH_REQUIRE(event != nullptr, "event is NULL");
    EH_TRY(use_device(dev));
    hipEvent_t ev;
    EH_TRY_HIP(hipEventCreate(&ev));
    *event = (void *)ev;
    return 0;
}

int eddlhip_event_destroy(int dev, void *event) {
    if (!event) return 0;
    EH_TRY(use_device(dev));
    EH_TRY_HIP(hipEventDestroy((hipEvent_t)event));
    return 0;
}

int eddlhip_event_record(int dev, void *event) {
    EH_REQUIRE(event != nullptr, "event is NULL");
    EH_TRY(use_device(dev));
    EH_TRY_HIP(hipEventRecord((hipEvent_t)event, state(dev).stream));
    return 0;
}

int eddlhip_event_elapsed_ms(int dev, void *start, void *stop, float *ms) {
    EH_REQUIRE(start && stop && ms, "NULL argument");
    EH_TRY(use_device(dev));
    EH_TRY_HIP(hipEventSynchronize((hipEvent_t)stop));
    EH_TRY_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return 0;
}

}  // extern "C"

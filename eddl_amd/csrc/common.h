// Shared state and helpers of libeddlhip.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/eddlhip.h"

#define EDDLHIP_MAX_DEVICES 16
#define EDDLHIP_NUM_XCD 8  // MI355X: 256 CUs in 8 XCDs, workgroups are dealt to XCDs round-robin

namespace eddlhip {

struct DeviceState {
    bool inited = false;
    hipStream_t stream = nullptr;  // null stream unless the caller installed its own
    int num_cu = 0;
    void *workspace = nullptr;  // private, grow-only (repacked filters, split-K partials)
    size_t workspace_bytes = 0;
    unsigned long workspace_generation = 0;  // counts replacements of the workspace by a larger one
    bool capture_used_workspace = false;     // a call recorded into the graph being captured took the workspace
    void *flag = nullptr;  // one int of device memory for kernels that report a condition
    hipStream_t copy_stream[2] = {nullptr, nullptr};  // uploads, downloads: created on first use (non-blocking, default priority)
    // eddlhip_graph_begin .. _end: launches go to capture_stream and are recorded, not run
    bool capturing = false;
    hipStream_t capture_stream = nullptr;  // created on first use (non-blocking, default priority)
    hipStream_t stream_before_capture = nullptr;
};

DeviceState &state(int dev);
int set_error(int code, const char *fmt, ...);
// Empties the calling thread's error text (after a failure that was handled inside the library).
void clear_error();
// Makes `dev` current and initialises it on first use.
int use_device(int dev);
// Returns a workspace of at least `bytes` (contents undefined); waits for the stream before
// replacing a smaller one so that kernels still reading it finish first.
int get_workspace(int dev, size_t bytes, void **ptr);
// Waits for the stream and frees the workspace; the next get_workspace allocates what it needs.
int release_workspace(int dev);
// Hooks of the convolution's cache of repacked filters: the library's own copy / fill / free entry
// points report device ranges they write or release, so a registered filter tensor whose contents
// change is repacked before its next use and one that is freed is forgotten.
void conv_filters_written(int dev, const void *dst, size_t bytes);
void conv_filters_released(int dev, const void *base, size_t bytes);
// Per-device set-up of the convolution code (address of its fixed scratch array, kernel occupancies);
// use_device calls it once, when it initialises the device.
int conv_setup_device(int dev);

}  // namespace eddlhip

#define EH_TRY_HIP(expr)                                                                          \
    do {                                                                                          \
        hipError_t _e = (expr);                                                                   \
        if (_e != hipSuccess)                                                                     \
            return eddlhip::set_error(EDDLHIP_EHIP, "%s: %s (%s:%d)", #expr, hipGetErrorString(_e), \
                                      __FILE__, __LINE__);                                        \
    } while (0)

#define EH_TRY(expr)          \
    do {                      \
        int _r = (expr);      \
        if (_r != 0) return _r; \
    } while (0)

#define EH_REQUIRE(cond, ...)                                            \
    do {                                                                 \
        if (!(cond)) return eddlhip::set_error(EDDLHIP_EINVAL, __VA_ARGS__); \
    } while (0)

#define EH_CHECK_LAUNCH() EH_TRY_HIP(hipGetLastError())

// For entry points that wait for the device, allocate or free: not possible while a graph is being recorded.
#define EH_NOT_CAPTURING(dev, what)                                                                                   \
    EH_REQUIRE(!eddlhip::state(dev).capturing, "%s is not possible between eddlhip_graph_begin and eddlhip_graph_end", what)

static inline unsigned eh_blocks(size_t work, unsigned per_block, unsigned cap = 1u << 20) {
    size_t b = (work + per_block - 1) / per_block;
    if (b < 1) b = 1;
    if (b > cap) b = cap;
    return (unsigned)b;
}

// Device probes: what the matrix pipe and the memory system sustain on this device when nothing else runs.
// First, the rate of v_mfma_f32_32x32x2_f32.
// The published fp32 matrix peak assumes the top engine clock; under a stream of MFMAs whose
// operands change from instruction to instruction (as a convolution's do) the device lowers its
// clock, and the sustained rate is what a kernel can be measured against.  Not part of the
// reference's interface; the benchmark reports it beside the published peak.
#include "common.h"
#include "../../include/eddlhip_probe.h"

using namespace eddlhip;

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
constexpr int kMaxLaunches = 256;

// `in` holds 16 x 256 floats: eight A and eight B operand registers per thread.  With
// vary == 0 every MFMA reads the same two registers (the most favourable case for power).
__global__ __launch_bounds__(256) void mfma_f32_probe_kernel(const float *in, float *out, int iters, int vary) {
    floatx16 acc[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[i][v] = 0.0f;
    float a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        a[i] = in[(vary ? i : 0) * 256 + threadIdx.x];
        b[i] = in[(8 + (vary ? i : 0)) * 256 + threadIdx.x];
    }
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int u = 0; u < 8; u++) {
            acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u], b[u], acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u], b[(u + 3) & 7], acc[1], 0, 0, 0);
            acc[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[(u + 5) & 7], b[u], acc[2], 0, 0, 0);
            acc[3] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[(u + 5) & 7], b[(u + 3) & 7], acc[3], 0, 0, 0);
        }
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) s += acc[i][v];
    out[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

// Second, plain streams over device memory: read only, write only, copy.  Grid-stride loops with U 16-byte
// accesses in flight per thread; the host tries a few grid sizes and keeps the best, since the rate
// depends on how many wavefronts walk the memory at once.
typedef float fx4 __attribute__((ext_vector_type(4)));

template <int U, bool STREAMING>
__global__ __launch_bounds__(256) void hbm_read_kernel(const fx4 *__restrict__ a, float *out, size_t n4) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256;
    float acc = 0.0f;
    for (; i + (U - 1) * stride < n4; i += U * stride) {
        fx4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = STREAMING ? __builtin_nontemporal_load(a + i + u * stride) : a[i + u * stride];
#pragma unroll
        for (int u = 0; u < U; u++) acc += (v[u].x + v[u].y) + (v[u].z + v[u].w);
    }
    for (; i < n4; i += stride) acc += a[i].x;
    if (acc == 1.2345678e-30f) out[0] = acc;  // keeps the loads alive; the buffer holds zeros
}

__global__ __launch_bounds__(256) void hbm_write_kernel(fx4 *__restrict__ a, size_t n4) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256;
    const fx4 v = {0.0f, 0.0f, 0.0f, 0.0f};
    for (; i < n4; i += stride) a[i] = v;
}

template <int U, bool STREAMING>
__global__ __launch_bounds__(256) void hbm_copy_kernel(const fx4 *__restrict__ a, fx4 *__restrict__ b, size_t n4) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256;
    for (; i + (U - 1) * stride < n4; i += U * stride) {
        fx4 v[U];
#pragma unroll
        for (int u = 0; u < U; u++) v[u] = STREAMING ? __builtin_nontemporal_load(a + i + u * stride) : a[i + u * stride];
#pragma unroll
        for (int u = 0; u < U; u++) {
            if (STREAMING) __builtin_nontemporal_store(v[u], b + i + u * stride);
            else b[i + u * stride] = v[u];
        }
    }
    for (; i < n4; i += stride) b[i] = a[i];
}

// Mean duration (ms) of `reps` back-to-back launches after two untimed ones; < 0 on a HIP error.
template <typename Launch>
float stream_ms(hipStream_t st, hipEvent_t e0, hipEvent_t e1, int reps, Launch launch) {
    launch();
    launch();
    if (hipEventRecord(e0, st) != hipSuccess) return -1.0f;
    for (int r = 0; r < reps; r++) launch();
    if (hipEventRecord(e1, st) != hipSuccess || hipEventSynchronize(e1) != hipSuccess) return -1.0f;
    float ms = 0.0f;
    if (hipEventElapsedTime(&ms, e0, e1) != hipSuccess || hipGetLastError() != hipSuccess) return -1.0f;
    return ms / reps;
}

}  // namespace

extern "C" int eddlhip_probe_hbm(int dev, size_t bytes, float *read_gbs, float *write_gbs, float *copy_gbs) {
    EH_REQUIRE(read_gbs && write_gbs && copy_gbs, "probe_hbm: NULL result pointer");
    EH_REQUIRE(bytes >= ((size_t)1 << 26) && bytes <= ((size_t)1 << 33) && bytes % 4096 == 0,
               "probe_hbm: buffer size must be a multiple of 4096 between 64 MiB and 8 GiB");
    EH_TRY(use_device(dev));
    EH_NOT_CAPTURING(dev, "eddlhip_probe_hbm");
    hipStream_t st = state(dev).stream;
    const int cus = state(dev).num_cu;
    const size_t n4 = bytes / 16;
    fx4 *a = nullptr, *b = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int rc = 0;
    if (hipMalloc((void **)&a, bytes) != hipSuccess || hipMalloc((void **)&b, bytes) != hipSuccess) rc = EDDLHIP_ENOMEM;
    if (rc == 0 && (hipMemsetAsync(a, 0, bytes, st) != hipSuccess || hipMemsetAsync(b, 0, bytes, st) != hipSuccess)) rc = EDDLHIP_EHIP;
    if (rc == 0 && (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess)) rc = EDDLHIP_EHIP;
    float *flag = (float *)state(dev).flag;
    double best_r = 0.0, best_w = 0.0, best_c = 0.0;
    const int reps = 5;
    auto keep = [&](double &best, float ms, double moved) {
        if (ms < 0.0f) rc = EDDLHIP_EHIP;
        else if (ms > 0.0f && moved / ms / 1e6 > best) best = moved / ms / 1e6;
    };
    const unsigned whole = (unsigned)((n4 / 4 + 255) / 256);  // one 4-deep trip per thread
    for (int per_cu : {2, 4, 8, 32, 0}) {
        if (rc != 0) break;
        const unsigned grid = per_cu ? (unsigned)(cus * per_cu) : whole;
        keep(best_r, stream_ms(st, e0, e1, reps, [&] { hipLaunchKernelGGL((hbm_read_kernel<4, false>), dim3(grid), dim3(256), 0, st, a, flag, n4); }), (double)bytes);
        keep(best_r, stream_ms(st, e0, e1, reps, [&] { hipLaunchKernelGGL((hbm_read_kernel<4, true>), dim3(grid), dim3(256), 0, st, a, flag, n4); }), (double)bytes);
        keep(best_w, stream_ms(st, e0, e1, reps, [&] { hipLaunchKernelGGL(hbm_write_kernel, dim3(grid), dim3(256), 0, st, b, n4); }), (double)bytes);
        keep(best_c, stream_ms(st, e0, e1, reps, [&] { hipLaunchKernelGGL((hbm_copy_kernel<4, false>), dim3(grid), dim3(256), 0, st, a, b, n4); }), 2.0 * bytes);
        keep(best_c, stream_ms(st, e0, e1, reps, [&] { hipLaunchKernelGGL((hbm_copy_kernel<4, true>), dim3(grid), dim3(256), 0, st, a, b, n4); }), 2.0 * bytes);
    }
    if (rc == 0) {  // one access per thread, workgroups in address order: the shape of the element-wise kernels
        const unsigned flat = (unsigned)((n4 + 255) / 256);
        keep(best_r, stream_ms(st, e0, e1, reps, [&] { hipLaunchKernelGGL((hbm_read_kernel<1, false>), dim3(flat), dim3(256), 0, st, a, flag, n4); }), (double)bytes);
        keep(best_w, stream_ms(st, e0, e1, reps, [&] { hipLaunchKernelGGL(hbm_write_kernel, dim3(flat), dim3(256), 0, st, b, n4); }), (double)bytes);
        keep(best_c, stream_ms(st, e0, e1, reps, [&] { hipLaunchKernelGGL((hbm_copy_kernel<1, false>), dim3(flat), dim3(256), 0, st, a, b, n4); }), 2.0 * bytes);
    }
    (void)hipStreamSynchronize(st);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (a) (void)hipFree(a);
    if (b) (void)hipFree(b);
    if (rc == EDDLHIP_ENOMEM) {
        (void)hipGetLastError();
        return set_error(rc, "probe_hbm: two buffers of %zu bytes do not fit", bytes);
    }
    EH_REQUIRE(rc == 0, "probe_hbm: a HIP call failed: %s", hipGetErrorString(hipGetLastError()));
    *read_gbs = (float)best_r;
    *write_gbs = (float)best_w;
    *copy_gbs = (float)best_c;
    return 0;
}

extern "C" int eddlhip_probe_mfma_f32(int dev, int vary_operands, int launches, float *tflops_mean, float *tflops_best,
                                      float *tflops_worst) {
    EH_REQUIRE(launches >= 1 && launches <= kMaxLaunches, "probe_mfma_f32: launches must be 1..%d", kMaxLaunches);
    EH_REQUIRE(tflops_mean && tflops_best && tflops_worst, "probe_mfma_f32: NULL result pointer");
    EH_TRY(use_device(dev));
    hipStream_t st = state(dev).stream;
    const int blocks = state(dev).num_cu * 2, iters = 4000;
    // operands: a fixed pseudo-random sequence in (-3, 3) (the sums stay far from overflow)
    float host[16 * 256];
    unsigned x = 12345u;
    for (int i = 0; i < 16 * 256; i++) {
        x = x * 1664525u + 1013904223u;
        host[i] = ((x >> 8) * (1.0f / 16777216.0f) - 0.5f) * 6.0f;
    }
    EH_NOT_CAPTURING(dev, "eddlhip_probe_mfma_f32");
    void *ws = nullptr;
    EH_TRY(get_workspace(dev, sizeof(host) + (size_t)blocks * 256 * sizeof(float), &ws));
    float *in = (float *)ws, *out = in + 16 * 256;
    EH_TRY_HIP(hipMemcpyAsync(in, host, sizeof(host), hipMemcpyHostToDevice, st));
    EH_TRY_HIP(hipStreamSynchronize(st));
    // all launches are queued back to back (events between them) and awaited once at the end:
    // a host round trip per launch would give the device pauses that a real workload does not
    static hipEvent_t ev[kMaxLaunches + 1];
    int created = 0, rc = 0;
    for (; created <= launches && rc == 0; created++)
        if (hipEventCreate(&ev[created]) != hipSuccess) rc = -1;
    if (rc != 0) created--;
    const double flops = (double)blocks * 4.0 * iters * 8.0 * 4.0 * 4096.0;
    for (int l = 0; l < 2 && rc == 0; l++)  // two untimed launches first
        hipLaunchKernelGGL(mfma_f32_probe_kernel, dim3(blocks), dim3(256), 0, st, in, out, iters, vary_operands);
    if (rc == 0 && hipEventRecord(ev[0], st) != hipSuccess) rc = -1;
    for (int l = 0; l < launches && rc == 0; l++) {
        hipLaunchKernelGGL(mfma_f32_probe_kernel, dim3(blocks), dim3(256), 0, st, in, out, iters, vary_operands);
        if (hipEventRecord(ev[l + 1], st) != hipSuccess) rc = -1;
    }
    if (rc == 0 && hipEventSynchronize(ev[launches]) != hipSuccess) rc = -1;
    double total_ms = 0.0, best_ms = 1e30, worst_ms = 0.0;
    for (int l = 0; l < launches && rc == 0; l++) {
        float ms = 0.0f;
        if (hipEventElapsedTime(&ms, ev[l], ev[l + 1]) != hipSuccess) rc = -1;
        total_ms += ms;
        if (ms < best_ms) best_ms = ms;
        if (ms > worst_ms) worst_ms = ms;
    }
    for (int i = 0; i < created; i++) (void)hipEventDestroy(ev[i]);
    EH_REQUIRE(rc == 0, "probe_mfma_f32: a HIP call failed: %s", hipGetErrorString(hipGetLastError()));
    *tflops_mean = (float)(flops * launches / total_ms / 1e9);
    *tflops_best = (float)(flops / best_ms / 1e9);
    *tflops_worst = (float)(flops / worst_ms / 1e9);
    return 0;
}

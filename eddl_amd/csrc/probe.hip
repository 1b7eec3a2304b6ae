// Device probe: the rate v_mfma_f32_32x32x2_f32 sustains on this device when nothing else runs.
// The published fp32 matrix peak assumes the top engine clock; under a stream of MFMAs whose
// operands change from instruction to instruction (as a convolution's do) the device lowers its
// clock, and the sustained rate is what a kernel can be measured against.  Not part of the
// reference's interface; the benchmark reports it beside the published peak.
#include "common.h"

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

}  // namespace

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

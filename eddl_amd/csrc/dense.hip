// Dense forward: C[m,n] (+)= A[m,k] * B[k,n], row-major fp32, B = W[in, out]
// (what LDense::forward asks of mult2D: src/layers/core/layer_dense.cpp:65-73).
//
// At the batch sizes of CNN heads (m = 32..64 rows against a 25088 x 4096 weight matrix) the
// product is bound by streaming B from HBM once.  One wavefront owns a 32-row x 32-column
// output block over a slice of k and advances it with v_mfma_f32_32x32x2_f32: the B operand
// of a step is two 128-byte row segments read straight from global memory (coalesced), the A
// operand is two columns of the small activation matrix (L2-resident).  k is split over
// wavefronts so the whole device streams B; the per-slice partial blocks go to the private
// workspace and a second kernel adds them in slice order (fixed summation order, no atomics).
#include "common.h"

using namespace eddlhip;

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

// grid: (n tiles, k slices, m tiles); block: one wavefront
__global__ __launch_bounds__(64) void dense_partial_kernel(const float *__restrict__ A, const float *__restrict__ B,
                                                           float *__restrict__ part, int m, int k, int n, int kslice) {
    const int lane = threadIdx.x;
    const int n0 = blockIdx.x * 32, ks = blockIdx.y, m0 = blockIdx.z * 32;
    const int kbeg = ks * kslice;
    int kend = kbeg + kslice;
    if (kend > k) kend = k;
    const int row = m0 + (lane & 31), col = n0 + (lane & 31), half = lane >> 5;
    const bool rok = row < m, cok = col < n;
    const float *ap = A + (size_t)(rok ? row : 0) * k;
    const float *bp = B + (cok ? col : 0);
    floatx16 acc;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = 0.0f;
    int kk = kbeg;
    for (; kk + 16 <= kend; kk += 16) {
        float a[8], b[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int ki = kk + 2 * u + half;
            a[u] = rok ? ap[ki] : 0.0f;
            b[u] = cok ? bp[(size_t)ki * n] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 8; u++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u], b[u], acc, 0, 0, 0);
    }
    for (; kk < kend; kk += 2) {
        const int ki = kk + half;
        const bool kok = ki < kend;
        float a = (rok && kok) ? ap[ki] : 0.0f;
        float b = (cok && kok) ? bp[(size_t)ki * n] : 0.0f;
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
    }
    // part[ks][row][col]
    if (cok) {
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int r = m0 + 8 * (v / 4) + 4 * half + (v % 4);
            if (r < m) part[((size_t)ks * m + r) * n + col] = acc[v];
        }
    }
}

__global__ __launch_bounds__(256) void dense_reduce_kernel(const float *__restrict__ part, float *C, size_t mn, int nslices,
                                                           int incC) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x, stride = (size_t)gridDim.x * 256;
    for (size_t t = i; t < mn; t += stride) {
        float s = part[t];
        for (int ks = 1; ks < nslices; ks++) s = __fadd_rn(s, part[(size_t)ks * mn + t]);
        C[t] = incC ? __fadd_rn(C[t], s) : s;
    }
}

}  // namespace

extern "C" int eddlhip_mult2d(int dev, const float *A, const float *B, float *C, int m, int k, int n, int incC) {
    EH_REQUIRE(m >= 0 && k > 0 && n > 0, "mult2d: bad shape %dx%d * %dx%d", m, k, k, n);
    if (m == 0) return 0;
    EH_REQUIRE(A && B && C, "mult2d: NULL tensor");
    EH_TRY(use_device(dev));
    hipStream_t st = state(dev).stream;
    const int nt = (n + 31) / 32, mt = (m + 31) / 32;
    // enough wavefronts to cover the device several times over, slices of at least 64 taps
    long long want = 8LL * state(dev).num_cu;
    int nslices = (int)((want + (long long)nt * mt - 1) / ((long long)nt * mt));
    if (nslices < 1) nslices = 1;
    int max_slices = (k + 63) / 64;
    if (nslices > max_slices) nslices = max_slices;
    int kslice = ((k + nslices - 1) / nslices + 1) & ~1;  // even, so MFMA tap pairs do not straddle slices
    nslices = (k + kslice - 1) / kslice;
    EH_REQUIRE(nslices <= 65535 && mt <= 65535, "mult2d: shape out of range");
    void *ws = nullptr;
    EH_TRY(get_workspace(dev, (size_t)nslices * m * n * sizeof(float), &ws));
    hipLaunchKernelGGL(dense_partial_kernel, dim3(nt, nslices, mt), dim3(64), 0, st, A, B, (float *)ws, m, k, n, kslice);
    EH_CHECK_LAUNCH();
    size_t mn = (size_t)m * n;
    hipLaunchKernelGGL(dense_reduce_kernel, dim3(eh_blocks(mn, 256, 65536)), dim3(256), 0, st, (const float *)ws, C, mn, nslices, incC);
    EH_CHECK_LAUNCH();
    return 0;
}

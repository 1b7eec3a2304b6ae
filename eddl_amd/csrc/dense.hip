// Dense forward: C[m,n] (+)= A[m,k] * B[k,n], row-major fp32, B = W[in, out]
// (what LDense::forward asks of mult2D: src/layers/core/layer_dense.cpp:65-73).
//
// At the batch sizes of CNN heads (m = 32..64 rows against a 25088 x 4096 weight matrix) the
// product is bound by streaming B from HBM once.  One wavefront owns a 32-row x 128-column
// output block over a slice of k: per pair of k it loads ONE float4 of B per lane (lane l of a
// half wavefront covers columns 4l..4l+3: 512 contiguous bytes per k row) and one dword of the
// transposed activations, and issues four v_mfma_f32_32x32x2_f32, one per column phase
// (accumulator j holds columns 4l + j).  The activations are transposed first (At[k][32], a few
// MB, L2-resident) so that their loads are coalesced too.  k is split over wavefronts so the
// whole device streams B; the per-slice partial blocks go to the private workspace and a second
// kernel adds them in slice order (fixed summation order, no atomics).
#include <algorithm>

#include "common.h"

using namespace eddlhip;

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// A[m][k] -> At[mt][k][32] (mt = 32-row block), zero-padded rows
__global__ __launch_bounds__(256) void dense_transpose_kernel(const float *__restrict__ A, float *__restrict__ At, int m, int k) {
    __shared__ float tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;
    const int k0 = blockIdx.x * 32, mt = blockIdx.y;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int r = mt * 32 + ty + 8 * j, kk = k0 + tx;
        tile[ty + 8 * j][tx] = (r < m && kk < k) ? A[(size_t)r * k + kk] : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int kk = k0 + ty + 8 * j;
        if (kk < k) At[((size_t)mt * k + kk) * 32 + tx] = tile[tx][ty + 8 * j];
    }
}

// grid: (column tiles of 128, k slices, groups of MT row tiles of 32); block: one wavefront, which multiplies every
// float4 of weights it loads into MT accumulator sets: one pass over B serves MT x 32 rows (a batch of up to 128 rows
// reads the weights once; the activations, transposed, are small and come from L2).
// VEC: n is a multiple of 4 and B is 16-byte aligned, so a lane's four columns are one float4.
// STREAM (with VEC): the weights are read with the streaming (non-temporal) hint - for matrices larger than
// the device's caches, which no later kernel finds there anyway (25088 x 4096: 96 -> 88 us).
template <bool VEC, bool STREAM, int MT>
__global__ __launch_bounds__(64) void dense_partial_kernel(const float *__restrict__ At, const float *__restrict__ B,
                                                           float *__restrict__ part, int m, int k, int n, int kslice) {
    const int lane = threadIdx.x, half = lane >> 5, l = lane & 31;
    const int n0 = blockIdx.x * 128, ks = blockIdx.y, mt0 = blockIdx.z * MT;
    const int kbeg = ks * kslice;
    int kend = kbeg + kslice;
    if (kend > k) kend = k;
    const int col0 = n0 + 4 * l;
    const int mtiles = (m + 31) / 32;
    // row tile mt0 + t of this group, or the last existing one again (its results are not stored)
    const float *ap[MT];
#pragma unroll
    for (int t = 0; t < MT; t++) ap[t] = At + (size_t)(mt0 + t < mtiles ? mt0 + t : mtiles - 1) * k * 32 + l;
    floatx16 acc[MT][4];
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[t][j][v] = 0.0f;
    auto load_b = [&](int ki) -> floatx4 {
        floatx4 b = {0.0f, 0.0f, 0.0f, 0.0f};
        if (ki < kend) {
            const float *row = B + (size_t)ki * n;
            if (VEC) {
                if (col0 < n) b = *reinterpret_cast<const floatx4 *>(row + col0);
            } else {
                if (col0 + 0 < n) b.x = row[col0 + 0];
                if (col0 + 1 < n) b.y = row[col0 + 1];
                if (col0 + 2 < n) b.z = row[col0 + 2];
                if (col0 + 3 < n) b.w = row[col0 + 3];
            }
        }
        return b;
    };
    auto multiply = [&](const float (&a)[MT], const floatx4 &b) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < MT; t++) {
            acc[t][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t], b.x, acc[t][0], 0, 0, 0);
            acc[t][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t], b.y, acc[t][1], 0, 0, 0);
            acc[t][2] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t], b.z, acc[t][2], 0, 0, 0);
            acc[t][3] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t], b.w, acc[t][3], 0, 0, 0);
        }
    };
    constexpr int U = MT == 1 ? 8 : 4;  // k pairs (float4 of weights per lane) in flight
    int kk = kbeg;
    for (; kk + 2 * U <= kend; kk += 2 * U) {
        float a[U][MT];
        floatx4 b[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int ki = kk + 2 * u + half;
#pragma unroll
            for (int t = 0; t < MT; t++) a[u][t] = ap[t][(size_t)ki * 32];
            const float *row = B + (size_t)ki * n;
            if (VEC) {
                const floatx4 *src = reinterpret_cast<const floatx4 *>(row + col0);
                b[u] = col0 < n ? (STREAM ? __builtin_nontemporal_load(src) : *src) : floatx4{0.0f, 0.0f, 0.0f, 0.0f};
            } else {
                b[u] = load_b(ki);
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) multiply(a[u], b[u]);
    }
    for (; kk < kend; kk += 2) {
        const int ki = kk + half;
        float a[MT];
#pragma unroll
        for (int t = 0; t < MT; t++) a[t] = ki < kend ? ap[t][(size_t)ki * 32] : 0.0f;
        multiply(a, load_b(ki));
    }
    // part[ks][row][col]: accumulator j, lane column l -> column col0 + j; rows 8*(v/4) + 4*half + v%4
#pragma unroll
    for (int t = 0; t < MT; t++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int r = (mt0 + t) * 32 + 8 * (v / 4) + 4 * half + (v % 4);
            if (r < m) {
                float *dst = part + ((size_t)ks * m + r) * n + col0;
                if (VEC) {
                    if (col0 < n) *reinterpret_cast<floatx4 *>(dst) = floatx4{acc[t][0][v], acc[t][1][v], acc[t][2][v], acc[t][3][v]};
                } else {
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        if (col0 + j < n) dst[j] = acc[t][j][v];
                }
            }
        }
}

// Adds the K slices in slice order; then, in the reference's order, C += (incC), + bias[column]
// (sum2D_rowwise) and ReLU - each an fp32 operation of its own, so the fused tail equals the
// separate launches bit for bit.
__global__ __launch_bounds__(256) void dense_reduce_kernel(const float *__restrict__ part, float *C, size_t mn, int nslices,
                                                           int incC, const float *__restrict__ bias, int n, int relu) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x, stride = (size_t)gridDim.x * 256;
    for (size_t t = i; t < mn; t += stride) {
        // eight slices' loads in flight at a time; the additions keep the slice order
        float s = part[t];
        int ks = 1;
        for (; ks + 8 <= nslices; ks += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = part[(size_t)(ks + u) * mn + t];
#pragma unroll
            for (int u = 0; u < 8; u++) s = __fadd_rn(s, v[u]);
        }
        for (; ks < nslices; ks++) s = __fadd_rn(s, part[(size_t)ks * mn + t]);
        if (incC) s = __fadd_rn(C[t], s);
        if (bias) s = __fadd_rn(s, bias[t % (size_t)n]);
        if (relu) s = s > 0.0f ? s : 0.0f;
        C[t] = s;
    }
}

}  // namespace

namespace {

int dense_impl(int dev, const float *A, const float *B, float *C, int m, int k, int n, int incC, const float *bias, int relu,
               const char *what) {
    EH_REQUIRE(m >= 0 && k > 0 && n > 0, "%s: bad shape %dx%d * %dx%d", what, m, k, k, n);
    if (m == 0) return 0;
    EH_REQUIRE(A && B && C, "%s: NULL tensor", what);
    EH_TRY(use_device(dev));
    hipStream_t st = state(dev).stream;
    const int nt = (n + 127) / 128, mt = (m + 31) / 32;
    // Wavefronts to cover the device eight times over, in slices of at least 128 taps (shorter
    // slices cost more in partial blocks written and read back than they gain) - unless that
    // leaves fewer than four wavefronts per CU, when slices go down to 64 taps.
    const int MT = mt >= 3 ? 4 : mt;  // row tiles one wavefront serves with each float4 of weights it loads
    const int mgroups = (mt + MT - 1) / MT;
    const long long blocks = (long long)nt * mgroups;
    const long long num_cu = state(dev).num_cu;
    long long nsl = (8 * num_cu + blocks - 1) / blocks;
    const long long max128 = (k + 127) / 128, max64 = (k + 63) / 64;
    if (nsl > max128) nsl = std::max(max128, std::min((4 * num_cu + blocks - 1) / blocks, max64));
    int nslices = (int)std::max(1LL, nsl);
    int kslice = ((k + nslices - 1) / nslices + 1) & ~1;  // even, so MFMA tap pairs do not straddle slices
    nslices = (k + kslice - 1) / kslice;
    EH_REQUIRE(nslices <= 65535 && mgroups <= 65535, "%s: shape out of range", what);
    const size_t at_bytes = ((size_t)mt * k * 32 * sizeof(float) + 255) & ~(size_t)255;
    void *ws = nullptr;
    EH_TRY(get_workspace(dev, at_bytes + (size_t)nslices * m * n * sizeof(float), &ws));
    float *At = (float *)ws, *part = (float *)((char *)ws + at_bytes);
    hipLaunchKernelGGL(dense_transpose_kernel, dim3((k + 31) / 32, mt), dim3(256), 0, st, A, At, m, k);
    EH_CHECK_LAUNCH();
    const bool vec = (n % 4 == 0) && (((uintptr_t)B & 15u) == 0);
    const bool stream = vec && (size_t)k * n * sizeof(float) > ((size_t)256 << 20);  // beyond the 256 MB last-level cache
    typedef void (*partial_fn)(const float *, const float *, float *, int, int, int, int);
    static const partial_fn kernels[3][3] = {
        {dense_partial_kernel<false, false, 1>, dense_partial_kernel<true, false, 1>, dense_partial_kernel<true, true, 1>},
        {dense_partial_kernel<false, false, 2>, dense_partial_kernel<true, false, 2>, dense_partial_kernel<true, true, 2>},
        {dense_partial_kernel<false, false, 4>, dense_partial_kernel<true, false, 4>, dense_partial_kernel<true, true, 4>}};
    const partial_fn kern = kernels[MT == 1 ? 0 : MT == 2 ? 1 : 2][!vec ? 0 : (stream ? 2 : 1)];
    hipLaunchKernelGGL(kern, dim3(nt, nslices, mgroups), dim3(64), 0, st, At, B, part, m, k, n, kslice);
    EH_CHECK_LAUNCH();
    size_t mn = (size_t)m * n;
    hipLaunchKernelGGL(dense_reduce_kernel, dim3(eh_blocks(mn, 256, 65536)), dim3(256), 0, st, (const float *)part, C, mn, nslices, incC,
                       bias, n, relu);
    EH_CHECK_LAUNCH();
    return 0;
}

}  // namespace

extern "C" int eddlhip_mult2d(int dev, const float *A, const float *B, float *C, int m, int k, int n, int incC) {
    return dense_impl(dev, A, B, C, m, k, n, incC, nullptr, 0, "mult2d");
}

extern "C" int eddlhip_dense_fwd(int dev, const float *A, const float *W, const float *bias, float *C, int m, int k, int n, int relu) {
    return dense_impl(dev, A, W, C, m, k, n, 0, bias, relu, "dense_fwd");
}

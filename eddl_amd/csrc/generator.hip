// Random fills and scalar arithmetic that EDDL's parameter initialisers run on the device:
// gpu_rand_uniform / gpu_rand_signed_uniform / gpu_rand_normal / gpu_rand_binary
// (include/eddl/hardware/gpu/gpu_hw.h:58-61, called from src/tensor/tensor_generator.cpp:25-110) and
// gpu_mult(A, B, v) / gpu_add(A, B, v) (gpu_hw.h:89,106; Tensor::mult_ / add_ in the initialisers,
// src/initializers/initializer_glorot_uniform.cpp:35-60, initializer_random_uniform.cpp:35-37).
//
// The value of element i depends on (seed, i) only - Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random
// numbers: as easy as 1, 2, 3", SC'11), key = the 64-bit seed, counter = (i / 4, kind of fill, 0): one block of four
// 32-bit words serves four consecutive elements.  A fill is therefore reproducible whatever the launch shape, and
// two fills with different seeds are independent streams.  The reference draws from cuRAND (MRG32k3a, seed 1234,
// src/hardware/gpu/gpu_tensor.cu:179-185) on the GPU and from std::mt19937 seeded by std::random_device on the CPU
// (src/random.cpp:25-26): its streams cannot be reproduced and are not part of its contract; the distributions are.
//
// Distributions (CPU semantics, src/hardware/cpu/cpu_generator.cpp:14-49, with u = (word >> 8) * 2^-24 in [0, 1)):
//   uniform         A[i] = u * v
//   signed uniform  A[i] = (2u - 1) * v
//   binary          A[i] = u < v ? 1 : 0
//   normal          A[i] = z * s + m,  z standard normal by Box-Muller from two words:
//                   r = sqrt(-2 ln u1), u1 = ((w0 >> 8) + 1) * 2^-24 in (0, 1];  z = r cos(2 pi u2), r sin(2 pi u2).
//                   (The reference's CPU generator leaves out the factor 2 under the root, src/random.cpp:40-48, and so
//                   draws values of standard deviation s / sqrt(2); its GPU path, cuRAND, draws N(m, s^2) as the
//                   function's name says.  This file draws N(m, s^2).)
#include <math.h>

#include "common.h"

using namespace eddlhip;

namespace {

constexpr int TPB = 256;
constexpr unsigned PHILOX_M0 = 0xD2511F53u, PHILOX_M1 = 0xCD9E8D57u;
constexpr unsigned PHILOX_W0 = 0x9E3779B9u, PHILOX_W1 = 0xBB67AE85u;

struct Words4 {
    unsigned x, y, z, w;
};

__device__ __forceinline__ Words4 philox4x32_10(Words4 c, unsigned k0, unsigned k1) {
#pragma unroll
    for (int round = 0; round < 10; round++) {
        const unsigned hi0 = __umulhi(PHILOX_M0, c.x), lo0 = PHILOX_M0 * c.x;
        const unsigned hi1 = __umulhi(PHILOX_M1, c.z), lo1 = PHILOX_M1 * c.z;
        c = Words4{hi1 ^ c.y ^ k0, lo1, hi0 ^ c.w ^ k1, lo0};
        k0 += PHILOX_W0;
        k1 += PHILOX_W1;
    }
    return c;
}

__device__ __forceinline__ float unit_interval(unsigned word) { return (float)(word >> 8) * 0x1p-24f; }

enum Kind { UNIFORM = 0, SIGNED_UNIFORM = 1, BINARY = 2, NORMAL = 3, RAW = 4 };

// Thread t of the grid produces elements 4t .. 4t+3 (grid-stride over blocks of four).
template <int KIND>
__global__ __launch_bounds__(TPB) void rand_fill_kernel(float *A, size_t n, float p0, float p1, unsigned k0, unsigned k1,
                                                        unsigned long long first_block, unsigned c2, unsigned c3) {
    const size_t blocks4 = (n + 3) / 4;
    for (size_t b = (size_t)blockIdx.x * TPB + threadIdx.x; b < blocks4; b += (size_t)gridDim.x * TPB) {
        const unsigned long long ctr = first_block + b;
        const Words4 r = philox4x32_10(Words4{(unsigned)ctr, (unsigned)(ctr >> 32), c2, c3}, k0, k1);
        float v[4];
        if (KIND == NORMAL) {
            const float two_pi = 6.28318530717958647692f;
            const float r0 = sqrtf(-2.0f * logf((float)((r.x >> 8) + 1u) * 0x1p-24f));
            const float r1 = sqrtf(-2.0f * logf((float)((r.z >> 8) + 1u) * 0x1p-24f));
            float s0, c0, s1, c1;
            sincosf(two_pi * unit_interval(r.y), &s0, &c0);
            sincosf(two_pi * unit_interval(r.w), &s1, &c1);
            v[0] = __fadd_rn(__fmul_rn(__fmul_rn(r0, c0), p1), p0);
            v[1] = __fadd_rn(__fmul_rn(__fmul_rn(r0, s0), p1), p0);
            v[2] = __fadd_rn(__fmul_rn(__fmul_rn(r1, c1), p1), p0);
            v[3] = __fadd_rn(__fmul_rn(__fmul_rn(r1, s1), p1), p0);
        } else {
            const unsigned w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float u = unit_interval(w[j]);
                if (KIND == UNIFORM) v[j] = __fmul_rn(u, p0);
                else if (KIND == SIGNED_UNIFORM) v[j] = __fmul_rn(__fsub_rn(__fmul_rn(2.0f, u), 1.0f), p0);
                else if (KIND == BINARY) v[j] = u < p0 ? 1.0f : 0.0f;
                else v[j] = __uint_as_float(w[j]);  // RAW: the generator's words themselves (known-answer tests)
            }
        }
        const size_t i = b * 4;
        if (i + 4 <= n && (((size_t)A & 15) == 0)) {
            *reinterpret_cast<float4 *>(A + i) = make_float4(v[0], v[1], v[2], v[3]);
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (i + j < n) A[i + j] = v[j];
        }
    }
}

// B = A * v (OP 0) or A + v (OP 1); A and B may be the same tensor (Tensor::mult_, Tensor::add_)
template <int OP>
__global__ __launch_bounds__(TPB) void scalar_kernel(const float *A, float *B, size_t n, float v, int vec) {
    const size_t i = (size_t)blockIdx.x * TPB + threadIdx.x, stride = (size_t)gridDim.x * TPB;
    auto f = [v](float a) -> float { return OP == 0 ? __fmul_rn(a, v) : __fadd_rn(a, v); };
    const size_t n4 = vec ? n / 4 : 0;
    for (size_t j = i; j < n4; j += stride) {
        const float4 a = reinterpret_cast<const float4 *>(A)[j];
        reinterpret_cast<float4 *>(B)[j] = make_float4(f(a.x), f(a.y), f(a.z), f(a.w));
    }
    for (size_t j = n4 * 4 + i; j < n; j += stride) B[j] = f(A[j]);
}

template <int KIND>
int rand_fill(int dev, float *A, size_t n, float p0, float p1, unsigned long long seed, const char *what,
              unsigned long long first_block = 0, unsigned long long counter_hi = KIND) {
    if (n == 0) return 0;
    EH_REQUIRE(A != nullptr, "%s: NULL tensor", what);
    EH_TRY(use_device(dev));
    conv_filters_written(dev, A, n * sizeof(float));
    hipLaunchKernelGGL(rand_fill_kernel<KIND>, dim3(eh_blocks((n + 3) / 4, TPB, 65536)), dim3(TPB), 0, state(dev).stream, A, n, p0, p1,
                       (unsigned)(seed & 0xffffffffu), (unsigned)(seed >> 32), first_block, (unsigned)(counter_hi & 0xffffffffu),
                       (unsigned)(counter_hi >> 32));
    EH_CHECK_LAUNCH();
    return 0;
}

template <int OP>
int scalar_op(int dev, const float *A, float *B, size_t n, float v, const char *what) {
    if (n == 0) return 0;
    EH_REQUIRE(A && B, "%s: NULL tensor", what);
    EH_TRY(use_device(dev));
    conv_filters_written(dev, B, n * sizeof(float));
    const int vec = (((size_t)A | (size_t)B) & 15) == 0;
    hipLaunchKernelGGL(scalar_kernel<OP>, dim3(eh_blocks(n / 4 + 1, TPB, 65536)), dim3(TPB), 0, state(dev).stream, A, B, n, v, vec);
    EH_CHECK_LAUNCH();
    return 0;
}

}  // namespace

extern "C" {

int eddlhip_rand_uniform(int dev, float *A, size_t n, float v, unsigned long long seed) {
    return rand_fill<UNIFORM>(dev, A, n, v, 0.0f, seed, "rand_uniform");
}

int eddlhip_rand_signed_uniform(int dev, float *A, size_t n, float v, unsigned long long seed) {
    return rand_fill<SIGNED_UNIFORM>(dev, A, n, v, 0.0f, seed, "rand_signed_uniform");
}

int eddlhip_rand_binary(int dev, float *A, size_t n, float v, unsigned long long seed) {
    return rand_fill<BINARY>(dev, A, n, v, 0.0f, seed, "rand_binary");
}

int eddlhip_rand_normal(int dev, float *A, size_t n, float mean, float stddev, unsigned long long seed) {
    return rand_fill<NORMAL>(dev, A, n, mean, stddev, seed, "rand_normal");
}

int eddlhip_rand_words(int dev, float *A, size_t n, unsigned long long seed, unsigned long long first_block,
                       unsigned long long counter_hi) {
    return rand_fill<RAW>(dev, A, n, 0.0f, 0.0f, seed, "rand_words", first_block, counter_hi);
}

int eddlhip_mult_scalar(int dev, const float *A, float *B, size_t n, float v) { return scalar_op<0>(dev, A, B, n, v, "mult_scalar"); }

int eddlhip_add_scalar(int dev, const float *A, float *B, size_t n, float v) { return scalar_op<1>(dev, A, B, n, v, "add_scalar"); }

}  // extern "C"

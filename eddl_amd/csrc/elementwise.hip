// Bandwidth-bound operators of the CNN forward path: fill, ReLU, sigmoid, softmax,
// inference batch-norm, add/inc, concat, nearest resize, pad.  Each kernel moves every byte
// once, with 16-byte accesses where the shapes allow, and keeps the reference CPU path's
// per-element rounding sequence (this file is compiled with FMA contraction off).
#include <math.h>

#include "common.h"

using namespace eddlhip;

namespace {

constexpr int TPB = 256;
constexpr int kBnFlatBelow = 4096;  // planes shorter than this take the flat batch-norm kernel

__device__ __forceinline__ float relu_f(float x) { return x > 0.0f ? x : 0.0f; }

// ---------------------------------------------------------------- fill / relu / sigmoid / add / inc
__global__ __launch_bounds__(TPB) void fill_kernel(float *__restrict__ A, size_t n, float v, int vec) {
    size_t i = (size_t)blockIdx.x * TPB + threadIdx.x, stride = (size_t)gridDim.x * TPB;
    size_t n4 = vec ? n / 4 : 0;
    float4 v4 = make_float4(v, v, v, v);
    for (size_t j = i; j < n4; j += stride) reinterpret_cast<float4 *>(A)[j] = v4;
    for (size_t j = n4 * 4 + i; j < n; j += stride) A[j] = v;
}

template <int OP>  // 0 relu, 1 sigmoid
__global__ __launch_bounds__(TPB) void unary_kernel(const float *__restrict__ A, float *__restrict__ B, size_t n, int vec) {
    size_t i = (size_t)blockIdx.x * TPB + threadIdx.x, stride = (size_t)gridDim.x * TPB;
    auto f = [](float x) -> float {
        if (OP == 0) return relu_f(x);
        return 1.0f / (1.0f + expf(-x));
    };
    size_t n4 = vec ? n / 4 : 0;
    for (size_t j = i; j < n4; j += stride) {
        float4 a = reinterpret_cast<const float4 *>(A)[j];
        reinterpret_cast<float4 *>(B)[j] = make_float4(f(a.x), f(a.y), f(a.z), f(a.w));
    }
    for (size_t j = n4 * 4 + i; j < n; j += stride) B[j] = f(A[j]);
}

// C (+)= scA*A + scB*B : two products, one sum, (one more sum when accumulating)
__global__ __launch_bounds__(TPB) void add_kernel(float scA, const float *__restrict__ A, float scB,
                                                  const float *__restrict__ B, float *C, int incC, size_t n, int vec) {
    size_t i = (size_t)blockIdx.x * TPB + threadIdx.x, stride = (size_t)gridDim.x * TPB;
    auto f = [&](float a, float b, float c) -> float {
        float s = __fadd_rn(__fmul_rn(scA, a), __fmul_rn(scB, b));
        return incC ? __fadd_rn(c, s) : s;
    };
    size_t n4 = vec ? n / 4 : 0;
    for (size_t j = i; j < n4; j += stride) {
        float4 a = reinterpret_cast<const float4 *>(A)[j];
        float4 b = reinterpret_cast<const float4 *>(B)[j];
        float4 c = make_float4(0, 0, 0, 0);
        if (incC) c = reinterpret_cast<const float4 *>(C)[j];
        reinterpret_cast<float4 *>(C)[j] = make_float4(f(a.x, b.x, c.x), f(a.y, b.y, c.y), f(a.z, b.z, c.z), f(a.w, b.w, c.w));
    }
    for (size_t j = n4 * 4 + i; j < n; j += stride) C[j] = f(A[j], B[j], incC ? C[j] : 0.0f);
}

__global__ __launch_bounds__(TPB) void inc_kernel(const float *__restrict__ A, float *B, size_t n, int vec) {
    size_t i = (size_t)blockIdx.x * TPB + threadIdx.x, stride = (size_t)gridDim.x * TPB;
    size_t n4 = vec ? n / 4 : 0;
    for (size_t j = i; j < n4; j += stride) {
        float4 a = reinterpret_cast<const float4 *>(A)[j];
        float4 b = reinterpret_cast<float4 *>(B)[j];
        reinterpret_cast<float4 *>(B)[j] = make_float4(b.x + a.x, b.y + a.y, b.z + a.z, b.w + a.w);
    }
    for (size_t j = n4 * 4 + i; j < n; j += stride) B[j] = B[j] + A[j];
}

// ---------------------------------------------------------------- batch-norm (inference)
// One (image, channel) plane per blockIdx.y; threads stream the plane.  Rounding sequence
// per element: sub, div, [mul, add].
__global__ __launch_bounds__(TPB) void bn_inference_kernel(int plane0, int z, int rc, const float *__restrict__ in,
                                                           float *__restrict__ out, float *__restrict__ opa,
                                                           const float *__restrict__ gmean, const float *__restrict__ gvar,
                                                           const float *__restrict__ g, const float *__restrict__ bb,
                                                           float *__restrict__ variance, float eps, int vec) {
    const int plane = plane0 + blockIdx.y;  // b*z + c
    const int c = plane % z;
    const float sd = sqrtf(__fadd_rn(gvar[c], eps));
    const float mean = gmean[c];
    const bool affine = g != nullptr;
    const float gg = affine ? g[c] : 1.0f, bc = affine ? bb[c] : 0.0f;
    if (plane < z && blockIdx.x == 0 && threadIdx.x == 0) variance[c] = sd;
    const size_t base = (size_t)plane * rc;
    const int i0 = blockIdx.x * TPB + threadIdx.x, stride = gridDim.x * TPB;
    const int rc4 = vec ? rc / 4 : 0;
    auto norm = [&](float x) -> float { return __fdiv_rn(__fsub_rn(x, mean), sd); };
    auto aff = [&](float o) -> float { return __fadd_rn(__fmul_rn(o, gg), bc); };
    for (int j = i0; j < rc4; j += stride) {
        float4 x = reinterpret_cast<const float4 *>(in + base)[j];
        float4 o = make_float4(norm(x.x), norm(x.y), norm(x.z), norm(x.w));
        if (affine) {
            if (opa) reinterpret_cast<float4 *>(opa + base)[j] = o;
            o = make_float4(aff(o.x), aff(o.y), aff(o.z), aff(o.w));
        }
        reinterpret_cast<float4 *>(out + base)[j] = o;
    }
    for (int j = rc4 * 4 + i0; j < rc; j += stride) {
        float o = norm(in[base + j]);
        if (affine) {
            if (opa) opa[base + j] = o;
            o = aff(o);
        }
        out[base + j] = o;
    }
}

// Small planes (a 7x7 plane would leave most of a workgroup idle above): one float4 of the whole tensor per
// thread, whatever plane it falls into.  A float4 may cross from one plane into the next (planes of at
// least 4 elements: at most one crossing), so the constants of both channels are at hand.  Same operations
// per element as above.  IDX: 32-bit element arithmetic when the tensor allows it.
template <typename IDX>
__global__ __launch_bounds__(TPB) void bn_inference_flat_kernel(IDX total, int z, int rc, const float *__restrict__ in,
                                                                float *__restrict__ out, float *__restrict__ opa,
                                                                const float *__restrict__ gmean, const float *__restrict__ gvar,
                                                                const float *__restrict__ g, const float *__restrict__ bb,
                                                                float *__restrict__ variance, float eps) {
    const bool affine = g != nullptr;
    const IDX n4 = total / 4;
    const IDX i0 = (IDX)blockIdx.x * TPB + threadIdx.x, stride = (IDX)gridDim.x * TPB;
    for (IDX j = i0; j < n4; j += stride) {
        const IDX e0 = j * 4;
        const IDX plane = e0 / (IDX)rc;
        const int r0 = (int)(e0 - plane * (IDX)rc);
        const int c0 = (int)(plane % (IDX)z);
        const bool crosses = r0 + 3 >= rc;  // components from rc - r0 on belong to the next plane
        const int c1 = crosses ? (c0 + 1 == z ? 0 : c0 + 1) : c0;
        const float sd0 = sqrtf(__fadd_rn(gvar[c0], eps)), sd1 = sqrtf(__fadd_rn(gvar[c1], eps));
        const float m0 = gmean[c0], m1 = gmean[c1];
        const float g0 = affine ? g[c0] : 1.0f, g1 = affine ? g[c1] : 1.0f;
        const float b0 = affine ? bb[c0] : 0.0f, b1 = affine ? bb[c1] : 0.0f;
        if (r0 == 0 && plane < (IDX)z) variance[c0] = sd0;
        if (crosses && plane + 1 < (IDX)z) variance[c1] = sd1;
        const float4 x = reinterpret_cast<const float4 *>(in)[j];
        const float xs[4] = {x.x, x.y, x.z, x.w};
        float o[4], y[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const bool first = r0 + k < rc;
            o[k] = __fdiv_rn(__fsub_rn(xs[k], first ? m0 : m1), first ? sd0 : sd1);
            y[k] = affine ? __fadd_rn(__fmul_rn(o[k], first ? g0 : g1), first ? b0 : b1) : o[k];
        }
        if (affine && opa) reinterpret_cast<float4 *>(opa)[j] = make_float4(o[0], o[1], o[2], o[3]);
        reinterpret_cast<float4 *>(out)[j] = make_float4(y[0], y[1], y[2], y[3]);
    }
    for (IDX e = n4 * 4 + i0; e < total; e += stride) {  // the last total % 4 elements
        const IDX plane = e / (IDX)rc;
        const int c = (int)(plane % (IDX)z);
        const float sd = sqrtf(__fadd_rn(gvar[c], eps));
        if (e == plane * (IDX)rc && plane < (IDX)z) variance[c] = sd;
        float o = __fdiv_rn(__fsub_rn(in[e], gmean[c]), sd);
        if (affine) {
            if (opa) opa[e] = o;
            o = __fadd_rn(__fmul_rn(o, g[c]), bb[c]);
        }
        out[e] = o;
    }
}

// ---------------------------------------------------------------- softmax
// One wavefront per sample (a sample = one line along the axis).  max and sum are wavefront
// reductions, so the denominator's summation order differs from a sequential loop (covered
// by the stated floating-point tolerance); it starts from the same 1.19209e-07 seed.
__global__ __launch_bounds__(64) void softmax_kernel(const float *__restrict__ A, float *__restrict__ B, int n_samples,
                                                     int len, int inner, int stable) {
    const int si = blockIdx.x;
    if (si >= n_samples) return;
    const int lane = threadIdx.x;
    const size_t start = (size_t)(si % inner) + (size_t)(si / inner) * ((size_t)len * inner);
    if (len <= 64 * 16) {
        // lines of up to 1024 entries stay in registers: one read, one write, the same operations in the same order
        float v[16];
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const int i = lane + 64 * j;
            v[j] = i < len ? A[start + (size_t)i * inner] : 0.0f;
        }
        float mx = -3.40282e+38f;
        if (stable) {
#pragma unroll
            for (int j = 0; j < 16; j++)
                if (lane + 64 * j < len && v[j] > mx) mx = v[j];
            for (int off = 32; off > 0; off >>= 1) {
                float o = __shfl_xor(mx, off, 64);
                if (o > mx) mx = o;
            }
        }
        float sum = 0.0f;
#pragma unroll
        for (int j = 0; j < 16; j++)
            if (lane + 64 * j < len) {
                v[j] = expf(v[j] - mx);
                sum += v[j];
            }
        for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
        const float den = 1.19209e-07f + sum;
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const int i = lane + 64 * j;
            if (i < len) B[start + (size_t)i * inner] = __fdiv_rn(v[j], den);
        }
        return;
    }
    float mx = -3.40282e+38f;
    if (stable) {
        for (int i = lane; i < len; i += 64) {
            float v = A[start + (size_t)i * inner];
            if (v > mx) mx = v;
        }
        for (int off = 32; off > 0; off >>= 1) {
            float o = __shfl_xor(mx, off, 64);
            if (o > mx) mx = o;
        }
    }
    float sum = 0.0f;
    for (int i = lane; i < len; i += 64) {
        float e = expf(A[start + (size_t)i * inner] - mx);
        B[start + (size_t)i * inner] = e;
        sum += e;
    }
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    const float den = 1.19209e-07f + sum;
    for (int i = lane; i < len; i += 64) {
        size_t p = start + (size_t)i * inner;
        B[p] = __fdiv_rn(B[p], den);
    }
}

// ---------------------------------------------------------------- concat
// Copies one input into its slot of the destination.  Element j of the source goes to
// (j / src_stride) * steps + j % src_stride + offset.  With vec, all of src_stride, steps and
// offset are multiples of 4 and whole float4 groups move.
__global__ __launch_bounds__(TPB) void concat_kernel(float *__restrict__ dest, const float *__restrict__ src, size_t size,
                                                     size_t src_stride, size_t steps, int vec) {
    size_t i = (size_t)blockIdx.x * TPB + threadIdx.x, stride = (size_t)gridDim.x * TPB;
    if (vec) {
        size_t n4 = size / 4, ss4 = src_stride / 4, st4 = steps / 4;
        for (size_t j = i; j < n4; j += stride) {
            size_t blk = j / ss4, k = j - blk * ss4;
            reinterpret_cast<float4 *>(dest)[blk * st4 + k] = reinterpret_cast<const float4 *>(src)[j];
        }
    } else {
        for (size_t j = i; j < size; j += stride) {
            size_t blk = j / src_stride, k = j - blk * src_stride;
            dest[blk * steps + k] = src[j];
        }
    }
}

// ---------------------------------------------------------------- nearest resize (asymmetric)
// One thread per TWO horizontally adjacent destination elements (float2 store when aligned).
__global__ __launch_bounds__(TPB) void scale_nearest_kernel(const float *__restrict__ A, float *__restrict__ B, int planes,
                                                            int H, int W, int OH, int OW, float scale_y, float scale_x,
                                                            int off0, int off1) {
    const int OW2 = (OW + 1) / 2;
    size_t total = (size_t)planes * OH * OW2;
    size_t i = (size_t)blockIdx.x * TPB + threadIdx.x, stride = (size_t)gridDim.x * TPB;
    for (size_t t = i; t < total; t += stride) {
        int bj2 = (int)(t % OW2);
        size_t r = t / OW2;
        int bi = (int)(r % OH);
        size_t plane = r / OH;
        int ai = (int)__fdiv_rn((float)(bi + off0), scale_y);
        const float *src = A + plane * H * W;
        float *dst = B + (plane * OH + bi) * OW;
        int bj = bj2 * 2;
        int aj0 = (int)__fdiv_rn((float)(bj + off1), scale_x);
        int aj1 = (int)__fdiv_rn((float)(bj + 1 + off1), scale_x);
        bool rowok = ai >= 0 && ai < H;
        bool ok0 = rowok && aj0 >= 0 && aj0 < W;
        bool ok1 = rowok && (bj + 1 < OW) && aj1 >= 0 && aj1 < W;
        if (ok0) dst[bj] = src[(size_t)ai * W + aj0];
        if (ok1) dst[bj + 1] = src[(size_t)ai * W + aj1];
    }
}

// Exact doubling (source row = destination row / 2, same for columns; even W, aligned rows): a
// thread reads two neighbouring source pixels and writes them as one float4 into each of the two
// destination rows they cover.
__global__ __launch_bounds__(TPB) void scale_double_kernel(const float *__restrict__ A, float *__restrict__ B, size_t total_pairs,
                                                           int H, int W2) {
    size_t i = (size_t)blockIdx.x * TPB + threadIdx.x, stride = (size_t)gridDim.x * TPB;
    for (size_t t = i; t < total_pairs; t += stride) {
        const int j2 = (int)(t % W2);
        const size_t row = t / W2;  // plane * H + source row
        const float2 v = *reinterpret_cast<const float2 *>(A + row * (size_t)(2 * W2) + 2 * j2);
        const float4 o = make_float4(v.x, v.x, v.y, v.y);
        float *dst = B + (row * 2) * (size_t)(4 * W2) + 4 * j2;  // destination rows 2*row' and 2*row'+1 of the same plane
        *reinterpret_cast<float4 *>(dst) = o;
        *reinterpret_cast<float4 *>(dst + 4 * W2) = o;
    }
}

// ---------------------------------------------------------------- pad (interior copy)
__global__ __launch_bounds__(TPB) void pad_kernel(const float *__restrict__ A, float *__restrict__ B, size_t total, int H,
                                                  int W, int OH, int OW, int top, int left) {
    size_t i = (size_t)blockIdx.x * TPB + threadIdx.x, stride = (size_t)gridDim.x * TPB;
    for (size_t t = i; t < total; t += stride) {
        int w = (int)(t % W);
        size_t r = t / W;
        int h = (int)(r % H);
        size_t plane = r / H;
        B[(plane * OH + (h + top)) * OW + (w + left)] = A[t];
    }
}

// Rows of at least 64 pixels: one wavefront per source row, lanes on consecutive pixels (256 contiguous
// bytes per load and per store, whatever the destination row's alignment), four loads in flight per
// lane, and one division per row instead of three per pixel.
__global__ __launch_bounds__(TPB) void pad_rows_kernel(const float *__restrict__ A, float *__restrict__ B, size_t rows, int H,
                                                       int W, int OH, int OW, int top, int left) {
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    constexpr int WAVES = TPB / 64;
    for (size_t r = (size_t)blockIdx.x * WAVES + wv; r < rows; r += (size_t)gridDim.x * WAVES) {
        const size_t plane = r / H;
        const int h = (int)(r - plane * H);
        const float *src = A + r * W;
        float *dst = B + (plane * OH + (h + top)) * OW + left;
        int j = lane;
        for (; j + 192 < W; j += 256) {
            const float v0 = src[j], v1 = src[j + 64], v2 = src[j + 128], v3 = src[j + 192];
            dst[j] = v0;
            dst[j + 64] = v1;
            dst[j + 128] = v2;
            dst[j + 192] = v3;
        }
        for (; j < W; j += 64) dst[j] = src[j];
    }
}

__global__ __launch_bounds__(TPB) void sum2d_rowwise_kernel(const float *A, const float *__restrict__ B, float *C,
                                                            size_t total, int cols) {
    size_t i = (size_t)blockIdx.x * TPB + threadIdx.x, stride = (size_t)gridDim.x * TPB;
    for (size_t t = i; t < total; t += stride) C[t] = __fadd_rn(A[t], B[t % cols]);
}

inline bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

}  // namespace

extern "C" {

int eddlhip_fill(int dev, float *A, size_t n, float v) {
    if (n == 0) return 0;
    EH_REQUIRE(A != nullptr, "fill: NULL tensor");
    EH_TRY(use_device(dev));
    conv_filters_written(dev, A, n * sizeof(float));
    hipLaunchKernelGGL(fill_kernel, dim3(eh_blocks(n / 4 + 1, TPB, 65536)), dim3(TPB), 0, state(dev).stream, A, n, v,
                       (int)aligned16(A));
    EH_CHECK_LAUNCH();
    return 0;
}

int eddlhip_relu(int dev, const float *A, float *B, size_t n) {
    if (n == 0) return 0;
    EH_REQUIRE(A && B, "relu: NULL tensor");
    EH_TRY(use_device(dev));
    int vec = aligned16(A) && aligned16(B);
    hipLaunchKernelGGL(unary_kernel<0>, dim3(eh_blocks(n / 4 + 1, TPB, 65536)), dim3(TPB), 0, state(dev).stream, A, B, n, vec);
    EH_CHECK_LAUNCH();
    return 0;
}

int eddlhip_sigmoid(int dev, const float *A, float *B, size_t n) {
    if (n == 0) return 0;
    EH_REQUIRE(A && B, "sigmoid: NULL tensor");
    EH_TRY(use_device(dev));
    int vec = aligned16(A) && aligned16(B);
    hipLaunchKernelGGL(unary_kernel<1>, dim3(eh_blocks(n / 4 + 1, TPB, 65536)), dim3(TPB), 0, state(dev).stream, A, B, n, vec);
    EH_CHECK_LAUNCH();
    return 0;
}

int eddlhip_softmax(int dev, const float *A, float *B, int outer, int len, int inner, int stable) {
    EH_REQUIRE(outer >= 0 && len > 0 && inner > 0, "softmax: bad shape outer=%d len=%d inner=%d", outer, len, inner);
    if (outer == 0) return 0;
    EH_REQUIRE(A && B, "softmax: NULL tensor");
    EH_REQUIRE((long long)outer * inner <= 0x7fffffffLL, "softmax: too many samples");
    EH_TRY(use_device(dev));
    int n_samples = outer * inner;
    hipLaunchKernelGGL(softmax_kernel, dim3(n_samples), dim3(64), 0, state(dev).stream, A, B, n_samples, len, inner, stable);
    EH_CHECK_LAUNCH();
    return 0;
}

int eddlhip_batchnorm_inference(int dev, int b, int z, int rc, const float *input, float *output, float *opa,
                                const float *global_mean, const float *global_variance, const float *affine_g,
                                const float *affine_b, float *variance, float epsilon) {
    EH_REQUIRE(b >= 0 && z > 0 && rc > 0, "batchnorm: bad shape b=%d z=%d rc=%d", b, z, rc);
    EH_REQUIRE(global_mean && global_variance && variance, "batchnorm: NULL statistics");
    EH_REQUIRE((affine_g == nullptr) == (affine_b == nullptr), "batchnorm: affine_g and affine_b must come together");
    if (b == 0) return 0;
    EH_REQUIRE(input && output, "batchnorm: NULL tensor");
    EH_REQUIRE((long long)b * z <= 0x7fffffffLL, "batchnorm: too many planes");
    EH_TRY(use_device(dev));
    const bool all_aligned = aligned16(input) && aligned16(output) && (!opa || aligned16(opa));
    long long planes = (long long)b * z;
    if (rc >= 4 && rc < kBnFlatBelow && all_aligned) {
        const size_t total = (size_t)planes * rc;
        const unsigned grid = eh_blocks(total / 4 + 1, TPB, 1u << 20);
        if (total < 0x7fffffffULL)
            hipLaunchKernelGGL(bn_inference_flat_kernel<unsigned>, dim3(grid), dim3(TPB), 0, state(dev).stream, (unsigned)total, z, rc,
                               input, output, opa, global_mean, global_variance, affine_g, affine_b, variance, epsilon);
        else
            hipLaunchKernelGGL(bn_inference_flat_kernel<size_t>, dim3(grid), dim3(TPB), 0, state(dev).stream, total, z, rc, input,
                               output, opa, global_mean, global_variance, affine_g, affine_b, variance, epsilon);
        EH_CHECK_LAUNCH();
        return 0;
    }
    int vec = (rc % 4 == 0) && all_aligned;
    // grid.y is limited to 65535: fold the rest into a loop of launches
    int gx = (int)eh_blocks((size_t)rc / 4 + 1, TPB, 64);
    for (long long p0 = 0; p0 < planes; p0 += 65535) {
        long long cnt = planes - p0;
        if (cnt > 65535) cnt = 65535;
        hipLaunchKernelGGL(bn_inference_kernel, dim3(gx, (unsigned)cnt), dim3(TPB), 0, state(dev).stream, (int)p0, z, rc, input,
                           output, opa, global_mean, global_variance, affine_g, affine_b, variance, epsilon, vec);
        EH_CHECK_LAUNCH();
    }
    return 0;
}

int eddlhip_add(int dev, float scA, const float *A, float scB, const float *B, float *C, int incC, size_t n) {
    if (n == 0) return 0;
    EH_REQUIRE(A && B && C, "add: NULL tensor");
    EH_TRY(use_device(dev));
    conv_filters_written(dev, C, n * sizeof(float));
    int vec = aligned16(A) && aligned16(B) && aligned16(C);
    hipLaunchKernelGGL(add_kernel, dim3(eh_blocks(n / 4 + 1, TPB, 65536)), dim3(TPB), 0, state(dev).stream, scA, A, scB, B, C,
                       incC, n, vec);
    EH_CHECK_LAUNCH();
    return 0;
}

int eddlhip_inc(int dev, const float *A, float *B, size_t n) {
    if (n == 0) return 0;
    EH_REQUIRE(A && B, "inc: NULL tensor");
    EH_TRY(use_device(dev));
    conv_filters_written(dev, B, n * sizeof(float));
    int vec = aligned16(A) && aligned16(B);
    hipLaunchKernelGGL(inc_kernel, dim3(eh_blocks(n / 4 + 1, TPB, 65536)), dim3(TPB), 0, state(dev).stream, A, B, n, vec);
    EH_CHECK_LAUNCH();
    return 0;
}

int eddlhip_concat(int dev, float *dest, const float *const *host_srcs, const int *host_axis_extent, int n_in, int outer,
                   int inner) {
    EH_REQUIRE(n_in >= 1 && host_srcs && host_axis_extent, "concat: no inputs");
    EH_REQUIRE(outer >= 0 && inner > 0, "concat: bad shape outer=%d inner=%d", outer, inner);
    EH_TRY(use_device(dev));
    size_t steps = 0;
    for (int i = 0; i < n_in; i++) {
        EH_REQUIRE(host_axis_extent[i] >= 0, "concat: negative extent");
        steps += (size_t)host_axis_extent[i] * inner;
    }
    if (outer == 0 || steps == 0) return 0;
    EH_REQUIRE(dest != nullptr, "concat: NULL destination");
    size_t offset = 0;
    for (int i = 0; i < n_in; i++) {
        size_t src_stride = (size_t)host_axis_extent[i] * inner;
        size_t size = src_stride * outer;
        if (size) {
            EH_REQUIRE(host_srcs[i] != nullptr, "concat: NULL input %d", i);
            int vec = (src_stride % 4 == 0) && (steps % 4 == 0) && (offset % 4 == 0) && aligned16(dest) && aligned16(host_srcs[i]);
            hipLaunchKernelGGL(concat_kernel, dim3(eh_blocks(size / (vec ? 4 : 1), TPB, 65536)), dim3(TPB), 0, state(dev).stream,
                               dest + offset, host_srcs[i], size, src_stride, steps, vec);
            EH_CHECK_LAUNCH();
        }
        offset += src_stride;
    }
    return 0;
}

int eddlhip_scale_nearest(int dev, const float *A, float *B, int N, int C, int H, int W, int OH, int OW, int newH, int newW) {
    EH_REQUIRE(N >= 0 && C > 0 && H > 0 && W > 0 && OH > 0 && OW > 0, "scale: bad shape");
    EH_REQUIRE(newH > 0 && newW > 0, "scale: the new shape must be greater than zero");
    if (N == 0) return 0;
    EH_REQUIRE(A && B, "scale: NULL tensor");
    const int off0 = (int)((newH - OH) / 2.0f), off1 = (int)((newW - OW) / 2.0f);
    const float scale_y = (float)newH / (float)H, scale_x = (float)newW / (float)W;
    // The mapping is separable: validate it on the host with the same IEEE arithmetic the
    // kernel uses.  Nearest wrapping has no rule for a source outside the image.
    bool doubling = OH == 2 * H && OW == 2 * W;  // stays true when the mapping is row/2, column/2 throughout
    for (int bi = 0; bi < OH; bi++) {
        int ai = (int)((float)(bi + off0) / scale_y);
        EH_REQUIRE(ai >= 0 && ai < H, "scale: destination row %d maps outside the source (nearest wrapping)", bi);
        doubling = doubling && ai == bi / 2;
    }
    for (int bj = 0; bj < OW; bj++) {
        int aj = (int)((float)(bj + off1) / scale_x);
        EH_REQUIRE(aj >= 0 && aj < W, "scale: destination column %d maps outside the source (nearest wrapping)", bj);
        doubling = doubling && aj == bj / 2;
    }
    EH_TRY(use_device(dev));
    if (doubling && W % 2 == 0 && ((uintptr_t)A & 7u) == 0 && ((uintptr_t)B & 15u) == 0) {
        // plane * H + row is one running index because every plane has H rows; destination row pairs likewise
        size_t pairs = (size_t)N * C * H * (W / 2);
        hipLaunchKernelGGL(scale_double_kernel, dim3(eh_blocks(pairs, TPB, 1u << 18)), dim3(TPB), 0, state(dev).stream, A, B, pairs, H,
                           W / 2);
        EH_CHECK_LAUNCH();
        return 0;
    }
    size_t total = (size_t)N * C * OH * ((OW + 1) / 2);
    hipLaunchKernelGGL(scale_nearest_kernel, dim3(eh_blocks(total, TPB, 1u << 18)), dim3(TPB), 0, state(dev).stream, A, B, N * C, H,
                       W, OH, OW, scale_y, scale_x, off0, off1);
    EH_CHECK_LAUNCH();
    return 0;
}

int eddlhip_pad(int dev, const float *A, float *B, int N, int C, int H, int W, int top, int right, int bottom, int left) {
    EH_REQUIRE(N >= 0 && C > 0 && H > 0 && W > 0, "pad: bad shape");
    EH_REQUIRE(top >= 0 && right >= 0 && bottom >= 0 && left >= 0, "pad: margins must be greater or equal than zero");
    if (N == 0) return 0;
    EH_REQUIRE(A && B, "pad: NULL tensor");
    EH_TRY(use_device(dev));
    size_t total = (size_t)N * C * H * W;
    if (W >= 64) {
        size_t rows = (size_t)N * C * H;
        hipLaunchKernelGGL(pad_rows_kernel, dim3(eh_blocks(rows, TPB / 64, 1u << 16)), dim3(TPB), 0, state(dev).stream, A, B, rows,
                           H, W, H + top + bottom, W + left + right, top, left);
    } else {
        hipLaunchKernelGGL(pad_kernel, dim3(eh_blocks(total, TPB, 1u << 18)), dim3(TPB), 0, state(dev).stream, A, B, total, H, W,
                           H + top + bottom, W + left + right, top, left);
    }
    EH_CHECK_LAUNCH();
    return 0;
}

int eddlhip_sum2d_rowwise(int dev, const float *A, const float *B, float *C, int rows, int cols) {
    EH_REQUIRE(rows >= 0 && cols > 0, "sum2d_rowwise: bad shape");
    if (rows == 0) return 0;
    EH_REQUIRE(A && B && C, "sum2d_rowwise: NULL tensor");
    EH_TRY(use_device(dev));
    size_t total = (size_t)rows * cols;
    hipLaunchKernelGGL(sum2d_rowwise_kernel, dim3(eh_blocks(total, TPB, 65536)), dim3(TPB), 0, state(dev).stream, A, B, C, total,
                       cols);
    EH_CHECK_LAUNCH();
    return 0;
}

}  // extern "C"

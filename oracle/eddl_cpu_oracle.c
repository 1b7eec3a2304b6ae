/*
 * CPU oracle for the CNN forward path of EDDL (deephealthproject/eddl v1.1).
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain C, the algorithm of the
 * reference's CPU backend for the operators on the CNN forward path.  It is the
 * checker the HIP kernels are compared against and the timed CPU baseline; nothing
 * in the shipped library links, loads or calls it.
 *
 * Build: -O2 -ffp-contract=off (no -ffast-math, no FMA contraction), so every
 * floating-point expression below is evaluated with the rounding steps written.
 *
 * Every function cites the reference file:line it follows (paths relative to the
 * reference tree).  What pins each function (reference-held vectors, closed forms,
 * library cross-checks) is listed next to it; a function that nothing pins says
 * "parity unpinned".
 *
 * Pin summary
 *   geometry             reference table tests/layers/conv/test_convol_sizes.cpp:18-30
 *   conv2d (direct)      reference vectors tests/layers/conv/test_conv2d.cpp:9-393,
 *                        torch conv2d cross-check, brute force
 *   conv2d (im2col+gemm) checked against conv2d direct
 *   maxpool (+argmax)    reference vectors tests/layers/pool/test_mpool.cpp:9-272 (forward
 *                        values; backward maps pin the argmax), torch max_pool2d
 *   avgpool              reference vectors tests/layers/pool/test_avgpool.cpp:8-277,
 *                        torch avg_pool2d(count_include_pad=True)
 *   pad                  reference vector tests/tensor/test_tensor_da.cpp:19-31 (symmetric);
 *                        (top,right,bottom,left) order is from source reading only
 *   softmax              reference vector tests/tensor/nn/test_tensor_nn.cpp:17-24 (1e-3; the
 *                        1.19209e-07 denominator seed is from source reading only)
 *   batchnorm inference  no reference vectors exist; closed form + torch batch_norm
 *                        cross-check + identity invariants.  The per-element rounding
 *                        sequence (sub, div, mul, add) is from source reading only.
 *   relu/add/concat/
 *   upsample/sigmoid     closed forms, torch cross-checks
 *   dense (mult2D)       no vector in the reference's tests; a textbook matrix product, pinned
 *                        by library routines: numpy float64 matmul, and PyTorch's Linear
 *                        through networks exported to ONNX with PyTorch's own outputs
 *   whole graphs         three PyTorch-exported networks (conv, batch norm, pools, upsample,
 *                        pad, concat, add, dense, softmax, sigmoid) reproduce PyTorch's outputs
 */
#include <math.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* include/eddl/tensor/tensor.h:57-58, include/eddl/hardware/cpu/nn/cpu_tensor_nn.h:20 */
#define ORACLE_LOWEST_FLOAT (-3.40282e+38f)
#define ORACLE_EPS_FLOAT (1.19209e-07f)
#define ORACLE_MIN_FLOAT (-3.402823466e+38F) /* -FLT_MAX */

int eddl_oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

static int g_inner_parallel = 0;
void eddl_oracle_set_inner_parallel(int on) { g_inner_parallel = on; }

void eddl_oracle_set_num_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

/* ------------------------------------------------------------------ geometry */

/* src/descriptors/descriptor_conv2D.cpp:295-307 (named padding; same code in
 * descriptor_pool2D.cpp:162-174).  same=1 for "same"/"zeros", 0 for "valid"/"none". */
int eddl_oracle_out_size_named(int same, int input_size, int kernel_size, int stride, int dilation) {
    if (same) return (int)ceilf((float)input_size / (float)stride);
    return (int)ceilf(((float)input_size - ((float)kernel_size - 1.0f) * (float)dilation) / (float)stride);
}

/* src/descriptors/descriptor_conv2D.cpp:325-327 (custom pads, float arithmetic then truncation) */
int eddl_oracle_out_size_custom(int pad0, int pad1, int input_size, int kernel_size, int stride, int dilation) {
    return (int)(((float)input_size - ((float)kernel_size - 1.0f) * (float)dilation + (float)pad0 + (float)pad1 - 1.0f) /
                     (float)stride +
                 1.0f);
}

/* src/descriptors/descriptor_conv2D.cpp:329-360 ("same" total pad, low half first).
 * The pooling variant (descriptor_pool2D.cpp:180-211) is the dilation=1 case. */
void eddl_oracle_same_pads(int output_size, int input_size, int kernel_size, int stride, int dilation, int *lo, int *hi) {
    int pad = (output_size - 1) * stride + kernel_size - input_size + (dilation - 1) * (kernel_size - 1);
    if (pad < 0) pad = 0;
    *lo = pad / 2;
    *hi = pad - pad / 2;
}

/* Number of window origins the pooling loops visit along one axis:
 * for (i = -pad_lo; i <= in + pad_hi - k; i += stride)  (src/hardware/cpu/nn/cpu_pool.cpp:89-90,
 * replayed by src/descriptors/descriptor_pool2D.cpp:113-117). */
int eddl_oracle_pool_loop_count(int in, int k, int stride, int pad_lo, int pad_hi) {
    int n = 0;
    for (int i = -pad_lo; i <= in + pad_hi - k; i += stride) n++;
    return n;
}

/* ------------------------------------------------------------------ conv2d */

/* Direct convolution in the reference's only fully order-defined form:
 * src/hardware/cpu/nn/cpu_conv.cpp:282-314 (cpu_low_mem_conv3D with depth 1):
 * one fp32 accumulator per output; for ky, for kx (out-of-bounds taps skipped), for c.
 * Cross-correlation (no kernel flip), NCHW input, OIHW filters.  Uses top/left pad only.
 * Bias is a separate pass over the finished output (cpu_conv.cpp:335-346). */
void eddl_oracle_conv2d_direct(const float *I, const float *K, const float *bias, float *O, int N, int C, int H, int W,
                               int Kf, int R, int S, int sr, int sc, int pt, int pl, int P, int Q) {
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < N; b++)
        for (int nk = 0; nk < Kf; nk++)
            for (int i = 0; i < P; i++)
                for (int j = 0; j < Q; j++) {
                    float s = 0;
                    for (int x = 0; x < R; x++) {
                        int px = i * sr + x - pt;
                        if (px >= 0 && px < H)
                            for (int y = 0; y < S; y++) {
                                int py = j * sc + y - pl;
                                if (py >= 0 && py < W) {
                                    for (int c = 0; c < C; c++)
                                        s += K[(((size_t)nk * C + c) * R + x) * S + y] *
                                             I[(((size_t)b * C + c) * H + px) * W + py];
                                }
                            }
                    }
                    O[(((size_t)b * Kf + nk) * P + i) * Q + j] = s;
                }
    if (bias) {
#pragma omp parallel for schedule(static)
        for (int b = 0; b < N; b++) {
            float *ptrO = O + (size_t)b * Kf * P * Q;
            for (int z = 0; z < Kf; z++)
                for (int rc = 0; rc < P * Q; rc++, ptrO++) (*ptrO) += bias[z];
        }
    }
}

/* Same arithmetic as eddl_oracle_conv2d_direct (bias included) at a list of output
 * coordinates only; idx holds npts quadruples (b, k, p, q).  Lets full-size layers be
 * spot-checked without computing every output on the CPU. */
void eddl_oracle_conv2d_direct_at(const float *I, const float *K, const float *bias, float *out, const int *idx,
                                  int npts, int N, int C, int H, int W, int Kf, int R, int S, int sr, int sc, int pt,
                                  int pl) {
    (void)N;
    (void)Kf;
#pragma omp parallel for schedule(static)
    for (int t = 0; t < npts; t++) {
        int b = idx[4 * t], nk = idx[4 * t + 1], i = idx[4 * t + 2], j = idx[4 * t + 3];
        float s = 0;
        for (int x = 0; x < R; x++) {
            int px = i * sr + x - pt;
            if (px >= 0 && px < H)
                for (int y = 0; y < S; y++) {
                    int py = j * sc + y - pl;
                    if (py >= 0 && py < W)
                        for (int c = 0; c < C; c++)
                            s += K[(((size_t)nk * C + c) * R + x) * S + y] * I[(((size_t)b * C + c) * H + px) * W + py];
                }
        }
        if (bias) s += bias[nk];
        out[t] = s;
    }
}

/* Lowering of one image, src/hardware/cpu/nn/cpu_conv.cpp:55-112 (im2col) with
 * get_pixel :25-40: row j of the lowered matrix is output pixel j (row-major over P x Q),
 * column i is tap (c = i/(R*S), ky = (i%(R*S))/S, kx = i%S); stored column-major
 * (element (j,i) at j + i*P*Q); out-of-bounds taps read 0. */
static void oracle_im2col(const float *img, float *col, int C, int H, int W, int R, int S, int sr, int sc, int pt,
                          int pl, int P, int Q, int inner) {
    const int PQ = P * Q, CRS = C * R * S, RS = R * S;
#pragma omp parallel for schedule(static) num_threads(inner) if (inner > 1)
    for (int i = 0; i < CRS; i++) {
        int pz = i / RS, ky = (i % RS) / S, kx = i % S;
        float *dst = col + (size_t)i * PQ;
        const float *src = img + (size_t)pz * H * W;
        for (int p = 0; p < P; p++) {
            int y = -pt + p * sr + ky;
            if (y < 0 || y >= H) {
                for (int q = 0; q < Q; q++) dst[p * Q + q] = 0.0f;
                continue;
            }
            for (int q = 0; q < Q; q++) {
                int x = -pl + q * sc + kx;
                dst[p * Q + q] = (x < 0 || x >= W) ? 0.0f : src[(size_t)y * W + x];
            }
        }
    }
}

/* Single-threaded fp32 GEMM  Out[PQ x Kf] = Col[PQ x CRS] * Wt[CRS x Kf], all three
 * column-major, which is what the Eigen maps of cpu_conv.cpp:210,218-223 describe
 * (Wt(i,k) = K[k][i] over OIHW memory; Out(p,k) = O[b][k][p] in NCHW).
 * The reference's product is Eigen 3.4.0's GEBP kernel (not vendored, absent here): its
 * blocked summation order is Eigen-internal.  This routine sums the CRS products of one
 * output strictly in increasing tap index i, one fp32 accumulator per output.
 * `inner` > 1 spreads the blocks of output pixels over that many more threads: every output is still summed by one
 * thread in the same order, so the result does not depend on it. */
static void oracle_sgemm_colmajor(const float *col, const float *Kw, float *out, int PQ, int CRS, int Kf, int inner) {
    enum { KB = 4, PB = 256 };
#pragma omp parallel for schedule(dynamic, 1) num_threads(inner) if (inner > 1)
    for (int p0 = 0; p0 < PQ; p0 += PB) {
        int pn = PQ - p0 < PB ? PQ - p0 : PB;
        int k = 0;
        for (; k + KB <= Kf; k += KB) {
            float acc[KB][PB];
            for (int kk = 0; kk < KB; kk++)
                for (int p = 0; p < pn; p++) acc[kk][p] = 0.0f;
            for (int i = 0; i < CRS; i++) {
                const float *c = col + (size_t)i * PQ + p0;
                float w0 = Kw[(size_t)(k + 0) * CRS + i], w1 = Kw[(size_t)(k + 1) * CRS + i];
                float w2 = Kw[(size_t)(k + 2) * CRS + i], w3 = Kw[(size_t)(k + 3) * CRS + i];
                for (int p = 0; p < pn; p++) {
                    float v = c[p];
                    acc[0][p] += v * w0;
                    acc[1][p] += v * w1;
                    acc[2][p] += v * w2;
                    acc[3][p] += v * w3;
                }
            }
            for (int kk = 0; kk < KB; kk++) memcpy(out + (size_t)(k + kk) * PQ + p0, acc[kk], sizeof(float) * pn);
        }
        for (; k < Kf; k++) {
            float acc[PB];
            for (int p = 0; p < pn; p++) acc[p] = 0.0f;
            for (int i = 0; i < CRS; i++) {
                const float *c = col + (size_t)i * PQ + p0;
                float w = Kw[(size_t)k * CRS + i];
                for (int p = 0; p < pn; p++) acc[p] += c[p] * w;
            }
            memcpy(out + (size_t)k * PQ + p0, acc, sizeof(float) * pn);
        }
    }
}

/* The reference's default CPU convolution, src/hardware/cpu/nn/cpu_conv.cpp:114-226 and
 * :316-346: "#pragma omp parallel for" over the batch; per image one im2col and one
 * single-threaded GEMM; bias added afterwards in a separate pass.  The reference keeps
 * one lowering buffer per image (descriptor_conv2D.cpp:170-177); this restatement keeps
 * one per thread.  Returns 0, or -1 if the scratch cannot be allocated. */
int eddl_oracle_conv2d_im2col(const float *I, const float *K, const float *bias, float *O, int N, int C, int H, int W,
                              int Kf, int R, int S, int sr, int sc, int pt, int pl, int P, int Q) {
    const size_t PQ = (size_t)P * Q, CRS = (size_t)C * R * S;
    int nthreads = eddl_oracle_num_threads();
    /* The reference runs one thread per image.  With eddl_oracle_set_inner_parallel(1) (checking runs on batches
     * smaller than the machine, never the timed baseline) the threads left over also share each image's lowering
     * and product, which changes no result. */
    int inner = 1;
    if (g_inner_parallel && N > 0 && nthreads > N) inner = nthreads / N;
    if (nthreads > N) nthreads = N;
    if (nthreads < 1) nthreads = 1;
#ifdef _OPENMP
    if (inner > 1) omp_set_max_active_levels(2);
#endif
    float *scratch = (float *)malloc(sizeof(float) * PQ * CRS * (size_t)nthreads);
    if (!scratch) return -1;
#pragma omp parallel for schedule(dynamic, 1) num_threads(nthreads)
    for (int b = 0; b < N; b++) {
#ifdef _OPENMP
        int tid = omp_get_thread_num();
#else
        int tid = 0;
#endif
        float *col = scratch + (size_t)tid * PQ * CRS;
        oracle_im2col(I + (size_t)b * C * H * W, col, C, H, W, R, S, sr, sc, pt, pl, P, Q, inner);
        oracle_sgemm_colmajor(col, K, O + (size_t)b * Kf * PQ, (int)PQ, (int)CRS, Kf, inner);
    }
    free(scratch);
    if (bias) {
#pragma omp parallel for schedule(static)
        for (int b = 0; b < N; b++) {
            float *ptrO = O + (size_t)b * Kf * PQ;
            for (int z = 0; z < Kf; z++)
                for (size_t rc = 0; rc < PQ; rc++, ptrO++) (*ptrO) += bias[z];
        }
    }
    return 0;
}

/* ------------------------------------------------------------------ batchnorm (inference) */

/* src/hardware/cpu/nn/cpu_bn.cpp:118-180, branch trmode==false (:154-163) then the
 * normalisation loop (:165-179): variance[j] = sqrt(global_variance[j] + eps) is WRITTEN
 * into the layer's batch-variance buffer; o = (x - mean)/sd; with affine: opa = o and
 * y = o*g + b (two roundings, no FMA).  b = batch, z = channels, rc = H*W.
 * affine_g == NULL means no affine (then opa is not written). */
void eddl_oracle_batchnorm_inference(int b, int z, int rc, const float *input, float *output, float *opa,
                                     const float *global_mean, const float *global_variance, const float *affine_g,
                                     const float *affine_b, float *variance, float epsilon) {
    const size_t rcz = (size_t)rc * z;
    for (int j = 0; j < z; j++) variance[j] = sqrtf(global_variance[j] + epsilon);
#pragma omp parallel for schedule(static)
    for (int i = 0; i < b; i++) {
        size_t p = (size_t)i * rcz;
        for (size_t k = 0; k < rcz; k++, p++) {
            int j = (int)(k / rc);
            float o = (input[p] - global_mean[j]) / variance[j];
            if (affine_g != NULL) {
                if (opa) opa[p] = o;
                float t = o * affine_g[j];
                output[p] = t + affine_b[j];
            } else {
                output[p] = o;
            }
        }
    }
}

/* ------------------------------------------------------------------ activations */

/* src/hardware/cpu/nn/cpu_activations.cpp:18-33: (x > 0.0) ? x : 0.0  =>  NaN -> 0, -0 -> +0 */
void eddl_oracle_relu(const float *A, float *B, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) {
        if (A[i] > 0.0) B[i] = A[i];
        else B[i] = 0.0;
    }
}

/* src/hardware/cpu/cpu_math.cpp:354-357 */
void eddl_oracle_sigmoid(const float *A, float *B, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) B[i] = 1.0f / (1.0f + expf(-A[i]));
}

/* src/hardware/cpu/nn/cpu_activations.cpp:329-375 (cpu_full_softmax_nd, stable or not) over
 * an axis of length `len` with stride `inner`; `outer` = product of the dimensions before
 * the axis.  Denominator starts at 1.19209e-07. */
void eddl_oracle_softmax(const float *A, float *B, int outer, int len, int inner, int stable) {
    const int n_samples = outer * inner;
#pragma omp parallel for schedule(static)
    for (int si = 0; si < n_samples; si++) {
        size_t start_b = (size_t)(si % inner) + (size_t)(si / inner) * ((size_t)len * inner);
        size_t end_b = start_b + (size_t)(len - 1) * inner;
        float max_value = ORACLE_LOWEST_FLOAT;
        if (stable) {
            for (size_t i = start_b; i <= end_b; i += inner)
                if (A[i] > max_value) max_value = A[i];
        }
        float denominator = ORACLE_EPS_FLOAT;
        for (size_t i = start_b; i <= end_b; i += inner) {
            float value = expf(A[i] - max_value);
            B[i] = value;
            denominator += value;
        }
        for (size_t i = start_b; i <= end_b; i += inner) B[i] /= denominator;
    }
}

/* ------------------------------------------------------------------ pooling */

/* src/hardware/cpu/nn/cpu_pool.cpp:74-121 with get_pixel :20-30.  Window origins step by
 * the stride from -pad; running maximum starts at -3.40282e+38f; out-of-image taps read
 * -FLT_MAX (never win); strict '>' so the first maximum in (ky, kx) scan order wins;
 * indX = absolute column, indY = absolute row, stored as floats; a window in which no tap
 * exceeds the start value leaves its two index slots untouched.  Outputs are written
 * densely in loop order (p++), loop counts from the four pads. */
void eddl_oracle_maxpool2d(const float *I, float *O, float *indX, float *indY, int N, int C, int H, int W, int kr,
                           int kc, int sr, int sc, int pt, int pb, int pl, int pr) {
    const int LP = eddl_oracle_pool_loop_count(H, kr, sr, pt, pb);
    const int LQ = eddl_oracle_pool_loop_count(W, kc, sc, pl, pr);
    const size_t size = (size_t)C * LP * LQ;
#pragma omp parallel for schedule(static)
    for (int b = 0; b < N; b++) {
        size_t p = (size_t)b * size;
        for (int k = 0; k < C; k++) {
            const float *img = I + ((size_t)b * C + k) * H * W;
            for (int i = -pt; i <= H + pb - kr; i += sr)
                for (int j = -pl; j <= W + pr - kc; j += sc, p++) {
                    float max = ORACLE_LOWEST_FLOAT;
                    for (int ki = 0; ki < kr; ki++)
                        for (int kj = 0; kj < kc; kj++) {
                            int px = j + kj, py = i + ki;
                            float v = (px < 0 || py < 0 || px >= W || py >= H) ? ORACLE_MIN_FLOAT
                                                                                : img[(size_t)py * W + px];
                            if (v > max) {
                                max = v;
                                indX[p] = (float)(j + kj);
                                indY[p] = (float)(i + ki);
                            }
                        }
                    O[p] = max;
                }
        }
    }
}

/* src/hardware/cpu/nn/cpu_pool.cpp:226-274: in-bounds taps summed in (ky, kx) order into one
 * fp32 accumulator, divided by kr*kc (padding counts in the divisor). */
void eddl_oracle_avgpool2d(const float *I, float *O, int N, int C, int H, int W, int kr, int kc, int sr, int sc,
                           int pt, int pb, int pl, int pr) {
    const int LP = eddl_oracle_pool_loop_count(H, kr, sr, pt, pb);
    const int LQ = eddl_oracle_pool_loop_count(W, kc, sc, pl, pr);
    const size_t size = (size_t)C * LP * LQ;
    const int ksize = kr * kc;
#pragma omp parallel for schedule(static)
    for (int b = 0; b < N; b++) {
        size_t p = (size_t)b * size;
        for (int k = 0; k < C; k++) {
            const float *img = I + ((size_t)b * C + k) * H * W;
            for (int i = -pt; i <= H + pb - kr; i += sr)
                for (int j = -pl; j <= W + pr - kc; j += sc, p++) {
                    float sum = 0.0f;
                    for (int ki = 0; ki < kr; ki++)
                        for (int kj = 0; kj < kc; kj++) {
                            int px = j + kj, py = i + ki;
                            if (px >= 0 && py >= 0 && px < W && py < H) sum += img[(size_t)py * W + px];
                        }
                    O[p] = sum / (float)ksize;
                }
        }
    }
}

/* ------------------------------------------------------------------ resize / concat / add / pad */

/* Nearest resize, "asymmetric" coordinate mode: src/hardware/cpu/cpu_da.cpp:88-137 (mode 3 branch
 * :113-117) called from cpu_scale :407-436 with offsets = (new_shape - B.shape)/2.  UpSampling2D
 * uses new_shape == B's spatial shape, so offsets are 0 (src/layers/core/layer_resize.cpp:22-47).
 * Source index = (int)((float)dst / ((float)new / in)).  Returns the number of destination
 * elements whose source fell outside A (the reference raises for those in this mode; 0 here
 * for every integer up-scaling). */
int eddl_oracle_scale_nearest(const float *A, float *B, int N, int C, int H, int W, int OH, int OW, int newH,
                              int newW) {
    int off0 = (int)((newH - OH) / 2.0f), off1 = (int)((newW - OW) / 2.0f);
    int bad = 0;
    float scale_y = (float)newH / H, scale_x = (float)newW / W;
    for (int b = 0; b < N; b++)
        for (int c = 0; c < C; c++)
            for (int Bi = 0; Bi < OH; Bi++)
                for (int Bj = 0; Bj < OW; Bj++) {
                    int Ai = Bi + off0, Aj = Bj + off1;
                    Ai = (int)(Ai / scale_y);
                    Aj = (int)(Aj / scale_x);
                    size_t bpos = (((size_t)b * C + c) * OH + Bi) * OW + Bj;
                    if (Ai >= 0 && Ai < H && Aj >= 0 && Aj < W) B[bpos] = A[(((size_t)b * C + c) * H + Ai) * W + Aj];
                    else bad++;
                }
    return bad;
}

/* src/hardware/cpu/cpu_core.cpp:368-396 (derivative == false).  A 4-D (or any) row-major
 * tensor is described around the concatenation axis by `outer` (product of dims before the
 * axis) and `inner` (stride of the axis); input i has axis extent ext[i]. */
void eddl_oracle_concat(float *dest_base, const float *const *srcs, const int *ext, int n_in, int outer, int inner) {
    size_t steps = 0;
    for (int i = 0; i < n_in; i++) steps += (size_t)ext[i] * inner;
    size_t offset = 0, src_stride = 0;
    for (int i = 0; i < n_in; i++) {
        offset += src_stride;
        src_stride = (size_t)ext[i] * inner;
        float *dest = dest_base + offset;
        const float *src = srcs[i];
        size_t size = src_stride * outer;
        for (size_t j = 0; j < size; j++) {
            size_t k = j % src_stride, stride_idx = j / src_stride;
            dest[stride_idx * steps + k] = src[j];
        }
    }
}

/* src/hardware/cpu/cpu_math.cpp:278-287: C (+)= scA*A + scB*B.  The residual Add of the
 * model graphs is this with scA = scB = 1, incC = 0 (src/layers/operators/layer_sum.cpp:73-78);
 * the n-ary LAdd is fill_(0) then inc per parent (src/layers/merge/layer_add.cpp:60-64,
 * cpu_math.cpp:291-298, cpu_core.cpp:250-257). */
void eddl_oracle_add(float scA, const float *A, float scB, const float *B, float *C, int incC, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) {
        float a = scA * A[i];
        float b = scB * B[i];
        if (incC) C[i] += a + b;
        else C[i] = a + b;
    }
}

void eddl_oracle_inc(const float *A, float *B, size_t n) {
    for (size_t i = 0; i < n; i++) B[i] += A[i];
}

void eddl_oracle_fill(float *A, float v, size_t n) {
    for (size_t i = 0; i < n; i++) A[i] = v;
}

/* src/hardware/cpu/cpu_da.cpp:502-517: interior copy only, pads = (top, right, bottom, left);
 * the border keeps whatever B held (the layer fills it with the constant once, at
 * construction: src/layers/da/layer_pad.cpp:23-41). */
void eddl_oracle_pad(const float *A, float *B, int N, int C, int H, int W, int top, int right, int bottom, int left) {
    const int OH = H + top + bottom, OW = W + left + right;
    for (int b = 0; b < N; b++)
        for (int c = 0; c < C; c++)
            for (int h = 0; h < H; h++)
                for (int w = 0; w < W; w++)
                    B[(((size_t)b * C + c) * OH + (h + top)) * OW + (w + left)] = A[(((size_t)b * C + c) * H + h) * W + w];
}

/* ------------------------------------------------------------------ dense */

/* src/hardware/cpu/cpu_math.cpp:302-328 as used by src/layers/core/layer_dense.cpp:65-73
 * (tA = tB = 0, incC = 0): C[m x n] = A[m x k] * B[k x n], row-major, B = W[in, out].
 * The reference's product is an Eigen GEMM (summation order Eigen-internal); this sums each
 * output's k products in increasing index with one fp32 accumulator.  The reference's tests
 * hold no vector for it; it is pinned as a textbook matrix product against numpy (float64)
 * and against PyTorch's Linear layers in the exported-network fixtures. */
void eddl_oracle_mult2d(const float *A, const float *B, float *C, int m, int k, int n) {
#pragma omp parallel for schedule(static)
    for (int j0 = 0; j0 < n; j0 += 256) {
        int jn = n - j0 < 256 ? n - j0 : 256;
        for (int i = 0; i < m; i++) {
            float acc[256];
            for (int j = 0; j < jn; j++) acc[j] = 0.0f;
            for (int l = 0; l < k; l++) {
                float a = A[(size_t)i * k + l];
                const float *brow = B + (size_t)l * n + j0;
                for (int j = 0; j < jn; j++) acc[j] += a * brow[j];
            }
            memcpy(C + (size_t)i * n + j0, acc, sizeof(float) * jn);
        }
    }
}

/* src/hardware/cpu/cpu_math.cpp:354-365 (cpu_sum2D_rowwise): C[i][j] = A[i][j] + B[j] */
void eddl_oracle_sum2d_rowwise(const float *A, const float *B, float *C, int rows, int cols) {
    for (int i = 0; i < rows; i++)
        for (int j = 0; j < cols; j++) C[(size_t)i * cols + j] = A[(size_t)i * cols + j] + B[j];
}

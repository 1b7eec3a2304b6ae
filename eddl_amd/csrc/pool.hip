// MaxPool2D (with argmax) and AvgPool2D forward.  Semantics of the reference's CPU loops
// (src/hardware/cpu/nn/cpu_pool.cpp:74-121 and :226-274): window origins step from -pad,
// taps scanned ky then kx, strict '>' so the first maximum wins, indices are absolute input
// coordinates stored as floats, average divides by kr*kc whatever the padding.
//
// Two kernels per operator:
//   * small windows: one thread per output, neighbouring lanes on neighbouring outputs so
//     loads and the three stores are coalesced; a 2x2/stride-2 fast path reads two input
//     rows as float4 and produces two outputs per thread;
//   * large windows (>= 64 taps, e.g. global pooling): one wavefront per output, lanes
//     stride over the taps in scan order and a wavefront (max, tap-index) reduction picks the
//     winner; ties go to the lower tap index, which is the first maximum of the scan.
#include "common.h"

using namespace eddlhip;

namespace {

constexpr int TPB = 256;
constexpr float LOWEST = -3.40282e+38f;  // the reference's running-maximum start value

struct PoolShape {
    int C, H, W, kr, kc, sr, sc, pt, pl, LP, LQ;
};

__global__ __launch_bounds__(TPB) void maxpool_kernel(const float *__restrict__ I, float *__restrict__ O,
                                                      float *__restrict__ indX, float *__restrict__ indY, size_t total,
                                                      PoolShape s) {
    size_t t0 = (size_t)blockIdx.x * TPB + threadIdx.x, stride = (size_t)gridDim.x * TPB;
    for (size_t p = t0; p < total; p += stride) {
        int oj = (int)(p % s.LQ);
        size_t r = p / s.LQ;
        int oi = (int)(r % s.LP);
        size_t plane = r / s.LP;  // b*C + k
        const float *img = I + plane * s.H * s.W;
        const int i = oi * s.sr - s.pt, j = oj * s.sc - s.pl;
        float mx = LOWEST;
        int bx = 0, by = 0;
        bool found = false;
        for (int ki = 0; ki < s.kr; ki++) {
            int py = i + ki;
            if (py < 0 || py >= s.H) continue;  // out-of-image taps read -FLT_MAX and never win
            for (int kj = 0; kj < s.kc; kj++) {
                int px = j + kj;
                if (px < 0 || px >= s.W) continue;
                float v = img[(size_t)py * s.W + px];
                if (v > mx) {
                    mx = v;
                    bx = px;
                    by = py;
                    found = true;
                }
            }
        }
        O[p] = mx;
        if (found) {
            indX[p] = (float)bx;
            indY[p] = (float)by;
        }
    }
}

// Window shape known at compile time (3x3 here): the KR*KC loads of an output are independent and all
// issued before the first comparison; a tap outside the image reads -FLT_MAX, which is below the
// running maximum's start value and so never wins - the reference's own rule (cpu_pool.cpp:20-30).
template <int KR, int KC>
__global__ __launch_bounds__(TPB) void maxpool_window_kernel(const float *__restrict__ I, float *__restrict__ O,
                                                             float *__restrict__ indX, float *__restrict__ indY, size_t total,
                                                             PoolShape s) {
    size_t t0 = (size_t)blockIdx.x * TPB + threadIdx.x, stride = (size_t)gridDim.x * TPB;
    for (size_t p = t0; p < total; p += stride) {
        const int oj = (int)(p % s.LQ);
        const size_t r = p / s.LQ;
        const int oi = (int)(r % s.LP);
        const size_t plane = r / s.LP;
        const float *img = I + plane * s.H * s.W;
        const int i = oi * s.sr - s.pt, j = oj * s.sc - s.pl;
        float v[KR][KC];
#pragma unroll
        for (int ki = 0; ki < KR; ki++)
#pragma unroll
            for (int kj = 0; kj < KC; kj++) {
                const int py = i + ki, px = j + kj;
                const bool in = (unsigned)py < (unsigned)s.H && (unsigned)px < (unsigned)s.W;
                v[ki][kj] = in ? img[py * s.W + px] : -3.402823466e+38f;
            }
        float mx = LOWEST;
        int bx = 0, by = 0;
        bool found = false;
#pragma unroll
        for (int ki = 0; ki < KR; ki++)
#pragma unroll
            for (int kj = 0; kj < KC; kj++)
                if (v[ki][kj] > mx) {
                    mx = v[ki][kj];
                    bx = j + kj;
                    by = i + ki;
                    found = true;
                }
        O[p] = mx;
        if (found) {
            indX[p] = (float)bx;
            indY[p] = (float)by;
        }
    }
}

// 2x2 window, stride 2, no padding, even W, 16-byte aligned rows: each thread reads a float4
// from two consecutive input rows and writes two outputs (float2 stores).
__global__ __launch_bounds__(TPB) void maxpool_2x2s2_kernel(const float *__restrict__ I, float *__restrict__ O,
                                                            float *__restrict__ indX, float *__restrict__ indY,
                                                            size_t total_pairs, int H, int W, int LP, int LQ) {
    const int LQ2 = LQ / 2;
    size_t t0 = (size_t)blockIdx.x * TPB + threadIdx.x, stride = (size_t)gridDim.x * TPB;
    for (size_t t = t0; t < total_pairs; t += stride) {
        int oj2 = (int)(t % LQ2);
        size_t r = t / LQ2;
        int oi = (int)(r % LP);
        size_t plane = r / LP;
        const float *row0 = I + (plane * H + 2 * oi) * W + 4 * oj2;
        float4 a = *reinterpret_cast<const float4 *>(row0);
        float4 b = *reinterpret_cast<const float4 *>(row0 + W);
        float2 o, ix, iy;
        const float x0 = (float)(4 * oj2), y0 = (float)(2 * oi);
        {
            float mx = LOWEST;
            float fx = 0.f, fy = 0.f;
            bool found = false;
            if (a.x > mx) { mx = a.x; fx = x0; fy = y0; found = true; }
            if (a.y > mx) { mx = a.y; fx = x0 + 1.f; fy = y0; found = true; }
            if (b.x > mx) { mx = b.x; fx = x0; fy = y0 + 1.f; found = true; }
            if (b.y > mx) { mx = b.y; fx = x0 + 1.f; fy = y0 + 1.f; found = true; }
            o.x = mx;
            size_t p = (plane * LP + oi) * LQ + 2 * oj2;
            if (!found) { fx = indX[p]; fy = indY[p]; }
            ix.x = fx; iy.x = fy;
        }
        {
            float mx = LOWEST;
            float fx = 0.f, fy = 0.f;
            bool found = false;
            if (a.z > mx) { mx = a.z; fx = x0 + 2.f; fy = y0; found = true; }
            if (a.w > mx) { mx = a.w; fx = x0 + 3.f; fy = y0; found = true; }
            if (b.z > mx) { mx = b.z; fx = x0 + 2.f; fy = y0 + 1.f; found = true; }
            if (b.w > mx) { mx = b.w; fx = x0 + 3.f; fy = y0 + 1.f; found = true; }
            o.y = mx;
            size_t p = (plane * LP + oi) * LQ + 2 * oj2 + 1;
            if (!found) { fx = indX[p]; fy = indY[p]; }
            ix.y = fx; iy.y = fy;
        }
        size_t p = (plane * LP + oi) * LQ + 2 * oj2;
        *reinterpret_cast<float2 *>(O + p) = o;
        *reinterpret_cast<float2 *>(indX + p) = ix;
        *reinterpret_cast<float2 *>(indY + p) = iy;
    }
}

// 3x3 window, stride 2, left padding PL of 0 or 1, W a multiple of 4, even LQ with 2*LQ <= W, aligned
// tensors (ResNet's stem pool).  A thread produces two neighbouring outputs from one float4 per input row
// (columns 4m .. 4m+3) plus one more column: 4m-1 with PL == 1, 4m+4 with PL == 0.  That column is the
// neighbouring lane's .w / .x, taken by a lane shuffle; the first / last thread of an output row and of a
// wavefront loads it itself (or takes -FLT_MAX outside the image).  Same scan order and strict '>' as above.
template <int PL>
__global__ __launch_bounds__(TPB) void maxpool_3x3s2_kernel(const float *__restrict__ I, float *__restrict__ O,
                                                            float *__restrict__ indX, float *__restrict__ indY,
                                                            size_t total_pairs, int H, int W, int LP, int LQ, int pt) {
    constexpr float OUTSIDE = -3.402823466e+38f;
    const int LQ2 = LQ / 2, lane = threadIdx.x & 63;
    size_t t0 = (size_t)blockIdx.x * TPB + threadIdx.x, stride = (size_t)gridDim.x * TPB;
    // every lane of a wavefront makes the same number of trips, so that the shuffles below always run
    // with all 64 lanes; lanes past the end compute on clamped coordinates and store nothing
    const size_t wave_first = t0 - lane;
    for (size_t tw = wave_first; tw < total_pairs; tw += stride) {
        const size_t tt = tw + lane;
        const bool live = tt < total_pairs;
        const size_t t = live ? tt : total_pairs - 1;
        const int m = (int)(t % LQ2);
        const size_t r = t / LQ2;
        const int oi = (int)(r % LP);
        const size_t plane = r / LP;
        const float *img = I + plane * (size_t)H * W;
        const int i = 2 * oi - pt;
        float4 c[3];
        float e[3];
#pragma unroll
        for (int ki = 0; ki < 3; ki++) {
            const int py = i + ki;
            const bool rowin = (unsigned)py < (unsigned)H;
            c[ki] = rowin ? *reinterpret_cast<const float4 *>(img + (size_t)py * W + 4 * m) : make_float4(OUTSIDE, OUTSIDE, OUTSIDE, OUTSIDE);
            if (PL == 1) {
                const float nb = __shfl_up(c[ki].w, 1, 64);
                const bool own = lane == 0 || m == 0;  // no left neighbour in this wavefront / in this output row
                e[ki] = own ? ((rowin && m > 0) ? img[(size_t)py * W + 4 * m - 1] : OUTSIDE) : nb;
            } else {
                const float nb = __shfl_down(c[ki].x, 1, 64);
                const bool own = lane == 63 || m == LQ2 - 1;
                e[ki] = own ? ((rowin && 4 * m + 4 < W) ? img[(size_t)py * W + 4 * m + 4] : OUTSIDE) : nb;
            }
        }
        float2 o, ix, iy;
        const size_t p = (plane * LP + oi) * LQ + 2 * m;
        const int j0 = 4 * m - PL;  // first column of the first output's window
        {
            float mx = LOWEST, fx = 0.f, fy = 0.f;
            bool found = false;
#pragma unroll
            for (int ki = 0; ki < 3; ki++) {
                const float w0 = PL ? e[ki] : c[ki].x, w1 = PL ? c[ki].x : c[ki].y, w2 = PL ? c[ki].y : c[ki].z;
                if (w0 > mx) { mx = w0; fx = (float)j0; fy = (float)(i + ki); found = true; }
                if (w1 > mx) { mx = w1; fx = (float)(j0 + 1); fy = (float)(i + ki); found = true; }
                if (w2 > mx) { mx = w2; fx = (float)(j0 + 2); fy = (float)(i + ki); found = true; }
            }
            o.x = mx;
            if (!found && live) { fx = indX[p]; fy = indY[p]; }
            ix.x = fx; iy.x = fy;
        }
        {
            float mx = LOWEST, fx = 0.f, fy = 0.f;
            bool found = false;
#pragma unroll
            for (int ki = 0; ki < 3; ki++) {
                const float w0 = PL ? c[ki].y : c[ki].z, w1 = PL ? c[ki].z : c[ki].w, w2 = PL ? c[ki].w : e[ki];
                if (w0 > mx) { mx = w0; fx = (float)(j0 + 2); fy = (float)(i + ki); found = true; }
                if (w1 > mx) { mx = w1; fx = (float)(j0 + 3); fy = (float)(i + ki); found = true; }
                if (w2 > mx) { mx = w2; fx = (float)(j0 + 4); fy = (float)(i + ki); found = true; }
            }
            o.y = mx;
            if (!found && live) { fx = indX[p + 1]; fy = indY[p + 1]; }
            ix.y = fx; iy.y = fy;
        }
        if (live) {
            *reinterpret_cast<float2 *>(O + p) = o;
            *reinterpret_cast<float2 *>(indX + p) = ix;
            *reinterpret_cast<float2 *>(indY + p) = iy;
        }
    }
}

// The same window on an even number of output rows: a thread produces a 2 x 2 patch of outputs (rows 2h, 2h+1) from five
// input rows instead of two times three - the row the two windows share is loaded once - with five float4 loads in
// flight.  Per output the scan order and the strict '>' are those of the kernel above.
template <int PL>
__global__ __launch_bounds__(TPB) void maxpool_3x3s2_rows_kernel(const float *__restrict__ I, float *__restrict__ O,
                                                                 float *__restrict__ indX, float *__restrict__ indY,
                                                                 size_t total_quads, int H, int W, int LP, int LQ, int pt) {
    constexpr float OUTSIDE = -3.402823466e+38f;
    const int LQ2 = LQ / 2, LP2 = LP / 2, lane = threadIdx.x & 63;
    size_t t0 = (size_t)blockIdx.x * TPB + threadIdx.x, stride = (size_t)gridDim.x * TPB;
    const size_t wave_first = t0 - lane;
    for (size_t tw = wave_first; tw < total_quads; tw += stride) {
        const size_t tt = tw + lane;
        const bool live = tt < total_quads;
        const size_t t = live ? tt : total_quads - 1;
        const int m = (int)(t % LQ2);
        const size_t r = t / LQ2;
        const int oh = (int)(r % LP2);
        const size_t plane = r / LP2;
        const float *img = I + plane * (size_t)H * W;
        const int i = 4 * oh - pt;  // first input row of the upper window
        float4 c[5];
        float e[5];
#pragma unroll
        for (int ki = 0; ki < 5; ki++) {
            const int py = i + ki;
            const bool rowin = (unsigned)py < (unsigned)H;
            c[ki] = rowin ? *reinterpret_cast<const float4 *>(img + (size_t)py * W + 4 * m) : make_float4(OUTSIDE, OUTSIDE, OUTSIDE, OUTSIDE);
        }
#pragma unroll
        for (int ki = 0; ki < 5; ki++) {
            const int py = i + ki;
            const bool rowin = (unsigned)py < (unsigned)H;
            if (PL == 1) {
                const float nb = __shfl_up(c[ki].w, 1, 64);
                const bool own = lane == 0 || m == 0;
                e[ki] = own ? ((rowin && m > 0) ? img[(size_t)py * W + 4 * m - 1] : OUTSIDE) : nb;
            } else {
                const float nb = __shfl_down(c[ki].x, 1, 64);
                const bool own = lane == 63 || m == LQ2 - 1;
                e[ki] = own ? ((rowin && 4 * m + 4 < W) ? img[(size_t)py * W + 4 * m + 4] : OUTSIDE) : nb;
            }
        }
        const int j0 = 4 * m - PL;
#pragma unroll
        for (int half = 0; half < 2; half++) {  // output rows 2*oh + half: input rows i + 2*half .. i + 2*half + 2
            const size_t p = (plane * LP + 2 * oh + half) * LQ + 2 * m;
            float2 o, ix, iy;
            {
                float mx = LOWEST, fx = 0.f, fy = 0.f;
                bool found = false;
#pragma unroll
                for (int kk = 0; kk < 3; kk++) {
                    const int ki = 2 * half + kk;
                    const float w0 = PL ? e[ki] : c[ki].x, w1 = PL ? c[ki].x : c[ki].y, w2 = PL ? c[ki].y : c[ki].z;
                    if (w0 > mx) { mx = w0; fx = (float)j0; fy = (float)(i + ki); found = true; }
                    if (w1 > mx) { mx = w1; fx = (float)(j0 + 1); fy = (float)(i + ki); found = true; }
                    if (w2 > mx) { mx = w2; fx = (float)(j0 + 2); fy = (float)(i + ki); found = true; }
                }
                o.x = mx;
                if (!found && live) { fx = indX[p]; fy = indY[p]; }
                ix.x = fx; iy.x = fy;
            }
            {
                float mx = LOWEST, fx = 0.f, fy = 0.f;
                bool found = false;
#pragma unroll
                for (int kk = 0; kk < 3; kk++) {
                    const int ki = 2 * half + kk;
                    const float w0 = PL ? c[ki].y : c[ki].z, w1 = PL ? c[ki].z : c[ki].w, w2 = PL ? c[ki].w : e[ki];
                    if (w0 > mx) { mx = w0; fx = (float)(j0 + 2); fy = (float)(i + ki); found = true; }
                    if (w1 > mx) { mx = w1; fx = (float)(j0 + 3); fy = (float)(i + ki); found = true; }
                    if (w2 > mx) { mx = w2; fx = (float)(j0 + 4); fy = (float)(i + ki); found = true; }
                }
                o.y = mx;
                if (!found && live) { fx = indX[p + 1]; fy = indY[p + 1]; }
                ix.y = fx; iy.y = fy;
            }
            if (live) {
                *reinterpret_cast<float2 *>(O + p) = o;
                *reinterpret_cast<float2 *>(indX + p) = ix;
                *reinterpret_cast<float2 *>(indY + p) = iy;
            }
        }
    }
}

// One wavefront per output.  Lane l visits taps l, l+64, ... in scan order (tap = ki*kc + kj),
// keeping its first maximum; the reduction keeps the larger value and, on equal values, the
// lower tap index.
__global__ __launch_bounds__(TPB) void maxpool_wave_kernel(const float *__restrict__ I, float *__restrict__ O,
                                                           float *__restrict__ indX, float *__restrict__ indY, size_t total,
                                                           PoolShape s) {
    const int lane = threadIdx.x & 63;
    const size_t wave = ((size_t)blockIdx.x * TPB + threadIdx.x) >> 6, nwaves = ((size_t)gridDim.x * TPB) >> 6;
    const int taps = s.kr * s.kc;
    for (size_t p = wave; p < total; p += nwaves) {
        int oj = (int)(p % s.LQ);
        size_t r = p / s.LQ;
        int oi = (int)(r % s.LP);
        size_t plane = r / s.LP;
        const float *img = I + plane * s.H * s.W;
        const int i = oi * s.sr - s.pt, j = oj * s.sc - s.pl;
        float mx = LOWEST;
        int best = 0x7fffffff;  // tap index of the winner; "none" sorts last
        for (int t = lane; t < taps; t += 64) {
            int ki = t / s.kc, kj = t - ki * s.kc;
            int py = i + ki, px = j + kj;
            if (py < 0 || py >= s.H || px < 0 || px >= s.W) continue;
            float v = img[(size_t)py * s.W + px];
            if (v > mx) {
                mx = v;
                best = t;
            }
        }
        for (int off = 32; off > 0; off >>= 1) {
            float omx = __shfl_xor(mx, off, 64);
            int obest = __shfl_xor(best, off, 64);
            if (omx > mx || (omx == mx && obest < best)) {
                mx = omx;
                best = obest;
            }
        }
        if (lane == 0) {
            O[p] = mx;
            if (best != 0x7fffffff) {
                int ki = best / s.kc, kj = best - ki * s.kc;
                indX[p] = (float)(j + kj);
                indY[p] = (float)(i + ki);
            }
        }
    }
}

// Sequential (ky,kx) sum of the in-image taps, one thread per output: bit-exact with the
// reference's accumulation order for every window size.
__global__ __launch_bounds__(TPB) void avgpool_kernel(const float *__restrict__ I, float *__restrict__ O, size_t total,
                                                      PoolShape s) {
    size_t t0 = (size_t)blockIdx.x * TPB + threadIdx.x, stride = (size_t)gridDim.x * TPB;
    const float ksize = (float)(s.kr * s.kc);
    for (size_t p = t0; p < total; p += stride) {
        int oj = (int)(p % s.LQ);
        size_t r = p / s.LQ;
        int oi = (int)(r % s.LP);
        size_t plane = r / s.LP;
        const float *img = I + plane * s.H * s.W;
        const int i = oi * s.sr - s.pt, j = oj * s.sc - s.pl;
        float sum = 0.0f;
        for (int ki = 0; ki < s.kr; ki++) {
            int py = i + ki;
            if (py < 0 || py >= s.H) continue;
            for (int kj = 0; kj < s.kc; kj++) {
                int px = j + kj;
                if (px < 0 || px >= s.W) continue;
                sum = __fadd_rn(sum, img[(size_t)py * s.W + px]);
            }
        }
        O[p] = __fdiv_rn(sum, ksize);
    }
}

// Window = the whole plane, no padding (GlobalAveragePool2D): one wavefront takes 64 planes, which
// are contiguous in memory, reads them with coalesced loads into LDS (row stride odd: no bank
// conflicts), and each lane then adds up its own plane in the same sequential order as above.
__global__ __launch_bounds__(64) void avgpool_plane_kernel(const float *__restrict__ I, float *__restrict__ O, size_t planes, int hw) {
    extern __shared__ float plane_tile[];
    const int lane = threadIdx.x, row = hw | 1;
    const size_t p0 = (size_t)blockIdx.x * 64;
    const int here = (int)(planes - p0 < 64 ? planes - p0 : 64);
    const float *src = I + p0 * hw;
    // element i belongs to plane i / hw, position i % hw: both advance by fixed steps from one load to the next.
    // Sixteen loads are requested before the first of them is stored, so a wavefront makes a handful of trips to memory.
    int pl = lane / hw, k = lane - pl * hw;
    const int dp = 64 / hw, dk = 64 - dp * hw;
    const int n = here * hw;
    for (int base = lane; base < n; base += 64 * 16) {
        float v[16];
#pragma unroll
        for (int u = 0; u < 16; u++) v[u] = base + 64 * u < n ? src[base + 64 * u] : 0.0f;
#pragma unroll
        for (int u = 0; u < 16; u++) {
            if (base + 64 * u < n) plane_tile[pl * row + k] = v[u];
            pl += dp;
            k += dk;
            if (k >= hw) {
                k -= hw;
                pl++;
            }
        }
    }
    __syncthreads();
    if (lane < here) {
        float sum = 0.0f;
#pragma unroll 8
        for (int k = 0; k < hw; k++) sum = __fadd_rn(sum, plane_tile[lane * row + k]);
        O[p0 + lane] = __fdiv_rn(sum, (float)hw);
    }
}

int loop_count(int in, int k, int stride, int pad_lo, int pad_hi) {
    long long last = (long long)in + pad_hi - k, first = -(long long)pad_lo;
    if (last < first) return 0;
    return (int)((last - first) / stride) + 1;
}

int check_pool(const char *name, int N, int C, int H, int W, int kr, int kc, int sr, int sc, int pt, int pb, int pl, int pr,
               PoolShape *s) {
    EH_REQUIRE(N >= 0 && C > 0 && H > 0 && W > 0, "%s: bad input shape", name);
    EH_REQUIRE(kr > 0 && kc > 0 && sr > 0 && sc > 0, "%s: bad window/stride", name);
    EH_REQUIRE(pt >= 0 && pb >= 0 && pl >= 0 && pr >= 0, "%s: negative padding", name);
    *s = PoolShape{C, H, W, kr, kc, sr, sc, pt, pl, loop_count(H, kr, sr, pt, pb), loop_count(W, kc, sc, pl, pr)};
    EH_REQUIRE((long long)C * H * W <= 0x7fffffffLL, "%s: image too large", name);
    return 0;
}

}  // namespace

extern "C" {

int eddlhip_pool2d_out_dims(int H, int W, int kr, int kc, int sr, int sc, int pad_top, int pad_bottom, int pad_left,
                            int pad_right, int *LP, int *LQ) {
    EH_REQUIRE(LP && LQ, "pool2d_out_dims: NULL output");
    EH_REQUIRE(H > 0 && W > 0 && kr > 0 && kc > 0 && sr > 0 && sc > 0, "pool2d_out_dims: bad shape");
    *LP = loop_count(H, kr, sr, pad_top, pad_bottom);
    *LQ = loop_count(W, kc, sc, pad_left, pad_right);
    return 0;
}

int eddlhip_maxpool2d(int dev, const float *I, float *O, float *indX, float *indY, int N, int C, int H, int W, int kr, int kc,
                      int sr, int sc, int pad_top, int pad_bottom, int pad_left, int pad_right) {
    PoolShape s;
    EH_TRY(check_pool("maxpool2d", N, C, H, W, kr, kc, sr, sc, pad_top, pad_bottom, pad_left, pad_right, &s));
    size_t total = (size_t)N * C * s.LP * s.LQ;
    if (total == 0) return 0;
    EH_REQUIRE(I && O && indX && indY, "maxpool2d: NULL tensor");
    EH_TRY(use_device(dev));
    hipStream_t st = state(dev).stream;
    auto al = [](const void *p, unsigned a) { return ((uintptr_t)p & (a - 1)) == 0; };
    if (kr == 2 && kc == 2 && sr == 2 && sc == 2 && !pad_top && !pad_left && !pad_bottom && !pad_right && W % 4 == 0 &&
        al(I, 16) && al(O, 8) && al(indX, 8) && al(indY, 8)) {
        size_t pairs = total / 2;
        hipLaunchKernelGGL(maxpool_2x2s2_kernel, dim3(eh_blocks(pairs, TPB, 1u << 18)), dim3(TPB), 0, st, I, O, indX, indY, pairs, H,
                           W, s.LP, s.LQ);
    } else if (kr == 3 && kc == 3 && sr == 2 && sc == 2 && pad_left <= 1 && W % 4 == 0 && s.LQ % 2 == 0 && 2 * s.LQ <= W &&
               al(I, 16) && al(O, 8) && al(indX, 8) && al(indY, 8)) {
        size_t pairs = total / 2;
        if (s.LP % 2 == 0) {
            auto kern = pad_left ? maxpool_3x3s2_rows_kernel<1> : maxpool_3x3s2_rows_kernel<0>;
            hipLaunchKernelGGL(kern, dim3(eh_blocks(pairs / 2, TPB, 1u << 18)), dim3(TPB), 0, st, I, O, indX, indY, pairs / 2, H, W, s.LP,
                               s.LQ, pad_top);
        } else {
            auto kern = pad_left ? maxpool_3x3s2_kernel<1> : maxpool_3x3s2_kernel<0>;
            hipLaunchKernelGGL(kern, dim3(eh_blocks(pairs, TPB, 1u << 18)), dim3(TPB), 0, st, I, O, indX, indY, pairs, H, W, s.LP, s.LQ,
                               pad_top);
        }
    } else if (kr == 3 && kc == 3 && (long long)H * W < (1LL << 31)) {
        hipLaunchKernelGGL((maxpool_window_kernel<3, 3>), dim3(eh_blocks(total, TPB, 1u << 18)), dim3(TPB), 0, st, I, O, indX, indY,
                           total, s);
    } else if (kr * kc >= 64) {
        hipLaunchKernelGGL(maxpool_wave_kernel, dim3(eh_blocks(total, TPB / 64, 1u << 18)), dim3(TPB), 0, st, I, O, indX, indY, total,
                           s);
    } else {
        hipLaunchKernelGGL(maxpool_kernel, dim3(eh_blocks(total, TPB, 1u << 18)), dim3(TPB), 0, st, I, O, indX, indY, total, s);
    }
    EH_CHECK_LAUNCH();
    return 0;
}

int eddlhip_avgpool2d(int dev, const float *I, float *O, int N, int C, int H, int W, int kr, int kc, int sr, int sc, int pad_top,
                      int pad_bottom, int pad_left, int pad_right) {
    PoolShape s;
    EH_TRY(check_pool("avgpool2d", N, C, H, W, kr, kc, sr, sc, pad_top, pad_bottom, pad_left, pad_right, &s));
    size_t total = (size_t)N * C * s.LP * s.LQ;
    if (total == 0) return 0;
    EH_REQUIRE(I && O, "avgpool2d: NULL tensor");
    EH_TRY(use_device(dev));
    const bool whole_plane = kr == H && kc == W && pad_top == 0 && pad_bottom == 0 && pad_left == 0 && pad_right == 0 && s.LP == 1 && s.LQ == 1;
    if (whole_plane && H * W <= 255 && total <= 0x7fffffffULL * 64) {
        const int hw = H * W;
        hipLaunchKernelGGL(avgpool_plane_kernel, dim3((unsigned)((total + 63) / 64)), dim3(64), (size_t)64 * (hw | 1) * sizeof(float),
                           state(dev).stream, I, O, total, hw);
    } else {
        hipLaunchKernelGGL(avgpool_kernel, dim3(eh_blocks(total, TPB, 1u << 18)), dim3(TPB), 0, state(dev).stream, I, O, total, s);
    }
    EH_CHECK_LAUNCH();
    return 0;
}

}  // extern "C"

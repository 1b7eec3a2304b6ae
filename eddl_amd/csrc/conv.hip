// Conv2D forward for gfx950: implicit GEMM on the fp32 matrix cores, no materialised
// lowering buffer, bias / inference batch-norm / residual add / ReLU fused into the store.
//
// GEMM view (the reference lowers to the same product, src/hardware/cpu/nn/cpu_conv.cpp:55-112,
// 210-223, but materialises the lowered matrix):
//     O[m][n] = sum_i  Wt[i][m] * Col[i][n]
//     m = output channel, n = flattened (image, p, q) output pixel,
//     i = (c, ky, kx) tap, c slowest  - the order of OIHW filter memory.
// Col is never stored: each workgroup gathers the 16 x BN slice it needs straight from the
// NCHW input into LDS (out-of-image taps become 0).  Filters are repacked once per call into
// a tap-major, zero-padded matrix Wp[i][m] (private workspace) so that the filter slice of a
// tile is 16 rows of contiguous floats: 16-byte global loads, 16-byte LDS stores.
//
// Tile: BM x BN outputs per 256-thread workgroup (4 wavefronts), K-step 16 taps, LDS
// double-buffered (one barrier per step), global loads of step t+1 issued before the MFMAs of
// step t.  Each wavefront owns TM x TN blocks of 32x32 outputs and advances them with
// v_mfma_f32_32x32x2_f32 (A = 32 channels x 2 taps, B = 2 taps x 32 pixels).
//
// Accumulation order per output: taps in increasing i, two per MFMA (the instruction adds
// both products of a pair into the fp32 accumulator), all in one accumulator from the first
// tap to the last; no split over taps.  The reference CPU order is ky,kx,c per output in its
// direct form and Eigen-internal in its GEMM form, so agreement is to a tolerance, not
// bit-for-bit; the scalar kernel at the end of this file follows the direct form's order and
// rounding exactly.
//
// Workgroups are numbered so that those running on one XCD (workgroup id mod 8) cover
// neighbouring pixel tiles for all channel tiles: the input slice they share stays in that
// XCD's L2.
#include "common.h"

using namespace eddlhip;

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BK = 16;       // taps per pipeline step
constexpr int M_ALIGN = 128; // packed filter rows are padded to this many channels

struct ConvParams {
    const float *I;
    const float *Wp;  // packed filters [CRSp][Mp]
    const float *K;   // original OIHW filters (scalar kernel only)
    float *O;
    const float *bias, *bn_g, *bn_b, *bn_mean, *bn_var, *residual;
    float bn_eps;
    int relu;
    int N, C, H, W, Kf, R, S, sr, sc, pt, pl, P, Q;
    int CRS, Mp, nsteps, PQ;
    long long npix;
    int gm, gn;
};

// The fused tail of a Conv -> BatchNorm(inference) -> Add -> ReLU chain; every step rounded
// to fp32, no contraction.  sd is sqrtf(var + eps) for channel k (unused without batch-norm).
struct ChannelEpilogue {
    float bias, mean, sd, g, b;
};

__device__ __forceinline__ ChannelEpilogue load_channel(const ConvParams &p, int k) {
    ChannelEpilogue e;
    e.bias = p.bias ? p.bias[k] : 0.0f;
    e.mean = 0.0f;
    e.sd = 1.0f;
    e.g = 1.0f;
    e.b = 0.0f;
    if (p.bn_mean) {
        e.mean = p.bn_mean[k];
        e.sd = sqrtf(__fadd_rn(p.bn_var[k], p.bn_eps));
        if (p.bn_g) {
            e.g = p.bn_g[k];
            e.b = p.bn_b[k];
        }
    }
    return e;
}

__device__ __forceinline__ float apply_epilogue(const ConvParams &p, const ChannelEpilogue &e, float v, size_t oidx) {
    if (p.bias) v = __fadd_rn(v, e.bias);
    if (p.bn_mean) {
        v = __fdiv_rn(__fsub_rn(v, e.mean), e.sd);
        if (p.bn_g) v = __fadd_rn(__fmul_rn(v, e.g), e.b);
    }
    if (p.residual) v = __fadd_rn(v, p.residual[oidx]);
    if (p.relu) v = v > 0.0f ? v : 0.0f;
    return v;
}

// ---------------------------------------------------------------- filter repack
// K[Kf][CRS] (OIHW memory) -> Wp[CRSp][Mp], zero-padded; 32x32 tiles through LDS so that
// both the read and the write are coalesced.
__global__ __launch_bounds__(256) void pack_filters_kernel(const float *__restrict__ K, float *__restrict__ Wp, int Kf, int CRS,
                                                           int Mp, int CRSp) {
    __shared__ float tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    const int i0 = blockIdx.x * 32, m0 = blockIdx.y * 32;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        int m = m0 + ty + 8 * j, i = i0 + tx;
        tile[ty + 8 * j][tx] = (m < Kf && i < CRS) ? K[(size_t)m * CRS + i] : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; j++) {
        int i = i0 + ty + 8 * j, m = m0 + tx;
        if (i < CRSp && m < Mp) Wp[(size_t)i * Mp + m] = tile[tx][ty + 8 * j];
    }
}

// ---------------------------------------------------------------- implicit GEMM, fp32 MFMA
template <int WM, int WN, int TM, int TN, int R_, int S_>
__global__ __launch_bounds__(256) void conv_igemm_kernel(const ConvParams p) {
    static_assert(WM * WN == 4, "four wavefronts per workgroup");
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    constexpr int LDA = BM + 32, LDB = BN + 32;  // +32 floats: the two half-wavefronts of an operand read hit different banks
    constexpr int AV = BM >= 64 ? BM / 64 : 1;   // float4 filter loads per thread per step
    constexpr int A_VECS = BK * BM / 4;          // float4 in one filter slice (fewer than 256 when BM = 32)
    constexpr int EPT = BN / 16;                 // gathered input elements per thread per step
    static_assert(BN >= 64, "a wavefront gathers one tap row slice");

    __shared__ __attribute__((aligned(16))) float As[2][BK * LDA];
    __shared__ __attribute__((aligned(16))) float Bs[2][BK * LDB];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int R = R_ ? R_ : p.R, S = S_ ? S_ : p.S, RS = R * S;

    // workgroup id -> tile, XCD-contiguous
    int vid;
    {
        const unsigned total = gridDim.x, bid = blockIdx.x;
        const unsigned q = total / EDDLHIP_NUM_XCD, r = total % EDDLHIP_NUM_XCD;
        const unsigned xcd = bid % EDDLHIP_NUM_XCD, slot = bid / EDDLHIP_NUM_XCD;
        vid = (int)((xcd < r ? xcd * (q + 1) : r * (q + 1) + (xcd - r) * q) + slot);
    }
    const int m_tile = vid % p.gm, n_tile = vid / p.gm;
    const int m0 = m_tile * BM;
    const long long n0 = (long long)n_tile * BN;

    // ---- this thread's gathered pixel (fixed for the whole kernel)
    const int bn_l = tid % BN;
    const int bg = __builtin_amdgcn_readfirstlane(tid / BN);  // tap group, uniform in a wavefront
    const long long ng = n0 + bn_l;
    const bool pvalid = ng < p.npix;
    int ih0, iw0;
    const float *in_img;
    {
        const long long ngc = pvalid ? ng : 0;
        const int img = (int)(ngc / p.PQ);
        const int pq = (int)(ngc - (long long)img * p.PQ);
        const int op = pq / p.Q, oq = pq - op * p.Q;
        ih0 = op * p.sr - p.pt;
        iw0 = oq * p.sc - p.pl;
        in_img = p.I + (size_t)img * p.C * p.H * p.W;
    }

    float4 areg[AV];
    float breg[EPT];

    auto load_a = [&](int step) {
#pragma unroll
        for (int j = 0; j < AV; j++) {
            const int f = tid + j * 256;
            const int kk = f / (BM / 4), m4 = (f % (BM / 4)) * 4;
            if (f < A_VECS) areg[j] = *reinterpret_cast<const float4 *>(p.Wp + (size_t)(step * BK + kk) * p.Mp + m0 + m4);
        }
    };
    auto load_b = [&](int step) {
        int i = step * BK + bg * EPT;
        int c = i / RS;
        int rem = i - c * RS;
        int ky = rem / S, kx = rem - ky * S;
#pragma unroll
        for (int e = 0; e < EPT; e++) {
            const int ih = ih0 + ky, iw = iw0 + kx;
            const bool ok = pvalid && c < p.C && (unsigned)ih < (unsigned)p.H && (unsigned)iw < (unsigned)p.W;
            float v = 0.0f;
            if (ok) v = in_img[((size_t)c * p.H + ih) * p.W + iw];
            breg[e] = v;
            if (++kx == S) {
                kx = 0;
                if (++ky == R) {
                    ky = 0;
                    ++c;
                }
            }
        }
    };
    auto store_ab = [&](int buf) {
#pragma unroll
        for (int j = 0; j < AV; j++) {
            const int f = tid + j * 256;
            const int kk = f / (BM / 4), m4 = (f % (BM / 4)) * 4;
            if (f < A_VECS) *reinterpret_cast<float4 *>(&As[buf][kk * LDA + m4]) = areg[j];
        }
#pragma unroll
        for (int e = 0; e < EPT; e++) Bs[buf][(bg * EPT + e) * LDB + bn_l] = breg[e];
    };

    floatx16 acc[TM][TN];
#pragma unroll
    for (int tm = 0; tm < TM; tm++)
#pragma unroll
        for (int tn = 0; tn < TN; tn++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[tm][tn][v] = 0.0f;

    load_a(0);
    load_b(0);
    store_ab(0);
    __syncthreads();

    const int a_off = (lane >> 5) * LDA + wm * TM * 32 + (lane & 31);
    const int b_off = (lane >> 5) * LDB + wn * TN * 32 + (lane & 31);

    for (int step = 0; step < p.nsteps; step++) {
        const int buf = step & 1;
        const bool more = step + 1 < p.nsteps;
        if (more) {
            load_a(step + 1);
            load_b(step + 1);
        }
#pragma unroll
        for (int ks = 0; ks < BK / 2; ks++) {
            float a[TM], b[TN];
#pragma unroll
            for (int tm = 0; tm < TM; tm++) a[tm] = As[buf][ks * 2 * LDA + a_off + tm * 32];
#pragma unroll
            for (int tn = 0; tn < TN; tn++) b[tn] = Bs[buf][ks * 2 * LDB + b_off + tn * 32];
#pragma unroll
            for (int tm = 0; tm < TM; tm++)
#pragma unroll
                for (int tn = 0; tn < TN; tn++)
                    acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[tm], b[tn], acc[tm][tn], 0, 0, 0);
        }
        if (more) store_ab(buf ^ 1);
        __syncthreads();
    }

    // ---- store: lane holds column (pixel) lane%32 and rows 8*(v/4) + 4*(lane/32) + v%4 of each 32x32 block
#pragma unroll
    for (int tn = 0; tn < TN; tn++) {
        const long long n = n0 + wn * TN * 32 + tn * 32 + (lane & 31);
        if (n >= p.npix) continue;
        const int img = (int)(n / p.PQ);
        const int pq = (int)(n - (long long)img * p.PQ);
        const size_t obase = (size_t)img * p.Kf * p.PQ + pq;
#pragma unroll
        for (int tm = 0; tm < TM; tm++) {
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = m0 + wm * TM * 32 + tm * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
                if (m < p.Kf) {
                    const ChannelEpilogue e = load_channel(p, m);
                    const size_t oidx = obase + (size_t)m * p.PQ;
                    p.O[oidx] = apply_epilogue(p, e, acc[tm][tn][v], oidx);
                }
            }
        }
    }
}

// ---------------------------------------------------------------- scalar direct kernel
// One thread per output, taps in the order ky, kx, c with a separate multiply and add per tap
// (src/hardware/cpu/nn/cpu_conv.cpp:282-314).  Slow; exists to check the MFMA kernels on the
// device and as a fallback nobody selects automatically.
__global__ __launch_bounds__(256) void conv_direct_kernel(const ConvParams p) {
    const size_t total = (size_t)p.npix * p.Kf;
    size_t t0 = (size_t)blockIdx.x * 256 + threadIdx.x, stride = (size_t)gridDim.x * 256;
    for (size_t o = t0; o < total; o += stride) {
        const int q = (int)(o % p.Q);
        size_t r = o / p.Q;
        const int pp = (int)(r % p.P);
        r /= p.P;
        const int k = (int)(r % p.Kf);
        const int b = (int)(r / p.Kf);
        const float *img = p.I + (size_t)b * p.C * p.H * p.W;
        const float *flt = p.K + (size_t)k * p.C * p.R * p.S;
        float s = 0.0f;
        for (int x = 0; x < p.R; x++) {
            const int px = pp * p.sr + x - p.pt;
            if (px < 0 || px >= p.H) continue;
            for (int y = 0; y < p.S; y++) {
                const int py = q * p.sc + y - p.pl;
                if (py < 0 || py >= p.W) continue;
                for (int c = 0; c < p.C; c++)
                    s = __fadd_rn(s, __fmul_rn(flt[((size_t)c * p.R + x) * p.S + y], img[((size_t)c * p.H + px) * p.W + py]));
            }
        }
        const ChannelEpilogue e = load_channel(p, k);
        p.O[o] = apply_epilogue(p, e, s, o);
    }
}

int g_algo = 0;
hipEvent_t g_prof_start = nullptr, g_prof_stop = nullptr;  // optional: bracket the main kernel of the next calls

template <int WM, int WN, int TM, int TN>
int launch_igemm(hipStream_t st, ConvParams &p) {
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    p.gm = (p.Kf + BM - 1) / BM;
    long long gn = (p.npix + BN - 1) / BN;
    EH_REQUIRE(gn * p.gm <= 0x7fffffffLL, "conv2d: too many tiles");
    p.gn = (int)gn;
    dim3 grid((unsigned)(gn * p.gm)), block(256);
    if (g_prof_start) EH_TRY_HIP(hipEventRecord(g_prof_start, st));
    if (p.R == 3 && p.S == 3) hipLaunchKernelGGL((conv_igemm_kernel<WM, WN, TM, TN, 3, 3>), grid, block, 0, st, p);
    else if (p.R == 1 && p.S == 1) hipLaunchKernelGGL((conv_igemm_kernel<WM, WN, TM, TN, 1, 1>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((conv_igemm_kernel<WM, WN, TM, TN, 0, 0>), grid, block, 0, st, p);
    EH_CHECK_LAUNCH();
    if (g_prof_stop) EH_TRY_HIP(hipEventRecord(g_prof_stop, st));
    return 0;
}

}  // namespace

extern "C" {

int eddlhip_conv2d_set_algo(int algo) {
    EH_REQUIRE(algo >= 0 && algo <= 2, "conv2d_set_algo: unknown algorithm %d", algo);
    g_algo = algo;
    return 0;
}

int eddlhip_conv2d_set_profile_events(void *start, void *stop) {
    EH_REQUIRE((start == nullptr) == (stop == nullptr), "conv2d_set_profile_events: give both events or neither");
    g_prof_start = (hipEvent_t)start;
    g_prof_stop = (hipEvent_t)stop;
    return 0;
}

int eddlhip_conv2d_fwd(int dev, const float *I, const float *K, const float *bias, float *O, int N, int C, int H, int W, int Kf,
                       int R, int S, int sr, int sc, int pad_top, int pad_left, int P, int Q, const float *bn_g, const float *bn_b,
                       const float *bn_mean, const float *bn_var, float bn_eps, const float *residual, int relu) {
    EH_REQUIRE(N >= 0 && C > 0 && H > 0 && W > 0, "conv2d: bad input shape %dx%dx%dx%d", N, C, H, W);
    EH_REQUIRE(Kf > 0 && R > 0 && S > 0, "conv2d: bad filter shape %dx%dx%dx%d", Kf, C, R, S);
    EH_REQUIRE(sr > 0 && sc > 0, "conv2d: strides must be positive");
    EH_REQUIRE(P > 0 && Q > 0, "conv2d: invalid output shape (%d x %d)", P, Q);
    EH_REQUIRE(pad_top >= 0 && pad_left >= 0, "conv2d: negative padding");
    EH_REQUIRE((bn_mean == nullptr) == (bn_var == nullptr), "conv2d: bn_mean and bn_var must come together");
    EH_REQUIRE((bn_g == nullptr) == (bn_b == nullptr), "conv2d: bn_g and bn_b must come together");
    EH_REQUIRE(bn_g == nullptr || bn_mean != nullptr, "conv2d: affine parameters without statistics");
    EH_REQUIRE((long long)C * H * W <= 0x7fffffffLL && (long long)C * R * S <= 0x7fffff00LL, "conv2d: image or filter too large");
    EH_REQUIRE((long long)P * Q <= 0x7fffffffLL, "conv2d: output plane too large");
    if (N == 0) return 0;
    EH_REQUIRE(I && K && O, "conv2d: NULL tensor");
    EH_TRY(use_device(dev));
    hipStream_t st = state(dev).stream;

    ConvParams p;
    p.I = I; p.K = K; p.O = O; p.Wp = nullptr;
    p.bias = bias; p.bn_g = bn_g; p.bn_b = bn_b; p.bn_mean = bn_mean; p.bn_var = bn_var; p.residual = residual;
    p.bn_eps = bn_eps; p.relu = relu;
    p.N = N; p.C = C; p.H = H; p.W = W; p.Kf = Kf; p.R = R; p.S = S; p.sr = sr; p.sc = sc; p.pt = pad_top; p.pl = pad_left;
    p.P = P; p.Q = Q;
    p.CRS = C * R * S;
    p.PQ = P * Q;
    p.npix = (long long)N * P * Q;
    p.gm = p.gn = 0;
    p.nsteps = (p.CRS + BK - 1) / BK;
    p.Mp = (Kf + M_ALIGN - 1) / M_ALIGN * M_ALIGN;

    if (g_algo == 2) {
        size_t total = (size_t)p.npix * Kf;
        hipLaunchKernelGGL(conv_direct_kernel, dim3(eh_blocks(total, 256, 1u << 20)), dim3(256), 0, st, p);
        EH_CHECK_LAUNCH();
        return 0;
    }

    // repack the filters (tap-major, zero-padded) into the private workspace
    const int CRSp = p.nsteps * BK;
    void *ws = nullptr;
    EH_TRY(get_workspace(dev, (size_t)CRSp * p.Mp * sizeof(float), &ws));
    p.Wp = (const float *)ws;
    hipLaunchKernelGGL(pack_filters_kernel, dim3((CRSp + 31) / 32, p.Mp / 32), dim3(256), 0, st, K, (float *)ws, Kf, p.CRS, p.Mp, CRSp);
    EH_CHECK_LAUNCH();

    // tile choice: the largest tile that still gives every CU about two workgroups
    const long long want = 2LL * state(dev).num_cu;
    auto tiles = [&](int bm, int bn) { return (long long)((Kf + bm - 1) / bm) * ((p.npix + bn - 1) / bn); };
    if (Kf > 64 && tiles(128, 128) >= want) return launch_igemm<2, 2, 2, 2>(st, p);
    if (Kf > 32 && tiles(64, 128) >= want) return launch_igemm<1, 4, 2, 1>(st, p);
    if (Kf > 32) return launch_igemm<2, 2, 1, 1>(st, p);
    return launch_igemm<1, 4, 1, 1>(st, p);
}

}  // extern "C"

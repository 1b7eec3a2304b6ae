// Conv2D forward for gfx950: implicit GEMM on the fp32 matrix cores, no materialised
// lowering buffer, bias / inference batch-norm / residual add / ReLU fused into the store.
//
// GEMM view (the reference lowers to the same product, src/hardware/cpu/nn/cpu_conv.cpp:55-112,
// 210-223, but materialises the lowered matrix):
//     O[m][n] = sum_i  Wt[i][m] * Col[i][n]
//     m = output channel, n = flattened (image, p, q) output pixel,
//     i = (c, ky, kx) tap, c slowest  - the order of OIHW filter memory.
// Col is never stored: each workgroup gathers the BK x BN slice it needs straight from the
// NCHW input into LDS.  The gather uses buffer loads: a tap that falls outside the image gets
// an out-of-range offset and the hardware returns 0 for it - no branch, no select.  Filters are
// repacked once per call into a tap-major, zero-padded matrix Wp[i][m] (private workspace) so
// that the filter slice of a tile is BK rows of contiguous floats (16-byte loads).
//
// Tile: BM x BN outputs per 256-thread workgroup (4 wavefronts), LDS double-buffered (one
// barrier per K-step), loads of step t+1 issued before the MFMAs of step t.  Each wavefront
// owns TM x TN blocks of 32x32 outputs and advances them with v_mfma_f32_32x32x2_f32
// (A = 32 channels x 2 taps, B = 2 taps x 32 pixels).
//
// Two kernels:
//   conv_tap_kernel  filter shape known at compile time (3x3, 1x1, 2x2): a K-step is CPB whole
//                    input channels; every thread gathers ONE fixed output pixel, so the R*S
//                    tap offsets (and their validity) are computed once, before the loop, and
//                    the per-step address work is one scalar offset per channel.  By default
//                    both operand slices go global -> LDS directly (buffer_load ... lds),
//                    skipping the register file; a register-staged form is kept for checking.
//   conv_gen_kernel  any filter shape, K-step 16 taps.  What a tap needs (its byte offset from
//                    the window origin, its channel's byte offset, its row and column in the
//                    filter) comes from a table written once per call and read with scalar
//                    loads, so a gathered element costs two bounds tests and one address add.
//                    Same LDS-direct loads as conv_tap_kernel.
//
// Accumulation order per output: taps in increasing i, two per MFMA (the instruction adds
// both products of a pair into the fp32 accumulator), one accumulator from the first tap to
// the last.  Tiles the launch plan divides along K (plan_conv) are summed slice by slice in
// increasing K order by conv_reduce_kernel: a fixed order too.  The reference CPU order is ky,kx,c per output in its direct
// form and Eigen-internal in its GEMM form, so agreement is to a tolerance, not bit-for-bit;
// the scalar kernel at the end of this file follows the direct form's order and rounding.
//
// Workgroups are numbered so that those running on one XCD (workgroup id mod 8) cover
// neighbouring pixel tiles for all channel tiles: the input slice they share stays in that
// XCD's L2.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <mutex>
#include <utility>
#include <vector>

#include "common.h"

using namespace eddlhip;

// Device memory of eddlhip_conv2d_fwd_noalloc: what eddlhip_conv2d_fwd takes from the library's grow-only
// workspace (repacked filters, tap table, partial tiles of a K-split launch) comes out of this fixed array
// instead, so that entry point never allocates.  Each device the library runs on holds its own copy, at its
// own address, until the process ends.  In host code the name is only a handle for hipGetSymbolAddress:
// conv_setup_device asks for the device address once per device and everything else uses that pointer.
static __device__ __align__(256) unsigned char scratch[EDDLHIP_CONV_NOALLOC_SCRATCH_BYTES];

namespace {

void *g_scratch_ptr[EDDLHIP_MAX_DEVICES];  // device address of `scratch` on each initialised device

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(3))) float lds_float;

constexpr int M_ALIGN = 128;                  // packed filter rows are padded to this many channels
constexpr int OOB = (int)0x80000000u;         // byte offset no buffer of <= 2 GiB contains
constexpr unsigned RSRC_WORD3 = 0x00020000u;  // raw buffer, 32-bit data format

typedef int int32x4 __attribute__((ext_vector_type(4)));

struct ConvParams {
    const float *I;
    // Two-tensor input (a channel Concat folded into the convolution): channels [0, Csplit) come from I,
    // channels [Csplit, C) from I2, both tensors holding Cimg = Csplit = C - Csplit channels per image.
    // One tensor: I2 == I, Csplit == C, Cimg == C.
    const float *I2;
    int Csplit, Cimg;
    // Nearest-neighbour upsampling folded into the gather: the convolution sees an image of H*uh x W*uw pixels
    // whose pixel (y, x) is the stored pixel (y / uh, x / uw).  uh == uw == 1: the stored image itself.
    int uh, uw;
    const float *Wp;  // packed filters [rows][Mp]
    // Image n of the launch multiplies by the packed matrix at Wp + n * w_img_stride (floats): 0 for a convolution (one
    // matrix for all images); the 16 products of a Winograd convolution run as ONE 1x1 launch over 16 "images", one
    // transformed filter matrix each (an image's pixel count is then a multiple of every tile width, so that no tile
    // holds pixels of two images).  conv_tap_kernel only.
    size_t w_img_stride;
    const float *K;   // original OIHW filters (scalar kernel only)
    float *O;
    const float *bias, *bn_g, *bn_b, *bn_mean, *bn_var, *residual;
    float bn_eps;
    int relu;
    // The output is written with the streaming (non-temporal) hint: set by the host for a layer that is bound by its
    // output traffic and whose output is larger than the last-level cache, so that keeping it there helps no reader.
    int stream_out;
    int N, C, H, W, Kf, R, S, sr, sc, pt, pl, P, Q;
    int CRS, Mp, nsteps, PQ;
    long long npix;
    int gm, gn;
    unsigned in_bytes, wp_bytes;  // sizes the input's and the packed filters' buffer descriptors cover
    // The first main_tiles workgroups of a launch compute one whole tile each (tiles 0..main_tiles-1).
    // The workgroups after them divide the remaining tiles along K: nslices workgroups per tile, of
    // slice_steps K-steps each, which write their raw accumulators to `partial`; conv_reduce_kernel
    // adds the slices and finishes those tiles.
    int main_tiles, nslices, slice_steps;
    float *partial;
    // conv_gen_kernel only: one entry per tap of the padded K range (tap_table_kernel)
    const int32x4 *taps;
    // eddlhip_conv2d_trace: eight 64-bit words per workgroup (see trace_mark), or nullptr
    unsigned long long *trace;
    // conv_tap_kernel<..., WINO = true> (the 16 products of a Winograd convolution and its output transform in one
    // launch): the K range is 16 runs of wspx steps, one per patch position; a pixel of the launch is a 2x2 block of the
    // wP x wQ output planes, wth x wtw of them per image, wT in all (see wino_fold / wino_store_tile).
    int wspx, wth, wtw, wT, wP, wQ;
    int wps;  // patch side: 4 (3x3 filters, 16 positions) or 3 (2x2 filters, 9 positions)
    // The Winograd epilogues only (a lane holds whole 2x2 blocks of outputs there; output planes with even sides): the
    // 2x2, stride-2 max-pool of the finished outputs with the coordinates of each maximum (the arithmetic of
    // maxpool_2x2s2_kernel), written next to the outputs - or instead of them when O is nullptr.
    float *pool_O, *pool_ix, *pool_iy;
};

// One 2x2 window of finished outputs (x00 x01 / x10 x11 at rows 2 ty, 2 ty + 1 and columns 2 tx, 2 tx + 1) pooled as
// eddlhip_maxpool2d does it: running maximum from -3.40282e38 in the order of the window scan, strictly greater wins,
// and when nothing is greater (a window of NaN) the coordinates are left as they are.
__device__ __forceinline__ void pool_block(const ConvParams &p, size_t pidx, int ty, int tx, float x00, float x01, float x10, float x11) {
    float mx = -3.40282e+38f, fx = 0.0f, fy = 0.0f;
    bool found = false;
    const float x0 = (float)(2 * tx), y0 = (float)(2 * ty);
    if (x00 > mx) { mx = x00; fx = x0; fy = y0; found = true; }
    if (x01 > mx) { mx = x01; fx = x0 + 1.0f; fy = y0; found = true; }
    if (x10 > mx) { mx = x10; fx = x0; fy = y0 + 1.0f; found = true; }
    if (x11 > mx) { mx = x11; fx = x0 + 1.0f; fy = y0 + 1.0f; found = true; }
    p.pool_O[pidx] = mx;
    if (found) {
        p.pool_ix[pidx] = fx;
        p.pool_iy[pidx] = fy;
    }
}

// Timeline of a workgroup for eddlhip_conv2d_trace: words 0..3 = the device's constant 100 MHz clock at the marks (entry,
// operands of the first K-step in LDS, end of the K loop, end of the kernel with its stores drained), word 4 = where the
// workgroup runs (HW_ID register in the low half, XCC_ID in the high half), words 5 and 6 = the shader clock at the
// first and the last mark (their difference over that of words 0 and 3 is the engine clock).
__device__ __forceinline__ void trace_mark(const ConvParams &p, int slot) {
    if (p.trace != nullptr && threadIdx.x == 0) {
        unsigned long long *w = p.trace + (size_t)blockIdx.x * 8;
        if (slot == 0) {
            w[4] = (unsigned long long)__builtin_amdgcn_s_getreg(0xF804) | ((unsigned long long)__builtin_amdgcn_s_getreg(0xF814) << 32);
            w[5] = __builtin_readcyclecounter();
        }
        if (slot == 3) w[6] = __builtin_readcyclecounter();
        w[slot] = __builtin_amdgcn_s_memrealtime();
    }
}

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

// LDS-direct load: the load unit writes the dword of lane i to LDS address dst + 4*i (out-of-range
// lanes write 0).  Written as inline assembly on purpose: the compiler's wait-count insertion
// makes every LDS read wait for ALL outstanding LDS-direct loads (it cannot tell the buffer being
// filled from the buffer being read), which would serialise the loads of step t+1 with the MFMAs
// of step t.  With the instruction opaque to it, the kernel places the one wait that is needed
// itself: vmcnt(0) before the barrier that publishes the buffer.
// The statements write M0 without declaring it: the compiler treats M0 as a reserved register, warns about it in
// a clobber list and does not promise to honour it there.  Its own uses of M0 (indexed register access, message
// sends, its LDS-direct builtin) set the register immediately before the instruction that reads it, and the
// kernels of this file contain none of them between these statements (every register array is indexed by
// compile-time constants after unrolling).
__device__ __forceinline__ int32x4 make_rsrc_words(const void *base, unsigned bytes) {
    const unsigned long long a = (unsigned long long)base;
    int32x4 r;
    r.x = __builtin_amdgcn_readfirstlane((int)(a & 0xffffffffu));
    r.y = __builtin_amdgcn_readfirstlane((int)((a >> 32) & 0xffffu));  // stride 0
    r.z = __builtin_amdgcn_readfirstlane((int)bytes);
    r.w = (int)RSRC_WORD3;
    return r;
}

__device__ __forceinline__ void lds_dma_b32(int32x4 rsrc, lds_float *dst, int voffset, int soffset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
                 :
                 : "s"((unsigned)(unsigned long long)dst), "v"(voffset), "s"(rsrc), "s"(soffset)
                 : "memory");
}

// 16 bytes per lane: lane l's four floats land at dst + 4*l .. 4*l + 3 (1 KB per wavefront instruction)
__device__ __forceinline__ void lds_dma_b128(int32x4 rsrc, lds_float *dst, int voffset, int soffset) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"((unsigned)(unsigned long long)dst), "v"(voffset), "s"(rsrc), "s"(soffset)
                 : "memory");
}

__device__ __forceinline__ float buf_load(__amdgpu_buffer_rsrc_t r, int voffset, int soffset) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voffset, soffset, 0));
}

// workgroup id -> (channel tile, pixel tile, K slice); ids that share an XCD get consecutive tiles.
// Workgroups are dealt to the XCDs round-robin by id, so within each of the two groups of a launch
// (whole tiles, then K slices) the ids that are congruent modulo the XCD count share an XCD.
__device__ __forceinline__ void tile_of_block(const ConvParams &p, int &m_tile, int &n_tile, int &local_tile, int &slice, bool &split) {
    unsigned total = (unsigned)p.main_tiles, bid = blockIdx.x;
    split = bid >= total;
    if (split) {
        bid -= total;
        total = gridDim.x - total;
    }
    const unsigned q = total / EDDLHIP_NUM_XCD, r = total % EDDLHIP_NUM_XCD;
    const unsigned xcd = bid % EDDLHIP_NUM_XCD, slot = bid / EDDLHIP_NUM_XCD;
    const int vid = (int)((xcd < r ? xcd * (q + 1) : r * (q + 1) + (xcd - r) * q) + slot);
    int tile;
    if (split) {
        slice = vid % p.nslices;
        local_tile = vid / p.nslices;
        tile = p.main_tiles + local_tile;
    } else {
        slice = 0;
        local_tile = vid;
        tile = vid;
    }
    m_tile = tile % p.gm;
    n_tile = tile / p.gm;
}

// Raw accumulators of one K slice of one tile, laid out [slice][tile][wave][block][v][lane] so
// that every store instruction of a wavefront writes 256 contiguous bytes.
template <int TM, int TN>
__device__ __forceinline__ void store_partial(const ConvParams &p, floatx16 (&acc)[TM][TN], int local_tile, int slice, int wave,
                                              int lane) {
    const size_t tiles = (gridDim.x - (unsigned)p.main_tiles) / p.nslices;
    float *dst = p.partial + (((size_t)slice * tiles + local_tile) * 4 + wave) * (TM * TN * 16 * 64) + lane;
#pragma unroll
    for (int tm = 0; tm < TM; tm++)
#pragma unroll
        for (int tn = 0; tn < TN; tn++)
#pragma unroll
            for (int v = 0; v < 16; v++) dst[((tm * TN + tn) * 16 + v) * 64] = acc[tm][tn][v];
}

// The per-channel constants of a tile's BM channels reach the epilogue through LDS (layout:
// bias[BM], mean[BM], sd[BM], g[BM], b[BM]).  Thread t < BM fetches those of channel m0 + t at the
// START of the kernel, so that their memory latency passes during the K loop instead of standing
// between the last MFMA and the first store, and writes them to LDS after the loop; the caller
// synchronises before and after that write.
template <int BM>
__device__ __forceinline__ ChannelEpilogue fetch_channel_constants(const ConvParams &p, int m0, int tid) {
    ChannelEpilogue e = {0.0f, 0.0f, 1.0f, 1.0f, 0.0f};
    if (tid < BM && m0 + tid < p.Kf) e = load_channel(p, m0 + tid);
    return e;
}
template <int BM>
__device__ __forceinline__ void put_channel_constants(float *epi, const ChannelEpilogue &e, int tid) {
    if (tid < BM) {
        epi[tid] = e.bias;
        epi[BM + tid] = e.mean;
        epi[2 * BM + tid] = e.sd;
        epi[3 * BM + tid] = e.g;
        epi[4 * BM + tid] = e.b;
    }
}
template <int BM>
__device__ __forceinline__ void stage_channel_constants(const ConvParams &p, float *epi, int m0, int tid) {
    put_channel_constants<BM>(epi, fetch_channel_constants<BM>(p, m0, tid), tid);
}

// The common case of store_tile below: every row and every pixel of the wavefront's blocks exists.
// No per-value bounds tests; one 64-bit address per pixel column, advanced by whole channel planes;
// the channel constants of four consecutive rows come from LDS in one read; which of batch norm,
// affine, residual and ReLU apply is decided once per group of four rows (the flags are the same for
// every lane) instead of once per value.  The arithmetic per value is that of store_tile, step by step.
template <int TM, int TN, int BM, bool HAS_RES>
__device__ __forceinline__ void store_tile_inside(const ConvParams &p, floatx16 (&acc)[TM][TN], const float *epi, int m0, int m_local,
                                                  int n_base, int lane) {
    const int half = lane >> 5;
    float *optr[TN];
    const float *rptr[TN];
    const size_t plane = (size_t)p.PQ;
#pragma unroll
    for (int tn = 0; tn < TN; tn++) {
        const unsigned n = (unsigned)(n_base + tn * 32 + (lane & 31));
        const unsigned img = n / (unsigned)p.PQ;
        const unsigned pq = n - img * (unsigned)p.PQ;
        const size_t idx = ((size_t)img * p.Kf + (size_t)(m0 + m_local + 4 * half)) * plane + pq;
        optr[tn] = p.O + idx;
        rptr[tn] = p.residual + idx;  // not dereferenced without a residual
    }
    const bool has_bias = p.bias != nullptr, has_bn = p.bn_mean != nullptr, affine = p.bn_g != nullptr;
    constexpr bool has_res = HAS_RES;
    const bool relu = p.relu != 0, stream_out = p.stream_out != 0;
#pragma unroll
    for (int tm = 0; tm < TM; tm++) {
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {  // rows 8*q4 + 4*half + 0..3 of the block: v = 4*q4 + j
            const int row0 = m_local + tm * 32 + 8 * q4 + 4 * half;
            const size_t roff = (size_t)(tm * 32 + 8 * q4) * plane;
            float res[4][TN];
            if constexpr (has_res) {
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int tn = 0; tn < TN; tn++) res[j][tn] = rptr[tn][roff + (size_t)j * plane];
            }
            float x[4][TN];
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int tn = 0; tn < TN; tn++) x[j][tn] = acc[tm][tn][4 * q4 + j];
            if (has_bias) {
                const floatx4 bias = *reinterpret_cast<const floatx4 *>(epi + row0);
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int tn = 0; tn < TN; tn++) x[j][tn] = __fadd_rn(x[j][tn], bias[j]);
            }
            if (has_bn) {
                const floatx4 mean = *reinterpret_cast<const floatx4 *>(epi + BM + row0);
                const floatx4 sd = *reinterpret_cast<const floatx4 *>(epi + 2 * BM + row0);
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int tn = 0; tn < TN; tn++) x[j][tn] = __fdiv_rn(__fsub_rn(x[j][tn], mean[j]), sd[j]);
                if (affine) {
                    const floatx4 g = *reinterpret_cast<const floatx4 *>(epi + 3 * BM + row0);
                    const floatx4 b = *reinterpret_cast<const floatx4 *>(epi + 4 * BM + row0);
#pragma unroll
                    for (int j = 0; j < 4; j++)
#pragma unroll
                        for (int tn = 0; tn < TN; tn++) x[j][tn] = __fadd_rn(__fmul_rn(x[j][tn], g[j]), b[j]);
                }
            }
            if constexpr (has_res) {
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int tn = 0; tn < TN; tn++) x[j][tn] = __fadd_rn(x[j][tn], res[j][tn]);
            }
            if (relu) {
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int tn = 0; tn < TN; tn++) x[j][tn] = x[j][tn] > 0.0f ? x[j][tn] : 0.0f;
            }
            if (stream_out) {
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int tn = 0; tn < TN; tn++) __builtin_nontemporal_store(x[j][tn], optr[tn] + roff + (size_t)j * plane);
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int tn = 0; tn < TN; tn++) optr[tn][roff + (size_t)j * plane] = x[j][tn];
            }
        }
    }
}

// Writes a wavefront's TM x TN blocks.  A lane holds column (pixel) lane%32 and rows
// 8*(v/4) + 4*(lane/32) + v%4 of each 32x32 block: for a fixed v the 32 lanes of a half
// wavefront store 32 consecutive pixels of one channel plane (128 contiguous bytes).
// `epi` holds the tile's channel constants (stage_channel_constants); m_local is the first of the
// wavefront's rows within the tile.  The residual values of a 32-row block are all requested
// before the first of them is used, so their latencies overlap.
// (The residual's presence is a template parameter of the two bodies so that the loads of the residual values and their
// uses sit in one branch: a kernel that goes on to further work after a tile then carries no load that looks pending.)
template <int TM, int TN, int BM, bool HAS_RES>
__device__ __forceinline__ void store_tile_edge(const ConvParams &p, floatx16 (&acc)[TM][TN], const float *epi, int m0, int m_local, int n_base,
                                                int lane);

template <int TM, int TN, int BM>
__device__ __forceinline__ void store_tile(const ConvParams &p, floatx16 (&acc)[TM][TN], const float *epi, int m0, int m_local, int n_base,
                                           int lane) {
    if (m0 + m_local + TM * 32 <= p.Kf && (long long)n_base + TN * 32 <= p.npix) {
        if (p.residual != nullptr) store_tile_inside<TM, TN, BM, true>(p, acc, epi, m0, m_local, n_base, lane);
        else store_tile_inside<TM, TN, BM, false>(p, acc, epi, m0, m_local, n_base, lane);
        return;
    }
    if (p.residual != nullptr) store_tile_edge<TM, TN, BM, true>(p, acc, epi, m0, m_local, n_base, lane);
    else store_tile_edge<TM, TN, BM, false>(p, acc, epi, m0, m_local, n_base, lane);
}

template <int TM, int TN, int BM, bool HAS_RES>
__device__ __forceinline__ void store_tile_edge(const ConvParams &p, floatx16 (&acc)[TM][TN], const float *epi, int m0, int m_local, int n_base,
                                                int lane) {
    size_t obase[TN];
    bool nok[TN];
#pragma unroll
    for (int tn = 0; tn < TN; tn++) {
        const int n = n_base + tn * 32 + (lane & 31);
        nok[tn] = n < (int)p.npix;
        const unsigned nc = nok[tn] ? (unsigned)n : 0u;
        const unsigned img = nc / (unsigned)p.PQ;
        const unsigned pq = nc - img * (unsigned)p.PQ;
        obase[tn] = (size_t)img * p.Kf * p.PQ + pq;
    }
    constexpr bool has_res = HAS_RES;
#pragma unroll
    for (int tm = 0; tm < TM; tm++) {
#pragma unroll
        for (int vh = 0; vh < 16; vh += 8) {  // eight rows at a time: their residual loads are in flight together
            float res[8][TN];
            if constexpr (has_res) {
#pragma unroll
                for (int vv = 0; vv < 8; vv++) {
                    const int v = vh + vv;
                    const int ml = m_local + tm * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
                    const bool mok = m0 + ml < p.Kf;
#pragma unroll
                    for (int tn = 0; tn < TN; tn++) {
                        const size_t oidx = (mok && nok[tn]) ? obase[tn] + (size_t)(m0 + ml) * p.PQ : 0;
                        res[vv][tn] = p.residual[oidx];
                    }
                }
            }
#pragma unroll
            for (int vv = 0; vv < 8; vv++) {
                const int v = vh + vv;
                const int ml = m_local + tm * 32 + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
                const bool mok = m0 + ml < p.Kf;
                const float bias = epi[ml], mean = epi[BM + ml], sd = epi[2 * BM + ml], g = epi[3 * BM + ml], b = epi[4 * BM + ml];
#pragma unroll
                for (int tn = 0; tn < TN; tn++) {
                    float x = acc[tm][tn][v];
                    if (p.bias) x = __fadd_rn(x, bias);
                    if (p.bn_mean) {
                        x = __fdiv_rn(__fsub_rn(x, mean), sd);
                        if (p.bn_g) x = __fadd_rn(__fmul_rn(x, g), b);
                    }
                    if constexpr (has_res) x = __fadd_rn(x, res[vv][tn]);
                    if (p.relu) x = x > 0.0f ? x : 0.0f;
                    if (mok && nok[tn]) p.O[obase[tn] + (size_t)(m0 + ml) * p.PQ] = x;
                }
            }
        }
    }
}

// ---------------------------------------------------------------- filter repack
// K[Kf][CRS] (OIHW memory) -> Wp[rows][Mp], zero-padded; 32x32 tiles through LDS so that
// both the read and the write are coalesced.
__global__ __launch_bounds__(256) void pack_filters_kernel(const float *__restrict__ K, float *__restrict__ Wp, int Kf, int CRS,
                                                           int Mp, int rows) {
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
        if (i < rows && m < Mp) Wp[(size_t)i * Mp + m] = tile[tx][ty + 8 * j];
    }
}

// ---------------------------------------------------------------- Winograd output transform inside the product launch
// Y = A^T M A with A^T = [1 1 1 0; 0 1 -1 -1]: the product M of patch position xi = 4 i + j reaches output (a, b) of the
// 2x2 block with the factor A^T[a][i] * A^T[b][j], which is 0, 1 or -1.  A workgroup that walks through all 16 positions
// therefore needs no M tensor: after the K run of a position it adds the accumulator into four running outputs, with
// those signs, and clears it.  Positions are taken in the order 0..15, so the sums are reproducible.
__device__ __forceinline__ void wino_fold(floatx16 (&y)[2][2], floatx16 &acc, int xi, int ps) {
    // ps = 4: A^T = [1 1 1 0; 0 1 -1 -1]; ps = 3 (2x2 filters): A^T = [1 1 0; 0 1 -1]
    const int i = xi / ps, j = xi - i * ps;
    const int ca[2] = {i < ps - 1 ? 1 : 0, i == 0 ? 0 : (i == 1 ? 1 : -1)};
    const int cb[2] = {j < ps - 1 ? 1 : 0, j == 0 ? 0 : (j == 1 ? 1 : -1)};
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++) {
            const int f = ca[a] * cb[b];  // the same for every lane
            if (f > 0) {
#pragma unroll
                for (int v = 0; v < 16; v++) y[a][b][v] = __fadd_rn(y[a][b][v], acc[v]);
            } else if (f < 0) {
#pragma unroll
                for (int v = 0; v < 16; v++) y[a][b][v] = __fsub_rn(y[a][b][v], acc[v]);
            }
        }
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = 0.0f;
}

// The 2x2 convolution of an image upsampled twice: output (2a + i, 2b + j) sees the stored pixels (a .. a + i, b .. b + j)
// only, each through the sum of the filter taps that land on it, so the four parities are four convolutions of the
// stored image with 1x1, 1x2, 2x1 and 2x2 filters - 9 multiplications per channel and block where the direct form has 16.
// The nine filter rows of channel c, U[9 c + r][column of filter m] (Mp columns, zero past Kf), from OIHW 2x2 filters:
// r = 0: (w00 + w01) + (w10 + w11) [output (0,0), tap 0]; 1, 2: w00 + w10, w01 + w11 [output (0,1), taps 0, 1];
// 3, 4: w00 + w01, w10 + w11 [output (1,0), taps 0, 2]; 5..8: w00, w01, w10, w11 [output (1,1), taps 0..3].
__global__ __launch_bounds__(256) void up2x2_filter_kernel(const float *__restrict__ K, float *__restrict__ U, int Kf, int C, int Mp) {
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)C * Mp) return;
    const int c = (int)(idx / Mp), m = (int)(idx - (size_t)c * Mp);
    float w00 = 0.0f, w01 = 0.0f, w10 = 0.0f, w11 = 0.0f;
    if (m < Kf) {
        const float *k = K + ((size_t)m * C + c) * 4;
        w00 = k[0], w01 = k[1], w10 = k[2], w11 = k[3];
    }
    const float r[9] = {__fadd_rn(__fadd_rn(w00, w01), __fadd_rn(w10, w11)), __fadd_rn(w00, w10), __fadd_rn(w01, w11), __fadd_rn(w00, w01), __fadd_rn(w10, w11),
                        w00, w01, w10, w11};
    // within each group of 64 filters (the tile of conv_up2x2_kernel) filter j of the first 32 and filter 32 + j sit side by side
    const int col = (m & ~63) + 2 * (m & 31) + ((m >> 5) & 1);
#pragma unroll
    for (int run = 0; run < 9; run++) U[((size_t)c * 9 + run) * Mp + col] = r[run];
}

// One filter row's four outputs of one 2x2 block (y00 y01 / y10 y11 at rows 2 ty, 2 ty + 1 and columns 2 tx, 2 tx + 1 of
// image `img`): the convolution's epilogue value by value (the arithmetic of apply_epilogue), two outputs of a row per
// store where the rows are aligned for it (`pair`), and the block's max-pool where one is asked for.  `e`: the channel
// constants of filter m.
__device__ __forceinline__ void wino_store_row(const ConvParams &p, const ChannelEpilogue &e, int m, int img, int ty, int tx, size_t plane, bool pair,
                                               float y00, float y01, float y10, float y11) {
    if (m >= p.Kf) return;
    const float bias = e.bias, mean = e.mean, sd = e.sd, g = e.g, b = e.b;
    const float yy[2][2] = {{y00, y01}, {y10, y11}};
    float fin[2][2] = {{0.0f, 0.0f}, {0.0f, 0.0f}};
#pragma unroll
    for (int a = 0; a < 2; a++) {
        const int oy = 2 * ty + a, ox = 2 * tx;
        if (oy >= p.wP) continue;
        const size_t oidx = ((size_t)img * p.Kf + (size_t)m) * plane + (size_t)oy * p.wQ + ox;
        float x0 = yy[a][0], x1 = yy[a][1];
        float r0 = 0.0f, r1 = 0.0f;
        if (p.residual) {
            if (pair) {
                const float2 rr = *reinterpret_cast<const float2 *>(p.residual + oidx);
                r0 = rr.x;
                r1 = rr.y;
            } else {
                r0 = p.residual[oidx];
                if (ox + 1 < p.wQ) r1 = p.residual[oidx + 1];
            }
        }
        if (p.bias) x0 = __fadd_rn(x0, bias), x1 = __fadd_rn(x1, bias);
        if (p.bn_mean) {
            x0 = __fdiv_rn(__fsub_rn(x0, mean), sd), x1 = __fdiv_rn(__fsub_rn(x1, mean), sd);
            if (p.bn_g) x0 = __fadd_rn(__fmul_rn(x0, g), b), x1 = __fadd_rn(__fmul_rn(x1, g), b);
        }
        if (p.residual) x0 = __fadd_rn(x0, r0), x1 = __fadd_rn(x1, r1);
        if (p.relu) x0 = x0 > 0.0f ? x0 : 0.0f, x1 = x1 > 0.0f ? x1 : 0.0f;
        fin[a][0] = x0;
        fin[a][1] = x1;
        if (p.O == nullptr) continue;
        if (pair) {
            *reinterpret_cast<float2 *>(p.O + oidx) = make_float2(x0, x1);
        } else {
            p.O[oidx] = x0;
            if (ox + 1 < p.wQ) p.O[oidx + 1] = x1;
        }
    }
    if (p.pool_O != nullptr)  // (even wP, wQ: both rows and both columns of the block exist)
        pool_block(p, (((size_t)img * p.Kf + (size_t)m) * p.wth + ty) * p.wtw + tx, ty, tx, fin[0][0], fin[0][1], fin[1][0], fin[1][1]);
}

// the constants of row ml of a tile as stage_channel_constants laid them out in LDS
template <int BM>
__device__ __forceinline__ ChannelEpilogue channel_from_lds(const float *epi, int ml) {
    ChannelEpilogue e;
    e.bias = epi[ml], e.mean = epi[BM + ml], e.sd = epi[2 * BM + ml], e.g = epi[3 * BM + ml], e.b = epi[4 * BM + ml];
    return e;
}

// NK (4 or 2) consecutive filter rows' outputs of one 2x2 block, x[k][a][b] = output (2 ty + a, 2 tx + b) of filter m + k -
// the common case of wino_store_row NK times over: all NK filters exist, the block lies inside the output plane, and the
// rows are aligned for 8-byte stores.  The arithmetic per value is wino_store_row's, step by step; which steps apply is
// decided once for the 4 NK values (the flags are the same for every lane), the channel constants of the rows come from
// LDS in one read each (`epi`: stage_channel_constants' layout, ml = the first row's place in the tile, a multiple of
// NK), one 64-bit address serves all stores, and the residual's loads are in flight together.
template <int BM, int NK>
__device__ __forceinline__ void wino_store_rows(const ConvParams &p, const float *epi, int ml, int m, int img, int ty, int tx, size_t plane,
                                                float (&x)[NK][2][2]) {
    static_assert(NK == 4 || NK == 2, "the constants of the rows are one 16-byte or one 8-byte read");
    typedef float vec_t __attribute__((ext_vector_type(NK)));
    const size_t o0 = ((size_t)img * p.Kf + (size_t)m) * plane + (size_t)(2 * ty) * p.wQ + 2 * tx;
    float2 rr[NK][2];
    if (p.residual) {
#pragma unroll
        for (int k = 0; k < NK; k++)
#pragma unroll
            for (int a = 0; a < 2; a++) rr[k][a] = *reinterpret_cast<const float2 *>(p.residual + o0 + (size_t)k * plane + (size_t)a * p.wQ);
    }
    if (p.bias) {
        const vec_t bias = *reinterpret_cast<const vec_t *>(epi + ml);
#pragma unroll
        for (int k = 0; k < NK; k++)
#pragma unroll
            for (int a = 0; a < 2; a++)
#pragma unroll
                for (int b = 0; b < 2; b++) x[k][a][b] = __fadd_rn(x[k][a][b], bias[k]);
    }
    if (p.bn_mean) {
        const vec_t mean = *reinterpret_cast<const vec_t *>(epi + BM + ml), sd = *reinterpret_cast<const vec_t *>(epi + 2 * BM + ml);
#pragma unroll
        for (int k = 0; k < NK; k++)
#pragma unroll
            for (int a = 0; a < 2; a++)
#pragma unroll
                for (int b = 0; b < 2; b++) x[k][a][b] = __fdiv_rn(__fsub_rn(x[k][a][b], mean[k]), sd[k]);
        if (p.bn_g) {
            const vec_t g = *reinterpret_cast<const vec_t *>(epi + 3 * BM + ml), bb = *reinterpret_cast<const vec_t *>(epi + 4 * BM + ml);
#pragma unroll
            for (int k = 0; k < NK; k++)
#pragma unroll
                for (int a = 0; a < 2; a++)
#pragma unroll
                    for (int b = 0; b < 2; b++) x[k][a][b] = __fadd_rn(__fmul_rn(x[k][a][b], g[k]), bb[k]);
        }
    }
    if (p.residual) {
#pragma unroll
        for (int k = 0; k < NK; k++)
#pragma unroll
            for (int a = 0; a < 2; a++) x[k][a][0] = __fadd_rn(x[k][a][0], rr[k][a].x), x[k][a][1] = __fadd_rn(x[k][a][1], rr[k][a].y);
    }
    if (p.relu) {
#pragma unroll
        for (int k = 0; k < NK; k++)
#pragma unroll
            for (int a = 0; a < 2; a++)
#pragma unroll
                for (int b = 0; b < 2; b++) x[k][a][b] = x[k][a][b] > 0.0f ? x[k][a][b] : 0.0f;
    }
    if (p.O != nullptr) {
#pragma unroll
        for (int k = 0; k < NK; k++)
#pragma unroll
            for (int a = 0; a < 2; a++)
                *reinterpret_cast<float2 *>(p.O + o0 + (size_t)k * plane + (size_t)a * p.wQ) = make_float2(x[k][a][0], x[k][a][1]);
    }
    if (p.pool_O != nullptr) {
#pragma unroll
        for (int k = 0; k < NK; k++)
            pool_block(p, (((size_t)img * p.Kf + (size_t)(m + k)) * p.wth + ty) * p.wtw + tx, ty, tx, x[k][0][0], x[k][0][1], x[k][1][0], x[k][1][1]);
    }
}

// A wavefront's 32 filters x 32 blocks: lane = block (column) lane % 32, filter rows 8 * (v / 4) + 4 * (lane / 32) + v % 4.
// `epi`: the tile's channel constants (stage_channel_constants); m_local: the wavefront's first row in the tile.
// NK: filter rows finished at a time (wino_store_rows), or 1 for a caller that has no registers for that.
template <int BM, int NK = 4>
__device__ __forceinline__ void wino_store_tile(const ConvParams &p, floatx16 (&y)[2][2], const float *epi, int m0, int m_local, int n_base,
                                                int lane) {
    const int n = n_base + (lane & 31);
    if (n >= p.wT) return;
    const int per_img = p.wth * p.wtw;
    const int img = n / per_img, r = n - img * per_img, ty = r / p.wtw, tx = r - ty * p.wtw;
    const size_t plane = (size_t)p.wP * p.wQ;
    const bool pair = (p.wQ % 2 == 0) && (((size_t)p.O | (size_t)(p.residual ? p.residual : p.O)) % 8 == 0);
    if constexpr (NK == 1) {  // row by row (a caller with no registers to spare)
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int ml = m_local + 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
            wino_store_row(p, channel_from_lds<BM>(epi, ml), m0 + ml, img, ty, tx, plane, pair, y[0][0][v], y[0][1][v], y[1][0][v], y[1][1][v]);
        }
    } else {
        const bool inside = pair && 2 * ty + 1 < p.wP && 2 * tx + 1 < p.wQ;
#pragma unroll
        for (int q = 0; q < 16 / NK; q++) {  // rows 8 (v / 4) + 4 (lane / 32) + v % 4 for v = NK q .. NK q + NK - 1
            const int v0 = NK * q;
            const int ml = m_local + 8 * (v0 / 4) + 4 * (lane >> 5) + (v0 % 4);
            if (inside && m0 + ml + NK - 1 < p.Kf) {
                float x[NK][2][2];
#pragma unroll
                for (int k = 0; k < NK; k++)
#pragma unroll
                    for (int a = 0; a < 2; a++)
#pragma unroll
                        for (int b = 0; b < 2; b++) x[k][a][b] = y[a][b][v0 + k];
                wino_store_rows<BM, NK>(p, epi, ml, m0 + ml, img, ty, tx, plane, x);
            } else {
#pragma unroll
                for (int k = 0; k < NK; k++) {
                    const int v = v0 + k;
                    wino_store_row(p, channel_from_lds<BM>(epi, ml + k), m0 + ml + k, img, ty, tx, plane, pair, y[0][0][v], y[0][1][v], y[1][0][v],
                                   y[1][1][v]);
                }
            }
        }
    }
}

// ---------------------------------------------------------------- MFMA kernel, compile-time filter shape
// K-step = CPB input channels x (R*S) taps.  Gather work is split by wavefront: a wavefront
// serves one 64-pixel segment of the tile (its lanes = 64 consecutive output pixels) and CPW of
// the step's channels; each of its loads is one (channel, tap) row segment of 64 floats.
// MODE: 0 = a convolution; 1 = the 16 (9) products of a Winograd convolution with the output transform folded in
// (wino_fold); 2 = a 2x2 convolution of an image upsampled twice, as four convolutions of the stored image, one per
// parity of the output row and column, on four accumulators (see up2x2_filter_kernel); 3 = the same, built with registers
// to spare for the epilogue that finishes four filter rows at a time.
template <int WM, int WN, int TM, int TN, int R, int S, int CPB, bool DIRECT, int MODE>
__device__ __forceinline__ void conv_tap_body(const ConvParams &p) {
    constexpr bool WINO = MODE == 1;  // the K range is a sequence of runs whose products end in the four outputs of a 2x2 block
    constexpr bool UP2 = MODE >= 2;  // (3: with registers to spare for the epilogue's four-row path)
    static_assert(WM * WN == 4, "four wavefronts per workgroup");
    static_assert(!WINO || (TM == 1 && TN == 1 && R == 1 && S == 1), "the Winograd products run on one 32x32 block per wavefront");
    static_assert(!UP2 || (DIRECT && R == 2 && S == 2 && TN == 1 && CPB % 2 == 0), "the upsampled form: 2x2 taps of the stored image, LDS-direct loads");
    constexpr int RS = R * S, BK = CPB * RS;
    constexpr int AK = UP2 ? CPB * 9 : BK;  // filter rows of a K-step (UP2: nine weight sums per channel where the pixel slice has four taps)
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    constexpr int NS = BN / 64;     // 64-pixel segments in a tile row
    constexpr int WPS = 4 / NS;     // wavefronts that share a segment
    constexpr int CPW = CPB / WPS;  // channels a wavefront gathers per step
    static_assert(BK % 2 == 0, "an MFMA consumes two taps");
    static_assert(NS == 1 || NS == 2 || NS == 4, "BN is 64, 128 or 256");
    static_assert(CPB % WPS == 0, "channels of a step divide over the wavefronts of a segment");
    // Rows are not padded: an operand read touches two rows (one per half wavefront) and the two
    // halves are served in separate passes, so they do not conflict (SQ_LDS_BANK_CONFLICT reads 0),
    // and without padding four workgroups fit in a CU's LDS instead of three.
    constexpr int LDA = BM, LDB = BN;
    constexpr int A_VECS = AK * BM / 4;          // float4 in one filter slice
    constexpr int AV = (A_VECS + 255) / 256;     // float4 filter loads per thread per step (last one partial)

    // (+256 floats after each filter slice: where the lanes past the end of a partial last load round park their float4)
    __shared__ __attribute__((aligned(16))) float As[2][AK * LDA + 256];
    __shared__ __attribute__((aligned(16))) float Bs[2][BK * LDB];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    int m_tile, n_tile, local_tile, slice;
    bool split;
    trace_mark(p, 0);
    tile_of_block(p, m_tile, n_tile, local_tile, slice, split);
    const int step_lo = split ? slice * p.slice_steps : 0;
    const int step_hi = split ? min(step_lo + p.slice_steps, p.nsteps) : p.nsteps;
    const int m0 = m_tile * BM;
    const long long n0 = (long long)n_tile * BN;
    ChannelEpilogue chan = {0.0f, 0.0f, 1.0f, 1.0f, 0.0f};
    if (!split && !UP2) chan = fetch_channel_constants<BM>(p, m0, tid);  // (UP2 has no register to spare in its K loop: fetched after it)

    const __amdgpu_buffer_rsrc_t rsrc_in = __builtin_amdgcn_make_buffer_rsrc((void *)p.I, 0, p.in_bytes, RSRC_WORD3);
    const __amdgpu_buffer_rsrc_t rsrc_in2 = __builtin_amdgcn_make_buffer_rsrc((void *)p.I2, 0, p.in_bytes, RSRC_WORD3);

    // ---- this thread's gathered pixel and its R*S tap offsets (bytes; OOB where the tap leaves the image)
    const int seg = wave % NS, cg = wave / NS;
    int voff[RS];
    // UP2: a "pixel" of the launch is pixel (a, b) of the stored image, i.e. the 2x2 block of outputs at (2a, 2b); tap
    // t = 2 ky + kx of it is the stored pixel (a + ky, b + kx), nothing where that leaves the image (the upsampled image
    // ends there: what follows is the zero padding below and to the right)
    if constexpr (UP2) {
        const int ng = (int)n0 + seg * 64 + lane;
        const bool pvalid = ng < p.wT;
        const unsigned ngc = pvalid ? (unsigned)ng : 0u;
        const unsigned per_img = (unsigned)(p.wth * p.wtw);
        const int img = (int)(ngc / per_img);
        const int r = (int)(ngc - (unsigned)img * per_img);
        const int a = (int)((unsigned)r / (unsigned)p.wtw), b = r - a * p.wtw;
        const int pix = img * (p.Cimg * p.H * p.W) + a * p.W + b;
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int ky = t >> 1, kx = t & 1;
            const bool ok = pvalid && a + ky < p.H && b + kx < p.W;
            voff[t] = ok ? (pix + ky * p.W + kx) * 4 : OOB;
        }
    } else {
        const int ng = (int)n0 + seg * 64 + lane;  // a launch covers fewer than 2^31 pixels
        const bool pvalid = ng < (int)p.npix;
        const unsigned ngc = pvalid ? (unsigned)ng : 0u;
        const int img = (int)(ngc / (unsigned)p.PQ);
        const int pq = (int)(ngc - (unsigned)img * (unsigned)p.PQ);
        const int op = (int)((unsigned)pq / (unsigned)p.Q), oq = pq - op * p.Q;
        const int ih0 = op * p.sr - p.pt, iw0 = oq * p.sc - p.pl;
        const int pix = img * (p.Cimg * p.H * p.W) + ih0 * p.W + iw0;
        if (p.uh == 1 && p.uw == 1) {
#pragma unroll
            for (int t = 0; t < RS; t++) {
                const int ky = t / S, kx = t % S;
                const bool ok = pvalid && (unsigned)(ih0 + ky) < (unsigned)p.H && (unsigned)(iw0 + kx) < (unsigned)p.W;
                voff[t] = ok ? (pix + ky * p.W + kx) * 4 : OOB;
            }
        } else {  // taps address the upsampled image; each reads the stored pixel it is a copy of
            const int base = img * (p.Cimg * p.H * p.W);
            const unsigned Hu = (unsigned)(p.H * p.uh), Wu = (unsigned)(p.W * p.uw);
#pragma unroll
            for (int t = 0; t < RS; t++) {
                const int ky = t / S, kx = t % S;
                const unsigned y = (unsigned)(ih0 + ky), x = (unsigned)(iw0 + kx);
                const bool ok = pvalid && y < Hu && x < Wu;
                voff[t] = ok ? (base + (int)(y / (unsigned)p.uh) * p.W + (int)(x / (unsigned)p.uw)) * 4 : OOB;
            }
        }
    }
    const int HW4 = p.H * p.W * 4;

    // ---- filter slice: float4 f of the slice is row f / (BM/4), channels 4*(f % (BM/4))
    // (plain 16-byte loads: the packed matrix is padded to whole steps and whole tiles, so every address exists)
    // Every thread loads in every round, without a condition: in a partial last round the lanes past
    // the end of the slice re-read their first element and park it behind the slice in LDS.
    const float *wp = p.Wp;
    if (p.w_img_stride != 0) wp += (size_t)((unsigned)n0 / (unsigned)p.PQ) * p.w_img_stride;  // the matrix of this tile's image
    const float *a_ptr[AV];
    int a_lds[AV];
#pragma unroll
    for (int j = 0; j < AV; j++) {
        const int f = tid + j * 256;
        const bool in_slice = f < A_VECS;
        const int fc = in_slice ? f : tid % A_VECS;
        const int kk = fc / (BM / 4), m4 = (fc % (BM / 4)) * 4;
        a_ptr[j] = wp + (size_t)kk * p.Mp + m0 + m4;
        a_lds[j] = in_slice ? kk * LDA + m4 : AK * LDA + lane * 4;
    }
    const int a_step = AK * p.Mp;

    floatx4 areg[DIRECT ? 1 : AV];
    float breg[DIRECT ? 1 : CPW * RS];

    // LDS-direct filter slice: a wavefront instruction moves 256 consecutive floats of the slice in LDS
    // (16 bytes per lane), i.e. RPI = 256 / BM whole rows; unit u (rows u*RPI ...) belongs to wavefront
    // u % 4.  The last unit may reach past the slice: it then reads rows of the next step (or zeros
    // past the end of the packed matrix, which the buffer descriptor bounds) into the parking area
    // behind the slice.
    constexpr int RPI = 256 / BM;
    constexpr int A_UNITS = (AK + RPI - 1) / RPI;
    constexpr int A_UPW = (A_UNITS + 3) / 4;
    static_assert((RPI - 1) * BM <= 256, "the parking area holds the surplus rows of the last unit");
    const int32x4 dma_w = make_rsrc_words(wp, p.wp_bytes), dma_in = make_rsrc_words(p.I, p.in_bytes);
    const int32x4 dma_in2 = make_rsrc_words(p.I2, p.in_bytes);
    const int a_voff_direct = ((lane / (BM / 4)) * p.Mp + m0 + 4 * (lane % (BM / 4))) * 4;

    auto load_a = [&](int step, lds_float *as) {
        if constexpr (DIRECT) {
#pragma unroll
            for (int j = 0; j < A_UPW; j++) {
                const int u = wave + 4 * j;
                if (A_UNITS % 4 == 0 || j < A_UPW - 1 || u < A_UNITS) {  // uniform in the wavefront
                    const int kk = u * RPI;
                    lds_dma_b128(dma_w, as + kk * LDA, a_voff_direct, (step * AK + kk) * p.Mp * 4);
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < AV; j++) areg[j] = *reinterpret_cast<const floatx4 *>(a_ptr[j] + (size_t)step * a_step);
        }
    };
    auto store_a = [&](lds_float *as) {
        if constexpr (!DIRECT) {
#pragma unroll
            for (int j = 0; j < AV; j++) {
                as[a_lds[j] + 0] = areg[j].x;
                as[a_lds[j] + 1] = areg[j].y;
                as[a_lds[j] + 2] = areg[j].z;
                as[a_lds[j] + 3] = areg[j].w;
            }
        }
    };
    // gather of one step; `checked` adds the test for channels past C (last step of an odd channel count)
    auto load_b = [&](int step, lds_float *bs, bool checked) {
        if constexpr (DIRECT) {
            // one input tensor and every channel of the step exists (nearly every step of every layer): the channel's
            // offset advances by one plane per load and nothing is selected
            if (!checked && p.Csplit == p.C) {
                int soff = (step * CPB + cg * CPW) * HW4;
#pragma unroll
                for (int jc = 0; jc < CPW; jc++) {
#pragma unroll
                    for (int t = 0; t < RS; t++) lds_dma_b32(dma_in, bs + ((cg * CPW + jc) * RS + t) * LDB + seg * 64, voff[t], soff);
                    soff += HW4;
                }
                return;
            }
        }
#pragma unroll
        for (int jc = 0; jc < CPW; jc++) {
            const int cl = cg * CPW + jc;
            const int c = step * CPB + cl;
            const bool cok = !checked || c < p.C;
            const bool second = c >= p.Csplit;  // uniform in the wavefront: the channel comes from the second tensor
            const int soff = (cok ? (second ? c - p.Csplit : c) : 0) * HW4;
#pragma unroll
            for (int t = 0; t < RS; t++) {
                const int vo = cok ? voff[t] : OOB;
                if constexpr (DIRECT) {
                    lds_dma_b32(second ? dma_in2 : dma_in, bs + (cl * RS + t) * LDB + seg * 64, vo, soff);
                } else {
                    breg[jc * RS + t] = second ? buf_load(rsrc_in2, vo, soff) : buf_load(rsrc_in, vo, soff);
                }
            }
        }
    };
    auto store_b = [&](lds_float *bs) {
        if constexpr (!DIRECT) {
#pragma unroll
            for (int jc = 0; jc < CPW; jc++)
#pragma unroll
                for (int t = 0; t < RS; t++) bs[((cg * CPW + jc) * RS + t) * LDB + seg * 64 + lane] = breg[jc * RS + t];
        }
    };

    floatx16 acc[UP2 ? 1 : TM][UP2 ? 1 : TN];
    if constexpr (!UP2) {
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
#pragma unroll
            for (int tn = 0; tn < TN; tn++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[tm][tn][v] = 0.0f;
    }
    floatx16 uy[UP2 ? TM : 1][2][2];  // UP2: per 32-filter block the outputs (2a + i, 2b + j) of the wavefront's stored pixels (a, b)
    if constexpr (UP2) {
#pragma unroll
        for (int tm = 0; tm < TM; tm++)
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
#pragma unroll
                    for (int v = 0; v < 16; v++) uy[tm][i][j][v] = 0.0f;
    }

    const int full_steps = p.C / CPB;  // steps whose channels all exist
    const int a_off = (lane >> 5) * LDA + wm * TM * 32 + (lane & 31);
    const int b_off = (lane >> 5) * LDB + wn * TN * 32 + (lane & 31);
    auto as_of = [&](int buf) { return (lds_float *)&As[buf][0]; };
    auto bs_of = [&](int buf) { return (lds_float *)&Bs[buf][0]; };

    // One K-step: start the loads of the next step into the other buffer, then the MFMAs of this one.
    auto do_step = [&](const lds_float *__restrict__ a_cur, const lds_float *__restrict__ b_cur, lds_float *__restrict__ a_nxt,
                       lds_float *__restrict__ b_nxt, int step, bool more) __attribute__((always_inline)) {
        if (more) {
            load_a(step + 1, a_nxt);
            if (step + 1 < full_steps) load_b(step + 1, b_nxt, false);
            else load_b(step + 1, b_nxt, true);
        }
        if constexpr (UP2) {
            // Filter rows of channel c: 9 c + {0: all four taps; 1, 2: the two rows of column 0, of column 1; 3, 4: the two
            // columns of row 0, of row 1; 5..8: taps 0..3}; pixel rows: 4 c + tap.  An MFMA consumes two rows, one per half
            // wavefront (h).  Per channel: output (1,1) takes taps (0,1) and (2,3), output (0,1) the column sums on taps
            // (0,1), output (1,0) the row sums on taps (0,2); per channel pair: output (0,0) the full sums on tap 0 of both.
            const int h = lane >> 5;
            static_assert(TM == 2, "the filter rows hold the two 32-filter blocks of a wavefront interleaved");
            typedef float floatx2 __attribute__((ext_vector_type(2)));
            typedef const __attribute__((address_space(3))) floatx2 *lds_f2;
            // (up2x2_filter_kernel lays a row's 64 filters out as 32 pairs {j, 32 + j}: both blocks' operands in one 8-byte read)
            const lds_float *ab = a_cur + 2 * (lane & 31), *bb = b_cur + wn * 32 + (lane & 31);
            // the operands of channel c + 1 are read from LDS while the MFMAs of channel c run (six read instructions: the
            // pixel rows (0,1) and (2,3) in one, rows (0,2), and the two filter blocks of each of the four row pairs in one)
            float bq[2][3], aq[2][4][TM], b00 = 0.0f, a_ee[TM];
            auto read_channel = [&](int c, int set) {
                bq[set][0] = bb[(4 * c + h) * LDB];
                bq[set][1] = bb[(4 * c + 2 + h) * LDB];
                bq[set][2] = bb[(4 * c + 2 * h) * LDB];
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const floatx2 a2 = *(lds_f2)(ab + (9 * c + 1 + 2 * r + h) * LDA);
                    aq[set][r][0] = a2.x;
                    aq[set][r][1] = a2.y;
                }
            };
            read_channel(0, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
#pragma unroll
            for (int c = 0; c < CPB; c++) {
                const int cur = c & 1, nxt = cur ^ 1;
                if (c + 1 < CPB) read_channel(c + 1, nxt);
                if (c % 2 == 1) {  // tap 0 of this channel and the one before, under the sums of all four taps
                    b00 = bb[(4 * (c - 1 + h)) * LDB];
                    const floatx2 a2 = *(lds_f2)(ab + (9 * (c - 1 + h)) * LDA);
                    a_ee[0] = a2.x;
                    a_ee[1] = a2.y;
                }
#pragma unroll
                for (int tm = 0; tm < TM; tm++) {
                    uy[tm][1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(aq[cur][2][tm], bq[cur][0], uy[tm][1][1], 0, 0, 0);
                    uy[tm][0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(aq[cur][0][tm], bq[cur][0], uy[tm][0][1], 0, 0, 0);
                    uy[tm][1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(aq[cur][1][tm], bq[cur][2], uy[tm][1][0], 0, 0, 0);
                }
#pragma unroll
                for (int tm = 0; tm < TM; tm++) uy[tm][1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(aq[cur][3][tm], bq[cur][1], uy[tm][1][1], 0, 0, 0);
                if (c % 2 == 1) {
#pragma unroll
                    for (int tm = 0; tm < TM; tm++) uy[tm][0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a_ee[tm], b00, uy[tm][0][0], 0, 0, 0);
                }
                // issue order: one read instruction of channel c + 1 behind each of the first MFMAs of channel c
                constexpr int kReadsNext = 6, kReadsSum = 2;
                const int reads = (c + 1 < CPB ? kReadsNext : 0) + (c % 2 == 1 ? kReadsSum : 0);
                const int mfmas = 4 * TM + (c % 2 == 1 ? TM : 0);
#pragma unroll
                for (int i = 0; i < mfmas; i++) {
                    if (i < reads) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                }
            }
            return;
        }
        // operands of tap pair ks+1 are read from LDS while the MFMAs of pair ks run
        float a[2][TM], b[2][TN];
#pragma unroll
        for (int tm = 0; tm < TM; tm++) a[0][tm] = (a_cur[a_off + tm * 32]);
#pragma unroll
        for (int tn = 0; tn < TN; tn++) b[0][tn] = (b_cur[b_off + tn * 32]);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // the two reads of pair 0
#pragma unroll
        for (int ks = 0; ks < BK / 2; ks++) {
            const int cur = ks & 1, nxt = cur ^ 1;
            if (ks + 1 < BK / 2) {
#pragma unroll
                for (int tm = 0; tm < TM; tm++) a[nxt][tm] = (a_cur[(ks + 1) * 2 * LDA + a_off + tm * 32]);
#pragma unroll
                for (int tn = 0; tn < TN; tn++) b[nxt][tn] = (b_cur[(ks + 1) * 2 * LDB + b_off + tn * 32]);
            }
#pragma unroll
            for (int tm = 0; tm < TM; tm++)
#pragma unroll
                for (int tn = 0; tn < TN; tn++)
                    acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][tm], b[cur][tn], acc[tm][tn], 0, 0, 0);
            // issue order: the LDS reads of pair ks+1 (two instructions: the TM and the TN operands
            // each pair up into one two-address read, or are one read), then the MFMAs of pair ks
            if (ks + 1 < BK / 2) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, TM * TN, 0);
        }
        if (more) {
            store_a(a_nxt);
            store_b(b_nxt);
        }
    };

    // A K range of exactly two steps (three or four input channels under a 3x3 filter) fits the two buffers: both are
    // requested before the first wait, and the loop then runs without a trip to memory between its two steps.
    const bool both = DIRECT && step_hi - step_lo == 2;
    load_a(step_lo, as_of(0));
    load_b(step_lo, bs_of(0), step_lo >= full_steps);
    if (both) {
        load_a(step_lo + 1, as_of(1));
        load_b(step_lo + 1, bs_of(1), step_lo + 1 >= full_steps);
    }
    store_a(as_of(0));
    store_b(bs_of(0));
    if constexpr (DIRECT) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wavefront's LDS-direct loads have landed
    __syncthreads();
    trace_mark(p, 1);

    floatx16 wy[WINO ? 2 : 1][WINO ? 2 : 1];  // WINO: the four outputs of every 2x2 block of this wavefront
    int wino_left = p.wspx, wino_xi = 0;        // steps left in the current patch position's run
    if constexpr (WINO) {
#pragma unroll
        for (int a = 0; a < 2; a++)
#pragma unroll
            for (int b = 0; b < 2; b++)
#pragma unroll
                for (int v = 0; v < 16; v++) wy[a][b][v] = 0.0f;
    }
    for (int step = step_lo; step < step_hi; step++) {
        const int buf = (step - step_lo) & 1;
        do_step(as_of(buf), bs_of(buf), as_of(buf ^ 1), bs_of(buf ^ 1), step, step + 1 < step_hi && !both);
        if constexpr (WINO) {
            if (--wino_left == 0) {  // this position's product is complete
                wino_fold(wy, acc[0][0], wino_xi, p.wps);
                wino_xi++;
                wino_left = p.wspx;
            }
        }
        // The barrier publishes the next buffer to the other wavefronts, so this wavefront's
        // LDS-direct loads into it must be complete first.
        if constexpr (DIRECT) __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
    }

    trace_mark(p, 2);
    if constexpr (WINO) {
        // (launched with whole tiles only)
        float *epi = &As[0][0];
        put_channel_constants<BM>(epi, chan, tid);
        __syncthreads();
        wino_store_tile<BM>(p, wy, epi, m0, wm * 32, (int)n0 + wn * 32, lane);
    } else if constexpr (UP2) {
        // (launched with whole tiles only; a lane holds the four outputs of a block like the Winograd forms)
        float *epi = &As[0][0];
        stage_channel_constants<BM>(p, epi, m0, tid);
        __syncthreads();
        // (the two blocks written out: the optimizer does not unroll a loop around this much code, and a runtime index
        // would put the accumulators in memory; four rows at a time only in the build whose register budget has room for
        // their values and constants beside the 128 accumulator registers)
        constexpr int NK = MODE == 3 ? 4 : 1;
        wino_store_tile<BM, NK>(p, uy[0], epi, m0, wm * TM * 32, (int)n0 + wn * 32, lane);
        wino_store_tile<BM, NK>(p, uy[TM - 1], epi, m0, wm * TM * 32 + 32, (int)n0 + wn * 32, lane);
    } else if (split) {
        store_partial<TM, TN>(p, acc, local_tile, slice, wave, lane);
    } else {
        float *epi = &As[0][0];  // the K loop ended with a barrier: the filter buffers are free
        put_channel_constants<BM>(epi, chan, tid);
        __syncthreads();
        store_tile<TM, TN, BM>(p, acc, epi, m0, wm * TM * 32, (int)n0 + wn * TN * 32, lane);
    }
    if (p.trace != nullptr) {
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        trace_mark(p, 3);
    }
}

template <int WM, int WN, int TM, int TN, int R, int S, int CPB, bool DIRECT, bool WINO = false>
__global__ __launch_bounds__(256, (TM * TN >= 4 ? 3 : 4)) void conv_tap_kernel(const ConvParams p) {  // registers for 3 (4) workgroups per CU
    conv_tap_body<WM, WN, TM, TN, R, S, CPB, DIRECT, WINO ? 1 : 0>(p);
}

// A 2x2 stride-1 convolution of an image upsampled twice (nearest neighbour), zero padding below and to the right only:
// 64 filters x 128 stored pixels per workgroup, four channels per K-step (conv_tap_body, MODE 2 / 3).  WGS: workgroups per CU
// the register budget is set for - three hide more of a short K loop's loads and stores; two run alike from the first
// to the last when the tile count is a whole number of generations that way and not the other.
template <int WGS>
__global__ __launch_bounds__(256, WGS) void conv_up2x2_kernel(const ConvParams p) {
    conv_tap_body<1, 4, 2, 1, 2, 2, 4, true, (WGS >= 3 ? 2 : 3)>(p);
}

// ---------------------------------------------------------------- MFMA kernel, any filter shape
// K-step = 16 taps.  Thread t gathers pixel t % BN for EPT consecutive taps of the step.  Which
// channel, filter row and filter column a tap is does not depend on the pixel, so it is worked out
// once per call, by tap_table_kernel, and the gather reads it back with scalar loads.
// Tap table of conv_gen_kernel: entry k of the padded K range (k = (c*R + ky)*S + kx) holds
// { byte offset of the tap relative to the window origin, byte offset of channel c, ky, kx }.
// Taps past C*R*S get a row offset no image reaches, so their gathers read zeros.
constexpr int TAP_NOWHERE = 0x40000000;
__global__ __launch_bounds__(256) void tap_table_kernel(int32x4 *table, int rows, int C, int R, int S, int W, int HW) {
    const int k = blockIdx.x * 256 + threadIdx.x;
    if (k >= rows) return;
    const int c = k / (R * S), rem = k - c * (R * S), ky = rem / S, kx = rem - ky * S;
    int32x4 t;
    if (c < C) {
        t.x = (ky * W + kx) * 4;
        t.y = c * HW * 4;
        t.z = ky;
        t.w = kx;
    } else {
        t.x = 0;
        t.y = 0;
        t.z = TAP_NOWHERE;
        t.w = 0;
    }
    table[k] = t;
}

template <int WM, int WN, int TM, int TN, bool DIRECT>
__global__ __launch_bounds__(256, (TM * TN >= 4 ? 3 : 4)) void conv_gen_kernel(const ConvParams p) {
    static_assert(WM * WN == 4, "four wavefronts per workgroup");
    constexpr int BK = 16;
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
    constexpr int LDA = BM, LDB = BN;
    constexpr int A_VECS = BK * BM / 4;
    constexpr int AV = (A_VECS + 255) / 256;
    constexpr int EPT = BN / 16;  // gathered elements per thread per step
    static_assert(BN >= 64 && BN <= 256, "a wavefront gathers whole tap rows");

    // (+256 floats after each filter slice: where the lanes past the end of a partial last load round park their float4)
    __shared__ __attribute__((aligned(16))) float As[2][BK * LDA + 256];
    __shared__ __attribute__((aligned(16))) float Bs[2][BK * LDB];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    int m_tile, n_tile, local_tile, slice;
    bool split;
    tile_of_block(p, m_tile, n_tile, local_tile, slice, split);
    const int step_lo = split ? slice * p.slice_steps : 0;
    const int step_hi = split ? min(step_lo + p.slice_steps, p.nsteps) : p.nsteps;
    const int m0 = m_tile * BM;
    const long long n0 = (long long)n_tile * BN;
    ChannelEpilogue chan = {0.0f, 0.0f, 1.0f, 1.0f, 0.0f};
    if (!split) chan = fetch_channel_constants<BM>(p, m0, tid);

    const __amdgpu_buffer_rsrc_t rsrc_in = __builtin_amdgcn_make_buffer_rsrc((void *)p.I, 0, p.in_bytes, RSRC_WORD3);

    const int bn_l = tid % BN;
    const int bg = __builtin_amdgcn_readfirstlane(tid / BN);           // tap group (BN >= 64: uniform in a wavefront)
    const int seg_off = __builtin_amdgcn_readfirstlane((tid - lane) % BN);  // first pixel column of this wavefront
    int ih0, iw0, pix4;
    {
        const int ng = (int)n0 + bn_l;  // a launch covers fewer than 2^31 pixels
        const bool pvalid = ng < (int)p.npix;
        const unsigned ngc = pvalid ? (unsigned)ng : 0u;
        const int img = (int)(ngc / (unsigned)p.PQ);
        const int pq = (int)(ngc - (unsigned)img * (unsigned)p.PQ);
        const int op = (int)((unsigned)pq / (unsigned)p.Q), oq = pq - op * p.Q;
        ih0 = pvalid ? op * p.sr - p.pt : TAP_NOWHERE;  // a pixel past the end of the launch gathers zeros
        iw0 = oq * p.sc - p.pl;
        pix4 = (img * (p.C * p.H * p.W) + (op * p.sr - p.pt) * p.W + iw0) * 4;
    }

    // (plain 16-byte loads: the packed matrix is padded to whole steps and whole tiles, so every address exists)
    // Every thread loads in every round, without a condition: in a partial last round the lanes past
    // the end of the slice re-read their first element and park it behind the slice in LDS.
    const float *a_ptr[AV];
    int a_lds[AV];
#pragma unroll
    for (int j = 0; j < AV; j++) {
        const int f = tid + j * 256;
        const bool in_slice = f < A_VECS;
        const int fc = in_slice ? f : tid % A_VECS;
        const int kk = fc / (BM / 4), m4 = (fc % (BM / 4)) * 4;
        a_ptr[j] = p.Wp + (size_t)kk * p.Mp + m0 + m4;
        a_lds[j] = in_slice ? kk * LDA + m4 : BK * LDA + lane * 4;
    }
    const int a_step = BK * p.Mp;
    floatx4 areg[DIRECT ? 1 : AV];
    float breg[DIRECT ? 1 : EPT];

    // LDS-direct filter slice, as in conv_tap_kernel: a wavefront instruction moves RPI = 256 / BM
    // whole rows; unit u belongs to wavefront u % 4; surplus rows of the last unit land in the
    // parking area behind the slice.
    constexpr int RPI = 256 / BM;
    constexpr int A_UNITS = (BK + RPI - 1) / RPI;
    constexpr int A_UPW = (A_UNITS + 3) / 4;
    static_assert((RPI - 1) * BM <= 256, "the parking area holds the surplus rows of the last unit");
    const int32x4 dma_w = make_rsrc_words(p.Wp, p.wp_bytes), dma_in = make_rsrc_words(p.I, p.in_bytes);
    const int a_voff_direct = ((lane / (BM / 4)) * p.Mp + m0 + 4 * (lane % (BM / 4))) * 4;

    auto load_a = [&](int step, lds_float *as) {
        if constexpr (DIRECT) {
#pragma unroll
            for (int j = 0; j < A_UPW; j++) {
                const int u = wave + 4 * j;
                if (A_UNITS % 4 == 0 || j < A_UPW - 1 || u < A_UNITS) {  // uniform in the wavefront
                    const int kk = u * RPI;
                    lds_dma_b128(dma_w, as + kk * LDA, a_voff_direct, (step * BK + kk) * p.Mp * 4);
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < AV; j++) areg[j] = *reinterpret_cast<const floatx4 *>(a_ptr[j] + (size_t)step * a_step);
        }
    };
    // the gather of one step: this wavefront's tap group, 64 pixels per tap row.  The table entries
    // are read through the constant address space with a wavefront-uniform index: scalar loads.
    typedef const __attribute__((address_space(4))) int32x4 *tap_table_ptr;
    const tap_table_ptr taps = (tap_table_ptr)p.taps;
    auto load_b = [&](int step, lds_float *bs) {
        const int i = step * BK + bg * EPT;
        int32x4 t[EPT];  // all entries first: the loads below are opaque to the compiler and would keep them apart
#pragma unroll
        for (int e = 0; e < EPT; e++) t[e] = taps[i + e];
#pragma unroll
        for (int e = 0; e < EPT; e++) {
            const bool ok = (unsigned)(ih0 + t[e].z) < (unsigned)p.H && (unsigned)(iw0 + t[e].w) < (unsigned)p.W;
            const int vo = ok ? pix4 + t[e].x : OOB;
            if constexpr (DIRECT) {
                lds_dma_b32(dma_in, bs + (bg * EPT + e) * LDB + seg_off, vo, t[e].y);
            } else {
                breg[e] = buf_load(rsrc_in, vo, t[e].y);
            }
        }
    };
    auto store_ab = [&](lds_float *as, lds_float *bs) {
        if constexpr (!DIRECT) {
#pragma unroll
            for (int j = 0; j < AV; j++) {
                as[a_lds[j] + 0] = areg[j].x;
                as[a_lds[j] + 1] = areg[j].y;
                as[a_lds[j] + 2] = areg[j].z;
                as[a_lds[j] + 3] = areg[j].w;
            }
#pragma unroll
            for (int e = 0; e < EPT; e++) bs[(bg * EPT + e) * LDB + bn_l] = breg[e];
        }
    };

    floatx16 acc[TM][TN];
#pragma unroll
    for (int tm = 0; tm < TM; tm++)
#pragma unroll
        for (int tn = 0; tn < TN; tn++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[tm][tn][v] = 0.0f;

    const int a_off = (lane >> 5) * LDA + wm * TM * 32 + (lane & 31);
    const int b_off = (lane >> 5) * LDB + wn * TN * 32 + (lane & 31);
    auto as_of = [&](int buf) { return (lds_float *)&As[buf][0]; };
    auto bs_of = [&](int buf) { return (lds_float *)&Bs[buf][0]; };

    load_a(step_lo, as_of(0));
    load_b(step_lo, bs_of(0));
    store_ab(as_of(0), bs_of(0));
    if constexpr (DIRECT) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wavefront's LDS-direct loads have landed
    __syncthreads();

    for (int step = step_lo; step < step_hi; step++) {
        const int buf = (step - step_lo) & 1;
        const bool more = step + 1 < step_hi;
        const lds_float *__restrict__ a_cur = as_of(buf);
        const lds_float *__restrict__ b_cur = bs_of(buf);
        if (more) {
            load_a(step + 1, as_of(buf ^ 1));
            load_b(step + 1, bs_of(buf ^ 1));
        }
        // operands of tap pair ks+1 are read from LDS while the MFMAs of pair ks run
        float a[2][TM], b[2][TN];
#pragma unroll
        for (int tm = 0; tm < TM; tm++) a[0][tm] = a_cur[a_off + tm * 32];
#pragma unroll
        for (int tn = 0; tn < TN; tn++) b[0][tn] = b_cur[b_off + tn * 32];
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
        for (int ks = 0; ks < BK / 2; ks++) {
            const int cur = ks & 1, nxt = cur ^ 1;
            if (ks + 1 < BK / 2) {
#pragma unroll
                for (int tm = 0; tm < TM; tm++) a[nxt][tm] = a_cur[(ks + 1) * 2 * LDA + a_off + tm * 32];
#pragma unroll
                for (int tn = 0; tn < TN; tn++) b[nxt][tn] = b_cur[(ks + 1) * 2 * LDB + b_off + tn * 32];
            }
#pragma unroll
            for (int tm = 0; tm < TM; tm++)
#pragma unroll
                for (int tn = 0; tn < TN; tn++)
                    acc[tm][tn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][tm], b[cur][tn], acc[tm][tn], 0, 0, 0);
            if (ks + 1 < BK / 2) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, TM * TN, 0);
        }
        if (more) store_ab(as_of(buf ^ 1), bs_of(buf ^ 1));
        // the barrier publishes the next buffer: this wavefront's LDS-direct loads into it must be complete
        if constexpr (DIRECT) __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
    }

    if (split) {
        store_partial<TM, TN>(p, acc, local_tile, slice, wave, lane);
    } else {
        float *epi = &As[0][0];  // the K loop ended with a barrier: the filter buffers are free
        put_channel_constants<BM>(epi, chan, tid);
        __syncthreads();
        store_tile<TM, TN, BM>(p, acc, epi, m0, wm * TM * 32, (int)n0 + wn * TN * 32, lane);
    }
}

// ---------------------------------------------------------------- finishing kernel of K-split tiles
// One workgroup per 32x32 block of a divided tile (4 wavefronts x TM x TN blocks per tile), same lane -> output
// mapping as the MFMA kernels, a quarter of the block's rows per wavefront (accumulator registers 4q .. 4q+3 of
// wavefront q): adds the slices in increasing K order (a fixed order: results do not depend on scheduling), then
// applies the fused tail and stores.  A wavefront has few values and therefore all slices' loads in flight at once
// (fifteen slices at a time): the kernel lasts about one trip to memory.
template <int WM, int WN, int TM, int TN>
__global__ __launch_bounds__(256) void conv_reduce_kernel(const ConvParams p) {
    constexpr int BM = WM * TM * 32, BN = WN * TN * 32, UNITS = 4 * TM * TN;
    const int lane = threadIdx.x & 63, q = threadIdx.x >> 6, half = lane >> 5;
    const int unit = blockIdx.x % UNITS, local_tile = blockIdx.x / UNITS;
    const int wave = unit / (TM * TN), blk = unit % (TM * TN);
    const int wm = wave / WN, wn = wave % WN, tm = blk / TN, tn = blk % TN;
    const int tile = p.main_tiles + local_tile;
    const int m_first = (tile % p.gm) * BM + (wm * TM + tm) * 32 + 8 * q + 4 * half;  // this lane's rows: m_first + 0..3
    const long long n = (long long)(tile / p.gm) * BN + (wn * TN + tn) * 32 + (lane & 31);
    const size_t tiles = gridDim.x / UNITS;
    // the channel constants are asked for first, then the slices
    ChannelEpilogue chan[4];
#pragma unroll
    for (int j = 0; j < 4; j++) chan[j] = load_channel(p, m_first + j < p.Kf ? m_first + j : p.Kf - 1);
    const size_t slice_stride = tiles * 4 * (TM * TN) * (16 * 64);
    const float *src = p.partial + (((size_t)local_tile * 4 + wave) * (TM * TN) + blk) * (16 * 64) + (4 * q) * 64 + lane;
    float acc[4];
#pragma unroll
    for (int j = 0; j < 4; j++) acc[j] = src[j * 64];  // the sum starts from slice 0's value, not from zero
    int sl = 1;
    for (; sl + 15 <= p.nslices; sl += 15) {
        float x[15][4];
#pragma unroll
        for (int u = 0; u < 15; u++)
#pragma unroll
            for (int j = 0; j < 4; j++) x[u][j] = src[(size_t)(sl + u) * slice_stride + j * 64];
#pragma unroll
        for (int u = 0; u < 15; u++)
#pragma unroll
            for (int j = 0; j < 4; j++) acc[j] = __fadd_rn(acc[j], x[u][j]);
    }
    {
        float x[14][4];
#pragma unroll
        for (int u = 0; u < 14; u++)
            if (sl + u < p.nslices) {
#pragma unroll
                for (int j = 0; j < 4; j++) x[u][j] = src[(size_t)(sl + u) * slice_stride + j * 64];
            }
#pragma unroll
        for (int u = 0; u < 14; u++)
            if (sl + u < p.nslices) {
#pragma unroll
                for (int j = 0; j < 4; j++) acc[j] = __fadd_rn(acc[j], x[u][j]);
            }
    }
    if (n >= p.npix) return;
    const unsigned img = (unsigned)n / (unsigned)p.PQ, pq = (unsigned)n - img * (unsigned)p.PQ;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int m = m_first + j;
        if (m < p.Kf) {
            const size_t oidx = ((size_t)img * p.Kf + m) * p.PQ + pq;
            p.O[oidx] = apply_epilogue(p, chan[j], acc[j], oidx);
        }
    }
}

// ---------------------------------------------------------------- 1x1 convolution onto a few filters
// A 1x1, stride-1, unpadded convolution with at most four filters (a segmentation head: 64 -> 1) reads C values and
// writes KF per pixel: no matrix-core tile has work for 32 filter rows, and the layer is a read stream.  One thread
// takes VEC consecutive pixels of one image for all KF filters and walks the channels with eight loads in flight;
// per output the products are added in increasing channel order with a separate multiply and add, which is the
// reference's direct form (src/hardware/cpu/nn/cpu_conv.cpp:296-311) for a one-tap filter, rounding for rounding.
template <int KF, int VEC>
__global__ __launch_bounds__(256) void conv_pointwise_few_kernel(const ConvParams p) {
    typedef float vec_t __attribute__((ext_vector_type(VEC)));
    const size_t PQ = (size_t)p.PQ, per_img = PQ / VEC, total = (size_t)p.N * per_img;
    ChannelEpilogue epi[KF];
#pragma unroll
    for (int k = 0; k < KF; k++) epi[k] = load_channel(p, k);
    for (size_t g = (size_t)blockIdx.x * 256 + threadIdx.x; g < total; g += (size_t)gridDim.x * 256) {
        const size_t img = g / per_img, pq = (g - img * per_img) * VEC;
        const float *src = p.I + img * (size_t)p.C * PQ + pq;
        float acc[KF][VEC];
#pragma unroll
        for (int k = 0; k < KF; k++)
#pragma unroll
            for (int v = 0; v < VEC; v++) acc[k][v] = 0.0f;
        for (int c0 = 0; c0 < p.C; c0 += 8) {
            vec_t x[8];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const int c = c0 + u < p.C ? c0 + u : p.C - 1;  // a short last group re-reads the last channel; unused below
                x[u] = __builtin_nontemporal_load(reinterpret_cast<const vec_t *>(src + (size_t)c * PQ));
            }
#pragma unroll
            for (int u = 0; u < 8; u++) {
                if (c0 + u < p.C) {
#pragma unroll
                    for (int k = 0; k < KF; k++) {
                        const float w = p.K[(size_t)k * p.C + c0 + u];
#pragma unroll
                        for (int v = 0; v < VEC; v++) acc[k][v] = __fadd_rn(acc[k][v], __fmul_rn(w, x[u][v]));
                    }
                }
            }
        }
#pragma unroll
        for (int k = 0; k < KF; k++) {
            const size_t o = (img * KF + k) * PQ + pq;
            vec_t y;
#pragma unroll
            for (int v = 0; v < VEC; v++) y[v] = apply_epilogue(p, epi[k], acc[k][v], o + v);
            *reinterpret_cast<vec_t *>(p.O + o) = y;
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
        const float *img = p.I + (size_t)b * p.Cimg * p.H * p.W, *img2 = p.I2 + (size_t)b * p.Cimg * p.H * p.W;
        const float *flt = p.K + (size_t)k * p.C * p.R * p.S;
        float s = 0.0f;
        for (int x = 0; x < p.R; x++) {
            const int pxu = pp * p.sr + x - p.pt;  // row in the (upsampled) image the convolution sees
            if (pxu < 0 || pxu >= p.H * p.uh) continue;
            const int px = pxu / p.uh;
            for (int y = 0; y < p.S; y++) {
                const int pyu = q * p.sc + y - p.pl;
                if (pyu < 0 || pyu >= p.W * p.uw) continue;
                const int py = pyu / p.uw;
                for (int c = 0; c < p.C; c++) {
                    const float v = c < p.Csplit ? img[((size_t)c * p.H + px) * p.W + py] : img2[((size_t)(c - p.Csplit) * p.H + px) * p.W + py];
                    s = __fadd_rn(s, __fmul_rn(flt[((size_t)c * p.R + x) * p.S + y], v));
                }
            }
        }
        const ChannelEpilogue e = load_channel(p, k);
        p.O[o] = apply_epilogue(p, e, s, o);
    }
}

// ---------------------------------------------------------------- Winograd F(2x2, 3x3) and F(2x2, 2x2)
// A 3x3 stride-1 convolution as 16 independent products of [Kf x C] by [C x tiles] matrices (Lavin & Gray's minimal
// filtering form): every 4x4 input patch d (stride 2, so neighbouring patches overlap by two pixels) becomes
// V = B^T d B, every filter g becomes U = G g G^T, M = U (.) V summed over the channels - position by position, which is
// what makes it 16 matrix products - and each 2x2 block of outputs is A^T M A.  2.25 times fewer multiplications than
// the direct form.  The products run as ONE launch of the 1x1 tile kernel over 16 "images" (ConvParams::w_img_stride);
// the two transforms are bandwidth kernels.  Sums are fp32 in a fixed order, so results are reproducible, and they
// differ from the direct form's by rounding only (a few 1e-7 of the largest output on this path's layers).
//   B^T = [1 0 -1 0; 0 1 1 0; 0 -1 1 0; 0 1 0 -1]   G = [1 0 0; .5 .5 .5; .5 -.5 .5; 0 0 1]   A^T = [1 1 1 0; 0 1 -1 -1]
// The same for a 2x2 filter (U-Net's convolutions behind its upsamplings): 3x3 patches, 9 products where the direct form
// multiplies 16 times, every factor 1 or -1:
//   B^T = [1 -1 0; 0 1 0; 0 1 -1]   G = [1 0; 1 1; 0 1]   A^T = [1 1 0; 0 1 -1]
// PS below is the patch side (filter size + 1), PS * PS the number of products ("positions").
struct WinoParams {
    const float *I, *I2;  // input as ConvParams describes it (second tensor of a folded Concat, folded upsampling)
    int Csplit, Cimg, uh, uw;
    int C, H, W, pt, pl;
    int th, tw;  // 2x2 output blocks per image, rows and columns
    int T, Tp;   // blocks in the launch; Tp = T rounded up to the widest tile: one "image" of the product launch
    float *V;    // [PS * PS][C][Tp]
};
constexpr int WINO_CH = 4;  // channels (input transform) or filters (output transform) per thread

// (cmajor: the layout of the one-launch form, U[c][position][Mp]; otherwise one packed matrix per position, U[position][rows][Mp])
template <int PS>
__global__ __launch_bounds__(256) void wino_filter_kernel(const float *__restrict__ K, float *__restrict__ U, int Kf, int C, int Mp, int rows, int cmajor) {
    constexpr int R = PS - 1;
    const int idx = blockIdx.x * 256 + threadIdx.x;  // (c, k), k fastest: row c of the packed matrices
    if (idx >= rows * Mp) return;
    const int c = idx / Mp, k = idx - c * Mp;
    float g[R * R];
#pragma unroll
    for (int i = 0; i < R * R; i++) g[i] = (c < C && k < Kf) ? K[((size_t)k * C + c) * (R * R) + i] : 0.0f;
    const size_t plane = (size_t)rows * Mp;
    auto at = [&](int e) -> float & { return cmajor ? U[((size_t)c * (PS * PS) + e) * Mp + k] : U[(size_t)e * plane + idx]; };
    if constexpr (PS == 4) {
        float t[4][3];
#pragma unroll
        for (int j = 0; j < 3; j++) {
            t[0][j] = g[j];
            t[1][j] = __fmul_rn(0.5f, __fadd_rn(__fadd_rn(g[j], g[3 + j]), g[6 + j]));
            t[2][j] = __fmul_rn(0.5f, __fadd_rn(__fsub_rn(g[j], g[3 + j]), g[6 + j]));
            t[3][j] = g[6 + j];
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            at(4 * i + 0) = t[i][0];
            at(4 * i + 1) = __fmul_rn(0.5f, __fadd_rn(__fadd_rn(t[i][0], t[i][1]), t[i][2]));
            at(4 * i + 2) = __fmul_rn(0.5f, __fadd_rn(__fsub_rn(t[i][0], t[i][1]), t[i][2]));
            at(4 * i + 3) = t[i][2];
        }
    } else {
        float t[3][2];
#pragma unroll
        for (int j = 0; j < 2; j++) {
            t[0][j] = g[j];
            t[1][j] = __fadd_rn(g[j], g[2 + j]);
            t[2][j] = g[2 + j];
        }
#pragma unroll
        for (int i = 0; i < 3; i++) {
            at(3 * i + 0) = t[i][0];
            at(3 * i + 1) = __fadd_rn(t[i][0], t[i][1]);
            at(3 * i + 2) = t[i][1];
        }
    }
}

// V = B^T d B of one PS x PS patch, written to the PS * PS planes (`plane` floats apart) at dst
template <int PS>
__device__ __forceinline__ void wino_input_store(const float (&d)[PS * PS], float *dst, size_t plane) {
    float u[PS * PS];  // B^T d
    if constexpr (PS == 4) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            u[0 + j] = __fsub_rn(d[0 + j], d[8 + j]);
            u[4 + j] = __fadd_rn(d[4 + j], d[8 + j]);
            u[8 + j] = __fsub_rn(d[8 + j], d[4 + j]);
            u[12 + j] = __fsub_rn(d[4 + j], d[12 + j]);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {  // (B^T d) B
            dst[(size_t)(4 * i + 0) * plane] = __fsub_rn(u[4 * i + 0], u[4 * i + 2]);
            dst[(size_t)(4 * i + 1) * plane] = __fadd_rn(u[4 * i + 1], u[4 * i + 2]);
            dst[(size_t)(4 * i + 2) * plane] = __fsub_rn(u[4 * i + 2], u[4 * i + 1]);
            dst[(size_t)(4 * i + 3) * plane] = __fsub_rn(u[4 * i + 1], u[4 * i + 3]);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 3; j++) {
            u[0 + j] = __fsub_rn(d[0 + j], d[3 + j]);
            u[3 + j] = d[3 + j];
            u[6 + j] = __fsub_rn(d[3 + j], d[6 + j]);
        }
#pragma unroll
        for (int i = 0; i < 3; i++) {
            dst[(size_t)(3 * i + 0) * plane] = __fsub_rn(u[3 * i + 0], u[3 * i + 1]);
            dst[(size_t)(3 * i + 1) * plane] = u[3 * i + 1];
            dst[(size_t)(3 * i + 2) * plane] = __fsub_rn(u[3 * i + 1], u[3 * i + 2]);
        }
    }
}

// The input transform with the image rows staged through LDS.  A workgroup takes 256 consecutive blocks, i.e. a run of
// whole rows of blocks in one image or a few small images, and `chans` channels.  Once per workgroup it writes, for every
// LDS slot (a pixel of the zero-padded, possibly upsampled rows its blocks touch; a row holds 2 tw + 2 pixels, the
// first being column -pad_left), where that pixel lies in a channel plane, or that it does not exist.  Then per channel:
// the slots are filled with coalesced loads - every pixel once, where the kernel below reads each four times through
// the cache with half of every line unused -, a thread reads its 4x4 patch from LDS, transforms and stores as below.
template <int KMAX, int PS>  // a thread fills at most KMAX slots: slots <= 256 * KMAX
__global__ __launch_bounds__(256) void wino_input_lds_kernel(const WinoParams w, int slots, int chans) {
    extern __shared__ int wino_lds[];
    int *soff = wino_lds;
    float *sval = reinterpret_cast<float *>(wino_lds + slots);
    const int tid = threadIdx.x;
    const int t0 = blockIdx.x * 256, t1 = min(t0 + 256, w.T), t = t0 + tid;
    const int per_img = w.th * w.tw, LW = 2 * w.tw + PS - 2;
    const unsigned Hu = (unsigned)(w.H * w.uh), Wu = (unsigned)(w.W * w.uw);
    const int n_first = t0 / per_img;
    const int img_elems = w.Cimg * w.H * w.W;
    const int my_n = t / per_img, my_r = t - my_n * per_img, my_ty = my_r / w.tw, my_tx = my_r - my_ty * w.tw;
    int my_base = 0, total = 0;
    for (int n = n_first; n * per_img < t1; n++) {  // the images this workgroup's blocks lie in (uniform)
        const int a = max(t0, n * per_img) - n * per_img, b = min(t1, (n + 1) * per_img) - n * per_img;
        const int ty_a = a / w.tw, ty_b = (b - 1) / w.tw;
        const int cells = (2 * (ty_b - ty_a) + PS) * LW;
        const int y_first = 2 * ty_a - w.pt, img_off = (n - n_first) * img_elems;
        for (int i = tid; i < cells; i += 256) {
            const int r = i / LW, xl = i - r * LW;
            const unsigned y = (unsigned)(y_first + r), x = (unsigned)(xl - w.pl);
            soff[total + i] = (y < Hu && x < Wu) ? img_off + (int)(y / (unsigned)w.uh) * w.W + (int)(x / (unsigned)w.uw) : -1;
        }
        if (my_n == n) my_base = total + 2 * (my_ty - ty_a) * LW + 2 * my_tx;
        total += cells;
    }
    __syncthreads();
    const size_t hw = (size_t)w.H * w.W, plane = (size_t)w.C * w.Tp;
    const int c0 = blockIdx.y * chans, c1 = min(c0 + chans, w.C);
    auto plane_of = [&](int c) {
        return c < w.Csplit ? w.I + ((size_t)n_first * w.Cimg + c) * hw : w.I2 + ((size_t)n_first * w.Cimg + (c - w.Csplit)) * hw;
    };
    // the next channel's pixels are requested while this channel's patches are transformed and stored
    float pre[KMAX];
    auto fetch = [&](int c) {
        const float *src = plane_of(c);
#pragma unroll
        for (int k = 0; k < KMAX; k++) {
            const int i = tid + 256 * k;
            pre[k] = 0.0f;
            if (i < total) {
                const int o = soff[i];
                if (o >= 0) pre[k] = src[o];
            }
        }
    };
    fetch(c0);
    for (int c = c0; c < c1; c++) {
#pragma unroll
        for (int k = 0; k < KMAX; k++)
            if (tid + 256 * k < total) sval[tid + 256 * k] = pre[k];
        __syncthreads();
        if (c + 1 < c1) fetch(c + 1);
        if (t < t1) {
            float d[PS * PS];
            if constexpr (PS == 4) {
#pragma unroll
                for (int i = 0; i < 4; i++) {  // (rows and the patch's first column are at even slots)
                    const float2 lo = *reinterpret_cast<const float2 *>(sval + my_base + i * LW);
                    const float2 hi = *reinterpret_cast<const float2 *>(sval + my_base + i * LW + 2);
                    d[4 * i + 0] = lo.x;
                    d[4 * i + 1] = lo.y;
                    d[4 * i + 2] = hi.x;
                    d[4 * i + 3] = hi.y;
                }
            } else {
#pragma unroll
                for (int i = 0; i < PS; i++)
#pragma unroll
                    for (int j = 0; j < PS; j++) d[PS * i + j] = sval[my_base + i * LW + j];
            }
            wino_input_store<PS>(d, w.V + (size_t)c * w.Tp + t, plane);
        }
        __syncthreads();
    }
}

// One thread: one 2x2 output block (its 4x4 input patch) for WINO_CH channels; lanes hold consecutive blocks, so the 16
// stores of a channel are 16 coalesced rows.  The patch offsets and which of its pixels exist are worked out once.
// (The general form: taken where the staged kernel's tables would not fit.)
template <int PS>
__global__ __launch_bounds__(256) void wino_input_kernel(const WinoParams w) {
    const int t = blockIdx.x * 256 + threadIdx.x;
    if (t >= w.T) return;
    const int per_img = w.th * w.tw;
    const int n = t / per_img, r = t - n * per_img, ty = r / w.tw, tx = r - ty * w.tw;
    const int y0 = 2 * ty - w.pt, x0 = 2 * tx - w.pl;
    const unsigned Hu = (unsigned)(w.H * w.uh), Wu = (unsigned)(w.W * w.uw);
    int off[PS * PS];
    unsigned mask = 0;
#pragma unroll
    for (int i = 0; i < PS; i++)
#pragma unroll
        for (int j = 0; j < PS; j++) {
            const unsigned y = (unsigned)(y0 + i), x = (unsigned)(x0 + j);
            const bool ok = y < Hu && x < Wu;
            int o = 0;
            if (ok) o = (w.uh == 1 && w.uw == 1) ? (int)(y * (unsigned)w.W + x) : (int)((y / (unsigned)w.uh) * (unsigned)w.W + x / (unsigned)w.uw);
            off[PS * i + j] = o;
            mask |= (ok ? 1u : 0u) << (PS * i + j);
        }
    const size_t hw = (size_t)w.H * w.W, plane = (size_t)w.C * w.Tp;
    const int c0 = blockIdx.y * WINO_CH;
#pragma unroll
    for (int cc = 0; cc < WINO_CH; cc++) {
        const int c = c0 + cc;
        if (c >= w.C) break;
        const float *src = c < w.Csplit ? w.I + ((size_t)n * w.Cimg + c) * hw : w.I2 + ((size_t)n * w.Cimg + (c - w.Csplit)) * hw;
        float d[PS * PS];
#pragma unroll
        for (int e = 0; e < PS * PS; e++) d[e] = ((mask >> e) & 1u) ? src[off[e]] : 0.0f;
        wino_input_store<PS>(d, w.V + (size_t)c * w.Tp + t, plane);
    }
}

// One thread: one 2x2 output block for WINO_CH filters: A^T M A, then the convolution's epilogue (the arithmetic of
// apply_epilogue, value by value) and the stores - both values of a row at once where the row pair is aligned.
template <int PS>
__global__ __launch_bounds__(256) void wino_output_kernel(const ConvParams p, const float *__restrict__ M, int th, int tw, int T, int Tp) {
    const int t = blockIdx.x * 256 + threadIdx.x;
    if (t >= T) return;
    const int per_img = th * tw;
    const int n = t / per_img, r = t - n * per_img, ty = r / tw, tx = r - ty * tw;
    const size_t plane = (size_t)p.Kf * Tp;
    const bool pair = (p.Q % 2 == 0) && (((size_t)p.O | (size_t)(p.residual ? p.residual : p.O)) % 8 == 0);  // PQ is then even, too
    const int k0 = blockIdx.y * WINO_CH;
#pragma unroll
    for (int cc = 0; cc < WINO_CH; cc++) {
        const int k = k0 + cc;
        if (k >= p.Kf) break;
        const float *src = M + (size_t)k * Tp + t;
        float m[PS * PS];
#pragma unroll
        for (int e = 0; e < PS * PS; e++) m[e] = src[(size_t)e * plane];
        float s[2][PS];
#pragma unroll
        for (int j = 0; j < PS; j++) {
            if constexpr (PS == 4) {
                s[0][j] = __fadd_rn(__fadd_rn(m[0 + j], m[4 + j]), m[8 + j]);
                s[1][j] = __fsub_rn(__fsub_rn(m[4 + j], m[8 + j]), m[12 + j]);
            } else {
                s[0][j] = __fadd_rn(m[0 + j], m[3 + j]);
                s[1][j] = __fsub_rn(m[3 + j], m[6 + j]);
            }
        }
        const ChannelEpilogue e = load_channel(p, k);
        float fin[2][2] = {{0.0f, 0.0f}, {0.0f, 0.0f}};
#pragma unroll
        for (int a = 0; a < 2; a++) {
            const int oy = 2 * ty + a, ox = 2 * tx;
            if (oy >= p.P) break;
            float v0, v1;
            if constexpr (PS == 4) {
                v0 = __fadd_rn(__fadd_rn(s[a][0], s[a][1]), s[a][2]);
                v1 = __fsub_rn(__fsub_rn(s[a][1], s[a][2]), s[a][3]);
            } else {
                v0 = __fadd_rn(s[a][0], s[a][1]);
                v1 = __fsub_rn(s[a][1], s[a][2]);
            }
            const size_t oidx = ((size_t)n * p.Kf + k) * p.PQ + (size_t)oy * p.Q + ox;
            if (pair) {  // Q even: column ox + 1 exists
                float r0 = 0.0f, r1 = 0.0f;
                if (p.residual) {
                    const float2 rr = *reinterpret_cast<const float2 *>(p.residual + oidx);
                    r0 = rr.x;
                    r1 = rr.y;
                }
                float x0 = v0, x1 = v1;
                if (p.bias) x0 = __fadd_rn(x0, e.bias), x1 = __fadd_rn(x1, e.bias);
                if (p.bn_mean) {
                    x0 = __fdiv_rn(__fsub_rn(x0, e.mean), e.sd), x1 = __fdiv_rn(__fsub_rn(x1, e.mean), e.sd);
                    if (p.bn_g) x0 = __fadd_rn(__fmul_rn(x0, e.g), e.b), x1 = __fadd_rn(__fmul_rn(x1, e.g), e.b);
                }
                if (p.residual) x0 = __fadd_rn(x0, r0), x1 = __fadd_rn(x1, r1);
                if (p.relu) x0 = x0 > 0.0f ? x0 : 0.0f, x1 = x1 > 0.0f ? x1 : 0.0f;
                fin[a][0] = x0;
                fin[a][1] = x1;
                if (p.O != nullptr) *reinterpret_cast<float2 *>(p.O + oidx) = make_float2(x0, x1);
            } else {
                fin[a][0] = apply_epilogue(p, e, v0, oidx);
                if (p.O != nullptr) p.O[oidx] = fin[a][0];
                if (ox + 1 < p.Q) {
                    fin[a][1] = apply_epilogue(p, e, v1, oidx + 1);
                    if (p.O != nullptr) p.O[oidx + 1] = fin[a][1];
                }
            }
        }
        if (p.pool_O != nullptr)  // (even P, Q: both rows and both columns of the block exist)
            pool_block(p, (((size_t)n * p.Kf + k) * th + ty) * tw + tx, ty, tx, fin[0][0], fin[0][1], fin[1][0], fin[1][1]);
    }
}

// Issue order of one channel pair of wino_fused_kernel (see there): H1 matrix instructions, each followed by its share of
// NDS LDS reads, then H2 matrix instructions, each followed by its share of NVALU vector instructions.
template <int NDS, int NVALU, int H1, int H2, int K>
__device__ __forceinline__ void wino_sched_pair() {
    if constexpr (K < H1) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        constexpr int n = (NDS * (K + 1)) / H1 - (NDS * K) / H1;
        if constexpr (n > 0) __builtin_amdgcn_sched_group_barrier(0x100, n, 0);
        wino_sched_pair<NDS, NVALU, H1, H2, K + 1>();
    } else if constexpr (K < H1 + H2) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        constexpr int n = (NVALU * (K - H1 + 1)) / H2 - (NVALU * (K - H1)) / H2;
        (void)n;  // (the additions are left to the scheduler: address arithmetic counts as vector work, too)
        wino_sched_pair<NDS, NVALU, H1, H2, K + 1>();
    }
}

// ---------------------------------------------------------------- Winograd F(2x2, 3x3) in one launch, no transformed input in memory
// The whole convolution - input transform, the 16 products, output transform, epilogue - in ONE kernel that reads the
// NCHW input itself.  The loop order is channels outermost: a workgroup owns a tile of 32 FM filters x 32 FN blocks (2x2
// output blocks, numbered image by image, row by row) and keeps the accumulators of ALL 16 patch positions of that tile,
// wavefront i those of position row i (positions 4 i .. 4 i + 3: 4 FM FN blocks of 32x32 per wavefront).  A K-step is CK
// input channels:
//   * the load unit writes the step's slice of the transformed filters, U[c][position][filter] (wino_filter_kernel's
//     channel-major layout: a step's slice of a filter tile is 16 CK rows of 32 FM floats), and the RAW 4x4 patches
//     of the tile's blocks, R[c][patch element][block], into LDS (buffer_load ... lds; a patch element outside the image,
//     or of a block past the end, has an out-of-range offset and arrives as 0, as in conv_tap_kernel's gather);
//   * a lane derives its B operands itself: position row i of V = B^T d B needs two patch rows (i = 0: row 0 - row 2,
//     1: row 1 + row 2, 2: row 2 - row 1, 3: row 1 - row 3), i.e. eight LDS reads and four additions give the row
//     combination u[0..3] of the lane's (block, channel), and four more give the wavefront's four operands
//     u0 - u2, u1 + u2, u2 - u1, u1 - u3 - the very operations, in the very order, of wino_input_store, so V has the bits
//     it has in the other Winograd forms; it is never stored.
// After the last channel the wavefronts combine their positions' products along the row (s0 = m0 + m1 + m2,
// s1 = m1 - m2 - m3), exchange s through LDS, and wavefront q finishes filter rows 8 q + 4 (lane / 32) + 0..3 of every
// block: y[a][b] = s[0][b] + s[1][b] + s[2][b] (a = 0), s[1][b] - s[2][b] - s[3][b] (a = 1), then the convolution's
// epilogue (wino_store_row).  Sums: channels in increasing order, two per matrix instruction, one accumulator per
// position from the first channel to the last; the output transform in the order just given.  Whole tiles only.
// WPE: wavefronts per SIMD the register budget is set for.  WIDE: the pixels come in 16 bytes per lane (two load instructions
// per channel where the 4-byte gather issues five), for launches whose image rows are a multiple of four pixels long.
template <int FM, int FN, int CK, int WPE, bool WIDE>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void wino_fused_kernel(const ConvParams p) {
    static_assert(CK % 4 == 0 && FN <= 2 && FM <= 2, "a wavefront stages whole channels; a lane gathers one block");
    constexpr int MF = 32 * FM, NB = 32 * FN;
    constexpr int U_FLOATS = CK * 16 * MF;  // a step's filter slice  [c][position][MF]
    constexpr int R_FLOATS = CK * 16 * NB;  // a step's raw patches   [c][patch element][NB]
    constexpr int BUF_FLOATS = U_FLOATS + R_FLOATS;
    constexpr int XCH_FLOATS = 4 * 2 * 16 * 64;  // the exchange of one 32x32 block: [position row][b][v][lane]
    constexpr int LDS_FLOATS = 2 * BUF_FLOATS > XCH_FLOATS ? 2 * BUF_FLOATS : XCH_FLOATS;
    __shared__ __attribute__((aligned(16))) float lds[LDS_FLOATS];
    __shared__ __attribute__((aligned(16))) float epi[5 * MF];

    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, half = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int m_tile, n_tile, local_tile, slice;
    bool split;
    trace_mark(p, 0);
    tile_of_block(p, m_tile, n_tile, local_tile, slice, split);
    const int m0 = m_tile * MF, n0 = n_tile * NB;
    // a tile the launch plan divides along the channels: this workgroup sums steps step_lo .. step_hi - 1 only
    const int step_lo = split ? slice * p.slice_steps : 0;
    const int step_hi = split ? min(step_lo + p.slice_steps, p.nsteps) : p.nsteps;
    // Requested first, used last: the step's filter slice needs nothing but the tile's place, so it is on its way while
    // the lanes work out where the pixels go (below); so are the channel constants, which reach LDS after that.
    ChannelEpilogue chan = {0.0f, 0.0f, 1.0f, 1.0f, 0.0f};

    // filter slice: a wavefront instruction moves 256 consecutive floats of the slice, i.e. RPI whole rows of MF
    constexpr int RPI = 256 / MF, U_UNITS = U_FLOATS / 256, UPW = U_UNITS / 4;
    const int32x4 dma_w = make_rsrc_words(p.Wp, p.wp_bytes);
    const int a_voff = ((lane / (MF / 4)) * p.Mp + m0 + 4 * (lane % (MF / 4))) * 4;
    auto load_filters = [&](int step, lds_float *us) {
#pragma unroll
        for (int j = 0; j < UPW; j++) {
            const int u = wave + 4 * j;
            lds_dma_b128(dma_w, us + u * 256, a_voff, (step * (CK * 16) + u * RPI) * p.Mp * 4);
        }
    };
    load_filters(step_lo, (lds_float *)&lds[0]);
    if (!split) chan = fetch_channel_constants<MF>(p, m0, tid);

    // ---- where the tile's pixels go in LDS, and where this lane's patches lie there.  The tile's blocks are a run of
    // consecutive blocks, i.e. a few SEGMENTS of block rows (a segment: cnt neighbouring blocks of one row of blocks of one
    // image).  A segment's blocks share pixels with their neighbours, so it is staged as the 4 pixel rows it touches,
    // 2 cnt + 2 pixels each, every pixel once: slot (segment base) + r (2 cnt + 2) + x is pixel (2 ty - pad_top + r,
    // 2 tx_first - pad_left + x).  The slots of a channel are consecutive LDS floats, slot k * 64 + lane is written by lane
    // `lane` of load k: its byte offset in a channel plane (or out of range: padding, a block past the end) is worked out
    // here once.  16 NB slots always suffice (a segment of one block takes 16).
    constexpr int SLOTS = 16 * NB, WLC = WIDE ? SLOTS / 256 : SLOTS / 64;
    const int per_img = p.wth * p.wtw;
    int voff[WLC], my_base[FN], my_stride[FN];
#pragma unroll
    for (int k = 0; k < WLC; k++) voff[k] = OOB;
#pragma unroll
    for (int fn = 0; fn < FN; fn++) my_base[fn] = 0, my_stride[fn] = 0;  // (a block past the end reads slot 0: never stored)
    int nload;
    {
        const int n_end = min(n0 + NB, p.wT);
        const unsigned Hu = (unsigned)(p.H * p.uh), Wu = (unsigned)(p.W * p.uw);
        const int img_elems = p.Cimg * p.H * p.W;
        const bool whole = p.uh == 1 && p.uw == 1;  // (the stored image itself: no division per slot)
        int base = 0;
        for (int seg_n = n0; seg_n < n_end;) {  // (uniform)
            const int row = seg_n / p.wtw, tx0 = seg_n - row * p.wtw;
            const int cnt = min(p.wtw - tx0, n_end - seg_n), width = 2 * cnt + 2;
            const int img = row / p.wth, ty = row - img * p.wth;
            const int y0 = 2 * ty - p.pt, x0 = 2 * tx0 - p.pl, gbase = img * img_elems;
            if constexpr (WIDE) {
                // 16 bytes per lane: a segment's pixel rows start at the multiple of four columns at or below x0 and are
                // a whole number of GROUPS of four columns long.  The launch has image rows of a multiple of four pixels
                // and 16-byte aligned tensors, so a group lies inside the image or outside it as a whole (out of range:
                // four zeros), every load is aligned, and a patch starts `shift` slots into its row (odd with one column
                // of padding: the patches are read with 4-byte alignment).  Group g of a channel is written by lane
                // g % 64 of load g / 64.  (The host launches this build only where 16 NB slots hold the widened rows.)
                const int xs = ((x0 + 4) & ~3) - 4, shift = x0 - xs, gpr = (shift + width + 3) >> 2, gb = base >> 2;
#pragma unroll
                for (int k = 0; k < WLC; k++) {
                    const int local = k * 64 + lane - gb;
                    const int r = (local >= gpr ? 1 : 0) + (local >= 2 * gpr ? 1 : 0) + (local >= 3 * gpr ? 1 : 0);
                    const unsigned y = (unsigned)(y0 + r), x = (unsigned)(xs + 4 * (local - r * gpr));
                    const bool ok = (unsigned)local < (unsigned)(4 * gpr) && y < Hu && x < Wu;
                    voff[k] = ok ? (gbase + (int)y * p.W + (int)x) * 4 : voff[k];
                }
#pragma unroll
                for (int fn = 0; fn < FN; fn++) {
                    const int n = n0 + fn * 32 + l32;
                    if (n >= seg_n && n < seg_n + cnt) my_base[fn] = base + shift + 2 * (n - seg_n), my_stride[fn] = 4 * gpr;
                }
                base += 16 * gpr;
            } else {
                // (only the loads that carry slots of this segment; selects instead of branches: this runs once per
                // workgroup, in front of everything else, on a SIMD that other workgroups keep busy)
                const int k_lo = base >> 6, k_hi = (base + 4 * width - 1) >> 6;
#pragma unroll
                for (int k = 0; k < WLC; k++) {
                    if (k < k_lo || k > k_hi) continue;  // (uniform)
                    const int local = k * 64 + lane - base;
                    const int r = (local >= width ? 1 : 0) + (local >= 2 * width ? 1 : 0) + (local >= 3 * width ? 1 : 0);
                    const unsigned y = (unsigned)(y0 + r), x = (unsigned)(x0 + local - r * width);
                    const bool ok = (unsigned)local < (unsigned)(4 * width) && y < Hu && x < Wu;
                    int off;
                    if (whole) off = (gbase + (int)y * p.W + (int)x) * 4;
                    else off = (gbase + (int)(y / (unsigned)p.uh) * p.W + (int)(x / (unsigned)p.uw)) * 4;
                    voff[k] = ok ? off : voff[k];
                }
#pragma unroll
                for (int fn = 0; fn < FN; fn++) {
                    const int n = n0 + fn * 32 + l32;
                    if (n >= seg_n && n < seg_n + cnt) my_base[fn] = base + 2 * (n - seg_n), my_stride[fn] = width;
                }
                base += 4 * width;
            }
            seg_n += cnt;
        }
        nload = WIDE ? (base + 255) >> 8 : (base + 63) >> 6;  // loads per channel that carry slots in use
    }
    const int HW4 = p.H * p.W * 4;
    const int32x4 dma_in = make_rsrc_words(p.I, p.in_bytes), dma_in2 = make_rsrc_words(p.I2, p.in_bytes);

    const bool whole_steps = p.Csplit == p.C || p.Csplit % CK == 0;
    auto load_step = [&](int step, lds_float *us, lds_float *rs, bool checked, bool filters = true) {
        if (filters) load_filters(step, us);
        // every channel of the step exists and lies in one tensor (nearly every step of every layer; a two-tensor input
        // whose first tensor ends on a step boundary): nothing is selected per load, the step picks its tensor once
        if (!checked && whole_steps) {
            const bool second = step * CK >= p.Csplit;
            const int32x4 dma = second ? dma_in2 : dma_in;
            const int c0 = step * CK - (second ? p.Csplit : 0);
#pragma unroll
            for (int jc = 0; jc < CK / 4; jc++) {
                const int cl = wave + 4 * jc;
                const int soff = (c0 + cl) * HW4;
#pragma unroll
                for (int k = 0; k < WLC; k++)
                    if (k < nload) {
                        if constexpr (WIDE) lds_dma_b128(dma, rs + cl * SLOTS + k * 256, voff[k], soff);
                        else lds_dma_b32(dma, rs + cl * SLOTS + k * 64, voff[k], soff);
                    }
            }
            return;
        }
#pragma unroll
        for (int jc = 0; jc < CK / 4; jc++) {
            const int cl = wave + 4 * jc, c = step * CK + cl;
            const bool cok = !checked || c < p.C;
            const bool second = c >= p.Csplit;  // uniform in the wavefront: the channel comes from the second tensor
            const int soff = (cok ? (second ? c - p.Csplit : c) : 0) * HW4;
#pragma unroll
            for (int k = 0; k < WLC; k++)
                if (k < nload) {
                    if constexpr (WIDE) lds_dma_b128(second ? dma_in2 : dma_in, rs + cl * SLOTS + k * 256, cok ? voff[k] : OOB, soff);
                    else lds_dma_b32(second ? dma_in2 : dma_in, rs + cl * SLOTS + k * 64, cok ? voff[k] : OOB, soff);
                }
        }
    };

    floatx16 acc[4][FM][FN];
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int fm = 0; fm < FM; fm++)
#pragma unroll
            for (int fn = 0; fn < FN; fn++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[j][fm][fn][v] = 0.0f;

    // position row i = wave: patch rows ra and rb, combined as d[ra] + d[rb] (i = 1) or d[ra] - d[rb]
    const int ra = wave == 0 ? 0 : (wave == 2 ? 2 : 1), rb = wave == 0 ? 2 : (wave == 1 ? 2 : (wave == 2 ? 1 : 3));
    const float sgn = wave == 1 ? 1.0f : -1.0f;
    const int a_off = (half * 16 + 4 * wave) * MF + l32;
    int ra_off[FN], rb_off[FN];  // this lane's two patch rows, as LDS offsets within a step's pixels (channel `half` of a pair)
#pragma unroll
    for (int fn = 0; fn < FN; fn++) {
        ra_off[fn] = half * SLOTS + my_base[fn] + ra * my_stride[fn];
        rb_off[fn] = half * SLOTS + my_base[fn] + rb * my_stride[fn];
    }

    // The K loop, software-pipelined over channel pairs and across K-steps: the operands of the pair after the current one
    // are read from LDS, and its B operands derived, while the matrix instructions of the current pair are issued (a
    // matrix instruction occupies its pipe for 64 cycles; the reads go first - their results are needed soonest).  Per
    // pair: 2 FM + 4 FN two-address LDS reads, 12 FN vector instructions, 4 FM FN matrix instructions.  The first pair of
    // a step is read right after the barrier that publishes the step's buffer, in front of the second half of the last
    // pair's matrix instructions of the step before.
    static_assert((CK / 2) % 2 == 0, "the first pair of a step always lands in operand set 0");
    float a[2][4][FM], d[2][4][FN], vv[2][4][FN];
    auto read_pair = [&](const lds_float *__restrict__ us, const lds_float *__restrict__ rs, int cp, int into) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int fm = 0; fm < FM; fm++) a[into][j][fm] = us[a_off + cp * (32 * MF) + j * MF + fm * 32];
#pragma unroll
        for (int fn = 0; fn < FN; fn++) {
            if constexpr (WIDE) {  // (a patch may start at an odd slot: pairs of 4-byte reads)
                const lds_float *pa = rs + ra_off[fn] + cp * (2 * SLOTS), *pb = rs + rb_off[fn] + cp * (2 * SLOTS);
                d[0][0][fn] = pa[0], d[0][1][fn] = pa[1], d[0][2][fn] = pa[2], d[0][3][fn] = pa[3];
                d[1][0][fn] = pb[0], d[1][1][fn] = pb[1], d[1][2][fn] = pb[2], d[1][3][fn] = pb[3];
            } else {  // (a patch starts at an even slot: 8-byte reads)
                typedef float floatx2 __attribute__((ext_vector_type(2)));
                typedef const __attribute__((address_space(3))) floatx2 *lds_f2;
                const floatx2 a0 = *(lds_f2)(rs + ra_off[fn] + cp * (2 * SLOTS)), a1 = *(lds_f2)(rs + ra_off[fn] + cp * (2 * SLOTS) + 2);
                const floatx2 b0 = *(lds_f2)(rs + rb_off[fn] + cp * (2 * SLOTS)), b1 = *(lds_f2)(rs + rb_off[fn] + cp * (2 * SLOTS) + 2);
                d[0][0][fn] = a0.x, d[0][1][fn] = a0.y, d[0][2][fn] = a1.x, d[0][3][fn] = a1.y;
                d[1][0][fn] = b0.x, d[1][1][fn] = b0.y, d[1][2][fn] = b1.x, d[1][3][fn] = b1.y;
            }
        }
    };
    auto transform = [&](int into) __attribute__((always_inline)) {
#pragma unroll
        for (int fn = 0; fn < FN; fn++) {
            float u[4];
#pragma unroll
            for (int s = 0; s < 4; s++) u[s] = __builtin_fmaf(d[1][s][fn], sgn, d[0][s][fn]);  // d[ra] + d[rb] or d[ra] - d[rb]: one rounding either way
            vv[into][0][fn] = __fsub_rn(u[0], u[2]);
            vv[into][1][fn] = __fadd_rn(u[1], u[2]);
            vv[into][2][fn] = __fsub_rn(u[2], u[1]);
            vv[into][3][fn] = __fsub_rn(u[1], u[3]);
        }
    };
    auto mfmas = [&](int cur, int j_lo, int j_hi) __attribute__((always_inline)) {  // positions j_lo .. j_hi - 1 of the row
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int fm = 0; fm < FM; fm++)
#pragma unroll
                for (int fn = 0; fn < FN; fn++)
                    if (j >= j_lo && j < j_hi)
                        acc[j][fm][fn] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][j][fm], vv[cur][j][fn], acc[j][fm][fn], 0, 0, 0);
    };
    constexpr int NDS = 2 * FM + 2 * FN, NVALU = 12 * FN, NMFMA = 4 * FM * FN;

    auto us_of = [&](int buf) { return (lds_float *)&lds[buf * BUF_FLOATS]; };
    auto rs_of = [&](int buf) { return (lds_float *)&lds[buf * BUF_FLOATS + U_FLOATS]; };
    const int full_steps = p.C / CK;
    constexpr int WAIT_ALL = 0x0F70;  // vmcnt(0): this wavefront's LDS-direct loads have landed
    load_step(step_lo, us_of(0), rs_of(0), step_lo >= full_steps, false);  // (its filters were requested at the start)
    if (!split) put_channel_constants<MF>(epi, chan, tid);  // (published by the barrier below)
    __builtin_amdgcn_s_waitcnt(WAIT_ALL);
    __syncthreads();
    trace_mark(p, 1);
    read_pair(us_of(0), rs_of(0), 0, 0);
    transform(0);
    for (int step = step_lo; step < step_hi; step++) {
        const int cur = (step - step_lo) & 1, nxt = cur ^ 1;
        if (step + 1 < step_hi) load_step(step + 1, us_of(nxt), rs_of(nxt), step + 1 >= full_steps);
        const lds_float *us = us_of(cur), *rs = rs_of(cur);
#pragma unroll
        for (int cp = 0; cp + 1 < CK / 2; cp++) {
            const int set = cp & 1;
            read_pair(us, rs, cp + 1, set ^ 1);
            transform(set ^ 1);
            mfmas(set, 0, 4);
            wino_sched_pair<NDS, NVALU, NMFMA / 2, NMFMA - NMFMA / 2, 0>();
        }
        // the last pair of the step: its matrix instructions straddle the barrier and the reads of the next step's first
        // pair (after the last step these reads fetch the other buffer's stale contents, which nothing uses)
        mfmas(1, 0, 2);
        __builtin_amdgcn_sched_barrier(0);  // (nothing moves across: the wait comes after the first half's matrix instructions)
        __builtin_amdgcn_s_waitcnt(WAIT_ALL);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        read_pair(us_of(nxt), rs_of(nxt), 0, 0);
        mfmas(1, 2, 4);
        transform(0);
        __builtin_amdgcn_sched_group_barrier(0x100, NDS, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, NMFMA / 2, 0);
    }
    trace_mark(p, 2);

    // ---- output transform: along the position row in registers, across the rows through LDS, then the epilogue
    const size_t plane = (size_t)p.wP * p.wQ;
    const bool pair = (p.wQ % 2 == 0) && (((size_t)p.O | (size_t)(p.residual ? p.residual : p.O)) % 8 == 0);
    float *xch = &lds[0];
#pragma unroll
    for (int fm = 0; fm < FM; fm++)
#pragma unroll
        for (int fn = 0; fn < FN; fn++) {
            if (fm + fn > 0) __syncthreads();  // the reads of the block before are done
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const float s0 = __fadd_rn(__fadd_rn(acc[0][fm][fn][v], acc[1][fm][fn][v]), acc[2][fm][fn][v]);
                const float s1 = __fsub_rn(__fsub_rn(acc[1][fm][fn][v], acc[2][fm][fn][v]), acc[3][fm][fn][v]);
                xch[((wave * 2 + 0) * 16 + v) * 64 + lane] = s0;
                xch[((wave * 2 + 1) * 16 + v) * 64 + lane] = s1;
            }
            __syncthreads();
            const int n = n0 + fn * 32 + l32;
            const int nc = n < p.wT ? n : 0;
            const int img = nc / per_img, r = nc - img * per_img, ty = r / p.wtw, tx = r - ty * p.wtw;
            float yk[4][2][2];  // [k][a][b]: output (2 ty + a, 2 tx + b) of filter row 8 wave + 4 half + k of the block
#pragma unroll
            for (int k = 0; k < 4; k++)
#pragma unroll
                for (int b = 0; b < 2; b++) {
                    float t[4];
#pragma unroll
                    for (int i = 0; i < 4; i++) t[i] = xch[((i * 2 + b) * 16 + 4 * wave + k) * 64 + lane];
                    yk[k][0][b] = __fadd_rn(__fadd_rn(t[0], t[1]), t[2]);
                    yk[k][1][b] = __fsub_rn(__fsub_rn(t[1], t[2]), t[3]);
                }
            const int ml0 = fm * 32 + 8 * wave + 4 * half;
            if (split) {
                // this slice's share of the four outputs, raw: wino_fused_reduce_kernel adds the slices and finishes
                // (layout [slice][tile][32x32 block][wavefront][k][lane] of four floats: a store writes 1 KB)
                const size_t tiles = (gridDim.x - (unsigned)p.main_tiles) / p.nslices;
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    floatx4 *dst = reinterpret_cast<floatx4 *>(p.partial) +
                                   (((((size_t)slice * tiles + local_tile) * (FM * FN) + fm * FN + fn) * 4 + wave) * 4 + k) * 64 + lane;
                    floatx4 yv;
                    yv.x = yk[k][0][0], yv.y = yk[k][0][1], yv.z = yk[k][1][0], yv.w = yk[k][1][1];
                    *dst = yv;
                }
            } else if (n < p.wT) {
                if (pair && 2 * ty + 1 < p.wP && 2 * tx + 1 < p.wQ && m0 + ml0 + 3 < p.Kf) {
                    wino_store_rows<MF, 4>(p, epi, ml0, m0 + ml0, img, ty, tx, plane, yk);
                } else {
#pragma unroll
                    for (int k = 0; k < 4; k++)
                        wino_store_row(p, channel_from_lds<MF>(epi, ml0 + k), m0 + ml0 + k, img, ty, tx, plane, pair, yk[k][0][0], yk[k][0][1], yk[k][1][0],
                                       yk[k][1][1]);
                }
            }
        }
    if (p.trace != nullptr) {
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        trace_mark(p, 3);
    }
}

// Finishes the tiles of wino_fused_kernel that the launch plan divided along the channels: one workgroup per 32x32 block of
// such a tile, the fused kernel's thread -> (filter row, block) mapping; adds the slices' four raw outputs in increasing
// channel order, starting from slice 0's values (a fixed order: results do not depend on scheduling), then the epilogue.
template <int FM, int FN>
__global__ __launch_bounds__(256) void wino_fused_reduce_kernel(const ConvParams p) {
    constexpr int MF = 32 * FM, NB = 32 * FN;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31, half = lane >> 5;
    const int blk = blockIdx.x % (FM * FN), local_tile = blockIdx.x / (FM * FN), fm = blk / FN, fn = blk % FN;
    const size_t tiles = gridDim.x / (FM * FN);
    const int tile = p.main_tiles + local_tile;
    const int m_first = (tile % p.gm) * MF + fm * 32 + 8 * wave + 4 * half;  // this lane's rows: m_first + 0..3
    const int n = (tile / p.gm) * NB + fn * 32 + l32;
    ChannelEpilogue chan[4];
#pragma unroll
    for (int k = 0; k < 4; k++) chan[k] = load_channel(p, m_first + k < p.Kf ? m_first + k : p.Kf - 1);
    const size_t slice_stride = tiles * (FM * FN) * 4 * 4 * 64;
    const floatx4 *src = reinterpret_cast<const floatx4 *>(p.partial) + ((((size_t)local_tile * (FM * FN) + blk) * 4 + wave) * 4) * 64 + lane;
    floatx4 y[4];
#pragma unroll
    for (int k = 0; k < 4; k++) y[k] = src[k * 64];
    for (int sl = 1; sl < p.nslices; sl++) {
        floatx4 x[4];
#pragma unroll
        for (int k = 0; k < 4; k++) x[k] = src[(size_t)sl * slice_stride + k * 64];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            y[k].x = __fadd_rn(y[k].x, x[k].x);
            y[k].y = __fadd_rn(y[k].y, x[k].y);
            y[k].z = __fadd_rn(y[k].z, x[k].z);
            y[k].w = __fadd_rn(y[k].w, x[k].w);
        }
    }
    if (n >= p.wT) return;
    const int per_img = p.wth * p.wtw;
    const int img = n / per_img, r = n - img * per_img, ty = r / p.wtw, tx = r - ty * p.wtw;
    const size_t plane = (size_t)p.wP * p.wQ;
    const bool pair = (p.wQ % 2 == 0) && (((size_t)p.O | (size_t)(p.residual ? p.residual : p.O)) % 8 == 0);
#pragma unroll
    for (int k = 0; k < 4; k++) wino_store_row(p, chan[k], m_first + k, img, ty, tx, plane, pair, y[k].x, y[k].y, y[k].z, y[k].w);
}

// ---------------------------------------------------------------- host side
int g_algo = 0;
// Measurement: while collecting, every launch of a convolution kernel (not the filter repack, not
// the K-split finishing kernel) is bracketed by its own pair of events on the launch stream.
bool g_prof_on = false;
std::vector<std::pair<hipEvent_t, hipEvent_t>> g_prof_pairs;  // recorded since collection was switched on
std::vector<std::pair<hipEvent_t, hipEvent_t>> g_prof_free;   // reusable

int prof_begin(hipStream_t st) {
    if (!g_prof_on) return 0;
    std::pair<hipEvent_t, hipEvent_t> pr;
    if (!g_prof_free.empty()) {
        pr = g_prof_free.back();
        g_prof_free.pop_back();
    } else {
        EH_TRY_HIP(hipEventCreate(&pr.first));
        EH_TRY_HIP(hipEventCreate(&pr.second));
    }
    g_prof_pairs.push_back(pr);
    EH_TRY_HIP(hipEventRecord(pr.first, st));
    return 0;
}

int prof_end(hipStream_t st) {
    if (!g_prof_on) return 0;
    EH_TRY_HIP(hipEventRecord(g_prof_pairs.back().second, st));
    return 0;
}
thread_local char g_last_kernel[128] = "";
int g_split = 1;  // divide the tiles left over after a whole number per CU along K (set_algo 5 turns it off)
bool g_wino = false;  // set_algo(7): the Winograd form wherever it applies (8: only where a searched plan asks for it)
bool g_wino_never = false;  // set_algo(9): no Winograd form at all, not in the plan search and not from a kept plan
thread_local int g_force_tile = -1, g_force_slices = -1;  // eddlhip_conv2d_force_plan (per calling thread: the plan search steers its own launches with them)
unsigned long long *g_trace = nullptr;       // eddlhip_conv2d_trace
long long g_trace_wgs = 0;

// eddlhip_conv2d_autotune: launch plans found by measurement, by device and geometry.  Neither the epilogue nor the form of
// the input is part of the key (image size and paddings - a folded Pad layer changes both -, one tensor or two, stored or
// upsampled image): what a plan fixes, tile shape and K slices, meets the same channels, filter and output pixels either
// way, and a convolution sums in the same order in a fused plan and in a layer-by-layer one.  One exception: a 2x2 filter
// on an input upsampled twice has a form that only that call can take (conv_up2x2_kernel), so it is a geometry of its own
// (kind + 2).
struct TunedPlan {
    int key[10];       // N C Kf R S sr sc P Q kind (0 / 1: register-staged / LDS-direct gather; + 2: see above)
    int tile, slices;  // tile -1: the planner's own choice was the fastest; tile 4: the Winograd form
};
bool g_autotune = false;
thread_local bool g_tuning = false;  // this thread is inside a plan search: the convolutions it times start no search of their own
std::vector<TunedPlan> g_tuned[EDDLHIP_MAX_DEVICES];

struct Variant {
    const char *name;
    int bm, bn, cpb;  // cpb = channels per K-step (0: the 16-tap kernel for any filter shape)
    void (*kernel)(const ConvParams);
    void (*reduce)(const ConvParams);
    mutable int occupancy;  // resident workgroups per CU, asked of the runtime on first use
};

#define TAP(WM, WN, TM, TN, R, S, CPB, D)                                                                                     \
    {                                                                                                                         \
        "conv_tap_kernel<" #WM "," #WN "," #TM "," #TN "," #R "," #S "," #CPB "," #D ">", WM *TM * 32, WN *TN * 32, CPB,       \
            conv_tap_kernel<WM, WN, TM, TN, R, S, CPB, D>, conv_reduce_kernel<WM, WN, TM, TN>, 0                              \
    }
#define GEN(WM, WN, TM, TN, D)                                                                                     \
    {                                                                                                              \
        "conv_gen_kernel<" #WM "," #WN "," #TM "," #TN "," #D ">", WM *TM * 32, WN *TN * 32, 0,                     \
            conv_gen_kernel<WM, WN, TM, TN, D>, conv_reduce_kernel<WM, WN, TM, TN>, 0                              \
    }

// Per filter shape: [gather kind: register-staged, LDS-direct][tile: 128x128, 64x128, 64x64, 32x128]
const Variant k3x3[2][4] = {
    {TAP(2, 2, 2, 2, 3, 3, 2, false), TAP(1, 4, 2, 1, 3, 3, 2, false), TAP(2, 2, 1, 1, 3, 3, 4, false), TAP(1, 4, 1, 1, 3, 3, 2, false)},
    {TAP(2, 2, 2, 2, 3, 3, 2, true), TAP(1, 4, 2, 1, 3, 3, 2, true), TAP(2, 2, 1, 1, 3, 3, 4, true), TAP(1, 4, 1, 1, 3, 3, 2, true)}};
const Variant k1x1[2][4] = {
    {TAP(2, 2, 2, 2, 1, 1, 16, false), TAP(1, 4, 2, 1, 1, 1, 16, false), TAP(2, 2, 1, 1, 1, 1, 16, false), TAP(1, 4, 1, 1, 1, 1, 16, false)},
    {TAP(2, 2, 2, 2, 1, 1, 16, true), TAP(1, 4, 2, 1, 1, 1, 16, true), TAP(2, 2, 1, 1, 1, 1, 16, true), TAP(1, 4, 1, 1, 1, 1, 16, true)}};
const Variant k2x2[2][4] = {
    {TAP(2, 2, 2, 2, 2, 2, 4, false), TAP(1, 4, 2, 1, 2, 2, 4, false), TAP(2, 2, 1, 1, 2, 2, 4, false), TAP(1, 4, 1, 1, 2, 2, 4, false)},
    {TAP(2, 2, 2, 2, 2, 2, 4, true), TAP(1, 4, 2, 1, 2, 2, 4, true), TAP(2, 2, 1, 1, 2, 2, 4, true), TAP(1, 4, 1, 1, 2, 2, 4, true)}};
const Variant kgen[2][4] = {{GEN(2, 2, 2, 2, false), GEN(1, 4, 2, 1, false), GEN(2, 2, 1, 1, false), GEN(1, 4, 1, 1, false)},
                            {GEN(2, 2, 2, 2, true), GEN(1, 4, 2, 1, true), GEN(2, 2, 1, 1, true), GEN(1, 4, 1, 1, true)}};

// The one-launch Winograd form's tile shapes: 32 FM filters x 32 FN blocks, CK channels per K-step.
struct FusedVariant {
    const char *name, *name_wide;
    int fm, fn, ck;
    void (*kernel)(const ConvParams);
    void (*kernel_wide)(const ConvParams);  // the build that loads the pixels 16 bytes per lane (conv2d_winograd_fused decides)
    void (*reduce)(const ConvParams);
};
#define FUSED(FM, FN, CK, WPE)                                                                                                       \
    {"wino_fused_kernel<" #FM "," #FN "," #CK "," #WPE ">", "wino_fused_kernel<" #FM "," #FN "," #CK "," #WPE ",true>", FM, FN, CK,  \
     wino_fused_kernel<FM, FN, CK, WPE, false>,         wino_fused_kernel<FM, FN, CK, WPE, true>, wino_fused_reduce_kernel<FM, FN>}
const FusedVariant kfused[] = {FUSED(1, 1, 4, 4), FUSED(2, 1, 4, 3)};
constexpr int NUM_FUSED = (int)(sizeof(kfused) / sizeof(kfused[0]));
constexpr int FUSED_TILE0 = 6;      // plan "tile" numbers 6 .. 6 + NUM_FUSED - 1 name these shapes (0..3: direct tiles, 4 / 5: the other Winograd forms)
constexpr int FUSED_ROW_ALIGN = 8;  // the transformed filters are padded to whole K-steps of every variant
constexpr int UP2X2_TILE = FUSED_TILE0 + NUM_FUSED;  // plan "tiles" of the upsampled-input form of a 2x2 convolution: conv_up2x2_kernel<3>, <2>
constexpr int NUM_PLAN_TILES = UP2X2_TILE + 2;

// K slices of the left-over tiles of a one-launch Winograd plan that asks for `slices` of them (T blocks in the launch):
// the tiles beyond a whole number per CU are divided, as in forced_plan; 1 = nothing is divided
int fused_slices(const FusedVariant &fv, int slices, long long T, int C, int Kf, int num_cu, long long *leftover_out = nullptr, int *slice_steps_out = nullptr) {
    const int nsteps = (C + fv.ck - 1) / fv.ck;
    const long long tiles = (long long)((Kf + 32 * fv.fm - 1) / (32 * fv.fm)) * ((T + 32 * fv.fn - 1) / (32 * fv.fn));
    const long long leftover = tiles % num_cu;
    const int want = slices < 1 ? 1 : (slices > nsteps ? nsteps : slices);
    int slice_steps = (nsteps + want - 1) / want;
    int nslices = (nsteps + slice_steps - 1) / slice_steps;
    if (leftover == 0) nslices = 1;
    if (nslices == 1) slice_steps = nsteps;
    if (leftover_out) *leftover_out = nslices > 1 ? leftover : 0;
    if (slice_steps_out) *slice_steps_out = slice_steps;
    return nslices;
}

// Launch plan: tile shape and, for the tiles that do not divide evenly over the CUs, the number
// of K slices.  The MFMA pipe of a CU is shared by its resident workgroups, so a launch takes as
// long as the busiest CU's share of the tiles: 784 tiles of 128x128 (28x28x512 at batch 32) on 256
// CUs cost four tile times where the average CU has 3.06 tiles.  The tiles beyond a whole number
// per CU ("leftover") can be divided along K over several workgroups each, so that they, too,
// spread over the whole device; conv_reduce_kernel then adds the slices in a fixed order.  The
// whole tiles come first in the grid and the slices after them, in ONE launch, so the slices fill
// CUs as whole tiles retire.  The plan minimises a simple time estimate over the four tile shapes
// and 1..16 slices:
//   a K-step of a tile costs its flops over (CU peak x tile efficiency); a workgroup costs its
//   K-steps plus a fixed prologue/epilogue; a CU with few resident workgroups hides less latency;
//   divided tiles add the traffic of their partial sums and one more launch.
struct Plan {
    int tile, nsteps, nslices, slice_steps;
    long long tiles, leftover;
    double cost_us;
};

Plan plan_conv(const Variant *family, int Kf, int C, int RS, long long npix, int num_cu, bool allow_split) {
    static const double kEff[4] = {0.90, 0.905, 0.87, 0.86};      // fraction of the MFMA peak a long K loop sustains, per tile shape
    static const double kOverheadUs[4] = {5.0, 3.0, 1.5, 2.0};   // prologue + epilogue of one workgroup (CU time)
    const double cu_flops_per_us = 157.3e6 / 256.0;
    const double bytes_per_us = 3.0e6;  // partial-sum traffic
    // a CU with fewer resident workgroups than it can hold hides less latency
    auto crowd = [](long long resident) { return resident >= 3 ? 1.0 : (resident == 2 ? 0.9 : 0.73); };
    Plan best;
    best.cost_us = -1.0;
    for (int t = 0; t < 4; t++) {
        const Variant &v = family[t];
        // wide tiles only pay off when the filters fill them
        if ((v.bm == 128 && Kf <= 64) || (v.bm == 64 && Kf <= 32)) continue;
        const int bk = v.cpb ? v.cpb * RS : 16;
        const int nsteps = v.cpb ? (C + v.cpb - 1) / v.cpb : (C * RS + 15) / 16;
        const long long tiles = (long long)((Kf + v.bm - 1) / v.bm) * ((npix + v.bn - 1) / v.bn);
        const long long full = tiles / num_cu, left = tiles % num_cu;
        const double step_us = 2.0 * v.bm * v.bn * bk / (cu_flops_per_us * kEff[t]);
        const double tile_us = nsteps * step_us + kOverheadUs[t];
        const int smax = (allow_split && left > 0) ? (nsteps / 4 < 16 ? nsteps / 4 : 16) : 1;
        for (int want = 1; want <= (smax < 1 ? 1 : smax); want++) {
            const int ss = (nsteps + want - 1) / want;
            const int sl = (nsteps + ss - 1) / ss;
            if (sl != want && want != 1) continue;  // same plan as a smaller `want`
            const long long wgs = left * sl;
            const long long per_cu = (wgs + num_cu - 1) / num_cu;
            // a CU works through its `full` whole tiles `occupancy` at a time; the last, smaller group
            // (plus the K slices, which are short) runs with fewer wavefronts to hide latency
            const long long occ = v.occupancy;
            const long long tail = full % occ;
            double cost = (double)(full - tail) * tile_us / crowd(occ);
            if (tail > 0) cost += (double)tail * tile_us / crowd(tail + (per_cu > 0 ? 1 : 0));
            if (per_cu > 0) {
                const long long resident = (tail > 0 ? tail : (full > 0 ? occ - 1 : 0)) + per_cu;
                cost += (double)per_cu * (ss * step_us + kOverheadUs[t]) / crowd(resident < occ ? resident : occ);
            }
            if (sl > 1) cost += (double)wgs * v.bm * v.bn * 8.0 / bytes_per_us + 6.0;
            if (best.cost_us < 0 || cost < best.cost_us) {
                best.tile = t;
                best.nsteps = nsteps;
                best.nslices = sl;
                best.slice_steps = ss;
                best.tiles = tiles;
                best.leftover = left;
                best.cost_us = cost;
            }
        }
    }
    return best;
}

// Resident workgroups per CU of each variant of a family, asked of the runtime once.
int family_occupancy(const Variant *family) {
    for (int t = 0; t < 4; t++) {
        if (family[t].occupancy == 0) {
            int occ = 0;
            EH_TRY_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, family[t].kernel, 256, 0));
            family[t].occupancy = occ > 0 ? occ : 1;
        }
    }
    return 0;
}

// A plan with a given tile shape and slice count (every leftover tile is divided; with fewer
// tiles than CUs that is every tile).
Plan forced_plan(const Variant *family, int tile, int slices, int Kf, int C, int RS, long long npix, int num_cu) {
    const Variant &v = family[tile];
    Plan pl;
    pl.tile = tile;
    pl.nsteps = v.cpb ? (C + v.cpb - 1) / v.cpb : (C * RS + 15) / 16;
    pl.tiles = (long long)((Kf + v.bm - 1) / v.bm) * ((npix + v.bn - 1) / v.bn);
    pl.leftover = pl.tiles % num_cu;
    int want = slices < 1 ? 1 : (slices > pl.nsteps ? pl.nsteps : slices);
    pl.slice_steps = (pl.nsteps + want - 1) / want;
    pl.nslices = (pl.nsteps + pl.slice_steps - 1) / pl.slice_steps;
    if (pl.leftover == 0) pl.nslices = 1, pl.slice_steps = pl.nsteps;
    pl.cost_us = 0.0;
    return pl;
}


// ---------------------------------------------------------------- cache of repacked filters
// A caller that keeps its filters fixed between calls (inference) registers them once
// (eddlhip_conv2d_cache_filters); eddlhip_conv2d_fwd then finds the repacked copy by the filter
// pointer and skips pack_filters_kernel.  Rows are in OIHW tap order for every kernel variant and
// only the zero padding behind them differs, so one copy padded for the largest K-step serves all.
struct CachedFilters {
    const float *K;
    int Kf, C, R, S, rows, Mp;
    float *Wp;
    float *Wwino;  // 3x3 (2x2) filters: the 16 (9) transformed matrices of the Winograd form [16][wino_rows][Mp], made on first use
    int wino_rows;
    float *Wfused;  // 3x3 filters: the transformed filters of the one-launch Winograd form [fused_rows][16][Mp], made on first use
    int fused_rows;
    float *Wup;  // 2x2 filters: the nine weight-sum rows per channel of the upsampled-input form [C][9][Mp] (up2x2_filter_kernel), made on first use
    bool stale;  // K was written through this library since the last repack
};
std::mutex g_cache_mutex;
std::vector<CachedFilters> g_cache[EDDLHIP_MAX_DEVICES];

int cache_rows(int C, int R, int S) {
    const int RS = R * S, crs = C * RS;
    int rows = (crs + 15) / 16 * 16;  // the 16-tap kernel
    for (int cpb : {2, 4, 16}) {
        const int r = (C + cpb - 1) / cpb * cpb * RS;
        if (r > rows) rows = r;
    }
    return rows;
}

int repack(int dev, CachedFilters &e) {
    hipLaunchKernelGGL(pack_filters_kernel, dim3((e.rows + 31) / 32, e.Mp / 32), dim3(256), 0, state(dev).stream, e.K, e.Wp, e.Kf,
                       e.C * e.R * e.S, e.Mp, e.rows);
    EH_CHECK_LAUNCH();
    if (e.Wwino != nullptr) {
        const dim3 grid((unsigned)(((size_t)e.wino_rows * e.Mp + 255) / 256));
        if (e.R == 3) hipLaunchKernelGGL(wino_filter_kernel<4>, grid, dim3(256), 0, state(dev).stream, e.K, e.Wwino, e.Kf, e.C, e.Mp, e.wino_rows, 0);
        else hipLaunchKernelGGL(wino_filter_kernel<3>, grid, dim3(256), 0, state(dev).stream, e.K, e.Wwino, e.Kf, e.C, e.Mp, e.wino_rows, 0);
        EH_CHECK_LAUNCH();
    }
    if (e.Wfused != nullptr) {
        const dim3 grid((unsigned)(((size_t)e.fused_rows * e.Mp + 255) / 256));
        hipLaunchKernelGGL(wino_filter_kernel<4>, grid, dim3(256), 0, state(dev).stream, e.K, e.Wfused, e.Kf, e.C, e.Mp, e.fused_rows, 1);
        EH_CHECK_LAUNCH();
    }
    if (e.Wup != nullptr) {
        hipLaunchKernelGGL(up2x2_filter_kernel, dim3((unsigned)(((size_t)e.C * e.Mp + 255) / 256)), dim3(256), 0, state(dev).stream, e.K, e.Wup, e.Kf, e.C, e.Mp);
        EH_CHECK_LAUNCH();
    }
    e.stale = false;
    return 0;
}

}  // namespace

namespace eddlhip {

// Called once per device from the library's initialisation, with that device current: looks up where this
// device keeps its copy of `scratch`, and asks the runtime how many workgroups of each kernel variant fit
// on a CU (the launch planner's input), so that eddlhip_conv2d_fwd_noalloc finds both ready.
int conv_setup_device(int dev) {
    void *ptr = nullptr;
    EH_TRY_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    EH_REQUIRE(ptr != nullptr, "device %d: no address for the convolution scratch array", dev);
    g_scratch_ptr[dev] = ptr;
    for (const Variant(*fam)[4] : {k3x3, k1x1, k2x2, kgen})
        for (int d = 0; d < 2; d++) EH_TRY(family_occupancy(fam[d]));
    return 0;
}

void conv_filters_written(int dev, const void *dst, size_t bytes) {
    if (dev < 0 || dev >= EDDLHIP_MAX_DEVICES) return;
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    const char *lo = (const char *)dst, *hi = lo + bytes;
    for (CachedFilters &e : g_cache[dev]) {
        const char *klo = (const char *)e.K, *khi = klo + (size_t)e.Kf * e.C * e.R * e.S * sizeof(float);
        if (lo < khi && klo < hi) e.stale = true;
    }
}

void conv_filters_released(int dev, const void *base, size_t bytes) {
    if (dev < 0 || dev >= EDDLHIP_MAX_DEVICES) return;
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    std::vector<CachedFilters> &c = g_cache[dev];
    const char *lo = (const char *)base, *hi = lo + bytes;
    for (size_t i = 0; i < c.size();) {
        if ((const char *)c[i].K >= lo && (const char *)c[i].K < hi) {
            // kernels still reading the packed copy finish first
            (void)hipStreamSynchronize(state(dev).stream);
            (void)hipFree(c[i].Wp);
            if (c[i].Wwino) (void)hipFree(c[i].Wwino);
            if (c[i].Wfused) (void)hipFree(c[i].Wfused);
            if (c[i].Wup) (void)hipFree(c[i].Wup);
            c[i] = c.back();
            c.pop_back();
        } else {
            i++;
        }
    }
}

}  // namespace eddlhip

extern "C" {

int eddlhip_conv2d_cache_filters(int dev, const float *K, int Kf, int C, int R, int S) {
    EH_REQUIRE(K != nullptr && Kf > 0 && C > 0 && R > 0 && S > 0, "conv2d_cache_filters: bad filter tensor %dx%dx%dx%d", Kf, C, R, S);
    EH_REQUIRE((long long)C * R * S <= (1LL << 24), "conv2d_cache_filters: filter too large");
    EH_TRY(use_device(dev));
    EH_NOT_CAPTURING(dev, "eddlhip_conv2d_cache_filters");
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    for (CachedFilters &e : g_cache[dev]) {
        if (e.K == K) {
            EH_REQUIRE(e.Kf == Kf && e.C == C && e.R == R && e.S == S,
                       "conv2d_cache_filters: pointer already registered with shape %dx%dx%dx%d", e.Kf, e.C, e.R, e.S);
            return repack(dev, e);
        }
    }
    CachedFilters e;
    e.K = K; e.Kf = Kf; e.C = C; e.R = R; e.S = S;
    e.rows = cache_rows(C, R, S);
    e.Mp = (Kf + M_ALIGN - 1) / M_ALIGN * M_ALIGN;
    e.Wp = nullptr;
    e.Wwino = nullptr;
    e.wino_rows = 0;
    e.Wfused = nullptr;
    e.fused_rows = 0;
    e.Wup = nullptr;
    e.stale = true;
    EH_REQUIRE((size_t)e.rows * e.Mp * sizeof(float) < ((size_t)1 << 31),
               "conv2d_cache_filters: the repacked filter matrix (%d taps x %d channels) exceeds the 2 GiB a buffer descriptor covers", e.rows, e.Mp);
    EH_TRY_HIP(hipMalloc((void **)&e.Wp, (size_t)e.rows * e.Mp * sizeof(float)));
    int rc = repack(dev, e);
    if (rc != 0) {
        (void)hipFree(e.Wp);
        return rc;
    }
    g_cache[dev].push_back(e);
    return 0;
}

int eddlhip_conv2d_uncache_filters(int dev, const float *K) {
    EH_TRY(use_device(dev));
    EH_NOT_CAPTURING(dev, "eddlhip_conv2d_uncache_filters");
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    std::vector<CachedFilters> &c = g_cache[dev];
    bool synced = false;
    for (size_t i = 0; i < c.size();) {
        if (K == nullptr || c[i].K == K) {
            if (!synced) EH_TRY_HIP(hipStreamSynchronize(state(dev).stream));
            synced = true;
            EH_TRY_HIP(hipFree(c[i].Wp));
            if (c[i].Wwino) EH_TRY_HIP(hipFree(c[i].Wwino));
            if (c[i].Wfused) EH_TRY_HIP(hipFree(c[i].Wfused));
            if (c[i].Wup) EH_TRY_HIP(hipFree(c[i].Wup));
            c[i] = c.back();
            c.pop_back();
        } else {
            i++;
        }
    }
    return 0;
}

int eddlhip_conv2d_force_plan(int tile, int slices) {
    EH_REQUIRE(tile >= -1 && tile < NUM_PLAN_TILES,
               "conv2d_force_plan: tile is -1 (automatic), 0..3, 4 .. %d (the Winograd forms where they apply) or %d, %d (a 2x2 filter on an input upsampled twice)",
               UP2X2_TILE - 1, UP2X2_TILE, UP2X2_TILE + 1);
    g_force_tile = tile;
    g_force_slices = slices;
    return 0;
}

int eddlhip_conv2d_trace(unsigned long long *words, long long workgroups) {
    EH_REQUIRE(workgroups >= 0 && (words != nullptr || workgroups == 0), "conv2d_trace: bad buffer");
    g_trace = workgroups > 0 ? words : nullptr;
    g_trace_wgs = workgroups;
    return 0;
}

int eddlhip_conv2d_autotune(int on) {
    g_autotune = on > 0;
    if (on < 0)
        for (auto &t : g_tuned) t.clear();
    return 0;
}

int eddlhip_conv2d_tuned_save(int dev, const char *host_path) {
    EH_REQUIRE(dev >= 0 && dev < EDDLHIP_MAX_DEVICES && host_path != nullptr, "conv2d_tuned_save: bad arguments");
    FILE *f = fopen(host_path, "w");
    EH_REQUIRE(f != nullptr, "conv2d_tuned_save: cannot write %s", host_path);
    fprintf(f, "# eddlhip tuned convolution plans: N C Kf R S sr sc P Q kind | tile slices\n");
    for (const TunedPlan &t : g_tuned[dev]) {
        for (int v : t.key) fprintf(f, "%d ", v);
        fprintf(f, "| %d %d\n", t.tile, t.slices);
    }
    const bool ok = fclose(f) == 0;
    EH_REQUIRE(ok, "conv2d_tuned_save: writing %s failed", host_path);
    return 0;
}

int eddlhip_conv2d_tuned_load(int dev, const char *host_path) {
    EH_REQUIRE(dev >= 0 && dev < EDDLHIP_MAX_DEVICES && host_path != nullptr, "conv2d_tuned_load: bad arguments");
    FILE *f = fopen(host_path, "r");
    EH_REQUIRE(f != nullptr, "conv2d_tuned_load: cannot read %s", host_path);
    std::vector<TunedPlan> read;
    char line[512];
    bool bad = false;
    while (fgets(line, sizeof(line), f) != nullptr) {
        if (line[0] == '#' || line[0] == '\n') continue;
        TunedPlan t;
        int *k = t.key;
        const int got = sscanf(line, "%d %d %d %d %d %d %d %d %d %d | %d %d", k, k + 1, k + 2, k + 3, k + 4, k + 5, k + 6, k + 7, k + 8, k + 9, &t.tile,
                               &t.slices);
        if (got != 12 || t.tile < -1 || t.tile >= NUM_PLAN_TILES || t.slices < 1 || t.slices > 16) {  // (no search tries more than 16 slices)
            bad = true;
            break;
        }
        read.push_back(t);
    }
    fclose(f);
    EH_REQUIRE(!bad, "conv2d_tuned_load: %s holds a line that is not a plan", host_path);
    for (const TunedPlan &t : read) {
        bool known = false;
        for (TunedPlan &have : g_tuned[dev])
            if (memcmp(have.key, t.key, sizeof(t.key)) == 0) {
                have = t;
                known = true;
            }
        if (!known) g_tuned[dev].push_back(t);
    }
    return 0;
}

int eddlhip_conv2d_tuned_plans(int dev) {
    EH_REQUIRE(dev >= 0 && dev < EDDLHIP_MAX_DEVICES, "conv2d_tuned_plans: bad device %d", dev);
    return (int)g_tuned[dev].size();
}

int eddlhip_conv2d_set_algo(int algo) {
    EH_REQUIRE(algo >= 0 && algo <= 9, "conv2d_set_algo: unknown algorithm %d", algo);
    if (algo == 5 || algo == 6) {
        g_split = (algo == 6);
        return 0;
    }
    if (algo >= 7 && algo <= 9) {
        g_wino = (algo == 7);
        g_wino_never = (algo == 9);
        return 0;
    }
    g_algo = algo;
    return 0;
}

int eddlhip_conv2d_profile(int collect) {
    for (auto &pr : g_prof_pairs) g_prof_free.push_back(pr);
    g_prof_pairs.clear();
    g_prof_on = collect != 0;
    return 0;
}

int eddlhip_conv2d_profile_read(int *launches, float *total_ms) {
    EH_REQUIRE(launches && total_ms, "conv2d_profile_read: NULL output");
    float sum = 0.0f;
    for (auto &pr : g_prof_pairs) {
        float ms = 0.0f;
        EH_TRY_HIP(hipEventSynchronize(pr.second));
        EH_TRY_HIP(hipEventElapsedTime(&ms, pr.first, pr.second));
        sum += ms;
    }
    *launches = (int)g_prof_pairs.size();
    *total_ms = sum;
    return 0;
}

const char *eddlhip_conv2d_last_kernel(void) { return g_last_kernel; }

}  // extern "C"

namespace {

// I2 == nullptr: the input is the one tensor I[N,C,H,W].  Otherwise channels [0, C/2) are I[N,C/2,H,W] and
// channels [C/2, C) are I2[N,C/2,H,W].
// uh, uw > 1: the convolution runs over I enlarged uh x uw times by nearest-neighbour repetition (H, W stay the stored size).
// no_alloc: take the scratch memory from the device's fixed array instead of the workspace, and refuse whatever
// would allocate (an uninitialised device, a need beyond the array, event pairs for the measurement hook).
// The 16 products of a Winograd convolution, run by conv2d_fwd_impl as a 1x1 convolution over 16 images: the packed
// transformed filters (one matrix per image, `stride` floats apart) come from the caller instead of the filter tensor.
struct GemmBatch {
    const float *Wp;
    size_t stride;
    // Workspace the launch may take (its partial tiles), which the Winograd driver leaves free in front of its own
    // buffers; with need_out set the call launches nothing and only reports what it would take: exactly, under the plan
    // that is fixed for its geometry, or the largest need of any plan while a search could still pick one.
    size_t reserve;
    size_t *need_out;
};
// eddlhip_conv2d_fwd_maxpool: the 2x2, stride-2 max-pool the caller wants of this thread's current convolution.  A
// Winograd form computes it in its epilogue and says so (`done`); after any other form the entry point launches the pool
// kernel on the convolution's output.
struct PoolRequest {
    float *O, *ix, *iy;
    bool keep;  // the unpooled output is wanted as well
    bool done;
};
thread_local PoolRequest *g_pool_req = nullptr;
// Workspace a product launch may take for the partial tiles of a K-split plan: fewer than one tile per CU left over,
// at most 16 slices each, 128 x 128 floats per tile.  The Winograd driver keeps its own buffers behind this much.
// The plan search tries the Winograd forms that keep a transformed input in memory only below this much workspace.
constexpr size_t WINO_SEARCH_CAP = (size_t)512 << 20;

int conv2d_winograd(bool fold, int fs, int dev, const float *I, const float *I2, int uh, int uw, const float *K, const float *bias, float *O, int N, int C,
                    int H, int W, int Kf, int pad_top, int pad_left, int P, int Q, const float *bn_g, const float *bn_b, const float *bn_mean,
                    const float *bn_var, float bn_eps, const float *residual, int relu);

int conv2d_winograd_fused(int variant, int slices, int dev, const float *I, const float *I2, int uh, int uw, const float *K, const float *bias, float *O,
                          int N, int C, int H, int W, int Kf, int pad_top, int pad_left, int P, int Q, const float *bn_g, const float *bn_b,
                          const float *bn_mean, const float *bn_var, float bn_eps, const float *residual, int relu);

int conv2d_up2x2(int variant, int dev, const float *I, const float *K, const float *bias, float *O, int N, int C, int H, int W, int Kf, int P, int Q, const float *bn_g,
                 const float *bn_b, const float *bn_mean, const float *bn_var, float bn_eps, const float *residual, int relu);

// Whether a convolution is the one conv_up2x2_kernel computes: a 2x2 stride-1 filter on ONE tensor upsampled twice in both
// directions, no padding above or to the left (below and to the right the image is followed by zeros, as many as the
// output size asks for), whole K-steps of 4 channels, and everything within 32-bit offsets.
bool up2x2_applies(int N, int C, int H, int W, int Kf, int R, int S, int sr, int sc, int uh, int uw, bool two, int pad_top, int pad_left, int P, int Q) {
    if (R != 2 || S != 2 || sr != 1 || sc != 1 || uh != 2 || uw != 2 || two || pad_top != 0 || pad_left != 0 || C % 4 != 0) return false;
    const long long T = (long long)N * ((P + 1) / 2) * ((Q + 1) / 2);
    const long long Mp = (Kf + M_ALIGN - 1) / M_ALIGN * M_ALIGN;
    return T <= 0x3fffff80LL && (long long)N * C * H * W * 4 < (1LL << 31) && 9LL * C * Mp * 4 < (1LL << 31);
}

// Whether the Winograd form can run this convolution: 3x3, stride 1, and the product launch within the limits of
// conv2d_fwd_impl (one "image" of transformed input or output below 1 GiB, fewer than 2^31 blocks).
bool winograd_applies(int N, int C, int Kf, int R, int S, int sr, int sc, int P, int Q) {
    if (R != S || (R != 3 && R != 2) || sr != 1 || sc != 1) return false;
    const long long T = (long long)N * ((P + 1) / 2) * ((Q + 1) / 2), Tp = (T + 127) / 128 * 128;
    return Tp <= 0x3fffff80LL && (long long)C * Tp <= (1LL << 28) && (long long)Kf * Tp <= (1LL << 28);
}
// ... with the output transform folded into the product launch (one launch over all 16 positions: the transformed input is
// then ONE image of 16 C channels, which a buffer descriptor must cover, and the channel runs must be whole K-steps)
bool winograd_fold_applies(int N, int C, int Kf, int R, int S, int sr, int sc, int P, int Q) {
    if (!winograd_applies(N, C, Kf, R, S, sr, sc, P, Q) || C % 16 != 0) return false;
    const long long T = (long long)N * ((P + 1) / 2) * ((Q + 1) / 2), Tp = (T + 127) / 128 * 128;
    const long long np = (R + 1) * (R + 1);
    return np * C * Tp * 4 < (1LL << 31) && np * C * ((Kf + M_ALIGN - 1) / M_ALIGN * M_ALIGN) * 4 < (1LL << 31);
}

int conv2d_fwd_impl(bool no_alloc, int dev, const float *I, const float *I2, int uh, int uw, const float *K, const float *bias, float *O, int N, int C,
                    int H, int W, int Kf, int R, int S, int sr, int sc, int pad_top, int pad_left, int P, int Q, const float *bn_g,
                    const float *bn_b, const float *bn_mean, const float *bn_var, float bn_eps, const float *residual, int relu,
                    const GemmBatch *gemm = nullptr);

// One convolution call, as the plan search repeats it.
struct ConvCall {
    int dev;
    const float *I, *I2;
    int uh, uw;
    const float *K, *bias;
    float *O;
    int N, C, H, W, Kf, R, S, sr, sc, pt, pl, P, Q;
    const float *bn_g, *bn_b, *bn_mean, *bn_var;
    float bn_eps;
    const float *residual;
    int relu;
};
int run_call(const ConvCall &c) {
    return conv2d_fwd_impl(false, c.dev, c.I, c.I2, c.uh, c.uw, c.K, c.bias, c.O, c.N, c.C, c.H, c.W, c.Kf, c.R, c.S, c.sr, c.sc, c.pt, c.pl, c.P, c.Q,
                           c.bn_g, c.bn_b, c.bn_mean, c.bn_var, c.bn_eps, c.residual, c.relu);
}

constexpr int kSearchSlices[8] = {1, 2, 3, 4, 6, 8, 12, 16};  // K-slice counts the search tries per tile shape

// What the Winograd forms that keep a transformed input take from the workspace (3x3: patch side 4, 2x2: 3): transformed
// filters unless kept, V, and for the three-kernel form M and room for the product launch's partial tiles.
size_t winograd_workspace(bool fold, int N, int C, int Kf, int fs, int P, int Q, int num_cu) {
    const size_t np = (size_t)(fs + 1) * (fs + 1);
    const size_t T = (size_t)N * ((P + 1) / 2) * ((Q + 1) / 2), Tp = (T + 127) / 128 * 128;
    const size_t rows = ((size_t)C + 15) / 16 * 16, Mp = ((size_t)Kf + M_ALIGN - 1) / M_ALIGN * M_ALIGN;
    size_t bytes = np * rows * Mp * 4 + np * C * Tp * 4;
    if (!fold) bytes += np * Kf * Tp * 4 + (size_t)16 * (num_cu - 1) * 128 * 128 * 4;
    return bytes;
}

// The plan search of eddlhip_conv2d_autotune (the reference finds its algorithm the same way, by measurement on a layer's
// first forward: src/hardware/gpu/nn/gpu_conv.cu:42-66, 211-213).  Runs the call under every launch plan on the call's own
// tensors (each plan writes the same output, up to the rounding of its summation order) in batches of about 0.3 ms of
// launches, after the planner's plan has run for 25 ms (settled clocks), re-times the plans near the front in turns, and
// takes each plan's FASTEST batch (noise only ever adds time).  Then, so that two searches of one geometry agree:
// of all plans within 3 % of the fastest one it keeps the first in a fixed order of preference - the planner's own plan,
// the one-launch Winograd form, the direct tiles, the Winograd forms with a transformed input in memory; within a form
// fewer K slices first.  Returns 0 with *out filled, 1 when these tensors cannot be searched on (the output overlaps an
// input: repeating the call would change what it reads), or minus the error code of a runtime failure.
int search_plan(const ConvCall &c, const Variant *family, const Plan &planned, long long chunk_pix, bool wino_ok, bool fold_ok, bool fused_ok, bool up_ok,
                TunedPlan *out) {
    {
        const size_t out_bytes = (size_t)c.N * c.Kf * c.P * c.Q * 4, in_bytes = (size_t)c.N * (c.I2 ? c.C / 2 : c.C) * c.H * c.W * 4;
        const char *o_lo = (const char *)c.O, *o_hi = o_lo + out_bytes;
        auto overlaps = [&](const float *ptr, size_t bytes) { return ptr != nullptr && (const char *)ptr < o_hi && o_lo < (const char *)ptr + bytes; };
        if (overlaps(c.I, in_bytes) || overlaps(c.I2, in_bytes) || overlaps(c.residual, out_bytes)) return 1;
    }
    hipStream_t st = state(c.dev).stream;
    const int num_cu = state(c.dev).num_cu;
    struct Cand {
        int rank, tile, slices;
        float ms;
    };
    std::vector<Cand> cands;
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess) return -set_error(EDDLHIP_EHIP, "conv2d plan search: hipEventCreate failed");
    if (hipEventCreate(&e1) != hipSuccess) {
        (void)hipEventDestroy(e0);
        return -set_error(EDDLHIP_EHIP, "conv2d plan search: hipEventCreate failed");
    }
    PoolRequest *const pool_req = g_pool_req;  // the candidates are timed as plain convolutions
    g_pool_req = nullptr;
    const int ft = g_force_tile, fs = g_force_slices;
    int fatal = 0;
    // `launches` back-to-back launches of the call under a plan between one pair of events: time per launch
    auto run_timed = [&](int tile, int slices, int launches, float *ms_per_launch) -> int {
        g_force_tile = tile;
        g_force_slices = slices;
        int rc = hipEventRecord(e0, st) == hipSuccess ? 0 : set_error(EDDLHIP_EHIP, "conv2d plan search: hipEventRecord failed");
        for (int i = 0; i < launches && rc == 0; i++) rc = run_call(c);
        float ms = 0.0f;
        if (rc == 0 && (hipEventRecord(e1, st) != hipSuccess || hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&ms, e0, e1) != hipSuccess))
            rc = set_error(EDDLHIP_EHIP, "conv2d plan search: timing a launch failed");
        g_force_tile = ft;
        g_force_slices = fs;
        *ms_per_launch = ms / (float)launches;
        return rc;
    };
    // a batch of launches lasts about 0.3 ms, so that the events' own cost and jitter stay small beside it
    auto batch_of = [](float ms) { return ms >= 0.3f ? 1 : (ms <= 0.0375f ? 8 : (int)(0.3f / ms + 0.999f)); };
    // First timing of a plan: one launch that also warms it up (filter transforms, workspace growth), then one batch.
    // EDDLHIP_EINVAL / EDDLHIP_ENOMEM: the plan does not apply here (skipped); any other failure ends the search.
    auto time_plan = [&](int rank, int tile, int slices) {
        if (fatal != 0) return;
        float first = 0.0f, ms = 0.0f;
        int rc = run_timed(tile, slices, 1, &first);
        if (rc == 0) rc = run_timed(tile, slices, batch_of(first), &ms);
        if (rc == 0) cands.push_back({rank, tile, slices, ms});
        else if (rc == EDDLHIP_EINVAL || rc == EDDLHIP_ENOMEM) clear_error();
        else fatal = rc;
    };
    g_tuning = true;
    {
        // the clocks settle under load within a few tens of milliseconds: the planner's plan runs that long first
        float ms = 0.0f, total = 0.0f;
        int rc = run_timed(-1, -1, 1, &ms);
        while (rc == 0 && total < 25.0f) {
            const int b = batch_of(ms);
            rc = run_timed(-1, -1, b, &ms);
            total += ms * (float)b + 0.01f;
        }
        if (rc != 0) fatal = rc;
    }
    time_plan(0, -1, -1);
    if (fatal == 0 && cands.empty()) fatal = set_error(EDDLHIP_EINVAL, "conv2d plan search: the planner's own plan did not run");
    if (up_ok) {  // (2x2 filters only: no rank shared with the one-launch Winograd form of 3x3 filters)
        time_plan(1, UP2X2_TILE, 1);
        time_plan(2, UP2X2_TILE + 1, 1);
    }
    if (fused_ok)  // the one-launch Winograd form: its tile shapes, each undivided and with the left-over tiles in K slices
        for (int fv = NUM_FUSED - 1; fv >= 0; fv--) {
            int last_slices = 0;
            for (int sl : kSearchSlices) {
                const int ns = fused_slices(kfused[fv], sl, (long long)c.N * ((c.P + 1) / 2) * ((c.Q + 1) / 2), c.C, c.Kf, num_cu);
                if (ns == last_slices) continue;  // the same plan as the one before
                last_slices = ns;
                time_plan(1 + (NUM_FUSED - 1 - fv), FUSED_TILE0 + fv, sl);
            }
        }
    for (int tile = 0; tile < 4; tile++) {
        int last_slices = 0;
        for (int sl : kSearchSlices) {
            const Plan fp = forced_plan(family, tile, sl, c.Kf, c.C, c.R * c.S, chunk_pix, num_cu);
            if (fp.nslices == last_slices) continue;
            last_slices = fp.nslices;
            if (tile == planned.tile && fp.nslices == planned.nslices && fp.slice_steps == planned.slice_steps) continue;  // the planner's own plan again
            time_plan(10 + tile, tile, sl);
        }
    }
    if (fold_ok && winograd_workspace(true, c.N, c.C, c.Kf, c.R, c.P, c.Q, num_cu) <= WINO_SEARCH_CAP) time_plan(20, 5, 1);
    if (wino_ok && fatal == 0 && winograd_workspace(false, c.N, c.C, c.Kf, c.R, c.P, c.Q, num_cu) <= WINO_SEARCH_CAP) {
        // the three-kernel form: its product launch is a geometry of its own, searched first (one untimed call with the
        // search open), then timed under what that search kept
        g_tuning = false;
        g_force_tile = 4;
        const int wrc = run_call(c);
        g_force_tile = ft;
        g_tuning = true;
        if (wrc == 0) time_plan(21, 4, 1);
        else if (wrc == EDDLHIP_EINVAL || wrc == EDDLHIP_ENOMEM) clear_error();
        else fatal = wrc;
    }
    // The plans within 10 % of the fastest are timed four more times, in turns (a drift of the clocks then meets all of them
    // alike), those within 6 % after that eight more times; a plan's time is its fastest batch.  While a plan then lies
    // within a per cent of the 3 % margin that decides below, it and the plans in front of it get up to sixteen turns more.
    if (fatal == 0) {
        for (int round = 0; round < 28 && fatal == 0; round++) {
            float lead = cands[0].ms;
            for (const Cand &k : cands) lead = k.ms < lead ? k.ms : lead;
            if (round >= 12) {
                bool grey = false;
                for (const Cand &k : cands) grey = grey || (k.ms > 1.02f * lead && k.ms < 1.04f * lead);
                if (!grey) break;
            }
            for (Cand &k : cands) {
                if (k.ms > (round < 4 ? 1.10f : (round < 12 ? 1.06f : 1.04f)) * lead) continue;
                float ms = 0.0f;
                const int rc = run_timed(k.tile, k.slices, batch_of(k.ms), &ms);
                if (rc != 0) {
                    fatal = rc;
                    break;
                }
                if (ms < k.ms) k.ms = ms;
            }
        }
    }
    g_tuning = false;
    g_pool_req = pool_req;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (fatal != 0) return -fatal;
    float fastest = cands[0].ms;
    for (const Cand &k : cands) fastest = k.ms < fastest ? k.ms : fastest;
    const Cand *pick = nullptr;
    for (const Cand &k : cands)
        if (k.ms <= 1.03f * fastest && (pick == nullptr || k.rank < pick->rank || (k.rank == pick->rank && k.slices < pick->slices))) pick = &k;
    out->tile = pick->tile;
    out->slices = pick->tile < 0 ? 1 : pick->slices;
    if (getenv("EDDLHIP_TUNE_VERBOSE"))
        fprintf(stderr, "tune %d %d %d %d -> %d %dx%d s%d: planned %.1f us, fastest %.1f us, kept %.1f us (tile %d x %d slices) of %zu plans\n", c.N, c.C,
                c.H, c.W, c.Kf, c.R, c.S, c.sr, cands[0].ms * 1e3f, fastest * 1e3f, pick->ms * 1e3f, out->tile, out->slices, cands.size());
    return 0;
}

int conv2d_fwd_impl(bool no_alloc, int dev, const float *I, const float *I2, int uh, int uw, const float *K, const float *bias, float *O, int N, int C,
                    int H, int W, int Kf, int R, int S, int sr, int sc, int pad_top, int pad_left, int P, int Q, const float *bn_g,
                    const float *bn_b, const float *bn_mean, const float *bn_var, float bn_eps, const float *residual, int relu,
                    const GemmBatch *gemm) {
    EH_REQUIRE(N >= 0 && C > 0 && H > 0 && W > 0, "conv2d: bad input shape %dx%dx%dx%d", N, C, H, W);
    EH_REQUIRE(Kf > 0 && R > 0 && S > 0, "conv2d: bad filter shape %dx%dx%dx%d", Kf, C, R, S);
    EH_REQUIRE(sr > 0 && sc > 0, "conv2d: strides must be positive");
    EH_REQUIRE(P > 0 && Q > 0, "conv2d: invalid output shape (%d x %d)", P, Q);
    EH_REQUIRE(pad_top >= 0 && pad_left >= 0, "conv2d: negative padding");
    EH_REQUIRE((bn_mean == nullptr) == (bn_var == nullptr), "conv2d: bn_mean and bn_var must come together");
    EH_REQUIRE((bn_g == nullptr) == (bn_b == nullptr), "conv2d: bn_g and bn_b must come together");
    EH_REQUIRE(bn_g == nullptr || bn_mean != nullptr, "conv2d: affine parameters without statistics");
    const bool two = I2 != nullptr;
    const int Cimg = two ? C / 2 : C;  // channels per image in each input tensor
    if (two) {
        EH_REQUIRE(C % 2 == 0, "conv2d: a two-tensor input needs an even channel count, got %d", C);
        EH_REQUIRE(g_algo == 2 || (R == S && (R == 1 || R == 2 || R == 3)),
                   "conv2d: a two-tensor input is taken by the 1x1, 2x2 and 3x3 kernels only (filter %dx%d): concatenate first", R, S);
    }
    if (uh != 1 || uw != 1) {
        EH_REQUIRE(uh >= 1 && uw >= 1 && (long long)H * uh <= (1 << 20) && (long long)W * uw <= (1 << 20), "conv2d: bad upsampling factors %d x %d", uh, uw);
        EH_REQUIRE(g_algo == 2 || (R == S && (R == 1 || R == 2 || R == 3)),
                   "conv2d: an upsampled input is taken by the 1x1, 2x2 and 3x3 kernels only (filter %dx%d): resize first", R, S);
        // the reference's mapping, source = (int)((float)dst / ((float)new / in)) (src/hardware/cpu/cpu_da.cpp:109-113), must be
        // the integer division the gather uses
        for (int axis = 0; axis < 2; axis++) {
            const int in = axis ? W : H, u = axis ? uw : uh;
            const float scale = (float)(in * u) / (float)in;
            for (int d = 0; d < in * u; d++)
                EH_REQUIRE((int)((float)d / scale) == d / u, "conv2d: upsampling %d -> %d is not a whole-pixel repetition at %d", in, in * u, d);
        }
    }
    const long long img_elems = (long long)Cimg * H * W;
    EH_REQUIRE(img_elems <= (1LL << 28), "conv2d: one image of %lld elements exceeds the 1 GiB a buffer descriptor may cover", img_elems);
    EH_REQUIRE((long long)C * R * S <= (1LL << 24), "conv2d: filter too large");
    EH_REQUIRE((long long)P * Q <= 0x7fffffffLL, "conv2d: output plane too large");
    if (N == 0) return 0;
    EH_REQUIRE(I && K && O, "conv2d: NULL tensor");
    if (no_alloc) {
        EH_REQUIRE(dev >= 0 && dev < EDDLHIP_MAX_DEVICES && state(dev).inited && g_scratch_ptr[dev] != nullptr,
                   "conv2d_fwd_noalloc: device %d is not initialised; call eddlhip_init(%d) first (initialisation allocates)", dev, dev);
        EH_REQUIRE(!g_prof_on, "conv2d_fwd_noalloc: not while eddlhip_conv2d_profile collects (its event pairs are allocated)");
    }
    EH_TRY(use_device(dev));
    EH_REQUIRE(!(g_prof_on && state(dev).capturing), "conv2d: launches cannot be timed (eddlhip_conv2d_profile) while a graph is being recorded");
    hipStream_t st = state(dev).stream;

    ConvParams p;
    p.I = I; p.I2 = two ? I2 : I; p.Csplit = two ? C / 2 : C; p.Cimg = Cimg;
    p.uh = uh; p.uw = uw;
    p.K = K; p.O = O; p.Wp = nullptr;
    p.bias = bias; p.bn_g = bn_g; p.bn_b = bn_b; p.bn_mean = bn_mean; p.bn_var = bn_var; p.residual = residual;
    p.bn_eps = bn_eps; p.relu = relu;
    {
        // bound by its output traffic (arithmetic intensity under the ridge of 157.3 TFLOP/s over 8 TB/s) and an output that
        // the 256 MB last-level cache cannot hold for the next layer anyway
        const double out_bytes = 4.0 * N * Kf * P * Q, in_bytes = 4.0 * N * C * H * W;
        const double flops = 2.0 * N * Kf * (double)C * R * S * P * Q;
        p.stream_out = (out_bytes >= 256e6 && out_bytes > 2 * in_bytes && flops / (out_bytes + in_bytes) < 19.7) ? 1 : 0;
    }
    p.N = N; p.C = C; p.H = H; p.W = W; p.Kf = Kf; p.R = R; p.S = S; p.sr = sr; p.sc = sc; p.pt = pad_top; p.pl = pad_left;
    p.P = P; p.Q = Q;
    p.CRS = C * R * S;
    p.PQ = P * Q;
    p.npix = (long long)N * P * Q;
    p.gm = p.gn = 0;
    p.nsteps = 0;
    p.Mp = (Kf + M_ALIGN - 1) / M_ALIGN * M_ALIGN;
    p.in_bytes = p.wp_bytes = 0;
    p.main_tiles = 0; p.nslices = 1; p.slice_steps = 0; p.partial = nullptr;
    p.trace = nullptr;
    p.w_img_stride = 0;

    if (g_algo == 2) {
        size_t total = (size_t)p.npix * Kf;
        snprintf(g_last_kernel, sizeof(g_last_kernel), "conv_direct_kernel");
        EH_TRY(prof_begin(st));
        hipLaunchKernelGGL(conv_direct_kernel, dim3(eh_blocks(total, 256, 1u << 20)), dim3(256), 0, st, p);
        EH_CHECK_LAUNCH();
        EH_TRY(prof_end(st));
        return 0;
    }

    // ---- a 1x1 convolution onto at most four filters: a read stream, no tile
    if (!gemm && g_algo == 0 && g_force_tile < 0 && R == 1 && S == 1 && sr == 1 && sc == 1 && pad_top == 0 && pad_left == 0 && Kf <= 4 && !two &&
        uh == 1 && uw == 1 && P == H && Q == W) {
        const bool vec4 = p.PQ % 4 == 0 && (((size_t)I | (size_t)O | (size_t)(residual ? residual : O)) & 15) == 0;
        void (*kern)(const ConvParams) = nullptr;
        switch (Kf * 2 + (vec4 ? 1 : 0)) {
            case 2: kern = conv_pointwise_few_kernel<1, 1>; break;
            case 3: kern = conv_pointwise_few_kernel<1, 4>; break;
            case 4: kern = conv_pointwise_few_kernel<2, 1>; break;
            case 5: kern = conv_pointwise_few_kernel<2, 4>; break;
            case 6: kern = conv_pointwise_few_kernel<3, 1>; break;
            case 7: kern = conv_pointwise_few_kernel<3, 4>; break;
            case 8: kern = conv_pointwise_few_kernel<4, 1>; break;
            default: kern = conv_pointwise_few_kernel<4, 4>; break;
        }
        const size_t groups = (size_t)N * (p.PQ / (vec4 ? 4 : 1));
        snprintf(g_last_kernel, sizeof(g_last_kernel), "conv_pointwise_few_kernel<%d,%d>", Kf, vec4 ? 4 : 1);
        EH_TRY(prof_begin(st));
        hipLaunchKernelGGL(kern, dim3(eh_blocks(groups, 256, 256 * 16)), dim3(256), 0, st, p);
        EH_CHECK_LAUNCH();
        EH_TRY(prof_end(st));
        return 0;
    }

    // ---- kernel variant and launch plan
    const int direct = (g_algo == 3) ? 0 : 1;  // default: the load unit writes LDS directly
    const Variant *family;
    if (R == 3 && S == 3) family = k3x3[direct];
    else if (R == 1 && S == 1) family = k1x1[direct];
    else if (R == 2 && S == 2) family = k2x2[direct];
    else family = kgen[direct];
    EH_TRY(family_occupancy(family));
    // a launch covers one batch chunk: input within the 2 GiB a buffer descriptor addresses with 32-bit
    // offsets, and fewer than 2^31 output pixels (32-bit pixel arithmetic in the kernels)
    long long max_imgs = (1LL << 29) / img_elems;
    if (max_imgs > 0x7ffffe00LL / p.PQ) max_imgs = 0x7ffffe00LL / p.PQ;
    EH_REQUIRE(max_imgs >= 1, "conv2d: one output plane of %d pixels is too large", p.PQ);
    const int chunk_imgs = (int)((N < max_imgs) ? N : max_imgs);
    Plan plan = plan_conv(family, Kf, C, R * S, (long long)chunk_imgs * p.PQ, state(dev).num_cu, g_split != 0);
    if (g_force_tile >= 0 && g_force_tile < 4)
        plan = forced_plan(family, g_force_tile, g_force_slices, Kf, C, R * S, (long long)chunk_imgs * p.PQ, state(dev).num_cu);
    // the Winograd form: asked for (force_plan(4, .), set_algo(7)) or found faster by the plan search (below); never from the
    // fixed scratch array, whose size it exceeds, and not for the scalar-order or register-staged algorithm switches
    const bool wino_ok = !gemm && !no_alloc && g_algo == 0 && !g_wino_never && winograd_applies(N, C, Kf, R, S, sr, sc, P, Q);
    const bool fold_ok = wino_ok && winograd_fold_applies(N, C, Kf, R, S, sr, sc, P, Q);
    // the one-launch form (3x3 filters only) needs no transformed copy of the input, so none of V's limits apply
    const bool fused_ok = !gemm && !no_alloc && g_algo == 0 && !g_wino_never && R == 3 && S == 3 && sr == 1 && sc == 1 &&
                          (long long)C * 16 * p.Mp * 4 < (1LL << 31);
    // the upsampled-input form of a 2x2 filter: a geometry of its own in the plans table (kind 2 / 3), since the same
    // shapes on a stored tensor cannot take it
    const bool up_ok = !gemm && !no_alloc && g_algo == 0 && up2x2_applies(N, C, H, W, Kf, R, S, sr, sc, uh, uw, two, pad_top, pad_left, P, Q);
    if (up_ok && (g_force_tile == UP2X2_TILE || g_force_tile == UP2X2_TILE + 1))
        return conv2d_up2x2(g_force_tile - UP2X2_TILE, dev, I, K, bias, O, N, C, H, W, Kf, P, Q, bn_g, bn_b, bn_mean, bn_var, bn_eps, residual, relu);
    if (fused_ok && g_force_tile >= FUSED_TILE0 && g_force_tile < FUSED_TILE0 + NUM_FUSED)
        return conv2d_winograd_fused(g_force_tile - FUSED_TILE0, g_force_slices, dev, I, two ? I2 : nullptr, uh, uw, K, bias, O, N, C, H, W, Kf, pad_top,
                                     pad_left, P, Q, bn_g, bn_b, bn_mean, bn_var, bn_eps, residual, relu);
    if ((wino_ok && (g_force_tile == 4 || (g_wino && g_force_tile < 0 && !g_tuning))) || (fold_ok && g_force_tile == 5))
        return conv2d_winograd(g_force_tile == 5, R, dev, I, two ? I2 : nullptr, uh, uw, K, bias, O, N, C, H, W, Kf, pad_top, pad_left, P, Q, bn_g, bn_b,
                               bn_mean, bn_var, bn_eps, residual, relu);
    const bool query = gemm != nullptr && gemm->need_out != nullptr;  // report the workspace need, launch nothing
    bool plan_open = false;                                         // a search could still pick any plan for this geometry
    if (g_autotune && g_force_tile < 0 && g_algo == 0 && g_split != 0) {
        const int key[10] = {N, C, Kf, R, S, sr, sc, P, Q, direct + (up_ok ? 2 : 0)};
        const TunedPlan *found = nullptr;
        for (const TunedPlan &t : g_tuned[dev])
            if (memcmp(t.key, key, sizeof(key)) == 0) found = &t;
        // (no search inside a search: a convolution being timed runs its product launch, a geometry of its own, under the
        // plan already kept for it)
        const bool can_search = found == nullptr && !g_tuning && !no_alloc && !state(dev).capturing && !g_prof_on;
        plan_open = can_search;
        if (can_search && !query) {
            const ConvCall call = {dev, I, I2, uh, uw, K, bias, O, N, C, H, W, Kf, R, S, sr, sc, pad_top, pad_left, P, Q,
                                   bn_g, bn_b, bn_mean, bn_var, bn_eps, residual, relu};
            TunedPlan best;
            memcpy(best.key, key, sizeof(key));
            const size_t ws_before = state(dev).workspace_bytes;
            const int src = search_plan(call, family, plan, (long long)chunk_imgs * p.PQ, wino_ok, fold_ok, fused_ok, up_ok, &best);
            if (src < 0) return -src;  // a runtime error inside the search
            // the candidates may have taken far more workspace than the plan that stays: let it grow back to what is needed
            // (not inside another convolution's call, whose buffers live there)
            if (!gemm && state(dev).workspace_bytes > ws_before) EH_TRY(release_workspace(dev));
            if (src == 0) {
                g_tuned[dev].push_back(best);
                found = &g_tuned[dev].back();
            }  // (src > 0: no search on these tensors - the planner's plan, nothing recorded)
        }
        if (found != nullptr && ((found->tile == 4 && wino_ok) || (found->tile == 5 && fold_ok)))
            return conv2d_winograd(found->tile == 5, R, dev, I, two ? I2 : nullptr, uh, uw, K, bias, O, N, C, H, W, Kf, pad_top, pad_left, P, Q, bn_g,
                                   bn_b, bn_mean, bn_var, bn_eps, residual, relu);
        if (found != nullptr && (found->tile == UP2X2_TILE || found->tile == UP2X2_TILE + 1) && up_ok)
            return conv2d_up2x2(found->tile - UP2X2_TILE, dev, I, K, bias, O, N, C, H, W, Kf, P, Q, bn_g, bn_b, bn_mean, bn_var, bn_eps, residual, relu);
        if (found != nullptr && found->tile >= FUSED_TILE0 && found->tile < FUSED_TILE0 + NUM_FUSED && fused_ok)
            return conv2d_winograd_fused(found->tile - FUSED_TILE0, found->slices, dev, I, two ? I2 : nullptr, uh, uw, K, bias, O, N, C, H, W, Kf, pad_top, pad_left, P, Q, bn_g,
                                         bn_b, bn_mean, bn_var, bn_eps, residual, relu);
        if (found != nullptr && found->tile >= 0 && found->tile < 4)
            plan = forced_plan(family, found->tile, found->slices, Kf, C, R * S, (long long)chunk_imgs * p.PQ, state(dev).num_cu);
    }
    if (query && plan_open) {
        // the largest partial-tile need of any plan the search tries
        size_t worst = 0;
        for (int tile = 0; tile < 4; tile++)
            for (int sl : kSearchSlices) {
                const Plan fp = forced_plan(family, tile, sl, Kf, C, R * S, (long long)chunk_imgs * p.PQ, state(dev).num_cu);
                const size_t need = fp.nslices > 1 ? (size_t)fp.nslices * fp.leftover * family[tile].bm * family[tile].bn * sizeof(float) : 0;
                if (need > worst) worst = need;
            }
        *gemm->need_out = worst;
        return 0;
    }
    const Variant *v = &family[plan.tile];
    const int bk = v->cpb ? v->cpb * R * S : 16;
    p.nsteps = plan.nsteps;
    const int gm = (Kf + v->bm - 1) / v->bm;
    EH_REQUIRE(plan.tiles <= 0x3fffffffLL, "conv2d: too many tiles");
    const long long leftover = plan.nslices > 1 ? plan.leftover : 0;
    const int nslices = plan.nslices, slice_steps = plan.slice_steps;
    const size_t tile_floats = (size_t)v->bm * v->bn;

    // ---- packed filters (the registered copy, or a repack into the workspace), then the partial
    // tiles of the K-split launch
    const int rows = p.nsteps * bk;
    // the kernels address the packed filters through a buffer descriptor with 32-bit byte offsets
    EH_REQUIRE((size_t)rows * p.Mp * sizeof(float) < ((size_t)1 << 31),
               "conv2d: the repacked filter matrix (%d taps x %d channels) exceeds the 2 GiB a buffer descriptor covers", rows, p.Mp);
    const float *cached = gemm ? gemm->Wp : nullptr;
    if (!gemm) {
        std::lock_guard<std::mutex> lock(g_cache_mutex);
        for (CachedFilters &e : g_cache[dev]) {
            if (e.K == K && e.Kf == Kf && e.C == C && e.R == R && e.S == S && rows <= e.rows) {
                if (e.stale) EH_TRY(repack(dev, e));
                cached = e.Wp;
                break;
            }
        }
    }
    const size_t wp_bytes = cached ? 0 : (((size_t)rows * p.Mp * sizeof(float) + 255) & ~(size_t)255);
    const size_t taps_bytes = v->cpb ? 0 : (((size_t)rows * sizeof(int32x4) + 255) & ~(size_t)255);
    const size_t partial_bytes = (size_t)nslices * leftover * tile_floats * sizeof(float);
    if (query) {
        *gemm->need_out = wp_bytes + taps_bytes + partial_bytes;
        return 0;
    }
    if (gemm)  // (checked before the workspace is touched: growing it would free the caller's buffers)
        EH_REQUIRE(wp_bytes + taps_bytes + partial_bytes <= gemm->reserve, "conv2d: internal error, workspace of a product launch");
    void *ws = nullptr;
    if (no_alloc) {
        const size_t need = wp_bytes + taps_bytes + partial_bytes;
        EH_REQUIRE(need <= (size_t)EDDLHIP_CONV_NOALLOC_SCRATCH_BYTES,
                   "conv2d_fwd_noalloc: this call needs %zu bytes of scratch memory (%zu repacked filters + %zu tap table + %zu partial "
                   "tiles); the fixed array holds %zu.  Register the filters (eddlhip_conv2d_cache_filters) or call eddlhip_conv2d_fwd",
                   need, wp_bytes, taps_bytes, partial_bytes, (size_t)EDDLHIP_CONV_NOALLOC_SCRATCH_BYTES);
        ws = g_scratch_ptr[dev];
    } else {
        EH_TRY(get_workspace(dev, wp_bytes + taps_bytes + partial_bytes, &ws));
    }
    p.Wp = cached ? cached : (const float *)ws;
    p.wp_bytes = (unsigned)((size_t)rows * p.Mp * sizeof(float));
    if (gemm) {
        EH_REQUIRE(v->cpb != 0 && gemm->stride == (size_t)rows * p.Mp && p.PQ % v->bn == 0,
                   "conv2d: internal error, the product launch of a Winograd convolution does not fit its operands");
        p.w_img_stride = gemm->stride;
    }
    p.taps = (const int32x4 *)((char *)ws + wp_bytes);
    p.partial = (float *)((char *)ws + wp_bytes + taps_bytes);
    if (taps_bytes) {
        hipLaunchKernelGGL(tap_table_kernel, dim3((rows + 255) / 256), dim3(256), 0, st, (int32x4 *)((char *)ws + wp_bytes), rows, C, R, S, W, H * W);
        EH_CHECK_LAUNCH();
    }
    if (!cached) {
        hipLaunchKernelGGL(pack_filters_kernel, dim3((rows + 31) / 32, p.Mp / 32), dim3(256), 0, st, K, (float *)ws, Kf, p.CRS, p.Mp, rows);
        EH_CHECK_LAUNCH();
    }

    for (long long b0 = 0; b0 < N; b0 += chunk_imgs) {
        const int nb = (int)((N - b0 < chunk_imgs) ? N - b0 : chunk_imgs);
        ConvParams q = p;
        q.N = nb;
        q.I = I + (size_t)b0 * img_elems;
        q.I2 = p.I2 + (size_t)b0 * img_elems;
        q.O = O + (size_t)b0 * Kf * p.PQ;
        q.Wp = p.Wp + (size_t)b0 * p.w_img_stride;
        if (residual) q.residual = residual + (size_t)b0 * Kf * p.PQ;
        q.npix = (long long)nb * p.PQ;
        q.in_bytes = (unsigned)((size_t)nb * img_elems * sizeof(float));
        q.gm = gm;
        const long long gn = (q.npix + v->bn - 1) / v->bn;
        q.gn = (int)gn;
        const long long tiles = gn * gm;
        const long long split_tiles = (nb == chunk_imgs) ? leftover : 0;  // a short last chunk runs unsplit
        const long long main_tiles = tiles - split_tiles;
        q.main_tiles = (int)main_tiles;
        q.nslices = split_tiles > 0 ? nslices : 1;
        q.slice_steps = split_tiles > 0 ? slice_steps : p.nsteps;
        q.trace = (g_trace != nullptr && main_tiles + split_tiles * q.nslices <= g_trace_wgs) ? g_trace : nullptr;
        EH_TRY(prof_begin(st));
        hipLaunchKernelGGL(v->kernel, dim3((unsigned)(main_tiles + split_tiles * q.nslices)), dim3(256), 0, st, q);
        EH_CHECK_LAUNCH();
        EH_TRY(prof_end(st));
        if (split_tiles > 0) {
            hipLaunchKernelGGL(v->reduce, dim3((unsigned)(split_tiles * (v->bm / 32) * (v->bn / 32))), dim3(256), 0, st, q);
            EH_CHECK_LAUNCH();
        }
    }
    if (leftover > 0) snprintf(g_last_kernel, sizeof(g_last_kernel), "%s +ksplit(%lld tiles x %d)", v->name, leftover, nslices);
    else snprintf(g_last_kernel, sizeof(g_last_kernel), "%s", v->name);
    return 0;
}

// The Winograd form of a 3x3 stride-1 convolution (kernels and algebra above): filter transform (kept with a registered
// filter tensor), input transform, ONE product launch through conv2d_fwd_impl (16 images of C channels and Tp pixels, a
// planned or searched 1x1 launch like any other), output transform with the convolution's epilogue.
// Workspace: [what the product launch may take][transformed filters unless kept][V][M].
int conv2d_winograd(bool fold, int fs, int dev, const float *I, const float *I2, int uh, int uw, const float *K, const float *bias, float *O, int N, int C,
                    int H, int W, int Kf, int pad_top, int pad_left, int P, int Q, const float *bn_g, const float *bn_b, const float *bn_mean,
                    const float *bn_var, float bn_eps, const float *residual, int relu) {
    hipStream_t st = state(dev).stream;
    // a max-pool asked for with this convolution is taken into the epilogue where every 2x2 block of outputs is whole
    PoolRequest *const pool = (g_pool_req != nullptr && !g_tuning && P % 2 == 0 && Q % 2 == 0) ? g_pool_req : nullptr;
    if (pool != nullptr) pool->done = true;
    const int ps = fs + 1, np = ps * ps;  // patch side and positions: 4 and 16 for 3x3 filters, 3 and 9 for 2x2
    const int th = (P + 1) / 2, tw = (Q + 1) / 2;
    const int T = N * th * tw, Tp = (T + 127) / 128 * 128;
    const int rows = (C + 15) / 16 * 16, Mp = (Kf + M_ALIGN - 1) / M_ALIGN * M_ALIGN;
    const size_t u_floats = (size_t)np * rows * Mp, v_floats = (size_t)np * C * Tp, m_floats = (size_t)np * Kf * Tp;
    EH_REQUIRE((size_t)rows * Mp * sizeof(float) < ((size_t)1 << 31), "conv2d: the transformed filter matrix (%d x %d) exceeds 2 GiB", rows, Mp);

    // ---- transformed filters: the registered copy (made here on first use, refreshed when the filters were written), or a
    // transform into the workspace
    const float *U = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_cache_mutex);
        for (CachedFilters &e : g_cache[dev]) {
            if (e.K == K && e.Kf == Kf && e.C == C && e.R == fs && e.S == fs) {
                if (e.Wwino == nullptr && !state(dev).capturing) {
                    if (hipMalloc((void **)&e.Wwino, u_floats * sizeof(float)) != hipSuccess) {
                        e.Wwino = nullptr;
                        (void)hipGetLastError();
                        break;  // no room to keep them: transform per call
                    }
                    e.wino_rows = rows;
                    e.stale = true;
                }
                if (e.Wwino != nullptr) {
                    if (e.stale) EH_TRY(repack(dev, e));
                    U = e.Wwino;
                }
                break;
            }
        }
    }
    const size_t u_bytes = U ? 0 : ((u_floats * sizeof(float) + 255) & ~(size_t)255);
    const size_t v_bytes = (v_floats * sizeof(float) + 255) & ~(size_t)255;
    const size_t m_bytes = fold ? 0 : ((m_floats * sizeof(float) + 255) & ~(size_t)255);  // folded: M is never written
    // what the product launch of the three-kernel form will take for its partial tiles lies in front of U, V and M
    size_t inner = 0;
    if (!fold) {
        const GemmBatch gq = {K, (size_t)rows * Mp, 0, &inner};
        const int ft = g_force_tile, fsl = g_force_slices;
        g_force_tile = -1;
        g_force_slices = -1;
        const int qrc = conv2d_fwd_impl(false, dev, K, nullptr, 1, 1, K, nullptr, O, np, C, 1, Tp, Kf, 1, 1, 1, 1, 0, 0, 1, Tp, nullptr, nullptr, nullptr, nullptr,
                                        0.0f, nullptr, 0, &gq);
        g_force_tile = ft;
        g_force_slices = fsl;
        if (qrc != 0) return qrc;
        inner = (inner + 255) & ~(size_t)255;
    }
    void *ws = nullptr;
    EH_TRY(get_workspace(dev, inner + u_bytes + v_bytes + m_bytes, &ws));
    char *base = (char *)ws + inner;
    float *Uw = (float *)base, *V = (float *)(base + u_bytes), *M = (float *)(base + u_bytes + v_bytes);
    if (U == nullptr) {
        const dim3 grid((unsigned)(((size_t)rows * Mp + 255) / 256));
        if (ps == 4) hipLaunchKernelGGL(wino_filter_kernel<4>, grid, dim3(256), 0, st, K, Uw, Kf, C, Mp, rows, 0);
        else hipLaunchKernelGGL(wino_filter_kernel<3>, grid, dim3(256), 0, st, K, Uw, Kf, C, Mp, rows, 0);
        EH_CHECK_LAUNCH();
        U = Uw;
    }

    // ---- input transform
    WinoParams w;
    w.I = I; w.I2 = I2 ? I2 : I; w.Csplit = I2 ? C / 2 : C; w.Cimg = I2 ? C / 2 : C;
    w.uh = uh; w.uw = uw;
    w.C = C; w.H = H; w.W = W; w.pt = pad_top; w.pl = pad_left;
    w.th = th; w.tw = tw; w.T = T; w.Tp = Tp;
    w.V = V;
    {
        // LDS slots of the staged kernel, an upper bound over its workgroups: 256 blocks lie in at most `segs` images and
        // 256 / tw whole rows of blocks, plus a partial row at either end of every image's run; a run of r rows of blocks
        // touches 2 r + 2 pixel rows of 2 tw + 2 slots
        const long long per_img = (long long)th * tw;
        const long long segs = std::min<long long>(N, 256 / per_img + 2);
        const long long block_rows = 256 / tw + 2 * segs;
        const long long slots = ((2 * block_rows + (ps - 2) * segs) * (2 * tw + ps - 2) + 1) & ~1LL;
        const long long img_elems = (long long)w.Cimg * H * W;
        constexpr int chans = 8;
        if (slots <= 256 * 30 && segs * img_elems < 0x7fffffffLL) {  // (offsets and values of 7680 slots: 60 KB of LDS)
            const dim3 grid((unsigned)((T + 255) / 256), (unsigned)((C + chans - 1) / chans));
            const size_t lds = (size_t)slots * 8;
            const int kmax = slots <= 256 * 8 ? 8 : (slots <= 256 * 16 ? 16 : 30);
            if (ps == 4 && kmax == 8) hipLaunchKernelGGL((wino_input_lds_kernel<8, 4>), grid, dim3(256), lds, st, w, (int)slots, chans);
            else if (ps == 4 && kmax == 16) hipLaunchKernelGGL((wino_input_lds_kernel<16, 4>), grid, dim3(256), lds, st, w, (int)slots, chans);
            else if (ps == 4) hipLaunchKernelGGL((wino_input_lds_kernel<30, 4>), grid, dim3(256), lds, st, w, (int)slots, chans);
            else if (kmax == 8) hipLaunchKernelGGL((wino_input_lds_kernel<8, 3>), grid, dim3(256), lds, st, w, (int)slots, chans);
            else if (kmax == 16) hipLaunchKernelGGL((wino_input_lds_kernel<16, 3>), grid, dim3(256), lds, st, w, (int)slots, chans);
            else hipLaunchKernelGGL((wino_input_lds_kernel<30, 3>), grid, dim3(256), lds, st, w, (int)slots, chans);
        } else {
            const dim3 grid((unsigned)((T + 255) / 256), (unsigned)((C + WINO_CH - 1) / WINO_CH));
            if (ps == 4) hipLaunchKernelGGL(wino_input_kernel<4>, grid, dim3(256), 0, st, w);
            else hipLaunchKernelGGL(wino_input_kernel<3>, grid, dim3(256), 0, st, w);
        }
    }
    EH_CHECK_LAUNCH();

    if (fold) {
        // ---- the 16 products and the output transform in one launch: a 1x1 "convolution" of ONE image of 16 C channels
        // and Tp pixels whose K range is 16 runs of C / 16 steps; conv_tap_kernel<..., WINO> folds each run's product
        // into the four outputs of a block and finishes with the convolution's epilogue (64x64 tiles, whole tiles only)
        ConvParams q;
        memset(&q, 0, sizeof(q));
        q.I = V; q.I2 = V; q.Csplit = np * C; q.Cimg = np * C; q.uh = 1; q.uw = 1;
        q.Wp = U; q.w_img_stride = 0; q.K = K; q.O = O;
        q.bias = bias; q.bn_g = bn_g; q.bn_b = bn_b; q.bn_mean = bn_mean; q.bn_var = bn_var; q.residual = residual;
        q.bn_eps = bn_eps; q.relu = relu;
        q.N = 1; q.C = np * C; q.H = 1; q.W = Tp; q.Kf = Kf; q.R = 1; q.S = 1; q.sr = 1; q.sc = 1; q.P = 1; q.Q = Tp;
        q.CRS = np * C; q.Mp = Mp; q.nsteps = np * C / 16; q.PQ = Tp; q.npix = Tp;
        q.gm = (Kf + 63) / 64; q.gn = Tp / 64;
        q.in_bytes = (unsigned)((size_t)np * C * Tp * sizeof(float));
        q.wp_bytes = (unsigned)((size_t)np * rows * Mp * sizeof(float));
        q.main_tiles = q.gm * q.gn; q.nslices = 1; q.slice_steps = q.nsteps;
        q.wspx = C / 16; q.wth = th; q.wtw = tw; q.wT = T; q.wP = P; q.wQ = Q; q.wps = ps;
        if (pool != nullptr) {
            q.pool_O = pool->O; q.pool_ix = pool->ix; q.pool_iy = pool->iy;
            if (!pool->keep) q.O = nullptr;
        }
        EH_REQUIRE(rows == C && (long long)q.gm * q.gn <= 0x3fffffffLL, "conv2d: internal error, folded Winograd launch");
        q.trace = (g_trace != nullptr && q.main_tiles <= g_trace_wgs) ? g_trace : nullptr;
        // K-steps of 32 channels where the runs divide into them: a workgroup's K loop is long here (16 C channels), few
        // workgroups share a CU (64 output registers per lane), and a step's matrix work then covers a trip to memory
        const bool wide = C % 32 == 0;
        if (wide) {
            q.nsteps = np * C / 32;
            q.slice_steps = q.nsteps;
            q.wspx = C / 32;
        }
        EH_TRY(prof_begin(st));
        if (wide) hipLaunchKernelGGL((conv_tap_kernel<2, 2, 1, 1, 1, 1, 32, true, true>), dim3((unsigned)q.main_tiles), dim3(256), 0, st, q);
        else hipLaunchKernelGGL((conv_tap_kernel<2, 2, 1, 1, 1, 1, 16, true, true>), dim3((unsigned)q.main_tiles), dim3(256), 0, st, q);
        EH_CHECK_LAUNCH();
        EH_TRY(prof_end(st));
        snprintf(g_last_kernel, sizeof(g_last_kernel), "winograd[conv_tap_kernel<2,2,1,1,1,1,%d,true,true>, %d blocks]", wide ? 32 : 16, Tp);
        return 0;
    }

    // ---- the 16 products: M[xi] = U[xi] x V[xi]
    {
        const GemmBatch gb = {U, (size_t)rows * Mp, inner, nullptr};
        const int ft = g_force_tile, fs = g_force_slices;
        g_force_tile = -1;
        g_force_slices = -1;
        const int rc = conv2d_fwd_impl(false, dev, V, nullptr, 1, 1, K, nullptr, M, np, C, 1, Tp, Kf, 1, 1, 1, 1, 0, 0, 1, Tp, nullptr, nullptr, nullptr,
                                       nullptr, 0.0f, nullptr, 0, &gb);
        g_force_tile = ft;
        g_force_slices = fs;
        if (rc != 0) return rc;
    }

    // ---- output transform + epilogue
    ConvParams p;
    memset(&p, 0, sizeof(p));
    p.O = O;
    p.bias = bias; p.bn_g = bn_g; p.bn_b = bn_b; p.bn_mean = bn_mean; p.bn_var = bn_var; p.residual = residual;
    p.bn_eps = bn_eps; p.relu = relu;
    p.N = N; p.Kf = Kf; p.P = P; p.Q = Q; p.PQ = P * Q;
    if (pool != nullptr) {
        p.pool_O = pool->O; p.pool_ix = pool->ix; p.pool_iy = pool->iy;
        if (!pool->keep) p.O = nullptr;
    }
    {
        const dim3 grid((unsigned)((T + 255) / 256), (unsigned)((Kf + WINO_CH - 1) / WINO_CH));
        if (ps == 4) hipLaunchKernelGGL(wino_output_kernel<4>, grid, dim3(256), 0, st, p, (const float *)M, th, tw, T, Tp);
        else hipLaunchKernelGGL(wino_output_kernel<3>, grid, dim3(256), 0, st, p, (const float *)M, th, tw, T, Tp);
    }
    EH_CHECK_LAUNCH();
    char product[sizeof(g_last_kernel)];
    snprintf(product, sizeof(product), "%s", g_last_kernel);
    snprintf(g_last_kernel, sizeof(g_last_kernel), "winograd[%.100s, %d blocks]", product, Tp);
    return 0;
}

// A 2x2 convolution of an input upsampled twice, as four convolutions of the stored image (conv_up2x2_kernel; see
// up2x2_filter_kernel).  Workspace: the nine filter rows per channel, unless a registered filter tensor keeps them.
int conv2d_up2x2(int variant, int dev, const float *I, const float *K, const float *bias, float *O, int N, int C, int H, int W, int Kf, int P, int Q, const float *bn_g,
                 const float *bn_b, const float *bn_mean, const float *bn_var, float bn_eps, const float *residual, int relu) {
    hipStream_t st = state(dev).stream;
    PoolRequest *const pool = (g_pool_req != nullptr && !g_tuning && P % 2 == 0 && Q % 2 == 0) ? g_pool_req : nullptr;
    if (pool != nullptr) pool->done = true;
    const int th = (P + 1) / 2, tw = (Q + 1) / 2;
    const int T = N * th * tw, Tp = (T + 127) / 128 * 128;
    const int Mp = (Kf + M_ALIGN - 1) / M_ALIGN * M_ALIGN;
    const size_t u_floats = (size_t)9 * C * Mp;
    const float *U = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_cache_mutex);
        for (CachedFilters &e : g_cache[dev]) {
            if (e.K == K && e.Kf == Kf && e.C == C && e.R == 2 && e.S == 2) {
                if (e.Wup == nullptr && !state(dev).capturing) {
                    if (hipMalloc((void **)&e.Wup, u_floats * sizeof(float)) != hipSuccess) {
                        e.Wup = nullptr;
                        (void)hipGetLastError();
                        break;  // no room to keep them: made per call
                    }
                    e.stale = true;
                }
                if (e.Wup != nullptr) {
                    if (e.stale) EH_TRY(repack(dev, e));
                    U = e.Wup;
                }
                break;
            }
        }
    }
    if (U == nullptr) {
        void *ws = nullptr;
        EH_TRY(get_workspace(dev, u_floats * sizeof(float), &ws));
        hipLaunchKernelGGL(up2x2_filter_kernel, dim3((unsigned)(((size_t)C * Mp + 255) / 256)), dim3(256), 0, st, K, (float *)ws, Kf, C, Mp);
        EH_CHECK_LAUNCH();
        U = (const float *)ws;
    }
    ConvParams q;
    memset(&q, 0, sizeof(q));
    q.I = I; q.I2 = I; q.Csplit = C; q.Cimg = C; q.uh = 1; q.uw = 1;
    q.Wp = U; q.w_img_stride = 0; q.K = K; q.O = O;
    q.bias = bias; q.bn_g = bn_g; q.bn_b = bn_b; q.bn_mean = bn_mean; q.bn_var = bn_var; q.residual = residual;
    q.bn_eps = bn_eps; q.relu = relu;
    q.N = N; q.C = C; q.H = H; q.W = W; q.Kf = Kf; q.R = 2; q.S = 2; q.sr = 1; q.sc = 1; q.P = 1; q.Q = Tp;
    q.CRS = 4 * C; q.Mp = Mp; q.PQ = Tp; q.npix = Tp;
    q.gm = (Kf + 63) / 64; q.gn = Tp / 128;
    q.in_bytes = (unsigned)((size_t)N * C * H * W * sizeof(float));
    q.wp_bytes = (unsigned)(u_floats * sizeof(float));
    q.main_tiles = q.gm * q.gn; q.nslices = 1;
    q.wth = th; q.wtw = tw; q.wT = T; q.wP = P; q.wQ = Q; q.wps = 3;
    if (pool != nullptr) {
        q.pool_O = pool->O; q.pool_ix = pool->ix; q.pool_iy = pool->iy;
        if (!pool->keep) q.O = nullptr;
    }
    EH_REQUIRE((long long)q.gm * q.gn <= 0x3fffffffLL, "conv2d: internal error, launch of the upsampled 2x2 form");
    q.nsteps = C / 4;
    q.slice_steps = q.nsteps;
    EH_TRY(prof_begin(st));
    if (variant == 0) hipLaunchKernelGGL(conv_up2x2_kernel<3>, dim3((unsigned)q.main_tiles), dim3(256), 0, st, q);
    else hipLaunchKernelGGL(conv_up2x2_kernel<2>, dim3((unsigned)q.main_tiles), dim3(256), 0, st, q);
    EH_CHECK_LAUNCH();
    EH_TRY(prof_end(st));
    snprintf(g_last_kernel, sizeof(g_last_kernel), "upsampled2x2[conv_up2x2_kernel<%d>, %d blocks]", variant == 0 ? 3 : 2, Tp);
    return 0;
}

// The one-launch Winograd form of a 3x3 stride-1 convolution (wino_fused_kernel).  Workspace: the transformed filters,
// unless a registered filter tensor keeps them, and the partial output tiles of a K-split plan.
int conv2d_winograd_fused(int variant, int slices, int dev, const float *I, const float *I2, int uh, int uw, const float *K, const float *bias, float *O,
                          int N, int C, int H, int W, int Kf, int pad_top, int pad_left, int P, int Q, const float *bn_g, const float *bn_b,
                          const float *bn_mean, const float *bn_var, float bn_eps, const float *residual, int relu) {
    hipStream_t st = state(dev).stream;
    const FusedVariant &fv = kfused[variant];
    // a max-pool asked for with this convolution is taken into the epilogue where every 2x2 block of outputs is whole
    PoolRequest *const pool = (g_pool_req != nullptr && !g_tuning && P % 2 == 0 && Q % 2 == 0) ? g_pool_req : nullptr;
    if (pool != nullptr) pool->done = true;
    const int th = (P + 1) / 2, tw = (Q + 1) / 2;
    const int rows = (C + FUSED_ROW_ALIGN - 1) / FUSED_ROW_ALIGN * FUSED_ROW_ALIGN, Mp = (Kf + M_ALIGN - 1) / M_ALIGN * M_ALIGN;
    const size_t u_floats = (size_t)16 * rows * Mp;
    EH_REQUIRE(u_floats * sizeof(float) < ((size_t)1 << 31), "conv2d: the transformed filters (16 x %d x %d) exceed 2 GiB", rows, Mp);

    // a launch covers one batch chunk: input within the 2 GiB a buffer descriptor addresses, fewer than 2^30 blocks
    const int Cimg = I2 ? C / 2 : C;
    const long long img_elems = (long long)Cimg * H * W, per_img = (long long)th * tw;
    long long max_imgs = (1LL << 29) / img_elems;
    if (max_imgs > 0x3ffffe00LL / per_img) max_imgs = 0x3ffffe00LL / per_img;
    EH_REQUIRE(max_imgs >= 1, "conv2d: one image of %lld elements is too large for the Winograd form", img_elems);
    const int chunk_imgs = (int)((N < max_imgs) ? N : max_imgs);
    long long leftover = 0;
    int slice_steps = 0;
    const int nslices = fused_slices(fv, slices, chunk_imgs * per_img, C, Kf, state(dev).num_cu, &leftover, &slice_steps);
    const size_t tile_floats = (size_t)32 * fv.fm * 32 * fv.fn * 4;  // four outputs per filter and block
    // The pixels come in 16 bytes per lane where a group of four columns that starts at a multiple of four lies inside the
    // image or outside it as a whole and is aligned in memory (image rows of a multiple of four pixels, stored as they are
    // read, 16-byte aligned tensors), and where rows of blocks are long enough that the widened pixel rows of a tile's
    // segments fit its 16 slots per block (at most 2 + 30 / tw segments, each pixel row at most 6 slots longer than it needs to be).
    const bool wide = uh == 1 && uw == 1 && W % 4 == 0 && tw >= 6 && pad_left <= 4 && (uintptr_t)I % 16 == 0 && (I2 == nullptr || (uintptr_t)I2 % 16 == 0);
    const size_t partial_bytes = (size_t)nslices * leftover * tile_floats * sizeof(float);

    const float *U = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_cache_mutex);
        for (CachedFilters &e : g_cache[dev]) {
            if (e.K == K && e.Kf == Kf && e.C == C && e.R == 3 && e.S == 3) {
                if (e.Wfused == nullptr && !state(dev).capturing) {
                    if (hipMalloc((void **)&e.Wfused, u_floats * sizeof(float)) != hipSuccess) {
                        e.Wfused = nullptr;
                        (void)hipGetLastError();
                        break;  // no room to keep them: transform per call
                    }
                    e.fused_rows = rows;
                    e.stale = true;
                }
                if (e.Wfused != nullptr) {
                    if (e.stale) EH_TRY(repack(dev, e));
                    U = e.Wfused;
                }
                break;
            }
        }
    }
    const size_t u_bytes = U ? 0 : ((u_floats * sizeof(float) + 255) & ~(size_t)255);
    void *ws = nullptr;
    if (u_bytes + partial_bytes > 0) EH_TRY(get_workspace(dev, u_bytes + partial_bytes, &ws));
    if (U == nullptr) {
        const dim3 grid((unsigned)(((size_t)rows * Mp + 255) / 256));
        hipLaunchKernelGGL(wino_filter_kernel<4>, grid, dim3(256), 0, st, K, (float *)ws, Kf, C, Mp, rows, 1);
        EH_CHECK_LAUNCH();
        U = (const float *)ws;
    }

    ConvParams q;
    memset(&q, 0, sizeof(q));
    q.Csplit = I2 ? C / 2 : C; q.Cimg = Cimg; q.uh = uh; q.uw = uw;
    q.Wp = U; q.K = K;
    q.bias = bias; q.bn_g = bn_g; q.bn_b = bn_b; q.bn_mean = bn_mean; q.bn_var = bn_var;
    q.bn_eps = bn_eps; q.relu = relu;
    q.C = C; q.H = H; q.W = W; q.Kf = Kf; q.R = 3; q.S = 3; q.sr = 1; q.sc = 1; q.pt = pad_top; q.pl = pad_left; q.P = P; q.Q = Q;
    q.CRS = C * 9; q.Mp = Mp; q.PQ = P * Q;
    q.nsteps = (C + fv.ck - 1) / fv.ck;
    q.wp_bytes = (unsigned)(u_floats * sizeof(float));
    q.wth = th; q.wtw = tw; q.wP = P; q.wQ = Q; q.wps = 4;
    q.gm = (Kf + 32 * fv.fm - 1) / (32 * fv.fm);
    q.partial = (float *)((char *)ws + u_bytes);
    for (long long b0 = 0; b0 < N; b0 += chunk_imgs) {
        const int nb = (int)((N - b0 < chunk_imgs) ? N - b0 : chunk_imgs);
        q.N = nb;
        q.I = I + (size_t)b0 * img_elems;
        q.I2 = (I2 ? I2 : I) + (size_t)b0 * img_elems;
        q.O = O + (size_t)b0 * Kf * q.PQ;
        q.residual = residual ? residual + (size_t)b0 * Kf * q.PQ : nullptr;
        q.in_bytes = (unsigned)((size_t)nb * img_elems * sizeof(float));
        q.wT = (int)(nb * per_img);
        q.npix = q.wT;
        q.gn = (q.wT + 32 * fv.fn - 1) / (32 * fv.fn);
        const long long tiles = (long long)q.gm * q.gn;
        EH_REQUIRE(tiles <= 0x3fffffffLL, "conv2d: too many tiles");
        const long long split_tiles = (nb == chunk_imgs) ? leftover : 0;  // a short last chunk runs undivided
        q.main_tiles = (int)(tiles - split_tiles);
        q.nslices = split_tiles > 0 ? nslices : 1;
        q.slice_steps = split_tiles > 0 ? slice_steps : q.nsteps;
        if (pool != nullptr) {
            const size_t po = (size_t)b0 * Kf * per_img;
            q.pool_O = pool->O + po; q.pool_ix = pool->ix + po; q.pool_iy = pool->iy + po;
            if (!pool->keep) q.O = nullptr;
        }
        const long long wgs = q.main_tiles + split_tiles * q.nslices;
        q.trace = (g_trace != nullptr && wgs <= g_trace_wgs) ? g_trace : nullptr;
        EH_TRY(prof_begin(st));
        hipLaunchKernelGGL(wide ? fv.kernel_wide : fv.kernel, dim3((unsigned)wgs), dim3(256), 0, st, q);
        EH_CHECK_LAUNCH();
        EH_TRY(prof_end(st));
        if (split_tiles > 0) {
            hipLaunchKernelGGL(fv.reduce, dim3((unsigned)(split_tiles * fv.fm * fv.fn)), dim3(256), 0, st, q);
            EH_CHECK_LAUNCH();
        }
    }
    const char *name = wide ? fv.name_wide : fv.name;
    if (leftover > 0) snprintf(g_last_kernel, sizeof(g_last_kernel), "winograd[%s +ksplit(%lld tiles x %d), %lld blocks]", name, leftover, nslices, (long long)N * per_img);
    else snprintf(g_last_kernel, sizeof(g_last_kernel), "winograd[%s, %lld blocks]", name, (long long)N * per_img);
    return 0;
}

}  // namespace

extern "C" {

int eddlhip_conv2d_fwd(int dev, const float *I, const float *K, const float *bias, float *O, int N, int C, int H, int W, int Kf,
                       int R, int S, int sr, int sc, int pad_top, int pad_left, int P, int Q, const float *bn_g, const float *bn_b,
                       const float *bn_mean, const float *bn_var, float bn_eps, const float *residual, int relu) {
    return conv2d_fwd_impl(false, dev, I, nullptr, 1, 1, K, bias, O, N, C, H, W, Kf, R, S, sr, sc, pad_top, pad_left, P, Q, bn_g, bn_b, bn_mean,
                           bn_var, bn_eps, residual, relu);
}

int eddlhip_conv2d_fwd_concat(int dev, const float *I_first, const float *I_second, const float *K, const float *bias, float *O,
                              int N, int C, int H, int W, int Kf, int R, int S, int sr, int sc, int pad_top, int pad_left, int P,
                              int Q, const float *bn_g, const float *bn_b, const float *bn_mean, const float *bn_var, float bn_eps,
                              const float *residual, int relu) {
    EH_REQUIRE(N == 0 || (I_first && I_second), "conv2d_fwd_concat: NULL input tensor");
    if (N == 0) return 0;
    return conv2d_fwd_impl(false, dev, I_first, I_second, 1, 1, K, bias, O, N, C, H, W, Kf, R, S, sr, sc, pad_top, pad_left, P, Q, bn_g, bn_b,
                           bn_mean, bn_var, bn_eps, residual, relu);
}

int eddlhip_conv2d_fwd_upsampled(int dev, const float *I, int up_h, int up_w, const float *K, const float *bias, float *O, int N, int C,
                                 int H, int W, int Kf, int R, int S, int sr, int sc, int pad_top, int pad_left, int P, int Q,
                                 const float *bn_g, const float *bn_b, const float *bn_mean, const float *bn_var, float bn_eps,
                                 const float *residual, int relu) {
    return conv2d_fwd_impl(false, dev, I, nullptr, up_h, up_w, K, bias, O, N, C, H, W, Kf, R, S, sr, sc, pad_top, pad_left, P, Q, bn_g, bn_b,
                           bn_mean, bn_var, bn_eps, residual, relu);
}

int eddlhip_conv2d_fwd_maxpool(int dev, const float *I, const float *I_second, int up_h, int up_w, const float *K, const float *bias, float *O,
                               int N, int C, int H, int W, int Kf, int R, int S, int sr, int sc, int pad_top, int pad_left, int P, int Q,
                               const float *bn_g, const float *bn_b, const float *bn_mean, const float *bn_var, float bn_eps,
                               const float *residual, int relu, float *pool_O, float *pool_indX, float *pool_indY, int keep_O) {
    EH_REQUIRE(P > 0 && Q > 0 && P % 2 == 0 && Q % 2 == 0, "conv2d_fwd_maxpool: the output planes must have even sides, got %d x %d", P, Q);
    EH_REQUIRE(N == 0 || (O && pool_O && pool_indX && pool_indY), "conv2d_fwd_maxpool: NULL output tensor");
    EH_REQUIRE(up_h >= 1 && up_w >= 1 && (I_second == nullptr || (up_h == 1 && up_w == 1)), "conv2d_fwd_maxpool: bad input form");
    if (N == 0) return 0;
    PoolRequest req = {pool_O, pool_indX, pool_indY, keep_O != 0, false};
    g_pool_req = &req;
    const int rc = conv2d_fwd_impl(false, dev, I, I_second, up_h, up_w, K, bias, O, N, C, H, W, Kf, R, S, sr, sc, pad_top, pad_left, P, Q, bn_g,
                                   bn_b, bn_mean, bn_var, bn_eps, residual, relu);
    g_pool_req = nullptr;
    if (rc != 0 || req.done) return rc;
    return eddlhip_maxpool2d(dev, O, pool_O, pool_indX, pool_indY, N, Kf, P, Q, 2, 2, 2, 2, 0, 0, 0, 0);
}

int eddlhip_conv2d_fwd_noalloc(int dev, const float *I, const float *K, const float *bias, float *O, int N, int C, int H, int W, int Kf,
                               int R, int S, int sr, int sc, int pad_top, int pad_left, int P, int Q, const float *bn_g,
                               const float *bn_b, const float *bn_mean, const float *bn_var, float bn_eps, const float *residual,
                               int relu) {
    return conv2d_fwd_impl(true, dev, I, nullptr, 1, 1, K, bias, O, N, C, H, W, Kf, R, S, sr, sc, pad_top, pad_left, P, Q, bn_g, bn_b,
                           bn_mean, bn_var, bn_eps, residual, relu);
}

}  // extern "C"

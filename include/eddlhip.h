/*
 * eddlhip.h - C ABI of libeddlhip.so, an MI355X (gfx950) backend for the CNN forward path
 * of EDDL (deephealthproject/eddl v1.1).
 *
 * The library replaces, for forward/inference, the family of `gpu_*` free functions that
 * EDDL's Tensor / tensorNN dispatchers call when a tensor lives on a GPU device
 * (declared in the reference's include/eddl/hardware/gpu/gpu_tensor.h:45-53,
 * include/eddl/hardware/gpu/gpu_hw.h:30-257 and include/eddl/hardware/gpu/nn/gpu_tensor_nn.h:26-147).
 * Those functions take Tensor* / Descriptor* C++ objects; thin C++ shims unpack the
 * objects into the flat calls below (plain pointers and sizes).
 *
 * Conventions
 *  - All tensors are fp32, contiguous, row-major: activations NCHW, filters OIHW,
 *    dense weights [in, out].  Pointers named `const float*`/`float*` are DEVICE pointers
 *    unless the parameter name starts with `host`.
 *  - Every function returns 0 on success or a negative EDDLHIP_E* code; a message for the
 *    last failure on the calling thread is available from eddlhip_last_error().
 *  - Kernels are launched asynchronously on one stream per device (the null stream unless
 *    eddlhip_set_stream was called); eddlhip_synchronize() waits for them.  The reference's
 *    wrappers synchronise after every launch (e.g. src/hardware/gpu/nn/gpu_pool.cu:27-33);
 *    the C++ shims reproduce that by calling eddlhip_synchronize() before returning.
 *  - The library never owns user-visible tensors.  It keeps one private, grow-only
 *    workspace per device (repacked filters); eddlhip_shutdown() releases it.
 *  - Calls on one device must not overlap from several threads (the reference drives one
 *    device from one thread: src/net/net_api.cpp:146-171).  Different devices may be driven
 *    from different threads.  The tuning and measurement switches (eddlhip_conv2d_set_algo,
 *    _autotune, _tuned_load / _tuned_save, _profile, _profile_read, _trace) act on the whole
 *    process: change them only while no other thread is inside the library.
 *    eddlhip_conv2d_force_plan acts on the calling thread only.
 */
#ifndef EDDLHIP_H
#define EDDLHIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define EDDLHIP_OK 0
#define EDDLHIP_EINVAL (-1)  /* bad argument (shape, null pointer, unsupported mode) */
#define EDDLHIP_EHIP (-2)    /* a HIP runtime call failed */
#define EDDLHIP_ENODEV (-3)  /* no such device */
#define EDDLHIP_ENOMEM (-4)  /* device allocation failed */

/* ------------------------------------------------------------------ runtime
 * Replaces gpu_devices / gpu_init / gpu_set_device / gpu_create_tensor / gpu_delete_tensor
 * (src/hardware/gpu/gpu_tensor.cu:121-240) and gpu_copy_to_gpu / gpu_copy_from_gpu /
 * gpu_copy_gpu / gpu_fill_ (src/hardware/gpu/gpu_core.cu:49-67,139-147). */
const char *eddlhip_version(void);
const char *eddlhip_last_error(void);
int eddlhip_device_count(int *count);
int eddlhip_init(int dev);
int eddlhip_shutdown(int dev);
int eddlhip_device_name(int dev, char *buf, size_t buflen);
int eddlhip_set_stream(int dev, void *hip_stream);
int eddlhip_synchronize(int dev);
int eddlhip_malloc(int dev, size_t bytes, void **dev_ptr);
int eddlhip_free(int dev, void *dev_ptr);
int eddlhip_memcpy_h2d(int dev, void *dev_dst, const void *host_src, size_t bytes);
int eddlhip_memcpy_d2h(int dev, void *host_dst, const void *dev_src, size_t bytes);
int eddlhip_memcpy_d2d(int dev, void *dev_dst, const void *dev_src, size_t bytes);
int eddlhip_fill(int dev, float *A, size_t n, float v);
/* Size of the library's private workspace on the device right now (it only grows; 0 before the first call that
 * needs one).  eddlhip_workspace_trim waits for the device's kernels and releases the workspace, so that it grows back
 * to what the calls from then on need (a plan search does this itself when its candidates have grown the workspace).
 * Not while a graph is being recorded; graphs recorded before name the released memory and refuse to launch.
 * No counterpart in the reference. */
int eddlhip_workspace_bytes(int dev, size_t *bytes);
int eddlhip_workspace_trim(int dev);

/* Batch staging.  The reference moves a batch to the device through pageable host tensors and
 * blocking copies (Net::distributeTensor / collectTensor, src/net/net_func.cpp:195-249; a D2H +
 * H2D round trip per batch, src/tensor/tensor_core.cpp:877-895).  These entry points let a host
 * overlap that traffic with the kernels: page-locked host buffers, copies queued on two more
 * streams of the device (one for uploads, one for downloads, so neither waits behind the other),
 * and events to order them against the compute stream.
 *   eddlhip_memcpy_h2d_async / _d2h_async: queue the copy on the upload / download stream and
 *     return; the host buffer should come from eddlhip_host_malloc (a pageable one makes the copy
 *     synchronous) and must stay untouched until done_event (recorded on that stream behind the
 *     copy; may be NULL) has completed.
 *   eddlhip_stream_wait_event: work queued later on the device's compute stream waits for event.
 *   eddlhip_upload_wait_event / eddlhip_download_wait_event: uploads / downloads queued later wait
 *     for event (e.g. one recorded with eddlhip_event_record after the kernels that last read the
 *     upload's destination, or that wrote the download's source). */
int eddlhip_host_malloc(int dev, void **host_ptr, size_t bytes);
int eddlhip_host_free(int dev, void *host_ptr);
int eddlhip_memcpy_h2d_async(int dev, void *dev_dst, const void *host_src, size_t bytes, void *done_event);
int eddlhip_memcpy_d2h_async(int dev, void *host_dst, const void *dev_src, size_t bytes, void *done_event);
int eddlhip_stream_wait_event(int dev, void *event);
int eddlhip_upload_wait_event(int dev, void *event);
int eddlhip_download_wait_event(int dev, void *event);
int eddlhip_event_synchronize(int dev, void *event);

/* Graphs.  A plan of short kernels (a small network, a small batch) can take longer to queue launch by
 * launch than to run.  Between eddlhip_graph_begin and eddlhip_graph_end the library's launches on the
 * device are recorded instead of run (stream capture on a stream of the library's own, default priority);
 * eddlhip_graph_end returns the recorded sequence as a graph that eddlhip_graph_launch replays, in one
 * call, on the device's stream - same kernels, same arguments, same order, hence the same results bit for
 * bit.  Pointers and shapes are frozen into the graph: replay only while the tensors it names are alive,
 * and record again after a resize.  Run the same calls once BEFORE recording, so that the workspace has
 * its final size and registered filters are repacked; calls that wait for the device, copy from or to the
 * host, allocate or free are refused while recording.  A call that fails while recording leaves the
 * recording open: close it with eddlhip_graph_end (which then reports the failure too).
 * A recorded convolution or dense call that took the library's workspace names it by address; when a later,
 * larger call has made the library replace that workspace, eddlhip_graph_launch refuses the graph with
 * EDDLHIP_EINVAL ("record again") instead of letting its kernels write into freed memory.
 * No counterpart in the reference, which synchronises after every kernel. */
int eddlhip_graph_begin(int dev);
int eddlhip_graph_end(int dev, void **graph);
int eddlhip_graph_launch(int dev, void *graph);
int eddlhip_graph_destroy(int dev, void *graph);

/* Events on the device's stream, for timing kernels where they run.  No counterpart in the
 * reference (its profiling is host wall-clock, include/eddl/profiling.h:27-66). */
int eddlhip_event_create(int dev, void **event);
int eddlhip_event_destroy(int dev, void *event);
int eddlhip_event_record(int dev, void *event);
int eddlhip_event_elapsed_ms(int dev, void *start, void *stop, float *ms);

/* ------------------------------------------------------------------ convolution
 * Replaces gpu_conv2D(ConvolDescriptor*) (src/hardware/gpu/nn/gpu_conv.cu:159-233; CPU
 * semantics src/hardware/cpu/nn/cpu_conv.cpp:55-112,114-226,316-346).
 *
 * Cross-correlation.  I[N,C,H,W], K[Kf,C,R,S], O[N,Kf,P,Q].  Output pixel (p,q) reads taps
 * (p*sr - pad_top + ky, q*sc - pad_left + kx); taps outside the image read 0.  P and Q come
 * from the descriptor (its geometry rules are not a closed form of the pads), so they are
 * arguments; only the top/left pads enter the arithmetic, as in the reference's lowering.
 * bias may be NULL (descriptor's use_bias == false).
 *
 * Fused epilogue (all optional; what a Conv -> BatchNorm(inference) -> Add -> ReLU chain of
 * layers computes, applied per output element in this order, each step rounded to fp32
 * with no fused multiply-add):
 *     v = acc;  if bias: v = v + bias[k]
 *     if bn_mean: v = ((v - bn_mean[k]) / sqrtf(bn_var[k] + bn_eps)) * bn_g[k] + bn_b[k]
 *                 (bn_g/bn_b NULL => no affine step)
 *     if residual: v = v + residual[same index as O]
 *     if relu: v = v > 0 ? v : 0
 * With the epilogue pointers NULL and relu 0 it is exactly the descriptor call. */
int eddlhip_conv2d_fwd(int dev, const float *I, const float *K, const float *bias, float *O,
                       int N, int C, int H, int W, int Kf, int R, int S, int sr, int sc,
                       int pad_top, int pad_left, int P, int Q,
                       const float *bn_g, const float *bn_b, const float *bn_mean, const float *bn_var,
                       float bn_eps, const float *residual, int relu);

/* A channel Concat of two tensors folded into the convolution that consumes it (no counterpart in the
 * reference, which materialises the concatenation: src/layers/merge/layer_concat.cpp:87-94 followed by
 * LConv::forward).  The input is I_first[N,C/2,H,W] for channels [0, C/2) and I_second[N,C/2,H,W] for
 * channels [C/2, C); C is the filters' channel count.  Every other argument, the fused epilogue and the
 * result are those of eddlhip_conv2d_fwd on the concatenated tensor, bit for bit (same taps in the same
 * order).  Taken by the 1x1, 2x2 and 3x3 kernels; other filter shapes are refused with EDDLHIP_EINVAL and
 * the caller concatenates first. */
int eddlhip_conv2d_fwd_concat(int dev, const float *I_first, const float *I_second, const float *K, const float *bias,
                              float *O, int N, int C, int H, int W, int Kf, int R, int S, int sr, int sc,
                              int pad_top, int pad_left, int P, int Q,
                              const float *bn_g, const float *bn_b, const float *bn_mean, const float *bn_var,
                              float bn_eps, const float *residual, int relu);

/* Nearest-neighbour UpSampling2D by whole factors folded into the convolution that consumes it (no counterpart in
 * the reference, which writes the enlarged tensor: src/layers/core/layer_resize.cpp:22-47 followed by
 * LConv::forward).  I[N,C,H,W] is the tensor BEFORE upsampling; the convolution runs over the image of
 * H*up_h x W*up_w pixels whose pixel (y, x) is I's pixel (y / up_h, x / up_w) - the mapping of the reference's
 * nearest / asymmetric scale for whole factors (src/hardware/cpu/cpu_da.cpp:109-113; checked on the host, the call
 * is refused where the two differ).  pad_top / pad_left, P and Q refer to the enlarged image.  Everything else,
 * and the result, are those of eddlhip_conv2d_fwd on the enlarged tensor, bit for bit.  Taken by the 1x1, 2x2 and
 * 3x3 kernels; other filter shapes are refused with EDDLHIP_EINVAL and the caller resizes first. */
int eddlhip_conv2d_fwd_upsampled(int dev, const float *I, int up_h, int up_w, const float *K, const float *bias, float *O,
                                 int N, int C, int H, int W, int Kf, int R, int S, int sr, int sc,
                                 int pad_top, int pad_left, int P, int Q,
                                 const float *bn_g, const float *bn_b, const float *bn_mean, const float *bn_var,
                                 float bn_eps, const float *residual, int relu);

/* A convolution (with its fused epilogue) whose output goes through a 2x2, stride-2, unpadded max-pool - the
 * Conv -> [BN] -> ReLU -> MaxPool(2, 2) step of the reference's VGG and U-Net encoders (LMaxPool::forward after
 * LConv::forward, src/layers/pool/layer_maxpool.cpp:62-64 and src/layers/conv/layer_conv2D.cpp:91-93) as one call.
 * O, pool_O, pool_indX and pool_indY receive exactly what eddlhip_conv2d_fwd (or _concat with I_second != NULL, or
 * _upsampled with up_h, up_w > 1) followed by eddlhip_maxpool2d(O, 2, 2, 2, 2, no padding) would write, bit for bit
 * for the convolution form the call takes.  P and Q must be even.  Where the convolution runs in a Winograd form its
 * epilogue holds whole 2x2 blocks of outputs and pools them itself: no pool launch, and with keep_O == 0 the unpooled
 * outputs are not written at all (O must still be a buffer of the full size: the other forms compute it and pool it
 * with the pool kernel; its contents after a call with keep_O == 0 are unspecified). */
int eddlhip_conv2d_fwd_maxpool(int dev, const float *I, const float *I_second, int up_h, int up_w, const float *K,
                               const float *bias, float *O, int N, int C, int H, int W, int Kf, int R, int S, int sr, int sc,
                               int pad_top, int pad_left, int P, int Q,
                               const float *bn_g, const float *bn_b, const float *bn_mean, const float *bn_var,
                               float bn_eps, const float *residual, int relu,
                               float *pool_O, float *pool_indX, float *pool_indY, int keep_O);

/* eddlhip_conv2d_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid it).  No counterpart in the reference.  Same arguments, same kernels,
 * same launch plan and therefore the same result, bit for bit, as eddlhip_conv2d_fwd; the difference is where
 * the call's scratch memory comes from (the repacked filters unless they are registered with
 * eddlhip_conv2d_cache_filters, the tap table of filter shapes other than 1x1 / 2x2 / 3x3, the partial tiles of
 * a K-split launch): a fixed array of EDDLHIP_CONV_NOALLOC_SCRATCH_BYTES in the library's device image, one copy
 * per device, instead of the grow-only workspace.  The call makes no hipMalloc / hipFree and no allocating
 * library call.  It returns EDDLHIP_EINVAL, and launches nothing, when
 *   - the device has not been initialised (call eddlhip_init(dev) once beforehand; that call allocates),
 *   - the scratch need exceeds the array (the message gives the figures),
 *   - eddlhip_conv2d_profile is collecting (its event pairs are allocated on demand).
 * Every call on a device uses that device's one array, which keeps the previous call's contents; each call
 * writes what it reads from it before reading, so nothing has to be cleared, but two calls that overlap on
 * one device (from two threads, or on two streams) race on it. */
#define EDDLHIP_CONV_NOALLOC_SCRATCH_BYTES (64u << 20)
int eddlhip_conv2d_fwd_noalloc(int dev, const float *I, const float *K, const float *bias, float *O,
                               int N, int C, int H, int W, int Kf, int R, int S, int sr, int sc,
                               int pad_top, int pad_left, int P, int Q,
                               const float *bn_g, const float *bn_b, const float *bn_mean, const float *bn_var,
                               float bn_eps, const float *residual, int relu);

/* Selects the convolution kernel: 0 = automatic; 1 = matrix-core (MFMA) implicit GEMM;
 * 2 = the scalar direct kernel (one thread per output; taps summed in the reference's ky,kx,c
 * order with its rounding - used to cross-check the MFMA kernels on the device);
 * 3 = MFMA with the operand slices staged through registers; 4 = MFMA with the operand slices
 * written by the load unit straight into LDS (what 0 and 1 select); 5 / 6 = switch off / on the
 * division along K of the tiles left over after a whole number of tiles per CU (on by default;
 * independent of 0-4); 7 / 8 = switch on / off the Winograd form for every convolution it applies to
 * (off by default; independent of 5 / 6; only under 0); 9 = no Winograd form at all: the plan search does not try
 * it and a kept plan that names it runs the planner's own choice instead (8 returns to the default).
 *
 * The Winograd form, F(2x2, 3x3): a 3x3 stride-1 convolution (any paddings, one or two input tensors, stored or
 * upsampled image) computed as an input transform, 16 products of [Kf x C] by [C x blocks of 2x2 outputs] matrices -
 * one launch of the 1x1 MFMA kernel - and an output transform that carries the fused epilogue: 2.25 times fewer
 * multiplications, the role of the WINOGRAD algorithms among those the reference lets cuDNN choose from
 * (src/hardware/gpu/nn/gpu_conv.cu:42-66).  Sums run in a fixed order (reproducible) and differ from the direct form's
 * by rounding: the result meets the same tolerance against the reference's CPU convolution, it is not bit-identical to
 * the direct form.  It takes workspace (16/4 of the input and of the output, plus what its product launch needs for the
 * partial tiles of a K-split plan), so eddlhip_conv2d_fwd_noalloc never uses it.  Chosen per geometry by the plan search
 * (below) where it is faster, or everywhere by 7, or by eddlhip_conv2d_force_plan(4, .).  A second form, for input channel
 * counts that are multiples of 16 (force_plan(5, .), or the search): one product launch walks through all 16 patch
 * positions and folds each product into the outputs as it completes, so the products are never written and there is no
 * output-transform launch; it sums the 16 positions in another order than the first form (same tolerance, not the same
 * bits).  A third form, for 3x3 filters (force_plan(6, .) / (7, .), or the search): ONE launch that reads the NCHW input
 * itself - raw pixels and transformed filters are staged through LDS, a lane derives its transformed operands from LDS
 * reads and additions, a workgroup keeps all 16 positions' products of its tile (32 or 64 filters x 32 blocks) in
 * registers and transforms them at the end - so no transformed input or product is ever in memory and the only
 * workspace is the transformed filters (unless registered) and the partial output tiles of a K-split plan.  Where the
 * stored image has rows of a multiple of four pixels and the input tensors are 16-byte aligned the kernel loads its pixels
 * 16 bytes per lane (its name in eddlhip_conv2d_last_kernel then ends in ",true>"), 4 bytes per lane otherwise: same sums,
 * same bits.  Non-finite inputs: the
 * transforms take differences of neighbouring pixels, so an infinity in the input can turn into NaN in outputs where the
 * direct form yields an infinity (all finite inputs give finite outputs as in the direct form); a caller that relies on
 * the propagation of infinities keeps the plan search off or calls eddlhip_conv2d_set_algo(9).
 *
 * The upsampled-input form of a 2x2 filter (force_plan(8, .) / (9, .), or the search): a 2x2 stride-1 convolution of ONE
 * tensor that eddlhip_conv2d_fwd_upsampled enlarges twice in both directions, without padding above or to the left (the
 * convolution behind each UpSampling2D of a U-Net decoder, with its Pad of one row below and one column to the right), is
 * computed on the stored image: output (2a + i, 2b + j) only sees the stored pixels (a .. a + i, b .. b + j), each under
 * the sum of the filter taps that land on it, so the four parities of the output position are four convolutions with
 * 1x1, 1x2, 2x1 and 2x2 filters - 9 multiplications per channel where the direct form has 16, no transform and no
 * workspace beyond the nine weight sums per filter and channel (kept with a registered filter tensor).  One launch, four
 * accumulators per lane, the epilogue of the Winograd forms (a lane holds whole 2x2 blocks of outputs; the 2x2 max-pool
 * can ride along).  The weight sums are rounded once in fp32, so the result differs from the direct form's by rounding
 * (same tolerance).  Because a convolution of the stored, enlarged tensor cannot take this form, such a call is a
 * geometry of its own in the plans table (kind 2 / 3 instead of 0 / 1): the same layer run after a stand-alone
 * UpSampling2D keeps its own plan, and the two agree to the convolution's tolerance, not bit for bit.
 *
 * eddlhip_conv2d_last_kernel() names the kernel the calling thread's last eddlhip_conv2d_fwd
 * launched, followed by " +ksplit(T tiles x S)" when T tiles were divided into S slices; for the Winograd form
 * "winograd[<kernel and plan of the product launch>, <blocks per product> blocks]", for the upsampled-input form
 * "upsampled2x2[<kernel>, <blocks> blocks]". */
int eddlhip_conv2d_set_algo(int algo);
const char *eddlhip_conv2d_last_kernel(void);

/* Plan search on first use.  eddlhip_conv2d_autotune(1): from now on the first eddlhip_conv2d_fwd* call with a geometry the
 * device has not seen (N, C, Kf, R, S, strides, output size P x Q) runs that convolution under every launch plan (tile
 * shape x K slices and the Winograd forms, every launch timed by itself, the fastest of three to nine launches per plan,
 * on the call's own tensors) and remembers one; later calls with that geometry take it.  Which one: of all plans within
 * 3 % of the fastest, the first in a fixed order of preference (the planner's own plan, the one-launch Winograd form, the
 * direct tiles, the Winograd forms that keep a transformed input in memory - those are tried only below 512 MB of
 * workspace; within a form fewer K slices first), so that two searches of one geometry agree unless two plans differ by
 * just that margin.  A caller that needs run-to-run identical bits loads a plans file instead of searching.  The call's
 * tensors must not alias: when the output overlaps an input or the residual, nothing is searched or recorded and the
 * planner's plan runs (repeating such a call would change what it reads).  The reference does the same on a layer's first forward, with
 * cudnnFindConvolutionForwardAlgorithm (src/hardware/gpu/nn/gpu_conv.cu:42-66, 211-213).  Neither the epilogue, nor the
 * image size and paddings (a folded Pad layer changes both), nor the form of the input (one tensor, two, upsampled) is
 * part of the geometry, so a layer computes the same sums in a fused plan and layer by layer - with the one exception of
 * a 2x2 filter on an input upsampled twice (above), whose own form exists only for the folded call.  A plan that divides tiles
 * along K adds its slices in another order than an undivided one, so results with and without the search agree to the
 * convolution's tolerance, not bit for bit.  Calls that must not allocate or wait (graph recording,
 * eddlhip_conv2d_fwd_noalloc, eddlhip_conv2d_profile collecting) do not search; they use what was found.
 * eddlhip_conv2d_autotune(0) stops searching and using the table, eddlhip_conv2d_autotune(-1) also empties it.
 * eddlhip_conv2d_tuned_plans(dev) = number of geometries in the table.  With EDDLHIP_TUNE_VERBOSE set in the environment every
 * search prints one line to stderr (geometry, the planner's time, the best time and plan). */
int eddlhip_conv2d_autotune(int on);
int eddlhip_conv2d_tuned_plans(int dev);
/* The table as a text file (one geometry and its plan per line), so that a later process starts from what an earlier
 * one found: _save writes the device's table, _load merges a file into it (a geometry already in the table takes the
 * file's plan).  A loaded plan is used like a found one while eddlhip_conv2d_autotune(1) is in force.  A file from
 * another device model is accepted (its plans are valid launches) but was not measured there. */
int eddlhip_conv2d_tuned_save(int dev, const char *host_path);
int eddlhip_conv2d_tuned_load(int dev, const char *host_path);

/* Overrides the launch planner of the MFMA kernels (tuning and tests): tile = 0 (128x128 outputs per
 * workgroup), 1 (64x128), 2 (64x64), 3 (32x128) or -1 to give the choice back to the planner;
 * slices = number of K slices the tiles left over after a whole number per CU are divided into
 * (1 = none).  tile = 4: the Winograd form wherever it applies (its product launch is planned or searched as usual),
 * 5: its folded form wherever that applies, 6 / 7: its one-launch form on tiles of 32 / 64 filters x 32 blocks, `slices`
 * K slices for the left-over tiles as above; 8 / 9: the upsampled-input form of a 2x2 filter, built for three / two
 * workgroups per CU; the planner's choice wherever a form does not apply.  Acts on the calling thread only. */
int eddlhip_conv2d_force_plan(int tile, int slices);

/* Filters that stay fixed between calls (inference).  Every eddlhip_conv2d_fwd first repacks its
 * filters into the kernels' tap-major layout (3-10 us per layer).  After
 * eddlhip_conv2d_cache_filters(dev, K, ...) the library keeps that repacked copy in device memory
 * of its own, and calls that pass the same K pointer and shape use it instead.  The caller
 * promises that K's contents change only through this library: eddlhip_memcpy_h2d/_d2d, _fill,
 * _add and _inc into a registered tensor mark its copy stale (it is repacked on the next use);
 * a kernel of the caller's own that writes K must be followed by another
 * eddlhip_conv2d_cache_filters call.  eddlhip_free of the tensor, eddlhip_conv2d_uncache_filters
 * (K == NULL: every tensor of the device) and eddlhip_shutdown drop the copy.
 * No counterpart in the reference, whose gpu_conv2D reads OIHW filters on every call
 * (src/hardware/gpu/nn/gpu_conv.cu:159-233); the C++ host layer does not register anything, so
 * training-style callers that update filters between calls see the reference's behaviour. */
int eddlhip_conv2d_cache_filters(int dev, const float *K, int Kf, int C, int R, int S);
int eddlhip_conv2d_uncache_filters(int dev, const float *K);

/* Measurement hook (no counterpart in the reference).  eddlhip_conv2d_profile(1) starts a
 * collection: from then on every launch of a convolution kernel made by eddlhip_conv2d_fwd
 * (one per batch chunk, so one per call for inputs up to 2 GiB; not the filter repack, not the
 * finishing kernel of a K-split) is bracketed by its own pair of events on the device's stream.
 * eddlhip_conv2d_profile_read waits for those launches and returns how many there were and the
 * sum of their durations; eddlhip_conv2d_profile(0) stops collecting.  Either call of
 * eddlhip_conv2d_profile forgets what was collected before. */
int eddlhip_conv2d_profile(int collect);
/* Measurement hook (no counterpart in the reference): while `words` (device memory, 8 x workgroups 64-bit words) is
 * set, every launch of a compile-time-filter-shape MFMA kernel (1x1, 2x2, 3x3) of at most `workgroups` workgroups
 * writes one record per workgroup, indexed by workgroup id: words 0..3 = the device's constant 100 MHz clock at entry,
 * when the operands of the first K-step are in LDS, at the end of the K loop and at the end of the kernel with its
 * stores drained (tracing adds that wait); word 4 = the HW_ID register (low half: wavefront slot, SIMD, CU, shader
 * engine) and the XCC_ID register (high half); words 5 and 6 = the shader clock at the first and the last mark.
 * A later launch overwrites the records.  eddlhip_conv2d_trace(NULL, 0) switches it off. */
int eddlhip_conv2d_trace(unsigned long long *words, long long workgroups);
int eddlhip_conv2d_profile_read(int *launches, float *total_ms);

/* ------------------------------------------------------------------ batch normalisation (inference)
 * Replaces gpu_batchnorm_forward(...) with trmode == false
 * (include/eddl/hardware/gpu/nn/gpu_tensor_nn.h:138-143, src/hardware/gpu/nn/gpu_bn.cu:65-98;
 * CPU semantics src/hardware/cpu/nn/cpu_bn.cpp:154-179).  b = batch, z = channels, rc = H*W.
 * Writes sd[c] = sqrtf(global_variance[c] + eps) into `variance` (the layer's bn_var), then
 * o = (x - global_mean[c]) / sd[c]; with affine (affine_g != NULL): opa = o (if opa != NULL)
 * and y = o*g[c] + b[c]. */
int eddlhip_batchnorm_inference(int dev, int b, int z, int rc, const float *input, float *output, float *opa,
                                const float *global_mean, const float *global_variance,
                                const float *affine_g, const float *affine_b, float *variance, float epsilon);

/* ------------------------------------------------------------------ activations
 * Replace gpu_relu / gpu_sigmoid / gpu_full_softmax
 * (include/eddl/hardware/gpu/nn/gpu_tensor_nn.h:26,44,59; CPU semantics
 * src/hardware/cpu/nn/cpu_activations.cpp:18-33,329-375, src/hardware/cpu/cpu_math.cpp:354-357).
 * Softmax runs over an axis of length `len` whose stride is `inner`; `outer` is the product
 * of the dimensions before it. */
int eddlhip_relu(int dev, const float *A, float *B, size_t n);
int eddlhip_sigmoid(int dev, const float *A, float *B, size_t n);
int eddlhip_softmax(int dev, const float *A, float *B, int outer, int len, int inner, int stable);

/* ------------------------------------------------------------------ pooling
 * Replace gpu_mpool2D / gpu_avgpool2D(PoolDescriptor*)
 * (src/hardware/gpu/nn/gpu_pool.cu:26-46,101-117; CPU semantics
 * src/hardware/cpu/nn/cpu_pool.cpp:74-121,226-274).  Window origins run
 * i = -pad_top; i <= H + pad_bottom - kr; i += sr (same for columns); outputs are written
 * densely in that loop order.  eddlhip_pool2d_out_dims returns the two loop counts.
 * Max: indX/indY receive the absolute column/row of the first maximum, as floats; a window
 * with no tap above -3.40282e+38f leaves its two index slots untouched.
 * Avg: in-image taps summed in (ky,kx) order, divided by kr*kc. */
int eddlhip_pool2d_out_dims(int H, int W, int kr, int kc, int sr, int sc,
                            int pad_top, int pad_bottom, int pad_left, int pad_right, int *LP, int *LQ);
int eddlhip_maxpool2d(int dev, const float *I, float *O, float *indX, float *indY,
                      int N, int C, int H, int W, int kr, int kc, int sr, int sc,
                      int pad_top, int pad_bottom, int pad_left, int pad_right);
int eddlhip_avgpool2d(int dev, const float *I, float *O,
                      int N, int C, int H, int W, int kr, int kc, int sr, int sc,
                      int pad_top, int pad_bottom, int pad_left, int pad_right);

/* ------------------------------------------------------------------ resize / concat / add / pad
 * eddlhip_scale_nearest replaces gpu_scale(A, B, new_shape, wrap, c, mode) for the only
 * combination UpSampling2D uses: nearest wrapping, "asymmetric" coordinates
 * (src/hardware/gpu/gpu_da.cu:61-76; CPU semantics src/hardware/cpu/cpu_da.cpp:88-137,407-436).
 * A[N,C,H,W] -> B[N,C,OH,OW]; source index = (int)((float)(dst + off) / ((float)new / in)),
 * off = (int)((new - out)/2.0f).  Destination elements whose source falls outside A are left
 * untouched and make the call fail with EDDLHIP_EINVAL (the reference raises there).
 *
 * eddlhip_concat replaces gpu_concat(A, t, axis, false) with the CPU backend's semantics
 * (src/hardware/cpu/cpu_core.cpp:368-396): n_in device pointers (host array), the axis extent
 * of each, `outer` = product of dims before the axis, `inner` = stride of the axis.
 *
 * eddlhip_add replaces gpu_add(scA, A, scB, B, C, incC) (src/hardware/gpu/gpu_math.cu:446-455;
 * CPU src/hardware/cpu/cpu_math.cpp:278-287); eddlhip_inc replaces gpu_inc.
 *
 * eddlhip_pad replaces gpu_pad(A, B, pads) (CPU src/hardware/cpu/cpu_da.cpp:502-517): interior
 * copy, pads in the reference's (top, right, bottom, left) order; B's border is not written. */
int eddlhip_scale_nearest(int dev, const float *A, float *B, int N, int C, int H, int W, int OH, int OW,
                          int newH, int newW);
int eddlhip_concat(int dev, float *dest, const float *const *host_srcs, const int *host_axis_extent, int n_in,
                   int outer, int inner);
int eddlhip_add(int dev, float scA, const float *A, float scB, const float *B, float *C, int incC, size_t n);
int eddlhip_inc(int dev, const float *A, float *B, size_t n);
int eddlhip_pad(int dev, const float *A, float *B, int N, int C, int H, int W,
                int top, int right, int bottom, int left);

/* ------------------------------------------------------------------ parameter initialisation on the device
 * What EDDL's initialisers run on a GPU tensor when eddl::build creates the device copy of a net
 * (Net::split -> make_graph -> do_initialize, src/net/net_build.cpp:235-237,401; e.g. IGlorotUniform::apply,
 * src/initializers/initializer_glorot_uniform.cpp:35-60): the four random fills
 * gpu_rand_uniform / gpu_rand_signed_uniform / gpu_rand_normal / gpu_rand_binary
 * (include/eddl/hardware/gpu/gpu_hw.h:58-61; distributions as src/hardware/cpu/cpu_generator.cpp:14-49) and the
 * scalar operations gpu_mult(A, B, v) and gpu_add(A, B, v) (gpu_hw.h:89,106) behind Tensor::mult_ / add_ / sub_.
 *
 * Random fills are counter-based (Philox4x32-10): element i of a fill is a function of (seed, i) alone, so a
 * fill is reproducible whatever the launch shape, and different seeds give independent streams; the caller
 * picks a new seed per fill (the C++ binding counts fills per device from a fixed base, as the reference's
 * cuRAND generator is seeded with a constant, src/hardware/gpu/gpu_tensor.cu:179-185).  With u uniform on
 * [0, 1) in steps of 2^-24:
 *   eddlhip_rand_uniform         A[i] = u * v
 *   eddlhip_rand_signed_uniform  A[i] = (2u - 1) * v
 *   eddlhip_rand_binary          A[i] = u < v ? 1 : 0
 *   eddlhip_rand_normal          A[i] = z * stddev + mean, z standard normal (Box-Muller)
 * The reference's own random streams (cuRAND MRG32k3a on the GPU, std::mt19937 seeded from std::random_device
 * on the CPU) are not reproduced: only the distributions are its contract.
 * eddlhip_rand_words writes the generator's raw 32-bit words (bit patterns stored in the float slots; block b of
 * four words is Philox4x32-10 with key = seed and counter = (first_block + b, counter_hi)): for known-answer tests.
 * eddlhip_mult_scalar: B = A * v;  eddlhip_add_scalar: B = A + v;  A == B is allowed. */
int eddlhip_rand_uniform(int dev, float *A, size_t n, float v, unsigned long long seed);
int eddlhip_rand_signed_uniform(int dev, float *A, size_t n, float v, unsigned long long seed);
int eddlhip_rand_binary(int dev, float *A, size_t n, float v, unsigned long long seed);
int eddlhip_rand_normal(int dev, float *A, size_t n, float mean, float stddev, unsigned long long seed);
int eddlhip_rand_words(int dev, float *A, size_t n, unsigned long long seed, unsigned long long first_block,
                       unsigned long long counter_hi);
int eddlhip_mult_scalar(int dev, const float *A, float *B, size_t n, float v);
int eddlhip_add_scalar(int dev, const float *A, float *B, size_t n, float v);

/* ------------------------------------------------------------------ dense
 * eddlhip_mult2d replaces gpu_mult2D(A, tA, B, tB, C, incC) for the forward case
 * tA = tB = 0 used by LDense::forward (src/layers/core/layer_dense.cpp:65-73,
 * src/hardware/gpu/gpu_math.cu:457-488): C[m,n] (+)= A[m,k] * B[k,n], row-major.
 * eddlhip_sum2d_rowwise replaces gpu_sum2D_rowwise: C[i][j] = A[i][j] + B[j]. */
int eddlhip_mult2d(int dev, const float *A, const float *B, float *C, int m, int k, int n, int incC);
int eddlhip_sum2d_rowwise(int dev, const float *A, const float *B, float *C, int rows, int cols);
/* LDense::forward in one call: C[m,n] = A[m,k] * W[k,n], then + bias[column] when bias != NULL
 * (sum2D_rowwise), then ReLU when relu != 0 (the LActivation that commonly follows; 
 * src/hardware/cpu/nn/cpu_activations.cpp:18-33).  Each step is the separate call's fp32 operation,
 * so the result equals eddlhip_mult2d + eddlhip_sum2d_rowwise + eddlhip_relu bit for bit. */
int eddlhip_dense_fwd(int dev, const float *A, const float *W, const float *bias, float *C, int m, int k, int n, int relu);

#ifdef __cplusplus
}
#endif
#endif /* EDDLHIP_H */

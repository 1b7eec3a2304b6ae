/* eddlhip_probe - device probes beside the C ABI of include/eddlhip.h, in a library of their own
 * (eddl_amd/libeddlhip_probe.so, built from eddl_amd/csrc/probe.hip and linked against libeddlhip.so, whose device state
 * and stream they use).  They are measurement tools of the benchmark, not part of the drop-in boundary: nothing in the
 * reference corresponds to them and no convolution, pooling or element-wise call needs this library.
 */
#ifndef EDDLHIP_PROBE_H
#define EDDLHIP_PROBE_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Device probe: TFLOP/s that v_mfma_f32_32x32x2_f32 sustains with nothing else running, over
 * `launches` back-to-back launches of about 7 ms each (mean, best launch, worst launch).
 * vary_operands == 0: every MFMA reads the same two registers; != 0: operands change from one
 * instruction to the next, as in a real product (the device then lowers its clock at times).
 * No counterpart in the reference; the benchmark reports the result beside the published peak. */
int eddlhip_probe_mfma_f32(int dev, int vary_operands, int launches, float *tflops_mean, float *tflops_best,
                           float *tflops_worst);
/* Device probe: GB/s that plain streams over device memory sustain with nothing else running - read only,
 * write only, and copy (bytes read + bytes written) - over two buffers of `bytes` each that the call
 * allocates and frees (choose them larger than the device's caches: 1 GiB).  16-byte accesses, four in
 * flight per thread or one, with and without the streaming (non-temporal) hint, several grid sizes; the best rate
 * of each kind is returned.  It is what the bandwidth-bound kernels can be measured against beside the
 * published 8 TB/s.  No counterpart in the reference. */
int eddlhip_probe_hbm(int dev, size_t bytes, float *read_gbs, float *write_gbs, float *copy_gbs);

#ifdef __cplusplus
}
#endif

#endif /* EDDLHIP_PROBE_H */

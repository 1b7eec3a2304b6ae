// Seeded synthetic tensors for the benchmark configurations: one generator that a C++ host and a Python host
// (ctypes) share, so that both build the same inputs and parameters from a seed alone.  Never EDDL's own generator,
// which cannot be seeded (src/random.cpp:25-26).
//
//   engine   std::mt19937(seed) - its output sequence is fixed by the C++ standard
//   uniform  u = (word >> 8) * 2^-24 in [0, 1), one word per value:  out = (float)(lo + (hi - lo) * u)
//   normal   Box-Muller, two words per PAIR of values: u1 = ((w0 >> 8) + 1) * 2^-24 in (0, 1], u2 = (w1 >> 8) * 2^-24,
//            r = sqrt(-2 ln u1);  out[2j] = (float)(mean + stddev * r cos(2 pi u2)),  out[2j+1] = ... r sin(2 pi u2)
//            (double arithmetic, one rounding to float at the end).  A fill of an odd count drops the last sine value:
//            every fill starts on a fresh pair.
// Values are drawn in row-major order, tensor after tensor in the order of the calls.
#pragma once
#include <stddef.h>
#include <stdint.h>

extern "C" {
typedef struct eddl_synth eddl_synth;
eddl_synth *eddl_synth_new(uint32_t seed);
void eddl_synth_free(eddl_synth *s);
void eddl_synth_words(eddl_synth *s, uint32_t *out, size_t n);  // the engine's raw output (tests)
void eddl_synth_uniform(eddl_synth *s, float *out, size_t n, float lo, float hi);
void eddl_synth_normal(eddl_synth *s, float *out, size_t n, float mean, float stddev);
}

namespace eddl_hip {
class Net;
// Fills every parameter of a net that has NOT been moved to a device yet (host tensors), layer by layer in the net's
// layer order, tensor by tensor in the layer's parameter order:
//   convolution  K ~ N(0, sqrt(2 / (C R S))) (He normal, src/initializers/initializer_he_normal.cpp:38-42), bias 0
//   dense        W ~ N(0, sqrt(2 / in)) (the 2-D rule, :35-37), bias 0
//   batch norm   gamma ~ U(0.8, 1.2), beta ~ N(0, 0.1) (when affine), running mean ~ N(0, 0.1), running variance ~ U(0.5, 1.5)
void synth_he_normal(Net *net, uint32_t seed);
}  // namespace eddl_hip

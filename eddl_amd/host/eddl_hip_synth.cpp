#include "eddl_hip_synth.h"

#include <cmath>
#include <random>
#include <vector>

#include "eddl_hip_net.h"

struct eddl_synth {
    std::mt19937 engine;
};

extern "C" {

eddl_synth *eddl_synth_new(uint32_t seed) { return new eddl_synth{std::mt19937(seed)}; }

void eddl_synth_free(eddl_synth *s) { delete s; }

void eddl_synth_words(eddl_synth *s, uint32_t *out, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = (uint32_t)s->engine();
}

void eddl_synth_uniform(eddl_synth *s, float *out, size_t n, float lo, float hi) {
    const double a = lo, span = (double)hi - (double)lo;
    for (size_t i = 0; i < n; i++) {
        const double u = (double)((uint32_t)s->engine() >> 8) * (1.0 / 16777216.0);
        out[i] = (float)(a + span * u);
    }
}

void eddl_synth_normal(eddl_synth *s, float *out, size_t n, float mean, float stddev) {
    const double two_pi = 6.283185307179586476925286766559, m = mean, sd = stddev;
    // the engine is sequential; the transform of a block of pairs is not, so it runs over all cores
    const size_t BLOCK = (size_t)1 << 16;  // pairs
    std::vector<uint32_t> w(2 * BLOCK);
    for (size_t p0 = 0; p0 * 2 < n; p0 += BLOCK) {
        const size_t pairs = std::min(BLOCK, (n - 2 * p0 + 1) / 2);
        for (size_t i = 0; i < 2 * pairs; i++) w[i] = (uint32_t)s->engine();
#pragma omp parallel for schedule(static)
        for (long j = 0; j < (long)pairs; j++) {
            const double u1 = ((double)(w[2 * j] >> 8) + 1.0) * (1.0 / 16777216.0), u2 = (double)(w[2 * j + 1] >> 8) * (1.0 / 16777216.0);
            const double r = std::sqrt(-2.0 * std::log(u1)), t = two_pi * u2;
            const size_t i = 2 * (p0 + (size_t)j);
            out[i] = (float)(m + sd * (r * std::cos(t)));
            if (i + 1 < n) out[i + 1] = (float)(m + sd * (r * std::sin(t)));
        }
    }
}

}  // extern "C"

namespace eddl_hip {

void synth_he_normal(Net *net, uint32_t seed) {
    eddl_synth *s = eddl_synth_new(seed);
    auto normal = [s](Tensor *t, float sd) {
        if (!t->isCPU()) msg("the parameters are on a device already: fill them before build", "synth_he_normal");
        eddl_synth_normal(s, t->ptr, t->size, 0.0f, sd);
    };
    auto uniform = [s](Tensor *t, float lo, float hi) { eddl_synth_uniform(s, t->ptr, t->size, lo, hi); };
    for (Layer *l : net->layers) {
        if (LConv *conv = dynamic_cast<LConv *>(l)) {
            const ConvolDescriptor *D = conv->cd;
            normal(D->K, (float)std::sqrt(2.0 / (double)(D->kz * D->kr * D->kc)));
            D->bias->fill_(0.0f);
        } else if (LDense *dense = dynamic_cast<LDense *>(l)) {
            normal(dense->W, (float)std::sqrt(2.0 / (double)dense->W->shape[0]));
            if (dense->use_bias) dense->bias->fill_(0.0f);
        } else if (LBatchNorm *bn = dynamic_cast<LBatchNorm *>(l)) {
            if (bn->affine) {
                uniform(bn->bn_g, 0.8f, 1.2f);
                normal(bn->bn_b, 0.1f);
            }
            normal(bn->mean, 0.1f);
            uniform(bn->variance, 0.5f, 1.5f);
        }
    }
    eddl_synth_free(s);
}

}  // namespace eddl_hip

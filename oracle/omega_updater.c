/*
 * CPU restatement of the reference's AdamW step.  TEST INFRASTRUCTURE ONLY: nothing the library ships may call it.
 *
 * Follows adamw_kernel (J/engine/updater/gpu/updater.cu:31-52) as AdamWKernel.updateW / updateB / updateGamma launch
 * it (J/engine/updater/gpu/AdamWKernel.java:177-195,301-320,380-399): eps = 1e-8f, the two bias corrections formed on
 * the host as (float)(1.0f - Math.pow(beta, train_time)).
 *
 * Pinned by tests/test_oracle_updater.py: torch.optim.AdamW in float64 over several steps (an independent
 * implementation of the same algebra), the closed form of the first step (m_hat = g, v_hat = g*g, so the step is
 * lr * (g / (|g| + eps) + wd * w)), and zero gradient = pure decay.  PARITY UNPINNED at the bit level: the CUDA
 * compiler contracts a*b + c into fused multiply-adds where it sees fit and the reference's binary is not here; the
 * two contractions written out below (the decay term and the final step) are the ones the source's expression shape
 * offers.  Against the float64 algebra the difference is a few ulp of the step.
 */
#include "oracle_common.h"

/* lerp(start, end, weight) = fma(weight, end, fma(-weight, start, start)): updater.cu:31-33 */
static inline float lerp_f(float start, float end, float weight) { return fmaf(weight, end, fmaf(-weight, start, start)); }

float orc_adamw_correction(float beta, int train_time) { return (float)(1.0 - pow((double)beta, (double)train_time)); }

void orc_adamw(float *w, const float *grad, float *mw, float *vw, long n, float lr, float beta1, float beta2, float b1c,
               float b2c, float eps, float wd)
{
    for (long i = 0; i < n; ++i) {
        const float g = grad[i];
        const float m = lerp_f(g, mw[i], beta1);
        const float v = lerp_f(g * g, vw[i], beta2);
        mw[i] = m;
        vw[i] = v;
        const float mh = m / b1c, vh = v / b2c;
        const float t = fmaf(wd, w[i], mh / (sqrtf(vh) + eps));
        w[i] = fmaf(-lr, t, w[i]);
    }
}

/*
 * ORACLE — test infrastructure only (see moe_oracle.c for the rules).
 *
 * Scalar C restatement of the compute block of MixedPrecisionAdamW.step,
 * optimus/optimizers.py:162-205 (formula restated at optimizers.py:1745-1760).
 * One torch elementwise op of the reference = one individually rounded fp32
 * operation here (-ffp-contract=off); the Python scalars (beta, 1-beta, the two
 * bias corrections, -lr, -lr*wd) are computed in double by the caller exactly as
 * the reference computes them and are narrowed to float when they meet a float
 * tensor, which is what torch does with a Python scalar operand.
 */
#include <stdint.h>
#include <string.h>
#include <math.h>

typedef uint16_t bf16_t;

static inline float bf16_to_f32(bf16_t h) {
    uint32_t u = ((uint32_t)h) << 16; float f; memcpy(&f, &u, 4); return f;
}
static inline bf16_t f32_to_bf16(float f) {
    uint32_t u; memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)0x7fc0;
    uint32_t lsb = (u >> 16) & 1u; u += 0x7fffu + lsb; return (bf16_t)(u >> 16);
}

/*
 * step is the 1-based step number t = step_id + 1.
 *   optimizers.py:190  g = float(grad)
 *   optimizers.py:193  m = m*b1 ; m = m + (1-b1)*g
 *   optimizers.py:194  v = v*b2 ; v = v + (1-b2)*g*g          (addcmul: value*t1*t2)
 *   optimizers.py:195  mh = m / (1 - b1^t)
 *   optimizers.py:196  vh = v / (1 - b2^t)
 *   optimizers.py:197  d  = sqrt(vh) + eps
 *   optimizers.py:198  w  = w + (-lr) * mh / d                (addcdiv: value*(t1/t2))
 *   optimizers.py:202  w  = w + (-lr*wd) * w                  (only when wd > 0)
 *   optimizers.py:205  p  = bf16(w)
 */
void orc_adamw_step_bf16(bf16_t *param, const bf16_t *grad, float *master,
                         float *exp_avg, float *exp_avg_sq, int64_t n,
                         double lr, double beta1, double beta2, double eps,
                         double weight_decay, int64_t step) {
    const float b1 = (float)beta1, b2 = (float)beta2;
    const float omb1 = (float)(1.0 - beta1), omb2 = (float)(1.0 - beta2);
    const float bc1 = (float)(1.0 - pow(beta1, (double)step));
    const float bc2 = (float)(1.0 - pow(beta2, (double)step));
    const float epsf = (float)eps, neg_lr = (float)(-lr);
    const float neg_lr_wd = (float)(-lr * weight_decay);
    for (int64_t i = 0; i < n; i++) {
        float g = bf16_to_f32(grad[i]);
        float m = exp_avg[i] * b1;
        m = m + omb1 * g;
        float v = exp_avg_sq[i] * b2;
        v = v + (omb2 * g) * g;
        float mh = m / bc1;
        float vh = v / bc2;
        float d = sqrtf(vh) + epsf;
        float w = master[i];
        w = w + neg_lr * (mh / d);
        if (weight_decay > 0.0) w = w + neg_lr_wd * w;
        exp_avg[i] = m; exp_avg_sq[i] = v; master[i] = w;
        param[i] = f32_to_bf16(w);
    }
}

/* fp32-dtype mode of the reference (optimizers.py:100-102): master aliases param. */
void orc_adamw_step_f32(float *param_master, const float *grad,
                        float *exp_avg, float *exp_avg_sq, int64_t n,
                        double lr, double beta1, double beta2, double eps,
                        double weight_decay, int64_t step) {
    const float b1 = (float)beta1, b2 = (float)beta2;
    const float omb1 = (float)(1.0 - beta1), omb2 = (float)(1.0 - beta2);
    const float bc1 = (float)(1.0 - pow(beta1, (double)step));
    const float bc2 = (float)(1.0 - pow(beta2, (double)step));
    const float epsf = (float)eps, neg_lr = (float)(-lr);
    const float neg_lr_wd = (float)(-lr * weight_decay);
    for (int64_t i = 0; i < n; i++) {
        float g = grad[i];
        float m = exp_avg[i] * b1;
        m = m + omb1 * g;
        float v = exp_avg_sq[i] * b2;
        v = v + (omb2 * g) * g;
        float mh = m / bc1;
        float vh = v / bc2;
        float d = sqrtf(vh) + epsf;
        float w = param_master[i];
        w = w + neg_lr * (mh / d);
        if (weight_decay > 0.0) w = w + neg_lr_wd * w;
        exp_avg[i] = m; exp_avg_sq[i] = v; param_master[i] = w;
    }
}

/* Same recurrence in double: the distance of the fp32 sequence from exact arithmetic. */
void orc_adamw_step_f64(const bf16_t *grad, double *master, double *exp_avg,
                        double *exp_avg_sq, int64_t n,
                        double lr, double beta1, double beta2, double eps,
                        double weight_decay, int64_t step) {
    const double bc1 = 1.0 - pow(beta1, (double)step);
    const double bc2 = 1.0 - pow(beta2, (double)step);
    for (int64_t i = 0; i < n; i++) {
        double g = (double)bf16_to_f32(grad[i]);
        double m = exp_avg[i] * beta1 + (1.0 - beta1) * g;
        double v = exp_avg_sq[i] * beta2 + (1.0 - beta2) * g * g;
        double d = sqrt(v / bc2) + eps;
        double w = master[i] - lr * (m / bc1) / d;
        if (weight_decay > 0.0) w = w - lr * weight_decay * w;
        exp_avg[i] = m; exp_avg_sq[i] = v; master[i] = w;
    }
}

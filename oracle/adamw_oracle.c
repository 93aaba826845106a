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

/*
 * Gradient norm and clip, optimizers.py:136-160: torch.nn.utils.get_total_norm over the
 * parameters' gradient views, then clip_grads_with_norm_(max_norm) when the step clips.
 * What those library calls compute for bf16 gradients (fp32 arithmetic inside each op, the
 * result of each op rounded to the tensor dtype):
 *   norm_i = bf16( sqrt( sum_j g_ij^2 ) )                 vector_norm of one gradient
 *   total  = bf16( sqrt( sum_i norm_i^2 ) )               vector_norm of the stacked norms
 *   coef   = min( bf16( bf16( 1 / bf16(total + 1e-6) ) * max_norm ), 1 )
 *            (max_norm / tensor is evaluated as tensor.reciprocal() * max_norm)
 *   g_ij   = bf16( g_ij * coef )                          in-place multiply by the 0-dim tensor
 * The sums are taken in double here and rounded once to float: the library's own summation order
 * is not specified, and any fp32 order differs from this by far less than one bf16 step except
 * exactly at a rounding boundary.
 */
void orc_grad_norm_clip_bf16(const bf16_t *grad, const int64_t *starts, const int64_t *sizes,
                             int64_t n_params, double max_norm, float *seg_norms,
                             float *total_norm, float *clip_coef) {
    double tot = 0.0;
    for (int64_t p = 0; p < n_params; p++) {
        double acc = 0.0;
        for (int64_t j = 0; j < sizes[p]; j++) {
            double g = (double)bf16_to_f32(grad[starts[p] + j]);
            acc += g * g;
        }
        float nrm = bf16_to_f32(f32_to_bf16(sqrtf((float)acc)));
        seg_norms[p] = nrm;
        tot += (double)nrm * (double)nrm;
    }
    float total = bf16_to_f32(f32_to_bf16(sqrtf((float)tot)));
    *total_norm = total;
    float x = bf16_to_f32(f32_to_bf16(total + 1e-6f));
    float r = bf16_to_f32(f32_to_bf16(1.0f / x));
    float c = bf16_to_f32(f32_to_bf16(r * (float)max_norm));
    *clip_coef = c > 1.0f ? 1.0f : c;
}

void orc_grad_norm_clip_f32(const float *grad, const int64_t *starts, const int64_t *sizes,
                            int64_t n_params, double max_norm, float *seg_norms,
                            float *total_norm, float *clip_coef) {
    double tot = 0.0;
    for (int64_t p = 0; p < n_params; p++) {
        double acc = 0.0;
        for (int64_t j = 0; j < sizes[p]; j++) {
            double g = (double)grad[starts[p] + j];
            acc += g * g;
        }
        float nrm = sqrtf((float)acc);
        seg_norms[p] = nrm;
        tot += (double)nrm * (double)nrm;
    }
    float total = sqrtf((float)tot);
    *total_norm = total;
    float x = total + 1e-6f;
    float r = 1.0f / x;
    float c = r * (float)max_norm;
    *clip_coef = c > 1.0f ? 1.0f : c;
}

/* The in-place multiply of clip_grads_with_norm_: g = cast(float(g) * coef). */
void orc_scale_grads_bf16(bf16_t *grad, int64_t n, float coef) {
    for (int64_t i = 0; i < n; i++) grad[i] = f32_to_bf16(bf16_to_f32(grad[i]) * coef);
}
void orc_scale_grads_f32(float *grad, int64_t n, float coef) {
    for (int64_t i = 0; i < n; i++) grad[i] = grad[i] * coef;
}

/*
 * Clip decision of the sharded optimizer, ShardedMixedPrecisionAdamW.step, optimizers.py:398-432.
 * The shard's norm is get_total_norm of ONE tensor (the rank's slice of the flat gradient), i.e.
 * bf16( sqrt( sum g^2 ) ) for bf16 gradients (orc_grad_norm_clip_* with a single segment gives it).
 *   mode 0, no process group (:404-405): grad_norm is that 0-dim tensor in the gradient dtype, and
 *     clip_coef = max_norm / (grad_norm + 1e-6) = (grad_norm + 1e-6).reciprocal() * max_norm is
 *     evaluated in that dtype: sum, reciprocal and product each rounded.
 *   mode 1, process group (:399-403): `value` is the all-reduced sum of float(norm)^2 over the ranks;
 *     grad_norm = sqrt(value), clip_coef = 1 / (grad_norm + 1e-6) * max_norm, all fp32.
 * :431-432 multiplies the shard in place only if clip_coef < 1.  Both operands of that mul_ live on
 * the device, so torch casts the 0-dim coefficient to the gradient dtype before the multiply (a CPU
 * 0-dim operand would be taken as an exact scalar instead; the reference's norm is a device tensor).
 * `multiplier` is therefore round(clip_coef) when clip_coef < 1 and 1 otherwise (NaN included).
 */
static float round_bf16(float x) { return bf16_to_f32(f32_to_bf16(x)); }
void orc_shard_clip_multiplier(float value, int mode, int grad_is_bf16, double max_norm,
                               float *grad_norm, float *multiplier) {
    float norm, c;
    if (mode == 0) {
        norm = value;
        if (grad_is_bf16) {
            float x = round_bf16(norm + 1e-6f);
            float r = round_bf16(1.0f / x);
            c = round_bf16(r * (float)max_norm);
        } else {
            c = (1.0f / (norm + 1e-6f)) * (float)max_norm;
        }
    } else {
        norm = sqrtf(value);
        c = (1.0f / (norm + 1e-6f)) * (float)max_norm;
    }
    *grad_norm = norm;
    *multiplier = (c < 1.0f) ? (grad_is_bf16 ? round_bf16(c) : c) : 1.0f;
}

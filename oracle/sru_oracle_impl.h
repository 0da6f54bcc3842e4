/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Body of the CPU oracle for the SRU elementwise recurrence, compiled twice by
 * sru_oracle.c: once with REAL=float (a serial restatement of the reference's
 * arithmetic in its own precision, used as the timed CPU baseline) and once with
 * REAL=double (the checker every parity test compares against).
 *
 * Tensor layouts are the reference's:
 *   U        (L, B, D', k)   k = 3 or 4 innermost       sru/modules.py:193-194
 *   x,h,c    (L, B, D')      D' = dirs*d, col = b*D' + dir*d + j
 *   weight_c (2, D')         or per-step V (L, B, D', 2) when is_custom
 *   bias     (2, D')
 *   c_init, mask_c, c_last, grad_last, grad_init  (B, D')
 *   mask_pad (L, B) bytes, non-zero = padded
 * Columns whose direction index is 1 walk time from L-1 down to 0
 * (sru/csrc/sru_cuda_kernel.cu:223-234, sru/csrc/sru_cpu_impl.cpp:190).
 */

/* sigmoid as the reference writes it: sru/csrc/sru_cpu_impl.cpp:229-231,
 * sru/csrc/sru_cuda_kernel.cu:8-11 */
static inline REAL FN(sigmoid)(REAL v) {
    return (REAL)1 / ((REAL)1 + EXP(-v));
}

/*
 * Forward scan. Follows the loop nest of sru/csrc/sru_cpu_impl.cpp:101-138 (uni)
 * and :186-224 (bi): time outermost, state (B, D') updated in place, a padded
 * (t, b) is skipped so that h stays 0 and the state carries over (:104, :191).
 * On top of that CPU routine it takes what only the GPU kernels of the reference
 * have: the dropout mask on the output gate (sru/csrc/sru_cuda_kernel.cu:413,:434),
 * the per-step state c (:436, kept for the backward pass) and skip_type 0/1/2
 * (:416,:429,:434). scale_x multiplies x only (sru/cuda_functional.py:76,
 * sru_cpu_impl.cpp:131). For a per-step V the reverse direction reads V at the
 * real time step, as sru_cuda_kernel.cu:631-634 and sru/ops.py:211-212 do (the
 * CPU routine of the reference indexes it by the loop counter, :202-203, which
 * disagrees with both).
 */
void FN(sru_oracle_forward)(
    const REAL *U, const REAL *x, const REAL *weight_c, const REAL *bias,
    const REAL *c_init, const REAL *mask_c, const uint8_t *mask_pad,
    int64_t L, int64_t B, int64_t d, int dirs, int k,
    int activation_type, int skip_type, int is_custom, REAL scale_x,
    REAL *h, REAL *c_all, REAL *c_last)
{
    const int64_t Dp = d * dirs;
    const int64_t ncols = B * Dp;
    for (int64_t i = 0; i < ncols; ++i) c_last[i] = c_init[i];
    for (int64_t i = 0; i < L * ncols; ++i) h[i] = 0;

    for (int64_t l = 0; l < L; ++l) {
        for (int64_t b = 0; b < B; ++b) {
            for (int64_t j = 0; j < Dp; ++j) {
                const int64_t t = (j < d) ? l : (L - 1 - l);
                const int64_t col = b * Dp + j;
                const int pad = mask_pad && mask_pad[t * B + b];
                REAL cur = c_last[col];
                if (!pad) {
                    const REAL *u = U + (t * ncols + col) * k;
                    const REAL u0 = u[0], u1 = u[1], u2 = u[2];
                    const REAL wc1 = is_custom ? weight_c[(t * ncols + col) * 2] : weight_c[j];
                    const REAL wc2 = is_custom ? weight_c[(t * ncols + col) * 2 + 1] : weight_c[Dp + j];
                    const REAL m = mask_c ? mask_c[col] : (REAL)1;
                    const REAL g1 = FN(sigmoid)(u1 + wc1 * cur + bias[j]);
                    const REAL g2 = FN(sigmoid)(u2 + wc2 * cur + bias[Dp + j]);
                    cur = (cur - u0) * g1 + u0;
                    const REAL val = activation_type ? TANH(cur) : cur;
                    REAL hv;
                    if (skip_type) {
                        const REAL xv = (skip_type == 1) ? x[t * ncols + col] * scale_x : u[3];
                        hv = (val - xv) * m * g2 + xv;
                    } else {
                        hv = val * m * g2;
                    }
                    h[t * ncols + col] = hv;
                    c_last[col] = cur;
                }
                if (c_all) c_all[t * ncols + col] = cur;
            }
        }
    }
}

/*
 * Backward scan, column by column in reverse walk order. Follows
 * sru/csrc/sru_cuda_kernel.cu:447-578 (uni) and :667-822 (bi): gates are
 * recomputed from u and the stored previous state (:522-523), padded steps
 * write nothing and leave the carried gradient alone (:511), grad_x is the
 * gradient w.r.t. x*scale_x times scale_x (sru/cuda_functional.py:253-255),
 * and the per-column sums of the weight_c / bias gradients (:572-576) are added
 * up over the batch (sru/cuda_functional.py:258-260) into (2, D') outputs.
 * With is_custom the weight_c gradient is per step, shape (L, B, D', 2)
 * (:533,:543), zero at padded steps.
 */
void FN(sru_oracle_backward)(
    const REAL *U, const REAL *x, const REAL *weight_c, const REAL *bias,
    const REAL *c_init, const REAL *mask_c, const uint8_t *mask_pad,
    const REAL *c_all, const REAL *grad_h, const REAL *grad_last,
    int64_t L, int64_t B, int64_t d, int dirs, int k,
    int activation_type, int skip_type, int is_custom, REAL scale_x,
    REAL *grad_u, REAL *grad_x, REAL *grad_wc, REAL *grad_bias, REAL *grad_init)
{
    const int64_t Dp = d * dirs;
    const int64_t ncols = B * Dp;
    for (int64_t i = 0; i < L * ncols * k; ++i) grad_u[i] = 0;
    if (grad_x) for (int64_t i = 0; i < L * ncols; ++i) grad_x[i] = 0;
    if (is_custom) for (int64_t i = 0; i < L * ncols * 2; ++i) grad_wc[i] = 0;
    else for (int64_t i = 0; i < 2 * Dp; ++i) grad_wc[i] = 0;
    for (int64_t i = 0; i < 2 * Dp; ++i) grad_bias[i] = 0;

    for (int64_t b = 0; b < B; ++b) {
        for (int64_t j = 0; j < Dp; ++j) {
            const int64_t col = b * Dp + j;
            const int flip = (j >= d);
            const REAL m = mask_c ? mask_c[col] : (REAL)1;
            const REAL b1 = bias[j], b2 = bias[Dp + j];
            REAL gwc1 = 0, gwc2 = 0, gb1 = 0, gb2 = 0;
            REAL cur = grad_last[col];
            /* the backward walk visits the forward walk's steps in reverse */
            for (int64_t s = L - 1; s >= 0; --s) {
                const int64_t t = flip ? (L - 1 - s) : s;
                if (mask_pad && mask_pad[t * B + b]) continue;
                const int64_t tprev = flip ? (t + 1) : (t - 1);
                const REAL cp = (s > 0) ? c_all[tprev * ncols + col] : c_init[col];
                const REAL cv = c_all[t * ncols + col];
                const REAL *u = U + (t * ncols + col) * k;
                const REAL u0 = u[0], u1 = u[1], u2 = u[2];
                const REAL wc1 = is_custom ? weight_c[(t * ncols + col) * 2] : weight_c[j];
                const REAL wc2 = is_custom ? weight_c[(t * ncols + col) * 2 + 1] : weight_c[Dp + j];
                const REAL xv = (skip_type == 0) ? (REAL)0
                              : (skip_type == 1) ? x[t * ncols + col] * scale_x : u[3];
                const REAL gh = grad_h[t * ncols + col];
                const REAL g1 = FN(sigmoid)(u1 + wc1 * cp + b1);
                const REAL g2 = FN(sigmoid)(u2 + wc2 * cp + b2);
                const REAL val = activation_type ? TANH(cv) : cv;
                const REAL dact = activation_type ? ((REAL)1 - val * val) : (REAL)1;

                const REAL gg2 = gh * (val - xv) * m * (g2 * ((REAL)1 - g2));
                gb2 += gg2;
                gwc2 += gg2 * cp;
                const REAL gc = gh * m * (g2 * dact) + cur;
                const REAL gg1 = gc * (cp - u0) * (g1 * ((REAL)1 - g1));
                gb1 += gg1;
                gwc1 += gg1 * cp;
                cur = gc * g1 + gg1 * wc1 + gg2 * wc2;

                REAL *gu = grad_u + (t * ncols + col) * k;
                gu[0] = gc * ((REAL)1 - g1);
                gu[1] = gg1;
                gu[2] = gg2;
                if (skip_type == 2) gu[3] = gh * ((REAL)1 - g2 * m);
                if (skip_type == 1) grad_x[t * ncols + col] = gh * ((REAL)1 - g2 * m) * scale_x;
                if (is_custom) {
                    grad_wc[(t * ncols + col) * 2] = gg1 * cp;
                    grad_wc[(t * ncols + col) * 2 + 1] = gg2 * cp;
                }
            }
            if (!is_custom) {
                grad_wc[j] += gwc1;
                grad_wc[Dp + j] += gwc2;
            }
            grad_bias[j] += gb1;
            grad_bias[Dp + j] += gb2;
            grad_init[col] = cur;
        }
    }
}

/* CPU oracle for the optimiser step.  TEST INFRASTRUCTURE ONLY (see oracle.c).
 *
 * Restates adam_step_individual_kernel of xyz-autodiff-cuda
 * (examples/mini-gaussian-splatting/gaussian_parameters.cu:260-320) and its
 * host launcher (:353-386: beta^t via powf, t = iteration), for one flat array
 * of parameters that share a learning rate.  The reference keeps an array of
 * structs and runs the same three statements on each of the nine fields; per
 * field the arithmetic is what is written here, in fp32:
 *
 *     lr_c = lr * sqrtf(1 - beta2^t) / (1 - beta1^t)
 *     m    = beta1 * m + (1 - beta1) * g
 *     v    = beta2 * v + (1 - beta2) * g * g
 *     p   -= lr_c * m / (sqrtf(v) + eps)
 *
 * No clamping is applied (the device kernel there applies none).
 */
#include <math.h>

void oracle_adam_step_f32(long n, float* p, const float* g, float* m, float* v, float lr, float beta1,
                          float beta2, float eps, int iteration) {
    float beta1_t = powf(beta1, (float)iteration);
    float beta2_t = powf(beta2, (float)iteration);
    float lr_c = lr * sqrtf(1.0f - beta2_t) / (1.0f - beta1_t);
#pragma omp parallel for schedule(static)
    for (long i = 0; i < n; ++i) {
        m[i] = beta1 * m[i] + (1.0f - beta1) * g[i];
        v[i] = beta2 * v[i] + (1.0f - beta2) * g[i] * g[i];
        p[i] -= lr_c * m[i] / (sqrtf(v[i]) + eps);
    }
}

/* Same recurrence in fp64, for error budgeting of the fp32 paths. */
void oracle_adam_step_f64(long n, double* p, const double* g, double* m, double* v, double lr, double beta1,
                          double beta2, double eps, int iteration) {
    double lr_c = lr * sqrt(1.0 - pow(beta2, iteration)) / (1.0 - pow(beta1, iteration));
    for (long i = 0; i < n; ++i) {
        m[i] = beta1 * m[i] + (1.0 - beta1) * g[i];
        v[i] = beta2 * v[i] + (1.0 - beta2) * g[i] * g[i];
        p[i] -= lr_c * m[i] / (sqrt(v[i]) + eps);
    }
}

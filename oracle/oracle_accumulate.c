/* CPU oracle for parallel gradient accumulation.  TEST INFRASTRUCTURE ONLY
 * (see oracle.c).
 *
 * The reference accumulates shared gradients by letting every thread call
 * VariableRef::add_grad, i.e. atomicAdd on the shared element
 * (include/xyz_autodiff/variable.cuh:48-50; the pattern is exercised by
 * tests/test_parallel_gradient_accumulation.cu:25-49).  Mathematically that is
 * a sum over threads per (slot, element); the order is unspecified.  Here the
 * sum is formed in fp64, so it serves as the order-independent truth:
 *
 *   sums[slot[i]][k]  += g_k(i)          k = 0..5: d w / d (sx, sy, theta, o, px, py)
 *   abs_sums[..][k]   += |g_k(i)|        the mass of the terms, to scale tolerances
 *
 * chain_in_double != 0: each thread's gradient is evaluated in fp64 from the
 * fp32 inputs (the exact answer); == 0: evaluated in fp32 exactly as the fp32
 * oracle does, then widened (isolates the error of the summation itself).
 * Slots outside [0, num_slots) are ignored.
 */
#include <stdlib.h>
#include <string.h>
#include <math.h>
#include <omp.h>

void oracle_chain_one_f32(const float* in, float* w_out, float* grads, float* q_out);
void oracle_chain_one_f64(const double* in, double* w_out, double* grads, double* q_out);

void oracle_accumulate_chain(long n, const float* sx, const float* sy, const float* theta, const float* o,
                             const float* px, const float* py, const int* slot, int num_slots,
                             int chain_in_double, double* sums, double* abs_sums) {
    size_t cells = (size_t)num_slots * 6;
    memset(sums, 0, cells * sizeof(double));
    memset(abs_sums, 0, cells * sizeof(double));
#pragma omp parallel
    {
        double* local = (double*)calloc(2 * cells, sizeof(double));
#pragma omp for schedule(static)
        for (long i = 0; i < n; ++i) {
            int s = slot[i];
            if (s < 0 || s >= num_slots) continue;
            double g[6];
            if (chain_in_double) {
                double in[6] = {sx[i], sy[i], theta[i], o[i], px[i], py[i]}, w;
                oracle_chain_one_f64(in, &w, g, 0);
            } else {
                float in[6] = {sx[i], sy[i], theta[i], o[i], px[i], py[i]}, w, gf[6];
                oracle_chain_one_f32(in, &w, gf, 0);
                for (int k = 0; k < 6; ++k) g[k] = gf[k];
            }
            for (int k = 0; k < 6; ++k) {
                local[(size_t)s * 6 + k] += g[k];
                local[cells + (size_t)s * 6 + k] += fabs(g[k]);
            }
        }
#pragma omp critical
        for (size_t c = 0; c < cells; ++c) {
            sums[c] += local[c];
            abs_sums[c] += local[cells + c];
        }
        free(local);
    }
}

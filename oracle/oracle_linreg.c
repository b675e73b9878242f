/* CPU oracle for the least-squares example.  TEST INFRASTRUCTURE ONLY (see
 * oracle.c): nothing that ships may call it.
 *
 * Restates, in fp64 and statement by statement, what xyz-autodiff-cuda computes
 * for one sample when compute_gradient_kernel
 * (examples/optimization/tests/test_linear_regression_gradient.cu:47-78) runs
 * its graph, using the forward and backward rules of the op logics involved:
 *
 *   SubConstantLogic  y = x - k;    x_bar += g          (operations/unary/sub_constant_logic.cuh:25-37)
 *   SquaredLogic      y = x * x;    x_bar += g * 2.0 * x (operations/unary/squared_logic.cuh:17-33)
 *   MulLogic          y = p * q;    p_bar += g * q; q_bar += g * p (operations/binary/mul_logic.cuh:25-39)
 *   AddLogic          y = p + q;    p_bar += g; q_bar += g         (operations/binary/add_logic.cuh:25-39)
 *
 * and the SGD loop of examples/optimization/linear_regression_sgd.cu: the
 * update of update_parameters_kernel (:126-134), the learning-rate schedule of
 * compute_learning_rate (:137-140).  The batch draw is passed in as explicit
 * rows (the reference draws them with cuRAND, :68-81, which has no CPU form).
 */
#include <math.h>

/* out[0..3] += d loss / d (a, b, c, d); returns the loss. */
static double linreg_one(const double p[4], double x1, double x2, double y, double out[4]) {
    /* forward, in the order the graph is nested */
    double a_minus_x1 = p[0] - x1;                  /* sub_constant(a, x1)     */
    double x1_term = a_minus_x1 * a_minus_x1;       /* squared                 */
    double c_minus_x2 = p[2] - x2;                  /* sub_constant(c, x2)     */
    double x2_squared = c_minus_x2 * c_minus_x2;    /* squared                 */
    double x2_term = p[1] * x2_squared;             /* mul(b, .)               */
    double both_terms = x1_term + x2_term;          /* add                     */
    double prediction = both_terms + p[3];          /* add(., d)               */
    double residual = prediction - y;               /* sub_constant(., y)      */
    double loss = residual * residual;              /* squared                 */

    /* backward from a seed of one on the loss */
    double g_residual = 1.0 * 2.0 * residual;       /* squared                 */
    double g_prediction = g_residual;               /* sub_constant            */
    double g_both = g_prediction;                   /* add: both operands      */
    double g_d = g_prediction;
    double g_x1_term = g_both;                      /* add: both operands      */
    double g_x2_term = g_both;
    double g_b = g_x2_term * x2_squared;            /* mul                     */
    double g_x2_squared = g_x2_term * p[1];
    double g_c_minus_x2 = g_x2_squared * 2.0 * c_minus_x2; /* squared          */
    double g_c = g_c_minus_x2;                      /* sub_constant            */
    double g_a_minus_x1 = g_x1_term * 2.0 * a_minus_x1;    /* squared          */
    double g_a = g_a_minus_x1;                      /* sub_constant            */

    out[0] += g_a;
    out[1] += g_b;
    out[2] += g_c;
    out[3] += g_d;
    return loss;
}

/* out[0..3] = sum of gradients, out[4] = sum of losses over n samples; sample i
 * is row rows[i] (or i when rows is null). */
void oracle_linreg_gradient_f64(long n, const double* x1, const double* x2, const double* y, const int* rows,
                                const double* params, double* out) {
    double sums[5] = {0.0, 0.0, 0.0, 0.0, 0.0};
    for (long i = 0; i < n; ++i) {
        long r = rows ? rows[i] : i;
        sums[4] += linreg_one(params, x1[r], x2[r], y[r], sums);
    }
    for (int k = 0; k < 5; ++k) out[k] = sums[k];
}

/* epochs steps; step e uses rows[e * batch .. (e + 1) * batch).  params is
 * updated in place; history (may be null) receives the mean loss before each
 * update. */
void oracle_linreg_sgd_f64(const double* x1, const double* x2, const double* y, const int* rows, double* params,
                           int batch, int epochs, double lr_first, double lr_last, double* history) {
    double decay_rate = log(lr_last / lr_first) / epochs;
    for (int e = 0; e < epochs; ++e) {
        double lr = lr_first * exp(decay_rate * e);
        double sums[5];
        oracle_linreg_gradient_f64(batch, x1, x2, y, rows + (long)e * batch, params, sums);
        for (int k = 0; k < 4; ++k) {
            double avg_grad = sums[k] / batch;
            params[k] -= lr * avg_grad;
        }
        if (history) history[e] = sums[4] / batch;
    }
}

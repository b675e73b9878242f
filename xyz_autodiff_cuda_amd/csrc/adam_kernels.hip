// Adam update over flat parameter arrays.
//
// The arithmetic per element is that of adam_step_individual_kernel in
// xyz-autodiff-cuda (examples/mini-gaussian-splatting/gaussian_parameters.cu:260-320):
//     lr_c = lr sqrt(1 - beta2^t) / (1 - beta1^t)
//     m = beta1 m + (1 - beta1) g;  v = beta2 v + (1 - beta2) g g;  p -= lr_c m / (sqrt(v) + eps)
// with beta^t formed on the host by powf (:353-356) and no clamping.  There the
// nine fields of an array of structs are updated by one lane per Gaussian with a
// learning rate per field group; here parameters, gradients and both moments
// are structure-of-arrays rows, so the update is one streaming pass over
// rows x n elements (28 bytes of traffic each) with a learning rate per row.
//
// The gated form reads one word of device memory first and leaves parameters and
// moments as they are when it is not zero, counting the update it withheld: a
// training loop that does not wait for the device hands it the word in which the
// step before it reports gradients that lack contributions (xad_splat_overflow_word).
#include <cmath>

#include "common.cuh"

namespace {

constexpr unsigned kBlock = 512;
constexpr int kMaxRows = 16;

struct RowRates {
    float lr_corrected[kMaxRows];
};

__global__ void __launch_bounds__(kBlock) adam_kernel(std::size_t n, int rows, float* __restrict__ p,
                                                      const float* __restrict__ g, float* __restrict__ m,
                                                      float* __restrict__ v, RowRates rates, float beta1, float beta2,
                                                      float eps, const std::uint32_t* __restrict__ hold_if_nonzero,
                                                      std::uint32_t* __restrict__ held_count) {
    const std::size_t i = static_cast<std::size_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (hold_if_nonzero != nullptr && *hold_if_nonzero != 0) {  // the same answer for every lane of the launch
        if (i == 0 && held_count != nullptr) atomicAdd(held_count, 1u);
        return;
    }
    if (i >= n) return;
    for (int r = 0; r < rows; ++r) {
        const std::size_t at = static_cast<std::size_t>(r) * n + i;
        const float grad = g[at];
        const float m_new = beta1 * m[at] + (1.0f - beta1) * grad;
        const float v_new = beta2 * v[at] + (1.0f - beta2) * grad * grad;
        m[at] = m_new;
        v[at] = v_new;
        p[at] -= rates.lr_corrected[r] * m_new / (::sqrtf(v_new) + eps);
    }
}

}  // namespace

namespace {

int adam_step(const char* who, std::size_t n, int rows, float* params, const float* grads, float* m, float* v,
              const float* row_learning_rates, float beta1, float beta2, float eps, int iteration,
              const std::uint32_t* hold_if_nonzero, std::uint32_t* held_count, void* stream) {
    if (n == 0 || rows == 0) return XAD_OK;
    XAD_REQUIRE(rows > 0 && rows <= kMaxRows, "%s: rows must be in 1..%d, got %d", who, kMaxRows, rows);
    XAD_REQUIRE(params && grads && m && v && row_learning_rates, "%s: null array", who);
    XAD_REQUIRE(iteration >= 1, "%s: iteration counts from 1, got %d", who, iteration);
    const float beta1_t = ::powf(beta1, static_cast<float>(iteration));
    const float beta2_t = ::powf(beta2, static_cast<float>(iteration));
    RowRates rates{};
    for (int r = 0; r < rows; ++r) rates.lr_corrected[r] = row_learning_rates[r] * ::sqrtf(1.0f - beta2_t) / (1.0f - beta1_t);
    hipLaunchKernelGGL(adam_kernel, dim3(xad::blocks_for(n, kBlock)), dim3(kBlock), 0, xad::as_stream(stream), n, rows,
                       params, grads, m, v, rates, beta1, beta2, eps, hold_if_nonzero, held_count);
    XAD_HIP_TRY(hipGetLastError());
    return XAD_OK;
}

}  // namespace

extern "C" int xad_adam_step_f32(std::size_t n, int rows, float* params, const float* grads, float* m, float* v,
                                 const float* row_learning_rates, float beta1, float beta2, float eps, int iteration,
                                 void* stream) {
    return adam_step("xad_adam_step_f32", n, rows, params, grads, m, v, row_learning_rates, beta1, beta2, eps, iteration,
                     nullptr, nullptr, stream);
}

extern "C" int xad_adam_step_gated_f32(std::size_t n, int rows, float* params, const float* grads, float* m, float* v,
                                       const float* row_learning_rates, float beta1, float beta2, float eps, int iteration,
                                       const std::uint32_t* hold_if_nonzero, std::uint32_t* held_count, void* stream) {
    XAD_REQUIRE(hold_if_nonzero, "xad_adam_step_gated_f32: hold_if_nonzero is null");
    return adam_step("xad_adam_step_gated_f32", n, rows, params, grads, m, v, row_learning_rates, beta1, beta2, eps, iteration,
                     hold_if_nonzero, held_count, stream);
}

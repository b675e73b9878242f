// Kernels in the shapes that users of the header library write, compiled for
// gfx950 only to read the compiler's resource report: every graph below has to
// stay in vector registers (no scratch, no LDS that the source did not ask for).
// Nothing here is launched.
#include <hip/hip_runtime.h>

#include <xyz_autodiff/xyz_autodiff.cuh>
#include <mini-gaussian-splatting/operations/covariance_generation.cuh>
#include <mini-gaussian-splatting/operations/mahalanobis_distance.cuh>

using namespace xyz_autodiff;

// Array-of-structures records as the caller of xyz-autodiff-cuda keeps them
// (examples/mini-gaussian-splatting/gaussian_parameters.h:12-18): 9 floats.
struct Splat {
    float centre[2];
    float log_scale[2];
    float angle[1];
    float rgb[3];
    float logit[1];
};

using Rgb = ConstArray<float, 3>;

// (1) forward-only loop: a per-pixel sum over all records, graph evaluated with
// forward() alone (shape of gaussian_splatting_kernel.cu:33-62).
extern "C" __global__ void resident_forward_loop(const Splat* splats, Rgb* image, int width, int height, int count) {
    const int x = blockIdx.x * blockDim.x + threadIdx.x;
    const int y = blockIdx.y * blockDim.y + threadIdx.y;
    if (x >= width || y >= height) return;
    Rgb pixel{};
    for (int i = 0; i < count; ++i) {
        Splat& s = const_cast<Splat&>(splats[i]);
        VariableRef<2, float> centre(s.centre, nullptr), log_scale(s.log_scale, nullptr);
        VariableRef<1, float> angle(s.angle, nullptr), logit(s.logit, nullptr);
        VariableRef<3, float> rgb(s.rgb, nullptr);
        auto scale = op::exp(log_scale);
        auto cov = op::scale_rotation_to_covariance_3param(scale, angle);
        auto inv = op::sym_matrix2_inv(cov);
        auto q = op::mahalanobis_distance_with_center(float(x), float(y), centre, inv);
        auto half = q * 0.5f;
        auto minus = op::neg(half);
        auto falloff = op::exp(minus);
        auto alpha = op::sigmoid(logit);
        auto weight = falloff * alpha;
        auto weight3 = op::broadcast<3>(weight);
        auto shaded = rgb * weight3;
        shaded.forward();
        pixel += shaded;
    }
    image[y * width + x] = pixel;
}

// (2) run() loop: the benchmark chain per record with atomics into shared gradients.
extern "C" __global__ void resident_run_loop(const Splat* splats, Splat* grads, int width, int height, int count) {
    const int x = blockIdx.x * blockDim.x + threadIdx.x;
    const int y = blockIdx.y * blockDim.y + threadIdx.y;
    if (x >= width || y >= height) return;
    for (int i = 0; i < count; ++i) {
        Splat& s = const_cast<Splat&>(splats[i]);
        Splat& g = grads[i];
        VariableRef<2, float> centre(s.centre, g.centre), log_scale(s.log_scale, g.log_scale);
        VariableRef<1, float> angle(s.angle, g.angle), logit(s.logit, g.logit);
        auto scale = op::exp(log_scale);
        auto cov = op::scale_rotation_to_covariance_3param(scale, angle);
        auto inv = op::sym_matrix2_inv(cov);
        auto q = op::mahalanobis_distance_with_center(float(x), float(y), centre, inv);
        auto half = q * 0.5f;
        auto minus = op::neg(half);
        auto falloff = op::exp(minus);
        auto alpha = op::sigmoid(logit);
        auto weight = falloff * alpha;
        weight.run();
    }
}

// (3) broadcast x colour - ConstArray -> l1_norm -> run(): the loss loop of
// gaussian_splatting_kernel.cu:73-111.
extern "C" __global__ void resident_broadcast_l1_run(const Splat* splats, Splat* grads, const Rgb* target, const Rgb* image,
                                                     int width, int height, int count) {
    const int x = blockIdx.x * blockDim.x + threadIdx.x;
    const int y = blockIdx.y * blockDim.y + threadIdx.y;
    if (x >= width || y >= height) return;
    const Rgb want = target[y * width + x];
    const Rgb have = image[y * width + x];
    for (int i = 0; i < count; ++i) {
        Splat& s = const_cast<Splat&>(splats[i]);
        Splat& g = grads[i];
        VariableRef<2, float> centre(s.centre, g.centre), log_scale(s.log_scale, g.log_scale);
        VariableRef<1, float> angle(s.angle, g.angle), logit(s.logit, g.logit);
        VariableRef<3, float> rgb(s.rgb, g.rgb);
        auto scale = op::exp(log_scale);
        auto cov = op::scale_rotation_to_covariance_3param(scale, angle);
        auto inv = op::sym_matrix2_inv(cov);
        auto q = op::mahalanobis_distance_with_center(float(x), float(y), centre, inv);
        if (q[0] > 8.0f) continue;
        auto half = q * 0.5f;
        auto minus = op::neg(half);
        auto falloff = op::exp(minus);
        auto alpha = op::sigmoid(logit);
        auto weight = falloff * alpha;
        auto weight3 = op::broadcast<3>(weight);
        auto shaded = rgb * weight3;
        Rgb rest = want - have;
        rest += shaded;
        auto diff = shaded - rest;
        auto loss = op::l1_norm(diff);
        loss.run();
    }
}

// (4) two roots over one shared node: forward both, seed both, backward both.
extern "C" __global__ void resident_two_roots(float* values, float* grads, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    VariableRef<2, float> a(values + 4 * i, grads + 4 * i), b(values + 4 * i + 2, grads + 4 * i + 2);
    auto shared = a * b;
    auto left = op::exp(shared);
    auto right = op::sin(shared);
    left.forward();
    right.forward();
    left.zero_grad();
    right.zero_grad();
    left.add_grad(0, 1.0f);
    left.add_grad(1, 1.0f);
    right.add_grad(0, 0.5f);
    right.add_grad(1, 0.5f);
    left.backward();
    right.backward();
}

// (5) a ternary node with a user-written logic (the shape of
// tests/operation/base/test_operation_chaining.cu:217-226: x*z + y).
struct FusedMulAddLogic {
    static constexpr std::size_t outputDim = 2;
    template <typename Out, typename X, typename Y, typename Z>
    __host__ __device__ void forward(Out& out, const X& x, const Y& y, const Z& z) const {
        for (std::size_t k = 0; k < 2; ++k) out[k] = x[k] * z[k] + y[k];
    }
    template <typename Out, typename X, typename Y, typename Z>
    __host__ __device__ void backward(const Out& out, X& x, Y& y, Z& z) const {
        for (std::size_t k = 0; k < 2; ++k) {
            x.add_grad(k, out.grad(k) * z[k]);
            y.add_grad(k, out.grad(k));
            z.add_grad(k, out.grad(k) * x[k]);
        }
    }
};

extern "C" __global__ void resident_ternary(float* values, float* grads, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    VariableRef<2, float> x(values + 6 * i, grads + 6 * i), y(values + 6 * i + 2, grads + 6 * i + 2),
        z(values + 6 * i + 4, grads + 6 * i + 4);
    auto ex = op::exp(x);
    TernaryOperation<2, FusedMulAddLogic, decltype(ex), decltype(y), decltype(z)> fma(FusedMulAddLogic{}, ex, y, z);
    auto total = op::sum(fma);
    total.run();
}

// (6) one graph object, leaves rewritten and forward() called again in a loop, a single
// backward at the end: the nodes carry their bookkeeping from trip to trip.
extern "C" __global__ void resident_repeated_forward(const float* samples, float* best, float* grads, int n, int trips) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    Variable<2, float> x;
    auto e = op::exp(x);
    auto s = op::squared(e);
    auto both = e + s;
    auto total = op::sum(both);
    float smallest = 3.0e38f;
    for (int t = 0; t < trips; ++t) {
        x[0] = samples[2 * (t * n + i)];
        x[1] = samples[2 * (t * n + i) + 1];
        total.forward();
        smallest = fminf(smallest, total[0]);
    }
    total.zero_grad();
    total.add_grad(0, 1.0f);
    total.backward();
    best[i] = smallest;
    grads[2 * i] = x.grad(0);
    grads[2 * i + 1] = x.grad(1);
}

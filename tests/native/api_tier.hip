// Test tier for the public operator API: runs the same case functions on the host
// cores and on the GPU, evaluates any op logic (values, analytic gradients,
// central-difference gradients) on either side, and reproduces the reference's
// concurrent-accumulation tests.  Built into tests/native/libxad_api_tier.so;
// not part of the shipped library.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>

#include "api_cases.cuh"
#include <xyz_autodiff/util/hip_managed_ptr.cuh>
#include "tester_suite.cuh"
#include "concept_checks.cuh"
#include "../../xyz_autodiff_cuda_amd/csrc/splat_staged.cuh"

using namespace xyz_autodiff;

namespace {

// ---- generic logic evaluation ---------------------------------------------
// in  = operand values, concatenated (plus trailing constants where the logic has any)
// up  = upstream gradient, one per output
// out = [outputs | analytic gradients | numerical gradients]; returns their total count
template <typename T, typename Logic, std::size_t In, std::size_t Out>
XAD_HD int eval_unary(const Logic& logic, const double* in, const double* up, double delta, double* out) {
    T x[In], g[Out], an[In], nu[In];
    for (std::size_t i = 0; i < In; ++i) x[i] = static_cast<T>(in[i]);
    for (std::size_t j = 0; j < Out; ++j) g[j] = static_cast<T>(up[j]);
    Variable<In, T> v(x);
    UnaryOperation<Out, Logic, Variable<In, T>> node(logic, v);
    node.forward();
    int n = 0;
    for (std::size_t j = 0; j < Out; ++j) out[n++] = node[j];
    testing::check_unary<Logic, In, Out, T>(logic, x, g, static_cast<T>(delta), an, nu);
    for (std::size_t i = 0; i < In; ++i) out[n++] = an[i];
    for (std::size_t i = 0; i < In; ++i) out[n++] = nu[i];
    return n;
}

template <typename T, typename Logic, std::size_t In1, std::size_t In2, std::size_t Out>
XAD_HD int eval_binary(const Logic& logic, const double* in, const double* up, double delta, double* out) {
    T a[In1], b[In2], g[Out], an[In1 + In2], nu[In1 + In2];
    for (std::size_t i = 0; i < In1; ++i) a[i] = static_cast<T>(in[i]);
    for (std::size_t i = 0; i < In2; ++i) b[i] = static_cast<T>(in[In1 + i]);
    for (std::size_t j = 0; j < Out; ++j) g[j] = static_cast<T>(up[j]);
    Variable<In1, T> va(a);
    Variable<In2, T> vb(b);
    BinaryOperation<Out, Logic, Variable<In1, T>, Variable<In2, T>> node(logic, va, vb);
    node.forward();
    int n = 0;
    for (std::size_t j = 0; j < Out; ++j) out[n++] = node[j];
    testing::check_binary<Logic, In1, In2, Out, T>(logic, a, b, g, static_cast<T>(delta), an, nu);
    for (std::size_t i = 0; i < In1 + In2; ++i) out[n++] = an[i];
    for (std::size_t i = 0; i < In1 + In2; ++i) out[n++] = nu[i];
    return n;
}

template <typename T>
XAD_HD int eval_logic(int logic, const double* in, const double* up, double delta, double* out) {
    using V1 = Variable<1, T>;
    using V2 = Variable<2, T>;
    using V3 = Variable<3, T>;
    using V4 = Variable<4, T>;
    using V6 = Variable<6, T>;
    using V9 = Variable<9, T>;
    switch (logic) {
        case 0: return eval_unary<T, op::ExpLogic<3>, 3, 3>({}, in, up, delta, out);
        case 1: return eval_unary<T, op::SinLogic<3>, 3, 3>({}, in, up, delta, out);
        case 2: return eval_unary<T, op::CosLogic<3>, 3, 3>({}, in, up, delta, out);
        case 3: return eval_unary<T, op::SigmoidLogic<3>, 3, 3>({}, in, up, delta, out);
        case 4: return eval_unary<T, op::NegLogic<3>, 3, 3>({}, in, up, delta, out);
        case 5: return eval_unary<T, op::SquaredLogic<3>, 3, 3>({}, in, up, delta, out);
        case 6: return eval_unary<T, op::SumLogic<4>, 4, 1>({}, in, up, delta, out);
        case 7: return eval_unary<T, op::L1NormLogic<4>, 4, 1>({}, in, up, delta, out);
        case 8: return eval_unary<T, op::L2NormLogic<4>, 4, 1>({}, in, up, delta, out);
        case 9: return eval_unary<T, op::AddConstantLogic<V3>, 3, 3>(op::AddConstantLogic<V3>(static_cast<T>(in[3])), in, up, delta, out);
        case 10: return eval_unary<T, op::SubConstantLogic<V3>, 3, 3>(op::SubConstantLogic<V3>(static_cast<T>(in[3])), in, up, delta, out);
        case 11: return eval_unary<T, op::MulConstantLogic<V3>, 3, 3>(op::MulConstantLogic<V3>(static_cast<T>(in[3])), in, up, delta, out);
        case 12: return eval_unary<T, op::DivConstantLogic<V3>, 3, 3>(op::DivConstantLogic<V3>(static_cast<T>(in[3])), in, up, delta, out);
        case 13:
        case 14: {
            ConstArray<T, 3> k;
            for (int i = 0; i < 3; ++i) k[i] = static_cast<T>(in[3 + i]);
            if (logic == 13) return eval_unary<T, op::ConstArrayAddLogic<3, ConstArray<T, 3>>, 3, 3>(op::ConstArrayAddLogic<3, ConstArray<T, 3>>(k), in, up, delta, out);
            return eval_unary<T, op::ConstArraySubLogic<3, ConstArray<T, 3>>, 3, 3>(op::ConstArraySubLogic<3, ConstArray<T, 3>>(k), in, up, delta, out);
        }
        case 15: return eval_unary<T, op::SymMatrix2InvLogic<3>, 3, 3>({}, in, up, delta, out);
        case 16: return eval_unary<T, op::QuaternionToRotationMatrixLogic<4>, 4, 9>({}, in, up, delta, out);
        case 17: return eval_unary<T, BroadcastLogic<4>, 1, 4>({}, in, up, delta, out);
        case 18: return eval_binary<T, op::AddLogic<V3, V3>, 3, 3, 3>({}, in, up, delta, out);
        case 19: return eval_binary<T, op::SubLogic<V3, V3>, 3, 3, 3>({}, in, up, delta, out);
        case 20: return eval_binary<T, op::MulLogic<V3, V3>, 3, 3, 3>({}, in, up, delta, out);
        case 21: return eval_binary<T, op::DivLogic<V3, V3>, 3, 3, 3>({}, in, up, delta, out);
        case 22: return eval_binary<T, op::MatMulLogic<2, 2, 2, V4, V4>, 4, 4, 4>({}, in, up, delta, out);
        case 23: return eval_binary<T, op::MatMulLogic<3, 3, 3, V9, V9>, 9, 9, 9>({}, in, up, delta, out);
        case 24: return eval_binary<T, op::MatMulLogic<2, 3, 1, V6, V3>, 6, 3, 2>({}, in, up, delta, out);  // matvec<2,3>
        case 25: return eval_binary<T, op::MatMulLogic<1, 3, 2, V3, V6>, 3, 6, 2>({}, in, up, delta, out);  // vecmat<3,2>
        case 26: return eval_binary<T, op::CovarianceMatrixGenerationLogic<V2, V1>, 2, 1, 4>({}, in, up, delta, out);
        case 27: return eval_unary<T, op::MatrixToCovariance3ParamLogic<V4>, 4, 3>({}, in, up, delta, out);
        case 28: return eval_binary<T, op::ScaleRotationToCovariance3ParamLogic<V2, V1>, 2, 1, 3>({}, in, up, delta, out);
        case 29: return eval_binary<T, op::MahalanobisDistanceLogic<V2, V3>, 2, 3, 1>({}, in, up, delta, out);
        case 30:
            return eval_binary<T, op::MahalanobisDistanceWithCenterLogic<V2, V3>, 2, 3, 1>(
                op::MahalanobisDistanceWithCenterLogic<V2, V3>(static_cast<T>(in[5]), static_cast<T>(in[6])), in, up, delta, out);
        // other operand sizes of the element-wise logics: tests/operation/base/test_gradient_verification.cu:14-39, :77-86
        case 31: return eval_unary<T, op::ExpLogic<1>, 1, 1>({}, in, up, delta, out);
        case 32: return eval_unary<T, op::ExpLogic<20>, 20, 20>({}, in, up, delta, out);
        case 33: return eval_unary<T, op::SigmoidLogic<1>, 1, 1>({}, in, up, delta, out);
        case 34: return eval_unary<T, op::SigmoidLogic<20>, 20, 20>({}, in, up, delta, out);
        case 35: return eval_binary<T, op::MulLogic<V1, V1>, 1, 1, 1>({}, in, up, delta, out);
        case 36: return eval_binary<T, op::MulLogic<Variable<5, T>, Variable<5, T>>, 5, 5, 5>({}, in, up, delta, out);
        case 37: return eval_binary<T, op::AddLogic<Variable<5, T>, Variable<5, T>>, 5, 5, 5>({}, in, up, delta, out);
        default: return -1;
    }
}

__global__ void case_kernel(int id, double* out, int* count) { *count = xad_test::run_case(id, out); }

__global__ void logic_kernel(int logic, int use_double, const double* in, const double* up, double delta, double* out, int* count) {
    *count = use_double ? eval_logic<double>(logic, in, up, delta, out) : eval_logic<float>(logic, in, up, delta, out);
}

// tests/test_parallel_gradient_accumulation.cu:25-49: every thread adds 1 to two shared
// gradients and (3 + 0.002 tid) to a third, through VariableRef::add_grad.
__global__ void parallel_accumulation_kernel(double* values, double* grads, std::size_t threads) {
    const std::size_t tid = static_cast<std::size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (tid >= threads) return;
    VariableRef<1, double> x(&values[0], &grads[0]), y(&values[1], &grads[1]), r(&values[2], &grads[2]);
    x.add_grad(0, 1.0);
    y.add_grad(0, 1.0);
    r.add_grad(0, (1.0 + tid * 0.001) + (2.0 + tid * 0.001));
}

// tests/test_shared_memory_atomic.cu:29-64 and :119-151: the same through LDS, per block.
__global__ void shared_accumulation_kernel(double* per_block) {
    __shared__ double x_data[1], x_grad[1], y_data[1], y_grad[1];
    if (threadIdx.x == 0) {
        x_data[0] = 5.0;
        x_grad[0] = 0.0;
        y_data[0] = 3.0;
        y_grad[0] = 0.0;
    }
    __syncthreads();
    VariableRef<1, double> x(x_data, x_grad), y(y_data, y_grad);
    x.add_grad(0, 1.0);
    y.add_grad(0, 2.0);
    __syncthreads();
    if (threadIdx.x == 0) {
        per_block[2 * blockIdx.x + 0] = x_grad[0];
        per_block[2 * blockIdx.x + 1] = y_grad[0];
    }
}

// VariableRef::add_grad from every thread on memory that the host can also reach (hipMallocManaged): the
// pairing the tests of xyz-autodiff-cuda use throughout (cuda_managed_ptr + VariableRef, e.g.
// tests/test_parallel_gradient_accumulation.cu:60-99).
template <typename T>
__global__ void managed_accumulation_kernel(T* values, T* grads, std::size_t threads) {
    const std::size_t tid = static_cast<std::size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (tid >= threads) return;
    VariableRef<2, T> v(values, grads);
    v.add_grad(0, T(1));
    v.add_grad(1, T(0.5) * v[1]);
}

bool ok(hipError_t e) { return e == hipSuccess; }

// The test that leaves a list entry out of a tile's compositing (csrc/splat_staged.cuh), on n (record, tile)
// pairs; fields: n x 6 floats (centre x, y; inverse covariance a, b, c; alpha0), tiles: n x 2 floats (the
// tile's first pixel).
XAD_HD int negligible_pair(const float* fields, const float* tiles, int i) {
    xad_splat::Record record{};
    record.cx = fields[6 * i];
    record.cy = fields[6 * i + 1];
    record.a = fields[6 * i + 2];
    record.b = fields[6 * i + 3];
    record.c = fields[6 * i + 4];
    record.alpha0 = fields[6 * i + 5];
    const xad_splat::Staged staged = xad_splat::stage_record(&record, 0);
    return xad_splat::negligible_in_tile(staged, tiles[2 * i], tiles[2 * i + 1]) ? 1 : 0;
}

__global__ void negligible_kernel(int n, const float* fields, const float* tiles, int* out) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = negligible_pair(fields, tiles, i);
}

template <typename T>
int managed_accumulation(std::size_t threads, double* out2) {
    auto values = makeHipManagedArray<T>(2);
    auto grads = makeHipManagedArray<T>(2);
    if (!values || !grads) return -2;
    values[0] = T(0);
    values[1] = T(4);  // written by the host, read by the device
    grads[0] = grads[1] = T(0);
    hipLaunchKernelGGL(managed_accumulation_kernel<T>, dim3(static_cast<unsigned>((threads + 255) / 256)), dim3(256), 0, 0,
                       values.get(), grads.get(), threads);
    if (!ok(hipGetLastError()) || !ok(hipDeviceSynchronize())) return -2;
    out2[0] = static_cast<double>(grads[0]);  // read by the host after the wait
    out2[1] = static_cast<double>(grads[1]);
    return 0;
}

}  // namespace

#ifndef XAD_TEST_SOURCE_DIGEST
#define XAD_TEST_SOURCE_DIGEST ""
#endif
extern "C" const char* xad_test_source_digest(void) { return XAD_TEST_SOURCE_DIGEST; }

// The gradient testers in this HIP translation unit: all cases of a tester call run in one kernel launch.
extern "C" int xad_test_tester_suite_device(char* text, std::size_t capacity, unsigned* self_checks) {
    return xad_suite::export_suite(text, capacity, self_checks);
}

extern "C" int xad_test_case_capacity(void) { return xad_test::kCaseCapacity; }

// side: 0 host, 1 device.  out: n ints, 1 where the entry would be left out.
extern "C" int xad_test_negligible_in_tile(int side, int n, const float* fields, const float* tiles, int* out) {
    if (side == 0) {
        for (int i = 0; i < n; ++i) out[i] = negligible_pair(fields, tiles, i);
        return 0;
    }
    float *d_fields = nullptr, *d_tiles = nullptr;
    int* d_out = nullptr;
    if (!ok(hipMalloc(&d_fields, sizeof(float) * 6 * n)) || !ok(hipMalloc(&d_tiles, sizeof(float) * 2 * n)) ||
        !ok(hipMalloc(&d_out, sizeof(int) * n)))
        return -2;
    (void)hipMemcpy(d_fields, fields, sizeof(float) * 6 * n, hipMemcpyHostToDevice);
    (void)hipMemcpy(d_tiles, tiles, sizeof(float) * 2 * n, hipMemcpyHostToDevice);
    hipLaunchKernelGGL(negligible_kernel, dim3((n + 255) / 256), dim3(256), 0, 0, n, d_fields, d_tiles, d_out);
    const int rc = ok(hipDeviceSynchronize()) && ok(hipMemcpy(out, d_out, sizeof(int) * n, hipMemcpyDeviceToHost)) ? 0 : -2;
    (void)hipFree(d_fields);
    (void)hipFree(d_tiles);
    (void)hipFree(d_out);
    return rc;
}

extern "C" int xad_test_run_case_host(int id, double* out) { return xad_test::run_case(id, out); }

extern "C" int xad_test_run_case_device(int id, double* out) {
    double* d_out = nullptr;
    int* d_count = nullptr;
    int count = -2;
    if (!ok(hipMalloc(&d_out, sizeof(double) * xad_test::kCaseCapacity)) || !ok(hipMalloc(&d_count, sizeof(int)))) return -2;
    (void)hipMemset(d_out, 0, sizeof(double) * xad_test::kCaseCapacity);
    hipLaunchKernelGGL(case_kernel, dim3(1), dim3(1), 0, 0, id, d_out, d_count);
    if (ok(hipDeviceSynchronize()) && ok(hipMemcpy(&count, d_count, sizeof(int), hipMemcpyDeviceToHost)))
        (void)hipMemcpy(out, d_out, sizeof(double) * xad_test::kCaseCapacity, hipMemcpyDeviceToHost);
    (void)hipFree(d_out);
    (void)hipFree(d_count);
    return count;
}

// side: 0 host, 1 device.  in: n_in doubles, up: n_up doubles, out: capacity 64.
extern "C" int xad_test_eval_logic(int side, int logic, int use_double, const double* in, int n_in, const double* up,
                                   int n_up, double delta, double* out) {
    if (side == 0) return use_double ? eval_logic<double>(logic, in, up, delta, out) : eval_logic<float>(logic, in, up, delta, out);
    double *d_in = nullptr, *d_up = nullptr, *d_out = nullptr;
    int* d_count = nullptr;
    int count = -2;
    if (!ok(hipMalloc(&d_in, sizeof(double) * (n_in + 1))) || !ok(hipMalloc(&d_up, sizeof(double) * (n_up + 1))) ||
        !ok(hipMalloc(&d_out, sizeof(double) * 64)) || !ok(hipMalloc(&d_count, sizeof(int))))
        return -2;
    (void)hipMemcpy(d_in, in, sizeof(double) * n_in, hipMemcpyHostToDevice);
    (void)hipMemcpy(d_up, up, sizeof(double) * n_up, hipMemcpyHostToDevice);
    hipLaunchKernelGGL(logic_kernel, dim3(1), dim3(1), 0, 0, logic, use_double, d_in, d_up, delta, d_out, d_count);
    if (ok(hipDeviceSynchronize()) && ok(hipMemcpy(&count, d_count, sizeof(int), hipMemcpyDeviceToHost)) && count > 0)
        (void)hipMemcpy(out, d_out, sizeof(double) * count, hipMemcpyDeviceToHost);
    (void)hipFree(d_in);
    (void)hipFree(d_up);
    (void)hipFree(d_out);
    (void)hipFree(d_count);
    return count;
}

extern "C" int xad_test_parallel_accumulation(std::size_t threads, int block, double* grads3) {
    double *d_values = nullptr, *d_grads = nullptr;
    if (!ok(hipMalloc(&d_values, 3 * sizeof(double))) || !ok(hipMalloc(&d_grads, 3 * sizeof(double)))) return -2;
    (void)hipMemset(d_values, 0, 3 * sizeof(double));
    (void)hipMemset(d_grads, 0, 3 * sizeof(double));
    hipLaunchKernelGGL(parallel_accumulation_kernel, dim3(static_cast<unsigned>((threads + block - 1) / block)), dim3(block), 0, 0,
                       d_values, d_grads, threads);
    const int rc = ok(hipDeviceSynchronize()) && ok(hipMemcpy(grads3, d_grads, 3 * sizeof(double), hipMemcpyDeviceToHost)) ? 0 : -2;
    (void)hipFree(d_values);
    (void)hipFree(d_grads);
    return rc;
}

// out4: the two gradients for float, then for double.
extern "C" int xad_test_managed_accumulation(std::size_t threads, double* out4) {
    if (int rc = managed_accumulation<float>(threads, out4)) return rc;
    return managed_accumulation<double>(threads, out4 + 2);
}

extern "C" int xad_test_shared_accumulation(int blocks, int threads, double* per_block) {
    double* d = nullptr;
    if (!ok(hipMalloc(&d, sizeof(double) * 2 * blocks))) return -2;
    hipLaunchKernelGGL(shared_accumulation_kernel, dim3(blocks), dim3(threads), 0, 0, d);
    const int rc = ok(hipDeviceSynchronize()) && ok(hipMemcpy(per_block, d, sizeof(double) * 2 * blocks, hipMemcpyDeviceToHost)) ? 0 : -2;
    (void)hipFree(d);
    return rc;
}

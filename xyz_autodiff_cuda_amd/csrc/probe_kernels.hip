// Hardware probe: cost of LDS atomic adds by element type and address pattern.
// The accumulator's choice of an fp64 LDS table rests on these numbers, so the
// measurement ships with the library and can be repeated on any device.
#include <vector>

#include "common.cuh"

namespace {

constexpr int kWaves = 16;
constexpr int kBlocks = 256;

template <typename T>
__global__ void __launch_bounds__(kWaves * 64) lds_atomic_probe_kernel(int pattern, int iterations, T* sink,
                                                                       long long* cycles) {
    __shared__ T table[4096];
    for (int i = threadIdx.x; i < 4096; i += blockDim.x) table[i] = T(0);
    __syncthreads();
    const int lane = threadIdx.x & 63;
    int at;
    switch (pattern) {
        case 0: at = lane; break;                   // 64 distinct consecutive addresses
        case 1: at = 0; break;                      // all lanes one address
        case 2: at = lane < 16 ? 0 : lane; break;   // 16 lanes share an address
        case 3: at = lane & 7; break;               // eight lanes per address
        default: at = lane * 6; break;              // stride of six elements
    }
    T v = T(1) + T(lane);
    const long long t0 = clock64();
    for (int i = 0; i < iterations; ++i) {
        atomicAdd(&table[at], v);
        v += T(1);
    }
    __syncthreads();
    const long long t1 = clock64();
    if (threadIdx.x == 0) cycles[blockIdx.x] = t1 - t0;
    if (threadIdx.x < 64) sink[blockIdx.x * 64 + threadIdx.x] = table[threadIdx.x];
}

template <typename T>
int run_probe(int pattern, double* cycles_per_instruction) {
    const int iterations = 1000;
    T* sink = nullptr;
    long long* cycles = nullptr;
    XAD_HIP_TRY(hipMalloc(&sink, sizeof(T) * kBlocks * 64));
    hipError_t st = hipMalloc(&cycles, sizeof(long long) * kBlocks);
    std::vector<long long> host(kBlocks);
    if (st == hipSuccess) {
        for (int rep = 0; rep < 2; ++rep)  // the second launch is the measurement
            hipLaunchKernelGGL(lds_atomic_probe_kernel<T>, dim3(kBlocks), dim3(kWaves * 64), 0, nullptr, pattern, iterations, sink,
                               cycles);
        st = hipDeviceSynchronize();
    }
    if (st == hipSuccess) st = hipMemcpy(host.data(), cycles, sizeof(long long) * kBlocks, hipMemcpyDeviceToHost);
    (void)hipFree(sink);
    (void)hipFree(cycles);
    if (st != hipSuccess) return xad::fail(XAD_ERR_HIP, "xad_probe_lds_atomic_cycles: %s", hipGetErrorString(st));
    double total = 0.0;
    for (long long c : host) total += static_cast<double>(c);
    // 16 wavefronts share one LDS pipeline: cycles the pipeline spends per wavefront instruction
    *cycles_per_instruction = total / kBlocks / iterations / kWaves;
    return XAD_OK;
}

}  // namespace

extern "C" int xad_probe_lds_atomic_cycles(int element, int pattern, double* cycles_per_instruction) {
    XAD_REQUIRE(cycles_per_instruction, "xad_probe_lds_atomic_cycles: output is null");
    XAD_REQUIRE(pattern >= 0 && pattern <= 4, "xad_probe_lds_atomic_cycles: pattern must be 0..4, got %d", pattern);
    switch (element) {
        case 0: return run_probe<float>(pattern, cycles_per_instruction);
        case 1: return run_probe<double>(pattern, cycles_per_instruction);
        case 2: return run_probe<unsigned int>(pattern, cycles_per_instruction);
        case 3: return run_probe<unsigned long long>(pattern, cycles_per_instruction);
        default: return xad::fail(XAD_ERR_INVALID_ARGUMENT, "xad_probe_lds_atomic_cycles: element must be 0..3, got %d", element);
    }
}

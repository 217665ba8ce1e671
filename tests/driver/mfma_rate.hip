// Sustained rate of back-to-back v_mfma_f32_32x32x16_f16 on the whole GPU as a function of the operand data.
// Test / measurement infrastructure: no memory traffic, 2 waves per SIMD, 4 independent accumulators per wave, i.e. the
// MFMA pipe is the only busy unit.  The rate depends on the data: with changing, random operands the power management
// of the MI355X lowers the clock well below what zero or constant operands run at, so the number printed for "random"
// is the ceiling a real attention kernel can approach, whatever its schedule.
// Prints one JSON line: {"zeros": T, "constant": T, "random": T} in TFLOP/s (best of 5 launches each).
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

#define HIP_CHECK(call)                                                                          \
    do {                                                                                         \
        hipError_t e_ = (call);                                                                  \
        if (e_ != hipSuccess) {                                                                  \
            std::fprintf(stderr, "HIP error: %s at line %d\n", hipGetErrorString(e_), __LINE__); \
            std::exit(1);                                                                        \
        }                                                                                        \
    } while (0)

// MODE 0: zeros; 1: one constant fragment pair; 2: 8 random A and 8 random B fragments per lane, cycled
template <int MODE>
__global__ void __launch_bounds__(256) mfma_loop(float* out, int iters)
{
    v8h a[8], b[8];
    unsigned s = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
    auto rnd = [&]() {
        s = s * 1664525u + 1013904223u;
        return ((int)((s >> 8) & 0xffff) - 32768) / 32768.0f;
    };
    for (int f = 0; f < 8; ++f)
        for (int e = 0; e < 8; ++e) {
            if (MODE == 0) {
                a[f][e] = 0;
                b[f][e] = 0;
            } else if (MODE == 1) {
                a[f][e] = (_Float16)(0.5f + 0.1f * e);
                b[f][e] = (_Float16)(0.25f * e);
            } else {
                a[f][e] = (_Float16)(rnd() * 2.0f);
                b[f][e] = (_Float16)(rnd() * 2.0f);
            }
        }
    v16f acc[4];
    for (int n = 0; n < 4; ++n)
        for (int r = 0; r < 16; ++r) acc[n][r] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int f = 0; f < 8; ++f)
#pragma unroll
            for (int n = 0; n < 4; ++n)
                acc[n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[(f + n) & 7], b[f], acc[n], 0, 0, 0);
    }
    float r_ = 0;
    for (int n = 0; n < 4; ++n)
        for (int r = 0; r < 16; ++r) r_ += acc[n][r];
    out[blockIdx.x * blockDim.x + threadIdx.x] = r_;
}

template <typename K>
double best_tflops(K kern, float* out, int n_cu)
{
    const int iters = 6000, grid = 2 * n_cu;  // 4 waves per work-group, 2 work-groups per CU
    hipLaunchKernelGGL(kern, grid, 256, 0, 0, out, 10);
    HIP_CHECK(hipDeviceSynchronize());
    hipEvent_t e0, e1;
    HIP_CHECK(hipEventCreate(&e0));
    HIP_CHECK(hipEventCreate(&e1));
    double best = 0;
    for (int rep = 0; rep < 5; ++rep) {
        HIP_CHECK(hipEventRecord(e0, 0));
        hipLaunchKernelGGL(kern, grid, 256, 0, 0, out, iters);
        HIP_CHECK(hipEventRecord(e1, 0));
        HIP_CHECK(hipEventSynchronize(e1));
        float ms;
        HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
        const double n_mfma = (double)grid * 4 * iters * 32;
        const double t = n_mfma * 32768.0 / ms / 1e9;
        if (t > best) best = t;
    }
    return best;
}

int main()
{
    hipDeviceProp_t prop;
    HIP_CHECK(hipGetDeviceProperties(&prop, 0));
    const int n_cu = prop.multiProcessorCount;
    float* out;
    HIP_CHECK(hipMalloc(&out, (size_t)2 * n_cu * 256 * sizeof(float)));
    const double z = best_tflops(mfma_loop<0>, out, n_cu);
    const double c = best_tflops(mfma_loop<1>, out, n_cu);
    const double r = best_tflops(mfma_loop<2>, out, n_cu);
    std::printf("{\"zeros\": %.1f, \"constant\": %.1f, \"random\": %.1f, \"unit\": \"TFLOP/s\", \"cus\": %d}\n", z, c, r, n_cu);
    HIP_CHECK(hipFree(out));
    return 0;
}

// Sustained rate of back-to-back v_mfma_f32_32x32x16_f16 on the whole GPU as a function of the operand data.
// Test / measurement infrastructure: no memory traffic, 2 waves per SIMD, 4 independent accumulators per wave, i.e. the
// MFMA pipe is the only busy unit.  The rate depends on the data: with changing, random operands the power management
// of the MI355X lowers the clock well below what zero or constant operands run at, so the number printed for "random"
// is the ceiling a real attention kernel can approach, whatever its schedule.
// Further figures relate that ceiling to the instruction mix of an attention loop at head dim 128 (8 waves per CU unless
// stated, no global memory traffic, no barriers, no masks; everything beside an MFMA is independent of it and of each
// other, so each figure is the ceiling of its mix, whatever the schedule):
//   random_mfma_lds             every MFMA is followed by the re-read of its A fragment from LDS (half of them
//                               ds_read_b128 as for K, half pairs of ds_read_b64_tr_b16 as for V): 32 query rows per wave
//   random_attention_mix        the same plus four fp32 fma/add and one v_exp_f32 per MFMA (the softmax of those scores)
//   random_attention_mix_64rows one wave per SIMD with 64 query rows: every fragment read feeds two MFMAs (two B operands,
//                               eight accumulators), the same four fma/add and one exp per MFMA
//   zeros_attention_mix, zeros_attention_mix_64rows: the last two on all-zero MFMA operands
// Prints one JSON line with these keys beside "zeros", "constant", "random", in TFLOP/s (best of 5 launches each).
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

// The MFMA stream of mfma_loop<2> with the companions of an attention loop (see the head of the file).  One work-group
// per CU: 8 waves with one MFMA per fragment read, or (k64Rows) 4 waves with two; 64 KiB of LDS hold four stages of
// random (kZero: zero) fp16 data that the fragment reads walk through.  kValu: the fma/add and exp companions are issued.
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef __fp16 v4hp __attribute__((__vector_size__(4 * sizeof(__fp16))));
#define LDS_AS __attribute__((address_space(3)))
template <bool k64Rows, bool kValu, bool kZero>
__global__ void __launch_bounds__(k64Rows ? 256 : 512) attention_mix_loop(float* out, int iters)
{
    constexpr int NB = k64Rows ? 2 : 1;  // MFMAs per fragment read
    extern __shared__ __attribute__((aligned(16))) char smem[];
    LDS_AS char* lds = (LDS_AS char*)smem;
    const int tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, g = lane >> 5;
    unsigned s = tid * 2654435761u + blockIdx.x * 40503u + 12345u;
    auto rnd2 = [&]() {  // two fp16 values of magnitude 0.125 .. 2 with random sign and mantissa
        auto h = [](unsigned x) { return (x & 0x8000u) | ((12u + ((x >> 10) & 3u)) << 10) | (x & 0x3ffu); };
        s = s * 1664525u + 1013904223u;
        const unsigned lo = s >> 16;
        s = s * 1664525u + 1013904223u;
        return kZero ? 0u : h(lo) | (h(s >> 16) << 16);
    };
    for (int i = tid; i < 16384; i += blockDim.x) ((LDS_AS unsigned*)lds)[i] = rnd2();
    __syncthreads();
    // lane parts of conflict-free fragment addresses in a row-major 64 x 128 fp16 tile with permuted 16-byte chunks
    const int k_rd = l32 * 256 + ((g ^ (l32 & 1)) << 4) + (((l32 & 15) >> 1) << 5);
    const int G = lane >> 4, e4 = (lane >> 2) & 3, j4 = lane & 3;
    const int v_rd = (4 * (G >> 1) + e4) * 256 + (((G & 1) ^ (G >> 1)) << 5) + 8 * j4 + (e4 << 6);
    union Frag { v4u u; v8h h; v4hp p[2]; };
    Frag fr[16], bq[NB];
    for (int i = 0; i < 16; ++i) fr[i].u = v4u{rnd2(), rnd2(), rnd2(), rnd2()};
    for (int i = 0; i < NB; ++i) bq[i].u = v4u{rnd2(), rnd2(), rnd2(), rnd2()};
    v16f acc[4 * NB];
    for (int n = 0; n < 4 * NB; ++n)
        for (int r = 0; r < 16; ++r) acc[n][r] = 0.f;
    float vr[8];
    for (int i = 0; i < 8; ++i) vr[i] = tid * 1e-3f + i;
    const float c1 = 0.999f, c0 = 0.01f;
    for (int it = 0; it < iters; ++it) {
        unsigned kb = (unsigned)k_rd + (it & 3) * 16384, vb = (unsigned)v_rd + (it & 3) * 16384;
        asm volatile("" : "+v"(kb), "+v"(vb));
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            // the fragment consumed here was requested one iteration ago; its refill is issued right behind the MFMAs
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                acc[NB * (u & 3) + nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fr[u].h, bq[nb].h, acc[NB * (u & 3) + nb], 0, 0, 0);
                if (kValu) {
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(vr[((NB * u + nb) * 4 + v) & 7]) : "v"(c1), "v"(c0));
                    asm volatile("v_exp_f32 %0, %0" : "+v"(vr[(NB * u + nb + 3) & 7]));
                }
            }
            if (u < 8) {
                fr[u].u = *(LDS_AS const v4u*)(lds + (kb ^ (unsigned)((u & 7) << 5)) + (u >> 3) * 8192);
            } else {
                LDS_AS char* p = lds + (vb ^ (unsigned)((u & 3) << 6)) + (u >> 2) * 4096;
                fr[u].p[0] = __builtin_amdgcn_ds_read_tr16_b64_v4f16((LDS_AS v4hp*)p);
                fr[u].p[1] = __builtin_amdgcn_ds_read_tr16_b64_v4f16((LDS_AS v4hp*)(p + 2048));
            }
        }
    }
    float r_ = 0;
    for (int n = 0; n < 4 * NB; ++n)
        for (int r = 0; r < 16; ++r) r_ += acc[n][r];
    for (int i = 0; i < 8; ++i) r_ += vr[i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = r_;
}

template <bool k64Rows, bool kValu, bool kZero>
double best_mix_tflops(float* out, int n_cu)
{
    const int iters = 12000, lds_bytes = 65536, threads = k64Rows ? 256 : 512;
    auto kern = attention_mix_loop<k64Rows, kValu, kZero>;
    HIP_CHECK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes));
    hipLaunchKernelGGL(kern, n_cu, threads, lds_bytes, 0, out, 10);
    HIP_CHECK(hipDeviceSynchronize());
    hipEvent_t e0, e1;
    HIP_CHECK(hipEventCreate(&e0));
    HIP_CHECK(hipEventCreate(&e1));
    double best = 0;
    for (int rep = 0; rep < 5; ++rep) {
        HIP_CHECK(hipEventRecord(e0, 0));
        hipLaunchKernelGGL(kern, n_cu, threads, lds_bytes, 0, out, iters);
        HIP_CHECK(hipEventRecord(e1, 0));
        HIP_CHECK(hipEventSynchronize(e1));
        float ms;
        HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
        // every wave issues 16 MFMAs per iteration and B operand
        const double t = (double)n_cu * (threads / 64) * iters * 16 * (k64Rows ? 2 : 1) * 32768.0 / ms / 1e9;
        if (t > best) best = t;
    }
    HIP_CHECK(hipEventDestroy(e0));
    HIP_CHECK(hipEventDestroy(e1));
    return best;
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
    const double ml = best_mix_tflops<false, false, false>(out, n_cu);
    const double m = best_mix_tflops<false, true, false>(out, n_cu);
    const double m64 = best_mix_tflops<true, true, false>(out, n_cu);
    const double mz = best_mix_tflops<false, true, true>(out, n_cu);
    const double m64z = best_mix_tflops<true, true, true>(out, n_cu);
    std::printf("{\"zeros\": %.1f, \"constant\": %.1f, \"random\": %.1f, \"random_mfma_lds\": %.1f, \"random_attention_mix\": %.1f, "
                "\"random_attention_mix_64rows\": %.1f, \"zeros_attention_mix\": %.1f, \"zeros_attention_mix_64rows\": %.1f, "
                "\"unit\": \"TFLOP/s\", \"cus\": %d}\n",
                z, c, r, ml, m, m64, mz, m64z, n_cu);
    HIP_CHECK(hipFree(out));
    return 0;
}

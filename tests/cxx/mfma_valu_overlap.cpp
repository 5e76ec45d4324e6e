// A premise of the matrix-product and attention kernels, as a measurement: on this GPU, FP32 MFMAs and FP32 vector
// instructions do not overlap -- neither between the two wavefronts that share a SIMD nor within one wavefront -- so
// every vector instruction inside an MFMA loop is paid in matrix time.
//
// A block is 8 wavefronts; wavefronts w and w + 4 share a SIMD.  Four timed runs of the same kernel, 256 blocks each:
//   mfma    wavefronts 0-3 issue 64 independent 16x16x4 MFMAs per iteration, wavefronts 4-7 idle
//   valu    wavefronts 4-7 issue 512 FP32 multiply-adds per iteration (eight independent chains), wavefronts 0-3 idle
//   both    the two at once, on the same SIMDs
//   mixed   wavefronts 0-3 issue both kinds, interleaved, independent of one another
// Prints the four durations in microseconds: "mfma <t> valu <t> both <t> mixed <t>".  With overlap, `both` would be
// near max(mfma, valu); without it, near their sum.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#define CK(x)                                                                  \
    do {                                                                       \
        hipError_t e_ = (x);                                                   \
        if (e_ != hipSuccess) {                                                \
            printf("%s failed: %s\n", #x, hipGetErrorString(e_));              \
            exit(1);                                                           \
        }                                                                      \
    } while (0)

typedef float float4_t __attribute__((ext_vector_type(4)));

enum { A_MFMA = 1, B_VALU = 2, A_MIXED = 4 };

__global__ __launch_bounds__(512) void overlap_kernel(float* out, int iters, int mode) {
    const unsigned wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const bool first_four = wave < 4;
    float4_t acc[8];
    for (int i = 0; i < 8; ++i) acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    float v[8];
    for (int i = 0; i < 8; ++i) v[i] = (float)lane * 0.001f + i;
    const float a = (float)lane, b = 1.0f / (1 + lane);
    if (first_four && (mode & A_MFMA)) {
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
#pragma unroll
                for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc[i], 0, 0, 0);
        }
    }
    if (!first_four && (mode & B_VALU)) {
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int r = 0; r < 64; ++r)
#pragma unroll
                for (int i = 0; i < 8; ++i) v[i] = v[i] * 1.0001f + 0.5f;
        }
    }
    if (first_four && (mode & A_MIXED)) {
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc[i], 0, 0, 0);
#pragma unroll
                    for (int q = 0; q < 8; ++q) v[(i + q) & 7] = v[(i + q) & 7] * 1.0001f + 0.5f;
                }
        }
    }
    float s = 0;
    for (int i = 0; i < 8; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3] + v[i];
    if (s == 1.2345f) out[threadIdx.x] = s;   // never true: keeps the arithmetic alive
}

int main() {
    float* out;
    CK(hipMalloc(&out, 4096));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    const int iters = 2000;
    const int modes[4] = {A_MFMA, B_VALU, A_MFMA | B_VALU, A_MIXED};
    const char* names[4] = {"mfma", "valu", "both", "mixed"};
    for (int m = 0; m < 4; ++m) {
        float best = 1e30f;
        for (int rep = 0; rep < 3; ++rep) {
            CK(hipEventRecord(e0));
            hipLaunchKernelGGL(overlap_kernel, dim3(256), dim3(512), 0, 0, out, iters, modes[m]);
            CK(hipEventRecord(e1));
            CK(hipEventSynchronize(e1));
            float ms;
            CK(hipEventElapsedTime(&ms, e0, e1));
            if (rep && ms < best) best = ms;
        }
        printf("%s %.1f%s", names[m], best * 1000, m == 3 ? "\n" : " ");
    }
    CK(hipFree(out));
    return 0;
}

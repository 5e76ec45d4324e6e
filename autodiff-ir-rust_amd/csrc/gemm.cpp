// FP32 matrix product for gfx950 on the matrix cores (v_mfma_f32_32x32x2_f32), LDS-tiled.
//
// The reference multiplies with one work-item per output element, a sequential k loop and two
// global loads per multiply-add (reference src/devices/opencl/kernels/dotprod.rs:23-53); transposed
// operands are folded into its index expressions.  Here both operands are described by strides
// (so x^T and W^T of the backward pass need no copy), staged through LDS in 128x128x16 tiles with
// register prefetch of the next tile, and each of the four wavefronts of a block owns a 64x64
// sub-tile = 2x2 MFMA blocks of 32x32.
#include "gemm.hpp"

#include "common.hpp"

namespace adhip {

std::string gemm_kernel_source(const GemmConfig& cfg, const std::string& entry) {
    std::string s;
    s += strf("#define A_KCONTIG %d\n#define B_KCONTIG %d\n#define EDGE %d\n", cfg.a_kcontig ? 1 : 0, cfg.b_kcontig ? 1 : 0,
              cfg.edge ? 1 : 0);
    s += strf("#define KERNEL_NAME %s\n", entry.c_str());
    s += R"(
#define BM 128
#define BN 128
#define BK 16
#define LDA (BM + 4)
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

// A is [M,K] with element strides (a_sm, a_sk); B is [K,N] with (b_sk, b_sn); C dense [M,N].
// A_KCONTIG: a_sk == 1 (else a_sm == 1).  B_KCONTIG: b_sk == 1 (else b_sn == 1).
// EDGE: M, N or K is not a multiple of the tile, or an operand is not 16-byte aligned; every
// access is then bounds-checked and scalar.
extern "C" __global__ __launch_bounds__(256) void KERNEL_NAME(
    const int* __restrict__ guard, float* __restrict__ C, const float* __restrict__ A, const float* __restrict__ B,
    long long M, long long N, long long K, long long a_off, long long a_sm, long long a_sk, long long b_off,
    long long b_sk, long long b_sn) {
    if (guard && *guard == 0) return;
    __shared__ __attribute__((aligned(16))) float As[2][BK][LDA];
    __shared__ __attribute__((aligned(16))) float Bs[2][BK][LDA];

    const unsigned tid = threadIdx.x;
    const unsigned lane = tid & 63u, wave = tid >> 6;
    const unsigned wm = wave >> 1, wn = wave & 1u;
    const unsigned li = lane & 31u, lh = lane >> 5;

    // Block -> tile.  Consecutive block ids go to different XCDs (8 of them, each with its own L2), so
    // ids are first regrouped per XCD and then walked in column-major groups of 8 tile rows, which
    // keeps the A and B panels one XCD works on small.
    const unsigned gm = (unsigned)((M + BM - 1) / BM), gn = (unsigned)((N + BN - 1) / BN);
    const unsigned nblk = gm * gn;
    unsigned pid = blockIdx.x;
    if ((nblk & 7u) == 0) pid = (pid & 7u) * (nblk >> 3) + (pid >> 3);
    const unsigned GROUP = 8;
    const unsigned per_group = GROUP * gn;
    const unsigned group = pid / per_group;
    const unsigned first_m = group * GROUP;
    const unsigned gsz = min(gm - first_m, GROUP);
    const unsigned tile_m = first_m + (pid % per_group) % gsz;
    const unsigned tile_n = (pid % per_group) / gsz;
    const long long bm = (long long)tile_m * BM, bn = (long long)tile_n * BN;

    A += a_off;
    B += b_off;

    float16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    float4_t ra[2], rb[2];

    auto load_a = [&](long long k0) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#if A_KCONTIG
            const unsigned kq = tid & 3u, mr = (tid >> 2) + 64u * i;
            const long long m = bm + mr, k = k0 + 4 * kq;
#if EDGE
            float4_t v = {0.f, 0.f, 0.f, 0.f};
            if (m < M) {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (k + j < K) v[j] = A[m * a_sm + (k + j) * a_sk];
            }
            ra[i] = v;
#else
            ra[i] = *(const float4_t*)(A + m * a_sm + k);
#endif
#else
            const unsigned mq = tid & 31u, kr = (tid >> 5) + 8u * i;
            const long long m = bm + 4 * mq, k = k0 + kr;
#if EDGE
            float4_t v = {0.f, 0.f, 0.f, 0.f};
            if (k < K) {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (m + j < M) v[j] = A[(m + j) * a_sm + k * a_sk];
            }
            ra[i] = v;
#else
            ra[i] = *(const float4_t*)(A + k * a_sk + m);
#endif
#endif
        }
    };
    auto load_b = [&](long long k0) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#if B_KCONTIG
            const unsigned kq = tid & 3u, nr = (tid >> 2) + 64u * i;
            const long long n = bn + nr, k = k0 + 4 * kq;
#if EDGE
            float4_t v = {0.f, 0.f, 0.f, 0.f};
            if (n < N) {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (k + j < K) v[j] = B[(k + j) * b_sk + n * b_sn];
            }
            rb[i] = v;
#else
            rb[i] = *(const float4_t*)(B + n * b_sn + k);
#endif
#else
            const unsigned nq = tid & 31u, kr = (tid >> 5) + 8u * i;
            const long long n = bn + 4 * nq, k = k0 + kr;
#if EDGE
            float4_t v = {0.f, 0.f, 0.f, 0.f};
            if (k < K) {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (n + j < N) v[j] = B[k * b_sk + (n + j) * b_sn];
            }
            rb[i] = v;
#else
            rb[i] = *(const float4_t*)(B + k * b_sk + n);
#endif
#endif
        }
    };
    auto store_tiles = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#if A_KCONTIG
            {
                const unsigned kq = tid & 3u, mr = (tid >> 2) + 64u * i;
#pragma unroll
                for (int j = 0; j < 4; ++j) As[buf][4 * kq + j][mr] = ra[i][j];
            }
#else
            {
                const unsigned mq = tid & 31u, kr = (tid >> 5) + 8u * i;
                *(float4_t*)&As[buf][kr][4 * mq] = ra[i];
            }
#endif
#if B_KCONTIG
            {
                const unsigned kq = tid & 3u, nr = (tid >> 2) + 64u * i;
#pragma unroll
                for (int j = 0; j < 4; ++j) Bs[buf][4 * kq + j][nr] = rb[i][j];
            }
#else
            {
                const unsigned nq = tid & 31u, kr = (tid >> 5) + 8u * i;
                *(float4_t*)&Bs[buf][kr][4 * nq] = rb[i];
            }
#endif
        }
    };

    const long long KT = (K + BK - 1) / BK;
    load_a(0);
    load_b(0);
    store_tiles(0);
    __syncthreads();

    for (long long kt = 0; kt < KT; ++kt) {
        const int cur = (int)(kt & 1);
        const bool more = kt + 1 < KT;
        if (more) {
            load_a((kt + 1) * BK);
            load_b((kt + 1) * BK);
        }
#pragma unroll
        for (int ks = 0; ks < BK / 2; ++ks) {
            const float a0 = As[cur][2 * ks + lh][wm * 64 + li];
            const float a1 = As[cur][2 * ks + lh][wm * 64 + 32 + li];
            const float b0 = Bs[cur][2 * ks + lh][wn * 64 + li];
            const float b1 = Bs[cur][2 * ks + lh][wn * 64 + 32 + li];
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
        }
        if (more) store_tiles(cur ^ 1);
        __syncthreads();
    }

    // acc[i][j][4g + r] holds C[row = 32i + 8g + 4*lh + r][col = 32j + li] of the wave's 64x64 tile
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const long long row = bm + wm * 64 + 32 * i + 8 * g + 4 * lh + r;
                    const long long col = bn + wn * 64 + 32 * j + li;
#if EDGE
                    if (row < M && col < N)
#endif
                        C[row * N + col] = acc[i][j][4 * g + r];
                }
}
)";
    return s;
}

}  // namespace adhip

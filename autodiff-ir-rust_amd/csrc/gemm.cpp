// FP32 matrix product for gfx950 on the matrix cores (v_mfma_f32_32x32x2_f32), LDS-tiled.
//
// The reference multiplies with one work-item per output element, a sequential k loop and two
// global loads per multiply-add (reference src/devices/opencl/kernels/dotprod.rs:23-53); transposed
// operands are folded into its index expressions.  Here both operands are described by strides
// (so x^T and W^T of the backward pass need no copy), staged through LDS in 128x128x16 or 256x128x16
// tiles with register prefetch of the next tile, and each of the four (eight) wavefronts of a block
// owns a 64x64 sub-tile = 2x2 MFMA blocks of 32x32.
#include "gemm.hpp"

#include "common.hpp"

namespace adhip {

std::string gemm_kernel_source(const GemmConfig& cfg, const std::string& entry, const GemmEpilogue* epilogue) {
    std::string s;
    if (epilogue) s += epilogue->prelude;
    s += strf("#define STORE_C %d\n#define EPI_PARAMS %s\n", (!epilogue || epilogue->store_c) ? 1 : 0,
              epilogue ? epilogue->params.c_str() : "");
    {
        // the epilogue statements become one macro (line continuations), expanded where an element is finished
        std::string body = epilogue ? epilogue->code : std::string();
        std::string m = "#define EPILOGUE";
        size_t pos = 0;
        while (pos < body.size()) {
            size_t nl = body.find('\n', pos);
            if (nl == std::string::npos) nl = body.size();
            m += " \\\n    " + body.substr(pos, nl - pos);
            pos = nl + 1;
        }
        s += m + "\n";
    }
    s += strf("#define A_KCONTIG %d\n#define B_KCONTIG %d\n#define EDGE %d\n", cfg.a_kcontig ? 1 : 0, cfg.b_kcontig ? 1 : 0,
              cfg.edge ? 1 : 0);
    s += strf("#define KERNEL_NAME %s\n#define BM %d\n", entry.c_str(), cfg.bm);
    s += R"(
#define BN 128
#define BK 16
#define LDA (BM + 4)
#define LDB (BN + 4)
#define NT (BM * 2)            /* threads: one wave per 64x64 sub-tile */
#define B_LOADS (512 / NT)     /* float4 loads of the B tile per thread */
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

// A is [M,K] with element strides (a_sm, a_sk); B is [K,N] with (b_sk, b_sn); C dense [M,N].
// A_KCONTIG: a_sk == 1 (else a_sm == 1).  B_KCONTIG: b_sk == 1 (else b_sn == 1).
// EDGE: M, N or K is not a multiple of the tile, or an operand is not 16-byte aligned; every
// access is then bounds-checked and scalar.
extern "C" __global__ __launch_bounds__(NT) void KERNEL_NAME(
    const int* __restrict__ guard, float* __restrict__ C, const float* __restrict__ A, const float* __restrict__ B,
    long long M, long long N, long long K, long long a_off, long long a_sm, long long a_sk, long long b_off,
    long long b_sk, long long b_sn EPI_PARAMS) {
    if (guard && *guard == 0) return;
    __shared__ __attribute__((aligned(16))) float As[2][BK][LDA];
    __shared__ __attribute__((aligned(16))) float Bs[2][BK][LDB];

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

    float4_t ra0[2], rb0[B_LOADS];

    auto load_a = [&](long long k0, float4_t* ra) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#if A_KCONTIG
            const unsigned kq = tid & 3u, mr = (tid >> 2) + (NT / 4) * i;
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
            const unsigned mq = tid % (BM / 4), kr = tid / (BM / 4) + 8u * i;
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
    auto load_b = [&](long long k0, float4_t* rb) {
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i) {
#if B_KCONTIG
            const unsigned kq = tid & 3u, nr = (tid >> 2) + (NT / 4) * i;
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
            const unsigned nq = tid & 31u, kr = (tid >> 5) + (NT / 32) * i;
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
    auto store_tiles = [&](int buf, const float4_t* ra, const float4_t* rb) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#if A_KCONTIG
            const unsigned kq = tid & 3u, mr = (tid >> 2) + (NT / 4) * i;
#pragma unroll
            for (int j = 0; j < 4; ++j) As[buf][4 * kq + j][mr] = ra[i][j];
#else
            const unsigned mq = tid % (BM / 4), kr = tid / (BM / 4) + 8u * i;
            *(float4_t*)&As[buf][kr][4 * mq] = ra[i];
#endif
        }
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i) {
#if B_KCONTIG
            const unsigned kq = tid & 3u, nr = (tid >> 2) + (NT / 4) * i;
#pragma unroll
            for (int j = 0; j < 4; ++j) Bs[buf][4 * kq + j][nr] = rb[i][j];
#else
            const unsigned nq = tid & 31u, kr = (tid >> 5) + (NT / 32) * i;
            *(float4_t*)&Bs[buf][kr][4 * nq] = rb[i];
#endif
        }
    };

    // One k-tile: 8 MFMA steps from LDS buffer `cur`; the operands of step ks+1 are fetched from LDS before the
    // four MFMAs of step ks are issued, and half way through the tile that was prefetched into registers (sa, sb)
    // is parked in the other LDS buffer, which nobody reads during this iteration.
    auto compute = [&](int cur, bool park, const float4_t* sa, const float4_t* sb) {
        float fa0[2], fa1[2], fb0[2], fb1[2];
        fa0[0] = As[cur][lh][wm * 64 + li];
        fa1[0] = As[cur][lh][wm * 64 + 32 + li];
        fb0[0] = Bs[cur][lh][wn * 64 + li];
        fb1[0] = Bs[cur][lh][wn * 64 + 32 + li];
#pragma unroll
        for (int ks = 0; ks < BK / 2; ++ks) {
            const int c = ks & 1, nx = c ^ 1;
            if (ks + 1 < BK / 2) {
                fa0[nx] = As[cur][2 * (ks + 1) + lh][wm * 64 + li];
                fa1[nx] = As[cur][2 * (ks + 1) + lh][wm * 64 + 32 + li];
                fb0[nx] = Bs[cur][2 * (ks + 1) + lh][wn * 64 + li];
                fb1[nx] = Bs[cur][2 * (ks + 1) + lh][wn * 64 + 32 + li];
            }
            __builtin_amdgcn_sched_barrier(0);  // keep the LDS reads ahead of the MFMAs that hide their latency
            acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa0[c], fb0[c], acc[0][0], 0, 0, 0);
            acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa0[c], fb1[c], acc[0][1], 0, 0, 0);
            acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa1[c], fb0[c], acc[1][0], 0, 0, 0);
            acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa1[c], fb1[c], acc[1][1], 0, 0, 0);
            if (ks == BK / 4 - 1 && park) store_tiles(cur ^ 1, sa, sb);
        }
    };

    // The next tile's global loads are issued before the current tile is multiplied (one tile ahead).
    const long long KT = (K + BK - 1) / BK;
    load_a(0, ra0);
    load_b(0, rb0);
    store_tiles(0, ra0, rb0);
    __syncthreads();

    for (long long kt = 0; kt < KT; ++kt) {
        const bool more = kt + 1 < KT;
        if (more) {
            load_a((kt + 1) * BK, ra0);
            load_b((kt + 1) * BK, rb0);
        }
        compute((int)(kt & 1), more, ra0, rb0);
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
                    {
                        const float sum_value = acc[i][j][4 * g + r];
#if STORE_C
                        C[row * N + col] = sum_value;
#endif
                        EPILOGUE
                    }
                }
}
)";
    return s;
}

}  // namespace adhip

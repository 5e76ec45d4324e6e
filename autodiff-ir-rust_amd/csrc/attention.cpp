// softmax(scale * Q K^T) V in one kernel, FP32 on the matrix cores: the attention of reference
// src/nn/transformer.rs:10-18 (`dot(softmax(dot(Q, K^T) / sqrt(d_model), -1), V)`), which the reference runs as two
// one-thread-per-element products with the softmax's element-wise and reduction kernels in between, every
// intermediate [Sq, Sk] matrix in memory.  Here the scores never leave the chip: a block owns 64 query rows (four
// wavefronts of 16), walks over the keys BN at a time with the K and V tiles in LDS (fetched one tile ahead into
// registers), multiplies with v_mfma_f32_16x16x4_f32, keeps a running maximum and sum per row (the arithmetic of the
// softmax the caller wrote: exp2((x - max) * log2 e), normalised by the sum) and rescales its accumulators when the
// maximum grows.  The probabilities go from the accumulator layout to the operand layout through the wavefront's own
// part of LDS.  blockIdx.y picks one of up to 16 problems of the same shape (the heads).
#include "attention.hpp"

#include "common.hpp"

namespace adhip {

std::string attention_kernel_source(const AttentionConfig& cfg, const std::string& entry) {
    std::string s;
    std::string params, pick = "switch (blockIdx.y) {";
    for (int i = 0; i < kAttentionSlots; ++i) {
        params += strf("float* o%d, const float* q%d, const float* k%d, const float* v%d, ", i, i, i, i);
        pick += strf(" case %d: O = o%d; Q = q%d; K = k%d; V = v%d; break;", i, i, i, i, i);
    }
    s += "#define GROUP_PARAMS " + params + "\n#define GROUP_PICK " + pick + " default: return; }\n";
    s += strf("#define KERNEL_NAME %s\n#define D %d\n#define DV %d\n#define BN %d\n", entry.c_str(), cfg.d, cfg.dv, cfg.bn);
    s += R"(
#define BM 64
#define KLD (D + 4)
#define VLD (DV + 16)
#define PLD (BN + 4)
typedef float float4_t __attribute__((ext_vector_type(4)));
// O[Sq, DV] = softmax_rows(scale * Q[Sq, D] K[Sk, D]^T) V[Sk, DV]; one block = 64 query rows, 4 wavefronts of 16 rows.
// MFMA 16x16x4 f32: A[i = lane % 16][k = lane / 16], B[k = lane / 16][j = lane % 16], C[4 * (lane / 16) + r][lane % 16].
extern "C" __global__ __launch_bounds__(256) void KERNEL_NAME(
    const int* __restrict__ guard, GROUP_PARAMS long long Sq, long long Sk, long long q_ld, long long k_ld, long long v_ld,
    float scale) {
    if (guard && *guard == 0) return;
    float* __restrict__ O;
    const float* __restrict__ Q;
    const float* __restrict__ K;
    const float* __restrict__ V;
    GROUP_PICK
    __shared__ __attribute__((aligned(16))) float Ks[BN][KLD];
    __shared__ __attribute__((aligned(16))) float Vs[BN][VLD];
    __shared__ __attribute__((aligned(16))) float Ps[4][16][PLD];
    const unsigned tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const unsigned li = lane & 15u, lq = lane >> 4;
    const long long row_base = (long long)blockIdx.x * BM + wave * 16;
    const float LOG2E = 1.44269502162933349609375f;  // the float nearest 1 / ln 2

    // this lane's part of the wavefront's 16 query rows: A[i = li][k = 4 s + lq]
    float qf[D / 4];
    {
        const long long row = row_base + li;
#pragma unroll
        for (int s = 0; s < D / 4; ++s) qf[s] = row < Sq ? Q[row * q_ld + 4 * s + lq] : 0.0f;
    }
    float4_t oacc[DV / 16];
#pragma unroll
    for (int nb = 0; nb < DV / 16; ++nb) oacc[nb] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_i[4], l_i[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) { m_i[r] = -__builtin_inff(); l_i[r] = 0.0f; }

    // The K and V tiles of the next iteration are fetched into registers while this iteration computes (one tile
    // ahead) and parked in LDS when everybody is done with the current ones.
    constexpr int KL = (BN * D / 4 + 255) / 256, VL = (BN * DV / 4 + 255) / 256;
    float4_t kr[KL], vr[VL];
    auto fetch = [&](long long k0) {
#pragma unroll
        for (int i = 0; i < KL; ++i) {
            const unsigned idx = tid + 256u * i, key = idx / (D / 4), f4 = idx % (D / 4);
            kr[i] = float4_t{0.f, 0.f, 0.f, 0.f};
            if (idx < BN * D / 4 && k0 + key < Sk) kr[i] = *(const float4_t*)(K + (k0 + key) * k_ld + 4 * f4);
        }
#pragma unroll
        for (int i = 0; i < VL; ++i) {
            const unsigned idx = tid + 256u * i, key = idx / (DV / 4), f4 = idx % (DV / 4);
            vr[i] = float4_t{0.f, 0.f, 0.f, 0.f};
            if (idx < BN * DV / 4 && k0 + key < Sk) vr[i] = *(const float4_t*)(V + (k0 + key) * v_ld + 4 * f4);
        }
    };
    auto park = [&]() {
#pragma unroll
        for (int i = 0; i < KL; ++i) {
            const unsigned idx = tid + 256u * i, key = idx / (D / 4), f4 = idx % (D / 4);
            if (idx < BN * D / 4) *(float4_t*)&Ks[key][4 * f4] = kr[i];
        }
#pragma unroll
        for (int i = 0; i < VL; ++i) {
            const unsigned idx = tid + 256u * i, key = idx / (DV / 4), f4 = idx % (DV / 4);
            if (idx < BN * DV / 4) *(float4_t*)&Vs[key][4 * f4] = vr[i];
        }
    };
    fetch(0);
    for (long long k0 = 0; k0 < Sk; k0 += BN) {
        __syncthreads();  // everybody is done with the previous tiles
        park();
        __syncthreads();
        if (k0 + BN < Sk) fetch(k0 + BN);

        // scores of 16 rows x BN keys
        float4_t sacc[BN / 16];
#pragma unroll
        for (int nb = 0; nb < BN / 16; ++nb) sacc[nb] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < D / 4; ++s) {
#pragma unroll
            for (int nb = 0; nb < BN / 16; ++nb)
                sacc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(qf[s], Ks[16 * nb + li][4 * s + lq], sacc[nb], 0, 0, 0);
        }
        // running maximum and sum of every row (rows 4 lq + r of this wavefront; 16 lanes share a row)
        float mx[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) mx[r] = -__builtin_inff();
#pragma unroll
        for (int nb = 0; nb < BN / 16; ++nb) {
            const bool valid = k0 + 16 * nb + li < Sk;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float x = valid ? sacc[nb][r] * scale : -__builtin_inff();
                sacc[nb][r] = x;
                mx[r] = fmaxf(mx[r], x);
            }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
#pragma unroll
            for (int o = 1; o < 16; o <<= 1) mx[r] = fmaxf(mx[r], __shfl_xor(mx[r], o, 64));
        }
        float alpha[4], rs[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float m_new = fmaxf(m_i[r], mx[r]);
            alpha[r] = exp2f((m_i[r] - m_new) * LOG2E);
            m_i[r] = m_new;
            rs[r] = 0.0f;
        }
#pragma unroll
        for (int nb = 0; nb < BN / 16; ++nb) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float p = exp2f((sacc[nb][r] - m_i[r]) * LOG2E);
                rs[r] += p;
                Ps[wave][4 * lq + r][16 * nb + li] = p;
            }
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
#pragma unroll
            for (int o = 1; o < 16; o <<= 1) rs[r] += __shfl_xor(rs[r], o, 64);
            l_i[r] = l_i[r] * alpha[r] + rs[r];
        }
#pragma unroll
        for (int nb = 0; nb < DV / 16; ++nb)
#pragma unroll
            for (int r = 0; r < 4; ++r) oacc[nb][r] *= alpha[r];
        // the probabilities go from the accumulator layout to the operand layout through this wavefront's own part of
        // LDS; a wavefront's LDS accesses are carried out in order, the compiler only has to keep them in order too
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int s = 0; s < BN / 4; ++s) {
            const float a = Ps[wave][li][4 * s + lq];
#pragma unroll
            for (int nb = 0; nb < DV / 16; ++nb)
                oacc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, Vs[4 * s + lq][16 * nb + li], oacc[nb], 0, 0, 0);
        }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const long long row = row_base + 4 * lq + r;
        const float inv = 1.0f / l_i[r];
        if (row < Sq) {
#pragma unroll
            for (int nb = 0; nb < DV / 16; ++nb) O[row * DV + 16 * nb + li] = oacc[nb][r] * inv;
        }
    }
}
)";
    return s;
}

}  // namespace adhip

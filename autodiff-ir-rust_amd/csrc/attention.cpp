// softmax(scale * Q K^T) V in one kernel, FP32 on the matrix cores: the attention of reference
// src/nn/transformer.rs:10-18 (`dot(softmax(dot(Q, K^T) / sqrt(d_model), -1), V)`), which the reference runs as two
// one-thread-per-element products with the softmax's element-wise and reduction kernels in between, every
// intermediate [Sq, Sk] matrix in memory.  Here the scores never leave the chip.
//
// A block is 4 WG wavefronts on 64 query rows: wavefront w works on rows 16 (w % 4) .. + 15 and, of every tile of BN
// keys, on keys (w / 4) BN / WG .. + BN / WG - 1; with WG = 2 the two halves keep their own running maximum, sum and
// accumulators, which are merged at the end (the same arithmetic as the softmax the caller wrote: exp2((x - max) *
// log2 e), normalised by the sum; accumulators are rescaled when the maximum grows).  K and V tiles live in two LDS
// stages: while one is computed on, the next tile (fetched into registers one iteration earlier) is parked in the
// other, with one barrier per tile.  The probabilities go from the accumulator layout to the operand layout through
// the wavefront's own part of LDS.  Operand reads from LDS run one MFMA step ahead of the MFMAs that use them.
//
// On this hardware FP32 MFMAs and ordinary vector instructions do not overlap (neither within a wavefront nor between
// the wavefronts of a SIMD: a loop of 64 MFMAs and a loop of 512 vector operations take as long together as one after
// the other), so every vector instruction in the loop costs matrix time: addresses are computed once outside the
// loop, ragged-edge masking and the rescaling of the accumulators only run when they are needed.
//
// MFMA 16x16x4 f32: A[i = lane % 16][k = lane / 16], B[k = lane / 16][j = lane % 16], C[4 (lane / 16) + r][lane % 16].
// With D % 16 == 0 the contraction index of the scores is spread over the lanes in runs of four (in step (S, u) lane
// group lq supplies element 16 S + 4 lq + u), so a lane's operands for four consecutive steps are one 128-bit LDS
// read; the weighted values use the same spreading over the keys of a tile.
#include "attention.hpp"

#include "common.hpp"

namespace adhip {

size_t attention_lds_bytes(const AttentionConfig& cfg) {
    const size_t stage = (size_t)cfg.bn * (size_t)(cfg.d + 4 + cfg.dv + 4);
    const size_t patches = (size_t)4 * cfg.wg * 16 * (size_t)(cfg.bn / cfg.wg + 4);
    return 4 * (2 * stage + patches);
}

std::string attention_kernel_source(const AttentionConfig& cfg, const std::string& entry) {
    std::string s;
    std::string params, pick = "switch (problem) {";
    for (int i = 0; i < kAttentionSlots; ++i) {
        params += strf("float* o%d, const float* q%d, const float* k%d, const float* v%d, ", i, i, i, i);
        if (cfg.mask) params += strf("const float* m%d, ", i);
        pick += strf(" case %d: O = o%d; Q = q%d; K = k%d; V = v%d;%s break;", i, i, i, i, i, cfg.mask ? strf(" Mk = m%d;", i).c_str() : "");
    }
    s += "#define GROUP_PARAMS " + params + "\n#define GROUP_PICK " + pick + " default: return; }\n";
    s += strf("#define KERNEL_NAME %s\n#define D %d\n#define DV %d\n#define BN %d\n#define WG %d\n#define MASK %d\n", entry.c_str(), cfg.d, cfg.dv, cfg.bn,
              cfg.wg, cfg.mask ? 1 : 0);
    s += cfg.mask ? "#define MASK_LD long long m_ld,\n" : "#define MASK_LD\n";
    s += "typedef float float4_t __attribute__((ext_vector_type(4)));\n";
    s += R"ATTN(
#define NT (256 * WG)
#define BNW (BN / WG)
#define KLD (D + 4)
#define VLD (DV + 4)
#define PLD (BNW + 4)
#define STAGE (BN * KLD + BN * VLD)
// Value of lane (16 q + perm(i)) for every lane 16 q + i; every lane has a source, so the "old" value never shows.
#define ROW16_FROM(x, ctrl) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, (x)), (ctrl), 0xF, 0xF, true))
static __device__ __forceinline__ float row16_max(float x) {
    // maximum over the 16 lanes that share an accumulator row (lanes 16 q .. 16 q + 15)
    x = fmaxf(x, ROW16_FROM(x, 0xB1));    // quad_perm [1,0,3,2]
    x = fmaxf(x, ROW16_FROM(x, 0x4E));    // quad_perm [2,3,0,1]
    x = fmaxf(x, ROW16_FROM(x, 0x141));   // row_half_mirror
    x = fmaxf(x, ROW16_FROM(x, 0x140));   // row_mirror
    return x;
}
static __device__ __forceinline__ float row16_sum(float x) {
    // every step adds a lane's value and its partner's, both partners in the same way: all 16 lanes end with the same bits
    x += ROW16_FROM(x, 0xB1);
    x += ROW16_FROM(x, 0x4E);
    x += ROW16_FROM(x, 0x141);
    x += ROW16_FROM(x, 0x140);
    return x;
}

extern "C" __global__ __launch_bounds__(NT) void KERNEL_NAME(
    const int* __restrict__ guard, GROUP_PARAMS long long Sq, long long Sk, long long q_ld, long long k_ld, long long v_ld,
    MASK_LD float scale, int row_blocks, int problems) {
    if (guard && *guard == 0) return;
    // Blocks are handed to the eight XCDs in turn; renumbering them so that an XCD's blocks are consecutive puts the row
    // blocks of one problem on one XCD, whose L2 then fetches that problem's K and V once.
    unsigned bid = blockIdx.x;
    {
        const unsigned total = (unsigned)row_blocks * (unsigned)problems;
        if (total % 8u == 0u) bid = (bid % 8u) * (total / 8u) + bid / 8u;
    }
    const unsigned problem = bid / (unsigned)row_blocks, row_block = bid % (unsigned)row_blocks;
    float* __restrict__ O;
    const float* __restrict__ Q;
    const float* __restrict__ K;
    const float* __restrict__ V;
#if MASK
    const float* __restrict__ Mk;
#endif
    GROUP_PICK
    __shared__ __attribute__((aligned(16))) float lds[2 * STAGE + 4 * WG * 16 * PLD];
    float (*Ps)[16][PLD] = (float (*)[16][PLD])(lds + 2 * STAGE);
    const unsigned tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const unsigned li = lane & 15u, lq = lane >> 4, rw = wave & 3u, kg = wave >> 2;
    const long long row_base = (long long)row_block * 64 + rw * 16;
    const float LOG2E = 1.44269502162933349609375f;  // the float nearest 1 / ln 2

    // this lane's part of the wavefront's 16 query rows
#if D % 16 == 0
    float4_t qf[D / 16];
    {
        const long long row = row_base + li;
#pragma unroll
        for (int S = 0; S < D / 16; ++S)
            qf[S] = row < Sq ? *(const float4_t*)(Q + row * q_ld + 16 * S + 4 * lq) : float4_t{0.f, 0.f, 0.f, 0.f};
    }
#else
    float qf[D / 4];
    {
        const long long row = row_base + li;
#pragma unroll
        for (int s = 0; s < D / 4; ++s) qf[s] = row < Sq ? Q[row * q_ld + 4 * s + lq] : 0.0f;
    }
#endif
    float4_t oacc[DV / 16];
#pragma unroll
    for (int nb = 0; nb < DV / 16; ++nb) oacc[nb] = float4_t{0.f, 0.f, 0.f, 0.f};
    float m_i[4], l_i[4];   // running maximum of the row; this lane's share of the running sum (added up at the end)
#pragma unroll
    for (int r = 0; r < 4; ++r) { m_i[r] = -__builtin_inff(); l_i[r] = 0.0f; }
#if MASK
    // where this lane's four accumulator rows start in the mask, at this key group's and lane's column (rows beyond Sq
    // are never stored: they read the last row)
    const float* mrow[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const long long row = row_base + 4 * lq + r;
        mrow[r] = Mk + (row < Sq ? row : Sq - 1) * m_ld + kg * BNW + li;
    }
#endif

    // The next tile travels through registers.  Where a thread's pieces sit inside a tile, in memory and in LDS, is
    // computed once; a tile's base is uniform.  Keys beyond Sk (last tile only) are fetched from the last valid row
    // instead: their scores are masked to -inf and their probabilities are 0, so what stands there only has to be finite.
    constexpr int KL = (BN * D / 4 + NT - 1) / NT, VL = (BN * DV / 4 + NT - 1) / NT;
    float4_t kr[KL], vr[VL];
    unsigned k_key[KL], k_mem[KL], k_lds[KL], v_key[VL], v_mem[VL], v_lds[VL];
#pragma unroll
    for (int i = 0; i < KL; ++i) {
        const unsigned idx = tid + NT * i, key = idx / (D / 4), f4 = idx % (D / 4);
        k_key[i] = key; k_mem[i] = key * (unsigned)k_ld + 4 * f4; k_lds[i] = key * KLD + 4 * f4;
    }
#pragma unroll
    for (int i = 0; i < VL; ++i) {
        const unsigned idx = tid + NT * i, key = idx / (DV / 4), f4 = idx % (DV / 4);
        v_key[i] = key; v_mem[i] = key * (unsigned)v_ld + 4 * f4; v_lds[i] = BN * KLD + key * VLD + 4 * f4;
    }
    auto fetch = [&](long long k0) {
        const float* kb = K + k0 * k_ld;
        const float* vb = V + k0 * v_ld;
        if (k0 + BN <= Sk) {
#pragma unroll
            for (int i = 0; i < KL; ++i)
                if (BN * D / 4 % NT == 0 || tid + NT * i < BN * D / 4) kr[i] = *(const float4_t*)(kb + k_mem[i]);
#pragma unroll
            for (int i = 0; i < VL; ++i)
                if (BN * DV / 4 % NT == 0 || tid + NT * i < BN * DV / 4) vr[i] = *(const float4_t*)(vb + v_mem[i]);
        } else {
            const unsigned last = (unsigned)(Sk - 1 - k0);
#pragma unroll
            for (int i = 0; i < KL; ++i)
                if (BN * D / 4 % NT == 0 || tid + NT * i < BN * D / 4) {
                    const unsigned back = k_key[i] > last ? k_key[i] - last : 0u;
                    kr[i] = *(const float4_t*)(kb + (k_mem[i] - back * (unsigned)k_ld));
                }
#pragma unroll
            for (int i = 0; i < VL; ++i)
                if (BN * DV / 4 % NT == 0 || tid + NT * i < BN * DV / 4) {
                    const unsigned back = v_key[i] > last ? v_key[i] - last : 0u;
                    vr[i] = *(const float4_t*)(vb + (v_mem[i] - back * (unsigned)v_ld));
                }
        }
    };
    auto park = [&](int stage) {
        float* base = lds + stage * STAGE;
#pragma unroll
        for (int i = 0; i < KL; ++i)
            if (BN * D / 4 % NT == 0 || tid + NT * i < BN * D / 4) *(float4_t*)(base + k_lds[i]) = kr[i];
#pragma unroll
        for (int i = 0; i < VL; ++i)
            if (BN * DV / 4 % NT == 0 || tid + NT * i < BN * DV / 4) *(float4_t*)(base + v_lds[i]) = vr[i];
    };
    fetch(0);
    park(0);
    if (BN < Sk) fetch(BN);
    int stage = 0;
    for (long long k0 = 0; k0 < Sk; k0 += BN, stage ^= 1) {
        // tile k0 is complete in this stage, and everybody is done with the other stage (the previous tile)
        __syncthreads();
        float (*Ks)[KLD] = (float (*)[KLD])(lds + stage * STAGE + kg * BNW * KLD);
        float (*Vs)[VLD] = (float (*)[VLD])(lds + stage * STAGE + BN * KLD + kg * BNW * VLD);
        if (k0 + BN < Sk) {
            park(stage ^ 1);
            if (k0 + 2 * BN < Sk) fetch(k0 + 2 * BN);
        }

        // ---- scores of 16 rows x BNW keys.  The K operands of step S + 1 are read while the MFMAs of step S run;
        // two accumulators per block of 16 keys (even and odd u) keep dependent MFMAs apart.
        float4_t sacc[BNW / 16], sodd[BNW / 16];
#pragma unroll
        for (int nb = 0; nb < BNW / 16; ++nb) { sacc[nb] = float4_t{0.f, 0.f, 0.f, 0.f}; sodd[nb] = float4_t{0.f, 0.f, 0.f, 0.f}; }
#if D % 16 == 0
        {
            float4_t kf[2][BNW / 16];
#pragma unroll
            for (int nb = 0; nb < BNW / 16; ++nb) kf[0][nb] = *(const float4_t*)&Ks[16 * nb + li][4 * lq];
#pragma unroll
            for (int S = 0; S < D / 16; ++S) {
                if (S + 1 < D / 16) {
#pragma unroll
                    for (int nb = 0; nb < BNW / 16; ++nb)
                        kf[(S + 1) & 1][nb] = *(const float4_t*)&Ks[16 * nb + li][16 * (S + 1) + 4 * lq];
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < 4; u += 2) {
#pragma unroll
                    for (int nb = 0; nb < BNW / 16; ++nb)
                        sacc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(qf[S][u], kf[S & 1][nb][u], sacc[nb], 0, 0, 0);
#pragma unroll
                    for (int nb = 0; nb < BNW / 16; ++nb)
                        sodd[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(qf[S][u + 1], kf[S & 1][nb][u + 1], sodd[nb], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
#else
#pragma unroll
        for (int s = 0; s < D / 4; ++s) {
#pragma unroll
            for (int nb = 0; nb < BNW / 16; ++nb) {
                if (s & 1) sodd[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(qf[s], Ks[16 * nb + li][4 * s + lq], sodd[nb], 0, 0, 0);
                else sacc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(qf[s], Ks[16 * nb + li][4 * s + lq], sacc[nb], 0, 0, 0);
            }
        }
#endif
        // ---- running maximum of every row (rows 4 lq + r of this wavefront; 16 lanes share a row)
        float mx[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) mx[r] = -__builtin_inff();
#if MASK
#pragma unroll
        for (int nb = 0; nb < BNW / 16; ++nb) {
            // the scaled score times the mask, in that order, as the caller wrote it; keys beyond Sk read nothing
            const bool inside = k0 + BN <= Sk || k0 + kg * BNW + 16 * nb + li < Sk;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float mv = inside ? mrow[r][k0 + 16 * nb] : 0.0f;
                sacc[nb][r] = ((sacc[nb][r] + sodd[nb][r]) * scale) * mv;
            }
        }
#else
#pragma unroll
        for (int nb = 0; nb < BNW / 16; ++nb)
#pragma unroll
            for (int r = 0; r < 4; ++r) sacc[nb][r] = (sacc[nb][r] + sodd[nb][r]) * scale;
#endif
        if (k0 + BN > Sk) {   // the last tile may reach beyond the keys
#pragma unroll
            for (int nb = 0; nb < BNW / 16; ++nb) {
                const bool valid = k0 + kg * BNW + 16 * nb + li < Sk;
#pragma unroll
                for (int r = 0; r < 4; ++r) sacc[nb][r] = valid ? sacc[nb][r] : -__builtin_inff();
            }
        }
#pragma unroll
        for (int nb = 0; nb < BNW / 16; ++nb)
#pragma unroll
            for (int r = 0; r < 4; ++r) mx[r] = fmaxf(mx[r], sacc[nb][r]);
        float m_new[4], mu[4];
        bool grew = false;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            m_new[r] = fmaxf(m_i[r], row16_max(mx[r]));
            grew = grew || m_new[r] != m_i[r];
            // a key group that has not seen a valid key yet keeps -inf; the exponentials are then taken against 0
            mu[r] = m_new[r] == -__builtin_inff() ? 0.0f : m_new[r];
        }
        if (__builtin_amdgcn_ballot_w64(grew) != 0ull) {
            // some row's maximum grew: what has been accumulated against the old maximum is rescaled
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float alpha = __builtin_amdgcn_exp2f((m_i[r] - mu[r]) * LOG2E);
                l_i[r] *= alpha;
#pragma unroll
                for (int nb = 0; nb < DV / 16; ++nb) oacc[nb][r] *= alpha;
                m_i[r] = m_new[r];
            }
        }
#pragma unroll
        for (int nb = 0; nb < BNW / 16; ++nb) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float p = __builtin_amdgcn_exp2f((sacc[nb][r] - mu[r]) * LOG2E);
                l_i[r] += p;
                Ps[wave][4 * lq + r][16 * nb + li] = p;
            }
        }
        // the probabilities go from the accumulator layout to the operand layout through this wavefront's own part of
        // LDS; a wavefront's LDS accesses are carried out in order, the compiler only has to keep them in order too
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        {
            // ---- weighted values: step t covers four keys of this wavefront's share (in the spread order); the V
            // operands of step t + 1 are read while the MFMAs of step t run
            float4_t a[BNW / 16];
#pragma unroll
            for (int S = 0; S < BNW / 16; ++S) a[S] = *(const float4_t*)&Ps[wave][li][16 * S + 4 * lq];
            float vb[2][DV / 16];
#pragma unroll
            for (int nb = 0; nb < DV / 16; ++nb) vb[0][nb] = Vs[4 * lq][16 * nb + li];
#pragma unroll
            for (int t = 0; t < BNW / 4; ++t) {
                if (t + 1 < BNW / 4) {
#pragma unroll
                    for (int nb = 0; nb < DV / 16; ++nb)
                        vb[(t + 1) & 1][nb] = Vs[16 * ((t + 1) / 4) + 4 * lq + ((t + 1) & 3)][16 * nb + li];
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int nb = 0; nb < DV / 16; ++nb)
                    oacc[nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[t / 4][t & 3], vb[t & 1][nb], oacc[nb], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) l_i[r] = row16_sum(l_i[r]);
#if WG == 2
    // the second key group hands its maximum, sum and accumulators to the first through LDS (the tiles are done with)
    __syncthreads();
    {
        float* mg = lds + (size_t)(rw * 64 + lane) * (DV / 4 + 8);
        if (kg == 1) {
#pragma unroll
            for (int r = 0; r < 4; ++r) { mg[r] = m_i[r]; mg[4 + r] = l_i[r]; }
#pragma unroll
            for (int nb = 0; nb < DV / 16; ++nb) *(float4_t*)(mg + 8 + 4 * nb) = oacc[nb];
        }
        __syncthreads();
        if (kg == 1) return;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float mb = mg[r], lb = mg[4 + r];
            const float m = fmaxf(m_i[r], mb);   // the first group always holds key 0: finite; a group without keys has -inf and sum 0
            const float ea = __builtin_amdgcn_exp2f((m_i[r] - m) * LOG2E), eb = __builtin_amdgcn_exp2f((mb - m) * LOG2E);
            l_i[r] = l_i[r] * ea + lb * eb;
#pragma unroll
            for (int nb = 0; nb < DV / 16; ++nb) oacc[nb][r] = oacc[nb][r] * ea + mg[8 + 4 * nb + r] * eb;
        }
    }
#endif
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
)ATTN";
    return s;
}

}  // namespace adhip

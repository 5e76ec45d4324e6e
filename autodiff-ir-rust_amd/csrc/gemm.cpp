// FP32 matrix product for gfx950 on the matrix cores (v_mfma_f32_32x32x2_f32), LDS-tiled.
//
// The reference multiplies with one work-item per output element, a sequential k loop and two
// global loads per multiply-add (reference src/devices/opencl/kernels/dotprod.rs:23-53); transposed
// operands are folded into its index expressions.  Here both operands are described by strides
// (so x^T and W^T of the backward pass need no copy), staged through LDS in 256x128x16, 128x128x16 or
// 64x64x16 tiles with the global loads two tiles ahead in registers.  A wavefront owns a 64x64 sub-tile (2x2 MFMA
// blocks of 32x32) in the two large tiles and one 32x32 block in the small one, which exists so that
// products with a small output still put a few hundred blocks on the chip.
#include "gemm.hpp"

#include <algorithm>
#include <cstdlib>

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
    s += strf("#define A_KCONTIG %d\n#define B_KCONTIG %d\n#define EDGE %d\n#define EDGE_VEC %d\n#define SPLITK %d\n#define GROUPED %d\n", cfg.a_kcontig ? 1 : 0,
              cfg.b_kcontig ? 1 : 0, cfg.edge ? 1 : 0, cfg.edge && cfg.edge_vec ? 1 : 0, cfg.split_k ? 1 : 0, cfg.grouped ? 1 : 0);
    if (cfg.grouped) {
        // one parameter triple per problem slot, and the (wave-uniform) choice among them by blockIdx.y
        std::string params, pick = "switch (blockIdx.y) {";
        for (int i = 0; i < kGemmGroupSlots; ++i) {
            params += strf("float* c%d, const float* a%d, const float* b%d, ", i, i, i);
            pick += strf(" case %d: C = c%d; A = a%d; B = b%d; break;", i, i, i, i);
        }
        s += "#define GROUP_PARAMS " + params + "\n#define GROUP_PICK " + pick + " default: return; }\n";
    }
    // tile geometry: BM x BN block tile, TM x TN MFMA blocks per wave, WGN waves along n
    const int bn = cfg.bn ? cfg.bn : (cfg.bm == 64 ? 64 : 128);
    const int tm = cfg.bm == 64 ? 1 : 2, tn = (bn == 64) ? 1 : 2;
    const int waves = (cfg.bm / (32 * tm)) * (bn / (32 * tn));
    s += strf("#define KERNEL_NAME %s\n#define BM %d\n#define BN %d\n#define TM %d\n#define TN %d\n#define NT %d\n", entry.c_str(),
              cfg.bm, bn, tm, tn, waves * 64);
    {
        // diagnostic: ADHIP_GEMM_AHEAD=1 keeps the global loads one k-tile ahead of the MFMAs instead of two
        int ahead = 2;
        if (const char* e = getenv("ADHIP_GEMM_AHEAD")) ahead = atoi(e) == 1 ? 1 : 2;
        s += strf("#define AHEAD %d\n", ahead);
    }
    s += R"(
#define BK 16
// An MFMA operand read from LDS.  Volatile and explicitly in the LDS address space: the compiler then issues one
// ds_read_b32 per operand with the whole tile offset in the instruction's 16-bit immediate field, instead of pairing
// neighbouring reads into ds_read2_b32, whose 8-bit offsets do not reach the next k-row, so that every pair needed a
// vector add for its base.  Vector ALU instructions and FP32 MFMAs do not overlap on a SIMD; the 14 adds per k-tile
// this removes are worth 2 % (4096^3: 0.827 -> 0.844 of the FP32 matrix peak).
#define LDS_OPERAND(x) (*(const volatile __attribute__((address_space(3))) float*)&(x))
#define LDA (BM + 4)
#define LDB (BN + 4)
#define WGN (BN / (32 * TN))            /* waves along n */
#define A_LOADS (BM * BK / 4 / NT)      /* float4 loads of the A tile per thread */
#define B_LOADS (BN * BK / 4 / NT)      /* float4 loads of the B tile per thread */
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
// 128 bits of an operand that is only known to be 4-byte aligned (an odd leading dim or offset): still one
// global_load_dwordx4, which the hardware splits where it crosses a cache line
typedef float4_t float4_ua __attribute__((aligned(4)));

#if EDGE
// Four operand elements p[off + j * step], j = 0..3, of which the first `valid` (any integer; <= 0: none) exist; the
// others read as 0.  `step` is the operand's unit stride (the four run along its contiguous dim).  With EDGE_VEC
// (the operands' contiguous extents are at least 4) a thread whose
// four elements all exist takes them with one 128-bit load, as the kernel without EDGE does, and only the threads on
// the ragged rim fall back to single elements.  The common load sits under no condition (a thread of the rim reads
// the operand's first elements there, and an element that does not exist is read at the first element and replaced),
// so that the loads of a tile are in flight together.  With EDGE_VEC the kernel calls this only for the last,
// ragged k-tile and for quads that straddle the end of M or N: everywhere else a row or column beyond the product
// is replaced by one inside it (what it contributes to is never stored) and the load is the plain 128-bit one.
static __device__ __forceinline__ float4_t edge_load4(const float* p, long long off, long long step, long long valid) {
    float4_t v;
#if EDGE_VEC
    const bool whole = valid >= 4;
    v = *(const float4_ua*)(p + (whole ? off : 0));
    if (!whole)
#endif
    {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bool ok = j < valid;
            const float x = p[ok ? off + j * step : 0];
            v[j] = ok ? x : 0.0f;
        }
    }
    return v;
}
#endif

// A is [M,K] with element strides (a_sm, a_sk); B is [K,N] with (b_sk, b_sn); C dense [M,N].
// A_KCONTIG: a_sk == 1 (else a_sm == 1).  B_KCONTIG: b_sk == 1 (else b_sn == 1).
// EDGE: M, N or K is not a multiple of the tile, or an operand is not 16-byte aligned.  Stores are bounds-checked;
// loads go through edge_load4 where an element may not exist (all of them without EDGE_VEC; with it, only the last
// ragged k-tile and quads that straddle the end of M or N).
// SPLITK: the block at blockIdx.y multiplies only k in [y*k_chunk, (y+1)*k_chunk) and writes slice y of a
// [gridDim.y][M][N] buffer; the caller adds the slices in a fixed order.  For products whose output alone gives
// too few blocks to hide the latency of the operand loads.
// GROUPED: several independent products of one shape and one set of strides in a single launch; the block row
// blockIdx.y works on problem y, whose three base pointers (operand offsets already applied) are parameters
// c<y>, a<y>, b<y>.  For the same kind of product when there are many of them (the per-head projections of
// multi-head attention).  With SPLITK the range of k is picked by blockIdx.z.
extern "C" __global__ __launch_bounds__(NT) void KERNEL_NAME(
#if GROUPED
    const int* __restrict__ guard, GROUP_PARAMS long long M, long long N, long long K, long long a_sm, long long a_sk,
    long long b_sk, long long b_sn
#if SPLITK
    , long long k_chunk
#endif
    ) {
    if (guard && *guard == 0) return;
    float* __restrict__ C;
    const float* __restrict__ A;
    const float* __restrict__ B;
    GROUP_PICK
    const long long a_off = 0, b_off = 0;
#else
    const int* __restrict__ guard, float* __restrict__ C, const float* __restrict__ A, const float* __restrict__ B,
    long long M, long long N, long long K, long long a_off, long long a_sm, long long a_sk, long long b_off,
    long long b_sk, long long b_sn
#if SPLITK
    , long long k_chunk
#endif
    EPI_PARAMS) {
    if (guard && *guard == 0) return;
#endif
#if SPLITK
#if GROUPED
    const unsigned slice = blockIdx.z;  // c<y> points at problem y's own [gridDim.z][M][N] slices
#else
    const unsigned slice = blockIdx.y;
#endif
    const long long k_lo = (long long)slice * k_chunk;
    const long long k_hi = min(K, k_lo + k_chunk);
    C += (long long)slice * M * N;
#else
    const long long k_lo = 0, k_hi = K;
#endif
    __shared__ __attribute__((aligned(16))) float As[2][BK][LDA];
    __shared__ __attribute__((aligned(16))) float Bs[2][BK][LDB];

    const unsigned tid = threadIdx.x;
    const unsigned lane = tid & 63u, wave = tid >> 6;
    const unsigned wm = wave / WGN, wn = wave % WGN;
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

    float16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    float4_t ra0[A_LOADS], rb0[B_LOADS];

    auto load_a = [&](long long k0, float4_t* ra) {
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
#if A_KCONTIG
            const unsigned kq = tid & 3u, mr = (tid >> 2) + (NT / 4) * i;
            const long long m = bm + mr, k = k0 + 4 * kq;
#if EDGE
            // rows beyond M only feed rows of the product that are never stored: they read the last row instead
            if (EDGE_VEC && k0 + BK <= k_hi) ra[i] = *(const float4_ua*)(A + min(m, M - 1) * a_sm + k);
            else ra[i] = edge_load4(A, m * a_sm + k * a_sk, a_sk, m < M ? k_hi - k : 0);
#else
            ra[i] = *(const float4_t*)(A + m * a_sm + k);
#endif
#else
            const unsigned mq = tid % (BM / 4), kr = tid / (BM / 4) + (NT / (BM / 4)) * i;
            const long long m = bm + 4 * mq, k = k0 + kr;
#if EDGE
            // a quad of rows that lies wholly beyond M reads the last whole quad instead; one that straddles M is
            // taken element by element
            if (EDGE_VEC && k0 + BK <= k_hi && (m + 4 <= M || m >= M)) ra[i] = *(const float4_ua*)(A + k * a_sk + min(m, (M - 4) & ~3ll));
            else ra[i] = edge_load4(A, m * a_sm + k * a_sk, a_sm, k < k_hi ? M - m : 0);
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
            if (EDGE_VEC && k0 + BK <= k_hi) rb[i] = *(const float4_ua*)(B + min(n, N - 1) * b_sn + k);
            else rb[i] = edge_load4(B, k * b_sk + n * b_sn, b_sk, n < N ? k_hi - k : 0);
#else
            rb[i] = *(const float4_t*)(B + n * b_sn + k);
#endif
#else
            const unsigned nq = tid % (BN / 4), kr = tid / (BN / 4) + (NT / (BN / 4)) * i;
            const long long n = bn + 4 * nq, k = k0 + kr;
#if EDGE
            if (EDGE_VEC && k0 + BK <= k_hi && (n + 4 <= N || n >= N)) rb[i] = *(const float4_ua*)(B + k * b_sk + min(n, (N - 4) & ~3ll));
            else rb[i] = edge_load4(B, k * b_sk + n * b_sn, b_sn, k < k_hi ? N - n : 0);
#else
            rb[i] = *(const float4_t*)(B + k * b_sk + n);
#endif
#endif
        }
    };
    auto store_tiles = [&](int buf, const float4_t* ra, const float4_t* rb) {
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
#if A_KCONTIG
            const unsigned kq = tid & 3u, mr = (tid >> 2) + (NT / 4) * i;
#pragma unroll
            for (int j = 0; j < 4; ++j) As[buf][4 * kq + j][mr] = ra[i][j];
#else
            const unsigned mq = tid % (BM / 4), kr = tid / (BM / 4) + (NT / (BM / 4)) * i;
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
            const unsigned nq = tid % (BN / 4), kr = tid / (BN / 4) + (NT / (BN / 4)) * i;
            *(float4_t*)&Bs[buf][kr][4 * nq] = rb[i];
#endif
        }
    };

    // One k-tile: 8 MFMA steps from LDS buffer `cur`; the operands of step ks+1 are fetched from LDS before the
    // four MFMAs of step ks are issued, and half way through the tile that was prefetched into registers (sa, sb)
    // is parked in the other LDS buffer, which nobody reads during this iteration.
    auto compute = [&](int cur, bool park, const float4_t* sa, const float4_t* sb) {
        float fa[TM][2], fb[TN][2];
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[i][0] = LDS_OPERAND(As[cur][lh][wm * (32 * TM) + 32 * i + li]);
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[j][0] = LDS_OPERAND(Bs[cur][lh][wn * (32 * TN) + 32 * j + li]);
#pragma unroll
        for (int ks = 0; ks < BK / 2; ++ks) {
            const int c = ks & 1, nx = c ^ 1;
            if (ks + 1 < BK / 2) {
#pragma unroll
                for (int i = 0; i < TM; ++i) fa[i][nx] = LDS_OPERAND(As[cur][2 * (ks + 1) + lh][wm * (32 * TM) + 32 * i + li]);
#pragma unroll
                for (int j = 0; j < TN; ++j) fb[j][nx] = LDS_OPERAND(Bs[cur][2 * (ks + 1) + lh][wn * (32 * TN) + 32 * j + li]);
            }
            __builtin_amdgcn_sched_barrier(0);  // keep the LDS reads ahead of the MFMAs that hide their latency
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][c], fb[j][c], acc[i][j], 0, 0, 0);
            if (ks == BK / 4 - 1 && park) store_tiles(cur ^ 1, sa, sb);
        }
    };

    const int KT = __builtin_amdgcn_readfirstlane((int)((k_hi - k_lo + BK - 1) / BK));   // (uniform: kept in a scalar register)
#if AHEAD == 2
    // Global loads run two k-tiles ahead of the MFMAs, in two register sets that take turns: during tile kt the loads
    // of tile kt + 2 are issued into the set that held tile kt (parked in LDS during tile kt - 1), and the set that
    // holds tile kt + 1, issued a whole tile earlier, is parked.  A load then has a k-tile and a half of MFMAs to
    // arrive instead of half a tile (which is some 500 cycles where a wavefront owns 64x32, less than a trip to
    // memory): 4096 x 1024 x 4096 in 276 / 268 / 251 us instead of 289 / 274 / 257, the MLP workload's step 1.2 % and
    // the encoder layer's 1.3 % shorter.  The loop is unrolled by two so that the sets and the LDS buffers are named,
    // not indexed.
    // Loads and parkings stand under no condition: beyond the last tile the loads fetch the last tile again and the
    // parking writes a tile nobody reads.  (Under a condition, the wait in front of a parking also waits for the
    // newest loads, or the compiler moves the loads down to the parking that consumes them.)
    int t_at = 0;   // the tile the next loads fetch
#if EDGE
    auto load_next = [&](float4_t* ra, float4_t* rb) {
        load_a(k_lo + (long long)t_at * BK, ra);
        load_b(k_lo + (long long)t_at * BK, rb);
        t_at += t_at + 1 < KT ? 1 : 0;
    };
#else
    // Without bounds checks an address is a wave-uniform pointer -- the tile's corner, moved on from tile to tile and
    // from one of a thread's loads to its next by scalar instructions -- plus one 32-bit offset per thread and
    // operand that never changes: no vector instruction per load (vector instructions are paid in matrix time).
    const unsigned oa = A_KCONTIG ? (tid >> 2) * (unsigned)a_sm + 4u * (tid & 3u) : (tid / (BM / 4)) * (unsigned)a_sk + 4u * (tid % (BM / 4));
    const unsigned ob = B_KCONTIG ? (tid >> 2) * (unsigned)b_sn + 4u * (tid & 3u) : (tid / (BN / 4)) * (unsigned)b_sk + 4u * (tid % (BN / 4));
    const float* Ab = A + (A_KCONTIG ? bm * a_sm + k_lo : k_lo * a_sk + bm);
    const float* Bb = B + (B_KCONTIG ? bn * b_sn + k_lo : k_lo * b_sk + bn);
    const long long ia = A_KCONTIG ? (NT / 4) * a_sm : (NT / (BM / 4)) * a_sk;   // from one of a thread's loads to its next
    const long long ib = B_KCONTIG ? (NT / 4) * b_sn : (NT / (BN / 4)) * b_sk;
    const long long step_a = A_KCONTIG ? BK : BK * a_sk, step_b = B_KCONTIG ? BK : BK * b_sk;
    auto load_next = [&](float4_t* ra, float4_t* rb) {
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) ra[i] = *(const float4_t*)((const char*)(Ab + i * ia) + (size_t)(4u * oa));
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i) rb[i] = *(const float4_t*)((const char*)(Bb + i * ib) + (size_t)(4u * ob));
        const bool go = t_at + 1 < KT;
        Ab += go ? step_a : 0;
        Bb += go ? step_b : 0;
        t_at += go ? 1 : 0;
    };
#endif
    float4_t ra1[A_LOADS], rb1[B_LOADS];
    load_next(ra0, rb0);
    store_tiles(0, ra0, rb0);
    load_next(ra1, rb1);
    __syncthreads();
    int kt = 0;
    for (; kt + 1 < KT; kt += 2) {
        load_next(ra0, rb0);
        compute(0, true, ra1, rb1);
        __syncthreads();
        load_next(ra1, rb1);
        compute(1, true, ra0, rb0);
        __syncthreads();
    }
    if (kt < KT) compute(0, false, ra1, rb1);   // an odd number of tiles: the last one sits in buffer 0
#else
    // The next tile's global loads are issued before the current tile is multiplied (one tile ahead).
    load_a(k_lo, ra0);
    load_b(k_lo, rb0);
    store_tiles(0, ra0, rb0);
    __syncthreads();

    for (long long kt = 0; kt < KT; ++kt) {
        const bool more = kt + 1 < KT;
        if (more) {
            load_a(k_lo + (kt + 1) * BK, ra0);
            load_b(k_lo + (kt + 1) * BK, rb0);
        }
        compute((int)(kt & 1), more, ra0, rb0);
        __syncthreads();
    }
#endif

    // acc[i][j][4g + r] holds C[row = 32i + 8g + 4*lh + r][col = 32j + li] of the wave's sub-tile
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const long long row = bm + wm * (32 * TM) + 32 * i + 8 * g + 4 * lh + r;
                    const long long col = bn + wn * (32 * TN) + 32 * j + li;
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

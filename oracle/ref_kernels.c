/*
 * TEST INFRASTRUCTURE ONLY -- not part of the product path.
 *
 * CPU restatement of the arithmetic the reference's OpenCL device executes, one function per
 * reference kernel.  Used by oracle/interp.py as the checker in tests/, in
 * __graft_entry__.smoke() and as bench.py's cpu_baseline leg.  Nothing under the product
 * package links or loads this file.
 *
 * Each function states which reference kernel template it follows.  Work-items of the
 * reference become loop iterations, parallelised with OpenMP over the work-item index.
 * Compile with -ffp-contract=off so that `value += a*b` is a separate multiply and add.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* One work-item per C element, sequential k, one f32 accumulator:
 * reference src/devices/opencl/kernels/dotprod.rs:23-53.
 * A is [m,k] with element strides (a_rs, a_cs); B is [k,n] with (b_rs, b_cs); C dense [m,n].
 * The reference folds transposes into the index expression; strides do the same here. */
void ref_dot(const float *A, int64_t a_rs, int64_t a_cs, const float *B, int64_t b_rs, int64_t b_cs,
             float *C, int64_t m, int64_t k, int64_t n)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t ty = 0; ty < m; ++ty) {
        for (int64_t tx = 0; tx < n; ++tx) {
            float value = 0.0f;
            for (int64_t kk = 0; kk < k; ++kk) {
                float ea = A[ty * a_rs + kk * a_cs];
                float eb = B[kk * b_rs + tx * b_cs];
                value += ea * eb;
            }
            C[ty * n + tx] = value;
        }
    }
}

/* One work-group per output element, `local` lanes, halving tree in local memory:
 * reference src/devices/opencl/kernels/reduce.rs:29-63.
 * The reference sizes the group as ceil(R/2)*2 and halves `offset = local/2; offset >>= 1`,
 * which only visits every element when that size is a power of two; the evident intent (a full
 * pairwise tree over zero-padded lanes) is what is restated: local = next power of two >= R.
 * Input is [vec, red] with element strides (rs, cs); output dense [vec]. */
void ref_reduce_sum(const float *a, int64_t rs, int64_t cs, float *out, int64_t vec, int64_t red)
{
    int64_t local = 1;
    while (local < red) local <<= 1;
#pragma omp parallel
    {
        float *scratch = (float *)malloc(sizeof(float) * (size_t)local);
#pragma omp for schedule(static)
        for (int64_t x = 0; x < vec; ++x) {
            for (int64_t y = 0; y < local; ++y)
                scratch[y] = (y < red) ? a[x * rs + y * cs] : 0.0f;
            for (int64_t offset = local / 2; offset > 0; offset >>= 1)
                for (int64_t y = 0; y < offset; ++y)
                    scratch[y] += scratch[y + offset];
            out[x] = scratch[0];
        }
        free(scratch);
    }
}

/* Unary kernels, one work-item per element: reference src/devices/opencl/kernels/unary.rs:4-17.
 * op: 0 exp2, 1 log2, 2 sin, 3 neg, 4 recip (1.0/x), 5 sqrt(fabs(x)), 6 ==0, 7 >0, 8 <0. */
void ref_unary(int op, const float *a, float *res, int64_t n)
{
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < n; ++g) {
        float x = a[g], r;
        switch (op) {
        case 0: r = exp2f(x); break;
        case 1: r = log2f(x); break;
        case 2: r = sinf(x); break;
        case 3: r = -x; break;
        case 4: r = (float)(1.0 / (double)x); break; /* `1.0/x` is a double expression in OpenCL C */
        case 5: r = sqrtf(fabsf(x)); break;
        case 6: r = (x == 0.0f) ? 1.0f : 0.0f; break;
        case 7: r = (x > 0.0f) ? 1.0f : 0.0f; break;
        default: r = (x < 0.0f) ? 1.0f : 0.0f; break;
        }
        res[g] = r;
    }
}

/* Binary kernels: reference src/devices/opencl/kernels/binary.rs:3-14.  op: 0 add, 1 multiply.
 * Either operand may be an inline constant (stride 0 with a one-element array). */
void ref_binary(int op, const float *a, int64_t a_stride, const float *b, int64_t b_stride, float *res, int64_t n)
{
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < n; ++g) {
        float x = a[g * a_stride], y = b[g * b_stride];
        res[g] = op ? x * y : x + y;
    }
}

int ref_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

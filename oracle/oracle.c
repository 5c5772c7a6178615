/*
 * oracle.c -- CPU restatement of ManagedLlama2's quantized batch-1 decode path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker that the HIP library is
 * compared against; nothing in the shipped library links, loads or calls it.
 * Only the test-suite, the smoke check and the CPU-baseline leg of the
 * benchmark use it.
 *
 * Two families of functions:
 *
 *   ref_*  -- line-for-line restatements of the reference's own C# CPU code
 *             (HostQWeight.Pack/Unpack and the xUnit tests' `Expected`
 *             loops): single-threaded, fp32 sequential accumulation,
 *             dequantised weights rounded to fp16, results rounded to fp16.
 *             These are also what the benchmark times as the CPU baseline.
 *
 *   f64_*  -- closed-form fp64 "dequantise-then-dot" versions of the same
 *             operators on the layout the reference's GPU kernels and model
 *             loader use (per-row padded zero words).  OpenMP over output
 *             rows.  These are the tolerance oracle (max rel. err 2e-3).
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the reference checkout).
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   qweight unpack ........ reference golden vector test/QWeightTestData.cs
 *                           (128 words, 8 scales, zero word 1770678440 ->
 *                           1024 fp32 bit patterns), bit-exact
 *   qweight pack .......... the six (range, scale, zero) round-trip cases of
 *                           test/QWeightTests.cs:9-18
 *   int4 GEMV family ...... integer regime (scale 1, zero 0: exact integer
 *                           matrix product, numpy int64), brute force on
 *                           128x128, linearity, residual-minus-plain,
 *                           fused==separate, per-row zero padding at
 *                           K=11008/13824
 *   fp16 GEMV / strided /
 *   vec-mat ............... numpy fp64 matmul on strided views
 *   softmax ............... rows sum to 1, shift invariance, two-point closed
 *                           form
 *   rmsnorm ............... the reference's inline vectors
 *                           test/RMSNormTests.cs:64-65 against hand-computed
 *                           closed forms
 *   rope .................. identity at pos 0, norm preservation, known angle
 *                           (pos*freq = pi/2 swaps a pair)
 *   argmax ................ numpy.argmax (first maximum)
 *   softmax_logits ........ two-point closed form, temperature scaling law
 *                           softmax(x/T), rows sum to 1, indices = 0..n-1
 *   sort .................. numpy stable argsort of the negated keys, python
 *                           sorted() on small inputs, permutation check
 *   cumulative_sum ........ numpy integer cumsum (exact regime of
 *                           test/CumulativeSumTests.cs:51-57), fp64 cumsum
 *   sample_top_p .......... brute force over all thresholds on small inputs
 *   sample ................ composition, checked against the empirical
 *                           distribution for a 4-token vocabulary
 *   repack_qdata .......... an integer matrix packed the way AWQ's GEMM
 *                           packer is published (column 8c+orderMap[i] in
 *                           nibble i), repacked, then unpacked by the
 *                           golden-pinned unpack: the matrix comes back; the
 *                           spill-over nibbles of ragged heights by brute force
 *   repack_scales ......... numpy transpose
 *   forward ............... composition checked module by module
 * Parity unpinned: the fp32 summation ORDER of the reference's CUB
 * warp/block reductions (it only matters below fp16 rounding and the
 * reference's own tests pin results to fp16 equality on tiny inputs only).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ */
/* fp16 <-> fp32, IEEE round-to-nearest-even (what C#'s (Half)x and     */
/* (float)h do; src/Extensions.cs:8-15).                                */
/* ------------------------------------------------------------------ */
static inline float h2f(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; ++e; } while (!(man & 0x400u));
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static inline uint16_t f2h(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax = x & 0x7FFFFFFFu;
    if (ax >= 0x7F800000u) /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | ((ax > 0x7F800000u) ? 0x200u : 0));
    if (ax >= 0x477FF000u) /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7C00u);
    if (ax < 0x33000001u) /* < 2^-25 (or exactly 2^-25, ties to even 0) */
        return sign;
    int32_t e = (int32_t)(ax >> 23) - 127;
    uint32_t man = (ax & 0x7FFFFFu) | 0x800000u;
    int shift;
    uint32_t base;
    if (e < -14) { /* subnormal result */
        shift = 13 + (-14 - e);
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        man &= 0x7FFFFFu;
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u)))
        ++q; /* may carry into the exponent, which is the right answer */
    return (uint16_t)(sign | (base + q));
}

/* double -> fp16 with a single rounding (used by the f64 oracle outputs). */
static inline uint16_t d2h(double d)
{
    uint64_t x;
    memcpy(&x, &d, 8);
    uint16_t sign = (uint16_t)((x >> 48) & 0x8000u);
    uint64_t ax = x & 0x7FFFFFFFFFFFFFFFull;
    if (ax >= 0x7FF0000000000000ull)
        return (uint16_t)(sign | 0x7C00u | ((ax > 0x7FF0000000000000ull) ? 0x200u : 0));
    int e = (int)(ax >> 52) - 1023;
    if (e > 15)
        return (uint16_t)(sign | 0x7C00u);
    if (e < -25)
        return sign;
    uint64_t man = (ax & 0xFFFFFFFFFFFFFull) | (1ull << 52);
    int shift;
    uint32_t base;
    if (e < -14) {
        shift = 42 + (-14 - e);
        base = 0;
    } else {
        shift = 42;
        base = (uint32_t)(e + 15) << 10;
        man &= 0xFFFFFFFFFFFFFull;
    }
    uint64_t q = man >> shift;
    uint64_t rem = man & ((1ull << shift) - 1ull);
    uint64_t halfway = 1ull << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1ull)))
        ++q;
    uint32_t r = base + (uint32_t)q;
    if (r >= 0x7C00u)
        r = 0x7C00u;
    return (uint16_t)(sign | r);
}

ORACLE_API float oracle_h2f(uint16_t h) { return h2f(h); }
ORACLE_API uint16_t oracle_f2h(float f) { return f2h(f); }
ORACLE_API uint16_t oracle_d2h(double d) { return d2h(d); }

ORACLE_API void oracle_set_threads(int n)
{
#ifdef _OPENMP
    omp_set_num_threads(n > 0 ? n : 1);
#else
    (void)n;
#endif
}

/* ------------------------------------------------------------------ */
/* Tensor sizes of one int4 row: src/TransformerWeights.cs:54-59,       */
/* src/MatVecResidual.cs:15-19.                                         */
/* ------------------------------------------------------------------ */
static inline int ceil_div(int a, int b) { return (a + (b - 1)) / b; }

ORACLE_API void oracle_qweight_sizes(int K, int* weights_size, int* scales_size, int* zeros_size)
{
    int ss = ceil_div(K, 128);
    *scales_size = ss;
    *weights_size = ceil_div(K, 32) * 4;
    *zeros_size = ceil_div(ss, 8);
}

/* ------------------------------------------------------------------ */
/* ref_qweight_unpack -- HostQWeight.Unpack, src/QWeight.cs:29-54.      */
/* Flat layout: n_words uint32 of nibbles, n_words/16 scales,           */
/* ceil(n_words/128) zero words; output n_words*8 fp16.                 */
/* The C# shift `>> (sIndex * nBits)` masks its count to 5 bits.        */
/* ------------------------------------------------------------------ */
ORACLE_API void ref_qweight_unpack(const uint32_t* W, const uint32_t* Z, const uint16_t* S,
                                   int n_words, uint16_t* out)
{
    const int iSize = 8, wSize = 4, zSize = 32, nBits = 4;
    const uint32_t mask = 0xF;
    int xSize = n_words / wSize;
    for (int x = 0; x < xSize; ++x) {
        int zIndex = x / zSize;
        int sIndex = x / wSize;
        int wIndex = x * wSize;
        int zero = (int)((Z[zIndex] >> ((sIndex * nBits) & 31)) & mask);
        float scale = h2f(S[sIndex]);
        for (int w = 0; w < wSize; ++w) {
            uint32_t weight = W[wIndex + w];
            int oIndex = wIndex * iSize + w * iSize;
            for (int i = 0; i < iSize; ++i) {
                int element = (int)((weight >> (i * nBits)) & mask);
                out[oIndex + i] = f2h((float)(element - zero) * scale);
            }
        }
    }
}

/* ------------------------------------------------------------------ */
/* ref_qweight_pack -- HostQWeight.Pack, src/QWeight.cs:56-92.          */
/* data: n_values fp16; scales/zeros: one per 128-group (n_groups).     */
/* Outputs: W[n_values/8], Z[n_values/8/128 (at least n_groups/8)],     */
/* S[n_values/128].                                                     */
/* ------------------------------------------------------------------ */
ORACLE_API void ref_qweight_pack(const uint16_t* data, int n_values, const float* scales,
                                 const uint32_t* zeros, int n_groups,
                                 uint32_t* W, uint32_t* Z, uint16_t* S)
{
    const int iSize = 8, wSize = 4, nBits = 4;
    const uint32_t mask = 0xF;
    (void)n_values;
    for (int i = 0; i < n_groups / iSize; ++i) {
        uint32_t combined = 0;
        int zIndex = i * iSize;
        for (int z = 0; z < iSize; ++z)
            combined |= (zeros[zIndex + z] & mask) << (z * nBits);
        Z[i] = combined;
    }
    int sSize = n_groups * wSize;
    for (int s = 0; s < sSize; ++s) {
        int sIndex = s / wSize;
        int wIndex = s * wSize;
        float scale = scales[sIndex];
        uint32_t zero = zeros[sIndex];
        for (int w = 0; w < wSize; ++w) {
            uint32_t weight = 0;
            int oIndex = wIndex * iSize + w * iSize;
            for (int i = 0; i < iSize; ++i) {
                /* C#: (uint)(((float)data[o] / scale) + zero); uint promotes to float */
                float v = (h2f(data[oIndex + i]) / scale) + (float)zero;
                uint32_t element = (uint32_t)(int64_t)v;
                weight |= (element & mask) << (i * nBits);
            }
            W[wIndex + w] = weight;
        }
        S[sIndex] = f2h(scale);
    }
}

/* ------------------------------------------------------------------ */
/* Row-padded layout used by the GPU kernels and the model loader:      */
/* native/mat_vec_kernel.cu:98-134, src/TransformerWeights.cs:54-69.    */
/* Row n owns ws words of nibbles, ss scales and zs zero words; the     */
/* zero of group g is nibble g%8 of Z[n*zs + g/8].                      */
/* ------------------------------------------------------------------ */
static inline int nib(uint32_t w, int i) { return (int)((w >> (4 * i)) & 0xFu); }

/* One row dequantised the way HostQWeight.Unpack does it (fp32 product, */
/* rounded to fp16): src/QWeight.cs:46-53 applied to a single row.      */
static void ref_unpack_row(const uint32_t* Wr, const uint32_t* Zr, const uint16_t* Sr,
                           int K, uint16_t* out)
{
    for (int k = 0; k < K; ++k) {
        int g = k / 128;
        int zero = nib(Zr[g / 8], g % 8);
        float scale = h2f(Sr[g]);
        int element = nib(Wr[k / 8], k % 8);
        out[k] = f2h((float)(element - zero) * scale);
    }
}

ORACLE_API void ref_qweight_unpack_rows(const uint32_t* W, const uint32_t* Z, const uint16_t* S,
                                        int K, int N, uint16_t* out)
{
    int ws, ss, zs;
    oracle_qweight_sizes(K, &ws, &ss, &zs);
    for (int n = 0; n < N; ++n)
        ref_unpack_row(W + (size_t)n * ws, Z + (size_t)n * zs, S + (size_t)n * ss, K,
                       out + (size_t)n * K);
}

ORACLE_API void f64_dequant_rows(const uint32_t* W, const uint32_t* Z, const uint16_t* S,
                                 int K, int N, double* out)
{
    int ws, ss, zs;
    oracle_qweight_sizes(K, &ws, &ss, &zs);
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n) {
        const uint32_t* Wr = W + (size_t)n * ws;
        const uint32_t* Zr = Z + (size_t)n * zs;
        const uint16_t* Sr = S + (size_t)n * ss;
        for (int k = 0; k < K; ++k) {
            int g = k / 128;
            out[(size_t)n * K + k] =
                (double)(nib(Wr[k / 8], k % 8) - nib(Zr[g / 8], g % 8)) * (double)h2f(Sr[g]);
        }
    }
}

/* ------------------------------------------------------------------ */
/* ref_matvec -- the tests' fp32 mat-vec `Expected`/`MatVec` loop on an  */
/* fp16 matrix stored [d][n] (output-major): test/MatVecTests.cs:41-56, */
/* test/QKVMatVecInt4Tests.cs:64-79.  out_f32[d] (not yet rounded).     */
/* ------------------------------------------------------------------ */
ORACLE_API void ref_matvec_f32(const uint16_t* w, const uint16_t* x, int n, int d, float* out)
{
    for (int i = 0; i < d; ++i) {
        float val = 0.0f;
        for (int j = 0; j < n; ++j)
            val += h2f(w[(size_t)i * n + j]) * h2f(x[j]);
        out[i] = val;
    }
}

/* fp16 classifier GEMV, result rounded to fp16: test/MatVecTests.cs:41-56. */
ORACLE_API void ref_matvec(const uint16_t* w, const uint16_t* x, int n, int d, uint16_t* out)
{
    float* tmp = (float*)malloc(sizeof(float) * (size_t)d);
    ref_matvec_f32(w, x, n, d, tmp);
    for (int i = 0; i < d; ++i)
        out[i] = f2h(tmp[i]);
    free(tmp);
}

/* int4 mat-vec with residual: HostQWeight.Unpack + test/MatVecInt4Tests.cs:48-70. */
/* out holds the residual on entry (fp16) and the result on exit.       */
ORACLE_API void ref_matvec_residual_int4(uint16_t* out, const uint16_t* x, const uint32_t* W,
                                         const uint32_t* Z, const uint16_t* S, int K, int N)
{
    uint16_t* w = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)K * N);
    float* xb2 = (float*)malloc(sizeof(float) * (size_t)N);
    ref_qweight_unpack_rows(W, Z, S, K, N, w);
    ref_matvec_f32(w, x, K, N, xb2);
    for (int i = 0; i < N; ++i)
        out[i] = f2h(h2f(out[i]) + xb2[i]);
    free(w);
    free(xb2);
}

/* plain int4 mat-vec (one of q/k/v): test/QKVMatVecInt4Tests.cs:64-87. */
ORACLE_API void ref_matvec_int4(uint16_t* out, const uint16_t* x, const uint32_t* W,
                                const uint32_t* Z, const uint16_t* S, int K, int N)
{
    uint16_t* w = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)K * N);
    ref_qweight_unpack_rows(W, Z, S, K, N, w);
    ref_matvec(w, x, K, N, out);
    free(w);
}

/* fused gate/up + SiLU*mul: test/SwiGLUMatVecInt4Tests.cs:55-92. */
ORACLE_API void ref_matvec_swiglu(uint16_t* out, const uint16_t* x,
                                  const uint32_t* Wg, const uint32_t* Zg, const uint16_t* Sg,
                                  const uint32_t* Wu, const uint32_t* Zu, const uint16_t* Su,
                                  int K, int N)
{
    uint16_t* w = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)K * N);
    float* g = (float*)malloc(sizeof(float) * (size_t)N);
    float* u = (float*)malloc(sizeof(float) * (size_t)N);
    ref_qweight_unpack_rows(Wg, Zg, Sg, K, N, w);
    ref_matvec_f32(w, x, K, N, g);
    ref_qweight_unpack_rows(Wu, Zu, Su, K, N, w);
    ref_matvec_f32(w, x, K, N, u);
    for (int i = 0; i < N; ++i) {
        float val = g[i];
        val *= 1.0f / (1.0f + expf(-val));
        val *= u[i];
        out[i] = f2h(val);
    }
    free(w);
    free(g);
    free(u);
}

/* attention scores: test/MatVecStridedTests.cs:43-72 (n_kv_heads == n_heads). */
/* att[h*seq_len + t], k rows of kv_dim halfs starting at k.            */
ORACLE_API void ref_matvec_strided(uint16_t* att, const uint16_t* q, const uint16_t* k,
                                   int dim, int n_heads, int n_kv_heads, int seq_len)
{
    int head_size = dim / n_heads;
    float scale = 1.0f / sqrtf((float)head_size);
    int kv_dim = dim * n_kv_heads / n_heads;
    int kv_mul = n_heads / n_kv_heads;
    for (int h = 0; h < n_heads; ++h) {
        int _q = h * head_size;
        int _att = h * seq_len;
        for (int t = 0; t < seq_len; ++t) {
            size_t _k = (size_t)t * kv_dim + (size_t)(h / kv_mul) * head_size;
            float score = 0.0f;
            for (int i = 0; i < head_size; ++i)
                score += h2f(q[_q + i]) * h2f(k[_k + i]);
            score *= scale;
            att[_att + t] = f2h(score);
        }
    }
}

/* weighted sum of values: test/VecMatTests.cs:44-73. out[dim]. */
ORACLE_API void ref_vecmat(uint16_t* out, const uint16_t* att, const uint16_t* v,
                           int dim, int n_heads, int n_kv_heads, int seq_len)
{
    int head_size = dim / n_heads;
    int kv_dim = dim * n_kv_heads / n_heads;
    int kv_mul = n_heads / n_kv_heads;
    float* xb = (float*)calloc((size_t)dim, sizeof(float));
    for (int h = 0; h < n_heads; ++h) {
        int _xb = h * head_size;
        int _att = h * seq_len;
        for (int t = 0; t < seq_len; ++t) {
            size_t _v = (size_t)t * kv_dim + (size_t)(h / kv_mul) * head_size;
            float a = h2f(att[_att + t]);
            for (int i = 0; i < head_size; ++i)
                xb[_xb + i] += a * h2f(v[_v + i]);
        }
    }
    for (int i = 0; i < dim; ++i)
        out[i] = f2h(xb[i]);
    free(xb);
}

/* softmax of one row, in place: test/SoftmaxTests.cs:31-59. */
ORACLE_API void ref_softmax(uint16_t* x1, int size)
{
    if (size <= 0)
        return;
    float* x = (float*)malloc(sizeof(float) * (size_t)size);
    for (int i = 0; i < size; ++i)
        x[i] = h2f(x1[i]);
    float max_val = x[0];
    for (int i = 1; i < size; ++i)
        if (x[i] > max_val)
            max_val = x[i];
    float sum = 0.0f;
    for (int i = 0; i < size; ++i) {
        x[i] = expf(x[i] - max_val);
        sum += x[i];
    }
    for (int i = 0; i < size; ++i)
        x1[i] = f2h(x[i] / sum);
    free(x);
}

/* RMSNorm: test/RMSNormTests.cs:34-51.  NB the C# reference squares in  */
/* Half (`input[i] * input[i]` is a Half product, rounded to fp16)       */
/* before widening; the GPU kernel (native/rmsnorm_kernel.cu:11-17)      */
/* squares in fp32.  `square_in_half` selects which.                     */
ORACLE_API void ref_rmsnorm(uint16_t* out, const uint16_t* input, const uint16_t* gamma,
                            int size, float eps, int square_in_half)
{
    float ss = 0.0f;
    for (int i = 0; i < size; ++i) {
        float v = h2f(input[i]);
        ss += square_in_half ? h2f(f2h(v * v)) : v * v;
    }
    ss /= (float)size;
    ss += eps;
    ss = 1.0f / sqrtf(ss);
    for (int i = 0; i < size; ++i)
        out[i] = f2h(h2f(gamma[i]) * (ss * h2f(input[i])));
}

/* RoPE, rotate-half pairing (i, i+head_size/2): test/RoPETests.cs:42-83, */
/* native/rope_kernel.cu:3-26.  k points at the row to rotate.          */
ORACLE_API void ref_rope(uint16_t* q, uint16_t* k, int dim, int n_heads, int n_kv_heads,
                         int pos, float theta)
{
    int kv_dim = dim * n_kv_heads / n_heads;
    int head_size = dim / n_heads;
    int size = head_size / 2;
    for (int h = 0; h < n_heads; ++h) {
        for (int t = 0; t < size; ++t) {
            int i = h * head_size + t;
            int j = size + i;
            int head_dim = i * 2 % head_size;
            float freq = 1.0f / powf(theta, (float)head_dim / (float)head_size);
            float val = (float)pos * freq;
            float fci = sinf(val);
            float fcr = cosf(val);
            float v0 = h2f(q[i]), v1 = h2f(q[j]);
            q[i] = f2h(v0 * fcr - v1 * fci);
            q[j] = f2h(v0 * fci + v1 * fcr);
            if (i < kv_dim) {
                v0 = h2f(k[i]);
                v1 = h2f(k[j]);
                k[i] = f2h(v0 * fcr - v1 * fci);
                k[j] = f2h(v0 * fci + v1 * fcr);
            }
        }
    }
}

/* first maximum with strict '>': test/ArgmaxTests.cs:33-46. */
ORACLE_API int ref_argmax(const uint16_t* logits, int n)
{
    int max_i = 0;
    float max_p = h2f(logits[0]);
    for (int i = 1; i < n; ++i) {
        float v = h2f(logits[i]);
        if (v > max_p) {
            max_i = i;
            max_p = v;
        }
    }
    return max_i;
}

/* table row copy: native/embedding_kernel.cu:3-12, test/EmbeddingTableTests.cs:40-50. */
ORACLE_API void ref_embedding(uint16_t* x, const uint16_t* table, int dim, const int* tokens, int pos)
{
    memcpy(x, table + (size_t)tokens[pos] * dim, sizeof(uint16_t) * (size_t)dim);
}

/* ================================================================== */
/* Stochastic sampler: src/Sampler.cs:48-67 and its four kernels.        */
/* ================================================================== */

/* SoftmaxLogits, in place: test/SoftmaxLogitsTests.cs:33-73; the same    */
/* three roundings to fp16 as native/softmax_logits_kernel.cu:12-53       */
/* (after the temperature division, after expf, after the normalisation); */
/* the sum runs over the unrounded exponentials.                          */
ORACLE_API void ref_softmax_logits(uint16_t* logits, int size, float temperature, int* indices)
{
    for (int i = 0; i < size; ++i) {
        indices[i] = i;
        float val = h2f(logits[i]);
        val /= temperature;
        logits[i] = f2h(val);
    }
    float max_val = h2f(logits[0]);
    for (int i = 1; i < size; ++i)
        if (h2f(logits[i]) > max_val)
            max_val = h2f(logits[i]);
    float sum = 0.0f;
    for (int i = 0; i < size; ++i) {
        float v = expf(h2f(logits[i]) - max_val);
        logits[i] = f2h(v);
        sum += v;
    }
    for (int i = 0; i < size; ++i)
        logits[i] = f2h(h2f(logits[i]) / sum);
}

/* Sort, descending by key, values carried along: test/SortTests.cs:38-43 */
/* (Array.Sort with a descending comparer).  The kernel is a radix sort   */
/* (native/sort_kernel.cu:28, cub::BlockRadixSort::SortDescending), which */
/* is STABLE; .NET's Array.Sort is not, which is why the reference's test */
/* leaves the indices unchecked (test/SortTests.cs:88-89).  This is the   */
/* stable sort: equal keys keep their input order.  Keys are ordered by   */
/* the radix sort's total order on fp16 bit patterns (+0 before -0, NaNs  */
/* at the two ends), which is the numeric order for everything else.      */
static inline uint32_t sort_rank(uint16_t k) /* larger rank = sorts first */
{
    return (k & 0x8000u) ? (uint32_t)(uint16_t)~k : (uint32_t)(k | 0x8000u);
}

ORACLE_API void ref_sort(uint16_t* keys, int* values, int size)
{
    size_t* start = (size_t*)calloc(65537, sizeof(size_t));
    uint16_t* k2 = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)size);
    int* v2 = (int*)malloc(sizeof(int) * (size_t)size);
    for (int i = 0; i < size; ++i)
        start[65535 - sort_rank(keys[i]) + 1]++; /* bucket 0 = largest key */
    for (int b = 0; b < 65536; ++b)
        start[b + 1] += start[b];
    for (int i = 0; i < size; ++i) {
        size_t at = start[65535 - sort_rank(keys[i])]++;
        k2[at] = keys[i];
        v2[at] = values[i];
    }
    memcpy(keys, k2, sizeof(uint16_t) * (size_t)size);
    memcpy(values, v2, sizeof(int) * (size_t)size);
    free(start);
    free(k2);
    free(v2);
}

/* CumulativeSum, in place: test/CumulativeSumTests.cs:37-49 (fp32 running */
/* sum, every prefix rounded to fp16).                                    */
ORACLE_API void ref_cumulative_sum(uint16_t* values, int size)
{
    float cdf = 0.0f;
    for (int i = 0; i < size; ++i) {
        cdf += h2f(values[i]);
        values[i] = f2h(cdf);
    }
}

/* SampleTopP: test/SampleTopPTests.cs:34-46 (first index whose value     */
/* reaches the threshold, the last index if none does).                   */
ORACLE_API int ref_sample_top_p(const uint16_t* logits, const int* indices, int size, float threshold)
{
    int min_index = size - 1;
    for (int i = 0; i < size; ++i)
        if (h2f(logits[i]) >= threshold && i < min_index)
            min_index = i;
    return indices[min_index];
}

/* Sampler.Sample: src/Sampler.cs:40-70.  `logits` and `indices` are      */
/* overwritten like runstate.logits / runstate.indices.  Returns the      */
/* token; generate_token == 0 returns -1 (the prompt token stays).        */
ORACLE_API int ref_argmax(const uint16_t* logits, int n);
ORACLE_API int ref_sample(uint16_t* logits, int* indices, int size, float temperature, float top_p,
                          float coin, int generate_token)
{
    if (!generate_token)
        return -1;
    if (temperature == 0.0f)
        return ref_argmax(logits, size);
    ref_softmax_logits(logits, size, temperature, indices);
    float threshold;
    if (top_p <= 0 || top_p >= 1) {
        threshold = coin;
    } else {
        ref_sort(logits, indices, size);
        threshold = coin * top_p;
    }
    ref_cumulative_sum(logits, size);
    return ref_sample_top_p(logits, indices, size, threshold);
}

/* The uniform number in [0, 1) a device-resident sampling loop draws for */
/* position `pos` from `seed` (splitmix64 of seed + pos, top 24 bits).    */
/* The reference draws from an unseeded System.Random (src/Sampler.cs:24, */
/* 42), so any uniform stream is as good as its own.                      */
ORACLE_API float oracle_coin(uint64_t seed, int pos)
{
    uint64_t z = seed + 0x9E3779B97F4A7C15ull * (uint64_t)(pos + 1);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (float)(z >> 40) * (1.0f / 16777216.0f);
}

/* ================================================================== */
/* Converter repack (the data format on the other side of the loader):   */
/* src/ModelConverter.cs:196-328.                                        */
/* ================================================================== */

/* RepackQData, src/ModelConverter.cs:277-317, line for line.  `in` is    */
/* the AWQ "GEMM" tensor [height][width/8] of uint32: nibble i of a word  */
/* holds column 8*(word index) + orderMap[i] (orderMap :19).  `out` is    */
/* [width][ceil(height/8)]: word y/8 of row x holds rows y..y+7 of column */
/* x.  When height is not a multiple of 8 (the zero points: height =      */
/* number of groups) the last word of a row picks up the first elements   */
/* of the NEXT column from the intermediate array (zero behind the last   */
/* column): those nibbles are don't-care for the kernels but they are     */
/* part of the file the reference writes, so they are reproduced.         */
ORACLE_API void ref_repack_qdata(const uint32_t* q_weight_in, int height, int width, uint32_t* q_weight_out)
{
    static const int orderMap[8] = {0, 2, 4, 6, 1, 3, 5, 7};
    uint32_t* packed = (uint32_t*)calloc((size_t)width * height + 8, sizeof(uint32_t));
    uint32_t q[8];
    for (int y = 0; y < height; ++y)
        for (int x = 0; x < width; x += 8) {
            size_t offset = (size_t)height * x + y;
            uint32_t packed_q_wt = q_weight_in[((size_t)y * width + x) / 8];
            for (int i = 0; i < 8; ++i) {
                q[orderMap[i]] = packed_q_wt & 0xF;
                packed_q_wt >>= 4;
            }
            for (int i = 0; i < 8; ++i)
                packed[offset + (size_t)height * i] = q[i];
        }
    int packed_wt_height = ceil_div(height, 8);
    for (int x = 0; x < width; ++x)
        for (int y = 0; y < height; y += 8) {
            size_t offset = (size_t)height * x + y;
            uint32_t packed_val = 0;
            for (int i = 0; i < 8; ++i)
                packed_val |= packed[offset + i] << (4 * i);
            q_weight_out[(size_t)x * packed_wt_height + y / 8] = packed_val;
        }
    free(packed);
}

/* RepackScales, src/ModelConverter.cs:319-328: [meta_height][width] ->   */
/* [width][meta_height].                                                  */
ORACLE_API void ref_repack_scales(const uint16_t* scales_in, int meta_height, int width, uint16_t* packed)
{
    for (int x = 0; x < width; ++x)
        for (int y = 0; y < meta_height; ++y)
            packed[(size_t)x * meta_height + y] = scales_in[(size_t)y * width + x];
}

/* Format.v1 scales, src/ModelConverter.cs:247-262: rows of               */
/* zeros_size*8 halfs compacted to rows of scales_size halfs.             */
ORACLE_API void ref_compact_scales_v1(const uint16_t* scales, int scales_size, int width, uint16_t* scales_t)
{
    int original_height = ceil_div(scales_size, 8) * 8;
    for (int x = 0; x < width; ++x)
        for (int y = 0; y < scales_size; ++y)
            scales_t[(size_t)x * scales_size + y] = scales[(size_t)x * original_height + y];
}

/* ================================================================== */
/* fp64 closed forms.  Outputs are double (pre-rounding) so a test can  */
/* apply its own error metric; *_h helpers round once to fp16.          */
/* ================================================================== */

/* y[n] = sum_k x[k] * (w-z)*s on the row-padded layout. */
ORACLE_API void f64_matvec_int4(double* y, const uint16_t* x, const uint32_t* W, const uint32_t* Z,
                                const uint16_t* S, int K, int N)
{
    int ws, ss, zs;
    oracle_qweight_sizes(K, &ws, &ss, &zs);
    double* xd = (double*)malloc(sizeof(double) * (size_t)K);
    for (int k = 0; k < K; ++k)
        xd[k] = (double)h2f(x[k]);
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n) {
        const uint32_t* Wr = W + (size_t)n * ws;
        const uint32_t* Zr = Z + (size_t)n * zs;
        const uint16_t* Sr = S + (size_t)n * ss;
        double acc = 0.0;
        for (int g = 0; g < ss; ++g) {
            int zero = nib(Zr[g / 8], g % 8);
            double scale = (double)h2f(Sr[g]);
            int k1 = (g + 1) * 128 < K ? (g + 1) * 128 : K;
            double part = 0.0;
            for (int k = g * 128; k < k1; ++k)
                part += xd[k] * (double)(nib(Wr[k / 8], k % 8) - zero);
            acc += part * scale;
        }
        y[n] = acc;
    }
    free(xd);
}

ORACLE_API void f64_matvec_f16(double* y, const uint16_t* x, const uint16_t* M, int K, int N)
{
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n) {
        double acc = 0.0;
        const uint16_t* row = M + (size_t)n * K;
        for (int k = 0; k < K; ++k)
            acc += (double)h2f(row[k]) * (double)h2f(x[k]);
        y[n] = acc;
    }
}

/* att[h*o_stride + t] = alpha * sum_r q[h*v_stride + r] * Km[t*m_row_stride + h*m_col_stride + r] */
/* (argument meaning of native/mat_vec_kernel.cu:51-76). */
ORACLE_API void f64_matvec_strided(double* att, const uint16_t* q, const uint16_t* Km, int rows,
                                   int cols, int v_stride, int m_col_stride, int m_row_stride,
                                   int o_stride, double alpha, int n_heads)
{
#pragma omp parallel for schedule(static)
    for (int h = 0; h < n_heads; ++h)
        for (int t = 0; t < cols; ++t) {
            double acc = 0.0;
            for (int r = 0; r < rows; ++r)
                acc += (double)h2f(q[(size_t)h * v_stride + r]) *
                       (double)h2f(Km[(size_t)t * m_row_stride + (size_t)h * m_col_stride + r]);
            att[(size_t)h * o_stride + t] = acc * alpha;
        }
}

/* out[h*o_stride + r] = sum_t att[h*cols + t] * V[t*m_row_stride + h*m_col_stride + r] */
/* (native/vec_mat_kernel.cu:8-42). */
ORACLE_API void f64_vecmat(double* out, const uint16_t* att, const uint16_t* V, int rows, int cols,
                           int m_col_stride, int o_stride, int m_row_stride, int n_heads)
{
#pragma omp parallel for schedule(static)
    for (int h = 0; h < n_heads; ++h)
        for (int r = 0; r < rows; ++r) {
            double acc = 0.0;
            for (int t = 0; t < cols; ++t)
                acc += (double)h2f(att[(size_t)h * cols + t]) *
                       (double)h2f(V[(size_t)t * m_row_stride + (size_t)h * m_col_stride + r]);
            out[(size_t)h * o_stride + r] = acc;
        }
}

ORACLE_API void f64_softmax(double* out, const uint16_t* x, int size, int n_rows)
{
    for (int r = 0; r < n_rows; ++r) {
        const uint16_t* xr = x + (size_t)r * size;
        double* o = out + (size_t)r * size;
        double m = (double)h2f(xr[0]);
        for (int i = 1; i < size; ++i)
            if ((double)h2f(xr[i]) > m)
                m = (double)h2f(xr[i]);
        double sum = 0.0;
        for (int i = 0; i < size; ++i) {
            o[i] = exp((double)h2f(xr[i]) - m);
            sum += o[i];
        }
        for (int i = 0; i < size; ++i)
            o[i] /= sum;
    }
}

/* SoftmaxLogits with exact exp and sum.  The two fp16 roundings that the */
/* in-place buffer forces on the INPUT of later steps are kept: the       */
/* temperature division (fp32, correctly rounded, then fp16) and the fp16 */
/* exponential that is normalised.  out = double(half(e)) / sum(e).       */
ORACLE_API void f64_softmax_logits(double* out, const uint16_t* logits, int size, float temperature)
{
    double m = -INFINITY;
    for (int i = 0; i < size; ++i) {
        out[i] = (double)h2f(f2h(h2f(logits[i]) / temperature));
        if (out[i] > m)
            m = out[i];
    }
    double sum = 0.0;
    for (int i = 0; i < size; ++i) {
        double e = exp(out[i] - m);
        sum += e;
        out[i] = (double)h2f(d2h(e));
    }
    for (int i = 0; i < size; ++i)
        out[i] /= sum;
}

ORACLE_API void f64_cumulative_sum(double* out, const uint16_t* values, int size)
{
    double cdf = 0.0;
    for (int i = 0; i < size; ++i) {
        cdf += (double)h2f(values[i]);
        out[i] = cdf;
    }
}

ORACLE_API void f64_rmsnorm(double* out, const uint16_t* x, const uint16_t* gamma, int size, double eps)
{
    double ss = 0.0;
    for (int i = 0; i < size; ++i)
        ss += (double)h2f(x[i]) * (double)h2f(x[i]);
    double r = 1.0 / sqrt(ss / (double)size + eps);
    for (int i = 0; i < size; ++i)
        out[i] = r * (double)h2f(gamma[i]) * (double)h2f(x[i]);
}

/* rotate-half RoPE in fp64 on q (n_heads) and k (n_kv_heads); outputs double. */
ORACLE_API void f64_rope(double* qo, double* ko, const uint16_t* q, const uint16_t* k, int n_heads,
                         int n_kv_heads, int head_size, int pos, double theta)
{
    int half_size = head_size / 2;
    for (int h = 0; h < n_heads; ++h)
        for (int t = 0; t < half_size; ++t) {
            int i = h * head_size + t, j = i + half_size;
            double freq = 1.0 / pow(theta, (double)((2 * t) % head_size) / (double)head_size);
            double a = (double)pos * freq, c = cos(a), s = sin(a);
            double v0 = (double)h2f(q[i]), v1 = (double)h2f(q[j]);
            qo[i] = v0 * c - v1 * s;
            qo[j] = v0 * s + v1 * c;
            if (h < n_kv_heads) {
                v0 = (double)h2f(k[i]);
                v1 = (double)h2f(k[j]);
                ko[i] = v0 * c - v1 * s;
                ko[j] = v0 * s + v1 * c;
            }
        }
}

ORACLE_API void oracle_round_d2h(const double* in, uint16_t* out, size_t n)
{
    for (size_t i = 0; i < n; ++i)
        out[i] = d2h(in[i]);
}

/* ================================================================== */
/* One decode step, composed as src/Transformer.cs:158-190 with          */
/* MultiHeadAttention :150-156: each module is evaluated in fp64 and its */
/* output rounded once to fp16, because every buffer between modules is  */
/* fp16 storage in the reference (src/RunState.cs:7-21).                 */
/* ================================================================== */
typedef struct {
    int dim, hidden_dim, n_layers, n_heads, n_kv_heads, vocab_size, seq_len;
    float rope_theta;
} oracle_config; /* src/Config.cs:6-19 */

typedef struct {
    const uint32_t* W;
    const uint32_t* Z;
    const uint16_t* S;
} oracle_qweight; /* src/QWeight.cs:5-10 */

typedef struct {
    oracle_qweight q, k, v, o, gate, up, down;
    const uint16_t* rms_att;
    const uint16_t* rms_ffn;
} oracle_layer; /* src/PerLayerWeight.cs:5-16 */

typedef struct {
    const uint16_t* embedding;
    const uint16_t* classifier;
    const uint16_t* rms_final;
    const oracle_layer* layers;
} oracle_weights; /* src/TransformerWeights.cs:8-14 */

typedef struct {
    uint16_t *x, *xb, *h, *q, *att, *logits, *key_cache, *value_cache;
    int* tokens;
} oracle_runstate; /* src/RunState.cs:7-25 */

static void mv4_h(uint16_t* out, const uint16_t* x, const oracle_qweight* w, int K, int N,
                  int residual, double* tmp)
{
    f64_matvec_int4(tmp, x, w->W, w->Z, w->S, K, N);
    for (int i = 0; i < N; ++i)
        out[i] = d2h(residual ? tmp[i] + (double)h2f(out[i]) : tmp[i]);
}

ORACLE_API void f64_forward(const oracle_config* c, const oracle_weights* w, oracle_runstate* s,
                            int position, int next_position)
{
    int dim = c->dim, hd = c->hidden_dim;
    int head_size = dim / c->n_heads;
    int kv_dim = dim * c->n_kv_heads / c->n_heads;
    double scale = 1.0 / sqrt((double)head_size);
    int big = hd > dim ? hd : dim;
    if (c->vocab_size > big)
        big = c->vocab_size;
    if (c->n_heads * next_position > big)
        big = c->n_heads * next_position;
    double* tmp = (double*)malloc(sizeof(double) * (size_t)big);
    double* tmp2 = (double*)malloc(sizeof(double) * (size_t)big);

    ref_embedding(s->x, w->embedding, dim, s->tokens, position); /* Transformer.cs:163 */
    for (int l = 0; l < c->n_layers; ++l) {
        const oracle_layer* L = &w->layers[l];
        f64_rmsnorm(tmp, s->x, L->rms_att, dim, 1e-5); /* :167 */
        oracle_round_d2h(tmp, s->xb, (size_t)dim);
        size_t loff = (size_t)l * c->seq_len * kv_dim; /* :169 */
        uint16_t* krow = s->key_cache + loff + (size_t)position * kv_dim;
        uint16_t* vrow = s->value_cache + loff + (size_t)position * kv_dim;
        mv4_h(s->q, s->xb, &L->q, dim, dim, 0, tmp); /* :171 */
        mv4_h(krow, s->xb, &L->k, dim, kv_dim, 0, tmp);
        mv4_h(vrow, s->xb, &L->v, dim, kv_dim, 0, tmp);
        f64_rope(tmp, tmp2, s->q, krow, c->n_heads, c->n_kv_heads, head_size, position,
                 (double)c->rope_theta); /* :173 */
        oracle_round_d2h(tmp, s->q, (size_t)dim);
        oracle_round_d2h(tmp2, krow, (size_t)kv_dim);
        int S = next_position; /* :175, attends rows 0..position */
        f64_matvec_strided(tmp, s->q, s->key_cache + loff, head_size, S, head_size, head_size,
                           kv_dim, S, scale, c->n_heads); /* :153 */
        oracle_round_d2h(tmp, s->att, (size_t)c->n_heads * S);
        f64_softmax(tmp, s->att, S, c->n_heads); /* :154 */
        oracle_round_d2h(tmp, s->att, (size_t)c->n_heads * S);
        f64_vecmat(tmp, s->att, s->value_cache + loff, head_size, S, head_size, head_size, kv_dim,
                   c->n_heads); /* :155 */
        oracle_round_d2h(tmp, s->xb, (size_t)dim);
        mv4_h(s->x, s->xb, &L->o, dim, dim, 1, tmp); /* :177 */
        f64_rmsnorm(tmp, s->x, L->rms_ffn, dim, 1e-5); /* :179 */
        oracle_round_d2h(tmp, s->xb, (size_t)dim);
        f64_matvec_int4(tmp, s->xb, L->gate.W, L->gate.Z, L->gate.S, dim, hd); /* :181 */
        f64_matvec_int4(tmp2, s->xb, L->up.W, L->up.Z, L->up.S, dim, hd);
        for (int i = 0; i < hd; ++i)
            s->h[i] = d2h(tmp[i] / (1.0 + exp(-tmp[i])) * tmp2[i]);
        mv4_h(s->x, s->h, &L->down, hd, dim, 1, tmp); /* :183 */
    }
    f64_rmsnorm(tmp, s->x, w->rms_final, dim, 1e-5); /* :187, in place */
    oracle_round_d2h(tmp, s->x, (size_t)dim);
    f64_matvec_f16(tmp, s->x, w->classifier, dim, c->vocab_size); /* :189 */
    oracle_round_d2h(tmp, s->logits, (size_t)c->vocab_size);
    free(tmp);
    free(tmp2);
}

/* ================================================================== */
/* CPU baseline: the reference's C# CPU path for one decoder layer's     */
/* mat-vec set (Unpack + Expected loops), single thread.                 */
/* q,k,v: K=dim,N=dim; o: residual; gate/up: N=hidden; down: K=hidden.   */
/* ================================================================== */
ORACLE_API void ref_layer_matvec_set(const oracle_layer* L, int dim, int hidden_dim,
                                     const uint16_t* xb, uint16_t* q, uint16_t* k, uint16_t* v,
                                     uint16_t* x, uint16_t* h)
{
    ref_matvec_int4(q, xb, L->q.W, L->q.Z, L->q.S, dim, dim);
    ref_matvec_int4(k, xb, L->k.W, L->k.Z, L->k.S, dim, dim);
    ref_matvec_int4(v, xb, L->v.W, L->v.Z, L->v.S, dim, dim);
    ref_matvec_residual_int4(x, xb, L->o.W, L->o.Z, L->o.S, dim, dim);
    ref_matvec_swiglu(h, xb, L->gate.W, L->gate.Z, L->gate.S, L->up.W, L->up.Z, L->up.S, dim,
                      hidden_dim);
    ref_matvec_residual_int4(x, h, L->down.W, L->down.Z, L->down.S, hidden_dim, dim);
}

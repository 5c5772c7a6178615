// AWQ-v1 int4 (group 128) mat-vec family for gfx950: plain, +residual, fused
// QKV, fused SwiGLU.  Replaces native/mat_vec_kernel.cu:83-234 of the reference.
//
// Shape of the computation (batch-1 GEMV, HBM-bound, no MFMA):
//   * a "chunk" is 16 bytes of one weight row = 4 uint32 = 32 nibbles; a
//     64-lane wavefront reads 64 consecutive chunks (1 KiB) per load
//     instruction, lane l taking chunk j*64+l (global_load_dwordx4);
//   * the input vector is staged once per workgroup in LDS, pre-permuted to
//     the order the nibble extraction produces, in four planes so that
//     consecutive lanes read consecutive 16-byte slots (conflict-free
//     ds_read_b128);
//   * nibbles become fp16 pairs with the exponent-OR trick
//     ((w & 0x000F000F) | 0x6400'6400 = 1024+n), the zero-point is removed
//     exactly in fp16 (v_pk_add_f16 / v_pk_fma_f16), products are accumulated
//     in fp32 with v_dot2_f32_f16, and each chunk's partial sum is multiplied
//     once by its group scale in fp32;
//   * lanes are reduced with DPP row operations, lane 63 owns the total.
#include "common.hpp"

namespace l2 {

constexpr int kWaves = 4;                // wavefronts per workgroup
constexpr int kThreads = kWaves * 64;    // 256
constexpr int kMaxLdsBytes = 64 * 1024;  // static+dynamic LDS we ask for

struct QW {
    const uint32_t* w;
    const uint32_t* z;
    const uint16_t* s;
};

struct Frag { // what one lane holds of one row for one chunk
    u32x4 w;
    uint32_t zword;
    uint16_t sbits;
};

__device__ __forceinline__ Frag load_frag(const QW& m, size_t row, int c, int ws, int ss, int zs, bool valid)
{
    Frag f;
    if (valid) {
        const int g = c >> 2;
        f.w = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(m.w + row * ws) + c);
        f.zword = m.z[row * zs + (g >> 3)];
        f.sbits = m.s[row * ss + g];
    } else {
        f.w = u32x4{0u, 0u, 0u, 0u};
        f.zword = 0u;
        f.sbits = 0;
    }
    return f;
}

// Partial dot product of one chunk (32 elements) of one row.
__device__ __forceinline__ float chunk_dot(const Frag& f, int c, const u32x4 (&x)[4])
{
    const uint32_t z = (f.zword >> (((c >> 2) & 7) * 4)) & 0xFu;
    // -(1024 + z) and -(64 + z) as fp16 pairs: ulp(1024) = 1, ulp(64) = 1/16
    const uint32_t neg_a = 0xE400E400u + z * 0x00010001u;
    const uint32_t neg_b = 0xD400D400u + z * 0x00100010u;
    const h2_t sixteenth = {static_cast<_Float16>(0.0625f), static_cast<_Float16>(0.0625f)};
    float acc0 = 0.0f, acc1 = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t w = f.w[i];
        const uint32_t w8 = w >> 8;
        // (n0,n4) (n1,n5) (n2,n6) (n3,n7), each minus the zero-point, exact in fp16
        const h2_t a0 = as_h2((w & 0x000F000Fu) | 0x64006400u) + as_h2(neg_a);
        const h2_t a1 = __builtin_elementwise_fma(as_h2((w & 0x00F000F0u) | 0x64006400u), sixteenth, as_h2(neg_b));
        const h2_t a2 = as_h2((w8 & 0x000F000Fu) | 0x64006400u) + as_h2(neg_a);
        const h2_t a3 = __builtin_elementwise_fma(as_h2((w8 & 0x00F000F0u) | 0x64006400u), sixteenth, as_h2(neg_b));
        acc0 = __builtin_amdgcn_fdot2(a0, as_h2(x[i][0]), acc0, false);
        acc1 = __builtin_amdgcn_fdot2(a1, as_h2(x[i][1]), acc1, false);
        acc0 = __builtin_amdgcn_fdot2(a2, as_h2(x[i][2]), acc0, false);
        acc1 = __builtin_amdgcn_fdot2(a3, as_h2(x[i][3]), acc1, false);
    }
    return (acc0 + acc1) * half_bits_to_float(f.sbits);
}

// Stage the K-element input in LDS as 4 planes of nchunks 16-byte slots:
// slot (i, c) holds elements 8*(4c+i)+{0,4,1,5,2,6,3,7}; elements >= K are 0.
__device__ __forceinline__ void stage_input(u32x4* xs, const uint16_t* x, int K, int nchunks)
{
    const int nwords = nchunks * 4;
    for (int e = threadIdx.x; e < nwords; e += kThreads) {
        u32x4 in;
        if (8 * e + 8 <= K) {
            in = *reinterpret_cast<const u32x4*>(x + 8 * e);
        } else {
            uint16_t t[8];
#pragma unroll
            for (int i = 0; i < 8; ++i)
                t[i] = (8 * e + i < K) ? x[8 * e + i] : uint16_t(0);
            in = u32x4{uint32_t(t[0]) | (uint32_t(t[1]) << 16), uint32_t(t[2]) | (uint32_t(t[3]) << 16),
                       uint32_t(t[4]) | (uint32_t(t[5]) << 16), uint32_t(t[6]) | (uint32_t(t[7]) << 16)};
        }
        u32x4 out;
        out[0] = (in[0] & 0xFFFFu) | (in[2] << 16);          // x0,x4
        out[1] = (in[0] >> 16) | (in[2] & 0xFFFF0000u);      // x1,x5
        out[2] = (in[1] & 0xFFFFu) | (in[3] << 16);          // x2,x6
        out[3] = (in[1] >> 16) | (in[3] & 0xFFFF0000u);      // x3,x7
        xs[(e & 3) * nchunks + (e >> 2)] = out;
    }
}

// R rows of one wavefront against the staged input; sums valid in every lane.
template <int R>
__device__ __forceinline__ void dot_rows(float (&sum)[R], const QW (&m)[R], const size_t (&row)[R],
                                         const u32x4* xs, const uint16_t* x, int K, int nchunks,
                                         int ws, int ss, int zs)
{
    const int lane = threadIdx.x & 63;
    Frag cur[R];
#pragma unroll
    for (int r = 0; r < R; ++r)
        cur[r] = load_frag(m[r], row[r], lane, ws, ss, zs, lane < nchunks);

    // weight loads are in flight while the input is staged
    stage_input(const_cast<u32x4*>(xs), x, K, nchunks);
    __syncthreads();

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r)
        acc[r] = 0.0f;

    for (int c = lane; c < nchunks + lane; c += 64) { // uniform trip count; c < nchunks masks lanes
        const int cn = c + 64;
        Frag nxt[R];
#pragma unroll
        for (int r = 0; r < R; ++r)
            nxt[r] = load_frag(m[r], row[r], cn, ws, ss, zs, cn < nchunks);
        if (c < nchunks) {
            u32x4 xv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                xv[i] = xs[i * nchunks + c];
#pragma unroll
            for (int r = 0; r < R; ++r)
                acc[r] += chunk_dot(cur[r], c, xv);
        }
#pragma unroll
        for (int r = 0; r < R; ++r)
            cur[r] = nxt[r];
    }
#pragma unroll
    for (int r = 0; r < R; ++r)
        sum[r] = wave_sum(acc[r]);
}

struct PlainArgs {
    QW m[3];
    uint16_t* out[3];
};

// blockIdx.y selects the tensor (1 for plain/residual, 3 for fused QKV);
// each wavefront owns R consecutive output rows.
template <int R, bool RESIDUAL>
__global__ __launch_bounds__(kThreads) void int4_matvec_kernel(PlainArgs a, const uint16_t* x, int K, int N,
                                                               int ws, int ss, int zs)
{
    extern __shared__ u32x4 xs[];
    const int nchunks = ws >> 2;
    const QW m = a.m[blockIdx.y];
    uint16_t* out = a.out[blockIdx.y];
    const int wave = threadIdx.x >> 6;
    const int n0 = (blockIdx.x * kWaves + wave) * R;
    QW ms[R];
    size_t rows[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        ms[r] = m;
        rows[r] = static_cast<size_t>(n0 + r < N ? n0 + r : N - 1);
    }
    float sum[R];
    dot_rows<R>(sum, ms, rows, xs, x, K, nchunks, ws, ss, zs);
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (lane == r && n0 + r < N) {
            float v = sum[r];
            if (RESIDUAL)
                v += half_bits_to_float(out[n0 + r]);
            out[n0 + r] = float_to_half_bits(v);
        }
    }
}

// Each wavefront owns O outputs: rows n of the gate and of the up tensor.
template <int O>
__global__ __launch_bounds__(kThreads) void int4_swiglu_kernel(QW g, QW u, uint16_t* out, const uint16_t* x,
                                                               int K, int N, int ws, int ss, int zs)
{
    extern __shared__ u32x4 xs[];
    const int nchunks = ws >> 2;
    const int wave = threadIdx.x >> 6;
    const int n0 = (blockIdx.x * kWaves + wave) * O;
    QW ms[2 * O];
    size_t rows[2 * O];
#pragma unroll
    for (int o = 0; o < O; ++o) {
        const size_t n = static_cast<size_t>(n0 + o < N ? n0 + o : N - 1);
        ms[2 * o] = g;
        ms[2 * o + 1] = u;
        rows[2 * o] = n;
        rows[2 * o + 1] = n;
    }
    float sum[2 * O];
    dot_rows<2 * O>(sum, ms, rows, xs, x, K, nchunks, ws, ss, zs);
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int o = 0; o < O; ++o) {
        if (lane == o && n0 + o < N) {
            float v = sum[2 * o];
            v *= 1.0f / (1.0f + expf(-v));
            v *= sum[2 * o + 1];
            out[n0 + o] = float_to_half_bits(v);
        }
    }
}

static int check_qweight_call(const char* fn, const void* out, const void* in, int rows, int cols,
                              int zeros_size, int scales_size, int weights_size)
{
    L2_CHECK(out && in, "%s: null activation pointer", fn);
    L2_CHECK(rows > 0 && cols > 0, "%s: rows=%d cols=%d must be positive", fn, rows, cols);
    const int ss = ceil_div(rows, 128), ws = ceil_div(rows, 32) * 4, zs = ceil_div(ss, 8);
    L2_CHECK(scales_size == ss && weights_size == ws && zeros_size == zs,
             "%s: sizes (zeros %d, scales %d, weights %d) do not match rows=%d (expected %d, %d, %d)", fn,
             zeros_size, scales_size, weights_size, rows, zs, ss, ws);
    L2_CHECK(aligned(in, 16), "%s: input must be 16-byte aligned", fn);
    L2_CHECK(aligned(out, 2), "%s: output must be 2-byte aligned", fn);
    if (static_cast<size_t>(ws) * 16 > static_cast<size_t>(kMaxLdsBytes))
        return fail(LLAMA2_ERR_UNSUPPORTED, "%s: rows=%d needs %d bytes of LDS, limit %d", fn, rows, ws * 16,
                    kMaxLdsBytes);
    return LLAMA2_OK;
}

static int check_qweight(const char* fn, const char* name, const uint32_t* w, const uint32_t* z,
                         const llama2_half* s)
{
    L2_CHECK(w && z && s, "%s: null pointer in %s tensor", fn, name);
    L2_CHECK(aligned(w, 16), "%s: %s weights must be 16-byte aligned", fn, name);
    L2_CHECK(aligned(z, 4) && aligned(s, 2), "%s: %s zeros/scales misaligned", fn, name);
    return LLAMA2_OK;
}

template <bool RESIDUAL>
static int launch_plain(const char* fn, int n_tensors, PlainArgs a, const llama2_half* input, int rows, int cols,
                        int zs, int ss, int ws)
{
    constexpr int R = 2;
    const dim3 grid(ceil_div(cols, kWaves * R), n_tensors);
    const size_t lds = static_cast<size_t>(ws) * 16; // nchunks * 64 bytes
    hipLaunchKernelGGL((int4_matvec_kernel<R, RESIDUAL>), grid, dim3(kThreads), lds, ctx().stream, a, input,
                       rows, cols, ws, ss, zs);
    L2_LAUNCH_CHECK(fn);
    return LLAMA2_OK;
}

} // namespace l2

using namespace l2;

extern "C" {

int llama2_mat_vec_residual_int4(llama2_half* output, const llama2_half* input, const uint32_t* weights,
                                 const uint32_t* zeros, const llama2_half* scales, int rows, int cols,
                                 int zeros_size, int scales_size, int weights_size)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_mat_vec_residual_int4";
    if (int rc = check_qweight_call(fn, output, input, rows, cols, zeros_size, scales_size, weights_size))
        return rc;
    if (int rc = check_qweight(fn, "matrix", weights, zeros, scales))
        return rc;
    L2_CHECK(!overlap(output, size_t(cols) * 2, input, size_t(rows) * 2),
             "%s: output overlaps input (other workgroups still read the input while rows are written)", fn);
    PlainArgs a{};
    a.m[0] = QW{weights, zeros, scales};
    a.out[0] = output;
    return launch_plain<true>(fn, 1, a, input, rows, cols, zeros_size, scales_size, weights_size);
}

int llama2_mat_vec_int4(llama2_half* output, const llama2_half* input, const uint32_t* weights,
                        const uint32_t* zeros, const llama2_half* scales, int rows, int cols, int zeros_size,
                        int scales_size, int weights_size)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_mat_vec_int4";
    if (int rc = check_qweight_call(fn, output, input, rows, cols, zeros_size, scales_size, weights_size))
        return rc;
    if (int rc = check_qweight(fn, "matrix", weights, zeros, scales))
        return rc;
    L2_CHECK(!overlap(output, size_t(cols) * 2, input, size_t(rows) * 2), "%s: output overlaps input", fn);
    PlainArgs a{};
    a.m[0] = QW{weights, zeros, scales};
    a.out[0] = output;
    return launch_plain<false>(fn, 1, a, input, rows, cols, zeros_size, scales_size, weights_size);
}

int llama2_qkv_mat_vec(llama2_half* q_output, llama2_half* k_output, llama2_half* v_output,
                       const llama2_half* input, const uint32_t* q_weight, const uint32_t* q_zeros,
                       const llama2_half* q_scales, const uint32_t* k_weight, const uint32_t* k_zeros,
                       const llama2_half* k_scales, const uint32_t* v_weight, const uint32_t* v_zeros,
                       const llama2_half* v_scales, int rows, int cols, int zeros_size, int scales_size,
                       int weights_size)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_qkv_mat_vec";
    if (int rc = check_qweight_call(fn, q_output, input, rows, cols, zeros_size, scales_size, weights_size))
        return rc;
    L2_CHECK(k_output && v_output, "%s: null k/v output", fn);
    if (int rc = check_qweight(fn, "query", q_weight, q_zeros, q_scales))
        return rc;
    if (int rc = check_qweight(fn, "key", k_weight, k_zeros, k_scales))
        return rc;
    if (int rc = check_qweight(fn, "value", v_weight, v_zeros, v_scales))
        return rc;
    for (llama2_half* o : {q_output, k_output, v_output})
        L2_CHECK(!overlap(o, size_t(cols) * 2, input, size_t(rows) * 2), "%s: an output overlaps the input", fn);
    PlainArgs a{};
    a.m[0] = QW{q_weight, q_zeros, q_scales};
    a.m[1] = QW{k_weight, k_zeros, k_scales};
    a.m[2] = QW{v_weight, v_zeros, v_scales};
    a.out[0] = q_output;
    a.out[1] = k_output;
    a.out[2] = v_output;
    return launch_plain<false>(fn, 3, a, input, rows, cols, zeros_size, scales_size, weights_size);
}

int llama2_mat_vec_swiglu(llama2_half* output, const llama2_half* input, const uint32_t* g_weight,
                          const uint32_t* g_zeros, const llama2_half* g_scales, const uint32_t* u_weight,
                          const uint32_t* u_zeros, const llama2_half* u_scales, int rows, int cols,
                          int zeros_size, int scales_size, int weights_size)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_mat_vec_swiglu";
    if (int rc = check_qweight_call(fn, output, input, rows, cols, zeros_size, scales_size, weights_size))
        return rc;
    if (int rc = check_qweight(fn, "gate", g_weight, g_zeros, g_scales))
        return rc;
    if (int rc = check_qweight(fn, "up", u_weight, u_zeros, u_scales))
        return rc;
    L2_CHECK(!overlap(output, size_t(cols) * 2, input, size_t(rows) * 2), "%s: output overlaps input", fn);
    constexpr int O = 1;
    const dim3 grid(ceil_div(cols, kWaves * O));
    const size_t lds = static_cast<size_t>(weights_size) * 16;
    hipLaunchKernelGGL((int4_swiglu_kernel<O>), grid, dim3(kThreads), lds, ctx().stream,
                       QW{g_weight, g_zeros, g_scales}, QW{u_weight, u_zeros, u_scales}, output, input, rows, cols,
                       weights_size, scales_size, zeros_size);
    L2_LAUNCH_CHECK(fn);
    return LLAMA2_OK;
}

} // extern "C"

// AWQ-v1 int4 (group 128) mat-vec family for gfx950: plain, +residual, fused
// QKV, fused SwiGLU.  Replaces native/mat_vec_kernel.cu:83-234 of the reference.
//
// Shape of the computation (batch-1 GEMV, HBM-bound, no MFMA):
//   * a "chunk" is 16 bytes of one weight row = 4 uint32 = 32 nibbles; a
//     64-lane wavefront reads 64 consecutive chunks (1 KiB) per load
//     instruction, lane l taking chunks l, l+64, ... (buffer_load_dwordx4
//     through a per-row buffer resource, so the ragged end of a row reads as
//     zero without any lane predication);
//   * wavefronts are persistent: each walks over its rows with the next row's
//     loads already in flight while the current one is reduced;
//   * the input vector is staged once per workgroup in LDS, pre-permuted to
//     the order the nibble extraction produces, in four planes so that
//     consecutive lanes read consecutive 16-byte slots (conflict-free
//     ds_read_b128), together with the fp32 sum of every 32-element chunk;
//   * a nibble masked in place (w & 0x000F000F, w & 0x00F000F0) IS an fp16
//     subnormal pair (n * 2^-24 resp. n * 2^-20): v_dot2_f32_f16 multiplies it
//     exactly with the fp16 input pair and accumulates in fp32, so dequantising
//     costs one v_and per pair.  The zero-point is applied per chunk as
//     -z * sum(x), the group scale once per chunk, all in fp32;
//   * lanes are reduced with DPP row operations.
#include "common.hpp"

namespace l2 {

struct QW {
    const uint32_t* w;
    const uint32_t* z;
    const uint16_t* s;
};

enum Mode { PLAIN = 0, RESIDUAL = 1, SWIGLU = 2 };

struct Int4Args {
    QW m[3];          // PLAIN/RESIDUAL: m[0] (QKV: q,k,v); SWIGLU: gate, up
    uint16_t* out[3]; // one output vector per tensor (SWIGLU: out[0])
    const uint16_t* x;
    int K, N, ws, ss, zs;
    int n_tensors;
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes)
{
    // raw buffer, 32-bit elements; out-of-range reads return 0
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, static_cast<int>(bytes), 0x00020000);
}

constexpr int kAuxStream = 2; // "nt": weights are touched once

template <int J, int R>
struct Frag { // what one lane holds of R rows: J chunks each + its group's zero word and scale
    u32x4 w[R][J];
    uint32_t zw[R][J];
    uint16_t sb[R][J];
};

template <int J>
__device__ __forceinline__ void load_row(u32x4 (&w)[J], uint32_t (&zw)[J], uint16_t (&sb)[J], const QW& m,
                                         size_t row, int ws, int ss, int zs, int lane)
{
    const __amdgpu_buffer_rsrc_t rw = make_rsrc(m.w + row * ws, ws * 4);
    const __amdgpu_buffer_rsrc_t rz = make_rsrc(m.z + row * zs, zs * 4);
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(m.s + row * ss, ss * 2);
#pragma unroll
    for (int j = 0; j < J; ++j) {
        // chunk c = lane + 64 j: group c/4, zero word c/32
        w[j] = __builtin_amdgcn_raw_buffer_load_b128(rw, lane * 16 + j * 1024, 0, kAuxStream);
        zw[j] = __builtin_amdgcn_raw_buffer_load_b32(rz, (lane >> 5) * 4 + j * 8, 0, 0);
        sb[j] = __builtin_amdgcn_raw_buffer_load_b16(rs, (lane >> 2) * 2 + j * 32, 0, 0);
    }
}

// Stage the input in LDS: xs[i*JC + c] holds elements 8*(4c+i)+{0,4,1,5,2,6,3,7}
// (JC = 64 J chunks, zero beyond K), sx[c] the fp32 sum of chunk c.
template <int J, int T>
struct XStage {
    static constexpr int JC = J * 64;
    static constexpr int XE = (JC * 4 + T - 1) / T;
    u32x4 in[XE];
    __device__ __forceinline__ void issue(const uint16_t* x, int K)
    {
        const __amdgpu_buffer_rsrc_t rx = make_rsrc(x, K * 2);
#pragma unroll
        for (int i = 0; i < XE; ++i)
            in[i] = __builtin_amdgcn_raw_buffer_load_b128(rx, (threadIdx.x + i * T) * 16, 0, 0);
    }
    __device__ __forceinline__ void commit(u32x4* xs, float* sx)
    {
#pragma unroll
        for (int i = 0; i < XE; ++i) {
            const int e = threadIdx.x + i * T;
            if (e < JC * 4) {
                const u32x4 v = in[i];
                u32x4 o;
                o[0] = (v[0] & 0xFFFFu) | (v[2] << 16);     // x0,x4
                o[1] = (v[0] >> 16) | (v[2] & 0xFFFF0000u); // x1,x5
                o[2] = (v[1] & 0xFFFFu) | (v[3] << 16);     // x2,x6
                o[3] = (v[1] >> 16) | (v[3] & 0xFFFF0000u); // x3,x7
                xs[(e & 3) * JC + (e >> 2)] = o;
                const h2_t one = {static_cast<_Float16>(1.0f), static_cast<_Float16>(1.0f)};
                float s = 0.0f;
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    s = __builtin_amdgcn_fdot2(as_h2(v[k]), one, s, false);
                s += dpp_f32<DPP_QUAD_XOR1>(s); // the 4 words of a chunk sit in one quad
                s += dpp_f32<DPP_QUAD_XOR2>(s);
                if ((e & 3) == 0)
                    sx[e >> 2] = s;
            }
        }
    }
};

// Dot products of R rows (J chunks per lane each) with the staged input.
template <int J, int R>
__device__ __forceinline__ void dot_frag(float (&acc)[R], const Frag<J, R>& f, const u32x4* xs, const float* sx,
                                         int lane, int zshift)
{
    constexpr int JC = J * 64;
#pragma unroll
    for (int r = 0; r < R; ++r)
        acc[r] = 0.0f;
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const int c = lane + 64 * j;
        u32x4 xv[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            xv[i] = xs[i * JC + c];
        const float sxv = sx[c];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float a0 = 0.0f, a1 = 0.0f; // a0: nibbles at bit 0 of a byte (x 2^-24), a1: at bit 4 (x 2^-20)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t w = f.w[r][j][i], w8 = w >> 8;
                a0 = __builtin_amdgcn_fdot2(as_h2(w & 0x000F000Fu), as_h2(xv[i][0]), a0, false);  // n0,n4
                a1 = __builtin_amdgcn_fdot2(as_h2(w & 0x00F000F0u), as_h2(xv[i][1]), a1, false);  // n1,n5
                a0 = __builtin_amdgcn_fdot2(as_h2(w8 & 0x000F000Fu), as_h2(xv[i][2]), a0, false); // n2,n6
                a1 = __builtin_amdgcn_fdot2(as_h2(w8 & 0x00F000F0u), as_h2(xv[i][3]), a1, false); // n3,n7
            }
            const float zf = static_cast<float>((f.zw[r][j] >> zshift) & 0xFu);
            float t = a0 * 16777216.0f;      // 2^24
            t = fmaf(a1, 1048576.0f, t);     // 2^20
            t = fmaf(-zf, sxv, t);           // sum x (n - z)
            acc[r] = fmaf(t, half_bits_to_float(f.sb[r][j]), acc[r]);
        }
    }
}

// PLAIN / RESIDUAL: item = one output row of tensor item / N (fused QKV has 3).
// SWIGLU: item = one output n; rows n of the gate and of the up tensor.
template <int J, int MODE, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void int4_matvec_kernel(Int4Args a)
{
    constexpr int R = MODE == SWIGLU ? 2 : 1;
    constexpr int JC = J * 64;
    constexpr int T = WAVES * 64;
    __shared__ u32x4 xs[4 * JC];
    __shared__ float sx[JC];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int total_waves = gridDim.x * WAVES;
    const int nitems = a.n_tensors * a.N;
    int item = blockIdx.x * WAVES + wave;

    auto load_item = [&](Frag<J, R>& f, uint16_t& res, int it) {
        it = __builtin_amdgcn_readfirstlane(it);
        if (MODE == SWIGLU) {
            load_row<J>(f.w[0], f.zw[0], f.sb[0], a.m[0], static_cast<size_t>(it), a.ws, a.ss, a.zs, lane);
            load_row<J>(f.w[R - 1], f.zw[R - 1], f.sb[R - 1], a.m[1], static_cast<size_t>(it), a.ws, a.ss, a.zs, lane);
        } else {
            const int t = it / a.N, n = it - t * a.N;
            load_row<J>(f.w[0], f.zw[0], f.sb[0], a.m[t], static_cast<size_t>(n), a.ws, a.ss, a.zs, lane);
            if (MODE == RESIDUAL)
                res = a.out[t][n];
        }
    };

    XStage<J, T> stage;
    stage.issue(a.x, a.K); // input first (L2), then the first item's weights (HBM)
    Frag<J, R> cur;
    uint16_t cur_res = 0;
    if (item < nitems)
        load_item(cur, cur_res, item);
    stage.commit(xs, sx);
    __syncthreads();

    const int zshift = ((lane >> 2) & 7) * 4; // nibble of the zero word: group (c/4) % 8, same for every j
    for (; item < nitems; item += total_waves) {
        Frag<J, R> nxt;
        uint16_t nxt_res = 0;
        if (item + total_waves < nitems)
            load_item(nxt, nxt_res, item + total_waves);
        float acc[R];
        dot_frag<J, R>(acc, cur, xs, sx, lane, zshift);
        if (MODE == SWIGLU) {
            const float g = wave_sum(acc[0]);
            const float u = wave_sum(acc[R - 1]);
            if (lane == 0) {
                float v = g;
                v *= 1.0f / (1.0f + expf(-v));
                v *= u;
                a.out[0][item] = float_to_half_bits(v);
            }
        } else {
            float v = wave_sum(acc[0]);
            if (lane == 0) {
                const int t = item / a.N, n = item - t * a.N;
                if (MODE == RESIDUAL)
                    v += half_bits_to_float(cur_res);
                a.out[t][n] = float_to_half_bits(v);
            }
        }
        cur = nxt;
        cur_res = nxt_res;
    }
}

// Any K (fallback beyond 8 chunk-columns per lane): runtime trip count, dynamic LDS.
template <int MODE>
__global__ __launch_bounds__(256) void int4_matvec_generic_kernel(Int4Args a)
{
    constexpr int R = MODE == SWIGLU ? 2 : 1;
    extern __shared__ u32x4 xs_dyn[];
    const int nchunks = a.ws >> 2;
    float* sx = reinterpret_cast<float*>(xs_dyn + 4 * nchunks);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int total_waves = gridDim.x * 4;
    const int nitems = a.n_tensors * a.N;
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(a.x, a.K * 2);
    for (int e = threadIdx.x; e < nchunks * 4; e += 256) {
        const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rx, e * 16, 0, 0);
        u32x4 o;
        o[0] = (v[0] & 0xFFFFu) | (v[2] << 16);
        o[1] = (v[0] >> 16) | (v[2] & 0xFFFF0000u);
        o[2] = (v[1] & 0xFFFFu) | (v[3] << 16);
        o[3] = (v[1] >> 16) | (v[3] & 0xFFFF0000u);
        xs_dyn[(e & 3) * nchunks + (e >> 2)] = o;
        const h2_t one = {static_cast<_Float16>(1.0f), static_cast<_Float16>(1.0f)};
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < 4; ++k)
            s = __builtin_amdgcn_fdot2(as_h2(v[k]), one, s, false);
        s += dpp_f32<DPP_QUAD_XOR1>(s);
        s += dpp_f32<DPP_QUAD_XOR2>(s);
        if ((e & 3) == 0)
            sx[e >> 2] = s;
    }
    __syncthreads();
    const int zshift = ((lane >> 2) & 7) * 4;
    for (int item = blockIdx.x * 4 + wave; item < nitems; item += total_waves) {
        const int it = __builtin_amdgcn_readfirstlane(item);
        const int t = MODE == SWIGLU ? 0 : it / a.N, n = MODE == SWIGLU ? it : it - t * a.N;
        float acc[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const QW& m = a.m[MODE == SWIGLU ? r : t];
            const __amdgpu_buffer_rsrc_t rw = make_rsrc(m.w + static_cast<size_t>(n) * a.ws, a.ws * 4);
            const __amdgpu_buffer_rsrc_t rz = make_rsrc(m.z + static_cast<size_t>(n) * a.zs, a.zs * 4);
            const __amdgpu_buffer_rsrc_t rs = make_rsrc(m.s + static_cast<size_t>(n) * a.ss, a.ss * 2);
            float s = 0.0f;
            for (int c0 = 0; c0 < nchunks; c0 += 64) {
                const int c = c0 + lane; // beyond nchunks the buffer reads 0, the LDS index is clamped
                const u32x4 w4 = __builtin_amdgcn_raw_buffer_load_b128(rw, c * 16, 0, kAuxStream);
                const uint32_t zw = __builtin_amdgcn_raw_buffer_load_b32(rz, (c >> 5) * 4, 0, 0);
                const uint16_t sb = __builtin_amdgcn_raw_buffer_load_b16(rs, (c >> 2) * 2, 0, 0);
                const int cc = c < nchunks ? c : nchunks - 1;
                float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const u32x4 xv = xs_dyn[i * nchunks + cc];
                    const uint32_t w = w4[i], w8 = w >> 8;
                    a0 = __builtin_amdgcn_fdot2(as_h2(w & 0x000F000Fu), as_h2(xv[0]), a0, false);
                    a1 = __builtin_amdgcn_fdot2(as_h2(w & 0x00F000F0u), as_h2(xv[1]), a1, false);
                    a0 = __builtin_amdgcn_fdot2(as_h2(w8 & 0x000F000Fu), as_h2(xv[2]), a0, false);
                    a1 = __builtin_amdgcn_fdot2(as_h2(w8 & 0x00F000F0u), as_h2(xv[3]), a1, false);
                }
                const float zf = static_cast<float>((zw >> zshift) & 0xFu);
                float tt = a0 * 16777216.0f;
                tt = fmaf(a1, 1048576.0f, tt);
                tt = fmaf(-zf, c < nchunks ? sx[cc] : 0.0f, tt);
                s = fmaf(tt, half_bits_to_float(sb), s);
            }
            acc[r] = wave_sum(s);
        }
        if (lane == 0) {
            float v = acc[0];
            if (MODE == SWIGLU) {
                v *= 1.0f / (1.0f + expf(-v));
                v *= acc[R - 1];
            } else if (MODE == RESIDUAL) {
                v += half_bits_to_float(a.out[t][n]);
            }
            a.out[t][n] = float_to_half_bits(v);
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
    L2_CHECK(rows % 8 == 0, "%s: rows=%d must be a multiple of 8 (the input is read 16 bytes at a time, as in the reference)",
             fn, rows);
    L2_CHECK(aligned(in, 16), "%s: input must be 16-byte aligned", fn);
    L2_CHECK(aligned(out, 2), "%s: output must be 2-byte aligned", fn);
    if (static_cast<size_t>(ws) * 17 > 64 * 1024)
        return fail(LLAMA2_ERR_UNSUPPORTED, "%s: rows=%d does not fit the 64 KiB LDS staging buffer", fn, rows);
    if (static_cast<long long>(cols) * 3 > 0x7FFFFFFFLL)
        return fail(LLAMA2_ERR_UNSUPPORTED, "%s: cols=%d too large", fn, cols);
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

template <int J, int MODE, int WAVES>
static void launch_j(const Int4Args& a, int max_waves)
{
    const int nitems = a.n_tensors * a.N;
    int waves = nitems < max_waves ? nitems : max_waves;
    const int grid = ceil_div(waves, WAVES);
    hipLaunchKernelGGL((int4_matvec_kernel<J, MODE, WAVES>), dim3(grid), dim3(WAVES * 64), 0, ctx().stream, a);
}

// Wavefronts kept resident per launch: 16 per CU while a lane holds up to 3
// chunks of a row, 8 per CU for longer rows (more bytes in flight per lane).
template <int MODE>
static int launch_int4(const char* fn, const Int4Args& a)
{
    const int nchunks = a.ws / 4;
    const int J = ceil_div(nchunks, 64);
    const int cus = ctx().num_cus > 0 ? ctx().num_cus : 256;
    switch (J) {
    case 1: launch_j<1, MODE, 4>(a, cus * 16); break;
    case 2: launch_j<2, MODE, 4>(a, cus * 16); break;
    case 3: launch_j<3, MODE, 4>(a, cus * 16); break;
    case 4: launch_j<4, MODE, 4>(a, cus * 8); break;
    case 5: launch_j<5, MODE, 4>(a, cus * 8); break;
    case 6: launch_j<6, MODE, 4>(a, cus * 8); break;
    case 7: launch_j<7, MODE, 4>(a, cus * 8); break;
    case 8: launch_j<8, MODE, 4>(a, cus * 8); break;
    default: {
        const int nitems = a.n_tensors * a.N;
        const int grid = ceil_div(nitems < cus * 8 ? nitems : cus * 8, 4);
        hipLaunchKernelGGL((int4_matvec_generic_kernel<MODE>), dim3(grid), dim3(256),
                           static_cast<size_t>(nchunks) * 68, ctx().stream, a);
    }
    }
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
    Int4Args a{};
    a.m[0] = QW{weights, zeros, scales};
    a.out[0] = output;
    a.x = input;
    a.K = rows, a.N = cols, a.ws = weights_size, a.ss = scales_size, a.zs = zeros_size, a.n_tensors = 1;
    return launch_int4<RESIDUAL>(fn, a);
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
    Int4Args a{};
    a.m[0] = QW{weights, zeros, scales};
    a.out[0] = output;
    a.x = input;
    a.K = rows, a.N = cols, a.ws = weights_size, a.ss = scales_size, a.zs = zeros_size, a.n_tensors = 1;
    return launch_int4<PLAIN>(fn, a);
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
    Int4Args a{};
    a.m[0] = QW{q_weight, q_zeros, q_scales};
    a.m[1] = QW{k_weight, k_zeros, k_scales};
    a.m[2] = QW{v_weight, v_zeros, v_scales};
    a.out[0] = q_output;
    a.out[1] = k_output;
    a.out[2] = v_output;
    a.x = input;
    a.K = rows, a.N = cols, a.ws = weights_size, a.ss = scales_size, a.zs = zeros_size, a.n_tensors = 3;
    return launch_int4<PLAIN>(fn, a);
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
    Int4Args a{};
    a.m[0] = QW{g_weight, g_zeros, g_scales};
    a.m[1] = QW{u_weight, u_zeros, u_scales};
    a.out[0] = output;
    a.x = input;
    a.K = rows, a.N = cols, a.ws = weights_size, a.ss = scales_size, a.zs = zeros_size, a.n_tensors = 1;
    return launch_int4<SWIGLU>(fn, a);
}

} // extern "C"

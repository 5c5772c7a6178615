// Module entry points of the AWQ-v1 int4 mat-vec family (plain, +residual, fused
// QKV, fused SwiGLU); the kernels live in int4_kernels.hpp.
#include "int4_kernels.hpp"

namespace l2 {

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
    return launch_int4<RESIDUAL, STAGE_X>(fn, a);
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
    return launch_int4<PLAIN, STAGE_X>(fn, a);
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
    return launch_int4<PLAIN, STAGE_X>(fn, a);
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
    return launch_int4<SWIGLU, STAGE_X>(fn, a);
}

} // extern "C"

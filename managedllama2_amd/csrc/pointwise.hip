// The latency-bound modules of the decode step: RMSNorm, RoPE, softmax, argmax,
// embedding.  Replaces native/rmsnorm_kernel.cu, rope_kernel.cu,
// softmax_kernel.cu, argmax_kernel.cu and embedding_kernel.cu of the reference.
#include "common.hpp"

#include <cfloat>

namespace l2 {

constexpr int kBlock = 1024; // the reference's block size for the single-workgroup modules
constexpr int kBlockWaves = kBlock / 64;

// Sum over a 1024-thread workgroup; result in every thread.
__device__ __forceinline__ float block_sum(float v, float* lds /* kBlockWaves floats */)
{
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0)
        lds[wave] = v;
    __syncthreads();
    float t = (threadIdx.x & 63) < kBlockWaves ? lds[threadIdx.x & 63] : 0.0f;
    t = wave_sum(t);
    __syncthreads(); // lds reusable after return
    return t;
}

__device__ __forceinline__ float block_max(float v, float* lds)
{
    v = wave_max(v);
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0)
        lds[wave] = v;
    __syncthreads();
    float t = (threadIdx.x & 63) < kBlockWaves ? lds[threadIdx.x & 63] : -INFINITY;
    t = wave_max(t);
    __syncthreads();
    return t;
}

// out[i] = half( (1/sqrtf(sum(x^2)/n + eps)) * gamma[i] * x[i] ), product order
// (rms*gamma)*x as in native/rmsnorm_kernel.cu:34.  Safe in place: every
// element is read (twice) and written by the same thread, after the barrier.
__global__ __launch_bounds__(kBlock) void rmsnorm_kernel(uint16_t* out, const uint16_t* x, const uint16_t* gamma,
                                                         int size, float eps)
{
    __shared__ float lds[kBlockWaves];
    float ss = 0.0f;
    for (int i = threadIdx.x; i < size; i += kBlock) {
        const float v = half_bits_to_float(x[i]);
        ss += v * v;
    }
    ss = block_sum(ss, lds);
    const float rms = 1.0f / sqrtf(ss / static_cast<float>(size) + eps);
    for (int i = threadIdx.x; i < size; i += kBlock)
        out[i] = float_to_half_bits(rms * half_bits_to_float(gamma[i]) * half_bits_to_float(x[i]));
}

// The same module for sizes that are multiples of 8 up to 16384: 256 threads,
// 16-byte accesses, and exactly the arithmetic (order included) that the fused
// decode kernels apply while staging their input, so both paths agree bit for bit.
template <int J>
__global__ __launch_bounds__(256) void rmsnorm_vec_kernel(uint16_t* out, const uint16_t* x, const uint16_t* gamma,
                                                          int size, float eps)
{
    __shared__ float red4[4];
    VecPieces<J> xp, gp;
    xp.load(x, size);
    gp.load(gamma, size);
    const float ss = block256_sum(xp.sum_squares(), red4);
    const float rms = 1.0f / sqrtf(ss / static_cast<float>(size) + eps);
    xp.scale(rms, gp);
    const __amdgpu_buffer_rsrc_t ro = make_rsrc(out, size * 2);
#pragma unroll
    for (int i = 0; i < J; ++i) // pieces beyond `size` fall outside the buffer and are dropped
        __builtin_amdgcn_raw_buffer_store_b128(xp.v[i], ro, (threadIdx.x + i * 256) * 16, 0, 0);
}

// One workgroup per head, one thread per rotated pair (t, t + head_size/2):
// native/rope_kernel.cu:3-26.
__global__ void rope_kernel(uint16_t* q, uint16_t* k, int n_kv_heads, int head_size, int pos, float theta)
{
    const int half_size = head_size >> 1;
    for (int t = threadIdx.x; t < half_size; t += blockDim.x) {
        const int i = blockIdx.x * head_size + t;
        const int j = i + half_size;
        const int head_dim = (t * 2) % head_size;
        const float freq = 1.0f / powf(theta, static_cast<float>(head_dim) / static_cast<float>(head_size));
        const float val = static_cast<float>(pos) * freq;
        const float fcr = cosf(val);
        const float fci = sinf(val);
        rope_rotate(q[i], q[j], half_bits_to_float(q[i]), half_bits_to_float(q[j]), fcr, fci);
        if (static_cast<int>(blockIdx.x) < n_kv_heads)
            rope_rotate(k[i], k[j], half_bits_to_float(k[i]), half_bits_to_float(k[j]), fcr, fci);
    }
}

// In-place softmax of row blockIdx.x; the row lives in LDS as fp32
// (native/softmax_kernel.cu:10-47).  The maximum is the true row maximum.
__global__ __launch_bounds__(kBlock) void softmax_kernel(uint16_t* v, int size)
{
    __shared__ float buf[LLAMA2_MAX_SOFTMAX_SIZE];
    __shared__ float lds[kBlockWaves];
    uint16_t* row = v + static_cast<size_t>(blockIdx.x) * size;
    float m = -INFINITY;
    for (int i = threadIdx.x; i < size; i += kBlock) {
        const float f = half_bits_to_float(row[i]);
        buf[i] = f;
        m = fmaxf(m, f);
    }
    m = block_max(m, lds);
    float sum = 0.0f;
    for (int i = threadIdx.x; i < size; i += kBlock) {
        const float e = expf(buf[i] - m);
        buf[i] = e;
        sum += e;
    }
    sum = block_sum(sum, lds);
    for (int i = threadIdx.x; i < size; i += kBlock)
        row[i] = float_to_half_bits(buf[i] / sum);
}

// Largest logit, lowest index among equals (test/ArgmaxTests.cs:33-46).
static_assert(kBlock == 1024, "block1024_argmax");
__global__ __launch_bounds__(kBlock) void argmax_kernel(const uint16_t* x, int size, int* result, int pos,
                                                        int write_token)
{
    __shared__ float sv[kBlockWaves];
    __shared__ int si[kBlockWaves];
    const int best = block1024_argmax(x, size, sv, si);
    if (threadIdx.x == 0 && write_token)
        result[pos] = best;
}

__global__ void embedding_kernel(uint16_t* out, const uint16_t* table, int size, const int* tokens, int pos)
{
    const int token = tokens[pos];
    const uint16_t* row = table + static_cast<size_t>(token) * size;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < size)
        out[i] = row[i];
}

} // namespace l2

using namespace l2;

extern "C" {

int llama2_rmsnorm(llama2_half* output, const llama2_half* input, const llama2_half* gamma, int size, float eps)
{
    L2_REQUIRE_INIT();
    L2_CHECK(output && input && gamma, "llama2_rmsnorm: null pointer");
    L2_CHECK(size > 0, "llama2_rmsnorm: size=%d must be positive", size);
    const int J = ceil_div(size, 2048);
    if (size % 8 == 0 && J <= 8 && aligned(output, 16) && aligned(input, 16) && aligned(gamma, 16)) {
#define L2_RMS_CASE(j)                                                                                           \
    case j:                                                                                                      \
        hipLaunchKernelGGL(rmsnorm_vec_kernel<j>, dim3(1), dim3(256), 0, ctx().stream, output, input, gamma, size, \
                           eps);                                                                                 \
        break;
        switch (J) {
            L2_RMS_CASE(1) L2_RMS_CASE(2) L2_RMS_CASE(3) L2_RMS_CASE(4) L2_RMS_CASE(5) L2_RMS_CASE(6) L2_RMS_CASE(7)
            L2_RMS_CASE(8)
        }
#undef L2_RMS_CASE
    } else {
        hipLaunchKernelGGL(rmsnorm_kernel, dim3(1), dim3(kBlock), 0, ctx().stream, output, input, gamma, size, eps);
    }
    L2_LAUNCH_CHECK("llama2_rmsnorm");
    return LLAMA2_OK;
}

int llama2_rope(llama2_half* q, llama2_half* k, int n_kv_heads, int head_size, int pos, float theta, int n_heads)
{
    L2_REQUIRE_INIT();
    L2_CHECK(q && k, "llama2_rope: null pointer");
    L2_CHECK(n_heads > 0 && n_kv_heads >= 0 && n_kv_heads <= n_heads, "llama2_rope: n_heads=%d n_kv_heads=%d",
             n_heads, n_kv_heads);
    L2_CHECK(head_size >= 2 && head_size % 2 == 0, "llama2_rope: head_size=%d must be even", head_size);
    L2_CHECK(pos >= 0, "llama2_rope: pos=%d is negative", pos);
    const int half_size = head_size / 2;
    const int block = half_size < 1024 ? ((half_size + 63) / 64) * 64 : 1024;
    hipLaunchKernelGGL(rope_kernel, dim3(n_heads), dim3(block), 0, ctx().stream, q, k, n_kv_heads, head_size, pos,
                       theta);
    L2_LAUNCH_CHECK("llama2_rope");
    return LLAMA2_OK;
}

int llama2_softmax(llama2_half* vector, int size, int n_rows)
{
    L2_REQUIRE_INIT();
    L2_CHECK(vector, "llama2_softmax: null pointer");
    L2_CHECK(size > 0 && n_rows > 0, "llama2_softmax: size=%d n_rows=%d must be positive", size, n_rows);
    if (size > LLAMA2_MAX_SOFTMAX_SIZE)
        return fail(LLAMA2_ERR_UNSUPPORTED, "llama2_softmax: size=%d exceeds %d", size, LLAMA2_MAX_SOFTMAX_SIZE);
    hipLaunchKernelGGL(softmax_kernel, dim3(n_rows), dim3(kBlock), 0, ctx().stream, vector, size);
    L2_LAUNCH_CHECK("llama2_softmax");
    return LLAMA2_OK;
}

int llama2_argmax(const llama2_half* input, int size, int* result, int pos, int write_token)
{
    L2_REQUIRE_INIT();
    L2_CHECK(input && result, "llama2_argmax: null pointer");
    L2_CHECK(size > 0 && pos >= 0, "llama2_argmax: size=%d pos=%d", size, pos);
    hipLaunchKernelGGL(argmax_kernel, dim3(1), dim3(kBlock), 0, ctx().stream, input, size, result, pos, write_token);
    L2_LAUNCH_CHECK("llama2_argmax");
    return LLAMA2_OK;
}

int llama2_embedding(llama2_half* output, const llama2_half* table, int size, const int* tokens, int pos)
{
    L2_REQUIRE_INIT();
    L2_CHECK(output && table && tokens, "llama2_embedding: null pointer");
    L2_CHECK(size > 0 && pos >= 0, "llama2_embedding: size=%d pos=%d", size, pos);
    hipLaunchKernelGGL(embedding_kernel, dim3(ceil_div(size, 256)), dim3(256), 0, ctx().stream, output, table, size,
                       tokens, pos);
    L2_LAUNCH_CHECK("llama2_embedding");
    return LLAMA2_OK;
}

} // extern "C"

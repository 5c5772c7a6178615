// The stochastic sampler's modules (src/SoftmaxLogits.cs, Sort.cs,
// CumulativeSum.cs, SampleTopP.cs; kernels native/softmax_logits_kernel.cu,
// sort_kernel.cu, cumulative_sum_kernel.cu, sample_top_p_kernel.cu) and the
// whole stochastic branch of Sampler.Sample (src/Sampler.cs:48-67) as one launch.
// Every kernel is one 1024-thread workgroup, like the reference's.
#include "sampler_kernels.hpp"

namespace l2 {

template <int CH>
__global__ __launch_bounds__(kSampBlock) void softmax_logits_kernel(uint16_t* logits, int size, float temperature,
                                                                    int* indices)
{
    __shared__ SamplerLds lds;
    softmax_logits_dev<CH>(logits, size, temperature, indices, lds);
}

template <int CH>
__global__ __launch_bounds__(kSampBlock) void sort_kernel(uint16_t* keys, int* values, int size, uint16_t* keys2,
                                                          int* values2)
{
    __shared__ SamplerLds lds;
    sort_dev<CH>(keys, values, size, keys2, values2, lds);
}

__global__ __launch_bounds__(kSampBlock) void sort_lds_kernel(uint16_t* keys, int* values, int size)
{
    __shared__ SamplerLds lds;
    __shared__ SortLds buf;
    sort_lds_dev<false>(keys, values, size, lds, buf);
}

template <int CH>
__global__ __launch_bounds__(kSampBlock) void cumulative_sum_kernel(uint16_t* values, int size)
{
    __shared__ SamplerLds lds;
    cumulative_sum_dev<CH>(values, size, lds);
}

template <int CH>
__global__ __launch_bounds__(kSampBlock) void sample_top_p_kernel(const uint16_t* logits, const int* indices, int size,
                                                                  float threshold, int* result, int pos)
{
    __shared__ SamplerLds lds;
    const int token = sample_top_p_dev<CH>(logits, indices, size, threshold, lds);
    if (threadIdx.x == 0)
        result[pos] = token;
}

template <bool HEAD_ONLY>
__global__ __launch_bounds__(kSampBlock) void sample_kernel(uint16_t* logits, int* indices, int size, float temperature,
                                                            float top_p, float coin, int* result, int pos)
{
    __shared__ SamplerLds lds;
    __shared__ SortLds buf;
    const int token =
        sample_dev<4, true, HEAD_ONLY>(logits, indices, size, temperature, top_p, coin, nullptr, nullptr, lds, &buf);
    if (threadIdx.x == 0)
        result[pos] = token;
}

__global__ __launch_bounds__(kSampBlock) void sample_big_kernel(uint16_t* logits, int* indices, int size,
                                                                float temperature, float top_p, float coin, int* result,
                                                                int pos, uint16_t* keys2, int* values2)
{
    __shared__ SamplerLds lds;
    const int token = sample_dev<8, false>(logits, indices, size, temperature, top_p, coin, keys2, values2, lds, nullptr);
    if (threadIdx.x == 0)
        result[pos] = token;
}

int check_sampler_size(const char* fn, int size)
{
    L2_CHECK(size > 0, "%s: size=%d must be positive", fn, size);
    if (size > LLAMA2_MAX_SAMPLER_SIZE)
        return fail(LLAMA2_ERR_UNSUPPORTED, "%s: size=%d exceeds %d", fn, size, LLAMA2_MAX_SAMPLER_SIZE);
    return LLAMA2_OK;
}

} // namespace l2

using namespace l2;

#define L2_TRY(expr)          \
    do {                      \
        int rc_ = (expr);     \
        if (rc_ != LLAMA2_OK) \
            return rc_;       \
    } while (0)

// 8-element chunks per thread: 4 cover 32768 elements, 8 cover 65536
#define L2_SAMPLER_LAUNCH(kernel, size, ...)                                                                   \
    do {                                                                                                       \
        if ((size) <= 4 * 8 * kSampBlock)                                                                      \
            hipLaunchKernelGGL(kernel<4>, dim3(1), dim3(kSampBlock), 0, ctx().stream, __VA_ARGS__);            \
        else                                                                                                   \
            hipLaunchKernelGGL(kernel<8>, dim3(1), dim3(kSampBlock), 0, ctx().stream, __VA_ARGS__);            \
    } while (0)

extern "C" {

int llama2_softmax_logits(llama2_half* logits, int size, float temperature, int* indices)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_softmax_logits";
    L2_CHECK(logits && indices, "%s: null pointer", fn);
    L2_TRY(check_sampler_size(fn, size));
    L2_CHECK(temperature > 0.0f, "%s: temperature=%g must be positive (temperature 0 is the argmax branch)", fn,
             static_cast<double>(temperature));
    L2_CHECK(aligned(logits, 16) && aligned(indices, 16), "%s: logits and indices must be 16-byte aligned", fn);
    L2_SAMPLER_LAUNCH(softmax_logits_kernel, size, logits, size, temperature, indices);
    L2_LAUNCH_CHECK(fn);
    return LLAMA2_OK;
}

int llama2_sort(llama2_half* keys, int* values, int size)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_sort";
    L2_CHECK(keys && values, "%s: null pointer", fn);
    L2_TRY(check_sampler_size(fn, size));
    L2_CHECK(aligned(keys, 16) && aligned(values, 16), "%s: keys and values must be 16-byte aligned", fn);
    if (size <= kSortLdsItems)
        hipLaunchKernelGGL(sort_lds_kernel, dim3(1), dim3(kSampBlock), 0, ctx().stream, keys, values, size);
    else
        L2_SAMPLER_LAUNCH(sort_kernel, size, keys, values, size, ctx().sort_keys, ctx().sort_values);
    L2_LAUNCH_CHECK(fn);
    return LLAMA2_OK;
}

int llama2_cumulative_sum(llama2_half* values, int size)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_cumulative_sum";
    L2_CHECK(values, "%s: null pointer", fn);
    L2_TRY(check_sampler_size(fn, size));
    L2_CHECK(aligned(values, 16), "%s: values must be 16-byte aligned", fn);
    L2_SAMPLER_LAUNCH(cumulative_sum_kernel, size, values, size);
    L2_LAUNCH_CHECK(fn);
    return LLAMA2_OK;
}

int llama2_sample_top_p(const llama2_half* logits, const int* indices, int size, float threshold, int* result, int pos)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_sample_top_p";
    L2_CHECK(logits && indices && result, "%s: null pointer", fn);
    L2_TRY(check_sampler_size(fn, size));
    L2_CHECK(pos >= 0, "%s: pos=%d is negative", fn, pos);
    L2_CHECK(aligned(logits, 16), "%s: logits must be 16-byte aligned", fn);
    L2_SAMPLER_LAUNCH(sample_top_p_kernel, size, logits, indices, size, threshold, result, pos);
    L2_LAUNCH_CHECK(fn);
    return LLAMA2_OK;
}

int llama2_sample(llama2_half* logits, int* indices, int size, float temperature, float top_p, float coin,
                  int* result, int pos)
{
    L2_REQUIRE_INIT();
    return sample_launch("llama2_sample", logits, indices, size, temperature, top_p, coin, result, pos, false);
}

} // extern "C"

namespace l2 {

int sample_launch(const char* fn, uint16_t* logits, int* indices, int size, float temperature, float top_p, float coin,
                  int* result, int pos, bool token_only)
{
    L2_CHECK(logits && indices && result, "%s: null pointer", fn);
    L2_TRY(check_sampler_size(fn, size));
    L2_CHECK(temperature > 0.0f, "%s: temperature=%g must be positive (temperature 0 is the argmax branch)", fn,
             static_cast<double>(temperature));
    L2_CHECK(pos >= 0, "%s: pos=%d is negative", fn, pos);
    L2_CHECK(aligned(logits, 16) && aligned(indices, 16), "%s: logits and indices must be 16-byte aligned", fn);
    if (size <= kSortLdsItems && token_only)
        hipLaunchKernelGGL(sample_kernel<true>, dim3(1), dim3(kSampBlock), 0, ctx().stream, logits, indices, size,
                           temperature, top_p, coin, result, pos);
    else if (size <= kSortLdsItems)
        hipLaunchKernelGGL(sample_kernel<false>, dim3(1), dim3(kSampBlock), 0, ctx().stream, logits, indices, size,
                           temperature, top_p, coin, result, pos);
    else
        hipLaunchKernelGGL(sample_big_kernel, dim3(1), dim3(kSampBlock), 0, ctx().stream, logits, indices, size,
                           temperature, top_p, coin, result, pos, ctx().sort_keys, ctx().sort_values);
    L2_LAUNCH_CHECK(fn);
    return LLAMA2_OK;
}

} // namespace l2

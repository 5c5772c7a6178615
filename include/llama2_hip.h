/*
 * llama2_hip.h -- C ABI of libllama2_hip.so, the MI355X (gfx950) implementation
 * of ManagedLlama2's quantized batch-1 decode path.
 *
 * The library takes the place of ManagedCuda + the embedded PTX modules
 * underneath the reference's C# module classes: every entry point below names
 * the reference interface it replaces (paths relative to the reference
 * checkout).  Kernel entry points keep the argument order of the reference's
 * `extern "C" __global__` prototypes (the native/<kernel>.cuh headers); what the reference
 * encoded in the launch grid (number of heads / rows) is an explicit trailing
 * int here, because grid and block shapes are chosen inside the library.
 *
 * Conventions
 *   - plain C, no C++ or framework types in any signature;
 *   - every function returns 0 (LLAMA2_OK) on success, a negative LLAMA2_ERR_*
 *     for rejected arguments / state, or a positive hipError_t value when the
 *     HIP runtime failed; llama2_last_error() describes the last failure of
 *     the calling thread;
 *   - `llama2_half` is IEEE binary16 storage (C# System.Half, CUDA half);
 *   - all pointers named out/x/q/... are DEVICE pointers obtained from
 *     llama2_malloc (or any hipMalloc'ed memory of the same device);
 *   - kernels are enqueued asynchronously on one library-owned stream, in
 *     call order; llama2_memcpy_d2h and llama2_sync wait for them.  The
 *     reference runs on a single NULL stream from one host thread; here host
 *     threads may share the library: every entry point takes one lock and
 *     binds the calling thread to the library's device, so calls take turns.
 */
#ifndef LLAMA2_HIP_H
#define LLAMA2_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

typedef uint16_t llama2_half;

#define LLAMA2_OK 0
#define LLAMA2_ERR_INVALID_ARGUMENT (-1) /* null / misaligned pointer, bad size, aliasing */
#define LLAMA2_ERR_NOT_INITIALIZED (-2)  /* llama2_init not called                        */
#define LLAMA2_ERR_UNSUPPORTED (-3)      /* shape outside what the kernels implement      */
#define LLAMA2_ERR_NO_DEVICE (-4)        /* no usable gfx950 device                        */
#define LLAMA2_ERR_STEP_FAILED (-5)      /* a persistent decode step gave up a bounded wait */

/* Largest softmax row, as in the reference (native/softmax_kernel.cu:5). */
#define LLAMA2_MAX_SOFTMAX_SIZE 8192
/* Largest `size` of the sampler modules (softmax_logits, sort, cumulative_sum,
 * sample_top_p): one 1024-thread workgroup holds the whole vector. */
#define LLAMA2_MAX_SAMPLER_SIZE 65536

/* ---------------------------------------------------------------- runtime */

/* new CudaContext(deviceID): src/Transformer.cs:48-49.  Idempotent per device. */
int llama2_init(int device);
/* Releases the stream and internal scratch.  Caller-owned buffers stay valid. */
int llama2_shutdown(void);
/* Text of the calling thread's last error ("" if none).  Never NULL. */
const char* llama2_last_error(void);

/* new CudaDeviceVariable<T>(n): src/RunState.cs:41-53.  256-byte aligned. */
int llama2_malloc(void** ptr, size_t bytes);
/* CudaDeviceVariable.Dispose. */
int llama2_free(void* ptr);
/* implicit T[] -> CudaDeviceVariable<T> (src/TransformerWeights.cs:61-66) and
 * CopyToDevice(src, 0, dstByteOffset, bytes) (src/Extensions.cs:23-24,
 * src/Transformer.cs:93,127).  Ordered after previously enqueued kernels. */
int llama2_memcpy_h2d(void* dst, size_t dst_offset_bytes, const void* src, size_t bytes);
/* explicit CudaDeviceVariable<T> -> T[] and the 1-element indexer read
 * `runstate.tokens[nextPosition]` (src/Sampler.cs:69).  Waits for the stream. */
int llama2_memcpy_d2h(void* dst, const void* src, size_t src_offset_bytes, size_t bytes);
/* CudaDeviceVariable.CopyToDevice(CudaDeviceVariable): asynchronous device-to-
 * device copy by a plain copy kernel (16-byte granularity, no overlap). */
int llama2_memcpy_d2d(void* dst, const void* src, size_t bytes);
/* Asynchronous fill (tests and RunState set-up; ManagedCuda's Memset). */
int llama2_memset(void* dst, int byte_value, size_t bytes);
/* CudaContext.GetFreeDeviceMemorySize(): src/RunState.cs:34. */
int llama2_mem_info(size_t* free_bytes, size_t* total_bytes);
/* CudaContext.Synchronize(). */
int llama2_sync(void);
/* The hipStream_t every entry point launches on (for callers that time or
 * order their own work against it).  NULL before llama2_init. */
void* llama2_stream(void);

/* HIP events on the library's stream, for timing the enqueued kernels. */
int llama2_event_create(void** event);
int llama2_event_record(void* event);
int llama2_event_elapsed_ms(void* start, void* stop, float* ms); /* waits for `stop` */
int llama2_event_destroy(void* event);

/* Stream capture of the calls made between begin and end into a hipGraph that
 * llama2_graph_launch replays with a single submission (no counterpart in the
 * reference, which pays one cuLaunchKernel per module call, src/Module.cs:21-22).
 * Only kernel entry points may be called while capturing: no malloc / free /
 * memcpy / sync, and llama2_vec_mat / llama2_multi_head_attention only for
 * shapes whose scratch already exists (call them once eagerly first).  The captured calls keep the argument
 * values they were made with, the scratch address included: the library never
 * frees a scratch buffer before llama2_shutdown, so a later eager call that
 * needs a larger one leaves earlier graphs valid. */
int llama2_graph_begin_capture(void);
int llama2_graph_end_capture(void** graph);
int llama2_graph_launch(void* graph);
int llama2_graph_destroy(void* graph);

/* ------------------------------------------------- int4 tensors ("QWeight")
 * Layout per output row n of a K-input tensor (src/TransformerWeights.cs:54-69,
 * native/mat_vec_kernel.cu:98-134):
 *   weights_size = ceil(K/32)*4 uint32, element k in bits 4*(k%8).. of word k/8
 *   scales_size  = ceil(K/128)   fp16,  scale of group g = k/128
 *   zeros_size   = ceil(scales_size/8) uint32, zero of group g = nibble g%8 of word g/8
 *   value(n,k)   = (w - z) * scale
 * `rows` is the INPUT length K and `cols` the number of outputs N, as in the
 * reference (src/MatVecResidual.cs:15-22).  The three *_size arguments must be
 * the values above (they are what the reference's modules pass); weight rows
 * must be 16-byte aligned.
 */

/* mat_vec_residual_int4_kernel (native/mat_vec_kernel.cuh:58-59), module
 * MatVecResidual.Forward (src/MatVecResidual.cs:15-22):
 *   output[n] = half(float(output[n]) + sum_k input[k]*(w-z)*s).
 * `output` must not overlap `input`. */
int llama2_mat_vec_residual_int4(llama2_half* output, const llama2_half* input,
                                 const uint32_t* weights, const uint32_t* zeros,
                                 const llama2_half* scales, int rows, int cols, int zeros_size,
                                 int scales_size, int weights_size);

/* The same dot product without the residual read (device function
 * mat_vec_int4, native/mat_vec_kernel.cu:166-177; one third of QKVMatVec). */
int llama2_mat_vec_int4(llama2_half* output, const llama2_half* input, const uint32_t* weights,
                        const uint32_t* zeros, const llama2_half* scales, int rows, int cols,
                        int zeros_size, int scales_size, int weights_size);

/* qkv_mat_vec_kernel (native/mat_vec_kernel.cuh:85-89), module QKVMatVec.Forward
 * (src/QKVMatVec.cs:19-31): three int4 mat-vecs of one input in one launch.
 * k_output / v_output are the KV-cache rows, i.e. the caller has already added
 * layerOffset + pos*kvDim (src/QKVMatVec.cs:25-26). */
int llama2_qkv_mat_vec(llama2_half* q_output, llama2_half* k_output, llama2_half* v_output,
                       const llama2_half* input, const uint32_t* q_weight, const uint32_t* q_zeros,
                       const llama2_half* q_scales, const uint32_t* k_weight,
                       const uint32_t* k_zeros, const llama2_half* k_scales,
                       const uint32_t* v_weight, const uint32_t* v_zeros,
                       const llama2_half* v_scales, int rows, int cols, int zeros_size,
                       int scales_size, int weights_size);

/* mat_vec_swiglu_kernel (native/mat_vec_kernel.cuh:113-116), module
 * MatVecSwiGLU.Forward (src/MatVecSwiGLU.cs:15-24):
 *   output[n] = half( silu(g.x) * (u.x) ),  silu(v) = v / (1 + expf(-v)). */
int llama2_mat_vec_swiglu(llama2_half* output, const llama2_half* input, const uint32_t* g_weight,
                          const uint32_t* g_zeros, const llama2_half* g_scales,
                          const uint32_t* u_weight, const uint32_t* u_zeros,
                          const llama2_half* u_scales, int rows, int cols, int zeros_size,
                          int scales_size, int weights_size);

/* ---------------------------------------------------------- fp16 mat-vecs */

/* mat_vec_kernel (native/mat_vec_kernel.cuh:17), module MatVec.Forward
 * (src/MatVec.cs:15-16): output[n] = sum_k matrix[n*rows + k] * vector[k];
 * rows % 8 == 0 as in the reference (native/mat_vec_kernel.cu:16,26). */
int llama2_mat_vec(llama2_half* output, const llama2_half* vector, const llama2_half* matrix,
                   int rows, int cols);

/* mat_vec_strided_kernel (native/mat_vec_kernel.cuh:37-38), module
 * MatVecStrided.Forward (src/MatVecStrided.cs:16-18); n_heads was gridDim.y:
 *   output[h*o_stride + t] = alpha * sum_{r<rows} vector[h*v_stride + r]
 *                                    * matrix[t*m_row_stride + h*m_col_stride + r]
 * for t < cols, h < n_heads. */
int llama2_mat_vec_strided(llama2_half* output, const llama2_half* vector,
                           const llama2_half* matrix, int rows, int cols, int v_stride,
                           int m_col_stride, int m_row_stride, int o_stride, float alpha,
                           int n_heads);

/* vec_mat_kernel (native/vec_mat_kernel.cuh:5-6), module VecMat.Forward
 * (src/VecMat.cs:17-19); n_heads was gridDim.y:
 *   output[h*o_stride + r] = sum_{t<cols} vector[h*cols + t]
 *                            * matrix[t*m_row_stride + h*m_col_stride + r],  r < rows. */
int llama2_vec_mat(llama2_half* output, const llama2_half* vector, const llama2_half* matrix,
                   int rows, int cols, int m_col_stride, int o_stride, int m_row_stride,
                   int n_heads);

/* llama2_vec_mat for callers that cannot allocate (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same
 * arguments, same kernels, same results bit for bit; but where llama2_vec_mat keeps the fp32
 * partial sums of a sequence split over workgroups in a buffer it allocates (and grows) on
 * demand, this entry point keeps them in a fixed array of LLAMA2_STATIC_VEC_MAT_BYTES inside
 * the library's code object (one copy per GPU, held until the process ends) and calls no
 * hipMalloc, hipFree or other allocating routine.  A call whose partial sums
 * (sequence blocks x n_heads x rows floats) do not fit returns LLAMA2_ERR_UNSUPPORTED
 * (32 heads of 128 rows fit at any sequence length; 40 heads up to about 3300 positions).
 * All calls on a GPU share the array: calls that overlap on one GPU (two streams, two
 * replaying graphs) race; calls on the library's one stream are in order and safe. */
#define LLAMA2_STATIC_VEC_MAT_BYTES 2097152
int llama2_vec_mat_static(llama2_half* output, const llama2_half* vector, const llama2_half* matrix,
                   int rows, int cols, int m_col_stride, int o_stride, int m_row_stride,
                   int n_heads);

/* Transformer.MultiHeadAttention (src/Transformer.cs:150-156) as ONE launch:
 * scores over `seq_length` rows of `key`, softmax, weighted sum of `value`
 * rows, without the round trip through the `attention` scratch.  key / value
 * are the cache slices of the layer (caller adds layerOffset), rows of `dim`
 * halfs; head h uses columns h*head_size .. of q, key, value and output.
 * Scores are rounded to fp16 as the reference's attention buffer does.
 * head_size must be 128; other sizes: LLAMA2_ERR_UNSUPPORTED, use the three
 * modules above. */
int llama2_multi_head_attention(llama2_half* output, const llama2_half* query, const llama2_half* key,
                                const llama2_half* value, int head_size, int dim, int seq_length,
                                float scale, int n_heads);

/* RoPERotation.Forward (src/RoPERotation.cs:13-21, native/rope_kernel.cu:3-26)
 * at position `pos` followed by MultiHeadAttention (src/Transformer.cs:172-175)
 * in ONE launch: the query and row seq_length - 1 of `key` (the row the step's
 * QKVMatVec has just written) are rotated inside the attention kernel and
 * written back rotated, as llama2_rope leaves them, so the call equals
 * llama2_rope(query, key + (seq_length - 1) * dim, n_heads, 128, pos, theta,
 * n_heads) + llama2_multi_head_attention(...) bit for bit, without the second
 * launch.  No counterpart in the reference, which launches four kernels here.
 * Same limits as llama2_multi_head_attention (head_size 128). */
int llama2_rope_multi_head_attention(llama2_half* output, llama2_half* query, llama2_half* key,
                                     const llama2_half* value, int head_size, int dim,
                                     int seq_length, float scale, int n_heads, int pos,
                                     float theta);

/* ------------------------------------------------------- pointwise modules */

/* rmsnorm_kernel (native/rmsnorm_kernel.cuh:5), module RMSNorm.Forward
 * (src/RMSNorm.cs:13-14): output[i] = half(1/sqrtf(mean(x^2)+eps) * gamma[i] * x[i]).
 * output may be the same buffer as input (src/Transformer.cs:187). */
int llama2_rmsnorm(llama2_half* output, const llama2_half* input, const llama2_half* gamma,
                   int size, float eps);

/* rope_kernel (native/rope_kernel.cuh:6), module RoPERotation.Forward
 * (src/RoPERotation.cs:19-24); n_heads was gridDim.x.  Rotates the pairs
 * (i, i + head_size/2) of every head of q, and of k for heads < n_kv_heads;
 * k is the cache row, already offset by layerOffset + pos*kvDim. */
int llama2_rope(llama2_half* q, llama2_half* k, int n_kv_heads, int head_size, int pos,
                float theta, int n_heads);

/* softmax_kernel (native/softmax_kernel.cuh:5), module Softmax.Forward
 * (src/Softmax.cs:13-14); n_rows was gridDim.x: in-place softmax of
 * vector[r*size .. r*size+size) for r < n_rows; size <= LLAMA2_MAX_SOFTMAX_SIZE. */
int llama2_softmax(llama2_half* vector, int size, int n_rows);

/* argmax_kernel (native/argmax_kernel.cuh:5), module Argmax.Forward
 * (src/Argmax.cs:13-14): result[pos] = index of the largest input iff
 * write_token.  Ties resolve to the LOWEST index, deterministically (the
 * reference's CPU check, test/ArgmaxTests.cs:33-46; its kernel races). */
int llama2_argmax(const llama2_half* input, int size, int* result, int pos, int write_token);

/* embedding_kernel (native/embedding_kernel.cuh:5), module Embedding.Forward
 * (src/Embedding.cs:13-14): output[i] = table[tokens[pos]*size + i]; the token
 * id is read on the device. */
int llama2_embedding(llama2_half* output, const llama2_half* table, int size, const int* tokens,
                     int pos);

/* ------------------------------------------------ stochastic sampler modules
 * The four kernels of Sampler.Sample's temperature / top-p branch
 * (src/Sampler.cs:48-67).  1 <= size <= LLAMA2_MAX_SAMPLER_SIZE (the
 * reference's launch shapes fix size to a multiple of 125 resp. 32 up to
 * 32000; any size works here).  fp16 and int buffers 16-byte aligned. */

/* softmax_logits_kernel (native/softmax_logits_kernel.cuh:5), module
 * SoftmaxLogits.Forward (src/SoftmaxLogits.cs:14-15): indices[t] = t;
 * logits <- softmax(logits / temperature) in place with the reference's three
 * fp16 roundings (after the division, after expf, after the normalisation).
 * temperature > 0. */
int llama2_softmax_logits(llama2_half* logits, int size, float temperature, int* indices);

/* sort_kernel (native/sort_kernel.cuh:4), module Sort.Forward
 * (src/Sort.cs:14-15): sorts keys in DESCENDING order, in place, carrying
 * values along.  Stable (equal keys keep their order), like the reference's
 * cub::BlockRadixSort; keys are ordered as the radix sort orders fp16 bit
 * patterns (numeric order, +0 before -0, NaNs at the two ends). */
int llama2_sort(llama2_half* keys, int* values, int size);

/* cumulative_sum_kernel (native/cumulative_sum_kernel.cuh:5), module
 * CumulativeSum.Forward (src/CumulativeSum.cs:14-15): in-place inclusive
 * prefix sums, accumulated in fp32, each rounded to fp16. */
int llama2_cumulative_sum(llama2_half* values, int size);

/* sample_top_p_kernel (native/sample_top_p_kernel.cuh:5), module
 * SampleTopP.Forward (src/SampleTopP.cs:14-15): result[pos] = indices[m], m the
 * first position with float(logits[m]) >= threshold, or size-1 if none. */
int llama2_sample_top_p(const llama2_half* logits, const int* indices, int size, float threshold,
                        int* result, int pos);

/* The stochastic branch of Sampler.Sample (src/Sampler.cs:50-66) as ONE launch:
 * softmax_logits; if 0 < top_p < 1: sort and threshold = coin * top_p, else
 * threshold = coin; cumulative_sum; sample_top_p into result[pos].  logits and
 * indices are overwritten exactly as by the four module calls (same device
 * code).  coin is the caller's uniform number in [0, 1). */
int llama2_sample(llama2_half* logits, int* indices, int size, float temperature, float top_p,
                  float coin, int* result, int pos);

/* ------------------------------------------------------- converter repack
 * The tensor transformations of ModelConverter.RepackQWeightByName
 * (src/ModelConverter.cs:196-275) on device buffers: what turns an AWQ
 * checkpoint's tensors into the layout every entry point above reads.  All
 * asynchronous on the library's stream; out and in must not overlap. */

/* RepackQData (src/ModelConverter.cs:277-317).  in: [height][width/8] words of
 * the AWQ "GEMM" format (nibble i of a word = column 8c + {0,2,4,6,1,3,5,7}[i]);
 * out: [width][ceil(height/8)] words, word y/8 of row x = rows y..y+7 of column
 * x.  Used for qweight (height = K) and qzeros (height = K/128).  When height
 * is not a multiple of 8 the unused nibbles of a row's last word are filled as
 * the reference fills them (first rows of the next column, zero behind the
 * last column), so converted files are byte-identical.  width % 8 == 0. */
int llama2_repack_qdata(uint32_t* out, const uint32_t* in, int height, int width);

/* RepackScales (src/ModelConverter.cs:319-328): [meta_height][width] halfs ->
 * [width][meta_height]. */
int llama2_repack_scales(llama2_half* out, const llama2_half* in, int meta_height, int width);

/* The Format.v1 branch (src/ModelConverter.cs:247-262): scale rows stored with
 * ceil(scales_size/8)*8 halfs each -> rows of scales_size halfs. */
int llama2_compact_scales_v1(llama2_half* out, const llama2_half* in, int scales_size, int width);

/* ------------------------------------------------------------ decode step */

/* src/Config.cs:6-19 -- the 32-byte model-file header, same field order. */
typedef struct llama2_config {
    int dim;
    int hidden_dim;
    int n_layers;
    int n_heads;
    int n_kv_heads;
    int vocab_size;
    int seq_len;
    float rope_theta;
} llama2_config;

/* src/QWeight.cs:5-10 */
typedef struct llama2_qweight {
    const uint32_t* weight;
    const uint32_t* zeros;
    const llama2_half* scales;
} llama2_qweight;

/* src/PerLayerWeight.cs:5-16 */
typedef struct llama2_layer_weights {
    llama2_qweight query, key, value, output, gate, up, down;
    const llama2_half* rms_attention;
    const llama2_half* rms_feed_forward;
} llama2_layer_weights;

/* src/TransformerWeights.cs:8-14 */
typedef struct llama2_transformer_weights {
    const llama2_half* token_embedding_table;
    const llama2_half* classifier_weights;
    const llama2_half* rms_final_weight;
    const llama2_layer_weights* layers; /* host array of n_layers entries */
} llama2_transformer_weights;

/* src/RunState.cs:7-25.  attention holds n_heads*max(dim, seq_len) halfs,
 * key/value caches n_layers*seq_len*kv_dim halfs, tokens seq_len+1 ints,
 * indices vocab_size ints (only the stochastic sampler uses it: may be null
 * for greedy decoding). */
typedef struct llama2_run_state {
    llama2_half* x;
    llama2_half* xb;
    llama2_half* h;
    llama2_half* q;
    llama2_half* attention;
    llama2_half* logits;
    llama2_half* key_cache;
    llama2_half* value_cache;
    int* tokens;
    int* indices;
} llama2_run_state;

typedef struct llama2_decoder llama2_decoder;

/* How llama2_decode_forward issues the step. */
#define LLAMA2_DECODE_MODULES 0 /* the 10 module launches per layer of Transformer.Forward */
#define LLAMA2_DECODE_FUSED 1   /* fused kernels (norm+QKV+RoPE, attention, norm+SwiGLU, ...) */
#define LLAMA2_DECODE_GRAPH 2   /* OR-able: replay the step as a captured hipGraph (one per attention launch shape) */
/* OR-able with LLAMA2_DECODE_FUSED: the whole of Transformer.Forward
 * (src/Transformer.cs:158-190) as ONE persistent launch -- one workgroup per
 * compute unit walks through all layers, the vectors between the modules are
 * handed from workgroup to workgroup inside the launch, and the weight stream
 * never stops at a module boundary.  Same arithmetic as LLAMA2_DECODE_FUSED, and
 * the same results bit for bit up to 1024 attended rows (beyond, the launch
 * sequence merges attention blocks of 256 rows and this step blocks of 128).  Serves histories of up to 3072 rows (longer ones fall
 * back to the launch sequence, step by step) and the shapes it has kernels for
 * (Llama-2-7B: dim 4096, hidden_dim 11008, 32 heads on 256 compute units; and
 * small models of at most one row per wavefront and phase: on 256 compute units
 * dim <= 640 and hidden_dim <= 2048); otherwise llama2_decode_create
 * returns LLAMA2_ERR_UNSUPPORTED.  The launch needs the GPU to itself: all its
 * workgroups must be resident at once.  Every wait inside it is bounded; a step
 * that gives up raises a sticky flag: llama2_decode_sample and
 * llama2_decode_sample_top_p return LLAMA2_ERR_STEP_FAILED from then on, and
 * after the asynchronous llama2_decode_run / _run_sampled the caller asks
 * llama2_decode_check. */
#define LLAMA2_DECODE_PERSISTENT 4

/* Binds a config, a weight set and a run state (all borrowed, all must outlive
 * the decoder) to the per-step launch sequence of Transformer.Forward
 * (src/Transformer.cs:158-190).  GQA is rejected like the reference does
 * (src/Transformer.cs:53-56). */
int llama2_decode_create(llama2_decoder** decoder, const llama2_config* config,
                         const llama2_transformer_weights* weights,
                         const llama2_run_state* state, int mode);
/* Transformer.Forward(position, nextPosition): leaves fp16 logits in
 * state->logits.  Asynchronous. */
int llama2_decode_forward(llama2_decoder* decoder, int position, int next_position);
/* Sampler.Sample greedy branch (src/Sampler.cs:44-47,69): argmax into
 * tokens[next_position] iff generate_token, then reads that token back
 * (the one host synchronisation per token).  The token after the last row of
 * the context (next_position == seq_len) has no slot in `tokens`
 * (src/RunState.cs:52): it is returned without being stored, and the
 * device-resident loops below do not store it either. */
int llama2_decode_sample(llama2_decoder* decoder, int next_position, int generate_token,
                         int* token);
/* Sampler.Sample with temperature and top-p (src/Sampler.cs:40-70): the greedy
 * branch when temperature == 0 or !generate_token, otherwise the token that
 * llama2_sample picks on state->logits / state->indices with the caller's
 * uniform `coin` in [0, 1); then reads tokens[next_position] back.  Only the
 * token is defined: the sort stops at the head of the distribution that holds
 * top_p of the mass, so logits / indices are left partly sorted. */
int llama2_decode_sample_top_p(llama2_decoder* decoder, int next_position, int generate_token,
                               float temperature, float top_p, float coin, int* token);
/* The uniform number the device-resident sampling loop draws for the token at
 * `position` from `seed` (splitmix64 of seed + position, top 24 bits); exported
 * so that a host loop can reproduce llama2_decode_run_sampled step by step. */
float llama2_sampler_coin(unsigned long long seed, int position);
/* `steps` iterations of forward + greedy sample starting at `position`
 * without any host synchronisation in between (tokens stay on the device;
 * positions below n_prompt keep their prompt token, as Transformer.Generate
 * does, src/Transformer.cs:96-104).  Does not stop on token < 3. */
int llama2_decode_run(llama2_decoder* decoder, int position, int steps, int n_prompt);
/* The same loop with the stochastic sampler: the token at next_position p is
 * drawn with coin = llama2_sampler_coin(seed, p).  temperature == 0 is
 * llama2_decode_run.  (The reference draws from an unseeded System.Random,
 * src/Sampler.cs:24,42, on the host; this keeps the loop on the device.)
 * The tokens are those of llama2_decode_sample_top_p with the same coins; what
 * state->logits and state->indices hold afterwards is not: when a short head of
 * the sorted distribution carries more than top_p of the mass, only that head
 * is sorted and summed. */
int llama2_decode_run_sampled(llama2_decoder* decoder, int position, int steps, int n_prompt,
                              float temperature, float top_p, unsigned long long seed);
/* Waits for the enqueued steps and reports LLAMA2_ERR_STEP_FAILED if a
 * persistent step (LLAMA2_DECODE_PERSISTENT) gave up a wait; LLAMA2_OK for the
 * other modes.  No counterpart in the reference (its kernels cannot fail this
 * way). */
int llama2_decode_check(llama2_decoder* decoder);
/* Number of unsuccessful polls (about a microsecond each) after which a wait
 * inside the persistent step gives up; default 2^21.  Clears the failure flag.
 * For tests of the failure path and for hosts that want a tighter bound. */
int llama2_decode_set_wait_limit(llama2_decoder* decoder, int polls);
/* The int4 mat-vec set of every layer of the decoder's model -- RMSNorm + fused
 * QKV (native/mat_vec_kernel.cu:166-203), o-proj + residual (:144-164), RMSNorm
 * + fused SwiGLU (:206-234), down-proj + residual -- chained through all layers
 * in one persistent launch, exactly as the persistent step runs them, but
 * without attention: the o-projection takes q as its input.  input: dim halfs
 * (the residual stream entering layer 0); output: dim halfs (the residual
 * stream after the last layer).  Needs LLAMA2_DECODE_PERSISTENT.  This is the
 * measurement and parity handle for the mat-vec family inside the persistent
 * step; the KV cache is not touched. */
int llama2_decode_matvec_chain(llama2_decoder* decoder, const llama2_half* input,
                               llama2_half* output);
int llama2_decode_destroy(llama2_decoder* decoder);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif

#ifdef __cplusplus
}
#endif
#endif /* LLAMA2_HIP_H */

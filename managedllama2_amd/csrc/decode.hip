// The decode step: Transformer.Forward (src/Transformer.cs:158-190) with
// MultiHeadAttention (:150-156) and the greedy branch of Sampler.Sample
// (src/Sampler.cs:44-47,69), issued on the library's stream.
//
// Two ways of issuing the step:
//   LLAMA2_DECODE_MODULES  the reference's launch sequence, module by module
//                          (1 + 10 L + 2 launches per token);
//   LLAMA2_DECODE_FUSED    5 launches per layer: RMSNorm + QKV + RoPE + cache
//                          write | split-sequence attention | o-proj + residual |
//                          RMSNorm + SwiGLU | down-proj + residual.  Everything
//                          that depends on the position is read from a small
//                          device-resident state block, so the launch sequence
//                          is identical for every token and is replayed as a
//                          hipGraph (LLAMA2_DECODE_GRAPH): one graph per size of
//                          the attention grid, chosen by the host's copy of the
//                          position.
#include "int4_kernels.hpp"
#include "persist.hpp"
#include "sampler_kernels.hpp"

#include <climits>
#include <cstdlib>
#include <cmath>
#include <new>
#include <vector>

namespace l2 {

// ---------------------------------------------------------------- fused attention
// One workgroup of WAVES wavefronts per (head, block of 32 * WAVES timesteps).  Every
// byte of K and V the workgroup needs is requested before the first score is computed
// (up to 16 loads of 16 bytes per lane; rows outside the block are out of the
// buffer's range and cost no traffic), 16 lanes share one timestep, scores are
// rounded to fp16 like the reference's `attention` buffer, softmax statistics
// are per block and the blocks of a head are merged by whichever workgroup
// finishes last (fixed merge order: deterministic).
//
// One compute unit pulls only a few tens of GB/s, so a short sequence wants
// many small blocks (4 wavefronts, 128 rows); the exchange between workgroups
// costs about 3 us whatever their number, and a long sequence wants fewer
// merges.  Measured on 32 heads (one launch, RoPE inside), 64 / 128 / 256 / 512
// rows per block: 512 rows 7.4 / 7.3 / 8.8 / 11.0 us, 2048 rows 17.7 / 12.1 /
// 11.4 / 15.5 us, 4096 rows 31.2 / 21.5 / 17.3 / 19.4 us: 128-row blocks up to
// 1024 rows, 256-row blocks (8 wavefronts) beyond.  Dispatching workgroups
// that find nothing to do is not free: a grid sized for the whole context costs
// several microseconds per launch at short lengths.  The position lives on the
// device, but the host always knows an upper bound for it, so it picks the
// launch shape (block size, number of blocks) from a short list by that bound.
// Measured in the decode loop: one 256-row block of 8 wavefronts for 129 .. 256 rows
// is as fast as two 128-row blocks and a merge, two 256-row blocks for 257 .. 512 rows
// lose 1.2 % against four 128-row blocks.
constexpr int kAttnWaves = 16;
constexpr int kSplitT = 32 * kAttnWaves; // 512: only for contexts beyond 64 blocks of 256 rows
constexpr int kMidWaves = 8;
constexpr int kMidSplitT = 32 * kMidWaves; // 256
constexpr int kSmallWaves = 4;
constexpr int kSmallSplitT = 32 * kSmallWaves; // 128
constexpr int kMaxSplits = 64; // one lane per block in the merge
constexpr int kPartStride = kRopeHeadSize + 2; // 128 partial outputs, block max, block sum

inline int attn_max_splits(int seq_len) { return ceil_div(seq_len, kSplitT); }
constexpr int kSmallBlockMaxSeq = 1024;                   // 128-row blocks up to this length,
constexpr int kMidBlockMaxSeq = kMaxSplits * kMidSplitT;  // 256-row blocks up to this one (16384), 512-row blocks beyond

// Launch shapes of the decode step: 1, 2, 4, 8 blocks of 128 rows; 8, 16, 32, 64 blocks
// of 256 rows; 512-row blocks over the whole context.
constexpr int ceil_log2(int v) { return v <= 1 ? 0 : 1 + ceil_log2((v + 1) / 2); }
constexpr int kSmallShapes = ceil_log2(kSmallBlockMaxSeq / kSmallSplitT) + 1;             // 4
constexpr int kMidFirstLog = ceil_log2(kSmallBlockMaxSeq / kMidSplitT) + 1;               // 3: 8 blocks
constexpr int kMidShapes = ceil_log2(kMaxSplits) - kMidFirstLog + 1;                      // 4
constexpr int kAttnShapes = kSmallShapes + kMidShapes + 1;
struct AttnShape {
    int waves;
    int splits;
};
inline int attn_shape_index(int rows)
{
    if (rows <= kSmallBlockMaxSeq)
        return ceil_log2(ceil_div(rows, kSmallSplitT));
    if (rows <= kMidBlockMaxSeq) {
        const int b = ceil_log2(ceil_div(rows, kMidSplitT));
        return kSmallShapes + (b > kMidFirstLog ? b - kMidFirstLog : 0);
    }
    return kAttnShapes - 1;
}
inline AttnShape attn_shape(int index, int seq_len)
{
    if (index < kSmallShapes)
        return AttnShape{kSmallWaves, 1 << index};
    if (index < kSmallShapes + kMidShapes)
        return AttnShape{kMidWaves, 1 << (kMidFirstLog + index - kSmallShapes)};
    return AttnShape{kAttnWaves, attn_max_splits(seq_len)};
}

struct AttnArgs;
void launch_attn(const AttnShape& shape, int n_heads, const AttnArgs& a);

struct AttnArgs {
    const uint16_t* q;
    const uint16_t* kcache; // layer base, rows of `dim` halfs
    const uint16_t* vcache;
    uint16_t* out; // [n_heads * 128]
    float* part;   // [n_heads][max_splits][kPartStride]
    unsigned* counters; // [n_heads], zero between launches
    const int* pos_ptr; // device-resident position, or null: attend `seq` rows
    int seq;
    int dim;
    int max_splits;
    float scale;
    // ROPE variant only: the rotation of native/rope_kernel.cu:3-26 at position rope_pos is applied to
    // the query and to row S - 1 of the key cache inside the launch, and both are written back rotated
    uint16_t* q_rw;
    uint16_t* k_rw;
    int rope_pos;
    float theta;
};

// Rotates the 8 elements a lane holds of a head's 128 (lane l16 of a 16-lane group: elements
// 8 l16 .. 8 l16 + 7; the partner of element t < 64 is element t + 64, held by lane l16 ^ 8).
__device__ __forceinline__ u32x4 rope_lane8(u32x4 mine, int l16, const float* tab /* LDS: (cos, sin) of t < 64 */)
{
    u32x4 other, r;
#pragma unroll
    for (int k = 0; k < 4; ++k)
        other[k] = static_cast<uint32_t>(__shfl_xor(static_cast<int>(mine[k]), 8, 64));
    const bool low = l16 < 8;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        uint32_t packed = 0;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int t = (l16 & 7) * 8 + 2 * k + e;
            const uint16_t m = static_cast<uint16_t>(mine[k] >> (16 * e)), o = static_cast<uint16_t>(other[k] >> (16 * e));
            const float v0 = half_bits_to_float(low ? m : o), v1 = half_bits_to_float(low ? o : m);
            uint16_t b0, b1;
            rope_rotate(b0, b1, v0, v1, tab[2 * t], tab[2 * t + 1]);
            packed |= static_cast<uint32_t>(low ? b0 : b1) << (16 * e);
        }
        r[k] = packed;
    }
    return r;
}

template <int WAVES, bool ROPE>
__global__ __launch_bounds__(WAVES * 64) void fused_attn_kernel(AttnArgs a)
{
    constexpr int GROUPS = WAVES * 4;   // 16-lane groups, one timestep each per pass
    constexpr int SPLIT_T = GROUPS * 8; // timesteps per workgroup
    __shared__ float sc[SPLIT_T];
    __shared__ float red[WAVES][kRopeHeadSize];
    __shared__ int is_last;
    const int split = blockIdx.x, h = blockIdx.y;
    const int S = a.pos_ptr ? a.pos_ptr[0] + 1 : a.seq; // attends rows 0..pos (src/Transformer.cs:175)
    const int nsplit = (S + SPLIT_T - 1) / SPLIT_T;
    if (split >= nsplit)
        return;
    const int t0 = split * SPLIT_T;
    const int t1 = S < t0 + SPLIT_T ? S : t0 + SPLIT_T;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l16 = lane & 15, grp = wave * 4 + (lane >> 4);
    const int col = h * kRopeHeadSize + l16 * 8;

    const uint32_t cache_bytes = static_cast<uint32_t>(t1) * a.dim * 2; // rows of this block only; < 2^31: checked on the host
    const __amdgpu_buffer_rsrc_t rk = make_rsrc(a.kcache, cache_bytes), rv = make_rsrc(a.vcache, cache_bytes);
    u32x4 qv = *reinterpret_cast<const u32x4*>(a.q + col);
    u32x4 kv[8], vv[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
        kv[i] = __builtin_amdgcn_raw_buffer_load_b128(rk, ((t0 + i * GROUPS + grp) * a.dim + col) * 2, 0,
                                                      kAuxNonTemporal);
#pragma unroll
    for (int i = 0; i < 8; ++i)
        vv[i] = __builtin_amdgcn_raw_buffer_load_b128(rv, ((t0 + i * GROUPS + grp) * a.dim + col) * 2, 0,
                                                      kAuxNonTemporal);
    if constexpr (ROPE) {
        // the angles while the cache rows are on their way; every block of a head rotates the query
        // for itself (in registers), the block that holds row S - 1 rotates that row and stores it
        __shared__ float rope_tab[kRopeHeadSize];
        if (threadIdx.x < kRopeHeadSize / 2) {
            float c, sn;
            rope_cos_sin(c, sn, threadIdx.x, kRopeHeadSize, a.rope_pos, a.theta);
            rope_tab[2 * threadIdx.x] = c;
            rope_tab[2 * threadIdx.x + 1] = sn;
        }
        __syncthreads();
        qv = rope_lane8(qv, l16, rope_tab);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int row = t0 + i * GROUPS + grp;
            if (row == S - 1) { // the same for the 16 lanes of a group
                kv[i] = rope_lane8(kv[i], l16, rope_tab);
                *reinterpret_cast<u32x4*>(a.k_rw + static_cast<size_t>(row) * a.dim + col) = kv[i];
            }
        }
    }
    float s[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float acc = 0.0f;
#pragma unroll
        for (int k = 0; k < 4; ++k)
            acc = dot2(kv[i][k], qv[k], acc);
        acc = row16_sum(acc) * a.scale; // native/mat_vec_kernel.cu:71-74
        s[i] = t0 + i * GROUPS + grp < t1 ? half_bits_to_float(float_to_half_bits(acc)) : -INFINITY;
        if (l16 == 0)
            sc[i * GROUPS + grp] = s[i];
    }
    __syncthreads();
    float m = -INFINITY;
#pragma unroll
    for (int k = 0; k < SPLIT_T / 64; ++k)
        m = fmaxf(m, sc[lane + 64 * k]);
    m = wave_max(m);
    float l = 0.0f;
#pragma unroll
    for (int k = 0; k < SPLIT_T / 64; ++k)
        l += expf(sc[lane + 64 * k] - m);
    l = wave_sum(l);
    float o[8];
#pragma unroll
    for (int k = 0; k < 8; ++k)
        o[k] = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float p = expf(s[i] - m); // 0 for masked timesteps
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const h2_t v2 = as_h2(vv[i][k]);
            o[2 * k] = fmaf(p, static_cast<float>(v2[0]), o[2 * k]);
            o[2 * k + 1] = fmaf(p, static_cast<float>(v2[1]), o[2 * k + 1]);
        }
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) { // the 4 groups of a wavefront, then the wavefronts through LDS
        o[k] += __shfl_xor(o[k], 16, 64);
        o[k] += __shfl_xor(o[k], 32, 64);
    }
    if (lane < 16) {
#pragma unroll
        for (int k = 0; k < 8; ++k)
            red[wave][l16 * 8 + k] = o[k];
    }
    __syncthreads();
    float val = 0.0f;
    if (threadIdx.x < kRopeHeadSize) {
#pragma unroll
        for (int g = 0; g < WAVES; ++g)
            val += red[g][threadIdx.x];
    }
    uint16_t* out = a.out + static_cast<size_t>(h) * kRopeHeadSize;
    if (nsplit == 1) {
        if (threadIdx.x < kRopeHeadSize)
            out[threadIdx.x] = float_to_half_bits(val / l);
        if constexpr (ROPE) { // the only block of the head: all its wavefronts used the query before the barriers above
            if (threadIdx.x < 16)
                *reinterpret_cast<u32x4*>(a.q_rw + col) = qv;
        }
        return;
    }
    float* P = a.part + (static_cast<size_t>(h) * a.max_splits + split) * kPartStride;
    if (threadIdx.x < kRopeHeadSize)
        store_agent(P + threadIdx.x, val);
    if (threadIdx.x == 0) {
        store_agent(P + kRopeHeadSize, m);
        store_agent(P + kRopeHeadSize + 1, l);
    }
    wait_agent_stores(); // the partials are visible device-wide before they are announced
    __syncthreads();
    if (threadIdx.x == 0)
        is_last = add_agent(&a.counters[h], 1u) == static_cast<unsigned>(nsplit - 1);
    __syncthreads();
    if (!is_last)
        return;
    if (threadIdx.x == 0)
        store_agent(&a.counters[h], 0u); // ready for the next launch
    if constexpr (ROPE) {
        // every other block of the head read the query before it announced its partials
        if (threadIdx.x < 16)
            *reinterpret_cast<u32x4*>(a.q_rw + col) = qv;
    }
    // Merge the blocks of this head.  The partials are read with agent-scope
    // buffer loads (they were written by other workgroups of this launch); a read
    // beyond the last block returns 0, so the loads are unconditional, and the
    // first eight blocks' outputs are requested before the weights are known.
    const __amdgpu_buffer_rsrc_t rp = make_rsrc(a.part + static_cast<size_t>(h) * a.max_splits * kPartStride,
                                                static_cast<uint32_t>(nsplit) * kPartStride * sizeof(float));
    float* wsh = sc;         // per-block weights exp(m_i - M)   (nsplit <= kMaxSplits <= SPLIT_T)
    float* lsh = &red[0][0]; // the merged denominator
    const int j = threadIdx.x & (kRopeHeadSize - 1);
    float v[8] = {};
    if (threadIdx.x < kRopeHeadSize) {
#pragma unroll
        for (int u = 0; u < 8; ++u)
            v[u] = __builtin_bit_cast(float,
                                      __builtin_amdgcn_raw_buffer_load_b32(rp, (u * kPartStride + j) * 4, 0, kAuxAgent));
    }
    if (threadIdx.x < 64) { // one wavefront: block i in lane i
        const int off = (threadIdx.x * kPartStride + kRopeHeadSize) * 4;
        const bool have = static_cast<int>(threadIdx.x) < nsplit;
        const float mi = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rp, off, 0, kAuxAgent));
        const float li = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rp, off + 4, 0, kAuxAgent));
        const float M = wave_max(have ? mi : -INFINITY);
        const float w = have ? expf(mi - M) : 0.0f;
        wsh[threadIdx.x] = w;
        const float L = wave_sum(w * li);
        if (threadIdx.x == 0)
            lsh[0] = L;
    }
    __syncthreads();
    if (threadIdx.x < kRopeHeadSize) {
        float O = 0.0f;
        for (int i0 = 0;;) { // block order is fixed: deterministic
#pragma unroll
            for (int u = 0; u < 8; ++u)
                O = fmaf(i0 + u < nsplit ? wsh[i0 + u] : 0.0f, v[u], O);
            i0 += 8;
            if (i0 >= nsplit)
                break;
#pragma unroll
            for (int u = 0; u < 8; ++u)
                v[u] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                                     rp, ((i0 + u) * kPartStride + j) * 4, 0, kAuxAgent));
        }
        out[threadIdx.x] = float_to_half_bits(O / lsh[0]);
    }
}

template <int WAVES>
static void launch_attn_waves(const dim3 grid, const AttnArgs& a)
{
    if (a.q_rw)
        hipLaunchKernelGGL((fused_attn_kernel<WAVES, true>), grid, dim3(WAVES * 64), 0, ctx().stream, a);
    else
        hipLaunchKernelGGL((fused_attn_kernel<WAVES, false>), grid, dim3(WAVES * 64), 0, ctx().stream, a);
}

void launch_attn(const AttnShape& shape, int n_heads, const AttnArgs& a)
{
    const dim3 grid(shape.splits, n_heads);
    switch (shape.waves) {
    case 2: launch_attn_waves<2>(grid, a); break;
    case 4: launch_attn_waves<4>(grid, a); break;
    case 8: launch_attn_waves<8>(grid, a); break;
    default: launch_attn_waves<kAttnWaves>(grid, a); break;
    }
}

// ---------------------------------------------------------------- step state
// state[0] = position, state[1] = first position whose token is generated,
// state[2] = 1 to advance the position after sampling, state[3] = number of
// token slots (the context length: the token after the last row has no slot and
// is not stored), state[4] = a spare slot for that token when the host asks for
// it, state[5] = the number of persistent steps so far, incremented by a one-thread
// launch right before each of them and by nothing else (the persistent step derives
// its hand-over tags from it: successive tags of a word differ by 1 .. n_layers + 2),
// state[6] = the persistent step's error flag (persist.hpp names the indices);
// the 128 floats behind the 8 ints hold (cos, sin) of the position's RoPE
// angles, so the 32 QKV launches of a step do not each call powf/cosf/sinf.
constexpr size_t kStateBytes = kStateInts * sizeof(int) + kRopeHeadSize * sizeof(float);

__device__ __forceinline__ void write_rope_table(int* state, int i, int pos, float theta)
{
    float c, s;
    rope_cos_sin(c, s, i, kRopeHeadSize, pos, theta);
    float* tab = reinterpret_cast<float*>(state + kStateInts);
    tab[2 * i] = c;
    tab[2 * i + 1] = s;
}

__global__ void set_state_kernel(int* state, int pos, int n_prompt, int advance, int n_slots, float theta)
{
    if (threadIdx.x == 0) {
        state[0] = pos;
        state[1] = n_prompt;
        state[2] = advance;
        state[3] = n_slots;
    }
    if (threadIdx.x < kRopeHeadSize / 2)
        write_rope_table(state, threadIdx.x, pos, theta);
}

__global__ void bump_serial_kernel(int* state)
{
    if (threadIdx.x == 0)
        state[kStateSerial] = state[kStateSerial] + 1;
}

// Sampler.Sample greedy branch (src/Sampler.cs:44-47) against the device state:
// tokens[pos+1] = argmax(logits) iff pos+1 >= n_prompt; lowest index wins ties.
__global__ __launch_bounds__(1024) void argmax_step_kernel(const uint16_t* x, int size, int* tokens, int* state,
                                                           float theta)
{
    __shared__ float sv[16];
    __shared__ int si[16];
    // read by every thread before thread 0 updates the position (one 16-byte scalar load)
    const int pos0 = state[0], n_prompt = state[1], advance0 = state[2], n_slots = state[3];
    if (advance0 && threadIdx.x >= 64 && threadIdx.x < 64 + kRopeHeadSize / 2)
        write_rope_table(state, threadIdx.x - 64, pos0 + 1, theta); // for the next step
    const int best = block1024_argmax(x, size, sv, si);
    if (threadIdx.x == 0) {
        if (pos0 + 1 >= n_prompt && pos0 + 1 < n_slots)
            tokens[pos0 + 1] = best;
        if (advance0)
            state[0] = pos0 + 1;
    }
}

// Sampler.Sample's stochastic branch (src/Sampler.cs:48-67) against the device
// state: the token at pos+1 is drawn with the coin of (seed, pos+1) iff
// pos+1 >= n_prompt; then the position advances like in argmax_step_kernel.
struct SampleStepArgs {
    uint16_t* logits;
    int* indices;
    int size;
    int* tokens;
    int* state;
    uint16_t* keys2; // second buffer of the global-memory sort (vocabularies beyond kSortLdsItems)
    int* values2;
    float temperature, top_p;
    unsigned long long seed;
    float theta;
};

template <bool LDS_SORT>
__device__ __forceinline__ void sample_step(const SampleStepArgs& a, SamplerLds& lds, SortLds* buf)
{
    const int pos0 = a.state[0], n_prompt = a.state[1], advance0 = a.state[2], n_slots = a.state[3];
    if (advance0 && threadIdx.x >= 64 && threadIdx.x < 64 + kRopeHeadSize / 2)
        write_rope_table(a.state, threadIdx.x - 64, pos0 + 1, a.theta); // for the next step
    if (pos0 + 1 >= n_prompt && pos0 + 1 < n_slots) { // uniform over the workgroup
        const float coin = sampler_coin(a.seed, pos0 + 1);
        const int token = sample_dev<LDS_SORT ? 4 : 8, LDS_SORT, true>(a.logits, a.indices, a.size, a.temperature, a.top_p,
                                                                 coin, a.keys2, a.values2, lds, buf);
        if (threadIdx.x == 0)
            a.tokens[pos0 + 1] = token;
    }
    __syncthreads(); // every thread has read the state
    if (threadIdx.x == 0) {
        if (advance0)
            a.state[0] = pos0 + 1;
    }
}

__global__ __launch_bounds__(kSampBlock) void sample_step_kernel(SampleStepArgs a)
{
    __shared__ SamplerLds lds;
    __shared__ SortLds buf;
    sample_step<true>(a, lds, &buf);
}

__global__ __launch_bounds__(kSampBlock) void sample_step_big_kernel(SampleStepArgs a)
{
    __shared__ SamplerLds lds;
    sample_step<false>(a, lds, nullptr);
}

} // namespace l2

struct llama2_decoder {
    llama2_config cfg;
    std::vector<llama2_layer_weights> layers;
    llama2_transformer_weights w;
    llama2_run_state s;
    int mode;
    int kv_dim;
    int head_size;
    // fused path
    int* state = nullptr;
    float* attn_part = nullptr;
    unsigned* counters = nullptr;
    // One captured graph per (kind, attention launch shape).  Kinds: Transformer.Forward;
    // Forward + greedy sample + position advance; Forward + stochastic sample + position
    // advance, captured for the parameters below.
    enum { kGraphForward, kGraphStep, kGraphStepSampled, kGraphKinds };
    // the last shape index is the persistent step (one launch for any history up to kPMaxRows rows)
    hipGraphExec_t graphs[kGraphKinds][l2::kAttnShapes + 1] = {};
    float sampled_temperature = 0.0f, sampled_top_p = 0.0f;
    unsigned long long sampled_seed = 0;
    // persistent step (LLAMA2_DECODE_PERSISTENT): kernel variant, per-layer pointer table and
    // hand-over buffers on the device, and the launch arguments
    int persist_variant = -1;
    l2::PersistLayer* persist_layers = nullptr;
    void* persist_scratch = nullptr;
    l2::PersistArgs pa{};
};

using namespace l2;

namespace {

int check_qw(const llama2_qweight& q, const char* what, int layer)
{
    L2_CHECK(q.weight && q.zeros && q.scales, "llama2_decode_create: layer %d %s tensor has a null pointer", layer,
             what);
    L2_CHECK(aligned(q.weight, 16), "llama2_decode_create: layer %d %s weights must be 16-byte aligned", layer, what);
    return LLAMA2_OK;
}

#define L2_TRY(expr)          \
    do {                      \
        int rc_ = (expr);     \
        if (rc_ != LLAMA2_OK) \
            return rc_;       \
    } while (0)

// The ten module calls per layer, in the reference's order and with the
// reference's argument derivations (file:line beside each call).
int forward_modules(llama2_decoder* d, int position, int next_position)
{
    const llama2_config& c = d->cfg;
    const llama2_run_state& s = d->s;
    const int dim = c.dim, hidden = c.hidden_dim, hs = d->head_size, kv = d->kv_dim;
    const float scale = 1.0f / sqrtf(static_cast<float>(hs)); // Transformer.cs:161
    const int ss = ceil_div(dim, 128), ws = ceil_div(dim, 32) * 4, zs = ceil_div(ss, 8);
    const int hss = ceil_div(hidden, 128), hws = ceil_div(hidden, 32) * 4, hzs = ceil_div(hss, 8);

    L2_TRY(llama2_embedding(s.x, d->w.token_embedding_table, dim, s.tokens, position)); // :163
    for (int i = 0; i < c.n_layers; ++i) {
        const llama2_layer_weights& L = d->layers[i];
        L2_TRY(llama2_rmsnorm(s.xb, s.x, L.rms_attention, dim, 1e-5f)); // :167
        const size_t layer_offset = static_cast<size_t>(i) * c.seq_len * kv; // :169
        const size_t row = layer_offset + static_cast<size_t>(position) * kv; // QKVMatVec.cs:25
        L2_TRY(llama2_qkv_mat_vec(s.q, s.key_cache + row, s.value_cache + row, s.xb, L.query.weight, L.query.zeros,
                                  L.query.scales, L.key.weight, L.key.zeros, L.key.scales, L.value.weight,
                                  L.value.zeros, L.value.scales, dim, dim, zs, ss, ws)); // :171
        L2_TRY(llama2_rope(s.q, s.key_cache + row, c.n_kv_heads, hs, position, c.rope_theta, c.n_heads)); // :173
        const int seq = next_position; // :175
        L2_TRY(llama2_mat_vec_strided(s.attention, s.q, s.key_cache + layer_offset, hs, seq, hs, hs, dim, seq, scale,
                                      c.n_heads)); // :153, MatVecStrided.cs:18
        L2_TRY(llama2_softmax(s.attention, seq, c.n_heads)); // :154
        L2_TRY(llama2_vec_mat(s.xb, s.attention, s.value_cache + layer_offset, hs, seq, hs, hs, dim,
                              c.n_heads)); // :155, VecMat.cs:19
        L2_TRY(llama2_mat_vec_residual_int4(s.x, s.xb, L.output.weight, L.output.zeros, L.output.scales, dim, dim, zs,
                                            ss, ws)); // :177
        L2_TRY(llama2_rmsnorm(s.xb, s.x, L.rms_feed_forward, dim, 1e-5f)); // :179
        L2_TRY(llama2_mat_vec_swiglu(s.h, s.xb, L.gate.weight, L.gate.zeros, L.gate.scales, L.up.weight, L.up.zeros,
                                     L.up.scales, dim, hidden, zs, ss, ws)); // :181
        L2_TRY(llama2_mat_vec_residual_int4(s.x, s.h, L.down.weight, L.down.zeros, L.down.scales, hidden, dim, hzs,
                                            hss, hws)); // :183
    }
    L2_TRY(llama2_rmsnorm(s.x, s.x, d->w.rms_final_weight, dim, 1e-5f)); // :187
    L2_TRY(llama2_mat_vec(s.logits, s.x, d->w.classifier_weights, dim, c.vocab_size)); // :189
    return LLAMA2_OK;
}

QW qw(const llama2_qweight& q) { return QW{q.weight, q.zeros, q.scales}; }

constexpr int kPersistShape = kAttnShapes; // index of the persistent step among the launch shapes

// Device-side tables and hand-over buffers of the persistent step.
int persist_setup(llama2_decoder* d)
{
    const llama2_config& c = d->cfg;
    std::vector<PersistLayer> table(c.n_layers);
    for (int i = 0; i < c.n_layers; ++i) {
        const llama2_layer_weights& L = d->layers[i];
        table[i] = PersistLayer{qw(L.query), qw(L.key),  qw(L.value),     qw(L.output),      qw(L.gate),
                                qw(L.up),    qw(L.down), L.rms_attention, L.rms_feed_forward};
    }
    const size_t table_bytes = sizeof(PersistLayer) * table.size();
    L2_HIP(hipMalloc(reinterpret_cast<void**>(&d->persist_layers), table_bytes));
    L2_HIP(hipMemcpyAsync(d->persist_layers, table.data(), table_bytes, hipMemcpyHostToDevice, ctx().stream));
    const size_t scratch_bytes = persist_scratch_bytes(c.dim, c.hidden_dim, c.n_heads);
    L2_HIP(hipMalloc(&d->persist_scratch, scratch_bytes));
    L2_HIP(hipMemsetAsync(d->persist_scratch, 0, scratch_bytes, ctx().stream)); // tag 0: no word is ready
    L2_HIP(hipStreamSynchronize(ctx().stream)); // `table` goes out of scope
    PersistArgs& a = d->pa;
    a = PersistArgs{};
    a.layers = d->persist_layers;
    a.n_layers = c.n_layers, a.dim = c.dim, a.hidden = c.hidden_dim, a.n_heads = c.n_heads, a.vocab = c.vocab_size;
    a.seq_len = c.seq_len;
    a.ss_d = ceil_div(c.dim, 128), a.ws_d = ceil_div(c.dim, 32) * 4, a.zs_d = ceil_div(a.ss_d, 8);
    a.ss_h = ceil_div(c.hidden_dim, 128), a.ws_h = ceil_div(c.hidden_dim, 32) * 4, a.zs_h = ceil_div(a.ss_h, 8);
    a.eps = 1e-5f;
    a.scale = 1.0f / sqrtf(static_cast<float>(d->head_size));
    a.embedding = d->w.token_embedding_table, a.tokens = d->s.tokens;
    a.rms_final = d->w.rms_final_weight, a.classifier = d->w.classifier_weights, a.logits = d->s.logits;
    a.kcache = d->s.key_cache, a.vcache = d->s.value_cache;
    a.state = d->state;
    a.spin_limit = kPersistSpinLimit;
    persist_bind_scratch(a, d->persist_scratch);
#ifdef L2_PERSIST_TRACE
    a.trace = nullptr;
    if (const char* addr = getenv("LLAMA2_PERSIST_TRACE")) // a device buffer of n_layers * 4 * kPTracePoints 64-bit words
        a.trace = reinterpret_cast<unsigned long long*>(strtoull(addr, nullptr, 0));
#endif
    return LLAMA2_OK;
}

// The same step in 5 launches per layer; the position comes from d->state, and
// `shape` (attn_shape_index of an upper bound of position + 1) sizes the attention grid.
int forward_fused(llama2_decoder* d, int shape)
{
    if (shape == kPersistShape) { // the whole step in one launch, behind the bump of its own step counter
        hipLaunchKernelGGL(bump_serial_kernel, dim3(1), dim3(64), 0, ctx().stream, d->state);
        L2_LAUNCH_CHECK("bump_serial_kernel");
        return persist_launch(d->persist_variant, d->pa, ctx().num_cus);
    }
    const AttnShape as = attn_shape(shape, d->cfg.seq_len);
    const llama2_config& c = d->cfg;
    const llama2_run_state& s = d->s;
    const int dim = c.dim, hidden = c.hidden_dim;
    const int ss = ceil_div(dim, 128), ws = ceil_div(dim, 32) * 4, zs = ceil_div(ss, 8);
    const int hss = ceil_div(hidden, 128), hws = ceil_div(hidden, 32) * 4, hzs = ceil_div(hss, 8);
    for (int i = 0; i < c.n_layers; ++i) {
        const llama2_layer_weights& L = d->layers[i];
        const size_t layer_offset = static_cast<size_t>(i) * c.seq_len * d->kv_dim;
        {
            Int4Args a{}; // :163 (layer 0) + :167 + :171 + :173
            a.m[0] = qw(L.query), a.m[1] = qw(L.key), a.m[2] = qw(L.value);
            a.out[0] = s.q, a.out[1] = s.key_cache + layer_offset, a.out[2] = s.value_cache + layer_offset;
            a.x = s.x;
            a.K = dim, a.N = dim, a.ws = ws, a.ss = ss, a.zs = zs, a.n_tensors = 3;
            a.gamma = L.rms_attention, a.eps = 1e-5f;
            if (i == 0)
                a.embedding = d->w.token_embedding_table, a.tokens = s.tokens, a.vocab = c.vocab_size, a.x_out = s.x;
            a.pos_ptr = d->state;
            a.kv_dim = d->kv_dim, a.theta = c.rope_theta;
            a.rope_table = reinterpret_cast<const float*>(d->state + kStateInts);
            L2_TRY((launch_int4<QKV_ROPE, STAGE_RMSNORM>("fused qkv", a)));
        }
        {
            AttnArgs a{}; // :175 (MultiHeadAttention :150-156)
            a.q = s.q, a.kcache = s.key_cache + layer_offset, a.vcache = s.value_cache + layer_offset, a.out = s.xb;
            a.part = d->attn_part, a.counters = d->counters, a.pos_ptr = d->state;
            a.dim = dim, a.max_splits = as.splits;
            a.scale = 1.0f / sqrtf(static_cast<float>(d->head_size));
            launch_attn(as, c.n_heads, a);
            L2_LAUNCH_CHECK("fused attention");
        }
        {
            Int4Args a{}; // :177
            a.m[0] = qw(L.output), a.out[0] = s.x, a.x = s.xb;
            a.K = dim, a.N = dim, a.ws = ws, a.ss = ss, a.zs = zs, a.n_tensors = 1;
            L2_TRY((launch_int4<RESIDUAL, STAGE_X>("fused o-proj", a)));
        }
        {
            Int4Args a{}; // :179 + :181
            a.m[0] = qw(L.gate), a.m[1] = qw(L.up), a.out[0] = s.h, a.x = s.x;
            a.K = dim, a.N = hidden, a.ws = ws, a.ss = ss, a.zs = zs, a.n_tensors = 1;
            a.gamma = L.rms_feed_forward, a.eps = 1e-5f;
            L2_TRY((launch_int4<SWIGLU, STAGE_RMSNORM>("fused swiglu", a)));
        }
        {
            Int4Args a{}; // :183
            a.m[0] = qw(L.down), a.out[0] = s.x, a.x = s.h;
            a.K = hidden, a.N = dim, a.ws = hws, a.ss = hss, a.zs = hzs, a.n_tensors = 1;
            L2_TRY((launch_int4<RESIDUAL, STAGE_X>("fused down-proj", a)));
        }
    }
    L2_TRY(llama2_rmsnorm(s.x, s.x, d->w.rms_final_weight, dim, 1e-5f)); // :187
    L2_TRY(llama2_mat_vec(s.logits, s.x, d->w.classifier_weights, dim, c.vocab_size)); // :189
    return LLAMA2_OK;
}

int launch_argmax_step(llama2_decoder* d)
{
    hipLaunchKernelGGL(argmax_step_kernel, dim3(1), dim3(1024), 0, ctx().stream, d->s.logits, d->cfg.vocab_size,
                       d->s.tokens, d->state, d->cfg.rope_theta);
    L2_LAUNCH_CHECK("argmax_step_kernel");
    return LLAMA2_OK;
}

int launch_sample_step(llama2_decoder* d, float temperature, float top_p, unsigned long long seed)
{
    SampleStepArgs a{d->s.logits, d->s.indices, d->cfg.vocab_size, d->s.tokens, d->state, ctx().sort_keys,
                     ctx().sort_values, temperature, top_p, seed, d->cfg.rope_theta};
    if (a.size <= kSortLdsItems)
        hipLaunchKernelGGL(sample_step_kernel, dim3(1), dim3(kSampBlock), 0, ctx().stream, a);
    else
        hipLaunchKernelGGL(sample_step_big_kernel, dim3(1), dim3(kSampBlock), 0, ctx().stream, a);
    L2_LAUNCH_CHECK("sample_step_kernel");
    return LLAMA2_OK;
}

int check_sampling(const char* fn, const llama2_decoder* d, float temperature)
{
    L2_CHECK(temperature > 0.0f, "%s: temperature=%g must be positive", fn, static_cast<double>(temperature));
    L2_CHECK(d->s.indices, "%s: the run state has no indices buffer (vocab_size ints)", fn);
    L2_CHECK(aligned(d->s.indices, 16), "%s: run-state indices must be 16-byte aligned", fn);
    if (d->cfg.vocab_size > LLAMA2_MAX_SAMPLER_SIZE)
        return fail(LLAMA2_ERR_UNSUPPORTED, "%s: vocab_size=%d exceeds the sampler limit %d", fn, d->cfg.vocab_size,
                    LLAMA2_MAX_SAMPLER_SIZE);
    return LLAMA2_OK;
}

// Where the token of `next_position` goes: its slot of the run state's tokens, or, for the token
// after the last row of the context (the reference's tokens buffer has no slot for it,
// src/RunState.cs:52), a spare slot of the decoder's own.
struct TokenSlot {
    int* tokens;
    int index;
};
TokenSlot token_slot(llama2_decoder* d, int next_position)
{
    if (next_position < d->cfg.seq_len)
        return TokenSlot{d->s.tokens, next_position};
    return TokenSlot{d->state, kSpareTokenSlot};
}

int set_state(llama2_decoder* d, int pos, int n_prompt, int advance)
{
    hipLaunchKernelGGL(set_state_kernel, dim3(1), dim3(64), 0, ctx().stream, d->state, pos, n_prompt, advance,
                       d->cfg.seq_len, d->cfg.rope_theta);
    L2_LAUNCH_CHECK("set_state_kernel");
    return LLAMA2_OK;
}

int capture(hipGraphExec_t* exec, llama2_decoder* d, int kind, int shape)
{
    L2_HIP(hipStreamBeginCapture(ctx().stream, hipStreamCaptureModeThreadLocal));
    ctx().capturing = true;
    int rc = forward_fused(d, shape);
    if (rc == LLAMA2_OK && kind == llama2_decoder::kGraphStepSampled)
        rc = launch_sample_step(d, d->sampled_temperature, d->sampled_top_p, d->sampled_seed);
    else if (rc == LLAMA2_OK && kind == llama2_decoder::kGraphStep)
        rc = launch_argmax_step(d);
    ctx().capturing = false;
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(ctx().stream, &g);
    if (rc != LLAMA2_OK) {
        if (g)
            (void)hipGraphDestroy(g);
        return rc;
    }
    if (e != hipSuccess)
        return hip_fail(e, "hipStreamEndCapture");
    e = hipGraphInstantiate(exec, g, nullptr, nullptr, 0);
    (void)hipGraphDestroy(g);
    if (e != hipSuccess)
        return hip_fail(e, "hipGraphInstantiate");
    return LLAMA2_OK;
}

// The shape for a step at `position`.  While the caller captures a graph of its own the
// step may be replayed at any later position, so it gets the shape of the whole context.
int step_shape(const llama2_decoder* d, int position)
{
    const int rows = ctx().capturing ? d->cfg.seq_len : position + 1;
    if (d->persist_variant >= 0 && rows <= kPMaxRows)
        return kPersistShape;
    return attn_shape_index(rows);
}

// Launches one step of `kind`: the captured graph of that shape (captured on first use)
// in graph mode, the same launches otherwise.
int launch_step(llama2_decoder* d, int kind, int position)
{
    const int shape = step_shape(d, position);
    if ((d->mode & LLAMA2_DECODE_GRAPH) && !ctx().capturing) {
        hipGraphExec_t& g = d->graphs[kind][shape];
        if (!g)
            L2_TRY(capture(&g, d, kind, shape));
        L2_HIP(hipGraphLaunch(g, ctx().stream));
        return LLAMA2_OK;
    }
    L2_TRY(forward_fused(d, shape));
    if (kind == llama2_decoder::kGraphStepSampled)
        return launch_sample_step(d, d->sampled_temperature, d->sampled_top_p, d->sampled_seed);
    if (kind == llama2_decoder::kGraphStep)
        return launch_argmax_step(d);
    return LLAMA2_OK;
}

void release(llama2_decoder* d)
{
    for (auto& kind : d->graphs)
        for (hipGraphExec_t g : kind)
            if (g)
                (void)hipGraphExecDestroy(g);
    if (d->state)
        (void)hipFree(d->state);
    if (d->persist_layers)
        (void)hipFree(d->persist_layers);
    if (d->persist_scratch)
        (void)hipFree(d->persist_scratch);
    if (d->attn_part)
        (void)hipFree(d->attn_part);
    if (d->counters)
        (void)hipFree(d->counters);
    delete d;
}

// Argument checks shared by the two attention entry points; on success *shape is the launch
// shape the decode step would pick for this length, with exactly the blocks it needs.
int check_attention(const char* fn, const void* output, const void* query, const void* key, const void* value,
                    int head_size, int dim, int seq_length, int n_heads, AttnShape* shape)
{
    L2_CHECK(output && query && key && value, "%s: null pointer", fn);
    L2_CHECK(seq_length > 0 && n_heads > 0 && dim > 0, "%s: seq_length=%d n_heads=%d dim=%d must be positive", fn,
             seq_length, n_heads, dim);
    if (head_size != kRopeHeadSize)
        return fail(LLAMA2_ERR_UNSUPPORTED, "%s: head_size=%d, only 128 is implemented (use the three modules)", fn,
                    head_size);
    L2_CHECK(dim % 8 == 0 && dim >= n_heads * head_size, "%s: dim=%d must be a multiple of 8 and hold %d heads", fn, dim,
             n_heads);
    L2_CHECK(aligned(query, 16) && aligned(key, 16) && aligned(value, 16), "%s: q/k/v must be 16-byte aligned", fn);
    L2_CHECK(n_heads <= kMaxAttnHeads, "%s: n_heads=%d exceeds %d", fn, n_heads, kMaxAttnHeads);
    L2_CHECK((static_cast<long long>(seq_length) + kSplitT) * dim * 2 < (1ll << 31),
             "%s: seq_length * dim = %lld is too large", fn, static_cast<long long>(seq_length) * dim);
    L2_CHECK(seq_length <= kMaxSplits * kSplitT, "%s: seq_length=%d exceeds %d", fn, seq_length, kMaxSplits * kSplitT);
    *shape = attn_shape(attn_shape_index(seq_length), seq_length);
    const int forced = ctx().attn_waves; // LLAMA2_ATTN_WAVES: 2, 4, 8 or 16 wavefronts (64 .. 512 rows) per block
    if ((forced == 2 || forced == 4 || forced == 8 || forced == 16) && ceil_div(seq_length, forced * 32) <= kMaxSplits)
        shape->waves = forced;
    shape->splits = ceil_div(seq_length, shape->waves * 32);
    return LLAMA2_OK;
}

} // namespace

extern "C" {

int llama2_multi_head_attention(llama2_half* output, const llama2_half* query, const llama2_half* key,
                                const llama2_half* value, int head_size, int dim, int seq_length, float scale,
                                int n_heads)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_multi_head_attention";
    AttnShape shape{};
    L2_TRY(check_attention(fn, output, query, key, value, head_size, dim, seq_length, n_heads, &shape));
    if (shape.splits > 1)
        L2_TRY(ensure_attn_partials(sizeof(float) * static_cast<size_t>(n_heads) * shape.splits * kPartStride));
    AttnArgs a{};
    a.q = query, a.kcache = key, a.vcache = value, a.out = output;
    a.part = ctx().attn_partials, a.counters = ctx().attn_counters, a.pos_ptr = nullptr, a.seq = seq_length;
    a.dim = dim, a.max_splits = shape.splits, a.scale = scale;
    launch_attn(shape, n_heads, a);
    L2_LAUNCH_CHECK(fn);
    return LLAMA2_OK;
}

int llama2_rope_multi_head_attention(llama2_half* output, llama2_half* query, llama2_half* key,
                                     const llama2_half* value, int head_size, int dim, int seq_length, float scale,
                                     int n_heads, int pos, float theta)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_rope_multi_head_attention";
    AttnShape shape{};
    L2_TRY(check_attention(fn, output, query, key, value, head_size, dim, seq_length, n_heads, &shape));
    L2_CHECK(pos >= 0, "%s: pos=%d is negative", fn, pos);
    L2_CHECK(!overlap(output, static_cast<size_t>(n_heads) * head_size * 2, query, static_cast<size_t>(n_heads) * head_size * 2),
             "%s: output and query overlap", fn);
    if (shape.splits > 1)
        L2_TRY(ensure_attn_partials(sizeof(float) * static_cast<size_t>(n_heads) * shape.splits * kPartStride));
    AttnArgs a{};
    a.q = query, a.kcache = key, a.vcache = value, a.out = output;
    a.part = ctx().attn_partials, a.counters = ctx().attn_counters, a.pos_ptr = nullptr, a.seq = seq_length;
    a.dim = dim, a.max_splits = shape.splits, a.scale = scale;
    a.q_rw = query, a.k_rw = key, a.rope_pos = pos, a.theta = theta;
    launch_attn(shape, n_heads, a);
    L2_LAUNCH_CHECK(fn);
    return LLAMA2_OK;
}

int llama2_decode_create(llama2_decoder** decoder, const llama2_config* config,
                         const llama2_transformer_weights* weights, const llama2_run_state* state, int mode)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_decode_create";
    L2_CHECK(decoder && config && weights && state, "%s: null argument", fn);
    *decoder = nullptr;
    L2_CHECK(!ctx().capturing, "%s: not allowed during graph capture", fn);
    const llama2_config& c = *config;
    L2_CHECK(c.dim > 0 && c.hidden_dim > 0 && c.n_layers > 0 && c.n_heads > 0 && c.n_kv_heads > 0 &&
                 c.vocab_size > 0 && c.seq_len > 0,
             "%s: non-positive field in config", fn);
    L2_CHECK(c.dim % c.n_heads == 0, "%s: dim=%d is not a multiple of n_heads=%d", fn, c.dim, c.n_heads);
    L2_CHECK(c.rope_theta == 10000.0f, "%s: Invalid model config (rope_theta=%g, expected 10000)", fn,
             static_cast<double>(c.rope_theta)); // src/Config.cs:27-28
    const int kv_dim = c.dim * c.n_kv_heads / c.n_heads;
    if (kv_dim != c.dim) // src/Transformer.cs:53-56
        return fail(LLAMA2_ERR_UNSUPPORTED, "%s: Differing kvDim dimention not currently supported (kv_dim=%d, dim=%d)",
                    fn, kv_dim, c.dim);
    if (c.seq_len > LLAMA2_MAX_SOFTMAX_SIZE)
        return fail(LLAMA2_ERR_UNSUPPORTED, "%s: seq_len=%d exceeds the softmax limit %d", fn, c.seq_len,
                    LLAMA2_MAX_SOFTMAX_SIZE);
    L2_CHECK(mode >= 0 && mode <= (LLAMA2_DECODE_FUSED | LLAMA2_DECODE_GRAPH | LLAMA2_DECODE_PERSISTENT),
             "%s: unknown mode %d", fn, mode);
    const bool fused = (mode & LLAMA2_DECODE_FUSED) != 0;
    if ((mode & (LLAMA2_DECODE_GRAPH | LLAMA2_DECODE_PERSISTENT)) && !fused)
        return fail(LLAMA2_ERR_UNSUPPORTED,
                    "%s: LLAMA2_DECODE_GRAPH and LLAMA2_DECODE_PERSISTENT need LLAMA2_DECODE_FUSED (the module sequence "
                    "takes the position by value)", fn);
    int variant = -1;
    if (mode & LLAMA2_DECODE_PERSISTENT) {
        variant = persist_variant(c.dim, c.hidden_dim, c.n_heads, ctx().num_cus);
        if (variant < 0)
            return fail(LLAMA2_ERR_UNSUPPORTED,
                        "%s: no persistent step for dim %d, hidden_dim %d, %d heads on %d compute units; drop "
                        "LLAMA2_DECODE_PERSISTENT", fn, c.dim, c.hidden_dim, c.n_heads, ctx().num_cus);
    }
    if (fused) {
        const int head_size = c.dim / c.n_heads;
        if (head_size != kRopeHeadSize || c.dim % 8 || c.hidden_dim % 8 ||
            chunk_columns(ceil_div(c.dim, 32) * 4) > kMaxChunkColumns ||
            chunk_columns(ceil_div(c.hidden_dim, 32) * 4) > kMaxChunkColumns)
            return fail(LLAMA2_ERR_UNSUPPORTED,
                        "%s: the fused step needs head_size 128 and dim, hidden_dim multiples of 8 up to 16384 "
                        "(got head_size %d, dim %d, hidden_dim %d); use LLAMA2_DECODE_MODULES",
                        fn, head_size, c.dim, c.hidden_dim);
        if (attn_max_splits(c.seq_len) > kMaxSplits ||
            (static_cast<long long>(c.seq_len) + kSplitT) * c.dim * 2 >= (1ll << 31))
            return fail(LLAMA2_ERR_UNSUPPORTED, "%s: seq_len=%d is too long for the fused attention (dim %d)", fn,
                        c.seq_len, c.dim);
    }
    L2_CHECK(weights->token_embedding_table && weights->classifier_weights && weights->rms_final_weight &&
                 weights->layers,
             "%s: null pointer in weights", fn);
    for (int i = 0; i < c.n_layers; ++i) {
        const llama2_layer_weights& L = weights->layers[i];
        L2_TRY(check_qw(L.query, "query", i));
        L2_TRY(check_qw(L.key, "key", i));
        L2_TRY(check_qw(L.value, "value", i));
        L2_TRY(check_qw(L.output, "output", i));
        L2_TRY(check_qw(L.gate, "gate", i));
        L2_TRY(check_qw(L.up, "up", i));
        L2_TRY(check_qw(L.down, "down", i));
        L2_CHECK(L.rms_attention && L.rms_feed_forward, "%s: layer %d has a null rmsnorm weight", fn, i);
    }
    L2_CHECK(state->x && state->xb && state->h && state->q && state->attention && state->logits &&
                 state->key_cache && state->value_cache && state->tokens,
             "%s: null pointer in run state", fn);
    for (const void* p : {static_cast<const void*>(state->x), static_cast<const void*>(state->xb),
                          static_cast<const void*>(state->h), static_cast<const void*>(state->q),
                          static_cast<const void*>(state->key_cache), static_cast<const void*>(state->value_cache),
                          static_cast<const void*>(state->logits)})
        L2_CHECK(aligned(p, 16), "%s: run-state buffers must be 16-byte aligned", fn);
    llama2_decoder* d = new (std::nothrow) llama2_decoder();
    L2_CHECK(d, "%s: out of host memory", fn);
    d->cfg = c;
    d->layers.assign(weights->layers, weights->layers + c.n_layers);
    d->w = *weights;
    d->w.layers = d->layers.data();
    d->s = *state;
    d->mode = mode;
    d->kv_dim = kv_dim;
    d->head_size = c.dim / c.n_heads;
    {
        hipError_t e = hipMalloc(reinterpret_cast<void**>(&d->state), kStateBytes);
        if (e == hipSuccess)
            e = hipMemsetAsync(d->state, 0, kStateBytes, ctx().stream);
        if (e == hipSuccess)
            e = hipStreamSynchronize(ctx().stream);
        if (e != hipSuccess) {
            release(d);
            return hip_fail(e, "llama2_decode_create: state allocation");
        }
    }
    if (fused) {
        hipError_t e = hipMalloc(reinterpret_cast<void**>(&d->attn_part),
                          sizeof(float) * static_cast<size_t>(c.n_heads) * kMaxSplits * kPartStride);
        if (e == hipSuccess)
            e = hipMalloc(reinterpret_cast<void**>(&d->counters), sizeof(unsigned) * c.n_heads);
        if (e == hipSuccess)
            e = hipMemsetAsync(d->counters, 0, sizeof(unsigned) * c.n_heads, ctx().stream);
        if (e == hipSuccess)
            e = hipStreamSynchronize(ctx().stream);
        if (e != hipSuccess) {
            release(d);
            return hip_fail(e, "llama2_decode_create: scratch allocation");
        }
        if (variant >= 0) {
            const int rc = persist_setup(d);
            if (rc != LLAMA2_OK) {
                release(d);
                return rc;
            }
            d->persist_variant = variant;
        }
        if (mode & LLAMA2_DECODE_GRAPH) { // every shape this context can reach, so that no step pays for a capture
            int rc = LLAMA2_OK;
            if (variant >= 0) {
                rc = capture(&d->graphs[llama2_decoder::kGraphForward][kPersistShape], d, llama2_decoder::kGraphForward,
                             kPersistShape);
                if (rc == LLAMA2_OK)
                    rc = capture(&d->graphs[llama2_decoder::kGraphStep][kPersistShape], d, llama2_decoder::kGraphStep,
                                 kPersistShape);
            }
            // the launch sequence serves what the persistent step does not: histories beyond kPMaxRows rows
            const int first = variant >= 0 ? attn_shape_index(kPMaxRows + 1) : 0;
            for (int shape = first; shape <= attn_shape_index(c.seq_len) && rc == LLAMA2_OK; ++shape) {
                rc = capture(&d->graphs[llama2_decoder::kGraphForward][shape], d, llama2_decoder::kGraphForward, shape);
                if (rc == LLAMA2_OK)
                    rc = capture(&d->graphs[llama2_decoder::kGraphStep][shape], d, llama2_decoder::kGraphStep, shape);
            }
            if (rc != LLAMA2_OK) {
                release(d);
                return rc;
            }
        }
    }
    *decoder = d;
    return LLAMA2_OK;
}

// The persistent step's failure flag is sticky (every later wait gives up at once): wherever the
// library hands a token back to the host, which waits for the GPU anyway, the flag comes with it.
static int persist_status(llama2_decoder* d, const char* fn)
{
    if (d->persist_variant < 0)
        return LLAMA2_OK;
    int flag = 0;
    L2_TRY(llama2_memcpy_d2h(&flag, d->state, static_cast<size_t>(kStateError) * sizeof(int), sizeof(int)));
    if (flag != 0)
        return fail(LLAMA2_ERR_STEP_FAILED,
                    "%s: a persistent step gave up waiting for data from another workgroup; the decoder's results "
                    "are undefined from that step on (llama2_decode_check has the details)", fn);
    return LLAMA2_OK;
}

int llama2_decode_forward(llama2_decoder* d, int position, int next_position)
{
    L2_REQUIRE_INIT();
    L2_CHECK(d, "llama2_decode_forward: null decoder");
    L2_CHECK(position >= 0 && position < d->cfg.seq_len, "llama2_decode_forward: position=%d outside [0,%d)",
             position, d->cfg.seq_len);
    L2_CHECK(next_position == position + 1, "llama2_decode_forward: next_position=%d must be position+1=%d",
             next_position, position + 1);
    if (!(d->mode & LLAMA2_DECODE_FUSED))
        return forward_modules(d, position, next_position);
    L2_TRY(set_state(d, position, INT_MAX, 0));
    return launch_step(d, llama2_decoder::kGraphForward, position);
}

int llama2_decode_sample(llama2_decoder* d, int next_position, int generate_token, int* token)
{
    L2_REQUIRE_INIT();
    L2_CHECK(d && token, "llama2_decode_sample: null argument");
    L2_CHECK(next_position >= 0 && next_position <= d->cfg.seq_len, "llama2_decode_sample: next_position=%d",
             next_position);
    const TokenSlot slot = token_slot(d, next_position);
    L2_CHECK(slot.tokens == d->s.tokens || generate_token,
             "llama2_decode_sample: next_position=%d is past the last token of the context", next_position);
    L2_TRY(llama2_argmax(d->s.logits, d->cfg.vocab_size, slot.tokens, slot.index, generate_token));
    L2_TRY(llama2_memcpy_d2h(token, slot.tokens, static_cast<size_t>(slot.index) * sizeof(int), sizeof(int)));
    return persist_status(d, "llama2_decode_sample");
}

int llama2_decode_sample_top_p(llama2_decoder* d, int next_position, int generate_token, float temperature,
                               float top_p, float coin, int* token)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_decode_sample_top_p";
    L2_CHECK(d && token, "%s: null argument", fn);
    if (temperature == 0.0f || !generate_token) // src/Sampler.cs:44-47
        return llama2_decode_sample(d, next_position, generate_token, token);
    L2_CHECK(next_position >= 0 && next_position <= d->cfg.seq_len, "%s: next_position=%d", fn, next_position);
    L2_TRY(check_sampling(fn, d, temperature));
    const TokenSlot slot = token_slot(d, next_position);
    L2_TRY(sample_launch(fn, d->s.logits, d->s.indices, d->cfg.vocab_size, temperature, top_p, coin, slot.tokens,
                         slot.index, true)); // :50-66
    L2_TRY(llama2_memcpy_d2h(token, slot.tokens, static_cast<size_t>(slot.index) * sizeof(int), sizeof(int))); // :69
    return persist_status(d, fn);
}

float llama2_sampler_coin(unsigned long long seed, int position) { return sampler_coin(seed, position); }

int llama2_decode_run_sampled(llama2_decoder* d, int position, int steps, int n_prompt, float temperature,
                              float top_p, unsigned long long seed)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_decode_run_sampled";
    L2_CHECK(d, "%s: null decoder", fn);
    if (temperature == 0.0f)
        return llama2_decode_run(d, position, steps, n_prompt);
    L2_CHECK(position >= 0 && steps >= 0 && position + steps <= d->cfg.seq_len,
             "%s: position=%d steps=%d exceed seq_len=%d", fn, position, steps, d->cfg.seq_len);
    L2_TRY(check_sampling(fn, d, temperature));
    if (!(d->mode & LLAMA2_DECODE_FUSED)) {
        for (int pos = position; pos < position + steps; ++pos) {
            L2_TRY(forward_modules(d, pos, pos + 1));
            if (pos + 1 >= n_prompt && pos + 1 < d->cfg.seq_len) // the token after the last row has no slot
                L2_TRY(sample_launch(fn, d->s.logits, d->s.indices, d->cfg.vocab_size, temperature, top_p,
                                     sampler_coin(seed, pos + 1), d->s.tokens, pos + 1, true));
        }
        return LLAMA2_OK;
    }
    if (d->sampled_temperature != temperature || d->sampled_top_p != top_p || d->sampled_seed != seed) {
        // the sampling parameters are kernel arguments of the captured steps: drop those when they change
        bool any = false;
        for (hipGraphExec_t g : d->graphs[llama2_decoder::kGraphStepSampled])
            any |= g != nullptr;
        if (any) {
            L2_CHECK(!ctx().capturing, "%s: the sampling parameters cannot change during graph capture", fn);
            L2_HIP(hipStreamSynchronize(ctx().stream));
            for (hipGraphExec_t& g : d->graphs[llama2_decoder::kGraphStepSampled]) {
                if (g)
                    (void)hipGraphExecDestroy(g);
                g = nullptr;
            }
        }
        d->sampled_temperature = temperature, d->sampled_top_p = top_p, d->sampled_seed = seed;
    }
    L2_TRY(set_state(d, position, n_prompt, 1));
    for (int i = 0; i < steps; ++i)
        L2_TRY(launch_step(d, llama2_decoder::kGraphStepSampled, position + i));
    return LLAMA2_OK;
}

int llama2_decode_run(llama2_decoder* d, int position, int steps, int n_prompt)
{
    L2_REQUIRE_INIT();
    L2_CHECK(d, "llama2_decode_run: null decoder");
    L2_CHECK(position >= 0 && steps >= 0 && position + steps <= d->cfg.seq_len,
             "llama2_decode_run: position=%d steps=%d exceed seq_len=%d", position, steps, d->cfg.seq_len);
    if (!(d->mode & LLAMA2_DECODE_FUSED)) {
        for (int pos = position; pos < position + steps; ++pos) {
            L2_TRY(forward_modules(d, pos, pos + 1));
            if (pos + 1 < d->cfg.seq_len) // the token after the last row has no slot
                L2_TRY(llama2_argmax(d->s.logits, d->cfg.vocab_size, d->s.tokens, pos + 1, pos + 1 >= n_prompt));
        }
        return LLAMA2_OK;
    }
    L2_TRY(set_state(d, position, n_prompt, 1));
    for (int i = 0; i < steps; ++i)
        L2_TRY(launch_step(d, llama2_decoder::kGraphStep, position + i));
    return LLAMA2_OK;
}

int llama2_decode_check(llama2_decoder* d)
{
    L2_REQUIRE_INIT();
    L2_CHECK(d, "llama2_decode_check: null decoder");
    L2_CHECK(!ctx().capturing, "llama2_decode_check: not allowed during graph capture");
    int flag = 0;
    L2_HIP(hipMemcpyAsync(&flag, d->state + kStateError, sizeof(int), hipMemcpyDeviceToHost, ctx().stream));
    L2_HIP(hipStreamSynchronize(ctx().stream));
    if (flag != 0)
        return fail(LLAMA2_ERR_STEP_FAILED,
                    "llama2_decode_check: a persistent step gave up waiting for data from another workgroup (its "
                    "workgroups were not all resident, or the wait limit is too low); the decoder's results are "
                    "undefined from that step on");
    return LLAMA2_OK;
}

int llama2_decode_set_wait_limit(llama2_decoder* d, int polls)
{
    L2_REQUIRE_INIT();
    L2_CHECK(d, "llama2_decode_set_wait_limit: null decoder");
    L2_CHECK(polls >= 0, "llama2_decode_set_wait_limit: polls=%d must not be negative", polls);
    L2_CHECK(!ctx().capturing, "llama2_decode_set_wait_limit: not allowed during graph capture");
    if (d->persist_variant < 0)
        return fail(LLAMA2_ERR_UNSUPPORTED, "llama2_decode_set_wait_limit: the decoder has no persistent step");
    L2_HIP(hipStreamSynchronize(ctx().stream));
    d->pa.spin_limit = polls;
    for (auto& kind : d->graphs) { // the limit is a kernel argument of the captured persistent steps
        if (kind[kPersistShape])
            (void)hipGraphExecDestroy(kind[kPersistShape]);
        kind[kPersistShape] = nullptr;
    }
    L2_HIP(hipMemsetAsync(d->state + kStateError, 0, sizeof(int), ctx().stream));
    L2_HIP(hipStreamSynchronize(ctx().stream));
    return LLAMA2_OK;
}

int llama2_decode_matvec_chain(llama2_decoder* d, const llama2_half* input, llama2_half* output)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_decode_matvec_chain";
    L2_CHECK(d && input && output, "%s: null argument", fn);
    L2_CHECK(aligned(input, 16) && aligned(output, 16), "%s: input and output must be 16-byte aligned", fn);
    if (d->persist_variant < 0)
        return fail(LLAMA2_ERR_UNSUPPORTED, "%s: the decoder was not created with LLAMA2_DECODE_PERSISTENT", fn);
    hipLaunchKernelGGL(bump_serial_kernel, dim3(1), dim3(64), 0, ctx().stream, d->state);
    L2_LAUNCH_CHECK("bump_serial_kernel");
    PersistArgs a = d->pa;
    a.skip_attention = 1;
    a.embedding = nullptr, a.tokens = nullptr, a.x_in = input;
    a.classifier = nullptr, a.logits = nullptr, a.x_out = output;
    return persist_launch(d->persist_variant, a, ctx().num_cus);
}

int llama2_decode_destroy(llama2_decoder* d)
{
    if (!d)
        return LLAMA2_OK;
    std::lock_guard<std::recursive_mutex> lock(api_mutex());
    if (ctx().ready)
        L2_HIP(hipStreamSynchronize(ctx().stream));
    release(d);
    return LLAMA2_OK;
}

} // extern "C"

// The decode step of Transformer.Forward (src/Transformer.cs:158-190) as ONE persistent
// launch: one 8-wavefront workgroup per compute unit walks through every layer
//   RMSNorm + QKV | attention (RoPE, cache write, scores, softmax, weighted sum) | [merge] |
//   o-proj + residual | RMSNorm + SwiGLU | down-proj + residual
// and then the final RMSNorm and the classifier, without a kernel boundary in between.
//
// Why: a kernel boundary costs about 2.5 us on this part (drain, dispatch, ramp, caches
// invalidated) and a step has 5 L + 3 of them; a grid barrier costs more (agent-scope atomics
// serialise).  Here nothing is counted and nobody waits for "everyone": the vector a phase
// produces is handed over as TAGGED WORDS -- every 32-bit word carries its fp16 value and a
// 16-bit tag of the (step, layer) that wrote it, stored with one agent-scope store -- and a
// consumer simply re-reads the words it needs until all of them carry the tag it expects.
// No fence, no atomic, no flag: a word is its own "ready" bit (the scheme of RCCL's LL
// protocol).  Attention partials are fp32 and travel as 64-bit words (value, 32-bit tag).
//
// The weight stream does not stop at a phase boundary: a wavefront knows which rows it will
// take in every phase, and requests them one or two phases ahead, so that while a vector is
// being handed over the memory system still has tens of megabytes of weights in flight.
//
// Every wait is bounded: after `spin_limit` unsuccessful polls a thread raises the error flag
// in the state block and goes on with what it has; every later wait sees the flag and gives
// up at once, so the grid always drains.  The host reports the flag as an error.
//
// The arithmetic of every module is the one of the stand-alone kernels (int4_kernels.hpp,
// f16_matvec.hip, fused_attn_kernel in decode.hip), operation for operation: the results are
// bit-identical to the launch sequence LLAMA2_DECODE_FUSED.
#include "persist.hpp"

namespace l2 {

constexpr int kPThreads = kPWaves * 64;

__device__ __forceinline__ uint32_t tag16(uint32_t t) { return (t % 65535u) + 1u; } // never 0: a zeroed word is never ready
__device__ __forceinline__ uint32_t tag32(uint32_t t) { return t | 0x80000000u; }

// One unsuccessful poll more.  Returns true when the wait has to be given up.
__device__ __forceinline__ bool give_up(int* err, int& spins, int spin_limit)
{
    ++spins;
    if (spins == 1 || (spins & 255) == 0) {
        if (__hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0)
            return true;
    }
    if (spins > spin_limit) {
        __hip_atomic_store(err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return true;
    }
    __builtin_amdgcn_s_sleep(1);
    return false;
}

// Copies n tagged words (n % 4 == 0) from `src` into fp16 LDS vectors `dst` (and `dst2` if not
// null) once each of them carries `tag`.  Called by the `nthreads` threads of a polling group
// with their number t in it; each owns 16-byte pieces.
// `src` is the same in every lane; `first_word` (a multiple of 4, may differ from lane to lane)
// is where this thread's vector starts in it.
__device__ __forceinline__ void poll_words(const uint32_t* src, int n, uint32_t tag, uint16_t* dst, uint16_t* dst2,
                                           int t, int nthreads, int* err, int spin_limit, int first_word = 0)
{
    const __amdgpu_buffer_rsrc_t r = make_rsrc(uniform_ptr(src), 0x7FFFFFFCu);
    if (t < 0 || t >= nthreads)
        return;
    for (int p = t; p * 4 < n; p += nthreads) {
        u32x4 v;
        int spins = 0;
        for (;;) {
            v = __builtin_amdgcn_raw_buffer_load_b128(r, (first_word + p * 4) * 4, 0, kAuxAgent);
            const uint32_t bad = ((v[0] >> 16) ^ tag) | ((v[1] >> 16) ^ tag) | ((v[2] >> 16) ^ tag) | ((v[3] >> 16) ^ tag);
            if (bad == 0u || give_up(err, spins, spin_limit))
                break;
        }
        u32x2 o;
        o[0] = (v[0] & 0xFFFFu) | (v[1] << 16);
        o[1] = (v[2] & 0xFFFFu) | (v[3] << 16);
        *reinterpret_cast<u32x2*>(dst + p * 4) = o;
        if (dst2)
            *reinterpret_cast<u32x2*>(dst2 + p * 4) = o;
    }
}

__device__ __forceinline__ void put_word(uint32_t* dst, uint32_t tag, uint16_t bits)
{
    store_agent(dst, (tag << 16) | bits);
}

__device__ __forceinline__ void put_part(unsigned long long* dst, uint32_t tag, float v)
{
    const unsigned long long w =
        (static_cast<unsigned long long>(tag) << 32) | static_cast<unsigned long long>(__builtin_bit_cast(uint32_t, v));
    __hip_atomic_store(dst, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ float poll_part(const unsigned long long* src, uint32_t tag, int* err, int spin_limit)
{
    int spins = 0;
    unsigned long long w;
    for (;;) {
        w = __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (static_cast<uint32_t>(w >> 32) == tag || give_up(err, spins, spin_limit))
            break;
    }
    return __builtin_bit_cast(float, static_cast<uint32_t>(w));
}

// The first 256 threads turn the fp16 vector `raw` (LDS, K halfs) into the LDS image the int4
// dot product reads, optionally through RMSNorm with the preloaded weights `gp`: the arithmetic
// of the 256-thread stand-alone kernels, order included.  All threads call, with their number tid.
template <int J>
__device__ __forceinline__ void stage_int4(const uint16_t* raw, int K, bool norm, const uint16_t* gam, float eps,
                                           u32x4* xs, float* sx, float* red4, int tid)
{
    const bool worker = tid < 256;
    VecPieces<J> xp, gp;
#pragma unroll
    for (int i = 0; i < J; ++i) {
        const int e = tid + i * 256;
        xp.v[i] = (worker && e * 8 < K) ? *reinterpret_cast<const u32x4*>(raw + e * 8) : u32x4{0u, 0u, 0u, 0u};
    }
    if (norm) { // uniform
        const float part = wave_sum(worker ? xp.sum_squares() : 0.0f);
        if (worker && (tid & 63) == 0)
            red4[tid >> 6] = part;
        __syncthreads();
        const float ss = (red4[0] + red4[1]) + (red4[2] + red4[3]);
        const float rms = 1.0f / sqrtf(ss / static_cast<float>(K) + eps); // native/rmsnorm_kernel.cu:25-27
#pragma unroll
        for (int i = 0; i < J; ++i) {
            const int e = tid + i * 256;
            gp.v[i] = (worker && e * 8 < K) ? *reinterpret_cast<const u32x4*>(gam + e * 8) : u32x4{0u, 0u, 0u, 0u};
        }
        xp.scale(rms, gp);
    }
    if (worker)
        commit_pieces_t<J>(xs, sx, xp, tid);
    __syncthreads();
}

// RMSNorm weights on their way to LDS: requested by all threads before the wait for the input
// vector (one 16-byte piece per thread and round), written to `gam` once that wait is over.
template <int J>
struct GammaPieces {
    static constexpr int GP = (J * 256 + kPThreads - 1) / kPThreads;
    u32x4 v[GP];
    __device__ __forceinline__ void load(const uint16_t* gamma, int K, int tid)
    {
        const __amdgpu_buffer_rsrc_t r = make_rsrc(uniform_ptr(gamma), K * 2);
#pragma unroll
        for (int i = 0; i < GP; ++i)
            v[i] = __builtin_amdgcn_raw_buffer_load_b128(r, (tid + i * kPThreads) * 16, 0, 0);
    }
    __device__ __forceinline__ void store(uint16_t* gam, int tid) const
    {
#pragma unroll
        for (int i = 0; i < GP; ++i)
            if (tid + i * kPThreads < J * 256)
                *reinterpret_cast<u32x4*>(gam + (tid + i * kPThreads) * 8) = v[i];
    }
};

// The per-layer pointer table is read through the constant address space: nothing writes it while
// the kernel runs, and saying so lets the compiler fetch the pointers with scalar loads.  Read
// through a plain pointer they would be vector loads -- and a vector load in the middle of the
// weight stream makes the wavefront wait for every weight load it has in flight (loads complete in
// order) before it can even form the next address.
typedef const __attribute__((address_space(4))) PersistLayer* LayerTable;
__device__ __forceinline__ QW table_qw(const __attribute__((address_space(4))) QW& q) { return QW{q.w, q.z, q.s}; }

template <int JD, int JH, int RQ, int RO, int RS, int RD>
__global__ __launch_bounds__(kPThreads) void decode_persist_kernel(PersistArgs a)
{
    constexpr int JX = JD > JH ? JD : JH;
    constexpr int CL = 4 * JD; // 16-byte chunks of a classifier row per lane
    __shared__ u32x4 xs[4 * JX * 64];
    __shared__ float sx[JX * 64];
    __shared__ uint16_t rawv[JX * 2048] __attribute__((aligned(16)));
    // the residual stream entering the layer (read by the o-proj rows) and after the o-projection
    // (read by the down-proj rows): two buffers, because a fast wavefront stages the next one
    // while a slow one still reads the previous
    __shared__ uint16_t xres[JD * 2048] __attribute__((aligned(16)));
    __shared__ uint16_t xres1[JD * 2048] __attribute__((aligned(16)));
    __shared__ uint16_t gam[JD * 2048] __attribute__((aligned(16))); // RMSNorm weights of the stage at hand
    __shared__ float red4[4];
    __shared__ float rope_tab[kRopeHeadSize];
    __shared__ float sc[kPUnits][kPBlockRows];
    __shared__ float red[kPUnits][4][kRopeHeadSize];
    __shared__ uint16_t qkv_s[kPUnits][3][kRopeHeadSize] __attribute__((aligned(16)));
    __shared__ float mrg[kPMaxBlocks * kPPartStride];
    __shared__ float mrg_w[64];
    __shared__ float mrg_l;

    const int lane0 = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
    const int G = gridDim.x, W = G * kPWaves;
    const int gw0 = blockIdx.x * kPWaves + wave;
    const int N = a.dim, NH = a.hidden, L = a.n_layers;
    const int nQ = 3 * N;
    const int wg0 = blockIdx.x * kPWaves; // the workgroup's first wavefront: it takes part in a phase iff wg0 < items
    const bool wgQ = wg0 < nQ, wgO = wg0 < N, wgS = wg0 < NH;
    int* err = a.state + kStateError;
    const int spin_limit = a.spin_limit;
    const int pos = a.state[kStatePos];
    const uint32_t tbase = static_cast<uint32_t>(a.state[kStateSerial]) * static_cast<uint32_t>(L + 2);
    if (threadIdx.x < kRopeHeadSize)
        rope_tab[threadIdx.x] = reinterpret_cast<const float*>(a.state + kStateInts)[threadIdx.x];
    __syncthreads();
#ifdef L2_PERSIST_TRACE
    const int trace_slot = blockIdx.x == 0 ? 0 : blockIdx.x == 1 ? 1 : blockIdx.x == 100 ? 2 : blockIdx.x == 255 ? 3 : -1;
#define L2_TRACE(layer, point)                                                                                   \
    do {                                                                                                         \
        if (a.trace && trace_slot >= 0 && threadIdx.x == 0)                                                      \
            a.trace[(static_cast<size_t>(layer) * 4 + trace_slot) * kPTracePoints + (point)] = __builtin_amdgcn_s_memrealtime(); \
    } while (0)
#else
#define L2_TRACE(layer, point) do { } while (0)
#endif

    // attention geometry of this step
    const int S = pos + 1; // attends rows 0..pos (src/Transformer.cs:175)
    const int nblk = (S + kPBlockRows - 1) / kPBlockRows;
    const int natt = a.skip_attention ? 0 : a.n_heads * nblk; // (head, block) items, taken kPUnits * G at a time
    const int q4 = wave >> 2, wq = wave & 3; // q4: the attention unit of this wavefront
    const int mrg_h = G - 1 - static_cast<int>(blockIdx.x); // the head whose blocks this workgroup merges
    const bool wgM = !a.skip_attention && nblk > 1 && mrg_h < a.n_heads;

    const LayerTable layers = (LayerTable)a.layers;
    auto issue_q_row = [&](CFrag<JD, 1> (&fq)[RQ], int layer, bool have_layer, int r, int lane, int gw) {
        if (r < RQ) {
            const int it = gw + r * W;
            const int t = (it >= N) + (it >= 2 * N), n = it - t * N;
            const QW mq = table_qw(layers[layer].q), mk = table_qw(layers[layer].k), mv = table_qw(layers[layer].v);
            const QW m = t == 0 ? mq : (t == 1 ? mk : mv);
            load_row_c<JD>(fq[r].w[0], fq[r].zwv[0], fq[r].sbv[0], m, n, have_layer && it < nQ, a.ws_d, a.ss_d, a.zs_d, lane);
        }
    };

    CFrag<JD, 1> fq[RQ];
#pragma unroll
    for (int r = 0; r < RQ; ++r)
        issue_q_row(fq, 0, true, r, lane0, gw0);

    for (int l = 0; l < L; ++l) {
        // Opaque copies of the thread and wavefront numbers, taken anew in every layer: whatever is
        // derived from them (LDS and buffer addresses, shuffle indices, row numbers -- dozens of
        // values) is recomputed per layer with a few scalar and vector instructions instead of being
        // hoisted out of the loop, where it would occupy registers across the whole layer or be
        // spilled to scratch memory -- and a reload from scratch waits behind every weight load the
        // wavefront has in flight.
        int tid_o = static_cast<int>(threadIdx.x), gw_o = gw0;
        asm volatile("" : "+v"(tid_o));
        asm volatile("" : "+s"(gw_o));
        const int tid = tid_o, lane = tid & 63, tq = tid & 255, gw = gw_o;
        const int zshift = ((lane >> 2) & 7) * 4;
        const QW Po = table_qw(layers[l].o), Pgate = table_qw(layers[l].gate), Pup = table_qw(layers[l].up),
                 Pdown = table_qw(layers[l].down);
        const uint16_t* const rms_att = layers[l].rms_att;
        const uint16_t* const rms_ffn = layers[l].rms_ffn;
        const uint32_t tag = tag16(tbase + static_cast<uint32_t>(l));
        const uint32_t tag_next = tag16(tbase + static_cast<uint32_t>(l) + 1u);

        // ------------------------------------------------ layer input: RMSNorm while staging
        L2_TRACE(l, 0);
        if (wgQ) {
            GammaPieces<JD> gp;
            gp.load(rms_att, N, tid);
            if (l == 0) {
                const uint16_t* src = a.x_in;
                if (a.embedding) { // native/embedding_kernel.cu:9-11
                    int token = a.tokens[pos];
                    token = token < 0 ? 0 : (token >= a.vocab ? a.vocab - 1 : token); // never read outside the table
                    src = a.embedding + static_cast<size_t>(token) * N;
                }
                for (int p = tid; p * 8 < N; p += kPThreads) {
                    const u32x4 v = *reinterpret_cast<const u32x4*>(src + p * 8);
                    *reinterpret_cast<u32x4*>(rawv + p * 8) = v;
                    *reinterpret_cast<u32x4*>(xres + p * 8) = v;
                }
            } else {
                poll_words(a.ll_x0, N, tag, rawv, xres, tid, kPThreads, err, spin_limit);
            }
            gp.store(gam, tid);
            __syncthreads();
            L2_TRACE(l, 1);
            stage_int4<JD>(rawv, N, true, gam, a.eps, xs, sx, red4, tid);
        }
        L2_TRACE(l, 2);

        // o-proj rows and the first SwiGLU pair are requested now, two phases ahead of their use
        CFrag<JD, 1> fo[RO];
#pragma unroll
        for (int r = 0; r < RO; ++r) {
            const int n = gw + r * W;
            load_row_c<JD>(fo[r].w[0], fo[r].zwv[0], fo[r].sbv[0], Po, n, n < N, a.ws_d, a.ss_d, a.zs_d, lane);
        }
        CFrag<JD, 2> fs[RS];
        auto issue_s = [&](int r) {
            const int n = gw + r * W;
            load_row_c<JD>(fs[r].w[0], fs[r].zwv[0], fs[r].sbv[0], Pgate, n, n < NH, a.ws_d, a.ss_d, a.zs_d, lane);
            load_row_c<JD>(fs[r].w[1], fs[r].zwv[1], fs[r].sbv[1], Pup, n, n < NH, a.ws_d, a.ss_d, a.zs_d, lane);
        };
        // SwiGLU pairs [0, S_A) are requested after the q/k/v rows are computed (in flight during
        // attention), [S_A, S_B) after the o-projection, the rest while earlier pairs are computed
        constexpr int S_A = RS < 2 ? RS : 2, S_B = RS < 3 ? RS : 3;

        // ------------------------------------------------ q, k, v rows (unrotated, fp16) as tagged words
        // The results of a phase are collected, row r in lane r, and stored once after the last row: a
        // store issued between the rows would make every later wait for weights a wait for ALL memory
        // operations in flight (loads and stores share one in-order counter and complete out of order
        // with respect to each other), the freshly requested rows and the store's own
        // acknowledgement included.  Nothing is lost: the consumers need the whole vector anyway.
        uint32_t outw = 0;
#pragma unroll
        for (int r = 0; r < RQ; ++r) {
            const int it = gw + r * W;
            if (it < nQ) {
                float acc[1];
                Frag<JD, 1> f;
                expand<JD, 1>(f, fq[r], lane);
                dot_frag<JD, 1>(acc, f, xs, sx, lane, zshift);
                const float v = wave_sum(acc[0]);
                outw = lane == r ? float_to_half_bits(v) : outw;
            }
        }
        if (lane < RQ && gw + lane * W < nQ)
            put_word(a.ll_qkv + gw + lane * W, tag, static_cast<uint16_t>(outw));

        L2_TRACE(l, 3);
#pragma unroll
        for (int r = 0; r < S_A; ++r)
            issue_s(r);

        // ------------------------------------------------ attention: four wavefronts per (head, block of 128 rows)
        for (int it0 = static_cast<int>(blockIdx.x); it0 < natt; it0 += kPUnits * G) { // uniform over the workgroup
            const int att_item = it0 + q4 * G;
            const bool att_act = att_item < natt;
            const int att_h = att_act ? att_item / nblk : 0, att_b = att_act ? att_item - att_h * nblk : 0;
            const int t0 = att_b * kPBlockRows;
            const int t1 = S < t0 + kPBlockRows ? S : t0 + kPBlockRows;
            const int l16 = lane & 15, grp = wq * 4 + (lane >> 4);
            const int col = att_h * kRopeHeadSize + l16 * 8;
            const bool last = att_act && att_b == nblk - 1; // the block that holds the step's own row
            uint16_t* kc = a.kcache + static_cast<size_t>(l) * a.seq_len * N;
            uint16_t* vc = a.vcache + static_cast<size_t>(l) * a.seq_len * N;
            u32x4 kv[8], vv[8];
            if (att_act) { // earlier rows come from the cache and are requested before q exists
                const uint32_t cache_bytes = static_cast<uint32_t>(t1) * N * 2;
                const __amdgpu_buffer_rsrc_t rk = make_rsrc(kc, cache_bytes), rv = make_rsrc(vc, cache_bytes);
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    kv[i] = __builtin_amdgcn_raw_buffer_load_b128(rk, ((t0 + i * 16 + grp) * N + col) * 2, 0, kAuxNonTemporal);
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    vv[i] = __builtin_amdgcn_raw_buffer_load_b128(rv, ((t0 + i * 16 + grp) * N + col) * 2, 0, kAuxNonTemporal);
                // this head's q, and for the last block the new k and v, 32 threads each
                const int part = tq >> 5;
                if (part < (last ? 3 : 1))
                    poll_words(a.ll_qkv, kRopeHeadSize, tag, qkv_s[q4][part], nullptr, tq - part * 32, 32, err, spin_limit,
                               part * N + att_h * kRopeHeadSize);
            }
            __syncthreads();
            if (att_act) { // RoPE (native/rope_kernel.cu:3-26) and the cache row of this position
                const int i = tq & 63, which = tq >> 6;
                if (which == 0 || (which == 1 && last)) {
                    uint16_t* v = qkv_s[q4][which];
                    uint16_t b0, b1;
                    rope_rotate(b0, b1, half_bits_to_float(v[i]), half_bits_to_float(v[i + 64]), rope_tab[2 * i],
                                rope_tab[2 * i + 1]);
                    v[i] = b0;
                    v[i + 64] = b1;
                    if (which == 1) {
                        uint16_t* dst = kc + static_cast<size_t>(pos) * N + att_h * kRopeHeadSize;
                        dst[i] = b0;
                        dst[i + 64] = b1;
                    }
                } else if (which == 2 && last) {
                    uint16_t* dst = vc + static_cast<size_t>(pos) * N + att_h * kRopeHeadSize;
                    dst[i] = qkv_s[q4][2][i];
                    dst[i + 64] = qkv_s[q4][2][i + 64];
                }
            }
            __syncthreads();
            float s[8], m = 0.0f, lsum = 0.0f;
            if (att_act) {
                const u32x4 qv = *reinterpret_cast<const u32x4*>(&qkv_s[q4][0][l16 * 8]);
                if (last) {
                    const u32x4 kn = *reinterpret_cast<const u32x4*>(&qkv_s[q4][1][l16 * 8]);
                    const u32x4 vn = *reinterpret_cast<const u32x4*>(&qkv_s[q4][2][l16 * 8]);
#pragma unroll
                    for (int i = 0; i < 8; ++i)
                        if (t0 + i * 16 + grp == pos) {
                            kv[i] = kn;
                            vv[i] = vn;
                        }
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    float acc = 0.0f;
#pragma unroll
                    for (int k = 0; k < 4; ++k)
                        acc = dot2(kv[i][k], qv[k], acc);
                    acc = row16_sum(acc) * a.scale; // native/mat_vec_kernel.cu:71-74
                    s[i] = t0 + i * 16 + grp < t1 ? half_bits_to_float(float_to_half_bits(acc)) : -INFINITY;
                    if (l16 == 0)
                        sc[q4][i * 16 + grp] = s[i];
                }
            }
            __syncthreads();
            if (att_act) {
                m = -INFINITY;
#pragma unroll
                for (int k = 0; k < kPBlockRows / 64; ++k)
                    m = fmaxf(m, sc[q4][lane + 64 * k]);
                m = wave_max(m);
#pragma unroll
                for (int k = 0; k < kPBlockRows / 64; ++k)
                    lsum += expf(sc[q4][lane + 64 * k] - m);
                lsum = wave_sum(lsum);
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
                for (int k = 0; k < 8; ++k) {
                    o[k] += __shfl_xor(o[k], 16, 64);
                    o[k] += __shfl_xor(o[k], 32, 64);
                }
                if (lane < 16) {
#pragma unroll
                    for (int k = 0; k < 8; ++k)
                        red[q4][wq][l16 * 8 + k] = o[k];
                }
            }
            __syncthreads();
            if (att_act && tq < kRopeHeadSize) {
                float val = 0.0f;
#pragma unroll
                for (int g = 0; g < 4; ++g)
                    val += red[q4][g][tq];
                if (nblk == 1) {
                    put_word(a.ll_att + att_h * kRopeHeadSize + tq, tag, float_to_half_bits(val / lsum));
                } else {
                    unsigned long long* Pp =
                        a.ll_part + (static_cast<size_t>(att_h) * kPMaxBlocks + att_b) * kPPartStride;
                    const uint32_t t32 = tag32(tbase + static_cast<uint32_t>(l));
                    put_part(Pp + tq, t32, val);
                    if (tq == 0) {
                        put_part(Pp + kRopeHeadSize, t32, m);
                        put_part(Pp + kRopeHeadSize + 1, t32, lsum);
                    }
                }
            }
        }

        // ------------------------------------------------ merge of a head's blocks (fixed order: deterministic)
        if (wgM) {
            const uint32_t t32 = tag32(tbase + static_cast<uint32_t>(l));
            const unsigned long long* Pp = a.ll_part + static_cast<size_t>(mrg_h) * kPMaxBlocks * kPPartStride;
            if (q4 == kPUnits - 1)
                for (int e = tq; e < nblk * kPPartStride; e += 256)
                    mrg[e] = poll_part(Pp + e, t32, err, spin_limit);
            __syncthreads();
            if (wave == 4 * (kPUnits - 1)) { // block i in lane i
                const bool have = lane < nblk;
                const float mi = have ? mrg[lane * kPPartStride + kRopeHeadSize] : -INFINITY;
                const float li = have ? mrg[lane * kPPartStride + kRopeHeadSize + 1] : 0.0f;
                const float M = wave_max(mi);
                const float w = have ? expf(mi - M) : 0.0f;
                mrg_w[lane] = w;
                const float Lm = wave_sum(w * li);
                if (lane == 0)
                    mrg_l = Lm;
            }
            __syncthreads();
            if (q4 == kPUnits - 1 && tq < kRopeHeadSize) {
                float O = 0.0f;
                for (int i = 0; i < nblk; ++i)
                    O = fmaf(mrg_w[i], mrg[i * kPPartStride + tq], O);
                put_word(a.ll_att + mrg_h * kRopeHeadSize + tq, tag, float_to_half_bits(O / mrg_l));
            }
        }

        // ------------------------------------------------ o-proj + residual
        L2_TRACE(l, 4);
        if (wgO) {
            poll_words(a.skip_attention ? a.ll_qkv : a.ll_att, N, tag, rawv, nullptr, tid, kPThreads, err, spin_limit);
            __syncthreads();
            L2_TRACE(l, 5);
            stage_int4<JD>(rawv, N, false, gam, a.eps, xs, sx, red4, tid);
        }
        L2_TRACE(l, 6);
#pragma unroll
        for (int r = 0; r < RO; ++r) {
            const int n = gw + r * W;
            if (n < N) {
                float acc[1];
                Frag<JD, 1> f;
                expand<JD, 1>(f, fo[r], lane);
                dot_frag<JD, 1>(acc, f, xs, sx, lane, zshift);
                float v = wave_sum(acc[0]);
                v += half_bits_to_float(xres[n]);
                outw = lane == r ? float_to_half_bits(v) : outw;
            }
        }
        if (lane < RO && gw + lane * W < N)
            put_word(a.ll_x1 + gw + lane * W, tag, static_cast<uint16_t>(outw));
#pragma unroll
        for (int r = S_A; r < S_B; ++r)
            issue_s(r);

        // ------------------------------------------------ RMSNorm + SwiGLU
        L2_TRACE(l, 7);
        if (wgS) { // every workgroup with down-proj rows has SwiGLU rows too (hidden >= dim: checked on the host)
            GammaPieces<JD> gp;
            gp.load(rms_ffn, N, tid);
            poll_words(a.ll_x1, N, tag, rawv, xres1, tid, kPThreads, err, spin_limit);
            gp.store(gam, tid);
            __syncthreads();
            L2_TRACE(l, 8);
            stage_int4<JD>(rawv, N, true, gam, a.eps, xs, sx, red4, tid);
        }
        L2_TRACE(l, 9);
        CFrag<JH, 1> fd[RD];
        constexpr int NS2 = RS - S_B, NI = NS2 + RD + RQ, PER = (NI + RS - 1) / RS;
        const bool have_next = l + 1 < L;
        const int next_layer = have_next ? l + 1 : l;
        auto issue_ahead = [&](int i) {
            if (i < NS2) {
                issue_s(S_B + i);
            } else if (i < NS2 + RD) {
                const int nd = gw + (i - NS2) * W;
                load_row_c<JH>(fd[i - NS2].w[0], fd[i - NS2].zwv[0], fd[i - NS2].sbv[0], Pdown, nd, nd < N, a.ws_h, a.ss_h,
                               a.zs_h, lane);
            } else if (i < NI) {
                issue_q_row(fq, next_layer, have_next, i - NS2 - RD, lane, gw);
            }
        };
#pragma unroll
        for (int r = 0; r < RS; ++r) {
            const int n = gw + r * W;
            if (n < NH) {
                float acc[2];
                Frag<JD, 2> f;
                expand<JD, 2>(f, fs[r], lane);
                dot_frag<JD, 2>(acc, f, xs, sx, lane, zshift);
                const float g = wave_sum(acc[0]), u = wave_sum(acc[1]);
                float v = g;
                v *= 1.0f / (1.0f + expf(-v)); // native/mat_vec_kernel.cu:219-221
                v *= u;
                outw = lane == r ? float_to_half_bits(v) : outw;
            }
            // the registers a computed pair frees take, in this order, the remaining pairs, the down-proj
            // rows and the next layer's q/k/v rows, PER of them per pair
#pragma unroll
            for (int k = 0; k < PER; ++k)
                issue_ahead(r * PER + k);
        }
#pragma unroll
        for (int i = RS * PER; i < NI; ++i)
            issue_ahead(i);
        if (lane < RS && gw + lane * W < NH)
            put_word(a.ll_h + gw + lane * W, tag, static_cast<uint16_t>(outw));

        // ------------------------------------------------ down-proj + residual
        L2_TRACE(l, 10);
        if (wgO) {
            poll_words(a.ll_h, NH, tag, rawv, nullptr, tid, kPThreads, err, spin_limit);
            __syncthreads();
            L2_TRACE(l, 11);
            stage_int4<JH>(rawv, NH, false, gam, a.eps, xs, sx, red4, tid);
        }
        L2_TRACE(l, 12);
#pragma unroll
        for (int r = 0; r < RD; ++r) {
            const int n = gw + r * W;
            if (n < N) {
                float acc[1];
                Frag<JH, 1> f;
                expand<JH, 1>(f, fd[r], lane);
                dot_frag<JH, 1>(acc, f, xs, sx, lane, zshift);
                float v = wave_sum(acc[0]);
                v += half_bits_to_float(xres1[n]);
                outw = lane == r ? float_to_half_bits(v) : outw;
            }
        }
        if (lane < RD && gw + lane * W < N)
            put_word(a.ll_x0 + gw + lane * W, tag_next, static_cast<uint16_t>(outw));
        L2_TRACE(l, 13);
    }

    // ---------------------------------------------------- final RMSNorm + classifier (src/Transformer.cs:187-189)
    const int lane = lane0, gw = gw0;
    const uint32_t tag = tag16(tbase + static_cast<uint32_t>(L));
    if (!a.classifier) {
        if (blockIdx.x == 0) { // the mat-vec chain alone: hand the residual stream back as plain fp16
            poll_words(a.ll_x0, N, tag, rawv, nullptr, static_cast<int>(threadIdx.x), kPThreads, err, spin_limit);
            __syncthreads();
            for (int p = threadIdx.x; p * 8 < N; p += kPThreads)
                *reinterpret_cast<u32x4*>(a.x_out + p * 8) = *reinterpret_cast<const u32x4*>(rawv + p * 8);
        }
        return;
    }
    if (wg0 >= a.vocab)
        return;
    const int nchunks = N >> 3;
    u32x4 cur[CL], nxt[CL];
    auto issue_row = [&](u32x4 (&m)[CL], int n) {
        const __amdgpu_buffer_rsrc_t rm =
            make_rsrc(uniform_ptr(a.classifier + static_cast<size_t>(n) * N), static_cast<uint32_t>(N) * 2u);
#pragma unroll
        for (int u = 0; u < CL; ++u)
            m[u] = __builtin_amdgcn_raw_buffer_load_b128(rm, (lane + 64 * u) * 16, 0, kAuxNonTemporal);
    };
    if (gw < a.vocab)
        issue_row(cur, gw);
    {
        VecPieces<JD> gp, xp;
        GammaPieces<JD> gq;
        gq.load(a.rms_final, N, static_cast<int>(threadIdx.x));
        poll_words(a.ll_x0, N, tag, rawv, nullptr, static_cast<int>(threadIdx.x), kPThreads, err, spin_limit);
        gq.store(gam, static_cast<int>(threadIdx.x));
        __syncthreads();
        const bool worker = threadIdx.x < 256;
#pragma unroll
        for (int i = 0; i < JD; ++i) {
            const int e = threadIdx.x + i * 256;
            xp.v[i] = (worker && e * 8 < N) ? *reinterpret_cast<const u32x4*>(rawv + e * 8) : u32x4{0u, 0u, 0u, 0u};
        }
        const float part = wave_sum(worker ? xp.sum_squares() : 0.0f);
        if (worker && lane == 0)
            red4[threadIdx.x >> 6] = part;
        __syncthreads();
        const float ss = (red4[0] + red4[1]) + (red4[2] + red4[3]);
        const float rms = 1.0f / sqrtf(ss / static_cast<float>(N) + a.eps);
#pragma unroll
        for (int i = 0; i < JD; ++i) {
            const int e = threadIdx.x + i * 256;
            gp.v[i] = (worker && e * 8 < N) ? *reinterpret_cast<const u32x4*>(gam + e * 8) : u32x4{0u, 0u, 0u, 0u};
        }
        xp.scale(rms, gp);
        if (worker) {
#pragma unroll
            for (int i = 0; i < JD; ++i) {
                const int e = threadIdx.x + i * 256;
                if (e < nchunks)
                    xs[e] = xp.v[i];
            }
        }
        __syncthreads();
    }
    uint32_t outw = 0; // logits of this wavefront's rows, row k in lane k % 64, stored 64 at a time
    int k = 0;
    for (int n = gw; n < a.vocab; n += W, ++k) {
        const int nn = n + W;
        if (nn < a.vocab)
            issue_row(nxt, nn);
        float acc = 0.0f;
#pragma unroll
        for (int u = 0; u < CL; ++u) {
            const int c = lane + 64 * u;
            if (c < nchunks) {
                const u32x4 xv = xs[c];
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    acc = dot2(cur[u][i], xv[i], acc);
            }
        }
        const float sum = wave_sum(acc);
        outw = lane == (k & 63) ? float_to_half_bits(sum) : outw;
        if ((k & 63) == 63 || nn >= a.vocab) {
            const int row = gw + ((k & ~63) + lane) * W;
            if (lane <= (k & 63))
                a.logits[row] = static_cast<uint16_t>(outw);
        }
#pragma unroll
        for (int u = 0; u < CL; ++u)
            cur[u] = nxt[u];
    }
}

// ------------------------------------------------------------------ host side
namespace {

struct Variant {
    int jd, jh, rq, ro, rs, rd;
    void (*kernel)(PersistArgs);
};

const Variant kVariants[] = {
    {1, 1, 1, 1, 1, 1, decode_persist_kernel<1, 1, 1, 1, 1, 1>}, // small models: at most one row per wavefront and phase
    {2, 6, 6, 2, 6, 2, decode_persist_kernel<2, 6, 6, 2, 6, 2>}, // Llama-2-7B on 256 compute units
};

} // namespace

int persist_variant(int dim, int hidden, int n_heads, int num_cus)
{
    if (num_cus <= 0 || dim % 8 || hidden % 8 || hidden < dim || dim != n_heads * kRopeHeadSize)
        return -1;
    const int W = num_cus * kPWaves;
    if (n_heads > num_cus)
        return -1;
    const int jd = chunk_columns(ceil_div(dim, 32) * 4), jh = chunk_columns(ceil_div(hidden, 32) * 4);
    const int rq = ceil_div(3 * dim, W), ro = ceil_div(dim, W), rs = ceil_div(hidden, W);
    for (size_t i = 0; i < sizeof(kVariants) / sizeof(kVariants[0]); ++i) {
        const Variant& v = kVariants[i];
        if (v.jd == jd && v.jh == jh && v.rq == rq && v.ro == ro && v.rs == rs && v.rd == ro)
            return static_cast<int>(i);
    }
    return -1;
}

static size_t align256(size_t v) { return (v + 255) & ~static_cast<size_t>(255); }

size_t persist_scratch_bytes(int dim, int hidden, int n_heads)
{
    return align256(sizeof(uint32_t) * dim) * 3 + align256(sizeof(uint32_t) * 3 * dim) + align256(sizeof(uint32_t) * hidden) +
           align256(sizeof(unsigned long long) * n_heads * kPMaxBlocks * kPPartStride);
}

void persist_bind_scratch(PersistArgs& a, void* base)
{
    char* p = static_cast<char*>(base);
    a.ll_x0 = reinterpret_cast<uint32_t*>(p), p += align256(sizeof(uint32_t) * a.dim);
    a.ll_att = reinterpret_cast<uint32_t*>(p), p += align256(sizeof(uint32_t) * a.dim);
    a.ll_x1 = reinterpret_cast<uint32_t*>(p), p += align256(sizeof(uint32_t) * a.dim);
    a.ll_qkv = reinterpret_cast<uint32_t*>(p), p += align256(sizeof(uint32_t) * 3 * a.dim);
    a.ll_h = reinterpret_cast<uint32_t*>(p), p += align256(sizeof(uint32_t) * a.hidden);
    a.ll_part = reinterpret_cast<unsigned long long*>(p);
}

int persist_launch(int variant, const PersistArgs& a, int num_cus)
{
    if (variant < 0 || variant >= static_cast<int>(sizeof(kVariants) / sizeof(kVariants[0])))
        return fail(LLAMA2_ERR_UNSUPPORTED, "persistent decode step: no kernel for these shapes");
    hipLaunchKernelGGL(kVariants[variant].kernel, dim3(num_cus), dim3(kPThreads), 0, ctx().stream, a);
    L2_LAUNCH_CHECK("decode_persist_kernel");
    return LLAMA2_OK;
}

} // namespace l2

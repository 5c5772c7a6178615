// AWQ-v1 int4 (group 128) mat-vec kernels for gfx950, shared by the module entry
// points (int4_matvec.hip) and the fused decode step (decode.hip).
// Replaces native/mat_vec_kernel.cu:83-234 of the reference.
//
// Shape of the computation (batch-1 GEMV, HBM-bound, no MFMA):
//   * a "chunk" is 16 bytes of one weight row = 4 uint32 = 32 nibbles; a
//     64-lane wavefront reads 64 consecutive chunks (1 KiB) per load
//     instruction, lane l taking chunks l, l+64, ... (buffer_load_dwordx4
//     through a per-row buffer resource, so the ragged end of a row reads as
//     zero without any lane predication);
//   * a wavefront owns a span of consecutive rows, all wavefronts resident at once, the row
//     sequence fully unrolled with the next row's loads in flight while the current one is
//     reduced (int4_matvec_span_kernel: every shape the decoder and the benches launch); the
//     two older kernels (persistent wavefronts that stride over the rows, one row or a block of
//     rows per item) take the launches it refuses;
//   * the input vector is staged once per workgroup in LDS, pre-permuted to
//     the order the nibble extraction produces, in four planes so that
//     consecutive lanes read consecutive 16-byte slots (conflict-free
//     ds_read_b128), together with the fp32 sum of every 32-element chunk.
//     The staging step can apply RMSNorm on the way (fused decode step);
//   * a nibble masked in place (w & 0x000F000F, w & 0x00F000F0) IS an fp16
//     subnormal pair (n * 2^-24 resp. n * 2^-20): v_dot2_f32_f16 multiplies it
//     exactly with the fp16 input pair and accumulates in fp32, so dequantising
//     costs one v_and per pair.  The zero-point is applied per chunk as
//     -z * sum(x), the group scale once per chunk, all in fp32;
//   * lanes are reduced with DPP row operations.
#pragma once

#include "common.hpp"

namespace l2 {

struct QW {
    const uint32_t* w;
    const uint32_t* z;
    const uint16_t* s;
};

// What the wavefront does with its dot products.
enum Mode {
    PLAIN = 0,    // out[t][n] = half(sum)                     (1 or 3 tensors)
    RESIDUAL = 1, // out[0][n] = half(sum + float(out[0][n]))
    SWIGLU = 2,   // out[0][n] = half(silu(gate.x) * (up.x))
    QKV_ROPE = 3, // q/k/v rows (i, i+64) of a head; q and k rotated; k, v written to the cache row of *pos
};
// Where the staged input comes from.
enum Stage {
    STAGE_X = 0,       // x as given
    STAGE_RMSNORM = 1, // half(rms * gamma * x), x = a.x or (layer 0) the embedding row of tokens[*pos]
};

constexpr int kRopeHeadSize = 128; // QKV_ROPE assumes head_size 128 (pairs i, i+64)

struct Int4Args {
    QW m[3];          // PLAIN/RESIDUAL: m[0] (QKV: q,k,v); SWIGLU: gate, up
    uint16_t* out[3]; // one output vector per tensor; QKV_ROPE: q, key-cache layer base, value-cache layer base
    const uint16_t* x;
    int K, N, ws, ss, zs;
    int n_tensors;
    // STAGE_RMSNORM
    const uint16_t* gamma;
    float eps;
    const uint16_t* embedding; // non-null: x = embedding[tokens[*pos] * K ..], also copied to x_out
    const int* tokens;
    int vocab;
    uint16_t* x_out;
    // device-resident step state: pos_ptr[0] = position
    const int* pos_ptr;
    // QKV_ROPE
    int kv_dim;
    float theta;
    const float* rope_table; // (cos, sin) of the step's position for i < 64, or null: computed here from theta
};

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

// LDS image of the input for J chunk-columns per lane:
//   xs[i*JC + c] holds elements 8*(4c+i)+{0,4,1,5,2,6,3,7} (JC = 64 J, zero beyond K),
//   sx[c] the fp32 sum of the 32 elements of chunk c.
// 8 consecutive inputs (words `word` and the three after it of a chunk's 16) in the order the nibble
// extraction produces them: (x0,x4), (x1,x5), (x2,x6), (x3,x7).
//
// v_dot2_f32_f16 does not round its fp32 result to nearest: it drops what lies below about 2^-40
// (an ABSOLUTE position, whatever the magnitude of the operands) towards minus infinity.  The sums
// of nibble * 2^-24 * x live just above that position, and a mat-vec of 11008 terms came out low
// by 4.0e-5 +- 0.5e-5 in every single output, whatever the signs of the inputs.  Therefore the
// second half of every chunk (words 2 and 3) is staged with the inputs of those sums NEGATED and
// added up in an accumulator of its own, which is subtracted: the two halves lose the same on
// average and the bias cancels (the sums of nibble * 2^-20 * x lose 16 times less and are left alone).
__device__ __forceinline__ u32x4 staged_order(const u32x4 v, int word)
{
    const uint32_t flip = word >= 2 ? 0x80008000u : 0u;
    u32x4 o;
    o[0] = ((v[0] & 0xFFFFu) | (v[2] << 16)) ^ flip; // x0, x4 (meet the nibbles at bit 0 of a byte)
    o[1] = (v[0] >> 16) | (v[2] & 0xFFFF0000u);      // x1, x5
    o[2] = ((v[1] & 0xFFFFu) | (v[3] << 16)) ^ flip; // x2, x6 (bit 0 of a byte after the shift by 8)
    o[3] = (v[1] >> 16) | (v[3] & 0xFFFF0000u);      // x3, x7
    return o;
}

// One thread's pieces of the input into the LDS image; `tid` < 256.
template <int J>
__device__ __forceinline__ void commit_pieces_t(u32x4* xs, float* sx, const VecPieces<J>& p, int tid)
{
    constexpr int JC = J * 64;
#pragma unroll
    for (int i = 0; i < J; ++i) { // JC*4 pieces over 256 threads = J per thread
        const int e = tid + i * 256;
        const u32x4 v = p.v[i];
        xs[(e & 3) * JC + (e >> 2)] = staged_order(v, e & 3);
        const h2_t one = {static_cast<_Float16>(1.0f), static_cast<_Float16>(1.0f)};
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < 4; ++k)
            s = __builtin_amdgcn_fdot2(as_h2(v[k]), one, s, false);
        s += dpp_f32<DPP_QUAD_XOR1>(s); // the 4 words of a chunk sit in one quad of lanes
        s += dpp_f32<DPP_QUAD_XOR2>(s);
        if ((e & 3) == 0)
            sx[e >> 2] = s;
    }
}

template <int J>
__device__ __forceinline__ void commit_pieces(u32x4* xs, float* sx, const VecPieces<J>& p)
{
    commit_pieces_t<J>(xs, sx, p, static_cast<int>(threadIdx.x));
}

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
            // a0, a0n: nibbles at bit 0 of a byte (x 2^-24) of words 0-1 and, inputs negated, of words 2-3;
            // a1: nibbles at bit 4 (x 2^-20)
            float a0 = 0.0f, a0n = 0.0f, a1 = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t w = f.w[r][j][i], w8 = w >> 8;
                float& lo = i < 2 ? a0 : a0n;
                lo = __builtin_amdgcn_fdot2(as_h2(w & 0x000F000Fu), as_h2(xv[i][0]), lo, false);  // n0,n4
                a1 = __builtin_amdgcn_fdot2(as_h2(w & 0x00F000F0u), as_h2(xv[i][1]), a1, false);  // n1,n5
                lo = __builtin_amdgcn_fdot2(as_h2(w8 & 0x000F000Fu), as_h2(xv[i][2]), lo, false); // n2,n6
                a1 = __builtin_amdgcn_fdot2(as_h2(w8 & 0x00F000F0u), as_h2(xv[i][3]), a1, false); // n3,n7
            }
            const float zf = static_cast<float>((f.zw[r][j] >> zshift) & 0xFu);
            float t = a0 * 16777216.0f;      // 2^24
            t = fmaf(a0n, -16777216.0f, t);
            t = fmaf(a1, 1048576.0f, t);     // 2^20
            t = fmaf(-zf, sxv, t);       // sum x (n - z)
            acc[r] = fmaf(t, half_bits_to_float(f.sb[r][j]), acc[r]);
        }
    }
}

// cos/sin of pos * theta^(-2i/head_size) for i < head_size/2, the float
// expression of native/rope_kernel.cu:8-12.
__device__ __forceinline__ void rope_cos_sin(float& fcr, float& fci, int i, int head_size, int pos, float theta)
{
    const int head_dim = (i * 2) % head_size;
    const float freq = 1.0f / powf(theta, static_cast<float>(head_dim) / static_cast<float>(head_size));
    const float val = static_cast<float>(pos) * freq;
    fcr = cosf(val);
    fci = sinf(val);
}

template <int J, int MODE, int STAGE>
__global__ __launch_bounds__(256) void int4_matvec_kernel(Int4Args a)
{
    // Two rows per item (QKV_ROPE: rows i and i + 64 of a head; SWIGLU: gate row and up row) are taken
    // one after the other by the same wavefront (PAIRED), except where the input is normalised while it
    // is staged: there holding both rows of SwiGLU at once (R = 2) measured faster.
    constexpr bool PAIRED = MODE == QKV_ROPE || (MODE == SWIGLU && STAGE == STAGE_X);
    constexpr int R = (MODE == SWIGLU && !PAIRED) ? 2 : 1;
    constexpr int JC = J * 64;
    constexpr int WAVES = 4;
    __shared__ u32x4 xs[4 * JC];
    __shared__ float sx[JC];
    __shared__ float red4[4];
    __shared__ float rope_tab[MODE == QKV_ROPE ? kRopeHeadSize : 2]; // (cos, sin) pairs
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int total_waves = gridDim.x * WAVES;
    const int pairs = a.N >> 1; // QKV_ROPE: (i, i+64) row pairs per tensor
    const int nitems = MODE == QKV_ROPE ? 3 * pairs : a.n_tensors * a.N;
    int item = blockIdx.x * WAVES + wave;
    int half = 0; // PAIRED: which row of the item's pair is being worked on

    auto load_item = [&](Frag<J, R>& f, uint16_t& res, int it, int hf) {
        it = __builtin_amdgcn_readfirstlane(it);
        hf = __builtin_amdgcn_readfirstlane(hf);
        if (MODE == SWIGLU && PAIRED) { // half 0: gate row, half 1: up row
            load_row<J>(f.w[0], f.zw[0], f.sb[0], a.m[hf], static_cast<size_t>(it), a.ws, a.ss, a.zs, lane);
        } else if (MODE == SWIGLU) {
            load_row<J>(f.w[0], f.zw[0], f.sb[0], a.m[0], static_cast<size_t>(it), a.ws, a.ss, a.zs, lane);
            load_row<J>(f.w[R - 1], f.zw[R - 1], f.sb[R - 1], a.m[1], static_cast<size_t>(it), a.ws, a.ss, a.zs, lane);
        } else if (MODE == QKV_ROPE) {
            const int t = (it >= pairs) + (it >= 2 * pairs), rem = it - t * pairs;
            const int n0 = (rem >> 6) * kRopeHeadSize + (rem & 63);
            load_row<J>(f.w[0], f.zw[0], f.sb[0], a.m[t], static_cast<size_t>(n0 + 64 * hf), a.ws, a.ss, a.zs, lane);
        } else {
            const int t = (it >= a.N) + (it >= 2 * a.N), n = it - t * a.N; // at most 3 tensors
            load_row<J>(f.w[0], f.zw[0], f.sb[0], a.m[t], static_cast<size_t>(n), a.ws, a.ss, a.zs, lane);
            if (MODE == RESIDUAL)
                res = a.out[t][n];
        }
    };

    // input first (served by L2), then the first item's weights (HBM)
    VecPieces<J> xp;
    const uint16_t* xsrc = a.x;
    if (STAGE == STAGE_RMSNORM && a.embedding) { // native/embedding_kernel.cu:9-11
        int token = a.tokens[a.pos_ptr ? a.pos_ptr[0] : 0];
        token = token < 0 ? 0 : (token >= a.vocab ? a.vocab - 1 : token); // never read outside the table
        xsrc = a.embedding + static_cast<size_t>(token) * a.K;
    }
    xp.load(xsrc, a.K);
    VecPieces<J> gp;
    if (STAGE == STAGE_RMSNORM)
        gp.load(a.gamma, a.K);
    // The RoPE table is requested before the weights as well: loads return in order, so a value
    // requested after them would hold up the staging below until the first weights have arrived.
    float rope_entry = 0.0f;
    if (MODE == QKV_ROPE && a.rope_table && threadIdx.x < kRopeHeadSize)
        rope_entry = a.rope_table[threadIdx.x];
    Frag<J, R> cur;
    uint16_t cur_res = 0;
    if (item < nitems)
        load_item(cur, cur_res, item, 0);

    // The position lives in device memory: outside layer 0 it is read only here, after the weight
    // loads above were issued.
    const int pos = MODE == QKV_ROPE && a.pos_ptr ? a.pos_ptr[0] : 0;
    if (MODE == QKV_ROPE) {
        if (a.rope_table) { // prepared by the kernel that set the position
            if (threadIdx.x < kRopeHeadSize)
                rope_tab[threadIdx.x] = rope_entry;
        } else if (threadIdx.x < kRopeHeadSize / 2) {
            float c, s;
            rope_cos_sin(c, s, threadIdx.x, kRopeHeadSize, pos, a.theta);
            rope_tab[2 * threadIdx.x] = c;
            rope_tab[2 * threadIdx.x + 1] = s;
        }
    }
    if (STAGE == STAGE_RMSNORM) {
        if (a.embedding && blockIdx.x == 0) { // the residual stream starts as the embedding row
            const __amdgpu_buffer_rsrc_t ro = make_rsrc(a.x_out, a.K * 2);
#pragma unroll
            for (int i = 0; i < J; ++i)
                __builtin_amdgcn_raw_buffer_store_b128(xp.v[i], ro, (threadIdx.x + i * 256) * 16, 0, 0);
        }
        const float ss = block256_sum(xp.sum_squares(), red4);
        const float rms = 1.0f / sqrtf(ss / static_cast<float>(a.K) + a.eps); // native/rmsnorm_kernel.cu:25-27
        xp.scale(rms, gp);
    }
    commit_pieces<J>(xs, sx, xp);
    __syncthreads();

    const int zshift = ((lane >> 2) & 7) * 4; // nibble of the zero word: group (c/4) % 8, same for every j
    float v_first = 0.0f;
    while (item < nitems) {
        const int nitem = (!PAIRED || half) ? item + total_waves : item;
        const int nhalf = PAIRED ? half ^ 1 : 0;
        Frag<J, R> nxt;
        uint16_t nxt_res = 0;
        if (nitem < nitems)
            load_item(nxt, nxt_res, nitem, nhalf);
        float acc[R];
        dot_frag<J, R>(acc, cur, xs, sx, lane, zshift);
        if (MODE == SWIGLU) {
            float g = wave_sum(acc[0]), u = 0.0f;
            if (PAIRED) {
                if (half == 0)
                    v_first = g;
                u = g;
                g = v_first;
            } else {
                u = wave_sum(acc[R - 1]);
            }
            if ((!PAIRED || half == 1) && lane == 0) {
                float v = g;
                v *= 1.0f / (1.0f + expf(-v)); // native/mat_vec_kernel.cu:219-221
                v *= u;
                a.out[0][item] = float_to_half_bits(v);
            }
        } else if (MODE == QKV_ROPE) {
            // the unfused path stores q/k as fp16 and RoPE reads them back: keep that rounding
            const float v = half_bits_to_float(float_to_half_bits(wave_sum(acc[0])));
            if (half == 0)
                v_first = v;
            const float v0 = v_first, v1 = v;
            if (half == 1 && lane == 0) {
                const int t = (item >= pairs) + (item >= 2 * pairs), rem = item - t * pairs;
                const int i = rem & 63, n0 = (rem >> 6) * kRopeHeadSize + i;
                uint16_t* dst = t == 0 ? a.out[0] : a.out[t] + static_cast<size_t>(pos) * a.kv_dim;
                uint16_t b0 = float_to_half_bits(v0), b1 = float_to_half_bits(v1);
                if (t < 2) // native/rope_kernel.cu:14-26
                    rope_rotate(b0, b1, v0, v1, rope_tab[2 * i], rope_tab[2 * i + 1]);
                dst[n0] = b0;
                dst[n0 + 64] = b1;
            }
        } else {
            float v = wave_sum(acc[0]);
            if (lane == 0) {
                const int t = (item >= a.N) + (item >= 2 * a.N), n = item - t * a.N;
                if (MODE == RESIDUAL)
                    v += half_bits_to_float(cur_res);
                a.out[t][n] = float_to_half_bits(v);
            }
        }
        cur = nxt;
        cur_res = nxt_res;
        item = nitem;
        half = nhalf;
    }
}

// ---------------------------------------------------------------------------------------------
// Blocks of consecutive rows per wavefront.
//
// What limits a batch-1 mat-vec on this part is neither arithmetic nor bandwidth as such but the
// number of vector-memory INSTRUCTIONS a compute unit can have in flight (a few dozen, whatever
// their size): a 16-byte-per-lane load carries 1 KiB, a 4- or 2-byte-per-lane load carries a
// fraction of that and takes the same slot.  Reading a row of 4096 inputs as 2 loads of weights
// plus 2 of zero words plus 2 of scales puts 0.35 KiB in flight per slot; a pure read achieves 1.
// Hence:
//   * an item is a block of RB consecutive rows: their scales are one contiguous run (RB x ss
//     fp16, at most 256 bytes), their zero words another, so ONE 4-byte-per-lane load fetches all
//     scales of the block and one more all zero words -- RB J + 2 slots for RB rows instead of
//     6 J RB.  The lanes that need a scale or a zero word fetch it from the lane that holds it
//     (ds_bpermute) when the row is computed;
//   * the rows of a block share the reads of the staged input (dot_frag over RB rows at once);
//   * no store between the items of a wavefront: loads and stores share one counter (vmcnt) and
//     complete out of order with respect to each other, so after a store the compiler can only
//     wait for "all memory operations done", the next block's loads included.  Results are
//     collected, one per lane, and stored once;
//   * descriptors are made scalar explicitly (uniform_ptr); a descriptor in vector registers
//     costs a readfirstlane loop per load.
// ---------------------------------------------------------------------------------------------

// A pointer that is the same in every lane, moved to scalar registers.
template <class T>
__device__ __forceinline__ T* uniform_ptr(T* p)
{
    const unsigned long long v = reinterpret_cast<unsigned long long>(p);
    const unsigned lo = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(v));
    const unsigned hi = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(v >> 32));
    return reinterpret_cast<T*>((static_cast<unsigned long long>(hi) << 32) | lo);
}

// What a lane keeps of R rows while they are in flight (persistent decode step): J chunks of
// weights per row, its share of the row's zero words (word l) and of its scales (scale l + 64 k).
template <int J, int R>
struct CFrag {
    static constexpr int SV = (J + 3) / 4; // 64 scales (4 chunk columns) per register
    u32x4 w[R][J];
    uint32_t zwv[R];
    uint32_t sbv[R][SV];
};

// Requests row `row` of tensor m; a row that does not exist (the wavefront has no item in this
// round) is read through buffers of zero length, which return zero and cost no traffic.
template <int J>
__device__ __forceinline__ void load_row_c(u32x4 (&w)[J], uint32_t& zwv, uint32_t (&sbv)[(J + 3) / 4], const QW m, int row,
                                           bool valid, int ws, int ss, int zs, int lane)
{
    const size_t r = valid ? static_cast<size_t>(row) : 0;
    const uint32_t on = valid ? 1u : 0u;
    const __amdgpu_buffer_rsrc_t rw = make_rsrc(uniform_ptr(m.w + r * ws), on * ws * 4);
    const __amdgpu_buffer_rsrc_t rz = make_rsrc(uniform_ptr(m.z + r * zs), on * zs * 4);
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(uniform_ptr(m.s + r * ss), on * ss * 2);
#pragma unroll
    for (int j = 0; j < J; ++j)
        w[j] = __builtin_amdgcn_raw_buffer_load_b128(rw, lane * 16 + j * 1024, 0, kAuxStream);
    zwv = __builtin_amdgcn_raw_buffer_load_b32(rz, lane * 4, 0, 0);
#pragma unroll
    for (int k = 0; k < (J + 3) / 4; ++k)
        sbv[k] = __builtin_amdgcn_raw_buffer_load_b16(rs, lane * 2 + k * 128, 0, 0);
}

// The fragment layout the dot product reads: chunk column j of lane l belongs to group
// (l >> 2) + 16 j, whose zero point sits in zero word (l >> 5) + 2 j.
template <int J, int R>
__device__ __forceinline__ void expand(Frag<J, R>& f, const CFrag<J, R>& c, int lane)
{
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int j = 0; j < J; ++j) {
            f.w[r][j] = c.w[r][j];
            f.zw[r][j] = static_cast<uint32_t>(
                __builtin_amdgcn_ds_bpermute(((lane >> 5) + 2 * j) * 4, static_cast<int>(c.zwv[r])));
            f.sb[r][j] = static_cast<uint16_t>(
                __builtin_amdgcn_ds_bpermute((((lane >> 2) + 16 * j) & 63) * 4, static_cast<int>(c.sbv[r][j >> 2])));
        }
}

// Rows per block: what fits in 8 weight loads (32 registers) per item; RB x ss <= 128 scales
// then always fit the one scale load (ss <= 16 J).
constexpr int block_rows(int J, int groups) { return 8 / (J * groups) < 1 ? 1 : 8 / (J * groups); }

// What a lane holds of an item: G groups (tensors, or the two halves of a RoPE pair) of RB
// consecutive rows, J chunks each; of every group's scales the pair (2 l, 2 l + 1) of its run of
// RB x ss, of its zero words word l of its run of RB x zs.
template <int J, int G, int RB>
struct BFrag {
    u32x4 w[G][RB][J];
    uint32_t sv[G];
    uint32_t zv[G];
};

template <int J, int RB>
__device__ __forceinline__ void load_block(u32x4 (&w)[RB][J], uint32_t& sv, uint32_t& zv, const QW m, int row0, int n_rows,
                                           int ws, int ss, int zs, int lane)
{
    // rows [row0, row0 + RB) of a tensor with n_rows rows; rows beyond the tensor read as zero
    const int have = n_rows - row0 < RB ? n_rows - row0 : RB;
    const size_t r0 = static_cast<size_t>(row0);
#pragma unroll
    for (int r = 0; r < RB; ++r) {
        // one descriptor per row: the ragged end of a row (K not a multiple of 2048) reads as zero
        const __amdgpu_buffer_rsrc_t rw = make_rsrc(uniform_ptr(m.w + (r0 + r) * ws), r < have ? ws * 4 : 0);
#pragma unroll
        for (int j = 0; j < J; ++j)
            w[r][j] = __builtin_amdgcn_raw_buffer_load_b128(rw, lane * 16 + j * 1024, 0, kAuxStream);
    }
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(uniform_ptr(m.s + r0 * ss), have * ss * 2);
    const __amdgpu_buffer_rsrc_t rz = make_rsrc(uniform_ptr(m.z + r0 * zs), have * zs * 4);
    sv = __builtin_amdgcn_raw_buffer_load_b32(rs, lane * 4, 0, 0);
    zv = __builtin_amdgcn_raw_buffer_load_b32(rz, lane * 4, 0, 0);
}

// Row r of a group in the layout the dot product reads.
template <int J, int RB>
__device__ __forceinline__ void expand_row(u32x4 (&fw)[J], uint32_t (&fzw)[J], uint16_t (&fsb)[J], const u32x4 (&w)[RB][J],
                                           uint32_t sv, uint32_t zv, int r, int ss, int zs, int lane)
{
#pragma unroll
    for (int j = 0; j < J; ++j) {
        fw[j] = w[r][j];
        const int si = r * ss + (lane >> 2) + 16 * j; // scale of group (l >> 2) + 16 j of row r
        const uint32_t pair = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute((si >> 1) * 4, static_cast<int>(sv)));
        fsb[j] = static_cast<uint16_t>(pair >> ((si & 1) * 16));
        const int zi = r * zs + (lane >> 5) + 2 * j;
        fzw[j] = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(zi * 4, static_cast<int>(zv)));
    }
}

template <int J, int MODE, int STAGE>
__global__ __launch_bounds__(256) void int4_matvec_block_kernel(Int4Args a)
{
    constexpr int G = (MODE == SWIGLU || MODE == QKV_ROPE) ? 2 : 1; // row groups per item
    constexpr int RB = block_rows(J, G);
    constexpr int OUT = MODE == QKV_ROPE ? 2 * RB : RB; // results per item
    constexpr int JC = J * 64;
    constexpr int WAVES = 4;
    __shared__ u32x4 xs[4 * JC];
    __shared__ float sx[JC];
    __shared__ float red4[4];
    __shared__ float rope_tab[MODE == QKV_ROPE ? kRopeHeadSize : 2]; // (cos, sin) pairs
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
    const int total_waves = gridDim.x * WAVES;
    const int first_item = blockIdx.x * WAVES + wave;
    // PLAIN / RESIDUAL / SWIGLU: blocks of RB rows per tensor; QKV_ROPE: blocks of RB (i, i + 64) pairs
    const int per_tensor = MODE == QKV_ROPE ? (a.N >> 1) / RB : (a.N + RB - 1) / RB;
    const int nitems = MODE == QKV_ROPE ? 3 * per_tensor : (MODE == SWIGLU ? per_tensor : a.n_tensors * per_tensor);

    auto item_tensor = [&](int it) { return MODE == SWIGLU ? 0 : (it >= per_tensor) + (it >= 2 * per_tensor); };
    auto item_row0 = [&](int it, int t) { // first row of group 0
        const int b = it - t * per_tensor;
        if (MODE == QKV_ROPE) {
            const int rem = b * RB; // 64 pairs per head, 64 % RB == 0
            return (rem >> 6) * kRopeHeadSize + (rem & 63);
        }
        return b * RB;
    };
    auto tensor = [&](int t) -> QW { return t == 0 ? a.m[0] : (t == 1 ? a.m[1] : a.m[2]); };
    auto load_item = [&](BFrag<J, G, RB>& f, uint32_t& res, int it) {
        it = __builtin_amdgcn_readfirstlane(it);
        const int t = item_tensor(it), row0 = item_row0(it, t);
        if (MODE == SWIGLU) {
            load_block<J, RB>(f.w[0], f.sv[0], f.zv[0], a.m[0], row0, a.N, a.ws, a.ss, a.zs, lane);
            load_block<J, RB>(f.w[G - 1], f.sv[G - 1], f.zv[G - 1], a.m[1], row0, a.N, a.ws, a.ss, a.zs, lane);
        } else if (MODE == QKV_ROPE) {
            load_block<J, RB>(f.w[0], f.sv[0], f.zv[0], tensor(t), row0, a.N, a.ws, a.ss, a.zs, lane);
            load_block<J, RB>(f.w[G - 1], f.sv[G - 1], f.zv[G - 1], tensor(t), row0 + 64, a.N, a.ws, a.ss, a.zs, lane);
        } else {
            load_block<J, RB>(f.w[0], f.sv[0], f.zv[0], tensor(t), row0, a.N, a.ws, a.ss, a.zs, lane);
            if (MODE == RESIDUAL) { // the residuals of the block, row r in lane r
                const int have = a.N - row0 < RB ? a.N - row0 : RB;
                const __amdgpu_buffer_rsrc_t ro = make_rsrc(uniform_ptr(a.out[0] + row0), have * 2);
                res = __builtin_amdgcn_raw_buffer_load_b16(ro, lane * 2, 0, 0);
            }
        }
    };

    // input first (served by L2), then the first item's weights (HBM)
    VecPieces<J> xp;
    const uint16_t* xsrc = a.x;
    if (STAGE == STAGE_RMSNORM && a.embedding) { // native/embedding_kernel.cu:9-11
        int token = a.tokens[a.pos_ptr ? a.pos_ptr[0] : 0];
        token = token < 0 ? 0 : (token >= a.vocab ? a.vocab - 1 : token); // never read outside the table
        xsrc = a.embedding + static_cast<size_t>(token) * a.K;
    }
    xp.load(xsrc, a.K);
    VecPieces<J> gp;
    if (STAGE == STAGE_RMSNORM)
        gp.load(a.gamma, a.K);
    // The RoPE table is requested before the weights as well: loads return in order, so a value
    // requested after them would hold up the staging below until the first weights have arrived.
    float rope_entry = 0.0f;
    if (MODE == QKV_ROPE && a.rope_table && threadIdx.x < kRopeHeadSize)
        rope_entry = a.rope_table[threadIdx.x];
    asm volatile("" ::: "memory"); // the input stays ahead of the weights in the memory queue
    BFrag<J, G, RB> cur;
    uint32_t cur_res = 0;
    int item = first_item;
    if (item < nitems)
        load_item(cur, cur_res, item);

    // The position lives in device memory: outside layer 0 it is read only here, after the weight
    // loads above were issued.
    const int pos = MODE == QKV_ROPE && a.pos_ptr ? a.pos_ptr[0] : 0;
    if (MODE == QKV_ROPE) {
        if (a.rope_table) { // prepared by the kernel that set the position
            if (threadIdx.x < kRopeHeadSize)
                rope_tab[threadIdx.x] = rope_entry;
        } else if (threadIdx.x < kRopeHeadSize / 2) {
            float c, s;
            rope_cos_sin(c, s, threadIdx.x, kRopeHeadSize, pos, a.theta);
            rope_tab[2 * threadIdx.x] = c;
            rope_tab[2 * threadIdx.x + 1] = s;
        }
    }
    if (STAGE == STAGE_RMSNORM) {
        if (a.embedding && blockIdx.x == 0) { // the residual stream starts as the embedding row
            const __amdgpu_buffer_rsrc_t ro = make_rsrc(a.x_out, a.K * 2);
#pragma unroll
            for (int i = 0; i < J; ++i)
                __builtin_amdgcn_raw_buffer_store_b128(xp.v[i], ro, (threadIdx.x + i * 256) * 16, 0, 0);
        }
        const float ss = block256_sum(xp.sum_squares(), red4);
        const float rms = 1.0f / sqrtf(ss / static_cast<float>(a.K) + a.eps); // native/rmsnorm_kernel.cu:25-27
        xp.scale(rms, gp);
    }
    commit_pieces<J>(xs, sx, xp);
    __syncthreads();

    const int zshift = ((lane >> 2) & 7) * 4; // nibble of the zero word: group (c/4) % 8, same for every j
    uint32_t outw = 0; // result p of this wavefront in lane p: item k contributes lanes [k OUT, (k + 1) OUT)
    int filled = 0, flushed_items = 0;

    // Stores what has been collected: lane p holds result p % OUT of item first_item + (flushed_items + p / OUT) total_waves.
    auto flush = [&]() {
        const int k = lane / OUT, o = lane - k * OUT;
        const int it = first_item + (flushed_items + k) * total_waves;
        if (lane < filled && it < nitems) {
            const int t = item_tensor(it), row0 = item_row0(it, t);
            if (MODE == QKV_ROPE) {
                uint16_t* dst = t == 0 ? a.out[0] : (t == 1 ? a.out[1] : a.out[2]) + static_cast<size_t>(pos) * a.kv_dim;
                const int row = row0 + (o % RB) + 64 * (o / RB);
                dst[row] = static_cast<uint16_t>(outw);
            } else {
                uint16_t* dst = t == 0 ? a.out[0] : (t == 1 ? a.out[1] : a.out[2]);
                if (row0 + o < a.N)
                    dst[row0 + o] = static_cast<uint16_t>(outw);
            }
        }
        flushed_items += filled / OUT;
        filled = 0;
    };

    while (item < nitems) {
        const int nitem = item + total_waves;
        BFrag<J, G, RB> nxt;
        uint32_t nxt_res = 0;
        if (nitem < nitems)
            load_item(nxt, nxt_res, nitem);
        // the RB rows of the block (and of its partner group) against the staged input, together
        Frag<J, G * RB> f;
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int r = 0; r < RB; ++r)
                expand_row<J, RB>(f.w[g * RB + r], f.zw[g * RB + r], f.sb[g * RB + r], cur.w[g], cur.sv[g], cur.zv[g], r, a.ss,
                                  a.zs, lane);
        float acc[G * RB];
        dot_frag<J, G * RB>(acc, f, xs, sx, lane, zshift);
        const int t = item_tensor(item);
#pragma unroll
        for (int r = 0; r < RB; ++r) {
            if (MODE == SWIGLU) {
                const float g = wave_sum(acc[r]), u = wave_sum(acc[RB + r]);
                float v = g;
                v *= 1.0f / (1.0f + expf(-v)); // native/mat_vec_kernel.cu:219-221
                v *= u;
                outw = lane == filled + r ? float_to_half_bits(v) : outw;
            } else if (MODE == QKV_ROPE) {
                // the unfused path stores q/k as fp16 and RoPE reads them back: keep that rounding
                const float v0 = half_bits_to_float(float_to_half_bits(wave_sum(acc[r])));
                const float v1 = half_bits_to_float(float_to_half_bits(wave_sum(acc[RB + r])));
                const int i = ((item - t * per_tensor) * RB + r) & 63;
                uint16_t b0 = float_to_half_bits(v0), b1 = float_to_half_bits(v1);
                if (t < 2) // native/rope_kernel.cu:14-26
                    rope_rotate(b0, b1, v0, v1, rope_tab[2 * i], rope_tab[2 * i + 1]);
                outw = lane == filled + r ? b0 : outw;
                outw = lane == filled + RB + r ? b1 : outw;
            } else {
                float v = wave_sum(acc[r]);
                if (MODE == RESIDUAL)
                    v += half_bits_to_float(static_cast<uint16_t>(__builtin_amdgcn_readlane(static_cast<int>(cur_res), r)));
                outw = lane == filled + r ? float_to_half_bits(v) : outw;
            }
        }
        filled += OUT;
        if (filled + OUT > 64)
            flush();
        cur = nxt;
        cur_res = nxt_res;
        item = nitem;
    }
    flush();
}

// ---------------------------------------------------------------------------------------------
// Spans of consecutive rows per wavefront, statically scheduled.
//
// Measured on the 7B shapes against a pure read of the same bytes (which takes 2.7 / 5.2 / 8.0 /
// 4.7 us for the o-proj / QKV / SwiGLU / down-proj tensors), the kernels above lose their time in
// fixed costs, not in the streaming rate:
//   * a 2-byte result stored by 64 different workgroups into one 128-byte line, from all 8 XCDs
//     (workgroups are dealt to the XCDs round-robin), leaves that line partially dirty in 8 L2s:
//     0.45 us per launch at the kernel's end.  Here runs of 16 consecutive workgroups are mapped to
//     one XCD, so a line of the output is merged in ONE L2 and written back whole;
//   * the per-row scale / zero-word loads: a wavefront owns ROWS consecutive rows of each tensor,
//     so their scales are one contiguous run and their zero words another, fetched once per
//     wavefront (one or two 4-byte-per-lane loads each), parked in a wave-private piece of LDS and
//     read per row from there.  Per row only the J 16-byte weight loads remain;
//   * a conditional prefetch ("if there is a next row, request it") makes the compiler wait for
//     ALL outstanding loads where the two paths merge.  Here the row sequence is fully unrolled and
//     every load is unconditional (a row that does not exist is read through a descriptor of
//     length zero: no traffic), so the number of loads in flight is known at every point and
//     each wait is for exactly the loads that are needed; the staging of the input no longer
//     waits for the first weights either;
//   * results stay in lanes (row i of the span in lane i) and are stored once, after the last row;
//     residual add and SwiGLU run lane-parallel there;
//   * the first row of a span is found without a division (base / remainder from the host);
//   * what the instruction stream showed, once read: a load of the position placed after the first
//     row's requests had become "vector load, wait for everything"; the kernel arguments were
//     fetched in five dependent round trips; with one row per wavefront the compiler mixed the dot
//     product into the staging code.  See the comments at those three places below.
// QKV_ROPE: a workgroup of 8 wavefronts takes rows n .. n + 3 and n + 64 .. n + 67 of a head (of
// q, k and v), the two halves of four RoPE pairs, and exchanges the fp16-rounded results through LDS.
// ---------------------------------------------------------------------------------------------

struct SpanPlan {
    int grid;      // workgroups
    int base, rem; // rows per wavefront: base, one more for the first rem wavefronts
};

// Scale words (pairs of fp16) a lane fetches per tensor: ROWS rows of at most 16 J scales each.
constexpr int span_scale_words(int J, int ROWS) { return (ROWS * 16 * J + 127) / 128; }

template <int J, int MODE, int STAGE, int TN, int WAVES, int ROWS>
__global__ __launch_bounds__(WAVES * 64) void int4_matvec_span_kernel(Int4Args a, SpanPlan plan)
{
    static_assert(MODE != QKV_ROPE || (WAVES == 8 && ROWS == 1 && TN == 3), "RoPE pairs: 8 wavefronts, one row each");
    constexpr int SD = span_scale_words(J, ROWS);
    constexpr int JC = J * 64;
    constexpr int Q = ROWS * TN; // row loads per wavefront
    __shared__ u32x4 xs[4 * JC];
    __shared__ float sx[JC];
    __shared__ float red4[4];
    __shared__ uint32_t meta_s[WAVES][TN][SD * 64];
    __shared__ uint32_t meta_z[WAVES][TN][64];
    __shared__ float rope_tab[MODE == QKV_ROPE ? kRopeHeadSize : 2]; // (cos, sin) pairs
    __shared__ float pair_val[MODE == QKV_ROPE ? 2 * WAVES : 2];     // q and k of every wavefront's row
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
    // Workgroups go to the 8 XCDs round-robin: within every aligned group of 128 workgroups, give each
    // XCD a run of 16 consecutive ones (64 or more consecutive rows: whole lines of the output).
    int bx = blockIdx.x;
    if (bx < static_cast<int>(gridDim.x & ~127u)) {
        const int k = bx >> 3;
        bx = (k >> 4) * 128 + (bx & 7) * 16 + (k & 15);
    }
    int r0, n;
    if (MODE == QKV_ROPE) { // 16 workgroups per head: rows 4 b .. 4 b + 3 (wavefronts 0-3) and + 64 (wavefronts 4-7)
        r0 = (bx >> 4) * kRopeHeadSize + (bx & 15) * 4 + (wave & 3) + (wave >> 2) * 64;
        n = r0 < a.N ? 1 : 0;
    } else {
        const int gw = bx * WAVES + wave;
        r0 = gw * plan.base + (gw < plan.rem ? gw : plan.rem);
        n = plan.base + (gw < plan.rem ? 1 : 0); // ROWS or ROWS - 1; 0 beyond the tensor
        if (r0 >= a.N)
            n = 0;
    }

    auto load_w = [&](u32x4 (&w)[J], int q) { // q = i TN + t: constants after unrolling
        const int i = q / TN, t = q % TN;
        const __amdgpu_buffer_rsrc_t rw =
            make_rsrc(uniform_ptr(a.m[t].w + static_cast<size_t>(r0 + i) * a.ws), i < n ? a.ws * 4 : 0);
#pragma unroll
        for (int j = 0; j < J; ++j)
            w[j] = __builtin_amdgcn_raw_buffer_load_b128(rw, lane * 16 + j * 1024, 0, kAuxStream);
    };

    // The decode step's kernels (RMSNorm in the staging) fetch every kernel argument they read in one
    // round trip: left to itself the compiler fetches them where they are first used, five dependent
    // round trips to the scalar cache before the first weight is requested (decode 910 -> 917 tok/s).
    // The kernels that stage the input as given have shorter chains and lose 1 .. 3 % with it.
    if (STAGE == STAGE_RMSNORM) {
        asm volatile("" ::"s"(a.m[0].w), "s"(a.m[0].z), "s"(a.m[0].s), "s"(a.out[0]), "s"(a.x), "s"(a.K), "s"(a.N),
                     "s"(a.ws), "s"(a.ss), "s"(a.zs), "s"(a.gamma), "s"(a.eps), "s"(a.embedding));
        if (TN > 1)
            asm volatile("" ::"s"(a.m[1].w), "s"(a.m[1].z), "s"(a.m[1].s), "s"(a.out[1]));
        if (TN > 2)
            asm volatile("" ::"s"(a.m[2].w), "s"(a.m[2].z), "s"(a.m[2].s), "s"(a.out[2]));
        if (MODE == QKV_ROPE)
            asm volatile("" ::"s"(a.pos_ptr), "s"(a.kv_dim), "s"(a.rope_table));
    }
    // The position of the step, for the cache row of k and v: requested ahead of everything else as a
    // vector load and taken into a scalar register only where it is used.  Vector loads return in order
    // and are waited for by count; read where it is used (`a.pos_ptr[0]` after the first row's requests)
    // it made the wavefront wait for that whole row before the input could be staged.
    uint32_t pos_bits = 0;
    if (MODE == QKV_ROPE)
        pos_bits = __builtin_amdgcn_raw_buffer_load_b32(make_rsrc(a.pos_ptr, a.pos_ptr ? 4 : 0), 0, 0, 0);
    auto position = [&]() -> int {
        asm volatile("" : "+v"(pos_bits)); // stays where it is written
        return __builtin_amdgcn_readfirstlane(static_cast<int>(pos_bits)); // 0 without pos_ptr: nothing was read
    };
    // input next, then the span's scales / zero words / residuals, then the first row
    const bool stager = WAVES == 4 || threadIdx.x < 256;
    VecPieces<J> xp, gp;
    const uint16_t* xsrc = a.x;
    if (STAGE == STAGE_RMSNORM && a.embedding) { // native/embedding_kernel.cu:9-11
        int token = a.tokens[a.pos_ptr ? a.pos_ptr[0] : 0];
        token = token < 0 ? 0 : (token >= a.vocab ? a.vocab - 1 : token); // never read outside the table
        xsrc = a.embedding + static_cast<size_t>(token) * a.K;
    }
    if (stager) {
        xp.load(xsrc, a.K);
        if (STAGE == STAGE_RMSNORM)
            gp.load(a.gamma, a.K);
    }
    float rope_entry = 0.0f;
    if (MODE == QKV_ROPE && a.rope_table && threadIdx.x < kRopeHeadSize)
        rope_entry = a.rope_table[threadIdx.x];
    uint32_t sreg[TN][SD], zreg[TN], res = 0;
#pragma unroll
    for (int t = 0; t < TN; ++t) {
        const __amdgpu_buffer_rsrc_t rs = make_rsrc(uniform_ptr(a.m[t].s + static_cast<size_t>(r0) * a.ss), n * a.ss * 2);
        const __amdgpu_buffer_rsrc_t rz = make_rsrc(uniform_ptr(a.m[t].z + static_cast<size_t>(r0) * a.zs), n * a.zs * 4);
#pragma unroll
        for (int k = 0; k < SD; ++k)
            sreg[t][k] = __builtin_amdgcn_raw_buffer_load_b32(rs, lane * 4 + k * 256, 0, 0);
        zreg[t] = __builtin_amdgcn_raw_buffer_load_b32(rz, lane * 4, 0, 0);
    }
    if (MODE == RESIDUAL) {
        const __amdgpu_buffer_rsrc_t ro = make_rsrc(uniform_ptr(a.out[0] + r0), n * 2);
        res = __builtin_amdgcn_raw_buffer_load_b16(ro, lane * 2, 0, 0);
    }
    asm volatile("" ::: "memory"); // the small loads stay ahead of the weights in the memory queue
    u32x4 ring[2][J];
    load_w(ring[0], 0);
    asm volatile("" ::: "memory");

    if (MODE == QKV_ROPE) {
        if (a.rope_table) { // prepared by the kernel that set the position
            if (threadIdx.x < kRopeHeadSize)
                rope_tab[threadIdx.x] = rope_entry;
        } else {
            const int pos = position(); // all threads: the value is moved from lane 0
            if (threadIdx.x < kRopeHeadSize / 2) {
                float c, sn;
                rope_cos_sin(c, sn, threadIdx.x, kRopeHeadSize, pos, a.theta);
                rope_tab[2 * threadIdx.x] = c;
                rope_tab[2 * threadIdx.x + 1] = sn;
            }
        }
    }
    if (STAGE == STAGE_RMSNORM) {
        if (a.embedding && blockIdx.x == 0 && stager) { // the residual stream starts as the embedding row
            const __amdgpu_buffer_rsrc_t ro = make_rsrc(a.x_out, a.K * 2);
#pragma unroll
            for (int i = 0; i < J; ++i)
                __builtin_amdgcn_raw_buffer_store_b128(xp.v[i], ro, (threadIdx.x + i * 256) * 16, 0, 0);
        }
        // the sum of the stand-alone RMSNorm: wavefronts 0-3 each a quarter, added in its order
        float part = stager ? wave_sum(xp.sum_squares()) : 0.0f;
        if (stager && lane == 0)
            red4[wave] = part;
        __syncthreads();
        const float ss = (red4[0] + red4[1]) + (red4[2] + red4[3]);
        const float rms = 1.0f / sqrtf(ss / static_cast<float>(a.K) + a.eps); // native/rmsnorm_kernel.cu:25-27
        if (stager)
            xp.scale(rms, gp);
    }
    if (stager)
        commit_pieces_t<J>(xs, sx, xp, threadIdx.x);
#pragma unroll
    for (int t = 0; t < TN; ++t) {
#pragma unroll
        for (int k = 0; k < SD; ++k)
            meta_s[wave][t][lane + 64 * k] = sreg[t][k];
        meta_z[wave][t][lane] = zreg[t];
    }
    __syncthreads();

    const int zshift = ((lane >> 2) & 7) * 4; // nibble of the zero word: group (c/4) % 8, same for every j
    float outv[TN];
#pragma unroll
    for (int t = 0; t < TN; ++t)
        outv[t] = 0.0f;
#pragma unroll
    for (int q = 0; q < Q; ++q) {
        if (q + 1 < Q)
            load_w(ring[(q + 1) & 1], q + 1);
        // One row per wavefront: nothing of the dot product is moved up into the staging code (measured:
        // o-proj 3.88 -> 3.68 us, down-proj 6.39 -> 6.29).  With more rows the same fence lets the
        // compiler pull the requests of row q + 2 into the arithmetic of row q, which costs the
        // SwiGLU launch 4 .. 10 %: there the order is left to the compiler.
        if (Q == 1)
            __builtin_amdgcn_sched_barrier(0);
        const int i = q / TN, t = q % TN;
        Frag<J, 1> cur;
        const uint16_t* sp = reinterpret_cast<const uint16_t*>(&meta_s[wave][t][0]) + i * a.ss + (lane >> 2);
        const uint32_t* zp = &meta_z[wave][t][0] + i * a.zs + (lane >> 5);
#pragma unroll
        for (int j = 0; j < J; ++j) {
            cur.w[0][j] = ring[q & 1][j];
            cur.sb[0][j] = sp[16 * j];
            cur.zw[0][j] = zp[2 * j];
        }
        float acc[1];
        dot_frag<J, 1>(acc, cur, xs, sx, lane, zshift);
        const float s = wave_sum(acc[0]);
        outv[t] = lane == i ? s : outv[t];
    }

    if (MODE == QKV_ROPE) {
        // the unfused path stores q/k as fp16 and RoPE reads them back: keep that rounding
        const float qv = half_bits_to_float(float_to_half_bits(__builtin_bit_cast(
            float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, outv[0])))));
        const float kv = half_bits_to_float(float_to_half_bits(__builtin_bit_cast(
            float, __builtin_amdgcn_readfirstlane(__builtin_bit_cast(int, outv[TN > 1 ? 1 : 0])))));
        if (lane == 0) {
            pair_val[2 * wave] = qv;
            pair_val[2 * wave + 1] = kv;
        }
        __syncthreads();
        const int pos = position();
        if (lane == 0 && n) {
            const int partner = wave ^ 4, i = r0 & 63; // pair index within the head
            const float c = rope_tab[2 * i], sn = rope_tab[2 * i + 1];
            uint16_t* kdst = a.out[1] + static_cast<size_t>(pos) * a.kv_dim;
            uint16_t* vdst = a.out[TN > 2 ? 2 : 0] + static_cast<size_t>(pos) * a.kv_dim;
            uint16_t b0, b1;
            // native/rope_kernel.cu:14-26: (v0, v1) = rows (i, i + 64) of the head
            if (wave < 4) {
                rope_rotate(b0, b1, qv, pair_val[2 * partner], c, sn);
                a.out[0][r0] = b0;
                rope_rotate(b0, b1, kv, pair_val[2 * partner + 1], c, sn);
                kdst[r0] = b0;
            } else {
                rope_rotate(b0, b1, pair_val[2 * partner], qv, c, sn);
                a.out[0][r0] = b1;
                rope_rotate(b0, b1, pair_val[2 * partner + 1], kv, c, sn);
                kdst[r0] = b1;
            }
            vdst[r0] = float_to_half_bits(outv[TN > 2 ? 2 : 0]);
        }
    } else if (lane < n) {
        if (MODE == SWIGLU) {
            float v = outv[0];
            v *= 1.0f / (1.0f + expf(-v)); // native/mat_vec_kernel.cu:219-221
            v *= outv[TN - 1];
            a.out[0][r0 + lane] = float_to_half_bits(v);
        } else if (MODE == RESIDUAL) {
            a.out[0][r0 + lane] = float_to_half_bits(outv[0] + half_bits_to_float(static_cast<uint16_t>(res)));
        } else {
#pragma unroll
            for (int t = 0; t < TN; ++t)
                a.out[t][r0 + lane] = float_to_half_bits(outv[t]);
        }
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
        xs_dyn[(e & 3) * nchunks + (e >> 2)] = staged_order(v, e & 3);
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
        const int t = MODE == SWIGLU ? 0 : (it >= a.N) + (it >= 2 * a.N), n = it - t * a.N;
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
                float a0 = 0.0f, a0n = 0.0f, a1 = 0.0f;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const u32x4 xv = xs_dyn[i * nchunks + cc];
                    const uint32_t w = w4[i], w8 = w >> 8;
                    float& lo = i < 2 ? a0 : a0n;
                    lo = __builtin_amdgcn_fdot2(as_h2(w & 0x000F000Fu), as_h2(xv[0]), lo, false);
                    a1 = __builtin_amdgcn_fdot2(as_h2(w & 0x00F000F0u), as_h2(xv[1]), a1, false);
                    lo = __builtin_amdgcn_fdot2(as_h2(w8 & 0x000F000Fu), as_h2(xv[2]), lo, false);
                    a1 = __builtin_amdgcn_fdot2(as_h2(w8 & 0x00F000F0u), as_h2(xv[3]), a1, false);
                }
                const float zf = static_cast<float>((zw >> zshift) & 0xFu);
                float tt = a0 * 16777216.0f;
                tt = fmaf(a0n, -16777216.0f, tt);
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

// Wavefronts of a 256-thread kernel that fit on the GPU at once.  The kernels here are persistent
// (a wavefront walks over its rows until none is left), so a grid larger than that is not "more
// parallelism": the workgroups that do not fit start when the first ones are done, a second round
// that nobody overlaps with (13B QKV: 13.4 us with 20 wavefronts per CU requested and 16 resident,
// 11.0 us with 16 requested).
template <auto Kernel, int THREADS = 256>
inline int resident_waves()
{
    static int waves = 0, for_cus = -1; // per kernel instantiation; recomputed if the device changed
    const int cus = ctx().num_cus > 0 ? ctx().num_cus : 256;
    if (for_cus != cus) {
        int blocks = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, Kernel, THREADS, 0) != hipSuccess || blocks <= 0)
            blocks = 1;
        waves = blocks * (THREADS / 64) * cus;
        for_cus = cus;
    }
    return waves;
}

// The span kernel for this launch, if the shape suits it: scales readable 4 bytes at a time, and
// all wavefronts resident at once with ROWS rows each.
template <int J, int MODE, int STAGE, int TN, int WAVES, int ROWS>
inline bool try_span(const Int4Args& a)
{
    constexpr auto kernel = int4_matvec_span_kernel<J, MODE, STAGE, TN, WAVES, ROWS>;
    SpanPlan plan{};
    if (MODE == QKV_ROPE) {
        if (a.N % kRopeHeadSize)
            return false;
        plan.grid = a.N / 8;
    } else {
        int waves = ceil_div(a.N, ROWS);
        waves = ceil_div(waves, WAVES * 8) * (WAVES * 8);
        plan.grid = waves / WAVES;
        plan.base = a.N / waves, plan.rem = a.N % waves;
    }
    if (plan.grid * WAVES > resident_waves<kernel, WAVES * 64>())
        return false;
    hipLaunchKernelGGL(kernel, dim3(plan.grid), dim3(WAVES * 64), 0, ctx().stream, a, plan);
    return true;
}

template <int J, int MODE, int STAGE>
inline bool launch_span(const Int4Args& a)
{
    if (ctx().int4_no_span || ctx().int4_narrow || ctx().int4_blocks || (a.ss & 1))
        return false;
    const int tn = MODE == SWIGLU ? 2 : a.n_tensors;
    for (int t = 0; t < tn; ++t)
        if (!aligned(a.m[t].s, 4))
            return false;
    // Rows per wavefront and wavefronts per workgroup as measured on the 7B / 13B shapes: one row per
    // wavefront where that many wavefronts fit, three for the SwiGLU pair of tensors.
    if constexpr (MODE == QKV_ROPE) {
        return a.n_tensors == 3 && try_span<J, MODE, STAGE, 3, 8, 1>(a);
    } else if constexpr (MODE == SWIGLU) {
        return try_span<J, MODE, STAGE, 2, 8, 3>(a) || try_span<J, MODE, STAGE, 2, 8, 4>(a);
    } else if constexpr (MODE == PLAIN) {
        if (a.n_tensors == 3)
            return try_span<J, MODE, STAGE, 3, 8, 1>(a) || try_span<J, MODE, STAGE, 3, 8, 2>(a);
        if (a.n_tensors != 1)
            return false;
    }
    if constexpr (MODE == PLAIN || MODE == RESIDUAL) {
        constexpr int W = J <= 3 ? 4 : 8;
        return try_span<J, MODE, STAGE, 1, W, 1>(a) || try_span<J, MODE, STAGE, 1, W, 2>(a);
    }
    return false;
}

template <int J, int MODE, int STAGE>
inline void launch_j(const Int4Args& a, int max_waves)
{
    if (launch_span<J, MODE, STAGE>(a))
        return;
    // Rows of up to 6144 inputs (J <= 3) measured faster one row per item (more wavefronts, each with
    // one row in flight): 7.0 against 7.8 us for the 7B QKV launch, 10.1 against 11.7 us for SwiGLU;
    // longer rows faster in blocks with the shared scale and zero loads (down-proj 7.4 against 7.8 us).
    if (ctx().int4_narrow || (J <= 3 && !ctx().int4_blocks)) {
        const int nitems = MODE == QKV_ROPE ? 3 * (a.N / 2) : a.n_tensors * a.N;
        const int fit = resident_waves<int4_matvec_kernel<J, MODE, STAGE>>();
        const int cap = max_waves < fit ? max_waves : fit;
        const int waves = nitems < cap ? nitems : cap;
        hipLaunchKernelGGL((int4_matvec_kernel<J, MODE, STAGE>), dim3(ceil_div(waves, 4)), dim3(256), 0, ctx().stream, a);
        return;
    }
    constexpr int G = (MODE == SWIGLU || MODE == QKV_ROPE) ? 2 : 1;
    constexpr int RB = block_rows(J, G);
    const int per_tensor = MODE == QKV_ROPE ? (a.N / 2) / RB : ceil_div(a.N, RB);
    const int nitems = MODE == QKV_ROPE ? 3 * per_tensor : (MODE == SWIGLU ? per_tensor : a.n_tensors * per_tensor);
    const int fit = resident_waves<int4_matvec_block_kernel<J, MODE, STAGE>>();
    const int cap = max_waves < fit ? max_waves : fit;
    const int waves = nitems < cap ? nitems : cap;
    hipLaunchKernelGGL((int4_matvec_block_kernel<J, MODE, STAGE>), dim3(ceil_div(waves, 4)), dim3(256), 0, ctx().stream, a);
}

// Number of chunk-columns a lane holds per row for a K-input tensor.
inline int chunk_columns(int ws) { return ceil_div(ws / 4, 64); }
constexpr int kMaxChunkColumns = 8; // K <= 16384 on the unrolled kernels

// Wavefronts kept resident per launch: 16 per CU while a lane holds up to 3
// chunks of a row (20 for the three-tensor QKV launch of single rows), 8 per CU
// for longer rows (more bytes in flight per lane).  Measured on the 7B shapes:
// 12 .. 24 per CU are within 5 % of each other.
template <int MODE, int STAGE>
inline int launch_int4(const char* fn, const Int4Args& a)
{
    const int J = chunk_columns(a.ws);
    const int cus = ctx().num_cus > 0 ? ctx().num_cus : 256;
    const int short_rows = cus * ((MODE == PLAIN && a.n_tensors == 3) ? 20 : 16); // capped to what fits: launch_j
    switch (J) {
    case 1: launch_j<1, MODE, STAGE>(a, short_rows); break;
    case 2: launch_j<2, MODE, STAGE>(a, short_rows); break;
    case 3: launch_j<3, MODE, STAGE>(a, short_rows); break;
    case 4: launch_j<4, MODE, STAGE>(a, cus * 8); break;
    case 5: launch_j<5, MODE, STAGE>(a, cus * 8); break;
    case 6: launch_j<6, MODE, STAGE>(a, cus * 8); break;
    case 7: launch_j<7, MODE, STAGE>(a, cus * 8); break;
    case 8: launch_j<8, MODE, STAGE>(a, cus * 8); break;
    default: {
        if (MODE == QKV_ROPE || STAGE != STAGE_X)
            return fail(LLAMA2_ERR_UNSUPPORTED, "%s: rows=%d exceeds the fused kernels' limit of %d", fn, a.K,
                        kMaxChunkColumns * 2048);
        const int nitems = a.n_tensors * a.N;
        const int grid = ceil_div(nitems < cus * 8 ? nitems : cus * 8, 4);
        constexpr int GM = (MODE == QKV_ROPE) ? PLAIN : MODE;
        hipLaunchKernelGGL((int4_matvec_generic_kernel<GM>), dim3(grid), dim3(256),
                           static_cast<size_t>(a.ws / 4) * 68, ctx().stream, a);
    }
    }
    L2_LAUNCH_CHECK(fn);
    return LLAMA2_OK;
}

} // namespace l2

// Shared host/device helpers of libllama2_hip.so (gfx950 only).
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <mutex>

#include "../../include/llama2_hip.h"

namespace l2 {

// ------------------------------------------------------------------ host side
constexpr int kMaxRetiredPartials = 32;

struct Context {
    bool ready = false;
    int device = -1;
    hipStream_t stream = nullptr;
    int num_cus = 0;
    bool capturing = false; // between llama2_graph_begin_capture and _end_capture
    // A/B switches of the int4 mat-vec launches: LLAMA2_INT4_NARROW=1 one row per item for every
    // shape, LLAMA2_INT4_BLOCKS=1 blocks of rows for every shape (default: by row length)
    // LLAMA2_INT4_NO_SPAN=1: never the span kernel (the shapes it does not take always go this way)
    bool int4_narrow = false;
    bool int4_blocks = false;
    bool int4_no_span = false;
    int attn_waves = 0; // LLAMA2_ATTN_WAVES: block size of the attention entry points, for sweeps (0: by length)
    // fp32 partial sums of the sequence-split attention kernels
    float* attn_partials = nullptr;
    size_t attn_partials_bytes = 0;
    // earlier, smaller buffers: a graph captured by the caller may still hold their address,
    // so they stay allocated until llama2_shutdown
    float* retired_partials[kMaxRetiredPartials] = {};
    int n_retired_partials = 0;
    // per-head arrival counters of llama2_multi_head_attention (zero between launches)
    unsigned* attn_counters = nullptr;
    // second buffer of the sampler's radix sort (LLAMA2_MAX_SAMPLER_SIZE keys and payloads)
    uint16_t* sort_keys = nullptr;
    int* sort_values = nullptr;
};

constexpr int kMaxAttnHeads = 1024;

Context& ctx();
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
int hip_fail(hipError_t e, const char* what);
int ensure_attn_partials(size_t bytes);
// Device address of llama2_vec_mat_static's scratch array on `device` (current), asked for once at llama2_init.
int resolve_vec_mat_static_scratch(int device);
// Sampler.Sample's stochastic branch in one launch (sampler.hip).  token_only: the caller reads the
// token alone, so the sort may stop at the head of the distribution that holds top_p of the mass.
int sample_launch(const char* fn, uint16_t* logits, int* indices, int size, float temperature, float top_p, float coin,
                  int* result, int pos, bool token_only);

// HIP's current device is a per-thread setting: a host thread other than the one that called
// llama2_init (a thread-pool worker of the managed host, say) is bound to the library's device on
// its first call.
int bind_thread();

// Every entry point runs under one recursive lock (entry points call each other): host threads
// that share the library -- one Transformer per connection, say -- take turns.  The GPU work is in
// order on one stream either way; what the lock protects is the stream-capture state and the lazily
// captured graphs.  llama2_graph_begin_capture keeps the lock until llama2_graph_end_capture.
std::recursive_mutex& api_mutex();

#define L2_REQUIRE_INIT()                                                          \
    std::lock_guard<std::recursive_mutex> l2_api_lock_(::l2::api_mutex());         \
    do {                                                                           \
        if (!::l2::ctx().ready)                                                    \
            return ::l2::fail(LLAMA2_ERR_NOT_INITIALIZED, "%s: llama2_init has not been called", __func__); \
        if (int rc_bind_ = ::l2::bind_thread())                                    \
            return rc_bind_;                                                       \
    } while (0)

#define L2_CHECK(cond, ...)                                                        \
    do {                                                                           \
        if (!(cond))                                                               \
            return ::l2::fail(LLAMA2_ERR_INVALID_ARGUMENT, __VA_ARGS__);           \
    } while (0)

#define L2_HIP(expr)                                                               \
    do {                                                                           \
        hipError_t e_ = (expr);                                                    \
        if (e_ != hipSuccess)                                                      \
            return ::l2::hip_fail(e_, #expr);                                      \
    } while (0)

#define L2_LAUNCH_CHECK(name)                                                      \
    do {                                                                           \
        hipError_t e_ = hipGetLastError();                                         \
        if (e_ != hipSuccess)                                                      \
            return ::l2::hip_fail(e_, name);                                       \
    } while (0)

inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }
inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline bool overlap(const void* a, size_t na, const void* b, size_t nb)
{
    auto pa = reinterpret_cast<uintptr_t>(a), pb = reinterpret_cast<uintptr_t>(b);
    return pa < pb + nb && pb < pa + na;
}

// ---------------------------------------------------------------- device side
#if defined(__HIPCC__)

typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ h2_t as_h2(uint32_t v) { return __builtin_bit_cast(h2_t, v); }
__device__ __forceinline__ uint32_t as_u32(h2_t v) { return __builtin_bit_cast(uint32_t, v); }

// fp32 += a.x*b.x + a.y*b.y  (v_dot2_f32_f16: fp16 products, fp32 accumulate)
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc)
{
    return __builtin_amdgcn_fdot2(as_h2(a), as_h2(b), acc, false);
}

__device__ __forceinline__ float half_bits_to_float(uint16_t h)
{
    return static_cast<float>(__builtin_bit_cast(_Float16, h));
}
__device__ __forceinline__ uint16_t float_to_half_bits(float f)
{
    return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f)); // v_cvt_f16_f32, RNE
}

// The rotation of native/rope_kernel.cu:14-26, rounded the way the reference rounds it: the fp32
// value first, then __float2half of it.  The multiply-adds are spelled out and the fp32 results are
// made opaque before the conversion, so that every kernel that inlines this produces the same bits:
// left alone, the compiler fuses some of these multiply-adds with the conversion (v_fma_mixlo_f16,
// ONE rounding straight to fp16) and not others, depending on the surrounding code, and a value
// near an fp16 tie then rounds differently from kernel to kernel.
__device__ __forceinline__ void rope_rotate(uint16_t& b0, uint16_t& b1, float v0, float v1, float fcr, float fci)
{
    float o0 = __builtin_fmaf(v0, fcr, -(v1 * fci));
    float o1 = __builtin_fmaf(v0, fci, v1 * fcr);
    asm volatile("" : "+v"(o0), "+v"(o1));
    b0 = float_to_half_bits(o0);
    b1 = float_to_half_bits(o1);
}

// DPP controls (GCN3/CDNA encoding)
constexpr int DPP_QUAD_XOR1 = 0xB1;        // quad_perm:[1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;        // quad_perm:[2,3,0,1]
constexpr int DPP_ROW_HALF_MIRROR = 0x141; // lane i <- lane 7-i within 8
constexpr int DPP_ROW_MIRROR = 0x140;      // lane i <- lane 15-i within 16
constexpr int DPP_ROW_BCAST15 = 0x142;     // lane 15 of each row -> next row
constexpr int DPP_ROW_BCAST31 = 0x143;     // lane 31 -> rows 2,3

template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ float dpp_f32(float v)
{
    // lanes whose row is masked out (or whose source is invalid) read 0
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, false));
}

// Sum over each 16-lane row; every lane of the row ends with the row total.
__device__ __forceinline__ float row16_sum(float v)
{
    v += dpp_f32<DPP_QUAD_XOR1>(v);
    v += dpp_f32<DPP_QUAD_XOR2>(v);
    v += dpp_f32<DPP_ROW_HALF_MIRROR>(v);
    v += dpp_f32<DPP_ROW_MIRROR>(v);
    return v;
}

// Sum over the 64-lane wavefront, returned in every lane (as a scalar).
__device__ __forceinline__ float wave_sum(float v)
{
    v = row16_sum(v);
    v += dpp_f32<DPP_ROW_BCAST15, 0xA>(v);
    v += dpp_f32<DPP_ROW_BCAST31, 0xC>(v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
        v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// Data handed from one workgroup to another INSIDE a kernel (attention partials,
// arrival counters) moves through agent-scope accesses: the store is written
// through to the level every XCD sees, the load bypasses this XCD's possibly
// stale L2 lines.  That replaces __threadfence(), whose L2 write-back +
// invalidate costs tens of microseconds on this part.  Ordering: a producer
// calls wait_agent_stores() before it announces its data with an atomic.
__device__ __forceinline__ void store_agent(float* p, float v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_agent(const float* p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_agent(unsigned* p, unsigned v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned add_agent(unsigned* p, unsigned v)
{
    return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void wait_agent_stores() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Sum over a 256-thread workgroup (4 wavefronts), identical in every thread and
// independent of which kernel calls it: RMSNorm is evaluated both by the
// stand-alone module and inside the fused mat-vec kernels, and the two must
// agree bit for bit.  `lds4` holds 4 floats.
__device__ __forceinline__ float block256_sum(float v, float* lds4)
{
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0)
        lds4[threadIdx.x >> 6] = v;
    __syncthreads();
    const float t = (lds4[0] + lds4[1]) + (lds4[2] + lds4[3]);
    __syncthreads();
    return t;
}

// Cache-policy bits of the raw buffer load/store builtins on gfx94x/gfx950.
constexpr int kAuxNonTemporal = 2; // "nt": streamed once, do not keep
constexpr int kAuxAgent = 16;      // "sc1": coherent at agent scope (sees other workgroups' sc1 stores)

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes)
{
    // raw buffer, 32-bit elements; out-of-range reads return 0
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, static_cast<int>(bytes), 0x00020000);
}

// One thread's share of a K-element fp16 vector read 16 bytes at a time by a
// 256-thread workgroup: piece i covers elements 8*(tid + 256 i) .. +7.
template <int PIECES>
struct VecPieces {
    u32x4 v[PIECES];
    __device__ __forceinline__ void load(const uint16_t* p, int K)
    {
        const __amdgpu_buffer_rsrc_t r = make_rsrc(p, K * 2);
#pragma unroll
        for (int i = 0; i < PIECES; ++i)
            v[i] = __builtin_amdgcn_raw_buffer_load_b128(r, (threadIdx.x + i * 256) * 16, 0, 0);
    }
    __device__ __forceinline__ float sum_squares() const
    {
        float ss = 0.0f;
#pragma unroll
        for (int i = 0; i < PIECES; ++i)
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const h2_t p = as_h2(v[i][k]);
                const float a = static_cast<float>(p[0]), b = static_cast<float>(p[1]);
                ss += a * a;
                ss += b * b;
            }
        return ss;
    }
    // v <- half(rms * gamma * v), the product order of native/rmsnorm_kernel.cu:34
    __device__ __forceinline__ void scale(float rms, const VecPieces& gamma)
    {
#pragma unroll
        for (int i = 0; i < PIECES; ++i)
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const h2_t x = as_h2(v[i][k]), g = as_h2(gamma.v[i][k]);
                h2_t o;
                o[0] = static_cast<_Float16>(rms * static_cast<float>(g[0]) * static_cast<float>(x[0]));
                o[1] = static_cast<_Float16>(rms * static_cast<float>(g[1]) * static_cast<float>(x[1]));
                v[i][k] = as_u32(o);
            }
    }
};

// Largest fp16 value of x[0..size), lowest index among equals, by a workgroup of 1024 threads;
// valid in thread 0 (0 when every entry is NaN).  A candidate is the pair (value, index); `better`
// is a strict total order, so every reduction order yields the same winner (no race, unlike
// native/argmax_kernel.cu:32-36).  `sv`, `si`: 16 entries of LDS each.
__device__ __forceinline__ bool better(float va, int ia, float vb, int ib)
{
    return va > vb || (va == vb && ia < ib);
}

__device__ __forceinline__ int block1024_argmax(const uint16_t* x, int size, float* sv, int* si)
{
    float bv = -INFINITY;
    int bi = 0x7FFFFFFF;
    // 16 bytes per load while whole groups of 8 remain (when x is 16-byte aligned), the rest one by one
    const int n8 = (reinterpret_cast<uintptr_t>(x) & 15) == 0 ? size >> 3 : 0;
    for (int g = threadIdx.x; g < n8; g += 1024) {
        const u32x4 v = reinterpret_cast<const u32x4*>(x)[g];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float f = half_bits_to_float(static_cast<uint16_t>(v[k >> 1] >> (16 * (k & 1))));
            if (better(f, g * 8 + k, bv, bi)) {
                bv = f;
                bi = g * 8 + k;
            }
        }
    }
    for (int i = n8 * 8 + threadIdx.x; i < size; i += 1024) {
        const float f = half_bits_to_float(x[i]);
        if (better(f, i, bv, bi)) {
            bv = f;
            bi = i;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, 64);
        const int oi = __shfl_xor(bi, off, 64);
        if (better(ov, oi, bv, bi)) {
            bv = ov;
            bi = oi;
        }
    }
    if ((threadIdx.x & 63) == 0) {
        sv[threadIdx.x >> 6] = bv;
        si[threadIdx.x >> 6] = bi;
    }
    __syncthreads();
    if (threadIdx.x < 64) {
        bv = threadIdx.x < 16 ? sv[threadIdx.x] : -INFINITY;
        bi = threadIdx.x < 16 ? si[threadIdx.x] : 0x7FFFFFFF;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ov = __shfl_xor(bv, off, 64);
            const int oi = __shfl_xor(bi, off, 64);
            if (better(ov, oi, bv, bi)) {
                bv = ov;
                bi = oi;
            }
        }
    }
    return bi == 0x7FFFFFFF ? 0 : bi;
}

#endif // __HIPCC__


} // namespace l2

// The stochastic sampler of src/Sampler.cs:48-67 as device functions for one
// 1024-thread workgroup: softmax_logits, sort, cumulative_sum, sample_top_p
// (native/softmax_logits_kernel.cu, sort_kernel.cu, cumulative_sum_kernel.cu,
// sample_top_p_kernel.cu).  Each module kernel calls one of them; the decode
// step calls all four from a single launch.
//
// 32000 logits are 64 KB: the work is latency-bound, so every phase touches
// global memory once for reading and once for writing, 16 bytes per access,
// and keeps its share in registers in between.  CH is the number of 8-element
// chunks a thread holds: 4 up to 32768 elements, 8 up to 65536.
#pragma once

#include "common.hpp"

namespace l2 {

constexpr int kSampBlock = 1024;
constexpr int kSampWaves = kSampBlock / 64;

struct SamplerLds {
    float redf[kSampWaves];
    int redi[kSampWaves];
    uint16_t counts[16 * kSampBlock]; // sort: per (digit, thread) counters, then scatter cursors
};

// ---- 8-element chunks of fp16 / int32 -----------------------------------------------
// Whole chunks move as 16-byte accesses, the ragged last chunk element by element.
__device__ __forceinline__ void load_half8(float (&f)[8], const uint16_t* p, int base, int size, float fill)
{
    if (base + 8 <= size) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(p + base);
#pragma unroll
        for (int k = 0; k < 8; ++k)
            f[k] = half_bits_to_float(static_cast<uint16_t>(v[k >> 1] >> (16 * (k & 1))));
    } else {
#pragma unroll
        for (int k = 0; k < 8; ++k)
            f[k] = base + k < size ? half_bits_to_float(p[base + k]) : fill;
    }
}

__device__ __forceinline__ void load_bits8(uint16_t (&b)[8], const uint16_t* p, int base, int size)
{
    if (base + 8 <= size) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(p + base);
#pragma unroll
        for (int k = 0; k < 8; ++k)
            b[k] = static_cast<uint16_t>(v[k >> 1] >> (16 * (k & 1)));
    } else {
#pragma unroll
        for (int k = 0; k < 8; ++k)
            b[k] = base + k < size ? p[base + k] : static_cast<uint16_t>(0);
    }
}

__device__ __forceinline__ void store_half8(uint16_t* p, int base, int size, const uint16_t (&b)[8])
{
    if (base + 8 <= size) {
        u32x4 v;
#pragma unroll
        for (int k = 0; k < 4; ++k)
            v[k] = static_cast<uint32_t>(b[2 * k]) | (static_cast<uint32_t>(b[2 * k + 1]) << 16);
        *reinterpret_cast<u32x4*>(p + base) = v;
    } else {
#pragma unroll
        for (int k = 0; k < 8; ++k)
            if (base + k < size)
                p[base + k] = b[k];
    }
}

__device__ __forceinline__ void load_int8(int (&o)[8], const int* p, int base, int size)
{
    if (base + 8 <= size) {
        const u32x4 a = *reinterpret_cast<const u32x4*>(p + base), b = *reinterpret_cast<const u32x4*>(p + base + 4);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            o[k] = static_cast<int>(a[k]);
            o[4 + k] = static_cast<int>(b[k]);
        }
    } else {
#pragma unroll
        for (int k = 0; k < 8; ++k)
            o[k] = base + k < size ? p[base + k] : 0;
    }
}

__device__ __forceinline__ void store_int8(int* p, int base, int size, const int (&o)[8])
{
    if (base + 8 <= size) {
        u32x4 a, b;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            a[k] = static_cast<uint32_t>(o[k]);
            b[k] = static_cast<uint32_t>(o[4 + k]);
        }
        *reinterpret_cast<u32x4*>(p + base) = a;
        *reinterpret_cast<u32x4*>(p + base + 4) = b;
    } else {
#pragma unroll
        for (int k = 0; k < 8; ++k)
            if (base + k < size)
                p[base + k] = o[k];
    }
}

// ---- reductions and scans over the 1024 threads -------------------------------------
__device__ __forceinline__ float samp_block_sum(float v, float* lds)
{
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0)
        lds[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = (threadIdx.x & 63) < kSampWaves ? lds[threadIdx.x & 63] : 0.0f;
    t = wave_sum(t);
    __syncthreads();
    return t;
}

__device__ __forceinline__ float samp_block_max(float v, float* lds)
{
    v = wave_max(v);
    if ((threadIdx.x & 63) == 0)
        lds[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = (threadIdx.x & 63) < kSampWaves ? lds[threadIdx.x & 63] : -INFINITY;
    t = wave_max(t);
    __syncthreads();
    return t;
}

__device__ __forceinline__ int samp_block_min(int v, int* lds)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const int o = __shfl_xor(v, off, 64);
        v = o < v ? o : v;
    }
    if ((threadIdx.x & 63) == 0)
        lds[threadIdx.x >> 6] = v;
    __syncthreads();
    int t = (threadIdx.x & 63) < kSampWaves ? lds[threadIdx.x & 63] : 0x7FFFFFFF;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const int o = __shfl_xor(t, off, 64);
        t = o < t ? o : t;
    }
    __syncthreads();
    return t;
}

// Exclusive prefix of one value per thread, in thread order (fixed association:
// within a wavefront by doubling, then over the 16 wavefront totals).
template <typename T>
__device__ __forceinline__ T samp_block_exclusive_scan(T v, T* lds /* kSampWaves */)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    T inc = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const T o = __shfl_up(inc, off, 64);
        if (lane >= off)
            inc += o;
    }
    if (lane == 63)
        lds[wave] = inc;
    __syncthreads();
    T before = 0; // total of the wavefronts in front of this one
#pragma unroll
    for (int w = 0; w < kSampWaves; ++w)
        before += w < wave ? lds[w] : static_cast<T>(0);
    __syncthreads();
    return before + inc - v;
}

// ---- softmax_logits (native/softmax_logits_kernel.cu:8-53) ---------------------------
// indices[t] = t; logits <- half(logits / temperature); p = expf(l - max) rounded to
// fp16; logits <- half(float(half(p)) / sum of the unrounded p).  The three fp16
// roundings are the ones the reference's in-place buffer forces.
template <int CH>
__device__ __forceinline__ void softmax_logits_dev(uint16_t* logits, int size, float temperature, int* indices,
                                                   SamplerLds& lds)
{
    float f[CH][8];
    float m = -INFINITY;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int base = (threadIdx.x + c * kSampBlock) * 8;
        if (base < size) {
            load_half8(f[c], logits, base, size, -INFINITY);
            int idx[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                idx[k] = base + k;
                if (base + k < size) {
                    f[c][k] = half_bits_to_float(float_to_half_bits(f[c][k] / temperature));
                    m = fmaxf(m, f[c][k]);
                }
            }
            store_int8(indices, base, size, idx);
        }
    }
    m = samp_block_max(m, lds.redf);
    float sum = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int base = (threadIdx.x + c * kSampBlock) * 8;
        if (base < size) {
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if (base + k < size) {
                    const float v = expf(f[c][k] - m);
                    sum += v;
                    f[c][k] = half_bits_to_float(float_to_half_bits(v));
                }
        }
    }
    sum = samp_block_sum(sum, lds.redf);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int base = (threadIdx.x + c * kSampBlock) * 8;
        if (base < size) {
            uint16_t b[8];
#pragma unroll
            for (int k = 0; k < 8; ++k)
                b[k] = float_to_half_bits(f[c][k] / sum);
            store_half8(logits, base, size, b);
        }
    }
}

// ---- sort (native/sort_kernel.cu:13-37) ---------------------------------------------
// Stable descending radix sort of fp16 keys with int payloads: four passes of
// four bits over the keys' total order (sign-flipped bit pattern; +0 before -0).
// Thread t owns the 8*CH consecutive items starting at 8*CH*t, so "thread order,
// then item order" is the input order and the scatter is stable.  Even passes
// write (keys2, values2), odd passes write back: the result ends in place.
__device__ __forceinline__ uint32_t sort_rank(uint16_t k) // larger = sorts first
{
    return (k & 0x8000u) ? static_cast<uint32_t>(static_cast<uint16_t>(~k)) : static_cast<uint32_t>(k) | 0x8000u;
}

template <int CH>
__device__ __forceinline__ void sort_dev(uint16_t* keys, int* values, int size, uint16_t* keys2, int* values2,
                                         SamplerLds& lds)
{
    const int first = threadIdx.x * 8 * CH;
    uint16_t* kin = keys;
    int* vin = values;
    uint16_t* kout = keys2;
    int* vout = values2;
    for (int pass = 0; pass < 4; ++pass) {
        const int shift = 4 * pass;
        uint16_t kb[CH][8];
        uint32_t cnt[4] = {0u, 0u, 0u, 0u}; // 16 byte-wide counters (a thread owns at most 64 items)
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int base = first + c * 8;
            if (base < size) {
                load_bits8(kb[c], kin, base, size);
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    if (base + k < size) {
                        const uint32_t d = 15u - ((sort_rank(kb[c][k]) >> shift) & 15u); // bucket 0 = largest digit
                        const uint32_t inc = 1u << ((d & 3u) * 8u);
                        cnt[0] += (d >> 2) == 0u ? inc : 0u;
                        cnt[1] += (d >> 2) == 1u ? inc : 0u;
                        cnt[2] += (d >> 2) == 2u ? inc : 0u;
                        cnt[3] += (d >> 2) == 3u ? inc : 0u;
                    }
            }
        }
#pragma unroll
        for (int d = 0; d < 16; ++d)
            lds.counts[d * kSampBlock + threadIdx.x] = static_cast<uint16_t>((cnt[d >> 2] >> ((d & 3) * 8)) & 0xFFu);
        __syncthreads();
        // exclusive scan of the 16 x 1024 counters in (digit, thread) order: 16 consecutive per thread
        {
            uint16_t* mine = lds.counts + threadIdx.x * 16;
            int local[16], total = 0;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                local[i] = total;
                total += mine[i];
            }
            const int before = samp_block_exclusive_scan<int>(total, lds.redi);
#pragma unroll
            for (int i = 0; i < 16; ++i)
                mine[i] = static_cast<uint16_t>(before + local[i]); // < 65536: positions of a sort of at most 65536 items
        }
        __syncthreads();
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int base = first + c * 8;
            if (base < size) {
                int vb[8];
                load_int8(vb, vin, base, size);
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    if (base + k < size) {
                        const uint32_t d = 15u - ((sort_rank(kb[c][k]) >> shift) & 15u);
                        uint16_t* cursor = &lds.counts[d * kSampBlock + threadIdx.x]; // only this thread touches it
                        const int at = *cursor;
                        *cursor = static_cast<uint16_t>(at + 1);
                        kout[at] = kb[c][k];
                        vout[at] = vb[k];
                    }
            }
        }
        __syncthreads(); // the scattered items are visible to the whole workgroup
        uint16_t* tk = kin;
        kin = kout;
        kout = tk;
        int* tv = vin;
        vin = vout;
        vout = tv;
    }
}

// The same sort with every pass inside LDS, for up to kSortLdsItems items (a
// 32000-entry vocabulary fits).  Scattering 2- and 4-byte items to global memory
// from one compute unit costs one cache-line transaction per lane and made the
// sort above take 140 us for 32000 items; in LDS a scatter is a bank access.
// An item is (rank << 16) | original position; a thread owns 32 consecutive
// positions, kept in registers between passes.  Slot p lives at word
// p ^ ((p >> 5) & 31), so a thread reading its 32 consecutive slots and the 64
// lanes of a wavefront reading slot k of 64 threads both spread over all banks.
constexpr int kSortLdsThreads = 1008;
constexpr int kSortLdsItems = kSortLdsThreads * 32; // 32256: data + counters fill the 160 KB of LDS

struct SortLds {
    uint32_t item[kSortLdsItems];
};

__device__ __forceinline__ int sort_slot(int p) { return p ^ ((p >> 5) & 31); }
__device__ __forceinline__ uint16_t sort_key_of_rank(uint32_t rank)
{
    return static_cast<uint16_t>((rank & 0x8000u) ? rank ^ 0x8000u : ~rank);
}

// The four passes over items held C per thread (thread t owns positions C*t .. C*t + C - 1;
// C = 32 is the full vocabulary, smaller C a short list).  On return the thread holds the
// sorted items of its positions.
template <int C>
__device__ __forceinline__ void sort_passes(uint32_t (&it)[C], bool active, SamplerLds& lds, SortLds& buf)
{
    const int first = threadIdx.x * C;
    // Between the read-back of one pass and the scatter of the next the item
    // buffer is idle: its first 16 x 1024 words serve as 32-bit (bucket, thread)
    // counters, filled with fire-and-forget LDS adds.
    static_assert(kSortLdsItems >= 16 * kSampBlock, "the counters borrow the item buffer");
    uint32_t* cnt32 = buf.item;
    for (int pass = 0; pass < 4; ++pass) {
        const int shift = 16 + 4 * pass;
#pragma unroll
        for (int d = 0; d < 16; ++d)
            cnt32[d * kSampBlock + threadIdx.x] = 0u;
        // own words only: no barrier needed before the adds below
        if (active) {
#pragma unroll
            for (int k = 0; k < C; ++k) {
                const uint32_t d = 15u - ((it[k] >> shift) & 15u); // bucket 0 = largest digit
                __hip_atomic_fetch_add(&cnt32[d * kSampBlock + threadIdx.x], 1u, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_WORKGROUP);
            }
        }
        __syncthreads();
        {
            // exclusive scan in (bucket, thread) order: 16 consecutive counters per thread
            const u32x4* mine = reinterpret_cast<const u32x4*>(cnt32 + threadIdx.x * 16);
            int local[16], total = 0;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const u32x4 c4 = mine[q];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    local[q * 4 + i] = total;
                    total += static_cast<int>(c4[i]);
                }
            }
            const int before = samp_block_exclusive_scan<int>(total, lds.redi);
            u32x4* out = reinterpret_cast<u32x4*>(lds.counts + threadIdx.x * 16);
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                u32x4 w;
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    w[i] = static_cast<uint32_t>(before + local[q * 8 + 2 * i]) |
                           (static_cast<uint32_t>(before + local[q * 8 + 2 * i + 1]) << 16);
                out[q] = w; // 16-bit cursors: positions stay below 32256
            }
        }
        __syncthreads();
        if (active) {
            // the cursor of (bucket, thread) is one half of a 32-bit word shared with the neighbouring
            // thread: an LDS add on the word returns the old cursor and advances it in one operation
            uint32_t* words = reinterpret_cast<uint32_t*>(lds.counts);
            const uint32_t one = (threadIdx.x & 1) ? 0x10000u : 1u;
            const int hshift = (threadIdx.x & 1) * 16;
#pragma unroll
            for (int k = 0; k < C; ++k) {
                const uint32_t d = 15u - ((it[k] >> shift) & 15u);
                const uint32_t old = __hip_atomic_fetch_add(&words[(d * kSampBlock + threadIdx.x) >> 1], one,
                                                            __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                const int at = static_cast<int>((old >> hshift) & 0xFFFFu);
                buf.item[sort_slot(at)] = it[k];
                if ((k & 7) == 7)
                    asm volatile("" ::: "memory"); // at most 8 cursors in flight: keeps the items in registers
            }
        }
        __syncthreads();
        if (active) {
#pragma unroll
            for (int k = 0; k < C; ++k)
                it[k] = buf.item[sort_slot(first + k)];
        }
        __syncthreads(); // everyone has its items back before the buffer turns into counters again
    }
}

// The thread's 32 consecutive keys as sort items: (rank << 16) | position.
__device__ __forceinline__ void sort_load_items(uint32_t (&it)[32], const uint16_t* keys, int size)
{
    const int first = threadIdx.x * 32;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        uint16_t kb[8];
        load_bits8(kb, keys, first + c * 8, size);
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int idx = first + c * 8 + k;
            // padding up to the thread's 32 items: smallest rank, behind every real item (stable)
            it[c * 8 + k] = (idx < size ? sort_rank(kb[k]) << 16 : 0u) | static_cast<uint32_t>(idx);
        }
    }
}

// IDENTITY: values[i] == i on entry (as softmax_logits leaves them), so the
// sorted payload is the original position itself and no gather is needed.
template <bool IDENTITY>
__device__ __forceinline__ void sort_lds_dev(uint16_t* keys, int* values, int size, SamplerLds& lds, SortLds& buf)
{
    const int first = threadIdx.x * 32;
    const bool active = first < size; // threads beyond the (padded) input own nothing
    uint32_t it[32];
    if (active)
        sort_load_items(it, keys, size);
    sort_passes<32>(it, active, lds, buf);
    if (active) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            uint16_t kb[8];
#pragma unroll
            for (int k = 0; k < 8; ++k)
                kb[k] = sort_key_of_rank(it[c * 8 + k] >> 16);
            store_half8(keys, first + c * 8, size, kb);
        }
    }
    if (IDENTITY) {
        if (active) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                int vb[8];
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    vb[k] = static_cast<int>(it[c * 8 + k] & 0xFFFFu);
                store_int8(values, first + c * 8, size, vb);
            }
        }
        __syncthreads();
        return;
    }
    // payloads: stage the input values in LDS (every thread has read its items back), gather by position
    __syncthreads();
    if (active) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            int vb[8];
            load_int8(vb, values, first + c * 8, size);
#pragma unroll
            for (int k = 0; k < 8; ++k)
                buf.item[sort_slot(first + c * 8 + k)] = static_cast<uint32_t>(vb[k]);
        }
    }
    __syncthreads();
    if (active) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            int vb[8];
#pragma unroll
            for (int k = 0; k < 8; ++k)
                vb[k] = static_cast<int>(buf.item[sort_slot(static_cast<int>(it[c * 8 + k] & 0xFFFFu))]);
            store_int8(values, first + c * 8, size, vb);
        }
    }
    __syncthreads(); // the sorted arrays are visible to the whole workgroup
}

// ---- the head of the sorted order only ------------------------------------------------
// Sampler.Sample (src/Sampler.cs:56-66) reads the sorted probabilities only up to the first
// position whose cumulative sum reaches coin * topP < topP.  When the largest probabilities
// alone add up to more than topP, sorting them is enough: the head of a stable sort does not
// depend on the tail, and neither do the prefix sums over it.
//
// The keys must be probabilities (fp16 in [0, 1]).  Each is put in a bucket by how many
// binades it lies below the largest one (subnormals included: most of a 32000-entry
// distribution is subnormal in fp16); the exact mass of every bucket (integers in units
// of 2^-24, the smallest fp16 subnormal) tells how many buckets are needed to reach `need`;
// their items are compacted in input order, sorted C <= 16 per thread and written to the head
// of keys / values (values[i] == i on entry).  Returns the length n of that head, whose exact
// sum is at least `need`, or 0 when it did nothing (no such head within 15 binades and half
// the buffer, or keys that are no probabilities): then the caller sorts everything.
template <int C>
__device__ __noinline__ void sort_head_finish(uint16_t* keys, int* values, int n, SamplerLds* lds, SortLds* buf)
{
    const int first = threadIdx.x * C;
    const bool active = first < n;
    uint32_t it[C];
#pragma unroll
    for (int k = 0; k < C; ++k) {
        const int p = first + k;
        it[k] = (active && p < n) ? buf->item[sort_slot(p)] : static_cast<uint32_t>(p & 0xFFFF);
    }
    __syncthreads(); // the compacted items are in registers before the buffer turns into counters
    sort_passes<C>(it, active, *lds, *buf);
#pragma unroll
    for (int k = 0; k < C; ++k) {
        const int p = first + k;
        if (active && p < n) {
            keys[p] = sort_key_of_rank(it[k] >> 16);
            values[p] = static_cast<int>(it[k] & 0xFFFFu);
        }
    }
    __syncthreads();
}

// Binade of a non-negative fp16 key: the exponent field for normal numbers, continued downwards
// through the subnormals by the position of the leading mantissa bit (zero: below all of them).
__device__ __forceinline__ int sort_head_binade(uint32_t rank)
{
    const int e = static_cast<int>((rank >> 10) & 31u);
    const uint32_t mant = rank & 0x3FFu;
    return e ? e : (mant ? 22 - __clz(mant) : -10); // mant in [2^k, 2^(k+1)): k - 9
}

__device__ __forceinline__ int sort_head_bucket(uint32_t item, int emax)
{
    const uint32_t r = item >> 16;
    const int below = emax - sort_head_binade(r);
    return (r < 0x8000u || below > 15) ? 15 : below; // padding and negative keys: last bucket
}

__device__ __noinline__ int sort_head_call(uint16_t* keys, int* values, int size, float need, SamplerLds* lds_,
                                           SortLds* buf_)
{
    SamplerLds& lds = *lds_;
    SortLds& buf = *buf_;
    const bool active = static_cast<int>(threadIdx.x) * 32 < size;
    uint32_t it[32];
    int top = 0;
    if (active) {
        sort_load_items(it, keys, size);
#pragma unroll
        for (int k = 0; k < 32; ++k)
            top = max(top, static_cast<int>(it[k] >> 16));
    }
    top = 0xFFFF - samp_block_min(0xFFFF - top, lds.redi);
    if (top > 0xBC00 || top < 0x8000) // something above 1.0 (or NaN), or nothing positive
        return 0;
    const int emax = sort_head_binade(static_cast<uint32_t>(top));
    uint32_t* mass = buf.item; // [16][kSampBlock], own words only
#pragma unroll
    for (int d = 0; d < 16; ++d)
        mass[d * kSampBlock + threadIdx.x] = 0u;
    if (active) {
#pragma unroll
        for (int k = 0; k < 32; ++k) {
            const uint32_t r = it[k] >> 16;
            const uint32_t e = (r >> 10) & 31u, mant = r & 0x3FFu;
            uint32_t units = e ? (0x400u | mant) << (e - 1) : mant; // value * 2^24, exact
            if (r < 0x8000u)
                units = 0u;
            __hip_atomic_fetch_add(&mass[sort_head_bucket(it[k], emax) * kSampBlock + threadIdx.x], units,
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
    }
    __syncthreads();
    {
        // wavefront d adds up bucket d: 64 lanes x 16 consecutive words
        const u32x4* mine = reinterpret_cast<const u32x4*>(mass + threadIdx.x * 16);
        uint32_t sum = 0;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const u32x4 m4 = mine[q];
            sum += m4[0] + m4[1] + m4[2] + m4[3];
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1)
            sum += __shfl_xor(sum, off, 64);
        if ((threadIdx.x & 63) == 0)
            lds.redi[threadIdx.x >> 6] = static_cast<int>(sum); // the whole vocabulary stays below 2^31 units
    }
    __syncthreads();
    const float need_units = ceilf(need * 16777216.0f);
    int last_bucket = -1;
    {
        float cum = 0.0f; // sums of integers below 2^25 in fp32 lose at most a unit or two: `need` carries a margin
#pragma unroll
        for (int d = 0; d < 15; ++d) {
            cum += static_cast<float>(lds.redi[d]);
            if (last_bucket < 0 && cum >= need_units)
                last_bucket = d;
        }
    }
    __syncthreads();
    if (last_bucket < 0)
        return 0;
    int keep = 0;
    if (active) {
#pragma unroll
        for (int k = 0; k < 32; ++k)
            keep += sort_head_bucket(it[k], emax) <= last_bucket;
    }
    const int before = samp_block_exclusive_scan<int>(keep, lds.redi);
    if (threadIdx.x == kSampBlock - 1)
        lds.redi[0] = before + keep;
    __syncthreads();
    const int n = lds.redi[0];
    __syncthreads();
    if (n > kSortLdsThreads * 16)
        return 0;
    if (active) {
        int at = before;
#pragma unroll
        for (int k = 0; k < 32; ++k)
            if (sort_head_bucket(it[k], emax) <= last_bucket)
                buf.item[sort_slot(at++)] = it[k];
    }
    __syncthreads();
    if (n <= kSortLdsThreads)
        sort_head_finish<1>(keys, values, n, lds_, buf_);
    else if (n <= kSortLdsThreads * 2)
        sort_head_finish<2>(keys, values, n, lds_, buf_);
    else if (n <= kSortLdsThreads * 4)
        sort_head_finish<4>(keys, values, n, lds_, buf_);
    else if (n <= kSortLdsThreads * 8)
        sort_head_finish<8>(keys, values, n, lds_, buf_);
    else
        sort_head_finish<16>(keys, values, n, lds_, buf_);
    return n;
}

// ---- cumulative_sum (native/cumulative_sum_kernel.cu:8-26) ---------------------------
// Inclusive prefix sums in fp32, each rounded to fp16, in place.  A thread sums
// its 8*CH consecutive values in order, the thread totals are scanned in thread
// order, prefix + running sum is stored.
template <int CH>
__device__ __forceinline__ void cumulative_sum_dev(uint16_t* values, int size, SamplerLds& lds)
{
    const int first = threadIdx.x * 8 * CH;
    float f[CH][8];
    float run = 0.0f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int base = first + c * 8;
        if (base < size) {
            load_half8(f[c], values, base, size, 0.0f);
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                run += f[c][k];
                f[c][k] = run;
            }
        }
    }
    const float before = samp_block_exclusive_scan<float>(run, lds.redf);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int base = first + c * 8;
        if (base < size) {
            uint16_t b[8];
#pragma unroll
            for (int k = 0; k < 8; ++k)
                b[k] = float_to_half_bits(before + f[c][k]);
            store_half8(values, base, size, b);
        }
    }
}

// ---- sample_top_p (native/sample_top_p_kernel.cu:8-21) -------------------------------
// The value at the first position whose entry reaches the threshold (the last
// position if none does) of `indices`; returned in every thread.
template <int CH>
__device__ __forceinline__ int sample_top_p_dev(const uint16_t* logits, const int* indices, int size, float threshold,
                                                SamplerLds& lds)
{
    int best = size - 1;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int base = (threadIdx.x + c * kSampBlock) * 8;
        if (base < size) {
            float f[8];
            load_half8(f, logits, base, size, -INFINITY);
#pragma unroll
            for (int k = 7; k >= 0; --k)
                if (base + k < size && f[k] >= threshold && base + k < best)
                    best = base + k;
        }
    }
    best = samp_block_min(best, lds.redi);
    return indices[best];
}

// Uniform number in [0, 1) for position `pos` of the stream `seed`: splitmix64
// of seed + pos, top 24 bits.  (The reference draws from an unseeded
// System.Random, src/Sampler.cs:24,42.)
__host__ __device__ inline float sampler_coin(unsigned long long seed, int pos)
{
    unsigned long long z = seed + 0x9E3779B97F4A7C15ull * static_cast<unsigned long long>(pos + 1);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return static_cast<float>(z >> 40) * (1.0f / 16777216.0f);
}

// Sampler.Sample's stochastic branch (src/Sampler.cs:48-67) on one workgroup.
// LDS_SORT: size <= kSortLdsItems and `buf` is there; otherwise the sort runs
// through the second global buffer (keys2, values2).
// Each phase is a call, not inlined: inlined together the phases' register arrays
// overlap in the allocator's view and two hundred registers spill.
template <int CH>
__device__ __noinline__ void softmax_logits_call(uint16_t* logits, int size, float temperature, int* indices,
                                                 SamplerLds* lds)
{
    softmax_logits_dev<CH>(logits, size, temperature, indices, *lds);
}
// TAG: one copy per calling kernel.  Shared between two kernels of a translation unit the same code
// was compiled with 4.4 KB of scratch memory per lane (against 0.4 KB), and a kernel with that
// much scratch costs over a millisecond per launch.
template <bool TAG>
__device__ __noinline__ void sort_lds_identity_call(uint16_t* keys, int* values, int size, SamplerLds* lds, SortLds* buf)
{
    sort_lds_dev<true>(keys, values, size, *lds, *buf);
}
template <int CH>
__device__ __noinline__ void sort_call(uint16_t* keys, int* values, int size, uint16_t* keys2, int* values2,
                                       SamplerLds* lds)
{
    sort_dev<CH>(keys, values, size, keys2, values2, *lds);
}
template <int CH>
__device__ __noinline__ void cumulative_sum_call(uint16_t* values, int size, SamplerLds* lds)
{
    cumulative_sum_dev<CH>(values, size, *lds);
}

// HEAD_ONLY: the caller needs the token alone, not the sorted arrays and their prefix sums: when a
// short head of the sorted order holds more than top_p of the mass, only that head is sorted and
// summed (the token is the same; what logits / indices hold afterwards is not).
template <int CH, bool LDS_SORT, bool HEAD_ONLY = false>
__device__ __forceinline__ int sample_dev(uint16_t* logits, int* indices, int size, float temperature, float top_p,
                                          float coin, uint16_t* keys2, int* values2, SamplerLds& lds, SortLds* buf)
{
    softmax_logits_call<CH>(logits, size, temperature, indices, &lds);
    __syncthreads();
    float threshold = coin;
    int n = size;
    if (!(top_p <= 0.0f || top_p >= 1.0f)) {
        // The prefix sums are rounded to fp16 (2^-11) after a blocked fp32 summation (a few 2^-24):
        // a head whose exact mass is 1.004 top_p reaches top_p > coin * top_p in that arithmetic too.
        int head = 0;
        if (LDS_SORT && HEAD_ONLY)
            head = sort_head_call(logits, indices, size, top_p * 1.004f, &lds, buf);
        if (head)
            n = head;
        else if (LDS_SORT)
            sort_lds_identity_call<HEAD_ONLY>(logits, indices, size, &lds, buf); // indices are 0..size-1 here
        else
            sort_call<CH>(logits, indices, size, keys2, values2, &lds);
        threshold = coin * top_p;
    }
    cumulative_sum_call<CH>(logits, n, &lds);
    __syncthreads();
    return sample_top_p_dev<CH>(logits, indices, n, threshold, lds);
}

} // namespace l2

// fp16 mat-vecs of the decode path: the classifier GEMV, the attention score
// mat-vec over the key cache and the probability-weighted sum over the value
// cache.  Replaces native/mat_vec_kernel.cu:14-81 and native/vec_mat_kernel.cu.
//
// All three are HBM-bound streams of an fp16 matrix read exactly once with
// 16-byte loads; fp32 accumulation; fp16 results.
#include "common.hpp"

namespace l2 {

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;

// ------------------------------------------------------------------ classifier
// One wavefront per R consecutive output rows; input staged once per workgroup
// in LDS; lane l of a wavefront reads 16-byte chunks l, l+64, ... of each row.
template <int R, int U>
__global__ __launch_bounds__(kThreads) void f16_matvec_kernel(uint16_t* out, const uint16_t* x,
                                                              const uint16_t* M, int K, int N)
{
    extern __shared__ u32x4 xs[];
    const int nchunks = K >> 3;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n0 = (blockIdx.x * kWaves + wave) * R;
    const u32x4* rowp[R];
#pragma unroll
    for (int r = 0; r < R; ++r)
        rowp[r] = reinterpret_cast<const u32x4*>(M + static_cast<size_t>(n0 + r < N ? n0 + r : N - 1) * K);

    // first block of matrix loads goes out before the input is staged
    u32x4 m[R][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int c = lane + 64 * u;
#pragma unroll
        for (int r = 0; r < R; ++r)
            m[r][u] = c < nchunks ? __builtin_nontemporal_load(rowp[r] + c) : u32x4{0u, 0u, 0u, 0u};
    }
    for (int e = threadIdx.x; e < nchunks; e += kThreads)
        xs[e] = reinterpret_cast<const u32x4*>(x)[e];
    __syncthreads();

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r)
        acc[r] = 0.0f;

    for (int c0 = 0; c0 < nchunks; c0 += 64 * U) {
        u32x4 nxt[R][U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int c = c0 + 64 * U + lane + 64 * u;
#pragma unroll
            for (int r = 0; r < R; ++r)
                nxt[r][u] = c < nchunks ? __builtin_nontemporal_load(rowp[r] + c) : u32x4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int c = c0 + lane + 64 * u;
            if (c < nchunks) {
                const u32x4 xv = xs[c];
#pragma unroll
                for (int r = 0; r < R; ++r) {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        acc[r] = dot2(m[r][u][i], xv[i], acc[r]);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int r = 0; r < R; ++r)
                m[r][u] = nxt[r][u];
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const float s = wave_sum(acc[r]);
        if (lane == r && n0 + r < N)
            out[n0 + r] = float_to_half_bits(s);
    }
}

// ------------------------------------------------------------- attention scores
// 16 lanes per (timestep, head): each lane holds 16 bytes of q per CH chunk
// and dots it with 16 bytes of the key row; a wavefront covers 4 heads of one
// timestep per step (1 KiB contiguous when heads are packed), unrolled over U
// timesteps.  Requires rows % 8 == 0, rows <= 128*CH and 16-byte aligned strides.
template <int CH, int U>
__global__ __launch_bounds__(kThreads) void scores_kernel(uint16_t* out, const uint16_t* q, const uint16_t* Km,
                                                          int rows, int cols, int v_stride, int m_col_stride,
                                                          int m_row_stride, int o_stride, float alpha,
                                                          int n_heads, int t_per_wg)
{
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int l16 = lane & 15;
    const int h = blockIdx.y * 4 + (lane >> 4);
    const bool head_ok = h < n_heads;
    const int hh = head_ok ? h : n_heads - 1;
    const int rchunks = rows >> 3;

    u32x4 qv[CH];
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
        const int ci = l16 + 16 * ch;
        qv[ch] = ci < rchunks ? *reinterpret_cast<const u32x4*>(q + static_cast<size_t>(hh) * v_stride + ci * 8)
                              : u32x4{0u, 0u, 0u, 0u};
    }
    const uint16_t* kbase = Km + static_cast<size_t>(hh) * m_col_stride;
    const int t_begin = blockIdx.x * t_per_wg;
    const int t_end = min(cols, t_begin + t_per_wg);

    for (int t0 = t_begin + wave * U; t0 < t_end; t0 += kWaves * U) {
        u32x4 kv[U][CH];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int t = t0 + u;
#pragma unroll
            for (int ch = 0; ch < CH; ++ch) {
                const int ci = l16 + 16 * ch;
                kv[u][ch] = (t < t_end && ci < rchunks)
                                ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(
                                      kbase + static_cast<size_t>(t) * m_row_stride + ci * 8))
                                : u32x4{0u, 0u, 0u, 0u};
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float acc = 0.0f;
#pragma unroll
            for (int ch = 0; ch < CH; ++ch)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    acc = dot2(kv[u][ch][i], qv[ch][i], acc);
            acc = row16_sum(acc);
            const int t = t0 + u;
            if (l16 == 0 && head_ok && t < t_end)
                out[static_cast<size_t>(h) * o_stride + t] = float_to_half_bits(acc * alpha);
        }
    }
}

// Any shape / stride: one wavefront per (timestep, head), 2-byte loads.
__global__ __launch_bounds__(kThreads) void scores_generic_kernel(uint16_t* out, const uint16_t* q,
                                                                  const uint16_t* Km, int rows, int cols,
                                                                  int v_stride, int m_col_stride, int m_row_stride,
                                                                  int o_stride, float alpha)
{
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * kWaves + (threadIdx.x >> 6);
    const int h = blockIdx.y;
    const int tt = t < cols ? t : cols - 1;
    float acc = 0.0f;
    for (int r = lane; r < rows; r += 64)
        acc += half_bits_to_float(Km[static_cast<size_t>(tt) * m_row_stride + static_cast<size_t>(h) * m_col_stride + r]) *
               half_bits_to_float(q[static_cast<size_t>(h) * v_stride + r]);
    acc = wave_sum(acc);
    if (lane == 0 && t < cols)
        out[static_cast<size_t>(h) * o_stride + t] = float_to_half_bits(acc * alpha);
}

// ------------------------------------------------------- weighted sum of values
// Lane owns 8 consecutive outputs (one 16-byte chunk of a value row); 16 lanes
// per head, 4 heads per wavefront; blockIdx.z selects a 128-wide block of r.
// The sequence is split over blockIdx.x; the 4 wavefronts of a workgroup take
// timesteps round-robin and are combined through LDS.  With more than one
// split, fp32 partials go to `partials[split][n_heads*rows]` and
// vecmat_reduce_kernel adds them in a fixed order (deterministic).
template <int U>
__global__ __launch_bounds__(kThreads) void vecmat_kernel(uint16_t* out, float* partials, const uint16_t* att,
                                                          const uint16_t* V, int rows, int cols, int m_col_stride,
                                                          int o_stride, int m_row_stride, int n_heads, int t_per_wg)
{
    __shared__ float red[kWaves][64][8 + 1];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int l16 = lane & 15;
    const int h = blockIdx.y * 4 + (lane >> 4);
    const int hh = h < n_heads ? h : n_heads - 1;
    const int r0 = blockIdx.z * 128 + l16 * 8;
    const bool r_ok = r0 < rows; // rows % 8 == 0
    const uint16_t* vbase = V + static_cast<size_t>(hh) * m_col_stride + (r_ok ? r0 : 0);
    const uint16_t* abase = att + static_cast<size_t>(hh) * cols;
    const int t_begin = blockIdx.x * t_per_wg;
    const int t_end = min(cols, t_begin + t_per_wg);

    float acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
        acc[i] = 0.0f;

    for (int t0 = t_begin + wave * U; t0 < t_end; t0 += kWaves * U) {
        u32x4 vv[U];
        float a[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int t = t0 + u;
            const bool ok = t < t_end;
            vv[u] = ok ? __builtin_nontemporal_load(
                             reinterpret_cast<const u32x4*>(vbase + static_cast<size_t>(t) * m_row_stride))
                       : u32x4{0u, 0u, 0u, 0u};
            a[u] = ok ? half_bits_to_float(abase[t]) : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const h2_t p = as_h2(vv[u][i]);
                acc[2 * i] += a[u] * static_cast<float>(p[0]);
                acc[2 * i + 1] += a[u] * static_cast<float>(p[1]);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
        red[wave][lane][i] = acc[i];
    __syncthreads();
    // 512 outputs per workgroup: thread -> (lane slot, element) pairs
    for (int o = threadIdx.x; o < 512; o += kThreads) {
        const int sl = o >> 3, i = o & 7;
        const float s = (red[0][sl][i] + red[1][sl][i]) + (red[2][sl][i] + red[3][sl][i]);
        const int ho = blockIdx.y * 4 + (sl >> 4);
        const int ro = blockIdx.z * 128 + (sl & 15) * 8 + i;
        if (ho < n_heads && ro < rows) {
            if (partials)
                partials[(static_cast<size_t>(blockIdx.x) * n_heads + ho) * rows + ro] = s;
            else
                out[static_cast<size_t>(ho) * o_stride + ro] = float_to_half_bits(s);
        }
    }
}

// Short sequences of 128-wide heads (cols <= 512): one workgroup of 16 wavefronts per head and no
// partial sums in memory.  16 lanes share a timestep (16 bytes of its value row each), the 64 groups
// take the timesteps round-robin, every load is issued before the first use, and the groups are
// combined in a fixed order (within the wavefront by shuffles, across wavefronts through LDS).
constexpr int kHeadVecMatCols = 512;
__global__ __launch_bounds__(1024) void vecmat_head_kernel(uint16_t* out, const uint16_t* att, const uint16_t* V,
                                                           int cols, int m_col_stride, int o_stride,
                                                           int m_row_stride)
{
    constexpr int PASSES = kHeadVecMatCols / 64;
    __shared__ float red[16][128];
    const int h = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l16 = lane & 15, grp = wave * 4 + (lane >> 4);
    const uint16_t* vbase = V + static_cast<size_t>(h) * m_col_stride + l16 * 8;
    const uint16_t* abase = att + static_cast<size_t>(h) * cols;
    u32x4 vv[PASSES];
    float a[PASSES];
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
        const int t = i * 64 + grp;
        const bool ok = t < cols;
        vv[i] = ok ? __builtin_nontemporal_load(
                         reinterpret_cast<const u32x4*>(vbase + static_cast<size_t>(t) * m_row_stride))
                   : u32x4{0u, 0u, 0u, 0u};
        a[i] = ok ? half_bits_to_float(abase[t]) : 0.0f;
    }
    float acc[8];
#pragma unroll
    for (int k = 0; k < 8; ++k)
        acc[k] = 0.0f;
#pragma unroll
    for (int i = 0; i < PASSES; ++i) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const h2_t p = as_h2(vv[i][k]);
            acc[2 * k] += a[i] * static_cast<float>(p[0]);
            acc[2 * k + 1] += a[i] * static_cast<float>(p[1]);
        }
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        acc[k] += __shfl_xor(acc[k], 16, 64);
        acc[k] += __shfl_xor(acc[k], 32, 64);
    }
    if (lane < 16) {
#pragma unroll
        for (int k = 0; k < 8; ++k)
            red[wave][l16 * 8 + k] = acc[k];
    }
    __syncthreads();
    if (threadIdx.x < 128) {
        float s = 0.0f;
#pragma unroll
        for (int w = 0; w < 16; ++w)
            s += red[w][threadIdx.x];
        out[static_cast<size_t>(h) * o_stride + threadIdx.x] = float_to_half_bits(s);
    }
}

// One workgroup adds up 64 consecutive outputs: wavefront w takes the splits w, w + 16, ... (one
// coalesced 256-byte row of partials each, independent loads), then the 16 wavefront sums are
// added in wavefront order (fixed association: deterministic).
constexpr int kReduceWaves = 16;
__global__ __launch_bounds__(kReduceWaves * 64) void vecmat_reduce_kernel(uint16_t* out, const float* partials,
                                                                          int rows, int o_stride, int n_heads,
                                                                          int splits)
{
    __shared__ float red[kReduceWaves][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int total = n_heads * rows;
    const int i = blockIdx.x * 64 + lane;
    float s = 0.0f;
    if (i < total) {
#pragma unroll 8
        for (int k = wave; k < splits; k += kReduceWaves)
            s += partials[static_cast<size_t>(k) * total + i];
    }
    red[wave][lane] = s;
    __syncthreads();
    if (wave == 0 && i < total) {
        float t = 0.0f;
#pragma unroll
        for (int w = 0; w < kReduceWaves; ++w)
            t += red[w][lane];
        out[static_cast<size_t>(i / rows) * o_stride + (i % rows)] = float_to_half_bits(t);
    }
}

// Any shape / stride: one thread per output element.
__global__ void vecmat_generic_kernel(uint16_t* out, const uint16_t* att, const uint16_t* V, int rows, int cols,
                                      int m_col_stride, int o_stride, int m_row_stride, int n_heads)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_heads * rows)
        return;
    const int h = i / rows, r = i % rows;
    float s = 0.0f;
    for (int t = 0; t < cols; ++t)
        s += half_bits_to_float(att[static_cast<size_t>(h) * cols + t]) *
             half_bits_to_float(V[static_cast<size_t>(t) * m_row_stride + static_cast<size_t>(h) * m_col_stride + r]);
    out[static_cast<size_t>(h) * o_stride + r] = float_to_half_bits(s);
}

// Workgroups wanted to keep 256 CUs busy with a few wavefronts each.
constexpr int kTargetWorkgroups = 1024;

static int pick_t_per_wg(int cols, int other_dim_wgs, int min_t)
{
    int along_t = ceil_div(kTargetWorkgroups, other_dim_wgs);
    int t = ceil_div(cols, along_t);
    if (t < min_t)
        t = min_t;
    return ceil_div(t, 4) * 4;
}

} // namespace l2

using namespace l2;

// ---------------------------------------------------------------- static scratch
// llama2_vec_mat_static allocates nothing: the fp32 partial sums of a sequence split over
// workgroups live in this file-scope device array (one copy per GPU, at its own address, held
// until the process ends).  In host code the array's name is only a stand-in; its device address
// is asked for once per device, at llama2_init with that device current, and every later use
// goes through that pointer.  Nothing in the array has to start at zero: the first launch writes
// every partial sum the second one reads.
static __device__ __align__(256) float scratch[LLAMA2_STATIC_VEC_MAT_BYTES / sizeof(float)];

namespace l2 {

constexpr int kMaxStaticDevices = 64;
static float* g_static_partials[kMaxStaticDevices] = {};

int resolve_vec_mat_static_scratch(int device)
{
    if (device < 0 || device >= kMaxStaticDevices)
        return fail(LLAMA2_ERR_INVALID_ARGUMENT, "llama2_init: device %d beyond the %d the static scratch tracks", device,
                    kMaxStaticDevices);
    void* ptr = nullptr;
    L2_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr)
        return fail(LLAMA2_ERR_NO_DEVICE, "llama2_init: the static scratch has no address on device %d", device);
    g_static_partials[device] = static_cast<float*>(ptr);
    return LLAMA2_OK;
}

// VecMat.Forward; `static_partials`: the caller's scratch for the partial sums (LLAMA2_STATIC_VEC_MAT_BYTES of
// it), or null: the library's growing buffer.
static int vec_mat(const char* fn, llama2_half* output, const llama2_half* vector, const llama2_half* matrix, int rows,
                   int cols, int m_col_stride, int o_stride, int m_row_stride, int n_heads, float* static_partials)
{
    L2_CHECK(output && vector && matrix, "%s: null pointer", fn);
    L2_CHECK(rows > 0 && cols > 0 && n_heads > 0, "%s: rows=%d cols=%d n_heads=%d must be positive", fn, rows, cols,
             n_heads);
    L2_CHECK(m_col_stride >= 0 && m_row_stride >= 0 && o_stride >= 0, "%s: negative stride", fn);
    const bool fast =
        rows % 8 == 0 && m_col_stride % 8 == 0 && m_row_stride % 8 == 0 && aligned(matrix, 16);
    if (fast && rows == 128 && cols <= kHeadVecMatCols) {
        hipLaunchKernelGGL(vecmat_head_kernel, dim3(n_heads), dim3(1024), 0, ctx().stream, output, vector, matrix, cols,
                           m_col_stride, o_stride, m_row_stride);
        L2_LAUNCH_CHECK(fn);
    } else if (fast) {
        const int hq = ceil_div(n_heads, 4), rb = ceil_div(rows, 128);
        const int t_per_wg = pick_t_per_wg(cols, hq * rb, 32);
        const int splits = ceil_div(cols, t_per_wg);
        const dim3 grid(splits, hq, rb);
        float* partials = nullptr;
        if (splits > 1) {
            const size_t bytes = static_cast<size_t>(splits) * n_heads * rows * sizeof(float);
            if (static_partials) {
                if (bytes > LLAMA2_STATIC_VEC_MAT_BYTES)
                    return fail(LLAMA2_ERR_UNSUPPORTED,
                                "%s: %d sequence blocks x %d heads x %d rows of partial sums (%zu bytes) exceed the static "
                                "scratch of %d bytes; use llama2_vec_mat", fn, splits, n_heads, rows, bytes,
                                LLAMA2_STATIC_VEC_MAT_BYTES);
                partials = static_partials;
            } else {
                if (int rc = ensure_attn_partials(bytes))
                    return rc;
                partials = ctx().attn_partials;
            }
        }
        hipLaunchKernelGGL((vecmat_kernel<4>), grid, dim3(kThreads), 0, ctx().stream, output, partials, vector,
                           matrix, rows, cols, m_col_stride, o_stride, m_row_stride, n_heads, t_per_wg);
        L2_LAUNCH_CHECK(fn);
        if (splits > 1) {
            hipLaunchKernelGGL(vecmat_reduce_kernel, dim3(ceil_div(n_heads * rows, 64)), dim3(kReduceWaves * 64), 0,
                               ctx().stream, output, partials, rows, o_stride, n_heads, splits);
            L2_LAUNCH_CHECK("vecmat_reduce_kernel");
        }
    } else {
        hipLaunchKernelGGL(vecmat_generic_kernel, dim3(ceil_div(n_heads * rows, 256)), dim3(256), 0, ctx().stream,
                           output, vector, matrix, rows, cols, m_col_stride, o_stride, m_row_stride, n_heads);
        L2_LAUNCH_CHECK(fn);
    }
    return LLAMA2_OK;
}

} // namespace l2

extern "C" {

int llama2_mat_vec(llama2_half* output, const llama2_half* vector, const llama2_half* matrix, int rows, int cols)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_mat_vec";
    L2_CHECK(output && vector && matrix, "%s: null pointer", fn);
    L2_CHECK(rows > 0 && cols > 0, "%s: rows=%d cols=%d must be positive", fn, rows, cols);
    L2_CHECK(rows % 8 == 0, "%s: rows=%d must be a multiple of 8 (16-byte loads, as in the reference)", fn, rows);
    L2_CHECK(aligned(vector, 16) && aligned(matrix, 16), "%s: vector and matrix must be 16-byte aligned", fn);
    if (static_cast<size_t>(rows) * 2 > 64 * 1024)
        return fail(LLAMA2_ERR_UNSUPPORTED, "%s: rows=%d does not fit the 64 KiB LDS staging buffer", fn, rows);
    L2_CHECK(!overlap(output, size_t(cols) * 2, vector, size_t(rows) * 2), "%s: output overlaps vector", fn);
    constexpr int R = 2, U = 2;
    hipLaunchKernelGGL((f16_matvec_kernel<R, U>), dim3(ceil_div(cols, kWaves * R)), dim3(kThreads),
                       static_cast<size_t>(rows) * 2, ctx().stream, output, vector, matrix, rows, cols);
    L2_LAUNCH_CHECK(fn);
    return LLAMA2_OK;
}

int llama2_mat_vec_strided(llama2_half* output, const llama2_half* vector, const llama2_half* matrix, int rows,
                           int cols, int v_stride, int m_col_stride, int m_row_stride, int o_stride, float alpha,
                           int n_heads)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_mat_vec_strided";
    L2_CHECK(output && vector && matrix, "%s: null pointer", fn);
    L2_CHECK(rows > 0 && cols > 0 && n_heads > 0, "%s: rows=%d cols=%d n_heads=%d must be positive", fn, rows, cols,
             n_heads);
    L2_CHECK(v_stride >= 0 && m_col_stride >= 0 && m_row_stride >= 0 && o_stride >= 0, "%s: negative stride", fn);
    const bool fast = rows % 8 == 0 && rows <= 256 && v_stride % 8 == 0 && m_col_stride % 8 == 0 &&
                      m_row_stride % 8 == 0 && aligned(vector, 16) && aligned(matrix, 16);
    if (fast) {
        const int hq = ceil_div(n_heads, 4);
        const int t_per_wg = pick_t_per_wg(cols, hq, 16);
        const dim3 grid(ceil_div(cols, t_per_wg), hq);
        if (rows <= 128)
            hipLaunchKernelGGL((scores_kernel<1, 4>), grid, dim3(kThreads), 0, ctx().stream, output, vector, matrix,
                               rows, cols, v_stride, m_col_stride, m_row_stride, o_stride, alpha, n_heads, t_per_wg);
        else
            hipLaunchKernelGGL((scores_kernel<2, 2>), grid, dim3(kThreads), 0, ctx().stream, output, vector, matrix,
                               rows, cols, v_stride, m_col_stride, m_row_stride, o_stride, alpha, n_heads, t_per_wg);
    } else {
        hipLaunchKernelGGL(scores_generic_kernel, dim3(ceil_div(cols, kWaves), n_heads), dim3(kThreads), 0,
                           ctx().stream, output, vector, matrix, rows, cols, v_stride, m_col_stride, m_row_stride,
                           o_stride, alpha);
    }
    L2_LAUNCH_CHECK(fn);
    return LLAMA2_OK;
}

int llama2_vec_mat(llama2_half* output, const llama2_half* vector, const llama2_half* matrix, int rows, int cols,
                   int m_col_stride, int o_stride, int m_row_stride, int n_heads)
{
    L2_REQUIRE_INIT();
    return vec_mat("llama2_vec_mat", output, vector, matrix, rows, cols, m_col_stride, o_stride, m_row_stride, n_heads,
                   nullptr);
}

int llama2_vec_mat_static(llama2_half* output, const llama2_half* vector, const llama2_half* matrix, int rows, int cols,
                          int m_col_stride, int o_stride, int m_row_stride, int n_heads)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_vec_mat_static";
    const int device = ctx().device;
    float* sp = device >= 0 && device < kMaxStaticDevices ? g_static_partials[device] : nullptr;
    if (!sp)
        return fail(LLAMA2_ERR_NOT_INITIALIZED, "%s: the static scratch of device %d was not resolved at llama2_init", fn,
                    device);
    return vec_mat(fn, output, vector, matrix, rows, cols, m_col_stride, o_stride, m_row_stride, n_heads, sp);
}

} // extern "C"

// The converter's repack step on the GPU (src/ModelConverter.cs:196-328): AWQ
// "GEMM" tensors [K][N/8] -> the output-major int4 layout [N][K/8] the decode
// kernels read, scales [K/128][N] -> [N][K/128].  Pure byte shuffling, HBM-bound:
// every input word is read once and every output word written once, both in
// 128-byte runs, with the nibble transpose done in registers and the word
// transpose in LDS.
#include "common.hpp"

namespace l2 {

// Nibble i of an input word holds column 8c + orderMap[i], orderMap = {0,2,4,6,1,3,5,7}
// (src/ModelConverter.cs:19, 289-293): column j of the word sits in nibble kNibbleOf[j].
__device__ __forceinline__ int nibble_of_column(int j) { return (j & 1) ? 4 + (j >> 1) : (j >> 1); }

constexpr int kTile = 32; // words per tile side: 32 x 32 cells of 8 x 8 nibbles

// height % 8 == 0.  One workgroup transposes 256 input rows x 32 input words
// (= 256 output rows x 32 output words).
__global__ __launch_bounds__(256) void repack_qdata_tile_kernel(uint32_t* out, const uint32_t* in, int H8, int W8)
{
    __shared__ uint32_t tile[8 * kTile * kTile]; // [8 * nwl + j][kbl ^ nwl]
    const int kb0 = blockIdx.x * kTile, nw0 = blockIdx.y * kTile;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int c = threadIdx.x + 256 * r;
        const int nwl = c & 31, kbl = c >> 5;
        const int kb = kb0 + kbl, nw = nw0 + nwl;
        uint32_t w[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
            w[i] = (kb < H8 && nw < W8) ? __builtin_nontemporal_load(in + (static_cast<size_t>(kb) * 8 + i) * W8 + nw)
                                        : 0u;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int sh = 4 * nibble_of_column(j);
            uint32_t o = 0;
#pragma unroll
            for (int i = 0; i < 8; ++i)
                o |= ((w[i] >> sh) & 0xFu) << (4 * i);
            tile[(8 * nwl + j) * kTile + (kbl ^ nwl)] = o;
        }
    }
    __syncthreads();
    const int kbl = threadIdx.x & 31;
#pragma unroll
    for (int r = 0; r < 32; ++r) {
        const int nl = (threadIdx.x >> 5) + 8 * r; // output row within the tile
        const int n = nw0 * 8 + nl, kb = kb0 + kbl;
        if (n < W8 * 8 && kb < H8)
            __builtin_nontemporal_store(tile[nl * kTile + (kbl ^ (nl >> 3))], out + static_cast<size_t>(n) * H8 + kb);
    }
}

// Any height: one thread per output word.  Element (column x, row y) of the
// column-major intermediate array of the reference has linear index
// L = height * x + y; an output word takes L .. L+7, which runs into the next
// column when height is not a multiple of 8 and reads zero behind the last one
// (src/ModelConverter.cs:283-311).
__global__ __launch_bounds__(256) void repack_qdata_generic_kernel(uint32_t* out, const uint32_t* in, int height,
                                                                   int width, int H8)
{
    const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    const size_t total = static_cast<size_t>(width) * H8;
    if (idx >= total)
        return;
    const int x = static_cast<int>(idx / H8), yb = static_cast<int>(idx % H8);
    const size_t elements = static_cast<size_t>(width) * height;
    const int W8 = width >> 3;
    uint32_t o = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const size_t L = static_cast<size_t>(height) * x + 8 * yb + i;
        if (L < elements) {
            const int col = static_cast<int>(L / height), row = static_cast<int>(L % height);
            const uint32_t w = in[static_cast<size_t>(row) * W8 + (col >> 3)];
            o |= ((w >> (4 * nibble_of_column(col & 7))) & 0xFu) << (4 * i);
        }
    }
    out[idx] = o;
}

// [rows][cols] -> [cols][rows] of 16-bit values, 64 x 64 tiles.
__global__ __launch_bounds__(256) void transpose_u16_kernel(uint16_t* out, const uint16_t* in, int rows, int cols)
{
    __shared__ uint16_t tile[64][66];
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
        const int r = r0 + ty + 4 * k, c = c0 + tx;
        if (r < rows && c < cols)
            tile[ty + 4 * k][tx] = in[static_cast<size_t>(r) * cols + c];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; ++k) {
        const int c = c0 + ty + 4 * k, r = r0 + tx;
        if (r < rows && c < cols)
            out[static_cast<size_t>(c) * rows + r] = tile[tx][ty + 4 * k];
    }
}

// Format.v1 scales (src/ModelConverter.cs:247-262): rows of `in_stride` halfs -> rows of `scales_size` halfs.
__global__ __launch_bounds__(256) void compact_rows_u16_kernel(uint16_t* out, const uint16_t* in, int scales_size,
                                                               int in_stride, size_t total)
{
    const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total)
        return;
    const size_t x = idx / scales_size, y = idx % scales_size;
    out[idx] = in[x * in_stride + y];
}

} // namespace l2

using namespace l2;

extern "C" {

int llama2_repack_qdata(uint32_t* out, const uint32_t* in, int height, int width)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_repack_qdata";
    L2_CHECK(out && in, "%s: null pointer", fn);
    L2_CHECK(height > 0 && width > 0, "%s: height=%d width=%d must be positive", fn, height, width);
    L2_CHECK(width % 8 == 0, "%s: width=%d must be a multiple of 8 (8 columns per input word)", fn, width);
    const int H8 = ceil_div(height, 8), W8 = width / 8;
    const size_t in_bytes = static_cast<size_t>(height) * W8 * 4, out_bytes = static_cast<size_t>(width) * H8 * 4;
    L2_CHECK(!overlap(out, out_bytes, in, in_bytes), "%s: out and in overlap", fn);
    L2_CHECK(static_cast<size_t>(width) * H8 < (static_cast<size_t>(1) << 40), "%s: tensor too large", fn);
    if (height % 8 == 0 && H8 >= 8 && W8 >= 8) {
        hipLaunchKernelGGL(repack_qdata_tile_kernel, dim3(ceil_div(H8, kTile), ceil_div(W8, kTile)), dim3(256), 0,
                           ctx().stream, out, in, H8, W8);
    } else {
        const size_t total = static_cast<size_t>(width) * H8;
        hipLaunchKernelGGL(repack_qdata_generic_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0,
                           ctx().stream, out, in, height, width, H8);
    }
    L2_LAUNCH_CHECK(fn);
    return LLAMA2_OK;
}

int llama2_repack_scales(llama2_half* out, const llama2_half* in, int meta_height, int width)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_repack_scales";
    L2_CHECK(out && in, "%s: null pointer", fn);
    L2_CHECK(meta_height > 0 && width > 0, "%s: meta_height=%d width=%d must be positive", fn, meta_height, width);
    const size_t bytes = static_cast<size_t>(meta_height) * width * 2;
    L2_CHECK(!overlap(out, bytes, in, bytes), "%s: out and in overlap", fn);
    hipLaunchKernelGGL(transpose_u16_kernel, dim3(ceil_div(width, 64), ceil_div(meta_height, 64)), dim3(256), 0,
                       ctx().stream, out, in, meta_height, width);
    L2_LAUNCH_CHECK(fn);
    return LLAMA2_OK;
}

int llama2_compact_scales_v1(llama2_half* out, const llama2_half* in, int scales_size, int width)
{
    L2_REQUIRE_INIT();
    const char* fn = "llama2_compact_scales_v1";
    L2_CHECK(out && in, "%s: null pointer", fn);
    L2_CHECK(scales_size > 0 && width > 0, "%s: scales_size=%d width=%d must be positive", fn, scales_size, width);
    const int in_stride = ceil_div(scales_size, 8) * 8;
    const size_t total = static_cast<size_t>(scales_size) * width;
    L2_CHECK(!overlap(out, total * 2, in, static_cast<size_t>(in_stride) * width * 2), "%s: out and in overlap", fn);
    hipLaunchKernelGGL(compact_rows_u16_kernel, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0,
                       ctx().stream, out, in, scales_size, in_stride, total);
    L2_LAUNCH_CHECK(fn);
    return LLAMA2_OK;
}

} // extern "C"

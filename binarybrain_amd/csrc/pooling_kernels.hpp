// MaxPooling and UpSampling over images held as rows (channel, y, x) of frames, and Shuffle, a permutation of whole rows
// (reference: include/bb/MaxPooling.h:251-284, 340-370, 478-506, 551-579; include/bb/UpSampling.h:223-259, 321-353;
// include/bb/Shuffle.h:166-185, 225-243; entry points include/bbcu/bbcu.h:949-1016, 1024-1069, 1194-1216).
//
// Windows of filter_h x filter_w tile the image without overlap (the last ones are cut off at the border), so every input
// element belongs to one window and every kernel writes each output element once: streaming maps with one thread per W
// consecutive frames of a window (W = 4 with 128-bit accesses where rows are 16-byte aligned, else 1) or, for packed
// rows, per 32-frame word.  The loads of a window are issued before the first comparison; 2 x 2 windows, the usual case,
// are compiled with constant bounds.  Selections and fixed-order sums: the bits of the reference's host loops.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "bn_kernels.hpp"
#include "tile_divisor.hpp"

namespace bbhip {

constexpr int kPoolBlock   = 256;
constexpr int kPoolMaxTaps = 9;         // windows up to 3 x 3 are held in registers

struct WindowArgs {
    void const  *x;             // forward: input rows (fp32 or packed words); packed backward: the forward input
    int const   *argmax_in;     // fp32 backward
    float const *dy;            // backward
    void        *out;           // forward: y; backward: dx
    int         *argmax_out;    // fp32 forward
    int fh, fw, w, h, ow, oh, frame_size, x_stride, out_stride;
    int fill;                   // UpSampling
    TileDivisor f_blocks;       // workgroups per row of the launch's index space
    TileDivisor row_w, row_h;   // row of the index space -> (channel, y, x)
};

// row of the launch's index space -> (channel, y, x) with extents (row_h.count, row_w.count)
__device__ __forceinline__ void split_pixel(int node, WindowArgs const &a, int &c, int &y, int &x)
{
    int plane;
    split_tile(node, a.row_w, plane, x);
    split_tile(plane, a.row_h, c, y);
}

// ---- MaxPooling, fp32 ----------------------------------------------------------------------------------------------
// One thread per (window, W frames): the largest value found with a strict > from the lowest float in (fy, fx) order, and
// the position of its first occurrence counted over the positions inside the image.
template <int W, bool TWO>
__global__ __launch_bounds__(kPoolBlock) void max_pooling_forward_kernel(WindowArgs a)
{
    int node, block, c, oy, ox;
    split_tile(blockIdx.x, a.f_blocks, node, block);
    int const f = (block * kPoolBlock + threadIdx.x) * W;
    if (f >= a.frame_size) { return; }
    split_pixel(node, a, c, oy, ox);
    int const fh = TWO ? 2 : a.fh, fw = TWO ? 2 : a.fw;
    float const *__restrict__ x = static_cast<float const *>(a.x);
    float best[W];
    int arg_best[W];
#pragma unroll
    for (int j = 0; j < W; ++j) { best[j] = -3.402823466e+38f; arg_best[j] = 0; }
    int arg = 0;
    if (TWO || (fh <= 3 && fw <= 3)) {
        float v[TWO ? 4 : kPoolMaxTaps][W];
#pragma unroll
        for (int fy = 0; fy < (TWO ? 2 : 3); ++fy) {
#pragma unroll
            for (int fx = 0; fx < (TWO ? 2 : 3); ++fx) {
                int const iy = oy * fh + fy, ix = ox * fw + fx;
                if (fy < fh && fx < fw && iy < a.h && ix < a.w) {
                    bn_load<W>(x + (size_t)((c * a.h + iy) * a.w + ix) * a.x_stride, f, a.frame_size, v[fy * (TWO ? 2 : 3) + fx]);
                }
            }
        }
#pragma unroll
        for (int fy = 0; fy < (TWO ? 2 : 3); ++fy) {
#pragma unroll
            for (int fx = 0; fx < (TWO ? 2 : 3); ++fx) {
                int const iy = oy * fh + fy, ix = ox * fw + fx;
                if (fy < fh && fx < fw && iy < a.h && ix < a.w) {
#pragma unroll
                    for (int j = 0; j < W; ++j) {
                        float const t = v[fy * (TWO ? 2 : 3) + fx][j];
                        if (t > best[j]) { best[j] = t; arg_best[j] = arg; }
                    }
                    ++arg;
                }
            }
        }
    }
    else {
        for (int fy = 0; fy < fh; ++fy) {
            int const iy = oy * fh + fy;
            if (iy >= a.h) { break; }
            for (int fx = 0; fx < fw; ++fx) {
                int const ix = ox * fw + fx;
                if (ix >= a.w) { break; }
                float t[W];
                bn_load<W>(x + (size_t)((c * a.h + iy) * a.w + ix) * a.x_stride, f, a.frame_size, t);
#pragma unroll
                for (int j = 0; j < W; ++j) { if (t[j] > best[j]) { best[j] = t[j]; arg_best[j] = arg; } }
                ++arg;
            }
        }
    }
    float as_float[W];
#pragma unroll
    for (int j = 0; j < W; ++j) { as_float[j] = __int_as_float(arg_best[j]); }
    bn_store<W>(static_cast<float *>(a.out) + (size_t)node * a.out_stride, f, a.frame_size, best);
    bn_store<W>(reinterpret_cast<float *>(a.argmax_out) + (size_t)node * a.out_stride, f, a.frame_size, as_float);
}

// dx of the recorded position = dy, of the window's other positions 0
template <int W>
__global__ __launch_bounds__(kPoolBlock) void max_pooling_backward_kernel(WindowArgs a)
{
    int node, block, c, oy, ox;
    split_tile(blockIdx.x, a.f_blocks, node, block);
    int const f = (block * kPoolBlock + threadIdx.x) * W;
    if (f >= a.frame_size) { return; }
    split_pixel(node, a, c, oy, ox);
    float g[W], which[W];
    bn_load<W>(a.dy + (size_t)node * a.out_stride, f, a.frame_size, g);
    bn_load<W>(reinterpret_cast<float const *>(a.argmax_in) + (size_t)node * a.out_stride, f, a.frame_size, which);
    float *__restrict__ dx = static_cast<float *>(a.out);
    int arg = 0;
    for (int fy = 0; fy < a.fh; ++fy) {
        int const iy = oy * a.fh + fy;
        if (iy >= a.h) { break; }
        for (int fx = 0; fx < a.fw; ++fx) {
            int const ix = ox * a.fw + fx;
            if (ix >= a.w) { break; }
            float v[W];
#pragma unroll
            for (int j = 0; j < W; ++j) { v[j] = (__float_as_int(which[j]) == arg) ? g[j] : 0.0f; }
            bn_store<W>(dx + (size_t)((c * a.h + iy) * a.w + ix) * a.out_stride, f, a.frame_size, v);
            ++arg;
        }
    }
}

// ---- MaxPooling, packed bits ---------------------------------------------------------------------------------------
// y = the OR of the window; one thread per (window, word), the (window, word) pairs numbered through: a packed row of a
// training batch is a few words, far fewer than a workgroup has threads
__global__ __launch_bounds__(kPoolBlock) void max_pooling_bit_forward_kernel(WindowArgs a, int words, long long total)
{
    long long const gid = (long long)blockIdx.x * kPoolBlock + threadIdx.x;
    if (gid >= total) { return; }
    int node, wd, c, oy, ox;
    split_tile((int)gid, a.f_blocks, node, wd);         // f_blocks holds the words per row here
    split_pixel(node, a, c, oy, ox);
    uint32_t const *__restrict__ x = static_cast<uint32_t const *>(a.x);
    uint32_t any = 0;
    for (int fy = 0; fy < a.fh; ++fy) {
        int const iy = oy * a.fh + fy;
        if (iy >= a.h) { break; }
        for (int fx = 0; fx < a.fw; ++fx) {
            int const ix = ox * a.fw + fx;
            if (ix >= a.w) { break; }
            any |= x[(size_t)((c * a.h + iy) * a.w + ix) * a.x_stride + wd];
        }
    }
    if (wd == words - 1 && (a.frame_size & 31)) { any &= (1u << (a.frame_size & 31)) - 1u; }       // bits past the last frame are 0
    static_cast<uint32_t *>(a.out)[(size_t)node * a.out_stride + wd] = any;
}

// dy goes to the first set input of the window in (fy, fx) order, 0 to the others; one thread per (window, frame)
__global__ __launch_bounds__(kPoolBlock) void max_pooling_bit_backward_kernel(WindowArgs a)
{
    int node, block, c, oy, ox;
    split_tile(blockIdx.x, a.f_blocks, node, block);
    int const f = block * kPoolBlock + threadIdx.x;
    if (f >= a.frame_size) { return; }
    split_pixel(node, a, c, oy, ox);
    uint32_t const *__restrict__ x = static_cast<uint32_t const *>(a.x);
    float *__restrict__ dx = static_cast<float *>(a.out);
    float grad = a.dy[(size_t)node * a.out_stride + f];
    for (int fy = 0; fy < a.fh; ++fy) {
        int const iy = oy * a.fh + fy;
        if (iy >= a.h) { break; }
        for (int fx = 0; fx < a.fw; ++fx) {
            int const ix = ox * a.fw + fx;
            if (ix >= a.w) { break; }
            size_t const in_node = (size_t)((c * a.h + iy) * a.w + ix);
            bool const sig = (x[in_node * a.x_stride + (f >> 5)] >> (f & 31)) & 1u;
            dx[in_node * a.out_stride + f] = sig ? grad : 0.0f;
            if (sig) { grad = 0.0f; }
        }
    }
}

// ---- UpSampling ----------------------------------------------------------------------------------------------------
// Output pixel (oy, ox) reads input pixel (oy / fh, ox / fw): all of the block (fill) or only its position (fh / 2, fw / 2)
// with zeros around.  One thread per (output pixel, W frames) or, packed, per (output pixel, word).
template <bool BIT, int W>
__global__ __launch_bounds__(kPoolBlock) void up_sampling_forward_kernel(WindowArgs a, int items, long long total)
{
    int node, f, c, oy, ox;
    if constexpr (BIT) {                                // (pixel, word) pairs numbered through, f_blocks = words per row
        long long const gid = (long long)blockIdx.x * kPoolBlock + threadIdx.x;
        if (gid >= total) { return; }
        split_tile((int)gid, a.f_blocks, node, f);
    }
    else {
        int block;
        split_tile(blockIdx.x, a.f_blocks, node, block);
        f = (block * kPoolBlock + threadIdx.x) * W;
        if (f >= items) { return; }
    }
    split_pixel(node, a, c, oy, ox);                    // extents: the output image
    int const iy = oy / a.fh, ix = ox / a.fw;
    bool const take = a.fill || (oy - iy * a.fh == a.fh / 2 && ox - ix * a.fw == a.fw / 2);
    size_t const in_node = (size_t)((c * a.h + iy) * a.w + ix);
    if constexpr (BIT) {
        uint32_t const v = take ? static_cast<uint32_t const *>(a.x)[in_node * a.x_stride + f] : 0u;
        static_cast<uint32_t *>(a.out)[(size_t)node * a.out_stride + f] = v;
    }
    else {
        float v[W];
        if (take) { bn_load<W>(static_cast<float const *>(a.x) + in_node * a.x_stride, f, items, v); }
        else {
#pragma unroll
            for (int j = 0; j < W; ++j) { v[j] = 0.0f; }
        }
        bn_store<W>(static_cast<float *>(a.out) + (size_t)node * a.out_stride, f, items, v);
    }
}

// dx = the sum of dy over the block in (fy, fx) order (fill), or dy at the block's position (fh / 2, fw / 2)
template <int W>
__global__ __launch_bounds__(kPoolBlock) void up_sampling_backward_kernel(WindowArgs a)
{
    int node, block, c, iy, ix;
    split_tile(blockIdx.x, a.f_blocks, node, block);
    int const f = (block * kPoolBlock + threadIdx.x) * W;
    if (f >= a.frame_size) { return; }
    split_pixel(node, a, c, iy, ix);                    // extents: the input image
    int const ow = a.w * a.fw, oh = a.h * a.fh;
    float sum[W];
#pragma unroll
    for (int j = 0; j < W; ++j) { sum[j] = 0.0f; }
    if (a.fill) {
        for (int fy = 0; fy < a.fh; ++fy) {
            for (int fx = 0; fx < a.fw; ++fx) {
                float g[W];
                bn_load<W>(a.dy + (size_t)((c * oh + iy * a.fh + fy) * ow + ix * a.fw + fx) * a.out_stride, f, a.frame_size, g);
#pragma unroll
                for (int j = 0; j < W; ++j) { sum[j] += g[j]; }
            }
        }
    }
    else {
        float g[W];
        bn_load<W>(a.dy + (size_t)((c * oh + iy * a.fh + a.fh / 2) * ow + ix * a.fw + a.fw / 2) * a.out_stride, f, a.frame_size, g);
#pragma unroll
        for (int j = 0; j < W; ++j) { sum[j] += g[j]; }          // 0 + dy, as the host loop adds it
    }
    bn_store<W>(static_cast<float *>(a.out) + (size_t)node * a.out_stride, f, a.frame_size, sum);
}

// ---- Shuffle -------------------------------------------------------------------------------------------------------
// Destination row group * unit.count + u takes source row u * group_size + group: the rows, seen as a [unit][group] matrix,
// are transposed.  The backward pass is the same copy with the two extents exchanged.  Rows are copied whole, whatever they
// hold; one thread per (destination row, piece of V words), pieces numbered through so that short rows still fill the chip.
struct ShuffleArgs {
    uint32_t const *src;
    uint32_t       *dst;
    TileDivisor     pieces;     // per row
    TileDivisor     unit;
    int             group_size;
    int             stride;     // words per row
};

template <int V>
__global__ __launch_bounds__(kPoolBlock) void row_shuffle_kernel(ShuffleArgs a, long long total)
{
    long long const gid = (long long)blockIdx.x * kPoolBlock + threadIdx.x;
    if (gid >= total) { return; }
    int row, piece, group, u;
    split_tile((int)gid, a.pieces, row, piece);
    split_tile(row, a.unit, group, u);
    size_t const from = ((size_t)u * a.group_size + group) * a.stride, to = (size_t)row * a.stride;
    if constexpr (V == 4) { reinterpret_cast<uint4 *>(a.dst + to)[piece] = reinterpret_cast<uint4 const *>(a.src + from)[piece]; }
    else                  { a.dst[to + piece] = a.src[from + piece]; }
}

}  // namespace bbhip

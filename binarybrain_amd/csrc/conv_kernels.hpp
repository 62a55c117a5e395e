// Convolution plumbing around the LUT layers: Im2Col, Col2Im, StochasticMaxPooling2x2.
//
// A convolution in this framework is Im2Col -> LUT layers -> Col2Im: Im2Col turns every filter window position of every
// image into its own frame (frame' = (frame, oy, ox), node' = (c, fy, fx)), Col2Im turns them back into pixels
// (node = (c, y, x)).  Both are permutations between the pixel index and the frame index of node-major, frame-minor
// buffers, i.e. transposes whose two sides are contiguous along different indices.  The fp32 kernels stage 64 x 64
// tiles through LDS so that reads and writes are both made of contiguous runs; the packed-bit kernels assemble each
// output word from 32 single-bit gathers.  (Reference semantics: the host paths of include/bb/ConvolutionIm2Col.h:370-452,
// ConvolutionCol2Im.h:203-293, StochasticMaxPooling2x2.h:190-306.)
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "vector_kernels.hpp"
#include "bn_kernels.hpp"

namespace bbhip {

constexpr int kConvBlock = 256;
constexpr int kTile = 64;

struct Im2ColArgs {
    void const *x;          // [c*h*w][input_frame_stride]
    void       *y;          // [c*fh*fw][output_frame_stride], frames*oh*ow frames
    int x_stride, y_stride, x_offset, y_offset;
    int input_frame_size, input_frame_stride;
    int w, h, c, ow, oh, output_frame_stride, fw, fh;
    int border_mode;
    float border_value;
    int q_tiles, f_tiles;      // q_tiles: 64-position tiles of the flattened output plane (forward)
};

// include/bb/ConvolutionIm2Col.h:251-286
__device__ __forceinline__ bool im2col_border(int mode, int &x, int &y, int w, int h)
{
    switch (mode) {
    case 1: if (x < 0) { x = -x - 1; } if (y < 0) { y = -y - 1; } if (x >= w) { x = (w - 1) - (x - w); } if (y >= h) { y = (h - 1) - (y - h); } return true;
    case 2: if (x < 0) { x = -x; }     if (y < 0) { y = -y; }     if (x >= w) { x = (w - 2) - (x - w); } if (y >= h) { y = (h - 2) - (y - h); } return true;
    case 3: if (x < 0) { x = 0; }      if (y < 0) { y = 0; }      if (x >= w) { x = w - 1; }             if (y >= h) { y = h - 1; }             return true;
    case 4: if (x < 0) { x += w; }     if (y < 0) { y += h; }     if (x >= w) { x -= w; }                if (y >= h) { y -= h; }                return true;
    default: return false;
    }
}

// input pixel of window position (oy, ox), tap (fy, fx); false = the constant border value applies
__device__ __forceinline__ bool im2col_source(Im2ColArgs const &a, int oy, int ox, int fy, int fx, int &iy, int &ix)
{
    iy = oy * a.y_stride - a.y_offset + fy;
    ix = ox * a.x_stride - a.x_offset + fx;
    if (iy >= 0 && iy < a.h && ix >= 0 && ix < a.w) { return true; }
    return im2col_border(a.border_mode, ix, iy, a.w, a.h);
}

// block = (output node, 64 window positions of the flattened (oy, ox) plane, 64 input frames): rows of the input are read
// along the frames, the tile is written along the window positions, which are contiguous in the output
__global__ __launch_bounds__(kConvBlock) void im2col_forward_kernel(Im2ColArgs a)
{
    __shared__ float tile[kTile][kTile + 1];                 // [window position][frame]
    int b = blockIdx.x;
    int const ft = b % a.f_tiles;  b /= a.f_tiles;
    int const qt = b % a.q_tiles;  b /= a.q_tiles;
    int const node = b;                                      // (c*fh + fy)*fw + fx
    int const fx = node % a.fw, fy = (node / a.fw) % a.fh, c = node / (a.fw * a.fh);
    int const lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int const f0 = ft * kTile, q0 = qt * kTile;
    int const plane = a.oh * a.ow;
    float const *x = static_cast<float const *>(a.x);
    float *y = static_cast<float *>(a.y);

    // all loads of a wavefront's 16 rows are issued before the first of them is used (one round trip instead of sixteen)
    constexpr int kRows = kTile / (kConvBlock / 64);
    float v[kRows];
    int oy = (q0 + wave) / a.ow, ox = (q0 + wave) - oy * a.ow;      // of the wavefront's first row; the next rows step on from it
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
        int const q = q0 + wave + r * (kConvBlock / 64);
        v[r] = a.border_value;
        if (r > 0) {
            ox += kConvBlock / 64;
            while (ox >= a.ow) { ox -= a.ow; ++oy; }
        }
        if (q < plane) {
            int iy, ix;
            bool const have = im2col_source(a, oy, ox, fy, fx, iy, ix);  // wave-uniform
            if (have && f0 + lane < a.input_frame_size) {
                v[r] = x[((size_t)(c * a.h + iy) * a.w + ix) * a.input_frame_stride + f0 + lane];
            }
        }
    }
#pragma unroll
    for (int r = 0; r < kRows; ++r) { tile[wave + r * (kConvBlock / 64)][lane] = v[r]; }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
        int const f = wave + r * (kConvBlock / 64);
        if (f0 + f < a.input_frame_size && q0 + lane < plane) {
            y[(size_t)node * a.output_frame_stride + (size_t)(f0 + f) * plane + q0 + lane] = tile[lane][f];
        }
    }
}

// one thread per output word (32 consecutive output frames of one node)
__global__ __launch_bounds__(kConvBlock) void im2col_forward_bit_kernel(Im2ColArgs a, int words_per_node, long long total_words)
{
    long long const t = (long long)blockIdx.x * kConvBlock + threadIdx.x;
    if (t >= total_words) { return; }
    int const wd = (int)(t % words_per_node);
    int const node = (int)(t / words_per_node);
    int const fx = node % a.fw, fy = (node / a.fw) % a.fh, c = node / (a.fw * a.fh);
    uint32_t const *x = static_cast<uint32_t const *>(a.x);
    long long const plane = (long long)a.oh * a.ow;
    long long const frames = (long long)a.input_frame_size * plane;
    uint32_t out = 0;
    for (int bit = 0; bit < 32; ++bit) {
        long long const of = (long long)wd * 32 + bit;
        if (of >= frames) { break; }
        int const in_frame = (int)(of / plane);
        int const f = (int)(of % plane);
        int iy, ix;
        if (im2col_source(a, f / a.ow, f % a.ow, fy, fx, iy, ix)) {
            uint32_t const word = x[((size_t)(c * a.h + iy) * a.w + ix) * a.input_frame_stride + (in_frame >> 5)];
            out |= ((word >> (in_frame & 31)) & 1u) << bit;
        }
    }
    static_cast<uint32_t *>(a.y)[(size_t)node * a.output_frame_stride + wd] = out;
}

// dx[(c, y, x)][f] = sum over the taps (fy, fx) whose window holds (y, x), in (fy, fx) order, of dy[(c, fy, fx)][(f, oy, ox)]
// (include/bb/ConvolutionIm2Col.h:411-452: border replicas carry no gradient).  block = (c, 64 pixels of the flattened
// image, 64 frames): one lane per pixel forms the sums (pixels of one image row are contiguous along ox in dy), which are
// then transposed through LDS so that the stores run along the frames.  Flattening keeps the lanes busy for images
// narrower than a wavefront; TF (frames per block) is 64, or 16 when the batch is too small to fill the device otherwise.
template <int TF>
__global__ __launch_bounds__(kConvBlock) void im2col_backward_kernel(Im2ColArgs a, int p_tiles)
{
    __shared__ float tile[kTile][TF + 1];                    // [pixel][frame]
    int b = blockIdx.x;
    int const ft = b % a.f_tiles; b /= a.f_tiles;
    int const pt = b % p_tiles;   b /= p_tiles;
    int const c  = b;
    int const lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int const f0 = ft * TF, p0 = pt * kTile;
    int const hw = a.h * a.w;
    int const p = p0 + lane;
    float const *dy = static_cast<float const *>(a.x);       // the gradient buffer comes in through the first slot
    float *dx = static_cast<float *>(a.y);
    constexpr int kWaves = kConvBlock / 64;
    constexpr int kPer = TF / kWaves;                        // frames per thread
    float acc[kPer];
#pragma unroll
    for (int j = 0; j < kPer; ++j) { acc[j] = 0.0f; }

    int const iy_limit = (a.oh - 1) * a.y_stride, ix_limit = (a.ow - 1) * a.x_stride;
    size_t const plane = (size_t)a.oh * a.ow;
    if (kPer <= 4 && a.x_stride == 1 && a.y_stride == 1 && a.fh <= 3 && a.fw <= 3) {
        // Filters up to 3 x 3 at stride 1 (workgroup-uniform): the loads of all taps go out together — nine round trips become one —
        // and the sums are formed in the same (fy, fx) order afterwards.  A tap outside the window contributes +0, which leaves a
        // sum that started at +0 unchanged.
        float v[3][3][kPer];
        int const y = (p < hw) ? p / a.w : 0, x = (p < hw) ? p - y * a.w : 0;
#pragma unroll
        for (int fy = 0; fy < 3; ++fy) {
#pragma unroll
            for (int fx = 0; fx < 3; ++fx) {
                int const iy = y - fy + a.y_offset, ix = x - fx + a.x_offset;
                bool const have = (p < hw) && fy < a.fh && fx < a.fw && iy >= 0 && iy <= iy_limit && ix >= 0 && ix <= ix_limit;
                float const *row = dy + (size_t)((c * a.fh + fy) * a.fw + fx) * a.output_frame_stride + (size_t)iy * a.ow + ix;
#pragma unroll
                for (int j = 0; j < kPer; ++j) {
                    int const f = f0 + wave + j * kWaves;
                    v[fy][fx][j] = (have && f < a.input_frame_size) ? row[(size_t)f * plane] : 0.0f;
                }
            }
        }
#pragma unroll
        for (int fy = 0; fy < 3; ++fy) {
#pragma unroll
            for (int fx = 0; fx < 3; ++fx) {
#pragma unroll
                for (int j = 0; j < kPer; ++j) { acc[j] += v[fy][fx][j]; }
            }
        }
    }
    else if (p < hw) {
        int const y = p / a.w, x = p - y * a.w;
        int const x_align = x % a.x_stride, y_align = y % a.y_stride;
        for (int fy = y_align; fy < a.fh; fy += a.y_stride) {
            int const iy = y - fy + a.y_offset;
            if (iy < 0 || iy > iy_limit) { continue; }
            for (int fx = x_align; fx < a.fw; fx += a.x_stride) {
                int const ix = x - fx + a.x_offset;
                if (ix < 0 || ix > ix_limit) { continue; }
                float const *row = dy + (size_t)((c * a.fh + fy) * a.fw + fx) * a.output_frame_stride
                                      + (size_t)(iy / a.y_stride) * a.ow + (ix / a.x_stride);
#pragma unroll
                for (int j = 0; j < kPer; ++j) {
                    int const f = f0 + wave + j * kWaves;
                    if (f < a.input_frame_size) { acc[j] += row[(size_t)f * plane]; }
                }
            }
        }
    }
#pragma unroll
    for (int j = 0; j < kPer; ++j) { tile[lane][wave + j * kWaves] = acc[j]; }
    __syncthreads();
    // TF consecutive threads store the TF frames of one pixel
    constexpr int kPixelsPerPass = kConvBlock / TF;
    int const fl = threadIdx.x % TF, pl = threadIdx.x / TF;
    for (int i = pl; i < kTile; i += kPixelsPerPass) {
        if (p0 + i < hw && f0 + fl < a.input_frame_size) {
            dx[((size_t)c * hw + p0 + i) * a.input_frame_stride + f0 + fl] = tile[i][fl];
        }
    }
}

// y[(c, xy)][f] = x[c][f*hw + xy]  (forward)  /  dx[c][f*hw + xy] = dy[(c, xy)][f]  (backward): a [frames][hw] <-> [hw][frames]
// transpose per channel.  block = (c, 64 pixels, 64 frames).  `narrow` is the [c][frames*hw] side, `wide` the [c*hw][frames] side.
template <bool FORWARD>
__global__ __launch_bounds__(kConvBlock) void col2im_kernel(float const *__restrict__ src, float *__restrict__ dst, int hw, int c_size,
                                                           int narrow_stride, int frames, int wide_stride, int xy_tiles, int f_tiles)
{
    __shared__ float tile[kTile][kTile + 1];
    int b = blockIdx.x;
    int const ft = b % f_tiles;  b /= f_tiles;
    int const xt = b % xy_tiles; b /= xy_tiles;
    int const c = b;
    int const lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int const f0 = ft * kTile, xy0 = xt * kTile;
    // all loads of a wavefront's 16 rows are issued before the first of them is used (one round trip instead of sixteen)
    constexpr int kStep = kConvBlock / 64, kRows = kTile / kStep;
    float v[kRows];
    if (FORWARD) {
#pragma unroll
        for (int r = 0; r < kRows; ++r) {                                                  // lanes along xy: contiguous in src
            int const f = wave + r * kStep;
            v[r] = (f0 + f < frames && xy0 + lane < hw) ? src[(size_t)c * narrow_stride + (size_t)(f0 + f) * hw + xy0 + lane] : 0.0f;
        }
#pragma unroll
        for (int r = 0; r < kRows; ++r) { tile[wave + r * kStep][lane] = v[r]; }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kRows; ++r) {                                                  // lanes along frames: contiguous in dst
            int const i = wave + r * kStep;
            if (xy0 + i < hw && f0 + lane < frames) { dst[((size_t)c * hw + xy0 + i) * wide_stride + f0 + lane] = tile[lane][i]; }
        }
    }
    else {
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
            int const i = wave + r * kStep;
            v[r] = (xy0 + i < hw && f0 + lane < frames) ? src[((size_t)c * hw + xy0 + i) * wide_stride + f0 + lane] : 0.0f;
        }
#pragma unroll
        for (int r = 0; r < kRows; ++r) { tile[wave + r * kStep][lane] = v[r]; }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kRows; ++r) {
            int const f = wave + r * kStep;
            if (f0 + f < frames && xy0 + lane < hw) { dst[(size_t)c * narrow_stride + (size_t)(f0 + f) * hw + xy0 + lane] = tile[lane][f]; }
        }
    }
}

// one thread per output word of the [c*hw][frames] side
__global__ __launch_bounds__(kConvBlock) void col2im_forward_bit_kernel(uint32_t const *__restrict__ x, uint32_t *__restrict__ y, int hw,
                                                                       int input_frame_stride, int frames, int output_frame_stride,
                                                                       int words_per_node, long long total_words)
{
    long long const t = (long long)blockIdx.x * kConvBlock + threadIdx.x;
    if (t >= total_words) { return; }
    int const wd = (int)(t % words_per_node);
    long long const node = t / words_per_node;           // c*hw + xy
    int const xy = (int)(node % hw);
    long long const c = node / hw;
    uint32_t out = 0;
    for (int bit = 0; bit < 32; ++bit) {
        int const f = wd * 32 + bit;
        if (f >= frames) { break; }
        long long const in_frame = (long long)f * hw + xy;
        uint32_t const word = x[(size_t)c * input_frame_stride + (in_frame >> 5)];
        out |= ((word >> (in_frame & 31)) & 1u) << bit;
    }
    y[(size_t)node * output_frame_stride + wd] = out;
}

struct PoolArgs {
    float const *x;
    float const *dy;
    float       *out;       // y (forward) or dx (backward)
    int w, h, ow, oh, c, frame_size, frame_stride;
};

// y = 1 - prod over the window taps inside the image, (fy, fx) ascending, of (1 - x): the probability that at least one
// of four independent binary inputs is 1 (include/bb/StochasticMaxPooling2x2.h:190-218).  One thread per (output node,
// W frames), W = 4 with 128-bit accesses where rows are 16-byte aligned; the four taps are loaded before the first is used.
template <int W>
__global__ __launch_bounds__(kConvBlock) void stochastic_maxpool2x2_forward_kernel(PoolArgs a, int f_blocks)
{
    int const f = ((int)(blockIdx.x % f_blocks) * kConvBlock + threadIdx.x) * W;
    int const node = blockIdx.x / f_blocks;
    if (f >= a.frame_size) { return; }
    int const ox = node % a.ow, oy = (node / a.ow) % a.oh, c = node / (a.ow * a.oh);
    float v[2][2][W];
#pragma unroll
    for (int fy = 0; fy < 2; ++fy) {
#pragma unroll
        for (int fx = 0; fx < 2; ++fx) {
            int const iy = oy * 2 + fy, ix = ox * 2 + fx;
            if (iy < a.h && ix < a.w) { bn_load<W>(a.x + ((size_t)(c * a.h + iy) * a.w + ix) * a.frame_stride, f, a.frame_size, v[fy][fx]); }
        }
    }
    float out[W];
#pragma unroll
    for (int j = 0; j < W; ++j) { out[j] = 1.0f; }
#pragma unroll
    for (int fy = 0; fy < 2; ++fy) {
#pragma unroll
        for (int fx = 0; fx < 2; ++fx) {
            int const iy = oy * 2 + fy, ix = ox * 2 + fx;
            if (iy < a.h && ix < a.w) {
                // the product is rounded on its own (not fused into the final 1 - out)
#pragma unroll
                for (int j = 0; j < W; ++j) { out[j] = rounded_mul(out[j], 1.0f - v[fy][fx][j]); }
            }
        }
    }
#pragma unroll
    for (int j = 0; j < W; ++j) { out[j] = 1.0f - out[j]; }
    bn_store<W>(a.out + (size_t)node * a.frame_stride, f, a.frame_size, out);
}

// dx of each tap = dy * prod over the other three taps of (1 - x), the product evaluated in double and rounded once, taps
// outside the image reading as 0 (include/bb/StochasticMaxPooling2x2.h:262-306)
template <int W>
__global__ __launch_bounds__(kConvBlock) void stochastic_maxpool2x2_backward_kernel(PoolArgs a, int f_blocks)
{
    int const f = ((int)(blockIdx.x % f_blocks) * kConvBlock + threadIdx.x) * W;
    int const node = blockIdx.x / f_blocks;
    if (f >= a.frame_size) { return; }
    int const ox = node % a.ow, oy = (node / a.ow) % a.oh, c = node / (a.ow * a.oh);
    float v[2][2][W], gv[W];
#pragma unroll
    for (int fy = 0; fy < 2; ++fy) {
#pragma unroll
        for (int fx = 0; fx < 2; ++fx) {
            int const iy = oy * 2 + fy, ix = ox * 2 + fx;
            if (iy < a.h && ix < a.w) { bn_load<W>(a.x + ((size_t)(c * a.h + iy) * a.w + ix) * a.frame_stride, f, a.frame_size, v[fy][fx]); }
            else {
#pragma unroll
                for (int j = 0; j < W; ++j) { v[fy][fx][j] = 0.0f; }
            }
        }
    }
    bn_load<W>(a.dy + (size_t)node * a.frame_stride, f, a.frame_size, gv);
    float gr[2][2][W];
#pragma unroll
    for (int j = 0; j < W; ++j) {
        double const g = (double)gv[j];
        double const i00 = (double)v[0][0][j], i01 = (double)v[0][1][j], i10 = (double)v[1][0][j], i11 = (double)v[1][1][j];
        gr[0][0][j] = (float)(g * (1.0 - i01) * (1.0 - i10) * (1.0 - i11));
        gr[0][1][j] = (float)(g * (1.0 - i00) * (1.0 - i10) * (1.0 - i11));
        gr[1][0][j] = (float)(g * (1.0 - i00) * (1.0 - i01) * (1.0 - i11));
        gr[1][1][j] = (float)(g * (1.0 - i00) * (1.0 - i01) * (1.0 - i10));
    }
#pragma unroll
    for (int fy = 0; fy < 2; ++fy) {
#pragma unroll
        for (int fx = 0; fx < 2; ++fx) {
            int const iy = oy * 2 + fy, ix = ox * 2 + fx;
            if (iy < a.h && ix < a.w) { bn_store<W>(a.out + ((size_t)(c * a.h + iy) * a.w + ix) * a.frame_stride, f, a.frame_size, gr[fy][fx]); }
        }
    }
}

}  // namespace bbhip

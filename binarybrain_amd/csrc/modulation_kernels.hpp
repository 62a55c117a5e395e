// The layers at either end of a binary network and the activations between its layers:
//   RealToBinary  (reference: include/bb/RealToBinary.h:300-344, cuda/RealToBinary.cu:140-260; entry points include/bbcu/bbcu.h:1337-1370)
//   BinaryToReal  (include/bb/BinaryToReal.h:262-290 forward, :333-352 backward; bbcu.h:1376-1413)
//   Binarize      (include/bb/Binarize.h:196-213; bbcu.h:1223-1246), HardTanh (include/bb/HardTanh.h:176-193, :253-271; bbcu.h:1253-1276)
//
// All of them stream node-major, frame-minor rows once: a thread owns W consecutive frames of one row (W = 4 with 128-bit
// accesses where rows are 16-byte aligned, else 1), a workgroup 256 * W frames, and the launch is a flat list of
// (row, frame block) pairs, so that the row count is not bounded by a grid dimension.  Packed outputs are assembled in
// registers: a thread's W bits are shifted to their place in the 32-bit word that neighbouring lanes share, the lanes'
// parts are combined by exchanges, and one lane per word stores it.
//
// Arithmetic follows the host loops of the reference operation by operation (every product rounded on its own, min and max
// as std::min / std::max evaluate them), so results are the bits of the reference's C++ expressions in fp32.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "bn_kernels.hpp"
#include "tile_divisor.hpp"
#include "vector_kernels.hpp"

namespace bbhip {

constexpr int kModBlock = 256;

// ---- elementwise maps over rows ------------------------------------------------------------------------------------
enum { kMapBinarize = 0, kMapHardTanh = 1, kMapHardTanhBackward = 2 };

struct RowMapArgs {
    float const *x;
    float const *dy;            // kMapHardTanhBackward only
    float       *out;
    int frame_size, x_stride, out_stride;
    float p0, p1, p2;           // Binarize: threshold, low, high; HardTanh: min, max
    TileDivisor f_blocks;       // workgroups per row
};

template <int OP, int W>
__global__ __launch_bounds__(kModBlock) void row_map_kernel(RowMapArgs a)
{
    int node, block;
    split_tile(blockIdx.x, a.f_blocks, node, block);
    int const f = (block * kModBlock + threadIdx.x) * W;
    if (f >= a.frame_size) { return; }
    float v[W], g[W];
    bn_load<W>(a.x + (size_t)node * a.x_stride, f, a.frame_size, v);
    if (OP == kMapHardTanhBackward) { bn_load<W>(a.dy + (size_t)node * a.out_stride, f, a.frame_size, g); }
#pragma unroll
    for (int j = 0; j < W; ++j) {
        if (OP == kMapBinarize) { v[j] = (v[j] > a.p0) ? a.p2 : a.p1; }
        if (OP == kMapHardTanh) {
            if (v[j] <= a.p0) { v[j] = a.p0; }
            if (v[j] >= a.p1) { v[j] = a.p1; }
        }
        if (OP == kMapHardTanhBackward) { v[j] = (v[j] <= a.p0 || v[j] >= a.p1) ? 0.0f : g[j]; }
    }
    bn_store<W>(a.out + (size_t)node * a.out_stride, f, a.frame_size, v);
}

// A thread's W bits (bit j = frame f + j, W = 4 or 1) -> the words of the workgroup's frames.  With W = 4 eight
// neighbouring lanes share a word and combine their nibbles by three exchanges; with W = 1 the wavefront's ballot is its
// two words.  Every lane of the workgroup calls this (lanes past the row's end with bits = 0): words past y_stride are not
// stored, bits past the last frame are stored as 0.
template <int W>
__device__ __forceinline__ void store_packed_bits(uint32_t bits, uint32_t *__restrict__ row, int f, int y_stride)
{
    if constexpr (W == 4) {
        uint32_t v = bits << (4 * (threadIdx.x & 7));
        v |= __shfl_xor(v, 1, 64);
        v |= __shfl_xor(v, 2, 64);
        v |= __shfl_xor(v, 4, 64);
        int const w = f >> 5;
        if ((threadIdx.x & 7) == 0 && w < y_stride) { row[w] = v; }
    }
    else {
        uint64_t const m = __ballot(bits != 0);
        int const lane = threadIdx.x & (kWave - 1);
        int const w = (f & ~(kWave - 1)) >> 5;
        if (lane == 0  && w     < y_stride) { row[w]     = (uint32_t)m; }
        if (lane == 32 && w + 1 < y_stride) { row[w + 1] = (uint32_t)(m >> 32); }
    }
}

// fp32 rows -> packed bits of x > threshold.  The launch covers whole words of every row (frames up to 32 * words).
template <int W>
__global__ __launch_bounds__(kModBlock) void binarize_bits_kernel(float const *__restrict__ x, uint32_t *__restrict__ y, float threshold,
                                                                  int frame_size, int x_stride, int y_stride, TileDivisor f_blocks)
{
    int node, block;
    split_tile(blockIdx.x, f_blocks, node, block);
    int const f = (block * kModBlock + threadIdx.x) * W;
    uint32_t bits = 0;
    if (f < frame_size) {
        float v[W];
        bn_load<W>(x + (size_t)node * x_stride, f, frame_size, v);
#pragma unroll
        for (int j = 0; j < W; ++j) { if (f + j < frame_size && v[j] > threshold) { bits |= 1u << j; } }
    }
    store_packed_bits<W>(bits, y + (size_t)node * y_stride, f, y_stride);
}

// ---- RealToBinary --------------------------------------------------------------------------------------------------
struct RealToBinaryArgs {
    float const *x;
    void        *y;                 // fp32 rows or rows of packed words
    int x_frame_size, y_frame_size, x_stride, y_stride;
    TileDivisor points;             // output node -> (depth plane, point)
    TileDivisor depth_modulation;   // depth plane -> (input depth, depth step)
    float lo, x_scale, depth_step, depth_step_recip, frame_step, frame_step_recip;
    float threshold;                // packed output: 0.5 in binary mode, else 0 (the bit of the clamped value, v > 0)
    int binarize;                   // fp32 output: +1 / -1 by v > 0.5
    TileDivisor f_blocks;           // workgroups per output row
    TileDivisor frame_modulation;   // output frame -> (input frame, step within the modulation)
};

// The value of an input before the frame step: brought to [0, 1] and through the depth step d (include/bb/RealToBinary.h:318-324)
__device__ __forceinline__ float real_to_binary_depth_value(float x, float d, RealToBinaryArgs const &a)
{
    float const v = rounded_mul(x - a.lo, a.x_scale);
    return rounded_mul(v - rounded_mul(d, a.depth_step), a.depth_step_recip);
}

// ... and through frame step r, clamped (:326-330)
__device__ __forceinline__ float real_to_binary_frame_value(float t, float r, RealToBinaryArgs const &a)
{
    float v = rounded_mul(t - rounded_mul(r, a.frame_step), a.frame_step_recip);
    v = (v < 1.0f) ? v : 1.0f;      // std::min(1, v): a NaN becomes 1
    v = (0.0f < v) ? v : 0.0f;      // std::max(0, v)
    return v;
}

// A thread's W output frames are consecutive, so their (input frame, frame step) pairs follow from the first by counting:
// one division per thread.  The inputs of all W frames are requested before the first is used (neighbouring frames mostly
// share one, which the cache serves; a load that waits for the previous frame's arithmetic would cost a round trip each).
template <bool BIT, int W>
__global__ __launch_bounds__(kModBlock) void real_to_binary_kernel(RealToBinaryArgs a)
{
    int node, block;
    split_tile(blockIdx.x, a.f_blocks, node, block);
    // output node = (c * dm + d) * points + p  reads input node c * points + p
    int plane, p, c, d;
    split_tile(node, a.points, plane, p);
    split_tile(plane, a.depth_modulation, c, d);
    float const *__restrict__ xr = a.x + (size_t)(c * a.points.count + p) * a.x_stride;
    int const f = (block * kModBlock + threadIdx.x) * W;
    float v[W];
    uint32_t bits = 0;
    if (f < a.y_frame_size) {
        int g, r;
        split_tile(f, a.frame_modulation, g, r);
        float xv[W];
        int step[W];
#pragma unroll
        for (int j = 0; j < W; ++j) {
            xv[j] = xr[g];
            step[j] = r;
            if (++r == a.frame_modulation.count) {
                r = 0;
                g = (g + 1 < a.x_frame_size) ? g + 1 : g;          // frames past the end of the row are computed but not stored
            }
        }
#pragma unroll
        for (int j = 0; j < W; ++j) {
            v[j] = real_to_binary_frame_value(real_to_binary_depth_value(xv[j], (float)d, a), (float)step[j], a);
            if (BIT) { if (f + j < a.y_frame_size && v[j] > a.threshold) { bits |= 1u << j; } }
            else if (a.binarize) { v[j] = (v[j] > 0.5f) ? 1.0f : -1.0f; }
        }
    }
    if constexpr (BIT) { store_packed_bits<W>(bits, static_cast<uint32_t *>(a.y) + (size_t)node * a.y_stride, f, a.y_stride); }
    else {
        if (f < a.y_frame_size) { bn_store<W>(static_cast<float *>(a.y) + (size_t)node * a.y_stride, f, a.y_frame_size, v); }
    }
}

// ---- BinaryToReal --------------------------------------------------------------------------------------------------
struct BinaryToRealArgs {
    void const *x;                  // forward: fp32 rows or packed words; backward: unused
    float const *dy;                // backward
    float       *out;               // forward: y; backward: dx
    int node_mux_size, frame_mux_size, y_node_size;
    int x_stride, y_frame_size, y_stride;
    float denominator;              // forward: (float)(node_mux_size * frame_mux_size)
    float gain;                     // backward
    TileDivisor f_blocks;           // workgroups per row of `out`
    TileDivisor frame_mux;          // backward: input frame -> output frame
};

// y[o][g] = (number of inputs > 0 among nodes o, O + o, ... and frames g * fmux ... g * fmux + fmux - 1) / their number
template <bool BIT>
__global__ __launch_bounds__(kModBlock) void binary_to_real_forward_kernel(BinaryToRealArgs a)
{
    int o, block;
    split_tile(blockIdx.x, a.f_blocks, o, block);
    int const g = block * kModBlock + threadIdx.x;
    if (g >= a.y_frame_size) { return; }
    int const first = g * a.frame_mux_size;
    float count = 0.0f;                                 // whole numbers below 2^24: exact in any order
    for (int m = 0; m < a.node_mux_size; ++m) {
        size_t const row = (size_t)(m * a.y_node_size + o) * a.x_stride;
        if (BIT) {
            uint32_t const *__restrict__ xr = static_cast<uint32_t const *>(a.x) + row;
            int f = first, left = a.frame_mux_size;
            while (left > 0) {                          // the set bits of [f, f + left) word by word
                int const at = f & 31, take = (32 - at < left) ? 32 - at : left;
                uint32_t const mask = (take == 32) ? 0xffffffffu : (((1u << take) - 1u) << at);
                count += (float)__popc(xr[f >> 5] & mask);
                f += take; left -= take;
            }
        }
        else {
            float const *__restrict__ xr = static_cast<float const *>(a.x) + row + first;
            for (int i = 0; i < a.frame_mux_size; ++i) { count += (xr[i] > 0.0f) ? 1.0f : 0.0f; }
        }
    }
    a.out[(size_t)o * a.y_stride + g] = count / a.denominator;
}

// dx[node][f] = dy[node % O][f / fmux] * gain
template <int W>
__global__ __launch_bounds__(kModBlock) void binary_to_real_backward_kernel(BinaryToRealArgs a, int x_frame_size)
{
    int node, block;
    split_tile(blockIdx.x, a.f_blocks, node, block);
    int const f = (block * kModBlock + threadIdx.x) * W;
    if (f >= x_frame_size) { return; }
    float const *__restrict__ dyr = a.dy + (size_t)(node % a.y_node_size) * a.y_stride;
    float v[W];
#pragma unroll
    for (int j = 0; j < W; ++j) {
        int g, r;
        split_tile(f + j, a.frame_mux, g, r);
        v[j] = (f + j < x_frame_size) ? rounded_mul(dyr[g], a.gain) : 0.0f;
    }
    bn_store<W>(a.out + (size_t)node * a.x_stride, f, x_frame_size, v);
}

}  // namespace bbhip

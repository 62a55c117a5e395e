// The tail of a LUT classifier: AverageLut (sum / vote over n wired inputs), softmax cross entropy and categorical accuracy.
//
// All of it is streaming work over node-major, frame-minor buffers: one lane per frame (or per 32-frame word), rows read
// as contiguous runs.  Results follow the reference's host loops (include/bb/AverageLut.h:320-345, 386-406;
// LossSoftmaxCrossEntropy.h:159-211; MetricsCategoricalAccuracy.h:144-173): AverageLut writes the SUM when the output is
// not binarized, gradients are dy / n added node ascending then input ascending, each product that the host code rounds
// on its own is rounded on its own here.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "vector_kernels.hpp"

namespace bbhip {

constexpr int kTailBlock = 256;

// one thread per (output node, frame)
// scale: what an un-binarized sum is multiplied by — 1 (the host loop of the reference writes the sum) or the fp32
// reciprocal of n (its CUDA kernel writes sum * (1 / n), cuda/AverageLut.cu:46-54)
__global__ __launch_bounds__(kTailBlock) void average_lut_forward_kernel(float const *x, float *y, int const *idx, int n, int frame_size,
                                                                         int frame_stride, int binarize_input, int binarize_output, int f_blocks,
                                                                         float scale)
{
    int const f = (int)(blockIdx.x % f_blocks) * kTailBlock + threadIdx.x;
    int const node = blockIdx.x / f_blocks;
    if (f >= frame_size) { return; }
    int const *row = idx + (size_t)node * n;
    float sum = 0.0f;
    for (int i = 0; i < n; ++i) {
        float v = x[(size_t)row[i] * frame_stride + f];
        if (binarize_input) { v = (v > 0.0f) ? 1.0f : -1.0f; }
        sum += v;
    }
    if (binarize_output) { sum = (sum > 0.0f) ? 1.0f : -1.0f; }
    else                 { sum = rounded_mul(sum, scale); }
    y[(size_t)node * frame_stride + f] = sum;
}

// Packed bits, one thread per (output node, 32-frame word): the n input words are added into P bit planes (plane p holds
// bit p of each frame's count of ones) and the count is compared with floor(n / 2): ones > n / 2 is the strict majority
// that the host loop computes as (ones - zeros) > 0.
template <int P>
__global__ __launch_bounds__(kTailBlock) void average_lut_forward_bit_kernel(int const *x, int *y, int const *idx, int n, int words,
                                                                             int frame_stride, int w_blocks)
{
    int const w = (int)(blockIdx.x % w_blocks) * kTailBlock + threadIdx.x;
    int const node = blockIdx.x / w_blocks;
    if (w >= words) { return; }
    int const *row = idx + (size_t)node * n;
    uint32_t plane[P];
#pragma unroll
    for (int p = 0; p < P; ++p) { plane[p] = 0u; }
    for (int i = 0; i < n; ++i) {
        uint32_t carry = (uint32_t)x[(size_t)row[i] * frame_stride + w];
#pragma unroll
        for (int p = 0; p < P; ++p) {
            uint32_t const t = plane[p] & carry;
            plane[p] ^= carry;
            carry = t;
        }
    }
    uint32_t const threshold = (uint32_t)n >> 1;
    uint32_t gt = 0u, eq = ~0u;
#pragma unroll
    for (int p = P - 1; p >= 0; --p) {
        uint32_t const tb = ((threshold >> p) & 1u) ? ~0u : 0u;
        gt |= eq & plane[p] & ~tb;
        eq &= ~(plane[p] ^ tb);
    }
    y[(size_t)node * frame_stride + w] = (int)gt;
}

// any n: per frame bit, count the ones directly
__global__ __launch_bounds__(kTailBlock) void average_lut_forward_bit_wide_kernel(int const *x, int *y, int const *idx, int n, int words,
                                                                                  int frame_stride, int w_blocks)
{
    int const w = (int)(blockIdx.x % w_blocks) * kTailBlock + threadIdx.x;
    int const node = blockIdx.x / w_blocks;
    if (w >= words) { return; }
    int const *row = idx + (size_t)node * n;
    uint32_t out = 0u;
    for (int base = 0; base < 32; base += 4) {               // four frame bits per sweep over the inputs
        int ones[4] = {0, 0, 0, 0};
        for (int i = 0; i < n; ++i) {
            uint32_t const v = (uint32_t)x[(size_t)row[i] * frame_stride + w] >> base;
#pragma unroll
            for (int b = 0; b < 4; ++b) { ones[b] += (int)((v >> b) & 1u); }
        }
#pragma unroll
        for (int b = 0; b < 4; ++b) { out |= (2 * ones[b] > n) ? (1u << (base + b)) : 0u; }
    }
    y[(size_t)node * frame_stride + w] = (int)out;
}

// Reverse wiring for the backward pass, built on the device: for input node i, offsets[i] = number of table entries that
// name a smaller input, and list[offsets[i] ...] = the output nodes wired to i in table order (node ascending, input
// position ascending).  One thread per input node (plus one for the end offset) sweeps the whole table twice; the block
// stages the table through LDS in pieces, so a sweep is one coalesced load per piece and broadcast LDS reads.
// Entries outside [0, input_node_size) match no thread.
constexpr int kReversePiece = 2048;

// copy `count` table entries into LDS and fill up to the next multiple of four with -1, which matches no input node
__device__ __forceinline__ void stage_piece(int *piece, int const *__restrict__ src, int count)
{
    int const padded = (count + 3) & ~3;
    for (int k = threadIdx.x; k < padded; k += kTailBlock) { piece[k] = (k < count) ? src[k] : -1; }
}

// entry_ids: the list holds table positions (node * n + input position) instead of output nodes
__global__ __launch_bounds__(kTailBlock) void average_lut_reverse_kernel(int const *__restrict__ idx, int total, int n, int input_node_size,
                                                                         int *__restrict__ offsets, int *__restrict__ list, int entry_ids)
{
    __shared__ __attribute__((aligned(16))) int piece[kReversePiece];
    int const i = blockIdx.x * kTailBlock + threadIdx.x;
    bool const live = (i <= input_node_size);
    int below = 0;
    for (int base = 0; base < total; base += kReversePiece) {
        int const count = min(kReversePiece, total - base);
        __syncthreads();
        stage_piece(piece, idx + base, count);
        __syncthreads();
#pragma unroll 2
        for (int k = 0; k < count; k += 4) {
            int4 const e = *reinterpret_cast<int4 const *>(&piece[k]);
            below += ((uint32_t)e.x < (uint32_t)i) + ((uint32_t)e.y < (uint32_t)i) + ((uint32_t)e.z < (uint32_t)i) + ((uint32_t)e.w < (uint32_t)i);
        }
    }
    if (live) { offsets[i] = below; }
    int at = below;
    for (int base = 0; base < total; base += kReversePiece) {
        int const count = min(kReversePiece, total - base);
        __syncthreads();
        stage_piece(piece, idx + base, count);
        __syncthreads();
        if (live && i < input_node_size) {
#pragma unroll 2
            for (int k = 0; k < count; k += 4) {
                int4 const e = *reinterpret_cast<int4 const *>(&piece[k]);
                if (e.x == i) { list[at++] = entry_ids ? (base + k)     : (base + k) / n; }
                if (e.y == i) { list[at++] = entry_ids ? (base + k + 1) : (base + k + 1) / n; }
                if (e.z == i) { list[at++] = entry_ids ? (base + k + 2) : (base + k + 2) / n; }
                if (e.w == i) { list[at++] = entry_ids ? (base + k + 3) : (base + k + 3) / n; }
            }
        }
    }
}

// one thread per (input node, column of the row pitch): dx = sum over the wired output nodes, in table order, of dy / n
__global__ __launch_bounds__(kTailBlock) void average_lut_backward_kernel(float const *dy, float *dx, int const *offsets, int const *list,
                                                                          int n, int frame_size, int frame_stride, int f_blocks)
{
    int const f = (int)(blockIdx.x % f_blocks) * kTailBlock + threadIdx.x;
    int const in = blockIdx.x / f_blocks;
    if (f >= frame_stride) { return; }
    if (f >= frame_size) { dx[(size_t)in * frame_stride + f] = 0.0f; return; }      // the row's padding reads as zero, as after the host's FillZero
    int const begin = offsets[in], end = offsets[in + 1];
    float const fn = (float)n;
    float acc = 0.0f;
    for (int k = begin; k < end; ++k) { acc += dy[(size_t)list[k] * frame_stride + f] / fn; }
    dx[(size_t)in * frame_stride + f] = acc;
}

// The same for a table of at most kReversePiece entries, without the reverse wiring: every workgroup (one input node, kTailBlock
// columns) stages the whole table in LDS and walks it in table order; the comparison is the same for all its threads.  For the
// tails of classifiers (tens of entries) this saves the launch that builds the reverse wiring, which costs more than the walk.
__global__ __launch_bounds__(kTailBlock) void average_lut_backward_small_kernel(float const *dy, float *dx, int const *__restrict__ idx, int total,
                                                                                int n, int frame_size, int frame_stride, int f_blocks)
{
    __shared__ __attribute__((aligned(16))) int piece[kReversePiece];
    stage_piece(piece, idx, total);
    __syncthreads();
    int const f = (int)(blockIdx.x % f_blocks) * kTailBlock + threadIdx.x;
    int const in = blockIdx.x / f_blocks;
    if (f >= frame_stride) { return; }
    if (f >= frame_size) { dx[(size_t)in * frame_stride + f] = 0.0f; return; }
    float const fn = (float)n;
    float acc = 0.0f;
    for (int k = 0; k < total; ++k) {
        if (piece[k] == in) { acc += dy[(size_t)(k / n) * frame_stride + f] / fn; }
    }
    dx[(size_t)in * frame_stride + f] = acc;
}

// MaxLut: the largest of the n wired inputs, starting from -1 and replaced by strictly larger values only (reference host
// loop: include/bb/MaxLut.h:293-318); binarize_input as in the reference's device kernel (cuda/MaxLut.cu:33-36).
// One thread per (output node, frame).
__global__ __launch_bounds__(kTailBlock) void max_lut_forward_kernel(float const *x, float *y, int const *idx, int n, int frame_size,
                                                                     int frame_stride, int binarize_input, int binarize_output, int f_blocks)
{
    int const f = (int)(blockIdx.x % f_blocks) * kTailBlock + threadIdx.x;
    int const node = blockIdx.x / f_blocks;
    if (f >= frame_size) { return; }
    int const *row = idx + (size_t)node * n;
    float max_val = -1.0f;
    for (int i = 0; i < n; ++i) {
        float v = x[(size_t)row[i] * frame_stride + f];
        if (binarize_input) { v = (v > 0.0f) ? 1.0f : -1.0f; }
        if (v > max_val) { max_val = v; }
    }
    if (binarize_output) { max_val = (max_val > 0.0f) ? 1.0f : -1.0f; }
    y[(size_t)node * frame_stride + f] = max_val;
}

// packed bits, one thread per (output node, 32-frame word): the OR of the n input words
__global__ __launch_bounds__(kTailBlock) void max_lut_forward_bit_kernel(int const *x, int *y, int const *idx, int n, int words,
                                                                         int frame_stride, int w_blocks)
{
    int const w = (int)(blockIdx.x % w_blocks) * kTailBlock + threadIdx.x;
    int const node = blockIdx.x / w_blocks;
    if (w >= words) { return; }
    int const *row = idx + (size_t)node * n;
    uint32_t any = 0u;
    for (int i = 0; i < n; ++i) { any |= (uint32_t)x[(size_t)row[i] * frame_stride + w]; }
    y[(size_t)node * frame_stride + w] = (int)any;
}

// One thread per (input node, column of the dx row pitch): over the table positions that name this input, in table order, add
// the node's dy where this position holds the node's first largest input (include/bb/MaxLut.h:394-424).  BITS: x is packed, the
// first largest input is the first one that is set (position 0 when none is).
// the position of a node's first largest input at frame f (BITS: the first input that is set; position 0 when none is)
template <bool BITS>
__device__ __forceinline__ int max_lut_winner(void const *x_buf, int const *row, int n, int f, int x_stride, int binarize_input)
{
    int first = 0;
    if (BITS) {
        uint32_t const *xb = static_cast<uint32_t const *>(x_buf);
        for (int i = 0; i < n; ++i) {
            if ((xb[(size_t)row[i] * x_stride + (f >> 5)] >> (f & 31)) & 1u) { first = i; break; }
        }
    }
    else {
        float const *xf = static_cast<float const *>(x_buf);
        float max_val = -1.0f;
        for (int i = 0; i < n; ++i) {
            float v = xf[(size_t)row[i] * x_stride + f];
            if (binarize_input) { v = (v > 0.0f) ? 1.0f : -1.0f; }
            if (v > max_val) { max_val = v; first = i; }
        }
    }
    return first;
}

// One thread per (input node, column of the dx row pitch): over the table positions that name this input, in table order, add
// the node's dy where this position holds the node's first largest input (include/bb/MaxLut.h:394-424).
template <bool BITS>
__global__ __launch_bounds__(kTailBlock) void max_lut_backward_kernel(void const *x_buf, float const *dy, float *dx, int const *idx,
                                                                      int const *offsets, int const *list, int n, int frame_size,
                                                                      int x_stride, int dy_stride, int binarize_input, int f_blocks)
{
    int const f = (int)(blockIdx.x % f_blocks) * kTailBlock + threadIdx.x;
    int const in = blockIdx.x / f_blocks;
    if (f >= dy_stride) { return; }
    if (f >= frame_size) { dx[(size_t)in * dy_stride + f] = 0.0f; return; }         // the row's padding reads as zero, as after the host's FillZero
    int const begin = offsets[in], end = offsets[in + 1];
    float acc = 0.0f;
    for (int k = begin; k < end; ++k) {
        int const entry = list[k], node = entry / n, pos = entry - node * n;
        if (max_lut_winner<BITS>(x_buf, idx + (size_t)node * n, n, f, x_stride, binarize_input) == pos) { acc += dy[(size_t)node * dy_stride + f]; }
    }
    dx[(size_t)in * dy_stride + f] = acc;
}

// the same for a table of at most kReversePiece entries, walked from LDS without the reverse wiring (see average_lut_backward_small_kernel)
template <bool BITS>
__global__ __launch_bounds__(kTailBlock) void max_lut_backward_small_kernel(void const *x_buf, float const *dy, float *dx, int const *__restrict__ idx,
                                                                            int total, int n, int frame_size, int x_stride, int dy_stride,
                                                                            int binarize_input, int f_blocks)
{
    __shared__ __attribute__((aligned(16))) int piece[kReversePiece];
    stage_piece(piece, idx, total);
    __syncthreads();
    int const f = (int)(blockIdx.x % f_blocks) * kTailBlock + threadIdx.x;
    int const in = blockIdx.x / f_blocks;
    if (f >= dy_stride) { return; }
    if (f >= frame_size) { dx[(size_t)in * dy_stride + f] = 0.0f; return; }
    float acc = 0.0f;
    for (int k = 0; k < total; ++k) {
        if (piece[k] != in) { continue; }
        int const node = k / n, pos = k - node * n;
        if (max_lut_winner<BITS>(x_buf, piece + node * n, n, f, x_stride, binarize_input) == pos) { acc += dy[(size_t)node * dy_stride + f]; }
    }
    dx[(size_t)in * dy_stride + f] = acc;
}

// Reduce: output node o is the mean of the input nodes o, O + o, 2 O + o, ... (reference host loop: include/bb/Reduce.h:172-190;
// the reference has no device code for this layer).  One thread per (output node, frame); BITS: packed input read as +1 / -1.
template <bool BITS>
__global__ __launch_bounds__(kTailBlock) void reduce_forward_kernel(void const *x_buf, float *y, int mux, int output_node_size, int frame_size,
                                                                    int x_stride, int y_stride, int f_blocks)
{
    int const f = (int)(blockIdx.x % f_blocks) * kTailBlock + threadIdx.x;
    int const o = blockIdx.x / f_blocks;
    if (f >= frame_size) { return; }
    float sum = 0.0f;
    for (int i = 0; i < mux; ++i) {
        size_t const row = (size_t)output_node_size * i + o;
        if (BITS) { sum += ((static_cast<uint32_t const *>(x_buf)[row * x_stride + (f >> 5)] >> (f & 31)) & 1u) ? 1.0f : -1.0f; }
        else      { sum += static_cast<float const *>(x_buf)[row * x_stride + f]; }
    }
    y[(size_t)o * y_stride + f] = sum / (float)mux;
}

// dx[input node] = dy[input node mod O] / mux (include/bb/Reduce.h:229-247); one thread per (input node, frame)
__global__ __launch_bounds__(kTailBlock) void reduce_backward_kernel(float const *dy, float *dx, int mux, int output_node_size, int frame_size,
                                                                     int frame_stride, int f_blocks)
{
    int const f = (int)(blockIdx.x % f_blocks) * kTailBlock + threadIdx.x;
    int const in = blockIdx.x / f_blocks;
    if (f >= frame_size) { return; }
    dx[(size_t)in * frame_stride + f] = dy[(size_t)(in % output_node_size) * frame_stride + f] / (float)mux;
}

// Mean squared error.  One thread per (group of kMseNodes nodes, frame): dy = (y - t) * grad_scale, and the group's share of the
// frame's loss, node ascending, in double: partial[group][frame] = sum of (float)(y - t)^2 * loss_scale (LOSS: NaN squares left
// out, as the reference's loss does, include/bb/LossMeanSquaredError.h:150-169; else sum of (float)(t - y)^2 / node_size, as its
// metric, MetricsMeanSquaredError.h:66-85).
constexpr int kMseNodes = 64;

template <bool LOSS>
__global__ __launch_bounds__(kTailBlock) void mean_squared_error_kernel(float const *y, float const *t, float *dy, double *partial,
                                                                        float grad_scale, double loss_scale, int node_size, int frame_size,
                                                                        int frame_stride, int f_blocks)
{
    int const f = (int)(blockIdx.x % f_blocks) * kTailBlock + threadIdx.x;
    int const group = blockIdx.x / f_blocks;
    if (f >= frame_size) { return; }
    int const first = group * kMseNodes, last = min(first + kMseNodes, node_size);
    double acc = 0.0;
    for (int node = first; node < last; ++node) {
        size_t const at = (size_t)node * frame_stride + f;
        if (LOSS) {
            float const grad = y[at] - t[at];
            float const error = rounded_mul(grad, grad);
            dy[at] = rounded_mul(grad, grad_scale);
            if (error == error) { acc += (double)error * loss_scale; }
        }
        else {
            float const grad = t[at] - y[at];
            acc += (double)rounded_mul(grad, grad) / loss_scale;
        }
    }
    partial[(size_t)group * frame_size + f] = acc;
}

// buf[s] += the partial sums of the frames s, s + buf_size, s + 2 buf_size, ...: frames ascending, groups ascending within a frame
__global__ __launch_bounds__(kTailBlock) void mean_squared_error_sum_kernel(double const *partial, double *buf, int buf_size, int groups,
                                                                            int frame_size)
{
    int const s = blockIdx.x * kTailBlock + threadIdx.x;
    if (s >= buf_size || s >= frame_size) { return; }
    double acc = 0.0;
    for (int f = s; f < frame_size; f += buf_size) {
        for (int g = 0; g < groups; ++g) { acc += partial[(size_t)g * frame_size + f]; }
    }
    buf[s] += acc;
}

// Softmax cross entropy, one thread per (pixel, frame); node = ch * pix_size + pix.  partial[pix * frame_size + frame]
// receives sum over the channels with t > 0 of log(softmax + eps) * t_max in double; with one pixel that is loss_buf itself.
__global__ __launch_bounds__(kTailBlock) void softmax_cross_entropy_kernel(float const *y, float const *t, float *dy, double *partial,
                                                                           float t_sum, int pix_size, int ch_size, int frame_size,
                                                                           int frame_stride, int f_blocks)
{
    int const f = (int)(blockIdx.x % f_blocks) * kTailBlock + threadIdx.x;
    int const pix = blockIdx.x / f_blocks;
    if (f >= frame_size) { return; }
    float const eps = 1.0e-7f;
    size_t const node_step = (size_t)pix_size * frame_stride;
    size_t const first = (size_t)pix * frame_stride + f;
    float c = -3.402823466e+38f;
    for (int ch = 0; ch < ch_size; ++ch) {
        float const v = y[first + ch * node_step];
        c = (c < v) ? v : c;
    }
    float y_sum = 0.0f, t_max = 0.0f;
    for (int ch = 0; ch < ch_size; ++ch) {
        y_sum += expf(y[first + ch * node_step] - c);
        t_max += t[first + ch * node_step];
    }
    if (y_sum <= eps) { y_sum = eps; }
    double loss = 0.0;
    for (int ch = 0; ch < ch_size; ++ch) {
        size_t const at = first + ch * node_step;
        float const tv = t[at];
        float const softmax = expf(y[at] - c) / y_sum;
        if (tv > 0.0f) { loss += (double)rounded_mul(logf(softmax + eps), t_max); }
        dy[at] = (rounded_mul(t_max, softmax) - tv) / t_sum;
    }
    partial[(size_t)pix * frame_size + f] = loss;
}

// The same arithmetic for at most CH channels with every y and t of the (pixel, frame) loaded first: the loads of the three passes
// above depend on nothing, but issued one pass after the other their latencies add up, which is what a small batch pays for.
template <int CH>
__global__ __launch_bounds__(kTailBlock) void softmax_cross_entropy_few_kernel(float const *y, float const *t, float *dy, double *partial,
                                                                               float t_sum, int pix_size, int ch_size, int frame_size,
                                                                               int frame_stride, int f_blocks)
{
    int const f = (int)(blockIdx.x % f_blocks) * kTailBlock + threadIdx.x;
    int const pix = blockIdx.x / f_blocks;
    if (f >= frame_size) { return; }
    float const eps = 1.0e-7f;
    size_t const node_step = (size_t)pix_size * frame_stride;
    size_t const first = (size_t)pix * frame_stride + f;
    float yv[CH], tv[CH];
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
        yv[ch] = (ch < ch_size) ? y[first + ch * node_step] : 0.0f;
        tv[ch] = (ch < ch_size) ? t[first + ch * node_step] : 0.0f;
    }
    float c = -3.402823466e+38f;
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) { if (ch < ch_size) { c = (c < yv[ch]) ? yv[ch] : c; } }
    float y_sum = 0.0f, t_max = 0.0f;
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
        if (ch < ch_size) {
            yv[ch] = expf(yv[ch] - c);
            y_sum += yv[ch];
            t_max += tv[ch];
        }
    }
    if (y_sum <= eps) { y_sum = eps; }
    double loss = 0.0;
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
        if (ch < ch_size) {
            float const softmax = yv[ch] / y_sum;
            if (tv[ch] > 0.0f) { loss += (double)rounded_mul(logf(softmax + eps), t_max); }
            dy[first + ch * node_step] = (rounded_mul(t_max, softmax) - tv[ch]) / t_sum;
        }
    }
    partial[(size_t)pix * frame_size + f] = loss;
}

// The whole tail of a LUT classifier in one launch: AverageLut forward over the last layer's output (un-binarized: the logits), softmax
// cross entropy against t, categorical accuracy, and the AverageLut backward pass of the loss gradient — four launches of a few
// microseconds each when called one by one, which at training batch sizes cost their launch latencies rather than their work.
// A workgroup of kClassifierTailWaves wavefronts owns 64 frames of ALL nodes, one frame per lane.
//   1. the table is staged in LDS;
//   2. wavefront w computes the logits of the channels ch = w, w + waves, ...: the sum of the channel's n inputs in table order, times
//      `scale` (as average_lut_forward_kernel), eight loads in flight at a time, and leaves them in LDS;
//   3. every wavefront takes all logits and computes the loss terms (as softmax_cross_entropy_few_kernel, pix_size 1) and the accuracy
//      (as categorical_accuracy_kernel) — the same values in each, cheaper than a second exchange; wavefront 0 stores them;
//   4. the gradient dy / n of every logit goes through the table once more, in table order, into per-input sums in LDS
//      (acc[input][lane] += dy[node] / n: the order of the host loop, include/bb/AverageLut.h:395-404, and of
//      average_lut_backward_kernel); wavefront w takes the inputs with input % waves == w, so the chain of dependent LDS updates is a
//      quarter as long, and writes their rows.
// Columns between frame_size and frame_stride of dx are written as 0, as the backward kernels do.  Same bits as the four entries called
// one after the other.  LDS: (input_node_size + 2 CH) x 64 floats + the table (padded to a multiple of four entries).
constexpr int kClassifierTailWaves = 4;

template <int CH>
__global__ __launch_bounds__(64 * kClassifierTailWaves) void classifier_tail_kernel(float const *__restrict__ x, float *__restrict__ y, float *__restrict__ dx,
                                                             int const *__restrict__ idx, float const *__restrict__ t,
                                                             float *__restrict__ dy_out, double *__restrict__ loss_buf,
                                                             int *__restrict__ accuracy_buf, int *__restrict__ category_buf,
                                                             float t_sum, float scale, int n, int input_node_size, int ch_size,
                                                             int frame_size, int frame_stride, int binarize_input)
{
    extern __shared__ __attribute__((aligned(16))) float tail_lds[];
    constexpr int WAVES = kClassifierTailWaves;
    int const lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int const total = ch_size * n, padded = (total + 3) & ~3;
    float *acc   = tail_lds;                                                    // [input_node_size][64]
    float *logit = tail_lds + (size_t)input_node_size * 64;                     // [CH][64]
    float *dyn   = logit + CH * 64;                                             // [CH][64]: dy / n of the lane's frame
    int *piece   = reinterpret_cast<int *>(dyn + CH * 64);                      // [padded]: the table
    int const f = blockIdx.x * 64 + lane;
    bool const in_row = f < frame_stride, live = f < frame_size;
    int const fc = live ? f : 0;                                                // (a lane without a frame loads frame 0 and stores nothing)
    for (int k = threadIdx.x; k < padded; k += 64 * WAVES) { piece[k] = (k < total) ? idx[k] : -1; }
    // the targets do not depend on anything computed here: requested ahead of the logits
    float tv[CH];
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) { tv[ch] = (ch < ch_size) ? t[(size_t)ch * frame_stride + fc] : 0.0f; }
    __syncthreads();
    {
        // the wavefront's channels together, so that their loads are in flight together (a channel's sum stays in table order)
        constexpr int PER = (CH + WAVES - 1) / WAVES;
        float sum[PER];
        int const *row[PER];
#pragma unroll
        for (int q = 0; q < PER; ++q) {
            int const ch = wave + q * WAVES;
            sum[q] = 0.0f;
            row[q] = piece + ((ch < ch_size) ? ch : 0) * n;         // (a channel that does not exist reads channel 0's rows and stores nothing)
        }
        for (int i0 = 0; i0 < n; i0 += 8) {
            float v[PER][8];
#pragma unroll
            for (int q = 0; q < PER; ++q) {
#pragma unroll
                for (int j = 0; j < 8; ++j) { v[q][j] = x[(size_t)row[q][(i0 + j < n) ? i0 + j : 0] * frame_stride + fc]; }
            }
#pragma unroll
            for (int q = 0; q < PER; ++q) {
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    if (i0 + j < n) {
                        float u = v[q][j];
                        if (binarize_input) { u = (u > 0.0f) ? 1.0f : -1.0f; }
                        sum[q] += u;
                    }
                }
            }
        }
#pragma unroll
        for (int q = 0; q < PER; ++q) {
            int const ch = wave + q * WAVES;
            if (ch < ch_size) {
                float const out = rounded_mul(sum[q], scale);
                logit[ch * 64 + lane] = out;
                if (live && y != nullptr) { y[(size_t)ch * frame_stride + f] = out; }
            }
        }
    }
    __syncthreads();
    float const eps = 1.0e-7f;
    bool const first = (wave == 0) && live;
    float yv[CH];
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) { yv[ch] = (ch < ch_size) ? logit[ch * 64 + lane] : 0.0f; }
    // accuracy: the first largest logit sits on a channel with a positive target (one pixel per frame)
    if (first) {
        float max_y = -3.402823466e+38f, max_t = -3.402823466e+38f;
        bool valid = false;
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) {
            if (ch < ch_size) {
                valid = valid || (tv[ch] > 0.0f);
                if (yv[ch] > max_y) { max_y = yv[ch]; max_t = tv[ch]; }
            }
        }
        if (accuracy_buf != nullptr) { accuracy_buf[f] = (valid && max_t > 0.0f) ? 1 : 0; }
        if (category_buf != nullptr) { category_buf[f] = valid ? 1 : 0; }
    }
    // softmax cross entropy
    float c = -3.402823466e+38f;
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) { if (ch < ch_size) { c = (c < yv[ch]) ? yv[ch] : c; } }
    float y_sum = 0.0f, t_max = 0.0f;
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
        if (ch < ch_size) {
            yv[ch] = expf(yv[ch] - c);
            y_sum += yv[ch];
            t_max += tv[ch];
        }
    }
    if (y_sum <= eps) { y_sum = eps; }
    double loss = 0.0;
    float const fn = (float)n;
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
        if (ch < ch_size) {
            float const softmax = yv[ch] / y_sum;
            if (tv[ch] > 0.0f) { loss += (double)rounded_mul(logf(softmax + eps), t_max); }
            float const g = (rounded_mul(t_max, softmax) - tv[ch]) / t_sum;
            if (first && dy_out != nullptr) { dy_out[(size_t)ch * frame_stride + f] = g; }
            dyn[ch * 64 + lane] = g / fn;           // (every wavefront writes the same values; each reads them after its own writes)
        }
    }
    if (first) { loss_buf[f] = loss; }
    // backward through the table, in table order; a lane only ever touches its own column of acc and dyn
    for (int in = wave; in < input_node_size; in += WAVES) { acc[in * 64 + lane] = 0.0f; }
    int node = 0, pos = 0;
    for (int k = 0; k < padded; k += 4) {
        int4 const e4 = *reinterpret_cast<int4 const *>(&piece[k]);
        int const e[4] = {e4.x, e4.y, e4.z, e4.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int const in = e[j];                            // the same for every lane
            if ((unsigned)in < (unsigned)input_node_size && (in % WAVES) == wave) { acc[in * 64 + lane] += dyn[node * 64 + lane]; }
            if (++pos == n) { pos = 0; ++node; }
        }
    }
    if (in_row) {
        for (int in = wave; in < input_node_size; in += WAVES) { dx[(size_t)in * frame_stride + f] = live ? acc[in * 64 + lane] : 0.0f; }
    }
}

// loss_buf[frame] = sum over the pixels, ascending, of the per-pixel terms
__global__ __launch_bounds__(kTailBlock) void loss_pixel_sum_kernel(double const *partial, double *loss_buf, int pix_size, int frame_size)
{
    int const f = blockIdx.x * kTailBlock + threadIdx.x;
    if (f >= frame_size) { return; }
    double loss = 0.0;
    for (int pix = 0; pix < pix_size; ++pix) { loss += partial[(size_t)pix * frame_size + f]; }
    loss_buf[f] = loss;
}

// Per frame: pixels with a positive target (category) and, of those, pixels whose first largest y sits on a channel with
// a positive target (accuracy).  One thread per frame.
__global__ __launch_bounds__(kTailBlock) void categorical_accuracy_kernel(float const *y, float const *t, int *accuracy_buf, int *category_buf,
                                                                          int pix_size, int ch_size, int frame_size, int frame_stride)
{
    int const f = blockIdx.x * kTailBlock + threadIdx.x;
    if (f >= frame_size) { return; }
    size_t const node_step = (size_t)pix_size * frame_stride;
    int accuracy = 0, category = 0;
    for (int pix = 0; pix < pix_size; ++pix) {
        size_t const first = (size_t)pix * frame_stride + f;
        float max_y = -3.402823466e+38f, max_t = -3.402823466e+38f;
        bool valid = false;
        for (int ch = 0; ch < ch_size; ++ch) {
            float const yv = y[first + ch * node_step], tv = t[first + ch * node_step];
            valid = valid || (tv > 0.0f);
            if (yv > max_y) { max_y = yv; max_t = tv; }
        }
        if (valid) { category += 1; accuracy += (max_t > 0.0f) ? 1 : 0; }
    }
    accuracy_buf[f] = accuracy;
    category_buf[f] = category;
}

}  // namespace bbhip

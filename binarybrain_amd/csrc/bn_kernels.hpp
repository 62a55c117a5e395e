// StochasticBatchNormalization: every node (a row of frames) is normalised with its own batch statistics and then mapped by
// one scalar gamma and beta — the unfused form of the normalisation inside DifferentiableLutN
// (reference: include/bb/StochasticBatchNormalization.h: training forward :535-597, re-forward :655-678, backward :815-851;
// entry points include/bbcu/bbcu.h:883-942).
//
// Streaming work over node-major, frame-minor rows: a row belongs to one workgroup, which reads it once with 128-bit
// loads, keeps it in registers (rows of up to kBnBlock * 4 * kBnHeld frames), forms the mean, then the variance about
// that mean (two passes over the registers, as the reference's two loops over the row), and writes the output: 4 bytes
// read and 4 written per element, the minimum.  Longer rows are read again for each pass; a row is at most a few
// hundred KB then and stays in L2 between the passes.  Sums are taken lane-wise, then across the wavefront, then across
// the workgroup's wavefronts in a fixed order: the same input gives the same bits on every run, and results differ from the
// reference's frame-order sums only in rounding.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "lut_kernels.hpp"

namespace bbhip {

constexpr int kBnBlock     = 256;       // rows kept in registers, and the elementwise passes
constexpr int kBnLongBlock = 1024;      // rows that are read once per pass: four times the loads in flight per row
constexpr int kBnHeld      = 8;         // float4 (W = 4) or float (W = 1) values a thread keeps of its row

struct BnArgs {
    float const *x;
    float const *dy;            // backward only
    float       *out;           // y or dx
    float       *mean;          // batch statistics: written by the training pass, read by re-forward and backward
    float       *rstd;
    float       *running_mean;  // training: updated; inference: read
    float       *running_var;
    float gamma, beta, momentum, reciprocal_frame_size;
    int   frame_size, x_stride, out_stride;
};

// the sum of v over the workgroup of BLOCK threads, the same value in every thread; `share` holds one float per wavefront
template <int BLOCK>
__device__ __forceinline__ float bn_block_sum(float v, float *share)
{
    v = wave_sum(v);
    __syncthreads();                                    // the previous sum has been read by everyone
    if ((threadIdx.x & (kWave - 1)) == 0) { share[threadIdx.x / kWave] = v; }
    __syncthreads();
    float s = 0.0f;
#pragma unroll
    for (int w = 0; w < BLOCK / kWave; ++w) { s += share[w]; }
    return s;
}

// W consecutive frames starting at f: one 128-bit access where all of them exist, else frame by frame (absent ones read 0)
template <int W>
__device__ __forceinline__ void bn_load(float const *__restrict__ row, int f, int frame_size, float (&v)[W])
{
    if constexpr (W == 4) {
        if (f + 3 < frame_size) {
            float4 const t = *reinterpret_cast<float4 const *>(row + f);
            v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
            return;
        }
    }
#pragma unroll
    for (int j = 0; j < W; ++j) { v[j] = (f + j < frame_size) ? row[f + j] : 0.0f; }
}

template <int W>
__device__ __forceinline__ void bn_store(float *__restrict__ row, int f, int frame_size, float const (&v)[W])
{
    if constexpr (W == 4) {
        if (f + 3 < frame_size) {
            *reinterpret_cast<float4 *>(row + f) = make_float4(v[0], v[1], v[2], v[3]);
            return;
        }
    }
#pragma unroll
    for (int j = 0; j < W; ++j) { if (f + j < frame_size) { row[f + j] = v[j]; } }
}

// Training forward, one workgroup per node.  HELD: the row is kept in registers (frame_size <= kBnBlock * W * kBnHeld,
// kBnBlock threads); otherwise it is read once per pass, by kBnLongBlock threads.
template <int W, bool HELD>
__global__ __launch_bounds__(HELD ? kBnBlock : kBnLongBlock) void bn_forward_training_kernel(BnArgs a)
{
    constexpr int BLOCK = HELD ? kBnBlock : kBnLongBlock;
    __shared__ float share[BLOCK / kWave];
    int const node = blockIdx.x;
    float const *__restrict__ xr = a.x + (size_t)node * a.x_stride;
    float *__restrict__ yr = a.out + (size_t)node * a.out_stride;
    int const F = a.frame_size;
    constexpr int kStep = BLOCK * W;
    int const f0 = threadIdx.x * W;

    float v[HELD ? kBnHeld : 1][W];
    float s = 0.0f;
    if (HELD) {
#pragma unroll
        for (int r = 0; r < kBnHeld; ++r) { bn_load<W>(xr, f0 + r * kStep, F, v[r]); }
#pragma unroll
        for (int r = 0; r < kBnHeld; ++r) {
#pragma unroll
            for (int j = 0; j < W; ++j) { s += v[r][j]; }
        }
    }
    else {
        for (int f = f0; f < F; f += kStep) {
            bn_load<W>(xr, f, F, v[0]);
#pragma unroll
            for (int j = 0; j < W; ++j) { s += v[0][j]; }
        }
    }
    float const mean = bn_block_sum<BLOCK>(s, share) / (float)F;

    float q = 0.0f;
    if (HELD) {
#pragma unroll
        for (int r = 0; r < kBnHeld; ++r) {
#pragma unroll
            for (int j = 0; j < W; ++j) {
                float const xc = (f0 + r * kStep + j < F) ? v[r][j] - mean : 0.0f;
                q = __builtin_fmaf(xc, xc, q);
            }
        }
    }
    else {
        for (int f = f0; f < F; f += kStep) {
            bn_load<W>(xr, f, F, v[0]);
#pragma unroll
            for (int j = 0; j < W; ++j) {
                float const xc = (f + j < F) ? v[0][j] - mean : 0.0f;
                q = __builtin_fmaf(xc, xc, q);
            }
        }
    }
    float const var  = fmaxf(0.0f, bn_block_sum<BLOCK>(q, share) / (float)F);
    float const rstd = 1.0f / (sqrtf(var) + 1.0e-7f);

    if (threadIdx.x == 0) {
        a.running_mean[node] = a.running_mean[node] * a.momentum + mean * (1.0f - a.momentum);
        a.running_var[node]  = a.running_var[node]  * a.momentum + var  * (1.0f - a.momentum);
        a.mean[node] = mean;
        a.rstd[node] = rstd;
    }

    if (HELD) {
#pragma unroll
        for (int r = 0; r < kBnHeld; ++r) {
#pragma unroll
            for (int j = 0; j < W; ++j) { v[r][j] = ((v[r][j] - mean) * rstd) * a.gamma + a.beta; }
            bn_store<W>(yr, f0 + r * kStep, F, v[r]);
        }
    }
    else {
        for (int f = f0; f < F; f += kStep) {
            bn_load<W>(xr, f, F, v[0]);
#pragma unroll
            for (int j = 0; j < W; ++j) { v[0][j] = ((v[0][j] - mean) * rstd) * a.gamma + a.beta; }
            bn_store<W>(yr, f, F, v[0]);
        }
    }
}

// y = ((x - mean) * rstd) * gamma + beta with given statistics: re-forward (mean / rstd of the training pass) and
// inference (FROM_RUNNING: mean = running mean, rstd = 1 / (sqrt(running var) + 1e-7)).  One thread per W frames.
template <int W, bool FROM_RUNNING>
__global__ __launch_bounds__(kBnBlock) void bn_apply_kernel(BnArgs a, int f_blocks)
{
    int const node = blockIdx.x / f_blocks;
    int const f = ((int)(blockIdx.x % f_blocks) * kBnBlock + threadIdx.x) * W;
    if (f >= a.frame_size) { return; }
    float mean, rstd;
    if (FROM_RUNNING) { mean = a.running_mean[node]; rstd = 1.0f / (sqrtf(a.running_var[node]) + 1.0e-7f); }
    else              { mean = a.mean[node];         rstd = a.rstd[node]; }
    float v[W];
    bn_load<W>(a.x + (size_t)node * a.x_stride, f, a.frame_size, v);
#pragma unroll
    for (int j = 0; j < W; ++j) { v[j] = ((v[j] - mean) * rstd) * a.gamma + a.beta; }
    bn_store<W>(a.out + (size_t)node * a.out_stride, f, a.frame_size, v);
}

// Backward, one workgroup per node: with dxn = gamma dy and xc = x - mean,
//   dstd = -sum dxn xc rstd^2,  dmeanx = -sum dxn rstd,  dvar = dstd rstd,  dmean = (dmeanx - mean dvar) / F,
//   dx = dxn rstd + dmean + x dvar / F.
template <int W, bool HELD>
__global__ __launch_bounds__(HELD ? kBnBlock : kBnLongBlock) void bn_backward_kernel(BnArgs a)
{
    constexpr int BLOCK = HELD ? kBnBlock : kBnLongBlock;
    __shared__ float share[BLOCK / kWave];
    int const node = blockIdx.x;
    float const *__restrict__ xr  = a.x  + (size_t)node * a.x_stride;
    float const *__restrict__ dyr = a.dy + (size_t)node * a.out_stride;
    float *__restrict__ dxr = a.out + (size_t)node * a.out_stride;
    int const F = a.frame_size;
    constexpr int kStep = BLOCK * W;
    int const f0 = threadIdx.x * W;
    float const mean = a.mean[node], rstd = a.rstd[node];
    float const rstd2 = rstd * rstd;

    float xv[HELD ? kBnHeld : 1][W], gv[HELD ? kBnHeld : 1][W];
    float s_std = 0.0f, s_mean = 0.0f;
    if (HELD) {
#pragma unroll
        for (int r = 0; r < kBnHeld; ++r) { bn_load<W>(xr, f0 + r * kStep, F, xv[r]); bn_load<W>(dyr, f0 + r * kStep, F, gv[r]); }
#pragma unroll
        for (int r = 0; r < kBnHeld; ++r) {
#pragma unroll
            for (int j = 0; j < W; ++j) {
                float const dxn = a.gamma * gv[r][j];               // 0 for frames that do not exist
                s_std  -= (dxn * (xv[r][j] - mean)) * rstd2;
                s_mean -= dxn * rstd;
            }
        }
    }
    else {
        for (int f = f0; f < F; f += kStep) {
            bn_load<W>(xr, f, F, xv[0]); bn_load<W>(dyr, f, F, gv[0]);
#pragma unroll
            for (int j = 0; j < W; ++j) {
                float const dxn = a.gamma * gv[0][j];
                s_std  -= (dxn * (xv[0][j] - mean)) * rstd2;
                s_mean -= dxn * rstd;
            }
        }
    }
    float const dstd   = bn_block_sum<BLOCK>(s_std, share);
    float const dmeanx = bn_block_sum<BLOCK>(s_mean, share);
    float const dvar   = dstd * rstd;
    float const dmean  = (dmeanx - mean * dvar) * a.reciprocal_frame_size;

    if (HELD) {
#pragma unroll
        for (int r = 0; r < kBnHeld; ++r) {
#pragma unroll
            for (int j = 0; j < W; ++j) { gv[r][j] = ((gv[r][j] * a.gamma) * rstd + dmean) + (xv[r][j] * dvar) * a.reciprocal_frame_size; }
            bn_store<W>(dxr, f0 + r * kStep, F, gv[r]);
        }
    }
    else {
        for (int f = f0; f < F; f += kStep) {
            bn_load<W>(xr, f, F, xv[0]); bn_load<W>(dyr, f, F, gv[0]);
#pragma unroll
            for (int j = 0; j < W; ++j) { gv[0][j] = ((gv[0][j] * a.gamma) * rstd + dmean) + (xv[0][j] * dvar) * a.reciprocal_frame_size; }
            bn_store<W>(dxr, f, F, gv[0]);
        }
    }
}

}  // namespace bbhip

// HIP kernels of the differentiable-LUT path for gfx950 (wave64).
//
// Data layout (the FrameBuffer layout of the reference, include/bb/FrameBuffer.h:28-46): node-major, frame-minor.
// Element (node n, frame f) of an fp32 buffer is p[n*stride + f]; of a packed buffer, bit (f & 31) of word
// p[n*stride_words + (f >> 5)].  A wavefront always works on 64 consecutive frames of ONE output node: the node's
// table and its N connection indices are wave-uniform (scalar registers / scalar loads), the N gathered input rows
// are read as coalesced 256-byte segments, and the result row is written the same way.
//
// Work decomposition: a *unit* is (output node, chunk of frames); a workgroup of 4 waves takes 4 consecutive nodes of
// one chunk.  Workgroups are numbered so that the ones an XCD receives (hardware deals consecutive workgroup ids
// round-robin over the 8 XCDs) cover a contiguous range of chunks: every input row segment is then gathered by one
// XCD only and the ~N-fold re-reads of a row by its consumers are served by that XCD's L2.
#pragma once

#include "lut_math.hpp"
#include "tile_divisor.hpp"

namespace bbhip {

constexpr int kBlock        = 256;                 // threads per workgroup
constexpr int kWavesPerBlk  = kBlock / kWave;      // = nodes per workgroup
constexpr int kXcd          = 8;

// logical workgroup index for hardware workgroup id b of a grid of B: XCD x (= b % 8) owns a contiguous range
__device__ __forceinline__ int xcd_remap(int b, int B)
{
    // (unsigned: the shifts and masks of a division by 8 without the sign fix-ups, which cost the scalar unit a dozen instructions)
    uint32_t const q = (uint32_t)B / kXcd, r = (uint32_t)B % kXcd;
    uint32_t const x = (uint32_t)b % kXcd, k = (uint32_t)b / kXcd;
    return (int)(x * q + (x < r ? x : r) + k);
}

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) { v += __shfl_xor(v, o, 64); }
    return v;
}

// ------------------------------------------------------------------------------------------------
//  table preparation from W' (W' = lut_binarize ? W > 0.5 : W):
//    C = coefficients in the centred monomial basis,  y = sum_S C[S] prod_{j in S} (x_j - 1/2)
//  (the plain-basis coefficients P,  y = sum_S P[S] prod_{j in S} x_j,  are formed inside term_table_block)
// ------------------------------------------------------------------------------------------------
//  For two-valued inputs (x_j = 1/2 -+ bias) the layer is a table of 2^N values, V[p] = y at the corner whose bit j says
//  which value input j takes: one more butterfly over C, (a, b) -> (a - bias b, a + bias b) per variable.
//  clamp_W != nullptr: the table is first clamped to [clamp_lo, clamp_hi] and written back there (the model classes clamp
//  their table in place before every forward pass, include/bb/StochasticLutN.h:451; folded in here the clamp costs no
//  launch of its own).  clamp_W is W itself, so neither pointer is declared unaliased.
// entry i of a table held by 2^N neighbouring lanes: W' -> centred coefficients, (a, b) -> ((a + b) / 2, b - a) per index bit ...
template <int N>
__device__ __forceinline__ float centred_butterfly(float v, int i)
{
#pragma unroll
    for (int j = 0; j < N; ++j) {
        float const o = __shfl_xor(v, 1 << j, 64);
        v = ((i >> j) & 1) ? (v - o) : (v + o) * 0.5f;
    }
    return v;
}

// ... and centred coefficients -> corner values, (a, b) -> (a - bias b, a + bias b) per index bit
template <int N>
__device__ __forceinline__ float corner_butterfly(float v, int i, float bias)
{
#pragma unroll
    for (int j = 0; j < N; ++j) {
        float const o = __shfl_xor(v, 1 << j, 64);
        v = ((i >> j) & 1) ? __builtin_fmaf(bias, v, o) : __builtin_fmaf(-bias, o, v);
    }
    return v;
}

template <int N>
__device__ __forceinline__ void table_prep_block(float const *W, float *__restrict__ C, int node_size, int lut_binarize,
                                                 float *__restrict__ V, float bias, int block,
                                                 float *clamp_W = nullptr, float clamp_lo = 0.0f, float clamp_hi = 0.0f)
{
    constexpr int NN = 1 << N;
    int const t = block * kBlock + threadIdx.x;
    int const total = node_size * NN;
    float v = 0.0f;
    if (t < total) {
        v = W[t];
        if (clamp_W != nullptr) {
            float const w = fminf(clamp_hi, fmaxf(clamp_lo, v));        // as clamp_kernel
            if (w != v) { clamp_W[t] = w; }
            v = w;
        }
        if (lut_binarize) { v = (v > 0.5f) ? 1.0f : 0.0f; }
    }
    int const i = t & (NN - 1);
    v = centred_butterfly<N>(v, i);
    if (t < total) { C[t] = v; }
    if (V == nullptr) { return; }           // same for every thread of the launch
    v = corner_butterfly<N>(v, i, bias);
    if (t < total) { V[t] = v; }
}

template <int N>
__global__ __launch_bounds__(kBlock) void table_prep_kernel(float const *W, float *__restrict__ C,
                                                           int node_size, int lut_binarize,
                                                           float *__restrict__ V = nullptr, float bias = 0.0f,
                                                           float *clamp_W = nullptr, float clamp_lo = 0.0f, float clamp_hi = 0.0f)
{
    table_prep_block<N>(W, C, node_size, lut_binarize, V, bias, blockIdx.x, clamp_W, clamp_lo, clamp_hi);
}

// dW[node][i] += (T^T sum_s partial[s][node])[i]   (T = the butterfly above; deterministic slab order); overwrite: = instead of +=
template <int N>
__device__ __forceinline__ void dw_finalize_block(float const *__restrict__ partial, float *__restrict__ dW, int node_size, int slab_count, int block,
                                                  int overwrite = 0)
{
    constexpr int NN = 1 << N;
    int const t = block * kBlock + threadIdx.x;
    int const total = node_size * NN;
    float v = 0.0f;
    if (t < total) {
#pragma unroll 8
        for (int s = 0; s < slab_count; ++s) { v += partial[(size_t)s * total + t]; }
    }
    int const i = t & (NN - 1);
#pragma unroll
    for (int j = 0; j < N; ++j) {
        float const o = __shfl_xor(v, 1 << j, 64);
        v = ((i >> j) & 1) ? (o * 0.5f + v) : (v * 0.5f - o);
    }
    if (t < total) { dW[t] = overwrite ? v : dW[t] + v; }
}

template <int N>
__global__ __launch_bounds__(kBlock) void dw_finalize_kernel(float const *__restrict__ partial, float *__restrict__ dW,
                                                            int node_size, int slab_count, int overwrite)
{
    dw_finalize_block<N>(partial, dW, node_size, slab_count, blockIdx.x, overwrite);
}

// ------------------------------------------------------------------------------------------------
//  gather of one frame's inputs
// ------------------------------------------------------------------------------------------------
template <int N, int XMODE>
struct Gather {
    using Raw = uint32_t;

    // rows[k]: wave-uniform pointer to the input row of connection k.  f0 is the wavefront step's first frame; the
    // frame index of a lane is clamped into the buffer, so every lane loads unconditionally and the N loads are
    // issued back to back.
    // The element offset is an unsigned 32-bit byte offset from the wave-uniform row pointer, which lets the load use the
    // scalar-base + vector-offset addressing form (no per-load 64-bit vector add).
    __device__ __forceinline__ static void load_raw(void const *(&rows)[N], int f0, int lane, int f_last, Raw (&raw)[N])
    {
        uint32_t const off = (uint32_t)min(f0 + lane, f_last) * 4u;
#pragma unroll
        for (int k = 0; k < N; ++k) {
            raw[k] = *reinterpret_cast<uint32_t const *>(reinterpret_cast<char const *>(rows[k]) + off);
        }
    }

    __device__ __forceinline__ static void centre_all(Raw const (&raw)[N], float bias, float (&z)[N])
    {
#pragma unroll
        for (int k = 0; k < N; ++k) { z[k] = centre<XMODE>(__uint_as_float(raw[k]), bias); }
    }
};

// Packed bits: the 64 frames of a wavefront step (f0 a multiple of 64) are the two words f0 / 32 and f0 / 32 + 1 of the
// row, the same for every lane, and bit l of the pair belongs to lane l.  They are fetched with scalar loads through the
// constant address space (the input is not written by the kernels that gather) and used directly as the lane mask of a
// select between -bias and +bias: no vector memory instruction and one vector ALU instruction per input.
// Where the second word would hold no frame of the buffer the first is loaded in its place: lanes beyond the last frame
// get bits of the row's padding or of other frames, and their results are discarded by the callers.
template <int N>
struct Gather<N, kXBit> {
    using Raw = uint64_t;
    typedef __attribute__((address_space(4))) uint32_t const const_u32;

    __device__ __forceinline__ static void load_raw(void const *(&rows)[N], int f0, int, int f_last, Raw (&raw)[N])
    {
        int const  w0     = min(f0, f_last) >> 5;
        bool const second = ((w0 + 1) << 5) <= f_last;
#pragma unroll
        for (int k = 0; k < N; ++k) {
            const_u32 *p = (const_u32 *)rows[k] + w0;
            uint32_t const lo = p[0];
            uint32_t const hi = p[second ? 1 : 0];          // always a word of the row
            raw[k] = (uint64_t)lo | ((uint64_t)hi << 32);
        }
    }

    __device__ __forceinline__ static void centre_all(Raw const (&raw)[N], float bias, float (&z)[N])
    {
#pragma unroll
        for (int k = 0; k < N; ++k) { z[k] = __builtin_amdgcn_inverse_ballot_w64(raw[k]) ? bias : -bias; }
    }
};

struct FwdArgs {
    void const  *x;
    void        *y;
    int const   *idx;
    float const *C;             // [O][2^N] centred coefficients
    float const *V;             // [O][2^N] corner values (two-valued inputs: lut_forward_corner_kernel)
    float const *mean;          // BN: per node (nullptr otherwise)
    float const *rstd;
    float       *stat_partial;  // STATS: [O][chunk][2] partial sums of (v - C0), (v - C0)^2;  kind 3: of g, g (v - mean)
    float const *dy;            // kind 3: [O][dy_stride]
    int   dy_stride;
    int   node_size, frame_size;
    int   x_stride, y_stride;   // elements per node row (floats or words)
    int   chunk;                // frames per unit, multiple of 64
    int   chunk_count;
    TileDivisor tiles;
    float bias, gamma, beta;
    // where kind 1 takes the batch-norm statistics of a node from (see forward_statistics)
    int   stat_mode;            // kStatGiven: mean / rstd;  kStatRunning: mean = running mean, rstd holds the running variance;
                                // kStatPartial: from the partial sums that a kind 2 launch of the same shape left in stat_partial
    float momentum;             // kStatPartial: the wavefront of a node's first unit also stores the statistics:
    float *mean_out, *rstd_out, *running_mean, *running_var;
    // Not null (plain output, one unit per node, widths whose table fits one vector register): no table-preparation launch has
    // run; the wavefront brings its node's table W' into the centred basis itself — 2^N loads, one per lane, and the
    // butterfly of table_prep_block over the lanes.  A call of a few hundred frames is two launches' worth of latency, not work.
    // With clamp_W (below) the table is first clamped and written back, as in the corner-value kernel.
    float const *W_inline;
    int   lut_binarize;
    // lut_forward_corner_kernel with W_inline: the node's tables go to C_out / V_out as well (the wavefront of the node's first unit
    // stores them: for a later launch of the same call, and for the caller that keeps them for the backward pass), and the table is
    // first clamped to [clamp_lo, clamp_hi] and written back where clamp_W (W itself) is given — all as table_prep_block does
    float *C_out, *V_out;
    float *clamp_W;  float clamp_lo, clamp_hi;
    // Not null (binarized fp32 output): the binarized output also goes here as packed bits, rows of y_bits_stride words — the packed
    // copy that the next layer would otherwise make of y before it reads it
    uint32_t *y_bits;
    int   y_bits_stride;
    // lut_forward_corner_kernel on fp32 frames, statistics kind: not null = the corner index that each lane forms of its frame's
    // inputs is kept, one byte per (node, frame) (the index times 4, as ds_bpermute takes it): word (f / 256) * 64 + l of a node's
    // row of own_stride words holds frames f + l, f + 64 + l, f + 128 + l, f + 192 + l.  The output launch of the same call
    // (own_index: the same buffer) then reads a word per lane and four steps instead of gathering the fp32 frames a second time.
    // Units of both launches begin at multiples of 256 frames.  Needs no count of the input's rows.
    // The statistics pass of a backward call (kind 3, passes of four steps) keeps them the same way for lut_dx_indexed_kernel.
    uint32_t       *own_index_out;
    uint32_t const *own_index;
    int   own_stride;
    // kStatPartial: units per node of the launch that left the partial sums, where the output launch has other units (0: the same)
    int   stat_units;
};

// kStatInline: the call has one unit per node, so the wavefront that writes a node's output first sums the node's statistics
// itself (a pass of its own over the unit) instead of reading them from a statistics launch
enum StatMode : int { kStatGiven = 0, kStatRunning = 1, kStatPartial = 2, kStatInline = 3 };
constexpr int kInlineUnitPasses = 4;         // kStatInline: passes (of 256 frames) whose corner indices a wavefront keeps in registers
constexpr int kInlineStatUnits = 4 * kWave; // most units whose partial sums a wavefront adds up itself: up to four loads per lane

// What a forward kernel does with the LUT output v of (node, frame f = f0 + lane): accumulate statistics (kinds 2, 3) or
// apply the batch-norm output stage (kind 1) and store.  ok: the frame belongs to the unit; live: the node exists.
// bits_mask (binarized fp32 output with a packed copy): where given, the lane mask of the step's binarized output is handed back
// instead of stored, and the caller stores the words of several steps together.
// the batch-norm output of a LUT output v (reference: DifferentiableLutN.h:831-835); one expression for every kernel that forms it
__device__ __forceinline__ float batch_norm_output(float v, float mean, float rstd, float gamma, float beta)
{
    return ((v - mean) * rstd) * gamma + beta;
}

template <int YMODE, int FWD_KIND>
__device__ __forceinline__ void forward_stage(FwdArgs const &a, float v, bool ok, bool live, int lane, int node, int f0, int f, int f_end,
                                              float mean, float rstd, float c0, float dyv, float &s1, float &s2, uint64_t *bits_mask = nullptr)
{
    if (FWD_KIND == 2) {
        float const d = ok ? (v - c0) : 0.0f;
        s1 += d;
        s2 = __builtin_fmaf(d, d, s2);
        return;
    }
    if (FWD_KIND == 3) {
        float const t = batch_norm_output(v, mean, rstd, a.gamma, a.beta);
        float d = ok ? dyv : 0.0f;
        if (t <= 0.0f || t >= 1.0f) { d = 0.0f; }
        s1 += d;
        s2 = __builtin_fmaf(d, v - mean, s2);
        return;
    }
    if (FWD_KIND == 1) { v = batch_norm_output(v, mean, rstd, a.gamma, a.beta); }
    if (!live) { return; }
    if (YMODE == kYBit) {
        uint64_t const m = __ballot(ok && (v > 0.5f));
        uint32_t *yr = reinterpret_cast<uint32_t *>(a.y) + (size_t)node * a.y_stride + (f0 >> 5);
        if (lane == 0)                          { yr[0] = (uint32_t)m; }
        if (lane == 32 && (f0 + 32) < f_end)    { yr[1] = (uint32_t)(m >> 32); }
    }
    else {
        if (YMODE == kYBinarize) {
            if (a.y_bits != nullptr) {                // wave-uniform
                uint64_t const m = __ballot(ok && (v > 0.5f));
                if (bits_mask != nullptr) { *bits_mask = m; }
                else {
                    uint32_t *yr = a.y_bits + (size_t)node * a.y_bits_stride + (f0 >> 5);
                    if (lane == 0)                          { yr[0] = (uint32_t)m; }
                    if (lane == 32 && (f0 + 32) < f_end)    { yr[1] = (uint32_t)(m >> 32); }
                }
            }
            v = (v > 0.5f) ? 1.0f : 0.0f;
        }
        else { v = __builtin_amdgcn_fmed3f(v, 0.0f, 1.0f); }
        if (ok) { __builtin_nontemporal_store(v, reinterpret_cast<float *>(a.y) + (size_t)node * a.y_stride + f); }
    }
}

// Packed copy of the output: the words of a node's row behind its last frame are written as 0 by the wavefront of the node's last
// unit (the words of the frames themselves are whole: bits past the last frame are 0 in the ballot), as the packing kernels leave them.
__device__ __forceinline__ void zero_packed_tail(FwdArgs const &a, int ck, int node, bool live, int lane)
{
    if (a.y_bits == nullptr || ck != a.chunk_count - 1 || !live) { return; }
    for (int w = ((a.frame_size + 31) >> 5) + lane; w < a.y_bits_stride; w += kWave) { a.y_bits[(size_t)node * a.y_bits_stride + w] = 0u; }
}

// per (unit, node) partial sums of the statistics kinds
__device__ __forceinline__ void forward_store_stats(FwdArgs const &a, int ck, int node, bool live, int lane, float s1, float s2)
{
    float const t1 = wave_sum(s1), t2 = wave_sum(s2);
    if (lane == 0 && live) {
        float *q = a.stat_partial + ((size_t)node * a.chunk_count + ck) * 2;     // a node's units side by side: who adds them up reads a contiguous run
        q[0] = t1;
        q[1] = t2;
    }
}

// Sum of the per-unit partial sums [node_size][count][2] of one node by one wavefront, count <= kInlineStatUnits: lane l
// adds units l, l + 64, l + 128, l + 192 in that order and wave_sum adds the lanes, a fixed order: every wavefront that sums a node
// gets the same bits.  This costs a wavefront a few loads and a dozen cross-lane steps, less than the launch that would do it once per node.
__device__ __forceinline__ void wave_stat_sums(float const *__restrict__ stat_partial, int node_size, int count, int node, int lane,
                                               float &s1, float &s2)
{
    float2 v = make_float2(0.0f, 0.0f);
    if (count <= kWave) {
        if (lane < count) { v = *reinterpret_cast<float2 const *>(stat_partial + ((size_t)node * count + lane) * 2); }
    }
    else {
        float2 p[kInlineStatUnits / kWave];
#pragma unroll
        for (int q = 0; q < kInlineStatUnits / kWave; ++q) {
            int const u = lane + q * kWave;
            p[q] = (u < count) ? *reinterpret_cast<float2 const *>(stat_partial + ((size_t)node * count + u) * 2) : make_float2(0.0f, 0.0f);
        }
#pragma unroll
        for (int q = 0; q < kInlineStatUnits / kWave; ++q) { v.x += p[q].x; v.y += p[q].y; }
    }
    s1 = wave_sum(v.x);
    s2 = wave_sum(v.y);
}

// mean, var (>= 1e-5) and rstd of a node from the sums of (v - C0) and (v - C0)^2 over the frames
// (reference: include/bb/DifferentiableLutN.h:804-806)
__device__ __forceinline__ void batch_statistics(float s1, float s2, float c0, int frame_size, float &mean, float &var, float &rstd)
{
    float const r  = 1.0f / (float)frame_size;
    float const m0 = s1 * r;                                  // mean of (v - C0)
    mean = c0 + m0;
    var  = fmaxf(1.0e-5f, s2 * r - m0 * m0);
    rstd = 1.0f / sqrtf(var);
}

// running statistics and the stored mean / rstd of a training pass (reference: DifferentiableLutN.h:809-812)
__device__ __forceinline__ void store_statistics(float *__restrict__ mean_out, float *__restrict__ rstd_out,
                                                 float *__restrict__ running_mean, float *__restrict__ running_var,
                                                 int node, float mean, float var, float rstd, float momentum)
{
    running_mean[node] = running_mean[node] * momentum + mean * (1.0f - momentum);
    running_var[node]  = running_var[node]  * momentum + var  * (1.0f - momentum);
    mean_out[node] = mean;
    rstd_out[node] = rstd;
}

// batch-norm statistics of a node for the output stage (kind 1), by the mode of the call; var only with kStatPartial
__device__ __forceinline__ void forward_statistics(FwdArgs const &a, int node, int lane, float c0, float &mean, float &var, float &rstd)
{
    var = 0.0f;
    if (a.stat_mode == kStatPartial) {
        float s1, s2;
        wave_stat_sums(a.stat_partial, a.node_size, a.stat_units > 0 ? a.stat_units : a.chunk_count, node, lane, s1, s2);
        batch_statistics(s1, s2, c0, a.frame_size, mean, var, rstd);
    }
    else {
        mean = a.mean[node];
        rstd = a.rstd[node];
        if (a.stat_mode == kStatRunning) { rstd = 1.0f / sqrtf(rstd); }       // reference: DifferentiableLutN.h:866-868
    }
    // the same in every lane: kept in scalar registers, as when they are read from memory
    mean = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(mean)));
    var  = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(var)));
    rstd = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(rstd)));
}

// kStatPartial: the wavefront of a node's first unit stores the statistics.  Called at the end of the kernel: a store ahead
// of the wave-uniform loads of the set-up would take them off the scalar path.
__device__ __forceinline__ void forward_store_statistics(FwdArgs const &a, int node, bool live, int ck, int lane, float mean, float var, float rstd)
{
    if ((a.stat_mode == kStatPartial || a.stat_mode == kStatInline) && ck == 0 && lane == 0 && live) {
        store_statistics(a.mean_out, a.rstd_out, a.running_mean, a.running_var, node, mean, var, rstd, a.momentum);
    }
}

// FWD_KIND: 0 = plain LUT output, 1 = LUT + batch-norm (mean/rstd/gamma/beta) output, 2 = statistics only,
//           3 = statistics of the backward pass through batch-norm: per node the sums of g and g (v - mean), where g = dy gated by
//               the hard-tanh window 0 < t < 1 of the batch-norm output t (reference: DifferentiableLutN.h:1206-1222)
// NPW: nodes per wavefront.  A wavefront issues the loads of NPW nodes x U steps together (NPW x U = 4); with two nodes the
// set-up of a wavefront (index and table loads, two memory latencies before the first gather can go out) is shared by twice
// the work.
template <int N, int XMODE, int YMODE, int FWD_KIND, int NPW>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(2))) void lut_forward_kernel(FwdArgs a)
{
    using D = LutDims<N>;
    int const B    = a.chunk_count * a.tiles.count;
    int const lid  = xcd_remap(blockIdx.x, B);
    int ck, tile;
    split_tile(lid, a.tiles, ck, tile);
    int const node0 = __builtin_amdgcn_readfirstlane((tile * kWavesPerBlk + (int)(threadIdx.x / kWave)) * NPW);
    if (node0 >= a.node_size) { return; }
    int const lane = threadIdx.x & (kWave - 1);

    constexpr bool kMatrix = LutMatrixQ<N>::kUsable;
    float C[NPW][kMatrix ? 1 : D::NN], cv[NPW][D::H];
    LutMatrixQ<N> mq[NPW];
    void const *rows[NPW][N];
    float mean[NPW], rstd[NPW], var[NPW], c0[NPW];
    int node[NPW];
    bool live[NPW];
    bool clamp_store[NPW];
    float clamp_w[NPW];
#pragma unroll
    for (int p = 0; p < NPW; ++p) { clamp_store[p] = false; clamp_w[p] = 0.0f; }
    // (the statistics first: what they need in registers is gone before the tables arrive)
#pragma unroll
    for (int p = 0; p < NPW; ++p) {
        live[p] = (node0 + p < a.node_size);
        node[p] = live[p] ? node0 + p : node0;              // a wavefront past the last node repeats its first one and stores nothing
        mean[p] = 0.0f; rstd[p] = 1.0f; var[p] = 0.0f;
        c0[p] = (FWD_KIND == 0) ? 0.0f : a.C[(size_t)node[p] * D::NN];      // (the plain output does not use it)
        if (FWD_KIND == 1) { forward_statistics(a, node[p], lane, c0[p], mean[p], var[p], rstd[p]); }
        if (FWD_KIND == 3) { mean[p] = a.mean[node[p]]; rstd[p] = a.rstd[node[p]]; }
    }
#pragma unroll
    for (int p = 0; p < NPW; ++p) {
        if constexpr (kMatrix) {
            if (FWD_KIND == 0 && a.W_inline != nullptr) {
                float v = a.W_inline[(size_t)node[p] * D::NN + (lane & (D::NN - 1))];
                if (a.clamp_W != nullptr) {                   // the table clamped in place as well, by the wavefront of the node's first unit
                    float const wc = fminf(a.clamp_hi, fmaxf(a.clamp_lo, v));
                    clamp_store[p] = (ck == 0) && live[p] && (lane < D::NN) && (wc != v);
                    v = wc;
                    clamp_w[p] = wc;
                }
                if (a.lut_binarize) { v = (v > 0.5f) ? 1.0f : 0.0f; }
#pragma unroll
                for (int j = 0; j < N; ++j) {                 // as table_prep_block: (a, b) -> ((a + b) / 2, b - a) per index bit
                    float const o = __shfl_xor(v, 1 << j, 64);
                    v = ((lane >> j) & 1) ? (v - o) : (v + o) * 0.5f;
                }
                mq[p].take(v, lane);
                C[p][0] = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(v)));
            }
            else {
                mq[p].load(a.C + (size_t)node[p] * D::NN, lane);
                C[p][0] = a.C[(size_t)node[p] * D::NN];
            }
        }
        else {
            LutEval<N>::load_table(a.C + (size_t)node[p] * D::NN, C[p]);
            LutEval<N>::pin_constants(C[p], cv[p]);
        }
#pragma unroll
        for (int k = 0; k < N; ++k) {
            int const in = a.idx[node[p] * N + k];
            rows[p][k] = (XMODE == kXBit) ? (void const *)(reinterpret_cast<uint32_t const *>(a.x) + (size_t)in * a.x_stride)
                                          : (void const *)(reinterpret_cast<float const *>(a.x) + (size_t)in * a.x_stride);
        }
    }

    int const f_begin = ck * a.chunk;
    int const f_end   = min(f_begin + a.chunk, a.frame_size);
    float s1[NPW], s2[NPW];
#pragma unroll
    for (int p = 0; p < NPW; ++p) { s1[p] = 0.0f; s2[p] = 0.0f; }

    // wavefront-steps whose loads are issued together; packed-bit inputs arrive as scalar lane masks, two registers each
    constexpr int U = (XMODE == kXBit) ? 2 / NPW : 4 / NPW;
    int const f_last = a.frame_size - 1;
    for (int fb = f_begin; fb < f_end; fb += kWave * U) {
        typename Gather<N, XMODE>::Raw raw[NPW][U][N];
        float dyv[NPW][U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (fb + u * kWave < f_end) {            // wave-uniform: steps beyond the unit load nothing
#pragma unroll
                for (int p = 0; p < NPW; ++p) {
                    int const fs = min(fb + u * kWave + lane, f_last);
                    Gather<N, XMODE>::load_raw(rows[p], fb + u * kWave, lane, f_last, raw[p][u]);
                    if (FWD_KIND == 3) { dyv[p][u] = a.dy[(size_t)node[p] * a.dy_stride + fs]; }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            int const f0 = fb + u * kWave;
            if (f0 >= f_end) { break; }
            int const  f  = f0 + lane;
            bool const ok = f < f_end;
#pragma unroll
            for (int p = 0; p < NPW; ++p) {
                float z[N];
                Gather<N, XMODE>::centre_all(raw[p][u], a.bias, z);
                float v;
                if constexpr (kMatrix) { v = mq[p].forward(z); }
                else                   { v = LutEval<N>::forward(C[p], cv[p], z); }

                forward_stage<YMODE, FWD_KIND>(a, v, ok, live[p], lane, node[p], f0, f, f_end, mean[p], rstd[p], c0[p],
                                               (FWD_KIND == 3) ? dyv[p][u] : 0.0f, s1[p], s2[p]);
            }
        }
    }

    if (FWD_KIND == 2 || FWD_KIND == 3) {
#pragma unroll
        for (int p = 0; p < NPW; ++p) { forward_store_stats(a, ck, node[p], live[p], lane, s1[p], s2[p]); }
    }
    if (FWD_KIND == 1) {
#pragma unroll
        for (int p = 0; p < NPW; ++p) { forward_store_statistics(a, node[p], live[p], ck, lane, mean[p], var[p], rstd[p]); }
    }
    if (YMODE == kYBinarize && (FWD_KIND == 0 || FWD_KIND == 1)) {
#pragma unroll
        for (int p = 0; p < NPW; ++p) { zero_packed_tail(a, ck, node[p], live[p], lane); }
    }
    if (FWD_KIND == 0 && kMatrix) {           // (at the end: a store ahead of the unit's loads would be waited for with them)
#pragma unroll
        for (int p = 0; p < NPW; ++p) {
            if (clamp_store[p]) { a.clamp_W[(size_t)node[p] * D::NN + lane] = clamp_w[p]; }
        }
    }
}

// ------------------------------------------------------------------------------------------------
//  helpers of the kernels for two-valued inputs
// ------------------------------------------------------------------------------------------------
// lane masks of four wavefront-steps (256 frames from fb, a multiple of 256) of N packed rows: one 32-byte scalar load per row
template <int N>
__device__ __forceinline__ void corner_masks_wide(void const *(&rows)[N], int fb, uint64_t (&raw)[4][N])
{
    typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
    typedef __attribute__((address_space(4))) u32x8 const const_u32x8;
#pragma unroll
    for (int k = 0; k < N; ++k) {
        u32x8 const w = *(const_u32x8 *)(reinterpret_cast<uint32_t const *>(rows[k]) + (fb >> 5));
#pragma unroll
        for (int u = 0; u < 4; ++u) { raw[u][k] = (uint64_t)w[2 * u] | ((uint64_t)w[2 * u + 1] << 32); }
    }
}

// corner index of the lane's frame, most significant input first: index = 2 index + bit, one add-with-carry per input
// with the input's lane mask as the carry
template <int N, int XMODE, typename Raw>
__device__ __forceinline__ uint32_t corner_index(Raw const (&raw)[N])
{
    uint32_t index = 0;
#pragma unroll
    for (int k = N - 1; k >= 0; --k) {
        uint64_t mask, carry;
        if constexpr (XMODE == kXBit) { mask = raw[k]; }
        else                          { mask = __ballot(__uint_as_float(raw[k]) > 0.5f); }
        asm("v_addc_co_u32_e64 %0, %1, %2, %2, %3" : "=v"(index), "=s"(carry) : "v"(index), "s"(mask));
    }
    return index;
}

// What a corner-value wavefront looks up per frame.  The LUT output of a frame is one of the node's 2^N corner values, so everything
// that a kind computes from it alone is computed once per corner — by lane p for corner p, with the operations the polynomial
// kernels apply per frame (same bits) — and the frames fetch the finished value from the lane that holds it:
//   kinds 0, 1: tab0 = the output (batch-norm stage for kind 1, then clamped to [0, 1], or 1 / 0 where the output is binarized)
//   kind 2    : tab0 = V - C0, the term of the statistics sums
//   kind 3    : tab0 = 1 / 0, whether the batch-norm output lies inside the hard-tanh window;  tab1 = V - mean
struct CornerTables { int tab0, tab1; };

template <int YMODE, int KIND>
__device__ __forceinline__ CornerTables corner_tables(FwdArgs const &a, float v, float mean, float rstd, float c0)
{
    CornerTables t{0, 0};
    if (KIND == 2) { t.tab0 = __float_as_int(v - c0); }
    else if (KIND == 3) {
        float const b = batch_norm_output(v, mean, rstd, a.gamma, a.beta);
        t.tab0 = __float_as_int((b <= 0.0f || b >= 1.0f) ? 0.0f : 1.0f);
        t.tab1 = __float_as_int(v - mean);
    }
    else {
        float y = (KIND == 1) ? batch_norm_output(v, mean, rstd, a.gamma, a.beta) : v;
        if (YMODE == kYClamp) { y = __builtin_amdgcn_fmed3f(y, 0.0f, 1.0f); }
        else                  { y = (y > 0.5f) ? 1.0f : 0.0f; }
        t.tab0 = __float_as_int(y);
    }
    return t;
}

// A corner-value wavefront's pass over U wavefront-steps from frame fb of its unit (see lut_forward_corner_kernel).
// OWN: where the corner indices come from.  kOwnNone: from the gathered inputs; kOwnMemory: from the bytes that the statistics launch
// of the call kept (FwdArgs::own_index); kOwnRegister: from `own`, which an earlier pass of the same wavefront over the same frames
// left there.  `own` always returns the indices of the pass, byte u = 4 x the index of frame fb + 64 u + lane.
enum OwnIndex : int { kOwnNone = 0, kOwnMemory = 1, kOwnRegister = 2 };
// RAGGED: the pass may reach beyond the unit's last frame (else all of its U steps are whole, and nothing is masked)
template <int N, int XMODE, int YMODE, int KIND, bool WIDE, int OWN, bool RAGGED = true>
__device__ __forceinline__ void corner_pass(FwdArgs const &a, void const *(&rows)[N], CornerTables tabs, int node, int lane, int fb,
                                            int f_end, int f_last, float &s1, float &s2, uint32_t &own)
{
    constexpr int U = (XMODE == kXBit && !WIDE && OWN == kOwnNone) ? 2 : 4;  // wavefront-steps whose loads are issued together
    typename Gather<N, XMODE>::Raw raw[U][N];
    float dyv[U];
    if constexpr (OWN == kOwnNone)   { own = 0; }
    if constexpr (OWN == kOwnMemory) { own = a.own_index[(size_t)node * a.own_stride + (fb >> 8) * kWave + lane]; }
    if constexpr (WIDE && OWN == kOwnNone) { corner_masks_wide<N>(rows, fb, raw); }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        if (!RAGGED || fb + u * kWave < f_end) {            // wave-uniform: steps beyond the unit load nothing
            if constexpr (!WIDE && OWN == kOwnNone) { Gather<N, XMODE>::load_raw(rows, fb + u * kWave, lane, f_last, raw[u]); }
            if (KIND == 3) { dyv[u] = a.dy[(size_t)node * a.dy_stride + (RAGGED ? min(fb + u * kWave + lane, f_last) : fb + u * kWave + lane)]; }
        }
    }
    constexpr bool kPackedCopy = (YMODE == kYBinarize) && (KIND == 0 || KIND == 1);
    uint32_t words = 0;                                  // lane l < 2 U: word l of the pass's packed output
#pragma unroll
    for (int u = 0; u < U; ++u) {
        int const f0 = fb + u * kWave;
        if (RAGGED && f0 >= f_end) { break; }
        int const  f  = f0 + lane;
        bool const ok = !RAGGED || f < f_end;
        uint32_t index4;
        if constexpr (OWN != kOwnNone) { index4 = (own >> (8 * u)) & 0xffu; }
        else {
            index4 = corner_index<N, XMODE>(raw[u]) << 2;
            if (U == 4) { own |= index4 << (8 * u); }
        }
        float const t0 = __int_as_float(__builtin_amdgcn_ds_bpermute((int)index4, tabs.tab0));
        if (KIND == 2) {
            float const d = ok ? t0 : 0.0f;
            s1 += d;
            s2 = __builtin_fmaf(d, d, s2);
        }
        else if (KIND == 3) {
            // (reference: DifferentiableLutN.h:1206-1222: dy behind the hard-tanh window, summed alone and times the centred output)
            float const t1 = __int_as_float(__builtin_amdgcn_ds_bpermute((int)index4, tabs.tab1));
            float const d  = (ok && t0 != 0.0f) ? dyv[u] : 0.0f;
            s1 += d;
            s2 = __builtin_fmaf(d, t1, s2);
        }
        else if (YMODE == kYBit) {
            uint64_t const m = __ballot(ok && (t0 > 0.5f));
            asm("s_nop 3\n\tv_writelane_b32 %0, %1, %2" : "+v"(words) : "s"((uint32_t)m), "n"(2 * u));         // (as below)
            asm("s_nop 3\n\tv_writelane_b32 %0, %1, %2" : "+v"(words) : "s"((uint32_t)(m >> 32)), "n"(2 * u + 1));
        }
        else {
            if (kPackedCopy && a.y_bits != nullptr) {         // wave-uniform
                uint64_t const m = __ballot(ok && (t0 > 0.5f));
                // words[lane 2u] = low half, words[lane 2u + 1] = high half.  The mask may come straight from a vector compare, and
                // v_writelane_b32 must not read a scalar register in the wait states after a vector instruction wrote it (the
                // compiler does not look into the asm): both instructions wait for themselves.
                asm("s_nop 3\n\tv_writelane_b32 %0, %1, %2" : "+v"(words) : "s"((uint32_t)m), "n"(2 * u));
                asm("s_nop 3\n\tv_writelane_b32 %0, %1, %2" : "+v"(words) : "s"((uint32_t)(m >> 32)), "n"(2 * u + 1));
            }
            if (ok) { __builtin_nontemporal_store(t0, reinterpret_cast<float *>(a.y) + (size_t)node * a.y_stride + f); }
        }
    }
    // the packed copy of the pass: its 2 U words by one store (a store per step would double the kernel's store instructions)
    if (kPackedCopy && a.y_bits != nullptr && lane < 2 * U && (!RAGGED || fb + 32 * lane < f_end)) {
        a.y_bits[(size_t)node * a.y_bits_stride + (fb >> 5) + lane] = words;
    }
    // packed output: the same, to the words of the output row that hold frames of the unit
    if (YMODE == kYBit && (KIND == 0 || KIND == 1) && lane < 2 * U && (!RAGGED || fb + 32 * lane < f_end)) {
        reinterpret_cast<uint32_t *>(a.y)[(size_t)node * a.y_stride + (fb >> 5) + lane] = words;
    }
}

// corner_pass, whole or ragged as the pass lies in the unit (wave-uniform)
template <int N, int XMODE, int YMODE, int KIND, bool WIDE, int OWN>
__device__ __forceinline__ void corner_pass_any(FwdArgs const &a, void const *(&rows)[N], CornerTables tabs, int node, int lane, int fb,
                                                int f_end, int f_last, float &s1, float &s2, uint32_t &own)
{
    constexpr int U = (XMODE == kXBit && !WIDE && OWN == kOwnNone) ? 2 : 4;
    if (fb + kWave * U <= f_end) { corner_pass<N, XMODE, YMODE, KIND, WIDE, OWN, false>(a, rows, tabs, node, lane, fb, f_end, f_last, s1, s2, own); }
    else                         { corner_pass<N, XMODE, YMODE, KIND, WIDE, OWN, true>(a, rows, tabs, node, lane, fb, f_end, f_last, s1, s2, own); }
}

// The passes of a corner-value wavefront over its unit.  OWN as in corner_pass (kOwnNone or kOwnMemory); the statistics kind over
// fp32 frames keeps its corner indices for the output launch where the call asks for it (FwdArgs::own_index_out).
template <int N, int XMODE, int YMODE, int KIND, bool WIDE, int OWN = kOwnNone>
__device__ __forceinline__ void corner_unit_pass(FwdArgs const &a, void const *(&rows)[N], CornerTables tabs, int node, int lane,
                                                 int f_begin, int f_end, int f_last, float &s1, float &s2)
{
    constexpr int U = (XMODE == kXBit && !WIDE && OWN == kOwnNone) ? 2 : 4;
    // passes of four steps leave their corner indices in `own`: the statistics kinds keep them where the call asks for it
    // (kind 2 over fp32 frames: for the output launch; kind 3: for the dx kernel of the same backward call, lut_dx_indexed_kernel)
    constexpr bool kKeepIndex = (U == 4) && (OWN == kOwnNone) && ((XMODE == kXBinary && KIND == 2) || KIND == 3);
    for (int fb = f_begin; fb < f_end; fb += kWave * U) {
        uint32_t own;
        corner_pass_any<N, XMODE, YMODE, KIND, WIDE, OWN>(a, rows, tabs, node, lane, fb, f_end, f_last, s1, s2, own);
        if (kKeepIndex && a.own_index_out != nullptr) {      // (wave-uniform; steps beyond the unit left their byte 0)
            a.own_index_out[(size_t)node * a.own_stride + (fb >> 8) * kWave + lane] = own;
        }
    }
}

// ------------------------------------------------------------------------------------------------
//  Forward for two-valued inputs (packed bits, or fp32 frames binarized at 0.5): the LUT output is one of the 2^N corner
//  values V of the node.  A lane builds the corner index of its frame from the N input bits (one add-with-carry per input:
//  index = 2 index + bit, the bit arriving as a lane mask in a scalar register pair) and fetches V[index] from the lane
//  that holds it (ds_bpermute): N + 2 instructions per (node, 64 frames) instead of the polynomial's 45.
//  One wavefront = one node x one unit of frames; kinds and output modes as in lut_forward_kernel.
// ------------------------------------------------------------------------------------------------
//  WIDE (packed bits, row pitch a multiple of 8 words, units a multiple of 256 frames): the bits of 256 frames of an input
//  are one 32-byte scalar load, so a unit costs N scalar loads per four steps instead of 2 N per step.
//  OWN (output launch of a batch-norm training pass over fp32 frames): the corner indices are read from the bytes that the
//  statistics launch kept (FwdArgs::own_index); instantiated on the packed-bit mode, whose gathers it does not use.
template <int N, int XMODE, int YMODE, int FWD_KIND, bool WIDE = false, int OWN = kOwnNone>
__global__ __launch_bounds__(kBlock) void lut_forward_corner_kernel(FwdArgs a)
{
    static_assert(XMODE == kXBit || XMODE == kXBinary, "corner values need two-valued inputs");
    static_assert(!WIDE || XMODE == kXBit, "wide loads are for packed bits");
    static_assert(OWN == kOwnNone || (OWN == kOwnMemory && XMODE == kXBit && !WIDE && FWD_KIND == 1), "kept corner indices: output launch only");
    constexpr int NN = 1 << N;
    int const B    = a.chunk_count * a.tiles.count;
    int const lid  = xcd_remap(blockIdx.x, B);
    int ck, tile;
    split_tile(lid, a.tiles, ck, tile);
    int const node = __builtin_amdgcn_readfirstlane(tile * kWavesPerBlk + (int)(threadIdx.x / kWave));
    if (node >= a.node_size) { return; }
    int const lane = threadIdx.x & (kWave - 1);

    int corner;                                                                         // lane p holds V[p]
    float c0 = 0.0f, table_c = 0.0f, table_w = 0.0f;
    bool clamp_store = false;
    if (a.W_inline != nullptr) {
        // no table launch has run: the wavefront derives its node's tables itself, as table_prep_block would (same operations on
        // the same values: same bits), and the wavefront of the node's first unit stores what later launches and the caller read
        int const i = lane & (NN - 1);
        float w = a.W_inline[(size_t)node * NN + i];
        if (a.clamp_W != nullptr) {
            float const wc = fminf(a.clamp_hi, fmaxf(a.clamp_lo, w));
            clamp_store = (ck == 0) && (lane < NN) && (wc != w);
            w = wc;
        }
        table_w = w;
        if (a.lut_binarize) { w = (w > 0.5f) ? 1.0f : 0.0f; }
        float const c = centred_butterfly<N>(w, i);
        float const v = corner_butterfly<N>(c, i, a.bias);
        table_c = c;                                        // stored at the end of the kernel: a store ahead of the unit's loads would be waited for with them
        c0 = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(c)));
        corner = __float_as_int(v);
    }
    else { corner = __float_as_int(a.V[(size_t)node * NN + (lane & (NN - 1))]); }
    void const *rows[N];
#pragma unroll
    for (int k = 0; k < N; ++k) {
        int const in = (OWN == kOwnMemory) ? 0 : a.idx[node * N + k];
        rows[k] = (XMODE == kXBit) ? (void const *)(reinterpret_cast<uint32_t const *>(a.x) + (size_t)in * a.x_stride)
                                   : (void const *)(reinterpret_cast<float const *>(a.x) + (size_t)in * a.x_stride);
    }
    float mean = 0.0f, rstd = 1.0f;
    if (a.W_inline == nullptr && (FWD_KIND == 2 || (FWD_KIND == 1 && (a.stat_mode == kStatPartial || a.stat_mode == kStatInline)))) {
        c0 = a.C[(size_t)node * NN];
    }
    float var = 0.0f;

    int const f_begin = ck * a.chunk;
    int const f_end   = min(f_begin + a.chunk, a.frame_size);
    int const f_last  = a.frame_size - 1;
    float s1 = 0.0f, s2 = 0.0f;
    bool f_done = false;

    if (FWD_KIND == 1) {
        if (a.stat_mode == kStatInline) {
            // one unit per node: the sums of the statistics kind, by the same steps in the same order, then what the
            // statistics launch and the partial-sum read would have delivered (same bits)
            // up to kInlineUnitPasses passes of four steps: the corner indices of the passes stay in registers for the output pass,
            // which then gathers nothing
            constexpr bool kKeep = (XMODE == kXBinary || WIDE) && (OWN == kOwnNone);
            bool const keep = kKeep && (f_end - f_begin <= kInlineUnitPasses * 4 * kWave);      // wave-uniform
            uint32_t kept[kInlineUnitPasses];
            CornerTables const stat_tabs = corner_tables<YMODE, 2>(a, __int_as_float(corner), 0.0f, 1.0f, c0);
            if (keep) {
                if constexpr (kKeep) {
#pragma unroll
                    for (int q = 0; q < kInlineUnitPasses; ++q) {
                        int const fb = f_begin + q * 4 * kWave;
                        kept[q] = 0;
                        if (fb < f_end) { corner_pass_any<N, XMODE, YMODE, 2, WIDE, kOwnNone>(a, rows, stat_tabs, node, lane, fb, f_end, f_last, s1, s2, kept[q]); }
                    }
                }
            }
            else { corner_unit_pass<N, XMODE, YMODE, 2, WIDE, OWN>(a, rows, stat_tabs, node, lane, f_begin, f_end, f_last, s1, s2); }
            batch_statistics(wave_sum(s1), wave_sum(s2), c0, a.frame_size, mean, var, rstd);
            mean = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(mean)));
            var  = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(var)));
            rstd = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(rstd)));
            s1 = 0.0f; s2 = 0.0f;
            if (keep) {
                if constexpr (kKeep) {
                    CornerTables const out_tabs = corner_tables<YMODE, FWD_KIND>(a, __int_as_float(corner), mean, rstd, c0);
#pragma unroll
                    for (int q = 0; q < kInlineUnitPasses; ++q) {
                        int const fb = f_begin + q * 4 * kWave;
                        if (fb < f_end) { corner_pass_any<N, XMODE, YMODE, FWD_KIND, WIDE, kOwnRegister>(a, rows, out_tabs, node, lane, fb, f_end, f_last, s1, s2, kept[q]); }
                    }
                }
                f_done = true;
            }
        }
        else { forward_statistics(a, node, lane, c0, mean, var, rstd); }
    }
    if (FWD_KIND == 3) { mean = a.mean[node]; rstd = a.rstd[node]; }

    if (!f_done) {
        CornerTables const tabs = corner_tables<YMODE, FWD_KIND>(a, __int_as_float(corner), mean, rstd, c0);
        corner_unit_pass<N, XMODE, YMODE, FWD_KIND, WIDE, OWN>(a, rows, tabs, node, lane, f_begin, f_end, f_last, s1, s2);
    }
    if (FWD_KIND == 2 || FWD_KIND == 3) { forward_store_stats(a, ck, node, true, lane, s1, s2); }
    if (FWD_KIND == 1) { forward_store_statistics(a, node, true, ck, lane, mean, var, rstd); }
    if (YMODE == kYBinarize && (FWD_KIND == 0 || FWD_KIND == 1)) { zero_packed_tail(a, ck, node, true, lane); }
    if (a.W_inline != nullptr && ck == 0 && lane < NN) {
        if (clamp_store)         { a.clamp_W[(size_t)node * NN + lane] = table_w; }
        if (a.C_out != nullptr)  { a.C_out[(size_t)node * NN + lane] = table_c; }
        if (a.V_out != nullptr)  { a.V_out[(size_t)node * NN + lane] = __int_as_float(corner); }
    }
}

// Sum of the per-unit partial sums [node_size][count][2] of one node.  A workgroup owns nodes_per_block consecutive nodes
// (a power of two up to kBlock) and splits the units over its kBlock / nodes_per_block thread groups: group g adds units
// g, g + G, ... in ascending order and the groups are added in ascending order through LDS — a fixed order, so the result
// does not depend on the launch.  Returns true in
// the one thread per node that holds the sums.
__device__ __forceinline__ bool sum_stat_partials(float const *__restrict__ stat_partial, int node_size, int count,
                                                  int nodes_per_block, int &node, float &s1, float &s2)
{
    __shared__ float2 red[kBlock];
    int const n_local = threadIdx.x % nodes_per_block, g = threadIdx.x / nodes_per_block, groups = kBlock / nodes_per_block;
    node = blockIdx.x * nodes_per_block + n_local;
    float a = 0.0f, b = 0.0f;
    if (node < node_size) {
#pragma unroll 4
        for (int c = g; c < count; c += groups) {
            float2 const v = *reinterpret_cast<float2 const *>(stat_partial + ((size_t)node * count + c) * 2);
            a += v.x;
            b += v.y;
        }
    }
    red[threadIdx.x] = make_float2(a, b);                  // index = g * nodes_per_block + n_local
    __syncthreads();
    if (g != 0 || node >= node_size) { return false; }
    s1 = 0.0f; s2 = 0.0f;
    for (int k = 0; k < groups; ++k) {
        float2 const v = red[k * nodes_per_block + n_local];
        s1 += v.x;
        s2 += v.y;
    }
    return true;
}

// per node: mean, var (>= 1e-5), rstd, running statistics (reference: include/bb/DifferentiableLutN.h:804-812)
__global__ __launch_bounds__(kBlock) void bn_forward_finalize_kernel(float const *__restrict__ stat_partial, float const *__restrict__ C, int nn,
                                                                    float *__restrict__ mean, float *__restrict__ rstd,
                                                                    float *__restrict__ running_mean, float *__restrict__ running_var,
                                                                    float momentum, int node_size, int chunk_count, int frame_size,
                                                                    int nodes_per_block)
{
    int node;
    float s1, s2;
    if (!sum_stat_partials(stat_partial, node_size, chunk_count, nodes_per_block, node, s1, s2)) { return; }
    float m, var, rs;
    batch_statistics(s1, s2, C[(size_t)node * nn], frame_size, m, var, rs);
    store_statistics(mean, rstd, running_mean, running_var, node, m, var, rs, momentum);
}

// Term table for the input-centric dx kernel: for input node `in` and its t-th consumer connection (t-th entry of
// the reverse-table row, e = node*N + k) one record of kTermHead + 2^(N-1) dwords at
// ((in * max_fan + t) * record):  dwords [2j, 2j+1], j < N-1: the 64-bit device address of the row of the consumer's
// other input j (ascending connection order, k skipped); dwords [2(N-1), 2(N-1)+1]: the address of the consumer's dy
// row; rest of the head unused; then the 2^(N-1) coefficients Dk (entries of the consumer's plain-basis table P).  The addresses
// are final, so the dx kernel spends no scalar arithmetic on them.  All records of one input node are contiguous, so a
// wavefront reads its whole work list from one base address with scalar loads.
constexpr int kTermHead = 12;

struct TermArgs {
    float const *W;             // [O][2^N]
    int const   *idx;           // [O][N]
    int const   *rev;           // reverse table [I][rev_stride]
    int         *term;          // the records
    unsigned long long x_base, x_row_pitch_bytes, dy_base, dy_row_pitch_bytes;
    int lut_binarize, rev_stride, input_node_size;
    TileDivisor fan;            // division by the slots per input, rev_stride - 1
    int blocks;                 // workgroups that build records (kWavesPerBlk * kTermRecordsPerWave records each); 0 = nothing to build
    int corner;                 // 1: records hold the derivative's corner values for two-valued inputs (lut_dx_corner_kernel)
    float lo, hi;               //    the two input values, 1/2 -+ bias
    // node_size > 0: the records are built node by node (term_table_node_block: `blocks` then counts workgroups of kWavesPerBlk nodes) —
    // coefficient records (corner = 0) from W, value records from the nodes' corner values V, which the call then has at hand
    float const *V;             // [O][2^N], or null
    int node_size;
    // ... and indexed != 0: the records are those of lut_dx_indexed_kernel: kTermHead + 2^N dwords, head = the address of the consumer's
    // row of kept corner indices (x_base / x_row_pitch_bytes describe that buffer) and of its dy row, then the value at every corner of
    // the node (all N inputs: the two corners that differ in input k hold the same)
    int indexed;
};

// input j of a node's connections with connection k left out (j < N - 1, may differ per lane; k and the array index are compile-time)
template <int N>
__device__ __forceinline__ int ins_other(int const (&ins)[N], int k, int j)
{
    int r = 0;
#pragma unroll
    for (int q = 0; q < N - 1; ++q) { if (j == q) { r = ins[(q < k) ? q : q + 1]; } }
    return r;
}

// A wavefront builds kTermRecordsPerWave consecutive records: lane i holds entry i of a consumer's table while it is
// brought into the plain basis.  The records' loads go out together — reverse-table entries, then wiring and tables — so a
// wavefront pays the two memory round trips of a record once for all of them (one record per wavefront made the builder
// the longest part of the table-gradient launch of a layer with few nodes and many connections per input).
// Slots beyond an input's fan-out are never read by the dx kernel and are left alone.
constexpr int kTermRecordsPerWave = 4;

template <int N>
__device__ __forceinline__ void term_table_block(TermArgs const &a, int block)
{
    static_assert(2 * N <= kTermHead && kTermHead <= kWave, "head size");
    constexpr int NN = 1 << N, HN = NN / 2, REC = kTermHead + HN, R = kTermRecordsPerWave;
    int const total = a.fan.count * a.input_node_size;          // records, below 2^31 (checked on the host)
    int const rec0  = __builtin_amdgcn_readfirstlane((block * kWavesPerBlk + (int)(threadIdx.x / kWave)) * R);
    if (rec0 >= total) { return; }
    int const lane = threadIdx.x & (kWave - 1);
    // wave-uniform loads of tables that no kernel of the call writes: scalar loads through the constant address space
    typedef __attribute__((address_space(4))) int const const_int;
    const_int *rev = (const_int *)a.rev;

    int in[R], slot[R], cnt[R], e[R];
#pragma unroll
    for (int q = 0; q < R; ++q) {
        int const rec = min(rec0 + q, total - 1);               // (a wavefront past the last record repeats it and stores nothing)
        split_tile(rec, a.fan, in[q], slot[q]);                 // rec = in * max_fan + slot
        const_int *r = rev + (size_t)in[q] * a.rev_stride;
        cnt[q] = r[0];
        e[q]   = r[1 + slot[q]];                                // inside the row for every slot
    }
    bool  live[R];
    int   k[R], node[R], head[R];
    float v[R];
#pragma unroll
    for (int q = 0; q < R; ++q) {
        live[q] = (rec0 + q < total) && (slot[q] < cnt[q]);
        int const eq = live[q] ? e[q] : 0;                      // (whatever an unused slot holds is not followed)
        k[q]    = eq % N;
        node[q] = eq / N;
        head[q] = 0;
        if (lane < 2 * N) {
            int const j = lane >> 1;
            unsigned long long const addr = (j < N - 1) ? a.x_base + (unsigned long long)(unsigned)a.idx[node[q] * N + ((j < k[q]) ? j : j + 1)] * a.x_row_pitch_bytes
                                                        : a.dy_base + (unsigned long long)(unsigned)node[q] * a.dy_row_pitch_bytes;
            head[q] = (lane & 1) ? (int)(addr >> 32) : (int)(addr & 0xffffffffULL);
        }
        v[q] = 0.0f;
        if (lane < NN) { v[q] = a.W[(size_t)node[q] * NN + lane]; }
    }
#pragma unroll
    for (int q = 0; q < R; ++q) {
        if (!live[q]) { continue; }                             // wave-uniform
        int *out = a.term + (size_t)(rec0 + q) * REC;
        if (lane < kTermHead) { out[lane] = head[q]; }
        // P = plain-basis coefficients of W' (W' = lut_binarize ? W > 0.5 : W): the butterfly (a, b) -> (a, b - a) per index bit.
        // For two-valued inputs the record holds values instead of coefficients: dy/dx_k at the corner where every other
        // input j takes lo or hi.  W' is the table of y at x in {0, 1}^N and y is linear in each input, so input j != k
        // interpolates, (a, b) -> (a + lo (b - a), a + hi (b - a)), and input k differentiates, (a, b) -> (., b - a).
        float w = v[q];
        if (a.lut_binarize) { w = (w > 0.5f) ? 1.0f : 0.0f; }
#pragma unroll
        for (int j = 0; j < N; ++j) {
            float const o   = __shfl_xor(w, 1 << j, 64);
            bool const  up  = (lane >> j) & 1;
            if (a.corner && j != k[q]) {
                float const lower = up ? o : w, step = up ? (w - o) : (o - w);
                w = __builtin_fmaf(up ? a.hi : a.lo, step, lower);
            }
            else {
                w = up ? (w - o) : w;
            }
        }
        if (lane < NN && ((lane >> k[q]) & 1)) {
            int const sidx = (lane & ((1 << k[q]) - 1)) | ((lane >> (k[q] + 1)) << k[q]);      // the entry's index with bit k taken out
            out[kTermHead + sidx] = __float_as_int(w);
        }
    }
}

// The same records built node by node: a wavefront takes a node, and for each of its N connections finds the connection's place in the
// reverse-table row of its input (the lanes compare a row's entries with the connection id), and writes the record there.  Coefficient
// records share one butterfly per node (the plain-basis table does not depend on the connection).  Value records (two-valued inputs) are
// built where the call has already derived the node's corner values V: y is linear in input k between its two values, so dy/dx_k at a
// corner of the other inputs is (V[k at hi] - V[k at lo]) / (hi - lo), one cross-lane exchange instead of a butterfly per record.  The
// work is O x N records, not I x (largest fan-out) slots, and a fraction of the instructions per record: for a layer of 784 inputs and
// 6144 nodes 2.5 us instead of 10.5 us.
template <int N>
__device__ __forceinline__ void term_table_node_block(TermArgs const &a, int block)
{
    constexpr int NN = 1 << N, HN = NN / 2;
    int const REC = kTermHead + (a.indexed ? NN : HN);
    int const node = __builtin_amdgcn_readfirstlane(block * kWavesPerBlk + (int)(threadIdx.x / kWave));
    if (node >= a.node_size) { return; }
    int const lane = threadIdx.x & (kWave - 1);
    typedef __attribute__((address_space(4))) int const const_int;
    const_int *rev = (const_int *)a.rev;
    const_int *idx = (const_int *)a.idx;
    float v;
    if (a.V != nullptr) { v = a.V[(size_t)node * NN + (lane & (NN - 1))]; }
    else {
        // coefficient records: P = plain-basis coefficients of W' (W' = lut_binarize ? W > 0.5 : W), the butterfly (a, b) -> (a, b - a)
        // per index bit, as term_table_block forms them per record (same operations: same bits); a record takes the entries whose
        // index has the connection's bit set
        v = a.W[(size_t)node * NN + (lane & (NN - 1))];
        if (a.lut_binarize) { v = (v > 0.5f) ? 1.0f : 0.0f; }
#pragma unroll
        for (int j = 0; j < N; ++j) {
            float const o = __shfl_xor(v, 1 << j, 64);
            v = ((lane >> j) & 1) ? (v - o) : v;
        }
    }
    float const inv_step = 1.0f / (a.hi - a.lo);
    int ins[N], cnt[N];
#pragma unroll
    for (int k = 0; k < N; ++k) { ins[k] = idx[node * N + k]; }
#pragma unroll
    for (int k = 0; k < N; ++k) { cnt[k] = rev[(size_t)ins[k] * a.rev_stride]; }
#pragma unroll
    for (int k = 0; k < N; ++k) {
        int const e = node * N + k;
        int const *row = a.rev + (size_t)ins[k] * a.rev_stride + 1;
        int slot = -1;
        for (int base = 0; base < cnt[k] && slot < 0; base += kWave) {          // wave-uniform; a row holds a connection once
            int const r = (base + lane < cnt[k]) ? row[base + lane] : -1;
            uint64_t const m = __ballot(r == e);
            if (m != 0) { slot = base + (int)__builtin_ctzll(m); }
        }
        if (slot < 0) { continue; }                                             // (a reverse table that does not list the connection: nothing to write)
        int *out = a.term + ((size_t)ins[k] * a.fan.count + slot) * REC;
        float const other = __shfl_xor(v, 1 << k, 64);
        if (a.indexed) {
            // the node's row of kept corner indices and its dy row; the value at every corner of the node (both corners of input k)
            if (lane < 4) {
                unsigned long long const addr = (lane < 2) ? a.x_base + (unsigned long long)(unsigned)node * a.x_row_pitch_bytes
                                                           : a.dy_base + (unsigned long long)(unsigned)node * a.dy_row_pitch_bytes;
                out[lane] = (lane & 1) ? (int)(addr >> 32) : (int)(addr & 0xffffffffULL);
            }
            float const step = ((lane >> k) & 1) ? (v - other) : (other - v);
            if (lane < NN) { out[kTermHead + lane] = __float_as_int(step * inv_step); }
            continue;
        }
        if (lane < 2 * N) {
            int const j = lane >> 1;
            unsigned long long const addr = (j < N - 1) ? a.x_base + (unsigned long long)(unsigned)ins_other<N>(ins, k, j) * a.x_row_pitch_bytes
                                                        : a.dy_base + (unsigned long long)(unsigned)node * a.dy_row_pitch_bytes;
            out[lane] = (lane & 1) ? (int)(addr >> 32) : (int)(addr & 0xffffffffULL);
        }
        if (lane < NN && ((lane >> k) & 1)) {
            int const sidx = (lane & ((1 << k) - 1)) | ((lane >> (k + 1)) << k);          // the corner's index with bit k taken out
            out[kTermHead + sidx] = __float_as_int((a.V != nullptr) ? (v - other) * inv_step : v);
        }
    }
}

// ------------------------------------------------------------------------------------------------
//  backward
// ------------------------------------------------------------------------------------------------
struct BwdArgs {
    void const  *x;
    float const *dy;
    float       *dx;            // kDxAtomic: dx [I][stride], zero-filled;  kDxTmp: dx_tmp [O*N][tmp_stride];
                                // kDxNone + batch-norm: dL/d(LUT output) [O][dx_stride] for the input-centric dx kernel
    int const   *idx;
    float const *C;
    float       *dw_partial;    // [slab][O][2^N]   (BWD_KIND 0,1)
    float const *mean;          // BN
    float const *rstd;
    float const *dmean;         // BN phase 1
    float const *dvar;
    int   node_size, frame_size;
    int   x_stride, dy_stride, dx_stride;
    int   f_base, f_limit;      // frame range handled by this launch
    int   slab;                 // frames per unit, multiple of 64
    int   slab_first;           // index of the first slab of this launch in dw_partial
    int   slab_count;
    TileDivisor tiles;
    float bias, gamma, beta, inv_frames;
    TermArgs tt;                // kDxNone: the last tt.blocks workgroups of the launch build the dx kernel's term table
    float const *V;             // [O][2^N] corner values (CORNER variant)
    float const *stat_partial;  // BN, not null: dmean / dvar come from the stat_count (<= kInlineStatUnits) partial sums
    int   stat_count;           //     [unit][O][2] that the kind 3 launch left, added up by every wavefront for its node
};

// dvar and dmean of a node from the sums of g and g (v - mean) over the frames (reference: DifferentiableLutN.h:1218-1222)
__device__ __forceinline__ void batch_gradient_statistics(float s0, float s1, float mean, float rstd, float gamma, int frame_size,
                                                          float &dmean, float &dvar)
{
    float const dstd   = -(gamma * s1) * (rstd * rstd);
    float const dmeanx = -(gamma * s0) * rstd;
    dvar  = dstd * rstd;
    dmean = (dmeanx - mean * dvar) * (1.0f / (float)frame_size);
}

enum DxMode : int { kDxAtomic = 0, kDxTmp = 1, kDxNone = 2 };

// BWD_KIND: 0 = plain LUT backward, 1 = backward through batch-norm (its statistics pass is kind 3 of the forward kernel)
// DXMODE  : how (whether) the per-connection input gradients leave the kernel
// CORNER (packed bits, batch-norm, dx left to the dx kernel): the LUT output that the batch-norm window needs comes from
// the node's corner values (index by add-with-carry from the lane masks, ds_bpermute) instead of the 64-term polynomial,
// and the table leaves the scalar registers.
template <int N, int XMODE, int BWD_KIND, int DXMODE, bool CORNER = false>
__global__ __launch_bounds__(kBlock) void lut_backward_kernel(BwdArgs a)
{
    using D = LutDims<N>;
    __shared__ float red[kWavesPerBlk][16][kWave + 1];

    // The term table of the dx kernel that follows depends on nothing this kernel computes: its workgroups ride at the
    // end of this launch, where they fill the device while the last slabs drain, instead of taking a launch of their own.
    int const bid = blockIdx.x;
    int const B   = a.slab_count * a.tiles.count;
    if (DXMODE == kDxNone) {
        if (bid >= B) {
            if (a.tt.node_size > 0) { term_table_node_block<N>(a.tt, bid - B); }
            else                   { term_table_block<N>(a.tt, bid - B); }
            return;
        }
    }
    int const lid  = xcd_remap(bid, B);
    int sl, tile;
    split_tile(lid, a.tiles, sl, tile);
    int const wv   = threadIdx.x / kWave;
    int const node = __builtin_amdgcn_readfirstlane(tile * kWavesPerBlk + wv);
    if (node >= a.node_size) { return; }
    int const lane = threadIdx.x & (kWave - 1);

    // the table itself enters only the batch-norm kinds (the LUT output is recomputed) and the per-connection gradients
    static_assert(!CORNER || (XMODE == kXBit && BWD_KIND != 0 && DXMODE == kDxNone), "corner values: packed bits, batch-norm, no dx here");
    constexpr bool kNeedTable = ((BWD_KIND != 0) || (DXMODE != kDxNone)) && !CORNER;
    // (the partial sums stay on the vector ALU here: the matrix unit's operand registers would cost this kernel a wavefront of
    // occupancy, which measured slower; the batch-norm statistics pass, which only recomputes the LUT output, runs in the
    // forward kernel instead)
    float C[D::NN], cv[D::H];
    if (kNeedTable) {
        LutEval<N>::load_table(a.C + (size_t)node * D::NN, C);
        LutEval<N>::pin_constants(C, cv);
    }
    int corner = 0;
    if (CORNER) { corner = __float_as_int(a.V[(size_t)node * D::NN + (lane & (D::NN - 1))]); }      // lane p holds V[p]
    void const *rows[N];
    int ins[N];
#pragma unroll
    for (int k = 0; k < N; ++k) {
        ins[k] = a.idx[node * N + k];
        rows[k] = (XMODE == kXBit) ? (void const *)(reinterpret_cast<uint32_t const *>(a.x) + (size_t)ins[k] * a.x_stride)
                                   : (void const *)(reinterpret_cast<float const *>(a.x) + (size_t)ins[k] * a.x_stride);
    }
    float const *__restrict__ dyr = a.dy + (size_t)node * a.dy_stride;

    float mean = 0.0f, rstd = 1.0f, dmean = 0.0f, dvarf = 0.0f;
    if (BWD_KIND != 0) { mean = a.mean[node]; rstd = a.rstd[node]; }
    if (BWD_KIND == 1) {
        if (a.stat_partial) {
            float s0, s1, dv;
            wave_stat_sums(a.stat_partial, a.node_size, a.stat_count, node, lane, s0, s1);
            batch_gradient_statistics(s0, s1, mean, rstd, a.gamma, a.frame_size, dmean, dv);
            dvarf = dv * a.inv_frames;
        }
        else { dmean = a.dmean[node]; dvarf = a.dvar[node] * a.inv_frames; }
        dmean = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(dmean)));       // the same in every lane
        dvarf = __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(dvarf)));
    }
    float const grs = a.gamma * rstd;
    int corner_open = 0;        // lane p: 1 where the batch-norm output of corner p lies inside the hard-tanh window, else 0
    if (CORNER) {
        float const t = batch_norm_output(__int_as_float(corner), mean, rstd, a.gamma, a.beta);
        corner_open = (t <= 0.0f || t >= 1.0f) ? 0 : 1;
    }

    int const f_begin = a.f_base + sl * a.slab;
    int const f_end   = min(f_begin + a.slab, a.f_limit);
    int const f_last  = a.frame_size - 1;

    float acc[D::NN];
#pragma unroll
    for (int i = 0; i < D::NN; ++i) { acc[i] = 0.0f; }

    constexpr int U = 2;                         // wavefront-steps whose loads are issued together
    // packed-bit inputs are scalar lane masks: where the table already fills the scalar registers they are fetched step by step
    constexpr bool kLateGather = (XMODE == kXBit) && kNeedTable;
    for (int fb = f_begin; fb < f_end; fb += kWave * U) {
        typename Gather<N, XMODE>::Raw raw[U][N];
        float dyv[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            int const fs = min(fb + u * kWave + lane, f_last);
            if (!kLateGather) { Gather<N, XMODE>::load_raw(rows, fb + u * kWave, lane, f_last, raw[u]); }
            dyv[u] = *reinterpret_cast<float const *>(reinterpret_cast<char const *>(dyr) + (uint32_t)fs * 4u);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            int const f0 = fb + u * kWave;
            if (f0 >= f_end) { break; }
            int const  f  = f0 + lane;
            bool const ok = f < f_end;
            float z[N];
            if (kLateGather) { Gather<N, XMODE>::load_raw(rows, f0, lane, f_last, raw[u]); }
            Gather<N, XMODE>::centre_all(raw[u], a.bias, z);
            float d = ok ? dyv[u] : 0.0f;

            float zl[D::NL], zh[D::NH];
#pragma unroll
            for (int k = 0; k < D::NL; ++k) { zl[k] = z[k]; }
#pragma unroll
            for (int k = 0; k < D::NH; ++k) { zh[k] = z[D::NL + k]; }
            float l[D::L], h[D::H], q[D::H];
            monomials<D::NL>(zl, l);
            monomials<D::NH>(zh, h);
            if (kNeedTable) { LutEval<N>::partial_q(C, cv, l, q); }

            if (BWD_KIND != 0) {
                // hard-tanh window on the batch-norm output (reference: DifferentiableLutN.h:1206-1211, 1241-1246)
                float v;
                if constexpr (CORNER) {
                    // the window depends on the corner alone: lane p decided it for corner p before the loop (same operations)
                    int const index4 = (int)(corner_index<N, XMODE>(raw[u]) << 2);
                    v = __int_as_float(__builtin_amdgcn_ds_bpermute(index4, corner));
                    if (__builtin_amdgcn_ds_bpermute(index4, corner_open) == 0) { d = 0.0f; }
                }
                else {
                    v = LutEval<N>::combine(h, q);
                    float const t = batch_norm_output(v, mean, rstd, a.gamma, a.beta);
                    if (t <= 0.0f || t >= 1.0f) { d = 0.0f; }
                }
                // dL/d(LUT output) (reference: DifferentiableLutN.h:1248-1250)
                d = ok ? (__builtin_fmaf(d, grs, dmean) + v * dvarf) : 0.0f;
                if (DXMODE == kDxNone && ok) { a.dx[(size_t)node * a.dx_stride + f] = d; }
            }

            float g[D::H];
            g[0] = d;
#pragma unroll
            for (int j = 1; j < D::H; ++j) { g[j] = d * h[j]; }

            // table gradient in the centred basis
#pragma unroll
            for (int j = 0; j < D::H; ++j) {
                acc[j * D::L] += g[j];
#pragma unroll
                for (int i = 1; i < D::L; ++i) { acc[j * D::L + i] = __builtin_fmaf(g[j], l[i], acc[j * D::L + i]); }
            }

            if (DXMODE == kDxNone) { continue; }

            // input gradients
            float p[D::L];
#pragma unroll
            for (int i = 0; i < D::L; ++i) {
                float s = g[0] * C[i];
#pragma unroll
                for (int j = 1; j < D::H; ++j) { s = __builtin_fmaf(g[j], C[j * D::L + i], s); }
                p[i] = s;
            }
            float dxl[D::NL], dxh[D::NH];
            LutEval<N>::template group_grad<D::NL>(l, p, dxl);
            LutEval<N>::template group_grad<D::NH>(h, q, dxh);
#pragma unroll
            for (int k = 0; k < D::NH; ++k) { dxh[k] *= d; }

            if (ok) {
#pragma unroll
                for (int k = 0; k < N; ++k) {
                    float const val = (k < D::NL) ? dxl[k < D::NL ? k : 0] : dxh[k >= D::NL ? k - D::NL : 0];
                    if (DXMODE == kDxAtomic) {
                        unsafeAtomicAdd(a.dx + (size_t)ins[k] * a.dx_stride + f, val);
                    }
                    else {
                        a.dx[(size_t)(node * N + k) * a.dx_stride + (f - a.f_base)] = val;
                    }
                }
            }
        }
    }

    // frame reduction of the 2^N per-lane accumulators through LDS, 16 at a time:
    // lane i sums accumulator (i / 4), lanes (i % 4) * 16 .. + 15, then the 4 quarter sums are combined.
    float *out = a.dw_partial + ((size_t)(a.slab_first + sl) * a.node_size + node) * D::NN;
    constexpr int PASS = (D::NN + 15) / 16;
#pragma unroll
    for (int ps = 0; ps < PASS; ++ps) {
        constexpr int CNT = D::NN < 16 ? D::NN : 16;
#pragma unroll
        for (int r = 0; r < CNT; ++r) { red[wv][r][lane] = acc[ps * 16 + r]; }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        int const r  = lane >> 2;
        int const qd = lane & 3;
        float s = 0.0f;
        if (r < CNT) {
#pragma unroll
            for (int t = 0; t < 16; ++t) { s += red[wv][r][qd * 16 + t]; }
        }
        s += __shfl_xor(s, 1, 64);
        s += __shfl_xor(s, 2, 64);
        if (qd == 0 && r < CNT) { out[ps * 16 + r] = s; }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
}

struct DxArgs {
    void const  *x;
    float const *dy;            // dL/d(LUT output) [O][dy_stride]
    float       *dx;            // [I][dx_stride]
    int const   *rev;           // reverse table [I][rev_stride]: count, then connection ids node*N + k
    int const   *term;          // term table, see term_table_block
    int   rev_stride, input_node_size, frame_size;
    int   x_stride, dy_stride, dx_stride;
    int   chunk, chunk_count;
    TileDivisor tiles;
    float bias;
    // split != 0: the four wavefronts of a workgroup share ONE input node and a quarter of its work list each; their sums are
    // added in wavefront order through LDS.  For layers with few input nodes and long lists (784 inputs feeding 6144 nodes:
    // 47 consumers each), where one wavefront per (input, unit) leaves most of the device idle behind a long serial walk.
    // tiles then counts input nodes, not groups of four.
    int   split;
    // the last fin_blocks workgroups of the launch fold the table-gradient partial sums into dW (dw_finalize_block)
    float const *fin_partial;
    float       *fin_dW;
    int   fin_node_size, fin_slab_count, fin_blocks;
    int   fin_overwrite;        // dW = instead of dW += (the caller's dW holds nothing: bbhip_HintTableGradientOverwrite)
    int   own_stride;           // lut_dx_indexed_kernel: words per node row of the kept corner indices
};

// ------------------------------------------------------------------------------------------------
//  input-centric dx: one wavefront owns dx[input node][64 frames x U] and walks the node's fan-out list
//  (the reverse table, in its ascending (node, input) order), re-evaluating dy/dx_k of each consumer from that
//  consumer's other N-1 inputs.  By multilinearity dy/dx_k is itself a LUT over the other inputs; in the plain
//  monomial basis  y = sum_S P[S] prod_{j in S} x_j  its coefficients are the entries of P with bit k set:
//  Dk[s] = P[insert_zero_bit(s, k) | (1 << k)].  This kernel uses the plain basis (no centring subtraction per
//  operand; |P| <= 2^N |W| keeps the rounding error of the 2^(N-1)-term sum near 1e-6 of the gradient scale).
//  The low ML variables are expanded into monomials (wave-uniform coefficients, one FMA each), the high MH variables
//  are folded by Horner's rule.  No scratch traffic, no atomics; every dx element is written exactly once, summed in
//  the reference's order.
//
//  Rows are read through buffer descriptors (base = the row, extent = its valid bytes): the vector offset stays a
//  32-bit register shared by all loads of a pass, and lanes beyond the last frame read 0 instead of needing a clamp.
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ __amdgpu_buffer_rsrc_t row_descriptor(void const *base, int row, int stride_elems, uint32_t row_bytes)
{
    char const *p = reinterpret_cast<char const *>(base) + (size_t)row * (size_t)stride_elems * 4u;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(p), 0, (int)row_bytes, 0x00020000);
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t address_descriptor(uint32_t addr_lo, uint32_t addr_hi, uint32_t row_bytes)
{
    uint64_t const p = ((uint64_t)addr_hi << 32) | addr_lo;
    return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<char *>(p), 0, (int)row_bytes, 0x00020000);
}

// value of one input as the LUT sees it (reference: include/bb/StochasticLutN.h:536-553)
template <int XMODE>
__device__ __forceinline__ float input_value(uint32_t raw, int bit, float lo, float hi)
{
    if (XMODE == kXClamp)  { return __builtin_amdgcn_fmed3f(__uint_as_float(raw), 0.0f, 1.0f); }
    if (XMODE == kXBinary) { return (__uint_as_float(raw) > 0.5f) ? hi : lo; }
    return ((raw >> bit) & 1u) ? hi : lo;
}

// One term of the work list.  The gathered rows live in a Stage (vector registers); the coefficients are fetched
// into scalar registers right before the term is evaluated.
template <int N, int XMODE, int U>          // U wavefront-steps per pass
struct DxTerm {
    static constexpr int M  = N - 1;        // variables of the derivative LUT
    static constexpr int ML = M / 2, MH = M - ML;
    static constexpr int L = 1 << ML, H = 1 << MH, HN = 1 << M, REC = kTermHead + HN;

    struct Stage {
        uint32_t raw[U][M];
        float    dyv[U];
    };

    // vector loads of the U x (M + 1) operands of the record at rec (its head is read with scalar loads).
    // xoff / yoff: byte offset of this lane's element (word for packed rows) in the first step of the pass
    template <typename RecPtr>
    __device__ __forceinline__ static void issue(RecPtr rec, uint32_t xoff, uint32_t yoff,
                                                 uint32_t x_row_bytes, uint32_t y_row_bytes, Stage &st)
    {
        constexpr uint32_t xstep = (XMODE == kXBit) ? (kWave / 32) * 4u : kWave * 4u;
#pragma unroll
        for (int j = 0; j < M; ++j) {
            __amdgpu_buffer_rsrc_t const r = address_descriptor((uint32_t)rec[2 * j], (uint32_t)rec[2 * j + 1], x_row_bytes);
#pragma unroll
            for (int u = 0; u < U; ++u) { st.raw[u][j] = __builtin_amdgcn_raw_buffer_load_b32(r, xoff + u * xstep, 0, 0); }
        }
        __amdgpu_buffer_rsrc_t const dyr = address_descriptor((uint32_t)rec[2 * M], (uint32_t)rec[2 * M + 1], y_row_bytes);
#pragma unroll
        for (int u = 0; u < U; ++u) { st.dyv[u] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(dyr, yoff + u * (kWave * 4u), 0, 0)); }
    }

    template <typename RecPtr>
    __device__ __forceinline__ static void load_coefficients(RecPtr rec, float (&Dk)[HN])
    {
#pragma unroll
        for (int sidx = 0; sidx < HN; ++sidx) { Dk[sidx] = __int_as_float(rec[kTermHead + sidx]); }
    }

    __device__ __forceinline__ static void accumulate(Stage const &st, float const (&Dk)[HN], int bit, float lo, float hi, float (&acc)[U])
    {
        // constant terms of the H partial sums in vector registers: an FMA reads at most one scalar register
        float cv[H];
        if (L > 1) {
#pragma unroll
            for (int j = 0; j < H; ++j) { asm("v_mov_b32 %0, %1" : "=v"(cv[j]) : "s"(Dk[j * L])); }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            float xv[M];
#pragma unroll
            for (int k = 0; k < M; ++k) { xv[k] = input_value<XMODE>(st.raw[u][k], bit, lo, hi); }
            float xl[ML > 0 ? ML : 1];
#pragma unroll
            for (int k = 0; k < ML; ++k) { xl[k] = xv[k]; }
            float l[L];
            monomials<ML>(xl, l);
            float q[H];
#pragma unroll
            for (int j = 0; j < H; ++j) {
                float s = (L > 1) ? cv[j] : Dk[j * L];
#pragma unroll
                for (int i = 1; i < L; ++i) { s = __builtin_fmaf(l[i], Dk[j * L + i], s); }
                q[j] = s;
            }
            // Horner over the high variables: bit v of j belongs to xv[ML + v]
#pragma unroll
            for (int v = 0; v < MH; ++v) {
#pragma unroll
                for (int s = 0; s < (H >> (v + 1)); ++s) { q[s] = __builtin_fmaf(xv[ML + v], q[2 * s + 1], q[2 * s]); }
            }
            acc[u] = __builtin_fmaf(st.dyv[u], q[0], acc[u]);
        }
    }
};

// The wavefront's share of an input node's work list (the whole list, or a quarter of it in split mode) ...
__device__ __forceinline__ void dx_list_share(DxArgs const &a, int tile, int wave, int &in, int &t_scale)
{
    // (the wavefront's number within the workgroup is the same in all its lanes; saying so keeps everything derived from it —
    // list bounds, record addresses — in scalar registers and on scalar loads)
    int const w = __builtin_amdgcn_readfirstlane(wave);
    in      = __builtin_amdgcn_readfirstlane(a.split ? tile : tile * kWavesPerBlk + w);
    t_scale = a.split ? w : -1;
}
__device__ __forceinline__ void dx_list_range(int cnt, int share, int &t_begin, int &t_end)
{
    t_begin = (share < 0) ? 0   : (cnt * share) / kWavesPerBlk;
    t_end   = (share < 0) ? cnt : (cnt * (share + 1)) / kWavesPerBlk;
}

// ... and the end of a pass: the lane's U sums go to dx — directly, or in split mode added over the workgroup's wavefronts
// in wavefront order (a fixed order: results do not depend on timing) by the first of them.  Every wavefront of the
// workgroup must come here (the barrier).
template <int U>
__device__ __forceinline__ void dx_store_pass(DxArgs const &a, float (&part)[kWavesPerBlk][U][kWave], int in, int wave, int lane,
                                              int f_begin, float (&acc)[U])
{
    if (a.split) {
#pragma unroll
        for (int u = 0; u < U; ++u) { part[wave][u][lane] = acc[u]; }
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float sum = part[0][u][lane];
#pragma unroll
                for (int w = 1; w < kWavesPerBlk; ++w) { sum += part[w][u][lane]; }
                acc[u] = sum;
            }
        }
        __syncthreads();                    // the next pass writes part again
        if (wave != 0) { return; }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        int const f = f_begin + u * kWave + lane;
        if (f < a.frame_size) { __builtin_nontemporal_store(acc[u], a.dx + (size_t)in * a.dx_stride + f); }
    }
}

template <int N, int XMODE, int U>
__global__ __launch_bounds__(kBlock) void lut_dx_kernel(DxArgs a)
{
    using T = DxTerm<N, XMODE, U>;
    // the table-gradient partial sums are complete before this launch and independent of it: folding them into dW rides at
    // the end of this launch instead of taking a launch of its own
    int const bid = blockIdx.x;
    int const B   = a.chunk_count * a.tiles.count;
    if (bid >= B) { dw_finalize_block<N>(a.fin_partial, a.fin_dW, a.fin_node_size, a.fin_slab_count, bid - B, a.fin_overwrite); return; }
    int const lid  = xcd_remap(bid, B);
    int ck, tile;
    split_tile(lid, a.tiles, ck, tile);
    __shared__ float part[kWavesPerBlk][U][kWave];
    int const wave = threadIdx.x / kWave;
    int in, share;
    dx_list_share(a, tile, wave, in, share);
    if (in >= a.input_node_size) { return; }            // (workgroup-uniform in split mode)
    int const lane = threadIdx.x & (kWave - 1);

    int const cnt = a.rev[(size_t)in * a.rev_stride];
    int t_begin, t_end;
    dx_list_range(cnt, share, t_begin, t_end);
    // The term table is read through the constant address space: its wave-uniform loads stay scalar loads wherever
    // they are placed relative to the stores of this kernel (the table is written by an earlier kernel).
    typedef __attribute__((address_space(4))) int const const_int;
    const_int *rec = (const_int *)(a.term + (size_t)in * (a.rev_stride - 1) * T::REC);
    uint32_t const y_row_bytes = (uint32_t)a.frame_size * 4u;
    uint32_t const x_row_bytes = (XMODE == kXBit) ? (uint32_t)((a.frame_size + 31) >> 5) * 4u : y_row_bytes;
    float const lo = 0.5f - a.bias, hi = 0.5f + a.bias;
    int const bit = lane & 31;

    // a unit is a.chunk frames = several passes of 64 * U frames; the node's work list is walked once per pass.
    // (Requesting the operands of later terms ahead of time — a ring of stages — was measured slower at every depth:
    // with 8 wavefronts per SIMD the other wavefronts already cover the latency, and more loads in flight only
    // lengthen the queues.)
    for (int f_begin = ck * a.chunk; f_begin < min((ck + 1) * a.chunk, a.frame_size); f_begin += kWave * U) {
        uint32_t const f0   = (uint32_t)(f_begin + lane);
        uint32_t const yoff = f0 * 4u;
        uint32_t const xoff = (XMODE == kXBit) ? (f0 >> 5) * 4u : yoff;
        float acc[U];
#pragma unroll
        for (int u = 0; u < U; ++u) { acc[u] = 0.0f; }

        // the head (row addresses) of the next term is requested while the current term is evaluated, so that a term's
        // loads do not wait for a scalar-memory round trip first
        constexpr int HEAD = 2 * T::M + 2;
        int head_next[HEAD];
        if (t_begin < t_end) {
#pragma unroll
            for (int i = 0; i < HEAD; ++i) { head_next[i] = rec[(size_t)t_begin * T::REC + i]; }
        }
        for (int t = t_begin; t < t_end; ++t) {
            typename T::Stage st;
            float Dk[T::HN];
            int head[HEAD];
#pragma unroll
            for (int i = 0; i < HEAD; ++i) { head[i] = head_next[i]; }
            if (t + 1 < t_end) {
#pragma unroll
                for (int i = 0; i < HEAD; ++i) { head_next[i] = rec[(size_t)(t + 1) * T::REC + i]; }
            }
            T::issue(head, xoff, yoff, x_row_bytes, y_row_bytes, st);
            T::load_coefficients(rec + (size_t)t * T::REC, Dk);
            T::accumulate(st, Dk, bit, lo, hi, acc);
        }
        dx_store_pass<U>(a, part, in, wave, lane, f_begin, acc);
    }
}

// ------------------------------------------------------------------------------------------------
//  Input-centric dx for two-valued inputs (packed bits, fp32 binarized at 0.5).  A term's dy/dx_k is one of 2^(N-1)
//  values, chosen by the other inputs' bits: the term record holds that table (term_table_block with corner = 1), lane p
//  keeps entry p, and a lane fetches the entry of its frame with ds_bpermute: about a dozen vector instructions per term
//  and step instead of the polynomial's 43.  Units, work list and the dW rider are those of lut_dx_kernel; fp32 rows are
//  loaded as there and compared with 0.5, packed rows take one load per row and pass (see below).
// ------------------------------------------------------------------------------------------------
template <int N, int XMODE, int U, bool WIDE = false>
__global__ __launch_bounds__(kBlock) void lut_dx_corner_kernel(DxArgs a)
{
    static_assert(XMODE == kXBit || XMODE == kXBinary, "corner values need two-valued inputs");
    static_assert(!WIDE || XMODE == kXBit, "scalar loads of whole passes are for packed rows");
    using T = DxTerm<N, XMODE, U>;
    int const bid = blockIdx.x;
    int const B   = a.chunk_count * a.tiles.count;
    if (bid >= B) { dw_finalize_block<N>(a.fin_partial, a.fin_dW, a.fin_node_size, a.fin_slab_count, bid - B, a.fin_overwrite); return; }
    int const lid  = xcd_remap(bid, B);
    int ck, tile;
    split_tile(lid, a.tiles, ck, tile);
    __shared__ float part[kWavesPerBlk][U][kWave];
    int const wave = threadIdx.x / kWave;
    int in, share;
    dx_list_share(a, tile, wave, in, share);
    if (in >= a.input_node_size) { return; }            // (workgroup-uniform in split mode)
    int const lane = threadIdx.x & (kWave - 1);

    int const cnt = a.rev[(size_t)in * a.rev_stride];
    int t_begin, t_end;
    dx_list_range(cnt, share, t_begin, t_end);
    typedef __attribute__((address_space(4))) int const const_int;
    const_int *rec = (const_int *)(a.term + (size_t)in * (a.rev_stride - 1) * T::REC);
    int const *rec_v = a.term + (size_t)in * (a.rev_stride - 1) * T::REC + kTermHead + (lane & (T::HN - 1));
    uint32_t const y_row_bytes = (uint32_t)a.frame_size * 4u;
    uint32_t const x_row_bytes = (XMODE == kXBit) ? (uint32_t)((a.frame_size + 31) >> 5) * 4u : y_row_bytes;

    for (int f_begin = ck * a.chunk; f_begin < min((ck + 1) * a.chunk, a.frame_size); f_begin += kWave * U) {
        uint32_t const f0   = (uint32_t)(f_begin + lane);
        uint32_t const yoff = f0 * 4u;
        uint32_t const xoff = (XMODE == kXBit) ? (f0 >> 5) * 4u : yoff;
        uint32_t const wordoff = ((uint32_t)(f_begin >> 5) + (uint32_t)(lane & (2 * U - 1))) * 4u;      // packed rows: word (lane mod 2 U) of the pass
        float acc[U];
#pragma unroll
        for (int u = 0; u < U; ++u) { acc[u] = 0.0f; }

        // Packed rows: a term is a round trip — its head (row addresses, scalar loads), then the rows' words and dy — and a few
        // dozen instructions, so the walk is bound by latency.  Two terms are in flight: while term t is evaluated, the rows of
        // term t + 1 have been requested and the head of term t + 2 is on its way.
        if constexpr (XMODE == kXBit) {
            // The 64 U frames of a pass are 2 U words of a packed row, the same for every lane: one load per row brings them
            // in (lane i holds word i of the pass), each step's two words are read back as a lane mask, and the index costs
            // one add-with-carry per input.  Per term and pass: M + U + 1 vector memory instructions instead of (M + 1) U + 1.
            constexpr int HEAD = 2 * T::M + 2;
            int head[HEAD];
            uint32_t w_next[T::M];
            float dy_next[U];
            int values_next = 0;
            auto load_head = [&](int t) {
#pragma unroll
                for (int i = 0; i < HEAD; ++i) { head[i] = rec[(size_t)t * T::REC + i]; }
            };
            auto request_rows = [&](int t) {                      // of the term whose head is in `head`
#pragma unroll
                for (int j = 0; j < T::M; ++j) {
                    __amdgpu_buffer_rsrc_t const d = address_descriptor((uint32_t)head[2 * j], (uint32_t)head[2 * j + 1], x_row_bytes);
                    w_next[j] = __builtin_amdgcn_raw_buffer_load_b32(d, wordoff, 0, 0);
                }
                __amdgpu_buffer_rsrc_t const dyr = address_descriptor((uint32_t)head[2 * T::M], (uint32_t)head[2 * T::M + 1], y_row_bytes);
#pragma unroll
                for (int u = 0; u < U; ++u) { dy_next[u] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(dyr, yoff + u * (kWave * 4u), 0, 0)); }
                values_next = rec_v[(size_t)t * T::REC];        // lane p: the term's value at corner p
            };
            if constexpr (WIDE) {
                // Row pitch a multiple of 2 U words: the 2 U words of a pass are ONE scalar load per row (32 bytes with U = 4), each
                // step's lane mask is a register pair of it, and the 2 M U read-lanes of the form below go away (a third of this
                // kernel's instructions).  A term's corner indices are formed one term ahead, as soon as its words are there,
                // so only the head of term t + 2 and the words of term t + 1 sit in scalar registers.
                typedef uint32_t u32x8 __attribute__((ext_vector_type(2 * U)));
                typedef __attribute__((address_space(4))) u32x8 const const_u32x8;
                uint32_t index_next[U];
                auto request_wide = [&](int t) {                  // of the term whose head is in `head`: its indices, dy, values
                    u32x8 wq[T::M];
#pragma unroll
                    for (int j = 0; j < T::M; ++j) {
                        uint64_t const row = ((uint64_t)(uint32_t)head[2 * j + 1] << 32) | (uint32_t)head[2 * j];
                        wq[j] = *(const_u32x8 *)(row + (uint64_t)(uint32_t)(f_begin >> 5) * 4u);
                    }
                    __amdgpu_buffer_rsrc_t const dyr = address_descriptor((uint32_t)head[2 * T::M], (uint32_t)head[2 * T::M + 1], y_row_bytes);
#pragma unroll
                    for (int u = 0; u < U; ++u) { dy_next[u] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(dyr, yoff + u * (kWave * 4u), 0, 0)); }
                    values_next = rec_v[(size_t)t * T::REC];
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        uint32_t index = 0;                        // most significant input first: index = 2 index + bit
#pragma unroll
                        for (int j = T::M - 1; j >= 0; --j) {
                            uint64_t const mask = (uint64_t)wq[j][2 * u] | ((uint64_t)wq[j][2 * u + 1] << 32);
                            uint64_t carry;
                            asm("v_addc_co_u32_e64 %0, %1, %2, %2, %3" : "=v"(index), "=s"(carry) : "v"(index), "s"(mask));
                        }
                        index_next[u] = index << 2;
                    }
                };
                if (t_begin < t_end) {
                    load_head(t_begin);
                    request_wide(t_begin);
                    if (t_begin + 1 < t_end) { load_head(t_begin + 1); }
                }
                for (int t = t_begin; t < t_end; ++t) {
                    uint32_t idx4[U];
                    float dyv[U];
#pragma unroll
                    for (int u = 0; u < U; ++u) { idx4[u] = index_next[u]; dyv[u] = dy_next[u]; }
                    int const values = values_next;
                    if (t + 1 < t_end) {
                        request_wide(t + 1);
                        if (t + 2 < t_end) { load_head(t + 2); }
                    }
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        float const d = __int_as_float(__builtin_amdgcn_ds_bpermute((int)idx4[u], values));
                        acc[u] = __builtin_fmaf(dyv[u], d, acc[u]);
                    }
                }
                dx_store_pass<U>(a, part, in, wave, lane, f_begin, acc);
                continue;
            }
            if (t_begin < t_end) {
                load_head(t_begin);
                request_rows(t_begin);
                if (t_begin + 1 < t_end) { load_head(t_begin + 1); }
            }
            for (int t = t_begin; t < t_end; ++t) {
                uint32_t w[T::M];
                float dyv[U];
#pragma unroll
                for (int j = 0; j < T::M; ++j) { w[j] = w_next[j]; }
#pragma unroll
                for (int u = 0; u < U; ++u) { dyv[u] = dy_next[u]; }
                int const values = values_next;
                if (t + 1 < t_end) {
                    request_rows(t + 1);
                    if (t + 2 < t_end) { load_head(t + 2); }
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    uint32_t index = 0;                            // most significant input first: index = 2 index + bit
#pragma unroll
                    for (int j = T::M - 1; j >= 0; --j) {
                        uint64_t const mask = (uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)w[j], 2 * u) |
                                              ((uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)w[j], 2 * u + 1) << 32);
                        uint64_t carry;
                        asm("v_addc_co_u32_e64 %0, %1, %2, %2, %3" : "=v"(index), "=s"(carry) : "v"(index), "s"(mask));
                    }
                    float const d = __int_as_float(__builtin_amdgcn_ds_bpermute((int)(index << 2), values));
                    acc[u] = __builtin_fmaf(dyv[u], d, acc[u]);
                }
            }
            dx_store_pass<U>(a, part, in, wave, lane, f_begin, acc);
            continue;
        }
        for (int t = t_begin; t < t_end; ++t) {
            int const values = rec_v[(size_t)t * T::REC];          // lane p: the term's value at corner p
            typename T::Stage st;
            T::issue(rec + (size_t)t * T::REC, xoff, yoff, x_row_bytes, y_row_bytes, st);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                uint32_t index = 0;
#pragma unroll
                for (int j = 0; j < T::M; ++j) { index |= (__uint_as_float(st.raw[u][j]) > 0.5f) ? (4u << j) : 0u; }
                float const d = __int_as_float(__builtin_amdgcn_ds_bpermute((int)index, values));
                acc[u] = __builtin_fmaf(st.dyv[u], d, acc[u]);
            }
        }
        dx_store_pass<U>(a, part, in, wave, lane, f_begin, acc);
    }
}

// ------------------------------------------------------------------------------------------------
//  Input-centric dx from kept corner indices (batch-norm backward over two-valued inputs).  The statistics pass of the same
//  call has formed the corner index of every (node, frame) and kept it, a byte each (FwdArgs::own_index_out); a term's
//  dy/dx_k is its record's value at that corner (term_table_node_block with indexed = 1), so a term costs per pass one word of
//  indices and four of dy per lane, and per step a byte extract, ds_bpermute and the multiply-add: no row of the other inputs
//  is read and no index is formed.  Units (multiples of 256 frames), work list, split mode and the dW rider are those of
//  lut_dx_corner_kernel, and so is the order of the sums: the same bits.
// ------------------------------------------------------------------------------------------------
template <int N>
__global__ __launch_bounds__(kBlock) void lut_dx_indexed_kernel(DxArgs a)
{
    constexpr int U = 4, NN = 1 << N, REC = kTermHead + NN, HEAD = 4;
    int const bid = blockIdx.x;
    int const B   = a.chunk_count * a.tiles.count;
    if (bid >= B) { dw_finalize_block<N>(a.fin_partial, a.fin_dW, a.fin_node_size, a.fin_slab_count, bid - B, a.fin_overwrite); return; }
    int const lid  = xcd_remap(bid, B);
    int ck, tile;
    split_tile(lid, a.tiles, ck, tile);
    __shared__ float part[kWavesPerBlk][U][kWave];
    int const wave = threadIdx.x / kWave;
    int in, share;
    dx_list_share(a, tile, wave, in, share);
    if (in >= a.input_node_size) { return; }            // (workgroup-uniform in split mode)
    int const lane = threadIdx.x & (kWave - 1);

    int const cnt = a.rev[(size_t)in * a.rev_stride];
    int t_begin, t_end;
    dx_list_range(cnt, share, t_begin, t_end);
    typedef __attribute__((address_space(4))) int const const_int;
    const_int *rec = (const_int *)(a.term + (size_t)in * (a.rev_stride - 1) * REC);
    int const *rec_v = a.term + (size_t)in * (a.rev_stride - 1) * REC + kTermHead + (lane & (NN - 1));
    uint32_t const y_row_bytes = (uint32_t)a.frame_size * 4u;
    uint32_t const i_row_bytes = (uint32_t)a.own_stride * 4u;

    for (int f_begin = ck * a.chunk; f_begin < min((ck + 1) * a.chunk, a.frame_size); f_begin += kWave * U) {
        uint32_t const yoff = (uint32_t)(f_begin + lane) * 4u;
        uint32_t const ioff = ((uint32_t)(f_begin >> 8) * kWave + (uint32_t)lane) * 4u;     // byte u of the word: frame f_begin + 64 u + lane
        float acc[U];
#pragma unroll
        for (int u = 0; u < U; ++u) { acc[u] = 0.0f; }

        // two terms in flight, as in lut_dx_corner_kernel: while term t is evaluated, the words of term t + 1 have been
        // requested and the head of term t + 2 is on its way (four in flight measured slower: 136 vs 128 us at 4096 x 4096 x 8192)
        int head[HEAD];
        uint32_t iw_next = 0;
        float dy_next[U];
        int values_next = 0;
        auto load_head = [&](int t) {
#pragma unroll
            for (int i = 0; i < HEAD; ++i) { head[i] = rec[(size_t)t * REC + i]; }
        };
        auto request = [&](int t) {                           // of the term whose head is in `head`
            __amdgpu_buffer_rsrc_t const ir = address_descriptor((uint32_t)head[0], (uint32_t)head[1], i_row_bytes);
            iw_next = __builtin_amdgcn_raw_buffer_load_b32(ir, ioff, 0, 0);
            __amdgpu_buffer_rsrc_t const dyr = address_descriptor((uint32_t)head[2], (uint32_t)head[3], y_row_bytes);
#pragma unroll
            for (int u = 0; u < U; ++u) { dy_next[u] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(dyr, yoff + u * (kWave * 4u), 0, 0)); }
            values_next = rec_v[(size_t)t * REC];              // lane p: the term's value at corner p
        };
        if (t_begin < t_end) {
            load_head(t_begin);
            request(t_begin);
            if (t_begin + 1 < t_end) { load_head(t_begin + 1); }
        }
        for (int t = t_begin; t < t_end; ++t) {
            uint32_t const iw = iw_next;
            float dyv[U];
#pragma unroll
            for (int u = 0; u < U; ++u) { dyv[u] = dy_next[u]; }
            int const values = values_next;
            if (t + 1 < t_end) {
                request(t + 1);
                if (t + 2 < t_end) { load_head(t + 2); }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float const d = __int_as_float(__builtin_amdgcn_ds_bpermute((int)((iw >> (8 * u)) & 0xffu), values));
                acc[u] = __builtin_fmaf(dyv[u], d, acc[u]);
            }
        }
        dx_store_pass<U>(a, part, in, wave, lane, f_begin, acc);
    }
}

// per node: dvar, dmean from the phase-0 sums (reference: DifferentiableLutN.h:1218-1222)
__global__ __launch_bounds__(kBlock) void bn_backward_finalize_kernel(float const *__restrict__ stat_partial,
                                                                     float const *__restrict__ mean, float const *__restrict__ rstd,
                                                                     float *__restrict__ dmean, float *__restrict__ dvar,
                                                                     float gamma, int node_size, int slab_count, int frame_size,
                                                                     int nodes_per_block)
{
    int node;
    float s0, s1;
    if (!sum_stat_partials(stat_partial, node_size, slab_count, nodes_per_block, node, s0, s1)) { return; }
    float dm, dv;
    batch_gradient_statistics(s0, s1, mean[node], rstd[node], gamma, frame_size, dm, dv);
    dvar[node]  = dv;
    dmean[node] = dm;
}

// dx[in][f] = sum_k tmp[rev[in][k]][f - base], k = 1 .. rev[in][0]  (the reference's reverse-table order,
// cuda/Common.cuh:174-202 and include/bb/FixedSizeConnectionTable.h:198-214); overwrites dx
__global__ __launch_bounds__(kBlock) void dx_gather_kernel(float const *__restrict__ tmp, float *__restrict__ dx,
                                                          int const *__restrict__ rev, int rev_stride, int input_node_size,
                                                          int f_base, int f_limit, int dx_stride, int tmp_stride)
{
    int const f  = f_base + blockIdx.x * kBlock + threadIdx.x;
    if (f >= f_limit) { return; }
    for (int in = blockIdx.y; in < input_node_size; in += gridDim.y) {
        int const *r = rev + (size_t)in * rev_stride;
        int const cnt = r[0];
        float s = 0.0f;
        for (int k = 1; k <= cnt; ++k) { s += tmp[(size_t)r[k] * tmp_stride + (f - f_base)]; }
        dx[(size_t)in * dx_stride + f] = s;
    }
}

// ------------------------------------------------------------------------------------------------
//  elementwise helpers
// ------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kBlock) void fill_kernel(float *__restrict__ dst, float v, size_t size)
{
    size_t const i4 = ((size_t)blockIdx.x * kBlock + threadIdx.x) * 4;
    if (i4 + 3 < size && ((uintptr_t)dst & 15) == 0) {
        *reinterpret_cast<float4 *>(dst + i4) = make_float4(v, v, v, v);
    }
    else {
        for (size_t i = i4; i < size && i < i4 + 4; ++i) { dst[i] = v; }
    }
}

__global__ __launch_bounds__(kBlock) void clamp_kernel(float *__restrict__ dst, float const *__restrict__ src, float lo, float hi, int size)
{
    int const i = blockIdx.x * kBlock + threadIdx.x;
    if (i < size) { dst[i] = fminf(hi, fmaxf(lo, src[i])); }
}

// fp32 frames -> packed bits, bit = x > 0.5 (the binarization of binary mode, include/bb/StochasticLutN.h:539): one lane per
// frame, a wavefront writes two words.  Rows of `bits` are y_stride words long; bits beyond the last frame are 0.
__global__ __launch_bounds__(kBlock) void binarize_pack_kernel(float const *__restrict__ x, uint32_t *__restrict__ bits,
                                                               int frame_size, int x_stride, int y_stride)
{
    int const f    = blockIdx.x * kBlock + threadIdx.x;
    int const node = blockIdx.y;
    bool const on  = (f < frame_size) && (x[(size_t)node * x_stride + (f < frame_size ? f : 0)] > 0.5f);
    uint64_t const m = __ballot(on);
    int const lane = threadIdx.x & (kWave - 1);
    int const w = (f & ~(kWave - 1)) >> 5;                 // first word of the wavefront's 64 frames
    if (lane == 0  && w     < y_stride) { bits[(size_t)node * y_stride + w]     = (uint32_t)m; }
    if (lane == 32 && w + 1 < y_stride) { bits[(size_t)node * y_stride + w + 1] = (uint32_t)(m >> 32); }
}

// the same with four frames per lane (16-byte loads; rows 16-byte aligned, x_stride a multiple of 4): a lane's four bits
// are shifted to their place in the word that eight neighbouring lanes share and the eight are combined by three exchanges
__device__ __forceinline__ void binarize_pack4_block(float const *__restrict__ x, uint32_t *__restrict__ bits,
                                                     int frame_size, int x_stride, int y_stride, int node, int block)
{
    int const q    = block * kBlock + threadIdx.x;          // group of four frames
    int const f    = q * 4;
    uint32_t v = 0;
    if (f < frame_size) {
        float4 const t = *reinterpret_cast<float4 const *>(x + (size_t)node * x_stride + f);
        v = (t.x > 0.5f ? 1u : 0u) | ((f + 1 < frame_size && t.y > 0.5f) ? 2u : 0u) |
            ((f + 2 < frame_size && t.z > 0.5f) ? 4u : 0u) | ((f + 3 < frame_size && t.w > 0.5f) ? 8u : 0u);
    }
    v <<= 4 * (threadIdx.x & 7);
    v |= __shfl_xor(v, 1, 64);
    v |= __shfl_xor(v, 2, 64);
    v |= __shfl_xor(v, 4, 64);
    int const w = q >> 3;
    if ((threadIdx.x & 7) == 0 && w < y_stride) { bits[(size_t)node * y_stride + w] = v; }
}

__global__ __launch_bounds__(kBlock) void binarize_pack4_kernel(float const *__restrict__ x, uint32_t *__restrict__ bits,
                                                                int frame_size, int x_stride, int y_stride)
{
    binarize_pack4_block(x, bits, frame_size, x_stride, y_stride, blockIdx.y, blockIdx.x);
}

// Packing and table preparation in one launch: they are independent, and a launch of its own costs each of them more than
// its work.  Workgroups [0, rows * row_blocks.count) pack, the rest prepare the tables.
struct PackPrepArgs {
    float const *x;  uint32_t *bits;  int frame_size, x_stride, y_stride;
    TileDivisor row_blocks;     // workgroups per packed row
    int pack_blocks;            // rows * row_blocks.count
    float const *W;  float *C;  float *V;  int node_size, lut_binarize;  float bias;
    float *clamp_W;  float clamp_lo, clamp_hi;      // see table_prep_block
};

template <int N>
__global__ __launch_bounds__(kBlock) void binarize_pack4_prep_kernel(PackPrepArgs a)
{
    int const bid = blockIdx.x;
    if (bid < a.pack_blocks) {
        int row, block;
        split_tile(bid, a.row_blocks, row, block);
        binarize_pack4_block(a.x, a.bits, a.frame_size, a.x_stride, a.y_stride, row, block);
        return;
    }
    table_prep_block<N>(a.W, a.C, a.node_size, a.lut_binarize, a.V, a.bias, bid - a.pack_blocks, a.clamp_W, a.clamp_lo, a.clamp_hi);
}

// packed bits -> fp32 values (reference: cuda/ConvBitToReal.cu, include/bb/FrameBuffer.h:850-866)
__global__ __launch_bounds__(kBlock) void conv_bit_to_real_kernel(uint32_t const *__restrict__ x, float *__restrict__ y, float v0, float v1,
                                                                 int frame_size, int x_stride, int y_stride)
{
    int const f    = blockIdx.x * kBlock + threadIdx.x;
    int const node = blockIdx.y;
    if (f >= frame_size) { return; }
    uint32_t const w = x[(size_t)node * x_stride + (f >> 5)];
    y[(size_t)node * y_stride + f] = ((w >> (f & 31)) & 1u) ? v1 : v0;
}

// ------------------------------------------------------------------------------------------------
//  BinaryLut6: y = table[x5 x4 x3 x2 x1 x0] on 32 frames per word
//  (reference semantics: include/bb/BinaryLutN.h:436-463 — input k is index bit k, entries 0-31 in table word 0).
//  Evaluated as a 6-level multiplexer tree whose first two levels are replaced by a register lookup: they turn each
//  group of four table entries into one of the 16 Boolean functions of (x0, x1), and which one is the group's table
//  nibble, the same for every frame.  Per word the kernel forms all 16 functions once (12 three-input bit operations),
//  picks the group values out of that register array with the nibbles as wave-uniform register indices while
//  multiplexing by x2 (16 instructions), and finishes with the last three levels (7 bit-selects): 35 vector
//  instructions per word where the plain tree takes 63; the table is held as eight scalar registers per node, one 16-bit
//  index field per nibble.
// ------------------------------------------------------------------------------------------------
// bit-select d = (s & hi) | (~s & lo): one instruction per multiplexer of the tree
__device__ __forceinline__ uint32_t bfi_vvv(uint32_t s, uint32_t hi, uint32_t lo)
{
    uint32_t d;
    asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(d) : "v"(s), "v"(hi), "v"(lo));
    return d;
}

struct BinArgs {
    uint32_t const *x;
    uint32_t       *y;
    int const      *idx;
    int const      *table;      // [O][2]: entries 0-31 in word 0
    int node_size, frame_size, word_count, stride;
    int chunk;                  // words per unit, multiple of 64
    int chunk_count;
    TileDivisor tiles;
};

typedef uint32_t bin_u32x16 __attribute__((ext_vector_type(16)));

// value of a two-input function as x1 varies, for fixed x0: (at x1 = 0, at x1 = 1) -> one of 0, ~0, x1, ~x1
__device__ __forceinline__ uint32_t bin_pick(int at0, int at1, uint32_t x1, uint32_t nx1)
{
    return at0 ? (at1 ? 0xffffffffu : nx1) : (at1 ? x1 : 0u);
}

// The eight level-2 multiplexers t_j = x2 ? fn[nibble 2j+1] : fn[nibble 2j] of a node (sixteen groups of four table
// entries).  The function values sit in fixed registers v48..v63 and are picked with the vector-register index mode:
// while it is on for source 0, source 0 of a vector instruction names register v48 + M0[7:0].  One move fetches the
// x2 = 0 value, one three-input bit operation (truth table 0xe2: source 1 selects between source 0 and source 2)
// fetches the x2 = 1 value and multiplexes.  The mode stays on across the block and M0 is written whole for every pick:
// the node's table is kept as eight scalar registers of two 16-bit fields 0x1000 | nibble (bits 15:12 = index source 0,
// bits 7:0 = the index; bin_index_words), so that a pick costs one scalar instruction (and / shift into M0) where
// extracting the nibble from the packed table and setting the index took two.
__device__ __forceinline__ void bin_select_level2(bin_u32x16 const &fn, uint32_t const (&iw)[8], uint32_t x2, uint32_t (&t)[8])
{
    uint32_t tmp;
    asm volatile(
        "s_set_gpr_idx_on %[w0], gpr_idx(SRC0)\n\t"
        "v_mov_b32 %[tmp], v48\n\t"
        "s_lshr_b32 m0, %[w0], 16\n\t"
        "v_bitop3_b32 %[t0], v48, %[x2], %[tmp] bitop3:0xe2\n\t"
        "s_and_b32 m0, %[w1], 0xffff\n\t"
        "v_mov_b32 %[tmp], v48\n\t"
        "s_lshr_b32 m0, %[w1], 16\n\t"
        "v_bitop3_b32 %[t1], v48, %[x2], %[tmp] bitop3:0xe2\n\t"
        "s_and_b32 m0, %[w2], 0xffff\n\t"
        "v_mov_b32 %[tmp], v48\n\t"
        "s_lshr_b32 m0, %[w2], 16\n\t"
        "v_bitop3_b32 %[t2], v48, %[x2], %[tmp] bitop3:0xe2\n\t"
        "s_and_b32 m0, %[w3], 0xffff\n\t"
        "v_mov_b32 %[tmp], v48\n\t"
        "s_lshr_b32 m0, %[w3], 16\n\t"
        "v_bitop3_b32 %[t3], v48, %[x2], %[tmp] bitop3:0xe2\n\t"
        "s_and_b32 m0, %[w4], 0xffff\n\t"
        "v_mov_b32 %[tmp], v48\n\t"
        "s_lshr_b32 m0, %[w4], 16\n\t"
        "v_bitop3_b32 %[t4], v48, %[x2], %[tmp] bitop3:0xe2\n\t"
        "s_and_b32 m0, %[w5], 0xffff\n\t"
        "v_mov_b32 %[tmp], v48\n\t"
        "s_lshr_b32 m0, %[w5], 16\n\t"
        "v_bitop3_b32 %[t5], v48, %[x2], %[tmp] bitop3:0xe2\n\t"
        "s_and_b32 m0, %[w6], 0xffff\n\t"
        "v_mov_b32 %[tmp], v48\n\t"
        "s_lshr_b32 m0, %[w6], 16\n\t"
        "v_bitop3_b32 %[t6], v48, %[x2], %[tmp] bitop3:0xe2\n\t"
        "s_and_b32 m0, %[w7], 0xffff\n\t"
        "v_mov_b32 %[tmp], v48\n\t"
        "s_lshr_b32 m0, %[w7], 16\n\t"
        "v_bitop3_b32 %[t7], v48, %[x2], %[tmp] bitop3:0xe2\n\t"
        "s_set_gpr_idx_off"
        : [t0] "=&v"(t[0]), [t1] "=&v"(t[1]), [t2] "=&v"(t[2]), [t3] "=&v"(t[3]),
          [t4] "=&v"(t[4]), [t5] "=&v"(t[5]), [t6] "=&v"(t[6]), [t7] "=&v"(t[7]), [tmp] "=&v"(tmp)
        : [w0] "s"(iw[0]), [w1] "s"(iw[1]), [w2] "s"(iw[2]), [w3] "s"(iw[3]), [w4] "s"(iw[4]), [w5] "s"(iw[5]), [w6] "s"(iw[6]), [w7] "s"(iw[7]),
          [x2] "v"(x2),
          "{v48}"(fn[0]), "{v49}"(fn[1]), "{v50}"(fn[2]), "{v51}"(fn[3]), "{v52}"(fn[4]), "{v53}"(fn[5]), "{v54}"(fn[6]), "{v55}"(fn[7]),
          "{v56}"(fn[8]), "{v57}"(fn[9]), "{v58}"(fn[10]), "{v59}"(fn[11]), "{v60}"(fn[12]), "{v61}"(fn[13]), "{v62}"(fn[14]), "{v63}"(fn[15])
        : "scc");                // (M0 is written too: it is reserved, the compiler keeps nothing there across statements)
}

// The index words of a node's table for bin_select_level2: word j holds 0x1000 | nibble 2j in its low half and
// 0x1000 | nibble 2j+1 in its high half (nibble k = table entries 4k .. 4k+3).  Lane j < 8 forms word j with a few vector
// instructions and the eight words are read back into scalar registers: the vector unit has the room, the scalar unit
// does not.
__device__ __forceinline__ void bin_index_words(uint32_t table_lo, uint32_t table_hi, int lane, uint32_t (&iw)[8])
{
    uint32_t const w    = (lane & 4) ? table_hi : table_lo;
    uint32_t const byte = (w >> ((lane & 3) * 8)) & 0xffu;
    uint32_t const v    = 0x10001000u | (byte & 15u) | ((byte >> 4) << 16);
#pragma unroll
    for (int j = 0; j < 8; ++j) { iw[j] = (uint32_t)__builtin_amdgcn_readlane((int)v, j); }
}

template <int NPW, bool EXACT>   // nodes per wavefront; EXACT: the node count is a multiple of NPW, no wavefront has nodes to skip
__global__ __launch_bounds__(kBlock) void binary_lut6_kernel(BinArgs a)
{
    int const B    = a.chunk_count * a.tiles.count;
    int const lid  = xcd_remap(blockIdx.x, B);
    int ck, tile;
    split_tile(lid, a.tiles, ck, tile);
    int const node0 = __builtin_amdgcn_readfirstlane((tile * kWavesPerBlk + (int)(threadIdx.x / kWave)) * NPW);
    if (node0 >= a.node_size) { return; }
    int const lane = threadIdx.x & (kWave - 1);

    uint32_t const row_bytes    = (uint32_t)a.word_count * 4u;
    uint32_t const stride_bytes = (uint32_t)a.stride * 4u;
    // wiring and tables are read through the constant address space: wave-uniform scalar loads wherever the compiler
    // places them relative to the stores of this kernel (neither is written here)
    typedef __attribute__((address_space(4))) int const const_int;
    const_int *idxc = (const_int *)a.idx + (size_t)node0 * 6;
    const_int *tabc = (const_int *)a.table + (size_t)node0 * 2;
    uint32_t iw[NPW][8];                    // the node's table as index words (bin_index_words)
    char const *rows[NPW][6];               // wave-uniform row bases: loads take a scalar base and a 32-bit lane offset
    bool live[NPW];
#pragma unroll
    for (int p = 0; p < NPW; ++p) {
        live[p] = EXACT || (node0 + p < a.node_size);
        int const rel = live[p] ? p : 0;                    // a wavefront past the last node repeats its first one and stores nothing
        bin_index_words((uint32_t)tabc[rel * 2], (uint32_t)tabc[rel * 2 + 1], lane, iw[p]);
#pragma unroll
        for (int k = 0; k < 6; ++k) {
            // unsigned 32 x 32 -> 64 bit: two scalar multiplies and an add with carry per row (the wiring is validated
            // as non-negative by whoever builds it; a signed 64-bit product costs the scalar unit three times as much)
            rows[p][k] = reinterpret_cast<char const *>(a.x) + (uint64_t)(uint32_t)idxc[rel * 6 + k] * (uint64_t)stride_bytes;
        }
    }
    // Outputs of the wavefront's nodes go through one buffer descriptor over their NPW rows, the node's row added as the
    // scalar offset of the store (the range check covers that offset too, so the extent cannot end with a row: lanes
    // beyond the end of a row are masked in the one step of a row that has them).
    __amdgpu_buffer_rsrc_t const yr = row_descriptor(a.y, node0, a.stride, (uint32_t)NPW * stride_bytes);

    int const w_begin = ck * a.chunk;
    int const w_end   = min(w_begin + a.chunk, a.word_count);
    int const w_last  = a.word_count - 1;
    uint32_t const tail_mask = (a.frame_size & 31) ? ((1u << (a.frame_size & 31)) - 1u) : 0xffffffffu;

    uint32_t const last_off = (uint32_t)w_last * 4u;        // lanes beyond the row re-read its last word and store nothing
    uint32_t off = (uint32_t)(w_begin + lane) * 4u;
    for (int w0 = w_begin; w0 < w_end; w0 += kWave, off += kWave * 4u) {
        uint32_t xv[NPW][6];
        uint32_t const at = min(off, last_off);
#pragma unroll
        for (int p = 0; p < NPW; ++p) {
#pragma unroll
            for (int k = 0; k < 6; ++k) { xv[p][k] = *reinterpret_cast<uint32_t const *>(rows[p][k] + at); }
        }
        bool const has_tail = (w0 + kWave > w_last);            // wave-uniform: only the last step of a row
#pragma unroll
        for (int p = 0; p < NPW; ++p) {
            uint32_t const x0 = xv[p][0], x1 = xv[p][1], nx1 = ~x1;
            bin_u32x16 fn;
#pragma unroll
            for (int c = 0; c < 16; ++c) {
                // table position q = x0 + 2 * x1: bit q of c is the function's value there
                uint32_t const g0 = bin_pick(c & 1, (c >> 2) & 1, x1, nx1);          // x0 = 0
                uint32_t const g1 = bin_pick((c >> 1) & 1, (c >> 3) & 1, x1, nx1);   // x0 = 1
                fn[c] = (x0 & g1) | (~x0 & g0);
            }
            uint32_t t[8];
            bin_select_level2(fn, iw[p], xv[p][2], t);
            // the next node's functions are formed after this point, straight into the fixed registers that are free
            // again now (formed earlier, they would have to be moved there: fifteen moves per node)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int lv = 3; lv < 6; ++lv) {
#pragma unroll
                for (int k = 0; k < (32 >> lv); ++k) { t[k] = bfi_vvv(xv[p][lv], t[2 * k + 1], t[2 * k]); }
            }
            uint32_t r = t[0];
            // streamed once (non-temporal): keep it from displacing x rows in L2
            if (live[p]) {
                if (!has_tail) { __builtin_amdgcn_raw_buffer_store_b32(r, yr, off, (uint32_t)p * stride_bytes, 2); }
                else {
                    if (w0 + lane == w_last) { r &= tail_mask; }
                    if (w0 + lane <= w_last) { __builtin_amdgcn_raw_buffer_store_b32(r, yr, off, (uint32_t)p * stride_bytes, 2); }
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
//  BinaryLutN for N = 2 .. 5 (reference: the generic loop of BinaryLutN<N>::Forward, include/bb/BinaryLutN.h:436-463; the
//  reference has a device kernel for N = 6 only).  A table of 2^N <= 32 entries is one word per node.  One thread per (node, word of
//  32 frames): the N input words are the select lines of a multiplexer tree over the table's entries, each entry spread to a word of
//  all ones or all zeros — 2^N - 1 bit-selects per word, whose first level folds into constants.  The node (blockIdx.y), its wiring
//  and its table are the same for the whole workgroup: scalar loads.  Bits of the last word beyond frame_size are written as 0.
// ------------------------------------------------------------------------------------------------
template <int N>
__global__ __launch_bounds__(kBlock) void binary_lutn_kernel(uint32_t const *__restrict__ x, uint32_t *__restrict__ y, int const *__restrict__ idx,
                                                            int const *__restrict__ table, int node0, int frame_size, int stride)
{
    static_assert(N >= 2 && N <= 5, "one table word per node");
    int const node = node0 + (int)blockIdx.y;
    int const w = blockIdx.x * kBlock + threadIdx.x;
    int const words = (frame_size + 31) >> 5;
    if (w >= words) { return; }
    uint32_t const t = (uint32_t)table[node];
    uint32_t sel[N];
#pragma unroll
    for (int k = 0; k < N; ++k) { sel[k] = x[(size_t)idx[node * N + k] * stride + w]; }
    uint32_t v[1 << N];
#pragma unroll
    for (int i = 0; i < (1 << N); ++i) { v[i] = ((t >> i) & 1u) ? 0xffffffffu : 0u; }
#pragma unroll
    for (int k = 0; k < N; ++k) {
#pragma unroll
        for (int i = 0; i < (1 << (N - 1 - k)); ++i) { v[i] = (sel[k] & v[2 * i + 1]) | (~sel[k] & v[2 * i]); }
    }
    uint32_t out = v[0];
    if (w == words - 1 && (frame_size & 31)) { out &= (1u << (frame_size & 31)) - 1u; }
    y[(size_t)node * stride + w] = out;
}

}  // namespace bbhip

// Bench-only instrumentation, not part of the library: bench.py builds this file into bench_gather_probe.so and loads it itself
// (workload "gather_ceiling").  It measures the rate at which the GPU delivers gathered row segments from L2 to the compute
// units, which is the practical ceiling of a kernel with the access pattern of the input-centric dx kernel.
//
//   hipcc --offload-arch=gfx950 -O3 -std=c++17 -fPIC -shared -Xclang -target-feature -Xclang -packed-fp32-ops \
//         bench_gather_probe.hip -o bench_gather_probe.so

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "binarybrain_amd/csrc/tile_divisor.hpp"

namespace bbhip {

constexpr int kWave = 64, kBlock = 256, kWavesPerBlk = kBlock / kWave, kXcd = 8;

// logical workgroup index for hardware workgroup id b of a grid of B: XCD x (= b % 8) owns a contiguous range (as in the library)
__device__ __forceinline__ int xcd_remap(int b, int B)
{
    uint32_t const q = (uint32_t)B / kXcd, r = (uint32_t)B % kXcd;
    uint32_t const x = (uint32_t)b % kXcd, k = (uint32_t)b / kXcd;
    return (int)(x * q + (x < r ? x : r) + k);
}

// ------------------------------------------------------------------------------------------------
//  The gather pattern of lut_dx_kernel without its arithmetic.  One wavefront per (row, unit of P x 64 frames;
//  P = 2 is the dx kernel's unit), units dealt to the XCDs as everywhere; it reads `loads` pseudo-randomly chosen rows'
//  segments of its frame window (P x 256 bytes each), six rows' loads in flight at a time like a dx term, and adds them up.  What this kernel sustains is the rate at
//  which this GPU delivers gathered row segments from L2 to the compute units — the practical ceiling of any kernel with
//  the dx kernel's access pattern.
// ------------------------------------------------------------------------------------------------
template <int P>
__global__ __launch_bounds__(kBlock) void row_gather_probe_kernel(float const *__restrict__ x, float *__restrict__ sink, int rows, int stride,
                                                                  int frame_size, int chunk_count, TileDivisor tiles, int loads)
{
    // P: 64-frame steps per row segment (a segment is P x 256 bytes, read with P loads in flight)
    int const B   = chunk_count * tiles.count;
    int const lid = xcd_remap(blockIdx.x, B);
    int ck, tile;
    split_tile(lid, tiles, ck, tile);
    int const lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    if (tile * kWavesPerBlk + wave >= rows) { return; }
    uint32_t s = (uint32_t)(lid * kWavesPerBlk + wave) * 2654435761u + 12345u;
    int const f_last = frame_size - 1;
    uint32_t off[P];
#pragma unroll
    for (int q = 0; q < P; ++q) { off[q] = (uint32_t)min(ck * (P * kWave) + q * kWave + lane, f_last) * 4u; }
    float acc = 0.0f;
    for (int r = 0; r < loads; r += 6) {
        float v[6][P];
#pragma unroll
        for (int j = 0; j < 6; ++j) {
            s = s * 1664525u + 1013904223u;
            int const row = __builtin_amdgcn_readfirstlane((int)((s >> 8) % (uint32_t)rows));
            char const *p = reinterpret_cast<char const *>(x + (size_t)row * stride);
#pragma unroll
            for (int q = 0; q < P; ++q) { v[j][q] = *reinterpret_cast<float const *>(p + off[q]); }
        }
#pragma unroll
        for (int j = 0; j < 6; ++j) {
#pragma unroll
            for (int q = 0; q < P; ++q) { acc += v[j][q]; }
        }
    }
    if (acc == 123.456f) { sink[0] = acc; }                 // (never true for the buffers it is run on; keeps the loads alive)
}

}  // namespace bbhip

using namespace bbhip;

// Runs `warmup` untimed and `reps` timed launches on `stream` and writes the mean launch-to-launch duration (HIP events around the
// timed launches, on that stream) to *mean_ms.  One wavefront per (row, window of segment_frames frames) reads loads_per_unit
// (rounded up to a multiple of 6) pseudo-randomly chosen rows' segments of that window from dev_x [row_count][frame_stride] and
// discards them: row_count * ceil(frame_size / segment_frames) * loads_per_unit * segment_frames * 4 bytes per launch.
// dev_sink: one float that is never written in practice.  Returns 0, or a HIP error code / -1 for a rejected argument.
extern "C" int bench_row_gather_probe(float const *dev_x, float *dev_sink, int row_count, int frame_size, int frame_stride, int loads_per_unit,
                                      int segment_frames, int warmup, int reps, float *mean_ms, void *stream)
{
    if (!(dev_x && dev_sink && mean_ms && row_count > 0 && frame_size > 0 && frame_stride >= frame_size && loads_per_unit > 0 && reps > 0 && warmup >= 0)) { return -1; }
    if (!(segment_frames == 64 || segment_frames == 128 || segment_frames == 256 || segment_frames == 512)) { return -1; }
    int const chunk_count = (frame_size + segment_frames - 1) / segment_frames, tile_count = (row_count + kWavesPerBlk - 1) / kWavesPerBlk;
    if ((long long)chunk_count * tile_count > 0x7fffffffLL) { return -1; }
    hipStream_t st = static_cast<hipStream_t>(stream);
    dim3 const grid((unsigned)(chunk_count * tile_count)), block(kBlock);
    TileDivisor const tiles = make_tile_divisor(tile_count);
    hipEvent_t e0, e1;
    hipError_t err;
    if ((err = hipEventCreate(&e0)) != hipSuccess) { return (int)err; }
    if ((err = hipEventCreate(&e1)) != hipSuccess) { (void)hipEventDestroy(e0); return (int)err; }
    for (int i = 0; i < warmup + reps; ++i) {
        if (i == warmup) { (void)hipEventRecord(e0, st); }
        switch (segment_frames / kWave) {
        case 1: hipLaunchKernelGGL(row_gather_probe_kernel<1>, grid, block, 0, st, dev_x, dev_sink, row_count, frame_stride, frame_size, chunk_count, tiles, loads_per_unit); break;
        case 2: hipLaunchKernelGGL(row_gather_probe_kernel<2>, grid, block, 0, st, dev_x, dev_sink, row_count, frame_stride, frame_size, chunk_count, tiles, loads_per_unit); break;
        case 4: hipLaunchKernelGGL(row_gather_probe_kernel<4>, grid, block, 0, st, dev_x, dev_sink, row_count, frame_stride, frame_size, chunk_count, tiles, loads_per_unit); break;
        default: hipLaunchKernelGGL(row_gather_probe_kernel<8>, grid, block, 0, st, dev_x, dev_sink, row_count, frame_stride, frame_size, chunk_count, tiles, loads_per_unit); break;
        }
    }
    (void)hipEventRecord(e1, st);
    err = hipGetLastError();
    if (err == hipSuccess) { err = hipEventSynchronize(e1); }
    float ms = 0.0f;
    if (err == hipSuccess) { err = hipEventElapsedTime(&ms, e0, e1); }
    (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
    *mean_ms = ms / (float)reps;
    return (int)err;
}

// Elementwise fp32 kernels: the vector operations behind the reference's Tensor arithmetic and the Adam step.
// All of them stream their operands once (HBM-bound); a thread handles four consecutive elements with 128-bit
// accesses where the pointers allow it.  Every arithmetic step is individually rounded (see rounded_mul), so results equal the reference's C++ expressions evaluated in fp32
// operation by operation (reference: include/bb/TensorOperator.h:41-238, include/bb/OptimizerAdam.h:168-178).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bbhip {

constexpr int kVecBlock = 256;

enum VecOp : int {
    kVecAddEx = 0,   // a*s0 + b*s1 + c
    kVecMulEx,       // a*s0*s1 + b
    kVecDivEx,       // (a*s0 + b) / (c*s1 + d)
    kVecSqrt,        // sqrt(s0)
    kVecExp,         // exp(s0)
    kVecMin,         // min(s0, s1)
    kVecMinV,        // min(s0, a)
    kVecMax,         // max(s0, s1)
    kVecMaxV,        // max(s0, a)
};

// A product that must be rounded on its own: the empty asm makes the value opaque, so the compiler cannot contract the
// multiplication with a following addition (this build contracts across statements and ignores the contract pragma).
__device__ __forceinline__ float rounded_mul(float x, float y)
{
    float t = x * y;
    asm("" : "+v"(t));
    return t;
}

template <int OP>
__device__ __forceinline__ float vec_apply(float s0, float s1, float a, float b, float c, float d)
{
    if (OP == kVecAddEx) { return (rounded_mul(a, s0) + rounded_mul(b, s1)) + c; }
    if (OP == kVecMulEx) { return rounded_mul(rounded_mul(a, s0), s1) + b; }
    if (OP == kVecDivEx) { return (rounded_mul(a, s0) + b) / (rounded_mul(c, s1) + d); }
    if (OP == kVecSqrt)  { return sqrtf(s0); }
    if (OP == kVecExp)   { return expf(s0); }
    // std::min(x, y) = (y < x) ? y : x,  std::max(x, y) = (x < y) ? y : x   (so a NaN in the second operand is dropped)
    if (OP == kVecMin)   { return (s1 < s0) ? s1 : s0; }
    if (OP == kVecMinV)  { return (a < s0) ? a : s0; }
    if (OP == kVecMax)   { return (s0 < s1) ? s1 : s0; }
    return (s0 < a) ? a : s0;
}

template <int OP>
constexpr bool vec_binary(void) { return OP == kVecAddEx || OP == kVecMulEx || OP == kVecDivEx || OP == kVecMin || OP == kVecMax; }

template <int OP>
__global__ __launch_bounds__(kVecBlock) void vector_op_kernel(float *__restrict__ dst, float const *src0, float const *src1,
                                                             float a, float b, float c, float d, size_t size, int aligned)
{
    size_t const i4 = ((size_t)blockIdx.x * kVecBlock + threadIdx.x) * 4;
    if (i4 >= size) { return; }
    if (aligned && i4 + 3 < size) {
        float4 const x = *reinterpret_cast<float4 const *>(src0 + i4);
        float4 y = x;
        if (vec_binary<OP>()) { y = *reinterpret_cast<float4 const *>(src1 + i4); }
        float4 r;
        r.x = vec_apply<OP>(x.x, y.x, a, b, c, d);
        r.y = vec_apply<OP>(x.y, y.y, a, b, c, d);
        r.z = vec_apply<OP>(x.z, y.z, a, b, c, d);
        r.w = vec_apply<OP>(x.w, y.w, a, b, c, d);
        *reinterpret_cast<float4 *>(dst + i4) = r;
    }
    else {
        for (size_t i = i4; i < size && i < i4 + 4; ++i) {
            float const x = src0[i];
            float const y = vec_binary<OP>() ? src1[i] : x;
            dst[i] = vec_apply<OP>(x, y, a, b, c, d);
        }
    }
}

// One Adam update of every tensor of a parameter list (reference: include/bb/OptimizerAdam.h:168-178, the host path;
// entry point cuda/OptimizerAdam.cu:12-84).  blockIdx.y = tensor, the blocks of a row stride over its elements.
//     m += (1-beta1)*(g - m);  v += (1-beta2)*(g*g - v);  p -= (lr_t*m) / (sqrt(v) + 1e-7)
__device__ __forceinline__ void adam_update(float &p, float g, float &m, float &v, float lr_t, float nb1, float nb2)
{
    m = m + rounded_mul(nb1, g - m);
    v = v + rounded_mul(nb2, rounded_mul(g, g) - v);
    p = p - rounded_mul(lr_t, m) / (sqrtf(v) + 1.0e-7f);
}

// ZERO: the gradients are set to zero once they have been used — the optimizer's Update() is Step() followed by ZeroGrad()
// (include/bb/Optimizer.h:31-35); done here, the zeroing costs four bytes per element instead of a launch per tensor.
template <bool ZERO>
__global__ __launch_bounds__(kVecBlock) void adam_kernel(int const *__restrict__ size_table, float *const *__restrict__ params_table,
                                                        float *const *__restrict__ grads_table, float *const *__restrict__ m_table,
                                                        float *const *__restrict__ v_table, float lr_t, float nb1, float nb2)
{
    int const t = blockIdx.y;
    int const size = size_table[t];
    float       *__restrict__ p = params_table[t];
    float       *__restrict__ g = grads_table[t];
    float       *__restrict__ m = m_table[t];
    float       *__restrict__ v = v_table[t];
    bool const aligned = ((reinterpret_cast<uintptr_t>(p) | reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(m) |
                           reinterpret_cast<uintptr_t>(v)) & 15) == 0;
    int const quads = aligned ? size / 4 : 0;          // elements handled four at a time with 128-bit accesses
    for (int q = blockIdx.x * kVecBlock + threadIdx.x; q < quads; q += gridDim.x * kVecBlock) {
        float4 pi = reinterpret_cast<float4 *>(p)[q];
        float4 const gi = reinterpret_cast<float4 const *>(g)[q];
        float4 mi = reinterpret_cast<float4 *>(m)[q];
        float4 vi = reinterpret_cast<float4 *>(v)[q];
        adam_update(pi.x, gi.x, mi.x, vi.x, lr_t, nb1, nb2);
        adam_update(pi.y, gi.y, mi.y, vi.y, lr_t, nb1, nb2);
        adam_update(pi.z, gi.z, mi.z, vi.z, lr_t, nb1, nb2);
        adam_update(pi.w, gi.w, mi.w, vi.w, lr_t, nb1, nb2);
        reinterpret_cast<float4 *>(p)[q] = pi;
        reinterpret_cast<float4 *>(m)[q] = mi;
        reinterpret_cast<float4 *>(v)[q] = vi;
        if (ZERO) { reinterpret_cast<float4 *>(g)[q] = make_float4(0.0f, 0.0f, 0.0f, 0.0f); }
    }
    for (int i = quads * 4 + blockIdx.x * kVecBlock + threadIdx.x; i < size; i += gridDim.x * kVecBlock) {
        float pi = p[i], mi = m[i], vi = v[i];
        adam_update(pi, g[i], mi, vi, lr_t, nb1, nb2);
        p[i] = pi; m[i] = mi; v[i] = vi;
        if (ZERO) { g[i] = 0.0f; }
    }
}

}  // namespace bbhip

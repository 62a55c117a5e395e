// Device-side arithmetic of the differentiable LUT, shared by every kernel of the library.
//
// The layer computes, per (output node, frame),
//     y = sum_{i < 2^N} W[i] * prod_{j < N} (bit_j(i) ? x_j : 1 - x_j)
// (reference: include/bb/StochasticOperation.h:95-114).  The sum is a multilinear polynomial in x_0..x_{N-1}.
// Instead of the 2^N products of the defining formula the kernels evaluate the same polynomial in the
// *centred monomial basis*
//     y = sum_{S subset of {0..N-1}} C[S] * prod_{j in S} z_j ,      z_j = x_j - 1/2 ,
// where C is obtained from W once per call by an N-stage butterfly (a, b) -> ((a + b) / 2, b - a)
// (table_prep_kernel in lut_kernels.hip).  The butterfly is an orthogonal transform up to powers of two, so no
// cancellation is introduced, and the evaluation needs one fused multiply-add per coefficient:
//     l[i] = monomials of the low  NL variables,   h[j] = monomials of the high NH variables (index = subset mask)
//     q[j] = sum_i C[j*L + i] * l[i]               (C is wave-uniform: scalar registers)
//     y    = sum_j h[j] * q[j]
// Backward, with d = dL/dy for this (node, frame):
//     g[j]        = d * h[j]
//     dC[j*L + i] += g[j] * l[i]                   (per-lane accumulators, reduced over frames afterwards)
//     p[i]        = sum_j C[j*L + i] * g[j]
//     dL/dx_k     = sum_{i : bit k of i set} l[i ^ (1<<k)] * p[i]                   for low  variables
//     dL/dx_k     = d * sum_{j : bit k' of j set} h[j ^ (1<<k')] * q[j]             for high variables (k' = k - NL)
// and dW = T^T dC is applied once per node after the frame reduction.  Results agree with the reference's
// association to a few ulp (fp32), well inside the 1e-5 / 1e-4 parity tolerances.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bbhip {

constexpr int kWave = 64;

template <int N>
struct LutDims {
    static constexpr int NL = N / 2;          // variables 0 .. NL-1 form the low group
    static constexpr int NH = N - NL;         // variables NL .. N-1 form the high group
    static constexpr int L  = 1 << NL;
    static constexpr int H  = 1 << NH;
    static constexpr int NN = 1 << N;
};

// how a kernel reads its inputs
enum XMode : int {
    kXClamp  = 0,   // fp32 frames, clamp to [0,1]                 (StochasticLutN.h:542)
    kXBinary = 1,   // fp32 frames, x > 0.5 ? 0.5+bias : 0.5-bias  (StochasticLutN.h:539)
    kXBit    = 2,   // bit-packed frames, same mapping
};

// how a kernel writes its output
enum YMode : int {
    kYClamp    = 0,   // fp32, clamp to [0,1]
    kYBinarize = 1,   // fp32, v > 0.5 ? 1 : 0
    kYBit      = 2,   // bit-packed, v > 0.5
};

// all monomials of K variables: m[mask] = prod_{k in mask} z[k], m[0] = 1
template <int K>
__device__ __forceinline__ void monomials(float const (&z)[K > 0 ? K : 1], float (&m)[1 << K])
{
    m[0] = 1.0f;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        m[1 << k] = z[k];
#pragma unroll
        for (int i = 1; i < (1 << k); ++i) {
            m[(1 << k) + i] = m[i] * z[k];
        }
    }
}

// centred input of one frame
template <int XMODE>
__device__ __forceinline__ float centre(float v, float bias)
{
    if (XMODE == kXClamp) {
        return __builtin_amdgcn_fmed3f(v, 0.0f, 1.0f) - 0.5f;
    }
    return (v > 0.5f) ? bias : -bias;
}

__device__ __forceinline__ float centre_bit(uint32_t word, int bit, float bias)
{
    return ((word >> bit) & 1u) ? bias : -bias;
}

template <int N>
struct LutEval {
    using D = LutDims<N>;

    // the node's coefficients, read once through a wave-uniform pointer before any store of the kernel so that
    // they are fetched with scalar loads and stay in scalar registers for the whole frame loop
    __device__ __forceinline__ static void load_table(float const *__restrict__ Cg, float (&C)[D::NN])
    {
#pragma unroll
        for (int i = 0; i < D::NN; ++i) { C[i] = Cg[i]; }
    }

    // Vector-register copies of the H constant terms C[j*L].  A fused multiply-add may read only one scalar
    // register, so "C[j*L] + l[1]*C[j*L+1]" needs one of the two coefficients in a vector register; copying them once
    // per unit (instead of once per frame step) takes H moves out of the frame loop.  The asm keeps the compiler from
    // re-materialising the copy inside the loop.
    __device__ __forceinline__ static void pin_constants(float const (&C)[D::NN], float (&cv)[D::H])
    {
#pragma unroll
        for (int j = 0; j < D::H; ++j) {
            asm("v_mov_b32 %0, %1" : "=v"(cv[j]) : "s"(C[j * D::L]));
        }
    }

    // q[j] = sum_i C[j*L+i] * l[i], cv[j] = C[j*L] held in a vector register
    __device__ __forceinline__ static void partial_q(float const (&C)[D::NN], float const (&cv)[D::H], float const (&l)[D::L], float (&q)[D::H])
    {
#pragma unroll
        for (int j = 0; j < D::H; ++j) {
            float a = cv[j];
#pragma unroll
            for (int i = 1; i < D::L; ++i) {
                a = __builtin_fmaf(l[i], C[j * D::L + i], a);
            }
            q[j] = a;
        }
    }

    __device__ __forceinline__ static float combine(float const (&h)[D::H], float const (&q)[D::H])
    {
        float y = q[0];
#pragma unroll
        for (int j = 1; j < D::H; ++j) {
            y = __builtin_fmaf(h[j], q[j], y);
        }
        return y;
    }

    // y for one frame from the centred inputs z[0..N-1]
    __device__ __forceinline__ static float forward(float const (&C)[D::NN], float const (&cv)[D::H], float const (&z)[N])
    {
        float zl[D::NL > 0 ? D::NL : 1], zh[D::NH];
#pragma unroll
        for (int k = 0; k < D::NL; ++k) { zl[k] = z[k]; }
#pragma unroll
        for (int k = 0; k < D::NH; ++k) { zh[k] = z[D::NL + k]; }
        float l[D::L], h[D::H], q[D::H];
        monomials<D::NL>(zl, l);
        monomials<D::NH>(zh, h);
        partial_q(C, cv, l, q);
        return combine(h, q);
    }

    // d(sum)/dz for the variables of one group: out[k] = sum_{i : bit k} m[i ^ (1<<k)] * v[i]
    template <int K>
    __device__ __forceinline__ static void group_grad(float const (&m)[1 << K], float const (&v)[1 << K], float (&out)[K > 0 ? K : 1])
    {
#pragma unroll
        for (int k = 0; k < K; ++k) {
            float a = 0.0f;
            bool first = true;
#pragma unroll
            for (int i = 0; i < (1 << K); ++i) {
                if ((i >> k) & 1) {
                    int const o = i ^ (1 << k);
                    if (first)       { a = (o == 0) ? v[i] : m[o] * v[i]; first = false; }
                    else             { a = __builtin_fmaf(m[o], v[i], a); }
                }
            }
            out[k] = a;
        }
    }
};

}  // namespace bbhip

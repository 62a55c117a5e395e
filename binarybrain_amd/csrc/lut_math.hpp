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
        float l[D::L], q[D::H];
        monomials<D::NL>(zl, l);
        partial_q(C, cv, l, q);
        return fold_high(zh, q);
    }

    // Horner's rule over the high variables: sum_j h[j] q[j] with h the monomials of zh, bit v of j belonging to zh[v];
    // H - 1 fused multiply-adds and no monomial products.  q is consumed.
    __device__ __forceinline__ static float fold_high(float const (&zh)[D::NH], float (&q)[D::H])
    {
#pragma unroll
        for (int v = 0; v < D::NH; ++v) {
#pragma unroll
            for (int s = 0; s < (D::H >> (v + 1)); ++s) { q[s] = __builtin_fmaf(zh[v], q[2 * s + 1], q[2 * s]); }
        }
        return q[0];
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

// ------------------------------------------------------------------------------------------------
//  The partial sums q[j] = sum_i C[j*L + i] * l[i] on the matrix unit.
//
//  v_mfma_f32_4x4x1_16b_f32 performs, for each of the 16 lane quads b of a wavefront, the rank-1 update
//      D_b[r][c] += A_b[r] * B_b[c],      A_b[r] = srcA of lane 4b + r,   B_b[c] = srcB of lane 4b + c,
//  and returns D_b[r][c] in result register r of lane 4b + c.  With srcB = l[i] of the lane's own frame and
//  srcA = C[(4g + r)*L + i] (the same for every quad), L such updates (l[0] = 1) leave q[4g + r] of the lane's own
//  frame in result register r: 4 coefficients per lane and instruction instead of 1, with the frames staying one per
//  lane and no data movement between lanes.  The instruction's broadcast control (cbsz = 4, abid = s) makes all 16
//  quads take their A values from quad s of the source register, so the coefficients of 16 updates sit in one register.
// ------------------------------------------------------------------------------------------------
typedef float mfma_f4 __attribute__((ext_vector_type(4)));

// One update with the A operand broadcast from lane quad SLOT to all 16 quads (cbsz = 4, abid = SLOT):
//     D[r] (own lane) += A(lane 4 SLOT + r) * B(own lane)
// A single vector register then carries 16 updates' worth of coefficients: a whole 64-entry table.
template <int SLOT>
__device__ __forceinline__ mfma_f4 mfma_broadcast(float a, float b, mfma_f4 d)
{
    static_assert(SLOT >= 0 && SLOT < 16, "a register holds 16 quads");
    return __builtin_amdgcn_mfma_f32_4x4x1f32(a, b, d, 4, SLOT, 0);
}

// sum over i < COUNT of A(quad BASE + i) * b[i], four results per lane (the quad index must be a compile-time constant)
template <int BASE, int COUNT, int I = 0>
__device__ __forceinline__ mfma_f4 mfma_broadcast_chain(float a, float const (&b)[COUNT], mfma_f4 d)
{
    d = mfma_broadcast<BASE + I>(a, b[I], d);
    if constexpr (I + 1 < COUNT) { return mfma_broadcast_chain<BASE, COUNT, I + 1>(a, b, d); }
    else                         { return d; }
}

// out[4 g + v] = sum_i A(quad g * COUNT + i)[v] * b[i] for g < GROUPS
template <int GROUPS, int COUNT, int G = 0>
__device__ __forceinline__ void mfma_broadcast_matvec(float a, float const (&b)[COUNT], float (&out)[GROUPS * 4])
{
    mfma_f4 const d = mfma_broadcast_chain<G * COUNT, COUNT>(a, b, mfma_f4{0.0f, 0.0f, 0.0f, 0.0f});
#pragma unroll
    for (int v = 0; v < 4; ++v) { out[4 * G + v] = d[v]; }
    if constexpr (G + 1 < GROUPS) { mfma_broadcast_matvec<GROUPS, COUNT, G + 1>(a, b, out); }
}

// The node's whole table in ONE vector register: lane 4 s + r holds C[(4 g + r) * L + i] for update s = g * L + i, and each
// update takes its A operand from quad s of that register (the loads of a wavefront cover the table's 2^N consecutive
// floats once, in permuted order).
template <int N>
struct LutMatrixQ {
    using D = LutDims<N>;
    static constexpr bool kUsable = (D::H % 4 == 0) && (D::L >= 4) && ((D::H / 4) * D::L <= 16);
    static constexpr int  G = (D::H >= 4) ? D::H / 4 : 1;     // groups of 4 partial sums

    float t;

    __device__ __forceinline__ static int table_index(int lane)
    {
        int const s = lane >> 2, r = lane & 3;
        int const g = s / D::L, i = s % D::L;
        int const e = (4 * g + r) * D::L + i;
        return e < D::NN ? e : D::NN - 1;                      // (lanes beyond the updates of a narrow table: any entry)
    }

    __device__ __forceinline__ void load(float const *__restrict__ Cg, int lane) { t = Cg[table_index(lane)]; }
    // the same from a table held one entry per lane (lane e: entry e)
    __device__ __forceinline__ void take(float entry_of_lane, int lane)
    {
        t = __int_as_float(__builtin_amdgcn_ds_bpermute(table_index(lane) << 2, __float_as_int(entry_of_lane)));
    }

    __device__ __forceinline__ void partial_q(float const (&l)[D::L], float (&q)[D::H]) const
    {
        mfma_broadcast_matvec<G, D::L>(t, l, q);
    }

    // y for one frame from the centred inputs z[0..N-1]
    __device__ __forceinline__ float forward(float const (&z)[N]) const
    {
        float zl[D::NL > 0 ? D::NL : 1], zh[D::NH];
#pragma unroll
        for (int k = 0; k < D::NL; ++k) { zl[k] = z[k]; }
#pragma unroll
        for (int k = 0; k < D::NH; ++k) { zh[k] = z[D::NL + k]; }
        float l[D::L], q[D::H];
        monomials<D::NL>(zl, l);
        partial_q(l, q);
        return LutEval<N>::fold_high(zh, q);
    }
};

}  // namespace bbhip

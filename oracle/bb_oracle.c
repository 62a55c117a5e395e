/*
 * TEST INFRASTRUCTURE — CPU oracle for the differentiable-LUT hot path.
 *
 * This file is a plain-C restatement of BinaryBrain's *CPU* implementation of
 * StochasticLutN / DifferentiableLutN / BinaryLutN<6> and of the connection
 * reverse table.  It exists so that parity tests, the smoke check and the
 * cpu_baseline leg of the benchmark have a fixed side to compare the HIP
 * library against on machines where the reference tree is absent.  Nothing in
 * the shipped library may call it.
 *
 * Build: gcc -O2 -mavx2 -mfma -fopenmp -ffp-contract=off (see oracle/Makefile).
 * -ffp-contract=off keeps every multiply/add a separate IEEE operation; fused
 * multiply-adds appear only where the reference uses _mm256_fmadd_ps and are
 * written as fmaf().
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   - *_StochasticLut_Forward/Backward, simd order : bit-exact against the real
 *     reference headers (oracle/_ref) where that library is built, against the
 *     committed vectors in tests/golden/ elsewhere, plus closed forms
 *     (x in {0,1}^N picks W[index]; constant W; sum_i dW[i] = sum_f dy;
 *     multilinear finite differences for dx) and an fp64 brute force.
 *   - generic order, DifferentiableLutN *: same vectors with a few-ulp
 *     tolerance (the reference's generic loops are subject to the compiler's
 *     contraction choices), textbook mean/variance, BN gradient invariants.
 *   - BinaryLut6, reverse table: bit-exact against oracle/_ref and golden
 *     vectors; BinaryLut6 also against StochasticLut with W,x in {0,1}.
 *   - MaxLut *: bit-exact against the reference's class (oracle/_ref), vectors
 *     written from it (tests/golden/maxlut.npz), the known answers of
 *     tests/gtest/MaxLutTest.cpp and numpy max / argmax.
 *   - Reduce *, LossMeanSquaredError, MetricsMeanSquaredError: bit-exact (double
 *     accumulators included) against the reference's classes and vectors
 *     written from them (tests/golden/reduce_mse.npz); numpy means in fp64.
 *   - StochasticBatchNormalization *: the reference's class (oracle/_ref) and
 *     vectors written from it (tests/golden/bn.npz) to 1e-6 of the terms that
 *     cancel (contraction, as above; the batch mean bit-exact), fp64 textbook
 *     statistics, the gradient's two vanishing sums and a finite difference.
 *   - RealToBinary, BinaryToReal, Binarize, HardTanh: bit-exact against the
 *     reference's classes (oracle/_ref), vectors written from them
 *     (tests/golden/modulation.npz), the known answers of
 *     tests/gtest/RealToBinaryTest.cpp, BinaryToRealTest.cpp, BinarizeTest.cpp,
 *     and numpy restatements.
 *   - MaxPooling *, UpSampling *: bit-exact against the reference's classes
 *     (oracle/_ref), vectors written from them (tests/golden/pooling.npz), the
 *     known answers of tests/gtest/MaxPoolingTest.cpp and UpSamplingTest.cpp, numpy.
 *   - Shuffle *: bit-exact against the reference's class (oracle/_ref), the known
 *     answer of tests/gtest/ShuffleTest.cpp, numpy's transpose of the rows seen as
 *     a [unit][group] matrix, and backward(forward(x)) == x.
 *
 * Array conventions (the reference's FrameBuffer layout, include/bb/FrameBuffer.h:28-46,
 * 927-939): node-major, frame-minor; element (node n, frame f) of an fp32
 * buffer is p[n*stride + f]; of a bit buffer, bit (f & 31) of the 32-bit word
 * p[n*stride_words + (f >> 5)] (include/bb/DataType.h:612-647).
 */

#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define MAXN   6
#define MAXNN  64

static inline float clamp01(float v) { return fminf(1.0f, fmaxf(0.0f, v)); }

/* include/bb/StochasticOperation.h:95-114 */
static inline float lut_forward_generic(float const *x, float const *W, int N)
{
    float acc = 0.0f;
    for (int i = 0; i < (1 << N); ++i) {
        float w = W[i];
        for (int j = 0; j < N; ++j) {
            w *= ((i >> j) & 1) ? x[j] : (1.0f - x[j]);
        }
        acc += w;
    }
    return acc;
}

/* include/bb/StochasticOperation.h:118-152 */
static inline void lut_backward_generic(float const *x, float *dx, float dy, float const *W, float *dW, int N)
{
    for (int i = 0; i < (1 << N); ++i) {
        float dw = dy;
        for (int j = 0; j < N; ++j) {
            dw *= ((i >> j) & 1) ? x[j] : (1.0f - x[j]);
        }
        dW[i] += dw;
    }
    for (int i = 0; i < N; ++i) {
        dx[i] = 0;
        for (int j = 0; j < (1 << N); ++j) {
            float w = ((j >> i) & 1) ? +W[j] : -W[j];
            for (int k = 0; k < N; ++k) {
                if (i != k) {
                    w *= ((j >> k) & 1) ? x[k] : (1.0f - x[k]);
                }
            }
            dx[i] += w;
        }
        dx[i] *= dy;
    }
}

/* One frame of simd_fp32_StochasticLut6_Forward (include/bb/StochasticLutSimd.h:77-154):
 * pair products xk_ab = x[2k+1]? * x[2k]?, then y = W0*(x2*(x1*x0)) followed by 63 fmadd in index order. */
static inline float lut6_forward_simd_order(float const xp[6], float const W[64])
{
    float xn[6], pr[3][4];
    for (int i = 0; i < 6; ++i) { xn[i] = 1.0f - xp[i]; }
    for (int k = 0; k < 3; ++k) {
        pr[k][0] = xn[2 * k + 1] * xn[2 * k];
        pr[k][1] = xn[2 * k + 1] * xp[2 * k];
        pr[k][2] = xp[2 * k + 1] * xn[2 * k];
        pr[k][3] = xp[2 * k + 1] * xp[2 * k];
    }
    float y = 0.0f;
    for (int i = 0; i < 64; ++i) {
        float p = pr[2][(i >> 4) & 3] * (pr[1][(i >> 2) & 3] * pr[0][i & 3]);
        y = (i == 0) ? (W[0] * p) : fmaf(W[i], p, y);
    }
    return y;
}

/* One frame of simd_fp32_StochasticLut6_Backward (StochasticLutSimd.h:240-433). dWacc is the per-lane accumulator. */
static inline void lut6_backward_simd_order(float const xp[6], float grad, float const W[64], float dWacc[64], float dx[6])
{
    float xn[6], pr[3][4], d[3][4];
    for (int i = 0; i < 6; ++i) { xn[i] = 1.0f - xp[i]; }
    for (int k = 0; k < 3; ++k) {
        pr[k][0] = xn[2 * k + 1] * xn[2 * k];
        pr[k][1] = xn[2 * k + 1] * xp[2 * k];
        pr[k][2] = xp[2 * k + 1] * xn[2 * k];
        pr[k][3] = xp[2 * k + 1] * xp[2 * k];
        d[k][0] = d[k][1] = d[k][2] = d[k][3] = 0.0f;
    }
    for (int i = 0; i < 64; ++i) {
        float p = pr[2][(i >> 4) & 3] * (pr[1][(i >> 2) & 3] * pr[0][i & 3]);
        dWacc[i] = fmaf(grad, p, dWacc[i]);
    }
    for (int i = 0; i < 64; ++i) {
        int a = i & 3, b = (i >> 2) & 3, c = (i >> 4) & 3;
        float dxi = W[i] * grad;
        d[0][a] = fmaf(dxi, pr[2][c] * pr[1][b], d[0][a]);
        d[1][b] = fmaf(dxi, pr[2][c] * pr[0][a], d[1][b]);
        d[2][c] = fmaf(dxi, pr[1][b] * pr[0][a], d[2][c]);
    }
    for (int k = 0; k < 3; ++k) {
        /* even input of the pair (StochasticLutSimd.h:399-403, 411-415, 423-427) */
        float dxn = d[k][0] * xn[2 * k + 1];
        dxn = fmaf(d[k][2], xp[2 * k + 1], dxn);
        float dxp = d[k][1] * xn[2 * k + 1];
        dxp = fmaf(d[k][3], xp[2 * k + 1], dxp);
        dx[2 * k] = dxp - dxn;
        /* odd input of the pair (:405-409, 417-421, 429-433) */
        dxn = d[k][0] * xn[2 * k];
        dxn = fmaf(d[k][1], xp[2 * k], dxn);
        dxp = d[k][2] * xn[2 * k];
        dxp = fmaf(d[k][3], xp[2 * k], dxp);
        dx[2 * k + 1] = dxp - dxn;
    }
}

/* bb_mm256_hsum_ps (include/bb/SimdSupport.h:93-100): ((a0+a1)+(a2+a3)) + ((a4+a5)+(a6+a7)) */
static inline float hsum8(float const a[8])
{
    return ((a[0] + a[1]) + (a[2] + a[3])) + ((a[4] + a[5]) + (a[6] + a[7]));
}

static inline float read_x_fp32(float const *row, int f, int input_binary, float bias)
{
    float v = row[f];
    if (input_binary) { return 0.5f + ((v > 0.5f) ? +bias : -bias); }
    return clamp01(v);
}

static inline int read_bit(int32_t const *row, int f)
{
    return (int)(((uint32_t)row[f >> 5] >> (f & 31)) & 1u);
}

static inline float read_x_bit(int32_t const *row, int f, float bias)
{
    float v = read_bit(row, f) ? 1.0f : 0.0f;
    return 0.5f + ((v > 0.5f) ? +bias : -bias);
}

static inline void write_bit(int32_t *row, int f, int v)
{
    uint32_t m = 1u << (f & 31);
    uint32_t w = (uint32_t)row[f >> 5];
    row[f >> 5] = (int32_t)(v ? (w | m) : (w & ~m));
}

static void load_W(float *Wl, float const *W, int node, int NN, int lut_binarize)
{
    for (int i = 0; i < NN; ++i) {
        float w = W[(size_t)node * NN + i];
        if (lut_binarize) { w = (w > 0.5f) ? 1.0f : 0.0f; }
        Wl[i] = w;
    }
}


/* Tensor::Clamp_inplace as used on W (include/bb/StochasticLutN.h:451) */
void oracle_fp32_Vector_clamp(float *dst, float const *src, float lo, float hi, int size)
{
    for (int i = 0; i < size; ++i) { dst[i] = fminf(hi, fmaxf(lo, src[i])); }
}


/* StochasticLutN<N,float>::Forward, host path (include/bb/StochasticLutN.h:504-559).
 * simd != 0 and n == 6 selects the AVX2 association (StochasticLutSimd.h:25-163). W is used as given. */
void oracle_fp32_StochasticLut_Forward(int n, float const *x, float *y, int32_t const *idx, float const *W,
                                       int node_size, int frame_size, int frame_stride,
                                       int input_binary, int lut_binarize, float bias, int simd)
{
    int const NN = 1 << n;
    #pragma omp parallel for
    for (int node = 0; node < node_size; ++node) {
        float Wl[MAXNN];
        load_W(Wl, W, node, NN, lut_binarize);
        for (int f = 0; f < frame_size; ++f) {
            float xv[MAXN];
            for (int i = 0; i < n; ++i) {
                xv[i] = read_x_fp32(x + (size_t)idx[node * n + i] * frame_stride, f, input_binary, bias);
            }
            float v = (simd && n == 6) ? lut6_forward_simd_order(xv, Wl) : lut_forward_generic(xv, Wl, n);
            if (simd && n == 6) { v = fminf(fmaxf(v, 0.0f), 1.0f); }       /* StochasticLutSimd.h:157-158 */
            else                { v = fmaxf(0.0f, v); v = fminf(1.0f, v); } /* StochasticLutN.h:551-552 */
            y[(size_t)node * frame_stride + f] = v;
        }
    }
}

/* StochasticLutN<N,Bit>::Forward generic path: x bit-packed, y fp32 (StochasticLutN.h:512-559) */
void oracle_bit_fp32_StochasticLut_Forward(int n, int32_t const *x, float *y, int32_t const *idx, float const *W,
                                           int node_size, int frame_size, int frame_stride, int bin_frame_stride,
                                           int lut_binarize, float bias)
{
    int const NN = 1 << n;
    #pragma omp parallel for
    for (int node = 0; node < node_size; ++node) {
        float Wl[MAXNN];
        load_W(Wl, W, node, NN, lut_binarize);
        for (int f = 0; f < frame_size; ++f) {
            float xv[MAXN];
            for (int i = 0; i < n; ++i) {
                xv[i] = read_x_bit(x + (size_t)idx[node * n + i] * bin_frame_stride, f, bias);
            }
            float v = lut_forward_generic(xv, Wl, n);
            v = fmaxf(0.0f, v); v = fminf(1.0f, v);
            y[(size_t)node * frame_stride + f] = v;
        }
    }
}

/* DifferentiableLutN<N,Bit> forward without batch-norm: bit in, bit out, y = (LUT > 0.5)
 * (include/bb/DifferentiableLutN.h:959-1008 with BinType = Bit). Bits of frames >= frame_size are left untouched. */
void oracle_bit_bit_fp32_StochasticLut_Forward(int n, int32_t const *x, int32_t *y, int32_t const *idx, float const *W,
                                               int node_size, int frame_size, int frame_stride,
                                               int lut_binarize, float bias)
{
    int const NN = 1 << n;
    #pragma omp parallel for
    for (int node = 0; node < node_size; ++node) {
        float Wl[MAXNN];
        load_W(Wl, W, node, NN, lut_binarize);
        for (int f = 0; f < frame_size; ++f) {
            float xv[MAXN];
            for (int i = 0; i < n; ++i) {
                xv[i] = read_x_bit(x + (size_t)idx[node * n + i] * frame_stride, f, bias);
            }
            float v = lut_forward_generic(xv, Wl, n);
            write_bit(y + (size_t)node * frame_stride, f, v > 0.5f);
        }
    }
}


static void backward_core(int n, float const *x_fp32, int32_t const *x_bit, float const *dy, float *dx,
                          int32_t const *idx, float const *W, float *dW,
                          int input_node_size, int output_node_size, int frame_size,
                          int frame_stride, int bin_frame_stride,
                          int input_binary, int lut_binarize, float bias, int simd)
{
    int const NN = 1 << n;
    size_t const tmp_rows = (size_t)output_node_size * n;
    float *tmp = (float *)malloc(sizeof(float) * tmp_rows * (size_t)frame_size);

    #pragma omp parallel for
    for (int node = 0; node < output_node_size; ++node) {
        float Wl[MAXNN];
        load_W(Wl, W, node, NN, lut_binarize);
        if (simd && n == 6 && !x_bit) {
            /* StochasticLutSimd.h:195-440: 8 independent lanes over frames, horizontal sum at the end */
            float acc[8][64];
            memset(acc, 0, sizeof(acc));
            for (int f = 0; f < frame_size; ++f) {
                float xv[6], dxv[6];
                for (int i = 0; i < 6; ++i) {
                    xv[i] = read_x_fp32(x_fp32 + (size_t)idx[node * 6 + i] * frame_stride, f, input_binary, bias);
                }
                lut6_backward_simd_order(xv, dy[(size_t)node * frame_stride + f], Wl, acc[f & 7], dxv);
                for (int i = 0; i < 6; ++i) { tmp[((size_t)node * 6 + i) * frame_size + f] = dxv[i]; }
            }
            for (int i = 0; i < 64; ++i) {
                float lanes[8];
                for (int l = 0; l < 8; ++l) { lanes[l] = acc[l][i]; }
                dW[(size_t)node * 64 + i] += hsum8(lanes);
            }
        }
        else {
            /* StochasticLutN.h:692-736 */
            float dWl[MAXNN];
            memset(dWl, 0, sizeof(dWl));
            for (int f = 0; f < frame_size; ++f) {
                float xv[MAXN], dxv[MAXN];
                for (int i = 0; i < n; ++i) {
                    int in = idx[node * n + i];
                    xv[i] = x_bit ? read_x_bit(x_bit + (size_t)in * bin_frame_stride, f, bias)
                                  : read_x_fp32(x_fp32 + (size_t)in * frame_stride, f, input_binary, bias);
                }
                lut_backward_generic(xv, dxv, dy[(size_t)node * frame_stride + f], Wl, dWl, n);
                for (int i = 0; i < n; ++i) { tmp[((size_t)node * n + i) * frame_size + f] = dxv[i]; }
            }
            for (int i = 0; i < NN; ++i) { dW[(size_t)node * NN + i] += dWl[i]; }
        }
    }

    /* integrate: zero-filled dx, contributions added in ascending (node, input) order
     * (StochasticLutSimd.h:179, 442-454; StochasticLutN.h:680, 738-749) */
    for (int in = 0; in < input_node_size; ++in) {
        memset(dx + (size_t)in * frame_stride, 0, sizeof(float) * (size_t)frame_size);
    }
    #pragma omp parallel for
    for (int f = 0; f < frame_size; ++f) {
        for (int node = 0; node < output_node_size; ++node) {
            for (int i = 0; i < n; ++i) {
                dx[(size_t)idx[node * n + i] * frame_stride + f] += tmp[((size_t)node * n + i) * frame_size + f];
            }
        }
    }
    free(tmp);
}

/* StochasticLutN<N,float>::Backward host path (StochasticLutN.h:668-752). dW accumulates; dx is overwritten. */
void oracle_fp32_StochasticLut_Backward(int n, float const *x, float const *dy, float *dx, int32_t const *idx,
                                        float const *W, float *dW,
                                        int input_node_size, int output_node_size, int frame_size, int frame_stride,
                                        int input_binary, int lut_binarize, float bias, int simd)
{
    backward_core(n, x, NULL, dy, dx, idx, W, dW, input_node_size, output_node_size, frame_size,
                  frame_stride, 0, input_binary, lut_binarize, bias, simd);
}

/* StochasticLutN<N,Bit>::Backward generic path */
void oracle_bit_fp32_StochasticLut_Backward(int n, int32_t const *x, float const *dy, float *dx, int32_t const *idx,
                                            float const *W, float *dW,
                                            int input_node_size, int output_node_size, int frame_size,
                                            int frame_stride, int bin_frame_stride, int lut_binarize, float bias)
{
    backward_core(n, NULL, x, dy, dx, idx, W, dW, input_node_size, output_node_size, frame_size,
                  frame_stride, bin_frame_stride, 1, lut_binarize, bias, 0);
}


/* ---- DifferentiableLutN ------------------------------------------------------------------ */

static inline float dl_read_x(float const *x_fp32, int32_t const *x_bit, int in, int f,
                              int frame_stride, int bin_frame_stride, int binary_mode, float bias)
{
    float v = x_bit ? (read_bit(x_bit + (size_t)in * bin_frame_stride, f) ? 1.0f : 0.0f)
                    : x_fp32[(size_t)in * frame_stride + f];
    if (binary_mode) { return 0.5f + ((v > 0.5f) ? +bias : -bias); }
    return clamp01(v);
}

static inline float dl_activate(float v, int binary_mode)
{
    if (binary_mode) { return (v > 0.5f) ? 1.0f : 0.0f; }
    v = fminf(v, 1.0f);
    v = fmaxf(v, 0.0f);
    return v;
}

static void dl_forward_core(int n, float const *x_fp32, int32_t const *x_bit, float *y_fp32, int32_t *y_bit,
                            int32_t const *idx, float const *W,
                            float *mean_out, float *rstd_out, float *running_mean, float *running_var,
                            float gamma, float beta, float momentum, float bias,
                            int node_size, int frame_size, int frame_stride, int bin_frame_stride,
                            int lut_binarize, int binary_mode, int train)
{
    int const NN = 1 << n;
    float const reciprocal_frame_size = 1.0f / (float)frame_size;

    #pragma omp parallel for
    for (int node = 0; node < node_size; ++node) {
        float Wl[MAXNN];
        load_W(Wl, W, node, NN, lut_binarize);
        float mean, rstd;
        if (train) {
            /* include/bb/DifferentiableLutN.h:775-812: Kahan-compensated sums in frame order */
            float s1 = 0, c1 = 0, y1, t1;
            float s2 = 0, c2 = 0, y2, t2;
            for (int f = 0; f < frame_size; ++f) {
                float xv[MAXN];
                for (int i = 0; i < n; ++i) {
                    xv[i] = dl_read_x(x_fp32, x_bit, idx[node * n + i], f, frame_stride, bin_frame_stride, binary_mode, bias);
                }
                float v = lut_forward_generic(xv, Wl, n);
                y1 = v - c1;       t1 = s1 + y1; c1 = (t1 - s1) - y1; s1 = t1;
                y2 = (v * v) - c2; t2 = s2 + y2; c2 = (t2 - s2) - y2; s2 = t2;
            }
            mean = s1 * reciprocal_frame_size;
            float var = fmaxf(1.0e-5f, (s2 * reciprocal_frame_size) - (mean * mean));
            rstd = 1.0f / sqrtf(var);
            running_mean[node] = running_mean[node] * momentum + mean * (1.0f - momentum);
            running_var[node]  = running_var[node]  * momentum + var  * (1.0f - momentum);
            mean_out[node] = mean;
            rstd_out[node] = rstd;
        }
        else {
            /* :866-868 */
            mean = running_mean[node];
            rstd = 1.0f / sqrtf(running_var[node]);
        }
        for (int f = 0; f < frame_size; ++f) {
            float xv[MAXN];
            for (int i = 0; i < n; ++i) {
                xv[i] = dl_read_x(x_fp32, x_bit, idx[node * n + i], f, frame_stride, bin_frame_stride, binary_mode, bias);
            }
            float v = lut_forward_generic(xv, Wl, n);
            v = (v - mean) * rstd;
            v = v * gamma + beta;
            v = dl_activate(v, binary_mode);
            if (y_bit) { write_bit(y_bit + (size_t)node * bin_frame_stride, f, v != 0.0f); }
            else       { y_fp32[(size_t)node * frame_stride + f] = v; }
        }
    }
}

/* DifferentiableLutN<N,float>::Forward(train=true), batch_norm on (DifferentiableLutN.h:754-847) */
void oracle_fp32_DifferentiableLutN_ForwardTraining(int n, float const *x, float *y, int32_t const *idx, float const *W,
        float *mean, float *rstd, float *running_mean, float *running_var,
        float gamma, float beta, float momentum, float bias,
        int node_size, int frame_size, int frame_stride, int lut_binarize, int binary_mode)
{
    dl_forward_core(n, x, NULL, y, NULL, idx, W, mean, rstd, running_mean, running_var, gamma, beta, momentum, bias,
                    node_size, frame_size, frame_stride, 0, lut_binarize, binary_mode, 1);
}

/* DifferentiableLutN<N,Bit>::Forward(train=true): bit in, bit out; binary_mode is forced on for Bit (:116-118) */
void oracle_bit_fp32_DifferentiableLutN_ForwardTraining(int n, int32_t const *x, int32_t *y, int32_t const *idx, float const *W,
        float *mean, float *rstd, float *running_mean, float *running_var,
        float gamma, float beta, float momentum, float bias,
        int node_size, int frame_size, int frame_stride, int lut_binarize)
{
    dl_forward_core(n, NULL, x, NULL, y, idx, W, mean, rstd, running_mean, running_var, gamma, beta, momentum, bias,
                    node_size, frame_size, 0, frame_stride, lut_binarize, 1, 1);
}

/* DifferentiableLutN::Forward(train=false), batch_norm on (:848-902) */
void oracle_fp32_DifferentiableLutN_ForwardInference(int n, float const *x, float *y, int32_t const *idx, float const *W,
        float const *running_mean, float const *running_var,
        float gamma, float beta, float bias,
        int node_size, int frame_size, int frame_stride, int lut_binarize, int binary_mode)
{
    dl_forward_core(n, x, NULL, y, NULL, idx, W, NULL, NULL, (float *)running_mean, (float *)running_var, gamma, beta, 0.0f, bias,
                    node_size, frame_size, frame_stride, 0, lut_binarize, binary_mode, 0);
}

void oracle_bit_fp32_DifferentiableLutN_ForwardInference(int n, int32_t const *x, int32_t *y, int32_t const *idx, float const *W,
        float const *running_mean, float const *running_var,
        float gamma, float beta, float bias,
        int node_size, int frame_size, int frame_stride, int lut_binarize)
{
    dl_forward_core(n, NULL, x, NULL, y, idx, W, NULL, NULL, (float *)running_mean, (float *)running_var, gamma, beta, 0.0f, bias,
                    node_size, frame_size, 0, frame_stride, lut_binarize, 1, 0);
}

/* DifferentiableLutN<N,float> forward without batch-norm (:959-1008): out = binary ? (y > 0.5) : clip(y, 0, 1) */
void oracle_fp32_DifferentiableLutN_ForwardNoBn(int n, float const *x, float *y, int32_t const *idx, float const *W,
        float bias, int node_size, int frame_size, int frame_stride, int lut_binarize, int binary_mode)
{
    int const NN = 1 << n;
    #pragma omp parallel for
    for (int node = 0; node < node_size; ++node) {
        float Wl[MAXNN];
        load_W(Wl, W, node, NN, lut_binarize);
        for (int f = 0; f < frame_size; ++f) {
            float xv[MAXN];
            for (int i = 0; i < n; ++i) {
                xv[i] = dl_read_x(x, NULL, idx[node * n + i], f, frame_stride, 0, binary_mode, bias);
            }
            y[(size_t)node * frame_stride + f] = dl_activate(lut_forward_generic(xv, Wl, n), binary_mode);
        }
    }
}

static void dl_backward_core(int n, float const *x_fp32, int32_t const *x_bit, float const *dy, float *dx,
                             int32_t const *idx, float const *W, float *dW,
                             float const *mean_in, float const *rstd_in,
                             float gamma, float beta, float bias,
                             int input_node_size, int output_node_size, int frame_size,
                             int frame_stride, int bin_frame_stride, int lut_binarize, int binary_mode)
{
    /* include/bb/DifferentiableLutN.h:1157-1266: single-threaded in the reference; kept sequential here so the
     * dx accumulation order (node, frame, input) is the reference's. */
    int const NN = 1 << n;
    float const reciprocal_frame_size = 1.0f / (float)frame_size;

    for (int in = 0; in < input_node_size; ++in) {
        memset(dx + (size_t)in * frame_stride, 0, sizeof(float) * (size_t)frame_size);
    }
    for (int node = 0; node < output_node_size; ++node) {
        float Wl[MAXNN], dWl[MAXNN];
        load_W(Wl, W, node, NN, lut_binarize);
        memset(dWl, 0, sizeof(dWl));

        float mean = mean_in[node];
        float rstd = rstd_in[node];
        float rstd2 = rstd * rstd;
        float dmeanx = 0;
        float dstd = 0;
        for (int f = 0; f < frame_size; ++f) {
            float xv[MAXN];
            for (int i = 0; i < n; ++i) {
                xv[i] = dl_read_x(x_fp32, x_bit, idx[node * n + i], f, frame_stride, bin_frame_stride, binary_mode, bias);
            }
            float v = lut_forward_generic(xv, Wl, n);
            float tanh_x = ((v - mean) * rstd) * gamma + beta;
            float g = dy[(size_t)node * frame_stride + f];
            if (tanh_x <= 0.0f) { g = 0.0f; }
            if (tanh_x >= 1.0f) { g = 0.0f; }
            float xc = v - mean;
            float dxn = gamma * g;
            dstd   += -(dxn * xc * rstd2);
            dmeanx += -(dxn * rstd);
        }
        float dvar  = dstd * rstd;
        float dmean = (dmeanx - (mean * dvar)) * reciprocal_frame_size;

        for (int f = 0; f < frame_size; ++f) {
            float xv[MAXN], dxv[MAXN];
            for (int i = 0; i < n; ++i) {
                xv[i] = dl_read_x(x_fp32, x_bit, idx[node * n + i], f, frame_stride, bin_frame_stride, binary_mode, bias);
            }
            float v = lut_forward_generic(xv, Wl, n);
            float tanh_x = ((v - mean) * rstd) * gamma + beta;
            float g = dy[(size_t)node * frame_stride + f];
            if (tanh_x <= 0.0f) { g = 0.0f; }
            if (tanh_x >= 1.0f) { g = 0.0f; }
            float dxn = g * gamma;
            float dxc = dxn * rstd;
            float d   = dxc + dmean + (v * dvar * reciprocal_frame_size);
            lut_backward_generic(xv, dxv, d, Wl, dWl, n);
            for (int i = 0; i < n; ++i) {
                dx[(size_t)idx[node * n + i] * frame_stride + f] += dxv[i];
            }
        }
        for (int i = 0; i < NN; ++i) { dW[(size_t)node * NN + i] += dWl[i]; }
    }
}

/* DifferentiableLutN<N,float>::Backward with batch-norm (:1157-1266); mean/rstd are the values Forward(train) stored */
void oracle_fp32_DifferentiableLutN_Backward(int n, float const *x, float const *dy, float *dx, int32_t const *idx,
        float const *W, float *dW, float const *mean, float const *rstd,
        float gamma, float beta, float bias,
        int input_node_size, int output_node_size, int frame_size, int frame_stride,
        int lut_binarize, int binary_mode)
{
    dl_backward_core(n, x, NULL, dy, dx, idx, W, dW, mean, rstd, gamma, beta, bias,
                     input_node_size, output_node_size, frame_size, frame_stride, 0, lut_binarize, binary_mode);
}

void oracle_bit_fp32_DifferentiableLutN_Backward(int n, int32_t const *x, float const *dy, float *dx, int32_t const *idx,
        float const *W, float *dW, float const *mean, float const *rstd,
        float gamma, float beta, float bias,
        int input_node_size, int output_node_size, int frame_size, int frame_stride, int x_frame_stride,
        int lut_binarize)
{
    dl_backward_core(n, NULL, x, dy, dx, idx, W, dW, mean, rstd, gamma, beta, bias,
                     input_node_size, output_node_size, frame_size, frame_stride, x_frame_stride, lut_binarize, 1);
}


/* ---- BinaryLutN<6> ------------------------------------------------------------------------- */

/* Generic loop of BinaryLutN<6,Bit>::Forward (include/bb/BinaryLutN.h:436-463): input k is table-index bit k,
 * entries 0-31 live in table word 0 (:170-171, 279-284). Only bits of frames < frame_size are written. */
void oracle_bit_BinaryLut6_Forward(int32_t const *x, int32_t *y, int32_t const *idx, int32_t const *table,
                                   int node_size, int frame_size, int frame_stride)
{
    #pragma omp parallel for
    for (int node = 0; node < node_size; ++node) {
        for (int f = 0; f < frame_size; ++f) {
            int index = 0, mask = 1;
            for (int i = 0; i < 6; ++i) {
                if (read_bit(x + (size_t)idx[node * 6 + i] * frame_stride, f)) { index |= mask; }
                mask <<= 1;
            }
            int v = (int)(((uint32_t)table[node * 2 + (index >> 5)] >> (index & 31)) & 1u);
            write_bit(y + (size_t)node * frame_stride, f, v);
        }
    }
}

/* The same loop for any width n = 2 .. 6 (BinaryLutN<N,Bit>::Forward is this loop for every N but 6 with host_simd,
 * include/bb/BinaryLutN.h:436-463): a node's table is (2^n + 31) / 32 words, entry i = bit i & 31 of word i >> 5 (:43-46, 170-171). */
void oracle_bit_BinaryLutN_Forward(int n, int32_t const *x, int32_t *y, int32_t const *idx, int32_t const *table,
                                   int node_size, int frame_size, int frame_stride)
{
    int const unit = ((1 << n) + 31) / 32;
    #pragma omp parallel for
    for (int node = 0; node < node_size; ++node) {
        for (int f = 0; f < frame_size; ++f) {
            int index = 0, mask = 1;
            for (int i = 0; i < n; ++i) {
                if (read_bit(x + (size_t)idx[node * n + i] * frame_stride, f)) { index |= mask; }
                mask <<= 1;
            }
            int v = (int)(((uint32_t)table[node * unit + (index >> 5)] >> (index & 31)) & 1u);
            write_bit(y + (size_t)node * frame_stride, f, v);
        }
    }
}

/* Word-parallel form of the AVX2 loop (BinaryLutN.h:322-433): y = OR_k (T_k & AND_j (bit_j(k) ? x_j : ~x_j)),
 * evaluated on whole 32-bit words, padding bits included — used as the timed CPU baseline. */
void oracle_bit_BinaryLut6_Forward_words(int32_t const *x, int32_t *y, int32_t const *idx, int32_t const *table,
                                         int node_size, int word_size, int frame_stride)
{
    #pragma omp parallel for
    for (int node = 0; node < node_size; ++node) {
        uint32_t const t0 = (uint32_t)table[node * 2 + 0], t1 = (uint32_t)table[node * 2 + 1];
        uint32_t const *xr[6];
        for (int i = 0; i < 6; ++i) { xr[i] = (uint32_t const *)x + (size_t)idx[node * 6 + i] * frame_stride; }
        uint32_t *yr = (uint32_t *)y + (size_t)node * frame_stride;
        for (int w = 0; w < word_size; ++w) {
            uint32_t xv[6];
            for (int i = 0; i < 6; ++i) { xv[i] = xr[i][w]; }
            uint32_t acc = 0;
            for (int k = 0; k < 64; ++k) {
                uint32_t lut = (((k < 32 ? t0 : t1) >> (k & 31)) & 1u) ? 0xffffffffu : 0u;
                for (int j = 0; j < 6; ++j) { lut &= ((k >> j) & 1) ? xv[j] : ~xv[j]; }
                acc |= lut;
            }
            yr[w] = acc;
        }
    }
}


/* ---- connection tables --------------------------------------------------------------------- */

/* FixedSizeConnectionTable<N>::BuildReverseTable (include/bb/FixedSizeConnectionTable.h:180-215).
 * Returns the row stride 1 + max fan-out. When rev != NULL and stride*input_node_size <= rev_cap the table is
 * written: row r = [count, node*N+input ... in ascending (node,input) order, zero tail]. */
int oracle_ReverseTable(int n, int32_t const *idx, int input_node_size, int output_node_size, int32_t *rev, int rev_cap)
{
    int *cnt = (int *)calloc((size_t)input_node_size, sizeof(int));
    for (int node = 0; node < output_node_size; ++node) {
        for (int i = 0; i < n; ++i) { cnt[idx[node * n + i]]++; }
    }
    int max_n = 0;
    for (int r = 0; r < input_node_size; ++r) { if (cnt[r] > max_n) { max_n = cnt[r]; } }
    free(cnt);
    int stride = max_n + 1;
    if (rev && (long long)stride * input_node_size <= rev_cap) {
        memset(rev, 0, sizeof(int32_t) * (size_t)stride * (size_t)input_node_size);
        for (int node = 0; node < output_node_size; ++node) {
            for (int i = 0; i < n; ++i) {
                int32_t r = idx[node * n + i];
                int32_t c = rev[(size_t)r * stride] + 1;
                rev[(size_t)r * stride]     = c;
                rev[(size_t)r * stride + c] = (int32_t)(node * n + i);
            }
        }
    }
    return stride;
}


/* ---- timed CPU baseline (port) ----------------------------------------------------------------- */
#include <time.h>

/* One warm-up, then `reps` repetitions of StochasticLut6 forward+backward (AVX2 association), wall-clock around the
 * two calls only. */
void oracle_fp32_StochasticLut6_Time(float const *x, float const *dy, int32_t const *idx, float const *W,
                                     int input_node_size, int output_node_size, int frame_size, int reps, double *seconds)
{
    float *y  = (float *)malloc(sizeof(float) * (size_t)output_node_size * frame_size);
    float *dx = (float *)malloc(sizeof(float) * (size_t)input_node_size * frame_size);
    float *dW = (float *)calloc((size_t)output_node_size * 64, sizeof(float));
    for (int r = -1; r < reps; ++r) {
        struct timespec t0, t1;
        clock_gettime(CLOCK_MONOTONIC, &t0);
        oracle_fp32_StochasticLut_Forward(6, x, y, idx, W, output_node_size, frame_size, frame_size, 0, 0, 0.25f, 1);
        oracle_fp32_StochasticLut_Backward(6, x, dy, dx, idx, W, dW, input_node_size, output_node_size, frame_size, frame_size, 0, 0, 0.25f, 1);
        clock_gettime(CLOCK_MONOTONIC, &t1);
        if (r >= 0) { seconds[r] = (double)(t1.tv_sec - t0.tv_sec) + 1e-9 * (double)(t1.tv_nsec - t0.tv_nsec); }
    }
    free(y); free(dx); free(dW);
}

/* ------------------------------------------------------------------------------------------------
 * Elementwise vector operations of the reference's Tensor arithmetic (include/bb/TensorOperator.h:41-238) and the
 * Adam update (include/bb/OptimizerAdam.h:166-180, host path).  Evaluated in fp32 operation by operation (this file
 * is built with -ffp-contract=off).  Pinned by: numpy closed forms in fp32 (tests/test_oracle.py), the reference's
 * own Tensor operators and OptimizerAdam through oracle/_ref where it is built, the model in the reference's
 * optimizer test (tests/gtest/OptimizerAdamTest.cpp:10-40) restated in the test, and tests/golden/adam.npz.
 * op: 0 add_ex, 1 mul_ex, 2 div_ex, 3 sqrt, 4 exp, 5 min, 6 min_v, 7 max, 8 max_v (std::min / std::max semantics)
 * ------------------------------------------------------------------------------------------------ */
void oracle_fp32_Vector_op(int op, float *dst, float const *src0, float const *src1, float a, float b, float c, float d, int size)
{
    for (int i = 0; i < size; ++i) {
        float const x = src0[i];
        float const y = src1 ? src1[i] : 0.0f;
        float r;
        switch (op) {
        case 0:  r = a * x + b * y + c; break;                       /* TensorOperator.h:54 */
        case 1:  r = a * x * y + b; break;                           /* :91 */
        case 2:  r = (a * x + b) / (c * y + d); break;               /* :110 */
        case 3:  r = sqrtf(x); break;                                /* :137 */
        case 4:  r = expf(x); break;                                 /* :164 */
        case 5:  r = (y < x) ? y : x; break;                         /* :179 std::min(src0, src1) */
        case 6:  r = (a < x) ? a : x; break;                         /* :193 */
        case 7:  r = (x < y) ? y : x; break;                         /* :208 std::max(src0, src1) */
        default: r = (x < a) ? a : x; break;                         /* :222 */
        }
        dst[i] = r;
    }
}

/* One Adam step on one tensor; lr_t is computed by the caller as the reference does (OptimizerAdam.h:171). */
void oracle_fp32_OptimizerAdam(int size, float *param, float const *grad, float *m, float *v, float lr_t, float beta1, float beta2)
{
    float const nb1 = 1.0f - beta1, nb2 = 1.0f - beta2;
    for (int i = 0; i < size; ++i) {
        float const g = grad[i];
        float t = g - m[i];          t = nb1 * t;   m[i] = m[i] + t;          /* m += (1-b1)*(g - m)   :173 */
        float u = g * g;  u = u - v[i]; u = nb2 * u; v[i] = v[i] + u;         /* v += (1-b2)*(g*g - v) :174 */
        float num = lr_t * m[i];
        float den = sqrtf(v[i]) + 1.0e-7f;
        param[i] = param[i] - num / den;                                       /* p -= lr_t*m/(sqrt(v)+1e-7) :176 */
    }
}


/* ------------------------------------------------------------------------------------------------
 * Convolution plumbing around the LUT layers: Im2Col, Col2Im, StochasticMaxPooling2x2 (host paths of
 * include/bb/ConvolutionIm2Col.h:317-470, ConvolutionCol2Im.h:203-300, StochasticMaxPooling2x2.h:190-320).
 * Buffers are node-major, frame-minor with explicit strides (floats, or 32-bit words for packed bits).
 * Pinned by: the known answers of the reference's tests (tests/gtest/ConvolutionIm2ColTest.cpp:20-200,
 * ConvolutionCol2ImTest.cpp), restated in tests/test_oracle_conv.py; the reference's own classes through
 * oracle/_ref where built; tests/golden/conv.npz; permutation identities (Col2Im backward inverts forward,
 * Im2Col backward = transpose of forward on constant borders, pooling = 1 - prod(1 - x)).
 * border_mode: 0 constant, 1 reflect, 2 reflect_101, 3 replicate, 4 wrap (include/bb/DataType.h BB_BORDER_*).
 * ------------------------------------------------------------------------------------------------ */
static int im2col_border(int mode, int *x, int *y, int w, int h)        /* ConvolutionIm2Col.h:251-286 */
{
    switch (mode) {
    case 1: if (*x < 0) { *x = -*x - 1; } if (*y < 0) { *y = -*y - 1; }
            if (*x >= w) { *x = (w - 1) - (*x - w); } if (*y >= h) { *y = (h - 1) - (*y - h); } return 1;
    case 2: if (*x < 0) { *x = -*x; } if (*y < 0) { *y = -*y; }
            if (*x >= w) { *x = (w - 2) - (*x - w); } if (*y >= h) { *y = (h - 2) - (*y - h); } return 1;
    case 3: if (*x < 0) { *x = 0; } if (*y < 0) { *y = 0; } if (*x >= w) { *x = w - 1; } if (*y >= h) { *y = h - 1; } return 1;
    case 4: if (*x < 0) { *x += w; } if (*y < 0) { *y += h; } if (*x >= w) { *x -= w; } if (*y >= h) { *y -= h; } return 1;
    default: return 0;
    }
}

static int get_bit(int const *row, long long f) { return (row[f >> 5] >> (f & 31)) & 1; }
static void set_bit(int *row, long long f, int v)
{
    unsigned int const m = 1u << (f & 31);
    unsigned int w = (unsigned int)row[f >> 5];
    w = v ? (w | m) : (w & ~m);
    row[f >> 5] = (int)w;
}

/* is_bit = 0: fp32 buffers; 1: packed bits (border_value is then 0/1) */
static void im2col_forward(int is_bit, void const *x, void *y, int x_stride, int y_stride, int x_offset, int y_offset,
                           int input_frame_size, int input_frame_stride, int w, int h, int c_size, int ow, int oh,
                           int output_frame_stride, int fw, int fh, int border_mode, float border_value)
{
    long long const output_size = (long long)oh * ow;
    long long const output_frame_size = (long long)input_frame_size * output_size;
    for (int c = 0; c < c_size; ++c) {
        for (int fy = 0; fy < fh; ++fy) {
            for (int fx = 0; fx < fw; ++fx) {
                long long const out_node = ((long long)c * fh + fy) * fw + fx;
                for (long long of = 0; of < output_frame_size; ++of) {
                    long long const in_frame = of / output_size;
                    long long const f = of % output_size;
                    int iy = (int)(f / ow) * y_stride - y_offset + fy;
                    int ix = (int)(f % ow) * x_stride - x_offset + fx;
                    int have = (iy >= 0 && iy < h && ix >= 0 && ix < w);
                    if (!have) { have = im2col_border(border_mode, &ix, &iy, w, h); }
                    long long const in_node = ((long long)c * h + iy) * w + ix;
                    if (is_bit) {
                        int const v = have ? get_bit((int const *)x + in_node * input_frame_stride, in_frame) : (border_value > 0.5f);
                        set_bit((int *)y + out_node * output_frame_stride, of, v);
                    }
                    else {
                        float const v = have ? ((float const *)x)[in_node * input_frame_stride + in_frame] : border_value;
                        ((float *)y)[out_node * output_frame_stride + of] = v;
                    }
                }
            }
        }
    }
}

void oracle_fp32_Im2Col_Forward(float const *x, float *y, int x_stride, int y_stride, int x_offset, int y_offset,
                                int input_frame_size, int input_frame_stride, int w, int h, int c, int ow, int oh,
                                int output_frame_stride, int fw, int fh, int border_mode, float border_value)
{
    im2col_forward(0, x, y, x_stride, y_stride, x_offset, y_offset, input_frame_size, input_frame_stride, w, h, c, ow, oh,
                   output_frame_stride, fw, fh, border_mode, border_value);
}

void oracle_bit_Im2Col_Forward(int const *x, int *y, int x_stride, int y_stride, int x_offset, int y_offset,
                               int input_frame_size, int input_frame_stride, int w, int h, int c, int ow, int oh,
                               int output_frame_stride, int fw, int fh, int border_mode)
{
    im2col_forward(1, x, y, x_stride, y_stride, x_offset, y_offset, input_frame_size, input_frame_stride, w, h, c, ow, oh,
                   output_frame_stride, fw, fh, border_mode, 0.0f);
}

/* ConvolutionIm2Col.h:411-452: only in-range taps contribute (border replicas carry no gradient); sums in (fy, fx) order */
void oracle_fp32_Im2Col_Backward(float const *dy, float *dx, int x_stride, int y_stride, int x_offset, int y_offset,
                                 int input_frame_size, int input_frame_stride, int w, int h, int c_size, int ow, int oh,
                                 int output_frame_stride, int fw, int fh)
{
    int const iy_limit = (oh - 1) * y_stride, ix_limit = (ow - 1) * x_stride;
    for (int c = 0; c < c_size; ++c) {
        for (int y = 0; y < h; ++y) {
            for (int x = 0; x < w; ++x) {
                long long const in_node = ((long long)c * h + y) * w + x;
                int const x_align = x % x_stride, y_align = y % y_stride;
                for (int f = 0; f < input_frame_size; ++f) {
                    float s = 0.0f;
                    for (int fy = y_align; fy < fh; fy += y_stride) {
                        int const iy = y - fy + y_offset;
                        if (iy < 0 || iy > iy_limit) { continue; }
                        for (int fx = x_align; fx < fw; fx += x_stride) {
                            int const ix = x - fx + x_offset;
                            if (ix < 0 || ix > ix_limit) { continue; }
                            long long const of = ((long long)f * oh + (iy / y_stride)) * ow + (ix / x_stride);
                            long long const out_node = ((long long)c * fh + fy) * fw + fx;
                            s += dy[out_node * output_frame_stride + of];
                        }
                    }
                    dx[in_node * input_frame_stride + f] = s;
                }
            }
        }
    }
}

/* ConvolutionCol2Im.h:203-217: y[(c, xy)][f] = x[c][f*hw + xy] */
void oracle_fp32_Col2Im_Forward(float const *x, float *y, int w, int h, int c_size, int input_frame_stride,
                                int output_frame_size, int output_frame_stride)
{
    long long const hw = (long long)h * w;
    for (int c = 0; c < c_size; ++c) {
        for (long long xy = 0; xy < hw; ++xy) {
            for (int f = 0; f < output_frame_size; ++f) {
                y[(c * hw + xy) * output_frame_stride + f] = x[(long long)c * input_frame_stride + f * hw + xy];
            }
        }
    }
}

void oracle_bit_Col2Im_Forward(int const *x, int *y, int w, int h, int c_size, int input_frame_stride,
                               int output_frame_size, int output_frame_stride)
{
    long long const hw = (long long)h * w;
    for (int c = 0; c < c_size; ++c) {
        for (long long xy = 0; xy < hw; ++xy) {
            for (int f = 0; f < output_frame_size; ++f) {
                set_bit(y + (c * hw + xy) * output_frame_stride, f, get_bit(x + (long long)c * input_frame_stride, f * hw + xy));
            }
        }
    }
}

/* ConvolutionCol2Im.h:279-293: dx[c][f*hw + xy] = dy[(c, xy)][f].  input_* describe dx, output_* describe dy. */
void oracle_fp32_Col2Im_Backward(float const *dy, float *dx, int w, int h, int c_size, int input_frame_stride,
                                 int output_frame_size, int output_frame_stride)
{
    long long const hw = (long long)h * w;
    for (int c = 0; c < c_size; ++c) {
        for (long long xy = 0; xy < hw; ++xy) {
            for (int f = 0; f < output_frame_size; ++f) {
                dx[(long long)c * input_frame_stride + f * hw + xy] = dy[(c * hw + xy) * output_frame_stride + f];
            }
        }
    }
}

/* StochasticMaxPooling2x2.h:190-218: y = 1 - prod over the window (taps inside the image, (fy, fx) ascending) of (1 - x) */
void oracle_fp32_StochasticMaxPooling2x2_Forward(float const *x, float *y, int w, int h, int ow, int oh, int c_size,
                                                 int frame_size, int frame_stride)
{
    for (int c = 0; c < c_size; ++c) {
        for (int oy = 0; oy < oh; ++oy) {
            for (int ox = 0; ox < ow; ++ox) {
                for (int f = 0; f < frame_size; ++f) {
                    float out = 1.0f;
                    for (int fy = 0; fy < 2; ++fy) {
                        int const iy = oy * 2 + fy;
                        if (iy >= h) { continue; }
                        for (int fx = 0; fx < 2; ++fx) {
                            int const ix = ox * 2 + fx;
                            if (ix >= w) { continue; }
                            out *= (1.0f - x[(((long long)c * h + iy) * w + ix) * frame_stride + f]);
                        }
                    }
                    y[(((long long)c * oh + oy) * ow + ox) * frame_stride + f] = 1.0f - out;
                }
            }
        }
    }
}

/* StochasticMaxPooling2x2.h:262-306: in_grad = (float)(dy * (1.0 - other taps ...)) evaluated in double; taps outside the
 * image read as 0 */
void oracle_fp32_StochasticMaxPooling2x2_Backward(float const *x, float const *dy, float *dx, int w, int h, int ow, int oh,
                                                  int c_size, int frame_size, int frame_stride)
{
    for (int c = 0; c < c_size; ++c) {
        for (int oy = 0; oy < oh; ++oy) {
            for (int ox = 0; ox < ow; ++ox) {
                for (int f = 0; f < frame_size; ++f) {
                    float in[2][2] = {{0, 0}, {0, 0}};
                    for (int fy = 0; fy < 2; ++fy) {
                        for (int fx = 0; fx < 2; ++fx) {
                            int const iy = oy * 2 + fy, ix = ox * 2 + fx;
                            if (iy < h && ix < w) { in[fy][fx] = x[(((long long)c * h + iy) * w + ix) * frame_stride + f]; }
                        }
                    }
                    float const g = dy[(((long long)c * oh + oy) * ow + ox) * frame_stride + f];
                    float gr[2][2];
                    gr[0][0] = (float)(g * (1.0 - in[0][1]) * (1.0 - in[1][0]) * (1.0 - in[1][1]));
                    gr[0][1] = (float)(g * (1.0 - in[0][0]) * (1.0 - in[1][0]) * (1.0 - in[1][1]));
                    gr[1][0] = (float)(g * (1.0 - in[0][0]) * (1.0 - in[0][1]) * (1.0 - in[1][1]));
                    gr[1][1] = (float)(g * (1.0 - in[0][0]) * (1.0 - in[0][1]) * (1.0 - in[1][0]));
                    for (int fy = 0; fy < 2; ++fy) {
                        for (int fx = 0; fx < 2; ++fx) {
                            int const iy = oy * 2 + fy, ix = ox * 2 + fx;
                            if (iy < h && ix < w) { dx[(((long long)c * h + iy) * w + ix) * frame_stride + f] = gr[fy][fx]; }
                        }
                    }
                }
            }
        }
    }
}


/* ---------------------------------------------------------------------------------------------------------------------
 * AverageLut, LossSoftmaxCrossEntropy, MetricsCategoricalAccuracy: the host loops of the reference.
 *
 * Pinned by: bit-exact agreement with the reference's own classes (oracle/_ref) and the vectors written from them
 * (tests/golden/tail.npz); the NumPy known answers held by the reference's loss test
 * (tests/gtest/LossSoftmaxCrossEntropyTest.cpp:8-92: loss 2.29783..., dy table, tolerances 1e-4 / 1e-6); closed forms
 * (AverageLut of +-1 inputs = sign of the count; backward column sums = n * dy / n; softmax rows sum to 1 so each
 * frame's dy sums to (t_max - sum t)/t_sum = 0 for one-hot targets; uniform logits give loss log(ch); accuracy of
 * y = t is 1).
 * ------------------------------------------------------------------------------------------------------------------ */

/* AverageLut.h:320-345 (host loop; the value written without binarize_output is the SUM, not the mean) */
void oracle_fp32_AverageLut_Forward(float const *x, float *y, int32_t const *idx, int n, int node_size, int frame_size,
                                    int frame_stride, int binarize_input, int binarize_output)
{
    for (int node = 0; node < node_size; ++node) {
        for (int f = 0; f < frame_size; ++f) {
            float sum = 0;
            for (int i = 0; i < n; ++i) {
                float val = x[(long long)idx[node * n + i] * frame_stride + f];
                if (binarize_input) { val = (val > 0) ? 1.0f : -1.0f; }
                sum += val;
            }
            if (binarize_output) { sum = (sum > 0) ? 1.0f : -1.0f; }
            y[(long long)node * frame_stride + f] = sum;
        }
    }
}

/* The same loop on packed bits: a Bit reads as +1 / -1 (DataType.h:302-303) and is written as (sum > 0)
 * (DataType.h:277-278), so the flags do not matter and the result is the strict majority of the n inputs. */
void oracle_bit_AverageLut_Forward(int const *x, int *y, int32_t const *idx, int n, int node_size, int frame_size,
                                   int frame_stride)
{
    for (int node = 0; node < node_size; ++node) {
        for (int f = 0; f < frame_size; ++f) {
            float sum = 0;
            for (int i = 0; i < n; ++i) {
                sum += get_bit(x + (long long)idx[node * n + i] * frame_stride, f) ? 1.0f : -1.0f;
            }
            set_bit(y + (long long)node * frame_stride, f, sum > 0);
        }
    }
}

/* AverageLut.h:386-406: dx = 0, then node ascending, input ascending: dx[input] += dy / n */
void oracle_fp32_AverageLut_Backward(float const *dy, float *dx, int32_t const *idx, int n, int input_node_size,
                                     int output_node_size, int frame_size, int frame_stride)
{
    memset(dx, 0, sizeof(float) * (size_t)input_node_size * (size_t)frame_stride);
    for (int node = 0; node < output_node_size; ++node) {
        for (int f = 0; f < frame_size; ++f) {
            float const g = dy[(long long)node * frame_stride + f] / n;
            for (int i = 0; i < n; ++i) {
                dx[(long long)idx[node * n + i] * frame_stride + f] += g;
            }
        }
    }
}

/* LossSoftmaxCrossEntropy.h:150-156: the host path's sum of the targets, frame outer, node inner, in float */
float oracle_fp32_LossSoftmaxCrossEntropy_TSum(float const *t, int node_size, int frame_size, int frame_stride)
{
    float t_sum = 0;
    for (int f = 0; f < frame_size; ++f) {
        for (int node = 0; node < node_size; ++node) { t_sum += t[(long long)node * frame_stride + f]; }
    }
    return t_sum;
}

/* LossSoftmaxCrossEntropy.h:159-211: node = ch * pix_size + pix; per frame loss_buf += log(softmax + eps) * t_max over
 * the channels with t > 0; dy = (t_max * softmax - t) / t_sum.  The caller negates and sums loss_buf (:213-219). */
void oracle_fp32_LossSoftmaxCrossEntropy(float const *y, float const *t, float *dy, double *loss_buf, float t_sum,
                                         int pix_size, int ch_size, int frame_size, int frame_stride)
{
    float const eps = 1.0e-7f;
    for (int f = 0; f < frame_size; ++f) {
        loss_buf[f] = 0;
        for (int pix = 0; pix < pix_size; ++pix) {
            float c = -3.402823466e+38f;
            for (int ch = 0; ch < ch_size; ++ch) {
                float const v = y[(long long)(ch * pix_size + pix) * frame_stride + f];
                c = (c < v) ? v : c;                                           /* std::max(c, v) */
            }
            float y_sum = 0, t_max = 0;
            for (int ch = 0; ch < ch_size; ++ch) {
                long long const at = (long long)(ch * pix_size + pix) * frame_stride + f;
                y_sum += expf(y[at] - c);
                t_max += t[at];
            }
            if (y_sum <= eps) { y_sum = eps; }
            for (int ch = 0; ch < ch_size; ++ch) {
                long long const at = (long long)(ch * pix_size + pix) * frame_stride + f;
                float const softmax = expf(y[at] - c) / y_sum;
                if (t[at] > 0) { loss_buf[f] += logf(softmax + eps) * t_max; }
                dy[at] = (t_max * softmax - t[at]) / t_sum;
            }
        }
    }
}

/* MetricsCategoricalAccuracy.h:144-173: per pixel the first channel holding the largest y decides; pixels whose targets
 * are all <= 0 are not counted */
void oracle_fp32_MetricsCategoricalAccuracy(float const *y, float const *t, int *accuracy_buf, int *category_buf,
                                            int pix_size, int ch_size, int frame_size, int frame_stride)
{
    for (int f = 0; f < frame_size; ++f) {
        int accuracy = 0, category = 0;
        for (int pix = 0; pix < pix_size; ++pix) {
            float max_y = -3.402823466e+38f, max_t = -3.402823466e+38f;
            int valid = 0;
            for (int ch = 0; ch < ch_size; ++ch) {
                long long const at = (long long)(ch * pix_size + pix) * frame_stride + f;
                if (t[at] > 0) { valid = 1; }
                if (y[at] > max_y) { max_y = y[at]; max_t = t[at]; }
            }
            if (valid) { category += 1; if (max_t > 0) { accuracy += 1; } }
        }
        accuracy_buf[f] = accuracy;
        category_buf[f] = category;
    }
}

/* ---------------------------------------------------------------------------------------------------------------------
 *  StochasticBatchNormalization: per-node batch normalisation with scalar gamma / beta, the unfused twin of the
 *  normalisation inside DifferentiableLutN (reference host path, include/bb/StochasticBatchNormalization.h: training forward
 *  :535-597, re-forward :655-678, backward :815-851).  fp32 sums in frame order, as the reference's generic loops.
 *  Pinned by tests/test_oracle_bn.py: the reference's own class where oracle/_ref is built, tests/golden/bn.npz elsewhere,
 *  textbook mean / variance in fp64, the invariants sum_f dx = 0 and sum_f dx (x - mean) = 0.
 *  Inference: y = ((x - running_mean) * rstd) * gamma + beta with rstd = 1 / (sqrt(running_var) + 1e-7), the form of the
 *  reference's re-forward, its ForwardNode (:319-341) and its CUDA kernel.  The reference's generic host inference (:599-616)
 *  folds the same into gain * x + offset but takes the mean of the LAST TRAINING BATCH for the offset where every other path
 *  takes the running mean; that is not reproduced.
 * ------------------------------------------------------------------------------------------------------------------- */
void oracle_fp32_StochasticBatchNormalization_ForwardTraining(float const *x, float *y, float *mean_buf, float *rstd_buf,
                                                              float *running_mean, float *running_var, float gamma, float beta,
                                                              float momentum, int node_size, int frame_size, int frame_stride)
{
    for (int node = 0; node < node_size; ++node) {
        float const *xr = x + (size_t)node * frame_stride;
        float *yr = y + (size_t)node * frame_stride;
        float mean = 0.0f;
        for (int f = 0; f < frame_size; ++f) { mean += xr[f]; }
        mean /= (float)frame_size;
        float var = 0.0f;
        for (int f = 0; f < frame_size; ++f) { float const xc = xr[f] - mean; var += xc * xc; }
        var /= (float)frame_size;
        var = fmaxf(0.0f, var);
        float const rstd = 1.0f / (sqrtf(var) + 1.0e-7f);
        running_mean[node] = running_mean[node] * momentum + mean * (1.0f - momentum);
        running_var[node]  = running_var[node]  * momentum + var  * (1.0f - momentum);
        mean_buf[node] = mean;
        rstd_buf[node] = rstd;
        for (int f = 0; f < frame_size; ++f) {
            float v = (xr[f] - mean) * rstd;
            yr[f] = v * gamma + beta;
        }
    }
}

/* re-forward with stored statistics (:655-678) */
void oracle_fp32_StochasticBatchNormalization_ReForward(float const *x, float *y, float const *mean_buf, float const *rstd_buf,
                                                        float gamma, float beta, int node_size, int frame_size, int frame_stride)
{
    for (int node = 0; node < node_size; ++node) {
        float const mean = mean_buf[node], rstd = rstd_buf[node];
        for (int f = 0; f < frame_size; ++f) {
            float v = (x[(size_t)node * frame_stride + f] - mean) * rstd;
            y[(size_t)node * frame_stride + f] = v * gamma + beta;
        }
    }
}

void oracle_fp32_StochasticBatchNormalization_ForwardInference(float const *x, float *y, float const *running_mean,
                                                               float const *running_var, float gamma, float beta,
                                                               int node_size, int frame_size, int frame_stride)
{
    for (int node = 0; node < node_size; ++node) {
        float const mean = running_mean[node];
        float const rstd = 1.0f / (sqrtf(running_var[node]) + 1.0e-7f);
        for (int f = 0; f < frame_size; ++f) {
            float v = (x[(size_t)node * frame_stride + f] - mean) * rstd;
            y[(size_t)node * frame_stride + f] = v * gamma + beta;
        }
    }
}

/* backward (:815-851): dstd = -sum dxn xc rstd^2, dmeanx = -sum dxn rstd with dxn = gamma dy;
 * dvar = dstd rstd; dmean = (dmeanx - mean dvar) / F; dx = dxn rstd + dmean + x dvar / F */
void oracle_fp32_StochasticBatchNormalization_Backward(float const *x, float const *dy, float *dx, float const *mean_buf,
                                                       float const *rstd_buf, float gamma, int node_size, int frame_size,
                                                       int frame_stride, int x_frame_stride)
{
    for (int node = 0; node < node_size; ++node) {
        float const *xr = x + (size_t)node * x_frame_stride;
        float const *dyr = dy + (size_t)node * frame_stride;
        float *dxr = dx + (size_t)node * frame_stride;
        float const mean = mean_buf[node], rstd = rstd_buf[node];
        float dmeanx = 0.0f, dstd = 0.0f;
        for (int f = 0; f < frame_size; ++f) {
            float const xc = xr[f] - mean;
            float const dxn = gamma * dyr[f];
            dstd   += -(dxn * xc * (rstd * rstd));
            dmeanx += -(dxn * rstd);
        }
        float const dvar  = dstd * rstd;
        float const dmean = (dmeanx - (mean * dvar)) / (float)frame_size;
        for (int f = 0; f < frame_size; ++f) {
            float const dxn = dyr[f] * gamma;
            float const dxc = dxn * rstd;
            dxr[f] = dxc + dmean + (xr[f] * dvar / (float)frame_size);
        }
    }
}

/* ---------------------------------------------------------------------------------------------------------------------
 *  MaxLut: the largest of n wired inputs (reference host path, include/bb/MaxLut.h: forward :293-318, backward :394-424).
 *  The running maximum starts at BB_BINARY_LO = -1 (DataType.h:49) and is replaced by a strictly larger value, so the
 *  output is never below -1 and the gradient goes to the FIRST largest input (to input 0 when none exceeds -1).
 *  binarize_output: +1 where the maximum is positive, else -1.  The host loop does not look at binarize_input; the
 *  reference's device kernel does (cuda/MaxLut.cu:33-36: x = x > 0 ? +1 : -1 before the comparison) and the flag is
 *  restated here in that meaning — with the flag off this is the host loop.
 *  Packed bits: a Bit is +1 / -1, so the maximum is the OR of the inputs and the gradient goes to the first input
 *  that is set (input 0 when none is).
 *  Pinned by tests/test_oracle_maxlut.py: the reference's class (oracle/_ref) and vectors written from it
 *  (tests/golden/maxlut.npz), the known answers of tests/gtest/MaxLutTest.cpp:15-139, numpy max / argmax.
 * ------------------------------------------------------------------------------------------------------------------- */
void oracle_fp32_MaxLut_Forward(float const *x, float *y, int32_t const *idx, int n, int node_size, int frame_size,
                                int frame_stride, int binarize_input, int binarize_output)
{
    for (int node = 0; node < node_size; ++node) {
        for (int f = 0; f < frame_size; ++f) {
            float max_val = -1.0f;
            for (int i = 0; i < n; ++i) {
                float val = x[(long long)idx[node * n + i] * frame_stride + f];
                if (binarize_input) { val = (val > 0) ? 1.0f : -1.0f; }
                if (val > max_val) { max_val = val; }
            }
            if (binarize_output) { max_val = (max_val > 0) ? 1.0f : -1.0f; }
            y[(long long)node * frame_stride + f] = max_val;
        }
    }
}

void oracle_bit_MaxLut_Forward(int const *x, int *y, int32_t const *idx, int n, int node_size, int frame_size, int frame_stride)
{
    for (int node = 0; node < node_size; ++node) {
        for (int f = 0; f < frame_size; ++f) {
            int any = 0;
            for (int i = 0; i < n; ++i) { any |= get_bit(x + (long long)idx[node * n + i] * frame_stride, f); }
            set_bit(y + (long long)node * frame_stride, f, any);
        }
    }
}

/* dx = 0, then node ascending: dx[first largest input] += dy */
void oracle_fp32_MaxLut_Backward(float const *x, float const *dy, float *dx, int32_t const *idx, int n, int input_node_size,
                                 int output_node_size, int frame_size, int frame_stride, int binarize_input)
{
    memset(dx, 0, sizeof(float) * (size_t)input_node_size * (size_t)frame_stride);
    for (int node = 0; node < output_node_size; ++node) {
        for (int f = 0; f < frame_size; ++f) {
            float max_val = -1.0f;
            int max_idx = 0;
            for (int i = 0; i < n; ++i) {
                float val = x[(long long)idx[node * n + i] * frame_stride + f];
                if (binarize_input) { val = (val > 0) ? 1.0f : -1.0f; }
                if (val > max_val) { max_val = val; max_idx = i; }
            }
            dx[(long long)idx[node * n + max_idx] * frame_stride + f] += dy[(long long)node * frame_stride + f];
        }
    }
}

void oracle_bit_MaxLut_Backward(int const *x, float const *dy, float *dx, int32_t const *idx, int n, int input_node_size,
                                int output_node_size, int frame_size, int x_frame_stride, int dy_frame_stride)
{
    memset(dx, 0, sizeof(float) * (size_t)input_node_size * (size_t)dy_frame_stride);
    for (int node = 0; node < output_node_size; ++node) {
        for (int f = 0; f < frame_size; ++f) {
            int max_idx = 0;
            for (int i = 0; i < n; ++i) {
                if (get_bit(x + (long long)idx[node * n + i] * x_frame_stride, f)) { max_idx = i; break; }
            }
            dx[(long long)idx[node * n + max_idx] * dy_frame_stride + f] += dy[(long long)node * dy_frame_stride + f];
        }
    }
}

/* ---------------------------------------------------------------------------------------------------------------------
 *  Reduce: output node o is the mean of the input nodes o, O + o, 2 O + o, ... (reference host loop,
 *  include/bb/Reduce.h:172-190; backward :229-247: every one of them receives dy / mux).  Packed bits read as +1 / -1
 *  (DataType.h:302-303).  fp32 sums in input order, one division.
 *  LossMeanSquaredError (include/bb/LossMeanSquaredError.h:150-169): frame outer, node inner; dy = 2 (y - t) * grad_reduction
 *  in fp32; the loss accumulator (double) += (float)(y - t)^2 * loss_reduction unless that square is NaN.
 *  MetricsMeanSquaredError (include/bb/MetricsMeanSquaredError.h:66-85): accumulator (double) += (float)(t - y)^2 / node_size.
 *  Pinned by tests/test_oracle_reduce_mse.py: the reference's classes (oracle/_ref), vectors written from them
 *  (tests/golden/reduce_mse.npz), numpy means in fp64.
 * ------------------------------------------------------------------------------------------------------------------- */
void oracle_fp32_Reduce_Forward(float const *x, float *y, int input_node_size, int output_node_size, int frame_size, int frame_stride)
{
    int const mux = input_node_size / output_node_size;
    for (int o = 0; o < output_node_size; ++o) {
        for (int f = 0; f < frame_size; ++f) {
            float sum = 0;
            for (int i = 0; i < mux; ++i) { sum += x[(long long)(output_node_size * i + o) * frame_stride + f]; }
            y[(long long)o * frame_stride + f] = sum / (float)mux;
        }
    }
}

void oracle_bit_fp32_Reduce_Forward(int const *x, float *y, int input_node_size, int output_node_size, int frame_size,
                                    int x_frame_stride, int y_frame_stride)
{
    int const mux = input_node_size / output_node_size;
    for (int o = 0; o < output_node_size; ++o) {
        for (int f = 0; f < frame_size; ++f) {
            float sum = 0;
            for (int i = 0; i < mux; ++i) { sum += get_bit(x + (long long)(output_node_size * i + o) * x_frame_stride, f) ? 1.0f : -1.0f; }
            y[(long long)o * y_frame_stride + f] = sum / (float)mux;
        }
    }
}

void oracle_fp32_Reduce_Backward(float const *dy, float *dx, int input_node_size, int output_node_size, int frame_size, int frame_stride)
{
    int const mux = input_node_size / output_node_size;
    for (int o = 0; o < output_node_size; ++o) {
        for (int f = 0; f < frame_size; ++f) {
            float const g = dy[(long long)o * frame_stride + f] / (float)mux;
            for (int i = 0; i < mux; ++i) { dx[(long long)(output_node_size * i + o) * frame_stride + f] = g; }
        }
    }
}

void oracle_fp32_LossMeanSquaredError(float const *y, float const *t, float *dy, double *loss, int node_size, int frame_size,
                                      int frame_stride, float grad_reduction, double loss_reduction)
{
    for (int f = 0; f < frame_size; ++f) {
        for (int node = 0; node < node_size; ++node) {
            float const grad = y[(long long)node * frame_stride + f] - t[(long long)node * frame_stride + f];
            float const error = grad * grad;
            dy[(long long)node * frame_stride + f] = 2 * grad * grad_reduction;
            if (!isnan(error)) { *loss += error * loss_reduction; }
        }
    }
}

void oracle_fp32_MetricsMeanSquaredError(float const *y, float const *t, double *accuracy, int node_size, int frame_size, int frame_stride)
{
    for (int f = 0; f < frame_size; ++f) {
        for (int node = 0; node < node_size; ++node) {
            float const grad = t[(long long)node * frame_stride + f] - y[(long long)node * frame_stride + f];
            float const error = grad * grad;
            *accuracy += error / (double)node_size;
        }
    }
}

/* ---------------------------------------------------------------------------------------------------------------------
 *  The layers at either end of a binary network and the activations between its layers.
 *
 *  RealToBinary without a value generator (host loop include/bb/RealToBinary.h:300-344): input node (depth c, point p),
 *  input frame g; output node (depth c * dm + d, point p), output frame g * fm + f:
 *      v = (x - lo) * (1 / (hi - lo));  v = (v - d * (1/dm)) * dm;  v = (v - f * (1/fm)) * fm;  v = max(0, min(1, v))
 *  every operation rounded to fp32 on its own, min and max as std::min / std::max evaluate them (a NaN becomes 1), and
 *  in binary mode +1 where v > 0.5, else -1.  Packed output takes the bit of that value as Bit(v) does (DataType.h:278):
 *  v > 0, which is v > 0.5 before the +1 / -1 in binary mode and v > 0 after the clamp otherwise.
 *  BinaryToReal (include/bb/BinaryToReal.h:262-290, backward :333-352): output node o, frame g counts the inputs that are
 *  > 0 (set bits) among input nodes o, O + o, 2 O + o, ... and frames g * fmux ... g * fmux + fmux - 1 and divides the count by their
 *  number; backward sends dy * gain to each of them, gain = O / (I * fmux) in fp32.
 *  Binarize (include/bb/Binarize.h:196-213): y = x > th ? high : low; its backward is HardTanh's with the layer's own window
 *  (:268-285).  HardTanh (include/bb/HardTanh.h:176-193, :253-271): x <= min -> min, x >= max -> max; dx = 0 there, dy elsewhere.
 *  Pinned by tests/test_oracle_modulation.py: the reference's classes (oracle/_ref), vectors written from them
 *  (tests/golden/modulation.npz), the known answers of tests/gtest/RealToBinaryTest.cpp, BinaryToRealTest.cpp and
 *  BinarizeTest.cpp, and numpy restatements in fp64 where fp32 rounding cannot matter.
 * ------------------------------------------------------------------------------------------------------------------- */
static inline float std_min_f(float a, float b) { return (b < a) ? b : a; }     /* std::min(a, b) */
static inline float std_max_f(float a, float b) { return (a < b) ? b : a; }     /* std::max(a, b) */

static inline float real_to_binary_value(float x, long long d, long long f, float lo, float x_scale, float depth_step,
                                         float depth_step_recip, float frame_step, float frame_step_recip)
{
    float v = (x - lo) * x_scale;
    v = (v - (float)((float)d * depth_step)) * depth_step_recip;
    v = (v - (float)((float)f * frame_step)) * frame_step_recip;
    return std_max_f(0.0f, std_min_f(1.0f, v));
}

void oracle_fp32_RealToBinary_Forward(float const *x, float *y, int depth_modulation_size, int frame_modulation_size,
                                      float input_range_lo, float input_range_hi, int point_size, int x_depth_size,
                                      int x_frame_size, int x_frame_stride, int y_frame_stride, int binarize)
{
    float const frame_step = 1.0f / (float)frame_modulation_size, frame_step_recip = (float)frame_modulation_size;
    float const depth_step = 1.0f / (float)depth_modulation_size, depth_step_recip = (float)depth_modulation_size;
    float const x_scale = 1.0f / (input_range_hi - input_range_lo);
    for (int g = 0; g < x_frame_size; ++g) {
        for (int f = 0; f < frame_modulation_size; ++f) {
            long long const out_frame = (long long)g * frame_modulation_size + f;
            for (int c = 0; c < x_depth_size; ++c) {
                for (int p = 0; p < point_size; ++p) {
                    float const xv = x[((long long)c * point_size + p) * x_frame_stride + g];
                    for (int d = 0; d < depth_modulation_size; ++d) {
                        long long const out_node = ((long long)c * depth_modulation_size + d) * point_size + p;
                        float v = real_to_binary_value(xv, d, f, input_range_lo, x_scale, depth_step, depth_step_recip, frame_step, frame_step_recip);
                        if (binarize) { v = (v > 0.5f) ? 1.0f : -1.0f; }
                        y[out_node * y_frame_stride + out_frame] = v;
                    }
                }
            }
        }
    }
}

/* y rows are y_frame_stride words; the caller clears them (bits past the last frame stay 0) */
void oracle_bit_RealToBinary_Forward(float const *x, int *y, int depth_modulation_size, int frame_modulation_size,
                                     float input_range_lo, float input_range_hi, int point_size, int x_depth_size,
                                     int x_frame_size, int x_frame_stride, int y_frame_stride, int binarize)
{
    float const frame_step = 1.0f / (float)frame_modulation_size, frame_step_recip = (float)frame_modulation_size;
    float const depth_step = 1.0f / (float)depth_modulation_size, depth_step_recip = (float)depth_modulation_size;
    float const x_scale = 1.0f / (input_range_hi - input_range_lo);
    for (int g = 0; g < x_frame_size; ++g) {
        for (int f = 0; f < frame_modulation_size; ++f) {
            long long const out_frame = (long long)g * frame_modulation_size + f;
            for (int c = 0; c < x_depth_size; ++c) {
                for (int p = 0; p < point_size; ++p) {
                    float const xv = x[((long long)c * point_size + p) * x_frame_stride + g];
                    for (int d = 0; d < depth_modulation_size; ++d) {
                        long long const out_node = ((long long)c * depth_modulation_size + d) * point_size + p;
                        float v = real_to_binary_value(xv, d, f, input_range_lo, x_scale, depth_step, depth_step_recip, frame_step, frame_step_recip);
                        if (binarize) { v = (v > 0.5f) ? 1.0f : -1.0f; }
                        if (v > 0) { y[out_node * y_frame_stride + (out_frame >> 5)] |= (int)(1u << (out_frame & 31)); }
                    }
                }
            }
        }
    }
}

void oracle_fp32_BinaryToReal_Forward(float const *x, float *y, int node_mux_size, int frame_mux_size, int y_node_size,
                                      int x_frame_stride, int y_frame_size, int y_frame_stride)
{
    for (int g = 0; g < y_frame_size; ++g) {
        for (int o = 0; o < y_node_size; ++o) {
            float v = 0;
            int n = 0;
            for (int m = 0; m < node_mux_size; ++m) {
                for (int i = 0; i < frame_mux_size; ++i) {
                    float const sig = x[((long long)m * y_node_size + o) * x_frame_stride + (long long)g * frame_mux_size + i];
                    v += (sig > 0) ? 1 : 0;
                    n += 1;
                }
            }
            y[(long long)o * y_frame_stride + g] = v / (float)n;
        }
    }
}

void oracle_bit_fp32_BinaryToReal_Forward(int const *x, float *y, int node_mux_size, int frame_mux_size, int y_node_size,
                                          int x_frame_stride, int y_frame_size, int y_frame_stride)
{
    for (int g = 0; g < y_frame_size; ++g) {
        for (int o = 0; o < y_node_size; ++o) {
            float v = 0;
            int n = 0;
            for (int m = 0; m < node_mux_size; ++m) {
                for (int i = 0; i < frame_mux_size; ++i) {
                    v += get_bit(x + ((long long)m * y_node_size + o) * x_frame_stride, (long long)g * frame_mux_size + i) ? 1 : 0;
                    n += 1;
                }
            }
            y[(long long)o * y_frame_stride + g] = v / (float)n;
        }
    }
}

void oracle_fp32_BinaryToReal_Backward(float const *dy, float *dx, int node_mux_size, int frame_mux_size, int y_node_size,
                                       int x_frame_stride, int y_frame_size, int y_frame_stride)
{
    float const gain = (float)y_node_size / ((float)((long long)node_mux_size * y_node_size) * (float)frame_mux_size);
    for (long long node = 0; node < (long long)node_mux_size * y_node_size; ++node) {
        for (int g = 0; g < y_frame_size; ++g) {
            for (int i = 0; i < frame_mux_size; ++i) {
                float grad = dy[(node % y_node_size) * y_frame_stride + g];
                grad *= gain;
                dx[node * x_frame_stride + (long long)g * frame_mux_size + i] = grad;
            }
        }
    }
}

void oracle_fp32_Binarize_Forward(float const *x, float *y, float binary_th, float binary_low, float binary_high,
                                  int node_size, int frame_size, int frame_stride)
{
    for (int node = 0; node < node_size; ++node) {
        for (int f = 0; f < frame_size; ++f) {
            y[(long long)node * frame_stride + f] = x[(long long)node * frame_stride + f] > binary_th ? binary_high : binary_low;
        }
    }
}

/* y rows are y_frame_stride words; the caller clears them */
void oracle_fp32_bit_Binarize_Forward(float const *x, int *y, float binary_th, int node_size, int frame_size,
                                      int x_frame_stride, int y_frame_stride)
{
    for (int node = 0; node < node_size; ++node) {
        for (int f = 0; f < frame_size; ++f) {
            if (x[(long long)node * x_frame_stride + f] > binary_th) { y[(long long)node * y_frame_stride + (f >> 5)] |= (int)(1u << (f & 31)); }
        }
    }
}

void oracle_fp32_HardTanh_Forward(float const *x, float *y, float limit_min, float limit_max, int node_size, int frame_size, int frame_stride)
{
    for (int node = 0; node < node_size; ++node) {
        for (int f = 0; f < frame_size; ++f) {
            float v = x[(long long)node * frame_stride + f];
            if (v <= limit_min) { v = limit_min; }
            if (v >= limit_max) { v = limit_max; }
            y[(long long)node * frame_stride + f] = v;
        }
    }
}

void oracle_fp32_HardTanh_Backward(float const *x, float const *dy, float *dx, float limit_min, float limit_max,
                                   int node_size, int frame_size, int frame_stride)
{
    for (int node = 0; node < node_size; ++node) {
        for (int f = 0; f < frame_size; ++f) {
            float g = dy[(long long)node * frame_stride + f];
            float const v = x[(long long)node * frame_stride + f];
            if (v <= limit_min || v >= limit_max) { g = 0.0f; }
            dx[(long long)node * frame_stride + f] = g;
        }
    }
}

/* ---------------------------------------------------------------------------------------------------------------------
 *  MaxPooling (include/bb/MaxPooling.h): windows of filter_h x filter_w tile the image without overlap, the last ones cut off at
 *  the border (output = ceil(input / filter)).  fp32 forward (:251-284): the largest value of the window, found with a strict >
 *  from the lowest float in (fy, fx) order, and the position of its first occurrence counted over the positions inside the image;
 *  backward (:478-506): that position receives dy, the others 0.  Packed bits, windows below 32 positions (:340-370 forward: the
 *  OR of the window; :551-579 backward: dy goes to the first set input in (fy, fx) order, nothing when none is set).
 *  UpSampling (include/bb/UpSampling.h:223-259, :321-353): every input pixel becomes a filter_h x filter_w block, all of it (fill)
 *  or only its position (filter_h / 2, filter_w / 2) with zeros around; backward sums dy over the block in (fy, fx) order in fp32,
 *  or takes that one position.
 *  Pinned by tests/test_oracle_pooling.py: the reference's classes (oracle/_ref), vectors written from them
 *  (tests/golden/pooling.npz), the known answers of tests/gtest/MaxPoolingTest.cpp and UpSamplingTest.cpp, numpy.
 * ------------------------------------------------------------------------------------------------------------------- */
void oracle_fp32_MaxPooling_Forward(float const *x, float *y, int *argmax, int filter_h_size, int filter_w_size, int input_w_size,
                                    int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size, int frame_stride)
{
    for (int c = 0; c < c_size; ++c) {
        for (int oy = 0; oy < output_h_size; ++oy) {
            for (int ox = 0; ox < output_w_size; ++ox) {
                long long const out = (((long long)c * output_h_size + oy) * output_w_size + ox) * frame_stride;
                for (int f = 0; f < frame_size; ++f) {
                    float max_val = -3.402823466e+38f;      /* std::numeric_limits<float>::lowest() */
                    int best = 0, arg = 0;
                    for (int fy = 0; fy < filter_h_size; ++fy) {
                        int const iy = oy * filter_h_size + fy;
                        if (iy >= input_h_size) { continue; }
                        for (int fx = 0; fx < filter_w_size; ++fx) {
                            int const ix = ox * filter_w_size + fx;
                            if (ix >= input_w_size) { continue; }
                            float const v = x[(((long long)c * input_h_size + iy) * input_w_size + ix) * frame_stride + f];
                            if (v > max_val) { max_val = v; best = arg; }
                            ++arg;
                        }
                    }
                    y[out + f] = max_val;
                    argmax[out + f] = best;
                }
            }
        }
    }
}

void oracle_fp32_MaxPooling_Backward(int const *argmax, float const *dy, float *dx, int filter_h_size, int filter_w_size, int input_w_size,
                                     int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size, int frame_stride)
{
    for (int c = 0; c < c_size; ++c) {
        for (int oy = 0; oy < output_h_size; ++oy) {
            for (int ox = 0; ox < output_w_size; ++ox) {
                long long const out = (((long long)c * output_h_size + oy) * output_w_size + ox) * frame_stride;
                for (int f = 0; f < frame_size; ++f) {
                    int arg = 0;
                    for (int fy = 0; fy < filter_h_size; ++fy) {
                        int const iy = oy * filter_h_size + fy;
                        if (iy >= input_h_size) { continue; }
                        for (int fx = 0; fx < filter_w_size; ++fx) {
                            int const ix = ox * filter_w_size + fx;
                            if (ix >= input_w_size) { continue; }
                            dx[(((long long)c * input_h_size + iy) * input_w_size + ix) * frame_stride + f] = (arg == argmax[out + f]) ? dy[out + f] : 0.0f;
                            ++arg;
                        }
                    }
                }
            }
        }
    }
}

/* y rows are frame_stride words; the caller clears them */
void oracle_bit_MaxPooling_Forward(int const *x, int *y, int filter_h_size, int filter_w_size, int input_w_size, int input_h_size,
                                   int output_w_size, int output_h_size, int c_size, int frame_size, int frame_stride)
{
    for (int c = 0; c < c_size; ++c) {
        for (int oy = 0; oy < output_h_size; ++oy) {
            for (int ox = 0; ox < output_w_size; ++ox) {
                int *yr = y + (((long long)c * output_h_size + oy) * output_w_size + ox) * frame_stride;
                for (int f = 0; f < frame_size; ++f) {
                    int any = 0;
                    for (int fy = 0; fy < filter_h_size; ++fy) {
                        int const iy = oy * filter_h_size + fy;
                        if (iy >= input_h_size) { continue; }
                        for (int fx = 0; fx < filter_w_size; ++fx) {
                            int const ix = ox * filter_w_size + fx;
                            if (ix >= input_w_size) { continue; }
                            any |= get_bit(x + (((long long)c * input_h_size + iy) * input_w_size + ix) * frame_stride, f);
                        }
                    }
                    set_bit(yr, f, any);
                }
            }
        }
    }
}

void oracle_bit_fp32_MaxPooling_Backward(int const *x, float const *dy, float *dx, int filter_h_size, int filter_w_size, int input_w_size,
                                         int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size,
                                         int forward_frame_stride, int backward_frame_stride)
{
    for (int c = 0; c < c_size; ++c) {
        for (int oy = 0; oy < output_h_size; ++oy) {
            for (int ox = 0; ox < output_w_size; ++ox) {
                long long const out = (((long long)c * output_h_size + oy) * output_w_size + ox) * backward_frame_stride;
                for (int f = 0; f < frame_size; ++f) {
                    float grad = dy[out + f];
                    for (int fy = 0; fy < filter_h_size; ++fy) {
                        int const iy = oy * filter_h_size + fy;
                        if (iy >= input_h_size) { continue; }
                        for (int fx = 0; fx < filter_w_size; ++fx) {
                            int const ix = ox * filter_w_size + fx;
                            if (ix >= input_w_size) { continue; }
                            long long const in_node = ((long long)c * input_h_size + iy) * input_w_size + ix;
                            int const sig = get_bit(x + in_node * forward_frame_stride, f);
                            dx[in_node * backward_frame_stride + f] = sig ? grad : 0.0f;
                            if (sig) { grad = 0.0f; }
                        }
                    }
                }
            }
        }
    }
}

void oracle_fp32_UpSampling_Forward(float const *x, float *y, int input_w_size, int input_h_size, int c_size, int filter_w_size,
                                    int filter_h_size, int fill, int frame_size, int frame_stride)
{
    int const output_h_size = input_h_size * filter_h_size, output_w_size = input_w_size * filter_w_size;
    for (int c = 0; c < c_size; ++c) {
        for (int iy = 0; iy < input_h_size; ++iy) {
            for (int ix = 0; ix < input_w_size; ++ix) {
                long long const in_node = ((long long)c * input_h_size + iy) * input_w_size + ix;
                for (int f = 0; f < frame_size; ++f) {
                    float const v = x[in_node * frame_stride + f];
                    for (int fy = 0; fy < filter_h_size; ++fy) {
                        for (int fx = 0; fx < filter_w_size; ++fx) {
                            long long const out_node = ((long long)c * output_h_size + iy * filter_h_size + fy) * output_w_size + ix * filter_w_size + fx;
                            int const centre = (fx == filter_w_size / 2 && fy == filter_h_size / 2);
                            y[out_node * frame_stride + f] = (fill || centre) ? v : 0.0f;
                        }
                    }
                }
            }
        }
    }
}

/* y rows are frame_stride words; the caller clears them */
void oracle_bit_UpSampling_Forward(int const *x, int *y, int input_w_size, int input_h_size, int c_size, int filter_w_size,
                                   int filter_h_size, int fill, int frame_size, int frame_stride)
{
    int const output_h_size = input_h_size * filter_h_size, output_w_size = input_w_size * filter_w_size;
    for (int c = 0; c < c_size; ++c) {
        for (int iy = 0; iy < input_h_size; ++iy) {
            for (int ix = 0; ix < input_w_size; ++ix) {
                long long const in_node = ((long long)c * input_h_size + iy) * input_w_size + ix;
                for (int f = 0; f < frame_size; ++f) {
                    int const v = get_bit(x + in_node * frame_stride, f);
                    for (int fy = 0; fy < filter_h_size; ++fy) {
                        for (int fx = 0; fx < filter_w_size; ++fx) {
                            long long const out_node = ((long long)c * output_h_size + iy * filter_h_size + fy) * output_w_size + ix * filter_w_size + fx;
                            int const centre = (fx == filter_w_size / 2 && fy == filter_h_size / 2);
                            set_bit(y + out_node * frame_stride, f, (fill || centre) ? v : 0);
                        }
                    }
                }
            }
        }
    }
}

void oracle_fp32_UpSampling_Backward(float const *dy, float *dx, int input_w_size, int input_h_size, int c_size, int filter_w_size,
                                     int filter_h_size, int fill, int frame_size, int frame_stride)
{
    int const output_h_size = input_h_size * filter_h_size, output_w_size = input_w_size * filter_w_size;
    for (int c = 0; c < c_size; ++c) {
        for (int iy = 0; iy < input_h_size; ++iy) {
            for (int ix = 0; ix < input_w_size; ++ix) {
                long long const in_node = ((long long)c * input_h_size + iy) * input_w_size + ix;
                for (int f = 0; f < frame_size; ++f) {
                    float sum = 0;
                    for (int fy = 0; fy < filter_h_size; ++fy) {
                        for (int fx = 0; fx < filter_w_size; ++fx) {
                            long long const out_node = ((long long)c * output_h_size + iy * filter_h_size + fy) * output_w_size + ix * filter_w_size + fx;
                            int const centre = (fx == filter_w_size / 2 && fy == filter_h_size / 2);
                            if (fill || centre) { sum += dy[out_node * frame_stride + f]; }
                        }
                    }
                    dx[in_node * frame_stride + f] = sum;
                }
            }
        }
    }
}

/* ------------------------------------------------------------------------------------------------------------------------------------
 *  Shuffle (include/bb/Shuffle.h:166-185, :225-243): a permutation of whole rows, whatever their element type.  With
 *  x_unit_size = node_size / y_unit_size, output row i * y_unit_size + j is input row j * x_unit_size + i; backward undoes it.
 *  Rows are frame_stride 32-bit words and are copied whole, as the reference's memcpy of one stride does.
 * ---------------------------------------------------------------------------------------------------------------------------------- */
void oracle_Shuffle_Forward(int const *x, int *y, int y_unit_size, int node_size, int frame_stride)
{
    int const x_unit_size = node_size / y_unit_size;
    for (int i = 0; i < x_unit_size; ++i) {
        for (int j = 0; j < y_unit_size; ++j) {
            memcpy(y + (size_t)(i * y_unit_size + j) * frame_stride, x + (size_t)(j * x_unit_size + i) * frame_stride, (size_t)frame_stride * sizeof(int));
        }
    }
}

void oracle_Shuffle_Backward(int const *dy, int *dx, int y_unit_size, int node_size, int frame_stride)
{
    int const x_unit_size = node_size / y_unit_size;
    for (int i = 0; i < y_unit_size; ++i) {
        for (int j = 0; j < x_unit_size; ++j) {
            memcpy(dx + (size_t)(i * x_unit_size + j) * frame_stride, dy + (size_t)(j * y_unit_size + i) * frame_stride, (size_t)frame_stride * sizeof(int));
        }
    }
}

// TEST INFRASTRUCTURE — not part of the shipped library.
//
// Thin extern "C" harness around the *unmodified* BinaryBrain CPU headers
// (compiled with -I/root/reference/include, no BB_WITH_CUDA).  It lets the
// parity tests and the CPU-baseline leg of bench.py run the reference's own
// host implementation of the three LUT layers on caller-provided dense
// arrays.  Every array is node-major, frame-minor: element (node n, frame f)
// of an fp32 buffer is p[n*frames + f]; bit buffers are rows of `words`
// 32-bit words per node, frame f at word f>>5 bit f&31 (the reference's own
// packing, include/bb/DataType.h:612-647).
//
// Built only where the reference tree is present; see oracle/Makefile.

#include <chrono>
#include <cstring>
#include <cstdint>
#include <vector>
#include <string>
#include <sstream>

#include "bb/StochasticLutN.h"
#include "bb/DifferentiableLutN.h"
#include "bb/BinaryLutN.h"
#include "bb/FixedSizeConnectionTable.h"
#include "bb/OptimizerAdam.h"
#include "bb/ConvolutionIm2Col.h"
#include "bb/ConvolutionCol2Im.h"
#include "bb/StochasticMaxPooling2x2.h"
#include "bb/TensorOperator.h"
#include "bb/AverageLut.h"
#include "bb/MaxLut.h"
#include "bb/Reduce.h"
#include "bb/LossMeanSquaredError.h"
#include "bb/MetricsMeanSquaredError.h"
#include "bb/LossSoftmaxCrossEntropy.h"
#include "bb/MetricsCategoricalAccuracy.h"
#include "bb/Convolution2d.h"
#include "bb/Sequential.h"
#include "bb/StochasticBatchNormalization.h"
#include "bb/RealToBinary.h"
#include "bb/BinaryToReal.h"
#include "bb/Binarize.h"
#include "bb/HardTanh.h"
#include "bb/BinaryModulation.h"
#include "bb/DifferentiableLutDiscreteN.h"
#include "bb/MaxPooling.h"
#include "bb/UpSampling.h"
#include "bb/Shuffle.h"

namespace {

using bb::index_t;

void put_fp32(bb::FrameBuffer &buf, float const *src, index_t nodes, index_t frames)
{
    auto ptr = buf.Lock<float>(true);
    index_t stride = buf.GetFrameStride() / (index_t)sizeof(float);
    for (index_t n = 0; n < nodes; ++n) {
        float *row = ptr.GetAddr(n);
        std::memcpy(row, src + n * frames, sizeof(float) * (size_t)frames);
        for (index_t f = frames; f < stride; ++f) { row[f] = 0.0f; }
    }
}

void get_fp32(bb::FrameBuffer &buf, float *dst, index_t nodes, index_t frames)
{
    auto ptr = buf.LockConst<float>();
    for (index_t n = 0; n < nodes; ++n) {
        std::memcpy(dst + n * frames, ptr.GetAddr(n), sizeof(float) * (size_t)frames);
    }
}

void put_bit(bb::FrameBuffer &buf, std::int32_t const *src, index_t nodes, index_t words)
{
    auto ptr = buf.Lock<bb::Bit>(true);
    index_t stride_bytes = buf.GetFrameStride();
    for (index_t n = 0; n < nodes; ++n) {
        auto *row = (std::uint8_t *)ptr.GetAddr(n);
        std::memset(row, 0, (size_t)stride_bytes);
        index_t nbytes = std::min(stride_bytes, words * 4);
        std::memcpy(row, src + n * words, (size_t)nbytes);
    }
}

void get_bit(bb::FrameBuffer &buf, std::int32_t *dst, index_t nodes, index_t words)
{
    auto ptr = buf.LockConst<bb::Bit>();
    index_t stride_bytes = buf.GetFrameStride();
    for (index_t n = 0; n < nodes; ++n) {
        auto const *row = (std::uint8_t const *)ptr.GetAddr(n);
        std::memset(dst + n * words, 0, (size_t)words * 4);
        index_t nbytes = std::min(stride_bytes, words * 4);
        std::memcpy(dst + n * words, row, (size_t)nbytes);
    }
}

std::string onoff(int v) { return v ? "true" : "false"; }

template <int N, typename BinType>
int run_stochastic(int I, int O, int F, void const *x, std::int32_t const *idx, float *W,
                   float const *dy, float *y, float *dx, float *dW,
                   int binary_mode, int lut_binarize, int host_simd)
{
    auto lut = bb::StochasticLutN<N, BinType, float>::Create((index_t)O);
    lut->SendCommand("host_only true");
    lut->SendCommand("host_simd " + onoff(host_simd));
    lut->SendCommand("lut_binarize " + onoff(lut_binarize));
    lut->SendCommand("binary " + onoff(binary_mode));

    int const xtype = bb::DataType<BinType>::type;
    bb::FrameBuffer x_buf((index_t)F, {(index_t)I}, xtype, true);
    lut->SetInputShape(x_buf.GetShape());
    for (int n = 0; n < O; ++n) {
        for (int i = 0; i < N; ++i) { lut->SetNodeConnectionIndex(n, i, idx[n * N + i]); }
    }
    {
        auto Wp = lut->lock_W();
        for (int n = 0; n < O; ++n) for (int i = 0; i < (1 << N); ++i) { Wp(n, i) = W[n * (1 << N) + i]; }
    }
    if (dW) {
        auto dWp = lut->lock_dW();
        for (int n = 0; n < O; ++n) for (int i = 0; i < (1 << N); ++i) { dWp(n, i) = dW[n * (1 << N) + i]; }
    }
    if (xtype == BB_TYPE_BIT) { put_bit(x_buf, (std::int32_t const *)x, I, (F + 31) / 32); }
    else                      { put_fp32(x_buf, (float const *)x, I, F); }

    auto y_buf = lut->Forward(x_buf, dy != nullptr);
    get_fp32(y_buf, y, O, F);
    {
        auto Wp = lut->lock_W_const();
        for (int n = 0; n < O; ++n) for (int i = 0; i < (1 << N); ++i) { W[n * (1 << N) + i] = Wp(n, i); }
    }
    if (dy) {
        bb::FrameBuffer dy_buf((index_t)F, {(index_t)O}, BB_TYPE_FP32, true);
        put_fp32(dy_buf, dy, O, F);
        auto dx_buf = lut->Backward(dy_buf);
        get_fp32(dx_buf, dx, I, F);
        auto dWp = lut->lock_dW_const();
        for (int n = 0; n < O; ++n) for (int i = 0; i < (1 << N); ++i) { dW[n * (1 << N) + i] = dWp(n, i); }
    }
    return 0;
}

template <int N, typename BinType>
int run_differentiable(int I, int O, int F, void const *x, std::int32_t const *idx, float *W,
                       float const *dy, void *y, float *dx, float *dW,
                       float *mean, float *rstd, float *running_mean, float *running_var,
                       float gamma, float beta, float momentum,
                       int batch_norm, int binary_mode, int lut_binarize, int train)
{
    typename bb::DifferentiableLutN<N, BinType, float>::create_t cr;
    cr.output_shape = {(index_t)O};
    cr.batch_norm   = batch_norm != 0;
    cr.binary       = binary_mode != 0;
    cr.momentum     = momentum;
    cr.gamma        = gamma;
    cr.beta         = beta;
    auto lut = bb::DifferentiableLutN<N, BinType, float>::Create(cr);
    lut->SendCommand("host_only true");
    lut->SendCommand("lut_binarize " + onoff(lut_binarize));

    int const xtype = bb::DataType<BinType>::type;
    bb::FrameBuffer x_buf((index_t)F, {(index_t)I}, xtype, true);
    lut->SetInputShape(x_buf.GetShape());
    for (int n = 0; n < O; ++n) {
        for (int i = 0; i < N; ++i) { lut->SetNodeConnectionIndex(n, i, idx[n * N + i]); }
    }
    {
        auto Wp = lut->lock_W();
        for (int n = 0; n < O; ++n) for (int i = 0; i < (1 << N); ++i) { Wp(n, i) = W[n * (1 << N) + i]; }
    }
    if (dW) {
        auto dWp = lut->lock_dW();
        for (int n = 0; n < O; ++n) for (int i = 0; i < (1 << N); ++i) { dWp(n, i) = dW[n * (1 << N) + i]; }
    }
    {
        auto rm = lut->lock_mean();
        auto rv = lut->lock_var();
        for (int n = 0; n < O; ++n) { rm[n] = running_mean[n]; rv[n] = running_var[n]; }
    }
    if (xtype == BB_TYPE_BIT) { put_bit(x_buf, (std::int32_t const *)x, I, (F + 31) / 32); }
    else                      { put_fp32(x_buf, (float const *)x, I, F); }

    auto y_buf = lut->Forward(x_buf, train != 0);
    if (xtype == BB_TYPE_BIT) { get_bit(y_buf, (std::int32_t *)y, O, (F + 31) / 32); }
    else                      { get_fp32(y_buf, (float *)y, O, F); }
    {
        auto rm = lut->lock_mean_const();
        auto rv = lut->lock_var_const();
        for (int n = 0; n < O; ++n) { running_mean[n] = rm[n]; running_var[n] = rv[n]; }
    }
    if (batch_norm && train) {
        auto tm = lut->lock_tmp_mean_const();
        auto tr = lut->lock_tmp_rstd_const();
        for (int n = 0; n < O; ++n) { mean[n] = tm[n]; rstd[n] = tr[n]; }
    }
    if (dy) {
        bb::FrameBuffer dy_buf((index_t)F, {(index_t)O}, BB_TYPE_FP32, true);
        put_fp32(dy_buf, dy, O, F);
        auto dx_buf = lut->Backward(dy_buf);
        get_fp32(dx_buf, dx, I, F);
        auto dWp = lut->lock_dW_const();
        for (int n = 0; n < O; ++n) for (int i = 0; i < (1 << N); ++i) { dW[n * (1 << N) + i] = dWp(n, i); }
    }
    return 0;
}

}  // namespace


// BinaryLutN<N,Bit>::Forward for any width N = 2 .. 6 (host path; N = 6 with its AVX2 loop); table [O][(2^N + 31) / 32] words
template <int N>
static int binary_lut_n(int I, int O, int F, std::int32_t const *x, std::int32_t const *idx, std::int32_t const *table, std::int32_t *y)
{
    auto lut = bb::BinaryLutN<N, bb::Bit, float>::Create((index_t)O);
    lut->SendCommand("host_only true");
    bb::FrameBuffer x_buf((index_t)F, {(index_t)I}, BB_TYPE_BIT, true);
    lut->SetInputShape(x_buf.GetShape());
    int const unit = ((1 << N) + 31) / 32;
    for (int nd = 0; nd < O; ++nd) {
        for (int i = 0; i < N; ++i) { lut->SetNodeConnectionIndex(nd, i, idx[nd * N + i]); }
        for (int b = 0; b < (1 << N); ++b) { lut->SetLutTable(nd, b, ((table[nd * unit + (b >> 5)] >> (b & 31)) & 1) != 0); }
    }
    put_bit(x_buf, x, I, (F + 31) / 32);
    auto y_buf = lut->Forward(x_buf, false);
    get_bit(y_buf, y, O, (F + 31) / 32);
    return 0;
}

extern "C" {

// StochasticLutN<N,float|Bit,float>::Forward (+Backward when dy != NULL) on the host-only path.
// W is clamped in place exactly as Forward does (include/bb/StochasticLutN.h:451).
int bbref_StochasticLut(int n, int bit_input, int I, int O, int F,
                        void const *x, std::int32_t const *idx, float *W,
                        float const *dy, float *y, float *dx, float *dW,
                        int binary_mode, int lut_binarize, int host_simd)
{
#define BBREF_CASE(NN) \
    case NN: return bit_input ? run_stochastic<NN, bb::Bit>(I, O, F, x, idx, W, dy, y, dx, dW, binary_mode, lut_binarize, host_simd) \
                              : run_stochastic<NN, float  >(I, O, F, x, idx, W, dy, y, dx, dW, binary_mode, lut_binarize, host_simd);
    switch (n) { BBREF_CASE(2) BBREF_CASE(3) BBREF_CASE(4) BBREF_CASE(5) BBREF_CASE(6) default: return -1; }
#undef BBREF_CASE
}

// Times StochasticLutN<6,float>::Forward + Backward (AVX2/OpenMP host path) on caller data: one warm-up, then
// `reps` repetitions timed with steady_clock around Forward+Backward only; seconds[r] receives each repetition.
int bbref_StochasticLut6_Time(int I, int O, int F, float const *x, std::int32_t const *idx, float const *W,
                              float const *dy, int lut_binarize, int reps, double *seconds)
{
    auto lut = bb::StochasticLutN<6, float, float>::Create((index_t)O);
    lut->SendCommand("host_only true");
    lut->SendCommand("lut_binarize " + onoff(lut_binarize));
    bb::FrameBuffer x_buf((index_t)F, {(index_t)I}, BB_TYPE_FP32, true);
    lut->SetInputShape(x_buf.GetShape());
    for (int n = 0; n < O; ++n) for (int i = 0; i < 6; ++i) { lut->SetNodeConnectionIndex(n, i, idx[n * 6 + i]); }
    {
        auto Wp = lut->lock_W();
        for (int n = 0; n < O; ++n) for (int i = 0; i < 64; ++i) { Wp(n, i) = W[n * 64 + i]; }
    }
    put_fp32(x_buf, x, I, F);
    bb::FrameBuffer dy_buf((index_t)F, {(index_t)O}, BB_TYPE_FP32, true);
    put_fp32(dy_buf, dy, O, F);
    for (int r = -1; r < reps; ++r) {
        auto t0 = std::chrono::steady_clock::now();
        auto y_buf  = lut->Forward(x_buf, true);
        auto dx_buf = lut->Backward(dy_buf);
        auto t1 = std::chrono::steady_clock::now();
        if (r >= 0) { seconds[r] = std::chrono::duration<double>(t1 - t0).count(); }
    }
    return 0;
}

// DifferentiableLutN<N,float|Bit,float>::Forward (+Backward when dy != NULL), host-only generic path.
int bbref_DifferentiableLut(int n, int bit_input, int I, int O, int F,
                            void const *x, std::int32_t const *idx, float *W,
                            float const *dy, void *y, float *dx, float *dW,
                            float *mean, float *rstd, float *running_mean, float *running_var,
                            float gamma, float beta, float momentum,
                            int batch_norm, int binary_mode, int lut_binarize, int train)
{
#define BBREF_CASE(NN) \
    case NN: return bit_input ? run_differentiable<NN, bb::Bit>(I, O, F, x, idx, W, dy, y, dx, dW, mean, rstd, running_mean, running_var, gamma, beta, momentum, batch_norm, binary_mode, lut_binarize, train) \
                              : run_differentiable<NN, float  >(I, O, F, x, idx, W, dy, y, dx, dW, mean, rstd, running_mean, running_var, gamma, beta, momentum, batch_norm, binary_mode, lut_binarize, train);
    switch (n) { BBREF_CASE(2) BBREF_CASE(4) BBREF_CASE(6) default: return -1; }
#undef BBREF_CASE
}

// BinaryLutN<6,Bit>::Forward, host-only; host_simd selects the AVX2 or the generic loop.
int bbref_BinaryLut6(int I, int O, int F, std::int32_t const *x, std::int32_t const *idx,
                     std::int32_t const *table /*[O][2]*/, std::int32_t *y, int host_simd)
{
    auto lut = bb::BinaryLutN<6, bb::Bit, float>::Create((index_t)O);
    lut->SendCommand("host_only true");
    lut->SendCommand("host_simd " + onoff(host_simd));
    bb::FrameBuffer x_buf((index_t)F, {(index_t)I}, BB_TYPE_BIT, true);
    lut->SetInputShape(x_buf.GetShape());
    for (int nd = 0; nd < O; ++nd) {
        for (int i = 0; i < 6; ++i) { lut->SetNodeConnectionIndex(nd, i, idx[nd * 6 + i]); }
        for (int b = 0; b < 64; ++b) { lut->SetLutTable(nd, b, ((table[nd * 2 + (b >> 5)] >> (b & 31)) & 1) != 0); }
    }
    put_bit(x_buf, x, I, (F + 31) / 32);
    auto y_buf = lut->Forward(x_buf, false);
    get_bit(y_buf, y, O, (F + 31) / 32);
    return 0;
}

int bbref_BinaryLutN(int n, int I, int O, int F, std::int32_t const *x, std::int32_t const *idx, std::int32_t const *table, std::int32_t *y)
{
    switch (n) {
    case 2: return binary_lut_n<2>(I, O, F, x, idx, table, y);
    case 3: return binary_lut_n<3>(I, O, F, x, idx, table, y);
    case 4: return binary_lut_n<4>(I, O, F, x, idx, table, y);
    case 5: return binary_lut_n<5>(I, O, F, x, idx, table, y);
    case 6: return binary_lut_n<6>(I, O, F, x, idx, table, y);
    }
    return 1;
}

// FixedSizeConnectionTable<6>: reverse table for a given input table.
// Returns the row stride (1 + max fan-out); fills rev (capacity rev_cap int32) when it fits.
int bbref_ReverseTable6(int I, int O, std::int32_t const *idx, std::int32_t *rev, int rev_cap)
{
    bb::FixedSizeConnectionTable<6> tbl;
    tbl.SetShape({(index_t)I}, {(index_t)O});
    for (int nd = 0; nd < O; ++nd) for (int i = 0; i < 6; ++i) { tbl.SetInputConnection(nd, i, idx[nd * 6 + i]); }
    auto ptr = tbl.LockConst_ReverseTable();
    int stride = (int)tbl.GetReverseTableStride();
    if ((long long)stride * I <= rev_cap) {
        for (int r = 0; r < I; ++r) for (int c = 0; c < stride; ++c) { rev[r * stride + c] = ptr(r, c); }
    }
    return stride;
}

// Seeded default wiring of StochasticLutN<6>::SetInputShape (random ShuffleSet policy) — used only
// to check that injected wiring satisfies the same invariants (distinct inputs per node).
int bbref_DefaultWiring6(int I, int O, std::uint64_t seed, std::int32_t *idx)
{
    auto lut = bb::StochasticLutN<6, float, float>::Create((index_t)O, "", seed);
    lut->SendCommand("host_only true");
    lut->SetInputShape({(index_t)I});
    for (int nd = 0; nd < O; ++nd) for (int i = 0; i < 6; ++i) { idx[nd * 6 + i] = (std::int32_t)lut->GetNodeConnectionIndex(nd, i); }
    return 0;
}


// Seeded wiring by policy.  kind 0: FixedSizeConnectionTable<6>::InitializeConnection(seed, policy) (the table behind
// StochasticLutN / DifferentiableLutN, include/bb/ConnectionTable.h:150-284); kind 1: BinaryLutN<6, Bit> created with
// (output_shape, policy, seed) and given its input shape, which draws the wiring seed and then the table seed from the
// layer's generator (include/bb/BinaryLutN.h:201-218, SparseModel.h:97-233, BinaryLutModel.h:45-59) — `table` then
// receives the layer's random truth tables, int32 [O][2].  Shapes have `dims` entries.  idx: int32 [O][6].
int bbref_Wiring6(int kind, int dims, long long const *in_shape, long long const *out_shape, std::uint64_t seed, char const *policy,
                  std::int32_t *idx, std::int32_t *table)
{
    bb::indices_t in((size_t)dims), out((size_t)dims);
    for (int i = 0; i < dims; ++i) { in[(size_t)i] = (index_t)in_shape[i]; out[(size_t)i] = (index_t)out_shape[i]; }
    index_t const O = bb::CalcShapeSize(out);
    if (kind == 0) {
        bb::FixedSizeConnectionTable<6> tbl;
        tbl.SetShape(in, out);
        tbl.InitializeConnection(seed, policy);
        for (index_t nd = 0; nd < O; ++nd) for (int i = 0; i < 6; ++i) { idx[nd * 6 + i] = (std::int32_t)tbl.GetInputConnection(nd, i); }
        return 0;
    }
    typename bb::BinaryLutN<6, bb::Bit>::create_t create;
    create.output_shape = out;
    create.connection   = policy;
    create.seed         = seed;
    auto lut = bb::BinaryLutN<6, bb::Bit>::Create(create);
    lut->SetInputShape(in);
    for (index_t nd = 0; nd < O; ++nd) {
        for (int i = 0; i < 6; ++i) { idx[nd * 6 + i] = (std::int32_t)lut->GetNodeConnectionIndex(nd, i); }
        std::uint32_t w[2] = {0, 0};
        for (int b = 0; b < 64; ++b) { if (lut->GetLutTable(nd, b)) { w[b / 32] |= (1u << (b % 32)); } }
        table[nd * 2] = (std::int32_t)w[0]; table[nd * 2 + 1] = (std::int32_t)w[1];
    }
    return 0;
}


// bb::OptimizerAdam<float> (host path, include/bb/OptimizerAdam.h:142-180): `steps` updates of one fp32 tensor of
// `size` elements; grads is [steps][size]; param is updated in place.
int bbref_OptimizerAdam(int size, int steps, float *param, float const *grads, float learning_rate, float beta1, float beta2)
{
    auto opt = bb::OptimizerAdam<float>::Create(learning_rate, beta1, beta2);
    auto p = std::shared_ptr<bb::Tensor>(new bb::Tensor(bb::indices_t({(bb::index_t)size}), BB_TYPE_FP32, true));
    auto g = std::shared_ptr<bb::Tensor>(new bb::Tensor(bb::indices_t({(bb::index_t)size}), BB_TYPE_FP32, true));
    bb::Variables pv, gv;
    pv.PushBack(p);
    gv.PushBack(g);
    opt->SetVariables(pv, gv);
    { auto ptr = p->Lock<float>(); for (int i = 0; i < size; ++i) { ptr(i) = param[i]; } }
    for (int s = 0; s < steps; ++s) {
        { auto ptr = g->Lock<float>(); for (int i = 0; i < size; ++i) { ptr(i) = grads[(size_t)s * size + i]; } }
        opt->Update();
    }
    { auto ptr = p->LockConst<float>(); for (int i = 0; i < size; ++i) { param[i] = ptr(i); } }
    return 0;
}

// The reference's elementwise kernels of its Tensor arithmetic, host versions (include/bb/TensorOperator.h:41-238).
// op: 0 add_ex, 1 mul_ex, 2 div_ex, 3 sqrt, 4 exp, 5 min, 6 min_v, 7 max, 8 max_v
int bbref_Vector_op(int op, float *dst, float const *src0, float const *src1, float a, float b, float c, float d, int size)
{
    bb::index_t const n = size;
    switch (op) {
    case 0: bb::Tensor_Vector_add_ex<float>(dst, src0, src1, a, b, c, n); return 0;
    case 1: bb::Tensor_Vector_mul_ex<float>(dst, src0, src1, a, b, n); return 0;
    case 2: bb::Tensor_Vector_div_ex<float>(dst, src0, src1, a, b, c, d, n); return 0;
    case 3: bb::Tensor_Vector_sqrt<float>(dst, src0, n); return 0;
    case 4: bb::Tensor_Vector_exp<float>(dst, src0, n); return 0;
    case 5: bb::Tensor_Vector_min<float>(dst, src0, src1, n); return 0;
    case 6: bb::Tensor_Vector_min_v<float>(dst, src0, a, n); return 0;
    case 7: bb::Tensor_Vector_max<float>(dst, src0, src1, n); return 0;
    case 8: bb::Tensor_Vector_max_v<float>(dst, src0, a, n); return 0;
    }
    return -1;
}


}  // extern "C"

// ConvolutionIm2Col<float|Bit, float> (host path).  x: [c*h*w][frames] dense (fp32) or [c*h*w][words] (bits);
// y: [c*fh*fw][frames*oh*ow]; when dy != NULL (fp32 only) Backward is run and dx [c*h*w][frames] is returned.
// out_hw receives {oh, ow}.
template <typename FT>
static int run_im2col(int c, int h, int w, int frames, int fh, int fw, int ys, int xs, char const *padding, char const *border,
                      void const *x, void *y, float const *dy, float *dx, int *out_hw)
{
    auto m = bb::ConvolutionIm2Col<FT, float>::Create(fh, fw, ys, xs, padding, border);
    m->SendCommand("host_only true");
    bb::indices_t shape({(index_t)c, (index_t)h, (index_t)w});
    bb::FrameBuffer xb(frames, shape, bb::DataType<FT>::type, true);
    index_t const in_nodes = (index_t)c * h * w;
    if (std::is_same<FT, bb::Bit>::value) { put_bit(xb, (std::int32_t const *)x, in_nodes, (frames + 31) / 32); }
    else                                   { put_fp32(xb, (float const *)x, in_nodes, frames); }
    bb::FrameBuffer yb = m->Forward(xb, true);
    index_t const out_nodes = (index_t)c * fh * fw;
    index_t const out_frames = yb.GetFrameSize();
    index_t const o = out_frames / frames;            // oh * ow
    (void)o;
    if (std::is_same<FT, bb::Bit>::value) { get_bit(yb, (std::int32_t *)y, out_nodes, (out_frames + 31) / 32); }
    else                                   { get_fp32(yb, (float *)y, out_nodes, out_frames); }
    if (dy) {
        bb::FrameBuffer dyb(out_frames, bb::indices_t({(index_t)c, (index_t)fh, (index_t)fw}), BB_TYPE_FP32, true);
        put_fp32(dyb, dy, out_nodes, out_frames);
        bb::FrameBuffer dxb = m->Backward(dyb);
        get_fp32(dxb, dx, in_nodes, frames);
    }
    if (out_hw) {
        std::string pad(padding);
        out_hw[0] = pad == "same" ? (h + ys - 1) / ys : ((h - fh + 1) + (ys - 1)) / ys;
        out_hw[1] = pad == "same" ? (w + xs - 1) / xs : ((w - fw + 1) + (xs - 1)) / xs;
    }
    return (int)out_frames;
}

extern "C" int bbref_Im2Col(int bit, int c, int h, int w, int frames, int fh, int fw, int ys, int xs, char const *padding, char const *border,
                 void const *x, void *y, float const *dy, float *dx, int *out_hw)
{
    return bit ? run_im2col<bb::Bit>(c, h, w, frames, fh, fw, ys, xs, padding, border, x, y, dy, dx, out_hw)
               : run_im2col<float>(c, h, w, frames, fh, fw, ys, xs, padding, border, x, y, dy, dx, out_hw);
}

// ConvolutionCol2Im<float|Bit, float> (host path).  x: [c][frames*h*w]; y: [c*h*w][frames]; dy/dx likewise (fp32).
template <typename FT>
static int run_col2im(int c, int h, int w, int frames, void const *x, void *y, float const *dy, float *dx)
{
    auto m = bb::ConvolutionCol2Im<FT, float>::Create(h, w);
    m->SendCommand("host_only true");
    m->SetInputShape(bb::indices_t({(index_t)c}));      // Forward does not derive the channel count itself
    index_t const in_frames = (index_t)frames * h * w;
    bb::FrameBuffer xb(in_frames, bb::indices_t({(index_t)c}), bb::DataType<FT>::type, true);
    if (std::is_same<FT, bb::Bit>::value) { put_bit(xb, (std::int32_t const *)x, c, (in_frames + 31) / 32); }
    else                                   { put_fp32(xb, (float const *)x, c, in_frames); }
    bb::FrameBuffer yb = m->Forward(xb, true);
    index_t const out_nodes = (index_t)c * h * w;
    if (std::is_same<FT, bb::Bit>::value) { get_bit(yb, (std::int32_t *)y, out_nodes, (frames + 31) / 32); }
    else                                   { get_fp32(yb, (float *)y, out_nodes, frames); }
    if (dy) {
        bb::FrameBuffer dyb(frames, bb::indices_t({(index_t)c, (index_t)h, (index_t)w}), BB_TYPE_FP32, true);
        put_fp32(dyb, dy, out_nodes, frames);
        bb::FrameBuffer dxb = m->Backward(dyb);
        get_fp32(dxb, dx, c, in_frames);
    }
    return 0;
}

extern "C" int bbref_Col2Im(int bit, int c, int h, int w, int frames, void const *x, void *y, float const *dy, float *dx)
{
    return bit ? run_col2im<bb::Bit>(c, h, w, frames, x, y, dy, dx) : run_col2im<float>(c, h, w, frames, x, y, dy, dx);
}

// StochasticMaxPooling2x2<float, float> (host path).  x: [c*h*w][frames]; y: [c*oh*ow][frames]
extern "C" int bbref_StochasticMaxPooling2x2(int c, int h, int w, int frames, float const *x, float *y, float const *dy, float *dx)
{
    auto m = bb::StochasticMaxPooling2x2<float, float>::Create();
    m->SendCommand("host_only true");
    bb::FrameBuffer xb(frames, bb::indices_t({(index_t)c, (index_t)h, (index_t)w}), BB_TYPE_FP32, true);
    put_fp32(xb, x, (index_t)c * h * w, frames);
    bb::FrameBuffer yb = m->Forward(xb, true);
    int const oh = (h + 1) / 2, ow = (w + 1) / 2;
    get_fp32(yb, y, (index_t)c * oh * ow, frames);
    if (dy) {
        bb::FrameBuffer dyb(frames, bb::indices_t({(index_t)c, (index_t)oh, (index_t)ow}), BB_TYPE_FP32, true);
        put_fp32(dyb, dy, (index_t)c * oh * ow, frames);
        bb::FrameBuffer dxb = m->Backward(dyb);
        get_fp32(dxb, dx, (index_t)c * h * w, frames);
    }
    return 0;
}

// AverageLut<BinType, float> (host path).  x: [I][frames] (fp32) or [I][words] (bits); y likewise for O nodes.
namespace {
template <typename BinType>
int run_average_lut(int n, int I, int O, int F, void const *x, std::int32_t const *idx, int binarize_input, int binarize_output,
                    void *y, float const *dy, float *dx)
{
    auto m = bb::AverageLut<BinType, float>::Create(n, bb::indices_t({(index_t)O}));
    m->SendCommand("host_only true");
    m->SendCommand("binarize_input " + onoff(binarize_input));
    m->SendCommand("binarize_output " + onoff(binarize_output));
    int const xtype = bb::DataType<BinType>::type;
    bb::FrameBuffer xb((index_t)F, bb::indices_t({(index_t)I}), xtype, true);
    m->SetInputShape(xb.GetShape());
    for (int o = 0; o < O; ++o) { for (int i = 0; i < n; ++i) { m->SetNodeConnectionIndex(o, i, idx[o * n + i]); } }
    if (xtype == BB_TYPE_BIT) { put_bit(xb, (std::int32_t const *)x, I, (F + 31) / 32); }
    else                      { put_fp32(xb, (float const *)x, I, F); }
    bb::FrameBuffer yb = m->Forward(xb, true);
    if (xtype == BB_TYPE_BIT) { get_bit(yb, (std::int32_t *)y, O, (F + 31) / 32); }
    else                      { get_fp32(yb, (float *)y, O, F); }
    if (dy) {
        bb::FrameBuffer dyb((index_t)F, bb::indices_t({(index_t)O}), BB_TYPE_FP32, true);
        put_fp32(dyb, dy, O, F);
        bb::FrameBuffer dxb = m->Backward(dyb);
        get_fp32(dxb, dx, I, F);
    }
    return 0;
}
}  // namespace

extern "C" int bbref_AverageLut(int bit, int n, int I, int O, int F, void const *x, std::int32_t const *idx, int binarize_input,
                                int binarize_output, void *y, float const *dy, float *dx)
{
    return bit ? run_average_lut<bb::Bit>(n, I, O, F, x, idx, binarize_input, binarize_output, y, dy, dx)
               : run_average_lut<float>(n, I, O, F, x, idx, binarize_input, binarize_output, y, dy, dx);
}

// LossSoftmaxCrossEntropy<float> and MetricsCategoricalAccuracy<float> (host paths) on [ch][pix] nodes.
// loss = GetLoss(), metric = GetMetrics() after one batch.
extern "C" int bbref_LossAndAccuracy(int ch, int pix, int F, float const *y, float const *t, float *dy, double *loss, double *metric)
{
    bb::indices_t const shape({(index_t)ch, (index_t)pix});
    bb::FrameBuffer yb((index_t)F, shape, BB_TYPE_FP32, true), tb((index_t)F, shape, BB_TYPE_FP32, true);
    put_fp32(yb, y, (index_t)ch * pix, F);
    put_fp32(tb, t, (index_t)ch * pix, F);
    auto lossFunc = bb::LossSoftmaxCrossEntropy<float>::Create();
    lossFunc->Clear();
    bb::FrameBuffer dyb = lossFunc->CalculateLoss(yb, tb, (index_t)F);
    get_fp32(dyb, dy, (index_t)ch * pix, F);
    *loss = lossFunc->GetLoss();
    auto metrics = bb::MetricsCategoricalAccuracy<float>::Create();
    metrics->Clear();
    metrics->CalculateMetrics(yb, tb);
    *metric = metrics->GetMetrics();
    return 0;
}

// ---------------------------------------------------------------------------------------------------------------------
// Object serialization of the three LUT layers (Object::DumpObject / LoadObject): a layer with the given wiring and
// parameters is built through the reference's API and written to bytes, or read back from bytes and taken apart.
// kind 0 = StochasticLutN<6>, 1 = DifferentiableLutN<6>, 2 = BinaryLutN<6, Bit, float>; bit selects BinType = Bit for
// kinds 0 and 1.  flags: bit 0 = binary, bit 1 = lut_binarize, bit 2 = batch_norm.  scalars = {momentum, gamma, beta}.
// params: W [O][64] fp32 (kinds 0, 1) or the truth table [O][2] int32 (kind 2).
// ---------------------------------------------------------------------------------------------------------------------
namespace {

template <class M>
void put_wiring(M &m, int O, std::int32_t const *idx)
{
    for (int o = 0; o < O; ++o) { for (int i = 0; i < 6; ++i) { m.SetNodeConnectionIndex(o, i, idx[o * 6 + i]); } }
}
template <class M>
void get_wiring(M const &m, int O, std::int32_t *idx)
{
    for (int o = 0; o < O; ++o) { for (int i = 0; i < 6; ++i) { idx[o * 6 + i] = (std::int32_t)m.GetNodeConnectionIndex(o, i); } }
}
long emit(bb::Object const &obj, unsigned char *out, long cap)
{
    std::ostringstream os(std::ios::binary);
    obj.DumpObject(os);
    std::string const bytes = os.str();
    if ((long)bytes.size() > cap) { return -(long)bytes.size(); }
    std::memcpy(out, bytes.data(), bytes.size());
    return (long)bytes.size();
}

template <typename BinType>
long dump_stochastic(int I, int O, std::int32_t const *idx, float const *W, int flags, char const *name, unsigned char *out, long cap)
{
    auto m = bb::StochasticLutN<6, BinType, float>::Create((index_t)O);
    if (name && *name) { m->SetName(name); }
    m->SetInputShape({(index_t)I});
    put_wiring(*m, O, idx);
    { auto Wp = m->lock_W(); for (int i = 0; i < O * 64; ++i) { Wp(i / 64, i % 64) = W[i]; } }
    m->SendCommand("binary " + onoff(flags & 1));
    m->SendCommand("lut_binarize " + onoff(flags & 2));
    return emit(*m, out, cap);
}
template <typename BinType>
int load_stochastic(unsigned char const *bytes, long size, int O, std::int32_t *idx, float *W, char *name, int name_cap)
{
    auto m = bb::StochasticLutN<6, BinType, float>::Create((index_t)O);
    std::istringstream is(std::string((char const *)bytes, (size_t)size), std::ios::binary);
    m->LoadObject(is);
    if ((int)m->GetOutputNodeSize() != O) { return -1; }
    get_wiring(*m, O, idx);
    { auto Wp = m->lock_W_const(); for (int i = 0; i < O * 64; ++i) { W[i] = Wp(i / 64, i % 64); } }
    std::snprintf(name, (size_t)name_cap, "%s", m->GetName().c_str());
    return (int)m->GetInputNodeSize();
}

template <typename BinType>
long dump_differentiable(int I, int O, std::int32_t const *idx, float const *W, float const *mean, float const *var, int flags,
                         float const *scalars, char const *name, unsigned char *out, long cap)
{
    typename bb::DifferentiableLutN<6, BinType, float>::create_t c;
    c.output_shape = {(index_t)O};
    c.batch_norm = (flags & 4) != 0;
    c.binary = (flags & 1) != 0;
    c.momentum = scalars[0]; c.gamma = scalars[1]; c.beta = scalars[2];
    auto m = bb::DifferentiableLutN<6, BinType, float>::Create(c);
    if (name && *name) { m->SetName(name); }
    m->SetInputShape({(index_t)I});
    put_wiring(*m, O, idx);
    { auto Wp = m->lock_W(); for (int i = 0; i < O * 64; ++i) { Wp(i / 64, i % 64) = W[i]; } }
    { auto p = m->lock_mean(); for (int o = 0; o < O; ++o) { p[o] = mean[o]; } }
    { auto p = m->lock_var();  for (int o = 0; o < O; ++o) { p[o] = var[o]; } }
    m->SendCommand("lut_binarize " + onoff(flags & 2));
    return emit(*m, out, cap);
}
template <typename BinType>
int load_differentiable(unsigned char const *bytes, long size, int O, std::int32_t *idx, float *W, float *mean, float *var, char *name, int name_cap)
{
    auto m = bb::DifferentiableLutN<6, BinType, float>::Create((index_t)O);
    std::istringstream is(std::string((char const *)bytes, (size_t)size), std::ios::binary);
    m->LoadObject(is);
    if ((int)m->GetOutputNodeSize() != O) { return -1; }
    get_wiring(*m, O, idx);
    { auto Wp = m->lock_W_const(); for (int i = 0; i < O * 64; ++i) { W[i] = Wp(i / 64, i % 64); } }
    { auto p = m->lock_mean_const(); for (int o = 0; o < O; ++o) { mean[o] = p[o]; } }
    { auto p = m->lock_var_const();  for (int o = 0; o < O; ++o) { var[o] = p[o]; } }
    std::snprintf(name, (size_t)name_cap, "%s", m->GetName().c_str());
    return (int)m->GetInputNodeSize();
}

}  // namespace

extern "C" long bbref_DumpLutObject(int kind, int bit, int I, int O, std::int32_t const *idx, void const *params, float const *mean,
                                    float const *var, int flags, float const *scalars, char const *name, unsigned char *out, long cap)
{
    if (kind == 0) { return bit ? dump_stochastic<bb::Bit>(I, O, idx, (float const *)params, flags, name, out, cap)
                                : dump_stochastic<float>(I, O, idx, (float const *)params, flags, name, out, cap); }
    if (kind == 1) { return bit ? dump_differentiable<bb::Bit>(I, O, idx, (float const *)params, mean, var, flags, scalars, name, out, cap)
                                : dump_differentiable<float>(I, O, idx, (float const *)params, mean, var, flags, scalars, name, out, cap); }
    auto m = bb::BinaryLutN<6, bb::Bit, float>::Create((index_t)O);
    if (name && *name) { m->SetName(name); }
    m->SetInputShape({(index_t)I});
    put_wiring(*m, O, idx);
    std::int32_t const *table = (std::int32_t const *)params;
    for (int o = 0; o < O; ++o) { for (int b = 0; b < 64; ++b) { m->SetLutTable(o, b, ((table[o * 2 + b / 32] >> (b % 32)) & 1) != 0); } }
    return emit(*m, out, cap);
}

// returns the input node count of the loaded layer (negative on a mismatch)
extern "C" int bbref_LoadLutObject(int kind, int bit, unsigned char const *bytes, long size, int O, std::int32_t *idx, void *params,
                                   float *mean, float *var, char *name, int name_cap)
{
    if (kind == 0) { return bit ? load_stochastic<bb::Bit>(bytes, size, O, idx, (float *)params, name, name_cap)
                                : load_stochastic<float>(bytes, size, O, idx, (float *)params, name, name_cap); }
    if (kind == 1) { return bit ? load_differentiable<bb::Bit>(bytes, size, O, idx, (float *)params, mean, var, name, name_cap)
                                : load_differentiable<float>(bytes, size, O, idx, (float *)params, mean, var, name, name_cap); }
    auto m = bb::BinaryLutN<6, bb::Bit, float>::Create((index_t)O);
    std::istringstream is(std::string((char const *)bytes, (size_t)size), std::ios::binary);
    m->LoadObject(is);
    if ((int)m->GetOutputNodeSize() != O) { return -1; }
    get_wiring(*m, O, idx);
    std::int32_t *table = (std::int32_t *)params;
    for (int o = 0; o < O; ++o) {
        table[o * 2] = table[o * 2 + 1] = 0;
        for (int b = 0; b < 64; ++b) { if (m->GetLutTable(o, b)) { table[o * 2 + b / 32] |= (std::int32_t)(1u << (b % 32)); } }
    }
    std::snprintf(name, (size_t)name_cap, "%s", m->GetName().c_str());
    return (int)m->GetInputNodeSize();
}

// ---- container objects: the convolution wrapper around one LUT layer or a list of two, the list alone, Im2Col, Col2Im ----
// kind 0: Convolution2d over one DifferentiableLut6; 1: Convolution2d over a Sequential of two DifferentiableLut6 layers;
// 2: that Sequential alone (input shape {c * fh * fw}); 3: ConvolutionIm2Col; 4: ConvolutionCol2Im (after SetInputShape({o2})).
// The layers are wired and initialised by the reference with the given seed; their contents only have to survive.
extern "C" long bbref_DumpContainerObject(int kind, int c, int h, int w, int fh, int fw, int ys, int xs, int same, char const *border_mode,
                                          int o1, int o2, int seed, char const *name, unsigned char *out, long cap)
{
    std::string const padding = same ? "same" : "valid";
    auto make_lut = [&](int o, int s) {
        typename bb::DifferentiableLutN<6, float, float>::create_t cr;
        cr.output_shape = {(index_t)o};
        cr.seed = (std::uint64_t)s;
        return bb::DifferentiableLutN<6, float, float>::Create(cr);
    };
    if (kind == 3) {
        auto m = bb::ConvolutionIm2Col<float, float>::Create((index_t)fh, (index_t)fw, (index_t)ys, (index_t)xs, padding, border_mode);
        if (name && *name) { m->SetName(name); }
        m->SetInputShape({(index_t)c, (index_t)h, (index_t)w});
        return emit(*m, out, cap);
    }
    if (kind == 4) {
        auto m = bb::ConvolutionCol2Im<float, float>::Create((index_t)h, (index_t)w);
        if (name && *name) { m->SetName(name); }
        m->SetInputShape({(index_t)o2});
        return emit(*m, out, cap);
    }
    std::shared_ptr<bb::Model> sub;
    if (kind == 0) { sub = make_lut(o2, seed); }
    else {
        auto seq = bb::Sequential::Create();
        seq->Add(make_lut(o1, seed));
        seq->Add(make_lut(o2, seed + 1));
        if (kind == 2 && name && *name) { seq->SetName(name); }
        sub = seq;
    }
    if (kind == 2) {
        sub->SetInputShape({(index_t)(c * fh * fw)});
        return emit(*sub, out, cap);
    }
    auto m = bb::Convolution2d<float, float>::Create(sub, (index_t)fh, (index_t)fw, (index_t)ys, (index_t)xs, padding, border_mode);
    if (name && *name) { m->SetName(name); }
    m->SetInputShape({(index_t)c, (index_t)h, (index_t)w});
    return emit(*m, out, cap);
}

// Loads a container object written elsewhere into the reference's own classes (rebuilt from the type names in the stream) and
// dumps it again: returns the size of the re-dumped object, negative if the reference could not load it.
extern "C" long bbref_ReloadContainerObject(unsigned char const *bytes, long size, unsigned char *out, long cap)
{
    std::istringstream is(std::string((char const *)bytes, (size_t)size), std::ios::binary);
    auto obj = bb::Object_Load(is);
    if (!obj) { return -1; }
    return emit(*obj, out, cap);
}

// StochasticBatchNormalization<float> (generic host path: host_only, no SIMD).  x, y, dy, dx: [nodes][frames].
// The running statistics start at running_mean / running_var (in) and come back updated; mean / rstd are the batch statistics
// kept for the backward pass.  train == 0 runs the inference formula; it takes its offset from the batch mean of the last
// training pass, so a caller that wants the running mean there runs one training pass with momentum 0 on the same batch first.
// object_out (may be null) receives the layer dumped after the passes; returns its size (0 without object_out), negative on error.
extern "C" long bbref_StochasticBatchNormalization(int nodes, int frames, float momentum, float gamma, float beta, int train,
                                                   float const *x, float *running_mean, float *running_var, float *y, float *mean,
                                                   float *rstd, float const *dy, float *dx, char const *name,
                                                   unsigned char *object_out, long cap)
{
    auto m = bb::StochasticBatchNormalization<float>::Create(momentum, gamma, beta);
    m->SendCommand("host_only true");
    if (name && *name) { m->SetName(name); }
    m->SetInputShape({(index_t)nodes});
    {
        auto rm = m->lock_mean();
        auto rv = m->lock_var();
        for (int n = 0; n < nodes; ++n) { rm[n] = running_mean[n]; rv[n] = running_var[n]; }
    }
    bb::FrameBuffer xb((index_t)frames, bb::indices_t({(index_t)nodes}), BB_TYPE_FP32, true);
    put_fp32(xb, x, nodes, frames);
    bb::FrameBuffer yb = m->Forward(xb, train != 0);
    get_fp32(yb, y, nodes, frames);
    {
        auto rm = m->lock_mean_const();
        auto rv = m->lock_var_const();
        for (int n = 0; n < nodes; ++n) { running_mean[n] = rm[n]; running_var[n] = rv[n]; }
    }
    if (train) {
        auto bm = m->lock_tmp_mean_const();
        auto br = m->lock_tmp_rstd_const();
        for (int n = 0; n < nodes; ++n) { mean[n] = bm[n]; rstd[n] = br[n]; }
    }
    if (train && dy) {
        bb::FrameBuffer dyb((index_t)frames, bb::indices_t({(index_t)nodes}), BB_TYPE_FP32, true);
        put_fp32(dyb, dy, nodes, frames);
        bb::FrameBuffer dxb = m->Backward(dyb);
        get_fp32(dxb, dx, nodes, frames);
    }
    return object_out ? emit(*m, object_out, cap) : 0;
}

// MaxLut<BinType, float> (host path).  x: [I][frames] (fp32) or [I][words] (bits); y likewise for O nodes; dx is fp32 either way.
// object_out (may be null) receives the layer dumped after the passes; returns its size (0 without), negative on error.
namespace {
template <typename BinType>
long run_max_lut(int n, int I, int O, int F, void const *x, std::int32_t const *idx, int binarize_input, int binarize_output,
                 void *y, float const *dy, float *dx, char const *name, unsigned char *object_out, long cap)
{
    auto m = bb::MaxLut<BinType, float>::Create(n, bb::indices_t({(index_t)O}));
    m->SendCommand("host_only true");
    m->SendCommand("binarize_input " + onoff(binarize_input));
    m->SendCommand("binarize_output " + onoff(binarize_output));
    if (name && *name) { m->SetName(name); }
    int const xtype = bb::DataType<BinType>::type;
    bb::FrameBuffer xb((index_t)F, bb::indices_t({(index_t)I}), xtype, true);
    m->SetInputShape(xb.GetShape());
    for (int o = 0; o < O; ++o) { for (int i = 0; i < n; ++i) { m->SetNodeConnectionIndex(o, i, idx[o * n + i]); } }
    if (xtype == BB_TYPE_BIT) { put_bit(xb, (std::int32_t const *)x, I, (F + 31) / 32); }
    else                      { put_fp32(xb, (float const *)x, I, F); }
    bb::FrameBuffer yb = m->Forward(xb, true);
    if (xtype == BB_TYPE_BIT) { get_bit(yb, (std::int32_t *)y, O, (F + 31) / 32); }
    else                      { get_fp32(yb, (float *)y, O, F); }
    if (dy) {
        bb::FrameBuffer dyb((index_t)F, bb::indices_t({(index_t)O}), BB_TYPE_FP32, true);
        put_fp32(dyb, dy, O, F);
        bb::FrameBuffer dxb = m->Backward(dyb);
        get_fp32(dxb, dx, I, F);
    }
    return object_out ? emit(*m, object_out, cap) : 0;
}
}  // namespace

extern "C" long bbref_MaxLut(int bit, int n, int I, int O, int F, void const *x, std::int32_t const *idx, int binarize_input,
                             int binarize_output, void *y, float const *dy, float *dx, char const *name, unsigned char *object_out, long cap)
{
    return bit ? run_max_lut<bb::Bit>(n, I, O, F, x, idx, binarize_input, binarize_output, y, dy, dx, name, object_out, cap)
               : run_max_lut<float>(n, I, O, F, x, idx, binarize_input, binarize_output, y, dy, dx, name, object_out, cap);
}

// An AverageLut<BinType, float> with the given wiring, dumped: returns the object's size, negative on error.
extern "C" long bbref_AverageLutObject(int bit, int n, int I, int O, std::int32_t const *idx, int binarize_input, int binarize_output,
                                       char const *name, unsigned char *out, long cap)
{
    auto fill = [&](auto m) {
        m->SendCommand("binarize_input " + onoff(binarize_input));
        m->SendCommand("binarize_output " + onoff(binarize_output));
        if (name && *name) { m->SetName(name); }
        m->SetInputShape(bb::indices_t({(index_t)I}));
        for (int o = 0; o < O; ++o) { for (int i = 0; i < n; ++i) { m->SetNodeConnectionIndex(o, i, idx[o * n + i]); } }
        return emit(*m, out, cap);
    };
    if (bit) { return fill(bb::AverageLut<bb::Bit, float>::Create(n, bb::indices_t({(index_t)O}))); }
    return fill(bb::AverageLut<float, float>::Create(n, bb::indices_t({(index_t)O})));
}

// Reduce<BinType, float> (host path).  x: [I][frames] fp32 or [I][words] bits; y, dy: [O][frames]; dx: [I][frames].
// integration_size 0: the output shape {O} is given; otherwise the layer derives it from the input shape {I}.
namespace {
template <typename BinType>
long run_reduce(int I, int O, int F, int integration_size, void const *x, float *y, float const *dy, float *dx, char const *name,
                unsigned char *object_out, long cap)
{
    auto m = bb::Reduce<BinType, float>::Create(bb::indices_t({(index_t)O}), (index_t)integration_size);
    if (name && *name) { m->SetName(name); }
    int const xtype = bb::DataType<BinType>::type;
    bb::FrameBuffer xb((index_t)F, bb::indices_t({(index_t)I}), xtype, true);
    m->SetInputShape(xb.GetShape());
    if (m->GetOutputNodeSize() != O) { return -2; }
    if (xtype == BB_TYPE_BIT) { put_bit(xb, (std::int32_t const *)x, I, (F + 31) / 32); }
    else                      { put_fp32(xb, (float const *)x, I, F); }
    bb::FrameBuffer yb = m->Forward(xb, true);
    get_fp32(yb, y, O, F);
    if (dy) {
        bb::FrameBuffer dyb((index_t)F, bb::indices_t({(index_t)O}), BB_TYPE_FP32, true);
        put_fp32(dyb, dy, O, F);
        bb::FrameBuffer dxb = m->Backward(dyb);
        get_fp32(dxb, dx, I, F);
    }
    return object_out ? emit(*m, object_out, cap) : 0;
}
}  // namespace

extern "C" long bbref_Reduce(int bit, int I, int O, int F, int integration_size, void const *x, float *y, float const *dy, float *dx,
                             char const *name, unsigned char *object_out, long cap)
{
    return bit ? run_reduce<bb::Bit>(I, O, F, integration_size, x, y, dy, dx, name, object_out, cap)
               : run_reduce<float>(I, O, F, integration_size, x, y, dy, dx, name, object_out, cap);
}

// LossMeanSquaredError<float> and MetricsMeanSquaredError<float> (host paths) over `batches` equal batches of F frames held one
// after the other in y and t ([nodes][batches * F]); dy likewise.  loss = GetLoss(), metric = GetMetrics() after all of them.
extern "C" int bbref_MeanSquaredError(int nodes, int F, int batches, int reduction_sum, float const *y, float const *t, float *dy,
                                      double *loss, double *metric)
{
    auto lossFunc = bb::LossMeanSquaredError<float>::Create(reduction_sum ? "sum" : "");
    auto metrics = bb::MetricsMeanSquaredError<float>::Create();
    lossFunc->Clear();
    metrics->Clear();
    std::vector<float> ys((size_t)nodes * F), ts((size_t)nodes * F), ds((size_t)nodes * F);
    for (int b = 0; b < batches; ++b) {
        for (int n = 0; n < nodes; ++n) {
            std::memcpy(&ys[(size_t)n * F], y + ((size_t)n * batches + b) * F, sizeof(float) * (size_t)F);
            std::memcpy(&ts[(size_t)n * F], t + ((size_t)n * batches + b) * F, sizeof(float) * (size_t)F);
        }
        bb::FrameBuffer yb((index_t)F, bb::indices_t({(index_t)nodes}), BB_TYPE_FP32, true), tb((index_t)F, bb::indices_t({(index_t)nodes}), BB_TYPE_FP32, true);
        put_fp32(yb, ys.data(), nodes, F);
        put_fp32(tb, ts.data(), nodes, F);
        bb::FrameBuffer dyb = lossFunc->CalculateLoss(yb, tb, (index_t)F);
        get_fp32(dyb, ds.data(), nodes, F);
        for (int n = 0; n < nodes; ++n) { std::memcpy(dy + ((size_t)n * batches + b) * F, &ds[(size_t)n * F], sizeof(float) * (size_t)F); }
        metrics->CalculateMetrics(yb, tb);
    }
    *loss = lossFunc->GetLoss();
    *metric = metrics->GetMetrics();
    return 0;
}

// RealToBinary<BinType, float> (host path, no value generator).  x: [depth * points][F]; y: [depth * depth_mod * points][F * frame_mod]
// as fp32 or as rows of ceil(F * frame_mod / 32) words.
namespace {
template <typename BinType>
long run_real_to_binary(int depth, int points, int F, int frame_mod, int depth_mod, float lo, float hi, int binary_mode,
                        float const *x, void *y, char const *name, unsigned char *object_out, long cap)
{
    auto m = bb::RealToBinary<BinType, float>::Create((index_t)frame_mod, (index_t)depth_mod, nullptr, false, lo, hi);
    if (name && *name) { m->SetName(name); }
    m->SendCommand("binary " + onoff(binary_mode));
    bb::FrameBuffer xb((index_t)F, bb::indices_t({(index_t)depth, (index_t)points}), BB_TYPE_FP32, true);
    m->SetInputShape(xb.GetShape());
    put_fp32(xb, x, (index_t)depth * points, F);
    bb::FrameBuffer yb = m->Forward(xb, true);
    index_t const out_nodes = (index_t)depth * depth_mod * points, out_frames = (index_t)F * frame_mod;
    if (yb.GetNodeSize() != out_nodes || yb.GetFrameSize() != out_frames) { return -2; }
    if (bb::DataType<BinType>::type == BB_TYPE_BIT) { get_bit(yb, (std::int32_t *)y, out_nodes, (out_frames + 31) / 32); }
    else                                            { get_fp32(yb, (float *)y, out_nodes, out_frames); }
    return object_out ? emit(*m, object_out, cap) : 0;
}

template <typename BinType>
long run_binary_to_real(int I, int O, int F, int frame_mux, void const *x, float *y, float const *dy, float *dx, char const *name,
                        unsigned char *object_out, long cap)
{
    auto m = bb::BinaryToReal<BinType, float>::Create((index_t)frame_mux, bb::indices_t({(index_t)O}));
    if (name && *name) { m->SetName(name); }
    int const xtype = bb::DataType<BinType>::type;
    bb::FrameBuffer xb((index_t)F, bb::indices_t({(index_t)I}), xtype, true);
    m->SetInputShape(xb.GetShape());
    if (xtype == BB_TYPE_BIT) { put_bit(xb, (std::int32_t const *)x, I, (F + 31) / 32); }
    else                      { put_fp32(xb, (float const *)x, I, F); }
    bb::FrameBuffer yb = m->Forward(xb, true);
    if (yb.GetNodeSize() != O || yb.GetFrameSize() != F / frame_mux) { return -2; }
    get_fp32(yb, y, O, F / frame_mux);
    if (dy) {
        bb::FrameBuffer dyb((index_t)(F / frame_mux), bb::indices_t({(index_t)O}), BB_TYPE_FP32, true);
        put_fp32(dyb, dy, O, F / frame_mux);
        bb::FrameBuffer dxb = m->Backward(dyb);
        if (dxb.GetNodeSize() != I || dxb.GetFrameSize() != F) { return -3; }
        get_fp32(dxb, dx, I, F);
    }
    return object_out ? emit(*m, object_out, cap) : 0;
}

// kind 0: Binarize<BinType>(th, low, high, lo, hi); kind 1: HardTanh<BinType>(lo, hi); kind 2: HardTanh in binary mode
template <typename BinType>
long run_activation(int kind, int nodes, int F, float th, float low, float high, float lo, float hi, float const *x, void *y,
                    float const *dy, float *dx, char const *name, unsigned char *object_out, long cap)
{
    std::shared_ptr<bb::Binarize<BinType, float>> m;
    if (kind == 0) { m = bb::Binarize<BinType, float>::Create(th, (double)low, (double)high, lo, hi); }
    else {
        m = bb::HardTanh<BinType, float>::Create(lo, hi);
        if (kind == 2) { m->SendCommand("binary true"); }
    }
    if (name && *name) { m->SetName(name); }
    bb::FrameBuffer xb((index_t)F, bb::indices_t({(index_t)nodes}), BB_TYPE_FP32, true);
    m->SetInputShape(xb.GetShape());
    put_fp32(xb, x, nodes, F);
    bb::FrameBuffer yb = m->Forward(xb, true);
    if (yb.GetType() == BB_TYPE_BIT) { get_bit(yb, (std::int32_t *)y, nodes, (F + 31) / 32); }
    else                             { get_fp32(yb, (float *)y, nodes, F); }
    if (dy) {
        bb::FrameBuffer dyb((index_t)F, bb::indices_t({(index_t)nodes}), BB_TYPE_FP32, true);
        put_fp32(dyb, dy, nodes, F);
        bb::FrameBuffer dxb = m->Backward(dyb);
        get_fp32(dxb, dx, nodes, F);
    }
    return object_out ? emit(*m, object_out, cap) : 0;
}
}  // namespace

extern "C" long bbref_RealToBinary(int bit, int depth, int points, int F, int frame_mod, int depth_mod, float lo, float hi, int binary_mode,
                                   float const *x, void *y, char const *name, unsigned char *object_out, long cap)
{
    return bit ? run_real_to_binary<bb::Bit>(depth, points, F, frame_mod, depth_mod, lo, hi, binary_mode, x, y, name, object_out, cap)
               : run_real_to_binary<float>(depth, points, F, frame_mod, depth_mod, lo, hi, binary_mode, x, y, name, object_out, cap);
}

// BinaryToReal<BinType, float> (host path) with output shape {O}.  x: [I][F] fp32 or bits; y, dy: [O][F / frame_mux]; dx: [I][F].
extern "C" long bbref_BinaryToReal(int bit, int I, int O, int F, int frame_mux, void const *x, float *y, float const *dy, float *dx,
                                   char const *name, unsigned char *object_out, long cap)
{
    return bit ? run_binary_to_real<bb::Bit>(I, O, F, frame_mux, x, y, dy, dx, name, object_out, cap)
               : run_binary_to_real<float>(I, O, F, frame_mux, x, y, dy, dx, name, object_out, cap);
}

// Binarize / HardTanh (host paths), see run_activation.  y: fp32 [nodes][F], or bits when the layer's output type is Bit.
extern "C" long bbref_Activation(int kind, int bit, int nodes, int F, float th, float low, float high, float lo, float hi,
                                 float const *x, void *y, float const *dy, float *dx, char const *name, unsigned char *object_out, long cap)
{
    return bit ? run_activation<bb::Bit>(kind, nodes, F, th, low, high, lo, hi, x, y, dy, dx, name, object_out, cap)
               : run_activation<float>(kind, nodes, F, th, low, high, lo, hi, x, y, dy, dx, name, object_out, cap);
}

// A BinaryModulation<BinType, float> around a Sequential of two DifferentiableLut6 layers (I -> o1 -> o2 nodes, wired and initialised
// by the reference from the seed), dumped after SetInputShape({I}) and, with run_inference, after one inference pass over four zero
// frames (which leaves the converters at the inference modulation size).  Returns the object's size, negative on error.
namespace {
template <typename BinType>
long dump_binary_modulation(int I, int o1, int o2, int train_mod, int infer_mod, int depth_mod, int seed, int run_inference, char const *name,
                            unsigned char *out, long cap)
{
    auto make_lut = [&](int o, int s) {
        typename bb::DifferentiableLutN<6, BinType, float>::create_t cr;
        cr.output_shape = {(index_t)o};
        cr.seed = (std::uint64_t)s;
        return bb::DifferentiableLutN<6, BinType, float>::Create(cr);
    };
    auto body = bb::Sequential::Create();
    body->Add(make_lut(o1, seed));
    body->Add(make_lut(o2, seed + 1));
    auto m = bb::BinaryModulation<BinType, float>::Create(body, (index_t)train_mod, (index_t)infer_mod, (index_t)depth_mod);
    if (name && *name) { m->SetName(name); }
    m->SendCommand("host_only true");
    m->SetInputShape(bb::indices_t({(index_t)I}));
    if (run_inference) {
        bb::FrameBuffer xb((index_t)4, bb::indices_t({(index_t)I}), BB_TYPE_FP32, true);
        xb.FillZero();
        (void)m->Forward(xb, false);
    }
    return emit(*m, out, cap);
}
}  // namespace

extern "C" long bbref_DumpBinaryModulationObject(int bit, int I, int o1, int o2, int train_mod, int infer_mod, int depth_mod, int seed,
                                                 int run_inference, char const *name, unsigned char *out, long cap)
{
    return bit ? dump_binary_modulation<bb::Bit>(I, o1, o2, train_mod, infer_mod, depth_mod, seed, run_inference, name, out, cap)
               : dump_binary_modulation<float>(I, o1, o2, train_mod, infer_mod, depth_mod, seed, run_inference, name, out, cap);
}

// A DifferentiableLutDiscreteN<6, BinType, float> (StochasticLutN -> StochasticBatchNormalization -> HardTanh), wired and initialised
// by the reference from the seed, dumped after SetInputShape({I}).  Returns the object's size, negative on error.
extern "C" long bbref_DumpDiscreteLutObject(int bit, int I, int O, int seed, int batch_norm, int memory_saving, char const *name,
                                            unsigned char *out, long cap)
{
    auto fill = [&](auto m) {
        if (name && *name) { m->SetName(name); }
        m->SendCommand("memory_saving " + onoff(memory_saving));
        m->SetInputShape(bb::indices_t({(index_t)I}));
        return emit(*m, out, cap);
    };
    if (bit) { return fill(bb::DifferentiableLutDiscreteN<6, bb::Bit, float>::Create((index_t)O, batch_norm != 0, "", (std::uint64_t)seed)); }
    return fill(bb::DifferentiableLutDiscreteN<6, float, float>::Create((index_t)O, batch_norm != 0, "", (std::uint64_t)seed));
}

// MaxPooling<BinType, float> and UpSampling<BinType, float> (host paths).  x: [c * h * w][F] fp32 or bits; dy, y: the output shape.
namespace {
template <typename BinType>
long run_max_pooling(int c, int h, int w, int fh, int fw, int F, void const *x, void *y, float const *dy, float *dx, char const *name,
                     unsigned char *object_out, long cap)
{
    auto m = bb::MaxPooling<BinType, float>::Create((index_t)fh, (index_t)fw);
    m->SendCommand("host_only true");
    if (name && *name) { m->SetName(name); }
    int const xtype = bb::DataType<BinType>::type;
    bb::FrameBuffer xb((index_t)F, bb::indices_t({(index_t)c, (index_t)h, (index_t)w}), xtype, true);
    auto out_shape = m->SetInputShape(xb.GetShape());
    index_t const I = (index_t)c * h * w, O = bb::CalcShapeSize(out_shape);
    if (xtype == BB_TYPE_BIT) { put_bit(xb, (std::int32_t const *)x, I, (F + 31) / 32); }
    else                      { put_fp32(xb, (float const *)x, I, F); }
    bb::FrameBuffer yb = m->Forward(xb, true);
    if (yb.GetNodeSize() != O) { return -2; }
    if (xtype == BB_TYPE_BIT) { get_bit(yb, (std::int32_t *)y, O, (F + 31) / 32); }
    else                      { get_fp32(yb, (float *)y, O, F); }
    if (dy) {
        bb::FrameBuffer dyb((index_t)F, out_shape, BB_TYPE_FP32, true);
        put_fp32(dyb, dy, O, F);
        bb::FrameBuffer dxb = m->Backward(dyb);
        get_fp32(dxb, dx, I, F);
    }
    return object_out ? emit(*m, object_out, cap) : 0;
}

template <typename BinType>
long run_up_sampling(int c, int h, int w, int fh, int fw, int fill, int F, void const *x, void *y, float const *dy, float *dx, char const *name,
                     unsigned char *object_out, long cap)
{
    auto m = bb::UpSampling<BinType, float>::Create((index_t)fh, (index_t)fw, fill != 0);
    m->SendCommand("host_only true");
    if (name && *name) { m->SetName(name); }
    int const xtype = bb::DataType<BinType>::type;
    bb::FrameBuffer xb((index_t)F, bb::indices_t({(index_t)c, (index_t)h, (index_t)w}), xtype, true);
    auto out_shape = m->SetInputShape(xb.GetShape());
    index_t const I = (index_t)c * h * w, O = bb::CalcShapeSize(out_shape);
    if (xtype == BB_TYPE_BIT) { put_bit(xb, (std::int32_t const *)x, I, (F + 31) / 32); }
    else                      { put_fp32(xb, (float const *)x, I, F); }
    bb::FrameBuffer yb = m->Forward(xb, true);
    if (yb.GetNodeSize() != O) { return -2; }
    if (xtype == BB_TYPE_BIT) { get_bit(yb, (std::int32_t *)y, O, (F + 31) / 32); }
    else                      { get_fp32(yb, (float *)y, O, F); }
    if (dy) {
        bb::FrameBuffer dyb((index_t)F, out_shape, BB_TYPE_FP32, true);
        put_fp32(dyb, dy, O, F);
        bb::FrameBuffer dxb = m->Backward(dyb);
        get_fp32(dxb, dx, I, F);
    }
    return object_out ? emit(*m, object_out, cap) : 0;
}
}  // namespace

extern "C" long bbref_MaxPooling(int bit, int c, int h, int w, int fh, int fw, int F, void const *x, void *y, float const *dy, float *dx,
                                 char const *name, unsigned char *object_out, long cap)
{
    return bit ? run_max_pooling<bb::Bit>(c, h, w, fh, fw, F, x, y, dy, dx, name, object_out, cap)
               : run_max_pooling<float>(c, h, w, fh, fw, F, x, y, dy, dx, name, object_out, cap);
}

extern "C" long bbref_UpSampling(int bit, int c, int h, int w, int fh, int fw, int fill, int F, void const *x, void *y, float const *dy,
                                 float *dx, char const *name, unsigned char *object_out, long cap)
{
    return bit ? run_up_sampling<bb::Bit>(c, h, w, fh, fw, fill, F, x, y, dy, dx, name, object_out, cap)
               : run_up_sampling<float>(c, h, w, fh, fw, fill, F, x, y, dy, dx, name, object_out, cap);
}

// Shuffle (host path): x [node_size][F] fp32 or bits -> y; dy of the same type -> dx.  output_node_size > 0 asks for that output
// shape, 0 keeps the input shape.
extern "C" long bbref_Shuffle(int bit, int shuffle_unit, int node_size, int F, void const *x, void *y, void const *dy, void *dx,
                              char const *name, unsigned char *object_out, long cap)
{
    auto m = bb::Shuffle::Create((index_t)shuffle_unit);
    m->SendCommand("host_only true");
    if (name && *name) { m->SetName(name); }
    int const xtype = bit ? BB_TYPE_BIT : BB_TYPE_FP32;
    index_t const N = (index_t)node_size;
    bb::FrameBuffer xb((index_t)F, bb::indices_t({N}), xtype, true);
    auto out_shape = m->SetInputShape(xb.GetShape());
    if (bb::CalcShapeSize(out_shape) != N) { return -2; }
    if (bit) { put_bit(xb, (std::int32_t const *)x, N, (F + 31) / 32); }
    else     { put_fp32(xb, (float const *)x, N, F); }
    bb::FrameBuffer yb = m->Forward(xb, true);
    if (bit) { get_bit(yb, (std::int32_t *)y, N, (F + 31) / 32); }
    else     { get_fp32(yb, (float *)y, N, F); }
    if (dy) {
        bb::FrameBuffer dyb((index_t)F, out_shape, xtype, true);
        if (bit) { put_bit(dyb, (std::int32_t const *)dy, N, (F + 31) / 32); }
        else     { put_fp32(dyb, (float const *)dy, N, F); }
        bb::FrameBuffer dxb = m->Backward(dyb);
        if (bit) { get_bit(dxb, (std::int32_t *)dx, N, (F + 31) / 32); }
        else     { get_fp32(dxb, (float *)dx, N, F); }
    }
    return object_out ? emit(*m, object_out, cap) : 0;
}

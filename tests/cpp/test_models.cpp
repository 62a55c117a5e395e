// GPU test of the C++ model classes (bb::StochasticLutN, bb::DifferentiableLutN, bb::BinaryLutN) in the shape of the
// reference's own parity test (tests/gtest/StochasticLutNTest.cpp:15-246): random wiring/table/input injected into the
// model, Forward/Backward on the device, results compared with the CPU oracle (oracle/bb_oracle.c, linked as the
// checker only).  Exit status 0 = all checks passed.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <sstream>
#include <vector>

#include "bb/StochasticLutN.h"
#include "bb/DifferentiableLutN.h"
#include "bb/BinaryLutN.h"
#include "bb/OptimizerAdam.h"
#include "bb/ConvolutionIm2Col.h"
#include "bb/ConvolutionCol2Im.h"
#include "bb/StochasticMaxPooling2x2.h"
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
#include "bb/Binarize.h"
#include "bb/HardTanh.h"
#include "bb/RealToBinary.h"
#include "bb/BinaryToReal.h"
#include "bb/BinaryModulation.h"
#include "bb/DifferentiableLutDiscreteN.h"
#include "bb/MaxPooling.h"
#include "bb/UpSampling.h"
#include "bb/Shuffle.h"
#include "bb/ObjectLoader.h"

extern "C" {
void oracle_fp32_AverageLut_Forward(float const *x, float *y, std::int32_t const *idx, int n, int node_size, int frame_size, int frame_stride, int binarize_input, int binarize_output);
void oracle_bit_AverageLut_Forward(int const *x, int *y, std::int32_t const *idx, int n, int node_size, int frame_size, int frame_stride);
void oracle_fp32_AverageLut_Backward(float const *dy, float *dx, std::int32_t const *idx, int n, int input_node_size, int output_node_size, int frame_size, int frame_stride);
void oracle_fp32_Im2Col_Backward(float const *dy, float *dx, int x_stride, int y_stride, int x_offset, int y_offset, int input_frame_size,
                                 int input_frame_stride, int w, int h, int c, int ow, int oh, int output_frame_stride, int fw, int fh);
void oracle_fp32_StochasticMaxPooling2x2_Forward(float const *x, float *y, int w, int h, int ow, int oh, int c, int frame_size, int frame_stride);
void oracle_fp32_StochasticMaxPooling2x2_Backward(float const *x, float const *dy, float *dx, int w, int h, int ow, int oh, int c, int frame_size, int frame_stride);
void oracle_fp32_OptimizerAdam(int size, float *param, float const *grad, float *m, float *v, float lr_t, float beta1, float beta2);
void oracle_fp32_StochasticLut_Forward(int n, float const *x, float *y, std::int32_t const *idx, float const *W, int node_size, int frame_size, int frame_stride, int input_binary, int lut_binarize, float bias, int simd);
void oracle_fp32_StochasticLut_Backward(int n, float const *x, float const *dy, float *dx, std::int32_t const *idx, float const *W, float *dW, int input_node_size, int output_node_size, int frame_size, int frame_stride, int input_binary, int lut_binarize, float bias, int simd);
void oracle_fp32_DifferentiableLutN_ForwardTraining(int n, float const *x, float *y, std::int32_t const *idx, float const *W, float *mean, float *rstd, float *running_mean, float *running_var, float gamma, float beta, float momentum, float bias, int node_size, int frame_size, int frame_stride, int lut_binarize, int binary_mode);
void oracle_fp32_DifferentiableLutN_Backward(int n, float const *x, float const *dy, float *dx, std::int32_t const *idx, float const *W, float *dW, float const *mean, float const *rstd, float gamma, float beta, float bias, int input_node_size, int output_node_size, int frame_size, int frame_stride, int lut_binarize, int binary_mode);
void oracle_fp32_StochasticBatchNormalization_ForwardTraining(float const *x, float *y, float *mean, float *rstd, float *running_mean, float *running_var, float gamma, float beta, float momentum, int node_size, int frame_size, int frame_stride);
void oracle_fp32_StochasticBatchNormalization_ForwardInference(float const *x, float *y, float const *running_mean, float const *running_var, float gamma, float beta, int node_size, int frame_size, int frame_stride);
void oracle_fp32_StochasticBatchNormalization_Backward(float const *x, float const *dy, float *dx, float const *mean, float const *rstd, float gamma, int node_size, int frame_size, int frame_stride, int x_frame_stride);
void oracle_fp32_MaxLut_Forward(float const *x, float *y, std::int32_t const *idx, int n, int node_size, int frame_size, int frame_stride, int binarize_input, int binarize_output);
void oracle_fp32_MaxLut_Backward(float const *x, float const *dy, float *dx, std::int32_t const *idx, int n, int input_node_size, int output_node_size, int frame_size, int frame_stride, int binarize_input);
void oracle_fp32_Reduce_Forward(float const *x, float *y, int input_node_size, int output_node_size, int frame_size, int frame_stride);
void oracle_fp32_Reduce_Backward(float const *dy, float *dx, int input_node_size, int output_node_size, int frame_size, int frame_stride);
void oracle_fp32_LossMeanSquaredError(float const *y, float const *t, float *dy, double *loss, int node_size, int frame_size, int frame_stride, float grad_reduction, double loss_reduction);
void oracle_fp32_MetricsMeanSquaredError(float const *y, float const *t, double *accuracy, int node_size, int frame_size, int frame_stride);
void oracle_fp32_RealToBinary_Forward(float const *x, float *y, int depth_modulation_size, int frame_modulation_size, float input_range_lo, float input_range_hi, int point_size, int x_depth_size, int x_frame_size, int x_frame_stride, int y_frame_stride, int binarize);
void oracle_bit_RealToBinary_Forward(float const *x, int *y, int depth_modulation_size, int frame_modulation_size, float input_range_lo, float input_range_hi, int point_size, int x_depth_size, int x_frame_size, int x_frame_stride, int y_frame_stride, int binarize);
void oracle_fp32_BinaryToReal_Forward(float const *x, float *y, int node_mux_size, int frame_mux_size, int y_node_size, int x_frame_stride, int y_frame_size, int y_frame_stride);
void oracle_fp32_BinaryToReal_Backward(float const *dy, float *dx, int node_mux_size, int frame_mux_size, int y_node_size, int x_frame_stride, int y_frame_size, int y_frame_stride);
void oracle_fp32_Binarize_Forward(float const *x, float *y, float binary_th, float binary_low, float binary_high, int node_size, int frame_size, int frame_stride);
void oracle_fp32_HardTanh_Forward(float const *x, float *y, float limit_min, float limit_max, int node_size, int frame_size, int frame_stride);
void oracle_fp32_HardTanh_Backward(float const *x, float const *dy, float *dx, float limit_min, float limit_max, int node_size, int frame_size, int frame_stride);
void oracle_fp32_MaxPooling_Forward(float const *x, float *y, int *argmax, int filter_h_size, int filter_w_size, int input_w_size, int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size, int frame_stride);
void oracle_fp32_MaxPooling_Backward(int const *argmax, float const *dy, float *dx, int filter_h_size, int filter_w_size, int input_w_size, int input_h_size, int output_w_size, int output_h_size, int c_size, int frame_size, int frame_stride);
void oracle_fp32_UpSampling_Forward(float const *x, float *y, int input_w_size, int input_h_size, int c_size, int filter_w_size, int filter_h_size, int fill, int frame_size, int frame_stride);
void oracle_fp32_UpSampling_Backward(float const *dy, float *dx, int input_w_size, int input_h_size, int c_size, int filter_w_size, int filter_h_size, int fill, int frame_size, int frame_stride);
void oracle_bit_BinaryLut6_Forward(std::int32_t const *x, std::int32_t *y, std::int32_t const *idx, std::int32_t const *table, int node_size, int frame_size, int frame_stride);
}

static int g_fail = 0;
#define CHECK(cond, ...) do { if (!(cond)) { ++g_fail; std::printf("FAIL %s:%d: ", __FILE__, __LINE__); std::printf(__VA_ARGS__); std::printf("\n"); } } while (0)

static double max_abs(std::vector<float> const &a) { double m = 0; for (float v : a) { m = std::max(m, (double)std::fabs(v)); } return m; }
static double max_diff(std::vector<float> const &a, std::vector<float> const &b) { double m = 0; for (size_t i = 0; i < a.size(); ++i) { m = std::max(m, (double)std::fabs(a[i] - b[i])); } return m; }

template <int N>
static void wire(std::mt19937_64 &mt, int I, int O, std::vector<std::int32_t> &idx)
{
    idx.resize((size_t)O * N);
    for (int o = 0; o < O; ++o) {
        for (int i = 0; i < N; ++i) {
            for (;;) {
                std::int32_t c = (std::int32_t)(mt() % (std::uint64_t)I);
                bool dup = false;
                for (int j = 0; j < i; ++j) { dup = dup || idx[(size_t)o * N + j] == c; }
                if (!dup) { idx[(size_t)o * N + i] = c; break; }
            }
        }
    }
}

static void read_fp32(bb::FrameBuffer &buf, std::vector<float> &out)
{
    auto p = buf.LockConst<float>();
    out.assign((size_t)(buf.GetNodeSize() * buf.GetFrameSize()), 0.0f);
    for (bb::index_t n = 0; n < buf.GetNodeSize(); ++n) for (bb::index_t f = 0; f < buf.GetFrameSize(); ++f) { out[(size_t)(n * buf.GetFrameSize() + f)] = p.Get(f, n); }
}

template <int N>
static void test_stochastic(int I, int O, int F, bool lut_binarize, bool binary)
{
    std::mt19937_64 mt(12345 + I + O + F);
    std::uniform_real_distribution<float> uni(-0.1f, 1.1f);
    std::normal_distribution<float> nrm(0.0f, 1.0f);
    constexpr int NN = 1 << N;

    auto lut = bb::StochasticLutN<N, float>::Create(O);
    lut->SendCommand(std::string("lut_binarize ") + (lut_binarize ? "true" : "false"));
    lut->SendCommand(std::string("binary ") + (binary ? "true" : "false"));
    bb::FrameBuffer x_buf(F, {I}, BB_TYPE_FP32);
    lut->SetInputShape(x_buf.GetShape());

    std::vector<std::int32_t> idx; wire<N>(mt, I, O, idx);
    for (int o = 0; o < O; ++o) for (int i = 0; i < N; ++i) { lut->SetNodeConnectionIndex(o, i, idx[(size_t)o * N + i]); }
    std::vector<float> W((size_t)O * NN), x((size_t)I * F), dy((size_t)O * F);
    // the layer gets table entries in [-0.1, 1.1]: Forward clamps them to [0, 1] in place first (reference: StochasticLutN.h:451),
    // so the oracle works on the clamped table and the layer's own table must equal it afterwards
    { auto Wp = lut->lock_W(); for (int o = 0; o < O; ++o) for (int i = 0; i < NN; ++i) { float const w = uni(mt); Wp(o, i) = w; W[(size_t)o * NN + i] = std::min(1.0f, std::max(0.0f, w)); } }
    { auto xp = x_buf.Lock<float>(true); for (int n = 0; n < I; ++n) for (int f = 0; f < F; ++f) { x[(size_t)n * F + f] = uni(mt); xp.Set(f, n, x[(size_t)n * F + f]); } }
    bb::FrameBuffer dy_buf(F, {O}, BB_TYPE_FP32);
    { auto dp = dy_buf.Lock<float>(true); for (int n = 0; n < O; ++n) for (int f = 0; f < F; ++f) { dy[(size_t)n * F + f] = nrm(mt); dp.Set(f, n, dy[(size_t)n * F + f]); } }

    for (int loop = 0; loop < 2; ++loop) {            // dW accumulates over the loops, as in the reference test
        auto y_buf = lut->Forward(x_buf);
        auto dx_buf = lut->Backward(dy_buf);
        std::vector<float> y, dx;
        read_fp32(y_buf, y); read_fp32(dx_buf, dx);
        std::vector<float> y_ref((size_t)O * F), dx_ref((size_t)I * F), dW_ref((size_t)O * NN, 0.0f);
        oracle_fp32_StochasticLut_Forward(N, x.data(), y_ref.data(), idx.data(), W.data(), O, F, F, binary, lut_binarize, 0.25f, 0);
        for (int l = 0; l <= loop; ++l) {
            oracle_fp32_StochasticLut_Backward(N, x.data(), dy.data(), dx_ref.data(), idx.data(), W.data(), dW_ref.data(), I, O, F, F, binary, lut_binarize, 0.25f, 0);
        }
        std::vector<float> dW((size_t)O * NN);
        { auto p = lut->lock_dW_const(); for (int o = 0; o < O; ++o) for (int i = 0; i < NN; ++i) { dW[(size_t)o * NN + i] = p(o, i); } }
        {
            auto Wp = lut->lock_W_const();
            size_t bad = 0;
            for (int o = 0; o < O; ++o) for (int i = 0; i < NN; ++i) { bad += (Wp(o, i) != W[(size_t)o * NN + i]); }
            CHECK(bad == 0, "StochasticLut%d: %zu table entries differ from the clamped table after Forward", N, bad);
        }
        CHECK(max_diff(y, y_ref) <= 1e-5, "StochasticLut%d %dx%dx%d y err %g", N, I, O, F, max_diff(y, y_ref));
        CHECK(max_diff(dx, dx_ref) <= 1e-4 * max_abs(dx_ref), "StochasticLut%d dx err %g", N, max_diff(dx, dx_ref));
        CHECK(max_diff(dW, dW_ref) <= 1e-4 * max_abs(dW_ref), "StochasticLut%d dW err %g (loop %d)", N, max_diff(dW, dW_ref), loop);
    }
    // ForwardNode agrees with the frame path on corner inputs
    {
        std::vector<double> v((size_t)N, 1.0);
        double r = lut->ForwardNode(0, v)[0];
        float w = W[(size_t)NN - 1]; if (lut_binarize) { w = w > 0.5f ? 1.0f : 0.0f; }
        if (!binary) { CHECK(std::fabs(r - w) < 1e-6, "ForwardNode corner value %g vs %g", r, (double)w); }
    }
    // host-only execution is refused, not emulated
    lut->SendCommand("host_only true");
    bool threw = false;
    try { lut->Forward(x_buf); } catch (bb::Exception const &) { threw = true; }
    CHECK(threw, "host_only forward must throw");
}

template <int N>
static void test_differentiable(int I, int O, int F, bool binary)
{
    std::mt19937_64 mt(777 + I + O + F);
    std::uniform_real_distribution<float> uni(0.0f, 1.0f);
    std::normal_distribution<float> nrm(0.0f, 1.0f);
    constexpr int NN = 1 << N;
    typename bb::DifferentiableLutN<N, float>::create_t cr;
    cr.output_shape = {O}; cr.binary = binary;
    auto lut = bb::DifferentiableLutN<N, float>::Create(cr);
    bb::FrameBuffer x_buf(F, {I}, BB_TYPE_FP32);
    lut->SetInputShape(x_buf.GetShape());
    std::vector<std::int32_t> idx; wire<N>(mt, I, O, idx);
    for (int o = 0; o < O; ++o) for (int i = 0; i < N; ++i) { lut->SetNodeConnectionIndex(o, i, idx[(size_t)o * N + i]); }
    std::vector<float> W((size_t)O * NN), x((size_t)I * F), dy((size_t)O * F);
    { auto Wp = lut->lock_W(); for (size_t k = 0; k < W.size(); ++k) { W[k] = uni(mt); Wp[(bb::index_t)k] = W[k]; } }
    { auto xp = x_buf.Lock<float>(true); for (int n = 0; n < I; ++n) for (int f = 0; f < F; ++f) { x[(size_t)n * F + f] = uni(mt); xp.Set(f, n, x[(size_t)n * F + f]); } }
    bb::FrameBuffer dy_buf(F, {O}, BB_TYPE_FP32);
    { auto dp = dy_buf.Lock<float>(true); for (int n = 0; n < O; ++n) for (int f = 0; f < F; ++f) { dy[(size_t)n * F + f] = nrm(mt); dp.Set(f, n, dy[(size_t)n * F + f]); } }

    auto y_buf = lut->Forward(x_buf, true);
    auto dx_buf = lut->Backward(dy_buf);
    std::vector<float> y, dx; read_fp32(y_buf, y); read_fp32(dx_buf, dx);
    std::vector<float> y_ref((size_t)O * F), mean((size_t)O), rstd((size_t)O), rm((size_t)O, 0.0f), rv((size_t)O, 1.0f), dx_ref((size_t)I * F), dW_ref((size_t)O * NN, 0.0f);
    oracle_fp32_DifferentiableLutN_ForwardTraining(N, x.data(), y_ref.data(), idx.data(), W.data(), mean.data(), rstd.data(), rm.data(), rv.data(), 0.3f, 0.5f, 0.9f, 0.25f, O, F, F, 0, binary);
    oracle_fp32_DifferentiableLutN_Backward(N, x.data(), dy.data(), dx_ref.data(), idx.data(), W.data(), dW_ref.data(), mean.data(), rstd.data(), 0.3f, 0.5f, 0.25f, I, O, F, F, 0, binary);
    std::vector<float> dW((size_t)O * NN), rm_gpu((size_t)O), rv_gpu((size_t)O), mean_gpu((size_t)O);
    { auto p = lut->lock_dW_const(); for (size_t k = 0; k < dW.size(); ++k) { dW[k] = p[(bb::index_t)k]; } }
    { auto a = lut->lock_mean_const(); auto b = lut->lock_var_const(); auto c = lut->lock_tmp_mean_const(); for (int o = 0; o < O; ++o) { rm_gpu[(size_t)o] = a[o]; rv_gpu[(size_t)o] = b[o]; mean_gpu[(size_t)o] = c[o]; } }
    if (binary) {
        size_t mism = 0; for (size_t k = 0; k < y.size(); ++k) { mism += (y[k] != y_ref[k]); }
        CHECK(mism <= 2 + y.size() / 10000, "DifferentiableLut%d binary y mismatches %zu of %zu", N, mism, y.size());
    }
    else {
        CHECK(max_diff(y, y_ref) <= 2e-4, "DifferentiableLut%d y err %g", N, max_diff(y, y_ref));
    }
    CHECK(max_diff(mean_gpu, mean) <= 1e-5, "batch mean err %g", max_diff(mean_gpu, mean));
    CHECK(max_diff(rm_gpu, rm) <= 1e-5 && max_diff(rv_gpu, rv) <= 1e-5, "running statistics err %g %g", max_diff(rm_gpu, rm), max_diff(rv_gpu, rv));
    CHECK(max_diff(dx, dx_ref) <= 1e-4 * max_abs(dx_ref), "DifferentiableLut%d dx err %g of %g", N, max_diff(dx, dx_ref), max_abs(dx_ref));
    CHECK(max_diff(dW, dW_ref) <= 1e-4 * max_abs(dW_ref), "DifferentiableLut%d dW err %g of %g", N, max_diff(dW, dW_ref), max_abs(dW_ref));
    // a frozen layer passes nothing back and holds no gradient of its own
    lut->SendCommand("backward_break true");
    lut->Forward(x_buf, true);
    bb::FrameBuffer none = lut->Backward(dy_buf);
    { auto p = lut->lock_dW_const(); for (size_t k = 0; k < dW.size(); ++k) { dW[k] = p[(bb::index_t)k]; } }
    CHECK(none.Empty() && max_abs(dW) == 0.0, "backward_break: the layer must return an empty buffer and zero its table gradient");
}

// Two DifferentiableLut6 layers in binary mode on fp32 frames: the first layer's forward call writes the packed copy of its binarized
// output beside it and the copy travels with the buffer (FrameBuffer::GetPackedTwin), so the second layer packs nothing, forward or
// backward.  A writable lock on the buffer in between makes the copy stale — the second layer then packs the values itself — and no
// output may differ by a bit between the two ways; a frozen layer keeps nothing from its forward passes.
static bool same_bits(bb::FrameBuffer &a, bb::FrameBuffer &b);
static void test_packed_twin(int I, int H, int O, int F)
{
    std::mt19937_64 mt(4242 + I + H + O + F);
    std::uniform_real_distribution<float> uni(0.0f, 1.0f);
    std::normal_distribution<float> nrm(0.0f, 1.0f);
    bb::FrameBuffer x_buf(F, {I}, BB_TYPE_FP32), dy_buf(F, {O}, BB_TYPE_FP32);
    { auto xp = x_buf.Lock<float>(true); for (int n = 0; n < I; ++n) for (int f = 0; f < F; ++f) { xp.Set(f, n, uni(mt)); } }
    { auto dp = dy_buf.Lock<float>(true); for (int n = 0; n < O; ++n) for (int f = 0; f < F; ++f) { dp.Set(f, n, nrm(mt)); } }
    std::vector<float> y[2], dx[2], dW1[2], dW2[2];
    for (int pass = 0; pass < 2; ++pass) {
        typename bb::DifferentiableLutN<6, float>::create_t c1, c2;
        c1.output_shape = {H}; c1.seed = 11; c2.output_shape = {O}; c2.seed = 12;
        auto l1 = bb::DifferentiableLutN<6, float>::Create(c1);
        auto l2 = bb::DifferentiableLutN<6, float>::Create(c2);
        l1->SetInputShape({I}); l2->SetInputShape({H});
        for (int step = 0; step < 2; ++step) {                 // (the second step runs with the table clamp inside the forward entry)
            bb::FrameBuffer h_buf = l1->Forward(x_buf, true);
            if (step == 0) {
                CHECK(!h_buf.GetPackedTwin().Empty(), "binary-mode layer on fp32 frames: the output carries no packed copy");
                bb::FrameBuffer copy = h_buf;                   // the copy travels with copies of the buffer
                CHECK(!copy.GetPackedTwin().Empty(), "the packed copy does not travel with a copy of the buffer");
            }
            if (pass == 1) {
                h_buf.LockDeviceMemory();                       // somebody may have written: the packed copy is no longer trusted
                CHECK(h_buf.GetPackedTwin().Empty(), "a writable lock must retire the packed copy");
            }
            bb::FrameBuffer y_buf = l2->Forward(h_buf, true);
            bb::FrameBuffer dh_buf = l2->Backward(dy_buf);
            bb::FrameBuffer dx_buf = l1->Backward(dh_buf);
            if (step == 1) {
                read_fp32(y_buf, y[pass]); read_fp32(dx_buf, dx[pass]);
                { auto p = l1->lock_dW_const(); dW1[pass].resize((size_t)H * 64); for (size_t k = 0; k < dW1[pass].size(); ++k) { dW1[pass][k] = p[(bb::index_t)k]; } }
                { auto p = l2->lock_dW_const(); dW2[pass].resize((size_t)O * 64); for (size_t k = 0; k < dW2[pass].size(); ++k) { dW2[pass][k] = p[(bb::index_t)k]; } }
            }
            else {
                // an optimizer step's worth of change, so that the clamp has something to do
                auto Wp = l1->lock_W(); for (bb::index_t k = 0; k < (bb::index_t)H * 64; k += 7) { Wp[k] = Wp[k] * 1.5f - 0.2f; }
            }
        }
        // inference takes the copy as well
        bb::FrameBuffer h_inf = l1->Forward(x_buf, false);
        CHECK(!h_inf.GetPackedTwin().Empty(), "inference output carries no packed copy");
        bb::FrameBuffer y_a = l2->Forward(h_inf, false);
        h_inf.LockDeviceMemory();
        bb::FrameBuffer y_b = l2->Forward(h_inf, false);
        CHECK(same_bits(y_a, y_b), "inference: output differs with and without the packed copy");
    }
    CHECK(y[0] == y[1] && dx[0] == dx[1] && dW1[0] == dW1[1] && dW2[0] == dW2[1], "results differ with and without the packed copy of the hidden layer");
}

static void test_binary(int I, int O, int F)
{
    std::mt19937_64 mt(99 + I + O + F);
    auto lut = bb::BinaryLutN<6, bb::Bit>::Create(O);
    bb::FrameBuffer x_buf(F, {I}, BB_TYPE_BIT);
    lut->SetInputShape(x_buf.GetShape());
    int const words = (F + 31) / 32;
    std::vector<std::int32_t> idx((size_t)O * 6), table((size_t)O * 2), x((size_t)I * words, 0), y_ref((size_t)O * words, 0);
    for (int o = 0; o < O; ++o) {
        for (int i = 0; i < 6; ++i) { idx[(size_t)o * 6 + i] = (std::int32_t)lut->GetNodeConnectionIndex(o, i); }
        for (int b = 0; b < 64; ++b) { if (lut->GetLutTable(o, b)) { table[(size_t)o * 2 + b / 32] |= (std::int32_t)(1u << (b % 32)); } }
    }
    { auto xp = x_buf.Lock<bb::Bit>(true); for (int n = 0; n < I; ++n) for (int f = 0; f < F; ++f) { bool b = (mt() & 1) != 0; xp.Set(f, n, bb::Bit(b)); if (b) { x[(size_t)n * words + f / 32] |= (std::int32_t)(1u << (f % 32)); } } }
    auto y_buf = lut->Forward(x_buf);
    oracle_bit_BinaryLut6_Forward(x.data(), y_ref.data(), idx.data(), table.data(), O, F, words);
    auto yp = y_buf.LockConst<bb::Bit>();
    size_t mism = 0;
    for (int n = 0; n < O; ++n) for (int f = 0; f < F; ++f) { mism += ((bool)yp.Get(f, n) != (((std::uint32_t)y_ref[(size_t)n * words + f / 32] >> (f % 32)) & 1u)); }
    CHECK(mism == 0, "BinaryLut6 %dx%dx%d: %zu mismatching bits", I, O, F, mism);
}

// trained-layer hand-off at every width: a StochasticLut<N> with binarized tables tabulated into a BinaryLut<N> gives the same bits,
// and the tabulated layer survives a trip through a stream under its own type name
template <int N>
static void test_import_layer(void)
{
    int const I = 32, O = 24, F = 200;
    std::mt19937_64 mt(5 + N);
    std::uniform_real_distribution<float> uni(0.0f, 1.0f);
    auto src = bb::StochasticLutN<N, bb::Bit>::Create(O);
    src->SendCommand("lut_binarize true");
    bb::FrameBuffer x_buf(F, {I}, BB_TYPE_BIT);
    src->SetInputShape(x_buf.GetShape());
    { auto Wp = src->lock_W(); for (int k = 0; k < O * (1 << N); ++k) { Wp[k] = uni(mt); } }
    { auto xp = x_buf.Lock<bb::Bit>(true); for (int n = 0; n < I; ++n) for (int f = 0; f < F; ++f) { xp.Set(f, n, bb::Bit((mt() & 1) != 0)); } }
    auto dst = bb::BinaryLutN<N, bb::Bit>::Create(O);
    dst->SetInputShape(x_buf.GetShape());
    CHECK(dst->GetLutTableSize(0) == (1 << N) && dst->GetNodeConnectionSize(0) == N, "BinaryLut%d: table size and fan-in", N);
    dst->ImportLayer(src);
    auto y_src = src->Forward(x_buf, false);          // fp32 in [0,1]; with binarized tables and bits at 0.5+-0.25 it is > 0.5 iff the table bit is 1
    auto y_dst = dst->Forward(x_buf);
    {
        auto a = y_src.template LockConst<float>(); auto b = y_dst.template LockConst<bb::Bit>();
        size_t mism = 0;
        for (int n = 0; n < O; ++n) for (int f = 0; f < F; ++f) { mism += ((a.Get(f, n) > 0.5f) != (bool)b.Get(f, n)); }
        CHECK(mism == 0, "ImportLayer<%d>: %zu mismatching bits", N, mism);
    }
    std::stringstream ss;
    dst->DumpObject(ss);
    auto again = std::dynamic_pointer_cast<bb::BinaryLutN<N, bb::Bit>>(bb::Object_Load(ss));
    CHECK((bool)again && again->GetObjectName() == "BinaryLut" + std::to_string(N) + "_bit_fp32", "BinaryLut%d does not come back from a stream", N);
    if (again) {
        auto y_again = again->Forward(x_buf);
        auto a = y_dst.template LockConst<bb::Bit>(); auto b = y_again.template LockConst<bb::Bit>();
        size_t mism = 0;
        for (int n = 0; n < O; ++n) for (int f = 0; f < F; ++f) { mism += ((bool)a.Get(f, n) != (bool)b.Get(f, n)); }
        CHECK(mism == 0, "BinaryLut%d: output differs after a trip through a stream (%zu bits)", N, mism);
    }
}

// Shaped like the reference's optimizer test (tests/gtest/OptimizerAdamTest.cpp:44-96): parameters follow a model of the
// update step by step; here the model is the CPU oracle and the list holds several tensors of different sizes.
static void test_adam(void)
{
    float const lr = 0.001f, beta1 = 0.9f, beta2 = 0.999f;
    int const sizes[] = {1, 70 * 64, 1024 * 64, 5};
    auto opt = bb::OptimizerAdam<float>::Create(lr, beta1, beta2);
    std::vector<std::shared_ptr<bb::Tensor>> params, grads;
    bb::Variables pv, gv;
    std::mt19937_64 mt(1);
    std::normal_distribution<float> norm(0.0001f, 2.0f);
    std::vector<std::vector<float>> p_ref, m_ref, v_ref;
    for (int n : sizes) {
        auto p = std::make_shared<bb::Tensor>(bb::indices_t({(bb::index_t)n}), BB_TYPE_FP32);
        auto g = std::make_shared<bb::Tensor>(bb::indices_t({(bb::index_t)n}), BB_TYPE_FP32);
        std::vector<float> init((size_t)n);
        { auto ptr = p->Lock<float>(true); for (int i = 0; i < n; ++i) { init[(size_t)i] = ptr[i] = 0.1f + 0.001f * (float)(i % 97); } }
        g->FillZero();
        params.push_back(p); grads.push_back(g); pv.PushBack(p); gv.PushBack(g);
        p_ref.push_back(init); m_ref.emplace_back((size_t)n, 0.0f); v_ref.emplace_back((size_t)n, 0.0f);
    }
    opt->SetVariables(pv, gv);
    float b1 = beta1, b2 = beta2;
    for (int step = 0; step < 10; ++step) {
        float const lr_t = lr * std::sqrt(1.0f - b2) / (1.0f - b1);
        for (size_t t = 0; t < params.size(); ++t) {
            int const n = sizes[t];
            std::vector<float> g((size_t)n);
            for (auto &x : g) { x = norm(mt); }
            { auto ptr = grads[t]->Lock<float>(true); for (int i = 0; i < n; ++i) { ptr[i] = g[(size_t)i]; } }
            oracle_fp32_OptimizerAdam(n, p_ref[t].data(), g.data(), m_ref[t].data(), v_ref[t].data(), lr_t, beta1, beta2);
        }
        opt->Update();
        b1 *= beta1; b2 *= beta2;
        for (size_t t = 0; t < params.size(); ++t) {
            auto ptr = params[t]->LockConst<float>();
            size_t bad = 0;
            for (int i = 0; i < sizes[t]; ++i) { bad += (ptr[i] != p_ref[t][(size_t)i]); }
            CHECK(bad == 0, "Adam step %d tensor %zu: %zu of %d parameters differ from the oracle", step, t, bad, sizes[t]);
            auto gp = grads[t]->LockConst<float>();
            CHECK(gp[0] == 0.0f && gp[sizes[t] - 1] == 0.0f, "Update must clear the gradients");
        }
    }
}

// The reference's Im2Col test (tests/gtest/ConvolutionIm2ColTest.cpp:19-190): 2 frames of {2, 3, 4} images whose pixels
// encode their own coordinates, filter 2 x 3; then a conv block Im2Col -> Col2Im -> pooling against the oracle.
static void test_conv_plumbing(void)
{
    auto im2col = bb::ConvolutionIm2Col<>::Create(2, 3);
    bb::FrameBuffer x(2, {2, 3, 4}, BB_TYPE_FP32);
    for (int f = 0; f < 2; ++f) for (int c = 0; c < 2; ++c) for (int y = 0; y < 3; ++y) for (int xx = 0; xx < 4; ++xx) {
        x.SetFP32(f, (c * 3 + y) * 4 + xx, (float)(1000 * f + 100 * c + 10 * y + xx));
    }
    bb::FrameBuffer y = im2col->Forward(x);
    CHECK(y.GetFrameSize() == 8 && y.GetNodeSize() == 12, "Im2Col output %d frames x %d nodes", (int)y.GetFrameSize(), (int)y.GetNodeSize());
    int const base[8] = {0, 1, 10, 11, 1000, 1001, 1010, 1011};
    size_t bad = 0;
    for (int of = 0; of < 8; ++of) for (int c = 0; c < 2; ++c) for (int fy = 0; fy < 2; ++fy) for (int fx = 0; fx < 3; ++fx) {
        bad += (y.GetFP32(of, (c * 2 + fy) * 3 + fx) != (float)(base[of] + 100 * c + 10 * fy + fx));
    }
    CHECK(bad == 0, "Im2Col known answers: %zu wrong", bad);
    bb::FrameBuffer dy(8, {2, 2, 3}, BB_TYPE_FP32);
    std::vector<float> dyv(12 * 8);
    for (int of = 0; of < 8; ++of) for (int n = 0; n < 12; ++n) { dyv[(size_t)n * 8 + of] = (float)(1000 * of + n); dy.SetFP32(of, n, dyv[(size_t)n * 8 + of]); }
    bb::FrameBuffer dx = im2col->Backward(dy);
    std::vector<float> dx_ref(24 * 2);
    oracle_fp32_Im2Col_Backward(dyv.data(), dx_ref.data(), 1, 1, 0, 0, 2, 2, 4, 3, 2, 2, 2, 8, 3, 2);
    bad = 0;
    for (int f = 0; f < 2; ++f) for (int n = 0; n < 24; ++n) { bad += (dx.GetFP32(f, n) != dx_ref[(size_t)n * 2 + f]); }
    CHECK(bad == 0, "Im2Col backward: %zu wrong", bad);

    // 1 x 1 Im2Col and Col2Im invert each other; pooling against the oracle
    int const C = 3, H = 5, W = 7, F = 70;
    std::mt19937_64 mt(5);
    std::uniform_real_distribution<float> uni(0.0f, 1.0f);
    bb::FrameBuffer img(F, {C, H, W}, BB_TYPE_FP32);
    std::vector<float> dense((size_t)C * H * W * F);
    for (int n = 0; n < C * H * W; ++n) for (int f = 0; f < F; ++f) { dense[(size_t)n * F + f] = uni(mt); img.SetFP32(f, n, dense[(size_t)n * F + f]); }
    auto one = bb::ConvolutionIm2Col<>::Create(1, 1);
    auto col2im = bb::ConvolutionCol2Im<>::Create(H, W);
    bb::FrameBuffer back = col2im->Forward(one->Forward(img));
    bad = 0;
    for (int n = 0; n < C * H * W; ++n) for (int f = 0; f < F; ++f) { bad += (back.GetFP32(f, n) != dense[(size_t)n * F + f]); }
    CHECK(bad == 0 && back.GetShape() == bb::indices_t({C, H, W}), "Im2Col(1x1) -> Col2Im round trip: %zu wrong", bad);
    auto pool = bb::StochasticMaxPooling2x2<>::Create();
    bb::FrameBuffer py = pool->Forward(img);
    int const OH = 3, OW = 4;
    std::vector<float> py_ref((size_t)C * OH * OW * F), pdy((size_t)C * OH * OW * F), pdx_ref(dense.size());
    oracle_fp32_StochasticMaxPooling2x2_Forward(dense.data(), py_ref.data(), W, H, OW, OH, C, F, F);
    bb::FrameBuffer pdy_buf(F, {C, OH, OW}, BB_TYPE_FP32);
    bad = 0;
    for (int n = 0; n < C * OH * OW; ++n) for (int f = 0; f < F; ++f) {
        bad += (py.GetFP32(f, n) != py_ref[(size_t)n * F + f]);
        pdy[(size_t)n * F + f] = uni(mt) - 0.5f; pdy_buf.SetFP32(f, n, pdy[(size_t)n * F + f]);
    }
    CHECK(bad == 0, "StochasticMaxPooling2x2 forward: %zu wrong", bad);
    bb::FrameBuffer pdx = pool->Backward(pdy_buf);
    oracle_fp32_StochasticMaxPooling2x2_Backward(dense.data(), pdy.data(), pdx_ref.data(), W, H, OW, OH, C, F, F);
    bad = 0;
    for (int n = 0; n < C * H * W; ++n) for (int f = 0; f < F; ++f) { bad += (pdx.GetFP32(f, n) != pdx_ref[(size_t)n * F + f]); }
    CHECK(bad == 0, "StochasticMaxPooling2x2 backward: %zu wrong", bad);
}

// The convolution wrapper (reference: include/bb/Convolution2d.h:278-309): Convolution2d over a list of two DifferentiableLut6
// layers gives, bit for bit, what Im2Col -> layer -> layer -> Col2Im give when called one by one on copies of the same layers
// (forward, backward down to the image gradient, table gradients); its shapes, parameter list and a trip through a stream.
static bool same_bits(bb::FrameBuffer &a, bb::FrameBuffer &b)
{
    if (a.GetShape() != b.GetShape() || a.GetFrameSize() != b.GetFrameSize()) { return false; }
    std::vector<float> va, vb;
    read_fp32(a, va); read_fp32(b, vb);
    return std::memcmp(va.data(), vb.data(), va.size() * sizeof(float)) == 0;
}

static void test_convolution2d(void)
{
    int const C = 3, H = 8, W = 9, F = 5, O1 = 24, O2 = 8, OH = 6, OW = 7;
    auto lut1 = bb::DifferentiableLutN<6, float>::Create(O1);
    auto lut2 = bb::DifferentiableLutN<6, float>::Create(O2);
    auto body = bb::Sequential::Create();
    body->Add(lut1); body->Add(lut2);
    auto conv = bb::Convolution2d<>::Create(body, 3, 3);
    bb::indices_t const out_shape = conv->SetInputShape({C, H, W});
    CHECK(out_shape == bb::indices_t({O2, OH, OW}) && conv->GetOutputShape() == out_shape && conv->GetInputShape() == bb::indices_t({C, H, W}),
          "Convolution2d shapes");
    CHECK(lut1->GetInputShape() == bb::indices_t({C, 3, 3}) && lut2->GetInputNodeSize() == O1, "Convolution2d hands the shapes through");
    CHECK(conv->GetParameters().GetSize() == lut1->GetParameters().GetSize() + lut2->GetParameters().GetSize() &&
          conv->GetGradients().GetSize() == conv->GetParameters().GetSize(), "Convolution2d parameter list");

    // copies of the two layers through their serialized form, and the plumbing by hand
    auto copy_of = [](std::shared_ptr<bb::Model> const &m) {
        std::stringstream ss(std::ios::in | std::ios::out | std::ios::binary);
        m->DumpObject(ss);
        return std::dynamic_pointer_cast<bb::Model>(bb::Object_Load(ss));
    };
    auto lut1b = copy_of(lut1), lut2b = copy_of(lut2);
    auto im2col = bb::ConvolutionIm2Col<>::Create(3, 3);
    auto col2im = bb::ConvolutionCol2Im<>::Create(OH, OW);

    std::mt19937_64 mt(77);
    std::uniform_real_distribution<float> uni(0.0f, 1.0f);
    bb::FrameBuffer x(F, {C, H, W}, BB_TYPE_FP32), dy(F, {O2, OH, OW}, BB_TYPE_FP32);
    for (int n = 0; n < C * H * W; ++n) for (int f = 0; f < F; ++f) { x.SetFP32(f, n, uni(mt)); }
    for (int n = 0; n < O2 * OH * OW; ++n) for (int f = 0; f < F; ++f) { dy.SetFP32(f, n, uni(mt) - 0.5f); }

    bb::FrameBuffer y = conv->Forward(x);
    bb::FrameBuffer dx = conv->Backward(dy);
    bb::FrameBuffer a = im2col->Forward(x);
    col2im->SetInputShape(lut2b->SetInputShape(lut1b->SetInputShape(a.GetShape())));
    bb::FrameBuffer y2 = col2im->Forward(lut2b->Forward(lut1b->Forward(a)));
    bb::FrameBuffer dx2 = im2col->Backward(lut1b->Backward(lut2b->Backward(col2im->Backward(dy))));
    CHECK(y.GetShape() == out_shape && y.GetFrameSize() == F, "Convolution2d output %d frames", (int)y.GetFrameSize());
    CHECK(same_bits(y, y2), "Convolution2d forward differs from the layers called one by one");
    CHECK(same_bits(dx, dx2), "Convolution2d backward differs from the layers called one by one");
    {
        auto g = conv->GetGradients(), gb1 = lut1b->GetGradients(), gb2 = lut2b->GetGradients();
        auto p = g[0].LockConst<float>(); auto q = gb1[0].LockConst<float>();
        size_t bad = 0;
        for (bb::index_t i = 0; i < g[0].GetSize(); ++i) { bad += (p[i] != q[i]); }
        auto p2 = g[g.GetSize() / 2].LockConst<float>(); auto q2 = gb2[0].LockConst<float>();
        for (bb::index_t i = 0; i < gb2[0].GetSize(); ++i) { bad += (p2[i] != q2[i]); }
        CHECK(bad == 0, "Convolution2d table gradients: %zu differ", bad);
    }
    // through a stream: the rebuilt wrapper (layers rebuilt from their type names) computes the same output
    {
        std::stringstream ss(std::ios::in | std::ios::out | std::ios::binary);
        conv->DumpObject(ss);
        auto again = std::dynamic_pointer_cast<bb::Model>(bb::Object_Load(ss));
        CHECK((bool)again && again->GetObjectName() == "Convolution2d_fp32_fp32", "Convolution2d reload");
        if (again) {
            bb::FrameBuffer y3 = again->Forward(x, false), y4 = conv->Forward(x, false);
            CHECK(same_bits(y3, y4), "reloaded Convolution2d differs in inference");
        }
    }
}

// The tail of a classifier through the host classes: AverageLut against the oracle, and the reference's own known-answer test
// of the loss (tests/gtest/LossSoftmaxCrossEntropyTest.cpp:8-92, NumPy goldens: loss within 1e-4, dy within 1e-6).
// StochasticBatchNormalization: two training passes (the running statistics move twice), backward, the pass repeated from the
// stored statistics, inference, the gain / offset form of inference, and a round trip through a stream
static void test_stochastic_batch_normalization(void)
{
    int const C = 5, H = 3, W = 4, NODES = C * H * W, F = 200;
    float const momentum = 0.8f, gamma = 0.25f, beta = 0.5f;
    auto bn = bb::StochasticBatchNormalization<>::Create(momentum, gamma, beta);
    CHECK(bn->SetInputShape({C, H, W}) == bb::indices_t({C, H, W}) && bn->GetOutputNodeSize() == NODES, "normalisation shapes");
    CHECK(bn->GetParameters().GetSize() == 0 && bn->GetGradients().GetSize() == 0, "normalisation has no trained parameters");
    std::mt19937_64 mt(5);
    std::uniform_real_distribution<float> uni(0.0f, 1.0f);
    std::vector<float> rm((size_t)NODES, 0.0f), rv((size_t)NODES, 1.0f), mean((size_t)NODES), rstd((size_t)NODES);
    std::vector<float> x, y, dy, dx, y_ref((size_t)NODES * F), dx_ref((size_t)NODES * F);
    bb::FrameBuffer x_buf(F, {C, H, W}, BB_TYPE_FP32), dy_buf(F, {C, H, W}, BB_TYPE_FP32);
    for (int pass = 0; pass < 2; ++pass) {
        for (int n = 0; n < NODES; ++n) for (int f = 0; f < F; ++f) { x_buf.SetFP32(f, n, uni(mt) * (0.2f + 0.1f * (float)(n % 7))); dy_buf.SetFP32(f, n, uni(mt) - 0.5f); }
        read_fp32(x_buf, x); read_fp32(dy_buf, dy);
        bb::FrameBuffer y_buf = bn->Forward(x_buf, true);
        read_fp32(y_buf, y);
        oracle_fp32_StochasticBatchNormalization_ForwardTraining(x.data(), y_ref.data(), mean.data(), rstd.data(), rm.data(), rv.data(), gamma, beta, momentum, NODES, F, F);
        CHECK(max_diff(y, y_ref) <= 2e-6 * (1.0 + max_abs(y_ref)) * 4, "normalisation y err %g (pass %d)", max_diff(y, y_ref), pass);
        {
            auto pm = bn->lock_mean_const(); auto pv = bn->lock_var_const(); auto bm = bn->lock_tmp_mean_const(); auto br = bn->lock_tmp_rstd_const();
            double e = 0;
            for (int n = 0; n < NODES; ++n) {
                e = std::max(e, (double)std::fabs(pm[n] - rm[n])); e = std::max(e, (double)std::fabs(pv[n] - rv[n]));
                e = std::max(e, (double)std::fabs(bm[n] - mean[n])); e = std::max(e, (double)std::fabs(br[n] - rstd[n]) / rstd[n]);
            }
            CHECK(e <= 5e-6, "normalisation statistics err %g (pass %d)", e, pass);
        }
        // the pass again from the stored statistics pushes the input a second time: two backward passes follow
        bb::FrameBuffer y2_buf = bn->ReForward(x_buf);
        CHECK(same_bits(y_buf, y2_buf), "normalisation: the repeated pass differs");
        bb::FrameBuffer dx_buf = bn->Backward(dy_buf);
        bb::FrameBuffer dx2_buf = bn->Backward(dy_buf);
        CHECK(same_bits(dx_buf, dx2_buf), "normalisation: the two backward passes differ");
        read_fp32(dx_buf, dx);
        {
            std::vector<float> bmean((size_t)NODES), brstd((size_t)NODES);
            auto bm = bn->lock_tmp_mean_const(); auto br = bn->lock_tmp_rstd_const();
            for (int n = 0; n < NODES; ++n) { bmean[(size_t)n] = bm[n]; brstd[(size_t)n] = br[n]; }
            oracle_fp32_StochasticBatchNormalization_Backward(x.data(), dy.data(), dx_ref.data(), bmean.data(), brstd.data(), gamma, NODES, F, F, F);
        }
        CHECK(max_diff(dx, dx_ref) <= 1e-5 * max_abs(dx_ref), "normalisation dx err %g of %g", max_diff(dx, dx_ref), max_abs(dx_ref));
    }
    // inference from the running statistics, also as gain * x + offset and node by node
    bb::FrameBuffer yi_buf = bn->Forward(x_buf, false);
    read_fp32(yi_buf, y);
    oracle_fp32_StochasticBatchNormalization_ForwardInference(x.data(), y_ref.data(), rm.data(), rv.data(), gamma, beta, NODES, F, F);
    CHECK(max_diff(y, y_ref) <= 1e-5, "normalisation inference err %g", max_diff(y, y_ref));
    {
        double e = 0;
        for (int n = 0; n < NODES; n += 7) {
            double const v = (double)x[(size_t)n * F + 3];
            e = std::max(e, std::fabs((double)bn->GetNormalizeGain(n) * v + (double)bn->GetNormalizeOffset(n) - (double)y[(size_t)n * F + 3]));
            e = std::max(e, std::fabs(bn->ForwardNode(n, {v})[0] - (double)y[(size_t)n * F + 3]));
        }
        CHECK(e <= 1e-5, "normalisation gain / offset / ForwardNode err %g", e);
    }
    // through a stream, rebuilt from the type name: the same inference output, bit for bit
    {
        std::stringstream ss(std::ios::in | std::ios::out | std::ios::binary);
        bn->DumpObject(ss);
        auto again = std::dynamic_pointer_cast<bb::Model>(bb::Object_Load(ss));
        CHECK((bool)again && again->GetObjectName() == "StochasticBatchNormalization_fp32" && again->GetInputShape() == bb::indices_t({C, H, W}), "normalisation reload");
        if (again) {
            bb::FrameBuffer y3 = again->Forward(x_buf, false);
            CHECK(same_bits(y3, yi_buf), "reloaded normalisation differs in inference");
        }
    }
    // commands: gamma and beta can be changed; host-only execution is refused, not emulated
    bn->SendCommand("set_gamma 0.5");
    bn->SendCommand("set_beta 0.25");
    CHECK(bn->GetGamma() == 0.5f && bn->GetBeta() == 0.25f, "set_gamma / set_beta");
    bn->SendCommand("host_only true");
    bool threw = false;
    try { bn->Forward(x_buf); } catch (std::exception const &) { threw = true; }
    CHECK(threw, "host_only normalisation must throw");
}

// MaxLut: the known answers of the reference's own test on packed bits (tests/gtest/MaxLutTest.cpp:15-139), then a wired fp32
// layer against the oracle, bit for bit, and a trip through a stream
static void test_max_lut(void)
{
    {
        auto lut = bb::MaxLut<bb::Bit>::Create(6, bb::indices_t({2}), "serial");
        bb::FrameBuffer x(3, {2, 6}, BB_TYPE_BIT);
        lut->SetInputShape(x.GetShape());
        for (int f = 0; f < 3; ++f) for (int n = 0; n < 12; ++n) { x.SetBit(f, n, false); }
        x.SetBit(0, 2, true);
        x.SetBit(1, 1, true); x.SetBit(1, 5, true); x.SetBit(1, 11, true);
        x.SetBit(2, 6, true);
        bb::FrameBuffer y = lut->Forward(x);
        bool const want_y[2][3] = {{true, true, false}, {false, true, true}};
        for (int n = 0; n < 2; ++n) for (int f = 0; f < 3; ++f) { CHECK(y.GetBit(f, n) == want_y[n][f], "MaxLut bits y(%d, %d)", f, n); }
        bb::FrameBuffer dy(3, {2}, BB_TYPE_FP32);
        float const g[2][3] = {{0.1f, 0.2f, 0.3f}, {0.4f, 0.5f, 0.6f}};
        for (int n = 0; n < 2; ++n) for (int f = 0; f < 3; ++f) { dy.SetFP32(f, n, g[n][f]); }
        bb::FrameBuffer dx = lut->Backward(dy);
        int const winner[2][3] = {{2, 1, 0}, {6, 11, 6}};       // the set input, the first of two set inputs, input 0 of the node when none is set
        for (int n = 0; n < 12; ++n) for (int f = 0; f < 3; ++f) {
            float const want = (winner[n / 6][f] == n) ? g[n / 6][f] : 0.0f;
            CHECK(dx.GetFP32(f, n) == want, "MaxLut bits dx(%d, %d) = %g, want %g", f, n, (double)dx.GetFP32(f, n), (double)want);
        }
    }
    int const N = 5, I = 60, O = 24, F = 150;
    auto lut = bb::MaxLut<float>::Create(N, bb::indices_t({O}), "random", false);
    bb::FrameBuffer x_buf(F, {I}, BB_TYPE_FP32), dy_buf(F, {O}, BB_TYPE_FP32);
    lut->SetInputShape(x_buf.GetShape());
    std::vector<std::int32_t> idx((size_t)O * N);
    {
        std::vector<int> uses((size_t)I, 0);
        for (int o = 0; o < O; ++o) for (int i = 0; i < N; ++i) {
            idx[(size_t)o * N + i] = (std::int32_t)lut->GetNodeConnectionIndex(o, i);
            uses[(size_t)idx[(size_t)o * N + i]] += 1;
        }
        int lo = 1 << 30, hi = 0;
        for (int u : uses) { lo = std::min(lo, u); hi = std::max(hi, u); }
        CHECK(hi - lo <= 1, "MaxLut random wiring uses the inputs %d to %d times", lo, hi);      // dealt from shuffled decks
    }
    std::mt19937_64 mt(9);
    std::uniform_real_distribution<float> uni(-2.0f, 1.0f);
    for (int n = 0; n < I; ++n) for (int f = 0; f < F; ++f) { x_buf.SetFP32(f, n, (f % 5 == 0) ? std::round(uni(mt)) : uni(mt)); }
    for (int n = 0; n < O; ++n) for (int f = 0; f < F; ++f) { dy_buf.SetFP32(f, n, uni(mt)); }
    std::vector<float> x, dy, y, dx, y_ref((size_t)O * F), dx_ref((size_t)I * F);
    read_fp32(x_buf, x); read_fp32(dy_buf, dy);
    bb::FrameBuffer y_buf = lut->Forward(x_buf);
    bb::FrameBuffer dx_buf = lut->Backward(dy_buf);
    read_fp32(y_buf, y); read_fp32(dx_buf, dx);
    oracle_fp32_MaxLut_Forward(x.data(), y_ref.data(), idx.data(), N, O, F, F, 0, 0);
    oracle_fp32_MaxLut_Backward(x.data(), dy.data(), dx_ref.data(), idx.data(), N, I, O, F, F, 0);
    CHECK(max_diff(y, y_ref) == 0.0, "MaxLut y differs by %g", max_diff(y, y_ref));
    CHECK(max_diff(dx, dx_ref) == 0.0, "MaxLut dx differs by %g", max_diff(dx, dx_ref));
    lut->SendCommand("binarize_output true");
    bb::FrameBuffer yb_buf = lut->Forward(x_buf, false);
    read_fp32(yb_buf, y);
    oracle_fp32_MaxLut_Forward(x.data(), y_ref.data(), idx.data(), N, O, F, F, 0, 1);
    CHECK(max_diff(y, y_ref) == 0.0, "MaxLut binarized y differs by %g", max_diff(y, y_ref));
    {
        std::stringstream ss(std::ios::in | std::ios::out | std::ios::binary);
        lut->DumpObject(ss);
        auto again = std::dynamic_pointer_cast<bb::Model>(bb::Object_Load(ss));
        CHECK((bool)again && again->GetObjectName() == "MaxLut_fp32_fp32" && again->GetOutputNodeSize() == O, "MaxLut reload");
        if (again) {
            bb::FrameBuffer y3 = again->Forward(x_buf, false);
            CHECK(same_bits(y3, yb_buf), "reloaded MaxLut differs");
        }
    }
    lut->SendCommand("host_only true");
    bool threw = false;
    try { lut->Forward(x_buf); } catch (bb::Exception const &) { threw = true; }
    CHECK(threw, "host_only MaxLut must throw");
}

// Reduce (output shape given, and derived from an integration size), then the mean-squared-error loss and metric over two batches
static void test_reduce_and_mean_squared_error(void)
{
    int const I = 70, O = 10, F = 90;
    std::mt19937_64 mt(17);
    std::uniform_real_distribution<float> uni(0.0f, 1.0f);
    auto fold = bb::Reduce<>::Create((bb::index_t)O);
    auto fold7 = bb::Reduce<>::Create(bb::indices_t(), 7);
    bb::FrameBuffer x_buf(F, {I}, BB_TYPE_FP32), dy_buf(F, {O}, BB_TYPE_FP32), t_buf(F, {O}, BB_TYPE_FP32);
    CHECK(fold->SetInputShape({I}) == bb::indices_t({O}) && fold7->SetInputShape({I}) == bb::indices_t({O}), "Reduce shapes");
    auto loss = bb::LossMeanSquaredError<>::Create();
    auto metric = bb::MetricsMeanSquaredError<>::Create();
    double loss_ref = 0, metric_ref = 0;
    std::vector<float> x, y, dy, dx, t, g, y_ref((size_t)O * F), dx_ref((size_t)I * F), g_ref((size_t)O * F);
    for (int batch = 0; batch < 2; ++batch) {
        for (int n = 0; n < I; ++n) for (int f = 0; f < F; ++f) { x_buf.SetFP32(f, n, uni(mt)); }
        for (int n = 0; n < O; ++n) for (int f = 0; f < F; ++f) { dy_buf.SetFP32(f, n, uni(mt) - 0.5f); t_buf.SetFP32(f, n, (uni(mt) > 0.5f) ? 1.0f : 0.0f); }
        read_fp32(x_buf, x); read_fp32(dy_buf, dy); read_fp32(t_buf, t);
        bb::FrameBuffer y_buf = fold->Forward(x_buf);
        bb::FrameBuffer y7_buf = fold7->Forward(x_buf);
        bb::FrameBuffer dx_buf = fold->Backward(dy_buf);
        read_fp32(y_buf, y); read_fp32(dx_buf, dx);
        oracle_fp32_Reduce_Forward(x.data(), y_ref.data(), I, O, F, F);
        oracle_fp32_Reduce_Backward(dy.data(), dx_ref.data(), I, O, F, F);
        CHECK(max_diff(y, y_ref) == 0.0 && same_bits(y_buf, y7_buf), "Reduce forward differs by %g", max_diff(y, y_ref));
        CHECK(max_diff(dx, dx_ref) == 0.0, "Reduce backward differs by %g", max_diff(dx, dx_ref));
        bb::FrameBuffer g_buf = loss->CalculateLoss(y_buf, t_buf, F);
        metric->CalculateMetrics(y_buf, t_buf);
        read_fp32(g_buf, g);
        oracle_fp32_LossMeanSquaredError(y.data(), t.data(), g_ref.data(), &loss_ref, O, F, F, 1.0f / (float)(O * F), 1.0 / O);
        oracle_fp32_MetricsMeanSquaredError(y.data(), t.data(), &metric_ref, O, F, F);
        CHECK(max_diff(g, g_ref) == 0.0, "mean squared error gradient differs by %g", max_diff(g, g_ref));
    }
    double const want_loss = loss_ref / (2.0 * F), want_metric = metric_ref / (2.0 * F);
    CHECK(std::fabs(loss->GetLoss() - want_loss) <= 1e-12 * want_loss, "mean squared error loss %.17g vs %.17g", loss->GetLoss(), want_loss);
    CHECK(std::fabs(metric->GetMetrics() - want_metric) <= 1e-12 * want_metric, "mean squared error metric %.17g vs %.17g", metric->GetMetrics(), want_metric);
    loss->Clear(); metric->Clear();
    auto sum_loss = bb::LossMeanSquaredError<>::Create("sum");
    bb::FrameBuffer y_buf = fold->Forward(x_buf);
    sum_loss->CalculateLoss(y_buf, t_buf, F);
    double sum_ref = 0;
    oracle_fp32_LossMeanSquaredError(y.data(), t.data(), g_ref.data(), &sum_ref, O, F, F, 1.0f, 1.0);
    CHECK(std::fabs(sum_loss->GetLoss() - sum_ref) <= 1e-12 * sum_ref, "summed squared error %.17g vs %.17g", sum_loss->GetLoss(), sum_ref);
    {
        std::stringstream ss(std::ios::in | std::ios::out | std::ios::binary);
        fold7->DumpObject(ss);
        auto again = std::dynamic_pointer_cast<bb::Model>(bb::Object_Load(ss));
        CHECK((bool)again && again->GetObjectName() == "Reduce_fp32_fp32" && again->GetOutputNodeSize() == O, "Reduce reload");
        if (again) { bb::FrameBuffer y3 = again->Forward(x_buf); CHECK(same_bits(y3, y_buf), "reloaded Reduce differs"); }
    }
}

// The converters at either end of a binary network, the activations, and the three-part container around a layer list.
static void test_binary_modulation(void)
{
    std::mt19937_64 mt(23);
    std::uniform_real_distribution<float> uni(-0.1f, 1.1f);
    std::vector<float> x, y, dy, dx, ref;
    {   // RealToBinary over shape {2, 5}: 3 frames and 2 depth steps per input; fp32 and packed outputs, binary and real mode
        int const D = 2, P = 5, F = 37, fm = 3, dm = 2;
        bb::FrameBuffer x_buf(F, {D, P}, BB_TYPE_FP32);
        for (int n = 0; n < D * P; ++n) for (int f = 0; f < F; ++f) { x_buf.SetFP32(f, n, uni(mt)); }
        read_fp32(x_buf, x);
        auto r2b = bb::RealToBinary<float>::Create(fm, dm);
        auto r2b_bit = bb::RealToBinary<bb::Bit>::Create(fm, dm);
        CHECK(r2b->SetInputShape({D, P}) == bb::indices_t({D * dm, P}), "RealToBinary output shape");
        for (int binary = 1; binary >= 0; --binary) {
            r2b->SendCommand(binary ? "binary true" : "binary false"); r2b_bit->SendCommand(binary ? "binary true" : "binary false");
            bb::FrameBuffer y_buf = r2b->Forward(x_buf), yb_buf = r2b_bit->Forward(x_buf);
            CHECK(y_buf.GetFrameSize() == F * fm && y_buf.GetNodeSize() == D * dm * P && yb_buf.GetType() == BB_TYPE_BIT, "RealToBinary output size");
            read_fp32(y_buf, y);
            ref.assign(y.size(), 0.0f);
            oracle_fp32_RealToBinary_Forward(x.data(), ref.data(), dm, fm, 0.0f, 1.0f, P, D, F, F, F * fm, binary);
            CHECK(max_diff(y, ref) == 0.0, "RealToBinary (binary %d) differs by %g", binary, max_diff(y, ref));
            size_t bad = 0;
            // the packed output is Bit(v), v > 0, of the fp32 output: of +1 / -1 in binary mode, of the clamped value otherwise
            for (int n = 0; n < D * dm * P; ++n) for (int f = 0; f < F * fm; ++f) { bad += (yb_buf.GetBit(f, n) != (ref[(size_t)n * F * fm + f] > 0.0f)); }
            CHECK(bad == 0, "RealToBinary packed output (binary %d): %zu bits differ", binary, bad);
        }
        auto plain = bb::RealToBinary<float>::Create(fm);
        plain->SendCommand("binary false");
        bb::FrameBuffer same = plain->Forward(x_buf);
        CHECK(same_bits(same, x_buf), "RealToBinary out of binary mode without depth modulation hands its input through");
    }
    {   // BinaryToReal: 70 nodes fold into 10, 7 frames into 1; fp32 and packed input, backward
        int const I = 70, O = 10, Fy = 33, fm = 7, F = Fy * fm;
        bb::FrameBuffer x_buf(F, {I}, BB_TYPE_FP32), xb_buf(F, {I}, BB_TYPE_BIT), dy_buf(Fy, {O}, BB_TYPE_FP32);
        for (int n = 0; n < I; ++n) for (int f = 0; f < F; ++f) { float const v = uni(mt) - 0.5f; x_buf.SetFP32(f, n, v); xb_buf.SetBit(f, n, v > 0); }
        for (int n = 0; n < O; ++n) for (int f = 0; f < Fy; ++f) { dy_buf.SetFP32(f, n, uni(mt) - 0.5f); }
        read_fp32(x_buf, x); read_fp32(dy_buf, dy);
        auto b2r = bb::BinaryToReal<float>::Create(fm, bb::indices_t({O}));
        auto b2r_bit = bb::BinaryToReal<bb::Bit>::Create(fm, bb::indices_t({O}));
        bb::FrameBuffer y_buf = b2r->Forward(x_buf), yb_buf = b2r_bit->Forward(xb_buf);
        read_fp32(y_buf, y);
        ref.assign((size_t)O * Fy, 0.0f);
        oracle_fp32_BinaryToReal_Forward(x.data(), ref.data(), I / O, fm, O, F, Fy, Fy);
        CHECK(max_diff(y, ref) == 0.0 && same_bits(y_buf, yb_buf), "BinaryToReal forward differs by %g", max_diff(y, ref));
        bb::FrameBuffer dx_buf = b2r->Backward(dy_buf);
        read_fp32(dx_buf, dx);
        ref.assign((size_t)I * F, 0.0f);
        oracle_fp32_BinaryToReal_Backward(dy.data(), ref.data(), I / O, fm, O, F, Fy, Fy);
        CHECK(dx_buf.GetFrameSize() == F && max_diff(dx, ref) == 0.0, "BinaryToReal backward differs by %g", max_diff(dx, ref));
        auto by_depth = bb::BinaryToReal<float>::Create(fm, 7);
        CHECK(by_depth->SetInputShape({I}) == bb::indices_t({O}), "BinaryToReal output shape from the depth integration size");
    }
    {   // Binarize and HardTanh
        int const N = 9, F = 130;
        bb::FrameBuffer x_buf(F, {N}, BB_TYPE_FP32), dy_buf(F, {N}, BB_TYPE_FP32);
        for (int n = 0; n < N; ++n) for (int f = 0; f < F; ++f) { x_buf.SetFP32(f, n, 3.0f * (uni(mt) - 0.5f)); dy_buf.SetFP32(f, n, uni(mt)); }
        read_fp32(x_buf, x); read_fp32(dy_buf, dy);
        auto bin = bb::Binarize<float>::Create(0.1f, 0.0, 1.0, -0.7f, 0.9f);
        auto bin_bit = bb::Binarize<bb::Bit>::Create(0.1f);
        auto tanh = bb::HardTanh<float>::Create(-0.5f, 0.75f);
        bb::FrameBuffer y_buf = bin->Forward(x_buf), yb_buf = bin_bit->Forward(x_buf, false), t_buf = tanh->Forward(x_buf);
        read_fp32(y_buf, y);
        ref.assign(x.size(), 0.0f);
        oracle_fp32_Binarize_Forward(x.data(), ref.data(), 0.1f, 0.0f, 1.0f, N, F, F);
        size_t bad = 0;
        for (int n = 0; n < N; ++n) for (int f = 0; f < F; ++f) { bad += (yb_buf.GetBit(f, n) != (ref[(size_t)n * F + f] > 0.5f)); }
        CHECK(max_diff(y, ref) == 0.0 && bad == 0, "Binarize forward differs by %g, %zu bits", max_diff(y, ref), bad);
        bb::FrameBuffer dx_buf = bin->Backward(dy_buf);
        read_fp32(dx_buf, dx);
        oracle_fp32_HardTanh_Backward(x.data(), dy.data(), ref.data(), -0.7f, 0.9f, N, F, F);
        CHECK(max_diff(dx, ref) == 0.0, "Binarize backward differs by %g", max_diff(dx, ref));
        read_fp32(t_buf, y);
        oracle_fp32_HardTanh_Forward(x.data(), ref.data(), -0.5f, 0.75f, N, F, F);
        CHECK(max_diff(y, ref) == 0.0, "HardTanh forward differs by %g", max_diff(y, ref));
        dx_buf = tanh->Backward(dy_buf);
        read_fp32(dx_buf, dx);
        oracle_fp32_HardTanh_Backward(x.data(), dy.data(), ref.data(), -0.5f, 0.75f, N, F, F);
        CHECK(max_diff(dx, ref) == 0.0, "HardTanh backward differs by %g", max_diff(dx, ref));
        tanh->SendCommand("binary true");
        t_buf = tanh->Forward(x_buf, false);
        read_fp32(t_buf, y);
        oracle_fp32_Binarize_Forward(x.data(), ref.data(), 0.125f, -1.0f, 1.0f, N, F, F);
        CHECK(max_diff(y, ref) == 0.0, "HardTanh in binary mode differs by %g", max_diff(y, ref));
        CHECK(tanh->ForwardNode(0, {0.2, 0.1})[0] == 0.75 && tanh->ForwardNode(0, {0.2, 0.1})[1] == -0.5, "HardTanh::ForwardNode in binary mode");
    }
    {   // BinaryModulation around two layers = its three parts called one after the other; training and inference sizes; a reload
        int const I = 20, O1 = 36, O2 = 12, F = 50, train_mod = 3, infer_mod = 5;
        auto make_body = [&](void) {
            auto body = bb::Sequential::Create();
            body->Add(bb::DifferentiableLutN<6, float>::Create((bb::index_t)O1));
            body->Add(bb::DifferentiableLutN<6, float>::Create((bb::index_t)O2));
            return body;
        };
        auto net = bb::BinaryModulation<float>::Create(make_body(), train_mod, infer_mod);
        CHECK(net->SetInputShape({I}) == bb::indices_t({O2}), "BinaryModulation output shape");
        auto body = make_body();
        {   // a second copy of the layers with the same contents, for the parts called by hand
            std::stringstream ss(std::ios::in | std::ios::out | std::ios::binary);
            net->GetLayer()->DumpObject(ss);
            body->SetInputShape({I});
            body->LoadObject(ss);
        }
        bb::FrameBuffer x_buf(F, {I}, BB_TYPE_FP32), dy_buf(F, {O2}, BB_TYPE_FP32);
        for (int n = 0; n < I; ++n) for (int f = 0; f < F; ++f) { x_buf.SetFP32(f, n, uni(mt)); }
        for (int n = 0; n < O2; ++n) for (int f = 0; f < F; ++f) { dy_buf.SetFP32(f, n, uni(mt) - 0.5f); }
        auto r2b = bb::RealToBinary<float>::Create(train_mod);
        auto b2r = bb::BinaryToReal<float>::Create(train_mod, bb::indices_t({O2}));
        bb::FrameBuffer y_buf = net->Forward(x_buf, true);
        bb::FrameBuffer h_buf = b2r->Forward(body->Forward(r2b->Forward(x_buf, true), true), true);
        CHECK(y_buf.GetFrameSize() == F && same_bits(y_buf, h_buf), "BinaryModulation forward differs from its three parts");
        bb::FrameBuffer dx_buf = net->Backward(dy_buf);
        bb::FrameBuffer g_buf = body->Backward(b2r->Backward(dy_buf));
        CHECK(dx_buf.GetFrameSize() == F && dx_buf.GetNodeSize() == I && g_buf.GetFrameSize() == F * train_mod, "BinaryModulation backward shapes");
        {
            auto a = net->GetGradients(), b = body->GetGradients();
            CHECK(a.GetSize() == b.GetSize() && a.GetSize() == 2, "BinaryModulation hands the layers' gradients through");
        }
        r2b->SetModulationSize(infer_mod); b2r->SetFrameIntegrationSize(infer_mod);
        y_buf = net->Forward(x_buf, false);
        h_buf = b2r->Forward(body->Forward(r2b->Forward(x_buf, false), false), false);
        CHECK(y_buf.GetFrameSize() == F && same_bits(y_buf, h_buf), "BinaryModulation inference differs from its three parts");
        std::stringstream ss(std::ios::in | std::ios::out | std::ios::binary);
        net->DumpObject(ss);
        auto again = std::dynamic_pointer_cast<bb::Model>(bb::Object_Load(ss));
        CHECK((bool)again && again->GetObjectName() == "BinaryModulation_fp32_fp32" && again->GetOutputNodeSize() == O2, "BinaryModulation reload");
        if (again) { bb::FrameBuffer y3 = again->Forward(x_buf, false); CHECK(same_bits(y3, y_buf), "reloaded BinaryModulation differs"); }
        net->SendCommand("binary false");
        y_buf = net->Forward(x_buf, false);
        CHECK(y_buf.GetFrameSize() == F, "BinaryModulation out of binary mode runs the layer on the unconverted input");
    }
}

// The LUT layer put together from its parts (StochasticLutN -> StochasticBatchNormalization -> HardTanh) against the fused
// DifferentiableLutN with the same wiring and table, in the shape of the reference's own comparison of the two
// (tests/gtest/SparseLutNTest.cpp:19-299), and with memory saving (intermediate results recomputed in the backward pass) against
// without, which must give the same bits.
template <int N>
static void test_discrete(int I, int O, int F, bool binary)
{
    std::mt19937_64 mt(4242 + I + O + F + (binary ? 1 : 0));
    std::uniform_real_distribution<float> uni(0.0f, 1.0f);
    constexpr int NN = 1 << N;
    typename bb::DifferentiableLutN<N, float>::create_t fc;
    fc.output_shape = {O}; fc.binary = binary; fc.momentum = 0.9f;
    auto fused = bb::DifferentiableLutN<N, float>::Create(fc);
    typename bb::DifferentiableLutDiscreteN<N, float>::create_t dc;
    dc.output_shape = {O}; dc.momentum = 0.9f;
    auto parts = bb::DifferentiableLutDiscreteN<N, float>::Create(dc);
    auto saving = bb::DifferentiableLutDiscreteN<N, float>::Create(dc);
    saving->SendCommand("memory_saving true");
    std::vector<std::int32_t> idx; wire<N>(mt, I, O, idx);
    std::vector<float> W((size_t)O * NN);
    for (auto &w : W) { w = uni(mt); }
    auto set_up = [&](auto &m) {
        m->SendCommand(binary ? "binary true" : "binary false");
        m->SendCommand("lut_binarize false");
        m->SetInputShape({I});
        for (int o = 0; o < O; ++o) for (int i = 0; i < N; ++i) { m->SetNodeConnectionIndex(o, i, idx[(size_t)o * N + i]); }
        auto Wp = m->lock_W();
        for (size_t k = 0; k < W.size(); ++k) { Wp[(bb::index_t)k] = W[k]; }
    };
    set_up(fused); set_up(parts); set_up(saving);
    bb::FrameBuffer x_buf(F, {I}, BB_TYPE_FP32), dy_buf(F, {O}, BB_TYPE_FP32);
    for (int loop = 0; loop < 2; ++loop) {
        for (int n = 0; n < I; ++n) for (int f = 0; f < F; ++f) { x_buf.SetFP32(f, n, uni(mt)); }
        for (int n = 0; n < O; ++n) for (int f = 0; f < F; ++f) { dy_buf.SetFP32(f, n, uni(mt) - 0.5f); }
        bb::FrameBuffer y0 = fused->Forward(x_buf, true), y1 = parts->Forward(x_buf, true), y2 = saving->Forward(x_buf, true);
        bb::FrameBuffer dx0 = fused->Backward(dy_buf), dx1 = parts->Backward(dy_buf), dx2 = saving->Backward(dy_buf);
        CHECK(same_bits(y1, y2) && same_bits(dx1, dx2), "DifferentiableLutDiscrete%d: memory saving changes the result", N);
        std::vector<float> a, b;
        read_fp32(y0, a); read_fp32(y1, b);
        if (binary) {
            size_t mism = 0;
            for (size_t k = 0; k < a.size(); ++k) { mism += ((a[k] > 0.5f) != (b[k] > 0.0f)); }     // the fused layer writes 1 / 0, the activation +1 / -1
            CHECK(mism <= 2 + a.size() / 10000, "DifferentiableLutDiscrete%d binary y: %zu of %zu differ from the fused layer", N, mism, a.size());
        }
        else {
            CHECK(max_diff(a, b) <= 1e-5, "DifferentiableLutDiscrete%d y differs from the fused layer by %g", N, max_diff(a, b));
            read_fp32(dx0, a); read_fp32(dx1, b);
            CHECK(max_diff(a, b) <= 1e-4 * std::max(1e-3, max_abs(a)), "DifferentiableLutDiscrete%d dx differs from the fused layer by %g of %g", N, max_diff(a, b), max_abs(a));
            std::vector<float> g0((size_t)O * NN), g1((size_t)O * NN);
            { auto p = fused->lock_dW_const(); auto q = parts->lock_dW_const(); for (size_t k = 0; k < g0.size(); ++k) { g0[k] = p[(bb::index_t)k]; g1[k] = q[(bb::index_t)k]; } }
            CHECK(max_diff(g0, g1) <= 1e-4 * std::max(1e-3, max_abs(g0)), "DifferentiableLutDiscrete%d dW differs from the fused layer by %g of %g", N, max_diff(g0, g1), max_abs(g0));
        }
        std::vector<float> m0((size_t)O), m1((size_t)O), v0((size_t)O), v1((size_t)O);
        { auto p = fused->lock_mean_const(); auto q = parts->lock_mean_const(); auto r = fused->lock_var_const(); auto t = parts->lock_var_const();
          for (int o = 0; o < O; ++o) { m0[(size_t)o] = p[o]; m1[(size_t)o] = q[o]; v0[(size_t)o] = r[o]; v1[(size_t)o] = t[o]; } }
        CHECK(max_diff(m0, m1) <= 1e-5 && max_diff(v0, v1) <= 2e-5, "DifferentiableLutDiscrete%d running statistics differ by %g, %g", N, max_diff(m0, m1), max_diff(v0, v1));
        { auto p = parts->lock_dW_const(); auto q = saving->lock_dW_const(); size_t bad = 0; for (bb::index_t k = 0; k < (bb::index_t)O * NN; ++k) { bad += (p[k] != q[k]); }
          CHECK(bad == 0, "DifferentiableLutDiscrete%d: memory saving changes %zu table gradients", N, bad); }
    }
    // through a stream and back
    std::stringstream ss(std::ios::in | std::ios::out | std::ios::binary);
    parts->DumpObject(ss);
    auto again = std::dynamic_pointer_cast<bb::Model>(bb::Object_Load(ss));
    CHECK((bool)again && again->GetObjectName() == parts->GetObjectName() && again->GetOutputNodeSize() == O, "DifferentiableLutDiscrete reload");
    if (again) {
        bb::FrameBuffer y1 = parts->Forward(x_buf, false), y3 = again->Forward(x_buf, false);
        CHECK(same_bits(y1, y3), "reloaded DifferentiableLutDiscrete%d differs", N);
    }
}

// MaxPooling and UpSampling through the classes: fp32 against the oracle, the packed forms against the fp32 forms on 0 / 1 images
// (OR = max; the first set input = the first largest value), shapes, and a trip through a stream.
static void test_pooling(void)
{
    int const C = 3, H = 5, Wd = 7, FH = 2, FW = 3, F = 70;
    int const OH = (H + FH - 1) / FH, OW = (Wd + FW - 1) / FW;
    std::mt19937_64 mt(31);
    std::uniform_real_distribution<float> uni(-1.0f, 1.0f);
    bb::FrameBuffer x_buf(F, {C, H, Wd}, BB_TYPE_FP32), dy_buf(F, {C, OH, OW}, BB_TYPE_FP32);
    for (int n = 0; n < C * H * Wd; ++n) for (int f = 0; f < F; ++f) { x_buf.SetFP32(f, n, (mt() % 5 == 0) ? 0.25f : uni(mt)); }
    for (int n = 0; n < C * OH * OW; ++n) for (int f = 0; f < F; ++f) { dy_buf.SetFP32(f, n, uni(mt)); }
    std::vector<float> x, dy, y, dx, y_ref((size_t)C * OH * OW * F), dx_ref((size_t)C * H * Wd * F);
    std::vector<int> arg_ref(y_ref.size());
    read_fp32(x_buf, x); read_fp32(dy_buf, dy);
    auto pool = bb::MaxPooling<>::Create(FH, FW);
    CHECK(pool->SetInputShape({C, H, Wd}) == bb::indices_t({C, OH, OW}), "MaxPooling output shape");
    bb::FrameBuffer y_buf = pool->Forward(x_buf), dx_buf = pool->Backward(dy_buf);
    read_fp32(y_buf, y); read_fp32(dx_buf, dx);
    oracle_fp32_MaxPooling_Forward(x.data(), y_ref.data(), arg_ref.data(), FH, FW, Wd, H, OW, OH, C, F, F);
    oracle_fp32_MaxPooling_Backward(arg_ref.data(), dy.data(), dx_ref.data(), FH, FW, Wd, H, OW, OH, C, F, F);
    CHECK(max_diff(y, y_ref) == 0.0 && max_diff(dx, dx_ref) == 0.0, "MaxPooling differs by %g, %g", max_diff(y, y_ref), max_diff(dx, dx_ref));
    {   // packed: a 0 / 1 image pooled as bits = the fp32 pooling of the same image
        bb::FrameBuffer b_buf(F, {C, H, Wd}, BB_TYPE_BIT), f_buf(F, {C, H, Wd}, BB_TYPE_FP32);
        for (int n = 0; n < C * H * Wd; ++n) for (int f = 0; f < F; ++f) { bool const v = (mt() % 4 == 0); b_buf.SetBit(f, n, v); f_buf.SetFP32(f, n, v ? 1.0f : 0.0f); }
        auto pool_bit = bb::MaxPooling<bb::Bit>::Create(FH, FW);
        auto pool_f = bb::MaxPooling<>::Create(FH, FW);
        bb::FrameBuffer yb = pool_bit->Forward(b_buf), yf = pool_f->Forward(f_buf);
        size_t bad = 0;
        for (int n = 0; n < C * OH * OW; ++n) for (int f = 0; f < F; ++f) { bad += (yb.GetBit(f, n) != (yf.GetFP32(f, n) > 0.5f)); }
        CHECK(yb.GetType() == BB_TYPE_BIT && bad == 0, "packed MaxPooling forward: %zu bits differ", bad);
        bb::FrameBuffer gb = pool_bit->Backward(dy_buf), gf = pool_f->Backward(dy_buf);
        // where a window holds a one both send dy to its first one; an empty window sends nothing (packed) or dy to its first input (fp32)
        bad = 0;
        for (int c = 0; c < C; ++c) for (int iy = 0; iy < H; ++iy) for (int ix = 0; ix < Wd; ++ix) for (int f = 0; f < F; ++f) {
            int const n = (c * H + iy) * Wd + ix, o = (c * OH + iy / FH) * OW + ix / FW;
            float const want = yb.GetBit(f, o) ? gf.GetFP32(f, n) : 0.0f;
            bad += (gb.GetFP32(f, n) != want);
        }
        CHECK(bad == 0, "packed MaxPooling backward: %zu values differ", bad);
    }
    for (int fill = 1; fill >= 0; --fill) {
        auto up = bb::UpSampling<>::Create(FH, FW, fill != 0);
        CHECK(up->SetInputShape({C, OH, OW}) == bb::indices_t({C, OH * FH, OW * FW}), "UpSampling output shape");
        bb::FrameBuffer u_buf = up->Forward(dy_buf);
        bb::FrameBuffer g_buf(F, {C, OH * FH, OW * FW}, BB_TYPE_FP32);
        for (int n = 0; n < C * OH * FH * OW * FW; ++n) for (int f = 0; f < F; ++f) { g_buf.SetFP32(f, n, uni(mt)); }
        bb::FrameBuffer d_buf = up->Backward(g_buf);
        std::vector<float> u, g, d, u_ref((size_t)C * OH * FH * OW * FW * F), d_ref(dy.size());
        read_fp32(u_buf, u); read_fp32(g_buf, g); read_fp32(d_buf, d);
        oracle_fp32_UpSampling_Forward(dy.data(), u_ref.data(), OW, OH, C, FW, FH, fill, F, F);
        oracle_fp32_UpSampling_Backward(g.data(), d_ref.data(), OW, OH, C, FW, FH, fill, F, F);
        CHECK(max_diff(u, u_ref) == 0.0 && max_diff(d, d_ref) == 0.0, "UpSampling (fill %d) differs by %g, %g", fill, max_diff(u, u_ref), max_diff(d, d_ref));
        std::stringstream ss(std::ios::in | std::ios::out | std::ios::binary);
        up->DumpObject(ss);
        pool->DumpObject(ss);
        auto up2 = std::dynamic_pointer_cast<bb::Model>(bb::Object_Load(ss));
        auto pool2 = std::dynamic_pointer_cast<bb::Model>(bb::Object_Load(ss));
        CHECK((bool)up2 && (bool)pool2 && up2->GetObjectName() == "UpSampling_fp32_fp32" && pool2->GetObjectName() == "MaxPooling_fp32_fp32", "pooling reload");
        if (up2 && pool2) {
            bb::FrameBuffer u2 = up2->Forward(dy_buf, false), y2 = pool2->Forward(x_buf, false);
            CHECK(same_bits(u2, u_buf) && same_bits(y2, y_buf), "reloaded pooling layers differ");
        }
    }
}

// Shuffle through the class: fp32 and packed frames against the closed form (output node i * unit + j = input node
// j * (nodes / unit) + i), backward(forward(x)) == x, and a trip through a stream.
static void test_shuffle(void)
{
    int const N = 84, U = 7, X = N / U, F = 70;
    std::mt19937_64 mt(47);
    std::uniform_real_distribution<float> uni(-1.0f, 1.0f);
    bb::FrameBuffer x_buf(F, {N}, BB_TYPE_FP32), b_buf(F, {N}, BB_TYPE_BIT);
    for (int n = 0; n < N; ++n) for (int f = 0; f < F; ++f) { x_buf.SetFP32(f, n, uni(mt)); b_buf.SetBit(f, n, mt() % 2 == 0); }
    auto shuffle = bb::Shuffle::Create(U, bb::indices_t({4, 21}));
    CHECK(shuffle->SetInputShape({N}) == bb::indices_t({4, 21}), "Shuffle output shape");
    bb::FrameBuffer y_buf = shuffle->Forward(x_buf), yb_buf = shuffle->Forward(b_buf);
    CHECK(y_buf.GetType() == BB_TYPE_FP32 && yb_buf.GetType() == BB_TYPE_BIT && y_buf.GetShape() == bb::indices_t({4, 21}), "Shuffle output type");
    size_t bad = 0;
    for (int i = 0; i < X; ++i) for (int j = 0; j < U; ++j) for (int f = 0; f < F; ++f) {
        bad += (y_buf.GetFP32(f, i * U + j) != x_buf.GetFP32(f, j * X + i));
        bad += (yb_buf.GetBit(f, i * U + j) != b_buf.GetBit(f, j * X + i));
    }
    CHECK(bad == 0, "Shuffle forward: %zu values differ", bad);
    bb::FrameBuffer dx_buf = shuffle->Backward(y_buf), dxb_buf = shuffle->Backward(yb_buf);
    bad = 0;
    for (int n = 0; n < N; ++n) for (int f = 0; f < F; ++f) { bad += (dx_buf.GetFP32(f, n) != x_buf.GetFP32(f, n)) + (dxb_buf.GetBit(f, n) != b_buf.GetBit(f, n)); }
    CHECK(bad == 0 && dx_buf.GetShape() == bb::indices_t({N}), "Shuffle backward does not undo forward: %zu values differ", bad);
    std::stringstream ss(std::ios::in | std::ios::out | std::ios::binary);
    shuffle->DumpObject(ss);
    auto again = std::dynamic_pointer_cast<bb::Model>(bb::Object_Load(ss));
    CHECK((bool)again && again->GetObjectName() == "Shuffle" && again->GetOutputShape() == bb::indices_t({4, 21}), "Shuffle reload");
    if (again) { bb::FrameBuffer y2 = again->Forward(x_buf, false); CHECK(same_bits(y2, y_buf), "reloaded Shuffle differs"); }
}

static void test_tail(void)
{
    int const n = 7, O = 10, I = 70, F = 100;
    std::mt19937_64 mt(9);
    std::uniform_real_distribution<float> uni(-1.0f, 1.0f);
    std::vector<std::int32_t> idx((size_t)O * n);
    for (auto &v : idx) { v = (std::int32_t)(mt() % (std::uint64_t)I); }
    std::vector<float> x((size_t)I * F), dy((size_t)O * F), y_ref((size_t)O * F), dx_ref((size_t)I * F), got;
    for (auto &v : x) { v = uni(mt); }
    for (auto &v : dy) { v = uni(mt); }
    bb::FrameBuffer x_buf(F, {I}, BB_TYPE_FP32), dy_buf(F, {O}, BB_TYPE_FP32);
    for (int i = 0; i < I; ++i) for (int f = 0; f < F; ++f) { x_buf.SetFP32(f, i, x[(size_t)i * F + f]); }
    for (int o = 0; o < O; ++o) for (int f = 0; f < F; ++f) { dy_buf.SetFP32(f, o, dy[(size_t)o * F + f]); }
    for (int binarize = 0; binarize < 2; ++binarize) {
        auto avg = bb::AverageLut<>::Create(n, (bb::index_t)O, "", binarize != 0);
        avg->SetInputShape({I});
        for (int o = 0; o < O; ++o) for (int i = 0; i < n; ++i) { avg->SetNodeConnectionIndex(o, i, idx[(size_t)o * n + i]); }
        // the class follows the reference's device path: sum * (1 / n) where the output is not binarized; "host_sum true" gives
        // the host loop's plain sum, which is what the oracle restates
        oracle_fp32_AverageLut_Forward(x.data(), y_ref.data(), idx.data(), n, O, F, F, 0, binarize);
        bb::FrameBuffer y_buf = avg->Forward(x_buf);
        read_fp32(y_buf, got);
        {
            std::vector<float> y_mean(y_ref);
            float const reciprocal = 1.0f / (float)n;
            if (!binarize) { for (auto &v : y_mean) { v = v * reciprocal; } }
            CHECK(got == y_mean, "AverageLut forward, device convention (binarize %d)", binarize);
        }
        avg->SendCommand("host_sum true");
        y_buf = avg->Forward(x_buf);
        read_fp32(y_buf, got);
        CHECK(got == y_ref, "AverageLut forward, host convention (binarize %d)", binarize);
        bb::FrameBuffer dx_buf = avg->Backward(dy_buf);
        oracle_fp32_AverageLut_Backward(dy.data(), dx_ref.data(), idx.data(), n, I, O, F, F);
        read_fp32(dx_buf, got);
        CHECK(got == dx_ref, "AverageLut backward");
    }
    {
        auto avg = bb::AverageLut<bb::Bit>::Create(n, (bb::index_t)O);
        avg->SetInputShape({I});
        for (int o = 0; o < O; ++o) for (int i = 0; i < n; ++i) { avg->SetNodeConnectionIndex(o, i, idx[(size_t)o * n + i]); }
        int const words = (F + 31) / 32;
        std::vector<std::int32_t> xb((size_t)I * words, 0), yb_ref((size_t)O * words, 0);
        bb::FrameBuffer xb_buf(F, {I}, BB_TYPE_BIT);
        xb_buf.FillZero();
        for (int i = 0; i < I; ++i) for (int f = 0; f < F; ++f) {
            bool const v = x[(size_t)i * F + f] > 0;
            if (v) { xb[(size_t)i * words + (f >> 5)] |= (std::int32_t)(1u << (f & 31)); }
            xb_buf.SetBit(f, i, v);
        }
        bb::FrameBuffer yb_buf = avg->Forward(xb_buf);
        oracle_bit_AverageLut_Forward(xb.data(), yb_ref.data(), idx.data(), n, O, F, words);
        size_t bad = 0;
        for (int o = 0; o < O; ++o) for (int f = 0; f < F; ++f) { bad += (yb_buf.GetBit(f, o) != (((yb_ref[(size_t)o * words + (f >> 5)] >> (f & 31)) & 1) != 0)); }
        CHECK(bad == 0, "AverageLut bit forward: %zu wrong", bad);
        CHECK(avg->GetLutTable(0, 0x0f) && !avg->GetLutTable(0, 0x07), "AverageLut table view: majority of 7 index bits");
    }

    float const x_table[5][10] = {
        {0.03682449f, 0.7174495f, 0.9130372f, 0.6275032f, 0.11995261f, 0.25850186f, 0.9942376f, 0.23910977f, 0.75574166f, 0.38816985f},
        {0.59729785f, 0.7654758f, 0.35820892f, 0.0122047f, 0.05050702f, 0.323845f, 0.6889169f, 0.16161442f, 0.06116614f, 0.769033f},
        {0.94036084f, 0.25700864f, 0.73131865f, 0.58721095f, 0.78960747f, 0.29338115f, 0.36369365f, 0.5750651f, 0.81494033f, 0.05262487f},
        {0.98256797f, 0.15146895f, 0.51034707f, 0.38718516f, 0.18072742f, 0.7927627f, 0.13334593f, 0.03729849f, 0.20618507f, 0.9241972f},
        {0.713539f, 0.48547512f, 0.27168426f, 0.54288715f, 0.6140953f, 0.67773014f, 0.03847398f, 0.7239832f, 0.64887875f, 0.42749837f}};
    int const x_label[5] = {2, 5, 6, 3, 4};
    float const dx_table[5][10] = {
        {0.01189111f, 0.02348626f, -0.17144011f, 0.02146598f, 0.01292184f, 0.0148421f, 0.03097572f, 0.01455706f, 0.02440304f, 0.016897f},
        {0.02385998f, 0.02822986f, 0.01878603f, 0.01329129f, 0.01381026f, -0.18184856f, 0.02614928f, 0.01543317f, 0.01395825f, 0.02833046f},
        {0.02876907f, 0.01452612f, 0.0233421f, 0.02020946f, 0.02474312f, 0.0150642f, -0.18383847f, 0.01996549f, 0.02537794f, 0.01184096f},
        {0.03275547f, 0.01426731f, 0.02042683f, -0.18194023f, 0.01469092f, 0.02709271f, 0.01401107f, 0.01272795f, 0.01506971f, 0.03089824f},
        {0.02392219f, 0.01904382f, 0.01537821f, 0.02016916f, -0.17834225f, 0.02308072f, 0.01217935f, 0.02417335f, 0.02242433f, 0.01797112f}};
    bb::FrameBuffer y_buf(5, {10}, BB_TYPE_FP32), t_buf(5, {10}, BB_TYPE_FP32);
    for (int i = 0; i < 5; ++i) for (int j = 0; j < 10; ++j) {
        y_buf.SetFP32(i, j, x_table[i][j]);
        t_buf.SetFP32(i, j, (j == x_label[i]) ? 1.0f : 0.0f);
    }
    auto lossFunc = bb::LossSoftmaxCrossEntropy<float>::Create();
    lossFunc->Clear();
    bb::FrameBuffer dyb = lossFunc->CalculateLoss(y_buf, t_buf, y_buf.GetFrameSize());
    CHECK(std::fabs(lossFunc->GetLoss() - 2.297830009460449) < 0.0001, "loss %.9f, expected 2.297830009", lossFunc->GetLoss());
    double worst = 0;
    for (int i = 0; i < 5; ++i) for (int j = 0; j < 10; ++j) { worst = std::max(worst, (double)std::fabs(dyb.GetFP32(i, j) - dx_table[i][j])); }
    CHECK(worst < 0.000001, "loss gradient off by %.3g", worst);
    auto metrics = bb::MetricsCategoricalAccuracy<float>::Create();
    metrics->CalculateMetrics(t_buf, t_buf);
    CHECK(metrics->GetMetrics() == 1.0, "accuracy of the targets themselves: %f", metrics->GetMetrics());
    metrics->Clear();
    metrics->CalculateMetrics(y_buf, t_buf);
    int hits = 0;
    for (int i = 0; i < 5; ++i) { int best = 0; for (int j = 1; j < 10; ++j) { if (x_table[i][j] > x_table[i][best]) { best = j; } } hits += (best == x_label[i]); }
    CHECK(metrics->GetMetrics() == hits / 5.0, "accuracy %f, expected %f", metrics->GetMetrics(), hits / 5.0);
}

// The trained-layer hand-off end to end through files: a DifferentiableLut6 on packed bits is written as a `.bb_net` object,
// reconstructed from the file by its recorded name, gives the same inference output, is tabulated into a BinaryLut6
// (ImportLayer), which is written and read back as well and reproduces those bits on the device.
static void test_hand_off_through_files(void)
{
    int const I = 48, O = 40, F = 300;
    std::mt19937_64 mt(17);
    std::uniform_real_distribution<float> uni(0.0f, 1.0f);
    auto src = bb::DifferentiableLutN<6, bb::Bit>::Create(O);
    src->SetName("trained");
    bb::FrameBuffer x_buf(F, {I}, BB_TYPE_BIT);
    src->SetInputShape(x_buf.GetShape());
    { auto Wp = src->lock_W(); for (int k = 0; k < O * 64; ++k) { Wp[k] = uni(mt); } }
    { auto m = src->lock_mean(); auto v = src->lock_var(); for (int o = 0; o < O; ++o) { m[o] = 0.35f + 0.3f * uni(mt); v[o] = 0.02f + 0.1f * uni(mt); } }
    { auto xp = x_buf.Lock<bb::Bit>(true); for (int n = 0; n < I; ++n) for (int f = 0; f < F; ++f) { xp.Set(f, n, bb::Bit((mt() & 1) != 0)); } }
    std::string const dir = "/tmp/";
    CHECK(src->DumpToFile(dir + "bbhip_hand_off_layer.bb_net"), "DumpToFile");
    auto loaded = std::dynamic_pointer_cast<bb::DifferentiableLutN<6, bb::Bit>>(bb::Object_LoadFromFile(dir + "bbhip_hand_off_layer.bb_net"));
    CHECK((bool)loaded, "Object_LoadFromFile did not reconstruct a DifferentiableLut6_bit_fp32");
    if (!loaded) { return; }
    CHECK(loaded->GetName() == "trained", "name %s", loaded->GetName().c_str());
    auto y_src = src->Forward(x_buf, false);
    auto y_loaded = loaded->Forward(x_buf, false);
    auto dst = bb::BinaryLutN<6, bb::Bit>::Create(O);
    dst->SetInputShape(x_buf.GetShape());
    dst->ImportLayer(loaded);
    CHECK(dst->DumpToFile(dir + "bbhip_hand_off_table.bb_net"), "DumpToFile");
    auto table = std::dynamic_pointer_cast<bb::BinaryLutN<6, bb::Bit>>(bb::Object_LoadFromFile(dir + "bbhip_hand_off_table.bb_net"));
    CHECK((bool)table, "Object_LoadFromFile did not reconstruct a BinaryLut6_bit_fp32");
    if (!table) { return; }
    auto y_table = table->Forward(x_buf);
    auto a = y_src.LockConst<bb::Bit>(); auto b = y_loaded.LockConst<bb::Bit>(); auto c = y_table.LockConst<bb::Bit>();
    size_t reload = 0, tabulated = 0, ones = 0;
    for (int n = 0; n < O; ++n) for (int f = 0; f < F; ++f) {
        reload += ((bool)a.Get(f, n) != (bool)b.Get(f, n));
        tabulated += ((bool)a.Get(f, n) != (bool)c.Get(f, n));
        ones += (bool)a.Get(f, n);
    }
    CHECK(reload == 0, "reloaded layer: %zu mismatching bits", reload);
    CHECK(tabulated == 0, "tabulated layer: %zu mismatching bits", tabulated);
    CHECK(ones > (size_t)O * F / 10 && ones < (size_t)O * F * 9 / 10, "degenerate outputs (%zu ones)", ones);
    std::remove((dir + "bbhip_hand_off_layer.bb_net").c_str());
    std::remove((dir + "bbhip_hand_off_table.bb_net").c_str());
}

int main(void)
{
    if (!bb::Manager::IsDeviceAvailable()) { std::printf("no device available\n"); return 2; }
    try {
        // shapes of tests/gtest/StochasticLutNTest.cpp:235-246
        int const shapes[][3] = {{6, 1, 1}, {14, 16, 8}, {14, 1024, 8}, {14, 1024, 3}, {13, 17, 1529}};
        for (auto &s : shapes) {
            test_stochastic<6>(s[0], s[1], s[2], true, false);
            test_stochastic<6>(s[0], s[1], s[2], false, false);
            test_stochastic<6>(s[0], s[1], s[2], false, true);
        }
        test_stochastic<4>(14, 33, 100, false, false);
        test_stochastic<2>(14, 33, 100, true, false);
        for (int dx_mode = 0; dx_mode <= 2; ++dx_mode) {
            bbhip_SetDxMode(dx_mode);
            test_stochastic<6>(40, 33, 300, false, false);
            test_differentiable<6>(24, 20, 1024, true);
            test_differentiable<6>(24, 20, 131, false);
            test_differentiable<4>(24, 20, 64, true);
        }
        bbhip_SetDxMode(0);
        test_packed_twin(40, 70, 20, 1000);
        test_packed_twin(27, 216, 36, 5000);
        test_binary(16, 16, 32);
        test_binary(70, 33, 1000);
        test_import_layer<6>();
        test_import_layer<5>();
        test_import_layer<4>();
        test_import_layer<3>();
        test_import_layer<2>();
        test_adam();
        test_conv_plumbing();
        test_convolution2d();
        test_stochastic_batch_normalization();
        test_max_lut();
        test_reduce_and_mean_squared_error();
        test_binary_modulation();
        test_pooling();
        test_shuffle();
        test_discrete<6>(24, 16, 200, false);
        test_discrete<6>(24, 16, 200, true);
        test_discrete<4>(12, 30, 1024, false);
        test_discrete<6>(6, 1, 39, false);
        test_tail();
        test_hand_off_through_files();
    }
    catch (std::exception const &e) {
        std::printf("exception: %s\n", e.what());
        return 1;
    }
    std::printf("%s (%d failed checks)\n", g_fail ? "FAILED" : "OK", g_fail);
    return g_fail ? 1 : 0;
}

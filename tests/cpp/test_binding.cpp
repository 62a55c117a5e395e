// The binding header include/bbcu_hip_binding.h against the reference's declarations (include/bbcu/bbcu.h), restated here
// as function-pointer types: every entry must have exactly the reference's parameter list, its template defaults (N = 6,
// T = float) and its stream default.  Compile-time checks; the program only prints how many it made.  With `--gpu` it also
// runs one StochasticLut6 forward + backward THROUGH the reference-named templates and compares with the bbhip_ entry
// points called directly (bit-identical: the wrappers only forward).
#include <cstdio>
#include <cstring>
#include <random>
#include <type_traits>
#include <vector>

#include "bbcu_hip_binding.h"

#define SAME(expr, ...) static_assert(std::is_same<decltype(expr), __VA_ARGS__>::value, #expr " has the reference's signature")

typedef cudaStream_t S;
// device manager and heap, bbcu.h:49-67
SAME(&bbcu_GetDeviceCount, int (*)(void));
SAME(&bbcu_GetDevice, int (*)(void));
SAME(&bbcu_SetDevice, void (*)(int));
SAME(&bbcu_SetHostOnly, void (*)(bool));
SAME(&bbcu_IsHostOnly, bool (*)(void));
SAME(&bbcu_IsDeviceAvailable, bool (*)(void));
SAME(&bbcu_LocalHeap_Malloc, void *(*)(size_t));
SAME(&bbcu_LocalHeap_Free, void (*)(void *));
SAME(&bbcu_LocalHeap_GetMaxAllocSize, size_t (*)(void));
SAME(&bbcu_LocalHeap_GetAllocatedSize, size_t (*)(void));
SAME(&bbcu_LocalHeap_GarbageCollect, void (*)(void));
// vector operations, bbcu.h:89-198
SAME(&bbcu_fp32_Vector_set, int (*)(float *, float, int, S));
SAME(&bbcu_fp32_Vector_add_ex, int (*)(float *, const float *, const float *, float, float, float, int, S));
SAME(&bbcu_fp32_Vector_mul_ex, int (*)(float *, const float *, const float *, float, float, int, S));
SAME(&bbcu_fp32_Vector_div_ex, int (*)(float *, float const *, float const *, float, float, float, float, int, S));
SAME(&bbcu_fp32_Vector_sqrt, int (*)(float *, float const *, int, S));
SAME(&bbcu_fp32_Vector_exp, int (*)(float *, float const *, int, S));
SAME(&bbcu_fp32_Vector_min, int (*)(float *, float const *, float const *, int, S));
SAME(&bbcu_fp32_Vector_min_v, int (*)(float *, float const *, float, int, S));
SAME(&bbcu_fp32_Vector_max, int (*)(float *, float const *, float const *, int, S));
SAME(&bbcu_fp32_Vector_max_v, int (*)(float *, float const *, float, int, S));
SAME(&bbcu_fp32_Vector_clamp, int (*)(float *, float const *, float, float, int, S));
// bbcu.h:246-258, 285-295, 321-361
SAME(&bbcu_ConvBitToReal<>, int (*)(int const *, float *, float, float, int, int, int, int, S));
SAME(&bbcu_ConvBitToReal<float>, int (*)(int const *, float *, float, float, int, int, int, int, S));
SAME(&bbcu_bit_BinatyLut6_Forward, int (*)(int const *, int *, int const *, int const *, int, int, int, S));
SAME(&bbcu_AverageLut_Forward<float>, int (*)(float const *, float *, int const *, int, int, int, int, bool, bool, S));
SAME(&bbcu_bit_AverageLut_Forward, int (*)(int const *, int *, int const *, int, int, int, int, S));
SAME(&bbcu_AverageLut_Backward<float>, int (*)(float const *, float *, int const *, int, int, int, int, int, S));
SAME(&bbcu_MaxLut_Forward<float>, int (*)(float const *, float *, int const *, int, int, int, int, bool, bool, S));
SAME(&bbcu_bit_MaxLut_Forward, int (*)(int const *, int *, int const *, int, int, int, int, S));
SAME(&bbcu_MaxLut_Backward<float>, int (*)(float const *, float const *, float *, int const *, int, int, int, int, int, bool, S));
SAME(&bbcu_bit_MaxLut_Backward<float>, int (*)(int const *, float const *, float *, int const *, int, int, int, int, int, int, S));

// the LUT entries, bbcu.h:518-761: one block of checks per width, and the default width
template <int N>
struct LutSignatures {
    SAME(&bbcu_fp32_DifferentiableLutN_ForwardTraining<N>,
         int (*)(float const *, float *, int const *, float const *, float *, float *, float *, float *, float, float, float, float, int, int, int, int, int, S));
    SAME(&bbcu_bit_fp32_DifferentiableLutN_ForwardTraining<N>,
         int (*)(int const *, int *, int const *, float const *, float *, float *, float *, float *, float, float, float, float, int, int, int, int, S));
    SAME(&bbcu_fp32_DifferentiableLutN_ForwardInference<N>,
         int (*)(float const *, float *, int const *, float const *, float const *, float const *, float, float, float, int, int, int, int, int, S));
    SAME(&bbcu_bit_fp32_DifferentiableLutN_ForwardInference<N>,
         int (*)(int const *, int *, int const *, float const *, float const *, float const *, float, float, float, int, int, int, int, S));
    SAME(&bbcu_fp32_DifferentiableLutN_Backward<N>,
         int (*)(float const *, float const *, float *, float *, int const *, int const *, float const *, float *, float const *, float const *, float *,
                 float *, float, float, float, int, int, int, int, int, int, int, int, int, S));
    SAME(&bbcu_bit_fp32_DifferentiableLutN_Backward<N>,
         int (*)(int const *, float const *, float *, float *, int const *, int const *, float const *, float *, float const *, float const *, float *,
                 float *, float, float, float, int, int, int, int, int, int, int, int, int, S));
    SAME(&bbcu_fp32_StochasticLut_Forward<N>, int (*)(const float *, float *, int const *, float const *, int, int, int, int, int, float, S));
    SAME(&bbcu_bit_fp32_StochasticLut_Forward<N>, int (*)(int const *, float *, int const *, float const *, int, int, int, int, int, float, S));
    SAME(&bbcu_bit_bit_fp32_StochasticLut_Forward<N>, int (*)(int const *, int *, int const *, float const *, int, int, int, int, float, S));
    SAME(&bbcu_fp32_StochasticLut_Backward<N>,
         int (*)(float const *, float const *, float *, float *, int const *, int const *, float const *, float *, int, int, int, int, int, int, int,
                 int, int, float, S));
    SAME(&bbcu_bit_fp32_StochasticLut_Backward<N>,
         int (*)(int const *, float const *, float *, float *, int const *, int const *, float const *, float *, int, int, int, int, int, int, int,
                 int, int, float, S));
    static constexpr int kChecks = 11;
};
template struct LutSignatures<2>;
template struct LutSignatures<3>;
template struct LutSignatures<4>;
template struct LutSignatures<5>;
template struct LutSignatures<6>;
// the default width is 6 (template <int N = 6>)
SAME(&bbcu_fp32_StochasticLut_Forward<>, decltype(&bbcu_fp32_StochasticLut_Forward<6>));
SAME(&bbcu_fp32_StochasticLut_Backward<>, decltype(&bbcu_fp32_StochasticLut_Backward<6>));
SAME(&bbcu_fp32_DifferentiableLutN_ForwardTraining<>, decltype(&bbcu_fp32_DifferentiableLutN_ForwardTraining<6>));
SAME(&bbcu_fp32_DifferentiableLutN_Backward<>, decltype(&bbcu_fp32_DifferentiableLutN_Backward<6>));

// bbcu.h:768-796, 1076-1186, 1506-1572
SAME(&bbcu_fp32_StochasticMaxPooling2x2_Forward, int (*)(float const *, float *, int, int, int, int, int, int, int, S));
SAME(&bbcu_fp32_StochasticMaxPooling2x2_Backward, int (*)(float const *, float const *, float *, int, int, int, int, int, int, int, S));
SAME(&bbcu_fp32_LossMeanSquaredError, int (*)(const float *, const float *, float *, double *, int, int, int, int, float, double, S));
SAME(&bbcu_fp32_StochasticBatchNormalization_ForwardTraining, int (*)(float const *, float *, float *, float *, float *, float *, float, float, float, int, int, int, S));
SAME(&bbcu_fp32_StochasticBatchNormalization_ReForward, int (*)(float const *, float *, float const *, float const *, float, float, int, int, int, S));
SAME(&bbcu_fp32_StochasticBatchNormalization_ForwardInference, int (*)(float const *, float *, float const *, float const *, float, float, int, int, int, S));
SAME(&bbcu_fp32_StochasticBatchNormalization_Backward, int (*)(float const *, float const *, float *, float const *, float const *, float, float, int, int, int, int, S));
// bbcu.h:1223-1276, 1337-1413
SAME(&bbcu_fp32_Binarize_Forward, int (*)(const float *, float *, float, float, float, int, int, int, S));
SAME(&bbcu_fp32_bit_Binarize_Forward, int (*)(float const *, int *, float, int, int, int, int, S));
SAME(&bbcu_fp32_HardTanh_Forward, int (*)(float const *, float *, float, float, int, int, int, S));
SAME(&bbcu_fp32_HardTanh_Backward, int (*)(const float *, const float *, float *, float, float, int, int, int, S));
SAME(&bbcu_RealToBinary_Forward<float>, int (*)(float const *, float *, unsigned int, unsigned int, float, float, unsigned int, unsigned int, unsigned int, unsigned int, unsigned int, bool, S));
SAME(&bbcu_RealToBinary_Forward<>, decltype(&bbcu_RealToBinary_Forward<float>));
SAME(&bbcu_bit_RealToBinary_Forward<float>, int (*)(float const *, int *, unsigned int, unsigned int, float, float, unsigned int, unsigned int, unsigned int, unsigned int, unsigned int, S));
SAME(&bbcu_fp32_BinaryToReal_Forward, int (*)(float const *, float *, int, int, int, int, int, int, S));
SAME(&bbcu_bit_fp32_BinaryToReal_Forward, int (*)(int const *, float *, int, int, int, int, int, int, S));
SAME(&bbcu_fp32_BinaryToReal_Backward, int (*)(float const *, float *, int, int, int, int, int, int, S));
// bbcu.h:949-1068
SAME(&bbcu_fp32_MaxPooling_Forward, int (*)(float const *, float *, int *, int, int, int, int, int, int, int, int, int, S));
SAME(&bbcu_bit_MaxPooling_Forward, int (*)(int const *, int *, int, int, int, int, int, int, int, int, int, S));
SAME(&bbcu_fp32_MaxPooling_Backward, int (*)(int const *, float const *, float *, int, int, int, int, int, int, int, int, int, S));
SAME(&bbcu_bit_fp32_MaxPooling_Backward, int (*)(int const *, float const *, float *, int, int, int, int, int, int, int, int, int, int, S));
SAME(&bbcu_fp32_UpSampling_Forward, int (*)(float const *, float *, int, int, int, int, int, int, int, int, S));
SAME(&bbcu_bit_UpSampling_Forward, int (*)(int const *, int *, int, int, int, int, int, int, int, int, S));
SAME(&bbcu_fp32_UpSampling_Backward, int (*)(float const *, float *, int, int, int, int, int, int, int, int, S));
SAME(&bbcu_fp32_Im2Col_Forward, int (*)(float const *, float *, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, float, S));
SAME(&bbcu_bit_Im2Col_Forward, int (*)(int const *, int *, int, int, int, int, int, int, int, int, int, int, int, int, int, int, int, S));
SAME(&bbcu_fp32_Im2Col_Backward, int (*)(float const *, float *, int, int, int, int, int, int, int, int, int, int, int, int, int, int, S));
SAME(&bbcu_fp32_Col2Im_Forward, int (*)(float const *, float *, int, int, int, int, int, int, S));
SAME(&bbcu_bit_Col2Im_Forward, int (*)(int const *, int *, int, int, int, int, int, int, S));
SAME(&bbcu_fp32_Col2Im_Backward, int (*)(float const *, float *, int, int, int, int, int, int, S));
SAME(&bbcu_Shuffle_Forward<int>, int (*)(int const *, int *, unsigned int, unsigned int, unsigned int, unsigned int, S));
SAME(&bbcu_Shuffle_Forward<float>, int (*)(float const *, float *, unsigned int, unsigned int, unsigned int, unsigned int, S));
SAME(&bbcu_Shuffle_Backward<int>, int (*)(int const *, int *, unsigned int, unsigned int, unsigned int, unsigned int, S));
SAME(&bbcu_Shuffle_Backward<float>, int (*)(float const *, float *, unsigned int, unsigned int, unsigned int, unsigned int, S));
SAME(&bbcu_LossSoftmaxCrossEntropy<float>, int (*)(float const *, float const *, float *, double *, float, int, int, int, int, S));
SAME(&bbcu_MetricsCategoricalAccuracy<float>, int (*)(float const *, float const *, int *, int *, int, int, int, int, S));
SAME(&bbcu_fp32_OptimizerAdam, int (*)(int, int const *, float *const *, float *const *, float *const *, float *const *, float, float, float, S));

// the stream argument may be left out, as every call site in the reference does (e.g. include/bb/StochasticLutN.h:463-474)
static int call_with_default_stream(float *d)
{
    return bbcu_fp32_Vector_set(d, 0.0f, 0);       // size 0: returns before any device work
}

static int run_on_gpu(void)
{
    constexpr int N = 6, NN = 64, I = 40, O = 33, F = 300, S_ = 320;
    std::mt19937_64 mt(7);
    std::uniform_real_distribution<float> uni(0.0f, 1.0f);
    std::vector<int> idx(O * N), rev;
    for (int o = 0; o < O; ++o) for (int i = 0; i < N; ++i) { idx[o * N + i] = (o * 7 + i * 5) % I; }
    // reverse table: [I][1 + max fan-out], count then node * N + k in ascending order
    std::vector<std::vector<int>> fan(I);
    for (int o = 0; o < O; ++o) for (int i = 0; i < N; ++i) { fan[idx[o * N + i]].push_back(o * N + i); }
    size_t maxf = 0; for (auto &v : fan) { maxf = v.size() > maxf ? v.size() : maxf; }
    int const rs = (int)maxf + 1;
    rev.assign((size_t)I * rs, 0);
    for (int in = 0; in < I; ++in) { rev[(size_t)in * rs] = (int)fan[in].size(); for (size_t t = 0; t < fan[in].size(); ++t) { rev[(size_t)in * rs + 1 + t] = fan[in][t]; } }
    std::vector<float> W(O * NN), x((size_t)I * S_), dy((size_t)O * S_);
    for (auto &v : W) { v = uni(mt); } for (auto &v : x) { v = uni(mt); } for (auto &v : dy) { v = uni(mt) - 0.5f; }
    void *dW_[2], *dx_[2], *y_[2], *px, *pdy, *pidx, *prev, *pW;
    bbcu::Malloc(&px, x.size() * 4); bbcu::Malloc(&pdy, dy.size() * 4); bbcu::Malloc(&pidx, idx.size() * 4);
    bbcu::Malloc(&prev, rev.size() * 4); bbcu::Malloc(&pW, W.size() * 4);
    bbcu::Memcpy(px, x.data(), x.size() * 4, 1); bbcu::Memcpy(pdy, dy.data(), dy.size() * 4, 1); bbcu::Memcpy(pidx, idx.data(), idx.size() * 4, 1);
    bbcu::Memcpy(prev, rev.data(), rev.size() * 4, 1); bbcu::Memcpy(pW, W.data(), W.size() * 4, 1);
    for (int v = 0; v < 2; ++v) {
        bbcu::Malloc(&dW_[v], W.size() * 4); bbcu::Malloc(&dx_[v], x.size() * 4); bbcu::Malloc(&y_[v], dy.size() * 4);
        if (bbhip_Memset(dW_[v], 0, W.size() * 4) || bbhip_Memset(dx_[v], 0, x.size() * 4) || bbhip_Memset(y_[v], 0, dy.size() * 4)) { return 1; }
    }
    // through the reference's names (width by default and explicitly, stream left out) ...
    bbcu_fp32_StochasticLut_Forward<>((float const *)px, (float *)y_[0], (int const *)pidx, (float const *)pW, O, F, S_, 0, 0, 0.25f);
    bbcu_fp32_StochasticLut_Backward<6>((float const *)px, (float const *)pdy, (float *)dx_[0], nullptr, (int const *)pidx, (int const *)prev,
                                        (float const *)pW, (float *)dW_[0], rs, I, O, F, S_, F, S_, 0, 0, 0.25f);
    // ... and the C ABI directly
    if (bbhip_fp32_StochasticLut_Forward(N, (float const *)px, (float *)y_[1], (int const *)pidx, (float const *)pW, O, F, S_, 0, 0, 0.25f, nullptr)) { return 1; }
    if (bbhip_fp32_StochasticLut_Backward(N, (float const *)px, (float const *)pdy, (float *)dx_[1], nullptr, (int const *)pidx, (int const *)prev,
                                          (float const *)pW, (float *)dW_[1], rs, I, O, F, S_, F, S_, 0, 0, 0.25f, nullptr)) { return 1; }
    if (bbhip_DeviceSynchronize()) { return 1; }
    int bad = 0;
    std::vector<float> a, b;
    auto same = [&](void *p, void *q, size_t n, char const *name) {
        a.resize(n); b.resize(n);
        bbcu::Memcpy(a.data(), p, n * 4, 2); bbcu::Memcpy(b.data(), q, n * 4, 2);
        double mx = 0; for (float v : a) { mx = v > mx ? v : (-v > mx ? -v : mx); }
        if (std::memcmp(a.data(), b.data(), n * 4) != 0 || mx == 0) { std::printf("FAIL: %s through the binding differs from the C ABI (or is all zero)\n", name); ++bad; }
    };
    same(y_[0], y_[1], dy.size(), "y"); same(dx_[0], dx_[1], x.size(), "dx"); same(dW_[0], dW_[1], W.size(), "dW");
    // a rejected call surfaces as an exception
    bool threw = false;
    try { bbcu_fp32_StochasticLut_Forward<6>(nullptr, nullptr, nullptr, nullptr, 1, 1, 1, 0, 0, 0.25f); } catch (std::runtime_error const &) { threw = true; }
    if (!threw) { std::printf("FAIL: a rejected call must throw\n"); ++bad; }
    for (int v = 0; v < 2; ++v) { bbcu::Free(dW_[v]); bbcu::Free(dx_[v]); bbcu::Free(y_[v]); }
    bbcu::Free(px); bbcu::Free(pdy); bbcu::Free(pidx); bbcu::Free(prev); bbcu::Free(pW);
    return bad;
}

int main(int argc, char **argv)
{
    int const checks = 11 + 11 + 6 + 4 + 5 * LutSignatures<6>::kChecks + 4 + 4 + 1 + 11 + 10 + 7 + 4;
    if (argc > 1 && !std::strcmp(argv[1], "--gpu")) {
        if (!bbcu_IsDeviceAvailable()) { std::printf("no device available\n"); return 2; }
        int const bad = run_on_gpu();
        std::printf("%s\n", bad ? "FAILED" : "binding on the GPU OK");
        return bad ? 1 : 0;
    }
    (void)&call_with_default_stream;
    std::printf("binding header: %d signatures equal the reference's declarations\n", checks);
    return 0;
}

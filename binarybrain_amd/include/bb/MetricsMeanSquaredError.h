// Mean squared error as a metric, accumulated over batches (reference API: include/bb/MetricsMeanSquaredError.h:20-91: Create,
// Clear, CalculateMetrics, GetMetrics = mean over frames of the mean over nodes of (t - y)^2, GetMetricsString "MSE").
// The reference loops over the buffers on the host; here the sums are taken on the device into 1024 partial sums.
#pragma once

#include "bb/MetricsCategoricalAccuracy.h"

namespace bb {

template <typename T = float>
class MetricsMeanSquaredError : public MetricsFunction {
    static_assert(std::is_same<T, float>::value, "the device path is fp32");
    static constexpr int kBufSize = 1024;

    Tensor_<double> m_accuracy_buf;
    index_t         m_frames = 0;

    MetricsMeanSquaredError()
    {
        m_accuracy_buf.Resize(kBufSize);
        m_accuracy_buf.FillZero();
    }

public:
    static std::string MetricsFunctionName(void) { return "MetricsMeanSquaredError"; }
    std::string GetMetricsFunctionName(void) const override { return MetricsFunctionName(); }
    std::string GetMetricsString(void) { return "MSE"; }

    static std::shared_ptr<MetricsMeanSquaredError> Create(void) { return std::shared_ptr<MetricsMeanSquaredError>(new MetricsMeanSquaredError); }

    void Clear(void) override { m_accuracy_buf.FillZero(); m_frames = 0; }

    double GetMetrics(void) const override
    {
        double sum = 0;
        auto p = m_accuracy_buf.LockConst();
        for (int i = 0; i < kBufSize; ++i) { sum += p[i]; }
        return sum / (double)m_frames;
    }

    void CalculateMetrics(FrameBuffer y_buf, FrameBuffer t_buf) override
    {
        BB_ASSERT(y_buf.GetType() == BB_TYPE_FP32 && t_buf.GetType() == BB_TYPE_FP32);
        BB_ASSERT(y_buf.GetNodeSize() == t_buf.GetNodeSize() && y_buf.GetFrameSize() == t_buf.GetFrameSize());
        BB_ASSERT(y_buf.GetFrameStride() == t_buf.GetFrameStride());
        if (!Manager::IsDeviceAvailable()) {
            throw Exception("MetricsMeanSquaredError: host-only execution is not provided by this library (device path only)");
        }
        auto y_ptr = y_buf.LockDeviceMemoryConst();
        auto t_ptr = t_buf.LockDeviceMemoryConst();
        auto a_ptr = m_accuracy_buf.LockDeviceMemory();
        CheckDevice(bbhip_fp32_MetricsMeanSquaredError((float const *)y_ptr.GetAddr(), (float const *)t_ptr.GetAddr(), (double *)a_ptr.GetAddr(), kBufSize,
                        (int)y_buf.GetNodeSize(), (int)y_buf.GetFrameSize(), (int)(y_buf.GetFrameStride() / sizeof(float)), nullptr),
                    "bbhip_fp32_MetricsMeanSquaredError");
        m_frames += y_buf.GetFrameSize();
    }
};

}  // namespace bb

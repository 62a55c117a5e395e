// Share of labeled pixels whose largest output sits on a channel with a positive target, accumulated over batches
// (reference API: include/bb/MetricsCategoricalAccuracy.h:20-180: Create, Clear, CalculateMetrics, GetMetrics).
#pragma once

#include "bb/Model.h"

namespace bb {

class MetricsFunction {
public:
    virtual ~MetricsFunction() {}
    virtual std::string GetMetricsFunctionName(void) const = 0;
    virtual void        Clear(void) = 0;
    virtual double      GetMetrics(void) const = 0;
    virtual void        CalculateMetrics(FrameBuffer y_buf, FrameBuffer t_buf) = 0;
};

template <typename T = float>
class MetricsCategoricalAccuracy : public MetricsFunction {
    static_assert(std::is_same<T, float>::value, "the device path is fp32");

    int m_accuracy = 0;
    int m_category_count = 0;

    MetricsCategoricalAccuracy() { Clear(); }

public:
    static std::string MetricsFunctionName(void) { return "MetricsCategoricalAccuracy"; }
    std::string GetMetricsFunctionName(void) const override { return MetricsFunctionName(); }

    static std::shared_ptr<MetricsCategoricalAccuracy> Create(void) { return std::shared_ptr<MetricsCategoricalAccuracy>(new MetricsCategoricalAccuracy); }

    void   Clear(void) override { m_accuracy = 0; m_category_count = 0; }
    double GetMetrics(void) const override { return (m_category_count == 0) ? 0 : (double)m_accuracy / m_category_count; }

    void CalculateMetrics(FrameBuffer y_buf, FrameBuffer t_buf) override
    {
        BB_ASSERT(y_buf.GetType() == BB_TYPE_FP32 && t_buf.GetType() == BB_TYPE_FP32);
        BB_ASSERT(y_buf.GetNodeSize() == t_buf.GetNodeSize() && y_buf.GetFrameSize() == t_buf.GetFrameSize());
        if (!Manager::IsDeviceAvailable()) {
            throw Exception("MetricsCategoricalAccuracy: host-only execution is not provided by this library (device path only)");
        }
        index_t const frame_size = t_buf.GetFrameSize(), node_size = t_buf.GetNodeSize();
        index_t const ch_size = t_buf.GetShape()[0], pix_size = node_size / ch_size;
        FrameBuffer accuracy_buf(frame_size, indices_t({1}), BB_TYPE_INT32);
        FrameBuffer category_buf(frame_size, indices_t({1}), BB_TYPE_INT32);
        {
            auto y_ptr = y_buf.LockDeviceMemoryConst();
            auto t_ptr = t_buf.LockDeviceMemoryConst();
            auto a_ptr = accuracy_buf.LockDeviceMemory(true);
            auto c_ptr = category_buf.LockDeviceMemory(true);
            CheckDevice(bbhip_fp32_MetricsCategoricalAccuracy((float const *)y_ptr.GetAddr(), (float const *)t_ptr.GetAddr(), (int *)a_ptr.GetAddr(),
                            (int *)c_ptr.GetAddr(), (int)pix_size, (int)ch_size, (int)frame_size, (int)(y_buf.GetFrameStride() / sizeof(float)), nullptr),
                        "bbhip_fp32_MetricsCategoricalAccuracy");
        }
        m_accuracy       += (int)accuracy_buf.Sum();
        m_category_count += (int)category_buf.Sum();
    }
};

}  // namespace bb

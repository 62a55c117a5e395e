// Softmax cross entropy over the channel index of [ch][pix] nodes, accumulated over batches (reference API:
// include/bb/LossSoftmaxCrossEntropy.h:20-226: Create, Clear, CalculateLoss -> dy, GetLoss = -sum(log(softmax) * t) / sum(t)).
// As on the reference's device path the target sum and the per-frame loss terms are added up on the host in double.
#pragma once

#include "bb/Model.h"

namespace bb {

class LossFunction {
public:
    virtual ~LossFunction() {}
    virtual std::string GetLossFunctionName(void) const = 0;
    virtual void        Clear(void) = 0;
    virtual double      GetLoss(void) const = 0;
    virtual FrameBuffer CalculateLoss(FrameBuffer y_buf, FrameBuffer t_buf, index_t batch_size) = 0;
};

template <typename T = float>
class LossSoftmaxCrossEntropy : public LossFunction {
    static_assert(std::is_same<T, float>::value, "the device path is fp32");

    Tensor_<double> m_loss_buf;
    double          m_loss = 0;
    double          m_frame_count = 0;

    LossSoftmaxCrossEntropy() { Clear(); }

public:
    static std::string LossFunctionName(void) { return "LossSoftmaxCrossEntropy"; }
    std::string GetLossFunctionName(void) const override { return LossFunctionName(); }

    static std::shared_ptr<LossSoftmaxCrossEntropy> Create(void) { return std::shared_ptr<LossSoftmaxCrossEntropy>(new LossSoftmaxCrossEntropy); }

    void   Clear(void) override { m_loss = 0; m_frame_count = 0; }
    double GetLoss(void) const override { return (m_frame_count == 0) ? 0 : m_loss / m_frame_count; }

    FrameBuffer CalculateLoss(FrameBuffer y_buf, FrameBuffer t_buf, index_t) override
    {
        BB_ASSERT(y_buf.GetType() == BB_TYPE_FP32 && t_buf.GetType() == BB_TYPE_FP32);
        BB_ASSERT(y_buf.GetNodeSize() == t_buf.GetNodeSize() && y_buf.GetFrameSize() == t_buf.GetFrameSize());
        if (!Manager::IsDeviceAvailable()) {
            throw Exception("LossSoftmaxCrossEntropy: host-only execution is not provided by this library (device path only)");
        }
        FrameBuffer dy_buf(y_buf.GetFrameSize(), y_buf.GetShape(), BB_TYPE_FP32);
        index_t const frame_size = t_buf.GetFrameSize(), node_size = t_buf.GetNodeSize();
        index_t const ch_size = t_buf.GetShape()[0], pix_size = node_size / ch_size;
        m_loss_buf.Resize(frame_size);
        T const t_sum = (T)t_buf.Sum();
        {
            auto y_ptr    = y_buf.LockDeviceMemoryConst();
            auto t_ptr    = t_buf.LockDeviceMemoryConst();
            auto dy_ptr   = dy_buf.LockDeviceMemory(true);
            auto loss_ptr = m_loss_buf.LockDeviceMemory(true);
            CheckDevice(bbhip_fp32_LossSoftmaxCrossEntropy((float const *)y_ptr.GetAddr(), (float const *)t_ptr.GetAddr(), (float *)dy_ptr.GetAddr(),
                            (double *)loss_ptr.GetAddr(), t_sum, (int)pix_size, (int)ch_size, (int)frame_size,
                            (int)(y_buf.GetFrameStride() / sizeof(float)), nullptr), "bbhip_fp32_LossSoftmaxCrossEntropy");
        }
        double loss_sum = 0;
        {
            auto p = m_loss_buf.LockConst();
            for (index_t frame = 0; frame < frame_size; ++frame) { loss_sum += p[frame]; }
        }
        m_loss += -loss_sum;
        m_frame_count += t_sum;
        return dy_buf;
    }
};

}  // namespace bb

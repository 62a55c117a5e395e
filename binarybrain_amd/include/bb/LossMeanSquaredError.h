// Mean squared error, accumulated over batches (reference API: include/bb/LossMeanSquaredError.h:20-185: Create(reduction),
// Clear, CalculateLoss -> dy, GetLoss).  Default reduction: dy = 2 (y - t) / (nodes * batch), loss = mean over nodes and frames;
// reduction "sum": dy = 2 (y - t), loss = the sum.  As on the reference's device path the loss is kept in 1024 partial sums in
// device memory and added up on the host when it is asked for.
#pragma once

#include "bb/LossSoftmaxCrossEntropy.h"

namespace bb {

template <typename T = float>
class LossMeanSquaredError : public LossFunction {
    static_assert(std::is_same<T, float>::value, "the device path is fp32");
    static constexpr int kLossBufSize = 1024;

    double          m_frames = 0;
    Tensor_<double> m_loss_buf;
    bool            m_reduction_sum = false;

public:
    struct create_t {
        std::string reduction;
    };

protected:
    explicit LossMeanSquaredError(create_t const &create) : m_reduction_sum(create.reduction == "sum")
    {
        m_loss_buf.Resize(kLossBufSize);
        m_loss_buf.FillZero();
    }

public:
    static std::string LossFunctionName(void) { return "LossMeanSquaredError"; }
    std::string GetLossFunctionName(void) const override { return LossFunctionName(); }

    static std::shared_ptr<LossMeanSquaredError> Create(create_t const &create) { return std::shared_ptr<LossMeanSquaredError>(new LossMeanSquaredError(create)); }
    static std::shared_ptr<LossMeanSquaredError> Create(std::string reduction = "")
    {
        create_t c;
        c.reduction = reduction;
        return Create(c);
    }

    void Clear(void) override { m_loss_buf.FillZero(); m_frames = 0; }

    double GetLoss(void) const override
    {
        double loss = 0;
        auto p = m_loss_buf.LockConst();
        for (int i = 0; i < kLossBufSize; ++i) { loss += p[i]; }
        return m_reduction_sum ? loss : loss / m_frames;
    }

    FrameBuffer CalculateLoss(FrameBuffer y_buf, FrameBuffer t_buf, index_t batch_size) override
    {
        BB_ASSERT(y_buf.GetType() == BB_TYPE_FP32 && t_buf.GetType() == BB_TYPE_FP32);
        BB_ASSERT(y_buf.GetNodeSize() == t_buf.GetNodeSize() && y_buf.GetFrameSize() == t_buf.GetFrameSize());
        BB_ASSERT(y_buf.GetFrameStride() == t_buf.GetFrameStride());
        if (!Manager::IsDeviceAvailable()) {
            throw Exception("LossMeanSquaredError: host-only execution is not provided by this library (device path only)");
        }
        index_t const frame_size = y_buf.GetFrameSize(), node_size = y_buf.GetNodeSize();
        FrameBuffer dy_buf(frame_size, y_buf.GetShape(), BB_TYPE_FP32);
        T      const grad_reduction = m_reduction_sum ? (T)1.0 : (T)1.0 / (T)(node_size * batch_size);
        double const loss_reduction = m_reduction_sum ? 1.0 : 1.0 / (double)node_size;
        auto y_ptr    = y_buf.LockDeviceMemoryConst();
        auto t_ptr    = t_buf.LockDeviceMemoryConst();
        auto dy_ptr   = dy_buf.LockDeviceMemory(true);
        auto loss_ptr = m_loss_buf.LockDeviceMemory();
        CheckDevice(bbhip_fp32_LossMeanSquaredError((float const *)y_ptr.GetAddr(), (float const *)t_ptr.GetAddr(), (float *)dy_ptr.GetAddr(),
                        (double *)loss_ptr.GetAddr(), kLossBufSize, (int)node_size, (int)frame_size, (int)(y_buf.GetFrameStride() / sizeof(float)),
                        (float)2 * grad_reduction, loss_reduction, nullptr), "bbhip_fp32_LossMeanSquaredError");
        m_frames += (double)frame_size;
        return dy_buf;
    }
};

}  // namespace bb

// 2 x 2 pooling of probabilities: the output is the probability that at least one of the four (independent, binary)
// inputs is 1, y = 1 - prod(1 - x); on {0,1} inputs it is max pooling (reference API:
// include/bb/StochasticMaxPooling2x2.h:23-320).  Shapes {c, h, w} -> {c, ceil(h/2), ceil(w/2)}.
#pragma once

#include "bb/Model.h"

namespace bb {

template <typename FT = float, typename BT = float>
class StochasticMaxPooling2x2 : public Model {
    static_assert(std::is_same<FT, float>::value && std::is_same<BT, float>::value, "the device path is fp32");

    bool      m_host_only = false;
    indices_t m_input_shape, m_output_shape;
    index_t   m_input_c_size = 0, m_input_h_size = 0, m_input_w_size = 0;
    index_t   m_output_h_size = 0, m_output_w_size = 0;

    void CommandProc(std::vector<std::string> args) override
    {
        Model::CommandProc(args);
        if (args.size() == 2 && args[0] == "host_only") { m_host_only = EvalBool(args[1]); }
    }

    StochasticMaxPooling2x2() {}

public:
    static std::string ModelName(void) { return "StochasticMaxPooling2x2"; }
    std::string GetModelName(void) const override { return ModelName(); }

    static std::shared_ptr<StochasticMaxPooling2x2> Create(void) { return std::shared_ptr<StochasticMaxPooling2x2>(new StochasticMaxPooling2x2); }

    indices_t SetInputShape(indices_t shape) override
    {
        BB_ASSERT(shape.size() == 3);
        m_input_c_size = shape[0]; m_input_h_size = shape[1]; m_input_w_size = shape[2];
        m_output_w_size = (m_input_w_size + 2 - 1) / 2;
        m_output_h_size = (m_input_h_size + 2 - 1) / 2;
        m_input_shape = shape;
        m_output_shape = indices_t({m_input_c_size, m_output_h_size, m_output_w_size});
        return m_output_shape;
    }
    indices_t GetInputShape(void) const override { return m_input_shape; }
    indices_t GetOutputShape(void) const override { return m_output_shape; }

    FrameBuffer Forward(FrameBuffer x_buf, bool train = true) override
    {
        BB_ASSERT(x_buf.GetType() == BB_TYPE_FP32);
        if (x_buf.GetShape() != m_input_shape) { SetInputShape(x_buf.GetShape()); }
        if (m_host_only || !x_buf.IsDeviceAvailable()) { throw std::runtime_error("StochasticMaxPooling2x2: no host path in this build"); }
        if (train) { PushFrameBuffer(x_buf); }
        FrameBuffer y_buf(x_buf.GetFrameSize(), m_output_shape, BB_TYPE_FP32);
        BB_ASSERT(y_buf.GetFrameStride() == x_buf.GetFrameStride());
        auto px = x_buf.LockDeviceMemoryConst();
        auto py = y_buf.LockDeviceMemory(true);
        CheckDevice(bbhip_fp32_StochasticMaxPooling2x2_Forward((float const *)px.GetAddr(), (float *)py.GetAddr(), (int)m_input_w_size, (int)m_input_h_size,
                (int)m_output_w_size, (int)m_output_h_size, (int)m_input_c_size, (int)y_buf.GetFrameSize(), (int)(y_buf.GetFrameStride() / 4), nullptr),
                "bbhip_fp32_StochasticMaxPooling2x2_Forward");
        return y_buf;
    }

    FrameBuffer Backward(FrameBuffer dy_buf) override
    {
        if (dy_buf.Empty()) { return FrameBuffer(); }
        BB_ASSERT(dy_buf.GetType() == BB_TYPE_FP32 && dy_buf.GetShape().size() == 3);
        if (m_host_only || !dy_buf.IsDeviceAvailable()) { throw std::runtime_error("StochasticMaxPooling2x2: no host path in this build"); }
        FrameBuffer x_buf = PopFrameBuffer();
        FrameBuffer dx_buf(dy_buf.GetFrameSize(), m_input_shape, BB_TYPE_FP32);
        auto px  = x_buf.LockDeviceMemoryConst();
        auto pdy = dy_buf.LockDeviceMemoryConst();
        auto pdx = dx_buf.LockDeviceMemory(true);
        CheckDevice(bbhip_fp32_StochasticMaxPooling2x2_Backward((float const *)px.GetAddr(), (float const *)pdy.GetAddr(), (float *)pdx.GetAddr(),
                (int)m_input_w_size, (int)m_input_h_size, (int)m_output_w_size, (int)m_output_h_size, (int)m_input_c_size,
                (int)dy_buf.GetFrameSize(), (int)(dy_buf.GetFrameStride() / 4), nullptr), "bbhip_fp32_StochasticMaxPooling2x2_Backward");
        return dx_buf;
    }
};

}  // namespace bb

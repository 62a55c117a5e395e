// Col2Im: the inverse regrouping of Im2Col on the output side of a convolution — frames (image, y, x) of c-node
// vectors become images of shape {c, h, w} (reference API: include/bb/ConvolutionCol2Im.h:22-300).
#pragma once

#include "bb/Model.h"

namespace bb {

template <typename FT = float, typename BT = float>
class ConvolutionCol2Im : public Model {
    static_assert(std::is_same<BT, float>::value, "gradients are fp32");

    bool      m_host_only = false;
    indices_t m_input_shape;
    index_t   m_c_size = 1, m_h_size = 1, m_w_size = 1;

    void CommandProc(std::vector<std::string> args) override
    {
        Model::CommandProc(args);
        if (args.size() == 2 && args[0] == "host_only") { m_host_only = EvalBool(args[1]); }
    }

public:
    struct create_t {
        index_t h_size = 1;
        index_t w_size = 1;
    };

protected:
    explicit ConvolutionCol2Im(create_t const &create) : m_h_size(create.h_size), m_w_size(create.w_size) {}

    // version 1 | Model part | image height, width | input shape (reference: include/bb/ConvolutionCol2Im.h:334-367)
    void DumpObjectData(std::ostream &os) const override
    {
        SaveValue(os, (std::int64_t)1);
        Model::DumpObjectData(os);
        SaveValue(os, (std::int64_t)m_h_size);
        SaveValue(os, (std::int64_t)m_w_size);
        SaveIndices(os, m_input_shape);
    }
    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = -1, h = 0, w = 0;
        LoadValue(is, ver);
        BB_ASSERT(ver == 1);
        Model::LoadObjectData(is);
        LoadValue(is, h);
        LoadValue(is, w);
        BB_ASSERT(is.good() && h >= 1 && w >= 1);
        m_h_size = (index_t)h; m_w_size = (index_t)w;
        m_input_shape = LoadIndices(is);
        m_c_size = CalcShapeSize(m_input_shape);
    }

public:
    static std::string ModelName(void)  { return "ConvolutionCol2Im"; }
    static std::string ObjectName(void) { return ModelName() + "_" + DataType<FT>::Name() + "_" + DataType<BT>::Name(); }
    std::string GetModelName(void) const override  { return ModelName(); }
    std::string GetObjectName(void) const override { return ObjectName(); }

    static std::shared_ptr<ConvolutionCol2Im> Create(create_t const &create) { return std::shared_ptr<ConvolutionCol2Im>(new ConvolutionCol2Im(create)); }
    static std::shared_ptr<ConvolutionCol2Im> Create(index_t h_size = 1, index_t w_size = 1)
    {
        create_t c; c.h_size = h_size; c.w_size = w_size;
        return Create(c);
    }

    void SetOutputSize(index_t h_size, index_t w_size) { m_h_size = h_size; m_w_size = w_size; }
    index_t GetChannel(void) const { return m_c_size; }
    index_t GetHeight(void) const { return m_h_size; }
    index_t GetWidth(void) const { return m_w_size; }

    indices_t SetInputShape(indices_t shape) override
    {
        m_input_shape = shape;
        m_c_size = CalcShapeSize(shape);
        return indices_t({m_c_size, m_h_size, m_w_size});
    }
    indices_t GetInputShape(void) const override { return m_input_shape; }
    indices_t GetOutputShape(void) const override { return indices_t({m_c_size, m_h_size, m_w_size}); }

    FrameBuffer Forward(FrameBuffer x_buf, bool train = true) override
    {
        (void)train;
        BB_ASSERT(x_buf.GetType() == DataType<FT>::type);
        if (x_buf.GetShape() != m_input_shape) { SetInputShape(x_buf.GetShape()); }       // the reference leaves this to the caller
        if (m_host_only || !x_buf.IsDeviceAvailable()) { throw std::runtime_error("ConvolutionCol2Im: no host path in this build"); }
        index_t const input_frame_size = x_buf.GetFrameSize();
        BB_ASSERT(input_frame_size % (m_h_size * m_w_size) == 0);
        index_t const output_frame_size = input_frame_size / (m_h_size * m_w_size);
        FrameBuffer y_buf(output_frame_size, indices_t({m_c_size, m_h_size, m_w_size}), x_buf.GetType());
        auto px = x_buf.LockDeviceMemoryConst();
        auto py = y_buf.LockDeviceMemory(true);
        if (std::is_same<FT, Bit>::value) {
            CheckDevice(bbhip_bit_Col2Im_Forward((int const *)px.GetAddr(), (int *)py.GetAddr(), (int)m_w_size, (int)m_h_size, (int)m_c_size,
                    (int)(x_buf.GetFrameStride() / 4), (int)output_frame_size, (int)(y_buf.GetFrameStride() / 4), nullptr), "bbhip_bit_Col2Im_Forward");
        }
        else {
            CheckDevice(bbhip_fp32_Col2Im_Forward((float const *)px.GetAddr(), (float *)py.GetAddr(), (int)m_w_size, (int)m_h_size, (int)m_c_size,
                    (int)(x_buf.GetFrameStride() / 4), (int)output_frame_size, (int)(y_buf.GetFrameStride() / 4), nullptr), "bbhip_fp32_Col2Im_Forward");
        }
        return y_buf;
    }

    FrameBuffer Backward(FrameBuffer dy_buf) override
    {
        if (dy_buf.Empty()) { return dy_buf; }
        BB_ASSERT(dy_buf.GetType() == BB_TYPE_FP32);
        if (m_host_only || !dy_buf.IsDeviceAvailable()) { throw std::runtime_error("ConvolutionCol2Im: no host path in this build"); }
        index_t const output_frame_size = dy_buf.GetFrameSize();
        index_t const input_frame_size = output_frame_size * (m_h_size * m_w_size);
        FrameBuffer dx_buf(input_frame_size, indices_t({m_c_size}), BB_TYPE_FP32);
        auto pdy = dy_buf.LockDeviceMemoryConst();
        auto pdx = dx_buf.LockDeviceMemory(true);
        CheckDevice(bbhip_fp32_Col2Im_Backward((float const *)pdy.GetAddr(), (float *)pdx.GetAddr(), (int)m_w_size, (int)m_h_size, (int)m_c_size,
                (int)(dx_buf.GetFrameStride() / 4), (int)output_frame_size, (int)(dy_buf.GetFrameStride() / 4), nullptr), "bbhip_fp32_Col2Im_Backward");
        return dx_buf;
    }
};

}  // namespace bb

// BinaryToReal: the exit of a binary network.  Output node o of output frame g is the share of ones among the input nodes
// o, O + o, 2 O + o, ... and the frame_integration_size input frames that fold into g; the backward pass hands every one of
// them dy * O / (I * frame_integration_size) (reference API: include/bb/BinaryToReal.h:30-383: Create(frame_integration_size,
// [depth_integration_size,] output_shape), SetFrameIntegrationSize, SetInputShape, Forward, Backward, commands "binary",
// "host_only").  With depth_integration_size > 0 the output shape is the input shape with its first extent divided by it.
// Serialized as  version 1 | Model part | host_only | binary_mode | frame integration | depth integration | input shape |
// output shape  (reference :352-380).
#pragma once

#include "bb/Model.h"

namespace bb {

template <typename BinType = float, typename RealType = float>
class BinaryToReal : public Model {
    static_assert(std::is_same<RealType, float>::value, "outputs and gradients are fp32");
    static_assert(std::is_same<BinType, float>::value || std::is_same<BinType, Bit>::value, "inputs are fp32 or packed bits");

    bool      m_host_only = false;
    bool      m_binary_mode = true;
    index_t   m_frame_integration_size = 1;
    index_t   m_depth_integration_size = 0;
    indices_t m_input_shape, m_output_shape;

public:
    struct create_t {
        indices_t output_shape;
        index_t   frame_integration_size = 1;
        index_t   depth_integration_size = 0;       // 0: the output shape is given
    };

protected:
    explicit BinaryToReal(create_t const &create)
        : m_frame_integration_size(create.frame_integration_size), m_depth_integration_size(create.depth_integration_size),
          m_output_shape(create.output_shape)
    {
        BB_ASSERT(m_frame_integration_size > 0 && m_depth_integration_size >= 0);
    }

    void CommandProc(std::vector<std::string> args) override
    {
        Model::CommandProc(args);
        if (args.size() == 2 && args[0] == "binary")    { m_binary_mode = EvalBool(args[1]); }
        if (args.size() == 2 && args[0] == "host_only") { m_host_only = EvalBool(args[1]); }
    }

    void DumpObjectData(std::ostream &os) const override
    {
        SaveValue(os, (std::int64_t)1);
        Model::DumpObjectData(os);
        SaveValue(os, m_host_only);
        SaveValue(os, m_binary_mode);
        SaveValue(os, (std::int64_t)m_frame_integration_size);
        SaveValue(os, (std::int64_t)m_depth_integration_size);
        SaveIndices(os, m_input_shape);
        SaveIndices(os, m_output_shape);
    }

    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = -1, frames = -1, depth = -1;
        LoadValue(is, ver);
        BB_ASSERT(ver == 1);
        Model::LoadObjectData(is);
        LoadValue(is, m_host_only);
        LoadValue(is, m_binary_mode);
        LoadValue(is, frames);
        LoadValue(is, depth);
        m_input_shape = LoadIndices(is);
        m_output_shape = LoadIndices(is);
        BB_ASSERT(is.good() && frames > 0 && depth >= 0);
        m_frame_integration_size = (index_t)frames; m_depth_integration_size = (index_t)depth;
        index_t const I = CalcShapeSize(m_input_shape), O = CalcShapeSize(m_output_shape);
        BB_ASSERT(m_input_shape.empty() || (O > 0 && I % O == 0));
    }

    void RequireDevice(FrameBuffer const &buf, char const *what) const
    {
        if (m_host_only || !buf.IsDeviceAvailable() || !Manager::IsDeviceAvailable()) {
            throw Exception(std::string(what) + ": host-only execution is not provided by this library (device path only)");
        }
    }

public:
    static std::string ModelName(void)  { return "BinaryToReal"; }
    static std::string ObjectName(void) { return ModelName() + "_" + DataType<BinType>::Name() + "_" + DataType<RealType>::Name(); }
    std::string GetModelName(void) const override  { return ModelName(); }
    std::string GetObjectName(void) const override { return ObjectName(); }

    static std::shared_ptr<BinaryToReal> Create(create_t const &create) { return std::shared_ptr<BinaryToReal>(new BinaryToReal(create)); }
    static std::shared_ptr<BinaryToReal> Create(index_t frame_integration_size, indices_t output_shape)
    {
        create_t c;
        c.output_shape = output_shape; c.frame_integration_size = frame_integration_size;
        return Create(c);
    }
    static std::shared_ptr<BinaryToReal> Create(index_t frame_integration_size = 1, index_t depth_integration_size = 0,
                                                indices_t output_shape = indices_t())
    {
        create_t c;
        c.output_shape = output_shape; c.frame_integration_size = frame_integration_size; c.depth_integration_size = depth_integration_size;
        return Create(c);
    }

    void SetFrameIntegrationSize(index_t frame_integration_size) { BB_ASSERT(frame_integration_size > 0); m_frame_integration_size = frame_integration_size; }
    index_t GetFrameIntegrationSize(void) const { return m_frame_integration_size; }

    indices_t SetInputShape(indices_t shape) override
    {
        if (shape == m_input_shape) { return m_output_shape; }
        m_input_shape = shape;
        if (m_output_shape.empty()) { m_output_shape = m_input_shape; }
        if (m_depth_integration_size > 0) {
            if (m_output_shape.empty() || CalcShapeSize(m_output_shape) != CalcShapeSize(m_input_shape) * m_depth_integration_size) {
                m_output_shape = m_input_shape;
                BB_ASSERT(!m_output_shape.empty() && m_output_shape[0] % m_depth_integration_size == 0);
                m_output_shape[0] /= m_depth_integration_size;
            }
        }
        BB_ASSERT(CalcShapeSize(m_output_shape) > 0 && CalcShapeSize(m_input_shape) >= CalcShapeSize(m_output_shape));
        BB_ASSERT(CalcShapeSize(m_input_shape) % CalcShapeSize(m_output_shape) == 0);
        return m_output_shape;
    }
    indices_t GetInputShape(void) const override  { return m_input_shape; }
    indices_t GetOutputShape(void) const override { return m_output_shape; }

    FrameBuffer Forward(FrameBuffer x_buf, bool = true) override
    {
        if (std::is_same<BinType, RealType>::value && !m_binary_mode) { return x_buf; }        // reference :207-209
        BB_ASSERT(x_buf.GetType() == DataType<BinType>::type);
        RequireDevice(x_buf, "BinaryToReal::Forward");
        if (x_buf.GetShape() != m_input_shape) { SetInputShape(x_buf.GetShape()); }
        BB_ASSERT(x_buf.GetFrameSize() % m_frame_integration_size == 0);
        FrameBuffer y_buf(x_buf.GetFrameSize() / m_frame_integration_size, m_output_shape, BB_TYPE_FP32);
        int const node_mux = (int)(CalcShapeSize(m_input_shape) / CalcShapeSize(m_output_shape));
        auto x_ptr = x_buf.LockDeviceMemoryConst();
        auto y_ptr = y_buf.LockDeviceMemory(true);
        if (DataType<BinType>::type == BB_TYPE_BIT) {
            CheckDevice(bbhip_bit_fp32_BinaryToReal_Forward((int const *)x_ptr.GetAddr(), (float *)y_ptr.GetAddr(), node_mux,
                            (int)m_frame_integration_size, (int)y_buf.GetNodeSize(), (int)(x_buf.GetFrameStride() / sizeof(int)),
                            (int)y_buf.GetFrameSize(), (int)(y_buf.GetFrameStride() / sizeof(float)), nullptr), "bbhip_bit_fp32_BinaryToReal_Forward");
        }
        else {
            CheckDevice(bbhip_fp32_BinaryToReal_Forward((float const *)x_ptr.GetAddr(), (float *)y_ptr.GetAddr(), node_mux,
                            (int)m_frame_integration_size, (int)y_buf.GetNodeSize(), (int)(x_buf.GetFrameStride() / sizeof(float)),
                            (int)y_buf.GetFrameSize(), (int)(y_buf.GetFrameStride() / sizeof(float)), nullptr), "bbhip_fp32_BinaryToReal_Forward");
        }
        return y_buf;
    }

    FrameBuffer Backward(FrameBuffer dy_buf) override
    {
        if (dy_buf.Empty()) { return dy_buf; }
        if (!m_binary_mode || (m_frame_integration_size == 1 && m_input_shape == m_output_shape)) { return dy_buf; }   // reference :303-305
        BB_ASSERT(dy_buf.GetType() == BB_TYPE_FP32 && dy_buf.GetNodeSize() == this->GetOutputNodeSize());
        RequireDevice(dy_buf, "BinaryToReal::Backward");
        FrameBuffer dx_buf(dy_buf.GetFrameSize() * m_frame_integration_size, m_input_shape, BB_TYPE_FP32);
        auto dy_ptr = dy_buf.LockDeviceMemoryConst();
        auto dx_ptr = dx_buf.LockDeviceMemory(true);
        CheckDevice(bbhip_fp32_BinaryToReal_Backward((float const *)dy_ptr.GetAddr(), (float *)dx_ptr.GetAddr(),
                        (int)(CalcShapeSize(m_input_shape) / CalcShapeSize(m_output_shape)), (int)m_frame_integration_size,
                        (int)dy_buf.GetNodeSize(), (int)(dx_buf.GetFrameStride() / sizeof(float)), (int)dy_buf.GetFrameSize(),
                        (int)(dy_buf.GetFrameStride() / sizeof(float)), nullptr), "bbhip_fp32_BinaryToReal_Backward");
        return dx_buf;
    }
};

}  // namespace bb

// Reduce: output node o is the mean of the input nodes o, O + o, 2 O + o, ...; the usual last layer of a LUT classifier whose
// final LUT layer has several nodes per class (reference API: include/bb/Reduce.h:21-332: Create(output_shape | output_node,
// integration_size), SetInputShape, Forward, Backward).  With integration_size > 0 the output shape follows from the input shape
// (its first extent divided by integration_size).  The reference runs this layer on the host; here it is a device kernel.
// Serialized as  version 1 | Model part | host_only | input shape | output shape | int64 integration_size  (reference :287-317).
#pragma once

#include "bb/Model.h"

namespace bb {

template <typename BinType = float, typename RealType = float>
class Reduce : public Model {
    static_assert(std::is_same<RealType, float>::value, "outputs and gradients are fp32");
    static_assert(std::is_same<BinType, float>::value || std::is_same<BinType, Bit>::value, "inputs are fp32 or packed bits");

    bool      m_host_only = false;
    indices_t m_input_shape, m_output_shape;
    index_t   m_integration_size = 0;

public:
    struct create_t {
        indices_t output_shape;
        index_t   integration_size = 0;
    };

protected:
    explicit Reduce(create_t const &create) : m_output_shape(create.output_shape), m_integration_size(create.integration_size) {}

    void CommandProc(std::vector<std::string> args) override
    {
        Model::CommandProc(args);
        if (args.size() == 2 && args[0] == "host_only") { m_host_only = EvalBool(args[1]); }
    }

    void DumpObjectData(std::ostream &os) const override
    {
        SaveValue(os, (std::int64_t)1);
        Model::DumpObjectData(os);
        SaveValue(os, m_host_only);
        SaveIndices(os, m_input_shape);
        SaveIndices(os, m_output_shape);
        SaveValue(os, (std::int64_t)m_integration_size);
    }

    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = -1, integration = -1;
        LoadValue(is, ver);
        BB_ASSERT(ver == 1);
        Model::LoadObjectData(is);
        LoadValue(is, m_host_only);
        m_input_shape = LoadIndices(is);
        m_output_shape = LoadIndices(is);
        LoadValue(is, integration);
        BB_ASSERT(is.good() && integration >= 0);
        m_integration_size = (index_t)integration;
        index_t const I = CalcShapeSize(m_input_shape), O = CalcShapeSize(m_output_shape);
        BB_ASSERT(m_input_shape.empty() || (O > 0 && I % O == 0));
    }

public:
    static std::string ModelName(void)  { return "Reduce"; }
    static std::string ObjectName(void) { return ModelName() + "_" + DataType<BinType>::Name() + "_" + DataType<RealType>::Name(); }
    std::string GetModelName(void) const override  { return ModelName(); }
    std::string GetObjectName(void) const override { return ObjectName(); }

    static std::shared_ptr<Reduce> Create(create_t const &create) { return std::shared_ptr<Reduce>(new Reduce(create)); }
    static std::shared_ptr<Reduce> Create(index_t output_node, index_t integration_size = 0)
    {
        create_t c;
        c.output_shape = indices_t({output_node}); c.integration_size = integration_size;
        return Create(c);
    }
    static std::shared_ptr<Reduce> Create(indices_t output_shape, index_t integration_size = 0)
    {
        create_t c;
        c.output_shape = output_shape; c.integration_size = integration_size;
        return Create(c);
    }
    static std::shared_ptr<Reduce> Create(void) { return Create(create_t()); }

    indices_t SetInputShape(indices_t shape) override
    {
        if (shape == m_input_shape) { return m_output_shape; }
        m_input_shape = shape;
        if (m_integration_size > 0) {
            m_output_shape = shape;
            BB_ASSERT(!shape.empty() && m_output_shape[0] % m_integration_size == 0);
            m_output_shape[0] /= m_integration_size;
        }
        BB_ASSERT(CalcShapeSize(m_output_shape) > 0 && CalcShapeSize(m_input_shape) >= CalcShapeSize(m_output_shape));
        BB_ASSERT(CalcShapeSize(m_input_shape) % CalcShapeSize(m_output_shape) == 0);
        return m_output_shape;
    }
    indices_t GetInputShape(void) const override  { return m_input_shape; }
    indices_t GetOutputShape(void) const override { return m_output_shape; }

    FrameBuffer Forward(FrameBuffer x_buf, bool = true) override
    {
        BB_ASSERT(x_buf.GetType() == DataType<BinType>::type);
        if (m_host_only || !Manager::IsDeviceAvailable()) {
            throw Exception("Reduce::Forward: host-only execution is not provided by this library (device path only)");
        }
        if (x_buf.GetShape() != m_input_shape) { SetInputShape(x_buf.GetShape()); }
        FrameBuffer y_buf(x_buf.GetFrameSize(), m_output_shape, BB_TYPE_FP32);
        auto x_ptr = x_buf.LockDeviceMemoryConst();
        auto y_ptr = y_buf.LockDeviceMemory(true);
        if (DataType<BinType>::type == BB_TYPE_BIT) {
            CheckDevice(bbhip_bit_fp32_Reduce_Forward((int const *)x_ptr.GetAddr(), (float *)y_ptr.GetAddr(), (int)x_buf.GetNodeSize(),
                            (int)y_buf.GetNodeSize(), (int)y_buf.GetFrameSize(), (int)(x_buf.GetFrameStride() / sizeof(int)),
                            (int)(y_buf.GetFrameStride() / sizeof(float)), nullptr), "bbhip_bit_fp32_Reduce_Forward");
        }
        else {
            BB_ASSERT(x_buf.GetFrameStride() == y_buf.GetFrameStride());
            CheckDevice(bbhip_fp32_Reduce_Forward((float const *)x_ptr.GetAddr(), (float *)y_ptr.GetAddr(), (int)x_buf.GetNodeSize(),
                            (int)y_buf.GetNodeSize(), (int)y_buf.GetFrameSize(), (int)(y_buf.GetFrameStride() / sizeof(float)), nullptr),
                        "bbhip_fp32_Reduce_Forward");
        }
        return y_buf;
    }

    FrameBuffer Backward(FrameBuffer dy_buf) override
    {
        if (dy_buf.Empty()) { return FrameBuffer(); }
        BB_ASSERT(dy_buf.GetType() == BB_TYPE_FP32 && dy_buf.GetNodeSize() == this->GetOutputNodeSize());
        if (m_host_only || !Manager::IsDeviceAvailable()) {
            throw Exception("Reduce::Backward: host-only execution is not provided by this library (device path only)");
        }
        FrameBuffer dx_buf(dy_buf.GetFrameSize(), m_input_shape, BB_TYPE_FP32);
        BB_ASSERT(dx_buf.GetFrameStride() == dy_buf.GetFrameStride());
        auto dy_ptr = dy_buf.LockDeviceMemoryConst();
        auto dx_ptr = dx_buf.LockDeviceMemory(true);
        CheckDevice(bbhip_fp32_Reduce_Backward((float const *)dy_ptr.GetAddr(), (float *)dx_ptr.GetAddr(), (int)dx_buf.GetNodeSize(),
                        (int)dy_buf.GetNodeSize(), (int)dy_buf.GetFrameSize(), (int)(dy_buf.GetFrameStride() / sizeof(float)), nullptr),
                    "bbhip_fp32_Reduce_Backward");
        return dx_buf;
    }
};

}  // namespace bb

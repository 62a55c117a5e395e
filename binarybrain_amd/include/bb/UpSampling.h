// UpSampling: every pixel becomes a filter_h x filter_w block — all of it (fill), or only the block's position
// (filter_h / 2, filter_w / 2) with zeros around; the backward pass sums the gradient over the block, or takes that one
// position (reference API: include/bb/UpSampling.h:22-405: Create(filter_h_size, filter_w_size, fill), SetInputShape,
// Forward, Backward).  Shapes {c, h, w} -> {c, h fh, w fw}; fp32 or packed-bit images, fp32 gradients.
// Serialized as  version 1 | Model part | host_only | input shape | filter h, w | fill  (reference :357-383).
#pragma once

#include <stack>

#include "bb/Model.h"

namespace bb {

template <typename FT = float, typename BT = float>
class UpSampling : public Model {
    static_assert(std::is_same<BT, float>::value, "gradients are fp32");
    static_assert(std::is_same<FT, float>::value || std::is_same<FT, Bit>::value, "images are fp32 or packed bits");

    bool      m_host_only = false;
    indices_t m_input_shape;
    std::stack<indices_t> m_shapes;
    index_t   m_filter_h_size = 1, m_filter_w_size = 1;
    bool      m_fill = true;

public:
    struct create_t {
        index_t filter_h_size = 1;
        index_t filter_w_size = 1;
        bool    fill = true;
    };

protected:
    explicit UpSampling(create_t const &create) : m_filter_h_size(create.filter_h_size), m_filter_w_size(create.filter_w_size), m_fill(create.fill)
    {
        BB_ASSERT(m_filter_h_size > 0 && m_filter_w_size > 0);
    }

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
        SaveValue(os, (std::int64_t)m_filter_h_size);
        SaveValue(os, (std::int64_t)m_filter_w_size);
        SaveValue(os, m_fill);
    }

    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = -1, fh = -1, fw = -1;
        LoadValue(is, ver);
        BB_ASSERT(ver == 1);
        Model::LoadObjectData(is);
        LoadValue(is, m_host_only);
        m_input_shape = LoadIndices(is);
        LoadValue(is, fh);
        LoadValue(is, fw);
        LoadValue(is, m_fill);
        BB_ASSERT(is.good() && fh > 0 && fw > 0 && (m_input_shape.empty() || m_input_shape.size() == 3));
        m_filter_h_size = (index_t)fh; m_filter_w_size = (index_t)fw;
    }

    void RequireDevice(FrameBuffer const &buf, char const *what) const
    {
        if (m_host_only || !buf.IsDeviceAvailable() || !Manager::IsDeviceAvailable()) {
            throw Exception(std::string(what) + ": host-only execution is not provided by this library (device path only)");
        }
    }

    indices_t OutputShapeOf(indices_t shape) const
    {
        if (shape.size() == 3) { shape[1] *= m_filter_h_size; shape[2] *= m_filter_w_size; }
        return shape;
    }

public:
    static std::string ModelName(void)  { return "UpSampling"; }
    static std::string ObjectName(void) { return ModelName() + "_" + DataType<FT>::Name() + "_" + DataType<BT>::Name(); }
    std::string GetModelName(void) const override  { return ModelName(); }
    std::string GetObjectName(void) const override { return ObjectName(); }

    static std::shared_ptr<UpSampling> Create(create_t const &create) { return std::shared_ptr<UpSampling>(new UpSampling(create)); }
    static std::shared_ptr<UpSampling> Create(index_t filter_h_size, index_t filter_w_size, bool fill = true)
    {
        create_t c;
        c.filter_h_size = filter_h_size; c.filter_w_size = filter_w_size; c.fill = fill;
        return Create(c);
    }
    static std::shared_ptr<UpSampling> Create(void) { return Create(create_t()); }

    indices_t SetInputShape(indices_t shape) override
    {
        if (shape == m_input_shape) { return OutputShapeOf(shape); }
        BB_ASSERT(shape.size() == 3);
        m_input_shape = shape;
        return OutputShapeOf(shape);
    }
    indices_t GetInputShape(void) const override  { return m_input_shape; }
    indices_t GetOutputShape(void) const override { return OutputShapeOf(m_input_shape); }

    void Clear(void) override
    {
        Model::Clear();
        while (!m_shapes.empty()) { m_shapes.pop(); }
    }

    FrameBuffer Forward(FrameBuffer x_buf, bool = true) override
    {
        BB_ASSERT(x_buf.GetType() == DataType<FT>::type);
        RequireDevice(x_buf, "UpSampling::Forward");
        indices_t const input_shape = x_buf.GetShape();
        BB_ASSERT(input_shape.size() == 3);
        if (input_shape != m_input_shape) { SetInputShape(input_shape); }
        m_shapes.push(input_shape);
        FrameBuffer y_buf(x_buf.GetFrameSize(), OutputShapeOf(input_shape), DataType<FT>::type);
        BB_ASSERT(y_buf.GetFrameStride() == x_buf.GetFrameStride());
        auto x_ptr = x_buf.LockDeviceMemoryConst();
        auto y_ptr = y_buf.LockDeviceMemory(true);
        if (DataType<FT>::type == BB_TYPE_BIT) {
            CheckDevice(bbhip_bit_UpSampling_Forward((int const *)x_ptr.GetAddr(), (int *)y_ptr.GetAddr(), (int)input_shape[2], (int)input_shape[1],
                            (int)input_shape[0], (int)m_filter_w_size, (int)m_filter_h_size, m_fill ? 1 : 0, (int)x_buf.GetFrameSize(),
                            (int)(x_buf.GetFrameStride() / sizeof(int)), nullptr), "bbhip_bit_UpSampling_Forward");
        }
        else {
            CheckDevice(bbhip_fp32_UpSampling_Forward((float const *)x_ptr.GetAddr(), (float *)y_ptr.GetAddr(), (int)input_shape[2], (int)input_shape[1],
                            (int)input_shape[0], (int)m_filter_w_size, (int)m_filter_h_size, m_fill ? 1 : 0, (int)x_buf.GetFrameSize(),
                            (int)(x_buf.GetFrameStride() / sizeof(float)), nullptr), "bbhip_fp32_UpSampling_Forward");
        }
        return y_buf;
    }

    FrameBuffer Backward(FrameBuffer dy_buf) override
    {
        if (dy_buf.Empty()) { return FrameBuffer(); }
        BB_ASSERT(!m_shapes.empty());
        indices_t const input_shape = m_shapes.top();
        m_shapes.pop();
        BB_ASSERT(dy_buf.GetType() == BB_TYPE_FP32 && dy_buf.GetShape() == OutputShapeOf(input_shape));
        RequireDevice(dy_buf, "UpSampling::Backward");
        FrameBuffer dx_buf(dy_buf.GetFrameSize(), input_shape, BB_TYPE_FP32);
        auto dy_ptr = dy_buf.LockDeviceMemoryConst();
        auto dx_ptr = dx_buf.LockDeviceMemory(true);
        CheckDevice(bbhip_fp32_UpSampling_Backward((float const *)dy_ptr.GetAddr(), (float *)dx_ptr.GetAddr(), (int)input_shape[2], (int)input_shape[1],
                        (int)input_shape[0], (int)m_filter_w_size, (int)m_filter_h_size, m_fill ? 1 : 0, (int)dy_buf.GetFrameSize(),
                        (int)(dy_buf.GetFrameStride() / sizeof(float)), nullptr), "bbhip_fp32_UpSampling_Backward");
        return dx_buf;
    }
};

}  // namespace bb

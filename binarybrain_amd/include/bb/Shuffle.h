// Shuffle: a fixed permutation of a frame's nodes that deals the inputs of neighbouring groups out to different LUTs of the
// next layer — output node i * shuffle_unit + j is input node j * (nodes / shuffle_unit) + i; the backward pass undoes it
// (reference API: include/bb/Shuffle.h:18-309: Create(shuffle_unit, output_shape), SetInputShape, Forward, Backward).
// Frames of any type move as whole rows; an output shape of another size than the input's is replaced by the input shape.
// Serialized as  version 1 | Model part | host_only | input shape | output shape | shuffle_unit  (reference :270-301).
#pragma once

#include "bb/Model.h"

namespace bb {

class Shuffle : public Model {
    bool      m_host_only = false;
    indices_t m_input_shape;
    indices_t m_output_shape;
    index_t   m_shuffle_unit = 0;

public:
    struct create_t {
        index_t   shuffle_unit = 0;
        indices_t output_shape;
    };

protected:
    explicit Shuffle(create_t const &create) : m_output_shape(create.output_shape), m_shuffle_unit(create.shuffle_unit) {}

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
        SaveValue(os, (std::int64_t)m_shuffle_unit);
    }

    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = -1, unit = -1;
        LoadValue(is, ver);
        BB_ASSERT(ver == 1);
        Model::LoadObjectData(is);
        LoadValue(is, m_host_only);
        m_input_shape  = LoadIndices(is);
        m_output_shape = LoadIndices(is);
        LoadValue(is, unit);
        BB_ASSERT(is.good() && unit >= 0);
        BB_ASSERT(m_input_shape.empty() || (unit > 0 && CalcShapeSize(m_output_shape) == CalcShapeSize(m_input_shape)
                                            && CalcShapeSize(m_output_shape) % unit == 0));
        m_shuffle_unit = (index_t)unit;
    }

    void RequireDevice(FrameBuffer const &buf, char const *what) const
    {
        if (m_host_only || !buf.IsDeviceAvailable() || !Manager::IsDeviceAvailable()) {
            throw Exception(std::string(what) + ": host-only execution is not provided by this library (device path only)");
        }
    }

public:
    static std::string ModelName(void)  { return "Shuffle"; }
    static std::string ObjectName(void) { return ModelName(); }
    std::string GetModelName(void) const override  { return ModelName(); }
    std::string GetObjectName(void) const override { return ObjectName(); }

    static std::shared_ptr<Shuffle> Create(create_t const &create) { return std::shared_ptr<Shuffle>(new Shuffle(create)); }
    static std::shared_ptr<Shuffle> Create(index_t shuffle_unit, indices_t output_shape = indices_t())
    {
        create_t c;
        c.shuffle_unit = shuffle_unit; c.output_shape = output_shape;
        return Create(c);
    }
    static std::shared_ptr<Shuffle> Create(index_t shuffle_unit, index_t output_node_size) { return Create(shuffle_unit, indices_t({output_node_size})); }
    static std::shared_ptr<Shuffle> Create(void) { return Create(create_t()); }

    indices_t SetInputShape(indices_t shape) override
    {
        m_input_shape = shape;
        if (m_output_shape.empty() || CalcShapeSize(shape) != CalcShapeSize(m_output_shape)) { m_output_shape = m_input_shape; }
        BB_ASSERT(m_shuffle_unit > 0 && CalcShapeSize(m_output_shape) % m_shuffle_unit == 0);
        return m_output_shape;
    }
    indices_t GetInputShape(void) const override  { return m_input_shape; }
    indices_t GetOutputShape(void) const override { return m_output_shape; }

    FrameBuffer Forward(FrameBuffer x_buf, bool = true) override
    {
        RequireDevice(x_buf, "Shuffle::Forward");
        if (x_buf.GetShape() != m_input_shape) { SetInputShape(x_buf.GetShape()); }
        FrameBuffer y_buf(x_buf.GetFrameSize(), m_output_shape, x_buf.GetType());
        BB_ASSERT(y_buf.GetFrameStride() == x_buf.GetFrameStride());
        auto x_ptr = x_buf.LockDeviceMemoryConst();
        auto y_ptr = y_buf.LockDeviceMemory(true);
        CheckDevice(bbhip_Shuffle_Forward((int const *)x_ptr.GetAddr(), (int *)y_ptr.GetAddr(), (unsigned int)m_shuffle_unit,
                        (unsigned int)x_buf.GetNodeSize(), (unsigned int)x_buf.GetFrameSize(),
                        (unsigned int)(x_buf.GetFrameStride() / sizeof(int)), nullptr), "bbhip_Shuffle_Forward");
        return y_buf;
    }

    FrameBuffer Backward(FrameBuffer dy_buf) override
    {
        if (dy_buf.Empty()) { return FrameBuffer(); }
        BB_ASSERT(dy_buf.GetNodeSize() == CalcShapeSize(m_input_shape));
        RequireDevice(dy_buf, "Shuffle::Backward");
        FrameBuffer dx_buf(dy_buf.GetFrameSize(), m_input_shape, dy_buf.GetType());
        BB_ASSERT(dx_buf.GetFrameStride() == dy_buf.GetFrameStride());
        auto dy_ptr = dy_buf.LockDeviceMemoryConst();
        auto dx_ptr = dx_buf.LockDeviceMemory(true);
        CheckDevice(bbhip_Shuffle_Backward((int const *)dy_ptr.GetAddr(), (int *)dx_ptr.GetAddr(), (unsigned int)m_shuffle_unit,
                        (unsigned int)dy_buf.GetNodeSize(), (unsigned int)dy_buf.GetFrameSize(),
                        (unsigned int)(dy_buf.GetFrameStride() / sizeof(int)), nullptr), "bbhip_Shuffle_Backward");
        return dx_buf;
    }
};

}  // namespace bb

// RealToBinary: the entry of a binary network.  Every input value becomes frame_modulation_size frames (and
// depth_modulation_size nodes along the first axis of the shape) of a binary signal whose share of ones follows the value:
// step f of F compares the value, brought to [0, 1], with (f + 1/2) / F (reference API: include/bb/RealToBinary.h:33-556:
// Create(frame_modulation_size[, depth_modulation_size], value_generator, framewise, input_range_lo, input_range_hi),
// SetModulationSize, SetInputShape, Forward, Backward, command "binary").
// Thresholds drawn from a value generator exist only as a host loop in the reference (:346-388) and are not provided here:
// the argument must be empty, as it is in every use the reference's samples make of the layer.
// The backward pass returns a buffer of the input's shape whose contents are unspecified, as in the reference (:467-497:
// nothing reads the gradient of the network's input).
// Serialized as  version 1 | Model part | binary_mode | input shape | output shape | point size | input depth | output depth |
// frame modulation | depth modulation | framewise | range lo | range hi | has value generator (0)  (reference :501-548).
#pragma once

#include "bb/Model.h"

namespace bb {

template <typename BinType = float, typename RealType = float>
class RealToBinary : public Model {
    static_assert(std::is_same<RealType, float>::value, "inputs are fp32");
    static_assert(std::is_same<BinType, float>::value || std::is_same<BinType, Bit>::value, "outputs are fp32 or packed bits");

    bool      m_binary_mode = true;
    indices_t m_x_node_shape, m_y_node_shape;
    index_t   m_point_size = 0, m_x_depth_size = 0, m_y_depth_size = 0;
    index_t   m_frame_modulation_size = 1, m_depth_modulation_size = 1;
    bool      m_framewise = false;
    RealType  m_input_range_lo = (RealType)0.0, m_input_range_hi = (RealType)1.0;

public:
    // the record that BinaryModulation keeps of how its converter is set up (reference :62-103)
    struct create_t {
        index_t  frame_modulation_size = 1;
        index_t  depth_modulation_size = 1;
        std::shared_ptr<Object> value_generator;        // must stay empty
        bool     framewise = false;
        RealType input_range_lo = (RealType)0.0;
        RealType input_range_hi = (RealType)1.0;

        void ObjectDump(std::ostream &os) const
        {
            SaveValue(os, (std::int64_t)frame_modulation_size);
            SaveValue(os, (std::int64_t)depth_modulation_size);
            SaveValue(os, framewise);
            SaveValue(os, input_range_lo);
            SaveValue(os, input_range_hi);
            SaveValue(os, false);
        }
        void ObjectLoad(std::istream &is)
        {
            std::int64_t fm = -1, dm = -1;
            bool has_generator = true;
            LoadValue(is, fm);
            LoadValue(is, dm);
            LoadValue(is, framewise);
            LoadValue(is, input_range_lo);
            LoadValue(is, input_range_hi);
            LoadValue(is, has_generator);
            BB_ASSERT(is.good() && fm > 0 && dm > 0);
            if (has_generator) { throw Exception("RealToBinary: a serialized value generator is not supported (thresholds are the fixed steps)"); }
            frame_modulation_size = (index_t)fm; depth_modulation_size = (index_t)dm;
        }
    };

protected:
    explicit RealToBinary(create_t const &create)
        : m_frame_modulation_size(create.frame_modulation_size), m_depth_modulation_size(create.depth_modulation_size),
          m_framewise(create.framewise), m_input_range_lo(create.input_range_lo), m_input_range_hi(create.input_range_hi)
    {
        if (create.value_generator) { throw Exception("RealToBinary: value generators are not supported (thresholds are the fixed steps)"); }
        BB_ASSERT(m_frame_modulation_size > 0 && m_depth_modulation_size > 0);
    }

    void CommandProc(std::vector<std::string> args) override
    {
        Model::CommandProc(args);
        if (args.size() == 2 && args[0] == "binary") { m_binary_mode = EvalBool(args[1]); }
    }

    void DumpObjectData(std::ostream &os) const override
    {
        SaveValue(os, (std::int64_t)1);
        Model::DumpObjectData(os);
        SaveValue(os, m_binary_mode);
        SaveIndices(os, m_x_node_shape);
        SaveIndices(os, m_y_node_shape);
        SaveValue(os, (std::int64_t)m_point_size);
        SaveValue(os, (std::int64_t)m_x_depth_size);
        SaveValue(os, (std::int64_t)m_y_depth_size);
        SaveValue(os, (std::int64_t)m_frame_modulation_size);
        SaveValue(os, (std::int64_t)m_depth_modulation_size);
        SaveValue(os, m_framewise);
        SaveValue(os, m_input_range_lo);
        SaveValue(os, m_input_range_hi);
        SaveValue(os, false);
    }

    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = -1, v[5] = {-1, -1, -1, -1, -1};
        bool has_generator = true;
        LoadValue(is, ver);
        BB_ASSERT(ver == 1);
        Model::LoadObjectData(is);
        LoadValue(is, m_binary_mode);
        m_x_node_shape = LoadIndices(is);
        m_y_node_shape = LoadIndices(is);
        for (auto &e : v) { LoadValue(is, e); }
        LoadValue(is, m_framewise);
        LoadValue(is, m_input_range_lo);
        LoadValue(is, m_input_range_hi);
        LoadValue(is, has_generator);
        BB_ASSERT(is.good() && v[3] > 0 && v[4] > 0);
        if (has_generator) { throw Exception("RealToBinary: a serialized value generator is not supported (thresholds are the fixed steps)"); }
        m_point_size = v[0]; m_x_depth_size = v[1]; m_y_depth_size = v[2]; m_frame_modulation_size = v[3]; m_depth_modulation_size = v[4];
        if (!m_x_node_shape.empty()) {          // the sizes must be the ones SetInputShape derives from the shape
            BB_ASSERT(m_x_depth_size == m_x_node_shape[0] && m_x_depth_size > 0 && m_point_size * m_x_depth_size == CalcShapeSize(m_x_node_shape));
            BB_ASSERT(m_y_depth_size == m_x_depth_size * m_depth_modulation_size && m_point_size * m_y_depth_size == CalcShapeSize(m_y_node_shape));
        }
    }

public:
    static std::string ModelName(void)  { return "RealToBinary"; }
    static std::string ObjectName(void) { return ModelName() + "_" + DataType<BinType>::Name() + "_" + DataType<RealType>::Name(); }
    std::string GetModelName(void) const override  { return ModelName(); }
    std::string GetObjectName(void) const override { return ObjectName(); }

    static std::shared_ptr<RealToBinary> Create(create_t const &create) { return std::shared_ptr<RealToBinary>(new RealToBinary(create)); }
    static std::shared_ptr<RealToBinary> Create(index_t frame_modulation_size = 1, std::shared_ptr<Object> value_generator = nullptr,
                                                bool framewise = false, RealType input_range_lo = (RealType)0.0,
                                                RealType input_range_hi = (RealType)1.0)
    {
        create_t c;
        c.frame_modulation_size = frame_modulation_size; c.value_generator = value_generator; c.framewise = framewise;
        c.input_range_lo = input_range_lo; c.input_range_hi = input_range_hi;
        return Create(c);
    }
    static std::shared_ptr<RealToBinary> Create(index_t frame_modulation_size, index_t depth_modulation_size,
                                                std::shared_ptr<Object> value_generator = nullptr, bool framewise = false,
                                                RealType input_range_lo = (RealType)0.0, RealType input_range_hi = (RealType)1.0)
    {
        create_t c;
        c.frame_modulation_size = frame_modulation_size; c.depth_modulation_size = depth_modulation_size; c.value_generator = value_generator;
        c.framewise = framewise; c.input_range_lo = input_range_lo; c.input_range_hi = input_range_hi;
        return Create(c);
    }

    void SetModulationSize(index_t modulation_size) { BB_ASSERT(modulation_size > 0); m_frame_modulation_size = modulation_size; }
    void SetValueGenerator(std::shared_ptr<Object> value_generator)
    {
        if (value_generator) { throw Exception("RealToBinary: value generators are not supported (thresholds are the fixed steps)"); }
    }
    index_t GetModulationSize(void) const { return m_frame_modulation_size; }

    indices_t SetInputShape(indices_t shape) override
    {
        if (shape == m_x_node_shape) { return m_y_node_shape; }
        BB_ASSERT(shape.size() > 0 && shape[0] > 0);
        m_x_node_shape = shape;
        m_x_depth_size = shape[0];
        m_point_size   = CalcShapeSize(shape) / m_x_depth_size;
        m_y_depth_size = m_x_depth_size * m_depth_modulation_size;
        m_y_node_shape = shape;
        m_y_node_shape[0] = m_y_depth_size;
        return m_y_node_shape;
    }
    indices_t GetInputShape(void) const override  { return m_x_node_shape; }
    indices_t GetOutputShape(void) const override { return m_y_node_shape; }

    FrameBuffer Forward(FrameBuffer x_buf, bool = true) override
    {
        if (!m_binary_mode && m_depth_modulation_size == 1) { return x_buf; }       // reference :268-270
        BB_ASSERT(x_buf.GetType() == DataType<RealType>::type);
        if (!x_buf.IsDeviceAvailable() || !Manager::IsDeviceAvailable()) {
            throw Exception("RealToBinary::Forward: host-only execution is not provided by this library (device path only)");
        }
        if (x_buf.GetShape() != m_x_node_shape) { SetInputShape(x_buf.GetShape()); }
        FrameBuffer y_buf(x_buf.GetFrameSize() * m_frame_modulation_size, m_y_node_shape, DataType<BinType>::type);
        auto x_ptr = x_buf.LockDeviceMemoryConst();
        auto y_ptr = y_buf.LockDeviceMemory(true);
        if (DataType<BinType>::type == BB_TYPE_BIT) {
            CheckDevice(bbhip_fp32_bit_RealToBinary_Forward((float const *)x_ptr.GetAddr(), (int *)y_ptr.GetAddr(), (unsigned)m_depth_modulation_size,
                            (unsigned)m_frame_modulation_size, (float)m_input_range_lo, (float)m_input_range_hi, (unsigned)m_point_size,
                            (unsigned)m_x_depth_size, (unsigned)x_buf.GetFrameSize(), (unsigned)(x_buf.GetFrameStride() / sizeof(float)),
                            (unsigned)(y_buf.GetFrameStride() / sizeof(int)), m_binary_mode ? 1 : 0, nullptr), "bbhip_fp32_bit_RealToBinary_Forward");
        }
        else {
            CheckDevice(bbhip_fp32_RealToBinary_Forward((float const *)x_ptr.GetAddr(), (float *)y_ptr.GetAddr(), (unsigned)m_depth_modulation_size,
                            (unsigned)m_frame_modulation_size, (float)m_input_range_lo, (float)m_input_range_hi, (unsigned)m_point_size,
                            (unsigned)m_x_depth_size, (unsigned)x_buf.GetFrameSize(), (unsigned)(x_buf.GetFrameStride() / sizeof(float)),
                            (unsigned)(y_buf.GetFrameStride() / sizeof(float)), m_binary_mode ? 1 : 0, nullptr), "bbhip_fp32_RealToBinary_Forward");
        }
        return y_buf;
    }

    FrameBuffer Backward(FrameBuffer dy_buf) override
    {
        if (dy_buf.Empty()) { return FrameBuffer(); }
        if (m_depth_modulation_size == 1 && (!m_binary_mode || m_frame_modulation_size == 1)) { return dy_buf; }
        BB_ASSERT(dy_buf.GetType() == DataType<RealType>::type);
        return FrameBuffer(dy_buf.GetFrameSize() / m_frame_modulation_size, m_x_node_shape, DataType<RealType>::type);
    }
};

}  // namespace bb

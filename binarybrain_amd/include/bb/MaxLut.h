// MaxLut: every output node takes the largest of n wired inputs; with binarize_output it writes +1 / -1 on maximum > 0, on
// packed bits it is the OR of the n inputs.  The gradient of a node goes to its first largest input.
// Reference API: include/bb/MaxLut.h:22-502 (Create(n, output_shape, connection, binarize, binarize_input, seed); commands
// binary / binarize_input / binarize_output / host_only; connection get/set; GetLutTable = majority of the index bits, as
// the reference has it).  Frame work runs in the HIP library only.
// Serialized as  version 1 | Model part | int32 n | host_only | connection policy | input shape | output shape |
// binarize_input | binarize_output | the wiring as a Tensor_int32 object  (reference :428-465).
#pragma once

#include <random>

#include "bb/ConnectionPolicy.h"
#include "bb/Model.h"

namespace bb {

template <typename BinType = float, typename RealType = float>
class MaxLut : public Model {
    static_assert(std::is_same<RealType, float>::value, "gradients are fp32");
    static_assert(std::is_same<BinType, float>::value || std::is_same<BinType, Bit>::value, "inputs are fp32 or packed bits");

protected:
    bool        m_host_only = false;
    bool        m_binarize_input = false;
    bool        m_binarize_output = true;
    int         m_n = 6;
    std::string m_connection;
    indices_t   m_input_shape, m_output_shape;
    Tensor_<std::int32_t> m_input_index;    // [output nodes][n]
    std::mt19937_64 m_mt;

    void CommandProc(std::vector<std::string> args) override
    {
        Model::CommandProc(args);
        if (args.size() == 2 && args[0] == "host_only")       { m_host_only = EvalBool(args[1]); }
        if (args.size() == 2 && args[0] == "binary")          { m_binarize_input = m_binarize_output = EvalBool(args[1]); }
        if (args.size() == 2 && args[0] == "binarize_input")  { m_binarize_input = EvalBool(args[1]); }
        if (args.size() == 2 && args[0] == "binarize_output") { m_binarize_output = EvalBool(args[1]); }
    }

    void DumpObjectData(std::ostream &os) const override
    {
        SaveValue(os, (std::int64_t)1);
        Model::DumpObjectData(os);
        SaveValue(os, (std::int32_t)m_n);
        SaveValue(os, m_host_only);
        SaveValue(os, m_connection);
        SaveIndices(os, m_input_shape);
        SaveIndices(os, m_output_shape);
        SaveValue(os, m_binarize_input);
        SaveValue(os, m_binarize_output);
        m_input_index.DumpObject(os);
    }

    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = -1;
        std::int32_t n = 0;
        LoadValue(is, ver);
        BB_ASSERT(ver == 1);
        Model::LoadObjectData(is);
        LoadValue(is, n);
        LoadValue(is, m_host_only);
        LoadValue(is, m_connection);
        m_input_shape = LoadIndices(is);
        m_output_shape = LoadIndices(is);
        LoadValue(is, m_binarize_input);
        LoadValue(is, m_binarize_output);
        m_input_index.LoadObject(is);
        BB_ASSERT(is.good() && n > 0);
        m_n = (int)n;
        BB_ASSERT(m_input_index.GetShape() == indices_t({CalcShapeSize(m_output_shape), (index_t)m_n}));
        // a wiring entry outside the input nodes would be read out of bounds on the device
        index_t const I = CalcShapeSize(m_input_shape);
        auto idx = m_input_index.LockConst();
        for (index_t k = 0; k < m_input_index.GetSize(); ++k) { BB_ASSERT(I == 0 || (idx[k] >= 0 && idx[k] < I)); }
    }

public:
    struct create_t {
        int           n = 6;
        indices_t     output_shape;
        std::string   connection = "";
        bool          binarize_input = false;
        bool          binarize_output = true;
        std::uint64_t seed = 1;
    };

protected:
    explicit MaxLut(create_t const &create)
    {
        BB_ASSERT(!create.output_shape.empty() && create.n > 0);
        m_mt.seed(create.seed);
        m_n = create.n;
        m_output_shape = create.output_shape;
        m_connection = create.connection;
        m_binarize_input = create.binarize_input;
        m_binarize_output = create.binarize_output;
        m_input_index.Resize(CalcShapeSize(m_output_shape), (index_t)m_n);
    }

public:
    static std::string ModelName(void)  { return "MaxLut"; }
    static std::string ObjectName(void) { return ModelName() + "_" + DataType<BinType>::Name() + "_" + DataType<RealType>::Name(); }
    std::string GetModelName(void) const override  { return ModelName(); }
    std::string GetObjectName(void) const override { return ObjectName(); }

    static std::shared_ptr<MaxLut> Create(create_t const &create) { return std::shared_ptr<MaxLut>(new MaxLut(create)); }
    static std::shared_ptr<MaxLut> Create(int n, indices_t const &output_shape, std::string connection = "", bool binarize = true,
                                          bool binarize_input = false, std::uint64_t seed = 1)
    {
        create_t c;
        c.n = n; c.output_shape = output_shape; c.connection = connection; c.binarize_input = binarize_input; c.binarize_output = binarize; c.seed = seed;
        return Create(c);
    }
    static std::shared_ptr<MaxLut> Create(int n, index_t output_node_size, std::string connection = "", bool binarize = true,
                                          bool binarize_input = false, std::uint64_t seed = 1)
    {
        return Create(n, indices_t({output_node_size}), connection, binarize, binarize_input, seed);
    }
    static std::shared_ptr<MaxLut> Create(void)
    {
        create_t c;
        c.output_shape = indices_t({1});
        return Create(c);
    }

    auto lock_InputIndex(void)             { return m_input_index.Lock(); }
    auto lock_InputIndex_const(void) const { return m_input_index.LockConst(); }

    index_t GetNodeConnectionSize(index_t) const { return m_n; }
    void SetNodeConnectionIndex(index_t node, index_t input_index, index_t input_node)
    {
        BB_ASSERT(node >= 0 && node < this->GetOutputNodeSize() && input_index >= 0 && input_index < m_n);
        BB_ASSERT(input_node >= 0 && input_node < this->GetInputNodeSize());
        m_input_index.Lock()(node, input_index) = (std::int32_t)input_node;
    }
    index_t GetNodeConnectionIndex(index_t node, index_t input_index) const
    {
        BB_ASSERT(node >= 0 && node < this->GetOutputNodeSize() && input_index >= 0 && input_index < m_n);
        return (index_t)m_input_index.LockConst()(node, input_index);
    }

    // the layer as a look-up table, as the reference tabulates it (:190-206: the majority of the index bits)
    int  GetLutTableSize(index_t) const { return 1 << m_n; }
    void SetLutTable(index_t, int, bool) {}
    bool GetLutTable(index_t, int bitpos) const
    {
        int count = 0;
        for (int i = 0; i < m_n; ++i) { count += (bitpos & 1) ? +1 : -1; bitpos >>= 1; }
        return count > 0;
    }

    // seeded wiring by the reference's policies (bb/ConnectionPolicy.h; reference: SparseModel.h:97-233); a repeated shape keeps it
    indices_t SetInputShape(indices_t shape) override
    {
        if (shape == m_input_shape) { return m_output_shape; }
        m_input_shape = shape;
        index_t const I = CalcShapeSize(shape);
        BB_ASSERT(I > 0);
        auto idx = m_input_index.Lock(true);
        connection_policy::Initialize(m_mt(), m_connection, m_input_shape, m_output_shape, m_n, connection_policy::Layout::kChannelLast,
                                      [&](index_t node, int i, index_t input) {
                                          BB_ASSERT(input >= 0 && input < I);
                                          idx(node, (index_t)i) = (std::int32_t)input;
                                      });
        return m_output_shape;
    }
    void SetOutputShape(indices_t const &shape)
    {
        BB_ASSERT(CalcShapeSize(shape) == this->GetOutputNodeSize());
        m_output_shape = shape;
    }
    indices_t GetInputShape(void) const override  { return m_input_shape; }
    indices_t GetOutputShape(void) const override { return m_output_shape; }

    FrameBuffer Forward(FrameBuffer x_buf, bool train = true) override
    {
        BB_ASSERT(x_buf.GetType() == DataType<BinType>::type);
        if (m_host_only || !Manager::IsDeviceAvailable()) {
            throw Exception("MaxLut::Forward: host-only execution is not provided by this library (device path only)");
        }
        if (x_buf.GetShape() != m_input_shape) { SetInputShape(x_buf.GetShape()); }
        if (train) { PushFrameBuffer(x_buf); }
        FrameBuffer y_buf(x_buf.GetFrameSize(), m_output_shape, DataType<BinType>::type);
        BB_ASSERT(x_buf.GetFrameStride() == y_buf.GetFrameStride());
        auto x_ptr   = x_buf.LockDeviceMemoryConst();
        auto y_ptr   = y_buf.LockDeviceMemory(true);
        auto idx_ptr = m_input_index.LockDeviceMemoryConst();
        if (DataType<BinType>::type == BB_TYPE_BIT) {
            CheckDevice(bbhip_bit_MaxLut_Forward((int const *)x_ptr.GetAddr(), (int *)y_ptr.GetAddr(), (int const *)idx_ptr.GetAddr(), m_n,
                            (int)y_buf.GetNodeSize(), (int)y_buf.GetFrameSize(), (int)(y_buf.GetFrameStride() / sizeof(int)), nullptr),
                        "bbhip_bit_MaxLut_Forward");
        }
        else {
            CheckDevice(bbhip_fp32_MaxLut_Forward((float const *)x_ptr.GetAddr(), (float *)y_ptr.GetAddr(), (int const *)idx_ptr.GetAddr(), m_n,
                            (int)y_buf.GetNodeSize(), (int)y_buf.GetFrameSize(), (int)(y_buf.GetFrameStride() / sizeof(float)),
                            m_binarize_input ? 1 : 0, m_binarize_output ? 1 : 0, nullptr), "bbhip_fp32_MaxLut_Forward");
        }
        return y_buf;
    }

    FrameBuffer Backward(FrameBuffer dy_buf) override
    {
        if (dy_buf.Empty()) { return dy_buf; }
        BB_ASSERT(dy_buf.GetType() == BB_TYPE_FP32);
        if (m_host_only || !Manager::IsDeviceAvailable()) {
            throw Exception("MaxLut::Backward: host-only execution is not provided by this library (device path only)");
        }
        FrameBuffer x_buf = PopFrameBuffer();
        BB_ASSERT(x_buf.GetType() == DataType<BinType>::type && x_buf.GetFrameSize() == dy_buf.GetFrameSize());
        FrameBuffer dx_buf(dy_buf.GetFrameSize(), m_input_shape, BB_TYPE_FP32);
        BB_ASSERT(dx_buf.GetFrameStride() == dy_buf.GetFrameStride());
        auto x_ptr   = x_buf.LockDeviceMemoryConst();
        auto dy_ptr  = dy_buf.LockDeviceMemoryConst();
        auto dx_ptr  = dx_buf.LockDeviceMemory(true);
        auto idx_ptr = m_input_index.LockDeviceMemoryConst();
        if (DataType<BinType>::type == BB_TYPE_BIT) {
            CheckDevice(bbhip_bit_fp32_MaxLut_Backward((int const *)x_ptr.GetAddr(), (float const *)dy_ptr.GetAddr(), (float *)dx_ptr.GetAddr(),
                            (int const *)idx_ptr.GetAddr(), m_n, (int)dx_buf.GetNodeSize(), (int)dy_buf.GetNodeSize(), (int)dy_buf.GetFrameSize(),
                            (int)(x_buf.GetFrameStride() / sizeof(int)), (int)(dy_buf.GetFrameStride() / sizeof(float)), nullptr),
                        "bbhip_bit_fp32_MaxLut_Backward");
        }
        else {
            BB_ASSERT(x_buf.GetFrameStride() == dy_buf.GetFrameStride());
            CheckDevice(bbhip_fp32_MaxLut_Backward((float const *)x_ptr.GetAddr(), (float const *)dy_ptr.GetAddr(), (float *)dx_ptr.GetAddr(),
                            (int const *)idx_ptr.GetAddr(), m_n, (int)dx_buf.GetNodeSize(), (int)dy_buf.GetNodeSize(), (int)dy_buf.GetFrameSize(),
                            (int)(dy_buf.GetFrameStride() / sizeof(float)), m_binarize_input ? 1 : 0, nullptr), "bbhip_fp32_MaxLut_Backward");
        }
        return dx_buf;
    }
};

}  // namespace bb

// BinaryLutN<N, Bit>, N = 2 .. 6: inference-only layer of N-input binary look-up tables on bit-packed frames, with the reference's
// model API (include/bb/BinaryLutN.h:20-523, table helpers in include/bb/BinaryLutModel.h:45-91): Create, SetInputShape,
// connection get/set, GetLutTable / SetLutTable, ImportLayer, Forward.  Input k of a node is bit k of the table index;
// a node's table is (2^N + 31) / 32 words of its int32 row, entry i = bit i & 31 of word i >> 5 (one word up to N = 5, two for N = 6).
// Frame work runs in the HIP library only (the reference has a device kernel for N = 6 and runs the other widths on the host).
#pragma once

#include <random>

#include "bb/ConnectionPolicy.h"
#include "bb/Model.h"

namespace bb {

template <int N = 6, typename FT = Bit, typename BT = float>
class BinaryLutN : public Model {
    static_assert(N >= 2 && N <= 6 && std::is_same<FT, Bit>::value, "the device path covers 2- to 6-input tables on packed bits");
    static constexpr int kTableSize = 1 << N;
    static constexpr int kTableUnit = (kTableSize + 31) / 32;

protected:
    bool        m_host_only = false;
    bool        m_host_simd = true;             // carried through serialization only: there is no host path here
    std::string m_connection;
    indices_t   m_input_shape, m_output_shape;
    Tensor_<std::int32_t> m_table;          // [output nodes][kTableUnit]
    Tensor_<std::int32_t> m_input_index;    // [output nodes][N]
    std::mt19937_64 m_mt;

    void CommandProc(std::vector<std::string> args) override
    {
        Model::CommandProc(args);
        if (args.size() == 2 && args[0] == "host_only") { m_host_only = EvalBool(args[1]); }
        if (args.size() == 2 && args[0] == "host_simd") { m_host_simd = EvalBool(args[1]); }     // kept and serialized only
    }

public:
    struct create_t {
        indices_t     output_shape;
        std::string   connection = "";
        std::uint64_t seed = 1;
    };

protected:
    explicit BinaryLutN(create_t const &create)
    {
        BB_ASSERT(!create.output_shape.empty());
        m_mt.seed(create.seed);
        m_output_shape = create.output_shape;
        m_connection = create.connection;
        m_input_index.Resize(CalcShapeSize(m_output_shape), (index_t)N);
        m_table.Resize(CalcShapeSize(m_output_shape), (index_t)kTableUnit);
        m_table = 0;
    }

    // the reference's object layout (include/bb/BinaryLutN.h:481-519): version, Model part, flags, connection policy, shapes,
    // truth table object, input index object
    void DumpObjectData(std::ostream &os) const override
    {
        SaveValue(os, (std::int64_t)1);
        Model::DumpObjectData(os);
        SaveValue(os, m_host_only);
        SaveValue(os, m_host_simd);
        SaveValue(os, m_connection);
        SaveValue(os, m_input_shape);
        SaveValue(os, m_output_shape);
        m_table.DumpObject(os);
        m_input_index.DumpObject(os);
    }
    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = 0;
        LoadValue(is, ver); BB_ASSERT(ver == 1);
        Model::LoadObjectData(is);
        LoadValue(is, m_host_only);
        LoadValue(is, m_host_simd);
        LoadValue(is, m_connection);
        LoadValue(is, m_input_shape);
        LoadValue(is, m_output_shape);
        m_table.LoadObject(is);
        m_input_index.LoadObject(is);
        index_t const O = CalcShapeSize(m_output_shape), I = CalcShapeSize(m_input_shape);
        BB_ASSERT(m_table.GetShape() == indices_t({O, (index_t)kTableUnit}) && m_input_index.GetShape() == indices_t({O, (index_t)N}));
        // wiring read from a file is checked before any kernel follows it
        auto idx = m_input_index.LockConst();
        for (index_t i = 0; i < O * N; ++i) { BB_ASSERT(idx[i] >= 0 && idx[i] < I); }
    }

public:
    static std::string ModelName(void) { return "BinaryLut" + std::to_string(N); }
    static std::string ObjectName(void) { return ModelName() + "_" + DataType<FT>::Name() + "_" + DataType<BT>::Name(); }
    std::string GetModelName(void) const override { return ModelName(); }
    std::string GetObjectName(void) const override { return ObjectName(); }

    static std::shared_ptr<BinaryLutN> Create(create_t const &create) { return std::shared_ptr<BinaryLutN>(new BinaryLutN(create)); }
    static std::shared_ptr<BinaryLutN> Create(indices_t const &output_shape, std::uint64_t seed = 1)
    {
        create_t c; c.output_shape = output_shape; c.seed = seed;
        return Create(c);
    }
    static std::shared_ptr<BinaryLutN> Create(index_t output_node_size, std::uint64_t seed = 1) { return Create(indices_t({output_node_size}), seed); }

    index_t GetNodeConnectionSize(index_t) const { return N; }
    void SetNodeConnectionIndex(index_t node, index_t input_index, index_t input_node)
    {
        BB_ASSERT(node >= 0 && node < this->GetOutputNodeSize() && input_index >= 0 && input_index < N);
        BB_ASSERT(input_node >= 0 && input_node < this->GetInputNodeSize());
        m_input_index.Lock()(node, input_index) = (std::int32_t)input_node;
    }
    index_t GetNodeConnectionIndex(index_t node, index_t input_index) const
    {
        BB_ASSERT(node >= 0 && node < this->GetOutputNodeSize() && input_index >= 0 && input_index < N);
        return (index_t)m_input_index.LockConst()(node, input_index);
    }

    int  GetLutTableSize(index_t) const { return kTableSize; }
    void SetLutTable(index_t node, int bitpos, bool value)
    {
        BB_ASSERT(node >= 0 && node < this->GetOutputNodeSize() && bitpos >= 0 && bitpos < kTableSize);
        auto p = m_table.Lock();
        std::uint32_t w = (std::uint32_t)p(node, bitpos / 32);
        std::uint32_t const m = 1u << (bitpos % 32);
        p(node, bitpos / 32) = (std::int32_t)(value ? (w | m) : (w & ~m));
    }
    bool GetLutTable(index_t node, int bitpos) const
    {
        BB_ASSERT(node >= 0 && node < this->GetOutputNodeSize() && bitpos >= 0 && bitpos < kTableSize);
        return (((std::uint32_t)m_table.LockConst()(node, bitpos / 32) >> (bitpos % 32)) & 1u) != 0;
    }

    indices_t SetInputShape(indices_t shape) override
    {
        if (shape == m_input_shape) { return m_output_shape; }
        m_input_shape = shape;
        index_t const I = CalcShapeSize(shape), O = this->GetOutputNodeSize();
        BB_ASSERT(I >= N);
        // seeded wiring by policy, then random tables: one draw of the layer's generator seeds each, and the table bits come
        // from a generator of their own, entry by entry (reference: BinaryLutN.h:201-218, SparseModel.h:97-233,
        // BinaryLutModel.h:45-59)
        {
            auto idx = m_input_index.Lock(true);
            connection_policy::Initialize(m_mt(), m_connection, m_input_shape, m_output_shape, N, connection_policy::Layout::kChannelLast,
                                          [&](index_t node, int i, index_t input) {
                                              BB_ASSERT(input >= 0 && input < I);
                                              idx(node, (index_t)i) = (std::int32_t)input;
                                          });
        }
        {
            std::mt19937_64 mt(m_mt());
            std::uniform_int_distribution<int> coin(0, 1);
            auto tbl = m_table.Lock(true);
            for (index_t o = 0; o < O; ++o) {
                for (int u = 0; u < kTableUnit; ++u) { tbl(o, u) = 0; }
                for (int i = 0; i < kTableSize; ++i) {
                    if (coin(mt) != 0) { tbl(o, i / 32) = (std::int32_t)((std::uint32_t)tbl(o, i / 32) | (1u << (i % 32))); }
                }
            }
        }
        return m_output_shape;
    }
    indices_t GetInputShape(void) const override  { return m_input_shape; }
    indices_t GetOutputShape(void) const override { return m_output_shape; }

    // Tabulate a trained layer: same wiring, table bit i = (ForwardNode(node, bits of i as 0.0 / 1.0) >= 0.5)
    // (reference: BinaryLutModel::ImportLayer, include/bb/BinaryLutModel.h:63-91)
    template <class SrcModel>
    void ImportLayer(std::shared_ptr<SrcModel> src)
    {
        BB_ASSERT(src->GetInputShape() == m_input_shape || m_input_shape.empty());
        BB_ASSERT(src->GetOutputNodeSize() == this->GetOutputNodeSize());
        if (m_input_shape.empty()) { SetInputShape(src->GetInputShape()); }
        for (index_t node = 0; node < this->GetOutputNodeSize(); ++node) {
            for (int i = 0; i < N; ++i) { SetNodeConnectionIndex(node, i, src->GetNodeConnectionIndex(node, i)); }
            for (int i = 0; i < kTableSize; ++i) {
                std::vector<double> vec((std::size_t)N);
                for (int bit = 0; bit < N; ++bit) { vec[(std::size_t)bit] = ((i >> bit) & 1) ? 1.0 : 0.0; }
                SetLutTable(node, i, src->ForwardNode(node, vec)[0] >= 0.5);
            }
        }
    }

    FrameBuffer Forward(FrameBuffer x_buf, bool = true) override
    {
        BB_ASSERT(x_buf.GetType() == BB_TYPE_BIT);
        if (m_host_only || !Manager::IsDeviceAvailable()) {
            throw Exception("BinaryLutN::Forward: host-only execution is not provided by this library (device path only)");
        }
        if (x_buf.GetShape() != m_input_shape) { SetInputShape(x_buf.GetShape()); }
        FrameBuffer y_buf(x_buf.GetFrameSize(), m_output_shape, BB_TYPE_BIT);
        BB_ASSERT(x_buf.GetFrameStride() == y_buf.GetFrameStride());
        auto x_ptr   = x_buf.LockDeviceMemoryConst();
        auto y_ptr   = y_buf.LockDeviceMemory(true);
        auto idx_ptr = m_input_index.LockDeviceMemoryConst();
        auto tbl_ptr = m_table.LockDeviceMemoryConst();
        CheckDevice(bbhip_bit_BinaryLutN_Forward(N, (int const *)x_ptr.GetAddr(), (int *)y_ptr.GetAddr(), (int const *)idx_ptr.GetAddr(),
                        (int const *)tbl_ptr.GetAddr(), (int)y_buf.GetNodeSize(), (int)y_buf.GetFrameSize(),
                        (int)(y_buf.GetFrameStride() / sizeof(int)), nullptr), "bbhip_bit_BinaryLutN_Forward");
        return y_buf;
    }

    // there is no backward pass; the shape-only buffer of the reference is returned (BinaryLutN.h:467-475)
    FrameBuffer Backward(FrameBuffer dy_buf) override
    {
        if (dy_buf.Empty()) { return dy_buf; }
        return FrameBuffer(dy_buf.GetFrameSize(), m_input_shape, DataType<BT>::type);
    }
};

}  // namespace bb

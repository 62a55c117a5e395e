// What AverageLut and MaxLut share: n wired inputs per output node (no trained table), the commands, the view as a look-up
// table and the serialized form.  Reference: both classes derive from BinaryLutModel and repeat this code
// (include/bb/AverageLut.h:36-257, 412-458; include/bb/MaxLut.h:36-250, 428-465).
// Serialized as  version 1 | Model part | int32 n | host_only | connection policy | input shape | output shape |
// binarize_input | binarize_output | the wiring as a Tensor_int32 object.
#pragma once

#include <random>

#include "bb/ConnectionPolicy.h"
#include "bb/Model.h"

namespace bb {

class WiredSelectModel : public Model {
protected:
    bool        m_host_only = false;
    bool        m_binarize_input = false;
    bool        m_binarize_output = true;
    int         m_n = 6;
    std::string m_connection;
    indices_t   m_input_shape, m_output_shape;
    Tensor_<std::int32_t> m_input_index;    // [output nodes][n]
    std::mt19937_64 m_mt;

    WiredSelectModel(int n, indices_t const &output_shape, std::string const &connection, bool binarize_input, bool binarize_output,
                     std::uint64_t seed)
    {
        BB_ASSERT(!output_shape.empty() && n > 0);
        m_mt.seed(seed);
        m_n = n;
        m_output_shape = output_shape;
        m_connection = connection;
        m_binarize_input = binarize_input;
        m_binarize_output = binarize_output;
        m_input_index.Resize(CalcShapeSize(m_output_shape), (index_t)m_n);
    }

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

    // the layer as a look-up table, as the reference tabulates both layers: entry `bitpos` is the majority of its n index bits
    // (AverageLut.h:190-206, MaxLut.h:190-206)
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
};

}  // namespace bb

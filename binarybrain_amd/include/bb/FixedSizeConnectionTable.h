// Wiring of a sparse layer with exactly N inputs per output node: the input table int32 [output_nodes][N] and, built
// lazily from it, the reverse table int32 [input_nodes][1 + max fan-out] whose row r is
// [count, node*N + input ... in ascending (node, input) order, zero tail]
// (reference: include/bb/FixedSizeConnectionTable.h:24-216, reverse table :180-215; policies in
// include/bb/ConnectionTable.h:150-284).  Index bookkeeping stays on the host; the device sees the two tables.
#pragma once

#include <algorithm>

#include "bb/ConnectionPolicy.h"
#include "bb/Core.h"
#include "bb/Tensor.h"

namespace bb {

template <int N, typename IndexType = std::int32_t>
class FixedSizeConnectionTable : public Object {
    indices_t           m_input_shape, m_output_shape;
    index_t             m_input_node_size = 0, m_output_node_size = 0;
    Tensor_<IndexType>  m_input_table;
    Tensor_<IndexType>  m_reverse_table;
    bool                m_reverse_table_dirty = true;

public:
    void SetShape(indices_t input_shape, indices_t output_shape)
    {
        m_input_shape = input_shape;
        m_output_shape = output_shape;
        m_input_node_size = CalcShapeSize(input_shape);
        m_output_node_size = CalcShapeSize(output_shape);
        m_input_table.Resize(m_output_node_size, (index_t)N);
        m_reverse_table_dirty = true;
    }
    index_t GetInputNodeSize(void) const  { return m_input_node_size; }
    index_t GetOutputNodeSize(void) const { return m_output_node_size; }
    index_t GetInputConnectionSize(index_t) const { return N; }

    index_t GetInputConnection(index_t output_node, index_t connection_index) const
    {
        BB_ASSERT(output_node >= 0 && output_node < m_output_node_size && connection_index >= 0 && connection_index < N);
        return (index_t)m_input_table.LockConst()(output_node, connection_index);
    }
    void SetInputConnection(index_t output_node, index_t connection_index, index_t input_node)
    {
        BB_ASSERT(output_node >= 0 && output_node < m_output_node_size && connection_index >= 0 && connection_index < N);
        BB_ASSERT(input_node >= 0 && input_node < m_input_node_size);
        m_input_table.Lock()(output_node, connection_index) = (IndexType)input_node;
        m_reverse_table_dirty = true;
    }

    // Seeded wiring by policy ("" or "random", "serial", "pointwise", "depthwise", "gauss": bb/ConnectionPolicy.h; reference:
    // include/bb/ConnectionTable.h:150-284).  An unknown policy string throws.
    void InitializeConnection(std::uint64_t seed, std::string const &connection = "")
    {
        BB_ASSERT(m_input_node_size >= 1);
        auto tbl = m_input_table.Lock(true);
        index_t const inputs = m_input_node_size;
        connection_policy::Initialize(seed, connection, m_input_shape, m_output_shape, N, connection_policy::Layout::kChannelFirst,
                                      [&](index_t node, int i, index_t input) {
                                          BB_ASSERT(input >= 0 && input < inputs);
                                          tbl(node, (index_t)i) = (IndexType)input;
                                      });
        m_reverse_table_dirty = true;
    }

    auto Lock_InputTable(void)            { m_reverse_table_dirty = true; return m_input_table.Lock(); }
    auto LockConst_InputTable(void) const { return m_input_table.LockConst(); }
    auto LockDeviceMemConst_InputTable(void) const { return m_input_table.LockDeviceMemoryConst(); }

    auto LockConst_ReverseTable(void)          { BuildReverseTable(); return m_reverse_table.LockConst(); }
    auto LockDeviceMemConst_ReverseTable(void) { BuildReverseTable(); return m_reverse_table.LockDeviceMemoryConst(); }
    index_t GetReverseTableStride(void)        { BuildReverseTable(); return m_reverse_table.GetShape()[1]; }

    std::string GetObjectName(void) const override { return "FixedSizeConnectionTable" + std::to_string(N) + "_" + DataType<IndexType>::Name(); }

protected:
    // version | ConnectionTable part: version, Object version 0, input shape, output shape | input table object
    // (reference: include/bb/FixedSizeConnectionTable.h:50-82, ConnectionTable.h:47-74)
    void DumpObjectData(std::ostream &os) const override
    {
        SaveValue(os, (std::int64_t)1);
        SaveValue(os, (std::int64_t)1);
        SaveValue(os, (std::int64_t)0);
        SaveIndices(os, m_input_shape);
        SaveIndices(os, m_output_shape);
        m_input_table.DumpObject(os);
    }
    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = 0, parent = 0, base = -1;
        LoadValue(is, ver);    BB_ASSERT(ver == 1);
        LoadValue(is, parent); BB_ASSERT(parent == 1);
        LoadValue(is, base);   BB_ASSERT(base == 0);
        indices_t const input_shape = LoadIndices(is), output_shape = LoadIndices(is);
        SetShape(input_shape, output_shape);
        m_input_table.LoadObject(is);
        BB_ASSERT(m_input_table.GetShape() == indices_t({m_output_node_size, (index_t)N}));
        // wiring read from a file is checked before any kernel follows it
        auto tbl = m_input_table.LockConst();
        for (index_t i = 0; i < m_output_node_size * N; ++i) { BB_ASSERT(tbl[i] >= 0 && tbl[i] < m_input_node_size); }
        m_reverse_table_dirty = true;
    }

    void BuildReverseTable(void)
    {
        if (!m_reverse_table_dirty) { return; }
        m_reverse_table_dirty = false;
        auto in_tbl = m_input_table.LockConst();
        std::vector<index_t> fan((std::size_t)m_input_node_size, 0);
        for (index_t o = 0; o < m_output_node_size; ++o) {
            for (int i = 0; i < N; ++i) { fan[(std::size_t)in_tbl(o, i)]++; }
        }
        index_t const width = 1 + (fan.empty() ? 0 : *std::max_element(fan.begin(), fan.end()));
        m_reverse_table.Resize(m_input_node_size, width);
        auto rev = m_reverse_table.Lock(true);
        std::fill(rev.GetAddr(), rev.GetAddr() + m_input_node_size * width, (IndexType)0);
        for (index_t o = 0; o < m_output_node_size; ++o) {
            for (int i = 0; i < N; ++i) {
                index_t const r = in_tbl(o, i);
                IndexType const c = rev(r, 0) + 1;
                rev(r, 0) = c;
                rev(r, c) = (IndexType)(o * N + i);
            }
        }
    }
};

}  // namespace bb

// AverageLut: every output node adds up n wired inputs; with binarize_output it votes (+1 / -1 on sum > 0), on packed bits
// it is the strict majority of the n inputs.  Reference API: include/bb/AverageLut.h:22-458 (Create(n, output_shape,
// connection, binarize, binarize_input, seed); commands binary / binarize_input / binarize_output / host_only; connection
// get/set; GetLutTable = majority of the index bits).  Frame work runs in the HIP library only.
#pragma once

#include <algorithm>
#include <numeric>
#include <random>

#include "bb/Model.h"

namespace bb {

template <typename BinType = float, typename RealType = float>
class AverageLut : public Model {
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
    explicit AverageLut(create_t const &create)
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
    static std::string ModelName(void) { return "AverageLut"; }
    std::string GetModelName(void) const override { return ModelName(); }

    static std::shared_ptr<AverageLut> Create(create_t const &create) { return std::shared_ptr<AverageLut>(new AverageLut(create)); }
    static std::shared_ptr<AverageLut> Create(int n, indices_t const &output_shape, std::string connection = "", bool binarize = true,
                                              bool binarize_input = false, std::uint64_t seed = 1)
    {
        create_t c;
        c.n = n; c.output_shape = output_shape; c.connection = connection; c.binarize_input = binarize_input; c.binarize_output = binarize; c.seed = seed;
        return Create(c);
    }
    static std::shared_ptr<AverageLut> Create(int n, index_t output_node_size, std::string connection = "", bool binarize = true,
                                              bool binarize_input = false, std::uint64_t seed = 1)
    {
        return Create(n, indices_t({output_node_size}), connection, binarize, binarize_input, seed);
    }

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

    // the layer as a look-up table: entry `bitpos` is the majority of its n index bits (AverageLut.h:190-206)
    int  GetLutTableSize(index_t) const { return 1 << m_n; }
    void SetLutTable(index_t, int, bool) {}
    bool GetLutTable(index_t, int bitpos) const
    {
        int count = 0;
        for (int i = 0; i < m_n; ++i) { count += (bitpos & 1) ? +1 : -1; bitpos >>= 1; }
        return count > 0;
    }

    // Seeded wiring.  "serial": node o reads inputs (o*n + i) mod I.  Anything else: inputs are dealt from reshuffled decks
    // of all input nodes, so every input is used about equally often (the permutation itself depends on the random-number
    // library; inject wiring with SetNodeConnectionIndex where it has to match another implementation).
    indices_t SetInputShape(indices_t shape) override
    {
        if (shape == m_input_shape) { return m_output_shape; }
        m_input_shape = shape;
        index_t const I = CalcShapeSize(shape), O = this->GetOutputNodeSize();
        BB_ASSERT(I > 0);
        auto idx = m_input_index.Lock(true);
        if (m_connection == "serial") {
            for (index_t o = 0; o < O; ++o) { for (int i = 0; i < m_n; ++i) { idx(o, i) = (std::int32_t)((o * m_n + i) % I); } }
        }
        else {
            std::mt19937_64 mt(m_mt());
            std::vector<std::int32_t> deck((std::size_t)I);
            std::iota(deck.begin(), deck.end(), 0);
            std::size_t pos = deck.size();
            for (index_t o = 0; o < O; ++o) {
                for (int i = 0; i < m_n; ++i) {
                    if (pos >= deck.size()) { std::shuffle(deck.begin(), deck.end(), mt); pos = 0; }
                    idx(o, i) = deck[pos++];
                }
            }
        }
        return m_output_shape;
    }
    void SetOutputShape(indices_t const &shape)
    {
        BB_ASSERT(CalcShapeSize(shape) == this->GetOutputNodeSize());
        m_output_shape = shape;
    }
    indices_t GetInputShape(void) const override  { return m_input_shape; }
    indices_t GetOutputShape(void) const override { return m_output_shape; }

    FrameBuffer Forward(FrameBuffer x_buf, bool = true) override
    {
        BB_ASSERT(x_buf.GetType() == DataType<BinType>::type);
        if (m_host_only || !Manager::IsDeviceAvailable()) {
            throw Exception("AverageLut::Forward: host-only execution is not provided by this library (device path only)");
        }
        if (x_buf.GetShape() != m_input_shape) { SetInputShape(x_buf.GetShape()); }
        FrameBuffer y_buf(x_buf.GetFrameSize(), m_output_shape, DataType<BinType>::type);
        BB_ASSERT(x_buf.GetFrameStride() == y_buf.GetFrameStride());
        auto x_ptr   = x_buf.LockDeviceMemoryConst();
        auto y_ptr   = y_buf.LockDeviceMemory(true);
        auto idx_ptr = m_input_index.LockDeviceMemoryConst();
        if (DataType<BinType>::type == BB_TYPE_BIT) {
            CheckDevice(bbhip_bit_AverageLut_Forward((int const *)x_ptr.GetAddr(), (int *)y_ptr.GetAddr(), (int const *)idx_ptr.GetAddr(), m_n,
                            (int)y_buf.GetNodeSize(), (int)y_buf.GetFrameSize(), (int)(y_buf.GetFrameStride() / sizeof(int)), nullptr),
                        "bbhip_bit_AverageLut_Forward");
        }
        else {
            CheckDevice(bbhip_fp32_AverageLut_Forward((float const *)x_ptr.GetAddr(), (float *)y_ptr.GetAddr(), (int const *)idx_ptr.GetAddr(), m_n,
                            (int)y_buf.GetNodeSize(), (int)y_buf.GetFrameSize(), (int)(y_buf.GetFrameStride() / sizeof(float)),
                            m_binarize_input ? 1 : 0, m_binarize_output ? 1 : 0, nullptr), "bbhip_fp32_AverageLut_Forward");
        }
        return y_buf;
    }

    FrameBuffer Backward(FrameBuffer dy_buf) override
    {
        if (dy_buf.Empty()) { return dy_buf; }
        BB_ASSERT(dy_buf.GetType() == BB_TYPE_FP32);
        if (m_host_only || !Manager::IsDeviceAvailable()) {
            throw Exception("AverageLut::Backward: host-only execution is not provided by this library (device path only)");
        }
        FrameBuffer dx_buf(dy_buf.GetFrameSize(), m_input_shape, BB_TYPE_FP32);
        auto dy_ptr  = dy_buf.LockDeviceMemoryConst();
        auto dx_ptr  = dx_buf.LockDeviceMemory(true);
        auto idx_ptr = m_input_index.LockDeviceMemoryConst();
        CheckDevice(bbhip_fp32_AverageLut_Backward((float const *)dy_ptr.GetAddr(), (float *)dx_ptr.GetAddr(), (int const *)idx_ptr.GetAddr(), m_n,
                        (int)dx_buf.GetNodeSize(), (int)dy_buf.GetNodeSize(), (int)dy_buf.GetFrameSize(),
                        (int)(dy_buf.GetFrameStride() / sizeof(float)), nullptr), "bbhip_fp32_AverageLut_Backward");
        return dx_buf;
    }
};

}  // namespace bb

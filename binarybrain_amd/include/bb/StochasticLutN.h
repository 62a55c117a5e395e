// StochasticLutN<N, BinType, RealType>: a layer of N-input differentiable look-up tables
//     y = clip( sum_i W[i] * prod_j (bit_j(i) ? x_j : 1 - x_j), 0, 1 )
// with the reference's model API (include/bb/StochasticLutN.h:26-754: Create, SetInputShape, Forward, Backward,
// SendCommand keys binary / lut_binarize / host_only, W/dW access, connection get/set, ForwardNode).
// All frame work runs in the HIP library through the C ABI (include/bbhip.h); there is no host implementation of
// Forward/Backward here — with "host_only true" or without a device the calls throw.
#pragma once

#include <random>

#include "bb/Model.h"
#include "bb/FixedSizeConnectionTable.h"

namespace bb {

template <int N = 6, typename BinType = float, typename RealType = float>
class StochasticLutN : public Model {
    static_assert(std::is_same<RealType, float>::value, "fp32 tables only");
    static constexpr int NN = 1 << N;
    static constexpr bool kBitInput = std::is_same<BinType, Bit>::value;

protected:
    bool        m_host_only = false;
    bool        m_host_simd = true;                 // carried through serialization only: there is no host path here
    bool        m_y_binarize = false;               // likewise
    bool        m_binary_mode = kBitInput;
    bool        m_lut_binarize = true;              // class default of the reference (StochasticLutN.h:45)
    RealType    m_unbinarize_bias = (RealType)0.25;
    index_t     m_max_tmp_mem_size = 256 * 1024 * 1024;
    std::string m_connection;
    indices_t   m_input_shape, m_output_shape;
    FrameBuffer m_x_buf;
    FrameBuffer m_bits_buf;     // the packed copy of m_x_buf that the forward entry made (binary mode on fp32 frames)
    FixedSizeConnectionTable<N> m_connection_table;
    std::shared_ptr<Tensor> m_W, m_dW;
    std::mt19937_64 m_mt;

    void CommandProc(std::vector<std::string> args) override
    {
        Model::CommandProc(args);
        if (!kBitInput && args.size() == 2 && args[0] == "binary") { m_binary_mode = EvalBool(args[1]); }
        if (args.size() == 2 && args[0] == "lut_binarize")         { m_lut_binarize = EvalBool(args[1]); }
        if (args.size() == 2 && args[0] == "host_only")            { m_host_only = EvalBool(args[1]); }
        // kept and serialized as in the reference (StochasticLutN.h:105-120), where no computation reads the first either
        if (args.size() == 2 && args[0] == "y_binarize")           { m_y_binarize = EvalBool(args[1]); }
        if (args.size() == 2 && args[0] == "host_simd")            { m_host_simd = EvalBool(args[1]); }
    }

    void RequireDevice(char const *what) const
    {
        if (m_host_only || !Manager::IsDeviceAvailable()) {
            throw Exception(std::string(what) + ": host-only execution is not provided by this library (device path only)");
        }
    }

public:
    struct create_t {
        indices_t     output_shape;
        std::string   connection;
        std::uint64_t seed = 1;
    };

protected:
    explicit StochasticLutN(create_t const &create)
    {
        BB_ASSERT(!create.output_shape.empty());
        m_output_shape = create.output_shape;
        m_connection = create.connection;
        m_mt.seed(create.seed);
        m_W = std::make_shared<Tensor>();
        m_dW = std::make_shared<Tensor>();
    }

    // the reference's object layout (include/bb/StochasticLutN.h:170-223): version, Model part, flags, tmp size, connection
    // policy, bias, shapes, connection table object, W object
    void DumpObjectData(std::ostream &os) const override
    {
        SaveValue(os, (std::int64_t)1);
        Model::DumpObjectData(os);
        SaveValue(os, m_host_only);
        SaveValue(os, m_host_simd);
        SaveValue(os, m_binary_mode);
        SaveValue(os, m_lut_binarize);
        SaveValue(os, m_y_binarize);
        SaveValue(os, (std::int64_t)m_max_tmp_mem_size);
        SaveValue(os, m_connection);
        SaveValue(os, m_unbinarize_bias);
        SaveValue(os, m_input_shape);
        SaveValue(os, m_output_shape);
        m_connection_table.DumpObject(os);
        m_W->DumpObject(os);
    }
    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = 0, tmp = 0;
        LoadValue(is, ver); BB_ASSERT(ver == 1);
        Model::LoadObjectData(is);
        LoadValue(is, m_host_only);
        LoadValue(is, m_host_simd);
        LoadValue(is, m_binary_mode);
        LoadValue(is, m_lut_binarize);
        LoadValue(is, m_y_binarize);
        LoadValue(is, tmp); m_max_tmp_mem_size = (index_t)tmp;
        LoadValue(is, m_connection);
        LoadValue(is, m_unbinarize_bias);
        LoadValue(is, m_input_shape);
        LoadValue(is, m_output_shape);
        m_connection_table.LoadObject(is);
        m_W->LoadObject(is);
        index_t const O = CalcShapeSize(m_output_shape);
        BB_ASSERT(m_connection_table.GetOutputNodeSize() == O && m_connection_table.GetInputNodeSize() == CalcShapeSize(m_input_shape));
        BB_ASSERT(m_W->GetType() == DataType<RealType>::type && m_W->GetShape() == indices_t({O, (index_t)NN}));
        if (kBitInput) { m_binary_mode = true; }
        m_dW->Resize({O, (index_t)NN}, DataType<RealType>::type);
        m_dW->FillZero();
    }

public:
    static std::string ModelName(void) { return "StochasticLut" + std::to_string(N); }
    static std::string ObjectName(void) { return ModelName() + "_" + DataType<BinType>::Name() + "_" + DataType<RealType>::Name(); }
    std::string GetModelName(void) const override { return ModelName(); }
    std::string GetObjectName(void) const override { return ObjectName(); }

    static std::shared_ptr<StochasticLutN> Create(create_t const &create) { return std::shared_ptr<StochasticLutN>(new StochasticLutN(create)); }
    static std::shared_ptr<StochasticLutN> Create(indices_t const &output_shape, std::string connection = "", std::uint64_t seed = 1)
    {
        create_t c; c.output_shape = output_shape; c.connection = connection; c.seed = seed;
        return Create(c);
    }
    static std::shared_ptr<StochasticLutN> Create(index_t output_node_size, std::string connection = "", std::uint64_t seed = 1)
    {
        return Create(indices_t({output_node_size}), connection, seed);
    }

    Tensor &W(void)  { return *m_W; }
    Tensor &dW(void) { return *m_dW; }
    auto lock_W(void)              { return m_W->Lock<RealType>(); }
    auto lock_W_const(void) const  { return m_W->LockConst<RealType>(); }
    auto lock_dW(void)             { return m_dW->Lock<RealType>(); }
    auto lock_dW_const(void) const { return m_dW->LockConst<RealType>(); }

    index_t GetNodeConnectionSize(index_t) const { return N; }
    void    SetNodeConnectionIndex(index_t node, index_t input_index, index_t input_node) { m_connection_table.SetInputConnection(node, input_index, input_node); }
    index_t GetNodeConnectionIndex(index_t node, index_t input_index) const { return m_connection_table.GetInputConnection(node, input_index); }

    indices_t SetInputShape(indices_t shape) override
    {
        if (shape == m_input_shape) { return m_output_shape; }
        m_input_shape = shape;
        m_connection_table.SetShape(m_input_shape, m_output_shape);
        m_connection_table.InitializeConnection(m_mt(), m_connection);
        m_W->Resize({CalcShapeSize(m_output_shape), (index_t)NN}, DataType<RealType>::type);
        m_W->InitNormalDistribution(0.5, 0.01, m_mt());                     // reference: StochasticLutN.h:335
        m_dW->Resize({CalcShapeSize(m_output_shape), (index_t)NN}, DataType<RealType>::type);
        m_dW->FillZero();
        return m_output_shape;
    }
    indices_t GetInputShape(void) const override  { return m_input_shape; }
    indices_t GetOutputShape(void) const override { return m_output_shape; }

    Variables GetParameters(void) override { Variables v; v.PushBack(m_W);  return v; }
    Variables GetGradients(void) override  { Variables v; v.PushBack(m_dW); return v; }

    // one node, one input vector, evaluated on the host with the defining formula (reference: StochasticLutN.h:384-429)
    std::vector<double> ForwardNode(index_t node, std::vector<double> input_value) const override
    {
        BB_ASSERT((int)input_value.size() == N);
        auto Wp = lock_W_const();
        RealType x[N][2];
        for (int i = 0; i < N; ++i) {
            RealType v = (RealType)input_value[(std::size_t)i];
            v = m_binary_mode ? ((RealType)0.5 + ((v > (RealType)0.5) ? +m_unbinarize_bias : -m_unbinarize_bias))
                              : std::min((RealType)1, std::max((RealType)0, v));
            x[i][0] = (RealType)1 - v;
            x[i][1] = v;
        }
        RealType y = 0;
        for (int i = 0; i < NN; ++i) {
            RealType w = std::min((RealType)1, std::max((RealType)0, Wp(node, i)));
            if (m_lut_binarize) { w = (w > (RealType)0.5) ? (RealType)1 : (RealType)0; }
            for (int j = 0; j < N; ++j) { w *= x[j][(i >> j) & 1]; }
            y += w;
        }
        y = std::min((RealType)1, std::max((RealType)0, y));
        return std::vector<double>(1, (double)y);
    }

    FrameBuffer Forward(FrameBuffer x_buf, bool train = true) override
    {
        BB_ASSERT(x_buf.GetType() == DataType<BinType>::type);
        RequireDevice("StochasticLutN::Forward");
        if (x_buf.GetShape() != m_input_shape) { SetInputShape(x_buf.GetShape()); }
        FrameBuffer y_buf(x_buf.GetFrameSize(), m_output_shape, DataType<RealType>::type);
        if (train) {
            m_x_buf = x_buf;
            // in binary mode the layer reads fp32 frames as bits: the forward entry packs them into a buffer that is kept beside
            // the input and handed back to the backward entry, which then does not pack again (bbhip_HintPackedInput)
            m_bits_buf = FrameBuffer();
            if (!kBitInput && m_binary_mode) { m_bits_buf.Resize(x_buf.GetFrameSize(), m_input_shape, BB_TYPE_BIT); }
        }

        // The table is clamped to [0, 1] in place before every forward pass (reference: StochasticLutN.h:451): for fp32 frames
        // by the forward entry itself, in its table-preparation launch; for packed frames by a call of its own.
        auto x_ptr   = x_buf.LockDeviceMemoryConst();
        auto y_ptr   = y_buf.LockDeviceMemory(true);
        auto idx_ptr = m_connection_table.LockDeviceMemConst_InputTable();
        if (kBitInput) {
            m_W->Clamp_inplace(0.0f, 1.0f);
            auto W_ptr = m_W->LockDeviceMemoryConst();
            CheckDevice(bbhip_bit_fp32_StochasticLut_Forward(N, (int const *)x_ptr.GetAddr(), (float *)y_ptr.GetAddr(),
                            (int const *)idx_ptr.GetAddr(), (float const *)W_ptr.GetAddr(),
                            (int)y_buf.GetNodeSize(), (int)y_buf.GetFrameSize(), (int)(y_buf.GetFrameStride() / sizeof(float)),
                            (int)(x_buf.GetFrameStride() / sizeof(int)), m_lut_binarize ? 1 : 0, (float)m_unbinarize_bias, nullptr),
                        "bbhip_bit_fp32_StochasticLut_Forward");
        }
        else {
            BB_ASSERT(x_buf.GetFrameStride() == y_buf.GetFrameStride());
            auto W_ptr = m_W->LockDeviceMemory();
            if (train && !m_bits_buf.Empty()) {
                auto bits_ptr = m_bits_buf.LockDeviceMemory(true);
                bbhip_HintPackedInput((int *)bits_ptr.GetAddr(), (int)x_buf.GetNodeSize(), (int)(m_bits_buf.GetFrameStride() / sizeof(int)), 0);
            }
            else { bbhip_HintInputNodeSize((int)x_buf.GetNodeSize()); }     // the forward signatures do not carry the input's row count
            CheckDevice(bbhip_fp32_StochasticLut_ForwardClampW(N, (float const *)x_ptr.GetAddr(), (float *)y_ptr.GetAddr(),
                            (int const *)idx_ptr.GetAddr(), (float *)W_ptr.GetAddr(),
                            (int)y_buf.GetNodeSize(), (int)y_buf.GetFrameSize(), (int)(y_buf.GetFrameStride() / sizeof(float)),
                            m_binary_mode ? 1 : 0, m_lut_binarize ? 1 : 0, (float)m_unbinarize_bias, 0.0f, 1.0f, nullptr),
                        "bbhip_fp32_StochasticLut_ForwardClampW");
        }
        return y_buf;
    }

    void Clear(void) override { Model::Clear(); m_x_buf = FrameBuffer(); m_bits_buf = FrameBuffer(); }

    FrameBuffer Backward(FrameBuffer dy_buf) override
    {
        if (dy_buf.Empty()) { return FrameBuffer(); }       // (the reference also drops its dW tensor here — a defect, not kept)
        BB_ASSERT(dy_buf.GetType() == DataType<RealType>::type);
        RequireDevice("StochasticLutN::Backward");
        FrameBuffer x_buf = m_x_buf, bits_buf = m_bits_buf;
        m_x_buf = FrameBuffer();
        m_bits_buf = FrameBuffer();
        BB_ASSERT(!x_buf.Empty() && x_buf.GetFrameSize() == dy_buf.GetFrameSize());
        FrameBuffer dx_buf(dy_buf.GetFrameSize(), m_input_shape, DataType<RealType>::type);

        // scratch for the reference's dx scheme is only allocated when that mode is selected
        FrameBuffer tmp_buf;
        index_t tmp_frame_size = 0;
        if (bbhip_GetDxMode() == 2) {
            tmp_frame_size = m_max_tmp_mem_size / (index_t)(sizeof(float) * (std::size_t)this->GetOutputNodeSize() * N);
            tmp_frame_size = std::max(tmp_frame_size, (index_t)32);
            tmp_frame_size = (tmp_frame_size + 31) & ~(index_t)0x1f;
            tmp_frame_size = std::min(tmp_frame_size, dy_buf.GetFrameSize());
            tmp_buf.Resize(tmp_frame_size, {this->GetOutputNodeSize() * N}, DataType<RealType>::type);
        }

        auto x_ptr   = x_buf.LockDeviceMemoryConst();
        auto dy_ptr  = dy_buf.LockDeviceMemoryConst();
        auto dx_ptr  = dx_buf.LockDeviceMemory(true);
        auto rev_ptr = m_connection_table.LockDeviceMemConst_ReverseTable();
        auto idx_ptr = m_connection_table.LockDeviceMemConst_InputTable();
        auto W_ptr   = m_W->LockDeviceMemoryConst();
        auto dW_ptr  = m_dW->LockDeviceMemory();
        float *tmp_addr = nullptr;
        std::unique_ptr<DevicePtr> tmp_ptr;
        if (!tmp_buf.Empty()) { tmp_ptr.reset(new DevicePtr(tmp_buf.LockDeviceMemory(true))); tmp_addr = (float *)tmp_ptr->GetAddr(); }

        if (kBitInput) {
            CheckDevice(bbhip_bit_fp32_StochasticLut_Backward(N, (int const *)x_ptr.GetAddr(), (float const *)dy_ptr.GetAddr(),
                            (float *)dx_ptr.GetAddr(), tmp_addr, (int const *)idx_ptr.GetAddr(), (int const *)rev_ptr.GetAddr(),
                            (float const *)W_ptr.GetAddr(), (float *)dW_ptr.GetAddr(), (int)m_connection_table.GetReverseTableStride(),
                            (int)dx_buf.GetNodeSize(), (int)dy_buf.GetNodeSize(), (int)dx_buf.GetFrameSize(),
                            (int)(dx_buf.GetFrameStride() / sizeof(float)), (int)(x_buf.GetFrameStride() / sizeof(int)),
                            (int)tmp_frame_size, (int)(tmp_buf.GetFrameStride() / sizeof(float)),
                            m_lut_binarize ? 1 : 0, (float)m_unbinarize_bias, nullptr),
                        "bbhip_bit_fp32_StochasticLut_Backward");
        }
        else {
            if (!bits_buf.Empty() && m_binary_mode && bits_buf.GetFrameSize() == x_buf.GetFrameSize()) {
                auto bits_ptr = bits_buf.LockDeviceMemory();
                bbhip_HintPackedInput((int *)bits_ptr.GetAddr(), (int)x_buf.GetNodeSize(), (int)(bits_buf.GetFrameStride() / sizeof(int)), 1);
            }
            CheckDevice(bbhip_fp32_StochasticLut_Backward(N, (float const *)x_ptr.GetAddr(), (float const *)dy_ptr.GetAddr(),
                            (float *)dx_ptr.GetAddr(), tmp_addr, (int const *)idx_ptr.GetAddr(), (int const *)rev_ptr.GetAddr(),
                            (float const *)W_ptr.GetAddr(), (float *)dW_ptr.GetAddr(), (int)m_connection_table.GetReverseTableStride(),
                            (int)dx_buf.GetNodeSize(), (int)dy_buf.GetNodeSize(), (int)dx_buf.GetFrameSize(),
                            (int)(dx_buf.GetFrameStride() / sizeof(float)),
                            (int)tmp_frame_size, (int)(tmp_buf.GetFrameStride() / sizeof(float)),
                            m_binary_mode ? 1 : 0, m_lut_binarize ? 1 : 0, (float)m_unbinarize_bias, nullptr),
                        "bbhip_fp32_StochasticLut_Backward");
        }
        return dx_buf;
    }
};

}  // namespace bb

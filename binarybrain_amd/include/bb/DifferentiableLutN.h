// DifferentiableLutN<N, BinType, RealType>: the N-input differentiable LUT fused with per-node batch normalisation
// (scalar gamma / beta) and a binarize or hard-tanh output stage, with the reference's model API
// (include/bb/DifferentiableLutN.h:35-1398: create_t, Create, SetInputShape, Forward(train), Backward, commands
// binary / lut_binarize / batch_norm / momentum / backward_break / host_only / parameter_lock, running statistics).
// Numerical semantics are those of the reference's CPU path (:754-1008 forward, :1157-1396 backward): training
// statistics mean / max(1e-5, var) / rstd, running = running*m + stat*(1-m), inference rstd = 1/sqrt(running_var),
// hard-tanh window on dy in both binary and non-binary mode.  Frame work runs in the HIP library only.
#pragma once

#include <stack>

#include <random>

#include "bb/Model.h"
#include "bb/FixedSizeConnectionTable.h"

namespace bb {

template <int N = 6, typename BinType = float, typename RealType = float>
class DifferentiableLutN : public Model {
    static_assert(std::is_same<RealType, float>::value, "fp32 tables only");
    static constexpr int NN = 1 << N;
    static constexpr bool kBitType = std::is_same<BinType, Bit>::value;

protected:
    bool        m_host_only = false;
    bool        m_lut_binarize = false;
    bool        m_binary_mode = true;
    bool        m_batch_norm = true;
    bool        m_backward_break = false;
    bool        m_flagClamp = false;            // W is clamped lazily, once after each backward (reference :605-608, :1022)
    RealType    m_unbinarize_bias = (RealType)0.25;
    index_t     m_max_tmp_mem_size = 256 * 1024 * 1024;
    std::string m_connection;
    indices_t   m_input_shape, m_output_shape;
    FixedSizeConnectionTable<N> m_connection_table;
    std::shared_ptr<Tensor> m_W, m_dW;
    RealType    m_momentum, m_gamma, m_beta;
    Tensor_<RealType> m_mean, m_rstd, m_running_mean, m_running_var;
    std::mt19937_64 m_mt;

    void CommandProc(std::vector<std::string> args) override
    {
        Model::CommandProc(args);
        if (!kBitType && args.size() == 2 && args[0] == "binary") { m_binary_mode = EvalBool(args[1]); }
        if (args.size() == 2 && args[0] == "lut_binarize")   { m_lut_binarize = EvalBool(args[1]); }
        if (args.size() == 2 && args[0] == "host_only")      { m_host_only = EvalBool(args[1]); }
        if (args.size() == 2 && args[0] == "batch_norm")     { m_batch_norm = EvalBool(args[1]); }
        if (args.size() == 2 && args[0] == "momentum")       { m_momentum = (RealType)std::stod(args[1]); }
        if (args.size() == 2 && args[0] == "backward_break") { m_backward_break = EvalBool(args[1]); }
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
        bool          batch_norm = true;
        bool          binary = true;
        std::string   connection;
        RealType      momentum = (RealType)0.9;
        RealType      gamma = (RealType)0.3;
        RealType      beta = (RealType)0.5;
        std::uint64_t seed = 1;
    };

protected:
    explicit DifferentiableLutN(create_t const &create)
    {
        m_output_shape = create.output_shape;
        m_connection = create.connection;
        m_batch_norm = create.batch_norm;
        m_binary_mode = create.binary || kBitType;
        m_momentum = create.momentum;
        m_gamma = create.gamma;
        m_beta = create.beta;
        m_mt.seed(create.seed);
        m_W = std::make_shared<Tensor>();
        m_dW = std::make_shared<Tensor>();
    }

    // the reference's object layout (include/bb/DifferentiableLutN.h:266-334): version, Model part, flags, shapes, connection
    // table object, W object, bias, momentum, gamma, beta, running mean and variance objects
    void DumpObjectData(std::ostream &os) const override
    {
        SaveValue(os, (std::int64_t)1);
        Model::DumpObjectData(os);
        SaveValue(os, m_host_only);
        SaveValue(os, m_lut_binarize);
        SaveValue(os, m_binary_mode);
        SaveValue(os, m_batch_norm);
        SaveValue(os, m_flagClamp);
        SaveValue(os, m_input_shape);
        SaveValue(os, m_output_shape);
        m_connection_table.DumpObject(os);
        m_W->DumpObject(os);
        SaveValue(os, m_unbinarize_bias);
        SaveValue(os, m_momentum);
        SaveValue(os, m_gamma);
        SaveValue(os, m_beta);
        m_running_mean.DumpObject(os);
        m_running_var.DumpObject(os);
    }
    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = 0;
        LoadValue(is, ver); BB_ASSERT(ver == 1);
        Model::LoadObjectData(is);
        LoadValue(is, m_host_only);
        LoadValue(is, m_lut_binarize);
        LoadValue(is, m_binary_mode);
        LoadValue(is, m_batch_norm);
        LoadValue(is, m_flagClamp);
        LoadValue(is, m_input_shape);
        LoadValue(is, m_output_shape);
        m_connection_table.LoadObject(is);
        m_W->LoadObject(is);
        LoadValue(is, m_unbinarize_bias);
        LoadValue(is, m_momentum);
        LoadValue(is, m_gamma);
        LoadValue(is, m_beta);
        m_running_mean.LoadObject(is);
        m_running_var.LoadObject(is);
        index_t const O = CalcShapeSize(m_output_shape);
        BB_ASSERT(m_connection_table.GetOutputNodeSize() == O && m_connection_table.GetInputNodeSize() == CalcShapeSize(m_input_shape));
        BB_ASSERT(m_W->GetType() == DataType<RealType>::type && m_W->GetShape() == indices_t({O, (index_t)NN}));
        BB_ASSERT(m_running_mean.GetSize() == O && m_running_var.GetSize() == O);
        if (kBitType) { m_binary_mode = true; }
        m_dW->Resize(m_W->GetShape(), DataType<RealType>::type);
        m_dW->FillZero();
        m_mean.Resize(m_output_shape);
        m_rstd.Resize(m_output_shape);
    }

public:
    static std::string ModelName(void) { return "DifferentiableLut" + std::to_string(N); }
    static std::string ObjectName(void) { return ModelName() + "_" + DataType<BinType>::Name() + "_" + DataType<RealType>::Name(); }
    std::string GetModelName(void) const override { return ModelName(); }
    std::string GetObjectName(void) const override { return ObjectName(); }

    static std::shared_ptr<DifferentiableLutN> Create(create_t const &create) { return std::shared_ptr<DifferentiableLutN>(new DifferentiableLutN(create)); }
    static std::shared_ptr<DifferentiableLutN> Create(indices_t const &output_shape, bool batch_norm = true, std::string connection = "")
    {
        create_t c; c.output_shape = output_shape; c.batch_norm = batch_norm; c.connection = connection;
        return Create(c);
    }
    static std::shared_ptr<DifferentiableLutN> Create(index_t output_node_size, bool batch_norm = true, std::string connection = "")
    {
        return Create(indices_t({output_node_size}), batch_norm, connection);
    }

    Tensor &W(void)  { return *m_W; }
    Tensor &dW(void) { return *m_dW; }
    auto lock_W(void)              { return m_W->Lock<RealType>(); }
    auto lock_W_const(void) const  { return m_W->LockConst<RealType>(); }
    auto lock_dW(void)             { return m_dW->Lock<RealType>(); }
    auto lock_dW_const(void) const { return m_dW->LockConst<RealType>(); }
    auto lock_mean(void)                  { return m_running_mean.Lock(); }
    auto lock_mean_const(void) const      { return m_running_mean.LockConst(); }
    auto lock_var(void)                   { return m_running_var.Lock(); }
    auto lock_var_const(void) const       { return m_running_var.LockConst(); }
    auto lock_tmp_mean_const(void) const  { return m_mean.LockConst(); }
    auto lock_tmp_rstd_const(void) const  { return m_rstd.LockConst(); }
    double GetGamma(void) const { return (double)m_gamma; }
    double GetBeta(void) const  { return (double)m_beta; }

    index_t GetNodeConnectionSize(index_t) const { return N; }
    void    SetNodeConnectionIndex(index_t node, index_t input_index, index_t input_node) { m_connection_table.SetInputConnection(node, input_index, input_node); }
    index_t GetNodeConnectionIndex(index_t node, index_t input_index) const { return m_connection_table.GetInputConnection(node, input_index); }

    indices_t SetInputShape(indices_t shape) override
    {
        if (shape == m_input_shape) { return m_output_shape; }
        m_input_shape = shape;
        m_connection_table.SetShape(m_input_shape, m_output_shape);
        m_connection_table.InitializeConnection(m_mt(), m_connection);
        m_W->Resize({this->GetOutputNodeSize(), (index_t)NN}, DataType<RealType>::type);
        m_W->InitNormalDistribution(0.5, 0.01, m_mt());
        m_dW->Resize({this->GetOutputNodeSize(), (index_t)NN}, DataType<RealType>::type);
        m_dW->FillZero();
        m_mean.Resize(m_output_shape);
        m_rstd.Resize(m_output_shape);
        m_running_mean.Resize(m_output_shape); m_running_mean = (RealType)0.0;
        m_running_var.Resize(m_output_shape);  m_running_var = (RealType)1.0;
        return m_output_shape;
    }
    indices_t GetInputShape(void) const override  { return m_input_shape; }
    indices_t GetOutputShape(void) const override { return m_output_shape; }

    Variables GetParameters(void) override { Variables v; if (!m_parameter_lock) { v.PushBack(m_W); }  return v; }
    Variables GetGradients(void) override  { Variables v; if (!m_parameter_lock) { v.PushBack(m_dW); } return v; }

    // one node on the host with the running statistics (reference: DifferentiableLutN.h:527-586)
    std::vector<double> ForwardNode(index_t node, std::vector<double> input_value) const override
    {
        BB_ASSERT((int)input_value.size() == N);
        auto Wp = lock_W_const();
        RealType x[N];
        for (int i = 0; i < N; ++i) {
            RealType v = (RealType)input_value[(std::size_t)i];
            x[i] = m_binary_mode ? ((RealType)0.5 + ((v > (RealType)0.5) ? +m_unbinarize_bias : -m_unbinarize_bias))
                                 : std::min((RealType)1, std::max((RealType)0, v));
        }
        RealType y = 0;
        for (int i = 0; i < NN; ++i) {
            RealType w = Wp(node, i);
            if (m_flagClamp) { w = std::min((RealType)1, std::max((RealType)0, w)); }
            if (m_lut_binarize) { w = (w > (RealType)0.5) ? (RealType)1 : (RealType)0; }
            for (int j = 0; j < N; ++j) { w *= ((i >> j) & 1) ? x[j] : ((RealType)1 - x[j]); }
            y += w;
        }
        if (m_batch_norm) {
            RealType const mean = lock_mean_const()[node];
            RealType const rstd = (RealType)1 / std::sqrt(lock_var_const()[node]);
            y = (y - mean) * rstd;
            y = y * m_gamma + m_beta;
        }
        y = m_binary_mode ? ((y > (RealType)0.5) ? (RealType)1 : (RealType)0) : std::max((RealType)0, std::min((RealType)1, y));
        return std::vector<double>(1, (double)y);
    }

private:
    // A layer on fp32 frames in binary mode reads its input as bits.  The forward entry packs them into a buffer that the layer
    // keeps beside the input it keeps anyway, and hands it back to the backward entry, which then does not pack again
    // (bbhip_HintPackedInput).  One packed buffer per kept input, in the same order.
    std::stack<FrameBuffer> m_packed_bufs;

    // the hint for a call on x_buf: with `bits` the packed copy's place (or the copy itself, holds_input), else only the row count
    void HintInput(FrameBuffer const &x_buf, FrameBuffer *bits, bool holds_input)
    {
        if (bits != nullptr && !bits->Empty()) {
            int const rows = (int)x_buf.GetNodeSize(), words = (int)(bits->GetFrameStride() / 4);
            if (holds_input) { bbhip_HintPackedInput((int *)bits->LockDeviceMemoryConst().GetAddr(), rows, words, 1); }
            else             { bbhip_HintPackedInput((int *)bits->LockDeviceMemory(true).GetAddr(), rows, words, 0); }
        }
        else { bbhip_HintInputNodeSize((int)x_buf.GetNodeSize()); }         // the forward signatures do not carry the input's row count
    }

    // A layer in binary mode on fp32 frames binarizes its output; the layer behind it, if it is one of these too, reads that output as
    // bits.  The forward entry writes the packed copy in the launch that binarizes (bbhip_HintPackedOutput) and it travels with the
    // output buffer (FrameBuffer::AttachPackedTwin): the next layer's forward and backward calls then pack nothing.
    FrameBuffer OfferPackedOutput(FrameBuffer const &y_buf)
    {
        FrameBuffer bits;
        if (kBitType || !m_binary_mode) { return bits; }
        bits.Resize(y_buf.GetFrameSize(), m_output_shape, BB_TYPE_BIT);
        bbhip_HintPackedOutput((int *)bits.LockDeviceMemory(true).GetAddr(), (int)y_buf.GetNodeSize(), (int)(bits.GetFrameStride() / 4));
        return bits;
    }

    // The tables that the entry points derive from W before their kernels run (centred coefficients, corner values) are the same
    // for every call between two changes of W.  A batch-norm training forward call writes them into a buffer of the layer's, and the
    // backward calls that follow take them from there instead of preparing them again (bbhip_HintPreparedTables) — as long as nobody
    // took a writable lock on W since and the layer's modes are those of the call that filled the buffer.
    std::shared_ptr<Memory>                  m_tables;
    std::pair<void const *, std::uint64_t>   m_tables_stamp{nullptr, 0};
    int                                      m_tables_modes = -1;
    float                                    m_tables_bias = 0.0f;      // the corner values depend on unbinarize_bias

    int TableModes(void) const { return (m_lut_binarize ? 1 : 0) | (m_binary_mode ? 2 : 0); }

    // before a training forward call, after its locks on W were taken
    void OfferTables(void)
    {
        std::size_t const bytes = bbhip_PreparedTablesBytes(N, (int)this->GetOutputNodeSize());
        if (bytes == 0) { return; }
        if (!m_tables || m_tables->GetSize() != bytes) { m_tables = Memory::Create(bytes); }
        bbhip_HintPreparedTables((float *)m_tables->LockDevice(true), bytes, 0);
        m_tables_modes = -1;            // not filled yet: KeepTables() after the entry has returned success
    }

    // after the training forward entry returned success: the buffer holds the tables of this W and these modes
    void KeepTables(void)
    {
        if (!m_tables) { return; }
        m_tables_stamp = m_W->WriteStamp();
        m_tables_modes = TableModes();
        m_tables_bias  = m_unbinarize_bias;
    }

    // before a backward call
    void ReturnTables(void)
    {
        if (m_tables && m_tables_modes == TableModes() && m_tables_bias == m_unbinarize_bias && m_tables_stamp == m_W->WriteStamp()) {
            bbhip_HintPreparedTables((float *)m_tables->LockDevice(), m_tables->GetSize(), 1);
        }
    }

public:
    void Clear(void) override
    {
        Model::Clear();
        while (!m_packed_bufs.empty()) { m_packed_bufs.pop(); }
        m_tables_modes = -1;
    }

    FrameBuffer Forward(FrameBuffer x_buf, bool train = true) override
    {
        RequireDevice("DifferentiableLutN::Forward");
        if (x_buf.GetShape() != m_input_shape) { SetInputShape(x_buf.GetShape()); }
        FrameBuffer y_buf(x_buf.GetFrameSize(), m_output_shape, DataType<BinType>::type);
        if (train) { this->PushFrameBuffer(x_buf); }
        // The table is clamped to [0, 1] once after each backward pass (reference :605-608): by the training-forward entry
        // itself, in its table-preparation launch, on the batch-norm training path; by a call of its own otherwise.
        bool const clamp_in_entry = m_flagClamp && m_batch_norm && train;
        if (m_flagClamp && !clamp_in_entry) { m_W->Clamp_inplace(0.0f, 1.0f); }
        m_flagClamp = false;
        if (!kBitType && x_buf.GetType() == BB_TYPE_BIT) { x_buf = x_buf.ConvertBitToFP32(); }      // reference :610-613
        BB_ASSERT(x_buf.GetType() == DataType<BinType>::type);

        int const O = (int)y_buf.GetNodeSize(), F = (int)y_buf.GetFrameSize();
        int const y_stride = (int)(y_buf.GetFrameStride() / 4), x_stride = (int)(x_buf.GetFrameStride() / 4);
        if (!kBitType) { BB_ASSERT(x_stride == y_stride); }
        // the packed copy of a binarized fp32 input: the one that came with the buffer from the layer that wrote it, else (training) a
        // place for the entry to pack into; kept for the backward pass of a training call
        FrameBuffer bits_buf;
        bool have_bits = false;
        if (!kBitType && m_binary_mode) {
            bits_buf = x_buf.GetPackedTwin();
            have_bits = !bits_buf.Empty();
            if (!have_bits && train && !m_backward_break) { bits_buf.Resize(x_buf.GetFrameSize(), m_input_shape, BB_TYPE_BIT); }
        }
        if (train) { m_packed_bufs.push(bits_buf); }
        auto x_ptr   = x_buf.LockDeviceMemoryConst();
        auto y_ptr   = y_buf.LockDeviceMemory(true);
        FrameBuffer y_bits;
        auto idx_ptr = m_connection_table.LockDeviceMemConst_InputTable();
        if (clamp_in_entry) {
            auto W_mut    = m_W->LockDeviceMemory();
            auto mean_ptr = m_mean.LockDeviceMemory(true);
            auto rstd_ptr = m_rstd.LockDeviceMemory(true);
            auto rm_ptr   = m_running_mean.LockDeviceMemory();
            auto rv_ptr   = m_running_var.LockDeviceMemory();
            OfferTables();
            if (kBitType) {
                CheckDevice(bbhip_bit_fp32_DifferentiableLutN_ForwardTrainingClampW(N, (int const *)x_ptr.GetAddr(), (int *)y_ptr.GetAddr(),
                                (int const *)idx_ptr.GetAddr(), (float *)W_mut.GetAddr(), (float *)mean_ptr.GetAddr(), (float *)rstd_ptr.GetAddr(),
                                (float *)rm_ptr.GetAddr(), (float *)rv_ptr.GetAddr(), m_gamma, m_beta, m_momentum, m_unbinarize_bias,
                                O, F, y_stride, m_lut_binarize ? 1 : 0, 0.0f, 1.0f, nullptr), "bbhip_bit_fp32_DifferentiableLutN_ForwardTrainingClampW");
            }
            else {
                HintInput(x_buf, &bits_buf, have_bits);
                y_bits = OfferPackedOutput(y_buf);
                CheckDevice(bbhip_fp32_DifferentiableLutN_ForwardTrainingClampW(N, (float const *)x_ptr.GetAddr(), (float *)y_ptr.GetAddr(),
                                (int const *)idx_ptr.GetAddr(), (float *)W_mut.GetAddr(), (float *)mean_ptr.GetAddr(), (float *)rstd_ptr.GetAddr(),
                                (float *)rm_ptr.GetAddr(), (float *)rv_ptr.GetAddr(), m_gamma, m_beta, m_momentum, m_unbinarize_bias,
                                O, F, y_stride, m_lut_binarize ? 1 : 0, m_binary_mode ? 1 : 0, 0.0f, 1.0f, nullptr),
                            "bbhip_fp32_DifferentiableLutN_ForwardTrainingClampW");
            }
            KeepTables();
            if (!y_bits.Empty()) { y_buf.AttachPackedTwin(y_bits); }
            return y_buf;
        }
        auto W_ptr   = m_W->LockDeviceMemoryConst();

        if (m_batch_norm && train) {
            auto mean_ptr = m_mean.LockDeviceMemory(true);
            auto rstd_ptr = m_rstd.LockDeviceMemory(true);
            auto rm_ptr   = m_running_mean.LockDeviceMemory();
            auto rv_ptr   = m_running_var.LockDeviceMemory();
            OfferTables();
            if (kBitType) {
                CheckDevice(bbhip_bit_fp32_DifferentiableLutN_ForwardTraining(N, (int const *)x_ptr.GetAddr(), (int *)y_ptr.GetAddr(),
                                (int const *)idx_ptr.GetAddr(), (float const *)W_ptr.GetAddr(), (float *)mean_ptr.GetAddr(), (float *)rstd_ptr.GetAddr(),
                                (float *)rm_ptr.GetAddr(), (float *)rv_ptr.GetAddr(), m_gamma, m_beta, m_momentum, m_unbinarize_bias,
                                O, F, y_stride, m_lut_binarize ? 1 : 0, nullptr), "bbhip_bit_fp32_DifferentiableLutN_ForwardTraining");
            }
            else {
                HintInput(x_buf, &bits_buf, have_bits);
                y_bits = OfferPackedOutput(y_buf);
                CheckDevice(bbhip_fp32_DifferentiableLutN_ForwardTraining(N, (float const *)x_ptr.GetAddr(), (float *)y_ptr.GetAddr(),
                                (int const *)idx_ptr.GetAddr(), (float const *)W_ptr.GetAddr(), (float *)mean_ptr.GetAddr(), (float *)rstd_ptr.GetAddr(),
                                (float *)rm_ptr.GetAddr(), (float *)rv_ptr.GetAddr(), m_gamma, m_beta, m_momentum, m_unbinarize_bias,
                                O, F, y_stride, m_lut_binarize ? 1 : 0, m_binary_mode ? 1 : 0, nullptr), "bbhip_fp32_DifferentiableLutN_ForwardTraining");
            }
            KeepTables();
        }
        else if (m_batch_norm) {
            auto rm_ptr = m_running_mean.LockDeviceMemoryConst();
            auto rv_ptr = m_running_var.LockDeviceMemoryConst();
            if (kBitType) {
                CheckDevice(bbhip_bit_fp32_DifferentiableLutN_ForwardInference(N, (int const *)x_ptr.GetAddr(), (int *)y_ptr.GetAddr(),
                                (int const *)idx_ptr.GetAddr(), (float const *)W_ptr.GetAddr(), (float const *)rm_ptr.GetAddr(), (float const *)rv_ptr.GetAddr(),
                                m_gamma, m_beta, m_unbinarize_bias, O, F, y_stride, m_lut_binarize ? 1 : 0, nullptr),
                            "bbhip_bit_fp32_DifferentiableLutN_ForwardInference");
            }
            else {
                HintInput(x_buf, &bits_buf, have_bits);
                y_bits = OfferPackedOutput(y_buf);
                CheckDevice(bbhip_fp32_DifferentiableLutN_ForwardInference(N, (float const *)x_ptr.GetAddr(), (float *)y_ptr.GetAddr(),
                                (int const *)idx_ptr.GetAddr(), (float const *)W_ptr.GetAddr(), (float const *)rm_ptr.GetAddr(), (float const *)rv_ptr.GetAddr(),
                                m_gamma, m_beta, m_unbinarize_bias, O, F, y_stride, m_lut_binarize ? 1 : 0, m_binary_mode ? 1 : 0, nullptr),
                            "bbhip_fp32_DifferentiableLutN_ForwardInference");
            }
        }
        else if (kBitType) {
            CheckDevice(bbhip_bit_bit_fp32_StochasticLut_Forward(N, (int const *)x_ptr.GetAddr(), (int *)y_ptr.GetAddr(),
                            (int const *)idx_ptr.GetAddr(), (float const *)W_ptr.GetAddr(), O, F, y_stride,
                            m_lut_binarize ? 1 : 0, m_unbinarize_bias, nullptr), "bbhip_bit_bit_fp32_StochasticLut_Forward");
        }
        else {
            HintInput(x_buf, &bits_buf, have_bits);
            y_bits = OfferPackedOutput(y_buf);
            CheckDevice(bbhip_fp32_DifferentiableLutN_ForwardNoBn(N, (float const *)x_ptr.GetAddr(), (float *)y_ptr.GetAddr(),
                            (int const *)idx_ptr.GetAddr(), (float const *)W_ptr.GetAddr(), m_unbinarize_bias, O, F, y_stride,
                            m_lut_binarize ? 1 : 0, m_binary_mode ? 1 : 0, nullptr), "bbhip_fp32_DifferentiableLutN_ForwardNoBn");
        }
        if (!y_bits.Empty()) { y_buf.AttachPackedTwin(y_bits); }
        return y_buf;
    }

    FrameBuffer Backward(FrameBuffer dy_buf) override
    {
        if (m_backward_break || dy_buf.Empty()) {          // a frozen layer: no gradient of its own, none passed on (reference :1015-1018)
            m_dW->FillZero();
            // (what the matching forward pass kept is let go, or a frozen layer would hold one input and one packed copy per step)
            if (!this->m_bufs.empty()) { this->m_bufs.pop(); }
            if (!m_packed_bufs.empty()) { m_packed_bufs.pop(); }
            return FrameBuffer();
        }
        BB_ASSERT(dy_buf.GetType() == DataType<RealType>::type);
        RequireDevice("DifferentiableLutN::Backward");
        m_flagClamp = true;
        FrameBuffer x_buf = this->PopFrameBuffer();
        FrameBuffer bits_buf;
        if (!m_packed_bufs.empty()) { bits_buf = m_packed_bufs.top(); m_packed_bufs.pop(); }
        if (!kBitType && x_buf.GetType() == BB_TYPE_BIT) { x_buf = x_buf.ConvertBitToFP32(); }
        BB_ASSERT(x_buf.GetType() == DataType<BinType>::type && x_buf.GetFrameSize() == dy_buf.GetFrameSize());
        if (!bits_buf.Empty() && (bits_buf.GetFrameSize() != x_buf.GetFrameSize() || !m_binary_mode)) { bits_buf = FrameBuffer(); }
        FrameBuffer dx_buf(dy_buf.GetFrameSize(), m_input_shape, DataType<RealType>::type);

        FrameBuffer tmp_buf;
        index_t tmp_frame_size = 0;
        if (bbhip_GetDxMode() == 2) {
            tmp_frame_size = m_max_tmp_mem_size / (index_t)(sizeof(float) * (std::size_t)this->GetOutputNodeSize() * N);
            tmp_frame_size = std::max(tmp_frame_size, (index_t)32);
            tmp_frame_size = (tmp_frame_size + 31) & ~(index_t)0x1f;
            tmp_frame_size = std::min(tmp_frame_size, dy_buf.GetFrameSize());
            tmp_buf.Resize(tmp_frame_size, {this->GetOutputNodeSize() * N}, DataType<RealType>::type);
        }
        float *tmp_addr = nullptr;
        std::unique_ptr<DevicePtr> tmp_ptr;
        if (!tmp_buf.Empty()) { tmp_ptr.reset(new DevicePtr(tmp_buf.LockDeviceMemory(true))); tmp_addr = (float *)tmp_ptr->GetAddr(); }

        int const I = (int)dx_buf.GetNodeSize(), O = (int)dy_buf.GetNodeSize(), F = (int)dy_buf.GetFrameSize();
        int const stride = (int)(dx_buf.GetFrameStride() / 4), x_stride = (int)(x_buf.GetFrameStride() / 4);
        int const tmp_stride = (int)(tmp_buf.GetFrameStride() / 4);
        auto x_ptr   = x_buf.LockDeviceMemoryConst();
        auto dy_ptr  = dy_buf.LockDeviceMemoryConst();
        auto dx_ptr  = dx_buf.LockDeviceMemory(true);
        auto rev_ptr = m_connection_table.LockDeviceMemConst_ReverseTable();
        auto idx_ptr = m_connection_table.LockDeviceMemConst_InputTable();
        auto W_ptr   = m_W->LockDeviceMemoryConst();
        auto dW_ptr  = m_dW->LockDeviceMemory();
        int const rev_stride = (int)m_connection_table.GetReverseTableStride();

        if (m_batch_norm) {
            // with a locked parameter set the statistics of inference are used (reference :1048-1051)
            Tensor_<RealType> mean(m_output_shape), rstd(m_output_shape);
            if (m_parameter_lock) {
                auto rm = m_running_mean.LockConst(); auto rv = m_running_var.LockConst();
                auto mp = mean.Lock(true); auto rp = rstd.Lock(true);
                for (index_t n = 0; n < O; ++n) { mp[n] = rm[n]; rp[n] = (RealType)1 / std::sqrt(rv[n] + (RealType)1.0e-7); }
            }
            auto mean_ptr = m_parameter_lock ? mean.LockDeviceMemoryConst() : m_mean.LockDeviceMemoryConst();
            auto rstd_ptr = m_parameter_lock ? rstd.LockDeviceMemoryConst() : m_rstd.LockDeviceMemoryConst();
            Tensor_<RealType> dmean(m_output_shape), dvar(m_output_shape);
            auto dmean_ptr = dmean.LockDeviceMemory(true);
            auto dvar_ptr  = dvar.LockDeviceMemory(true);
            ReturnTables();
            if (kBitType) {
                CheckDevice(bbhip_bit_fp32_DifferentiableLutN_Backward(N, (int const *)x_ptr.GetAddr(), (float const *)dy_ptr.GetAddr(), (float *)dx_ptr.GetAddr(),
                                tmp_addr, (int const *)idx_ptr.GetAddr(), (int const *)rev_ptr.GetAddr(), (float const *)W_ptr.GetAddr(), (float *)dW_ptr.GetAddr(),
                                (float const *)mean_ptr.GetAddr(), (float const *)rstd_ptr.GetAddr(), (float *)dmean_ptr.GetAddr(), (float *)dvar_ptr.GetAddr(),
                                m_gamma, m_beta, m_unbinarize_bias, rev_stride, I, O, F, stride, x_stride, (int)tmp_frame_size, tmp_stride,
                                m_lut_binarize ? 1 : 0, nullptr), "bbhip_bit_fp32_DifferentiableLutN_Backward");
            }
            else {
                if (!bits_buf.Empty()) { HintInput(x_buf, &bits_buf, true); }
                CheckDevice(bbhip_fp32_DifferentiableLutN_Backward(N, (float const *)x_ptr.GetAddr(), (float const *)dy_ptr.GetAddr(), (float *)dx_ptr.GetAddr(),
                                tmp_addr, (int const *)idx_ptr.GetAddr(), (int const *)rev_ptr.GetAddr(), (float const *)W_ptr.GetAddr(), (float *)dW_ptr.GetAddr(),
                                (float const *)mean_ptr.GetAddr(), (float const *)rstd_ptr.GetAddr(), (float *)dmean_ptr.GetAddr(), (float *)dvar_ptr.GetAddr(),
                                m_gamma, m_beta, m_unbinarize_bias, rev_stride, I, O, F, stride, (int)tmp_frame_size, tmp_stride,
                                m_lut_binarize ? 1 : 0, m_binary_mode ? 1 : 0, nullptr), "bbhip_fp32_DifferentiableLutN_Backward");
            }
        }
        else if (kBitType) {
            CheckDevice(bbhip_bit_fp32_StochasticLut_Backward(N, (int const *)x_ptr.GetAddr(), (float const *)dy_ptr.GetAddr(), (float *)dx_ptr.GetAddr(),
                            tmp_addr, (int const *)idx_ptr.GetAddr(), (int const *)rev_ptr.GetAddr(), (float const *)W_ptr.GetAddr(), (float *)dW_ptr.GetAddr(),
                            rev_stride, I, O, F, stride, x_stride, (int)tmp_frame_size, tmp_stride, m_lut_binarize ? 1 : 0, m_unbinarize_bias, nullptr),
                        "bbhip_bit_fp32_StochasticLut_Backward");
        }
        else {
            if (!bits_buf.Empty()) { HintInput(x_buf, &bits_buf, true); }
            CheckDevice(bbhip_fp32_StochasticLut_Backward(N, (float const *)x_ptr.GetAddr(), (float const *)dy_ptr.GetAddr(), (float *)dx_ptr.GetAddr(),
                            tmp_addr, (int const *)idx_ptr.GetAddr(), (int const *)rev_ptr.GetAddr(), (float const *)W_ptr.GetAddr(), (float *)dW_ptr.GetAddr(),
                            rev_stride, I, O, F, stride, (int)tmp_frame_size, tmp_stride, m_binary_mode ? 1 : 0, m_lut_binarize ? 1 : 0,
                            m_unbinarize_bias, nullptr), "bbhip_fp32_StochasticLut_Backward");
        }
        return dx_buf;
    }
};

}  // namespace bb

// DifferentiableLutDiscreteN: the differentiable LUT layer put together from its three parts, StochasticLutN ->
// StochasticBatchNormalization -> HardTanh over [0, 1] (which binarizes at 0.5 in binary mode and with Bit output) — what
// DifferentiableLutN computes in fused kernels (reference API: include/bb/DifferentiableLutDiscreteN.h:30-470:
// Create(output_shape | output_node_size, batch_norm, connection, seed), the table / wiring / statistics accessors of its
// parts, Forward, Backward, command "memory_saving").  With "memory_saving true" a training pass keeps only the layer's
// input and the backward pass recomputes the intermediate results with the batch statistics of the first pass.
// Serialized as  version 1 | Model part | memory_saving | batch_norm | activation | StochasticLutN object |
// [StochasticBatchNormalization object] | [HardTanh object]  (reference :392-425).
#pragma once

#include "bb/StochasticLutN.h"
#include "bb/StochasticBatchNormalization.h"
#include "bb/HardTanh.h"

namespace bb {

template <int N = 6, typename BinType = float, typename RealType = float>
class DifferentiableLutDiscreteN : public Model {
    bool m_memory_saving = false;
    bool m_bn_enable = true;
    bool m_act_enable = true;
    std::shared_ptr<StochasticLutN<N, BinType, RealType>>   m_lut;
    std::shared_ptr<StochasticBatchNormalization<RealType>> m_batch_norm;
    std::shared_ptr<HardTanh<BinType, RealType>>            m_activation;

public:
    struct create_t {
        indices_t     output_shape;
        std::string   connection;
        bool          batch_norm = true;
        bool          activation = true;
        RealType      momentum = (RealType)0.0;
        RealType      gamma = (RealType)0.3;
        RealType      beta = (RealType)0.5;
        std::uint64_t seed = 1;
    };

protected:
    explicit DifferentiableLutDiscreteN(create_t const &create) : m_bn_enable(create.batch_norm), m_act_enable(create.activation)
    {
        typename StochasticLutN<N, BinType, RealType>::create_t lut_create;
        lut_create.output_shape = create.output_shape;
        lut_create.connection   = create.connection;
        lut_create.seed         = create.seed;
        m_lut        = StochasticLutN<N, BinType, RealType>::Create(lut_create);
        m_batch_norm = StochasticBatchNormalization<RealType>::Create(create.momentum, create.gamma, create.beta);
        m_activation = HardTanh<BinType, RealType>::Create((RealType)0, (RealType)1);
    }

    void CommandProc(std::vector<std::string> args) override
    {
        Model::CommandProc(args);
        if (args.size() == 2 && args[0] == "memory_saving") { m_memory_saving = EvalBool(args[1]); }
    }

    void DumpObjectData(std::ostream &os) const override
    {
        SaveValue(os, (std::int64_t)1);
        Model::DumpObjectData(os);
        SaveValue(os, m_memory_saving);
        SaveValue(os, m_bn_enable);
        SaveValue(os, m_act_enable);
        m_lut->DumpObject(os);
        if (m_bn_enable)  { m_batch_norm->DumpObject(os); }
        if (m_act_enable) { m_activation->DumpObject(os); }
    }

    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = -1;
        LoadValue(is, ver);
        BB_ASSERT(ver == 1);
        Model::LoadObjectData(is);
        LoadValue(is, m_memory_saving);
        LoadValue(is, m_bn_enable);
        LoadValue(is, m_act_enable);
        BB_ASSERT(is.good());
        m_lut->LoadObject(is);
        if (m_bn_enable)  { m_batch_norm->LoadObject(is); }
        if (m_act_enable) { m_activation->LoadObject(is); }
    }

public:
    static std::string ModelName(void)  { return "DifferentiableLutDiscrete" + std::to_string(N); }
    static std::string ObjectName(void) { return ModelName() + "_" + DataType<BinType>::Name() + "_" + DataType<RealType>::Name(); }
    std::string GetModelName(void) const override  { return ModelName(); }
    std::string GetObjectName(void) const override { return ObjectName(); }

    static std::shared_ptr<DifferentiableLutDiscreteN> Create(create_t const &create)
    {
        return std::shared_ptr<DifferentiableLutDiscreteN>(new DifferentiableLutDiscreteN(create));
    }
    static std::shared_ptr<DifferentiableLutDiscreteN> Create(indices_t const &output_shape, bool batch_norm = true, std::string connection = "",
                                                              std::uint64_t seed = 1)
    {
        create_t c;
        c.output_shape = output_shape; c.connection = connection; c.batch_norm = batch_norm; c.seed = seed;
        return Create(c);
    }
    static std::shared_ptr<DifferentiableLutDiscreteN> Create(index_t output_node_size, bool batch_norm = true, std::string connection = "",
                                                              std::uint64_t seed = 1)
    {
        return Create(indices_t({output_node_size}), batch_norm, connection, seed);
    }
    static std::shared_ptr<DifferentiableLutDiscreteN> Create(void) { return Create(create_t()); }

    void SendCommand(std::string command, std::string send_to = "all") override
    {
        Model::SendCommand(command, send_to);
        m_lut->SendCommand(command, send_to);
        m_batch_norm->SendCommand(command, send_to);
        m_activation->SendCommand(command, send_to);
    }

    Tensor &W(void)  { return m_lut->W(); }
    Tensor &dW(void) { return m_lut->dW(); }
    auto lock_W(void)                    { return m_lut->lock_W(); }
    auto lock_W_const(void) const        { return m_lut->lock_W_const(); }
    auto lock_dW(void)                   { return m_lut->lock_dW(); }
    auto lock_dW_const(void) const       { return m_lut->lock_dW_const(); }
    auto lock_mean(void)                 { return m_batch_norm->lock_mean(); }
    auto lock_mean_const(void) const     { return m_batch_norm->lock_mean_const(); }
    auto lock_var(void)                  { return m_batch_norm->lock_var(); }
    auto lock_var_const(void) const      { return m_batch_norm->lock_var_const(); }
    auto lock_tmp_mean_const(void) const { return m_batch_norm->lock_tmp_mean_const(); }
    auto lock_tmp_rstd_const(void) const { return m_batch_norm->lock_tmp_rstd_const(); }

    Variables GetParameters(void) override { return m_lut->GetParameters(); }
    Variables GetGradients(void) override  { return m_lut->GetGradients(); }

    indices_t SetInputShape(indices_t shape) override
    {
        shape = m_lut->SetInputShape(shape);
        if (m_bn_enable)  { shape = m_batch_norm->SetInputShape(shape); }
        if (m_act_enable) { shape = m_activation->SetInputShape(shape); }
        return shape;
    }
    indices_t GetInputShape(void) const override  { return m_lut->GetInputShape(); }
    indices_t GetOutputShape(void) const override { return m_lut->GetOutputShape(); }

    index_t GetNodeConnectionSize(index_t node) const { return m_lut->GetNodeConnectionSize(node); }
    void    SetNodeConnectionIndex(index_t node, index_t input_index, index_t input_node) { m_lut->SetNodeConnectionIndex(node, input_index, input_node); }
    index_t GetNodeConnectionIndex(index_t node, index_t input_index) const { return m_lut->GetNodeConnectionIndex(node, input_index); }

    std::vector<double> ForwardNode(index_t node, std::vector<double> x_vec) const override
    {
        BB_ASSERT(GetNodeConnectionSize(node) == (index_t)x_vec.size());
        x_vec = m_lut->ForwardNode(node, x_vec);
        if (m_bn_enable)  { x_vec = m_batch_norm->ForwardNode(node, x_vec); }
        if (m_act_enable) { x_vec = m_activation->ForwardNode(node, x_vec); }
        return x_vec;
    }

    FrameBuffer Forward(FrameBuffer x_buf, bool train = true) override
    {
        bool const saving = m_memory_saving && train && (m_bn_enable || m_act_enable);
        if (saving) { this->PushFrameBuffer(x_buf); }
        x_buf = m_lut->Forward(x_buf, train);
        if (saving) { m_lut->Clear(); }
        if (m_bn_enable) {
            x_buf = m_batch_norm->Forward(x_buf, train);
            if (saving) { m_batch_norm->Clear(); }
        }
        if (m_act_enable) {
            x_buf = m_activation->Forward(x_buf, train);
            if (saving) { m_activation->Clear(); }
        }
        return x_buf;
    }

    FrameBuffer Backward(FrameBuffer dy_buf) override
    {
        if (dy_buf.Empty()) { return dy_buf; }
        if (m_memory_saving && (m_bn_enable || m_act_enable)) {
            FrameBuffer x_buf = this->PopFrameBuffer();
            x_buf = m_lut->ReForward(x_buf);
            if (m_bn_enable)  { x_buf = m_batch_norm->ReForward(x_buf); }
            if (m_act_enable) { m_activation->ReForward(x_buf); }
        }
        if (m_act_enable) { dy_buf = m_activation->Backward(dy_buf); }
        if (m_bn_enable)  { dy_buf = m_batch_norm->Backward(dy_buf); }
        return m_lut->Backward(dy_buf);
    }
};

}  // namespace bb

// BinaryModulation: a binary network between its two converters, RealToBinary -> layer -> BinaryToReal, with one modulation
// size for training and one for inference; the converters are re-sized when a forward pass changes from one to the other
// (reference API: include/bb/BinaryModulation.h:22-473: Create(layer, train_modulation_size, inference_modulation_size,
// depth_modulation_size), GetLayer, Forward, Backward, command "binary" (fp32 activations only)).  Out of binary mode the
// layer runs on the unconverted input.
// Serialized as  version 1 | Model part | binary_mode | training | modulation size | the two converter set-ups |
// RealToBinary object | BinaryToReal object | has layer | layer object  (reference :370-420); an empty layer slot that is
// loaded is rebuilt from the type name in the stream (bb/ObjectLoader.h).
#pragma once

#include "bb/RealToBinary.h"
#include "bb/BinaryToReal.h"

namespace bb {

template <typename BinType = float, typename RealType = float>
class BinaryModulation : public Model {
    using R2B = RealToBinary<BinType, RealType>;
    using B2R = BinaryToReal<BinType, RealType>;

    bool    m_binary_mode = true;
    bool    m_training = true;
    index_t m_modulation_size = 1;
    typename R2B::create_t m_training_create, m_inference_create;
    std::shared_ptr<R2B>   m_real2bin;
    std::shared_ptr<Model> m_layer;
    std::shared_ptr<B2R>   m_bin2real;

public:
    struct create_t {
        std::shared_ptr<Model> layer;
        indices_t output_shape;
        index_t   depth_modulation_size = 1;
        index_t   training_modulation_size = 1;
        std::shared_ptr<Object> training_value_generator;       // must stay empty, see bb/RealToBinary.h
        bool      training_framewise = true;
        RealType  training_input_range_lo = (RealType)0.0, training_input_range_hi = (RealType)1.0;
        index_t   inference_modulation_size = 1;
        std::shared_ptr<Object> inference_value_generator;
        bool      inference_framewise = true;
        RealType  inference_input_range_lo = (RealType)0.0, inference_input_range_hi = (RealType)1.0;
    };

protected:
    explicit BinaryModulation(create_t const &create)
    {
        m_training_create.depth_modulation_size = create.depth_modulation_size;
        m_training_create.frame_modulation_size = create.training_modulation_size;
        m_training_create.value_generator       = create.training_value_generator;
        m_training_create.framewise             = create.training_framewise;
        m_training_create.input_range_lo        = create.training_input_range_lo;
        m_training_create.input_range_hi        = create.training_input_range_hi;
        m_inference_create.depth_modulation_size = create.depth_modulation_size;
        m_inference_create.frame_modulation_size = create.inference_modulation_size;
        m_inference_create.value_generator       = create.inference_value_generator;
        m_inference_create.framewise             = create.inference_framewise;
        m_inference_create.input_range_lo        = create.inference_input_range_lo;
        m_inference_create.input_range_hi        = create.inference_input_range_hi;
        if (create.inference_value_generator) { throw Exception("BinaryModulation: value generators are not supported"); }
        m_modulation_size = create.training_modulation_size;
        m_real2bin = R2B::Create(m_training_create);
        m_layer    = create.layer;
        m_bin2real = B2R::Create(m_modulation_size, create.output_shape);
    }

    void CommandProc(std::vector<std::string> args) override
    {
        Model::CommandProc(args);
        if (DataType<BinType>::type != BB_TYPE_BIT && args.size() == 2 && args[0] == "binary") { m_binary_mode = EvalBool(args[1]); }
    }

    void DumpObjectData(std::ostream &os) const override
    {
        SaveValue(os, (std::int64_t)1);
        Model::DumpObjectData(os);
        SaveValue(os, m_binary_mode);
        SaveValue(os, m_training);
        SaveValue(os, (std::int64_t)m_modulation_size);
        m_training_create.ObjectDump(os);
        m_inference_create.ObjectDump(os);
        m_real2bin->DumpObject(os);
        m_bin2real->DumpObject(os);
        SaveValue(os, (bool)m_layer);
        if (m_layer) { m_layer->DumpObject(os); }
    }

    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = -1, size = -1;
        bool has_layer = false;
        LoadValue(is, ver);
        BB_ASSERT(ver == 1);
        Model::LoadObjectData(is);
        LoadValue(is, m_binary_mode);
        LoadValue(is, m_training);
        LoadValue(is, size);
        BB_ASSERT(is.good() && size > 0);
        m_modulation_size = (index_t)size;
        m_training_create.ObjectLoad(is);
        m_inference_create.ObjectLoad(is);
        m_real2bin->LoadObject(is);
        m_bin2real->LoadObject(is);
        LoadValue(is, has_layer);
        BB_ASSERT(is.good());
        if (has_layer) {
            if (m_layer) { m_layer->LoadObject(is); }
            else {
                m_layer = std::dynamic_pointer_cast<Model>(Object_Load(is));
                if (!m_layer) { throw Exception("BinaryModulation: the stream holds a layer of a type that is not known here"); }
            }
        }
    }

public:
    static std::string ModelName(void)  { return "BinaryModulation"; }
    static std::string ObjectName(void) { return ModelName() + "_" + DataType<BinType>::Name() + "_" + DataType<RealType>::Name(); }
    std::string GetModelName(void) const override  { return ModelName(); }
    std::string GetObjectName(void) const override { return ObjectName(); }

    static std::shared_ptr<BinaryModulation> Create(create_t const &create) { return std::shared_ptr<BinaryModulation>(new BinaryModulation(create)); }
    static std::shared_ptr<BinaryModulation> Create(std::shared_ptr<Model> layer, index_t train_modulation_size, index_t inference_modulation_size = 0,
                                                    index_t depth_modulation_size = 1)
    {
        BB_ASSERT(train_modulation_size > 0);
        create_t c;
        c.layer = layer;
        c.training_modulation_size  = train_modulation_size;
        c.inference_modulation_size = inference_modulation_size > 0 ? inference_modulation_size : train_modulation_size;
        c.depth_modulation_size     = depth_modulation_size;
        return Create(c);
    }
    static std::shared_ptr<BinaryModulation> Create(void) { return Create(create_t()); }

    std::shared_ptr<Model> GetLayer(void) { return m_layer; }

    void SendCommand(std::string command, std::string send_to = "all") override
    {
        Model::SendCommand(command, send_to);
        m_real2bin->SendCommand(command, send_to);
        if (m_layer) { m_layer->SendCommand(command, send_to); }
        m_bin2real->SendCommand(command, send_to);
    }

    Variables GetParameters(void) override { return m_layer ? m_layer->GetParameters() : Variables(); }
    Variables GetGradients(void) override  { return m_layer ? m_layer->GetGradients() : Variables(); }

    indices_t SetInputShape(indices_t shape) override
    {
        BB_ASSERT(m_layer);
        if (shape == this->GetInputShape()) { return this->GetOutputShape(); }
        shape = m_real2bin->SetInputShape(shape);
        shape = m_layer->SetInputShape(shape);
        return m_bin2real->SetInputShape(shape);
    }
    indices_t GetInputShape(void) const override  { return m_real2bin->GetInputShape(); }
    indices_t GetOutputShape(void) const override { return m_bin2real->GetOutputShape(); }

    FrameBuffer Forward(FrameBuffer x_buf, bool train = true) override
    {
        BB_ASSERT(m_layer);
        if (!m_binary_mode) { return m_layer->Forward(x_buf, train); }
        if (train != m_training) {
            m_training = train;
            m_modulation_size = train ? m_training_create.frame_modulation_size : m_inference_create.frame_modulation_size;
            m_real2bin->SetModulationSize(m_modulation_size);
            m_bin2real->SetFrameIntegrationSize(m_modulation_size);
        }
        x_buf = m_real2bin->Forward(x_buf, train);
        x_buf = m_layer->Forward(x_buf, train);
        return m_bin2real->Forward(x_buf, train);
    }

    FrameBuffer Backward(FrameBuffer dy_buf) override
    {
        BB_ASSERT(m_layer);
        if (!m_binary_mode) { return m_layer->Backward(dy_buf); }
        dy_buf = m_bin2real->Backward(dy_buf);
        dy_buf = m_layer->Backward(dy_buf);
        return m_real2bin->Backward(dy_buf);
    }
};

}  // namespace bb

#include "bb/ObjectLoader.h"

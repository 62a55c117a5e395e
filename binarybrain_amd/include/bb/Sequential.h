// A list of layers run one after the other (reference API: include/bb/Sequential.h:24-330).  Forward walks the list,
// Backward walks it in reverse; shapes, commands, parameter and gradient lists are handed through to the layers.
// Serialized as  version 2 | Model part | int64 layer count | the layers as objects  (reference :239-288); an empty
// list that is loaded rebuilds its layers from the type names in the stream (bb/ObjectLoader.h).
#pragma once

#include "bb/Model.h"

namespace bb {

class Sequential : public Model {
    std::vector<std::shared_ptr<Model>> m_layers;

protected:
    Sequential() {}

    void DumpObjectData(std::ostream &os) const override
    {
        SaveValue(os, (std::int64_t)2);
        Model::DumpObjectData(os);
        SaveValue(os, (std::int64_t)m_layers.size());
        for (auto const &layer : m_layers) { layer->DumpObject(os); }
    }

    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = -1;
        LoadValue(is, ver);
        BB_ASSERT(ver == 1 || ver == 2);
        if (ver == 2) { Model::LoadObjectData(is); }
        std::int64_t count = -1;
        LoadValue(is, count);
        BB_ASSERT(is.good() && count >= 0 && count < (1 << 20));
        if (m_layers.empty()) {
            for (std::int64_t i = 0; i < count; ++i) {
                auto layer = std::dynamic_pointer_cast<Model>(Object_Load(is));
                if (!layer) { throw Exception("Sequential: the stream holds a layer of a type that is not known here"); }
                m_layers.push_back(layer);
            }
            return;
        }
        BB_ASSERT(count == (std::int64_t)m_layers.size());
        for (auto &layer : m_layers) { layer->LoadObject(is); }
    }

public:
    static std::string ModelName(void)  { return "Sequential"; }
    static std::string ObjectName(void) { return ModelName(); }
    std::string GetModelName(void) const override { return ModelName(); }

    static std::shared_ptr<Sequential> Create(void) { return std::shared_ptr<Sequential>(new Sequential()); }

    void Add(std::shared_ptr<Model> layer) { BB_ASSERT(layer); m_layers.push_back(layer); }
    int  GetSize(void) const { return (int)m_layers.size(); }
    std::shared_ptr<Model> Get(int index) const
    {
        BB_ASSERT(index >= 0 && index < (int)m_layers.size());
        return m_layers[(std::size_t)index];
    }

    void SendCommand(std::string command, std::string send_to = "all") override
    {
        Model::SendCommand(command, send_to);
        for (auto &layer : m_layers) { layer->SendCommand(command, send_to); }
    }

    Variables GetParameters(void) override
    {
        Variables v;
        for (auto &layer : m_layers) { v.PushBack(layer->GetParameters()); }
        return v;
    }
    Variables GetGradients(void) override
    {
        Variables v;
        for (auto &layer : m_layers) { v.PushBack(layer->GetGradients()); }
        return v;
    }

    indices_t SetInputShape(indices_t shape) override
    {
        for (auto &layer : m_layers) { shape = layer->SetInputShape(shape); }
        return shape;
    }
    indices_t GetInputShape(void) const override  { return m_layers.empty() ? indices_t() : m_layers.front()->GetInputShape(); }
    indices_t GetOutputShape(void) const override { return m_layers.empty() ? indices_t() : m_layers.back()->GetOutputShape(); }

    FrameBuffer Forward(FrameBuffer x_buf, bool train = true) override
    {
        for (auto &layer : m_layers) { x_buf = layer->Forward(x_buf, train); }
        return x_buf;
    }
    FrameBuffer Backward(FrameBuffer dy_buf) override
    {
        for (auto it = m_layers.rbegin(); it != m_layers.rend(); ++it) { dy_buf = (*it)->Backward(dy_buf); }
        return dy_buf;
    }
};

}  // namespace bb

#include "bb/ObjectLoader.h"

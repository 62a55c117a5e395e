// Base class of the layers (reference API: include/bb/Model.h:30-400): string commands, input/output shape,
// Forward/Backward on FrameBuffers, parameter and gradient lists, and a stack that keeps forward inputs for backward.
#pragma once

#include <stack>

#include "bb/Core.h"
#include "bb/FrameBuffer.h"
#include "bb/Tensor.h"

namespace bb {

class Model : public Object {
protected:
    std::string             m_name;
    bool                    m_parameter_lock = false;
    std::stack<FrameBuffer> m_bufs;

    // "key value" commands addressed to this layer; derived classes extend it
    virtual void CommandProc(std::vector<std::string> args)
    {
        if (args.size() == 2 && args[0] == "parameter_lock") { m_parameter_lock = EvalBool(args[1]); }
    }

    void        PushFrameBuffer(FrameBuffer buf) { m_bufs.push(buf); }
    FrameBuffer PopFrameBuffer(void)
    {
        BB_ASSERT(!m_bufs.empty());
        FrameBuffer buf = m_bufs.top();
        m_bufs.pop();
        return buf;
    }

    // version 1 | int64 length of the name | name (reference: include/bb/Model.h:392-426; a version 0 record carries no name)
    void DumpObjectData(std::ostream &os) const override
    {
        SaveValue(os, (std::int64_t)1);
        SaveValue(os, (std::int64_t)m_name.size());
        os.write(m_name.data(), (std::streamsize)m_name.size());
    }
    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = -1;
        LoadValue(is, ver);
        BB_ASSERT(ver == 0 || ver == 1);
        if (ver == 1) {
            std::int64_t size = -1;
            LoadValue(is, size);
            BB_ASSERT(is.good() && size >= 0 && size < (1ll << 20));
            std::string name((std::size_t)size, '\0');
            if (size > 0) { is.read(&name[0], (std::streamsize)size); }
            if (m_name.empty()) { m_name = name; }          // a name given before loading is kept
        }
    }

public:
    virtual ~Model() {}

    virtual std::string GetModelName(void) const = 0;
    // serialized type name; layers with element types append them (e.g. "StochasticLut6_fp32_fp32")
    std::string GetObjectName(void) const override { return GetModelName(); }
    virtual void        SetName(std::string const &name) { m_name = name; }
    virtual std::string GetName(void) const { return m_name.empty() ? GetModelName() : m_name; }

    virtual void SendCommand(std::string command, std::string send_to = "all")
    {
        if (send_to == "all" || send_to == GetModelName() || send_to == GetName()) { CommandProc(SplitString(command)); }
    }

    virtual indices_t SetInputShape(indices_t shape) = 0;
    virtual indices_t GetInputShape(void) const = 0;
    virtual indices_t GetOutputShape(void) const = 0;
    index_t GetInputNodeSize(void) const  { return CalcShapeSize(GetInputShape()); }
    index_t GetOutputNodeSize(void) const { return CalcShapeSize(GetOutputShape()); }

    virtual Variables GetParameters(void) { return Variables(); }
    virtual Variables GetGradients(void)  { return Variables(); }

    virtual FrameBuffer Forward(FrameBuffer x_buf, bool train = true) = 0;
    virtual FrameBuffer Backward(FrameBuffer dy_buf) = 0;
    // the training pass again on the same batch, with whatever the first pass fixed (batch statistics) kept
    // (reference: include/bb/Model.h:312-315)
    virtual FrameBuffer ReForward(FrameBuffer x_buf) { return Forward(x_buf, true); }

    // drops what a training forward pass kept for the backward pass (reference: include/bb/Model.h:362-367); used by layers
    // that recompute their intermediate results instead of keeping them
    virtual void Clear(void) { while (!m_bufs.empty()) { m_bufs.pop(); } }

    // value of one output node for one vector of input values (used to tabulate a trained layer)
    virtual std::vector<double> ForwardNode(index_t, std::vector<double> input_value) const { return input_value; }
};

}  // namespace bb

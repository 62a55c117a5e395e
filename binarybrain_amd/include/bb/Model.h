// Base class of the layers (reference API: include/bb/Model.h:30-400): string commands, input/output shape,
// Forward/Backward on FrameBuffers, parameter and gradient lists, and a stack that keeps forward inputs for backward.
#pragma once

#include <stack>

#include "bb/Core.h"
#include "bb/FrameBuffer.h"
#include "bb/Tensor.h"

namespace bb {

class Model {
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

public:
    virtual ~Model() {}

    virtual std::string GetModelName(void) const = 0;
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

    // value of one output node for one vector of input values (used to tabulate a trained layer)
    virtual std::vector<double> ForwardNode(index_t, std::vector<double> input_value) const { return input_value; }
};

}  // namespace bb

// Batch normalisation of probabilities: every node is normalised with the statistics of its batch and mapped by one scalar
// gamma and beta shared by the whole layer; the layer has no trained parameters (reference API:
// include/bb/StochasticBatchNormalization.h:38-860).  DifferentiableLutN computes the same inside its own kernels; this class
// is the separate layer for networks that are put together from StochasticLutN, a normalisation and an activation.
// Inference takes the running statistics, y = ((x - running_mean) / (sqrt(running_var) + 1e-7)) * gamma + beta, as the
// reference's ForwardNode (:319-341) and its device kernel do.
// Serialized as  version 1 | [version 1 | Model part | shape] | host_only, host_simd | gamma, beta, momentum |
// running mean | running variance (both as typed tensor objects)  (reference :143-183, include/bb/Activation.h:79-109).
#pragma once

#include <cstdlib>

#include "bb/Model.h"

namespace bb {

template <typename T = float>
class StochasticBatchNormalization : public Model {
    static_assert(std::is_same<T, float>::value, "the device path is fp32");

    bool      m_host_only = false;
    bool      m_host_simd = false;      // carried through serialization only
    indices_t m_shape;
    T         m_gamma = (T)0.2, m_beta = (T)0.5, m_momentum = (T)0.9;
    Tensor_<T> m_mean, m_rstd;          // batch statistics of the last training pass
    Tensor_<T> m_running_mean, m_running_var;

public:
    struct create_t {
        T momentum = (T)0.9;
        T gamma    = (T)0.2;
        T beta     = (T)0.5;
    };

protected:
    explicit StochasticBatchNormalization(create_t const &create)
        : m_gamma(create.gamma), m_beta(create.beta), m_momentum(create.momentum) {}

    void CommandProc(std::vector<std::string> args) override
    {
        Model::CommandProc(args);
        if (args.size() == 2 && args[0] == "host_only") { m_host_only = EvalBool(args[1]); }
        if (args.size() == 2 && args[0] == "host_simd") { m_host_simd = EvalBool(args[1]); }
        if (args.size() == 2 && args[0] == "set_gamma") { m_gamma = (T)std::atof(args[1].c_str()); }
        if (args.size() == 2 && args[0] == "set_beta")  { m_beta  = (T)std::atof(args[1].c_str()); }
    }

    void DumpObjectData(std::ostream &os) const override
    {
        SaveValue(os, (std::int64_t)1);
        SaveValue(os, (std::int64_t)1);             // the activation part: version, Model part, shape
        Model::DumpObjectData(os);
        SaveIndices(os, m_shape);
        SaveValue(os, m_host_only);
        SaveValue(os, m_host_simd);
        SaveValue(os, m_gamma);
        SaveValue(os, m_beta);
        SaveValue(os, m_momentum);
        m_running_mean.DumpObject(os);
        m_running_var.DumpObject(os);
    }

    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = -1, act_ver = -1;
        LoadValue(is, ver);
        LoadValue(is, act_ver);
        BB_ASSERT(ver == 1 && act_ver == 1);
        Model::LoadObjectData(is);
        m_shape = LoadIndices(is);
        LoadValue(is, m_host_only);
        LoadValue(is, m_host_simd);
        LoadValue(is, m_gamma);
        LoadValue(is, m_beta);
        LoadValue(is, m_momentum);
        m_running_mean.LoadObject(is);
        m_running_var.LoadObject(is);
        index_t const nodes = CalcShapeSize(m_shape);
        BB_ASSERT(is.good() && m_running_mean.GetSize() == nodes && m_running_var.GetSize() == nodes);
        m_mean.Resize(m_shape);
        m_rstd.Resize(m_shape);
    }

    void RequireDevice(FrameBuffer const &buf) const
    {
        BB_ASSERT(buf.GetType() == BB_TYPE_FP32);
        if (m_host_only || !buf.IsDeviceAvailable()) { throw std::runtime_error("StochasticBatchNormalization: no host path in this build"); }
    }

public:
    static std::string ModelName(void)  { return "StochasticBatchNormalization"; }
    static std::string ObjectName(void) { return ModelName() + "_" + DataType<T>::Name(); }
    std::string GetModelName(void) const override  { return ModelName(); }
    std::string GetObjectName(void) const override { return ObjectName(); }

    static std::shared_ptr<StochasticBatchNormalization> Create(create_t const &create)
    {
        return std::shared_ptr<StochasticBatchNormalization>(new StochasticBatchNormalization(create));
    }
    static std::shared_ptr<StochasticBatchNormalization> Create(T momentum = (T)0.9, T gamma = (T)0.2, T beta = (T)0.5)
    {
        create_t c;
        c.momentum = momentum; c.gamma = gamma; c.beta = beta;
        return Create(c);
    }

    T GetGamma(void) const    { return m_gamma; }
    T GetBeta(void) const     { return m_beta; }
    T GetMomentum(void) const { return m_momentum; }

    auto lock_mean(void)                 { return m_running_mean.Lock(); }
    auto lock_mean_const(void) const     { return m_running_mean.LockConst(); }
    auto lock_var(void)                  { return m_running_var.Lock(); }
    auto lock_var_const(void) const      { return m_running_var.LockConst(); }
    auto lock_tmp_mean_const(void) const { return m_mean.LockConst(); }
    auto lock_tmp_rstd_const(void) const { return m_rstd.LockConst(); }

    // reference :268-287: a repeated shape changes nothing; a new one starts the running statistics at mean 0, variance 1
    indices_t SetInputShape(indices_t shape) override
    {
        if (shape == m_shape) { return m_shape; }
        m_shape = shape;
        m_mean.Resize(shape);
        m_rstd.Resize(shape);
        m_running_mean.Resize(shape); m_running_mean = (T)0.0;
        m_running_var.Resize(shape);  m_running_var  = (T)1.0;
        return m_shape;
    }
    indices_t GetInputShape(void) const override  { return m_shape; }
    indices_t GetOutputShape(void) const override { return m_shape; }

    // y = gain * x + offset at inference (reference :307-317)
    T GetNormalizeGain(index_t node) const
    {
        auto var = m_running_var.LockConst();
        return m_gamma / ((T)std::sqrt(var[node]) + (T)1.0e-7);
    }
    T GetNormalizeOffset(index_t node) const
    {
        auto mean = m_running_mean.LockConst();
        auto var  = m_running_var.LockConst();
        return m_beta - (m_gamma * mean[node] / ((T)std::sqrt(var[node]) + (T)1.0e-7));
    }

    std::vector<double> ForwardNode(index_t node, std::vector<double> x_vec) const override
    {
        BB_ASSERT(node >= 0 && node < CalcShapeSize(m_shape));
        auto mean = m_running_mean.LockConst();
        auto var  = m_running_var.LockConst();
        std::vector<double> y_vec(x_vec.size());
        for (std::size_t i = 0; i < x_vec.size(); ++i) {
            T x = (T)x_vec[i];
            x -= mean[node];
            x /= (T)std::sqrt(var[node]) + (T)1.0e-7;
            x  = x * m_gamma + m_beta;
            y_vec[i] = (double)x;
        }
        return y_vec;
    }

    FrameBuffer Forward(FrameBuffer x_buf, bool train = true) override
    {
        RequireDevice(x_buf);
        if (x_buf.GetShape() != m_shape) { SetInputShape(x_buf.GetShape()); }
        FrameBuffer y_buf(x_buf.GetFrameSize(), x_buf.GetShape(), x_buf.GetType());
        if (train) { PushFrameBuffer(x_buf); }
        auto px = x_buf.LockDeviceMemoryConst();
        auto py = y_buf.LockDeviceMemory(true);
        int const nodes = (int)x_buf.GetNodeSize(), frames = (int)x_buf.GetFrameSize(), stride = (int)(x_buf.GetFrameStride() / 4);
        if (train) {
            auto pm  = m_mean.LockDeviceMemory(true);
            auto pr  = m_rstd.LockDeviceMemory(true);
            auto prm = m_running_mean.LockDeviceMemory();
            auto prv = m_running_var.LockDeviceMemory();
            CheckDevice(bbhip_fp32_StochasticBatchNormalization_ForwardTraining((float const *)px.GetAddr(), (float *)py.GetAddr(),
                    (float *)pm.GetAddr(), (float *)pr.GetAddr(), (float *)prm.GetAddr(), (float *)prv.GetAddr(), (float)m_gamma, (float)m_beta,
                    (float)m_momentum, nodes, frames, stride, nullptr), "bbhip_fp32_StochasticBatchNormalization_ForwardTraining");
        }
        else {
            auto prm = m_running_mean.LockDeviceMemoryConst();
            auto prv = m_running_var.LockDeviceMemoryConst();
            CheckDevice(bbhip_fp32_StochasticBatchNormalization_ForwardInference((float const *)px.GetAddr(), (float *)py.GetAddr(),
                    (float const *)prm.GetAddr(), (float const *)prv.GetAddr(), (float)m_gamma, (float)m_beta, nodes, frames, stride, nullptr),
                    "bbhip_fp32_StochasticBatchNormalization_ForwardInference");
        }
        return y_buf;
    }

    // the output again from the statistics that the training pass stored (reference :621-680)
    FrameBuffer ReForward(FrameBuffer x_buf) override
    {
        RequireDevice(x_buf);
        BB_ASSERT(x_buf.GetShape() == m_shape);
        FrameBuffer y_buf(x_buf.GetFrameSize(), x_buf.GetShape(), x_buf.GetType());
        PushFrameBuffer(x_buf);
        auto px = x_buf.LockDeviceMemoryConst();
        auto py = y_buf.LockDeviceMemory(true);
        auto pm = m_mean.LockDeviceMemoryConst();
        auto pr = m_rstd.LockDeviceMemoryConst();
        CheckDevice(bbhip_fp32_StochasticBatchNormalization_ReForward((float const *)px.GetAddr(), (float *)py.GetAddr(),
                (float const *)pm.GetAddr(), (float const *)pr.GetAddr(), (float)m_gamma, (float)m_beta, (int)x_buf.GetNodeSize(),
                (int)x_buf.GetFrameSize(), (int)(x_buf.GetFrameStride() / 4), nullptr), "bbhip_fp32_StochasticBatchNormalization_ReForward");
        return y_buf;
    }

    FrameBuffer Backward(FrameBuffer dy_buf) override
    {
        if (dy_buf.Empty()) { return FrameBuffer(); }
        RequireDevice(dy_buf);
        FrameBuffer x_buf = PopFrameBuffer();
        BB_ASSERT(x_buf.GetFrameSize() == dy_buf.GetFrameSize() && x_buf.GetNodeSize() == dy_buf.GetNodeSize());
        FrameBuffer dx_buf(dy_buf.GetFrameSize(), dy_buf.GetShape(), dy_buf.GetType());
        auto px  = x_buf.LockDeviceMemoryConst();
        auto pdy = dy_buf.LockDeviceMemoryConst();
        auto pdx = dx_buf.LockDeviceMemory(true);
        auto pm  = m_mean.LockDeviceMemoryConst();
        auto pr  = m_rstd.LockDeviceMemoryConst();
        CheckDevice(bbhip_fp32_StochasticBatchNormalization_Backward((float const *)px.GetAddr(), (float const *)pdy.GetAddr(), (float *)pdx.GetAddr(),
                (float const *)pm.GetAddr(), (float const *)pr.GetAddr(), (float)m_gamma, 1.0f / (float)dy_buf.GetFrameSize(), (int)dy_buf.GetNodeSize(),
                (int)dy_buf.GetFrameSize(), (int)(dy_buf.GetFrameStride() / 4), (int)(x_buf.GetFrameStride() / 4), nullptr),
                "bbhip_fp32_StochasticBatchNormalization_Backward");
        return dx_buf;
    }
};

}  // namespace bb

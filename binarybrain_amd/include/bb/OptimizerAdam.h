// Adam optimizer over a list of parameter / gradient tensors (reference API: include/bb/OptimizerAdam.h:20-184,
// include/bb/Optimizer.h:19-40).  The update of all tensors is one device call (bbhip_fp32_OptimizerAdam); the
// bias-correction products beta1^t, beta2^t are kept on the host in fp32 exactly as the reference keeps them.
#pragma once

#include <cmath>

#include "bb/Core.h"
#include "bb/Tensor.h"

namespace bb {

class Optimizer {
public:
    virtual ~Optimizer() {}
    virtual std::string GetOptimizerName(void) const = 0;
    virtual void SetVariables(Variables params, Variables grads) = 0;
    virtual void ZeroGrad(void) = 0;
    virtual void Step(void) = 0;
    virtual void Update(void) { Step(); ZeroGrad(); }
    virtual void SetLearningRate(double learning_rate) = 0;
};


template <typename T = float>
class OptimizerAdam : public Optimizer {
    static_assert(std::is_same<T, float>::value, "the device step is fp32");

    T         m_learning_rate, m_beta1, m_beta2;
    T         m_b1, m_b2;                       // beta1^t, beta2^t
    Variables m_params, m_grads;
    std::vector<std::shared_ptr<Tensor>> m_m, m_v;
    // device tables of the call: element counts and the four pointer lists
    std::shared_ptr<Memory> m_size_table, m_param_table, m_grad_table, m_m_table, m_v_table;

    OptimizerAdam(T learning_rate, T beta1, T beta2)
        : m_learning_rate(learning_rate), m_beta1(beta1), m_beta2(beta2), m_b1(beta1), m_b2(beta2) {}

    static std::shared_ptr<Memory> pointer_table(std::vector<void *> const &ptrs)
    {
        auto mem = Memory::Create(ptrs.size() * sizeof(void *));
        std::memcpy(mem->Lock(true), ptrs.data(), ptrs.size() * sizeof(void *));
        return mem;
    }

public:
    struct create_t {
        T learning_rate = (T)0.001;
        T beta1         = (T)0.9;
        T beta2         = (T)0.999;
    };

    static std::shared_ptr<OptimizerAdam> Create(create_t const &create)
    {
        return std::shared_ptr<OptimizerAdam>(new OptimizerAdam(create.learning_rate, create.beta1, create.beta2));
    }
    static std::shared_ptr<OptimizerAdam> Create(T learning_rate = (T)0.001, T beta1 = (T)0.9, T beta2 = (T)0.999)
    {
        return std::shared_ptr<OptimizerAdam>(new OptimizerAdam(learning_rate, beta1, beta2));
    }

    std::string GetOptimizerName(void) const override { return "OptimizerAdam"; }

    void SetLearningRate(double learning_rate) override { m_learning_rate = (T)learning_rate; }

    // Binds the parameter list; the moment estimates start at zero (reference: OptimizerAdam.h:120-130).
    // The tensors must keep their storage (no Resize) while the optimizer is in use.
    void SetVariables(Variables params, Variables grads) override
    {
        BB_ASSERT(params.GetSize() == grads.GetSize());
        m_params = params;
        m_grads  = grads;
        m_m.clear(); m_v.clear();
        index_t const n = params.GetSize();
        std::vector<std::int32_t> sizes;
        std::vector<void *> pp, gp, mp, vp;
        for (index_t i = 0; i < n; ++i) {
            BB_ASSERT(params[i].GetType() == BB_TYPE_FP32 && grads[i].GetType() == BB_TYPE_FP32);
            BB_ASSERT(params[i].GetSize() == grads[i].GetSize() && params[i].GetSize() <= 0x7fffffff);
            if (!params[i].IsDeviceAvailable()) { throw std::runtime_error("OptimizerAdam: no device path for host-only tensors"); }
            auto m = std::make_shared<Tensor>(params[i].GetShape(), BB_TYPE_FP32);
            auto v = std::make_shared<Tensor>(params[i].GetShape(), BB_TYPE_FP32);
            m->FillZero(); v->FillZero();
            m_m.push_back(m); m_v.push_back(v);
            sizes.push_back((std::int32_t)params[i].GetSize());
            pp.push_back(params[i].LockDeviceMemory().GetAddr());
            gp.push_back(grads[i].LockDeviceMemory().GetAddr());
            mp.push_back(m->LockDeviceMemory().GetAddr());
            vp.push_back(v->LockDeviceMemory().GetAddr());
        }
        m_size_table = Memory::Create(sizes.size() * sizeof(std::int32_t));
        if (n > 0) { std::memcpy(m_size_table->Lock(true), sizes.data(), sizes.size() * sizeof(std::int32_t)); }
        m_param_table = pointer_table(pp); m_grad_table = pointer_table(gp);
        m_m_table = pointer_table(mp);     m_v_table = pointer_table(vp);
    }

    void ZeroGrad(void) override { m_grads.FillZero(); }

    void Step(void) override { Apply(false); }

    // Step() followed by ZeroGrad() (reference: Optimizer.h:31-35), as one launch: the update kernel zeroes each gradient
    // element once it has used it.
    void Update(void) override { Apply(true); }

private:
    void Apply(bool zero_grads)
    {
        index_t const n = m_params.GetSize();
        if (n == 0) { return; }
        if (!Manager::IsDeviceAvailable()) { throw std::runtime_error("OptimizerAdam: no device available (there is no host path)"); }
        // make the device copies current (a host-side edit of a parameter or gradient marks them stale)
        for (index_t i = 0; i < n; ++i) {
            m_params[i].LockDeviceMemory();
            if (zero_grads) { m_grads[i].LockDeviceMemory(); } else { m_grads[i].LockDeviceMemoryConst(); }
            m_m[(std::size_t)i]->LockDeviceMemory();
            m_v[(std::size_t)i]->LockDeviceMemory();
        }
        T const lr_t = m_learning_rate * std::sqrt((T)1.0 - m_b2) / ((T)1.0 - m_b1);        // OptimizerAdam.h:171
        auto const entry = zero_grads ? bbhip_fp32_OptimizerAdam_Update : bbhip_fp32_OptimizerAdam;
        CheckDevice(entry((int)n, (int const *)m_size_table->LockDeviceConst(),
                          (float *const *)m_param_table->LockDeviceConst(), (float *const *)m_grad_table->LockDeviceConst(),
                          (float *const *)m_m_table->LockDeviceConst(), (float *const *)m_v_table->LockDeviceConst(),
                          lr_t, m_beta1, m_beta2, nullptr), zero_grads ? "bbhip_fp32_OptimizerAdam_Update" : "bbhip_fp32_OptimizerAdam");
        m_b1 *= m_beta1;
        m_b2 *= m_beta2;
    }
};

}  // namespace bb

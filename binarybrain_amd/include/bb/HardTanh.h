// HardTanh: y = min(max(x, lo), hi), dx = dy inside (lo, hi) and 0 elsewhere.  In binary mode ("binary true"), and always with
// Bit output, it is Binarize with the threshold in the middle of the window (reference API: include/bb/HardTanh.h:21-292).
// Serialized as  version 1 | Binarize part | binary_mode  (reference :262-289).
#pragma once

#include "bb/Binarize.h"

namespace bb {

template <typename BinType = float, typename RealType = float>
class HardTanh : public Binarize<BinType, RealType> {
    using _super = Binarize<BinType, RealType>;
    using _super::m_binary_th;
    using _super::m_hardtanh_min;
    using _super::m_hardtanh_max;

    bool m_binary_mode = false;

public:
    struct create_t {
        RealType hardtanh_min = (RealType)-1.0;
        RealType hardtanh_max = (RealType)+1.0;
    };

protected:
    explicit HardTanh(create_t const &create)
    {
        m_hardtanh_min = create.hardtanh_min;
        m_hardtanh_max = create.hardtanh_max;
        m_binary_th    = (m_hardtanh_min + m_hardtanh_max) / (RealType)2;
    }

    void CommandProc(std::vector<std::string> args) override
    {
        _super::CommandProc(args);
        if (args.size() == 2 && args[0] == "binary") { m_binary_mode = EvalBool(args[1]); }
    }

    void DumpObjectData(std::ostream &os) const override
    {
        SaveValue(os, (std::int64_t)1);
        _super::DumpObjectData(os);
        SaveValue(os, m_binary_mode);
    }

    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = -1;
        LoadValue(is, ver);
        BB_ASSERT(ver == 1);
        _super::LoadObjectData(is);
        LoadValue(is, m_binary_mode);
        BB_ASSERT(is.good());
    }

public:
    static std::string ModelName(void)  { return "HardTanh"; }
    static std::string ObjectName(void) { return ModelName() + "_" + DataType<BinType>::Name() + "_" + DataType<RealType>::Name(); }
    std::string GetModelName(void) const override  { return ModelName(); }
    std::string GetObjectName(void) const override { return ObjectName(); }

    static std::shared_ptr<HardTanh> Create(create_t const &create) { return std::shared_ptr<HardTanh>(new HardTanh(create)); }
    static std::shared_ptr<HardTanh> Create(RealType hardtanh_min = (RealType)-1, RealType hardtanh_max = (RealType)+1)
    {
        create_t c;
        c.hardtanh_min = hardtanh_min; c.hardtanh_max = hardtanh_max;
        return Create(c);
    }

    std::vector<double> ForwardNode(index_t node, std::vector<double> x_vec) const override
    {
        if (m_binary_mode) { return _super::ForwardNode(node, x_vec); }
        for (auto &x : x_vec) {
            if (x <= (double)m_hardtanh_min) { x = (double)m_hardtanh_min; }
            if (x >= (double)m_hardtanh_max) { x = (double)m_hardtanh_max; }
        }
        return x_vec;
    }

    FrameBuffer Forward(FrameBuffer x_buf, bool train = true) override
    {
        if (DataType<BinType>::type == BB_TYPE_BIT || m_binary_mode) { return this->BinarizeForward(x_buf, train); }
        this->RequireDevice(x_buf, "HardTanh::Forward");
        if (x_buf.GetShape() != this->m_shape) { this->SetInputShape(x_buf.GetShape()); }
        if (train) { this->PushFrameBuffer(x_buf); }
        FrameBuffer y_buf(x_buf.GetFrameSize(), x_buf.GetShape(), BB_TYPE_FP32);
        auto x_ptr = x_buf.LockDeviceMemoryConst();
        auto y_ptr = y_buf.LockDeviceMemory(true);
        CheckDevice(bbhip_fp32_HardTanh_Forward((float const *)x_ptr.GetAddr(), (float *)y_ptr.GetAddr(), (float)m_hardtanh_min,
                        (float)m_hardtanh_max, (int)y_buf.GetNodeSize(), (int)y_buf.GetFrameSize(), (int)(y_buf.GetFrameStride() / sizeof(float)),
                        nullptr), "bbhip_fp32_HardTanh_Forward");
        return y_buf;
    }

    FrameBuffer Backward(FrameBuffer dy_buf) override { return this->WindowBackward(dy_buf); }
};

}  // namespace bb

// Binarize: y = x > threshold ? high : low (fp32 output) or the packed bit of x > threshold (Bit output); its backward is the
// straight-through estimator with a window, dx = dy where hardtanh_min < x < hardtanh_max and 0 elsewhere
// (reference API: include/bb/Binarize.h:21-310: Create(binary_th, binary_low, binary_high, hardtanh_min, hardtanh_max),
// Forward, Backward, ForwardNode).  Forward keeps its input for the backward pass when `train` is set.
// Serialized as  version 1 | [version 1 | Model part | shape] | host_only | binary_th | hardtanh_min | hardtanh_max
// (reference :286-308, include/bb/Activation.h:79-104); binary_low and binary_high are not part of the record.
#pragma once

#include "bb/Model.h"

namespace bb {

template <typename BinType = float, typename RealType = float>
class Binarize : public Model {
    static_assert(std::is_same<RealType, float>::value, "inputs and gradients are fp32");
    static_assert(std::is_same<BinType, float>::value || std::is_same<BinType, Bit>::value, "outputs are fp32 or packed bits");

protected:
    bool      m_host_only = false;
    indices_t m_shape;
    RealType  m_binary_th    = (RealType)0;
    RealType  m_binary_low   = (RealType)BB_BINARY_LO;
    RealType  m_binary_high  = (RealType)BB_BINARY_HI;
    RealType  m_hardtanh_min = (RealType)-1.0;
    RealType  m_hardtanh_max = (RealType)+1.0;

public:
    struct create_t {
        RealType binary_th    = (RealType)0;
        double   binary_low   = (double)BB_BINARY_LO;
        double   binary_high  = (double)BB_BINARY_HI;
        RealType hardtanh_min = (RealType)-1.0;
        RealType hardtanh_max = (RealType)+1.0;
    };

protected:
    Binarize() {}
    explicit Binarize(create_t const &create)
        : m_binary_th(create.binary_th), m_binary_low((RealType)create.binary_low), m_binary_high((RealType)create.binary_high),
          m_hardtanh_min(create.hardtanh_min), m_hardtanh_max(create.hardtanh_max) {}

    void CommandProc(std::vector<std::string> args) override
    {
        Model::CommandProc(args);
        if (args.size() == 2 && args[0] == "host_only") { m_host_only = EvalBool(args[1]); }
    }

    void DumpObjectData(std::ostream &os) const override
    {
        SaveValue(os, (std::int64_t)1);
        SaveValue(os, (std::int64_t)1);             // the activation part: version, Model part, shape
        Model::DumpObjectData(os);
        SaveIndices(os, m_shape);
        SaveValue(os, m_host_only);
        SaveValue(os, m_binary_th);
        SaveValue(os, m_hardtanh_min);
        SaveValue(os, m_hardtanh_max);
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
        LoadValue(is, m_binary_th);
        LoadValue(is, m_hardtanh_min);
        LoadValue(is, m_hardtanh_max);
        BB_ASSERT(is.good());
    }

    void RequireDevice(FrameBuffer const &buf, char const *what) const
    {
        BB_ASSERT(buf.GetType() == BB_TYPE_FP32);
        if (m_host_only || !buf.IsDeviceAvailable() || !Manager::IsDeviceAvailable()) {
            throw Exception(std::string(what) + ": host-only execution is not provided by this library (device path only)");
        }
    }

    // the straight-through window, shared with HardTanh
    FrameBuffer WindowBackward(FrameBuffer dy_buf)
    {
        if (dy_buf.Empty()) { return dy_buf; }
        RequireDevice(dy_buf, "Binarize::Backward");
        FrameBuffer x_buf = this->PopFrameBuffer();
        BB_ASSERT(x_buf.GetNodeSize() == dy_buf.GetNodeSize() && x_buf.GetFrameSize() == dy_buf.GetFrameSize());
        FrameBuffer dx_buf(dy_buf.GetFrameSize(), dy_buf.GetShape(), BB_TYPE_FP32);
        auto x_ptr  = x_buf.LockDeviceMemoryConst();
        auto dy_ptr = dy_buf.LockDeviceMemoryConst();
        auto dx_ptr = dx_buf.LockDeviceMemory(true);
        CheckDevice(bbhip_fp32_HardTanh_Backward((float const *)x_ptr.GetAddr(), (float const *)dy_ptr.GetAddr(), (float *)dx_ptr.GetAddr(),
                        (float)m_hardtanh_min, (float)m_hardtanh_max, (int)dx_buf.GetNodeSize(), (int)dx_buf.GetFrameSize(),
                        (int)(dx_buf.GetFrameStride() / sizeof(float)), nullptr), "bbhip_fp32_HardTanh_Backward");
        return dx_buf;
    }

    FrameBuffer BinarizeForward(FrameBuffer x_buf, bool train)
    {
        RequireDevice(x_buf, "Binarize::Forward");
        if (x_buf.GetShape() != m_shape) { SetInputShape(x_buf.GetShape()); }
        if (train) { this->PushFrameBuffer(x_buf); }
        FrameBuffer y_buf(x_buf.GetFrameSize(), x_buf.GetShape(), DataType<BinType>::type);
        auto x_ptr = x_buf.LockDeviceMemoryConst();
        auto y_ptr = y_buf.LockDeviceMemory(true);
        if (DataType<BinType>::type == BB_TYPE_BIT) {
            CheckDevice(bbhip_fp32_bit_Binarize_Forward((float const *)x_ptr.GetAddr(), (int *)y_ptr.GetAddr(), (float)m_binary_th,
                            (int)x_buf.GetNodeSize(), (int)x_buf.GetFrameSize(), (int)(x_buf.GetFrameStride() / sizeof(float)),
                            (int)(y_buf.GetFrameStride() / sizeof(int)), nullptr), "bbhip_fp32_bit_Binarize_Forward");
        }
        else {
            CheckDevice(bbhip_fp32_Binarize_Forward((float const *)x_ptr.GetAddr(), (float *)y_ptr.GetAddr(), (float)m_binary_th,
                            (float)m_binary_low, (float)m_binary_high, (int)y_buf.GetNodeSize(), (int)y_buf.GetFrameSize(),
                            (int)(y_buf.GetFrameStride() / sizeof(float)), nullptr), "bbhip_fp32_Binarize_Forward");
        }
        return y_buf;
    }

public:
    static std::string ModelName(void)  { return "Binarize"; }
    static std::string ObjectName(void) { return ModelName() + "_" + DataType<BinType>::Name() + "_" + DataType<RealType>::Name(); }
    std::string GetModelName(void) const override  { return ModelName(); }
    std::string GetObjectName(void) const override { return ObjectName(); }

    static std::shared_ptr<Binarize> Create(create_t const &create) { return std::shared_ptr<Binarize>(new Binarize(create)); }
    static std::shared_ptr<Binarize> Create(RealType binary_th = (RealType)0, double binary_low = (double)BB_BINARY_LO,
                                            double binary_high = (double)BB_BINARY_HI, RealType hardtanh_min = (RealType)-1.0,
                                            RealType hardtanh_max = (RealType)+1.0)
    {
        create_t c;
        c.binary_th = binary_th; c.binary_low = binary_low; c.binary_high = binary_high; c.hardtanh_min = hardtanh_min; c.hardtanh_max = hardtanh_max;
        return Create(c);
    }

    indices_t SetInputShape(indices_t shape) override { m_shape = shape; return m_shape; }
    indices_t GetInputShape(void) const override  { return m_shape; }
    indices_t GetOutputShape(void) const override { return m_shape; }

    // the layer as a table entry sees it: the window's upper or lower end (reference :125-132)
    std::vector<double> ForwardNode(index_t, std::vector<double> x_vec) const override
    {
        for (auto &x : x_vec) { x = (x > (double)m_binary_th) ? (double)m_hardtanh_max : (double)m_hardtanh_min; }
        return x_vec;
    }

    FrameBuffer Forward(FrameBuffer x_buf, bool train = true) override { return BinarizeForward(x_buf, train); }
    FrameBuffer Backward(FrameBuffer dy_buf) override { return WindowBackward(dy_buf); }
};

}  // namespace bb

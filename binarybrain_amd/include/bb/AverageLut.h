// AverageLut: every output node adds up n wired inputs; with binarize_output it votes (+1 / -1 on sum > 0), on packed bits
// it is the strict majority of the n inputs.  Reference API: include/bb/AverageLut.h:22-458 (Create(n, output_shape,
// connection, binarize, binarize_input, seed); commands binary / binarize_input / binarize_output / host_only; connection
// get/set; GetLutTable = majority of the index bits; wiring policies and serialized form: bb/WiredSelectModel.h).
// Frame work runs in the HIP library only.  Without binarize_output the reference disagrees with itself: its CUDA kernel writes
// sum * (1 / n) (cuda/AverageLut.cu:46-54), its host loop the plain sum (include/bb/AverageLut.h:331-343).  The class follows
// the device path, which is what the reference's class runs where a GPU is present; the command "host_sum true" selects the
// host loop's sum (a run-time choice like host_only: not part of the serialized object).
#pragma once

#include "bb/WiredSelectModel.h"

namespace bb {

template <typename BinType = float, typename RealType = float>
class AverageLut : public WiredSelectModel {
    static_assert(std::is_same<RealType, float>::value, "gradients are fp32");
    static_assert(std::is_same<BinType, float>::value || std::is_same<BinType, Bit>::value, "inputs are fp32 or packed bits");

public:
    struct create_t {
        int           n = 6;
        indices_t     output_shape;
        std::string   connection = "";
        bool          binarize_input = false;
        bool          binarize_output = true;
        std::uint64_t seed = 1;
    };

protected:
    bool m_host_sum = false;

    explicit AverageLut(create_t const &create)
        : WiredSelectModel(create.n, create.output_shape, create.connection, create.binarize_input, create.binarize_output, create.seed) {}

    void CommandProc(std::vector<std::string> args) override
    {
        WiredSelectModel::CommandProc(args);
        if (args.size() == 2 && args[0] == "host_sum") { m_host_sum = EvalBool(args[1]); }
    }

public:
    static std::string ModelName(void)  { return "AverageLut"; }
    static std::string ObjectName(void) { return ModelName() + "_" + DataType<BinType>::Name() + "_" + DataType<RealType>::Name(); }
    std::string GetModelName(void) const override  { return ModelName(); }
    std::string GetObjectName(void) const override { return ObjectName(); }

    static std::shared_ptr<AverageLut> Create(create_t const &create) { return std::shared_ptr<AverageLut>(new AverageLut(create)); }
    static std::shared_ptr<AverageLut> Create(int n, indices_t const &output_shape, std::string connection = "", bool binarize = true,
                                              bool binarize_input = false, std::uint64_t seed = 1)
    {
        create_t c;
        c.n = n; c.output_shape = output_shape; c.connection = connection; c.binarize_input = binarize_input; c.binarize_output = binarize; c.seed = seed;
        return Create(c);
    }
    static std::shared_ptr<AverageLut> Create(int n, index_t output_node_size, std::string connection = "", bool binarize = true,
                                              bool binarize_input = false, std::uint64_t seed = 1)
    {
        return Create(n, indices_t({output_node_size}), connection, binarize, binarize_input, seed);
    }
    static std::shared_ptr<AverageLut> Create(void)
    {
        create_t c;
        c.output_shape = indices_t({1});
        return Create(c);
    }

    FrameBuffer Forward(FrameBuffer x_buf, bool = true) override
    {
        BB_ASSERT(x_buf.GetType() == DataType<BinType>::type);
        if (m_host_only || !Manager::IsDeviceAvailable()) {
            throw Exception("AverageLut::Forward: host-only execution is not provided by this library (device path only)");
        }
        if (x_buf.GetShape() != m_input_shape) { SetInputShape(x_buf.GetShape()); }
        FrameBuffer y_buf(x_buf.GetFrameSize(), m_output_shape, DataType<BinType>::type);
        BB_ASSERT(x_buf.GetFrameStride() == y_buf.GetFrameStride());
        auto x_ptr   = x_buf.LockDeviceMemoryConst();
        auto y_ptr   = y_buf.LockDeviceMemory(true);
        auto idx_ptr = m_input_index.LockDeviceMemoryConst();
        if (DataType<BinType>::type == BB_TYPE_BIT) {
            CheckDevice(bbhip_bit_AverageLut_Forward((int const *)x_ptr.GetAddr(), (int *)y_ptr.GetAddr(), (int const *)idx_ptr.GetAddr(), m_n,
                            (int)y_buf.GetNodeSize(), (int)y_buf.GetFrameSize(), (int)(y_buf.GetFrameStride() / sizeof(int)), nullptr),
                        "bbhip_bit_AverageLut_Forward");
        }
        else {
            auto const entry = m_host_sum ? bbhip_fp32_AverageLut_ForwardSum : bbhip_fp32_AverageLut_Forward;
            CheckDevice(entry((float const *)x_ptr.GetAddr(), (float *)y_ptr.GetAddr(), (int const *)idx_ptr.GetAddr(), m_n,
                            (int)y_buf.GetNodeSize(), (int)y_buf.GetFrameSize(), (int)(y_buf.GetFrameStride() / sizeof(float)),
                            m_binarize_input ? 1 : 0, m_binarize_output ? 1 : 0, nullptr), "bbhip_fp32_AverageLut_Forward");
        }
        return y_buf;
    }

    FrameBuffer Backward(FrameBuffer dy_buf) override
    {
        if (dy_buf.Empty()) { return dy_buf; }
        BB_ASSERT(dy_buf.GetType() == BB_TYPE_FP32);
        if (m_host_only || !Manager::IsDeviceAvailable()) {
            throw Exception("AverageLut::Backward: host-only execution is not provided by this library (device path only)");
        }
        FrameBuffer dx_buf(dy_buf.GetFrameSize(), m_input_shape, BB_TYPE_FP32);
        auto dy_ptr  = dy_buf.LockDeviceMemoryConst();
        auto dx_ptr  = dx_buf.LockDeviceMemory(true);
        auto idx_ptr = m_input_index.LockDeviceMemoryConst();
        CheckDevice(bbhip_fp32_AverageLut_Backward((float const *)dy_ptr.GetAddr(), (float *)dx_ptr.GetAddr(), (int const *)idx_ptr.GetAddr(), m_n,
                        (int)dx_buf.GetNodeSize(), (int)dy_buf.GetNodeSize(), (int)dy_buf.GetFrameSize(),
                        (int)(dy_buf.GetFrameStride() / sizeof(float)), nullptr), "bbhip_fp32_AverageLut_Backward");
        return dx_buf;
    }
};

}  // namespace bb

// Im2Col: every window position of every image becomes a frame of its own, so that the LUT layers of a convolution
// see a plain (filter taps) -> (outputs) problem (reference API: include/bb/ConvolutionIm2Col.h:26-470).
// Input shape {c, h, w}; output shape {c, filter_h, filter_w}; output frames = input frames * oh * ow, frame index
// (input frame, oy, ox) row-major.  FT is float or Bit (packed forward only); the backward type is float.
#pragma once

#include "bb/Model.h"

namespace bb {

#define BB_BORDER_CONSTANT      0
#define BB_BORDER_REFLECT       1
#define BB_BORDER_REFLECT_101   2
#define BB_BORDER_REPLICATE     3
#define BB_BORDER_WRAP          4

template <typename FT = float, typename BT = float>
class ConvolutionIm2Col : public Model {
    static_assert(std::is_same<BT, float>::value, "gradients are fp32");

    bool        m_host_only = false;
    indices_t   m_input_shape, m_output_shape;
    index_t     m_input_frame_size = 1, m_output_frame_size = 1;
    index_t     m_input_c_size = 1, m_input_h_size = 1, m_input_w_size = 1;
    index_t     m_filter_h_size = 1, m_filter_w_size = 1;
    index_t     m_y_stride = 1, m_x_stride = 1, m_y_offset = 0, m_x_offset = 0;
    index_t     m_output_h_size = 1, m_output_w_size = 1;
    std::string m_padding = "valid";
    int         m_border_mode = BB_BORDER_REFLECT_101;
    FT          m_border_value = (FT)0;

    static int BorderConv(std::string const &mode)
    {
        if (mode == "constant")    { return BB_BORDER_CONSTANT; }
        if (mode == "reflect")     { return BB_BORDER_REFLECT; }
        if (mode == "reflect_101") { return BB_BORDER_REFLECT_101; }
        if (mode == "replicate")   { return BB_BORDER_REPLICATE; }
        if (mode == "wrap")        { return BB_BORDER_WRAP; }
        throw std::runtime_error("ConvolutionIm2Col: unknown border mode " + mode);
    }

    void CommandProc(std::vector<std::string> args) override
    {
        Model::CommandProc(args);
        if (args.size() == 2 && args[0] == "host_only") { m_host_only = EvalBool(args[1]); }
    }

public:
    struct create_t {
        index_t     filter_h_size = 1;
        index_t     filter_w_size = 1;
        index_t     x_stride = 1;
        index_t     y_stride = 1;
        std::string padding = "valid";
        std::string border_mode = "reflect_101";
        FT          border_value = (FT)0;
    };

protected:
    explicit ConvolutionIm2Col(create_t const &create)
    {
        m_filter_h_size = create.filter_h_size;
        m_filter_w_size = create.filter_w_size;
        m_x_stride = create.x_stride;
        m_y_stride = create.y_stride;
        m_padding = create.padding;
        m_border_mode = BorderConv(create.border_mode);
        m_border_value = create.border_value;
    }

    // version 1 | Model part | host_only, frame sizes of the last pass, input c/h/w, filter h/w, strides y/x, padding, border mode
    // and value (reference: include/bb/ConvolutionIm2Col.h:492-563); the shapes are rebuilt from them
    void DumpObjectData(std::ostream &os) const override
    {
        SaveValue(os, (std::int64_t)1);
        Model::DumpObjectData(os);
        SaveValue(os, m_host_only);
        SaveValue(os, (std::int64_t)m_input_frame_size);  SaveValue(os, (std::int64_t)m_output_frame_size);
        SaveValue(os, (std::int64_t)m_input_c_size);      SaveValue(os, (std::int64_t)m_input_h_size);  SaveValue(os, (std::int64_t)m_input_w_size);
        SaveValue(os, (std::int64_t)m_filter_h_size);     SaveValue(os, (std::int64_t)m_filter_w_size);
        SaveValue(os, (std::int64_t)m_y_stride);          SaveValue(os, (std::int64_t)m_x_stride);
        SaveValue(os, m_padding);
        SaveValue(os, (std::int32_t)m_border_mode);
        SaveValue(os, m_border_value);
    }
    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = -1;
        LoadValue(is, ver);
        BB_ASSERT(ver == 1);
        Model::LoadObjectData(is);
        auto load_index = [&is](index_t &v) { std::int64_t e = 0; LoadValue(is, e); v = (index_t)e; };
        LoadValue(is, m_host_only);
        load_index(m_input_frame_size); load_index(m_output_frame_size);
        index_t c = 1, h = 1, w = 1;
        load_index(c); load_index(h); load_index(w);
        load_index(m_filter_h_size); load_index(m_filter_w_size);
        load_index(m_y_stride); load_index(m_x_stride);
        LoadValue(is, m_padding);
        std::int32_t mode = 0;
        LoadValue(is, mode);
        LoadValue(is, m_border_value);
        BB_ASSERT(is.good() && c >= 1 && h >= 1 && w >= 1 && m_filter_h_size >= 1 && m_filter_w_size >= 1 && m_y_stride >= 1 && m_x_stride >= 1);
        BB_ASSERT(mode >= BB_BORDER_CONSTANT && mode <= BB_BORDER_WRAP);
        m_border_mode = (int)mode;
        SetInputShape(indices_t({c, h, w}));
    }

public:
    static std::string ModelName(void)  { return "ConvolutionIm2Col"; }
    static std::string ObjectName(void) { return ModelName() + "_" + DataType<FT>::Name() + "_" + DataType<BT>::Name(); }
    std::string GetModelName(void) const override  { return ModelName(); }
    std::string GetObjectName(void) const override { return ObjectName(); }

    static std::shared_ptr<ConvolutionIm2Col> Create(create_t const &create) { return std::shared_ptr<ConvolutionIm2Col>(new ConvolutionIm2Col(create)); }
    static std::shared_ptr<ConvolutionIm2Col> Create(index_t filter_h_size, index_t filter_w_size, index_t y_stride = 1, index_t x_stride = 1,
                                                     std::string padding = "valid", std::string border_mode = "reflect_101")
    {
        create_t c;
        c.filter_h_size = filter_h_size; c.filter_w_size = filter_w_size; c.y_stride = y_stride; c.x_stride = x_stride;
        c.padding = padding; c.border_mode = border_mode;
        return Create(c);
    }

    index_t GetFilterSizeH(void) const { return m_filter_h_size; }
    index_t GetFilterSizeW(void) const { return m_filter_w_size; }
    index_t GetStrideX(void) const { return m_x_stride; }
    index_t GetStrideY(void) const { return m_y_stride; }
    index_t GetOutputSizeH(void) const { return m_output_h_size; }
    index_t GetOutputSizeW(void) const { return m_output_w_size; }
    std::string GetPadding(void) const { return m_padding; }

    // reference: include/bb/ConvolutionIm2Col.h:169-207
    indices_t SetInputShape(indices_t shape) override
    {
        BB_ASSERT(shape.size() == 3);
        m_input_shape = shape;
        m_input_c_size = shape[0]; m_input_h_size = shape[1]; m_input_w_size = shape[2];
        if (m_padding == "valid") {
            m_output_h_size = ((m_input_h_size - m_filter_h_size + 1) + (m_y_stride - 1)) / m_y_stride;
            m_output_w_size = ((m_input_w_size - m_filter_w_size + 1) + (m_x_stride - 1)) / m_x_stride;
            m_y_offset = 0; m_x_offset = 0;
        }
        else if (m_padding == "same") {
            m_output_h_size = (m_input_h_size + (m_y_stride - 1)) / m_y_stride;
            m_output_w_size = (m_input_w_size + (m_x_stride - 1)) / m_x_stride;
            m_y_offset = (m_filter_h_size - 1) / 2; m_x_offset = (m_filter_w_size - 1) / 2;
        }
        else { throw std::runtime_error("ConvolutionIm2Col: padding must be valid or same"); }
        m_output_shape = indices_t({m_input_c_size, m_filter_h_size, m_filter_w_size});
        return m_output_shape;
    }
    indices_t GetInputShape(void) const override { return m_input_shape; }
    indices_t GetOutputShape(void) const override { return m_output_shape; }

    FrameBuffer Forward(FrameBuffer x_buf, bool train = true) override
    {
        (void)train;
        BB_ASSERT(x_buf.GetType() == DataType<FT>::type);
        if (x_buf.GetShape() != m_input_shape) { SetInputShape(x_buf.GetShape()); }
        if (m_host_only || !x_buf.IsDeviceAvailable()) { throw std::runtime_error("ConvolutionIm2Col: no host path in this build"); }
        m_input_frame_size = x_buf.GetFrameSize();
        m_output_frame_size = m_input_frame_size * m_output_h_size * m_output_w_size;
        FrameBuffer y_buf(m_output_frame_size, m_output_shape, x_buf.GetType());
        auto px = x_buf.LockDeviceMemoryConst();
        auto py = y_buf.LockDeviceMemory(true);
        if (std::is_same<FT, Bit>::value) {
            CheckDevice(bbhip_bit_Im2Col_Forward((int const *)px.GetAddr(), (int *)py.GetAddr(), (int)m_x_stride, (int)m_y_stride, (int)m_x_offset,
                    (int)m_y_offset, (int)m_input_frame_size, (int)(x_buf.GetFrameStride() / 4), (int)m_input_w_size, (int)m_input_h_size,
                    (int)m_input_c_size, (int)m_output_w_size, (int)m_output_h_size, (int)(y_buf.GetFrameStride() / 4), (int)m_filter_w_size,
                    (int)m_filter_h_size, m_border_mode, nullptr), "bbhip_bit_Im2Col_Forward");
        }
        else {
            CheckDevice(bbhip_fp32_Im2Col_Forward((float const *)px.GetAddr(), (float *)py.GetAddr(), (int)m_x_stride, (int)m_y_stride, (int)m_x_offset,
                    (int)m_y_offset, (int)m_input_frame_size, (int)(x_buf.GetFrameStride() / 4), (int)m_input_w_size, (int)m_input_h_size,
                    (int)m_input_c_size, (int)m_output_w_size, (int)m_output_h_size, (int)(y_buf.GetFrameStride() / 4), (int)m_filter_w_size,
                    (int)m_filter_h_size, m_border_mode, (float)m_border_value, nullptr), "bbhip_fp32_Im2Col_Forward");
        }
        return y_buf;
    }

    FrameBuffer Backward(FrameBuffer dy_buf) override
    {
        if (dy_buf.Empty()) { return dy_buf; }
        BB_ASSERT(dy_buf.GetType() == BB_TYPE_FP32);
        if (m_host_only || !dy_buf.IsDeviceAvailable()) { throw std::runtime_error("ConvolutionIm2Col: no host path in this build"); }
        FrameBuffer dx_buf(m_input_frame_size, m_input_shape, BB_TYPE_FP32);
        auto pdy = dy_buf.LockDeviceMemoryConst();
        auto pdx = dx_buf.LockDeviceMemory(true);
        CheckDevice(bbhip_fp32_Im2Col_Backward((float const *)pdy.GetAddr(), (float *)pdx.GetAddr(), (int)m_x_stride, (int)m_y_stride, (int)m_x_offset,
                (int)m_y_offset, (int)m_input_frame_size, (int)(dx_buf.GetFrameStride() / 4), (int)m_input_w_size, (int)m_input_h_size,
                (int)m_input_c_size, (int)m_output_w_size, (int)m_output_h_size, (int)(dy_buf.GetFrameStride() / 4), (int)m_filter_w_size,
                (int)m_filter_h_size, nullptr), "bbhip_fp32_Im2Col_Backward");
        return dx_buf;
    }
};

}  // namespace bb

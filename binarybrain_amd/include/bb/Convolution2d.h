// A convolution as three layers: Im2Col turns every window position of every image into a frame, any layer (or list of
// layers) maps the window's taps to the output channels, Col2Im gathers the frames back into images
// (reference API: include/bb/Convolution2d.h:24-480; Forward / Backward :278-309).
// Serialized as  version 1 | Im2Col object | Col2Im object | bool: a layer follows | the layer object  (reference :355-409).
#pragma once

#include "bb/ConvolutionCol2Im.h"
#include "bb/ConvolutionIm2Col.h"
#include "bb/Model.h"

namespace bb {

template <typename FT = float, typename BT = float>
class Convolution2d : public Model {
    using Im2Col = ConvolutionIm2Col<FT, BT>;
    using Col2Im = ConvolutionCol2Im<FT, BT>;

    index_t     m_filter_h_size = 1, m_filter_w_size = 1;
    index_t     m_y_stride = 1, m_x_stride = 1;
    index_t     m_output_h_size = 1, m_output_w_size = 1;
    std::string m_padding = "valid";

    std::shared_ptr<Im2Col> m_im2col;
    std::shared_ptr<Model>  m_layer;
    std::shared_ptr<Col2Im> m_col2im;
    std::stack<indices_t>   m_input_shapes;         // one per forward pass in training mode, taken back by Backward

public:
    struct create_t {
        std::shared_ptr<Model> layer;
        index_t     filter_h_size = 1;
        index_t     filter_w_size = 1;
        index_t     x_stride = 1;
        index_t     y_stride = 1;
        std::string padding = "valid";
        std::string border_mode = "reflect_101";
        FT          border_value = (FT)0;
    };

protected:
    explicit Convolution2d(create_t const &create)
        : m_filter_h_size(create.filter_h_size), m_filter_w_size(create.filter_w_size), m_y_stride(create.y_stride),
          m_x_stride(create.x_stride), m_padding(create.padding), m_layer(create.layer)
    {
        typename Im2Col::create_t c;
        c.filter_h_size = create.filter_h_size; c.filter_w_size = create.filter_w_size;
        c.x_stride = create.x_stride; c.y_stride = create.y_stride;
        c.padding = create.padding; c.border_mode = create.border_mode; c.border_value = create.border_value;
        m_im2col = Im2Col::Create(c);
        m_col2im = Col2Im::Create();                // its image size follows from the input shape
    }

    void DumpObjectData(std::ostream &os) const override
    {
        SaveValue(os, (std::int64_t)1);
        m_im2col->DumpObject(os);
        m_col2im->DumpObject(os);
        bool const has_layer = (bool)m_layer;
        SaveValue(os, has_layer);
        if (has_layer) { m_layer->DumpObject(os); }
    }

    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = -1;
        LoadValue(is, ver);
        BB_ASSERT(ver == 1);
        m_im2col->LoadObject(is);
        m_col2im->LoadObject(is);
        bool has_layer = false;
        LoadValue(is, has_layer);
        if (has_layer) {
            if (m_layer) { m_layer->LoadObject(is); }
            else {
                m_layer = std::dynamic_pointer_cast<Model>(Object_Load(is));
                if (!m_layer) { throw Exception("Convolution2d: the stream holds a layer of a type that is not known here"); }
            }
        }
        m_filter_h_size = m_im2col->GetFilterSizeH(); m_filter_w_size = m_im2col->GetFilterSizeW();
        m_y_stride = m_im2col->GetStrideY();          m_x_stride = m_im2col->GetStrideX();
        m_padding = m_im2col->GetPadding();
        m_output_h_size = m_col2im->GetHeight();      m_output_w_size = m_col2im->GetWidth();
    }

public:
    static std::string ModelName(void)  { return "Convolution2d"; }
    static std::string ObjectName(void) { return ModelName() + "_" + DataType<FT>::Name() + "_" + DataType<BT>::Name(); }
    std::string GetModelName(void) const override  { return ModelName(); }
    std::string GetObjectName(void) const override { return ObjectName(); }

    static std::shared_ptr<Convolution2d> Create(create_t const &create) { return std::shared_ptr<Convolution2d>(new Convolution2d(create)); }
    static std::shared_ptr<Convolution2d> Create(std::shared_ptr<Model> layer, index_t filter_h_size, index_t filter_w_size,
                                                 index_t y_stride = 1, index_t x_stride = 1, std::string padding = "valid",
                                                 std::string border_mode = "reflect_101", FT border_value = (FT)0)
    {
        create_t c;
        c.layer = layer; c.filter_h_size = filter_h_size; c.filter_w_size = filter_w_size; c.y_stride = y_stride; c.x_stride = x_stride;
        c.padding = padding; c.border_mode = border_mode; c.border_value = border_value;
        return Create(c);
    }
    static std::shared_ptr<Convolution2d> Create(void) { return Create(create_t()); }

    std::shared_ptr<Model> GetSubLayer(void) const { return m_layer; }
    index_t GetFilterHeight(void) const { return m_filter_h_size; }
    index_t GetFilterWidth(void) const  { return m_filter_w_size; }

    void SendCommand(std::string command, std::string send_to = "all") override
    {
        m_im2col->SendCommand(command, send_to);
        if (m_layer) { m_layer->SendCommand(command, send_to); }
        m_col2im->SendCommand(command, send_to);
    }

    Variables GetParameters(void) override { return m_layer ? m_layer->GetParameters() : Variables(); }
    Variables GetGradients(void) override  { return m_layer ? m_layer->GetGradients() : Variables(); }

    // reference: include/bb/Convolution2d.h:213-250 (a repeated shape changes nothing)
    indices_t SetInputShape(indices_t shape) override
    {
        if (shape == GetInputShape()) { return GetOutputShape(); }
        BB_ASSERT(shape.size() == 3 && m_layer);
        index_t const h = shape[1], w = shape[2];
        if (m_padding == "valid") {
            m_output_h_size = ((h - m_filter_h_size + 1) + (m_y_stride - 1)) / m_y_stride;
            m_output_w_size = ((w - m_filter_w_size + 1) + (m_x_stride - 1)) / m_x_stride;
        }
        else if (m_padding == "same") {
            m_output_h_size = (h + (m_y_stride - 1)) / m_y_stride;
            m_output_w_size = (w + (m_x_stride - 1)) / m_x_stride;
        }
        else { throw std::runtime_error("Convolution2d: padding must be valid or same"); }
        m_col2im->SetOutputSize(m_output_h_size, m_output_w_size);
        shape = m_im2col->SetInputShape(shape);
        shape = m_layer->SetInputShape(shape);
        return m_col2im->SetInputShape(shape);
    }
    indices_t GetInputShape(void) const override  { return m_im2col->GetInputShape(); }
    indices_t GetOutputShape(void) const override { return m_col2im->GetOutputShape(); }

    FrameBuffer Forward(FrameBuffer x_buf, bool train = true) override
    {
        indices_t const shape = x_buf.GetShape();
        SetInputShape(shape);
        if (train) { m_input_shapes.push(shape); }
        x_buf = m_im2col->Forward(x_buf, train);
        x_buf = m_layer->Forward(x_buf, train);
        return m_col2im->Forward(x_buf, train);
    }

    FrameBuffer Backward(FrameBuffer dy_buf) override
    {
        BB_ASSERT(!m_input_shapes.empty());
        indices_t const shape = m_input_shapes.top();
        m_input_shapes.pop();
        SetInputShape(shape);
        dy_buf = m_col2im->Backward(dy_buf);
        dy_buf = m_layer->Backward(dy_buf);
        return m_im2col->Backward(dy_buf);
    }
};

}  // namespace bb

#include "bb/ObjectLoader.h"

// Node-major, frame-minor mini-batch buffer (reference API: include/bb/FrameBuffer.h:269-1868; layout :28-46, :927-939).
//
// Element (frame f, node n) lives at  base + n * frame_stride + f * sizeof(T)  for fp32 and at bit (f & 7) of byte
// base + n * frame_stride + (f >> 3)  for Bit (equivalently bit f & 31 of 32-bit word f >> 5).  frame_stride is in
// BYTES, as in the reference.  It is rounded up to a 256-byte multiple — one wavefront of fp32 frames — so that every
// node row starts on a wavefront boundary, and rows whose pitch would be a multiple of 2 KiB are lengthened by 512
// (fp32) / 384 (Bit) bytes: rows a power of two apart alias in the L2 of the GPU and the gathered rows evict each other.
// (The reference rounds to 32 bytes, include/bb/FrameBuffer.h:414-417; strides are arguments of every device entry point,
// so both choices are valid at the boundary.)
#pragma once

#include "bb/Core.h"
#include "bb/Tensor.h"

namespace bb {

class FrameBuffer;

template <typename T, bool CONST>
class FrameBufferView {
    using BytePtr = typename std::conditional<CONST, std::uint8_t const *, std::uint8_t *>::type;
    std::shared_ptr<Memory> m_mem;
    BytePtr                 m_base;
    index_t                 m_stride;       // bytes
public:
    FrameBufferView(std::shared_ptr<Memory> mem, BytePtr base, index_t stride) : m_mem(mem), m_base(base), m_stride(stride) {}

    // row of node `node` as the storage type (float, or bytes of packed bits)
    auto GetAddr(index_t node) const
    {
        using Elem = typename std::conditional<std::is_same<T, Bit>::value, std::uint8_t, T>::type;
        using Ptr  = typename std::conditional<CONST, Elem const *, Elem *>::type;
        return reinterpret_cast<Ptr>(m_base + node * m_stride);
    }
    auto GetAddr(void) const { return GetAddr(0); }

    T Get(index_t frame, index_t node) const
    {
        if (std::is_same<T, Bit>::value) {
            std::uint8_t const *row = reinterpret_cast<std::uint8_t const *>(m_base + node * m_stride);
            return T((row[frame >> 3] >> (frame & 7)) & 1);
        }
        return reinterpret_cast<T const *>(m_base + node * m_stride)[frame];
    }

    template <bool C = CONST>
    typename std::enable_if<!C>::type Set(index_t frame, index_t node, T value) const
    {
        if (std::is_same<T, Bit>::value) {
            std::uint8_t *row = reinterpret_cast<std::uint8_t *>(m_base + node * m_stride);
            std::uint8_t const m = (std::uint8_t)(1u << (frame & 7));
            if ((bool)value) { row[frame >> 3] |= m; } else { row[frame >> 3] &= (std::uint8_t)~m; }
            return;
        }
        reinterpret_cast<T *>(m_base + node * m_stride)[frame] = value;
    }
};


class FrameBuffer {
    int                     m_type = BB_TYPE_FP32;
    index_t                 m_frame_size = 0;
    index_t                 m_frame_stride = 0;     // bytes per node row
    index_t                 m_node_size = 0;
    indices_t               m_shape;
    bool                    m_host_only = false;
    std::shared_ptr<Memory> m_mem;
    // The packed copy (bit = value > 0.5) of a binarized fp32 buffer, written by the layer that produced the buffer in the same launch
    // (bbhip_HintPackedOutput).  It travels with the buffer's copies and holds good while nobody has taken a writable lock on the
    // fp32 memory since it was attached: the layer that reads the buffer next then takes the bits instead of packing the values again.
    struct PackedTwin { std::shared_ptr<FrameBuffer> bits; std::uint64_t writes; };
    std::shared_ptr<PackedTwin> m_twin;

public:
    // bits: a BB_TYPE_BIT buffer of the same shape and frame count.  Called by the producing layer after its launch, while the
    // writable lock it took on this buffer for that launch is the last one handed out.
    void AttachPackedTwin(FrameBuffer const &bits);
    // the packed copy, or an empty buffer when there is none or the fp32 memory may have been written since
    FrameBuffer GetPackedTwin(void) const;

    static index_t CalcFrameStride(int type, index_t frame_size)
    {
        index_t bytes = ((frame_size * DataType_GetBitSize(type) + 2047) / 2048) * 256;
        if (bytes > 0 && bytes % 2048 == 0) { bytes += (type == BB_TYPE_BIT) ? 384 : 512; }
        return bytes;
    }

    explicit FrameBuffer(index_t frame_size = 0, indices_t shape = indices_t(), int type = BB_TYPE_FP32, bool host_only = false)
        : m_host_only(host_only)
    {
        Resize(frame_size, shape, type);
    }

    void Resize(index_t frame_size, indices_t shape, int type)
    {
        m_type = type;
        m_frame_size = frame_size;
        m_shape = shape;
        m_node_size = shape.empty() ? 0 : CalcShapeSize(shape);
        m_frame_stride = CalcFrameStride(type, frame_size);
        m_mem = Memory::Create((std::size_t)(m_node_size * m_frame_stride), m_host_only);
        m_twin.reset();
    }

    bool      Empty(void) const          { return m_frame_size == 0 || m_node_size == 0; }
    int       GetType(void) const        { return m_type; }
    index_t   GetFrameSize(void) const   { return m_frame_size; }
    index_t   GetFrameStride(void) const { return m_frame_stride; }
    index_t   GetNodeSize(void) const    { return m_node_size; }
    indices_t GetShape(void) const       { return m_shape; }
    bool      IsHostOnly(void) const     { return m_host_only; }
    bool      IsDeviceAvailable(void) const { return m_mem->IsDeviceAvailable(); }

    template <typename T> auto Lock(bool discard = false)
    {
        BB_ASSERT(DataType<T>::type == m_type);
        return FrameBufferView<T, false>(m_mem, static_cast<std::uint8_t *>(m_mem->Lock(discard)), m_frame_stride);
    }
    template <typename T> auto LockConst(void) const
    {
        BB_ASSERT(DataType<T>::type == m_type);
        return FrameBufferView<T, true>(m_mem, static_cast<std::uint8_t const *>(m_mem->LockConst()), m_frame_stride);
    }
    DevicePtr      LockDeviceMemory(bool discard = false) { return DevicePtr(m_mem, m_mem->LockDevice(discard)); }
    DeviceConstPtr LockDeviceMemoryConst(void) const      { return DeviceConstPtr(m_mem, m_mem->LockDeviceConst()); }

    void FillZero(void) { m_mem->FillZero(); }

    // element access by value; each call takes and releases a host lock, keep it out of hot loops
    void  SetFP32(index_t frame, index_t node, float v) { Lock<float>().Set(frame, node, v); }
    float GetFP32(index_t frame, index_t node) const    { return LockConst<float>().Get(frame, node); }
    void  SetBit(index_t frame, index_t node, bool v)   { Lock<Bit>().Set(frame, node, Bit(v)); }
    bool  GetBit(index_t frame, index_t node) const     { return (bool)LockConst<Bit>().Get(frame, node); }

    // sum of all elements in double, taken on the host (reference: Tensor_<T>::Sum, include/bb/Tensor.h:918-926)
    double Sum(void) const
    {
        double sum = 0;
        if (m_type == BB_TYPE_FP32) {
            auto p = LockConst<float>();
            for (index_t node = 0; node < m_node_size; ++node) { float const *row = p.GetAddr(node); for (index_t f = 0; f < m_frame_size; ++f) { sum += row[f]; } }
        }
        else if (m_type == BB_TYPE_INT32) {
            auto p = LockConst<std::int32_t>();
            for (index_t node = 0; node < m_node_size; ++node) { std::int32_t const *row = p.GetAddr(node); for (index_t f = 0; f < m_frame_size; ++f) { sum += row[f]; } }
        }
        else {
            throw Exception("FrameBuffer::Sum: fp32 and int32 buffers only");
        }
        return sum;
    }

    // packed bits -> fp32 0/1 on the device (reference: FrameBuffer::ConvertTo, include/bb/FrameBuffer.h:838-900)
    FrameBuffer ConvertBitToFP32(void) const
    {
        BB_ASSERT(m_type == BB_TYPE_BIT);
        FrameBuffer dst(m_frame_size, m_shape, BB_TYPE_FP32, m_host_only);
        auto src_ptr = LockDeviceMemoryConst();
        auto dst_ptr = dst.LockDeviceMemory(true);
        CheckDevice(bbhip_fp32_ConvBitToReal((int const *)src_ptr.GetAddr(), (float *)dst_ptr.GetAddr(), 0.0f, 1.0f,
                                             (int)m_node_size, (int)m_frame_size, (int)(m_frame_stride / 4),
                                             (int)(dst.GetFrameStride() / 4), nullptr), "bbhip_fp32_ConvBitToReal");
        return dst;
    }
};

inline void FrameBuffer::AttachPackedTwin(FrameBuffer const &bits)
{
    BB_ASSERT(bits.GetType() == BB_TYPE_BIT && bits.GetFrameSize() == m_frame_size && bits.GetNodeSize() == m_node_size);
    m_twin = std::make_shared<PackedTwin>(PackedTwin{std::make_shared<FrameBuffer>(bits), m_mem->WriteCount()});
}

inline FrameBuffer FrameBuffer::GetPackedTwin(void) const
{
    if (m_twin && m_twin->bits && m_mem && m_twin->writes == m_mem->WriteCount() && m_twin->bits->GetFrameSize() == m_frame_size &&
        m_twin->bits->GetNodeSize() == m_node_size) {
        return *m_twin->bits;
    }
    return FrameBuffer();
}

}  // namespace bb

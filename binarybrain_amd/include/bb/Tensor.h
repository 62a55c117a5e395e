// Dense row-major tensors over a mirrored Memory block, plus the list-of-tensors type used for parameters and
// gradients (reference API: include/bb/Tensor.h:304-608 `Tensor_<T>` / `Tensor`, include/bb/Variables.h:20-120).
// Only what the LUT layers use is provided: shape handling, typed host accessors, raw device pointers, zero fill,
// clamp, seeded initialisation.
#pragma once

#include <cmath>
#include <random>

#include "bb/Core.h"
#include "bb/Object.h"

namespace bb {

// typed host view of a tensor; element (i0, i1) of a 2-d tensor is at i0 * shape[1] + i1 (row-major)
template <typename T, typename VoidPtr>
class TensorView {
    std::shared_ptr<Memory> m_mem;      // keeps the block alive while the view exists
    VoidPtr                 m_ptr;
    indices_t               m_shape;
public:
    TensorView(std::shared_ptr<Memory> mem, VoidPtr ptr, indices_t shape) : m_mem(mem), m_ptr(ptr), m_shape(shape) {}
    auto GetAddr(void) const { return reinterpret_cast<typename std::conditional<std::is_const<typename std::remove_pointer<VoidPtr>::type>::value, T const *, T *>::type>(m_ptr); }
    auto &operator[](index_t i) const { return GetAddr()[i]; }
    auto &operator()(index_t i0) const { return GetAddr()[i0]; }
    auto &operator()(index_t i0, index_t i1) const { return GetAddr()[i0 * m_shape[1] + i1]; }
};

class DevicePtr {
    std::shared_ptr<Memory> m_mem;
    void                   *m_ptr;
public:
    DevicePtr(std::shared_ptr<Memory> mem, void *ptr) : m_mem(mem), m_ptr(ptr) {}
    void *GetAddr(void) const { return m_ptr; }
};

class DeviceConstPtr {
    std::shared_ptr<Memory> m_mem;
    void const             *m_ptr;
public:
    DeviceConstPtr(std::shared_ptr<Memory> mem, void const *ptr) : m_mem(mem), m_ptr(ptr) {}
    void const *GetAddr(void) const { return m_ptr; }
};


class Tensor : public Object {
protected:
    int                     m_type = BB_TYPE_FP32;
    indices_t               m_shape;
    index_t                 m_size = 0;
    bool                    m_host_only = false;
    std::shared_ptr<Memory> m_mem;

public:
    explicit Tensor(bool host_only = false) : m_host_only(host_only), m_mem(Memory::Create(0, host_only)) {}
    Tensor(indices_t shape, int type, bool host_only = false) : m_host_only(host_only) { Resize(shape, type); }

    void Resize(indices_t shape, int type)
    {
        m_type  = type;
        m_shape = shape;
        m_size  = CalcShapeSize(shape);
        m_mem   = Memory::Create((std::size_t)m_size * (std::size_t)(DataType_GetBitSize(type) / 8), m_host_only);
    }

    std::string GetObjectName(void) const override { return "Tensor"; }

protected:
    // the layout of the reference's typed tensor (include/bb/Tensor.h:614-651): version, parent version, element offset,
    // element count, shape, row-major strides, elements
    void DumpTypedData(std::ostream &os) const
    {
        SaveValue(os, (std::int64_t)1);
        SaveValue(os, (std::int64_t)0);
        SaveValue(os, (std::int64_t)0);
        SaveValue(os, (std::int64_t)m_size);
        SaveIndices(os, m_shape);
        indices_t stride(m_shape.size());
        index_t total = 1;
        for (std::size_t i = m_shape.size(); i-- > 0;) { stride[i] = total; total *= m_shape[i]; }
        SaveIndices(os, stride);
        if (m_size > 0) { os.write(static_cast<char const *>(m_mem->LockConst()), (std::streamsize)(m_size * (DataType_GetBitSize(m_type) / 8))); }
    }
    void LoadTypedData(std::istream &is, int type)
    {
        std::int64_t ver = 0, parent = -1, offset = -1, size = -1;
        LoadValue(is, ver);    BB_ASSERT(ver == 1);
        LoadValue(is, parent); BB_ASSERT(parent == 0);
        LoadValue(is, offset); BB_ASSERT(offset == 0);
        LoadValue(is, size);
        indices_t const shape = LoadIndices(is);
        BB_ASSERT(is.good() && size == CalcShapeSize(shape));
        Resize(shape, type);
        (void)LoadIndices(is);
        if (m_size > 0) { is.read(static_cast<char *>(m_mem->Lock(true)), (std::streamsize)(m_size * (DataType_GetBitSize(type) / 8))); }
    }
    // untyped tensor: version, parent version, element type code, then the typed layout (include/bb/Tensor.h:2159-2211)
    void DumpObjectData(std::ostream &os) const override
    {
        SaveValue(os, (std::int64_t)1);
        SaveValue(os, (std::int64_t)0);
        SaveValue(os, (std::int32_t)m_type);
        DumpTypedData(os);
    }
    void LoadObjectData(std::istream &is) override
    {
        std::int64_t ver = 0, parent = -1;
        std::int32_t type = 0;
        LoadValue(is, ver);    BB_ASSERT(ver == 1);
        LoadValue(is, parent); BB_ASSERT(parent == 0);
        LoadValue(is, type);
        (void)DataType_GetBitSize(type);        // throws on a type code this library does not hold
        LoadTypedData(is, type);
    }

public:
    int       GetType(void) const  { return m_type; }
    indices_t GetShape(void) const { return m_shape; }
    index_t   GetSize(void) const  { return m_size; }
    bool      IsDeviceAvailable(void) const { return m_mem->IsDeviceAvailable(); }
    std::shared_ptr<Memory> GetMemory(void) const { return m_mem; }

    template <typename T> auto Lock(bool discard = false)
    {
        BB_ASSERT(DataType<T>::type == m_type);
        return TensorView<T, void *>(m_mem, m_mem->Lock(discard), m_shape);
    }
    template <typename T> auto LockConst(void) const
    {
        BB_ASSERT(DataType<T>::type == m_type);
        return TensorView<T, void const *>(m_mem, m_mem->LockConst(), m_shape);
    }
    // identifies the contents: the same stamp at two moments = no writable lock was taken and no new block was put in between
    std::pair<void const *, std::uint64_t> WriteStamp(void) const { return {m_mem.get(), m_mem ? m_mem->WriteCount() : 0}; }
    DevicePtr      LockDeviceMemory(bool discard = false) { return DevicePtr(m_mem, m_mem->LockDevice(discard)); }
    DeviceConstPtr LockDeviceMemoryConst(void) const      { return DeviceConstPtr(m_mem, m_mem->LockDeviceConst()); }

    void FillZero(void) { m_mem->FillZero(); }

    // in-place clamp on the device (the forward pass of the stochastic LUT clamps its table first,
    // reference: include/bb/StochasticLutN.h:451 -> include/bb/Tensor.h:1266-1271)
    void Clamp_inplace(float lo, float hi)
    {
        BB_ASSERT(m_type == BB_TYPE_FP32);
        if (m_size == 0) { return; }
        BB_ASSERT(m_size <= 0x7fffffff);
        float *p = static_cast<float *>(m_mem->LockDevice());
        CheckDevice(bbhip_fp32_Vector_clamp(p, p, lo, hi, (int)m_size, nullptr), "bbhip_fp32_Vector_clamp");
    }

    // seeded initialisation (reference: include/bb/Tensor.h:540-565; the exact stream is a property of the C++ library)
    void InitNormalDistribution(double mean, double stddev, std::uint64_t seed)
    {
        std::mt19937_64 mt(seed);
        std::normal_distribution<double> dist(mean, stddev);
        auto p = Lock<float>(true);
        for (index_t i = 0; i < m_size; ++i) { p[i] = (float)dist(mt); }
    }
    void InitUniformDistribution(double lo, double hi, std::uint64_t seed)
    {
        std::mt19937_64 mt(seed);
        std::uniform_real_distribution<double> dist(lo, hi);
        auto p = Lock<float>(true);
        for (index_t i = 0; i < m_size; ++i) { p[i] = (float)dist(mt); }
    }
};


// tensor with a fixed element type
template <typename T>
class Tensor_ : public Tensor {
public:
    explicit Tensor_(bool host_only = false) : Tensor(host_only) { m_type = DataType<T>::type; }
    explicit Tensor_(indices_t shape, bool host_only = false) : Tensor(shape, DataType<T>::type, host_only) {}
    void Resize(indices_t shape) { Tensor::Resize(shape, DataType<T>::type); }
    void Resize(index_t i0) { Resize(indices_t({i0})); }
    void Resize(index_t i0, index_t i1) { Resize(indices_t({i0, i1})); }
    auto Lock(bool discard = false) { return Tensor::Lock<T>(discard); }
    auto LockConst(void) const { return Tensor::LockConst<T>(); }
    std::string GetObjectName(void) const override { return "Tensor_" + DataType<T>::Name(); }
protected:
    void DumpObjectData(std::ostream &os) const override { DumpTypedData(os); }
    void LoadObjectData(std::istream &is) override { LoadTypedData(is, DataType<T>::type); }
public:
    Tensor_ &operator=(T value)
    {
        auto p = Lock(true);
        for (index_t i = 0; i < m_size; ++i) { p[i] = value; }
        return *this;
    }
};


// ordered list of shared tensors: a layer's parameters or their gradients
class Variables {
    std::vector<std::shared_ptr<Tensor>> m_tensors;
public:
    void PushBack(std::shared_ptr<Tensor> t) { m_tensors.push_back(t); }
    void PushBack(Variables const &v) { for (auto &t : v.m_tensors) { m_tensors.push_back(t); } }
    index_t GetSize(void) const { return (index_t)m_tensors.size(); }
    Tensor &operator[](index_t i) { return *m_tensors[(std::size_t)i]; }
    Tensor const &operator[](index_t i) const { return *m_tensors[(std::size_t)i]; }
    void FillZero(void) { for (auto &t : m_tensors) { t->FillZero(); } }
};

}  // namespace bb

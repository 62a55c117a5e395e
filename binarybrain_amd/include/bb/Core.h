// Host-side plumbing shared by the LUT model classes: scalar types and type codes, assertions, string helpers,
// the device manager switch and a host/device mirrored memory block.
//
// The names and semantics follow BinaryBrain's host API so that model code written against it reads the same
// (reference: include/bb/DataType.h:30-54, 271-315; include/bb/Manager.h:17-40; include/bb/Memory.h:45-823;
// include/bb/Assert.h:26-33).  Everything device-side goes through the C ABI in include/bbhip.h — this header
// needs no HIP headers and compiles with a plain host compiler.
#pragma once

#include <cstdint>
#include <cstring>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "bbhip.h"

// numeric codes of the element types (same values as the reference, they appear in serialized objects)
#define BB_TYPE_BIT     (0x0000 + 1)
#define BB_TYPE_BINARY  (0x0000 + 2)
#define BB_TYPE_FP32    (0x0100 + 32)
#define BB_TYPE_FP64    (0x0100 + 64)
#define BB_TYPE_INT32   (0x0200 + 32)
#define BB_TYPE_UINT8   (0x0300 + 8)

// the two values of a binary signal held as a number (reference: include/bb/DataType.h:48-49)
#define BB_BINARY_HI    (+1)
#define BB_BINARY_LO    (-1)

namespace bb {

using index_t   = std::int64_t;
using indices_t = std::vector<index_t>;

class Exception : public std::runtime_error {
public:
    explicit Exception(std::string const &what) : std::runtime_error(what) {}
};

// failed preconditions throw (the reference does this under BB_ASSERT_EXCEPTION, include/bb/Assert.h:26-33)
#define BB_ASSERT(cond) \
    do { if (!(cond)) { throw bb::Exception(std::string("BB_ASSERT(" #cond ") failed at ") + __FILE__ + ":" + std::to_string(__LINE__)); } } while (0)

// a failing device call carries the library's message
inline void CheckDevice(int rc, char const *what)
{
    if (rc != 0) { throw Exception(std::string(what) + ": " + bbhip_GetLastErrorString()); }
}

// one frame of a packed buffer (reference: include/bb/DataType.h:271-315)
class Bit {
    bool m_v = false;
public:
    Bit() {}
    Bit(bool v) : m_v(v) {}
    Bit(int v) : m_v(v != 0) {}
    Bit(float v) : m_v(v > 0.5f) {}
    operator bool() const { return m_v; }
};

template <typename T> struct DataType {};
template <> struct DataType<float>        { static constexpr int type = BB_TYPE_FP32;  static constexpr int bits = 32; static std::string Name() { return "fp32"; } };
template <> struct DataType<double>       { static constexpr int type = BB_TYPE_FP64;  static constexpr int bits = 64; static std::string Name() { return "fp64"; } };
template <> struct DataType<std::int32_t> { static constexpr int type = BB_TYPE_INT32; static constexpr int bits = 32; static std::string Name() { return "int32"; } };
template <> struct DataType<std::uint8_t> { static constexpr int type = BB_TYPE_UINT8; static constexpr int bits = 8;  static std::string Name() { return "uint8"; } };
template <> struct DataType<Bit>          { static constexpr int type = BB_TYPE_BIT;   static constexpr int bits = 1;  static std::string Name() { return "bit"; } };

inline int DataType_GetBitSize(int type)
{
    switch (type) {
    case BB_TYPE_BIT:   return 1;
    case BB_TYPE_UINT8: return 8;
    case BB_TYPE_FP32:  return 32;
    case BB_TYPE_FP64:  return 64;
    case BB_TYPE_INT32: return 32;
    }
    throw Exception("unsupported data type code " + std::to_string(type));
}

inline index_t CalcShapeSize(indices_t const &shape)
{
    index_t n = 1;
    for (auto s : shape) { n *= s; }
    return n;
}

inline std::vector<std::string> SplitString(std::string const &text)
{
    std::istringstream ss(text);
    std::vector<std::string> out;
    std::string tok;
    while (ss >> tok) { out.push_back(tok); }
    return out;
}

inline bool EvalBool(std::string const &s)
{
    return s == "true" || s == "True" || s == "TRUE" || s == "1" || s == "on" || s == "ON";
}

// global switch between device and host-only buffers (reference: include/bb/Manager.h:17-40)
class Manager {
public:
    static bool IsDeviceAvailable(void) { return bbhip_IsDeviceAvailable() != 0; }
    static void SetHostOnly(bool host_only) { bbhip_SetHostOnly(host_only ? 1 : 0); }
    static bool IsHostOnly(void) { return bbhip_IsHostOnly() != 0; }
};


// A block of bytes mirrored between host and device.  Each side is allocated on first use; a write lock on one side
// marks the other side stale, and a later lock on the stale side copies the block over first (the lazy mirroring of
// the reference's Memory class, include/bb/Memory.h:524-662).  Host and device locks must not be held together.
class Memory {
    std::size_t m_size = 0;
    bool        m_host_only = false;
    void       *m_host = nullptr;
    void       *m_dev = nullptr;
    bool        m_host_valid = false;   // host copy holds the current contents
    bool        m_dev_valid = false;    // device copy holds the current contents
    bool        m_host_pinned = false;
    std::uint64_t m_writes = 0;         // writable locks handed out (WriteCount)

    void alloc_host(void)
    {
        if (m_host || m_size == 0) { return; }
        if (!m_host_only && Manager::IsDeviceAvailable()) {
            CheckDevice(bbhip_MallocHost(&m_host, m_size), "bbhip_MallocHost");
            m_host_pinned = true;
        }
        else {
            m_host = ::operator new(m_size);
        }
    }
    void alloc_dev(void)
    {
        if (m_dev || m_size == 0) { return; }
        BB_ASSERT(IsDeviceAvailable());
        CheckDevice(bbhip_Malloc(&m_dev, m_size), "bbhip_Malloc");
    }
    void release(void)
    {
        if (m_host) { if (m_host_pinned) { bbhip_FreeHost(m_host); } else { ::operator delete(m_host); } }
        if (m_dev)  { bbhip_Free(m_dev); }
        m_host = m_dev = nullptr;
        m_host_valid = m_dev_valid = m_host_pinned = false;
    }

public:
    explicit Memory(std::size_t size = 0, bool host_only = false) : m_size(size), m_host_only(host_only) {}
    ~Memory() { release(); }
    Memory(Memory const &) = delete;
    Memory &operator=(Memory const &) = delete;

    static std::shared_ptr<Memory> Create(std::size_t size, bool host_only = false) { return std::make_shared<Memory>(size, host_only); }

    std::size_t GetSize(void) const { return m_size; }
    bool IsHostOnly(void) const { return m_host_only; }
    bool IsDeviceAvailable(void) const { return !m_host_only && Manager::IsDeviceAvailable(); }

    void Resize(std::size_t size) { release(); m_size = size; ++m_writes; }

    // how many writable locks were handed out so far: unchanged between two moments = nothing could write in between
    std::uint64_t WriteCount(void) const { return m_writes; }

    // host side, read-write (discard = old contents not needed)
    void *Lock(bool discard = false)
    {
        ++m_writes;
        alloc_host();
        if (!discard && !m_host_valid && m_dev_valid) { CheckDevice(bbhip_Memcpy(m_host, m_dev, m_size, 2), "bbhip_Memcpy(D2H)"); }
        m_host_valid = true;
        m_dev_valid = false;
        return m_host;
    }
    void const *LockConst(void)
    {
        alloc_host();
        if (!m_host_valid && m_dev_valid) { CheckDevice(bbhip_Memcpy(m_host, m_dev, m_size, 2), "bbhip_Memcpy(D2H)"); }
        m_host_valid = true;
        return m_host;
    }
    // device side
    void *LockDevice(bool discard = false)
    {
        ++m_writes;
        alloc_dev();
        if (!discard && !m_dev_valid && m_host_valid) { CheckDevice(bbhip_Memcpy(m_dev, m_host, m_size, 1), "bbhip_Memcpy(H2D)"); }
        m_dev_valid = true;
        m_host_valid = false;
        return m_dev;
    }
    void const *LockDeviceConst(void)
    {
        alloc_dev();
        if (!m_dev_valid && m_host_valid) { CheckDevice(bbhip_Memcpy(m_dev, m_host, m_size, 1), "bbhip_Memcpy(H2D)"); }
        m_dev_valid = true;
        return m_dev;
    }

    void FillZero(void)
    {
        if (m_size == 0) { return; }
        if (IsDeviceAvailable()) { CheckDevice(bbhip_Memset(LockDevice(true), 0, m_size), "bbhip_Memset"); }
        else                     { std::memset(Lock(true), 0, m_size); }
    }
};

}  // namespace bb

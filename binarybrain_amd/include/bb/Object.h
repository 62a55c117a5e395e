// Binary object serialization in the reference's `.bb_net` layout (include/bb/Object.h:28-179, value helpers
// include/bb/DataType.h:58-70, 215-236, 670-741).  An object is
//     "BB_OBJ" | int64 header version (1) | uint64 name length | name | object data
// and object data is, class by class from the most derived one down: int64 version, the parent's data, the members.
// Scalars are written in host byte order and width (bool as one byte), strings and vectors as a uint64 count followed by the
// elements, index lists as int64 count and int64 elements.  Files written here load in the reference and the other way round.
#pragma once

#include <fstream>
#include <istream>
#include <ostream>

#include "bb/Core.h"

namespace bb {

template <typename T>
inline void SaveValue(std::ostream &os, T const &val) { os.write(reinterpret_cast<char const *>(&val), sizeof(T)); }
template <typename T>
inline void LoadValue(std::istream &is, T &val) { is.read(reinterpret_cast<char *>(&val), sizeof(T)); }

inline void SaveValue(std::ostream &os, bool const &val) { std::int8_t v = (std::int8_t)val; os.write(reinterpret_cast<char const *>(&v), 1); }
inline void LoadValue(std::istream &is, bool &val)       { std::int8_t v = 0; is.read(reinterpret_cast<char *>(&v), 1); val = (v != 0); }

inline void SaveValue(std::ostream &os, std::string const &str)
{
    std::uint64_t const size = (std::uint64_t)str.size();
    SaveValue(os, size);
    if (size > 0) { os.write(str.data(), (std::streamsize)size); }
}
inline void LoadValue(std::istream &is, std::string &str)
{
    std::uint64_t size = 0;
    LoadValue(is, size);
    BB_ASSERT(is.good() && size < (1ull << 32));
    str.resize((std::size_t)size);
    if (size > 0) { is.read(&str[0], (std::streamsize)size); }
}

template <typename T>
inline void SaveValue(std::ostream &os, std::vector<T> const &vec)
{
    std::uint64_t const size = (std::uint64_t)vec.size();
    SaveValue(os, size);
    if (size > 0) { os.write(reinterpret_cast<char const *>(vec.data()), (std::streamsize)(size * sizeof(T))); }
}
template <typename T>
inline void LoadValue(std::istream &is, std::vector<T> &vec)
{
    std::uint64_t size = 0;
    LoadValue(is, size);
    BB_ASSERT(is.good() && size < (1ull << 32));
    vec.resize((std::size_t)size);
    if (size > 0) { is.read(reinterpret_cast<char *>(vec.data()), (std::streamsize)(size * sizeof(T))); }
}

inline void SaveIndices(std::ostream &os, indices_t const &indices)
{
    SaveValue(os, (std::int64_t)indices.size());
    for (auto v : indices) { SaveValue(os, (std::int64_t)v); }
}
inline indices_t LoadIndices(std::istream &is)
{
    std::int64_t size = 0;
    LoadValue(is, size);
    BB_ASSERT(is.good() && size >= 0 && size < (1ll << 32));
    indices_t indices((std::size_t)size);
    for (auto &v : indices) { std::int64_t e = 0; LoadValue(is, e); v = (index_t)e; }
    return indices;
}


class Object;
inline std::shared_ptr<Object> Object_Load(std::istream &is);       // bb/ObjectLoader.h

class Object {
    friend std::shared_ptr<Object> Object_Load(std::istream &is);

    static std::string ReadHeader(std::istream &is)
    {
        char tag[6] = {0, 0, 0, 0, 0, 0};
        is.read(tag, 6);
        BB_ASSERT(is.good() && std::memcmp(tag, "BB_OBJ", 6) == 0);
        std::int64_t ver = 0;
        LoadValue(is, ver);
        std::string name;
        LoadValue(is, name);
        return name;
    }

public:
    virtual ~Object() {}
    virtual std::string GetObjectName(void) const = 0;

    void DumpObject(std::ostream &os) const
    {
        os.write("BB_OBJ", 6);
        SaveValue(os, (std::int64_t)1);
        SaveValue(os, GetObjectName());
        DumpObjectData(os);
    }

    void LoadObject(std::istream &is)
    {
        std::string const name = ReadHeader(is);
        if (name != GetObjectName()) { throw Exception("LoadObject: the stream holds a " + name + ", expected a " + GetObjectName()); }
        LoadObjectData(is);
        BB_ASSERT(!is.fail());
    }

    bool DumpToFile(std::string filename) const
    {
        std::ofstream ofs(filename, std::ios::binary);
        if (!ofs.is_open()) { return false; }
        DumpObject(ofs);
        return true;
    }
    bool LoadFromFile(std::string filename)
    {
        std::ifstream ifs(filename, std::ios::binary);
        if (!ifs.is_open()) { return false; }
        LoadObject(ifs);
        return true;
    }

protected:
    // a class without members of its own marks itself with version 0
    virtual void DumpObjectData(std::ostream &os) const { SaveValue(os, (std::int64_t)0); }
    virtual void LoadObjectData(std::istream &is)
    {
        std::int64_t ver = -1;
        LoadValue(is, ver);
        BB_ASSERT(ver == 0);
    }
};

}  // namespace bb

// Command-line driver for the serialization tests (CPU only): builds, loads, re-writes and takes apart serialized LUT layers
// with the host classes, so that the Python tests can compare bytes and contents with the reference's
// (tests/test_serialization.py).  Contents travel as raw little-endian files <prefix>.idx / .params / .mean / .var.
//
//   object_tool make      <kind> <bit> <I> <O> <flags> <name|-> <prefix> <out.bb_net>
//   object_tool roundtrip <kind> <bit> <in.bb_net> <out.bb_net>
//   object_tool describe  <kind> <bit> <in.bb_net> <prefix>          prints "I O name" on one line
//   object_tool wiring    <kind> <seed> <policy|-> <dims> <input shape ...> <output shape ...> <prefix>
//                         seeded wiring of a fresh layer (kind 0: the connection table of StochasticLutN / DifferentiableLutN,
//                         2: BinaryLutN created with that seed, 3: StochasticLutN created with that seed): writes <prefix>.idx and, for BinaryLutN, <prefix>.params
//
// kind 0 = StochasticLutN<6>, 1 = DifferentiableLutN<6>, 2 = BinaryLutN<6, Bit>; bit selects BinType = Bit for kinds 0, 1.
// flags: bit 0 = binary, bit 1 = lut_binarize, bit 2 = batch_norm.  DifferentiableLut scalars are fixed: momentum 0.75,
// gamma 0.4, beta 0.6.  Exit status 0 on success, 1 with a message on stderr when an object is rejected.
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <string>
#include <vector>

#include "bb/StochasticLutN.h"
#include "bb/DifferentiableLutN.h"
#include "bb/BinaryLutN.h"
#include "bb/ObjectLoader.h"

template <typename T>
static std::vector<T> read_raw(std::string const &path, size_t count)
{
    std::vector<T> v(count);
    std::ifstream f(path, std::ios::binary);
    if (!f.is_open()) { throw bb::Exception("cannot open " + path); }
    f.read(reinterpret_cast<char *>(v.data()), (std::streamsize)(count * sizeof(T)));
    if ((size_t)f.gcount() != count * sizeof(T)) { throw bb::Exception("short file " + path); }
    return v;
}
template <typename T>
static void write_raw(std::string const &path, std::vector<T> const &v)
{
    std::ofstream f(path, std::ios::binary);
    f.write(reinterpret_cast<char const *>(v.data()), (std::streamsize)(v.size() * sizeof(T)));
}

template <class M>
static void put_wiring(M &m, int O, std::vector<std::int32_t> const &idx)
{
    for (int o = 0; o < O; ++o) { for (int i = 0; i < 6; ++i) { m.SetNodeConnectionIndex(o, i, idx[(size_t)o * 6 + i]); } }
}
template <class M>
static std::vector<std::int32_t> get_wiring(M const &m)
{
    int const O = (int)m.GetOutputNodeSize();
    std::vector<std::int32_t> idx((size_t)O * 6);
    for (int o = 0; o < O; ++o) { for (int i = 0; i < 6; ++i) { idx[(size_t)o * 6 + i] = (std::int32_t)m.GetNodeConnectionIndex(o, i); } }
    return idx;
}

template <typename BinType>
struct Stochastic {
    using Model = bb::StochasticLutN<6, BinType, float>;
    static std::shared_ptr<Model> blank(int O) { return Model::Create((bb::index_t)O); }
    static void fill(Model &m, int I, int O, int flags, std::string const &prefix)
    {
        m.SetInputShape({(bb::index_t)I});
        put_wiring(m, O, read_raw<std::int32_t>(prefix + ".idx", (size_t)O * 6));
        auto W = read_raw<float>(prefix + ".params", (size_t)O * 64);
        { auto p = m.lock_W(); for (size_t k = 0; k < W.size(); ++k) { p[(bb::index_t)k] = W[k]; } }
        m.SendCommand(std::string("binary ") + ((flags & 1) ? "true" : "false"));
        m.SendCommand(std::string("lut_binarize ") + ((flags & 2) ? "true" : "false"));
    }
    static void take_apart(Model const &m, std::string const &prefix)
    {
        write_raw(prefix + ".idx", get_wiring(m));
        std::vector<float> W((size_t)m.GetOutputNodeSize() * 64);
        { auto p = m.lock_W_const(); for (size_t k = 0; k < W.size(); ++k) { W[k] = p[(bb::index_t)k]; } }
        write_raw(prefix + ".params", W);
    }
};

template <typename BinType>
struct Differentiable {
    using Model = bb::DifferentiableLutN<6, BinType, float>;
    static std::shared_ptr<Model> blank(int O) { return Model::Create((bb::index_t)O); }
    static std::shared_ptr<Model> configured(int O, int flags)
    {
        typename Model::create_t c;
        c.output_shape = {(bb::index_t)O};
        c.batch_norm = (flags & 4) != 0;
        c.binary = (flags & 1) != 0;
        c.momentum = 0.75f; c.gamma = 0.4f; c.beta = 0.6f;
        return Model::Create(c);
    }
    static void fill(Model &m, int I, int O, int flags, std::string const &prefix)
    {
        m.SetInputShape({(bb::index_t)I});
        put_wiring(m, O, read_raw<std::int32_t>(prefix + ".idx", (size_t)O * 6));
        auto W = read_raw<float>(prefix + ".params", (size_t)O * 64);
        { auto p = m.lock_W(); for (size_t k = 0; k < W.size(); ++k) { p[(bb::index_t)k] = W[k]; } }
        auto mean = read_raw<float>(prefix + ".mean", (size_t)O), var = read_raw<float>(prefix + ".var", (size_t)O);
        { auto p = m.lock_mean(); for (int o = 0; o < O; ++o) { p[o] = mean[(size_t)o]; } }
        { auto p = m.lock_var();  for (int o = 0; o < O; ++o) { p[o] = var[(size_t)o]; } }
        m.SendCommand(std::string("lut_binarize ") + ((flags & 2) ? "true" : "false"));
    }
    static void take_apart(Model const &m, std::string const &prefix)
    {
        size_t const O = (size_t)m.GetOutputNodeSize();
        write_raw(prefix + ".idx", get_wiring(m));
        std::vector<float> W(O * 64), mean(O), var(O);
        { auto p = m.lock_W_const(); for (size_t k = 0; k < W.size(); ++k) { W[k] = p[(bb::index_t)k]; } }
        { auto p = m.lock_mean_const(); for (size_t o = 0; o < O; ++o) { mean[o] = p[(bb::index_t)o]; } }
        { auto p = m.lock_var_const();  for (size_t o = 0; o < O; ++o) { var[o] = p[(bb::index_t)o]; } }
        write_raw(prefix + ".params", W); write_raw(prefix + ".mean", mean); write_raw(prefix + ".var", var);
    }
};

struct Binary {
    using Model = bb::BinaryLutN<6, bb::Bit, float>;
    static std::shared_ptr<Model> blank(int O) { return Model::Create((bb::index_t)O); }
    static void fill(Model &m, int I, int O, int, std::string const &prefix)
    {
        m.SetInputShape({(bb::index_t)I});
        put_wiring(m, O, read_raw<std::int32_t>(prefix + ".idx", (size_t)O * 6));
        auto table = read_raw<std::int32_t>(prefix + ".params", (size_t)O * 2);
        for (int o = 0; o < O; ++o) { for (int b = 0; b < 64; ++b) { m.SetLutTable(o, b, ((table[(size_t)o * 2 + b / 32] >> (b % 32)) & 1) != 0); } }
    }
    static void take_apart(Model const &m, std::string const &prefix)
    {
        int const O = (int)m.GetOutputNodeSize();
        write_raw(prefix + ".idx", get_wiring(m));
        std::vector<std::int32_t> table((size_t)O * 2, 0);
        for (int o = 0; o < O; ++o) { for (int b = 0; b < 64; ++b) { if (m.GetLutTable(o, b)) { table[(size_t)o * 2 + b / 32] |= (std::int32_t)(1u << (b % 32)); } } }
        write_raw(prefix + ".params", table);
    }
};

template <class K, class MakeModel>
static int run(std::string const &cmd, char **a, MakeModel make_model)
{
    if (cmd == "make") {
        int const I = std::atoi(a[0]), O = std::atoi(a[1]), flags = std::atoi(a[2]);
        std::string const name = a[3], prefix = a[4], out = a[5];
        auto m = make_model(O, flags);
        if (name != "-") { m->SetName(name); }
        K::fill(*m, I, O, flags, prefix);
        return m->DumpToFile(out) ? 0 : 1;
    }
    auto m = K::blank(1);
    if (!m->LoadFromFile(a[0])) { std::fprintf(stderr, "cannot open %s\n", a[0]); return 1; }
    if (cmd == "roundtrip") { return m->DumpToFile(a[1]) ? 0 : 1; }
    if (cmd == "describe") {
        K::take_apart(*m, a[1]);
        std::printf("%d %d %s\n", (int)m->GetInputNodeSize(), (int)m->GetOutputNodeSize(), m->GetName().c_str());
        return 0;
    }
    std::fprintf(stderr, "unknown command %s\n", cmd.c_str());
    return 1;
}

// object_tool wiring <kind> <seed> <policy|-> <dims> <input shape ...> <output shape ...> <prefix>
static int wiring(int argc, char **argv)
{
    if (argc < 6) { std::fprintf(stderr, "usage: object_tool wiring <kind> <seed> <policy|-> <dims> <shapes ...> <prefix>\n"); return 1; }
    int const kind = std::atoi(argv[2]);
    std::uint64_t const seed = std::strtoull(argv[3], nullptr, 10);
    std::string const policy = std::string(argv[4]) == "-" ? "" : argv[4];
    int const dims = std::atoi(argv[5]);
    if (dims < 1 || argc != 6 + 2 * dims + 1) { std::fprintf(stderr, "wiring: %d shape entries and a prefix expected\n", 2 * dims); return 1; }
    bb::indices_t in((size_t)dims), out((size_t)dims);
    for (int i = 0; i < dims; ++i) { in[(size_t)i] = std::atoll(argv[6 + i]); out[(size_t)i] = std::atoll(argv[6 + dims + i]); }
    std::string const prefix = argv[6 + 2 * dims];
    bb::index_t const O = bb::CalcShapeSize(out);
    std::vector<std::int32_t> idx((size_t)O * 6);
    if (kind == 0) {
        bb::FixedSizeConnectionTable<6> tbl;
        tbl.SetShape(in, out);
        tbl.InitializeConnection(seed, policy);
        for (bb::index_t o = 0; o < O; ++o) { for (int i = 0; i < 6; ++i) { idx[(size_t)o * 6 + i] = (std::int32_t)tbl.GetInputConnection(o, i); } }
    }
    else if (kind == 3) {           // a whole StochasticLutN created with the seed: its generator's first draw seeds the table
        auto lut = bb::StochasticLutN<6, float, float>::Create(out, policy, seed);
        lut->SetInputShape(in);
        idx = get_wiring(*lut);
    }
    else {
        bb::BinaryLutN<6, bb::Bit>::create_t create;
        create.output_shape = out; create.connection = policy; create.seed = seed;
        auto lut = bb::BinaryLutN<6, bb::Bit>::Create(create);
        lut->SetInputShape(in);
        idx = get_wiring(*lut);
        std::vector<std::int32_t> table((size_t)O * 2, 0);
        for (bb::index_t o = 0; o < O; ++o) {
            for (int b = 0; b < 64; ++b) { if (lut->GetLutTable(o, b)) { table[(size_t)o * 2 + b / 32] = (std::int32_t)((std::uint32_t)table[(size_t)o * 2 + b / 32] | (1u << (b % 32))); } }
        }
        write_raw(prefix + ".params", table);
    }
    write_raw(prefix + ".idx", idx);
    return 0;
}

int main(int argc, char **argv)
{
    if (argc < 4) { std::fprintf(stderr, "usage: object_tool make|roundtrip|describe|wiring <kind> ... | reload <in> <out>\n"); return 1; }
    bb::Manager::SetHostOnly(true);             // serialization is host work; no device is touched
    std::string const cmd = argv[1];
    if (cmd == "reload") {
        // object_tool reload <in> <out>: any object this library knows, rebuilt from the type names in the file, written again
        auto obj = bb::Object_LoadFromFile(argv[2]);
        if (!obj) { std::fprintf(stderr, "cannot load %s\n", argv[2]); return 1; }
        if (auto m = std::dynamic_pointer_cast<bb::Model>(obj)) {
            std::printf("%s %s in %d out %d\n", m->GetObjectName().c_str(), m->GetName().c_str(), (int)m->GetInputNodeSize(), (int)m->GetOutputNodeSize());
        }
        return obj->DumpToFile(argv[3]) ? 0 : 1;
    }
    if (argc < 6) { std::fprintf(stderr, "usage: object_tool make|roundtrip|describe|wiring <kind> ...\n"); return 1; }
    if (cmd == "wiring") {
        try { return wiring(argc, argv); }
        catch (std::exception const &e) { std::fprintf(stderr, "rejected: %s\n", e.what()); return 1; }
    }
    int const kind = std::atoi(argv[2]), bit = std::atoi(argv[3]);
    char **rest = argv + 4;
    try {
        if (kind == 0 && !bit) { return run<Stochastic<float>>(cmd, rest, [](int O, int) { return Stochastic<float>::blank(O); }); }
        if (kind == 0 && bit)  { return run<Stochastic<bb::Bit>>(cmd, rest, [](int O, int) { return Stochastic<bb::Bit>::blank(O); }); }
        if (kind == 1 && !bit) { return run<Differentiable<float>>(cmd, rest, [](int O, int f) { return Differentiable<float>::configured(O, f); }); }
        if (kind == 1 && bit)  { return run<Differentiable<bb::Bit>>(cmd, rest, [](int O, int f) { return Differentiable<bb::Bit>::configured(O, f); }); }
        if (kind == 2)         { return run<Binary>(cmd, rest, [](int O, int) { return Binary::blank(O); }); }
        std::fprintf(stderr, "unknown kind %d\n", kind);
        return 1;
    }
    catch (std::exception const &e) {
        std::fprintf(stderr, "rejected: %s\n", e.what());
        return 1;
    }
}

// CPU test of the host-side plumbing (no device needed): frame-buffer layout and bit packing, tensors, the connection
// table and its reverse table against the oracle, command handling, and the refusal to run without a device.
#include <cstdio>
#include <map>
#include <set>
#include <sstream>
#include <vector>

#include "bb/StochasticLutN.h"
#include "bb/DifferentiableLutN.h"
#include "bb/BinaryLutN.h"
#include "bb/ObjectLoader.h"
#include "bb/BinaryModulation.h"
#include "bb/DifferentiableLutDiscreteN.h"
#include "bb/MaxPooling.h"
#include "bb/UpSampling.h"
#include "bb/Shuffle.h"
#include "../../binarybrain_amd/csrc/tile_divisor.hpp"

extern "C" int oracle_ReverseTable(int n, std::int32_t const *idx, int input_node_size, int output_node_size, std::int32_t *rev, int rev_cap);

static int g_fail = 0;
#define CHECK(cond) do { if (!(cond)) { ++g_fail; std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond); } } while (0)

int main(void)
{
    bb::Manager::SetHostOnly(true);
    CHECK(!bb::Manager::IsDeviceAvailable());

    // frame buffer: node-major rows, stride a 256-byte multiple and never a 2 KiB multiple
    {
        bb::FrameBuffer buf(100, {3, 5}, BB_TYPE_FP32, true);
        CHECK(buf.GetNodeSize() == 15 && buf.GetFrameSize() == 100 && buf.GetFrameStride() == 512);
        CHECK(bb::FrameBuffer::CalcFrameStride(BB_TYPE_FP32, 8192) == 32768 + 512);
        CHECK(bb::FrameBuffer::CalcFrameStride(BB_TYPE_BIT, 262144) == 32768 + 384);
        CHECK(bb::FrameBuffer::CalcFrameStride(BB_TYPE_BIT, 1) == 256);
        buf.SetFP32(99, 14, 3.5f);
        buf.SetFP32(0, 0, -1.0f);
        CHECK(buf.GetFP32(99, 14) == 3.5f && buf.GetFP32(0, 0) == -1.0f);
        auto p = buf.LockConst<float>();
        CHECK(p.GetAddr(14)[99] == 3.5f);
        CHECK((char const *)p.GetAddr(1) - (char const *)p.GetAddr(0) == 512);
        bb::FrameBuffer alias = buf;                       // copies share storage, as in the reference
        alias.SetFP32(1, 1, 7.0f);
        CHECK(buf.GetFP32(1, 1) == 7.0f);
    }
    // packed bits: frame f is bit f & 7 of byte f >> 3 (bit f & 31 of little-endian word f >> 5)
    {
        bb::FrameBuffer buf(70, {4}, BB_TYPE_BIT, true);
        buf.FillZero();
        buf.SetBit(0, 2, true); buf.SetBit(33, 2, true); buf.SetBit(69, 2, true);
        auto p = buf.LockConst<bb::Bit>();
        std::uint32_t const *w = reinterpret_cast<std::uint32_t const *>(p.GetAddr(2));
        CHECK(w[0] == 1u && w[1] == 2u && w[2] == (1u << 5));
        CHECK(buf.GetBit(33, 2) && !buf.GetBit(34, 2) && !buf.GetBit(33, 1));
        buf.SetBit(33, 2, false);
        CHECK(!buf.GetBit(33, 2));
        bool threw = false;
        try { buf.Lock<float>(); } catch (bb::Exception const &) { threw = true; }
        CHECK(threw);                                      // typed access checks the element type
    }
    // tensors
    {
        bb::Tensor_<float> t(bb::indices_t({4, 8}), true);
        t = 0.25f;
        auto p = t.Lock();
        p(3, 7) = 1.0f;
        CHECK(p[31] == 1.0f && p(0, 0) == 0.25f && t.GetSize() == 32);
        bb::Tensor w({16, 64}, BB_TYPE_FP32, true);
        w.InitNormalDistribution(0.5, 0.01, 1);
        double s = 0; { auto q = w.LockConst<float>(); for (int i = 0; i < 1024; ++i) { s += q[i]; } }
        CHECK(std::abs(s / 1024 - 0.5) < 0.01);
    }
    // connection table: distinct inputs per node, balanced use of inputs, reverse table equal to the oracle's
    for (std::string policy : {"", "random", "serial"}) {
        int const I = 50, O = 37;
        bb::FixedSizeConnectionTable<6> tbl;
        tbl.SetShape({I}, {O});
        tbl.InitializeConnection(3, policy);
        std::vector<std::int32_t> idx((size_t)O * 6);
        std::map<int, int> use;
        for (int o = 0; o < O; ++o) {
            std::set<int> seen;
            for (int i = 0; i < 6; ++i) { int v = (int)tbl.GetInputConnection(o, i); CHECK(v >= 0 && v < I); seen.insert(v); use[v]++; idx[(size_t)o * 6 + i] = v; }
            CHECK(seen.size() == 6);
        }
        int lo = 1 << 30, hi = 0;
        for (int v = 0; v < I; ++v) { lo = std::min(lo, use[v]); hi = std::max(hi, use[v]); }
        CHECK(hi - lo <= 2);                               // every input used about equally often
        int const stride = oracle_ReverseTable(6, idx.data(), I, O, nullptr, 0);
        std::vector<std::int32_t> rev((size_t)I * stride);
        oracle_ReverseTable(6, idx.data(), I, O, rev.data(), (int)rev.size());
        CHECK(tbl.GetReverseTableStride() == stride);
        auto p = tbl.LockConst_ReverseTable();
        bool same = true;
        for (int r = 0; r < I; ++r) for (int c = 0; c < stride; ++c) { same = same && (p(r, c) == rev[(size_t)r * stride + c]); }
        CHECK(same);
        tbl.SetInputConnection(0, 0, (tbl.GetInputConnection(0, 0) + 1) % I);     // editing the wiring rebuilds the reverse table
        idx[0] = (std::int32_t)tbl.GetInputConnection(0, 0);
        int const stride2 = oracle_ReverseTable(6, idx.data(), I, O, nullptr, 0);
        std::vector<std::int32_t> rev2((size_t)I * stride2);
        oracle_ReverseTable(6, idx.data(), I, O, rev2.data(), (int)rev2.size());
        auto p2 = tbl.LockConst_ReverseTable();
        same = (tbl.GetReverseTableStride() == stride2);
        for (int r = 0; same && r < I; ++r) for (int c = 0; c < stride2; ++c) { same = same && (p2(r, c) == rev2[(size_t)r * stride2 + c]); }
        CHECK(same);
    }
    // models: shapes, parameters, commands, ForwardNode, and no silent host execution
    {
        auto lut = bb::StochasticLutN<6, float>::Create(10);
        CHECK(lut->GetModelName() == "StochasticLut6");
        CHECK(lut->SetInputShape({4, 5}) == bb::indices_t({10}));
        CHECK(lut->GetInputNodeSize() == 20 && lut->GetOutputNodeSize() == 10);
        CHECK(lut->GetParameters().GetSize() == 1 && lut->GetGradients().GetSize() == 1);
        CHECK(lut->W().GetShape() == bb::indices_t({10, 64}));
        { auto W = lut->lock_W(); for (int i = 0; i < 64; ++i) { W(3, i) = (i == 37) ? 0.9f : 0.1f; } }
        std::vector<double> in(6);
        for (int b = 0; b < 6; ++b) { in[(size_t)b] = (37 >> b) & 1; }
        CHECK(lut->ForwardNode(3, in)[0] == 1.0);                                // lut_binarize is on by default
        lut->SendCommand("lut_binarize false");
        CHECK(std::abs(lut->ForwardNode(3, in)[0] - 0.9) < 1e-6);
        in[0] = 1.0 - in[0];
        CHECK(std::abs(lut->ForwardNode(3, in)[0] - 0.1) < 1e-6);
        bool threw = false;
        try { lut->Forward(bb::FrameBuffer(8, {4, 5}, BB_TYPE_FP32, true)); } catch (bb::Exception const &) { threw = true; }
        CHECK(threw);
        auto dl = bb::DifferentiableLutN<6, bb::Bit>::Create(12);
        CHECK(dl->GetModelName() == "DifferentiableLut6");
        dl->SetInputShape({30});
        CHECK(dl->GetParameters().GetSize() == 1);
        dl->SendCommand("parameter_lock true");
        CHECK(dl->GetParameters().GetSize() == 0);
        { auto v = dl->lock_var_const(); auto m = dl->lock_mean_const(); CHECK(v[0] == 1.0f && m[11] == 0.0f); }
        auto bl = bb::BinaryLutN<6, bb::Bit>::Create(5);
        bl->SetInputShape({9});
        bl->SetLutTable(2, 40, true);  CHECK(bl->GetLutTable(2, 40));
        bl->SetLutTable(2, 40, false); CHECK(!bl->GetLutTable(2, 40));
        std::set<bb::index_t> seen;
        for (int i = 0; i < 6; ++i) { seen.insert(bl->GetNodeConnectionIndex(4, i)); }
        CHECK(seen.size() == 6);
        CHECK(bl->Backward(bb::FrameBuffer(8, {5}, BB_TYPE_FP32, true)).GetNodeSize() == 9);
    }
    // serialization, in the shape of the reference's tests (tests/gtest/DifferentiableLutTest.cpp:10-53: dump, load into a
    // fresh layer, compare; tests/gtest/ObjectTest.cpp:191-216: reconstruct by the recorded name)
    {
        auto lut0 = bb::DifferentiableLutN<6, float>::Create(16);
        lut0->SetInputShape({16});
        { auto W = lut0->lock_W(); W(5, 9) = 0.125f; }
        { auto v = lut0->lock_var(); v[3] = 2.5f; }
        std::stringstream ss(std::ios::in | std::ios::out | std::ios::binary);
        lut0->DumpObject(ss);
        auto lut1 = bb::DifferentiableLutN<6, float>::Create(16);
        lut1->LoadObject(ss);
        CHECK(lut0->GetGamma() == lut1->GetGamma() && lut0->GetBeta() == lut1->GetBeta());
        CHECK(lut0->GetOutputShape() == lut1->GetOutputShape() && lut0->GetInputShape() == lut1->GetInputShape());
        bool same = true;
        for (bb::index_t o = 0; o < lut0->GetOutputNodeSize(); ++o) {
            for (bb::index_t i = 0; i < lut0->GetNodeConnectionSize(o); ++i) { same = same && (lut0->GetNodeConnectionIndex(o, i) == lut1->GetNodeConnectionIndex(o, i)); }
        }
        CHECK(same);
        { auto a = lut0->lock_W_const(); auto b = lut1->lock_W_const(); for (int k = 0; k < 16 * 64; ++k) { same = same && (a[k] == b[k]); } }
        { auto v = lut1->lock_var_const(); same = same && (v[3] == 2.5f) && (v[4] == 1.0f); }
        CHECK(same);
        CHECK(lut1->GetGradients().GetSize() == 1 && lut1->dW().GetShape() == bb::indices_t({16, 64}));

        auto model = bb::DifferentiableLutN<6, bb::Bit, float>::Create(bb::indices_t({1, 2, 3}));
        model->SetInputShape({32, 8});
        CHECK(model->GetObjectName() == "DifferentiableLut6_bit_fp32");
        std::stringstream s2(std::ios::in | std::ios::out | std::ios::binary);
        model->DumpObject(s2);
        auto obj = std::dynamic_pointer_cast<bb::DifferentiableLutN<6, bb::Bit, float>>(bb::Object_Load(s2));
        CHECK((bool)obj);
        if (obj) {
            CHECK(obj->GetObjectName() == model->GetObjectName());
            CHECK(obj->GetInputShape() == bb::indices_t({32, 8}) && obj->GetOutputShape() == bb::indices_t({1, 2, 3}));
        }
        // a layer of another class or width does not load into this one, and a name nobody knows reconstructs to nothing
        std::stringstream s3(std::ios::in | std::ios::out | std::ios::binary);
        model->DumpObject(s3);
        bool threw = false;
        try { bb::StochasticLutN<6, bb::Bit>::Create(6)->LoadObject(s3); } catch (bb::Exception const &) { threw = true; }
        CHECK(threw);
        std::stringstream s4(std::ios::in | std::ios::out | std::ios::binary);
        s4.write("BB_OBJ", 6); bb::SaveValue(s4, (std::int64_t)1); bb::SaveValue(s4, std::string("NoSuchLayer"));
        CHECK(!bb::Object_Load(s4));
        // tensors on their own
        bb::Tensor_<std::int32_t> t(bb::indices_t({2, 3}), true);
        { auto p = t.Lock(); for (int k = 0; k < 6; ++k) { p[k] = k + 1; } }
        std::stringstream s5(std::ios::in | std::ios::out | std::ios::binary);
        t.DumpObject(s5);
        auto t2 = std::dynamic_pointer_cast<bb::Tensor_<std::int32_t>>(bb::Object_Load(s5));
        CHECK(t2 && t2->GetShape() == bb::indices_t({2, 3}));
        if (t2) { auto p = t2->LockConst(); CHECK(p(1, 1) == 5 && p(1, 2) == 6); }          // ObjectTest.cpp:185-186
    }
    // the layers around the LUT layers: shapes, commands, refusals, and the device path's refusal without a device
    {
        auto r2b = bb::RealToBinary<bb::Bit>::Create(7, 3);
        CHECK(r2b->SetInputShape({2, 4, 5}) == bb::indices_t({6, 4, 5}) && r2b->GetInputNodeSize() == 40 && r2b->GetOutputNodeSize() == 120);
        CHECK(r2b->GetObjectName() == "RealToBinary_bit_fp32" && r2b->GetModulationSize() == 7);
        bool threw = false;
        try { bb::RealToBinary<float>::Create(2, std::make_shared<bb::Tensor>()); } catch (bb::Exception const &) { threw = true; }
        CHECK(threw);                                                   // thresholds from a value generator are not provided
        auto b2r = bb::BinaryToReal<bb::Bit>::Create(7, bb::indices_t({10}));
        CHECK(b2r->SetInputShape({70}) == bb::indices_t({10}));
        auto by_depth = bb::BinaryToReal<float>::Create(1, 7);
        CHECK(by_depth->SetInputShape({70, 2}) == bb::indices_t({10, 2}));
        threw = false;
        try { bb::BinaryToReal<float>::Create(1, bb::indices_t({9}))->SetInputShape({70}); } catch (bb::Exception const &) { threw = true; }
        CHECK(threw);                                                   // 70 inputs do not fold into 9 outputs
        auto pool = bb::MaxPooling<bb::Bit>::Create(2, 3);
        CHECK(pool->SetInputShape({4, 5, 7}) == bb::indices_t({4, 3, 3}) && pool->GetFilterHeight() == 2 && pool->GetFilterWidth() == 3);
        auto up = bb::UpSampling<>::Create(2, 3, false);
        CHECK(up->SetInputShape({4, 5, 7}) == bb::indices_t({4, 10, 21}) && up->GetOutputNodeSize() == 840);
        auto shuffle = bb::Shuffle::Create(3, bb::indices_t({2, 6}));
        CHECK(shuffle->SetInputShape({12}) == bb::indices_t({2, 6}) && shuffle->SetInputShape({6}) == bb::indices_t({6}));
        {
            std::stringstream ss(std::ios::in | std::ios::out | std::ios::binary);
            shuffle->DumpObject(ss);
            auto back = std::dynamic_pointer_cast<bb::Model>(bb::Object_Load(ss));
            CHECK((bool)back && back->GetObjectName() == "Shuffle" && back->GetOutputShape() == bb::indices_t({6}));
        }
        threw = false;
        try { bb::Shuffle::Create(4)->SetInputShape({6}); } catch (bb::Exception const &) { threw = true; }
        CHECK(threw);                                                   // 6 nodes do not split into units of 4
        {   // the stamp that says whether a tensor could have been written to since it was last looked at
            bb::Tensor_<float> t(bb::indices_t({4}));
            { auto w = t.Lock(true); w[0] = 1.0f; }
            auto const s0 = t.WriteStamp();
            { auto r = t.LockConst(); CHECK(r[0] == 1.0f); }
            CHECK(t.WriteStamp() == s0);                                // reading does not move it
            { auto w = t.Lock(); w[1] = 2.0f; }
            CHECK(t.WriteStamp() != s0);                                // a writable lock does
            auto const s1 = t.WriteStamp();
            t.Resize(bb::indices_t({8}));
            CHECK(t.WriteStamp() != s1);                                // and so does a new block
        }
        auto tanh = bb::HardTanh<>::Create(0.0f, 1.0f);
        CHECK(tanh->ForwardNode(0, {-0.5, 0.25, 2.0}) == std::vector<double>({0.0, 0.25, 1.0}));
        tanh->SendCommand("binary true");
        CHECK(tanh->ForwardNode(0, {0.4, 0.6}) == std::vector<double>({0.0, 1.0}));
        auto body = bb::Sequential::Create();
        body->Add(bb::DifferentiableLutN<6, bb::Bit>::Create((bb::index_t)36));
        body->Add(bb::DifferentiableLutDiscreteN<6, bb::Bit>::Create((bb::index_t)12));
        auto net = bb::BinaryModulation<bb::Bit>::Create(body, 7, 15);
        CHECK(net->SetInputShape({20}) == bb::indices_t({12}) && net->GetInputNodeSize() == 20 && net->GetLayer() == body);
        CHECK(net->GetParameters().GetSize() == 2 && net->GetGradients().GetSize() == 2);
        std::stringstream ss(std::ios::in | std::ios::out | std::ios::binary);
        net->DumpObject(ss);
        auto again = std::dynamic_pointer_cast<bb::Model>(bb::Object_Load(ss));
        CHECK((bool)again && again->GetObjectName() == "BinaryModulation_bit_fp32" && again->GetOutputNodeSize() == 12);
        std::stringstream s1(std::ios::in | std::ios::out | std::ios::binary), s2(std::ios::in | std::ios::out | std::ios::binary);
        net->DumpObject(s1);
        if (again) { again->DumpObject(s2); CHECK(s1.str() == s2.str()); }
        bb::FrameBuffer x(8, {20}, BB_TYPE_FP32, true);
        threw = false;
        try { net->Forward(x); } catch (bb::Exception const &) { threw = true; }
        CHECK(threw);                                                   // no device: the layers refuse instead of computing on the host
    }
    // workgroup index -> (frame chunk, node tile) without an integer division: exact for every index below 2^31
    {
        int const divisors[] = {1, 2, 3, 5, 7, 64, 255, 256, 257, 1000, 1024, 1536, 4096, 65535, 1 << 20, (1 << 20) + 1, 0x3fffffff, 0x7fffffff};
        std::uint64_t state = 0x9e3779b97f4a7c15ull;
        for (int d : divisors) {
            bbhip::TileDivisor const t = bbhip::make_tile_divisor(d);
            auto check = [&](std::uint32_t n) {
                int outer, tile;
                bbhip::split_tile((int)n, t, outer, tile);
                if (outer != (int)(n / (std::uint32_t)d) || tile != (int)(n % (std::uint32_t)d)) { CHECK(!"split_tile"); }
            };
            for (std::uint32_t n = 0; n < 70000; ++n) { check(n); }
            for (std::uint32_t k = 1; k < 200; ++k) {                 // around multiples of d and at the top of the range
                std::uint64_t const m = (std::uint64_t)k * (std::uint64_t)d;
                if (m < 0x7fffffffull) { check((std::uint32_t)m); check((std::uint32_t)m - 1); check((std::uint32_t)m + 1 < 0x80000000u ? (std::uint32_t)m + 1 : 0); }
                check(0x7fffffffu - k);
            }
            for (int i = 0; i < 200000; ++i) {
                state ^= state << 13; state ^= state >> 7; state ^= state << 17;
                check((std::uint32_t)(state >> 33));
            }
            check(0x7fffffffu);
        }
    }

    std::printf("%s (%d failed checks)\n", g_fail ? "FAILED" : "OK", g_fail);
    return g_fail ? 1 : 0;
}

// Seeded wiring policies of the sparse layers: which input nodes each output node reads.
//
// Policies and their random draws follow the reference so that a layer built here from the same seed, shapes and policy
// string is wired exactly like one built there (given the same C++ standard library, whose std::shuffle and
// std::normal_distribution the draws go through): include/bb/ConnectionTable.h:150-284 for the layers that keep a
// FixedSizeConnectionTable (StochasticLutN, DifferentiableLutN), include/bb/SparseModel.h:97-233 for BinaryLutN, and
// include/bb/ShuffleSet.h:26-103 for the dealing of input nodes.
//
//   ""/"random"  every input node is dealt from a shuffled deck that is reshuffled when it runs out, so all inputs are used
//                about equally often and the inputs of one node are distinct;
//   "serial"     output node o reads inputs o*n, o*n + 1, ... (mod the input node count);
//   "pointwise"  3-d shapes with equal spatial extents: a node reads channels of its own pixel only (one deck per pixel);
//   "depthwise"  3-d shapes with equal channel count: a node reads pixels of its own channel only (one deck per channel);
//   "gauss"      inputs drawn around the node's own position scaled into the input shape, normally distributed with
//                sigma = input extent / output extent per axis, wrapped around the edges, distinct per node.
// Any other policy string is an error.
#pragma once

#include <algorithm>
#include <cctype>
#include <cstdint>
#include <random>
#include <set>
#include <string>
#include <vector>

#include "bb/Core.h"

namespace bb {

// Dealer of the indices 0 .. size-1: a shuffled deck (`m_deck`, dealt from `m_next` on), the cards that earlier hands have
// used (`m_used`) and, during a hand, the cards of that hand (`hand`).  When the deck runs out it is refilled with the
// reshuffled used cards, and if there are none (a hand larger than the deck) with the reshuffled cards of the hand itself.
template <typename INDEX>
class ShuffleSet {
    std::mt19937_64     m_mt;
    std::vector<INDEX>  m_deck;
    std::size_t         m_next = 0;
    std::vector<INDEX>  m_used;

    void Refill(std::vector<INDEX> &from)
    {
        m_deck.assign(from.begin(), from.end());
        std::shuffle(m_deck.begin(), m_deck.end(), m_mt);
        m_next = 0;
        from.clear();
    }

public:
    ShuffleSet() {}
    ShuffleSet(INDEX size, std::uint64_t seed = 1) { Setup(size, seed); }

    void Setup(INDEX size, std::uint64_t seed = 1)
    {
        m_mt.seed(seed);
        m_used.clear();
        m_deck.resize((std::size_t)size);
        for (std::size_t i = 0; i < m_deck.size(); ++i) { m_deck[i] = (INDEX)i; }
        std::shuffle(m_deck.begin(), m_deck.end(), m_mt);
        m_next = 0;
    }

    std::vector<INDEX> GetRandomSet(INDEX n)
    {
        std::vector<INDEX> hand;
        std::vector<INDEX> recycled;        // what the hand holds since the deck was last refilled from it
        for (INDEX i = 0; i < n; ++i) {
            if (m_next >= m_deck.size()) { Refill(m_used); }
            if (m_next >= m_deck.size()) { Refill(recycled); }
            BB_ASSERT(m_next < m_deck.size());
            INDEX const card = m_deck[m_next++];
            hand.push_back(card);
            recycled.push_back(card);
        }
        m_used.insert(m_used.end(), recycled.begin(), recycled.end());
        return hand;
    }
};

namespace connection_policy {

inline std::vector<std::string> Words(std::string const &text)
{
    std::vector<std::string> out;
    std::string w;
    for (char ch : text) {
        if (std::isspace((unsigned char)ch)) { if (!w.empty()) { out.push_back(w); w.clear(); } }
        else { w.push_back(ch); }
    }
    if (!w.empty()) { out.push_back(w); }
    return out;
}

// row-major position of `indices` in `shape` (last index fastest)
inline index_t Flatten(indices_t const &indices, indices_t const &shape)
{
    index_t pos = 0;
    for (std::size_t i = 0; i < shape.size(); ++i) { pos = pos * shape[i] + indices[i]; }
    return pos;
}

// Which axis of a 3-d shape counts channels.  The connection-table layers keep (channel, y, x) (ConnectionTable.h:160-212),
// BinaryLutN's base class keeps (x, y, channel) (SparseModel.h:109-157); the walk over the output nodes differs accordingly.
enum class Layout { kChannelFirst, kChannelLast };

// set(output_node, connection, input_node) is called once for every connection of every output node.
template <typename SetFn>
void Initialize(std::uint64_t seed, std::string const &policy, indices_t const &input_shape, indices_t const &output_shape, int n,
                Layout layout, SetFn set)
{
    index_t const input_nodes = CalcShapeSize(input_shape), output_nodes = CalcShapeSize(output_shape);
    std::vector<std::string> const argv = Words(policy);
    std::string const rule = argv.empty() ? "random" : argv[0];
    bool const first = (layout == Layout::kChannelFirst);
    int const ch = first ? 0 : 2, ax = first ? 2 : 0;           // channel axis and x axis (y is axis 1 in both layouts)

    if (rule == "pointwise") {
        BB_ASSERT(input_shape.size() == 3 && output_shape.size() == 3);
        BB_ASSERT(input_shape[1] == output_shape[1] && input_shape[(std::size_t)ax] == output_shape[(std::size_t)ax]);
        std::mt19937_64 mt(seed);
        for (index_t y = 0; y < output_shape[1]; ++y) {
            for (index_t x = 0; x < output_shape[(std::size_t)ax]; ++x) {
                ShuffleSet<index_t> deck(input_shape[(std::size_t)ch], mt());      // the channels of this pixel
                for (index_t c = 0; c < output_shape[(std::size_t)ch]; ++c) {
                    auto const hand = deck.GetRandomSet(n);
                    indices_t out(3), in(3);
                    out[(std::size_t)ch] = c; out[1] = y; out[(std::size_t)ax] = x;
                    in[1] = y; in[(std::size_t)ax] = x;
                    for (int i = 0; i < n; ++i) {
                        in[(std::size_t)ch] = hand[(std::size_t)i];
                        set(Flatten(out, output_shape), i, Flatten(in, input_shape));
                    }
                }
            }
        }
        return;
    }
    if (rule == "depthwise") {
        BB_ASSERT(input_shape.size() == 3 && output_shape.size() == 3);
        BB_ASSERT(input_shape[(std::size_t)ch] == output_shape[(std::size_t)ch]);
        index_t const in_w = input_shape[(std::size_t)ax];
        std::mt19937_64 mt(seed);
        for (index_t c = 0; c < output_shape[(std::size_t)ch]; ++c) {
            ShuffleSet<index_t> deck(input_shape[1] * in_w, mt());                 // the pixels of this channel
            for (index_t y = 0; y < output_shape[1]; ++y) {
                for (index_t x = 0; x < output_shape[(std::size_t)ax]; ++x) {
                    auto const hand = deck.GetRandomSet(n);
                    indices_t out(3), in(3);
                    out[(std::size_t)ch] = c; out[1] = y; out[(std::size_t)ax] = x;
                    in[(std::size_t)ch] = c;
                    for (int i = 0; i < n; ++i) {
                        in[1] = hand[(std::size_t)i] / in_w;
                        in[(std::size_t)ax] = hand[(std::size_t)i] % in_w;
                        set(Flatten(out, output_shape), i, Flatten(in, input_shape));
                    }
                }
            }
        }
        return;
    }
    if (rule == "gauss") {
        BB_ASSERT(input_shape.size() == output_shape.size());
        std::size_t const dims = input_shape.size();
        std::vector<double> step(dims), sigma(dims);
        for (std::size_t d = 0; d < dims; ++d) {
            // (an output extent of 1 would divide by zero in the reference; its only node then sits at position 0)
            step[d]  = output_shape[d] > 1 ? (double)(input_shape[d] - 1) / (double)(output_shape[d] - 1) : 0.0;
            sigma[d] = (double)input_shape[d] / (double)output_shape[d];
        }
        std::mt19937_64 mt(seed);
        std::normal_distribution<double> gauss(0.0, 1.0);
        indices_t out(dims, 0);
        for (;;) {
            index_t const node = Flatten(out, output_shape);
            std::set<index_t> taken;
            for (int i = 0; i < n; ++i) {
                for (;;) {
                    indices_t in(dims);
                    std::vector<double> pos(dims);
                    for (std::size_t d = 0; d < dims; ++d) { pos[d] = (double)out[d] * step[d] + gauss(mt) * sigma[d]; }
                    // wrap around: negatives are lifted by whole extents, then the integer part is taken modulo the extent
                    for (std::size_t d = dims; d-- > 0;) {
                        while (pos[d] < 0) { pos[d] += (double)input_shape[d]; }
                        in[d] = (index_t)pos[d] % input_shape[d];
                    }
                    index_t const candidate = Flatten(in, input_shape);
                    if (taken.insert(candidate).second) { set(node, i, candidate); break; }
                }
            }
            // next output position, last axis fastest
            std::size_t d = dims;
            while (d-- > 0) { if (++out[d] < output_shape[d]) { break; } out[d] = 0; }
            if (d == (std::size_t)-1) { break; }
        }
        return;
    }
    if (rule == "serial") {
        index_t in = 0;
        for (index_t o = 0; o < output_nodes; ++o) {
            for (int i = 0; i < n; ++i) { set(o, i, in % input_nodes); ++in; }
        }
        return;
    }
    if (rule == "random") {
        ShuffleSet<index_t> deck(input_nodes, seed);
        for (index_t o = 0; o < output_nodes; ++o) {
            auto const hand = deck.GetRandomSet(n);
            for (int i = 0; i < n; ++i) { set(o, i, hand[(std::size_t)i]); }
        }
        return;
    }
    throw Exception("unknown connection rule: \"" + rule + "\"");
}

}  // namespace connection_policy
}  // namespace bb

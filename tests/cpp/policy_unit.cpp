// Replays the reference's own unit tests of the prefix tree
// (crates/retrograd-infer/src/kv.rs:558-700) and of the incremental
// detokenizer (crates/retrograd-infer/src/detok.rs:134-210) on the product's
// C++ classes. Every expected value is the reference's. Exits 0 when all hold.
#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "../../retrograd_amd/csrc/sched/detok.hpp"
#include "../../retrograd_amd/csrc/sched/prefix_tree.hpp"

using namespace sched;

static int g_failed = 0;
#define CHECK(cond) do { if (!(cond)) { std::fprintf(stderr, "FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); ++g_failed; } } while (0)

using V = std::vector<int32_t>;

static PrefixTree tree_with(const std::vector<V> & paths) {
    PrefixTree tree;
    for (size_t i = 0; i < paths.size(); ++i) tree.insert(0, paths[i].data(), paths[i].size(), (int32_t)(i + 1));
    return tree;
}
static std::optional<std::pair<size_t, size_t>> lp(const PrefixTree & t, Namespace ns, const V & tokens, bool partial,
                                                   const std::function<bool(size_t, size_t)> & usable) {
    return t.longest_prefix(ns, tokens.data(), tokens.size(), partial, usable);
}

static void longest_prefix_walks_edges_and_splits_on_divergence() {
    auto all = [](size_t, size_t) { return true; };
    {
        PrefixTree tree = tree_with({{1, 2, 3, 4}, {1, 2, 9, 9}});
        auto r = lp(tree, 0, {1, 2, 3, 4, 5}, true, all);
        CHECK(r && r->first == 1 && r->second == 4);
        r = lp(tree, 0, {1, 2, 9, 8}, true, all);
        CHECK(r && r->second == 3);
        r = lp(tree, 0, {1, 2, 9, 8}, false, all);
        CHECK(r && r->second == 2);
    }
    {
        PrefixTree tree = tree_with({{1, 2, 3, 4}});
        auto r = lp(tree, 0, {1, 2}, true, all);
        CHECK(r && r->first == 1 && r->second == 2);
        CHECK(!lp(tree, 0, {1, 2}, false, all));
    }
    {
        PrefixTree tree = tree_with({{1, 2, 3}, {1, 2, 9}});
        auto with_slots = [&](size_t node, size_t) { return tree.slot(node).has_value(); };
        auto r = lp(tree, 0, {1, 2, 7}, true, with_slots);
        CHECK(r && r->second == 2);
        CHECK(!lp(tree, 0, {1, 2, 7}, false, with_slots));
    }
    {
        PrefixTree tree = tree_with({{1, 2, 3}, {1, 2, 3, 4}});
        auto r = lp(tree, 0, {1, 2, 3, 4, 5}, false, [](size_t node, size_t) { return node != 2; });
        CHECK(r && r->first == 1 && r->second == 3);
    }
}

static void insert_attaches_once_and_pin_protects_from_eviction() {
    PrefixTree tree = tree_with({{7, 7, 7}});
    const V p{7, 7, 7};
    auto ins = tree.insert(0, p.data(), p.size(), 42);
    CHECK(!ins.second);
    CHECK(tree.slot(ins.first) == std::optional<int32_t>(1));
    auto pin = tree.pin_at(0, p.data(), p.size());
    CHECK(pin.has_value());
    CHECK(!tree.eviction_candidate());
    CHECK(tree.unpin(*pin));
    CHECK(tree.eviction_candidate() == std::optional<size_t>(ins.first));
    CHECK(!tree.unpin(*pin));
    const V q{8, 8};
    CHECK(!tree.pin_at(0, q.data(), q.size()));
}

static void clear_releases_every_slot_and_snapshot_bytes() {
    PrefixTree tree = tree_with({{1}, {1, 2}});
    tree.attach_snapshot(2, std::make_shared<const std::vector<uint8_t>>(100, 0));
    CHECK(tree.snapshot_bytes() == 100);
    CHECK(tree.clear().size() == 2);
    CHECK(tree.node_count() == 0);
    CHECK(tree.snapshot_bytes() == 0);
}

static void remove_prunes_up_to_the_root_and_recycles_indices() {
    PrefixTree tree = tree_with({{1, 2}, {5, 6}});
    const V p{1, 2};
    auto ins = tree.insert(0, p.data(), p.size(), 9);
    tree.remove(ins.first);
    CHECK(tree.node_count() == 1);
    CHECK(!lp(tree, 0, {1, 2, 3}, true, [](size_t, size_t) { return true; }));
    const V q{7, 8};
    auto again = tree.insert(0, q.data(), q.size(), 3);
    CHECK(again.second);
    CHECK(again.first == ins.first);
    CHECK(tree.node_count() == 2);
}

static void namespaces_share_no_prefix_and_drop_alone() {
    PrefixTree tree;
    const V a{1, 2, 3, 4}, b{1, 2, 9};
    tree.insert(0, a.data(), a.size(), 1);
    tree.insert(7, a.data(), a.size(), 2);
    tree.insert(7, b.data(), b.size(), 3);
    auto all = [](size_t, size_t) { return true; };
    auto r = lp(tree, 0, {1, 2, 3, 4, 5}, false, all);
    CHECK(r && tree.slot(r->first) == std::optional<int32_t>(1) && r->second == 4);
    r = lp(tree, 7, {1, 2, 3, 4, 5}, false, all);
    CHECK(r && tree.slot(r->first) == std::optional<int32_t>(2) && r->second == 4);
    CHECK(!lp(tree, 8, {1, 2, 3, 4}, true, all));
    CHECK(tree.node_count() == 4);
    auto pin = tree.pin_at(7, b.data(), b.size());
    CHECK(pin.has_value());
    std::vector<int32_t> slots = tree.drop_namespace(7);
    std::sort(slots.begin(), slots.end());
    CHECK((slots == std::vector<int32_t>{2, 3}));
    CHECK(!tree.unpin(*pin));
    CHECK(!lp(tree, 7, {1, 2, 3, 4}, true, all));
    CHECK(tree.node_count() == 1);
    CHECK((tree.resident_slots() == std::vector<int32_t>{1}));
    const V c{5, 6};
    tree.insert(7, c.data(), c.size(), 4);
    CHECK(tree.node_count() == 2);
}

static void detokenizer_tests() {
    const std::string party = "\xF0\x9F\x8E\x89";      // U+1F389
    {
        Detokenizer d(std::vector<std::string>{});
        auto r = d.push_bytes("ok ");
        CHECK(r.first == "ok " && !r.second);
        r = d.push_bytes(party.substr(0, 2));
        CHECK(r.first.empty() && !r.second);
        r = d.push_bytes(party.substr(2));
        CHECK(r.first == party && !r.second);
    }
    {
        Detokenizer d({"STOP"});
        auto r = d.push_bytes("abcST");
        CHECK(r.first == "abc" && !r.second);
        r = d.push_bytes("OP");
        CHECK(r.first.empty() && r.second);
        r = d.push_bytes("xyz");
        CHECK(r.first.empty() && r.second);
    }
    {
        Detokenizer d({"</end>"});
        auto r = d.push_bytes("answer</end>ignored");
        CHECK(r.first == "answer" && r.second);
    }
    {
        Detokenizer d({"STOP"});
        auto r = d.push_bytes("abST");
        CHECK(r.first == "ab");
        CHECK(d.finish() == "ST");
    }
    {
        Detokenizer d({"abc"});
        std::string emitted;
        for (const char * piece : {"x", "a", "b", "d", "e"}) {
            auto r = d.push_bytes(piece);
            CHECK(!r.second);
            emitted += r.first;
        }
        emitted += d.finish();
        CHECK(emitted == "xabde");
    }
    {
        // malformed and incomplete UTF-8 match lossy decoding
        const std::string rep = "\xEF\xBF\xBD";
        struct Case { std::vector<std::string> pieces; std::string lossy; };
        const std::vector<Case> cases = {
            {{"\xFFvalid"}, rep + "valid"},
            {{"\xF0\x9F", "ok"}, rep + "ok"},
            {{"ok\xF0\x9F"}, "ok" + rep},
        };
        for (const Case & c : cases) {
            Detokenizer d(std::vector<std::string>{});
            std::string text;
            for (const std::string & p : c.pieces) text += d.push_bytes(p).first;
            text += d.finish();
            CHECK(text == c.lossy);
        }
    }
    {
        Detokenizer d({"abcdef"});
        auto r = d.push_bytes("zzabc");
        CHECK(r.first == "zz" && !r.second);
        r = d.push_bytes("x");
        CHECK(r.first == "abcx" && !r.second);
    }
}

int main() {
    longest_prefix_walks_edges_and_splits_on_divergence();
    insert_attaches_once_and_pin_protects_from_eviction();
    clear_releases_every_slot_and_snapshot_bytes();
    remove_prunes_up_to_the_root_and_recycles_indices();
    namespaces_share_no_prefix_and_drop_alone();
    detokenizer_tests();
    if (g_failed) { std::fprintf(stderr, "%d checks failed\n", g_failed); return 1; }
    std::puts("ok");
    return 0;
}

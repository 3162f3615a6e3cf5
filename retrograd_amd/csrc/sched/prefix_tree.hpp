// The prefix cache's data structure: a radix tree of resident prefixes
// (reference crates/retrograd-infer/src/kv.rs:140-535). Pure data plus
// decisions; every backend operation is performed by the scheduler.
//
// A node with a slot owns a dormant sequence slot whose KV is frozen exactly at
// the node's end position (span [0, depth)); a swapped node kept only a host
// snapshot. Each adapter id is a namespace with its own root; namespace 0
// holds the rows decoded under the context's own adapter set.
#pragma once

#include <cstdint>
#include <functional>
#include <map>
#include <memory>
#include <optional>
#include <unordered_map>
#include <vector>

namespace sched {

using PinId = uint64_t;
using Namespace = uint64_t;
using Snapshot = std::shared_ptr<const std::vector<uint8_t>>;

// kv.rs:100-118
struct KvStats {
    uint64_t hits = 0, misses = 0, prefilled_cells = 0, prompt_cells = 0, evictions = 0, swaps = 0;
    size_t nodes = 0, resident_slots = 0;
    uint64_t snapshot_bytes = 0;
};

class PrefixTree {
public:
    PrefixTree();

    // The longest prefix of `tokens` that has a usable node, as (node, hit),
    // hit <= n. partial_ok allows a mid-sequence hit (hit < depth, served by a
    // partial-range copy). usable(node, hit) is the caller's backend-side check.
    std::optional<std::pair<size_t, size_t>> longest_prefix(
        Namespace ns, const int32_t * tokens, size_t n, bool partial_ok,
        const std::function<bool(size_t, size_t)> & usable) const;

    void touch(size_t node);
    // Inserts the full path and attaches `slot` at its end node: (node,
    // attached); attached is false when the end node already owned a slot.
    std::pair<size_t, bool> insert(Namespace ns, const int32_t * tokens, size_t n, int32_t slot);
    void attach_snapshot(size_t node, Snapshot snapshot);
    const Snapshot & snapshot(size_t node) const { return nodes_[node].snapshot; }
    std::optional<int32_t> slot(size_t node) const { return nodes_[node].slot; }
    void detach_slot(size_t node) { nodes_[node].slot.reset(); }
    size_t depth(size_t node) const { return nodes_[node].depth; }

    std::optional<PinId> pin_at(Namespace ns, const int32_t * tokens, size_t n);
    PinId pin_node(size_t node);
    bool unpin(PinId id);

    // LRU unpinned node owning a slot / LRU unpinned swapped-only node.
    std::optional<size_t> eviction_candidate() const;
    std::optional<size_t> snapshot_eviction_candidate() const;

    // Drops a node's payload and prunes it and its now-childless, payload-free,
    // unpinned ancestors up to the root.
    void remove(size_t node);

    std::vector<int32_t> resident_slots() const;
    uint64_t resident_cells() const;
    // Drops every node and pin; returns the slots the caller must seq_rm.
    std::vector<int32_t> clear();
    std::vector<int32_t> drop_namespace(Namespace ns);

    size_t node_count() const { return nodes_.size() - 1 - roots_.size() - free_.size(); }
    size_t resident_slot_count() const { return resident_slots().size(); }
    uint64_t snapshot_bytes() const { return snapshot_bytes_; }

private:
    struct Node {
        std::vector<int32_t> edge;
        size_t parent = 0;
        size_t depth = 0;
        std::optional<int32_t> slot;
        Snapshot snapshot;
        uint64_t last_use = 0;
        uint32_t pins = 0;
        std::map<int32_t, size_t> children;   // first token of the child edge -> child
    };
    std::optional<size_t> root(Namespace ns) const;
    size_t root_or_insert(Namespace ns);
    bool is_root(size_t node) const { return nodes_[node].edge.empty(); }
    uint64_t tick() { return ++clock_; }
    size_t alloc(Node node);
    std::optional<size_t> deepest_slot_in_subtree(size_t node) const;
    std::optional<size_t> find_exact(Namespace ns, const int32_t * tokens, size_t n) const;
    std::optional<size_t> lru(const std::function<bool(const Node &)> & eligible) const;

    std::vector<Node> nodes_;
    std::vector<size_t> free_;
    std::unordered_map<PinId, size_t> pins_;
    PinId next_pin_ = 1;
    uint64_t clock_ = 0;
    uint64_t snapshot_bytes_ = 0;
    std::unordered_map<Namespace, size_t> roots_;
};

}  // namespace sched

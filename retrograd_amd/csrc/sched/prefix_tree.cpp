#include "prefix_tree.hpp"

#include <algorithm>

namespace sched {

namespace {
constexpr size_t kRoot = 0;

size_t common_len(const std::vector<int32_t> & edge, const int32_t * tokens, size_t n) {
    size_t i = 0;
    while (i < edge.size() && i < n && edge[i] == tokens[i]) ++i;
    return i;
}
}  // namespace

PrefixTree::PrefixTree() { nodes_.emplace_back(); }

std::optional<size_t> PrefixTree::root(Namespace ns) const {
    if (ns == 0) return kRoot;
    auto it = roots_.find(ns);
    if (it == roots_.end()) return std::nullopt;
    return it->second;
}

size_t PrefixTree::root_or_insert(Namespace ns) {
    if (auto r = root(ns)) return *r;
    const size_t r = alloc(Node());
    nodes_[r].parent = r;
    roots_[ns] = r;
    return r;
}

size_t PrefixTree::alloc(Node node) {
    if (!free_.empty()) {
        const size_t index = free_.back();
        free_.pop_back();
        nodes_[index] = std::move(node);
        return index;
    }
    nodes_.push_back(std::move(node));
    return nodes_.size() - 1;
}

// kv.rs:213-268
std::optional<std::pair<size_t, size_t>> PrefixTree::longest_prefix(
    Namespace ns, const int32_t * tokens, size_t n, bool partial_ok,
    const std::function<bool(size_t, size_t)> & usable) const {
    std::optional<std::pair<size_t, size_t>> best;
    const auto start = root(ns);
    if (!start) return std::nullopt;
    size_t cur = *start;
    size_t pos = 0;
    for (;;) {
        const size_t depth = nodes_[cur].depth;
        if (depth > 0 && usable(cur, depth)) best = std::make_pair(cur, depth);
        // the child that continues the prompt, and how much of its edge the prompt shares
        bool has_next = false;
        size_t child = 0, matched = 0;
        if (pos < n) {
            auto it = nodes_[cur].children.find(tokens[pos]);
            if (it != nodes_[cur].children.end()) {
                has_next = true;
                child = it->second;
                matched = common_len(nodes_[child].edge, tokens + pos, n - pos);
            }
        }
        if (has_next && matched == nodes_[child].edge.size()) {
            cur = child;
            pos += matched;
            continue;
        }
        // The walk stops here. A mid-sequence hit is still possible: the prompt
        // shares pos + matched tokens with every path below the continuing child
        // (or pos with any child), served by a partial copy [0, hit) from a
        // slot-bearing node there.
        if (partial_ok) {
            std::optional<size_t> sub;
            size_t m = 0;
            if (has_next) {
                sub = child;
                m = matched;
            } else if (!nodes_[cur].children.empty()) {
                sub = nodes_[cur].children.begin()->second;
            }
            const size_t hit = pos + m;
            if (sub && hit > 0 && (!best || hit > best->second)) {
                const auto slot_node = deepest_slot_in_subtree(*sub);
                if (slot_node && usable(*slot_node, hit)) best = std::make_pair(*slot_node, hit);
            }
        }
        return best;
    }
}

// kv.rs:273-286: depth-first from a stack; children are pushed in ascending
// key order, a strictly deeper slot-bearing node replaces the best so far.
std::optional<size_t> PrefixTree::deepest_slot_in_subtree(size_t node) const {
    std::optional<size_t> best;
    std::vector<size_t> stack{node};
    while (!stack.empty()) {
        const size_t current = stack.back();
        stack.pop_back();
        if (nodes_[current].slot && (!best || nodes_[current].depth > nodes_[*best].depth)) best = current;
        for (const auto & kv : nodes_[current].children) stack.push_back(kv.second);
    }
    return best;
}

void PrefixTree::touch(size_t node) { nodes_[node].last_use = tick(); }

// kv.rs:297-348
std::pair<size_t, bool> PrefixTree::insert(Namespace ns, const int32_t * tokens, size_t n, int32_t slot) {
    size_t cur = root_or_insert(ns);
    size_t pos = 0;
    while (pos < n) {
        const int32_t first = tokens[pos];
        auto it = nodes_[cur].children.find(first);
        if (it != nodes_[cur].children.end()) {
            const size_t child = it->second;
            const size_t matched = common_len(nodes_[child].edge, tokens + pos, n - pos);
            if (matched < nodes_[child].edge.size()) {
                // split the edge at `matched`: a new mid node takes the shared
                // head, the old child moves under it with the tail
                std::vector<int32_t> tail(nodes_[child].edge.begin() + (ptrdiff_t)matched, nodes_[child].edge.end());
                std::vector<int32_t> head(nodes_[child].edge.begin(), nodes_[child].edge.begin() + (ptrdiff_t)matched);
                nodes_[child].edge = std::move(tail);
                Node mid_node;
                mid_node.edge = std::move(head);
                mid_node.parent = cur;
                mid_node.depth = nodes_[cur].depth + matched;
                const size_t mid = alloc(std::move(mid_node));
                const int32_t tail_first = nodes_[child].edge[0];
                nodes_[mid].children[tail_first] = child;
                nodes_[child].parent = mid;
                nodes_[cur].children[first] = mid;
                cur = mid;
            } else {
                cur = child;
            }
            pos += matched;
        } else {
            Node leaf;
            leaf.edge.assign(tokens + pos, tokens + n);
            leaf.parent = cur;
            leaf.depth = n;
            const size_t fresh = alloc(std::move(leaf));
            nodes_[cur].children[first] = fresh;
            cur = fresh;
            pos = n;
        }
    }
    const bool attached = !is_root(cur) && !nodes_[cur].slot;
    if (attached) {
        nodes_[cur].slot = slot;
        nodes_[cur].last_use = tick();
    }
    return {cur, attached};
}

void PrefixTree::attach_snapshot(size_t node, Snapshot snapshot) {
    snapshot_bytes_ += snapshot->size();
    if (nodes_[node].snapshot) {
        const uint64_t old = nodes_[node].snapshot->size();
        snapshot_bytes_ = snapshot_bytes_ >= old ? snapshot_bytes_ - old : 0;
    }
    nodes_[node].snapshot = std::move(snapshot);
}

std::optional<PinId> PrefixTree::pin_at(Namespace ns, const int32_t * tokens, size_t n) {
    const auto node = find_exact(ns, tokens, n);
    if (!node) return std::nullopt;
    return pin_node(*node);
}

PinId PrefixTree::pin_node(size_t node) {
    nodes_[node].pins += 1;
    nodes_[node].last_use = tick();
    const PinId id = next_pin_++;
    pins_[id] = node;
    return id;
}

bool PrefixTree::unpin(PinId id) {
    auto it = pins_.find(id);
    if (it == pins_.end()) return false;
    nodes_[it->second].pins -= 1;
    pins_.erase(it);
    return true;
}

std::optional<size_t> PrefixTree::find_exact(Namespace ns, const int32_t * tokens, size_t n) const {
    const auto start = root(ns);
    if (!start) return std::nullopt;
    size_t cur = *start;
    size_t pos = 0;
    while (pos < n) {
        auto it = nodes_[cur].children.find(tokens[pos]);
        if (it == nodes_[cur].children.end()) return std::nullopt;
        const std::vector<int32_t> & edge = nodes_[it->second].edge;
        if (n - pos < edge.size() || !std::equal(edge.begin(), edge.end(), tokens + pos)) return std::nullopt;
        cur = it->second;
        pos += edge.size();
    }
    if (is_root(cur)) return std::nullopt;
    return cur;
}

std::optional<size_t> PrefixTree::eviction_candidate() const {
    return lru([](const Node & node) { return node.slot.has_value(); });
}

std::optional<size_t> PrefixTree::snapshot_eviction_candidate() const {
    return lru([](const Node & node) { return !node.slot && node.snapshot; });
}

// kv.rs:420-428: the first node of the least last_use among the eligible ones.
std::optional<size_t> PrefixTree::lru(const std::function<bool(const Node &)> & eligible) const {
    std::optional<size_t> best;
    for (size_t i = 1; i < nodes_.size(); ++i) {
        const Node & node = nodes_[i];
        if (node.pins != 0 || !eligible(node)) continue;
        if (!best || node.last_use < nodes_[*best].last_use) best = i;
    }
    return best;
}

// kv.rs:433-456
void PrefixTree::remove(size_t node) {
    if (nodes_[node].snapshot) {
        const uint64_t len = nodes_[node].snapshot->size();
        snapshot_bytes_ = snapshot_bytes_ >= len ? snapshot_bytes_ - len : 0;
        nodes_[node].snapshot.reset();
    }
    nodes_[node].slot.reset();
    size_t child = node;
    while (!is_root(child)) {
        const Node & current = nodes_[child];
        if (!current.children.empty() || current.slot || current.snapshot || current.pins > 0) break;
        const size_t parent = current.parent;
        const int32_t first = current.edge[0];
        nodes_[parent].children.erase(first);
        nodes_[child] = Node();
        free_.push_back(child);
        child = parent;
    }
}

std::vector<int32_t> PrefixTree::resident_slots() const {
    std::vector<int32_t> out;
    for (const Node & node : nodes_) if (node.slot) out.push_back(*node.slot);
    return out;
}

uint64_t PrefixTree::resident_cells() const {
    uint64_t sum = 0;
    for (const Node & node : nodes_) if (node.slot) sum += node.depth;
    return sum;
}

std::vector<int32_t> PrefixTree::clear() {
    std::vector<int32_t> slots = resident_slots();
    nodes_.resize(1);
    nodes_[kRoot] = Node();
    free_.clear();
    pins_.clear();
    roots_.clear();
    snapshot_bytes_ = 0;
    return slots;
}

// kv.rs:491-525
std::vector<int32_t> PrefixTree::drop_namespace(Namespace ns) {
    const auto r = root(ns);
    if (!r) return {};
    const size_t rootn = *r;
    std::vector<int32_t> slots;
    std::vector<size_t> dropped;
    std::vector<size_t> stack;
    for (const auto & kv : nodes_[rootn].children) stack.push_back(kv.second);
    while (!stack.empty()) {
        const size_t node = stack.back();
        stack.pop_back();
        for (const auto & kv : nodes_[node].children) stack.push_back(kv.second);
        if (nodes_[node].slot) slots.push_back(*nodes_[node].slot);
        if (nodes_[node].snapshot) {
            const uint64_t len = nodes_[node].snapshot->size();
            snapshot_bytes_ = snapshot_bytes_ >= len ? snapshot_bytes_ - len : 0;
        }
        dropped.push_back(node);
    }
    for (size_t node : dropped) nodes_[node].pins = 0;
    for (auto it = pins_.begin(); it != pins_.end();) {
        if (nodes_[it->second].pins == 0) it = pins_.erase(it); else ++it;
    }
    for (size_t node : dropped) {
        nodes_[node] = Node();
        free_.push_back(node);
    }
    nodes_[rootn].children.clear();
    if (rootn != kRoot) {
        roots_.erase(ns);
        nodes_[rootn] = Node();
        free_.push_back(rootn);
    }
    return slots;
}

}  // namespace sched

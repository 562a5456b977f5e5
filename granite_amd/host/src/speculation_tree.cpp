// SpeculationTree (reference: src/llm/speculation_tree.cpp:13-150).
#include <algorithm>
#include <deque>

#include "granite/kv_cache.h"

namespace granite {

void SpeculationTree::build(int, int) {}

int SpeculationTree::add_node(int32_t token, int parent_idx, float log_prob) {
    const int idx = static_cast<int>(nodes_.size());
    Node n{token, parent_idx, 0, log_prob, {}};
    if (parent_idx >= 0) {
        n.depth = nodes_[parent_idx].depth + 1;
        nodes_[parent_idx].children.push_back(idx);
    }
    nodes_.push_back(std::move(n));
    return idx;
}

std::vector<int> SpeculationTree::get_leaves() const {
    std::vector<int> leaves;
    for (size_t i = 0; i < nodes_.size(); ++i)
        if (nodes_[i].children.empty()) leaves.push_back(static_cast<int>(i));
    return leaves;
}

std::vector<int> SpeculationTree::get_path(int node_idx) const {
    std::vector<int> path;
    for (int at = node_idx; at >= 0; at = nodes_[at].parent_idx) path.push_back(at);
    std::reverse(path.begin(), path.end());
    return path;
}

std::vector<int> SpeculationTree::get_parent_indices() const {
    std::vector<int> parents(nodes_.size());
    for (size_t i = 0; i < nodes_.size(); ++i) parents[i] = nodes_[i].parent_idx;
    return parents;
}

std::vector<int32_t> SpeculationTree::flatten_tokens() const {
    std::vector<int32_t> tokens;
    if (nodes_.empty()) return tokens;
    tokens.reserve(nodes_.size());
    std::deque<int> frontier{0};
    while (!frontier.empty()) {
        const Node& n = nodes_[frontier.front()];
        frontier.pop_front();
        tokens.push_back(n.token);
        frontier.insert(frontier.end(), n.children.begin(), n.children.end());
    }
    return tokens;
}

int SpeculationTree::max_depth() const {
    int deepest = 0;
    for (const Node& n : nodes_) deepest = std::max(deepest, n.depth);
    return deepest;
}

namespace {
// Depth-first walk; `path` is the accepted prefix on entry.
void walk(const SpeculationTree& tree, int idx, size_t pos, const std::vector<int32_t>& choices,
          std::vector<int32_t>& path, std::vector<int32_t>& best) {
    auto consider = [&] {
        if (path.size() > best.size()) best = path;
    };
    if (pos >= choices.size()) {
        consider();
        return;
    }
    const SpeculationTree::Node& n = tree.node(idx);
    if (n.token != choices[pos]) {  // the target's token ends this branch
        path.push_back(choices[pos]);
        consider();
        path.pop_back();
        return;
    }
    path.push_back(n.token);
    if (n.children.empty()) consider();
    for (int child : n.children) walk(tree, child, pos + 1, choices, path, best);
    path.pop_back();
}
}  // namespace

std::vector<int32_t> SpeculationTree::find_accepted_path(
    const std::vector<int32_t>& target_choices) const {
    std::vector<int32_t> best, path;
    if (nodes_.empty() || target_choices.empty()) return best;
    walk(*this, 0, 0, target_choices, path, best);
    return best;
}

std::vector<int> SpeculationTree::find_accepted_nodes(const std::vector<int32_t>& target_choices) const {
    // Replays the accepted token path from the root: position i of the path is the child of
    // the previous node whose token the target chose.
    std::vector<int> nodes;
    const std::vector<int32_t> tokens = find_accepted_path(target_choices);
    if (nodes_.empty() || tokens.empty()) return nodes;
    int cur = 0;
    for (size_t i = 0; i < tokens.size(); ++i) {
        if (i == 0) {
            if (nodes_[0].token != tokens[0]) break;  // the root itself was replaced
        } else {
            int next = -1;
            for (int child : nodes_[cur].children)
                if (nodes_[child].token == tokens[i]) {
                    next = child;
                    break;
                }
            if (next < 0) break;  // the closing token of a mismatch: no node
            cur = next;
        }
        nodes.push_back(cur);
    }
    return nodes;
}

}  // namespace granite

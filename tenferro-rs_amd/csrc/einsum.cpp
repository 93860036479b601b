// einsum.cpp -- the einsum front end and executor of the Hip backend:
//   Subscripts::{new, parse}                 tenferro-einsum/src/lib.rs:239-284
//   ContractionTree::{optimize, from_pairs}  tenferro-einsum/src/lib.rs:297-356
//   einsum_with_plan_into                    tenferro-einsum/src/lib.rs:584-621
// The executor enqueues every pairwise contraction of the tree on one stream; intermediates live in
// device memory taken from the stream's block cache and are laid out so that the step that consumes
// them reads its contracted modes contiguously.  The host never waits.
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <functional>
#include <list>
#include <map>
#include <mutex>
#include <set>
#include <string>
#include <unordered_map>

#include "internal.hpp"

using namespace tfh;

// A parse/ordering tree over operand indices: leaf >= 0, or a group of children.
struct NestNode {
    int leaf = -1;
    std::vector<int> children;  // indices into tfh_subscripts::nest
};

struct tfh_subscripts {
    std::vector<std::vector<uint32_t>> inputs;
    std::vector<uint32_t> output;
    std::vector<NestNode> nest;   // nest[root] is the top-level group
    int root = -1;
    bool has_parens = false;
};

struct TreeStep {
    int lhs, rhs;
};
struct TreeNode {
    std::vector<uint32_t> labels;   // memory order (row-major: last label fastest) for intermediates
    std::vector<int64_t> dims;
};
struct tfh_tree {
    int n_inputs = 0;
    std::vector<std::vector<uint32_t>> input_labels;   // as given (may repeat a label)
    std::vector<std::vector<int64_t>> input_dims;
    std::vector<uint32_t> output_labels;               // as given (may repeat a label)
    std::vector<int64_t> output_dims;
    std::map<uint32_t, int64_t> extent;
    std::vector<TreeNode> nodes;    // inputs after diagonal/pre-reduction (unique labels), then intermediates
    std::vector<TreeStep> steps;
    double macs = 0, peak = 0;
    std::atomic<int> refs{1};   // the creator's reference; the tree cache and each of its hits hold one more
    // One cache of routed launches per step (contract_cache.cpp): executions of the tree on operands with the strides of
    // an earlier execution enqueue that execution's kernels again without routing.  Made on first use (under step_mu);
    // an entry that could not be made stays null and its step routes every time.
    mutable std::mutex step_mu;
    mutable std::vector<tfh::ContractCache*> step_cache;
    ~tfh_tree() {
        for (tfh::ContractCache* c : step_cache) tfh::contract_cache_destroy(c);
    }
};

namespace {

int find(const std::vector<uint32_t>& m, uint32_t l) {
    for (size_t i = 0; i < m.size(); ++i)
        if (m[i] == l) return (int)i;
    return -1;
}
std::vector<uint32_t> unique_labels(const std::vector<uint32_t>& m) {
    std::vector<uint32_t> r;
    for (uint32_t l : m)
        if (find(r, l) < 0) r.push_back(l);
    return r;
}

// ---- parser ------------------------------------------------------------------------------------------
struct Parser {
    const char* s;
    size_t pos = 0;
    tfh_subscripts* out;
    std::string err;
    explicit Parser(const char* str, tfh_subscripts* o) : s(str), out(o) {}
    void skip() {
        while (s[pos] == ' ' || s[pos] == '\t') ++pos;
    }
    static bool is_label(char c) { return (c >= 'a' && c <= 'z') || (c >= 'A' && c <= 'Z'); }
    // group := item (',' item)* ; item := '(' group ')' | labels
    int parse_group(bool top) {
        int id = (int)out->nest.size();
        out->nest.emplace_back();
        for (;;) {
            skip();
            int child;
            if (s[pos] == '(') {
                ++pos;
                out->has_parens = true;
                child = parse_group(false);
                if (child < 0) return -1;
                skip();
                if (s[pos] != ')') {
                    err = "missing ')'";
                    return -1;
                }
                ++pos;
            } else {
                std::vector<uint32_t> labels;
                while (is_label(s[pos]) || s[pos] == ' ' || s[pos] == '\t') {
                    if (is_label(s[pos])) labels.push_back((uint32_t)(unsigned char)s[pos]);
                    ++pos;
                }
                child = (int)out->nest.size();
                out->nest.emplace_back();
                out->nest[child].leaf = (int)out->inputs.size();
                out->inputs.push_back(labels);
            }
            out->nest[id].children.push_back(child);
            skip();
            if (s[pos] == ',') {
                ++pos;
                continue;
            }
            if (top ? (s[pos] == '-' || s[pos] == 0) : s[pos] == ')') return id;
            err = std::string("unexpected character '") + (s[pos] ? s[pos] : '$') + "'";
            return -1;
        }
    }
};

int32_t check_output_labels(const tfh_subscripts& s) {
    for (uint32_t l : s.output) {
        bool found = false;
        for (auto& in : s.inputs) found |= find(in, l) >= 0;
        if (!found) return set_error(TFH_ERR_INVALID_ARGUMENT, "einsum: output label %u appears in no input", l);
    }
    return TFH_OK;
}

// ---- tree construction ---------------------------------------------------------------------------------
struct Item {          // a node while the order is being chosen
    int node;
    std::set<uint32_t> labels;
};

struct Builder {
    tfh_tree& t;
    explicit Builder(tfh_tree& tree) : t(tree) {}

    double size_of(const std::set<uint32_t>& ls) const {
        double p = 1;
        for (uint32_t l : ls) p *= (double)t.extent.at(l);
        return p;
    }
    // Labels of the result of contracting `a` and `b` when `others` (and the output) remain.
    std::set<uint32_t> result_labels(const std::set<uint32_t>& a, const std::set<uint32_t>& b,
                                     const std::vector<const std::set<uint32_t>*>& others) const {
        std::set<uint32_t> r;
        auto needed = [&](uint32_t l) {
            if (find(t.output_labels, l) >= 0) return true;
            for (auto* o : others)
                if (o->count(l)) return true;
            return false;
        };
        for (uint32_t l : a)
            if (needed(l)) r.insert(l);
        for (uint32_t l : b)
            if (needed(l)) r.insert(l);
        return r;
    }
    // Records one pairwise step; returns the new node index.  Label order of the node is fixed later.
    int add_step(int lhs, int rhs, const std::set<uint32_t>& labels, const std::set<uint32_t>& la, const std::set<uint32_t>& lb) {
        std::set<uint32_t> all = la;
        all.insert(lb.begin(), lb.end());
        t.macs += size_of(all);
        TreeNode n;
        n.labels.assign(labels.begin(), labels.end());
        for (uint32_t l : n.labels) n.dims.push_back(t.extent.at(l));
        t.nodes.push_back(n);
        t.steps.push_back({lhs, rhs});
        return (int)t.nodes.size() - 1;
    }

    // Contracts `items` down to one item in the cheapest order (total multiply-add count; ties by the
    // size of the largest intermediate).  `outside`: label sets of everything not in `items`.
    Item reduce_items(std::vector<Item> items, const std::vector<const std::set<uint32_t>*>& outside) {
        const int n = (int)items.size();
        if (n == 1) return items[0];
        if (n <= 12) {
            // exhaustive dynamic programme over subsets
            const int full = (1 << n) - 1;
            std::vector<double> cost((size_t)full + 1, INFINITY), peak((size_t)full + 1, 0);
            std::vector<int> best((size_t)full + 1, 0);
            std::vector<std::set<uint32_t>> lab((size_t)full + 1);
            for (int m = 1; m <= full; ++m) {
                // labels of subset m that the rest of the network (or the output) still needs
                std::set<uint32_t> in;
                for (int i = 0; i < n; ++i)
                    if (m >> i & 1) in.insert(items[i].labels.begin(), items[i].labels.end());
                std::vector<const std::set<uint32_t>*> others = outside;
                for (int i = 0; i < n; ++i)
                    if (!(m >> i & 1)) others.push_back(&items[i].labels);
                if ((m & (m - 1)) == 0) {
                    lab[m] = in;   // a single item keeps all its labels
                    cost[m] = 0;
                    continue;
                }
                lab[m] = result_labels(in, {}, others);
            }
            for (int m = 1; m <= full; ++m) {
                if ((m & (m - 1)) == 0) continue;
                for (int s1 = (m - 1) & m; s1 > 0; s1 = (s1 - 1) & m) {
                    int s2 = m ^ s1;
                    if (s1 < s2) continue;   // each split once
                    std::set<uint32_t> all = lab[s1];
                    all.insert(lab[s2].begin(), lab[s2].end());
                    double c = cost[s1] + cost[s2] + size_of(all);
                    double pk = std::max({peak[s1], peak[s2], m == full ? 0.0 : size_of(lab[m])});
                    if (c < cost[m] || (c == cost[m] && pk < peak[m])) {
                        cost[m] = c;
                        peak[m] = pk;
                        best[m] = s1;
                    }
                }
            }
            // emit steps bottom-up
            std::function<Item(int)> emit = [&](int m) -> Item {
                if ((m & (m - 1)) == 0) {
                    int i = 0;
                    while (!(m >> i & 1)) ++i;
                    return items[i];
                }
                Item a = emit(best[m]), b = emit(m ^ best[m]);
                Item r;
                r.labels = lab[m];
                r.node = add_step(a.node, b.node, r.labels, a.labels, b.labels);
                return r;
            };
            return emit(full);
        }
        // greedy: cheapest pair first
        while (items.size() > 1) {
            double bc = INFINITY, bs = INFINITY;
            size_t bi = 0, bj = 1;
            std::set<uint32_t> bl;
            for (size_t i = 0; i < items.size(); ++i)
                for (size_t j = i + 1; j < items.size(); ++j) {
                    std::vector<const std::set<uint32_t>*> others = outside;
                    for (size_t k = 0; k < items.size(); ++k)
                        if (k != i && k != j) others.push_back(&items[k].labels);
                    std::set<uint32_t> all = items[i].labels;
                    all.insert(items[j].labels.begin(), items[j].labels.end());
                    std::set<uint32_t> rl = result_labels(items[i].labels, items[j].labels, others);
                    double c = size_of(all), sz = size_of(rl);
                    if (c < bc || (c == bc && sz < bs)) {
                        bc = c; bs = sz; bi = i; bj = j; bl = rl;
                    }
                }
            Item r;
            r.labels = bl;
            r.node = add_step(items[bi].node, items[bj].node, bl, items[bi].labels, items[bj].labels);
            items.erase(items.begin() + bj);
            items.erase(items.begin() + bi);
            items.push_back(r);
        }
        return items[0];
    }

    // Follows the nesting of the subscripts: a group's children are reduced first, then the group.
    Item reduce_nest(const tfh_subscripts& s, int id, const std::vector<const std::set<uint32_t>*>& outside,
                     const std::vector<std::set<uint32_t>>& leaf_labels) {
        const NestNode& nn = s.nest[id];
        if (nn.leaf >= 0) return Item{nn.leaf, leaf_labels[nn.leaf]};
        // label sets of the leaves under each child, to know what is "outside" of a child
        std::vector<std::vector<int>> leaves(nn.children.size());
        std::function<void(int, std::vector<int>&)> collect = [&](int n, std::vector<int>& out) {
            if (s.nest[n].leaf >= 0) out.push_back(s.nest[n].leaf);
            for (int c : s.nest[n].children) collect(c, out);
        };
        for (size_t c = 0; c < nn.children.size(); ++c) collect(nn.children[c], leaves[c]);
        std::vector<Item> items;
        for (size_t c = 0; c < nn.children.size(); ++c) {
            std::vector<const std::set<uint32_t>*> out2 = outside;
            for (size_t o = 0; o < nn.children.size(); ++o)
                if (o != c)
                    for (int lf : leaves[o]) out2.push_back(&leaf_labels[lf]);
            items.push_back(reduce_nest(s, nn.children[c], out2, leaf_labels));
        }
        return reduce_items(items, outside);
    }
};

int32_t bind_tree_inputs(tfh_tree& t, const tfh_subscripts* s, const int64_t* const* shapes, const int32_t* ranks, int32_t n_inputs) {
    if (!s || (n_inputs > 0 && (!shapes || !ranks))) return set_error(TFH_ERR_INVALID_ARGUMENT, "null argument");
    if (n_inputs != (int)s->inputs.size())
        return set_error(TFH_ERR_INVALID_ARGUMENT, "subscripts name %d operands, %d shapes given", (int)s->inputs.size(), n_inputs);
    if (n_inputs < 1) return set_error(TFH_ERR_INVALID_ARGUMENT, "einsum needs at least one operand");
    if (int32_t e = check_output_labels(*s)) return e;
    t.n_inputs = n_inputs;
    t.input_labels = s->inputs;
    t.output_labels = s->output;
    for (int i = 0; i < n_inputs; ++i) {
        if (ranks[i] != (int)s->inputs[i].size()) return set_rank_mismatch((int64_t)s->inputs[i].size(), ranks[i]);
        if (ranks[i] > TFH_MAX_RANK) return set_error(TFH_ERR_INVALID_ARGUMENT, "operand %d has more than %d axes", i, TFH_MAX_RANK);
        std::vector<int64_t> dims(shapes[i], shapes[i] + ranks[i]), expected = dims;
        bool bad = false;
        for (int d = 0; d < ranks[i]; ++d) {
            if (dims[d] < 0) return set_error(TFH_ERR_INVALID_ARGUMENT, "operand %d has a negative extent", i);
            auto it = t.extent.find(s->inputs[i][d]);
            if (it == t.extent.end()) t.extent[s->inputs[i][d]] = dims[d];
            else if (it->second != dims[d]) {
                expected[d] = it->second;
                bad = true;
            }
        }
        if (bad) return set_shape_mismatch(expected.data(), ranks[i], dims.data(), ranks[i]);
        t.input_dims.push_back(dims);
    }
    if ((int)s->output.size() > TFH_MAX_RANK) return set_error(TFH_ERR_INVALID_ARGUMENT, "output has more than %d axes", TFH_MAX_RANK);
    for (uint32_t l : s->output) t.output_dims.push_back(t.extent.at(l));
    return TFH_OK;
}

// Leaf nodes: unique labels of each operand minus the labels only it carries and the output lacks
// (those are summed before any contraction).
void make_leaves(tfh_tree& t) {
    for (int i = 0; i < t.n_inputs; ++i) {
        TreeNode n;
        for (uint32_t l : unique_labels(t.input_labels[i])) {
            bool elsewhere = find(t.output_labels, l) >= 0;
            for (int j = 0; j < t.n_inputs && !elsewhere; ++j)
                if (j != i && find(t.input_labels[j], l) >= 0) elsewhere = true;
            if (elsewhere || t.n_inputs == 1) {
                if (t.n_inputs == 1 && find(t.output_labels, l) < 0) continue;   // single operand: summed directly
                n.labels.push_back(l);
                n.dims.push_back(t.extent.at(l));
            }
        }
        t.nodes.push_back(n);
    }
}

// Memory order of the intermediates.  Walking the steps backwards, an intermediate T consumed with
// sibling Z into U is laid out [batch | free, in U's order | contracted, largest extent innermost], so
// the consumer reads its contracted modes contiguously and writes U in long runs.
void choose_layouts(tfh_tree& t) {
    const int ns = (int)t.steps.size();
    if (ns == 0) return;
    // the last node is the result: unique output labels in output order
    t.nodes.back().labels = unique_labels(t.output_labels);
    t.nodes.back().dims.clear();
    for (uint32_t l : t.nodes.back().labels) t.nodes.back().dims.push_back(t.extent.at(l));
    for (int s = ns - 1; s >= 0; --s) {
        const TreeNode& U = t.nodes[(size_t)t.n_inputs + s];
        for (int side = 0; side < 2; ++side) {
            int ti = side ? t.steps[s].rhs : t.steps[s].lhs, zi = side ? t.steps[s].lhs : t.steps[s].rhs;
            if (ti < t.n_inputs) continue;   // inputs keep the caller's layout
            TreeNode& T = t.nodes[ti];
            const TreeNode& Z = t.nodes[zi];
            std::vector<uint32_t> batch, fre, con;
            for (uint32_t l : U.labels)
                if (find(T.labels, l) >= 0) (find(Z.labels, l) >= 0 ? batch : fre).push_back(l);
            for (uint32_t l : T.labels)
                if (find(U.labels, l) < 0) con.push_back(l);
            std::stable_sort(con.begin(), con.end(), [&](uint32_t x, uint32_t y) { return t.extent.at(x) < t.extent.at(y); });
            std::vector<uint32_t> order = batch;
            order.insert(order.end(), fre.begin(), fre.end());
            order.insert(order.end(), con.begin(), con.end());
            T.labels = order;
            T.dims.clear();
            for (uint32_t l : order) T.dims.push_back(t.extent.at(l));
        }
    }
}

void finish_tree(tfh_tree& t) {
    choose_layouts(t);
    t.peak = 0;
    for (size_t i = (size_t)t.n_inputs; i + 1 < t.nodes.size(); ++i) {
        double p = 1;
        for (int64_t d : t.nodes[i].dims) p *= (double)d;
        t.peak = std::max(t.peak, p);
    }
}

}  // namespace

// ---- tree cache: the allocating / string forms of einsum optimise the same network on every call
namespace {
constexpr size_t TREE_CACHE_ENTRIES = 512;
struct TreeCache {
    std::mutex mu;
    std::list<std::string> order;   // most recently used first
    std::unordered_map<std::string, std::pair<tfh_tree*, std::list<std::string>::iterator>> map;
    int64_t hits = 0, misses = 0;
};
TreeCache& tree_cache() {
    static TreeCache* c = new TreeCache();   // never destroyed: trees may be released during process exit
    return *c;
}
void put_u64(std::string& k, uint64_t v) { k.append(reinterpret_cast<const char*>(&v), sizeof v); }
}  // namespace

extern "C" {

int32_t tfh_subscripts_new(const uint32_t* labels, const int32_t* ranks, int32_t n_inputs, const uint32_t* output,
                           int32_t n_output, tfh_subscripts** out) {
    if (!out) return set_error(TFH_ERR_INVALID_ARGUMENT, "null output pointer");
    *out = nullptr;
    if (n_inputs < 0 || n_output < 0 || (n_inputs > 0 && !ranks)) return set_error(TFH_ERR_INVALID_ARGUMENT, "bad subscripts");
    auto* s = new (std::nothrow) tfh_subscripts();
    if (!s) return set_error(TFH_ERR_DEVICE, "out of host memory");
    s->nest.emplace_back();
    s->root = 0;
    const uint32_t* p = labels;
    for (int i = 0; i < n_inputs; ++i) {
        if (ranks[i] < 0) {
            delete s;
            return set_error(TFH_ERR_INVALID_ARGUMENT, "negative rank");
        }
        s->inputs.emplace_back(p, p + ranks[i]);
        p += ranks[i];
        NestNode leaf;
        leaf.leaf = i;
        s->nest.push_back(leaf);
        s->nest[0].children.push_back((int)s->nest.size() - 1);
    }
    if (n_output > 0) s->output.assign(output, output + n_output);
    *out = s;
    clear_error();
    return TFH_OK;
}

int32_t tfh_subscripts_parse(const char* notation, tfh_subscripts** out) {
    if (!out) return set_error(TFH_ERR_INVALID_ARGUMENT, "null output pointer");
    *out = nullptr;
    if (!notation) return set_error(TFH_ERR_INVALID_ARGUMENT, "null notation");
    auto* s = new (std::nothrow) tfh_subscripts();
    if (!s) return set_error(TFH_ERR_DEVICE, "out of host memory");
    Parser ps(notation, s);
    s->root = ps.parse_group(true);
    if (s->root < 0) {
        delete s;
        return set_error(TFH_ERR_INVALID_ARGUMENT, "einsum notation \"%s\": %s at position %zu", notation, ps.err.c_str(), ps.pos);
    }
    if (notation[ps.pos] != '-' || notation[ps.pos + 1] != '>') {
        delete s;
        return set_error(TFH_ERR_INVALID_ARGUMENT, "einsum notation \"%s\": expected \"->\" at position %zu", notation, ps.pos);
    }
    ps.pos += 2;
    for (; notation[ps.pos]; ++ps.pos) {
        char c = notation[ps.pos];
        if (c == ' ' || c == '\t') continue;
        if (!Parser::is_label(c)) {
            delete s;
            return set_error(TFH_ERR_INVALID_ARGUMENT, "einsum notation \"%s\": unexpected character '%c' in the output at position %zu", notation, c, ps.pos);
        }
        s->output.push_back((uint32_t)(unsigned char)c);
    }
    if (int32_t e = check_output_labels(*s)) {
        delete s;
        return e;
    }
    *out = s;
    clear_error();
    return TFH_OK;
}

void tfh_subscripts_destroy(tfh_subscripts* s) { delete s; }
int32_t tfh_subscripts_n_inputs(const tfh_subscripts* s) { return s ? (int32_t)s->inputs.size() : 0; }
int32_t tfh_subscripts_input_rank(const tfh_subscripts* s, int32_t i) {
    return (s && i >= 0 && i < (int)s->inputs.size()) ? (int32_t)s->inputs[i].size() : -1;
}
int32_t tfh_subscripts_labels(const tfh_subscripts* s, int32_t i, uint32_t* out, int32_t cap) {
    if (!s || i < -1 || i >= (int)s->inputs.size()) return -1;
    const std::vector<uint32_t>& v = i < 0 ? s->output : s->inputs[i];
    for (int d = 0; d < (int)v.size() && d < cap; ++d) out[d] = v[d];
    return (int32_t)v.size();
}
int32_t tfh_subscripts_nesting(const tfh_subscripts* s, char* buf, size_t cap) {
    if (!s || !buf || !cap) return set_error(TFH_ERR_INVALID_ARGUMENT, "null argument");
    std::string r;
    std::function<void(int, bool)> emit = [&](int n, bool top) {
        if (s->nest[n].leaf >= 0) {
            r += std::to_string(s->nest[n].leaf);
            return;
        }
        if (!top) r += "(";
        for (size_t c = 0; c < s->nest[n].children.size(); ++c) {
            if (c) r += ",";
            emit(s->nest[n].children[c], false);
        }
        if (!top) r += ")";
    };
    emit(s->root, true);
    snprintf(buf, cap, "%s", r.c_str());
    return TFH_OK;
}

int32_t tfh_tree_optimize(const tfh_subscripts* s, const int64_t* const* shapes, const int32_t* ranks, int32_t n_inputs,
                          tfh_tree** out) {
    if (!out) return set_error(TFH_ERR_INVALID_ARGUMENT, "null output pointer");
    *out = nullptr;
    auto* t = new (std::nothrow) tfh_tree();
    if (!t) return set_error(TFH_ERR_DEVICE, "out of host memory");
    if (int32_t e = bind_tree_inputs(*t, s, shapes, ranks, n_inputs)) {
        delete t;
        return e;
    }
    make_leaves(*t);
    if (n_inputs > 1) {
        std::vector<std::set<uint32_t>> leaf_labels;
        for (int i = 0; i < n_inputs; ++i) leaf_labels.emplace_back(t->nodes[i].labels.begin(), t->nodes[i].labels.end());
        Builder b(*t);
        b.reduce_nest(*s, s->root, {}, leaf_labels);
    }
    finish_tree(*t);
    *out = t;
    clear_error();
    return TFH_OK;
}

int32_t tfh_tree_from_pairs(const tfh_subscripts* s, const int64_t* const* shapes, const int32_t* ranks, int32_t n_inputs,
                            const int32_t* pairs, int32_t n_pairs, tfh_tree** out) {
    if (!out) return set_error(TFH_ERR_INVALID_ARGUMENT, "null output pointer");
    *out = nullptr;
    auto* t = new (std::nothrow) tfh_tree();
    if (!t) return set_error(TFH_ERR_DEVICE, "out of host memory");
    if (int32_t e = bind_tree_inputs(*t, s, shapes, ranks, n_inputs)) {
        delete t;
        return e;
    }
    if (n_pairs != n_inputs - 1 || (n_pairs > 0 && !pairs)) {
        delete t;
        return set_error(TFH_ERR_INVALID_ARGUMENT, "from_pairs: %d operands need %d pairs, got %d", n_inputs, n_inputs - 1, n_pairs);
    }
    make_leaves(*t);
    Builder b(*t);
    std::vector<char> alive((size_t)n_inputs, 1);
    std::vector<std::set<uint32_t>> labels;
    for (int i = 0; i < n_inputs; ++i) labels.emplace_back(t->nodes[i].labels.begin(), t->nodes[i].labels.end());
    for (int p = 0; p < n_pairs; ++p) {
        int i = pairs[2 * p], j = pairs[2 * p + 1];
        // intermediates are numbered from n_inputs upward (tenferro-einsum/src/lib.rs:322-324)
        if (i < 0 || j < 0 || i >= (int)alive.size() || j >= (int)alive.size() || i == j || !alive[i] || !alive[j]) {
            delete t;
            return set_error(TFH_ERR_INVALID_ARGUMENT, "from_pairs: pair %d = (%d, %d) does not name two distinct live operands", p, i, j);
        }
        alive[i] = alive[j] = 0;
        std::vector<const std::set<uint32_t>*> others;
        for (size_t k = 0; k < alive.size(); ++k)
            if (alive[k]) others.push_back(&labels[k]);
        std::set<uint32_t> rl = b.result_labels(labels[i], labels[j], others);
        b.add_step(i, j, rl, labels[i], labels[j]);
        labels.push_back(rl);
        alive.push_back(1);
    }
    finish_tree(*t);
    *out = t;
    clear_error();
    return TFH_OK;
}

void tfh_tree_destroy(tfh_tree* t) {
    if (t && t->refs.fetch_sub(1, std::memory_order_acq_rel) == 1) delete t;
}

int32_t tfh_tree_optimize_cached(const tfh_subscripts* s, const int64_t* const* shapes, const int32_t* ranks, int32_t n_inputs,
                                 tfh_tree** out) {
    if (!out) return set_error(TFH_ERR_INVALID_ARGUMENT, "null output pointer");
    *out = nullptr;
    if (!s || n_inputs != (int32_t)s->inputs.size() || (n_inputs > 0 && (!shapes || !ranks)))
        return tfh_tree_optimize(s, shapes, ranks, n_inputs, out);   // reports the error
    // key: the labels of every operand and of the output, the grouping the parentheses spell, and the extents
    std::string key;
    put_u64(key, (uint64_t)n_inputs);
    for (int i = 0; i < n_inputs; ++i) {
        if (ranks[i] != (int32_t)s->inputs[i].size() || (ranks[i] > 0 && !shapes[i])) return tfh_tree_optimize(s, shapes, ranks, n_inputs, out);
        put_u64(key, (uint64_t)ranks[i]);
        for (int d = 0; d < ranks[i]; ++d) {
            put_u64(key, s->inputs[i][d]);
            put_u64(key, (uint64_t)shapes[i][d]);
        }
    }
    put_u64(key, (uint64_t)s->output.size());
    for (uint32_t l : s->output) put_u64(key, l);
    if (s->has_parens) {
        std::function<void(int)> emit = [&](int n) {
            if (s->nest[n].leaf >= 0) {
                put_u64(key, (uint64_t)s->nest[n].leaf);
                return;
            }
            put_u64(key, ~(uint64_t)0);
            for (int c : s->nest[n].children) emit(c);
            put_u64(key, ~(uint64_t)1);
        };
        emit(s->root);
    }
    TreeCache& c = tree_cache();
    {
        std::lock_guard<std::mutex> lk(c.mu);
        auto it = c.map.find(key);
        if (it != c.map.end()) {
            c.order.splice(c.order.begin(), c.order, it->second.second);
            it->second.first->refs.fetch_add(1, std::memory_order_relaxed);
            *out = it->second.first;
            ++c.hits;
            clear_error();
            return TFH_OK;
        }
    }
    tfh_tree* t = nullptr;
    if (int32_t e = tfh_tree_optimize(s, shapes, ranks, n_inputs, &t)) return e;
    {
        std::lock_guard<std::mutex> lk(c.mu);
        ++c.misses;
        if (c.map.find(key) == c.map.end()) {   // (another thread may have inserted the same network meanwhile)
            while (c.map.size() >= TREE_CACHE_ENTRIES) {
                auto victim = c.map.find(c.order.back());
                tfh_tree_destroy(victim->second.first);   // callers that still hold it keep it alive
                c.map.erase(victim);
                c.order.pop_back();
            }
            c.order.push_front(key);
            t->refs.fetch_add(1, std::memory_order_relaxed);
            c.map.emplace(key, std::make_pair(t, c.order.begin()));
        }
    }
    *out = t;
    return TFH_OK;
}

int32_t tfh_tree_cache_stats(int64_t* hits, int64_t* misses, int64_t* entries) {
    TreeCache& c = tree_cache();
    std::lock_guard<std::mutex> lk(c.mu);
    if (hits) *hits = c.hits;
    if (misses) *misses = c.misses;
    if (entries) *entries = (int64_t)c.map.size();
    return TFH_OK;
}

int32_t tfh_tree_cache_clear(void) {
    TreeCache& c = tree_cache();
    std::lock_guard<std::mutex> lk(c.mu);
    for (auto& kv : c.map) tfh_tree_destroy(kv.second.first);
    c.map.clear();
    c.order.clear();
    return TFH_OK;
}
int32_t tfh_tree_n_inputs(const tfh_tree* t) { return t ? t->n_inputs : 0; }
int32_t tfh_tree_n_steps(const tfh_tree* t) { return t ? (int32_t)t->steps.size() : 0; }
int32_t tfh_tree_step(const tfh_tree* t, int32_t i, int32_t* lhs, int32_t* rhs) {
    if (!t || i < 0 || i >= (int)t->steps.size()) return set_error(TFH_ERR_INVALID_ARGUMENT, "step %d out of range", i);
    if (lhs) *lhs = t->steps[i].lhs;
    if (rhs) *rhs = t->steps[i].rhs;
    return TFH_OK;
}
int32_t tfh_tree_node(const tfh_tree* t, int32_t node, uint32_t* labels, int64_t* dims, int32_t cap) {
    if (!t || node < 0 || node >= (int)t->nodes.size()) return -1;
    const TreeNode& n = t->nodes[node];
    for (int d = 0; d < (int)n.labels.size() && d < cap; ++d) {
        if (labels) labels[d] = n.labels[d];
        if (dims) dims[d] = n.dims[d];
    }
    return (int32_t)n.labels.size();
}
int32_t tfh_tree_output_rank(const tfh_tree* t) { return t ? (int32_t)t->output_dims.size() : -1; }
int32_t tfh_tree_output_dims(const tfh_tree* t, int64_t* dims, int32_t cap) {
    if (!t) return -1;
    for (int d = 0; d < (int)t->output_dims.size() && d < cap; ++d) dims[d] = t->output_dims[d];
    return (int32_t)t->output_dims.size();
}
double tfh_tree_mac_count(const tfh_tree* t) { return t ? t->macs : 0; }
double tfh_tree_peak_intermediate(const tfh_tree* t) { return t ? t->peak : 0; }

// ---- executor ----------------------------------------------------------------------------------------------
}  // extern "C"

namespace {
struct Operand {          // a node as the executor sees it: unique labels + strides
    std::vector<uint32_t> labels;
    std::vector<int64_t> dims, strides;
    char* ptr = nullptr;
    void* owned = nullptr;   // pool block to release once consumed
    bool conj = false;       // read as conj(element): an input view flagged TFH_VIEW_CONJ (complex dtypes)
};

// Diagonal view over repeated labels (zero-copy, tenferro-tensor/src/lib.rs:518-529).
Operand unique_view(const std::vector<uint32_t>& labels, const int64_t* dims, const int64_t* strides, char* ptr) {
    Operand o;
    o.ptr = ptr;
    for (size_t d = 0; d < labels.size(); ++d) {
        int j = find(o.labels, labels[d]);
        if (j < 0) {
            o.labels.push_back(labels[d]);
            o.dims.push_back(dims[d]);
            o.strides.push_back(strides[d]);
        } else
            o.strides[j] += strides[d];
    }
    return o;
}

int64_t count(const std::vector<int64_t>& dims) {
    int64_t n = 1;
    for (int64_t d : dims) n *= d;
    return n;
}

// dst[dst_labels] = alpha * sum over missing labels of op(src) + beta*dst, op = conj when src.conj
int32_t reduce_or_copy(int dtype, const Operand& src, const Operand& dst, Scalar alpha, Scalar beta, void* stream) {
    std::vector<Axis> kept, red;
    for (size_t d = 0; d < dst.labels.size(); ++d) {
        int j = find(src.labels, dst.labels[d]);
        kept.push_back(Axis{dst.dims[d], {src.strides[j], dst.strides[d], 0}, dst.labels[d]});
    }
    for (size_t j = 0; j < src.labels.size(); ++j)
        if (find(dst.labels, src.labels[j]) < 0) red.push_back(Axis{src.dims[j], {src.strides[j], 0, 0}, src.labels[j]});
    if (red.empty()) return launch_copy(dtype, src.ptr, dst.ptr, kept, alpha, beta, src.conj, stream);
    if (!src.conj) return launch_reduce(dtype, src.ptr, dst.ptr, kept, red, TFH_REDUCE_SUM, alpha, beta, stream);
    // a flagged operand that is summed: a conjugated dense copy first (the reduction kernels do not conjugate)
    std::vector<Axis> all;
    int64_t n = 1;
    for (size_t j = src.labels.size(); j-- > 0;) {
        all.push_back(Axis{src.dims[j], {src.strides[j], n, 0}, src.labels[j]});
        n *= src.dims[j];
    }
    void* tmp = nullptr;
    if (int32_t e = pool_alloc(stream, (size_t)std::max<int64_t>(n, 1) * dtype_size(dtype), &tmp)) return e;
    int32_t e = launch_copy(dtype, src.ptr, tmp, all, Scalar{1, 0}, Scalar{0, 0}, true, stream);
    if (!e) {
        Operand dense = src;
        dense.ptr = (char*)tmp;
        dense.conj = false;
        int64_t st = 1;
        for (size_t j = src.labels.size(); j-- > 0;) {
            dense.strides[j] = st;
            st *= src.dims[j];
        }
        e = reduce_or_copy(dtype, dense, dst, alpha, beta, stream);
    }
    pool_free(stream, tmp);
    return e;
}
}  // namespace

extern "C" {

int32_t tfh_einsum_execute(int32_t dtype, const tfh_tree* tree, const tfh_view* operands, int32_t n_operands,
                           const void* alpha, const void* beta, tfh_view* output, uint64_t donate_mask, tfh_stream stream) {
    if (!tree || !alpha || !beta || !output || (n_operands > 0 && !operands)) return set_error(TFH_ERR_INVALID_ARGUMENT, "null argument");
    if (dtype < TFH_F32 || dtype > TFH_C128) return set_error(TFH_ERR_INVALID_ARGUMENT, "unknown dtype %d", dtype);
    const tfh_tree& t = *tree;
    if (n_operands != t.n_inputs) return set_error(TFH_ERR_INVALID_ARGUMENT, "tree was built for %d operands, got %d", t.n_inputs, n_operands);
    for (int i = 0; i < n_operands; ++i) {
        if (int32_t e = check_view_against(t.input_dims[i], operands[i], "operand")) return e;
        if (!operands[i].base) return set_error(TFH_ERR_INVALID_ARGUMENT, "operand %d has a null base pointer", i);
    }
    if (int32_t e = check_view_against(t.output_dims, *output, "output")) return e;
    if (!output->base) return set_error(TFH_ERR_INVALID_ARGUMENT, "output has a null base pointer");
    if (output->flags & TFH_VIEW_CONJ) return set_error(TFH_ERR_INVALID_ARGUMENT, "TFH_VIEW_CONJ on an output view");
    const Scalar al = load_scalar(dtype, alpha), be = load_scalar(dtype, beta);
    const size_t eb = dtype_size(dtype);
    const Scalar one{1, 0}, zero{0, 0};

    // the output as a unique-label view; a repeated output label addresses a diagonal, everything off the
    // diagonal receives beta*output only
    Operand outv = unique_view(t.output_labels, output->dims, output->strides, view_ptr(*output, dtype));
    Scalar be_final = be;
    if (outv.labels.size() != t.output_labels.size()) {
        std::vector<Axis> all;
        for (int d = 0; d < output->rank; ++d) all.push_back(Axis{output->dims[d], {output->strides[d], output->strides[d], 0}, 0});
        int32_t e = TFH_OK;
        if (be.is_zero()) e = launch_fill(dtype, outv.ptr, all, zero, stream);
        else if (!be.is_one()) e = launch_copy(dtype, outv.ptr, outv.ptr, all, be, zero, false, stream);
        if (e) return e;
        be_final = one;
    }

    std::vector<Operand> nodes((size_t)t.nodes.size());
    std::vector<void*> to_free;
    auto release_all = [&]() {
        for (void* p : to_free) pool_free(stream, p);
    };
    // leaves: diagonal views; labels private to one operand are summed into a temporary first
    for (int i = 0; i < n_operands; ++i) {
        Operand v = unique_view(t.input_labels[i], operands[i].dims, operands[i].strides, view_ptr(operands[i], dtype));
        v.conj = (operands[i].flags & TFH_VIEW_CONJ) && is_complex(dtype);
        const TreeNode& leaf = t.nodes[i];
        if (n_operands == 1 || v.labels.size() == leaf.labels.size()) {
            nodes[i] = v;
            continue;
        }
        Operand r;
        r.labels = leaf.labels;
        r.dims = leaf.dims;
        r.strides.assign(r.labels.size(), 0);
        int64_t n = 1;
        for (int d = (int)r.labels.size() - 1; d >= 0; --d) {
            r.strides[d] = n;
            n *= r.dims[d];
        }
        void* p = nullptr;
        if (int32_t e = pool_alloc(stream, (size_t)std::max<int64_t>(n, 1) * eb, &p)) {
            release_all();
            return e;
        }
        to_free.push_back(p);
        r.ptr = (char*)p;
        if (int32_t e = reduce_or_copy(dtype, v, r, one, zero, stream)) {
            release_all();
            return e;
        }
        nodes[i] = r;
    }
    if (t.steps.empty()) {
        // single operand: permute / diagonal / trace / reduce straight into the output
        int32_t e = reduce_or_copy(dtype, nodes[0], outv, al, be_final, stream);
        release_all();
        if (!e) clear_error();
        return e;
    }
    const int ns = (int)t.steps.size();
    // Donated operands (the *_owned variants, tenferro-einsum/src/lib.rs:436-498): once the step that consumes one
    // has been enqueued, its buffer is dead and may hold a later intermediate.  Only a dense view qualifies (its
    // elements occupy one contiguous block), and the kernels that read it precede the writer on the same stream.
    struct Donated { char* ptr; size_t bytes; int consumed_at; bool used; };
    std::vector<Donated> donated;
    for (int i = 0; i < n_operands && i < 64; ++i) {
        if (!((donate_mask >> i) & 1)) continue;
        const tfh_view& v = operands[i];
        std::vector<std::pair<int64_t, int64_t>> ax;   // (|stride|, extent) of the non-trivial axes
        bool dense = true;
        int64_t count = 1;
        for (int d = 0; d < v.rank; ++d) {
            count *= v.dims[d];
            if (v.dims[d] > 1) {
                if (v.strides[d] <= 0) dense = false;
                ax.emplace_back(v.strides[d], v.dims[d]);
            }
        }
        std::sort(ax.begin(), ax.end());
        int64_t expect = 1;
        for (auto& a : ax) {
            if (a.first != expect) dense = false;
            expect *= a.second;
        }
        if (!dense || count == 0) continue;
        int consumed = -1;
        for (int s = 0; s < ns; ++s)
            if (t.steps[s].lhs == i || t.steps[s].rhs == i) consumed = s;
        if (consumed < 0) continue;
        // the block must be this operand's alone: no other operand and not the output may reach into it
        auto range = [&](const tfh_view& w, const char*& lo, const char*& hi) {
            int64_t a = 0, b = 0;
            for (int d = 0; d < w.rank; ++d) {
                if (w.dims[d] <= 1) continue;
                const int64_t e = (w.dims[d] - 1) * w.strides[d];
                (e < 0 ? a : b) += e;
            }
            lo = view_ptr(w, dtype) + a * (int64_t)eb;
            hi = view_ptr(w, dtype) + (b + 1) * (int64_t)eb;
        };
        const char* lo = view_ptr(v, dtype);
        const char* hi = lo + (size_t)count * eb;
        bool alone = true;
        for (int j = 0; j <= n_operands && alone; ++j) {
            if (j == i) continue;
            const char *l2, *h2;
            range(j < n_operands ? operands[j] : *output, l2, h2);
            if (l2 < hi && lo < h2) alone = false;
        }
        if (!alone) continue;
        donated.push_back(Donated{view_ptr(v, dtype), (size_t)count * eb, consumed, false});
    }
    ContractCache* const* step_caches = nullptr;
    {
        std::lock_guard<std::mutex> lk(t.step_mu);
        if (t.step_cache.empty() && ns > 0) {
            t.step_cache.resize((size_t)ns, nullptr);
            for (auto& c : t.step_cache) c = contract_cache_create();
        }
        step_caches = t.step_cache.data();   // (the vector is sized once and never touched again)
    }
    for (int s = 0; s < ns; ++s) {
        const bool last = s == ns - 1;
        const Operand& A = nodes[t.steps[s].lhs];
        const Operand& B = nodes[t.steps[s].rhs];
        const TreeNode& tn = t.nodes[(size_t)t.n_inputs + s];
        Operand C;
        if (last) {
            C = outv;
        } else {
            C.labels = tn.labels;
            C.dims = tn.dims;
            C.strides.assign(C.labels.size(), 0);
            int64_t n = 1;
            for (int d = (int)C.labels.size() - 1; d >= 0; --d) {
                C.strides[d] = n;
                n *= C.dims[d];
            }
            const size_t need = (size_t)std::max<int64_t>(n, 1) * eb;
            Donated* reuse = nullptr;
            for (auto& dn : donated)   // smallest donated buffer that fits and whose reader is already enqueued
                if (!dn.used && dn.consumed_at < s && dn.bytes >= need && (!reuse || dn.bytes < reuse->bytes)) reuse = &dn;
            if (reuse) {
                reuse->used = true;
                C.ptr = reuse->ptr;
            } else {
                void* p = nullptr;
                if (int32_t e = pool_alloc(stream, need, &p)) {
                    release_all();
                    return e;
                }
                C.ptr = (char*)p;
                C.owned = p;
            }
        }
        int32_t e = execute_contract(step_caches[s], dtype, A.labels, A.dims.data(), A.strides.data(), A.ptr, B.labels, B.dims.data(),
                                     B.strides.data(), B.ptr, C.labels, C.dims.data(), C.strides.data(), C.ptr, last ? al : one,
                                     last ? be_final : zero, stream, (A.conj ? 1 : 0) | (B.conj ? 2 : 0));
        // operands of this step are dead once its kernels are enqueued (stream order protects them)
        for (int side = 0; side < 2; ++side) {
            Operand& o = nodes[side ? t.steps[s].rhs : t.steps[s].lhs];
            if (o.owned) {
                pool_free(stream, o.owned);
                o.owned = nullptr;
            }
        }
        if (e) {
            if (C.owned) pool_free(stream, C.owned);
            release_all();
            return e;
        }
        nodes[(size_t)t.n_inputs + s] = C;
    }
    release_all();
    clear_error();
    return TFH_OK;
}

}  // extern "C"

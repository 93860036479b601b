// plan.cpp -- TensorPrims::plan for the Hip backend: validates a PrimDescriptor against the shapes
// (tenferro-prims/src/lib.rs:282-298) and keeps the normalised descriptor.  Pure host code.
#include <algorithm>
#include <cstring>
#include <map>
#include <set>

#include "internal.hpp"

tfh_plan::~tfh_plan() {
    if (grouped) tfh::grouped_state_destroy(grouped);
    if (contract_cache) tfh::contract_cache_destroy(contract_cache);
}

namespace tfh {
namespace {

int find(const std::vector<uint32_t>& m, uint32_t l) {
    for (size_t i = 0; i < m.size(); ++i)
        if (m[i] == l) return (int)i;
    return -1;
}
bool repeats(const std::vector<uint32_t>& m) {
    std::set<uint32_t> s(m.begin(), m.end());
    return s.size() != m.size();
}
std::vector<uint32_t> modes_of(const uint32_t* p, int n) { return p && n > 0 ? std::vector<uint32_t>(p, p + n) : std::vector<uint32_t>(); }

// Checks rank == number of modes and that every label has one extent across the tensors.
// The "expected" shape of a tensor is what the labels seen so far imply for it.
int32_t bind_extents(const std::vector<uint32_t>& modes, const std::vector<int64_t>& shape,
                     std::map<uint32_t, int64_t>& ext) {
    if (modes.size() != shape.size()) return set_rank_mismatch((int64_t)modes.size(), (int64_t)shape.size());
    bool bad = false;
    std::vector<int64_t> expected = shape;
    for (size_t d = 0; d < modes.size(); ++d) {
        auto it = ext.find(modes[d]);
        if (it == ext.end()) ext[modes[d]] = shape[d];
        else if (it->second != shape[d]) {
            expected[d] = it->second;
            bad = true;
        }
    }
    if (bad) return set_shape_mismatch(expected.data(), (int)expected.size(), shape.data(), (int)shape.size());
    return TFH_OK;
}

int32_t need_tensors(int32_t n_tensors, int32_t want, const char* op) {
    if (n_tensors != want) return set_error(TFH_ERR_INVALID_ARGUMENT, "%s takes %d shapes (inputs then output), got %d", op, want, n_tensors);
    return TFH_OK;
}

}  // namespace

int32_t check_view_against(const std::vector<int64_t>& shape, const tfh_view& v, const char* what) {
    if (v.rank < 0 || v.rank > TFH_MAX_RANK) return set_error(TFH_ERR_INVALID_ARGUMENT, "%s: rank %d out of range", what, v.rank);
    if ((size_t)v.rank != shape.size()) return set_rank_mismatch((int64_t)shape.size(), v.rank);
    for (int d = 0; d < v.rank; ++d)
        if (v.dims[d] != shape[d]) return set_shape_mismatch(shape.data(), (int)shape.size(), v.dims, v.rank);
    return TFH_OK;
}

int32_t classify_contract(const std::vector<uint32_t>& ma, const int64_t* dims_a, const int64_t* str_a,
                          const std::vector<uint32_t>& mb, const int64_t* dims_b, const int64_t* str_b,
                          const std::vector<uint32_t>& mc, const int64_t* dims_c, const int64_t* str_c,
                          ContractAxes& out) {
    std::set<uint32_t> seen;
    auto add = [&](uint32_t l) {
        if (!seen.insert(l).second) return;
        int ia = find(ma, l), ib = find(mb, l), ic = find(mc, l);
        int64_t n = ia >= 0 ? dims_a[ia] : (ib >= 0 ? dims_b[ib] : dims_c[ic]);
        Axis ax{n, {ia >= 0 ? str_a[ia] : 0, ib >= 0 ? str_b[ib] : 0, ic >= 0 ? str_c[ic] : 0}, l};
        // modes shared between inputs and output are batch/free dimensions; modes present only in
        // inputs are contracted (tenferro-prims/src/lib.rs:136-138)
        if (ic >= 0) {
            if (ia >= 0 && ib >= 0) out.batch.push_back(ax);
            else if (ia >= 0) out.M.push_back(ax);
            else out.N.push_back(ax);
        } else
            out.K.push_back(ax);  // an input that lacks a summed mode sees it with stride 0
    };
    // group order follows the output first (so that fused output indices walk C's memory), then A, then B
    for (uint32_t l : mc) add(l);
    for (uint32_t l : ma) add(l);
    for (uint32_t l : mb) add(l);
    return TFH_OK;
}

void fuse_axes(std::vector<Axis>& ax, int nslots) {
    std::vector<Axis> r;
    for (const Axis& a : ax) {
        if (a.n == 1) continue;
        if (!r.empty()) {
            Axis& p = r.back();
            bool ok = true;
            for (int s = 0; s < nslots; ++s) ok &= p.s[s] == a.s[s] * a.n;
            if (ok) {
                p.n *= a.n;
                for (int s = 0; s < nslots; ++s) p.s[s] = a.s[s];
                continue;
            }
        }
        r.push_back(a);
    }
    ax.swap(r);
}

int32_t make_plan(int32_t dtype, const tfh_desc* desc, const int64_t* const* shapes, const int32_t* ranks,
                  int32_t n_tensors, tfh_plan& plan) {
    if (dtype < TFH_F32 || dtype > TFH_C128) return set_error(TFH_ERR_INVALID_ARGUMENT, "unknown dtype %d", dtype);
    if (!desc) return set_error(TFH_ERR_INVALID_ARGUMENT, "null descriptor");
    if (n_tensors < 0 || (n_tensors > 0 && (!shapes || !ranks))) return set_error(TFH_ERR_INVALID_ARGUMENT, "null shapes");
    plan.dtype = dtype;
    plan.op = desc->op;
    plan.reduce_op = desc->reduce_op;
    plan.shapes.clear();
    for (int t = 0; t < n_tensors; ++t) {
        if (ranks[t] < 0 || ranks[t] > TFH_MAX_RANK)
            return set_error(TFH_ERR_INVALID_ARGUMENT, "tensor %d has rank %d; at most %d axes are supported", t, ranks[t], TFH_MAX_RANK);
        plan.shapes.emplace_back(shapes[t], shapes[t] + ranks[t]);
        for (int64_t d : plan.shapes.back())
            if (d < 0) return set_error(TFH_ERR_INVALID_ARGUMENT, "tensor %d has a negative extent", t);
    }
    plan.modes_a = modes_of(desc->modes_a, desc->n_modes_a);
    plan.modes_b = modes_of(desc->modes_b, desc->n_modes_b);
    plan.modes_c = modes_of(desc->modes_c, desc->n_modes_c);
    plan.pairs.clear();
    for (int p = 0; p < desc->n_pairs; ++p) plan.pairs.emplace_back(desc->paired[2 * p], desc->paired[2 * p + 1]);
    std::map<uint32_t, int64_t> ext;
    const auto& sh = plan.shapes;
    switch (desc->op) {
        case TFH_OP_BATCHED_GEMM: {
            if (int32_t e = need_tensors(n_tensors, 3, "BatchedGemm")) return e;
            if (desc->n_batch_dims < 0 || desc->n_batch_dims + 2 > TFH_MAX_RANK || desc->m < 0 || desc->n < 0 || desc->k < 0)
                return set_error(TFH_ERR_INVALID_ARGUMENT, "BatchedGemm: bad batch_dims/m/n/k");
            // C[batch, m, n] = alpha*A[batch, m, k]*B[batch, k, n] + beta*C (tenferro-prims/src/lib.rs:156-168)
            uint32_t nb = (uint32_t)desc->n_batch_dims;
            std::vector<int64_t> ea, eb, ec;
            plan.modes_a.clear(); plan.modes_b.clear(); plan.modes_c.clear();
            for (uint32_t i = 0; i < nb; ++i) {
                plan.modes_a.push_back(i); plan.modes_b.push_back(i); plan.modes_c.push_back(i);
                ea.push_back(desc->batch_dims[i]); eb.push_back(desc->batch_dims[i]); ec.push_back(desc->batch_dims[i]);
            }
            uint32_t lm = nb, ln = nb + 1, lk = nb + 2;
            plan.modes_a.push_back(lm); plan.modes_a.push_back(lk); ea.push_back(desc->m); ea.push_back(desc->k);
            plan.modes_b.push_back(lk); plan.modes_b.push_back(ln); eb.push_back(desc->k); eb.push_back(desc->n);
            plan.modes_c.push_back(lm); plan.modes_c.push_back(ln); ec.push_back(desc->m); ec.push_back(desc->n);
            const std::vector<int64_t>* want[3] = {&ea, &eb, &ec};
            for (int t = 0; t < 3; ++t) {
                if (sh[t].size() != want[t]->size()) return set_rank_mismatch((int64_t)want[t]->size(), (int64_t)sh[t].size());
                if (sh[t] != *want[t]) return set_shape_mismatch(want[t]->data(), (int)want[t]->size(), sh[t].data(), (int)sh[t].size());
            }
            plan.n_inputs = 2;
            break;
        }
        case TFH_OP_CONTRACT: {
            if (int32_t e = need_tensors(n_tensors, 3, "Contract")) return e;
            if (repeats(plan.modes_a) || repeats(plan.modes_b) || repeats(plan.modes_c))
                return set_error(TFH_ERR_INVALID_ARGUMENT, "Contract: a mode label is repeated inside one operand");
            if (int32_t e = bind_extents(plan.modes_a, sh[0], ext)) return e;
            if (int32_t e = bind_extents(plan.modes_b, sh[1], ext)) return e;
            for (uint32_t l : plan.modes_c)
                if (find(plan.modes_a, l) < 0 && find(plan.modes_b, l) < 0)
                    return set_error(TFH_ERR_INVALID_ARGUMENT, "Contract: output mode %u appears in no input", l);
            if (int32_t e = bind_extents(plan.modes_c, sh[2], ext)) return e;
            plan.n_inputs = 2;
            break;
        }
        case TFH_OP_PERMUTE: {
            if (int32_t e = need_tensors(n_tensors, 2, "Permute")) return e;
            if (repeats(plan.modes_a) || repeats(plan.modes_c))
                return set_error(TFH_ERR_INVALID_ARGUMENT, "Permute: a mode label is repeated");
            if (int32_t e = bind_extents(plan.modes_a, sh[0], ext)) return e;
            if (plan.modes_c.size() != plan.modes_a.size())
                return set_rank_mismatch((int64_t)plan.modes_a.size(), (int64_t)plan.modes_c.size());
            for (uint32_t l : plan.modes_c)
                if (find(plan.modes_a, l) < 0)
                    return set_error(TFH_ERR_INVALID_ARGUMENT, "Permute: output mode %u is not an input mode", l);
            if (int32_t e = bind_extents(plan.modes_c, sh[1], ext)) return e;
            plan.n_inputs = 1;
            break;
        }
        case TFH_OP_REDUCE: {
            if (int32_t e = need_tensors(n_tensors, 2, "Reduce")) return e;
            if (desc->reduce_op < TFH_REDUCE_SUM || desc->reduce_op > TFH_REDUCE_MIN)
                return set_error(TFH_ERR_INVALID_ARGUMENT, "Reduce: unknown reduce_op %d", desc->reduce_op);
            if (is_complex(dtype) && desc->reduce_op != TFH_REDUCE_SUM)
                return set_error(TFH_ERR_INVALID_ARGUMENT, "Reduce: max/min are undefined for complex types");
            if (repeats(plan.modes_a) || repeats(plan.modes_c))
                return set_error(TFH_ERR_INVALID_ARGUMENT, "Reduce: a mode label is repeated");
            if (int32_t e = bind_extents(plan.modes_a, sh[0], ext)) return e;
            for (uint32_t l : plan.modes_c)
                if (find(plan.modes_a, l) < 0)
                    return set_error(TFH_ERR_INVALID_ARGUMENT, "Reduce: output mode %u is not an input mode (modes_c must be a subset of modes_a)", l);
            if (int32_t e = bind_extents(plan.modes_c, sh[1], ext)) return e;
            plan.n_inputs = 1;
            break;
        }
        case TFH_OP_ELEMENTWISE_MUL: {
            if (int32_t e = need_tensors(n_tensors, 3, "ElementwiseMul")) return e;
            for (int t = 0; t < 2; ++t) {
                if (sh[t].size() != sh[2].size()) return set_rank_mismatch((int64_t)sh[2].size(), (int64_t)sh[t].size());
                if (sh[t] != sh[2]) return set_shape_mismatch(sh[2].data(), (int)sh[2].size(), sh[t].data(), (int)sh[t].size());
            }
            plan.n_inputs = 2;
            break;
        }
        case TFH_OP_TRACE:
        case TFH_OP_ANTI_TRACE:
        case TFH_OP_ANTI_DIAG: {
            const char* name = desc->op == TFH_OP_TRACE ? "Trace" : desc->op == TFH_OP_ANTI_TRACE ? "AntiTrace" : "AntiDiag";
            if (int32_t e = need_tensors(n_tensors, 2, name)) return e;
            if (repeats(plan.modes_a) || repeats(plan.modes_c))
                return set_error(TFH_ERR_INVALID_ARGUMENT, "%s: a mode label is repeated", name);
            if (desc->n_pairs < 0 || (desc->n_pairs > 0 && !desc->paired)) return set_error(TFH_ERR_INVALID_ARGUMENT, "%s: bad pairs", name);
            // the tensor that carries both members of each pair: the input for Trace, the output otherwise
            bool fwd = desc->op == TFH_OP_TRACE;
            const std::vector<uint32_t>& full = fwd ? plan.modes_a : plan.modes_c;
            const std::vector<uint32_t>& small = fwd ? plan.modes_c : plan.modes_a;
            if (int32_t e = bind_extents(full, sh[fwd ? 0 : 1], ext)) return e;
            std::set<uint32_t> used;
            for (auto& pr : plan.pairs) {
                int i = find(full, pr.first), j = find(full, pr.second);
                if (i < 0 || j < 0 || i == j || !used.insert(pr.first).second || !used.insert(pr.second).second)
                    return set_error(TFH_ERR_INVALID_ARGUMENT, "%s: pair (%u,%u) must name two distinct, unpaired modes of the %s",
                                     name, pr.first, pr.second, fwd ? "input" : "output");
                if (ext[pr.first] != ext[pr.second]) {
                    std::vector<int64_t> want = sh[fwd ? 0 : 1];
                    want[j] = want[i];
                    return set_shape_mismatch(want.data(), (int)want.size(), sh[fwd ? 0 : 1].data(), (int)want.size());
                }
                bool i_in_small = find(small, pr.first) >= 0, j_in_small = find(small, pr.second) >= 0;
                bool want_i = desc->op == TFH_OP_ANTI_DIAG;  // AntiDiag's input still carries mode i
                if (j_in_small || i_in_small != want_i)
                    return set_error(TFH_ERR_INVALID_ARGUMENT, "%s: paired modes (%u,%u) are misplaced in the %s modes", name,
                                     pr.first, pr.second, fwd ? "output" : "input");
            }
            for (uint32_t l : small)
                if (find(full, l) < 0) return set_error(TFH_ERR_INVALID_ARGUMENT, "%s: mode %u is missing from the %s", name, l, fwd ? "input" : "output");
            if (!fwd)
                for (uint32_t l : full)
                    if (find(small, l) < 0 && !used.count(l))
                        return set_error(TFH_ERR_INVALID_ARGUMENT, "%s: output mode %u is neither paired nor an input mode", name, l);
            if (int32_t e = bind_extents(small, sh[fwd ? 1 : 0], ext)) return e;
            plan.n_inputs = 1;
            break;
        }
        default:
            return set_error(TFH_ERR_INVALID_ARGUMENT, "unknown operation %d", desc->op);
    }
    return TFH_OK;
}

}  // namespace tfh

extern "C" {

int32_t tfh_has_extension(int32_t dtype, int32_t ext) {
    // Fused contraction and element-wise multiplication exist for the whole Standard-algebra dtype
    // set (tenferro-prims/src/lib.rs:322-339; tenferro-algebra/src/lib.rs:58-72).
    if (dtype < TFH_F32 || dtype > TFH_C128) return 0;
    return ext == TFH_EXT_CONTRACT || ext == TFH_EXT_ELEMENTWISE_MUL;
}

int32_t tfh_plan_create(int32_t dtype, const tfh_desc* desc, const int64_t* const* shapes, const int32_t* ranks,
                        int32_t n_tensors, tfh_plan** out) {
    if (!out) return tfh::set_error(TFH_ERR_INVALID_ARGUMENT, "null output pointer");
    *out = nullptr;
    tfh_plan* p = new (std::nothrow) tfh_plan();
    if (!p) return tfh::set_error(TFH_ERR_DEVICE, "out of host memory");
    int32_t e = tfh::make_plan(dtype, desc, shapes, ranks, n_tensors, *p);
    if (e) {
        delete p;
        return e;
    }
    // kernel selection happens at the first execute with a given set of view strides and is kept here (a plan that
    // could not get the cache still works: every execute then routes afresh)
    if (p->op == TFH_OP_CONTRACT || p->op == TFH_OP_BATCHED_GEMM) p->contract_cache = tfh::contract_cache_create();
    *out = p;
    tfh::clear_error();
    return TFH_OK;
}

int32_t tfh_plan_create_grouped(int32_t dtype, const tfh_desc* desc, int32_t n_groups, const int64_t* const* shapes,
                                const int32_t* ranks, int32_t n_tensors, tfh_plan** out) {
    if (!out) return tfh::set_error(TFH_ERR_INVALID_ARGUMENT, "null output pointer");
    *out = nullptr;
    if (n_groups <= 0) return tfh::set_error(TFH_ERR_INVALID_ARGUMENT, "grouped plan needs at least one group");
    if (!desc || (desc->op != TFH_OP_CONTRACT && desc->op != TFH_OP_BATCHED_GEMM))
        return tfh::set_error(TFH_ERR_INVALID_ARGUMENT, "grouped execution exists for Contract and BatchedGemm only");
    if (n_tensors != 3) return tfh::set_error(TFH_ERR_INVALID_ARGUMENT, "grouped contraction takes 3 shapes per group");
    tfh_plan* p = new (std::nothrow) tfh_plan();
    if (!p) return tfh::set_error(TFH_ERR_DEVICE, "out of host memory");
    std::vector<std::vector<int64_t>> all;
    for (int g = 0; g < n_groups; ++g) {
        tfh_desc d = *desc;
        if (desc->op == TFH_OP_BATCHED_GEMM) {
            // extents of a grouped BatchedGemm come from each group's shapes, not from the descriptor
            const int64_t* sa = shapes[g * 3 + 0];
            const int64_t* sb = shapes[g * 3 + 1];
            int nb = desc->n_batch_dims;
            if (ranks[0] != nb + 2 || ranks[1] != nb + 2 || ranks[2] != nb + 2) {
                delete p;
                return tfh::set_rank_mismatch(nb + 2, ranks[0] != nb + 2 ? ranks[0] : ranks[1] != nb + 2 ? ranks[1] : ranks[2]);
            }
            d.batch_dims = sa;
            d.m = sa[nb];
            d.k = sa[nb + 1];
            d.n = sb[nb + 1];
        }
        int32_t e = tfh::make_plan(dtype, &d, shapes + (size_t)g * 3, ranks, 3, *p);
        if (e) {
            delete p;
            return e;
        }
        for (auto& s : p->shapes) all.push_back(s);
    }
    p->shapes.swap(all);
    p->n_groups = n_groups;
    int32_t e = tfh::grouped_plan_init(*p);
    if (e) {
        delete p;
        return e;
    }
    *out = p;
    tfh::clear_error();
    return TFH_OK;
}

void tfh_plan_destroy(tfh_plan* plan) { delete plan; }

}  // extern "C"

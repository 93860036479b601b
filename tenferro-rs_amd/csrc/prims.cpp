// prims.cpp -- TensorPrims::execute for the Hip backend (tenferro-prims/src/lib.rs:300-320):
// output = alpha*op(inputs) + beta*output, dispatched on the plan's descriptor to the kernel
// launchers.  Also Tensor::conj and zeros/ones on device memory.
#include <algorithm>
#include <cstring>

#include "internal.hpp"

namespace tfh {
namespace {

int find(const std::vector<uint32_t>& m, uint32_t l) {
    for (size_t i = 0; i < m.size(); ++i)
        if (m[i] == l) return (int)i;
    return -1;
}

// Collapses each pair (i, j) on a view into the single mode i whose stride is the sum of both strides:
// the zero-copy diagonal of tenferro-tensor/src/lib.rs:518-529.
struct ModedView {
    std::vector<uint32_t> modes;
    std::vector<int64_t> dims, strides;
};
ModedView diagonal_view(const tfh_view& v, const std::vector<uint32_t>& modes, const std::vector<std::pair<uint32_t, uint32_t>>& pairs) {
    ModedView r;
    r.modes = modes;
    r.dims.assign(v.dims, v.dims + v.rank);
    r.strides.assign(v.strides, v.strides + v.rank);
    for (auto& pr : pairs) {
        int i = find(r.modes, pr.first), j = find(r.modes, pr.second);
        r.strides[i] += r.strides[j];
        r.modes.erase(r.modes.begin() + j);
        r.dims.erase(r.dims.begin() + j);
        r.strides.erase(r.strides.begin() + j);
    }
    return r;
}

int32_t exec_permute(const tfh_plan& p, Scalar alpha, const tfh_view& a, Scalar beta, tfh_view& b, void* stream) {
    std::vector<Axis> ax;
    for (int d = 0; d < b.rank; ++d) {
        int j = find(p.modes_a, p.modes_c[d]);
        ax.push_back(Axis{b.dims[d], {a.strides[j], b.strides[d], 0}, p.modes_c[d]});
    }
    const bool conj = (a.flags & TFH_VIEW_CONJ) && is_complex(p.dtype);
    return launch_copy(p.dtype, view_ptr(a, p.dtype), view_ptr(b, p.dtype), ax, alpha, beta, conj, stream);
}

int32_t reduce_moded(int dtype, const char* a_ptr, const ModedView& a, char* c_ptr, const tfh_view& c,
                     const std::vector<uint32_t>& modes_c, int op, Scalar alpha, Scalar beta, void* stream) {
    std::vector<Axis> kept, red;
    for (int d = 0; d < c.rank; ++d) {
        int j = find(a.modes, modes_c[d]);
        kept.push_back(Axis{c.dims[d], {a.strides[j], c.strides[d], 0}, modes_c[d]});
    }
    for (size_t j = 0; j < a.modes.size(); ++j)
        if (find(modes_c, a.modes[j]) < 0) red.push_back(Axis{a.dims[j], {a.strides[j], 0, 0}, a.modes[j]});
    return launch_reduce(dtype, a_ptr, c_ptr, kept, red, op, alpha, beta, stream);
}

// AntiTrace / AntiDiag: C = beta*C everywhere, then diagonal(C) += alpha*A (A broadcast over a pair label
// it does not carry).  tenferro-prims/src/lib.rs:204-222.
int32_t exec_anti(const tfh_plan& p, Scalar alpha, const tfh_view& a, Scalar beta, tfh_view& c, void* stream) {
    std::vector<Axis> all;
    for (int d = 0; d < c.rank; ++d) all.push_back(Axis{c.dims[d], {c.strides[d], c.strides[d], 0}, p.modes_c[d]});
    char* cp = view_ptr(c, p.dtype);
    int32_t e;
    if (beta.is_zero()) e = launch_fill(p.dtype, cp, all, Scalar{0, 0}, stream);
    else if (beta.is_one()) e = TFH_OK;
    else e = launch_copy(p.dtype, cp, cp, all, beta, Scalar{0, 0}, false, stream);
    if (e) return e;
    ModedView dv = diagonal_view(c, p.modes_c, p.pairs);
    std::vector<Axis> ax;
    for (size_t d = 0; d < dv.modes.size(); ++d) {
        int j = find(p.modes_a, dv.modes[d]);
        ax.push_back(Axis{dv.dims[d], {j >= 0 ? a.strides[j] : 0, dv.strides[d], 0}, dv.modes[d]});
    }
    return launch_copy(p.dtype, view_ptr(a, p.dtype), cp, ax, alpha, Scalar{1, 0}, false, stream);
}

}  // namespace
}  // namespace tfh

using namespace tfh;

extern "C" {

int32_t tfh_execute(const tfh_plan* plan, const void* alpha, const tfh_view* inputs, int32_t n_inputs, const void* beta,
                    tfh_view* output, tfh_stream stream) {
    if (!plan || !alpha || !beta || !output || (n_inputs > 0 && !inputs)) return set_error(TFH_ERR_INVALID_ARGUMENT, "null argument");
    if (plan->n_groups) return set_error(TFH_ERR_INVALID_ARGUMENT, "grouped plan: use tfh_execute_grouped");
    if (n_inputs != plan->n_inputs) return set_error(TFH_ERR_INVALID_ARGUMENT, "plan takes %d inputs, got %d", plan->n_inputs, n_inputs);
    for (int t = 0; t < n_inputs; ++t)
        if (int32_t e = check_view_against(plan->shapes[t], inputs[t], "input")) return e;
    if (int32_t e = check_view_against(plan->shapes[n_inputs], *output, "output")) return e;
    auto empty = [](const tfh_view& v) {
        for (int d = 0; d < v.rank; ++d)
            if (v.dims[d] == 0) return true;
        return false;
    };
    for (int t = 0; t < n_inputs; ++t)
        if (!inputs[t].base && !empty(inputs[t])) return set_error(TFH_ERR_INVALID_ARGUMENT, "input %d has a null base pointer", t);
    if (!output->base && !empty(*output)) return set_error(TFH_ERR_INVALID_ARGUMENT, "output has a null base pointer");
    const int dt = plan->dtype;
    const Scalar al = load_scalar(dt, alpha), be = load_scalar(dt, beta);
    int32_t e = TFH_OK;
    // TFH_VIEW_CONJ: inputs of Contract, BatchedGemm and Permute only
    if (output->flags & TFH_VIEW_CONJ) return set_error(TFH_ERR_INVALID_ARGUMENT, "TFH_VIEW_CONJ on an output view");
    int conj = 0;
    for (int t = 0; t < n_inputs; ++t)
        if ((inputs[t].flags & TFH_VIEW_CONJ) && is_complex(dt)) conj |= 1 << t;
    if (conj && plan->op != TFH_OP_CONTRACT && plan->op != TFH_OP_BATCHED_GEMM && plan->op != TFH_OP_PERMUTE)
        return set_error(TFH_ERR_INVALID_ARGUMENT, "TFH_VIEW_CONJ is honoured by Contract, BatchedGemm and Permute only (operation %d)", plan->op);
    switch (plan->op) {
        case TFH_OP_PERMUTE: e = exec_permute(*plan, al, inputs[0], be, *output, stream); break;
        case TFH_OP_REDUCE: {
            ModedView a{plan->modes_a, {inputs[0].dims, inputs[0].dims + inputs[0].rank}, {inputs[0].strides, inputs[0].strides + inputs[0].rank}};
            e = reduce_moded(dt, view_ptr(inputs[0], dt), a, view_ptr(*output, dt), *output, plan->modes_c, plan->reduce_op, al, be, stream);
            break;
        }
        case TFH_OP_TRACE: {
            ModedView a = diagonal_view(inputs[0], plan->modes_a, plan->pairs);
            // the surviving pair label is summed like any other mode missing from the output
            e = reduce_moded(dt, view_ptr(inputs[0], dt), a, view_ptr(*output, dt), *output, plan->modes_c, TFH_REDUCE_SUM, al, be, stream);
            break;
        }
        case TFH_OP_ANTI_TRACE:
        case TFH_OP_ANTI_DIAG: e = exec_anti(*plan, al, inputs[0], be, *output, stream); break;
        case TFH_OP_ELEMENTWISE_MUL: {
            std::vector<Axis> ax;
            for (int d = 0; d < output->rank; ++d)
                ax.push_back(Axis{output->dims[d], {inputs[0].strides[d], inputs[1].strides[d], output->strides[d]}, (uint32_t)d});
            e = launch_emul(dt, view_ptr(inputs[0], dt), view_ptr(inputs[1], dt), view_ptr(*output, dt), ax, al, be, stream);
            break;
        }
        case TFH_OP_CONTRACT:
        case TFH_OP_BATCHED_GEMM: {
            e = execute_contract(plan->contract_cache, dt, plan->modes_a, inputs[0].dims, inputs[0].strides, view_ptr(inputs[0], dt),
                                 plan->modes_b, inputs[1].dims, inputs[1].strides, view_ptr(inputs[1], dt), plan->modes_c, output->dims,
                                 output->strides, view_ptr(*output, dt), al, be, stream, conj);
            break;
        }
        default: e = set_error(TFH_ERR_INVALID_ARGUMENT, "unknown operation %d", plan->op);
    }
    if (!e) clear_error();
    return e;
}

int32_t tfh_execute_grouped(const tfh_plan* plan, const void* alpha, const tfh_view* inputs, int32_t n_inputs,
                            const void* beta, tfh_view* outputs, tfh_stream stream) {
    if (!plan || !alpha || !beta || !outputs || !inputs) return set_error(TFH_ERR_INVALID_ARGUMENT, "null argument");
    if (!plan->n_groups) return set_error(TFH_ERR_INVALID_ARGUMENT, "not a grouped plan");
    if (n_inputs != 2) return set_error(TFH_ERR_INVALID_ARGUMENT, "grouped contraction takes 2 inputs per group, got %d", n_inputs);
    for (int i = 0; i < plan->n_groups; ++i)
        if ((inputs[2 * i].flags | inputs[2 * i + 1].flags | outputs[i].flags) & TFH_VIEW_CONJ)
            return set_error(TFH_ERR_INVALID_ARGUMENT, "TFH_VIEW_CONJ is not taken by a grouped plan (group %d)", i);
    int32_t e = launch_grouped(*plan, load_scalar(plan->dtype, alpha), inputs, load_scalar(plan->dtype, beta), outputs, stream);
    if (!e) clear_error();
    return e;
}

int32_t tfh_plan_cache_stats(const tfh_plan* plan, int64_t* hits, int64_t* misses, int32_t* entries) {
    if (!plan) return set_error(TFH_ERR_INVALID_ARGUMENT, "null plan");
    contract_cache_stats(plan->contract_cache, hits, misses, entries);
    return TFH_OK;
}

int32_t tfh_plan_describe(const tfh_plan* plan, char* buf, size_t cap) {
    if (!plan || !buf || !cap) return set_error(TFH_ERR_INVALID_ARGUMENT, "null argument");
    static const char* ops[] = {"BatchedGemm", "Reduce", "Trace", "Permute", "AntiTrace", "AntiDiag", "Contract", "ElementwiseMul"};
    static const char* dts[] = {"f32", "f64", "c64", "c128"};
    // kernel selection is kept per set of view strides from the first execute on: the routes the plan holds so far
    const std::string routes = contract_cache_routes(plan->contract_cache);
    snprintf(buf, cap, "%s<%s> inputs=%d groups=%d%s%s", ops[plan->op], dts[plan->dtype], plan->n_inputs, plan->n_groups,
             routes.empty() ? "" : " routes: ", routes.c_str());
    return TFH_OK;
}

static int32_t view_axes(const tfh_view* v, std::vector<Axis>& ax, int slot) {
    if (!v || !v->base) return set_error(TFH_ERR_INVALID_ARGUMENT, "null view");
    if (v->rank < 0 || v->rank > TFH_MAX_RANK) return set_error(TFH_ERR_INVALID_ARGUMENT, "rank %d out of range", v->rank);
    if (ax.empty())
        for (int d = 0; d < v->rank; ++d) ax.push_back(Axis{v->dims[d], {0, 0, 0}, (uint32_t)d});
    for (int d = 0; d < v->rank; ++d) ax[d].s[slot] = v->strides[d];
    return TFH_OK;
}

int32_t tfh_conj(int32_t dtype, const tfh_view* in, tfh_view* out, tfh_stream stream) {
    if (dtype < TFH_F32 || dtype > TFH_C128) return set_error(TFH_ERR_INVALID_ARGUMENT, "unknown dtype %d", dtype);
    if (!in || !out) return set_error(TFH_ERR_INVALID_ARGUMENT, "null view");
    if (in->rank != out->rank) return set_rank_mismatch(in->rank, out->rank);
    for (int d = 0; d < in->rank; ++d)
        if (in->dims[d] != out->dims[d]) return set_shape_mismatch(in->dims, in->rank, out->dims, out->rank);
    std::vector<Axis> ax;
    if (int32_t e = view_axes(in, ax, 0)) return e;
    if (int32_t e = view_axes(out, ax, 1)) return e;
    if (out->flags & TFH_VIEW_CONJ) return set_error(TFH_ERR_INVALID_ARGUMENT, "TFH_VIEW_CONJ on an output view");
    // (the conjugate of a view that is already read conjugated is a plain copy)
    const bool conj = !((in->flags & TFH_VIEW_CONJ) && is_complex(dtype));
    int32_t e = launch_copy(dtype, view_ptr(*in, dtype), view_ptr(*out, dtype), ax, Scalar{1, 0}, Scalar{0, 0}, conj, stream);
    if (!e) clear_error();
    return e;
}

int32_t tfh_fill(int32_t dtype, const void* value, tfh_view* out, tfh_stream stream) {
    if (dtype < TFH_F32 || dtype > TFH_C128) return set_error(TFH_ERR_INVALID_ARGUMENT, "unknown dtype %d", dtype);
    if (!value) return set_error(TFH_ERR_INVALID_ARGUMENT, "null value");
    std::vector<Axis> ax;
    if (int32_t e = view_axes(out, ax, 0)) return e;
    int32_t e = launch_fill(dtype, view_ptr(*out, dtype), ax, load_scalar(dtype, value), stream);
    if (!e) clear_error();
    return e;
}

}  // extern "C"

// tenferro.hpp -- C++17 mirror of tenferro-rs's public interface for the contraction hot path, header-only,
// over the C ABI of tenferro_hip.h.  It keeps the reference's names, argument meaning and error behaviour so that
// code written against the Rust crates reads the same here:
//
//   tenferro-device  (tenferro-device/src/lib.rs:30-162)    LogicalMemorySpace, ComputeDevice, OpKind, Error,
//                                                           preferred_compute_devices
//   tenferro-prims   (tenferro-prims/src/lib.rs:100-340)    ReduceOp, Extension, PrimDescriptor, TensorPrims as the
//                                                           static interface of HipBackend {plan, execute,
//                                                           has_extension_for}
//   tenferro-tensor  (tenferro-tensor/src/lib.rs:122-713)   MemoryOrder, CompletionEvent, Tensor<T>
//   tenferro-einsum  (tenferro-einsum/src/lib.rs:239-621)   Subscripts, ContractionTree, the nine einsum* functions
//
// Scalars: float, double, std::complex<float>, std::complex<double> (the Standard algebra,
// tenferro-algebra/src/lib.rs:58-72).  Rust's Result<T> becomes an exception of type tenferro::Error.
// This library computes on HIP devices only: a MainMemory tensor can be created, copied to a GPU memory space and
// back, but an operation on it raises NoCompatibleComputeDevice.
#pragma once
#include <complex>
#include <cstdint>
#include <cstring>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "tenferro_hip.h"

namespace tenferro {

// ---------------------------------------------------------------------------------------------- tenferro-device
struct LogicalMemorySpace {   // tenferro-device/src/lib.rs:30-38
    enum Kind { MainMemoryKind = TFH_SPACE_MAIN_MEMORY, GpuMemoryKind = TFH_SPACE_GPU_MEMORY } kind = MainMemoryKind;
    size_t space_id = 0;
    static LogicalMemorySpace MainMemory() { return {MainMemoryKind, 0}; }
    static LogicalMemorySpace GpuMemory(size_t space_id) { return {GpuMemoryKind, space_id}; }
    bool operator==(const LogicalMemorySpace& o) const { return kind == o.kind && (kind == MainMemoryKind || space_id == o.space_id); }
    bool operator!=(const LogicalMemorySpace& o) const { return !(*this == o); }
    std::string to_string() const { return kind == MainMemoryKind ? "MainMemory" : "GpuMemory { space_id: " + std::to_string(space_id) + " }"; }
};

struct ComputeDevice {   // tenferro-device/src/lib.rs:46-72
    enum Kind { Cpu = TFH_DEVICE_CPU, Cuda = TFH_DEVICE_CUDA, Hip = TFH_DEVICE_HIP } kind = Hip;
    size_t device_id = 0;
    bool operator==(const ComputeDevice& o) const { return kind == o.kind && device_id == o.device_id; }
    std::string to_string() const {   // Display: "cpu:0", "cuda:1", "hip:0"
        char buf[64];
        tfh_compute_device_format((int32_t)kind, (int64_t)device_id, buf, sizeof buf);
        return buf;
    }
};

enum class OpKind {   // tenferro-device/src/lib.rs:77-90
    Contract = TFH_KIND_CONTRACT, BatchedGemm = TFH_KIND_BATCHED_GEMM, Reduce = TFH_KIND_REDUCE,
    Trace = TFH_KIND_TRACE, Permute = TFH_KIND_PERMUTE, ElementwiseMul = TFH_KIND_ELEMENTWISE_MUL
};

class Error : public std::runtime_error {   // tenferro-device/src/lib.rs:108-159
public:
    enum class Kind {
        ShapeMismatch = TFH_ERR_SHAPE_MISMATCH, RankMismatch = TFH_ERR_RANK_MISMATCH, DeviceError = TFH_ERR_DEVICE,
        NoCompatibleComputeDevice = TFH_ERR_NO_COMPATIBLE_DEVICE, CrossMemorySpaceOperation = TFH_ERR_CROSS_MEMORY_SPACE,
        InvalidArgument = TFH_ERR_INVALID_ARGUMENT, Strided = TFH_ERR_STRIDED
    };
    Kind kind;
    std::vector<size_t> expected, got;   // ShapeMismatch: shapes; RankMismatch: one entry each
    Error(Kind k, const std::string& msg, std::vector<size_t> e = {}, std::vector<size_t> g = {})
        : std::runtime_error(msg), kind(k), expected(std::move(e)), got(std::move(g)) {}
    static Error InvalidArgument(const std::string& m) { return Error(Kind::InvalidArgument, "invalid argument: " + m); }
    static Error NoCompatibleComputeDevice(const LogicalMemorySpace& s, const char* op) {
        return Error(Kind::NoCompatibleComputeDevice, std::string("no compatible compute device for ") + op + " on " + s.to_string());
    }
    static Error CrossMemorySpaceOperation(const LogicalMemorySpace& l, const LogicalMemorySpace& r) {
        return Error(Kind::CrossMemorySpaceOperation, "cross-memory-space operation between " + l.to_string() + " and " + r.to_string());
    }
};

// Turns a tfh_status into the Error variant it stands for (payload from the calling thread's last error).
inline void check(int32_t status) {
    if (status == TFH_OK) return;
    tfh_error_info info;
    tfh_last_error(&info);
    std::vector<size_t> e, g;
    for (int i = 0; i < info.n_expected && i < TFH_MAX_RANK; ++i) e.push_back((size_t)info.expected[i]);
    for (int i = 0; i < info.n_got && i < TFH_MAX_RANK; ++i) g.push_back((size_t)info.got[i]);
    throw Error((Error::Kind)status, info.message, std::move(e), std::move(g));
}

inline std::vector<ComputeDevice> preferred_compute_devices(LogicalMemorySpace space, OpKind op) {   // :92-105
    tfh_compute_device out[8];
    int32_t n = 0;
    check(tfh_preferred_compute_devices((int32_t)space.kind, (int64_t)space.space_id, (int32_t)op, out, 8, &n));
    std::vector<ComputeDevice> r;
    for (int i = 0; i < n; ++i) r.push_back({(ComputeDevice::Kind)out[i].kind, (size_t)out[i].device_id});
    return r;
}

// ---------------------------------------------------------------------------------------------- scalar tags
template <class T> struct ScalarTag;
template <> struct ScalarTag<float> { static constexpr int32_t value = TFH_F32; };
template <> struct ScalarTag<double> { static constexpr int32_t value = TFH_F64; };
template <> struct ScalarTag<std::complex<float>> { static constexpr int32_t value = TFH_C64; };
template <> struct ScalarTag<std::complex<double>> { static constexpr int32_t value = TFH_C128; };

// ---------------------------------------------------------------------------------------------- tenferro-prims
enum class ReduceOp { Sum = TFH_REDUCE_SUM, Max = TFH_REDUCE_MAX, Min = TFH_REDUCE_MIN };                    // :100-107
enum class Extension { Contract = TFH_EXT_CONTRACT, ElementwiseMul = TFH_EXT_ELEMENTWISE_MUL };             // :123-128

struct PrimDescriptor {   // tenferro-prims/src/lib.rs:152-245; one named constructor per variant
    int32_t op = TFH_OP_CONTRACT;
    ReduceOp reduce_op = ReduceOp::Sum;
    std::vector<size_t> batch_dims;
    size_t m = 0, n = 0, k = 0;
    std::vector<uint32_t> modes_a, modes_b, modes_c;
    std::vector<std::pair<uint32_t, uint32_t>> paired;

    static PrimDescriptor BatchedGemm(std::vector<size_t> batch_dims, size_t m, size_t n, size_t k) {
        PrimDescriptor d; d.op = TFH_OP_BATCHED_GEMM; d.batch_dims = std::move(batch_dims); d.m = m; d.n = n; d.k = k; return d;
    }
    static PrimDescriptor Reduce(std::vector<uint32_t> modes_a, std::vector<uint32_t> modes_c, ReduceOp op) {
        PrimDescriptor d; d.op = TFH_OP_REDUCE; d.modes_a = std::move(modes_a); d.modes_c = std::move(modes_c); d.reduce_op = op; return d;
    }
    static PrimDescriptor Trace(std::vector<uint32_t> modes_a, std::vector<uint32_t> modes_c, std::vector<std::pair<uint32_t, uint32_t>> paired) {
        return with_pairs(TFH_OP_TRACE, std::move(modes_a), std::move(modes_c), std::move(paired));
    }
    static PrimDescriptor Permute(std::vector<uint32_t> modes_a, std::vector<uint32_t> modes_b) {
        PrimDescriptor d; d.op = TFH_OP_PERMUTE; d.modes_a = std::move(modes_a); d.modes_c = std::move(modes_b); return d;
    }
    static PrimDescriptor AntiTrace(std::vector<uint32_t> modes_a, std::vector<uint32_t> modes_c, std::vector<std::pair<uint32_t, uint32_t>> paired) {
        return with_pairs(TFH_OP_ANTI_TRACE, std::move(modes_a), std::move(modes_c), std::move(paired));
    }
    static PrimDescriptor AntiDiag(std::vector<uint32_t> modes_a, std::vector<uint32_t> modes_c, std::vector<std::pair<uint32_t, uint32_t>> paired) {
        return with_pairs(TFH_OP_ANTI_DIAG, std::move(modes_a), std::move(modes_c), std::move(paired));
    }
    static PrimDescriptor Contract(std::vector<uint32_t> modes_a, std::vector<uint32_t> modes_b, std::vector<uint32_t> modes_c) {
        PrimDescriptor d; d.op = TFH_OP_CONTRACT; d.modes_a = std::move(modes_a); d.modes_b = std::move(modes_b); d.modes_c = std::move(modes_c); return d;
    }
    static PrimDescriptor ElementwiseMul() { PrimDescriptor d; d.op = TFH_OP_ELEMENTWISE_MUL; return d; }

private:
    static PrimDescriptor with_pairs(int32_t op, std::vector<uint32_t> a, std::vector<uint32_t> c, std::vector<std::pair<uint32_t, uint32_t>> p) {
        PrimDescriptor d; d.op = op; d.modes_a = std::move(a); d.modes_c = std::move(c); d.paired = std::move(p); return d;
    }
};

// The StridedView / StridedViewMut contract (tenferro-tensor/src/lib.rs:169-171, 219-221) over DEVICE memory:
// element (i0, i1, ...) lives at data[offset + sum_d i_d * strides[d]].
template <class T>
struct StridedView {
    T* data = nullptr;
    std::vector<size_t> dims;
    std::vector<ptrdiff_t> strides;
    ptrdiff_t offset = 0;
    bool conj = false;   // read as the complex conjugate (TFH_VIEW_CONJ): Contract / Permute inputs and einsum operands only
    StridedView conjugated() const { StridedView v = *this; v.conj = !conj; return v; }
    tfh_view raw() const {
        if (dims.size() > TFH_MAX_RANK) throw Error::InvalidArgument("rank above 16");
        tfh_view v;
        std::memset(&v, 0, sizeof v);
        v.base = (void*)data;
        v.rank = (int32_t)dims.size();
        v.offset = offset;
        v.flags = conj ? TFH_VIEW_CONJ : 0;
        for (size_t i = 0; i < dims.size(); ++i) { v.dims[i] = (int64_t)dims[i]; v.strides[i] = (int64_t)strides[i]; }
        return v;
    }
};
template <class T> using StridedViewMut = StridedView<T>;

template <class T>
class HipPlan {   // TensorPrims::Plan<T> of the Hip backend
public:
    explicit HipPlan(tfh_plan* p) : p_(p, tfh_plan_destroy) {}
    const tfh_plan* get() const { return p_.get(); }
    std::string describe() const { char buf[256]; tfh_plan_describe(p_.get(), buf, sizeof buf); return buf; }
private:
    std::shared_ptr<tfh_plan> p_;
};

namespace detail {
struct DescHolder {   // keeps the arrays a tfh_desc points into alive
    tfh_desc d;
    std::vector<int64_t> batch;
    std::vector<uint32_t> pairs;
    explicit DescHolder(const PrimDescriptor& s) {
        std::memset(&d, 0, sizeof d);
        d.op = s.op;
        d.reduce_op = (int32_t)s.reduce_op;
        for (size_t b : s.batch_dims) batch.push_back((int64_t)b);
        d.batch_dims = batch.data(); d.n_batch_dims = (int32_t)batch.size();
        d.m = (int64_t)s.m; d.n = (int64_t)s.n; d.k = (int64_t)s.k;
        d.modes_a = s.modes_a.data(); d.n_modes_a = (int32_t)s.modes_a.size();
        d.modes_b = s.modes_b.data(); d.n_modes_b = (int32_t)s.modes_b.size();
        d.modes_c = s.modes_c.data(); d.n_modes_c = (int32_t)s.modes_c.size();
        for (auto& p : s.paired) { pairs.push_back(p.first); pairs.push_back(p.second); }
        d.paired = pairs.data(); d.n_pairs = (int32_t)s.paired.size();
    }
};
struct Shapes {
    std::vector<std::vector<int64_t>> store;
    std::vector<const int64_t*> ptrs;
    std::vector<int32_t> ranks;
    explicit Shapes(const std::vector<std::vector<size_t>>& shapes) {
        for (auto& s : shapes) store.emplace_back(s.begin(), s.end());
        for (auto& s : store) { ptrs.push_back(s.data()); ranks.push_back((int32_t)s.size()); }
    }
};
}  // namespace detail

// impl TensorPrims<Standard> for HipBackend (tenferro-prims/src/lib.rs:278-340)
struct HipBackend {
    template <class T>
    static HipPlan<T> plan(const PrimDescriptor& desc, const std::vector<std::vector<size_t>>& shapes) {   // :282-298
        detail::DescHolder h(desc);
        detail::Shapes s(shapes);
        tfh_plan* p = nullptr;
        check(tfh_plan_create(ScalarTag<T>::value, &h.d, s.ptrs.data(), s.ranks.data(), (int32_t)shapes.size(), &p));
        return HipPlan<T>(p);
    }
    template <class T>
    static void execute(const HipPlan<T>& plan, T alpha, const std::vector<const StridedView<T>*>& inputs, T beta,
                        StridedViewMut<T>& output, tfh_stream stream = nullptr) {   // :300-320
        std::vector<tfh_view> in;
        for (auto* v : inputs) in.push_back(v->raw());
        tfh_view out = output.raw();
        check(tfh_execute(plan.get(), &alpha, in.data(), (int32_t)in.size(), &beta, &out, stream));
    }
    template <class T>
    static bool has_extension_for(Extension ext) { return tfh_has_extension(ScalarTag<T>::value, (int32_t)ext) != 0; }   // :322-339

    // Grouped (variable-size) contraction: no counterpart in the reference protocol; shapes and views are group-major.
    template <class T>
    static HipPlan<T> plan_grouped(const PrimDescriptor& desc, const std::vector<std::vector<std::vector<size_t>>>& group_shapes) {
        detail::DescHolder h(desc);
        std::vector<std::vector<size_t>> flat;
        for (auto& g : group_shapes) for (auto& s : g) flat.push_back(s);
        detail::Shapes s(flat);
        tfh_plan* p = nullptr;
        const int32_t per = group_shapes.empty() ? 0 : (int32_t)group_shapes[0].size();
        check(tfh_plan_create_grouped(ScalarTag<T>::value, &h.d, (int32_t)group_shapes.size(), s.ptrs.data(), s.ranks.data(), per, &p));
        return HipPlan<T>(p);
    }
    template <class T>
    static void execute_grouped(const HipPlan<T>& plan, T alpha, const std::vector<StridedView<T>>& inputs, int n_inputs_per_group,
                                T beta, std::vector<StridedViewMut<T>>& outputs, tfh_stream stream = nullptr) {
        std::vector<tfh_view> in, out;
        for (auto& v : inputs) in.push_back(v.raw());
        for (auto& v : outputs) out.push_back(v.raw());
        check(tfh_execute_grouped(plan.get(), &alpha, in.data(), n_inputs_per_group, &beta, out.data(), stream));
    }
};

// ---------------------------------------------------------------------------------------------- tenferro-tensor
enum class MemoryOrder { ColumnMajor, RowMajor };   // tenferro-tensor/src/lib.rs:122-127

class CompletionEvent {   // :301-309
public:
    CompletionEvent() { tfh_event e = nullptr; check(tfh_event_create(&e)); e_ = std::shared_ptr<void>(e, [](void* p) { tfh_event_destroy(p); }); }
    void record(tfh_stream s) const { check(tfh_event_record(e_.get(), s)); }
    void wait() const { check(tfh_event_synchronize(e_.get())); }
    bool is_ready() const { int32_t r = 0; check(tfh_event_query(e_.get(), &r)); return r != 0; }
    tfh_event raw() const { return e_.get(); }
private:
    std::shared_ptr<void> e_;
};

template <class T> class TensorView;

template <class T>
class Tensor {   // tenferro-tensor/src/lib.rs:167-181
    friend class TensorView<T>;
public:
    // ---- constructors (:336-369)
    static Tensor zeros(const std::vector<size_t>& dims, LogicalMemorySpace space, MemoryOrder order) { return filled(dims, space, order, T(0)); }
    static Tensor ones(const std::vector<size_t>& dims, LogicalMemorySpace space, MemoryOrder order) { return filled(dims, space, order, T(1)); }
    // `data` is laid out in `order`; the tensor lives in main memory (move it with to_memory_space_async)
    static Tensor from_slice(const std::vector<T>& data, const std::vector<size_t>& dims, MemoryOrder order) {
        if (data.size() != count(dims)) throw Error(Error::Kind::ShapeMismatch, "shape mismatch: expected " + std::to_string(count(dims)) + " elements, got " + std::to_string(data.size()), {count(dims)}, {data.size()});
        Tensor t = uninit(dims, LogicalMemorySpace::MainMemory(), order);
        if (!data.empty()) std::memcpy(t.buf_->host.data(), data.data(), data.size() * sizeof(T));
        return t;
    }

    // ---- metadata (:378-411)
    const std::vector<size_t>& dims() const { return dims_; }
    const std::vector<ptrdiff_t>& strides() const { return strides_; }
    size_t ndim() const { return dims_.size(); }
    size_t len() const { return count(dims_); }
    bool is_empty() const { return len() == 0; }
    LogicalMemorySpace logical_memory_space() const { return space_; }
    std::optional<ComputeDevice> preferred_compute_device() const { return preferred_; }
    void set_preferred_compute_device(std::optional<ComputeDevice> d) { preferred_ = d; }
    std::vector<ComputeDevice> effective_compute_devices(OpKind op) const {   // :420-436
        if (preferred_) return {*preferred_};
        return preferred_compute_devices(space_, op);
    }
    ptrdiff_t offset() const { return offset_; }
    // true when no other tensor (a permute/broadcast/diagonal view, a copy) shares this tensor's buffer
    bool sole_owner() const { return buf_ && buf_.use_count() == 1; }

    // ---- views (:445-460): device views; waits for a pending transfer first
    StridedView<T> view() const {
        wait();
        if (space_.kind != LogicalMemorySpace::GpuMemoryKind) throw Error::NoCompatibleComputeDevice(space_, "view");
        return StridedView<T>{(T*)buf_->dev, dims_, strides_, offset_};
    }
    StridedViewMut<T> view_mut() { return view(); }
    TensorView<T> tensor_view() const;   // :455-470: waits, then a borrowed view without a pending event

    // ---- zero-copy metadata operations (:502-548)
    Tensor permute(const std::vector<size_t>& perm) const {
        if (perm.size() != ndim()) throw Error(Error::Kind::RankMismatch, "rank mismatch: expected " + std::to_string(ndim()) + ", got " + std::to_string(perm.size()), {ndim()}, {perm.size()});
        std::vector<bool> seen(ndim(), false);
        Tensor t = *this;
        for (size_t i = 0; i < perm.size(); ++i) {
            if (perm[i] >= ndim() || seen[perm[i]]) throw Error::InvalidArgument("permute: not a permutation");
            seen[perm[i]] = true;
            t.dims_[i] = dims_[perm[i]];
            t.strides_[i] = strides_[perm[i]];
        }
        return t;
    }
    Tensor broadcast(const std::vector<size_t>& target) const {
        if (target.size() < ndim()) throw Error(Error::Kind::RankMismatch, "rank mismatch: expected at least " + std::to_string(ndim()) + ", got " + std::to_string(target.size()), {ndim()}, {target.size()});
        Tensor t = *this;
        const size_t lead = target.size() - ndim();
        t.dims_ = target;
        t.strides_.assign(target.size(), 0);
        for (size_t i = 0; i < ndim(); ++i) {
            if (dims_[i] == target[lead + i]) t.strides_[lead + i] = strides_[i];
            else if (dims_[i] != 1) throw Error(Error::Kind::ShapeMismatch, "shape mismatch: cannot broadcast", dims_, target);
        }
        return t;
    }
    Tensor diagonal(const std::vector<std::pair<size_t, size_t>>& axes) const {
        Tensor t = *this;
        std::vector<bool> drop(ndim(), false);
        for (auto& p : axes) {
            if (p.first >= ndim() || p.second >= ndim() || p.first == p.second || drop[p.first] || drop[p.second]) throw Error::InvalidArgument("diagonal: bad axis pair");
            if (dims_[p.first] != dims_[p.second]) throw Error(Error::Kind::ShapeMismatch, "shape mismatch: diagonal axes differ", {dims_[p.first]}, {dims_[p.second]});
            t.strides_[p.first] += t.strides_[p.second];
            drop[p.second] = true;
        }
        std::vector<size_t> d; std::vector<ptrdiff_t> s;
        for (size_t i = 0; i < ndim(); ++i) if (!drop[i]) { d.push_back(t.dims_[i]); s.push_back(t.strides_[i]); }
        t.dims_ = d; t.strides_ = s;
        return t;
    }
    Tensor reshape(const std::vector<size_t>& new_dims) const {
        if (count(new_dims) != len()) throw Error(Error::Kind::ShapeMismatch, "shape mismatch: reshape changes the element count", dims_, new_dims);
        MemoryOrder order;
        if (!contiguous_order(order)) throw Error::InvalidArgument("reshape needs a contiguous tensor");
        Tensor t = *this;
        t.dims_ = new_dims;
        t.strides_ = natural_strides(new_dims, order);
        return t;
    }
    bool is_contiguous() const { MemoryOrder o; return contiguous_order(o); }   // :602

    // ---- materialising operations (device kernels; the result carries a CompletionEvent)
    Tensor contiguous(MemoryOrder order) const {   // :552-592
        require_gpu("contiguous");
        Tensor out = uninit(dims_, space_, order);
        std::vector<uint32_t> modes(ndim());
        for (size_t i = 0; i < ndim(); ++i) modes[i] = (uint32_t)i;
        std::vector<std::vector<size_t>> shapes = {dims_, dims_};
        auto plan = HipBackend::plan<T>(PrimDescriptor::Permute(modes, modes), shapes);
        StridedView<T> in = view();
        StridedViewMut<T> ov{(T*)out.buf_->dev, out.dims_, out.strides_, 0};
        HipBackend::execute<T>(plan, T(1), {&in}, T(0), ov, nullptr);
        out.mark(nullptr);
        return out;
    }
    Tensor into_contiguous(MemoryOrder order) && { return contiguous(order); }   // :594
    Tensor conj() const {   // :622-651
        require_gpu("conj");
        Tensor out = uninit(dims_, space_, MemoryOrder::RowMajor);
        tfh_view in = view().raw();
        tfh_view ov = StridedView<T>{(T*)out.buf_->dev, out.dims_, out.strides_, 0}.raw();
        check(tfh_conj(ScalarTag<T>::value, &in, &ov, nullptr));
        out.mark(nullptr);
        return out;
    }
    Tensor into_conj() && {   // :653-658: in place
        require_gpu("into_conj");
        tfh_view v = view().raw();
        check(tfh_conj(ScalarTag<T>::value, &v, &v, nullptr));
        mark(nullptr);
        return std::move(*this);
    }
    // Asynchronous copy to another memory space (:660-671); same space: a shallow copy.  The layout is preserved for a
    // contiguous tensor; a strided GPU tensor is compacted first.
    Tensor to_memory_space_async(LogicalMemorySpace target) const {
        if (target == space_) return *this;
        MemoryOrder order = MemoryOrder::RowMajor;
        Tensor src = *this;
        if (!contiguous_order(order)) {
            if (space_.kind != LogicalMemorySpace::GpuMemoryKind) throw Error::InvalidArgument("to_memory_space_async: a strided main-memory tensor cannot be transferred");
            src = contiguous(MemoryOrder::RowMajor);
        }
        src.wait();
        Tensor out = uninit(src.dims_, target, order);
        out.strides_ = src.strides_;
        const size_t bytes = src.len() * sizeof(T);
        if (bytes) {
            if (target.kind == LogicalMemorySpace::GpuMemoryKind && space_.kind == LogicalMemorySpace::MainMemoryKind)
                check(tfh_memcpy_h2d(out.buf_->dev, src.buf_->host.data() + src.offset_, bytes, nullptr));
            else if (target.kind == LogicalMemorySpace::MainMemoryKind)
                check(tfh_memcpy_d2h(out.buf_->host.data(), (const T*)src.buf_->dev + src.offset_, bytes, nullptr));
            else
                check(tfh_memcpy_d2d(out.buf_->dev, (const T*)src.buf_->dev + src.offset_, bytes, nullptr));
        }
        out.mark(nullptr);
        return out;
    }
    void wait() const { if (event_) event_->wait(); }                        // :701-704
    bool is_ready() const { return !event_ || event_->is_ready(); }          // :711-713

    // Host copy of the elements in row-major order of dims() (test helper, no counterpart in the reference).
    std::vector<T> to_vec() const {
        Tensor h = space_.kind == LogicalMemorySpace::GpuMemoryKind ? contiguous(MemoryOrder::RowMajor).to_memory_space_async(LogicalMemorySpace::MainMemory()) : *this;
        h.wait();
        std::vector<T> out(h.len());
        std::vector<size_t> idx(h.ndim(), 0);
        for (size_t n = 0; n < out.size(); ++n) {
            ptrdiff_t off = h.offset_;
            for (size_t d = 0; d < h.ndim(); ++d) off += (ptrdiff_t)idx[d] * h.strides_[d];
            out[n] = h.buf_->host[(size_t)off];
            for (size_t d = h.ndim(); d-- > 0;) { if (++idx[d] < h.dims_[d]) break; idx[d] = 0; }
        }
        return out;
    }
    // Uninitialised tensor (used by the einsum front end for outputs).
    static Tensor uninit(const std::vector<size_t>& dims, LogicalMemorySpace space, MemoryOrder order) {
        Tensor t;
        t.dims_ = dims;
        t.strides_ = natural_strides(dims, order);
        t.space_ = space;
        t.buf_ = std::make_shared<Buffer>();
        const size_t n = count(dims);
        if (space.kind == LogicalMemorySpace::GpuMemoryKind) {
            check(tfh_set_device((int32_t)space.space_id));
            check(tfh_malloc(n * sizeof(T) > 0 ? n * sizeof(T) : 16, &t.buf_->dev));
        } else {
            t.buf_->host.resize(n);
        }
        return t;
    }
    void mark(tfh_stream s) { event_ = std::make_shared<CompletionEvent>(); event_->record(s); }

private:
    struct Buffer {   // DataBuffer (:133-137): host array or device allocation
        std::vector<T> host;
        void* dev = nullptr;
        ~Buffer() { if (dev) tfh_free(dev); }
    };
    std::shared_ptr<Buffer> buf_;
    std::vector<size_t> dims_;
    std::vector<ptrdiff_t> strides_;
    ptrdiff_t offset_ = 0;
    LogicalMemorySpace space_;
    std::optional<ComputeDevice> preferred_;
    std::shared_ptr<CompletionEvent> event_;

    static size_t count(const std::vector<size_t>& d) { size_t n = 1; for (size_t x : d) n *= x; return n; }
    static std::vector<ptrdiff_t> natural_strides(const std::vector<size_t>& dims, MemoryOrder order) {
        std::vector<ptrdiff_t> s(dims.size());
        ptrdiff_t acc = 1;
        if (order == MemoryOrder::RowMajor) for (size_t i = dims.size(); i-- > 0;) { s[i] = acc; acc *= (ptrdiff_t)dims[i]; }
        else for (size_t i = 0; i < dims.size(); ++i) { s[i] = acc; acc *= (ptrdiff_t)dims[i]; }
        return s;
    }
    bool contiguous_order(MemoryOrder& order) const {
        auto match = [&](MemoryOrder o) {
            auto s = natural_strides(dims_, o);
            for (size_t i = 0; i < dims_.size(); ++i) if (dims_[i] > 1 && s[i] != strides_[i]) return false;
            return true;
        };
        if (match(MemoryOrder::RowMajor)) { order = MemoryOrder::RowMajor; return true; }
        if (match(MemoryOrder::ColumnMajor)) { order = MemoryOrder::ColumnMajor; return true; }
        return false;
    }
    void require_gpu(const char* op) const { if (space_.kind != LogicalMemorySpace::GpuMemoryKind) throw Error::NoCompatibleComputeDevice(space_, op); }
    static Tensor filled(const std::vector<size_t>& dims, LogicalMemorySpace space, MemoryOrder order, T value) {
        Tensor t = uninit(dims, space, order);
        if (space.kind == LogicalMemorySpace::GpuMemoryKind) {
            tfh_view v = StridedView<T>{(T*)t.buf_->dev, t.dims_, t.strides_, 0}.raw();
            check(tfh_fill(ScalarTag<T>::value, &value, &v, nullptr));
            t.mark(nullptr);
        } else {
            std::fill(t.buf_->host.begin(), t.buf_->host.end(), value);
        }
        return t;
    }
};

// Borrowed counterpart of Tensor (tenferro-tensor/src/lib.rs:183-300): shares the source's buffer (a reference count
// stands in for the borrow), carries no pending event, offers the zero-copy view operations and the copying
// to_tensor / contiguous / conj.
template <class T>
class TensorView {
public:
    const std::vector<size_t>& dims() const { return t_.dims(); }
    const std::vector<ptrdiff_t>& strides() const { return t_.strides(); }
    size_t ndim() const { return t_.ndim(); }
    LogicalMemorySpace logical_memory_space() const { return t_.logical_memory_space(); }
    std::optional<ComputeDevice> preferred_compute_device() const { return t_.preferred_compute_device(); }
    TensorView permute(const std::vector<size_t>& perm) const { return TensorView(t_.permute(perm)); }                              // :250
    TensorView broadcast(const std::vector<size_t>& target) const { return TensorView(t_.broadcast(target)); }                      // :262
    TensorView diagonal(const std::vector<std::pair<size_t, size_t>>& axes) const { return TensorView(t_.diagonal(axes)); }         // :272
    Tensor<T> to_tensor(MemoryOrder order) const { return t_.contiguous(order); }    // :281: always a fresh buffer
    Tensor<T> contiguous(MemoryOrder order) const { return t_.contiguous(order); }   // :286
    Tensor<T> conj() const { return t_.conj(); }                                     // :293
private:
    friend class Tensor<T>;
    explicit TensorView(Tensor<T> t) : t_(std::move(t)) { t_.event_.reset(); }
    Tensor<T> t_;
};
template <class T>
TensorView<T> Tensor<T>::tensor_view() const {
    wait();
    return TensorView<T>(*this);
}

// ---------------------------------------------------------------------------------------------- tenferro-einsum
class Subscripts {   // tenferro-einsum/src/lib.rs:239-283
public:
    Subscripts(const std::vector<std::vector<uint32_t>>& inputs, const std::vector<uint32_t>& output) {   // Subscripts::new
        std::vector<uint32_t> flat;
        std::vector<int32_t> ranks;
        for (auto& in : inputs) { flat.insert(flat.end(), in.begin(), in.end()); ranks.push_back((int32_t)in.size()); }
        tfh_subscripts* s = nullptr;
        check(tfh_subscripts_new(flat.data(), ranks.data(), (int32_t)inputs.size(), output.data(), (int32_t)output.size(), &s));
        s_ = std::shared_ptr<tfh_subscripts>(s, tfh_subscripts_destroy);
    }
    static Subscripts parse(const std::string& notation) {
        tfh_subscripts* s = nullptr;
        check(tfh_subscripts_parse(notation.c_str(), &s));
        return Subscripts(std::shared_ptr<tfh_subscripts>(s, tfh_subscripts_destroy));
    }
    std::vector<std::vector<uint32_t>> inputs() const {
        std::vector<std::vector<uint32_t>> r;
        for (int i = 0; i < tfh_subscripts_n_inputs(s_.get()); ++i) r.push_back(labels(i));
        return r;
    }
    std::vector<uint32_t> output() const { return labels(-1); }
    const tfh_subscripts* get() const { return s_.get(); }
private:
    explicit Subscripts(std::shared_ptr<tfh_subscripts> s) : s_(std::move(s)) {}
    std::vector<uint32_t> labels(int i) const {
        uint32_t buf[TFH_MAX_RANK];
        int n = tfh_subscripts_labels(s_.get(), i, buf, TFH_MAX_RANK);
        return std::vector<uint32_t>(buf, buf + (n > 0 ? n : 0));
    }
    std::shared_ptr<tfh_subscripts> s_;
};

class ContractionTree {   // tenferro-einsum/src/lib.rs:297-355
public:
    static ContractionTree optimize(const Subscripts& subscripts, const std::vector<std::vector<size_t>>& shapes) {
        detail::Shapes s(shapes);
        tfh_tree* t = nullptr;
        check(tfh_tree_optimize(subscripts.get(), s.ptrs.data(), s.ranks.data(), (int32_t)shapes.size(), &t));
        return ContractionTree(t);
    }
    // The tree `optimize` returns, shared through the library's cache of optimised networks (no counterpart in the
    // reference: the einsum functions that take no plan use it so that a repeated call does not search again).
    static ContractionTree optimize_cached(const Subscripts& subscripts, const std::vector<std::vector<size_t>>& shapes) {
        detail::Shapes s(shapes);
        tfh_tree* t = nullptr;
        check(tfh_tree_optimize_cached(subscripts.get(), s.ptrs.data(), s.ranks.data(), (int32_t)shapes.size(), &t));
        return ContractionTree(t);
    }
    static ContractionTree from_pairs(const Subscripts& subscripts, const std::vector<std::vector<size_t>>& shapes,
                                      const std::vector<std::pair<size_t, size_t>>& pairs) {
        detail::Shapes s(shapes);
        std::vector<int32_t> flat;
        for (auto& p : pairs) { flat.push_back((int32_t)p.first); flat.push_back((int32_t)p.second); }
        tfh_tree* t = nullptr;
        check(tfh_tree_from_pairs(subscripts.get(), s.ptrs.data(), s.ranks.data(), (int32_t)shapes.size(), flat.data(), (int32_t)pairs.size(), &t));
        return ContractionTree(t);
    }
    size_t n_inputs() const { return (size_t)tfh_tree_n_inputs(t_.get()); }
    std::vector<std::pair<size_t, size_t>> steps() const {
        std::vector<std::pair<size_t, size_t>> r;
        for (int i = 0; i < tfh_tree_n_steps(t_.get()); ++i) { int32_t a, b; tfh_tree_step(t_.get(), i, &a, &b); r.emplace_back((size_t)a, (size_t)b); }
        return r;
    }
    std::vector<size_t> output_dims() const {
        int64_t d[TFH_MAX_RANK];
        int n = tfh_tree_output_dims(t_.get(), d, TFH_MAX_RANK);
        return std::vector<size_t>(d, d + (n > 0 ? n : 0));
    }
    double mac_count() const { return tfh_tree_mac_count(t_.get()); }
    double peak_intermediate() const { return tfh_tree_peak_intermediate(t_.get()); }
    const tfh_tree* get() const { return t_.get(); }
private:
    explicit ContractionTree(tfh_tree* t) : t_(t, tfh_tree_destroy) {}
    std::shared_ptr<tfh_tree> t_;
};

namespace detail {
template <class T>
LogicalMemorySpace common_space(const std::vector<const Tensor<T>*>& operands) {
    if (operands.empty()) throw Error::InvalidArgument("einsum needs at least one operand");
    const LogicalMemorySpace s = operands[0]->logical_memory_space();
    for (auto* t : operands)
        if (t->logical_memory_space() != s) throw Error::CrossMemorySpaceOperation(s, t->logical_memory_space());
    if (s.kind != LogicalMemorySpace::GpuMemoryKind) throw Error::NoCompatibleComputeDevice(s, "Contract");
    return s;
}
template <class T>
std::vector<std::vector<size_t>> shapes_of(const std::vector<const Tensor<T>*>& operands) {
    std::vector<std::vector<size_t>> s;
    for (auto* t : operands) s.push_back(t->dims());
    return s;
}
template <class T>
void run_tree(const ContractionTree& tree, const std::vector<const Tensor<T>*>& operands, T alpha, T beta, Tensor<T>& output, uint64_t donate) {
    const LogicalMemorySpace s = common_space(operands);
    if (output.logical_memory_space() != s) throw Error::CrossMemorySpaceOperation(s, output.logical_memory_space());
    std::vector<tfh_view> views;
    for (auto* t : operands) views.push_back(t->view().raw());   // view() waits for pending transfers
    tfh_view out = output.view_mut().raw();
    check(tfh_einsum_execute(ScalarTag<T>::value, tree.get(), views.data(), (int32_t)views.size(), &alpha, &beta, &out, donate, nullptr));
    output.mark(nullptr);
}
template <class T>
std::vector<const Tensor<T>*> pointers(const std::vector<Tensor<T>>& owned) {
    std::vector<const Tensor<T>*> p;
    for (auto& t : owned) p.push_back(&t);
    return p;
}
}  // namespace detail

// einsum_with_plan_into (:584-621): output = alpha * einsum(operands) + beta * output
template <class T>
void einsum_with_plan_into(const ContractionTree& tree, const std::vector<const Tensor<T>*>& operands, T alpha, T beta, Tensor<T>& output) {
    detail::run_tree(tree, operands, alpha, beta, output, 0);
}
template <class T>
void einsum_with_subscripts_into(const Subscripts& subscripts, const std::vector<const Tensor<T>*>& operands, T alpha, T beta, Tensor<T>& output) {   // :545-582
    detail::common_space(operands);
    einsum_with_plan_into(ContractionTree::optimize_cached(subscripts, detail::shapes_of(operands)), operands, alpha, beta, output);
}
template <class T>
void einsum_into(const std::string& notation, const std::vector<const Tensor<T>*>& operands, T alpha, T beta, Tensor<T>& output) {   // :500-543
    einsum_with_subscripts_into(Subscripts::parse(notation), operands, alpha, beta, output);
}
// allocating variants (:393-434): the result is column-major (the order of the reference's examples) in the operands' memory space
template <class T>
Tensor<T> einsum_with_plan(const ContractionTree& tree, const std::vector<const Tensor<T>*>& operands) {
    const LogicalMemorySpace s = detail::common_space(operands);
    Tensor<T> out = Tensor<T>::uninit(tree.output_dims(), s, MemoryOrder::ColumnMajor);
    detail::run_tree(tree, operands, T(1), T(0), out, 0);
    return out;
}
template <class T>
Tensor<T> einsum_with_subscripts(const Subscripts& subscripts, const std::vector<const Tensor<T>*>& operands) {
    detail::common_space(operands);
    return einsum_with_plan(ContractionTree::optimize_cached(subscripts, detail::shapes_of(operands)), operands);
}
template <class T>
Tensor<T> einsum(const std::string& notation, const std::vector<const Tensor<T>*>& operands) {
    return einsum_with_subscripts(Subscripts::parse(notation), operands);
}
// consuming variants (:436-498): the operands' buffers may be reused by the implementation
template <class T>
Tensor<T> einsum_with_plan_owned(const ContractionTree& tree, std::vector<Tensor<T>> operands) {
    auto ptrs = detail::pointers(operands);
    const LogicalMemorySpace s = detail::common_space(ptrs);
    Tensor<T> out = Tensor<T>::uninit(tree.output_dims(), s, MemoryOrder::ColumnMajor);
    uint64_t donate = 0;   // only buffers nobody else can see may be overwritten
    for (size_t i = 0; i < operands.size() && i < 64; ++i)
        if (operands[i].sole_owner()) donate |= 1ull << i;
    detail::run_tree(tree, ptrs, T(1), T(0), out, donate);
    out.wait();   // the operands are released when this function returns
    return out;
}
template <class T>
Tensor<T> einsum_with_subscripts_owned(const Subscripts& subscripts, std::vector<Tensor<T>> operands) {
    auto ptrs = detail::pointers(operands);
    detail::common_space(ptrs);
    auto tree = ContractionTree::optimize_cached(subscripts, detail::shapes_of(ptrs));
    return einsum_with_plan_owned(tree, std::move(operands));
}
template <class T>
Tensor<T> einsum_owned(const std::string& notation, std::vector<Tensor<T>> operands) {
    return einsum_with_subscripts_owned(Subscripts::parse(notation), std::move(operands));
}

}  // namespace tenferro

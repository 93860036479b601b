// Exercises include/tenferro.hpp (the C++ mirror of the reference's interface) the way the reference's own doc
// examples use the Rust crates: `test_mirror host` needs no GPU (plans, subscripts, trees, error variants),
// `test_mirror gpu` runs the hot path on device 0 and checks it against plain loops on the host.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <string>

#include "tenferro.hpp"

using namespace tenferro;
typedef std::complex<double> c128;

static int g_failed = 0, g_checked = 0;
#define CHECK(cond)                                                                      \
    do {                                                                                 \
        ++g_checked;                                                                     \
        if (!(cond)) { ++g_failed; std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); } \
    } while (0)
template <class F>
static bool raises(Error::Kind kind, F f) {
    try { f(); } catch (const Error& e) { return e.kind == kind; }
    return false;
}

static uint64_t g_state = 0x9e3779b97f4a7c15ull;
static double uniform() {   // splitmix64 -> [-1, 1)
    uint64_t z = (g_state += 0x9e3779b97f4a7c15ull);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    z ^= z >> 31;
    return (double)(z >> 11) / 4503599627370496.0 - 1.0;
}
template <class T> static T draw();
template <> double draw<double>() { return uniform(); }
template <> float draw<float>() { return (float)uniform(); }
template <> c128 draw<c128>() { double a = uniform(), b = uniform(); return c128(a, b); }
template <class T> static std::vector<T> random_vec(size_t n) { std::vector<T> v(n); for (auto& x : v) x = draw<T>(); return v; }
template <class T> static double rel_frobenius(const std::vector<T>& x, const std::vector<T>& ref) {
    double d = 0, n = 0;
    for (size_t i = 0; i < x.size(); ++i) { d += std::norm(std::complex<double>(x[i]) - std::complex<double>(ref[i])); n += std::norm(std::complex<double>(ref[i])); }
    return n > 0 ? std::sqrt(d / n) : std::sqrt(d);
}
static std::vector<uint32_t> lab(const char* s) { std::vector<uint32_t> v; for (; *s; ++s) v.push_back((uint32_t)*s); return v; }

static void host_checks() {
    // plan(): shapes are validated against the descriptor without touching a device (tenferro-prims/src/lib.rs:282-298)
    auto p = HipBackend::plan<double>(PrimDescriptor::Contract(lab("ij"), lab("jk"), lab("ik")), {{3, 4}, {4, 5}, {3, 5}});
    CHECK(!p.describe().empty());
    CHECK(raises(Error::Kind::ShapeMismatch, [] { HipBackend::plan<double>(PrimDescriptor::Contract(lab("ij"), lab("jk"), lab("ik")), {{3, 4}, {5, 5}, {3, 5}}); }));
    CHECK(raises(Error::Kind::RankMismatch, [] { HipBackend::plan<double>(PrimDescriptor::Contract(lab("ij"), lab("jk"), lab("ik")), {{3, 4, 2}, {4, 5}, {3, 5}}); }));
    CHECK(raises(Error::Kind::InvalidArgument, [] { HipBackend::plan<double>(PrimDescriptor::Permute(lab("ij"), lab("jj")), {{3, 4}, {4, 4}}); }));
    HipBackend::plan<float>(PrimDescriptor::BatchedGemm({2}, 3, 5, 4), {{2, 3, 4}, {2, 4, 5}, {2, 3, 5}});
    HipBackend::plan<c128>(PrimDescriptor::Reduce(lab("ijk"), lab("ik"), ReduceOp::Sum), {{2, 3, 4}, {2, 4}});
    HipBackend::plan<double>(PrimDescriptor::Trace(lab("ijk"), lab("j"), {{'i', 'k'}}), {{3, 4, 3}, {4}});   // sum over the (i,k) diagonal
    HipBackend::plan<double>(PrimDescriptor::ElementwiseMul(), {{3, 4}, {3, 4}, {3, 4}});
    CHECK(HipBackend::has_extension_for<double>(Extension::Contract));
    CHECK(HipBackend::has_extension_for<c128>(Extension::ElementwiseMul));

    // Subscripts (tenferro-einsum/src/lib.rs:253-283)
    Subscripts s = Subscripts::parse("ij,jk->ik");
    CHECK(s.inputs().size() == 2 && s.inputs()[0] == lab("ij") && s.output() == lab("ik"));
    Subscripts s2({{0, 1}, {1, 2}}, {0, 2});
    CHECK(s2.inputs()[1] == (std::vector<uint32_t>{1, 2}));
    CHECK(raises(Error::Kind::InvalidArgument, [] { Subscripts::parse("ij,jk"); }));
    CHECK(raises(Error::Kind::InvalidArgument, [] { Subscripts::parse("ij,(jk->ik"); }));

    // ContractionTree (:303-355): the chain (8x2)(2x8)(8x2): contracting the last two first costs 8*2*... fewer multiply-adds
    Subscripts chain = Subscripts::parse("ij,jk,kl->il");
    std::vector<std::vector<size_t>> shapes = {{64, 2}, {2, 64}, {64, 2}};
    ContractionTree t = ContractionTree::optimize(chain, shapes);
    CHECK(t.n_inputs() == 3 && t.steps().size() == 2);
    CHECK(t.steps()[0].first + t.steps()[0].second == 3 && t.steps()[0].first != 0);   // (jk,kl) first: 2*64*2 + 64*2*2 = 512 MACs
    CHECK(t.mac_count() == 2.0 * 64 * 2 + 64.0 * 2 * 2);
    ContractionTree forced = ContractionTree::from_pairs(chain, shapes, {{0, 1}, {3, 2}});
    CHECK(forced.mac_count() == 64.0 * 2 * 64 + 64.0 * 64 * 2);
    CHECK(t.output_dims() == (std::vector<size_t>{64, 2}));
    CHECK(raises(Error::Kind::ShapeMismatch, [&] { ContractionTree::optimize(chain, {{64, 2}, {3, 64}, {64, 2}}); }));

    // device model (tenferro-device/src/lib.rs:46-105)
    CHECK((ComputeDevice{ComputeDevice::Hip, 0}).to_string() == "hip:0");
    CHECK((ComputeDevice{ComputeDevice::Cpu, 3}).to_string() == "cpu:3");
    CHECK(raises(Error::Kind::NoCompatibleComputeDevice, [] { preferred_compute_devices(LogicalMemorySpace::MainMemory(), OpKind::Contract); }));

    // Tensor metadata operations in main memory (:502-548, :602)
    std::vector<double> data(24);
    for (size_t i = 0; i < 24; ++i) data[i] = (double)i;
    auto a = Tensor<double>::from_slice(data, {2, 3, 4}, MemoryOrder::RowMajor);
    CHECK(a.strides() == (std::vector<ptrdiff_t>{12, 4, 1}) && a.is_contiguous() && a.len() == 24 && !a.is_empty());
    auto ap = a.permute({2, 0, 1});
    CHECK(ap.dims() == (std::vector<size_t>{4, 2, 3}) && ap.strides() == (std::vector<ptrdiff_t>{1, 12, 4}) && !ap.is_contiguous());
    CHECK(ap.to_vec()[1 * 6 + 1 * 3 + 2] == data[1 * 12 + 2 * 4 + 1]);
    CHECK(a.reshape({6, 4}).strides() == (std::vector<ptrdiff_t>{4, 1}));
    CHECK(raises(Error::Kind::ShapeMismatch, [&] { a.reshape({5, 5}); }));
    CHECK(raises(Error::Kind::InvalidArgument, [&] { ap.reshape({24}); }));
    // column-major from_slice([1..6], [2,3]) is [[1,3,5],[2,4,6]] (tenferro-tensor/src/lib.rs:34-39)
    CHECK(Tensor<double>::from_slice({1, 2, 3, 4, 5, 6}, {2, 3}, MemoryOrder::ColumnMajor).to_vec() == (std::vector<double>{1, 3, 5, 2, 4, 6}));
    auto col = Tensor<double>::from_slice(data, {2, 3, 4}, MemoryOrder::ColumnMajor);
    CHECK(col.strides() == (std::vector<ptrdiff_t>{1, 2, 6}) && col.is_contiguous());
    auto sq = Tensor<double>::from_slice(std::vector<double>(data.begin(), data.begin() + 9), {3, 3}, MemoryOrder::RowMajor);
    auto dg = sq.diagonal({{0, 1}});
    CHECK(dg.dims() == (std::vector<size_t>{3}) && dg.strides() == (std::vector<ptrdiff_t>{4}) && dg.to_vec() == (std::vector<double>{0, 4, 8}));
    auto row = Tensor<double>::from_slice({1, 2, 3}, {3}, MemoryOrder::RowMajor).broadcast({2, 3});
    CHECK(row.strides() == (std::vector<ptrdiff_t>{0, 1}) && row.to_vec() == (std::vector<double>{1, 2, 3, 1, 2, 3}));
    CHECK(raises(Error::Kind::ShapeMismatch, [] { Tensor<double>::from_slice({1, 2, 3}, {2, 2}, MemoryOrder::RowMajor); }));
    // TensorView (:183-300): borrowed metadata view, zero-copy permute / broadcast / diagonal
    {
        auto v = a.tensor_view();
        CHECK(v.dims() == a.dims() && v.strides() == a.strides() && v.ndim() == 3 && v.logical_memory_space() == a.logical_memory_space());
        auto vp = v.permute({2, 0, 1});
        CHECK(vp.dims() == ap.dims() && vp.strides() == ap.strides());
        CHECK(sq.tensor_view().diagonal({{0, 1}}).strides() == (std::vector<ptrdiff_t>{4}));
        CHECK(Tensor<double>::from_slice({1, 2, 3}, {3}, MemoryOrder::RowMajor).tensor_view().broadcast({2, 3}).strides() == (std::vector<ptrdiff_t>{0, 1}));
        CHECK(raises(Error::Kind::InvalidArgument, [&] { v.permute({0, 0, 1}); }));
        CHECK(raises(Error::Kind::NoCompatibleComputeDevice, [&] { v.to_tensor(MemoryOrder::RowMajor); }));
    }
    // no CPU compute in this library: an operation on main-memory operands names the missing device
    CHECK(raises(Error::Kind::NoCompatibleComputeDevice, [&] { einsum<double>("ij,jk->ik", {&sq, &sq}); }));
    CHECK(raises(Error::Kind::NoCompatibleComputeDevice, [&] { sq.conj(); }));
}

static void gpu_checks() {
    const LogicalMemorySpace gpu = LogicalMemorySpace::GpuMemory(0), host = LogicalMemorySpace::MainMemory();
    CHECK(preferred_compute_devices(gpu, OpKind::Contract) == (std::vector<ComputeDevice>{{ComputeDevice::Hip, 0}}));

    // configuration 0: einsum "ij,jk->ik", f64, i=j=k=512, uniform[-1,1) (tenferro-einsum/src/lib.rs:393-406)
    const size_t n = 512;
    auto ha = random_vec<double>(n * n), hb = random_vec<double>(n * n);
    auto A = Tensor<double>::from_slice(ha, {n, n}, MemoryOrder::RowMajor).to_memory_space_async(gpu);
    auto B = Tensor<double>::from_slice(hb, {n, n}, MemoryOrder::RowMajor).to_memory_space_async(gpu);
    CHECK(A.logical_memory_space() == gpu && A.preferred_compute_device() == std::nullopt);
    CHECK(A.effective_compute_devices(OpKind::Contract)[0].to_string() == "hip:0");
    auto Cg = einsum<double>("ij,jk->ik", {&A, &B});
    std::vector<double> ref(n * n, 0.0);
    for (size_t i = 0; i < n; ++i)
        for (size_t k = 0; k < n; ++k) {
            const double aik = ha[i * n + k];
            for (size_t j = 0; j < n; ++j) ref[i * n + j] += aik * hb[k * n + j];
        }
    Cg.wait();
    CHECK(Cg.is_ready() && Cg.dims() == (std::vector<size_t>{n, n}));
    CHECK(rel_frobenius(Cg.to_vec(), ref) < 1e-12);

    // einsum_into with alpha/beta, a transposed view as an operand, a pre-built plan, and the owned variant
    auto C2 = Tensor<double>::ones({n, n}, gpu, MemoryOrder::RowMajor);
    auto At = A.permute({1, 0});
    einsum_into<double>("ji,jk->ik", {&At, &B}, 0.5, -2.0, C2);
    std::vector<double> ref2(n * n);
    for (size_t i = 0; i < n * n; ++i) ref2[i] = 0.5 * ref[i] - 2.0;
    CHECK(rel_frobenius(C2.to_vec(), ref2) < 1e-12);
    Subscripts subs = Subscripts::parse("ij,jk->ik");
    ContractionTree tree = ContractionTree::optimize(subs, {{n, n}, {n, n}});
    CHECK(rel_frobenius(einsum_with_plan<double>(tree, {&A, &B}).to_vec(), ref) < 1e-12);
    CHECK(rel_frobenius(einsum_with_subscripts<double>(subs, {&A, &B}).to_vec(), ref) < 1e-12);
    CHECK(rel_frobenius(einsum_owned<double>("ij,jk->ik", {A, B}).to_vec(), ref) < 1e-12);
    {   // TensorView on the device: a permuted view materialised in either order, and its conjugate-free copy
        auto v = A.tensor_view().permute({1, 0});
        auto tr = v.to_tensor(MemoryOrder::RowMajor);
        CHECK(tr.is_contiguous() && tr.dims() == (std::vector<size_t>{n, n}) && tr.strides() == (std::vector<ptrdiff_t>{(ptrdiff_t)n, 1}));
        auto got = tr.to_vec();
        bool same = true;
        for (size_t i = 0; i < n && same; ++i)
            for (size_t j = 0; j < n; ++j) same = same && got[i * n + j] == ha[j * n + i];
        CHECK(same);
        CHECK(v.contiguous(MemoryOrder::ColumnMajor).strides() == (std::vector<ptrdiff_t>{1, (ptrdiff_t)n}));
    }
    {   // the plan-less forms share one cached tree per network: a repeated call is a hit and gives the same result
        int64_t h0 = 0, m0 = 0, h1 = 0, m1 = 0;
        tfh_tree_cache_stats(&h0, &m0, nullptr);
        CHECK(rel_frobenius(einsum<double>("ij,jk->ik", {&A, &B}).to_vec(), ref) < 1e-12);
        CHECK(rel_frobenius(einsum<double>("ij,jk->ik", {&A, &B}).to_vec(), ref) < 1e-12);
        tfh_tree_cache_stats(&h1, &m1, nullptr);
        CHECK(h1 - h0 == 2 && m1 == m0);
    }
    // the copies handed over above share A's and B's buffers, so nothing was donated and both are intact
    CHECK(A.to_vec() == ha && B.to_vec() == hb);
    {   // a chain whose operands are moved in: each is the sole owner of its buffer, which may then hold an intermediate
        auto mm = [n](const std::vector<double>& x, const std::vector<double>& y) {
            std::vector<double> z(n * n, 0.0);
            for (size_t i = 0; i < n; ++i)
                for (size_t k = 0; k < n; ++k)
                    for (size_t j = 0; j < n; ++j) z[i * n + j] += x[i * n + k] * y[k * n + j];
            return z;
        };
        std::vector<Tensor<double>> ops;
        for (int r = 0; r < 4; ++r)
            ops.push_back(Tensor<double>::from_slice(r % 2 ? hb : ha, {n, n}, MemoryOrder::RowMajor).to_memory_space_async(gpu));
        CHECK(ops[0].sole_owner() && ops[3].sole_owner());
        auto keep = ops[1].permute({1, 0});          // shares operand 1's buffer: that one must survive
        CHECK(!ops[1].sole_owner());
        auto chain = einsum_owned<double>("ij,jk,kl,lm->im", std::move(ops));
        CHECK(rel_frobenius(chain.to_vec(), mm(mm(mm(ha, hb), ha), hb)) < 1e-12);
        std::vector<double> hbt(n * n);
        for (size_t i = 0; i < n; ++i)
            for (size_t j = 0; j < n; ++j) hbt[j * n + i] = hb[i * n + j];
        CHECK(keep.to_vec() == hbt);
    }

    // three operands with an explicit pairwise order, complex128, one operand conjugated (Tensor::conj, :622-651)
    {
        const size_t p = 24, q = 17, r = 9, s = 13;
        auto hx = random_vec<c128>(p * q), hy = random_vec<c128>(q * r), hz = random_vec<c128>(r * s);
        auto X = Tensor<c128>::from_slice(hx, {p, q}, MemoryOrder::RowMajor).to_memory_space_async(gpu);
        auto Y = Tensor<c128>::from_slice(hy, {q, r}, MemoryOrder::RowMajor).to_memory_space_async(gpu);
        auto Z = Tensor<c128>::from_slice(hz, {r, s}, MemoryOrder::RowMajor).to_memory_space_async(gpu);
        auto Yc = Y.conj();
        auto out = einsum<c128>("ij,(jk,kl)->il", {&X, &Yc, &Z});
        std::vector<c128> expect(p * s, c128(0));
        for (size_t i = 0; i < p; ++i)
            for (size_t l = 0; l < s; ++l) {
                c128 acc = 0;
                for (size_t j = 0; j < q; ++j)
                    for (size_t k = 0; k < r; ++k) acc += hx[i * q + j] * std::conj(hy[j * r + k]) * hz[k * s + l];
                expect[i * s + l] = acc;
            }
        CHECK(rel_frobenius(out.to_vec(), expect) < 1e-12);
        auto Yback = std::move(Yc).into_conj();
        CHECK(Yback.to_vec() == hy);   // conj twice is the identity, bit for bit
        // the same conjugate without a copy: a view flagged conjugate-on-load as an input of Contract
        auto XY = Tensor<c128>::zeros({p, r}, gpu, MemoryOrder::RowMajor);
        auto cplan = HipBackend::plan<c128>(PrimDescriptor::Contract({0, 1}, {1, 2}, {0, 2}), {{p, q}, {q, r}, {p, r}});
        auto xv = X.view();
        auto yv = Yback.view().conjugated();
        auto xyv = XY.view_mut();
        HipBackend::execute<c128>(cplan, c128(1), {&xv, &yv}, c128(0), xyv);
        XY.mark(nullptr);
        std::vector<c128> exy(p * r, c128(0));
        for (size_t i = 0; i < p; ++i)
            for (size_t k = 0; k < r; ++k)
                for (size_t j = 0; j < q; ++j) exy[i * r + k] += hx[i * q + j] * std::conj(hy[j * r + k]);
        CHECK(rel_frobenius(XY.to_vec(), exy) < 1e-12);
    }

    // TensorPrims::plan / execute on views: Permute is bit-exact, Reduce and ElementwiseMul follow alpha/beta
    {
        const size_t d0 = 6, d1 = 33, d2 = 20;
        auto hv = random_vec<float>(d0 * d1 * d2);
        auto V = Tensor<float>::from_slice(hv, {d0, d1, d2}, MemoryOrder::RowMajor).to_memory_space_async(gpu);
        auto P = Tensor<float>::zeros({d2, d0, d1}, gpu, MemoryOrder::RowMajor);
        auto plan = HipBackend::plan<float>(PrimDescriptor::Permute({0, 1, 2}, {2, 0, 1}), {{d0, d1, d2}, {d2, d0, d1}});
        auto vin = V.view();
        auto vout = P.view_mut();
        HipBackend::execute<float>(plan, 1.0f, {&vin}, 0.0f, vout);
        P.mark(nullptr);
        std::vector<float> pref(hv.size());
        for (size_t i = 0; i < d0; ++i) for (size_t j = 0; j < d1; ++j) for (size_t k = 0; k < d2; ++k) pref[(k * d0 + i) * d1 + j] = hv[(i * d1 + j) * d2 + k];
        CHECK(P.to_vec() == pref);

        auto R = Tensor<float>::ones({d0, d2}, gpu, MemoryOrder::RowMajor);
        auto rplan = HipBackend::plan<float>(PrimDescriptor::Reduce({0, 1, 2}, {0, 2}, ReduceOp::Sum), {{d0, d1, d2}, {d0, d2}});
        auto rout = R.view_mut();
        HipBackend::execute<float>(rplan, 2.0f, {&vin}, 3.0f, rout);
        R.mark(nullptr);
        std::vector<float> rref(d0 * d2);
        for (size_t i = 0; i < d0; ++i) for (size_t k = 0; k < d2; ++k) { double acc = 0; for (size_t j = 0; j < d1; ++j) acc += hv[(i * d1 + j) * d2 + k]; rref[i * d2 + k] = (float)(2.0 * acc + 3.0); }
        CHECK(rel_frobenius(R.to_vec(), rref) < 1e-5);

        auto M = Tensor<float>::zeros({d0, d1, d2}, gpu, MemoryOrder::RowMajor);
        auto mplan = HipBackend::plan<float>(PrimDescriptor::ElementwiseMul(), {{d0, d1, d2}, {d0, d1, d2}, {d0, d1, d2}});
        auto mout = M.view_mut();
        HipBackend::execute<float>(mplan, 1.0f, {&vin, &vin}, 0.0f, mout);
        M.mark(nullptr);
        std::vector<float> mref(hv.size());
        for (size_t i = 0; i < hv.size(); ++i) mref[i] = hv[i] * hv[i];
        CHECK(M.to_vec() == mref);

        // execute() checks the views against the plan's shapes (tenferro-prims/src/lib.rs:309-312)
        auto wrong = Tensor<float>::zeros({d2, d0, d1 + 1}, gpu, MemoryOrder::RowMajor);
        CHECK(raises(Error::Kind::ShapeMismatch, [&] { auto w = wrong.view_mut(); HipBackend::execute<float>(plan, 1.0f, {&vin}, 0.0f, w); }));
    }

    // BatchedGemm (:156-168), column-major result tensor, contiguous()
    {
        const size_t b = 3, m = 20, k = 11, nn = 14;
        auto ha2 = random_vec<double>(b * m * k), hb2 = random_vec<double>(b * k * nn);
        auto A2 = Tensor<double>::from_slice(ha2, {b, m, k}, MemoryOrder::RowMajor).to_memory_space_async(gpu);
        auto B2 = Tensor<double>::from_slice(hb2, {b, k, nn}, MemoryOrder::RowMajor).to_memory_space_async(gpu);
        auto Cc = Tensor<double>::zeros({b, m, nn}, gpu, MemoryOrder::ColumnMajor);
        auto plan = HipBackend::plan<double>(PrimDescriptor::BatchedGemm({b}, m, nn, k), {{b, m, k}, {b, k, nn}, {b, m, nn}});
        auto va = A2.view(), vb = B2.view();
        auto vc = Cc.view_mut();
        HipBackend::execute<double>(plan, 1.0, {&va, &vb}, 0.0, vc);
        Cc.mark(nullptr);
        std::vector<double> expect(b * m * nn, 0.0);
        for (size_t x = 0; x < b; ++x) for (size_t i = 0; i < m; ++i) for (size_t j = 0; j < nn; ++j) { double acc = 0; for (size_t l = 0; l < k; ++l) acc += ha2[(x * m + i) * k + l] * hb2[(x * k + l) * nn + j]; expect[(x * m + i) * nn + j] = acc; }
        CHECK(rel_frobenius(Cc.to_vec(), expect) < 1e-12);
        auto Cr = Cc.contiguous(MemoryOrder::RowMajor);
        CHECK(Cr.strides() == (std::vector<ptrdiff_t>{(ptrdiff_t)(m * nn), (ptrdiff_t)nn, 1}) && Cr.to_vec() == Cc.to_vec());
    }

    // operands in different memory spaces (tenferro-device/src/lib.rs:142-150)
    auto Ah = Tensor<double>::from_slice(ha, {n, n}, MemoryOrder::RowMajor);
    CHECK(raises(Error::Kind::CrossMemorySpaceOperation, [&] { einsum<double>("ij,jk->ik", {&A, &Ah}); }));
    CHECK(A.to_memory_space_async(host).to_vec() == ha);
}

int main(int argc, char** argv) {
    const std::string mode = argc > 1 ? argv[1] : "host";
    try {
        host_checks();
        if (mode == "gpu") gpu_checks();
    } catch (const Error& e) {
        std::printf("unexpected tenferro::Error: %s\n", e.what());
        return 2;
    }
    std::printf("%s: %d checks, %d failed\n", mode.c_str(), g_checked, g_failed);
    return g_failed ? 1 : 0;
}

"""CPU-only checks of the host side of the backend through the C ABI: the library loads and exports
every symbol the header declares, descriptor validation and error payloads, the subscript parser and
the contraction-tree optimiser.  No kernel is launched."""
import ctypes
import itertools
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def tf():
    import tenferro_rs_amd as tf
    if not os.path.exists(tf.LIB_PATH):
        import importlib.util
        spec = importlib.util.spec_from_file_location("tfh_build", os.path.join(ROOT, "tenferro-rs_amd", "build.py"))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build()
    tf.lib()
    return tf


def lab(s):
    return [ord(c) for c in s]


def test_library_exports_every_declared_symbol(tf):
    header = open(os.path.join(ROOT, "include", "tenferro_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    names = set(re.findall(r"\b(tfh_[a-z0-9_]+)\s*\(", header))
    assert len(names) > 40
    L = ctypes.CDLL(tf.LIB_PATH)
    missing = [n for n in sorted(names) if not hasattr(L, n)]
    assert not missing, missing


def test_dtype_sizes_extensions_and_device_display(tf):
    L = tf.lib()
    assert [L.tfh_dtype_size(d) for d in (tf.F32, tf.F64, tf.C64, tf.C128)] == [4, 8, 8, 16]
    # has_extension_for (tenferro-prims/src/lib.rs:322-339): both extended ops for the Standard dtype set
    for dt in (np.float32, np.float64, np.complex64, np.complex128):
        assert tf.HipBackend.has_extension_for(dt, tf.Extension.Contract)
        assert tf.HipBackend.has_extension_for(dt, tf.Extension.ElementwiseMul)
    assert not tf.HipBackend.has_extension_for(17, tf.Extension.Contract)
    # Display for ComputeDevice (tenferro-device/src/lib.rs:12-18, 64-72)
    assert str(tf.ComputeDevice.Cpu(0)) == "cpu:0"
    assert str(tf.ComputeDevice.Cuda(1)) == "cuda:1"
    assert str(tf.ComputeDevice.Hip(0)) == "hip:0"
    assert L.tfh_status_name(1) == b"ShapeMismatch" and L.tfh_status_name(6) == b"InvalidArgument"


def test_preferred_compute_devices_main_memory_has_none(tf):
    # this library computes on HIP devices only
    with pytest.raises(tf.NoCompatibleComputeDevice) as e:
        tf.preferred_compute_devices(tf.MainMemory, tf.OpKind.Reduce)
    assert str(e.value) == "no compatible compute device for Reduce on MainMemory"
    # the variant's two fields come back as data, not only as text (tenferro-device/src/lib.rs:134-140)
    assert e.value.space == tf.MainMemory and e.value.op == tf.OpKind.Reduce


# ---------------------------------------------------------------------------------------------- plan validation
def test_plan_accepts_the_reference_examples(tf):
    P, D = tf.HipBackend.plan, tf.PrimDescriptor
    # tenferro-prims/src/lib.rs:266-269, 292-296, 408-411, 142-151
    P(np.float64, D.BatchedGemm([], 3, 5, 4), [[3, 4], [4, 5], [3, 5]])
    P(np.float64, D.Reduce([0, 1], [0], tf.ReduceOp.Sum), [[3, 4], [3]])
    P(np.float64, D.Permute([0, 1], [1, 0]), [[3, 4], [4, 3]])
    P(np.float64, D.Contract([0, 1], [1, 2], [0, 2]), [[3, 4], [4, 5], [3, 5]])
    P(np.complex128, D.ElementwiseMul(), [[2, 3], [2, 3], [2, 3]])
    P(np.float32, D.Trace([0, 1, 2], [2], [(0, 1)]), [[4, 4, 3], [3]])
    P(np.float32, D.AntiTrace([2], [0, 1, 2], [(0, 1)]), [[3], [4, 4, 3]])
    P(np.float32, D.AntiDiag([0, 2], [0, 1, 2], [(0, 1)]), [[4, 3], [4, 4, 3]])
    assert "Contract<f64>" in P(np.float64, D.Contract([0, 1], [1, 2], [0, 2]), [[3, 4], [4, 5], [3, 5]]).describe()


def test_plan_shape_and_rank_mismatch_payloads(tf):
    P, D = tf.HipBackend.plan, tf.PrimDescriptor
    with pytest.raises(tf.ShapeMismatch) as e:
        P(np.float64, D.Contract([0, 1], [1, 2], [0, 2]), [[3, 4], [5, 6], [3, 6]])
    assert e.value.expected == [4, 6] and e.value.got == [5, 6]
    assert str(e.value) == "shape mismatch: expected [4, 6], got [5, 6]"      # tenferro-device/src/lib.rs:111
    with pytest.raises(tf.RankMismatch) as e:
        P(np.float64, D.Contract([0, 1], [1, 2], [0, 2]), [[3, 4], [4, 5, 1], [3, 5]])
    assert (e.value.expected, e.value.got) == (2, 3)
    assert str(e.value) == "rank mismatch: expected 2, got 3"                  # :119
    with pytest.raises(tf.ShapeMismatch):
        P(np.float64, D.BatchedGemm([7], 3, 5, 4), [[7, 3, 4], [7, 4, 5], [7, 3, 6]])
    with pytest.raises(tf.RankMismatch):
        P(np.float64, D.BatchedGemm([7], 3, 5, 4), [[3, 4], [7, 4, 5], [7, 3, 5]])
    with pytest.raises(tf.ShapeMismatch):
        P(np.float64, D.Permute([0, 1], [1, 0]), [[3, 4], [3, 4]])
    with pytest.raises(tf.ShapeMismatch):
        P(np.float64, D.ElementwiseMul(), [[3, 4], [3, 5], [3, 4]])
    with pytest.raises(tf.ShapeMismatch):
        P(np.float64, D.Trace([0, 1], [], [(0, 1)]), [[3, 4], []])


@pytest.mark.parametrize("desc,shapes", [
    (lambda D: D.Contract([0, 0], [0, 2], [0, 2]), [[3, 3], [3, 5], [3, 5]]),        # repeated label in an operand
    (lambda D: D.Contract([0, 1], [1, 2], [0, 9]), [[3, 4], [4, 5], [3, 5]]),        # output label in no input
    (lambda D: D.Contract([0, 1], [1, 2], [0, 2]), [[3, 4], [4, 5]]),                # wrong number of shapes
    (lambda D: D.Permute([0, 1], [0, 2]), [[3, 4], [3, 4]]),                         # not a permutation
    (lambda D: D.Permute([0, 1], [1, 1]), [[3, 4], [4, 4]]),
    (lambda D: D.Reduce([0, 1], [2], 0), [[3, 4], [3]]),                             # modes_c not a subset
    (lambda D: D.Reduce([0, 1], [0], 7), [[3, 4], [3]]),                             # unknown reduce op
    (lambda D: D.Trace([0, 1], [0], [(0, 1)]), [[3, 3], [3]]),                       # paired mode in the output
    (lambda D: D.Trace([0, 1], [], [(0, 5)]), [[3, 3], []]),                         # pair names a missing mode
    (lambda D: D.AntiDiag([2], [0, 1, 2], [(0, 1)]), [[3], [4, 4, 3]]),              # AntiDiag input must carry mode i
    (lambda D: D.AntiTrace([0, 2], [0, 1, 2], [(0, 1)]), [[4, 3], [4, 4, 3]]),       # AntiTrace input must not
    (lambda D: tfpd(D, 42), [[3]]),                                                   # unknown op
])
def test_plan_invalid_argument(tf, desc, shapes):
    with pytest.raises(tf.InvalidArgument) as e:
        tf.HipBackend.plan(np.float64, desc(tf.PrimDescriptor), shapes)
    assert str(e.value).startswith("invalid argument: ")                        # tenferro-device/src/lib.rs:152


def tfpd(D, op):
    return D(op)


def test_plan_complex_max_is_rejected_and_bad_dtype(tf):
    with pytest.raises(tf.InvalidArgument):
        tf.HipBackend.plan(np.complex128, tf.PrimDescriptor.Reduce([0, 1], [0], tf.ReduceOp.Max), [[3, 4], [3]])
    with pytest.raises(tf.InvalidArgument):
        tf.HipBackend.plan(9, tf.PrimDescriptor.Reduce([0, 1], [0], tf.ReduceOp.Sum), [[3, 4], [3]])
    with pytest.raises(tf.InvalidArgument):
        tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Permute(list(range(17)), list(range(17))), [[1] * 17, [1] * 17])


def test_grouped_plan_validation(tf):
    D = tf.PrimDescriptor
    desc = D.Contract(lab("ij"), lab("jk"), lab("ik"))
    p = tf.HipBackend.plan_grouped(np.float64, desc, [[[64, 128], [128, 32], [64, 32]], [[5, 7], [7, 3], [5, 3]]])
    assert p.n_groups == 2
    with pytest.raises(tf.ShapeMismatch):
        tf.HipBackend.plan_grouped(np.float64, desc, [[[64, 128], [128, 32], [64, 32]], [[5, 7], [8, 3], [5, 3]]])
    with pytest.raises(tf.InvalidArgument):
        tf.HipBackend.plan_grouped(np.float64, D.Contract(lab("bij"), lab("bjk"), lab("bik")), [[[2, 3, 4], [2, 4, 5], [2, 3, 5]]])
    with pytest.raises(tf.InvalidArgument):
        tf.HipBackend.plan_grouped(np.float64, D.Permute([0], [0]), [[[2], [2], [2]]])


# ---------------------------------------------------------------------------------------------- Subscripts
def test_subscripts_new_reference_doctest(tf):
    # tenferro-einsum/src/lib.rs:222-229
    s = tf.Subscripts.new([[0, 1], [1, 2]], [0, 2])
    assert len(s.inputs) == 2 and s.output == [0, 2]


@pytest.mark.parametrize("notation,inputs,output,nesting", [
    ("ij,jk->ik", ["ij", "jk"], "ik", "0,1"),                      # :235-236, :268
    ("ii->i", ["ii"], "i", "0"),                                   # :269
    ("ijk->", ["ijk"], "", "0"),                                   # :270
    ("ij,(jk,kl)->il", ["ij", "jk", "kl"], "il", "0,(1,2)"),       # :271
    ("((ab,bc),cd),de->ae", ["ab", "bc", "cd", "de"], "ae", "((0,1),2),3"),
    (" i j , j k -> i k ", ["ij", "jk"], "ik", "0,1"),
    ("aB,Bc->ac", ["aB", "Bc"], "ac", "0,1"),
    (",i->i", ["", "i"], "i", "0,1"),                              # a scalar operand
])
def test_subscripts_parse(tf, notation, inputs, output, nesting):
    s = tf.Subscripts.parse(notation)
    assert s.inputs == [lab(t) for t in inputs]
    assert s.output == lab(output)
    assert s.nesting() == nesting


@pytest.mark.parametrize("bad", ["ij,jk", "ij,jk->ik->i", "ij,(jk,kl->il", "ij,jk)->ik", "i1,jk->ik", "ij,jk->i(k)", "ij->iz",
                                 "ij;jk->ik", "ij,jk-ik", "ij,(jk,kl))->il"])
def test_subscripts_parse_malformed(tf, bad):
    with pytest.raises(tf.InvalidArgument):
        tf.Subscripts.parse(bad)


# ---------------------------------------------------------------------------------------------- ContractionTree
def brute_force_min_macs(terms, out, ext):
    """Minimum multiply-add count over every pairwise order, by exhaustive recursion."""
    def rec(items):
        if len(items) == 1:
            return 0.0
        best = float("inf")
        for i, j in itertools.combinations(range(len(items)), 2):
            rest = [items[k] for k in range(len(items)) if k not in (i, j)]
            needed = set(out).union(*rest) if rest else set(out)
            both = items[i] | items[j]
            cost = float(np.prod([ext[l] for l in both])) if both else 1.0
            best = min(best, cost + rec(rest + [frozenset(l for l in both if l in needed)]))
        return best
    return rec([frozenset(t) for t in terms])


def test_tree_config3_is_the_minimum_flop_tree(tf):
    # "awc,asx,wstv,cty->xvy" at chi=1024, D=16, d=2: 558.3 G real flops (8 per complex multiply-add)
    ext = dict(a=1024, c=1024, x=1024, y=1024, w=16, v=16, s=2, t=2)
    terms, out = ["awc", "asx", "wstv", "cty"], "xvy"
    s = tf.Subscripts.parse(",".join(terms) + "->" + out)
    tree = tf.ContractionTree.optimize(s, [[ext[l] for l in t] for t in terms])
    assert tree.mac_count == brute_force_min_macs(terms, out, ext)
    assert abs(8 * tree.mac_count - 558.3e9) < 0.1e9
    assert tree.peak_intermediate * 16 == 536870912
    assert tree.output_dims == [1024, 16, 1024]
    assert len(tree.steps) == 3 and tree.n_inputs == 4


@pytest.mark.parametrize("seed", range(6))
def test_tree_optimize_matches_exhaustive_search_on_random_networks(tf, seed):
    rng = np.random.default_rng(100 + seed)
    labels = "abcdefgh"
    ext = {l: int(rng.integers(2, 9)) for l in labels}
    n = int(rng.integers(3, 6))
    terms = ["".join(sorted(rng.choice(list(labels), size=int(rng.integers(2, 4)), replace=False))) for _ in range(n)]
    used = sorted(set("".join(terms)))
    counts = {l: sum(l in t for t in terms) for l in used}
    out = "".join(l for l in used if counts[l] == 1 or rng.random() < 0.2)
    s = tf.Subscripts.parse(",".join(terms) + "->" + out)
    tree = tf.ContractionTree.optimize(s, [[ext[l] for l in t] for t in terms])
    # labels private to one operand and absent from the output are summed before any contraction
    pre = [frozenset(l for l in t if counts[l] > 1 or l in out) for t in terms]
    assert tree.mac_count == brute_force_min_macs(pre, out, ext)


def test_tree_from_pairs_numbering_and_errors(tf):
    # tenferro-einsum/src/lib.rs:335-343: B*C -> T(index=3), then A*T -> D
    subs = tf.Subscripts.new([[0, 1], [1, 2], [2, 3]], [0, 3])
    shapes = [[3, 4], [4, 100], [100, 5]]
    tree = tf.ContractionTree.from_pairs(subs, shapes, [(1, 2), (0, 3)])
    assert tree.steps == [(1, 2), (0, 3)]
    assert tree.mac_count == 4 * 100 * 5 + 3 * 4 * 5
    labels, dims = tree.node(3)
    assert sorted(labels) == [1, 3] and sorted(dims) == [4, 5]
    assert tree.output_dims == [3, 5]
    other = tf.ContractionTree.from_pairs(subs, shapes, [(0, 1), (3, 2)])
    assert other.mac_count == 3 * 4 * 100 + 3 * 100 * 5
    assert tf.ContractionTree.optimize(subs, shapes).mac_count == tree.mac_count
    for bad in ([(1, 2)], [(1, 2), (0, 1)], [(1, 1), (0, 3)], [(1, 2), (0, 4)], [(1, 2), (0, 3), (4, 0)]):
        with pytest.raises(tf.InvalidArgument):
            tf.ContractionTree.from_pairs(subs, shapes, bad)
    with pytest.raises(tf.ShapeMismatch):
        tf.ContractionTree.optimize(subs, [[3, 4], [5, 100], [100, 5]])
    with pytest.raises(tf.RankMismatch):
        tf.ContractionTree.optimize(subs, [[3, 4], [4, 100, 1], [100, 5]])
    with pytest.raises(tf.InvalidArgument):
        tf.ContractionTree.optimize(subs, [[3, 4], [4, 100]])


def test_tree_parenthesised_order_is_respected(tf):
    s = tf.Subscripts.parse("ij,(jk,kl)->il")
    shapes = [[3, 4], [4, 5], [5, 100]]            # the unforced optimum contracts A*B first
    forced = tf.ContractionTree.optimize(s, shapes)
    assert forced.steps[0] == (2, 1) or forced.steps[0] == (1, 2)
    free = tf.ContractionTree.optimize(tf.Subscripts.parse("ij,jk,kl->il"), shapes)
    assert free.mac_count == 3 * 4 * 5 + 3 * 5 * 100 < forced.mac_count


def test_tree_greedy_beyond_twelve_operands(tf):
    n = 14
    terms = [chr(97 + i) + chr(98 + i) for i in range(n)]         # a chain of matrices
    s = tf.Subscripts.parse(",".join(terms) + "->" + "a" + chr(97 + n))
    tree = tf.ContractionTree.optimize(s, [[4, 4]] * n)
    assert len(tree.steps) == n - 1 and tree.mac_count == (n - 1) * 64


def test_tree_cache_shares_a_network_and_tells_networks_apart(tf):
    # the plan-less einsum functions take their tree from a cache keyed on labels, grouping and extents: the same
    # network is searched once, every differing ingredient is its own entry, errors are reported as by optimize
    L = tf.lib()
    L.tfh_tree_cache_clear()
    h0, m0, e0 = tf.tree_cache_stats()
    assert e0 == 0
    net, shapes = "awc,asx,wstv,cty->xvy", [[8, 4, 8], [8, 2, 8], [4, 2, 2, 4], [8, 2, 8]]
    t1 = tf.ContractionTree.optimize_cached(tf.Subscripts.parse(net), shapes)
    t2 = tf.ContractionTree.optimize_cached(tf.Subscripts.parse(net), shapes)       # another Subscripts object, same key
    fresh = tf.ContractionTree.optimize(tf.Subscripts.parse(net), shapes)
    assert t1._h == t2._h != fresh._h
    assert t1.steps == fresh.steps and t1.mac_count == fresh.mac_count and t1.output_dims == fresh.output_dims
    h1, m1, e1 = tf.tree_cache_stats()
    assert (h1 - h0, m1 - m0, e1) == (1, 1, 1)
    others = [tf.ContractionTree.optimize_cached(tf.Subscripts.parse(n), sh) for n, sh in [
        (net, [[8, 4, 8], [8, 2, 16], [4, 2, 2, 4], [8, 2, 16]]),              # other extents
        ("awc,asx,wstv,cty->xyv", shapes),                                        # other output order
        ("awc,asx,wstv,cyt->xvy", [[8, 4, 8], [8, 2, 8], [4, 2, 2, 4], [8, 8, 2]]),   # other operand labels
        ("(awc,asx),(wstv,cty)->xvy", shapes),                                    # forced grouping
        ("(awc,cty),(asx,wstv)->xvy", [shapes[0], shapes[3], shapes[1], shapes[2]])]]   # another grouping and operand order
    handles = {t1._h} | {t._h for t in others}
    assert len(handles) == 6 and tf.tree_cache_stats()[2] == 6
    # integer-label subscripts with the same labels hit the entry of the parsed string
    ints = tf.Subscripts.new([[ord(c) for c in term] for term in "awc,asx,wstv,cty".split(",")], [ord(c) for c in "xvy"])
    assert tf.ContractionTree.optimize_cached(ints, shapes)._h == t1._h
    with pytest.raises(tf.ShapeMismatch):
        tf.ContractionTree.optimize_cached(tf.Subscripts.parse("ij,jk->ik"), [[3, 4], [5, 6]])
    with pytest.raises(tf.RankMismatch):
        tf.ContractionTree.optimize_cached(tf.Subscripts.parse("ij,jk->ik"), [[3, 4], [4, 6, 1]])
    with pytest.raises(tf.InvalidArgument):
        tf.ContractionTree.optimize_cached(tf.Subscripts.parse("ij,jk->ik"), [[3, 4]])
    assert tf.tree_cache_stats()[2] == 6          # failures leave no entry


def test_tree_cache_drops_the_least_recently_used_and_holders_keep_their_tree(tf):
    L = tf.lib()
    L.tfh_tree_cache_clear()
    s = tf.Subscripts.parse("ij,jk,kl->il")
    first = tf.ContractionTree.optimize_cached(s, [[2, 3], [3, 4], [4, 1000]])
    steps, macs = first.steps, first.mac_count
    for n in range(1, 700):                        # more networks than the cache keeps (512)
        tf.ContractionTree.optimize_cached(s, [[2, 3], [3, 4], [4, n]])
        if n % 100 == 0:                           # keep one entry in use: it must survive
            tf.ContractionTree.optimize_cached(s, [[2, 3], [3, 4], [4, 1]])
    hits, misses, entries = tf.tree_cache_stats()
    assert entries == 512
    assert first.steps == steps and first.mac_count == macs      # dropped by the cache, alive for its holder
    again = tf.ContractionTree.optimize_cached(s, [[2, 3], [3, 4], [4, 1000]])
    assert again._h != first._h and again.steps == steps         # searched again after the drop
    h2 = tf.tree_cache_stats()[0]
    tf.ContractionTree.optimize_cached(s, [[2, 3], [3, 4], [4, 1]])
    assert tf.tree_cache_stats()[0] == h2 + 1                    # the entry kept in use is still cached
    L.tfh_tree_cache_clear()
    assert tf.tree_cache_stats()[2] == 0 and again.steps == steps


def test_tree_cache_is_safe_from_several_threads(tf):
    import threading
    tf.lib().tfh_tree_cache_clear()
    s = tf.Subscripts.parse("ab,bc,cd,de->ae")
    ref = {n: tf.ContractionTree.optimize(s, [[n, 5], [5, 7], [7, 3], [3, n]]).steps for n in range(1, 40)}
    bad = []
    def work(seed):
        rng = np.random.default_rng(seed)
        for _ in range(400):
            n = int(rng.integers(1, 40))
            t = tf.ContractionTree.optimize_cached(s, [[n, 5], [5, 7], [7, 3], [3, n]])
            if t.steps != ref[n]:
                bad.append(n)
    threads = [threading.Thread(target=work, args=(i,)) for i in range(8)]
    for t in threads: t.start()
    for t in threads: t.join()
    assert not bad and tf.tree_cache_stats()[2] == 39


# ---------------------------------------------------------------------------------------------- Tensor metadata
def test_tensor_metadata_reference_doc_examples(tf):
    T, col = tf.Tensor, tf.MemoryOrder.ColumnMajor
    # tenferro-tensor/src/lib.rs:34-39: column-major from_slice([1..6], [2,3]) is [[1,3,5],[2,4,6]]
    m = T.from_slice(np.arange(1.0, 7.0), [2, 3], col)
    assert np.array_equal(m.to_numpy(), np.array([[1.0, 3, 5], [2, 4, 6]]))
    assert m.logical_memory_space() == tf.MainMemory and m.strides() == [1, 2]
    assert m.permute([1, 0]).dims() == [3, 2]                                   # :45-47
    assert m.reshape([6]).dims() == [6]                                         # :49-51
    b = T.from_slice(np.arange(3.0), [3, 1], col).broadcast([3, 4])             # :57-61
    assert b.dims() == [3, 4] and b.strides()[1] == 0
    d = T.from_slice(np.arange(16.0), [4, 4], col).diagonal([(0, 1)])           # :86-91
    assert d.dims() == [4] and np.array_equal(d.to_numpy(), np.array([0.0, 5, 10, 15]))
    at = m.permute([1, 0])                                                       # :578-592
    assert at.is_contiguous()          # a transposed 2-d tensor is contiguous in the other order
    sl = T(m._buf, [2, 2], [1, 4], 0, tf.MainMemory, m.dtype)
    assert not sl.is_contiguous() and sl.contiguous(col).is_contiguous()
    c = T.from_slice(np.array([1 + 2j, 3 - 4j]), [2], col).conj()               # :612-620
    assert np.array_equal(c.to_numpy(), np.array([1 - 2j, 3 + 4j]))
    with pytest.raises(tf.ShapeMismatch):
        T.from_slice(np.arange(5.0), [2, 3], col)
    with pytest.raises(tf.InvalidArgument):
        m.permute([0, 0])
    assert m.wait() is None and m.is_ready()
    m.set_preferred_compute_device(tf.ComputeDevice.Hip(0))
    assert m.effective_compute_devices(tf.OpKind.Contract) == [tf.ComputeDevice.Hip(0)]


def test_seeded_inputs_are_pure_functions_of_the_index():
    from tenferro_rs_amd import inputs
    # SplitMix64 known answers (seed 0: first outputs of the reference generator)
    x = inputs.splitmix64(np.array([0], dtype=np.uint64))
    assert int(x[0]) == 0xE220A8397B1DCDAF
    a = inputs.uniform(7, 3, (4, 5))
    assert a.min() >= -1 and a.max() < 1
    assert np.array_equal(a.ravel()[:7], inputs.uniform(7, 3, (7,)))
    assert not np.array_equal(a, inputs.uniform(7, 4, (4, 5)))
    z = inputs.normal(5, 0, (200000,))
    assert abs(z.mean()) < 0.01 and abs(z.std() - 1) < 0.01
    c = inputs.complex_normal(5, 1, (100000,), sigma=1 / 32)
    assert abs(c.real.std() * 32 - 1) < 0.02 and abs(c.imag.std() * 32 - 1) < 0.02 and abs(np.corrcoef(c.real, c.imag)[0, 1]) < 0.02
    dims = inputs.draw_block_dims(1004, 128)
    assert len(dims) == 128 and all(v % 64 == 0 and 64 <= v <= 1024 for d in dims for v in d)


def test_tensor_view_and_host_views(tf):
    # TensorView (tenferro-tensor/src/lib.rs:183-300) and view()/view_mut() (:445-454) on main-memory tensors
    T, row, col = tf.Tensor, tf.MemoryOrder.RowMajor, tf.MemoryOrder.ColumnMajor
    data = np.arange(24.0)
    a = T.from_slice(data, [2, 3, 4], row)
    v = a.tensor_view()
    assert v.dims() == [2, 3, 4] and v.strides() == [12, 4, 1] and v.ndim() == 3
    assert v.logical_memory_space() == tf.MainMemory and v.preferred_compute_device() is None
    vp = v.permute([2, 0, 1])
    assert vp.dims() == [4, 2, 3] and vp.strides() == [1, 12, 4]
    t = vp.to_tensor(row)                                   # a copy, contiguous in the requested order
    assert t.strides() == [6, 3, 1] and np.array_equal(t.to_numpy(), data.reshape(2, 3, 4).transpose(2, 0, 1))
    assert vp.contiguous(col).strides() == [1, 4, 8]
    assert np.array_equal(vp.contiguous(col).to_numpy(), data.reshape(2, 3, 4).transpose(2, 0, 1))
    same = v.to_tensor(row)                                 # already contiguous: still a fresh buffer
    assert same._buf is not a._buf and np.array_equal(same.to_numpy(), a.to_numpy())
    sq = T.from_slice(np.arange(9.0), [3, 3], row)
    d = sq.tensor_view().diagonal([(0, 1)])
    assert d.dims() == [3] and d.strides() == [4] and list(d.to_tensor(row).to_numpy()) == [0.0, 4.0, 8.0]
    b = T.from_slice(np.array([1.0, 2.0, 3.0]), [3, 1], row).tensor_view().broadcast([3, 4])
    assert b.strides() == [1, 0] and b.to_tensor(row).to_numpy().tolist() == [[1.0] * 4, [2.0] * 4, [3.0] * 4]
    z = T.from_slice(np.array([1 + 2j, 3 - 4j]), [2], row).tensor_view().conj()
    assert z.to_numpy().tolist() == [1 - 2j, 3 + 4j]       # :617-620
    with pytest.raises(tf.InvalidArgument):
        v.permute([0, 0, 1])
    # view(): the strided element view of a main-memory tensor
    w = a.permute([1, 2, 0]).view()
    assert w.shape == (3, 4, 2) and np.array_equal(w, data.reshape(2, 3, 4).transpose(1, 2, 0)) and not w.flags.writeable
    m = a.view_mut()
    m[1, 2, 3] = -1.0
    assert a.to_numpy()[1, 2, 3] == -1.0

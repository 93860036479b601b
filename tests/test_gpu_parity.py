"""GPU parity: the HIP backend, called through the C ABI, against the CPU oracle on the same seeded
inputs.  Bit-exact for data movement; relative Frobenius error <= 1e-12 for f64/complex128 and
<= 1e-5 for f32/complex64 (the tolerances the backend is specified to)."""
import itertools
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TOL = {np.float32: 1e-5, np.float64: 1e-12, np.complex64: 1e-5, np.complex128: 1e-12}
ALL = [np.float32, np.float64, np.complex64, np.complex128]


@pytest.fixture(scope="module")
def tf():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import tenferro_rs_amd as tf
    tf.lib()
    return tf


# Every randomized test draws from seeded_rng(n): n is the test's own number, TFH_TEST_SEED (default 0: the inputs these
# tests have always run on) is added to it, so another set of inputs can be tried without editing this file.
SEED_OFFSET = int(os.environ.get("TFH_TEST_SEED", "0"))


def seeded_rng(n):
    return np.random.default_rng(n + SEED_OFFSET)


def rand(rng, shape, dtype):
    x = rng.standard_normal(shape)
    if np.issubdtype(dtype, np.complexfloating):
        x = x + 1j * rng.standard_normal(shape)
    return x.astype(dtype)


def relerr(x, ref):
    d = np.linalg.norm((np.asarray(x, np.complex128) - ref).ravel())
    n = np.linalg.norm(np.asarray(ref).ravel())
    return d / n if n > 0 else d


def contraction_within_tolerance(x, ref, dtype, scale, k):
    """The parity rule for a contraction result.  The stated tolerance (TOL) is a relative Frobenius error against the
    norm of the reference, and a well-conditioned output meets it.  An output whose terms cancel cannot: two backends
    that each round every one of k products and partial sums (the CPU restatement accumulates f32 in f32 inside a cache
    block, the matrix cores accumulate f32 in f32) may differ by the textbook bound on a rounded inner product,
    2 * gamma with gamma = (k + 2) * u (u = 2^-24 or 2^-53; 4 real operations per complex one) times `scale`, the
    same contraction over absolute values |alpha| * |A| . |B| + |beta| * |C0|.  A wrong or dropped term is of the
    order scale / k, far above that."""
    d = np.linalg.norm((np.asarray(x, np.complex128) - ref).ravel())
    n = np.linalg.norm(np.asarray(ref).ravel())
    if d <= TOL[dtype] * n:
        return True
    u = 2.0 ** -24 if dtype in (np.float32, np.complex64) else 2.0 ** -53
    ops = 4 if np.issubdtype(dtype, np.complexfloating) else 1
    return d <= 2 * ops * (k + 2) * u * np.linalg.norm(np.asarray(scale).ravel())


def copy_kernel_is_fast(label):
    """Whether a copy_kernel label names the variant without bounds checks: the seventh template argument of
    copy_kernel<V, Op, EPT, VR, VW, READ_OLD, FAST, threads, FULL>."""
    assert label.startswith("(copy_kernel<"), label
    args, depth, cur = [], 0, ""
    for ch in label[len("(copy_kernel<"):-2]:
        if ch == "<":
            depth += 1
        elif ch == ">":
            depth -= 1
        if ch == "," and depth == 0:
            args.append(cur.strip())
            cur = ""
        else:
            cur += ch
    args.append(cur.strip())
    return args[6] == "true"


def dev(tf, arr):
    """Device Tensor with the same dims, element strides and offset as the numpy view `arr`."""
    import torch
    root = arr
    while root.base is not None:
        root = root.base
    flat = np.ascontiguousarray(root).reshape(-1) if root.flags.c_contiguous else None
    if flat is None or (arr.size and not np.shares_memory(flat, arr)):
        arr = np.ascontiguousarray(arr)
        flat = arr.reshape(-1)
    isz = arr.dtype.itemsize
    off = (arr.ctypes.data - flat.ctypes.data) // isz if arr.size else 0
    buf = torch.from_numpy(flat.copy()).cuda()
    return tf.Tensor(buf, list(arr.shape), [s // isz for s in arr.strides], off, tf.GpuMemory(0), tf.dtype_code(arr.dtype))


def lab(s):
    return [ord(c) for c in s]


# ------------------------------------------------------------------------------------------------ permute
@pytest.mark.parametrize("dtype", ALL)
def test_permute_all_rank4_perms_bit_exact(tf, oracle, dtype):
    rng = seeded_rng(21)
    a = rand(rng, (5, 12, 7, 9), dtype)
    da = dev(tf, a)
    for perm in itertools.permutations(range(4)):
        shape = [a.shape[p] for p in perm]
        out = tf.Tensor.empty(shape, tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Permute([0, 1, 2, 3], list(perm)), [a.shape, shape])
        tf.HipBackend.execute(plan, 1.0, [da], 0.0, out)
        ref = np.empty(shape, dtype)
        oracle.permute(a, [0, 1, 2, 3], ref, list(perm))
        assert out.to_numpy().tobytes() == ref.tobytes(), perm


@pytest.mark.parametrize("shape,perm", [((33, 65), (1, 0)), ((1, 7, 1, 5), (3, 2, 1, 0)), ((130, 3, 70), (2, 0, 1)),
                                        ((4, 4, 4, 4, 4, 4, 4), (6, 2, 4, 0, 5, 1, 3)), ((2000,), (0,)), ((3, 1000), (1, 0)),
                                        ((0, 5), (1, 0)), ((), ())])
def test_permute_shapes_bit_exact(tf, oracle, shape, perm):
    rng = seeded_rng(22)
    a = rng.standard_normal(shape)
    oshape = [shape[p] for p in perm]
    out = tf.Tensor.empty(oshape, tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64)
    modes = list(range(len(shape)))
    plan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Permute(modes, list(perm)), [shape, oshape])
    tf.HipBackend.execute(plan, 1.0, [dev(tf, a)], 0.0, out)
    ref = np.empty(oshape)
    if a.size:
        oracle.permute(a, modes, ref, list(perm))
    assert out.to_numpy().tobytes() == ref.tobytes()


def test_permute_special_values_bitwise(tf):
    a = np.array([[0.0, -0.0, np.inf, 1.0], [-np.inf, np.nan, 5e-324, -1.0]])
    out = tf.Tensor.empty([4, 2], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64)
    plan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Permute([0, 1], [1, 0]), [[2, 4], [4, 2]])
    tf.HipBackend.execute(plan, 1.0, [dev(tf, a)], 0.0, out)
    assert out.to_numpy().tobytes() == np.ascontiguousarray(a.T).tobytes()


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.complex128])
def test_permute_strided_negative_alpha_beta_and_column_major(tf, oracle, dtype):
    rng = seeded_rng(23)
    big = rand(rng, (16, 18, 20), dtype)
    a = big[::2, ::-1, 1:19:3]
    b0 = np.asfortranarray(rand(rng, (a.shape[2], a.shape[0], a.shape[1]), dtype))   # column-major output
    alpha, beta = (0.5 - 2j, 1.5 + 1j) if np.iscomplexobj(a) else (0.5, -1.5)
    ref = b0.copy(order="F")
    oracle.permute(a, [0, 1, 2], ref, [2, 0, 1], alpha=alpha, beta=beta)
    db = dev(tf, b0.T).permute([2, 1, 0])
    plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Permute([0, 1, 2], [2, 0, 1]), [a.shape, b0.shape])
    tf.HipBackend.execute(plan, alpha, [dev(tf, a)], beta, db)
    assert relerr(db.to_numpy(), ref) < TOL[dtype]


def test_permute_config2_full_size_bit_exact(tf, oracle):
    # the 16^6 f64 tensor permuted to (5,2,0,4,1,3): bit-exact against the oracle, and the inverse permutation
    # restores the input (involution)
    from tenferro_rs_amd import inputs
    a = inputs.uniform(1002, 0, (16,) * 6)
    perm = [5, 2, 0, 4, 1, 3]
    da = dev(tf, a)
    out = tf.Tensor.empty([16] * 6, tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64)
    plan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Permute(list(range(6)), perm), [[16] * 6, [16] * 6])
    tf.HipBackend.execute(plan, 1.0, [da], 0.0, out)
    ref = np.empty((16,) * 6)
    oracle.permute(a, list(range(6)), ref, perm)
    got = out.to_numpy()
    assert got.tobytes() == ref.tobytes()
    back = tf.Tensor.empty([16] * 6, tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64)
    inv = [int(i) for i in np.argsort(perm)]
    plan2 = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Permute(list(range(6)), inv), [[16] * 6, [16] * 6])
    tf.HipBackend.execute(plan2, 1.0, [out], 0.0, back)
    assert back.to_numpy().tobytes() == a.tobytes()


# ------------------------------------------------------------------------------------------------ reduce
@pytest.mark.parametrize("dtype", ALL)
def test_reduce_sum_keep_sets(tf, oracle, dtype):
    rng = seeded_rng(24)
    a = rand(rng, (6, 17, 5, 33), dtype)
    da = dev(tf, a)
    for keep in [(0,), (1, 3), (3, 0), (2, 1, 0), (), (0, 1, 2, 3), (3,), (2,)]:
        shape = [a.shape[k] for k in keep]
        ref = np.empty(shape, dtype)
        oracle.reduce(a, range(4), ref, list(keep))
        out = tf.Tensor.empty(shape, tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Reduce([0, 1, 2, 3], list(keep), tf.ReduceOp.Sum), [a.shape, shape])
        tf.HipBackend.execute(plan, 1.0, [da], 0.0, out)
        assert relerr(out.to_numpy(), ref) < TOL[dtype], keep


def test_reduce_closed_forms_exact_and_long_reductions(tf):
    # integers: exact in f64 whatever the summation order
    shape = (6, 50, 4, 30)
    a = np.arange(np.prod(shape), dtype=np.float64).reshape(shape)
    out = tf.Tensor.empty([6, 4], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64)
    plan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Reduce([0, 1, 2, 3], [0, 2], tf.ReduceOp.Sum), [shape, [6, 4]])
    tf.HipBackend.execute(plan, 1.0, [dev(tf, a)], 0.0, out)
    assert np.array_equal(out.to_numpy(), a.sum(axis=(1, 3)))
    # full reduction of 2^22 ones -> split over blocks, two passes
    ones = np.ones(1 << 22)
    s = tf.Tensor.empty([], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64)
    plan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Reduce([0], [], tf.ReduceOp.Sum), [[1 << 22], []])
    tf.HipBackend.execute(plan, 1.0, [dev(tf, ones)], 0.0, s)
    assert s.to_numpy() == float(1 << 22)
    # few outputs, long strided reduction
    b = np.arange(3 * 70000, dtype=np.float64).reshape(70000, 3)
    o = tf.Tensor.empty([3], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64)
    plan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Reduce([0, 1], [1], tf.ReduceOp.Sum), [[70000, 3], [3]])
    tf.HipBackend.execute(plan, 1.0, [dev(tf, b)], 0.0, o)
    assert np.array_equal(o.to_numpy(), b.sum(axis=0))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_reduce_max_min_alpha_beta_strided(tf, oracle, dtype):
    rng = seeded_rng(25)
    big = rand(rng, (14, 40, 18), dtype)
    a = big[::2, ::-1, ::3]
    da = dev(tf, a)
    for op, name in [(tf.ReduceOp.Max, oracle.MAX), (tf.ReduceOp.Min, oracle.MIN)]:
        ref = np.empty((a.shape[2], a.shape[0]), dtype)
        oracle.reduce(a, [0, 1, 2], ref, [2, 0], op=name)
        out = tf.Tensor.empty(list(ref.shape), tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Reduce([0, 1, 2], [2, 0], op), [a.shape, ref.shape])
        tf.HipBackend.execute(plan, 1.0, [da], 0.0, out)
        assert np.array_equal(out.to_numpy(), ref)
    c0 = rand(rng, (a.shape[2], a.shape[0]), dtype)
    ref = c0.copy()
    oracle.reduce(a, [0, 1, 2], ref, [2, 0], alpha=2.0, beta=-0.5)
    dc = dev(tf, c0)
    plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Reduce([0, 1, 2], [2, 0], tf.ReduceOp.Sum), [a.shape, c0.shape])
    tf.HipBackend.execute(plan, 2.0, [da], -0.5, dc)
    assert relerr(dc.to_numpy(), ref) < TOL[dtype]


def test_reduce_config2_full_size(tf, oracle):
    # sum over axes 1 and 4 of the permuted 16^6 tensor: <= 1e-12 against the oracle; all-ones gives 256 exactly
    from tenferro_rs_amd import inputs
    p = inputs.uniform(1002, 0, (16,) * 6).transpose(5, 2, 0, 4, 1, 3).copy()
    modes_a, modes_c = [5, 2, 0, 4, 1, 3], [5, 0, 4, 3]
    ref = np.empty((16,) * 4)
    oracle.reduce(p, modes_a, ref, modes_c)
    out = tf.Tensor.empty([16] * 4, tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64)
    plan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Reduce(modes_a, modes_c, tf.ReduceOp.Sum), [[16] * 6, [16] * 4])
    tf.HipBackend.execute(plan, 1.0, [dev(tf, p)], 0.0, out)
    assert relerr(out.to_numpy(), ref) < 1e-12
    tf.HipBackend.execute(plan, 1.0, [dev(tf, np.ones((16,) * 6))], 0.0, out)
    assert np.all(out.to_numpy() == 256.0)


# ------------------------------------------------------------------------------------------------ contract
CASES = [
    ("mk", "kn", "mn", dict(m=37, k=53, n=29)),
    ("km", "nk", "nm", dict(m=20, k=300, n=17)),
    ("mk", "kn", "mn", dict(m=300, k=77, n=260)),                  # 128x128 tiles with ragged edges
    ("km", "kn", "mn", dict(m=200, k=45, n=136)),                  # both operands contiguous along the row index
    ("mk", "nk", "nm", dict(m=130, k=100, n=150)),                 # output contiguous along m: operands swap
    ("bmk", "bkn", "bmn", dict(b=3, m=70, k=31, n=40)),
    ("ajbk", "kcj", "abc", dict(a=6, j=8, b=7, k=12, c=20)),       # config-1 pattern: multi-mode M and K
    ("awc", "asx", "wcsx", dict(a=33, w=3, c=10, s=2, x=9)),       # config-3 step 1
    ("mk", "k", "m", dict(m=150, k=300)),
    ("i", "i", "", dict(i=5000)),                                  # split-K down to a scalar
    ("i", "j", "ij", dict(i=19, j=23)),
    ("bij", "jk", "bik", dict(b=4, i=30, j=14, k=25)),
    ("abij", "abjk", "abik", dict(a=2, b=3, i=14, j=15, k=16)),
    ("xmk", "kn", "mn", dict(x=4, m=16, k=7, n=15)),
    ("mk", "kn", "mn", dict(m=64, k=4096, n=64)),                  # split-K
]


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("case", CASES, ids=[c[0] + "," + c[1] + "->" + c[2] + str(i) for i, c in enumerate(CASES)])
def test_contract_against_oracle(tf, oracle, dtype, case):
    ma, mb, mc, ext = case
    rng = seeded_rng(26)
    a = rand(rng, [ext[l] for l in ma], dtype)
    b = rand(rng, [ext[l] for l in mb], dtype)
    cshape = [ext[l] for l in mc]
    ref = np.empty(cshape, dtype)
    oracle.contract(a, lab(ma), b, lab(mb), ref, lab(mc))
    out = dev(tf, np.full(cshape, np.nan, dtype))      # beta == 0 must not read the NaNs
    plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab(ma), lab(mb), lab(mc)), [a.shape, b.shape, cshape])
    tf.HipBackend.execute(plan, 1.0, [dev(tf, a), dev(tf, b)], 0.0, out)
    assert relerr(out.to_numpy(), ref) < TOL[dtype]


@pytest.mark.parametrize("dtype", ALL)
def test_contract_integer_inputs_exact(tf, dtype):
    # small integers: products and sums are exact, so MFMA accumulation order cannot matter
    rng = seeded_rng(27)

    def ints(shape):
        x = rng.integers(-3, 4, shape).astype(np.float64)
        if np.issubdtype(dtype, np.complexfloating):
            x = x + 1j * rng.integers(-3, 4, shape)
        return x.astype(dtype)

    a, b = ints((150, 90, 3)), ints((90, 3, 140))
    out = tf.Tensor.empty([3, 150, 140], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
    plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract([0, 1, 2], [1, 2, 3], [2, 0, 3]), [a.shape, b.shape, [3, 150, 140]])
    tf.HipBackend.execute(plan, 1.0, [dev(tf, a), dev(tf, b)], 0.0, out)
    assert np.array_equal(out.to_numpy(), np.einsum("mkb,kbn->bmn", a, b).astype(dtype))


@pytest.mark.parametrize("dtype", [np.float64, np.complex128, np.float32])
def test_contract_alpha_beta_strided_views(tf, oracle, dtype):
    rng = seeded_rng(28)
    alpha, beta = (0.7 - 1.1j, -0.3 + 0.2j) if np.issubdtype(dtype, np.complexfloating) else (0.7, -0.3)
    big = rand(rng, (140, 90), dtype)
    av = big[::2, ::-2]                       # 70 x 45, negative stride
    b = rand(rng, (45, 50), dtype)
    c0 = rand(rng, (70, 100), dtype)
    cv = c0[:, ::2]                           # strided output
    ref = c0.copy()
    oracle.contract(av, [0, 1], b, [1, 2], ref[:, ::2], [0, 2], alpha=alpha, beta=beta)
    dc = dev(tf, cv)
    plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract([0, 1], [1, 2], [0, 2]), [av.shape, b.shape, cv.shape])
    tf.HipBackend.execute(plan, alpha, [dev(tf, av), dev(tf, b)], beta, dc)
    assert relerr(dc.to_numpy(), ref[:, ::2]) < TOL[dtype]
    # broadcast (stride-0) operand
    row = rand(rng, (1, 45), dtype)
    bc = np.broadcast_to(row, (70, 45))
    ref2 = np.empty((70, 50), dtype)
    oracle.contract(bc, [0, 1], b, [1, 2], ref2, [0, 2])
    out = tf.Tensor.empty([70, 50], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
    tbc = dev(tf, row).broadcast([70, 45])
    plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract([0, 1], [1, 2], [0, 2]), [[70, 45], b.shape, [70, 50]])
    tf.HipBackend.execute(plan, 1.0, [tbc, dev(tf, b)], 0.0, out)
    assert relerr(out.to_numpy(), ref2) < TOL[dtype]


@pytest.mark.parametrize("dtype", ALL)
def test_batched_gemm(tf, oracle, dtype):
    rng = seeded_rng(29)
    a, b = rand(rng, (2, 3, 50, 70), dtype), rand(rng, (2, 3, 70, 40), dtype)
    ref = np.empty((2, 3, 50, 40), dtype)
    oracle.batched_gemm(a, b, ref, n_batch=2)
    out = tf.Tensor.empty([2, 3, 50, 40], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
    plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.BatchedGemm([2, 3], 50, 40, 70), [a.shape, b.shape, ref.shape])
    tf.HipBackend.execute(plan, 1.0, [dev(tf, a), dev(tf, b)], 0.0, out)
    assert relerr(out.to_numpy(), ref) < TOL[dtype]


def colmajor(x):
    """The values of x laid out column-major (first index contiguous): a numpy view that dev() uploads as it is."""
    return np.ascontiguousarray(x.transpose()).transpose()


# the batched patterns of the reference's einsum documentation (tenferro-einsum/src/lib.rs:74-93) in the layout its
# examples allocate (MemoryOrder::ColumnMajor): the batch index is the contiguous one in all three tensors
BATCH_FIRST = [
    ("bij,bjk->bik", lambda b: dict(b=b, i=3, j=4, k=5)),
    ("abij,abjk->abik", lambda b: dict(a=2, b=b, i=4, j=5, k=6)),
    ("bij,jk->bik", lambda b: dict(b=b, i=3, j=4, k=5)),
    ("bij,bjk->bik", lambda b: dict(b=b, i=33, j=7, k=45)),      # ragged tiles, a partial k stage
    ("bij,bkj->bki", lambda b: dict(b=b, i=40, j=13, k=50)),     # k innermost of the free axes, output transposed
    ("bij,bjk->bik", lambda b: dict(b=b, i=64, j=64, k=64)),
]


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("nb", [10, 1023, 1024, 1100])
@pytest.mark.parametrize("case", range(len(BATCH_FIRST)))
def test_column_major_batched_products(tf, oracle, dtype, nb, case):
    sub, ext_of = BATCH_FIRST[case]
    ext = ext_of(nb)
    if case == 5 and nb > 100:
        ext["b"] = 136 if nb % 2 == 0 else 135
    rng = seeded_rng(201 + case)
    terms, out_l = sub.split("->")[0].split(","), sub.split("->")[1]
    hs = [colmajor(rand(rng, [ext[l] for l in t], dtype)) for t in terms]
    cshape = [ext[l] for l in out_l]
    ref = np.empty(cshape, dtype)
    oracle.contract(hs[0], lab(terms[0]), hs[1], lab(terms[1]), ref, lab(out_l))
    out = dev(tf, colmajor(np.full(cshape, np.nan, dtype)))      # beta == 0 must not read the NaNs
    tf.einsum_into(sub, [dev(tf, h) for h in hs], 1.0, 0.0, out)
    kernel = tf.last_kernel()
    assert relerr(out.to_numpy(), ref) < TOL[dtype]
    # the batch-first kernel takes whole 16-byte chunks of batch entries and at least two 128-byte lines of them
    nbf = int(np.prod([ext[l] for l in out_l if l in terms[0] and l in terms[1]]))
    per_chunk = 16 // np.dtype(dtype).itemsize
    batch_first = nbf % per_chunk == 0 and nbf >= 16 * per_chunk
    assert kernel.startswith("(gemm_bfirst_kernel") == batch_first, (kernel, nbf)
    # alpha and beta (complex for complex dtypes) on top of an existing output
    cx = np.issubdtype(dtype, np.complexfloating)
    alpha, beta = (0.5 - 0.25j, 2.0 + 1.0j) if cx else (0.5, 2.0)
    c0 = colmajor(rand(rng, cshape, dtype))
    out = dev(tf, c0)
    tf.einsum_into(sub, [dev(tf, h) for h in hs], alpha, beta, out)
    ref2 = (alpha * ref.astype(np.complex128 if cx else np.float64) + beta * c0).astype(dtype)
    scale = np.abs(alpha) * np.einsum(sub, np.abs(hs[0]).astype(np.float64), np.abs(hs[1]).astype(np.float64)) + np.abs(beta) * np.abs(c0)
    assert contraction_within_tolerance(out.to_numpy(), ref2, dtype, scale, ext["j"])


@pytest.mark.parametrize("dtype", ALL)
def test_batch_first_kernel_exact_on_integers_with_views_and_conj(tf, dtype):
    """Small integers (exact products and sums): the batch-first kernel against numpy on operands that are views -- an
    outer batch axis that does not fuse with the contiguous one, row and k strides that skip elements, a conjugated
    operand -- and on a batch extent that leaves the last group of lines partly filled."""
    rng = seeded_rng(207)
    cx = np.issubdtype(dtype, np.complexfloating)

    def ints(shape):
        x = rng.integers(-3, 4, shape).astype(np.float64)
        if cx:
            x = x + 1j * rng.integers(-3, 4, shape)
        return x.astype(dtype)

    nb, no = 72, 3
    # buffers [k or n][m or k][outer][batch] with the batch contiguous; views take every second row / k
    abuf, bbuf = ints((2 * 9, 2 * 21, no, nb)), ints((no, 37, 2 * 9, nb))
    a = abuf[::2, ::2].transpose(2, 3, 1, 0)          # [o, b, m=21, k=9]: (o, b) would fuse here ...
    b = bbuf[:, :, ::2].transpose(0, 3, 2, 1)         # [o, b, k=9, n=37]: ... but not here, where o is the outermost axis
    cbuf = ints((37, 21, no, nb))
    c = cbuf.transpose(2, 3, 1, 0)                    # [o, b, m, n]
    out = dev(tf, c)
    ops = [dev(tf, a), dev(tf, b)]
    if cx:
        ops[1] = ops[1].conj_on_load()
    tf.einsum_into("obmk,obkn->obmn", ops, 2.0, -1.0, out)
    assert tf.last_kernel().startswith("(gemm_bfirst_kernel"), tf.last_kernel()
    expect = 2.0 * np.einsum("obmk,obkn->obmn", a, np.conj(b)) - c
    assert np.array_equal(out.to_numpy(), expect.astype(dtype))


@pytest.mark.parametrize("dtype", ALL)
def test_plan_keeps_the_routed_launch_per_stride_set(tf, oracle, dtype):
    """Kernel selection lives in the plan (tenferro-prims/src/lib.rs:8, :284): the first execute with a set of view strides
    routes, later ones replay the routed launch on their own buffers -- bit-identical results, also for a route with
    offset tables and split-K partials, and after tfh_release_workspaces has taken the tables away."""
    rng = seeded_rng(211)
    cases = [("ij", "jk", "ik", dict(i=200, j=96, k=180)),                       # one launch
             ("ij", "jk", "ik", dict(i=128, j=4096, k=128)),                     # split-K: partials + fold
             ("ajbk", "kcj", "abc", dict(a=12, j=16, b=10, k=20, c=150)),        # multi-axis groups: offset tables (and a pack)
             ("awc", "asx", "wcsx", dict(a=40, w=4, c=24, s=2, x=36))]
    for ma, mb, mc, ext in cases:
        shapes = [[ext[l] for l in m] for m in (ma, mb, mc)]
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab(ma), lab(mb), lab(mc)), shapes)
        results = []
        for rep in range(4):
            a, b = rand(rng, shapes[0], dtype), rand(rng, shapes[1], dtype)
            ref = np.empty(shapes[2], dtype)
            oracle.contract(a, lab(ma), b, lab(mb), ref, lab(mc))
            out = dev(tf, np.full(shapes[2], np.nan, dtype))
            tf.HipBackend.execute(plan, 1.0, [dev(tf, a), dev(tf, b)], 0.0, out)
            if rep == 0:
                first_kernel = tf.last_kernel()
            assert tf.last_kernel() == first_kernel
            assert relerr(out.to_numpy(), ref) < TOL[dtype], (ma, rep)
            # the same operands once more: the replayed launch gives the same bits
            out2 = dev(tf, np.full(shapes[2], np.nan, dtype))
            tf.HipBackend.execute(plan, 1.0, [dev(tf, a), dev(tf, b)], 0.0, out2)
            assert out.to_numpy().tobytes() == out2.to_numpy().tobytes()
            results.append(out2)
            if rep == 1:
                import torch
                torch.cuda.synchronize()
                assert tf.lib().tfh_release_workspaces() == 0      # a record that names cached tables goes stale here
        hits, misses, entries = plan.cache_stats()
        assert hits + misses == 8 and entries <= 2
        assert (entries == 0) == ("routes:" not in plan.describe()), plan.describe()
        if entries:
            assert first_kernel in plan.describe(), plan.describe()
        if "kernel" in first_kernel and ma != "ajbk":
            assert hits >= 5, (ma, hits, misses)
        # column-major views of the same extents are a second route in the same plan
        a, b = rand(rng, shapes[0], dtype), rand(rng, shapes[1], dtype)
        ref = np.empty(shapes[2], dtype)
        oracle.contract(a, lab(ma), b, lab(mb), ref, lab(mc))
        for rep in range(2):
            out = dev(tf, colmajor(np.zeros(shapes[2], dtype)))
            tf.HipBackend.execute(plan, 1.0, [dev(tf, colmajor(a)), dev(tf, colmajor(b))], 0.0, out)
            assert relerr(out.to_numpy(), ref) < TOL[dtype]


def test_config0_matmul_512_f64(tf, oracle):
    from tenferro_rs_amd import inputs
    a, b = inputs.uniform(1000, 0, (512, 512)), inputs.uniform(1000, 1, (512, 512))
    ref = np.empty((512, 512))
    oracle.contract(a, lab("ij"), b, lab("jk"), ref, lab("ik"))
    c = tf.einsum("ij,jk->ik", [dev(tf, a), dev(tf, b)])
    assert c.dims() == [512, 512]
    assert relerr(c.to_numpy(), ref) < 1e-12


def test_config1_full_size_f32(tf, oracle):
    # "ajbk,kcj->abc", a=64 j=128 b=64 k=96 c=256, standard normal f32: <= 1e-5 against the oracle
    # (the oracle accumulates f32 products in f64)
    from tenferro_rs_amd import inputs
    A = inputs.normal(1001, 0, (64, 128, 64, 96), np.float32)
    B = inputs.normal(1001, 1, (96, 256, 128), np.float32)
    ref = np.empty((64, 64, 256), np.float32)
    oracle.contract(A, lab("ajbk"), B, lab("kcj"), ref, lab("abc"))
    c = tf.einsum("ajbk,kcj->abc", [dev(tf, A), dev(tf, B)])
    assert relerr(c.to_numpy(), ref) < 1e-5


# ------------------------------------------------------------------------------------------------ grouped
def _grouped_case(tf, oracle, dims, dtype, seed):
    from tenferro_rs_amd import inputs
    As = [inputs.uniform(seed, 3 * g, (i, j), dtype) for g, (i, j, k) in enumerate(dims)]
    Bs = [inputs.uniform(seed, 3 * g + 1, (j, k), dtype) for g, (i, j, k) in enumerate(dims)]
    outs = [tf.Tensor.empty([i, k], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype) for (i, j, k) in dims]
    desc = tf.PrimDescriptor.Contract(lab("ij"), lab("jk"), lab("ik"))
    plan = tf.HipBackend.plan_grouped(dtype, desc, [[[i, j], [j, k], [i, k]] for (i, j, k) in dims])
    tf.HipBackend.execute_grouped(plan, 1.0, [(dev(tf, a), dev(tf, b)) for a, b in zip(As, Bs)], 0.0, outs)
    worst = 0.0
    for a, b, o in zip(As, Bs, outs):
        ref = np.empty((a.shape[0], b.shape[1]), dtype)
        oracle.contract(a, lab("ij"), b, lab("jk"), ref, lab("ik"))
        worst = max(worst, relerr(o.to_numpy(), ref))
    return worst


def test_grouped_small_ragged(tf, oracle):
    dims = [(5, 7, 3), (64, 64, 64), (130, 33, 70), (1, 1, 1), (200, 128, 17)]
    assert _grouped_case(tf, oracle, dims, np.float64, 77) < 1e-12


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_grouped_odd_extents_on_128_tiles(tf, oracle, dtype):
    # one grouped launch over problems whose extents are not multiples of the tile, the stage or the vector length
    # (k tails of 1, 2, 5, 6 and 7 elements; edges of 1 and 3 rows), all large enough for 128x128 tiles
    dims = [(129, 1031, 133), (255, 66, 257), (193, 1058, 97), (300, 5, 310), (131, 130, 129), (257, 1025, 129), (300, 6, 310)]
    assert _grouped_case(tf, oracle, dims, dtype, 78) < TOL[dtype]
    assert "gemm128_kernel" in tf.last_kernel() or "gemm128_grouped_kernel" in tf.last_kernel(), tf.last_kernel()


@pytest.mark.parametrize("dtype", ALL)
def test_grouped_tile_shapes_for_last_strips(tf, oracle, dtype):
    # extents that leave a last strip of at most 64 rows or 64 real columns (odd multiples of 64, a strip of 1, of 63, of
    # exactly 64; for complex a strip of 32 elements is 64 real columns) get tiles of that shape -- the row strip runs as
    # the transposed product -- next to extents whose strip is wider than 64 and stays a padded 128 x 128 tile, extents
    # below one tile on one side, and a corner where both strips meet; alpha and beta applied
    dims = [(192, 80, 320), (320, 96, 192), (448, 40, 448), (129, 64, 191), (256, 33, 256), (191, 50, 129), (160, 72, 97),
            (224, 24, 100), (100, 56, 224), (128, 16, 64), (64, 16, 128), (576, 8, 1088)]
    from tenferro_rs_amd import inputs
    As = [inputs.uniform(81, 3 * g, (i, j), dtype) for g, (i, j, k) in enumerate(dims)]
    Bs = [inputs.uniform(81, 3 * g + 1, (j, k), dtype) for g, (i, j, k) in enumerate(dims)]
    C0 = [inputs.uniform(81, 3 * g + 2, (i, k), dtype) for g, (i, j, k) in enumerate(dims)]
    outs = [dev(tf, c) for c in C0]
    desc = tf.PrimDescriptor.Contract(lab("ij"), lab("jk"), lab("ik"))
    plan = tf.HipBackend.plan_grouped(dtype, desc, [[[i, j], [j, k], [i, k]] for (i, j, k) in dims])
    alpha, beta = (0.7 - 1.1j, -0.3 + 0.2j) if np.issubdtype(dtype, np.complexfloating) else (0.7, -0.3)
    tf.HipBackend.execute_grouped(plan, alpha, [(dev(tf, a), dev(tf, b)) for a, b in zip(As, Bs)], beta, outs)
    assert "gemm128_grouped_kernel" in tf.last_kernel(), tf.last_kernel()
    for a, b, c0, o, d in zip(As, Bs, C0, outs, dims):
        ref = c0.copy()
        oracle.contract(a, lab("ij"), b, lab("jk"), ref, lab("ik"), alpha=alpha, beta=beta)
        assert relerr(o.to_numpy(), ref) < TOL[dtype], d


def test_grouped_column_major_operands_and_views(tf, oracle):
    # column-major blocks (A contiguous along its rows, B along k) and blocks cut out of larger buffers: the other
    # loader layouts of the grouped kernel, with last strips in both directions
    rng = seeded_rng(82)
    dims = [(192, 70, 320), (320, 130, 192), (256, 64, 200), (200, 90, 256)]
    As = [np.asfortranarray(rng.standard_normal((i, j))) for (i, j, k) in dims]
    Bs = [np.asfortranarray(rng.standard_normal((j, k))) for (i, j, k) in dims]
    outs = [tf.Tensor.empty([i, k], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64) for (i, j, k) in dims]
    desc = tf.PrimDescriptor.Contract(lab("ij"), lab("jk"), lab("ik"))
    plan = tf.HipBackend.plan_grouped(np.float64, desc, [[[i, j], [j, k], [i, k]] for (i, j, k) in dims])
    ins = [(dev(tf, a.T).permute([1, 0]), dev(tf, b.T).permute([1, 0])) for a, b in zip(As, Bs)]
    tf.HipBackend.execute_grouped(plan, 1.0, ins, 0.0, outs)
    for a, b, o in zip(As, Bs, outs):
        assert relerr(o.to_numpy(), a @ b) < 1e-12
    big = [rng.standard_normal((i + 3, j + 8)) for (i, j, k) in dims]
    bigb = [rng.standard_normal((j + 2, k + 6)) for (i, j, k) in dims]
    As = [x[1:1 + i, 4:4 + j] for x, (i, j, k) in zip(big, dims)]
    Bs = [x[2:2 + j, 2:2 + k] for x, (i, j, k) in zip(bigb, dims)]
    tf.HipBackend.execute_grouped(plan, 1.0, [(dev(tf, a), dev(tf, b)) for a, b in zip(As, Bs)], 0.0, outs)
    for a, b, o in zip(As, Bs, outs):
        assert relerr(o.to_numpy(), a @ b) < 1e-12


def test_grouped_plan_on_two_streams_with_different_operands(tf, oracle):
    # one plan, two streams, two operand sets in flight at the same time: the problem records of a call live in the
    # workspace of its own stream, so neither call sees the other's pointers
    import ctypes
    import torch
    dims = [(192, 256, 320), (320, 192, 192), (256, 128, 256), (128, 320, 448)] * 6
    rng = seeded_rng(83)
    sets = []
    for s in range(2):
        As = [rng.standard_normal((i, j)) for (i, j, k) in dims]
        Bs = [rng.standard_normal((j, k)) for (i, j, k) in dims]
        outs = [tf.Tensor.empty([i, k], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64) for (i, j, k) in dims]
        sets.append((As, Bs, [(dev(tf, a), dev(tf, b)) for a, b in zip(As, Bs)], outs))
    desc = tf.PrimDescriptor.Contract(lab("ij"), lab("jk"), lab("ik"))
    plan = tf.HipBackend.plan_grouped(np.float64, desc, [[[i, j], [j, k], [i, k]] for (i, j, k) in dims])
    streams = []
    for _ in range(2):
        st = ctypes.c_void_p()
        assert tf.lib().tfh_stream_create(ctypes.byref(st)) == 0
        streams.append(st)
    torch.cuda.synchronize()
    try:
        for rep in range(4):   # alternate the streams so that launches of both are queued together
            for (As, Bs, ins, outs), st in zip(sets, streams):
                tf.HipBackend.execute_grouped(plan, 1.0, ins, 0.0, outs, stream=st.value)
        for st in streams:
            assert tf.lib().tfh_stream_synchronize(st) == 0
        for As, Bs, ins, outs in sets:
            for a, b, o in zip(As, Bs, outs):
                assert relerr(o.to_numpy(), a @ b) < 1e-12
    finally:
        for st in streams:
            tf.lib().tfh_stream_destroy(st)


@pytest.mark.parametrize("ma,mb,mc", [("ij", "jk", "ik"), ("ji", "kj", "ki"), ("ij", "kj", "ki"), ("aij", "jk", "aik"), ("ijl", "jlk", "ik")])
def test_grouped_label_orders_and_fusable_modes(tf, oracle, ma, mb, mc):
    # The roles of a matrix product's axes come from the plan's labels, in any order (transposed operands, transposed
    # result); operands with more than two modes are plain matrices once their modes fuse (a leading free mode, two
    # summed modes), and go through the general classification.
    rng = seeded_rng(85)
    ext_sets = [dict(i=70, j=33, k=130, a=3, l=4), dict(i=5, j=64, k=7, a=2, l=2), dict(i=128, j=128, k=64, a=1, l=8), dict(i=1, j=9, k=257, a=4, l=1)]
    shapes, As, Bs, outs = [], [], [], []
    for ext in ext_sets:
        sa, sb, sc = [ext[c] for c in ma], [ext[c] for c in mb], [ext[c] for c in mc]
        shapes.append([sa, sb, sc])
        As.append(rng.standard_normal(sa)); Bs.append(rng.standard_normal(sb))
        outs.append(tf.Tensor.empty(sc, tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64))
    plan = tf.HipBackend.plan_grouped(np.float64, tf.PrimDescriptor.Contract(lab(ma), lab(mb), lab(mc)), shapes)
    tf.HipBackend.execute_grouped(plan, 1.0, [(dev(tf, a), dev(tf, b)) for a, b in zip(As, Bs)], 0.0, outs)
    for a, b, o in zip(As, Bs, outs):
        assert relerr(o.to_numpy(), np.einsum(f"{ma},{mb}->{mc}", a, b)) < 1e-12, (ma, mb, mc, a.shape)


def test_grouped_records_are_kept_for_repeated_calls(tf, oracle):
    # A grouped call whose operands, outputs and strides equal those of an earlier call of the plan reuses the problem
    # records that call wrote to the device; new operand sets get records of their own, and once the plan holds as many
    # sets as it keeps, further ones are written per call again.  Twelve operand sets, each run three times in an
    # interleaved order, one of them also from a second stream, and a set whose output alone differs: every result is
    # that of its own operands.
    import ctypes
    dims = [(96, 64, 80), (33, 70, 129), (128, 128, 128), (17, 5, 260)] * 3
    rng = seeded_rng(84)
    desc = tf.PrimDescriptor.Contract(lab("ij"), lab("jk"), lab("ik"))
    plan = tf.HipBackend.plan_grouped(np.float64, desc, [[[i, j], [j, k], [i, k]] for (i, j, k) in dims])
    sets = []
    for s_ in range(12):
        As = [rng.standard_normal((i, j)) for (i, j, k) in dims]
        Bs = [rng.standard_normal((j, k)) for (i, j, k) in dims]
        outs = [tf.Tensor.empty([i, k], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64) for (i, j, k) in dims]
        sets.append((As, Bs, [(dev(tf, a), dev(tf, b)) for a, b in zip(As, Bs)], outs))
    for rep in range(3):
        for As, Bs, ins, outs in (sets if rep != 1 else sets[::-1]):
            for o in outs:
                o._buf.zero_()
            tf.HipBackend.execute_grouped(plan, 1.0, ins, 0.0, outs)
            for a, b, o in zip(As, Bs, outs):
                assert relerr(o.to_numpy(), a @ b) < 1e-12, rep
    # the first set again, from another stream (its records were written on the default stream), with alpha and beta
    st = ctypes.c_void_p()
    assert tf.lib().tfh_stream_create(ctypes.byref(st)) == 0
    try:
        As, Bs, ins, outs = sets[0]
        before = [o.to_numpy() for o in outs]
        import torch
        torch.cuda.synchronize()
        tf.HipBackend.execute_grouped(plan, 2.0, ins, -1.0, outs, stream=st.value)
        assert tf.lib().tfh_stream_synchronize(st) == 0
        for a, b, o, c0 in zip(As, Bs, outs, before):
            assert relerr(o.to_numpy(), 2.0 * (a @ b) - c0) < 1e-12
    finally:
        tf.lib().tfh_stream_destroy(st)
    # same inputs, other outputs: different records
    As, Bs, ins, outs = sets[1]
    outs2 = [tf.Tensor.empty([i, k], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64) for (i, j, k) in dims]
    tf.HipBackend.execute_grouped(plan, 1.0, ins, 0.0, outs2)
    for a, b, o in zip(As, Bs, outs2):
        assert relerr(o.to_numpy(), a @ b) < 1e-12


@pytest.mark.parametrize("dtype", ALL)
def test_grouped_tiny_problems_take_the_wave_kernel(tf, oracle, dtype):
    # 300 problems with every extent between 1 and 32 (a block-sparse tensor with small blocks): one grouped launch,
    # one wave per 32x32 tile
    rng = seeded_rng(79)
    dims = [tuple(int(v) for v in rng.integers(1, 33, 3)) for _ in range(300)]
    assert _grouped_case(tf, oracle, dims, dtype, 79) < TOL[dtype]
    assert "gemm_wave_kernel" in tf.last_kernel(), tf.last_kernel()


def test_config4_grouped_full_size(tf, oracle):
    # 128 blocks, i,j,k iid from {64,...,1024}: every block <= 1e-12 against the oracle, one launch
    from tenferro_rs_amd import inputs
    dims = inputs.draw_block_dims(1004, 128)
    assert _grouped_case(tf, oracle, dims, np.float64, 1004) < 1e-12


# ------------------------------------------------------------------------------------------------ elementwise, conj, fill, trace family
@pytest.mark.parametrize("dtype", ALL)
def test_elementwise_mul_conj_fill(tf, oracle, dtype):
    rng = seeded_rng(30)
    a, b = rand(rng, (9, 40, 21), dtype), rand(rng, (21, 40, 9), dtype).transpose(2, 1, 0)
    c0 = rand(rng, (9, 40, 21), dtype)
    ref = c0.copy()
    oracle.elementwise_mul(a, b, ref, alpha=2.0, beta=1.0)
    dc = dev(tf, c0)
    plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.ElementwiseMul(), [a.shape, b.shape, c0.shape])
    tf.HipBackend.execute(plan, 2.0, [dev(tf, a), dev(tf, b)], 1.0, dc)
    assert relerr(dc.to_numpy(), ref) < TOL[dtype]
    da = dev(tf, a)
    assert np.array_equal(da.conj().to_numpy(), np.conj(a))
    assert np.array_equal(da.into_conj().to_numpy(), np.conj(a))
    ones = tf.Tensor.ones([7, 33], tf.GpuMemory(0), tf.MemoryOrder.ColumnMajor, dtype)
    assert np.array_equal(ones.to_numpy(), np.ones((7, 33), dtype))
    assert ones.strides() == [1, 7]


@pytest.mark.parametrize("dtype", ALL)
def test_elementwise_mul_second_operand_in_another_axis_order(tf, oracle, dtype):
    # the second operand's contiguous axis is neither A's nor the output's: it is brought into the output's axis order
    # first (a pool block, released in stream order); strided / reversed / broadcast operands and an output that is
    # a view are covered, and the operands must come out unchanged
    rng = seeded_rng(130)
    shape = (70, 50, 60)
    a = rand(rng, shape, dtype)
    cases = {
        "reversed modes": rand(rng, shape[::-1], dtype).transpose(2, 1, 0),
        "middle axis contiguous": rand(rng, (70, 60, 50), dtype).transpose(0, 2, 1),
        "reversed and stepped": rand(rng, (60, 100, 70), dtype)[::-1, ::2, :].transpose(2, 1, 0),
        "broadcast": np.broadcast_to(rand(rng, (1, 50, 1), dtype), shape),
    }
    for name, b in cases.items():
        for alpha, beta in [(1.0, 0.0), (0.5, -1.5)]:
            big = rand(rng, (70, 50, 120), dtype)
            c0 = big[:, :, ::2]                                   # the output is a stepped view
            ref = c0.copy()
            oracle.elementwise_mul(a, np.ascontiguousarray(b), ref, alpha=alpha, beta=beta)
            da, db, dc = dev(tf, a), dev(tf, b), dev(tf, c0)
            plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.ElementwiseMul(), [a.shape, b.shape, c0.shape])
            tf.HipBackend.execute(plan, alpha, [da, db], beta, dc)
            assert relerr(dc.to_numpy(), ref) < TOL[dtype], (name, alpha, beta)
            assert np.array_equal(db.to_numpy(), b) and np.array_equal(da.to_numpy(), a), name
    # through einsum: a Hadamard product whose operands list their modes in different orders
    x, y = rand(rng, (64, 48, 40), dtype), rand(rng, (40, 48, 64), dtype)
    got = tf.einsum("ijk,kji->ijk", [dev(tf, x), dev(tf, y)])
    assert relerr(got.to_numpy(), x * y.transpose(2, 1, 0)) < TOL[dtype]


def test_conj_reference_doc_example(tf):
    # tenferro-tensor/src/lib.rs:612-620
    a = dev(tf, np.array([1 + 2j, 3 - 4j]))
    assert np.array_equal(a.conj().to_numpy(), np.array([1 - 2j, 3 + 4j]))


@pytest.mark.parametrize("dtype", [np.float64, np.complex128])
def test_trace_anti_trace_anti_diag(tf, oracle, dtype):
    rng = seeded_rng(31)
    a = rand(rng, (14, 5, 14, 3), dtype)
    ref = np.empty((3, 5), dtype)
    oracle.trace(a, [0, 1, 2, 3], ref, [3, 1], pairs=[(0, 2)])
    out = tf.Tensor.empty([3, 5], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
    plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Trace([0, 1, 2, 3], [3, 1], [(0, 2)]), [a.shape, [3, 5]])
    tf.HipBackend.execute(plan, 1.0, [dev(tf, a)], 0.0, out)
    assert relerr(out.to_numpy(), ref) < 1e-12
    g = rand(rng, (3, 5), dtype)
    back0 = rand(rng, (14, 5, 14, 3), dtype)
    for op_, ofn, am, av in [(tf.PrimDescriptor.AntiTrace, oracle.anti_trace, [3, 1], g),
                             (tf.PrimDescriptor.AntiDiag, oracle.anti_diag, [3, 1, 0], rand(rng, (3, 5, 14), dtype))]:
        for alpha, beta in [(1.0, 0.0), (2.0, 1.0), (0.5, -1.5)]:
            ref = back0.copy()
            ofn(av, am, ref, [0, 1, 2, 3], pairs=[(0, 2)], alpha=alpha, beta=beta)
            dc = dev(tf, back0)
            plan = tf.HipBackend.plan(dtype, op_(am, [0, 1, 2, 3], [(0, 2)]), [av.shape, back0.shape])
            tf.HipBackend.execute(plan, alpha, [dev(tf, av)], beta, dc)
            assert relerr(dc.to_numpy(), ref) < 1e-12


# ------------------------------------------------------------------------------------------------ einsum
PATTERNS = ["ij,jk->ik", "ii->", "i,j->ij", "i,i->", "ij,j->i", "ii->i", "ijk->", "bij,bjk->bik", "abij,abjk->abik",
            "bij,jk->bik", "ij,jk,kl->il", "ij->ji", "ij,ij->ij", "iij,jk->ik", "i->ii", "i->iii", "ij,(jk,kl)->il",
            "ijx,jk->ik"]


@pytest.mark.parametrize("dtype", [np.float64, np.complex128, np.float32])
@pytest.mark.parametrize("pattern", PATTERNS)
def test_einsum_pattern_catalogue(tf, oracle, dtype, pattern):
    # tenferro-einsum/src/lib.rs:37-93, against the brute-force einsum of the oracle
    rng = seeded_rng(32)
    ext = dict(i=13, j=14, k=15, l=6, a=2, b=3, x=4)
    ins, out = pattern.replace("(", "").replace(")", "").split("->")
    terms = ins.split(",")
    ops = [rand(rng, [ext[l] for l in t], dtype) for t in terms]
    oshape = [ext[l] for l in out]
    ref = np.empty(oshape, dtype)
    oracle.einsum_naive(ops, [lab(t) for t in terms], ref, lab(out))
    res = tf.einsum(pattern, [dev(tf, o) for o in ops])
    assert res.dims() == oshape
    assert relerr(res.to_numpy(), ref) < TOL[dtype]


def test_einsum_reference_doc_examples(tf):
    # tenferro-einsum/src/lib.rs:52-63, 76-93
    v = dev(tf, np.array([1.0, 2.0, 3.0]))
    d = tf.einsum("i->ii", [v])
    assert d.dims() == [3, 3] and np.array_equal(d.to_numpy(), np.diag([1.0, 2.0, 3.0]))
    assert tf.einsum("i->iii", [v]).dims() == [3, 3, 3]
    z = lambda *s: tf.Tensor.zeros(list(s), tf.GpuMemory(0), tf.MemoryOrder.ColumnMajor)
    assert tf.einsum("bij,bjk->bik", [z(10, 3, 4), z(10, 4, 5)]).dims() == [10, 3, 5]
    assert tf.einsum("abij,abjk->abik", [z(2, 3, 4, 5), z(2, 3, 5, 6)]).dims() == [2, 3, 4, 6]
    assert tf.einsum("bij,jk->bik", [z(10, 3, 4), z(4, 5)]).dims() == [10, 3, 5]


@pytest.mark.parametrize("dtype", [np.float64, np.complex128])
def test_einsum_every_tree_of_a_small_network_agrees(tf, oracle, dtype):
    rng = seeded_rng(33)
    ext = dict(a=9, c=8, x=7, y=6, w=3, v=4, s=2, t=2)
    terms, out = ["awc", "asx", "wstv", "cty"], "xvy"
    ops = [rand(rng, [ext[l] for l in t], dtype) for t in terms]
    ref = np.empty([ext[l] for l in out], dtype)
    oracle.einsum_naive(ops, [lab(t) for t in terms], ref, lab(out))
    subs = tf.Subscripts.new([lab(t) for t in terms], lab(out))
    dops = [dev(tf, o) for o in ops]
    orders = [[(0, 1), (4, 2), (5, 3)], [(0, 2), (1, 4), (5, 3)], [(1, 2), (0, 3), (4, 5)], [(2, 3), (0, 1), (4, 5)], [(0, 3), (4, 2), (5, 1)]]
    for pairs in orders:
        tree = tf.ContractionTree.from_pairs(subs, [o.shape for o in ops], pairs)
        res = tf.einsum_with_plan(tree, dops)
        assert relerr(res.to_numpy(), ref) < 1e-12, pairs
    # alpha/beta into a pre-allocated output, twice (accumulate)
    tree = tf.ContractionTree.optimize(subs, [o.shape for o in ops])
    c0 = rand(rng, ref.shape, dtype)
    dc = dev(tf, c0)
    tf.einsum_with_plan_into(tree, dops, 2.0, -1.0, dc)
    assert relerr(dc.to_numpy(), 2 * ref - c0) < 1e-12
    tf.einsum_with_plan_into(tree, dops, 1.0, 1.0, dc)
    assert relerr(dc.to_numpy(), 3 * ref - c0) < 1e-12


def _random_network(rng):
    """A random einsum of 2-5 operands over a pool of labels: repeated labels inside an operand (diagonals), labels
    held by one operand only and absent from the output (summed), labels shared by three operands, a random output
    order, sometimes a repeated output label or an empty output."""
    pool = list("abcdefg")
    ext = {l: int(rng.integers(1, 7)) for l in pool}
    n = int(rng.integers(2, 6))
    terms = []
    for _ in range(n):
        r = int(rng.integers(1, 4))
        t = [str(rng.choice(pool)) for _ in range(r)] if rng.integers(0, 4) == 0 else [str(x) for x in rng.choice(pool, r, replace=False)]
        terms.append("".join(t))
    used = sorted(set("".join(terms)))
    k = int(rng.integers(0, min(4, len(used)) + 1))
    out = [str(x) for x in rng.choice(used, k, replace=False)]
    if out and rng.integers(0, 6) == 0:
        out.append(out[0])
    rng.shuffle(out)
    return terms, "".join(out), ext


@pytest.mark.parametrize("dtype", [np.float64, np.complex128, np.float32])
def test_einsum_random_networks(tf, oracle, dtype):
    # the executor end to end (parser, optimiser, layouts of intermediates, diagonal views, reductions, output
    # diagonals, alpha/beta into a strided output) against the oracle's single-loop-nest einsum
    rng = seeded_rng(59)
    for case in range(60):
        terms, out, ext = _random_network(rng)
        ops = [_random_view(rng, [ext[l] for l in t], dtype) for t in terms]
        oshape = [ext[l] for l in out]
        pattern = ",".join(terms) + "->" + out
        ref = np.empty(oshape, dtype)
        oracle.einsum_naive(ops, [lab(t) for t in terms], ref, lab(out))
        dops = [dev(tf, o) for o in ops]
        res = tf.einsum(pattern, dops)
        assert res.dims() == oshape, pattern
        assert relerr(res.to_numpy(), ref) < 10 * TOL[dtype], (case, pattern, ext)
        if oshape and case % 3 == 0:
            c0 = _random_view(rng, oshape, dtype)
            dc = dev(tf, c0)
            tf.einsum_into(pattern, dops, 0.5, -2.0, dc)
            assert relerr(dc.to_numpy(), 0.5 * ref - 2.0 * c0) < 10 * TOL[dtype], (case, pattern, ext, "into")


def test_einsum_async_chaining(tf):
    # tenferro-einsum/src/lib.rs:158-177: the second call chains on the first result's event
    rng = seeded_rng(34)
    a, b = rng.standard_normal((300, 400)), rng.standard_normal((400, 400))
    da, db = dev(tf, a), dev(tf, b)
    c = tf.einsum("ij,jk->ik", [da, db])
    assert c.event is not None
    d = tf.einsum("ij,jk->ik", [c, db])
    d.wait()
    assert d.is_ready() and d.event is None
    assert relerr(d.to_numpy(), a @ b @ b) < 1e-12


@pytest.mark.parametrize("nb,label", [(0, "(gemm128_kernel"), (6, "(gemm128_kernel, 64x64 tiles)")])
@pytest.mark.parametrize("dtype", ALL)
def test_large_tile_kernel_stage_and_tile_boundaries(tf, dtype, nb, label):
    # The large-tile kernel treats a last k stage that is full, and a tile that lies wholly inside the matrix, like
    # interior ones (plain loads and stores, no predicates); everything else takes the masked paths.  Extents on and
    # around those boundaries -- k a whole number of stages or one element off, rows and columns a whole number of tiles,
    # of 16-byte vectors, or neither -- in the four storage-order combinations of the operands and both orders of the
    # result, with and without an old result to add, against numpy.  Once with enough batch entries for its 128 x 128
    # tiles at every extent below (8-byte reals with so little k change to the small tiles until a launch holds more
    # than 1536 large ones), once with so few that it runs with 64 x 64 tiles.
    if nb == 0:
        nb = {np.float32: 80, np.complex64: 80, np.float64: 385, np.complex128: 257}[dtype]
    rng = seeded_rng(71)
    tol = TOL[dtype]
    stage = {np.float32: 32, np.float64: 16, np.complex64: 16, np.complex128: 8}[dtype]
    seen = set()
    shapes, ks = [(256, 256), (384, 130), (257, 255), (130, 384), (129, 131)], (stage, 2 * stage, 3 * stage, 3 * stage - 1, 2 * stage + 1)
    if nb > 100:   # (hundreds of batch entries: fewer combinations, the same boundaries)
        shapes, ks = [(256, 256), (257, 255), (129, 131)], (stage, 3 * stage - 1, 2 * stage + 1)
    for (m, n) in shapes:
        for k in ks:
            for a_kfast, b_kfast in [(True, True), (True, False), (False, True), (False, False)]:
                a = rand(rng, (nb, m, k), dtype) if a_kfast else rand(rng, (nb, k, m), dtype).transpose(0, 2, 1)
                b = rand(rng, (nb, n, k), dtype).transpose(0, 2, 1) if b_kfast else rand(rng, (nb, k, n), dtype)
                c_row = (m * 7 + n + k) % 2 == 0
                c0 = rand(rng, (nb, m, n), dtype) if c_row else rand(rng, (nb, n, m), dtype).transpose(0, 2, 1)
                beta = 0.0 if (m + k) % 3 == 0 else 0.5
                out = dev(tf, c0)
                plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("bmk"), lab("bkn"), lab("bmn")), [a.shape, b.shape, c0.shape])
                tf.HipBackend.execute(plan, 1.25, [dev(tf, a), dev(tf, b)], beta, out)
                seen.add(tf.last_kernel().split("<")[0])
                wide = np.complex128 if np.iscomplexobj(a) else np.float64
                ref = 1.25 * np.matmul(a.astype(wide), b.astype(wide)) + beta * c0
                err = relerr(out.to_numpy(), ref)
                assert err < tol, (m, n, k, a_kfast, b_kfast, c_row, beta, err, tf.last_kernel())
    assert seen == {label}, seen


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.complex64, np.complex128])
def test_small_products_across_split_counts(tf, dtype):
    # Products with fewer than 256 tiles of 64 x 64 choose their number of k splits from an estimate of the run time: from
    # none (few stages) to hundreds (one tile with a long k).  Whatever it chooses, the result is that of the product:
    # extents that give one tile and many, k from one stage to thousands of elements, ragged in every direction, with
    # alpha and an old result to add, against numpy.
    rng = seeded_rng(83)
    tol = TOL[dtype]
    for (m, n, k) in [(64, 64, 4096), (64, 64, 4099), (128, 128, 128), (256, 256, 256), (200, 200, 2000), (100, 60, 5000),
                      (384, 384, 384), (512, 512, 512), (300, 260, 1103), (33, 47, 129), (64, 64, 33), (1000, 90, 70)]:
        a, b, c0 = rand(rng, (m, k), dtype), rand(rng, (k, n), dtype), rand(rng, (m, n), dtype)
        for alpha, beta in ((1.0, 0.0), (0.75, -0.5)):
            out = dev(tf, c0)
            plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("mk"), lab("kn"), lab("mn")), [a.shape, b.shape, c0.shape])
            tf.HipBackend.execute(plan, alpha, [dev(tf, a), dev(tf, b)], beta, out)
            wide = np.complex128 if np.iscomplexobj(a) else np.float64
            ref = alpha * np.matmul(a.astype(wide), b.astype(wide)) + beta * c0
            err = relerr(out.to_numpy(), ref)
            assert err < tol, (m, n, k, alpha, beta, err, tf.last_kernel())


# ------------------------------------------------------------------------------------------------ conj on load
def _contract_np(a, ma, b, mb, mc):
    return np.einsum(f"{ma},{mb}->{mc}", a, b, optimize=True)


@pytest.mark.parametrize("dtype", [np.complex64, np.complex128])
def test_conj_on_load_in_every_contraction_kernel(tf, dtype):
    # TFH_VIEW_CONJ (Tensor.conj_on_load): the operand is read as its conjugate, with no conjugated copy, by the four MFMA
    # contraction kernels; shapes that go to the other kernels get a conjugated copy first.  Each shape with the flag on
    # A, on B and on both, alpha and beta complex, against numpy on explicitly conjugated operands; the routing is
    # checked so that every kernel's sign flip is exercised, including the paths that exchange the operands.
    rng = seeded_rng(61)
    tol = TOL[dtype]
    cases = [   # (modes a, modes b, modes c, extents, substring of the kernel label expected)
        ("mk", "kn", "mn", dict(m=2000, k=600, n=1500), ", 128>)"),
        ("mk", "kn", "nm", dict(m=2000, k=600, n=1500), ", 128>)"),             # C's fastest axis is m: operands exchanged
        ("km", "nk", "mn", dict(m=2000, k=600, n=1500), ", 128>)"),             # A column-contiguous, B k-contiguous
        ("mk", "kn", "mn", dict(m=32768, k=64, n=40), "128x64 tiles"),                # thin right-hand side: 128x64 tiles
        ("mk", "kn", "mn", dict(m=40, k=64, n=32768), "128x64 tiles"),                # thin left-hand side: exchanged
        ("mk", "kn", "mn", dict(m=40, k=30, n=50), "64x64 tiles"),
        ("bmk", "bkn", "bmn", dict(b=70, m=20, k=24, n=18), "gemm_wave_kernel"),
        ("xk", "mk", "xm", dict(x=4096, k=16, m=12), None),                     # small operator on a long tensor
        ("mk", "k", "m", dict(m=500, k=300), None),                              # matrix . vector: conjugated copy, then the reduction kernel
        ("ab", "xby", "xay", dict(a=2, b=2, x=300, y=300), None),               # tiny operator: conjugated copy
        ("asx", "x", "asx", dict(a=30, s=2, x=40), None),                        # nothing summed: conjugated copy
    ]
    if dtype == np.complex128:
        cases.append(("mk", "xk", "xm", dict(m=16, k=32, x=8192), "gemm_skinny_kernel"))
        cases.append(("xk", "km", "xm", dict(m=16, k=32, x=8192), "gemm_skinny_kernel"))
    seen = set()
    for ma, mb, mc, ext, want in cases:
        a = rand(rng, [ext[l] for l in ma], dtype)
        b = rand(rng, [ext[l] for l in mb], dtype)
        c0 = rand(rng, [ext[l] for l in mc], dtype)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab(ma), lab(mb), lab(mc)), [a.shape, b.shape, c0.shape])
        alpha, beta = 0.7 - 1.1j, -0.3 + 0.2j
        da, db = dev(tf, a), dev(tf, b)
        for ca, cb in [(True, False), (False, True), (True, True)]:
            out = dev(tf, c0)
            tf.HipBackend.execute(plan, alpha, [da.conj_on_load() if ca else da, db.conj_on_load() if cb else db], beta, out)
            label = tf.last_kernel()
            if want is not None:
                assert want in label, (ma, mb, mc, want, label)
                seen.add(want)
            ref = alpha * _contract_np(np.conj(a) if ca else a, ma, np.conj(b) if cb else b, mb, mc) + beta * c0
            assert relerr(out.to_numpy(), ref) < tol, (ma, mb, mc, ca, cb, label)
    assert {", 128>)", "128x64 tiles", "64x64 tiles", "gemm_wave_kernel"} <= seen
    # the kernel with 64-bit offsets takes what the others cannot address: rows of A 2 GiB apart (a view of a large
    # buffer of which only those rows are ever touched; more than eight rows, or a conjugated copy would be made first)
    import torch
    m, k, n = 9, 30, 50
    gap = (1 << 31) // np.dtype(dtype).itemsize
    big = torch.empty((m - 1) * gap + k, dtype=torch.complex64 if dtype == np.complex64 else torch.complex128, device="cuda")
    a = rand(rng, (m, k), dtype)
    for r in range(m):
        big[r * gap:r * gap + k] = torch.from_numpy(a[r]).cuda()
    A = tf.Tensor(big, [m, k], [gap, 1], 0, tf.GpuMemory(0), tf.dtype_code(np.dtype(dtype)))
    b = rand(rng, (k, n), dtype)
    c0 = rand(rng, (m, n), dtype)
    plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("mk"), lab("kn"), lab("mn")), [[m, k], [k, n], [m, n]])
    for ca, cb in [(True, False), (False, True), (True, True)]:
        out = dev(tf, c0)
        tf.HipBackend.execute(plan, alpha, [A.conj_on_load() if ca else A, dev(tf, b).conj_on_load() if cb else dev(tf, b)], beta, out)
        assert "(gemm_kernel" in tf.last_kernel(), tf.last_kernel()
        ref = alpha * ((np.conj(a) if ca else a) @ (np.conj(b) if cb else b)) + beta * c0
        assert relerr(out.to_numpy(), ref) < tol, (ca, cb)


def test_conj_on_load_views_einsum_permute_and_rejections(tf, oracle):
    rng = seeded_rng(62)
    a = rand(rng, (12, 2, 14), np.complex128)
    L = rand(rng, (12, 5, 12), np.complex128)
    W = rand(rng, (5, 2, 2, 5), np.complex128)
    dA, dL, dW = dev(tf, a), dev(tf, L), dev(tf, W)
    # the benchmark's network with its fourth operand as a flagged view of the second: equal to the explicit conj(A)
    lazy = tf.einsum("awc,asx,wstv,cty->xvy", [dL, dA, dW, dA.conj_on_load()])
    eager = tf.einsum("awc,asx,wstv,cty->xvy", [dL, dA, dW, dA.conj()])
    ref = np.einsum("awc,asx,wstv,cty->xvy", L, a, W, np.conj(a))
    assert relerr(lazy.to_numpy(), ref) < 1e-12 and relerr(eager.to_numpy(), ref) < 1e-12
    # views of a flagged tensor keep the flag; to_numpy shows the logical values; conj() of it is a plain copy
    v = dA.conj_on_load().permute([2, 0, 1])
    assert np.array_equal(v.to_numpy(), np.conj(a).transpose(2, 0, 1))
    assert np.array_equal(dA.conj_on_load().conj().to_numpy(), a)
    w = dA.conj_on_load()
    assert w.into_conj() is w and np.array_equal(w.to_numpy(), a)
    # Permute honours the flag (bit-exact sign flip), with alpha and beta too
    out = tf.Tensor.empty([14, 12, 2], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.complex128)
    plan = tf.HipBackend.plan(np.complex128, tf.PrimDescriptor.Permute([0, 1, 2], [2, 0, 1]), [a.shape, [14, 12, 2]])
    tf.HipBackend.execute(plan, 1.0, [dA.conj_on_load()], 0.0, out)
    assert out.to_numpy().tobytes() == np.ascontiguousarray(np.conj(a).transpose(2, 0, 1)).tobytes()
    # a labelled sum of a flagged operand inside einsum (conj of the sum)
    s = tf.einsum("asx->ax", [dA.conj_on_load()])
    assert relerr(s.to_numpy(), np.conj(a).sum(axis=1)) < 1e-12
    p = tf.einsum("asx,x->as", [dA.conj_on_load(), dev(tf, a[0, 0, :].copy())])
    assert relerr(p.to_numpy(), np.einsum("asx,x->as", np.conj(a), a[0, 0, :])) < 1e-12
    # real tensors: the flag is not set at all
    r = dev(tf, rng.standard_normal((4, 4)))
    assert r.conj_on_load()._conj is False
    # not taken: other operations, outputs
    red = tf.HipBackend.plan(np.complex128, tf.PrimDescriptor.Reduce([0, 1, 2], [0, 2], tf.ReduceOp.Sum), [a.shape, [12, 14]])
    o2 = tf.Tensor.empty([12, 14], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.complex128)
    with pytest.raises(tf.InvalidArgument):
        tf.HipBackend.execute(red, 1.0, [dA.conj_on_load()], 0.0, o2)
    with pytest.raises(tf.InvalidArgument):
        tf.HipBackend.execute(plan, 1.0, [dA], 0.0, out.conj_on_load())


def _new_streams(tf, n):
    import ctypes
    out = []
    for _ in range(n):
        st = ctypes.c_void_p()
        assert tf.lib().tfh_stream_create(ctypes.byref(st)) == 0
        out.append(st)
    return out


def test_chaining_across_two_streams_through_the_completion_event(tf):
    # tenferro-einsum/src/lib.rs:146-177: the producer runs on one stream, the consumer on another, and the only thing
    # that orders them is the producer's completion event, which the consumer's stream is made to wait for.  The producer
    # is long (2 x 2048^3 f64 per call, four calls queued) and the consumer is enqueued at once: without the wait it
    # would read a half-written operand.  Both the einsum path and TensorPrims::execute.
    import torch
    rng = seeded_rng(35)
    n = 2048
    a = rng.standard_normal((n, n)) / 32
    b = rng.standard_normal((n, n)) / 32
    da, db = dev(tf, a), dev(tf, b)
    sa, sb = _new_streams(tf, 2)
    torch.cuda.synchronize()
    try:
        c = da
        for _ in range(4):
            c = tf.einsum("ij,jk->ik", [c, db], stream=sa.value)
        assert c.event is not None
        d = tf.einsum("ij,jk->ki", [c, db], stream=sb.value)       # consumer on the other stream
        d.wait()
        ref = a @ b @ b @ b @ b
        assert relerr(d.to_numpy(), (ref @ b).T) < 1e-12
        # the same through execute(): output.event is set by the producer and waited for by the consumer
        plan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Contract(lab("ij"), lab("jk"), lab("ik")), [[n, n], [n, n], [n, n]])
        x = tf.Tensor.empty([n, n], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64)
        y = tf.Tensor.empty([n, n], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64)
        z = tf.Tensor.empty([n, n], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64)
        torch.cuda.synchronize()
        tf.HipBackend.execute(plan, 1.0, [da, db], 0.0, x, stream=sa.value)
        tf.HipBackend.execute(plan, 1.0, [x, db], 0.0, y, stream=sa.value)
        assert y.event is not None
        tf.HipBackend.execute(plan, 1.0, [y, db], 0.0, z, stream=sb.value)
        z.wait()
        assert relerr(z.to_numpy(), a @ b @ b @ b) < 1e-12
    finally:
        torch.cuda.synchronize()
        for st in (sa, sb):
            tf.lib().tfh_stream_destroy(st)


def test_host_transfers_pageable_and_pinned_round_trip(tf):
    # tfh_memcpy_h2d / tfh_memcpy_d2h (Tensor::to_memory_space_async): pageable memory goes through the stream's pinned
    # staging buffers in 16 MiB chunks (sizes below, at and above one and two chunks, odd byte counts), pinned memory
    # from tfh_host_malloc directly; data comes back bit for bit
    import ctypes
    import torch
    L = tf.lib()
    (st,) = _new_streams(tf, 1)
    rng = seeded_rng(36)
    try:
        for nbytes in [1, 4097, (16 << 20) - 3, 16 << 20, (16 << 20) + 5, (40 << 20) + 1]:
            src = rng.integers(0, 256, nbytes, dtype=np.uint8)
            dbuf = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
            back = np.zeros(nbytes, np.uint8)
            assert L.tfh_memcpy_h2d(dbuf.data_ptr(), src.ctypes.data, nbytes, st) == 0
            assert L.tfh_memcpy_d2h(back.ctypes.data, dbuf.data_ptr(), nbytes, st) == 0   # returns with the data in place
            assert np.array_equal(back, src), nbytes
            assert np.array_equal(dbuf.cpu().numpy(), src), nbytes
        # pinned: the calls return at once; the stream orders the copies
        nbytes = (24 << 20) + 7
        hp, hq = ctypes.c_void_p(), ctypes.c_void_p()
        assert L.tfh_host_malloc(nbytes, ctypes.byref(hp)) == 0 and L.tfh_host_malloc(nbytes, ctypes.byref(hq)) == 0
        src = rng.integers(0, 256, nbytes, dtype=np.uint8)
        ctypes.memmove(hp.value, src.ctypes.data, nbytes)
        dbuf = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        assert L.tfh_memcpy_h2d(dbuf.data_ptr(), hp, nbytes, st) == 0
        assert L.tfh_memcpy_d2h(hq, dbuf.data_ptr(), nbytes, st) == 0
        assert L.tfh_stream_synchronize(st) == 0
        back = np.ctypeslib.as_array(ctypes.cast(hq.value, ctypes.POINTER(ctypes.c_uint8)), shape=(nbytes,))
        assert np.array_equal(back, src)
        assert L.tfh_host_free(hp) == 0 and L.tfh_host_free(hq) == 0
    finally:
        L.tfh_stream_destroy(st)


def test_two_host_threads_copy_pageable_memory_on_one_stream(tf):
    # both threads stage through the stream's two pinned buffers: a transfer holds them from its first chunk to its last,
    # so neither carries the other's bytes; uploads and downloads, several chunks each, on the null stream and on a created one
    import threading
    import torch
    L = tf.lib()
    (st,) = _new_streams(tf, 1)
    rng = seeded_rng(136)
    try:
        for stream in (None, st):
            nbytes = [(40 << 20) + 3, (33 << 20) + 1]
            srcs = [rng.integers(0, 256, n, dtype=np.uint8) for n in nbytes]
            dbufs = [torch.empty(n, dtype=torch.uint8, device="cuda") for n in nbytes]
            backs = [np.zeros(n, np.uint8) for n in nbytes]
            rcs = [[], []]

            def work(i):
                for _ in range(3):
                    rcs[i].append(L.tfh_memcpy_h2d(dbufs[i].data_ptr(), srcs[i].ctypes.data, nbytes[i], stream))
                    rcs[i].append(L.tfh_memcpy_d2h(backs[i].ctypes.data, dbufs[i].data_ptr(), nbytes[i], stream))
            threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
            for t in threads:
                t.start()
            for t in threads:
                t.join()
            assert L.tfh_stream_synchronize(stream) == 0
            for i in range(2):
                assert rcs[i] == [0] * 6
                assert np.array_equal(backs[i], srcs[i]), i
                assert np.array_equal(dbufs[i].cpu().numpy(), srcs[i]), i
    finally:
        assert L.tfh_stream_destroy(st) == 0
    # a destroyed stream leaves no staging buffers behind, and the null stream's go with tfh_release_workspaces
    torch.cuda.synchronize()
    assert L.tfh_release_workspaces() == 0


def test_host_to_device_copy_runs_beside_a_contraction_on_another_stream(tf):
    # a staged transfer from pageable memory on stream A and contractions on stream B, each alone and then together
    # (the transfer from a second host thread, because its host side is busy copying into the staging buffers): together
    # they must take clearly less than one after the other
    import threading
    import time
    import torch
    L = tf.lib()
    sa, sb = _new_streams(tf, 2)
    n = 3072
    da = tf.Tensor.from_torch(torch.randn(n, n, dtype=torch.float64, device="cuda"))
    db = tf.Tensor.from_torch(torch.randn(n, n, dtype=torch.float64, device="cuda"))
    dc = tf.Tensor.empty([n, n], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64)
    plan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Contract(lab("ij"), lab("jk"), lab("ik")), [[n, n], [n, n], [n, n]])
    nbytes = 192 << 20
    src = np.ones(nbytes, np.uint8)
    dbuf = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()

    def copy():
        assert L.tfh_memcpy_h2d(dbuf.data_ptr(), src.ctypes.data, nbytes, sa) == 0
        assert L.tfh_stream_synchronize(sa) == 0

    def timed(fn):
        t0 = time.perf_counter()
        fn()
        return time.perf_counter() - t0

    try:
        copy()                                                        # staging buffers allocated, pages touched
        t_copy = min(timed(copy) for _ in range(3))
        reps = 1
        def compute():
            for _ in range(reps):
                tf.HipBackend.execute(plan, 1.0, [da, db], 0.0, dc, stream=sb.value)
            assert L.tfh_stream_synchronize(sb) == 0
        compute()
        t_one = min(timed(compute) for _ in range(3))
        reps = max(1, int(round(t_copy / t_one)))                     # about as much compute as the copy takes
        t_comp = min(timed(compute) for _ in range(3))

        def both():
            th = threading.Thread(target=copy)
            th.start()
            compute()
            th.join()
        t_both = min(timed(both) for _ in range(3))
        print("copy %.2f ms, compute %.2f ms, together %.2f ms" % (t_copy * 1e3, t_comp * 1e3, t_both * 1e3))
        assert t_both < t_copy + t_comp - 0.4 * min(t_copy, t_comp), (t_copy, t_comp, t_both)
    finally:
        torch.cuda.synchronize()
        for st in (sa, sb):
            L.tfh_stream_destroy(st)


def test_execute_errors(tf):
    a = tf.Tensor.zeros([3, 4], tf.GpuMemory(0), tf.MemoryOrder.RowMajor)
    b = tf.Tensor.zeros([4, 5], tf.GpuMemory(0), tf.MemoryOrder.RowMajor)
    c = tf.Tensor.zeros([3, 5], tf.GpuMemory(0), tf.MemoryOrder.RowMajor)
    plan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Contract([0, 1], [1, 2], [0, 2]), [[3, 4], [4, 5], [3, 5]])
    with pytest.raises(tf.ShapeMismatch) as e:
        tf.HipBackend.execute(plan, 1.0, [b, b], 0.0, c)
    assert e.value.expected == [3, 4] and e.value.got == [4, 5]
    with pytest.raises(tf.RankMismatch):
        tf.HipBackend.execute(plan, 1.0, [a, b], 0.0, tf.Tensor.zeros([15], tf.GpuMemory(0), tf.MemoryOrder.RowMajor))
    with pytest.raises(tf.InvalidArgument):
        tf.HipBackend.execute(plan, 1.0, [a], 0.0, c)
    with pytest.raises(tf.Strided):
        tf.HipBackend.execute(plan, 1.0, [a, b], 0.0, tf.Tensor.zeros([3, 1], tf.GpuMemory(0), tf.MemoryOrder.RowMajor).broadcast([3, 5]))
    host = tf.Tensor.from_slice(np.zeros(12), [3, 4], tf.MemoryOrder.ColumnMajor)
    with pytest.raises(tf.CrossMemorySpaceOperation):
        tf.einsum("ij,jk->ik", [host, b])
    with pytest.raises(tf.NoCompatibleComputeDevice):
        tf.einsum("ij,jk->ik", [host, tf.Tensor.from_slice(np.zeros(20), [4, 5], tf.MemoryOrder.ColumnMajor)])
    assert [str(d) for d in tf.preferred_compute_devices(tf.GpuMemory(0), tf.OpKind.Contract)] == ["hip:0"]
    with pytest.raises(tf.NoCompatibleComputeDevice):
        tf.preferred_compute_devices(tf.GpuMemory(99), tf.OpKind.Contract)


# ------------------------------------------------------------------------------------------------ kernel-variant coverage
def _permute_check(tf, oracle, a, perm, alpha=1.0, beta=0.0, b0=None):
    shape = [a.shape[p] for p in perm]
    modes = list(range(a.ndim))
    ref = np.zeros(shape, a.dtype) if b0 is None else b0.copy()
    oracle.permute(a, modes, ref, list(perm), alpha=alpha, beta=beta)
    out = dev(tf, np.zeros(shape, a.dtype) if b0 is None else b0)
    plan = tf.HipBackend.plan(a.dtype, tf.PrimDescriptor.Permute(modes, list(perm)), [a.shape, shape])
    tf.HipBackend.execute(plan, alpha, [dev(tf, a)], beta, out)
    return out.to_numpy(), ref


@pytest.mark.parametrize("dtype,shape", [(np.float32, (16,) * 6), (np.float64, (16, 16, 16, 16, 16, 8)), (np.complex128, (16, 16, 16, 8, 16, 8)),
                                         (np.float64, (4, 16, 16, 16, 16, 16))])
def test_permute_large_tiles_for_far_apart_rows_bit_exact(tf, oracle, dtype, shape):
    # an axis that is contiguous on one side and the slowest on the other: every tile touches rows megabytes apart,
    # and the copy takes the large-tile variant (512 threads, four times the tile, the longer run on the scattered
    # side).  Bit-exact against numpy's transpose; the identity and a near-identity stay on the ordinary tiles.
    rng = seeded_rng(44)
    a = rand(rng, shape, dtype)
    da = dev(tf, a)
    large = 0
    for perm in [(5, 2, 0, 4, 1, 3), (1, 2, 3, 4, 5, 0), (2, 4, 1, 5, 3, 0), (5, 0, 1, 2, 3, 4), (0, 1, 2, 3, 4, 5), (0, 1, 2, 5, 3, 4)]:
        oshape = [shape[p] for p in perm]
        out = tf.Tensor.empty(oshape, tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Permute(list(range(6)), list(perm)), [shape, oshape])
        tf.HipBackend.execute(plan, 1.0, [da], 0.0, out)
        label = tf.last_kernel()
        is_large = label.endswith("512, true>)")
        large += is_large
        assert out.to_numpy().tobytes() == np.ascontiguousarray(a.transpose(perm)).tobytes(), (perm, label)
        if perm in [(0, 1, 2, 3, 4, 5), (0, 1, 2, 5, 3, 4)]:
            assert not is_large, (perm, label)
    assert large >= 2, large


@pytest.mark.parametrize("dtype", ALL)
def test_permute_power_of_two_shapes_take_the_vector_path(tf, oracle, dtype):
    # every tile full, contiguous fastest axes on both sides: 16-byte accesses, no bounds checks
    rng = seeded_rng(41)
    a = rand(rng, (32, 8, 64, 16), dtype)
    for perm in [(3, 1, 0, 2), (0, 1, 2, 3), (2, 3, 0, 1), (1, 0, 3, 2)]:
        got, ref = _permute_check(tf, oracle, a, perm)
        assert copy_kernel_is_fast(tf.last_kernel()), tf.last_kernel()
        assert got.tobytes() == ref.tobytes(), perm
    b0 = rand(rng, (16, 8, 32, 64), dtype)
    alpha, beta = (0.5 - 2j, 1.5 + 1j) if np.issubdtype(dtype, np.complexfloating) else (0.5, -1.5)
    got, ref = _permute_check(tf, oracle, a, (3, 1, 0, 2), alpha, beta, b0)
    assert relerr(got, ref) < TOL[dtype]


def test_permute_misaligned_base_and_odd_inner_extent(tf, oracle):
    # a view that starts one element into its buffer is only 8-byte aligned: the scalar path must be used
    rng = seeded_rng(42)
    big = rng.standard_normal(64 * 64 * 16 + 1)
    a = big[1:].reshape(64, 64, 16)
    got, ref = _permute_check(tf, oracle, a, (2, 0, 1))
    assert got.tobytes() == ref.tobytes()
    b = rng.standard_normal((64, 30, 17))            # partial tiles on every axis
    got, ref = _permute_check(tf, oracle, b, (2, 1, 0))
    assert not copy_kernel_is_fast(tf.last_kernel()), tf.last_kernel()      # bounds-checked
    assert got.tobytes() == ref.tobytes()


def _reduce_check(tf, oracle, a, modes_a, modes_c, op_tf, op_or, alpha=1.0, beta=0.0, c0=None):
    ext = dict(zip(modes_a, a.shape))
    shape = [ext[m] for m in modes_c]
    ref = np.zeros(shape, a.dtype) if c0 is None else c0.copy()
    oracle.reduce(a, modes_a, ref, modes_c, op=op_or, alpha=alpha, beta=beta)
    out = dev(tf, np.full(shape, np.nan, a.dtype) if c0 is None else c0)
    plan = tf.HipBackend.plan(a.dtype, tf.PrimDescriptor.Reduce(list(modes_a), list(modes_c), op_tf), [a.shape, shape])
    tf.HipBackend.execute(plan, alpha, [dev(tf, a)], beta, out)
    return out.to_numpy(), ref


@pytest.mark.parametrize("dtype", ALL)
def test_reduce_fast_path_variants(tf, oracle, dtype):
    rng = seeded_rng(43)
    a = rand(rng, (8, 16, 4, 16, 32), dtype)
    m = [0, 1, 2, 3, 4]
    cases = [[0, 1, 2, 3],          # contiguous axis reduced, few addends: block-serial kept indices
             [0, 2, 4],             # contiguous axis kept, two reduced axes
             [4, 0],                # output order differs from input order
             [1, 2, 3, 4],          # slowest axis reduced
             [3]]
    for mc in cases:
        got, ref = _reduce_check(tf, oracle, a, m, mc, tf.ReduceOp.Sum, oracle.SUM)
        # the first two and the fourth must take the tiled fast path for every dtype, and so must the 16-output case
        # ([3]: the serial range is split over blocks and folded by a second launch)
        if mc in ([0, 1, 2, 3], [0, 2, 4], [1, 2, 3, 4], [3]):
            assert "reduce_fast_kernel" in tf.last_kernel(), (mc, tf.last_kernel())
        assert relerr(got, ref) < TOL[dtype], mc
    c0 = rand(rng, (8, 4, 32), dtype)
    got, ref = _reduce_check(tf, oracle, a, m, [0, 2, 4], tf.ReduceOp.Sum, oracle.SUM, alpha=2.0, beta=-0.5, c0=c0)
    assert relerr(got, ref) < TOL[dtype]
    if np.issubdtype(dtype, np.complexfloating):
        got, ref = _reduce_check(tf, oracle, a, m, [0, 2, 4], tf.ReduceOp.Sum, oracle.SUM, alpha=0.5 - 1j, beta=0.25j, c0=c0)
        assert relerr(got, ref) < TOL[dtype]          # complex alpha/beta: general kernel
    else:
        for op_tf, op_or in [(tf.ReduceOp.Max, oracle.MAX), (tf.ReduceOp.Min, oracle.MIN)]:
            got, ref = _reduce_check(tf, oracle, a, m, [0, 2, 4], op_tf, op_or)
            assert np.array_equal(got, ref)


def test_reduce_misaligned_base_and_split_reductions(tf, oracle):
    rng = seeded_rng(44)
    big = rng.standard_normal(16 * 16 * 64 + 1)
    a = big[1:].reshape(16, 16, 64)                   # 8-byte aligned only
    got, ref = _reduce_check(tf, oracle, a, [0, 1, 2], [0, 2], tf.ReduceOp.Sum, oracle.SUM)
    assert relerr(got, ref) < 1e-12
    # few outputs, long reductions: split over blocks + second pass, every dtype of accumulator layout
    b = rng.standard_normal((5, 300000))
    got, ref = _reduce_check(tf, oracle, b, [0, 1], [0], tf.ReduceOp.Sum, oracle.SUM)
    assert relerr(got, ref) < 1e-12
    got, ref = _reduce_check(tf, oracle, b, [0, 1], [0], tf.ReduceOp.Max, oracle.MAX)
    assert np.array_equal(got, ref)
    z = (rng.standard_normal(1 << 20) + 1j * rng.standard_normal(1 << 20))
    got, ref = _reduce_check(tf, oracle, z, [0], [], tf.ReduceOp.Sum, oracle.SUM, alpha=1 - 2j)
    assert relerr(got, ref) < 1e-12
    c = rng.standard_normal((4096, 48))
    got, ref = _reduce_check(tf, oracle, c, [0, 1], [1], tf.ReduceOp.Sum, oracle.SUM)
    assert relerr(got, ref) < 1e-12


BIG_CASES = [
    # enough 128x128 tiles and k stages (tiles x stages / 8 > 128) that they are preferred to 64x64 tiles and split over k
    ("ajbk,kcj->abc", dict(a=48, j=24, b=16, k=48, c=672)),     # two-mode k through offset tables, packed B
    ("mk,kn->mn", dict(m=812, k=1103, n=772)),                   # ragged edges and a k tail
    ("km,nk->mn", dict(m=768, k=1040, n=896)),
    ("mk,nk->nm", dict(m=712, k=1030, n=642)),                   # operands swap
    ("bmk,kbn->bmn", dict(b=3, m=386, k=1050, n=396)),           # batch
]


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("case", BIG_CASES, ids=[c[0] for c in BIG_CASES])
def test_contract_128_tile_kernel(tf, oracle, dtype, case):
    pattern, ext = case
    ins, mc = pattern.split("->")
    ma, mb = ins.split(",")
    rng = seeded_rng(45)
    a = rand(rng, [ext[l] for l in ma], dtype)
    b = rand(rng, [ext[l] for l in mb], dtype)
    cshape = [ext[l] for l in mc]
    alpha, beta = (0.7 - 1.1j, -0.3 + 0.2j) if np.issubdtype(dtype, np.complexfloating) else (0.7, -0.3)
    c0 = rand(rng, cshape, dtype)
    ref = c0.copy()
    oracle.contract(a, lab(ma), b, lab(mb), ref, lab(mc), alpha=alpha, beta=beta)
    out = dev(tf, c0)
    plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab(ma), lab(mb), lab(mc)), [a.shape, b.shape, cshape])
    tf.HipBackend.execute(plan, alpha, [dev(tf, a), dev(tf, b)], beta, out)
    assert "gemm128_kernel" in tf.last_kernel(), tf.last_kernel()
    assert relerr(out.to_numpy(), ref) < TOL[dtype]


@pytest.mark.parametrize("dtype", [np.float64, np.complex128])
def test_contract_128_tile_negative_strides_and_offsets(tf, oracle, dtype):
    # reversed views: the kernel rebases each operand to its lowest address
    rng = seeded_rng(46)
    abig, bbig = rand(rng, (400, 310), dtype), rand(rng, (310, 280), dtype)
    av, bv = abig[::-2, ::-1][:, 5:], bbig[::-1, ::-2][5:, :]      # 200 x 305, 305 x 140
    ref = np.empty((200, 140), dtype)
    oracle.contract(av, lab("mk"), bv, lab("kn"), ref, lab("mn"))
    out = tf.Tensor.empty([200, 140], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
    plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("mk"), lab("kn"), lab("mn")), [av.shape, bv.shape, [200, 140]])
    tf.HipBackend.execute(plan, 1.0, [dev(tf, av), dev(tf, bv)], 0.0, out)
    assert relerr(out.to_numpy(), ref) < TOL[dtype]


def test_config3_full_size_complex128(tf, oracle):
    # "awc,asx,wstv,cty->xvy", chi=1024, D=16, d=2: the optimiser's tree on the GPU against the oracle along the same tree
    from tenferro_rs_amd import inputs
    chi, D, d = 1024, 16, 2
    sig = 1.0 / np.sqrt(chi)
    L = inputs.complex_normal(1003, 0, (chi, D, chi), sig)
    A = inputs.complex_normal(1003, 1, (chi, d, chi), sig)
    W = inputs.complex_normal(1003, 2, (D, d, d, D), sig)
    host = [L, A, W, np.conj(A)]
    terms, out = ["awc", "asx", "wstv", "cty"], "xvy"
    subs = tf.Subscripts.parse(",".join(terms) + "->" + out)
    tree = tf.ContractionTree.optimize(subs, [x.shape for x in host])
    assert abs(8 * tree.mac_count - 558.3e9) < 0.1e9
    res = tf.einsum_with_plan(tree, [dev(tf, x) for x in host])
    ref = np.empty((chi, D, chi), np.complex128)
    oracle.einsum_pairs(host, [lab(t) for t in terms], ref, lab(out), tree.steps)
    assert relerr(res.to_numpy(), ref) < 1e-12


# sizes that the launcher gives to the 128x128 kernel: a long k (>= 32 stages) over few tiles, or many tiles over a k
# shorter than one vector
# (the last three leave fewer k than one vector in the final stage: its window then starts inside the previous stage)
ODD_SIZES = [(641, 1031, 645), (767, 1077, 769), (1801, 5, 1795), (1810, 3, 1811), (1793, 4, 1800), (4673, 1058, 97),
             (769, 1025, 641), (642, 1027, 643), (1801, 66, 1795)]
LAYOUTS = [("mk", "kn"), ("mk", "nk"), ("km", "kn"), ("km", "nk")]


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("layout", LAYOUTS, ids=["NN", "NT", "TN", "TT"])
def test_contract_odd_extents_take_the_straddling_vector_path(tf, oracle, dtype, layout):
    # extents that are not multiples of the 16-byte vector length: the last vector of a row or column straddles the
    # end of the operand and is loaded from a window moved back inside it (k smaller than one vector: scalar path)
    ma, mb = layout
    rng = seeded_rng(47)
    for m, k, n in ODD_SIZES:
        ext = dict(m=m, k=k, n=n)
        a = rand(rng, [ext[l] for l in ma], dtype)
        b = rand(rng, [ext[l] for l in mb], dtype)
        ref = np.empty((m, n), dtype)
        oracle.contract(a, lab(ma), b, lab(mb), ref, lab("mn"))
        out = dev(tf, np.full((m, n), np.nan, dtype))
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab(ma), lab(mb), lab("mn")), [a.shape, b.shape, [m, n]])
        tf.HipBackend.execute(plan, 1.0, [dev(tf, a), dev(tf, b)], 0.0, out)
        assert "gemm128_kernel" in tf.last_kernel(), (m, k, n, tf.last_kernel())
        assert relerr(out.to_numpy(), ref) < TOL[dtype], (m, k, n)


THIN_SIZES = [(257, 1025, 33), (130, 523, 64), (300, 1040, 95), (47, 1031, 260), (64, 520, 1300), (1801, 66, 67), (513, 5, 80),
              # a last tile with fewer valid rows than a 16-byte vector and a short k: the vector moved back at the
              # edge starts before its tile
              (257, 40, 65), (385, 100, 65), (130, 24, 67), (65, 40, 257)]


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("layout", LAYOUTS, ids=["NN", "NT", "TN", "TT"])
def test_contract_thin_side_takes_128x64_tiles(tf, oracle, dtype, layout):
    # one free group of 33..95 real columns and a long other side: 128x64 tiles of the large-tile kernel, whichever
    # operand is the thin one (the operands are exchanged so that it becomes the right-hand side)
    ma, mb = layout
    rng = seeded_rng(147)
    ec = 2 if np.issubdtype(dtype, np.complexfloating) else 1
    for m, k, n in THIN_SIZES:
        ext = dict(m=m, k=k, n=n)
        a = rand(rng, [ext[l] for l in ma], dtype)
        b = rand(rng, [ext[l] for l in mb], dtype)
        c0 = rand(rng, (m, n), dtype)
        ref = c0.copy()
        oracle.contract(a, lab(ma), b, lab(mb), ref, lab("mn"), alpha=0.5, beta=-1.5)
        out = dev(tf, c0)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab(ma), lab(mb), lab("mn")), [a.shape, b.shape, [m, n]])
        print("thin", dtype.__name__, ma, mb, m, k, n, flush=True)
        tf.HipBackend.execute(plan, 0.5, [dev(tf, a), dev(tf, b)], -1.5, out)
        thin = min(m, n)
        if 33 <= thin * ec < 96:
            assert "gemm128_kernel, 128x64" in tf.last_kernel(), (m, k, n, tf.last_kernel())
        assert relerr(out.to_numpy(), ref) < TOL[dtype], (m, k, n, tf.last_kernel())


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("layout", LAYOUTS, ids=["NN", "NT", "TN", "TT"])
def test_contract_odd_extents_few_tiles(tf, oracle, dtype, layout):
    # the same kind of extents with so few tiles that the 64x64 kernel (or, for complex128, the large-tile one) is chosen
    ma, mb = layout
    rng = seeded_rng(148)
    for m, k, n in [(129, 1031, 133), (255, 1077, 257), (193, 1058, 97), (257, 1025, 129), (130, 1027, 131), (131, 37, 129), (300, 5, 310)]:
        ext = dict(m=m, k=k, n=n)
        a = rand(rng, [ext[l] for l in ma], dtype)
        b = rand(rng, [ext[l] for l in mb], dtype)
        ref = np.empty((m, n), dtype)
        oracle.contract(a, lab(ma), b, lab(mb), ref, lab("mn"))
        out = dev(tf, np.full((m, n), np.nan, dtype))
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab(ma), lab(mb), lab("mn")), [a.shape, b.shape, [m, n]])
        tf.HipBackend.execute(plan, 1.0, [dev(tf, a), dev(tf, b)], 0.0, out)
        assert relerr(out.to_numpy(), ref) < TOL[dtype], (m, k, n, tf.last_kernel())


def test_contract_operand_ending_at_the_end_of_its_allocation(tf, oracle):
    # the operands are the tail of exactly-sized device buffers: a read past the last element would leave the buffer
    rng = seeded_rng(48)
    for dtype, m, k, n in [(np.float32, 643, 1033, 641), (np.float64, 641, 523, 643)]:
        for ma, mb in LAYOUTS:
            ext = dict(m=m, k=k, n=n)
            a = rand(rng, [ext[l] for l in ma], dtype)
            b = rand(rng, [ext[l] for l in mb], dtype)
            ref = np.empty((m, n), dtype)
            oracle.contract(a, lab(ma), b, lab(mb), ref, lab("mn"))
            out = dev(tf, np.zeros((m, n), dtype))
            plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab(ma), lab(mb), lab("mn")), [a.shape, b.shape, [m, n]])
            tf.HipBackend.execute(plan, 1.0, [dev(tf, a), dev(tf, b)], 0.0, out)
            assert "gemm128_kernel" in tf.last_kernel(), tf.last_kernel()
            assert relerr(out.to_numpy(), ref) < TOL[dtype], (dtype, ma, mb)


@pytest.mark.parametrize("dtype", ALL)
def test_permute_extents_with_divisor_tiles(tf, oracle, dtype):
    # extents that are not powers of two but have useful divisors (15, 50, 60, 250): tiled without partial tiles
    rng = seeded_rng(49)
    for shape, perm in [((15, 15, 15, 15), (3, 1, 0, 2)), ((60, 50, 70), (2, 0, 1)), ((250, 130), (1, 0)), ((6, 250, 9, 20), (1, 3, 0, 2)),
                        ((33, 257), (1, 0)), ((12, 100, 35), (0, 2, 1))]:
        a = rand(rng, shape, dtype)
        got, ref = _permute_check(tf, oracle, a, perm)
        assert got.tobytes() == ref.tobytes(), (shape, perm)
    a = rand(rng, (60, 50, 70), dtype)
    b0 = rand(rng, (70, 60, 50), dtype)
    alpha, beta = (0.5 - 2j, 1.5 + 1j) if np.issubdtype(dtype, np.complexfloating) else (0.5, -1.5)
    got, ref = _permute_check(tf, oracle, a, (2, 0, 1), alpha, beta, b0)
    assert relerr(got, ref) < TOL[dtype]
    # a view whose rows start at odd element offsets: 16-byte accesses that are only element-aligned
    big = rand(rng, (64, 131), dtype)
    got, ref = _permute_check(tf, oracle, big[:, 1:129], (1, 0))
    assert got.tobytes() == ref.tobytes()
    # extents with a power-of-two divisor of at least 128 bytes (96 = 3 x 32, 160 = 5 x 32, 48 = 3 x 16): the tiles are
    # cut to that divisor, every tile is full and the launch stays on the kernel's fast path
    # (the last shape's divisor tiles would hold 256 elements only: it takes the table-driven tiles or the general path)
    for shape, perm, fast in [((96, 96, 96), (2, 1, 0), True), ((96, 256, 128), (1, 2, 0), True), ((160, 3, 160), (2, 1, 0), True),
                              ((192, 5, 320), (2, 0, 1), True), ((48, 48, 48, 16), (3, 1, 0, 2), False)]:
        a = rand(rng, shape, dtype)
        got, ref = _permute_check(tf, oracle, a, perm)
        assert got.tobytes() == ref.tobytes(), (shape, perm)
        if np.dtype(dtype).itemsize >= 8:
            if fast:
                assert copy_kernel_is_fast(tf.last_kernel()), (shape, perm, tf.last_kernel())
            else:
                assert "tabcopy_kernel" in tf.last_kernel() or "perm_kernel" in tf.last_kernel() or not copy_kernel_is_fast(tf.last_kernel()), (shape, perm, tf.last_kernel())


@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.complex128])
def test_permute_large_ragged_tensors_split_into_interior_and_border(tf, oracle, dtype):
    # more than 2^20 elements with extents just off the tile grid: whole tiles go through the fast path, the border
    # slabs are copied separately; every element must be written exactly once
    rng = seeded_rng(50)
    for shape, perm in [((1030, 1100), (1, 0)), ((101, 103, 107), (2, 0, 1)), ((65, 129, 131), (1, 2, 0)), ((3, 1025, 515), (2, 1, 0))]:
        a = rand(rng, shape, dtype)
        got, ref = _permute_check(tf, oracle, a, perm)
        assert got.tobytes() == ref.tobytes(), (shape, perm)
    a = rand(rng, (1030, 1100), dtype)
    b0 = rand(rng, (1100, 1030), dtype)
    alpha, beta = (0.5 - 2j, 1.5 + 1j) if np.issubdtype(dtype, np.complexfloating) else (0.5, -1.5)
    got, ref = _permute_check(tf, oracle, a, (1, 0), alpha, beta, b0)
    assert relerr(got, ref) < TOL[dtype]
    v = rand(rng, (1200, 1300), dtype)[7:1037, 3:1103]          # strided view in, strided view out is covered by dev()
    got, ref = _permute_check(tf, oracle, v, (1, 0))
    assert got.tobytes() == ref.tobytes()


def _random_contraction(rng, big):
    """Random binary contraction: labels split into batch / free-A / free-B / contracted groups, random extents,
    operands stored in a random axis order and seen through random strided (possibly reversed) views."""
    labels = list("abcdefgh")
    rng.shuffle(labels)
    nb, nm, nn, nk = rng.integers(0, 2), rng.integers(0, 3), rng.integers(0, 3), rng.integers(0, 3)
    groups, pos = [], 0
    for cnt in (nb, nm, nn, nk):
        groups.append(labels[pos:pos + cnt])
        pos += cnt
    batch, fm, fn, kk = groups
    top = 150 if big else 12
    ext = {l: int(rng.integers(1, top + 1)) for l in labels[:pos]}
    if big:   # keep the work bounded: at most two large extents per group product
        for grp in (batch, fm, fn, kk):
            for l in grp[1:]:
                ext[l] = int(rng.integers(1, 7))
        for l in batch:
            ext[l] = int(rng.integers(1, 4))
    ma = batch + fm + kk
    mb = batch + kk + fn
    mc = batch + fm + fn
    rng.shuffle(ma); rng.shuffle(mb); rng.shuffle(mc)
    return "".join(ma), "".join(mb), "".join(mc), ext


def _random_view(rng, shape, dtype):
    """A tensor of the given shape seen through a random view of a larger buffer (steps 1, 2 or -1, offsets)."""
    steps = [int(rng.choice([1, 1, 1, 2, -1])) for _ in shape]
    pads = [int(rng.integers(0, 3)) for _ in shape]
    big_shape = [n * abs(st) + p for n, st, p in zip(shape, steps, pads)]
    big = rand(rng, big_shape, dtype)
    idx = []
    for n, st, p in zip(shape, steps, pads):
        lo = int(rng.integers(0, p + 1))
        if st > 0:
            idx.append(slice(lo, lo + n * st, st))
        else:
            idx.append(slice(lo + n - 1, lo - 1 if lo > 0 else None, -1))
    v = big[tuple(idx)]
    assert list(v.shape) == list(shape)
    return v


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("big", [False, True], ids=["small", "large"])
def test_contract_random_label_patterns_and_views(tf, oracle, dtype, big):
    rng = seeded_rng(51 + (7 if big else 0))
    for case in range(25 if big else 40):
        ma, mb, mc, ext = _random_contraction(rng, big)
        while not ma or not mb:   # rank-0 operands are not views of anything
            ma, mb, mc, ext = _random_contraction(rng, big)
        a = _random_view(rng, [ext[l] for l in ma], dtype)
        b = _random_view(rng, [ext[l] for l in mb], dtype)
        cshape = [ext[l] for l in mc]
        use_beta = bool(rng.integers(0, 2)) and len(cshape) > 0
        alpha, beta = (0.7 - 1.1j, (-0.3 + 0.2j) if use_beta else 0.0) if np.issubdtype(dtype, np.complexfloating) else (0.7, -0.3 if use_beta else 0.0)
        c0 = rand(rng, cshape, dtype) if use_beta else np.full(cshape, np.nan, dtype)
        ref = c0.copy()
        oracle.contract(a, lab(ma), b, lab(mb), ref, lab(mc), alpha=alpha, beta=beta)
        out = dev(tf, c0) if cshape else tf.Tensor.empty([], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab(ma), lab(mb), lab(mc)), [a.shape, b.shape, cshape])
        tf.HipBackend.execute(plan, alpha, [dev(tf, a), dev(tf, b)], beta, out)
        # the same contraction over absolute values, in f64: the scale of the rounding-error bound
        scale = np.abs(c0).astype(np.float64) if use_beta else np.zeros(cshape)
        oracle.contract(np.abs(a).astype(np.float64), lab(ma), np.abs(b).astype(np.float64), lab(mb), scale, lab(mc),
                        alpha=abs(alpha), beta=abs(beta) if use_beta else 0.0)
        k = int(np.prod([ext[l] for l in set(ma) & set(mb) - set(mc)], dtype=np.int64))
        assert contraction_within_tolerance(out.to_numpy(), ref, dtype, scale, k), (case, ma, mb, mc, ext, relerr(out.to_numpy(), ref))
        # once more through the same plan on fresh device buffers: where the plan kept the routed launch this is its
        # replay (operands exchanged, tables, split-K and all), and it must give the same bits
        out2 = dev(tf, c0) if cshape else tf.Tensor.empty([], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
        tf.HipBackend.execute(plan, alpha, [dev(tf, a), dev(tf, b)], beta, out2)
        assert out.to_numpy().tobytes() == out2.to_numpy().tobytes(), (case, ma, mb, mc, ext, plan.cache_stats())


def _cancelling():
    import os
    return np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "cancelling_f32.npz"))


def test_f32_cancelling_dot_product_regression(tf, oracle):
    # "dc,dc->" (d = 6, c = 5), alpha = 0.7, thirty f32 terms whose sum is 1/1428 of the sum of their magnitudes.  A
    # randomized run once reported 2.18e-5 between the device and the CPU restatement on it: the restatement adds f32
    # products in f32 inside a cache block and carries all of that error; a product with an empty free group runs as a
    # reduction that accumulates in f64 on the device, which returns the exact result rounded once.
    fx = _cancelling()
    a, b, alpha = fx["dot_a"], fx["dot_b"], float(fx["alpha"])
    exact, scale = float(fx["dot_exact"]), float(fx["dot_abs"])
    out = tf.Tensor.empty([], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float32)
    plan = tf.HipBackend.plan(np.float32, tf.PrimDescriptor.Contract(lab("dc"), lab("dc"), []), [a.shape, b.shape, []])
    tf.HipBackend.execute(plan, alpha, [dev(tf, a), dev(tf, b)], 0.0, out)
    got = float(out.to_numpy())
    assert "dot" in tf.last_kernel() or "reduce" in tf.last_kernel(), tf.last_kernel()
    assert abs(got - exact) <= 2.0 ** -23 * abs(exact)          # one rounding of the result and one of alpha
    ref = np.empty([], np.float32)
    oracle.contract(a, lab("dc"), b, lab("dc"), ref, [], alpha=alpha)
    assert abs(float(ref) - exact) > 1e-5 * abs(exact)          # the restatement is the side that misses 1e-5 here ...
    assert contraction_within_tolerance(got, ref, np.float32, scale, 30)   # ... and is inside the rounding bound


def test_f32_cancelling_sums_on_the_matrix_cores(tf, oracle):
    # the same thirty terms under two free axes ("fdc,dce->fe"): the f32 matrix-core kernel accumulates in f32, so on
    # these outputs it is held to the rounding bound, not to 1e-5 of the (cancelled) result
    fx = _cancelling()
    a, b, alpha = fx["mat_a"], fx["mat_b"], float(fx["alpha"])
    exact, scale = fx["mat_exact"], fx["mat_abs"]
    out = tf.Tensor.empty([2, 3], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float32)
    plan = tf.HipBackend.plan(np.float32, tf.PrimDescriptor.Contract(lab("fdc"), lab("dce"), lab("fe")), [a.shape, b.shape, [2, 3]])
    tf.HipBackend.execute(plan, alpha, [dev(tf, a), dev(tf, b)], 0.0, out)
    assert "gemm" in tf.last_kernel(), tf.last_kernel()
    got = out.to_numpy().astype(np.float64)
    assert np.linalg.norm(got - exact) <= (30 + 2) * 2.0 ** -24 * np.linalg.norm(scale)
    ref = np.empty([2, 3], np.float32)
    oracle.contract(a, lab("fdc"), b, lab("dce"), ref, lab("fe"), alpha=alpha)
    assert contraction_within_tolerance(out.to_numpy(), ref, np.float32, scale, 30)


@pytest.mark.parametrize("dtype", ALL)
def test_contract_random_layouts_on_the_128_tile_kernel(tf, oracle, dtype):
    # random shapes sized for the 128x128 kernel (both free products >= 700, k of a thousand or more: enough tiles and stages):
    # one or two modes per group, random axis orders, random strided / reversed / offset views, odd extents.  Most
    # cases are contiguous along some operand direction (16-byte loads with their tail handling), the stepped views are not.
    rng = seeded_rng(58)
    on128 = 0
    for case in range(14):
        labels = list("abcdefgh")
        rng.shuffle(labels)
        nb, nm, nn, nk = int(rng.integers(0, 2)), int(rng.integers(1, 3)), int(rng.integers(1, 3)), int(rng.integers(1, 3))
        batch, fm, fn, kk = labels[:nb], labels[nb:nb + nm], labels[nb + nm:nb + nm + nn], labels[nb + nm + nn:nb + nm + nn + nk]
        ext = {}
        for grp, lo, hi in ((fm, 700, 860), (fn, 700, 860), (kk, 1000, 1100)):
            ext[grp[0]] = int(rng.integers(lo, hi + 1))
            for l in grp[1:]:
                ext[l] = int(rng.integers(1, 4))
        for l in batch:
            ext[l] = int(rng.integers(1, 3))
        ma, mb, mc = batch + fm + kk, batch + kk + fn, batch + fm + fn
        rng.shuffle(ma); rng.shuffle(mb); rng.shuffle(mc)
        plain = case % 2 == 0            # every other case: dense operands (the vector paths); else random views
        mk = (lambda shape: rand(rng, shape, dtype)) if plain else (lambda shape: _random_view(rng, shape, dtype))
        a, b = mk([ext[l] for l in ma]), mk([ext[l] for l in mb])
        cshape = [ext[l] for l in mc]
        use_beta = bool(rng.integers(0, 2))
        alpha, beta = (0.7 - 1.1j, (-0.3 + 0.2j) if use_beta else 0.0) if np.issubdtype(dtype, np.complexfloating) else (0.7, -0.3 if use_beta else 0.0)
        c0 = rand(rng, cshape, dtype) if use_beta else np.full(cshape, np.nan, dtype)
        ref = c0.copy()
        oracle.contract(a, lab(ma), b, lab(mb), ref, lab(mc), alpha=alpha, beta=beta)
        out = dev(tf, c0)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab(ma), lab(mb), lab(mc)), [a.shape, b.shape, cshape])
        print("case", case, "".join(ma), "".join(mb), "".join(mc), ext, "plain" if plain else "views", flush=True)
        tf.HipBackend.execute(plan, alpha, [dev(tf, a), dev(tf, b)], beta, out)
        on128 += "gemm128_kernel" in tf.last_kernel()
        err = relerr(out.to_numpy(), ref)
        assert err < TOL[dtype], (case, ma, mb, mc, ext, err)
    assert on128 >= 12, on128


@pytest.mark.parametrize("dtype", ALL)
def test_permute_and_reduce_random_shapes_and_views(tf, oracle, dtype):
    rng = seeded_rng(52)
    for case in range(30):
        rank = int(rng.integers(1, 6))
        shape = [int(rng.integers(1, 24)) for _ in range(rank)]
        if case % 5 == 0:
            shape[int(rng.integers(0, rank))] = int(rng.integers(100, 400))
        a = _random_view(rng, shape, dtype)
        modes = list(range(rank))
        perm = [int(p) for p in rng.permutation(rank)]
        ref = np.empty([shape[p] for p in perm], dtype)
        oracle.permute(a, modes, ref, perm)
        out = tf.Tensor.empty([shape[p] for p in perm], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Permute(modes, perm), [shape, [shape[p] for p in perm]])
        tf.HipBackend.execute(plan, 1.0, [dev(tf, a)], 0.0, out)
        assert out.to_numpy().tobytes() == ref.tobytes(), (case, shape, perm)
        keep = [m for m in perm if rng.integers(0, 2)]
        kshape = [shape[m] for m in keep]
        rref = np.empty(kshape, dtype)
        oracle.reduce(a, modes, rref, keep)
        rout = tf.Tensor.empty(kshape, tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
        rplan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Reduce(modes, keep, tf.ReduceOp.Sum), [shape, kshape])
        tf.HipBackend.execute(rplan, 1.0, [dev(tf, a)], 0.0, rout)
        assert relerr(rout.to_numpy(), rref) < 20 * TOL[dtype], (case, shape, keep)


def test_calls_are_capturable_in_a_hip_graph_and_replay_correctly(tf, oracle):
    # After one eager pass on the capture stream (which sizes the per-stream workspace and the intermediate pool), the
    # calls allocate nothing and synchronise nothing: a contraction with operand packing, offset tables and split-K, a
    # permute, a reduction and a three-operand einsum are captured into one graph and replayed on new input contents,
    # with eager work and synchronisation between the replays; every replay must equal the eager result.
    import torch
    rng = seeded_rng(53)
    ext = dict(a=8, j=32, b=16, k=48, c=64)
    A = rand(rng, [ext[l] for l in "ajbk"], np.float64)
    B = rand(rng, [ext[l] for l in "kcj"], np.float64)
    X = rand(rng, (16, 12, 20, 8), np.float64)
    E1, E2, E3 = rand(rng, (24, 30), np.complex128), rand(rng, (30, 18), np.complex128), rand(rng, (18, 40), np.complex128)
    tA, tB, tX = (torch.from_numpy(x).cuda() for x in (A, B, X))
    tE = [torch.from_numpy(x).cuda() for x in (E1, E2, E3)]
    dA, dB, dX = tf.Tensor.from_torch(tA), tf.Tensor.from_torch(tB), tf.Tensor.from_torch(tX)
    dE = [tf.Tensor.from_torch(t) for t in tE]
    gpu0 = tf.GpuMemory(0)
    oC = tf.Tensor.empty([8, 16, 64], gpu0, tf.MemoryOrder.RowMajor, np.float64)
    oP = tf.Tensor.empty([8, 16, 20, 12], gpu0, tf.MemoryOrder.RowMajor, np.float64)
    oR = tf.Tensor.empty([12, 8], gpu0, tf.MemoryOrder.RowMajor, np.float64)
    oE = tf.Tensor.empty([24, 40], gpu0, tf.MemoryOrder.RowMajor, np.complex128)
    pc = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Contract(lab("ajbk"), lab("kcj"), lab("abc")), [A.shape, B.shape, [8, 16, 64]])
    pp = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Permute([0, 1, 2, 3], [3, 0, 2, 1]), [X.shape, [8, 16, 20, 12]])
    pr = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Reduce([0, 1, 2, 3], [1, 3], tf.ReduceOp.Sum), [X.shape, [12, 8]])
    subs = tf.Subscripts.parse("ij,jk,kl->il")
    tree = tf.ContractionTree.optimize(subs, [E1.shape, E2.shape, E3.shape])

    def work():
        tf.HipBackend.execute(pc, 1.0, [dA, dB], 0.0, oC)
        tf.HipBackend.execute(pp, 1.0, [dX], 0.0, oP)
        tf.HipBackend.execute(pr, 1.0, [dX], 0.0, oR)
        tf.einsum_with_plan_into(tree, dE, 1.0, 0.0, oE)

    def expected():
        c = np.empty((8, 16, 64)); oracle.contract(tA.cpu().numpy(), lab("ajbk"), tB.cpu().numpy(), lab("kcj"), c, lab("abc"))
        x = tX.cpu().numpy()
        p = np.empty((8, 16, 20, 12)); oracle.permute(x, [0, 1, 2, 3], p, [3, 0, 2, 1])
        r = np.empty((12, 8)); oracle.reduce(x, [0, 1, 2, 3], r, [1, 3])
        e = np.empty((24, 40), np.complex128)
        oracle.einsum_pairs([t.cpu().numpy() for t in tE], [lab("ij"), lab("jk"), lab("kl")], e, lab("il"), tree.steps)
        return c, p, r, e

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        work()                                    # eager pass on the capture stream
    side.synchronize()
    for t in (oC, oP, oR, oE):
        t.event = None                            # completed; an event recorded outside the capture must not be waited on inside it
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        work()
    for replay in range(3):
        for t in [tA, tB, tX] + tE:               # new contents, same buffers
            t.mul_(-0.5).add_(0.25 * (replay + 1))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        c, p, r, e = expected()
        assert relerr(oC.to_numpy(), c) < 1e-12, replay
        assert oP.to_numpy().tobytes() == p.tobytes(), replay
        assert relerr(oR.to_numpy(), r) < 1e-12, replay
        assert relerr(oE.to_numpy(), e) < 1e-12, replay


def test_graph_replays_after_the_workspace_grew_and_the_caches_were_released(tf, oracle):
    # A captured graph holds the addresses of the workspace, the offset tables and the intermediates its calls were
    # given.  Later eager work on the same stream that needs a larger workspace, and tfh_release_workspaces, must leave
    # those buffers alone (they are retired or passed over, never freed): the graph is replayed afterwards on new
    # contents and must still give the eager result.
    import torch
    rng = seeded_rng(55)
    A = rand(rng, (8, 32, 16, 48), np.float64)        # "ajbk,kcj->abc": packing, offset tables, split-K partials
    B = rand(rng, (48, 64, 32), np.float64)
    E1, E2, E3 = rand(rng, (40, 50), np.float64), rand(rng, (50, 30), np.float64), rand(rng, (30, 20), np.float64)
    tA, tB = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    tE = [torch.from_numpy(x).cuda() for x in (E1, E2, E3)]
    dA, dB = tf.Tensor.from_torch(tA), tf.Tensor.from_torch(tB)
    dE = [tf.Tensor.from_torch(t) for t in tE]
    gpu0 = tf.GpuMemory(0)
    oC = tf.Tensor.empty([8, 16, 64], gpu0, tf.MemoryOrder.RowMajor, np.float64)
    oE = tf.Tensor.empty([40, 20], gpu0, tf.MemoryOrder.RowMajor, np.float64)
    pc = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Contract(lab("ajbk"), lab("kcj"), lab("abc")), [A.shape, B.shape, [8, 16, 64]])
    tree = tf.ContractionTree.optimize(tf.Subscripts.parse("ij,jk,kl->il"), [E1.shape, E2.shape, E3.shape])

    def work():
        tf.HipBackend.execute(pc, 1.0, [dA, dB], 0.0, oC)
        tf.einsum_with_plan_into(tree, dE, 1.0, 0.0, oE)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        work()
    side.synchronize()
    oC.event = oE.event = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        work()
    # eager work on the capture stream that needs a much larger workspace (a long k over few tiles: split-K partials)
    big_a = tf.Tensor.from_torch(torch.randn(256, 1 << 15, dtype=torch.float64, device="cuda"))
    big_b = tf.Tensor.from_torch(torch.randn(1 << 15, 256, dtype=torch.float64, device="cuda"))
    big_c = tf.Tensor.empty([256, 256], gpu0, tf.MemoryOrder.RowMajor, np.float64)
    pbig = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Contract(lab("mk"), lab("kn"), lab("mn")), [[256, 1 << 15], [1 << 15, 256], [256, 256]])
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        tf.HipBackend.execute(pbig, 1.0, [big_a, big_b], 0.0, big_c)
    side.synchronize()
    assert tf.lib().tfh_release_workspaces() == 0
    # fresh allocations that would land in freed memory if anything of the graph's had been freed
    filler = [torch.full((1 << 20,), float("nan"), dtype=torch.float64, device="cuda") for _ in range(8)]
    for replay in range(2):
        for t in [tA, tB] + tE:
            t.mul_(-0.5).add_(0.25 * (replay + 1))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        c = np.empty((8, 16, 64))
        oracle.contract(tA.cpu().numpy(), lab("ajbk"), tB.cpu().numpy(), lab("kcj"), c, lab("abc"))
        e = tE[0].cpu().numpy() @ tE[1].cpu().numpy() @ tE[2].cpu().numpy()
        assert relerr(oC.to_numpy(), c) < 1e-12, replay
        assert relerr(oE.to_numpy(), e) < 1e-12, replay
    del filler


def test_owned_variant_keeps_intermediates_in_donated_operand_buffers(tf, oracle):
    # einsum_with_plan_owned (tenferro-einsum/src/lib.rs:493-498): the operands are consumed, so an intermediate that fits
    # may live in the buffer of an operand whose step is already enqueued.  The result is unchanged; a donated buffer
    # ends up overwritten; the borrowing variant leaves its operands intact; a buffer that another tensor shares, or
    # that the caller wrapped from their own torch tensor, is never written.
    import torch
    rng = seeded_rng(54)
    host = [rand(rng, (64, 64), np.float64) for _ in range(4)]
    subs = tf.Subscripts.parse("ij,jk,kl,lm->im")
    tree = tf.ContractionTree.from_pairs(subs, [h.shape for h in host], [(0, 1), (4, 2), (5, 3)])
    ref = np.empty((64, 64))
    oracle.einsum_pairs(host, [lab(t) for t in ("ij", "jk", "kl", "lm")], ref, lab("im"), tree.steps)

    def upload():
        return [tf.Tensor.from_slice(h, h.shape, tf.MemoryOrder.RowMajor).to_memory_space_async(tf.GpuMemory(0)) for h in host]

    ops = upload()
    out = tf.einsum_with_plan(tree, ops)
    assert relerr(out.to_numpy(), ref) < 1e-12
    assert all(np.array_equal(o.to_numpy(), h) for o, h in zip(ops, host))               # borrowed: untouched

    # the test's own window onto the memory: the raw device addresses (the blocks stay mapped in torch's caching
    # allocator after the tensors are dropped)
    addrs = [o._buf.data_ptr() for o in ops]
    assert all(o._sole_owner() for o in ops)
    out2 = tf.einsum_with_plan_owned(tree, ops)
    assert ops == []                                                                     # consumed
    assert relerr(out2.to_numpy(), ref) < 1e-12
    torch.cuda.synchronize()
    after = [np.empty_like(h) for h in host]
    for a, dst in zip(addrs, after):
        assert tf.lib().tfh_memcpy_d2h(dst.ctypes.data, a, dst.nbytes, None) == 0
    torch.cuda.synchronize()
    assert any(not np.array_equal(a, h) for a, h in zip(after, host))                    # one holds an intermediate

    # shared buffers: a permuted view of operand 0 is alive, so operand 0 is not donated; the others still are
    ops = upload()
    keep = ops[0].permute([1, 0])
    assert not ops[0]._sole_owner() and ops[1]._sole_owner()
    out3 = tf.einsum_with_plan_owned(tree, ops)
    assert relerr(out3.to_numpy(), ref) < 1e-12
    assert np.array_equal(keep.to_numpy(), host[0].T)

    # caller-owned torch memory is never donated
    bufs = [torch.from_numpy(h).cuda() for h in host]
    out4 = tf.einsum_with_plan_owned(tree, [tf.Tensor.from_torch(b) for b in bufs])
    assert relerr(out4.to_numpy(), ref) < 1e-12
    assert all(np.array_equal(b.cpu().numpy(), h) for b, h in zip(bufs, host))

    # the raw C entry point with every bit set and one buffer given as all four operands: overlap is detected
    sq = torch.from_numpy(host[0]).cuda()
    same = [tf.Tensor.from_torch(sq)] * 4
    ref4 = host[0] @ host[0] @ host[0] @ host[0]
    out5 = tf.einsum_with_plan(tree, same, None, 0xF)
    assert relerr(out5.to_numpy(), ref4) < 1e-12
    assert np.array_equal(sq.cpu().numpy(), host[0])


def test_offset_tables_are_kept_per_layout_and_survive_a_release(tf, oracle):
    # The offset tables of a multi-mode contraction are built once per (dims, strides) and stream and reused by later
    # calls.  Two layouts of the same shapes alternate through one plan: each call must use its own layout's tables;
    # releasing the library's scratch memory in between drops them and the next call builds them again.
    rng = seeded_rng(77)
    sa, sb, sc = (16, 40, 8, 24), (24, 130, 40), (16, 8, 130)                  # "ajbk,kcj->abc": 128x128 tiles
    a1, b1 = rand(rng, sa, np.float64), rand(rng, sb, np.float64)
    a2 = np.ascontiguousarray(rand(rng, (24, 8, 40, 16), np.float64)).transpose(3, 2, 1, 0)      # same dims, reversed strides
    b2 = np.ascontiguousarray(rand(rng, (40, 130, 24), np.float64)).transpose(2, 1, 0)
    plan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Contract(lab("ajbk"), lab("kcj"), lab("abc")), [sa, sb, sc])
    pairs = [(a1, b1), (a2, b2), (a1, b2), (a2, b1)]
    refs = []
    for a, b in pairs:
        r = np.empty(sc)
        oracle.contract(a, lab("ajbk"), b, lab("kcj"), r, lab("abc"))
        refs.append(r)
    devs = [(dev(tf, a), dev(tf, b)) for a, b in pairs]
    out = tf.Tensor.empty(list(sc), tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64)
    for rnd in range(3):
        for (da, db), r in zip(devs, refs):
            tf.HipBackend.execute(plan, 1.0, [da, db], 0.0, out)
            assert relerr(out.to_numpy(), r) < 1e-12
        if rnd == 1:
            assert tf.lib().tfh_release_workspaces() == 0


def whole_chunks(dtype, n):
    # n elements fill a whole number of 16-byte chunks
    return (n * np.dtype(dtype).itemsize) % 16 == 0


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("m,k,x,c", [(32, 32, 8, 1024), (20, 13, 64, 80), (16, 32, 1, 4096), (7, 6, 16, 512), (32, 2, 32, 160),
                                     (32, 32, 16, 500), (16, 8, 64, 100), (20, 16, 100, 50), (5, 4, 5, 1000), (8, 6, 300, 17)])
def test_contract_small_operator_applied_to_a_long_tensor(tf, oracle, dtype, m, k, x, c):
    # T[x, c, k] . W[k, m] -> out[x, m, c]: few rows, little k, a long n = (x, c) whose fastest output axis is c -- the
    # shape of an operator applied to every fibre of a large tensor, which takes the streaming kernel.  Odd m and k,
    # general alpha/beta, and a W that is a strided view are covered; a row of k must fill whole 16-byte chunks for that
    # kernel (any k for complex128, even k for f64 and complex64, k a multiple of 4 for f32), otherwise the tiled ones
    # take the product (k = 13).  The kernel works on units of 16 consecutive c: extents that are no
    # multiple of 16 (500, 100, 50, 1000: bond dimensions are rarely powers of two) end each run on a partly filled unit;
    # a run shorter than three units (17) is left to the tiled kernels.
    rng = seeded_rng(91)
    t = rand(rng, (x, c, k), dtype)
    w = rand(rng, (k, 2 * m), dtype)[:, ::2]
    ref = rand(rng, (x, m, c), dtype)
    out0 = ref.copy()
    cplx = np.iscomplexobj(t)
    for alpha, beta in [(1.0, 0.0), ((0.5 - 2j, 1.5 + 1j) if cplx else (0.5, -1.5))]:
        ref = out0.copy()
        oracle.contract(t, lab("xck"), w, lab("km"), ref, lab("xmc"), alpha=alpha, beta=beta)
        dout = dev(tf, out0)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("xck"), lab("km"), lab("xmc")), [t.shape, w.shape, ref.shape])
        tf.HipBackend.execute(plan, alpha, [dev(tf, t), dev(tf, w)], beta, dout)
        streamed = whole_chunks(dtype, k) and (c % 16 == 0 or c >= 48)
        assert ("gemm_skinny_kernel" in tf.last_kernel()) == streamed, tf.last_kernel()
        assert relerr(dout.to_numpy(), ref) < TOL[dtype], (alpha, beta)


def test_contract_small_operator_exact_on_integer_inputs(tf):
    # small integers: every product and sum is exact, so the streaming kernel must agree with numpy to the bit, and a
    # wrong sign in the complex expansion or a misplaced k would show
    rng = seeded_rng(92)
    t = (rng.integers(-4, 5, (4, 1024, 32)) + 1j * rng.integers(-4, 5, (4, 1024, 32))).astype(np.complex128)
    w = (rng.integers(-4, 5, (32, 32)) + 1j * rng.integers(-4, 5, (32, 32))).astype(np.complex128)
    out = tf.Tensor.empty([4, 32, 1024], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.complex128)
    plan = tf.HipBackend.plan(np.complex128, tf.PrimDescriptor.Contract(lab("xck"), lab("km"), lab("xmc")), [t.shape, w.shape, [4, 32, 1024]])
    tf.HipBackend.execute(plan, 1.0, [dev(tf, t), dev(tf, w)], 0.0, out)
    assert "gemm_skinny_kernel" in tf.last_kernel()
    assert np.array_equal(out.to_numpy(), np.einsum("xck,km->xmc", t, w))


@pytest.mark.parametrize("dtype", ALL)
def test_contract_small_operator_strided_rows_and_split_k_order(tf, oracle, dtype):
    # the streaming kernel's addressing: rows of the long operand reversed along c and padded (a view of a larger buffer),
    # its k split over two modes that the small operand holds in the opposite order (its k goes through the offset table),
    # the small operand's rows split over two modes of the output
    rng = seeded_rng(93)
    x, c, s_, w_, t_, v_ = 16, 320, 2, 8, 2, 7
    t1 = rand(rng, (x, c, s_, w_), dtype)[:, ::-1]                                        # contiguous k per row, rows reversed
    wop = rand(rng, (w_, s_, t_, v_), dtype)
    ref = np.empty((x, v_, t_, c), dtype)
    oracle.contract(t1, lab("xcsw"), wop, lab("wstv"), ref, lab("xvtc"))
    out = tf.Tensor.empty([x, v_, t_, c], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
    plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("xcsw"), lab("wstv"), lab("xvtc")), [t1.shape, wop.shape, ref.shape])
    tf.HipBackend.execute(plan, 1.0, [dev(tf, t1), dev(tf, wop)], 0.0, out)
    assert "gemm_skinny_kernel" in tf.last_kernel()
    assert relerr(out.to_numpy(), ref) < TOL[dtype]
    # padded rows: each (x, c) row is the first 16 elements of a 24-element row of a larger buffer
    bigk = rand(rng, (x, c, 24), dtype)
    t2 = bigk[:, :, :16]
    w2 = rand(rng, (16, 20), dtype)
    ref2 = np.empty((x, 20, c), dtype)
    oracle.contract(t2, lab("xck"), w2, lab("km"), ref2, lab("xmc"))
    out2 = tf.Tensor.empty([x, 20, c], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
    plan2 = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("xck"), lab("km"), lab("xmc")), [t2.shape, w2.shape, ref2.shape])
    tf.HipBackend.execute(plan2, 1.0, [dev(tf, t2), dev(tf, w2)], 0.0, out2)
    assert "gemm_skinny_kernel" in tf.last_kernel()
    assert relerr(out2.to_numpy(), ref2) < TOL[dtype]


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("m,k,x,c", [(32, 32, 8, 1024), (20, 13, 64, 80), (16, 32, 1, 4096), (7, 6, 16, 512), (32, 2, 32, 160), (2, 64, 4, 2048),
                                     (32, 32, 9, 500), (16, 8, 7, 700), (4, 4, 1, 4099)])
def test_contract_small_operator_with_the_result_contiguous_along_its_columns(tf, oracle, dtype, m, k, x, c):
    # the other orientation of the same product: T[x, c, k] . W[k, m] -> out[x, c, m], the few columns m adjacent in the
    # output.  The streaming kernel then transposes each unit's results through LDS.  Rows of k and of m must fill
    # whole 16-byte chunks for it.
    # (x, c) is one run of x * c here: 9 * 500, 7 * 700 and 4099 leave a partly filled last unit.
    cplx = np.issubdtype(dtype, np.complexfloating)
    if k > 32 and cplx:
        k = 32
    rng = seeded_rng(94)
    t = rand(rng, (x, c, k), dtype)
    w = rand(rng, (k, m), dtype)
    out0 = rand(rng, (x, c, m), dtype)
    for alpha, beta in [(1.0, 0.0), ((0.5 - 2j, 1.5 + 1j) if cplx else (0.5, -1.5))]:
        ref = out0.copy()
        oracle.contract(t, lab("xck"), w, lab("km"), ref, lab("xcm"), alpha=alpha, beta=beta)
        dout = dev(tf, out0)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("xck"), lab("km"), lab("xcm")), [t.shape, w.shape, ref.shape])
        tf.HipBackend.execute(plan, alpha, [dev(tf, t), dev(tf, w)], beta, dout)
        streamed = whole_chunks(dtype, k) and whole_chunks(dtype, m)
        assert ("gemm_skinny_kernel" in tf.last_kernel()) == streamed, tf.last_kernel()
        assert relerr(dout.to_numpy(), ref) < TOL[dtype], (alpha, beta)
    # the same with the output rows padded (a view of a wider buffer) and the long operand's rows reversed
    wide = rand(rng, (x, c, m + 2), dtype)
    view = wide[:, :, :m]
    ref = view.copy()
    tr = t[:, ::-1]
    oracle.contract(tr, lab("xck"), w, lab("km"), ref, lab("xcm"), alpha=1.0, beta=0.0)
    dwide = dev(tf, wide)
    dview = tf.Tensor(dwide._buf, [x, c, m], dwide.strides(), 0, tf.GpuMemory(0), tf.dtype_code(dtype))
    tf.HipBackend.execute(plan, 1.0, [dev(tf, tr), dev(tf, w)], 0.0, dview)
    got = dwide.to_numpy()
    assert relerr(got[:, :, :m], ref) < TOL[dtype]
    assert np.array_equal(got[:, :, m:], wide[:, :, m:])          # the padding is untouched


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("out_modes", ["xmc", "xcm"])
@pytest.mark.parametrize("m,k,c", [(32, 32, 24000), (20, 12, 24008), (12, 10, 30001), (8, 6, 30001), (4, 8, 160000)])
def test_contract_small_operator_every_wave_streams_several_units(tf, oracle, dtype, out_modes, m, k, c):
    # The streaming kernel launches at most 2048 waves; with more units than that (3 x 1500 and more here) a wave works
    # through several, loads the next unit while it multiplies and stores a unit's results during the MFMAs of the
    # following one (the last unit's after the loop).  Both output orientations, whole and partly filled last units,
    # general alpha / beta.
    cplx = np.issubdtype(dtype, np.complexfloating)
    if not cplx:
        k *= 2
    if np.dtype(dtype).itemsize <= 8 and dtype != np.float64:
        k *= 2          # whole chunks of four f32 / two complex64
    if dtype == np.float32 and out_modes == "xcm":
        m = (m + 3) // 4 * 4
    rng = seeded_rng(95)
    x = 3
    t = rand(rng, (x, c, k), dtype)
    w = rand(rng, (k, m), dtype)
    out0 = rand(rng, (x, m, c) if out_modes == "xmc" else (x, c, m), dtype)
    for alpha, beta in [(1.0, 0.0), ((0.5 - 2j, 1.5 + 1j) if cplx else (0.5, -1.5))]:
        ref = out0.copy()
        oracle.contract(t, lab("xck"), w, lab("km"), ref, lab(out_modes), alpha=alpha, beta=beta)
        dout = dev(tf, out0)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("xck"), lab("km"), lab(out_modes)), [t.shape, w.shape, ref.shape])
        tf.HipBackend.execute(plan, alpha, [dev(tf, t), dev(tf, w)], beta, dout)
        assert "gemm_skinny_kernel" in tf.last_kernel(), tf.last_kernel()
        assert relerr(dout.to_numpy(), ref) < TOL[dtype], (alpha, beta)


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("out_modes", ["xmc", "xcm"])
@pytest.mark.parametrize("m,k,c", [(8, 8, 4096), (4, 4, 4096), (2, 2, 4096), (8, 4, 4096), (3, 6, 4096), (4, 2, 4096), (8, 8, 17)])
def test_contract_tiny_operator_on_the_last_leg_of_a_long_tensor(tf, oracle, dtype, out_modes, m, k, c):
    # a gate on the last leg: T[x, c, k] . W[k, m], at most 8 x 8, the rows of T contiguous runs of k.  Two kernels can
    # take it: the tiny-operator kernel (lanes a whole row apart) and the streaming kernel (whole rows per lane group);
    # which one is faster depends on the extents and on the output's orientation, and a product the streaming kernel
    # is preferred for but cannot take (runs of 17 columns) still goes to the tiny-operator kernel.
    cplx = np.issubdtype(dtype, np.complexfloating)
    rows = out_modes == "xcm"
    rng = seeded_rng(96)
    x = 32 if c > 100 else 4096
    t = rand(rng, (x, c, k), dtype)
    w = rand(rng, (k, m), dtype)
    out0 = rand(rng, (x, c, m) if rows else (x, m, c), dtype)
    if dtype == np.complex128:
        prefer = (m >= 3 or k >= 4) if rows else k >= 4
    elif dtype == np.float32:
        prefer = (m >= 4 or k >= 8) if rows else k >= 8
    else:
        prefer = (m >= 4 or k >= 6) if rows else k >= 6
    prefer = prefer and k >= 2 and whole_chunks(dtype, k)
    can = (whole_chunks(dtype, m) or not rows) and (rows or c >= 48)
    for alpha, beta in [(1.0, 0.0), ((0.5 - 2j, 1.5 + 1j) if cplx else (0.5, -1.5))]:
        ref = out0.copy()
        oracle.contract(t, lab("xck"), w, lab("km"), ref, lab(out_modes), alpha=alpha, beta=beta)
        dout = dev(tf, out0)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("xck"), lab("km"), lab(out_modes)), [t.shape, w.shape, ref.shape])
        tf.HipBackend.execute(plan, alpha, [dev(tf, t), dev(tf, w)], beta, dout)
        want = "gemm_skinny_kernel" if prefer and can else "tiny_operator_kernel"
        assert want in tf.last_kernel(), (tf.last_kernel(), want)
        assert relerr(dout.to_numpy(), ref) < TOL[dtype], (alpha, beta)


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("a_,k,m,c", [(64, 16, 16, 1024), (33, 12, 8, 2000), (3, 20, 12, 30001), (100, 32, 20, 777), (9, 32, 32, 4000),
                                      (6, 3, 5, 48 * 16), (5, 10, 9, 30002)])
def test_contract_small_operator_on_a_middle_leg(tf, oracle, dtype, a_, k, m, c):
    # T[a, k, c] . W[m, k] -> out[a, m, c]: the operator acts on a leg that is not the last, so the long operand is
    # contiguous along n = c like the output, and its k is strided.  The streaming kernel parks such a unit as [k][16 c];
    # its 16-byte loads run along c, so the runs of c must hold whole chunks (any c for complex128, even c for f64 and
    # complex64, multiples of 4 for f32), otherwise the tiled kernels take the product.  Whole and partly filled last
    # units, several units per wave (30001, 30002), general alpha / beta; then k split over two modes that the operator
    # holds in the other order, and a view of every second a with a conjugated operator.
    cplx = np.issubdtype(dtype, np.complexfloating)
    streamed = whole_chunks(dtype, c)
    rng = seeded_rng(97)
    t = rand(rng, (a_, k, c), dtype)
    w = rand(rng, (m, k), dtype)
    out0 = rand(rng, (a_, m, c), dtype)
    for alpha, beta in [(1.0, 0.0), ((0.5 - 2j, 1.5 + 1j) if cplx else (0.5, -1.5))]:
        ref = out0.copy()
        oracle.contract(t, lab("akc"), w, lab("mk"), ref, lab("amc"), alpha=alpha, beta=beta)
        dout = dev(tf, out0)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("akc"), lab("mk"), lab("amc")), [t.shape, w.shape, ref.shape])
        tf.HipBackend.execute(plan, alpha, [dev(tf, t), dev(tf, w)], beta, dout)
        assert ("gemm_skinny_kernel" in tf.last_kernel() and ", true>" in tf.last_kernel()) == streamed, tf.last_kernel()
        assert relerr(dout.to_numpy(), ref) < TOL[dtype], (alpha, beta)
    if k % 4 == 0:
        s_, w_ = 4, k // 4
        t4 = rand(rng, (a_, s_, w_, c), dtype)
        wop = rand(rng, (w_, m, s_), dtype)
        ref = np.empty((a_, m, c), dtype)
        oracle.contract(t4, lab("aswc"), wop, lab("wms"), ref, lab("amc"))
        out = tf.Tensor.empty([a_, m, c], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("aswc"), lab("wms"), lab("amc")), [t4.shape, wop.shape, ref.shape])
        tf.HipBackend.execute(plan, 1.0, [dev(tf, t4), dev(tf, wop)], 0.0, out)
        assert ("gemm_skinny_kernel" in tf.last_kernel()) == streamed, tf.last_kernel()
        assert relerr(out.to_numpy(), ref) < TOL[dtype]
    # a view of every second a and a conjugated operator
    tv = t[::2]
    ref = np.empty((tv.shape[0], m, c), dtype)
    oracle.contract(tv, lab("akc"), np.conj(w), lab("mk"), ref, lab("amc"))
    out = tf.Tensor.empty(list(ref.shape), tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
    plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("akc"), lab("mk"), lab("amc")), [tv.shape, w.shape, ref.shape])
    tf.HipBackend.execute(plan, 1.0, [dev(tf, tv), dev(tf, w).conj_on_load()], 0.0, out)
    assert relerr(out.to_numpy(), ref) < TOL[dtype]


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("a_,k,m,c", [(64, 8, 8, 1024), (300, 2, 8, 256), (33, 3, 4, 2048), (5, 8, 6, 25600), (70, 4, 3, 1024), (66, 8, 8, 1000)])
def test_contract_tiny_operator_with_the_acted_leg_moved_last(tf, oracle, dtype, a_, k, m, c):
    # T[a, k, c] . W[m, k] -> out[a, c, m]: a gate on a middle leg whose result carries that leg last.  A thread of the
    # tiny-operator kernel then holds m adjacent output elements and its neighbours are m elements away; where the rows
    # of m are packed, fill whole 16-byte pieces and the innermost long axis holds whole blocks of 256, the block's
    # results leave through an LDS tile in address order (the kernel's last template argument); elsewhere the direct
    # stores remain (c = 1000; three f64 per row) or another kernel takes the product.
    cplx = np.issubdtype(dtype, np.complexfloating)
    rng = seeded_rng(98)
    t = rand(rng, (a_, k, c), dtype)
    w = rand(rng, (m, k), dtype)
    out0 = rand(rng, (a_, c, m), dtype)
    tiled = m >= 3 and c % 256 == 0 and whole_chunks(dtype, m)
    for alpha, beta in [(1.0, 0.0), ((0.5 - 2j, 1.5 + 1j) if cplx else (0.5, -1.5))]:
        ref = out0.copy()
        oracle.contract(t, lab("akc"), w, lab("mk"), ref, lab("acm"), alpha=alpha, beta=beta)
        dout = dev(tf, out0)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("akc"), lab("mk"), lab("acm")), [t.shape, w.shape, ref.shape])
        tf.HipBackend.execute(plan, alpha, [dev(tf, t), dev(tf, w)], beta, dout)
        if "tiny_operator_kernel" in tf.last_kernel():
            assert tf.last_kernel().rstrip(")").endswith(", true>") == tiled, tf.last_kernel()
        else:
            assert not tiled, tf.last_kernel()
        assert relerr(dout.to_numpy(), ref) < TOL[dtype], (alpha, beta)


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("a_,k,m,c", [(64, 16, 16, 1024), (30, 12, 32, 2000), (3, 20, 12, 30001), (100, 32, 20, 776), (9, 32, 32, 4000),
                                      (5, 10, 9, 30002), (64, 8, 8, 1000)])
def test_contract_small_operator_on_a_middle_leg_with_that_leg_moved_last(tf, oracle, dtype, a_, k, m, c):
    # T[a, k, c] . W[m, k] -> out[a, c, m]: the long operand contiguous along c, the result along the operator's rows.
    # The streaming kernel parks [k][16 c] and writes through its transposing tile; runs of c and rows of m must hold
    # whole 16-byte chunks (any for complex128).
    cplx = np.issubdtype(dtype, np.complexfloating)
    streamed = whole_chunks(dtype, c) and whole_chunks(dtype, m)
    rng = seeded_rng(99)
    t = rand(rng, (a_, k, c), dtype)
    w = rand(rng, (m, k), dtype)
    out0 = rand(rng, (a_, c, m), dtype)
    for alpha, beta in [(1.0, 0.0), ((0.5 - 2j, 1.5 + 1j) if cplx else (0.5, -1.5))]:
        ref = out0.copy()
        oracle.contract(t, lab("akc"), w, lab("mk"), ref, lab("acm"), alpha=alpha, beta=beta)
        dout = dev(tf, out0)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("akc"), lab("mk"), lab("acm")), [t.shape, w.shape, ref.shape])
        tf.HipBackend.execute(plan, alpha, [dev(tf, t), dev(tf, w)], beta, dout)
        assert ("gemm_skinny_kernel" in tf.last_kernel() and ", true>" in tf.last_kernel()) == streamed, tf.last_kernel()
        assert relerr(dout.to_numpy(), ref) < TOL[dtype], (alpha, beta)


@pytest.mark.parametrize("dtype", ALL)
def test_reduce_rows_and_inner_axes_take_the_butterfly_fold(tf, oracle, dtype):
    # sums over the contiguous axis (row sums) and over an inner axis next to a short kept one: nothing is left to loop
    # over, so a block handles eight outputs per lane group and folds them with the transposing butterfly.  Exact
    # integer inputs make a misrouted accumulator visible; max/min and alpha/beta go the same way.
    rng = seeded_rng(95)
    cplx = np.issubdtype(dtype, np.complexfloating)
    def ints(shape):
        x = rng.integers(-9, 10, shape).astype(np.float64)
        return (x + 1j * rng.integers(-9, 10, shape)).astype(dtype) if cplx else x.astype(dtype)
    cases = [((32768, 256), [0, 1], [0]),                      # row sums, 128 lanes per row
             ((16, 16, 16, 16, 16, 16), list(range(6)), [0, 1, 2, 3, 5]),   # inner axis of 16 next to a kept axis of 16
             ((65536, 64), [0, 1], [0]),                       # two rows per wave
             ((512, 8, 32, 16), [0, 1, 2, 3], [0, 1, 3])]
    for shape, ma, mc in cases:
        a = ints(shape)
        got, ref = _reduce_check(tf, oracle, a, ma, mc, tf.ReduceOp.Sum, oracle.SUM)
        if dtype == np.float64:      # (the other element sizes tile these shapes differently; they are checked for their results)
            assert ", 8, true, " in tf.last_kernel(), (shape, tf.last_kernel())
        assert np.array_equal(got, ref), shape
    a = rand(rng, (32768, 256), dtype)
    c0 = rand(rng, (32768,), dtype)
    got, ref = _reduce_check(tf, oracle, a, [0, 1], [0], tf.ReduceOp.Sum, oracle.SUM, alpha=2.0, beta=-0.5, c0=c0)
    assert relerr(got, ref) < TOL[dtype]
    if not cplx:
        for op_tf, op_or in [(tf.ReduceOp.Max, oracle.MAX), (tf.ReduceOp.Min, oracle.MIN)]:
            got, ref = _reduce_check(tf, oracle, a, [0, 1], [0], op_tf, op_or)
            assert dtype != np.float64 or ", 8, true, " in tf.last_kernel()
            assert np.array_equal(got, ref)


@pytest.mark.parametrize("dtype", ALL)
def test_reduce_few_outputs_split_over_blocks(tf, oracle, dtype):
    # few outputs and a long reduction: the serial range is split over blocks (raw partials) and a second launch folds
    # the partials in a fixed order.  Exact integer inputs: any lost or doubled chunk changes the sum.
    rng = seeded_rng(96)
    cplx = np.issubdtype(dtype, np.complexfloating)
    def ints(shape):
        x = rng.integers(-9, 10, shape).astype(np.float64)
        return (x + 1j * rng.integers(-9, 10, shape)).astype(dtype) if cplx else x.astype(dtype)
    cases = [((1 << 21,), [0], []),                                   # full sum, one output
             ((2048, 512), [0, 1], [1]),                              # column sums
             ((32, 64, 64, 32), [0, 1, 2, 3], [0, 3]),                # two middle axes
             ((3, 1 << 19), [0, 1], [0])]                             # three long rows
    for shape, ma, mc in cases:
        a = ints(shape)
        got, ref = _reduce_check(tf, oracle, a, ma, mc, tf.ReduceOp.Sum, oracle.SUM)
        assert "reduce_fast_kernel" in tf.last_kernel(), (shape, tf.last_kernel())
        assert np.array_equal(got, ref), shape
        got2, _ = _reduce_check(tf, oracle, a, ma, mc, tf.ReduceOp.Sum, oracle.SUM)
        assert np.array_equal(got, got2)                              # same bits on every run
    a = rand(rng, (2048, 512), dtype)
    c0 = rand(rng, (512,), dtype)
    got, ref = _reduce_check(tf, oracle, a, [0, 1], [1], tf.ReduceOp.Sum, oracle.SUM, alpha=2.0, beta=-0.5, c0=c0)
    assert relerr(got, ref) < TOL[dtype]
    if not cplx:
        for op_tf, op_or in [(tf.ReduceOp.Max, oracle.MAX), (tf.ReduceOp.Min, oracle.MIN)]:
            got, ref = _reduce_check(tf, oracle, a, [0, 1], [1], op_tf, op_or)
            assert np.array_equal(got, ref)
            got, ref = _reduce_check(tf, oracle, a.reshape(-1), [0], [], op_tf, op_or)
            assert np.array_equal(got, ref)


@pytest.mark.parametrize("dtype", ALL)
def test_contract_one_tile_with_a_very_long_k_and_many_batches(tf, oracle, dtype):
    # a single output tile under a k of several hundred thousand: the range is split hundreds of ways and the partials
    # are folded by the many-splits kernel (fixed order: two runs give the same bits); and a batch count above 65535
    # (more (batch, split) pairs than one grid dimension holds)
    rng = seeded_rng(97)
    m, n, k = 40, 24, 300000
    a, b = rand(rng, (m, k), dtype), rand(rng, (n, k), dtype)
    ref = np.empty((m, n), dtype)
    oracle.contract(a, lab("mk"), b, lab("nk"), ref, lab("mn"))
    plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("mk"), lab("nk"), lab("mn")), [a.shape, b.shape, [m, n]])
    da, db = dev(tf, a), dev(tf, b)
    runs = []
    for _ in range(2):
        out = tf.Tensor.empty([m, n], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
        tf.HipBackend.execute(plan, 1.0, [da, db], 0.0, out)
        runs.append(out.to_numpy())
    assert relerr(runs[0], ref) < 10 * TOL[dtype]
    assert runs[0].tobytes() == runs[1].tobytes()
    c0 = rand(rng, (m, n), dtype)
    ref2 = c0.copy()
    oracle.contract(a, lab("mk"), b, lab("nk"), ref2, lab("mn"), alpha=0.5, beta=-1.0)
    dc = dev(tf, c0)
    tf.HipBackend.execute(plan, 0.5, [da, db], -1.0, dc)
    assert relerr(dc.to_numpy(), ref2) < 10 * TOL[dtype]
    # 70000 batches of a 3 x 5 x 4 product
    nb = 70000
    x, y = rand(rng, (nb, 3, 5), dtype), rand(rng, (nb, 5, 4), dtype)
    ref3 = np.empty((nb, 3, 4), dtype)
    oracle.contract(x, lab("bik"), y, lab("bkj"), ref3, lab("bij"))
    out3 = tf.Tensor.empty([nb, 3, 4], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
    plan3 = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("bik"), lab("bkj"), lab("bij")), [x.shape, y.shape, [nb, 3, 4]])
    tf.HipBackend.execute(plan3, 1.0, [dev(tf, x), dev(tf, y)], 0.0, out3)
    assert relerr(out3.to_numpy(), ref3) < TOL[dtype]


DOT_CASES = [
    ("mk,k->m", dict(m=512, k=1024)),                 # matrix-vector, rows contiguous in k
    ("km,k->m", dict(m=512, k=1024)),                 # ... columns: lanes along m, the vector element broadcast
    ("k,kn->n", dict(n=2048, k=256)),                 # vector-matrix
    ("k,k->", dict(k=1 << 18)),                       # dot product: one output, the range split over blocks
    ("bi,bi->b", dict(b=4096, i=256)),                # batched dot
    ("bmk,bk->bm", dict(b=16, m=64, k=512)),          # batched matrix-vector
    ("abk,kb->ab", dict(a=32, b=64, k=128)),          # the second operand holds the modes in another order
    ("mk,k->m", dict(m=100, k=36)),                   # extents that do not tile: the tiled kernels take it
]


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("case", DOT_CASES, ids=[c[0] + "-" + "x".join(str(v) for v in c[1].values()) for c in DOT_CASES])
def test_contract_with_an_empty_free_group_takes_the_product_reduction_kernel(tf, oracle, dtype, case):
    pattern, ext = case
    ins, mc = pattern.split("->")
    ma, mb = ins.split(",")
    rng = seeded_rng(98)
    a = rand(rng, [ext[l] for l in ma], dtype)
    b = rand(rng, [ext[l] for l in mb], dtype)
    cshape = [ext[l] for l in mc]
    cplx = np.issubdtype(dtype, np.complexfloating)
    tol = 10 * TOL[dtype]
    for alpha, beta in [(1.0, 0.0), ((0.7 - 1.1j, -0.3 + 0.2j) if cplx else (0.7, -0.3))]:
        c0 = rand(rng, cshape, dtype) if cshape else np.array(rng.standard_normal(), dtype)
        ref = c0.copy()
        oracle.contract(a, lab(ma), b, lab(mb), ref, lab(mc), alpha=alpha, beta=beta)
        out = dev(tf, c0) if cshape else tf.Tensor.zeros([], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
        if not cshape:
            ref = np.empty([], dtype)
            oracle.contract(a, lab(ma), b, lab(mb), ref, lab(mc), alpha=alpha, beta=0.0)
            beta = 0.0
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab(ma), lab(mb), lab(mc)), [a.shape, b.shape, cshape])
        tf.HipBackend.execute(plan, alpha, [dev(tf, a), dev(tf, b)], beta, out)
        tiled = "dot_fast_kernel" in tf.last_kernel()
        assert tiled == (ext.get("k", 0) != 36), tf.last_kernel()
        assert relerr(out.to_numpy(), ref) < tol, (alpha, beta)


@pytest.mark.parametrize("dtype", [np.float64, np.complex128, np.float32])
def test_product_reduction_on_strided_and_reversed_views(tf, oracle, dtype):
    # operands seen through stepped, reversed and offset views: scalar loads, negative strides
    rng = seeded_rng(99)
    big = rand(rng, (256, 2 * 512 + 3), dtype)
    a = big[::-1, 1:1025:2]                       # [256, 512], rows reversed, every other column
    x = rand(rng, (3 * 512,), dtype)[::3]
    ref = np.empty((256,), dtype)
    oracle.contract(a, lab("mk"), x, lab("k"), ref, lab("m"))
    out = tf.Tensor.empty([256], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
    plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("mk"), lab("k"), lab("m")), [a.shape, x.shape, [256]])
    tf.HipBackend.execute(plan, 1.0, [dev(tf, a), dev(tf, x)], 0.0, out)
    assert "dot_fast_kernel" in tf.last_kernel()
    assert relerr(out.to_numpy(), ref) < 10 * TOL[dtype]
    # integer inputs: exact, and a mode of the vector that the matrix lacks is summed too ("mk,kj->m")
    ai = rng.integers(-5, 6, (128, 256)).astype(dtype)
    bi = rng.integers(-5, 6, (256, 4)).astype(dtype)
    out2 = tf.Tensor.empty([128], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
    plan2 = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("mk"), lab("kj"), lab("m")), [ai.shape, bi.shape, [128]])
    tf.HipBackend.execute(plan2, 1.0, [dev(tf, ai), dev(tf, bi)], 0.0, out2)
    assert np.array_equal(out2.to_numpy(), np.einsum("mk,kj->m", ai, bi))


def _pow2_extent(rng, big):
    """Extents that tile without partial tiles: a power of two, sometimes times 3 or 5 on a large one."""
    e = int(2 ** rng.integers(0, 8 if big else 4))
    if big and e >= 16 and rng.integers(0, 3) == 0:
        e *= int(rng.choice([3, 5]))
    return e


@pytest.mark.parametrize("dtype", ALL)
def test_product_reduction_random_shapes(tf, oracle, dtype):
    # random contractions with one free group empty, over extents the product-reduction kernel tiles: random mode
    # structure (batch modes, modes only one operand has, several contracted modes), random axis orders, dense or
    # stepped / reversed views, alpha/beta.  Most cases must reach that kernel.
    rng = seeded_rng(101)
    hits = 0
    ncase = 40
    for case in range(ncase):
        labels = list("abcdefgh")
        rng.shuffle(labels)
        nb, nfree, nk = int(rng.integers(0, 3)), int(rng.integers(0, 3)), int(rng.integers(1, 4))
        batch, free, kk = labels[:nb], labels[nb:nb + nfree], labels[nb + nfree:nb + nfree + nk]
        ext = {l: _pow2_extent(rng, True) for l in batch + free + kk}
        while np.prod([ext[l] for l in batch + free + kk], dtype=np.float64) > 4e6:
            l = max(ext, key=ext.get)
            ext[l] = max(1, ext[l] // 4)
        # the free modes belong to the first operand; the second holds batch and contracted modes (and sometimes lacks one)
        ma, mb, mc = batch + free + kk, batch + kk, batch + free
        if len(kk) > 1 and rng.integers(0, 4) == 0:
            mb = batch + kk[:-1]                      # a contracted mode only the first operand has: summed over it
        if rng.integers(0, 2):
            ma, mb = mb, ma
        ma, mb, mc = list(ma), list(mb), list(mc)
        rng.shuffle(ma); rng.shuffle(mb); rng.shuffle(mc)
        if not ma or not mb:
            continue
        plain = case % 3 != 0
        mk = (lambda shape: rand(rng, shape, dtype)) if plain else (lambda shape: _random_view(rng, shape, dtype))
        a, b = mk([ext[l] for l in ma]), mk([ext[l] for l in mb])
        cshape = [ext[l] for l in mc]
        cplx = np.issubdtype(dtype, np.complexfloating)
        use_beta = bool(rng.integers(0, 2)) and len(cshape) > 0
        alpha, beta = ((0.7 - 1.1j, (-0.3 + 0.2j) if use_beta else 0.0) if cplx else (0.7, -0.3 if use_beta else 0.0))
        c0 = rand(rng, cshape, dtype) if use_beta else np.full(cshape, np.nan, dtype)
        ref = c0.copy()
        oracle.contract(a, lab(ma), b, lab(mb), ref, lab(mc), alpha=alpha, beta=beta)
        out = dev(tf, c0) if cshape else tf.Tensor.empty([], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab(ma), lab(mb), lab(mc)), [a.shape, b.shape, cshape])
        print("case", case, "".join(ma), "".join(mb), "".join(mc), ext, "plain" if plain else "views", flush=True)
        tf.HipBackend.execute(plan, alpha, [dev(tf, a), dev(tf, b)], beta, out)
        hits += "dot_fast_kernel" in tf.last_kernel()
        err = relerr(out.to_numpy(), ref)
        assert err < 10 * TOL[dtype], (case, ma, mb, mc, ext, err, tf.last_kernel())
    assert hits >= ncase // 2, hits


@pytest.mark.parametrize("dtype", ALL)
def test_reduce_random_shapes_that_tile(tf, oracle, dtype):
    # random reductions over power-of-two-friendly extents: every variant of the fast kernel (vector / scalar loads,
    # contiguous axis kept or reduced, eight block-serial outputs with the butterfly fold, the serial range split over
    # blocks) is reached by some case; sums, max/min, alpha/beta, dense and strided views
    rng = seeded_rng(102)
    kernels = set()
    cplx = np.issubdtype(dtype, np.complexfloating)
    for case in range(60):
        rank = int(rng.integers(1, 6))
        shape = [_pow2_extent(rng, True) for _ in range(rank)]
        while np.prod(shape, dtype=np.float64) > 4e6:
            shape[int(np.argmax(shape))] //= 4
        keep = [d for d in range(rank) if rng.integers(0, 2)]
        rng.shuffle(keep)
        a = rand(rng, shape, dtype) if case % 3 else _random_view(rng, shape, dtype)
        op_tf, op_or = (tf.ReduceOp.Sum, oracle.SUM)
        if not cplx and case % 5 == 0:
            op_tf, op_or = [(tf.ReduceOp.Max, oracle.MAX), (tf.ReduceOp.Min, oracle.MIN)][case % 2]
        oshape = [shape[d] for d in keep]
        use_beta = case % 4 == 0 and op_or == oracle.SUM and len(oshape) > 0
        c0 = rand(rng, oshape, dtype) if use_beta else None
        print("case", case, shape, keep, flush=True)
        got, ref = _reduce_check(tf, oracle, a, list(range(rank)), keep, op_tf, op_or, alpha=2.0 if use_beta else 1.0,
                                 beta=-0.5 if use_beta else 0.0, c0=c0)
        kernels.add(tf.last_kernel())
        if op_or == oracle.SUM:
            assert relerr(got, ref) < 10 * TOL[dtype], (case, shape, keep, tf.last_kernel())
        else:
            assert np.array_equal(got, ref), (case, shape, keep)
    assert any("reduce_fast_kernel" in k for k in kernels), kernels


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("m,k,n,nbatch", [(8, 8, 8, 500), (16, 16, 16, 300), (32, 32, 32, 100), (5, 7, 3, 1000), (1, 9, 17, 200),
                                          (20, 50, 31, 128), (32, 1, 32, 64), (3, 200, 2, 400)])
def test_batches_of_tiny_products_take_the_wave_kernel(tf, oracle, dtype, m, k, n, nbatch):
    # many products with both free extents at most 32: one wave per 32x32 tile, operands loaded straight into the MFMA
    # layout with bounds masks.  Odd extents, k that is not a multiple of the step, alpha/beta, operand orders.
    rng = seeded_rng(103)
    cplx = np.issubdtype(dtype, np.complexfloating)
    for ma, mb, mc in [("bmk", "bkn", "bmn"), ("kbm", "nbk", "bnm")]:
        ext = dict(b=nbatch, m=m, k=k, n=n)
        a, b = rand(rng, [ext[l] for l in ma], dtype), rand(rng, [ext[l] for l in mb], dtype)
        cshape = [ext[l] for l in mc]
        for alpha, beta in [(1.0, 0.0), ((0.7 - 1.1j, -0.3 + 0.2j) if cplx else (0.7, -0.3))]:
            c0 = rand(rng, cshape, dtype)
            ref = c0.copy()
            oracle.contract(a, lab(ma), b, lab(mb), ref, lab(mc), alpha=alpha, beta=beta)
            out = dev(tf, c0)
            plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab(ma), lab(mb), lab(mc)), [a.shape, b.shape, cshape])
            tf.HipBackend.execute(plan, alpha, [dev(tf, a), dev(tf, b)], beta, out)
            if m > 1 and n > 1:      # (an empty free group goes to the product-reduction kernels instead)
                assert "gemm_wave_kernel" in tf.last_kernel(), tf.last_kernel()
            assert relerr(out.to_numpy(), ref) < TOL[dtype], (ma, mb, mc, alpha, beta)
    # BatchedGemm descriptor, exact on small integers
    ai = rng.integers(-4, 5, (nbatch, m, k)).astype(dtype)
    bi = rng.integers(-4, 5, (nbatch, k, n)).astype(dtype)
    out = tf.Tensor.empty([nbatch, m, n], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
    plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.BatchedGemm([nbatch], m, n, k), [ai.shape, bi.shape, [nbatch, m, n]])
    tf.HipBackend.execute(plan, 1.0, [dev(tf, ai), dev(tf, bi)], 0.0, out)
    assert np.array_equal(out.to_numpy(), np.matmul(ai, bi))


def test_calls_from_several_host_threads_on_their_own_streams(tf, oracle):
    # the library's state (per-stream workspaces, pools, table caches, error slots) is process-global behind a mutex and
    # calls are documented as thread-safe: four host threads, each with its own stream, run a mix of contractions
    # (tables, split-K, packing), einsum trees, permutes and reductions at once; every result is checked
    import threading
    import torch
    rng = seeded_rng(104)
    work = []
    for t in range(4):
        a, b = rand(rng, (24, 8, 20, 12 + t), np.float64), rand(rng, (12 + t, 30, 8), np.float64)      # "ajbk,kcj->abc"
        ref = np.empty((24, 20, 30))
        oracle.contract(a, lab("ajbk"), b, lab("kcj"), ref, lab("abc"))
        p = rand(rng, (16, 8 + t, 16, 8), np.float64)
        pref = np.ascontiguousarray(p.transpose(3, 1, 0, 2))
        rref = p.sum(axis=(1, 3))
        ops = [rand(rng, s_, np.complex128) for s_ in [(9, 3, 8 + t), (9, 2, 7), (3, 2, 2, 4), (8 + t, 2, 6)]]
        eref = np.einsum("awc,asx,wstv,cty->xvy", *ops)
        work.append((a, b, ref, p, pref, rref, ops, eref))
    errors = []

    def body(t):
        try:
            a, b, ref, p, pref, rref, ops, eref = work[t]
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                st = stream.cuda_stream
                da, db, dp = dev(tf, a), dev(tf, b), dev(tf, p)
                dops = [dev(tf, o) for o in ops]
                stream.synchronize()
                plan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Contract(lab("ajbk"), lab("kcj"), lab("abc")), [a.shape, b.shape, ref.shape])
                pplan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Permute([0, 1, 2, 3], [3, 1, 0, 2]), [p.shape, pref.shape])
                rplan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Reduce([0, 1, 2, 3], [0, 2], tf.ReduceOp.Sum), [p.shape, rref.shape])
                for it in range(25):
                    out = tf.Tensor.empty(list(ref.shape), tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64)
                    pout = tf.Tensor.empty(list(pref.shape), tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64)
                    rout = tf.Tensor.empty(list(rref.shape), tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float64)
                    tf.HipBackend.execute(plan, 1.0, [da, db], 0.0, out, st)
                    tf.HipBackend.execute(pplan, 1.0, [dp], 0.0, pout, st)
                    tf.HipBackend.execute(rplan, 1.0, [dp], 0.0, rout, st)
                    e = tf.einsum("awc,asx,wstv,cty->xvy", dops, st)
                    stream.synchronize()
                    assert relerr(out.to_numpy(), ref) < 1e-12
                    assert pout.to_numpy().tobytes() == pref.tobytes()
                    assert relerr(rout.to_numpy(), rref) < 1e-12
                    assert relerr(e.to_numpy(), eref) < 1e-12
        except BaseException as ex:      # noqa: BLE001 -- reported by the main thread
            errors.append((t, repr(ex)))

    threads = [threading.Thread(target=body, args=(t,)) for t in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors


def test_operand_above_4_gib(tf, oracle):
    # An f32 matrix of 40000 x 30000 (4.8 GB): element byte offsets pass 2^32, so the large-tile kernel's 32-bit
    # addressing does not apply and the kernels with 64-bit addressing take over.  The tensor is too large for the
    # oracle as a whole: data movement is checked through the involution (bit for bit, on the device) and arithmetic
    # against the oracle on sampled rows, some of them beyond the 4 GiB mark and on tile boundaries.
    import torch
    m, k = 40000, 30000
    gen = torch.Generator(device="cuda").manual_seed(7)
    x = torch.randn(m, k, dtype=torch.float32, device="cuda", generator=gen)
    X = tf.Tensor.from_torch(x)
    rows = [0, 1, 63, 64, 127, 128, 20011, 35791, 35792, 39935, 39936, 39999]
    xs = x[rows].cpu().numpy()
    rng = seeded_rng(111)

    t = tf.Tensor.empty([k, m], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float32)
    back = tf.Tensor.empty([m, k], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float32)
    tf.HipBackend.execute(tf.HipBackend.plan(np.float32, tf.PrimDescriptor.Permute([0, 1], [1, 0]), [[m, k], [k, m]]), 1.0, [X], 0.0, t)
    tf.HipBackend.execute(tf.HipBackend.plan(np.float32, tf.PrimDescriptor.Permute([0, 1], [1, 0]), [[k, m], [m, k]]), 1.0, [t], 0.0, back)
    assert torch.equal(back._buf.view(m, k), x)
    assert np.array_equal(t._buf.view(k, m)[:, rows].cpu().numpy(), xs.T)
    del back, t

    def sampled(out, width):
        return out._buf.view(m, width)[rows].cpu().numpy() if width else out._buf[rows].cpu().numpy()

    v = rand(rng, (k,), np.float32)
    out = tf.Tensor.empty([m], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float32)
    tf.HipBackend.execute(tf.HipBackend.plan(np.float32, tf.PrimDescriptor.Contract(lab("mk"), lab("k"), lab("m")), [[m, k], [k], [m]]), 1.0, [X, dev(tf, v)], 0.0, out)
    ref = np.empty(len(rows), np.float32)
    oracle.contract(xs, lab("mk"), v, lab("k"), ref, lab("m"))
    assert relerr(sampled(out, 0), ref) < 1e-5, tf.last_kernel()

    tf.HipBackend.execute(tf.HipBackend.plan(np.float32, tf.PrimDescriptor.Reduce([0, 1], [0], tf.ReduceOp.Sum), [[m, k], [m]]), 1.0, [X], 0.0, out)
    oracle.reduce(xs, [0, 1], ref, [0])
    assert relerr(sampled(out, 0), ref) < 1e-5, tf.last_kernel()

    for n in (64, 256):      # a thin and a wide right-hand side
        # rows and k of the big operand have one stride each: the large-tile kernel folds the tile's first row and the
        # stage's first k into its 64-bit base, so its 32-bit offsets only span a tile
        w = rand(rng, (k, n), np.float32)
        out = tf.Tensor.empty([m, n], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float32)
        tf.HipBackend.execute(tf.HipBackend.plan(np.float32, tf.PrimDescriptor.Contract(lab("mk"), lab("kn"), lab("mn")), [[m, k], [k, n], [m, n]]), 1.0, [X, dev(tf, w)], 0.0, out)
        assert "gemm128_kernel" in tf.last_kernel(), tf.last_kernel()
        ref = np.empty((len(rows), n), np.float32)
        oracle.contract(xs, lab("mk"), w, lab("kn"), ref, lab("mn"))
        assert relerr(sampled(out, n), ref) < 1e-5, n
        # the big operand on the right (k-contiguous rows of B), the output transposed
        out = tf.Tensor.empty([n, m], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float32)
        tf.HipBackend.execute(tf.HipBackend.plan(np.float32, tf.PrimDescriptor.Contract(lab("kn"), lab("mk"), lab("nm")), [[k, n], [m, k], [n, m]]), 1.0, [dev(tf, w), X], 0.0, out)
        assert "gemm128_kernel" in tf.last_kernel(), tf.last_kernel()
        assert relerr(out._buf.view(n, m)[:, rows].cpu().numpy(), ref.T) < 1e-5, n
    # the same matrix as a [200, 199, k] view of [200, 200, k]: the row group has two strides that do not fuse, its
    # 32-bit table would have to span the whole operand -- the kernel with 64-bit offsets takes it
    n = 256
    X3 = tf.Tensor(x.view(-1), [200, 199, k], [200 * k, k, 1], 0, tf.GpuMemory(0), tf.dtype_code(np.dtype(np.float32)))
    out = tf.Tensor.empty([200, 199, n], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, np.float32)
    tf.HipBackend.execute(tf.HipBackend.plan(np.float32, tf.PrimDescriptor.Contract(lab("abk"), lab("kn"), lab("abn")), [[200, 199, k], [k, n], [200, 199, n]]), 1.0, [X3, dev(tf, w)], 0.0, out)
    assert "(gemm_kernel" in tf.last_kernel(), tf.last_kernel()
    pick = [(0, 0), (0, 198), (1, 0), (99, 57), (178, 190), (179, 0), (199, 198)]
    xs3 = np.stack([x[a_ * 200 + b_].cpu().numpy() for a_, b_ in pick])
    ref = np.empty((len(pick), n), np.float32)
    oracle.contract(xs3, lab("mk"), w, lab("kn"), ref, lab("mn"))
    got = np.stack([out._buf.view(200, 199, n)[a_, b_].cpu().numpy() for a_, b_ in pick])
    assert relerr(got, ref) < 1e-5


def test_long_grids_and_high_rank(tf, oracle):
    # extents past the 65535 limit of a grid's y and z dimensions, many small outputs, a rank-12 permutation
    rng = seeded_rng(112)
    x = rand(rng, (70000, 3, 5), np.float64)
    out = dev(tf, np.zeros((5, 70000, 3)))
    tf.HipBackend.execute(tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Permute([0, 1, 2], [2, 0, 1]), [x.shape, out.dims()]), 1.0, [dev(tf, x)], 0.0, out)
    assert out.to_numpy().tobytes() == np.ascontiguousarray(x.transpose(2, 0, 1)).tobytes()
    for shape, keep in [((300000, 7), 0), ((7, 300000), 1)]:
        y = rand(rng, shape, np.float64)
        ref = np.empty(300000)
        oracle.reduce(y, [0, 1], ref, [keep])
        out = dev(tf, np.zeros(300000))
        tf.HipBackend.execute(tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Reduce([0, 1], [keep], tf.ReduceOp.Sum), [list(shape), [300000]]), 1.0, [dev(tf, y)], 0.0, out)
        assert relerr(out.to_numpy(), ref) < 1e-12, shape
    a, b = rand(rng, (70000, 3, 4), np.float64), rand(rng, (70000, 4, 5), np.float64)
    ref = np.empty((70000, 3, 5))
    oracle.contract(a, lab("bij"), b, lab("bjk"), ref, lab("bik"))
    got = tf.einsum("bij,bjk->bik", [dev(tf, a), dev(tf, b)])
    assert relerr(got.to_numpy(), ref) < 1e-12, tf.last_kernel()
    shape = [2, 3] * 6
    perm = [11, 0, 9, 2, 7, 4, 5, 6, 3, 8, 1, 10]
    z = rand(rng, shape, np.float64)
    oshape = [shape[q] for q in perm]
    out = dev(tf, np.zeros(oshape))
    tf.HipBackend.execute(tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Permute(list(range(12)), perm), [shape, oshape]), 1.0, [dev(tf, z)], 0.0, out)
    assert out.to_numpy().tobytes() == np.ascontiguousarray(z.transpose(perm)).tobytes()


def test_tensor_view_materialises_on_the_device(tf, oracle):
    # TensorView (tenferro-tensor/src/lib.rs:183-300) over device memory: zero-copy permute / diagonal / broadcast, then
    # to_tensor / contiguous / conj run the copy kernels; bit-exact against the oracle's permute
    rng = seeded_rng(120)
    x = rand(rng, (6, 5, 6, 4), np.complex128)
    v = dev(tf, x).tensor_view()
    assert v.logical_memory_space() == tf.GpuMemory(0) and v.dims() == [6, 5, 6, 4]
    p = v.permute([3, 0, 2, 1])
    ref = np.empty((4, 6, 6, 5), np.complex128)
    oracle.permute(x, [0, 1, 2, 3], ref, [3, 0, 2, 1])
    for order in (tf.MemoryOrder.RowMajor, tf.MemoryOrder.ColumnMajor):
        t = p.to_tensor(order)
        assert t.is_contiguous() and t.to_numpy().tobytes() == ref.tobytes()
        assert p.contiguous(order).to_numpy().tobytes() == ref.tobytes()
    d = v.diagonal([(0, 2)])                   # axes 0 and 2 merged: dims [6, 5, 4]
    assert d.dims() == [6, 5, 4]
    assert d.to_tensor(tf.MemoryOrder.RowMajor).to_numpy().tobytes() == np.ascontiguousarray(np.einsum("ijik->ijk", x)).tobytes()
    b = dev(tf, x[:, :1]).tensor_view().broadcast([6, 5, 6, 4])
    assert b.to_tensor(tf.MemoryOrder.RowMajor).to_numpy().tobytes() == np.ascontiguousarray(np.broadcast_to(x[:, :1], x.shape)).tobytes()
    assert p.conj().to_numpy().tobytes() == np.conj(ref).tobytes()


def test_contract_tiny_operator_applied_to_a_long_tensor(tf):
    # One operand with at most 8 free and 8 contracted indices, the other long (a gate on one or two legs of a state):
    # the streaming kernel, against numpy's einsum in double precision.  Legs at the front, in the middle and at the end,
    # extents 2, 3 and 8, either operand order, two-leg gates, alpha/beta, a sliced long operand, an output whose
    # contiguous axis is not the long operand's (scalar accesses), all four dtypes; exact on small integers.
    rng = seeded_rng(134)
    lab = lambda t: [ord(ch) for ch in t]

    def run(sub, sa, sb, dtype, alpha=1.0, beta=0.0, views=None, out_order="C", exact=False):
        ia, ib, ic = sub.replace("->", ",").split(",")
        if exact:
            x, y = rng.integers(-3, 4, size=sa).astype(dtype), rng.integers(-3, 4, size=sb).astype(dtype)
        else:
            x, y = rand(rng, sa, dtype), rand(rng, sb, dtype)
        if views:
            x, y = views(x, y)
        ref = np.einsum(sub, x.astype(np.complex128), y.astype(np.complex128))
        c0 = rand(rng, ref.shape, dtype)
        c0 = np.asfortranarray(c0) if out_order == "F" else c0
        out = dev(tf, c0 if beta != 0.0 else np.full_like(c0, np.nan))
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab(ia), lab(ib), lab(ic)), [list(x.shape), list(y.shape), list(ref.shape)])
        tf.HipBackend.execute(plan, alpha, [dev(tf, x), dev(tf, y)], beta, out)
        assert "tiny_operator_kernel" in tf.last_kernel(), (sub, sa, sb, tf.last_kernel())
        want = alpha * ref + (beta * c0 if beta != 0.0 else 0.0)
        if exact:
            assert np.array_equal(out.to_numpy(), want.real.astype(dtype)), (sub, sa, sb, dtype)
        else:
            assert relerr(out.to_numpy(), want) < TOL[dtype], (sub, sa, sb, dtype)

    for dtype in ALL:
        run("ab,xby->xay", (2, 2), (64, 2, 1024), dtype)
        run("ab,xby->xay", (2, 2), (1, 2, 131072), dtype)
        run("ab,xby->xay", (2, 2), (131072, 2, 1), dtype)
        run("ab,xby->xay", (3, 3), (243, 3, 729), dtype)
        run("xby,ba->xay", (64, 2, 1024), (2, 2), dtype)                       # the operator second
        run("abcd,xcydz->xaybz", (2, 2, 2, 2), (32, 2, 32, 2, 64), dtype)       # two legs
        run("ab,xby->xay", (8, 8), (64, 8, 1024), dtype, alpha=-0.5, beta=2.0)
        run("ab,xby->xay", (5, 3), (100, 3, 700), dtype)                       # rectangular, nothing a power of two
        run("ab,xby->xay", (2, 2), (65, 2, 1023), dtype)                       # odd inner extent: scalar accesses
        run("ab,xby->xay", (2, 2), (64, 2, 1024), dtype, out_order="F")         # the output contiguous along x
        run("ab,xby->xay", (4, 4), (70, 4, 1100), dtype, views=lambda x, y: (x.T, y[3:67, :, 50:1074]))   # transposed operator, sliced tensor
        run("ab,xby->yax", (2, 2), (64, 2, 1024), dtype)                       # the long axes exchanged in the output
    run("ab,xby->xay", (2, 2), (64, 2, 1024), np.float64, exact=True)
    run("abcd,xcydz->xaybz", (2, 2, 2, 2), (32, 2, 32, 2, 64), np.float32, exact=True)
    if True:
        z = (rng.integers(-2, 3, size=(2, 2)) + 1j * rng.integers(-2, 3, size=(2, 2))).astype(np.complex128)
        t = (rng.integers(-2, 3, size=(32, 2, 2048)) + 1j * rng.integers(-2, 3, size=(32, 2, 2048))).astype(np.complex128)
        out = dev(tf, np.zeros((32, 2, 2048), np.complex128))
        tf.HipBackend.execute(tf.HipBackend.plan(np.complex128, tf.PrimDescriptor.Contract(lab("ab"), lab("xby"), lab("xay")), [[2, 2], [32, 2, 2048], [32, 2, 2048]]), 1.0, [dev(tf, z), dev(tf, t)], 0.0, out)
        assert "tiny_operator_kernel" in tf.last_kernel() and np.array_equal(out.to_numpy(), np.einsum("ab,xby->xay", z, t))


def test_contract_without_a_summed_index_scales_through_the_elementwise_kernel(tf):
    # "asx,x->asx", "ij,i->ij": a tensor scaled along some of its axes.  One free group is empty and nothing is summed, so
    # the elementwise kernel does it with the missing axes as broadcast axes; extents that tile and extents that do not,
    # alpha/beta, all dtypes (4-byte elements keep the product-reduction kernel where the extents tile).
    rng = seeded_rng(135)
    lab = lambda t: [ord(ch) for ch in t]
    for dtype in ALL:
        for sub, sa, sb in (("asx,x->asx", (100, 3, 1000), (1000,)), ("asx,a->asx", (128, 2, 1024), (128,)), ("ij,j->ij", (1021, 1031), (1031,)),
                            ("ij,i->ji", (512, 300), (512,)), ("abcd,ca->abcd", (16, 9, 32, 40), (32, 16))):
            ia, ib, ic = sub.replace("->", ",").split(",")
            x, y = rand(rng, sa, dtype), rand(rng, sb, dtype)
            ref = np.einsum(sub, x.astype(np.complex128), y.astype(np.complex128))
            c0 = rand(rng, ref.shape, dtype)
            out = dev(tf, c0)
            plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab(ia), lab(ib), lab(ic)), [list(sa), list(sb), list(ref.shape)])
            tf.HipBackend.execute(plan, 2.0, [dev(tf, x), dev(tf, y)], -1.0, out)
            if np.dtype(dtype).itemsize >= 8 or sa in ((100, 3, 1000), (1021, 1031), (512, 300), (16, 9, 32, 40)):
                assert "emul_kernel" in tf.last_kernel(), (sub, sa, dtype, tf.last_kernel())
            assert relerr(out.to_numpy(), 2.0 * ref - c0) < TOL[dtype], (sub, sa, dtype)


def test_permute_tensors_of_many_short_axes(tf):
    # Tensors of many small extents (spins, qubits): the tile is a product of whole axes and its position-to-offset maps
    # come from cached tables.  Bit-exact against numpy for reversals, a cyclic shift and neighbour exchanges, extents that
    # are and are not powers of two, 4-, 8- and 16-byte elements, a sliced operand (strides that are not the dense ones),
    # the second call on a layout (tables from the cache) and a call after the caches were released.
    rng = seeded_rng(133)
    cases = [((3,) * 14, tuple(reversed(range(14))), np.float64), ((3,) * 12, tuple(reversed(range(12))), np.complex128),
             ((3,) * 13, (0, 2, 1, 3, 5, 4, 6, 8, 7, 9, 11, 10, 12), np.float32), ((5,) * 8, tuple(reversed(range(8))), np.float64),
             ((3, 4) * 5, tuple(reversed(range(10))), np.float64), ((2, 3) * 7, tuple(reversed(range(14))), np.float64),
             ((4,) * 10, tuple(reversed(range(10))), np.float32), ((2,) * 16, tuple(reversed(range(16))), np.complex64),
             ((6,) * 7, (3, 4, 5, 6, 0, 1, 2), np.float64), ((100, 50, 20, 17), (0, 1, 3, 2), np.float64)]
    used = 0
    for shape, perm, dtype in cases:
        x = rand(rng, shape, dtype)
        oshape = [shape[q] for q in perm]
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Permute(list(range(len(shape))), list(perm)), [list(shape), oshape])
        for rep in range(2):
            out = dev(tf, np.zeros(oshape, dtype))
            tf.HipBackend.execute(plan, 1.0, [dev(tf, x)], 0.0, out)
            used += "tabcopy_kernel" in tf.last_kernel() or "perm_kernel" in tf.last_kernel()
            assert out.to_numpy().tobytes() == np.ascontiguousarray(x.transpose(perm)).tobytes(), (shape, perm, dtype, tf.last_kernel())
    assert used >= 14, used            # most of these shapes take the table-driven or the two-sided tiles, on both calls
    # a slice of a larger tensor: strides of the operand are not those of a dense tensor
    big = rand(rng, (4,) + (3,) * 11, np.float64)      # (under 4 MB: the table tiles' size)
    x = big[1]
    perm = tuple(reversed(range(11)))
    plan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Permute(list(range(11)), list(perm)), [[3] * 11, [3] * 11])
    out = dev(tf, np.zeros((3,) * 11))
    tf.HipBackend.execute(plan, 1.0, [dev(tf, x)], 0.0, out)
    assert out.to_numpy().tobytes() == np.ascontiguousarray(x.transpose(perm)).tobytes()
    assert tf.lib().tfh_release_workspaces() == 0
    tf.HipBackend.execute(plan, 1.0, [dev(tf, x)], 0.0, out)
    assert "tabcopy_kernel" in tf.last_kernel() and out.to_numpy().tobytes() == np.ascontiguousarray(x.transpose(perm)).tobytes()
    # alpha/beta and conj keep the masked tiles (the table path moves raw bits only)
    z = rand(rng, (3,) * 12, np.complex128)
    perm = tuple(reversed(range(12)))
    got = dev(tf, np.zeros((3,) * 12, np.complex128))
    tf.HipBackend.execute(tf.HipBackend.plan(np.complex128, tf.PrimDescriptor.Permute(list(range(12)), list(perm)), [[3] * 12, [3] * 12]), 2.0, [dev(tf, z)], 0.0, got)
    assert "tabcopy_kernel" not in tf.last_kernel() and np.array_equal(got.to_numpy(), 2.0 * z.transpose(perm))


def test_reduce_over_short_contiguous_rows(tf, oracle):
    # A reduced contiguous axis of 2..32 elements inside a long kept axis, extents that do not tile (17, 31, 3; an even 6
    # under an odd row count): 256 rows per block go through LDS and every thread adds up its own row.  Sum (exact on
    # small integers, and against the oracle on random data), max/min, alpha/beta on a permuted output, a sliced operand
    # whose outer axes do not merge, both real dtypes; complex and rows longer than 32 stay on the general kernel.
    rng = seeded_rng(132)
    for dtype in (np.float64, np.float32):
        for shape, red in (((100, 100, 100, 17), (3,)), ((15, 17, 33, 65, 31), (4,)), ((4097, 333, 3), (2,)), ((1001, 1025, 6), (2,)),
                           ((3000, 32), (1,)), ((70000, 2), (1,))):
            a = rng.integers(-3, 4, size=shape).astype(dtype)
            modes = list(range(len(shape)))
            kept = [m for m in modes if m not in red]
            oshape = [shape[m] for m in kept]
            out = dev(tf, np.full(oshape, np.nan, dtype))
            tf.HipBackend.execute(tf.HipBackend.plan(dtype, tf.PrimDescriptor.Reduce(modes, kept, tf.ReduceOp.Sum), [list(shape), oshape]), 1.0, [dev(tf, a)], 0.0, out)
            assert "reduce_shortrow_kernel" in tf.last_kernel(), (shape, tf.last_kernel())
            assert np.array_equal(out.to_numpy(), a.sum(axis=red, dtype=np.float64).astype(dtype)), (shape, dtype)
        x = rand(rng, (37, 1500, 17), dtype)
        got, ref = _reduce_check(tf, oracle, x, [0, 1, 2], [0, 1], tf.ReduceOp.Sum, oracle.SUM)
        assert "reduce_shortrow_kernel" in tf.last_kernel() and relerr(got, ref) < TOL[dtype]
        for op_tf, op_or in [(tf.ReduceOp.Max, oracle.MAX), (tf.ReduceOp.Min, oracle.MIN)]:
            got, ref = _reduce_check(tf, oracle, x, [0, 1, 2], [0, 1], op_tf, op_or)
            assert "reduce_shortrow_kernel" in tf.last_kernel() and np.array_equal(got, ref)
        # output axes exchanged (C strides 1 and 37), alpha and beta
        c0 = rand(rng, (1500, 37), dtype)
        got, ref = _reduce_check(tf, oracle, x, [0, 1, 2], [1, 0], tf.ReduceOp.Sum, oracle.SUM, alpha=-1.5, beta=0.25, c0=c0)
        assert "reduce_shortrow_kernel" in tf.last_kernel() and relerr(got, ref) < TOL[dtype]
        # a slice: the outer axis does not merge with the rows' axis
        big = rand(rng, (9, 1400, 13), dtype)
        got, ref = _reduce_check(tf, oracle, big[:, 100:1300, :], [0, 1, 2], [0, 1], tf.ReduceOp.Sum, oracle.SUM)
        assert "reduce_shortrow_kernel" in tf.last_kernel() and relerr(got, ref) < TOL[dtype]
        # rows that are not dense (every second one): the general kernel
        got, ref = _reduce_check(tf, oracle, big[:, ::2, :], [0, 1, 2], [0, 1], tf.ReduceOp.Sum, oracle.SUM)
        assert "reduce_shortrow_kernel" not in tf.last_kernel() and relerr(got, ref) < TOL[dtype]
    z = rand(rng, (2000, 17), np.complex128)
    got, ref = _reduce_check(tf, oracle, z, [0, 1], [0], tf.ReduceOp.Sum, oracle.SUM)
    assert "reduce_shortrow_kernel" not in tf.last_kernel() and relerr(got, ref) < 1e-12
    w = rand(rng, (2000, 33), np.float64)
    got, ref = _reduce_check(tf, oracle, w, [0, 1], [0], tf.ReduceOp.Sum, oracle.SUM)
    assert "reduce_shortrow_kernel" not in tf.last_kernel() and relerr(got, ref) < 1e-12


def test_rotated_serial_starts_sum_every_index_exactly_once(tf):
    # The fast reduction and product-reduction kernels start the serial range of a block group (or of a chunk of a
    # split range) at a rotated index and wrap round.  Small-integer inputs make every sum exact in f64 and f32, so a
    # serial index that is skipped or taken twice -- counts that are not powers of two, a last chunk shorter than the
    # others -- shows as an inequality.  Shapes: a middle axis of 12 and of 7 with serial steps of 128 KB under >= 512
    # blocks (rotation by block group), 1000 and 777 rows summed into few outputs (rotation by chunk).
    rng = seeded_rng(131)
    lab = lambda t: [ord(ch) for ch in t]

    def ints(shape, dtype):
        return rng.integers(-3, 4, size=shape).astype(dtype)

    for dtype in (np.float64, np.float32):
        for shape, red in (((24, 12, 16, 1024), (1,)), ((40, 7, 32, 512), (1,)), ((1000, 96, 128), (0,)), ((777, 2048), (0,)),
                           ((6, 5, 9, 16, 2048), (1, 2))):
            a = ints(shape, dtype)
            modes = list(range(len(shape)))
            kept = [m for m in modes if m not in red]
            out = dev(tf, np.full([shape[m] for m in kept], np.nan, dtype))
            plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Reduce(modes, kept, tf.ReduceOp.Sum), [list(shape), [shape[m] for m in kept]])
            tf.HipBackend.execute(plan, 1.0, [dev(tf, a)], 0.0, out)
            assert "reduce_fast_kernel" in tf.last_kernel(), (shape, tf.last_kernel())
            assert np.array_equal(out.to_numpy(), a.sum(axis=red, dtype=np.float64).astype(dtype)), (shape, red, dtype)
        # the same through the product reduction: a vector contracted with a middle axis, vector x matrix
        for sub, sa, sb in (("ajbi,j->abi", (24, 12, 16, 1024), (12,)), ("ajbi,j->abi", (40, 7, 32, 512), (7,)),
                            ("i,ij->j", (1000,), (1000, 4096)), ("i,ij->j", (777,), (777, 2048))):
            ia, ib, ic = sub.replace("->", ",").split(",")
            x, y = ints(sa, dtype), ints(sb, dtype)
            ref = np.einsum(sub, x.astype(np.float64), y.astype(np.float64))
            out = dev(tf, np.full(ref.shape, np.nan, dtype))
            plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab(ia), lab(ib), lab(ic)), [list(sa), list(sb), list(ref.shape)])
            tf.HipBackend.execute(plan, 1.0, [dev(tf, x), dev(tf, y)], 0.0, out)
            assert "dot_fast_kernel" in tf.last_kernel(), (sub, sa, tf.last_kernel())
            assert np.array_equal(out.to_numpy(), ref.astype(dtype)), (sub, sa, dtype)


def test_intermediates_cached_for_reuse_are_given_back_when_the_device_runs_out_of_memory(tf):
    # The intermediates of a contraction tree come from a per-stream cache of device blocks that keeps them after the
    # call.  With the device nearly full, a tree whose intermediate fits no cached block and no free memory must still
    # run: the cached blocks are released and the allocation is tried again.  The free memory is bounded with one large
    # untouched allocation; the three intermediates (2.0, 2.6, 3.4 GiB) each exceed what the earlier ones can hold.
    import torch
    assert tf.lib().tfh_release_workspaces() == 0
    torch.cuda.empty_cache()
    gib = 1 << 30
    free, _ = torch.cuda.mem_get_info()
    if free < 16 * gib:
        pytest.skip("needs 16 GiB of free device memory")
    try:
        ballast = torch.empty(free - 6 * gib, dtype=torch.uint8, device="cuda")
    except RuntimeError:
        pytest.skip("one allocation of all but 6 GiB of the free device memory is not available")
    try:
        rng = seeded_rng(130)
        subs = tf.Subscripts.parse("ij,jk,kl->il")
        for step, n in enumerate((16384, 18688, 21376)):
            a, b, c = rand(rng, (n, 2), np.float64), rand(rng, (2, n), np.float64), rand(rng, (n, 3), np.float64)
            tree = tf.ContractionTree.from_pairs(subs, [a.shape, b.shape, c.shape], [(0, 1), (3, 2)])   # (A B) first: n x n
            assert tree.peak_intermediate == n * n
            if step == 2:
                torch.cuda.synchronize()
                assert torch.cuda.mem_get_info()[0] < n * n * 8   # the cached blocks hold what this step would need
            out = tf.einsum_with_plan(tree, [dev(tf, a), dev(tf, b), dev(tf, c)])
            assert relerr(out.to_numpy(), a @ (b @ c)) < 1e-12
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] < 6 * gib - 21376 * 21376 * 8 + gib   # the last intermediate stays cached
        import ctypes
        p = ctypes.c_void_p()
        assert tf.lib().tfh_malloc(4 * gib, ctypes.byref(p)) == 0 and p.value     # tfh_malloc gives the cache back too
        assert tf.lib().tfh_free(p) == 0
    finally:
        del ballast
        assert tf.lib().tfh_release_workspaces() == 0
        torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype", ALL)
def test_reduce_dense_runs_of_any_extent(tf, oracle, dtype):
    # Extents that are no powers of two on a contiguous operand: the tiles are contiguous runs of memory with one ragged
    # edge, folded over the reduced axes inside the tile in LDS.  Integer inputs: every sum is exact, so a dropped or
    # doubled element (a ragged last range, the odd reals behind the last 16-byte vector, a split walk) changes the result.
    rng = seeded_rng(131)
    cplx = np.issubdtype(dtype, np.complexfloating)
    def ints(shape):
        x = rng.integers(-9, 10, shape).astype(np.float64)
        return (x + 1j * rng.integers(-9, 10, shape)).astype(dtype) if cplx else x.astype(dtype)
    cases = [((37, 141, 147), [2]),            # kept innermost axis under one long fused reduced axis: split walk
             ((41, 83, 1891), [0, 1]),         # long reduced rows, a tile per row
             ((53, 42, 19, 79), [1, 2, 3]),    # outermost axis reduced, a range of the fused kept axis per tile
             ((27, 90, 5, 21, 13), [0, 1, 3, 4]),   # a short reduced axis between kept ones
             ((9, 25, 26, 11, 6, 9), [4]),     # nearly everything reduced, kept axis inside the tile
             ((12, 10, 9, 7, 17, 5, 5), [0, 1, 4, 5, 6]),
             ((5, 9, 33, 10, 21, 7), [3, 4, 5]),
             ((358, 481, 3), [0, 2]),          # reduced middle axis, short kept rows
             ((101, 29, 141, 9), [0]),
             ((11, 139, 46, 3, 7), [2, 4]),
             ((7, 37, 17, 19, 9, 3), [5]),
             ((70001,), []),                   # one output
             ((3, 70001), [0]),
             ((66000, 3), [1])]
    ran = 0
    for shape, keep in cases:
        a = ints(shape)
        m = list(range(len(shape)))
        got, ref = _reduce_check(tf, oracle, a, m, keep, tf.ReduceOp.Sum, oracle.SUM)
        ran += "reduce_run_kernel" in tf.last_kernel()
        assert np.array_equal(got, ref), (shape, keep, tf.last_kernel())
        got2, _ = _reduce_check(tf, oracle, a, m, keep, tf.ReduceOp.Sum, oracle.SUM)
        assert np.array_equal(got, got2), (shape, keep)                   # same bits on every run
        perm = [int(p) for p in rng.permutation(len(keep))]                # outputs in another axis order
        got3, ref3 = _reduce_check(tf, oracle, a, m, [keep[p] for p in perm], tf.ReduceOp.Sum, oracle.SUM)
        assert np.array_equal(got3, ref3), (shape, keep, perm)
    assert ran >= 10, ran
    a = rand(rng, (37, 141, 147), dtype)
    c0 = rand(rng, (147, 37), dtype)
    alpha, beta = (0.5 - 2.0j, 1.5 + 0.25j) if cplx else (2.0, -0.5)
    got, ref = _reduce_check(tf, oracle, a, [0, 1, 2], [2, 0], tf.ReduceOp.Sum, oracle.SUM, alpha=alpha, beta=beta, c0=c0)
    assert relerr(got, ref) < TOL[dtype]
    # the operand starts at an odd element of its buffer, so no tile starts on a 16-byte boundary
    base = ints((37 * 141 * 147 + 3,))
    a = base[3:].reshape(37, 141, 147)
    got, ref = _reduce_check(tf, oracle, a, [0, 1, 2], [1], tf.ReduceOp.Sum, oracle.SUM)
    assert np.array_equal(got, ref)
    if not cplx:
        a = rand(rng, (41, 83, 189), dtype)
        for op_tf, op_or in [(tf.ReduceOp.Max, oracle.MAX), (tf.ReduceOp.Min, oracle.MIN)]:
            for keep in ([0, 1], [2], [1], []):
                got, ref = _reduce_check(tf, oracle, a, [0, 1, 2], keep, op_tf, op_or)
                assert np.array_equal(got, ref), (keep, tf.last_kernel())


@pytest.mark.parametrize("dtype", ALL)
def test_permute_table_tiles_with_ranged_axes(tf, oracle, dtype):
    # Long extents that are no powers of two: a tile holds a range of such an axis, and only the last range is ragged
    # (its positions past the edge are left out through the coordinate tables).  Bit-exact against the oracle; every
    # element of the output starts as NaN, so a position that is never written shows.
    rng = seeded_rng(137)
    cases = [((27, 46, 141), (2, 0, 1)), ((27, 46, 141), (1, 0, 2)), ((27, 46, 141), (2, 1, 0)), ((27, 46, 141), (0, 2, 1)),
             ((193, 25, 47), (2, 0, 1)), ((53, 42, 19, 7), (2, 0, 3, 1)), ((27, 9, 5, 21, 13), (1, 0, 2, 4, 3)),
             ((81, 59, 74), (1, 0, 2)), ((11, 29, 14, 9), (3, 1, 2, 0)), ((17, 43, 35, 13), (1, 2, 0, 3)),
             ((3, 7, 28, 6, 22, 9), (1, 5, 0, 2, 3, 4)), ((33, 17, 296, 2), (0, 2, 3, 1)), ((4, 5, 22, 18, 17, 2), (0, 4, 2, 5, 3, 1)),
             ((1031, 67), (1, 0)), ((67, 1031), (1, 0)), ((2, 70001), (1, 0)), ((263, 259), (1, 0)), ((131, 3, 257), (2, 1, 0))]
    ran = 0
    for shape, perm in cases:
        a = rand(rng, shape, dtype)
        oshape = [shape[p] for p in perm]
        ref = np.empty(oshape, dtype)
        oracle.permute(a, list(range(len(shape))), ref, list(perm))
        out = dev(tf, np.full(oshape, np.nan, dtype))
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Permute(list(range(len(shape))), list(perm)), [list(shape), oshape])
        tf.HipBackend.execute(plan, 1.0, [dev(tf, a)], 0.0, out)
        ran += "tabcopy_kernel" in tf.last_kernel()
        assert out.to_numpy().tobytes() == ref.tobytes(), (shape, perm, tf.last_kernel())
        tf.HipBackend.execute(plan, 1.0, [dev(tf, a)], 0.0, out)            # second call: the cached tables
        assert out.to_numpy().tobytes() == ref.tobytes(), (shape, perm, "second call")
    assert ran >= 10, ran


@pytest.mark.parametrize("dtype", ALL)
def test_permute_two_sided_tiles_of_long_odd_extents(tf, oracle, dtype):
    # Seventeen million elements and more with extents that are no powers of two: 64 KB tiles whose read run and write run are
    # ranges of long axes, ragged at the last range (lanes past the end of a run and rows past the edge are left out of
    # the stores).  Bit-exact against the oracle on an output that starts as NaN; the last shapes share the fastest axis
    # between input and output, or have a run of three elements on one side.
    rng = seeded_rng(139)
    cases = [((27, 466, 1401), (2, 0, 1)), ((193, 1255, 71), (2, 1, 0)), ((53, 42, 191, 41), (2, 0, 3, 1)),
             ((27, 90, 5, 21, 67), (1, 0, 2, 4, 3)), ((12, 10, 9, 7, 17, 5, 29), (6, 1, 2, 0, 5, 4, 3)), ((810, 592, 37), (1, 0, 2)),
             ((33, 17, 2969, 11), (0, 2, 3, 1)), ((4099, 4111), (1, 0)), ((3, 5600001), (1, 0)), ((5600001, 3), (1, 0)),
             ((14, 90, 5, 21, 134), (1, 0, 2, 4, 3)), ((9000, 45, 43), (0, 2, 1))]   # batched transposes of small matrices: the write run through its table
    ran = 0
    for shape, perm in cases:
        a = rand(rng, shape, dtype)
        oshape = [shape[p] for p in perm]
        ref = np.empty(oshape, dtype)
        oracle.permute(a, list(range(len(shape))), ref, list(perm))
        out = dev(tf, np.full(oshape, np.nan, dtype))
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Permute(list(range(len(shape))), list(perm)), [list(shape), oshape])
        tf.HipBackend.execute(plan, 1.0, [dev(tf, a)], 0.0, out)
        ran += "perm_kernel" in tf.last_kernel()
        assert out.to_numpy().tobytes() == ref.tobytes(), (shape, perm, tf.last_kernel())
        del a, ref, out
    assert ran >= 4, ran


@pytest.mark.parametrize("dtype", ALL)
def test_permute_two_sided_tiles_of_random_shapes_and_views(tf, oracle, dtype):
    # Seeded random tensors of rank 3..6 with five to twelve million elements and extents off the powers of two, a random
    # axis order each; every other input is a view that leaves out indices at both ends of two axes (rows that do not
    # abut, bases that are not aligned).  The tile planner picks among read runs of one row or of the whole tile,
    # write runs in registers or through the table, ranges that end ragged on one or two axes: whatever it picks, the
    # move is bit-exact against the oracle on an output that starts as NaN.
    rng = seeded_rng(143)
    ran = conj_ran = 0
    for case in range(8):
        rank = int(rng.integers(3, 7))
        target = int(rng.integers(5_000_000, 12_000_000))
        w = rng.dirichlet(np.ones(rank)) * np.log(target)
        shape = [max(3, int(round(np.exp(x)))) | 1 for x in w]
        while int(np.prod(shape)) > 14_000_000:
            shape[int(np.argmax(shape))] = shape[int(np.argmax(shape))] * 3 // 4 | 1
        perm = [int(x) for x in rng.permutation(rank)]
        if perm == list(range(rank)):
            perm = perm[::-1]
        full = rand(rng, shape, dtype)
        a = full
        if case % 2:
            cut = [slice(None)] * rank
            for ax in rng.choice(rank, 2, replace=False):
                if shape[ax] > 8:
                    cut[int(ax)] = slice(1, shape[ax] - 2)
            a = full[tuple(cut)]
        oshape = [a.shape[p] for p in perm]
        ref = np.empty(oshape, dtype)
        oracle.permute(np.ascontiguousarray(a), list(range(rank)), ref, list(perm))
        assert np.array_equal(ref, np.transpose(a, perm))
        out = dev(tf, np.full(oshape, np.nan, dtype))
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Permute(list(range(rank)), list(perm)), [list(a.shape), oshape])
        tf.HipBackend.execute(plan, 1.0, [dev(tf, a)], 0.0, out)
        ran += "perm_kernel" in tf.last_kernel()
        assert out.to_numpy().tobytes() == ref.tobytes(), (shape, perm, case, tf.last_kernel())
        if np.issubdtype(dtype, np.complexfloating) and case % 3 == 0:
            # the same move of an operand behind the conjugate-on-load flag: only the sign of the imaginary parts changes
            out = dev(tf, np.full(oshape, np.nan, dtype))
            tf.HipBackend.execute(plan, 1.0, [dev(tf, a).conj_on_load()], 0.0, out)
            conj_ran += "perm_kernel" in tf.last_kernel()
            assert out.to_numpy().tobytes() == np.conj(ref).tobytes(), (shape, perm, case, tf.last_kernel())
        del full, a, ref, out
    assert ran >= 3, ran
    assert conj_ran >= 1 or not np.issubdtype(dtype, np.complexfloating), conj_ran


@pytest.mark.parametrize("dtype", ALL)
def test_contract_long_operand_against_a_small_one_beyond_the_register_kernel(tf, oracle, dtype):
    # More k (over 32 16-byte chunks) than the register-resident streaming kernel holds against at most 32 real rows, far
    # too thin for tiles: the small operand is staged in LDS as MFMA operands (complex types as the real matrix
    # [[re, -im], [im, re]]) and every wave streams rows of the long one.  Both output orientations, either operand in
    # either position, a long extent that ends on a partly filled unit, k that ends inside a register set, rows that
    # are no multiple of 16, a strided small operand, general alpha / beta, and the conjugate-on-load flags.
    rng = seeded_rng(141)
    cplx = np.issubdtype(dtype, np.complexfloating)
    q = 16 // (np.dtype(dtype).itemsize // (2 if cplx else 1))      # reals per 16-byte chunk
    kq = q // (2 if cplx else 1) or 1                               # elements of k per chunk (1 for complex128)
    mmax = 16 if cplx else 32
    cases = [("nk", "mk", "nm", mmax, 40 * kq, 5000), ("nk", "mk", "mn", mmax, 40 * kq, 5000), ("mk", "nk", "mn", 12, 130 * kq, 4099),
             ("mk", "nk", "nm", 9 if cplx else 17, 36 * kq, 4112), ("nk", "km", "nm", mmax - 3, 64 * kq, 8192),
             ("mk", "nk", "mn", 5, 200 * kq, 6000), ("nk", "mk", "nm", mmax, 8 * kq, 4096 + 16),
             ("nk", "mk", "nm", mmax, 300 * kq, 4200), ("mk", "nk", "mn", mmax - 1, 517 * kq, 4100)]   # over 64 KB: passes over slices of k
    used = 0
    for la, lb, lc, m, k, n in cases:
        ext = dict(m=m, k=k, n=n)
        a = rand(rng, [ext[c] for c in la], dtype)
        b = rand(rng, [ext[c] for c in lb], dtype)
        c0 = rand(rng, [ext[c] for c in lc], dtype)
        for alpha, beta in [(1.0, 0.0), ((0.5 - 2j, 1.5 + 1j) if cplx else (0.5, -1.5))]:
            ref = c0.copy()
            oracle.contract(a, lab(la), b, lab(lb), ref, lab(lc), alpha=alpha, beta=beta)
            dout = dev(tf, c0)
            plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab(la), lab(lb), lab(lc)), [a.shape, b.shape, ref.shape])
            tf.HipBackend.execute(plan, alpha, [dev(tf, a), dev(tf, b)], beta, dout)
            used += "gemm_thin_kernel" in tf.last_kernel()
            assert relerr(dout.to_numpy(), ref) < TOL[dtype], (la, lb, lc, m, k, n, alpha, tf.last_kernel())
    assert used >= 10, used
    # exact on small integers: a misplaced k, a wrong sign in the complex expansion or a dropped chunk would show
    m, k, n = (14 if cplx else 30), 40 * kq, 4100
    def ints(shape):
        x = rng.integers(-4, 5, shape).astype(np.float64)
        return (x + 1j * rng.integers(-4, 5, shape)).astype(dtype) if cplx else x.astype(dtype)
    a, b = ints((n, k)), ints((m, k))
    for conj_a, conj_b in ([(False, False), (True, False), (False, True), (True, True)] if cplx else [(False, False)]):
        out = tf.Tensor.empty([n, m], tf.GpuMemory(0), tf.MemoryOrder.RowMajor, dtype)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("nk"), lab("mk"), lab("nm")), [a.shape, b.shape, [n, m]])
        da, db = dev(tf, a), dev(tf, b)
        tf.HipBackend.execute(plan, 1.0, [da.conj_on_load() if conj_a else da, db.conj_on_load() if conj_b else db], 0.0, out)
        assert "gemm_thin_kernel" in tf.last_kernel(), tf.last_kernel()
        want = np.einsum("nk,mk->nm", a.conj() if conj_a else a, b.conj() if conj_b else b)
        assert np.array_equal(out.to_numpy(), want), (conj_a, conj_b)

"""Pins the CPU oracle (oracle/tfo_oracle.cpp) without the reference, which has no implementation
(tenferro-prims/src/lib.rs:419-439 are todo!()): numpy as an independent library routine, closed
forms, brute force, identities, and the known answers in the reference's doc comments.
Each check is chosen so that a plausible mistake (transposed operand, dropped term, wrong sign,
wrong stride) fails it."""
import itertools

import numpy as np
import pytest

RTOL = {np.float32: 2e-6, np.float64: 1e-13, np.complex64: 2e-6, np.complex128: 1e-13}
ALL = [np.float32, np.float64, np.complex64, np.complex128]


def rand(rng, shape, dtype):
    x = rng.standard_normal(shape)
    if np.issubdtype(dtype, np.complexfloating):
        x = x + 1j * rng.standard_normal(shape)
    return x.astype(dtype)


def relerr(x, ref):
    d = np.linalg.norm((x - ref).ravel())
    n = np.linalg.norm(ref.ravel())
    return d / n if n > 0 else d


LET = "abcdefghijklmnopqrstuvwxyz"


# ---------------------------------------------------------------- permute
@pytest.mark.parametrize("dtype", ALL)
def test_permute_matches_numpy_all_perms_rank4(oracle, dtype):
    rng = np.random.default_rng(1)
    a = rand(rng, (3, 4, 5, 2), dtype)
    for perm in itertools.permutations(range(4)):
        b = np.full([a.shape[p] for p in perm], np.nan, dtype)
        # NumPy convention: output axis n carries label modes_b[n] (tenferro-prims/src/lib.rs:194-202,408-411)
        oracle.permute(a, [0, 1, 2, 3], b, list(perm))
        assert np.array_equal(b, a.transpose(perm))


def test_permute_reference_doc_example_shapes(oracle):
    # tenferro-prims/src/lib.rs:408-415: modes [0,1] -> [1,0], shapes [3,4] -> [4,3]
    a = np.arange(12, dtype=np.float64).reshape(3, 4)
    b = np.empty((4, 3))
    oracle.permute(a, [0, 1], b, [1, 0])
    assert np.array_equal(b, a.T)


def test_permute_bit_exact_index_fill_and_involution(oracle):
    # fill with the linear index: out[idx] must be the gathered input index, bit for bit
    shape = (4, 3, 5, 2, 6)
    a = np.arange(np.prod(shape), dtype=np.float64).reshape(shape)
    perm = (4, 1, 0, 3, 2)
    b = np.empty([shape[p] for p in perm])
    oracle.permute(a, range(5), b, perm)
    for idx in itertools.product(*[range(n) for n in b.shape]):
        src = [0] * 5
        for n, p in enumerate(perm):
            src[p] = idx[n]
        assert b[idx] == a[tuple(src)]
    inv = np.argsort(perm)
    c = np.empty(shape)
    oracle.permute(b, range(5), c, inv)
    assert a.tobytes() == c.tobytes()


def test_permute_special_values_are_copied_bitwise(oracle):
    a = np.array([[0.0, -0.0, np.inf], [-np.inf, np.nan, 5e-324]])
    b = np.empty((3, 2))
    oracle.permute(a, [0, 1], b, [1, 0])
    assert b.tobytes() == np.ascontiguousarray(a.T).tobytes()


@pytest.mark.parametrize("dtype", [np.float64, np.complex128])
def test_permute_strided_negative_and_alpha_beta(oracle, dtype):
    rng = np.random.default_rng(2)
    big = rand(rng, (8, 9, 10), dtype)
    a = big[::2, ::-1, 1:9:3]            # strided, negative stride
    b0 = rand(rng, (a.shape[2], a.shape[0], a.shape[1]), dtype)
    b = b0.copy()
    alpha, beta = (0.5 - 2j, 1.5 + 1j) if np.issubdtype(dtype, np.complexfloating) else (0.5, -1.5)
    oracle.permute(a, [0, 1, 2], b, [2, 0, 1], alpha=alpha, beta=beta)
    assert relerr(b, alpha * a.transpose(2, 0, 1) + beta * b0) < RTOL[dtype]


def test_permute_rejects_bad_modes(oracle):
    a = np.zeros((2, 3))
    with pytest.raises(oracle.OracleError):
        oracle.permute(a, [0, 1], np.zeros((3, 2)), [1, 1])
    with pytest.raises(oracle.OracleError):
        oracle.permute(a, [0, 1], np.zeros((2, 3)), [1, 0])   # extents do not match the labels
    with pytest.raises(oracle.OracleError):
        oracle.permute(a, [0, 1], np.zeros((3,)), [1])


# ---------------------------------------------------------------- reduce
@pytest.mark.parametrize("dtype", ALL)
def test_reduce_sum_matches_numpy(oracle, dtype):
    rng = np.random.default_rng(3)
    a = rand(rng, (4, 5, 6, 3), dtype)
    for keep in [(0,), (1, 3), (3, 0), (2, 1, 0), (), (0, 1, 2, 3)]:
        red = tuple(d for d in range(4) if d not in keep)
        ref = a.astype(np.complex128 if np.iscomplexobj(a) else np.float64).sum(axis=red) if red else a.copy()
        # order the kept axes as requested
        kept_sorted = [d for d in range(4) if d in keep]
        ref = np.asarray(ref).transpose([kept_sorted.index(k) for k in keep]) if keep else np.asarray(ref)
        c = np.full(ref.shape, np.nan, dtype)
        oracle.reduce(a, range(4), c, list(keep))
        assert relerr(c, ref) < RTOL[dtype]


def test_reduce_closed_forms_exact(oracle):
    # all ones -> the number of addends; linear-index fill -> arithmetic series; both exact in f64
    shape = (6, 5, 4, 3)
    ones = np.ones(shape)
    c = np.empty((6, 4))
    oracle.reduce(ones, [0, 1, 2, 3], c, [0, 2])
    assert np.all(c == 15.0)
    a = np.arange(np.prod(shape), dtype=np.float64).reshape(shape)
    oracle.reduce(a, [0, 1, 2, 3], c, [0, 2])
    i, k = np.meshgrid(np.arange(6), np.arange(4), indexing="ij")
    # sum_{j<5, l<3} (i*60 + j*12 + k*3 + l) = 15*(60 i + 3 k) + 12*3*10 + 5*3
    assert np.array_equal(c, 15.0 * (60 * i + 3 * k) + 360 + 15)


def test_reduce_max_min_alpha_beta(oracle):
    rng = np.random.default_rng(4)
    a = rng.standard_normal((7, 8, 9))
    c = np.empty((9, 7))
    oracle.reduce(a, [0, 1, 2], c, [2, 0], op=oracle.MAX)
    assert np.array_equal(c, a.max(axis=1).T)
    oracle.reduce(a, [0, 1, 2], c, [2, 0], op=oracle.MIN)
    assert np.array_equal(c, a.min(axis=1).T)
    c0 = rng.standard_normal((9, 7))
    c = c0.copy()
    oracle.reduce(a, [0, 1, 2], c, [2, 0], alpha=2.0, beta=-0.5)
    assert relerr(c, 2.0 * a.sum(axis=1).T - 0.5 * c0) < 1e-14
    with pytest.raises(oracle.OracleError):
        oracle.reduce(a.astype(np.complex128), [0, 1, 2], np.empty((9, 7), np.complex128), [2, 0], op=oracle.MAX)
    with pytest.raises(oracle.OracleError):
        oracle.reduce(a, [0, 1, 2], c, [2, 5])


# ---------------------------------------------------------------- contract
CASES = [
    # (modes_a, modes_b, modes_c, extents)
    ("mk", "kn", "mn", dict(m=37, k=53, n=29)),
    ("km", "nk", "nm", dict(m=20, k=300, n=17)),
    ("bmk", "bkn", "bmn", dict(b=3, m=10, k=11, n=12)),
    ("ajbk", "kcj", "abc", dict(a=4, j=8, b=5, k=6, c=7)),          # the config-1 pattern
    ("awc", "asx", "wcsx", dict(a=9, w=3, c=5, s=2, x=7)),         # config-3 step 1
    ("mk", "k", "m", dict(m=13, k=300)),                           # matrix-vector
    ("i", "i", "", dict(i=1000)),                                  # dot product
    ("i", "j", "ij", dict(i=19, j=23)),                            # outer product
    ("bij", "jk", "bik", dict(b=4, i=3, j=4, k=5)),                # broadcast batch (einsum/src/lib.rs:88-93)
    ("abij", "abjk", "abik", dict(a=2, b=3, i=4, j=5, k=6)),       # two batch dims (:82-86)
    ("xmk", "kn", "mn", dict(x=4, m=6, k=7, n=5)),                 # x only in A: summed
]


@pytest.mark.parametrize("dtype", ALL)
@pytest.mark.parametrize("case", CASES, ids=[c[0] + "," + c[1] + "->" + c[2] for c in CASES])
def test_contract_matches_numpy_einsum(oracle, dtype, case):
    ma, mb, mc, ext = case
    rng = np.random.default_rng(5)
    a = rand(rng, [ext[l] for l in ma], dtype)
    b = rand(rng, [ext[l] for l in mb], dtype)
    wide = np.complex128 if np.iscomplexobj(a) else np.float64
    ref = np.einsum(f"{ma},{mb}->{mc}", a.astype(wide), b.astype(wide))
    lab = lambda s: [ord(ch) for ch in s]
    c = np.full([ext[l] for l in mc], np.nan, dtype)
    oracle.contract(a, lab(ma), b, lab(mb), c, lab(mc))
    assert relerr(c, ref) < RTOL[dtype]
    c2 = np.full([ext[l] for l in mc], np.nan, dtype)
    oracle.contract(a, lab(ma), b, lab(mb), c2, lab(mc), naive=True)
    assert relerr(c2, ref) < RTOL[dtype]


@pytest.mark.parametrize("dtype", ALL)
def test_contract_integer_inputs_exact_blocked_vs_brute_force(oracle, dtype):
    # small integers: every product and partial sum is exactly representable, so the blocked
    # evaluator, the brute-force evaluator and numpy must agree bit for bit
    rng = np.random.default_rng(6)
    def ints(shape):
        x = rng.integers(-3, 4, shape).astype(np.float64)
        if np.issubdtype(dtype, np.complexfloating):
            x = x + 1j * rng.integers(-3, 4, shape)
        return x.astype(dtype)
    a, b = ints((23, 31, 4)), ints((31, 4, 19))
    c1 = np.empty((4, 23, 19), dtype)
    c2 = np.empty((4, 23, 19), dtype)
    oracle.contract(a, [0, 1, 2], b, [1, 2, 3], c1, [2, 0, 3])
    oracle.contract(a, [0, 1, 2], b, [1, 2, 3], c2, [2, 0, 3], naive=True)
    ref = np.einsum("mkb,kbn->bmn", a, b)
    assert np.array_equal(c1, c2) and np.array_equal(c1, ref.astype(dtype))


@pytest.mark.parametrize("dtype", [np.float64, np.complex128])
def test_contract_identities_alpha_beta_strides(oracle, dtype):
    rng = np.random.default_rng(7)
    a = rand(rng, (12, 9), dtype)
    eye = np.eye(9, dtype=dtype)
    c = np.empty((12, 9), dtype)
    oracle.contract(a, [0, 1], eye, [1, 2], c, [0, 2])
    assert np.array_equal(c, a)                                           # A.I = A
    b = rand(rng, (9, 7), dtype)
    ab = np.empty((12, 7), dtype)
    bta = np.empty((7, 12), dtype)
    oracle.contract(a, [0, 1], b, [1, 2], ab, [0, 2])
    oracle.contract(b.T, [2, 1], a.T, [1, 0], bta, [2, 0])                # (AB)^T = B^T A^T, transposed views
    assert relerr(bta.T, ab) < 1e-14
    # non-commuting complex alpha/beta, strided + negative-stride operands, accumulate into c0
    alpha, beta = (0.7 - 1.1j, -0.3 + 0.2j) if np.iscomplexobj(a) else (0.7, -0.3)
    big = rand(rng, (24, 18), dtype)
    av = big[::2, ::-2]
    c0 = rand(rng, (12, 7), dtype)
    c = c0.copy()
    oracle.contract(av, [0, 1], b, [1, 2], c, [0, 2], alpha=alpha, beta=beta)
    assert relerr(c, alpha * (av @ b) + beta * c0) < 1e-13
    # broadcast operand (stride 0)
    row = rand(rng, (1, 9), dtype)
    bc = np.broadcast_to(row, (12, 9))
    oracle.contract(bc, [0, 1], b, [1, 2], c, [0, 2])
    assert relerr(c, bc @ b) < 1e-13


def test_contract_complex_sign_conventions(oracle):
    # (a+ib)(c+id) on Gaussian integers is exact; a wrong sign on the imaginary cross terms fails
    a = np.array([[1 + 2j, 3 - 1j]], np.complex128)
    b = np.array([[2 - 1j], [-1 + 4j]], np.complex128)
    c = np.empty((1, 1), np.complex128)
    oracle.contract(a, [0, 1], b, [1, 2], c, [0, 2])
    assert c[0, 0] == (1 + 2j) * (2 - 1j) + (3 - 1j) * (-1 + 4j)
    x = np.array([1 + 2j, -3 + 0.5j])
    xc = np.empty_like(x)
    oracle.conj(x, xc)
    d = np.empty((), np.complex128)
    oracle.contract(x, [0], xc, [0], d, [])
    assert d.imag == 0 and d.real == 1 + 4 + 9 + 0.25


def test_contract_errors(oracle):
    a, b = np.zeros((3, 4)), np.zeros((5, 6))
    with pytest.raises(oracle.OracleError):
        oracle.contract(a, [0, 1], b, [1, 2], np.zeros((3, 6)), [0, 2])       # k extents differ
    with pytest.raises(oracle.OracleError):
        oracle.contract(a, [0, 1], np.zeros((4, 6)), [1, 2], np.zeros((3, 6)), [0, 9])  # label 9 nowhere
    with pytest.raises(oracle.OracleError):
        oracle.contract(a, [0, 0], np.zeros((4, 6)), [1, 2], np.zeros((3, 6)), [0, 2])  # repeated label


@pytest.mark.parametrize("dtype", ALL)
def test_batched_gemm_matches_matmul(oracle, dtype):
    rng = np.random.default_rng(8)
    a, b = rand(rng, (2, 3, 5, 7), dtype), rand(rng, (2, 3, 7, 4), dtype)
    c = np.full((2, 3, 5, 4), np.nan, dtype)
    oracle.batched_gemm(a, b, c, n_batch=2)
    wide = np.complex128 if np.iscomplexobj(a) else np.float64
    assert relerr(c, a.astype(wide) @ b.astype(wide)) < RTOL[dtype]
    a2, b2 = rand(rng, (3, 4), dtype), rand(rng, (4, 5), dtype)   # tenferro-prims/src/lib.rs:266-269 shapes
    c2 = np.empty((3, 5), dtype)
    oracle.batched_gemm(a2, b2, c2, n_batch=0)
    assert relerr(c2, a2.astype(wide) @ b2.astype(wide)) < RTOL[dtype]


# ---------------------------------------------------------------- elementwise, conj, trace family
@pytest.mark.parametrize("dtype", ALL)
def test_elementwise_mul_and_conj(oracle, dtype):
    rng = np.random.default_rng(9)
    a, b = rand(rng, (5, 6, 7), dtype), rand(rng, (5, 6, 7), dtype)
    c0 = rand(rng, (5, 6, 7), dtype)
    c = c0.copy()
    oracle.elementwise_mul(a.transpose(0, 1, 2), b, c, alpha=2.0, beta=1.0)
    assert relerr(c, 2 * a * b + c0) < RTOL[dtype]
    bt = rand(rng, (7, 6, 5), dtype).transpose(2, 1, 0)      # permuted operand, broadcast operand
    row = np.broadcast_to(rand(rng, (1, 1, 7), dtype), (5, 6, 7))
    c = np.full((5, 6, 7), np.nan, dtype)
    oracle.elementwise_mul(bt, row, c)
    assert relerr(c, bt * row) < RTOL[dtype]
    out = np.empty_like(a)
    oracle.conj(a, out)
    assert np.array_equal(out, np.conj(a))


def test_conj_reference_doc_example(oracle):
    # tenferro-tensor/src/lib.rs:612-620: conj([1+2i, 3-4i]) = [1-2i, 3+4i]
    a = np.array([1 + 2j, 3 - 4j])
    out = np.empty_like(a)
    oracle.conj(a, out)
    assert np.array_equal(out, np.array([1 - 2j, 3 + 4j]))


@pytest.mark.parametrize("dtype", [np.float64, np.complex128])
def test_trace_anti_trace_anti_diag(oracle, dtype):
    rng = np.random.default_rng(10)
    a = rand(rng, (4, 5, 4, 3), dtype)                       # modes i=0, k=1, j=2, l=3
    c = np.full((3, 5), np.nan, dtype)
    oracle.trace(a, [0, 1, 2, 3], c, [3, 1], pairs=[(0, 2)])
    assert relerr(c, np.einsum("ikil->lk", a)) < 1e-14
    sq = rand(rng, (6, 6), dtype)
    s = np.empty((), dtype)
    oracle.trace(sq, [0, 1], s, [], pairs=[(0, 1)])
    assert abs(s - np.trace(sq)) < 1e-13
    # AntiTrace is the adjoint of Trace: <trace(A), G> == <A, anti_trace(G)>
    g = rand(rng, (3, 5), dtype)
    back = np.full((4, 5, 4, 3), np.nan, dtype)
    oracle.anti_trace(g, [3, 1], back, [0, 1, 2, 3], pairs=[(0, 2)])
    ref = np.zeros((4, 5, 4, 3), dtype)
    for i in range(4):
        ref[i, :, i, :] = g.T
    assert np.array_equal(back, ref)
    assert abs(np.vdot(c, g) - np.vdot(a, back)) < 1e-12
    # AntiDiag: adjoint of "ii->i" -- C[i,j] = delta_ij A[i]
    v = rand(rng, (5,), dtype)
    m = np.full((5, 5), np.nan, dtype)
    oracle.anti_diag(v, [0], m, [0, 1], pairs=[(0, 1)])
    assert np.array_equal(m, np.diag(v))
    m0 = rand(rng, (5, 5), dtype)
    m = m0.copy()
    oracle.anti_diag(v, [0], m, [0, 1], pairs=[(0, 1)], alpha=2.0, beta=1.0)
    assert relerr(m, 2 * np.diag(v) + m0) < 1e-14


# ---------------------------------------------------------------- einsum
PATTERNS = ["ij,jk->ik", "ii->", "i,j->ij", "i,i->", "ij,j->i", "ii->i", "ijk->", "bij,bjk->bik",
            "abij,abjk->abik", "bij,jk->bik", "ij,jk,kl->il", "ij->ji", "ij,ij->ij", "iij,jk->ik"]


@pytest.mark.parametrize("dtype", [np.float64, np.complex128])
@pytest.mark.parametrize("pattern", PATTERNS)
def test_einsum_naive_matches_numpy_catalogue(oracle, dtype, pattern):
    # the pattern catalogue of tenferro-einsum/src/lib.rs:37-93
    rng = np.random.default_rng(11)
    ext = {l: n for l, n in zip("ijklab", (3, 4, 5, 6, 2, 3))}
    ext["b"] = 3
    ins, out = pattern.split("->")
    ops = [rand(rng, [ext[l] for l in term], dtype) for term in ins.split(",")]
    ref = np.einsum(pattern, *ops)
    res = np.full(np.shape(ref), np.nan, dtype)
    oracle.einsum_naive(ops, [[ord(l) for l in t] for t in ins.split(",")], res, [ord(l) for l in out])
    assert relerr(res, ref) < 1e-13


def test_einsum_naive_output_diagonals_reference_doc_examples(oracle):
    # tenferro-einsum/src/lib.rs:52-63: "i->ii" of v=[1,2,3] is diag(1,2,3) with dims [3,3]; "i->iii" dims [3,3,3]
    v = np.array([1.0, 2.0, 3.0])
    d = np.full((3, 3), np.nan)
    oracle.einsum_naive([v], [[0]], d, [0, 0])
    assert np.array_equal(d, np.diag(v))
    t = np.full((3, 3, 3), np.nan)
    oracle.einsum_naive([v], [[0]], t, [0, 0, 0])
    ref = np.zeros((3, 3, 3))
    for i in range(3):
        ref[i, i, i] = v[i]
    assert np.array_equal(t, ref)


@pytest.mark.parametrize("dtype", [np.float64, np.complex128])
def test_einsum_pairs_every_order_matches_numpy(oracle, dtype):
    # a 4-operand network shaped like the MPS-MPO environment update, tiny extents
    rng = np.random.default_rng(12)
    ext = dict(a=5, c=4, x=3, y=6, w=2, v=3, s=2, t=2)
    terms = ["awc", "asx", "wstv", "cty"]
    out = "xvy"
    ops = [rand(rng, [ext[l] for l in t], dtype) for t in terms]
    ref = np.einsum(",".join(terms) + "->" + out, *ops)
    lab = [[ord(l) for l in t] for t in terms]
    orders = [[(0, 1), (4, 2), (5, 3)], [(0, 2), (1, 4), (5, 3)], [(1, 2), (0, 3), (4, 5)],
              [(2, 3), (0, 1), (4, 5)], [(0, 3), (4, 2), (5, 1)]]
    for pairs in orders:
        res = np.full(ref.shape, np.nan, dtype)
        oracle.einsum_pairs(ops, lab, res, [ord(l) for l in out], pairs)
        assert relerr(res, ref) < 1e-13, pairs
    naive = np.full(ref.shape, np.nan, dtype)
    oracle.einsum_naive(ops, lab, naive, [ord(l) for l in out])
    assert relerr(naive, ref) < 1e-13
    r0 = rand(rng, ref.shape, dtype)
    res = r0.copy()
    oracle.einsum_pairs(ops, lab, res, [ord(l) for l in out], orders[0], alpha=2.0, beta=-1.0)
    assert relerr(res, 2 * ref - r0) < 1e-13
    with pytest.raises(oracle.OracleError):
        oracle.einsum_pairs(ops, lab, res, [ord(l) for l in out], [(0, 1), (0, 2), (5, 3)])   # operand 0 reused


def test_beta_zero_never_reads_the_output(oracle):
    # NaN-poisoned outputs: beta == 0 must overwrite (tenferro-prims/src/lib.rs:306-309)
    rng = np.random.default_rng(13)
    a, b = rng.standard_normal((6, 7)), rng.standard_normal((7, 5))
    c = np.full((6, 5), np.nan)
    oracle.contract(a, [0, 1], b, [1, 2], c, [0, 2])
    assert np.isfinite(c).all()
    r = np.full((6,), np.nan)
    oracle.reduce(a, [0, 1], r, [0])
    assert np.isfinite(r).all()
    e = np.full((6, 7), np.nan)
    oracle.elementwise_mul(a, a, e)
    assert np.isfinite(e).all()
    p = np.full((7, 6), np.nan)
    oracle.permute(a, [0, 1], p, [1, 0], alpha=2.0)
    assert np.isfinite(p).all()


# ------------------------------------------------------------------------------------------------ f32 under cancellation
def lab(s):
    return [ord(c) for c in s]


def _cancelling():
    import os
    return np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "cancelling_f32.npz"))


def test_f32_cancelling_sums_blocked_path_within_the_rounding_bound_and_brute_force_exact(oracle):
    # tests/golden/cancelling_f32.npz: thirty f32 terms whose sum is 1/1428 of the sum of their magnitudes, with the
    # exact result from numpy in f64.  The blocked path adds f32 products in f32 inside a cache block: its error is
    # bounded by (k + 2) * 2^-24 * sum|a||b| -- and on the first case it is 2.2e-5 of the result, i.e. this path cannot
    # meet a 1e-5 tolerance that is measured against a cancelled result.  The brute-force path (long double) is exact.
    fx = _cancelling()
    alpha = float(fx["alpha"])
    for a, ma, b, mb, mc, exact, scale in [(fx["dot_a"], "dc", fx["dot_b"], "dc", "", fx["dot_exact"], fx["dot_abs"]),
                                           (fx["mat_a"], "fdc", fx["mat_b"], "dce", "fe", fx["mat_exact"], fx["mat_abs"])]:
        shape = [dict(zip(ma + mb, a.shape + b.shape))[l] for l in mc]
        got = np.empty(shape, np.float32)
        oracle.contract(a, lab(ma), b, lab(mb), got, lab(mc), alpha=alpha)
        assert np.linalg.norm(got - exact) <= 32 * 2.0 ** -24 * np.linalg.norm(scale)
        gold = np.empty(shape, np.float32)
        oracle.contract(a, lab(ma), b, lab(mb), gold, lab(mc), alpha=alpha, naive=True)
        assert np.all(np.abs(gold - exact) <= 2.0 ** -23 * np.abs(exact))
    got = np.empty([], np.float32)
    oracle.contract(fx["dot_a"], lab("dc"), fx["dot_b"], lab("dc"), got, [], alpha=alpha)
    assert 1e-5 < abs(float(got) - float(fx["dot_exact"])) / abs(float(fx["dot_exact"])) < 1e-4


@pytest.mark.parametrize("dtype", [np.float32, np.complex64])
def test_f32_alpha_beta_epilogue_is_exact_on_dyadic_cancelling_sums(oracle, dtype):
    # quarter-integers in [-2, 2]: every product, partial sum and the alpha/beta combination below is exactly
    # representable in f32, so whatever the order of additions the blocked path must return numpy's f64 result bit for
    # bit -- a wrong sign, a dropped beta term or alpha applied twice cannot hide behind rounding.  Columns of B are
    # arranged in +/- pairs so that most sums cancel to small values.
    rng = np.random.default_rng(77)
    m, n, k = 37, 29, 96
    def draw(shape):
        x = rng.integers(-8, 9, shape).astype(np.float64) / 4.0
        if np.issubdtype(dtype, np.complexfloating):
            x = x + 1j * rng.integers(-8, 9, shape).astype(np.float64) / 4.0
        return x
    a = draw((m, k))
    a[:, k // 2:] = a[:, :k // 2]                 # a row is its first half twice ...
    b = draw((k, n))
    b[k // 2:, : n // 2] = -b[:k // 2, : n // 2]  # ... and the left columns of B change sign half way: those sums are exactly 0
    c0 = draw((m, n))
    alpha, beta = (0.5 - 0.25j, -0.25 + 2j) if np.issubdtype(dtype, np.complexfloating) else (0.5, -0.25)
    want = (alpha * (a @ b) + beta * c0).astype(dtype)
    assert np.all((a @ b)[:, : n // 2] == 0)
    got = c0.astype(dtype)
    oracle.contract(a.astype(dtype), lab("mk"), b.astype(dtype), lab("kn"), got, lab("mn"), alpha=alpha, beta=beta)
    assert got.tobytes() == want.tobytes()


# ------------------------------------------------------------------------------------------------ several cache blocks, all threads
@pytest.mark.parametrize("dtype", [np.float64, np.complex128, np.float32])
def test_contract_blocked_path_across_cache_blocks_against_numpy(oracle, dtype):
    # 700 x 1100 x 900: several blocks along every loop of the blocked kernel (with edge blocks that are not full),
    # all threads at work -- the code path that produces the full-size references of the benchmark.  numpy's matmul (BLAS)
    # is the independent check; f32 is compared with the f64 product rounded once.
    rng = np.random.default_rng(91)
    m, k, n = 700, 1100, 900
    a = rng.standard_normal((m, k))
    b = rng.standard_normal((k, n))
    if np.issubdtype(dtype, np.complexfloating):
        a = a + 1j * rng.standard_normal((m, k))
        b = b + 1j * rng.standard_normal((k, n))
    a, b = a.astype(dtype), b.astype(dtype)
    c0 = rng.standard_normal((m, n)).astype(dtype)
    wide = np.complex128 if np.issubdtype(dtype, np.complexfloating) else np.float64
    want = 0.5 * (a.astype(wide) @ b.astype(wide)) - 1.5 * c0.astype(wide)
    got = c0.copy()
    oracle.contract(a, lab("mk"), b, lab("kn"), got, lab("mn"), alpha=0.5, beta=-1.5)
    err = np.linalg.norm(got - want) / np.linalg.norm(want)
    assert err < (2e-6 if dtype == np.float32 else 1e-14), err
    # transposed storage of both operands and of the output (the packing routines' other branches)
    got_t = np.asfortranarray(c0.copy())
    oracle.contract(np.asfortranarray(a), lab("mk"), np.asfortranarray(b), lab("kn"), got_t, lab("mn"), alpha=0.5, beta=-1.5)
    assert np.linalg.norm(got_t - want) / np.linalg.norm(want) < (2e-6 if dtype == np.float32 else 1e-14)


def test_contract_benchmark_pattern_with_fused_groups_against_numpy(oracle):
    # "ajbk,kcj->abc" with a = 16 (the f32 benchmark configuration at a quarter of its rows): fused row and k groups
    # with different orders in the two operands, K = 12288 over many cache blocks; against numpy's einsum in f64
    rng = np.random.default_rng(92)
    a_, j, b_, k, c = 16, 128, 64, 96, 256
    A = rng.standard_normal((a_, j, b_, k)).astype(np.float32)
    B = rng.standard_normal((k, c, j)).astype(np.float32)
    want = np.einsum("ajbk,kcj->abc", A.astype(np.float64), B.astype(np.float64), optimize=True)
    got = np.empty((a_, b_, c), np.float32)
    oracle.contract(A, lab("ajbk"), B, lab("kcj"), got, lab("abc"))
    err = np.linalg.norm(got - want) / np.linalg.norm(want)
    assert err < 2e-6, err   # f32 accumulation inside a cache block, f64 across blocks

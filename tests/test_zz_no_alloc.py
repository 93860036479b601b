"""tfh_execute_static -- TensorPrims::execute without device allocations (its scratch is a fixed array inside the
library) -- against tfh_execute on the same inputs, through the C ABI.  Both run the same kernels with the same
splits in the same order, so the results must agree bit for bit; each case makes two calls in a row, the second on a
smaller input, because every call on a device reuses the one array and finds the previous call's contents in it."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TOL = {np.float32: 1e-5, np.float64: 1e-12, np.complex64: 1e-5, np.complex128: 1e-12}


@pytest.fixture(scope="module")
def tf():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import tenferro_rs_amd as tf
    tf.lib()
    return tf


def lab(s):
    return [ord(c) for c in s]


def gpu(tf, x):
    import torch
    return tf.Tensor.from_torch(torch.from_numpy(np.ascontiguousarray(x)).cuda())


def relerr(x, ref):
    return np.linalg.norm((x - ref).ravel()) / np.linalg.norm(ref.ravel())


def both_ways(tf, plan, alpha, ins, beta, out0):
    """Runs the plan through tfh_execute and through tfh_execute_static from the same initial output; returns both."""
    import torch
    o1, o2 = gpu(tf, out0), gpu(tf, out0)
    d_ins = [gpu(tf, x) for x in ins]
    tf.HipBackend.execute(plan, alpha, d_ins, beta, o1)
    k1 = tf.last_kernel()
    tf.HipBackend.execute_static(plan, alpha, d_ins, beta, o2)
    k2 = tf.last_kernel()
    torch.cuda.synchronize()
    assert k1 == k2
    return o1.to_numpy(), o2.to_numpy(), k1


def test_static_scratch_size_is_the_declared_one(tf):
    assert tf.lib().tfh_static_scratch_bytes() == 64 << 20


@pytest.mark.parametrize("dtype", [np.float32, np.complex128])
def test_contract_split_k_tables_and_packing_two_calls(tf, oracle, dtype):
    # "ajbk,kcj->abc": multi-axis row and k groups (offset tables) and a long k over few tiles (split-K partials); the
    # second call is smaller, so it finds the larger call's tables and partials in the array
    rng = np.random.default_rng(7)
    for (a, j, b, k, c) in [(16, 64, 16, 48, 160), (8, 32, 12, 24, 96)]:
        A = rng.standard_normal((a, j, b, k)).astype(dtype)
        B = rng.standard_normal((k, c, j)).astype(dtype)
        if np.iscomplexobj(A):
            A = A + 1j * rng.standard_normal(A.shape).astype(dtype)
            B = B + 1j * rng.standard_normal(B.shape).astype(dtype)
        C0 = rng.standard_normal((a, b, c)).astype(dtype)
        plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab("ajbk"), lab("kcj"), lab("abc")), [A.shape, B.shape, C0.shape])
        for alpha, beta in [(1.0, 0.0), (0.5, -1.5)]:
            r1, r2, kern = both_ways(tf, plan, alpha, [A, B], beta, C0)
            assert r1.tobytes() == r2.tobytes(), (kern, a, alpha)
            ref = C0.copy()
            oracle.contract(A, lab("ajbk"), B, lab("kcj"), ref, lab("abc"), alpha=alpha, beta=beta)
            assert relerr(r2.astype(np.complex128), ref) < TOL[dtype]


def test_reduce_split_partials_two_calls(tf, oracle):
    # few outputs over a long reduction: the serial range is split over blocks, partials go through the scratch
    rng = np.random.default_rng(8)
    for shape in [(4, 1 << 20), (3, 70001)]:
        A = rng.standard_normal(shape)
        C0 = np.zeros(shape[0])
        plan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Reduce([0, 1], [0], tf.ReduceOp.Sum), [A.shape, C0.shape])
        r1, r2, kern = both_ways(tf, plan, 1.0, [A], 0.0, C0)
        assert r1.tobytes() == r2.tobytes(), kern
        ref = C0.copy()
        oracle.reduce(A, [0, 1], ref, [0])
        assert relerr(r2, ref) < 1e-12


def test_permute_and_matrix_vector_two_calls(tf, oracle):
    rng = np.random.default_rng(9)
    for n in [48, 20]:
        A = rng.standard_normal((n, 16, n, 8))
        out = np.zeros((8, n, 16, n))
        plan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Permute([0, 1, 2, 3], [3, 2, 1, 0]), [A.shape, out.shape])
        r1, r2, _ = both_ways(tf, plan, 1.0, [A], 0.0, out)
        assert r1.tobytes() == r2.tobytes() == np.ascontiguousarray(A.transpose(3, 2, 1, 0)).tobytes()
    for (m, k) in [(8, 300000), (5, 4099)]:   # vector . matrix with a long k: split reduction of a product
        A = rng.standard_normal((m, k))
        x = rng.standard_normal(k)
        y0 = np.zeros(m)
        plan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Contract(lab("mk"), lab("k"), lab("m")), [A.shape, x.shape, y0.shape])
        r1, r2, kern = both_ways(tf, plan, 1.0, [A, x], 0.0, y0)
        assert r1.tobytes() == r2.tobytes(), kern
        assert relerr(r2, A @ x) < 1e-12


def test_more_scratch_than_the_array_is_an_error_and_the_next_call_works(tf, oracle):
    import torch
    # 2304 x 2304 x 8192 f64: 324 tiles of 128 x 128 fill 63 % of one round, so k is split and the partials take
    # a multiple of 42 MB -- more than the array holds
    M = N = 2304
    K = 8192
    A = tf.Tensor.from_torch(torch.randn(M, K, dtype=torch.float64, device="cuda"))
    B = tf.Tensor.from_torch(torch.randn(K, N, dtype=torch.float64, device="cuda"))
    Cd = tf.Tensor.from_torch(torch.zeros(M, N, dtype=torch.float64, device="cuda"))
    plan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Contract(lab("mk"), lab("kn"), lab("mn")), [[M, K], [K, N], [M, N]])
    with pytest.raises(tf.InvalidArgument, match="static scratch"):
        tf.HipBackend.execute_static(plan, 1.0, [A, B], 0.0, Cd)
    torch.cuda.synchronize()
    rng = np.random.default_rng(10)
    a = rng.standard_normal((40, 1000))
    b = rng.standard_normal((1000, 50))
    c0 = np.zeros((40, 50))
    p2 = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Contract(lab("mk"), lab("kn"), lab("mn")), [a.shape, b.shape, c0.shape])
    r1, r2, _ = both_ways(tf, p2, 1.0, [a, b], 0.0, c0)
    assert r1.tobytes() == r2.tobytes()
    assert relerr(r2, a @ b) < 1e-12


def test_static_call_leaves_free_device_memory_unchanged(tf):
    # on a stream the library has never seen (no cached workspace for it), a split-K contraction through the static
    # entry point must not change the device's free memory; the same call through tfh_execute allocates its workspace
    import ctypes
    import torch
    st = ctypes.c_void_p()
    assert tf.lib().tfh_stream_create(ctypes.byref(st)) == 0
    try:
        M, N, K = 256, 256, 1 << 15
        A = tf.Tensor.from_torch(torch.randn(M, K, dtype=torch.float64, device="cuda"))
        B = tf.Tensor.from_torch(torch.randn(K, N, dtype=torch.float64, device="cuda"))
        C1 = tf.Tensor.from_torch(torch.zeros(M, N, dtype=torch.float64, device="cuda"))
        C2 = tf.Tensor.from_torch(torch.zeros(M, N, dtype=torch.float64, device="cuda"))
        plan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Contract(lab("mk"), lab("kn"), lab("mn")), [[M, K], [K, N], [M, N]])
        torch.cuda.synchronize()
        # the first launches on a new stream make the HIP runtime set up the stream itself (queue, kernel-argument
        # memory): one unmeasured call takes that out of the comparison
        tf.HipBackend.execute_static(plan, 1.0, [A, B], 0.0, C1, stream=st.value)
        assert tf.lib().tfh_stream_synchronize(st) == 0
        free0 = torch.cuda.mem_get_info()[0]
        tf.HipBackend.execute_static(plan, 1.0, [A, B], 0.0, C1, stream=st.value)
        assert tf.lib().tfh_stream_synchronize(st) == 0
        free1 = torch.cuda.mem_get_info()[0]
        assert free1 == free0
        tf.HipBackend.execute(plan, 1.0, [A, B], 0.0, C2, stream=st.value)
        assert tf.lib().tfh_stream_synchronize(st) == 0
        free2 = torch.cuda.mem_get_info()[0]
        assert free2 < free1   # the ordinary entry point took a workspace for this stream: the check above can see one
        assert C1.to_numpy().tobytes() == C2.to_numpy().tobytes()
    finally:
        tf.lib().tfh_release_workspaces()
        tf.lib().tfh_stream_destroy(st)

"""Golden vectors (tests/golden/cases.{json,npz}, written by tests/golden/make_fixtures.py from numpy alone).

Without a GPU: the CPU oracle reproduces every vector, so the oracle and the fixtures pin each other through an
independent library.  On the GPU: the HIP backend, through the C ABI, reproduces the same vectors.
Data movement (permute, conj) and the exactly representable f32 cases are compared bit for bit; the rest by
relative Frobenius error (1e-12 for f64/complex128, 1e-5 for f32/complex64)."""
import json
import os

import numpy as np
import pytest

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DT = {"f32": np.float32, "f64": np.float64, "c64": np.complex64, "c128": np.complex128}
TOL = {"f32": 1e-5, "f64": 1e-12, "c64": 1e-5, "c128": 1e-12}

with open(os.path.join(HERE, "cases.json")) as _f:
    CASES = json.load(_f)
_NPZ = np.load(os.path.join(HERE, "cases.npz"))          # allow_pickle stays False: arrays only


def _label(case):
    what = case.get("subscripts") or case.get("op") or ""
    return f"{case['id']}-{case['kind']}-{what}-{case['dtype']}"


def _load(case):
    cid = case["id"]
    ins = [_NPZ[f"{cid}_in{i}"] for i in range(case["n_inputs"])]
    before = _NPZ[f"{cid}_before"] if f"{cid}_before" in _NPZ.files else None
    return ins, before, _NPZ[f"{cid}_expected"]


def _scalars(case):
    cplx = case["dtype"] in ("c64", "c128")
    mk = (lambda p: complex(p[0], p[1])) if cplx else (lambda p: float(p[0]))
    return mk(case["alpha"]), mk(case["beta"])


def _compare(case, got, expected):
    assert got.shape == expected.shape and got.dtype == expected.dtype
    if case["kind"] in ("permute", "conj") or case.get("exact"):
        assert got.tobytes() == expected.tobytes()
        return
    if case["kind"] == "reduce" and case["op"] in ("max", "min"):
        assert np.array_equal(got, expected)
        return
    d = np.linalg.norm((got.astype(np.complex128) - expected).ravel())
    n = np.linalg.norm(expected.ravel())
    assert (d / n if n > 0 else d) < TOL[case["dtype"]]


def _labels(sub):
    ins, out = sub.replace("(", "").replace(")", "").split("->")
    return [[ord(c) for c in t] for t in ins.split(",")], [ord(c) for c in out]


def test_fixture_files_are_consistent():
    assert len(CASES) > 100
    for case in CASES:
        ins, before, expected = _load(case)
        assert all(x.dtype == DT[case["dtype"]] for x in ins) and expected.dtype == DT[case["dtype"]]
        assert before is None or before.shape == expected.shape
    # the shape-level known answers of the reference's doc comments hold in the vectors
    # (tenferro-einsum/src/lib.rs:52-55, :60-63, :76-93)
    by_sub = {}
    for case in CASES:
        if case["kind"] == "einsum":
            by_sub.setdefault(case["subscripts"], _load(case)[2].shape)
    assert by_sub["i->ii"] == (3, 3) and by_sub["i->iii"] == (3, 3, 3)
    assert by_sub["bij,bjk->bik"] == (10, 3, 5) and by_sub["bij,jk->bik"] == (10, 3, 5)
    assert by_sub["abij,abjk->abik"] == (2, 3, 4, 6)


# ------------------------------------------------------------------------------------------------ CPU oracle
@pytest.mark.parametrize("case", CASES, ids=_label)
def test_oracle_reproduces_golden_vector(oracle, case):
    ins, before, expected = _load(case)
    alpha, beta = _scalars(case)
    out = np.array(before, copy=True) if before is not None else np.full(expected.shape, np.nan, expected.dtype)
    kind = case["kind"]
    if kind == "einsum":
        in_labels, out_labels = _labels(case["subscripts"])
        oracle.einsum_naive(ins, in_labels, out, out_labels, alpha=alpha, beta=beta)
    elif kind == "permute":
        oracle.permute(ins[0], case["modes_a"], out, case["modes_b"])
    elif kind == "reduce":
        op = {"sum": oracle.SUM, "max": oracle.MAX, "min": oracle.MIN}[case["op"]]
        oracle.reduce(ins[0], case["modes_a"], out, case["modes_c"], op=op)
    elif kind == "batched_gemm":
        oracle.batched_gemm(ins[0], ins[1], out, n_batch=len(case["batch_dims"]), alpha=alpha, beta=beta)
    elif kind == "elementwise_mul":
        oracle.elementwise_mul(ins[0], ins[1], out, alpha=alpha, beta=beta)
    elif kind == "trace":
        oracle.trace(ins[0], case["modes_a"], out, case["modes_c"], pairs=[tuple(p) for p in case["paired"]])
    elif kind == "conj":
        oracle.conj(ins[0], out)
    else:
        raise AssertionError(kind)
    _compare(case, out, expected)


# ------------------------------------------------------------------------------------------------ HIP backend
@pytest.fixture(scope="module")
def tf():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import tenferro_rs_amd as tf
    tf.lib()
    return tf


def _dev(tf, arr):
    return tf.Tensor.from_slice(arr, list(arr.shape), tf.MemoryOrder.RowMajor).to_memory_space_async(tf.GpuMemory(0))


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES, ids=_label)
def test_hip_backend_reproduces_golden_vector(tf, case):
    ins, before, expected = _load(case)
    alpha, beta = _scalars(case)
    dt, kind = DT[case["dtype"]], case["kind"]
    gpu = tf.GpuMemory(0)
    dins = [_dev(tf, x) for x in ins]
    if kind == "einsum" and before is None:
        out = tf.einsum(case["subscripts"], dins)
        assert out.dims() == list(expected.shape)
        _compare(case, np.array(out.to_numpy(), order="C"), expected)
        return
    if kind == "conj":
        _compare(case, np.array(dins[0].conj().to_numpy(), order="C"), expected)
        return
    out = _dev(tf, before) if before is not None else tf.Tensor.empty(list(expected.shape), gpu, tf.MemoryOrder.RowMajor, dt)
    if kind == "einsum":
        tf.einsum_into(case["subscripts"], dins, alpha, beta, out)
    else:
        shapes = [list(x.shape) for x in ins] + [list(expected.shape)]
        if kind == "permute":
            desc = tf.PrimDescriptor.Permute(case["modes_a"], case["modes_b"])
        elif kind == "reduce":
            op = {"sum": tf.ReduceOp.Sum, "max": tf.ReduceOp.Max, "min": tf.ReduceOp.Min}[case["op"]]
            desc = tf.PrimDescriptor.Reduce(case["modes_a"], case["modes_c"], op)
        elif kind == "batched_gemm":
            desc = tf.PrimDescriptor.BatchedGemm(case["batch_dims"], case["m"], case["n"], case["k"])
        elif kind == "elementwise_mul":
            desc = tf.PrimDescriptor.ElementwiseMul()
        elif kind == "trace":
            desc = tf.PrimDescriptor.Trace(case["modes_a"], case["modes_c"], [tuple(p) for p in case["paired"]])
        else:
            raise AssertionError(kind)
        plan = tf.HipBackend.plan(dt, desc, shapes)
        tf.HipBackend.execute(plan, alpha, dins, beta, out)
    _compare(case, np.array(out.to_numpy(), order="C"), expected)

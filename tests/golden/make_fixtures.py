"""Writes the golden vectors in this directory: cases.json (what each case is) and cases.npz (its
inputs and expected output).

The reference holds no numeric vectors for this path (its bodies are todo!(), tenferro-prims/src/lib.rs:419-439;
tenferro-einsum/src/lib.rs:393-621), so the expected outputs come from an independent library, numpy: np.einsum,
np.transpose, np.sum/max/min, np.matmul, all in the case's own dtype except that f32/c64 cases are evaluated in
f64/c128 and rounded once.  Repeated output labels ("i->ii"), which np.einsum rejects, are written by explicit
index loops.  The einsum strings are the pattern catalogue of tenferro-einsum/src/lib.rs:37-93 plus small
versions of the benchmark configurations.

Run from the repository root:  python tests/golden/make_fixtures.py
Neither the library under test nor its CPU oracle is imported here."""
import itertools
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
DT = {"f32": np.float32, "f64": np.float64, "c64": np.complex64, "c128": np.complex128}
WIDE = {"f32": np.float64, "f64": np.float64, "c64": np.complex128, "c128": np.complex128}


def draw(rng, shape, dt, exact=False):
    def real():
        if exact:                       # small dyadic rationals: every product and sum below is exact in f32
            return rng.integers(-8, 9, shape).astype(np.float64) / 4.0
        return rng.standard_normal(shape)
    x = real()
    if dt in ("c64", "c128"):
        x = x + 1j * real()
    return np.array(x, dtype=DT[dt], order="C")                # (ascontiguousarray would turn rank 0 into rank 1)


def einsum_expected(sub, ops, dt):
    ins, out = sub.replace("(", "").replace(")", "").split("->")
    wide = [o.astype(WIDE[dt]) for o in ops]
    if len(set(out)) == len(out):
        return np.asarray(np.einsum(ins + "->" + out, *wide))
    # repeated output labels: the unique-label result scattered on the diagonal, zero elsewhere
    uniq = "".join(dict.fromkeys(out))
    inner = np.asarray(np.einsum(ins + "->" + uniq, *wide))
    size = {c: inner.shape[uniq.index(c)] for c in uniq}
    res = np.zeros([size[c] for c in out], WIDE[dt])
    for idx in itertools.product(*[range(size[c]) for c in uniq]):
        at = dict(zip(uniq, idx))
        res[tuple(at[c] for c in out)] = inner[idx]
    return res


EINSUM = [   # (subscripts, shapes)
    ("ij,jk->ik", [(7, 5), (5, 9)]),
    ("ij,jk->ik", [(64, 48), (48, 80)]),
    ("ij,jk->ki", [(33, 17), (17, 20)]),
    ("bij,bjk->bik", [(10, 3, 4), (10, 4, 5)]),
    ("abij,abjk->abik", [(2, 3, 4, 5), (2, 3, 5, 6)]),
    ("bij,jk->bik", [(10, 3, 4), (4, 5)]),
    ("ii->", [(6, 6)]),
    ("ii->i", [(6, 6)]),
    ("i->ii", [(3,)]),
    ("i->iii", [(3,)]),
    ("ij->ji", [(5, 8)]),
    ("ij->", [(5, 8)]),
    ("ij->j", [(5, 8)]),
    ("ijk->kij", [(4, 5, 6)]),
    ("i,i->i", [(11,), (11,)]),
    ("i,i->", [(11,), (11,)]),
    ("i,j->ij", [(4,), (7,)]),
    ("ij,ij->ij", [(4, 7), (4, 7)]),
    ("iij,jk->ik", [(4, 4, 5), (5, 3)]),
    ("ajbk,kcj->abc", [(4, 8, 4, 6), (6, 16, 8)]),
    ("awc,asx,wstv,cty->xvy", [(8, 4, 8), (8, 2, 8), (4, 2, 2, 4), (8, 2, 8)]),
    ("ij,(jk,kl)->il", [(6, 7), (7, 8), (8, 9)]),
    ("(ij,jk),(kl,lm)->im", [(3, 4), (4, 5), (5, 6), (6, 7)]),
]


def main():
    rng = np.random.default_rng(20240611)
    cases, arrays = [], {}

    def add(case, ins, before, expected):
        cid = f"c{len(cases):03d}"
        case["id"], case["n_inputs"] = cid, len(ins)
        for i, x in enumerate(ins):
            arrays[f"{cid}_in{i}"] = x
        if before is not None:
            arrays[f"{cid}_before"] = before
        arrays[f"{cid}_expected"] = np.array(expected, dtype=DT[case["dtype"]], order="C")     # keeps rank 0
        cases.append(case)

    # ---- einsum front end: output = einsum(operands)
    for sub, shapes in EINSUM:
        for dt in DT:
            ops = [draw(rng, s, dt) for s in shapes]
            add({"kind": "einsum", "subscripts": sub, "dtype": dt, "alpha": [1, 0], "beta": [0, 0]}, ops, None,
                einsum_expected(sub, ops, dt))
    # exact inputs: the f32 result has no rounding, so every implementation must agree to the bit
    for sub, shapes in EINSUM[:6]:
        ops = [draw(rng, s, "f32", exact=True) for s in shapes]
        add({"kind": "einsum", "subscripts": sub, "dtype": "f32", "alpha": [1, 0], "beta": [0, 0], "exact": True}, ops,
            None, einsum_expected(sub, ops, "f32"))
    # ---- einsum_into: output = alpha * einsum(operands) + beta * output
    for (sub, shapes), dt in zip(EINSUM[:8], itertools.cycle(DT)):
        ops = [draw(rng, s, dt) for s in shapes]
        plain = einsum_expected(sub, ops, dt)
        before = draw(rng, plain.shape, dt)
        cplx = dt in ("c64", "c128")
        alpha, beta = (complex(0.5, -2.0), complex(1.5, 1.0)) if cplx else (0.5, -1.5)
        add({"kind": "einsum", "subscripts": sub, "dtype": dt, "alpha": [alpha.real, alpha.imag] if cplx else [alpha, 0],
             "beta": [beta.real, beta.imag] if cplx else [beta, 0]}, ops, before,
            alpha * plain + beta * before.astype(WIDE[dt]))

    # ---- Permute (tenferro-prims/src/lib.rs:194-202): B[modes_b] = A[modes_a], a pure copy
    for dt in DT:
        a = draw(rng, (2, 3, 4, 3, 2, 5), dt)
        perm = [5, 2, 0, 4, 1, 3]
        add({"kind": "permute", "dtype": dt, "modes_a": list(range(6)), "modes_b": perm, "alpha": [1, 0], "beta": [0, 0]},
            [a], None, np.transpose(a, perm))
    # ---- Reduce (:170-180): C[modes_c] = op over the modes of A that C lacks
    for dt, op in itertools.product(DT, ("sum", "max", "min")):
        if op != "sum" and dt in ("c64", "c128"):
            continue
        a = draw(rng, (6, 5, 4, 7), dt)
        fn = {"sum": np.sum, "max": np.max, "min": np.min}[op]
        red = fn(a.astype(WIDE[dt]), axis=(1, 3))                 # keeps modes 0, 2
        add({"kind": "reduce", "dtype": dt, "op": op, "modes_a": [0, 1, 2, 3], "modes_c": [2, 0], "alpha": [1, 0],
             "beta": [0, 0]}, [a], None, red.T)
    # ---- BatchedGemm (:156-168): C[batch,m,n] = alpha A[batch,m,k] B[batch,k,n] + beta C
    for dt in DT:
        a, b = draw(rng, (2, 3, 9, 11), dt), draw(rng, (2, 3, 11, 6), dt)
        before = draw(rng, (2, 3, 9, 6), dt)
        add({"kind": "batched_gemm", "dtype": dt, "batch_dims": [2, 3], "m": 9, "n": 6, "k": 11, "alpha": [2, 0],
             "beta": [-0.5, 0]}, [a, b], before,
            2 * np.matmul(a.astype(WIDE[dt]), b.astype(WIDE[dt])) - 0.5 * before.astype(WIDE[dt]))
    # ---- ElementwiseMul (:241-244): C = alpha A.B + beta C
    for dt in DT:
        a, b, before = draw(rng, (5, 6, 7), dt), draw(rng, (5, 6, 7), dt), draw(rng, (5, 6, 7), dt)
        add({"kind": "elementwise_mul", "dtype": dt, "alpha": [2, 0], "beta": [1, 0]}, [a, b], before,
            2 * a.astype(WIDE[dt]) * b.astype(WIDE[dt]) + before.astype(WIDE[dt]))
    # ---- Trace (:182-192): C[modes_c] = sum over paired modes set equal
    for dt in DT:
        a = draw(rng, (5, 4, 5), dt)                               # modes 0 and 2 paired, mode 1 kept
        add({"kind": "trace", "dtype": dt, "modes_a": [0, 1, 2], "modes_c": [1], "paired": [[0, 2]], "alpha": [1, 0],
             "beta": [0, 0]}, [a], None, np.einsum("iji->j", a.astype(WIDE[dt])))
    # ---- Tensor::conj (tenferro-tensor/src/lib.rs:606-647)
    for dt in ("c64", "c128"):
        a = draw(rng, (4, 5), dt)
        add({"kind": "conj", "dtype": dt, "alpha": [1, 0], "beta": [0, 0]}, [a], None, np.conj(a))

    with open(os.path.join(HERE, "cases.json"), "w") as f:
        json.dump(cases, f, indent=0)
    np.savez_compressed(os.path.join(HERE, "cases.npz"), **arrays)
    print(len(cases), "cases,", sum(a.nbytes for a in arrays.values()), "bytes of vectors")


if __name__ == "__main__":
    main()

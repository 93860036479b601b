"""Writes cancelling_f32.npz: f32 contractions whose sums cancel (the sum of |products| is ~1400 times the result).

Case "dot": the thirty-term product "dc,dc->" (d = 6, c = 5, alpha = 0.7) on which a randomized f32 parity run once
reported 2.18e-5 relative to the result.  Its operands are kept below as f32 bit patterns.  Evaluated here in f64
(products of f32 values are exact in f64, thirty of them add up with error ~1e-16): the exact result, and the same
sum over |a|.|b|.  Case "mat": the same thirty terms under two free axes, "fdc,dce->fe" (f = 2, e = 3), every output
cancelling the same way, so that the products run on a matrix-core kernel instead of a reduction kernel.

Run from the repository root:  python tests/golden/make_cancelling_f32.py      (numpy only)"""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
A_BITS = [3215052049, 3189937206, 1067278427, 1049619128, 1056259701, 3211744669, 3216664229, 3205288054, 3169484181, 1071888700,
          1043830563, 3207127370, 3220928091, 1029502990, 3205332298, 3201494992, 3207601677, 3219084288, 3210826054, 1067481894,
          1030896027, 3217104002, 3200313841, 3201024616, 1043173747, 3187190811, 3201426631, 1047306986, 1067230564, 1065875494]
B_BITS = [3184231536, 1070598132, 3204827593, 1012356136, 3172383767, 3219491813, 1058152720, 3196017543, 1065457905, 1060115301,
          3215041646, 3214994061, 3217803906, 1066132350, 3201598862, 3213441505, 3195755683, 3203012359, 1061128994, 3217379159,
          3200760632, 1066177624, 3203022975, 1070668112, 1067060870, 1060292856, 1064608376, 3179250164, 3205883741, 3212945387]

a = np.array(A_BITS, dtype=np.uint32).view(np.float32).reshape(6, 5)
b = np.array(B_BITS, dtype=np.uint32).view(np.float32).reshape(6, 5)
alpha = 0.7
a64, b64 = a.astype(np.float64), b.astype(np.float64)
out = {
    "dot_a": a, "dot_b": b, "alpha": np.float64(alpha),
    "dot_exact": np.float64(alpha * np.sum(a64 * b64)),
    "dot_abs": np.float64(alpha * np.sum(np.abs(a64 * b64))),
}
# two free axes: powers of two scale every term exactly, so each output cancels like the dot product does
a3 = np.stack([a, -2.0 * a]).astype(np.float32)                       # [f, d, c]
b3 = np.stack([b, 0.5 * b, -4.0 * b], axis=-1).astype(np.float32)     # [d, c, e]
out.update({
    "mat_a": a3, "mat_b": b3,
    "mat_exact": alpha * np.einsum("fdc,dce->fe", a3.astype(np.float64), b3.astype(np.float64)),
    "mat_abs": alpha * np.einsum("fdc,dce->fe", np.abs(a3).astype(np.float64), np.abs(b3).astype(np.float64)),
})
np.savez(os.path.join(HERE, "cancelling_f32.npz"), **out)
print({k: (v.shape, v.dtype) for k, v in out.items()})
print("dot exact", out["dot_exact"], "cancellation ratio", out["dot_abs"] / abs(out["dot_exact"]))

#!/usr/bin/env python3
"""Benchmark of the tensor-contraction hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--configs c1,c2,c3,c4] [--no-cpu]

Prints ONE JSON line.  The headline (`value`) is configuration 3 of the benchmark definition, the largest one --
the complex128 MPS-MPO environment update "awc,asx,wstv,cty->xvy" at bond dimension 1024 (558.3 GFLOP along the
minimum-flop tree) -- as whole-step TFLOP/s through einsum_with_plan_into with operands resident in HBM;
`all_configs` carries the same measurements for configurations 1 (f32 "ajbk,kcj->abc"), 2 (permute + reduce of a
16^6 f64 tensor) and 4 (128-block grouped f64 GEMM).  A "step" is one pass of the workload: one einsum tree, one
contraction, one permute+reduce, one grouped launch.

`roofline` describes the kernel that takes most of the step's time: `achieved` is its algorithmic flops (or bytes) per
launch divided by its average duration, measured from the begin/end timestamps of its own dispatches on the launch
stream over a second pass of the same K steps (the K timed steps themselves carry no events: launching a kernel with
them costs 4-5 us of stream time, which is not the library's); `kernel` is the label the library reported for those
dispatches.  `traffic` is read
from profiles/bench_hbm_traffic_pmc.txt (a profiler cannot run inside this script) and is null when the kernel that
ran is not the one that file was measured on.  `cpu_baseline` is the CPU oracle (a port: the reference has no CPU
backend to time) on the host cores of this machine, on the same inputs; its result is also the parity check of the run.
"""
import argparse
import ctypes as C
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK = {"hbm": 8000.0, "f32": 157.3, "f64": 78.6}   # GB/s, TFLOP/s (MI355X published peaks)
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "bench_hbm_traffic_pmc.txt")
SPINUP_S = 0.3   # seconds of untimed device spin-up per configuration
METRIC = "contraction TFLOP/s & % MFMA peak (f64/f32); permute/reduce GB/s & % HBM peak"


def load_traffic(path=TRAFFIC_FILE):
    """{key: (HBM bytes per launch, kernel label)} from the lines "traffic <key> <bytes> <label>" of the committed
    rocprofv3 --pmc summary (FETCH_SIZE + WRITE_SIZE, each scaled by its reading for a plain copy of known size)."""
    out = {}
    if os.path.exists(path):
        for line in open(path):
            m = re.match(r"\s*traffic\s+(\S+)\s+(\d+)\s+(\(.*\))\s*$", line)
            if m:
                out[m.group(1)] = (float(m.group(2)), m.group(3))
    return out


TRAFFIC = load_traffic()


def traffic_of(key, label):
    """Bytes per launch measured for `key`, or None when no measurement exists for the kernel that ran."""
    t = TRAFFIC.get(key)
    return t[0] if t and t[1] == label else None


def lab(s):
    return [ord(c) for c in s]


def relerr(x, ref):
    d = np.linalg.norm((x - ref).ravel())
    n = np.linalg.norm(ref.ravel())
    return float(d / n) if n > 0 else float(d)


def dominant(recs):
    """The record (label, ms per launch, launches per step) with the largest share of the step."""
    return max(recs, key=lambda r: r[1] * r[2])


def roofline(bound, peak_key, work_per_launch, rec, traffic_key):
    label, ms, per_step = rec
    scale = 1e12 if bound == "mfma" else 1e9
    achieved = work_per_launch / (ms * 1e-3) / scale
    return {"bound": bound, "achieved": achieved, "peak": PEAK[peak_key], "unit": "TFLOP/s" if bound == "mfma" else "GB/s",
            "frac": achieved / PEAK[peak_key], "traffic": traffic_of(traffic_key, label),
            "traffic_unit": "HBM bytes per launch (FETCH_SIZE + WRITE_SIZE, calibrated; profiles/bench_hbm_traffic_pmc.txt)",
            "kernel": label, "kernel_ms": ms, "launches_per_step": per_step,
            "work_per_launch": work_per_launch}


class Harness:
    def __init__(self, steps, warmup, cpu):
        import torch
        import tenferro_rs_amd as tf
        from tenferro_rs_amd import inputs
        self.torch, self.tf, self.inputs = torch, tf, inputs
        self.steps, self.warmup, self.cpu = steps, warmup, cpu
        tf.lib()
        if cpu:
            from oracle import tfo
            tfo.lib()
            self.tfo = tfo
            self.cores = tfo.num_threads()

    def gpu(self, arr, cm=False):
        """Device tensor with the values of arr, row-major, or column-major (first index contiguous) when cm."""
        if not cm:
            return self.tf.Tensor.from_torch(self.torch.from_numpy(np.ascontiguousarray(arr)).cuda())
        t = self.torch.from_numpy(np.ascontiguousarray(arr.transpose())).cuda()
        return self.tf.Tensor.from_torch(t.permute(*reversed(range(arr.ndim))))

    def empty(self, shape, dtype, cm=False):
        order = self.tf.MemoryOrder.ColumnMajor if cm else self.tf.MemoryOrder.RowMajor
        return self.tf.Tensor.empty(list(shape), self.tf.GpuMemory(0), order, dtype)

    def timed(self, step, kinds):
        """step(i) enqueues one pass.  Returns (ms per step, {kind: [(kernel label, ms per launch, launches per step)]})."""
        torch, tf = self.torch, self.tf
        # device spin-up, untimed: the first ~20 ms of work after an idle period run at lower clocks (the same kernel
        # measures 250 us in the first 30 launches and 226 us from the 60th on), so the workload is repeated for
        # SPINUP_S seconds before the W warm-up steps
        t_end = time.perf_counter() + SPINUP_S
        i = 0
        while time.perf_counter() < t_end:
            for _ in range(8):
                step(i)
                i += 1
            torch.cuda.synchronize()
        for i in range(self.warmup):
            step(i)
        torch.cuda.synchronize()
        # the timed region: exactly K steps, nothing but the workload on the stream
        t0 = time.perf_counter()
        for i in range(self.steps):
            step(self.warmup + i)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        # per-kernel durations: the same K steps once more with a pair of HIP events around every dominant kernel, on the
        # stream it is launched on.  The events are kept out of the region above because they are not free: launching a
        # kernel with them costs 4-5 us of stream time per kernel (0.245 ms instead of 0.2355 ms per step for
        # configuration 1), which would be charged to the library.
        tf.profile_enable(True)
        t2 = time.perf_counter()
        for i in range(self.steps):
            step(self.warmup + self.steps + i)
        torch.cuda.synchronize()
        t3 = time.perf_counter()
        out = {}
        for k in kinds:
            out[k] = [(name, ms / n, n / self.steps) for name, ms, n in tf.profile_kernels(k)]
            tf.profile_collect(k)
        tf.profile_enable(False)
        self.last_ms_with_events = (t3 - t2) * 1e3 / self.steps
        return (t1 - t0) * 1e3 / self.steps, out

    def cpu_time(self, fn, reps):
        best = None
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        return best

    def bound_execute(self, plan, inputs, output, alpha=1.0, beta=0.0):
        """Pre-marshalled tfh_execute call: the hot loop does no Python-side packing."""
        tf = self.tf
        L = tf.lib()
        views = (tf.tfh_view * len(inputs))(*[tf.view_of(t) for t in inputs])
        vo = tf.view_of(output)
        al, be = tf._scalar_c(plan.dtype, alpha), tf._scalar_c(plan.dtype, beta)
        st = tf.current_stream()
        n = len(inputs)

        def call():
            rc = L.tfh_execute(plan._h, al, views, n, be, C.byref(vo), st)
            if rc:
                tf._check(rc)
        call.keep = (views, vo, al, be, inputs, output, plan)
        return call


# ------------------------------------------------------------------------------------------------- config 1
def run_c1(h, cm=False, ref_out=None):
    tf, inputs = h.tf, h.inputs
    a, j, b, k, c = 64, 128, 64, 96, 256
    A = inputs.normal(1001, 0, (a, j, b, k), np.float32)
    B = inputs.normal(1001, 1, (k, c, j), np.float32)
    flops = 2.0 * a * b * c * j * k
    algo_bytes = 4.0 * (A.size + B.size + a * b * c)
    nset = 3   # rotate operand sets so the 201 MB operand is not served from the 256 MB last-level cache
    As = [h.gpu(A, cm) for _ in range(nset)]
    Bd = h.gpu(B, cm)
    outs = [h.empty((a, b, c), np.float32, cm) for _ in range(nset)]
    plan = tf.HipBackend.plan(np.float32, tf.PrimDescriptor.Contract(lab("ajbk"), lab("kcj"), lab("abc")),
                              [A.shape, B.shape, (a, b, c)])
    calls = [h.bound_execute(plan, [As[i], Bd], outs[i]) for i in range(nset)]
    ms, prof = h.timed(lambda i: calls[i % nset](), [tf.PROF_CONTRACT, tf.PROF_COPY])
    rec = dominant(prof[tf.PROF_CONTRACT])
    res = {
        "workload": "einsum ajbk,kcj->abc f32 a=64 j=128 b=64 k=96 c=256 (GEMM view M=4096 N=256 K=12288)" + LAYOUT_NOTE[cm],
        "dtype": "f32", "ms_per_step": ms, "ms_per_step_with_kernel_events": h.last_ms_with_events, "value": flops / (ms * 1e-3) / 1e12, "unit": "TFLOP/s",
        "whole_step_frac_of_peak": flops / (ms * 1e-3) / 1e12 / PEAK["f32"],
        "flops_per_step": flops, "algorithmic_bytes": algo_bytes,
        "roofline": roofline("mfma", "f32", flops, rec, "c1"),
        "other_kernels": [r for kind in prof.values() for r in kind if r is not rec],
    }
    res["_out"] = outs[0].to_numpy()
    if ref_out is not None:
        res["parity"] = {"vs_row_major_rel_frobenius": relerr(res["_out"].astype(np.float64), ref_out.astype(np.float64)), "tolerance": 1e-5}
    elif h.cpu:
        ref = np.empty((a, b, c), np.float32)
        t = h.cpu_time(lambda: h.tfo.contract(A, lab("ajbk"), B, lab("kcj"), ref, lab("abc")), 20)
        res["cpu_baseline"] = {"value": flops / t / 1e12, "unit": "TFLOP/s", "cores": h.cores, "kind": "port",
                               "sample": "the full contraction (25.8 GFLOP), best of 20", "seconds": t}
        res["parity"] = {"rel_frobenius": relerr(outs[0].to_numpy().astype(np.float64), ref.astype(np.float64)), "tolerance": 1e-5}
    return res


# ------------------------------------------------------------------------------------------------- config 2
def run_c2(h):
    tf, inputs = h.tf, h.inputs
    shape = (16,) * 6
    perm = [5, 2, 0, 4, 1, 3]
    X = inputs.uniform(1002, 0, shape)
    nset = 6   # permuted buffers in rotation: the reduce of step i reads the one written FOUR steps earlier
    lag = 4    # 4 x (134 MB read + 134 MB written by the permutes between) = 1.07 GB through the 256 MB last-level cache
    Xs = [h.gpu(X) for _ in range(3)]
    Ps = [h.empty(shape, np.float64) for _ in range(nset)]
    Rs = [h.empty((16,) * 4, np.float64) for _ in range(nset)]
    pplan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Permute(list(range(6)), perm), [shape, shape])
    modes_a, modes_c = perm, [5, 0, 4, 3]          # sum over output axes 1 and 4 of the permuted tensor
    rplan = tf.HipBackend.plan(np.float64, tf.PrimDescriptor.Reduce(modes_a, modes_c, tf.ReduceOp.Sum), [shape, (16,) * 4])
    pcalls = [h.bound_execute(pplan, [Xs[i % 3]], Ps[i]) for i in range(nset)]
    rcalls = [h.bound_execute(rplan, [Ps[i]], Rs[i]) for i in range(nset)]
    pbytes = 2.0 * X.nbytes
    rbytes = float(X.nbytes + 16 ** 4 * 8)
    for c in pcalls:    # every permuted buffer holds the permuted tensor before anything is timed
        c()

    def step_cold(i):
        # the reduce reads a buffer that no kernel has touched for `lag` steps: its input comes from HBM
        pcalls[i % nset]()
        rcalls[(i - lag) % nset]()

    def step_chained(i):
        # the reduce reads what the permute has just written (part of it still sits in the last-level cache)
        pcalls[i % nset]()
        rcalls[i % nset]()
    ms_chained, prof_chained = h.timed(step_chained, [tf.PROF_COPY, tf.PROF_REDUCE])
    ms_chained_events = h.last_ms_with_events
    ms, prof = h.timed(step_cold, [tf.PROF_COPY, tf.PROF_REDUCE])
    prec, rrec = dominant(prof[tf.PROF_COPY]), dominant(prof[tf.PROF_REDUCE])
    rrec_chained = dominant(prof_chained[tf.PROF_REDUCE])
    res = {
        "workload": "f64 16^6 tensor: permute to (5,2,0,4,1,3), then sum over output axes 1 and 4 "
                    "(six permuted buffers in rotation; the timed reduce reads the one written four steps earlier, i.e. from HBM)",
        "dtype": "f64", "ms_per_step": ms, "ms_per_step_with_kernel_events": h.last_ms_with_events, "value": (pbytes + rbytes) / (ms * 1e-3) / 1e9, "unit": "GB/s",
        "permute": {"roofline": roofline("hbm", "hbm", pbytes, prec, "c2_permute"), "algorithmic_bytes": pbytes},
        "reduce": {"roofline": roofline("hbm", "hbm", rbytes, rrec, "c2_reduce"), "algorithmic_bytes": rbytes,
                   "input": "cold: written four steps (1.07 GB of other traffic) before it is read"},
        "reduce_chained": {"roofline": roofline("hbm", "hbm", rbytes, rrec_chained, "c2_reduce"), "algorithmic_bytes": rbytes,
                           "ms_per_step": ms_chained, "ms_per_step_with_kernel_events": ms_chained_events,
                           "input": "warm: the buffer the preceding permute has just written (not the roofline figure)"},
    }
    if h.cpu:
        P = np.empty(shape)
        R = np.empty((16,) * 4)
        tp = h.cpu_time(lambda: h.tfo.permute(X, list(range(6)), P, perm), 20)
        tr = h.cpu_time(lambda: h.tfo.reduce(P, modes_a, R, modes_c), 20)
        res["cpu_baseline"] = {"permute": {"value": pbytes / tp / 1e9, "unit": "GB/s", "seconds": tp},
                               "reduce": {"value": rbytes / tr / 1e9, "unit": "GB/s", "seconds": tr},
                               "cores": h.cores, "kind": "port", "sample": "the full 16^6 tensor, best of 20"}
        res["parity"] = {"permute_bit_exact": bool(Ps[0].to_numpy().tobytes() == P.tobytes()),
                         "reduce_rel_frobenius": relerr(Rs[0].to_numpy(), R), "tolerance": 1e-12}
    return res


# ------------------------------------------------------------------------------------------------- config 3
def run_c3(h, cm=False, ref_out=None):
    tf, inputs = h.tf, h.inputs
    chi, D, d = 1024, 16, 2
    sig = 1.0 / np.sqrt(chi)
    Lh = inputs.complex_normal(1003, 0, (chi, D, chi), sig)
    Ah = inputs.complex_normal(1003, 1, (chi, d, chi), sig)
    Wh = inputs.complex_normal(1003, 2, (D, d, d, D), sig)
    terms, out = ["awc", "asx", "wstv", "cty"], "xvy"
    subs = tf.Subscripts.parse(",".join(terms) + "->" + out)
    shapes = [Lh.shape, Ah.shape, Wh.shape, Ah.shape]
    tree = tf.ContractionTree.optimize(subs, shapes)
    flops = 8.0 * tree.mac_count
    # per-step work of the tree: 8 real flops per complex multiply-add over the union of the two operands' labels
    step_flops = []
    for si, (lhs, rhs) in enumerate(tree.steps):
        ext = {}
        for node in (lhs, rhs):
            labels, dims = tree.node(node)
            ext.update(zip(labels, dims))
        step_flops.append(8.0 * float(np.prod([float(v) for v in ext.values()])))
    Ld, Ad, Wd = h.gpu(Lh, cm), h.gpu(Ah, cm), h.gpu(Wh, cm)
    # 4th operand: A itself behind the conjugate-on-load flag (no conjugated copy is made; the contraction kernel that
    # reads it flips the sign of the imaginary parts as it stages them).  The explicit copy (Tensor::conj) is timed
    # beside it, and one pass over it, for comparison.
    Acd = Ad.conj()
    h.torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(20):
        Acd = Ad.conj()
    h.torch.cuda.synchronize()
    conj_ms = (time.perf_counter() - t0) * 1e3 / 20
    res_t = h.empty((chi, D, chi), np.complex128, cm)
    ops_copy = [Ld, Ad, Wd, Acd]
    ms_copy, _ = h.timed(lambda i: tf.einsum_with_plan_into(tree, ops_copy, 1.0, 0.0, res_t), [tf.PROF_CONTRACT])
    copy_result = res_t.to_numpy()
    ops = [Ld, Ad, Wd, Ad.conj_on_load()]
    ms, prof = h.timed(lambda i: tf.einsum_with_plan_into(tree, ops, 1.0, 0.0, res_t), [tf.PROF_CONTRACT])
    recs = prof[tf.PROF_CONTRACT]
    rec = dominant(recs)
    total_kms = sum(r[1] * r[2] for r in recs)
    # the dominant kernel runs the large steps of the tree (equal work each); the remaining step has its own kernel
    n_dom = int(round(rec[2]))
    dom_flops = sorted(step_flops, reverse=True)[:n_dom]
    res = {
        "workload": "einsum awc,asx,wstv,cty->xvy complex128 chi=1024 D=16 d=2 via einsum_with_plan_into (tree from the optimiser; "
                    "4th operand is A behind the conjugate-on-load flag: no conjugated copy exists)" + LAYOUT_NOTE[cm],
        "dtype": "c128", "ms_per_step": ms, "ms_per_step_with_kernel_events": h.last_ms_with_events, "value": flops / (ms * 1e-3) / 1e12, "unit": "TFLOP/s",
        "whole_step_frac_of_peak": flops / (ms * 1e-3) / 1e12 / PEAK["f64"],
        "flops_per_step": flops, "tree_steps": tree.steps, "step_flops": step_flops, "min_flop_tree": bool(abs(flops - 558.3e9) < 0.1e9),
        "peak_intermediate_bytes": tree.peak_intermediate * 16,
        "with_conj_copy": {"ms_per_step": ms_copy, "conj_ms": conj_ms,
                           "same_result": bool(relerr(res_t.to_numpy(), copy_result) < 1e-14)},
        "roofline": roofline("mfma", "f64", sum(dom_flops) / max(n_dom, 1), rec, "c3"),
        "all_kernels": {"kernel_ms_per_step": total_kms, "frac_of_peak": flops / (total_kms * 1e-3) / 1e12 / PEAK["f64"],
                        "kernels": recs},
    }
    res["_out"] = res_t.to_numpy()
    if ref_out is not None:
        res["parity"] = {"vs_row_major_rel_frobenius": relerr(res["_out"], ref_out), "tolerance": 1e-12}
    elif h.cpu:
        host = [Lh, Ah, Wh, np.conj(Ah)]
        ref = np.empty((chi, D, chi), np.complex128)
        t = h.cpu_time(lambda: h.tfo.einsum_pairs(host, [lab(t_) for t_ in terms], ref, lab(out), tree.steps), 3)
        res["cpu_baseline"] = {"value": flops / t / 1e12, "unit": "TFLOP/s", "cores": h.cores, "kind": "port",
                               "sample": "the full tree (558.3 GFLOP), best of 3", "seconds": t}
        res["parity"] = {"rel_frobenius": relerr(res_t.to_numpy(), ref),
                         "conj_bit_exact": bool(Acd.to_numpy().tobytes() == np.conj(Ah).tobytes()), "tolerance": 1e-12}
    return res


# ------------------------------------------------------------------------------------------------- config 4
def run_c4(h, cm=False, ref_out=None):
    tf, inputs = h.tf, h.inputs
    dims = inputs.draw_block_dims(1004, 128)
    As = [inputs.uniform(1004, 3 * g, (i, j)) for g, (i, j, k) in enumerate(dims)]
    Bs = [inputs.uniform(1004, 3 * g + 1, (j, k)) for g, (i, j, k) in enumerate(dims)]
    flops = float(sum(2 * i * j * k for i, j, k in dims))
    algo_bytes = float(sum(8 * (i * j + j * k + i * k) for i, j, k in dims))
    dA, dB = [h.gpu(x, cm) for x in As], [h.gpu(x, cm) for x in Bs]
    outs = [h.empty((i, k), np.float64, cm) for i, j, k in dims]
    plan = tf.HipBackend.plan_grouped(np.float64, tf.PrimDescriptor.Contract(lab("ij"), lab("jk"), lab("ik")),
                                      [[[i, j], [j, k], [i, k]] for i, j, k in dims])
    pairs = list(zip(dA, dB))
    ms, prof = h.timed(lambda i: tf.HipBackend.execute_grouped(plan, 1.0, pairs, 0.0, outs), [tf.PROF_CONTRACT])
    rec = dominant(prof[tf.PROF_CONTRACT])
    res = {
        "workload": "128 independent ij,jk->ik f64 blocks, i,j,k iid from {64,...,1024}, one grouped launch" + LAYOUT_NOTE[cm],
        "dtype": "f64", "ms_per_step": ms, "ms_per_step_with_kernel_events": h.last_ms_with_events, "value": flops / (ms * 1e-3) / 1e12, "unit": "TFLOP/s",
        "flops_per_step": flops, "algorithmic_bytes": algo_bytes,
        "roofline": roofline("mfma", "f64", flops, rec, "c4"),
    }
    res["_out"] = [o.to_numpy() for o in outs]
    if ref_out is not None:
        res["parity"] = {"vs_row_major_max_rel_frobenius": max(relerr(o, r) for o, r in zip(res["_out"], ref_out)), "tolerance": 1e-12}
    elif h.cpu:
        refs = [np.empty((i, k)) for i, j, k in dims]

        def cpu():
            for a, b, r in zip(As, Bs, refs):
                h.tfo.contract(a, lab("ij"), b, lab("jk"), r, lab("ik"))
        t = h.cpu_time(cpu, 5)
        res["cpu_baseline"] = {"value": flops / t / 1e12, "unit": "TFLOP/s", "cores": h.cores, "kind": "port",
                               "sample": "all 128 blocks, best of 5", "seconds": t}
        res["parity"] = {"max_rel_frobenius": max(relerr(o.to_numpy(), r) for o, r in zip(outs, refs)), "tolerance": 1e-12}
    return res


# ------------------------------------------------------------------------------------------------- config 0 and batched products
def run_matmul(h, cm=False, ref_out=None):
    """Configuration 0 (the CPU-runnable plumbing case, 512^3 f64 through einsum) on the GPU, for the layout comparison."""
    tf, inputs = h.tf, h.inputs
    A, B = inputs.uniform(1000, 0, (512, 512)), inputs.uniform(1000, 1, (512, 512))
    Ad, Bd = h.gpu(A, cm), h.gpu(B, cm)
    out = h.empty((512, 512), np.float64, cm)
    tree = tf.ContractionTree.optimize(tf.Subscripts.parse("ij,jk->ik"), [A.shape, B.shape])
    ms, prof = h.timed(lambda i: tf.einsum_with_plan_into(tree, [Ad, Bd], 1.0, 0.0, out), [tf.PROF_CONTRACT])
    rec = dominant(prof[tf.PROF_CONTRACT])
    flops = 2.0 * 512 ** 3
    res = {"workload": "einsum ij,jk->ik f64 512^3" + LAYOUT_NOTE[cm], "dtype": "f64", "ms_per_step": ms, "value": flops / (ms * 1e-3) / 1e12,
           "unit": "TFLOP/s", "roofline": roofline("mfma", "f64", flops, rec, "c0"), "_out": out.to_numpy()}
    if ref_out is not None:
        res["parity"] = {"vs_row_major_rel_frobenius": relerr(res["_out"], ref_out), "tolerance": 1e-12}
    elif h.cpu:
        ref = np.empty((512, 512))
        t = h.cpu_time(lambda: h.tfo.contract(A, lab("ij"), B, lab("jk"), ref, lab("ik")), 20)
        res["cpu_baseline"] = {"value": flops / t / 1e12, "unit": "TFLOP/s", "cores": h.cores, "kind": "port", "sample": "the full product, best of 20", "seconds": t}
        res["parity"] = {"rel_frobenius": relerr(res["_out"], ref), "tolerance": 1e-12}
    return res


def run_batched(h, dtype, nb, n, cm=False, ref_out=None):
    """einsum bij,bjk->bik, nb products of n^3 (the batched pattern of the reference's einsum documentation); column-major
    is the layout the reference's examples allocate: the batch index is then the contiguous one in all three tensors."""
    tf = h.tf
    rng = np.random.default_rng(1005)
    cx = np.dtype(dtype).kind == "c"

    def draw(shape):
        x = rng.standard_normal(shape)
        return (x + 1j * rng.standard_normal(shape)).astype(dtype) if cx else x.astype(dtype)
    A, B = draw((nb, n, n)), draw((nb, n, n))
    Ad, Bd = h.gpu(A, cm), h.gpu(B, cm)
    out = h.empty((nb, n, n), dtype, cm)
    tree = tf.ContractionTree.optimize(tf.Subscripts.parse("bij,bjk->bik"), [A.shape, B.shape])
    ms, prof = h.timed(lambda i: tf.einsum_with_plan_into(tree, [Ad, Bd], 1.0, 0.0, out), [tf.PROF_CONTRACT, tf.PROF_COPY])
    rec = dominant(prof[tf.PROF_CONTRACT])
    flops = (8.0 if cx else 2.0) * nb * n ** 3
    nbytes = 3.0 * A.nbytes
    res = {"workload": "einsum bij,bjk->bik %s b=%d i=j=k=%d" % (np.dtype(dtype).name, nb, n) + LAYOUT_NOTE[cm],
           "dtype": "c128" if cx else "f64", "ms_per_step": ms, "value": flops / (ms * 1e-3) / 1e12, "unit": "TFLOP/s",
           "algorithmic_bytes": nbytes, "effective_GBps": nbytes / (ms * 1e-3) / 1e9,
           "roofline": roofline("mfma", "f64", flops, rec, "batched"),
           "operand_pack_kernels": [r for r in prof[tf.PROF_COPY]], "_out": out.to_numpy()}
    if ref_out is not None:
        res["parity"] = {"vs_row_major_rel_frobenius": relerr(res["_out"], ref_out), "tolerance": 1e-12}
    elif h.cpu:
        # a bounded sample of the batch on the CPU: the first 64 products
        m = min(nb, 64)
        ref = np.empty((m, n, n), dtype)
        As, Bs = np.ascontiguousarray(A[:m]), np.ascontiguousarray(B[:m])
        t = h.cpu_time(lambda: h.tfo.contract(As, lab("bij"), Bs, lab("bjk"), ref, lab("bik")), 5)
        res["cpu_baseline"] = {"value": flops * m / nb / t / 1e12, "unit": "TFLOP/s", "cores": h.cores, "kind": "port",
                               "sample": "the first %d of the %d products, best of 5" % (m, nb), "seconds": t}
        res["parity"] = {"rel_frobenius": relerr(res["_out"][:m], ref), "tolerance": 1e-12}
    return res


# ------------------------------------------------------------------------------------------------- permutes and reductions of general shapes
def random_shape(rng, rank, elems):
    """`rank` extents, none a power of two on purpose, whose product is close to `elems`."""
    w = rng.uniform(0.3, 1.0, rank)
    ext = np.maximum(2, np.round(np.exp(np.log(elems) * w / w.sum()))).astype(np.int64)
    for d in range(rank):      # nudge powers of two to their odd neighbours: the tile grid of the fast paths must not fit by luck
        if ext[d] & (ext[d] - 1) == 0:
            ext[d] += 1
    order = np.argsort(-ext)
    k = 0
    while np.prod(ext.astype(np.float64)) < elems:      # grow the largest extents until the tensor is large enough
        ext[order[k % rank]] += max(1, ext[order[k % rank]] // 16)
        k += 1
    return [int(x) for x in ext]


def shape_sweep(h, n_shapes=24, min_bytes=128 << 20, ops=("permute", "reduce"), dtypes=("f32", "f64", "c64", "c128")):
    """python bench.py --shape-sweep: permutes (random axis orders) and sum-reductions (random sets of reduced axes) of
    seeded random tensors of rank 3..7 and at least 128 MB, whose extents are not powers of two, for all four dtypes, as
    the fraction of the HBM peak that the bytes each must move (in + out) reach.  One line per shape, then min / median
    per dtype and operation."""
    tf, torch = h.tf, h.torch
    names = {np.float32: "f32", np.float64: "f64", np.complex64: "c64", np.complex128: "c128"}
    print("%-5s %-8s %-34s %-22s %9s %8s %8s %6s  %s" % ("dtype", "op", "shape", "perm / reduced axes", "MB moved", "us", "kernel us", "% HBM",
                                                         "last kernel"))
    summary = []
    for dtype in (np.float32, np.float64, np.complex64, np.complex128):
        if names[dtype] not in dtypes:
            continue
        rng = np.random.default_rng(1006)      # the same shapes for every dtype (scaled to the element size)
        fr = {"permute": [], "reduce": []}
        for i in range(n_shapes):
            rank = 3 + i % 5
            shape = random_shape(rng, rank, min_bytes // np.dtype(dtype).itemsize)
            perm = [int(x) for x in rng.permutation(rank)]
            while perm == list(range(rank)):
                perm = [int(x) for x in rng.permutation(rank)]
            nred = int(rng.integers(1, rank))
            red = sorted(int(x) for x in rng.choice(rank, nred, replace=False))
            n = int(np.prod(shape))
            src = torch.empty(n, dtype={np.float32: torch.float32, np.float64: torch.float64, np.complex64: torch.complex64,
                                        np.complex128: torch.complex128}[dtype], device="cuda")
            src.view(torch.float32 if np.dtype(dtype).itemsize % 8 else torch.float64).uniform_(-1.0, 1.0)
            X = tf.Tensor(src, shape, tf._contig_strides(shape, tf.MemoryOrder.RowMajor), 0, tf.GpuMemory(0), tf.dtype_code(dtype))
            for op in ops:
                if op == "permute":
                    oshape = [shape[p] for p in perm]
                    plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Permute(list(range(rank)), perm), [shape, oshape])
                    what, kind = str(tuple(perm)), tf.PROF_COPY
                else:
                    kept = [d for d in range(rank) if d not in red]
                    oshape = [shape[d] for d in kept]
                    plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Reduce(list(range(rank)), kept, tf.ReduceOp.Sum), [shape, oshape])
                    what, kind = "sum over " + str(tuple(red)), tf.PROF_REDUCE
                out = h.empty(oshape, dtype)
                call = h.bound_execute(plan, [X], out)
                ms, prof = h.timed(lambda i: call(), [kind])
                us = ms * 1e3
                kus = sum(m * c for (_, m, c) in prof[kind]) * 1e3      # the kernels alone, from HIP events around each
                nbytes = (n + int(np.prod(oshape))) * np.dtype(dtype).itemsize
                frac = nbytes / (us * 1e-6) / 1e9 / PEAK["hbm"]
                fr[op].append(frac)
                print("%-5s %-8s %-34s %-22s %9.1f %8.1f %8.1f %6.1f  %s" % (names[dtype], op, "x".join(map(str, shape)), what, nbytes / 1e6, us,
                                                                             kus, 100 * frac, tf.last_kernel()[:60]), flush=True)
                del out
            del X, src
            torch.cuda.empty_cache()
        for op in ops:
            summary.append("%-5s %-8s %2d shapes: min %5.1f %%  median %5.1f %%  max %5.1f %% of the 8 TB/s HBM peak" %
                           (names[dtype], op, len(fr[op]), 100 * min(fr[op]), 100 * float(np.median(fr[op])), 100 * max(fr[op])))
    print()
    print("\n".join(summary))


# ------------------------------------------------------------------------------------------------- host cost of a call
def host_overhead(h):
    """Microseconds of host time per enqueue (python bench.py --host-overhead): the first execute of a plan (routing, table
    build, workspace growth) against repeated ones (the plan keeps the routed launch per set of view strides), for a small
    contraction that is one launch, 128^3 f64 (split-K: two launches), configuration 1 (an operand pack, offset tables,
    split-K: not replayed) and a grouped plan of 1024 small problems.  Bursts of 200 calls on an idle stream, so that the
    launch queue never fills; every figure includes the ctypes call itself, measured beside them on tfh_version()."""
    tf, inputs, torch = h.tf, h.inputs, h.torch
    L = tf.lib()
    lines = []

    def measure(name, make_call, n=200, first_note=""):
        call = make_call()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        call()
        t_first = (time.perf_counter() - t0) * 1e6
        torch.cuda.synchronize()
        for _ in range(20):
            call()
        torch.cuda.synchronize()
        best = None
        for _ in range(5):
            t0 = time.perf_counter()
            for _ in range(n):
                call()
            t1 = time.perf_counter()
            torch.cuda.synchronize()
            t2 = time.perf_counter()
            rep = ((t1 - t0) * 1e6 / n, (t2 - t0) * 1e6 / n)
            best = rep if best is None or rep[0] < best[0] else best
        lines.append("%-58s first call %8.1f us   repeated enqueue %5.2f us   with drain %6.2f us   %s%s" %
                     (name, t_first, best[0], best[1], tf.last_kernel()[:44], first_note))

    t0 = time.perf_counter()
    for _ in range(20000):
        L.tfh_version()
    floor = (time.perf_counter() - t0) * 1e6 / 20000
    lines.append("measured from Python through ctypes (a call of a function that does nothing, tfh_version: %.2f us; marshalling the" % floor)
    lines.append("seven arguments of tfh_execute costs about a microsecond more):")

    def contraction(ma, mb, mc, ext, dtype):
        def make():
            rng = np.random.default_rng(3)
            A = rng.standard_normal([ext[c] for c in ma]).astype(dtype)
            B = rng.standard_normal([ext[c] for c in mb]).astype(dtype)
            out = h.empty([ext[c] for c in mc], dtype)
            plan = tf.HipBackend.plan(dtype, tf.PrimDescriptor.Contract(lab(ma), lab(mb), lab(mc)), [A.shape, B.shape, [ext[c] for c in mc]])
            call = h.bound_execute(plan, [h.gpu(A), h.gpu(B)], out)
            make.plan = plan
            return call
        return make
    m = contraction("ij", "jk", "ik", dict(i=64, j=64, k=64), np.float64)
    measure("Contract ij,jk->ik f64 64^3 (one launch)", m)
    lines.append("    plan.cache_stats() (hits, misses, routes kept): %r" % (m.plan.cache_stats(),))
    m = contraction("ij", "jk", "ik", dict(i=128, j=128, k=128), np.float64)
    measure("Contract ij,jk->ik f64 128^3 (split-K + fold: two launches)", m)
    lines.append("    plan.cache_stats(): %r" % (m.plan.cache_stats(),))
    m = contraction("ajbk", "kcj", "abc", dict(a=64, j=128, b=64, k=96, c=256), np.float32)
    measure("configuration 1 (pack of B, tables, split-K 8)", m)
    lines.append("    plan.cache_stats(): %r  (a route with an operand pack is not kept: every call routes)" % (m.plan.cache_stats(),))

    def grouped():
        rng = np.random.default_rng(4)
        dims = [(int(rng.integers(8, 40)), int(rng.integers(8, 40)), int(rng.integers(8, 40))) for _ in range(1024)]
        As = [h.gpu(rng.standard_normal((i, j))) for i, j, k in dims]
        Bs = [h.gpu(rng.standard_normal((j, k))) for i, j, k in dims]
        outs = [h.empty((i, k), np.float64) for i, j, k in dims]
        plan = tf.HipBackend.plan_grouped(np.float64, tf.PrimDescriptor.Contract(lab("ij"), lab("jk"), lab("ik")),
                                          [[[i, j], [j, k], [i, k]] for i, j, k in dims])
        pairs = list(zip(As, Bs))
        # marshalled once: the views of all 1024 problems
        views = (tf.tfh_view * (2 * len(dims)))(*[tf.view_of(t) for pr in pairs for t in pr])
        vouts = (tf.tfh_view * len(dims))(*[tf.view_of(t) for t in outs])
        al, be = tf._scalar_c(plan.dtype, 1.0), tf._scalar_c(plan.dtype, 0.0)
        st = tf.current_stream()

        def call():
            rc = L.tfh_execute_grouped(plan._h, al, views, 2, be, vouts, st)
            if rc:
                tf._check(rc)
        call.keep = (views, vouts, al, be, pairs, outs, plan)
        return call
    measure("grouped plan, 1024 problems of 8..40 (f64)", grouped, n=100)
    print("\n".join(lines))
    # the same from C, without the interpreter and ctypes between the calls (tests/cpp/host_overhead.cpp, built by
    # __graft_entry__.build())
    prog = os.path.join(ROOT, "tests", "cpp", "host_overhead")
    if os.path.exists(prog):
        import subprocess
        torch.cuda.synchronize()
        print("\nfrom C (tests/cpp/host_overhead):")
        sys.stdout.flush()
        subprocess.run([prog], check=False)


LAYOUT_NOTE = {False: "; operands and result row-major", True: "; operands and result column-major (MemoryOrder::ColumnMajor, the order of the reference's examples)"}
RUNNERS = {"c1": run_c1, "c2": run_c2, "c3": run_c3, "c4": run_c4, "c0": run_matmul,
           "b64": lambda h, cm=False, ref_out=None: run_batched(h, np.float64, 4096, 64, cm, ref_out),
           "b128": lambda h, cm=False, ref_out=None: run_batched(h, np.complex128, 1024, 128, cm, ref_out)}
HAS_LAYOUTS = ("c0", "c1", "c3", "c4", "b64", "b128")   # configurations that are also run column-major
HEADLINE = "c3"   # the largest configuration that fits one GPU


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--configs", default="c3,c1,c2,c4,c0,b64,b128")
    ap.add_argument("--no-colmajor", action="store_true", help="skip the column-major variants of the configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline / parity leg")
    ap.add_argument("--sweep-ops", default="permute,reduce", help="operations of --shape-sweep (permute, reduce)")
    ap.add_argument("--sweep-dtypes", default="f32,f64,c64,c128", help="dtypes of --shape-sweep")
    ap.add_argument("--sweep-mb", type=int, default=128, help="least size of a tensor of --shape-sweep, in MB")
    ap.add_argument("--shape-sweep", action="store_true",
                    help="permutes and reductions of seeded random tensors (rank 3..7, >= 128 MB, extents that are no powers of two)")
    ap.add_argument("--host-overhead", action="store_true",
                    help="print the host cost of tfh_execute per call (first against repeated) instead of running the benchmark")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also launch three plain 1 GiB device-to-device copies (torch's elementwise copy kernel): under "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE their readings give the counter's scale for known traffic")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.stderr.write("bench.py: this build runs on ONE GPU (no collectives, no sharding); --gpus %d is not supported\n" % args.gpus)
        sys.exit(2)
    h = Harness(args.steps, args.warmup, not args.no_cpu and not args.host_overhead and not args.shape_sweep)
    if args.shape_sweep:
        shape_sweep(h, min_bytes=args.sweep_mb << 20, ops=tuple(args.sweep_ops.split(",")), dtypes=tuple(args.sweep_dtypes.split(",")))
        return
    if args.host_overhead:
        host_overhead(h)
        return
    if args.pmc_calibration:
        src = h.torch.ones(1 << 28, dtype=h.torch.float32, device="cuda")
        dst = h.torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        h.torch.cuda.synchronize()
        del src, dst
    wanted = [c.strip() for c in args.configs.split(",") if c.strip()]
    if HEADLINE not in wanted:
        wanted.insert(0, HEADLINE)
    results = {}
    def release():
        h.torch.cuda.synchronize()
        h.torch.cuda.empty_cache()
        h.tf.lib().tfh_release_workspaces()
    for name in wanted:
        results[name] = RUNNERS[name](h)
        release()
        if name in HAS_LAYOUTS and not args.no_colmajor:
            # the same configuration with every operand and the result column-major; its result is checked against the
            # row-major run's (which the CPU oracle has checked), its fraction of the roofline is reported beside it
            r = RUNNERS[name](h, True, results[name]["_out"])
            base = results[name]
            r["vs_row_major"] = {"ms_per_step_ratio": r["ms_per_step"] / base["ms_per_step"],
                                 "roofline_frac": r["roofline"]["frac"], "row_major_roofline_frac": base["roofline"]["frac"]}
            r.pop("_out", None)
            results[name + "_colmajor"] = r
            release()
        results[name].pop("_out", None)
    top = results[HEADLINE]
    line = {
        "metric": METRIC, "value": top["value"], "unit": top["unit"], "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": top["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": top["dtype"], "data": "synthetic",
        "config": {"workload": "config 3: " + top["workload"],
                   "inputs": "seeded complex N(0, 1/chi), resident in HBM (268 MB + 34 MB + 34 MB operands, 268 MB output, two 537 MB intermediates)",
                   "spinup_s": SPINUP_S,
                   "kernel_timing": "the K timed steps carry no events; the per-kernel durations of `roofline` come from a second "
                                    "pass of K steps with a pair of HIP events around each dominant kernel on its own stream"},
        "roofline": top["roofline"],
        "cpu_baseline": top.get("cpu_baseline"),
        "parity": top.get("parity"),
        "all_configs": results,
    }
    print(json.dumps(line))
    bad = []
    for name, r in results.items():
        p = r.get("parity") or {}
        for k, v in p.items():
            if k.endswith("frobenius") and v > p["tolerance"]:
                bad.append((name, k, v))
            if k.endswith("bit_exact") and not v:
                bad.append((name, k, v))
    if bad:
        sys.stderr.write("PARITY FAILURE: %r\n" % bad)
        sys.exit(1)


if __name__ == "__main__":
    main()

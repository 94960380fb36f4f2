#!/usr/bin/env python3
"""Benchmark of the annotated-loop hot path on one MI355X.

``python bench.py [--gpus 1] [--steps K] [--warmup W]`` prints ONE JSON line.

Headline (``value``): achieved HBM GB/s of the ``shared()`` scalar reduction
``vector_sum`` over float32 N = 2^28 (1 GiB), inputs resident in HBM, one step
= clear the float64 accumulator + one launch of the generated kernel, timed
over K steps between device synchronisations.  ``roofline`` gives the same
kernel's algorithmic bytes per launch divided by its mean launch duration
measured with HIP events on the launch stream, against the 8 TB/s HBM peak.
``kernels`` lists the same figures for the other generated kernels
(vec_add at 2^24 and 2^27, masked_sum, GEMV, CSR SpMV uniform and power-law, CSR SpMM), each
checked against the float64 oracle on the identical inputs in the same run; a launch
that is a sequence of kernels (CSR loops) is timed as a whole.  The CSR SpMV workloads are
measured twice: with every launch reading the raw arrays (``kernel_ms`` / ``frac`` /
``ms_no_reuse``, the figure of record, which ``roofline.frac_configs_1_4`` uses; ``first_launch_ms``
is the form a launch takes that knows nothing of its rows yet), and with the order of the elements
worked out once and kept between launches, as launches on unchanged GPU tensors run from their second
sighting on (``inspector_ms`` once, then ``ms_reused`` / ``frac_reused`` per launch).
``roofline`` also says which kernel of configs 1-4 is furthest from the roofline and
which of their bars are met.  HBM traffic per launch comes from the committed
summary of the rocprofv3 counter runs of this program (``profiles/``).
``cpu_baseline`` times the oracle (NumPy, one core) on the host.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_BPS = 8.0e12  # MI355X HBM3E, bytes per second

# HBM traffic per launch at the default sizes is not measured in a bench run (counters are
# collected in runs of their own): it is read from the committed summary of the rocprofv3 counter
# runs of this same program, which names the kernel shape each figure belongs to.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "bench_kernels_pmc_fetch_write_size.txt")


def load_profile_traffic(path=TRAFFIC_PROFILE):
    """{workload: (kernel shape tag, bytes per launch)} from the lines
    ``traffic <workload> spec=<tag> fetch_kib=<FETCH_SIZE> write_kib=<WRITE_SIZE>`` of the profile
    summary, scaled by its ``calibration fetch_scale=<f> write_scale=<f>`` line (what the two
    counters read for the plain copy kernel of known size)."""
    out, fs, ws = {}, None, None
    try:
        with open(path) as fh:
            lines = fh.read().splitlines()
    except OSError:
        return out
    for ln in lines:
        parts = ln.split()
        if parts[:1] == ["calibration"]:
            kv = dict(p.split("=", 1) for p in parts[1:] if "=" in p)
            fs, ws = float(kv["fetch_scale"]), float(kv["write_scale"])
    if fs is None:
        return out
    for ln in lines:
        parts = ln.split()
        if parts[:1] == ["traffic"] and len(parts) >= 5:
            kv = dict(p.split("=", 1) for p in parts[2:] if "=" in p)
            out[parts[1]] = (kv["spec"], int((float(kv["fetch_kib"]) * fs + float(kv["write_kib"]) * ws) * 1024))
    return out


REQUESTS_PROFILE = os.path.join(ROOT, "profiles", "bench_kernels_pmc_read_requests.txt")


def load_profile_requests(path=REQUESTS_PROFILE):
    """{workload: (kernel shape tag, L2 requests per launch)} from the lines
    ``<workload> spec=<tag> ... L2_requests=<TCC_REQ>`` of the summary of the request counter runs."""
    out = {}
    try:
        with open(path) as fh:
            lines = fh.read().splitlines()
    except OSError:
        return out
    for ln in lines:
        parts = ln.split()
        if len(parts) > 2 and parts[1].startswith("spec=") and "L2_requests=" in ln:
            kv = {}
            for i, p in enumerate(parts):
                if p.endswith("=") and i + 1 < len(parts):
                    kv[p[:-1]] = parts[i + 1]
                elif "=" in p:
                    a, b = p.split("=", 1)
                    kv[a] = b
            out[parts[0]] = (kv["spec"], int(kv["L2_requests"]))
    return out


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=50)
    p.add_argument("--warmup", type=int, default=5)
    p.add_argument("--workloads", default="vector_sum,masked_sum,copy,vec_add,vec_add_2p27,gemv,gemv_columns,gather,spmv_uniform,spmv_powerlaw,spmv_powerlaw16,spmm",
                   help="comma separated subset; vector_sum is always run (headline) unless --no-headline is given")
    p.add_argument("--no-headline", action="store_true",
                   help="profiling runs of single workloads: do not add vector_sum (the JSON line then has no headline)")
    p.add_argument("--spmv-forms", default="both", choices=("both", "no_reuse", "reused"),
                   help="profiling runs: measure the CSR SpMV workloads only with launches that read the raw arrays, "
                        "or only with the kept order of the elements")
    p.add_argument("--no-first-launch", action="store_true",
                   help="profiling runs: do not time the form a CSR SpMV launch takes before anything is known of its rows "
                        "(its kernels share their names with those of the later launches)")
    p.add_argument("--scale", type=float, default=1.0, help="shrink every size by this factor (debugging)")
    p.add_argument("--no-cpu-baseline", action="store_true")
    return p.parse_args()


class Runner:
    """Times one compiled loop on resident inputs."""

    def __init__(self, torch, rt, cg):
        self.torch, self.rt, self.cg = torch, rt, cg

    def loop_of(self, before):
        new = [k for k in self.cg.code_cache if k not in before]
        assert len(new) == 1, f"expected one new compiled loop, got {len(new)}"
        return self.cg.code_cache[new[0]][0]

    def measure(self, loop, vals, nbytes, steps, warmup, clear=None):
        """Returns dict(ms_per_step, gbps_step, kernel_ms, gbps_kernel, frac, spec, grid)."""
        torch, rt = self.torch, self.rt
        launch = loop.prepare(vals)

        def step():
            if clear is not None:
                clear.zero_()           # fill kernel on the same (current) stream
            launch.launch_only()

        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / steps
        # kernel time from HIP events on the launch stream: five batches of back-to-back
        # launches (short kernels need many launches between two events); median and
        # minimum of the batch means
        reps = max(20, min(steps, 50))
        batches = sorted(launch.time_kernel(warmup=2, reps=reps) for _ in range(5))
        kernel_ms = batches[len(batches) // 2]
        info = rt.func_info(launch.function())
        return {
            "ms_per_step": dt * 1e3,
            "gbps_step": nbytes / dt / 1e9,
            "kernel_ms": kernel_ms,
            "kernel_ms_min": batches[0],
            "kernel_launches_timed": 5 * reps,
            "gbps_kernel": nbytes / (kernel_ms * 1e-3) / 1e9,
            "frac": nbytes / (kernel_ms * 1e-3) / HBM_PEAK_BPS,
            "algorithmic_bytes": int(nbytes),
            "spec": launch.spec.tag(),
            "grid": launch.grid[0],
            "vgprs": info["num_vgprs"],
            "scratch_bytes": info["scratch_bytes"],
        }


def _blas_threads():
    """Threads NumPy's BLAS may use (only `A @ x` of the per-kernel CPU figures is multi-threaded)."""
    try:
        from threadpoolctl import threadpool_info

        return max([p.get("num_threads", 1) for p in threadpool_info() if p.get("user_api") == "blas"] or [1])
    except Exception:
        return int(os.environ.get("OMP_NUM_THREADS", "0")) or None


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as fh:
            for line in fh:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return None


def cpu_time(fn, reps=3):
    """Best wall time of ``fn`` over ``reps`` runs, seconds."""
    best = 1e30
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        best = min(best, time.perf_counter() - t0)
    return best


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported in this build "
              "(every kernel here is a single-device kernel)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import __graft_entry__

    __graft_entry__.ensure_built()      # loads what is built; builds only if nothing is
    from appy_amd.backends.hip import codegen as cg
    from appy_amd.backends.hip import runtime as rt
    from appy_amd.backends.hip import selfcheck
    from oracle import loops as olo
    from oracle import vectorised as vo
    from oracle import workloads as wl
    from oracle.device_workloads import device_csr

    if not torch.cuda.is_available() or rt.device_count() < 1:
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    props = rt.device_props(0)
    log(f"device: {props['name']} {props['arch']} CUs={props['compute_units']} HBM={props['hbm_bytes'] / 2**30:.0f} GiB")

    k = selfcheck.kernels()
    run = Runner(torch, rt, cg)
    want = set(args.workloads.split(","))
    if not args.no_headline:
        want.add("vector_sum")
    sc = args.scale
    results = {}
    parity = {}
    K, W = args.steps, args.warmup

    def shrink(n, lo=1024):
        return max(lo, int(n * sc))

    # ---------------- config 2a / 2b: shared() scalar reductions ----------------------
    s_d = torch.zeros(1, dtype=torch.float64, device="cuda")
    cpu_baseline = None
    cpu_kernels = {}
    do_cpu = not args.no_cpu_baseline
    n = shrink(1 << 28)
    if {"vector_sum", "masked_sum"} & want:
        t0 = time.time()
        A, M = wl.reduce_inputs(n)
        log(f"reduce inputs N={n} generated in {time.time() - t0:.1f}s")
        A_d = torch.from_numpy(A).cuda()

        before = set(cg.code_cache)
        got = k.vector_sum(A_d)                                # product path end to end
        loop = run.loop_of(before)
        ref, budget = vo.vector_sum(A)
        parity["vector_sum"] = {"abs_err": abs(got - ref), "bound": vo.TOL * budget, "ok": abs(got - ref) <= vo.TOL * budget}
        results["vector_sum"] = run.measure(loop, {"s": s_d, "A": A_d, "A_shape_0": n}, 4 * n + 8, K, W, clear=s_d)
        # end-to-end call of the decorated function (shared scalar travels host<->device)
        # (steady state: the mean of 50 calls after three that are not timed; every call waits for its result)
        for _ in range(3):
            k.vector_sum(A_d)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(50):
            k.vector_sum(A_d)
        results["vector_sum"]["jit_call_ms"] = (time.perf_counter() - t0) / 50 * 1e3
        log("vector_sum", results["vector_sum"], parity["vector_sum"])

        if not args.no_cpu_baseline:
            # oracle (NumPy float64 accumulation, one core) on the full array, best of 3,
            # and the literal interpreter loop on a 2^20 sample
            best = 1e30
            for _ in range(3):
                t0 = time.perf_counter()
                A.sum(dtype=np.float64)
                best = min(best, time.perf_counter() - t0)
            m = min(n, 1 << 20)
            t0 = time.perf_counter()
            olo.vector_sum(A[:m])
            lit = (time.perf_counter() - t0) / m * 1e9
            cpu_baseline = {
                "value": (4 * n + 8) / best / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"oracle A.sum(dtype=float64) over all N={n} float32, best of 3 ({best * 1e3:.1f} ms); "
                          f"literal interpreter loop on the first {m} elements: {lit:.0f} ns/element",
                "host_cpus": os.cpu_count(), "affinity": len(os.sched_getaffinity(0)),
                "blas_threads": _blas_threads(), "cpu_model": _cpu_model(),
            }
            log("cpu_baseline", cpu_baseline)

        if "masked_sum" in want:
            M_d = torch.from_numpy(M).cuda()
            before = set(cg.code_cache)
            got = k.masked_sum(A_d, M_d)
            loop = run.loop_of(before)
            ref, budget = vo.masked_sum(A, M)
            parity["masked_sum"] = {"abs_err": abs(got - ref), "bound": vo.TOL * budget, "ok": abs(got - ref) <= vo.TOL * budget}
            results["masked_sum"] = run.measure(loop, {"s": s_d, "A": A_d, "M": M_d, "A_shape_0": n}, 5 * n + 8, K, W, clear=s_d)
            log("masked_sum", results["masked_sum"], parity["masked_sum"])
            if do_cpu:
                t = cpu_time(lambda: np.where(M, A, np.float32(0)).sum(dtype=np.float64), 2)
                cpu_kernels["masked_sum"] = {"ms": t * 1e3, "gbps": (5 * n + 8) / t / 1e9,
                                             "what": "np.where(M, A, 0).sum(dtype=float64), full size, 1 core"}
            del M_d
        del A_d, A, M
        torch.cuda.empty_cache()

    # ---------------- calibration: plain copy of known size -------------------------------
    # c[i] = a[i] over 2^28 float32: 1 GiB read + 1 GiB written.  Used to scale the
    # FETCH_SIZE / WRITE_SIZE counters of profiling runs and as the streaming reference.
    if "copy" in want:
        nc = shrink(1 << 28)
        a_d = torch.empty(nc, dtype=torch.float32, device="cuda").uniform_(-1, 1)
        c_d = torch.empty_like(a_d)
        before = set(cg.code_cache)
        selfcheck.kernels().copy(a_d, c_d)
        loop = run.loop_of(before)
        ok = bool(torch.equal(a_d, c_d))
        parity["copy"] = {"bit_exact": ok, "ok": ok}
        results["copy"] = run.measure(loop, {"c": c_d, "a": a_d, "a_shape_0": nc}, 8 * nc, K, W)
        log("copy", results["copy"], parity["copy"])
        del a_d, c_d
        torch.cuda.empty_cache()

    # ---------------- config 1: vec_add ---------------------------------------------------
    if "vec_add" in want:
        n1 = shrink(1 << 24)
        a, b = wl.vec_add(n1)
        a_d, b_d = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
        before = set(cg.code_cache)
        c_d = k.vec_add(a_d, b_d)
        loop = run.loop_of(before)
        ok = bool(np.array_equal(c_d.cpu().numpy(), vo.vec_add(a, b)))
        parity["vec_add"] = {"bit_exact": ok, "ok": ok}
        results["vec_add"] = run.measure(loop, {"c": c_d, "a": a_d, "b": b_d, "a_shape_0": n1}, 12 * n1, K, W)
        log("vec_add", results["vec_add"], parity["vec_add"])
        if do_cpu:
            out = np.empty_like(a)
            t = cpu_time(lambda: np.add(a, b, out=out), 5)
            m1 = min(n1, 1 << 20)
            t0 = time.perf_counter()
            olo.vec_add(a[:m1], b[:m1])
            cpu_kernels["vec_add"] = {"ms": t * 1e3, "gbps": 12 * n1 / t / 1e9, "what": "np.add(a, b, out=c), full size, 1 core",
                                      "literal_loop_ns_per_element": (time.perf_counter() - t0) / m1 * 1e9}
        del a_d, b_d, c_d

    # ---------------- config 1 beyond the memory-side cache: N = 2^27 (1.5 GiB touched) -------
    # (at the config's own N = 2^24 the three arrays, 192 MiB, fit the 256 MiB memory-side cache and
    #  are relaunched in place; this row shows the same kernel on streams that cannot be served from it)
    if "vec_add_2p27" in want:
        n7 = shrink(1 << 27)
        a_d = torch.empty(n7, dtype=torch.float32, device="cuda").uniform_(-1, 1)
        b_d = torch.empty(n7, dtype=torch.float32, device="cuda").uniform_(-1, 1)
        before = set(cg.code_cache)
        c_d = k.vec_add(a_d, b_d)
        new_loops = [kk for kk in cg.code_cache if kk not in before]
        loop = cg.code_cache[new_loops[0]][0] if new_loops else [v[0] for kk, v in cg.code_cache.items() if kk[-1] == "vec_add"][-1]
        ok = bool(torch.equal(c_d, a_d + b_d))
        parity["vec_add_2p27"] = {"bit_exact": ok, "ok": ok}
        results["vec_add_2p27"] = run.measure(loop, {"c": c_d, "a": a_d, "b": b_d, "a_shape_0": n7}, 12 * n7, K, W)
        log("vec_add_2p27", results["vec_add_2p27"], parity["vec_add_2p27"])
        del a_d, b_d, c_d
        torch.cuda.empty_cache()

    # ---------------- config 3: GEMV ---------------------------------------------------------
    if "gemv" in want:
        r = shrink(16384, 64)
        t0 = time.time()
        Am, x = wl.gemv(r, r)
        log(f"gemv inputs {r}x{r} generated in {time.time() - t0:.1f}s")
        A_d, x_d = torch.from_numpy(Am).cuda(), torch.from_numpy(x).cuda()
        before = set(cg.code_cache)
        y_d = k.gemv(A_d, x_d)
        loop = run.loop_of(before)
        ref, budget = vo.gemv(Am, x)
        ok, worst = vo.within_budget(y_d.cpu().numpy(), ref, budget)
        parity["gemv"] = {"worst_err_over_bound": worst, "ok": ok}
        vals = {"A": A_d, "x": x_d, "y": y_d, "A_shape_0": r, "A_shape_1": r}
        results["gemv"] = run.measure(loop, vals, 4 * (r * r + r + r), K, W)
        log("gemv", results["gemv"], parity["gemv"])
        if do_cpu:
            t = cpu_time(lambda: Am @ x, 3)
            rr = min(r, 256)
            t0 = time.perf_counter()
            olo.gemv(1.0, Am[:rr, :rr], x[:rr])
            cpu_kernels["gemv"] = {"ms": t * 1e3, "gbps": 4 * (r * r + 2 * r) / t / 1e9,
                                   "what": f"A @ x (BLAS sgemv, up to {len(os.sched_getaffinity(0))} threads), full size",
                                   "literal_loop_ns_per_element": (time.perf_counter() - t0) / (rr * rr) * 1e9}
        del A_d, x_d, y_d, Am, ref, budget
        torch.cuda.empty_cache()

    # ---------------- column form of GEMV (second loop of gemver): the strip kernel shape -------
    if "gemv_columns" in want:
        r = shrink(16384, 64)
        Am, yv = wl.gemv(r, r)
        A_d, y_d = torch.from_numpy(Am).cuda(), torch.from_numpy(yv).cuda()
        before = set(cg.code_cache)
        x_d = k.gemv_columns(A_d, y_d)
        loop = run.loop_of(before)
        ref, budget = vo.gemv(Am.T, yv)
        ok, worst = vo.within_budget(x_d.cpu().numpy(), ref, budget)
        parity["gemv_columns"] = {"worst_err_over_bound": worst, "ok": ok}
        vals = {"A": A_d, "y": y_d, "x": x_d, "A_shape_0": r, "A_shape_1": r}
        results["gemv_columns"] = run.measure(loop, vals, 4 * (r * r + r + r), K, W)
        log("gemv_columns", results["gemv_columns"], parity["gemv_columns"])
        del A_d, y_d, x_d, Am, ref, budget
        torch.cuda.empty_cache()

    # ---------------- config 4: CSR SpMV -----------------------------------------------------
    def spmv_case(name, data_d, indptr_d, indices_d, x_d, m, ncol):
        import appy_amd as appy

        nnz = data_d.numel()
        nbytes = 8 * nnz + 4 * (m + 1) + 4 * ncol + 4 * m
        t0 = time.time()
        h_data, h_ptr, h_idx, h_x = (data_d.cpu().numpy(), indptr_d.cpu().numpy(), indices_d.cpu().numpy(),
                                      x_d.cpu().numpy())
        ref, budget = vo.spmv_csr(h_data, h_ptr, h_idx, h_x, (m, ncol))
        log(f"{name}: oracle in {time.time() - t0:.1f}s")
        if do_cpu:
            import scipy.sparse as sp

            A32 = sp.csr_matrix((h_data, h_idx, h_ptr), shape=(m, ncol))
            t = cpu_time(lambda: A32 @ h_x, 2)
            mm = min(m, 1 << 12)
            t0 = time.perf_counter()
            olo.spmv_csr(h_data, h_ptr, h_idx, h_x, mm, ncol)
            cpu_kernels[name] = {"ms": t * 1e3, "gbps": nbytes / t / 1e9,
                                 "what": "scipy.sparse.csr_matrix (float32) @ x, full size, 1 core",
                                 "literal_loop_ns_per_nnz": (time.perf_counter() - t0) / max(1, int(h_ptr[mm])) * 1e9}
            del A32
        del h_data, h_ptr, h_idx, h_x
        lens = (indptr_d[1:] - indptr_d[:-1])
        worst_all, ok_all = 0.0, True

        def check(y_d):
            nonlocal worst_all, ok_all
            ok, worst = vo.within_budget(y_d.cpu().numpy(), ref, budget)
            worst_all, ok_all = max(worst_all, worst), bool(ok_all and ok)

        def steps_of(launch):
            seq = launch.sequence
            return sum(1 for step in seq if step[0] is not None) if seq else 1

        def loop_for(kernels, reuse):
            before = set(cg.code_cache)
            y_d = kernels.spmv(data_d, indptr_d, indices_d, x_d, m, ncol)
            new = [kk for kk in cg.code_cache if kk not in before]
            if new:
                spmv_case.loops[reuse] = cg.code_cache[new[0]][0]
            return spmv_case.loops[reuse], y_d

        rec = {"nnz": int(nnz), "rows": m, "mean_row": float(nnz) / m, "max_row": int(lens.max().item())}
        if args.spmv_forms in ("both", "no_reuse"):
            # every launch reads the raw arrays: the figure of record
            loop, y_d = loop_for(selfcheck.kernels(hip_reuse=False), False)
            check(y_d)
            vals = {"A_data": data_d, "A_indptr": indptr_d, "A_indices": indices_d, "x": x_d, "y": y_d, "M": m}
            # a launch that has been told nothing about the lengths of its rows (the first launch of a loop over these arrays)
            if not args.no_first_launch:
                loop._hint_key.clear()
                first = loop.prepare(vals)
                firsts = sorted(first.time_kernel(warmup=1, reps=10) for _ in range(3))
                torch.cuda.synchronize()
                check(y_d)
                rec.update({"first_launch_ms": firsts[1], "first_launch_kernels": steps_of(first)})
            # and the launches after it, which leave out the kernels that would run empty
            y_d = selfcheck.kernels(hip_reuse=False).spmv(data_d, indptr_d, indices_d, x_d, m, ncol)
            torch.cuda.synchronize()
            vals["y"] = y_d
            rec.update(run.measure(loop, vals, nbytes, K, W))
            check(y_d)
            rec.update({"ms_no_reuse": rec["kernel_ms"],
                        "kernels_per_launch": steps_of(loop.last_launch),
                        "giga_nnz_per_s": nnz / rec["kernel_ms"] / 1e6, "scratch_bytes_device": loop.scratch_bytes(0)})
            loop.release()
        if args.spmv_forms in ("both", "reused"):
            # unchanged GPU tensors seen a second time: the order of the elements is worked out (inspector) and kept
            loop, y_d = loop_for(selfcheck.kernels(), True)
            check(y_d)
            y_d = selfcheck.kernels().spmv(data_d, indptr_d, indices_d, x_d, m, ncol)
            torch.cuda.synchronize()
            check(y_d)
            plan = loop.last_launch.plan
            assert plan is not None, "no row plan was built"
            inspector_ms = [plan.inspector_ms]
            if not args.no_first_launch:
                # once more: the first inspector run of a process also loads the code of the library's sort for this size
                loop.release_plans()
                for _ in range(2):
                    y_d = selfcheck.kernels().spmv(data_d, indptr_d, indices_d, x_d, m, ncol)
                torch.cuda.synchronize()
                check(y_d)
                plan = loop.last_launch.plan
                assert plan is not None, "no row plan was built"
                inspector_ms.append(plan.inspector_ms)
            vals = {"A_data": data_d, "A_indptr": indptr_d, "A_indices": indices_d, "x": x_d, "y": y_d, "M": m}
            r = run.measure(loop, vals, nbytes, K, W)
            check(y_d)
            assert loop.last_launch.plan is plan
            reused = {"inspector_ms": min(inspector_ms), "inspector_ms_first_in_process": inspector_ms[0], "ms_reused": r["kernel_ms"], "ms_reused_min": r["kernel_ms_min"],
                      "frac_reused": r["frac"], "gbps_reused": r["gbps_kernel"], "giga_nnz_per_s_reused": nnz / r["kernel_ms"] / 1e6,
                      "spec_reused": r["spec"], "grid_reused": r["grid"], "vgprs_reused": r["vgprs"],
                      "kernels_per_launch_reused": steps_of(loop.last_launch),
                      "plan_bytes_device": plan.nbytes, "scratch_bytes_device_reused": loop.scratch_bytes(0)}
            if "kernel_ms" not in rec:
                rec.update(r)           # a run of the reused form only: its figures stand for the workload
            rec.update(reused)
            if rec.get("ms_no_reuse", 0) > reused["ms_reused"]:
                # launches after which working the order out has paid for itself
                rec["inspector_break_even_launches"] = reused["inspector_ms"] / (rec["ms_no_reuse"] - reused["ms_reused"])
            loop.release()
        rec["forms"] = ("kernel_ms, frac, ms_no_reuse, first_launch_ms: every launch reads the raw arrays (hip_reuse=False); "
                        "inspector_ms once, then ms_reused, frac_reused per launch: the kept order of the elements "
                        "(the default for unchanged GPU tensors from their second launch on)")
        results[name] = rec
        parity[name] = {"worst_err_over_bound": worst_all, "ok": ok_all}
        log(name, results[name], parity[name])
        appy.release()

    # ---------------- calibration: random gathers without rows ---------------------------------
    # s += v[i] * x[idx[i]] over 2^26 (value, index) pairs with uniformly random indices into
    # 2^22 floats: the memory behaviour of a CSR SpMV that walks the uniform matrix row by row (8 streamed
    # bytes and one 4-byte gather from a 16 MiB vector per non-zero) without its row structure.
    if "gather" in want:
        ng, nx = shrink(1 << 26), shrink(1 << 22)
        gx = torch.Generator(device="cuda"); gx.manual_seed(43)
        v_d = torch.randn(ng, generator=gx, device="cuda", dtype=torch.float32)
        idx_d = torch.randint(0, nx, (ng,), generator=gx, device="cuda", dtype=torch.int32)
        xg_d = torch.randn(nx, generator=gx, device="cuda", dtype=torch.float32)
        before = set(cg.code_cache)
        got = k.gather_dot(v_d, idx_d, xg_d)
        loop = run.loop_of(before)
        ref, budget = vo.gather_dot(v_d.cpu().numpy(), idx_d.cpu().numpy(), xg_d.cpu().numpy())
        parity["gather"] = {"abs_err": abs(got - ref), "bound": vo.TOL * budget, "ok": abs(got - ref) <= vo.TOL * budget}
        vals = {"s": s_d, "v": v_d, "idx": idx_d, "x": xg_d, "v_shape_0": ng}
        results["gather"] = run.measure(loop, vals, 8 * ng + 4 * nx + 8, K, W, clear=s_d)
        results["gather"]["giga_gathers_per_s"] = ng / results["gather"]["kernel_ms"] / 1e6
        log("gather", results["gather"], parity["gather"])
        del v_d, idx_d, xg_d
        torch.cuda.empty_cache()

    spmv_case.loops = {}
    if {"spmv_uniform", "spmv_powerlaw", "spmv_powerlaw16"} & want and args.spmv_forms != "no_reuse":
        # a small plan first: the library loads the code of its inspector kernels when they are first launched,
        # which is not what `inspector_ms` is about
        mw = 1 << 16
        dw, pw, iw = device_csr(torch, np.full(mw, 8, dtype=np.int64), 1 << 20, seed=3)
        xw = torch.randn(1 << 20, device="cuda", dtype=torch.float32)
        warm = selfcheck.kernels(hip_reuse="now")
        warm.spmv(dw, pw, iw, xw, mw, 1 << 20)
        torch.cuda.synchronize()
        del dw, pw, iw, xw
    if "spmv_uniform" in want:
        m4 = shrink(1 << 22)
        lengths = np.full(m4, 16, dtype=np.int64)
        data_d, indptr_d, indices_d = device_csr(torch, lengths, m4, seed=4)
        gx = torch.Generator(device="cuda"); gx.manual_seed(40)
        x_d = torch.randn(m4, generator=gx, device="cuda", dtype=torch.float32)
        spmv_case("spmv_uniform", data_d, indptr_d, indices_d, x_d, m4, m4)
        del data_d, indptr_d, indices_d, x_d
        torch.cuda.empty_cache()
    if "spmv_powerlaw" in want:
        m4 = shrink(1 << 22)
        rng = np.random.default_rng(104)
        lengths = np.clip(rng.zipf(1.5, m4), 1, min(4096, m4)).astype(np.int64)
        t0 = time.time()
        data_d, indptr_d, indices_d = device_csr(torch, lengths, m4, seed=5)
        log(f"power-law CSR nnz={data_d.numel()} built in {time.time() - t0:.1f}s")
        gx = torch.Generator(device="cuda"); gx.manual_seed(41)
        x_d = torch.randn(m4, generator=gx, device="cuda", dtype=torch.float32)
        spmv_case("spmv_powerlaw", data_d, indptr_d, indices_d, x_d, m4, m4)
        del data_d, indptr_d, indices_d, x_d
        torch.cuda.empty_cache()

    if "spmv_powerlaw16" in want:
        # same recipe with exponent 1.79: the power-law matrix whose mean row length is the
        # 16 non-zeros the config text quotes (exponent 1.5 with clip 4096 gives a mean of 97)
        m4 = shrink(1 << 22)
        rng = np.random.default_rng(105)
        lengths = np.clip(rng.zipf(1.79, m4), 1, min(4096, m4)).astype(np.int64)
        data_d, indptr_d, indices_d = device_csr(torch, lengths, m4, seed=7)
        log(f"power-law(1.79) CSR nnz={data_d.numel()}")
        gx = torch.Generator(device="cuda"); gx.manual_seed(42)
        x_d = torch.randn(m4, generator=gx, device="cuda", dtype=torch.float32)
        spmv_case("spmv_powerlaw16", data_d, indptr_d, indices_d, x_d, m4, m4)
        del data_d, indptr_d, indices_d, x_d
        torch.cuda.empty_cache()

    # ---------------- config 5: CSR SpMM -------------------------------------------------------
    if "spmm" in want:
        m5 = shrink(1 << 20)
        rng = np.random.default_rng(5)
        lengths = np.minimum(rng.poisson(32, m5), m5).astype(np.int64)
        data_d, indptr_d, indices_d = device_csr(torch, lengths, m5, seed=6)
        gx = torch.Generator(device="cuda"); gx.manual_seed(42)
        B_d = torch.randn((m5, 128), generator=gx, device="cuda", dtype=torch.float32)
        Y_d = torch.empty((m5, 128), device="cuda", dtype=torch.float32)
        before = set(cg.code_cache)
        k.spmm(data_d, indptr_d, indices_d, B_d, Y_d, m5)
        loop = run.loop_of(before)
        # oracle on a row sample (the full float64 product needs ~10 s of one core)
        rows = np.unique(np.concatenate([np.arange(min(m5, 4096)), rng.integers(0, m5, 4096)]))
        ip = indptr_d.cpu().numpy().astype(np.int64)
        sel = np.concatenate([np.arange(ip[r0], ip[r0 + 1]) for r0 in rows]) if len(rows) else np.empty(0, np.int64)
        sub_ptr = np.zeros(len(rows) + 1, dtype=np.int64)
        np.cumsum(ip[rows + 1] - ip[rows], out=sub_ptr[1:])
        ref, budget = vo.spmm_csr(data_d.cpu().numpy()[sel], sub_ptr, indices_d.cpu().numpy()[sel],
                                  B_d.cpu().numpy(), (len(rows), m5))
        ok, worst = vo.within_budget(Y_d.cpu().numpy()[rows], ref, budget)
        parity["spmm"] = {"worst_err_over_bound": worst, "ok": ok, "rows_checked": int(len(rows))}
        if do_cpu:
            import scipy.sparse as sp

            # bounded sample: the first 2^16 rows of A against all of B (the full product needs ~10 s of one core)
            ms_rows = min(m5, 1 << 16)
            e = int(ip[ms_rows])
            Asub = sp.csr_matrix((data_d[:e].cpu().numpy(), indices_d[:e].cpu().numpy(), ip[:ms_rows + 1]), shape=(ms_rows, m5))
            Bh = B_d.cpu().numpy()
            t = cpu_time(lambda: Asub @ Bh, 2)
            sub_bytes = 8 * e + 4 * (ms_rows + 1) + 512 * m5 + 512 * ms_rows
            cpu_kernels["spmm"] = {"ms": t * 1e3, "gbps": sub_bytes / t / 1e9,
                                   "what": f"scipy csr (float32) @ B on the first {ms_rows} rows (nnz {e}), 1 core"}
            del Asub, Bh
        nnz = data_d.numel()
        nbytes = 8 * nnz + 4 * (m5 + 1) + 4 * m5 * 128 + 4 * m5 * 128
        vals = {"A_data": data_d, "A_indptr": indptr_d, "A_indices": indices_d, "B": B_d, "y": Y_d, "M": m5}
        results["spmm"] = run.measure(loop, vals, nbytes, max(5, K // 5), min(W, 2))
        results["spmm"].update({"nnz": int(nnz), "gather_model_bytes": int(nnz * (8 + 512) + 4 * (m5 + 1) + 512 * m5)})
        log("spmm", results["spmm"], parity["spmm"])

    traffic = load_profile_traffic() if sc == 1.0 else {}
    for name, r in results.items():
        # HBM traffic per launch from the committed counter runs, if they were made with this kernel shape
        spec_tag, nbytes_prof = traffic.get(name, (None, None))
        r["traffic_profile_spec"] = spec_tag
        r["traffic_bytes_rocprof"] = nbytes_prof if spec_tag == r["spec"] else None
        if "spec_reused" in r:
            tag2, nbytes2 = traffic.get(name + "_reused", (None, None))
            r["traffic_bytes_rocprof_reused"] = nbytes2 if tag2 == r["spec_reused"] else None
    # L2 requests per second of the launches whose request counts the committed counter runs hold (same kernel
    # shape), against one request per L2 channel and clock (16 channels in each of 8 XCDs)
    requests = load_profile_requests() if sc == 1.0 else {}
    l2_peak = 128 * props["clock_khz"] * 1e3
    for name, r in results.items():
        for suffix, spec_key, ms_key in (("", "spec", "kernel_ms"), ("_reused", "spec_reused", "ms_reused")):
            tag, nreq = requests.get(name + suffix, (None, None))
            if tag is not None and tag == r.get(spec_key) and r.get(ms_key):
                r["l2_requests_per_launch" + suffix] = nreq
                r["l2_requests_per_s" + suffix] = nreq / (r[ms_key] * 1e-3)
                r["l2_request_rate_frac" + suffix] = nreq / (r[ms_key] * 1e-3) / l2_peak
    all_ok = all(p["ok"] for p in parity.values())
    # the bar of the goal: every generated kernel of configs 1-4 against the HBM roofline
    bar = {"vec_add": 0.85, "vector_sum": 0.85, "masked_sum": 0.85, "gemv": 0.70, "spmv_uniform": 0.70, "spmv_powerlaw": 0.70}
    measured = {name: results[name]["frac"] for name in bar if name in results}
    worst = min(measured, key=measured.get) if measured else None
    head = results.get("vector_sum")
    line = {
        "metric": "achieved HBM GB/s of the generated shared()-reduction kernel (vector_sum), 1 GPU",
        "value": head["gbps_step"] if head else None,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": head["ms_per_step"] if head else None,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32 loads, f64 accumulate",
        "data": "synthetic",
        "config": {"workload": f"configs[1](a) shared() scalar reduction vector_sum, float32 N={n}, uniform[0,1), seed 2",
                   "step": "clear float64 accumulator + one kernel launch, inputs resident in HBM"},
        "roofline": None if head is None else {
            "bound": "hbm", "achieved": head["gbps_kernel"], "peak": HBM_PEAK_BPS / 1e9, "unit": "GB/s",
            "frac": head["frac"], "traffic": head["traffic_bytes_rocprof"],
            # the kernel of configs 1-4 that is furthest from the roofline, and which bars are met
            "min_frac_configs_1_4": measured[worst] if worst else None, "min_frac_kernel": worst,
            "frac_configs_1_4": measured,
            # config 4 once the order of the elements is kept between launches (not the figure of record)
            "frac_reused_config_4": {name: results[name]["frac_reused"] for name in ("spmv_uniform", "spmv_powerlaw")
                                     if name in results and "frac_reused" in results[name]},
            "bars_configs_1_4": {name: {"bar": bar[name], "met": measured[name] >= bar[name]} for name in measured},
        },
        "cpu_baseline": cpu_baseline,
        "cpu_kernels": cpu_kernels,
        "parity_ok": all_ok,
        "parity": parity,
        "kernels": results,
        "device": {"name": props["name"], "arch": props["arch"], "compute_units": props["compute_units"]},
    }
    print(json.dumps(line), flush=True)
    if not all_ok:
        sys.exit(3)


if __name__ == "__main__":
    main()

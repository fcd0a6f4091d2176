#!/usr/bin/env python3
"""Benchmark of the Muon + AdamW optimizer step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (config.workload = "qwen3-0.6b-hybrid-step"): the full Qwen3-0.6B-shaped
parameter set, 596,049,920 parameters -- Muon on the 196 projection matrices
(q 1024x2048, k/v 1024x1024, o 2048x1024, gate/up 1024x3072, down 3072x1024 per layer),
AdamW on the tied embedding 151936x1024 and the RMSNorm / q,k-norm gains; fp32 master
weights, bf16 gradients ~N(0,1e-3) with 1% of rows scaled x100, global grad-norm clip at 1.0,
stochastic-rounded bf16 weight downcast, 5 Polar-Express Newton-Schulz iterations.
A step = grad-norm + clip scale + Muon (momentum, NS chain, update) + AdamW, with every
tensor already resident in HBM when the timed region starts.

Prints ONE JSON line. `value` is milliseconds per step (lower is better). `roofline` is the
dominant kernel, the bf16 matrix-core GEMM of the Newton-Schulz chain: executed FLOPs over
the summed duration of its launches, measured with HIP events on the launch stream, against
the 2.5 PFLOP/s dense bf16 peak. `cpu_baseline` times the numpy restatement of the
reference's host path on a bounded sample and scales it to the full step. `configs` holds the
other BASELINE configurations measured in the same run (the Newton-Schulz chain alone, the MoE
family, the flat AdamW buffer) and config 2 under Keller's coefficients and on gradients that
send every matrix through the chain's wide gate; `--no-configs` skips them.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "Qwen3-0.6B Muon+AdamW step ms; AdamW HBM GB/s; NS-GEMM MFMA util %"
PEAK_BF16_TFLOPS = 2500.0      # MI355X dense bf16 matrix-core peak
PEAK_HBM_GBPS = 8000.0         # MI355X HBM3E peak


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def synth(shapes, seed=0, idle_experts=4):
    """Synthetic weights (fp32) and gradients (bf16 bits) of the workload: weights 0.02 N(0,1), gains
    1 + 0.05 N(0,1), gradients N(0, 1e-3) with 1 % of the rows of every matrix x100. A stacked
    [E, K, N] expert tensor is E matrices; per MoE layer `idle_experts` of its experts (the same ones
    in the layer's three tensors, drawn from the seeded generator) have an all-zero gradient."""
    from ancora_cutile_amd.bf16 import bf16_bits
    rng = np.random.default_rng(seed)
    params, grads, idle = {}, {}, {}
    for name, shape in shapes.items():
        n = int(np.prod(shape))
        if len(shape) == 1:
            p = (1.0 + 0.05 * rng.standard_normal(n, dtype=np.float32)).reshape(shape)
        else:
            p = (0.02 * rng.standard_normal(n, dtype=np.float32)).reshape(shape)
        g = (1e-3 * rng.standard_normal(n, dtype=np.float32)).reshape(shape)
        if len(shape) >= 2:                      # 1% of rows carry a x100 outlier scale
            g2 = g.reshape(-1, shape[-1])
            rows = g2.shape[0]
            k = max(1, rows // 100)
            g2[rng.choice(rows, k, replace=False)] *= 100.0
        if len(shape) == 3 and idle_experts:
            layer = name.split(".")[0]
            if layer not in idle:
                idle[layer] = np.sort(rng.choice(shape[0], min(idle_experts, shape[0]), replace=False))
            g[idle[layer]] = 0.0
        params[name] = p
        grads[name] = bf16_bits(g).reshape(shape)
    return params, grads


def read_sclk_mhz():
    """Current shader clock in MHz from sysfs (read-only, no child process), or None."""
    from ancora_cutile_amd.sysfs import sclk_mhz
    return sclk_mhz()


def sustained_sclk(run_steps, seconds=1.5):
    """(median shader clock in MHz, median package power in W) while `run_steps(n)` keeps the GPU
    busy with optimizer steps: a sampler thread polls the board's sysfs entries, the main thread
    keeps launching (launches are asynchronous and the library calls drop the GIL). Outside the
    timed region. None where sysfs gives nothing."""
    import threading
    from ancora_cutile_amd.sysfs import power_w
    clocks, watts, stop = [], [], threading.Event()

    def poll():
        time.sleep(0.4)                      # let the clock settle under load
        while not stop.is_set():
            v, w = read_sclk_mhz(), power_w()
            if v:
                clocks.append(v)
            if w:
                watts.append(w)
            time.sleep(0.01)

    th = threading.Thread(target=poll, daemon=True)
    th.start()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        run_steps(5)
    stop.set()
    th.join(timeout=15)
    clocks = sorted(v for v in clocks if v > 300)   # drop samples taken while the GPU idled
    watts = sorted(watts)
    return (clocks[len(clocks) // 2] if clocks else None,
            round(watts[len(watts) // 2], 1) if watts else None)


def gemm_bytes_from_counter_db(path, ctr):
    """(bytes per k_ns_gemm_big launch, launches, KiB per count) from a rocprofv3 results database
    that holds counter `ctr` for the GEMM launches and for the 1 GiB copy kernel of the same run
    (which moves 1 GiB each way: its reading fixes the counter's unit)."""
    import sqlite3
    rows = sqlite3.connect(path).execute(
        "select kernel_name, count(*), sum(value) from counters_collection where counter_name = ? "
        "group by kernel_name", (ctr,)).fetchall()
    copy = [r for r in rows if "k_copy16" in r[0]]
    gemm = [r for r in rows if "k_ns_gemm_big" in r[0]]
    if not copy or not gemm:
        raise RuntimeError(f"{ctr}: copy or GEMM kernel missing from the counter table")
    unit_kib = (1 << 20) / (sum(r[2] for r in copy) / sum(r[1] for r in copy))
    n = sum(r[1] for r in gemm)
    return sum(r[2] for r in gemm) * unit_kib * 1024.0 / n, n, unit_kib


def measure_gemm_traffic(workload):
    """HBM bytes per k_ns_gemm_big launch, measured now: two child runs of this script under
    `rocprofv3 --pmc` (FETCH_SIZE, then WRITE_SIZE: the profiler does not split counters over
    passes), each scaled by what the same counter reads for the 1 GiB copy kernel the run contains.
    Called before this process touches the GPU. Returns (bytes_per_launch, detail dict)."""
    import shutil
    import signal
    import subprocess
    import tempfile
    if shutil.which("rocprofv3") is None:
        raise RuntimeError("rocprofv3 not found")
    top = tempfile.mkdtemp(prefix="anc_traffic_", dir="/tmp")
    res = {}
    for ctr in ("FETCH_SIZE", "WRITE_SIZE"):
        cmd = ["rocprofv3", "--pmc", ctr, "-d", os.path.join(top, ctr), "-o", ctr, "--",
               "python3", os.path.abspath(__file__), "--workload", workload, "--serial", "--steps", "3",
               "--warmup", "1", "--no-cpu", "--no-clock", "--no-configs"]
        log(" ".join(cmd))
        pr = subprocess.Popen(cmd, cwd="/tmp", env={**os.environ, "TMPDIR": "/tmp"}, start_new_session=True,
                              stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
        try:
            rc = pr.wait(timeout=280)
        except subprocess.TimeoutExpired:
            os.killpg(pr.pid, signal.SIGKILL)
            raise RuntimeError(f"rocprofv3 --pmc {ctr} did not finish")
        if rc != 0:
            raise RuntimeError(f"rocprofv3 --pmc {ctr} exited with {rc}")
        dbs = [os.path.join(d, f) for d, _, fs in os.walk(os.path.join(top, ctr)) for f in fs if f.endswith("_results.db")]
        if not dbs:
            raise RuntimeError(f"no results database under {top}/{ctr}")
        res[ctr] = gemm_bytes_from_counter_db(dbs[0], ctr)
    shutil.rmtree(top, ignore_errors=True)
    total = int(res["FETCH_SIZE"][0] + res["WRITE_SIZE"][0])
    return total, {"read_bytes_per_launch": int(res["FETCH_SIZE"][0]), "write_bytes_per_launch": int(res["WRITE_SIZE"][0]),
                   "launches_counted": res["FETCH_SIZE"][1], "fetch_unit_kib": round(res["FETCH_SIZE"][2], 4),
                   "write_unit_kib": round(res["WRITE_SIZE"][2], 4)}


def kernel_source_sha16():
    """Hash of the Newton-Schulz kernel sources: ties a recorded counter figure to the code it was
    measured on."""
    import hashlib
    h = hashlib.sha256()
    for f in ("ns_common.h", "ns.hip", "ns_gemm_big.hip"):
        with open(os.path.join(ROOT, "ancora-cutile_amd", "csrc", f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


def cpu_baseline(shapes, lr_adam=3e-4):
    """Numpy restatement of the reference host path (Muon.step + host_ns, AdamW test-oracle
    formula) timed on a bounded sample: one matrix of each Newton-Schulz shape and a 16M-element
    AdamW slice, scaled by the counts of the full parameter set."""
    from oracle.adamw_ref import adamw_step_div
    from oracle.muon_ref import muon_momentum, ns_any_shape, muon_update, PE_SCHEDULE
    try:
        from threadpoolctl import threadpool_info
        blas = [i for i in threadpool_info() if i.get("user_api") == "blas"]
        threads = max([i["num_threads"] for i in blas], default=1)
    except Exception:
        threads = 1
    rng = np.random.default_rng(0)
    groups = {}
    adam_elems = 0
    from ancora_cutile_amd.hybrid import resident_is_muon

    class _Shape:                     # what the routing predicate looks at
        def __init__(self, shape):
            self.shape, self.ndim = shape, len(shape)

    for name, shape in shapes.items():
        if len(shape) == 2 and resident_is_muon(name, _Shape(shape)):
            groups[shape] = groups.get(shape, 0) + 1
        else:
            adam_elems += int(np.prod(shape))
    total_ms = 0.0
    for shape, count in groups.items():
        W = (0.02 * rng.standard_normal(shape)).astype(np.float32)
        g = (1e-3 * rng.standard_normal(shape)).astype(np.float32)
        buf = np.zeros(shape, np.float32)
        t0 = time.perf_counter()
        buf, u = muon_momentum(buf, g)
        o = ns_any_shape(u, PE_SCHEDULE, 5)
        W = muon_update(W, o, 0.02)
        total_ms += (time.perf_counter() - t0) * 1e3 * count
    n = 1 << 24
    p = rng.standard_normal(n).astype(np.float32)
    m = np.zeros(n, np.float32)
    v = np.zeros(n, np.float32)
    g = (1e-3 * rng.standard_normal(n)).astype(np.float32)
    t0 = time.perf_counter()
    adamw_step_div(p, m, v, g, lr_adam, 0.9, 0.95, 1e-8, 0.1, 1)
    total_ms += (time.perf_counter() - t0) * 1e3 * adam_elems / n
    return {"value": round(total_ms, 1), "unit": "ms/step", "cores": int(threads), "kind": "port",
            "sample": "numpy oracle: one momentum+NS+update per Muon shape x its count "
                      f"({', '.join(f'{c}x{s}' for s, c in groups.items())}) + AdamW on a 16.8M-element "
                      f"slice scaled to {adam_elems} elements; host has {os.cpu_count()} cpus, "
                      f"{len(os.sched_getaffinity(0))} usable, BLAS threads {threads}"}


def ns_config(steps):
    """BASELINE config 3: the 196 Newton-Schulz matrices of the Qwen3-0.6B set through the fp32-input
    chain entry, group by group, in the bf16 matrix-core mode and in the fp32 validation mode."""
    from ancora_cutile_amd import DevBuf, PE_SCHEDULE, _lib
    from ancora_cutile_amd.muon_ns import ns_batched, ns_flops
    e0, e1 = _lib.Event(), _lib.Event()
    groups = ((1024, 1024, 56), (1024, 2048, 56), (1024, 3072, 84))
    res = {}
    for mode in ("bf16", "fp32"):
        k = steps if mode == "bf16" else 1
        total_ms, ex_t, de_t = 0.0, 0.0, 0.0
        for (M, N, E) in groups:
            one = np.random.default_rng(M + N).standard_normal((M, N)).astype(np.float32)
            X = DevBuf.empty((E * M, N), np.float32)
            for e in range(E):
                X.at_pos(e * M).upload(one)
            ns_batched(X, E, M, N, 0, schedule=PE_SCHEDULE, mode=mode)
            e0.record(0)
            for _ in range(k):
                ns_batched(X, E, M, N, 0, schedule=PE_SCHEDULE, mode=mode)
            e1.record(0)
            e1.sync()
            total_ms += e0.elapsed_ms(e1) / k
            ex, de = ns_flops(E, M, N, 5, mode)
            ex_t += ex
            de_t += de
            X.free()
        res[mode] = {"ms": round(total_ms, 3), "executed_tflop": round(ex_t / 1e12, 3),
                     "dense_tflop": round(de_t / 1e12, 3),
                     "executed_tflops_per_s": round(ex_t / total_ms / 1e9, 1)}
    return res, groups


def adamw_flat_config(steps, warmup):
    """BASELINE config 5, clean-gradient variant: grad-norm + clip + AdamW + stochastic bf16 downcast
    over one flat 1.2e9-element buffer, step counter at 1000."""
    import ctypes
    from ancora_cutile_amd import DevBuf, StepGuard, _lib
    from ancora_cutile_amd.adamw import hyper_div
    from ancora_cutile_amd.bf16 import bf16_bits
    e0, e1 = _lib.Event(), _lib.Event()
    n = 1_200_000_000
    rng = np.random.default_rng(0)
    chunk = bf16_bits(1e-3 * rng.standard_normal(1 << 24, dtype=np.float32))
    g = DevBuf.empty((n,), np.uint16)
    for off in range(0, n, 1 << 24):
        k = min(1 << 24, n - off)
        DevBuf(shape=(k,), dtype=np.uint16, ptr=g.ptr + 2 * off).upload(chunk[:k])
    m, v, p = (DevBuf.zeros((n,), np.float32) for _ in range(3))
    p16 = DevBuf.zeros((n,), np.uint16)
    guard = StepGuard(1.0)

    def step(t):
        guard.compute([g], 0)
        h = hyper_div(3e-4, 0.9, 0.95, 1e-8, 1000 + t, sr=True, seed_base=t)
        _lib.api.anc_adamw(g.ptr, m.ptr, v.ptr, p.ptr, p16.ptr, n, _lib.BF16, ctypes.byref(h), 0.1, 0,
                           guard.ptr, 0)
    for t in range(warmup):
        step(t)
    e0.record(0)
    for t in range(steps):
        step(t)
    e1.record(0)
    e1.sync()
    ms = e0.elapsed_ms(e1) / steps
    _lib.profile_enable(True)
    step(0)
    pr = _lib.profile_read()
    _lib.profile_enable(False)
    a_ms, g_ms = pr["adamw"][0], pr["gradnorm_partials"][0]
    out = {"elements": n, "ms": ms, "gbps": round(30.0 * n / (ms * 1e-3) / 1e9, 1),
           "frac": round(30.0 * n / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4),
           "adamw_kernel": {"ms": round(a_ms, 3), "gbps": round(28.0 * n / (a_ms * 1e-3) / 1e9, 1)},
           "gradnorm_kernel": {"ms": round(g_ms, 3), "gbps": round(2.0 * n / (g_ms * 1e-3) / 1e9, 1)},
           "clip_scale": guard.read(0)["clip_scale"]}
    for b in (g, m, v, p, p16):
        b.free()
    guard.free()
    return out


GEMM_KINDS = ("ns_gemm_gram", "ns_gemm_bmat", "ns_gemm_bx", "ns_gemm_bx_update")


def chain_work(opt, schedule):
    """(executed FLOPs, dense FLOPs, matrices that took a conditioning gate) of the optimizer's last
    step, from the plan of the mode it ran in and the gate decisions left in the workspaces."""
    from ancora_cutile_amd.muon_ns import ns_flops, ns_hard_info
    executed = dense = 0.0
    hard = 0
    for b in opt.muon.engine.batches:
        ex, de = ns_flops(b.E, b.M, b.Nn, 5, "bf16", schedule=schedule)
        nh, extra = ns_hard_info(b.ws.buf.ptr, b.E, b.M, b.Nn, 5, "bf16", schedule=schedule)
        executed += ex + extra
        dense += de
        hard += nh
    return executed, dense, hard


def hybrid_config(opt, gdev, schedule, steps=5, warmup=2):
    """A compact measurement of the hybrid step as `opt` stands: ms per step over `steps` steps
    (HIP events, steps queued without host synchronisation), and the matrix-core GEMM launches'
    summed duration and executed work from one step under the per-launch event timer."""
    from ancora_cutile_amd import _lib
    for _ in range(warmup):
        opt.step(gdev, 0)
    _lib.api.anc_device_sync()
    t_before = opt.step_count()
    e0, e1 = _lib.Event(), _lib.Event()
    e0.record(0)
    for _ in range(steps):
        opt.step(gdev, 0, sync=False)
    e1.record(0)
    e1.sync()
    ms = e0.elapsed_ms(e1) / steps
    if opt.step_count() != t_before + steps:
        raise RuntimeError("the guard skipped a timed step (non-finite gradient norm)")
    opt.muon.engine.serial = True
    opt.step(gdev, 0)
    _lib.profile_enable(True)
    opt.step(gdev, 0)
    prof = _lib.profile_read()
    _lib.profile_enable(False)
    opt.muon.engine.serial = False
    gemm_ms = sum(prof[k][0] for k in GEMM_KINDS)
    executed, dense, hard = chain_work(opt, schedule)
    tf = executed / (gemm_ms * 1e-3) / 1e12
    return {"ms": round(ms, 3), "ns_gemm_ms": round(gemm_ms, 3), "executed_tflop": round(executed / 1e12, 3),
            "dense_tflop": round(dense / 1e12, 3), "ns_gemm_tflops_per_s": round(tf, 1),
            "ns_gemm_frac": round(tf / PEAK_BF16_TFLOPS, 4),
            "muon_matrices": sum(b.E for b in opt.muon.engine.batches), "gated_hard_matrices": hard}


def wide_spectrum_grad(K, N, rng, decades=3.0):
    """(K, N) bf16 gradient whose singular values are log-uniform over `decades` decades: the kind of
    input the chain's wide gate exists for (every residual term from iteration 1 on)."""
    from ancora_cutile_amd.bf16 import bf16_bits
    M, L = min(K, N), max(K, N)
    U, _ = np.linalg.qr(rng.standard_normal((M, M)).astype(np.float32))
    V, _ = np.linalg.qr(rng.standard_normal((L, M)).astype(np.float32))
    sv = np.logspace(0.0, -decades, M).astype(np.float32)
    G = (U * sv) @ V.T                                    # (M, L)
    G = (1e-3 * np.sqrt(M * L) / np.linalg.norm(G)) * G    # entries of the size of the other gradients
    return bf16_bits(np.ascontiguousarray(G.T if K > N else G).astype(np.float32)).reshape(K, N)


def other_configs(opt, gdev, args):
    """The non-headline numbers, measured in the same run: config 2 under the reference's default
    schedule (Keller) and on gradients that send every matrix through the wide gate, then configs
    4, 3 and 5. `opt` (the headline optimizer) is freed on the way."""
    from ancora_cutile_amd import HybridOptimizer, PE_SCHEDULE, _lib
    from ancora_cutile_amd.hybrid import resident_is_muon
    from ancora_cutile_amd.shapes import moe_shapes
    cfg = {}
    # config 2 under Keller's coefficients: the host layer runs the chain in its late-3 plan
    opt.muon.schedule = None
    r = hybrid_config(opt, gdev, None)
    r["note"] = ("config 2, the reference's default schedule (Keller, ancora/kernels/muon_ns.py:21,51-65): "
                 "the chain runs its bf16_late3 plan")
    cfg["c2_keller"] = r
    opt.muon.schedule = PE_SCHEDULE
    log(f"configs: c2_keller {r['ms']} ms")
    # config 2 with a three-decade spectrum in every Muon gradient: every matrix takes the wide gate
    rng = np.random.default_rng(5)
    by_shape = {}
    for n in opt.muon_names:
        s = opt.muon.st[n]
        K, N = s["K"], s["N"]
        if (K, N) not in by_shape:
            by_shape[(K, N)] = wide_spectrum_grad(K, N, rng)
        s["g"].upload(by_shape[(K, N)])
        s["buf"].fill_zero(0)
    r = hybrid_config(opt, gdev, PE_SCHEDULE)
    r["note"] = ("config 2 with singular values log-uniform over three decades in every Muon gradient "
                 "(momentum buffers zeroed first): the worst-case Polar-Express step")
    cfg["c2_all_wide_gate"] = r
    log(f"configs: c2_all_wide_gate {r['ms']} ms, {r['gated_hard_matrices']} of {r['muon_matrices']} gated")
    opt.free()
    # config 4: the 16-layer MoE family
    shapes = moe_shapes(layers=16)
    params, grads = synth(shapes)
    n_params = sum(p.size for p in params.values())
    mo = HybridOptimizer(params, is_muon=resident_is_muon,
                         muon_kw=dict(lr=0.02, momentum=0.95, ns_steps=5, schedule=PE_SCHEDULE, sr=True, seed=1),
                         adamw_kw=dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, wd=0.1, sr=True, seed=2),
                         max_grad_norm=1.0, grad_dtype=np.uint16)
    del params
    gd = {}
    for part, names in ((mo.muon, mo.muon_names), (mo.adamw, mo.adamw_names)):
        for n in names:
            st = part.st[n]
            st["g"].upload(grads[n].reshape(st["g"].shape))
            gd[n] = st["g"]
    del grads
    r = hybrid_config(mo, gd, PE_SCHEDULE)
    r["params"] = n_params
    r["note"] = "config 4: 16 layers alternating dense / MoE (E = 16), grad-norm + clip + Muon + AdamW"
    cfg["c4_moe_16l"] = r
    log(f"configs: c4_moe_16l {r['ms']} ms")
    mo.free()
    # config 3: the Newton-Schulz chain alone, both modes
    res, _ = ns_config(3)
    cfg["c3_ns_196"] = {"bf16_ms": res["bf16"]["ms"], "fp32_ms": res["fp32"]["ms"],
                        "bf16_executed_tflops_per_s": res["bf16"]["executed_tflops_per_s"],
                        "fp32_tflops_per_s": res["fp32"]["executed_tflops_per_s"],
                        "note": "config 3: 196 matrices through the fp32-input chain entry, 5 Polar-Express steps"}
    log(f"configs: c3_ns_196 {res['bf16']['ms']} / {res['fp32']['ms']} ms")
    # config 5: the flat AdamW buffer
    r = adamw_flat_config(5, 2)
    cfg["c5_adamw_flat"] = {"ms": round(r["ms"], 3), "gbps": r["gbps"], "frac_of_8tbps": r["frac"],
                            "adamw_kernel": r["adamw_kernel"], "gradnorm_kernel": r["gradnorm_kernel"],
                            "note": "config 5, clean gradients: 1.2e9 elements, 30 B per element"}
    log(f"configs: c5_adamw_flat {r['ms']:.3f} ms")
    return cfg


def side_workload(args):
    """Configs 3 and 5 as stand-alone timings (same JSON shape, their own metric names)."""
    from ancora_cutile_amd import DevBuf, StepGuard, PE_SCHEDULE, _lib
    from ancora_cutile_amd.muon_ns import ns_batched, ns_flops
    _lib.init(0)
    info = _lib.device_info()
    e0, e1 = _lib.Event(), _lib.Event()
    if args.workload == "ns":
        res, groups = ns_config(args.steps)
        out = {"metric": "196-matrix Newton-Schulz chain ms (5 x Polar-Express)", "value": res["bf16"]["ms"],
               "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": 1, "ms_per_step": res["bf16"]["ms"],
               "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
               "data": "synthetic", "config": {"workload": "ns-196-matrices", "groups": [list(g) for g in groups]},
               "modes": res}
    elif args.workload == "dw":
        # the weight-gradient GEMMs of the 28 Qwen3-0.6B layers at `--tokens` tokens per micro-batch;
        # buffers of one layer reused for all layers. --dw-launch layer: one call per layer with
        # its 7 weights, one token segment each (480 workgroups); group: as the backward pass
        # reaches them, per layer [q,k,v] (shared activations), [o], [gate,up] (shared), [down],
        # every weight cut into the token segments that let it fill the GPU alone
        from ancora_cutile_amd.grads import gemm_dW, DwWorkspace, dw_info
        from ancora_cutile_amd.bf16 import bf16_bits
        T = args.tokens
        rng = np.random.default_rng(0)
        groups = ((1024, (2048, 1024, 1024)), (2048, (1024,)), (1024, (3072, 3072)), (3072, (1024,)))
        calls, flops = [], 0.0
        for K, Ns in groups:
            xT = DevBuf(bf16_bits((0.1 * rng.standard_normal((K, T))).astype(np.float32)))
            xkey = "xT"
            if args.dw_acts == "x":                # the activations as they lie, (T, K)
                xkey, old = "x", xT
                xT = DevBuf(np.ascontiguousarray(old.to_numpy().T))
                old.free()
            probs = []
            for N in Ns:
                probs.append(dict(**{xkey: xT}, dy=DevBuf(bf16_bits((0.1 * rng.standard_normal((T, N))).astype(np.float32))),
                                  dW=DevBuf.zeros((K, N), np.float32), g16=DevBuf.zeros((K, N), np.uint16),
                                  T=T, K=K, N=N, workspace=DwWorkspace(), accumulate=True))
                flops += dw_info(T, K, N)[0]
            calls.append(probs)
        layers = 28
        per_layer = [p for probs in calls for p in probs]

        side = [_lib.stream_create() for _ in calls] if args.dw_launch == "group" else []
        main_st = _lib.stream_create() if args.dw_launch == "group" else 0
        fork, joins = _lib.Event(), [_lib.Event() for _ in calls]

        def step():
            for _ in range(layers):
                if args.dw_launch == "layer":
                    gemm_dW(per_layer, 0, segments=1)
                elif args.dw_launch == "group":
                    # one call per group of weights, no token segments (the bits of `layer`); the four
                    # calls of a layer go to four streams, as a backward pass that keeps its
                    # weight-gradient GEMMs off the critical path would issue them
                    fork.record(main_st)
                    for st, ev, probs in zip(side, joins, calls):
                        fork.wait_on(st)
                        gemm_dW(probs, st, segments=1)
                        ev.record(st)
                    for ev in joins:
                        ev.wait_on(main_st)
                elif args.dw_launch == "group-serial":
                    for probs in calls:
                        gemm_dW(probs, 0, segments=1)
                else:
                    for probs in calls:
                        gemm_dW(probs, 0, segments="fill" if args.dw_launch == "group-fill" else "shape")
        for _ in range(max(1, args.warmup // 2)):
            step()
        _lib.api.anc_device_sync()
        e0.record(main_st)
        for _ in range(args.steps):
            step()
        e1.record(main_st)
        e1.sync()
        ms = e0.elapsed_ms(e1) / args.steps
        _lib.profile_enable(True)
        step()
        pr = _lib.profile_read()
        _lib.profile_enable(False)
        g_ms, r_ms = pr["dw_gemm"][0], pr["dw_reduce"][0]
        # the (T, K) -> (K, T) transposes of the activations that the GEMM's A operand layout asks
        # for (once per group of weights that share them), timed apart: not in `value`
        from ancora_cutile_amd.grads import transpose_acts
        xs = [(DevBuf.zeros((T, K), np.uint16), DevBuf.zeros((K, T), np.uint16), K) for (K, _), probs in zip(groups, calls)]
        for x, xT, K in xs:
            transpose_acts(x, xT, T, K, 0)
        e0.record(0)
        for _ in range(layers):
            for x, xT, K in xs:
                transpose_acts(x, xT, T, K, 0)
        e1.record(0)
        e1.sync()
        tr_ms = e0.elapsed_ms(e1)
        tr_bytes = layers * sum(4 * T * K for _, _, K in xs)
        tf = layers * flops / (ms * 1e-3) / 1e12
        gtf = layers * flops / (g_ms * 1e-3) / 1e12
        nparams = sum(K * N for K, Ns in groups for N in Ns) * layers
        out = {"metric": "Qwen3-0.6B weight-gradient GEMMs (dW += x^T dy, 196 weights) ms per micro-batch",
               "value": round(ms, 3), "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
               "ms_per_step": round(ms, 3), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
               "dtype": "bf16", "data": "synthetic",
               "config": {"workload": "qwen3-0.6b-weight-gradients", "tokens": T, "weights": 7 * layers,
                          "params": nparams, "launch": args.dw_launch,
                          "launches_per_layer": 1 if args.dw_launch == "layer" else 4,
                          "token_segments": {"layer": 1, "group": 1, "group-serial": 1, "group-split": "shape rule",
                                             "group-fill": "per launch, <= 512 workgroups"}[args.dw_launch],
                          "streams": 4 if args.dw_launch == "group" else 1,
                          "accumulate": True, "bf16_copy": True,
                          "activations": "x (T,K) as they lie" if args.dw_acts == "x" else "x^T (K,T), transposed by the caller"},
               "roofline": {"bound": "mfma", "achieved": round(gtf, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                            "frac": round(gtf / PEAK_BF16_TFLOPS, 4), "traffic": None,
                            "kernel": "k_ns_gemm_big<EPI_BX, ..., VAR_PLAIN> (partial tiles of x^T dy)",
                            "launches_per_step": pr["dw_gemm"][1], "avg_launch_ms": round(g_ms / pr["dw_gemm"][1], 4),
                            "tflop_per_step": round(layers * flops / 1e12, 3)},
               "whole_tflops_per_s": round(tf, 1),
               "reduce_kernel": {"ms": round(r_ms, 3), "launches": pr["dw_reduce"][1]},
               "activation_transposes": {"ms": round(tr_ms, 3), "launches": layers * len(xs),
                                         "gbps": round(tr_bytes / (tr_ms * 1e-3) / 1e9, 1),
                                         "note": "what a caller of the x^T form pays on top: x (T,K) -> x^T (K,T) once per group of weights sharing x; never in value"}}
    else:
        r = adamw_flat_config(args.steps, args.warmup)
        n, ms = r["elements"], r["ms"]
        out = {"metric": "flat 1.2e9-element grad-norm + clip + AdamW + SR downcast ms", "value": round(ms, 3),
               "unit": "ms", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 3),
               "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
               "data": "synthetic", "config": {"workload": "adamw-flat-1.2e9", "step": 1000},
               "roofline": {"bound": "hbm", "achieved": r["gbps"], "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                            "frac": r["frac"], "traffic": None, "bytes_per_elem": 30},
               "adamw_kernel": r["adamw_kernel"], "gradnorm_kernel": r["gradnorm_kernel"],
               "clip_scale": r["clip_scale"]}
    out["device"] = {"name": info["name"] or info["arch"].split(":")[0], "arch": info["arch"], "cus": info["cu_count"]}
    print(json.dumps(out), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--layers", type=int, default=28, help=argparse.SUPPRESS)   # smaller sets for debugging
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the `configs` block (configs 3, 4, 5 and the two other config-2 steps)")
    ap.add_argument("--no-clock", action="store_true",
                    help="skip the sustained-clock sampling")
    ap.add_argument("--traffic", action="store_true",
                    help="measure roofline.traffic now: two extra runs of this script under rocprofv3 --pmc "
                         "(about a minute); without it the figure recorded under profiles/ is reported while "
                         "the kernel sources are the ones it was taken with")
    ap.add_argument("--write-traffic", action="store_true",
                    help="with --traffic: also rewrite profiles/ns_gemm_traffic.json from the measurement")
    ap.add_argument("--tokens", type=int, default=8192, help="tokens per micro-batch of --workload dw")
    ap.add_argument("--dw-acts", default="x", choices=("x", "xT"),
                    help="--workload dw: activations as they lie (T,K), or transposed by the caller")
    ap.add_argument("--dw-launch", default="layer", choices=("layer", "group", "group-serial", "group-split", "group-fill"),
                    help="--workload dw: one call per layer (7 weights); or 4 calls per layer: `group` on four "
                         "streams, `group-serial` on one, both without token segments (same bits as `layer`); "
                         "`group-split` / `group-fill` cut the token axis (shape rule / per launch): other bits")
    ap.add_argument("--workload", default="qwen3", choices=("qwen3", "moe", "ns", "adamw", "dw"),
                    help="qwen3: the headline hybrid step (default). moe: the 16-layer MoE family "
                         "(config 4). ns: the 196-matrix Newton-Schulz stress, bf16 and fp32 modes "
                         "(config 3). adamw: one flat 1.2e9-element buffer (config 5)")
    ap.add_argument("--serial", action="store_true",
                    help="run the per-shape Newton-Schulz chains on one stream also in the timed steps "
                         "(what the rocprofv3 kernel summaries under profiles/ were taken with)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this optimizer step runs on one GPU; --gpus must be 1 "
                 "(no multi-GPU path is built: every box has one GPU and the step needs no collective)")

    if args.workload in ("ns", "adamw", "dw"):
        return side_workload(args)
    live_traffic = None
    if args.traffic:          # child processes first: this one has not touched the GPU yet
        live_traffic = measure_gemm_traffic(args.workload)
        log(f"HBM bytes per k_ns_gemm_big launch, measured: {live_traffic[0]} {live_traffic[1]}")
    from ancora_cutile_amd import HybridOptimizer, DevBuf, PE_SCHEDULE, _lib
    from ancora_cutile_amd.hybrid import resident_is_muon
    from ancora_cutile_amd.muon_ns import ns_flops, ns_product_flops, ns_hard_info
    from ancora_cutile_amd.shapes import qwen3_shapes, moe_shapes

    _lib.init(0)
    info = _lib.device_info()
    log(f"device: {info['name']} {info['arch']} cus={info['cu_count']} clock={info['clock_khz']} kHz")
    if args.workload == "moe":
        shapes = moe_shapes(layers=16)
    else:
        shapes = qwen3_shapes(layers=args.layers)
    t0 = time.perf_counter()
    params, grads = synth(shapes)
    n_params = sum(p.size for p in params.values())
    log(f"synthetic set: {n_params} params in {len(params)} tensors ({time.perf_counter() - t0:.1f} s)")

    opt = HybridOptimizer(params, is_muon=resident_is_muon,
                          muon_kw=dict(lr=0.02, momentum=0.95, ns_steps=5, schedule=PE_SCHEDULE,
                                       sr=True, seed=1),
                          adamw_kw=dict(lr=3e-4, betas=(0.9, 0.95), eps=1e-8, wd=0.1, sr=True, seed=2),
                          max_grad_norm=1.0, grad_dtype=np.uint16)
    n_muon = sum(params[n].size for n in opt.muon_names)
    n_adam = sum(params[n].size for n in opt.adamw_names)
    del params
    # gradients resident in HBM before anything is timed
    gdev = {}
    for opt_part, names in ((opt.muon, opt.muon_names), (opt.adamw, opt.adamw_names)):
        for n in names:
            s = opt_part.st[n]
            s["g"].upload(grads[n].reshape(s["g"].shape))
            gdev[n] = s["g"]
    del grads
    _lib.stream_sync(0)
    log(f"muon params {n_muon}, adamw params {n_adam}; state resident")

    # one plain 1 GiB copy kernel: the known-size reference that HBM traffic counters
    # (FETCH_SIZE / WRITE_SIZE) of a profiled run are scaled by
    cal_a, cal_b = DevBuf.empty((1 << 28,), np.float32), DevBuf.empty((1 << 28,), np.float32)
    cal_a.fill_zero(0)
    e0, e1 = _lib.Event(), _lib.Event()
    _lib.api.anc_copy_kernel(cal_b.ptr, cal_a.ptr, 1 << 30, 0)
    e0.record(0)
    _lib.api.anc_copy_kernel(cal_b.ptr, cal_a.ptr, 1 << 30, 0)
    e1.record(0)
    e1.sync()
    copy_gbps = 2 * (1 << 30) / (e0.elapsed_ms(e1) * 1e-3) / 1e9
    cal_a.free()
    cal_b.free()

    opt.muon.engine.serial = bool(args.serial)
    for _ in range(args.warmup):
        opt.step(gdev, 0)
    _lib.api.anc_device_sync()
    e0, e1 = _lib.Event(), _lib.Event()
    t_before = opt.step_count()
    t0 = time.perf_counter()
    e0.record(0)
    for _ in range(args.steps):
        # queued without a host synchronisation: the steps are counted on the device, the guard's
        # block is read once, after the timed region
        opt.step(gdev, 0, sync=False)
    e1.record(0)
    e1.sync()
    _lib.api.anc_device_sync()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    skipped = t_before + args.steps - opt.step_count()
    if skipped:       # a skipped step returns early from every kernel and would time as falsely fast
        sys.exit(f"bench.py: the guard skipped {skipped} of {args.steps} timed steps (non-finite gradient norm)")
    ev_ms = e0.elapsed_ms(e1) / args.steps
    ms_per_step = max(wall_ms, ev_ms)
    ctl = opt.last_ctl

    # per-kernel durations: HIP events around every launch, on the launch stream, with the
    # per-shape chains serialised onto one stream so that a launch is timed running alone
    opt.muon.engine.serial = True
    opt.step(gdev, 0)
    _lib.profile_enable(True)
    prof_steps = 2
    for _ in range(prof_steps):
        opt.step(gdev, 0)
    prof = _lib.profile_read()
    _lib.profile_enable(False)
    kind_ms = {k: v[0] / prof_steps for k, v in prof.items() if v[1]}
    launches = {k: v[1] // prof_steps for k, v in prof.items() if v[1]}

    executed = dense = last_bx = lower128 = 0.0
    hard = 0           # matrices that took the extra terms of the conditioning gate in the last step
    for b in opt.muon.engine.batches:
        ex, de = ns_flops(b.E, b.M, b.Nn, 5, "bf16")
        nh, extra = ns_hard_info(b.ws.buf.ptr, b.E, b.M, b.Nn, 5, "bf16")
        executed += ex + extra
        dense += de
        hard += nh
        ex128, _ = ns_flops(b.E, b.M, b.Nn, 5, "bf16_tile128")    # the same chain counted in 128x128 tiles
        nh128, extra128 = ns_hard_info(b.ws.buf.ptr, b.E, b.M, b.Nn, 5, "bf16_tile128")
        lower128 += ex128 + extra128
        last_bx += ns_product_flops(b.E, b.M, b.Nn, 4, 2, 5, "bf16")
    # What the board sustains: the shader clock while the step runs (the nominal 2.4 GHz is not
    # held under the power limit) and the matrix pipe's register-only rate on zero / random operands
    opt.muon.engine.serial = bool(args.serial)

    def run_steps(n):
        for _ in range(n):
            opt.step(gdev, 0)
        _lib.stream_sync(0)

    sclk, watts = (None, None) if args.no_clock else sustained_sclk(run_steps)

    # every launch of k_ns_gemm_big; with the fused update one of them (kind ns_gemm_bx_update, the
    # last X = a X + B X) also reads and writes the weights
    gemm_kinds = ("ns_gemm_gram", "ns_gemm_bmat", "ns_gemm_bx", "ns_gemm_bx_update")
    gemm_ms = sum(kind_ms.get(k, 0.0) for k in gemm_kinds)
    gemm_launches = sum(launches.get(k, 0) for k in gemm_kinds)
    achieved = executed / (gemm_ms * 1e-3) / 1e12 if gemm_ms else 0.0
    pure_ms = gemm_ms - kind_ms.get("ns_gemm_bx_update", 0.0)
    pure_launches = gemm_launches - launches.get("ns_gemm_bx_update", 0)
    pure_flops = executed - (last_bx if "ns_gemm_bx_update" in kind_ms else 0.0)
    pure_achieved = pure_flops / (pure_ms * 1e-3) / 1e12 if pure_ms else 0.0
    adamw_gbps = 28.0 * n_adam / (kind_ms["adamw"] * 1e-3) / 1e9
    gn_gbps = 2.0 * n_params / (kind_ms["gradnorm_partials"] * 1e-3) / 1e9
    # With the fused update the last X = a X + B X launch of the chain applies W -= lr*O itself:
    # no update kernel exists and its traffic (10 B per parameter) is inside that GEMM launch.
    upd_fused = "muon_update" not in kind_ms
    elem_ms = kind_ms["muon_momentum"] + kind_ms.get("muon_update", 0.0)
    # algorithmic bytes of the momentum stage: bf16 g + fp32 momentum read, fp32 momentum + bf16 u
    # written = 12 B; this kernel writes u as a bf16 pair, so it moves 14 B
    elem_bytes = 12.0 if upd_fused else 24.0
    elem_moved = 14.0 if upd_fused else 26.0
    elem_gbps = elem_bytes * n_muon / (elem_ms * 1e-3) / 1e9

    # HBM bytes per k_ns_gemm_big launch: NOT measured by this run (hardware counters need the
    # profiler). The figure comes from two rocprofv3 --pmc runs of this same command (FETCH_SIZE,
    # WRITE_SIZE, scaled by the copy kernel; summary under profiles/) and is reported only while
    # the kernel sources still have the hash those runs were taken with; otherwise null.
    traffic, traffic_note = None, "not measured in this run"
    tpath = os.path.join(ROOT, "profiles", "ns_gemm_traffic.json")
    if live_traffic is not None:
        traffic = live_traffic[0]
        traffic_note = ("measured in this run: rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE child runs of this command, "
                        f"scaled by the 1 GiB copy kernel {live_traffic[1]}")
        if args.write_traffic and args.workload == "qwen3" and args.layers == 28:
            with open(tpath, "w") as f:
                json.dump({"kernel": "k_ns_gemm_big", "hbm_bytes_per_launch": traffic, **live_traffic[1],
                           "source": "profiles/hybrid_step_qwen3_0p6b_hbm_traffic.md",
                           "source_sha16": kernel_source_sha16(),
                           "command": "python3 bench.py --traffic --write-traffic --no-cpu"}, f, indent=1)
                f.write("\n")
    elif args.workload == "qwen3" and args.layers == 28 and os.path.exists(tpath):
        with open(tpath) as f:
            tj = json.load(f)
        if tj.get("source_sha16") == kernel_source_sha16():
            traffic = tj.get("hbm_bytes_per_launch")
            traffic_note = "static: rocprofv3 FETCH_SIZE + WRITE_SIZE runs recorded in " + tj.get("source", "profiles/")
        else:
            traffic_note = "profiles/ns_gemm_traffic.json was taken with other kernel sources: dropped"

    out = {
        "metric": METRIC if args.workload == "qwen3" else "MoE-16L Muon+AdamW step ms",
        "value": round(ms_per_step, 3), "unit": "ms", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "qwen3-0.6b-hybrid-step" if args.workload == "qwen3" else "moe-16l-hybrid-step",
                   "params": n_params, "muon_params": n_muon,
                   "adamw_params": n_adam, "muon_matrices": sum(b.E for b in opt.muon.engine.batches),
                   "grads": "bf16 resident in HBM, 1% rows x100", "clip": 1.0,
                   "weight_downcast": "stochastic bf16", "ns": "5 x polar-express",
                   "layers": 16 if args.workload == "moe" else args.layers},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(achieved / PEAK_BF16_TFLOPS, 4), "traffic": traffic,
                     "traffic_source": traffic_note, "gated_hard_matrices": hard,
                     "kernel": "k_ns_gemm_big (gram, bmat, bx launches of the Newton-Schulz chain)",
                     "timed": "HIP events around each launch, chains serialised on one stream"
                              + ("; the last of the 15 launches also carries the fused weight update" if upd_fused else ""),
                     "launches_per_step": gemm_launches,
                     "without_fused_update_launch": {"launches": pure_launches, "achieved": round(pure_achieved, 1),
                                                     "frac": round(pure_achieved / PEAK_BF16_TFLOPS, 4),
                                                     "avg_launch_ms": round(pure_ms / max(1, pure_launches), 4)},
                     "avg_launch_ms": round(gemm_ms / max(1, gemm_launches), 4),
                     # context, not the fraction asked for: the board holds `sustained_sclk_mhz`, not
                     # its nominal clock, under the step's load
                     "frac_of_peak_at_sustained_clock": (round(achieved / (PEAK_BF16_TFLOPS * sclk * 1e3 / info["clock_khz"]), 4)
                                                         if sclk and info["clock_khz"] else None),
                     "executed_tflop_per_step": round(executed / 1e12, 3),
                     "executed_counts": "what the kernels multiply: residual and gated terms, and of the symmetric "
                                        "products the 256x256 tiles on or below the diagonal, each in full "
                                        "(= the profiler's matrix-instruction count)",
                     "lower_triangle_128_tflop_per_step": round(lower128 / 1e12, 3),
                     "frac_on_lower_triangle_128": round(lower128 / (gemm_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4) if gemm_ms else 0.0,
                     "dense_tflop_per_step": round(dense / 1e12, 3)},
        "adamw_hbm": {"bound": "hbm", "achieved": round(adamw_gbps, 1), "peak": PEAK_HBM_GBPS,
                      "unit": "GB/s", "frac": round(adamw_gbps / PEAK_HBM_GBPS, 4),
                      "bytes_per_elem": 28, "ms": round(kind_ms["adamw"], 4)},
        "gradnorm_hbm": {"achieved": round(gn_gbps, 1), "unit": "GB/s",
                         "frac": round(gn_gbps / PEAK_HBM_GBPS, 4), "bytes_per_elem": 2,
                         "ms": round(kind_ms["gradnorm_partials"], 4)},
        "muon_elementwise_hbm": {"achieved": round(elem_gbps, 1), "unit": "GB/s",
                                 "frac": round(elem_gbps / PEAK_HBM_GBPS, 4), "bytes_per_param": int(elem_bytes),
                                 "moved_bytes_per_param": int(elem_moved),
                                 "moved_gbps": round(elem_gbps * elem_moved / elem_bytes, 1),
                                 "ms": round(elem_ms, 4),
                                 "kernels": "momentum; the update runs in the epilogue of the chain's last GEMM"
                                 if upd_fused else "momentum + update"},
        "ns_mfma_util_pct": round(100 * achieved / PEAK_BF16_TFLOPS, 2),
        "kernel_ms_per_step": {k: round(v, 4) for k, v in kind_ms.items()},
        "event_ms_per_step": round(ev_ms, 3), "wall_ms_per_step": round(wall_ms, 3),
        "streams": "serial" if args.serial else "one: the Newton-Schulz chains of all shape groups advance together (grouped launches)",
        "host_sync": "none inside the timed region: the steps are counted on the device and queued back to back",
        "copy_kernel_gbps": round(copy_gbps, 1),
        "sustained_sclk_mhz": sclk,
        "sustained_power_w": watts,
        "grad_norm": ctl["norm"], "clip_scale": ctl["clip_scale"],
        "device": {"name": info["name"] or info["arch"].split(":")[0], "arch": info["arch"], "cus": info["cu_count"],
                   "clock_khz": info["clock_khz"]},
    }
    if args.workload == "qwen3" and args.layers == 28 and not args.no_configs:
        out["configs"] = other_configs(opt, gdev, args)        # frees opt on the way
    else:
        opt.free()
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(shapes)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()

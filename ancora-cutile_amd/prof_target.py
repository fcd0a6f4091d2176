"""Single-kernel profiling targets for rocprofv3 (the role of the reference's Nsight Compute
targets, tests/hardware/_ncu_train_target.py:1-3,50-57).

    python3 -m ancora_cutile_amd.prof_target ns M N E [mode] [calls] [times]   Newton-Schulz chain
                                      (a last word `times` adds one call under the library's
                                      per-launch event timer and prints ms per kernel kind)
    python3 -m ancora_cutile_amd.prof_target adamw NUMEL [calls]         fused AdamW, bf16 grads, SR
    python3 -m ancora_cutile_amd.prof_target gradnorm NUMEL [calls]      grad-norm partials + finalize
    python3 -m ancora_cutile_amd.prof_target quant K N E [cm] [calls]    MXFP8 weight re-quantisation
                                      (prints GB/s from HIP events around the calls)
    python3 -m ancora_cutile_amd.prof_target dwlayer [T] [calls] [x|xT]  weight-gradient GEMMs of one layer in one call
    python3 -m ancora_cutile_amd.prof_target dw T K N1[,N2,..] [calls]   weight-gradient GEMM of up to 8
                                      weights (K, Ni) that share the activations, T tokens

    python3 -m ancora_cutile_amd.prof_target embed [V] [H] [TOKENS] [steps]  sorted-scatter embedding
                                      gradient + row-sparse AdamW step beside the dense AdamW sweep
                                      of the same table (prints us per call from HIP events)

Each target allocates its operands, runs the kernel(s) `calls` times on the null stream and
synchronises; nothing is checked here (parity lives in tests/).
"""
import ctypes
import sys

import numpy as np


def main(argv):
    from . import DevBuf, StepGuard, _lib
    from .adamw import hyper_div
    from .muon_ns import ns_batched, PE_SCHEDULE
    _lib.init(0)
    what = argv[0]
    if what == "ns":
        M, N, E = int(argv[1]), int(argv[2]), int(argv[3])
        mode = argv[4] if len(argv) > 4 else "bf16"
        calls = int(argv[5]) if len(argv) > 5 else 2
        one = np.random.default_rng(0).standard_normal((M, N)).astype(np.float32)
        X = DevBuf.empty((E * M, N), np.float32)
        for e in range(E):
            X.at_pos(e * M).upload(one)
        for _ in range(calls):
            ns_batched(X, E, M, N, 0, schedule=PE_SCHEDULE, mode=mode)
        if len(argv) > 6 and argv[6] == "times":
            _lib.stream_sync(0)
            _lib.profile_enable(True)
            ns_batched(X, E, M, N, 0, schedule=PE_SCHEDULE, mode=mode)
            pr = _lib.profile_read()
            _lib.profile_enable(False)
            print("  ".join(f"{k}={v[0]:.3f}ms/{v[1]}" for k, v in pr.items() if v[1]))
    elif what == "adamw":
        n = int(argv[1]) // 64 * 64
        calls = int(argv[2]) if len(argv) > 2 else 3
        g = DevBuf.zeros((n,), np.uint16)
        m, v, p = (DevBuf.zeros((n,), np.float32) for _ in range(3))
        p16 = DevBuf.zeros((n,), np.uint16)
        for t in range(1, calls + 1):
            h = hyper_div(3e-4, 0.9, 0.95, 1e-8, 1000 + t, sr=True, seed_base=t)
            _lib.api.anc_adamw(g.ptr, m.ptr, v.ptr, p.ptr, p16.ptr, n, _lib.BF16, ctypes.byref(h),
                               0.1, 0, 0, 0)
    elif what == "gradnorm":
        n = int(argv[1])
        calls = int(argv[2]) if len(argv) > 2 else 3
        g = DevBuf.zeros((n,), np.uint16)
        guard = StepGuard(1.0)
        for _ in range(calls):
            guard.compute([g], 0)
    elif what == "quant":
        K, N, E = int(argv[1]), int(argv[2]), int(argv[3])
        cm = len(argv) > 4 and argv[4] == "cm"
        calls = int(argv[5]) if len(argv) > 5 else 5
        wb = (np.random.default_rng(0).standard_normal((K, N)) * 0.05).astype(np.float32)
        wb = (wb.view(np.uint32) >> 16).astype(np.uint16)
        w = DevBuf.empty((E * K, N), np.uint16)
        for e in range(E):
            w.at_pos(e * K).upload(wb)
        f8 = DevBuf.zeros((E * K * N,), np.uint8)
        sc = DevBuf.zeros((E * K * N // 32,), np.uint8)
        t0, t1 = _lib.Event(), _lib.Event()
        _lib.api.anc_quant_mxfp8_w(w.ptr, f8.ptr, sc.ptr, E, K, N, int(cm), 0)
        t0.record(0)
        for _ in range(calls):
            _lib.api.anc_quant_mxfp8_w(w.ptr, f8.ptr, sc.ptr, E, K, N, int(cm), 0)
        t1.record(0)
        t1.sync()
        ms = t0.elapsed_ms(t1) / calls
        nbytes = E * K * N * (2 + 1 + 1 / 32)
        print(f"quant_mxfp8_w {'column-major' if cm else 'row-major'} {E}x({K},{N}): {ms * 1e3:.1f} us per call, "
              f"{nbytes / ms / 1e9:.2f} TB/s of {nbytes / 1e9:.3f} GB algorithmic")
    elif what == "dw":
        from .grads import gemm_dW, DwWorkspace, dw_info
        T, K = int(argv[1]), int(argv[2])
        Ns = [int(v) for v in argv[3].split(",")]
        calls = int(argv[4]) if len(argv) > 4 else 5
        rng = np.random.default_rng(0)
        bits = lambda a: (a.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        xT = DevBuf(bits(0.1 * rng.standard_normal((K, T))))
        probs = [dict(xT=xT, dy=DevBuf(bits(0.1 * rng.standard_normal((T, N)))), dW=DevBuf.zeros((K, N), np.float32),
                      g16=DevBuf.zeros((K, N), np.uint16), T=T, K=K, N=N, workspace=DwWorkspace()) for N in Ns]
        gemm_dW(probs)
        _lib.stream_sync(0)
        _lib.profile_enable(True)
        for _ in range(calls):
            gemm_dW(probs)
        pr = _lib.profile_read()
        _lib.profile_enable(False)
        fl = sum(dw_info(T, K, N)[0] for N in Ns)
        gms, rms = pr["dw_gemm"][0] / calls, pr["dw_reduce"][0] / calls
        print(f"dW T={T} K={K} N={Ns} segments={[dw_info(T, K, N)[1] for N in Ns]}: gemm {gms * 1e3:.1f} us "
              f"({fl / gms / 1e9:.1f} TFLOP/s), reduce {rms * 1e3:.1f} us, together {fl / (gms + rms) / 1e9:.1f} TFLOP/s")
    elif what == "dwlayer":
        # the 7 weights of one Qwen3-0.6B layer in one call, one token segment each
        from .grads import gemm_dW, DwWorkspace, dw_info
        T = int(argv[1]) if len(argv) > 1 else 8192
        calls = int(argv[2]) if len(argv) > 2 else 5
        xkey = argv[3] if len(argv) > 3 else "x"          # x: activations (T, K) as they lie; xT: (K, T)
        rng = np.random.default_rng(0)
        bits = lambda a: (a.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        probs, fl = [], 0.0
        for K, Ns in ((1024, (2048, 1024, 1024)), (2048, (1024,)), (1024, (3072, 3072)), (3072, (1024,))):
            xT = DevBuf(bits(0.1 * rng.standard_normal((T, K) if xkey == "x" else (K, T))))
            for N in Ns:
                probs.append(dict(**{xkey: xT}, dy=DevBuf(bits(0.1 * rng.standard_normal((T, N)))),
                                  dW=DevBuf.zeros((K, N), np.float32), g16=DevBuf.zeros((K, N), np.uint16),
                                  T=T, K=K, N=N, workspace=DwWorkspace(), accumulate=True))
                fl += dw_info(T, K, N)[0]
        gemm_dW(probs, 0, segments=1)
        _lib.stream_sync(0)
        _lib.profile_enable(True)
        for _ in range(calls):
            gemm_dW(probs, 0, segments=1)
        pr = _lib.profile_read()
        _lib.profile_enable(False)
        gms, rms = pr["dw_gemm"][0] / calls, pr["dw_reduce"][0] / calls
        print(f"dW of one layer (7 weights, T={T}, 1 segment, 480 workgroups): gemm {gms * 1e3:.1f} us "
              f"({fl / gms / 1e9:.1f} TFLOP/s), finish {rms * 1e3:.1f} us, together {fl / (gms + rms) / 1e9:.1f} TFLOP/s")
    elif what == "embed":
        from .adamw import AdamW
        from .embed import IdGroups, RowSparseAdamW, embed_dw_scatter
        from .bf16 import bf16_bits
        V = int(argv[1]) if len(argv) > 1 else 151936
        H = int(argv[2]) if len(argv) > 2 else 1024
        T = int(argv[3]) if len(argv) > 3 else 8192
        steps = int(argv[4]) if len(argv) > 4 else 20
        rng = np.random.default_rng(0)
        W = (0.02 * rng.standard_normal((V, H))).astype(np.float32)
        sparse = RowSparseAdamW(W, sr=True, seed=1)
        dense = AdamW({"embed": W}, sr=True, seed=1, grad_dtype=np.float32)
        dy = DevBuf(bf16_bits((1e-2 * rng.standard_normal((T, H))).astype(np.float32)))
        compact = DevBuf.zeros((T, H), np.float32)
        gdense = DevBuf.zeros((V, H), np.float32)
        e = [_lib.Event() for _ in range(4)]
        t_sc = t_sp = t_de = t_cu = 0.0
        uniq = 0
        for it in range(steps + 1):
            ids = np.minimum((V * rng.random(T) ** 2).astype(np.int32), V - 1)      # skewed token ids
            grp = IdGroups(ids)
            e[0].record(0)
            sparse.catch_up(ids, 0)
            e[1].record(0)
            embed_dw_scatter(grp, dy, 0, compact=compact)
            e[2].record(0)
            sparse.step(grp.gid, grp.n_groups, compact, 0)
            e[3].record(0)
            e[3].sync()
            if it:                                          # first round warms up
                t_cu += e[0].elapsed_ms(e[1]); t_sc += e[1].elapsed_ms(e[2]); t_sp += e[2].elapsed_ms(e[3])
                uniq += grp.n_groups
            e[0].record(0)
            dense.launch({"embed": gdense}, 0)
            e[1].record(0)
            e[1].sync()
            if it:
                t_de += e[0].elapsed_ms(e[1])
            grp.free()
        print(f"(V, H) = ({V}, {H}), {T} tokens per step, {uniq / steps:.0f} distinct rows on average, {steps} steps")
        print(f"  catch-up of the rows the forward gathers  {t_cu / steps * 1e3:8.1f} us (includes the upload of the row list)")
        print(f"  sorted-scatter gradient rows              {t_sc / steps * 1e3:8.1f} us")
        print(f"  row-sparse AdamW step                     {t_sp / steps * 1e3:8.1f} us (includes the 16-byte step-table upload)")
        print(f"  dense AdamW sweep of the same table       {t_de / steps * 1e3:8.1f} us ({28.0 * V * H / (t_de / steps) / 1e9:.2f} TB/s)")
    else:
        raise SystemExit(__doc__)
    _lib.api.anc_device_sync()
    print("done")


if __name__ == "__main__":
    main(sys.argv[1:])

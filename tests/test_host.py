"""Host-side checks that need no GPU: the C ABI library loads and exports every symbol the
header declares, struct layouts match, routing, and the absence of any CPU fallback."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "anc_optim.h")


def _declared():
    txt = open(HEADER).read()
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    return sorted(set(re.findall(r"\b(anc_[a-z0-9_]+)\s*\(", txt)))


def test_library_exports_every_declared_symbol():
    from ancora_cutile_amd import _lib
    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = _declared()
    assert len(names) >= 35
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/anc_optim.h but not exported"
    assert sorted(_lib.EXPORTS) == names, "ctypes prototypes and header disagree"
    _lib.load()
    assert _lib.api.anc_abi_version() == _lib.ABI_VERSION == 3


def test_struct_sizes_match_header():
    from ancora_cutile_amd import _lib
    assert ctypes.sizeof(_lib.StepCtl) == 32
    assert ctypes.sizeof(_lib.AdamWHyper) == 56
    assert ctypes.sizeof(_lib.AdamWDesc) == 72
    assert ctypes.sizeof(_lib.GnDesc) == 40
    assert ctypes.sizeof(_lib.MuonDesc) == 80
    assert ctypes.sizeof(_lib.DeviceInfo) == 24 + 16 + 128


def test_header_is_plain_c_and_layouts_match_ctypes(tmp_path):
    """include/anc_optim.h compiles as C99 with gcc (no C++ in the boundary) and every struct has
    the size and the field offsets the ctypes mirror assumes."""
    import shutil
    import subprocess
    from ancora_cutile_amd import _lib
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    pairs = [("anc_step_ctl_t", _lib.StepCtl), ("anc_adamw_hyper_t", _lib.AdamWHyper),
             ("anc_adamw_step_t", _lib.AdamWStepEntry),
             ("anc_adamw_desc_t", _lib.AdamWDesc), ("anc_gn_desc_t", _lib.GnDesc),
             ("anc_muon_desc_t", _lib.MuonDesc), ("anc_ns_problem_t", _lib.NsProblem),
             ("anc_dw_problem_t", _lib.DwProblem),
             ("anc_device_info_t", _lib.DeviceInfo)]
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "anc_optim.h"', 'int main(void) {']
    for cname, ct in pairs:
        lines.append(f'  printf("{cname} %zu", sizeof({cname}));')
        for fname, _ in ct._fields_:
            lines.append(f'  printf(" %zu", offsetof({cname}, {fname}));')
        lines.append('  printf("\\n");')
    lines += ['  return 0;', '}']
    src = tmp_path / "abi.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "abi"
    subprocess.run([gcc, "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"),
                    str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split("\n")
    for (cname, ct), line in zip(pairs, out):
        vals = line.split()
        assert vals[0] == cname and int(vals[1]) == ctypes.sizeof(ct), line
        for (fname, _), off in zip(ct._fields_, vals[2:]):
            assert int(off) == getattr(ct, fname).offset, (cname, fname)


def test_no_gpu_means_error_not_fallback():
    """Without a GPU the product path must raise; it never computes on the CPU."""
    from ancora_cutile_amd import _lib
    if os.path.exists("/dev/kfd"):
        pytest.skip("a GPU is present")
    from ancora_cutile_amd import AdamW
    with pytest.raises(_lib.AncoraError):
        AdamW({"w": np.zeros((64,), np.float32)})


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "ancora-cutile_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                src = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", src, flags=re.M), f
                assert "oracle/" not in src and "oracle." not in src.replace("oracle. ", ""), f


def test_routing_predicates():
    from ancora_cutile_amd import default_is_muon, resident_is_muon
    from oracle.muon_ref import default_is_muon as ref
    names = ["embed", "lm_head", "final_norm", "layer0.input_ln", "layer0.q_norm", "layer0.q_proj",
             "layer1.o_proj", "layer5.down_proj", "layer1.ffn.router", "layer1.ffn.gate_proj"]
    for n in names:
        for arr in (np.zeros((128, 256)), np.zeros(64), np.zeros((4, 128, 128)), np.zeros((1024, 16))):
            assert default_is_muon(n, arr) == ref(n, arr)
    assert resident_is_muon("layer1.ffn.gate_proj", np.zeros((16, 128, 128)))
    assert not resident_is_muon("layer1.ffn.router", np.zeros((1024, 16)))
    assert not resident_is_muon("layer1.ffn.router", np.zeros((1024, 128)))
    assert not resident_is_muon("embed", np.zeros((1024, 128)))
    assert resident_is_muon("layer0.o_proj", np.zeros((2048, 1024)))


def test_schedule_toggle_and_constants():
    from ancora_cutile_amd import muon_ns
    assert (muon_ns.NTM, muon_ns.NTN, muon_ns.NTK) == (128, 128, 64)
    prev = muon_ns.set_polar_express(True)
    assert prev is None and muon_ns._resolve(muon_ns._KELLER) is muon_ns.PE_SCHEDULE
    assert muon_ns._resolve(None) is None                      # explicit None still means Keller
    # Keller's coefficients turn "bf16" into the late-three plan; Polar Express keeps the gated one
    assert muon_ns.effective_mode("bf16", None) == "bf16_late3"
    assert muon_ns.effective_mode("bf16", [(3.4445, -4.7750, 2.0315)] * 5) == "bf16_late3"
    assert muon_ns.effective_mode("bf16", muon_ns.PE_SCHEDULE) == "bf16"
    for m in ("bf16_gated", "bf16_fast", "bf16_x3", "fp32"):
        assert muon_ns.effective_mode(m, None) == m
    assert muon_ns.set_polar_express(False) is muon_ns.PE_SCHEDULE
    assert muon_ns._coef_at(muon_ns.PE_SCHEDULE, 7) == muon_ns.PE_SCHEDULE[-1]
    assert muon_ns._coef_at(None, 0) == (3.4445, -4.7750, 2.0315)
    from ancora_cutile_amd.adamw import _pick_otm, C
    assert C == 64 and _pick_otm(256) == 128 and _pick_otm(3) == 1 and _pick_otm(6) == 2


def test_bf16_host_helpers_match_oracle():
    from ancora_cutile_amd.bf16 import bf16_bits, bits_f32
    from oracle.bf16_ref import bf16_rne_bits, bits_to_f32
    x = np.random.default_rng(0).standard_normal(1000).astype(np.float32)
    assert np.array_equal(bf16_bits(x), bf16_rne_bits(x))
    assert np.array_equal(bits_f32(bf16_bits(x)), bits_to_f32(bf16_rne_bits(x)))


def test_flop_accounting_matches_the_tiles_the_kernels_multiply():
    """Host arithmetic only. (1024, 3072), 5 steps, no residual terms: per step the symmetric
    products multiply 10 lower 256x256 tiles (36 lower 128x128 tiles on the small-tile kernel) over
    K = N and K = M, the third product all of 2 M^2 N."""
    from ancora_cutile_amd.muon_ns import ns_flops, ns_product_flops
    M, N, E = 1024, 3072, 3
    ex, de = ns_flops(E, M, N, 5, "bf16_fast")
    assert de == E * 5 * (4.0 * M * M * N + 2.0 * M ** 3)
    assert ex == E * 5 * (10 * 2 * 256 * 256 * (N + M) + 2.0 * M * M * N)
    ex128, _ = ns_flops(E, M, N, 5, "bf16_fast_tile128")
    assert ex128 == E * 5 * (36 * 2 * 128 * 128 * (N + M) + 2.0 * M * M * N)
    assert ns_flops(E, 384, 768, 5, "bf16_fast")[0] == E * 5 * (6 * 2 * 128 * 128 * (768 + 384) + 2.0 * 384 * 384 * 768)
    assert sum(ns_product_flops(E, M, N, k, p, 5, "bf16_fast") for k in range(5) for p in range(3)) == ex
    # 1024 x 1024: iteration 4 carries the residual of X for every matrix (3 terms in A = X X^T, 2 in
    # X = a X + B X); iteration 3 only for matrices above the low gate (anc_ns_hard_info adds those)
    ex_sq, _ = ns_flops(1, M, M, 5, "bf16")
    sym = 10 * 2 * 256 * 256 * M
    assert ex_sq == 4 * (2 * sym + 2.0 * M ** 3) + 1 * (3 * sym + sym + 2 * 2.0 * M ** 3)
    assert ns_flops(1, M, M, 5, "fp32")[0] == ns_flops(1, M, M, 5, "fp32")[1]


def test_bench_reads_gemm_traffic_from_a_counter_database(tmp_path):
    """bench.py --traffic: bytes per GEMM launch = counter sum over the GEMM launches, in the unit the
    1 GiB copy kernel of the same run fixes. A hand-made database with a known answer."""
    import sqlite3
    import sys
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench
    db = str(tmp_path / "x_results.db")
    con = sqlite3.connect(db)
    con.execute("create table counters_collection (kernel_name text, counter_name text, value real)")
    rows = [("k_copy16(a, b, long)", "FETCH_SIZE", 524288.0), ("k_copy16(a, b, long)", "FETCH_SIZE", 524288.0),
            ("void k_ns_gemm_big<0, 256>(NsGemmMulti)", "FETCH_SIZE", 1000.0),
            ("void k_ns_gemm_big<2, 128>(NsGemmMulti)", "FETCH_SIZE", 3000.0),
            ("void k_ns_gemm_big<2, 128>(NsGemmMulti)", "WRITE_SIZE", 77.0),
            ("k_adamw_multi", "FETCH_SIZE", 5.0)]
    con.executemany("insert into counters_collection values (?, ?, ?)", rows)
    con.commit()
    con.close()
    per_launch, n, unit = bench.gemm_bytes_from_counter_db(db, "FETCH_SIZE")
    assert unit == 2.0 and n == 2 and per_launch == (1000.0 + 3000.0) * 2.0 * 1024.0 / 2
    with pytest.raises(RuntimeError):
        bench.gemm_bytes_from_counter_db(db, "WRITE_SIZE")          # no copy kernel row for this counter

"""CPU-side checks of the product's host layer: the C ABI library loads and exports every symbol the
header declares, and its layout/planner routines agree with the oracle byte for byte. No device
compute is called here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = set()
    for header in sorted(os.listdir(os.path.join(ROOT, "include"))):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(tsp_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_library_exports_every_declared_symbol(tsp):
    dll = tsp.dll()
    names = declared_symbols()
    assert len(names) >= 20
    missing = [n for n in names if not hasattr(dll, n)]
    assert not missing, missing
    assert dll.tsp_abi_version() >= 1


def test_struct_sizes_match_reference_abi(tsp):
    # include/tokspur/grouped_mm.hpp:8-13 (56-byte args) and planar_pack_v3.hpp:48-61.
    assert C.sizeof(tsp.GroupedMmPlan) == 120 and C.sizeof(tsp.PlanarSpec) == 80


def test_encoding_table(tsp, orc):
    for t in (0, 1, 2, 3, 6, 7, 8, 10, 11, 12, 13, 14, 20, 23, 24, 25, 26, 27, 28, 30):
        assert tsp.encoding(t) == orc.encoding(t)
    with pytest.raises(tsp.FormatError):
        tsp.encoding(9)


@pytest.mark.parametrize("t,cols,rows", [(12, 512, 8), (13, 256, 12), (8, 64, 8), (7, 96, 4)])
def test_planar_pack_matches_oracle(tsp, orc, synth, t, cols, rows):
    mine, theirs = tsp.make_expert_spec(t, cols, rows), orc.make_expert_spec(t, cols, rows)
    assert bytes(mine) == bytes(theirs)
    raw = synth.matrix(t, 500 + t, rows, cols)
    planar = tsp.pack_expert(mine, raw)
    assert np.array_equal(planar, orc.pack_expert(theirs, raw))
    assert np.array_equal(tsp.unpack_expert(mine, planar), raw)
    bad = planar.copy()
    if t in (12, 13):
        bad[mine.sm_offset + 3] |= 0x40
        with pytest.raises(tsp.FormatError):
            tsp.unpack_expert(mine, bad)


def test_spec_refusals_match_oracle(tsp, orc):
    from oracle.oracle import FormatError as OracleRefusal
    for args in ((12, 2048, 6), (12, 300, 8), (8, 32, 4), (12, 2048, 0), (7, 48, 8), (2, 256, 8)):
        with pytest.raises(OracleRefusal):
            orc.make_expert_spec(*args)
        with pytest.raises(tsp.FormatError):
            tsp.make_expert_spec(*args)


def test_q6k_planar_extension_round_trip(tsp, orc, synth):
    # Not a reference layout: pinned by bijection (byte-exact unpack) and plane geometry.
    cols, rows = 512, 16
    s = tsp.make_expert_spec(14, cols, rows)
    nb = rows * cols // 256
    assert (s.qs_offset, s.qh_offset, s.sm_offset, s.dm_offset, s.planar_expert_bytes) == (0, 128 * nb, 192 * nb, 208 * nb, 210 * nb)
    raw = synth.matrix(14, 77, rows, cols)
    planar = tsp.pack_expert(s, raw)
    assert np.array_equal(tsp.unpack_expert(s, planar), raw)
    blocks = raw.reshape(nb, 210)
    assert np.array_equal(planar[:128 * nb].reshape(nb, 128), blocks[:, :128])
    assert np.array_equal(planar[128 * nb:192 * nb].reshape(nb, 64), blocks[:, 128:192])
    assert np.array_equal(planar[192 * nb:208 * nb].reshape(nb, 16), blocks[:, 192:208])
    assert np.array_equal(planar[208 * nb:].reshape(nb, 2), blocks[:, 208:])
    with pytest.raises(tsp.FormatError):
        tsp.make_expert_spec(14, 256, 4)  # 4 blocks: planes would not be 16-byte aligned


def test_sm16_matches_oracle(tsp, orc):
    rng = np.random.default_rng(2)
    for h in rng.integers(0, 256, size=(2000, 12), dtype=np.uint8):
        sm = tsp.pack_sm16(h)
        assert np.array_equal(sm, orc.pack_sm16(h)) and np.array_equal(tsp.unpack_sm16(sm), h)


def test_coloc_matches_oracle(tsp, orc, synth):
    cols, rows, experts = 256, 8, 4
    spec_t, spec_o = tsp.make_expert_spec(12, cols, rows), orc.make_expert_spec(12, cols, rows)
    gate, up = synth.matrix(12, 61, rows * experts, cols), synth.matrix(12, 62, rows * experts, cols)
    for half in (0, 1):
        assert np.array_equal(tsp.pack_coloc_half(spec_t, gate, up, experts, half), orc.pack_coloc_half(spec_o, gate, up, experts, half))
    with pytest.raises(tsp.FormatError):
        tsp.pack_coloc_half(spec_t, gate, up, 3, 0)


@pytest.mark.parametrize("cols", [32, 512, 2048, 544])
def test_q8_lanes_matches_oracle(tsp, orc, synth, cols):
    raw = synth.matrix(8, 71, 3, cols)
    packed = tsp.q8_lanes_pack_rows(cols, raw)
    assert np.array_equal(packed, orc.q8_lanes_pack_rows(cols, raw))
    assert np.array_equal(tsp.q8_lanes_unpack_rows(cols, packed), raw)
    for b in (0, cols // 32 - 1):
        for i in (0, 31):
            assert tsp.q8_lanes_quant_offset(cols, b, i) == orc.q8_lanes_quant_offset(cols, b, i)


@pytest.mark.parametrize("cols", [32, 640, 2048, 544])
def test_q51_lanes_matches_oracle(tsp, orc, synth, cols):
    raw = synth.matrix(7, 72, 3, cols)
    packed = tsp.q51_lanes_pack_rows(cols, raw)
    assert np.array_equal(packed, orc.q51_lanes_pack_rows(cols, raw))
    assert np.array_equal(tsp.q51_lanes_unpack_rows(cols, packed), raw)
    for b in (0, cols // 32 - 1):
        for i in (0, 15):
            assert tsp.q51_lanes_quant_offset(cols, b, i) == orc.q51_lanes_quant_offset(cols, b, i)
    with pytest.raises(tsp.FormatError):
        tsp.q51_lanes_quant_offset(cols, 0, 16)
    with pytest.raises(tsp.FormatError):
        tsp.q51_lanes_pack_rows(cols, raw[:-1])


def test_planners_match_oracle(tsp, orc):
    from oracle.oracle import FormatError as OracleRefusal
    rng = np.random.default_rng(9)
    for _ in range(300):
        args = (int(rng.choice([7, 8, 12, 13, 14])), int(rng.choice([0, 0, 1, 2])), int(rng.choice([32, 256, 640, 2048, 2560, 300])),
                int(rng.integers(1, 3000)), int(rng.choice([1, 2, 8, 512, 600])), int(rng.integers(1, 18)),
                int(rng.choice([1, 31, 512, 600, 2048])), int(rng.choice([128, 8192, 10240, 10272])), int(rng.choice([16, 8192, 12000])),
                bool(rng.integers(0, 2)), bool(rng.integers(0, 2)))
        try:
            want = bytes(orc.grouped_mm_plan(*args))
        except OracleRefusal:
            with pytest.raises(tsp.FormatError):
                tsp.grouped_mm_plan(*args)
            continue
        assert bytes(tsp.grouped_mm_plan(*args)) == want
    # native/tests/test_moe_mm_many.cpp:13-31 byte goldens through the product's planner.
    views, total = tsp.moe_mm_many_bytes(2560, 640, 512, 10, 512)
    assert views == [1048576, 20480, 20480, 13107200, 13107200, 52428800, 1310720, 1310720, 5242880, 2048, 1048576, 2048, 5384]
    assert total == sum(views)
    for args in ((2560, 640, 512, 10, 1025), (2560, 640, 512, 6, 2048), (2560, 640, 8, 10, 512), (2561, 640, 512, 10, 512)):
        with pytest.raises(tsp.FormatError):
            tsp.moe_mm_many_bytes(*args)
    assert tsp.moe_mm_many_bytes(2048, 512, 512, 10, 2048, True) == orc.moe_mm_many_bytes(2048, 512, 512, 10, 2048, True)
    # dense plan: native/src/grouped_mm.cpp:48-54
    p = tsp.dense_mm_q8_plan(0, 2048, 4096, 100, 8192, 16384)
    assert (p.maximum_tasks, p.grid_y, p.indices_bytes, p.tasks_bytes) == (4, 4, 0, 0)
    assert [tsp.q8_many_width(n) for n in (1, 2, 3, 4, 7, 8, 16)] == [1, 2, 2, 4, 4, 8, 8]
    assert [tsp.q8_many_chunks(n) for n in (1, 3, 15, 16)] == [1, 2, 4, 2]


def test_missing_library_fails_loudly(tsp, monkeypatch, tmp_path):
    monkeypatch.setattr(tsp, "_dll", None)
    monkeypatch.setattr(tsp, "LIB_PATH", str(tmp_path / "absent.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        tsp.dll()


def test_host_class_library_exports_graph_operators():
    """libtokspur_graph.so (tokspur::HipGraph, the C++ mirror of the engine's graph class) carries every operator of the path."""
    import subprocess
    lib = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "tokspur-public_amd", "libtokspur_graph.so")
    assert os.path.exists(lib), "run __graft_entry__.build()"
    names = subprocess.run(["nm", "-D", "--demangle", lib], stdout=subprocess.PIPE, text=True, check=True).stdout
    for op in ("gemv", "gemv_rows", "q8_matvec_many", "route", "prefill_route_batch", "routed_gemv", "swiglu", "mixture", "prefill_mixture_batch",
               "register_planar_matrix", "planar_matrix_shape", "prepare_planar_moe_v3", "planar_moe_gate_up_swiglu_m8", "planar_moe_routed_m8",
               "planar_nax_grouped_moe", "dense_mm", "logit_topk", "validate_disjoint", "begin", "submit", "abort", "zeros", "upload", "release"):
        assert f"tokspur::HipGraph::{op}(" in names, op
    for fn in ("tokspur::encode_moe(", "tokspur::encode_moe_batch(", "tokspur::allocate_moe_scratch(", "tokspur::is_planar_moe("):
        assert fn in names, fn


def test_gemm_staging_waits_match_the_compiled_load_order(tmp_path):
    """The GEMM kernels bring activation slabs in with direct global -> LDS loads that no register dependency waits
    for: each K step waits with `s_waitcnt vmcnt(N)` where N is the number of younger vector-memory operations, written
    into the source as constants. This compiles gemm.hip to assembly and recounts, per kernel and loop: at an even step
    N must equal the other loads of the even step before; at an odd step, those of the even step three back plus the
    slab loads and the other loads of the step before."""
    import importlib
    import shutil
    import subprocess
    if shutil.which("hipcc") is None:
        pytest.skip("hipcc not on PATH")
    build = importlib.import_module("tokspur-public_amd.build")
    asm = tmp_path / "gemm.s"
    src = os.path.join(ROOT, "tokspur-public_amd", "csrc", "gemm.hip")
    flags = [f for f in build.HIP_FLAGS if f != "-fPIC"]
    subprocess.run(["hipcc", "-x", "hip", "-S", "--cuda-device-only", src, "-o", str(asm)] + flags, check=True,
                   stdout=subprocess.PIPE, stderr=subprocess.PIPE)
    kernels, name = {}, None
    for text in asm.read_text().splitlines():
        m = re.match(r"^(_Z\w*gemm_kernel\w*):", text)
        if m:
            name = m.group(1)
            kernels[name] = []
        elif name and text.startswith(".Lfunc_end"):  # a kernel may hold several s_endpgm (early exits)
            name = None
        elif name:
            kernels[name].append(text)
    assert len(kernels) >= 9
    loops_checked = 0
    for name, lines in kernels.items():
        loops, current = [], None
        for text in lines:
            if "Loop Header" in text:
                current = []
                loops.append(current)
            elif current is not None:
                current.append(text.strip())
                if text.strip().startswith("s_cbranch_scc"):
                    current = None
        for body in loops:
            steps, waits = [], []  # per K step: [slab loads, other loads]; wait constant at the top of the step
            for text in body:
                m = re.match(r"s_waitcnt vmcnt\((\d+)\) lgkmcnt\(0\)", text)
                if m:
                    waits.append(int(m.group(1)))
                    steps.append([0, 0])
                elif text.startswith("global_load_lds") and steps:
                    steps[-1][0] += 1
                elif (text.startswith("global_load") or text.startswith("buffer_load")) and steps:
                    steps[-1][1] += 1
            if len(waits) != 4:
                continue  # not a K loop
            loops_checked += 1
            for i in range(4):
                if i % 2 == 0:
                    want = steps[(i + 2) % 4][1]
                    assert steps[i][0] > 0 and steps[(i + 1) % 4] == [0, 0], (name, steps)
                else:
                    want = steps[(i + 1) % 4][1] + steps[(i + 3) % 4][0] + steps[(i + 3) % 4][1]
                assert waits[i] == want, (name, i, waits, steps)
    assert loops_checked >= 18  # two loops (one or two row tiles) in each of the nine kernels

"""Pins the oracle's Pack v3 planar layout, q8_lanes_v1 layout, expert permutation, union records,
row top-k and plan geometry against the reference's own checks:
native/tests/test_planar_pack_v3.cpp:194-280, native/tests/test_moe_mm_many.cpp:13-31,
native/tests/test_planar_union_metadata.mm:27-124, native/src/sampling.cpp:473-513."""
import numpy as np
import pytest

from test_oracle_routing import std_mt19937


def scale_min_k4(j, q):
    """The GGUF closed form for sub-block j of a 12-byte Q4_K/Q5_K scale header."""
    if j < 4:
        return q[j] & 63, q[j + 4] & 63
    return (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4), (q[j + 4] >> 4) | ((q[j] >> 6) << 4)


def test_pack_sm16_closed_form_and_round_trip(orc):
    # native/tests/test_planar_pack_v3.cpp:194-233
    from oracle.oracle import FormatError
    rng = np.random.default_rng(12)
    headers = rng.integers(0, 256, size=(65536, 12), dtype=np.uint8)
    for h in headers[:4096]:
        sm = orc.pack_sm16(h)
        for j in range(8):
            sc, mn = scale_min_k4(j, [int(v) for v in h])
            assert sm[j] == sc and sm[8 + j] == mn
        assert np.array_equal(orc.unpack_sm16(sm), h)
    sm = orc.pack_sm16(headers[0]).copy()
    for at in (0, 7, 8, 15):
        bad = sm.copy()
        bad[at] |= 64
        with pytest.raises(FormatError):
            orc.unpack_sm16(bad)


@pytest.mark.parametrize("t,cols,rows", [(12, 512, 8), (13, 256, 12), (8, 64, 8), (7, 96, 4)])
def test_planar_round_trip_and_dequant_equality(orc, cpu, synth, t, cols, rows):
    # native/tests/test_planar_pack_v3.cpp:236-280: unpack(pack(x)) == x, dequant(planar) == dequant(GGUF) bitwise,
    # for both the double and the float planar arithmetic; checked against oracle AND reference GGUF dequant.
    spec = orc.make_expert_spec(t, cols, rows)
    for raw in (synth.matrix(t, 300 + t, rows, cols), orc.fixture_weights(t, cols, rows, 1)):
        planar = orc.pack_expert(spec, raw)
        assert planar.size == spec.planar_expert_bytes and planar.size % 16 == 0
        assert np.array_equal(orc.unpack_expert(spec, planar), raw)
        want = cpu.dequantize(t, raw, rows * cols)
        for f32 in (False, True):
            got = orc.dequantize_expert_planar(spec, planar, f32=f32)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_spec_geometry(orc):
    from oracle.oracle import FormatError
    # Q4_K expert of the MoE configurations: 2048 columns x 512 rows.
    s = orc.make_expert_spec(12, 2048, 512)
    assert (s.blocks_per_row, s.planar_expert_bytes, s.sm_offset, s.dm_offset) == (8, 606208, 4096 * 128, 4096 * 144)
    assert s.source_expert_bytes == 4096 * 144
    s = orc.make_expert_spec(8, 512, 2048)
    assert s.planar_expert_bytes == s.source_expert_bytes == 2048 * 16 * 34 and s.dm_offset == 2048 * 16 * 32
    for bad in ((12, 2048, 6), (12, 300, 8), (8, 32, 4), (14, 256, 8), (12, 2048, 0)):
        with pytest.raises(FormatError):
            orc.make_expert_spec(*bad)


def test_coloc_halves(orc, synth):
    # native/tests/test_planar_pack_v3.cpp:401-424: pair_lo = experts 0..E/2-1 as [gate_e, up_e], pair_hi the rest.
    cols, rows, experts = 256, 8, 6
    spec = orc.make_expert_spec(12, cols, rows)
    gate = synth.matrix(12, 41, rows * experts, cols)
    up = synth.matrix(12, 42, rows * experts, cols)
    for half in (0, 1):
        out = orc.pack_coloc_half(spec, gate, up, experts, half)
        pb, sb = spec.planar_expert_bytes, spec.source_expert_bytes
        for k in range(experts // 2):
            e = half * (experts // 2) + k
            assert np.array_equal(orc.unpack_expert(spec, out[(2 * k) * pb:(2 * k + 1) * pb]), gate[e * sb:(e + 1) * sb])
            assert np.array_equal(orc.unpack_expert(spec, out[(2 * k + 1) * pb:(2 * k + 2) * pb]), up[e * sb:(e + 1) * sb])


@pytest.mark.parametrize("cols", [32, 512, 2048, 544])
def test_q8_lanes_layout(cpu, synth, cols):
    # native/src/expert_lanes.cpp:83-119: scales first, then runs of 16 blocks x 512 B, byte = index*width + block%16.
    blocks = cols // 32
    rows = 3
    raw = synth.matrix(8, 70, rows, cols)
    packed = cpu.q8_lanes_pack_rows(cols, raw)
    assert np.array_equal(cpu.q8_lanes_unpack_rows(cols, packed), raw)
    seen = set()
    for b in range(blocks):
        run, width = b // 16, min(16, blocks - (b // 16) * 16)
        for i in range(32):
            at = cpu.q8_lanes_quant_offset(cols, b, i)
            assert at == blocks * 2 + run * 512 + i * width + b % 16
            seen.add(at)
            assert packed[at] == raw[b * 34 + 2 + i]
        assert np.array_equal(packed[2 * b:2 * b + 2], raw[b * 34:b * 34 + 2])
    assert seen == set(range(blocks * 2, blocks * 34))


@pytest.mark.parametrize("cols", [32, 640, 2048, 544])
def test_q51_lanes_layout(cpu, synth, cols):
    # native/src/expert_lanes.cpp:75-95: 8-byte heads (d, m, qh) first, then runs of 16 blocks x 256 B, byte = index*width + block%16.
    blocks = cols // 32
    rows = 3
    raw = synth.matrix(7, 71, rows, cols)
    packed = cpu.q51_lanes_pack_rows(cols, raw)
    assert np.array_equal(cpu.q51_lanes_unpack_rows(cols, packed), raw)
    seen = set()
    for b in range(blocks):
        run, width = b // 16, min(16, blocks - (b // 16) * 16)
        for i in range(16):
            at = cpu.q51_lanes_quant_offset(cols, b, i)
            assert at == blocks * 8 + run * 256 + i * width + b % 16
            seen.add(at)
            assert packed[at] == raw[b * 24 + 8 + i]
        assert np.array_equal(packed[8 * b:8 * b + 8], raw[b * 24:b * 24 + 8])
    assert seen == set(range(blocks * 8, blocks * 24))
    # the second row starts a whole row later
    assert np.array_equal(packed[blocks * 24:blocks * 24 + 8], raw[blocks * 24:blocks * 24 + 8])


def brute_routes(ids, experts, selected, tokens):
    token_map = {}
    counts = []
    for e in range(experts):
        rids = [r for r in range(tokens * selected) if ids[r] == e]
        token_map[e] = rids  # ascending route id == ascending token, one slot per token
        counts.append(len(rids))
    return token_map, counts


def test_grouped_routes_and_tasks(orc):
    # kernels/grouped_mpp.metal:12-64, pinned by brute force + invariants (nothing in the reference pins it on CPU).
    rng = np.random.default_rng(8)
    for tokens, selected, experts in ((1, 1, 2), (5, 3, 8), (33, 4, 16), (100, 10, 64), (64, 2, 4)):
        ids = np.stack([rng.permutation(experts)[:selected] for _ in range(tokens)]).astype(np.uint32).reshape(-1)
        token_map, counts, err = orc.grouped_routes(ids, experts, selected, tokens)
        assert err == 0 and counts.sum() == tokens * selected
        want_map, want_counts = brute_routes(ids, experts, selected, tokens)
        assert list(counts) == want_counts
        for e in range(experts):
            got = token_map[e * tokens:e * tokens + counts[e]]
            assert list(got) == want_map[e]
            assert all(ids[r] == e for r in got) and list(got) == sorted(got)
            assert (token_map[e * tokens + counts[e]:(e + 1) * tokens] == 0xDEADBEEF).all()  # tail untouched
        tasks, err = orc.grouped_tasks(counts, experts, selected, tokens, 32)
        assert err == 0
        bound = tokens * selected // 32 + experts
        want = [(e, i * 32) for e in range(experts) for i in range((counts[e] + 31) // 32)]
        assert tasks[0] == len(want) <= bound and tasks[1] == tokens * selected
        for i, (e, start) in enumerate(want):
            assert (tasks[2 + 2 * i], tasks[3 + 2 * i]) == (e, start)
        assert (tasks[2 + 2 * len(want):] == 0xFFFFFFFF).all()
    # error bit 4: out-of-range id, duplicate expert inside one token, count mismatch.
    assert orc.grouped_routes(np.array([0, 9], dtype=np.uint32), 4, 2, 1)[2] == 4
    assert orc.grouped_routes(np.array([1, 1], dtype=np.uint32), 4, 2, 1)[2] == 4
    assert orc.grouped_tasks(np.array([1, 0, 0, 0], dtype=np.uint32), 4, 2, 1)[1] == 4


def union_spec(experts, selected, tokens, hidden, channels, ids, poison=0xBAADF00D):
    """native/tests/test_planar_union_metadata.mm:27-55, written as a dictionary of records and then laid out."""
    meta = np.full(2320, poison, dtype=np.uint32)
    meta[:8] = 0
    valid = (0 < experts <= 512 and experts % 2 == 0 and 0 < selected <= 16 and selected <= experts and 0 < tokens <= 8
             and all(i < experts for i in ids))
    if not valid:
        return meta, 4
    capacity = 4 if tokens <= 4 else 8
    records = []  # [expert, [flat routes]]
    for flat, e in enumerate(ids):
        rec = next((r for r in records if r[0] == e and len(r[1]) < capacity), None)
        if rec is None:
            rec = [e, []]
            records.append(rec)
        rec[1].append(flat)
    for slot, (e, flats) in enumerate(records):
        meta[8 + slot], meta[136 + slot] = e, len(flats)
        padded = flats + [flats[0]] * (8 - len(flats))
        meta[264 + 8 * slot:272 + 8 * slot] = [f // selected for f in padded]
        meta[1288 + 8 * slot:1296 + 8 * slot] = padded
    n = len(records)
    meta[:8] = [(hidden + 7) // 8, n, 1, (channels + 15) // 16, n, 1, n, 0]
    return meta, 0


def test_union_metadata_cases(orc):
    # native/tests/test_planar_union_metadata.mm:105-124, seed 1729, T = 1..8 x S = 1..16, four patterns each.
    bg = std_mt19937(1729)
    for tokens in range(1, 9):
        for selected in range(1, 17):
            n = tokens * selected
            cases = [[511] * n, [(511 - i) % 512 for i in range(n)]]
            mixed = [int(bg.random_raw()) % 7 if i % 3 else 511 for i in range(n)]
            cases.append(mixed)
            cases.append(mixed[:-1] + [512])
            for ids in cases:
                got, err = orc.union_metadata(512, selected, tokens, 639, 2559, ids)
                want, want_err = union_spec(512, selected, tokens, 639, 2559, ids)
                assert err == want_err and np.array_equal(got, want), (tokens, selected)
    assert orc.union_metadata(3, 1, 1, 640, 2560, [0])[1] == 4
    assert orc.union_metadata(2, 3, 1, 640, 2560, [0, 1, 0])[1] == 4


def test_logit_topk(cpu):
    # native/src/sampling.cpp:473-513: value desc, id asc, -0 == +0, non-finite skipped, first subnormal recorded.
    rng = np.random.default_rng(21)
    for n in (1, 5, 64, 65, 1000, 5000):
        x = np.round(rng.normal(size=n), 1).astype(np.float32)  # coarse grid: many ties
        if n >= 65:
            x[3], x[7], x[11] = np.inf, np.nan, -0.0
            x[20] = np.float32(1e-41)
        row = cpu.logit_topk_row(x)
        finite = [i for i in range(n) if np.isfinite(x[i])]
        order = sorted(finite, key=lambda i: (-(float(x[i]) + 0.0), i))[:64]
        assert row.count == len(order) and row.vocabulary == n
        assert list(row.ids[:row.count]) == order
        assert [np.float32(v).view(np.uint32) for v in row.logits[:row.count]] == [x[i].view(np.uint32) for i in order]
        nonfinite = [i for i in range(n) if not np.isfinite(x[i])]
        assert row.first_nonfinite_col == (nonfinite[0] if nonfinite else 0xFFFFFFFF)
        sub = [i for i in finite if x[i] != 0 and abs(float(x[i])) < 1.1754943508222875e-38]
        assert row.first_subnormal_col == (sub[0] if sub else 0xFFFFFFFF)


def test_plan_byte_goldens(cpu):
    # native/tests/test_moe_mm_many.cpp:13-31
    from oracle.oracle import FormatError
    views, total = cpu.moe_mm_many_bytes(2560, 640, 512, 10, 512)
    assert views[:3] == [1048576, 20480, 20480]
    assert views[3:6] == [13107200, 13107200, 52428800]
    assert views[6:10] == [1310720, 1310720, 5242880, 2048]
    assert views[10:] == [1048576, 2048, 5384]
    assert sum(views) == total < 96 * 1024 * 1024
    for n in (1, 3, 8, 16, 17, 31, 32, 33, 511, 512):
        for selected in (1, 3, 10, 16):
            v, _ = cpu.moe_mm_many_bytes(2560, 640, 512, selected, n)
            assert v[5] == n * selected * 2560 * 4 and v[10] == n * 512 * 4 and v[11] == 2048
            assert v[12] == (2 + 2 * (n * selected // 32 + 512)) * 4
    assert cpu.moe_mm_many_bytes(2560, 640, 512, 10, 1024)[1] <= 300 << 20
    assert cpu.moe_mm_many_bytes(2560, 640, 512, 5, 2048)[1] <= 300 << 20
    for bad in ((2560, 640, 512, 10, 1025), (2560, 640, 512, 10, 2048), (2560, 640, 512, 10, 0), (2560, 640, 512, 5, 2049),
                (2560, 640, 512, 6, 2048), (0, 640, 512, 10, 512), (2561, 640, 512, 10, 512), (2560, 641, 512, 10, 512),
                (2560, 640, 0, 10, 512), (2560, 640, 513, 10, 512), (2560, 640, 512, 17, 512), (2560, 640, 8, 10, 512)):
        with pytest.raises(FormatError):
            cpu.moe_mm_many_bytes(*bad)
    # The 2K-row MoE configuration needs the widened route cap.
    v, total = cpu.moe_mm_many_bytes(2048, 512, 512, 10, 2048, True)
    assert v[10] == 512 * 2048 * 4 and v[12] == (2 + 2 * (20480 // 32 + 512)) * 4
    # grouped_mm_plan: native/src/grouped_mm.cpp:24-47
    p = cpu.grouped_mm_plan(12, 0, 2048, 8192, 1, 1, 512, 8192, 32768, True)
    assert (p.row_bytes, p.expert_stride_bytes, p.maximum_tasks, p.grid_x, p.grid_y) == (1152, 1152 * 8192, 17, 128, 17)
    assert p.input_bytes == 511 * 8192 + 8192 and p.output_bytes == 511 * 32768 + 32768
    with pytest.raises(FormatError):
        cpu.grouped_mm_plan(14, 0, 2048, 8192, 1, 1, 512, 8192, 32768, True)
    with pytest.raises(FormatError):
        cpu.grouped_mm_plan(12, 0, 2048, 8192, 1, 1, 513, 8192, 32768, True)


def test_oracle_plans_equal_reference(orc, ref):
    from oracle.oracle import FormatError
    rng = np.random.default_rng(4)
    for _ in range(300):
        t = int(rng.choice([7, 8, 12, 13]))
        layout = int(rng.choice([0, 0, 1, 2]))
        args = (t, layout, int(rng.choice([32, 256, 640, 2048, 2560, 300])), int(rng.integers(1, 3000)),
                int(rng.choice([1, 2, 8, 512, 600])), int(rng.integers(1, 18)), int(rng.choice([1, 31, 512, 600, 2048])),
                int(rng.choice([128, 2048 * 4, 2560 * 4, 10272])), int(rng.choice([16, 8192, 12000])),
                bool(rng.integers(0, 2)), bool(rng.integers(0, 2)))
        results = []
        for lib in (orc, ref):
            try:
                p = lib.grouped_mm_plan(*args)
                results.append(bytes(p))
            except FormatError:
                results.append(None)
        assert results[0] == results[1], args


def test_round_bf16(orc, synth):
    # kernels/planar_moe_v3.metal:82-94; closed form: nearest bf16, ties to even mantissa.
    x = np.array([1.0, 1.00390625, 1.01171875, -3.14159, 1e-40, 65504.0, 3.3895313e38, 3.4e38], dtype=np.float32)
    for v in x:
        bits, bad = orc.round_bf16_bits_scalar(float(v))
        lo = int(v.view(np.uint32)) & 0xFFFF0000
        cands = [np.uint32(lo).view(np.float32), np.uint32((lo + 0x10000) & 0xFFFFFFFF).view(np.float32)]
        step = float(np.uint32(0x3F810000).view(np.float32) - 1.0) * 2.0 ** (((lo >> 23) & 255) - 127 if (lo >> 23) & 255 else -126)
        d = [float(v) - float(cands[0]), float(cands[0]) + (step if v >= 0 else -step) - float(v)]
        d = [abs(t) for t in d]
        pick = 0 if d[0] < d[1] else 1 if d[1] < d[0] else (0 if (lo >> 16) % 2 == 0 else 1)
        if not np.isfinite(cands[pick]):
            assert bad == 1
            continue
        assert bits == int(cands[pick].view(np.uint32)) >> 16 and bad == 0
        assert synth.round_bf16(np.array([v]))[0] == cands[pick]
    assert orc.round_bf16_bits_scalar(float("inf"))[1] == 1


def test_moe_routed_reference_brute_force(orc, synth):
    """The composed MoE reference (dequantize -> double dot -> float silu -> double dot) against a numpy
    restatement of native/tests/test_planar_pack_v3.cpp:519-547."""
    channels, hidden, experts, tokens, selected = 256, 32, 4, 3, 2
    gate = synth.matrix(12, 1, hidden * experts, channels)
    up = synth.matrix(12, 2, hidden * experts, channels)
    down = synth.matrix(14, 3, channels * experts, hidden * 8)[:0]  # placeholder, replaced below
    down = synth.matrix(8, 3, channels * experts, hidden)
    x = synth.activations_f32(4, (tokens, channels))
    ids = np.array([0, 3, 1, 0, 2, 3], dtype=np.uint32)
    h, y = orc.moe_routed_reference(12, 8, gate, up, down, channels, hidden, experts, ids, tokens, selected, x, threads=2)
    g = orc.dequantize(12, gate, gate.size // 144 * 256).reshape(experts, hidden, channels).astype(np.float64)
    u = orc.dequantize(12, up, up.size // 144 * 256).reshape(experts, hidden, channels).astype(np.float64)
    d = orc.dequantize(8, down, down.size // 34 * 32).reshape(experts, channels, hidden).astype(np.float64)
    for rid, e in enumerate(ids):
        xv = x[rid // selected].astype(np.float64)
        dg = np.array([sum(g[e, r] * xv) for r in range(hidden)])  # python sum: sequential
        du = np.array([sum(u[e, r] * xv) for r in range(hidden)])
        gf = dg.astype(np.float32)
        hh = (gf / (np.float32(1) + np.exp(-gf).astype(np.float32))) * du.astype(np.float32)
        # expf vs numpy's float exp differ by an ulp, and disagree on overflow right at exp(88.7): atol covers that.
        assert np.allclose(h[rid], hh.astype(np.float64), rtol=3e-7, atol=1e-30)
        yy = np.array([sum(d[e, r] * h[rid]) for r in range(channels)])
        assert np.allclose(y[rid], yy, rtol=1e-13, atol=1e-13)


def q6k_fields(blocks):
    """Independent numpy decode of Q6_K blocks -> (integer codes [nb, 256], int8 sub-scales [nb, 16], d [nb])."""
    blk = np.frombuffer(blocks, dtype=np.uint8).reshape(-1, 210)
    ql, qh = blk[:, :128].astype(np.int32), blk[:, 128:192].astype(np.int32)
    q = np.empty((blk.shape[0], 256), dtype=np.int32)
    for sec in range(2):
        for l in range(32):
            a, b, h = ql[:, sec * 64 + l], ql[:, sec * 64 + 32 + l], qh[:, sec * 32 + l]
            q[:, sec * 128 + l] = (a & 15) | ((h & 3) << 4)
            q[:, sec * 128 + 32 + l] = (b & 15) | (((h >> 2) & 3) << 4)
            q[:, sec * 128 + 64 + l] = (a >> 4) | (((h >> 4) & 3) << 4)
            q[:, sec * 128 + 96 + l] = (b >> 4) | (((h >> 6) & 3) << 4)
    return q, blk[:, 192:208].view(np.int8).astype(np.int32), blk[:, 208:210].copy().view(np.float16).astype(np.float64)[:, 0]


def test_matrix_core_staging_models(orc, synth):
    """stage_f16 = 2 (Q6_K rows as d * half(sc * (q - 32))) and the h = 256 * half(h / 256) carry restate the HIP
    kernels' staging; they have no counterpart in the reference, so they are checked against numpy's own half."""
    rows, cols, tokens = 24, 512, 5
    w = synth.matrix(14, 9100, rows, cols)
    x = synth.round_bf16(synth.activations_f32(9101, (tokens, cols)))
    q, sc, d = q6k_fields(w)
    prod = (q - 32) * np.repeat(sc, 16, axis=1)
    assert (np.abs(prod) > 2048).any()  # the case that rounds is present
    for stage, weights in ((0, prod.astype(np.float64)), (2, prod.astype(np.float16).astype(np.float64))):
        want = x.astype(np.float64) @ (weights * d[:, None]).reshape(rows, cols).T
        got = orc.staged_gemm(14, w, cols, x, nrows=rows, stage_f16=stage)
        assert np.allclose(got, want, rtol=1e-12, atol=1e-9)
    # h carry: stage 4 rounds h to the half nearest h / 256, stage 0 does not; the down product is then exact
    channels, hidden, experts = 256, 256, 2
    gate = synth.matrix(12, 9102, hidden * experts, channels)
    up = synth.matrix(12, 9103, hidden * experts, channels)
    down = synth.matrix(14, 9104, channels * experts, hidden)
    ids = np.array([1, 0, 1], dtype=np.uint32)
    xs = synth.round_bf16(synth.activations_f32(9105, (3, channels)))
    h0, _ = orc.moe_routed_reference(12, 14, gate, up, down, channels, hidden, experts, ids, 3, 1, xs, stage=0)
    h4, y4 = orc.moe_routed_reference(12, 14, gate, up, down, channels, hidden, experts, ids, 3, 1, xs, stage=4)
    carried = (h0.astype(np.float32) * np.float32(1 / 256)).astype(np.float16).astype(np.float64) * 256.0
    assert np.array_equal(h4, carried)
    qd, scd, dd = q6k_fields(down)
    wd = ((qd - 32) * np.repeat(scd, 16, axis=1) * dd[:, None]).reshape(experts, channels, hidden)
    want_y = np.stack([wd[ids[r]] @ carried[r] for r in range(3)])
    assert np.allclose(y4, want_y, rtol=1e-12, atol=1e-6)


@pytest.mark.parametrize("t,cols,rows", [(12, 512, 8), (13, 256, 12), (8, 256, 8), (7, 96, 4)])
def test_planar_plane_byte_positions(orc, synth, t, cols, rows):
    """Every plane byte at its place (native/src/planar_pack_v3.cpp:601-716): blocks in (row, block) order, nibbles and
    high bits verbatim, scales decoded one per byte, d / dmin verbatim. A round trip alone would also pass a pack and an
    unpack that agree on a wrong plane order."""
    raw = synth.matrix(t, 4200 + t, rows, cols)
    spec = orc.make_expert_spec(t, cols, rows)
    planar = orc.pack_expert(spec, raw)
    epb, bpb = orc.encoding(t)
    nb = rows * (cols // epb)
    blk = raw.reshape(nb, bpb)
    def plane(offset, width):
        return planar[offset:offset + nb * width].reshape(nb, width)
    if t == 12:
        assert np.array_equal(plane(spec.qs_offset, 128), blk[:, 16:144])
        want_sm = np.array([[scale_min_k4(j, [int(v) for v in b[4:16]])[0] for j in range(8)] +
                            [scale_min_k4(j, [int(v) for v in b[4:16]])[1] for j in range(8)] for b in blk], dtype=np.uint8)
        assert np.array_equal(plane(spec.sm_offset, 16), want_sm)
        assert np.array_equal(plane(spec.dm_offset, 4), blk[:, 0:4])
        assert (spec.qs_offset, spec.sm_offset, spec.dm_offset, spec.planar_expert_bytes) == (0, 128 * nb, 144 * nb, 148 * nb)
    elif t == 13:
        assert np.array_equal(plane(spec.qs_offset, 128), blk[:, 48:176])
        assert np.array_equal(plane(spec.qh_offset, 32), blk[:, 16:48])
        want_sm = np.array([[scale_min_k4(j, [int(v) for v in b[4:16]])[0] for j in range(8)] +
                            [scale_min_k4(j, [int(v) for v in b[4:16]])[1] for j in range(8)] for b in blk], dtype=np.uint8)
        assert np.array_equal(plane(spec.sm_offset, 16), want_sm)
        assert np.array_equal(plane(spec.dm_offset, 4), blk[:, 0:4])
        assert (spec.qs_offset, spec.qh_offset, spec.sm_offset, spec.dm_offset) == (0, 128 * nb, 160 * nb, 176 * nb)
    elif t == 8:
        assert np.array_equal(plane(spec.qs_offset, 32), blk[:, 2:34])
        assert np.array_equal(plane(spec.dm_offset, 2), blk[:, 0:2])
        assert (spec.qs_offset, spec.dm_offset, spec.planar_expert_bytes) == (0, 32 * nb, 34 * nb)
    else:
        assert np.array_equal(plane(spec.qs_offset, 16), blk[:, 8:24])
        assert np.array_equal(plane(spec.qh_offset, 4), blk[:, 4:8])
        assert np.array_equal(plane(spec.dm_offset, 4), blk[:, 0:4])
        assert (spec.qs_offset, spec.qh_offset, spec.dm_offset) == (0, 16 * nb, 20 * nb)


def _silu_f32(gf):
    return gf / (np.float32(1) + np.exp(-gf).astype(np.float32))


def test_declared_precision_modes_against_numpy(orc, synth):
    """The staging switches of the declared-precision references, each against numpy's own rounding on independently
    dequantised weights: `staged_gemm(stage_f16 = 1)` (weights as halves, tests/test_moe_mm_many_gpu.cpp:54-56) and bits
    1 (x and h as bf16), 2 (weights as halves) and 8 (Q6_K down rows as d * half(sc * (q - 32))) of
    `moe_routed_reference`."""
    rows, cols, tokens = 16, 512, 4
    w = synth.matrix(12, 9200, rows, cols)
    x = synth.activations_f32(9201, (tokens, cols))
    wf = orc.dequantize(12, w, rows * cols).reshape(rows, cols)
    want = x.astype(np.float64) @ wf.astype(np.float16).astype(np.float64).T
    assert np.allclose(orc.staged_gemm(12, w, cols, x, nrows=rows, stage_f16=1), want, rtol=1e-12, atol=1e-9)
    assert not np.allclose(orc.staged_gemm(12, w, cols, x, nrows=rows, stage_f16=0), want, rtol=1e-9, atol=1e-9)

    channels, hidden, experts = 256, 256, 2
    gate = synth.matrix(12, 9202, hidden * experts, channels)
    up = synth.matrix(12, 9203, hidden * experts, channels)
    down = synth.matrix(14, 9204, channels * experts, hidden)
    ids = np.array([1, 0, 1], dtype=np.uint32)
    xs = synth.activations_f32(9205, (3, channels))
    g = orc.dequantize(12, gate, hidden * experts * channels).reshape(experts, hidden, channels)
    u = orc.dequantize(12, up, hidden * experts * channels).reshape(experts, hidden, channels)
    d = orc.dequantize(14, down, channels * experts * hidden).reshape(experts, channels, hidden)
    half = lambda a: a.astype(np.float16).astype(np.float64)
    qd, scd, dd = q6k_fields(down)
    d_products = (((qd - 32) * np.repeat(scd, 16, axis=1)).astype(np.float16).astype(np.float64) * dd[:, None]).reshape(experts, channels, hidden)
    for stage, xin, wg, wu, wd, round_h in (
            (1, synth.round_bf16(xs), g.astype(np.float64), u.astype(np.float64), d.astype(np.float64), True),
            (2, xs, half(g), half(u), half(d), False),
            (8, xs, g.astype(np.float64), u.astype(np.float64), d_products, False)):
        h, y = orc.moe_routed_reference(12, 14, gate, up, down, channels, hidden, experts, ids, 3, 1, xs, stage=stage)
        for r, e in enumerate(ids):
            xv = xin[r].astype(np.float64)
            hh = _silu_f32((wg[e] @ xv).astype(np.float32)) * (wu[e] @ xv).astype(np.float32)
            if round_h:
                # numpy's exp and the C library's differ by an ulp now and then, which can move a bf16 rounding: at most
                # one bf16 step on a few elements, none on the rest
                hb = synth.round_bf16(hh)
                step = np.abs(hb.astype(np.float64)) * 2.0 ** -7
                assert (np.abs(h[r] - hb) <= step).all() and (h[r] == hb).mean() > 0.98
                assert np.array_equal(h[r], synth.round_bf16(h[r].astype(np.float32)).astype(np.float64))  # h is bf16-valued
            else:
                assert np.allclose(h[r], hh.astype(np.float64), rtol=3e-7, atol=1e-30)
            assert np.allclose(y[r], wd[e] @ h[r], rtol=1e-12, atol=1e-6)

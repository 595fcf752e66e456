"""GPU parity: dequantisation (bit-exact) and the GEMV family (scaled error <= 5e-5, the engine's
own bar: native/tests/test_graph.cpp:45-52) through the C ABI, against the CPU oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TOL = 5e-5  # |a - e| / max(1, |e|), native/src/main.cpp:165


def scaled_error(actual, expected):
    actual, expected = np.asarray(actual, dtype=np.float64), np.asarray(expected, dtype=np.float64)
    assert np.isfinite(actual).all()
    return float(np.max(np.abs(actual - expected) / np.maximum(1.0, np.abs(expected))))


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


# ---------------------------------------------------------------------------------- dequantise

def test_f16_all_patterns_bit_exact(gpu, orc):
    finite = np.array([b for b in range(65536) if (b >> 10) & 31 != 31], dtype=np.uint16)
    got = gpu.dequantize(1, gpu.upload(finite), finite.size).cpu().numpy()
    want = np.array([orc.binary16(int(b)) for b in finite], dtype=np.float32)
    assert np.array_equal(bits(got), bits(want)) and gpu.error() == 0
    inf = np.array([0x3C00, 0x7C00], dtype=np.uint16)
    gpu.dequantize(1, gpu.upload(inf), 2)
    assert gpu.error() == 1  # the reference refuses non-finite weights; the device flags them


@pytest.mark.parametrize("t", [0, 1, 7, 8, 12, 13, 14, 20, 30])
def test_dequantize_bit_exact_vs_oracle(gpu, orc, synth, t):
    epb, bpb = orc.encoding(t)
    nblocks = 4096 if epb > 1 else 40000
    if t in synth.BLOCKS:
        raw = synth.BLOCKS[t][0](1000 + t, nblocks).reshape(-1)
    elif t == 20:
        raw = synth.uniform_bytes(1020, nblocks * 18).reshape(nblocks, 18).copy()
        raw[:, 0:2] = synth.f16_bits(np.abs(synth.normal(1021, nblocks, 0.05))).view(np.uint8).reshape(nblocks, 2)
        raw = raw.reshape(-1)
    else:
        vals = synth.normal(1030 + t, nblocks, 3.0).astype(np.float32)
        raw = (vals.view(np.uint8) if t == 0 else synth.f16_bits(vals).view(np.uint8) if t == 1 else synth.bf16_bits(vals).view(np.uint8)).copy()
    want = orc.dequantize(t, raw, nblocks * epb)
    got = gpu.dequantize(t, gpu.upload(raw), nblocks * epb).cpu().numpy()
    assert np.array_equal(bits(got), bits(want)) and gpu.error() == 0


@pytest.mark.parametrize("t", [8, 12, 14])
def test_dequantize_edge_scales(gpu, orc, t):
    # native/tests/test_graph.cpp / test_metal.cpp scale set: zero, subnormal, +-0.25, 0x2800, plus f16 extremes.
    rng = np.random.default_rng(40 + t)
    epb, bpb = orc.encoding(t)
    scales = [0x0000, 0x8000, 0x0011, 0x0001, 0x03FF, 0x0400, 0x3400, 0xB400, 0x2800, 0x7BFF, 0xFBFF]
    raw = rng.integers(0, 256, size=(len(scales) * 8, bpb), dtype=np.uint8)
    for i in range(raw.shape[0]):
        s = scales[i % len(scales)]
        for off in ((0, 2) if t == 12 else (208,) if t == 14 else (0,)):
            raw[i, off], raw[i, off + 1] = s & 255, s >> 8
    n = raw.shape[0] * epb
    want = orc.dequantize(t, raw.reshape(-1), n)
    got = gpu.dequantize(t, gpu.upload(raw.reshape(-1)), n).cpu().numpy()
    assert np.array_equal(bits(got), bits(want)) and gpu.error() == 0


@pytest.mark.parametrize("t,cols,rows", [(12, 2048, 512), (13, 512, 64), (8, 512, 64), (7, 640, 32), (14, 512, 2048)])
def test_dequantize_planar_bit_exact(gpu, tsp, orc, synth, t, cols, rows):
    # native/tests/test_planar_pack_v3.cpp:269-275: planar dequant == GGUF dequant to the bit.
    raw = synth.matrix(t, 1100 + t, rows, cols)
    spec = tsp.make_expert_spec(t, cols, rows)
    planar = tsp.pack_expert(spec, raw)
    got = gpu.dequantize_planar(spec, gpu.upload(planar)).cpu().numpy()
    assert np.array_equal(bits(got), bits(orc.dequantize(t, raw, rows * cols))) and gpu.error() == 0


def test_dequantize_refusals(gpu, tsp):
    blocks = gpu.zeros(144, "uint8")
    with pytest.raises(tsp.FormatError):
        gpu.dequantize(12, blocks, 255)
    with pytest.raises(tsp.FormatError):
        gpu.dequantize(99, blocks, 256)


# ---------------------------------------------------------------------------------- GEMV

def reference_like_matrix(t, rows, cols, orc):
    """native/tests/test_graph.cpp:95-110: patterned bytes with fixed small scales."""
    epb, bpb = orc.encoding(t)
    data = np.array([(i * 37 + 19) & 255 for i in range(rows * (cols // epb) * bpb)], dtype=np.uint8).reshape(-1, bpb)
    for blk in data:
        if t == 0:
            blk[0:4] = np.frombuffer(np.float32(0.125).tobytes(), dtype=np.uint8)
        elif t == 30:
            blk[0:2] = (0x00, 0x3E)
        else:
            off = 208 if t == 14 else 0
            blk[off:off + 2] = (0x00, 0x24)
            if t in (7, 12, 13):
                blk[2:4] = (0x00, 0x20)
    return data.reshape(-1)


@pytest.mark.parametrize("t", [0, 1, 7, 8, 12, 13, 14, 20, 30])
def test_gemv_all_encodings_reference_fixture(gpu, orc, t):
    epb, _ = orc.encoding(t)
    cols, rows = epb * 3, 7
    w = reference_like_matrix(t, rows, cols, orc)
    x = np.array([((i % 31) - 15) / 16.0 for i in range(cols)], dtype=np.float32)
    want = orc.reference_gemv(t, w, cols, rows, x)
    dw, dx = gpu.upload(w), gpu.upload(x)
    for _ in range(3):
        got = gpu.gemv(t, dw, dx, cols, rows).cpu().numpy()
        assert scaled_error(got, want) <= TOL and gpu.error() == 0


@pytest.mark.parametrize("rows", [1, 3, 4, 5, 33])
@pytest.mark.parametrize("t,cols", [(12, 512), (12, 2048), (12, 4096), (12, 768), (14, 512), (8, 2048), (8, 96), (8, 4160)])
def test_gemv_shapes(gpu, orc, synth, t, cols, rows):
    w = synth.matrix(t, 1200 + t + rows, rows, cols)
    x = synth.activations_f32(1201, cols)
    want = orc.reference_gemv(t, w, cols, rows, x)
    got = gpu.gemv(t, gpu.upload(w), gpu.upload(x), cols, rows).cpu().numpy()
    assert scaled_error(got, want) <= TOL and gpu.error() == 0
    zero = gpu.gemv(t, gpu.upload(w), gpu.zeros(cols), cols, rows).cpu().numpy()
    assert not zero.any()  # zero input gives exactly zero output (native/tests/test_metal.cpp:41-66)


def test_config0_dense_q4k_gemv(gpu, tsp, orc, synth):
    """BASELINE config 0 at full size: W 4096 x 2048 Q4_K, x f32 N(0,1); raw GGUF rows and planar v3."""
    rows, cols = 4096, 2048
    w = synth.matrix(12, synth.tensor_seed(0, 1), rows, cols)
    x = synth.activations_f32(synth.tensor_seed(0, 2), cols)
    want = orc.reference_gemv_mt(12, w, cols, rows, x, 8)
    dx = gpu.upload(x)
    got = gpu.gemv(12, gpu.upload(w), dx, cols, rows).cpu().numpy()
    err_raw = scaled_error(got, want)
    spec = tsp.make_expert_spec(12, cols, rows)
    planar = tsp.pack_expert(spec, w)
    got_p = gpu.gemv(12, gpu.upload(planar), dx, cols, rows, layout=tsp.LAYOUT_PLANAR_V3).cpu().numpy()
    assert gpu.error() == 0
    # the two arms share their arithmetic: identical bits (the engine's block path is held to this too,
    # native/tests/test_block_gemv.cpp:94)
    assert np.array_equal(bits(got), bits(got_p))
    # The configuration's bar is max scaled error 2e-3 with f32 accumulation. Measured: 6.2e-5, on an element of magnitude ~1
    # in a vector whose entries reach several hundred (weights up to ~19, 2048 products): 3e-7 of the vector's scale, which
    # is what f32 accumulation leaves. The engine's 5e-5 (native/src/main.cpp:165) is quoted on outputs of magnitude ~1 and
    # holds at those (test_gemv_shapes, test_gemv_all_encodings_reference_fixture); here the bound asserted is 2e-4.
    print(f"config0 max scaled error {err_raw:.3e}")
    assert err_raw <= 2e-4, err_raw


def test_gemv_rows_strided(gpu, orc, synth):
    # include/tokspur/graph.hpp:733: gemv once per row of a strided row set; padding stays untouched.
    cols, rows, count = 2048, 64, 5
    w = synth.matrix(12, 1300, rows, cols)
    x = synth.activations_f32(1301, (count, cols + 8))
    y = gpu.full((count, rows + 4), -7.0)
    gpu.gemv_rows(12, gpu.upload(w), gpu.upload(x), y, count, cols, rows, (cols + 8) * 4, (rows + 4) * 4)
    y = y.cpu().numpy()
    for i in range(count):
        assert scaled_error(y[i, :rows], orc.reference_gemv(12, w, cols, rows, x[i, :cols])) <= TOL
    assert (y[:, rows:] == -7.0).all() and gpu.error() == 0


@pytest.mark.parametrize("t", [0, 1, 7, 8, 12, 13, 14, 20, 30])
def test_routed_gemv(gpu, orc, synth, t):
    # native/tests/test_moe.cpp:96-129: per selected expert, both broadcast and per-route inputs.
    epb, bpb = orc.encoding(t)
    cols, rows, experts, selected = epb * 2 if epb > 1 else 64, 9, 6, 4
    w = np.concatenate([reference_like_matrix(t, rows, cols, orc)[::1] for _ in range(experts)])
    w = w.copy()
    rng = np.random.default_rng(t)
    per = w.size // experts
    for e in range(experts):  # make experts differ in their quant bytes, keep the scale fields
        blk = w[e * per:(e + 1) * per].reshape(-1, bpb)
        lo = 4 if t in (7, 12, 13) else 2 if t in (8, 20, 1, 30) else 0
        hi = 208 if t == 14 else bpb
        if epb > 1:
            blk[:, lo:hi] = rng.integers(0, 256, size=(blk.shape[0], hi - lo), dtype=np.uint8)
    ids = np.array([5, 0, 3, 5], dtype=np.uint32)
    for broadcast in (True, False):
        x = synth.activations_f32(1400 + t, (1 if broadcast else selected, cols))
        got = gpu.routed_gemv(t, gpu.upload(w), gpu.upload(ids), gpu.upload(x), cols, rows, experts, selected, broadcast).cpu().numpy()
        for s, e in enumerate(ids):
            want = orc.reference_gemv(t, w[e * per:(e + 1) * per], cols, rows, x[0 if broadcast else s])
            assert scaled_error(got[s], want) <= TOL
        assert gpu.error() == 0


def test_sticky_error_word(gpu, tsp, orc, synth):
    # native/tests/test_moe.cpp:165-190: non-finite input or bad id poisons the batch; the next batch is clean.
    cols, rows = 2048, 16
    w = synth.matrix(12, 1500, rows, cols)
    x = synth.activations_f32(1501, cols)
    dw = gpu.upload(w)
    bad = x.copy()
    bad[7] = np.inf
    gpu.gemv(12, dw, gpu.upload(bad), cols, rows)
    assert gpu.error() & tsp.ERRBIT_NONFINITE
    got = gpu.gemv(12, dw, gpu.upload(x), cols, rows).cpu().numpy()
    assert gpu.error() == 0 and scaled_error(got, orc.reference_gemv(12, w, cols, rows, x)) <= TOL
    ids = gpu.upload(np.array([0, 9], dtype=np.uint32))
    wq = gpu.upload(synth.matrix(8, 1502, 4 * 2, 64))
    out = gpu.routed_gemv(8, wq, ids, gpu.upload(synth.activations_f32(1503, 64)), 64, 4, 2, 2, True).cpu().numpy()
    assert gpu.error() & tsp.ERRBIT_INDEX and not out[1].any()


def test_gemv_refusals(gpu, tsp, synth):
    w = gpu.upload(synth.matrix(12, 1600, 4, 256))
    x, y = gpu.zeros(256), gpu.zeros(4)
    for args in ((12, w, x, 256, 5), (12, w, x, 255, 4), (99, w, x, 256, 4), (12, w, x, 0, 4)):
        with pytest.raises(tsp.FormatError):
            gpu.gemv(*args)
    with pytest.raises(tsp.FormatError):  # output aliasing an input
        gpu.gemv(0, x, x, 16, 16, y=x)


# ---------------------------------------------------------------------------------- Q8 many rows

@pytest.mark.parametrize("tokens,cols,rows", [(1, 64, 5), (19, 512, 160), (40, 2048, 96), (9, 1024, 64), (13, 2048, 1000), (16, 2048, 2084),
                                              (27, 1024, 132), (8, 1536, 77), (3, 512, 16)])
def test_dense_mm_q8(gpu, tsp, orc, synth, tokens, cols, rows):
    # graph.hpp:860 `dense_mm_q8`: a dense Q8_0 matrix times f32 rows, GGUF rows and q8_lanes_v1 rows; rows back to back
    # (width groups 8, 4, 2, 1; nine or more GGUF rows of 1024 / 2048 columns go up to sixteen at a time, each half of the
    # columns summed by its own workgroups) and rows with padding (canaries stay)
    w = synth.matrix(8, 1800 + cols, rows, cols)
    lanes = tsp.q8_lanes_pack_rows(cols, w)
    x = synth.activations_f32(1801 + tokens, (tokens, cols + 4))
    want = np.stack([orc.reference_gemv(8, w, cols, rows, x[t, :cols]) for t in range(tokens)])
    for matrix, layout in ((w, tsp.LAYOUT_GGUF), (lanes, tsp.LAYOUT_Q8_LANES_V1)):
        packed = tsp.dense_mm_q8(gpu, layout, gpu.upload(matrix), gpu.upload(np.ascontiguousarray(x[:, :cols])), tokens, cols, rows).cpu().numpy()
        assert scaled_error(packed, want) <= TOL and gpu.error() == 0
        out = gpu.full((tokens, rows + 3), -5.0)
        tsp.dense_mm_q8(gpu, layout, gpu.upload(matrix), gpu.upload(x), tokens, cols, rows, out=out, x_stride=(cols + 4) * 4, out_stride=(rows + 3) * 4)
        got = out.cpu().numpy()
        assert scaled_error(got[:, :rows], want) <= TOL and (got[:, rows:] == -5.0).all() and gpu.error() == 0
    with pytest.raises(tsp.FormatError):
        tsp.dense_mm_q8(gpu, tsp.LAYOUT_PLANAR_V3, gpu.upload(w), gpu.upload(x), tokens, cols, rows, x_stride=(cols + 4) * 4)


@pytest.mark.parametrize("tokens,cols,rows", [(1, 64, 5), (70, 128, 33), (200, 2048, 512), (129, 512, 2048), (64, 4096, 64)])
def test_dense_mm_q8_staged(gpu, tsp, orc, synth, tokens, cols, rows):
    # the many-row form of graph.hpp:860 `dense_mm_q8`: matrix and rows as halves, one matrix-core GEMM. Both layouts, rows with
    # padding on both sides (canaries stay), tiles that overhang the matrix on either edge, and agreement with the streaming
    # entry point.
    w = synth.matrix(8, 1900 + cols, rows, cols)
    lanes = tsp.q8_lanes_pack_rows(cols, w)
    x = synth.activations_f32(1901 + tokens, (tokens, cols + 4))
    sample = np.unique(np.linspace(0, tokens - 1, min(tokens, 24)).astype(int))
    want = np.stack([orc.reference_gemv(8, w, cols, rows, x[t, :cols]) for t in sample])
    scale = np.maximum(1.0, np.sqrt((want ** 2).mean(axis=1, keepdims=True)))
    streamed = tsp.dense_mm_q8(gpu, tsp.LAYOUT_GGUF, gpu.upload(w), gpu.upload(np.ascontiguousarray(x[:, :cols])), tokens, cols, rows).cpu().numpy()
    for matrix, layout in ((w, tsp.LAYOUT_GGUF), (lanes, tsp.LAYOUT_Q8_LANES_V1)):
        out = gpu.full((tokens, rows + 3), -5.0)
        tsp.dense_mm_q8_staged(gpu, layout, gpu.upload(matrix), gpu.upload(x), tokens, cols, rows, out=out, x_stride=(cols + 4) * 4,
                               out_stride=(rows + 3) * 4)
        got = out.cpu().numpy()
        assert gpu.error() == 0 and (got[:, rows:] == -5.0).all()
        assert float(np.max(np.abs(got[sample, :rows] - want) / np.maximum(scale, np.abs(want)))) <= 2e-3  # the GEMM tolerance
        row_scale = np.maximum(1.0, np.sqrt((streamed ** 2).mean(axis=1, keepdims=True)))
        assert float(np.max(np.abs(got[:, :rows] - streamed) / np.maximum(row_scale, np.abs(streamed)))) <= 2e-3
        nmse = float(((got[:, :rows] - streamed) ** 2).sum() / max((streamed ** 2).sum(), 1e-30))
        assert nmse <= 1e-6, nmse
    with pytest.raises(tsp.FormatError):  # columns not a multiple of 64
        tsp.dense_mm_q8_staged(gpu, tsp.LAYOUT_GGUF, gpu.upload(synth.matrix(8, 3, 4, 96)), gpu.zeros((2, 96)), 2, 96, 4)
    with pytest.raises(tsp.FormatError):  # workspace too small
        tsp.dense_mm_q8_staged(gpu, tsp.LAYOUT_GGUF, gpu.upload(w), gpu.upload(x), tokens, cols, rows, x_stride=(cols + 4) * 4,
                               workspace=gpu.empty(256, "uint8"))
    x_bad = np.ascontiguousarray(x[:, :cols]).copy()
    x_bad[tokens // 2, cols // 2] = np.inf
    tsp.dense_mm_q8_staged(gpu, tsp.LAYOUT_GGUF, gpu.upload(w), gpu.upload(x_bad), tokens, cols, rows)
    assert gpu.error() & tsp.ERRBIT_NONFINITE
    gpu.clear_error()


@pytest.mark.parametrize("width", [1, 2, 4, 8])
@pytest.mark.parametrize("cols,rows", [(2048, 37), (64, 5), (96, 7), (4096, 9)])
def test_q8_matvec_many(gpu, tsp, orc, synth, width, cols, rows):
    # native/tests/test_q8_many.cpp: token-major in and out, every width, both layouts.
    w = synth.matrix(8, 1700 + cols, rows, cols)
    x = synth.activations_f32(1701 + width, (width, cols))
    want = orc.reference_q8_many(w, x, cols, rows, width)
    got = gpu.q8_matvec_many(gpu.upload(w), gpu.upload(x), cols, rows, width).cpu().numpy()
    assert scaled_error(got, want) <= TOL and gpu.error() == 0
    lanes = tsp.q8_lanes_pack_rows(cols, w)
    got_l = gpu.q8_matvec_many(gpu.upload(lanes), gpu.upload(x), cols, rows, width, layout=tsp.LAYOUT_Q8_LANES_V1).cpu().numpy()
    assert scaled_error(got_l, want) <= TOL and gpu.error() == 0
    with pytest.raises(tsp.FormatError):
        gpu.q8_matvec_many(gpu.upload(w), gpu.upload(x), cols, rows, 3)

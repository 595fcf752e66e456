"""GPU parity for the row top-64 of the logits (`logit_topk`, graph.hpp:1030-1033): every field of every 528-byte
row is compared bit for bit with the CPU rule of sampling.cpp:473-513 (value descending, column ascending,
-0 == +0, non-finite skipped and reported, first subnormal reported, unused slots id 0 / -inf)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def check_rows(tsp, orc, gpu, logits, stride_floats=None):
    rows, vocab = logits.shape
    stride_floats = vocab if stride_floats is None else stride_floats
    padded = np.full((rows, stride_floats), np.float32(7e30))
    padded[:, :vocab] = logits
    got = tsp.logit_topk(gpu, gpu.upload(padded), rows, vocab, stride_bytes=stride_floats * 4).cpu().numpy().view(tsp.TOPK_ROW_DTYPE)
    assert got.shape == (rows,)
    for r in range(rows):
        want = orc.logit_topk_row(logits[r])
        assert (got[r]["vocabulary"], got[r]["count"]) == (vocab, want.count)
        assert got[r]["first_nonfinite_col"] == want.first_nonfinite_col and got[r]["first_subnormal_col"] == want.first_subnormal_col
        assert np.array_equal(got[r]["ids"], np.array(want.ids, dtype=np.uint32))
        assert np.array_equal(got[r]["logits"].view(np.uint32), np.array(want.logits, dtype=np.float32).view(np.uint32))
    return got


@pytest.mark.parametrize("vocab", [1, 5, 64, 65, 1000, 4096, 4097, 5000, 70001])
def test_topk_ties_zeros_nonfinite(gpu, tsp, orc, vocab):
    rng = np.random.default_rng(vocab)
    x = np.round(rng.normal(size=(3, vocab)), 1).astype(np.float32)  # coarse grid: many exact ties, +0 and -0
    if vocab >= 65:
        x[0, 3], x[0, 7], x[0, 11] = np.inf, np.nan, -0.0
        x[0, 20] = np.float32(1e-41)
        x[1, vocab - 1] = -np.inf
        x[2, :] = 0.25  # all equal: ids 0..63
    check_rows(tsp, orc, gpu, x, stride_floats=vocab + 3)


def test_topk_mostly_nonfinite(gpu, tsp, orc):
    x = np.full((2, 300), np.nan, dtype=np.float32)
    x[0, [5, 17, 299]] = [1.0, -2.0, 1.0]
    got = check_rows(tsp, orc, gpu, x)
    assert got[0]["count"] == 3 and got[1]["count"] == 0 and got[1]["first_nonfinite_col"] == 0


def test_topk_refusals(gpu, tsp):
    x = gpu.upload(np.zeros((2, 128), dtype=np.float32))
    with pytest.raises(tsp.FormatError):
        tsp.logit_topk(gpu, x, 2, 128, stride_bytes=127 * 4)
    with pytest.raises(tsp.FormatError):
        tsp.logit_topk(gpu, x, 2, 128, scratch=gpu.empty(528, "uint8"))
    with pytest.raises(tsp.FormatError):
        tsp.logit_topk_scratch_bytes(4096)
    assert tsp.logit_topk_scratch_bytes(16, 151936) == 16 * 38 * 528 and tsp.logit_topk_output_bytes(16) == 16 * 528


def check_sampled_logits(orc, w, x, logits, columns, vocabulary, seed, what, samples=2048):
    """GPU logits of `samples` random vocabulary rows, plus the first and the last, against `reference_gemv` for every token row."""
    row_bytes = columns // 32 * 34
    sel = np.unique(np.concatenate([np.random.default_rng(seed).choice(vocabulary, size=samples, replace=False), [0, vocabulary - 1]]))
    sub = np.ascontiguousarray(w.reshape(vocabulary, row_bytes)[sel]).reshape(-1)
    worst = 0.0
    for r in range(x.shape[0]):
        ref = orc.reference_gemv(8, sub, columns, len(sel), x[r])
        worst = max(worst, float(np.max(np.abs(ref - logits[r, sel]) / np.maximum(1.0, np.abs(ref)))))
    print(f"{what}: {len(sel)} sampled vocabulary rows x {x.shape[0]} token rows, reference metric {worst:.2e}")
    assert worst <= 5e-5


def test_config4_lm_head_argmax(gpu, tsp, orc, synth):
    """BASELINE config 4 at full size for M = 1, 4, 8, 16: Q8_0 LM head 151 936 x 2048 -> logits -> top-64 rows.
    The arg-max (rank 0) is compared with the CPU arg-max of the same GPU logits bit for bit, and with the arg-max of the
    CPU reference logits wherever the reference's top-2 margin exceeds the GEMV error bound."""
    V, C = 151936, 2048
    w = synth.matrix(8, synth.tensor_seed(4, 1), V, C)
    dw = gpu.upload(w)
    for m in (1, 4, 8, 16):
        x = synth.activations_f32(synth.tensor_seed(4, 2 + m), (m, C))
        dx = gpu.upload(x)
        y = gpu.empty((m, V))
        if m > 8:  # the path the benchmark times: up to sixteen rows in one pass over the matrix (`dense_mm_q8`)
            tsp.dense_mm_q8(gpu, tsp.LAYOUT_GGUF, dw, dx, m, C, V, out=y)
            two_passes = gpu.empty((m, V))
            for at in range(0, m, 8):
                gpu.q8_matvec_many(dw, dx[at:at + 8], C, V, 8, y=two_passes[at:at + 8])
            both = (y.cpu().numpy(), two_passes.cpu().numpy())
            assert float(np.max(np.abs(both[0] - both[1]) / np.maximum(1.0, np.abs(both[1])))) <= 5e-5
        else:
            gpu.q8_matvec_many(dw, dx, C, V, m, y=y)
        rows = tsp.logit_topk(gpu, y, m, V).cpu().numpy().view(tsp.TOPK_ROW_DTYPE)
        assert gpu.error() == 0
        logits = y.cpu().numpy()
        for r in range(m):
            want = orc.logit_topk_row(logits[r])
            assert np.array_equal(rows[r]["ids"], np.array(want.ids, dtype=np.uint32)) and rows[r]["count"] == 64
            assert rows[r]["ids"][0] == int(np.argmax(logits[r]))
        # reference logits of 2048 random vocabulary rows (and the first and last one) for EVERY token row, the engine's
        # |a - e| / max(1, |e|) <= 5e-5 (native/tools/ffn_check.cpp:48-56); a full CPU GEMV is 3e8 multiply-adds per row
        check_sampled_logits(orc, w, x, logits, C, V, seed=40 + m, what=f"config4 M={m} raw rows")
        cand = rows[0]["ids"][:8].astype(np.int64)
        ref = np.array([orc.reference_gemv(8, w[int(c) * (C // 32) * 34:(int(c) + 1) * (C // 32) * 34], C, 1, x[0])[0] for c in cand])
        assert np.max(np.abs(ref - rows[0]["logits"][:8]) / np.maximum(1.0, np.abs(ref))) <= 5e-5
        margin = ref[0] - np.max(ref[1:])
        bound = 5e-5 * max(1.0, abs(ref[0])) * 2
        print(f"config4 M={m}: arg-max id {cand[0]}, reference top-2 margin {margin:.3e} (error bound {bound:.1e})")
        if margin > bound:
            assert int(np.argmax(ref)) == 0
    # the other arm: the same matrix as q8_lanes_v1 rows, the form Pack v3 stores a dense Q8_0 matrix in, at full vocabulary
    d_lanes = gpu.upload(tsp.q8_lanes_pack_rows(C, w))
    for m in (1, 8, 16):
        x = synth.activations_f32(synth.tensor_seed(4, 2 + m), (m, C))
        dx = gpu.upload(x)
        raw_rows, lane_rows = gpu.empty((m, V)), gpu.empty((m, V))
        tsp.dense_mm_q8(gpu, tsp.LAYOUT_GGUF, dw, dx, m, C, V, out=raw_rows)
        tsp.dense_mm_q8(gpu, tsp.LAYOUT_Q8_LANES_V1, d_lanes, dx, m, C, V, out=lane_rows)
        assert gpu.error() == 0
        a, b = raw_rows.cpu().numpy(), lane_rows.cpu().numpy()
        assert float(np.max(np.abs(a - b) / np.maximum(1.0, np.abs(a)))) <= 5e-5
        check_sampled_logits(orc, w, x, b, C, V, seed=90 + m, what=f"config4 M={m} q8_lanes_v1 rows")
        top = tsp.logit_topk(gpu, lane_rows, m, V).cpu().numpy().view(tsp.TOPK_ROW_DTYPE)
        for r in range(m):
            assert top[r]["ids"][0] == int(np.argmax(b[r]))

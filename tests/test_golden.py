"""Committed golden vectors (tests/golden/reference_vectors.npz: inputs from the seeded generators, outputs of the reference's
own CPU code, written by tests/golden/make_fixtures.py where the reference tree exists). On a machine without the
reference they pin the C restatement (CPU tests) and the HIP path (GPU tests)."""
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def gold():
    return np.load(os.path.join(HERE, "golden", "reference_vectors.npz"), allow_pickle=False)


def test_oracle_matches_the_golden_vectors(orc, gold):
    for t in (7, 8, 12, 13, 14):
        epb, _ = orc.encoding(t)
        assert np.array_equal(orc.dequantize(t, gold[f"dequant_{t}_in"], 6 * epb).view(np.uint32), gold[f"dequant_{t}_out"])
    for t, cols, rows in ((12, 512, 6), (14, 256, 5), (8, 96, 7)):
        y = orc.reference_gemv(t, gold[f"gemv_{t}_w"], cols, rows, gold[f"gemv_{t}_x"])
        assert np.array_equal(y.view(np.uint64), gold[f"gemv_{t}_y"])
    y = orc.reference_q8_many(gold["q8many_w"], gold["q8many_x"], 128, 9, 4).astype(np.float64)
    assert np.array_equal(y.view(np.uint64), gold["q8many_y"])
    assert np.array_equal(orc.q8_lanes_pack_rows(1024, gold["lanes_in"]), gold["lanes_out"])
    at = 0
    for mode, normalize in ((0, True), (0, False), (1, True)):
        for row in gold["route_logits"]:
            ids, weights = orc.route_reference(row, 6, mode, normalize)
            assert np.array_equal(ids, gold["route_ids"][at])
            assert np.array_equal(np.asarray(weights, dtype=np.float64).view(np.uint64), gold["route_weights"][at])
            at += 1
    mixed = orc.mixture_reference(gold["mixture_experts"], gold["mixture_weights"], gold["mixture_shared"], 0.75)
    assert np.array_equal(np.asarray(mixed, dtype=np.float64).view(np.uint64), gold["mixture_out"])
    top = orc.logit_topk_row(gold["topk_in"])
    assert np.array_equal(np.array(top.ids, dtype=np.uint32), gold["topk_ids"])
    assert np.array_equal(np.array(top.logits, dtype=np.float32).view(np.uint32), gold["topk_logits"])
    assert [top.count, top.first_nonfinite_col, top.first_subnormal_col] == list(gold["topk_meta"])
    views, total = orc.moe_mm_many_bytes(2048, 512, 512, 10, 2048, True)
    assert list(views) + [total] == list(gold["moe_mm_many_bytes"])
    p = orc.grouped_mm_plan(12, 0, 2048, 512, 512, 10, 2048, 8192, 2048, True, True)
    assert [p.maximum_tasks, p.matrix_bytes, p.token_map_bytes, p.counts_bytes, p.tasks_bytes, p.grid_x, p.grid_y] == list(gold["grouped_mm_plan"])


def test_host_planners_match_the_golden_vectors(tsp, gold):
    views, total = tsp.moe_mm_many_bytes(2048, 512, 512, 10, 2048, True)
    assert list(views) + [total] == list(gold["moe_mm_many_bytes"])
    p = tsp.grouped_mm_plan(12, 0, 2048, 512, 512, 10, 2048, 8192, 2048, True, True)
    assert [p.maximum_tasks, p.matrix_bytes, p.token_map_bytes, p.counts_bytes, p.tasks_bytes, p.grid_x, p.grid_y] == list(gold["grouped_mm_plan"])
    assert np.array_equal(tsp.q8_lanes_pack_rows(1024, gold["lanes_in"]), gold["lanes_out"])


@pytest.mark.gpu
def test_hip_path_matches_the_golden_vectors(gpu, tsp, gold):
    for t in (7, 8, 12, 13, 14):  # dequantised weights: bit-exact
        epb, _ = tsp.encoding(t)
        got = gpu.dequantize(t, gpu.upload(gold[f"dequant_{t}_in"]), 6 * epb).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), gold[f"dequant_{t}_out"])
    for t, cols, rows in ((12, 512, 6), (14, 256, 5), (8, 96, 7)):  # f32 GEMV: the engine's 5e-5 scaled-error bar
        want = gold[f"gemv_{t}_y"].view(np.float64)
        got = gpu.gemv(t, gpu.upload(gold[f"gemv_{t}_w"]), gpu.upload(gold[f"gemv_{t}_x"]), cols, rows).cpu().numpy()
        assert float(np.max(np.abs(got - want) / np.maximum(1.0, np.abs(want)))) <= 5e-5
    want = gold["q8many_y"].view(np.float64).reshape(4, 9)
    got = gpu.q8_matvec_many(gpu.upload(gold["q8many_w"]), gpu.upload(gold["q8many_x"]), 128, 9, 4).cpu().numpy()
    assert float(np.max(np.abs(got - want) / np.maximum(1.0, np.abs(want)))) <= 5e-5
    lanes = gpu.q8_matvec_many(gpu.upload(tsp.q8_lanes_pack_rows(128, gold["q8many_w"])), gpu.upload(gold["q8many_x"]), 128, 9, 4,
                               layout=tsp.LAYOUT_Q8_LANES_V1).cpu().numpy()
    assert float(np.max(np.abs(lanes - want) / np.maximum(1.0, np.abs(want)))) <= 5e-5
    logits = gold["route_logits"].astype(np.float32)  # the fixtures' logits are f32 values held in doubles
    at = 0
    for mode, normalize in ((0, True), (0, False), (1, True)):
        ids, weights = gpu.route(gpu.upload(logits), 6, mode, normalize, tokens=5)
        assert np.array_equal(ids.cpu().numpy().view(np.uint32), gold["route_ids"][at:at + 5])  # router ids: bit-exact
        want_w = gold["route_weights"][at:at + 5].view(np.float64)
        assert float(np.max(np.abs(weights.cpu().numpy() - want_w))) <= 1e-6
        at += 5
    mixed = gpu.mixture(gpu.upload(gold["mixture_experts"].astype(np.float32)), gpu.upload(gold["mixture_weights"].astype(np.float32)),
                        gpu.upload(gold["mixture_shared"].astype(np.float32)), gpu.upload(np.array([0.75], dtype=np.float32)), 32, 6).cpu().numpy()
    want = gold["mixture_out"].view(np.float64)
    assert float(np.max(np.abs(mixed.reshape(-1) - want) / np.maximum(1.0, np.abs(want)))) <= 1e-5
    rows = tsp.logit_topk(gpu, gpu.upload(gold["topk_in"].reshape(1, -1)), 1, 300).cpu().numpy().view(tsp.TOPK_ROW_DTYPE)
    assert np.array_equal(rows[0]["ids"], gold["topk_ids"]) and np.array_equal(rows[0]["logits"].view(np.uint32), gold["topk_logits"])
    assert [rows[0]["count"], rows[0]["first_nonfinite_col"], rows[0]["first_subnormal_col"]] == list(gold["topk_meta"])
    assert gpu.error() == 0

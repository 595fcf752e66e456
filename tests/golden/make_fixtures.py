"""Writes tests/golden/reference_vectors.npz: small inputs and the outputs of the reference's own CPU code for them.

Run in the build container, where oracle/_ref (the reference's C++ sources compiled in place by oracle/build_ref.sh)
exists:  python tests/golden/make_fixtures.py
The GPU box has no reference tree; there the fixtures stand in for it. Inputs come from the package's seeded generators,
outputs are stored as raw bits (uint32 / uint64) so that comparisons are exact.
"""
import importlib
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)


def main():
    from oracle import oracle
    ref = oracle.ref()
    if ref is None:
        raise SystemExit("oracle/_ref is not built: run oracle/build_ref.sh where the reference tree is present")
    synth = importlib.import_module("tokspur-public_amd.synth")
    out = {}
    # block decode: native/src/numeric.cpp:97-148
    for t in (7, 8, 12, 13, 14):
        epb, _ = ref.encoding(t)
        raw = synth.BLOCKS[t][0](7000 + t, 6).reshape(-1)
        out[f"dequant_{t}_in"] = raw
        out[f"dequant_{t}_out"] = ref.dequantize(t, raw, 6 * epb).view(np.uint32)
    # GEMV: native/src/numeric.cpp:150-184
    for t, cols, rows in ((12, 512, 6), (14, 256, 5), (8, 96, 7)):
        w = synth.matrix(t, 7100 + t, rows, cols)
        x = synth.activations_f32(7101 + t, cols)
        out[f"gemv_{t}_w"], out[f"gemv_{t}_x"] = w, x
        out[f"gemv_{t}_y"] = ref.reference_gemv(t, w, cols, rows, x).view(np.uint64)
    # Q8_0 many rows: native/src/q8_many.cpp:36-49
    w = synth.matrix(8, 7200, 9, 128)
    x = synth.activations_f32(7201, (4, 128))
    out["q8many_w"], out["q8many_x"] = w, x
    out["q8many_y"] = ref.reference_q8_many(w, x, 128, 9, 4).astype(np.float64).view(np.uint64)
    # q8_lanes_v1 rows: native/src/expert_lanes.cpp:60-119
    w = synth.matrix(8, 7300, 3, 1024)
    out["lanes_in"], out["lanes_out"] = w, ref.q8_lanes_pack_rows(1024, w)
    # router and mixture: native/src/routing.cpp:11-60
    logits = synth.activations_f32(7400, (5, 64)).astype(np.float64)
    logits[1, 7] = logits[1, 3] = logits[1, 40]  # exact ties: ascending id decides
    ids, weights = [], []
    for mode, normalize in ((0, True), (0, False), (1, True)):
        for row in logits:
            i, w_ = ref.route_reference(row, 6, mode, normalize)
            ids.append(i)
            weights.append(w_)
    out["route_logits"] = logits
    out["route_ids"] = np.array(ids, dtype=np.uint32)
    out["route_weights"] = np.array(weights, dtype=np.float64).view(np.uint64)
    experts = synth.activations_f32(7401, (6, 32)).astype(np.float64)
    shared = synth.activations_f32(7402, 32).astype(np.float64)
    out["mixture_experts"], out["mixture_shared"] = experts, shared
    out["mixture_weights"] = np.array(weights[0], dtype=np.float64)
    out["mixture_out"] = np.asarray(ref.mixture_reference(experts, np.array(weights[0]), shared, 0.75), dtype=np.float64).view(np.uint64)
    # row top-64: native/src/sampling.cpp:473-513
    row = np.round(synth.activations_f32(7500, 300), 1).astype(np.float32)
    row[[4, 9]] = [np.inf, np.nan]
    row[17] = np.float32(1e-41)
    top = ref.logit_topk_row(row)
    out["topk_in"] = row
    out["topk_ids"] = np.array(top.ids, dtype=np.uint32)
    out["topk_logits"] = np.array(top.logits, dtype=np.float32).view(np.uint32)
    out["topk_meta"] = np.array([top.count, top.first_nonfinite_col, top.first_subnormal_col], dtype=np.uint32)
    # plan geometry: native/src/grouped_mm.cpp:24-54, native/src/moe_mm_many_plan.cpp:28-52
    views, total = ref.moe_mm_many_bytes(2048, 512, 512, 10, 2048, True)
    out["moe_mm_many_bytes"] = np.array(list(views) + [total], dtype=np.uint64)
    p = ref.grouped_mm_plan(12, 0, 2048, 512, 512, 10, 2048, 8192, 2048, True, True)
    out["grouped_mm_plan"] = np.array([p.maximum_tasks, p.matrix_bytes, p.token_map_bytes, p.counts_bytes, p.tasks_bytes, p.grid_x, p.grid_y], dtype=np.uint64)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()

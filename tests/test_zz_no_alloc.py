"""GPU test of `tsp_logit_topk_static`, the row top-64 for callers that cannot allocate: its partial rows live in a device
array inside the library. Two calls in a row, the second on a smaller input, each bit-identical to `tsp_logit_topk` (which
takes the scratch as an argument) and to the CPU ordering rule; shapes beyond the array are refused."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _rows(seed, rows, vocab):
    rng = np.random.default_rng(seed)
    logits = rng.standard_normal((rows, vocab)).astype(np.float32)
    logits[0, :40] = 3.5          # ties: ascending column order decides
    logits[rows - 1, vocab // 2] = np.inf
    logits[rows - 1, 7] = np.float32(1e-41)
    return logits


def test_static_scratch_topk_matches_the_scratch_argument_form(gpu, tsp, orc):
    import torch
    fields = ("vocabulary", "count", "first_nonfinite_col", "first_subnormal_col", "ids", "logits")
    for seed, rows, vocab in ((1, 16, 151936), (2, 3, 5000)):  # the second call is smaller: stale partial rows must not be read
        logits = _rows(seed, rows, vocab)
        d = gpu.upload(logits)
        out = gpu.empty(tsp.logit_topk_output_bytes(rows), "uint8")
        torch.cuda.synchronize()
        # device-wide free bytes, not torch's own counter: a hipMalloc inside the library would not move the latter. The first
        # call on a device looks the array's address up (no allocation either: the array is part of the loaded code object).
        before, reserved = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
        tsp.logit_topk_static(gpu, d, rows, vocab, out=out)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == before and torch.cuda.memory_reserved() == reserved
        got = out.cpu().numpy().view(tsp.TOPK_ROW_DTYPE)
        ref = tsp.logit_topk(gpu, d, rows, vocab).cpu().numpy().view(tsp.TOPK_ROW_DTYPE)
        for name in fields:
            assert np.array_equal(got[name].view(np.uint32), ref[name].view(np.uint32)), (rows, vocab, name)
        for r in (0, rows - 1):
            want = orc.logit_topk_row(logits[r])
            assert (got[r]["vocabulary"], got[r]["count"]) == (vocab, want.count)
            assert got[r]["first_nonfinite_col"] == want.first_nonfinite_col and got[r]["first_subnormal_col"] == want.first_subnormal_col
            assert np.array_equal(got[r]["ids"], np.array(want.ids, dtype=np.uint32))
            assert np.array_equal(got[r]["logits"].view(np.uint32), np.array(want.logits, dtype=np.float32).view(np.uint32))


def test_static_scratch_topk_under_stream_capture(gpu, tsp, orc):
    """The use the entry point is for: after one eager call on the device, a call recorded into a HIP graph and replayed.
    Every replay, with new logits copied in between and eager work of the program's own around it, gives the rows of
    `tsp_logit_topk` bit for bit."""
    import torch
    fields = ("vocabulary", "count", "first_nonfinite_col", "first_subnormal_col", "ids", "logits")
    rows, vocab = 4, 40000
    d = gpu.upload(_rows(10, rows, vocab))
    out = gpu.empty(tsp.logit_topk_output_bytes(rows), "uint8")
    tsp.logit_topk_static(gpu, d, rows, vocab, out=out)  # eager: the address look-up happens here, outside capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        tsp.logit_topk_static(gpu, d, rows, vocab, out=out)
    for replay in range(4):
        logits = _rows(20 + replay, rows, vocab)
        d.copy_(gpu.upload(logits))
        out.fill_(0xEE)
        torch.cuda.synchronize()
        free = torch.cuda.mem_get_info()[0]
        graph.replay()
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free
        got = out.cpu().numpy().view(tsp.TOPK_ROW_DTYPE)
        ref = tsp.logit_topk(gpu, d, rows, vocab).cpu().numpy().view(tsp.TOPK_ROW_DTYPE)
        for name in fields:
            assert np.array_equal(got[name].view(np.uint32), ref[name].view(np.uint32)), (replay, name)
        want = orc.logit_topk_row(logits[0])
        assert np.array_equal(got[0]["ids"], np.array(want.ids, dtype=np.uint32))


def test_static_scratch_topk_refuses_what_does_not_fit(gpu, tsp):
    x = gpu.zeros((17, 128))
    with pytest.raises(tsp.FormatError):
        tsp.logit_topk_static(gpu, x, 17, 128)
    with pytest.raises(tsp.FormatError):
        tsp.logit_topk_static(gpu, x, 1, 262145, stride_bytes=262145 * 4)
    with pytest.raises(tsp.FormatError):
        tsp.logit_topk_static(gpu, x, 2, 128, out=gpu.empty(528, "uint8"))

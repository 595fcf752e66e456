"""GPU parity for the router (ids bit-exact), the expert permutation and prefix-sum offsets
(bit-exact), the T <= 8 union records (bit-exact), and the mixture / SwiGLU operators."""
import math

import numpy as np
import pytest

from test_oracle_pack import union_spec
from test_oracle_routing import std_mt19937

pytestmark = pytest.mark.gpu


def u32(t):
    return t.cpu().numpy().view(np.uint32)


# ---------------------------------------------------------------------------------- router

def test_route_reference_trials(gpu, orc):
    # native/tests/test_routing.cpp:24-48 trials, pushed through the device router; logits are multiples of 0.01
    # rounded to f32, so the f32 order (with its ties) is what the oracle sees too.
    bg = std_mt19937(0x726F7574)
    for trial in range(300):
        count = 1 + int(bg.random_raw()) % 1024
        selected = 1 + int(bg.random_raw()) % min(64, count)
        logits = ((bg.random_raw(count).astype(np.int64) % 2001 - 1000) / 100.0).astype(np.float32)
        mode, normalize = trial % 2, (trial // 2) % 2 == 0
        ids, w = gpu.route(gpu.upload(logits), selected, mode, normalize)
        want_ids, want_w = orc.route_reference(logits.astype(np.float64), selected, mode, normalize)
        assert np.array_equal(u32(ids)[0], want_ids), trial
        assert np.allclose(w.cpu().numpy()[0], want_w, rtol=2e-5, atol=1e-7), trial
    assert gpu.error() == 0


def test_route_goldens(gpu, orc):
    # native/tests/test_routing.cpp:49-51 tie golden; native/tests/test_moe_mm_many_gpu.cpp:252-253 all-zero logits.
    ids, _ = gpu.route(gpu.upload(np.array([3, 3, 2, 1, 3], dtype=np.float32)), 3, 0, True)
    assert list(u32(ids)[0]) == [0, 1, 4]
    ids, w = gpu.route(gpu.upload(np.zeros((4, 512), dtype=np.float32)), 10, 0, True, tokens=4)
    assert (u32(ids) == np.arange(10)).all() and np.allclose(w.cpu().numpy(), 0.1, rtol=1e-6)
    # -0.0 and +0.0 compare equal: ties go to the lower id
    ids, _ = gpu.route(gpu.upload(np.array([-0.0, 0.0, -0.0, 0.0], dtype=np.float32)), 2, 0, True)
    assert list(u32(ids)[0]) == [0, 1]
    # underflow cases, native/tests/test_routing.cpp:60-64
    _, w = gpu.route(gpu.upload(np.array([-1000.0], dtype=np.float32)), 1, 1, True)
    assert w.cpu().numpy()[0, 0] == 1.0
    _, w = gpu.route(gpu.upload(np.array([-1000.0], dtype=np.float32)), 1, 0, True)
    assert w.cpu().numpy()[0, 0] == 1.0 and gpu.error() == 0


@pytest.mark.parametrize("tokens,experts,selected", [(8, 512, 10), (2048, 512, 10), (33, 64, 4), (5, 200, 64)])
def test_route_batch_ids_bit_exact(gpu, orc, synth, tokens, experts, selected):
    """Configs 2 and 3: softmax, top-10 renormalised over 512 experts; Zipf-biased logits at T = 2048."""
    seed = synth.tensor_seed(3, 10 + tokens)
    logits = synth.zipf_router_logits(seed, tokens, experts, scale=synth.ZIPF_BIAS_SCALE) if tokens == 2048 else synth.activations_f32(seed, (tokens, experts))
    if tokens == 33:
        logits = np.round(logits * 2) / 2  # plenty of exact ties
    ids, w = gpu.route(gpu.upload(logits), selected, 0, True, tokens=tokens)
    ids, w = u32(ids), w.cpu().numpy()
    for t in range(tokens):
        want_ids, want_w = orc.route_reference(logits[t].astype(np.float64), selected, 0, True)
        assert np.array_equal(ids[t], want_ids), t
        assert np.allclose(w[t], want_w, rtol=2e-5, atol=1e-9), t
    assert gpu.error() == 0
    assert np.allclose(w.sum(axis=1), 1.0, rtol=1e-5)


def lcg_values(state, count):
    """`count` draws of the 32-bit generator x -> 1664525 x + 1013904223 as float(int(x % 1993) - 996) / 997, and the state."""
    out = np.empty(count, dtype=np.float64)
    for i in range(count):
        state = (state * 1664525 + 1013904223) & 0xFFFFFFFF
        out[i] = (state % 1993) - 996
    return (out / 997), state


def test_router_f32_batch_reference_controls(gpu, orc, tsp):
    """native/tests/test_moe_mm_many_gpu.cpp:194-262: dense non-binary f32 weights [512, 2560] and strided, poisoned rows;
    every logit within 5e-5 * max(1, |sum|) of the double sum and of the per-row f32 GEMV, padding untouched, the ten
    selected ids equal to the scalar path's and to the double route for both modes."""
    c, e, capacity = 2560, 512, 512
    xs, ys = c * 4 + 32, e * 4 + 32
    w64, state = lcg_values(44, c * e)
    weights = (w64.astype(np.float32) / np.float32(256)).reshape(e, c)
    x64, state = lcg_values(state, capacity * c)
    x_rows = np.full((capacity, xs // 4), -9876.25, dtype=np.float32)
    x_rows[:, :c] = x64.astype(np.float32).reshape(capacity, c)
    d_w, d_x = gpu.upload(weights), gpu.upload(x_rows)
    want = x_rows[:, :c].astype(np.float64) @ weights.astype(np.float64).T
    for n in (1, 2, 3, 8, 31, 32, 33, 511, 512):
        y = gpu.full((capacity, ys // 4), -7654.25)
        scalar = gpu.full((capacity, ys // 4), -7654.25)
        gpu.router_f32_batch(d_w, d_x, n, c, e, x_stride=xs, out=y, out_stride=ys)
        gpu.gemv_rows(0, d_w, d_x, scalar, n, c, e, xs, ys)
        got, legacy = y.cpu().numpy(), scalar.cpu().numpy()
        bound = 0.00005 * np.maximum(1.0, np.abs(want[:n]))
        assert np.isfinite(got[:n, :e]).all() and (np.abs(got[:n, :e] - want[:n]) <= bound).all(), n
        assert (np.abs(legacy[:n, :e] - want[:n]) <= bound).all() and (np.abs(got[:n, :e].astype(np.float64) - legacy[:n, :e]) <= bound).all(), n
        assert (got[:n, e:] == -7654.25).all() and (got[n:] == -7654.25).all(), "router output row padding / inactive rows"
        # tighter than the engine asks: f32 products and sums leave ~1e-6 of the sum of |w x|
        scale = np.abs(x_rows[:n, :c]).astype(np.float64) @ np.abs(weights).astype(np.float64).T
        assert (np.abs(got[:n, :e] - want[:n]) <= 2e-6 * scale).all(), n
        compact, compact_old = gpu.upload(np.ascontiguousarray(got[:n, :e])), gpu.upload(np.ascontiguousarray(legacy[:n, :e]))
        for mode in (0, 1):
            for normalise in (False, True):
                ids, wts = gpu.route(compact, 10, mode, normalise, tokens=n)
                old_ids, old_wts = gpu.route(compact_old, 10, mode, normalise, tokens=n)
                assert np.array_equal(u32(ids), u32(old_ids)), "router all-row selected IDs differ from actual scalar route"
                assert np.abs(wts.cpu().numpy() - old_wts.cpu().numpy()).max() <= 0.00005
                for t in range(0, n, max(1, n // 16)):
                    want_ids, want_w = orc.route_reference(want[t], 10, mode, normalise)
                    assert np.array_equal(u32(ids)[t], want_ids) and np.abs(wts.cpu().numpy()[t] - want_w).max() <= 0.00005
    # exact ties select low ids
    y = gpu.router_f32_batch(gpu.zeros((e, c)), d_x, 3, c, e, x_stride=xs)
    ids, _ = gpu.route(y, 10, 0, True, tokens=3)
    assert (u32(ids) == np.arange(10)).all() and gpu.error() == 0
    # refusals: short stride, output over an input, odd column count
    y = gpu.full((capacity, ys // 4), -7654.25)
    for call in (lambda: gpu.router_f32_batch(d_w, d_x, 3, c, e, x_stride=xs, out=y, out_stride=e * 4 - 4),
                 lambda: gpu.router_f32_batch(d_w, d_x, 3, c, e, x_stride=xs, out=d_x, out_stride=ys),
                 lambda: gpu.router_f32_batch(d_w, d_x, 3, c, e, x_stride=xs, out=d_w, out_stride=ys),
                 lambda: gpu.router_f32_batch(d_w, d_x, 3, c - 8, e, x_stride=xs, out=y, out_stride=ys),
                 lambda: gpu.router_f32_batch(d_w, d_x, 0, c, e, x_stride=xs, out=y, out_stride=ys)):
        with pytest.raises(tsp.FormatError):
            call()
    assert (y.cpu().numpy() == -7654.25).all(), "router refusal does not write output"


@pytest.mark.parametrize("tokens,columns,experts", [(1, 32, 1), (33, 96, 70), (130, 160, 65), (2048, 2048, 512)])
def test_router_f32_batch_shapes(gpu, synth, tokens, columns, experts):
    """Ragged tiles in every direction and the configs[3] chunk; a non-finite input raises the sticky bit."""
    w = synth.activations_f32(synth.tensor_seed(5, tokens), (experts, columns)) / np.float32(16)
    x = synth.activations_f32(synth.tensor_seed(6, tokens), (tokens, columns))
    pitch = (experts + 3) // 4 * 4  # output rows lie a multiple of 16 bytes apart, as the engine's planner demands

    def run(rows):
        out = gpu.full((tokens, pitch), -3.0)
        gpu.router_f32_batch(gpu.upload(w), gpu.upload(rows), tokens, columns, experts, out=out, out_stride=pitch * 4)
        out = out.cpu().numpy()
        assert (out[:, experts:] == -3.0).all()
        return np.ascontiguousarray(out[:, :experts])

    got = run(x)
    want = x.astype(np.float64) @ w.astype(np.float64).T
    scale = np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64).T
    assert (np.abs(got - want) <= 2e-6 * scale + 1e-30).all() and gpu.error() == 0
    assert np.array_equal(got.view(np.uint32), run(x).view(np.uint32))
    x[tokens // 2, columns - 1] = np.inf
    run(x)
    assert gpu.error() == 1


def test_route_errors(gpu, tsp):
    logits = np.zeros(16, dtype=np.float32)
    logits[3] = np.nan
    ids, _ = gpu.route(gpu.upload(logits), 2, 0, True)
    assert gpu.error() & tsp.ERRBIT_NONFINITE and list(u32(ids)[0]) == [0, 1]
    for args in ((0, 0, True), (17, 0, True), (2, 2, True)):
        with pytest.raises(tsp.FormatError):
            gpu.route(gpu.upload(np.zeros(16, dtype=np.float32)), *args)
    with pytest.raises(tsp.FormatError):
        gpu.route(gpu.upload(np.zeros((2, 600), dtype=np.float32)), 2, 0, True, tokens=2)


# ---------------------------------------------------------------------------------- permutation

def random_ids(rng, tokens, selected, experts, skew=False):
    out = np.empty((tokens, selected), dtype=np.uint32)
    p = None
    if skew:
        p = 1.0 / np.arange(1, experts + 1) ** 1.1
        p /= p.sum()
    for t in range(tokens):
        out[t] = rng.choice(experts, size=selected, replace=False, p=p)
    return out.reshape(-1)


@pytest.mark.parametrize("tokens,selected,experts", [(1, 1, 2), (5, 3, 8), (33, 4, 16), (100, 10, 64), (64, 2, 4), (257, 10, 512),
                                                     (2048, 10, 512), (544, 4, 8)])
def test_grouped_routes_and_tasks_bit_exact(gpu, orc, tokens, selected, experts):
    rng = np.random.default_rng(tokens * 31 + selected)
    ids = random_ids(rng, tokens, selected, experts, skew=tokens == 2048)
    want_map, want_counts, err = orc.grouped_routes(ids, experts, selected, tokens)
    assert err == 0
    token_map, counts = gpu.grouped_routes(gpu.upload(ids), experts, selected, tokens)
    assert np.array_equal(u32(counts), want_counts)
    assert np.array_equal(u32(token_map).reshape(-1), want_map)  # untouched tails keep the caller's fill on both sides
    want_tasks, err = orc.grouped_tasks(want_counts, experts, selected, tokens, 32)
    tasks = gpu.grouped_tasks(counts, experts, selected, tokens, 32)
    assert err == 0 and np.array_equal(u32(tasks), want_tasks) and gpu.error() == 0
    # size-independent invariants of the permutation
    tm = u32(token_map).reshape(experts, tokens)
    seen = np.concatenate([tm[e, :want_counts[e]] for e in range(experts)])
    assert np.array_equal(np.sort(seen), np.arange(tokens * selected))
    for e in range(experts):
        row = tm[e, :want_counts[e]]
        assert (ids[row] == e).all() and (np.diff(row.astype(np.int64)) > 0).all()


def test_grouping_error_bits(gpu, tsp):
    for ids in ([0, 9], [1, 1]):
        gpu.grouped_routes(gpu.upload(np.array(ids, dtype=np.uint32)), 4, 2, 1)
        assert gpu.error() == tsp.ERRBIT_INDEX
    gpu.grouped_tasks(gpu.upload(np.array([1, 0, 0, 0], dtype=np.uint32)), 4, 2, 1)
    assert gpu.error() == tsp.ERRBIT_INDEX
    gpu.grouped_tasks(gpu.upload(np.array([9, 0, 0, 0], dtype=np.uint32)), 4, 2, 4)
    assert gpu.error() == tsp.ERRBIT_INDEX


def test_union_metadata_all_cases_bit_exact(gpu, orc):
    # native/tests/test_planar_union_metadata.mm:105-124: T = 1..8 x S = 1..16, four id patterns each; untouched
    # words must keep the caller's poison and invalid ids must zero the header and raise bit 4.
    bg = std_mt19937(1729)
    for tokens in range(1, 9):
        for selected in range(1, 17):
            n = tokens * selected
            mixed = [int(bg.random_raw()) % 7 if i % 3 else 511 for i in range(n)]
            for ids in ([511] * n, [(511 - i) % 512 for i in range(n)], mixed, mixed[:-1] + [512]):
                got = u32(gpu.union_build(gpu.upload(np.array(ids, dtype=np.uint32)), 512, selected, tokens, 639, 2559))
                want, want_err = union_spec(512, selected, tokens, 639, 2559, ids)
                assert gpu.error() == want_err and np.array_equal(got, want), (tokens, selected)
                assert np.array_equal(got, orc.union_metadata(512, selected, tokens, 639, 2559, ids)[0])
    for shape, ids in (((3, 1, 1, 640, 2560), [0]), ((2, 3, 1, 640, 2560), [0, 1, 0])):
        got = u32(gpu.union_build(gpu.upload(np.array(ids, dtype=np.uint32)), *shape))
        assert gpu.error() == 4 and not got[:8].any() and (got[8:] == 0xBAADF00D).all()


# ---------------------------------------------------------------------------------- mixture / SwiGLU

def test_mixture_golden_and_rows(gpu, orc, synth):
    # native/tests/test_routing.cpp:52-55
    out = gpu.mixture(gpu.upload(np.array([1, 2, 3, 4], dtype=np.float32)), gpu.upload(np.array([0.25, 0.75], dtype=np.float32)),
                      gpu.upload(np.array([5, 6], dtype=np.float32)), gpu.upload(np.zeros(1, dtype=np.float32)), 2, 2)
    assert list(out.cpu().numpy()[0]) == [5.0, 6.5]
    tokens, selected, channels = 37, 10, 2048
    ex = synth.activations_f32(1, (tokens, selected, channels))
    w = np.abs(synth.activations_f32(2, (tokens, selected))) / 10
    sh = synth.activations_f32(3, (tokens, channels))
    sl = synth.activations_f32(4, tokens)
    out = gpu.full((tokens, channels + 16), -3.0)
    gpu.mixture(gpu.upload(ex), gpu.upload(w), gpu.upload(sh), gpu.upload(sl), channels, selected, tokens, out=out, out_stride=(channels + 16) * 4)
    out = out.cpu().numpy()
    for t in range(tokens):
        want = orc.mixture_reference(ex[t].astype(np.float64), w[t].astype(np.float64), sh[t].astype(np.float64), float(sl[t]))
        assert np.max(np.abs(out[t, :channels] - want) / np.maximum(1, np.abs(want))) <= 5e-6
    assert (out[:, channels:] == -3.0).all() and gpu.error() == 0


def test_mixture_errors(gpu, tsp):
    one = gpu.upload(np.ones(4, dtype=np.float32))
    gpu.mixture(gpu.upload(np.ones(8, dtype=np.float32)), gpu.upload(np.array([0.5, -0.5], dtype=np.float32)), one,
                gpu.upload(np.zeros(1, dtype=np.float32)), 4, 2)
    assert gpu.error() == tsp.ERRBIT_NONFINITE
    gpu.mixture(gpu.upload(np.ones(8, dtype=np.float32)), gpu.upload(np.array([0.5, 0.5], dtype=np.float32)), one,
                gpu.upload(np.array([np.inf], dtype=np.float32)), 4, 2)
    assert gpu.error() == tsp.ERRBIT_NONFINITE


def test_swiglu(gpu, tsp, orc):
    g = np.linspace(-30, 30, 4001).astype(np.float32)
    u = np.cos(np.arange(4001)).astype(np.float32) * 3
    out = gpu.swiglu(gpu.upload(g), gpu.upload(u), 0.5).cpu().numpy()
    want = np.array([orc.stable_silu(float(np.float32(a) * np.float32(0.5))) * float(b) for a, b in zip(g, u)])
    assert np.max(np.abs(out - want) / np.maximum(1, np.abs(want))) <= 2e-6 and gpu.error() == 0
    assert gpu.swiglu(gpu.upload(np.zeros(3, dtype=np.float32)), gpu.upload(np.ones(3, dtype=np.float32))).cpu().numpy().tolist() == [0, 0, 0]
    bad = g.copy()
    bad[5] = np.nan
    gpu.swiglu(gpu.upload(bad), gpu.upload(u))
    assert gpu.error() == tsp.ERRBIT_NONFINITE


# ---------------------------------------------------------------------------------- RMS, activations, residual streams

def scaled(got, want):
    return float(np.max(np.abs(np.asarray(got, dtype=np.float64) - want) / np.maximum(1.0, np.abs(want))))


@pytest.mark.parametrize("branches,channels,rank", [(1, 7, 3), (4, 9, 5), (3, 257, 16), (4, 2560, 320)])
def test_gated_residual_composition(gpu, orc, branches, channels, rank):
    """native/tests/test_graph.cpp:113-141: rms -> F32 GEMV -> SiLU(x / branches) in place -> two F32 GEMVs -> residual_read ->
    residual_write against gated_residual_reference / residual_write_reference, 5e-5 scaled error; the streams stay untouched."""
    rng = np.random.default_rng(branches * 1000 + channels)
    width = branches * channels
    streams = rng.uniform(-1, 1, width).astype(np.float32)
    gains = (1 + rng.uniform(-0.1, 0.1, width)).astype(np.float32)
    down = rng.uniform(-0.01, 0.01, (rank, width)).astype(np.float32)
    up = rng.uniform(-0.01, 0.01, (width, rank)).astype(np.float32)
    inject = rng.uniform(-0.01, 0.01, (branches, width)).astype(np.float32)
    epsilon = 1e-6
    want_read, want_scales = orc.gated_residual_reference(streams, gains, down, up, inject, branches, channels, rank, np.float32(epsilon))
    d_streams = gpu.upload(streams)
    normalized = gpu.rms(d_streams, gpu.upload(gains), channels, epsilon)
    bottleneck = gpu.gemv(0, gpu.upload(down), normalized, width, rank)
    gpu.activate(bottleneck, 1, 1.0 / branches, out=bottleneck)
    scores = gpu.gemv(0, gpu.upload(up), bottleneck, rank, width)
    logits = gpu.gemv(0, gpu.upload(inject), normalized, width, branches)
    read, scales = gpu.residual_read(normalized, scores, logits, branches, channels)
    written = gpu.residual_write(d_streams, read, scales, branches, channels)
    assert gpu.error() == 0
    assert scaled(read.cpu().numpy(), want_read) <= 5e-5 and scaled(scales.cpu().numpy(), want_scales) <= 5e-5
    assert scaled(written.cpu().numpy(), orc.residual_write_reference(streams, want_read, want_scales)) <= 5e-5
    assert np.array_equal(d_streams.cpu().numpy(), streams)
    # the streams updated in place give the same bits
    gpu.residual_write(d_streams, read, scales, branches, channels, out=d_streams)
    assert np.array_equal(d_streams.cpu().numpy().view(np.uint32), written.cpu().numpy().view(np.uint32))


def test_rms_activate_multiply(gpu, orc, tsp):
    rng = np.random.default_rng(77)
    for groups, width, shared in ((1, 1, False), (5, 128, True), (48, 128, True), (7, 333, False), (3, 65536, True)):
        x = rng.normal(size=groups * width).astype(np.float32)
        gains = rng.normal(size=width if shared else groups * width).astype(np.float32)
        gate = rng.normal(size=groups * width).astype(np.float32) * 3
        full_gains = np.tile(gains, groups) if shared else gains
        want = orc.group_rms_reference(x, full_gains, width, np.float32(1e-6))
        got = gpu.rms(gpu.upload(x), gpu.upload(gains), width, 1e-6).cpu().numpy()
        assert scaled(got, want) <= 5e-5, (groups, width)
        gated = gpu.rms(gpu.upload(x), gpu.upload(gains), width, 1e-6, gate=gpu.upload(gate)).cpu().numpy()
        assert scaled(gated, want / (1 + np.exp(-gate.astype(np.float64)))) <= 5e-5
        # the fused form is the composition of rms and multiply(sigmoid_gate) (kernels/graph.metal:249)
        two_step = gpu.multiply(gpu.upload(got), gpu.upload(gate), True).cpu().numpy()
        assert np.abs(gated - two_step).max() <= 1e-6 * max(1.0, np.abs(gated).max())
    x = np.concatenate([rng.normal(size=1000) * 10, [0.0, -0.0, 88.0, -88.0, 1e-30, -104.0, 30.0, -30.0]]).astype(np.float32)
    x64 = x.astype(np.float64)
    for kind, f in ((0, lambda v: v), (1, lambda v: v / (1 + np.exp(-v))), (2, lambda v: 1 / (1 + np.exp(-v))), (3, lambda v: np.maximum(v, 0) + np.log1p(np.exp(-np.abs(v))))):
        for scale in (1.0, 0.25):
            got = gpu.activate(gpu.upload(x), kind, scale).cpu().numpy()
            assert scaled(got, f(x64 * np.float32(scale))) <= 5e-5, kind
    # softplus keeps its tiny tail where 1 + e^-|x| rounds to 1
    tail = gpu.activate(gpu.upload(np.array([-30.0, -80.0], dtype=np.float32)), 3).cpu().numpy()
    assert tail[0] > 0 and abs(tail[0] / math.exp(-30.0) - 1) < 1e-5 and tail[1] > 0
    y = gpu.multiply(gpu.upload(x), gpu.upload(x[::-1].copy())).cpu().numpy()
    assert np.array_equal(y, x * x[::-1])
    assert gpu.error() == 0
    # error contract (kernels/graph.metal:18-21, 284-311): activate stores the non-finite operand itself and raises the flag;
    # multiply tests its operands first and leaves that destination alone; refusals on the host
    bad = x.copy()
    bad[3] = np.inf
    out = gpu.full(bad.size, -5.0)
    gpu.activate(gpu.upload(bad), 2, out=out)
    assert gpu.error() == 1 and out.cpu().numpy()[3] == np.inf and out.cpu().numpy()[4] != -5.0
    out = gpu.full(bad.size, -5.0)
    gpu.multiply(gpu.upload(x), gpu.upload(bad), out=out)
    assert gpu.error() == 1 and out.cpu().numpy()[3] == -5.0
    big = np.full(64, 3e38, dtype=np.float32)
    out = gpu.full(64, -5.0)
    gpu.rms(gpu.upload(big), gpu.upload(np.ones(64, dtype=np.float32)), 64, 1e-6, out=out)
    assert gpu.error() == 1 and (out.cpu().numpy() == -5.0).all()
    d = gpu.upload(x)
    for call in (lambda: gpu.rms(d, d, 11, 1e-6), lambda: gpu.rms(d, d, 8, 0.0), lambda: gpu.rms(d, d, 8, float("nan")), lambda: gpu.rms(d, d, 8, 1e-6, out=d),
                 lambda: gpu.activate(d, 4), lambda: gpu.activate(d, 1, float("inf")), lambda: gpu.residual_read(d, d, d, 65, 4), lambda: gpu.residual_write(d, d, d, 2, 70000)):
        with pytest.raises(tsp.FormatError):
            call()


def test_destination_contents_after_a_refused_batch(gpu, tsp):
    """kernels/graph.metal:18-21 `checked_store` stores a non-finite result and raises the flag; the operators that test their
    operands first (graph.metal:258-311, 340-347) raise it and store nothing for that element. A caller that looks at its
    buffers after a refused batch finds what the engine leaves there, in place forms included."""
    inf, nan = np.float32(np.inf), np.float32(np.nan)
    x = np.array([1.0, inf, -2.0, nan, 0.5, -inf, 3.0, 4.0], dtype=np.float32)
    for kind in (0, 1, 2, 3):  # activate: the scaled operand itself is what lands, never sigmoid(inf) = 1
        buf = gpu.upload(x)
        gpu.activate(buf, kind, 1.0, out=buf)
        got = buf.cpu().numpy()
        assert gpu.error() == tsp.ERRBIT_NONFINITE
        gpu.clear_error()
        assert got[1] == inf and np.isnan(got[3]) and got[5] == -inf and np.isfinite(got[[0, 2, 4, 6, 7]]).all()
    gate = np.array([1.0, 1.0, inf, 1.0, 2.0, 1.0, 1.0, 3e38], dtype=np.float32)
    big = np.array([1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 3e38], dtype=np.float32)
    out = gpu.full((8,), -9.0)
    gpu.multiply(gpu.upload(big), gpu.upload(gate), False, out=out)
    got = out.cpu().numpy()
    assert gpu.error() == tsp.ERRBIT_NONFINITE
    gpu.clear_error()
    assert got[2] == -9.0 and got[7] == inf and got[4] == 10.0  # bad operand: untouched; overflowing product: stored
    buf = gpu.upload(x)
    gpu.multiply(buf, gpu.upload(np.ones(8, dtype=np.float32)), False, out=buf)  # in place: the bad elements stay what they were
    got = buf.cpu().numpy()
    gpu.clear_error()
    assert got[1] == inf and np.isnan(got[3]) and got[0] == 1.0
    # rms: a group whose sum of squares is not finite stores nothing; a finite group beside it is normalised
    groups = np.array([1.0, 2.0, inf, 4.0, 3.0, 4.0, 0.0, 0.0], dtype=np.float32)
    out = gpu.full((8,), -9.0)
    gpu.rms(gpu.upload(groups), gpu.upload(np.ones(4, dtype=np.float32)), 4, 1e-6, out=out)
    got = out.cpu().numpy()
    assert gpu.error() == tsp.ERRBIT_NONFINITE
    gpu.clear_error()
    assert (got[:4] == -9.0).all() and abs(got[4] - 3.0 / np.sqrt(6.25)) <= 1e-6
    # rms_sigmoid_gate: a non-finite gate skips its element only
    out = gpu.full((4,), -9.0)
    gpu.rms(gpu.upload(np.array([3.0, 4.0, 0.0, 0.0], dtype=np.float32)), gpu.upload(np.ones(4, dtype=np.float32)), 4, 1e-6,
            gate=gpu.upload(np.array([0.0, nan, 0.0, 0.0], dtype=np.float32)), out=out)
    got = out.cpu().numpy()
    assert gpu.error() == tsp.ERRBIT_NONFINITE
    gpu.clear_error()
    assert got[1] == -9.0 and abs(got[0] - 0.5 * 3.0 / np.sqrt(6.25)) <= 1e-6
    # residual_read: the thread of a bad channel writes neither its channel nor the scale of the same index
    branches, channels = 2, 3
    normalized = np.array([[1.0, inf, 3.0], [1.0, 1.0, 1.0]], dtype=np.float32)
    scores = np.zeros((branches, channels), dtype=np.float32)
    read, scales = gpu.full((channels,), -9.0), gpu.full((branches,), -7.0)
    gpu.residual_read(gpu.upload(normalized), gpu.upload(scores), gpu.upload(np.zeros(branches, dtype=np.float32)), branches, channels, out=read, scales=scales)
    got, got_s = read.cpu().numpy(), scales.cpu().numpy()
    assert gpu.error() == tsp.ERRBIT_NONFINITE
    gpu.clear_error()
    assert got[0] == 0.5 and got[1] == -9.0 and got[2] == 1.0 and got_s[0] == 1.0 and got_s[1] == -7.0
    # residual_write: an overflowing sum is stored
    streams = np.array([3e38, 1.0], dtype=np.float32)
    written = gpu.residual_write(gpu.upload(streams), gpu.upload(np.array([3e38, 1.0], dtype=np.float32)), gpu.upload(np.array([1.0], dtype=np.float32)), 1, 2)
    got = written.cpu().numpy()
    assert gpu.error() == tsp.ERRBIT_NONFINITE
    gpu.clear_error()
    assert got[0] == inf and got[1] == 2.0

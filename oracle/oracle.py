"""ctypes doorway onto the CPU oracle (TEST INFRASTRUCTURE ONLY).

Only tests, the smoke check and the bench's cpu_baseline leg import this module. `lib()` is the C
restatement (liboracle.so, built by oracle/Makefile); `ref()` is the reference's own CPU code
(oracle/_ref/libtokspur_ref.so) when it has been built, else None. Both expose the same call shapes,
`orc_*` and `ref_*`, so a test can run one generic body against either.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_u8p, _f32p, _f64p, _u32p, _u64p = (C.POINTER(t) for t in (C.c_uint8, C.c_float, C.c_double, C.c_uint32, C.c_uint64))


class FormatError(RuntimeError):
    """The reference would have thrown tokspur::FormatError."""


class PlanarSpec(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("source_type", "columns", "rows", "blocks_per_row")] + \
               [(n, C.c_uint64) for n in ("source_row_bytes", "planar_row_bytes", "source_expert_bytes",
                                          "planar_expert_bytes", "qs_offset", "qh_offset", "sm_offset", "dm_offset")]


class TopKRow(C.Structure):
    _fields_ = [("vocabulary", C.c_uint32), ("count", C.c_uint32), ("first_nonfinite_col", C.c_uint32),
                ("first_subnormal_col", C.c_uint32), ("ids", C.c_uint32 * 64), ("logits", C.c_float * 64)]


class GroupedMmPlan(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("columns", "rows", "row_bytes", "experts", "selected", "tokens",
                                          "broadcast", "maximum_tasks")] + \
               [(n, C.c_uint64) for n in ("expert_stride_bytes", "input_stride_bytes", "output_stride_bytes",
                                          "matrix_bytes", "indices_bytes", "input_bytes", "output_bytes",
                                          "token_map_bytes", "counts_bytes", "tasks_bytes")] + \
               [("grid_x", C.c_uint32), ("grid_y", C.c_uint32)]


assert C.sizeof(TopKRow) == 528 and C.sizeof(GroupedMmPlan) == 120


def _p(a, t):
    return a.ctypes.data_as(t)


def _u8(a):
    a = np.ascontiguousarray(np.frombuffer(a, dtype=np.uint8) if isinstance(a, (bytes, bytearray)) else a)
    assert a.dtype == np.uint8
    return a


def _check(status):
    if status:
        raise FormatError(f"oracle status {status}")


class _Lib:
    def __init__(self, path, prefix):
        self.path, self.prefix = path, prefix
        self.dll = C.CDLL(path)
        self._f("binary16").restype = C.c_float
        self._f("binary16").argtypes = [C.c_uint16]

    def _f(self, name):
        return getattr(self.dll, self.prefix + name)  # attribute access caches the function object

    # ---- formats ----
    def binary16(self, bits):
        return float(self._f("binary16")(int(bits)))

    def encoding(self, t):
        e, b = C.c_uint32(), C.c_uint32()
        _check(self._f("encoding")(C.c_uint32(t), C.byref(e), C.byref(b)))
        return e.value, b.value

    def dequantize(self, t, data, nelem):
        data = _u8(data)
        out = np.empty(nelem, dtype=np.float32)
        _check(self._f("dequantize")(C.c_uint32(t), _p(data, _u8p), C.c_uint64(data.size), _p(out, _f32p), C.c_uint64(nelem)))
        return out

    def reference_gemv(self, t, matrix, columns, rows, x):
        matrix = _u8(matrix)
        y = np.empty(rows, dtype=np.float64)
        if np.asarray(x).dtype == np.float64:
            x = np.ascontiguousarray(x, dtype=np.float64)
            _check(self._f("reference_gemv_doubleinput")(C.c_uint32(t), _p(matrix, _u8p), C.c_uint64(matrix.size), C.c_uint32(columns),
                                                        C.c_uint32(rows), _p(x, _f64p), C.c_uint64(x.size), _p(y, _f64p)))
        else:
            x = np.ascontiguousarray(x, dtype=np.float32)
            _check(self._f("reference_gemv")(C.c_uint32(t), _p(matrix, _u8p), C.c_uint64(matrix.size), C.c_uint32(columns),
                                            C.c_uint32(rows), _p(x, _f32p), C.c_uint64(x.size), _p(y, _f64p)))
        return y

    def reference_q8_many(self, matrix, x, columns, rows, width):
        matrix = _u8(matrix)
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.empty((width, rows), dtype=np.float64)
        _check(self._f("reference_q8_many")(_p(matrix, _u8p), C.c_uint64(matrix.size), _p(x, _f32p), C.c_uint32(columns),
                                           C.c_uint32(rows), C.c_uint32(width), _p(out, _f64p)))
        return out

    def q8_many_width(self, remaining):
        w = C.c_uint32()
        _check(self._f("q8_many_width")(C.c_uint32(remaining), C.byref(w)))
        return w.value

    def q8_many_chunks(self, rows):
        w = C.c_uint32()
        _check(self._f("q8_many_chunks")(C.c_uint32(rows), C.byref(w)))
        return w.value

    def _scalar(self, name, v):
        out = C.c_double()
        _check(self._f(name)(C.c_double(v), C.byref(out)))
        return out.value

    def stable_sigmoid(self, v):
        return self._scalar("stable_sigmoid", v)

    def stable_silu(self, v):
        return self._scalar("stable_silu", v)

    def stable_softplus(self, v):
        return self._scalar("stable_softplus", v)

    # ---- operators around the sublayer ----
    def group_rms_reference(self, x, gains, group_width, epsilon):
        x = np.ascontiguousarray(x, dtype=np.float64).reshape(-1)
        gains = np.ascontiguousarray(gains, dtype=np.float64).reshape(-1)
        out = np.empty_like(x)
        _check(self._f("group_rms_reference")(_p(x, _f64p), _p(gains, _f64p), C.c_uint64(x.size), C.c_uint64(group_width), C.c_double(epsilon), _p(out, _f64p)))
        return out

    def gated_residual_reference(self, streams, gains, down, up, inject, branches, channels, rank, epsilon):
        arrays = [np.ascontiguousarray(a, dtype=np.float64).reshape(-1) for a in (streams, gains, down, up, inject)]
        read, scales = np.empty(channels, dtype=np.float64), np.empty(branches, dtype=np.float64)
        _check(self._f("gated_residual_reference")(*[_p(a, _f64p) for a in arrays], C.c_uint64(branches), C.c_uint64(channels), C.c_uint64(rank),
                                                   C.c_double(epsilon), _p(read, _f64p), _p(scales, _f64p)))
        return read, scales

    def residual_write_reference(self, streams, output, scales):
        streams = np.ascontiguousarray(streams, dtype=np.float64).reshape(-1)
        output = np.ascontiguousarray(output, dtype=np.float64).reshape(-1)
        scales = np.ascontiguousarray(scales, dtype=np.float64).reshape(-1)
        result = np.empty_like(streams)
        _check(self._f("residual_write_reference")(_p(streams, _f64p), _p(output, _f64p), _p(scales, _f64p), C.c_uint64(scales.size), C.c_uint64(output.size),
                                                   _p(result, _f64p)))
        return result

    # ---- routing ----
    def route_reference(self, logits, selected, mode=0, normalize=True):
        logits = np.ascontiguousarray(logits, dtype=np.float64)
        ids = np.empty(max(selected, 1), dtype=np.uint32)
        w = np.empty(max(selected, 1), dtype=np.float64)
        _check(self._f("route_reference")(_p(logits, _f64p), C.c_uint64(logits.size), C.c_uint64(selected), C.c_uint32(mode),
                                         C.c_int(bool(normalize)), _p(ids, _u32p), _p(w, _f64p)))
        return ids[:selected], w[:selected]

    def mixture_reference(self, experts, weights, shared, shared_logit):
        experts = np.ascontiguousarray(experts, dtype=np.float64)
        weights = np.ascontiguousarray(weights, dtype=np.float64)
        shared = np.ascontiguousarray(shared, dtype=np.float64)
        if experts.size != weights.size * shared.size:
            raise FormatError("mixture shape mismatch")
        out = np.empty(max(shared.size, 1), dtype=np.float64)
        _check(self._f("mixture_reference")(_p(experts, _f64p), _p(weights, _f64p), C.c_uint64(weights.size), _p(shared, _f64p),
                                           C.c_uint64(shared.size), C.c_double(shared_logit), _p(out, _f64p)))
        return out[:shared.size]

    # ---- q8 lanes ----
    def q8_lanes_quant_offset(self, columns, block, index):
        o = C.c_uint64()
        _check(self._f("q8_lanes_quant_offset")(C.c_uint32(columns), C.c_uint32(block), C.c_uint32(index), C.byref(o)))
        return o.value

    def q8_lanes_pack_rows(self, columns, original):
        original = _u8(original)
        out = np.empty_like(original)
        _check(self._f("q8_lanes_pack_rows")(C.c_uint32(columns), _p(original, _u8p), _p(out, _u8p), C.c_uint64(original.size)))
        return out

    def q8_lanes_unpack_rows(self, columns, packed):
        packed = _u8(packed)
        out = np.empty_like(packed)
        _check(self._f("q8_lanes_unpack_rows")(C.c_uint32(columns), _p(packed, _u8p), _p(out, _u8p), C.c_uint64(packed.size)))
        return out

    # ---- q51 lanes ----
    def q51_lanes_quant_offset(self, columns, block, index):
        o = C.c_uint64()
        _check(self._f("q51_lanes_quant_offset")(C.c_uint32(columns), C.c_uint32(block), C.c_uint32(index), C.byref(o)))
        return o.value

    def q51_lanes_pack_rows(self, columns, original):
        original = _u8(original)
        out = np.empty_like(original)
        _check(self._f("q51_lanes_pack_rows")(C.c_uint32(columns), _p(original, _u8p), _p(out, _u8p), C.c_uint64(original.size)))
        return out

    def q51_lanes_unpack_rows(self, columns, packed):
        packed = _u8(packed)
        out = np.empty_like(packed)
        _check(self._f("q51_lanes_unpack_rows")(C.c_uint32(columns), _p(packed, _u8p), _p(out, _u8p), C.c_uint64(packed.size)))
        return out

    # ---- top-k ----
    def logit_topk_row(self, logits):
        logits = np.ascontiguousarray(logits, dtype=np.float32)
        row = TopKRow()
        name = "logit_topk_row_cpu" if self.prefix == "orc_" else "logit_topk_row"
        _check(self._f(name)(_p(logits, _f32p), C.c_uint64(logits.size), C.byref(row)))
        return row

    # ---- plans ----
    def grouped_mm_plan(self, t, layout, columns, rows, experts, selected, tokens, in_stride, out_stride, broadcast, allow_2k=False):
        p = GroupedMmPlan()
        name = "grouped_mm_plan_make" if self.prefix == "orc_" else "grouped_mm_plan"
        _check(self._f(name)(C.c_uint32(t), C.c_uint32(layout), C.c_uint32(columns), C.c_uint32(rows), C.c_uint32(experts),
                             C.c_uint32(selected), C.c_uint32(tokens), C.c_uint64(in_stride), C.c_uint64(out_stride),
                             C.c_int(bool(broadcast)), C.c_int(bool(allow_2k)), C.byref(p)))
        return p

    def moe_mm_many_bytes(self, channels, hidden, experts, selected, capacity, allow_2k=False):
        views = (C.c_uint64 * 13)()
        total = C.c_uint64()
        _check(self._f("moe_mm_many_bytes")(C.c_uint32(channels), C.c_uint32(hidden), C.c_uint32(experts), C.c_uint32(selected),
                                           C.c_uint32(capacity), C.c_int(bool(allow_2k)), views, C.byref(total)))
        return list(views), total.value


class Oracle(_Lib):
    """The C restatement; adds the functions the reference only states as specifications or tests."""

    def __init__(self, path):
        super().__init__(path, "orc_")
        self.dll.orc_bf16_to_f32.restype = C.c_float
        self.dll.orc_bf16_to_f32.argtypes = [C.c_uint16]
        self.dll.orc_round_bf16_bits.restype = C.c_uint16
        self.dll.orc_round_bf16_bits.argtypes = [C.c_float, _u32p]

    def value(self, t, block, index):
        block = _u8(block)
        out = C.c_double()
        _check(self.dll.orc_value(C.c_uint32(t), _p(block, _u8p), C.c_uint32(index), C.byref(out)))
        return out.value

    def reference_gemv_mt(self, t, matrix, columns, rows, x, threads):
        matrix = _u8(matrix)
        x = np.ascontiguousarray(x, dtype=np.float32)
        y = np.empty(rows, dtype=np.float64)
        _check(self.dll.orc_reference_gemv_mt(C.c_uint32(t), _p(matrix, _u8p), C.c_uint64(matrix.size), C.c_uint32(columns),
                                              C.c_uint32(rows), _p(x, _f32p), C.c_uint64(x.size), _p(y, _f64p), C.c_uint32(threads)))
        return y

    def make_expert_spec(self, source_type, columns, rows):
        s = PlanarSpec()
        _check(self.dll.orc_make_expert_spec(C.c_uint32(source_type), C.c_uint32(columns), C.c_uint32(rows), C.byref(s)))
        return s

    def pack_sm16(self, s12):
        s12 = _u8(s12)
        assert s12.size == 12
        out = np.empty(16, dtype=np.uint8)
        self.dll.orc_pack_sm16(_p(s12, _u8p), _p(out, _u8p))
        return out

    def unpack_sm16(self, sm):
        sm = _u8(sm)
        assert sm.size == 16
        out = np.empty(12, dtype=np.uint8)
        _check(self.dll.orc_unpack_sm16(_p(sm, _u8p), _p(out, _u8p)))
        return out

    def pack_expert(self, spec, gguf):
        gguf = _u8(gguf)
        out = np.zeros(spec.planar_expert_bytes, dtype=np.uint8)
        _check(self.dll.orc_pack_expert_planar_v3(C.byref(spec), _p(gguf, _u8p), C.c_uint64(gguf.size), _p(out, _u8p), C.c_uint64(out.size)))
        return out

    def unpack_expert(self, spec, planar):
        planar = _u8(planar)
        out = np.zeros(spec.source_expert_bytes, dtype=np.uint8)
        _check(self.dll.orc_unpack_expert_planar_v3(C.byref(spec), _p(planar, _u8p), C.c_uint64(planar.size), _p(out, _u8p), C.c_uint64(out.size)))
        return out

    def dequantize_expert_planar(self, spec, planar, f32=False):
        planar = _u8(planar)
        n = spec.rows * spec.columns
        out = np.empty(n, dtype=np.float32)
        fn = self.dll.orc_dequantize_expert_planar_v3_f32 if f32 else self.dll.orc_dequantize_expert_planar_v3
        _check(fn(C.byref(spec), _p(planar, _u8p), C.c_uint64(planar.size), _p(out, _f32p), C.c_uint64(n)))
        return out

    def pack_coloc_half(self, spec, gate, up, experts, half):
        gate, up = _u8(gate), _u8(up)
        out = np.zeros((experts // 2) * 2 * spec.planar_expert_bytes, dtype=np.uint8)
        _check(self.dll.orc_pack_coloc_half(C.byref(spec), _p(gate, _u8p), _p(up, _u8p), C.c_uint32(experts), C.c_uint32(half),
                                            _p(out, _u8p), C.c_uint64(out.size)))
        return out

    def grouped_routes(self, ids, experts, selected, tokens):
        ids = np.ascontiguousarray(ids, dtype=np.uint32)
        token_map = np.full(experts * tokens, 0xdeadbeef, dtype=np.uint32)
        counts = np.zeros(experts, dtype=np.uint32)
        err = C.c_uint32(0)
        _check(self.dll.orc_grouped_routes(_p(ids, _u32p), C.c_uint32(experts), C.c_uint32(selected), C.c_uint32(tokens),
                                           _p(token_map, _u32p), _p(counts, _u32p), C.byref(err)))
        return token_map, counts, err.value

    def grouped_tasks(self, counts, experts, selected, tokens, tile=32):
        counts = np.ascontiguousarray(counts, dtype=np.uint32)
        bound = tokens * selected // tile + experts
        tasks = np.zeros(2 + 2 * bound, dtype=np.uint32)
        err = C.c_uint32(0)
        _check(self.dll.orc_grouped_tasks(_p(counts, _u32p), C.c_uint32(experts), C.c_uint32(selected), C.c_uint32(tokens),
                                          C.c_uint32(tile), _p(tasks, _u32p), C.byref(err)))
        return tasks, err.value

    def union_metadata(self, experts, selected, tokens, hidden, channels, ids, poison=0xbaadf00d):
        ids = np.ascontiguousarray(ids, dtype=np.uint32)
        meta = np.full(2320, poison, dtype=np.uint32)
        err = C.c_uint32(0)
        _check(self.dll.orc_union_metadata(C.c_uint32(experts), C.c_uint32(selected), C.c_uint32(tokens), C.c_uint32(hidden),
                                           C.c_uint32(channels), _p(ids, _u32p), _p(meta, _u32p), C.byref(err)))
        return meta, err.value

    def round_bf16(self, a):
        """RNE bf16 rounding of finite floats, returned as float32 (vectorised numpy restatement is checked against the C one in tests)."""
        a = np.ascontiguousarray(a, dtype=np.float32)
        bits = a.view(np.uint32).astype(np.uint64)
        r = ((bits + 0x7fff + ((bits >> 16) & 1)) >> 16).astype(np.uint32) << 16
        return r.astype(np.uint32).view(np.float32).reshape(a.shape)

    def round_bf16_bits_scalar(self, v):
        bad = C.c_uint32(0)
        return int(self.dll.orc_round_bf16_bits(C.c_float(v), C.byref(bad))), bad.value

    def round_f16(self, a):
        """float32 -> float16 (RNE) -> float32, element-wise through the C routine."""
        a = np.ascontiguousarray(a, dtype=np.float32)
        out = np.empty_like(a)
        f = self.dll.orc_round_f16
        f.restype, f.argtypes = C.c_float, [C.c_float]
        flat_in, flat_out = a.reshape(-1), out.reshape(-1)
        for i in range(flat_in.size):
            flat_out[i] = f(float(flat_in[i]))
        return out

    def staged_gemm(self, t, matrix, columns, x, rows_sel=None, nrows=None, stage_f16=True, threads=8):
        """out[m][i] = sum_k stage(dec(W[rows_sel[i], k])) * x[m, k] in double; x is [tokens, columns] float32.
        stage_f16: False/0 none, True/1 round weights to half, 2 Q6_K integer products as half (scale d kept f32)."""
        matrix = _u8(matrix)
        x = np.ascontiguousarray(x, dtype=np.float32)
        sel = None if rows_sel is None else np.ascontiguousarray(rows_sel, dtype=np.uint32)
        nsel = int(sel.size) if sel is not None else int(nrows)
        out = np.empty((x.shape[0], nsel), dtype=np.float64)
        _check(self.dll.orc_staged_gemm(C.c_uint32(t), _p(matrix, _u8p), C.c_uint32(columns), _p(sel, _u32p) if sel is not None else None,
                                        C.c_uint32(nsel), _p(x, _f32p), C.c_uint64(x.shape[1]), C.c_uint32(x.shape[0]), C.c_int(int(stage_f16)),
                                        _p(out, _f64p), C.c_uint32(threads)))
        return out

    def fixture_weights(self, t, k, r, e):
        epb, bpb = self.encoding(t)
        out = np.empty((k // epb) * bpb * r * e, dtype=np.uint8)
        _check(self.dll.orc_fixture_weights(C.c_uint32(t), C.c_uint32(k), C.c_uint32(r), C.c_uint32(e), _p(out, _u8p), C.c_uint64(out.size)))
        return out

    def moe_routed_reference(self, gu_type, dn_type, gate, up, down, channels, hidden, experts, ids, tokens, selected, x,
                             silu_f32=True, stage=0, threads=1, want_down=True):
        gate, up = _u8(gate), _u8(up)
        down = _u8(down) if down is not None else None
        ids = np.ascontiguousarray(ids, dtype=np.uint32)
        x = np.ascontiguousarray(x, dtype=np.float32)
        routes = tokens * selected
        h = np.empty((routes, hidden), dtype=np.float64)
        y = np.empty((routes, channels), dtype=np.float64) if (want_down and down is not None) else None
        _check(self.dll.orc_moe_routed_reference(
            C.c_uint32(gu_type), C.c_uint32(dn_type), _p(gate, _u8p), _p(up, _u8p), _p(down, _u8p) if down is not None else None,
            C.c_uint32(channels), C.c_uint32(hidden), C.c_uint32(experts), _p(ids, _u32p), C.c_uint32(tokens), C.c_uint32(selected),
            _p(x, _f32p), C.c_uint64(x.shape[-1] if x.ndim > 1 else channels), C.c_int(bool(silu_f32)), C.c_int(int(stage)),
            _p(h, _f64p), _p(y, _f64p) if y is not None else None, C.c_uint32(threads)))
        return h, y


_lib = None
_ref = False


def build():
    """Compile liboracle.so (and oracle/_ref when the reference tree is present)."""
    import subprocess
    subprocess.run(["make", "-C", _HERE, "all"], check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)


def lib():
    global _lib
    if _lib is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        _lib = Oracle(path)
    return _lib


def ref():
    """The reference's own CPU code, or None when oracle/_ref has not been built."""
    global _ref
    if _ref is False:
        path = os.path.join(_HERE, "_ref", "libtokspur_ref.so")
        _ref = _Lib(path, "ref_") if os.path.exists(path) else None
    return _ref

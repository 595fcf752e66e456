"""ctypes binding of the C ABI in include/tokspur_hip.h.

The library must have been built (python -m build step or __graft_entry__.build()); loading fails
loudly when libtokspur_hip.so is missing — there is no fallback path of any kind. `Device` wraps
torch tensors as device buffers and calls every device entry point on torch's current stream.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libtokspur_hip.so")

OK, ERR_FORMAT, ERR_HIP = 0, 1, 2
ERRBIT_NONFINITE, ERRBIT_INDEX = 1, 4
LAYOUT_GGUF, LAYOUT_Q8_LANES_V1, LAYOUT_Q51_LANES_V1, LAYOUT_PLANAR_V3 = 0, 1, 2, 3
u8p = C.POINTER(C.c_uint8)


class FormatError(RuntimeError):
    """A host-side refusal: what the engine reports as tokspur::FormatError."""


class HipError(RuntimeError):
    pass


class PlanarSpec(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("source_type", "columns", "rows", "blocks_per_row")] + \
               [(n, C.c_uint64) for n in ("source_row_bytes", "planar_row_bytes", "source_expert_bytes",
                                          "planar_expert_bytes", "qs_offset", "qh_offset", "sm_offset", "dm_offset")]


class GroupedMmPlan(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("columns", "rows", "row_bytes", "experts", "selected", "tokens",
                                          "broadcast", "maximum_tasks")] + \
               [(n, C.c_uint64) for n in ("expert_stride_bytes", "input_stride_bytes", "output_stride_bytes",
                                          "matrix_bytes", "indices_bytes", "input_bytes", "output_bytes",
                                          "token_map_bytes", "counts_bytes", "tasks_bytes")] + \
               [("grid_x", C.c_uint32), ("grid_y", C.c_uint32)]


_dll = None


def dll():
    global _dll
    if _dll is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with __graft_entry__.build() — there is no fallback")
        _dll = C.CDLL(LIB_PATH)
        _dll.tsp_last_error.restype = C.c_char_p
        _dll.tsp_abi_version.restype = C.c_uint32
    return _dll


def check(status):
    if status == OK:
        return
    message = dll().tsp_last_error().decode()
    raise (FormatError if status == ERR_FORMAT else HipError)(message)


def _np_u8(a):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.uint8
    return a


# ------------------------------------------------------------------ host functions

def encoding(t):
    e, b = C.c_uint32(), C.c_uint32()
    check(dll().tsp_encoding(C.c_uint32(t), C.byref(e), C.byref(b)))
    return e.value, b.value


def make_expert_spec(source_type, columns, rows):
    s = PlanarSpec()
    check(dll().tsp_make_expert_spec(C.c_uint32(source_type), C.c_uint32(columns), C.c_uint32(rows), C.byref(s)))
    return s


def pack_sm16(s12):
    s12 = _np_u8(s12)
    out = np.empty(16, dtype=np.uint8)
    dll().tsp_pack_sm16(s12.ctypes.data_as(u8p), out.ctypes.data_as(u8p))
    return out


def unpack_sm16(sm):
    sm = _np_u8(sm)
    out = np.empty(12, dtype=np.uint8)
    check(dll().tsp_unpack_sm16(sm.ctypes.data_as(u8p), out.ctypes.data_as(u8p)))
    return out


def pack_expert(spec, gguf):
    gguf = _np_u8(gguf)
    out = np.zeros(spec.planar_expert_bytes, dtype=np.uint8)
    check(dll().tsp_pack_expert_planar_v3(C.byref(spec), gguf.ctypes.data_as(u8p), C.c_uint64(gguf.size),
                                          out.ctypes.data_as(u8p), C.c_uint64(out.size)))
    return out


def unpack_expert(spec, planar):
    planar = _np_u8(planar)
    out = np.zeros(spec.source_expert_bytes, dtype=np.uint8)
    check(dll().tsp_unpack_expert_planar_v3(C.byref(spec), planar.ctypes.data_as(u8p), C.c_uint64(planar.size),
                                            out.ctypes.data_as(u8p), C.c_uint64(out.size)))
    return out


def pack_experts(spec, gguf_stack, experts):
    """[experts] contiguous planar experts (the layout of a down-projection tensor)."""
    gguf_stack = _np_u8(gguf_stack)
    sb = spec.source_expert_bytes
    return np.concatenate([pack_expert(spec, gguf_stack[e * sb:(e + 1) * sb]) for e in range(experts)])


def pack_coloc_half(spec, gate, up, experts, half):
    gate, up = _np_u8(gate), _np_u8(up)
    out = np.zeros((experts // 2) * 2 * spec.planar_expert_bytes, dtype=np.uint8)
    check(dll().tsp_pack_coloc_half(C.byref(spec), gate.ctypes.data_as(u8p), up.ctypes.data_as(u8p), C.c_uint32(experts),
                                    C.c_uint32(half), out.ctypes.data_as(u8p), C.c_uint64(out.size)))
    return out


def q8_lanes_quant_offset(columns, block, index):
    o = C.c_uint64()
    check(dll().tsp_q8_lanes_quant_offset(C.c_uint32(columns), C.c_uint32(block), C.c_uint32(index), C.byref(o)))
    return o.value


def q8_lanes_pack_rows(columns, original):
    original = _np_u8(original)
    out = np.empty_like(original)
    check(dll().tsp_q8_lanes_pack_rows(C.c_uint32(columns), original.ctypes.data_as(u8p), out.ctypes.data_as(u8p), C.c_uint64(original.size)))
    return out


def q51_lanes_quant_offset(columns, block, index):
    o = C.c_uint64()
    check(dll().tsp_q51_lanes_quant_offset(C.c_uint32(columns), C.c_uint32(block), C.c_uint32(index), C.byref(o)))
    return o.value


def q51_lanes_pack_rows(columns, original):
    original = _np_u8(original)
    out = np.empty_like(original)
    check(dll().tsp_q51_lanes_pack_rows(C.c_uint32(columns), original.ctypes.data_as(u8p), out.ctypes.data_as(u8p), C.c_uint64(original.size)))
    return out


def q51_lanes_unpack_rows(columns, packed):
    packed = _np_u8(packed)
    out = np.empty_like(packed)
    check(dll().tsp_q51_lanes_unpack_rows(C.c_uint32(columns), packed.ctypes.data_as(u8p), out.ctypes.data_as(u8p), C.c_uint64(packed.size)))
    return out


def q8_lanes_unpack_rows(columns, packed):
    packed = _np_u8(packed)
    out = np.empty_like(packed)
    check(dll().tsp_q8_lanes_unpack_rows(C.c_uint32(columns), packed.ctypes.data_as(u8p), out.ctypes.data_as(u8p), C.c_uint64(packed.size)))
    return out


def grouped_mm_plan(t, layout, columns, rows, experts, selected, tokens, in_stride, out_stride, broadcast, allow_2k=False):
    p = GroupedMmPlan()
    check(dll().tsp_grouped_mm_plan(C.c_uint32(t), C.c_uint32(layout), C.c_uint32(columns), C.c_uint32(rows), C.c_uint32(experts),
                                    C.c_uint32(selected), C.c_uint32(tokens), C.c_uint64(in_stride), C.c_uint64(out_stride),
                                    C.c_int(bool(broadcast)), C.c_int(bool(allow_2k)), C.byref(p)))
    return p


def dense_mm_q8_plan(layout, columns, rows, tokens, in_stride, out_stride, allow_2k=False):
    p = GroupedMmPlan()
    check(dll().tsp_dense_mm_q8_plan(C.c_uint32(layout), C.c_uint32(columns), C.c_uint32(rows), C.c_uint32(tokens),
                                     C.c_uint64(in_stride), C.c_uint64(out_stride), C.c_int(bool(allow_2k)), C.byref(p)))
    return p


def moe_mm_many_bytes(channels, hidden, experts, selected, capacity, allow_2k=False):
    views = (C.c_uint64 * 13)()
    total = C.c_uint64()
    check(dll().tsp_moe_mm_many_bytes(C.c_uint32(channels), C.c_uint32(hidden), C.c_uint32(experts), C.c_uint32(selected),
                                      C.c_uint32(capacity), C.c_int(bool(allow_2k)), views, C.byref(total)))
    return list(views), total.value


def q8_many_width(remaining):
    w = C.c_uint32()
    check(dll().tsp_q8_many_width(C.c_uint32(remaining), C.byref(w)))
    return w.value


def q8_many_chunks(rows):
    w = C.c_uint32()
    check(dll().tsp_q8_many_chunks(C.c_uint32(rows), C.byref(w)))
    return w.value


# ------------------------------------------------------------------ device side

class Device:
    """Device buffers are torch tensors on cuda:0; kernels run on torch's current stream."""

    def __init__(self):
        import torch
        self.torch = torch
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU: the HIP path cannot run and there is no CPU fallback")
        self.dev = torch.device("cuda", torch.cuda.current_device())
        self.err = torch.zeros(1, dtype=torch.int32, device=self.dev)
        dll()

    # -- memory
    def upload(self, a):
        a = np.ascontiguousarray(a)
        if a.dtype == np.uint32:
            return self.torch.from_numpy(a.view(np.int32)).to(self.dev)
        if a.dtype == np.uint16:
            return self.torch.from_numpy(a.view(np.int16)).to(self.dev)
        return self.torch.from_numpy(a).to(self.dev)

    def empty(self, shape, dtype="float32"):
        return self.torch.empty(shape, dtype=getattr(self.torch, dtype), device=self.dev)

    def zeros(self, shape, dtype="float32"):
        return self.torch.zeros(shape, dtype=getattr(self.torch, dtype), device=self.dev)

    def full(self, shape, value, dtype="float32"):
        shape = tuple(shape) if isinstance(shape, (tuple, list)) else (int(shape),)
        value = value.item() if hasattr(value, "item") else value
        return self.torch.full(shape, value, dtype=getattr(self.torch, dtype), device=self.dev)

    @staticmethod
    def ptr(t):
        return C.c_void_p(t.data_ptr()) if t is not None else None

    @staticmethod
    def nbytes(t):
        return t.numel() * t.element_size()

    def stream(self):
        return C.c_void_p(self.torch.cuda.current_stream().cuda_stream)

    def sync(self):
        self.torch.cuda.synchronize()

    def clear_error(self):
        self.err.zero_()

    def error(self):
        """Reads and clears the sticky error word (synchronises)."""
        value = int(self.err.item()) & 0xFFFFFFFF
        self.err.zero_()
        return value

    # -- operators
    def dequantize(self, t, blocks, nelem):
        out = self.empty(nelem)
        check(dll().tsp_dequantize(C.c_uint32(t), self.ptr(blocks), C.c_uint64(self.nbytes(blocks)), self.ptr(out),
                                   C.c_uint64(nelem), self.ptr(self.err), self.stream()))
        return out

    def dequantize_planar(self, spec, planar):
        out = self.empty(spec.rows * spec.columns)
        check(dll().tsp_dequantize_planar(C.byref(spec), self.ptr(planar), self.ptr(out), self.ptr(self.err), self.stream()))
        return out

    def gemv(self, t, matrix, x, columns, rows, layout=LAYOUT_GGUF, y=None, matrix_bytes=None):
        y = self.empty(rows) if y is None else y
        nbytes = self.nbytes(matrix) if matrix_bytes is None else matrix_bytes
        check(dll().tsp_gemv(C.c_uint32(t), C.c_uint32(layout), self.ptr(matrix), C.c_uint64(nbytes), self.ptr(x), self.ptr(y),
                             C.c_uint32(columns), C.c_uint32(rows), self.ptr(self.err), self.stream()))
        return y

    def gemv_rows(self, t, matrix, x, y, count, columns, rows, x_stride, y_stride, layout=LAYOUT_GGUF):
        check(dll().tsp_gemv_rows(C.c_uint32(t), C.c_uint32(layout), self.ptr(matrix), C.c_uint64(self.nbytes(matrix)), self.ptr(x),
                                  C.c_uint64(x_stride), self.ptr(y), C.c_uint64(y_stride), C.c_uint32(count), C.c_uint32(columns),
                                  C.c_uint32(rows), self.ptr(self.err), self.stream()))
        return y

    def q8_matvec_many(self, matrix, x, columns, rows, width, layout=LAYOUT_GGUF, y=None):
        y = self.empty((width, rows)) if y is None else y
        check(dll().tsp_q8_matvec_many(C.c_uint32(layout), self.ptr(matrix), C.c_uint64(self.nbytes(matrix)), self.ptr(x), self.ptr(y),
                                       C.c_uint32(columns), C.c_uint32(rows), C.c_uint32(width), self.ptr(self.err), self.stream()))
        return y

    def routed_gemv(self, t, matrices, ids, x, columns, rows, experts, selected, broadcast):
        y = self.empty((selected, rows))
        check(dll().tsp_routed_gemv(C.c_uint32(t), self.ptr(matrices), C.c_uint64(self.nbytes(matrices)), self.ptr(ids), self.ptr(x),
                                    self.ptr(y), C.c_uint32(columns), C.c_uint32(rows), C.c_uint32(experts), C.c_uint32(selected),
                                    C.c_int(bool(broadcast)), self.ptr(self.err), self.stream()))
        return y

    def router_f32_batch(self, weights, x, tokens, columns, experts, x_stride=None, out=None, out_stride=None):
        """logits[t, e] = sum_k weights[e, k] * x[t, k] for a whole chunk of token rows in one f32 GEMM."""
        out = self.empty((tokens, experts)) if out is None else out
        check(dll().tsp_router_f32_batch(self.ptr(weights), self.ptr(x), C.c_uint64(columns * 4 if x_stride is None else x_stride),
                                         self.ptr(out), C.c_uint64(experts * 4 if out_stride is None else out_stride), C.c_uint32(columns),
                                         C.c_uint32(experts), C.c_uint32(tokens), self.ptr(self.err), self.stream()))
        return out

    def route(self, logits, selected, mode=0, normalize=True, tokens=None, out=None):
        """logits [experts] (tokens=None: the single-row operator) or [tokens, experts]."""
        experts = logits.shape[-1]
        n = 1 if tokens is None else tokens
        ids, w = out if out is not None else (self.zeros((n, selected), "int32"), self.zeros((n, selected)))
        if tokens is None:
            check(dll().tsp_route(self.ptr(logits), self.ptr(ids), self.ptr(w), C.c_uint32(experts), C.c_uint32(selected), C.c_uint32(mode),
                                  C.c_int(bool(normalize)), self.ptr(self.err), self.stream()))
        else:
            check(dll().tsp_route_batch(self.ptr(logits), self.ptr(ids), self.ptr(w), C.c_uint32(experts), C.c_uint32(selected),
                                        C.c_uint32(tokens), C.c_uint32(mode), C.c_int(bool(normalize)), self.ptr(self.err), self.stream()))
        return ids, w

    def mixture(self, expert_out, weights, shared, shared_logit, channels, selected, tokens=1, out=None, out_stride=None):
        out = self.empty((tokens, channels)) if out is None else out
        stride = channels * 4 if out_stride is None else out_stride
        check(dll().tsp_mixture_batch(self.ptr(expert_out), self.ptr(weights), self.ptr(shared), self.ptr(shared_logit), self.ptr(out),
                                      C.c_uint64(stride), C.c_uint32(channels), C.c_uint32(selected), C.c_uint32(tokens),
                                      self.ptr(self.err), self.stream()))
        return out

    def swiglu(self, gate, up, scale=1.0, out=None):
        out = self.empty(gate.shape) if out is None else out
        check(dll().tsp_swiglu(self.ptr(gate), self.ptr(up), self.ptr(out), C.c_uint64(gate.numel()), C.c_float(scale),
                               self.ptr(self.err), self.stream()))
        return out

    def rms(self, x, gains, group_width, epsilon, gate=None, out=None):
        out = self.empty(x.shape) if out is None else out
        shared = int(gains.numel() == group_width and x.numel() != group_width)
        if gate is None:
            check(dll().tsp_rms(self.ptr(x), self.ptr(gains), self.ptr(out), C.c_uint64(x.numel()), C.c_uint32(group_width), C.c_int(shared),
                                C.c_float(epsilon), self.ptr(self.err), self.stream()))
        else:
            check(dll().tsp_rms_sigmoid_gate(self.ptr(x), self.ptr(gains), self.ptr(gate), self.ptr(out), C.c_uint64(x.numel()), C.c_uint32(group_width),
                                             C.c_int(shared), C.c_float(epsilon), self.ptr(self.err), self.stream()))
        return out

    def activate(self, x, kind, scale=1.0, out=None):
        out = self.empty(x.shape) if out is None else out
        check(dll().tsp_activate(self.ptr(x), self.ptr(out), C.c_uint64(x.numel()), C.c_uint32(kind), C.c_float(scale), self.ptr(self.err), self.stream()))
        return out

    def multiply(self, x, gate, sigmoid_gate=False, out=None):
        out = self.empty(x.shape) if out is None else out
        check(dll().tsp_multiply(self.ptr(x), self.ptr(gate), self.ptr(out), C.c_uint64(x.numel()), C.c_int(bool(sigmoid_gate)), self.ptr(self.err), self.stream()))
        return out

    def residual_read(self, normalized, scores, inject, branches, channels, out=None, scales=None):
        out = self.empty(channels) if out is None else out
        scales = self.empty(branches) if scales is None else scales
        check(dll().tsp_residual_read(self.ptr(normalized), self.ptr(scores), self.ptr(inject), self.ptr(out), self.ptr(scales), C.c_uint32(branches),
                                      C.c_uint32(channels), self.ptr(self.err), self.stream()))
        return out, scales

    def residual_write(self, streams, x, scales, branches, channels, out=None):
        out = self.empty(streams.shape) if out is None else out
        check(dll().tsp_residual_write(self.ptr(streams), self.ptr(x), self.ptr(scales), self.ptr(out), C.c_uint32(branches), C.c_uint32(channels),
                                       self.ptr(self.err), self.stream()))
        return out

    def grouped_routes(self, ids, experts, selected, tokens, fill=0xDEADBEEF):
        token_map = self.full((experts, tokens), np.int32(np.uint32(fill).view(np.int32)), "int32")
        counts = self.zeros(experts, "int32")
        check(dll().tsp_grouped_routes(self.ptr(ids), self.ptr(token_map), self.ptr(counts), C.c_uint32(experts), C.c_uint32(selected),
                                       C.c_uint32(tokens), self.ptr(self.err), self.stream()))
        return token_map, counts

    def grouped_tasks(self, counts, experts, selected, tokens, tile=32):
        bound = tokens * selected // tile + experts
        tasks = self.zeros(2 + 2 * bound, "int32")
        check(dll().tsp_grouped_tasks(self.ptr(counts), self.ptr(tasks), C.c_uint32(experts), C.c_uint32(selected), C.c_uint32(tokens),
                                      C.c_uint32(tile), self.ptr(self.err), self.stream()))
        return tasks

    def union_build(self, ids, experts, selected, tokens, hidden, channels, poison=0xBAADF00D):
        meta = self.full(2320, np.int32(np.uint32(poison).view(np.int32)), "int32")
        check(dll().tsp_planar_union_build(self.ptr(ids), self.ptr(meta), C.c_uint32(experts), C.c_uint32(selected), C.c_uint32(tokens),
                                           C.c_uint32(hidden), C.c_uint32(channels), self.ptr(self.err), self.stream()))
        return meta


class SmallMoe(C.Structure):
    _fields_ = [("pair_lo", C.c_void_p), ("pair_hi", C.c_void_p), ("down", C.c_void_p),
                ("gate_kind", C.c_uint32), ("up_kind", C.c_uint32), ("down_kind", C.c_uint32),
                ("channels", C.c_uint32), ("hidden", C.c_uint32), ("experts", C.c_uint32), ("selected", C.c_uint32),
                ("tokens", C.c_uint32), ("ids", C.c_void_p), ("x", C.c_void_p), ("x_stride_bytes", C.c_uint64),
                ("h", C.c_void_p), ("h_stride_bytes", C.c_uint64), ("y", C.c_void_p), ("y_stride_bytes", C.c_uint64),
                ("union_meta", C.c_void_p), ("error_word", C.c_void_p)]


COLOC_KINDS = {12: (2, 3), 13: (4, 5), 8: (6, 7)}
DOWN_KINDS = {7: 8, 8: 9, 14: 10}


class PlanarMoeWeights:
    """Device-resident planar v3 expert tensors of one MoE sublayer: pair_lo / pair_hi (co-located
    gate/up halves) and the [experts] down tensor, built from raw GGUF expert stacks on the host."""

    def __init__(self, dev, gu_type, dn_type, channels, hidden, experts, gate_raw, up_raw, down_raw):
        self.gu_type, self.dn_type = gu_type, dn_type
        self.channels, self.hidden, self.experts = channels, hidden, experts
        self.gu_spec = make_expert_spec(gu_type, channels, hidden)
        self.dn_spec = make_expert_spec(dn_type, hidden, channels)
        self.pair_lo = dev.upload(pack_coloc_half(self.gu_spec, gate_raw, up_raw, experts, 0))
        self.pair_hi = dev.upload(pack_coloc_half(self.gu_spec, gate_raw, up_raw, experts, 1))
        self.down = dev.upload(pack_experts(self.dn_spec, down_raw, experts))
        self.union_meta = dev.zeros(2320, "int32")


def _small_moe(dev, w, ids, x, tokens, selected, h, y, x_stride=None, h_stride=None, y_stride=None):
    gate_kind, up_kind = COLOC_KINDS[w.gu_type]
    m = SmallMoe(w.pair_lo.data_ptr(), w.pair_hi.data_ptr(), w.down.data_ptr() if y is not None else None,
                 gate_kind, up_kind, DOWN_KINDS[w.dn_type], w.channels, w.hidden, w.experts, selected, tokens,
                 ids.data_ptr(), x.data_ptr(), w.channels * 4 if x_stride is None else x_stride,
                 h.data_ptr(), w.hidden * 4 if h_stride is None else h_stride,
                 y.data_ptr() if y is not None else None, w.channels * 4 if y_stride is None else y_stride,
                 w.union_meta.data_ptr(), dev.err.data_ptr())
    return m


def planar_moe_gate_up_swiglu_m8(dev, w, ids, x, tokens, selected, h=None, **strides):
    h = dev.empty((tokens * selected, w.hidden)) if h is None else h
    m = _small_moe(dev, w, ids, x, tokens, selected, h, None, **strides)
    check(dll().tsp_planar_moe_gate_up_swiglu_m8(C.byref(m), dev.stream()))
    return h


class SharedRows(C.Structure):
    _fields_ = [("gate", C.c_void_p), ("up", C.c_void_p), ("down", C.c_void_p), ("h", C.c_void_p), ("h_stride_bytes", C.c_uint64),
                ("y", C.c_void_p), ("y_stride_bytes", C.c_uint64)]


def planar_moe_routed_m8(dev, w, ids, x, tokens, selected, h=None, y=None, shared=None, shared_h=None, shared_y=None, shared_y_stride=None,
                         **strides):
    """`planar_moe_routed_m8`; with `shared` (a PlanarSharedExpert) the always-on expert rides in the same launches and
    its rows [tokens, channels] come back as the third result."""
    h = dev.empty((tokens * selected, w.hidden)) if h is None else h
    y = dev.empty((tokens * selected, w.channels)) if y is None else y
    m = _small_moe(dev, w, ids, x, tokens, selected, h, y, **strides)
    if shared is None:
        check(dll().tsp_planar_moe_routed_m8(C.byref(m), dev.stream()))
        return h, y
    shared_h = dev.empty((tokens, w.hidden)) if shared_h is None else shared_h
    shared_y = dev.empty((tokens, w.channels)) if shared_y is None else shared_y
    e = SharedRows(shared.gate.data_ptr(), shared.up.data_ptr(), shared.down.data_ptr(), shared_h.data_ptr(), w.hidden * 4,
                   shared_y.data_ptr(), w.channels * 4 if shared_y_stride is None else shared_y_stride)
    check(dll().tsp_planar_moe_routed_m8_shared(C.byref(m), C.byref(e), dev.stream()))
    return h, y, shared_y


class GroupedMoe(C.Structure):
    _fields_ = [("pair_lo", C.c_void_p), ("pair_hi", C.c_void_p), ("down", C.c_void_p),
                ("gate_kind", C.c_uint32), ("up_kind", C.c_uint32), ("down_kind", C.c_uint32),
                ("channels", C.c_uint32), ("hidden", C.c_uint32), ("experts", C.c_uint32), ("selected", C.c_uint32),
                ("tokens", C.c_uint32), ("ids", C.c_void_p), ("x", C.c_void_p), ("x_stride_bytes", C.c_uint64),
                ("y", C.c_void_p), ("y_stride_bytes", C.c_uint64), ("token_map", C.c_void_p), ("counts", C.c_void_p),
                ("tasks", C.c_void_p), ("workspace", C.c_void_p), ("workspace_bytes", C.c_uint64), ("error_word", C.c_void_p)]


def dense_mm_q8(dev, layout, matrix, x, tokens, columns, rows, out=None, x_stride=None, out_stride=None):
    """Dense Q8_0 GEMM (`dense_mm_q8`): out[t] = W x[t], GGUF rows or q8_lanes_v1 rows, f32 rows with byte strides."""
    out = dev.empty((tokens, rows)) if out is None else out
    check(dll().tsp_dense_mm_q8(C.c_uint32(layout), dev.ptr(matrix), C.c_uint64(dev.nbytes(matrix)), dev.ptr(x),
                                C.c_uint64(columns * 4 if x_stride is None else x_stride), dev.ptr(out),
                                C.c_uint64(rows * 4 if out_stride is None else out_stride), C.c_uint32(tokens), C.c_uint32(columns),
                                C.c_uint32(rows), dev.ptr(dev.err), dev.stream()))
    return out


def dense_mm_q8_workspace_bytes(tokens, columns, rows):
    f = dll().tsp_dense_mm_q8_workspace_bytes
    f.restype = C.c_uint64
    return f(C.c_uint32(tokens), C.c_uint32(columns), C.c_uint32(rows))


def dense_mm_q8_staged(dev, layout, matrix, x, tokens, columns, rows, out=None, x_stride=None, out_stride=None, workspace=None):
    """Dense Q8_0 GEMM for many rows: matrix and rows staged as halves in `workspace`, one matrix-core GEMM."""
    f = dll().tsp_dense_mm_q8_workspace_bytes
    f.restype = C.c_uint64
    out = dev.empty((tokens, rows)) if out is None else out
    workspace = dev.empty(f(C.c_uint32(tokens), C.c_uint32(columns), C.c_uint32(rows)), "uint8") if workspace is None else workspace
    check(dll().tsp_dense_mm_q8_staged(C.c_uint32(layout), dev.ptr(matrix), C.c_uint64(dev.nbytes(matrix)), dev.ptr(x),
                                       C.c_uint64(columns * 4 if x_stride is None else x_stride), dev.ptr(out),
                                       C.c_uint64(rows * 4 if out_stride is None else out_stride), C.c_uint32(tokens), C.c_uint32(columns),
                                       C.c_uint32(rows), dev.ptr(workspace), C.c_uint64(dev.nbytes(workspace)), dev.ptr(dev.err), dev.stream()))
    return out


def dense_mm_workspace_bytes(tokens, columns):
    f = dll().tsp_dense_mm_workspace_bytes
    f.restype = C.c_uint64
    return f(C.c_uint32(tokens), C.c_uint32(columns))


def grouped_mm(dev, encoding, matrices, ids, x, columns, rows, experts, selected, tokens, broadcast, out=None, scratch=None,
               x_stride=None, out_stride=None, layout=LAYOUT_GGUF):
    """Grouped dequant-GEMM over expert stacks (`grouped_mm`): out[rid] = W[ids[rid]] x (x per token when broadcast, else per route)."""
    f = dll().tsp_grouped_mm_workspace_bytes
    f.restype = C.c_uint64
    routes = tokens * selected
    out = dev.empty((routes, rows)) if out is None else out
    if scratch is None:
        scratch = {"token_map": dev.zeros(experts * tokens, "int32"), "counts": dev.zeros(experts, "int32"),
                   "tasks": dev.zeros(2 + 2 * (routes // 32 + experts), "int32"),
                   "workspace": dev.empty(f(C.c_uint32(tokens), C.c_uint32(selected), C.c_uint32(experts), C.c_uint32(columns), C.c_int(bool(broadcast))), "uint8")}
    check(dll().tsp_grouped_mm(C.c_uint32(encoding), C.c_uint32(layout), dev.ptr(matrices), C.c_uint64(dev.nbytes(matrices)), dev.ptr(ids),
                               dev.ptr(x), C.c_uint64(columns * 4 if x_stride is None else x_stride), dev.ptr(out),
                               C.c_uint64(rows * 4 if out_stride is None else out_stride), dev.ptr(scratch["token_map"]), dev.ptr(scratch["counts"]),
                               dev.ptr(scratch["tasks"]), C.c_uint32(columns), C.c_uint32(rows), C.c_uint32(experts), C.c_uint32(selected),
                               C.c_uint32(tokens), C.c_int(bool(broadcast)), dev.ptr(scratch["workspace"]), C.c_uint64(dev.nbytes(scratch["workspace"])),
                               dev.ptr(dev.err), dev.stream()))
    return out, scratch


def planar_nax_workspace_bytes(tokens, selected, experts, channels, hidden):
    f = dll().tsp_planar_nax_workspace_bytes
    f.restype = C.c_uint64
    return f(C.c_uint32(tokens), C.c_uint32(selected), C.c_uint32(experts), C.c_uint32(channels), C.c_uint32(hidden))


def dense_mm(dev, encoding, layout, matrix, x, tokens, columns, rows, out=None, out_bf16=False, workspace=None,
             x_stride=None, out_stride=None):
    """x: f32 or bf16 rows. Returns out rows (f32, or bf16 bits as int16 when out_bf16)."""
    in_bf16 = x.dtype == dev.torch.bfloat16 or x.dtype == dev.torch.int16
    if out is None:
        out = dev.empty((tokens, rows), "int16" if out_bf16 else "float32")
    if workspace is None:
        workspace = dev.empty(dense_mm_workspace_bytes(tokens, columns), "uint8")
    xs = (columns * (2 if in_bf16 else 4)) if x_stride is None else x_stride
    os_ = (rows * (2 if out_bf16 else 4)) if out_stride is None else out_stride
    check(dll().tsp_dense_mm(C.c_uint32(encoding), C.c_uint32(layout), dev.ptr(matrix), C.c_uint64(dev.nbytes(matrix)), dev.ptr(x),
                             C.c_uint64(xs), C.c_int(bool(in_bf16)), dev.ptr(out), C.c_uint64(os_), C.c_int(bool(out_bf16)),
                             C.c_uint32(tokens), C.c_uint32(columns), C.c_uint32(rows), dev.ptr(workspace),
                             C.c_uint64(dev.nbytes(workspace)), dev.ptr(dev.err), dev.stream()))
    return out


class GroupedScratch:
    """Caller-owned outputs and scratch of planar_nax_grouped_moe for a given capacity (with_shared: room for the
    always-on expert's rows as well)."""

    def __init__(self, dev, tokens, selected, experts, channels, hidden, with_shared=False):
        self.token_map = dev.zeros(experts * tokens, "int32")
        self.counts = dev.zeros(experts, "int32")
        self.tasks = dev.zeros(2 + 2 * (tokens * selected // 32 + experts), "int32")
        f = dll().tsp_planar_nax_shared_workspace_bytes
        f.restype = C.c_uint64
        size = (f(C.c_uint32(tokens), C.c_uint32(selected), C.c_uint32(experts), C.c_uint32(channels), C.c_uint32(hidden)) if with_shared
                else planar_nax_workspace_bytes(tokens, selected, experts, channels, hidden))
        self.workspace = dev.empty(size, "uint8")


class SharedExpert(C.Structure):
    _fields_ = [("gate", C.c_void_p), ("up", C.c_void_p), ("down", C.c_void_p), ("y", C.c_void_p), ("y_stride_bytes", C.c_uint64)]


class PlanarSharedExpert:
    """One always-on expert in the routed experts' formats: Q4_K gate and up as one Pack v3 expert each, Q6_K planes down."""

    def __init__(self, dev, channels, hidden, gate_raw, up_raw, down_raw):
        self.channels, self.hidden = channels, hidden
        gu, dn = make_expert_spec(12, channels, hidden), make_expert_spec(14, hidden, channels)
        self.gate, self.up = dev.upload(pack_experts(gu, gate_raw, 1)), dev.upload(pack_experts(gu, up_raw, 1))
        self.down = dev.upload(pack_experts(dn, down_raw, 1))


def planar_nax_grouped_moe(dev, w, ids, x, tokens, selected, scratch, y=None, x_stride=None, y_stride=None, shared=None, shared_y=None,
                           shared_y_stride=None):
    """`planar_nax_grouped_moe`; with `shared` (a PlanarSharedExpert) the always-on expert rides in the same launches and its
    rows come back as the second result."""
    y = dev.empty((tokens * selected, w.channels)) if y is None else y
    gate_kind, up_kind = COLOC_KINDS[w.gu_type]
    m = GroupedMoe(w.pair_lo.data_ptr(), w.pair_hi.data_ptr(), w.down.data_ptr(), gate_kind, up_kind, DOWN_KINDS[w.dn_type],
                   w.channels, w.hidden, w.experts, selected, tokens, ids.data_ptr(), x.data_ptr(),
                   w.channels * 4 if x_stride is None else x_stride, y.data_ptr(), w.channels * 4 if y_stride is None else y_stride,
                   scratch.token_map.data_ptr(), scratch.counts.data_ptr(), scratch.tasks.data_ptr(), scratch.workspace.data_ptr(),
                   dev.nbytes(scratch.workspace), dev.err.data_ptr())
    if shared is None:
        check(dll().tsp_planar_nax_grouped_moe(C.byref(m), dev.stream()))
        return y
    shared_y = dev.empty((tokens, w.channels)) if shared_y is None else shared_y
    e = SharedExpert(shared.gate.data_ptr(), shared.up.data_ptr(), shared.down.data_ptr(), shared_y.data_ptr(),
                     w.channels * 4 if shared_y_stride is None else shared_y_stride)
    check(dll().tsp_planar_nax_grouped_moe_shared(C.byref(m), C.byref(e), dev.stream()))
    return y, shared_y


class KernelTime(C.Structure):
    _fields_ = [("name", C.c_char * 48), ("launches", C.c_uint32), ("total_ms", C.c_float), ("min_ms", C.c_float)]


def profile_begin():
    check(dll().tsp_profile_begin())


def profile_end():
    """{kernel name: (launches, total ms, min ms)} for every launch since profile_begin()."""
    rows = (KernelTime * 64)()
    n = C.c_uint32()
    check(dll().tsp_profile_end(rows, C.c_uint32(64), C.byref(n)))
    return {rows[i].name.decode(): (rows[i].launches, rows[i].total_ms, rows[i].min_ms) for i in range(min(n.value, 64))}


TOPK_ROW_DTYPE = np.dtype([("vocabulary", "<u4"), ("count", "<u4"), ("first_nonfinite_col", "<u4"), ("first_subnormal_col", "<u4"),
                           ("ids", "<u4", 64), ("logits", "<f4", 64)])


def logit_topk_scratch_bytes(max_rows, max_vocabulary=1 << 20):
    f = dll().tsp_logit_topk_scratch_bytes
    f.restype = C.c_uint64
    n = f(C.c_uint32(max_rows), C.c_uint32(max_vocabulary))
    if n == 0:
        raise FormatError(dll().tsp_last_error().decode())
    return n


def logit_topk_output_bytes(max_rows):
    f = dll().tsp_logit_topk_output_bytes
    f.restype = C.c_uint64
    n = f(C.c_uint32(max_rows))
    if n == 0:
        raise FormatError(dll().tsp_last_error().decode())
    return n


def logit_topk(dev, logits, rows, vocabulary, stride_bytes=None, scratch=None, out=None):
    """Row top-64 (`logit_topk`): returns the device buffer of 528-byte rows; view it with TOPK_ROW_DTYPE on the host."""
    stride_bytes = vocabulary * 4 if stride_bytes is None else stride_bytes
    scratch = dev.empty(logit_topk_scratch_bytes(rows, vocabulary), "uint8") if scratch is None else scratch
    out = dev.empty(logit_topk_output_bytes(rows), "uint8") if out is None else out
    check(dll().tsp_logit_topk(dev.ptr(logits), C.c_uint64(stride_bytes), C.c_uint32(rows), C.c_uint32(vocabulary), dev.ptr(scratch),
                               C.c_uint64(dev.nbytes(scratch)), dev.ptr(out), C.c_uint64(dev.nbytes(out)), dev.stream()))
    return out


def logit_topk_static(dev, logits, rows, vocabulary, stride_bytes=None, out=None):
    """`tsp_logit_topk_static`: the same rows with the partial rows kept in the library's own device array (no scratch
    argument, nothing allocated by the call when `out` is given)."""
    stride_bytes = vocabulary * 4 if stride_bytes is None else stride_bytes
    out = dev.empty(logit_topk_output_bytes(rows), "uint8") if out is None else out
    check(dll().tsp_logit_topk_static(dev.ptr(logits), C.c_uint64(stride_bytes), C.c_uint32(rows), C.c_uint32(vocabulary), dev.ptr(out),
                                      C.c_uint64(dev.nbytes(out)), dev.stream()))
    return out


def calibration_copy(dev, dst, src):
    """Plain copy kernel of a known size (scales a profiler's HBM byte counters)."""
    check(dll().tsp_calibration_copy(dev.ptr(dst), dev.ptr(src), C.c_uint64(dev.nbytes(src)), dev.stream()))


def as_u32(t):
    """Device int32 tensor -> host uint32 array."""
    return t.cpu().numpy().view(np.uint32)

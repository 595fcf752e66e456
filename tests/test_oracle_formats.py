"""Pins the CPU oracle's block decoders and GEMV against the reference's own known-answer tests
(native/tests/test_numeric.cpp) and against an independent bit-at-a-time decoder
(native/tests/raw_decode_reference.hpp). Every check runs against the C restatement and, where it
has been built, against the reference's own compiled CPU code."""
import math

import numpy as np
import pytest


def half_closed_form(bits):
    exponent, fraction = (bits >> 10) & 31, bits & 1023
    sign = -1.0 if bits & 0x8000 else 1.0
    if exponent == 31:
        return math.nan if fraction else sign * math.inf
    return sign * (math.ldexp(1 + fraction / 1024.0, exponent - 15) if exponent else math.ldexp(fraction, -24))


def test_binary16_all_patterns(cpu):
    # native/tests/test_numeric.cpp:40-54
    for bits in range(65536):
        actual, expected = cpu.binary16(bits), half_closed_form(bits)
        if math.isnan(expected):
            assert math.isnan(actual)
        else:
            assert actual == expected and math.copysign(1, actual) == math.copysign(1, expected), hex(bits)


def put(block, offset, value, width):
    for i in range(width):
        block[offset + i] = (value >> (8 * i)) & 255


def fixture_block(t):
    """native/tests/test_numeric.cpp:56-126: hand-encoded single blocks with exact expected floats.
    The encoder places logical values bit by bit; it shares nothing with the decoders under test."""
    geometry = {7: (32, 24), 8: (32, 34), 12: (256, 144), 13: (256, 176), 14: (256, 210), 20: (32, 18)}
    n, nbytes = geometry[t]
    block = np.zeros(nbytes, dtype=np.uint8)
    expected = np.zeros(n, dtype=np.float32)
    if t == 7:
        put(block, 0, 0x3800, 2)
        put(block, 2, 0xC000, 2)
        high = 0
        for i in range(32):
            code = (i * 13 + 7) % 32
            high |= (code // 16) << i
            block[8 + i % 16] |= (code % 16) << ((i // 16) * 4)
            expected[i] = np.float32(0.5) * np.float32(code) - np.float32(2)
        put(block, 4, high, 4)
    elif t == 8:
        put(block, 0, 0x3400, 2)
        for i in range(32):
            code = i * 8 - 128
            block[2 + i] = code & 255
            expected[i] = np.float32(0.25) * np.float32(code)
    elif t in (12, 13):
        put(block, 0, 0x3000, 2)
        put(block, 2, 0x3400, 2)
        for group in range(8):
            scale, minimum = (group * 11 + 3) % 64, (group * 7 + 5) % 64
            for bit in range(6):
                scale_byte = 4 + group if group < 4 else (8 + group if bit < 4 else group)
                min_byte = 8 + group if group < 4 else (8 + group if bit < 4 else 4 + group)
                scale_bit = bit if (group < 4 or bit < 4) else bit + 2
                min_bit = bit if group < 4 else (bit + 4 if bit < 4 else bit + 2)
                block[scale_byte] |= ((scale >> bit) & 1) << scale_bit
                block[min_byte] |= ((minimum >> bit) & 1) << min_bit
            for lane in range(32):
                code = (lane * 3 + group * 5) % (16 if t == 12 else 32)
                low_offset = 16 if t == 12 else 48
                block[low_offset + (group // 2) * 32 + lane] |= (code % 16) << ((group % 2) * 4)
                if t == 13:
                    block[16 + lane] |= (code // 16) << group
                expected[group * 32 + lane] = np.float32(np.float32(0.125) * np.float32(scale) * np.float32(code)) - \
                    np.float32(np.float32(0.25) * np.float32(minimum))
    elif t == 14:
        put(block, 208, 0x2800, 2)
        for i in range(256):
            code = (i * 7 + 1) % 64
            block[(i // 128) * 64 + (i % 64)] |= (code % 16) << ((i % 128 // 64) * 4)
            block[128 + (i // 128) * 32 + i % 32] |= (code // 16) << ((i % 128 // 32) * 2)
            scale = (i // 16) * 15 - 120
            block[192 + i // 16] = scale & 255
            expected[i] = np.float32(0.03125) * np.float32(scale) * np.float32(code - 32)
    else:
        put(block, 0, 0x3800, 2)
        alphabet = [-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113]
        for i in range(32):
            code = (i * 7) % 16
            block[2 + i % 16] |= code << ((i // 16) * 4)
            expected[i] = np.float32(0.5) * np.float32(alphabet[code])
    return block, expected


@pytest.mark.parametrize("t", [7, 8, 12, 13, 14, 20])
def test_single_block_fixtures(cpu, t):
    from oracle.oracle import FormatError
    block, expected = fixture_block(t)
    decoded = cpu.dequantize(t, block, expected.size)
    assert np.array_equal(decoded.view(np.uint32), expected.view(np.uint32))
    # native/tests/test_numeric.cpp:127-133: double GEMV over the fixture, float and double inputs.
    x = np.array([((i % 13) - 6) * 0.25 for i in range(expected.size)], dtype=np.float32)
    dot = 0.0
    for w, xi in zip(expected, x):
        dot += float(w) * float(xi)
    assert cpu.reference_gemv(t, block, expected.size, 1, x)[0] == dot
    assert cpu.reference_gemv(t, block, expected.size, 1, x.astype(np.float64))[0] == dot
    with pytest.raises(FormatError):
        cpu.dequantize(t, block[:-1], expected.size)


@pytest.mark.parametrize("t,patterns", [(0, (0x3F800000, 0xC0000000, 0x3E800000, 0x7F800000)),
                                        (1, (0x3C00, 0xC000, 0x3400, 0x7C00)), (30, (0x3F80, 0xC000, 0x3E80, 0x7F80))])
def test_float_decoders(cpu, t, patterns):
    # native/tests/test_numeric.cpp:134-145
    from oracle.oracle import FormatError
    width = 4 if t == 0 else 2
    data = np.zeros(width * 3, dtype=np.uint8)
    for i in range(3):
        put(data, width * i, patterns[i], width)
    assert list(cpu.dequantize(t, data, 3)) == [1.0, -2.0, 0.25]
    put(data, 0, patterns[3], width)
    with pytest.raises(FormatError):
        cpu.dequantize(t, data, 3)


def test_refusals(cpu):
    # native/tests/test_numeric.cpp:146-160
    from oracle.oracle import FormatError
    with pytest.raises(FormatError):
        cpu.dequantize(999, np.zeros(4, dtype=np.uint8), 1)
    f32 = np.zeros(4, dtype=np.uint8)
    with pytest.raises(FormatError):
        cpu.reference_gemv(0, f32, 1, 1, np.array([np.nan], dtype=np.float32))
    with pytest.raises(FormatError):
        cpu.reference_gemv(0, f32, 1, 1, np.array([np.nan], dtype=np.float64))
    put(f32, 0, 0x40000000, 4)
    precise = np.array([1 + 1e-12], dtype=np.float64)
    assert cpu.reference_gemv(0, f32, 1, 1, precise)[0] == precise[0] * 2
    with pytest.raises(FormatError):
        cpu.reference_gemv(0, f32, 1, 1, np.array([np.finfo(np.float64).max]))


def test_q8_multiblock_edge_scales(cpu):
    # native/tests/test_numeric.cpp:164-192: zero, negative zero, subnormal, extreme and negative scales.
    from oracle.oracle import FormatError
    scales = [0x0000, 0x8000, 0x0001, 0x03FF, 0x0400, 0x3555, 0xB555, 0x7BFF, 0xFBFF]
    encoded = np.zeros(len(scales) * 34, dtype=np.uint8)
    expected = np.zeros(len(scales) * 32, dtype=np.float32)
    for b, bits in enumerate(scales):
        put(encoded, b * 34, bits, 2)
        scale = half_closed_form(bits)
        for i in range(32):
            code = (b * 37 + i * 19) & 255
            encoded[b * 34 + 2 + i] = code
            expected[b * 32 + i] = np.float32(scale * (code if code < 128 else code - 256))
    decoded = cpu.dequantize(8, encoded, expected.size)
    assert np.array_equal(decoded.view(np.uint32), expected.view(np.uint32))
    for bad in (0x7C00, 0xFC00, 0x7E01):
        put(encoded, (len(scales) - 1) * 34, bad, 2)
        with pytest.raises(FormatError):
            cpu.dequantize(8, encoded, expected.size)


def bits_of(data, first, count):
    value = 0
    for bit in range(count):
        value |= ((int(data[(first + bit) // 8]) >> ((first + bit) % 8)) & 1) << bit
    return value


def independent_q4k(block, column):
    """native/tests/raw_decode_reference.hpp:14-49: every field read one bit at a time."""
    group = column // 32
    scale = minimum = 0
    for bit in range(6):
        scale_byte = 4 + group if group < 4 else (8 + group if bit < 4 else group)
        minimum_byte = 8 + group if group < 4 else (8 + group if bit < 4 else 4 + group)
        scale_bit = bit if (group < 4 or bit < 4) else bit + 2
        minimum_bit = bit if group < 4 else (bit + 4 if bit < 4 else bit + 2)
        scale |= bits_of(block, scale_byte * 8 + scale_bit, 1) << bit
        minimum |= bits_of(block, minimum_byte * 8 + minimum_bit, 1) << bit
    code = bits_of(block, 128 + (column // 64) * 256 + (column % 32) * 8 + ((column // 32) % 2) * 4, 4)
    return half_closed_form(bits_of(block, 0, 16)) * scale * code - half_closed_form(bits_of(block, 16, 16)) * minimum


def independent_q6k(block, i):
    """Bit-at-a-time Q6_K reader written from the format description (256 six-bit codes: four low
    bits in ql, two high bits in qh; sixteen int8 sub-scales; one f16 super-scale)."""
    section, within = i // 128, i % 128
    low = bits_of(block, (section * 64 + within % 64) * 8 + 4 * (within // 64), 4)
    high = bits_of(block, (128 + section * 32 + within % 32) * 8 + 2 * (within // 32), 2)
    sc = bits_of(block, (192 + i // 16) * 8, 8)
    sc = sc - 256 if sc >= 128 else sc
    return half_closed_form(bits_of(block, 208 * 8, 16)) * sc * ((low | (high << 4)) - 32)


def test_against_independent_decoders(cpu, synth):
    q4 = synth.q4k_blocks(101, 3)
    out = cpu.dequantize(12, q4.reshape(-1), 3 * 256)
    for b in range(3):
        for c in range(256):
            assert out[b * 256 + c] == np.float32(independent_q4k(q4[b], c))
    q6 = synth.q6k_blocks(102, 3)
    out = cpu.dequantize(14, q6.reshape(-1), 3 * 256)
    for b in range(3):
        for c in range(256):
            assert out[b * 256 + c] == np.float32(independent_q6k(q6[b], c))
    q8 = synth.q8_0_blocks(103, 5)
    out = cpu.dequantize(8, q8.reshape(-1), 5 * 32)
    for b in range(5):
        d = half_closed_form(int(q8[b, 0]) | (int(q8[b, 1]) << 8))
        for c in range(32):
            assert out[b * 32 + c] == np.float32(d * int(q8[b, 2 + c].view(np.int8)))


def test_half_times_int8_exact_in_f32(cpu):
    # native/tests/test_q8_layout.cpp:64-87 (invariant): half x int8 products are exact in fp32.
    rng = np.random.default_rng(5)
    halves = rng.integers(0, 0x7C00, size=4096, dtype=np.uint16)
    q = rng.integers(-128, 128, size=4096)
    for h, qi in zip(halves, q):
        exact = half_closed_form(int(h)) * int(qi)
        assert float(np.float32(exact)) == exact


@pytest.mark.parametrize("t", [8, 12, 14])
def test_gemv_brute_force(cpu, synth, t):
    rows, cols = 5, 512
    w = synth.matrix(t, 7 + t, rows, cols)
    x = synth.activations_f32(11, cols)
    dense = cpu.dequantize(t, w, rows * cols).reshape(rows, cols)
    y = cpu.reference_gemv(t, w, cols, rows, x)
    # Sequential double accumulation of float-rounded weights equals the reference unless the double
    # value needed rounding to fit a float; math.fsum bounds the association error instead.
    for r in range(rows):
        exact = math.fsum(float(a) * float(b) for a, b in zip(dense[r], x))
        assert abs(y[r] - exact) <= 1e-9 * max(1.0, abs(exact))


def test_oracle_equals_reference_on_random_blocks(orc, ref, synth):
    for t, n in ((7, 64), (8, 64), (12, 16), (13, 16), (14, 16)):
        rows, cols = 4, n * (32 if t in (7, 8) else 256) // 4
        w = synth.matrix(t, 900 + t, rows, cols)
        a, b = orc.dequantize(t, w, rows * cols), ref.dequantize(t, w, rows * cols)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
        x = synth.activations_f32(901, cols)
        assert np.array_equal(orc.reference_gemv(t, w, cols, rows, x), ref.reference_gemv(t, w, cols, rows, x))
    # Adversarial headers: raw random bytes (any scale pattern) with finite f16 fields.
    rng = np.random.default_rng(17)
    for t, bpb, epb in ((12, 144, 256), (14, 210, 256), (8, 34, 32)):
        raw = rng.integers(0, 256, size=(64, bpb), dtype=np.uint8)
        for off in ((0, 2) if t == 12 else (208,) if t == 14 else (0,)):
            raw[:, off + 1] &= 0x7B  # keep the f16 exponent below 31
        a, b = orc.dequantize(t, raw.reshape(-1), 64 * epb), ref.dequantize(t, raw.reshape(-1), 64 * epb)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_q8_many(cpu, synth):
    # native/src/q8_many.cpp:20-49
    assert [cpu.q8_many_width(n) for n in (1, 2, 3, 4, 5, 7, 8, 9, 16)] == [1, 2, 2, 4, 4, 4, 8, 8, 8]
    assert [cpu.q8_many_chunks(n) for n in (1, 3, 8, 15, 16)] == [1, 2, 1, 4, 2]
    rows, cols = 6, 128
    w = synth.matrix(8, 33, rows, cols)
    x = synth.activations_f32(34, (4, cols))
    out = cpu.reference_q8_many(w, x, cols, rows, 4)
    for tkn in range(4):
        assert np.array_equal(out[tkn], cpu.reference_gemv(8, w, cols, rows, x[tkn]))


def test_mt_gemv_matches_single_thread(orc, synth):
    w = synth.matrix(12, 55, 37, 512)
    x = synth.activations_f32(56, 512)
    assert np.array_equal(orc.reference_gemv_mt(12, w, 512, 37, x, 5), orc.reference_gemv(12, w, 512, 37, x))


def test_fixture_generator(orc, ref):
    # native/tests/grouped_mm_fixture.hpp:10-19: first bytes by hand (rng = 44, top byte of each LCG step).
    out = orc.fixture_weights(8, 64, 2, 1)
    rng, expect = 44, []
    for _ in range(out.size):
        rng = (rng * 1664525 + 1013904223) & 0xFFFFFFFF
        expect.append(rng >> 24)
    expect = np.array(expect, dtype=np.uint8).reshape(-1, 34)
    ds = [0x0401, 0x0568, 0x068E, 0x0AC2]
    for b in range(4):
        expect[b, 0], expect[b, 1] = ds[b] & 255, ds[b] >> 8
    assert np.array_equal(out.reshape(-1, 34), expect)
    q4 = orc.fixture_weights(12, 256, 4, 2).reshape(-1, 144)
    assert (q4[:, 2] == 0x03).all() and (q4[:, 3] == 0x1C).all()
    assert np.isfinite(ref.dequantize(12, q4.reshape(-1), 8 * 256)).all()

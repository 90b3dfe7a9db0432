"""Pins the CPU oracle's codecs (oracle/axq_oracle.c) without a GPU.

Sources of truth used here, none of which is the oracle's own formula retyped:
  * hand-computed known-answer blocks derived from the reference source
    (crates/axonml-quant/src/quantize.rs, dequantize.rs, types.rs) with scales
    chosen as powers of two so that every expected code is an obvious integer;
  * the inputs and tolerances of the reference's own unit tests
    (types.rs:344-389, quantize.rs:294-345, dequantize.rs:204-272);
  * numpy's float16 (an independent IEEE binary16 implementation) for the f16
    conversions the `half` crate performs;
  * the GGUF block spec, transcribed independently in numpy, for Q5_0/Q5_1/Q4_K.
"""
import numpy as np
import pytest

import oracle as o


def u16(p, i):
    return int(p[i]) | (int(p[i + 1]) << 8)


def f16_bits(v):
    return int(np.array([v], dtype=np.float32).astype(np.float16).view(np.uint16)[0])


# --------------------------------------------------------------------------- f16 conversion
def test_f32_to_f16_matches_numpy_at_every_boundary():
    # Every finite binary16 value, the midpoint to its successor, and one f32 ulp either side.
    h = np.arange(0, 0x7C00, dtype=np.uint16)
    v = h.view(np.float16).astype(np.float64)
    nxt = (h + 1).view(np.float16).astype(np.float64)
    nxt[-1] = 65536.0  # the rounding boundary to infinity is 65520
    mid = ((v + nxt) / 2).astype(np.float32)
    cand = np.concatenate([v.astype(np.float32), mid, np.nextafter(mid, np.float32(np.inf)),
                           np.nextafter(mid, np.float32(-np.inf))])
    cand = np.concatenate([cand, -cand, np.array([np.inf, -np.inf, 1e-10, -1e-10, 7e4, 6.0e-8, 2.9e-8, 3.0e-8],
                                                 dtype=np.float32)])
    want = cand.astype(np.float16).view(np.uint16)
    got = o.f32_to_f16_bits(cand)
    bad = np.nonzero(want != got)[0]
    assert bad.size == 0, f"{bad.size} mismatches, first: x={cand[bad[0]]!r} want={want[bad[0]]:#x} got={got[bad[0]]:#x}"


def test_f16_to_f32_matches_numpy_for_all_bit_patterns():
    h = np.arange(0, 0x10000, dtype=np.uint32).astype(np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = o.f16_bits_to_f32(h)
    finite = np.isfinite(want)
    assert np.array_equal(want[finite].view(np.uint32), got[finite].view(np.uint32))
    assert np.array_equal(np.isnan(want), np.isnan(got))
    assert np.array_equal(want[np.isinf(want)], got[np.isinf(want)])


def test_nan_keeps_being_nan():
    assert (o.f32_to_f16_bits(np.array([np.nan], dtype=np.float32))[0] & 0x7FFF) > 0x7C00


# --------------------------------------------------------------------------- registry (types.rs:45-78)
def test_registry_sizes():
    L = o.lib()
    expect = {o.Q8_0: (32, 34), o.Q4_0: (32, 18), o.Q4_1: (32, 20), o.Q5_0: (32, 22), o.Q5_1: (32, 24),
              o.F16: (1, 2), o.F32: (1, 4), o.Q4_K: (256, 144), o.Q6_K: (256, 210), o.Q5_K: (256, 176)}
    for t, (bs, bb) in expect.items():
        assert L.axo_block_size(t) == bs and L.axo_bytes_per_block(t) == bb
    # quantize.rs:294-313: 8 elements -> 1 block, 64 -> 2 blocks
    assert L.axo_num_blocks(o.Q8_0, 8) == 1 and L.axo_num_blocks(o.Q4_0, 64) == 2
    assert L.axo_block_size(99) == 0


# --------------------------------------------------------------------------- Q8_0 (quantize.rs:82-114)
def test_q8_0_zero_block_has_scale_one():
    p = o.quantize(o.Q8_0, np.zeros(32, np.float32))
    assert p[0] == 0x00 and p[1] == 0x3C  # f16 1.0, little endian (types.rs:144)
    assert not p[2:].any()


def test_q8_0_rounds_half_away_from_zero():
    # max_abs = 127 -> scale = 1.0 exactly, so q = round(x): Rust's f32::round, not round-half-even.
    x = np.zeros(32, np.float32)
    x[:10] = [127, -127, 0.5, -0.5, 1.5, 2.5, -2.5, 3.49, -3.51, 126.5]
    p = o.quantize(o.Q8_0, x)
    assert (p[0], p[1]) == (0x00, 0x3C)
    assert p[2:12].view(np.int8).tolist() == [127, -127, 1, -1, 2, 3, -3, 3, -4, 127]
    assert not p[12:].any()


def test_q8_0_power_of_two_scale_and_f16_rounding_of_scale():
    x = np.zeros(32, np.float32)
    x[:4] = [254, 1, 3, 5]  # scale = 2.0 -> 0x4000; 0.5 -> 1, 1.5 -> 2, 2.5 -> 3
    p = o.quantize(o.Q8_0, x)
    assert u16(p, 0) == 0x4000
    assert p[2:6].view(np.int8).tolist() == [127, 1, 2, 3]
    # the quantiser divides by the f32 scale but stores its f16 rounding (quantize.rs:100-109)
    x[:4] = [1.0, 0, 0, 0]
    p = o.quantize(o.Q8_0, x)
    assert u16(p, 0) == f16_bits(np.float32(1.0) / np.float32(127.0))
    assert p[2:3].view(np.int8)[0] == 127


def test_q8_0_tail_block_is_zero_padded_and_truncated():
    x = (np.arange(40, dtype=np.float32) - 20.0)
    p = o.quantize(o.Q8_0, x)
    assert p.size == 2 * 34
    assert not p[34 + 2 + 8:].any()  # codes 8..31 of the tail block (quantize.rs:103)
    y = o.dequantize(o.Q8_0, p, 40)
    assert y.shape == (40,)  # dequantize.rs:44-50
    assert np.abs(y - x).max() <= 20 / 127 / 2 + 20 * 2 ** -11


# --------------------------------------------------------------------------- Q4_0 (quantize.rs:121-156, types.rs:179-206)
def test_q4_0_zero_block():
    p = o.quantize(o.Q4_0, np.zeros(32, np.float32))
    assert (p[0], p[1]) == (0x00, 0x3C)
    assert (p[2:] == 0x88).all()  # code 0 + bias 8 in both nibbles


def test_q4_0_known_block_scale_one():
    # max_abs = 7 -> scale 1.0; pairs (2i, 2i+1) -> (low, high) nibble, bias 8 (types.rs:190-198)
    x = np.zeros(32, np.float32)
    x[:8] = [7, -7, 6.5, -6.5, 0.5, -0.5, 2.5, -1.4]
    p = o.quantize(o.Q4_0, x)
    assert (p[0], p[1]) == (0x00, 0x3C)
    # codes 7,-7,7,-7,1,-1,3,-1 -> nibbles 15,1,15,1,9,7,11,7
    assert p[2:6].tolist() == [0x1F, 0x1F, 0x79, 0x7B]
    assert (p[6:] == 0x88).all()


def test_q4_0_reference_pack_unpack_ramp():
    # types.rs:366-378: the ramp -8..7 twice, scale 1.0.  Bytes typed from Q4Block::pack by hand.
    img = bytes([0x00, 0x3C] + [0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE] * 2)
    y = o.dequantize(o.Q4_0, np.frombuffer(img, np.uint8), 32)
    assert y.tolist() == [float(v) for v in list(range(-8, 8)) * 2]


def test_q4_0_scale_is_max_abs_over_seven():
    x = np.zeros(32, np.float32)
    x[0], x[1] = -16.0, 16.0
    p = o.quantize(o.Q4_0, x)
    assert u16(p, 0) == f16_bits(np.float32(16.0) / np.float32(7.0)) == 0x4092
    assert p[2] == 0xF1  # -7 -> 1, +7 -> 15


# --------------------------------------------------------------------------- Q4_1 (quantize.rs:163-205, types.rs:238-255)
def test_q4_1_known_block():
    x = np.zeros(32, np.float32)
    x[:8] = [0, 15, 0.5, 1.5, 2.5, 14.5, 7, 8]
    p = o.quantize(o.Q4_1, x)
    assert u16(p, 0) == 0x3C00 and u16(p, 2) == 0x0000  # scale 1.0, min 0.0
    assert p[4:8].tolist() == [0xF0, 0x21, 0xF3, 0x87]
    assert not p[8:].any()


def test_q4_1_negative_min_and_constant_block():
    x = np.full(32, -3.0, np.float32)
    x[1] = 12.0  # range 15 -> scale 1.0, min -3.0
    p = o.quantize(o.Q4_1, x)
    assert u16(p, 0) == 0x3C00 and u16(p, 2) == 0xC200
    assert p[4] == 0xF0 and not p[5:].any()
    y = o.dequantize(o.Q4_1, p, 32)
    assert y[0] == -3.0 and y[1] == 12.0
    # max == min -> scale 1.0 (quantize.rs:179), min = the constant, all codes 0
    p = o.quantize(o.Q4_1, np.full(32, 2.5, np.float32))
    assert u16(p, 0) == 0x3C00 and u16(p, 2) == 0x4100
    assert not p[4:].any()


def test_q4_1_odd_tail_drops_last_code():
    # quantize.rs:190-194: the pack loop covers min(16, len/2) bytes; len = 3 -> one byte.
    x = np.zeros(35, np.float32)
    x[32:] = [1.0, 2.0, 4.0]
    p = o.quantize(o.Q4_1, x)
    tail = p[20:]
    assert u16(tail, 0) == f16_bits(np.float32(3.0) / np.float32(15.0))
    assert u16(tail, 2) == 0x3C00  # min 1.0
    assert tail[4] == 0x50 and not tail[5:].any()  # codes 0 and 5; the third element (code 15) is dropped
    y = o.dequantize(o.Q4_1, p, 35)
    assert y[34] == 1.0  # decodes as code 0 -> min


def test_q4_1_dequant_is_multiply_then_add():
    # scale = 0.1 (f16 0x2E66 = 0.0999755859375), min = 1/3 (f16 0x3555): q*scale + min in two f32 roundings.
    img = np.zeros(20, np.uint8)
    img[0:2] = [0x66, 0x2E]
    img[2:4] = [0x55, 0x35]
    img[4] = 0xF7
    y = o.dequantize(o.Q4_1, img, 32)
    s, m = np.float32(np.float16(0.1)), np.float32(np.float16(1 / 3))
    assert y[0] == np.float32(np.float32(7) * s) + m and y[1] == np.float32(np.float32(15) * s) + m


# --------------------------------------------------------------------------- the reference's own round-trip tests
def test_reference_roundtrip_tolerances():
    x = np.arange(64, dtype=np.float32) / np.float32(10.0)  # dequantize.rs:204-246
    y8 = o.dequantize(o.Q8_0, o.quantize(o.Q8_0, x), 64)
    assert np.abs(y8 - x).max() < 0.1
    y4 = o.dequantize(o.Q4_0, o.quantize(o.Q4_0, x), 64)
    assert np.abs(y4 - x).max() < 2.0
    v = np.array([1.0, 2.5, -3.0, 4.25], np.float32)  # dequantize.rs:248-272
    assert np.abs(o.dequantize(o.F16, o.quantize(o.F16, v), 4) - v).max() < 0.01
    assert np.array_equal(o.dequantize(o.F32, o.quantize(o.F32, v), 4), v)


def test_reference_q8_block_bytes_roundtrip():
    # types.rs:380-389: scale 0.5, zero codes
    img = np.zeros(34, np.uint8)
    img[0:2] = [0x00, 0x38]
    assert not o.dequantize(o.Q8_0, img, 32).any()
    img[2] = 0xFE  # -2 * 0.5
    assert o.dequantize(o.Q8_0, img, 32)[0] == -1.0


def test_compression_ordering():
    # quantize.rs:324-335
    n = 256
    assert n * 4 / o.packed_bytes(o.Q8_0, n) > 2.0
    assert o.packed_bytes(o.Q4_0, n) < o.packed_bytes(o.Q8_0, n)


# --------------------------------------------------------------------------- GGUF layouts, by hand-built blocks
def test_q5_0_layout_hand_block():
    img = np.zeros(22, np.uint8)
    img[0:2] = [0x00, 0x3C]  # d = 1.0
    img[2:6] = [0xFF, 0xFF, 0x00, 0x00]  # qh: elements 0..15 carry bit 4, 16..31 do not
    img[6:] = [j | ((15 - j) << 4) for j in range(16)]
    y = o.dequantize(o.Q5_0, img, 32)
    assert y[:16].tolist() == [float(j) for j in range(16)]  # (j | 16) - 16
    assert y[16:].tolist() == [float(15 - j - 16) for j in range(16)]


def test_q5_1_layout_hand_block():
    img = np.zeros(24, np.uint8)
    img[0:2] = [0x00, 0x38]  # d = 0.5
    img[2:4] = [0x00, 0xC0]  # m = -2.0
    img[4:8] = [0x01, 0x00, 0x00, 0x80]  # qh bit 0 (element 0) and bit 31 (element 31)
    img[8:] = [j | ((15 - j) << 4) for j in range(16)]
    y = o.dequantize(o.Q5_1, img, 32)
    want = [j * 0.5 - 2.0 for j in range(16)] + [(15 - j) * 0.5 - 2.0 for j in range(16)]
    want[0] = 16 * 0.5 - 2.0
    want[31] = (0 + 16) * 0.5 - 2.0
    assert y.tolist() == want


def test_q4_k_layout_hand_block():
    # 6-bit scales ls and mins lm chosen so that sub-blocks 4..7 use the split high bits.
    ls = [1, 2, 3, 4, 33, 34, 35, 36]
    lm = [5, 6, 7, 8, 37, 38, 39, 40]
    img = np.zeros(144, np.uint8)
    img[0:2] = [0x00, 0x3C]  # d = 1.0
    img[2:4] = [0x00, 0x38]  # dmin = 0.5
    # bytes typed by hand from ggml's get_scale_min_k4 packing
    img[4:16] = [129, 130, 131, 132, 133, 134, 135, 136, 0x51, 0x62, 0x73, 0x84]
    for p in range(4):
        for l in range(32):
            img[16 + 32 * p + l] = (l & 15) | (((l + 1) & 15) << 4)
    y = o.dequantize(o.Q4_K, img, 256)
    for s in range(8):
        for l in range(32):
            q = (l & 15) if s % 2 == 0 else ((l + 1) & 15)
            assert y[32 * s + l] == 1.0 * ls[s] * q - 0.5 * lm[s], (s, l)


def _gguf_dequant_numpy(qtype, packed, numel):
    """Independent numpy transcription of the GGUF block spec (not of the oracle)."""
    out = []
    if qtype == o.Q4_K:
        for b in packed.reshape(-1, 144):
            d, dmin = b[0:4].view(np.float16).astype(np.float32)
            sc, qs = b[4:16].astype(np.int32), b[16:]
            for j in range(8):
                if j < 4:
                    l, m = sc[j] & 63, sc[j + 4] & 63
                else:
                    l = (sc[j + 4] & 0xF) | ((sc[j - 4] >> 6) << 4)
                    m = (sc[j + 4] >> 4) | ((sc[j] >> 6) << 4)
                q = qs[32 * (j // 2):32 * (j // 2) + 32]
                q = (q >> 4) if j & 1 else (q & 0xF)
                out.append(np.float32(d * np.float32(l)) * q.astype(np.float32) - np.float32(dmin * np.float32(m)))
    else:
        hdr = 2 if qtype == o.Q5_0 else 4
        for b in packed.reshape(-1, hdr + 20):
            d = b[0:2].view(np.float16).astype(np.float32)[0]
            m = b[2:4].view(np.float16).astype(np.float32)[0] if qtype == o.Q5_1 else np.float32(0)
            qh = int(b[hdr:hdr + 4].view(np.uint32)[0])
            qs = b[hdr + 4:].astype(np.int32)
            hb = np.array([(qh >> e) & 1 for e in range(32)], dtype=np.int32)
            u = np.concatenate([(qs & 0xF) | (hb[:16] << 4), (qs >> 4) | (hb[16:] << 4)])
            if qtype == o.Q5_0:
                out.append((u - 16).astype(np.float32) * d)
            else:
                out.append(u.astype(np.float32) * d + m)
    return np.concatenate(out)[:numel]


@pytest.mark.parametrize("qtype", [o.Q5_0, o.Q5_1, o.Q4_K])
def test_gguf_types_dequant_matches_spec_on_random_quantised_data(qtype):
    rng = np.random.default_rng(7)
    x = (rng.standard_normal(2048) * 0.02).astype(np.float32)
    x[rng.random(2048) < 0.01] = 0.5
    p = o.quantize(qtype, x)
    assert np.array_equal(o.dequantize(qtype, p, 2048), _gguf_dequant_numpy(qtype, p, 2048))


def test_q4_k_six_bit_fields_roundtrip_all_values():
    # Drive every 6-bit scale value through every sub-block position: a superblock whose sub-block s
    # spans [0, 15*t] has scale t, so ls_s = round(63 * t_s / max t).
    for base in range(0, 64, 8):
        t = np.arange(base, base + 8, dtype=np.float32)
        t[t == 0] = 0.0
        x = np.zeros(256, np.float32)
        for s in range(8):
            x[32 * s + 1] = 15.0 * t[s]
        p = o.quantize(o.Q4_K, np.concatenate([x, np.full(256, 0, np.float32)]))[:144]
        sc = p[4:16].astype(np.int32)
        got = [(sc[j] & 63) if j < 4 else ((sc[j + 4] & 0xF) | ((sc[j - 4] >> 6) << 4)) for j in range(8)]
        tmax = t.max()
        want = [int(np.floor(63.0 * v / tmax + 0.5)) if tmax > 0 else 0 for v in t]
        assert got == want, (base, got, want)


# --------------------------------------------------------------------------- quantiser rules of the GGUF-only types, by hand
def _pack_q5(codes):
    """32 five-bit codes -> (qh, qs) in the GGUF order: element j < 16 in the low nibble of qs[j] and bit j of qh,
    element j + 16 in the high nibble of qs[j] and bit j + 16."""
    qh = sum(((c >> 4) & 1) << e for e, c in enumerate(codes))
    qs = [(codes[j] & 15) | ((codes[j + 16] & 15) << 4) for j in range(16)]
    return [qh & 255, (qh >> 8) & 255, (qh >> 16) & 255, qh >> 24], qs


def test_q5_0_known_block_with_half_way_values():
    # max |x| = 15 -> scale 1.0; q = round half away from zero, stored code = q + 16
    x = np.zeros(32, np.float32)
    x[:16] = [-15, 2.5, -2.5, 14.5, -14.5, 0, 1, -1, 0.49, -0.49, 7, -8, 0.5, -0.5, 15, 3]
    x[16], x[31] = 0.5, -0.5
    codes = [1, 19, 13, 31, 1, 16, 17, 15, 16, 16, 23, 8, 17, 15, 31, 19] + [17] + [16] * 14 + [15]
    qh, qs = _pack_q5(codes)
    assert qh == [0x6A, 0xD7, 0xFF, 0x7F]  # worked by hand from the bit 4 of each code
    assert o.quantize(o.Q5_0, x).tolist() == [0x00, 0x3C] + qh + qs
    # scale = max_abs / 15 is not a power of two in general: 7.5 / 15 = 0.5, -7.5 -> -15 -> code 1, 0.25 -> 0.5 -> 1 -> code 17
    y = np.zeros(32, np.float32)
    y[0], y[1], y[2] = -7.5, 0.25, -0.25
    qh, qs = _pack_q5([1, 17, 15] + [16] * 29)
    assert o.quantize(o.Q5_0, y).tolist() == [0x00, 0x38] + qh + qs
    # zero block: scale 1.0, every code 16
    qh, qs = _pack_q5([16] * 32)
    assert o.quantize(o.Q5_0, np.zeros(32, np.float32)).tolist() == [0x00, 0x3C] + qh + qs


def test_q5_1_known_block_with_half_way_values():
    # min -2, max 29 -> scale 31 / 31 = 1.0; code = round half away ((x - min) / scale)
    x = np.full(32, -2.0, np.float32)
    x[1], x[2], x[3], x[4], x[5], x[20], x[31] = 29, 0.5, -1.5, 27.5, -1.51, 13.49, 14.0
    codes = [0, 31, 3, 1, 30, 0] + [0] * 14 + [15] + [0] * 10 + [16]
    qh, qs = _pack_q5(codes)
    assert o.quantize(o.Q5_1, x).tolist() == [0x00, 0x3C, 0x00, 0xC0] + qh + qs
    # constant block: scale 1.0, min = the value, codes 0
    qh, qs = _pack_q5([0] * 32)
    assert o.quantize(o.Q5_1, np.full(32, 0.75, np.float32)).tolist() == [0x00, 0x3C, 0x00, 0x3A] + qh + qs
    # a span that is not a power of two: min 1, max 16.5 -> scale 0.5 (15.5 / 31), 1.25 -> 0.5 -> code 1, 1.24 -> code 0
    z = np.full(32, 1.0, np.float32)
    z[1], z[2], z[3] = 16.5, 1.25, 1.24
    qh, qs = _pack_q5([0, 31, 1, 0] + [0] * 28)
    assert o.quantize(o.Q5_1, z).tolist() == [0x00, 0x38, 0x00, 0x3C] + qh + qs


def _pack_q4k_codes(q):
    """256 four-bit codes -> qs[128]: pair p holds sub-block 2p in the low nibbles and 2p + 1 in the high."""
    return [q[64 * p + l] | (q[64 * p + 32 + l] << 4) for p in range(4) for l in range(32)]


def test_q4_k_known_superblock_worked_by_hand():
    """Sub-block s spans [-lm_s / 32, -lm_s / 32 + 15 ls_s / 64]: every quantity of the rule is an integer over a power
    of two.  max scale = 63/64 -> d = 1/64 (f16 0x2400), max min = 63/32 -> dmin = 1/32 (f16 0x2800), the 6-bit
    fields come back as the ls, lm chosen, and every code as placed (half-way values round away from zero)."""
    ls = [63, 1, 2, 32, 33, 47, 16, 0]  # sub-block 7 is constant: scale 0, codes 0
    lm = [63, 0, 5, 31, 32, 48, 17, 9]  # sub-block 1 has no negative value: min 0
    q = [[(7 * i + s) % 16 for i in range(32)] for s in range(8)]  # every code 0..15 twice per sub-block
    q[7] = [0] * 32
    x = np.zeros(256, np.float32)
    for s in range(8):
        for i in range(32):
            x[32 * s + i] = ls[s] / 64 * q[s][i] - lm[s] / 32
    # half-way values inside the range of sub-block 3 (step 1/2, offset 31/32): 6.5 steps -> 7, 13.5 steps -> 14
    x[96 + 5], x[96 + 6] = 0.5 * 6.5 - 31 / 32, 0.5 * 13.5 - 31 / 32
    q[3][5], q[3][6] = 7, 14
    scales = [191, 129, 66, 32, 191, 192, 69, 31, 1, 15, 16, 144]  # packed by hand from ls, lm (get_scale_min_k4 order)
    want = [0x00, 0x24, 0x00, 0x28] + scales + _pack_q4k_codes([c for sub in q for c in sub])
    got = o.quantize(o.Q4_K, x)
    assert got.tolist() == want
    y = o.dequantize(o.Q4_K, got, 256)
    keep = np.ones(256, bool)
    keep[[96 + 5, 96 + 6]] = False
    assert np.array_equal(y[keep], x[keep])  # everything but the two half-way values is a grid point
    assert y[96 + 5] == 0.5 * 7 - 31 / 32 and y[96 + 6] == 0.5 * 14 - 31 / 32


def test_q4_k_six_bit_rounding_is_to_nearest_half_away():
    # two sub-blocks with spans 15 and 7.5 -> scales 1 and 0.5 -> ls = 63 and round(31.5) = 32; mins 4 and 2.03 -> lm = 63 and
    # round(31.97) = 32; d = f16(1/63) = 0x2410 (2^-6 * (1 + 16/1024)), dmin = f16(4/63) = 0x2C10
    x = np.zeros(256, np.float32)
    x[0], x[1] = -4.0, 11.0
    x[32], x[33] = -2.03, np.float32(7.5) + np.float32(-2.03)
    p = o.quantize(o.Q4_K, x)
    assert p[:4].tolist() == [0x10, 0x24, 0x10, 0x2C]
    assert (p[4] & 63, p[5] & 63, p[8] & 63, p[9] & 63) == (63, 32, 63, 32)
    # codes with the stored d, dmin: sd = d * 63, sm = dmin * 63 for sub-block 0
    d, dmin = np.float32(0.015869140625), np.float32(0.0634765625)
    sd0, sm0 = float(d) * 63, float(dmin) * 63
    assert (p[16] & 15, p[17] & 15) == (int(np.floor((-4.0 + sm0) / sd0 + 0.5)), min(15, int(np.floor((11.0 + sm0) / sd0 + 0.5))))


# --------------------------------------------------------------------------- invariants, all types
@pytest.mark.parametrize("qtype", [o.Q8_0, o.Q4_0, o.Q4_1, o.Q5_0, o.Q5_1])
def test_roundtrip_error_bound(qtype):
    rng = np.random.default_rng(11)
    n = 4096
    x = (rng.standard_normal(n) * 0.02).astype(np.float32)
    y = o.dequantize(qtype, o.quantize(qtype, x), n)
    xb, yb = x.reshape(-1, 32), y.reshape(-1, 32)
    levels = {o.Q8_0: 127 * 2, o.Q4_0: 14, o.Q4_1: 15, o.Q5_0: 30, o.Q5_1: 31}[qtype]
    span = 2 * np.abs(xb).max(1) if qtype in (o.Q8_0, o.Q4_0, o.Q5_0) else xb.max(1) - xb.min(1)
    step = span / levels
    # half a step, plus the f16 rounding of the scale (and of the minimum) carried over the block's range
    assert (np.abs(xb - yb).max(1) <= step * 0.5 + np.abs(xb).max(1) * 2 ** -9).all()


def _q4k_fields(p):
    """(d, dmin, ls[8], lm[8]) of one 144-byte superblock, per the GGUF spec."""
    d, dmin = (float(v) for v in p[0:4].view(np.float16))
    sc = p[4:16].astype(np.int32)
    ls = [(sc[j] & 63) if j < 4 else ((sc[j + 4] & 0xF) | ((sc[j - 4] >> 6) << 4)) for j in range(8)]
    lm = [(sc[j + 4] & 63) if j < 4 else ((sc[j + 4] >> 4) | ((sc[j] >> 6) << 4)) for j in range(8)]
    return d, dmin, ls, lm


def test_q4_k_roundtrip_error_is_what_the_rule_implies():
    """From the stored fields: a value inside the code range is off by at most half a step sd; one pushed outside it by the
    6-bit rounding of the scale and the minimum is off by exactly how far outside it lies.  The stored 6-bit fields are the
    nearest ones: |sd - scale| <= d / 2 and |sm - min| <= dmin / 2, up to the f16 rounding of d and dmin."""
    rng = np.random.default_rng(12)
    n = 256 * 64
    x = (rng.standard_normal(n) * 0.02).astype(np.float32)
    x[rng.random(n) < 0.01] = 0.5
    x[256 * 5:256 * 5 + 64] = np.abs(x[256 * 5:256 * 5 + 64])  # two sub-blocks without a negative value
    packed = o.quantize(o.Q4_K, x)
    y = o.dequantize(o.Q4_K, packed, n)
    for b, p in enumerate(packed.reshape(-1, 144)):
        d, dmin, ls, lm = _q4k_fields(p)
        xs = x[256 * b:256 * b + 256].astype(np.float64).reshape(8, 32)
        ys = y[256 * b:256 * b + 256].astype(np.float64).reshape(8, 32)
        mins = np.maximum(0.0, -xs.min(1))
        scales = (xs.max(1) + mins) / 15
        assert abs(d - scales.max() / 63) <= scales.max() / 63 * 2 ** -11 and abs(dmin - mins.max() / 63) <= mins.max() / 63 * 2 ** -11
        for s in range(8):
            sd, sm = d * ls[s], dmin * lm[s]
            assert abs(sd - scales[s]) <= d * 0.5 + scales[s] * 2 ** -10, (b, s)
            assert abs(sm - mins[s]) <= dmin * 0.5 + mins[s] * 2 ** -10, (b, s)
            below = max(0.0, mins[s] - sm)                 # how far the smallest value lies under code 0
            above = max(0.0, xs[s].max() + sm - 15 * sd)   # ... and the largest above code 15
            bound = max(sd * 0.5, below, above) + 1e-6 * np.abs(xs[s]).max()
            assert np.abs(xs[s] - ys[s]).max() <= bound, (b, s)


def test_q8_0_requantising_dequantised_values_is_idempotent():
    rng = np.random.default_rng(3)
    x = rng.standard_normal(1024).astype(np.float32)
    p1 = o.quantize(o.Q8_0, x)
    p2 = o.quantize(o.Q8_0, o.dequantize(o.Q8_0, p1, 1024))
    # codes survive; scales may move by the f16 rounding of 127*f16(scale)/127
    assert np.array_equal(p1.reshape(-1, 34)[:, 2:], p2.reshape(-1, 34)[:, 2:])


def test_empty_input():
    for t in range(8):
        assert o.quantize(t, np.zeros(0, np.float32)).size == 0
        assert o.dequantize(t, np.zeros(0, np.uint8), 0).size == 0


# --------------------------------------------------------------------------- Q6_K (GGUF block; the reference has no such type)
def _q6k_dequant_numpy(packed, numel):
    """ggml's dequantize_row_q6_K, transcribed independently in numpy from its published loop: for each half n of
    the superblock and l in 0..31, four values at 128 n + l + {0, 32, 64, 96} out of ql[64 n + l], ql[64 n + l + 32]
    and qh[32 n + l], scales 8 n + l / 16 + {0, 2, 4, 6}."""
    out = []
    for b in packed.reshape(-1, 210):
        ql, qh, sc = b[:128].astype(np.int32), b[128:192].astype(np.int32), b[192:208].view(np.int8).astype(np.float32)
        d = b[208:210].view(np.float16).astype(np.float32)[0]
        y = np.zeros(256, np.float32)
        for n in range(2):
            for l in range(32):
                i = l // 16
                q1 = ((ql[64 * n + l] & 0xF) | (((qh[32 * n + l] >> 0) & 3) << 4)) - 32
                q2 = ((ql[64 * n + l + 32] & 0xF) | (((qh[32 * n + l] >> 2) & 3) << 4)) - 32
                q3 = ((ql[64 * n + l] >> 4) | (((qh[32 * n + l] >> 4) & 3) << 4)) - 32
                q4 = ((ql[64 * n + l + 32] >> 4) | (((qh[32 * n + l] >> 6) & 3) << 4)) - 32
                y[128 * n + l + 0] = np.float32(d * sc[8 * n + i + 0]) * np.float32(q1)
                y[128 * n + l + 32] = np.float32(d * sc[8 * n + i + 2]) * np.float32(q2)
                y[128 * n + l + 64] = np.float32(d * sc[8 * n + i + 4]) * np.float32(q3)
                y[128 * n + l + 96] = np.float32(d * sc[8 * n + i + 6]) * np.float32(q4)
        out.append(y)
    return np.concatenate(out)[:numel]


def test_q6_k_zero_superblock_bytes():
    # all codes q = 0 -> u = 32: low nibbles 0, every bit pair 0b10 -> qh bytes 0xAA; scales 0, d 0
    p = o.quantize(o.Q6_K, np.zeros(256, np.float32))
    assert p.tolist() == [0] * 128 + [0xAA] * 64 + [0] * 16 + [0, 0]
    assert not o.dequantize(o.Q6_K, p, 256).any()


def test_q6_k_layout_one_code_at_a_time():
    """A superblock of all-zero codes (u = 32) in which one element holds another code: which byte and which bits
    change, for elements of every (half, 32-group) and codes that exercise both the nibble and the bit pair."""
    base = np.array([0] * 128 + [0xAA] * 64 + [1] * 16 + [0x00, 0x3C], np.uint8)  # scales 1, d = 1.0
    assert not o.dequantize(o.Q6_K, base, 256).any()
    for e, u in [(0, 0), (1, 63), (31, 17), (32, 5), (63, 48), (64, 0x2B), (95, 1), (96, 62), (127, 15), (128, 63), (160 + 7, 0),
                 (192 + 16, 0x15), (224 + 31, 0x3A), (255, 0)]:
        n, c, l = e >> 7, (e >> 5) & 3, e & 31
        img = base.copy()
        qi, hi = 64 * n + 32 * (c & 1) + l, 128 + 32 * n + l
        img[qi] = (u & 15) << 4 if c >= 2 else (u & 15)
        img[hi] = (0xAA & ~(3 << (2 * c))) | ((u >> 4) << (2 * c))
        want = np.zeros(256, np.float32)
        want[e] = u - 32
        assert np.array_equal(o.dequantize(o.Q6_K, img, 256), want), (e, u)


def test_q6_k_signed_scales_and_d():
    # every int8 scale value, negative ones included, times d = 0.5; codes u = 33 (q = 1) everywhere
    for first in range(-128, 128, 16):
        sc = np.arange(first, first + 16, dtype=np.int8)
        img = np.concatenate([np.full(128, 0x11, np.uint8), np.full(64, 0xAA, np.uint8), sc.view(np.uint8), np.array([0x00, 0x38], np.uint8)])
        y = o.dequantize(o.Q6_K, img, 256)
        assert np.array_equal(y, np.repeat(sc.astype(np.float32) * np.float32(0.5), 16))


def test_q6_k_dequant_matches_ggml_loop_on_arbitrary_bytes():
    rng = np.random.default_rng(61)
    raw = rng.integers(0, 256, size=(64, 210), dtype=np.uint8)
    raw[:, 208:210] = (rng.standard_normal((64, 1)) * 0.1).astype(np.float16).view(np.uint8)
    assert np.array_equal(o.dequantize(o.Q6_K, raw.reshape(-1), 64 * 256), _q6k_dequant_numpy(raw.reshape(-1), 64 * 256))


def test_q6_k_known_superblock_by_hand():
    """Sub-block s holds multiples of its own step: max |x| = 31 * step_s with steps 2^-7 * ls_s for hand-picked ls
    (the largest 127), so max_scale = 127 / 128, d = f16(2^-7) exactly, every x an exact grid point."""
    ls = [127, 1, 2, 64, 100, 0, 33, 126, 5, 77, 127, 12, 90, 3, 50, 8]
    q = [[((11 * i + 5 * s) % 63) - 31 for i in range(16)] for s in range(16)]  # codes -31..31
    for s in range(16):
        q[s][3] = 31 if s % 2 else -31  # the sub-block's maximum magnitude is code 31 exactly
    x = np.zeros(256, np.float32)
    for s in range(16):
        for i in range(16):
            x[16 * s + i] = ls[s] / 128 * q[s][i]
    p = o.quantize(o.Q6_K, x)
    assert p[208:210].tolist() == [0x00, 0x20]  # 2^-7
    assert p[192:208].tolist() == ls
    got_q = np.rint(o.dequantize(o.Q6_K, p, 256).astype(np.float64) * 128).reshape(16, 16)
    for s in range(16):
        if ls[s]:
            assert (got_q[s] == np.array(q[s]) * ls[s]).all(), s
    # codes read straight from the bytes, per the layout
    for s in (0, 3, 9, 15):
        for i in (0, 3, 15):
            e = 16 * s + i
            n, c, l = e >> 7, (e >> 5) & 3, e & 31
            u = ((int(p[64 * n + 32 * (c & 1) + l]) >> (4 * (c >> 1))) & 15) | (((int(p[128 + 32 * n + l]) >> (2 * c)) & 3) << 4)
            assert u - 32 == q[s][i], (s, i)
    assert np.array_equal(o.dequantize(o.Q6_K, p, 256), x)


def test_q6_k_half_way_values_round_away_and_clamp():
    # sub-block 0: max |x| = 31 -> scale 1 = max_scale, d = f16(1 / 127), ls = 127, sd = d * 127 (in f32);
    # x = (k + 0.5) sd -> k + 1, -(k + 0.5) sd -> -(k + 1): half-way quotients round away from zero
    x = np.zeros(256, np.float32)
    x[0] = 31.0
    d = np.float32(np.float16(np.float32(1.0) / np.float32(127.0)))
    sd = np.float32(d * np.float32(127.0))
    vals = [0.5, 1.5, 2.5, -0.5, -1.5, 30.49, 7.0]
    for i, v in enumerate(vals):
        x[1 + i] = np.float32(v) * sd
    # sub-block 1: scale 1.4 / 127 of the maximum -> ls = round(1.4) = 1, sd = d: its extremes lie 43 steps out and clamp
    # to the ends of the code range, -32 and 31
    x[16], x[17] = -31 * 1.4 / 127, 31 * 1.4 / 127
    p = o.quantize(o.Q6_K, x)
    assert p[208:210].view(np.float16)[0] == d
    y = o.dequantize(o.Q6_K, p, 256)
    got = np.rint(y[1:1 + len(vals)] / sd).astype(int).tolist()
    assert got == [1, 2, 3, -1, -2, 30, 7]
    assert p[192] == 127 and p[193] == 1 and not p[194:208].any()
    code = lambda l: (int(p[l]) & 15) | ((int(p[128 + l]) & 3) << 4)  # elements 0..31: low nibble of ql[l], bits 0-1 of qh[l]
    assert code(16) == 0 and code(17) == 63 and code(18) == 32
    assert y[16] == -32 * d and y[17] == 31 * d


def test_q6_k_roundtrip_error_is_what_the_rule_implies():
    rng = np.random.default_rng(62)
    n = 256 * 64
    x = (rng.standard_normal(n) * 0.02).astype(np.float32)
    x[rng.random(n) < 0.01] = 0.5
    packed = o.quantize(o.Q6_K, x)
    y = o.dequantize(o.Q6_K, packed, n)
    assert np.array_equal(y, _q6k_dequant_numpy(packed, n))
    for b, p in enumerate(packed.reshape(-1, 210)):
        d = float(p[208:210].view(np.float16)[0])
        ls = p[192:208].view(np.int8).astype(np.float64)
        xs = x[256 * b:256 * b + 256].astype(np.float64).reshape(16, 16)
        ys = y[256 * b:256 * b + 256].astype(np.float64).reshape(16, 16)
        scales = np.abs(xs).max(1) / 31
        # f16 rounding of d; for weights of this size d is a subnormal f16 (spacing 2^-24), as it is in ggml's files
        d_err = max(scales.max() / 127 * 2 ** -11, 2.0 ** -25)
        assert abs(d - scales.max() / 127) <= d_err
        assert ls.max() == 127 and ls.min() >= 0
        for s in range(16):
            sd = d * ls[s]
            assert abs(sd - scales[s]) <= d * 0.5 + ls[s] * d_err + scales[s] * 2 ** -20, (b, s)
            above = max(0.0, np.abs(xs[s]).max() - 31 * sd)  # how far the 7-bit rounding of the scale pushed the maximum out
            assert np.abs(xs[s] - ys[s]).max() <= max(sd * 0.5, above) + 1e-6 * np.abs(xs[s]).max(), (b, s)


def test_q6_k_tail_superblock_is_zero_padded():
    x = (np.arange(300, dtype=np.float32) - 150) / 64
    p = o.quantize(o.Q6_K, x)
    assert p.size == 2 * 210
    full = o.quantize(o.Q6_K, np.concatenate([x, np.zeros(212, np.float32)]))
    assert np.array_equal(p, full)
    assert o.dequantize(o.Q6_K, p, 300).shape == (300,)


# --------------------------------------------------------------------------- Q5_K (GGUF block; the reference has no such type)
def _q5k_dequant_numpy(packed, numel):
    """ggml's dequantize_row_q5_K transcribed independently in numpy from its published loop: four chunks of 64, masks
    u1 = 1 << 2j and u2 = 2 << 2j into qh[l], low and high nibbles of ql[32j + l]."""
    out = []
    for b in packed.reshape(-1, 176):
        d, dmin = b[0:4].view(np.float16).astype(np.float32)
        sc, qh, ql = b[4:16].astype(np.int32), b[16:48].astype(np.int32), b[48:176].astype(np.int32)
        y = np.zeros(256, np.float32)
        for j in range(4):
            ls, lm = [], []
            for s in (2 * j, 2 * j + 1):
                if s < 4:
                    ls.append(sc[s] & 63), lm.append(sc[s + 4] & 63)
                else:
                    ls.append((sc[s + 4] & 0xF) | ((sc[s - 4] >> 6) << 4)), lm.append((sc[s + 4] >> 4) | ((sc[s] >> 6) << 4))
            d1, m1 = np.float32(d * np.float32(ls[0])), np.float32(dmin * np.float32(lm[0]))
            d2, m2 = np.float32(d * np.float32(ls[1])), np.float32(dmin * np.float32(lm[1]))
            u1, u2 = 1 << (2 * j), 2 << (2 * j)
            for l in range(32):
                y[64 * j + l] = d1 * np.float32((ql[32 * j + l] & 0xF) + (16 if qh[l] & u1 else 0)) - m1
                y[64 * j + 32 + l] = d2 * np.float32((ql[32 * j + l] >> 4) + (16 if qh[l] & u2 else 0)) - m2
        out.append(y)
    return np.concatenate(out)[:numel]


def test_q5_k_layout_one_code_at_a_time():
    # d = 1, dmin = 0, all eight 6-bit scales 1 (bytes typed from get_scale_min_k4's packing: sc[0..3] = 1, sc[8..11] = 1)
    base = np.zeros(176, np.uint8)
    base[0:2] = [0x00, 0x3C]
    base[4:8] = 1
    base[12:16] = 1
    assert not o.dequantize(o.Q5_K, base, 256).any()
    for e, u in [(0, 31), (1, 16), (31, 15), (32, 1), (63, 30), (64, 17), (100, 31), (127, 8), (128, 24), (191, 31), (192, 16), (255, 31)]:
        p, h, l = e >> 6, (e >> 5) & 1, e & 31
        img = base.copy()
        img[48 + 32 * p + l] = (u & 15) << (4 * h)
        img[16 + l] = (u >> 4) << (2 * p + h)
        want = np.zeros(256, np.float32)
        want[e] = u
        assert np.array_equal(o.dequantize(o.Q5_K, img, 256), want), (e, u)


def test_q5_k_dequant_matches_ggml_loop_on_arbitrary_bytes():
    rng = np.random.default_rng(51)
    raw = rng.integers(0, 256, size=(64, 176), dtype=np.uint8)
    raw[:, 0:4] = (rng.standard_normal((64, 2)) * 0.1).astype(np.float16).view(np.uint8)
    assert np.array_equal(o.dequantize(o.Q5_K, raw.reshape(-1), 64 * 256), _q5k_dequant_numpy(raw.reshape(-1), 64 * 256))


def test_q5_k_known_superblock_by_hand():
    """Q4_K's hand-worked superblock with 31 steps: sub-block s spans [-lm_s / 32, ls_s / 64 * 31 - lm_s / 32] with
    hand-picked 6-bit ls and lm (largest 63), so d = f16(63/64 / 63) = 2^-6, dmin = 2^-5, and every x is a grid point."""
    ls = [63, 1, 2, 32, 33, 47, 16, 0]  # sub-block 7 is constant: scale 0, codes 0
    lm = [63, 0, 5, 31, 32, 48, 17, 9]  # sub-block 1 has no negative value: min 0
    q = [[(7 * i + 3 * s) % 32 for i in range(32)] for s in range(8)]  # every code 0..31 once per sub-block
    q[7] = [0] * 32
    x = np.zeros(256, np.float32)
    for s in range(8):
        for i in range(32):
            x[32 * s + i] = ls[s] / 64 * q[s][i] - lm[s] / 32
    scales = [191, 129, 66, 32, 191, 192, 69, 31, 1, 15, 16, 144]  # as in the Q4_K block: the same ls, lm
    got = o.quantize(o.Q5_K, x)
    assert got[:4].tolist() == [0x00, 0x24, 0x00, 0x28] and got[4:16].tolist() == scales
    for s in range(8):
        for i in range(32):
            byte = int(got[48 + 32 * (s >> 1) + i])
            u = ((byte >> 4) if s & 1 else (byte & 15)) | (((int(got[16 + i]) >> s) & 1) << 4)
            assert u == q[s][i], (s, i)
    assert np.array_equal(o.dequantize(o.Q5_K, got, 256), x)


def test_q5_k_zero_and_tail_superblocks():
    p = o.quantize(o.Q5_K, np.zeros(256, np.float32))
    # as Q4_K's zero superblock: every field 0, dmin = -0.0 (the negated minimum of a block of zeros)
    assert p.tolist() == [0, 0, 0, 0x80] + [0] * 172 and not o.dequantize(o.Q5_K, p, 256).any()
    x = (np.arange(300, dtype=np.float32) - 150) / 64
    p = o.quantize(o.Q5_K, x)
    assert p.size == 2 * 176 and np.array_equal(p, o.quantize(o.Q5_K, np.concatenate([x, np.zeros(212, np.float32)])))
    # half-way quotients round away from zero: one sub-block 0..31 (scale 1 -> d = f16(1/63), ls = 63, sd = 63 d)
    x = np.zeros(256, np.float32)
    sd = np.float32(np.float32(np.float16(np.float32(1.0) / np.float32(63.0))) * np.float32(63.0))
    x[0] = 31.0
    for i, v in enumerate([0.5, 1.5, 2.5, 29.5, 30.49]):
        x[1 + i] = np.float32(v) * sd
    y = o.dequantize(o.Q5_K, o.quantize(o.Q5_K, x), 256)
    assert np.rint(y[1:6] / sd).astype(int).tolist() == [1, 2, 3, 30, 30]


def test_q5_k_roundtrip_error_is_what_the_rule_implies():
    rng = np.random.default_rng(53)
    n = 256 * 64
    x = (rng.standard_normal(n) * 0.02).astype(np.float32)
    x[rng.random(n) < 0.01] = 0.5
    packed = o.quantize(o.Q5_K, x)
    y = o.dequantize(o.Q5_K, packed, n)
    assert np.array_equal(y, _q5k_dequant_numpy(packed, n))
    for b, p in enumerate(packed.reshape(-1, 176)):
        d, dmin, ls, lm = _q4k_fields(p[:16])
        xs = x[256 * b:256 * b + 256].astype(np.float64).reshape(8, 32)
        ys = y[256 * b:256 * b + 256].astype(np.float64).reshape(8, 32)
        mins = np.maximum(0.0, -xs.min(1))
        scales = (xs.max(1) + mins) / 31
        # f16 rounding of d and dmin; with 31 steps d falls into f16's subnormal range (spacing 2^-24) for weights of this size
        d_err, m_err = max(scales.max() / 63 * 2 ** -11, 2.0 ** -25), max(mins.max() / 63 * 2 ** -11, 2.0 ** -25)
        assert abs(d - scales.max() / 63) <= d_err and abs(dmin - mins.max() / 63) <= m_err
        for s in range(8):
            sd, sm = d * ls[s], dmin * lm[s]
            assert abs(sd - scales[s]) <= d * 0.5 + ls[s] * d_err + scales[s] * 2 ** -20, (b, s)
            assert abs(sm - mins[s]) <= dmin * 0.5 + lm[s] * m_err + mins[s] * 2 ** -20, (b, s)
            below = max(0.0, mins[s] - sm)
            above = max(0.0, xs[s].max() + sm - 31 * sd)
            bound = max(sd * 0.5, below, above) + 1e-6 * np.abs(xs[s]).max()
            assert np.abs(xs[s] - ys[s]).max() <= bound, (b, s)

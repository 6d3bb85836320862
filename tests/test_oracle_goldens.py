"""Pins the CPU oracle against the reference's own golden vectors, known-answer
tests and closed forms.  Each test names the reference test it restates
(paths relative to the reference root)."""
import numpy as np
import pytest

import oracle as fo
from tests.refdata import k_quant_fixture, q8_0_sample_input

RNG = np.random.default_rng(20240607)


def hexbytes(s):
    return np.frombuffer(bytes.fromhex(s), np.uint8)


# ---------------------------------------------------------------- f16

def test_f16_to_f32_matches_ieee_for_every_bit_pattern():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([fo.f16_to_f32(int(b)) for b in bits], np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_rounds_to_nearest_even():
    # every f16 value's neighbourhood: exact, both half-way points, and one ulp either side
    cases = []
    for b in list(range(0, 0x7C00, 37)) + [0, 1, 2, 0x3FF, 0x400, 0x401, 0x7BFF]:
        lo = np.float32(np.uint16(b).view(np.float16))
        hi = np.float32(np.uint16(b + 1).view(np.float16)) if b + 1 < 0x7C00 else np.float32(65536.0)
        mid = np.float32((np.float64(lo) + np.float64(hi)) / 2)
        for v in (lo, mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(1e9))):
            cases += [v, -v]
    cases += list(RNG.standard_normal(4000).astype(np.float32) * np.float32(0.05))
    cases += [np.float32(65504.0), np.float32(65519.9), np.float32(65520.0), np.float32(1e9),
              np.float32(2.0 ** -25), np.float32(2.0 ** -24), np.float32(1e-10)]
    with np.errstate(over="ignore"):
        for v in cases:
            want = int(np.float32(v).astype(np.float16).view(np.uint16))
            assert fo.f32_to_f16(v) == want, (float(v), hex(want))


# ---------------------------------------------------------------- Q8_0 encoder
# crates/frink-quant/src/encode.rs:165-265

def test_q8_0_matches_llama_cpp_quantize_row_q8_0_ref(vectors):
    got = fo.encode_row(fo.Q8_0, q8_0_sample_input(64))
    assert got.tobytes() == bytes.fromhex(vectors["q8_0_encode_golden"])


def test_q8_0_scale_is_applied_as_a_reciprocal_multiply(vectors):
    x = np.array(vectors["q8_0_tie_block_f16_bits"], np.uint16).view(np.float16).astype(np.float32)
    got = fo.encode_row(fo.Q8_0, x)
    gold = bytes.fromhex(vectors["q8_0_tie_block_golden"])
    assert got.tobytes() == gold
    # the divide spelling differs on this block, so the golden asserts something
    d = np.float32(np.abs(x).max()) / np.float32(127.0)
    divided = np.array([int(np.sign(v) * np.floor(abs(v) + np.float32(0.5))) for v in (x / d)], np.int8)
    assert divided.tobytes() != gold[2:]


def test_q8_0_all_zero_block_is_34_zero_bytes():
    assert fo.encode_row(fo.Q8_0, np.zeros(32, np.float32)).tobytes() == bytes(34)


@pytest.mark.parametrize("kind,ragged", [(fo.Q8_0, 33), (fo.Q8_0, 1), (fo.Q4_K, 257), (fo.Q4_K, 32),
                                         (fo.Q5_K, 257), (fo.Q5_K, 32), (fo.Q6_K, 257), (fo.Q6_K, 16)])
def test_a_ragged_row_is_refused_and_an_empty_one_accepted(kind, ragged):
    assert fo.encode_row(kind, np.full(ragged, 0.5, np.float32)) is None
    assert fo.encode_row(kind, np.zeros(0, np.float32)).size == 0


def test_q8_0_round_trip_is_within_a_quantization_step():
    x = q8_0_sample_input(8 * 32)
    back = fo.dequant(fo.Q8_0, fo.encode_row(fo.Q8_0, x))
    for b in range(8):
        c = x[b * 32:(b + 1) * 32]
        bound = np.abs(c).max() / 127.0 * (0.5 + 127.0 * 2.0 ** -11)
        assert np.abs(c - back[b * 32:(b + 1) * 32]).max() <= bound


# ---------------------------------------------------------------- K-quant encoders
# crates/frink-quant/src/encode/q4_k.rs:152-362, encode/q6_k.rs:221-504

@pytest.fixture(scope="module")
def kfix(vectors):
    return k_quant_fixture(vectors["real_weight_blocks_f16_bits"])


def test_q4_k_matches_llama_cpp_quantize_row_q4_k_ref(vectors, kfix):
    got = fo.encode_row(fo.Q4_K, kfix).reshape(12, 144)
    gold = hexbytes(vectors["q4_k_encode_golden"]).reshape(12, 144)
    for b in range(12):
        assert got[b].tobytes() == gold[b].tobytes(), "super-block %d disagrees with llama.cpp" % b


# crates/frink-quant/src/encode/q5_k.rs:144-305
def test_q5_k_matches_llama_cpp_quantize_row_q5_k_ref(vectors, kfix):
    got = fo.encode_row(fo.Q5_K, kfix).reshape(12, 176)
    gold = hexbytes(vectors["q5_k_encode_golden"]).reshape(12, 176)
    for b in range(12):
        assert got[b].tobytes() == gold[b].tobytes(), "super-block %d disagrees with llama.cpp" % b
    # the fixture uses the fifth bit: some codes are above 15
    assert gold[:, 16:48].any()


def test_q6_k_matches_llama_cpp_quantize_row_q6_k_ref(vectors, kfix):
    got = fo.encode_row(fo.Q6_K, kfix).reshape(12, 210)
    gold = hexbytes(vectors["q6_k_encode_golden"]).reshape(12, 210)
    for b in range(12):
        assert got[b].tobytes() == gold[b].tobytes(), "super-block %d disagrees with llama.cpp" % b


def test_q6_k_all_zero_super_block_is_210_zero_bytes():
    assert fo.encode_row(fo.Q6_K, np.zeros(256, np.float32)).tobytes() == bytes(210)


def test_q6_k_group_scales_are_stored_signed(kfix):
    blocks = fo.encode_row(fo.Q6_K, kfix).reshape(12, 210)
    assert (blocks[:, 192:208].view(np.int8) < 0).any()


def test_q4_k_every_element_lands_on_its_nearest_level(kfix):
    data = fo.encode_row(fo.Q4_K, kfix)
    back = fo.dequant(fo.Q4_K, data)
    blocks = data.reshape(12, 144)
    for b in range(12):
        d = np.float32(blocks[b, 0:2].view(np.float16)[0])
        dmin = np.float32(blocks[b, 2:4].view(np.float16)[0])
        s = blocks[b, 4:16]
        for j in range(8):
            if j < 4:
                sc, m = s[j] & 63, s[j + 4] & 63
            else:
                sc = (s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4)
                m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4)
            dj, dm = d * np.float32(sc), dmin * np.float32(m)
            levels = dj * np.arange(16, dtype=np.float32) - dm
            sl = slice(b * 256 + 32 * j, b * 256 + 32 * j + 32)
            chosen = np.abs(kfix[sl] - back[sl])
            best = np.abs(kfix[sl][:, None] - levels[None, :]).min(axis=1)
            assert (best >= chosen).all(), (b, j)


def test_q6_k_every_element_lands_on_its_nearest_level(kfix):
    data = fo.encode_row(fo.Q6_K, kfix)
    back = fo.dequant(fo.Q6_K, data)
    blocks = data.reshape(12, 210)
    for b in range(12):
        d = np.float32(blocks[b, 208:210].view(np.float16)[0])
        for g in range(16):
            dg = d * np.float32(blocks[b, 192 + g].view(np.int8))
            levels = dg * np.arange(-32, 32, dtype=np.float32)
            sl = slice(b * 256 + 16 * g, b * 256 + 16 * g + 16)
            chosen = np.abs(kfix[sl] - back[sl])
            best = np.abs(kfix[sl][:, None] - levels[None, :]).min(axis=1)
            assert (best >= chosen).all(), (b, g)


# crates/frink-quant/src/encode/fit.rs:601-646
def test_nearest_int_rounds_ties_to_even():
    for f, want in [(0.5, 0), (1.5, 2), (2.5, 2), (-0.5, 0), (-1.5, -2), (3.7, 4), (-3.7, -4), (3.2, 3)]:
        assert fo.nearest_int(f) == want


def test_make_qx_quants_zero_group_and_sign_convention():
    s, l = fo.make_qx_quants(np.zeros(16, np.float32))
    assert s == 0.0 and (l == 0).all()
    x = np.array([1.0, -0.5, 0.25, 0.0, 0.125, -0.75, 0.5, -0.25, 0.0625, -0.0625, 0.3, -0.3, 0.9, -0.9,
                  0.7, -0.1], np.float32)
    s, l = fo.make_qx_quants(x)
    assert s < 0 and l[0] == 0 and l[13] > 32
    x2 = np.full(16, 0.001, np.float32)
    x2[0], x2[7] = 1.0, -0.4
    assert fo.make_qx_quants(x2, 32, 1)[0] != fo.make_qx_quants(x2, 32, 2)[0]


# ---------------------------------------------------------------- dequant
# crates/frink-quant/src/lib.rs:6297-6341, 6423-6529, 7108-7246 (goldens printed to 6 digits: 1e-3)

@pytest.mark.parametrize("kind,blk,gold", [
    (fo.Q4_K, "q4_k_test_block", "q4_k_golden"),
    (fo.Q5_K, "q5_k_test_block", "q5_k_golden"),
    (fo.Q6_K, "q6_k_test_block", "q6_k_golden"),
    (fo.Q6_K, "q6_k_signed_scales_test_block", "q6_k_signed_scales_golden"),
    (fo.Q6_K, "q6_k_signed_test_block", "q6_k_signed_golden"),
])
def test_dequant_matches_independent_python_reference(vectors, kind, blk, gold):
    got = fo.dequant(kind, hexbytes(vectors[blk]))
    want = np.array(vectors[gold], np.float32)
    assert got.shape == want.shape
    assert np.abs(got - want).max() < 1e-3


@pytest.mark.parametrize("kind", [fo.Q4_K, fo.Q5_K, fo.Q6_K])
def test_block_walk_and_index_formula_decoders_agree_bit_for_bit(kind):
    bb, be = fo.BLOCK[kind]
    for _ in range(64):
        blk = RNG.integers(0, 256, bb, dtype=np.uint8)
        # keep the f16 super-scales finite
        for off in ((208,) if kind == fo.Q6_K else (0, 2)):
            blk[off:off + 2] = np.frombuffer(np.float16(RNG.uniform(-0.01, 0.01)).tobytes(), np.uint8)
        walk = fo.dequant(kind, blk)
        elem = np.array([fo.element(kind, blk, i) for i in range(be)], np.float32)
        assert np.array_equal(walk.view(np.uint32), elem.view(np.uint32))


def test_q8_0_dequant_is_q_times_f16_scale():
    blk = RNG.integers(0, 256, 34 * 5, dtype=np.uint8).reshape(5, 34)
    blk[:, 0:2] = np.frombuffer(np.float16([0.01, -0.5, 1.0, 6e-6, 0.0]).tobytes(), np.uint8).reshape(5, 2)
    got = fo.dequant(fo.Q8_0, blk.ravel()).reshape(5, 32)
    want = blk[:, 2:].view(np.int8).astype(np.float32) * blk[:, 0:2].copy().view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


# crates/frink-quant/src/lib.rs:291-310, 5855-5864, 6277-6295: Q4_0 has no vector in the reference beyond closed forms
def test_q4_0_dequant_is_nibble_minus_eight_times_f16_scale():
    blk = np.concatenate([np.frombuffer(np.float16(1.0).tobytes(), np.uint8), np.zeros(16, np.uint8)])
    assert (fo.dequant(fo.Q4_0, blk) == -8.0).all()  # the reference's own case: nibble 0 is -8 * scale
    data = RNG.integers(0, 256, 18 * 7, dtype=np.uint8).reshape(7, 18)
    data[:, 0:2] = np.frombuffer(np.float16([0.01, -0.5, 1.0, 6e-6, 0.0, 3.0, 0.125]).tobytes(), np.uint8).reshape(7, 2)
    got = fo.dequant(fo.Q4_0, data.ravel()).reshape(7, 32)
    d = data[:, 0:2].copy().view(np.float16).astype(np.float32)
    lo = (data[:, 2:] & 15).astype(np.float32) - 8
    hi = (data[:, 2:] >> 4).astype(np.float32) - 8
    want = np.concatenate([lo, hi], axis=1) * d  # element i from byte i's low nibble, i + 16 from its high one
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_q4_0_dots_follow_the_dequantized_row():
    nb = 12
    data = RNG.integers(0, 256, 18 * nb, dtype=np.uint8).reshape(nb, 18)
    data[:, 0:2] = RNG.uniform(-0.05, 0.05, nb).astype(np.float16).view(np.uint8).reshape(nb, 2)
    row = data.ravel()
    x = RNG.standard_normal(32 * nb).astype(np.float32)
    w = fo.dequant(fo.Q4_0, row).astype(np.float64)
    assert abs(fo.dot_f32(fo.Q4_0, row, x) - float(np.dot(w, x.astype(np.float64)))) < 1e-4
    # f32 order: per block the sum of (nibble - 8) * x, elements i and i + 16 alternating, then times the scale
    acc = np.float32(0)
    for b in range(nb):
        blk = data[b]
        ba = np.float32(0)
        for i in range(16):
            ba = np.float32(ba + np.float32(np.float32(int(blk[2 + i] & 15) - 8) * x[32 * b + i]))
            ba = np.float32(ba + np.float32(np.float32(int(blk[2 + i] >> 4) - 8) * x[32 * b + i + 16]))
        acc = np.float32(acc + np.float32(ba * np.float32(blk[0:2].view(np.float16)[0])))
    assert np.float32(fo.dot_f32(fo.Q4_0, row, x)).view(np.uint32) == acc.view(np.uint32)
    # integer dot: exact integers times dw * da, in block order
    q, d = fo.quantize_q8_0(x)
    xa = q.astype(np.float64) * np.repeat(d.astype(np.float64), 32)
    want = float(np.dot(w, xa))
    assert abs(fo.dot_int(fo.Q4_0, row, (q, d)) - want) <= 2e-6 * float(np.abs(w * xa).sum())


def test_a_kind_without_an_encoder_is_refused_not_written_with_another_kinds_blocks():
    for kind in (fo.Q4_0, fo.Q5_0, fo.IQ4_XS, fo.MXFP4):
        with pytest.raises(ValueError):
            fo.encode_matrix(kind, np.zeros((2, 1024), np.float32))


def test_misaligned_buffers_are_refused():
    for kind in (fo.Q4_0, fo.Q8_0, fo.Q4_K, fo.Q5_K, fo.Q6_K):
        with pytest.raises(ValueError):
            fo.dequant(kind, np.zeros(5, np.uint8))


# fused dot == dequant-then-dot (crates/frink-quant/src/lib.rs:6544-6577, 7170-7246)
@pytest.mark.parametrize("kind,blk,freq,fn", [
    (fo.Q4_K, "q4_k_test_block", 0.017, np.sin),
    (fo.Q5_K, "q5_k_test_block", 0.019, np.cos),
    (fo.Q6_K, "q6_k_test_block", 0.021, np.cos),
    (fo.Q6_K, "q6_k_signed_test_block", 0.023, np.sin),
    (fo.Q6_K, "q6_k_signed_scales_test_block", 0.023, np.sin),
])
def test_fused_dot_matches_dequant_then_dot(vectors, kind, blk, freq, fn):
    b = hexbytes(vectors[blk])
    x = fn(np.arange(256, dtype=np.float32) * np.float32(freq)).astype(np.float32)
    expected = float(np.dot(fo.dequant(kind, b).astype(np.float64), x.astype(np.float64)))
    assert abs(fo.dot_f32(kind, b, x) - expected) < 1e-2


def test_q6_k_scalar_dot_matches_python_golden_with_negative_scales(vectors):
    x = np.sin(np.arange(256, dtype=np.float32) * np.float32(0.023)).astype(np.float32)
    expected = float(np.dot(np.array(vectors["q6_k_signed_scales_golden"], np.float64), x.astype(np.float64)))
    got = fo.dot_f32(fo.Q6_K, hexbytes(vectors["q6_k_signed_scales_test_block"]), x)
    assert abs(got - expected) < 1e-2


def _python_order_dot(kind, row, x):
    """dot_q4_k_f32_scalar's / dot_q5_k_f32_scalar's summation order in numpy float32, one op at a time."""
    acc = np.float32(0)
    w = fo.dequant(kind, row)
    for wi, xi in zip(w, x):
        acc = np.float32(acc + np.float32(wi * xi))
    return acc


@pytest.mark.parametrize("kind,blk", [(fo.Q4_K, "q4_k_test_block"), (fo.Q5_K, "q5_k_test_block")])
def test_f32_dot_is_the_sequential_sum_of_dequantized_products(vectors, kind, blk):
    row = np.tile(hexbytes(vectors[blk]), 3)
    x = RNG.standard_normal(768).astype(np.float32)
    got = np.float32(fo.dot_f32(kind, row, x))
    assert got.view(np.uint32) == _python_order_dot(kind, row, x).view(np.uint32)


# ---------------------------------------------------------------- activation quantizers
# crates/frink-quant/src/act_quant.rs:215-300 (libggml's own outputs)

def _block(head, n):
    x = np.zeros(n, np.float32)
    x[:len(head)] = head
    return x


def test_q8_k_rounds_ties_to_even():
    q, d, bs = fo.quantize_q8_k(_block([127.0, 2.5, -3.5, 0.5, -0.5, 126.5], 256))
    assert d[0] == 1.0
    assert list(q[:6]) == [127, 2, -4, 0, 0, 126]
    assert bs[0] == 127 + 2 - 4 + 126


def test_q8_k_takes_its_scale_from_the_inverse():
    amax = np.uint32(0x3FE46A64).view(np.float32)
    x = np.uint32(0x3DD7D365).view(np.float32)
    q, d, _ = fo.quantize_q8_k(_block([-amax, x], 256))
    assert d.view(np.uint32)[0] == 0x3C6636D1
    assert list(q[:2]) == [-127, 8]


def test_q8_k_scale_is_never_negative_and_quants_are_odd_symmetric():
    qn, dn, _ = fo.quantize_q8_k(_block([-127.0, 2.5], 256))
    qp, dp, _ = fo.quantize_q8_k(_block([127.0, -2.5], 256))
    assert (dn[0], dp[0]) == (1.0, 1.0)
    assert (qn[1], qp[1]) == (2, -2)
    assert np.array_equal(qn, -qp)


def test_q8_k_all_zero_block_is_all_zero():
    q, d, bs = fo.quantize_q8_k(np.zeros(256, np.float32))
    assert d[0] == 0.0 and not q.any() and not bs.any()


def test_q8_k_bsums_are_the_16_wide_sums_and_blocks_are_independent():
    x = RNG.standard_normal(1024).astype(np.float32)
    q, d, bs = fo.quantize_q8_k(x)
    assert np.array_equal(bs, q.reshape(-1, 16).astype(np.int32).sum(axis=1).astype(np.int16))
    q1, d1, bs1 = fo.quantize_q8_k(x[256:512])
    assert np.array_equal(q1, q[256:512]) and d1[0] == d[1] and np.array_equal(bs1, bs[16:32])
    # closed form, computed independently in numpy float32
    for b in range(4):
        c = x[b * 256:(b + 1) * 256]
        iscale = np.float32(127.0) / np.abs(c).max()
        assert d[b] == np.float32(1.0) / iscale
        assert np.array_equal(q[b * 256:(b + 1) * 256], np.rint(iscale * c).astype(np.int8))


def test_q8_0_act_forms():
    head = [127.0, 2.5, -3.5, 0.5, 1.5]
    q, d = fo.quantize_q8_0(_block(head, 32), fo.FORM_NEON)
    assert d[0] == 1.0 and list(q[:5]) == [127, 2, -4, 0, 2]
    assert list(fo.quantize_q8_0(_block(head, 32), fo.FORM_AVX)[0][:5]) == [127, 2, -4, 0, 2]
    assert list(fo.quantize_q8_0(_block(head, 32), fo.FORM_SCALAR)[0][:5]) == [127, 3, -4, 1, 2]
    q, d = fo.quantize_q8_0(_block([1.0, 0.5], 32), fo.FORM_NEON)
    assert d[0] == np.float32(np.uint16(0x2008).view(np.float16)) and d[0] != np.float32(1.0) / np.float32(127.0)
    assert list(q[:2]) == [127, 64]
    x = _block([np.uint32(0x4013E709).view(np.float32), np.uint32(0x3CDF99C0).view(np.float32)], 32)
    q, d = fo.quantize_q8_0(x, fo.FORM_NEON)
    assert d[0] == np.float32(np.uint16(0x24A9).view(np.float16)) and list(q[:2]) == [127, 2]
    assert fo.quantize_q8_0(x, fo.FORM_AVX)[0][1] == 1
    for form in (fo.FORM_NEON, fo.FORM_AVX, fo.FORM_SCALAR):
        q, d = fo.quantize_q8_0(np.zeros(32, np.float32), form)
        assert d[0] == 0.0 and not q.any()


# ---------------------------------------------------------------- integer dots
# No reference-held vector exists for these; pinned by the exact identity
#   int_dot(w, q8) == sum_i dequant(w)_i * (q8_i * d_act)      (in exact arithmetic)
# against the vector-pinned dequantizers, and by int-dot ~= f32-dot
# (crates/frink-quant/src/lib.rs:5624-5656, 5756-5808: rel < 0.05).

def _weights(kind, rows, cols, sigma=0.02):
    w = (RNG.standard_normal((rows, cols)) * sigma).astype(np.float32)
    return fo.encode_matrix(kind, w)


@pytest.mark.parametrize("kind", [fo.Q8_0, fo.Q4_K, fo.Q5_K, fo.Q6_K])
def test_int_dot_equals_dequant_dot_in_exact_arithmetic(kind):
    rows, cols = 6, 1024
    bb, be = fo.BLOCK[kind]
    data = _weights(kind, rows, cols)
    row_bytes = cols // be * bb
    x = RNG.standard_normal(cols).astype(np.float32)
    acts = fo.quantize_q8_0(x) if kind == fo.Q8_0 else fo.quantize_q8_k(x)
    q, d = acts[0], acts[1]
    xa = q.astype(np.float64) * np.repeat(d.astype(np.float64), be)
    for r in range(rows):
        row = data[r * row_bytes:(r + 1) * row_bytes]
        # exact-arithmetic value of the dequantized row: Q4_K's d*sc and dmin*m are rounded in the
        # dequantizer but not in the int dot, so rebuild the unrounded weights for Q4_K
        if kind == fo.Q4_K:
            wq = _q4_k_exact(row)
        elif kind == fo.Q5_K:
            wq = _q5_k_exact(row)
        else:
            wq = fo.dequant(kind, row).astype(np.float64)
            if kind == fo.Q6_K:
                wq = _q6_k_exact(row)
        want = float(np.dot(wq, xa))
        got = fo.dot_int(kind, row, acts)
        scale = float(np.abs(wq * xa).sum())
        assert abs(got - want) <= 2e-6 * scale + 1e-12, (kind, r, got, want)
        f32 = fo.dot_f32(kind, row, x)
        assert abs(got - f32) <= 0.05 * max(abs(f32), 0.5)


def _q4_k_exact(row):
    out = []
    for blk in row.reshape(-1, 144):
        d = float(blk[0:2].view(np.float16)[0])
        dmin = float(blk[2:4].view(np.float16)[0])
        s = blk[4:16].astype(int)
        for j in range(8):
            if j < 4:
                sc, m = s[j] & 63, s[j + 4] & 63
            else:
                sc = (s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4)
                m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4)
            qs = blk[16 + (j // 2) * 32:16 + (j // 2) * 32 + 32].astype(int)
            nib = (qs >> 4) if j & 1 else (qs & 15)
            out.append(d * sc * nib - dmin * m)
    return np.concatenate(out)


def _q5_k_exact(row):
    out = []
    for blk in row.reshape(-1, 176):
        d = float(blk[0:2].view(np.float16)[0])
        dmin = float(blk[2:4].view(np.float16)[0])
        s = blk[4:16].astype(int)
        qh = blk[16:48].astype(int)
        for j in range(8):
            if j < 4:
                sc, m = s[j] & 63, s[j + 4] & 63
            else:
                sc = (s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4)
                m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4)
            qs = blk[48 + (j // 2) * 32:48 + (j // 2) * 32 + 32].astype(int)
            code = ((qs >> 4) if j & 1 else (qs & 15)) + 16 * ((qh >> j) & 1)
            out.append(d * sc * code - dmin * m)
    return np.concatenate(out)


def _q6_k_exact(row):
    out = np.empty(row.size // 210 * 256)
    for b, blk in enumerate(row.reshape(-1, 210)):
        d = float(blk[208:210].view(np.float16)[0])
        sc = blk[192:208].view(np.int8).astype(int)
        for i in range(256):
            half, r = divmod(i, 128)
            quarter, l = divmod(r, 32)
            qlb = int(blk[half * 64 + (quarter & 1) * 32 + l])
            lo = (qlb >> 4) if quarter & 2 else (qlb & 15)
            hi = (int(blk[128 + half * 32 + l]) >> (2 * quarter)) & 3
            out[b * 256 + i] = d * sc[i // 16] * ((lo | (hi << 4)) - 32)
    return out


def test_exact_rebuilds_agree_with_the_dequantizers():
    # the float64 rebuilds above are themselves checked against the pinned dequantizers
    for kind, fn in ((fo.Q4_K, _q4_k_exact), (fo.Q5_K, _q5_k_exact), (fo.Q6_K, _q6_k_exact)):
        data = _weights(kind, 2, 512)
        assert np.abs(fn(data) - fo.dequant(kind, data)).max() < 1e-6


# ---------------------------------------------------------------- dispatch level
# crates/frink-core/src/weight_matrix.rs:4747-5350: apply_batch == N x apply; out is [batch][rows]

@pytest.mark.parametrize("kind", [fo.Q8_0, fo.Q4_K, fo.Q5_K, fo.Q6_K, fo.Q5_0, fo.IQ4_XS, fo.MXFP4])
@pytest.mark.parametrize("mode", [fo.F32_DOT, fo.INT_DOT])
def test_gemm_is_batch_times_gemv_and_output_is_batch_major(kind, mode):
    rows, cols, batch = 24, 512, 5
    data = _weights(kind, rows, cols) if kind in (fo.Q8_0, fo.Q4_K, fo.Q5_K, fo.Q6_K) else _random_blocks(kind, rows * cols // fo.BLOCK[kind][1], 77).ravel()
    x = RNG.standard_normal((batch, cols)).astype(np.float32)
    y = fo.gemm(kind, data, rows, cols, x, mode, threads=3)
    assert y.shape == (batch, rows)
    for b in range(batch):
        yb = fo.gemv(kind, data, rows, cols, x[b], mode, threads=1)
        assert np.array_equal(y[b].view(np.uint32), yb.view(np.uint32))
    part = fo.gemm(kind, data, rows, cols, x, mode, row0=8, nrows=8)
    assert np.array_equal(part, y[:, 8:16])
    # against a plain float64 matmul of the dequantized matrix
    w = fo.dequant(kind, data).reshape(rows, cols).astype(np.float64)
    ref = x.astype(np.float64) @ w.T
    tol = 1e-5 if mode == fo.F32_DOT else 0.05
    assert np.abs(y - ref).max() <= tol * np.abs(ref).max()


# ---------------------------------------------------------------- MoE
# crates/frink-moe/src/lib.rs:1345-1404

def test_route_top_k_softmax_kats():
    ids, w = fo.route_top_k_softmax([0.1, 5.0, 0.2, 3.0, -1.0], 2, True)
    assert list(ids) == [1, 3] and abs(w.sum() - 1) < 1e-5 and w[0] > w[1]
    logits = np.arange(1, 9, dtype=np.float32)
    for k in range(1, 9):
        assert abs(fo.route_top_k_softmax(logits, k, True)[1].sum() - 1) < 1e-5
    ids, w = fo.route_top_k_softmax(logits, 3, False)
    assert list(ids) == [7, 6, 5]
    assert np.abs(w - np.array([0.6323223, 0.2326232, 0.0855683], np.float32)).max() < 1e-4
    assert abs(w.sum() - 0.9505138) < 1e-4
    ids2, w2 = fo.route_top_k_softmax(logits, 3, True)
    assert list(ids2) == list(ids) and np.abs(w / w.sum() - w2).max() < 1e-4


def test_silu_and_swiglu_are_the_textbook_forms():
    g = RNG.standard_normal(100).astype(np.float32) * 3
    u = RNG.standard_normal(100).astype(np.float32)
    want = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64))) * u
    assert (np.abs(fo.swiglu(g, u) - want) <= 4e-7 * np.maximum(np.abs(want), 1)).all()
    assert fo.silu(0.0) == 0.0


def _expf_table():
    """2^(i/32) correctly rounded to double, i < 32, from integer arithmetic (the 32nd root of 2^(i + 32*400) by
    five integer square roots), with i/32 taken off the exponent field: the table of glibc's expf."""
    from math import isqrt
    out = []
    for i in range(32):
        v = 1 << (i + 32 * 400)
        for _ in range(5):
            v = isqrt(v)
        low = v & ((1 << 348) - 1)
        assert abs(low - (1 << 347)) > (1 << 300)          # nowhere near a tie: the floors above cannot matter
        m = (v + (1 << 347)) >> 348                         # 53 bits, the leading one included
        out.append((1023 << 52) + (m - (1 << 52)) - ((i << 52) // 32))
    return np.array(out, dtype=np.uint64)


def expf_table_algorithm(x):
    """expf as glibc >= 2.28 computes it (the algorithm the device kernels evaluate, restated in numpy's
    IEEE double arithmetic), with its three results outside the range of a finite, non-zero f32."""
    n = 32.0
    c0, c1, c2 = float.fromhex("0x1.c6af84b912394p-5") / n / n / n, float.fromhex("0x1.ebfce50fac4f3p-3") / n / n, \
        float.fromhex("0x1.62e42ff0c52d6p-1") / n
    inv_ln2_n, shift = float.fromhex("0x1.71547652b82fep+0") * n, float.fromhex("0x1.8p+52")
    x = np.asarray(x, np.float32)
    z = inv_ln2_n * x.astype(np.float64)
    kd = z + shift
    ki = kd.view(np.uint64)
    r = z - (kd - shift)
    s = (_expf_table()[(ki & np.uint64(31)).astype(np.int64)] + (ki << np.uint64(47))).view(np.float64)
    y = (c0 * r + c1) * (r * r) + (c2 * r + 1.0)
    with np.errstate(over="ignore", under="ignore", invalid="ignore"):
        e = (y * s).astype(np.float32)
    e = np.where(x > np.float32(float.fromhex("0x1.62e42ep6")), np.float32(np.inf), e)
    e = np.where(x < np.float32(float.fromhex("-0x1.9d1d9ep6")), np.float32(2.0 ** -149), e)  # glibc's "may underflow" value
    e = np.where(x < np.float32(float.fromhex("-0x1.9fe368p6")), np.float32(0.0), e)
    return e.astype(np.float32)


def test_the_devices_expf_algorithm_is_the_hosts_expf():
    """The device evaluates silu and the router's softmax with glibc's expf algorithm so that a quantizer
    downstream sees a Linux host's bits (Rust's f32::exp is the platform's expf).  Its restatement above,
    with a table derived here from integers, against the oracle's silu (x / (1 + expf(-x)) through this
    host's libm) on four million values: bit for bit."""
    x = np.concatenate([RNG.standard_normal(2_000_000).astype(np.float32) * 4,
                        RNG.uniform(-87.9, 87.9, 2_000_000).astype(np.float32),
                        RNG.uniform(-110, -86, 500_000).astype(np.float32), RNG.uniform(86, 92, 500_000).astype(np.float32),
                        np.array([0.0, -0.0, 1e-30, -1e-30, 87.99, -87.99, 1.0, -1.0, 1e-42, 200.0, -200.0, np.inf, -np.inf],
                                 np.float32)])
    with np.errstate(over="ignore", invalid="ignore"):
        mine = x / (np.float32(1.0) + expf_table_algorithm(-x))
    want = fo.swiglu(x, np.ones_like(x))
    assert np.array_equal(mine.view(np.uint32), want.view(np.uint32))
    # expf itself where silu hides it (1 + e rounds a small e away): softmax weights e(l) / (1 + e(l)) of two
    # logits 0 and l <= 0 through the oracle's router, down to the underflow and past it
    lo = np.concatenate([RNG.uniform(-110, -80, 20_000), RNG.uniform(-30, 0, 20_000)]).astype(np.float32)
    e = expf_table_algorithm(lo)
    for l, el in zip(lo[::40], e[::40]):
        _, w = fo.route_top_k_softmax(np.array([0.0, l], np.float32), 2, False)
        assert w[1].view(np.uint32) == (el / (np.float32(1.0) + el)).view(np.uint32)


def test_moe_batch_equals_per_token_experts_combined():
    E, k, hidden, ffn, batch = 6, 2, 256, 512, 9
    gate = _weights(fo.Q4_K, E * ffn, hidden)
    up = _weights(fo.Q4_K, E * ffn, hidden)
    down = _weights(fo.Q4_K, E * hidden, ffn)
    x = RNG.standard_normal((batch, hidden)).astype(np.float32)
    logits = RNG.standard_normal((batch, E)).astype(np.float32)
    routed = [fo.route_top_k_softmax(l, k, True) for l in logits]
    ids = np.stack([r[0] for r in routed])
    w = np.stack([r[1] for r in routed])
    got = fo.moe_ffn_batch(fo.Q4_K, gate, up, down, E, hidden, ffn, x, ids, w)
    gu = ffn * (hidden // 256) * 144
    dn = hidden * (ffn // 256) * 144
    for b in range(batch):
        acc = np.zeros(hidden, np.float32)
        # accumulation order in the batch path is expert id ascending
        for e in sorted(ids[b]):
            we = w[b][list(ids[b]).index(e)]
            g = fo.gemv(fo.Q4_K, gate[e * gu:(e + 1) * gu], ffn, hidden, x[b])
            u = fo.gemv(fo.Q4_K, up[e * gu:(e + 1) * gu], ffn, hidden, x[b])
            o = fo.gemv(fo.Q4_K, down[e * dn:(e + 1) * dn], hidden, ffn, fo.swiglu(g, u))
            acc = acc + we * o
        assert np.array_equal(got[b].view(np.uint32), acc.view(np.uint32))


def test_moe_per_position_adds_the_slots_in_routing_order():
    """Below 32 tokens the reference runs every position alone (ffn_batch.rs:355) and
    combine_expert_outputs (frink-moe/src/lib.rs:1246-1263) adds the routed slots in routing order;
    the batch path adds them in ascending expert id.  So the two paths agree bit for bit on a token
    whose routing order is ascending, and to rounding otherwise -- and a slot with an id outside the
    experts is left out of both."""
    E, k, hidden, ffn, batch = 8, 3, 256, 256, 7
    gate = _weights(fo.Q4_K, E * ffn, hidden)
    up = _weights(fo.Q4_K, E * ffn, hidden)
    down = _weights(fo.Q4_K, E * hidden, ffn)
    x = RNG.standard_normal((batch, hidden)).astype(np.float32)
    logits = RNG.standard_normal((batch, E)).astype(np.float32)
    routed = [fo.route_top_k_softmax(l, k, True) for l in logits]
    ids = np.stack([r[0] for r in routed]).astype(np.int32)
    w = np.stack([r[1] for r in routed])
    ids[0] = np.sort(ids[0])           # ascending routing order: both paths add in the same order
    ids[1] = np.sort(ids[1])[::-1]     # descending: the orders differ
    ids[2, 1] = E                      # an id outside the experts
    ids[3, 0] = -1
    per_pos = fo.moe_ffn_per_position(fo.Q4_K, gate, up, down, E, hidden, ffn, x, ids, w)
    bucket = fo.moe_ffn_batch(fo.Q4_K, gate, up, down, E, hidden, ffn, x, ids, w)
    assert np.array_equal(per_pos[0].view(np.uint32), bucket[0].view(np.uint32))
    assert np.abs(per_pos - bucket).max() <= 2e-6 * np.abs(bucket).max()
    gu, dn = ffn * (hidden // 256) * 144, hidden * (ffn // 256) * 144
    for b in range(batch):
        acc = np.zeros(hidden, np.float32)
        for s in range(k):  # routing order
            e = int(ids[b, s])
            if not 0 <= e < E:
                continue
            g = fo.gemv(fo.Q4_K, gate[e * gu:(e + 1) * gu], ffn, hidden, x[b])
            u = fo.gemv(fo.Q4_K, up[e * gu:(e + 1) * gu], ffn, hidden, x[b])
            o = fo.gemv(fo.Q4_K, down[e * dn:(e + 1) * dn], hidden, ffn, fo.swiglu(g, u))
            acc = acc + o * w[b, s]
        assert np.array_equal(per_pos[b].view(np.uint32), acc.view(np.uint32)), b
    # the dispatcher follows the reference's threshold
    assert np.array_equal(fo.moe_ffn(fo.Q4_K, gate, up, down, E, hidden, ffn, x, ids, w), per_pos)


def test_cpu_baseline_legs_agree_with_the_scalar_oracle():
    """The AVX2 forms bench.py times beside the GPU: the integer dot must equal the scalar oracle's bit
    for bit (exact integers, the same float expression); the f32 dot keeps eight partial sums a
    sub-block where the scalar form keeps one, so it is held to fp32 reassociation only (no vector of
    the reference pins it: it is timed, never used as a checker)."""
    if not fo.have_avx2():
        pytest.skip("no AVX2+FMA on this host")
    rng = np.random.default_rng(5)
    rows, cols = 96, 1024
    w = fo.encode_matrix(fo.Q4_K, (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32))
    x = rng.standard_normal((7, cols)).astype(np.float32)
    x[3] = 0.0
    got = fo.avx2_gemm_q4_k_q8k(w, rows, cols, x, threads=3)
    want = fo.gemm(fo.Q4_K, w, rows, cols, x, fo.INT_DOT, 2)
    assert np.array_equal(got, want)
    f = fo.avx2_gemv_q4_k_f32(w, rows, cols, x[0], threads=2)
    wf = fo.gemv(fo.Q4_K, w, rows, cols, x[0], fo.F32_DOT, 1)
    assert np.abs(f - wf).max() <= 2e-6 * np.abs(wf).max()


def test_bench_reads_the_host_cpu():
    import bench
    h = bench.host_cpu()
    assert 1 <= h["physical_cores"] <= h["logical_cpus"] and isinstance(h["cpu_model"], str)


# ---------------------------------------------------------------- Q5_0, IQ4_XS, MXFP4

def _vectors():
    import json
    import os
    return json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "frink_quant_vectors.json")))


def _random_blocks(kind, n, seed):
    """valid blocks of Q5_0 / IQ4_XS / MXFP4 with finite scales, all code values in play"""
    bb, _ = fo.BLOCK[kind]
    rng = np.random.default_rng(seed)
    blocks = rng.integers(0, 256, (n, bb), dtype=np.uint8)
    if kind == fo.MXFP4:
        blocks[:, 0] = rng.integers(100, 140, n)  # 2^-27 .. 2^12
    else:
        blocks[:, 0:2] = rng.uniform(-0.1, 0.1, n).astype(np.float16).view(np.uint8).reshape(n, 2)
    return blocks


def test_iq4_xs_dequant_matches_the_reference_golden():
    # iq4_xs_dequant_matches_independent_python_reference (crates/frink-quant/src/lib.rs:7480-7490); the golden is
    # printed to six digits
    v = _vectors()
    got = fo.dequant(fo.IQ4_XS, hexbytes(v["iq4_xs_test_block"]))
    want = np.array(v["iq4_xs_golden"], np.float32)
    assert np.abs(got - want).max() <= 6e-6 * np.abs(want).max() and np.abs(want).max() > 100


def test_mxfp4_dequant_matches_the_reference_goldens():
    # mxfp4_gguf_dequant_matches_independent_python_reference (lib.rs:7056-7066): powers of two, exact
    v = _vectors()
    got = fo.dequant(fo.MXFP4, hexbytes(v["mxfp4_gguf_test_blocks"]))
    assert np.array_equal(got, np.array(v["mxfp4_gguf_golden"], np.float32))
    # the two-buffer form's vectors (mxfp4_dequant_matches_independent_python_reference, lib.rs:7588-7599) through the block
    # form: scale bytes 0x00 (the subnormal 2^-127) and 0x82
    packed, scales = hexbytes(v["mxfp4_test_packed"]).reshape(2, 16), hexbytes(v["mxfp4_test_scales"])
    blocks = np.concatenate([np.concatenate([[scales[i]], packed[i]]) for i in range(2)]).astype(np.uint8)
    got = fo.dequant(fo.MXFP4, blocks)
    want = np.array(v["mxfp4_golden"], np.float64)
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max() and np.abs(got[:32]).max() < 1e-37
    # mxfp4_scale_byte_zero_and_max_match_the_e8m0_formula (lib.rs:7613-7620)
    assert fo.lib().fo_e8m0_scale(0) == 2.0 ** -127 and fo.lib().fo_e8m0_scale(127) == 1.0 and fo.lib().fo_e8m0_scale(254) == 2.0 ** 127


def test_q5_0_known_answers():
    # q5_0_fifth_bit_extends_range_past_a_plain_nibble (lib.rs:5886-5910)
    blk = np.zeros(22, np.uint8)
    blk[0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blk[2] = 1
    blk[6] = 0x0F
    out = fo.dequant(fo.Q5_0, blk)
    assert out[0] == 15.0 and (out[1:] == -16.0).all()
    # every element from the published layout by index arithmetic: q = nibble | bit (j or j + 16) of qh << 4
    blocks = _random_blocks(fo.Q5_0, 50, 5)
    got = fo.dequant(fo.Q5_0, blocks.ravel()).reshape(50, 32)
    for b in range(50):
        d = np.float32(blocks[b, 0:2].copy().view(np.float16)[0])
        qh = int(blocks[b, 2:6].copy().view(np.uint32)[0])
        for i in range(32):
            nib = (blocks[b, 6 + i % 16] >> (4 * (i // 16))) & 15
            q = int(nib) | (((qh >> i) & 1) << 4)
            assert got[b, i] == np.float32(q - 16) * d


@pytest.mark.parametrize("kind", [fo.Q5_0, fo.IQ4_XS, fo.MXFP4])
def test_f32_dots_of_the_other_kinds_are_the_dequantized_dot(kind):
    # (the reference's *_fused_dot_matches_dequant_then_dot tests, lib.rs:7068-7082, 7492-7502): the fused dot adds the
    # same products left to right, so it equals the dequantized row's sequential f32 dot bit for bit
    bb, be = fo.BLOCK[kind]
    cols = 1024
    blocks = _random_blocks(kind, 6 * cols // be, 11 + kind)
    x = np.random.default_rng(kind).standard_normal(cols).astype(np.float32)
    got = fo.gemv(kind, blocks.ravel(), 6, cols, x, fo.F32_DOT, 1)
    deq = fo.dequant(kind, blocks.ravel()).reshape(6, cols)
    for r in range(6):
        acc = np.float32(0)
        if kind == fo.Q5_0 or kind == fo.MXFP4 or kind == fo.IQ4_XS:
            # element pairs (j, j + 16) of each group of 32, in that order
            for g in range(cols // 32):
                for j in range(16):
                    acc = np.float32(acc + deq[r, 32 * g + j] * x[32 * g + j])
                    acc = np.float32(acc + deq[r, 32 * g + 16 + j] * x[32 * g + 16 + j])
        assert got[r] == acc


def test_the_integer_tiers_decoders_are_the_dequantizers_values():
    """legacy_q8.rs:108-161: a Q5_0 / MXFP4 block decodes to 32 small integers and one scale whose product is the
    dequantized value -- bit for bit, for every code, every fifth bit and every E8M0 scale byte (the doubled E2M1 table
    goes with the HALVED scale 2^(e - 128), subnormal patterns for e < 2 included)."""
    import ctypes as C
    L = fo.lib()
    w = np.zeros(32, np.int8)
    # MXFP4: every scale byte x every code (255 is not a finite scale)
    for e in range(255):
        blk = np.concatenate([[e], (np.arange(16) * 17) % 256]).astype(np.uint8)  # byte j = code j in both nibbles
        L.fo_decode_mxfp4_block(blk.ctypes.data_as(C.POINTER(C.c_uint8)), w.ctypes.data_as(C.POINTER(C.c_int8)))
        half = np.float32(L.fo_e8m0_half_scale(e))
        assert half == np.float32(2.0) ** np.float32(e - 128) or e < 2
        got, want = w.astype(np.float32) * half, fo.dequant(fo.MXFP4, blk)
        # (code 8 is -0.0 in the E2M1 table and the integer 0 here: equal as values, which is all a dot can see)
        nz = want != 0
        assert np.array_equal(got, want) and np.array_equal(got[nz].view(np.uint32), want[nz].view(np.uint32)), e
    assert np.float32(L.fo_e8m0_half_scale(0)).view(np.uint32) == 0x00200000 and np.float32(L.fo_e8m0_half_scale(1)).view(np.uint32) == 0x00400000
    assert w.tolist()[:16] == [0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12]
    # Q5_0: random blocks, scale 1.0 so that the dequantized values are the integers themselves
    blocks = _random_blocks(fo.Q5_0, 200, 21)
    blocks[:, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    deq = fo.dequant(fo.Q5_0, blocks.ravel()).reshape(200, 32)
    for b in range(200):
        L.fo_decode_q5_0_block(blocks[b].ctypes.data_as(C.POINTER(C.c_uint8)), w.ctypes.data_as(C.POINTER(C.c_int8)))
        assert np.array_equal(w.astype(np.float32), deq[b]) and w.min() >= -16 and w.max() <= 15


@pytest.mark.parametrize("kind", [fo.Q5_0, fo.MXFP4, fo.IQ4_XS])
def test_the_other_kinds_integer_dots_in_exact_arithmetic(kind):
    """dot_q5_0_q8 / dot_mxfp4_q8 (legacy_q8.rs:169-213, Q8_0 activation blocks) and dot_iq4_xs_q8_k
    (iq4_xs_q8.rs:67-98, Q8_K activations): the dot of the dequantized row with the dequantized activation, to f32
    rounding of a handful of operations per block -- exact integers inside a block, so a wrong element order, sign,
    sub-scale or scale shows at once.  And the reference's own invariant: within 5 % of the f32 dot."""
    bb, be = fo.BLOCK[kind]
    cols, rows = 1024, 8
    blocks = _random_blocks(kind, rows * cols // be, 31 + kind).reshape(rows, -1)
    x = np.random.default_rng(100 + kind).standard_normal(cols).astype(np.float32)
    if kind == fo.IQ4_XS:
        q, d, bs = fo.quantize_q8_k(x)
        acts = (q, d, bs)
        xa = q.astype(np.float64) * np.repeat(d.astype(np.float64), 256)
    else:
        q, d = fo.quantize_q8_0(x)
        acts = (q, d)
        xa = q.astype(np.float64) * np.repeat(d.astype(np.float64), 32)
    for r in range(rows):
        w = fo.dequant(kind, blocks[r]).astype(np.float64)
        want = float(np.dot(w, xa))
        got = fo.dot_int(kind, blocks[r], acts)
        assert abs(got - want) <= 2e-6 * float(np.abs(w * xa).sum())
        f32 = fo.dot_f32(kind, blocks[r], x)
        assert abs(got - f32) <= 0.05 * max(abs(f32), float(np.abs(w * xa).sum()) / np.sqrt(cols))
    # the dispatch level takes the same functions: gemv in integer mode, every row
    y = fo.gemv(kind, blocks.ravel(), rows, cols, x, fo.INT_DOT, 1)
    for r in range(rows):
        assert np.float32(fo.dot_int(kind, blocks[r], acts)).view(np.uint32) == y[r].view(np.uint32)
    # float order of one row, one operation at a time (scale * isum first, then the activation's scale)
    blk = blocks[0].reshape(-1, bb)
    acc = np.float32(0)
    if kind != fo.IQ4_XS:
        for b in range(cols // 32):
            wq = np.rint(fo.dequant(kind, blk[b]).astype(np.float64) / _unit_scale(kind, blk[b])).astype(np.int64)
            isum = int(np.dot(wq, q[32 * b:32 * b + 32].astype(np.int64)))
            acc = np.float32(acc + np.float32(d[b] * np.float32(np.float32(_unit_scale(kind, blk[b])) * np.float32(isum))))
        assert np.float32(fo.dot_int(kind, blocks[0], acts)).view(np.uint32) == acc.view(np.uint32)


def _unit_scale(kind, blk):
    if kind == fo.Q5_0:
        return float(blk[0:2].copy().view(np.float16)[0])
    return float(np.float32(fo.lib().fo_e8m0_half_scale(int(blk[0]))))

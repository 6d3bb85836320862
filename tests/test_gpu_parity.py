"""Parity of the HIP path against the CPU oracle, through the C ABI, on a real MI355X.

Gates (crates and lines are the reference's):
  * bit-exact: dequantized weights (dequant_q8_0 / dequant_q4_k / dequant_q6_k,
    crates/frink-quant/src/lib.rs:271-286, 334-364, 519-552) and activation quantization
    (quantize_activations_q8_k / quantize_activations_q8, crates/frink-quant/src/act_quant.rs:69-189);
  * fp32 outputs: max |err| <= 1e-3 * ||y||_inf per output row of the batch.
"""
import numpy as np
import pytest

import oracle as fo

pytestmark = pytest.mark.gpu

TOL = 1e-3  # of ||y||_inf, per activation row


@pytest.fixture(scope="module")
def fa():
    import torch
    assert torch.cuda.is_available(), "these tests need a GPU"
    import frink_amd
    info = frink_amd.probe()
    assert info["gcn_arch"].startswith("gfx950"), info
    print("device:", info, flush=True)
    return frink_amd


def to_dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def make_weights(kind, rows, cols, seed, sigma=0.02):
    from frink_amd import synth
    return fo.encode_matrix(kind, synth.weights(seed, rows, cols, sigma))


def record(what, value):
    """Measured worst-row figures survive `pytest -q` in a file, in the folder FRK_TEST_OUT names (if it does)."""
    import os
    d = os.environ.get("FRK_TEST_OUT", "")
    if d and os.path.isdir(d):
        with open(os.path.join(d, "parity_worst_rows.txt"), "a") as f:
            f.write("%s\t%.6g\n" % (what, value))


def assert_rows_close(got, want, what):
    got = np.asarray(got, np.float32).reshape(want.shape)
    for b in range(want.shape[0]):
        ninf = np.abs(want[b]).max()
        err = np.abs(got[b] - want[b]).max()
        assert err <= TOL * ninf, "%s: row %d max|err| %.3g > %.3g (||y||inf %.3g)" % (what, b, err, TOL * ninf, ninf)


# ------------------------------------------------------------------ dequant (bit-exact)

@pytest.mark.parametrize("kind,rows,cols", [
    (fo.Q4_K, 33, 4096), (fo.Q4_K, 5, 256), (fo.Q4_K, 7, 768),
    (fo.Q5_K, 33, 4096), (fo.Q5_K, 5, 256), (fo.Q5_K, 7, 768),
    (fo.Q6_K, 9, 14336), (fo.Q6_K, 5, 256), (fo.Q6_K, 3, 768),
    (fo.Q8_0, 17, 4096), (fo.Q8_0, 4, 32), (fo.Q8_0, 3, 96),
])
def test_dequant_is_bit_exact(fa, kind, rows, cols):
    data = make_weights(kind, rows, cols, seed=100 + kind)
    w = fa.Weights.from_host(kind, data, rows, cols)
    got = w.dequant().cpu().numpy()
    want = fo.dequant(kind, data).reshape(rows, cols)
    assert np.array_equal(bits(got), bits(want))
    w.release()


def test_dequant_of_arbitrary_block_bytes_is_bit_exact(fa):
    # any byte pattern is a structurally valid block; only the f16 super-scales are kept finite
    rng = np.random.default_rng(7)
    for kind, offs in ((fo.Q4_K, (0, 2)), (fo.Q5_K, (0, 2)), (fo.Q6_K, (208,)), (fo.Q8_0, (0,))):
        bb, be = fo.BLOCK[kind]
        rows, nb = 6, 4
        data = rng.integers(0, 256, rows * nb * bb, dtype=np.uint8).reshape(rows * nb, bb)
        for off in offs:
            data[:, off:off + 2] = rng.uniform(-0.05, 0.05, rows * nb).astype(np.float16).view(np.uint8).reshape(-1, 2)
        data = data.ravel()
        w = fa.Weights.from_host(kind, data, rows, nb * be)
        got = w.dequant().cpu().numpy()
        assert np.array_equal(bits(got), bits(fo.dequant(kind, data).reshape(rows, nb * be))), kind
        w.release()


def test_dequant_of_the_reference_golden_blocks(fa, vectors):
    for kind, blk, gold in ((fo.Q4_K, "q4_k_test_block", "q4_k_golden"), (fo.Q5_K, "q5_k_test_block", "q5_k_golden"),
                            (fo.Q6_K, "q6_k_test_block", "q6_k_golden"),
                            (fo.Q6_K, "q6_k_signed_scales_test_block", "q6_k_signed_scales_golden"),
                            (fo.Q6_K, "q6_k_signed_test_block", "q6_k_signed_golden")):
        data = np.frombuffer(bytes.fromhex(vectors[blk]), np.uint8)
        w = fa.Weights.from_host(kind, data, 1, 256)
        got = w.dequant().cpu().numpy().ravel()
        assert np.abs(got - np.array(vectors[gold], np.float32)).max() < 1e-3
        w.release()


@pytest.mark.parametrize("kind", [fo.Q4_0, fo.Q8_0, fo.Q4_K, fo.Q5_K, fo.Q6_K])
def test_get_rows_is_the_dequantized_row_bit_for_bit(fa, kind):
    """The embedding gather (crates/frink-cuda/src/get_rows.rs): row r of the output is the dequantized
    row ids[r] of the table -- repeated ids, the first and last rows, an empty list; the host form
    refuses an id outside the table, the device form reads the nearest row for it."""
    import torch
    rows, cols = 300, 768
    bb, be = fo.BLOCK[kind]
    rng = np.random.default_rng(kind)
    data = rng.integers(0, 256, rows * cols // be * bb, dtype=np.uint8).reshape(-1, bb)
    for off in {fo.Q6_K: (208,), fo.Q4_0: (0,), fo.Q8_0: (0,)}.get(kind, (0, 2)):
        data[:, off:off + 2] = rng.uniform(-0.05, 0.05, data.shape[0]).astype(np.float16).view(np.uint8).reshape(-1, 2)
    data = data.ravel()
    table = fo.dequant(kind, data).reshape(rows, cols)
    w = fa.Weights.from_host(kind, data, rows, cols)
    ids = np.array([0, 299, 17, 17, 150, 1, 298, 0], np.int32)
    got = w.get_rows(torch.from_numpy(ids).cuda()).cpu().numpy()
    assert np.array_equal(bits(got), bits(table[ids]))
    assert np.array_equal(bits(w.get_rows_host(ids)), bits(table[ids]))
    assert w.get_rows_host(np.zeros(0, np.int32)).shape == (0, cols)
    for bad in (300, -1):
        with pytest.raises(fa.BackendError) as e:
            w.get_rows_host(np.array([3, bad], np.int32))
        assert e.value.code == fa.ERR_SHAPE and "300 rows" in str(e.value)
    near = w.get_rows(torch.tensor([300, -5, 1 << 30], dtype=torch.int32).cuda()).cpu().numpy()
    assert np.array_equal(bits(near), bits(table[[299, 0, 299]]))
    w.release()


def test_weights_from_device_bytes_match_from_host(fa):
    data = make_weights(fo.Q6_K, 8, 512, seed=5)
    a = fa.Weights.from_host(fo.Q6_K, data, 8, 512)
    b = fa.Weights.from_device(fo.Q6_K, to_dev(data), 8, 512)
    assert np.array_equal(bits(a.dequant().cpu().numpy()), bits(b.dequant().cpu().numpy()))


# ------------------------------------------------------------------ activation quantizers (bit-exact)

def _q8k_cases():
    from frink_amd import synth
    head = lambda h: np.concatenate([np.array(h, np.float32), np.zeros(256 - len(h), np.float32)])
    amax = np.uint32(0x3FE46A64).view(np.float32)
    xx = np.uint32(0x3DD7D365).view(np.float32)
    return {
        "ties": head([127.0, 2.5, -3.5, 0.5, -0.5, 126.5]),
        "inverse_scale": head([-amax, xx]),
        "zero": np.zeros(256, np.float32),
        "normal": synth.activations(11, 8, 4096).ravel(),
        "outliers": synth.activations(12, 16, 4096, outlier_frac=0.01).ravel(),
        "tiny": synth.normal(13, 1024, 1e-30),
        "huge": synth.normal(14, 1024, 1e30),
        "wide": synth.activations(15, 2, 14336).ravel(),
        # f32::clamp keeps a NaN and `as i8` makes it 0; an infinity makes the inverse scale 0 and the scale infinite
        "nans": _with(synth.activations(16, 1, 2048).ravel(), {3: np.nan, 300: -np.nan, 511: np.nan, 1024: np.nan}),
        "infinities": _with(synth.activations(17, 1, 1024).ravel(), {5: np.inf, 6: -np.inf, 700: np.inf, 701: np.nan}),
        "all_nan": np.full(256, np.nan, np.float32),
        # a block of subnormal values: 127 / amax overflows to infinity, the clamp binds and the scale is zero
        "subnormal": (synth.normal(18, 512, 1.0) * np.float32(1e-40)).astype(np.float32),
        "smallest_normals": (synth.normal(19, 512, 1.0) * np.float32(3e-37)).astype(np.float32),
    }


def _with(x, values):
    x = x.copy()
    for i, v in values.items():
        x[i] = v
    return x


def test_quantize_q8_k_is_bit_exact(fa):
    for name, x in _q8k_cases().items():
        q, d, bs = fa.quantize_q8_k(to_dev(x))
        wq, wd, wbs = fo.quantize_q8_k(x)
        assert np.array_equal(q.cpu().numpy(), wq), name
        assert np.array_equal(bits(d.cpu().numpy()), bits(wd)), name
        assert np.array_equal(bs.cpu().numpy(), wbs), name


def test_quantize_q8_k_kats(fa):
    c = _q8k_cases()
    q, d, bs = fa.quantize_q8_k(to_dev(c["ties"]))
    assert d.cpu().numpy()[0] == 1.0 and list(q.cpu().numpy()[:6]) == [127, 2, -4, 0, 0, 126]
    assert bs.cpu().numpy()[0] == 251
    q, d, _ = fa.quantize_q8_k(to_dev(c["inverse_scale"]))
    assert bits(d.cpu().numpy())[0] == 0x3C6636D1 and list(q.cpu().numpy()[:2]) == [-127, 8]


def test_quantize_q8_0_is_bit_exact(fa):
    from frink_amd import synth
    head = lambda h: np.concatenate([np.array(h, np.float32), np.zeros(32 - len(h), np.float32)])
    cases = [head([127.0, 2.5, -3.5, 0.5, 1.5]), head([1.0, 0.5]), np.zeros(32, np.float32),
             head([np.uint32(0x4013E709).view(np.float32), np.uint32(0x3CDF99C0).view(np.float32)]),
             synth.activations(21, 4, 4096).ravel(), synth.normal(22, 320, 1e-6),
             _with(synth.activations(23, 1, 256).ravel(), {3: np.nan, 40: np.inf, 41: 1.0, 100: -np.nan}),
             np.full(32, np.nan, np.float32),
             (synth.normal(24, 320, 1.0) * np.float32(1e-40)).astype(np.float32),
             (synth.normal(25, 320, 1.0) * np.float32(3e-37)).astype(np.float32)]
    for x in cases:
        q, d = fa.quantize_q8_0(to_dev(x))
        wq, wd = fo.quantize_q8_0(x, fo.FORM_AVX)
        assert np.array_equal(q.cpu().numpy(), wq)
        assert np.array_equal(bits(d.cpu().numpy()), bits(wd))


# ------------------------------------------------------------------ GEMV

GEMV_SHAPES = [
    (fo.Q4_K, 64, 4096), (fo.Q4_K, 37, 4096), (fo.Q4_K, 19, 2048), (fo.Q4_K, 21, 768), (fo.Q4_K, 9, 256),
    (fo.Q4_K, 6, 14336),
    (fo.Q5_K, 64, 4096), (fo.Q5_K, 37, 4096), (fo.Q5_K, 19, 2048), (fo.Q5_K, 21, 768), (fo.Q5_K, 9, 256), (fo.Q5_K, 6, 14336),
    (fo.Q6_K, 48, 14336), (fo.Q6_K, 13, 4096), (fo.Q6_K, 11, 768), (fo.Q6_K, 9, 256), (fo.Q6_K, 5, 2048),
    (fo.Q8_0, 64, 4096), (fo.Q8_0, 7, 32), (fo.Q8_0, 9, 544), (fo.Q8_0, 5, 2048),
    (fo.Q8_0, 1030, 4096), (fo.Q8_0, 1025, 8192), (fo.Q8_0, 40, 8192), (fo.Q8_0, 1100, 5120), (fo.Q8_0, 33, 6144),
    (fo.Q8_0, 12, 16384),
    # Q8_0 rows of 8224 .. 16384 columns with at least 1024 rows: the activation shared through LDS, 11 to 16 units a lane
    (fo.Q8_0, 1024, 14336), (fo.Q8_0, 1500, 11008), (fo.Q8_0, 1027, 16384), (fo.Q8_0, 1100, 8704), (fo.Q8_0, 1030, 10240),
    (fo.Q8_0, 1025, 22016), (fo.Q8_0, 1030, 28672), (fo.Q8_0, 1024, 18432), (fo.Q8_0, 40, 28672), (fo.Q8_0, 1024, 28704),
    # (the wavefronts split the columns: rows that fill a workgroup's four or eight and do not, a last wavefront short of units)
    (fo.Q8_0, 1, 1056), (fo.Q8_0, 3, 16384), (fo.Q8_0, 4, 1088), (fo.Q8_0, 13, 3104), (fo.Q8_0, 9000, 2048), (fo.Q8_0, 8197, 4096),
]


@pytest.mark.parametrize("kind,rows,cols", GEMV_SHAPES)
def test_gemv_matches_the_oracle(fa, kind, rows, cols):
    from frink_amd import synth
    print("gemv", kind, rows, cols, flush=True)
    data = make_weights(kind, rows, cols, seed=rows * 7 + cols)
    x = synth.activations(rows + cols, 1, cols)[0]
    w = fa.Weights.from_host(kind, data, rows, cols)
    # K-quants: integer dots against Q8_K activations.  Q8_0: the f32 dot (no activation
    # quantization), and the integer tier as a second mode.
    mode = fo.F32_DOT if kind == fo.Q8_0 else fo.INT_DOT
    want = fo.gemv(kind, data, rows, cols, x, mode)
    got = w.gemv(to_dev(x), act_mode=fa.ACT_F32).cpu().numpy()
    assert_rows_close(got[None], want[None], "gemv kind %d %dx%d" % (kind, rows, cols))
    if kind == fo.Q8_0:
        want_i = fo.gemv(kind, data, rows, cols, x, fo.INT_DOT)
        got_i = w.gemv(to_dev(x), act_mode=fa.ACT_INT8).cpu().numpy()
        assert_rows_close(got_i[None], want_i[None], "gemv q8_0 int tier")
    w.release()


@pytest.mark.parametrize("rows,cols", [(1, 6144), (16, 6144), (17, 8192), (100, 11008), (31, 13824), (64, 14336), (33, 16384),
                                       (5, 6400), (40, 7168), (9, 256), (70, 1024), (33, 1792), (40, 2048), (21, 5120),
                                       (4101, 6144), (10243, 6144), (12290, 6144), (5120, 13824)])
def test_q6_k_gemv_with_the_columns_split_between_wavefronts(fa, rows, cols):
    """Q6_K rows of 20 blocks and more (and of 8 and fewer), one launch: a wavefront takes four blocks of columns of
    the workgroup's 4 .. 24 rows and quantizes exactly those blocks itself.  Row counts that fill a workgroup, fall
    short and leave a short last one, at every number of rows to a workgroup the launch picks (the large row counts:
    random block bytes, encoding that many rows takes too long); block counts that fill the last wavefront's four
    and do not."""
    from bench import random_blocks
    from frink_amd import synth
    data = random_blocks(fo.Q6_K, rows, cols, rows + cols) if rows > 2000 else make_weights(fo.Q6_K, rows, cols, seed=rows * 5 + cols)
    x = synth.activations(rows + 2 * cols, 1, cols, outlier_frac=0.01)[0]
    w = fa.Weights.from_host(fo.Q6_K, data, rows, cols)
    want = fo.gemv(fo.Q6_K, data, rows, cols, x, fo.INT_DOT)
    got = w.gemv(to_dev(x)).cpu().numpy()
    assert_rows_close(got[None], want[None], "q6_k columns form %dx%d" % (rows, cols))
    w.release()


@pytest.mark.parametrize("kind,rows,cols", [(fo.Q4_K, 40, 4096), (fo.Q4_K, 9, 1024), (fo.Q4_K, 20, 11008), (fo.Q5_K, 33, 4096),
                                            (fo.Q6_K, 20, 4096), (fo.Q6_K, 20, 14336), (fo.Q6_K, 7, 768)])
def test_gemv_quantizes_a_nan_to_zero_inside_the_launch(fa, kind, rows, cols):
    """quantize_activations_q8_k makes a NaN activation a zero quant (f32::clamp keeps the NaN, `as i8` makes it 0)
    and leaves it out of the block's maximum: the kernels that quantize inside the launch must do the same."""
    from frink_amd import synth
    data = make_weights(kind, rows, cols, seed=rows + cols)
    x = synth.activations(rows + cols + 1, 1, cols)[0].copy()
    x[[1, 77, 255, 256, cols - 1]] = np.nan
    w = fa.Weights.from_host(kind, data, rows, cols)
    want = fo.gemv(kind, data, rows, cols, x, fo.INT_DOT)
    assert np.isfinite(want).all()
    got = w.gemv(to_dev(x)).cpu().numpy()
    assert_rows_close(got[None], want[None], "gemv with NaN activations, kind %d %dx%d" % (kind, rows, cols))
    w.release()


@pytest.mark.parametrize("rows,cols", [(5, 2048), (8, 2048), (100, 2048), (1, 4096), (4, 4096), (131, 4096), (3, 8192), (50, 8192),
                                       (1, 16384), (33, 16384), (4100, 4096), (10301, 4096), (14336, 4096), (8200, 2048),
                                       (4096, 8192)])
@pytest.mark.parametrize("kind", [fo.Q4_K, fo.Q5_K])
def test_q4_k_gemv_over_whole_cache_lines(fa, kind, rows, cols):
    """Rows of 2048 .. 16384 columns take the kernel that gives a wavefront 64 consecutive blocks (8, 4, 2 or
    1 whole rows): row counts that fill a span, fall short of one, and leave a short last span -- with the
    quantization inside the launch and from activations quantized beforehand, which must agree bit for bit
    (the same integers, the same float order).  Q5_K runs on the same kernel, the fifth bits put over the
    nibbles on their way into the dot."""
    from bench import random_blocks
    from frink_amd import synth
    # (the row counts at which the launch changes its workgroups -- four, six or eight wavefronts, part of the span
    # behind the barrier -- need thousands of rows: random block bytes, encoding that many takes too long)
    data = random_blocks(kind, rows, cols, rows + cols) if rows > 2000 else make_weights(kind, rows, cols, seed=rows + cols)
    x = synth.activations(rows * 3 + cols, 1, cols, outlier_frac=0.01)[0]
    w = fa.Weights.from_host(kind, data, rows, cols)
    xd = to_dev(x)
    want = fo.gemv(kind, data, rows, cols, x)
    got = w.gemv(xd).cpu().numpy()
    assert_rows_close(got[None], want[None], "gemv over lines %dx%d" % (rows, cols))
    pre = w.gemv_q8k(fa.quantize_q8_k(xd)).cpu().numpy()
    # (rows of 64 blocks, and Q4_K rows of 32 blocks where the rows are few, take the kernel whose wavefronts split the
    # columns when the quantization is inside the launch: another order of the same terms)
    if cols > 8192 or (kind == fo.Q4_K and cols == 8192):
        assert_rows_close(pre[None], want[None], "gemv over lines from quantized activations %dx%d" % (rows, cols))
    else:
        assert np.array_equal(bits(pre), bits(got))
    w.release()


@pytest.mark.parametrize("kind,rows,cols,batches", [
    (fo.Q4_K, 200, 4096, (2, 8, 16, 17, 32)), (fo.Q4_K, 72, 512, (3, 9)), (fo.Q6_K, 136, 2048, (2, 8, 9, 24)),
    (fo.Q5_K, 100, 1024, (2, 16, 17, 32)), (fo.Q4_K, 50, 14336, (8,)),
])
def test_thin_gemm_from_activations_quantized_beforehand(fa, kind, rows, cols, batches):
    """frk_hip_gemm_q8k_dev (apply_batch_with_acts with BatchActs::Q8K, weight_matrix.rs:2481-2487, 757-768): a thin
    batch over Q8_K activations that frk_hip_quantize_q8_k_dev (or the producing kernel) wrote -- bit for bit
    frk_hip_gemm_dev's result (one row: frk_hip_gemv_q8k_dev's); a batch beyond the thin kernels' is refused with a
    message that names the entry to call."""
    from frink_amd import synth
    data = make_weights(kind, rows, cols, seed=rows + cols)
    w = fa.Weights.from_host(kind, data, rows, cols)
    x = synth.activations(rows + 7, max(batches), cols, outlier_frac=0.01)
    for batch in batches:
        xd = to_dev(x[:batch])
        want = w.gemm(xd).cpu().numpy()
        got = w.gemm_q8k(fa.quantize_q8_k(xd), batch).cpu().numpy()
        assert np.array_equal(bits(got), bits(want)), "batch %d" % batch
    acts = fa.quantize_q8_k(to_dev(x[0]))  # one row is frk_hip_gemv_q8k_dev
    assert np.array_equal(bits(w.gemm_q8k(acts, 1).cpu().numpy()[0]), bits(w.gemv_q8k(acts).cpu().numpy()))
    if kind == fo.Q4_K:
        xd = to_dev(synth.activations(3, 64, cols))
        with pytest.raises(fa.BackendError) as err:
            w.gemm_q8k(fa.quantize_q8_k(xd), 64)
        assert err.value.code == fa.ERR_UNSUPPORTED and "frk_hip_gemm_dev" in str(err.value)
    w.release()


@pytest.mark.parametrize("rows,cols", [(50, 14336), (300, 12288), (1000, 8448), (7, 16128), (64, 8192), (40, 2304),
                                       (1, 14336), (3, 11008), (131, 11008), (257, 13824), (5, 4352), (100, 5120), (129, 6144),
                                       (2, 7936), (63, 7680), (33, 16384), (10, 3072), (9, 2560)])
@pytest.mark.parametrize("kind", [fo.Q4_K, fo.Q5_K])
def test_gemv_at_rows_between_the_line_lengths(fa, kind, rows, cols):
    """Rows whose block count is not 8, 16 or 32.  From 17 blocks on (4352 columns) a wavefront takes the whole
    rows that fit its 64 lanes -- 3 rows of 20 blocks, one of 56 -- and adds a row's blocks with a segmented
    shuffle: in one launch up to 31 blocks (Q4_K: up to 20; longer rows take the kernel whose wavefronts split the
    columns), behind a quantization launch from 33 on (Q5_K, and Q4_K from quantized activations); shorter rows keep
    the per-lane kernel.  Row counts that fill spans, fall short of one and leave a short last span, for
    frk_hip_gemv_dev and frk_hip_gemv_q8k_dev (whose staging once stopped at 256 pairs of 16-wide sums: wrong
    results at 14336 columns)."""
    from frink_amd import synth
    data = make_weights(kind, rows, cols, seed=rows + cols)
    x = synth.activations(rows + cols, 1, cols, outlier_frac=0.01)[0]
    w = fa.Weights.from_host(kind, data, rows, cols)
    want = fo.gemv(kind, data, rows, cols, x)
    pre = w.gemv_q8k(fa.quantize_q8_k(to_dev(x))).cpu().numpy()
    got = w.gemv(to_dev(x)).cpu().numpy()
    if rows == 1:  # (a single output: nothing to take the norm over but itself)
        assert abs(pre[0] - want[0]) <= 1e-5 * np.abs(x).sum() * 1e-2 + 1e-6 and abs(got[0] - want[0]) <= 1e-5 * np.abs(x).sum() * 1e-2 + 1e-6
    else:
        assert_rows_close(pre[None], want[None], "gemv_q8k %dx%d" % (rows, cols))
        assert_rows_close(got[None], want[None], "gemv %dx%d" % (rows, cols))
    w.release()


@pytest.mark.parametrize("rows,cols", [(1, 5632), (8, 5632), (9, 16384), (3, 8192), (6200, 8192), (4101, 6144), (2050, 14336),
                                       (17, 11008), (24, 13824), (40, 16128), (100, 9472)])
@pytest.mark.parametrize("kind", [fo.Q4_K, fo.Q5_K])
def test_q4_k_gemv_with_the_columns_split_between_wavefronts(fa, kind, rows, cols):
    """Q4_K rows of more than 20 blocks (of 32 blocks: few or many rows) and Q5_K rows of more than 32, one launch (the
    other shapes in the list run on the kernels they had): a wavefront takes four blocks of
    columns of the workgroup's 8, 16 or 24 rows and quantizes exactly those blocks itself.  Row counts that fill a
    workgroup, fall short and leave a short last one, at every number of rows to a workgroup the launch picks (the
    large row counts: random block bytes); block counts that fill the last wavefront's four and do not."""
    from bench import random_blocks
    from frink_amd import synth
    data = random_blocks(kind, rows, cols, rows + cols) if rows > 2000 else make_weights(kind, rows, cols, seed=rows * 3 + cols)
    x = synth.activations(rows + 2 * cols, 1, cols, outlier_frac=0.01)[0]
    w = fa.Weights.from_host(kind, data, rows, cols)
    want = fo.gemv(kind, data, rows, cols, x, fo.INT_DOT)
    got = w.gemv(to_dev(x)).cpu().numpy()
    if rows == 1:
        assert abs(got[0] - want[0]) <= 1e-7 * np.abs(x).sum() + 1e-6
    else:
        assert_rows_close(got[None], want[None], "q4_k columns form %dx%d" % (rows, cols))
    w.release()


def test_gemv_outliers_and_zero_activation(fa):
    from frink_amd import synth
    data = make_weights(fo.Q4_K, 32, 4096, seed=3)
    w = fa.Weights.from_host(fo.Q4_K, data, 32, 4096)
    x = synth.activations(4, 1, 4096, outlier_frac=0.01)[0]
    assert_rows_close(w.gemv(to_dev(x)).cpu().numpy()[None], fo.gemv(fo.Q4_K, data, 32, 4096, x)[None], "outliers")
    z = np.zeros(4096, np.float32)
    assert not w.gemv(to_dev(z)).cpu().numpy().any()


@pytest.mark.parametrize("kind", [fo.Q4_K, fo.Q5_K, fo.Q6_K, fo.Q8_0])
def test_host_buffer_launch_matvec_is_the_drop_in(fa, kind):
    from frink_amd import synth
    rows, cols = 24, 1024
    bb, be = fo.BLOCK[kind]
    data = make_weights(kind, rows, cols, seed=9)
    x = synth.activations(10, 1, cols)[0]
    got = fa.launch_matvec(kind, data, x, rows, cols // be * bb)
    want = fo.gemv(kind, data, rows, cols, x, fo.F32_DOT if kind == fo.Q8_0 else fo.INT_DOT)
    assert_rows_close(got[None], want[None], "launch_matvec")
    # the resident copy is keyed by (pointer, length) and checked against sampled bytes: overwrite the
    # buffer in place and the next call must see the new weights
    data2 = make_weights(kind, rows, cols, seed=99)
    data[:] = data2
    got2 = fa.launch_matvec(kind, data, x, rows, cols // be * bb)
    want2 = fo.gemv(kind, data2, rows, cols, x, fo.F32_DOT if kind == fo.Q8_0 else fo.INT_DOT)
    assert_rows_close(got2[None], want2[None], "launch_matvec after the host bytes changed")


def test_q5_k_decode_and_batches_at_full_size(fa):
    """Q5_K (Q4_K's scale packing, a fifth bit per code from a separate plane): the FFN shape with
    arbitrary block bytes (every bit pattern of the fifth-bit plane) against the oracle on slices of
    rows, for one row (the decode kernel), 3, 16, 17 and 32 rows (the thin matrix-core kernel: 16 rows
    a workgroup, wider batches as a grid of 16-row groups in one launch), 33, 70 and 512 rows (the tiled
    matrix-core kernel with the fifth bits as a third int8 plane, its blocks split between workgroups for
    the small batches), and the whole output of a row against dequantized weights in float64."""
    from frink_amd import synth
    rows, cols = 14336, 4096
    data = _random_q5_k(rows, cols, 41)
    w = fa.Weights.from_host(fo.Q5_K, data, rows, cols)
    x = synth.activations(42, 512, cols, outlier_frac=0.01)
    for batch in (1, 3, 16, 17, 32, 33, 70, 512):
        print("q5_k batch", batch, flush=True)
        got = w.gemm(to_dev(x[:batch])).cpu().numpy()
        assert got.shape == (batch, rows)
        for row0 in (0, 7000, rows - 64):
            want = fo.gemm(fo.Q5_K, data, rows, cols, x[:batch], row0=row0, nrows=64)
            assert_rows_close(got[:, row0:row0 + 64], want, "q5_k batch %d rows %d.." % (batch, row0))
    one = w.gemv(to_dev(x[0])).cpu().numpy()
    wd = w.dequant().cpu().numpy().astype(np.float64)
    q, d, _ = fo.quantize_q8_k(x[0])
    xa = q.astype(np.float64) * np.repeat(d.astype(np.float64), 256)
    ref = wd @ xa
    assert np.abs(one - ref).max() <= 1e-3 * np.abs(ref).max()
    w.release()


@pytest.mark.parametrize("rows,cols,batch", [(72, 512, 2), (33, 768, 5), (100, 256, 16), (50, 2048, 9), (20, 14336, 4),
                                             (72, 512, 33), (40, 1024, 130), (200, 768, 130), (257, 1024, 200),
                                             (13000, 512, 300), (129, 256, 65)])
def test_q5_k_thin_batches_on_ragged_shapes(fa, rows, cols, batch):
    from frink_amd import synth
    data = make_weights(fo.Q5_K, rows, cols, seed=rows + cols)
    w = fa.Weights.from_host(fo.Q5_K, data, rows, cols)
    x = synth.activations(rows, batch, cols, outlier_frac=0.01)
    got = w.gemm(to_dev(x)).cpu().numpy()
    assert_rows_close(got, fo.gemm(fo.Q5_K, data, rows, cols, x), "q5_k thin %dx%d batch %d" % (rows, cols, batch))
    w.release()


def _random_q4_0(rows, cols, seed):
    rng = np.random.default_rng(seed)
    nb = rows * cols // 32
    data = rng.integers(0, 256, nb * 18, dtype=np.uint8).reshape(nb, 18)
    data[:, 0:2] = rng.uniform(-2e-3, 2e-3, nb).astype(np.float16).view(np.uint8).reshape(-1, 2)
    return data.ravel()


@pytest.mark.parametrize("rows,cols", [(64, 4096), (37, 4096), (7, 32), (9, 544), (5, 2048), (4096, 4096), (1, 2080), (13, 14336),
                                       (8200, 2048), (3, 32768), (10, 6176), (5, 34816)])
def test_q4_0_dequant_and_decode(fa, rows, cols):
    """Q4_0 (18-byte blocks: an f16 scale and 16 bytes of nibbles, value (nibble - 8) * d) is kept as a
    plane of nibbles and a plane of scales.  The reference holds no encoder for it, so the blocks are
    arbitrary bytes with finite scales: dequantization bit-exact, the f32 dot (decode on an x86 host)
    and the integer dot against Q8_0 activation blocks within the tolerance."""
    from frink_amd import synth
    print("q4_0", rows, cols, flush=True)
    data = _random_q4_0(rows, cols, rows + cols)
    w = fa.Weights.from_host(fo.Q4_0, data, rows, cols)
    assert np.array_equal(bits(w.dequant().cpu().numpy()), bits(fo.dequant(fo.Q4_0, data).reshape(rows, cols)))
    x = synth.activations(rows * 3 + cols, 3, cols, outlier_frac=0.01)
    n = min(rows, 64)
    for row0 in sorted({0, rows - n}):
        got = w.gemv(to_dev(x[0]), act_mode=fa.ACT_F32).cpu().numpy()
        want = fo.gemm(fo.Q4_0, data, rows, cols, x[:1], fo.F32_DOT, row0=row0, nrows=n)
        assert_rows_close(got[None, row0:row0 + n], want, "q4_0 f32 dot")
        got_i = w.gemv(to_dev(x[0]), act_mode=fa.ACT_INT8).cpu().numpy()
        want_i = fo.gemm(fo.Q4_0, data, rows, cols, x[:1], fo.INT_DOT, row0=row0, nrows=n)
        assert_rows_close(got_i[None, row0:row0 + n], want_i, "q4_0 integer dot")
    bb = fo.BLOCK[fo.Q4_0][0]
    host = fa.launch_matvec(fo.Q4_0, data, x[0], rows, cols // 32 * bb)
    assert np.array_equal(bits(host), bits(w.gemv(to_dev(x[0])).cpu().numpy()))
    w.release()


@pytest.mark.parametrize("rows,cols,batch", [(72, 512, 5), (100, 96, 33), (33, 288, 70), (64, 4096, 129),
                                             (1000, 1056, 300), (4096, 4096, 512)])
def test_gemm_q4_0_on_the_matrix_cores(fa, rows, cols, batch):
    """A Q4_0 batch is the Q8_0 GEMM kernel with the nibbles turned into signed bytes on their way to
    LDS (dot_q4_0_q8: Q8_0 activation blocks, exact integer sums): the three workgroup shapes, ragged
    tiles and rows that are not whole 256-column steps, arbitrary block bytes, against the oracle."""
    from frink_amd import synth
    print("gemm q4_0", rows, cols, batch, flush=True)
    data = _random_q4_0(rows, cols, rows + batch)
    x = synth.activations(rows * 11 + batch, batch, cols, outlier_frac=0.01)
    w = fa.Weights.from_host(fo.Q4_0, data, rows, cols)
    got = w.gemm(to_dev(x)).cpu().numpy()
    assert got.shape == (batch, rows)
    n = min(64, rows)
    for row0 in sorted({0, (rows // 2) // 32 * 32 + 5 if rows > 128 else 0, rows - n}):
        want = fo.gemm(fo.Q4_0, data, rows, cols, x, fo.INT_DOT, row0=row0, nrows=n)
        assert_rows_close(got[:, row0:row0 + n], want, "gemm q4_0 %dx%d batch %d rows %d.." % (rows, cols, batch, row0))
    half = w.gemm(to_dev(x * np.float32(0.5))).cpu().numpy()
    assert np.array_equal(bits(half), bits(got * np.float32(0.5)))
    w.release()


def _random_q5_k(rows, cols, seed):
    rng = np.random.default_rng(seed)
    nb = rows * cols // 256
    data = rng.integers(0, 256, nb * 176, dtype=np.uint8).reshape(nb, 176)
    data[:, 0:2] = rng.uniform(1e-4, 1e-3, nb).astype(np.float16).view(np.uint8).reshape(-1, 2)
    data[:, 2:4] = rng.uniform(1e-4, 1e-3, nb).astype(np.float16).view(np.uint8).reshape(-1, 2)
    return data.ravel()


def test_gemm_entry_point_is_batch_major(fa):
    from frink_amd import synth
    rows, cols, batch = 40, 1024, 3
    data = make_weights(fo.Q4_K, rows, cols, seed=17)
    x = synth.activations(18, batch, cols)
    got = fa.launch_mul_mm(fo.Q4_K, data, x, rows, cols, batch, cols // 256 * 144)
    want = fo.gemm(fo.Q4_K, data, rows, cols, x)
    assert got.shape == (batch, rows)
    assert_rows_close(got, want, "launch_mul_mm")


# ------------------------------------------------------------------ full-size configurations

FULL = [
    ("Q8_0 4096x4096", fo.Q8_0, 4096, 4096, 31),
    ("Q4_K 14336x4096 (gate/up)", fo.Q4_K, 14336, 4096, 32),
    ("Q6_K 4096x14336 (down)", fo.Q6_K, 4096, 14336, 33),
]


@pytest.mark.parametrize("name,kind,rows,cols,seed", FULL)
def test_full_size_gemv(fa, name, kind, rows, cols, seed):
    """The configured shapes: the whole output against the oracle (a few seconds of CPU), plus
    two size-independent properties: linearity in the output rows (a permutation of W's rows
    permutes y) is implied by per-row ownership, so check homogeneity instead -- scaling x by a
    power of two scales Q8_K's d exactly and leaves q unchanged, so y scales exactly."""
    from frink_amd import synth
    print("full", name, flush=True)
    data = make_weights(kind, rows, cols, seed)
    x = synth.activations(seed + 100, 1, cols)[0]
    w = fa.Weights.from_host(kind, data, rows, cols)
    mode = fo.F32_DOT if kind == fo.Q8_0 else fo.INT_DOT
    want = fo.gemv(kind, data, rows, cols, x, mode)
    y = w.gemv(to_dev(x)).cpu().numpy()
    assert_rows_close(y[None], want[None], name)
    y4 = w.gemv(to_dev(x * np.float32(4.0))).cpu().numpy()
    assert np.array_equal(bits(y4), bits(y * np.float32(4.0)))
    # and the dequantized matrix, every value
    got = w.dequant().cpu().numpy()
    assert np.array_equal(bits(got), bits(fo.dequant(kind, data).reshape(rows, cols)))
    w.release()


# ------------------------------------------------------------------ batched GEMM (int8 MFMA)

@pytest.mark.parametrize("rows,cols,batch", [(256, 1024, 128), (96, 512, 40), (64, 256, 16), (200, 768, 130),
                                             (128, 2048, 512)])
def test_gemm_mfma_matches_the_oracle(fa, rows, cols, batch):
    from frink_amd import synth
    print("gemm", rows, cols, batch, flush=True)
    data = make_weights(fo.Q4_K, rows, cols, seed=rows + cols + batch)
    x = synth.activations(rows * 3 + batch, batch, cols, outlier_frac=0.01)
    w = fa.Weights.from_host(fo.Q4_K, data, rows, cols)
    got = w.gemm(to_dev(x)).cpu().numpy()
    want = fo.gemm(fo.Q4_K, data, rows, cols, x)
    assert got.shape == (batch, rows)
    assert_rows_close(got, want, "gemm %dx%d batch %d" % (rows, cols, batch))
    w.release()


@pytest.mark.parametrize("rows,cols,batch", [(13000, 512, 500), (14336, 512, 320), (13001, 768, 1000)])
def test_gemm_large_tiles_with_ragged_edges(fa, rows, cols, batch):
    """Shapes that take the 256-row workgroup tiles (x128 tokens: 13000x500 and 13001x1000; x64:
    14336x320) with a last row tile and a last token tile that are partly empty: the first, a middle
    and the last 256 weight rows against the oracle, and zeros nowhere they do not belong."""
    from frink_amd import synth
    print("gemm large tiles", rows, cols, batch, flush=True)
    data = make_weights(fo.Q4_K, rows, cols, seed=rows + batch)
    x = synth.activations(rows + batch, batch, cols, outlier_frac=0.01)
    w = fa.Weights.from_host(fo.Q4_K, data, rows, cols)
    y = w.gemm(to_dev(x)).cpu().numpy()
    assert y.shape == (batch, rows)
    for row0 in (0, (rows // 2) // 32 * 32 + 7, rows - 256):
        want = fo.gemm(fo.Q4_K, data, rows, cols, x, row0=row0, nrows=256)
        assert_rows_close(y[:, row0:row0 + 256], want, "gemm %dx%d batch %d rows %d.." % (rows, cols, batch, row0))
    w.release()


@pytest.mark.parametrize("kind,rows,cols", [(fo.Q4_K, 70, 4096), (fo.Q5_K, 660, 4096), (fo.Q5_K, 40, 14336), (fo.Q6_K, 50, 2048),
                                            (fo.Q8_0, 64, 1024), (fo.Q4_0, 64, 1024)])
def test_a_batch_of_one_row_is_the_decode_path(fa, kind, rows, cols):
    """frk_hip_gemm_dev with one activation row returns the bits of frk_hip_gemv_dev (a Q5_K row of 16 blocks once took
    the generic kernel behind a quantization launch there); the batch-activations form returns frk_hip_gemv_q8k_dev's."""
    from frink_amd import synth
    data = _random_q4_0(rows, cols, rows) if kind == fo.Q4_0 else make_weights(kind, rows, cols, seed=rows)
    x = synth.activations(rows + 1, 1, cols, outlier_frac=0.01)
    w = fa.Weights.from_host(kind, data, rows, cols)
    one = w.gemv(to_dev(x[0])).cpu().numpy()
    assert np.array_equal(bits(w.gemm(to_dev(x)).cpu().numpy()[0]), bits(one))
    if kind in (fo.Q4_K, fo.Q5_K, fo.Q6_K):
        # (from quantized activations a long row takes another kernel than the one-launch form: the same integers,
        # added in another order)
        acts = fa.BatchActs(4, cols).quantize(to_dev(x))
        got = w.gemm_acts(acts).cpu().numpy()[0]
        assert np.abs(got - one).max() <= 1e-5 * np.abs(one).max()
        assert np.array_equal(bits(got), bits(w.gemv_q8k(fa.quantize_q8_k(to_dev(x[0]))).cpu().numpy()))
        acts.release()
    w.release()


def _oracle_gemm_all_rows(data, rows, cols, x):
    """The oracle's integer-dot GEMM over EVERY weight row.  Its AVX2 form is held bit-equal to the scalar
    functions by tests/test_oracle_goldens.py and does 14336 x 4096 x 512 in a fraction of a second; a host
    without AVX2 falls back to the scalar functions, threaded."""
    if fo.have_avx2():
        import os
        return fo.avx2_gemm_q4_k_q8k(data, rows, cols, x, threads=min(16, os.cpu_count() or 1))
    return fo.gemm(fo.Q4_K, data, rows, cols, x)


@pytest.mark.parametrize("rows,cols", [(4096, 4096), (14336, 4096)])
def test_full_size_prefill_gemm(fa, rows, cols):
    """M=512 with 1% outliers at +-20: every output of the batch, all weight rows, against the oracle,
    plus exact homogeneity."""
    from frink_amd import synth
    print("full gemm", rows, cols, flush=True)
    batch = 512
    data = make_weights(fo.Q4_K, rows, cols, seed=rows)
    x = synth.activations(77, batch, cols, outlier_frac=0.01)
    w = fa.Weights.from_host(fo.Q4_K, data, rows, cols)
    y = w.gemm(to_dev(x)).cpu().numpy()
    want = _oracle_gemm_all_rows(data, rows, cols, x)
    # (the scalar functions themselves on one slice, whatever the host)
    assert np.array_equal(bits(want[:, 512:544]), bits(fo.gemm(fo.Q4_K, data, rows, cols, x, row0=512, nrows=32)))
    ninf = np.abs(want).max(axis=1)
    err = np.abs(y - want).max(axis=1)
    record("Q4_K gemm M=512 %dx%d, all rows" % (rows, cols), float((err / ninf).max()))
    assert (err <= TOL * ninf).all(), float((err / ninf).max())
    y2 = w.gemm(to_dev(x * np.float32(0.5))).cpu().numpy()
    assert np.array_equal(bits(y2), bits(y * np.float32(0.5)))
    w.release()


# ------------------------------------------------------------------ MoE: routing, grouped expert GEMM

def _route(logits, k, norm=True):
    routed = [fo.route_top_k_softmax(l, k, norm) for l in logits]
    return np.stack([r[0] for r in routed]), np.stack([r[1] for r in routed])


def test_route_top_k_softmax_matches_the_oracle(fa):
    from frink_amd import synth
    logits = synth.normal(901, 512 * 128).reshape(512, 128)
    for norm in (True, False):
        ids, w = fa.route_top_k_softmax(to_dev(logits), 8, norm)
        want_ids, want_w = _route(logits, 8, norm)
        assert np.array_equal(ids.cpu().numpy(), want_ids)
        # bit for bit: the device evaluates expf the way the host's libm does, and adds in the oracle's order
        assert np.array_equal(bits(w.cpu().numpy()), bits(want_w))
    # logits far below the row's maximum: expf down to its subnormal results, glibc's underflow value and zero
    far = np.random.default_rng(5).uniform(-110, -80, (64, 16)).astype(np.float32)
    far[:, 0] = 0.0
    far[0, 1:6] = [-103.2, -103.3, -103.9, -104.0, -87.4]
    ids, w = fa.route_top_k_softmax(to_dev(far), 4, False)
    want_ids, want_w = _route(far, 4, False)
    assert np.array_equal(bits(w.cpu().numpy()), bits(want_w))
    assert np.array_equal(ids.cpu().numpy()[want_w > 0], want_ids[want_w > 0])  # (zeros tie: any order)
    # the reference's own known answers (crates/frink-moe/src/lib.rs:1345-1404)
    ids, w = fa.route_top_k_softmax(to_dev(np.arange(1, 9, dtype=np.float32)[None]), 3, False)
    assert ids.cpu().numpy().tolist() == [[7, 6, 5]]
    np.testing.assert_allclose(w.cpu().numpy()[0], [0.6323223, 0.2326232, 0.0855683], atol=1e-4)
    ids, _ = fa.route_top_k_softmax(to_dev(np.array([[0.1, 5.0, 0.2, 3.0, -1.0]], np.float32)), 2, True)
    assert ids.cpu().numpy().tolist() == [[1, 3]]


def _stacked_experts(n_experts, hidden, ffn, seed, random_blocks=False, sigma=0.05):
    """gate/up [E*ffn][hidden] and down [E*hidden][ffn] as Q4_K bytes."""
    shapes = ((n_experts * ffn, hidden), (n_experts * ffn, hidden), (n_experts * hidden, ffn))
    out = []
    for i, (rows, cols) in enumerate(shapes):
        if random_blocks:
            # any bytes are a valid block; keep the two f16 super-scales small and finite
            rng = np.random.default_rng(seed + i)
            nblk = rows * cols // 256
            data = rng.integers(0, 256, (nblk, 144), dtype=np.uint8)
            data[:, 0:2] = rng.uniform(0.0005, 0.002, nblk).astype(np.float16).view(np.uint8).reshape(-1, 2)
            data[:, 2:4] = rng.uniform(0.0005, 0.004, nblk).astype(np.float16).view(np.uint8).reshape(-1, 2)
            out.append(data.ravel())
        else:
            out.append(make_weights(fo.Q4_K, rows, cols, seed=seed + i, sigma=sigma))
    return out


def _grouped_case(kind, n_groups, rows_g, cols, counts, x_rows, seed, with_gather):
    """Weights of n_groups stacked matrices, x, the offsets of groups of the given sizes and a gather list (or none:
    pair p reads row p, so x has exactly one row per pair)."""
    from frink_amd import synth
    off = np.zeros(n_groups + 1, np.int32)
    off[1:] = np.cumsum(counts)
    pairs = int(off[-1])
    if not with_gather:
        x_rows = pairs
    data = make_weights(kind, n_groups * rows_g, cols, seed=seed)
    x = synth.activations(seed + 1, max(x_rows, 1), cols, outlier_frac=0.01)[:x_rows]
    gather = np.random.default_rng(seed + 2).integers(0, max(x_rows, 1), pairs).astype(np.int32) if with_gather else None
    return data, x, off, gather, pairs


def _grouped_oracle(kind, data, n_groups, rows_g, cols, x, off, gather):
    """enqueue_mul_mm_grouped_dev's contract (crates/frink-cuda/src/mul_mm_launch.rs:391-470) from the oracle's
    GEMM, one group at a time."""
    per = data.reshape(n_groups, -1)
    want = np.zeros((int(off[-1]), rows_g), np.float32)
    for g in range(n_groups):
        p0, p1 = int(off[g]), int(off[g + 1])
        if p1 > p0:
            src = gather[p0:p1] if gather is not None else np.arange(p0, p1)
            want[p0:p1] = fo.gemm(kind, per[g], rows_g, cols, x[src])
    return want


@pytest.mark.parametrize("kind", [fo.Q4_K, fo.Q6_K])
@pytest.mark.parametrize("with_gather", [True, False])
def test_grouped_gemm_on_its_own(fa, kind, with_gather):
    """Groups of 0, 1, 31..33, 64, 65 and 150 pairs (tiles of every fill, a group of several tiles, empty groups at
    both ends), rows that are not a multiple of the kernels' 256-row groups, a gather list that repeats rows."""
    counts = [0, 1, 31, 0, 32, 33, 64, 65, 150, 7, 0]
    n_groups, rows_g, cols = len(counts), 200, 768
    print("grouped gemm", kind, with_gather, flush=True)
    data, x, off, gather, pairs = _grouped_case(kind, n_groups, rows_g, cols, counts, 90, 77 + kind, with_gather)
    w = fa.Weights.from_host(kind, data, n_groups * rows_g, cols)
    import torch
    y = torch.full((pairs, rows_g), float("nan"), dtype=torch.float32, device="cuda")
    got = fa.gemm_grouped(w, n_groups, to_dev(off), to_dev(x), to_dev(gather) if with_gather else None, out=y).cpu().numpy()
    want = _grouped_oracle(kind, data, n_groups, rows_g, cols, x, off, gather)
    assert not np.isnan(got).any()  # every pair's row written
    assert_rows_close(got, want, "grouped gemm kind %d gather %s" % (kind, with_gather))
    # a second, smaller call on the same stream's scratch
    counts2 = [5, 0, 40]
    data2, x2, off2, gather2, pairs2 = _grouped_case(kind, 3, rows_g, cols, counts2, 20, 99, with_gather)
    w2 = fa.Weights.from_host(kind, data2, 3 * rows_g, cols)
    got2 = fa.gemm_grouped(w2, 3, to_dev(off2), to_dev(x2), to_dev(gather2) if with_gather else None).cpu().numpy()
    assert_rows_close(got2, _grouped_oracle(kind, data2, 3, rows_g, cols, x2, off2, gather2), "grouped gemm, second call")
    w.release()
    w2.release()


def test_grouped_gemm_at_the_expert_shape(fa):
    """128 groups of 768 x 2048 (the routed layer's gate experts), 4096 pairs of 512 rows: every output against the
    oracle."""
    from frink_amd import synth
    n_groups, rows_g, cols, x_rows, k = 128, 768, 2048, 512, 8
    print("grouped gemm 128 x 768 x 2048", flush=True)
    data = make_weights(fo.Q4_K, n_groups * rows_g, cols, seed=5)
    x = synth.activations(6, x_rows, cols, outlier_frac=0.01)
    rng = np.random.default_rng(7)
    ids = np.stack([rng.permutation(n_groups)[:k] for _ in range(x_rows)]).astype(np.int32)
    order = np.argsort(ids.ravel(), kind="stable")  # pairs by group, tokens ascending inside a group
    gather = (order // k).astype(np.int32)
    off = np.zeros(n_groups + 1, np.int32)
    off[1:] = np.cumsum(np.bincount(ids.ravel(), minlength=n_groups))
    w = fa.Weights.from_host(fo.Q4_K, data, n_groups * rows_g, cols)
    got = fa.gemm_grouped(w, n_groups, to_dev(off), to_dev(x), to_dev(gather)).cpu().numpy()
    want = _grouped_oracle(fo.Q4_K, data, n_groups, rows_g, cols, x, off, gather)
    assert_rows_close(got, want, "grouped gemm at the expert shape")
    w.release()


def test_grouped_gemm_over_more_rows_than_the_gathering_kernel_addresses(fa):
    """70000 activation rows (the gathering kernel's table holds 16-bit rows): the rows in use are gathered into the
    grouped order and quantized there."""
    counts = [3, 70, 0, 33]
    n_groups, rows_g, cols = len(counts), 64, 256
    print("grouped gemm, 70000 activation rows", flush=True)
    data, x, off, gather, pairs = _grouped_case(fo.Q4_K, n_groups, rows_g, cols, counts, 70000, 123, True)
    gather[:4] = [69999, 0, 65536, 65535]
    w = fa.Weights.from_host(fo.Q4_K, data, n_groups * rows_g, cols)
    got = fa.gemm_grouped(w, n_groups, to_dev(off), to_dev(x), to_dev(gather)).cpu().numpy()
    assert_rows_close(got, _grouped_oracle(fo.Q4_K, data, n_groups, rows_g, cols, x, off, gather), "grouped gemm, 70000 rows")
    w.release()


@pytest.mark.parametrize("kind,cols", [(fo.Q5_0, 96), (fo.MXFP4, 2880), (fo.IQ4_XS, 768), (fo.MXFP4, 256)])
@pytest.mark.parametrize("with_gather", [True, False])
def test_grouped_gemm_over_the_other_kinds(fa, kind, cols, with_gather):
    """The grouped entry over stacks of Q5_0 / MXFP4 / IQ4_XS matrices: the stack decoded to signed bytes per call, the
    activation rows quantized once (Q8_0 blocks; Q8_K for IQ4_XS), the grouped matrix-core kernel gathering through the
    list -- every pair against the integer tier of its kind (q8_row_dot / q8k_row_dot,
    crates/frink-core/src/weight_matrix.rs:392-420)."""
    from frink_amd import synth
    counts = [0, 1, 31, 0, 32, 33, 64, 65, 150, 7, 0]
    n_groups, rows_g = len(counts), 72
    print("grouped gemm, other kinds", kind, cols, with_gather, flush=True)
    off = np.zeros(n_groups + 1, np.int32)
    off[1:] = np.cumsum(counts)
    pairs = int(off[-1])
    x_rows = 90 if with_gather else pairs
    data = _other_kind_blocks(kind, n_groups * rows_g, cols, seed=kind + cols)
    if kind == fo.MXFP4:
        data.reshape(-1, 17)[:, 0] = 104 + data.reshape(-1, 17)[:, 0] % 40  # scales that are f16 values
    x = synth.activations(5, x_rows, cols, outlier_frac=0.01)
    gather = np.random.default_rng(6).integers(0, x_rows, pairs).astype(np.int32) if with_gather else None
    w = fa.Weights.from_host(kind, data, n_groups * rows_g, cols)
    import torch
    y = torch.full((pairs, rows_g), float("nan"), dtype=torch.float32, device="cuda")
    got = fa.gemm_grouped(w, n_groups, to_dev(off), to_dev(x), to_dev(gather) if with_gather else None, out=y).cpu().numpy()
    per = data.reshape(n_groups, -1)
    want = np.zeros((pairs, rows_g), np.float32)
    for g in range(n_groups):
        p0, p1 = int(off[g]), int(off[g + 1])
        if p1 > p0:
            src = gather[p0:p1] if with_gather else np.arange(p0, p1)
            want[p0:p1] = fo.gemm(kind, per[g], rows_g, cols, x[src], fo.INT_DOT)
    assert not np.isnan(got).any()  # every pair's row written
    assert_rows_close(got, want, "grouped gemm kind %d gather %s" % (kind, with_gather))
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max()
    w.release()


@pytest.mark.parametrize("kind", [fo.Q5_0, fo.IQ4_XS, fo.MXFP4])
def test_a_kept_decoded_copy_changes_no_bit(fa, kind):
    """frk_hip_weights_keep_decoded: the batched GEMM, the grouped GEMM and the MoE layer read the kept rows instead of
    decoding per call -- the same kernels over the same bytes, so every output bit is the same; kinds without a decoded
    form are refused."""
    from frink_amd import synth
    import torch
    E, k, hidden, ffn, batch = 4, 2, 512, 256, 70
    stacks = [_other_kind_blocks(kind, r, c, seed=60 + j) for j, (r, c) in enumerate(((E * ffn, hidden), (E * ffn, hidden), (E * hidden, ffn)))]
    for data in stacks:
        if kind == fo.MXFP4:
            data.reshape(-1, 17)[:, 0] = 110 + data.reshape(-1, 17)[:, 0] % 12
    x = synth.activations(63, batch, hidden)
    ids, wts = _route(synth.normal(64, batch * E).reshape(batch, E), k)
    off = to_dev(np.array([0, 10, 10, 50, 70], np.int32))

    def run(keep):
        ws = [fa.Weights.from_host(kind, d, r, c) for d, (r, c) in zip(stacks, ((E * ffn, hidden), (E * ffn, hidden), (E * hidden, ffn)))]
        if keep:
            for w in ws:
                w.keep_decoded()
                w.keep_decoded()  # (a second request: nothing to do)
        out = [ws[0].gemm(to_dev(x)).cpu().numpy(), fa.gemm_grouped(ws[0], E, off, to_dev(x)).cpu().numpy(),
               fa.moe_ffn(ws[0], ws[1], ws[2], E, to_dev(x), to_dev(ids.astype(np.int32)), to_dev(wts)).cpu().numpy()]
        for w in ws:
            w.release()
        return out
    for a, b in zip(run(False), run(True)):
        assert not np.isnan(a).any() and np.array_equal(bits(a), bits(b))
    w4 = fa.Weights.from_host(fo.Q4_K, make_weights(fo.Q4_K, 32, 256, seed=1), 32, 256)
    with pytest.raises(fa.BackendError):
        w4.keep_decoded()
    w4.release()
    if kind == fo.MXFP4:  # scales that are not f16 values: no decoded form
        stacks[0].reshape(-1, 17)[::5, 0] = 160
        wx = fa.Weights.from_host(kind, stacks[0], E * ffn, hidden)
        with pytest.raises(fa.BackendError):
            wx.keep_decoded()
        wx.release()


def test_grouped_gemm_refuses_what_it_cannot_run(fa):
    data = make_weights(fo.Q8_0, 64, 256, seed=1)
    w = fa.Weights.from_host(fo.Q8_0, data, 64, 256)
    off = to_dev(np.array([0, 1, 2], np.int32))
    x = to_dev(np.zeros((2, 256), np.float32))
    with pytest.raises(fa.BackendError):
        fa.gemm_grouped(w, 2, off, x)
    w.release()
    data = make_weights(fo.Q4_K, 96, 256, seed=1)
    w = fa.Weights.from_host(fo.Q4_K, data, 96, 256)
    with pytest.raises(fa.BackendError):  # 96 rows do not divide into 5 groups
        fa.gemm_grouped(w, 5, to_dev(np.zeros(6, np.int32)), x)
    # no pairs: nothing to do, no error
    y = fa.gemm_grouped(w, 2, to_dev(np.zeros(3, np.int32)), x, gather=to_dev(np.zeros(0, np.int32)))
    assert y.shape == (0, 48)
    w.release()


def _slot_order(ids_row, batch):
    """The order in which the reference adds a token's routed slots: ascending expert id on its bucket
    path (32 tokens and more, ffn_batch.rs:355, 388-423), routing order below that
    (combine_expert_outputs, crates/frink-moe/src/lib.rs:1246-1263)."""
    k = len(ids_row)
    if batch >= fo.MOE_BUCKET_FROM:
        return sorted(range(k), key=lambda s: (int(ids_row[s]), s))
    return list(range(k))


def _moe_oracle(down_kind, gate, up, down, n_experts, hidden, ffn, x, ids, w):
    """The layer as the reference runs a batch of this size (fo.moe_ffn); with the down experts in
    another kind than gate and up (a Q4_K_M checkpoint keeps some layers' down experts in Q6_K) from the
    oracle's own GEMMs and SwiGLU per expert, added per token in the same order."""
    if down_kind == fo.Q4_K:
        return fo.moe_ffn(fo.Q4_K, gate, up, down, n_experts, hidden, ffn, x, ids, w)
    gb, ub, db = (m.reshape(n_experts, -1) for m in (gate, up, down))
    batch, k = ids.shape
    pair_out = np.zeros((batch, k, hidden), np.float32)
    for e in range(n_experts):
        toks, slots = np.nonzero(ids == e)
        if toks.size == 0:
            continue
        g = fo.gemm(fo.Q4_K, gb[e], ffn, hidden, x[toks])
        u = fo.gemm(fo.Q4_K, ub[e], ffn, hidden, x[toks])
        act = fo.swiglu(g.ravel(), u.ravel()).reshape(toks.size, ffn)
        pair_out[toks, slots] = fo.gemm(down_kind, db[e], hidden, ffn, act)
    out = np.zeros((batch, hidden), np.float32)
    for t in range(batch):
        for sl in _slot_order(ids[t], batch):
            if 0 <= ids[t, sl] < n_experts:
                out[t] += w[t, sl] * pair_out[t, sl]
    return out


def _end_to_end_gate(got, want, what, strict):
    """The Q8_K quantizer between the two GEMMs is a step function: a last-bit difference in a gate
    output (any implementation that adds in another order than the oracle has them) can move an
    intermediate to the next int8 level, which shifts that output row by d_act*|w|, and the fewer
    columns the down projection has the larger that is against ||y||inf.  So the stage-by-stage gates
    are the strict ones, and end to end a full-size layer (strict) must hold the tolerance on at least
    99 % of its rows and one and a half times the tolerance on every row (measured on the 128-expert layer of
    2048/768: at most one row of 512 above 1e-3, the rest below 5e-7 apart from such flips;
    _report_flipped_levels prints the intermediate behind the worst row), the small test shapes on 90 % of the
    rows and ten times the tolerance on every row."""
    rel = np.abs(got - want).max(axis=1) / np.abs(want).max(axis=1)
    print("%s end-to-end: rows over 1e-3: %d of %d, worst %.3g" % (what, (rel > TOL).sum(), rel.size, rel.max()), flush=True)
    record(what, rel.max())
    record(what + ": rows over 1e-3", float((rel > TOL).sum()))
    if strict:
        assert (rel <= TOL).mean() >= 0.99 and rel.max() <= 1.5 * TOL, "%s: worst row %.3g of ||y||inf" % (what, rel.max())
    else:
        assert (rel <= TOL).mean() >= 0.9 and rel.max() <= 10 * TOL, "%s: worst row %.3g" % (what, rel.max())


def _moe_case(fa, n_experts, k, hidden, ffn, batch, seed, random_blocks=False, ids_override=None, down_kind=None,
              sigma=0.05, strict=False):
    """The quantizer between the two GEMMs is a step function, so a last-bit difference in a
    gate/up output can move one intermediate value to the next int8 level and shift a whole output
    row by d_act*|w|: the end-to-end comparison alone cannot hold 1e-3 on every row for any
    implementation that sums in another order than the oracle.  The layer is therefore gated as a
    chain in which each link starts from the device's own previous result:
      1. gate/up grouped GEMM outputs (row of every (token, slot) pair) vs the oracle's GEMM  [tolerance]
      2. silu(gate)*up (the oracle's, whose expf is the host's: the device evaluates glibc's algorithm) and its
         Q8_K quantization, from the device's gate/up                                          [bit-exact]
      3. down GEMM + weighted combine, from that same intermediate                            [tolerance]
    and end to end against the oracle's layer (_end_to_end_gate)."""
    from frink_amd import synth
    print("moe", n_experts, k, hidden, ffn, batch, flush=True)
    gate, up, down = _stacked_experts(n_experts, hidden, ffn, seed, random_blocks, sigma)
    down_kind = fo.Q4_K if down_kind is None else down_kind
    what = "moe E=%d k=%d %d/%d batch=%d down=%d" % (n_experts, k, hidden, ffn, batch, down_kind)
    if down_kind != fo.Q4_K:
        down = make_weights(down_kind, n_experts * hidden, ffn, seed=seed + 2, sigma=0.05)
    x = synth.activations(seed + 10, batch, hidden)
    logits = synth.normal(seed + 11, batch * n_experts).reshape(batch, n_experts)
    ids, w = _route(logits, k)
    if ids_override is not None:
        ids = ids_override(ids)
    ids = ids.astype(np.int32)
    wg = fa.Weights.from_host(fo.Q4_K, gate, n_experts * ffn, hidden)
    wu = fa.Weights.from_host(fo.Q4_K, up, n_experts * ffn, hidden)
    wd = fa.Weights.from_host(down_kind, down, n_experts * hidden, ffn)
    got = fa.moe_ffn(wg, wu, wd, n_experts, to_dev(x), to_dev(ids), to_dev(w)).cpu().numpy()
    if batch <= fa.MOE_PER_TOKEN_MAX_BATCH and down_kind == fo.Q4_K:
        for h in (wg, wu, wd):
            h.release()
        return _moe_per_token_checks(fa, got, gate, up, down, n_experts, k, hidden, ffn, batch, x, ids, w)
    if batch <= fa.MOE_PER_TOKEN_MAX_BATCH:  # grouped all the same, but the hook keeps no record of so few tokens
        for h in (wg, wu, wd):
            h.release()
        want = _moe_oracle(down_kind, gate, up, down, n_experts, hidden, ffn, x, ids, w)
        _end_to_end_gate(got, want, what, strict)
        return got, want
    g_out, u_out, act_q, act_d, pos = (t.cpu().numpy() for t in fa.moe_intermediates(batch, k, n_experts, hidden, ffn))
    for h in (wg, wu, wd):
        h.release()

    # the grouped order: experts ascending, tokens ascending inside an expert (ffn_batch.rs:362-386)
    order = sorted((int(ids[t, s]), t, s) for t in range(batch) for s in range(k))
    assert [int(pos[t, s]) for _, t, s in order] == list(range(batch * k))

    gb, ub, db = (m.reshape(n_experts, -1) for m in (gate, up, down))
    want_down = np.zeros((batch * k, hidden), np.float32)
    act = fo.swiglu(g_out.ravel(), u_out.ravel()).reshape(batch * k, ffn)
    for e in range(n_experts):
        rows = np.array([int(pos[t, s]) for ee, t, s in order if ee == e], dtype=np.int64)
        toks = np.array([t for ee, t, s in order if ee == e], dtype=np.int64)
        if rows.size == 0:
            continue
        assert_rows_close(g_out[rows], fo.gemm(fo.Q4_K, gb[e], ffn, hidden, x[toks]), "gate of expert %d" % e)
        assert_rows_close(u_out[rows], fo.gemm(fo.Q4_K, ub[e], ffn, hidden, x[toks]), "up of expert %d" % e)
        want_down[rows] = fo.gemm(down_kind, db[e], hidden, ffn, act[rows])
    q, d, _ = fo.quantize_q8_k(act.ravel())
    assert np.array_equal(act_q.ravel(), q) and np.array_equal(bits(act_d.ravel()), bits(d))
    chained = np.zeros((batch, hidden), np.float32)
    for t in range(batch):  # the reference's accumulation order for a batch of this size
        for s in _slot_order(ids[t], batch):
            chained[t] += w[t, s] * want_down[pos[t, s]]
    assert_rows_close(got, chained, "down+combine E=%d k=%d batch=%d" % (n_experts, k, batch))

    want = _moe_oracle(down_kind, gate, up, down, n_experts, hidden, ffn, x, ids, w)
    if strict:
        _report_flipped_levels(what, got, want, gb, ub, hidden, ffn, x, ids, pos, act_q)
    _end_to_end_gate(got, want, what, strict)
    return got, want


def _report_flipped_levels(what, got, want, gb, ub, hidden, ffn, x, ids, pos, act_q):
    """What stands behind the worst row of an end-to-end comparison: the oracle's own chain for that token (its gate
    and up, its SwiGLU, its Q8_K levels) beside the levels the device quantized from ITS gate and up.  A last-bit
    difference in a gate or up output that sits on a rounding boundary of the quantizer moves one int8 level; the
    line printed (and recorded) says how many of the token's k * ffn levels differ and by how much."""
    rel = np.abs(got - want).max(axis=1) / np.abs(want).max(axis=1)
    t = int(rel.argmax())
    flips = []
    for sl in range(ids.shape[1]):
        e = int(ids[t, sl])
        g = fo.gemm(fo.Q4_K, gb[e], ffn, hidden, x[t:t + 1])
        u = fo.gemm(fo.Q4_K, ub[e], ffn, hidden, x[t:t + 1])
        q, _, _ = fo.quantize_q8_k(fo.swiglu(g.ravel(), u.ravel()))
        dev = act_q.reshape(-1, ffn)[int(pos[t, sl])]
        for i in np.nonzero(q != dev)[0]:
            flips.append((sl, e, int(i), int(dev[i]), int(q[i])))
    line = "%s: worst row is token %d at %.3g of ||y||inf; of its %d intermediate levels %d differ from the oracle's own chain: %s" % (
        what, t, rel[t], ids.shape[1] * ffn, len(flips),
        "; ".join("slot %d expert %d column %d device %d oracle %d" % f for f in flips[:6]) or "none")
    print(line, flush=True)
    import os
    d = os.environ.get("FRK_TEST_OUT", "")
    if d and os.path.isdir(d):
        with open(os.path.join(d, "parity_worst_rows.txt"), "a") as f:
            f.write(line + "\n")


def _moe_per_token_checks(fa, got, gate, up, down, n_experts, k, hidden, ffn, batch, x, ids, w):
    """A token or a few run per (token, slot) pair on the decode kernels.  Each pair is then the dense
    SwiGLU FFN of its expert's three matrices -- the very kernels, so the layer must equal, bit for
    bit, the library's own frk_hip_ffn_swiglu_dev on the expert's slices added in routing order, as the
    reference's per-position path adds them (that FFN is gated against the oracle in
    test_dense_ffn_swiglu and the GEMV tests) -- and end to end it must agree with the oracle's
    per-position layer."""
    with pytest.raises(fa.BackendError) as e:
        fa.moe_intermediates(batch, k, n_experts, hidden, ffn)
    assert e.value.code == fa.ERR_UNSUPPORTED
    gb, ub, db = (m.reshape(n_experts, -1) for m in (gate, up, down))
    composed = np.zeros((batch, hidden), np.float32)
    cache = {}
    for t in range(batch):
        xd = to_dev(x[t])
        for s in range(k):  # routing order (combine_expert_outputs, crates/frink-moe/src/lib.rs:1246-1263)
            ex = int(ids[t, s])
            if ex not in cache:
                cache[ex] = (fa.Weights.from_host(fo.Q4_K, gb[ex], ffn, hidden), fa.Weights.from_host(fo.Q4_K, ub[ex], ffn, hidden),
                             fa.Weights.from_host(fo.Q4_K, db[ex], hidden, ffn))
            ge, ue, de = cache[ex]
            y = fa.ffn_swiglu(ge, ue, de, xd).cpu().numpy()
            composed[t] = composed[t] + np.float32(w[t, s]) * y
    for hs in cache.values():
        for h in hs:
            h.release()
    assert np.array_equal(bits(got), bits(composed)), np.abs(got - composed).max()
    want = fo.moe_ffn(fo.Q4_K, gate, up, down, n_experts, hidden, ffn, x, ids, w)
    _end_to_end_gate(got, want, "moe per token E=%d k=%d %d/%d batch=%d" % (n_experts, k, hidden, ffn, batch),
                     strict=hidden >= 2048)
    return got, want


@pytest.mark.parametrize("n_experts,k,hidden,ffn,batch", [
    (16, 4, 512, 768, 1), (8, 8, 256, 256, 2), (64, 6, 1024, 512, 4), (4, 1, 2048, 256, 3), (128, 8, 2048, 768, 1),
    (32, 4, 512, 512, 16),
])
def test_moe_ffn_of_a_few_tokens_runs_per_token(fa, n_experts, k, hidden, ffn, batch):
    _moe_case(fa, n_experts, k, hidden, ffn, batch, seed=n_experts * 10 + batch, random_blocks=n_experts >= 64)


@pytest.mark.parametrize("n_experts,k,hidden,ffn,batch", [
    (8, 2, 512, 256, 40),     # a few experts hold more than one 32-row tile
    (16, 4, 256, 512, 70),
    (4, 4, 256, 256, 33),     # every token visits every expert: 33 rows -> tiles of 32 + 1
    (32, 2, 256, 256, 17),    # just above the batches that run per token: most experts idle
])
def test_moe_ffn_matches_the_oracle(fa, n_experts, k, hidden, ffn, batch):
    _moe_case(fa, n_experts, k, hidden, ffn, batch, seed=n_experts * 100 + batch)


@pytest.mark.gpu
@pytest.mark.parametrize("n_experts,k,hidden,ffn,batch", [(8, 2, 256, 512, 40), (4, 2, 768, 256, 3), (16, 4, 512, 768, 130),
                                                         (32, 4, 256, 256, 200), (128, 8, 2048, 768, 1), (16, 4, 512, 768, 16),
                                                         (8, 2, 256, 4096, 2), (8, 2, 256, 2048, 5)])
def test_moe_ffn_with_q6_k_down_experts(fa, n_experts, k, hidden, ffn, batch):
    """Q4_K gate and up, Q6_K down: the down projection runs on the Q6_K matrix-core kernel by token tile,
    and for up to 16 tokens as one decode job per (token, slot) on the expert-indexed Q6_K kernel (16, 32 or
    64 lanes to a row, by the row's length)."""
    _moe_case(fa, n_experts, k, hidden, ffn, batch, seed=n_experts * 7 + batch, down_kind=fo.Q6_K)


@pytest.mark.parametrize("gate_kind,down_kind,n_experts,k,hidden,ffn,batch", [
    (fo.MXFP4, fo.MXFP4, 8, 2, 512, 256, 1), (fo.MXFP4, fo.MXFP4, 16, 4, 512, 768, 40), (fo.Q5_0, fo.Q5_0, 8, 2, 256, 512, 9),
    (fo.IQ4_XS, fo.IQ4_XS, 8, 3, 512, 256, 33), (fo.MXFP4, fo.Q5_0, 6, 2, 256, 256, 5),
    (fo.Q5_0, fo.Q5_0, 8, 2, 256, 512, 70), (fo.MXFP4, fo.Q5_0, 6, 2, 320, 96, 45), (fo.IQ4_XS, fo.Q5_0, 4, 2, 512, 160, 64),
    (fo.MXFP4, fo.IQ4_XS, 32, 4, 576, 512, 300), (fo.MXFP4, fo.MXFP4, 5, 2, 64, 64, 200),
])
def test_moe_ffn_with_experts_of_the_other_kinds(fa, gate_kind, down_kind, n_experts, k, hidden, ffn, batch):
    """Experts in MXFP4 / Q5_0 / IQ4_XS (run_expert takes any WeightMatrix, crates/frink-moe/src/lib.rs:1068-1165):
    every (token, slot) pair on the integer tier of its kind, the slots added in the reference's order for the batch
    size (routing order below 32 tokens, ascending expert id from 32 on), an id outside the experts left out.  Below 32
    tokens a decode job per pair; from 32 on the pairs bucketed by expert and the experts, decoded to signed bytes, on
    the grouped matrix-core kernel (tiles of every fill, several tiles an expert, experts nobody chose, rows that are
    not a multiple of the kernel's 256-column step)."""
    from frink_amd import synth
    print("moe, other kinds", gate_kind, down_kind, n_experts, k, hidden, ffn, batch, flush=True)
    gate = _other_kind_blocks(gate_kind, n_experts * ffn, hidden, seed=41)
    up = _other_kind_blocks(gate_kind, n_experts * ffn, hidden, seed=42)
    down = _other_kind_blocks(down_kind, n_experts * hidden, ffn, seed=43)
    for kind, data in ((gate_kind, gate), (gate_kind, up), (down_kind, down)):
        if kind == fo.MXFP4:  # weight-sized scales, 2^-17 .. 2^-6: the intermediate's Q8_0 scales are f16 values
            blk = data.reshape(-1, 17)
            blk[:, 0] = 110 + blk[:, 0] % 12
        if kind == fo.IQ4_XS and down_kind != fo.IQ4_XS:  # (the same: d * (ls - 32) * code reaches 200 at d = 0.05)
            blk = data.reshape(-1, 136)
            blk[:, 0:2] = np.random.default_rng(46).uniform(-5e-4, 5e-4, blk.shape[0]).astype(np.float16).view(np.uint8).reshape(-1, 2)
    x = synth.activations(44, batch, hidden)
    ids, w = _route(synth.normal(45, batch * n_experts).reshape(batch, n_experts), k)
    ids = ids.astype(np.int32)
    ids[0, 0] = n_experts + 3  # an id outside the experts contributes nothing
    wg = fa.Weights.from_host(gate_kind, gate, n_experts * ffn, hidden)
    wu = fa.Weights.from_host(gate_kind, up, n_experts * ffn, hidden)
    wd = fa.Weights.from_host(down_kind, down, n_experts * hidden, ffn)
    got = fa.moe_ffn(wg, wu, wd, n_experts, to_dev(x), to_dev(ids), to_dev(w)).cpu().numpy()
    gb, ub, db = (m.reshape(n_experts, -1) for m in (gate, up, down))
    pair_out = np.zeros((batch, k, hidden), np.float32)
    for e in range(n_experts):
        toks, slots = np.nonzero(ids == e)
        if toks.size:
            g = fo.gemm(gate_kind, gb[e], ffn, hidden, x[toks], fo.INT_DOT)
            u = fo.gemm(gate_kind, ub[e], ffn, hidden, x[toks], fo.INT_DOT)
            act = fo.swiglu(g.ravel(), u.ravel()).reshape(toks.size, ffn)
            pair_out[toks, slots] = fo.gemm(down_kind, db[e], hidden, ffn, act, fo.INT_DOT)
    want = np.zeros((batch, hidden), np.float32)
    for t in range(batch):
        for sl in _slot_order(ids[t], batch):
            if 0 <= ids[t, sl] < n_experts:
                want[t] += w[t, sl] * pair_out[t, sl]
    _end_to_end_gate(got, want, "moe kinds %d/%d E=%d k=%d %d/%d batch=%d" % (gate_kind, down_kind, n_experts, k, hidden, ffn, batch), False)
    for h in (wg, wu, wd):
        h.release()


def test_moe_ffn_refuses_other_expert_kinds(fa):
    w4 = fa.Weights.from_host(fo.Q4_K, make_weights(fo.Q4_K, 2 * 256, 256, seed=1), 2 * 256, 256)
    w8 = fa.Weights.from_host(fo.Q8_0, make_weights(fo.Q8_0, 2 * 256, 256, seed=2), 2 * 256, 256)
    x, ids, w = to_dev(np.zeros((20, 256), np.float32)), to_dev(np.zeros((20, 1), np.int32)), to_dev(np.ones((20, 1), np.float32))
    for gate, up, down in ((w4, w4, w8), (w8, w4, w4)):
        with pytest.raises(fa.BackendError) as e:
            fa.moe_ffn(gate, up, down, 2, x, ids, w)
        assert e.value.code == fa.ERR_UNSUPPORTED


def test_moe_ffn_with_idle_experts_and_one_hot_routing(fa):
    # all tokens on experts {1, 5}: the other buckets are empty and their tiles must not run
    _moe_case(fa, 8, 2, 256, 256, 50, seed=77, ids_override=lambda ids: np.tile(np.array([5, 1], np.int32), (50, 1)))


def test_moe_ffn_full_size_layer(fa):
    """The MoE configuration itself: 128 experts, top-8, hidden 2048, ffn 768, all Q4_K encoded from
    N(0, 0.02) of the documented generator (frink_amd/synth.py), 512 tokens N(0, 1): every stage and every token
    row against the oracle, and the whole layer end to end (_end_to_end_gate, strict)."""
    got, want = _moe_case(fa, 128, 8, 2048, 768, 512, seed=5, sigma=0.02, strict=True)
    assert np.isfinite(got).all()


def test_moe_ffn_full_size_layer_arbitrary_block_bytes(fa):
    """The same shape over arbitrary block bytes (every scale, min and nibble pattern): stage gates
    strict as always; end to end the larger cancellation of such weights leaves the relaxed gate."""
    got, want = _moe_case(fa, 128, 8, 2048, 768, 512, seed=5, random_blocks=True)
    assert np.isfinite(got).all()


@pytest.mark.parametrize("batch", [3, 40])
def test_moe_ffn_leaves_out_ids_outside_the_experts(fa, batch):
    """An id outside [0, n_experts) contributes nothing, on the per-token path (batch 3) and on the grouped
    path (batch 40) alike: the oracle with those slots dropped."""
    def spoil(ids):
        ids = ids.copy()
        ids[0, 0] = -1
        ids[1, 1] = 8
        ids[batch - 1, :] = np.array([8, -1], np.int32)  # a token with no valid slot: zeros
        return ids
    n_experts, k, hidden, ffn = 8, 2, 256, 256
    from frink_amd import synth
    gate, up, down = _stacked_experts(n_experts, hidden, ffn, 4242)
    x = synth.activations(4250, batch, hidden)
    ids, w = _route(synth.normal(4251, batch * n_experts).reshape(batch, n_experts), k)
    ids = spoil(ids.astype(np.int32))
    hs = [fa.Weights.from_host(fo.Q4_K, m, r, c) for m, r, c in ((gate, n_experts * ffn, hidden), (up, n_experts * ffn, hidden),
                                                                 (down, n_experts * hidden, ffn))]
    got = fa.moe_ffn(hs[0], hs[1], hs[2], n_experts, to_dev(x), to_dev(ids), to_dev(w)).cpu().numpy()
    for h in hs:
        h.release()
    want = fo.moe_ffn(fo.Q4_K, gate, up, down, n_experts, hidden, ffn, x, ids, w)
    assert not got[batch - 1].any() and not want[batch - 1].any()
    rel = np.abs(got[:-1] - want[:-1]).max(axis=1) / np.abs(want[:-1]).max(axis=1)
    assert (rel <= TOL).mean() >= 0.9 and rel.max() <= 10 * TOL, rel.max()


# ------------------------------------------------------------------ the C++ host mirror

def test_cpp_host_mirror_launches(fa):
    """tests/host_mirror_check.cpp --gpu: probe, launch_matvec and launch_mul_mm through
    frink_amd/host/frink_hip.hpp against closed forms."""
    import os
    import subprocess
    from frink_amd import build as fb
    if not os.path.exists(fb.HOST_CHECK_BIN):
        fb.build_host_check()
    env = {k: v for k, v in os.environ.items() if k != "FRINK_HIP"}
    r = subprocess.run([fb.HOST_CHECK_BIN, "--gpu"], env=env, text=True, capture_output=True, timeout=120)
    print(r.stdout, flush=True)
    assert r.returncode == 0 and "FAIL" not in r.stdout, r.stdout + r.stderr


# ------------------------------------------------------------------ Q5_0, IQ4_XS, MXFP4 (GGUF block form)

def _other_kind_blocks(kind, rows, cols, seed):
    """valid blocks with finite scales and every code value in play (these kinds have no encoder here)"""
    bb, be = fo.BLOCK[kind]
    n = rows * cols // be
    rng = np.random.default_rng(seed)
    blocks = rng.integers(0, 256, (n, bb), dtype=np.uint8)
    if kind == fo.MXFP4:
        blocks[:, 0] = rng.integers(100, 140, n)
        blocks[0, 0], blocks[1 % n, 0] = 0, 1  # the subnormal scales 2^-127 and 2^-126
    else:
        blocks[:, 0:2] = rng.uniform(-0.05, 0.05, n).astype(np.float16).view(np.uint8).reshape(n, 2)
    return blocks.ravel()


@pytest.mark.parametrize("kind,rows,cols", [
    (fo.Q5_0, 33, 4096), (fo.Q5_0, 5, 32), (fo.Q5_0, 7, 96), (fo.IQ4_XS, 33, 4096), (fo.IQ4_XS, 5, 256), (fo.IQ4_XS, 3, 768),
    (fo.MXFP4, 33, 4096), (fo.MXFP4, 5, 32), (fo.MXFP4, 9, 2880),
])
def test_other_kinds_dequant_and_get_rows_are_bit_exact(fa, kind, rows, cols):
    import torch
    data = _other_kind_blocks(kind, rows, cols, seed=kind + rows)
    w = fa.Weights.from_host(kind, data, rows, cols)
    want = fo.dequant(kind, data).reshape(rows, cols)
    assert np.array_equal(bits(w.dequant().cpu().numpy()), bits(want))
    ids = np.array([rows - 1, 0, rows // 2, 0], np.int32)
    assert np.array_equal(bits(w.get_rows(torch.from_numpy(ids).cuda()).cpu().numpy()), bits(want[ids]))
    w.release()


@pytest.mark.parametrize("kind,rows,cols,batch", [
    (fo.Q5_0, 70, 1024, 1), (fo.Q5_0, 300, 4096, 3), (fo.IQ4_XS, 70, 1024, 1), (fo.IQ4_XS, 130, 4096, 2), (fo.IQ4_XS, 9, 16384, 1),
    (fo.MXFP4, 70, 1024, 1), (fo.MXFP4, 64, 2880, 4),
])
def test_other_kinds_gemv_matches_the_oracle(fa, kind, rows, cols, batch):
    """The decode GEMV of Q5_0 / IQ4_XS / MXFP4 is the f32 dot of the reference's decode path."""
    from frink_amd import synth
    print("other kinds", kind, rows, cols, batch, flush=True)
    data = _other_kind_blocks(kind, rows, cols, seed=kind * 3 + rows)
    x = synth.activations(rows + cols, batch, cols, outlier_frac=0.01)
    w = fa.Weights.from_host(kind, data, rows, cols)
    # (a batch would take the integer tier: here every row through the decode entry point)
    got = np.stack([w.gemv(to_dev(x[b])).cpu().numpy() for b in range(batch)])
    want = fo.gemm(kind, data, rows, cols, x, fo.F32_DOT)
    assert_rows_close(got, want, "kind %d" % kind)
    deq = fo.dequant(kind, data).reshape(rows, cols).astype(np.float64)
    bound = 4e-6 * (np.abs(deq) @ np.abs(x.T).astype(np.float64)).T
    assert (np.abs(got - (deq @ x.T.astype(np.float64)).T) <= bound).all()
    w.release()


@pytest.mark.parametrize("kind,rows,cols", [
    (fo.Q5_0, 70, 1024), (fo.Q5_0, 300, 4096), (fo.Q5_0, 17, 96), (fo.Q5_0, 9, 16384), (fo.Q5_0, 2100, 512),
    (fo.IQ4_XS, 70, 1024), (fo.IQ4_XS, 130, 4096), (fo.IQ4_XS, 9, 16384), (fo.IQ4_XS, 5, 256), (fo.IQ4_XS, 33, 4352),
    (fo.MXFP4, 70, 1024), (fo.MXFP4, 64, 2880), (fo.MXFP4, 9, 16384), (fo.MXFP4, 5, 32),
])
def test_other_kinds_integer_gemv_matches_the_oracle(fa, kind, rows, cols):
    """FRK_ACT_INT8 on Q5_0 / MXFP4 (the activation as Q8_0 blocks: dot_q5_0_q8 / dot_mxfp4_q8) and IQ4_XS (as Q8_K:
    dot_iq4_xs_q8_k): rows of one block and of 512, more rows than one round of workgroups, unit counts that are
    not a multiple of 64 (the lanes of a wavefront's last round idle), the subnormal MXFP4 scales."""
    from frink_amd import synth
    print("other kinds, integer tier", kind, rows, cols, flush=True)
    data = _other_kind_blocks(kind, rows, cols, seed=kind * 5 + rows)
    x = synth.activations(rows + cols + 1, 1, cols, outlier_frac=0.01)[0]
    w = fa.Weights.from_host(kind, data, rows, cols)
    got = w.gemv(to_dev(x), act_mode=fa.ACT_INT8).cpu().numpy()
    want = fo.gemv(kind, data, rows, cols, x, fo.INT_DOT)
    assert_rows_close(got[None], want[None], "integer gemv kind %d %dx%d" % (kind, rows, cols))
    # the integers are exact and the float step is a handful of operations a block: far inside the tolerance
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max()
    # homogeneity: a power of two on the activation scales its Q8 scales exactly and leaves the quants alone
    y4 = w.gemv(to_dev(x * np.float32(4.0)), act_mode=fa.ACT_INT8).cpu().numpy()
    assert np.array_equal(bits(y4), bits(got * np.float32(4.0)))
    w.release()


@pytest.mark.parametrize("kind,rows,cols,batch", [
    (fo.Q5_0, 70, 1024, 2), (fo.Q5_0, 300, 4096, 3), (fo.Q5_0, 96, 512, 4), (fo.Q5_0, 200, 1056, 40), (fo.Q5_0, 130, 2048, 130),
    (fo.Q5_0, 64, 96, 33), (fo.MXFP4, 70, 1024, 2), (fo.MXFP4, 64, 2880, 4), (fo.MXFP4, 200, 1056, 40), (fo.MXFP4, 130, 2048, 130),
    (fo.MXFP4, 96, 32, 7), (fo.IQ4_XS, 70, 1024, 2), (fo.IQ4_XS, 130, 4096, 5), (fo.IQ4_XS, 40, 768, 17),
    (fo.IQ4_XS, 64, 256, 4), (fo.IQ4_XS, 100, 2304, 33), (fo.IQ4_XS, 200, 1280, 64), (fo.IQ4_XS, 130, 2048, 130),
    (fo.IQ4_XS, 33, 14336, 40), (fo.IQ4_XS, 1000, 512, 300),
])
def test_other_kinds_batches_take_the_integer_tier(fa, kind, rows, cols, batch):
    """A batch of Q5_0 / MXFP4 / IQ4_XS is the reference's integer tier (q8_row_dot / q8k_row_dot per (row, activation),
    crates/frink-core/src/weight_matrix.rs:392-420): up to three rows the decode kernel per row, from four on Q5_0 and
    MXFP4 decoded into the Q8_0 planar form and multiplied on the matrix cores -- every workgroup shape of that kernel,
    ragged tiles, rows that are not a multiple of its 256-column step -- and IQ4_XS decoded to signed bytes with their
    integer block scales, against Q8_K activations (the same kernel's form with a float scale per 256; long rows
    split between workgroups, grids of several token tiles)."""
    from frink_amd import synth
    print("other kinds, batch", kind, rows, cols, batch, flush=True)
    data = _other_kind_blocks(kind, rows, cols, seed=kind * 7 + rows + batch)
    if kind == fo.MXFP4:
        blk = data.reshape(-1, 17)
        blk[:2, 0] = (104, 143)  # the ends of the range whose halved scales are f16 values: 2^-24 and 2^15
    x = synth.activations(rows + cols + batch, batch, cols, outlier_frac=0.01)
    w = fa.Weights.from_host(kind, data, rows, cols)
    got = w.gemm(to_dev(x)).cpu().numpy()
    want = fo.gemm(kind, data, rows, cols, x, fo.INT_DOT)
    assert got.shape == (batch, rows)
    assert_rows_close(got, want, "batch of kind %d %dx%d x %d" % (kind, rows, cols, batch))
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max()
    half = w.gemm(to_dev(x * np.float32(0.5))).cpu().numpy()
    assert np.array_equal(bits(half), bits(got * np.float32(0.5)))
    w.release()


def test_mxfp4_batch_with_scales_outside_f16_keeps_the_decode_kernel(fa):
    """Halved E8M0 scales below 2^-24 or above 2^15 are not f16 values: such a matrix's batches run the integer decode
    kernel per row (f32 scales), with the same results to the tolerance."""
    from frink_amd import synth
    rows, cols, batch = 64, 1024, 9
    data = _other_kind_blocks(fo.MXFP4, rows, cols, seed=5)
    data.reshape(-1, 17)[::7, 0] = 160  # 2^32
    x = synth.activations(6, batch, cols, outlier_frac=0.01)
    w = fa.Weights.from_host(fo.MXFP4, data, rows, cols)
    got = w.gemm(to_dev(x)).cpu().numpy()
    assert_rows_close(got, fo.gemm(fo.MXFP4, data, rows, cols, x, fo.INT_DOT), "mxfp4 with wide scales")
    w.release()


def test_other_kinds_integer_gemv_refuses_rows_it_cannot_hold(fa):
    data = _other_kind_blocks(fo.Q5_0, 2, 32768, seed=1)
    w = fa.Weights.from_host(fo.Q5_0, data, 2, 32768)
    with pytest.raises(fa.BackendError) as e:
        w.gemv(to_dev(np.zeros(32768, np.float32)), act_mode=fa.ACT_INT8)
    assert e.value.code == fa.ERR_UNSUPPORTED
    w.release()


@pytest.mark.parametrize("kind", [fo.Q5_0, fo.IQ4_XS, fo.MXFP4])
def test_other_kinds_through_the_shared_activation_entry_points(fa, kind):
    """Q5_0 / IQ4_XS / MXFP4 matrices as q/k/v-style groups (frk_hip_gemv_multi_dev, alone and mixed with a K-quant)
    and as an FFN's projections (frk_hip_ffn_swiglu_dev and the host-buffer forms): the backend lists these kinds, so
    every entry point a model's projections go through must take them.  Each output against the oracle: the f32 dot
    for these kinds, the integer dot for the K-quant beside them."""
    from frink_amd import synth
    hidden, ffn = 512, 768
    bb, be = fo.BLOCK[kind]
    gate = _other_kind_blocks(kind, ffn, hidden, seed=kind + 1)
    up = _other_kind_blocks(kind, ffn, hidden, seed=kind + 2)
    down = _other_kind_blocks(kind, hidden, ffn, seed=kind + 3)
    kq = make_weights(fo.Q4_K, 96, hidden, seed=kind + 4)
    x = synth.activations(kind + 5, 1, hidden)[0]
    wg, wu, wd = (fa.Weights.from_host(kind, d, r, c) for d, r, c in ((gate, ffn, hidden), (up, ffn, hidden), (down, hidden, ffn)))
    wk = fa.Weights.from_host(fo.Q4_K, kq, 96, hidden)
    xd = to_dev(x)
    g_want = fo.gemv(kind, gate, ffn, hidden, x, fo.F32_DOT)
    u_want = fo.gemv(kind, up, ffn, hidden, x, fo.F32_DOT)
    k_want = fo.gemv(fo.Q4_K, kq, 96, hidden, x)
    for group, wants in (([wg, wu], [g_want, u_want]), ([wg, wk, wu], [g_want, k_want, u_want]), ([wk, wg], [k_want, g_want])):
        outs = fa.gemv_multi(group, xd)
        for i, (o, want) in enumerate(zip(outs, wants)):
            assert_rows_close(o.cpu().numpy()[None], want[None], "gemv_multi kind %d, matrix %d of %d" % (kind, i, len(group)))
    # the FFN: gate, up, SwiGLU, down -- each stage from the device's previous one
    y = fa.ffn_swiglu(wg, wu, wd, xd).cpu().numpy()
    g_dev, u_dev = (t.cpu().numpy() for t in fa.gemv_multi([wg, wu], xd))
    act = fo.swiglu(g_dev, u_dev)
    assert_rows_close(y[None], fo.gemv(kind, down, hidden, ffn, act, fo.F32_DOT)[None], "ffn_swiglu kind %d" % kind)
    # mixed: K-quant gate and up, a down projection of this kind
    g4, u4 = make_weights(fo.Q4_K, ffn, hidden, seed=kind + 6), make_weights(fo.Q4_K, ffn, hidden, seed=kind + 7)
    w4g, w4u = fa.Weights.from_host(fo.Q4_K, g4, ffn, hidden), fa.Weights.from_host(fo.Q4_K, u4, ffn, hidden)
    y = fa.ffn_swiglu(w4g, w4u, wd, xd).cpu().numpy()
    g_dev, u_dev = (t.cpu().numpy() for t in fa.gemv_multi([w4g, w4u], xd))
    assert_rows_close(y[None], fo.gemv(kind, down, hidden, ffn, fo.swiglu(g_dev, u_dev), fo.F32_DOT)[None], "ffn, down kind %d" % kind)
    # the host-buffer forms
    rb = hidden // be * bb
    outs = fa.launch_matvec_multi(x, [fa.MatvecLaunch.of(kind, gate, ffn, rb), fa.MatvecLaunch.of(fo.Q4_K, kq, 96, hidden // 256 * 144)])
    assert_rows_close(outs[0][None], g_want[None], "launch_matvec_multi kind %d" % kind)
    assert_rows_close(outs[1][None], k_want[None], "launch_matvec_multi beside kind %d" % kind)
    out = fa.launch_dense_ffn_swiglu(fa.MatvecLaunch.of(kind, gate, ffn, rb), fa.MatvecLaunch.of(kind, up, ffn, rb),
                                     fa.MatvecLaunch.of(kind, down, hidden, ffn // be * bb), x)
    want = fo.gemv(kind, down, hidden, ffn, fo.swiglu(g_want, u_want), fo.F32_DOT)
    rel = np.abs(out - want).max() / np.abs(want).max()
    assert rel <= 10 * TOL, rel  # (end to end over f32 stages: no quantizer between them, reassociation only)
    for h in (wg, wu, wd, wk, w4g, w4u):
        h.release()


# ------------------------------------------------------------------ the K-quants' f32 dot (the reference's x86 decode default)

@pytest.mark.parametrize("kind,rows,cols", [
    (fo.Q4_K, 70, 1024), (fo.Q4_K, 9, 256), (fo.Q4_K, 300, 4096), (fo.Q4_K, 17, 16384), (fo.Q4_K, 3, 11008), (fo.Q4_K, 1, 6400),
    (fo.Q5_K, 70, 1024), (fo.Q5_K, 33, 768), (fo.Q5_K, 128, 4096),
    (fo.Q6_K, 70, 1024), (fo.Q6_K, 5, 256), (fo.Q6_K, 64, 14336), (fo.Q6_K, 257, 2048),
])
def test_k_quant_f32_dot_gemv(fa, kind, rows, cols):
    """FRK_ACT_F32_DOT: dequantized weights times the f32 activation (dot_q4_k_f32 / dot_q5_k_f32 / dot_q6_k_f32).
    Against the oracle's f32 dot within the tolerance, and -- what tells it from the integer path, whose
    activation is rounded to eight bits -- against the product of the dequantized matrix in float64 to
    within float32 summation error."""
    from frink_amd import synth
    print("f32 dot", kind, rows, cols, flush=True)
    data = make_weights(kind, rows, cols, seed=kind * 31 + rows)
    x = synth.activations(rows + cols, 1, cols, outlier_frac=0.01)[0]
    w = fa.Weights.from_host(kind, data, rows, cols)
    got = w.gemv(to_dev(x), act_mode=fa.ACT_F32_DOT).cpu().numpy()
    want = fo.gemv(kind, data, rows, cols, x, fo.F32_DOT)
    assert_rows_close(got[None], want[None], "f32 dot kind %d" % kind)
    deq = fo.dequant(kind, data).reshape(rows, cols).astype(np.float64)
    exact = deq @ x.astype(np.float64)
    bound = 4e-6 * (np.abs(deq) @ np.abs(x).astype(np.float64))
    assert (np.abs(got - exact) <= bound).all(), float((np.abs(got - exact) / bound).max())
    ints = w.gemv(to_dev(x)).cpu().numpy()
    assert (np.abs(ints - exact) > bound).any(), "the integer path is not expected to be this close"
    w.release()


def test_k_quant_f32_dot_refuses_long_rows(fa):
    data = make_weights(fo.Q4_K, 2, 32768, seed=3)
    w = fa.Weights.from_host(fo.Q4_K, data, 2, 32768)
    with pytest.raises(fa.BackendError) as e:
        w.gemv(to_dev(np.zeros(32768, np.float32)), act_mode=fa.ACT_F32_DOT)
    assert e.value.code == fa.ERR_UNSUPPORTED
    w.release()


# ------------------------------------------------------------------ thin batched GEMM (batched decode)

@pytest.mark.parametrize("kind,rows,cols,batch", [
    (fo.Q4_K, 70, 1024, 2), (fo.Q4_K, 33, 512, 3), (fo.Q4_K, 128, 4096, 8), (fo.Q4_K, 64, 256, 5),
    (fo.Q4_K, 40, 2048, 11), (fo.Q4_K, 16, 768, 15), (fo.Q4_K, 100, 1024, 16), (fo.Q4_K, 17, 256, 16),
    (fo.Q4_K, 1000, 4096, 9), (fo.Q4_K, 31, 8192, 13), (fo.Q4_K, 20, 16384, 6), (fo.Q4_K, 18, 32768, 5),
    (fo.Q6_K, 70, 1024, 2), (fo.Q6_K, 33, 512, 3), (fo.Q6_K, 48, 14336, 8), (fo.Q6_K, 64, 256, 7),
    (fo.Q6_K, 40, 2048, 11), (fo.Q6_K, 24, 768, 40), (fo.Q6_K, 19, 28672, 4), (fo.Q6_K, 50, 4096, 5),
    # (the streamed Q6_K kernel: rows of 2, 6, 14 and 28 blocks -- one wavefront, uneven shares, a last row group partly empty)
    (fo.Q6_K, 37, 1536, 8), (fo.Q6_K, 20, 3584, 6), (fo.Q6_K, 16, 7168, 8), (fo.Q6_K, 33, 512, 17),
])
def test_thin_gemm_matches_the_oracle_and_the_gemv(fa, kind, rows, cols, batch):
    from frink_amd import synth
    print("thin gemm", kind, rows, cols, batch, flush=True)
    data = make_weights(kind, rows, cols, seed=kind * 1000 + rows + batch)
    x = synth.activations(rows + cols + batch, batch, cols, outlier_frac=0.01)
    w = fa.Weights.from_host(kind, data, rows, cols)
    xd = to_dev(x)
    got = w.gemm(xd).cpu().numpy()
    assert got.shape == (batch, rows)
    assert_rows_close(got, fo.gemm(kind, data, rows, cols, x), "thin gemm kind %d batch %d" % (kind, batch))
    # same integer sums, same scale expression, but a different lane-to-unit map than the decode
    # GEMV: equal to it within float summation order
    for b in (0, batch - 1):
        one = w.gemv(xd[b].contiguous()).cpu().numpy()
        assert np.abs(one - got[b]).max() <= 1e-5 * np.abs(one).max()
    w.release()


@pytest.mark.parametrize("kind", [fo.Q4_K, fo.Q5_K, fo.Q6_K, fo.Q8_0])
def test_gemm_at_every_batch_size_where_the_kernel_changes(fa, kind):
    """frk_hip_gemm_dev picks a kernel by the batch size (one row: the GEMV; 2: dot4; 3..16: thin on
    the matrix cores; wider: 8-row groups, or the MFMA GEMM from 33 rows (Q4_K) or from 25 or 41 (Q6_K, by the matrix's size); Q8_0:
    the MFMA GEMM from two rows, its token tile growing at 33 and 65): every size on either side of a threshold, on a ragged matrix, against the oracle."""
    from frink_amd import synth
    rows, cols = 72, 512
    data = make_weights(kind, rows, cols, seed=900 + kind)
    w = fa.Weights.from_host(kind, data, rows, cols)
    for batch in (1, 2, 3, 4, 5, 8, 9, 16, 17, 24, 25, 31, 32, 33, 40, 41, 47, 48, 49, 64, 65, 111, 112, 113, 129):
        print("gemm boundary", kind, batch, flush=True)
        x = synth.activations(901 + batch, batch, cols, outlier_frac=0.01)
        got = w.gemm(to_dev(x)).cpu().numpy()
        # one Q8_0 row is the f32 dot of the decode path, a Q8_0 batch the integer path
        want = fo.gemm(kind, data, rows, cols, x, fo.F32_DOT if kind == fo.Q8_0 and batch == 1 else fo.INT_DOT)
        assert got.shape == (batch, rows)
        assert_rows_close(got, want, "gemm kind %d batch %d" % (kind, batch))
    w.release()


@pytest.mark.parametrize("rows,cols,batch", [(100, 1024, 40), (33, 2048, 37), (50, 4096, 9), (4096, 14336, 64)])
def test_wide_q6_k_batch_is_one_launch_of_row_groups(fa, rows, cols, batch):
    """A Q6_K batch wider than the 8 rows one workgroup stages runs as a grid of 8-row groups (the
    last one ragged): every activation row against the oracle, on a slice of weight rows at full size."""
    from frink_amd import synth
    print("wide q6_k", rows, cols, batch, flush=True)
    data = make_weights(fo.Q6_K, rows, cols, seed=rows + batch)
    x = synth.activations(rows * 7 + batch, batch, cols, outlier_frac=0.01)
    w = fa.Weights.from_host(fo.Q6_K, data, rows, cols)
    got = w.gemm(to_dev(x)).cpu().numpy()
    assert got.shape == (batch, rows)
    for row0 in sorted({0, max(rows - 64, 0)}):
        n = min(64, rows - row0)
        want = fo.gemm(fo.Q6_K, data, rows, cols, x, row0=row0, nrows=n)
        assert_rows_close(got[:, row0:row0 + n], want, "wide q6_k %dx%d batch %d rows %d.." % (rows, cols, batch, row0))
    w.release()


@pytest.mark.parametrize("rows,cols,batch", [(300, 768, 130), (64, 256, 112), (13000, 512, 500), (257, 1024, 200),
                                             (4096, 14336, 512), (4096, 14336, 41), (4096, 14336, 128),
                                             (4096, 4096, 64), (500, 8192, 256), (96, 2048, 45)])
def test_gemm_q6_k_on_the_matrix_cores(fa, rows, cols, batch):
    """Q6_K batches from 25 rows on (41 for small matrices) take the int8 MFMA kernel (four pre-scaled
    planes per 16-weight group): both workgroup shapes (256 weight rows at 13000x512, 128 elsewhere),
    the blocks split between 2, 4 and 8 workgroups whose sums are added in order, ragged last row and
    token tiles, every activation row against the oracle on the first, a middle and the last
    weight rows, and exact homogeneity."""
    from frink_amd import synth
    print("gemm q6_k", rows, cols, batch, flush=True)
    data = make_weights(fo.Q6_K, rows, cols, seed=rows + batch)
    x = synth.activations(rows * 5 + batch, batch, cols, outlier_frac=0.01)
    w = fa.Weights.from_host(fo.Q6_K, data, rows, cols)
    got = w.gemm(to_dev(x)).cpu().numpy()
    assert got.shape == (batch, rows)
    n = min(64, rows)
    for row0 in sorted({0, (rows // 2) // 32 * 32 + 5 if rows > 128 else 0, rows - n}):
        want = fo.gemm(fo.Q6_K, data, rows, cols, x, row0=row0, nrows=n)
        assert_rows_close(got[:, row0:row0 + n], want, "gemm q6_k %dx%d batch %d rows %d.." % (rows, cols, batch, row0))
    half = w.gemm(to_dev(x * np.float32(0.5))).cpu().numpy()
    assert np.array_equal(bits(half), bits(got * np.float32(0.5)))
    w.release()


@pytest.mark.parametrize("rows,cols,batch", [(72, 512, 5), (100, 96, 33), (33, 288, 70), (64, 4096, 129),
                                             (1000, 1056, 300), (4096, 4096, 512), (4096, 14336, 512)])
def test_gemm_q8_0_on_the_matrix_cores(fa, rows, cols, batch):
    """A Q8_0 batch is quantized to Q8_0 activation blocks and multiplied on the int8 MFMA, one
    instruction per 32-wide block, the block's scales dw*da formed by an f16 MFMA: the three workgroup
    shapes, ragged row and token tiles, rows that are not a multiple of the 256-column step (96, 288,
    1056), every activation row against the oracle on the first, a middle and the last weight rows,
    and exact homogeneity."""
    from frink_amd import synth
    print("gemm q8_0", rows, cols, batch, flush=True)
    data = make_weights(fo.Q8_0, rows, cols, seed=rows + batch)
    x = synth.activations(rows * 7 + batch, batch, cols, outlier_frac=0.01)
    w = fa.Weights.from_host(fo.Q8_0, data, rows, cols)
    got = w.gemm(to_dev(x)).cpu().numpy()
    assert got.shape == (batch, rows)
    n = min(64, rows)
    for row0 in sorted({0, (rows // 2) // 32 * 32 + 5 if rows > 128 else 0, rows - n}):
        want = fo.gemm(fo.Q8_0, data, rows, cols, x, fo.INT_DOT, row0=row0, nrows=n)
        assert_rows_close(got[:, row0:row0 + n], want, "gemm q8_0 %dx%d batch %d rows %d.." % (rows, cols, batch, row0))
    half = w.gemm(to_dev(x * np.float32(0.5))).cpu().numpy()
    assert np.array_equal(bits(half), bits(got * np.float32(0.5)))
    w.release()


def test_gemm_q8_0_keeps_scales_below_the_f16_normal_range(fa):
    """Block scales under 2^-14 are subnormal f16 values: weights of size 2e-4 give such weight scales,
    activations of size 1e-3 such activation scales.  The scale product must not flush them."""
    from frink_amd import synth
    rows, cols, batch = 96, 512, 40
    data = make_weights(fo.Q8_0, rows, cols, seed=77, sigma=2e-4)
    d_bits = np.frombuffer(data, np.uint8).reshape(rows, cols // 32, 34)[:, :, :2].copy().view(np.uint16)
    assert ((d_bits & 0x7c00) == 0).all() and (d_bits & 0x3ff).any(), "the weight scales are meant to be subnormal"
    w = fa.Weights.from_host(fo.Q8_0, data, rows, cols)
    x = synth.activations(78, batch, cols, outlier_frac=0.0)
    got = w.gemm(to_dev(x)).cpu().numpy()
    assert_rows_close(got, fo.gemm(fo.Q8_0, data, rows, cols, x, fo.INT_DOT), "subnormal weight scales")
    assert np.abs(got).max() > 0
    w.release()
    data = make_weights(fo.Q8_0, rows, cols, seed=79)
    w = fa.Weights.from_host(fo.Q8_0, data, rows, cols)
    x = (x * np.float32(1e-3)).astype(np.float32)
    _, d = fo.quantize_q8_0(x.reshape(-1))
    assert (d < 2.0 ** -14).all() and (d > 0).any(), "the activation scales are meant to be subnormal"
    got = w.gemm(to_dev(x)).cpu().numpy()
    assert_rows_close(got, fo.gemm(fo.Q8_0, data, rows, cols, x, fo.INT_DOT), "subnormal activation scales")
    assert np.abs(got).max() > 0
    w.release()


@pytest.mark.parametrize("kind,rows,cols,seed", [(fo.Q4_K, 14336, 4096, 21), (fo.Q6_K, 4096, 14336, 22)])
def test_full_size_thin_gemm_m8(fa, kind, rows, cols, seed):
    """Batched decode, M=8, at the FFN shapes: every weight row against the oracle for every
    activation row (0.5 G multiply-adds: seconds on the threaded scalar oracle), and each batch row
    against the decode GEMV of that row."""
    from frink_amd import synth
    print("full thin gemm", kind, rows, cols, flush=True)
    data = make_weights(kind, rows, cols, seed=seed)
    x = synth.activations(seed + 1, 8, cols)
    w = fa.Weights.from_host(kind, data, rows, cols)
    xd = to_dev(x)
    y = w.gemm(xd).cpu().numpy()
    want = fo.gemm(kind, data, rows, cols, x)
    ninf = np.abs(want).max(axis=1)
    err = np.abs(y - want).max(axis=1)
    record("thin gemm M=8 kind %d %dx%d, all rows" % (kind, rows, cols), float((err / ninf).max()))
    assert (err <= TOL * ninf).all(), float((err / ninf).max())
    one = w.gemv(xd[5].contiguous()).cpu().numpy()
    assert np.abs(one - y[5]).max() <= 1e-5 * np.abs(one).max()
    w.release()


# ------------------------------------------------------------------ shared activation, fused FFN

def _ffn_oracle(gate, up, down, ffn, hidden, x):
    g = fo.gemv(fo.Q4_K, gate, ffn, hidden, x)
    u = fo.gemv(fo.Q4_K, up, ffn, hidden, x)
    return g, u, fo.swiglu(g, u)


def test_gemv_multi_shares_one_quantized_activation(fa):
    from frink_amd import synth
    hidden = 1024
    shapes = [(fo.Q4_K, 96), (fo.Q6_K, 40), (fo.Q8_0, 72), (fo.Q5_K, 24), (fo.Q4_K, 33)]
    datas = [make_weights(k, r, hidden, seed=300 + i) for i, (k, r) in enumerate(shapes)]
    ws = [fa.Weights.from_host(k, d, r, hidden) for (k, r), d in zip(shapes, datas)]
    x = synth.activations(301, 1, hidden, outlier_frac=0.01)[0]
    ys = fa.gemv_multi(ws, to_dev(x))
    for (k, r), d, y in zip(shapes, datas, ys):
        want = fo.gemv(k, d, r, hidden, x, fo.F32_DOT if k == fo.Q8_0 else fo.INT_DOT)
        assert_rows_close(y.cpu().numpy()[None], want[None], "gemv_multi kind %d" % k)
    # the host-buffer form (launch_matvec_multi)
    launches = [fa.MatvecLaunch.of(k, d, r, hidden // fo.BLOCK[k][1] * fo.BLOCK[k][0]) for (k, r), d in zip(shapes, datas)]
    outs = fa.launch_matvec_multi(x, launches)
    for o, y in zip(outs, ys):
        assert np.array_equal(bits(o), bits(y.cpu().numpy()))
    with pytest.raises(fa.BackendError) as e:
        fa.launch_matvec_multi(x[:512], launches)
    assert e.value.code == fa.ERR_SHAPE
    for w in ws:
        w.release()


@pytest.mark.parametrize("hidden,rows", [(4096, (4096, 1024, 1024)), (1024, (33, 7)), (2048, (100, 5, 64, 31, 9)),
                                         (16384, (40, 24)), (4096, (4, 8, 12, 4)), (4096, (132, 64, 6)), (2048, (8, 64, 16)),
                                         (2048, (512, 128, 128, 256, 8))])
def test_gemv_multi_groups_q4_k_matrices_in_one_launch(fa, hidden, rows):
    """q/k/v and other groups of Q4_K matrices (up to four per launch, a fifth starts the next): every
    output agrees with the oracle and with the lone GEMV of its matrix (to rounding: rows of 2048, 4096,
    8192 or 16384 columns take another kernel alone, which adds a row's blocks in another order)."""
    from frink_amd import synth
    print("gemv group", hidden, rows, flush=True)
    datas = [make_weights(fo.Q4_K, r, hidden, seed=700 + i) for i, r in enumerate(rows)]
    ws = [fa.Weights.from_host(fo.Q4_K, d, r, hidden) for r, d in zip(rows, datas)]
    x = synth.activations(701, 1, hidden, outlier_frac=0.01)[0]
    xd = to_dev(x)
    ys = fa.gemv_multi(ws, xd)
    for w, r, d, y in zip(ws, rows, datas, ys):
        got = y.cpu().numpy()
        assert got.shape == (r,)
        lone = w.gemv(xd).cpu().numpy()
        assert np.abs(got - lone).max() <= 2e-6 * np.abs(lone).max()
        # (rows of 2048 and 4096 columns in whole spans -- 8 or 4 rows -- run on the lone GEMV's own kernel as a list)
        if hidden not in (2048, 4096, 8192, 16384) or (hidden <= 4096 and all(q % (16384 // hidden) == 0 for q in rows[:4]) and len(rows) <= 4):
            assert np.array_equal(bits(got), bits(lone))
        if r <= 1024:
            assert_rows_close(got[None], fo.gemv(fo.Q4_K, d, r, hidden, x)[None], "grouped gemv %d rows" % r)
    for w in ws:
        w.release()


@pytest.mark.parametrize("hidden,ffn", [(512, 768), (4096, 14336)])
def test_dense_ffn_swiglu(fa, hidden, ffn):
    """gate/up Q4_K, down Q6_K (the Llama-3-8B FFN at full size): each stage from the device's own
    previous stage, as for the MoE layer -- the down projection quantizes its input, a step function."""
    from frink_amd import synth
    print("ffn", hidden, ffn, flush=True)
    gate = make_weights(fo.Q4_K, ffn, hidden, seed=401)
    up = make_weights(fo.Q4_K, ffn, hidden, seed=402)
    down = make_weights(fo.Q6_K, hidden, ffn, seed=403)
    x = synth.activations(404, 1, hidden)[0]
    wg, wu, wd = (fa.Weights.from_host(k, d, r, c) for k, d, r, c in
                  ((fo.Q4_K, gate, ffn, hidden), (fo.Q4_K, up, ffn, hidden), (fo.Q6_K, down, hidden, ffn)))
    xd = to_dev(x)
    y = fa.ffn_swiglu(wg, wu, wd, xd).cpu().numpy()
    g_dev, u_dev = (t.cpu().numpy() for t in fa.gemv_multi([wg, wu], xd))
    g, u, _ = _ffn_oracle(gate, up, down, ffn, hidden, x)
    assert_rows_close(g_dev[None], g[None], "gate")
    assert_rows_close(u_dev[None], u[None], "up")
    act = fo.swiglu(g_dev, u_dev)                      # the device's gate/up through the oracle's SwiGLU
    want = fo.gemv(fo.Q6_K, down, hidden, ffn, act)
    assert_rows_close(y[None], want[None], "down(silu(gate)*up)")
    # end to end against the oracle's own chain
    e2e = fo.gemv(fo.Q6_K, down, hidden, ffn, fo.swiglu(g, u))
    rel = np.abs(y - e2e).max() / np.abs(e2e).max()
    print("ffn end to end: %.3g of ||y||inf" % rel, flush=True)
    record("dense ffn %dx%d end to end" % (hidden, ffn), rel)
    # the full-size FFN holds the tolerance itself; the small one only ten times it (the quantizer
    # between the projections is a step function, see _end_to_end_gate)
    assert rel <= (TOL if hidden >= 4096 else 10 * TOL), rel
    if hidden == 512:  # the host-buffer form (launch_dense_ffn_swiglu)
        out = fa.launch_dense_ffn_swiglu(fa.MatvecLaunch.of(fo.Q4_K, gate, ffn, hidden // 256 * 144),
                                         fa.MatvecLaunch.of(fo.Q4_K, up, ffn, hidden // 256 * 144),
                                         fa.MatvecLaunch.of(fo.Q6_K, down, hidden, ffn // 256 * 210), x)
        assert np.array_equal(bits(out), bits(y))
    for w in (wg, wu, wd):
        w.release()


# ------------------------------------------------------------------ scratch memory per stream

def test_dev_calls_on_two_streams_from_two_threads(fa):
    """Two threads, each on a stream of its own, enqueue calls of different shapes that all use the
    library's scratch memory (quantized activations, split-K parts, MoE intermediates), a small shape
    first and a larger one after it, so that each stream's buffer is replaced while the other stream is
    busy.  Every result must be the one the same call gives alone, and agree with the oracle."""
    import threading
    import torch
    from frink_amd import synth
    shapes = {"a": (fo.Q4_K, 384, 1024, (40, 130)), "b": (fo.Q6_K, 256, 2048, (48, 200))}
    mats, xs, alone = {}, {}, {}
    for name, (kind, rows, cols, batches) in shapes.items():
        data = make_weights(kind, rows, cols, seed=900 + kind)
        mats[name] = (data, fa.Weights.from_host(kind, data, rows, cols))
        xs[name] = [to_dev(synth.activations(910 + b, b, cols)) for b in batches]
        alone[name] = [mats[name][1].gemm(x).cpu().numpy() for x in xs[name]]
    # a MoE layer on stream "a" as well (its intermediates live in the same scratch buffer)
    E, k, hidden, ffn, batch = 8, 2, 256, 256, 40
    gate, up, down = _stacked_experts(E, hidden, ffn, 930)
    hs = [fa.Weights.from_host(fo.Q4_K, m, r, c) for m, r, c in ((gate, E * ffn, hidden), (up, E * ffn, hidden), (down, E * hidden, ffn))]
    xm = to_dev(synth.activations(931, batch, hidden))
    ids, wts = _route(synth.normal(932, batch * E).reshape(batch, E), k)
    ids_d, wts_d = to_dev(ids.astype(np.int32)), to_dev(wts)
    moe_alone = fa.moe_ffn(hs[0], hs[1], hs[2], E, xm, ids_d, wts_d).cpu().numpy()
    torch.cuda.synchronize()

    results, errors = {}, []

    def work(name):
        try:
            stream = torch.cuda.Stream()  # default priority
            with torch.cuda.stream(stream):
                last = None
                for rep in range(12):
                    outs = [mats[name][1].gemm(x) for x in xs[name]]
                    if name == "a":
                        last = fa.moe_ffn(hs[0], hs[1], hs[2], E, xm, ids_d, wts_d)
                stream.synchronize()
            results[name] = [o.cpu().numpy() for o in outs] + ([last.cpu().numpy()] if last is not None else [])
        except Exception as e:  # noqa: BLE001 - reported in the main thread
            errors.append((name, repr(e)))

    threads = [threading.Thread(target=work, args=(n,)) for n in shapes]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
    assert not errors, errors
    for name, (kind, rows, cols, batches) in shapes.items():
        for got, want_alone, x in zip(results[name], alone[name], xs[name]):
            assert np.array_equal(bits(got), bits(want_alone)), "%s: differs from the same call alone" % name
            assert_rows_close(got, fo.gemm(kind, mats[name][0], rows, cols, x.cpu().numpy()), "two streams, %s" % name)
    assert np.array_equal(bits(results["a"][-1]), bits(moe_alone))
    for _, w in mats.values():
        w.release()
    for h in hs:
        h.release()


@pytest.mark.parametrize("kinds,rows,cols,batch", [
    ((fo.Q4_K, fo.Q4_K), (384, 200), 1024, 130),   # matrix cores, one quantization for both
    ((fo.Q4_K, fo.Q4_K), (96, 256), 2048, 40),     # the blocks split between workgroups: each GEMM its own parts
    ((fo.Q4_K, fo.Q4_K), (64, 64), 512, 8),        # thin kernel
    ((fo.Q4_K, fo.Q6_K), (128, 96), 1024, 64),     # kinds that do not share a quantized form
    ((fo.Q5_K, fo.Q4_K), (200, 136), 1024, 70),    # Q5_K's three planes beside Q4_K's two, one quantization
    ((fo.Q5_K, fo.Q5_K), (96, 160), 2048, 40),     # both with their blocks split
])
def test_gemm_pair_is_two_gemms_over_one_quantization(fa, kinds, rows, cols, batch):
    """frk_hip_gemm_pair_dev (apply_batch_pair_with_acts, weight_matrix.rs:2447-2479): bit for bit the two
    frk_hip_gemm_dev results, and within the tolerance of the oracle."""
    from frink_amd import synth
    datas = [make_weights(k, r, cols, seed=50 + i) for i, (k, r) in enumerate(zip(kinds, rows))]
    ws = [fa.Weights.from_host(k, d, r, cols) for k, d, r in zip(kinds, datas, rows)]
    x = synth.activations(77 + batch, batch, cols, outlier_frac=0.01)
    xd = to_dev(x)
    y0, y1 = fa.gemm_pair(ws[0], ws[1], xd)
    for w, k, d, r, y in zip(ws, kinds, datas, rows, (y0, y1)):
        assert np.array_equal(bits(y.cpu().numpy()), bits(w.gemm(xd).cpu().numpy()))
        assert_rows_close(y.cpu().numpy(), fo.gemm(k, d, r, cols, x), "gemm pair kind %d" % k)
        w.release()


def test_host_entry_points_from_four_threads(fa):
    """frk_hip_launch_matvec / frk_hip_launch_mul_mm called from four threads at once, the way the reference's rayon
    workers call the seam (crates/frink-core/src/weight_matrix/gpu_backend.rs:722-725): different kinds and shapes
    per thread, every result the oracle's."""
    import threading
    from frink_amd import synth
    jobs = []
    for t, (kind, rows, cols, batch) in enumerate(((fo.Q4_K, 200, 1024, 5), (fo.Q6_K, 120, 2048, 3), (fo.Q8_0, 150, 512, 4),
                                                   (fo.Q4_K, 64, 4096, 40))):
        bb, be = fo.BLOCK[kind]
        data = make_weights(kind, rows, cols, seed=1200 + t)
        x = synth.activations(1210 + t, batch, cols)
        mode = fo.F32_DOT if kind == fo.Q8_0 else fo.INT_DOT
        want_v = fo.gemv(kind, data, rows, cols, x[0], mode)
        want_m = fo.gemm(kind, data, rows, cols, x)  # (a Q8_0 batch is the integer path, as in the reference)
        jobs.append((kind, data, x, rows, cols, batch, cols // be * bb, want_v, want_m))
    errors = []

    def work(job):
        kind, data, x, rows, cols, batch, rb, want_v, want_m = job
        try:
            for rep in range(8):
                got = fa.launch_matvec(kind, data, x[0], rows, rb)
                assert_rows_close(got[None], want_v[None], "launch_matvec from a thread, kind %d" % kind)
                got = fa.launch_mul_mm(kind, data, x, rows, cols, batch, rb)
                assert_rows_close(got, want_m, "launch_mul_mm from a thread, kind %d" % kind)
        except Exception as e:  # noqa: BLE001 - reported in the main thread
            errors.append(repr(e))

    threads = [threading.Thread(target=work, args=(j,)) for j in jobs]
    for t in threads:
        t.start()
    for t in threads:
        t.join(180)
    assert not any(t.is_alive() for t in threads), "a thread is still running"
    assert not errors, errors


def test_a_captured_graph_survives_a_larger_call_on_its_stream(fa):
    """A graph captured from a stream replays the address of the stream's scratch buffer.  A larger call on the same
    stream afterwards gets a new buffer; the graph's one must stay allocated and untouched: every replay, with larger
    eager calls on that stream and on another between them, equals the eager result bit for bit."""
    import torch
    from frink_amd import synth
    rows, cols = 384, 1024
    data = make_weights(fo.Q4_K, rows, cols, seed=1301)
    w = fa.Weights.from_host(fo.Q4_K, data, rows, cols)
    big = fa.Weights.from_host(fo.Q4_K, make_weights(fo.Q4_K, 512, 2048, seed=1302), 512, 2048)
    x = to_dev(synth.activations(1303, 40, cols))
    xb = to_dev(synth.activations(1304, 300, 2048))
    stream, other = torch.cuda.Stream(), torch.cuda.Stream()
    with torch.cuda.stream(stream):
        eager = w.gemm(x).clone()          # (sizes the stream's buffer for this shape)
        y = torch.empty_like(eager)
        stream.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=stream):
            w.gemm(x, out=y)
        for rep in range(4):
            y.zero_()
            g.replay()
            stream.synchronize()
            assert np.array_equal(bits(y.cpu().numpy()), bits(eager.cpu().numpy())), rep
            big.gemm(xb)                   # a larger shape on the graph's stream: the buffer is replaced
            with torch.cuda.stream(other):
                big.gemm(xb)               # and one on another stream, which must not be handed the graph's buffer
            other.synchronize()
            stream.synchronize()
    want = fo.gemm(fo.Q4_K, data, rows, cols, x.cpu().numpy())
    assert_rows_close(eager.cpu().numpy(), want, "gemm under a graph")
    w.release()
    big.release()


@pytest.mark.parametrize("kind,rows,cols", [(fo.Q4_K, 384, 1024), (fo.Q6_K, 264, 2048), (fo.Q5_K, 200, 1024)])
def test_batch_acts_quantized_once_feed_any_batch(fa, kind, rows, cols):
    """quantize_batch_acts -> BatchActs::Q8K -> apply_batch_with_acts (weight_matrix.rs:2348-2426, 757-768,
    2481-2487): one quantization of a batch multiplied by several matrices, at every batch size -- one row, the
    thin kernels' batches, the batches where both forms are held, and the wide matrix-core batches.  Each result
    bit for bit frk_hip_gemm_dev's and within the tolerance of the oracle."""
    from frink_amd import synth
    data = make_weights(kind, rows, cols, seed=1400 + kind)
    data2 = make_weights(fo.Q4_K, 136, cols, seed=1410 + kind)
    w, w2 = fa.Weights.from_host(kind, data, rows, cols), fa.Weights.from_host(fo.Q4_K, data2, 136, cols)
    acts = fa.BatchActs(300, cols)
    for batch in (1, 2, 8, 16, 17, 25, 33, 64, 65, 130, 300):
        x = synth.activations(1420 + batch, batch, cols, outlier_frac=0.01)
        xd = to_dev(x)
        acts.quantize(xd)
        for ww, dd, rr, kk in ((w, data, rows, kind), (w2, data2, 136, fo.Q4_K)):
            got = ww.gemm_acts(acts).cpu().numpy()
            ref = ww.gemm(xd).cpu().numpy()
            assert np.array_equal(bits(got), bits(ref)), (batch, kk)
            assert_rows_close(got, fo.gemm(kk, dd, rr, cols, x), "gemm_acts kind %d batch %d" % (kk, batch))
    with pytest.raises(fa.BackendError) as e:
        acts.quantize(to_dev(np.zeros((301, cols), np.float32)))
    assert e.value.code == fa.ERR_SHAPE
    w8 = fa.Weights.from_host(fo.Q8_0, make_weights(fo.Q8_0, 40, cols, seed=3), 40, cols)
    acts.quantize(to_dev(np.zeros((4, cols), np.float32)))
    with pytest.raises(fa.BackendError) as e:
        w8.gemm_acts(acts)
    assert e.value.code == fa.ERR_UNSUPPORTED
    other = fa.Weights.from_host(fo.Q4_K, make_weights(fo.Q4_K, 40, 2 * cols, seed=4), 40, 2 * cols)
    with pytest.raises(fa.BackendError) as e:
        other.gemm_acts(acts)
    assert e.value.code == fa.ERR_SHAPE
    acts.release()
    for h in (w, w2, w8, other):
        h.release()


def test_batch_acts_at_the_prefill_shape(fa):
    """M=512 over 4096 x 4096 Q4_K: the GEMM over held activations equals frk_hip_gemm_dev bit for bit (the kernel
    bench.py times on its own through this entry point)."""
    from bench import random_blocks
    from frink_amd import synth
    rows = cols = 4096
    w = fa.Weights.from_host(fo.Q4_K, random_blocks(fo.Q4_K, rows, cols, 9), rows, cols)
    xd = to_dev(synth.activations(1500, 512, cols, outlier_frac=0.01))
    acts = fa.BatchActs(512, cols).quantize(xd)
    assert np.array_equal(bits(w.gemm_acts(acts).cpu().numpy()), bits(w.gemm(xd).cpu().numpy()))
    acts.release()
    w.release()

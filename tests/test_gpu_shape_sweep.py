"""A seeded walk over shapes nobody picked by hand: every dense entry point against the oracle on random
(kind, rows, columns, batch) combinations -- the row lengths and batch sizes at which the library changes
kernels are all inside the ranges drawn from.  (Two dispatch faults were found this way: a staging loop
sized for another workgroup, and a wait list that named a register twice.)"""
import numpy as np
import pytest

import oracle as fo
from test_gpu_parity import TOL, bits, fa, make_weights, to_dev  # noqa: F401 (fa: the module's fixture)

pytestmark = pytest.mark.gpu

COLS = [256, 512, 768, 1024, 1280, 2048, 2304, 3072, 4096, 4352, 5120, 6144, 7936, 8192, 8448, 11008, 12288, 14336, 16384, 20480]
ROWS = [1, 2, 7, 31, 33, 64, 100, 129, 257, 500, 1030]
BATCHES = [1, 1, 1, 2, 3, 8, 9, 15, 16, 17, 24, 25, 31, 32, 33, 40, 41, 64, 65, 128, 129, 200]


def _close(got, want, rows):
    # of the row's largest output; a lone output has nothing but itself to be measured against
    scale = np.abs(want).max(axis=-1, keepdims=True) if rows > 1 else np.abs(want).max() + 1.0
    return float((np.abs(got - want) / (scale + 1e-30)).max())


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_shapes_against_the_oracle(fa, seed):
    from bench import random_blocks
    from frink_amd import synth
    rng = np.random.default_rng(seed)
    done = 0
    while done < 45:
        kind = [fo.Q4_K, fo.Q5_K, fo.Q6_K, fo.Q8_0, fo.Q4_0][rng.integers(5)]
        cols = COLS[rng.integers(len(COLS))]
        if kind in (fo.Q8_0, fo.Q4_0) and rng.integers(3) == 0:
            cols = int(rng.integers(1, 200)) * 32
        rows, batch = ROWS[rng.integers(len(ROWS))], BATCHES[rng.integers(len(BATCHES))]
        if rows * cols * batch > 4.0e8:
            continue
        what = "kind %d, %d x %d, batch %d" % (kind, rows, cols, batch)
        print(what, flush=True)
        data = (random_blocks(kind, rows, cols, int(rng.integers(1 << 30))) if kind == fo.Q4_0
                else make_weights(kind, rows, cols, seed=int(rng.integers(1 << 30))))
        x = synth.activations(int(rng.integers(1 << 30)), batch, cols, outlier_frac=0.01)
        w = fa.Weights.from_host(kind, data, rows, cols)
        xd = to_dev(x)
        one_f32 = batch == 1 and kind in (fo.Q8_0, fo.Q4_0)  # (their single row is the f32 dot)
        want = fo.gemm(kind, data, rows, cols, x, fo.F32_DOT if one_f32 else fo.INT_DOT)
        got = w.gemm(xd).cpu().numpy()
        assert _close(got, want, rows) <= 2 * TOL, what + ": gemm"
        if batch == 1:
            assert _close(w.gemv(xd[0]).cpu().numpy()[None], want, rows) <= 2 * TOL, what + ": gemv"
        if kind in (fo.Q4_K, fo.Q5_K, fo.Q6_K):
            acts = fa.quantize_q8_k(xd)
            try:
                assert _close(w.gemm_q8k(acts, batch).cpu().numpy(), want, rows) <= 2 * TOL, what + ": gemm_q8k"
            except fa.BackendError as err:  # (a batch the thin kernels do not take)
                assert err.code == fa.ERR_UNSUPPORTED, what
            if batch > 1:
                w2 = fa.Weights.from_host(kind, data, rows, cols)
                y0, y1 = fa.gemm_pair(w, w2, xd)
                assert np.array_equal(bits(y0.cpu().numpy()), bits(got)) and np.array_equal(bits(y1.cpu().numpy()), bits(got)), what + ": pair"
                w2.release()
            elif cols <= 16384:
                f32 = w.gemv(xd[0], act_mode=fa.ACT_F32_DOT).cpu().numpy()[None]
                assert _close(f32, fo.gemm(kind, data, rows, cols, x, fo.F32_DOT), rows) <= 2 * TOL, what + ": f32 dot"
        w.release()
        done += 1

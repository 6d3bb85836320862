"""The entry point that allocates nothing (frk_hip_gemm_noalloc_dev) against frk_hip_gemm_dev: the same
kernels over a fixed scratch array inside the library's device image, so the outputs must be the same
bits -- on two calls in a row, the second with a smaller input (the array keeps the first call's
contents), for every kind and for batch sizes on each side of the dispatch thresholds."""
import numpy as np
import pytest

import oracle as fo

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fa():
    import torch
    assert torch.cuda.is_available(), "these tests need a GPU"
    import frink_amd
    assert frink_amd.probe()["gcn_arch"].startswith("gfx950")
    return frink_amd


def _bits(t):
    return t.cpu().numpy().view(np.uint32)


@pytest.mark.parametrize("kind,rows,cols,batches", [
    (fo.Q4_K, 384, 4096, (512, 40)),    # matrix-core GEMM, then a split one
    (fo.Q4_K, 200, 1024, (16, 3)),      # thin kernel
    (fo.Q6_K, 256, 2048, (130, 48)),    # split Q6_K GEMM both times
    (fo.Q6_K, 96, 1024, (8, 1)),        # thin kernel, then the decode kernel
    (fo.Q8_0, 128, 2048, (64, 2)),
    (fo.Q5_K, 160, 1024, (20, 5)),
    (fo.Q4_0, 64, 512, (33, 7)),
])
def test_gemm_noalloc_gives_the_bits_of_gemm(fa, kind, rows, cols, batches):
    import torch
    from frink_amd import synth
    print("no-alloc", kind, rows, cols, batches, flush=True)
    data = fo.encode_matrix(kind, synth.weights(4000 + kind, rows, cols)) if kind != fo.Q4_0 else \
        np.random.default_rng(5).integers(0, 256, rows * cols // 32 * 18, dtype=np.uint8)
    if kind == fo.Q4_0:
        blocks = data.reshape(-1, 18)
        blocks[:, 0:2] = np.random.default_rng(6).uniform(1e-3, 2e-3, blocks.shape[0]).astype(np.float16).view(np.uint8).reshape(-1, 2)
    w = fa.Weights.from_host(kind, data, rows, cols)
    for batch in batches:  # two calls in a row, the second smaller
        x = torch.from_numpy(synth.activations(4100 + batch, batch, cols)).cuda()
        want = w.gemm(x)
        got = torch.full((batch, rows), float("nan"), dtype=torch.float32, device="cuda")
        w.gemm_noalloc(x, got)
        assert np.array_equal(_bits(got), _bits(want)), (kind, batch)
        ref = fo.gemm(kind, data, rows, cols, x.cpu().numpy(), fo.INT_DOT if (kind not in (fo.Q8_0, fo.Q4_0) or batch > 1) else fo.F32_DOT)
        err = np.abs(got.cpu().numpy() - ref).max(axis=1) / np.abs(ref).max(axis=1)
        assert err.max() <= 1e-3, err.max()
    w.release()


def test_gemm_noalloc_refuses_a_shape_beyond_its_scratch(fa):
    import torch
    from frink_amd import synth
    rows, cols, batch = 64, 16384, 2048  # 2048 x 16384 quantized activations alone are 36 MiB
    w = fa.Weights.from_host(fo.Q4_K, fo.encode_matrix(fo.Q4_K, synth.weights(1, rows, cols)), rows, cols)
    x = torch.zeros((batch, cols), dtype=torch.float32, device="cuda")
    out = torch.zeros((batch, rows), dtype=torch.float32, device="cuda")
    with pytest.raises(fa.BackendError) as e:
        w.gemm_noalloc(x, out)
    assert e.value.code == fa.ERR_SHAPE and "scratch" in e.value.message
    w.release()

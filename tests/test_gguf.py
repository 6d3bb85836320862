"""The GGUF reader (frink_amd/gguf.py) against files written by its own writer and against hand-built
headers: the layout rules and the refusals of crates/frink-gguf/src/lib.rs:429-560."""
import struct

import numpy as np
import pytest

import oracle as fo
from frink_amd import gguf


def _blocks(kind, rows, cols, seed):
    bb, be = fo.BLOCK[kind]
    rng = np.random.default_rng(seed)
    data = rng.integers(0, 256, rows * cols // be * bb, dtype=np.uint8).reshape(-1, bb)
    for off in {fo.Q6_K: (208,), fo.Q4_0: (0,), fo.Q8_0: (0,)}.get(kind, (0, 2)):
        data[:, off:off + 2] = rng.uniform(-0.05, 0.05, data.shape[0]).astype(np.float16).view(np.uint8).reshape(-1, 2)
    return data.ravel()


@pytest.fixture()
def model(tmp_path):
    tensors = [("token_embd.weight", (512, 40), fo.Q6_K, _blocks(fo.Q6_K, 40, 512, 1)),
               ("blk.0.ffn_up.weight", (512, 24), fo.Q4_K, _blocks(fo.Q4_K, 24, 512, 2)),
               ("blk.0.attn_q.weight", (256, 16), fo.Q5_K, _blocks(fo.Q5_K, 16, 256, 3)),
               ("blk.0.attn_norm.weight", (512,), 0, np.arange(512, dtype=np.float32).tobytes()),
               ("output.weight", (64, 10), fo.Q8_0, _blocks(fo.Q8_0, 10, 64, 4))]
    path = tmp_path / "tiny.gguf"
    gguf.write_gguf(path, {"general.architecture": "llama", "llama.block_count": 1, "general.alignment": 64,
                           "llama.rope.freq_base": 10000.0, "flag": True}, tensors, alignment=64)
    return path, tensors


def test_header_metadata_and_tensor_table(model):
    path, tensors = model
    f = gguf.GgufFile(path)
    assert f.version == 3 and f.metadata["general.architecture"] == "llama" and f.metadata["llama.block_count"] == 1
    assert f.metadata["general.alignment"] == 64 and f.data_start % 64 == 0 and f.metadata["flag"] is True
    assert abs(f.metadata["llama.rope.freq_base"] - 10000.0) < 1e-3
    assert [t.name for t in f.tensors] == [t[0] for t in tensors]
    for (name, shape, tag, data), info in zip(tensors, f.tensors):
        assert info.shape == tuple(shape) and info.type_tag == tag and info.offset % 64 == 0
        assert f.tensor_bytes(name).tobytes() == bytes(data)
    assert f.info("token_embd.weight").type_name == "Q6_K" and f.info("token_embd.weight").byte_len == 40 * 2 * 210
    f.close()


def test_refusals(tmp_path, model):
    path, _ = model
    raw = bytearray(open(path, "rb").read())
    def variant(name, edit):
        b = bytearray(raw)
        edit(b)
        p = tmp_path / name
        p.write_bytes(b)
        return p
    with pytest.raises(gguf.GgufError, match="magic"):
        gguf.GgufFile(variant("magic", lambda b: b.__setitem__(slice(0, 4), b"GGML")))
    with pytest.raises(gguf.GgufError, match="version"):
        gguf.GgufFile(variant("version", lambda b: b.__setitem__(slice(4, 8), struct.pack("<I", 1))))
    with pytest.raises(gguf.GgufError, match="left"):
        f = gguf.GgufFile(variant("short", lambda b: b.__delitem__(slice(len(b) - 400, len(b)))))
        f.tensor_bytes("output.weight")
    with pytest.raises(gguf.GgufError, match="power of two"):
        p = tmp_path / "align.gguf"
        gguf.write_gguf(p, {"general.alignment": 48}, [], alignment=48)
        gguf.GgufFile(p)
    with pytest.raises(gguf.GgufError, match="can hold"):
        p = tmp_path / "huge.gguf"
        gguf.write_gguf(p, {}, [("w", (1 << 40, 1 << 20), fo.Q4_K, b"")])
        gguf.GgufFile(p)
    f = gguf.GgufFile(path)
    with pytest.raises(gguf.GgufError, match="no tensor"):
        f.tensor_bytes("missing")
    f.close()


@pytest.mark.gpu
def test_a_checkpoint_feeds_the_kernels(model):
    """Tensors of a GGUF file become resident weights straight from the mapped bytes: the embedding
    gather and a decode GEMV per kind against the oracle on the same bytes."""
    import torch
    import frink_amd as fa
    from frink_amd import synth
    path, tensors = model
    f = gguf.GgufFile(path)
    emb = f.weights("token_embd.weight")
    table = fo.dequant(fo.Q6_K, tensors[0][3]).reshape(40, 512)
    ids = np.array([3, 39, 0, 3], np.int32)
    assert np.array_equal(emb.get_rows(torch.from_numpy(ids).cuda()).cpu().numpy().view(np.uint32), table[ids].view(np.uint32))
    for name, (cols, rows), kind, data in (t for t in tensors if len(t[1]) == 2):
        w = f.weights(name)
        assert (w.rows, w.cols, w.kind) == (rows, cols, kind)
        x = synth.activations(rows, 1, cols)[0]
        got = w.gemv(torch.from_numpy(x).cuda()).cpu().numpy()
        want = fo.gemv(kind, np.frombuffer(bytes(data), np.uint8), rows, cols, x, fo.F32_DOT if kind == fo.Q8_0 else fo.INT_DOT)
        assert np.abs(got - want).max() <= 1e-3 * np.abs(want).max(), name
        w.release()
    with pytest.raises(gguf.GgufError, match="not a matrix"):
        f.weights("blk.0.attn_norm.weight")
    emb.release()
    f.close()


# ---------------------------------------------------------------- files the reader did not write
# Three of the reference's own test files (crates/frink-models/tests/fixtures/), copied as data: a
# dense two-layer model, its second split, and a four-expert MoE model, all with Q8_0 matrices.  What
# is asserted about them is what the reference's tests assert (crates/frink-models/tests/gguf_roundtrip.rs:
# 70-85 tensor count and kinds, :120-135 the packed expert tensor's raw shape) plus the layout rules of
# crates/frink-gguf/src/lib.rs:429-560 (alignment, offsets in order, byte lengths).
import os

GOLDEN_GGUF = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gguf")


def _open(name):
    return gguf.GgufFile(os.path.join(GOLDEN_GGUF, name))


def test_reference_dense_file_tensor_table():
    f = _open("frink_real_test.gguf")
    assert f.version == 3 and f.metadata["general.architecture"] == "ferroxtest" and f.metadata["general.alignment"] == 32
    # 1 embedding + 2 layers * (1 attn_norm + 4 attn + 1 ffn_norm + 3 ffn) + output_norm + output
    assert len(f.tensors) == 1 + 2 * 9 + 2
    assert sum(t.type_name == "Q8_0" for t in f.tensors) == 2 * 7
    assert f.data_start % 32 == 0 and f.data_start == 2048
    end = 0
    for t in f.tensors:
        assert t.offset % 32 == 0 and t.offset >= end
        n = int(np.prod(t.shape))
        assert t.byte_len == (n // 32 * 34 if t.type_name == "Q8_0" else n * 4)
        end = t.offset + t.byte_len
    assert f.data_start + end == os.path.getsize(os.path.join(GOLDEN_GGUF, "frink_real_test.gguf"))
    q = f.info("blk.0.attn_k.weight")
    assert q.shape == (32, 16) and q.type_tag == fo.Q8_0 and q.byte_len == 16 * 34  # 16 rows of one block
    # rms_norm epsilon is stored as an f32
    assert abs(f.metadata["ferroxtest.attention.layer_norm_rms_epsilon"] - 1e-5) < 1e-11
    f.close()


def test_reference_split_file_defaults_and_shares_its_tensors_bytes():
    whole, part = _open("frink_real_test.gguf"), _open("frink_real_test_split-00002-of-00003.gguf")
    assert "general.alignment" not in part.metadata and part.data_start % 32 == 0  # the default alignment
    assert part.metadata["split.no"] == 1 and part.metadata["split.count"] == 3 and part.metadata["split.tensors.count"] == 21
    assert [t.name for t in part.tensors] == [t.name for t in whole.tensors[:10]]
    for t in part.tensors:
        assert part.tensor_bytes(t.name).tobytes() == whole.tensor_bytes(t.name).tobytes()
    whole.close(), part.close()


def test_reference_moe_file_packed_expert_tensors():
    f = _open("frink_real_moe_test.gguf")
    g = f.info("blk.0.ffn_gate_exps.weight")
    assert g.shape == (32, 32, 4) and g.type_name == "Q8_0" and g.byte_len == 4 * 32 * 34  # [hidden, ffn, experts]
    assert f.info("blk.0.ffn_gate_inp.weight").shape == (32, 4) and f.metadata["ferroxtestmoe.expert_used_count"] == 2
    assert len(f.tensors) == 29 and sum(t.type_name == "Q8_0" for t in f.tensors) == 20
    f.close()


def test_reference_file_q8_0_bytes_dequantize_to_model_sized_weights():
    # the file's matrices were quantized from small random weights: every block's scale is a finite f16 and the
    # dequantized rows are what the index formula d * q gives (dequant_q8_0, crates/frink-quant/src/lib.rs:83-103)
    f = _open("frink_real_test.gguf")
    raw = np.frombuffer(f.tensor_bytes("blk.1.ffn_down.weight").tobytes(), np.uint8).reshape(32, 34)
    d = raw[:, :2].copy().view(np.float16).astype(np.float32).ravel()
    q = raw[:, 2:].copy().view(np.int8).astype(np.float32)
    want = d[:, None] * q
    got = fo.dequant(fo.Q8_0, raw.ravel()).reshape(32, 32)
    assert np.isfinite(d).all() and (d > 0).all() and np.array_equal(got, want) and 0.01 < np.abs(got).max() < 10
    f.close()


@pytest.mark.gpu
def test_reference_file_tensors_through_the_device():
    """A Q8_0 matrix straight from the reference's file: resident on the GPU, rows fetched back with
    get_rows bit for bit, and the matrix of packed experts read as 4 x 32 rows."""
    import torch
    import frink_amd as fa
    f = _open("frink_real_moe_test.gguf")
    for name, rows, cols in (("blk.0.attn_q.weight", 32, 32), ("blk.0.attn_k.weight", 16, 32),
                             ("blk.1.ffn_down_exps.weight", 4 * 32, 32)):
        raw = np.frombuffer(f.tensor_bytes(name).tobytes(), np.uint8)
        w = fa.Weights.from_host(fa.Q8_0, raw, rows, cols)
        ids = np.array([rows - 1, 0, 5, 5, rows // 2], np.int32)
        got = w.get_rows(torch.from_numpy(ids).cuda()).cpu().numpy()
        want = fo.dequant(fo.Q8_0, raw).reshape(rows, cols)[ids]
        assert np.array_equal(got, want), name
        w.release()
    f.close()

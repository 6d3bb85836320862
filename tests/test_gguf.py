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

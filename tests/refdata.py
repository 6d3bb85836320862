"""Input generators the reference's own tests use, restated so the golden
bytes can be checked against the inputs they were produced from."""
import numpy as np


def _xorshift32_stream(seed, n):
    """xorshift32 (13, 17, 5), mapped to [-1, 1) with 24 bits:
    ((state >> 8) as f32 / 8388608) - 1."""
    out = np.empty(n, np.float32)
    s = seed & 0xFFFFFFFF
    for i in range(n):
        s ^= (s << 13) & 0xFFFFFFFF
        s ^= s >> 17
        s ^= (s << 5) & 0xFFFFFFFF
        out[i] = np.float32(np.float32(s >> 8) / np.float32(8388608.0)) - np.float32(1.0)
    return out


def q8_0_sample_input(n):
    """crates/frink-quant/src/encode.rs:138-149 (seed 0x12345678)."""
    return _xorshift32_stream(0x12345678, n)


def k_quant_fixture(real_weight_blocks_f16_bits):
    """crates/frink-quant/src/encode/testdata.rs:90-119: four synthetic f16-shaped
    super-blocks (seed 0xb54cda26, special sub-blocks 8/9/10/11/17) followed by
    eight real-weight super-blocks given as f16 bit patterns."""
    gains = [np.float32(0.02), np.float32(0.05), np.float32(0.1), np.float32(0.25)]
    stream = _xorshift32_stream(0xB54CDA26, 4 * 8 * 32)
    out = []
    idx = 0
    for sub in range(32):
        for _ in range(32):
            v = stream[idx]
            idx += 1
            if sub == 8:
                shaped = np.float32(0.0)
            elif sub == 9:
                shaped = np.float32(0.125)
            elif sub == 10:
                shaped = np.float32(abs(v) * np.float32(0.05)) + np.float32(0.01)
            elif sub == 11:
                shaped = -(np.float32(abs(v) * np.float32(0.05)) + np.float32(0.01))
            elif sub == 17:
                shaped = v * np.float32(1e-4)
            else:
                shaped = v * gains[sub % 4]
            out.append(np.float32(np.float16(np.float32(shaped))))
    syn = np.array(out, np.float32)
    real = np.array(real_weight_blocks_f16_bits, np.uint16).view(np.float16).astype(np.float32)
    return np.concatenate([syn, real])

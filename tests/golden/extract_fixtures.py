#!/usr/bin/env python3
"""Extract the reference's own golden vectors for the quantized-matmul path.

Reads the reference's Rust test modules AS TEXT (nothing is compiled, imported
or executed) and copies the literal arrays they hold -- block bytes, f16 bit
patterns, expected f32 values -- into ``frink_quant_vectors.json`` beside this
script.  Only data is extracted; no reference code is kept.

Run once in a container that has the reference checked out:

    python tests/golden/extract_fixtures.py [/root/reference]

Sources (paths relative to the reference root):

* crates/frink-quant/src/encode.rs            Q8_0 encoder goldens, tie block
* crates/frink-quant/src/encode/q4_k.rs       llama.cpp Q4_K bytes for the k-quant fixture
* crates/frink-quant/src/encode/q5_k.rs       llama.cpp Q5_K bytes for the k-quant fixture
* crates/frink-quant/src/encode/q6_k.rs       llama.cpp Q6_K bytes for the k-quant fixture
* crates/frink-quant/src/encode/testdata.rs   8 real-weight super-blocks (f16 bits)
* crates/frink-quant/src/lib.rs               Q4_K / Q5_K / Q6_K dequant test blocks + goldens;
                                              IQ4_XS and MXFP4 (GGUF block form and two-buffer form) test
                                              blocks + goldens
"""
import json
import os
import re
import sys

ROOT = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
QUANT = os.path.join(ROOT, "crates", "frink-quant", "src")


def array_body(text, name):
    """Return the text between '[' and '];' of `const NAME: ... = [ ... ];`
    (or `= &[ ... ];`)."""
    m = re.search(r"const\s+" + re.escape(name) + r"\s*:[^=]*=\s*&?\[", text)
    if not m:
        raise KeyError(name)
    start = m.end()
    end = text.index("];", start)
    body = text[start:end]
    # strip // comments
    body = re.sub(r"//[^\n]*", "", body)
    return body


def ints(text, name):
    return [int(tok, 0) for tok in re.findall(r"0x[0-9a-fA-F]+|\b\d+\b", array_body(text, name))]


def floats(text, name):
    return [float(tok) for tok in re.findall(r"-?\d+\.?\d*(?:[eE][-+]?\d+)?", array_body(text, name))]


def main():
    out = {}
    enc = open(os.path.join(QUANT, "encode.rs")).read()
    out["q8_0_encode_golden"] = bytes(ints(enc, "LLAMA_CPP_Q8_0_GOLDEN")).hex()
    out["q8_0_tie_block_f16_bits"] = ints(enc, "TIE_BLOCK_F16_BITS")
    out["q8_0_tie_block_golden"] = bytes(ints(enc, "LLAMA_CPP_TIE_BLOCK_GOLDEN")).hex()

    q4 = open(os.path.join(QUANT, "encode", "q4_k.rs")).read()
    out["q4_k_encode_golden"] = bytes(ints(q4, "LLAMA_CPP_Q4_K_GOLDEN")).hex()
    q5 = open(os.path.join(QUANT, "encode", "q5_k.rs")).read()
    out["q5_k_encode_golden"] = bytes(ints(q5, "LLAMA_CPP_Q5_K_GOLDEN")).hex()
    q6 = open(os.path.join(QUANT, "encode", "q6_k.rs")).read()
    out["q6_k_encode_golden"] = bytes(ints(q6, "LLAMA_CPP_Q6_K_GOLDEN")).hex()

    td = open(os.path.join(QUANT, "encode", "testdata.rs")).read()
    out["real_weight_blocks_f16_bits"] = ints(td, "REAL_WEIGHT_BLOCKS")

    lib = open(os.path.join(QUANT, "lib.rs")).read()
    for blk, gold in [
        ("Q4_K_TEST_BLOCK", "Q4_K_GOLDEN"),
        ("Q5_K_TEST_BLOCK", "Q5_K_GOLDEN"),
        ("Q6_K_TEST_BLOCK", "Q6_K_GOLDEN"),
        ("Q6_K_SIGNED_SCALES_TEST_BLOCK", "Q6_K_SIGNED_SCALES_GOLDEN"),
        ("Q6_K_SIGNED_TEST_BLOCK", "Q6_K_SIGNED_GOLDEN"),
    ]:
        out[blk.lower()] = bytes(ints(lib, blk)).hex()
        out[gold.lower()] = floats(lib, gold)

    for blk, gold in [("IQ4_XS_TEST_BLOCK", "IQ4_XS_GOLDEN"), ("MXFP4_GGUF_TEST_BLOCKS", "MXFP4_GGUF_GOLDEN")]:
        out[blk.lower()] = bytes(ints(lib, blk)).hex()
        out[gold.lower()] = floats(lib, gold)
    out["mxfp4_test_packed"] = bytes(ints(lib, "MXFP4_TEST_PACKED")).hex()
    out["mxfp4_test_scales"] = bytes(ints(lib, "MXFP4_TEST_SCALES")).hex()
    out["mxfp4_golden"] = floats(lib, "MXFP4_GOLDEN")

    sizes = {
        "iq4_xs_test_block": 136, "iq4_xs_golden": 256, "mxfp4_gguf_test_blocks": 68, "mxfp4_gguf_golden": 128,
        "mxfp4_test_packed": 32, "mxfp4_test_scales": 2, "mxfp4_golden": 64,
        "q8_0_encode_golden": 2 * 34, "q8_0_tie_block_f16_bits": 32, "q8_0_tie_block_golden": 34,
        "q4_k_encode_golden": 12 * 144, "q5_k_encode_golden": 12 * 176, "q6_k_encode_golden": 12 * 210,
        "real_weight_blocks_f16_bits": 8 * 256,
        "q4_k_test_block": 144, "q4_k_golden": 256,
        "q6_k_test_block": 210, "q6_k_golden": 256,
        "q6_k_signed_scales_test_block": 210, "q6_k_signed_scales_golden": 256,
        "q6_k_signed_test_block": 210, "q6_k_signed_golden": 256,
    }
    for k, n in sizes.items():
        v = out[k]
        got = len(v) // 2 if isinstance(v, str) else len(v)
        assert got == n, (k, got, n)

    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "frink_quant_vectors.json")
    with open(dst, "w") as f:
        json.dump(out, f, indent=0, separators=(",", ":"))
    print("wrote", dst, os.path.getsize(dst), "bytes")


if __name__ == "__main__":
    main()

"""Writes golden input/output vectors by running the reference's own pure-torch helpers.

Run in the build container only (the reference checkout does not travel to the GPU box):

    python tests/golden/make_vectors.py [/root/reference]

It imports ``examples/dequantize_gemm/dequantize_utils.py`` (which imports only torch) and loads
``examples/dequantize_gemm/quantize/utils.py`` by file path (its package ``__init__`` pulls in the compiler and is
bypassed), calls four functions on fixed inputs and stores inputs and outputs in ``reference_vectors.npz`` next
to this script.  ``tests/test_oracle_pins.py`` loads that file and checks the oracle against every vector.  Nothing
of the reference's source is stored, only data.

Vectors:
* ``torch_convert``            every byte value (256) -> two bf16 bit patterns each
* ``torch_convert_bit_twiddling``  every 16-bit unit (65 536 byte pairs) -> four bf16 bit patterns each
* ``interleave_weight``        4096 int32 words drawn with seed 0, for every (nbits, target) the function handles
* ``general_compress``         a seeded matrix of codes for source_bits 1, 2 and 4
"""

import importlib.util
import os
import sys

import numpy as np
import torch


def _load(path, name):
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    here = os.path.dirname(os.path.abspath(__file__))
    dq = _load(os.path.join(ref, "examples", "dequantize_gemm", "dequantize_utils.py"), "ref_dequantize_utils")
    qu = _load(os.path.join(ref, "examples", "dequantize_gemm", "quantize", "utils.py"), "ref_quantize_utils")
    out = {}

    all_bytes = torch.arange(256, dtype=torch.int32).to(torch.uint8).reshape(1, 256)
    out["convert_in"] = all_bytes.numpy()
    out["convert_out_bits"] = dq.torch_convert(all_bytes).view(torch.int16).numpy().view(np.uint16)
    # with the block exponent of the scaled form: one scale per 32 outputs, values that reach the clamp at 255
    scale = torch.tensor([[0, 1, 7, 100, 125, 126, 127, 128, 200, 252, 253, 254, 255, 3, 2, 1]], dtype=torch.uint8)
    out["convert_scale"] = scale.numpy()
    out["convert_scaled_out_bits"] = dq.torch_convert(all_bytes, 32, scale).view(torch.int16).numpy().view(np.uint16)

    units = torch.arange(65536, dtype=torch.int32)
    pairs = torch.stack(((units >> 8) & 0xFF, units & 0xFF), dim=-1).to(torch.uint8).reshape(256, 512)  # byte 2j = high
    out["twiddling_in"] = pairs.numpy()
    out["twiddling_out_bits"] = dq.torch_convert_bit_twiddling(pairs).view(torch.int16).numpy().view(np.uint16)

    rng = np.random.default_rng(0)
    words = rng.integers(-(2 ** 31), 2 ** 31, size=(64, 64), dtype=np.int64).astype(np.int32)
    out["interleave_in"] = words
    # the byte-shuffle branches of the function ((2, float16), (1, float16), (1, int8)) call `torch.int32(...)`, which
    # raises TypeError in torch: the reference's own function cannot produce vectors for them
    raised = []
    for nbits, target in ((4, "float16"), (2, "float16"), (1, "float16"), (4, "int8"), (2, "int8"), (1, "int8")):
        q = torch.from_numpy(words.copy()).view(torch.int8)
        try:
            out[f"interleave_{nbits}_{target}"] = qu.interleave_weight(q, nbits, target).contiguous().numpy().view(np.int32)
        except TypeError as exc:
            raised.append(f"({nbits}, {target}): {exc}")
    out["interleave_cases_the_reference_raises_on"] = np.array(raised)

    for bits in (1, 2, 4):
        codes = rng.integers(0, 1 << bits, size=(8, 128), dtype=np.int64).astype(np.int8)
        out[f"compress_in_{bits}"] = codes
        out[f"compress_out_{bits}"] = qu.general_compress(torch.from_numpy(codes.copy()), source_bits=bits).numpy()

    path = os.path.join(here, "reference_vectors.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path}: " + ", ".join(f"{k}{list(v.shape)}" for k, v in out.items()))


if __name__ == "__main__":
    main()

"""Writes tests/golden/kv_golden.npz: small input/expected-output vectors for the quantize-pack
and decode path, produced by the CPU oracle of this repository (oracle/bitdecode_oracle.py).

The reference holds no fixtures for this path (its .gitignore excludes *.npy / *.pt and its
tests only print an error), and it cannot be built or imported in this image, so these
vectors pin the oracle's behaviour over time and give the GPU tests data that does not
depend on the oracle being importable.  Run from the repository root:

    python tests/golden/make_golden.py
"""
import math
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import bitdecode_oracle as O  # noqa: E402
from tests import helpers as H            # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kv_golden.npz")
B, H_Q, H_K, S, R = 1, 4, 2, 256, 48
CASES = [(4, 128), (4, 64), (4, 32), (2, 128), (2, 64), (2, 32)]


def main():
    q, k, v = O.make_inputs(B, H_Q, H_K, S, R, seed=2024)
    # edge groups: a constant K group, a constant V group, exact .5 ties, a large-range channel
    k[0, :32, 0, 11] = 0.625
    v[0, 17, 1, 32:64] = -1.25
    k[0, 128:160, 1, 5] = np.arange(32, dtype=np.float32) * np.float32(0.5)
    k[0, :, 0, 99] *= np.float32(30)
    k, v = O.round_to_storage(k, "fp16"), O.round_to_storage(v, "fp16")
    scale = 1.0 / math.sqrt(128)
    data = {
        "q": H.bits16(q, "fp16"), "k": H.bits16(k, "fp16"), "v": H.bits16(v, "fp16"),
        "softmax_scale": np.float32(scale), "packed_tokens": np.int32(S), "residual_tokens": np.int32(R),
    }
    for bits, gs in CASES:
        qkv = O.quantize_kv_ref(k[:, :S], v[:, :S], bits, gs)
        tag = f"b{bits}g{gs}"
        phys = H.oracle_physical(qkv)
        for name, arr in zip(("k_pack", "k_params", "v_pack", "v_params"), phys):
            data[f"{tag}_{name}"] = arr
        data[f"{tag}_k_codes"] = qkv.k_codes
        data[f"{tag}_v_codes"] = qkv.v_codes
        data[f"{tag}_k_scale"] = H.bits16(qkv.k_scale, "fp16")
        data[f"{tag}_k_zero"] = H.bits16(qkv.k_zero, "fp16")
        data[f"{tag}_v_scale"] = H.bits16(qkv.v_scale, "fp16")
        data[f"{tag}_v_zero"] = H.bits16(qkv.v_zero, "fp16")
        k_hat, v_hat = O.dequantize_ref(qkv)
        out, lse = O.attend_ref(q, k_hat, v_hat, scale, k[:, S:], v[:, S:])
        data[f"{tag}_out"] = out
        data[f"{tag}_lse"] = lse
    np.savez_compressed(OUT, **data)
    print(f"wrote {OUT} ({os.path.getsize(OUT) / 1024:.0f} KiB)")


if __name__ == "__main__":
    main()

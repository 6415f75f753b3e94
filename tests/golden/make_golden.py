"""Regenerate tests/golden/golden.json from the REAL upstream library.

Run in a container where the upstream sources are mounted and `make -C oracle ref` has
produced oracle/_ref/libxnor_nn_ref.so:

    python tests/golden/make_golden.py

For every case the upstream bcast path is driven through its public C API on inputs from
xnor_nn_amd.synth (bit-reproducible), and the SHA-256 of each tensor it produced is stored
together with a few sampled raw values.  The packed tensors are hashed in the upstream
CPU layout for a 256-bit host (16 filters per block with int16 words, 8 with int32).
Cases whose output-channel count the upstream bcast path cannot take (oc % 16 != 0, where
it silently runs its float algorithm instead) only record a, k, alpha and dst.
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import checkers  # noqa: E402
import shapes  # noqa: E402
from xnor_nn_amd import synth  # noqa: E402

KEYS = ("bin_src", "bin_weights", "a", "k", "alpha", "opc", "dst")


def digest(arr):
    return hashlib.sha256(np.ascontiguousarray(arr).tobytes()).hexdigest()


def samples(arr, n=8):
    flat = np.ascontiguousarray(arr).ravel()
    idx = np.linspace(0, flat.size - 1, n).astype(np.int64)
    vals = flat[idx]
    if flat.dtype == np.float32:
        vals = vals.view(np.uint32)
    return {"index": idx.tolist(), "bits": [int(v) for v in vals]}


def record(ref, dims, x, w):
    out = ref.forward(dims, x, w)
    keys = KEYS if out.get("bcast_applicable") else ("a", "k", "alpha", "dst")
    return {"dims": dims, "sha256": {k: digest(out[k]) for k in keys},
            "samples": {k: samples(out[k]) for k in keys}}


def main():
    ref = checkers.RefLib()
    golden = {"workloads": {}, "reference_test_shapes": {}}
    for name in synth.WORKLOADS:
        dims, x, w = synth.make_workload(name)
        dims = {k: v for k, v in dims.items() if k not in ("src", "wsigma")}
        golden["workloads"][name] = record(ref, dims, x, w)
        print(name, "done", flush=True)
    for t in shapes.COMPARE_WITH_REFERENCE:
        d = shapes.as_dims(t)
        x = synth.reference_test_src(d["mb"], d["ic"], d["ih"], d["iw"])
        w = synth.reference_test_weights(d["oc"], d["ic"], d["kh"], d["kw"])
        golden["reference_test_shapes"][shapes.shape_id(t)] = record(ref, d, x, w)
    # one tiny case stored in full: inputs and every output, as plain numbers
    dims = dict(mb=1, ic=5, oc=16, ih=4, iw=3, kh=3, kw=3, sh=1, sw=1, ph=1, pw=1)
    x = synth.normal(7, 1 * 5 * 4 * 3).reshape(1, 5, 4, 3)
    w = synth.normal(8, 16 * 5 * 3 * 3, 0.05).reshape(16, 5, 3, 3)
    out = ref.forward(dims, x, w)
    golden["tiny_full"] = {
        "dims": dims,
        "src_bits": x.view(np.uint32).ravel().tolist(),
        "weights_bits": w.view(np.uint32).ravel().tolist(),
        "bin_src": out["bin_src"].tolist(),
        "bin_weights": out["bin_weights"].tolist(),
        "a_bits": out["a"].view(np.uint32).ravel().tolist(),
        "k_bits": out["k"].view(np.uint32).ravel().tolist(),
        "alpha_bits": out["alpha"].view(np.uint32).ravel().tolist(),
        "opc": out["opc"].ravel().tolist(),
        "dst_bits": out["dst"].view(np.uint32).ravel().tolist(),
    }
    with open(os.path.join(HERE, "golden.json"), "w") as f:
        json.dump(golden, f, indent=0, sort_keys=True)
    print("wrote golden.json")


if __name__ == "__main__":
    main()

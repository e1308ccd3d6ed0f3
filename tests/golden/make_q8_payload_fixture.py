"""Writes tests/golden/q8_payload.npz: seeded fp32 weight matrices and the record bytes the
reference's own per-row int8 weight quantizer makes of them.

The quantizer is `q8_payload` (compiler/compile_minimindo_sensevoice_image.py:38-46): Python
on torch, with nothing in the reference's tests or C sources that fixes its rounding
(float32 row divided by a Python double, torch.round, the double scale packed as "<f").  No
closed form or other fixture pins those choices, so this script imports that one function from
the reference tree and records what it returns.

THIS SCRIPT EXECUTES REFERENCE CODE: importing the packer module runs that file's top-level
statements and its imports (torch among them).  Run it only in the sandboxed build container,
where the reference tree lives and nothing of value is within reach; never on a workstation
or the GPU box.  The tests read the committed .npz (numpy.load, allow_pickle=False) and never
the reference.

    python tests/golden/make_q8_payload_fixture.py
"""
import importlib.util
import sys
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
REFERENCE = Path("/root/reference/compiler/compile_minimindo_sensevoice_image.py")


def reference_q8_payload():
    spec = importlib.util.spec_from_file_location("reference_sensevoice_packer", REFERENCE)
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)  # defines functions only; its main() runs under __main__
    return module.q8_payload


def near_ties(rng, K):
    """A row whose quotients w/scale sit on and one float32 step either side of k + 0.5."""
    row = np.zeros(K, dtype=np.float32)
    row[0] = np.float32(1.27)  # the row maximum: scale = 0.01 (as a double, then as float32)
    scale32 = np.float32(np.float64(row[0]) / 127.0)
    targets = rng.integers(-126, 126, size=(K - 1) // 3 + 1).astype(np.float32) + np.float32(0.5)
    values = []
    for t in targets:
        centre = np.float32(t * scale32)
        values += [np.nextafter(centre, np.float32(-np.inf)), centre, np.nextafter(centre, np.float32(np.inf))]
    row[1:] = np.asarray(values[:K - 1], dtype=np.float32)
    return row


def main():
    import torch

    q8_payload = reference_q8_payload()
    rng = np.random.default_rng(20250103)
    cases = {}
    # N(0, 0.02) weights of the benchmark's kind, with an all-zero row and a constant row
    w = (rng.standard_normal((24, 160)) * 0.02).astype(np.float32)
    w[5] = 0.0
    w[6] = np.float32(-0.03125)
    cases["normal"] = w
    # rows built to land on rounding ties and one step beside them
    cases["ties"] = np.stack([near_ties(rng, 96) for _ in range(6)])
    # exact halves: maximum 127 makes the scale exactly 1
    halves = np.zeros((2, 32), dtype=np.float32)
    halves[0, :10] = [127.0, 0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5, 126.5, -126.5]
    halves[1, :6] = [-127.0, 125.5, -125.5, 64.5, 63.5, 1e-3]
    cases["halves"] = halves
    # wide dynamic range: tiny and huge row maxima, subnormal entries
    wide = (rng.standard_normal((8, 64))).astype(np.float32)
    wide *= np.float32(10.0) ** rng.integers(-30, 30, size=(8, 1)).astype(np.float32)
    wide[7, :4] = [1e-40, -1e-40, 3e-39, 0.0]
    cases["wide"] = wide
    out = {}
    for name, weights in cases.items():
        payload = q8_payload(torch.from_numpy(weights.copy()))
        records = np.frombuffer(payload, dtype=np.uint8)
        assert records.size == weights.shape[0] * (4 + weights.shape[1])
        out[f"{name}_w"] = weights
        out[f"{name}_records"] = records.copy()
    np.savez_compressed(HERE / "q8_payload.npz", **out)
    print("wrote", HERE / "q8_payload.npz", {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    sys.exit(main())

"""Writes the golden fixtures of tests/golden/ with the REFERENCE's own CPU prepacker.

Run in the build container only (it needs /root/reference to have been compiled into oracle/_ref by `make -C oracle`):

    python tests/golden/make_golden.py

What it writes
  prepack_<fmt>_<OC>x<IC>.npz : raw int32 weights (deterministic codes) and the bytes the reference's
                                weight_matrix_prepacking_fp_eXmY (utils/weight_prepacking.h:204-211) produced for them;
                                for e2m3 and e2m1, which that dispatcher does not admit, the bytes of the template it
                                dispatches to (weight_matrix_prepacking_x_bit, :118-196) instantiated for that (E, M).
  prepack_hashes.json         : SHA-256 of raw and reference-prepacked buffers at benchmark sizes
                                (config 1: 256x1024, config 2: 4096x4096), whose inputs any machine regenerates from
                                fp6_llm_amd.synth.uniform_codes(seed, ...).
The reference's dequantizer cannot be built in this image (its <cuda_fp16.h> needs <nv/target>), so there are no dequant
fixtures from it; the known answers that pin the dequantizer are the constants quoted in tests/test_oracle.py.
"""
import hashlib
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from fp6_llm_amd import quant, synth  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
FMT = {"e3m2": (3, 2), "e2m2": (2, 2), "e2m3": (2, 3), "e2m1": (2, 1)}


def main():
    if oracle.ref_lib() is None:
        raise SystemExit("oracle/_ref is not built: run `make -C oracle` where /root/reference exists")
    for name, (E, M) in FMT.items():
        for OC, IC, seed in ((64, 64, 101), (128, 192, 102), (256, 64, 103)):
            raw = quant.pack_raw(synth.uniform_codes(seed, OC, IC, E, M), E, M)
            packed = oracle.ref_prepack(raw, E, M)
            np.savez_compressed(os.path.join(HERE, "prepack_%s_%dx%d.npz" % (name, OC, IC)), raw=raw,
                                packed=packed.view(np.int32), seed=seed)
    hashes = {}
    for name, (E, M) in FMT.items():
        for OC, IC, seed in ((256, 1024, 1001), (4096, 4096, 2001)):
            raw = quant.pack_raw(synth.uniform_codes(seed, OC, IC, E, M), E, M)
            packed = oracle.ref_prepack(raw, E, M)
            hashes["%s_%dx%d_seed%d" % (name, OC, IC, seed)] = {
                "raw_sha256": hashlib.sha256(raw.tobytes()).hexdigest(),
                "packed_sha256": hashlib.sha256(packed.tobytes()).hexdigest(),
            }
    with open(os.path.join(HERE, "prepack_hashes.json"), "w") as f:
        json.dump(hashes, f, indent=1, sort_keys=True)
    print("wrote fixtures to", HERE)


if __name__ == "__main__":
    main()

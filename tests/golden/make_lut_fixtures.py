"""Write tests/golden/lut_fixtures.json from the reference checkout.

Run once in the build container (needs /root/reference; never on the GPU box):

    python tests/golden/make_lut_fixtures.py

Only the three load-time functions whose exact outputs depend on search /
iteration details are recorded, for bit widths 1, 2 and 4:

* get_codebook           (turboquant_utils/codebook.py:77-100)  -> fp16 centroids, fp32 boundaries
* build_fp8_codebook     (turboquant_utils/triton_kernels_fp8.py:35-87)  -> e4m3 bytes, scale
* build_e2m1_codebook    (turboquant_utils/triton_kernels_fp4.py:32-77)  -> nibbles, E0, residual
* build_int8_codebook    (turboquant_utils/triton_kernels_a8.py:526-550) -> int8 codes, step

The file holds inputs/outputs only (a few hundred bytes per entry).
"""

import json
import os
import sys

import torch

REF = os.environ.get("DARTMOQ_REFERENCE", "/root/reference")
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lut_fixtures.json")


def main():
    sys.path.insert(0, REF)
    from turboquant_utils.codebook import get_codebook
    from turboquant_utils.triton_kernels_a8 import build_int8_codebook
    from turboquant_utils.triton_kernels_fp8 import build_fp8_codebook
    from turboquant_utils.triton_kernels_fp4 import build_e2m1_codebook

    rec = {}
    for bit in (1, 2, 4):
        cents, bounds = get_codebook(bit)
        cb16 = cents.half()
        i8, step = build_int8_codebook(cb16)
        f8, f8_scale = build_fp8_codebook(cb16)
        nib, e0, resid, err = build_e2m1_codebook(cb16)
        rec[str(bit)] = {
            "codebook_fp16_bits": cb16.view(torch.int16).tolist(),
            "boundaries_fp32": [float(v) for v in bounds.tolist()],
            "int8": i8.tolist(), "int8_step": float(step),
            "e4m3_bytes": f8.view(torch.uint8).tolist(), "e4m3_scale": float(f8_scale),
            "e2m1_nib": nib.tolist(), "e2m1_e0": int(e0), "e2m1_residual": float(resid),
            "e2m1_relerr": float(err),
        }
    with open(OUT, "w") as fh:
        json.dump(rec, fh, indent=1)
    print("wrote", OUT)


if __name__ == "__main__":
    main()

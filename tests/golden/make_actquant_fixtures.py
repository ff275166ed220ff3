"""Write tests/golden/actquant_fixtures.json from the reference checkout.

Run once in the build container (needs /root/reference; never on the GPU box):

    python tests/golden/make_actquant_fixtures.py

Records what the reference's own torch code returns on small seeded inputs for

* quantize_act_per_token_group      (turboquant_utils/triton_kernels_a8.py:384-423)
* quantize_act_per_token_group_fp8  (turboquant_utils/triton_kernels_fp8.py:94-125)
* quantize_act_e2m1_per32           (turboquant_utils/triton_kernels_fp4.py:125-151)
* _build_merged_block_info          (turboquant_utils/triton_kernels_a8.py:938-956)

The inputs include rounding ties (values exactly between two codes), an all-zero group (the
scale floor), tiny groups below the floor and groups whose largest value is a power of two.
The file holds inputs (fp32 bit patterns) and outputs only.
"""

import json
import os
import sys

import torch

REF = os.environ.get("DARTMOQ_REFERENCE", "/root/reference")
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "actquant_fixtures.json")
E2M1_GRID = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)


def inputs(seed, rows, k):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, k, generator=g)
    x[0, :128] = 0.0                                         # scale floor
    x[0, 128:256] = torch.randn(128, generator=g) * 1e-10   # below the floor
    # int8 ties: the largest value 127 makes the scale exactly 1, the rest sit on k + 0.5
    x[1, :128] = (torch.arange(128) - 64).float() + 0.5
    x[1, 0] = 127.0
    # e4m3 ties: largest value 448 (scale 1), values halfway between neighbouring e4m3 codes
    x[1, 128:256] = torch.tensor([17.0, 19.0, 21.0, 23.0, 25.0, 27.0, 29.0, 31.0] * 16) * \
        torch.tensor([1.0, -1.0] * 64)
    x[1, 128] = 448.0
    # e2m1 ties: largest value 6 in each block of 32 (scale 1), the midpoints of the grid
    mids = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, -0.25, -0.75, -1.25, -1.75, -2.5,
                         -3.5, -5.0, 6.0, 0.0] * 2)
    x[2, :32] = mids
    x[2, 32:64] = mids * 4.0                                 # the same one scale step up
    x[2, 64:96] = mids / 3.0                                 # largest value 2: scale 2^-1
    x[2, 96:128] = 0.0
    x[2, 128:160] = 1e-35                                    # below the e2m1 quantizer's floor
    x[3] = x[3].half().float() * 37.0                        # fp16-representable inputs
    return x


def main():
    sys.path.insert(0, REF)
    from turboquant_utils.triton_kernels_a8 import quantize_act_per_token_group, _build_merged_block_info
    from turboquant_utils.triton_kernels_fp8 import quantize_act_per_token_group_fp8
    from turboquant_utils.triton_kernels_fp4 import quantize_act_e2m1_per32

    rec = {"act": [], "block_info": []}
    for seed, rows, k, extra in ((1, 6, 256, 1.0), (2, 5, 384, 0.0215203), (3, 4, 512, 0.0118931)):
        x = inputs(seed, rows, k)
        q8, s8 = quantize_act_per_token_group(x, 128, extra)
        qf, sf = quantize_act_per_token_group_fp8(x, 128, extra)
        p4, sb = quantize_act_e2m1_per32(x)
        rec["act"].append({
            "seed": seed, "rows": rows, "k": k, "extra_scale": extra,
            "x_fp32_bits": x.view(torch.int32).flatten().tolist(),
            "int8": q8.flatten().tolist(),
            "int8_scale_fp32_bits": s8.view(torch.int32).flatten().tolist(),
            "e4m3_bytes": qf.view(torch.uint8).flatten().tolist(),
            "e4m3_scale_fp32_bits": sf.view(torch.int32).flatten().tolist(),
            "e2m1_packed": p4.flatten().tolist(),
            "e2m1_scale_bytes": sb.flatten().tolist(),
        })
    cases = [
        ([(0, 5, 0, 1024), (5, 0, 1024, 1024), (5, 33, 2048, 1024), (38, 16, 3072, 1024)], 16, 64, 1024),
        ([(0, 1, 0, 512)], 32, 128, 512),
        ([(0, 70, 0, 4), (70, 3, 4, 0), (73, 129, 8, 4)], 64, 256, 2048),
        ([(0, 17, 0, 100)], 16, 64, 100),
    ]
    for info, bb, bn, ext in cases:
        out = _build_merged_block_info(info, bb, bn, ext, "cpu")
        rec["block_info"].append({"expert_info": [list(r) for r in info], "block_b": bb,
                                  "block_n": bn, "n_extent": ext, "blocks": out.tolist()})
    try:
        _build_merged_block_info([(0, 0, 0, 64), (0, 4, 64, 0)], 16, 64, 64, "cpu")
        rec["block_info_empty_raises"] = False
    except ValueError:
        rec["block_info_empty_raises"] = True
    with open(OUT, "w") as fh:
        json.dump(rec, fh, separators=(",", ":"))
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()

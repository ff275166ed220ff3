"""Write tests/golden/quant_fixtures.json from the reference checkout.

Run once in the build container (needs /root/reference; never on the GPU box):

    python tests/golden/make_quant_fixtures.py

Records, for small seeded matrices, what the reference's own quantizer and dequantizer produce
(turboquant_quantize_packed_full / turboquant_dequantize_packed{,_rows,_cols},
turboquant_utils/quantize.py:350-474, :478-826) for bit widths 1 / 2 / 4 / 8 and for the 8-bit
uniform grid (quantize.py:394-402), plus the helpers the int8 Linear path builds on
(uniform_codebook_step / is_uniform_codebook, quantization/wxa8/linear.py:35-66, and
build_int8_codebook of the 8-bit codebooks).  The file holds inputs and outputs only.
"""

import json
import os
import sys

import torch

REF = os.environ.get("DARTMOQ_REFERENCE", "/root/reference")
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "quant_fixtures.json")


def bits16(t):
    return t.contiguous().view(torch.int16).flatten().tolist()


def main():
    sys.path.insert(0, REF)
    from turboquant_utils.quantize import (turboquant_dequantize_packed, turboquant_dequantize_packed_cols,
                                           turboquant_dequantize_packed_rows, turboquant_quantize_packed_full)
    from turboquant_utils.triton_kernels_a8 import build_int8_codebook
    from quantization.wxa8.linear import is_uniform_codebook, uniform_codebook_step

    rec = {}
    for name, bit, uniform in (("1", 1, False), ("2", 2, False), ("4", 4, False), ("8", 8, False),
                               ("8u", 8, True)):
        g = torch.Generator().manual_seed(100 + bit + int(uniform))
        w = (torch.randn(4, 256, generator=g) * 0.02).half()
        seed = 40 + bit
        p = turboquant_quantize_packed_full(w, bit, group_size=128, seed=seed, uniform_codebook=uniform)
        full = turboquant_dequantize_packed(p)
        rows = turboquant_dequantize_packed_rows(p, 1, 3)
        cols = turboquant_dequantize_packed_cols(p, 128, 256)
        e = {
            "bit": bit, "uniform": uniform, "seed": seed, "shape": [4, 256],
            "w_fp16_bits": bits16(w),
            "indices_packed": p["indices_packed"].flatten().tolist(),
            "indices_packed_shape": list(p["indices_packed"].shape),
            "norms_fp16_bits": bits16(p["norms"]), "norms_shape": list(p["norms"].shape),
            "codebook_fp16_bits": bits16(p["codebook"]),
            "codebook_type": p.get("codebook_type"),
            "dequant_dtype": str(full.dtype),                 # the reference returns the weight dtype
            "dequant_fp16_bits": bits16(full.half()),
            "dequant_rows_1_3_fp16_bits": bits16(rows.half()),
            "dequant_cols_128_256_fp16_bits": bits16(cols.half()),
        }
        if bit == 8:
            e["is_uniform_codebook"] = bool(is_uniform_codebook(p["codebook"]))
            if uniform:
                e["uniform_codebook_step"] = float(uniform_codebook_step(p["codebook"]))
            i8, step = build_int8_codebook(p["codebook"])
            e["int8"] = i8.tolist()
            e["int8_step"] = float(step)
        rec[name] = e
    with open(OUT, "w") as fh:
        json.dump(rec, fh)
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()

"""CPU oracle for the DartMoQ quantized MoE FFN hot path.

TEST INFRASTRUCTURE ONLY.  This package is a CPU (torch / numpy) restatement of
the reference algorithm.  It is imported by tests/, by
``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of ``bench.py`` as
the *checker*; the shipped HIP path never imports it and never falls back to it.

Every function cites the reference file:line whose arithmetic it follows
(paths relative to the reference checkout).

Pinning status (what fixes each function independently of this restatement):

=====================================  =======================================
function                               pinned by
=====================================  =======================================
codebook.lloyd_max_gaussian            textbook N(0,1) Lloyd-Max levels, fixed
                                       point conditions, distortion values
packing.pack_nbit / unpack_nbit        closed form + brute force + round trip
packing.convert_to_group_first         closed form (index identity)
rotation.rotation_matrix               orthogonality, diag(R)>0 sign rule,
                                       seed determinism
turboquant.quantize / dequantize       Lloyd-Max relerr figures, matmul identity
luts.build_int8_codebook               closed form, published relerr
luts.build_fp8_codebook                published relerr, grid membership;
                                       exact scale choice: golden fixture
luts.build_e2m1_codebook               published relerr; exact (nib,E0,resid):
                                       golden fixture
luts.fold_indices_to_e2m1              closed form (byte identity)
actquant.quantize_act_int8             closed form, published relerr
actquant.quantize_act_fp8              torch float8_e4m3fn cast, published relerr
actquant.quantize_act_e2m1             8-point grid brute force, tie rule
routing.*                              torch.topk / stable sort, invariants
moe.reference_forward                  dense fp32 MoE on dequantized weights
moe.quantized_forward (A8/FP8/FP4)     published module-level relerr anchors
moe.shared_quantized_forward           dense SwiGLU MLP on dequantized Linears
norm.rms_norm                          unit RMS, scale invariance, hand case
=====================================  =======================================

The Triton code generation boundary of the reference (tl.dot accumulation
order, fp16 accumulators) is not restated: parity unpinned there by design,
fp16 outputs are compared within the stated tolerance against fp32 maths.
"""

from . import codebook, packing, rotation, turboquant, luts, actquant, routing, moe, norm  # noqa: F401

"""MI355X-native quantized-weight matmul path behind reinstinct's kernel API.

The product is `librein.so` (C ABI, see include/rein.h) plus the gfx950 code
object `rein_gfx950.hsaco`; this package is the thin host-side mirror used by
the tests and the benchmark:

    reinstinct_amd.quant     src/quant   (layouts, repack, synthetic quantizers)
    reinstinct_amd.hip       src/hip     (DeviceBuf, Stream, Event, Graph, Module)
    reinstinct_amd.runtime   launch sites of src/runtime/{qwen35,prefill}.rs

There is no CPU fallback: importing works anywhere, computing needs a GPU.
"""
from ._lib import ReinError, lib, load  # noqa: F401

Q4_0, Q8_0, Q4_K, Q5_K, Q6_K, IQ4_XS = 2, 8, 12, 13, 14, 23
# relabelled onto the Q5_K / IQ4_XS planes and kernels (src/quant/q5_1.rs, src/quant/iq3_s.rs):
# Q5_1 for MoE expert tensors only, IQ3_S for dense tensors only, as in the reference
Q5_1, IQ3_S = 7, 21
FORMATS = {"q4_0": Q4_0, "q4_k": Q4_K, "q5_k": Q5_K, "q6_k": Q6_K, "q8_0": Q8_0, "iq4_xs": IQ4_XS}

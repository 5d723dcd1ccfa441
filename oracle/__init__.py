"""CPU oracle for the quantized-weight linear / MoE expert path.

TEST INFRASTRUCTURE ONLY. Nothing in the shipped package imports this directory: it is the checker the HIP kernels
are compared against (tests/, the smoke check, and the CPU-baseline leg of the benchmark), never the thing that is
measured or shipped.

It restates, in plain numpy/torch on the CPU, the algorithms of the reference (paths relative to the reference tree):

  w3_format.py     hibana/kernels/w3.py:52-242        W3 codebooks, LUT, pack_codes, codes, group_scales, dequantize,
                                                      the nearest-level quantizer, interleave_rows
  nvfp4_format.py  hibana/weights/modelopt.py:84-156  E2M1 unpack, 128x4 block-scale swizzle (2-D and per expert),
                   hibana/kernels/w3_moe.py:97-110    pair_order
  layers.py        hibana/kernels/w3_moe.py:88-92,182-214, hibana/model/flashnext/moe.py:122-192,
                   hibana/kernels/flashnext_fused.py:278-319,506-571, tests/nemotron_reference.py:236-254,550-593,
                   hibana/kernels/csrc/w3_gemm.cu:710-782,1196-1213
                                                      weight-only dense products, expert-sorted plan, gated-SiLU and
                                                      ReLU^2 routed experts, combine, routing, latent MoE

Pinning (what each function is checked against, besides round trips) is listed per function in the module
docstrings; the checks live in tests/test_oracle_*.py.
"""

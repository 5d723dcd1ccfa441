"""MI355X-native quantized-weight linear and MoE expert kernels behind the reference's `hibana.kernels` op signatures.

  hibana_amd.kernels.w3       W3Weight, pack / pack_codes / codes / group_scales / dequantize / w3_linear / attach
  hibana_amd.kernels.w3_moe   W3Experts, w3_moe, fc1_order, moe layer
  hibana_amd.kernels.ops      nvfp4_linear, w3_decode, silu_and_mul, moe_combine(_pairs), route_topk
  hibana_amd.weights          Nvfp4Linear, unpack_fp4, block-scale swizzle, the Linear protocol

The compute is hand-written HIP for gfx950 in hibana_amd/csrc, loaded through a C ABI (include/hibana_hip.h).
There is no CPU fallback: calling an op without the built library or without a GPU raises.
"""
__version__ = "0.1.0"

"""nerva_amd: MI355X (gfx950) batch-1 decode backend behind the nerva C ABI.

The product is nerva_amd/libnerva_hip.so (HIP kernels + C ABI, see
include/nerva_hip_api.h). This package only loads it and offers thin numpy
plumbing for tests and benchmarks; all arithmetic runs in the HIP library and
importing a compute helper without the built library raises.
"""
from . import abi
from .runtime import (DeviceBuffer, Device, device_available, gemv, gemv_launch_shape, gemv_launch_plan, fp8_gemv, paged_attention, paged_attention_status,
                      argmax, argmax_static, sample, gemm_rows, gemm_rows_workspace_bytes, gemm_operand_order, gemm_operand_slots, moe_fp8_experts, moe_route_softmax, PagedKvCache)
from .session import DecodeSession, ModelWeights, Qwen3_8B, WeightPlan, hash_weight_blocks
from . import checkpoint

__all__ = ["abi", "checkpoint", "DeviceBuffer", "Device", "device_available", "gemv", "gemv_launch_shape", "gemv_launch_plan", "fp8_gemv",
           "paged_attention", "paged_attention_status", "argmax", "argmax_static", "sample", "gemm_rows", "gemm_rows_workspace_bytes", "gemm_operand_order", "gemm_operand_slots", "moe_fp8_experts", "moe_route_softmax", "PagedKvCache",
           "DecodeSession", "ModelWeights", "Qwen3_8B", "WeightPlan", "hash_weight_blocks"]

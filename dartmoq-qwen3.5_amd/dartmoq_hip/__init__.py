"""dartmoq_hip: MI355X-native kernels for DartMoQ's quantized MoE FFN layer."""

from . import _lib, checkpoint, hostprep, kernels, linear, ops, quantizer  # noqa: F401
from .linear import WxA16Linear, WxA8Linear, WxFP8Linear  # noqa: F401
from .moe import (BitPoolWeights, WxA16BitPartitionedGroupMoE, WxA8BitPartitionedGroupMoE,  # noqa: F401
                  WxFP4BitPartitionedGroupMoE, WxFP8BitPartitionedGroupMoE, convert_moe)

__all__ = [
    "ops", "hostprep", "kernels", "linear", "checkpoint", "quantizer", "WxA16Linear", "WxA8Linear", "WxFP8Linear", "BitPoolWeights", "WxA16BitPartitionedGroupMoE",
    "WxA8BitPartitionedGroupMoE", "WxFP8BitPartitionedGroupMoE", "WxFP4BitPartitionedGroupMoE",
    "convert_moe",
]

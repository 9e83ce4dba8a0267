"""MI355X (gfx950) mixture-of-experts layer behind RustingBrain's MoE interface."""
from .moe import (BackendUnavailable, Device, DeviceError, InvalidConfig, InvalidInput, Layout, MemoryBudget,
                  MoeCache, MoeConfig, MoeLayer, NetworkError, OutOfMemory, Unsupported, UNROUTED)
from .transformer import ParameterCounts, TransformerBuilder, TransformerConfig

__all__ = ["BackendUnavailable", "Device", "DeviceError", "InvalidConfig", "InvalidInput", "Layout",
           "MemoryBudget", "MoeCache", "MoeConfig", "MoeLayer", "NetworkError", "OutOfMemory", "Unsupported",
           "UNROUTED", "ParameterCounts", "TransformerBuilder", "TransformerConfig"]

"""MI355X-native mixture-of-experts layer path for Omega-AI: host side of libomega_hip.so."""
from . import configs, java_random, weights_json
from ._lib import LIB_PATH, load_library
from .moe_layer import Context, DeviceBuffer, MoELayer, bf16_bits_to_f32, f32_to_bf16_bits

__all__ = ["configs", "java_random", "weights_json", "LIB_PATH", "load_library", "Context", "DeviceBuffer", "MoELayer", "bf16_bits_to_f32",
           "f32_to_bf16_bits"]

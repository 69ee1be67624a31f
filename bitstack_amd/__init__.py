"""MI355X-native BitStack compressed-linear inference path.

Host side mirrors the reference's module and helper names; the device side is
hand-written HIP for gfx950 behind a C ABI (include/bitstack_hip.h), loaded with
ctypes from bitstack_amd/csrc/libbitstack_hip.so.
"""
from bitstack_amd.modules.BitStackLinear import BitStackLinear, ScaledActivation, compose_weight  # noqa: F401
from bitstack_amd.utils.pack_utils import pack_sign, unpack_sign  # noqa: F401

__all__ = ["BitStackLinear", "ScaledActivation", "compose_weight", "pack_sign", "unpack_sign"]

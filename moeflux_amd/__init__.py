"""MI355X-native attention path for moeflux: hand-written HIP kernels behind a C ABI.

``moeflux_amd.ffi`` binds ``lib/libmoeflux_attn_hip.so`` (declared in
``include/moeflux_attn.h``); ``moeflux_amd.ctx.Ctx`` mirrors, for the attention
core, the hooks of the reference's ``RsCtx`` (crates/moeflux/src/riir/mod.rs).
There is no CPU fallback: importing ``ffi`` without the built library raises.
"""
from .ctx import Ctx, Config, MfaError  # noqa: F401

__all__ = ["Ctx", "Config", "MfaError"]

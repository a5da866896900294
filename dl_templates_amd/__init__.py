"""MI355X-native attention hot path of dl_templates: tiled 2D sliding-window flash attention,
fused 2D rotary encoding and flash attention with separate qk / vo head dims.

Modules mirror the reference's ``src/`` files: ``tiled_swa``, ``fused_rope2d``, ``rope2d``,
``flash_attn``.  All device work is done by hand-written gfx950 HIP kernels in
``libdlt_hip.so`` (C ABI in ``include/dlt.h``)."""
__all__ = ["tiled_swa", "fused_rope2d", "rope2d", "flash_attn"]

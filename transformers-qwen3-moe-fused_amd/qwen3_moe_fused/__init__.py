"""MI355X-native drop-in for the ``qwen3_moe_fused`` hot path (moe_fused_linear and its
neighbours).  Module paths and public names follow the reference package; all device work
is done by ``libmoe_fused_linear.so`` (HIP, gfx950) through ``_lib``."""

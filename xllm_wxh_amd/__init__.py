"""MI355X-native paged-KV decode path for xLLM: KV write through slot_mapping and
paged-attention decode, hand-written HIP for gfx950 behind a C ABI."""

__all__ = ["ops", "build"]

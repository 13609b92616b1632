"""MI355X-native Hogwild! fragmented-KV attention: HIP kernels behind a C ABI, with the host-side
mirror of the reference operator interface in `inference_lib_amd.attention`."""
__all__ = ["attention", "cache", "cases", "model", "_lib"]

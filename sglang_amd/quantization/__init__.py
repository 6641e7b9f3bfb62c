"""Host-side callers of the operators, mirroring python/sglang/srt/layers/quantization."""

"""Serving-side surface: `core` (vLLM-independent: PackedShards, the shapequant::linear op) and
`plugin` (the vLLM quantization method; imports vLLM, so it is loaded only where vLLM exists)."""

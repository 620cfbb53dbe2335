"""MI355X-native codebook linear layer (learned weight-shape codebook: packed layout,
decode-time GEMV, small-batch path, prefill GEMM) behind the reference's packed-file layout and
its vLLM linear-method surface.  All device work runs in libsqhip.so (hand-written HIP for
gfx950); there is no CPU or PyTorch fallback: every op raises if the library is missing."""

__all__ = ["packed", "masks", "codebook", "kernels", "vllm_ext"]

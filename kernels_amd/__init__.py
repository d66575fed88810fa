"""MI355X-native kernels behind the PyTorch-facing API of alexdremov/kernels.

Only the streaming-attention operator lives here; `kernels_amd/streaming_attention`
mirrors `src/streaming_attention` of the reference and `kernels_amd/csrc` holds the HIP
kernels and their C ABI.
"""

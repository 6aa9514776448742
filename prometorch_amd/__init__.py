"""MI355X (gfx950) kernels for PromeTorch's GGUF Q4_K / Q6_K batch-1 decode path.

`prometorch_amd.ops` mirrors the reference's `at::cuda::launch_*` operators on top of the C ABI
of libptm_hip.so; `prometorch_amd.decode` wraps the decode runtime, `prometorch_amd.gguf` the file loader and
`prometorch_amd.tokenizer` the tokenizer.  `prometorch_amd.testing` (seeded synthetic super-blocks and models, a GGUF
writer) serves the tests and the benchmark only."""
__all__ = ["ops", "decode", "gguf", "tokenizer", "build"]

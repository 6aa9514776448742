"""MI355X (gfx950) kernels for PromeTorch's GGUF Q4_K / Q6_K batch-1 decode path.

`prometorch_amd.ops` mirrors the reference's `at::cuda::launch_*` operators on top of the C ABI
of libptm_hip.so; `prometorch_amd.decode` wraps the decode runtime; `prometorch_amd.synth`
generates the seeded synthetic super-blocks of the benchmark configurations."""
__all__ = ["ops", "decode", "synth", "build"]

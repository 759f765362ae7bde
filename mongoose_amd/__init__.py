"""mongoose_amd -- MI355X (gfx950) backend for mongoose's fused quantized decode path.

The product is libmongoose_hip.so (HIP kernels + C ABI, sources in csrc/);
`engine` mirrors the Go API over it.  Importing `engine` loads the library and
fails if it has not been built.
"""
__all__ = ["build", "engine", "lib", "configs"]

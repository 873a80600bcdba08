"""tatara_amd — MI355X (gfx950) backend for the attention-family hot path of
Tatara (full-attention and Gated DeltaNet layers of Qwen3.6-35B-A3B).

The product is the shared object `tatara_amd/lib/libtatara_hip.so` (hand-written
HIP kernels behind the C ABI declared in include/tatara_hip.h).  This package
only binds that C ABI with ctypes for Python hosts, mirroring the reference's
backend interface (include/tatara/backend/metal/{resources,pipeline,commands}.h).
There is no CPU or PyTorch fallback: importing `tatara_amd.backend` raises if the
library has not been built (`python -c "import __graft_entry__ as g; g.build()"`
or `make -C tatara_amd/csrc`)."""

__all__ = ["backend", "stack", "sweep", "q4_sweep"]

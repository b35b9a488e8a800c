"""dgpp_amd: the MI355X (gfx950) quantized MoE expert GEMV path behind the reference's launcher
surface. `dgpp_amd.launch` mirrors the operators, `dgpp_amd.hostgen` the host encoders; both go
through the C ABI of libdgpp_amd.so (include/dgpp_amd.h). Importing the package does not load the
library; the first call does, and fails loudly if it has not been built."""

__all__ = ["launch", "hostgen", "build"]

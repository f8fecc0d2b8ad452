"""camx: MI355X (gfx950) implementation of the fused per-layer row kernels of the Caminus inference engine, behind the
reference's own op entry points. The HIP kernels live in caminus_amd/csrc and are reached through the C ABI of
libcamx.so (include/camx.h); PyTorch is used for device memory and streams only."""
__version__ = '0.1.0'

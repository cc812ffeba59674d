"""vqtree_amd -- MI355X (gfx950) fused VQ-attention kernels behind the reference's `ops/` call surface.

The compute lives in `libvqattn_gfx950.so` (hand-written HIP, C ABI declared in include/vqattn.h); `vqtree_amd.ops`
mirrors the reference's operator modules and calls the library through ctypes.  There is no CPU fallback: every
operator raises if the library is not built or the tensors are not on a GPU.
"""
__version__ = "0.1.0"

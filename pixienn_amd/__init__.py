"""MI355X (gfx950) non-convolution layer kernels behind PixieNN's kernel/layer API.

capi     ctypes binding of the C ABI (include/pixienn_hip.h)
ops      torch-tensor front-end (argument checks + stream plumbing)
build    in-tree hipcc build of libpixienn_hip.so
"""
__all__ = ["capi", "ops", "build", "workloads"]

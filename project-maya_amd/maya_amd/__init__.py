"""Host side of the MI355X routed-MoE expert block: ctypes bindings of libmaya_moe.so (the C ABI of include/maya_moe.h)
and thin helpers that keep the reference's operator vocabulary (expert blobs, plans, entries, groups).

PyTorch is used for device memory and streams only; every computation runs in the library's HIP kernels.  There is no
CPU fallback: importing `maya_amd.lib` raises when the built library is missing.
"""
__all__ = ["lib", "exl3", "prefill", "expert_files", "build"]

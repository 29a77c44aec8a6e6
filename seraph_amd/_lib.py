"""Loads the in-tree native libraries.  There is no CPU fallback: if a library is
missing the import of anything that computes fails with a clear error."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
KERNEL_LIB = os.path.join(HERE, "lib", "libseraph_hip.so")
BACKEND_LIB = os.path.join(HERE, "lib", "libseraph_hip_backend.so")

_kernels = None
_backend = None


class SeraphError(RuntimeError):
    pass


def kernels():
    """ctypes handle of libseraph_hip.so (the C-ABI kernel library)."""
    global _kernels
    if _kernels is None:
        if not os.path.exists(KERNEL_LIB):
            raise SeraphError(f"{KERNEL_LIB} is not built; run `python -m seraph_amd.build` (needs hipcc)")
        lib = C.CDLL(KERNEL_LIB, mode=C.RTLD_GLOBAL)
        lib.seraph_hip_last_error.restype = C.c_char_p
        for name in ("seraph_attention_backward_ws_bytes", "seraph_attention_backward_ws_bytes_banded",
                     "seraph_rmsnorm_backward_ws_bytes", "seraph_embedding_backward_ws_bytes",
                     "seraph_gemm_scaled_ws_bytes", "seraph_rmsnorm_backward_static_max_bytes"):
            getattr(lib, name).restype = C.c_size_t
        lib.seraph_gemm_grouped_kernel_name.restype = C.c_char_p
        lib.seraph_gemm_chain_kernel_name.restype = C.c_char_p
        lib.seraph_gemm_kernel_name.restype = C.c_char_p
        _kernels = lib
    return _kernels


def backend():
    """ctypes handle of libseraph_hip_backend.so (vulkan_* compatible host backend + step drivers)."""
    global _backend
    if _backend is None:
        kernels()
        if not os.path.exists(BACKEND_LIB):
            raise SeraphError(f"{BACKEND_LIB} is not built; run `python -m seraph_amd.build`")
        _backend = C.CDLL(BACKEND_LIB, mode=C.RTLD_GLOBAL)
    return _backend


def check(rc, what=""):
    if rc != 0:
        msg = kernels().seraph_hip_last_error()
        raise SeraphError(f"{what} failed ({rc}): {msg.decode() if msg else ''}")

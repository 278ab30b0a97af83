"""ctypes binding of host/liblg_host.so (GGUF reader/writer, codecs, model geometry, generator)."""
import ctypes as C
import os
import subprocess

HOST_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "host")
_lib = None


def build():
    subprocess.run(["make", "-C", HOST_DIR, "-B", "liblg_host.so"], check=True,
                   stdout=subprocess.DEVNULL)


def lib():
    """The loaded host library; built first only when no built copy exists."""
    global _lib
    if _lib is None:
        path = os.path.join(HOST_DIR, "liblg_host.so")
        if not os.path.exists(path):
            build()
        _lib = C.CDLL(path)
        _lib.lg_synth_write.restype = C.c_int
        _lib.dequantize_into.restype = C.c_bool
        _lib.dequantize_into.argtypes = [C.c_uint32, C.c_void_p, C.c_void_p, C.c_int64]
        _lib.lg_quantize_q4_0.argtypes = [C.c_void_p, C.c_void_p, C.c_int64]
        _lib.lg_quantize_q4_0.restype = None
        _lib.load_gguf.restype = C.c_void_p
        _lib.load_gguf.argtypes = [C.c_char_p]
        _lib.free_gguf.argtypes = [C.c_void_p]
        _lib.free_gguf.restype = None
    return _lib

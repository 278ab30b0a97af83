"""placeholder"""
class HipError(RuntimeError):
    pass
class HipBackend:  # filled in with the HIP library
    pass
def load_hip():
    raise HipError("HIP library not built")

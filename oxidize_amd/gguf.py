"""GGUF model files through the C ABI (``oxh_gguf_*``): tensor views and
metadata, and the upload of every tensor the library has kernels for."""
import ctypes

from ._lib import DECLINED, OxhError, OxhTensor, check, lib


class GgufFile:
    def __init__(self, path):
        self.handle = ctypes.c_void_p()
        check(lib().oxh_gguf_open(str(path).encode(), ctypes.byref(self.handle)))
        ver, align, start = ctypes.c_uint32(), ctypes.c_uint64(), ctypes.c_uint64()
        nt, nm = ctypes.c_size_t(), ctypes.c_size_t()
        check(lib().oxh_gguf_info(self.handle, ctypes.byref(ver), ctypes.byref(align), ctypes.byref(start),
                                  ctypes.byref(nt), ctypes.byref(nm)))
        self.version, self.alignment, self.data_start = ver.value, align.value, start.value
        self.n_tensors, self.n_metadata = nt.value, nm.value

    def tensor_at(self, index):
        t = OxhTensor()
        check(lib().oxh_gguf_tensor_at(self.handle, index, ctypes.byref(t)))
        return t

    def tensors(self):
        return [self.tensor_at(i) for i in range(self.n_tensors)]

    def find(self, name):
        """The tensor of that name, or None."""
        t = OxhTensor()
        rc = lib().oxh_gguf_tensor_find(self.handle, name.encode(), ctypes.byref(t))
        if rc == DECLINED:
            return None
        check(rc)
        return t

    def meta_u64(self, key):
        v = ctypes.c_uint64()
        return v.value if lib().oxh_gguf_meta_u64(self.handle, key.encode(), ctypes.byref(v)) == 0 else None

    def meta_f64(self, key):
        v = ctypes.c_double()
        return v.value if lib().oxh_gguf_meta_f64(self.handle, key.encode(), ctypes.byref(v)) == 0 else None

    def meta_str(self, key):
        p, n = ctypes.c_void_p(), ctypes.c_size_t()
        if lib().oxh_gguf_meta_str(self.handle, key.encode(), ctypes.byref(p), ctypes.byref(n)) != 0:
            return None
        return ctypes.string_at(p.value, n.value)

    def register_all(self):
        """-> (tensors made resident, their bytes)"""
        n, b = ctypes.c_size_t(), ctypes.c_size_t()
        check(lib().oxh_gguf_register_all(self.handle, ctypes.byref(n), ctypes.byref(b)))
        return n.value, b.value

    def close(self):
        if self.handle:
            lib().oxh_gguf_close(self.handle)
            self.handle = ctypes.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()
        return False


__all__ = ["GgufFile", "OxhError"]

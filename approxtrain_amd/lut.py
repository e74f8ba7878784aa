"""LUT handle: the host-side counterpart of the reference's ``approx_mul_lut``
(approx_mul_lut.h:7-80): built from the ``mant_mul_lut`` file name attr, owns
the device copy of the table, exposes the derived mask / shifts."""
import ctypes as C
import threading

import numpy as np

from ._lib import check, load_library

_cache = {}
_cache_lock = threading.Lock()


class ApproxMulLut:
    """``ApproxMulLut('lut/MBM_7.bin')`` reads the file (mantissa width taken
    from the ``_<m>.bin`` suffix, approx_mul_lut.h:22-25) and uploads it to the
    current device.  ``ApproxMulLut.from_entries`` takes the table from memory
    (uint8 ``carry<<7|mantissa`` for m <= 7, or uint32 ``carry<<31|mantissa
    in place`` for m <= 11)."""

    def __init__(self, path=None, _handle=None):
        self._h = C.c_void_p()
        if _handle is not None:
            self._h = _handle
        else:
            if not path:
                raise ValueError("no mant lut file name given")
            check(load_library().amsim_lut_load_file(str(path).encode(), C.byref(self._h)))
        self.path = path
        lib = load_library()
        self.mant_width = lib.amsim_lut_mant_width(self._h)
        mask, a, b = C.c_uint32(), C.c_int(), C.c_int()
        check(lib.amsim_lut_params(self._h, C.byref(mask), C.byref(a), C.byref(b)))
        self.mant_mask, self.a_shift, self.b_shift = mask.value, a.value, b.value

    @classmethod
    def from_entries(cls, entries, mant_width):
        e = np.ascontiguousarray(entries)
        if e.dtype not in (np.uint8, np.uint32):
            raise TypeError("LUT entries must be uint8 or uint32")
        h = C.c_void_p()
        check(load_library().amsim_lut_create(e.ctypes.data_as(C.c_void_p), e.nbytes, int(mant_width),
                                              e.dtype.itemsize, C.byref(h)))
        return cls(_handle=h)

    @classmethod
    def cached(cls, path):
        """One handle per (device, file) instead of the reference's one copy per op node."""
        import torch
        key = (torch.cuda.current_device() if torch.cuda.is_available() else -1, str(path))
        with _cache_lock:
            if key not in _cache:
                _cache[key] = cls(path)
            return _cache[key]

    @property
    def handle(self):
        return self._h

    def close(self):
        if self._h:
            load_library().amsim_lut_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

"""MI355X-native HEMMer hot path: ctypes binding of libhemm.so (C ABI in include/hemm.h).

The shared library is the product; this module only loads it and gives device buffers
(torch tensors used as plain HBM allocations) a convenient shape.  There is no CPU
fallback: if the library or a GPU is missing, calls raise.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libhemm.so")
_lib = None


class HemmError(RuntimeError):
    pass


def lib():
    """Load libhemm.so (built by build.py); raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise HemmError("libhemm.so is missing: run __graft_entry__.build() first "
                            "(there is no CPU fallback)")
        # torch ships its own HIP runtime under the same soname; it has to be the one already
        # loaded when libhemm.so resolves libamdhip64, or the process ends up with two runtimes.
        import torch  # noqa: F401
        _lib = ctypes.CDLL(LIB_PATH)
        _declare(_lib)
    return _lib


u64p = ctypes.POINTER(ctypes.c_uint64)
u32p = ctypes.POINTER(ctypes.c_uint32)
vp = ctypes.c_void_p


def _declare(L):
    L.hemm_last_error.restype = ctypes.c_char_p
    L.hemm_context_create.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, u64p,
                                      ctypes.c_uint32, ctypes.POINTER(vp)]
    L.hemm_context_destroy.argtypes = [vp]
    L.hemm_context_psi.restype = ctypes.c_uint64
    L.hemm_context_psi.argtypes = [vp, ctypes.c_uint32]
    L.hemm_primes_below.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, u64p]
    L.hemm_ntt.argtypes = [vp, vp, u32p, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_int, vp]


def check(rc):
    if rc != 0:
        msg = lib().hemm_last_error().decode()
        if rc == 1:
            raise ValueError(msg)
        raise HemmError(msg)


class Context:
    """Owns a hemm_context (device twiddle tables for one parameter set)."""

    def __init__(self, log_n, q_primes, p_primes, dnum):
        L = lib()
        self.log_n, self.N = log_n, 1 << log_n
        self.q, self.p = [int(x) for x in q_primes], [int(x) for x in p_primes]
        self.nQ, self.nP, self.dnum = len(self.q), len(self.p), dnum
        mods = self.q + self.p
        arr = (ctypes.c_uint64 * len(mods))(*mods)
        h = vp()
        check(L.hemm_context_create(log_n, self.nQ, self.nP, arr, dnum, ctypes.byref(h)))
        self.h = h

    def close(self):
        if getattr(self, "h", None):
            lib().hemm_context_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def psi(self, idx):
        return lib().hemm_context_psi(self.h, idx)

    def ntt(self, data, prime_idx, inverse=False, stream=None):
        """In-place transform of a CUDA int64 tensor shaped [..., n_limbs, N]."""
        n_limbs = len(prime_idx)
        assert data.is_cuda and data.is_contiguous() and data.shape[-1] == self.N
        assert data.shape[-2] == n_limbs
        n_polys = data.numel() // (n_limbs * self.N)
        idx = (ctypes.c_uint32 * n_limbs)(*prime_idx)
        check(lib().hemm_ntt(self.h, vp(data.data_ptr()), idx, n_limbs, n_polys, int(inverse),
                             vp(stream or 0)))
        return data


def primes_below(bits, log_n, count):
    out = (ctypes.c_uint64 * count)()
    check(lib().hemm_primes_below(bits, log_n, count, out))
    return list(out)

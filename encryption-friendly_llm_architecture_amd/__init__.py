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


class RotTerm(ctypes.Structure):
    _fields_ = [("ext", vp), ("b", vp), ("evk", vp), ("mask", vp), ("galois", ctypes.c_uint32),
                ("mask_shift", ctypes.c_uint32), ("pt", vp), ("pt_galois", ctypes.c_uint32),
                ("flags", ctypes.c_uint32)]


class TensorGroup(ctypes.Structure):
    _fields_ = [("t1", vp), ("t2", vp), ("acc3", vp), ("n_pairs", ctypes.c_uint32), ("accumulate", ctypes.c_uint32)]


class LinTerm(ctypes.Structure):
    _fields_ = [("ct", vp), ("mask", vp), ("stride", ctypes.c_uint64), ("galois", ctypes.c_uint64)]


def _declare(L):
    L.hemm_last_error.restype = ctypes.c_char_p
    L.hemm_context_create.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, u64p,
                                      ctypes.c_uint32, ctypes.POINTER(vp)]
    L.hemm_context_destroy.argtypes = [vp]
    L.hemm_context_psi.restype = ctypes.c_uint64
    L.hemm_context_psi.argtypes = [vp, ctypes.c_uint32]
    L.hemm_primes_below.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, u64p]
    L.hemm_ntt.argtypes = [vp, vp, u32p, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_int, vp]
    sz, u32, u64, ci = ctypes.c_size_t, ctypes.c_uint32, ctypes.c_uint64, ctypes.c_int
    L.hemm_pointwise.argtypes = [vp, ci, vp, sz, vp, sz, vp, sz, u32, ci, u32, vp]
    L.hemm_mul_scalar.argtypes = [vp, vp, sz, u64p, vp, sz, u32, ci, u32, vp]
    L.hemm_encode.argtypes = [vp, vp, ctypes.c_double, u32, ci, u32, vp, vp]
    L.hemm_decode.argtypes = [vp, vp, u32, ctypes.c_double, vp, vp, vp]
    L.hemm_mul_imag_unit.argtypes = [vp, vp, sz, vp, sz, u32, u32, vp]
    L.hemm_tensor.argtypes = [vp, vp, sz, vp, sz, vp, sz, u32, ci, vp]
    L.hemm_automorphism.argtypes = [vp, vp, sz, vp, sz, u64, u32, u32, vp]
    L.hemm_modup.argtypes = [vp, vp, u32, vp, vp]
    L.hemm_inner_product.argtypes = [vp, vp, vp, u32, vp, vp]
    L.hemm_moddown.argtypes = [vp, vp, u32, u32, vp, sz, vp]
    L.hemm_keyswitch.argtypes = [vp, vp, vp, u32, vp, sz, vp, vp]
    L.hemm_rotate.argtypes = [vp, vp, sz, vp, u64, u32, vp, sz, vp]
    L.hemm_relinearize.argtypes = [vp, vp, sz, vp, u32, vp, sz, vp]
    L.hemm_rescale.argtypes = [vp, vp, sz, vp, sz, u32, u32, vp]
    L.hemm_rescale_static.argtypes = [vp, vp, sz, vp, sz, u32, u32, vp]
    L.hemm_sample_uniform.argtypes = [vp, u64p, u32p, u32, vp, vp]
    L.hemm_sample_error.argtypes = [vp, u64, u32p, u32, vp, vp]
    L.hemm_modup_batch.argtypes = [vp, vp, sz, u32, u32, vp, vp, vp]
    L.hemm_hoisted_terms.argtypes = [vp, ctypes.POINTER(RotTerm), u32p, u32, u32, vp, ci, vp]
    L.hemm_moddown_batch.argtypes = [vp, vp, u32, u32, ci, vp, sz, vp, vp]
    L.hemm_hoisted_moddown.argtypes = [vp, ctypes.POINTER(RotTerm), u32p, u32, u32, ci, ci, vp, vp, sz, vp, vp]
    L.hemm_masked_sum_batch.argtypes = [vp, ctypes.POINTER(LinTerm), u32p, u32, u32, u32, vp, vp]
    L.hemm_tensor_batch.argtypes = [vp, vp, vp, u32, u32, vp, ci, vp]
    L.hemm_tensor_batch_groups.argtypes = [vp, ctypes.POINTER(TensorGroup), u32, u32, sz, vp]
    L.hemm_compact_mask.argtypes = [vp, vp, u32, u32, vp, ctypes.POINTER(ci), vp]
    L.hemm_key_compact_words.argtypes = [vp]
    L.hemm_key_compact_words.restype = ctypes.c_size_t
    L.hemm_key_compact.argtypes = [vp, vp, vp, vp]
    L.hemm_sum_parts.argtypes = [vp, vp, u32, u32, u32, vp, vp]


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

    TRAFFIC_KINDS = ("transforms", "key_products", "basis_conversions", "tensor_accumulation", "masked_sums", "pointwise")

    def traffic(self, reset=False):
        """Algorithmic bytes and launch counts queued on this context since the last reset, by kind of work."""
        b = (ctypes.c_uint64 * 8)()
        n = (ctypes.c_uint64 * 8)()
        check(lib().hemm_traffic(self.h, b, n, int(reset)))
        return ({k: int(b[i]) for i, k in enumerate(self.TRAFFIC_KINDS)},
                {k: int(n[i]) for i, k in enumerate(self.TRAFFIC_KINDS)})

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


    def encode(self, slots, scale, nq, with_p=False):
        """slots: complex128 CUDA tensor [n_msgs][N/2] (or [N/2]) -> int64 [n_msgs][nq (+ n_p)][N] (NTT form)."""
        import torch
        z = slots.reshape(-1, self.N // 2).clone().contiguous()
        limbs = nq + (self.nP if with_p else 0)
        out = torch.empty((z.shape[0], limbs, self.N), dtype=torch.int64, device=z.device)
        check(lib().hemm_encode(self.h, vp(z.data_ptr()), ctypes.c_double(scale), nq, int(with_p), z.shape[0],
                                vp(out.data_ptr()), vp(0)))
        return out

    def decode(self, pt, scale, n_limbs=2):
        """pt: int64 CUDA tensor [>= n_limbs][N] (NTT form) -> complex128 CUDA tensor [N/2]."""
        import torch
        ws = torch.empty((n_limbs, self.N), dtype=torch.int64, device=pt.device)
        z = torch.empty(self.N // 2, dtype=torch.complex128, device=pt.device)
        check(lib().hemm_decode(self.h, vp(pt.data_ptr()), n_limbs, ctypes.c_double(scale), vp(ws.data_ptr()),
                                vp(z.data_ptr()), vp(0)))
        return z

    # ---- evaluator-level kernels on [polys][limbs][N] int64 CUDA tensors ---------------------
    def _new(self, polys, limbs, like):
        import torch
        return torch.empty((polys, limbs, self.N), dtype=torch.int64, device=like.device)

    @staticmethod
    def _ps(t):
        return t.stride(0) if t.dim() == 3 else 0

    def pointwise(self, op, a, b, nq, with_p=False, out=None, stream=None):
        """a: [P][>=nl][N]; b: same or a single [>=nl][N] polynomial (broadcast)."""
        nl = nq + (self.nP if with_p else 0)
        polys = a.shape[0]
        if out is None:
            out = self._new(polys, nl, a)
        check(lib().hemm_pointwise(self.h, op, vp(a.data_ptr()), self._ps(a),
                                   vp(b.data_ptr() if b is not None else 0),
                                   self._ps(b) if b is not None else 0, vp(out.data_ptr()),
                                   self._ps(out), nq, int(with_p), polys, vp(stream or 0)))
        return out

    def mul_scalar(self, a, scalars, nq, with_p=False, out=None):
        nl = nq + (self.nP if with_p else 0)
        if out is None:
            out = self._new(a.shape[0], nl, a)
        arr = (ctypes.c_uint64 * nl)(*[int(v) for v in scalars])
        check(lib().hemm_mul_scalar(self.h, vp(a.data_ptr()), self._ps(a), arr, vp(out.data_ptr()),
                                    self._ps(out), nq, int(with_p), a.shape[0], vp(0)))
        return out

    def mul_imag_unit(self, a, nq, out=None):
        if out is None:
            out = self._new(a.shape[0], nq, a)
        check(lib().hemm_mul_imag_unit(self.h, vp(a.data_ptr()), self._ps(a), vp(out.data_ptr()),
                                       self._ps(out), nq, a.shape[0], vp(0)))
        return out

    def tensor(self, c1, c2, nq, out=None, accumulate=False):
        if out is None:
            out = self._new(3, nq, c1)
        check(lib().hemm_tensor(self.h, vp(c1.data_ptr()), self._ps(c1), vp(c2.data_ptr()),
                                self._ps(c2), vp(out.data_ptr()), self._ps(out), nq,
                                int(accumulate), vp(0)))
        return out

    def automorphism(self, a, galois, n_limbs):
        polys = a.shape[0]
        out = self._new(polys, n_limbs, a)
        check(lib().hemm_automorphism(self.h, vp(a.data_ptr()), self._ps(a), vp(out.data_ptr()),
                                      self._ps(out), galois, n_limbs, polys, vp(0)))
        return out

    def beta(self, nq):
        alpha = -(-self.nQ // self.dnum)
        return -(-nq // alpha)

    def sample_uniform(self, stream_keys, prime_idx):
        """out[j] uniform mod prime prime_idx[j] from stream key stream_keys[j] (counter-based, masked rejection)"""
        import torch
        n = len(prime_idx)
        out = torch.empty((n, self.N), dtype=torch.int64, device="cuda")
        keys = (ctypes.c_uint64 * n)(*[int(k) for k in stream_keys])
        idx = (ctypes.c_uint32 * n)(*prime_idx)
        check(lib().hemm_sample_uniform(self.h, keys, idx, n, vp(out.data_ptr()), vp(0)))
        return out

    def sample_error(self, stream_key, prime_idx):
        """residues of the centred-binomial error polynomial of a stream (coefficient form)"""
        import torch
        n = len(prime_idx)
        out = torch.empty((n, self.N), dtype=torch.int64, device="cuda")
        idx = (ctypes.c_uint32 * n)(*prime_idx)
        check(lib().hemm_sample_error(self.h, int(stream_key), idx, n, vp(out.data_ptr()), vp(0)))
        return out

    def modup(self, poly, nq):
        import torch
        ext = torch.empty((self.beta(nq), nq + self.nP, self.N), dtype=torch.int64, device=poly.device)
        check(lib().hemm_modup(self.h, vp(poly.data_ptr()), nq, vp(ext.data_ptr()), vp(0)))
        return ext

    def inner_product(self, ext, evk, nq):
        acc = self._new(2, nq + self.nP, ext)
        check(lib().hemm_inner_product(self.h, vp(ext.data_ptr()), vp(evk.data_ptr()), nq,
                                       vp(acc.data_ptr()), vp(0)))
        return acc

    def moddown(self, acc, nq):
        out = self._new(acc.shape[0], nq, acc)
        check(lib().hemm_moddown(self.h, vp(acc.data_ptr()), nq, acc.shape[0], vp(out.data_ptr()),
                                 self._ps(out), vp(0)))
        return out

    def keyswitch(self, poly, evk, nq, add_b=None):
        out = self._new(2, nq, poly)
        check(lib().hemm_keyswitch(self.h, vp(poly.data_ptr()), vp(evk.data_ptr()), nq,
                                   vp(out.data_ptr()), self._ps(out),
                                   vp(add_b.data_ptr() if add_b is not None else 0), vp(0)))
        return out

    def rotate(self, ct, evk, galois, nq, out=None):
        if out is None:
            out = self._new(2, nq, ct)
        check(lib().hemm_rotate(self.h, vp(ct.data_ptr()), self._ps(ct), vp(evk.data_ptr()), galois,
                                nq, vp(out.data_ptr()), self._ps(out), vp(0)))
        return out

    def relinearize(self, ct3, evk, nq):
        out = self._new(2, nq, ct3)
        check(lib().hemm_relinearize(self.h, vp(ct3.data_ptr()), self._ps(ct3), vp(evk.data_ptr()),
                                     nq, vp(out.data_ptr()), self._ps(out), vp(0)))
        return out

    def rescale(self, ct, nq):
        out = self._new(ct.shape[0], nq - 1, ct)
        check(lib().hemm_rescale(self.h, vp(ct.data_ptr()), self._ps(ct), vp(out.data_ptr()),
                                 self._ps(out), nq, ct.shape[0], vp(0)))
        return out

    def rescale_static(self, ct, nq, out):
        """hemm_rescale_static: the caller brings the output buffer, the call allocates nothing."""
        check(lib().hemm_rescale_static(self.h, vp(ct.data_ptr()), self._ps(ct), vp(out.data_ptr()),
                                        self._ps(out), nq, ct.shape[0], vp(0)))
        return out


    # ---- batched / hoisted forms ------------------------------------------------------------
    def modup_batch(self, polys, nq):
        """polys: [n_in][>=nq][N] -> ext [n_in][beta][nq+K][N]"""
        import torch
        n_in = polys.shape[0]
        ext = torch.empty((n_in, self.beta(nq), nq + self.nP, self.N), dtype=torch.int64, device=polys.device)
        ws = torch.empty((n_in, nq, self.N), dtype=torch.int64, device=polys.device)
        check(lib().hemm_modup_batch(self.h, vp(polys.data_ptr()), polys.stride(0), nq, n_in,
                                     vp(ext.data_ptr()), vp(ws.data_ptr()), vp(0)))
        return ext

    def sum_parts(self, parts, n_parts, nq):
        """[n_out * n_parts][2][nq+K][N] partial hoisted sums -> [n_out][2][nq+K][N]"""
        import torch
        n_out = parts.shape[0] // n_parts
        y = torch.empty((n_out,) + tuple(parts.shape[1:]), dtype=torch.int64, device=parts.device)
        check(lib().hemm_sum_parts(self.h, vp(parts.data_ptr()), n_parts, n_out, nq, vp(y.data_ptr()), vp(0)))
        return y

    def compact_mask(self, mask, shift):
        """run table [limbs][N >> shift][2] = (value, floor(value * 2^64 / prime)) of a mask [limbs][N] over the extended
        basis that is constant over runs of 2^shift residues, or None"""
        import torch
        table = torch.empty((mask.shape[0], self.N >> shift, 2), dtype=torch.int64, device=mask.device)
        ok = ctypes.c_int(0)
        check(lib().hemm_compact_mask(self.h, vp(mask.data_ptr()), mask.shape[0], shift, vp(table.data_ptr()),
                                      ctypes.byref(ok), vp(0)))
        return table if ok.value else None

    def compact_key(self, evk):
        """The compact form of a key [dnum][2][nQ+nP][N] that the hoisted sums read (6 bytes per residue of a prime
        below 2^44): pass it as evk with compact_keys=True (or a list of flags, one per term in order; the library takes
        one layout per call)."""
        import torch
        out = torch.empty(lib().hemm_key_compact_words(self.h), dtype=torch.int64, device=evk.device)
        check(lib().hemm_key_compact(self.h, vp(evk.data_ptr()), vp(out.data_ptr()), vp(0)))
        return out

    def hoisted_terms(self, groups, nq, b_premultiplied=False, compact_keys=False):
        """groups: list of lists of (ext, b, evk, mask or None, galois[, mask_shift[, pt, pt_galois]]) -> y [n_out][2][nq+K][N];
        evk None: a term without a key switch, mask * P * (b, a) with the a-polynomial [nq][N] as ext."""
        import torch
        flat = [t for g in groups for t in g]
        flag = (lambda i: compact_keys[i]) if isinstance(compact_keys, (list, tuple)) else (lambda i: compact_keys)
        arr = (RotTerm * len(flat))()
        for i, (ext, b, evk, mask, gal, *more) in enumerate(flat):
            shift = more[0] if more else 0
            pt, pt_gal = (more[1], more[2]) if len(more) >= 3 else (None, 1)
            arr[i] = RotTerm(ext.data_ptr(), b.data_ptr() if b is not None else None, evk.data_ptr() if evk is not None else None,
                             mask.data_ptr() if mask is not None else None, gal, shift,
                             pt.data_ptr() if pt is not None else None, pt_gal, int(flag(i)))
        offs = [0]
        for g in groups:
            offs.append(offs[-1] + len(g))
        off = (ctypes.c_uint32 * len(offs))(*offs)
        y = torch.empty((len(groups), 2, nq + self.nP, self.N), dtype=torch.int64, device=flat[0][0].device)
        check(lib().hemm_hoisted_terms(self.h, arr, off, len(groups), nq, vp(y.data_ptr()), int(b_premultiplied), vp(0)))
        return y

    def hoisted_moddown(self, groups, nq, drop_last, b_premultiplied=False, compact_keys=False):
        """hoisted_terms + moddown_batch in one call -> [n_out][2][nq - drop_last][N]"""
        import torch
        flat = [t for g in groups for t in g]
        flag = (lambda i: compact_keys[i]) if isinstance(compact_keys, (list, tuple)) else (lambda i: compact_keys)
        arr = (RotTerm * len(flat))()
        for i, (ext, b, evk, mask, gal, *more) in enumerate(flat):
            shift = more[0] if more else 0
            pt, pt_gal = (more[1], more[2]) if len(more) >= 3 else (None, 1)
            arr[i] = RotTerm(ext.data_ptr(), b.data_ptr() if b is not None else None, evk.data_ptr() if evk is not None else None,
                             mask.data_ptr() if mask is not None else None, gal, shift,
                             pt.data_ptr() if pt is not None else None, pt_gal, int(flag(i)))
        offs = [0]
        for g in groups:
            offs.append(offs[-1] + len(g))
        off = (ctypes.c_uint32 * len(offs))(*offs)
        dev = flat[0][0].device
        nq_out = nq - 1 if drop_last else nq
        y = torch.empty((len(groups), 2, nq + self.nP, self.N), dtype=torch.int64, device=dev)
        out = torch.empty((len(groups), 2, nq_out, self.N), dtype=torch.int64, device=dev)
        ws = torch.empty_like(out)
        check(lib().hemm_hoisted_moddown(self.h, arr, off, len(groups), nq, int(b_premultiplied), int(drop_last),
                                         vp(y.data_ptr()), vp(out.data_ptr()), nq_out * self.N, vp(ws.data_ptr()), vp(0)))
        return out

    def moddown_batch(self, y, nq, drop_last, column_slab=False):
        """y: [..., nq+K, N] (clobbered) -> [..., nq - drop_last, N]; column_slab: the three-launch form
        (HEMM_MODDOWN_COLUMN_SLAB), same residues"""
        import torch
        n_polys = y.numel() // ((nq + self.nP) * self.N)
        nq_out = nq - 1 if drop_last else nq
        out = torch.empty(tuple(y.shape[:-2]) + (nq_out, self.N), dtype=torch.int64, device=y.device)
        ws = torch.empty_like(out)
        check(lib().hemm_moddown_batch(self.h, vp(y.data_ptr()), nq, n_polys, int(bool(drop_last)) | (2 if column_slab else 0),
                                       vp(out.data_ptr()), nq_out * self.N, vp(ws.data_ptr()), vp(0)))
        return out

    def masked_sum_batch(self, groups, nq, n_polys):
        """groups: list of lists of (ct [n_polys][>=nq][N], mask [>=nq][N] or None)"""
        import torch
        flat = [t for g in groups for t in g]
        arr = (LinTerm * len(flat))()
        for i, term in enumerate(flat):
            ct, mask = term[0], term[1]
            gal = term[2] if len(term) > 2 else 0
            arr[i] = LinTerm(ct.data_ptr(), mask.data_ptr() if mask is not None else None, ct.stride(0), gal)
        offs = [0]
        for g in groups:
            offs.append(offs[-1] + len(g))
        off = (ctypes.c_uint32 * len(offs))(*offs)
        out = torch.empty((len(groups), n_polys, nq, self.N), dtype=torch.int64, device=flat[0][0].device)
        check(lib().hemm_masked_sum_batch(self.h, arr, off, len(groups), nq, n_polys, vp(out.data_ptr()), vp(0)))
        return out

    def tensor_batch(self, t1, t2, nq, acc=None):
        import torch
        accumulate = acc is not None
        if acc is None:
            acc = torch.empty((3, nq, self.N), dtype=torch.int64, device=t1.device)
        check(lib().hemm_tensor_batch(self.h, vp(t1.data_ptr()), vp(t2.data_ptr()), t1.shape[0], nq,
                                      vp(acc.data_ptr()), int(accumulate), vp(0)))
        return acc

    def tensor_batch_groups(self, groups, nq, acc):
        """groups: list of (t1 [n_pairs][2][nq][N], t2 the same, index of the accumulator, accumulate) -- one launch;
        acc: [3][n_acc][nq][N], polynomial-major (accumulator i is acc[:, i])."""
        arr = (TensorGroup * len(groups))()
        for i, (t1, t2, idx, accumulate) in enumerate(groups):
            arr[i] = TensorGroup(t1.data_ptr(), t2.data_ptr(), acc[0, idx].data_ptr(), t1.shape[0], int(accumulate))
        check(lib().hemm_tensor_batch_groups(self.h, arr, len(groups), nq, acc.shape[1] * nq * self.N, vp(0)))
        return acc


ADD, SUB, MUL, NEG, MAC = 0, 1, 2, 3, 4


class Timer:
    """HIP-event stopwatch on the stream the kernels are launched on (default: the null stream)."""

    def __init__(self, stream=None):
        L = lib()
        L.hemm_timer_create.argtypes = [ctypes.POINTER(vp)]
        L.hemm_timer_start.argtypes = [vp, vp]
        L.hemm_timer_stop.argtypes = [vp, vp, ctypes.POINTER(ctypes.c_float)]
        L.hemm_timer_destroy.argtypes = [vp]
        self.t = vp()
        self.stream = vp(stream or 0)
        check(L.hemm_timer_create(ctypes.byref(self.t)))

    def start(self):
        check(lib().hemm_timer_start(self.t, self.stream))

    def stop(self):
        ms = ctypes.c_float()
        check(lib().hemm_timer_stop(self.t, self.stream, ctypes.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            lib().hemm_timer_destroy(self.t)
        except Exception:
            pass


def primes_below(bits, log_n, count):
    out = (ctypes.c_uint64 * count)()
    check(lib().hemm_primes_below(bits, log_n, count, out))
    return list(out)

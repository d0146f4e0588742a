"""TEST INFRASTRUCTURE ONLY -- Python driver over the CPU oracle (oracle/liboracle.so).

Provides the RNS-CKKS objects and evaluator operations that HEMMer's matrix
multiplication issues against HEaaN (ciphertext/external/include/HEaaN/HomEvaluator.hpp:
add :144, sub :223, mult :257-311, multWithoutRescale :478-491, tensor :518, relinearize
:524, rescale :540, levelDown :575, leftRotate/rightRotate :370-403, conjugate :465,
multImagUnit :330, multInteger :347, matmul :600; EnDecoder.hpp:51-66; Encryptor.hpp:84;
Decryptor.hpp:36; KeyGenerator.hpp:69-89).  HEaaN is closed source, so the arithmetic is
the published RNS-CKKS one; see ckks_oracle.cpp for what pins it.

Only tests, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this.
"""
import ctypes
import math
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

u64p = ctypes.POINTER(ctypes.c_uint64)
i64p = ctypes.POINTER(ctypes.c_int64)
i32p = ctypes.POINTER(ctypes.c_int)
f64p = ctypes.POINTER(ctypes.c_double)


def build(force=False):
    so = os.path.join(_HERE, "liboracle.so")
    src = os.path.join(_HERE, "ckks_oracle.cpp")
    if force or not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"],
                              stdout=subprocess.DEVNULL)
    return so


def lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(so):
            build()
        L = ctypes.CDLL(so)
        L.orc_create.restype = ctypes.c_void_p
        L.orc_create.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, u64p, ctypes.c_int]
        L.orc_destroy.argtypes = [ctypes.c_void_p]
        L.orc_psi.restype = ctypes.c_uint64
        L.orc_psi.argtypes = [ctypes.c_void_p, ctypes.c_int]
        L.orc_alpha.argtypes = [ctypes.c_void_p]
        L.orc_set_threads.argtypes = [ctypes.c_void_p, ctypes.c_int]
        L.orc_sm64.restype = ctypes.c_uint64
        L.orc_sm64.argtypes = [ctypes.c_uint64]
        L.orc_stream_key.restype = ctypes.c_uint64
        L.orc_stream_key.argtypes = [ctypes.c_uint64] * 4
        L.orc_sample_uniform.argtypes = [ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int, u64p]
        L.orc_sample_ternary.argtypes = [ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int, i32p]
        L.orc_sample_error.argtypes = [ctypes.c_void_p, ctypes.c_uint64, i32p]
        L.orc_lift_small.argtypes = [ctypes.c_void_p, i32p, ctypes.c_int, u64p]
        L.orc_ntt.argtypes = [ctypes.c_void_p, u64p, ctypes.c_int, ctypes.c_int]
        L.orc_ntt_batch.argtypes = [ctypes.c_void_p, u64p, i32p, ctypes.c_int, ctypes.c_int,
                                    ctypes.c_int, ctypes.c_int]
        L.orc_pointwise.argtypes = [ctypes.c_void_p, ctypes.c_int, u64p, u64p, u64p, ctypes.c_int]
        L.orc_mul_scalar.argtypes = [ctypes.c_void_p, u64p, ctypes.c_uint64, u64p, ctypes.c_int]
        L.orc_mul_imag_unit.argtypes = [ctypes.c_void_p, u64p, u64p, ctypes.c_int]
        L.orc_automorphism_coeff.argtypes = [ctypes.c_void_p, u64p, u64p, ctypes.c_uint64,
                                             ctypes.c_int]
        L.orc_automorphism_ntt.argtypes = [ctypes.c_void_p, u64p, u64p, ctypes.c_uint64]
        L.orc_modup.argtypes = [ctypes.c_void_p, u64p, ctypes.c_int, u64p]
        L.orc_inner_product.argtypes = [ctypes.c_void_p, u64p, u64p, ctypes.c_int, u64p]
        L.orc_moddown.argtypes = [ctypes.c_void_p, u64p, ctypes.c_int, u64p]
        L.orc_keyswitch.argtypes = [ctypes.c_void_p, u64p, u64p, ctypes.c_int, u64p, u64p]
        L.orc_rescale.argtypes = [ctypes.c_void_p, u64p, ctypes.c_int, u64p]
        L.orc_hoisted_term.argtypes = [ctypes.c_void_p, u64p, u64p, u64p, u64p, ctypes.c_uint64,
                                       ctypes.c_int, u64p, ctypes.c_int]
        L.orc_moddown_drop.argtypes = [ctypes.c_void_p, u64p, ctypes.c_int, ctypes.c_int, u64p]
        L.orc_tensor.argtypes = [ctypes.c_void_p, u64p, u64p, ctypes.c_int, u64p]
        L.orc_encode_coeffs.argtypes = [ctypes.c_void_p, f64p, ctypes.c_double, i64p]
        L.orc_decode_coeffs.argtypes = [ctypes.c_void_p, f64p, f64p]
        L.orc_lift_i64.argtypes = [ctypes.c_void_p, i64p, ctypes.c_int, u64p]
        L.orc_crt_to_double.argtypes = [ctypes.c_void_p, u64p, u64p, ctypes.c_int,
                                        ctypes.c_double, f64p]
        _LIB = L
    return _LIB


def _p(a, t=u64p):
    return a.ctypes.data_as(t)


# --------------------------------------------------------------------------------------
# primes (Python big-int arithmetic; independent of the C++ side)
# --------------------------------------------------------------------------------------
_MR_BASES = (2, 3, 5, 7, 11, 13, 17, 19, 23, 29, 31, 37)


def is_prime(n):
    if n < 2:
        return False
    for p in _MR_BASES:
        if n % p == 0:
            return n == p
    d, s = n - 1, 0
    while d % 2 == 0:
        d //= 2
        s += 1
    for a in _MR_BASES:
        x = pow(a, d, n)
        if x in (1, n - 1):
            continue
        for _ in range(s - 1):
            x = x * x % n
            if x == n - 1:
                break
        else:
            return False
    return True


def primes_below(bits, log_n, count, skip=()):
    """The `count` largest primes p < 2^bits with p = 1 (mod 2N), descending."""
    m = 2 << log_n
    p = (1 << bits) - ((1 << bits) % m) + 1
    while p >= (1 << bits):
        p -= m
    out = []
    while len(out) < count:
        if is_prime(p) and p not in skip:
            out.append(p)
        p -= m
    return out


def nearest_prime(target, log_n, skip=()):
    """Prime p = 1 (mod 2N) closest to `target` (ties go down), not in `skip`."""
    m = 2 << log_n
    base = int(target) - (int(target) % m) + 1
    k = 0
    while True:
        cands = [base - k * m, base + (k + 1) * m] if k else [base, base + m]
        cands = sorted(set(cands), key=lambda c: (abs(c - target), c))
        for c in cands:
            if c > 2 and c not in skip and is_prime(c):
                # make sure nothing closer was skipped over on the other side
                return c
        k += 1


def ckks_chain(log_n, n_q, n_p, base_bits=60, scale_bits=42, special_bits=60):
    """q_0 ~ 2^base_bits, q_1..q_L chosen top-down so the per-level scale
    Delta_{l-1} = Delta_l^2 / q_l stays next to 2^scale_bits, then n_p special primes."""
    q0 = primes_below(base_bits, log_n, 1)[0]
    used = {q0}
    L = n_q - 1
    qs = [0] * n_q
    qs[0] = q0
    delta = float(1 << scale_bits)
    for l in range(L, 0, -1):
        target = delta * delta / float(1 << scale_bits)
        q = nearest_prime(target, log_n, used)
        used.add(q)
        qs[l] = q
        delta = delta * delta / float(q)
    ps = primes_below(special_bits, log_n, n_p, skip=used)
    return qs, ps


# --------------------------------------------------------------------------------------
# objects
# --------------------------------------------------------------------------------------
class Ct:
    """Ciphertext: data[poly][limb][N] (NTT form), level = limbs-1, scale (float)."""

    def __init__(self, data, scale):
        self.data = data
        self.scale = scale

    @property
    def level(self):
        return self.data.shape[1] - 1

    @property
    def nq(self):
        return self.data.shape[1]

    def copy(self):
        return Ct(self.data.copy(), self.scale)


class Pt:
    """Plaintext: data[limb][N] (NTT form)."""

    def __init__(self, data, scale):
        self.data = data
        self.scale = scale

    @property
    def level(self):
        return self.data.shape[0] - 1

    def copy(self):
        return Pt(self.data.copy(), self.scale)


TAG_SK, TAG_EVK_A, TAG_EVK_E, TAG_ENC_A, TAG_ENC_E = 1, 2, 3, 4, 5


class Oracle:
    """Context + secret key + evaluator on the CPU."""

    def __init__(self, log_n, q_primes, p_primes, dnum, log_scale=42, threads=1):
        self.L = lib()
        self.log_n = log_n
        self.N = 1 << log_n
        self.slots = self.N // 2
        self.q = [int(x) for x in q_primes]
        self.p = [int(x) for x in p_primes]
        self.nQ, self.nP, self.dnum = len(self.q), len(self.p), dnum
        self.mods = self.q + self.p
        arr = (ctypes.c_uint64 * len(self.mods))(*self.mods)
        self.h = self.L.orc_create(log_n, self.nQ, self.nP, arr, dnum)
        self.alpha = self.L.orc_alpha(self.h)
        self.threads = threads
        self.L.orc_set_threads(self.h, threads)
        # fixed per-level scale: Delta_L = 2^log_scale, Delta_{l-1} = Delta_l^2 / q_l
        self.delta = [0.0] * self.nQ
        self.delta[self.nQ - 1] = float(1 << log_scale)
        for l in range(self.nQ - 1, 0, -1):
            self.delta[l - 1] = self.delta[l] * self.delta[l] / float(self.q[l])
        self.sk = None
        self.keys = {}

    def __del__(self):
        try:
            self.L.orc_destroy(self.h)
        except Exception:
            pass

    # ---- helpers -----------------------------------------------------------------
    def prime_of(self, j, nq):
        return j if j < nq else self.nQ + (j - nq)

    def ntt(self, data, primes, inverse=False):
        """In-place batched transform of data[..., limb, N]; primes = prime index per limb."""
        d = np.ascontiguousarray(data)
        assert d is data or d.base is data or True
        n_limbs = len(primes)
        n_polys = d.size // (n_limbs * self.N)
        idx = np.asarray(primes, dtype=np.int32)
        self.L.orc_ntt_batch(self.h, _p(d), _p(idx, i32p), n_limbs, n_polys, int(inverse),
                             self.threads)
        if d is not data:
            data[...] = d
        return data

    def galois(self, r):
        """Galois element of a left rotation by r slots."""
        return pow(5, r % self.slots, 2 * self.N)

    # ---- sampling ----------------------------------------------------------------
    def stream(self, seed, tag, a=0, b=0):
        return self.L.orc_stream_key(seed, tag, a, b)

    def uniform(self, key, prime_idx):
        out = np.empty(self.N, dtype=np.uint64)
        self.L.orc_sample_uniform(self.h, key, prime_idx, _p(out))
        return out

    def ternary(self, key, hw):
        out = np.empty(self.N, dtype=np.int32)
        self.L.orc_sample_ternary(self.h, key, hw, _p(out, i32p))
        return out

    def error(self, key):
        out = np.empty(self.N, dtype=np.int32)
        self.L.orc_sample_error(self.h, key, _p(out, i32p))
        return out

    def small_to_ntt(self, v, prime_indices):
        """Small signed coefficient vector -> NTT form for each prime: [len][N]."""
        v = np.ascontiguousarray(v, dtype=np.int32)
        out = np.empty((len(prime_indices), self.N), dtype=np.uint64)
        for j, pi in enumerate(prime_indices):
            self.L.orc_lift_small(self.h, _p(v, i32p), pi, _p(out[j]))
        self.ntt(out, prime_indices)
        return out

    # ---- keys --------------------------------------------------------------------
    def gen_secret(self, seed, hw=192):
        self.sk_coeffs = self.ternary(self.stream(seed, TAG_SK), min(hw, self.N // 2))
        self.sk = self.small_to_ntt(self.sk_coeffs, list(range(self.nQ + self.nP)))
        return self.sk

    def _gen_switch_key(self, seed, key_id, s_from):
        """evk[d] = (b_d, a_d) over all nQ+nP primes (NTT form):
        b_d = -a_d*s + e_d + [P mod q_i]*s_from on the limbs of digit d, -a_d*s + e_d elsewhere."""
        tot = self.nQ + self.nP
        evk = np.empty((self.dnum, 2, tot, self.N), dtype=np.uint64)
        P = 1
        for p in self.p:
            P *= p
        def limb(d, i, e_i):
            tmp = np.empty(self.N, dtype=np.uint64)
            a = self.uniform(self.stream(seed, TAG_EVK_A, key_id, d * tot + i), i)
            evk[d, 1, i] = a
            self.L.orc_pointwise(self.h, 2, _p(a), _p(self.sk[i]), _p(tmp), i)   # a*s
            self.L.orc_pointwise(self.h, 1, _p(e_i), _p(tmp), _p(evk[d, 0, i]), i)  # e - a*s
            if i < self.nQ and d * self.alpha <= i < (d + 1) * self.alpha:
                self.L.orc_mul_scalar(self.h, _p(s_from[i]), P % self.mods[i], _p(tmp), i)
                self.L.orc_pointwise(self.h, 0, _p(evk[d, 0, i]), _p(tmp), _p(evk[d, 0, i]), i)

        for d in range(self.dnum):
            e = self.small_to_ntt(self.error(self.stream(seed, TAG_EVK_E, key_id, d)),
                                  list(range(tot)))
            self._for_each(lambda i: limb(d, i, e[i]), range(tot))
        return evk

    def gen_mult_key(self, seed):
        tot = self.nQ + self.nP
        s2 = np.empty_like(self.sk)
        for i in range(tot):
            self.L.orc_pointwise(self.h, 2, _p(self.sk[i]), _p(self.sk[i]), _p(s2[i]), i)
        self.keys["mult"] = self._gen_switch_key(seed, 0, s2)

    def _for_each(self, fn, items):
        """fn over independent items (limbs), on self.threads worker threads (ctypes calls release the GIL)."""
        items = list(items)
        if self.threads <= 1 or len(items) <= 1:
            for it in items:
                fn(it)
            return
        from concurrent.futures import ThreadPoolExecutor
        with ThreadPoolExecutor(max_workers=min(self.threads, len(items))) as ex:
            list(ex.map(fn, items))

    def _sk_automorphism(self, g):
        out = np.empty_like(self.sk)
        self._for_each(lambda i: self.L.orc_automorphism_ntt(self.h, _p(self.sk[i]), _p(out[i]), g),
                       range(self.nQ + self.nP))
        return out

    def gen_rot_key(self, seed, r):
        """Key for a left rotation by r slots (key id = Galois element)."""
        g = self.galois(r)
        if ("gal", g) not in self.keys:
            self.keys[("gal", g)] = self._gen_switch_key(seed, g, self._sk_automorphism(g))

    def gen_rot_square_key(self, seed, g):
        """Key switching rho_g(s)^2 -> s (key id = Galois element with bit 40 set): rotates the degree-2
        component of an un-relinearised product directly."""
        if ("galsq", g) not in self.keys:
            tot = self.nQ + self.nP
            s2 = np.empty_like(self.sk)
            for i in range(tot):
                self.L.orc_pointwise(self.h, 2, _p(self.sk[i]), _p(self.sk[i]), _p(s2[i]), i)
            sg = np.empty_like(s2)
            for i in range(tot):
                self.L.orc_automorphism_ntt(self.h, _p(s2[i]), _p(sg[i]), g)
            self.keys[("galsq", g)] = self._gen_switch_key(seed, (1 << 40) | g, sg)
        return self.keys[("galsq", g)]

    def gen_conj_key(self, seed):
        g = 2 * self.N - 1
        self.keys[("gal", g)] = self._gen_switch_key(seed, g, self._sk_automorphism(g))

    # ---- encode / decode / encrypt / decrypt -------------------------------------------
    def encode(self, msg, level, scale=None):
        """msg: complex vector of N/2 slots -> Pt at `level` with scale Delta_level."""
        if scale is None:
            scale = self.delta[level]
        z = np.zeros(self.slots, dtype=np.complex128)
        m = np.asarray(msg)
        z[: m.size] = m.reshape(-1)
        sl = np.ascontiguousarray(z.view(np.float64))
        co = np.empty(self.N, dtype=np.int64)
        self.L.orc_encode_coeffs(self.h, _p(sl, f64p), float(scale), _p(co, i64p))
        out = np.empty((level + 1, self.N), dtype=np.uint64)
        for j in range(level + 1):
            self.L.orc_lift_i64(self.h, _p(co, i64p), j, _p(out[j]))
        self.ntt(out, list(range(level + 1)))
        return Pt(out, float(scale))

    def decode(self, pt):
        d = pt.data[: min(2, pt.data.shape[0])].copy()
        self.ntt(d, list(range(d.shape[0])), inverse=True)
        co = np.empty(self.N, dtype=np.float64)
        two = int(d.shape[0] > 1)
        self.L.orc_crt_to_double(self.h, _p(d[0]), _p(d[1] if two else d[0]), two,
                                 float(pt.scale), _p(co, f64p))
        sl = np.empty(self.N, dtype=np.float64)
        self.L.orc_decode_coeffs(self.h, _p(co, f64p), _p(sl, f64p))
        return sl.view(np.complex128).copy()

    def encrypt(self, pt, seed):
        """Secret-key encryption: (b, a) with b = -a*s + e + m  (Encryptor.hpp:81)."""
        nq = pt.data.shape[0]
        ct = np.empty((2, nq, self.N), dtype=np.uint64)
        e = self.small_to_ntt(self.error(self.stream(seed, TAG_ENC_E)), list(range(nq)))
        tmp = np.empty(self.N, dtype=np.uint64)
        for i in range(nq):
            a = self.uniform(self.stream(seed, TAG_ENC_A, i), i)
            ct[1, i] = a
            self.L.orc_pointwise(self.h, 2, _p(a), _p(self.sk[i]), _p(tmp), i)
            self.L.orc_pointwise(self.h, 1, _p(e[i]), _p(tmp), _p(ct[0, i]), i)
            self.L.orc_pointwise(self.h, 0, _p(ct[0, i]), _p(pt.data[i]), _p(ct[0, i]), i)
        return Ct(ct, pt.scale)

    def decrypt_pt(self, ct):
        nq = min(2, ct.nq)
        out = np.empty((nq, self.N), dtype=np.uint64)
        tmp = np.empty(self.N, dtype=np.uint64)
        for i in range(nq):
            self.L.orc_pointwise(self.h, 2, _p(ct.data[1, i]), _p(self.sk[i]), _p(tmp), i)
            self.L.orc_pointwise(self.h, 0, _p(ct.data[0, i]), _p(tmp), _p(out[i]), i)
            if ct.data.shape[0] == 3:
                s2 = np.empty(self.N, dtype=np.uint64)
                self.L.orc_pointwise(self.h, 2, _p(self.sk[i]), _p(self.sk[i]), _p(s2), i)
                self.L.orc_pointwise(self.h, 4, _p(ct.data[2, i]), _p(s2), _p(out[i]), i)
        return Pt(out, ct.scale)

    def decrypt(self, ct):
        return self.decode(self.decrypt_pt(ct))

    # ---- evaluator ------------------------------------------------------------------------
    def _binary(self, op, a, b):
        nq = min(a.shape[-2], b.shape[-2])
        a2 = a[..., :nq, :]
        b2 = b[..., :nq, :]
        out = np.empty(np.broadcast_shapes(a2.shape, b2.shape), dtype=np.uint64)
        a3 = np.broadcast_to(a2, out.shape)
        b3 = np.broadcast_to(b2, out.shape)
        flat_o = out.reshape(-1, nq, self.N)
        flat_a = np.ascontiguousarray(a3).reshape(-1, nq, self.N)
        flat_b = np.ascontiguousarray(b3).reshape(-1, nq, self.N)
        for k in range(flat_o.shape[0]):
            for i in range(nq):
                self.L.orc_pointwise(self.h, op, _p(flat_a[k, i]), _p(flat_b[k, i]),
                                     _p(flat_o[k, i]), i)
        return out

    def add(self, x, y):
        """ct+ct or ct+pt (pt adds to the b polynomial). Levels drop to the lower operand."""
        if isinstance(y, Pt):
            nq = min(x.nq, y.data.shape[0])
            out = x.data[:, :nq].copy()
            out[0] = self._binary(0, out[0], y.data[:nq])
            return Ct(out, x.scale)
        np_ = max(x.data.shape[0], y.data.shape[0])
        nq = min(x.nq, y.nq)
        out = np.zeros((np_, nq, self.N), dtype=np.uint64)
        out[: x.data.shape[0]] = x.data[:, :nq]
        k = y.data.shape[0]
        out[:k] = self._binary(0, out[:k], y.data[:, :nq])
        return Ct(out, x.scale)

    def sub(self, x, y):
        nq = min(x.nq, y.nq)
        return Ct(self._binary(1, x.data[:, :nq], y.data[:, :nq]), x.scale)

    def negate(self, x):
        z = np.zeros_like(x.data)
        return Ct(self._binary(1, z, x.data), x.scale)

    def mult_plain_no_rescale(self, x, pt):
        nq = min(x.nq, pt.data.shape[0])
        return Ct(self._binary(2, x.data[:, :nq], pt.data[None, :nq]), x.scale * pt.scale)

    def mult_scalar_residues(self, x, value):
        """Multiply every residue by the integer `value` (may be negative)."""
        out = np.empty_like(x.data)
        for k in range(x.data.shape[0]):
            for i in range(x.nq):
                self.L.orc_mul_scalar(self.h, _p(x.data[k, i]), int(value) % self.mods[i],
                                      _p(out[k, i]), i)
        return out

    def add_constant_residues(self, data, c, level):
        """data [polys][nq][N] + the NTT form of round(re Delta_level) + round(im Delta_level) X^(N/2) on polynomial 0:
        slot k of limb j gets re + im psi_j^(N/2) (-1)^(bitrev(k) & 1), i.e. the sign flips on the upper half."""
        def rnd(v):
            return int(math.floor(abs(v) + 0.5)) * (1 if v >= 0 else -1)      # llround: halves away from zero
        re, im = rnd(c.real * self.delta[level]), rnd(c.imag * self.delta[level])
        out = data.copy()
        nq = out.shape[1]
        cols = np.empty((nq, self.N), dtype=np.uint64)
        for j in range(nq):
            cols[j] = re % int(self.q[j])
        if im != 0:
            v = np.empty((nq, self.N), dtype=np.uint64)
            w = np.empty_like(v)
            for j in range(nq):
                v[j] = im % int(self.q[j])
                self.L.orc_mul_imag_unit(self.h, _p(v[j]), _p(w[j]), j)      # im X^(N/2) in NTT form
            cols = self._binary(0, cols, w)
        out[0] = self._binary(0, np.ascontiguousarray(out[0]), cols)
        return out

    def add_residues(self, a, b):
        """Limb-wise a + b of residue arrays [nq][N] over the chain primes 0 .. nq-1."""
        return self._binary(0, a, b)

    def mul_p_residues(self, a):
        """a [nq][N] times P = product of the special primes, limb-wise."""
        P = 1
        for p in self.p:
            P *= p
        out = np.empty_like(a)
        for i in range(a.shape[0]):
            self.L.orc_mul_scalar(self.h, _p(np.ascontiguousarray(a[i])), P % self.mods[i], _p(out[i]), i)
        return out

    def mult_integer(self, x, value):
        return Ct(self.mult_scalar_residues(x, value), x.scale)

    def mult_const(self, x, c):
        """ct * real constant: multiply by round(c*Delta_level) and rescale."""
        v = int(round(c * self.delta[x.level]))
        return self.rescale(Ct(self.mult_scalar_residues(x, v), x.scale * self.delta[x.level]))

    def mult_imag_unit(self, x):
        out = np.empty_like(x.data)
        for k in range(x.data.shape[0]):
            for i in range(x.nq):
                self.L.orc_mul_imag_unit(self.h, _p(x.data[k, i]), _p(out[k, i]), i)
        return Ct(out, x.scale)

    def tensor(self, x, y):
        nq = min(x.nq, y.nq)
        a = np.ascontiguousarray(x.data[:2, :nq])
        b = np.ascontiguousarray(y.data[:2, :nq])
        out = np.empty((3, nq, self.N), dtype=np.uint64)
        self.L.orc_tensor(self.h, _p(a), _p(b), nq, _p(out))
        return Ct(out, x.scale * y.scale)

    def keyswitch(self, poly, evk):
        nq = poly.shape[0]
        p = np.ascontiguousarray(poly)
        ob = np.empty((nq, self.N), dtype=np.uint64)
        oa = np.empty((nq, self.N), dtype=np.uint64)
        self.L.orc_keyswitch(self.h, _p(p), _p(evk), nq, _p(ob), _p(oa))
        return ob, oa

    def relinearize(self, x):
        ob, oa = self.keyswitch(x.data[2], self.keys["mult"])
        out = np.empty((2, x.nq, self.N), dtype=np.uint64)
        out[0] = self._binary(0, x.data[0], ob)
        out[1] = self._binary(0, x.data[1], oa)
        return Ct(out, x.scale)

    def rescale(self, x):
        nq = x.nq
        out = np.empty((x.data.shape[0], nq - 1, self.N), dtype=np.uint64)
        for k in range(x.data.shape[0]):
            src = np.ascontiguousarray(x.data[k])
            self.L.orc_rescale(self.h, _p(src), nq, _p(out[k]))
        return Ct(out, x.scale / float(self.q[nq - 1]))

    def mult(self, x, y):
        if isinstance(y, Pt):
            return self.rescale(self.mult_plain_no_rescale(x, y))
        return self.rescale(self.relinearize(self.tensor(x, y)))

    def mult_msg(self, x, msg):
        return self.mult(x, self.encode(msg, x.level))

    def apply_galois(self, x, g):
        """Automorphism on both polynomials + key switch of the a part."""
        nq = x.nq
        rb = np.empty((nq, self.N), dtype=np.uint64)
        ra = np.empty((nq, self.N), dtype=np.uint64)
        for i in range(nq):
            self.L.orc_automorphism_ntt(self.h, _p(np.ascontiguousarray(x.data[0, i])), _p(rb[i]), g)
            self.L.orc_automorphism_ntt(self.h, _p(np.ascontiguousarray(x.data[1, i])), _p(ra[i]), g)
        if ("gal", g) not in self.keys and getattr(self, "key_seed", None) is not None:
            # keys are a deterministic function of (seed, Galois element): derive on first use
            self.keys[("gal", g)] = self._gen_switch_key(self.key_seed, g, self._sk_automorphism(g))
        ob, oa = self.keyswitch(ra, self.keys[("gal", g)])
        out = np.empty((2, nq, self.N), dtype=np.uint64)
        out[0] = self._binary(0, rb, ob)
        out[1] = oa
        return Ct(out, x.scale)

    def left_rotate(self, x, r):
        r %= self.slots
        if r == 0:
            return x.copy()
        if isinstance(x, Pt):
            out = np.empty_like(x.data)
            g = self.galois(r)
            for i in range(x.data.shape[0]):
                self.L.orc_automorphism_ntt(self.h, _p(np.ascontiguousarray(x.data[i])),
                                            _p(out[i]), g)
            return Pt(out, x.scale)
        return self.apply_galois(x, self.galois(r))

    def right_rotate(self, x, r):
        return self.left_rotate(x, (self.slots - r % self.slots) % self.slots)

    def conjugate(self, x):
        return self.apply_galois(x, 2 * self.N - 1)

    def level_down(self, x, target):
        """Drop to `target`, keeping the fixed per-level scale: truncate to target+1 limbs,
        multiply by round(Delta_target * q_{target+1} / scale) and rescale."""
        if x.level == target:
            return x.copy()
        assert x.level > target
        t = Ct(np.ascontiguousarray(x.data[:, : target + 2]), x.scale)
        c = int(math.floor(self.delta[target] * float(self.q[target + 1]) / x.scale + 0.5))
        t = Ct(self.mult_scalar_residues(t, c), t.scale * c)
        r = self.rescale(t)
        r.scale = self.delta[target]
        return r

    def level_down_one(self, x):
        return self.level_down(x, x.level - 1)

    # ---- hoisted / merged forms (what the batched GPU launches compute) -------------------------
    def ext_primes(self, level):
        """Prime indices of the extended basis at `level`: q_0..q_level, then the special primes."""
        return list(range(level + 1)) + [self.nQ + k for k in range(self.nP)]

    def ext_plain_product(self, mask, pt, g):
        """mask * (pt read through the automorphism X -> X^g), limb-wise over the extended basis: the plaintext
        factor a hoisted term applies when it carries both a mask and a rotated plaintext (mask None: factor 1)."""
        level = pt.data.shape[0] - self.nP - 1
        out = np.empty_like(pt.data)
        for j, pi in enumerate(self.ext_primes(level)):
            rot = np.empty(self.N, dtype=np.uint64)
            self.L.orc_automorphism_ntt(self.h, _p(np.ascontiguousarray(pt.data[j])), _p(rot), int(g))
            if mask is None:
                out[j] = rot
            else:
                self.L.orc_pointwise(self.h, 2, _p(np.ascontiguousarray(mask.data[j])), _p(rot), _p(out[j]), pi)
        return Pt(out, pt.scale * (mask.scale if mask is not None else 1.0))

    def encode_ext(self, msg, level, scale=None):
        """Plaintext over the extended basis: limbs q_0..q_level then the special primes (scale: the level's fixed
        scale unless given)."""
        z = np.zeros(self.slots, dtype=np.complex128)
        m = np.asarray(msg)
        z[: m.size] = m.reshape(-1)
        sl = np.ascontiguousarray(z.view(np.float64))
        co = np.empty(self.N, dtype=np.int64)
        scale = self.delta[level] if scale is None else scale
        self.L.orc_encode_coeffs(self.h, _p(sl, f64p), float(scale), _p(co, i64p))
        primes = list(range(level + 1)) + [self.nQ + k for k in range(self.nP)]
        out = np.empty((len(primes), self.N), dtype=np.uint64)
        for j, pi in enumerate(primes):
            self.L.orc_lift_i64(self.h, _p(co, i64p), pi, _p(out[j]))
        self.ntt(out, primes)
        return Pt(out, float(scale))

    def modup(self, poly):
        nq = poly.shape[0]
        beta = (nq + self.alpha - 1) // self.alpha
        ext = np.empty((beta, nq + self.nP, self.N), dtype=np.uint64)
        self.L.orc_modup(self.h, _p(np.ascontiguousarray(poly)), nq, _p(ext))
        return ext

    def galois_key(self, g):
        if ("gal", g) not in self.keys and getattr(self, "key_seed", None) is not None:
            self.keys[("gal", g)] = self._gen_switch_key(self.key_seed, g, self._sk_automorphism(g))
        return self.keys[("gal", g)]

    def hoisted_sum(self, terms, nq):
        """terms: (ext, b or None, rotation r (left, in slots) or ('g', galois) or ('sq', galois): the key of
        rho_g(s)^2, or ('mult', 1): the multiplication key without rotation, or ('none',): no key switch at all, ext
        being the a-polynomial on the chain limbs; mask Pt over the extended basis or None).
        Returns y[2][nq+K][N] = sum mask * (<galois(ext), evk> + P galois(b))."""
        y = np.zeros((2, nq + self.nP, self.N), dtype=np.uint64)
        keyless = [t for t in terms if isinstance(t[2], tuple) and t[2][0] == "none"]
        terms = [t for t in terms if not (isinstance(t[2], tuple) and t[2][0] == "none")]
        for i, (ext, b, rot, mask) in enumerate(terms):
            g = rot[1] if isinstance(rot, tuple) else self.galois(rot)
            if isinstance(rot, tuple) and rot[0] == "sq":
                evk = self.gen_rot_square_key(self.key_seed, g)
            elif isinstance(rot, tuple) and rot[0] == "mult":      # the multiplication key, identity automorphism
                evk, g = self.keys["mult"], 1
            else:
                evk = self.galois_key(g)
            mk = _p(np.ascontiguousarray(mask.data)) if mask is not None else None
            bp = _p(np.ascontiguousarray(b)) if b is not None else None
            self.L.orc_hoisted_term(self.h, _p(np.ascontiguousarray(ext)), bp,
                                    _p(evk), mk, g, nq, _p(y), int(i > 0))
        # ('none',): a term without a key switch -- ext is the a-polynomial [nq][N] itself and the term is
        # mask * P * (b, a) on the chain limbs (exact residue arithmetic: where it joins the sum does not matter)
        for a, b, _, mask in keyless:
            for pol, src in ((0, b), (1, a)):
                if src is None:
                    continue
                t = self.mul_p_residues(np.ascontiguousarray(src[:nq]))
                if mask is not None:
                    t = self._binary(2, t, np.ascontiguousarray(mask.data[:nq]))
                y[pol, :nq] = self.add_residues(np.ascontiguousarray(y[pol, :nq]), t)
        return y

    def moddown_drop(self, y, nq, drop_last):
        nq_out = nq - 1 if drop_last else nq
        out = np.empty((y.shape[0], nq_out, self.N), dtype=np.uint64)
        for p in range(y.shape[0]):
            self.L.orc_moddown_drop(self.h, _p(np.ascontiguousarray(y[p])), nq, int(drop_last), _p(out[p]))
        return out

    def rotate_hoisted(self, x, r):
        """Rotation with the automorphism applied after ModUp (the order the batched launches use)."""
        r %= self.slots
        if r == 0:
            return x.copy()
        ext = self.modup(x.data[1])
        y = self.hoisted_sum([(ext, x.data[0], r, None)], x.nq)
        return Ct(self.moddown_drop(y, x.nq, False), x.scale)

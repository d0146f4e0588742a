"""ctypes binding of the HEMMer facade (include/hellm.h): the Python mirror of HELLM::HEMMer used by
the tests and bench.py.  Matrices are numpy float64 arrays; tensors are opaque device handles."""
import ctypes

import numpy as np

from . import check, lib

vp = ctypes.c_void_p
u32 = ctypes.c_uint32
u64 = ctypes.c_uint64
f64p = ctypes.POINTER(ctypes.c_double)
u64p = ctypes.POINTER(ctypes.c_uint64)
u32p = ctypes.POINTER(ctypes.c_uint32)
_declared = False


def _L():
    global _declared
    L = lib()
    if not _declared:
        pvp = ctypes.POINTER(vp)
        L.hellm_hemmer_create.argtypes = [u32, u32, u32, u64p, u32, u32, u32, u64, pvp]
        L.hellm_hemmer_create_preset.argtypes = [u64, pvp]
        L.hellm_hemmer_destroy.argtypes = [vp]
        L.hellm_hemmer_info.argtypes = [vp, u32p, u32p, u32p, u32p, u32p, u64p]
        L.hellm_secret_coeffs.argtypes = [vp, ctypes.POINTER(ctypes.c_int32)]
        L.hellm_export_key.argtypes = [vp, u64, u64p]
        L.hellm_ensure_rotation_keys.argtypes = [vp, u64p, u32]
        L.hellm_set_schedule.argtypes = [vp, ctypes.c_int, u32]
        L.hellm_graph_begin.argtypes = [vp]
        L.hellm_graph_end.argtypes = [vp, pvp]
        L.hellm_graph_launch.argtypes = [vp]
        L.hellm_graph_sync.argtypes = [vp]
        L.hellm_graph_nodes.argtypes = [vp, ctypes.POINTER(ctypes.c_uint64)]
        L.hellm_graph_destroy.argtypes = [vp]
        L.hellm_graph_destroy.restype = None
        L.hellm_key_bytes.argtypes = [vp] + [ctypes.POINTER(ctypes.c_uint64)] * 3
        L.hellm_phase_trace.argtypes = [vp, ctypes.c_int]
        L.hellm_phase_report.argtypes = [vp, ctypes.c_char_p, ctypes.c_size_t]
        L.hellm_assume_single_tile.argtypes = [vp, ctypes.c_int]
        L.hellm_traffic.argtypes = [vp, ctypes.POINTER(ctypes.c_uint64), ctypes.POINTER(ctypes.c_uint64), ctypes.c_int]
        L.hellm_encrypt.argtypes = [vp, f64p, u32, u32, pvp]
        L.hellm_encrypt2.argtypes = [vp, f64p, f64p, u32, u32, pvp]
        L.hellm_encode.argtypes = [vp, f64p, u32, u32, u32, pvp]
        L.hellm_encode2.argtypes = [vp, f64p, f64p, u32, u32, u32, pvp]
        L.hellm_encode_diagonal_to_row4.argtypes = [vp, f64p, f64p, f64p, f64p, u32, u32, u32, pvp]
        L.hellm_decrypt.argtypes = [vp, vp, f64p]
        L.hellm_decrypt2.argtypes = [vp, vp, f64p]
        L.hellm_decrypt_slots.argtypes = [vp, vp, f64p]
        L.hellm_ct_info.argtypes = [vp, u32p, u32p, u32p, u32p, u32p, u32p]
        L.hellm_ct_download.argtypes = [vp, u64p]
        L.hellm_ct_upload.argtypes = [vp, u64p, u32, u32, u32, u32, u32, u32, pvp]
        L.hellm_ct_clone.argtypes = [vp, pvp]
        L.hellm_ct_assign.argtypes = [vp, vp, vp]
        L.hellm_ct_destroy.argtypes = [vp]
        L.hellm_pt_destroy.argtypes = [vp]
        L.hellm_pt_download.argtypes = [vp, u32p, u64p]
        L.hellm_ctvec_destroy.argtypes = [vp]
        L.hellm_ctvec_size.argtypes = [vp, u32p]
        L.hellm_ctvec_get.argtypes = [vp, u32, u32, u32, u32, pvp]
        L.hellm_left_rotate.argtypes = [vp, vp, u64, pvp]
        for n in ("hellm_conjugate", "hellm_mult_imag_unit", "hellm_diagonal_to_column",
                  "hellm_diagonal_to_row"):
            getattr(L, n).argtypes = [vp, vp, pvp]
        for n in ("hellm_mult", "hellm_add", "hellm_complex_packing", "hellm_complex_packing_rev",
                  "hellm_complex_packing_pt", "hellm_repack_not_bts", "hellm_repack_lora_opti"):
            getattr(L, n).argtypes = [vp, vp, vp, pvp]
        for n in ("hellm_mult_const", "hellm_add_const"):
            getattr(L, n).argtypes = [vp, vp, ctypes.c_double, ctypes.c_double, pvp]
        L.hellm_matmul_high_low.argtypes = [vp, vp, vp, u32, u32, pvp]
        L.hellm_matmul_low_high.argtypes = [vp, vp, vp, u32, u32, pvp]
        L.hellm_matmul_low_low.argtypes = [vp, vp, vp, u32, u32, u32, pvp]
        L.hellm_low_rank_block.argtypes = [vp, vp, u32, u32, pvp]
        L.hellm_lora_rank2.argtypes = [vp, ctypes.c_int, ctypes.POINTER(vp), u32, vp, u32, u32, ctypes.POINTER(vp)]
        L.hellm_level_down.argtypes = [vp, vp, u32, pvp]
        L.hellm_transpose_inplace.argtypes = [vp, vp, u32]
        L.hellm_complex_packing_inplace.argtypes = [vp, vp]
        L.hellm_complex_packing_row_inplace.argtypes = [vp, vp]
        L.hellm_transpose_complex_packing_inplace.argtypes = [vp, vp, u32]
        L.hellm_split_in_two.argtypes = [vp, vp, pvp, pvp]
        for n in ("hellm_single_cc_matmul", "hellm_single_matmul", "hellm_packed_matmul",
                  "hellm_packed_matmul_cc_reuse", "hellm_matmul_reuse", "hellm_matmul_cc_reuse"):
            getattr(L, n).argtypes = [vp, vp, vp, u32, pvp]
        for n in ("hellm_packed_matmul_pre", "hellm_packed_matmul_pre_rot", "hellm_packed_matmul_pre_rev",
                  "hellm_matmul_pre", "hellm_matmul_pre_rev"):
            getattr(L, n).argtypes = [vp, vp, u32, pvp]
        L.hellm_repack_cc.argtypes = [vp, vp, pvp]
        dp = ctypes.POINTER(ctypes.c_double)
        L.hellm_reduce_row_sum_with_scaled_mask.argtypes = [vp, vp, dp, dp, u32, u32]
        L.hellm_one_mat_rot_sum_inplace.argtypes = [vp, vp, vp]
        L.hellm_mask_right_left.argtypes = [vp, vp, pvp, pvp]
        L.hellm_mask_first_col_inplace.argtypes = [vp, vp]
        L.hellm_row_moments.argtypes = [vp, ctypes.POINTER(vp), u32, ctypes.c_double, pvp, pvp]
        L.hellm_encode_weight_grid.argtypes = [vp, dp, u32, u32, u32, u32, ctypes.c_char_p]
        L.hellm_encode_weight_list.argtypes = [vp, dp, u32, u32, u32, ctypes.c_char_p]
        L.hellm_get_weight.argtypes = [vp, ctypes.c_char_p, u32, pvp]
        L.hellm_ct_save.argtypes = [vp, vp, ctypes.c_char_p]
        L.hellm_ct_load.argtypes = [vp, ctypes.c_char_p, pvp]
        L.hellm_exp_iter.argtypes = [vp, vp, ctypes.c_int, pvp]
        L.hellm_exp_iter_parallel.argtypes = [vp, pvp, ctypes.c_uint32, ctypes.c_int]
        L.hellm_eval_odd_polynomial.argtypes = [vp, vp, dp, u32, ctypes.c_int, ctypes.c_int, pvp]
        L.hellm_eval_chebyshev.argtypes = [vp, vp, dp, u32, u32, ctypes.c_double, pvp]
        L.hellm_linear_transform.argtypes = [vp, vp, ctypes.c_double, ctypes.c_double, pvp]
        _declared = True
    return L


def _m(a):
    a = np.ascontiguousarray(a, dtype=np.float64)
    return a, a.ctypes.data_as(f64p)


class _Handle:
    _destroy = None

    def __init__(self, owner, h):
        self.owner, self.h = owner, h

    def free(self):
        if self.h:
            getattr(_L(), self._destroy)(self.h)
            self.h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Ct(_Handle):
    _destroy = "hellm_ct_destroy"

    def info(self):
        v = [u32() for _ in range(6)]
        check(_L().hellm_ct_info(self.h, *[ctypes.byref(x) for x in v]))
        return dict(zip(("num_poly", "level", "rescale_counter", "rows", "cols", "block_width"),
                        [x.value for x in v]))

    @property
    def level(self):
        return self.info()["level"]

    def residues(self):
        i = self.info()
        out = np.empty((i["num_poly"], i["level"] + 1, self.owner.N), dtype=np.uint64)
        check(_L().hellm_ct_download(self.h, out.ctypes.data_as(u64p)))
        return out

    def clone(self):
        h = vp()
        check(_L().hellm_ct_clone(self.h, ctypes.byref(h)))
        return Ct(self.owner, h)


class Pt(_Handle):
    _destroy = "hellm_pt_destroy"

    def residues(self):
        lvl = u32()
        check(_L().hellm_pt_download(self.h, ctypes.byref(lvl), None))
        out = np.empty((lvl.value + 1, self.owner.N), dtype=np.uint64)
        check(_L().hellm_pt_download(self.h, ctypes.byref(lvl), out.ctypes.data_as(u64p)))
        return out


class CtVec(_Handle):
    _destroy = "hellm_ctvec_destroy"

    def __len__(self):
        n = u32()
        check(_L().hellm_ctvec_size(self.h, ctypes.byref(n)))
        return n.value

    def get(self, i, rows, cols, block_width):
        h = vp()
        check(_L().hellm_ctvec_get(self.h, i, rows, cols, block_width, ctypes.byref(h)))
        return Ct(self.owner, h)


def chebyshev_product_basis(coeffs, baby_steps):
    """Plain Chebyshev series (coeffs[k] multiplies T_k) -> the coefficient table HEaaN::Math::ChebyshevCoefficients
    holds for `baby_steps` baby steps (a power of two): entry bs * i + j multiplies T_j * prod_k T_{2^k bs}^{bit k of i}.
    Uses T_k = 2 T_m T_{k-m} - T_{2m-k} (m < k < 2m) from the top giant step down, so numpy's fits can be fed to
    eval_chebyshev the way the reference's Remez tables are."""
    bs = int(baby_steps)
    assert bs >= 1 and bs & (bs - 1) == 0, "baby_steps must be a power of two"
    c = [float(x) for x in coeffs]
    size = bs
    while size < len(c):
        size *= 2
    c += [0.0] * (size - len(c))

    def split(c):
        if len(c) == bs:
            return c
        m = len(c) // 2
        low = [c[0]] + [c[j] - c[2 * m - j] for j in range(1, m)]
        high = [c[m]] + [2.0 * c[m + j] for j in range(1, m)]
        return split(low) + split(high)

    return split(c)


class Graph:
    """A recorded sequence of HEMMer calls (hellm_graph_*): launch() replays it asynchronously on its own stream,
    sync() waits for it."""

    def __init__(self, owner, h, keep):
        self.owner, self.h, self.keep = owner, h, keep

    def launch(self):
        check(_L().hellm_graph_launch(self.h))

    def sync(self):
        check(_L().hellm_graph_sync(self.h))

    def nodes(self):
        n = ctypes.c_uint64()
        check(_L().hellm_graph_nodes(self.h, ctypes.byref(n)))
        return n.value

    def free(self):
        if self.h:
            _L().hellm_graph_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class HEMMer:
    """HELLM::HEMMer on the GPU.  preset=True builds the FGb-sized context (N = 2^16)."""

    def __init__(self, log_n=None, q_primes=None, p_primes=None, dnum=None, log_scale=42,
                 min_bootstrap_level=0, seed=0x5EED, preset=False):
        L = _L()
        h = vp()
        if preset:
            check(L.hellm_hemmer_create_preset(seed, ctypes.byref(h)))
        else:
            mods = [int(x) for x in q_primes] + [int(x) for x in p_primes]
            arr = (ctypes.c_uint64 * len(mods))(*mods)
            check(L.hellm_hemmer_create(log_n, len(q_primes), len(p_primes), arr, dnum, log_scale,
                                        min_bootstrap_level, seed, ctypes.byref(h)))
        self.h = h
        self.seed = seed
        v = [u32() for _ in range(5)]
        check(L.hellm_hemmer_info(h, *[ctypes.byref(x) for x in v], None))
        self.log_n, self.nQ, self.nP, self.dnum, self.dim = [x.value for x in v]
        self.N = 1 << self.log_n
        pr = (ctypes.c_uint64 * (self.nQ + self.nP))()
        check(L.hellm_hemmer_info(h, None, None, None, None, None, pr))
        self.q, self.p = list(pr)[: self.nQ], list(pr)[self.nQ:]

    def close(self):
        if getattr(self, "h", None):
            _L().hellm_hemmer_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_schedule(self, fused=True, batch=16):
        """fused: batched launches with hoisted rotations (default); False: the reference's call order."""
        check(_L().hellm_set_schedule(self.h, int(fused), batch))

    def assume_single_tile(self, on=True):
        """Promise that single_cc_matmul operands hold one tile block and nothing else (encrypt() outputs)."""
        check(_L().hellm_assume_single_tile(self.h, int(on)))

    def sync(self):
        check(_L().hellm_sync())

    TRAFFIC_KINDS = ("transforms", "key_products", "basis_conversions", "tensor_accumulation", "masked_sums", "pointwise")

    def assign(self, dst, src):
        """dst's residues = src's, in place (hellm_ct_assign)"""
        check(_L().hellm_ct_assign(self.h, dst.h, src.h))

    def record(self, fn):
        """Runs fn() with the calls on this HEMMer recorded into a HIP graph instead of executed; returns
        (Graph, fn's result).  fn's result and operands are kept alive by the graph object."""
        check(_L().hellm_graph_begin(self.h))
        try:
            res = fn()
        finally:
            g = vp()
            rc = _L().hellm_graph_end(self.h, ctypes.byref(g))
        check(rc)
        return Graph(self, g, res), res

    def key_bytes(self):
        """{'plain', 'compact', 'pool'}: device bytes of the evaluation keys by form and of the context's buffer pool"""
        a, b, c = ctypes.c_uint64(), ctypes.c_uint64(), ctypes.c_uint64()
        check(_L().hellm_key_bytes(self.h, ctypes.byref(a), ctypes.byref(b), ctypes.byref(c)))
        return {"plain": a.value, "compact": b.value, "pool": c.value}

    def phase_trace(self, on=True):
        """Record an event at each named point of the batched schedules from now on (off: stop and forget)."""
        check(_L().hellm_phase_trace(self.h, int(on)))

    def phase_report(self):
        """[(name, ms since the previous mark)] of the marks recorded so far; waits for the device."""
        buf = ctypes.create_string_buffer(1 << 16)
        check(_L().hellm_phase_report(self.h, buf, len(buf)))
        return [(l.split("\t")[0], float(l.split("\t")[1])) for l in buf.value.decode().splitlines()]

    def traffic(self, reset=False):
        """Algorithmic bytes and launch counts queued on the device context since the last reset, by kind of work."""
        b = (ctypes.c_uint64 * 8)()
        n = (ctypes.c_uint64 * 8)()
        check(_L().hellm_traffic(self.h, b, n, int(reset)))
        return ({k: int(b[i]) for i, k in enumerate(self.TRAFFIC_KINDS)},
                {k: int(n[i]) for i, k in enumerate(self.TRAFFIC_KINDS)})

    def secret_coeffs(self):
        out = np.empty(self.N, dtype=np.int32)
        check(_L().hellm_secret_coeffs(self.h, out.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))))
        return out

    def export_key(self, galois=0):
        out = np.empty((self.dnum, 2, self.nQ + self.nP, self.N), dtype=np.uint64)
        check(_L().hellm_export_key(self.h, galois, out.ctypes.data_as(u64p)))
        return out

    def ensure_rotation_keys(self, rots):
        arr = (ctypes.c_uint64 * len(rots))(*[int(r) for r in rots])
        check(_L().hellm_ensure_rotation_keys(self.h, arr, len(rots)))

    # ---- codec ------------------------------------------------------------------------------
    def _new(self, cls, fn, *args):
        h = vp()
        check(getattr(_L(), fn)(self.h, *args, ctypes.byref(h)))
        return cls(self, h)

    def encrypt(self, m):
        a, pa = _m(m)
        return self._new(Ct, "hellm_encrypt", pa, a.shape[0], a.shape[1])

    def encrypt2(self, m1, m2):
        a, pa = _m(m1)
        b, pb = _m(m2)
        return self._new(Ct, "hellm_encrypt2", pa, pb, a.shape[0], a.shape[1])

    def encode(self, m, level=0):
        a, pa = _m(m)
        return self._new(Pt, "hellm_encode", pa, a.shape[0], a.shape[1], level)

    def encode2(self, m1, m2, level=0):
        a, pa = _m(m1)
        b, pb = _m(m2)
        return self._new(Pt, "hellm_encode2", pa, pb, a.shape[0], a.shape[1], level)

    def encode_diagonal_to_row4(self, w1, w2, w3, w4, level=0):
        ms = [_m(w) for w in (w1, w2, w3, w4)]
        return self._new(Pt, "hellm_encode_diagonal_to_row4", *[p for _, p in ms],
                         ms[0][0].shape[0], ms[0][0].shape[1], level)

    def decrypt(self, ct):
        i = ct.info()
        out = np.empty((i["rows"], i["cols"]), dtype=np.float64)
        check(_L().hellm_decrypt(self.h, ct.h, out.ctypes.data_as(f64p)))
        return out

    def decrypt2(self, ct):
        i = ct.info()
        out = np.empty((2, i["rows"], i["cols"]), dtype=np.float64)
        check(_L().hellm_decrypt2(self.h, ct.h, out.ctypes.data_as(f64p)))
        return out

    def decrypt_slots(self, ct):
        out = np.empty(self.N, dtype=np.float64)
        check(_L().hellm_decrypt_slots(self.h, ct.h, out.ctypes.data_as(f64p)))
        return out.view(np.complex128).copy()

    def upload(self, residues, rows, cols, block_width, rescale_counter=0):
        r = np.ascontiguousarray(residues, dtype=np.uint64)
        return self._new(Ct, "hellm_ct_upload", r.ctypes.data_as(u64p), r.shape[0], r.shape[1] - 1,
                         rescale_counter, rows, cols, block_width)

    # ---- evaluator ----------------------------------------------------------------------------
    def left_rotate(self, a, rot):
        return self._new(Ct, "hellm_left_rotate", a.h, rot)

    def conjugate(self, a):
        return self._new(Ct, "hellm_conjugate", a.h)

    def mult_imag_unit(self, a):
        return self._new(Ct, "hellm_mult_imag_unit", a.h)

    def mult(self, a, b):
        return self._new(Ct, "hellm_mult", a.h, b.h)

    def add(self, a, b):
        return self._new(Ct, "hellm_add", a.h, b.h)

    def mult_const(self, a, c):
        """HomEvaluator::mult(ct, constant): a Gaussian-integer constant does not consume a level"""
        c = complex(c)
        return self._new(Ct, "hellm_mult_const", a.h, c.real, c.imag)

    def add_const(self, a, c):
        c = complex(c)
        return self._new(Ct, "hellm_add_const", a.h, c.real, c.imag)

    def reduce_row_sum_with_scaled_mask(self, a, mask_left, mask_right):
        import numpy as np
        ml = np.ascontiguousarray(mask_left, dtype=np.float64)
        mr = np.ascontiguousarray(mask_right, dtype=np.float64)
        dp = ctypes.POINTER(ctypes.c_double)
        check(_L().hellm_reduce_row_sum_with_scaled_mask(self.h, a.h, ml.ctypes.data_as(dp), mr.ctypes.data_as(dp),
                                                         ml.shape[0], ml.shape[1]))

    def one_mat_rot_sum_inplace(self, a, b):
        check(_L().hellm_one_mat_rot_sum_inplace(self.h, a.h, b.h))

    def mask_right_left(self, a):
        h1, h2 = vp(), vp()
        check(_L().hellm_mask_right_left(self.h, a.h, ctypes.byref(h1), ctypes.byref(h2)))
        return Ct(self, h1), Ct(self, h2)

    def mask_first_col_inplace(self, a):
        check(_L().hellm_mask_first_col_inplace(self.h, a.h))

    def row_moments(self, tiles, inv_count):
        arr = (vp * len(tiles))(*[t.h for t in tiles])
        h1, h2 = vp(), vp()
        check(_L().hellm_row_moments(self.h, arr, len(tiles), float(inv_count), ctypes.byref(h1), ctypes.byref(h2)))
        return Ct(self, h1), Ct(self, h2)

    def encode_weight(self, tiles, save_path):
        """HEMMer::encodeWeight: tiles [height][width][rows][cols] -> <save_path><i>_<j>.msg (diagonal-to-row
        packing of four tile rows), or [count][rows][cols] -> <save_path><i>.msg (pairs of tiles)."""
        import numpy as np
        t = np.ascontiguousarray(tiles, dtype=np.float64)
        p = t.ctypes.data_as(ctypes.POINTER(ctypes.c_double))
        if t.ndim == 4:
            check(_L().hellm_encode_weight_grid(self.h, p, t.shape[0], t.shape[1], t.shape[2], t.shape[3],
                                                str(save_path).encode()))
        elif t.ndim == 3:
            check(_L().hellm_encode_weight_list(self.h, p, t.shape[0], t.shape[1], t.shape[2], str(save_path).encode()))
        else:
            raise ValueError("tiles must have 3 or 4 dimensions")

    def get_weight(self, file, level):
        return self._new(Pt, "hellm_get_weight", str(file).encode(), level)

    def save_ct(self, ct, file):
        check(_L().hellm_ct_save(self.h, ct.h, str(file).encode()))

    def load_ct(self, file):
        return self._new(Ct, "hellm_ct_load", str(file).encode())

    def exp_iter(self, a, num_iter):
        """(1 + a / 2^num_iter)^(2^num_iter) on the slots (HELLM::Exp::exp_iter)"""
        return self._new(Ct, "hellm_exp_iter", a.h, num_iter)

    def exp_iter_parallel(self, cts, num_iter):
        """HELLM::Exp::exp_iter_Parallel: exp_iter on every tensor of the list in place, squared pair by pair"""
        arr = (vp * len(cts))(*[c.h for c in cts])
        check(_L().hellm_exp_iter_parallel(self.h, arr, len(cts), num_iter))

    def eval_odd_polynomial(self, a, coeffs, k, l):
        """sum over odd i of coeffs[i] a^i (HELLM::ReLU::evalOddPolynomial)"""
        c = (ctypes.c_double * len(coeffs))(*[float(x) for x in coeffs])
        return self._new(Ct, "hellm_eval_odd_polynomial", a.h, c, len(coeffs), k, l)

    def eval_chebyshev(self, a, coeffs, baby_steps, multiplier=1.0):
        """HEaaN::Math::evaluateChebyshevExpansion on ChebyshevCoefficients{coeffs, baby_steps}: coefficients in the
        baby-step / giant-step product basis (entry bs * i + j multiplies T_j * prod_k T_{2^k bs}^{bit k of i}), slot
        values in [-1, 1]; baby_steps = 0: one block, i.e. a plain Chebyshev series"""
        c = (ctypes.c_double * len(coeffs))(*[float(x) for x in coeffs])
        return self._new(Ct, "hellm_eval_chebyshev", a.h, c, len(coeffs), baby_steps, float(multiplier))

    def linear_transform(self, a, left, right):
        """HEaaN::Math::linearTransform: [left, right] -> [-1, 1]"""
        return self._new(Ct, "hellm_linear_transform", a.h, float(left), float(right))

    def level_down(self, a, target):
        return self._new(Ct, "hellm_level_down", a.h, target)

    # ---- transforms and products -----------------------------------------------------------------
    def diagonal_to_column(self, a):
        return self._new(Ct, "hellm_diagonal_to_column", a.h)

    def diagonal_to_row(self, a):
        return self._new(Ct, "hellm_diagonal_to_row", a.h)

    def transpose_inplace(self, a, target_level=0):
        check(_L().hellm_transpose_inplace(self.h, a.h, target_level))

    def complex_packing_inplace(self, a):
        check(_L().hellm_complex_packing_inplace(self.h, a.h))

    def complex_packing_row_inplace(self, a):
        check(_L().hellm_complex_packing_row_inplace(self.h, a.h))

    def transpose_complex_packing_inplace(self, a, target_level=0):
        check(_L().hellm_transpose_complex_packing_inplace(self.h, a.h, target_level))

    def split_in_two(self, a):
        h1, h2 = vp(), vp()
        check(_L().hellm_split_in_two(self.h, a.h, ctypes.byref(h1), ctypes.byref(h2)))
        return Ct(self, h1), Ct(self, h2)

    def single_cc_matmul(self, a, b, target_level=4):
        return self._new(Ct, "hellm_single_cc_matmul", a.h, b.h, target_level)

    def single_matmul(self, a, b_pt, target_level=4):
        return self._new(Ct, "hellm_single_matmul", a.h, b_pt.h, target_level)

    def packed_matmul(self, a, b, target_level=4):
        return self._new(Ct, "hellm_packed_matmul", a.h, b.h, target_level)

    def packed_matmul_pre(self, a, target_level=4):
        return self._new(Ct, "hellm_packed_matmul_pre", a.h, target_level)

    def packed_matmul_pre_rot(self, a, target_level=4):
        return self._new(CtVec, "hellm_packed_matmul_pre_rot", a.h, target_level)

    def packed_matmul_pre_rev(self, b, target_level=4):
        return self._new(Ct, "hellm_packed_matmul_pre_rev", b.h, target_level)

    def packed_matmul_cc_reuse(self, tmp, b, target_level=4):
        return self._new(Ct, "hellm_packed_matmul_cc_reuse", tmp.h, b.h, target_level)

    def repack_cc(self, a):
        return self._new(Ct, "hellm_repack_cc", a.h)

    def complex_packing(self, a, b):
        return self._new(Ct, "hellm_complex_packing", a.h, b.h)

    def complex_packing_rev(self, a, b):
        return self._new(Ct, "hellm_complex_packing_rev", a.h, b.h)

    def complex_packing_pt(self, a, b):
        """plaintexts: 0.5 a - 0.5 i b (HEMMer::complexPacking(PtxtTensor, PtxtTensor))"""
        return self._new(Pt, "hellm_complex_packing_pt", a.h, b.h)

    def repack_not_bts(self, a, b):
        return self._new(Ct, "hellm_repack_not_bts", a.h, b.h)

    def repack_lora_opti(self, a, b):
        return self._new(Ct, "hellm_repack_lora_opti", a.h, b.h)

    # LoRA low-rank path (rank 2): products with a thin operand and the block repacking around them
    def matmul_high_low(self, a, b, in_col_block, target_level):
        return self._new(Ct, "hellm_matmul_high_low", a.h, b.h, in_col_block, target_level)

    def matmul_low_high(self, a, b, in_row_block, target_level):
        return self._new(Ct, "hellm_matmul_low_high", a.h, b.h, in_row_block, target_level)

    def matmul_low_low(self, a, b, in_col_block, in_row_block, target_level=4):
        return self._new(Ct, "hellm_matmul_low_low", a.h, b.h, in_col_block, in_row_block, target_level)

    def repack_to_one_col(self, a, block):
        return self._new(Ct, "hellm_low_rank_block", a.h, 0, block)

    def repack_to_multi_col(self, a, block):
        return self._new(Ct, "hellm_low_rank_block", a.h, 1, block)

    def repack_to_one_row(self, a, block):
        return self._new(Ct, "hellm_low_rank_block", a.h, 2, block)

    def repack_to_multi_row(self, a, block):
        return self._new(Ct, "hellm_low_rank_block", a.h, 3, block)

    def get_low_col_block(self, a, block):
        return self._new(Ct, "hellm_low_rank_block", a.h, 4, block)

    def get_low_row_block(self, a, block):
        return self._new(Ct, "hellm_low_rank_block", a.h, 5, block)

    def _lora_rank2(self, up, cts, weight, n_out, weight_level):
        arr = (vp * len(cts))(*[t.h for t in cts])
        out = (vp * n_out)()
        check(_L().hellm_lora_rank2(self.h, up, arr, len(cts), weight.h, n_out, weight_level, out))
        return [Ct(self, vp(out[i])) for i in range(n_out)]

    def lora_rank2_down(self, cur, lora_wa, weight_level=9):
        """X a_0, X a_1 (column 0 of the left tile) from pair-layout activation tiles and the A weight tile."""
        return self._lora_rank2(0, cur, lora_wa, 2, weight_level)

    def lora_rank2_up(self, xa, lora_wb, n_out, weight_level=6):
        """(X A) B as n_out pair-layout ciphertexts from the two outputs of lora_rank2_down and the B weight tile."""
        return self._lora_rank2(1, xa, lora_wb, n_out, weight_level)

    def matmul_pre(self, a, target_level=4):
        return self._new(CtVec, "hellm_matmul_pre", a.h, target_level)

    def matmul_reuse(self, tmp, b_pt, target_level=4):
        return self._new(Ct, "hellm_matmul_reuse", tmp.h, b_pt.h, target_level)

    def matmul_pre_rev(self, b, target_level=4):
        return self._new(Ct, "hellm_matmul_pre_rev", b.h, target_level)

    def matmul_cc_reuse(self, tmp, b, target_level=4):
        return self._new(Ct, "hellm_matmul_cc_reuse", tmp.h, b.h, target_level)

"""TEST INFRASTRUCTURE ONLY -- CPU restatement of HEMMer's matrix-multiplication algorithms.

Restates, over an abstract evaluator, the slot-level algorithms of the reference's
ciphertext/src/MatrixUtils.cpp (mask families :90-578, sigma/tau transforms :776-1098, transpose
:671-739, multMatMat<Ciphertext> :1307-1446, multMatMat<Plaintext> :1448-1570, multPackedMatMat
:1100-1216, the Pre/ReUse family :1218-1305,:1572-1679) and the packing helpers of
ciphertext/src/HEMMer.cpp (:764-831, :964-1053).  Two evaluators run the same code:

  * SlotSim   -- "ciphertexts" are plain complex slot vectors (np.roll for rotations).  Pins every
                 mask and rotation index against float64 matrix algebra, independent of any crypto.
  * oracle.Oracle -- the CPU RNS-CKKS oracle; gives the residues the GPU path must reproduce bit
                 for bit when it issues the same operation sequence.

The operation order (masked rotations summed before one rescale; masks pre-rotated per
baby-step/giant-step group) is the one the GPU build documents for itself; decrypted results equal
the reference's A*B either way.
"""
import math

import numpy as np


def pow2ceil(v):
    p = 1
    while p < v:
        p <<= 1
    return p


# --------------------------------------------------------------------------------------------
# slot simulator
# --------------------------------------------------------------------------------------------
def rotate_sum_stages(count):
    """(rotations per stage, multiplier of the unit): one stage up to four terms, else i = i0 + b i1 with
    b = 2^ceil(log2(count) / 2)."""
    assert count >= 1 and count & (count - 1) == 0
    if count <= 4:
        return [(count, 1)]
    b = 1
    while b * b < count:
        b <<= 1
    return [(b, 1), (count // b, b)]


class SimCt:
    def __init__(self, z, level, rc=0):
        self.z, self.level, self.rc = np.asarray(z, dtype=np.complex128), level, rc


class SlotSim:
    """Evaluator over exact slot vectors, with the same level / rescale-counter bookkeeping."""

    def __init__(self, log_slots, top_level):
        self.slots = 1 << log_slots
        self.top = top_level

    def encrypt(self, z, level=None):
        v = np.zeros(self.slots, dtype=np.complex128)
        z = np.asarray(z).reshape(-1)
        v[: z.size] = z
        return SimCt(v, self.top if level is None else level)

    def encode(self, msg, level):
        return SimCt(np.asarray(msg, dtype=np.complex128).copy(), level)

    def decrypt(self, ct):
        return ct.z.copy()

    def level_of(self, x):
        return x.level

    def _lv(self, x, y):
        lo = min(x.level, y.level)
        return lo

    def add(self, x, y):
        assert x.rc == y.rc
        return SimCt(x.z + y.z, self._lv(x, y), x.rc)

    def sub(self, x, y):
        assert x.rc == y.rc
        return SimCt(x.z - y.z, self._lv(x, y), x.rc)

    def negate(self, x):
        return SimCt(-x.z, x.level, x.rc)

    def mult_plain_no_rescale(self, x, pt):
        assert x.rc == 0 and pt.level >= x.level
        return SimCt(x.z * pt.z, x.level, 1)

    def masked_sum(self, a, ma, b, mb):
        assert a.level == b.level
        return self.add(self.mult_plain_no_rescale(a, ma), self.mult_plain_no_rescale(b, mb))

    def rescale(self, x):
        assert x.rc >= 1 and x.level >= 1
        return SimCt(x.z, x.level - 1, x.rc - 1)

    def tensor(self, x, y):
        assert x.rc == 0 and y.rc == 0
        return SimCt(x.z * y.z, self._lv(x, y), 1)

    def relinearize(self, x):
        return x

    def mult(self, x, y):
        if isinstance(y, SimCt) and getattr(y, "is_pt", False):
            return self.rescale(self.mult_plain_no_rescale(x, y))
        return self.rescale(self.tensor(x, y))

    def mult_const(self, x, c):
        """HomEvaluator::mult(ct, constant): constants within 1e-8 of an integer do not use a level."""
        if abs(c - round(c)) <= 1e-8:
            return SimCt(x.z * round(c), x.level, x.rc)
        assert x.rc == 0 and x.level >= 1
        return SimCt(x.z * c, x.level - 1, 0)

    def mult_const_rescale(self, x, c):
        """multWithoutRescale(ct, constant) + rescale: always one level, however small or integral the constant."""
        assert x.rc == 0 and x.level >= 1
        return SimCt(x.z * c, x.level - 1, 0)

    def add_const(self, x, c):
        return SimCt(x.z + c, x.level, x.rc)

    def mult_pt(self, x, pt):
        return self.rescale(self.mult_plain_no_rescale(x, pt))

    def mult_imag_unit(self, x):
        return SimCt(1j * x.z, x.level, x.rc)

    def left_rotate(self, x, r):
        return SimCt(np.roll(x.z, -(r % self.slots)), x.level, x.rc)

    def right_rotate(self, x, r):
        return SimCt(np.roll(x.z, r % self.slots), x.level, x.rc)

    def rotate_sum(self, x, unit, count):
        """sum_{i < count} leftRotate(x, i * unit) (unit < 0: to the right)."""
        z = np.zeros_like(x.z)
        for i in range(count):
            z = z + np.roll(x.z, -((i * unit) % self.slots))
        return SimCt(z, x.level, x.rc)

    def conjugate(self, x):
        return SimCt(np.conj(x.z), x.level, x.rc)

    def level_down(self, x, target):
        assert target <= x.level
        return SimCt(x.z, target, x.rc)

    def level_down_one(self, x):
        return self.level_down(x, x.level - 1)

    # plaintext helpers (plaintexts are SimCt too)
    def pt_mult(self, a, b):
        return SimCt(a.z * b.z, min(a.level, b.level) - 1)

    def pt_add(self, a, b):
        return SimCt(a.z + b.z, min(a.level, b.level))

    def pt_reencode(self, pt, level):
        return SimCt(pt.z, level)

    def pt_values(self, pt):
        return pt.z


class OracleEval:
    """Adapter giving oracle.Oracle the interface the algorithms below use."""

    def __init__(self, orc):
        self.o = orc
        self.slots = orc.slots

    def encode(self, msg, level):
        return self.o.encode(msg, level)

    def level_of(self, x):
        return x.level

    def _same_level(self, x, y):
        if x.level > y.level:
            x = self.o.level_down(x, y.level)
        elif y.level > x.level:
            y = self.o.level_down(y, x.level)
        return x, y

    def add(self, x, y):
        x, y = self._same_level(x, y)
        return self.o.add(x, y)

    def sub(self, x, y):
        x, y = self._same_level(x, y)
        return self.o.sub(x, y)

    def negate(self, x):
        return self.o.negate(x)

    def mult_plain_no_rescale(self, x, pt):
        assert pt.level >= x.level
        return self.o.mult_plain_no_rescale(x, pt)

    def masked_sum(self, a, ma, b, mb):
        return self.o.add(self.o.mult_plain_no_rescale(a, ma), self.o.mult_plain_no_rescale(b, mb))

    def rescale(self, x):
        return self.o.rescale(x)

    def tensor(self, x, y):
        x, y = self._same_level(x, y)
        return self.o.tensor(x, y)

    def relinearize(self, x):
        return self.o.relinearize(x)

    def mult(self, x, y):
        return self.rescale(self.relinearize(self.tensor(x, y)))

    def mult_pt(self, x, pt):
        return self.rescale(self.mult_plain_no_rescale(x, pt))

    def mult_const(self, x, c):
        """HomEvaluator::mult(ct, real constant): an integer (within 1e-8) multiplies the residues and keeps
        the level; anything else is multiplied by round(c * Delta_level) and rescaled."""
        from .oracle import Ct
        r = math.floor(c + 0.5)
        if abs(c - r) <= 1e-8:
            return self.o.mult_integer(x, int(r))
        d = c * self.o.delta[x.level]
        v = int(math.floor(abs(d) + 0.5)) * (1 if d >= 0 else -1)      # llround: halves away from zero
        return self.o.rescale(Ct(self.o.mult_scalar_residues(x, v), x.scale * self.o.delta[x.level]))

    def mult_const_rescale(self, x, c):
        """multWithoutRescale(ct, real constant) + rescale: round(c * Delta_level) on the residues, one level."""
        from .oracle import Ct
        d = c * self.o.delta[x.level]
        v = int(math.floor(abs(d) + 0.5)) * (1 if d >= 0 else -1)      # llround: halves away from zero
        return self.o.rescale(Ct(self.o.mult_scalar_residues(x, v), x.scale * self.o.delta[x.level]))

    def add_const(self, x, c):
        """HomEvaluator::add(ct, Complex): the constant polynomial round(re Delta) + round(im Delta) X^(N/2) added to
        the first polynomial (what encoding a constant message gives, without the transform)."""
        from .oracle import Ct
        if self.o.N < 512:
            import numpy as _np
            return self.o.add(x, self.o.encode(_np.full(self.o.slots, c, dtype=_np.complex128), x.level))
        return Ct(self.o.add_constant_residues(x.data, complex(c), x.level), x.scale)

    def mult_imag_unit(self, x):
        return self.o.mult_imag_unit(x)

    def left_rotate(self, x, r):
        return self.o.left_rotate(x, r)

    def right_rotate(self, x, r):
        return self.o.right_rotate(x, r)

    def rotate_sum(self, x, unit, count):
        """sum_{i < count} leftRotate(x, i * unit) (unit < 0: to the right) as hoisted sums (rotateSumFused): at most
        two stages, i = i0 + b i1, each one ModUp, one sum of the stage's rotations with the unrotated input as a term
        without a key, and one ModDown."""
        from .oracle import Ct
        o = self.o
        for cnt, mul in rotate_sum_stages(count):
            if cnt <= 1:
                continue
            ext = o.modup(x.data[1])
            terms = []
            for i in range(1, cnt):
                r = (i * mul * unit) % o.slots
                terms.append((x.data[1], x.data[0], ("none",), None) if r == 0 else (ext, x.data[0], r, None))
            terms.append((x.data[1], x.data[0], ("none",), None))
            y = o.hoisted_sum(terms, x.nq)
            x = Ct(o.moddown_drop(y, x.nq, False), x.scale)
        return x

    def conjugate(self, x):
        return self.o.conjugate(x)

    def level_down(self, x, target):
        return self.o.level_down(x, target)

    def level_down_one(self, x):
        return self.o.level_down_one(x)

    def pt_mult(self, a, b):
        from .oracle import Ct, Pt
        lv = min(a.level, b.level)
        prod = self.o._binary(2, a.data[: lv + 1], b.data[: lv + 1])
        r = self.o.rescale(Ct(prod[None], a.scale * b.scale))
        return Pt(r.data[0], r.scale)

    def pt_add(self, a, b):
        from .oracle import Pt
        lv = min(a.level, b.level)
        return Pt(self.o._binary(0, a.data[: lv + 1], b.data[: lv + 1]), a.scale)

    def pt_reencode(self, pt, level):
        return self.o.encode(self.o.decode(pt), level)

    def pt_values(self, pt):
        return self.o.decode(pt)


# --------------------------------------------------------------------------------------------
# masks  (MatrixUtils.cpp:90-578)
# --------------------------------------------------------------------------------------------
H, V, PH, PV, DIAG = "horizontal", "vertical", "packed_horizontal", "packed_vertical", "diagonal"
DIAG_SIGNED = "diagonal_signed"   # the transpose's diagonals in the grouping of sigma / tau (batched transform)
# the complex packing followed by the packed transform as ONE linear map (one level instead of two)
PKH, PKV = "packing_horizontal", "packing_vertica"


def _dims(n):
    """Tile shape: an int is a square tile, a pair is (rows, cols)."""
    return (n, n) if isinstance(n, (int, np.integer)) else (int(n[0]), int(n[1]))


def geometry(kind, n, w):
    """(units, cell, bs, gs, step): diagonals in cells, cell size, BSGS sizes, slots per diagonal.
    For a rectangular tile (sigma / tau only, generateHorizontalMask :129-217, generateVerticalMask
    :330-419) `units` is the length a diagonal wraps over (columns for sigma, rows for tau) and the
    BSGS sizes come from the shorter side (sub_dim)."""
    rows, cols = _dims(n)
    if kind == DIAG:
        assert rows == cols
        count = 2 * rows - 1
        bs = math.ceil(math.sqrt(count))
        return rows, 1, bs, math.ceil(count / bs), w - 1
    cell = 2 if kind in (PH, PV) else 1
    assert cell == 1 or rows == cols
    assert kind not in (DIAG_SIGNED, PKH, PKV) or rows == cols
    units = (cols if kind in (H, PH, PKH) else rows) // cell
    sub = sub_dim(kind, n)
    bs = math.ceil(math.sqrt(2 * sub - 1))
    gs = math.ceil((sub - 1) / bs)
    step = w - 1 if kind == DIAG_SIGNED else cell * (w if kind in (V, PV, PKV) else 1)
    return units, cell, bs, gs, step


def sub_dim(kind, n):
    """Number of diagonals of one sign: the shorter side of the tile, in cells."""
    rows, cols = _dims(n)
    return min(rows, cols) // (2 if kind in (PH, PV) else 1)


def transform_mask(kind, n, w, slots, idx):
    """Slot pattern of diagonal idx (no pre-rotation)."""
    rows, cols = _dims(n)
    if kind in (PKH, PKV):
        # T_packed(P(x)) = sum_d mask_d rho^(2 d unit)(Z x + M_+ rho^unit x + M_- rho^-unit x): the coefficient of
        # rho^(idx unit)(x) collects the three ways of writing idx = 2 d + e, e in {0, +1, -1}
        by_rows = kind == PKV
        base, unit, cells = (PV if by_rows else PH), (w if by_rows else 1), (rows if by_rows else cols) // 2
        zmask, terms = packing_maps(slots, w, by_rows)
        part = {0: zmask, 1: terms[0][1], -1: terms[1][1]}
        m = np.zeros(slots, dtype=np.complex128)
        for e in (0, 1, -1):
            if (idx - e) % 2:
                continue
            d = (idx - e) // 2
            if d <= -cells or d >= cells:
                continue
            m += transform_mask(base, n, w, slots, d) * np.roll(part[e], -2 * d * unit)
        return m
    units, cell, _, _, _ = geometry(kind, n, w)
    sub = sub_dim(kind, n)
    r = np.arange(slots) // w
    c = np.arange(slots) % w
    R = (r % rows) // cell
    C = (c % cols) // cell
    if kind in (H, PH):
        R = R % sub                      # a tall tile repeats the pattern every sub_dim rows
        on = (R == idx) & (C < units - idx) if idx >= 0 else (R == units + idx) & (C >= -idx)
    elif kind in (V, PV):
        C = C % sub                      # a wide tile repeats it every sub_dim columns
        on = (C == idx) & (R < units - idx) if idx >= 0 else (C == units + idx) & (R >= -idx)
    else:
        on = (C - R) == idx
    return np.where(on, 0.5 if kind == PH else 1.0, 0.0).astype(np.complex128)


def prerotated_mask(kind, n, w, slots, idx):
    units, _, bs, _, step = geometry(kind, n, w)
    m = transform_mask(kind, n, w, slots, idx)
    if kind == DIAG:
        i = (idx + _dims(n)[0] - 1) // bs
        return np.roll(m, i * bs * step)
    if idx > 0:
        i = (idx - 1) // bs
        return np.roll(m, i * bs * step)
    if idx < 0:
        i = (idx + units - 1) // bs
        return np.roll(m, -((units - i * bs) * step))
    return m


def col_masks(n, slots):
    """[2i] wrapped part, [2i+1] main part of a cyclic column shift by i (generateColMask :554-578)."""
    j = np.arange(slots)
    out = []
    for i in range(n):
        main = (j % n < n - i)
        out += [(~main).astype(np.complex128), main.astype(np.complex128)]
    return out


def row_masks(n, w, slots):
    j = np.arange(slots)
    out = []
    for i in range(n):
        main = ((j // w) % n < n - i)
        out += [(~main).astype(np.complex128), main.astype(np.complex128)]
    return out


# --------------------------------------------------------------------------------------------
# transforms  (MatrixUtils.cpp:671-1098)
# --------------------------------------------------------------------------------------------
def diagonal_transform(ev, ct, kind, n, w):
    units, _, bs, gs, step = geometry(kind, n, w)
    sub = sub_dim(kind, n)
    level = ev.level_of(ct)
    enc = lambda idx: ev.encode(prerotated_mask(kind, n, w, ev.slots, idx), level)
    baby = []
    for j in range(bs):
        baby.append(ev.left_rotate(ct if j == 0 else baby[j - 1], step))
    res = ev.mult_plain_no_rescale(ct, enc(0))
    for i in range(gs):
        group = None
        for j in range(bs):
            d = 1 + i * bs + j - units
            if d >= sub - units:
                break
            t = ev.mult_plain_no_rescale(baby[j], enc(d))
            group = t if group is None else ev.add(group, t)
        if group is not None:
            res = ev.add(res, ev.right_rotate(group, (units - i * bs) * step))
        group = None
        for j in range(bs):
            d = 1 + i * bs + j
            if d >= sub:
                break
            t = ev.mult_plain_no_rescale(baby[j], enc(d))
            group = t if group is None else ev.add(group, t)
        if group is not None:
            if i > 0:
                group = ev.left_rotate(group, i * bs * step)
            res = ev.add(res, group)
    return ev.rescale(res)


def transpose(ev, ct, n, w):
    _, _, bs, gs, step = geometry(DIAG, n, w)
    level = ev.level_of(ct)
    baby = []
    for j in range(bs):
        baby.append(ev.right_rotate(ct, (n - 1) * step) if j == 0 else ev.left_rotate(baby[j - 1], step))
    res = None
    for i in range(gs):
        group = None
        for j in range(bs):
            e = 1 - n + i * bs + j
            if e >= n:
                break
            t = ev.mult_plain_no_rescale(baby[j], ev.encode(prerotated_mask(DIAG, n, w, ev.slots, e), level))
            group = t if group is None else ev.add(group, t)
        if group is None:
            continue
        if i > 0:
            group = ev.left_rotate(group, i * bs * step)
        res = group if res is None else ev.add(res, group)
    return ev.rescale(res)


# --------------------------------------------------------------------------------------------
# products  (MatrixUtils.cpp:1100-1679)
# --------------------------------------------------------------------------------------------
def mult_mat_mat_cc(ev, a, b, T, n, w):
    """multMatMat<Ciphertext> (:1307-1446): sum_k phi^k(sigma A) * psi^k(tau B)."""
    cm = [ev.encode(m, T + 2) for m in col_masks(n, ev.slots)]
    rm = [ev.encode(m, T + 2) for m in row_masks(n, w, ev.slots)]
    a = diagonal_transform(ev, a, H, n, w)
    b = diagonal_transform(ev, b, V, n, w)
    a = ev.level_down(a, T + 2)
    b = ev.level_down(b, T + 2)
    res = ev.mult(a, b)
    a = ev.left_rotate(a, 1)
    b = ev.left_rotate(b, w)
    a_wrap = ev.right_rotate(a, n)
    b_wrap = ev.right_rotate(b, n * w)
    acc = None
    for i in range(1, n):
        if i > 1:
            a = ev.left_rotate(a, 1)
            a_wrap = ev.left_rotate(a_wrap, 1)
            b = ev.left_rotate(b, w)
            b_wrap = ev.left_rotate(b_wrap, w)
        t1 = ev.rescale(ev.masked_sum(a, cm[2 * i + 1], a_wrap, cm[2 * i]))
        t2 = ev.rescale(ev.masked_sum(b, rm[2 * i + 1], b_wrap, rm[2 * i]))
        t = ev.tensor(t1, t2)
        acc = t if acc is None else ev.add(acc, t)
    out = ev.rescale(ev.relinearize(acc))
    return ev.add(res, out)


def tau_plain(values, n, w):
    """diagonalToRow<Plaintext> (:1072-1098): host permutation tau(B)[i,j] = B[(i+j) mod n, j]."""
    slots = values.size
    r = np.arange(slots) // w
    c = np.arange(slots) % w
    src = ((r - r % n) + (r % n + c % n) % n) * w + c
    return values[src]


def mult_mat_mat_pc(ev, a, b_pt, T, n, w):
    """multMatMat<Plaintext> (:1448-1570)."""
    cm = [ev.encode(m, T + 2) for m in col_masks(n, ev.slots)]
    rm = [ev.encode(m, T + 2) for m in row_masks(n, w, ev.slots)]
    a = diagonal_transform(ev, a, H, n, w)
    b = ev.encode(tau_plain(ev.pt_values(b_pt), n, w), ev.level_of(b_pt))
    a = ev.level_down(a, T + 2)
    b = ev.pt_reencode(b, T + 2)
    res = ev.mult_pt(a, b)
    a = ev.left_rotate(a, 1)
    b = ev.left_rotate(b, w)
    a_wrap = ev.right_rotate(a, n)
    b_wrap = ev.right_rotate(b, n * w)
    acc = None
    for i in range(1, n):
        if i > 1:
            a = ev.left_rotate(a, 1)
            a_wrap = ev.left_rotate(a_wrap, 1)
            b = ev.left_rotate(b, w)
            b_wrap = ev.left_rotate(b_wrap, w)
        t1 = ev.rescale(ev.masked_sum(a, cm[2 * i + 1], a_wrap, cm[2 * i]))
        p = ev.pt_add(ev.pt_mult(b, rm[2 * i + 1]), ev.pt_mult(b_wrap, rm[2 * i]))
        t = ev.mult_pt(t1, p)
        acc = t if acc is None else ev.add(acc, t)
    return ev.add(res, acc)


def complex_packing_cols(ev, t, n, w):
    """HEMMer::complexPackingInplace (HEMMer.cpp:764-777): columns (2c, 2c+1) -> a + i b in both."""
    even = (np.arange(ev.slots) % 2 == 0).astype(np.complex128)
    m = ev.encode(even, ev.level_of(t))
    e = ev.mult_pt(t, m)
    o = ev.mult_pt(ev.mult_imag_unit(ev.left_rotate(t, 1)), m)
    fus = ev.add(o, e)
    return ev.add(ev.right_rotate(fus, 1), fus)


def complex_packing_rows(ev, t, n, w):
    """HEMMer::complexPackingRowInplace (HEMMer.cpp:801-817): rows (2k, 2k+1) -> a - i b in both."""
    even = ((np.arange(ev.slots) // w) % 2 == 0).astype(np.complex128)
    m = ev.encode(even, ev.level_of(t))
    e = ev.mult_pt(t, m)
    o = ev.mult_pt(ev.negate(ev.mult_imag_unit(ev.left_rotate(t, w))), m)
    fus = ev.add(e, o)
    return ev.add(ev.right_rotate(fus, w), fus)


def mult_packed_mat_mat(ev, a, b, T, n, w):
    """multPackedMatMat (:1100-1216) on complex-packed operands."""
    cm = [ev.encode(m, T + 2) for m in col_masks(n, ev.slots)]
    a = ev.level_down(a, T + 3)
    b = ev.level_down(b, T + 2)
    a = diagonal_transform(ev, a, PH, n, w)
    b = diagonal_transform(ev, b, PV, n, w)
    res = ev.mult(a, b)
    a = ev.left_rotate(a, 2)
    b = ev.left_rotate(b, 2 * w)
    a_wrap = ev.right_rotate(a, n)
    acc = None
    for i in range(1, n // 2):
        if i > 1:
            a = ev.left_rotate(a, 2)
            a_wrap = ev.left_rotate(a_wrap, 2)
            b = ev.left_rotate(b, 2 * w)
        t1 = ev.rescale(ev.masked_sum(a, cm[4 * i + 1], a_wrap, cm[4 * i]))
        t = ev.tensor(t1, b)
        acc = t if acc is None else ev.add(acc, t)
    out = ev.rescale(ev.relinearize(acc))
    return ev.add(res, out)


def repack_cc(ev, t):
    """HEMMer::repackCC (HEMMer.cpp:964-969): x + conj(x)."""
    return ev.add(t, ev.conjugate(t))


def mult_mat_mat_pre(ev, a, T, n, w):
    """multMatMatPre (:1572-1610): all column shifts of sigma(A), at level T+1."""
    cm = [ev.encode(m, T + 2) for m in col_masks(n, ev.slots)]
    a = ev.level_down(a, T + 3)
    a = diagonal_transform(ev, a, H, n, w)
    tmp = [ev.level_down_one(a)]
    a = ev.left_rotate(a, 1)
    a_wrap = ev.right_rotate(a, n)
    for i in range(1, n):
        if i > 1:
            a = ev.left_rotate(a, 1)
            a_wrap = ev.left_rotate(a_wrap, 1)
        tmp.append(ev.rescale(ev.masked_sum(a, cm[2 * i + 1], a_wrap, cm[2 * i])))
    return tmp


def mult_mat_mat_reuse(ev, tmp, b_pt, T, step=None):
    """multMatMatReUse (:1612-1639) with eval.matmul spelled out:
    rescale(sum_k tmp[k] * leftRotate(pt, k * slots / len(tmp)))."""
    if ev.level_of(b_pt) != T + 1:
        b_pt = ev.pt_reencode(b_pt, T + 1)
    step = ev.slots // len(tmp) if step is None else step
    acc = None
    for k, c in enumerate(tmp):
        t = ev.mult_plain_no_rescale(c, ev.left_rotate(b_pt, k * step))
        acc = t if acc is None else ev.add(acc, t)
    return ev.rescale(acc)


def mult_mat_mat_pre_rev(ev, b, T, n, w, kind=V):
    """multMatMatPreRev (:1641-1649) / multPackedMatMatPreRev (:1266-1274, kind=PV): tau(B) after a levelDown to
    T+2; multPackedMatMatPre (:1218-1227) is the same at T+3 with kind=PH (pass T+1)."""
    return diagonal_transform(ev, ev.level_down(b, T + 2), kind, n, w)


def mult_mat_mat_cc_reuse(ev, tmp, b, step, rescale_after=False):
    """multMatMatCCReUse (:1651-1679; step = block width, no rescale) / multPackedMatMatCCReuse (:1276-1305;
    step = 2 * block width, rescale after the relinearisation): sum_k tmp[k] (x) leftRotate^k(tau B, step), the
    rotations chained one after the other."""
    acc = ev.tensor(tmp[0], b)
    for k in range(1, len(tmp)):
        b = ev.left_rotate(b, step)
        acc = ev.add(acc, ev.tensor(tmp[k], b))
    out = ev.relinearize(acc)
    return ev.rescale(out) if rescale_after else out


def mult_packed_mat_mat_pre_rot(ev, a, T, n, w):
    """multPackedMatMatPreRot (:1229-1264): the n/2 shifts by two columns of packed sigma(A), at level T+1."""
    cm = [ev.encode(m, T + 2) for m in col_masks(n, ev.slots)]
    tmp = [ev.level_down_one(a)]
    a = ev.left_rotate(a, 2)
    a_wrap = ev.right_rotate(a, n)
    for i in range(1, n // 2):
        if i > 1:
            a = ev.left_rotate(a, 2)
            a_wrap = ev.left_rotate(a_wrap, 2)
        tmp.append(ev.rescale(ev.masked_sum(a, cm[4 * i + 1], a_wrap, cm[4 * i])))
    return tmp


def transpose_complex_packing(ev, t, n, w, target_level=0, fused_orc=None):
    """HEMMer::transposeComplexPackingInplace (HEMMer.cpp:779-799): columns (2c, 2c+1) -> a - i b in both, an
    optional levelDown to target_level + 1, then the transpose (reference order, or the batched transform over
    `fused_orc` as the default schedule runs it)."""
    even = (np.arange(ev.slots) % 2 == 0).astype(np.complex128)
    m = ev.encode(even, ev.level_of(t))
    e = ev.mult_pt(t, m)
    o = ev.mult_pt(ev.negate(ev.mult_imag_unit(ev.left_rotate(t, 1))), m)
    fus = ev.add(o, e)
    out = ev.add(ev.right_rotate(fus, 1), fus)
    if target_level > 0:
        out = ev.level_down(out, 1 + target_level)
    if fused_orc is not None:
        return diagonal_transform_fused(fused_orc, out, DIAG_SIGNED, n, w)
    return transpose(ev, out, n, w)


# --------------------------------------------------------------------------------------------
# batched schedule of the same products, over the oracle only (residue-level definition of what the
# GPU's batched launches compute): rotations are applied after ModUp ("hoisted"), the two masked
# halves of a shift are combined in the extended basis and ModDown is merged with the rescale.
# --------------------------------------------------------------------------------------------
def diagonal_transform_fused(orc, ct, kind, n, w):
    from .oracle import Ct
    units, _, bs, gs, step = geometry(kind, n, w)
    sub = sub_dim(kind, n)
    level, nq = ct.level, ct.nq
    enc = lambda idx: orc.encode(prerotated_mask(kind, n, w, orc.slots, idx), level)
    ext = orc.modup(ct.data[1])
    baby = [Ct(orc.moddown_drop(orc.hoisted_sum([(ext, ct.data[0], (j + 1) * step, None)], nq), nq, False),
               ct.scale) for j in range(bs)]
    groups, rots = [[(ct, 0)]], [0]

    def push(terms, r):
        if not terms:
            return
        if r % orc.slots == 0:
            groups[0].extend(terms)
        else:
            groups.append(terms)
            rots.append(r)

    for i in range(gs):
        neg = [(baby[j], 1 + i * bs + j - units) for j in range(bs) if 1 + i * bs + j - units < sub - units]
        push(neg, -(units - i * bs) * step)
        pos = [(baby[j], 1 + i * bs + j) for j in range(bs) if 1 + i * bs + j < sub]
        push(pos, i * bs * step)
    sums = []
    for terms in groups:
        acc = None
        for c, d in terms:
            t = orc.mult_plain_no_rescale(c, enc(d))
            acc = t if acc is None else orc.add(acc, t)
        sums.append(acc)
    res = sums[0]
    if len(sums) > 1:
        # the group that is not rotated joins the rotated ones as a term without a key; one ModDown merged with the rescale
        terms = [(orc.modup(s.data[1]), s.data[0], r % orc.slots, None) for s, r in zip(sums[1:], rots[1:])]
        terms.append((res.data[1], res.data[0], ("none",), None))
        y = orc.hoisted_sum(terms, nq)
        return Ct(orc.moddown_drop(y, nq, True), res.scale / float(orc.q[nq - 1]))
    return orc.rescale(res)


def bsgs_baby_count(n):
    """Largest power of two g with g * g <= 2 n."""
    g = 1
    while 4 * g * g <= 2 * n:
        g <<= 1
    return g


def two_stage_split(units):
    """Smallest power of two b with b * b >= units."""
    b = 1
    while b * b < units:
        b <<= 1
    return b


def two_stage_mask(kind, n, w, slots, stage, r, part):
    """Masks of the two-stage sigma / tau: stage 1 selects the rows (sigma) / columns (tau) whose cell index
    is r mod b, stage 2 those whose cell index div b is r; part 0: all of them, 1: the positions that do
    not wrap under the stage's rotation (r cells, or r b cells), 2: those that do, 3: both."""
    cell = 2 if kind in (PH, PV) else 1
    u = n // cell
    b = two_stage_split(u)
    row, col = np.arange(slots) // w, np.arange(slots) % w
    Rc, Cc = (row % n) // cell, (col % n) // cell
    sel, pos = (Cc, Rc) if kind in (V, PV) else (Rc, Cc)
    on = (sel % b == r) if stage == 1 else (sel // b == r)
    amount = r if stage == 1 else r * b
    if part == 1:
        on = on & (pos < u - amount)
    elif part == 2:
        on = on & (pos >= u - amount)
    return np.where(on, 0.5 if (kind == PH and stage == 1) else 1.0, 0.0).astype(np.complex128)


def diagonal_transform_two_stage(orc, ct, kind, n, w, from_level=None, first_stage=1):
    """sigma / tau (square tiles) in two stages of one mask level each: row i is rotated by i mod b, then
    by b (i div b).  Every stage is one hoisted sum over its rotations of
    main_r rho^(r)(X) + wrap_r rho^(r - tile side)(X) (two keys per r, one source) and of mask_0 X for the rows that
    stay (a term without a key switch), with ModDown merged with the rescale.  Level L -> L - 2.
    from_level: the level whose scale the input still carries when it was only truncated from there (the masks of
    the first stage are then encoded at Delta_{L-1} q_L / Delta_from, so the stage ends at the scale of L - 1).
    first_stage = 2: only the second stage (ct is what a first stage left)."""
    from .oracle import Ct
    cell = 2 if kind in (PH, PV) else 1
    u = n // cell
    b = two_stage_split(u)
    step = cell * (w if kind in (V, PV) else 1)
    wrap = n * (w if kind in (V, PV) else 1)
    x = ct
    for stage, count, mul in ((1, b, 1), (2, u // b, b)):
        if stage < first_stage:
            continue
        nq, lvl = x.nq, x.level
        own = stage == 2 or from_level is None or from_level == lvl
        ms = orc.delta[lvl] if own else orc.delta[lvl - 1] * float(orc.q[lvl]) / orc.delta[from_level]
        mask = lambda r, part: orc.encode_ext(two_stage_mask(kind, n, w, orc.slots, stage, r, part), lvl, ms)
        if count <= 1:      # no rotation in this stage: mask and rescale
            x = orc.rescale(orc.mult_plain_no_rescale(
                x, orc.encode(two_stage_mask(kind, n, w, orc.slots, stage, 0, 0), lvl, ms)))
            x.scale = orc.delta[lvl - 1]
            continue
        ext = orc.modup(x.data[1])
        terms = []
        for r in range(1, count):
            r_main, r_wrap = (r * mul * step) % orc.slots, (r * mul * step - wrap) % orc.slots
            if r_main == r_wrap:        # the tile side is a whole turn: one term with both parts of the mask
                terms.append((ext, x.data[0], r_main, mask(r, 3)))
            else:
                terms.append((ext, x.data[0], r_main, mask(r, 1)))
                terms.append((ext, x.data[0], r_wrap, mask(r, 2)))
        terms.append((x.data[1], x.data[0], ("none",), mask(0, 0)))
        y = orc.hoisted_sum(terms, nq)
        x = Ct(orc.moddown_drop(y, nq, True), orc.delta[lvl - 1])
    return x


def packing_stage_one(orc, x, kind, n, w, from_level=None):
    """The complex packing (by rows for PV, by columns for PH) and the FIRST stage of the two-stage transform of `kind`
    as one linear map on the slots (MatrixTransformer::packingStageOne): one hoisted sum, one level.  The term that
    rotates by a slots carries the sum over (stage rotation r, packing shift e) with r + e = a of
    stage mask_r (.) rho^r(packing mask_e); a = 0 is the term without a key; rotations whose masks cancel are left out.
    from_level: the level whose scale a truncated input still carries (the masks then carry the change of scale)."""
    from .oracle import Ct
    nq, lvl = x.nq, x.level
    own = from_level is None or from_level == lvl
    ms = orc.delta[lvl] if own else orc.delta[lvl - 1] * float(orc.q[lvl]) / orc.delta[from_level]
    ext = orc.modup(x.data[1])
    terms = []
    for a, mask in packing_stage_one_maps(kind, n, w, orc.slots):
        m = orc.encode_ext(mask, lvl, ms)
        terms.append((x.data[1], x.data[0], ("none",), m) if a == 0 else (ext, x.data[0], a, m))
    y = orc.hoisted_sum(terms, nq)
    return Ct(orc.moddown_drop(y, nq, True), orc.delta[lvl - 1])


def packing_stage_one_maps(kind, n, w, slots):
    """[(left rotation a in slots, mask)] with stage_1(packing(x)) = sum_a mask_a (.) rho^a(x), in increasing a."""
    assert kind in (PH, PV)
    b = two_stage_split(n // 2)
    unit = w if kind == PV else 1
    step, wrap = 2 * unit, n * unit
    zmask, pterms = packing_maps(slots, w, rows=(kind == PV))
    pack = [(0, zmask)] + pterms
    acc = {}

    def add(stage_mask, a):
        for e, pm in pack:
            t = (a + e) % slots
            acc[t] = acc.get(t, 0) + stage_mask * np.roll(pm, -(a % slots))     # rho^a(pm)[s] = pm[s + a]

    add(two_stage_mask(kind, n, w, slots, 1, 0, 0), 0)
    for r in range(1, b):
        add(two_stage_mask(kind, n, w, slots, 1, r, 1), r * step)
        add(two_stage_mask(kind, n, w, slots, 1, r, 2), r * step - wrap)
    return [(a, acc[a]) for a in sorted(acc) if np.any(acc[a])]


def lower_and_transform_fused(orc, x, kind, n, w, end_level):
    """Batched transform ending at end_level: two stages from end_level + 2 when the operand is that high and
    the tile is square, otherwise one stage from end_level + 1."""
    from .oracle import Ct
    rows, cols = _dims(n)
    if x.level >= end_level + 2 and rows == cols:
        # an operand above the starting level is only truncated to it: the masks of the first stage absorb the change
        # of scale (no levelDown)
        cut = Ct(np.ascontiguousarray(x.data[:, : end_level + 3]), x.scale)
        return diagonal_transform_two_stage(orc, cut, kind, rows, w, from_level=x.level)
    return diagonal_transform_fused(orc, orc.level_down(x, end_level + 1), kind, n, w)


def _rotated_copy(orc, src, ext, r):
    """rot(src, r) with the automorphism after ModUp (one hoisted term, plain ModDown)."""
    from .oracle import Ct
    if r % orc.slots == 0:      # a whole turn: rows of a tile that fills the slot vector
        return src.copy()
    y = orc.hoisted_sum([(ext, src.data[0], r % orc.slots, None)], src.nq)
    return Ct(orc.moddown_drop(y, src.nq, False), src.scale)


def _assemble_shifts(orc, src, ext, back, shifts):
    """Cyclic shifts inside a tile: main_mask * rot(src, r) + wrap_mask * rot(src2, r) with
    src2 = rot(src, back) prepared once, so both halves use the key of r.
    shifts: (r, main_mask_ext, wrap_mask_ext) -> ciphertexts one level down."""
    from .oracle import Ct
    nq = src.nq
    src2 = _rotated_copy(orc, src, ext, back)
    ext2 = orc.modup(src2.data[1])
    out = []
    for r, m_main, m_wrap in shifts:
        terms = [(ext, src.data[0], r % orc.slots, m_main), (ext2, src2.data[0], r % orc.slots, m_wrap)]
        y = orc.hoisted_sum(terms, nq)
        out.append(Ct(orc.moddown_drop(y, nq, True), orc.delta[src.level - 1]))
    return out


def _bsgs_shift_product(orc, a, b_low, acc, cm, n, units, cu, w, spread_block=0, with_conj=False):
    """Baby-step / giant-step sum over the shift index i = i1 + g i2 (column shift cu * i slots, row rotation
    i * cu * w slots); `acc` holds the i = 0 term, a = sigma(A) at T+2, b_low = tau(B) at T+1.
    spread_block: tau(B) holds one tile block of that many slots and nothing else; every baby rotation then
    also gathers the copies rho^(-j spread_block) (further terms of the same hoisted sum), i.e. it is the
    rotation of tau(B) copied into every block.
    with_conj: returns x + conj(x) of that sum x: every term of the giant-step sum enters a second time under its
    Galois element times 2N - 1 (d1 of U_0, which needs no key switch in x, under the conjugation key)."""
    from .oracle import Ct
    ru = cu * w
    g = bsgs_baby_count(units)
    ext_a, ext_b = orc.modup(a.data[1]), orc.modup(b_low.data[1])
    copies = orc.slots // spread_block if spread_block else 1
    bb = []
    for i1 in range(g):
        terms = [(ext_b, b_low.data[0], (i1 * ru - j * spread_block) % orc.slots, None)
                 for j in range(copies) if not (i1 == 0 and j == 0)]
        if not terms:
            bb.append(b_low)
            continue
        moved = Ct(orc.moddown_drop(orc.hoisted_sum(terms, b_low.nq), b_low.nq, False), b_low.scale)
        bb.append(orc.add(moved, b_low) if i1 == 0 else moved)
    ta = _assemble_shifts(orc, a, ext_a, -n,
                          [((cu * i - g * (i // g) * ru) % orc.slots, cm[2 * cu * i + 1], cm[2 * cu * i])
                           for i in range(1, units)])
    U = [acc] + [None] * (units // g - 1)
    for i in range(1, units):
        t = orc.tensor(ta[i - 1], bb[i % g])
        U[i // g] = t if U[i // g] is None else orc.add(U[i // g], t)
    # The partial sums are rescaled first (three polynomials each), then one hoisted sum for everything, a level lower:
    # U_0 gives its d2 under the multiplication key (no rotation) and its d1, times P, is added to the second polynomial
    # of the sum before the plain ModDown
    U = [orc.rescale(u) for u in U]
    lo = b_low.nq - 1
    terms = [(orc.modup(U[0].data[2]), U[0].data[0], ("mult", 1), None)]
    for i2 in range(1, units // g):
        gal = orc.galois((i2 * g * ru) % orc.slots)
        u = U[i2]
        terms.append((orc.modup(u.data[1]), u.data[0], ("g", gal), None))
        terms.append((orc.modup(u.data[2]), None, ("sq", gal), None))
    if with_conj:
        cj, two_n = 2 * orc.N - 1, 2 * orc.N
        for i2 in range(units // g):
            gal = 1 if i2 == 0 else orc.galois((i2 * g * ru) % orc.slots)
            u = U[i2]
            terms.append((orc.modup(u.data[1]), u.data[0], ("g", gal * cj % two_n), None))
            terms.append((orc.modup(u.data[2]), None, ("sq", gal * cj % two_n), None))
    y = orc.hoisted_sum(terms, lo)
    y[1, :lo] = orc.add_residues(y[1, :lo], orc.mul_p_residues(U[0].data[1]))
    return Ct(orc.moddown_drop(y, lo, False), orc.delta[b_low.level - 1])


def mult_mat_mat_cc_fused(orc, a, b, T, n, w, single_tile=False):
    """single_tile: both operands hold one tile block and nothing else; tau(B) is then taken as copied into
    every block (the copies are gathered by the baby rotations), which makes its row shifts exact rotations."""
    from .oracle import Ct
    ev = OracleEval(orc)
    cm = [orc.encode_ext(m, T + 2) for m in col_masks(n, orc.slots)]
    lvl = min(a.level, b.level)            # both operands take the same route (they share the launches)
    a = lower_and_transform_fused(orc, orc.level_down(a, min(lvl, T + 4)), H, n, w, T + 2)
    b = lower_and_transform_fused(orc, orc.level_down(b, min(lvl, T + 4)), V, n, w, T + 2)
    # the k = 0 term joins the accumulator at the shifts' level
    b_low = orc.level_down_one(b)
    acc = orc.tensor(orc.level_down_one(a), b_low)
    ext_a = orc.modup(a.data[1])
    spread = single_tile and n * w < orc.slots and orc.slots % (n * w) == 0
    if n * w == orc.slots or spread:
        # The tile block fills the slot vector: row shifts are exact rotations rho^(k w) of tau(B) lowered to
        # T+1 (no mask, plain ModDown), which allows the baby-step / giant-step split k = k1 + g k2:
        #   C = sum_k2 rho^(g k2 w)(U_k2),  U_k2 = sum_k1 rho^(-g k2 w)(phi^k(sigma A)) (x) rho^(k1 w)(tau B).
        # The column shifts come out already rotated back by g k2 rows (another Galois element, same masks);
        # the un-relinearised U_k2 are rotated directly: d1 with the key of rho(s), d2 with a key of
        # rho(s)^2, all summed in the extended basis before one ModDown merged with the rescale.
        return _bsgs_shift_product(orc, a, b_low, acc, cm, n, n, 1, w, n * w if spread else 0)
    else:
        ta = _assemble_shifts(orc, a, ext_a, -n, [(i, cm[2 * i + 1], cm[2 * i]) for i in range(1, n)])
        rm = [orc.encode_ext(m, T + 2) for m in row_masks(n, w, orc.slots)]
        ext_b = orc.modup(b.data[1])
        tb = _assemble_shifts(orc, b, ext_b, -n * w, [(i * w, rm[2 * i + 1], rm[2 * i]) for i in range(1, n)])
    for x, y in zip(ta, tb):
        acc = orc.add(acc, orc.tensor(x, y))
    return orc.rescale(orc.relinearize(acc))


def mult_packed_mat_mat_fused(orc, a, b, T, n, w, single_tile=False, merge_packing=False, with_conj=False,
                              own_levels=False, first_stage=1):
    """single_tile: the operands hold one tile block and nothing else (see mult_mat_mat_cc_fused).
    merge_packing: a and b are NOT packed yet; the packing and the packed transform run as one composite one-stage
    transform from T+3 (kinds PKH / PKV).
    with_conj: returns x + conj(x) of the product x -- inside the giant-step sum where the schedule has one, by a
    conjugation afterwards otherwise.
    own_levels: sigma(A) ends at T+2 and tau(B) at T+1 from whatever levels they arrive at (the form for operands one
    level apart).
    first_stage = 2: a and b (at T+3) are what packing_stage_one left; only the second transform stage runs here."""
    from .oracle import Ct
    ev = OracleEval(orc)
    cm = [orc.encode_ext(m, T + 2) for m in col_masks(n, orc.slots)]
    spread = single_tile and n * w < orc.slots and orc.slots % (n * w) == 0
    lvl = min(a.level, b.level)
    rows, cols = _dims(n)
    # square tiles with A four and B three levels above the target take their own ways too (truncated to T+4 / T+3)
    if (first_stage == 1 and not merge_packing and a.level >= T + 4 and b.level >= T + 3 and rows == cols
            and n // 2 >= 4 and (n * w == orc.slots or spread)):
        own_levels = True
    if not own_levels and (merge_packing or lvl >= T + 3):
        if merge_packing:
            a = diagonal_transform_fused(orc, orc.level_down(a, T + 3), PKH, n, w)
            b = diagonal_transform_fused(orc, orc.level_down(b, T + 3), PKV, n, w)
        elif first_stage == 2:
            assert a.level == T + 3 == b.level
            a = diagonal_transform_two_stage(orc, a, PH, n, w, first_stage=2)
            b = diagonal_transform_two_stage(orc, b, PV, n, w, first_stage=2)
        # both operands a level above what B needs: sigma and tau share one launch chain and both end at T+2, as in
        # the unpacked product; tau(B) is lowered to T+1 with sigma(A)'s copy for the unshifted term
        else:
            a = lower_and_transform_fused(orc, orc.level_down(a, min(lvl, T + 4)), PH, n, w, T + 2)
            b = lower_and_transform_fused(orc, orc.level_down(b, min(lvl, T + 4)), PV, n, w, T + 2)
        if n * w != orc.slots and not spread:
            # row shifts wrap inside a tile block (stacked tiles, content not known to be a single tile): every shift
            # of tau(B) by a cell of two rows is a masked pair like the column shifts of sigma(A), n / 2 - 1 of each
            acc = orc.tensor(orc.level_down_one(a), orc.level_down_one(b))
            rm = [orc.encode_ext(m, T + 2) for m in row_masks(n, w, orc.slots)]
            ta = _assemble_shifts(orc, a, orc.modup(a.data[1]), -n,
                                  [(2 * i, cm[4 * i + 1], cm[4 * i]) for i in range(1, n // 2)])
            tb = _assemble_shifts(orc, b, orc.modup(b.data[1]), -n * w,
                                  [(2 * i * w, rm[4 * i + 1], rm[4 * i]) for i in range(1, n // 2)])
            for x, y in zip(ta, tb):
                acc = orc.add(acc, orc.tensor(x, y))
            res = orc.rescale(orc.relinearize(acc))
            return repack_cc(ev, res) if with_conj else res
        b = orc.level_down_one(b)
    else:
        a = lower_and_transform_fused(orc, a, PH, n, w, T + 2)
        b = lower_and_transform_fused(orc, b, PV, n, w, T + 1)
    # the k = 0 term joins the accumulator at the shifts' level
    acc = orc.tensor(orc.level_down_one(a), b)
    return _bsgs_shift_product(orc, a, b, acc, cm, n, n // 2, 2, w, n * w if spread else 0, with_conj)


def packing_maps(slots, w, rows):
    """The complex packing as a linear map on the slots, out = Z x + sum_r M_r rho^r(x):
    columns: fus = m (x + i rho^1 x), out = fus + rho^-1 fus with m = even columns;
    rows:    fus = m (x - i rho^w x), out = fus + rho^-w fus with m = even rows of width w.
    Returns (Z, [(r, M_r)])."""
    s = np.arange(slots)
    if rows:
        m = ((s // w) % 2 == 0).astype(np.complex128)
        prev = np.roll(m, w)
        return m - 1j * prev, [(w, -1j * m), (-w, prev)]
    m = (s % 2 == 0).astype(np.complex128)
    prev = np.roll(m, 1)
    return m + 1j * prev, [(1, 1j * m), (-1, prev)]


def complex_packing_hoisted(orc, x, w, rows):
    """complexPackingInplace / complexPackingRowInplace as ONE hoisted sum (both rotations from one ModUp and Z x as a
    term without a key switch, masks applied in the extended basis, ModDown merged with the rescale): one level, like
    the reference's two masked steps.  x may be a truncated ciphertext that still carries the scale of a higher level:
    the masks are then encoded at Delta_(l-1) q_l / scale(x) instead of Delta_l, so that the result has the fixed
    scale of level l - 1 without a levelDown in front."""
    from .oracle import Ct
    zmask, terms = packing_maps(orc.slots, w, rows)
    nq, lvl = x.nq, x.level
    ms = orc.delta[lvl] if x.scale == orc.delta[lvl] else orc.delta[lvl - 1] * float(orc.q[lvl]) / x.scale
    ext = orc.modup(x.data[1])
    y = orc.hoisted_sum([(ext, x.data[0], r % orc.slots, orc.encode_ext(m, lvl, ms)) for r, m in terms] +
                        [(x.data[1], x.data[0], ("none",), orc.encode_ext(zmask, lvl, ms))], nq)
    return Ct(orc.moddown_drop(y, nq, True), orc.delta[lvl - 1])


def mult_mat_mat_cc_packed(orc, a, b, T, n, w, single_tile):
    """mult_mat_mat_cc_packed_single for operands that may hold stacked tiles (single_tile = False): the packing and
    the transforms act on every tile block alike, the cells shift through masked pairs, and each block of the result
    is the product of the operands' blocks."""
    from .oracle import Ct
    ev = OracleEval(orc)
    cut = lambda x, lvl: Ct(np.ascontiguousarray(x.data[:, : lvl + 1]), x.scale)
    spread = single_tile and n * w < orc.slots and orc.slots % (n * w) == 0
    rows, cols = _dims(n)
    assert min(a.level, b.level) >= T + 3
    if rows == cols and n // 2 >= 4 and (n * w == orc.slots or spread):
        # exact row rotations: the operands go their own ways to T+2 (sigma(A)) and T+1 (tau(B)) -- side by side on the
        # GPU -- and only A's copy for the unshifted term is lowered.  Operands above the level their way starts from
        # are only truncated to it.
        if a.level >= T + 5 and b.level >= T + 4:
            # separate packing: B packed at T+4 and transformed in two stages, A packed at T+5 and transformed in two
            pa = complex_packing_hoisted(orc, cut(a, T + 5), w, rows=False)
            pb = complex_packing_hoisted(orc, cut(b, T + 4), w, rows=True)
            return mult_packed_mat_mat_fused(orc, pa, pb, T, n, w, single_tile=single_tile, with_conj=True,
                                             own_levels=True)
        # a level less than that: the packing and the first transform stage as one composite map, then the second
        # stage (B from T+3, A from T+4); an A at T+3 has one level for both: the composite one-stage transform
        tb = diagonal_transform_two_stage(orc, packing_stage_one(orc, cut(b, T + 3), PV, n, w, b.level), PV, n, w,
                                          first_stage=2)
        if a.level >= T + 4:
            sa = diagonal_transform_two_stage(orc, packing_stage_one(orc, cut(a, T + 4), PH, n, w, a.level), PH, n, w,
                                              first_stage=2)
        else:
            sa = diagonal_transform_fused(orc, a, PKH, n, w)
        cm = [orc.encode_ext(m, T + 2) for m in col_masks(n, orc.slots)]
        acc = orc.tensor(orc.level_down_one(sa), tb)
        return _bsgs_shift_product(orc, sa, tb, acc, cm, n, n // 2, 2, w, n * w if spread else 0, True)
    if min(a.level, b.level) == T + 3:   # one level short of a separate packing: packing and transform as one map
        return mult_packed_mat_mat_fused(orc, a, b, T, n, w, single_tile=single_tile, merge_packing=True, with_conj=True)
    lvl = min(a.level, b.level, T + 5)
    if lvl == T + 4 and rows == cols and n // 2 >= 4:
        # a level short of a separate packing in front of two-stage transforms: the packing and the first stage as one
        # composite map for both operands (T+4 -> T+3); the product runs the second stage
        pa = packing_stage_one(orc, cut(a, lvl), PH, n, w, a.level)
        pb = packing_stage_one(orc, cut(b, lvl), PV, n, w, b.level)
        return mult_packed_mat_mat_fused(orc, pa, pb, T, n, w, single_tile=single_tile, with_conj=True, first_stage=2)
    pa = complex_packing_hoisted(orc, cut(a, lvl), w, rows=False)
    pb = complex_packing_hoisted(orc, cut(b, lvl), w, rows=True)
    return mult_packed_mat_mat_fused(orc, pa, pb, T, n, w, single_tile=single_tile, with_conj=True)


def mult_mat_mat_cc_packed_single(orc, a, b, T, n, w):
    """One product through the complex-packed route: adjacent columns of A and adjacent rows of B are fused into
    complex slots (complexPackingInplace / complexPackingRowInplace, one level), the packed product then needs n / 2
    shifts instead of n, and x + conj(x) returns the real product (repackCC).  For operands that hold a single tile.
    Operands above the packing level are only truncated to it (the packing masks absorb the change of scale);
    operands three levels above the target take the packing and the packed transform as one composite transform."""
    return mult_mat_mat_cc_packed(orc, a, b, T, n, w, single_tile=True)


def mult_mat_mat_pre_fused(orc, a, T, n, w, first_block_only=False):
    """first_block_only: every mask (shift 0 included) is zero outside the first n * w slots."""
    masks = col_masks(n, orc.slots)
    block = np.zeros(orc.slots, dtype=np.complex128)
    block[: min(n * w, orc.slots)] = 1
    if first_block_only:
        masks = [m * block for m in masks]
    cm = [orc.encode_ext(m, T + 2) for m in masks]
    a = lower_and_transform_fused(orc, a, H, n, w, T + 2)
    ext = orc.modup(a.data[1])
    first = OracleEval(orc).mult_pt(a, orc.encode(block, T + 2)) if first_block_only else orc.level_down_one(a)
    return [first] + _assemble_shifts(
        orc, a, ext, -n, [(i, cm[2 * i + 1], cm[2 * i]) for i in range(1, n)])


def mult_mat_mat_pc_fused(orc, a, b_pt, T, n, w):
    """Batched plaintext x ciphertext product: hoisted column shifts of sigma(A), then
    rescale(sum_k shift_k (.) rot(tau(B), k w)).  The row shift of tau(B) is a whole rotation when all
    tile blocks (n * w slots) of the plaintext are equal; a plaintext that is zero outside its first block
    gets tau of that block copied into every block and masks restricted to the first block ("zero" and "equal"
    up to 2^-24).  Returns None
    for plaintexts of any other form (the product then takes the reference order)."""
    ev = OracleEval(orc)
    slots, block = orc.slots, n * w
    if block > slots or slots % block:
        return None
    v = ev.pt_values(b_pt)
    blocks = v.reshape(slots // block, block)
    tol = 2.0 ** -24            # decoded values carry the encoding's rounding noise
    rest_zero = bool(np.all(np.abs(blocks[1:]) < tol))
    rest_equal = bool(np.all(np.abs(blocks[1:] - blocks[0]) < tol))
    if not (rest_zero or rest_equal):
        return None
    first_block_only = rest_zero and block < slots
    if first_block_only:
        v = np.tile(blocks[0], slots // block)
    tmp = mult_mat_mat_pre_fused(orc, a, T, n, w, first_block_only)
    b = ev.encode(tau_plain(v, n, w), T + 1)
    return mult_mat_mat_reuse(ev, tmp, b, T, step=w)


def mult_packed_mat_mat_pre_rot_fused(orc, a, T, n, w):
    """multPackedMatMatPreRot through the hoisted launches: a = packed sigma(A) at level T+2 -> its n/2 column shifts
    (two columns each) at level T+1."""
    cm = [orc.encode_ext(m, T + 2) for m in col_masks(n, orc.slots)]
    ext = orc.modup(a.data[1])
    return [orc.level_down_one(a)] + _assemble_shifts(
        orc, a, ext, -n, [(2 * i, cm[4 * i + 1], cm[4 * i]) for i in range(1, n // 2)])


def mult_mat_mat_cc_reuse_fused(orc, tmp, b, step, rescale_after=False):
    """Batched ciphertext x ciphertext re-use product: sum_k tmp[k] (x) rho^(k step)(b), every rotation of b taken from
    one ModUp through its direct key (automorphism after ModUp, plain ModDown), relinearised at the end (packed
    form: rescaled as well)."""
    from .oracle import Ct
    ext = orc.modup(b.data[1])
    acc = orc.tensor(tmp[0], b)
    for k in range(1, len(tmp)):
        y = orc.hoisted_sum([(ext, b.data[0], (k * step) % orc.slots, None)], b.nq)
        acc = orc.add(acc, orc.tensor(tmp[k], Ct(orc.moddown_drop(y, b.nq, False), b.scale)))
    res = orc.relinearize(acc)
    return orc.rescale(res) if rescale_after else res


def mult_mat_mat_pc_lazy(orc, a, b_pt, T, n, w):
    """Plaintext x ciphertext product with ONE ModDown: every column shift of sigma(A) stays in the extended basis,
    is multiplied there by its column mask and by tau(B) rotated k w slots (a plaintext over the extended basis,
    encoded at the scale of level T+1), all n - 1 shifts are summed, the unshifted term P * (mask_0 tau(B)) sigma(A)
    is added on the chain limbs, and the sum is divided by P q_{T+2} (ModDown merged with the first rescale) and
    rescaled once more.  Same layout rules as mult_mat_mat_pc_fused; None for other plaintexts."""
    from .oracle import Ct, Pt
    ev = OracleEval(orc)
    slots, block = orc.slots, n * w
    if block > slots or slots % block:
        return None
    v = ev.pt_values(b_pt)
    blocks = v.reshape(slots // block, block)
    tol = 2.0 ** -24
    rest_zero = bool(np.all(np.abs(blocks[1:]) < tol))
    rest_equal = bool(np.all(np.abs(blocks[1:] - blocks[0]) < tol))
    if not (rest_zero or rest_equal):
        return None
    first_block_only = rest_zero and block < slots
    if first_block_only:
        v = np.tile(blocks[0], slots // block)
    masks = col_masks(n, slots)
    if first_block_only:
        keep = np.zeros(slots, dtype=np.complex128)
        keep[: min(block, slots)] = 1
        masks = [m * keep for m in masks]
    cm = [orc.encode_ext(m, T + 2) for m in masks]
    tau = orc.encode_ext(tau_plain(v, n, w), T + 2, scale=orc.delta[T + 1])
    a = lower_and_transform_fused(orc, a, H, n, w, T + 2)
    nq = a.nq
    ext = orc.modup(a.data[1])
    a2 = _rotated_copy(orc, a, ext, -n)
    ext2 = orc.modup(a2.data[1])
    terms = []
    for i in range(1, n):
        gp = orc.galois((i * w) % slots)
        terms.append((ext, a.data[0], i % slots, orc.ext_plain_product(cm[2 * i + 1], tau, gp)))
        terms.append((ext2, a2.data[0], i % slots, orc.ext_plain_product(cm[2 * i], tau, gp)))
    y = orc.hoisted_sum(terms, nq)
    # shift 0: P * (mask_0 * tau(B)) * sigma(A) on the chain limbs (zero on the special limbs)
    m0 = orc.ext_plain_product(cm[1], tau, 1)
    t0 = orc.mult_plain_no_rescale(a, Pt(m0.data[:nq], m0.scale))
    for pol in range(2):
        y[pol, :nq] = orc.add_residues(y[pol, :nq], orc.mul_p_residues(np.ascontiguousarray(t0.data[pol])))
    mid = Ct(orc.moddown_drop(y, nq, True), orc.delta[T + 1] * orc.delta[T + 1])
    res = orc.rescale(mid)
    res.scale = orc.delta[T]
    return res


def weights_diagonal_to_row4(w1, w2, w3, w4, slots):
    """HEMMer::msgDiagonalToRow4 (HEMMer.cpp:353-399)."""
    h, w = w1.shape
    msg = np.zeros(slots, dtype=np.complex128)
    left = 0.5 * (w1 - 1j * w3)
    right = 0.5 * (w2 - 1j * w4)
    for c in range(w):
        msg[np.arange(h) * 2 * w + c] = np.roll(left[:, c], -c)
        msg[np.arange(h) * 2 * w + w + c] = np.roll(right[:, c], -c)
    return msg


# ---- LoRA low-rank products (MatrixUtils.cpp:1681-1996) and their repacking (HEMMer.cpp:1055-1091, 2131-2332) ------
LOW_DIM = 2            # ModelArgs::LOW_DIM (ModelArgs.hpp:67)


def _low_rank_terms(ev, a, b, T, sa, sb, w, low_dim):
    """Shared tail of the three products: sigma(A) (.) tau(B) plus the low_dim - 1 shifted terms
    (e.g. :1716-1766): the full product's loop cut after low_dim terms."""
    cm = col_masks(sa[1], ev.slots)
    rm = row_masks(sb[0], w, ev.slots)
    res = ev.mult(a, b)
    a = ev.left_rotate(a, 1)
    b = ev.left_rotate(b, w)
    a_wrap = ev.right_rotate(a, w // 2)
    b_wrap = ev.right_rotate(b, sa[0] * w)
    acc = None
    for i in range(1, low_dim):
        if i > 1:
            a = ev.left_rotate(a, 1)
            a_wrap = ev.left_rotate(a_wrap, 1)
            b = ev.left_rotate(b, w)
            b_wrap = ev.left_rotate(b_wrap, w)
        enc = lambda m: ev.encode(m, T + 2)
        t1 = ev.rescale(ev.masked_sum(a, enc(cm[2 * i + 1]), a_wrap, enc(cm[2 * i])))
        t2 = ev.rescale(ev.masked_sum(b, enc(rm[2 * i + 1]), b_wrap, enc(rm[2 * i])))
        t = ev.tensor(t1, t2)
        acc = t if acc is None else ev.add(acc, t)
    if acc is None:
        return res
    return ev.add(res, ev.rescale(ev.relinearize(acc)))


def _lora_transform(ev, x, kind, shape, w, T, fused_orc):
    """Transform of an operand ending at T+2: reference order from T+3, or the batched form (two stages when
    the operand is high enough)."""
    if fused_orc is not None:
        return lower_and_transform_fused(fused_orc, x, kind, shape, w, T + 2)
    return diagonal_transform(ev, ev.level_down(x, T + 3), kind, shape, w)


def mult_mat_mat_high_low(ev, a, b, in_col_block, T, sa, sb, w, low_dim=LOW_DIM, fused_orc=None):
    """multMatMatHighLow (:1681-1770).  sa, sb = (rows, cols) of the operands' tile shapes.  B holds low_dim
    columns at column block in_col_block of every tile; tau runs on (rows, low_dim) tiles and the
    result is spread along the diagonal of column blocks before the truncated product."""
    a = _lora_transform(ev, a, H, sa, w, T, fused_orc)
    b = _lora_transform(ev, b, V, (sb[0], low_dim), w, T, fused_orc)
    pos, i = in_col_block, low_dim
    while i < w // 2:
        if pos % 2 == 0:
            tmp = ev.right_rotate(ev.left_rotate(b, i * w), i)
        else:
            tmp = ev.left_rotate(b, i)
            b = ev.left_rotate(b, i * w)
        b = ev.add(b, tmp)
        pos //= 2
        i <<= 1
    return _low_rank_terms(ev, a, b, T, sa, sb, w, low_dim)


def mult_mat_mat_low_high(ev, a, b, in_row_block, T, sa, sb, w, low_dim=LOW_DIM, fused_orc=None):
    """multMatMatLowHigh (:1772-1876): A holds low_dim rows at row block in_row_block; they are copied to
    every row block before sigma."""
    start = T + 4 if fused_orc is not None and min(ev.level_of(a), ev.level_of(b)) >= T + 4 else T + 3
    a = ev.level_down(a, start)
    pos, i = in_row_block, low_dim
    while i < w // 2:
        tmp = ev.right_rotate(a, i * w) if pos % 2 == 0 else ev.left_rotate(a, i * w)
        a = ev.add(a, tmp)
        pos //= 2
        i <<= 1
    a = _lora_transform(ev, a, H, sa, w, T, fused_orc)
    b = _lora_transform(ev, b, V, sb, w, T, fused_orc)
    return _low_rank_terms(ev, a, b, T, sa, sb, w, low_dim)


def mult_mat_mat_low_low(ev, a, b, in_col_block, in_row_block, T, sa, sb, w, low_dim=LOW_DIM, fused_orc=None):
    """multMatMatLowLow (:1878-1996): A (rows x low_dim at column block in_col_block) times B (low_dim x cols
    at row block in_row_block); sigma / tau run on the thin shapes and are then copied over the blocks."""
    a = _lora_transform(ev, a, H, (sa[0], low_dim), w, T, fused_orc)
    b = _lora_transform(ev, b, V, (low_dim, sb[1]), w, T, fused_orc)
    cpos, rpos, i = in_col_block, in_row_block, low_dim
    while i < w // 2:
        tmp = ev.right_rotate(a, i) if cpos % 2 == 0 else ev.left_rotate(a, i)
        a = ev.add(a, tmp)
        cpos //= 2
        tmp = ev.right_rotate(b, i * w) if rpos % 2 == 0 else ev.left_rotate(b, i * w)
        b = ev.add(b, tmp)
        rpos //= 2
        i <<= 1
    return _low_rank_terms(ev, a, b, T, sa, sb, w, low_dim)


def _mult_msg(ev, x, msg):
    return ev.mult_pt(x, ev.encode(msg, ev.level_of(x)))


def low_col_block_mask(rows, cols, w, block, slots, low_dim=LOW_DIM, every_tile=True):
    m = np.zeros(slots, dtype=np.complex128)
    for i in range(rows):
        for k in range(0, w if every_tile else 1, cols):
            m[i * w + k + block * low_dim: i * w + k + (block + 1) * low_dim] = 1
    return m


def low_row_block_mask(cols, w, block, slots, low_dim=LOW_DIM, width=None):
    m = np.zeros(slots, dtype=np.complex128)
    for i in range(block * low_dim, (block + 1) * low_dim):
        m[i * w: i * w + (w if width is None else width)] = 1
    return m


def get_low_col_block(ev, x, block, rows, cols, w, low_dim=LOW_DIM):
    """HEMMer::getLowColBlock (HEMMer.cpp:2294-2312)."""
    return _mult_msg(ev, x, low_col_block_mask(rows, cols, w, block, ev.slots, low_dim))


def get_low_row_block(ev, x, block, cols, w, low_dim=LOW_DIM):
    """HEMMer::getLowRowBlock (HEMMer.cpp:2314-2332)."""
    return _mult_msg(ev, x, low_row_block_mask(cols, w, block, ev.slots, low_dim))


def repack_to_one_col(ev, x, out_block, rows, cols, w, low_dim=LOW_DIM):
    """HEMMer::repackToOneCol (HEMMer.cpp:2137-2178)."""
    pos, i = out_block, low_dim
    while i < w:
        x = ev.add(x, ev.left_rotate(x, i) if pos % 2 == 0 else ev.right_rotate(x, i))
        pos //= 2
        i <<= 1
    x = _mult_msg(ev, x, low_col_block_mask(rows, cols, w, out_block, ev.slots, low_dim, every_tile=False))
    i = cols
    while i < w:
        x = ev.add(x, ev.right_rotate(x, cols))
        i <<= 1
    return x


def repack_to_multi_col(ev, x, out_block, rows, cols, w, low_dim=LOW_DIM):
    """HEMMer::repackToMultiCol (HEMMer.cpp:2180-2215)."""
    pos, i = out_block, low_dim
    while i < w // 2:
        x = ev.add(x, ev.left_rotate(x, i) if pos % 2 == 0 else ev.right_rotate(x, i))
        pos //= 2
        i <<= 1
    return _mult_msg(ev, x, low_col_block_mask(rows, cols, w, out_block, ev.slots, low_dim))


def repack_to_one_row(ev, x, out_block, rows, cols, w, low_dim=LOW_DIM):
    """HEMMer::repackToOneRow (HEMMer.cpp:2217-2259)."""
    pos, i = out_block, low_dim
    while i < rows:
        x = ev.add(x, ev.left_rotate(x, i * w) if pos % 2 == 0 else ev.right_rotate(x, i * w))
        pos //= 2
        i <<= 1
    i = cols
    while i < w:
        x = ev.add(x, ev.left_rotate(x, cols))
        i <<= 1
    x = _mult_msg(ev, x, low_row_block_mask(cols, w, out_block, ev.slots, low_dim, width=cols))
    i = cols
    while i < w:
        x = ev.add(x, ev.right_rotate(x, cols))
        i += cols
    return x


def repack_to_multi_row(ev, x, out_block, rows, w, low_dim=LOW_DIM):
    """HEMMer::repackToMultiRow (HEMMer.cpp:2261-2292)."""
    pos, i = out_block, low_dim
    while i < rows:
        x = ev.add(x, ev.left_rotate(x, i * w) if pos % 2 == 0 else ev.right_rotate(x, i * w))
        pos //= 2
        i <<= 1
    return _mult_msg(ev, x, low_row_block_mask(0, w, out_block, ev.slots, low_dim))


def repack_lora_opti(ev, t1, t2, n):
    """HEMMer::repack_loraOpti (HEMMer.cpp:1055-1091); both inputs arrive un-rescaled."""
    t1, t2 = ev.rescale(t1), ev.rescale(t2)
    out = ev.add(t1, ev.conjugate(t1))
    tmp = ev.mult_imag_unit(ev.add(t2, ev.conjugate(t2)))
    out = ev.add(out, tmp)
    tmp = ev.left_rotate(out, n)
    out = ev.add(out, tmp)
    conj = ev.conjugate(out)
    out = ev.add(out, conj)
    tmp = ev.mult_imag_unit(ev.sub(conj, tmp))
    half = _message2(np.full((n, n), 0.5), np.zeros((n, n)), ev.slots)
    tmp = _mult_msg(ev, tmp, half)
    out = _mult_msg(ev, out, half)
    return ev.add(out, ev.right_rotate(tmp, n))


def repack_not_bts(ev, t1, t2, n, rescale_first=True):
    """HEMMer::repack_notBTS (HEMMer.cpp:1025-1053): 2 Re(t1) + 2i Re(t2), the halves folded by a rotation of n,
    the left columns kept and the second half put back beside them.  rescale_first: the reference rescales both inputs
    (they arrive un-rescaled from a product); callers with rescaled inputs skip that step."""
    if rescale_first:
        t1, t2 = ev.rescale(t1), ev.rescale(t2)
    out = ev.add(t1, ev.conjugate(t1))
    tmp = ev.mult_imag_unit(ev.add(t2, ev.conjugate(t2)))
    out = ev.add(out, tmp)
    tmp = ev.left_rotate(out, n)
    out = ev.add(out, tmp)
    left = _message2(np.ones((n, n)), np.zeros((n, n)), ev.slots)        # mask_matmul_ (HEMMer.cpp:167-176)
    tmp = _mult_msg(ev, tmp, left)
    out = _mult_msg(ev, out, left)
    return ev.add(out, ev.right_rotate(tmp, n))


def split_in_two(ev, t, n):
    """HEMMer::splitInTwo (HEMMer.cpp:819-831): [A | B] -> [A | A], [B | B] (the unmasked operand is lowered to the
    product's level before the subtraction, as HomEvaluator::sub does with operands of two levels)."""
    left = _message2(np.ones((n, n)), np.zeros((n, n)), ev.slots)        # mask_left_half_
    tmp = _mult_msg(ev, t, left)
    t2 = ev.sub(ev.level_down(t, ev.level_of(tmp)), tmp)
    t1 = ev.add(ev.right_rotate(tmp, n), tmp)
    t2 = ev.add(t2, ev.left_rotate(t2, n))
    return t1, t2


# ---- rank-2 LoRA through element-wise products (TransformerBlock.cpp:2199-2365) ------------------------------------
def _first_row_mask(n, slots):
    m = np.zeros((n, n))
    m[0] = 1
    return _message2(m, m, slots)


def _first_col_only_mask(n, slots):
    m = np.zeros((n, n))
    m[:, 0] = 1
    return _message2(m, np.zeros((n, n)), slots)


def _split_weight_rows(ev, wt, count, n, w, hoisted=False):
    """Rows 2i and 2i+1 of the weight tile, each moved to row 0, masked and copied to all n rows
    (:2222-2251, :2294-2335)."""
    first = _first_row_mask(n, ev.slots)
    out = []
    for i in range(count):
        t = wt if i == 0 else ev.left_rotate(wt, i * 2 * w)
        pair = [_mult_msg(ev, t, first), _mult_msg(ev, ev.left_rotate(t, w), first)]
        out.append(pair)
    for pair in out:
        for j in range(2):
            if hoisted:
                pair[j] = ev.rotate_sum(pair[j], -w, n)
                continue
            rot = 1
            while rot < n:
                pair[j] = ev.add(pair[j], ev.right_rotate(pair[j], rot * w))
                rot <<= 1
    return out


def lora_rank2_down(ev, cur, wa, n, w, weight_level, hoisted=False):
    """X a_0 and X a_1 in column 0 of the left tile: row 2i+j of `wa` holds column j of A for the i-th pair
    of activation tiles (:2203-2283).  hoisted: every rotate-and-sum as hoisted sums (the batched schedule)."""
    wa = ev.level_down(wa, weight_level)
    wts = _split_weight_rows(ev, wa, len(cur), n, w, hoisted)
    out = []
    for j in range(2):
        acc = None
        for i, x in enumerate(cur):
            t = ev.mult(x, wts[i][j])
            acc = t if acc is None else ev.add(acc, t)
        if hoisted:
            acc = ev.rotate_sum(acc, 1, w)
        else:
            rot = 1
            while rot < w:
                acc = ev.add(acc, ev.left_rotate(acc, rot))
                rot <<= 1
        out.append(_mult_msg(ev, acc, _first_col_only_mask(n, ev.slots)))
    return out


def lora_rank2_up(ev, xa, wb, n_out, n, w, weight_level, hoisted=False):
    """(X A) B for n_out pairs of output tiles: row 2i+j of `wb` holds row j of B for output pair i
    (:2287-2358)."""
    wb = ev.level_down(wb, weight_level)
    wts = _split_weight_rows(ev, wb, n_out, n, w, hoisted)
    xa = list(xa)
    for j in range(2):
        if hoisted:
            xa[j] = ev.rotate_sum(xa[j], -1, w)
            continue
        rot = 1
        while rot < w:
            xa[j] = ev.add(xa[j], ev.right_rotate(xa[j], rot))
            rot <<= 1
    return [ev.add(ev.mult(xa[0], wts[i][0]), ev.mult(xa[1], wts[i][1])) for i in range(n_out)]


# ---- rotate-and-sum reductions on the pair layout (HEMMer.cpp:2512-2530, 882-919, 1245-1253, 1699-1760) -----------
def _message2(a, b, slots):
    """HEMMer::message2 (HEMMer.cpp:243-262): [A | B] row-major with block width 2 * cols."""
    n = a.shape[1]
    m = np.zeros(slots, dtype=np.complex128)
    m[: 2 * a.size] = np.concatenate([a, b], axis=1).reshape(-1)
    return m


def reduce_row_sum_with_scaled_mask(ev, x, mask_msg, w, hoisted=False):
    if hoisted:
        x = ev.rotate_sum(x, 1, w)
        x = ev.mult_pt(x, ev.encode(mask_msg, ev.level_of(x)))
        return ev.rotate_sum(x, -1, w)
    i = 1
    while i < w:
        x = ev.add(x, ev.left_rotate(x, i))
        i <<= 1
    x = ev.mult_pt(x, ev.encode(mask_msg, ev.level_of(x)))
    i = 1
    while i < w:
        x = ev.add(x, ev.right_rotate(x, i))
        i <<= 1
    return x


def one_mat_rot_sum(ev, a, b, n, hoisted=False):
    first, last = np.zeros((n, n)), np.zeros((n, n))
    first[:, 0] = 1.0
    last[:, n - 1] = 1.0
    if hoisted:
        a, b = ev.rotate_sum(a, 1, n // 2), ev.rotate_sum(b, -1, n // 2)
        a = ev.mult_pt(a, ev.encode(_message2(first, first, ev.slots), ev.level_of(a)))
        b = ev.mult_pt(b, ev.encode(_message2(last, last, ev.slots), ev.level_of(b)))
        return ev.rotate_sum(a, -1, n), ev.rotate_sum(b, 1, n)
    rot = 1
    while rot < n // 2:
        a = ev.add(a, ev.left_rotate(a, rot))
        b = ev.add(b, ev.right_rotate(b, rot))
        rot <<= 1
    a = ev.mult_pt(a, ev.encode(_message2(first, first, ev.slots), ev.level_of(a)))
    b = ev.mult_pt(b, ev.encode(_message2(last, last, ev.slots), ev.level_of(b)))
    rot = 1
    while rot < n:
        a = ev.add(a, ev.right_rotate(a, rot))
        b = ev.add(b, ev.left_rotate(b, rot))
        rot <<= 1
    return a, b


def mask_right_left(ev, x, n):
    left, right = np.zeros((n, n)), np.zeros((n, n))
    left[:, : n // 2] = 1.0
    right[:, n // 2:] = 1.0
    return (ev.mult_pt(x, ev.encode(_message2(left, left, ev.slots), ev.level_of(x))),
            ev.mult_pt(x, ev.encode(_message2(right, right, ev.slots), ev.level_of(x))))


def row_moments(ev, tiles, inv_count, n, hoisted=False):
    mean = tiles[0]
    sq = ev.tensor(tiles[0], tiles[0])
    for t in tiles[1:]:
        sq = ev.add(sq, ev.tensor(t, t))
        mean = ev.add(mean, t)
    sq = ev.rescale(ev.relinearize(sq))
    scaled = np.zeros((n, n))
    scaled[:, 0] = inv_count
    mask = _message2(scaled, np.zeros((n, n)), ev.slots)
    return (reduce_row_sum_with_scaled_mask(ev, mean, mask, 2 * n, hoisted),
            reduce_row_sum_with_scaled_mask(ev, sq, mask, 2 * n, hoisted))

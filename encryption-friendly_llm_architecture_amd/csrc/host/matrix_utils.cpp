// sigma / tau / transpose transforms and the matrix products of HELLM/MatrixUtils.hpp.
// Follows the algorithm of the reference's ciphertext/src/MatrixUtils.cpp (mask families :90-578,
// transforms :671-1098, products :1100-1679) restated over this build's evaluator.
#include <algorithm>
#include <cmath>
#include <cstring>

#include "HELLM/MatrixUtils.hpp"

namespace HELLM {

namespace {

i64 pow2ceil(i64 v) {
    i64 p = 1;
    while (p < v) p <<= 1;
    return p;
}

// baby-step / giant-step geometry of a transform kind
// Rectangular tiles (sigma and tau only; reference generateHorizontalMask / generateVerticalMask,
// ciphertext/src/MatrixUtils.cpp:129-217, 330-419): a diagonal wraps over the columns (sigma) or rows (tau)
// of the tile while the number of diagonals of one sign is the shorter side.
struct Geometry {
    i64 n;       // tile side (values) of a square tile; rows otherwise
    i64 rows, cols;
    i64 units;   // length a diagonal wraps over, in cells: n (plain) or n / 2 (packed)
    i64 sub;     // diagonals of one sign, in cells: min(rows, cols) / cell
    i64 cell;    // 1 or 2
    i64 bs, gs;
    i64 step;    // slots moved per unit diagonal
};

Geometry geometry(MaskKind kind, const TileTensorShape &s) {
    Geometry g{};
    const i64 rows = s.getNumRows(), cols = s.getNumCols(), w = s.getBlockWidth();
    const bool plain_sigma_tau = (kind == MaskKind::Horizontal || kind == MaskKind::Vertical);
    const bool packing = (kind == MaskKind::PackingHorizontal || kind == MaskKind::PackingVertical);
    if (rows != cols && !plain_sigma_tau)
        throw std::invalid_argument("[MatrixTransformer] packed transforms and transpose need square tiles");
    g.n = rows;
    g.rows = rows;
    g.cols = cols;
    if (kind == MaskKind::Diagonal) {
        g.sub = g.n;
        g.units = g.n;
        g.cell = 1;
        const i64 count = 2 * g.n - 1;
        g.bs = (i64)std::ceil(std::sqrt((double)count));
        g.gs = (i64)std::ceil((double)count / (double)g.bs);
        g.step = w - 1;
        return g;
    }
    const bool packed = (kind == MaskKind::PackedHorizontal || kind == MaskKind::PackedVertical);
    const bool vertical = (kind == MaskKind::Vertical || kind == MaskKind::PackedVertical || kind == MaskKind::PackingVertical);
    (void)packing;   // the composite kinds move by single columns / rows: the geometry of the plain transforms
    g.cell = packed ? 2 : 1;
    g.units = (vertical ? rows : cols) / g.cell;
    g.sub = std::min(rows, cols) / g.cell;
    g.bs = (i64)std::ceil(std::sqrt((double)(2 * g.sub - 1)));
    g.gs = (i64)std::ceil((double)(g.sub - 1) / (double)g.bs);
    g.step = kind == MaskKind::DiagonalSigned ? w - 1 : g.cell * (vertical ? w : 1);
    return g;
}

}  // namespace

Message packingMaskMessage(bool by_rows, i64 w, u64 log_slots, int part) {
    const u64 slots = u64(1) << log_slots, step = by_rows ? (u64)w : 1;
    Message m(log_slots, 0);
    const Complex iu(0, by_rows ? -1.0 : 1.0);
    for (u64 s = 0; s < slots; s++) {
        auto even = [&](u64 t) { return by_rows ? ((t / (u64)w) % 2 == 0) : (t % 2 == 0); };
        const double here = even(s) ? 1.0 : 0.0, prev = even((s + slots - step) % slots) ? 1.0 : 0.0;
        m[s] = part == 0 ? Complex(here, 0) + iu * prev : part == 1 ? iu * here : Complex(prev, 0);
    }
    return m;
}

Message transformMaskMessage(MaskKind kind, const TileTensorShape &shape, u64 log_slots, i64 idx) {
    if (kind == MaskKind::PackingHorizontal || kind == MaskKind::PackingVertical) {
        // T_packed(P(x)) = sum_d mask_d (.) rho^(2 d unit)(Z x + M_+ rho^unit x + M_- rho^-unit x): the coefficient of
        // rho^(idx unit)(x) collects the three ways of writing idx = 2 d + e
        const bool rows = kind == MaskKind::PackingVertical;
        const MaskKind base = rows ? MaskKind::PackedVertical : MaskKind::PackedHorizontal;
        const i64 w = shape.getBlockWidth(), slots = i64(1) << log_slots, unit = rows ? w : 1;
        const i64 cells = (rows ? shape.getNumRows() : shape.getNumCols()) / 2;
        Message m(log_slots, 0);
        const int parts[3] = {0, 1, 2};
        const i64 shift[3] = {0, 1, -1};
        for (int k = 0; k < 3; k++) {
            if (((idx - shift[k]) % 2) != 0) continue;
            const i64 d = (idx - shift[k]) / 2;
            if (d <= -cells || d >= cells) continue;
            const Message t = transformMaskMessage(base, shape, log_slots, d), pm = packingMaskMessage(rows, w, log_slots, parts[k]);
            const i64 r = ((2 * d * unit) % slots + slots) % slots;
            for (i64 s = 0; s < slots; s++) m[(u64)s] += t[(u64)s] * pm[(u64)((s + r) % slots)];
        }
        return m;
    }
    const Geometry g = geometry(kind, shape);
    const i64 w = shape.getBlockWidth(), slots = i64(1) << log_slots, height = slots / w;
    Message m(log_slots, 0);
    const double value = (kind == MaskKind::PackedHorizontal) ? 0.5 : 1.0;
    for (i64 r = 0; r < height; r++)
        for (i64 c = 0; c < w; c++) {
            const i64 R = (r % g.rows) / g.cell, C = (c % g.cols) / g.cell;
            bool on;
            switch (kind) {
                case MaskKind::Horizontal:
                case MaskKind::PackedHorizontal: {
                    const i64 Rs = R % g.sub;   // a tall tile repeats the pattern every `sub` rows
                    on = idx >= 0 ? (Rs == idx && C < g.units - idx) : (Rs == g.units + idx && C >= -idx);
                    break;
                }
                case MaskKind::Vertical:
                case MaskKind::PackedVertical: {
                    const i64 Cs = C % g.sub;   // a wide tile repeats it every `sub` columns
                    on = idx >= 0 ? (Cs == idx && R < g.units - idx) : (Cs == g.units + idx && R >= -idx);
                    break;
                }
                default:  // Diagonal: output positions with column - row == idx
                    on = (C - R == idx);
            }
            if (on) m[(u64)(r * w + c)] = value;
        }
    return m;
}

const Plaintext &MatrixTransformer::transformMask(const HomEvaluator &eval, MaskKind kind,
                                                  const TileTensorShape &shape, u64 level, i64 idx) {
    useChainOf(eval.getContext());
    Key key{(int)kind, shape, level, idx};
    auto it = masks_.find(key);
    if (it != masks_.end()) return it->second;
    const Context &ctx = eval.getContext();
    const u64 log_slots = getLogFullSlots(ctx);
    const Geometry g = geometry(kind, shape);
    Message m = transformMaskMessage(kind, shape, log_slots, idx);
    // pre-rotation so the mask can be applied before the giant-step rotation of its group
    if (kind == MaskKind::Diagonal) {
        const i64 i = (idx + (g.n - 1)) / g.bs;
        eval.rightRotate(m, (u64)(i * g.bs * g.step), m);
    } else if (idx > 0) {
        const i64 i = (idx - 1) / g.bs;
        eval.rightRotate(m, (u64)(i * g.bs * g.step), m);
    } else if (idx < 0) {
        const i64 i = (idx + g.units - 1) / g.bs;
        eval.leftRotate(m, (u64)((g.units - i * g.bs) * g.step), m);
    }
    auto res = masks_.emplace(key, EnDecoder(ctx).encode(m, level));
    return res.first->second;
}

std::vector<Plaintext> &MatrixTransformer::getColMask(const HomEvaluator &eval, const TileTensorShape &shape,
                                                      u64 level) {
    useChainOf(eval.getContext());
    auto key = std::make_pair(shape, level);
    auto it = col_masks_.find(key);
    if (it != col_masks_.end()) return it->second;
    const Context &ctx = eval.getContext();
    const u64 log_slots = getLogFullSlots(ctx);
    const i64 n = shape.getNumCols(), slots = i64(1) << log_slots;
    EnDecoder endec(ctx);
    std::vector<Plaintext> v;
    v.reserve((size_t)(2 * n));
    for (i64 i = 0; i < n; i++) {
        Message wrap(log_slots, 0), main(log_slots, 0);
        for (i64 j = 0; j < slots; j++) {
            if (j % n < n - i)
                main[(u64)j] = 1;
            else
                wrap[(u64)j] = 1;
        }
        v.push_back(endec.encode(wrap, level));
        v.push_back(endec.encode(main, level));
    }
    return col_masks_.emplace(key, std::move(v)).first->second;
}

std::vector<Plaintext> &MatrixTransformer::getRowMask(const HomEvaluator &eval, const TileTensorShape &shape,
                                                      u64 level) {
    useChainOf(eval.getContext());
    auto key = std::make_pair(shape, level);
    auto it = row_masks_.find(key);
    if (it != row_masks_.end()) return it->second;
    const Context &ctx = eval.getContext();
    const u64 log_slots = getLogFullSlots(ctx);
    const i64 n = shape.getNumRows(), w = shape.getBlockWidth(), slots = i64(1) << log_slots;
    EnDecoder endec(ctx);
    std::vector<Plaintext> v;
    v.reserve((size_t)(2 * n));
    for (i64 i = 0; i < n; i++) {
        Message wrap(log_slots, 0), main(log_slots, 0);
        for (i64 j = 0; j < slots; j++) {
            if ((j / w) % n < n - i)
                main[(u64)j] = 1;
            else
                wrap[(u64)j] = 1;
        }
        v.push_back(endec.encode(wrap, level));
        v.push_back(endec.encode(main, level));
    }
    return row_masks_.emplace(key, std::move(v)).first->second;
}

void MatrixTransformer::cleanUp() {
    masks_.clear();
    col_masks_.clear();
    row_masks_.clear();
    col_masks_ext_.clear();
    row_masks_ext_.clear();
    col_masks_ext_first_.clear();
    first_block_masks_.clear();
    two_stage_masks_.clear();
    packing_stage_one_masks_.clear();
    pack_masks_.clear();
    weight_tau_.clear();
    weight_tau_order_.clear();
    chain_.clear();
    last_context_ = Context();
}
size_t MatrixTransformer::cachedMasks() const {
    size_t n = masks_.size() + first_block_masks_.size() + two_stage_masks_.size() + pack_masks_.size();
    for (auto &kv : col_masks_) n += kv.second.size();
    for (auto &kv : row_masks_) n += kv.second.size();
    for (auto &kv : col_masks_ext_) n += kv.second.size();
    for (auto &kv : row_masks_ext_) n += kv.second.size();
    for (auto &kv : col_masks_ext_first_) n += kv.second.size();
    for (auto &kv : packing_stage_one_masks_) n += kv.second.size();
    return n;
}
void MatrixTransformer::useChainOf(const Context &c) {
    if (c.get() == last_context_.get()) return;
    last_context_ = c;
    std::vector<u64> sig{getDegree(c), getEncryptionLevel(c)};
    const std::vector<u64> primes = getPrimeList(c);
    sig.insert(sig.end(), primes.begin(), primes.end());
    for (Real d : getDefaultScaleFactorList(c)) {
        u64 bits;
        static_assert(sizeof(bits) == sizeof(d), "scale factors are doubles");
        std::memcpy(&bits, &d, sizeof(bits));
        sig.push_back(bits);
    }
    if (sig == chain_) return;
    if (!chain_.empty()) cleanUp();
    chain_ = std::move(sig);
    last_context_ = c;
}

// T(A) = M_0 * A + sum_{d != 0} M_d * rot_{d step}(A), d in (-units, units), grouped so that only
// bs baby rotations of A and 2 gs giant rotations of partial sums are key switched.  All products
// are summed at the doubled scale and rescaled once.
Ciphertext MatrixTransformer::diagonalTransform(const HomEvaluator &eval, const Ciphertext &in, MaskKind kind,
                                                const TileTensorShape &shape) {
    const Context &ctx = eval.getContext();
    const Geometry g = geometry(kind, shape);
    const u64 level = in.getLevel();
    if (level == 0) throw std::invalid_argument("[diagonalTransform] level >= 1 is needed.");
    std::vector<Ciphertext> baby;
    baby.reserve((size_t)g.bs);
    for (i64 j = 0; j < g.bs; j++) {
        baby.emplace_back(ctx);
        eval.leftRotate(j == 0 ? in : baby[(size_t)j - 1], (u64)g.step, baby[(size_t)j]);
    }
    Ciphertext res(ctx), group(ctx), tmp(ctx);
    eval.multWithoutRescale(in, transformMask(eval, kind, shape, level, 0), res);
    for (i64 i = 0; i < g.gs; i++) {
        // wrapped diagonals d = 1 + i bs + j - units < 0
        bool any = false;
        for (i64 j = 0; j < g.bs; j++) {
            const i64 d = 1 + i * g.bs + j - g.units;
            if (d >= g.sub - g.units) break;
            eval.multWithoutRescale(baby[(size_t)j], transformMask(eval, kind, shape, level, d), any ? tmp : group);
            if (any) eval.add(group, tmp, group);
            any = true;
        }
        if (any) {
            eval.rightRotate(group, (u64)((g.units - i * g.bs) * g.step), group);
            eval.add(res, group, res);
        }
        // diagonals d = 1 + i bs + j > 0
        any = false;
        for (i64 j = 0; j < g.bs; j++) {
            const i64 d = 1 + i * g.bs + j;
            if (d >= g.sub) break;
            eval.multWithoutRescale(baby[(size_t)j], transformMask(eval, kind, shape, level, d), any ? tmp : group);
            if (any) eval.add(group, tmp, group);
            any = true;
        }
        if (any) {
            if (i > 0) eval.leftRotate(group, (u64)(i * g.bs * g.step), group);
            eval.add(res, group, res);
        }
    }
    eval.rescale(res);
    return res;
}

template <>
CtxtTensor MatrixTransformer::diagonalToColumn<Ciphertext>(const HomEvaluator &eval, const CtxtTensor &op) {
    return CtxtTensor(op.getShape(), diagonalTransform(eval, op.get(), MaskKind::Horizontal, op.getShape()));
}
template <>
CtxtTensor MatrixTransformer::diagonalToRow<Ciphertext>(const HomEvaluator &eval, const CtxtTensor &op) {
    return CtxtTensor(op.getShape(), diagonalTransform(eval, op.get(), MaskKind::Vertical, op.getShape()));
}
CtxtTensor MatrixTransformer::packedDiagonalToColumn(const HomEvaluator &eval, const CtxtTensor &op) {
    return CtxtTensor(op.getShape(), diagonalTransform(eval, op.get(), MaskKind::PackedHorizontal, op.getShape()));
}
CtxtTensor MatrixTransformer::packedDiagonalToRow(const HomEvaluator &eval, const CtxtTensor &op) {
    return CtxtTensor(op.getShape(), diagonalTransform(eval, op.get(), MaskKind::PackedVertical, op.getShape()));
}

// plaintext operands are permuted on the host (decode -> permute -> encode)
template <>
PtxtTensor MatrixTransformer::diagonalToRow<Plaintext>(const HomEvaluator &eval, const PtxtTensor &op) {
    const Context &ctx = eval.getContext();
    EnDecoder endec(ctx);
    const Message src = endec.decode(op.get());
    Message dst(src.getLogSlots(), 0);
    const i64 n = op.getHeight(), w = op.getBlockWidth(), height = (i64)src.getSize() / w;
    for (i64 r = 0; r < height; r++)
        for (i64 c = 0; c < w; c++) {
            const i64 rb = r - r % n, cb = c - c % n, i = r % n, j = c % n;
            dst[(u64)(r * w + c)] = src[(u64)((rb + (i + j) % n) * w + cb + j)];
        }
    return PtxtTensor(op.getShape(), endec.encode(dst, op.getLevel()));
}
template <>
PtxtTensor MatrixTransformer::diagonalToColumn<Plaintext>(const HomEvaluator &eval, const PtxtTensor &op) {
    const Context &ctx = eval.getContext();
    EnDecoder endec(ctx);
    const Message src = endec.decode(op.get());
    Message dst(src.getLogSlots(), 0);
    const i64 n = op.getHeight(), w = op.getBlockWidth(), height = (i64)src.getSize() / w;
    for (i64 r = 0; r < height; r++)
        for (i64 c = 0; c < w; c++) {
            const i64 cb = c - c % n, i = r % n, j = c % n;
            dst[(u64)(r * w + c)] = src[(u64)(r * w + cb + (i + j) % n)];
        }
    return PtxtTensor(op.getShape(), endec.encode(dst, op.getLevel()));
}

// out(r, c) = in(c, r): sum over e = c - r of M_e * rot_{e (w - 1)}(in)
template <>
CtxtTensor MatrixTransformer::transpose<Ciphertext>(const HomEvaluator &eval, const CtxtTensor &op) {
    const Context &ctx = eval.getContext();
    const i64 n_out_cols = op.getHeight(), n_out_rows = op.getWidth(), w = op.getBlockWidth();
    if (n_out_cols > w) throw std::invalid_argument("[transpose] num_cols > width.");
    const TileTensorShape shape(n_out_rows, n_out_cols, w);
    const Geometry g = geometry(MaskKind::Diagonal, shape);
    const u64 level = op.getLevel();
    if (level == 0) throw std::invalid_argument("[transpose] level >= 1 is needed.");
    std::vector<Ciphertext> baby;
    baby.reserve((size_t)g.bs);
    for (i64 j = 0; j < g.bs; j++) {
        baby.emplace_back(ctx);
        if (j == 0)
            eval.rightRotate(op.get(), (u64)((g.n - 1) * g.step), baby[0]);
        else
            eval.leftRotate(baby[(size_t)j - 1], (u64)g.step, baby[(size_t)j]);
    }
    Ciphertext res(ctx), group(ctx), tmp(ctx);
    bool first = true;
    for (i64 i = 0; i < g.gs; i++) {
        bool any = false;
        for (i64 j = 0; j < g.bs; j++) {
            const i64 e = 1 - g.n + i * g.bs + j;
            if (e >= g.n) break;
            eval.multWithoutRescale(baby[(size_t)j], transformMask(eval, MaskKind::Diagonal, shape, level, e),
                                    any ? tmp : group);
            if (any) eval.add(group, tmp, group);
            any = true;
        }
        if (!any) continue;
        if (i > 0) eval.leftRotate(group, (u64)(i * g.bs * g.step), group);
        if (first)
            res = group;
        else
            eval.add(res, group, res);
        first = false;
    }
    eval.rescale(res);
    return CtxtTensor(shape, res);
}
template <>
PtxtTensor MatrixTransformer::transpose<Plaintext>(const HomEvaluator &eval, const PtxtTensor &op) {
    const Context &ctx = eval.getContext();
    const i64 n = op.getHeight(), w = op.getBlockWidth();
    if (n > w) throw std::invalid_argument("[transpose] num_cols > width.");
    EnDecoder endec(ctx);
    const Message src = endec.decode(op.get());
    Message dst(src.getLogSlots(), 0);
    const i64 height = (i64)src.getSize() / w;
    for (i64 r = 0; r < height; r++)
        for (i64 c = 0; c < w; c++) {
            const i64 rb = r - r % n, cb = c - c % n;
            dst[(u64)(r * w + c)] = src[(u64)((rb + c % n) * w + cb + r % n)];
        }
    return PtxtTensor(TileTensorShape(op.getWidth(), op.getHeight(), w), endec.encode(dst, op.getLevel()));
}

// ---- products ----------------------------------------------------------------------------------------
namespace {
template <class T1, class T2>
i64 commonInside(const HETensor<T1> &a, const HETensor<T2> &b) {
    if (a.getWidth() != b.getHeight()) throw std::invalid_argument("[getCommonInsideLength] different inside length.");
    return a.getWidth();
}
template <class T1, class T2>
i64 commonBlockWidth(const HETensor<T1> &a, const HETensor<T2> &b) {
    if (a.getBlockWidth() != b.getBlockWidth())
        throw std::invalid_argument("[getCommonBlockWidth] different block width");
    return a.getBlockWidth();
}
void checkLevel(u64 level, const Bootstrapper &btp) {
    if (level < 1 + btp.getMinLevelForBootstrap())
        throw std::invalid_argument("[multMatMat] level >= " + std::to_string(1 + btp.getMinLevelForBootstrap()) +
                                    " is needed.");
}
}  // namespace

template <>
CtxtTensor multMatMat<Ciphertext>(const HomEvaluator &eval, const Bootstrapper &btp, const CtxtTensor &op1,
                                  const CtxtTensor &op2, u64 T, MatrixTransformer &tr) {
    const Context &ctx = eval.getContext();
    const i64 rows = op1.getHeight(), cols = op2.getWidth();
    const i64 k = pow2ceil(commonInside(op1, op2)), w = commonBlockWidth(op1, op2);
    checkLevel(std::min(op1.getLevel(), op2.getLevel()), btp);
    CtxtTensor a{op1}, b{op2};
    a.setShape(rows, k);
    b.setShape(k, cols);
    if (std::min(a.getLevel(), b.getLevel()) < 4 + btp.getMinLevelForBootstrap()) {
        eval.multImagUnit(b.get(), b.get());
        eval.add(a.get(), b.get(), a.get());
        btp.bootstrapExtended(a.get(), a.get(), b.get());
    }
    std::vector<Plaintext> &col_mask = tr.getColMask(eval, a.getShape(), T + 2);
    std::vector<Plaintext> &row_mask = tr.getRowMask(eval, b.getShape(), T + 2);
    a = tr.diagonalToColumn(eval, a);
    b = tr.diagonalToRow(eval, b);
    if (std::min(a.getLevel(), b.getLevel()) < T + 2)
        throw std::invalid_argument("[multMatMat] level >= " + std::to_string(T + 3) + " is needed.");
    eval.levelDown(a.get(), T + 2, a.get());
    eval.levelDown(b.get(), T + 2, b.get());

    const i64 rows_p = std::max(k, pow2ceil(rows)), cols_p = std::max(k, pow2ceil(cols));
    CtxtTensor res(ctx, rows, cols, w);
    eval.mult(a.get(), b.get(), res.get());

    eval.leftRotate(a.get(), 1, a.get());
    eval.leftRotate(b.get(), (u64)w, b.get());
    Ciphertext a_wrap(ctx), b_wrap(ctx);
    eval.rightRotate(a.get(), (u64)cols_p, a_wrap);
    eval.rightRotate(b.get(), (u64)(rows_p * w), b_wrap);

    Ciphertext t1(ctx), t2(ctx), acc(ctx);
    for (i64 i = 1; i < k; i++) {
        if (i > 1) {
            eval.leftRotate(a.get(), 1, a.get());
            eval.leftRotate(a_wrap, 1, a_wrap);
            eval.leftRotate(b.get(), (u64)w, b.get());
            eval.leftRotate(b_wrap, (u64)w, b_wrap);
        }
        eval.maskedSum(a.get(), col_mask[(size_t)(2 * i + 1)], a_wrap, col_mask[(size_t)(2 * i)], t1);
        eval.rescale(t1);
        eval.maskedSum(b.get(), row_mask[(size_t)(2 * i + 1)], b_wrap, row_mask[(size_t)(2 * i)], t2);
        eval.rescale(t2);
        eval.tensorAccumulate(t1, t2, acc, i == 1);
    }
    if (k > 1) {
        eval.relinearize(acc, t1);
        eval.rescale(t1);
        eval.add(res.get(), t1, res.get());
    }
    return res;
}

// ---- LoRA low-rank products (reference ciphertext/src/MatrixUtils.cpp:1681-1996) -------------------------
// One operand has only `low_dim` columns (or rows) in use, sitting at a column (row) block of every tile.  The
// transforms of the thin operand run on the thin shape, its copies are spread over the blocks by log-step
// rotations, and the product loop stops after low_dim terms; the outputs of all column blocks still have to
// be summed (HEMMer::repackTo*).
namespace {
// transform of an operand ending at level T+2: batched (two stages when the operand is high enough, see
// MatrixTransformer::lowerAndTransformFused) or in the reference's order from level T+3
Ciphertext sigmaTau(const HomEvaluator &eval, MatrixTransformer &tr, const Ciphertext &in, MaskKind kind,
                    const TileTensorShape &shape, u64 T, bool fused) {
    if (fused) return tr.lowerAndTransformFused(eval, in, kind, shape, T + 2);
    Ciphertext x(eval.getContext());
    eval.levelDown(in, T + 3, x);
    CtxtTensor t(shape, x);
    return kind == MaskKind::Horizontal ? tr.diagonalToColumn(eval, t).get() : tr.diagonalToRow(eval, t).get();
}
// level the operands are lowered to before anything else: the batched transforms may start one level higher
u64 loraStartLevel(const CtxtTensor &op1, const CtxtTensor &op2, u64 T, bool fused) {
    return (fused && std::min(op1.getLevel(), op2.getLevel()) >= T + 4) ? T + 4 : T + 3;
}

// sigma(A) (.) tau(B) and the low_dim - 1 shifted terms (:1716-1766)
CtxtTensor lowRankTerms(const HomEvaluator &eval, Ciphertext &a, Ciphertext &b, const CtxtTensor &op1,
                        const CtxtTensor &op2, i64 w, u64 T, i64 low_dim, MatrixTransformer &tr) {
    const Context &ctx = eval.getContext();
    const i64 num_rows = op1.getHeight();
    CtxtTensor res(ctx, op1.getHeight(), op2.getWidth(), op2.getBlockWidth());
    eval.mult(a, b, res.get());
    if (low_dim < 2) return res;
    eval.leftRotate(a, 1, a);
    eval.leftRotate(b, (u64)w, b);
    Ciphertext a_wrap(ctx), b_wrap(ctx);
    eval.rightRotate(a, (u64)(w / 2), a_wrap);
    eval.rightRotate(b, (u64)(num_rows * w), b_wrap);
    std::vector<Plaintext> &col_mask = tr.getColMask(eval, op1.getShape(), T + 2);
    std::vector<Plaintext> &row_mask = tr.getRowMask(eval, op2.getShape(), T + 2);
    Ciphertext t1(ctx), t2(ctx), acc(ctx);
    for (i64 i = 1; i < low_dim; i++) {
        if (i > 1) {
            eval.leftRotate(a, 1, a);
            eval.leftRotate(a_wrap, 1, a_wrap);
            eval.leftRotate(b, (u64)w, b);
            eval.leftRotate(b_wrap, (u64)w, b_wrap);
        }
        eval.maskedSum(a, col_mask[(size_t)(2 * i + 1)], a_wrap, col_mask[(size_t)(2 * i)], t1);
        eval.rescale(t1);
        eval.maskedSum(b, row_mask[(size_t)(2 * i + 1)], b_wrap, row_mask[(size_t)(2 * i)], t2);
        eval.rescale(t2);
        eval.tensorAccumulate(t1, t2, acc, i == 1);
    }
    eval.relinearize(acc, t1);
    eval.rescale(t1);
    eval.add(res.get(), t1, res.get());
    return res;
}
}  // namespace

CtxtTensor multMatMatHighLow(const HomEvaluator &eval, const CtxtTensor &op1, const CtxtTensor &op2, u64 in_col_block,
                             u64 T, MatrixTransformer &tr, i64 low_dim, bool fused) {
    const Context &ctx = eval.getContext();
    const i64 w = op2.getBlockWidth();
    Ciphertext a(ctx), b(ctx), tmp(ctx);
    a = sigmaTau(eval, tr, op1.get(), MaskKind::Horizontal, op1.getShape(), T, fused);
    b = sigmaTau(eval, tr, op2.get(), MaskKind::Vertical, TileTensorShape(op2.getHeight(), low_dim, w), T, fused);
    u64 pos = in_col_block;
    for (i64 i = low_dim; i < w / 2; i <<= 1) {
        if (pos % 2 == 0) {
            eval.leftRotate(b, (u64)(i * w), tmp);
            eval.rightRotate(tmp, (u64)i, tmp);
        } else {
            eval.leftRotate(b, (u64)i, tmp);
            eval.leftRotate(b, (u64)(i * w), b);
        }
        eval.add(b, tmp, b);
        pos /= 2;
    }
    return lowRankTerms(eval, a, b, op1, op2, w, T, low_dim, tr);
}

CtxtTensor multMatMatLowHigh(const HomEvaluator &eval, const CtxtTensor &op1, const CtxtTensor &op2, u64 in_row_block,
                             u64 T, MatrixTransformer &tr, i64 low_dim, bool fused) {
    const Context &ctx = eval.getContext();
    const i64 w = commonBlockWidth(op1, op2);
    Ciphertext a(ctx), b(ctx), tmp(ctx);
    const u64 start = loraStartLevel(op1, op2, T, fused);
    eval.levelDown(op1.get(), start, a);
    u64 pos = in_row_block;
    for (i64 i = low_dim; i < w / 2; i <<= 1) {
        if (pos % 2 == 0)
            eval.rightRotate(a, (u64)(i * w), tmp);
        else
            eval.leftRotate(a, (u64)(i * w), tmp);
        eval.add(a, tmp, a);
        pos /= 2;
    }
    a = sigmaTau(eval, tr, a, MaskKind::Horizontal, op1.getShape(), T, fused);
    b = sigmaTau(eval, tr, op2.get(), MaskKind::Vertical, op2.getShape(), T, fused);
    return lowRankTerms(eval, a, b, op1, op2, w, T, low_dim, tr);
}

CtxtTensor multMatMatLowLow(const HomEvaluator &eval, const CtxtTensor &op1, const CtxtTensor &op2, u64 in_col_block,
                            u64 in_row_block, u64 T, MatrixTransformer &tr, i64 low_dim, bool fused) {
    const Context &ctx = eval.getContext();
    const i64 w = commonBlockWidth(op1, op2);
    Ciphertext a(ctx), b(ctx), tmp(ctx);
    a = sigmaTau(eval, tr, op1.get(), MaskKind::Horizontal, TileTensorShape(op1.getHeight(), low_dim, w), T, fused);
    b = sigmaTau(eval, tr, op2.get(), MaskKind::Vertical, TileTensorShape(low_dim, op2.getWidth(), w), T, fused);
    u64 cpos = in_col_block, rpos = in_row_block;
    for (i64 i = low_dim; i < w / 2; i <<= 1) {
        if (cpos % 2 == 0)
            eval.rightRotate(a, (u64)i, tmp);
        else
            eval.leftRotate(a, (u64)i, tmp);
        eval.add(a, tmp, a);
        cpos /= 2;
        if (rpos % 2 == 0)
            eval.rightRotate(b, (u64)(i * w), tmp);
        else
            eval.leftRotate(b, (u64)(i * w), tmp);
        eval.add(b, tmp, b);
        rpos /= 2;
    }
    return lowRankTerms(eval, a, b, op1, op2, w, T, low_dim, tr);
}

template <>
CtxtTensor multMatMat<Plaintext>(const HomEvaluator &eval, const Bootstrapper &btp, const CtxtTensor &op1,
                                 const PtxtTensor &op2, u64 T, MatrixTransformer &tr) {
    const Context &ctx = eval.getContext();
    const i64 rows = op1.getHeight(), cols = op2.getWidth();
    const i64 k = pow2ceil(commonInside(op1, op2)), w = commonBlockWidth(op1, op2);
    checkLevel(std::min(op1.getLevel(), op2.getLevel()), btp);
    CtxtTensor a{op1};
    PtxtTensor b{op2};
    a.setShape(rows, k);
    b.setShape(k, cols);
    if (a.getLevel() < 4 + btp.getMinLevelForBootstrap()) btp.bootstrapExtended(a.get(), a.get());
    a = tr.diagonalToColumn(eval, a);
    b = tr.diagonalToRow(eval, b);
    if (a.getLevel() < T + 2)
        throw std::invalid_argument("[multMatMat] level >= " + std::to_string(T + 3) + " is needed.");
    eval.levelDown(a.get(), T + 2, a.get());
    EnDecoder endec(ctx);
    b.get() = endec.encode(endec.decode(b.get()), T + 2);

    const i64 rows_p = std::max(k, pow2ceil(rows)), cols_p = std::max(k, pow2ceil(cols));
    std::vector<Plaintext> &col_mask = tr.getColMask(eval, a.getShape(), T + 2);
    std::vector<Plaintext> &row_mask = tr.getRowMask(eval, b.getShape(), T + 2);
    CtxtTensor res(ctx, rows, cols, w);
    eval.mult(a.get(), b.get(), res.get());

    eval.leftRotate(a.get(), 1, a.get());
    eval.leftRotate(b.get(), (u64)w, b.get());
    Ciphertext a_wrap(ctx);
    Plaintext b_wrap(ctx);
    eval.rightRotate(a.get(), (u64)cols_p, a_wrap);
    eval.rightRotate(b.get(), (u64)(rows_p * w), b_wrap);

    Ciphertext t1(ctx), prod(ctx), acc(ctx);
    Plaintext p1(ctx), p2(ctx);
    for (i64 i = 1; i < k; i++) {
        if (i > 1) {
            eval.leftRotate(a.get(), 1, a.get());
            eval.leftRotate(a_wrap, 1, a_wrap);
            eval.leftRotate(b.get(), (u64)w, b.get());
            eval.leftRotate(b_wrap, (u64)w, b_wrap);
        }
        eval.maskedSum(a.get(), col_mask[(size_t)(2 * i + 1)], a_wrap, col_mask[(size_t)(2 * i)], t1);
        eval.rescale(t1);
        eval.mult(b.get(), row_mask[(size_t)(2 * i + 1)], p1);
        eval.mult(b_wrap, row_mask[(size_t)(2 * i)], p2);
        eval.add(p1, p2, p1);
        eval.mult(t1, p1, prod);
        if (i == 1)
            acc = prod;
        else
            eval.add(acc, prod, acc);
    }
    if (k > 1) eval.add(res.get(), acc, res.get());
    return res;
}

CtxtTensor multPackedMatMat(const HomEvaluator &eval, const Bootstrapper &btp, const CtxtTensor &op1,
                            const CtxtTensor &op2, u64 T, MatrixTransformer &tr) {
    const Context &ctx = eval.getContext();
    const i64 rows = op1.getHeight(), cols = op2.getWidth();
    const i64 k = pow2ceil(commonInside(op1, op2)), w = commonBlockWidth(op1, op2);
    checkLevel(std::min(op1.getLevel(), op2.getLevel()), btp);
    if (op1.getLevel() < T + 3 || op2.getLevel() < T + 2)
        throw std::invalid_argument("[multPackedMatMat] levels >= " + std::to_string(T + 3) + " / " +
                                    std::to_string(T + 2) + " are needed.");
    CtxtTensor a{op1}, b{op2};
    a.setShape(rows, k);
    b.setShape(k, cols);
    std::vector<Plaintext> &col_mask = tr.getColMask(eval, a.getShape(), T + 2);
    eval.levelDown(a.get(), T + 3, a.get());
    eval.levelDown(b.get(), T + 2, b.get());
    a = tr.packedDiagonalToColumn(eval, a);
    b = tr.packedDiagonalToRow(eval, b);

    const i64 cols_p = std::max(k, pow2ceil(cols));
    CtxtTensor res(ctx, rows, cols, w);
    eval.mult(a.get(), b.get(), res.get());
    eval.leftRotate(a.get(), 2, a.get());
    eval.leftRotate(b.get(), (u64)(2 * w), b.get());
    Ciphertext a_wrap(ctx);
    eval.rightRotate(a.get(), (u64)cols_p, a_wrap);
    Ciphertext t1(ctx), acc(ctx);
    for (i64 i = 1; i < k / 2; i++) {
        if (i > 1) {
            eval.leftRotate(a.get(), 2, a.get());
            eval.leftRotate(a_wrap, 2, a_wrap);
            eval.leftRotate(b.get(), (u64)(2 * w), b.get());
        }
        eval.maskedSum(a.get(), col_mask[(size_t)(4 * i + 1)], a_wrap, col_mask[(size_t)(4 * i)], t1);
        eval.rescale(t1);
        eval.tensorAccumulate(t1, b.get(), acc, i == 1);
    }
    if (k / 2 > 1) {
        eval.relinearize(acc, t1);
        eval.rescale(t1);
        eval.add(res.get(), t1, res.get());
    }
    return res;
}

CtxtTensor multPackedMatMatPre(const HomEvaluator &eval, const CtxtTensor &a_in, u64 T, MatrixTransformer &tr) {
    CtxtTensor a(a_in);
    eval.levelDown(a.get(), T + 3, a.get());
    return tr.packedDiagonalToColumn(eval, a);
}

void multPackedMatMatPreRot(const HomEvaluator &eval, const CtxtTensor &a_in, std::vector<Ciphertext> &tmp, u64 T,
                            MatrixTransformer &tr) {
    const Context &ctx = eval.getContext();
    tmp.clear();
    const i64 n = a_in.getHeight();
    CtxtTensor a(a_in);
    Ciphertext first(ctx);
    eval.levelDownOne(a.get(), first);
    tmp.push_back(first);
    eval.leftRotate(a.get(), 2, a.get());
    Ciphertext a_wrap(ctx), t1(ctx);
    eval.rightRotate(a.get(), (u64)n, a_wrap);
    std::vector<Plaintext> &col_mask = tr.getColMask(eval, a.getShape(), T + 2);
    for (i64 i = 1; i < n / 2; i++) {
        if (i > 1) {
            eval.leftRotate(a.get(), 2, a.get());
            eval.leftRotate(a_wrap, 2, a_wrap);
        }
        eval.maskedSum(a.get(), col_mask[(size_t)(4 * i + 1)], a_wrap, col_mask[(size_t)(4 * i)], t1);
        eval.rescale(t1);
        tmp.push_back(t1);
    }
}

CtxtTensor multPackedMatMatPreRev(const HomEvaluator &eval, const CtxtTensor &b_in, u64 T, MatrixTransformer &tr) {
    CtxtTensor b(b_in);
    eval.levelDown(b.get(), T + 2, b.get());
    return tr.packedDiagonalToRow(eval, b);
}

CtxtTensor multPackedMatMatCCReuse(const HomEvaluator &eval, const std::vector<Ciphertext> &tmp,
                                   const CtxtTensor &b_in, u64, MatrixTransformer &) {
    const Context &ctx = eval.getContext();
    const i64 rows = b_in.getHeight(), cols = b_in.getWidth(), w = b_in.getBlockWidth();
    CtxtTensor b(b_in);
    b.setShape(pow2ceil(rows), cols);
    CtxtTensor res(ctx, rows, cols, w);
    Ciphertext acc(ctx);
    for (size_t i = 0; i < tmp.size(); i++) {
        if (i > 0) eval.leftRotate(b.get(), (u64)(2 * w), b.get());
        eval.tensorAccumulate(tmp[i], b.get(), acc, i == 0);
    }
    eval.relinearize(acc, res.get());
    eval.rescale(res.get());
    return res;
}

void multMatMatPre(const HomEvaluator &eval, const CtxtTensor &a_in, std::vector<Ciphertext> &tmp, u64 T,
                   MatrixTransformer &tr) {
    const Context &ctx = eval.getContext();
    tmp.clear();
    const i64 n = a_in.getHeight();
    CtxtTensor a(a_in);
    if (a.getLevel() < T + 3)
        throw std::invalid_argument("[multMatMatPre] level >= " + std::to_string(T + 3) + " is needed.");
    eval.levelDown(a.get(), T + 3, a.get());
    a = tr.diagonalToColumn(eval, a);
    Ciphertext first(ctx);
    eval.levelDownOne(a.get(), first);
    tmp.push_back(first);
    eval.leftRotate(a.get(), 1, a.get());
    Ciphertext a_wrap(ctx), t1(ctx);
    eval.rightRotate(a.get(), (u64)n, a_wrap);
    std::vector<Plaintext> &col_mask = tr.getColMask(eval, a.getShape(), T + 2);
    for (i64 i = 1; i < n; i++) {
        if (i > 1) {
            eval.leftRotate(a.get(), 1, a.get());
            eval.leftRotate(a_wrap, 1, a_wrap);
        }
        eval.maskedSum(a.get(), col_mask[(size_t)(2 * i + 1)], a_wrap, col_mask[(size_t)(2 * i)], t1);
        eval.rescale(t1);
        tmp.push_back(t1);
    }
}

CtxtTensor multMatMatReUse(const HomEvaluator &eval, const std::vector<Ciphertext> &tmp, const PtxtTensor &b_in,
                           u64 T, MatrixTransformer &) {
    const Context &ctx = eval.getContext();
    const i64 rows = b_in.getHeight(), cols = b_in.getWidth(), w = b_in.getBlockWidth();
    PtxtTensor b(b_in);
    if (b.getLevel() != T + 1) {
        EnDecoder endec(ctx);
        b.get() = endec.encode(endec.decode(b.get()), T + 1);
    }
    CtxtTensor res(ctx, rows, cols, w);
    eval.matmul(tmp, b.get(), res.get());
    return res;
}

CtxtTensor multMatMatPreRev(const HomEvaluator &eval, const CtxtTensor &b_in, u64 T, MatrixTransformer &tr) {
    CtxtTensor b(b_in);
    eval.levelDown(b.get(), T + 2, b.get());
    return tr.diagonalToRow(eval, b);
}

CtxtTensor multMatMatCCReUse(const HomEvaluator &eval, const std::vector<Ciphertext> &tmp, const CtxtTensor &b_in,
                             u64, MatrixTransformer &) {
    const Context &ctx = eval.getContext();
    const i64 rows = b_in.getHeight(), cols = b_in.getWidth(), w = b_in.getBlockWidth();
    CtxtTensor b(b_in);
    CtxtTensor res(ctx, rows, cols, w);
    Ciphertext acc(ctx);
    for (size_t i = 0; i < tmp.size(); i++) {
        if (i > 0) eval.leftRotate(b.get(), (u64)w, b.get());
        eval.tensorAccumulate(tmp[i], b.get(), acc, i == 0);
    }
    eval.relinearize(acc, res.get());
    return res;
}

}  // namespace HELLM

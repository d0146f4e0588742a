// Batched schedules of the HEMMer products: the algorithm of matrix_utils.cpp (reference:
// ciphertext/src/MatrixUtils.cpp:776-1098 transforms, :1307-1446 CCMM, :1100-1216 packed CCMM, :1572-1610
// hoisted pre-computation) re-scheduled for a 256-CU GPU.  One evaluator call of the reference is a
// 7-limb, ~100-workgroup launch chain; here all independent rotations of a phase share one launch chain.
#include <hip/hip_runtime.h>

#include <cmath>

#include "../../../include/hemm.h"
#include "HELLM/MatrixUtils.hpp"
#include "context_content.hpp"

namespace HELLM {

namespace {

void ck(int rc) {
    if (rc == 0) return;
    std::string m = hemm_last_error();
    if (rc == 1) throw std::invalid_argument(m);
    throw RuntimeException(m);
}
typedef unsigned __int128 u128;
u64 powmod(u64 a, u64 e, u64 q) {
    u64 r = 1 % q;
    a %= q;
    while (e) {
        if (e & 1) r = (u64)((u128)r * a % q);
        a = (u64)((u128)a * a % q);
        e >>= 1;
    }
    return r;
}
i64 pow2ceil(i64 v) {
    i64 p = 1;
    while (p < v) p <<= 1;
    return p;
}

struct Geo {
    i64 n, units, cell, bs, gs, step;
};
Geo geo(MaskKind kind, const TileTensorShape &s) {
    Geo g{};
    const i64 w = s.getBlockWidth();
    if (s.getNumRows() != s.getNumCols()) throw std::invalid_argument("[MatrixTransformer] only square tiles are supported");
    g.n = s.getNumRows();
    const bool packed = (kind == MaskKind::PackedHorizontal || kind == MaskKind::PackedVertical);
    const bool vertical = (kind == MaskKind::Vertical || kind == MaskKind::PackedVertical);
    g.cell = packed ? 2 : 1;
    g.units = g.n / g.cell;
    g.bs = (i64)std::ceil(std::sqrt((double)(2 * g.units - 1)));
    g.gs = (i64)std::ceil((double)(g.units - 1) / (double)g.bs);
    g.step = g.cell * (vertical ? w : 1);
    return g;
}

// left rotation amount (possibly negative) -> Galois element
struct Rot {
    const Context &c;
    u64 slots, M;
    explicit Rot(const Context &ctx) : c(ctx), slots(ctx->N / 2), M(2 * ctx->N) {}
    u64 norm(i64 r) const { return (u64)(((r % (i64)slots) + (i64)slots) % (i64)slots); }
    u64 galois(i64 r) const { return powmod(5, norm(r), M); }
};

hemm_rot_term term(const u64 *ext, const u64 *b, const KeyPack &pack, u64 galois, const Plaintext *mask) {
    hemm_rot_term t;
    t.ext = ext;
    t.b = b;
    t.evk = pack.galoisKey(galois);
    t.mask = mask ? mask->buf_.data() : nullptr;
    t.galois = galois;
    return t;
}

// P * b of a ciphertext's b-polynomial (limb j times P mod q_j), computed once per rotation source
DeviceBuffer timesP(const Context &c, const u64 *b, u64 nq) {
    DeviceBuffer out(c, nq * c->N);
    std::vector<u64> sc(nq);
    for (u64 j = 0; j < nq; j++) {
        u64 P = 1;
        for (u64 p : c->p) P = (u64)((u128)P * (p % c->q[j]) % c->q[j]);
        sc[j] = P;
    }
    ck(hemm_mul_scalar(c->dev, b, 0, sc.data(), out.data(), 0, (uint32_t)nq, 0, 1, nullptr));
    return out;
}

// ModUp of the a-polynomial of one ciphertext
DeviceBuffer modUpOne(const Context &c, const Ciphertext &ct) {
    const u64 nq = ct.level_ + 1, E = nq + c->nP, beta = (nq + c->alpha - 1) / c->alpha;
    DeviceBuffer ext(c, beta * E * c->N), ws(c, nq * c->N);
    ck(hemm_modup_batch(c->dev, ct.getPolyData(1), ct.polyStride(), (uint32_t)nq, 1, ext.data(), ws.data(), nullptr));
    return ext;
}

}  // namespace

std::vector<Plaintext> &MatrixTransformer::getColMaskExt(const HomEvaluator &eval, const TileTensorShape &shape,
                                                         u64 level) {
    auto key = std::make_pair(shape, level);
    auto it = col_masks_ext_.find(key);
    if (it != col_masks_ext_.end()) return it->second;
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
        v.push_back(endec.encodeExtended(wrap, level));
        v.push_back(endec.encodeExtended(main, level));
    }
    return col_masks_ext_.emplace(key, std::move(v)).first->second;
}
std::vector<Plaintext> &MatrixTransformer::getRowMaskExt(const HomEvaluator &eval, const TileTensorShape &shape,
                                                         u64 level) {
    auto key = std::make_pair(shape, level);
    auto it = row_masks_ext_.find(key);
    if (it != row_masks_ext_.end()) return it->second;
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
        v.push_back(endec.encodeExtended(wrap, level));
        v.push_back(endec.encodeExtended(main, level));
    }
    return row_masks_ext_.emplace(key, std::move(v)).first->second;
}

std::vector<u64> fusedRotations(const TileTensorShape &shape, u64 log_slots, bool packed, bool need_rows) {
    const i64 slots = i64(1) << log_slots, n = shape.getNumRows(), w = shape.getBlockWidth();
    std::vector<u64> r;
    auto left = [&](i64 v) { r.push_back((u64)(((v % slots) + slots) % slots)); };
    const i64 stride = packed ? 2 : 1, count = packed ? n / 2 : n;
    for (i64 i = 1; i < count; i++) {
        left(stride * i);
        left(stride * i - n);
        if (need_rows) {
            left(stride * i * w);
            if (!packed) left((stride * i - n) * w);
        }
    }
    return r;
}

// T(A) = M_0 A + sum_d M_d rot_{d step}(A) with:
//   1 ModUp of A, all bs baby rotations as hoisted terms in one launch + one batched ModDown;
//   one masked-sum launch for every (giant index, sign) group;
//   1 batched ModUp of the group sums, every giant rotation as a hoisted term of ONE output, so the
//   groups are summed in the extended basis and share a single ModDown; one rescale at the end.
Ciphertext MatrixTransformer::diagonalTransformFused(const HomEvaluator &eval, const Ciphertext &in, MaskKind kind,
                                                     const TileTensorShape &shape) {
    const Context &c = eval.getContext();
    const KeyPack &pack = eval.getKeyPack();
    const Geo g = geo(kind, shape);
    const Rot rot(c);
    const u64 level = in.getLevel(), nq = level + 1, N = c->N, K = c->nP, E = nq + K;
    if (level == 0) throw std::invalid_argument("[diagonalTransform] level >= 1 is needed.");
    if (in.getRescaleCounter() != 0) throw RuntimeException("diagonalTransform: operand must be rescaled first");
    const size_t ctw = 2 * nq * N;  // words per 2-poly ciphertext at this level

    // 1. baby steps
    DeviceBuffer ext = modUpOne(c, in);
    DeviceBuffer pb = timesP(c, in.getPolyData(0), nq);
    std::vector<hemm_rot_term> terms;
    std::vector<uint32_t> off{0};
    for (i64 j = 0; j < g.bs; j++) {
        terms.push_back(term(ext.data(), pb.data(), pack, rot.galois((j + 1) * g.step), nullptr));
        off.push_back((uint32_t)terms.size());
    }
    DeviceBuffer y(c, (size_t)g.bs * 2 * E * N), baby(c, (size_t)g.bs * ctw), ws(c, (size_t)g.bs * ctw);
    ck(hemm_hoisted_terms(c->dev, terms.data(), off.data(), (uint32_t)g.bs, (uint32_t)nq, y.data(), 1, nullptr));
    ck(hemm_moddown_batch(c->dev, y.data(), (uint32_t)nq, (uint32_t)(2 * g.bs), 0, baby.data(), nq * N, ws.data(),
                          nullptr));

    // 2. group sums: group 0 needs no rotation (d = 0, the positive diagonals of giant index 0, and any
    //    group whose rotation is a whole turn)
    std::vector<std::vector<hemm_lin_term>> groups(1);
    std::vector<i64> group_rot{0};  // left rotation still to apply to each group
    auto lin = [&](const u64 *ct, i64 d) {
        hemm_lin_term t;
        t.ct = ct;
        t.mask = transformMask(eval, kind, shape, level, d).buf_.data();
        t.stride = nq * N;
        t.galois = 0;
        return t;
    };
    auto push_group = [&](std::vector<hemm_lin_term> &&g_terms, i64 r) {
        if (g_terms.empty()) return;
        if (rot.norm(r) == 0) {
            for (auto &t : g_terms) groups[0].push_back(t);
        } else {
            groups.push_back(std::move(g_terms));
            group_rot.push_back(r);
        }
    };
    groups[0].push_back(lin(in.buf_.data(), 0));
    for (i64 i = 0; i < g.gs; i++) {
        std::vector<hemm_lin_term> neg, pos;
        for (i64 j = 0; j < g.bs; j++) {
            const i64 d = 1 + i * g.bs + j - g.units;
            if (d >= 0) break;
            neg.push_back(lin(baby.data() + (size_t)j * ctw, d));
        }
        push_group(std::move(neg), -(g.units - i * g.bs) * g.step);
        for (i64 j = 0; j < g.bs; j++) {
            const i64 d = 1 + i * g.bs + j;
            if (d >= g.units) break;
            pos.push_back(lin(baby.data() + (size_t)j * ctw, d));
        }
        push_group(std::move(pos), i * g.bs * g.step);
    }
    std::vector<hemm_lin_term> lt;
    std::vector<uint32_t> loff{0};
    for (auto &gr : groups) {
        for (auto &t : gr) lt.push_back(t);
        loff.push_back((uint32_t)lt.size());
    }
    const size_t n_groups = group_rot.size();
    DeviceBuffer sums(c, n_groups * ctw);
    ck(hemm_masked_sum_batch(c->dev, lt.data(), loff.data(), (uint32_t)n_groups, (uint32_t)nq, 2, sums.data(), nullptr));

    // 3. giant steps: every rotated group is a term of one output
    Ciphertext res(c);
    res.allocate(2, level, 1);
    if (n_groups > 1) {
        const size_t ng = n_groups - 1;
        const u64 beta = (nq + c->alpha - 1) / c->alpha;
        DeviceBuffer ext2(c, ng * beta * E * N), ws2(c, ng * nq * N);
        ck(hemm_modup_batch(c->dev, sums.data() + ctw + nq * N, ctw, (uint32_t)nq, (uint32_t)ng, ext2.data(), ws2.data(),
                            nullptr));
        std::vector<hemm_rot_term> gt;
        for (size_t k = 0; k < ng; k++)
            gt.push_back(term(ext2.data() + k * beta * E * N, sums.data() + (k + 1) * ctw, pack,
                              rot.galois(group_rot[k + 1]), nullptr));
        uint32_t goff[2] = {0, (uint32_t)ng};
        DeviceBuffer y2(c, 2 * E * N), ws3(c, ctw);
        ck(hemm_hoisted_terms(c->dev, gt.data(), goff, 1, (uint32_t)nq, y2.data(), 0, nullptr));
        ck(hemm_moddown_batch(c->dev, y2.data(), (uint32_t)nq, 2, 0, res.buf_.data(), nq * N, ws3.data(), nullptr));
        ck(hemm_pointwise(c->dev, HEMM_ADD, res.buf_.data(), nq * N, sums.data(), nq * N, res.buf_.data(), nq * N,
                          (uint32_t)nq, 0, 2, nullptr));
    } else {
        (void)hipMemcpyAsync(res.buf_.data(), sums.data(), ctw * 8, hipMemcpyDeviceToDevice, nullptr);
    }
    eval.rescale(res);
    return res;
}

namespace {

// Shifts of `src` (level l, rescale counter 0): for every entry two hoisted rotations of src combined
// with extended masks (second one optional), then ModDown merged with the rescale.  Output: entries.size()
// ciphertexts [2][l][N] (level l-1) packed in `out`.
struct Shift {
    i64 rot1;
    const Plaintext *mask1;
    i64 rot2;
    const Plaintext *mask2;  // nullptr: single-term shift
    bool two;
};
void assembleShifts(const HomEvaluator &eval, const Ciphertext &src, const DeviceBuffer &ext, const DeviceBuffer &pb,
                    const std::vector<Shift> &shifts, size_t first, size_t count, u64 *y, u64 *out, u64 *ws) {
    const Context &c = eval.getContext();
    const KeyPack &pack = eval.getKeyPack();
    const Rot rot(c);
    const u64 nq = src.getLevel() + 1, N = c->N;
    std::vector<hemm_rot_term> terms;
    std::vector<uint32_t> off{0};
    for (size_t k = first; k < first + count; k++) {
        const Shift &s = shifts[k];
        terms.push_back(term(ext.data(), pb.data(), pack, rot.galois(s.rot1), s.mask1));
        if (s.two) terms.push_back(term(ext.data(), pb.data(), pack, rot.galois(s.rot2), s.mask2));
        off.push_back((uint32_t)terms.size());
    }
    ck(hemm_hoisted_terms(c->dev, terms.data(), off.data(), (uint32_t)count, (uint32_t)nq, y, 1, nullptr));
    ck(hemm_moddown_batch(c->dev, y, (uint32_t)nq, (uint32_t)(2 * count), 1, out, (nq - 1) * N, ws, nullptr));
}

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

}  // namespace

CtxtTensor multMatMatFused(const HomEvaluator &eval, const Bootstrapper &btp, const CtxtTensor &op1,
                           const CtxtTensor &op2, u64 T, MatrixTransformer &tr, u64 batch) {
    const Context &c = eval.getContext();
    const i64 rows = op1.getHeight(), cols = op2.getWidth();
    const i64 k = pow2ceil(commonInside(op1, op2)), w = commonBlockWidth(op1, op2);
    const u64 min_level = std::min(op1.getLevel(), op2.getLevel());
    if (min_level < 1 + btp.getMinLevelForBootstrap())
        throw std::invalid_argument("[multMatMat] level >= " + std::to_string(1 + btp.getMinLevelForBootstrap()) +
                                    " is needed.");
    CtxtTensor a{op1}, b{op2};
    a.setShape(rows, k);
    b.setShape(k, cols);
    if (min_level < 4 + btp.getMinLevelForBootstrap()) btp.bootstrapExtended(a.get(), a.get(), b.get());
    if (min_level < T + 3)
        throw std::invalid_argument("[multMatMat] level >= " + std::to_string(T + 3) + " is needed.");
    // the transforms run at level T+3: lowering first gives the same values with 8 instead of 13 limbs
    eval.levelDown(a.get(), T + 3, a.get());
    eval.levelDown(b.get(), T + 3, b.get());
    std::vector<Plaintext> &cm = tr.getColMaskExt(eval, a.getShape(), T + 2);
    std::vector<Plaintext> &rm = tr.getRowMaskExt(eval, b.getShape(), T + 2);
    a.get() = tr.diagonalTransformFused(eval, a.get(), MaskKind::Horizontal, a.getShape());
    b.get() = tr.diagonalTransformFused(eval, b.get(), MaskKind::Vertical, b.getShape());

    CtxtTensor res(c, rows, cols, w);
    eval.mult(a.get(), b.get(), res.get());  // k = 0 term, level T+1
    if (k == 1) return res;

    const i64 n = k;
    std::vector<Shift> sa, sb;
    for (i64 i = 1; i < n; i++) {
        sa.push_back(Shift{i, &cm[(size_t)(2 * i + 1)], i - n, &cm[(size_t)(2 * i)], true});
        sb.push_back(Shift{i * w, &rm[(size_t)(2 * i + 1)], (i - n) * w, &rm[(size_t)(2 * i)], true});
    }
    const u64 nq = T + 3, N = c->N, E = nq + c->nP, lo = nq - 1;
    DeviceBuffer extA = modUpOne(c, a.get()), extB = modUpOne(c, b.get());
    DeviceBuffer pbA = timesP(c, a.get().getPolyData(0), nq), pbB = timesP(c, b.get().getPolyData(0), nq);
    const size_t G = std::max<u64>(1, std::min<u64>(batch, (u64)(n - 1)));
    DeviceBuffer y(c, 2 * G * 2 * E * N), t(c, 2 * G * 2 * lo * N), ws(c, 2 * G * 2 * lo * N);
    Ciphertext acc(c);
    acc.allocate(3, T + 1, 1);
    for (size_t first = 0; first < sa.size(); first += G) {
        const size_t cnt = std::min(G, sa.size() - first);
        assembleShifts(eval, a.get(), extA, pbA, sa, first, cnt, y.data(), t.data(), ws.data());
        assembleShifts(eval, b.get(), extB, pbB, sb, first, cnt, y.data() + G * 2 * E * N, t.data() + G * 2 * lo * N,
                       ws.data() + G * 2 * lo * N);
        ck(hemm_tensor_batch(c->dev, t.data(), t.data() + G * 2 * lo * N, (uint32_t)cnt, (uint32_t)lo, acc.buf_.data(),
                             first == 0 ? 0 : 1, nullptr));
    }
    Ciphertext out(c);
    eval.relinearize(acc, out);
    eval.rescale(out);
    eval.add(res.get(), out, res.get());
    return res;
}

CtxtTensor multPackedMatMatFused(const HomEvaluator &eval, const Bootstrapper &btp, const CtxtTensor &op1,
                                 const CtxtTensor &op2, u64 T, MatrixTransformer &tr, u64 batch) {
    const Context &c = eval.getContext();
    const i64 rows = op1.getHeight(), cols = op2.getWidth();
    const i64 k = pow2ceil(commonInside(op1, op2)), w = commonBlockWidth(op1, op2);
    if (std::min(op1.getLevel(), op2.getLevel()) < 1 + btp.getMinLevelForBootstrap())
        throw std::invalid_argument("[multMatMat] level >= " + std::to_string(1 + btp.getMinLevelForBootstrap()) +
                                    " is needed.");
    if (op1.getLevel() < T + 3 || op2.getLevel() < T + 2)
        throw std::invalid_argument("[multPackedMatMat] levels >= " + std::to_string(T + 3) + " / " +
                                    std::to_string(T + 2) + " are needed.");
    if ((u64)(k * w) != c->N / 2)
        throw std::invalid_argument("[multPackedMatMat] the row shift must be cyclic: rows * block width == slots");
    CtxtTensor a{op1}, b{op2};
    a.setShape(rows, k);
    b.setShape(k, cols);
    std::vector<Plaintext> &cm = tr.getColMaskExt(eval, a.getShape(), T + 2);
    eval.levelDown(a.get(), T + 3, a.get());
    eval.levelDown(b.get(), T + 2, b.get());
    a.get() = tr.diagonalTransformFused(eval, a.get(), MaskKind::PackedHorizontal, a.getShape());  // T+2
    b.get() = tr.diagonalTransformFused(eval, b.get(), MaskKind::PackedVertical, b.getShape());    // T+1
    CtxtTensor res(c, rows, cols, w);
    eval.mult(a.get(), b.get(), res.get());  // level T
    if (k / 2 <= 1) return res;

    const i64 n = k;
    std::vector<Shift> sa;
    for (i64 i = 1; i < n / 2; i++)
        sa.push_back(Shift{2 * i, &cm[(size_t)(4 * i + 1)], 2 * i - n, &cm[(size_t)(4 * i)], true});
    const u64 nqa = T + 3, nqb = T + 2, N = c->N, K = c->nP, lo = T + 2;  // both sides end at T+1 (lo limbs)
    DeviceBuffer extA = modUpOne(c, a.get()), extB = modUpOne(c, b.get());
    DeviceBuffer pbA = timesP(c, a.get().getPolyData(0), nqa), pbB = timesP(c, b.get().getPolyData(0), nqb);
    const KeyPack &pack = eval.getKeyPack();
    const Rot rot(c);
    const size_t G = std::max<u64>(1, std::min<u64>(batch, (u64)sa.size()));
    DeviceBuffer ya(c, G * 2 * (nqa + K) * N), yb(c, G * 2 * (nqb + K) * N), t1(c, G * 2 * lo * N), t2(c, G * 2 * lo * N),
        ws(c, G * 2 * lo * N);
    Ciphertext acc(c);
    acc.allocate(3, T + 1, 1);
    for (size_t first = 0; first < sa.size(); first += G) {
        const size_t cnt = std::min(G, sa.size() - first);
        assembleShifts(eval, a.get(), extA, pbA, sa, first, cnt, ya.data(), t1.data(), ws.data());
        // row shifts are exact rotations here: one unmasked hoisted term each, plain ModDown
        std::vector<hemm_rot_term> terms;
        std::vector<uint32_t> off{0};
        for (size_t q = first; q < first + cnt; q++) {
            terms.push_back(term(extB.data(), pbB.data(), pack, rot.galois((i64)(2 * (q + 1)) * w), nullptr));
            off.push_back((uint32_t)terms.size());
        }
        ck(hemm_hoisted_terms(c->dev, terms.data(), off.data(), (uint32_t)cnt, (uint32_t)nqb, yb.data(), 1, nullptr));
        ck(hemm_moddown_batch(c->dev, yb.data(), (uint32_t)nqb, (uint32_t)(2 * cnt), 0, t2.data(), lo * N, ws.data(),
                              nullptr));
        ck(hemm_tensor_batch(c->dev, t1.data(), t2.data(), (uint32_t)cnt, (uint32_t)lo, acc.buf_.data(),
                             first == 0 ? 0 : 1, nullptr));
    }
    Ciphertext out(c);
    eval.relinearize(acc, out);
    eval.rescale(out);
    eval.add(res.get(), out, res.get());
    return res;
}

void multMatMatPreFused(const HomEvaluator &eval, const CtxtTensor &a_in, std::vector<Ciphertext> &tmp, u64 T,
                        MatrixTransformer &tr, u64 batch) {
    const Context &c = eval.getContext();
    tmp.clear();
    const i64 n = a_in.getHeight();
    CtxtTensor a(a_in);
    if (a.getLevel() < T + 3)
        throw std::invalid_argument("[multMatMatPre] level >= " + std::to_string(T + 3) + " is needed.");
    eval.levelDown(a.get(), T + 3, a.get());
    std::vector<Plaintext> &cm = tr.getColMaskExt(eval, a.getShape(), T + 2);
    a.get() = tr.diagonalTransformFused(eval, a.get(), MaskKind::Horizontal, a.getShape());
    Ciphertext first_ct(c);
    eval.levelDownOne(a.get(), first_ct);
    tmp.push_back(first_ct);
    std::vector<Shift> sa;
    for (i64 i = 1; i < n; i++) sa.push_back(Shift{i, &cm[(size_t)(2 * i + 1)], i - n, &cm[(size_t)(2 * i)], true});
    const u64 nq = T + 3, N = c->N, E = nq + c->nP, lo = nq - 1;
    DeviceBuffer ext = modUpOne(c, a.get());
    DeviceBuffer pb = timesP(c, a.get().getPolyData(0), nq);
    const size_t G = std::max<u64>(1, std::min<u64>(batch, (u64)sa.size()));
    DeviceBuffer y(c, G * 2 * E * N), t(c, G * 2 * lo * N), ws(c, G * 2 * lo * N);
    for (size_t first = 0; first < sa.size(); first += G) {
        const size_t cnt = std::min(G, sa.size() - first);
        assembleShifts(eval, a.get(), ext, pb, sa, first, cnt, y.data(), t.data(), ws.data());
        for (size_t q = 0; q < cnt; q++) {
            Ciphertext ct(c);
            ct.allocate(2, T + 1, 0);
            (void)hipMemcpyAsync(ct.buf_.data(), t.data() + q * 2 * lo * N, 2 * lo * N * 8, hipMemcpyDeviceToDevice,
                                 nullptr);
            tmp.push_back(std::move(ct));
        }
    }
}

}  // namespace HELLM

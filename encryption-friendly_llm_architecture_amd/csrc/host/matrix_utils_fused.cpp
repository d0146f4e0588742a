// Batched schedules of the HEMMer products: the algorithm of matrix_utils.cpp (reference:
// ciphertext/src/MatrixUtils.cpp:776-1098 transforms, :1307-1446 CCMM, :1100-1216 packed CCMM, :1572-1610
// hoisted pre-computation) re-scheduled for a 256-CU GPU.  One evaluator call of the reference is a
// 7-limb, ~100-workgroup launch chain; here all independent rotations of a phase share one launch chain.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <map>
#include <set>

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

// baby-step count of the split of a product's n shifts: the largest power of two g with g * g <= 2 n
i64 bsgsBabyCount(i64 n) {
    i64 g = 1;
    while (4 * g * g <= 2 * n) g <<= 1;
    return g;
}

// units: length a diagonal wraps over (columns for sigma, rows for tau); sub: diagonals of one sign (the shorter
// side of a rectangular tile) -- both in cells
struct Geo {
    i64 n, units, sub, cell, bs, gs, step;
};
Geo geo(MaskKind kind, const TileTensorShape &s) {
    Geo g{};
    const i64 w = s.getBlockWidth(), rows = s.getNumRows(), cols = s.getNumCols();
    const bool packed = (kind == MaskKind::PackedHorizontal || kind == MaskKind::PackedVertical);
    const bool vertical = (kind == MaskKind::Vertical || kind == MaskKind::PackedVertical || kind == MaskKind::PackingVertical);
    const bool packing = (kind == MaskKind::PackingHorizontal || kind == MaskKind::PackingVertical);
    if (rows != cols && (packed || packing)) throw std::invalid_argument("[MatrixTransformer] packed transforms need square tiles");
    g.n = rows;
    g.cell = packed ? 2 : 1;
    g.units = (vertical ? rows : cols) / g.cell;
    g.sub = std::min(rows, cols) / g.cell;
    g.bs = (i64)std::ceil(std::sqrt((double)(2 * g.sub - 1)));
    g.gs = (i64)std::ceil((double)(g.sub - 1) / (double)g.bs);
    g.step = kind == MaskKind::DiagonalSigned ? w - 1 : g.cell * (vertical ? w : 1);
    if (kind == MaskKind::Diagonal) throw std::invalid_argument("[MatrixTransformer] the batched transform takes DiagonalSigned");
    if (kind == MaskKind::DiagonalSigned && rows != cols)
        throw std::invalid_argument("[MatrixTransformer] transpose needs square tiles");
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

// The key of a term of a hoisted sum (kind: 0 multiplication key, 1 key of X -> X^galois, 2 its square key): the
// compact form, a quarter less to read for the limbs of primes below 2^44, wherever the kernels take it (up to 6
// digits), else the plain one.
void set_key(hemm_rot_term &t, const KeyPack &pack, int kind, u64 galois) {
    if (pack.compactible()) {
        t.evk = pack.compactKey(kind, galois);
        t.flags = HEMM_ROT_COMPACT_KEY;
    } else {
        t.evk = kind == 0 ? pack.multKey() : kind == 1 ? pack.galoisKey(galois) : pack.galoisSquareKey(galois);
        t.flags = 0;
    }
}

hemm_rot_term term(const u64 *ext, const u64 *b, const KeyPack &pack, u64 galois, const Plaintext *mask) {
    hemm_rot_term t{};
    t.ext = ext;
    t.b = b;
    set_key(t, pack, 1, galois);
    t.mask = mask ? mask->buf_.data() : nullptr;
    t.galois = (uint32_t)galois;
    t.mask_shift = 0;
    if (mask && mask->compact_shift_ != 0) {
        t.mask = mask->compact_.data();
        t.mask_shift = mask->compact_shift_;
    }
    return t;
}

// mask * P * (b, a) on the chain limbs: a term of a hoisted sum that needs no key switch.  a is always given as it is;
// b as the launch takes every b (premultiplied or not), or nullptr
hemm_rot_term keylessTerm(const u64 *b, const u64 *a, const Plaintext *mask) {
    hemm_rot_term t{};
    t.ext = a;
    t.b = b;
    t.evk = nullptr;
    t.galois = 1;
    t.pt_galois = 1;
    if (mask) {
        t.mask = mask->buf_.data();
        if (mask->compact_shift_ != 0) {
            t.mask = mask->compact_.data();
            t.mask_shift = mask->compact_shift_;
        }
    }
    return t;
}

}  // namespace

const Plaintext &MatrixTransformer::firstBlockMask(const HomEvaluator &eval, const TileTensorShape &shape, u64 level) {
    useChainOf(eval.getContext());
    auto key = std::make_pair(shape, level);
    auto it = first_block_masks_.find(key);
    if (it != first_block_masks_.end()) return it->second;
    const Context &ctx = eval.getContext();
    const u64 log_slots = getLogFullSlots(ctx);
    const i64 first = shape.getNumRows() * shape.getBlockWidth(), slots = i64(1) << log_slots;
    Message m(log_slots, 0);
    for (i64 j = 0; j < std::min(first, slots); j++) m[(u64)j] = 1;
    return first_block_masks_.emplace(key, EnDecoder(ctx).encode(m, level)).first->second;
}

std::vector<Plaintext> &MatrixTransformer::getColMaskExt(const HomEvaluator &eval, const TileTensorShape &shape,
                                                         u64 level, bool first_block_only) {
    useChainOf(eval.getContext());
    auto key = std::make_pair(shape, level);
    auto &cache = first_block_only ? col_masks_ext_first_ : col_masks_ext_;
    auto it = cache.find(key);
    if (it != cache.end()) return it->second;
    const Context &ctx = eval.getContext();
    const u64 log_slots = getLogFullSlots(ctx);
    const i64 n = shape.getNumCols(), slots = i64(1) << log_slots;
    EnDecoder endec(ctx);
    std::vector<Plaintext> v;
    v.reserve((size_t)(2 * n));
    for (i64 i = 0; i < n; i++) {
        Message wrap(log_slots, 0), main(log_slots, 0);
        const i64 limit = first_block_only ? std::min(slots, shape.getNumRows() * shape.getBlockWidth()) : slots;
        for (i64 j = 0; j < limit; j++) {
            if (j % n < n - i)
                main[(u64)j] = 1;
            else
                wrap[(u64)j] = 1;
        }
        v.push_back(endec.encodeExtended(wrap, level));
        v.push_back(endec.encodeExtended(main, level));
    }
    // column patterns repeat every n slots: in NTT form such a mask is constant over long runs of residues, and
    // the hoisted sums then read one table entry per run instead of streaming the mask
    if (!first_block_only && (n & (n - 1)) == 0)
        for (Plaintext &pt : v) pt.makeCompact();
    return cache.emplace(key, std::move(v)).first->second;
}
std::vector<Plaintext> &MatrixTransformer::getRowMaskExt(const HomEvaluator &eval, const TileTensorShape &shape,
                                                         u64 level) {
    useChainOf(eval.getContext());
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

std::vector<u64> fusedCcmmRotations(const TileTensorShape &shape, u64 log_slots, std::vector<u64> &square_rots,
                                    bool packed, bool single_tile) {
    const i64 slots = i64(1) << log_slots, n = shape.getNumRows(), w = shape.getBlockWidth();
    square_rots.clear();
    const bool spread = single_tile && n * w < slots && slots % (n * w) == 0;
    if (n * w != slots && !spread) return fusedRotations(shape, log_slots, packed, true);
    std::vector<u64> r;
    auto left = [&](i64 v) { return (u64)(((v % slots) + slots) % slots); };
    const i64 cu = packed ? 2 : 1, units = n / cu, ru = cu * w, g = bsgsBabyCount(units);
    if (spread)     // baby rotations gather the block copies as well
        for (i64 i1 = 0; i1 < g; i1++)
            for (i64 j = 1; j < slots / (n * w); j++) r.push_back(left(i1 * ru - j * n * w));
    r.push_back(left(-n));
    for (i64 i = 1; i < units; i++) r.push_back(left(cu * i - g * (i / g) * ru));
    for (i64 i1 = 1; i1 < g; i1++) r.push_back(left(i1 * ru));
    for (i64 i2 = 1; i2 < units / g; i2++) {
        r.push_back(left(i2 * g * ru));
        square_rots.push_back(left(i2 * g * ru));
    }
    return r;
}

std::vector<u64> fusedRotations(const TileTensorShape &shape, u64 log_slots, bool packed, bool need_rows) {
    const i64 slots = i64(1) << log_slots, n = shape.getNumRows(), w = shape.getBlockWidth();
    std::vector<u64> r;
    auto left = [&](i64 v) { r.push_back((u64)(((v % slots) + slots) % slots)); };
    const i64 stride = packed ? 2 : 1, count = packed ? n / 2 : n;
    left(-n);
    if (need_rows) left(-n * w);
    for (i64 i = 1; i < count; i++) {
        left(stride * i);
        if (need_rows) left(stride * i * w);
    }
    return r;
}

// T(A) = M_0 A + sum_d M_d rot_{d step}(A) with:
//   1 ModUp of A, all bs baby rotations as hoisted terms in one launch + one batched ModDown;
//   one masked-sum launch for every (giant index, sign) group;
//   1 batched ModUp of the group sums, every giant rotation as a hoisted term of ONE output, so the
//   groups are summed in the extended basis together with the group that is not rotated (a term without a key) and
//   share a single ModDown merged with the rescale.
// Several transforms of operands at the same level (sigma(A) and tau(B) of one product) go through the
// same launches: `in` holds n_jobs ciphertexts [job][2][nq][N], `out` receives [job][2][nq-1][N].
void MatrixTransformer::diagonalTransformBatch(const HomEvaluator &eval, const u64 *in, size_t n_jobs, u64 level,
                                               const MaskKind *kinds, const TileTensorShape *shapes, u64 *out) {
    const Context &c = eval.getContext();
    const KeyPack &pack = eval.getKeyPack();
    const Rot rot(c);
    const u64 nq = level + 1, N = c->N, K = c->nP, E = nq + K, beta = (nq + c->alpha - 1) / c->alpha;
    if (level == 0) throw std::invalid_argument("[diagonalTransform] level >= 1 is needed.");
    const size_t ctw = 2 * nq * N;  // words per 2-poly ciphertext at this level
    std::vector<Geo> g;
    std::vector<size_t> baby_first{0};  // index of a job's first baby ciphertext
    for (size_t q = 0; q < n_jobs; q++) {
        g.push_back(geo(kinds[q], shapes[q]));
        baby_first.push_back(baby_first.back() + (size_t)g[q].bs);
    }
    const size_t n_baby = baby_first.back();

    // 1. baby steps
    DeviceBuffer ext(c, n_jobs * beta * E * N), pb(c, n_jobs * nq * N);
    {
        DeviceBuffer ws(c, n_jobs * nq * N);
        ck(hemm_modup_batch(c->dev, in + nq * N, ctw, (uint32_t)nq, (uint32_t)n_jobs, ext.data(), ws.data(), nullptr));
        std::vector<u64> sc(nq);
        for (u64 j = 0; j < nq; j++) {
            u64 P = 1;
            for (u64 p : c->p) P = (u64)((u128)P * (p % c->q[j]) % c->q[j]);
            sc[j] = P;
        }
        ck(hemm_mul_scalar(c->dev, in, ctw, sc.data(), pb.data(), nq * N, (uint32_t)nq, 0, (uint32_t)n_jobs, nullptr));
    }
    std::vector<hemm_rot_term> terms;
    std::vector<uint32_t> off{0};
    for (size_t q = 0; q < n_jobs; q++)
        for (i64 j = 0; j < g[q].bs; j++) {
            terms.push_back(term(ext.data() + q * beta * E * N, pb.data() + q * nq * N, pack,
                                 rot.galois((j + 1) * g[q].step), nullptr));
            off.push_back((uint32_t)terms.size());
        }
    DeviceBuffer y(c, n_baby * 2 * E * N), baby(c, n_baby * ctw), ws(c, n_baby * ctw);
    ck(hemm_hoisted_moddown(c->dev, terms.data(), off.data(), (uint32_t)n_baby, (uint32_t)nq, 1, 0, y.data(), baby.data(), nq * N, ws.data(), nullptr));
    c->mark("one-stage transform: baby rotations");

    // 2. group sums: a job's group 0 needs no rotation (d = 0, the positive diagonals of giant index 0, and
    //    any group whose rotation is a whole turn).  The unrotated groups of all jobs come first in `sums`,
    //    then every rotated group, so the rotated ones form one contiguous ModUp batch.
    std::vector<std::vector<hemm_lin_term>> plain(n_jobs), rotated;
    std::vector<i64> rotated_by;        // left rotation still to apply to each rotated group
    std::vector<size_t> rotated_first{0};
    for (size_t q = 0; q < n_jobs; q++) {
        const Geo &gq = g[q];
        const u64 *ct = in + q * ctw;
        const u64 *bb = baby.data() + baby_first[q] * ctw;
        auto lin = [&](const u64 *src, i64 d) {
            hemm_lin_term t;
            t.ct = src;
            t.mask = transformMask(eval, kinds[q], shapes[q], level, d).buf_.data();
            t.stride = nq * N;
            t.galois = 0;
            return t;
        };
        auto push_group = [&](std::vector<hemm_lin_term> &&g_terms, i64 r) {
            if (g_terms.empty()) return;
            if (rot.norm(r) == 0) {
                for (auto &t : g_terms) plain[q].push_back(t);
            } else {
                rotated.push_back(std::move(g_terms));
                rotated_by.push_back(r);
            }
        };
        plain[q].push_back(lin(ct, 0));
        for (i64 i = 0; i < gq.gs; i++) {
            std::vector<hemm_lin_term> neg, pos;
            for (i64 j = 0; j < gq.bs; j++) {
                const i64 d = 1 + i * gq.bs + j - gq.units;
                if (d >= gq.sub - gq.units) break;
                neg.push_back(lin(bb + (size_t)j * ctw, d));
            }
            push_group(std::move(neg), -(gq.units - i * gq.bs) * gq.step);
            for (i64 j = 0; j < gq.bs; j++) {
                const i64 d = 1 + i * gq.bs + j;
                if (d >= gq.sub) break;
                pos.push_back(lin(bb + (size_t)j * ctw, d));
            }
            push_group(std::move(pos), i * gq.bs * gq.step);
        }
        rotated_first.push_back(rotated.size());
    }
    std::vector<hemm_lin_term> lt;
    std::vector<uint32_t> loff{0};
    for (auto &gr : plain) {
        for (auto &t : gr) lt.push_back(t);
        loff.push_back((uint32_t)lt.size());
    }
    for (auto &gr : rotated) {
        for (auto &t : gr) lt.push_back(t);
        loff.push_back((uint32_t)lt.size());
    }
    const size_t ng = rotated.size(), n_groups = n_jobs + ng;
    DeviceBuffer sums(c, n_groups * ctw);
    ck(hemm_masked_sum_batch(c->dev, lt.data(), loff.data(), (uint32_t)n_groups, (uint32_t)nq, 2, sums.data(), nullptr));
    c->mark("one-stage transform: masked group sums");

    // 3. giant steps: every rotated group is a term of its job's output; the group that is not rotated joins the same
    // sum as a term without a key, and the sum takes one ModDown merged with the rescale
    bool every_job_rotates = ng > 0;
    for (size_t q = 0; q < n_jobs; q++) every_job_rotates = every_job_rotates && rotated_first[q + 1] > rotated_first[q];
    if (every_job_rotates) {
        const u64 *rs = sums.data() + n_jobs * ctw;
        DeviceBuffer ext2(c, ng * beta * E * N), ws2(c, ng * nq * N);
        ck(hemm_modup_batch(c->dev, rs + nq * N, ctw, (uint32_t)nq, (uint32_t)ng, ext2.data(), ws2.data(), nullptr));
        std::vector<hemm_rot_term> gt;
        std::vector<uint32_t> goff{0};
        for (size_t q = 0; q < n_jobs; q++) {
            for (size_t k = rotated_first[q]; k < rotated_first[q + 1]; k++)
                gt.push_back(term(ext2.data() + k * beta * E * N, rs + k * ctw, pack, rot.galois(rotated_by[k]), nullptr));
            gt.push_back(keylessTerm(sums.data() + q * ctw, sums.data() + q * ctw + nq * N, nullptr));
            goff.push_back((uint32_t)gt.size());
        }
        DeviceBuffer y2(c, n_jobs * 2 * E * N), ws3(c, n_jobs * ctw);
        ck(hemm_hoisted_moddown(c->dev, gt.data(), goff.data(), (uint32_t)n_jobs, (uint32_t)nq, 0, 1, y2.data(), out,
                                (nq - 1) * N, ws3.data(), nullptr));
    } else if (ng == 0) {
        ck(hemm_rescale(c->dev, sums.data(), nq * N, out, (nq - 1) * N, (uint32_t)nq, (uint32_t)(2 * n_jobs), nullptr));
    } else {
        throw RuntimeException("diagonalTransformBatch: jobs with and without giant steps cannot share a batch");
    }
    c->mark("one-stage transform: giant steps");
}

Ciphertext MatrixTransformer::diagonalTransformFused(const HomEvaluator &eval, const Ciphertext &in, MaskKind kind,
                                                     const TileTensorShape &shape) {
    if (in.getRescaleCounter() != 0) throw RuntimeException("diagonalTransform: operand must be rescaled first");
    if (in.getLevel() == 0) throw std::invalid_argument("[diagonalTransform] level >= 1 is needed.");
    Ciphertext res(eval.getContext());
    res.allocate(2, in.getLevel() - 1, 0);
    diagonalTransformBatch(eval, in.buf_.data(), 1, in.getLevel(), &kind, &shape, res.buf_.data());
    return res;
}

namespace {

// Rotation sources in the form the hoisted launches read: ModUp of the a-polynomial and P * b of
// n ciphertexts stored back to back ([n][2][nq][N]).
// premultiply = false leaves b as it is (pbOf points into the ciphertexts and the hoisted launch multiplies by P
// itself, `premultiplied()` = 0): one launch less for sources that a single short sum reads.
struct Sources {
    DeviceBuffer ext, pb;  // [n][beta][E][N], [n][nq][N]
    u64 nq, ext_words;
    const u64 *extOf(size_t q) const { return ext.data() + q * ext_words; }
    const u64 *pbOf(size_t q) const { return raw ? raw + q * 2 * nq * N_ : pb.data() + q * nq * N_; }
    int premultiplied() const { return raw ? 0 : 1; }
    u64 N_;
    const u64 *raw = nullptr;
};
Sources extendSources(const Context &c, const u64 *cts, size_t n, u64 nq, hipStream_t stream = nullptr,
                      bool premultiply = true) {
    const u64 N = c->N, E = nq + c->nP, beta = (nq + c->alpha - 1) / c->alpha, ctw = 2 * nq * N;
    Sources s{DeviceBuffer(c, n * beta * E * N), premultiply ? DeviceBuffer(c, n * nq * N) : DeviceBuffer(), nq,
              beta * E * N, N};
    DeviceBuffer ws(c, n * nq * N);
    ck(hemm_modup_batch(c->dev, cts + nq * N, ctw, (uint32_t)nq, (uint32_t)n, s.ext.data(), ws.data(), stream));
    if (!premultiply) {
        s.raw = cts;
        return s;
    }
    std::vector<u64> sc(nq);
    for (u64 j = 0; j < nq; j++) {
        u64 P = 1;
        for (u64 p : c->p) P = (u64)((u128)P * (p % c->q[j]) % c->q[j]);
        sc[j] = P;
    }
    ck(hemm_mul_scalar(c->dev, cts, ctw, sc.data(), s.pb.data(), nq * N, (uint32_t)nq, 0, (uint32_t)n, stream));
    return s;
}
// The same sources rotated left by rots[q] slots, as ciphertexts [n][2][nq][N]: one hoisted launch and one
// ModDown for all of them.
DeviceBuffer rotateSources(const HomEvaluator &eval, const Sources &src, const u64 *cts, size_t n, const i64 *rots,
                           hipStream_t stream = nullptr) {
    const Context &c = eval.getContext();
    const KeyPack &pack = eval.getKeyPack();
    const Rot rot(c);
    const u64 nq = src.nq, N = c->N, E = nq + c->nP, ctw = 2 * nq * N;
    DeviceBuffer out(c, n * ctw);
    std::vector<hemm_rot_term> terms;
    std::vector<uint32_t> off{0};
    std::vector<size_t> which;
    for (size_t q = 0; q < n; q++) {
        if (rot.norm(rots[q]) == 0) {  // a whole turn (rows of a tile that fills the slots): plain copy
            (void)hipMemcpyAsync(out.data() + q * ctw, cts + q * ctw, ctw * 8, hipMemcpyDeviceToDevice, c->on(stream));
            continue;
        }
        terms.push_back(term(src.extOf(q), src.pbOf(q), pack, rot.galois(rots[q]), nullptr));
        off.push_back((uint32_t)terms.size());
        which.push_back(q);
    }
    if (which.empty()) return out;
    const size_t m = which.size();
    DeviceBuffer y(c, m * 2 * E * N), ws(c, m * ctw);
    if (m == n) {   // every source rotated: the results land where they belong
        ck(hemm_hoisted_moddown(c->dev, terms.data(), off.data(), (uint32_t)m, (uint32_t)nq, 1, 0, y.data(), out.data(),
                                nq * N, ws.data(), stream));
        return out;
    }
    DeviceBuffer tmp(c, m * ctw);
    ck(hemm_hoisted_moddown(c->dev, terms.data(), off.data(), (uint32_t)m, (uint32_t)nq, 1, 0, y.data(), tmp.data(), nq * N, ws.data(), stream));
    for (size_t k = 0; k < m; k++)
        (void)hipMemcpyAsync(out.data() + which[k] * ctw, tmp.data() + k * ctw, ctw * 8, hipMemcpyDeviceToDevice, c->on(stream));
    return out;
}

// A cyclic shift by r inside a tile of period n (columns: unit 1, rows: unit w) is
//   main_mask * rot(X, r) + wrap_mask * rot(X, r - n unit)  =  main_mask * rot(X, r) + wrap_mask * rot(X', r)
// with X' = rot(X, -n unit) prepared once: both halves then use the key of r, which is streamed once.
struct Shift {
    i64 rot;
    const Plaintext *main_mask, *wrap_mask;
};
// terms of shifts[first, first + count) of source pair (x, x2) appended to `terms`
void pushShifts(const HomEvaluator &eval, const Sources &x, size_t ix, const Sources &x2, size_t ix2,
                const std::vector<Shift> &shifts, size_t first, size_t count, std::vector<hemm_rot_term> &terms,
                std::vector<uint32_t> &off) {
    const KeyPack &pack = eval.getKeyPack();
    const Rot rot(eval.getContext());
    for (size_t k = first; k < first + count; k++) {
        const u64 g = rot.galois(shifts[k].rot);
        terms.push_back(term(x.extOf(ix), x.pbOf(ix), pack, g, shifts[k].main_mask));
        terms.push_back(term(x2.extOf(ix2), x2.pbOf(ix2), pack, g, shifts[k].wrap_mask));
        off.push_back((uint32_t)terms.size());
    }
}

// the same without closing a group per shift: all shifts become terms of the output being assembled
void pushShiftGroup(const HomEvaluator &eval, const Sources &x, size_t ix, const Sources &x2, size_t ix2,
                    const std::vector<Shift> &shifts, std::vector<hemm_rot_term> &terms) {
    const KeyPack &pack = eval.getKeyPack();
    const Rot rot(eval.getContext());
    for (const Shift &sft : shifts) {
        const u64 g = rot.galois(sft.rot);
        terms.push_back(term(x.extOf(ix), x.pbOf(ix), pack, g, sft.main_mask));
        terms.push_back(term(x2.extOf(ix2), x2.pbOf(ix2), pack, g, sft.wrap_mask));
    }
}

// levelDown by one level of n_polys polynomials [n_polys][level+1][N] -> [n_polys][level][N]:
// multiply by round(Delta_{level-1} q_level / Delta_level), rescale (HomEvaluator::levelDown on a batch)
void levelDownOneBatch(const Context &c, const u64 *in, size_t n_polys, u64 level, u64 *out) {
    const u64 nq = level + 1, N = c->N;
    const i64 v = (i64)llround(c->delta[level - 1] * (Real)c->q[level] / c->delta[level]);
    std::vector<u64> sc(nq);
    for (u64 j = 0; j < nq; j++) sc[j] = v >= 0 ? (u64)v % c->q[j] : (c->q[j] - (u64)(-v) % c->q[j]) % c->q[j];
    DeviceBuffer t(c, n_polys * nq * N);
    ck(hemm_mul_scalar(c->dev, in, nq * N, sc.data(), t.data(), nq * N, (uint32_t)nq, 0, (uint32_t)n_polys, nullptr));
    ck(hemm_rescale(c->dev, t.data(), nq * N, out, (nq - 1) * N, (uint32_t)nq, (uint32_t)n_polys, nullptr));
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

// ---- two-stage sigma / tau ----------------------------------------------------------------------------------
i64 twoStageSplit(i64 units) {
    i64 b = 1;
    while (b * b < units) b <<= 1;
    return b;
}

Message twoStageMaskMessage(MaskKind kind, const TileTensorShape &shape, u64 log_slots, int stage, i64 r, int part) {
    const Geo g = geo(kind, shape);
    if (shape.getNumRows() != shape.getNumCols())
        throw std::invalid_argument("[MatrixTransformer] the two-stage transforms need square tiles");
    const bool vertical = (kind == MaskKind::Vertical || kind == MaskKind::PackedVertical);
    const i64 w = shape.getBlockWidth(), slots = i64(1) << log_slots, height = slots / w, n = g.n, u = g.units;
    const i64 b = twoStageSplit(u), amount = stage == 1 ? r : r * b;
    const double value = (kind == MaskKind::PackedHorizontal && stage == 1) ? 0.5 : 1.0;
    Message m(log_slots, 0);
    for (i64 row = 0; row < height; row++)
        for (i64 col = 0; col < w; col++) {
            const i64 Rc = (row % n) / g.cell, Cc = (col % n) / g.cell;
            const i64 sel = vertical ? Cc : Rc, pos = vertical ? Rc : Cc;
            bool on = stage == 1 ? (sel % b == r) : (sel / b == r);
            if (part == 1) on = on && pos < u - amount;
            if (part == 2) on = on && pos >= u - amount;   // part 3: both together (extended basis)
            if (on) m[(u64)(row * w + col)] = value;
        }
    return m;
}

const Plaintext &MatrixTransformer::twoStageMask(const HomEvaluator &eval, MaskKind kind, const TileTensorShape &shape,
                                                 u64 level, int stage, i64 r, int part, u64 from) {
    useChainOf(eval.getContext());
    if (from == level) from = 0;   // the level's own scale
    Key key{(int)kind, shape, level, ((i64)from * 4 + stage) * 4096 + r * 4 + part};
    auto it = two_stage_masks_.find(key);
    if (it != two_stage_masks_.end()) return it->second;
    const Context &ctx = eval.getContext();
    const Message m = twoStageMaskMessage(kind, shape, getLogFullSlots(ctx), stage, r, part);
    EnDecoder endec(ctx);
    if (from != 0) {
        const Real scale = ctx->delta[level - 1] * (Real)ctx->q[level] / ctx->delta[from];
        return two_stage_masks_.emplace(key, endec.encodeExtended(m, level, scale)).first->second;
    }
    return two_stage_masks_.emplace(key, part == 0 ? endec.encode(m, level) : endec.encodeExtended(m, level)).first->second;
}

std::vector<u64> MatrixTransformer::twoStageRotations(MaskKind kind, const TileTensorShape &shape, u64 log_slots) {
    const Geo g = geo(kind, shape);
    const bool vertical = (kind == MaskKind::Vertical || kind == MaskKind::PackedVertical);
    const i64 slots = i64(1) << log_slots, b = twoStageSplit(g.units);
    const i64 wrap = g.n * (vertical ? shape.getBlockWidth() : 1);
    std::vector<u64> r;
    auto left = [&](i64 v) { r.push_back((u64)(((v % slots) + slots) % slots)); };
    for (i64 i = 1; i < b; i++) {
        left(i * g.step);
        left(i * g.step - wrap);
    }
    for (i64 i = 1; i < g.units / b; i++) {
        left(i * b * g.step);
        left(i * b * g.step - wrap);
    }
    return r;
}

Ciphertext MatrixTransformer::lowerAndTransformFused(const HomEvaluator &eval, const Ciphertext &in, MaskKind kind,
                                                     const TileTensorShape &shape, u64 end_level) {
    const Context &c = eval.getContext();
    if (in.getLevel() < end_level + 1)
        throw std::invalid_argument("[diagonalTransform] level >= " + std::to_string(end_level + 1) + " is needed.");
    const bool two_stage = in.getLevel() >= end_level + 2 && shape.getNumRows() == shape.getNumCols();
    Ciphertext x(c), res(c);
    if (two_stage && in.getLevel() > end_level + 2 && in.getRescaleCounter() == 0 && in.getNumPoly() == 2) {
        // an operand above the starting level is only truncated to it (a copy of its first limbs): the masks of the
        // first stage absorb the change of scale, which saves the multiply-and-rescale of a levelDown
        const u64 L = end_level + 2, N = c->N, from = in.getLevel();
        DeviceBuffer cut(c, 2 * (L + 1) * N);
        const std::vector<u64> one(L + 1, 1);
        ck(hemm_mul_scalar(c->dev, in.buf_.data(), in.polyStride(), one.data(), cut.data(), (L + 1) * N, (uint32_t)(L + 1), 0, 2,
                           nullptr));
        res.allocate(2, end_level, 0);
        diagonalTransformTwoStage(eval, cut.data(), 1, L, &kind, &shape, res.buf_.data(), &from);
        return res;
    }
    eval.levelDown(in, end_level + (two_stage ? 2 : 1), x);
    if (!two_stage) return diagonalTransformFused(eval, x, kind, shape);
    res.allocate(2, end_level, 0);
    diagonalTransformTwoStage(eval, x.buf_.data(), 1, x.getLevel(), &kind, &shape, res.buf_.data());
    return res;
}

void MatrixTransformer::diagonalTransformTwoStage(const HomEvaluator &eval, const u64 *in, size_t n_jobs, u64 level,
                                                  const MaskKind *kinds, const TileTensorShape *shapes, u64 *out,
                                                  const u64 *scale_levels, int first_stage) {
    const Context &c = eval.getContext();
    if (level < 2) throw std::invalid_argument("[diagonalTransform] level >= 2 is needed.");
    const u64 N = c->N;
    if (first_stage != 1 && first_stage != 2) throw std::invalid_argument("[diagonalTransform] stage 1 or 2");
    DeviceBuffer mid;   // after stage 1: level - 1
    if (first_stage == 1) mid = DeviceBuffer(c, n_jobs * 2 * level * N);
    for (int stage = first_stage; stage <= 2; stage++) {
        const u64 lvl = stage == 1 ? level : level - 1, nq = lvl + 1, E = nq + c->nP, ctw = 2 * nq * N;
        const u64 *src = stage == first_stage ? in : mid.data();
        u64 *dst = stage == 1 ? mid.data() : out;
        auto from_of = [&](size_t q) -> u64 { return stage == 1 && scale_levels ? scale_levels[q] : 0; };
        // One rotation source per job (a single ModUp).  A stage's rotation by r cells wraps inside the tile, so it is
        //   main_r * rho^(r step)(X) + wrap_r * rho^(r step - tile side)(X):
        // two Galois elements per r with one key each; when they coincide (the tile side is a whole turn of the slot
        // vector) one term with the mask of both parts.
        // The rows that stay, mask_0 * X, need no key switch: they join the same sum as a term without a key
        // (mask_0 * P * (b, a) on the chain limbs) and share its ModDown and rescale.
        bool any_rotation = false;
        for (size_t q = 0; q < n_jobs; q++) {
            const Geo g = geo(kinds[q], shapes[q]);
            const i64 b = twoStageSplit(g.units);
            any_rotation = any_rotation || (stage == 1 ? b : g.units / b) > 1;
        }
        const Sources x = any_rotation ? extendSources(c, src, n_jobs, nq, nullptr, false) : Sources{};
        const KeyPack &pack = eval.getKeyPack();
        const Rot rot(c);
        std::vector<hemm_rot_term> terms;
        std::vector<uint32_t> off{0};
        for (size_t q = 0; any_rotation && q < n_jobs; q++) {
            const Geo g = geo(kinds[q], shapes[q]);
            const bool vertical = (kinds[q] == MaskKind::Vertical || kinds[q] == MaskKind::PackedVertical);
            const i64 wrap = g.n * (vertical ? shapes[q].getBlockWidth() : 1);
            const i64 b = twoStageSplit(g.units), count = stage == 1 ? b : g.units / b, mul = stage == 1 ? 1 : b;
            for (i64 r = 1; r < count; r++) {
                const i64 amount = r * mul * g.step;
                if (rot.norm(amount) == rot.norm(amount - wrap)) {
                    terms.push_back(term(x.extOf(q), x.pbOf(q), pack, rot.galois(amount),
                                         &twoStageMask(eval, kinds[q], shapes[q], lvl, stage, r, 3, from_of(q))));
                } else {
                    terms.push_back(term(x.extOf(q), x.pbOf(q), pack, rot.galois(amount),
                                         &twoStageMask(eval, kinds[q], shapes[q], lvl, stage, r, 1, from_of(q))));
                    terms.push_back(term(x.extOf(q), x.pbOf(q), pack, rot.galois(amount - wrap),
                                         &twoStageMask(eval, kinds[q], shapes[q], lvl, stage, r, 2, from_of(q))));
                }
            }
            terms.push_back(keylessTerm(src + q * ctw, src + q * ctw + nq * N, &twoStageMask(eval, kinds[q], shapes[q], lvl, stage, 0, 0, from_of(q))));
            off.push_back((uint32_t)terms.size());
        }
        if (any_rotation) {
            for (size_t q = 0; q + 1 < off.size(); q++)
                if (off[q + 1] == off[q] + 1)
                    throw RuntimeException("diagonalTransformTwoStage: jobs with and without rotations cannot share a batch");
            DeviceBuffer y(c, n_jobs * 2 * E * N), ws(c, n_jobs * 2 * (nq - 1) * N);
            ck(hemm_hoisted_moddown(c->dev, terms.data(), off.data(), (uint32_t)n_jobs, (uint32_t)nq, x.premultiplied(), 1,
                                    y.data(), dst, (nq - 1) * N, ws.data(), nullptr));
        } else {   // no rotation in this stage: mask and rescale
            std::vector<hemm_lin_term> zero_terms;
            std::vector<uint32_t> zoff{0};
            for (size_t q = 0; q < n_jobs; q++) {
                hemm_lin_term t;
                t.ct = src + q * ctw;
                t.mask = twoStageMask(eval, kinds[q], shapes[q], lvl, stage, 0, 0, from_of(q)).buf_.data();
                t.stride = nq * N;
                t.galois = 0;
                zero_terms.push_back(t);
                zoff.push_back((uint32_t)zero_terms.size());
            }
            DeviceBuffer zsum(c, n_jobs * ctw);
            ck(hemm_masked_sum_batch(c->dev, zero_terms.data(), zoff.data(), (uint32_t)n_jobs, (uint32_t)nq, 2, zsum.data(), nullptr));
            ck(hemm_rescale(c->dev, zsum.data(), nq * N, dst, (nq - 1) * N, (uint32_t)nq, (uint32_t)(2 * n_jobs), nullptr));
        }
        c->mark(stage == 1 ? "transform stage 1" : "transform stage 2");
    }
}

namespace {
// (left rotation in slots, mask) of the composite of the complex packing and the first transform stage
std::vector<std::pair<u64, Message>> packingStageOneMessages(MaskKind kind, const TileTensorShape &shape, u64 log_slots) {
    if (kind != MaskKind::PackedHorizontal && kind != MaskKind::PackedVertical)
        throw std::invalid_argument("[packingStageOne] a packed kind is needed");
    const Geo g = geo(kind, shape);
    const bool vertical = kind == MaskKind::PackedVertical;
    const i64 w = shape.getBlockWidth(), slots = i64(1) << log_slots, unit = vertical ? w : 1;
    const i64 b = twoStageSplit(g.units), wrap = g.n * (vertical ? w : 1);
    auto norm = [&](i64 v) { return (u64)(((v % slots) + slots) % slots); };
    const Message pm[3] = {packingMaskMessage(vertical, w, log_slots, 0), packingMaskMessage(vertical, w, log_slots, 1),
                           packingMaskMessage(vertical, w, log_slots, 2)};
    const i64 shift[3] = {0, unit, -unit};
    std::map<u64, Message> acc;
    auto add = [&](const Message &stage_mask, i64 a) {
        const u64 ra = norm(a);
        for (int e = 0; e < 3; e++) {
            auto it = acc.find(norm(a + shift[e]));
            if (it == acc.end()) it = acc.emplace(norm(a + shift[e]), Message(log_slots, 0)).first;
            Message &m = it->second;
            for (u64 s = 0; s < (u64)slots; s++) m[s] += stage_mask[s] * pm[e][(s + ra) % (u64)slots];
        }
    };
    add(twoStageMaskMessage(kind, shape, log_slots, 1, 0, 0), 0);
    for (i64 r = 1; r < b; r++) {
        add(twoStageMaskMessage(kind, shape, log_slots, 1, r, 1), r * g.step);
        add(twoStageMaskMessage(kind, shape, log_slots, 1, r, 2), r * g.step - wrap);
    }
    std::vector<std::pair<u64, Message>> out;
    for (auto &am : acc) {
        bool any = false;
        for (u64 s = 0; s < (u64)slots && !any; s++) any = am.second[s] != Complex(0, 0);
        if (any) out.emplace_back(am.first, std::move(am.second));   // (a rotation whose masks cancel is left out)
    }
    return out;
}
}  // namespace

std::vector<u64> MatrixTransformer::packingStageOneRotations(MaskKind kind, const TileTensorShape &shape, u64 log_slots) {
    // every stage rotation (0, r step, r step - wrap) shifted by the packing's 0, +unit, -unit
    const Geo g = geo(kind, shape);
    const bool vertical = kind == MaskKind::PackedVertical;
    const i64 w = shape.getBlockWidth(), slots = i64(1) << log_slots, unit = vertical ? w : 1;
    const i64 b = twoStageSplit(g.units), wrap = g.n * (vertical ? w : 1);
    std::set<u64> r;
    for (i64 i = 0; i < b; i++)
        for (i64 a : {i * g.step, i * g.step - wrap})
            for (i64 e : {i64(0), unit, -unit}) {
                const u64 v = (u64)((((a + e) % slots) + slots) % slots);
                if (v != 0 && (i > 0 || a == 0)) r.insert(v);
            }
    return std::vector<u64>(r.begin(), r.end());
}

void MatrixTransformer::packingStageOne(const HomEvaluator &eval, const u64 *in, size_t n_jobs, u64 level,
                                        const MaskKind *kinds, const TileTensorShape *shapes, u64 *out,
                                        const u64 *scale_levels) {
    const Context &c = eval.getContext();
    if (level < 1) throw std::invalid_argument("[packingStageOne] level >= 1 is needed.");
    const u64 nq = level + 1, N = c->N, E = nq + c->nP, ctw = 2 * nq * N;
    useChainOf(c);
    const Sources x = extendSources(c, in, n_jobs, nq, nullptr, false);
    const KeyPack &pack = eval.getKeyPack();
    const u64 M = 2 * N;
    std::vector<hemm_rot_term> terms;
    std::vector<uint32_t> off{0};
    for (size_t q = 0; q < n_jobs; q++) {
        const u64 scale_level = scale_levels && scale_levels[q] != 0 ? scale_levels[q] : level;
        if (scale_level < level)
            throw std::invalid_argument("[packingStageOne] the scale must come from the same or a higher level.");
        Key key{(int)kinds[q], shapes[q], level, (i64)(scale_level == level ? 0 : scale_level)};
        auto it = packing_stage_one_masks_.find(key);
        if (it == packing_stage_one_masks_.end()) {
            EnDecoder endec(c);
            // an input truncated from scale_level: the masks carry the change of scale (as in complexPackingBatch)
            const Real scale =
                scale_level == level ? c->delta[level] : c->delta[level - 1] * (Real)c->q[level] / c->delta[scale_level];
            std::vector<std::pair<u64, Plaintext>> v;
            for (const auto &am : packingStageOneMessages(kinds[q], shapes[q], getLogFullSlots(c)))
                v.emplace_back(am.first, endec.encodeExtended(am.second, level, scale));
            it = packing_stage_one_masks_.emplace(key, std::move(v)).first;
        }
        const u64 *ct = in + q * ctw;
        for (const auto &am : it->second) {
            if (am.first == 0)
                terms.push_back(keylessTerm(ct, ct + nq * N, &am.second));
            else
                terms.push_back(term(x.extOf(q), x.pbOf(q), pack, powmod(5, am.first, M), &am.second));
        }
        off.push_back((uint32_t)terms.size());
    }
    DeviceBuffer y(c, n_jobs * 2 * E * N), ws(c, n_jobs * 2 * (nq - 1) * N);
    ck(hemm_hoisted_moddown(c->dev, terms.data(), off.data(), (uint32_t)n_jobs, (uint32_t)nq, x.premultiplied(), 1, y.data(),
                            out, (nq - 1) * N, ws.data(), nullptr));
    c->mark("packing and transform stage 1");
}

// The complex packing as a linear map on the slots, out = Z x + M_+ rho^(step)(x) + M_- rho^(-step)(x):
//   columns (step 1):  fus = m (x + i rho^1 x), out = fus + rho^-1 fus, m = even columns
//   rows (step w):     fus = m (x - i rho^w x), out = fus + rho^-w fus, m = even rows of width w
// i.e. Z = m +- i m', M_+ = +- i m, M_- = m' with m'[s] = m[s - step].  One hoisted sum with three terms per job: the two
// rotations and Z x, which needs no key switch (a term without a key).
void MatrixTransformer::complexPackingBatch(const HomEvaluator &eval, const u64 *in, size_t n_jobs, u64 level,
                                            const bool *rows, i64 w, u64 *out, const u64 *scale_levels) {
    const Context &c = eval.getContext();
    if (level < 1) throw std::invalid_argument("[complexPacking] level >= 1 is needed.");
    const u64 nq = level + 1, N = c->N, E = nq + c->nP, ctw = 2 * nq * N;
    const u64 log_slots = getLogFullSlots(c);
    // All three masks of a job are encoded over the extended basis (the unrotated term reads the chain limbs only) at
    // the scale that takes the input's scale to the fixed scale of level - 1 across the rescale.
    useChainOf(c);
    auto mask = [&](bool by_rows, int part, u64 from) -> const Plaintext & {
        const auto key = std::make_tuple((int)by_rows, w, level, part, from);
        auto it = pack_masks_.find(key);
        if (it != pack_masks_.end()) return it->second;
        const Message m = packingMaskMessage(by_rows, w, log_slots, part);
        EnDecoder endec(c);
        const Real scale = from == level ? c->delta[level] : c->delta[level - 1] * (Real)c->q[level] / c->delta[from];
        return pack_masks_.emplace(key, endec.encodeExtended(m, level, scale)).first->second;
    };
    auto from_of = [&](size_t q) { return scale_levels ? scale_levels[q] : level; };
    for (size_t q = 0; q < n_jobs; q++)
        if (from_of(q) < level) throw std::invalid_argument("[complexPacking] the scale must come from the same or a higher level.");
    const Sources x = extendSources(c, in, n_jobs, nq, nullptr, false);
    const KeyPack &pack = eval.getKeyPack();
    const Rot rot(c);
    std::vector<hemm_rot_term> terms;
    std::vector<uint32_t> off{0};
    for (size_t q = 0; q < n_jobs; q++) {
        const i64 step = rows[q] ? w : 1;
        terms.push_back(term(x.extOf(q), x.pbOf(q), pack, rot.galois(step), &mask(rows[q], 1, from_of(q))));
        terms.push_back(term(x.extOf(q), x.pbOf(q), pack, rot.galois(-step), &mask(rows[q], 2, from_of(q))));
        terms.push_back(keylessTerm(in + q * ctw, in + q * ctw + nq * N, &mask(rows[q], 0, from_of(q))));   // Z x: no key switch
        off.push_back((uint32_t)terms.size());
    }
    DeviceBuffer y(c, n_jobs * 2 * E * N), ws(c, n_jobs * 2 * (nq - 1) * N);
    ck(hemm_hoisted_moddown(c->dev, terms.data(), off.data(), (uint32_t)n_jobs, (uint32_t)nq, x.premultiplied(), 1, y.data(),
                            out, (nq - 1) * N, ws.data(), nullptr));
}

namespace {
// Sum over the shift index of a product whose row shifts are exact rotations (the tile block fills the slot vector),
// split into baby and giant steps, i = i1 + g i2 over `units` shifts (column shift of i cells = cu * i slots, row
// shift of i cells = rho^(i ru)):
//   C = sum_i2 rho^(g i2 ru)( U_i2 ),   U_i2 = sum_i1 rho^(-g i2 ru)(phi^i(sigma A)) (x) rho^(i1 ru)(tau B)
// * tau(B), at level T+1, is rotated only g - 1 times (one chain, plain ModDown);
// * every column shift phi^i(sigma A) is produced already rotated back by g i2 row units: the column masks do not
//   depend on the row, so this only changes the Galois element of shift i (still one key per shift);
// * the un-relinearised sums U_i2 (three polynomials) are rotated by the giant steps directly: d1 under the key of
//   rho(s), d2 under a key of rho(s)^2, all 2 (units/g - 1) terms summed in the extended basis before a single
//   ModDown merged with the rescale.  U_0 (in `acc`, which arrives holding the i = 0 term) joins the same sum with
//   its d2 under the multiplication key.
// units + g + 2 units/g key switches instead of 2 units.
// sigma_a: [2][T+3][N] at level T+2; tau_b: [2][T+2][N] at level T+1; U_out receives U_1 .. (each [3][T+2][N]).
// spread_block != 0: tau_b holds one tile block of that many slots and nothing else; every baby rotation then also
// gathers the copies rho^(-j spread_block), j = 1 .. slots / spread_block - 1, as further terms of its output, which
// is the rotation of tau(B) copied into every block (row shifts of a periodic vector are exact rotations).
void bsgsShiftProduct(const HomEvaluator &eval, u64 T, const u64 *sigma_a, const u64 *tau_b, Ciphertext &acc,
                      std::vector<Plaintext> &cm, i64 n, i64 units, i64 cu, i64 w, u64 batch, DeviceBuffer *U_out,
                      i64 *g_out, u64 spread_block = 0, bool u_ready = false, hipStream_t b_stream = nullptr,
                      bool unshifted_last = false) {
    const Context &c = eval.getContext();
    const u64 nq = T + 3, N = c->N, K = c->nP, E = nq + K, lo = nq - 1;
    const i64 ru = cu * w;
    const i64 g = bsgsBabyCount(units), n_giant = units / g;
    const KeyPack &pack = eval.getKeyPack();
    const Rot rot(c);
    const u64 ctl = 2 * lo * N;   // words of a two-polynomial ciphertext at level T+1
    // The sources of the column shifts (sigma(A) and its copy rotated by -n, both extended) do not depend on the
    // baby rotations of tau(B): two chains of small launches side by side.  b_stream: the side chain is already open
    // and tau(B) is being produced on it; the baby rotations then follow it there and the sources of sigma(A) take the
    // context's stream, with no join in between.  Otherwise the side chain is opened here for the sources of sigma(A).
    const hipStream_t s_b = b_stream, s_a = b_stream ? nullptr : c->forkSide();
    struct JoinOnExit {
        const Context &c;
        ~JoinOnExit() { c->joinSide(); }   // also when a launch below throws
    } join_on_exit{c};
    const Sources xa = extendSources(c, sigma_a, 1, nq, s_a);
    const i64 back = -n;
    const DeviceBuffer a2 = rotateSources(eval, xa, sigma_a, 1, &back, s_a);
    const Sources xa2 = extendSources(c, a2.data(), 1, nq, s_a);
    // baby rotations of tau(B): bb[i1] = rho^(i1 ru)(tau B), summed over the block copies when tau(B) is spread
    DeviceBuffer bb(c, (u64)g * ctl);
    const i64 copies = spread_block ? (i64)((c->N / 2) / spread_block) : 1;
    if (g > 1 || copies > 1) {
        const Sources xb = extendSources(c, tau_b, 1, lo, s_b, false);
        std::vector<hemm_rot_term> terms;
        std::vector<uint32_t> off{0};
        const i64 first_out = copies > 1 ? 0 : 1;   // bb[0] needs a launch only for its copies
        for (i64 i1 = first_out; i1 < g; i1++) {
            for (i64 j = 0; j < copies; j++) {
                if (i1 == 0 && j == 0) continue;     // the operand itself joins below
                terms.push_back(term(xb.extOf(0), xb.pbOf(0), pack, rot.galois(i1 * ru - j * (i64)spread_block), nullptr));
            }
            if (i1 == 0) terms.push_back(keylessTerm(tau_b, tau_b + lo * N, nullptr));   // no key switch for itself
            off.push_back((uint32_t)terms.size());
        }
        const u64 n_out = (u64)(g - first_out);
        DeviceBuffer yb(c, n_out * 2 * (lo + K) * N), ws(c, n_out * ctl);
        ck(hemm_hoisted_moddown(c->dev, terms.data(), off.data(), (uint32_t)n_out, (uint32_t)lo, xb.premultiplied(), 0,
                                yb.data(), bb.data() + (u64)first_out * ctl, lo * N, ws.data(), s_b));
    }
    if (copies <= 1) (void)hipMemcpyAsync(bb.data(), tau_b, ctl * 8, hipMemcpyDeviceToDevice, c->on(s_b));
    // column shifts of sigma(A), shift i rotated back by g (i / g) row units
    std::vector<Shift> sa;
    for (i64 i = 1; i < units; i++)
        sa.push_back(Shift{cu * i - g * (i / g) * ru, &cm[(size_t)(2 * cu * i + 1)], &cm[(size_t)(2 * cu * i)]});
    const size_t G = std::max<u64>(1, std::min<u64>(2 * batch, (u64)std::max<i64>(1, units - 1)));
    // Chains of G shifts.  When the shifts split into exactly two chains, they are cut on a giant-step boundary (so
    // that they accumulate into different partial sums) and the second runs on the side stream beside the first, with
    // buffers of its own: each launch of one chain fills the part-empty last round of workgroups of the other's
    // (measured -1.3 % per product; staggering the chains so that one's inverse transforms meet the other's key
    // product gained nothing; three and four chains on as many streams cost 1.0 % and 2.3 %).
    std::vector<std::pair<size_t, size_t>> chains;   // (first, count)
    for (size_t first = 0; first < sa.size(); first += G) chains.push_back({first, std::min(G, sa.size() - first)});
    bool two_streams = false;
    // (chains of up to 32 shifts: their term lists travel in the kernel arguments; longer lists would be staged, each
    // stream through a region of its own, and copied from pageable memory, which waits for the stream)
    if (chains.size() == 2 && G <= 32) {
        const size_t cut = ((chains[0].second + 1) / (size_t)g) * (size_t)g;   // shift index q holds i = q + 1
        if (cut >= 1 && cut - 1 >= 1 && cut - 1 < sa.size() && sa.size() - (cut - 1) <= G && cut - 1 <= G) {
            chains[0] = {0, cut - 1};
            chains[1] = {cut - 1, sa.size() - (cut - 1)};
            two_streams = true;
        }
    }
    // The operands have come their own ways and the shifts run as two chains: the streams do not meet here.  The first
    // chain's sums (which need only the sources of sigma(A)) follow them on the context's stream and wait for the baby
    // rotations just before their products with them; the second chain follows the baby rotations on the side stream
    // once the sources of sigma(A) are there.  The large launches of a chain so fill the gaps of the other operand's
    // chain of small ones.
    const bool no_meeting = b_stream != nullptr && two_streams && unshifted_last;
    if (no_meeting) {
        c->markSide();
        c->sideWaitsForMain();
    } else {
        c->joinSide();
    }
    c->mark("rotation sources and baby rotations");
    // U, polynomial-major: polynomial p of U_i2 at (p * n_giant + i2) * lo * N, so that one ModUp batch later
    // covers d1 and d2 of all of them.  U_0 starts from `acc`, which holds the i = 0 term.
    const u64 pw = lo * N, us = (u64)n_giant * pw;
    if (unshifted_last) {     // the i = 0 term joins U_0 behind the first chain of shifts
        U_out->resize(c, 3 * us);
    } else if (!u_ready) {   // otherwise the caller has put the i = 0 term where U_0 lives
        U_out->resize(c, 3 * us);
        for (u64 p = 0; p < 3; p++)
            (void)hipMemcpyAsync(U_out->data() + p * us, acc.buf_.data() + p * pw, pw * 8, hipMemcpyDeviceToDevice, c->stream());
    }
    std::vector<bool> started((size_t)n_giant, false);
    started[0] = !unshifted_last;
    DeviceBuffer ya(c, G * 2 * E * N), t1(c, G * ctl), ws(c, G * ctl), ya2, t12, ws2, low_a;
    if (unshifted_last) low_a = DeviceBuffer(c, ctl);
    if (two_streams) {
        ya2 = DeviceBuffer(c, G * 2 * E * N);
        t12 = DeviceBuffer(c, G * ctl);
        ws2 = DeviceBuffer(c, G * ctl);
    }
    auto accumulate = [&](size_t first, size_t cnt, const u64 *tb, hipStream_t st) {
        // shift index q holds i = q + 1: consecutive i with the same i2 pair with consecutive baby rotations
        // one launch for the giant-step groups of the chain (each group its own accumulator)
        size_t q = first;
        std::vector<hemm_tensor_group> groups;
        auto flush = [&]() {
            if (!groups.empty())
                ck(hemm_tensor_batch_groups(c->dev, groups.data(), (uint32_t)groups.size(), (uint32_t)lo, us, st));
            groups.clear();
        };
        while (q < first + cnt) {
            const i64 ii = (i64)q + 1, i2 = ii / g, i1 = ii % g;
            const size_t run = std::min<size_t>(first + cnt - q, (size_t)(g - i1));
            if (N < 512) {
                ck(hemm_tensor_batch_strided(c->dev, tb + (q - first) * ctl, bb.data() + (u64)i1 * ctl, (uint32_t)run,
                                             (uint32_t)lo, U_out->data() + (u64)i2 * pw, us,
                                             started[(size_t)i2] ? 1 : 0, st));
            } else {
                // a group that continues an accumulator already in the list would race with it: close the list first
                for (const hemm_tensor_group &h : groups)
                    if (h.acc3 == U_out->data() + (u64)i2 * pw) {
                        flush();
                        break;
                    }
                groups.push_back(hemm_tensor_group{tb + (q - first) * ctl, bb.data() + (u64)i1 * ctl,
                                                   U_out->data() + (u64)i2 * pw, (uint32_t)run,
                                                   started[(size_t)i2] ? 1u : 0u});
                if (groups.size() == 8) flush();
            }
            started[(size_t)i2] = true;
            q += run;
        }
        flush();
    };
    // forked before the first chain is queued: the side stream waits only for what both chains depend on
    const hipStream_t side2 = !two_streams ? nullptr : no_meeting ? b_stream : c->forkSide();
    for (size_t ch = 0; ch < chains.size(); ch++) {
        const size_t first = chains[ch].first, cnt = chains[ch].second;
        const bool on_side = two_streams && ch == 1;
        const hipStream_t st = on_side ? side2 : nullptr;
        u64 *yap = on_side ? ya2.data() : ya.data(), *t1p = on_side ? t12.data() : t1.data(),
            *wsp = on_side ? ws2.data() : ws.data();
        std::vector<hemm_rot_term> terms;
        std::vector<uint32_t> off{0};
        pushShifts(eval, xa, 0, xa2, 0, sa, first, cnt, terms, off);
        ck(hemm_hoisted_moddown(c->dev, terms.data(), off.data(), (uint32_t)cnt, (uint32_t)nq, 1, 1, yap, t1p, lo * N,
                                wsp, st));
        if (no_meeting && !on_side) c->waitSideMark();
        accumulate(first, cnt, t1p, st);
    }
    if (unshifted_last) {
        // sigma(A) lowered to T+1 times tau(B), on the context's stream behind the chain that owns U_0: lowering it in
        // front of the rotation sources would lengthen the chain of small launches that the main loop waits for, here
        // it runs beside the second chain (sums of residues do not depend on their order).  The lowering is the only
        // call that works in the context's scratch region while the side chain is open.
        levelDownOneBatch(c, sigma_a, 2, T + 2, low_a.data());
        ck(hemm_tensor_batch_strided(c->dev, low_a.data(), tau_b, 1, (uint32_t)lo, U_out->data(), us,
                                     started[0] ? 1 : 0, nullptr));
    }
    if (two_streams) c->joinSide();
    *g_out = g;
}

// res = sum_i2 rho^(g i2 ru)(U_i2) relinearised and rescaled, all through one hoisted launch: U_i2 (i2 >= 1) gives
// the terms (d1 under the key of rho(s), d2 under the key of rho(s)^2); U_0 gives its d2 under the multiplication key
// with the identity automorphism, and its d1 is added to the second polynomial after the single ModDown.
// add_conj: the result is x + conj(x) for the sum x described above -- every term enters a second time under its
// Galois element times 2N - 1 (keys of the composite elements; d1 of U_0, which needs no key switch in x, is switched
// under the conjugation key), so the real part of a complex-packed product needs no key-switch round of its own.
void bsgsGiantSteps(const HomEvaluator &eval, u64 T, DeviceBuffer &U, i64 g, i64 n_giant, i64 ru, Ciphertext &acc,
                    CtxtTensor &res, bool add_conj = false) {
    const Context &c = eval.getContext();
    const u64 N = c->N, K = c->nP, lo = T + 1;
    const KeyPack &pack = eval.getKeyPack();
    const Rot rot(c);
    // The partial sums (three polynomials each, level T+1) are rescaled first: everything after runs on T+1 instead
    // of T+2 limbs -- one digit instead of two where that crosses a digit boundary -- and ends in a plain ModDown.
    // U is polynomial-major ([3][n_giant][.][N]): all 3 n_giant polynomials are rescaled by one launch chain, and d1 and
    // d2 of all partial sums are 2 n_giant polynomials in a row, extended by ONE ModUp batch (d1 of U_0 rides along
    // unused).
    (void)acc;
    const u64 m = (u64)n_giant, beta = (lo + c->alpha - 1) / c->alpha, El = lo + K, pw = lo * N, us = m * pw;
    {
        DeviceBuffer Ur(c, 3 * us);
        // a rescale call works in the context's scratch region of (dnum + 7) (nQ + nP) limbs
        const u64 cap = std::max<u64>(1, (c->dnum + 7) * (c->nQ + c->nP) / (lo + 1));
        for (u64 first = 0; first < 3 * m; first += cap) {
            const u64 cnt = std::min<u64>(cap, 3 * m - first);
            ck(hemm_rescale(c->dev, U.data() + first * (lo + 1) * N, (lo + 1) * N, Ur.data() + first * pw, pw,
                            (uint32_t)(lo + 1), (uint32_t)cnt, nullptr));
        }
        U = std::move(Ur);
    }
    DeviceBuffer ext(c, 2 * m * beta * El * N), wsu(c, 2 * m * lo * N);
    ck(hemm_modup_batch(c->dev, U.data() + us, pw, (uint32_t)lo, (uint32_t)(2 * m), ext.data(), wsu.data(), nullptr));
    const u64 *ext1 = ext.data(), *ext2 = ext.data() + m * beta * El * N;   // [i2][beta][El][N] each
    // d0 of every partial sum enters its term as it is (the launch multiplies by P); d1 of U_0, which needs no key
    // switch, joins the second polynomial as a term without a key (P d1 on the chain limbs)
    std::vector<hemm_rot_term> terms;
    terms.push_back(keylessTerm(nullptr, U.data() + us, nullptr));
    {
        hemm_rot_term t{};
        t.ext = ext2;
        t.b = U.data();
        set_key(t, pack, 0, 0);
        t.mask = nullptr;
        t.galois = 1;
        terms.push_back(t);
    }
    for (u64 i = 1; i < m; i++) {
        const u64 gal = rot.galois((i64)i * g * ru);
        hemm_rot_term t{};
        t.ext = ext1 + i * beta * El * N;
        t.b = U.data() + i * pw;
        set_key(t, pack, 1, gal);
        t.mask = nullptr;
        t.galois = gal;
        terms.push_back(t);
        t.ext = ext2 + i * beta * El * N;
        t.b = nullptr;
        set_key(t, pack, 2, gal);
        terms.push_back(t);
    }
    if (add_conj) {
        const u64 cj = 2 * N - 1;
        for (u64 i = 0; i < m; i++) {
            const u64 gal = i == 0 ? 1 : rot.galois((i64)i * g * ru), gc = (gal * cj) % (2 * N);
            hemm_rot_term t{};
            t.ext = ext1 + i * beta * El * N;
            t.b = U.data() + i * pw;
            set_key(t, pack, 1, gc);
            t.mask = nullptr;
            t.galois = gc;
            terms.push_back(t);
            t.ext = ext2 + i * beta * El * N;
            t.b = nullptr;
            set_key(t, pack, 2, gc);
            terms.push_back(t);
        }
    }
    const uint32_t off[2] = {0, (uint32_t)terms.size()};
    res.get().allocate(2, T, 0);
    DeviceBuffer yg(c, 2 * El * N), wsg(c, 2 * lo * N);
    ck(hemm_hoisted_terms(c->dev, terms.data(), off, 1, (uint32_t)lo, yg.data(), 0, nullptr));
    ck(hemm_moddown_batch(c->dev, yg.data(), (uint32_t)lo, 2, 0, res.get().buf_.data(), lo * N, wsg.data(), nullptr));
}

// The operands of a product on their own ways: B's chain is queued on the side stream -- the context's stream is
// pointed there for as long as B's calls are made -- and A's on the context's own.  On leaving (also by an exception)
// the context's stream is its own again, the side chain has joined and the phase marks, which the two interleaved
// chains would garble, are back on.
class OwnWays {
  public:
    explicit OwnWays(const Context &c)
        : c_(c), own_(hemm_context_stream(c->dev)), trace_(c->trace_on), side_(c->forkSide()) {
        c->trace_on = false;
    }
    ~OwnWays() {
        (void)hemm_context_set_stream(c_->dev, own_);
        c_->joinSide();
        c_->trace_on = trace_;
    }
    OwnWays(const OwnWays &) = delete;
    OwnWays &operator=(const OwnWays &) = delete;
    void toSide() const { ck(hemm_context_set_stream(c_->dev, side_)); }
    void toOwn() const { ck(hemm_context_set_stream(c_->dev, own_)); }
    void marksOn() const { c_->trace_on = trace_; }
    hipStream_t side() const { return side_; }

  private:
    const Context &c_;
    void *own_;
    bool trace_;
    hipStream_t side_;
};

// What follows the two chains: the baby rotations of tau(B) (level T+1) go on where it was made, on the side stream,
// while the rotation sources of sigma(A) (level T+2) are made on the context's; the chains meet in front of the main
// loop; the unshifted term, sigma(A) lowered to T+1 times tau(B), is taken behind the loop's first chain.
// Complex-packed cells: k / 2 shifts of two columns / rows.
CtxtTensor ownWaysShiftProduct(const HomEvaluator &eval, u64 T, const u64 *sigma_a, const u64 *tau_b,
                               std::vector<Plaintext> &cm, i64 rows, i64 cols, i64 k, i64 w, u64 batch, bool spread,
                               hipStream_t side, bool add_conj) {
    const Context &c = eval.getContext();
    DeviceBuffer U;
    Ciphertext acc(c);
    acc.allocate(3, T + 1, 1);
    CtxtTensor res(c, rows, cols, w);
    i64 g = 1;
    bsgsShiftProduct(eval, T, sigma_a, tau_b, acc, cm, k, k / 2, 2, w, batch, &U, &g, spread ? (u64)(k * w) : 0, false,
                     side, true);
    c->mark("main loop");
    bsgsGiantSteps(eval, T, U, g, (k / 2) / g, 2 * w, acc, res, add_conj);
    c->mark("giant steps");
    if (spread) res.get().occupied_ = (u64)(k * w);   // the product sits in the first block, the rest is empty
    return res;
}
}  // namespace

namespace {
// HomEvaluator::levelDown of two ciphertexts to level Lt into one buffer [2 cts][2][Lt+1][N]; when they share a higher
// level, both at once: multiply by round(Delta_Lt q_{Lt+1} / Delta_level) over Lt+2 limbs, then one rescale of the four
// polynomials straight into the buffer
void jointLevelDown(const HomEvaluator &eval, const Ciphertext &a, const Ciphertext &b, u64 Lt, u64 *joint) {
    const Context &c = eval.getContext();
    const u64 N = c->N, ctw_in = 2 * (Lt + 1) * N, la = a.getLevel(), lb = b.getLevel();
    if (la == lb && la > Lt && a.getRescaleCounter() == 0 && b.getRescaleCounter() == 0) {
        const u64 nl = Lt + 2;
        const i64 v = (i64)llround(c->delta[Lt] * (Real)c->q[Lt + 1] / c->delta[la]);
        std::vector<u64> sc(nl);
        for (u64 j = 0; j < nl; j++) sc[j] = v >= 0 ? (u64)v % c->q[j] : (c->q[j] - (u64)(-v) % c->q[j]) % c->q[j];
        DeviceBuffer t(c, 4 * nl * N);
        ck(hemm_mul_scalar(c->dev, a.buf_.data(), a.polyStride(), sc.data(), t.data(), nl * N, (uint32_t)nl, 0, 2, nullptr));
        ck(hemm_mul_scalar(c->dev, b.buf_.data(), b.polyStride(), sc.data(), t.data() + 2 * nl * N, nl * N, (uint32_t)nl, 0, 2, nullptr));
        ck(hemm_rescale(c->dev, t.data(), nl * N, joint, (nl - 1) * N, (uint32_t)nl, 4, nullptr));
    } else {
        Ciphertext la_ct(c), lb_ct(c);
        eval.levelDown(a, Lt, la_ct);
        eval.levelDown(b, Lt, lb_ct);
        (void)hipMemcpyAsync(joint, la_ct.buf_.data(), ctw_in * 8, hipMemcpyDeviceToDevice, c->stream());
        (void)hipMemcpyAsync(joint + ctw_in, lb_ct.buf_.data(), ctw_in * 8, hipMemcpyDeviceToDevice, c->stream());
    }
}

}  // namespace

namespace {
CtxtTensor ccmmFused(const HomEvaluator &eval, const Bootstrapper &btp, const CtxtTensor &op1, const CtxtTensor &op2, u64 T,
                     MatrixTransformer &tr, u64 batch, bool single_tile, bool packed, const u64 *pre = nullptr,
                     u64 pre_level = 0, bool merge_packing = false, bool add_conj = false, int first_stage = 1);
}
CtxtTensor multMatMatFused(const HomEvaluator &eval, const Bootstrapper &btp, const CtxtTensor &op1,
                           const CtxtTensor &op2, u64 T, MatrixTransformer &tr, u64 batch, bool single_tile) {
    return ccmmFused(eval, btp, op1, op2, T, tr, batch, single_tile, false);
}

namespace {
// packed: the operands are complex-packed (2 x 2 cells): sigma / tau of the packed kinds, n / 2 shifts of two columns /
// two rows each; otherwise the same schedule.  pre: both operands already side by side at pre_level (two ciphertexts
// of two polynomials, the layout the joint transforms read); op1 / op2 then only give the tile shapes.
// merge_packing (with packed): the operands are NOT packed yet; the complex packing and the packed transform run as one
// composite one-stage transform from T+3 (MaskKind::PackingHorizontal / PackingVertical), for operands with only
// three levels above the target.
// add_conj: the result is x + conj(x) of the product x (the real part, twice, of a complex-packed product): inside the
// giant-step sum where the schedule has one, by a conjugation afterwards otherwise.
// first_stage = 2 (with pre at T+3): pre is what the first stage of the two-stage transforms from T+4 left -- taken
// together with the packing, MatrixTransformer::packingStageOne -- and only the second stage runs here.
CtxtTensor ccmmFused(const HomEvaluator &eval, const Bootstrapper &btp, const CtxtTensor &op1, const CtxtTensor &op2, u64 T,
                     MatrixTransformer &tr, u64 batch, bool single_tile, bool packed, const u64 *pre, u64 pre_level,
                     bool merge_packing, bool add_conj, int first_stage) {
    const Context &c = eval.getContext();
    const i64 rows = op1.getHeight(), cols = op2.getWidth();
    const i64 k = pow2ceil(commonInside(op1, op2)), w = commonBlockWidth(op1, op2);
    const u64 min_level = pre ? pre_level : std::min(op1.getLevel(), op2.getLevel());
    if (min_level < 1 + btp.getMinLevelForBootstrap())
        throw std::invalid_argument("[multMatMat] level >= " + std::to_string(1 + btp.getMinLevelForBootstrap()) +
                                    " is needed.");
    if (pre && min_level < 4 + btp.getMinLevelForBootstrap())
        throw RuntimeException("bootstrapping is not part of this build");
    // the operands are only read: no working copies unless they have to be refreshed first
    const TileTensorShape shape_a(rows, k, w), shape_b(k, cols, w);
    const Ciphertext *pa = &op1.get(), *pb = &op2.get();
    Ciphertext own_a(c), own_b(c);
    if (min_level < 4 + btp.getMinLevelForBootstrap()) {
        own_a = op1.get();
        own_b = op2.get();
        btp.bootstrapExtended(own_a, own_a, own_b);
        pa = &own_a;
        pb = &own_b;
    }
    if (min_level < T + 3)
        throw std::invalid_argument("[multMatMat] level >= " + std::to_string(T + 3) + " is needed.");
    // The transforms end at level T+2.  With a level to spare they run in two stages from T+4 (far fewer rotations
    // and masks, MatrixTransformer::diagonalTransformTwoStage), otherwise in one from T+3; lowering the operands first
    // gives the same values with 9 or 8 instead of 13 limbs.
    std::vector<Plaintext> &cm = tr.getColMaskExt(eval, shape_a, T + 2);
    // sigma(A) and tau(B) through one launch chain; `ab` holds both results [2 cts][2][nq][N]
    const u64 nq = T + 3, N = c->N, E = nq + c->nP, lo = nq - 1, ctw = 2 * nq * N;
    const bool two_stage = !merge_packing && min_level >= T + 4 && shape_a.getNumRows() == shape_a.getNumCols() &&
                           shape_b.getNumRows() == shape_b.getNumCols();
    const u64 Lt = two_stage ? T + 4 : T + 3;   // level the transforms start from
    DeviceBuffer ab(c, 2 * ctw);
    if (first_stage == 2) {   // the first stage came with the packing: the second one from T+3
        if (!pre || pre_level != T + 3 || !packed || merge_packing)
            throw std::invalid_argument("[multMatMat] a second stage alone takes packed operands prepared at T+3.");
        const MaskKind kinds[2] = {MaskKind::PackedHorizontal, MaskKind::PackedVertical};
        const TileTensorShape shapes[2] = {shape_a, shape_b};
        tr.diagonalTransformTwoStage(eval, pre, 2, T + 4, kinds, shapes, ab.data(), nullptr, 2);
    } else {
        const u64 ctw_in = 2 * (Lt + 1) * N;
        DeviceBuffer joint;
        const u64 *src = pre;
        if (!pre || pre_level != Lt) {
            if (pre) throw std::invalid_argument("[multMatMat] prepared operands must be at the transforms' level.");
            joint = DeviceBuffer(c, 2 * ctw_in);
            jointLevelDown(eval, *pa, *pb, Lt, joint.data());
            src = joint.data();
        }
        const MaskKind kinds[2] = {merge_packing ? MaskKind::PackingHorizontal
                                   : packed      ? MaskKind::PackedHorizontal
                                                 : MaskKind::Horizontal,
                                   merge_packing ? MaskKind::PackingVertical
                                   : packed      ? MaskKind::PackedVertical
                                                 : MaskKind::Vertical};
        const TileTensorShape shapes[2] = {shape_a, shape_b};
        if (two_stage)
            tr.diagonalTransformTwoStage(eval, src, 2, Lt, kinds, shapes, ab.data());
        else
            tr.diagonalTransformBatch(eval, src, 2, Lt, kinds, shapes, ab.data());
    }
    // the k = 0 term sigma(A) (x) tau(B) joins the accumulator at the shifts' level T+1
    Ciphertext acc(c);
    acc.allocate(3, T + 1, 1);
    DeviceBuffer low(c, 2 * 2 * lo * N);   // sigma(A), tau(B) at level T+1
    levelDownOneBatch(c, ab.data(), 4, T + 2, low.data());
    const i64 cu = packed ? 2 : 1;
    const u64 slots = c->N / 2;
    const bool spread = single_tile && (u64)(k * w) < slots && slots % (u64)(k * w) == 0;
    const bool bsgs = k / cu > 1 && ((u64)(k * w) == slots || spread);
    DeviceBuffer U;
    if (bsgs) {   // the term goes straight to the first partial sum of the baby-step / giant-step split
        const u64 us = (u64)((k / cu) / bsgsBabyCount(k / cu)) * lo * N;
        U.resize(c, 3 * us);
        ck(hemm_tensor_batch_strided(c->dev, low.data(), low.data() + 2 * lo * N, 1, (uint32_t)lo, U.data(), us, 0, nullptr));
    } else {
        ck(hemm_tensor_batch(c->dev, low.data(), low.data() + 2 * lo * N, 1, (uint32_t)lo, acc.buf_.data(), 0, nullptr));
    }
    CtxtTensor res(c, rows, cols, w);
    auto finish = [&]() {
        eval.relinearize(acc, res.get());
        eval.rescale(res.get());
        if (add_conj) {
            Ciphertext cj(c);
            eval.conjugate(res.get(), cj);
            eval.add(res.get(), cj, res.get());
        }
    };
    if (k / cu <= 1) {
        finish();
        return res;
    }

    const i64 n = k;
    size_t G = std::max<u64>(1, std::min<u64>(batch, (u64)(n - 1)));
    // spread: tau(B) is copied into every tile block on the fly by the baby rotations (bsgsShiftProduct).  sigma(A)
    // stays as it is: rotated back by g k2 rows it spills into the empty block below and the giant step brings it
    // home, so the product comes out in the first block with the other blocks empty.
    if (bsgs) {
        i64 g = 1;
        c->mark("unshifted term");
        bsgsShiftProduct(eval, T, ab.data(), low.data() + 2 * lo * N, acc, cm, n, n / cu, cu, w, batch, &U, &g,
                         spread ? (u64)(n * w) : 0, true);
        c->mark("main loop");
        bsgsGiantSteps(eval, T, U, g, (n / cu) / g, cu * w, acc, res, add_conj);
        c->mark("giant steps");
        if (spread) res.get().occupied_ = (u64)(n * w);   // the product sits in the first block, the rest is empty
        return res;
    }
    // Row shifts that wrap inside a tile block (stacked tiles, or content that is not known to be a single tile):
    // every shift of tau(B) is a masked pair like the column shifts of sigma(A).  Complex-packed operands shift by
    // cells of two columns / two rows, so they need half as many.
    std::vector<Plaintext> &rm = tr.getRowMaskExt(eval, shape_b, T + 2);
    std::vector<Shift> sa, sb;
    for (i64 i = 1; i < n / cu; i++) {
        sa.push_back(Shift{cu * i, &cm[(size_t)(2 * cu * i + 1)], &cm[(size_t)(2 * cu * i)]});
        sb.push_back(Shift{cu * i * w, &rm[(size_t)(2 * cu * i + 1)], &rm[(size_t)(2 * cu * i)]});
    }
    G = std::max<u64>(1, std::min<u64>(batch, (u64)sa.size()));
    // rotation sources: sigma(A), tau(B) and their copies rotated by -n columns / -n rows
    const Sources x = extendSources(c, ab.data(), 2, nq);
    const i64 back[2] = {-n, -n * w};
    const DeviceBuffer ab2 = rotateSources(eval, x, ab.data(), 2, back);
    const Sources x2 = extendSources(c, ab2.data(), 2, nq);
    DeviceBuffer y(c, 2 * G * 2 * E * N), t(c, 2 * G * 2 * lo * N), ws(c, 2 * G * 2 * lo * N);
    for (size_t first = 0; first < sa.size(); first += G) {
        // cnt column shifts of sigma(A), then cnt row shifts of tau(B): one launch chain for all 2 cnt outputs
        const size_t cnt = std::min(G, sa.size() - first);
        std::vector<hemm_rot_term> terms;
        std::vector<uint32_t> off{0};
        pushShifts(eval, x, 0, x2, 0, sa, first, cnt, terms, off);
        pushShifts(eval, x, 1, x2, 1, sb, first, cnt, terms, off);
        ck(hemm_hoisted_moddown(c->dev, terms.data(), off.data(), (uint32_t)(2 * cnt), (uint32_t)nq, 1, 1, y.data(), t.data(), lo * N, ws.data(), nullptr));
        ck(hemm_tensor_batch(c->dev, t.data(), t.data() + cnt * 2 * lo * N, (uint32_t)cnt, (uint32_t)lo, acc.buf_.data(),
                             1, nullptr));
    }
    finish();
    return res;
}
}  // namespace

CtxtTensor multPackedMatMatFused(const HomEvaluator &eval, const Bootstrapper &btp, const CtxtTensor &op1,
                                 const CtxtTensor &op2, u64 T, MatrixTransformer &tr, u64 batch, bool single_tile) {
    const Context &c = eval.getContext();
    // Square tiles with A four levels and B three levels above the target: the operands go their own ways, as in the
    // complex-packed product.  tau(B) runs from T+3 to T+1 on the side stream, where the baby rotations follow it;
    // sigma(A) runs from T+4 to T+2 on the context's stream.  Operands above these levels are only truncated (the
    // first stage's masks absorb the change of scale), so nothing but sigma(A)'s copy for the unshifted term passes
    // through the context's scratch region while the side chain is open.
    if (op1.getLevel() >= T + 4 && op2.getLevel() >= T + 3 && op1.get().getRescaleCounter() == 0 &&
        op2.get().getRescaleCounter() == 0 && op1.get().getNumPoly() == 2 && op2.get().getNumPoly() == 2 &&
        std::min(op1.getLevel(), op2.getLevel()) >= 4 + btp.getMinLevelForBootstrap()) {
        const i64 rows = op1.getHeight(), cols = op2.getWidth();
        const i64 k = pow2ceil(commonInside(op1, op2)), w = commonBlockWidth(op1, op2);
        const u64 slots = c->N / 2, N = c->N, lo = T + 2;
        const bool spread = single_tile && (u64)(k * w) < slots && slots % (u64)(k * w) == 0;
        if (rows == k && cols == k && k / 2 >= 4 && ((u64)(k * w) == slots || spread)) {
            const TileTensorShape shape_a(rows, k, w), shape_b(k, cols, w);
            std::vector<Plaintext> &cm = tr.getColMaskExt(eval, shape_a, T + 2);
            OwnWays ways(c);
            ways.toSide();
            const Ciphertext tb = tr.lowerAndTransformFused(eval, op2.get(), MaskKind::PackedVertical, shape_b, T + 1);
            ways.toOwn();
            const Ciphertext sa = tr.lowerAndTransformFused(eval, op1.get(), MaskKind::PackedHorizontal, shape_a, T + 2);
            ways.marksOn();
            c->mark("transforms");
            return ownWaysShiftProduct(eval, T, sa.buf_.data(), tb.buf_.data(), cm, rows, cols, k, w, batch,
                                       spread, ways.side(), false);
        }
    }
    // both operands a level above what the reference asks of B: sigma and tau share one launch chain, as in the
    // unpacked product (tau(B) is then lowered to T+1 with sigma(A)'s copy for the unshifted term)
    if (std::min(op1.getLevel(), op2.getLevel()) >= T + 3 && op1.get().getRescaleCounter() == 0 &&
        op2.get().getRescaleCounter() == 0) {
        const u64 slots = c->N / 2;
        const i64 kk = pow2ceil(commonInside(op1, op2)), ww = commonBlockWidth(op1, op2);
        const bool spread = single_tile && (u64)(kk * ww) < slots && slots % (u64)(kk * ww) == 0;
        if ((u64)(kk * ww) == slots || spread) return ccmmFused(eval, btp, op1, op2, T, tr, batch, single_tile, true);
    }
    const i64 rows = op1.getHeight(), cols = op2.getWidth();
    const i64 k = pow2ceil(commonInside(op1, op2)), w = commonBlockWidth(op1, op2);
    if (std::min(op1.getLevel(), op2.getLevel()) < 1 + btp.getMinLevelForBootstrap())
        throw std::invalid_argument("[multMatMat] level >= " + std::to_string(1 + btp.getMinLevelForBootstrap()) +
                                    " is needed.");
    if (op1.getLevel() < T + 3 || op2.getLevel() < T + 2)
        throw std::invalid_argument("[multPackedMatMat] levels >= " + std::to_string(T + 3) + " / " +
                                    std::to_string(T + 2) + " are needed.");
    const u64 slots = c->N / 2;
    // one tile block in an otherwise empty slot vector: tau(B) is treated as copied into every block (the baby
    // rotations gather the copies), which makes its row shifts exact rotations, as in multMatMatFused
    const bool spread = single_tile && (u64)(k * w) < slots && slots % (u64)(k * w) == 0;
    if ((u64)(k * w) != slots && !spread)
        throw std::invalid_argument("[multPackedMatMat] the row shift must be cyclic: rows * block width == slots");
    CtxtTensor a{op1}, b{op2};
    a.setShape(rows, k);
    b.setShape(k, cols);
    std::vector<Plaintext> &cm = tr.getColMaskExt(eval, a.getShape(), T + 2);
    a.get() = tr.lowerAndTransformFused(eval, a.get(), MaskKind::PackedHorizontal, a.getShape(), T + 2);
    b.get() = tr.lowerAndTransformFused(eval, b.get(), MaskKind::PackedVertical, b.getShape(), T + 1);
    const u64 nqa = T + 3, nqb = T + 2, N = c->N, K = c->nP, lo = T + 2;  // both sides end at T+1 (lo limbs)
    // the k = 0 term joins the accumulator at level T+1: sigma(A) lowered one level, tau(B) as it is
    Ciphertext acc(c);
    acc.allocate(3, T + 1, 1);
    {
        DeviceBuffer low(c, 2 * lo * N);
        levelDownOneBatch(c, a.get().buf_.data(), 2, T + 2, low.data());
        ck(hemm_tensor_batch(c->dev, low.data(), b.get().buf_.data(), 1, (uint32_t)lo, acc.buf_.data(), 0, nullptr));
    }
    CtxtTensor res(c, rows, cols, w);
    auto finish = [&]() {
        eval.relinearize(acc, res.get());
        eval.rescale(res.get());
    };
    if (k / 2 <= 1) {
        finish();
        return res;
    }

    const i64 n = k;
    (void)nqa;
    (void)nqb;
    (void)N;
    (void)K;
    // column shifts of sigma(A) by 2 i, row rotations of tau(B) by 2 i w: baby-step / giant-step over i
    DeviceBuffer U;
    i64 g = 1;
    bsgsShiftProduct(eval, T, a.get().buf_.data(), b.get().buf_.data(), acc, cm, n, n / 2, 2, w, batch, &U, &g,
                     spread ? (u64)(n * w) : 0);
    bsgsGiantSteps(eval, T, U, g, (n / 2) / g, 2 * w, acc, res);
    if (spread) res.get().occupied_ = (u64)(n * w);
    return res;
}

void multMatMatPreFused(const HomEvaluator &eval, const CtxtTensor &a_in, std::vector<Ciphertext> &tmp, u64 T,
                        MatrixTransformer &tr, u64 batch, bool first_block_only) {
    const Context &c = eval.getContext();
    tmp.clear();
    const i64 n = a_in.getHeight();
    CtxtTensor a(a_in);
    if (a.getLevel() < T + 3)
        throw std::invalid_argument("[multMatMatPre] level >= " + std::to_string(T + 3) + " is needed.");
    std::vector<Plaintext> &cm = tr.getColMaskExt(eval, a.getShape(), T + 2, first_block_only);
    a.get() = tr.lowerAndTransformFused(eval, a.get(), MaskKind::Horizontal, a.getShape(), T + 2);
    Ciphertext first_ct(c);
    if (first_block_only)   // shift 0 is masked like the others so that it too is empty outside the first tile block
        eval.mult(a.get(), tr.firstBlockMask(eval, a.getShape(), T + 2), first_ct);
    else
        eval.levelDownOne(a.get(), first_ct);
    tmp.push_back(first_ct);
    std::vector<Shift> sa;
    for (i64 i = 1; i < n; i++) sa.push_back(Shift{i, &cm[(size_t)(2 * i + 1)], &cm[(size_t)(2 * i)]});
    const u64 nq = T + 3, N = c->N, E = nq + c->nP, lo = nq - 1;
    const Sources x = extendSources(c, a.get().buf_.data(), 1, nq);
    const i64 back = -n;
    const DeviceBuffer a2 = rotateSources(eval, x, a.get().buf_.data(), 1, &back);
    const Sources x2 = extendSources(c, a2.data(), 1, nq);
    const size_t G = std::max<u64>(1, std::min<u64>(batch, (u64)sa.size()));
    DeviceBuffer y(c, G * 2 * E * N), t(c, G * 2 * lo * N), ws(c, G * 2 * lo * N);
    for (size_t first = 0; first < sa.size(); first += G) {
        const size_t cnt = std::min(G, sa.size() - first);
        std::vector<hemm_rot_term> terms;
        std::vector<uint32_t> off{0};
        pushShifts(eval, x, 0, x2, 0, sa, first, cnt, terms, off);
        ck(hemm_hoisted_moddown(c->dev, terms.data(), off.data(), (uint32_t)cnt, (uint32_t)nq, 1, 1, y.data(), t.data(), lo * N, ws.data(), nullptr));
        for (size_t q = 0; q < cnt; q++) {
            Ciphertext ct(c);
            ct.allocate(2, T + 1, 0);
            (void)hipMemcpyAsync(ct.buf_.data(), t.data() + q * 2 * lo * N, 2 * lo * N * 8, hipMemcpyDeviceToDevice,
                                 c->stream());
            tmp.push_back(std::move(ct));
        }
    }
}

}  // namespace HELLM

namespace HELLM {

// multPackedMatMatPreRot with the batched launches: shift i moves the packed sigma(A) by 2 i columns inside its tile,
// main and wrapped part under the key of that one rotation (the copy rotated by -n is prepared once), 2 * batch
// shifts per hoisted launch, ModDown merged with the rescale of the mask product.
void multPackedMatMatPreRotFused(const HomEvaluator &eval, const CtxtTensor &a_in, std::vector<Ciphertext> &tmp, u64 T,
                                 MatrixTransformer &tr, u64 batch) {
    const Context &c = eval.getContext();
    tmp.clear();
    const i64 n = a_in.getHeight();
    if (a_in.getLevel() != T + 2 || a_in.get().getRescaleCounter() != 0)
        throw std::invalid_argument("[multPackedMatMatPreRot] operand must be at level " + std::to_string(T + 2) + ".");
    std::vector<Plaintext> &cm = tr.getColMaskExt(eval, a_in.getShape(), T + 2);
    Ciphertext first_ct(c);
    eval.levelDownOne(a_in.get(), first_ct);
    tmp.push_back(first_ct);
    std::vector<Shift> sa;
    for (i64 i = 1; i < n / 2; i++) sa.push_back(Shift{2 * i, &cm[(size_t)(4 * i + 1)], &cm[(size_t)(4 * i)]});
    if (sa.empty()) return;
    const u64 nq = T + 3, N = c->N, E = nq + c->nP, lo = nq - 1;
    const u64 *src = a_in.get().buf_.data();
    const Sources x = extendSources(c, src, 1, nq);
    const i64 back = -n;
    const DeviceBuffer a2 = rotateSources(eval, x, src, 1, &back);
    const Sources x2 = extendSources(c, a2.data(), 1, nq);
    const size_t G = std::max<u64>(1, std::min<u64>(2 * batch, (u64)sa.size()));
    DeviceBuffer y(c, G * 2 * E * N), t(c, G * 2 * lo * N), ws(c, G * 2 * lo * N);
    for (size_t first = 0; first < sa.size(); first += G) {
        const size_t cnt = std::min(G, sa.size() - first);
        std::vector<hemm_rot_term> terms;
        std::vector<uint32_t> off{0};
        pushShifts(eval, x, 0, x2, 0, sa, first, cnt, terms, off);
        ck(hemm_hoisted_moddown(c->dev, terms.data(), off.data(), (uint32_t)cnt, (uint32_t)nq, 1, 1, y.data(), t.data(), lo * N, ws.data(), nullptr));
        for (size_t q = 0; q < cnt; q++) {
            Ciphertext ct(c);
            ct.allocate(2, T + 1, 0);
            (void)hipMemcpyAsync(ct.buf_.data(), t.data() + q * 2 * lo * N, 2 * lo * N * 8, hipMemcpyDeviceToDevice, c->stream());
            tmp.push_back(std::move(ct));
        }
    }
}

void complexPackingPair(const HomEvaluator &eval, MatrixTransformer &tr, const Ciphertext &a, const Ciphertext &b, i64 w,
                        Ciphertext &pa, Ciphertext &pb, u64 pack_level) {
    const Context &c = eval.getContext();
    if (a.getRescaleCounter() != 0 || b.getRescaleCounter() != 0 || a.getNumPoly() != 2 || b.getNumPoly() != 2)
        throw std::invalid_argument("[complexPacking] operands must be rescaled.");
    // operands above pack_level are lowered first (both at once): the packing then runs on fewer limbs
    const u64 L = std::min<u64>(std::min(a.getLevel(), b.getLevel()), pack_level);
    const u64 N = c->N, ctw = 2 * (L + 1) * N, half = 2 * L * N;
    DeviceBuffer joint(c, 2 * ctw), packed(c, 2 * half);
    jointLevelDown(eval, a, b, L, joint.data());
    const bool by_rows[2] = {false, true};
    tr.complexPackingBatch(eval, joint.data(), 2, L, by_rows, w, packed.data());
    Ciphertext ra(c), rb(c);
    ra.allocate(2, L - 1, 0);
    rb.allocate(2, L - 1, 0);
    (void)hipMemcpyAsync(ra.buf_.data(), packed.data(), half * 8, hipMemcpyDeviceToDevice, c->stream());
    (void)hipMemcpyAsync(rb.buf_.data(), packed.data() + half, half * 8, hipMemcpyDeviceToDevice, c->stream());
    pa = std::move(ra);
    pb = std::move(rb);
}

CtxtTensor multMatMatComplexPackedFused(const HomEvaluator &eval, const Bootstrapper &btp, const CtxtTensor &a,
                                        const CtxtTensor &b, u64 T, MatrixTransformer &tr, u64 batch, bool single_tile,
                                        bool add_conj) {
    const Context &c = eval.getContext();
    c->mark("start");
    if (a.get().getRescaleCounter() != 0 || b.get().getRescaleCounter() != 0 || a.get().getNumPoly() != 2 ||
        b.get().getNumPoly() != 2)
        throw std::invalid_argument("[complexPacking] operands must be rescaled.");
    if (std::min(a.getLevel(), b.getLevel()) < T + 3)
        throw std::invalid_argument("[multMatMat] level >= " + std::to_string(T + 3) + " is needed.");
    {
        const i64 rows = a.getHeight(), cols = b.getWidth(), k = pow2ceil(commonInside(a, b)), w = commonBlockWidth(a, b);
        const u64 slots = c->N / 2, la = a.getLevel(), lb = b.getLevel();
        const bool spread = single_tile && (u64)(k * w) < slots && slots % (u64)(k * w) == 0;
        const bool bsgs = k / 2 > 1 && ((u64)(k * w) == slots || spread);
        // Exact row rotations (B's tile fills the slot vector or is spread over it) on square tiles: the product needs
        // sigma(A') at T+2 but tau(B') at T+1, and the two operands go their own ways there on two streams -- B on the
        // side stream, where the baby rotations follow its transform, A on the context's, where only its copy for the
        // unshifted term is lowered; the chains meet in front of the main loop.  Operands above the level their way
        // starts from are only truncated to it (the first masks on the way carry the change of scale).  The ways:
        //   * separate packing (A >= T+5, B >= T+4): packed at T+5 / T+4, then the two-stage transform -- three launch
        //     chains of few terms each;
        //   * packing and the first transform stage as one composite map (MatrixTransformer::packingStageOne), then the
        //     second stage: two chains, the first with about twice the terms -- for an A at T+4 and a B at T+3, which
        //     have a level less than the separate packing needs;
        //   * an A at T+3 has one level for packing and sigma together: the composite one-stage transform.
        // (k / 2 >= 4: every transform stage then has rotations; a stage without any rescales through the context's
        // scratch region, which only one of the two chains may use)
        if (bsgs && k / 2 >= 4 && rows == k && cols == k && std::min(la, lb) >= 4 + btp.getMinLevelForBootstrap()) {
            const bool separate = la >= T + 5 && lb >= T + 4;
            const u64 N = c->N, lo = T + 2;
            const TileTensorShape shape_a(rows, k, w), shape_b(k, cols, w);
            std::vector<Plaintext> &cm = tr.getColMaskExt(eval, shape_a, T + 2);
            DeviceBuffer sa(c, 2 * (T + 3) * N), tb(c, 2 * lo * N);
            const std::vector<u64> one(T + 6, 1);
            // the first L + 1 limbs of both polynomials of x, back to back
            auto truncated = [&](const Ciphertext &x, u64 L) {
                DeviceBuffer t(c, 2 * (L + 1) * N);
                ck(hemm_mul_scalar(c->dev, x.buf_.data(), x.polyStride(), one.data(), t.data(), (L + 1) * N, (uint32_t)(L + 1), 0,
                                   2, nullptr));
                return t;
            };
            OwnWays ways(c);
            ways.toSide();
            {
                const MaskKind kind = MaskKind::PackedVertical;
                if (separate) {   // truncated to T+4, packed by rows (T+3), tau in two stages (T+1)
                    const u64 Lb = T + 4;
                    const DeviceBuffer jb = truncated(b.get(), Lb);
                    DeviceBuffer pk(c, 2 * Lb * N);
                    const bool by_rows = true;
                    tr.complexPackingBatch(eval, jb.data(), 1, Lb, &by_rows, w, pk.data(), &lb);
                    tr.diagonalTransformTwoStage(eval, pk.data(), 1, Lb - 1, &kind, &shape_b, tb.data());
                } else {          // truncated to T+3, packing + first stage (T+2), second stage (T+1)
                    const u64 Lb = T + 3;
                    const DeviceBuffer jb = truncated(b.get(), Lb);
                    DeviceBuffer mid(c, 2 * Lb * N);
                    tr.packingStageOne(eval, jb.data(), 1, Lb, &kind, &shape_b, mid.data(), &lb);
                    tr.diagonalTransformTwoStage(eval, mid.data(), 1, Lb, &kind, &shape_b, tb.data(), nullptr, 2);
                }
            }
            ways.toOwn();
            if (separate) {       // truncated to T+5, packed by columns (T+4), sigma in two stages (T+2)
                const u64 La = T + 5;
                const DeviceBuffer ja = truncated(a.get(), La);
                DeviceBuffer pk(c, 2 * La * N);
                const bool by_rows = false;
                const MaskKind kind = MaskKind::PackedHorizontal;
                tr.complexPackingBatch(eval, ja.data(), 1, La, &by_rows, w, pk.data(), &la);
                tr.diagonalTransformTwoStage(eval, pk.data(), 1, La - 1, &kind, &shape_a, sa.data());
            } else if (la >= T + 4) {   // truncated to T+4, packing + first stage (T+3), second stage (T+2)
                const u64 La = T + 4;
                const DeviceBuffer ja = truncated(a.get(), La);
                DeviceBuffer mid(c, 2 * La * N);
                const MaskKind kind = MaskKind::PackedHorizontal;
                tr.packingStageOne(eval, ja.data(), 1, La, &kind, &shape_a, mid.data(), &la);
                tr.diagonalTransformTwoStage(eval, mid.data(), 1, La, &kind, &shape_a, sa.data(), nullptr, 2);
            } else {              // at T+3: packing and sigma as one composite one-stage transform (T+2)
                const MaskKind kind = MaskKind::PackingHorizontal;
                tr.diagonalTransformBatch(eval, a.get().buf_.data(), 1, T + 3, &kind, &shape_a, sa.data());
            }
            ways.marksOn();
            c->mark("packing and transforms of A");
            return ownWaysShiftProduct(eval, T, sa.data(), tb.data(), cm, rows, cols, k, w, batch, spread,
                                       ways.side(), add_conj);
        }
    }
    // one level short of a separate packing: the packing and the packed transform as one composite transform from T+3
    if (std::min(a.getLevel(), b.getLevel()) == T + 3)
        return ccmmFused(eval, btp, a, b, T, tr, batch, single_tile, true, nullptr, 0, true, add_conj);
    // pack at T+5 when the operands allow it, so that the transforms keep their two stages from T+4; the packed pair
    // is handed to the product where it lies.  Operands above the packing level are only truncated to it (a copy of
    // their first L+1 limbs): the packing masks absorb the change of scale, which saves the levelDown.
    const u64 L = std::min<u64>(std::min(a.getLevel(), b.getLevel()), T + 5);
    const u64 N = c->N, ctw = 2 * (L + 1) * N;
    DeviceBuffer joint(c, 2 * ctw), packed(c, 2 * 2 * L * N);
    const std::vector<u64> one(L + 1, 1);
    const Ciphertext *ops[2] = {&a.get(), &b.get()};
    for (int q = 0; q < 2; q++)
        ck(hemm_mul_scalar(c->dev, ops[q]->buf_.data(), ops[q]->polyStride(), one.data(), joint.data() + q * ctw, (L + 1) * N,
                           (uint32_t)(L + 1), 0, 2, nullptr));
    const bool by_rows[2] = {false, true};
    const u64 from[2] = {a.getLevel(), b.getLevel()};
    if (L == T + 4 && a.getHeight() == a.getWidth() && b.getHeight() == b.getWidth() && a.getHeight() == b.getHeight() &&
        pow2ceil(commonInside(a, b)) / 2 >= 4) {
        // a level short of a separate packing in front of two-stage transforms: the packing and the first stage as one
        // composite map for both operands (T+4 -> T+3); the product runs the second stage
        const MaskKind kinds[2] = {MaskKind::PackedHorizontal, MaskKind::PackedVertical};
        const i64 k = pow2ceil(commonInside(a, b)), w = commonBlockWidth(a, b);
        const TileTensorShape shapes[2] = {TileTensorShape(a.getHeight(), k, w), TileTensorShape(k, b.getWidth(), w)};
        tr.packingStageOne(eval, joint.data(), 2, L, kinds, shapes, packed.data(), from);
        return ccmmFused(eval, btp, a, b, T, tr, batch, single_tile, true, packed.data(), L - 1, false, add_conj, 2);
    }
    tr.complexPackingBatch(eval, joint.data(), 2, L, by_rows, a.getBlockWidth(), packed.data(), from);
    c->mark("complex packing");
    return ccmmFused(eval, btp, a, b, T, tr, batch, single_tile, true, packed.data(), L - 1, false, add_conj);
}

namespace {
// stages (rotations per stage, multiplier of the unit): one stage up to four terms, else i = i0 + b i1 with
// b = 2^ceil(log2(count) / 2)
std::vector<std::pair<u64, u64>> rotateSumStages(u64 count) {
    if (count == 0 || (count & (count - 1)) != 0) throw std::invalid_argument("[rotateSum] the count must be a power of two");
    if (count <= 4) return {{count, 1}};
    u64 b = 1;
    while (b * b < count) b <<= 1;
    return {{b, 1}, {count / b, b}};
}
}  // namespace

std::vector<u64> rotateSumRotations(i64 unit, u64 count, u64 log_slots) {
    const i64 slots = i64(1) << log_slots;
    std::vector<u64> r;
    for (const auto &st : rotateSumStages(count))
        for (u64 i = 1; i < st.first; i++) {
            const u64 v = (u64)((((i64)(i * st.second) * unit) % slots + slots) % slots);
            if (v != 0) r.push_back(v);
        }
    return r;
}

void rotateSumFused(const HomEvaluator &eval, const std::vector<RotateSumJob> &jobs, u64 count) {
    if (jobs.empty()) return;
    const Context &c = eval.getContext();
    const KeyPack &pack = eval.getKeyPack();
    const Rot rot(c);
    const size_t n = jobs.size();
    const u64 level = jobs[0].in->getLevel(), rc = jobs[0].in->getRescaleCounter();
    const u64 nq = level + 1, N = c->N, E = nq + c->nP, ctw = 2 * nq * N;
    for (const RotateSumJob &j : jobs)
        if (j.in == nullptr || j.out == nullptr || j.in->getNumPoly() != 2 || j.in->getLevel() != level ||
            j.in->getRescaleCounter() != rc)
            throw std::invalid_argument("[rotateSum] the operands must share one level and have two polynomials.");
    const auto stages = rotateSumStages(count);
    DeviceBuffer cur(c, n * ctw), nxt(c, n * ctw);
    for (size_t q = 0; q < n; q++)
        for (u64 p = 0; p < 2; p++)
            (void)hipMemcpyAsync(cur.data() + q * ctw + p * nq * N, jobs[q].in->buf_.data() + p * jobs[q].in->polyStride(),
                                 nq * N * 8, hipMemcpyDeviceToDevice, c->stream());
    for (const auto &st : stages) {
        if (st.first <= 1) continue;
        // raw b polynomials: the launch multiplies them by P itself (one launch less than premultiplied sources)
        const Sources x = extendSources(c, cur.data(), n, nq, nullptr, false);
        std::vector<hemm_rot_term> terms;
        std::vector<uint32_t> off{0};
        for (size_t q = 0; q < n; q++) {
            const u64 *b = cur.data() + q * ctw, *a = b + nq * N;
            for (u64 i = 1; i < st.first; i++) {
                const i64 amount = (i64)(i * st.second) * jobs[q].unit;
                if (rot.norm(amount) == 0)   // a whole turn: the input itself once more
                    terms.push_back(keylessTerm(b, a, nullptr));
                else
                    terms.push_back(term(x.extOf(q), x.pbOf(q), pack, rot.galois(amount), nullptr));
            }
            terms.push_back(keylessTerm(b, a, nullptr));   // i = 0: no key switch
            off.push_back((uint32_t)terms.size());
        }
        DeviceBuffer y(c, n * 2 * E * N), ws(c, n * ctw);
        ck(hemm_hoisted_moddown(c->dev, terms.data(), off.data(), (uint32_t)n, (uint32_t)nq, x.premultiplied(), 0, y.data(),
                                nxt.data(), nq * N, ws.data(), nullptr));
        std::swap(cur, nxt);
    }
    for (size_t q = 0; q < n; q++) {
        Ciphertext res(c);
        res.allocate(2, level, rc);
        (void)hipMemcpyAsync(res.buf_.data(), cur.data() + q * ctw, ctw * 8, hipMemcpyDeviceToDevice, c->stream());
        *jobs[q].out = std::move(res);   // (occupied slots: unknown, as allocate leaves them)
    }
}

// Ciphertext x ciphertext re-use product: sum_k tmp[k] (x) rho^(k step)(b) with tmp from multMatMatPre(Fused) and
// b = tau(B).  The reference rotates b by `step` in a chain, one key switch after the other; here every rotation
// comes from the same ModUp of b through its direct key (hoisted), 2 * batch rotations per launch chain with one
// plain ModDown for all of them.  The accumulator stays un-relinearised until the end.
CtxtTensor multMatMatCCReUseFused(const HomEvaluator &eval, const std::vector<Ciphertext> &tmp, const CtxtTensor &b,
                                  u64 step, bool rescale_after, u64 batch) {
    const Context &c = eval.getContext();
    if (tmp.empty()) throw std::invalid_argument("[multMatMatCCReUse] no shifted operands.");
    const u64 level = b.getLevel(), nq = level + 1, N = c->N, E = nq + c->nP, ctw = 2 * nq * N;
    for (const Ciphertext &t : tmp)
        if (t.getLevel() != level || t.getNumPoly() != 2 || t.getRescaleCounter() != b.get().getRescaleCounter())
            throw std::invalid_argument("[multMatMatCCReUse] operands must share one level.");
    const KeyPack &pack = eval.getKeyPack();
    const Rot rot(c);
    Ciphertext acc(c);
    acc.allocate(3, level, b.get().getRescaleCounter() + 1);
    ck(hemm_tensor_batch(c->dev, tmp[0].buf_.data(), b.get().buf_.data(), 1, (uint32_t)nq, acc.buf_.data(), 0, nullptr));
    const size_t n_rot = tmp.size() - 1;
    if (n_rot > 0) {
        const Sources xb = extendSources(c, b.get().buf_.data(), 1, nq);
        const size_t G = std::max<u64>(1, std::min<u64>(2 * batch, (u64)n_rot));
        DeviceBuffer y(c, G * 2 * E * N), rb(c, G * ctw), ws(c, G * ctw);
        for (size_t first = 0; first < n_rot; first += G) {
            const size_t cnt = std::min(G, n_rot - first);
            std::vector<hemm_rot_term> terms;
            std::vector<uint32_t> off{0};
            for (size_t q = 0; q < cnt; q++) {
                const i64 amount = (i64)((first + q + 1) * step);
                if (rot.norm(amount) == 0) throw std::invalid_argument("[multMatMatCCReUse] rotation by a whole turn.");
                terms.push_back(term(xb.extOf(0), xb.pbOf(0), pack, rot.galois(amount), nullptr));
                off.push_back((uint32_t)terms.size());
            }
            ck(hemm_hoisted_moddown(c->dev, terms.data(), off.data(), (uint32_t)cnt, (uint32_t)nq, 1, 0, y.data(), rb.data(),
                                    nq * N, ws.data(), nullptr));
            for (size_t q = 0; q < cnt; q++)
                ck(hemm_tensor_batch(c->dev, tmp[first + q + 1].buf_.data(), rb.data() + q * ctw, 1, (uint32_t)nq,
                                     acc.buf_.data(), 1, nullptr));
        }
    }
    CtxtTensor res(c, b.getHeight(), b.getWidth(), b.getBlockWidth());
    eval.relinearize(acc, res.get());
    if (rescale_after) eval.rescale(res.get());
    return res;
}

// Plaintext x ciphertext product with ONE ModDown.  Every column shift of sigma(A) stays in the extended basis; there
// it is multiplied by its column mask and by tau(B) rotated k w slots -- tau(B) is a plaintext over the extended basis
// that the hoisted kernel reads through the term's second automorphism, so the n rotated weights are never
// materialised -- and all shifts are summed.  The unshifted term P (mask_0 tau(B)) sigma(A) joins on the chain limbs,
// the sum is divided by P q_{T+2} (ModDown merged with the first rescale) and rescaled once more:
//     rescale(ModDown(sum_k [mask_k tau(B)_k] (.) KS_k(sigma A))).
// n - 1 key products, but 1 ModDown instead of n - 1 and no ciphertext ever leaves the extended basis in between.
// A row shift of tau(B) is a whole rotation when every tile block of the plaintext (rows * block width slots each)
// is the same.  The plaintext is known to the host, so the layouts are told apart there:
//   * one tile block fills the slot vector (pair layout), or all blocks are equal: as written above;
//   * only the first block is non-zero (HEMMer::encode of a single matrix): tau(B) is copied into every block
//     and the column-shift masks are restricted to the first block, so the product stays empty elsewhere
//     whatever the ciphertext carries there;
//   * anything else (different matrices stacked in one plaintext) returns false: the caller takes the
//     reference-order product.
// tau(B) is prepared once per weight (decode, permute, encode on the host as MatrixTransformer::diagonalToRow<Plaintext>
// does) and kept under a hash of the weight's residues.
namespace {
// two independent 64-bit digests of a plaintext's content (together a 128-bit key: an accidental collision between
// two weights is out of reach)
std::pair<u64, u64> hashResidues(const Context &c, const Plaintext &pt) {
    // limb 0 determines the plaintext (its coefficients are far below q_0 / 2)
    std::vector<u64> h(c->N);
    if (hipMemcpy(h.data(), pt.buf_.data(), h.size() * 8, hipMemcpyDeviceToHost) != hipSuccess)
        throw RuntimeException("hipMemcpy");
    u64 x = 0xcbf29ce484222325ull ^ pt.getLevel(), y = 0x9e3779b97f4a7c15ull + pt.getLevel();
    for (u64 v : h) {
        x ^= v;
        x *= 0x100000001b3ull;
        x ^= x >> 29;
        y = (y ^ (v + 0x632be59bd9b4e019ull)) * 0xff51afd7ed558ccdull;   // another multiplier, another mixing shift
        y ^= y >> 32;
    }
    return {x, y};
}
}  // namespace

bool multMatMatPlainFused(const HomEvaluator &eval, const Bootstrapper &btp, const CtxtTensor &op1, const PtxtTensor &op2,
                          u64 T, MatrixTransformer &tr, u64 batch, CtxtTensor &res_out) {
    const Context &c = eval.getContext();
    (void)batch;
    const i64 rows = op1.getHeight(), cols = op2.getWidth();
    const i64 k = pow2ceil(commonInside(op1, op2)), w = commonBlockWidth(op1, op2);
    if (std::min(op1.getLevel(), op2.getLevel()) < 1 + btp.getMinLevelForBootstrap())
        throw std::invalid_argument("[multMatMat] level >= " + std::to_string(1 + btp.getMinLevelForBootstrap()) +
                                    " is needed.");
    const i64 slots = (i64)(c->N / 2), block = k * w;
    if (block > slots || slots % block != 0) return false;
    if (op1.getLevel() < T + 3)
        throw std::invalid_argument("[multMatMat] level >= " + std::to_string(T + 3) + " is needed.");
    const TileTensorShape shape_a(rows, k, w), shape_b(k, cols, w);
    // ---- tau(B) over the extended basis at level T+2, scaled like a plaintext of level T+1
    // the hash needs a device-to-host copy and with it a drained queue: taken once per plaintext object
    const Plaintext &weight = op2.get();
    std::pair<u64, u64> weight_hash;
    if (weight.hash_state_ == 1) {
        weight_hash = {weight.content_hash_, weight.content_hash2_};
    } else {
        weight_hash = hashResidues(c, weight);
        if (weight.hash_state_ == 0) {
            weight.content_hash_ = weight_hash.first;
            weight.content_hash2_ = weight_hash.second;
            weight.hash_state_ = 1;
        }
    }
    tr.useChainOf(c);
    const auto key = std::make_tuple(weight_hash.first, weight_hash.second, shape_b, T);
    auto it = tr.weight_tau_.find(key);
    if (it == tr.weight_tau_.end()) {
        EnDecoder endec(c);
        const Message src = endec.decode(op2.get());
        // decoded values carry the encoding's rounding noise (about sqrt(N) / 2^43 at this scale): "zero" and "equal"
        // are taken up to 2^-24
        const double tol = std::ldexp(1.0, -24);
        bool rest_zero = true, rest_equal = true;
        for (i64 j = block; j < slots && (rest_zero || rest_equal); j++) {
            if (std::abs(src[(u64)j]) >= tol) rest_zero = false;
            if (std::abs(src[(u64)j] - src[(u64)(j % block)]) >= tol) rest_equal = false;
        }
        MatrixTransformer::WeightTau entry{Plaintext(c), 0};
        if (rest_zero || rest_equal) {
            const bool first_only = rest_zero && block < slots;
            Message dst(src.getLogSlots(), 0);
            const i64 height = slots / w;
            for (i64 r = 0; r < height; r++)
                for (i64 cc = 0; cc < w; cc++) {
                    const i64 cb = cc - cc % k, i = r % k, j = cc % k;
                    const i64 rb = first_only ? 0 : r - r % k;   // single matrix: every block takes the first one's tau
                    dst[(u64)(r * w + cc)] = src[(u64)((rb + (i + j) % k) * w + cb + j)];
                }
            entry.tau = endec.encodeExtended(dst, T + 2, c->delta[T + 1]);
            entry.layout = first_only ? 2 : 1;
        }
        if (tr.weight_tau_order_.size() >= 256) {   // bounded: the oldest weight is prepared again if it comes back
            tr.weight_tau_.erase(tr.weight_tau_order_.front());
            tr.weight_tau_order_.erase(tr.weight_tau_order_.begin());
        }
        tr.weight_tau_order_.push_back(key);
        it = tr.weight_tau_.emplace(key, std::move(entry)).first;
    }
    if (it->second.layout == 0) return false;
    const bool first_block_only = it->second.layout == 2;
    const Plaintext &tau = it->second.tau;
    std::vector<Plaintext> &cm = tr.getColMaskExt(eval, shape_a, T + 2, first_block_only);
    // ---- sigma(A) at level T+2 and its two rotation sources
    const u64 nq = T + 3, N = c->N, K = c->nP, E = nq + K, lo = nq - 1;
    Ciphertext own_a(c);
    const Ciphertext *pa = &op1.get();
    if (pa->getLevel() < 4 + btp.getMinLevelForBootstrap()) {
        own_a = *pa;
        btp.bootstrapExtended(own_a, own_a);
        pa = &own_a;
    }
    const Ciphertext sa = tr.lowerAndTransformFused(eval, *pa, MaskKind::Horizontal, shape_a, T + 2);
    const Sources x = extendSources(c, sa.buf_.data(), 1, nq);
    const i64 back = -k;
    const DeviceBuffer a2 = rotateSources(eval, x, sa.buf_.data(), 1, &back);
    const Sources x2 = extendSources(c, a2.data(), 1, nq);
    // ---- all shifts as terms of one sum, dealt to `parts` partial outputs
    const KeyPack &pack = eval.getKeyPack();
    const Rot rot(c);
    const u64 n_shift = (u64)(k - 1);
    const u64 parts = std::max<u64>(1, std::min<u64>(16, n_shift));
    DeviceBuffer y(c, 2 * E * N);
    if (n_shift > 0) {
        std::vector<hemm_rot_term> terms;
        std::vector<uint32_t> off{0};
        for (u64 p = 0; p < parts; p++) {
            for (u64 i = 1 + p * n_shift / parts; i < 1 + (p + 1) * n_shift / parts; i++) {
                const u64 g = rot.galois((i64)i), gp = rot.galois((i64)i * w);
                hemm_rot_term t1 = term(x.extOf(0), x.pbOf(0), pack, g, &cm[(size_t)(2 * i + 1)]);
                hemm_rot_term t2 = term(x2.extOf(0), x2.pbOf(0), pack, g, &cm[(size_t)(2 * i)]);
                t1.pt = t2.pt = tau.buf_.data();
                t1.pt_galois = t2.pt_galois = (uint32_t)gp;
                terms.push_back(t1);
                terms.push_back(t2);
            }
            if (p == 0) {   // shift 0 needs no key switch: P (mask_0 tau(B)) sigma(A) on the chain limbs
                hemm_rot_term t0 = keylessTerm(x.pbOf(0), sa.buf_.data() + nq * N, &cm[1]);
                t0.pt = tau.buf_.data();
                terms.push_back(t0);
            }
            off.push_back((uint32_t)terms.size());
        }
        DeviceBuffer yp(c, parts * 2 * E * N);
        ck(hemm_hoisted_terms(c->dev, terms.data(), off.data(), (uint32_t)parts, (uint32_t)nq, yp.data(), 1, nullptr));
        ck(hemm_sum_parts(c->dev, yp.data(), (uint32_t)parts, 1, (uint32_t)nq, y.data(), nullptr));
    } else {
        ck(hemm_zero(c->dev, y.data(), 2 * E * N, nullptr));
        // ---- no shift at all: P (mask_0 tau(B)) sigma(A) on the chain limbs
        DeviceBuffer m0(c, nq * N), t0(c, 2 * nq * N);
        ck(hemm_pointwise(c->dev, HEMM_MUL, cm[1].buf_.data(), 0, tau.buf_.data(), 0, m0.data(), 0, (uint32_t)nq, 0, 1, nullptr));
        ck(hemm_pointwise(c->dev, HEMM_MUL, sa.buf_.data(), nq * N, m0.data(), 0, t0.data(), nq * N, (uint32_t)nq, 0, 2, nullptr));
        std::vector<u64> sc(nq);
        for (u64 j = 0; j < nq; j++) {
            u64 P = 1;
            for (u64 p : c->p) P = (u64)((u128)P * (p % c->q[j]) % c->q[j]);
            sc[j] = P;
        }
        ck(hemm_mul_scalar(c->dev, t0.data(), nq * N, sc.data(), t0.data(), nq * N, (uint32_t)nq, 0, 2, nullptr));
        ck(hemm_pointwise(c->dev, HEMM_ADD, y.data(), E * N, t0.data(), nq * N, y.data(), E * N, (uint32_t)nq, 0, 2, nullptr));
    }
    // ---- one ModDown merged with the first rescale, then the second rescale
    DeviceBuffer mid(c, 2 * lo * N), ws(c, 2 * lo * N);
    ck(hemm_moddown_batch(c->dev, y.data(), (uint32_t)nq, 2, 1, mid.data(), lo * N, ws.data(), nullptr));
    CtxtTensor res(c, rows, cols, w);
    res.get().allocate(2, T, 0);
    ck(hemm_rescale(c->dev, mid.data(), lo * N, res.get().buf_.data(), (lo - 1) * N, (uint32_t)lo, 2, nullptr));
    res_out = res;
    return true;
}

}  // namespace HELLM

// HomEvaluator: level / scale bookkeeping on the host, arithmetic through the C ABI.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>

#include "../../../include/hemm.h"
#include "HEaaN/HEaaN.hpp"
#include "context_content.hpp"

namespace HEaaN {

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
// residues of a (possibly negative) integer for the first nq chain primes
std::vector<u64> int_residues(const Context &c, i64 v, u64 nq) {
    std::vector<u64> r(nq);
    for (u64 j = 0; j < nq; j++) {
        const u64 q = c->q[j];
        if (v >= 0)
            r[j] = (u64)v % q;
        else {
            u64 m = (u64)(-v) % q;
            r[j] = m ? q - m : 0;
        }
    }
    return r;
}
void require_rc0(const Ciphertext &a, const char *what) {
    if (a.getRescaleCounter() != 0) throw RuntimeException(std::string(what) + ": operand must be rescaled first");
}
}  // namespace

// out gets shape (polys, level); reuses out's buffer when the shape already matches (element-wise
// kernels tolerate aliasing), otherwise a fresh buffer replaces it after the kernel has been queued.
struct OutSlot {
    Ciphertext tmp;
    Ciphertext *dst;
    bool direct;
    OutSlot(const Context &c, Ciphertext &out, u64 polys, u64 level, u64 rc, bool allow_inplace,
            std::initializer_list<const Ciphertext *> inputs)
        : tmp(c), dst(&out) {
        bool aliases = false;
        for (auto *p : inputs) aliases |= (p == &out);
        direct = (!aliases || allow_inplace) && out.num_poly_ == polys && out.level_ == level && out.buf_.data();
        if (!direct && !aliases) {
            out.allocate(polys, level, rc);
            direct = true;
        }
        if (direct)
            out.rescale_counter_ = rc;
        else
            tmp.allocate(polys, level, rc);
    }
    Ciphertext &get() { return direct ? *dst : tmp; }
    // the result's known-empty slot range is `occupied` (all ones: nothing known); operations that are not
    // slot-wise leave the default
    void commit(u64 occupied = ~u64(0)) {
        if (!direct) *dst = std::move(tmp);
        dst->occupied_ = occupied;
    }
};

void HomEvaluator::negate(const Ciphertext &a, Ciphertext &out) const {
    const u64 occ = a.occupied_;
    OutSlot o(ctx_, out, a.num_poly_, a.level_, a.rescale_counter_, true, {&a});
    ck(hemm_pointwise(ctx_->dev, HEMM_NEG, a.buf_.data(), a.polyStride(), nullptr, 0, o.get().buf_.data(),
                      o.get().polyStride(), (uint32_t)a.level_ + 1, 0, (uint32_t)a.num_poly_, nullptr));
    o.commit(occ);
}

static void add_sub(const HomEvaluator &ev, const Context &c, int op, const Ciphertext &a0, const Ciphertext &b0,
                    Ciphertext &out) {
    if (a0.rescale_counter_ != b0.rescale_counter_)
        throw RuntimeException("add/sub: operands have different rescale counters");
    // operands at different levels: bring the higher one down to the lower level's scale first
    const Ciphertext *a = &a0, *b = &b0;
    Ciphertext la(c), lb(c);
    if (a0.level_ > b0.level_) {
        ev.levelDown(a0, b0.level_, la);
        a = &la;
    } else if (b0.level_ > a0.level_) {
        ev.levelDown(b0, a0.level_, lb);
        b = &lb;
    }
    const u64 polys = std::max(a->num_poly_, b->num_poly_), common = std::min(a->num_poly_, b->num_poly_);
    const u64 occ = std::max(a0.occupied_, b0.occupied_);
    OutSlot o(c, out, polys, a->level_, a->rescale_counter_, true, {&a0, &b0});
    Ciphertext &r = o.get();
    ck(hemm_pointwise(c->dev, op, a->buf_.data(), a->polyStride(), b->buf_.data(), b->polyStride(), r.buf_.data(),
                      r.polyStride(), (uint32_t)a->level_ + 1, 0, (uint32_t)common, nullptr));
    if (polys > common) {  // 3-poly +/- 2-poly: the third polynomial passes through (negated for 2 - 3)
        const Ciphertext *big = a->num_poly_ > b->num_poly_ ? a : b;
        const bool neg = (op == HEMM_SUB && big == b);
        const u64 *src = big->buf_.data() + 2 * big->polyStride();
        u64 *dst = r.buf_.data() + 2 * r.polyStride();
        if (neg)
            ck(hemm_pointwise(c->dev, HEMM_NEG, src, 0, nullptr, 0, dst, 0, (uint32_t)a->level_ + 1, 0, 1, nullptr));
        else if (src != dst)
            (void)hipMemcpyAsync(dst, src, r.polyStride() * 8, hipMemcpyDeviceToDevice, c->stream());
    }
    o.commit(occ);
}
void HomEvaluator::add(const Ciphertext &a, const Ciphertext &b, Ciphertext &out) const {
    add_sub(*this, ctx_, HEMM_ADD, a, b, out);
}
void HomEvaluator::sub(const Ciphertext &a, const Ciphertext &b, Ciphertext &out) const {
    add_sub(*this, ctx_, HEMM_SUB, a, b, out);
}
void HomEvaluator::add(const Ciphertext &a, const Plaintext &b, Ciphertext &out) const {
    if (b.level_ < a.level_) throw RuntimeException("add(ct, pt): plaintext level below the ciphertext level");
    const u64 occ = std::max(a.occupied_, b.occupied_);
    OutSlot o(ctx_, out, a.num_poly_, a.level_, a.rescale_counter_, true, {&a});
    Ciphertext &r = o.get();
    if (r.buf_.data() != a.buf_.data())
        (void)hipMemcpyAsync(r.buf_.data(), a.buf_.data(), a.buf_.words() * 8, hipMemcpyDeviceToDevice, ctx_->stream());
    ck(hemm_pointwise(ctx_->dev, HEMM_ADD, r.buf_.data(), 0, b.buf_.data(), 0, r.buf_.data(), 0,
                      (uint32_t)a.level_ + 1, 0, 1, nullptr));
    o.commit(occ);
}
void HomEvaluator::add(const Ciphertext &a, const Message &b, Ciphertext &out) const {
    add(a, EnDecoder(ctx_).encode(b, a.level_), out);
}
void HomEvaluator::add(const Ciphertext &a, const Complex &cst, Ciphertext &out) const {
    if (ctx_->N < 512) {
        Message m(getLogFullSlots(ctx_), cst);
        add(a, m, out);
        return;
    }
    // a constant in every slot is the polynomial round(re Delta) + round(im Delta) X^(N/2): added to the residues of
    // the first polynomial directly, no plaintext is encoded
    const Real delta = ctx_->delta[a.level_];
    const i64 re = (i64)llround(cst.real() * delta), im = (i64)llround(cst.imag() * delta);
    const u64 occ = (re != 0 || im != 0) ? (u64)ctx_->N / 2 : a.occupied_;
    OutSlot o(ctx_, out, a.num_poly_, a.level_, a.rescale_counter_, true, {&a});
    Ciphertext &r = o.get();
    if (r.buf_.data() != a.buf_.data())
        (void)hipMemcpyAsync(r.buf_.data(), a.buf_.data(), a.buf_.words() * 8, hipMemcpyDeviceToDevice, ctx_->stream());
    const auto rr = int_residues(ctx_, re, a.level_ + 1), ri = int_residues(ctx_, im, a.level_ + 1);
    ck(hemm_add_scalar(ctx_->dev, r.buf_.data(), rr.data(), im != 0 ? ri.data() : nullptr, r.buf_.data(),
                       (uint32_t)a.level_ + 1, 0, nullptr));
    o.commit(occ);
}
void HomEvaluator::sub(const Ciphertext &a, const Message &b, Ciphertext &out) const {
    Message nb(b);
    for (auto &z : nb) z = -z;
    add(a, nb, out);
}
void HomEvaluator::add(const Plaintext &a, const Plaintext &b, Plaintext &out) const {
    const u64 lvl = std::min(a.level_, b.level_);
    Plaintext r(ctx_);
    r.allocate(lvl, a.rescale_counter_);
    ck(hemm_pointwise(ctx_->dev, HEMM_ADD, a.buf_.data(), 0, b.buf_.data(), 0, r.buf_.data(), 0, (uint32_t)lvl + 1, 0,
                      1, nullptr));
    out = std::move(r);
}

void HomEvaluator::multWithoutRescale(const Ciphertext &a, const Plaintext &b, Ciphertext &out) const {
    require_rc0(a, "multWithoutRescale");
    if (b.level_ < a.level_) throw RuntimeException("mult(ct, pt): plaintext level below the ciphertext level");
    const u64 occ = std::min(a.occupied_, b.occupied_);   // a product is empty where either factor is
    OutSlot o(ctx_, out, a.num_poly_, a.level_, 1, true, {&a});
    ck(hemm_pointwise(ctx_->dev, HEMM_MUL, a.buf_.data(), a.polyStride(), b.buf_.data(), 0, o.get().buf_.data(),
                      o.get().polyStride(), (uint32_t)a.level_ + 1, 0, (uint32_t)a.num_poly_, nullptr));
    o.commit(occ);
}
void HomEvaluator::mult(const Ciphertext &a, const Plaintext &b, Ciphertext &out) const {
    multWithoutRescale(a, b, out);
    rescale(out);
}
void HomEvaluator::mult(const Ciphertext &a, const Message &b, Ciphertext &out) const {
    mult(a, EnDecoder(ctx_).encode(b, a.level_), out);
}
void HomEvaluator::maskedSum(const Ciphertext &a, const Plaintext &ma, const Ciphertext &b, const Plaintext &mb,
                             Ciphertext &out) const {
    require_rc0(a, "maskedSum");
    require_rc0(b, "maskedSum");
    if (a.level_ != b.level_ || ma.level_ < a.level_ || mb.level_ < a.level_)
        throw RuntimeException("maskedSum: level mismatch");
    OutSlot o(ctx_, out, 2, a.level_, 1, false, {&a, &b});
    Ciphertext &r = o.get();
    ck(hemm_pointwise(ctx_->dev, HEMM_MUL, a.buf_.data(), a.polyStride(), ma.buf_.data(), 0, r.buf_.data(),
                      r.polyStride(), (uint32_t)a.level_ + 1, 0, 2, nullptr));
    ck(hemm_pointwise(ctx_->dev, HEMM_MAC, b.buf_.data(), b.polyStride(), mb.buf_.data(), 0, r.buf_.data(),
                      r.polyStride(), (uint32_t)a.level_ + 1, 0, 2, nullptr));
    o.commit();
}

void HomEvaluator::multInteger(const Ciphertext &a, i64 v, Ciphertext &out) const {
    const u64 occ = a.occupied_;
    OutSlot o(ctx_, out, a.num_poly_, a.level_, a.rescale_counter_, true, {&a});
    auto sc = int_residues(ctx_, v, a.level_ + 1);
    ck(hemm_mul_scalar(ctx_->dev, a.buf_.data(), a.polyStride(), sc.data(), o.get().buf_.data(), o.get().polyStride(),
                       (uint32_t)a.level_ + 1, 0, (uint32_t)a.num_poly_, nullptr));
    o.commit(occ);
}
void HomEvaluator::multImagUnit(const Ciphertext &a, Ciphertext &out) const {
    const u64 occ = a.occupied_;
    OutSlot o(ctx_, out, a.num_poly_, a.level_, a.rescale_counter_, true, {&a});
    ck(hemm_mul_imag_unit(ctx_->dev, a.buf_.data(), a.polyStride(), o.get().buf_.data(), o.get().polyStride(),
                          (uint32_t)a.level_ + 1, (uint32_t)a.num_poly_, nullptr));
    o.commit(occ);
}
void HomEvaluator::multWithoutRescale(const Ciphertext &a, const Complex &cst, Ciphertext &out) const {
    require_rc0(a, "multWithoutRescale");
    const Real delta = ctx_->delta[a.level_];
    const i64 re = (i64)llround(cst.real() * delta), im = (i64)llround(cst.imag() * delta);
    Ciphertext r(ctx_);
    multInteger(a, re, r);
    if (im != 0) {
        Ciphertext t(ctx_);
        multImagUnit(a, t);
        multInteger(t, im, t);
        add(r, t, r);
    }
    r.rescale_counter_ = 1;
    out = std::move(r);
}
void HomEvaluator::mult(const Ciphertext &a, const Complex &cst, Ciphertext &out) const {
    // constants within 1e-8 of a Gaussian integer do not consume a level
    const Real rr = std::round(cst.real()), ri = std::round(cst.imag());
    if (std::fabs(cst.real() - rr) <= 1e-8 && std::fabs(cst.imag() - ri) <= 1e-8) {
        Ciphertext r(ctx_);
        multInteger(a, (i64)rr, r);
        if (ri != 0) {
            Ciphertext t(ctx_);
            multImagUnit(a, t);
            multInteger(t, (i64)ri, t);
            add(r, t, r);
        }
        out = std::move(r);
        return;
    }
    multWithoutRescale(a, cst, out);
    rescale(out);
}
void HomEvaluator::mult(const Plaintext &a, const Complex &cst, Plaintext &out) const {
    Message m = EnDecoder(ctx_).decode(a);
    for (auto &z : m) z *= cst;
    out = EnDecoder(ctx_).encode(m, a.level_);
}
void HomEvaluator::mult(const Plaintext &a, const Plaintext &b, Plaintext &out) const {
    const u64 lvl = std::min(a.level_, b.level_);
    if (lvl == 0) throw RuntimeException("mult(pt, pt): level 0 cannot be rescaled");
    Plaintext r(ctx_);
    r.allocate(lvl, 1);
    ck(hemm_pointwise(ctx_->dev, HEMM_MUL, a.buf_.data(), 0, b.buf_.data(), 0, r.buf_.data(), 0, (uint32_t)lvl + 1, 0,
                      1, nullptr));
    rescale(r);
    out = std::move(r);
}

void HomEvaluator::tensor(const Ciphertext &a, const Ciphertext &b, Ciphertext &out) const {
    require_rc0(a, "tensor");
    require_rc0(b, "tensor");
    if (a.num_poly_ != 2 || b.num_poly_ != 2) throw RuntimeException("tensor: operands must have two polynomials");
    const u64 lvl = std::min(a.level_, b.level_);
    const Ciphertext *pa = &a, *pb = &b;
    Ciphertext la(ctx_), lb(ctx_);
    if (a.level_ > lvl) {
        levelDown(a, lvl, la);
        pa = &la;
    }
    if (b.level_ > lvl) {
        levelDown(b, lvl, lb);
        pb = &lb;
    }
    const u64 occ = std::min(a.occupied_, b.occupied_);
    OutSlot o(ctx_, out, 3, lvl, 1, false, {&a, &b});
    ck(hemm_tensor(ctx_->dev, pa->buf_.data(), pa->polyStride(), pb->buf_.data(), pb->polyStride(),
                   o.get().buf_.data(), o.get().polyStride(), (uint32_t)lvl + 1, 0, nullptr));
    o.commit(occ);
}
void HomEvaluator::tensorAccumulate(const Ciphertext &a, const Ciphertext &b, Ciphertext &acc, bool first) const {
    if (first) {
        tensor(a, b, acc);
        return;
    }
    if (a.level_ != b.level_ || acc.level_ != a.level_ || acc.num_poly_ != 3 || acc.rescale_counter_ != 1)
        throw RuntimeException("tensorAccumulate: shape mismatch");
    ck(hemm_tensor(ctx_->dev, a.buf_.data(), a.polyStride(), b.buf_.data(), b.polyStride(), acc.buf_.data(),
                   acc.polyStride(), (uint32_t)a.level_ + 1, 1, nullptr));
    acc.occupied_ = std::max(acc.occupied_, std::min(a.occupied_, b.occupied_));
}
void HomEvaluator::relinearize(const Ciphertext &a, Ciphertext &out) const {
    if (a.num_poly_ != 3) throw RuntimeException("relinearize: operand must have three polynomials");
    Ciphertext r(ctx_);
    r.allocate(2, a.level_, a.rescale_counter_);
    ck(hemm_relinearize(ctx_->dev, a.buf_.data(), a.polyStride(), pack_.multKey(), (uint32_t)a.level_ + 1,
                        r.buf_.data(), r.polyStride(), nullptr));
    r.occupied_ = a.occupied_;
    out = std::move(r);
}
void HomEvaluator::rescale(Ciphertext &a) const {
    if (a.rescale_counter_ == 0) throw RuntimeException("rescale: nothing to rescale");
    if (a.level_ == 0) throw RuntimeException("rescale: level 0 cannot be rescaled");
    Ciphertext r(ctx_);
    r.allocate(a.num_poly_, a.level_ - 1, a.rescale_counter_ - 1);
    ck(hemm_rescale(ctx_->dev, a.buf_.data(), a.polyStride(), r.buf_.data(), r.polyStride(), (uint32_t)a.level_ + 1,
                    (uint32_t)a.num_poly_, nullptr));
    r.occupied_ = a.occupied_;
    a = std::move(r);
}
void HomEvaluator::rescale(Plaintext &a) const {
    if (a.rescale_counter_ == 0 || a.level_ == 0) throw RuntimeException("rescale: nothing to rescale");
    Plaintext r(ctx_);
    r.allocate(a.level_ - 1, a.rescale_counter_ - 1);
    ck(hemm_rescale(ctx_->dev, a.buf_.data(), 0, r.buf_.data(), 0, (uint32_t)a.level_ + 1, 1, nullptr));
    a = std::move(r);
}
void HomEvaluator::mult(const Ciphertext &a, const Ciphertext &b, Ciphertext &out) const {
    Ciphertext t(ctx_);
    tensor(a, b, t);
    relinearize(t, t);
    rescale(t);
    out = std::move(t);
}
void HomEvaluator::square(const Ciphertext &a, Ciphertext &out) const { mult(a, a, out); }

namespace {
// hemm_rescale of n_polys polynomials stored back to back, in as few calls as the context's scratch region allows
// ((dnum + 7) (nQ + nP) limbs per call)
void rescale_many(const Context &c, const u64 *in, u64 *out, u64 nq, size_t n_polys) {
    const u64 N = c->N;
    const size_t per_call = std::max<size_t>(1, (size_t)((c->dnum + 7) * (c->nQ + c->nP) / nq));
    for (size_t p0 = 0; p0 < n_polys; p0 += per_call) {
        const size_t np = std::min(per_call, n_polys - p0);
        ck(hemm_rescale(c->dev, in + p0 * nq * N, nq * N, out + p0 * (nq - 1) * N, (nq - 1) * N, (uint32_t)nq, (uint32_t)np,
                        nullptr));
    }
}
}  // namespace

void HomEvaluator::multRealBatch(const Ciphertext &a, const std::vector<Real> &csts, std::vector<Ciphertext> &out) const {
    require_rc0(a, "multRealBatch");
    if (a.num_poly_ != 2 || a.level_ == 0) throw RuntimeException("multRealBatch: two polynomials above level 0 are needed");
    const size_t n = csts.size();
    const u64 lvl = a.level_, nq = lvl + 1, N = ctx_->N;
    const Real delta = ctx_->delta[lvl];
    std::vector<Ciphertext> res;
    res.reserve(n);
    if (n == 0) {
        out = std::move(res);
        return;
    }
    DeviceBuffer t(ctx_, n * 2 * nq * N), low(ctx_, n * 2 * lvl * N);
    for (size_t i = 0; i < n; i++) {
        const auto sc = int_residues(ctx_, (i64)llround(csts[i] * delta), nq);
        ck(hemm_mul_scalar(ctx_->dev, a.buf_.data(), a.polyStride(), sc.data(), t.data() + i * 2 * nq * N, nq * N, (uint32_t)nq,
                           0, 2, nullptr));
    }
    rescale_many(ctx_, t.data(), low.data(), nq, 2 * n);
    for (size_t i = 0; i < n; i++) {
        res.emplace_back(ctx_);
        res.back().allocate(2, lvl - 1, 0);
        (void)hipMemcpyAsync(res.back().buf_.data(), low.data() + i * 2 * lvl * N, 2 * lvl * N * 8, hipMemcpyDeviceToDevice,
                             ctx_->stream());
        res.back().occupied_ = a.occupied_;
    }
    out = std::move(res);
}

void HomEvaluator::multBatch(const std::vector<const Ciphertext *> &a, const std::vector<const Ciphertext *> &b,
                             std::vector<Ciphertext> &out) const {
    const size_t n = a.size();
    if (n == 0 || n != b.size()) throw RuntimeException("multBatch: operand lists of different lengths");
    bool shared = n > 1 && ctx_->N >= 512;   // (the hoisted sums need N >= 512)
    for (size_t i = 0; i < n; i++) {
        if (a[i] == nullptr || b[i] == nullptr) throw RuntimeException("multBatch: null operand");
        shared = shared && a[i]->level_ == a[0]->level_ && b[i]->level_ == a[0]->level_ && a[i]->level_ > 0 &&
                 a[i]->rescale_counter_ == 0 && b[i]->rescale_counter_ == 0 && a[i]->num_poly_ == 2 && b[i]->num_poly_ == 2;
    }
    std::vector<Ciphertext> res;
    res.reserve(n);
    if (!shared) {
        for (size_t i = 0; i < n; i++) {
            res.emplace_back(ctx_);
            mult(*a[i], *b[i], res.back());
        }
        out = std::move(res);
        return;
    }
    const u64 lvl = a[0]->level_, nq = lvl + 1, N = ctx_->N, E = nq + ctx_->nP, beta = (nq + ctx_->alpha - 1) / ctx_->alpha;
    const u64 t3w = 3 * nq * N, ctw = 2 * nq * N;
    // tensor products, three polynomials each
    DeviceBuffer t3(ctx_, n * t3w);
    for (size_t i = 0; i < n; i++)
        ck(hemm_tensor(ctx_->dev, a[i]->buf_.data(), a[i]->polyStride(), b[i]->buf_.data(), b[i]->polyStride(),
                       t3.data() + i * t3w, nq * N, (uint32_t)nq, 0, nullptr));
    // relinearisation of all of them: d2 extended in one ModUp, <ext(d2), evk> + P (d0, d1) in one sum, one ModDown
    // (ModDown(P d + k) = d + ModDown(k) residue for residue: what relinearize() adds after its ModDown)
    DeviceBuffer ext(ctx_, n * beta * E * N), ws(ctx_, n * nq * N);
    ck(hemm_modup_batch(ctx_->dev, t3.data() + 2 * nq * N, t3w, (uint32_t)nq, (uint32_t)n, ext.data(), ws.data(), nullptr));
    std::vector<hemm_rot_term> terms;
    std::vector<uint32_t> off{0};
    for (size_t i = 0; i < n; i++) {
        hemm_rot_term t{};
        t.ext = ext.data() + i * beta * E * N;
        t.b = t3.data() + i * t3w;
        if (pack_.compactible()) {
            t.evk = pack_.compactKey(0, 0);
            t.flags = HEMM_ROT_COMPACT_KEY;
        } else {
            t.evk = pack_.multKey();
        }
        t.galois = 1;
        t.pt_galois = 1;
        terms.push_back(t);
        hemm_rot_term d1{};   // the second polynomial needs no key: P d1 on the chain limbs
        d1.ext = t3.data() + i * t3w + nq * N;
        d1.galois = 1;
        d1.pt_galois = 1;
        terms.push_back(d1);
        off.push_back((uint32_t)terms.size());
    }
    DeviceBuffer y(ctx_, n * 2 * E * N), r(ctx_, n * ctw), ws2(ctx_, n * ctw), low(ctx_, n * 2 * lvl * N);
    ck(hemm_hoisted_moddown(ctx_->dev, terms.data(), off.data(), (uint32_t)n, (uint32_t)nq, 0, 0, y.data(), r.data(), nq * N,
                            ws2.data(), nullptr));
    rescale_many(ctx_, r.data(), low.data(), nq, 2 * n);
    for (size_t i = 0; i < n; i++) {
        res.emplace_back(ctx_);
        res.back().allocate(2, lvl - 1, 0);
        (void)hipMemcpyAsync(res.back().buf_.data(), low.data() + i * 2 * lvl * N, 2 * lvl * N * 8, hipMemcpyDeviceToDevice,
                             ctx_->stream());
        res.back().occupied_ = std::min(a[i]->occupied_, b[i]->occupied_);
    }
    out = std::move(res);
}

// Drop to target_level keeping the fixed per-level scale: read the first target+2 limbs, multiply by
// round(Delta_target * q_{target+1} / Delta_level) and rescale by q_{target+1}.
void HomEvaluator::levelDown(const Ciphertext &a, u64 target, Ciphertext &out) const {
    if (target > a.level_) throw RuntimeException("levelDown: target above the current level");
    if (target == a.level_) {
        if (&out != &a) out = a;
        return;
    }
    require_rc0(a, "levelDown");
    const Real cst = ctx_->delta[target] * (Real)ctx_->q[target + 1] / ctx_->delta[a.level_];
    const i64 v = (i64)llround(cst);
    Ciphertext t(ctx_);
    t.allocate(a.num_poly_, target + 1, 1);
    auto sc = int_residues(ctx_, v, target + 2);
    ck(hemm_mul_scalar(ctx_->dev, a.buf_.data(), a.polyStride(), sc.data(), t.buf_.data(), t.polyStride(),
                       (uint32_t)target + 2, 0, (uint32_t)a.num_poly_, nullptr));
    t.occupied_ = a.occupied_;
    rescale(t);
    out = std::move(t);
}
void HomEvaluator::levelDownOne(const Ciphertext &a, Ciphertext &out) const {
    if (a.level_ == 0) throw RuntimeException("levelDownOne: already at level 0");
    levelDown(a, a.level_ - 1, out);
}

// ---- rotations -------------------------------------------------------------------------------------
void HomEvaluator::leftRotate(const Message &a, u64 rot, Message &out) const {
    const u64 n = a.getSize();
    rot %= n;
    Message r(a.getLogSlots());
    for (u64 i = 0; i < n; i++) r[i] = a[(i + rot) % n];
    out = std::move(r);
}
void HomEvaluator::rightRotate(const Message &a, u64 rot, Message &out) const {
    const u64 n = a.getSize();
    leftRotate(a, (n - rot % n) % n, out);
}
void HomEvaluator::leftRotate(const Plaintext &a, u64 rot, Plaintext &out) const {
    const u64 slots = ctx_->N / 2;
    rot %= slots;
    if (rot == 0) {
        if (&out != &a) out = a;
        return;
    }
    Plaintext r(ctx_);
    r.allocate(a.level_, a.rescale_counter_);
    r.scale_ = a.scale_;
    ck(hemm_automorphism(ctx_->dev, a.buf_.data(), 0, r.buf_.data(), 0, powmod(5, rot, 2 * ctx_->N),
                         (uint32_t)a.level_ + 1, 1, nullptr));
    out = std::move(r);
}
void HomEvaluator::rightRotate(const Plaintext &a, u64 rot, Plaintext &out) const {
    const u64 slots = ctx_->N / 2;
    leftRotate(a, (slots - rot % slots) % slots, out);
}
void HomEvaluator::applyGalois(const Ciphertext &a, u64 galois, Ciphertext &out) const {
    if (a.num_poly_ != 2) throw RuntimeException("rotate/conjugate: operand must have two polynomials");
    Ciphertext r(ctx_);
    r.allocate(2, a.level_, a.rescale_counter_);
    ck(hemm_rotate(ctx_->dev, a.buf_.data(), a.polyStride(), pack_.galoisKey(galois), galois, (uint32_t)a.level_ + 1,
                   r.buf_.data(), r.polyStride(), nullptr));
    out = std::move(r);
}
void HomEvaluator::leftRotate(const Ciphertext &a, u64 rot, Ciphertext &out) const {
    const u64 slots = ctx_->N / 2, M = 2 * ctx_->N;
    rot %= slots;
    if (rot == 0) {
        if (&out != &a) out = a;
        return;
    }
    const u64 g = powmod(5, rot, M);
    if (pack_.hasGaloisKey(g)) {
        applyGalois(a, g, out);
        return;
    }
    // no direct key: compose power-of-two rotations (left when the binary expansion is short,
    // right otherwise), the way a key bundle of powers of two is meant to be used
    const u64 right = slots - rot;
    const bool use_left = __builtin_popcountll(rot) <= __builtin_popcountll(right);
    const u64 amount = use_left ? rot : right;
    const Ciphertext *cur = &a;
    Ciphertext tmp(ctx_);
    for (u64 bit = 1; bit < slots; bit <<= 1) {
        if (!(amount & bit)) continue;
        const u64 step = use_left ? bit : slots - bit;
        const u64 gs = powmod(5, step, M);
        if (!pack_.hasGaloisKey(gs))
            throw RuntimeException("no rotation key for " + std::to_string(rot) + " nor for its power-of-two parts");
        applyGalois(*cur, gs, tmp);
        cur = &tmp;
    }
    out = tmp;
}
void HomEvaluator::rightRotate(const Ciphertext &a, u64 rot, Ciphertext &out) const {
    const u64 slots = ctx_->N / 2;
    leftRotate(a, (slots - rot % slots) % slots, out);
}
void HomEvaluator::conjugate(const Ciphertext &a, Ciphertext &out) const {
    const u64 occ = a.occupied_;   // conjugation acts on every slot by itself
    applyGalois(a, 2 * ctx_->N - 1, out);
    out.occupied_ = occ;
}
void HomEvaluator::leftRotateReduce(const Ciphertext &a, u64 idx_interval, u64 num_summation, Ciphertext &out) const {
    // sum_{k < num_summation} leftRotate(a, k * idx_interval), num_summation a power of two
    Ciphertext acc(a), t(ctx_);
    for (u64 step = 1; step < num_summation; step <<= 1) {
        leftRotate(acc, step * idx_interval, t);
        add(acc, t, acc);
    }
    out = std::move(acc);
}

// out = rescale( sum_k cts[k] * leftRotate(pt, k * slots / cts.size()) )
void HomEvaluator::matmul(const std::vector<Ciphertext> &cts, const Plaintext &pt, Ciphertext &out) const {
    matmul(cts, pt, out, 0);
}
void HomEvaluator::matmul(const std::vector<Ciphertext> &cts, const Plaintext &pt, Ciphertext &out, u64 step_in) const {
    if (cts.empty()) throw RuntimeException("matmul: empty operand list");
    const u64 slots = ctx_->N / 2, step = step_in ? step_in : slots / cts.size(), lvl = cts[0].level_;
    if (pt.level_ < lvl) throw RuntimeException("matmul: plaintext level below the ciphertext level");
    // one launch: every term reads its ciphertext and the plaintext through that term's automorphism
    Ciphertext acc(ctx_);
    acc.allocate(2, lvl, 1);
    std::vector<hemm_lin_term> terms(cts.size());
    for (size_t k = 0; k < cts.size(); k++) {
        if (cts[k].level_ != lvl || cts[k].rescale_counter_ != 0) throw RuntimeException("matmul: level mismatch");
        terms[k].ct = cts[k].buf_.data();
        terms[k].mask = pt.buf_.data();
        terms[k].stride = cts[k].polyStride();
        const u64 r = (k * step) % slots;
        terms[k].galois = r == 0 ? 0 : powmod(5, r, 2 * ctx_->N);
    }
    const uint32_t off[2] = {0, (uint32_t)cts.size()};
    ck(hemm_masked_sum_batch(ctx_->dev, terms.data(), off, 1, (uint32_t)lvl + 1, 2, acc.buf_.data(), nullptr));
    rescale(acc);
    out = std::move(acc);
}

void Bootstrapper::bootstrap(const Ciphertext &, Ciphertext &) const {
    throw RuntimeException("bootstrapping is not part of this build");
}
void Bootstrapper::bootstrap(const Ciphertext &, Ciphertext &, Ciphertext &) const {
    throw RuntimeException("bootstrapping is not part of this build");
}
void Bootstrapper::bootstrapExtended(const Ciphertext &, Ciphertext &) const {
    throw RuntimeException("bootstrapping is not part of this build");
}
void Bootstrapper::bootstrapExtended(const Ciphertext &, Ciphertext &, Ciphertext &) const {
    throw RuntimeException("bootstrapping is not part of this build");
}

}  // namespace HEaaN

// TEST INFRASTRUCTURE ONLY -- CPU oracle for the RNS-CKKS primitives under HEMMer's
// homomorphic matrix multiplication.
//
// The reference keeps every ring operation inside the closed HEaaN library (only call
// sites such as ciphertext/src/MatrixUtils.cpp:1378-1443 and the declarations in
// ciphertext/external/include/HEaaN/HomEvaluator.hpp:30-616 are visible), so this file
// restates the *published* RNS-CKKS algorithms those entry points name:
//   - negacyclic NTT/INTT (merged-twiddle Cooley-Tukey / Gentleman-Sande, Harvey lazy
//     butterflies)                          <- HomEvaluator.hpp: every NTT-form operand
//   - canonical-embedding encode/decode     <- EnDecoder.hpp:51,66
//   - sk-encrypt / decrypt                  <- Encryptor.hpp:81-84, Decryptor.hpp:36
//   - Galois automorphism + hybrid key switching (ModUp, evk inner product, ModDown)
//                                           <- HomEvaluator.hpp:383-403,465,524
//   - tensor / relinearize / rescale        <- HomEvaluator.hpp:510-540
// Only tests, the smoke check and the cpu_baseline leg of the benchmark may load this
// library.  Nothing in the shipped GPU path links, imports or calls it.
//
// Pins (see tests/test_oracle_*.py): modular arithmetic and NTT against Python big
// integers and the O(N^2) definition; basis conversion against exact CRT; encode/decode
// against the direct embedding sum; key switching / rescale through decryption
// identities.  Exact residues of the closed library cannot be pinned: parity unpinned
// for HEaaN's own RNG stream, rounding mode and key-switch variant.
//
// Data layout everywhere: [poly][limb][N] contiguous uint64 residues in [0, q).
// "limb j of an operand with nq active Q-limbs" uses prime j if j < nq, else the
// special prime nQ + (j - nq).

#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <vector>

typedef uint64_t u64;
typedef int64_t i64;
typedef unsigned __int128 u128;

namespace {

inline u64 mulmod(u64 a, u64 b, u64 q) { return (u64)((u128)a * b % q); }
inline u64 addmod(u64 a, u64 b, u64 q) {
    u64 s = a + b;
    return s >= q ? s - q : s;
}
inline u64 submod(u64 a, u64 b, u64 q) { return a >= b ? a - b : a + q - b; }
u64 powmod(u64 a, u64 e, u64 q) {
    u64 r = 1 % q;
    a %= q;
    while (e) {
        if (e & 1) r = mulmod(r, a, q);
        a = mulmod(a, a, q);
        e >>= 1;
    }
    return r;
}
inline u64 invmod(u64 a, u64 q) { return powmod(a, q - 2, q); }

inline unsigned bitrev(unsigned x, int bits) {
    unsigned r = 0;
    for (int i = 0; i < bits; i++) {
        r = (r << 1) | (x & 1);
        x >>= 1;
    }
    return r;
}

// splitmix64 finaliser used as a counter-based generator: draw(key, ctr) = sm64(key + ctr * golden-ratio constant).
inline u64 sm64(u64 x) {
    x += 0x9E3779B97F4A7C15ull;
    u64 z = x;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
inline u64 stream_key(u64 seed, u64 tag, u64 a, u64 b) {
    return sm64(sm64(sm64(seed + tag) + a) + b);
}
inline u64 draw(u64 key, u64 ctr) { return sm64(key + ctr * 0x9E3779B97F4A7C15ull); }

struct Prime {
    u64 q;
    u64 psi;                     // primitive 2N-th root of unity
    std::vector<u64> w, ws;      // psi^bitrev(i), Shoup quotient floor(w*2^64/q)
    std::vector<u64> iw, iws;    // inverse-transform table
    u64 ninv, ninv_s;
};

struct Ctx {
    int logN, N, nQ, nP, dnum, alpha;
    std::vector<Prime> pr;       // nQ chain primes then nP special primes
    std::vector<u64> rot_group;  // 5^j mod 2N
    std::vector<double> ksi_re, ksi_im;
    int threads = 1;             // limbs / coefficients are independent: the loops over them may run in parallel
};

inline u64 shoup(u64 w, u64 q) { return (u64)(((u128)w << 64) / q); }

// x*w mod q given ws = floor(w*2^64/q); result in [0, 2q) (lazy).
inline u64 mul_shoup_lazy(u64 x, u64 w, u64 ws, u64 q) {
    u64 hi = (u64)(((u128)x * ws) >> 64);
    return x * w - hi * q;
}

void build_prime(Prime &p, u64 q, int logN) {
    const int N = 1 << logN;
    p.q = q;
    // smallest g = 2,3,... whose (q-1)/2N-th power has order exactly 2N
    u64 psi = 0;
    for (u64 g = 2;; g++) {
        u64 c = powmod(g, (q - 1) / (2 * (u64)N), q);
        if (powmod(c, N, q) == q - 1) {
            psi = c;
            break;
        }
    }
    p.psi = psi;
    u64 ipsi = invmod(psi, q);
    p.w.resize(N);
    p.ws.resize(N);
    p.iw.resize(N);
    p.iws.resize(N);
    std::vector<u64> pw(N), ipw(N);
    pw[0] = 1;
    ipw[0] = 1;
    for (int i = 1; i < N; i++) {
        pw[i] = mulmod(pw[i - 1], psi, q);
        ipw[i] = mulmod(ipw[i - 1], ipsi, q);
    }
    for (int i = 0; i < N; i++) {
        unsigned r = bitrev((unsigned)i, logN);
        p.w[i] = pw[r];
        p.ws[i] = shoup(p.w[i], q);
        p.iw[i] = ipw[r];
        p.iws[i] = shoup(p.iw[i], q);
    }
    p.ninv = invmod((u64)N, q);
    p.ninv_s = shoup(p.ninv, q);
}

// Forward negacyclic NTT, natural order in, bit-reversed order out:
// out[k] = sum_j a[j] * psi^{(2*bitrev(k)+1) j}.
void ntt_fwd(const Prime &p, u64 *a, int N) {
    const u64 q = p.q, two_q = 2 * q;
    int t = N;
    for (int m = 1; m < N; m <<= 1) {
        t >>= 1;
        for (int i = 0; i < m; i++) {
            const u64 w = p.w[m + i], ws = p.ws[m + i];
            u64 *x = a + 2 * i * t, *y = x + t;
            for (int j = 0; j < t; j++) {
                u64 u = x[j];
                if (u >= two_q) u -= two_q;
                u64 v = mul_shoup_lazy(y[j], w, ws, q);
                x[j] = u + v;
                y[j] = u - v + two_q;
            }
        }
    }
    for (int j = 0; j < N; j++) {
        u64 v = a[j];
        if (v >= two_q) v -= two_q;
        if (v >= q) v -= q;
        a[j] = v;
    }
}

// Inverse of ntt_fwd (bit-reversed in, natural out), including the 1/N factor.
void ntt_inv(const Prime &p, u64 *a, int N) {
    const u64 q = p.q, two_q = 2 * q;
    int t = 1;
    for (int m = N >> 1; m >= 1; m >>= 1) {
        for (int i = 0; i < m; i++) {
            const u64 w = p.iw[m + i], ws = p.iws[m + i];
            u64 *x = a + 2 * i * t, *y = x + t;
            for (int j = 0; j < t; j++) {
                u64 u = x[j], v = y[j];
                u64 s = u + v;
                if (s >= two_q) s -= two_q;
                u64 d = u - v + two_q;
                x[j] = s;
                y[j] = mul_shoup_lazy(d, w, ws, q);
            }
        }
        t <<= 1;
    }
    for (int j = 0; j < N; j++) {
        u64 v = mul_shoup_lazy(a[j], p.ninv, p.ninv_s, q);
        if (v >= q) v -= q;
        a[j] = v;
    }
}

inline int prime_of(const Ctx *c, int j, int nq) { return j < nq ? j : c->nQ + (j - nq); }

// Fast basis conversion of coefficient-form residues x_i (i in src) to modulus index dst:
//   y = sum_i [x_i * (S/q_i)^{-1}]_{q_i} * (S/q_i)  mod q_dst,   S = prod_{i in src} q_i.
struct BConv {
    std::vector<int> src;
    std::vector<u64> qhat_inv;             // per src
    std::vector<std::vector<u64>> qhat;    // [dst][src]
    std::vector<int> dst;
};
BConv make_bconv(const Ctx *c, const std::vector<int> &src, const std::vector<int> &dst) {
    BConv b;
    b.src = src;
    b.dst = dst;
    for (size_t i = 0; i < src.size(); i++) {
        u64 qi = c->pr[src[i]].q, prod = 1;
        for (size_t j = 0; j < src.size(); j++)
            if (j != i) prod = mulmod(prod, c->pr[src[j]].q % qi, qi);
        b.qhat_inv.push_back(invmod(prod, qi));
    }
    for (size_t d = 0; d < dst.size(); d++) {
        u64 t = c->pr[dst[d]].q;
        std::vector<u64> row;
        for (size_t i = 0; i < src.size(); i++) {
            u64 prod = 1;
            for (size_t j = 0; j < src.size(); j++)
                if (j != i) prod = mulmod(prod, c->pr[src[j]].q % t, t);
            row.push_back(prod);
        }
        b.qhat.push_back(row);
    }
    return b;
}
// in: [src.size()][N] coefficient form; out: [dst.size()][N] coefficient form
void run_bconv(const Ctx *c, const BConv &b, const u64 *const *in, u64 *const *out) {
    const int N = c->N;
    const size_t ns = b.src.size();
    if (ns > 64) abort();
#pragma omp parallel for num_threads(c->threads) schedule(static)
    for (int n = 0; n < N; n++) {
        u64 v[64];
        for (size_t i = 0; i < ns; i++) v[i] = mulmod(in[i][n], b.qhat_inv[i], c->pr[b.src[i]].q);
        for (size_t d = 0; d < b.dst.size(); d++) {
            u64 t = c->pr[b.dst[d]].q;
            u128 acc = 0;
            for (size_t i = 0; i < ns; i++) acc += (u128)(v[i] % t) * b.qhat[d][i] % t;
            out[d][n] = (u64)(acc % t);
        }
    }
}

}  // namespace

extern "C" {

void *orc_create(int logN, int nQ, int nP, const u64 *primes, int dnum) {
    Ctx *c = new Ctx;
    c->logN = logN;
    c->N = 1 << logN;
    c->nQ = nQ;
    c->nP = nP;
    c->dnum = dnum;
    c->alpha = dnum > 0 ? (nQ + dnum - 1) / dnum : nQ;
    c->pr.resize(nQ + nP);
    for (int i = 0; i < nQ + nP; i++) build_prime(c->pr[i], primes[i], logN);
    const int n = c->N / 2, M = 2 * c->N;
    c->rot_group.resize(n);
    u64 g = 1;
    for (int j = 0; j < n; j++) {
        c->rot_group[j] = g;
        g = g * 5 % M;
    }
    c->ksi_re.resize(M + 1);
    c->ksi_im.resize(M + 1);
    // cos and sin in separate loops: called on one value side by side, an optimising compiler may replace the pair by a
    // single sincos call, whose results differ from cos / sin in the last bit for a few arguments
    for (int k = 0; k <= M; k++) c->ksi_re[k] = cos(2.0 * M_PI * (double)k / (double)M);
    for (int k = 0; k <= M; k++) c->ksi_im[k] = sin(2.0 * M_PI * (double)k / (double)M);
    return c;
}
void orc_destroy(void *h) { delete (Ctx *)h; }
// worker threads for the loops over independent limbs / coefficients (results do not depend on it)
void orc_set_threads(void *h, int threads) { ((Ctx *)h)->threads = threads < 1 ? 1 : threads; }
u64 orc_psi(void *h, int pi) { return ((Ctx *)h)->pr[pi].psi; }
int orc_alpha(void *h) { return ((Ctx *)h)->alpha; }

// ---- RNG primitives exposed so tests can pin them -------------------------------------
u64 orc_sm64(u64 x) { return sm64(x); }
u64 orc_stream_key(u64 seed, u64 tag, u64 a, u64 b) { return stream_key(seed, tag, a, b); }

// uniform residues in [0,q) for coefficient i: attempt t uses key sm64(key+t), counter i.
void orc_sample_uniform(void *h, u64 key, int prime_idx, u64 *out) {
    Ctx *c = (Ctx *)h;
    u64 q = c->pr[prime_idx].q;
    int bits = 64 - __builtin_clzll(q);
    u64 mask = bits >= 64 ? ~0ull : ((1ull << bits) - 1);
    for (int i = 0; i < c->N; i++) {
        for (u64 t = 0;; t++) {
            u64 x = draw(sm64(key + t), (u64)i) & mask;
            if (x < q) {
                out[i] = x;
                break;
            }
        }
    }
}
// ternary secret with exactly hw non-zeros: scan the stream, position = low bits,
// sign = top bit, skipping occupied positions.
void orc_sample_ternary(void *h, u64 key, int hw, int *out) {
    Ctx *c = (Ctx *)h;
    memset(out, 0, sizeof(int) * c->N);
    int placed = 0;
    for (u64 ctr = 0; placed < hw; ctr++) {
        u64 x = draw(key, ctr);
        int pos = (int)(x & (u64)(c->N - 1));
        if (out[pos]) continue;
        out[pos] = (x >> 63) ? -1 : 1;
        placed++;
    }
}
// centred binomial error, 21 bit pairs (variance 10.5).
void orc_sample_error(void *h, u64 key, int *out) {
    Ctx *c = (Ctx *)h;
    const u64 M21 = (1ull << 21) - 1;
    for (int i = 0; i < c->N; i++) {
        u64 x = draw(key, (u64)i);
        out[i] = __builtin_popcountll(x & M21) - __builtin_popcountll((x >> 21) & M21);
    }
}
// small signed coefficients -> residues of one prime (coefficient form)
void orc_lift_small(void *h, const int *v, int prime_idx, u64 *out) {
    Ctx *c = (Ctx *)h;
    u64 q = c->pr[prime_idx].q;
    for (int i = 0; i < c->N; i++) out[i] = v[i] >= 0 ? (u64)v[i] : q - (u64)(-v[i]);
}

// ---- NTT ------------------------------------------------------------------------------
void orc_ntt(void *h, u64 *a, int prime_idx, int inverse) {
    Ctx *c = (Ctx *)h;
    if (inverse)
        ntt_inv(c->pr[prime_idx], a, c->N);
    else
        ntt_fwd(c->pr[prime_idx], a, c->N);
}
// data [n_polys][n_limbs][N]; limb j uses prime prime_idx[j]
void orc_ntt_batch(void *h, u64 *data, const int *prime_idx, int n_limbs, int n_polys, int inverse,
                   int threads) {
    Ctx *c = (Ctx *)h;
    const int total = n_limbs * n_polys;
#pragma omp parallel for num_threads(threads) schedule(dynamic)
    for (int k = 0; k < total; k++) {
        int j = k % n_limbs;
        u64 *a = data + (size_t)k * c->N;
        if (inverse)
            ntt_inv(c->pr[prime_idx[j]], a, c->N);
        else
            ntt_fwd(c->pr[prime_idx[j]], a, c->N);
    }
}

// ---- pointwise (one limb) -------------------------------------------------------------
// op: 0 add, 1 sub, 2 mul, 3 neg(a), 4 mac (out += a*b)
void orc_pointwise(void *h, int op, const u64 *a, const u64 *b, u64 *out, int prime_idx) {
    Ctx *c = (Ctx *)h;
    const u64 q = c->pr[prime_idx].q;
    for (int i = 0; i < c->N; i++) {
        switch (op) {
            case 0: out[i] = addmod(a[i], b[i], q); break;
            case 1: out[i] = submod(a[i], b[i], q); break;
            case 2: out[i] = mulmod(a[i], b[i], q); break;
            case 3: out[i] = a[i] ? q - a[i] : 0; break;
            case 4: out[i] = addmod(out[i], mulmod(a[i], b[i], q), q); break;
        }
    }
}
void orc_mul_scalar(void *h, const u64 *a, u64 s, u64 *out, int prime_idx) {
    Ctx *c = (Ctx *)h;
    const u64 q = c->pr[prime_idx].q;
    s %= q;
    for (int i = 0; i < c->N; i++) out[i] = mulmod(a[i], s, q);
}
// multiply by the monomial X^{N/2} in NTT form: slot k holds the evaluation at
// psi^{2*bitrev(k)+1}, so the factor is psi^{(N/2)(2*bitrev(k)+1)}.
void orc_mul_imag_unit(void *h, const u64 *a, u64 *out, int prime_idx) {
    Ctx *c = (Ctx *)h;
    const Prime &p = c->pr[prime_idx];
    u64 I = powmod(p.psi, (u64)c->N / 2, p.q);  // I^2 = -1
    for (int k = 0; k < c->N; k++) {
        unsigned e = bitrev((unsigned)k, c->logN);
        u64 f = (e & 1) ? p.q - I : I;  // I^(2e+1) = I * (-1)^e
        out[k] = mulmod(a[k], f, p.q);
    }
}

// ---- automorphism X -> X^g (g odd) ------------------------------------------------------
void orc_automorphism_coeff(void *h, const u64 *in, u64 *out, u64 g, int prime_idx) {
    Ctx *c = (Ctx *)h;
    const u64 q = c->pr[prime_idx].q;
    const u64 M = 2 * (u64)c->N;
    for (int i = 0; i < c->N; i++) {
        u64 e = (u64)i * g % M;
        if (e < (u64)c->N)
            out[e] = in[i];
        else
            out[e - c->N] = in[i] ? q - in[i] : 0;
    }
}
// NTT form: out[k] = in[k'] with 2*br(k')+1 = (2*br(k)+1)*g mod 2N
void orc_automorphism_ntt(void *h, const u64 *in, u64 *out, u64 g) {
    Ctx *c = (Ctx *)h;
    const u64 M = 2 * (u64)c->N;
    for (int k = 0; k < c->N; k++) {
        u64 e = (2 * (u64)bitrev((unsigned)k, c->logN) + 1) * g % M;
        unsigned kp = bitrev((unsigned)((e - 1) / 2), c->logN);
        out[k] = in[kp];
    }
}

// ---- hybrid key switching ---------------------------------------------------------------
// ModUp: in [nq][N] NTT form (Q limbs 0..nq-1).  out [beta][nq+K][N] NTT form, digit d
// extended to all active limbs; beta = ceil(nq/alpha).
void orc_modup(void *h, const u64 *in, int nq, u64 *out) {
    Ctx *c = (Ctx *)h;
    const int N = c->N, K = c->nP, ext = nq + K;
    const int beta = (nq + c->alpha - 1) / c->alpha;
    std::vector<u64> coef((size_t)nq * N);
    memcpy(coef.data(), in, sizeof(u64) * (size_t)nq * N);
#pragma omp parallel for num_threads(c->threads) schedule(dynamic)
    for (int j = 0; j < nq; j++) ntt_inv(c->pr[j], coef.data() + (size_t)j * N, N);
    for (int d = 0; d < beta; d++) {
        int lo = d * c->alpha, hi = std::min(nq, lo + c->alpha);
        std::vector<int> src, dst, dst_limb;
        for (int j = lo; j < hi; j++) src.push_back(j);
        for (int j = 0; j < ext; j++) {
            if (j >= lo && j < hi) continue;
            dst.push_back(prime_of(c, j, nq));
            dst_limb.push_back(j);
        }
        BConv b = make_bconv(c, src, dst);
        std::vector<const u64 *> ip;
        std::vector<u64 *> op;
        for (int j = lo; j < hi; j++) ip.push_back(coef.data() + (size_t)j * N);
        u64 *od = out + (size_t)d * ext * N;
        for (size_t k = 0; k < dst.size(); k++) op.push_back(od + (size_t)dst_limb[k] * N);
        run_bconv(c, b, ip.data(), op.data());
#pragma omp parallel for num_threads(c->threads) schedule(dynamic)
        for (size_t k = 0; k < dst.size(); k++) ntt_fwd(c->pr[dst[k]], op[k], N);
        for (int j = lo; j < hi; j++)
            memcpy(od + (size_t)j * N, in + (size_t)j * N, sizeof(u64) * N);
    }
}
// evk layout [dnum][2][nQ+nP][N] (b then a); ext [beta][nq+K][N]; acc [2][nq+K][N]
void orc_inner_product(void *h, const u64 *ext, const u64 *evk, int nq, u64 *acc) {
    Ctx *c = (Ctx *)h;
    const int N = c->N, K = c->nP, e = nq + K, full = c->nQ + c->nP;
    const int beta = (nq + c->alpha - 1) / c->alpha;
#pragma omp parallel for num_threads(c->threads) collapse(2) schedule(dynamic)
    for (int pol = 0; pol < 2; pol++)
        for (int j = 0; j < e; j++) {
            int pi = prime_of(c, j, nq);
            const u64 q = c->pr[pi].q;
            u64 *o = acc + ((size_t)pol * e + j) * N;
            for (int n = 0; n < N; n++) {
                u64 s = 0;
                for (int d = 0; d < beta; d++) {
                    u64 x = ext[((size_t)d * e + j) * N + n];
                    u64 k = evk[(((size_t)d * 2 + pol) * full + pi) * N + n];
                    s = addmod(s, mulmod(x, k, q), q);
                }
                o[n] = s;
            }
        }
}
// ModDown: acc [nq+K][N] NTT -> out [nq][N] NTT, out = (acc_Q - BConv_{P->Q}(acc_P)) * P^{-1}
void orc_moddown(void *h, const u64 *acc, int nq, u64 *out) {
    Ctx *c = (Ctx *)h;
    const int N = c->N, K = c->nP;
    std::vector<u64> pc((size_t)K * N);
    memcpy(pc.data(), acc + (size_t)nq * N, sizeof(u64) * (size_t)K * N);
    std::vector<int> src, dst;
#pragma omp parallel for num_threads(c->threads) schedule(dynamic)
    for (int k = 0; k < K; k++) ntt_inv(c->pr[c->nQ + k], pc.data() + (size_t)k * N, N);
    for (int k = 0; k < K; k++) src.push_back(c->nQ + k);
    for (int j = 0; j < nq; j++) dst.push_back(j);
    BConv b = make_bconv(c, src, dst);
    std::vector<const u64 *> ip;
    std::vector<u64 *> op;
    for (int k = 0; k < K; k++) ip.push_back(pc.data() + (size_t)k * N);
    for (int j = 0; j < nq; j++) op.push_back(out + (size_t)j * N);
    run_bconv(c, b, ip.data(), op.data());
#pragma omp parallel for num_threads(c->threads) schedule(dynamic)
    for (int j = 0; j < nq; j++) {
        const u64 q = c->pr[j].q;
        ntt_fwd(c->pr[j], op[j], N);
        u64 pinv = 1;
        for (int k = 0; k < K; k++) pinv = mulmod(pinv, c->pr[c->nQ + k].q % q, q);
        pinv = invmod(pinv, q);
        const u64 *a = acc + (size_t)j * N;
        for (int n = 0; n < N; n++) op[j][n] = mulmod(submod(a[n], op[j][n], q), pinv, q);
    }
}
// full key switch of one NTT-form polynomial: out_b, out_a each [nq][N]
void orc_keyswitch(void *h, const u64 *in, const u64 *evk, int nq, u64 *out_b, u64 *out_a) {
    Ctx *c = (Ctx *)h;
    const int N = c->N, e = nq + c->nP;
    const int beta = (nq + c->alpha - 1) / c->alpha;
    std::vector<u64> ext((size_t)beta * e * N), acc((size_t)2 * e * N);
    orc_modup(h, in, nq, ext.data());
    orc_inner_product(h, ext.data(), evk, nq, acc.data());
    orc_moddown(h, acc.data(), nq, out_b);
    orc_moddown(h, acc.data() + (size_t)e * N, nq, out_a);
}

// ---- rescale: in [nq][N] NTT -> out [nq-1][N] NTT, out_i = (c_i - [c_last]_{q_i}) / q_last
void orc_rescale(void *h, const u64 *in, int nq, u64 *out) {
    Ctx *c = (Ctx *)h;
    const int N = c->N, last = nq - 1;
    std::vector<u64> lc(N), t(N);
    memcpy(lc.data(), in + (size_t)last * N, sizeof(u64) * N);
    ntt_inv(c->pr[last], lc.data(), N);
    const u64 ql = c->pr[last].q;
#pragma omp parallel for num_threads(c->threads) schedule(dynamic) firstprivate(t)
    for (int j = 0; j < last; j++) {
        const u64 q = c->pr[j].q;
        for (int n = 0; n < N; n++) t[n] = lc[n] % q;
        ntt_fwd(c->pr[j], t.data(), N);
        u64 qinv = invmod(ql % q, q);
        const u64 *a = in + (size_t)j * N;
        u64 *o = out + (size_t)j * N;
        for (int n = 0; n < N; n++) o[n] = mulmod(submod(a[n], t[n], q), qinv, q);
    }
}

// ---- tensor product of two 2-poly ciphertexts -> 3 polys (d0=b1b2, d1=a1b2+a2b1, d2=a1a2)
void orc_tensor(void *h, const u64 *ct1, const u64 *ct2, int nq, u64 *out) {
    Ctx *c = (Ctx *)h;
    const int N = c->N;
#pragma omp parallel for num_threads(c->threads) schedule(dynamic)
    for (int j = 0; j < nq; j++) {
        const u64 q = c->pr[j].q;
        const u64 *b1 = ct1 + (size_t)j * N, *a1 = ct1 + ((size_t)nq + j) * N;
        const u64 *b2 = ct2 + (size_t)j * N, *a2 = ct2 + ((size_t)nq + j) * N;
        u64 *d0 = out + (size_t)j * N, *d1 = out + ((size_t)nq + j) * N,
            *d2 = out + ((size_t)2 * nq + j) * N;
        for (int n = 0; n < N; n++) {
            d0[n] = mulmod(b1[n], b2[n], q);
            d1[n] = addmod(mulmod(a1[n], b2[n], q), mulmod(a2[n], b1[n], q), q);
            d2[n] = mulmod(a1[n], a2[n], q);
        }
    }
}

// ---- hoisted rotation term: y (+)= mask * ( <galois(ext), evk> + P * galois(b) ) -----------------
// ext [beta][nq+K][N] (ModUp output), b [nq][N], evk [dnum][2][nQ+nP][N], mask [nq+K][N] or null,
// y [2][nq+K][N].  The automorphism acts on the NTT-form limbs as the index map of
// orc_automorphism_ntt.
void orc_hoisted_term(void *h, const u64 *ext, const u64 *b, const u64 *evk, const u64 *mask, u64 g, int nq,
                      u64 *y, int accumulate) {
    Ctx *c = (Ctx *)h;
    const int N = c->N, K = c->nP, E = nq + K, full = c->nQ + c->nP;
    const int beta = (nq + c->alpha - 1) / c->alpha;
    const u64 M = 2 * (u64)N;
    std::vector<int> perm(N);
    for (int k = 0; k < N; k++) {
        u64 e = (2 * (u64)bitrev((unsigned)k, c->logN) + 1) * g % M;
        perm[k] = (int)bitrev((unsigned)((e - 1) / 2), c->logN);
    }
#pragma omp parallel for num_threads(c->threads) schedule(dynamic)
    for (int j = 0; j < E; j++) {
        const int pi = prime_of(c, j, nq);
        const u64 q = c->pr[pi].q;
        u64 P = 1;
        for (int k = 0; k < K; k++) P = mulmod(P, c->pr[c->nQ + k].q % q, q);
        for (int pol = 0; pol < 2; pol++) {
            u64 *o = y + ((size_t)pol * E + j) * N;
            for (int n = 0; n < N; n++) {
                u64 s = 0;
                for (int d = 0; d < beta; d++)
                    s = addmod(s, mulmod(ext[((size_t)d * E + j) * N + perm[n]],
                                         evk[(((size_t)d * 2 + pol) * full + pi) * N + n], q), q);
                if (pol == 0 && j < nq && b) s = addmod(s, mulmod(b[(size_t)j * N + perm[n]], P, q), q);
                if (mask) s = mulmod(s, mask[(size_t)j * N + n], q);
                o[n] = accumulate ? addmod(o[n], s, q) : s;
            }
        }
    }
}

// Division of an extended polynomial y [nq+K][N] (NTT) by P (drop_last = 0, result over nq limbs) or by
// P * q_{nq-1} (drop_last = 1, result over nq-1 limbs): out_j = (y_j - BConv_{D->q_j}(y_D)) * D^{-1}.
void orc_moddown_drop(void *h, const u64 *y, int nq, int drop_last, u64 *out) {
    Ctx *c = (Ctx *)h;
    const int N = c->N, K = c->nP, nq_out = drop_last ? nq - 1 : nq;
    std::vector<int> src, slot, dst;
    if (drop_last) {
        src.push_back(nq - 1);
        slot.push_back(nq - 1);
    }
    for (int k = 0; k < K; k++) {
        src.push_back(c->nQ + k);
        slot.push_back(nq + k);
    }
    std::vector<u64> dc(src.size() * (size_t)N);
    std::vector<const u64 *> ip;
    std::vector<u64 *> op;
#pragma omp parallel for num_threads(c->threads) schedule(dynamic)
    for (size_t i = 0; i < src.size(); i++) {
        memcpy(dc.data() + i * N, y + (size_t)slot[i] * N, sizeof(u64) * N);
        ntt_inv(c->pr[src[i]], dc.data() + i * N, N);
    }
    for (size_t i = 0; i < src.size(); i++) ip.push_back(dc.data() + i * N);
    for (int j = 0; j < nq_out; j++) {
        dst.push_back(j);
        op.push_back(out + (size_t)j * N);
    }
    BConv bc = make_bconv(c, src, dst);
    run_bconv(c, bc, ip.data(), op.data());
#pragma omp parallel for num_threads(c->threads) schedule(dynamic)
    for (int j = 0; j < nq_out; j++) {
        const u64 q = c->pr[j].q;
        ntt_fwd(c->pr[j], op[j], N);
        u64 D = 1;
        for (int s : src) D = mulmod(D, c->pr[s].q % q, q);
        const u64 dinv = invmod(D, q);
        const u64 *a = y + (size_t)j * N;
        for (int n = 0; n < N; n++) op[j][n] = mulmod(submod(a[n], op[j][n], q), dinv, q);
    }
}

// ---- encode / decode ---------------------------------------------------------------------
// slots: n = N/2 complex values (re, im interleaved).  Produces signed integer coefficients
// round(scale * coeff) as int64 (caller reduces per prime with orc_lift_i64).
static void bitrev_complex(double *re, double *im, int n) {
    for (int i = 1, j = 0; i < n; i++) {
        int bit = n >> 1;
        for (; j >= bit; bit >>= 1) j -= bit;
        j += bit;
        if (i < j) {
            std::swap(re[i], re[j]);
            std::swap(im[i], im[j]);
        }
    }
}
void orc_encode_coeffs(void *h, const double *slots, double scale, i64 *coeffs) {
    Ctx *c = (Ctx *)h;
    const int n = c->N / 2, M = 2 * c->N;
    std::vector<double> re(n), im(n);
    for (int i = 0; i < n; i++) {
        re[i] = slots[2 * i];
        im[i] = slots[2 * i + 1];
    }
    for (int len = n; len >= 2; len >>= 1) {
        int lenh = len >> 1, lenq = len << 2, gap = M / lenq;
        for (int i = 0; i < n; i += len)
            for (int j = 0; j < lenh; j++) {
                int idx = (lenq - (int)(c->rot_group[j] % (u64)lenq)) * gap;
                double ur = re[i + j] + re[i + j + lenh], ui = im[i + j] + im[i + j + lenh];
                double vr = re[i + j] - re[i + j + lenh], vi = im[i + j] - im[i + j + lenh];
                double kr = c->ksi_re[idx], ki = c->ksi_im[idx];
                re[i + j] = ur;
                im[i + j] = ui;
                re[i + j + lenh] = vr * kr - vi * ki;
                im[i + j + lenh] = vr * ki + vi * kr;
            }
    }
    bitrev_complex(re.data(), im.data(), n);
    for (int i = 0; i < n; i++) {
        coeffs[i] = (i64)llround(re[i] / (double)n * scale);
        coeffs[i + n] = (i64)llround(im[i] / (double)n * scale);
    }
}
// coefficient vector (doubles, already divided by the scale) -> slots
void orc_decode_coeffs(void *h, const double *coeffs, double *slots) {
    Ctx *c = (Ctx *)h;
    const int n = c->N / 2, M = 2 * c->N;
    std::vector<double> re(n), im(n);
    for (int i = 0; i < n; i++) {
        re[i] = coeffs[i];
        im[i] = coeffs[i + n];
    }
    bitrev_complex(re.data(), im.data(), n);
    for (int len = 2; len <= n; len <<= 1) {
        int lenh = len >> 1, lenq = len << 2, gap = M / lenq;
        for (int i = 0; i < n; i += len)
            for (int j = 0; j < lenh; j++) {
                int idx = (int)(c->rot_group[j] % (u64)lenq) * gap;
                double kr = c->ksi_re[idx], ki = c->ksi_im[idx];
                double xr = re[i + j + lenh], xi = im[i + j + lenh];
                double vr = xr * kr - xi * ki, vi = xr * ki + xi * kr;
                double ur = re[i + j], ui = im[i + j];
                re[i + j] = ur + vr;
                im[i + j] = ui + vi;
                re[i + j + lenh] = ur - vr;
                im[i + j + lenh] = ui - vi;
            }
    }
    for (int i = 0; i < n; i++) {
        slots[2 * i] = re[i];
        slots[2 * i + 1] = im[i];
    }
}
void orc_lift_i64(void *h, const i64 *v, int prime_idx, u64 *out) {
    Ctx *c = (Ctx *)h;
    const u64 q = c->pr[prime_idx].q;
    for (int i = 0; i < c->N; i++) {
        if (v[i] >= 0)
            out[i] = (u64)v[i] % q;
        else {
            u64 r = (u64)(-v[i]) % q;
            out[i] = r ? q - r : 0;
        }
    }
}
// centred CRT of limbs 0 (and 1 when two = 1), coefficient form, divided by scale.
void orc_crt_to_double(void *h, const u64 *l0, const u64 *l1, int two, double scale, double *out) {
    Ctx *c = (Ctx *)h;
    const u64 q0 = c->pr[0].q;
    if (!two) {
        for (int i = 0; i < c->N; i++) {
            u64 v = l0[i];
            out[i] = (v > q0 / 2 ? -(double)(q0 - v) : (double)v) / scale;
        }
        return;
    }
    const u64 q1 = c->pr[1].q;
    const u64 q0inv = invmod(q0 % q1, q1);
    const u128 Q = (u128)q0 * q1;
    for (int i = 0; i < c->N; i++) {
        // x = l0 + q0 * ((l1 - l0) * q0^{-1} mod q1)
        u64 d = submod(l1[i] % q1, l0[i] % q1, q1);
        u64 k = mulmod(d, q0inv, q1);
        u128 x = (u128)l0[i] + (u128)q0 * k;
        double v;
        if (x > Q / 2) {
            u128 y = Q - x;
            v = -((double)(u64)(y >> 64) * 18446744073709551616.0 + (double)(u64)y);
        } else
            v = (double)(u64)(x >> 64) * 18446744073709551616.0 + (double)(u64)x;
        out[i] = v / scale;
    }
}

}  // extern "C"

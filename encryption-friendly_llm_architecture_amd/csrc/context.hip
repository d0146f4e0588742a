// Context set-up: per-prime constants and twiddle tables, computed on the host once and kept
// resident in HBM (2 x 1 MiB per prime at N = 2^16).
#include <cstring>

#include "hemm_internal.hpp"

typedef unsigned __int128 u128;

u64 h_mulmod(u64 a, u64 b, u64 q) { return (u64)((u128)a * b % q); }
u64 h_powmod(u64 a, u64 e, u64 q) {
    u64 r = 1 % q;
    a %= q;
    while (e) {
        if (e & 1) r = h_mulmod(r, a, q);
        a = h_mulmod(a, a, q);
        e >>= 1;
    }
    return r;
}
u64 h_invmod(u64 a, u64 q) { return h_powmod(a % q, q - 2, q); }
static u64 h_shoup(u64 w, u64 q) { return (u64)(((u128)w << 64) / q); }

static bool h_is_prime(u64 n) {
    static const u64 bases[] = {2, 3, 5, 7, 11, 13, 17, 19, 23, 29, 31, 37};
    if (n < 2) return false;
    for (u64 p : bases) {
        if (n % p == 0) return n == p;
    }
    u64 d = n - 1;
    int s = 0;
    while ((d & 1) == 0) {
        d >>= 1;
        s++;
    }
    for (u64 a : bases) {
        u64 x = h_powmod(a, d, n);
        if (x == 1 || x == n - 1) continue;
        bool comp = true;
        for (int i = 1; i < s; i++) {
            x = h_mulmod(x, x, n);
            if (x == n - 1) {
                comp = false;
                break;
            }
        }
        if (comp) return false;
    }
    return true;
}

static unsigned bitrev(unsigned x, int bits) {
    unsigned r = 0;
    for (int i = 0; i < bits; i++) {
        r = (r << 1) | (x & 1);
        x >>= 1;
    }
    return r;
}

void hemm_primes_below_impl(int bits, int logN, int count, u64 *out) {
    const u64 m = 2ull << logN, top = 1ull << bits;
    u64 p = top - (top % m) + 1;
    while (p >= top) p -= m;
    int n = 0;
    while (n < count) {
        if (p < m) throw std::invalid_argument("not enough primes of that size");
        if (h_is_prime(p)) out[n++] = p;
        p -= m;
    }
}

LimbList limbs_default(const hemm_context *c, int nq, int with_p) {
    LimbList ll;
    memset(&ll, 0, sizeof(ll));
    int n = nq + (with_p ? c->nP : 0);
    for (int j = 0; j < n; j++) ll.idx[j] = (uint8_t)(j < nq ? j : c->nQ + (j - nq));
    return ll;
}

hemm_context *hemm_context_build(int logN, int nQ, int nP, const u64 *primes, int dnum) {
    if (logN < 6 || logN > 16) throw std::invalid_argument("log_n must be in [6, 16]");
    if (nQ < 1 || nP < 0 || nQ + nP > HEMM_MAX_PRIMES) throw std::invalid_argument("bad limb counts");
    if (dnum < 1 || dnum > nQ) throw std::invalid_argument("dnum must be in [1, n_q]");
    const int N = 1 << logN, T = nQ + nP;
    for (int i = 0; i < T; i++) {
        u64 q = primes[i];
        // Below 2^31 the one-step reductions of a 60-bit residue (or of a 128-bit product) to this prime would leave more
        // than the few multiples of q that their conditional subtractions remove.
        if (q >= (1ull << 61) || q < (1ull << 31) || (q - 1) % (2 * (u64)N) != 0 || !h_is_prime(q))
            throw std::invalid_argument("prime " + std::to_string(i) +
                                        " must be a prime in [2^31, 2^61) congruent to 1 mod 2N");
        for (int j = 0; j < i; j++)
            if (primes[j] == q) throw std::invalid_argument("primes must be distinct");
    }
    hemm_context *c = new hemm_context();
    HEMM_HIP(hipGetDevice(&c->device));
    c->logN = logN;
    c->N = N;
    c->nQ = nQ;
    c->nP = nP;
    c->dnum = dnum;
    c->alpha = (nQ + dnum - 1) / dnum;
    c->primes.assign(primes, primes + T);
    c->psi.resize(T);
    c->modq.resize(T);
    std::vector<u64> w((size_t)T * N * 2), iw((size_t)T * N * 2), ninv(T), ninv_s(T), im(T), im_s(T);
    std::vector<u64> pw(N), ipw(N);
    std::vector<double> fpc((size_t)T * 4);
    for (int i = 0; i < T; i++) {
        const u64 q = primes[i];
        u64 psi = 0;
        for (u64 g = 2;; g++) {
            u64 cnd = h_powmod(g, (q - 1) / (2 * (u64)N), q);
            if (h_powmod(cnd, (u64)N, q) == q - 1) {
                psi = cnd;
                break;
            }
        }
        c->psi[i] = psi;
        const u64 ipsi = h_invmod(psi, q);
        pw[0] = ipw[0] = 1;
        for (int j = 1; j < N; j++) {
            pw[j] = h_mulmod(pw[j - 1], psi, q);
            ipw[j] = h_mulmod(ipw[j - 1], ipsi, q);
        }
        u64 *wt = w.data() + (size_t)i * N * 2, *iwt = iw.data() + (size_t)i * N * 2;
        // Primes below 2^44 run the 2^16-point transform in double precision (exact: see ntt.hip); their
        // table is the N twiddles as doubles, packed into the first half of the prime's region (8 bytes per twiddle
        // instead of 16: the row passes read as many twiddle bytes as data, and the quotient w / q costs one multiply).
        const bool fp = (logN == 16) && (q >> 44) == 0;
        auto as_bits = [](double d) {
            u64 b;
            memcpy(&b, &d, 8);
            return b;
        };
        for (int j = 0; j < N; j++) {
            unsigned r = bitrev((unsigned)j, logN);
            if (fp) {
                wt[j] = as_bits((double)pw[r]);
                iwt[j] = as_bits((double)ipw[r]);
                wt[N + j] = iwt[N + j] = 0;
                continue;
            }
            wt[2 * j] = pw[r];
            wt[2 * j + 1] = h_shoup(pw[r], q);
            iwt[2 * j] = ipw[r];
            iwt[2 * j + 1] = h_shoup(ipw[r], q);
        }
        ninv[i] = h_invmod((u64)N, q);
        const bool small = (q >> 44) == 0;  // residues and products-by-parts are exact in double precision
        fpc[4 * i + 0] = small ? (double)q : 0.0;
        fpc[4 * i + 1] = small ? 1.0 / (double)q : 0.0;
        fpc[4 * i + 2] = (double)ninv[i];
        fpc[4 * i + 3] = (double)ninv[i] / (double)q;
        ninv_s[i] = h_shoup(ninv[i], q);
        im[i] = pw[N / 2];
        im_s[i] = h_shoup(im[i], q);
        ModQ m;
        m.q = q;
        m.k = 64 - (u32)__builtin_clzll(q);
        m.mu = (u64)((((u128)1) << (2 * m.k)) / q);
        m.pad = 0;
        m.mu3 = (m.k == 59 || m.k == 60) ? (u64)((((u128)1) << (2 * m.k + 3)) / q) : 0;
        m.r64 = (u64)((((u128)1) << 64) % q);
        c->modq[i] = m;
    }
    auto up = [&](const void *h, size_t bytes) -> void * {
        void *d = nullptr;
        HEMM_HIP(hipMalloc(&d, bytes));
        HEMM_HIP(hipMemcpy(d, h, bytes, hipMemcpyHostToDevice));
        return d;
    };
    c->key_off.assign(T + 1, 0);
    for (int i = 0; i < T; i++)
        c->key_off[i + 1] = c->key_off[i] + (fpc[4 * i] != 0.0 ? 3u : 4u);
    c->d_key_off = (u32 *)up(c->key_off.data(), c->key_off.size() * 4);
    c->d_w = (u64 *)up(w.data(), w.size() * 8);
    c->d_iw = (u64 *)up(iw.data(), iw.size() * 8);
    c->d_rw = c->d_irw = nullptr;
    if (logN == 16) {
        // per prime the same storage convention as the stage-ordered tables: 16-byte entries, or doubles packed into
        // the first half of the prime's region
        std::vector<u64> rw((size_t)T * N * 2, 0), irw((size_t)T * N * 2, 0);
        for (int i = 0; i < T; i++) {
            const bool fp = fpc[4 * i] != 0.0;
            const u64 *src[2] = {w.data() + (size_t)i * N * 2, iw.data() + (size_t)i * N * 2};
            u64 *dst[2] = {rw.data() + (size_t)i * N * 2, irw.data() + (size_t)i * N * 2};
            for (int dir = 0; dir < 2; dir++)
                for (u32 r = 0; r < 256; r++)
                    for (u32 l = 0; l < 4; l++)
                        for (u32 g = 0; g < (1u << l); g++)
                            for (u32 cc = 0; cc < 16; cc++) {
                                const size_t from = ((size_t)(16 * (256 + r) + cc) << l) + g;
                                const size_t to = ((size_t)r * 15 + (1u << l) - 1 + g) * 16 + cc;
                                if (fp) {
                                    dst[dir][to] = src[dir][from];
                                } else {
                                    dst[dir][2 * to] = src[dir][2 * from];
                                    dst[dir][2 * to + 1] = src[dir][2 * from + 1];
                                }
                            }
        }
        c->d_rw = (u64 *)up(rw.data(), rw.size() * 8);
        c->d_irw = (u64 *)up(irw.data(), irw.size() * 8);
    }
    c->d_ninv = (u64 *)up(ninv.data(), T * 8);
    c->d_ninv_s = (u64 *)up(ninv_s.data(), T * 8);
    c->d_imag = (u64 *)up(im.data(), T * 8);
    c->d_imag_s = (u64 *)up(im_s.data(), T * 8);
    c->d_modq = (ModQ *)up(c->modq.data(), T * sizeof(ModQ));
    c->d_fp = (double *)up(fpc.data(), fpc.size() * 8);
    c->d_scratch = nullptr;
    c->scratch_bytes = 0;
    memset(c->traffic, 0, sizeof(c->traffic));
    memset(c->launches, 0, sizeof(c->launches));
    return c;
}

void hemm_context_free(hemm_context *c) {
    if (!c) return;
    hipFree(c->d_key_off);
    hipFree(c->d_w);
    hipFree(c->d_iw);
    if (c->d_rw) hipFree(c->d_rw);
    if (c->d_irw) hipFree(c->d_irw);
    hipFree(c->d_ninv);
    hipFree(c->d_ninv_s);
    hipFree(c->d_imag);
    hipFree(c->d_imag_s);
    hipFree(c->d_modq);
    hipFree(c->d_fp);
    if (c->d_scratch) hipFree(c->d_scratch);
    for (auto &kv : c->d_desc) (void)hipFree(kv.second);
    if (c->aux) (void)hipStreamDestroy(c->aux);
    if (c->aux_fork) (void)hipEventDestroy(c->aux_fork);
    if (c->aux_join) (void)hipEventDestroy(c->aux_join);
    delete c;
}

// Device-side pieces shared by the hoisted key-switch kernels: the term descriptor, the NTT-domain index map
// of an automorphism, exact double-precision arithmetic for primes below 2^44, and the value of one output
// residue of a group of hoisted rotation terms.
#pragma once
#include "hemm_internal.hpp"

struct CstList {
    Cst c[HEMM_MAX_PRIMES];
};

struct RotTermDev {
    const u64 *ext;   // [beta][E][N] extended digits of the source a-polynomial
    const u64 *b;     // [nq][N] b-polynomial of the source (nullptr: none, single-source terms only)
    const u64 *evk;   // [dnum][2][nQ+K][N]; nullptr: a term without a key switch, mask * pt * P * (b, a) on the chain
                      // limbs with the a-polynomial [nq][N] in `ext`, always as it is (b may be premultiplied like any
                      // other b, or absent); single-source terms only; its mask needs nq limbs
    const u64 *mask;  // [E][N] plaintext over the extended basis, or nullptr
    u32 galois;
    u32 mask_shift;   // s > 0: mask (and mask2) are run tables [E][N >> s], one value per 2^s coefficients
    // optional second source rotated by the same Galois element with the same key (ext2 == nullptr: none):
    // the term is mask * rot(source) + mask2 * rot(source 2) and the key is read once for both
    const u64 *ext2, *b2, *mask2;
    // optional plaintext factor [E][N] of the whole term, read through its own automorphism (nullptr: none)
    const u64 *pt;
    u32 pt_galois;
    u32 flags;        // bit 0: evk is a compact key (see key_limb); bit 1 (single-source terms with a plain key only): ext
                      // already holds the digits of the rotated polynomial and is read as it is, only b is read through
                      // the automorphism
};
#define ROT_TERM_COMPACT_KEY 1u
#define ROT_TERM_EXT_ROTATED 2u

// Accesses to data that is touched once per launch (keys, masks, results): marked non-temporal so they do
// not push the rotation sources, which every output gathers from, out of the L2.
typedef u64 u64x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ ulonglong2 stream_load2(const u64 *p) {
    const u64x2 v = __builtin_nontemporal_load((const u64x2 *)p);
    return make_ulonglong2(v.x, v.y);
}
__device__ __forceinline__ u64 stream_load1(const u64 *p) { return __builtin_nontemporal_load(p); }
// mask residues of the pair (n, n+1) of limb j: streamed from a full mask, or one value of a run table (every
// lane of the workgroup reads the same one or two entries, which stay in cache).  A run table holds pairs
// (value, floor(value * 2^64 / q)): the second word lets integer limbs multiply by the value as by a constant.
__device__ __forceinline__ ulonglong2 load_mask2(const u64 *mask, const u32 shift, const int j, const u32 n, const int logN) {
    if (shift == 0) return stream_load2(mask + ((size_t)j << logN) + n);
    const u64 v = mask[(((size_t)j << (logN - shift)) + (n >> shift)) * 2];
    return make_ulonglong2(v, v);
}
// (value, Shoup companion) of the run that holds the pair (n, n+1)
__device__ __forceinline__ ulonglong2 load_mask_run(const u64 *mask, const u32 shift, const int j, const u32 n, const int logN) {
    return *(const ulonglong2 *)(mask + (((size_t)j << (logN - shift)) + (n >> shift)) * 2);
}
// x1 * w1 + x2 * w2 mod q for run-table constants, canonical
__device__ __forceinline__ u64 shoup_pair(u64 x1, const ulonglong2 w1, u64 x2, const ulonglong2 w2, u64 q) {
    const u64 z = mul_shoup_lazy_u(x1, w1.x, w1.y, q) + mul_shoup_lazy_u(x2, w2.x, w2.y, q);   // < 4q < 2^63
    return cond_sub_u(cond_sub_u(z, 2 * q), q);
}
// residues (n, n+1) of limb j of a plaintext read through the automorphism X -> X^g (an aligned pair stays an aligned
// pair, possibly swapped)
__device__ __forceinline__ ulonglong2 load_rotated2(const u64 *pt, const u32 g, const int j, const u32 n, const int logN) {
    const u32 np = g == 1u ? n : galois_index(n, g, logN);
    ulonglong2 v = *(const ulonglong2 *)(pt + ((size_t)j << logN) + (np & ~1u));
    if (np & 1u) {
        const u64 t = v.x;
        v.x = v.y;
        v.y = t;
    }
    return v;
}
__device__ __forceinline__ void stream_store2(u64 *p, u64 a, u64 b) {
    u64x2 v;
    v.x = a;
    v.y = b;
    __builtin_nontemporal_store(v, (u64x2 *)p);
}

// Exact arithmetic mod q in double precision for q < 2^44: a product is 6 FP64 operations (gfx950 issues one
// FP64 FMA per lane per clock; a 64-bit integer product plus its Barrett step is ~40 instructions).
#pragma clang fp contract(off)
struct FpMod {
    double q, qinv;
    // a * b mod q as a centred residue (|r| <= 0.54 q) for integers |a| < 2^48, |b| < 2^44
    __device__ __forceinline__ double mul(double a, double b) const {
        const double h = a * b;
        const double l = __builtin_fma(a, b, -h);
        const double c = __builtin_rint(h * qinv);
        return __builtin_fma(-c, q, h) + l;
    }
    __device__ __forceinline__ double reduce(double x) const { return __builtin_fma(-__builtin_rint(x * qinv), q, x); }
    __device__ __forceinline__ u64 canonical(double x) const {
        double r = reduce(x);
        r += r < 0.0 ? q : 0.0;
        return (u64)__double_as_longlong(r + 4503599627370496.0) & 0x000fffffffffffffull;
    }
};
__device__ __forceinline__ double u64_to_double(u64 v) {  // v < 2^52
    return __longlong_as_double((long long)(v | 0x4330000000000000ull)) - 4503599627370496.0;
}

// Evaluation keys come in two layouts.  Plain: [dnum][2][n_full][N] words.  Compact: every residue of a prime below
// 2^44 takes 6 bytes instead of 8 -- per (digit, polynomial) the limbs sit back to back, a limb of such a prime as
// N / 2 records of 12 bytes, one per residue pair (n, n+1): the two 32-bit low words, then the two 16-bit high
// halves in one word; every other limb as N words.  koff[prime] is the limb's offset and koff[n_full] the size of a
// (digit, polynomial) slice, both in units of 2N bytes.  A key is read once per launch and is most of what a key
// product moves: a quarter less of it for the double-precision limbs, in one 12-byte load per thread and stream
// (low and high parts in separate arrays, two loads per stream, ran 15 % slower than plain keys: the kernel is bound
// by the loads in flight, not by the bytes).
// (the layout is a property of the launch -- every term of a launch uses the same one -- and a template parameter of
// the kernels: with both forms behind a run-time test the mixed kernel spilled 24 registers)
//
// The double-precision path reads a key through a buffer resource: the key's base and the offset of the limb sit in scalar registers and a
// thread supplies only the 32-bit byte offset of its residue pair, shared by all key streams of the thread (with
// 64-bit addresses in vector registers every stream costs two registers and an add with carry per load): 70
// registers instead of 74, i.e. seven waves per SIMD instead of six.  The host checks that a key is below 4 GiB.
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t key_rsrc(const RotTermDev &T) {
    // raw buffer (stride 0), no range limit, 32-bit data format
    return __builtin_amdgcn_make_buffer_rsrc((void *)T.evk, 0, -1, 0x00020000);
}
// byte offset of limb `prime` of polynomial pol of digit d inside the key (keys are far below 4 GiB)
template <bool COMPACT>
__device__ __forceinline__ u32 key_limb(const u32 *__restrict__ koff, const int d, const int pol, const int prime,
                                        const int logN, const int n_full) {
    if (COMPACT) return (((u32)(d * 2 + pol) * koff[n_full] + koff[prime]) << (logN + 1));
    return ((u32)((d * 2 + pol) * n_full + prime)) << (logN + 3);
}
// residues (n, n+1) of a limb of any prime (compact keys: of a prime of 2^44 or more); streamed (non-temporal)
__device__ __forceinline__ ulonglong2 key_pair_u64(const __amdgpu_buffer_rsrc_t key, const u32 limb, const u32 n) {
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(key, n * 8u, limb, 2);
    return make_ulonglong2(((u64)v.y << 32) | v.x, ((u64)v.w << 32) | v.z);
}
// The integer path keeps plain pointers: it is short of scalar registers (106 of 102 usable with a resource per term,
// which spilled 18 vector registers), not of vector registers.
template <bool COMPACT>
__device__ __forceinline__ ulonglong2 key_pair_ptr(const RotTermDev &T, const u32 *__restrict__ koff, const int d,
                                                   const int pol, const int prime, const int logN, const int n_full,
                                                   const u32 n) {
    const char *limb = (const char *)T.evk + key_limb<COMPACT>(koff, d, pol, prime, logN, n_full);
    return stream_load2((const u64 *)limb + n);
}
typedef u32 u32x3 __attribute__((ext_vector_type(3), aligned(4)));

// One term with two masked sources under one key (integer path): residues (n, n+1) of limb j of
// <z, evk> + P (mask b + mask2 b2) with z_d = mask * x_d + mask2 * x2_d, canonical.  RUNS: the masks are run tables,
// i.e. constants with a Shoup companion: no wide product and no Barrett step for z_d; a plaintext factor of the term is
// then left to the caller, which multiplies the finished pair by it.
template <bool RUNS, bool COMPACT>
__device__ __forceinline__ void two_source_int(const RotTermDev &T, const u32 *__restrict__ koff, const ModQ m,
                                               const CstList &pmod, const int j,
                                               const int prime, const u32 n, const u32 base, const bool swap, int nq,
                                               int E, int beta, int n_full, int logN, int b_premultiplied,
                                               u64 (&rb)[2], u64 (&ra)[2]) {
    const size_t N = (size_t)1 << logN;
    ulonglong2 m1, m2;   // RUNS: (value, companion) of each mask; otherwise the mask residues of the pair
    if (RUNS) {
        m1 = load_mask_run(T.mask, T.mask_shift, j, n, logN);
        m2 = load_mask_run(T.mask2, T.mask_shift, j, n, logN);
    } else {
        m1 = load_mask2(T.mask, T.mask_shift, j, n, logN);
        m2 = load_mask2(T.mask2, T.mask_shift, j, n, logN);
        if (T.pt != nullptr) {
            const ulonglong2 pv = load_rotated2(T.pt, T.pt_galois, j, n, logN);
            m1.x = mulmod_u(m1.x, pv.x, m);
            m1.y = mulmod_u(m1.y, pv.y, m);
            m2.x = mulmod_u(m2.x, pv.x, m);
            m2.y = mulmod_u(m2.y, pv.y, m);
        }
    }
    u128_t pb[2] = {{0, 0}, {0, 0}}, pa[2] = {{0, 0}, {0, 0}};
    for (int d = 0; d < beta; d++) {
        ulonglong2 x1 = *(const ulonglong2 *)(T.ext + ((size_t)d * E + j) * N + base);
        ulonglong2 x2 = *(const ulonglong2 *)(T.ext2 + ((size_t)d * E + j) * N + base);
        if (swap) {
            u64 tmp = x1.x;
            x1.x = x1.y;
            x1.y = tmp;
            tmp = x2.x;
            x2.x = x2.y;
            x2.y = tmp;
        }
        u64 z0, z1;
        if (RUNS) {
            z0 = shoup_pair(x1.x, m1, x2.x, m2, m.q);
            z1 = shoup_pair(x1.y, m1, x2.y, m2, m.q);
        } else {
            u128_t t0 = mul64wide(m1.x, x1.x), t1 = mul64wide(m1.y, x1.y);
            add128(t0, mul64wide(m2.x, x2.x));
            add128(t1, mul64wide(m2.y, x2.y));
            z0 = barrett3_u(t0, m);
            z1 = barrett3_u(t1, m);
        }
        const ulonglong2 kb = key_pair_ptr<COMPACT>(T, koff, d, 0, prime, logN, n_full, n);
        const ulonglong2 ka = key_pair_ptr<COMPACT>(T, koff, d, 1, prime, logN, n_full, n);
        add128(pb[0], mul64wide(z0, kb.x));
        add128(pb[1], mul64wide(z1, kb.y));
        add128(pa[0], mul64wide(z0, ka.x));
        add128(pa[1], mul64wide(z1, ka.y));
    }
    if (beta <= 3) {   // at most 3 q^2: the short reduction applies
        rb[0] = barrett3_u(pb[0], m);
        rb[1] = barrett3_u(pb[1], m);
        ra[0] = barrett3_u(pa[0], m);
        ra[1] = barrett3_u(pa[1], m);
    } else {
        rb[0] = barrett128_u(pb[0], m);
        rb[1] = barrett128_u(pb[1], m);
        ra[0] = barrett128_u(pa[0], m);
        ra[1] = barrett128_u(pa[1], m);
    }
    if (j < nq) {
        ulonglong2 b1 = *(const ulonglong2 *)(T.b + (size_t)j * N + base);
        ulonglong2 b2 = *(const ulonglong2 *)(T.b2 + (size_t)j * N + base);
        if (swap) {
            u64 tmp = b1.x;
            b1.x = b1.y;
            b1.y = tmp;
            tmp = b2.x;
            b2.x = b2.y;
            b2.y = tmp;
        }
        if (!b_premultiplied) {
            b1.x = mul_shoup_u(b1.x, pmod.c[j].w, pmod.c[j].ws, m.q);
            b1.y = mul_shoup_u(b1.y, pmod.c[j].w, pmod.c[j].ws, m.q);
            b2.x = mul_shoup_u(b2.x, pmod.c[j].w, pmod.c[j].ws, m.q);
            b2.y = mul_shoup_u(b2.y, pmod.c[j].w, pmod.c[j].ws, m.q);
        }
        if (RUNS) {
            rb[0] = addmod_u(rb[0], shoup_pair(b1.x, m1, b2.x, m2, m.q), m.q);
            rb[1] = addmod_u(rb[1], shoup_pair(b1.y, m1, b2.y, m2, m.q), m.q);
        } else {
            u128_t t0 = mul64wide(m1.x, b1.x), t1 = mul64wide(m1.y, b1.y);
            add128(t0, mul64wide(m2.x, b2.x));
            add128(t1, mul64wide(m2.y, b2.y));
            rb[0] = addmod_u(rb[0], barrett3_u(t0, m), m.q);
            rb[1] = addmod_u(rb[1], barrett3_u(t1, m), m.q);
        }
    }
}

// Residues (n, n+1) of limb j of both polynomials of output o (integer path), canonical.
template <bool COMPACT>
__device__ __forceinline__ void hoisted_pair_int(const RotTermDev *__restrict__ terms,
                                                 const u32 *__restrict__ group_off, const u32 *__restrict__ koff,
                                                 const ModQ m, const CstList &pmod,
                                                 const int j, const int o, const int prime, const u32 n, int nq, int E,
                                                 int beta, int n_full, int logN, int b_premultiplied, u64 (&out_b)[2],
                                                 u64 (&out_a)[2]) {
    const size_t N = (size_t)1 << logN;
    u64 acc_b[2] = {0, 0}, acc_a[2] = {0, 0};
    u128_t lazy_b[2] = {{0, 0}, {0, 0}}, lazy_a[2] = {{0, 0}, {0, 0}};
    int pending = 0;
    for (u32 t = group_off[o]; t < group_off[o + 1]; t++) {
        const RotTermDev T = terms[t];
        // a term without a key lives on the chain limbs: its polynomials and its mask have nq limbs, nothing of it
        // is read for a special limb
        if (T.evk == nullptr && j >= nq) continue;
        const u32 np = galois_index(n, T.galois, logN);
        const u32 base = np & ~1u;
        const bool swap = (np & 1u) != 0;
        if (T.ext2 != nullptr) {
            // two masked sources under one key: z_d = mask * x_d + mask2 * x2_d, then one pass over the key
            u64 rb[2], ra[2];
            if (T.mask_shift != 0) {
                // run-table masks are constants: the plaintext factor of the term, if it has one, is common to both
                // sources and multiplies the finished pair once (same residues as masks multiplied by it beforehand)
                two_source_int<true, COMPACT>(T, koff, m, pmod, j, prime, n, base, swap, nq, E, beta, n_full, logN,
                                              b_premultiplied, rb, ra);
                if (T.pt != nullptr) {
                    const ulonglong2 pv = load_rotated2(T.pt, T.pt_galois, j, n, logN);
                    rb[0] = mulmod_u(rb[0], pv.x, m);
                    rb[1] = mulmod_u(rb[1], pv.y, m);
                    ra[0] = mulmod_u(ra[0], pv.x, m);
                    ra[1] = mulmod_u(ra[1], pv.y, m);
                }
            } else {
                two_source_int<false, COMPACT>(T, koff, m, pmod, j, prime, n, base, swap, nq, E, beta, n_full, logN,
                                               b_premultiplied, rb, ra);
            }
            acc_b[0] = addmod_u(acc_b[0], rb[0], m.q);
            acc_b[1] = addmod_u(acc_b[1], rb[1], m.q);
            acc_a[0] = addmod_u(acc_a[0], ra[0], m.q);
            acc_a[1] = addmod_u(acc_a[1], ra[1], m.q);
            continue;
        }
        u128_t sb[2] = {{0, 0}, {0, 0}}, sa[2] = {{0, 0}, {0, 0}};
        const bool keyless = T.evk == nullptr;
        const bool ext_as_is = !COMPACT && (T.flags & ROT_TERM_EXT_ROTATED) != 0;
        for (int d = 0; d < (keyless ? 0 : beta); d++) {
            ulonglong2 x = *(const ulonglong2 *)(T.ext + ((size_t)d * E + j) * N + (ext_as_is ? n : base));
            if (swap && !ext_as_is) {
                const u64 tmp = x.x;
                x.x = x.y;
                x.y = tmp;
            }
            const ulonglong2 kb = key_pair_ptr<COMPACT>(T, koff, d, 0, prime, logN, n_full, n);
            const ulonglong2 ka = key_pair_ptr<COMPACT>(T, koff, d, 1, prime, logN, n_full, n);
            add128(sb[0], mul64wide(x.x, kb.x));
            add128(sb[1], mul64wide(x.y, kb.y));
            add128(sa[0], mul64wide(x.x, ka.x));
            add128(sa[1], mul64wide(x.y, ka.y));
        }
        u64 rb[2], ra[2];
        if (beta <= 3) {
            rb[0] = barrett3_u(sb[0], m);
            rb[1] = barrett3_u(sb[1], m);
            ra[0] = barrett3_u(sa[0], m);
            ra[1] = barrett3_u(sa[1], m);
        } else {
            rb[0] = barrett128_u(sb[0], m);
            rb[1] = barrett128_u(sb[1], m);
            ra[0] = barrett128_u(sa[0], m);
            ra[1] = barrett128_u(sa[1], m);
        }
        if (j < nq && T.b != nullptr) {
            ulonglong2 bv = *(const ulonglong2 *)(T.b + (size_t)j * N + base);
            if (swap) {
                const u64 tmp = bv.x;
                bv.x = bv.y;
                bv.y = tmp;
            }
            if (!b_premultiplied) {
                bv.x = mul_shoup_u(bv.x, pmod.c[j].w, pmod.c[j].ws, m.q);
                bv.y = mul_shoup_u(bv.y, pmod.c[j].w, pmod.c[j].ws, m.q);
            }
            rb[0] = addmod_u(rb[0], bv.x, m.q);
            rb[1] = addmod_u(rb[1], bv.y, m.q);
        }
        if (keyless) {   // the a-polynomial enters as it is (times P): no key product above (j < nq here)
            ulonglong2 av = *(const ulonglong2 *)(T.ext + (size_t)j * N + base);
            if (swap) {
                const u64 tmp = av.x;
                av.x = av.y;
                av.y = tmp;
            }
            av.x = mul_shoup_u(av.x, pmod.c[j].w, pmod.c[j].ws, m.q);   // never premultiplied, whatever b is
            av.y = mul_shoup_u(av.y, pmod.c[j].w, pmod.c[j].ws, m.q);
            ra[0] = av.x;
            ra[1] = av.y;
        }
        if (T.mask != nullptr || T.pt != nullptr) {
            ulonglong2 mk = T.mask != nullptr ? load_mask2(T.mask, T.mask_shift, j, n, logN) : make_ulonglong2(1, 1);
            if (T.pt != nullptr) {
                const ulonglong2 pv = load_rotated2(T.pt, T.pt_galois, j, n, logN);
                if (T.mask != nullptr) {
                    mk.x = mulmod_u(mk.x, pv.x, m);
                    mk.y = mulmod_u(mk.y, pv.y, m);
                } else {
                    mk = pv;
                }
            }
            add128(lazy_b[0], mul64wide(rb[0], mk.x));
            add128(lazy_b[1], mul64wide(rb[1], mk.y));
            add128(lazy_a[0], mul64wide(ra[0], mk.x));
            add128(lazy_a[1], mul64wide(ra[1], mk.y));
            if (++pending == 4) {
                for (int i = 0; i < 2; i++) {
                    acc_b[i] = addmod_u(acc_b[i], barrett128_u(lazy_b[i], m), m.q);
                    acc_a[i] = addmod_u(acc_a[i], barrett128_u(lazy_a[i], m), m.q);
                    lazy_b[i].lo = lazy_b[i].hi = lazy_a[i].lo = lazy_a[i].hi = 0;
                }
                pending = 0;
            }
        } else {
            for (int i = 0; i < 2; i++) {
                acc_b[i] = addmod_u(acc_b[i], rb[i], m.q);
                acc_a[i] = addmod_u(acc_a[i], ra[i], m.q);
            }
        }
    }
    if (pending) {
        for (int i = 0; i < 2; i++) {
            acc_b[i] = addmod_u(acc_b[i], barrett128_u(lazy_b[i], m), m.q);
            acc_a[i] = addmod_u(acc_a[i], barrett128_u(lazy_a[i], m), m.q);
        }
    }
    out_b[0] = acc_b[0];
    out_b[1] = acc_b[1];
    out_a[0] = acc_a[0];
    out_a[1] = acc_a[1];
}

// The same sums in double precision for primes below 2^44 (exact, see the transform kernels): a product
// mod q is 6 FP64 operations instead of ~40 integer ones for a wide product plus its Barrett step.
struct D2 {
    double x, y;
};
__device__ __forceinline__ D2 to_d2(const ulonglong2 v) {
    D2 r;
    r.x = __longlong_as_double((long long)(v.x | 0x4330000000000000ull)) - 4503599627370496.0;
    r.y = __longlong_as_double((long long)(v.y | 0x4330000000000000ull)) - 4503599627370496.0;
    return r;
}
__device__ __forceinline__ D2 gather_d2(const u64 *p, const bool swap) {
    ulonglong2 v = *(const ulonglong2 *)p;
    if (swap) {
        const u64 tmp = v.x;
        v.x = v.y;
        v.y = tmp;
    }
    return to_d2(v);
}
// residues (n, n+1) of a key limb of a prime below 2^44 as doubles
template <bool COMPACT>
__device__ __forceinline__ D2 key_pair_fp(const __amdgpu_buffer_rsrc_t key, const u32 limb, const u32 n) {
    if (!COMPACT) return to_d2(key_pair_u64(key, limb, n));
    const u32x3 v = __builtin_amdgcn_raw_buffer_load_b96(key, n * 6u, limb, 2);   // one 12-byte load
    D2 r;
    r.x = __hiloint2double((int)((v.z & 0xffffu) | 0x43300000u), (int)v.x) - 4503599627370496.0;
    r.y = __hiloint2double((int)((v.z >> 16) | 0x43300000u), (int)v.y) - 4503599627370496.0;
    return r;
}
#pragma clang fp contract(off)
// The same residues in double precision (primes below 2^44); out_* are unreduced centred doubles.
template <bool COMPACT>
__device__ __forceinline__ void hoisted_pair_fp(const RotTermDev *__restrict__ terms,
                                                const u32 *__restrict__ group_off, const u32 *__restrict__ koff,
                                                const FpMod f, const double p_mod_q,
                                                const int j, const int o, const int prime, const u32 n, int nq, int E,
                                                int beta, int n_full, int logN, int b_premultiplied, double (&out_b)[2],
                                                double (&out_a)[2]) {
    const size_t N = (size_t)1 << logN;
    double acc_b0 = 0, acc_b1 = 0, acc_a0 = 0, acc_a1 = 0;
    int since = 0;
    for (u32 t = group_off[o]; t < group_off[o + 1]; t++) {
        const RotTermDev T = terms[t];
        if (T.evk == nullptr && j >= nq) continue;   // a term without a key: chain limbs only, mask included
        const __amdgpu_buffer_rsrc_t kr = key_rsrc(T);
        const u32 np = galois_index(n, T.galois, logN);
        const u32 base = np & ~1u;
        const bool swap = (np & 1u) != 0;
        double sb0 = 0, sb1 = 0, sa0 = 0, sa1 = 0;
        if (T.ext2 != nullptr) {
            D2 m1 = to_d2(load_mask2(T.mask, T.mask_shift, j, n, logN));
            D2 m2 = to_d2(load_mask2(T.mask2, T.mask_shift, j, n, logN));
            if (T.pt != nullptr) {
                const D2 pv = to_d2(load_rotated2(T.pt, T.pt_galois, j, n, logN));
                m1.x = f.mul(m1.x, pv.x);
                m1.y = f.mul(m1.y, pv.y);
                m2.x = f.mul(m2.x, pv.x);
                m2.y = f.mul(m2.y, pv.y);
            }
            for (int d = 0; d < beta; d++) {
                const D2 x1 = gather_d2(T.ext + ((size_t)d * E + j) * N + base, swap);
                const D2 x2 = gather_d2(T.ext2 + ((size_t)d * E + j) * N + base, swap);
                const double z0 = f.mul(m1.x, x1.x) + f.mul(m2.x, x2.x);
                const double z1 = f.mul(m1.y, x1.y) + f.mul(m2.y, x2.y);
                const D2 kb = key_pair_fp<COMPACT>(kr, key_limb<COMPACT>(koff, d, 0, prime, logN, n_full), n);
                const D2 ka = key_pair_fp<COMPACT>(kr, key_limb<COMPACT>(koff, d, 1, prime, logN, n_full), n);
                sb0 += f.mul(z0, kb.x);
                sb1 += f.mul(z1, kb.y);
                sa0 += f.mul(z0, ka.x);
                sa1 += f.mul(z1, ka.y);
            }
            if (j < nq) {
                D2 b1 = gather_d2(T.b + (size_t)j * N + base, swap);
                D2 b2 = gather_d2(T.b2 + (size_t)j * N + base, swap);
                if (!b_premultiplied) {
                    b1.x = f.mul(b1.x, p_mod_q);
                    b1.y = f.mul(b1.y, p_mod_q);
                    b2.x = f.mul(b2.x, p_mod_q);
                    b2.y = f.mul(b2.y, p_mod_q);
                }
                sb0 += f.mul(m1.x, b1.x) + f.mul(m2.x, b2.x);
                sb1 += f.mul(m1.y, b1.y) + f.mul(m2.y, b2.y);
            }
        } else {
            const bool keyless = T.evk == nullptr;
            const bool ext_as_is = !COMPACT && (T.flags & ROT_TERM_EXT_ROTATED) != 0;
            for (int d = 0; d < (keyless ? 0 : beta); d++) {
                const D2 x = gather_d2(T.ext + ((size_t)d * E + j) * N + (ext_as_is ? n : base), swap && !ext_as_is);
                const D2 kb = key_pair_fp<COMPACT>(kr, key_limb<COMPACT>(koff, d, 0, prime, logN, n_full), n);
                const D2 ka = key_pair_fp<COMPACT>(kr, key_limb<COMPACT>(koff, d, 1, prime, logN, n_full), n);
                sb0 += f.mul(x.x, kb.x);
                sb1 += f.mul(x.y, kb.y);
                sa0 += f.mul(x.x, ka.x);
                sa1 += f.mul(x.y, ka.y);
            }
            if (j < nq && T.b != nullptr) {
                D2 bv = gather_d2(T.b + (size_t)j * N + base, swap);
                if (!b_premultiplied) {
                    bv.x = f.mul(bv.x, p_mod_q);
                    bv.y = f.mul(bv.y, p_mod_q);
                }
                sb0 += bv.x;
                sb1 += bv.y;
            }
            if (keyless) {   // the a-polynomial enters as it is (times P); j < nq here
                D2 av = gather_d2(T.ext + (size_t)j * N + base, swap);
                av.x = f.mul(av.x, p_mod_q);   // never premultiplied, whatever b is
                av.y = f.mul(av.y, p_mod_q);
                sa0 = av.x;
                sa1 = av.y;
            }
            if (T.mask != nullptr) {
                const D2 mk = to_d2(load_mask2(T.mask, T.mask_shift, j, n, logN));
                sb0 = f.mul(sb0, mk.x);
                sb1 = f.mul(sb1, mk.y);
                sa0 = f.mul(sa0, mk.x);
                sa1 = f.mul(sa1, mk.y);
            }
            if (T.pt != nullptr) {
                const D2 pv = to_d2(load_rotated2(T.pt, T.pt_galois, j, n, logN));
                sb0 = f.mul(sb0, pv.x);
                sb1 = f.mul(sb1, pv.y);
                sa0 = f.mul(sa0, pv.x);
                sa1 = f.mul(sa1, pv.y);
            }
        }
        acc_b0 += sb0;
        acc_b1 += sb1;
        acc_a0 += sa0;
        acc_a1 += sa1;
        if (++since == 8) {  // a term adds at most (beta + 2) * 0.54 q: keep the running sums far below 2^52
            acc_b0 = f.reduce(acc_b0);
            acc_b1 = f.reduce(acc_b1);
            acc_a0 = f.reduce(acc_a0);
            acc_a1 = f.reduce(acc_a1);
            since = 0;
        }
    }
    out_b[0] = acc_b0;
    out_b[1] = acc_b1;
    out_a[0] = acc_a0;
    out_a[1] = acc_a1;
}


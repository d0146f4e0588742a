// Device-side modular arithmetic for RNS primes below 2^61 on gfx950.
//
// gfx950 has no 64x64->128 multiplier: every 64-bit product below is assembled by the
// compiler from 32-bit v_mad_u64_u32 / v_mul_hi_u32 pieces, so the code is written to keep
// the number of wide products per modular multiplication minimal:
//   * constant multiplicands (NTT twiddles, 1/N, P^-1, q_l^-1, basis-conversion factors) carry a
//     precomputed Shoup quotient floor(w * 2^64 / q): one high product + two low products;
//   * data x data products are kept as 128-bit values, summed lazily, and reduced once with a
//     Barrett step sized to the prime's bit length.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef unsigned long long u64;
typedef unsigned int u32;

struct u128_t {
    u64 lo, hi;
};

__device__ __forceinline__ u128_t mul64wide(u64 a, u64 b) {
    u128_t r;
    r.lo = a * b;
    r.hi = __umul64hi(a, b);
    return r;
}
__device__ __forceinline__ void add128(u128_t &acc, const u128_t &x) {
    u64 lo = acc.lo + x.lo;
    acc.hi += x.hi + (lo < acc.lo ? 1ull : 0ull);
    acc.lo = lo;
}

// Per-prime constants, passed to kernels by value or read from a small device table.
struct ModQ {
    u64 q;     // the prime
    u64 mu;    // floor(2^(2k) / q), k = bit length of q
    u32 k;     // bit length of q (q < 2^k, k <= 61)
    u32 pad;
    u64 mu3;   // floor(2^(2k+3) / q) for k = 59 or 60, else 0 (barrett_tight)
    u64 r64;   // 2^64 mod q
};

// x * w mod q for a constant w with ws = floor(w * 2^64 / q); result in [0, 2q).
__device__ __forceinline__ u64 mul_shoup_lazy(u64 x, u64 w, u64 ws, u64 q) {
    return x * w - __umul64hi(x, ws) * q;
}
__device__ __forceinline__ u64 mul_shoup(u64 x, u64 w, u64 ws, u64 q) {
    u64 r = mul_shoup_lazy(x, w, ws, q);
    return r >= q ? r - q : r;
}

// x * w - hi' * q with the quotient estimate hi' taken from three of the four 32-bit partial products of x * ws:
// hi' = xh wh + (xh wl >> 32) + (xl wh >> 32) is at most 2 below floor(x ws / 2^64), so the result lies in [0, 4q)
// instead of [0, 2q) for any 64-bit x.  One multiply-add and the carry chain of the exact high product are saved.
__device__ __forceinline__ u64 mul_shoup_lazy4(u64 x, u64 w, u64 ws, u64 q) {
    const u32 xl = (u32)x, xh = (u32)(x >> 32), sl = (u32)ws, sh = (u32)(ws >> 32);
    const u64 hi = ((u64)xh * sh + __umulhi(xh, sl)) + __umulhi(xl, sh);
    // x * w - hi * q = x * w + hi * (2^64 - q) mod 2^64 as one chain of 32-bit multiply-adds: the two low products
    // accumulate in one 64-bit register (a carry out of bit 64 is dropped, as it should be), the four cross products
    // only feed the high word; no 64-bit subtraction and none of its carry hazards
    const u64 nq = 0 - q;
    const u32 hl = (u32)hi, hh = (u32)(hi >> 32), wl = (u32)w, wh = (u32)(w >> 32), nl = (u32)nq, nh = (u32)(nq >> 32);
    const u64 t = (u64)hl * nl + (u64)xl * wl;
    const u32 top = (u32)(t >> 32) + xl * wh + xh * wl + hl * nh + hh * nl;
    return ((u64)top << 32) | (u32)t;
}
// v < 32q (q < 2^59) to [0, q)
__device__ __forceinline__ u64 reduce_below_32q(u64 v, const u64 q) {
#pragma unroll
    for (int m = 16; m >= 1; m >>= 1)
        if (v >= (u64)m * q) v -= (u64)m * q;
    return v;
}
// Barrett reduction of a 128-bit value T < 6 * 2^(2k) to [0, q).
__device__ __forceinline__ u64 barrett128(u128_t t, const ModQ &m) {
    const u32 k = m.k;
    u64 t1 = (t.hi << (65 - k)) | (t.lo >> (k - 1));
    u128_t p = mul64wide(t1, m.mu);
    u64 qhat = (p.hi << (63 - k)) | (p.lo >> (k + 1));
    u64 r = t.lo - qhat * m.q;
    const u64 q = m.q;
    if (r >= 4 * q) r -= 4 * q;
    if (r >= 2 * q) r -= 2 * q;
    if (r >= q) r -= q;
    return r;
}
// Barrett reduction of T < 3 * 2^(2k) to [0, q) for primes of 59 or 60 bits (m.mu3 != 0) with the three bits longer
// constant: qhat = floor(floor(T / 2^(k-2)) * mu3 / 2^(k+5)) misses floor(T / q) by less than
// T / 2^(2k+3) + 2^(k-2) / q + 1 < 3/8 + 1/2 + 1, i.e. by at most 1: only the high half of one product and a single
// correction, against a full product and three corrections in barrett128.
__device__ __forceinline__ u64 barrett_tight(u128_t t, const ModQ &m) {
    const u32 k = m.k;
    const u64 t1 = (t.hi << (66 - k)) | (t.lo >> (k - 2));
    const u64 qhat = __umul64hi(t1, m.mu3) >> (k - 59);
    const u64 r = t.lo - qhat * m.q;
    return r >= m.q ? r - m.q : r;
}
// T < 3 * 2^(2k)
__device__ __forceinline__ u64 barrett3(u128_t t, const ModQ &m) {
    return m.mu3 != 0 ? barrett_tight(t, m) : barrett128(t, m);
}
__device__ __forceinline__ u64 mulmod(u64 a, u64 b, const ModQ &m) {
    return barrett3(mul64wide(a, b), m);
}
// reduce an arbitrary 64-bit value
__device__ __forceinline__ u64 reduce64(u64 a, const ModQ &m) {
    u128_t t;
    t.lo = a;
    t.hi = 0;
    return barrett128(t, m);
}
// Lazy dot product sum_i v_i * h_i of up to 8 residues v_i < 2^60 with constants h_i < 2^60 (a target residue of a
// fast basis conversion).  The 32-bit halves are multiplied into three 64-bit accumulators -- s0 (weight 1, with a
// carry count), s1 (weight 2^32: 16 terms below 2^60 cannot overflow), s2 (weight 2^64) -- four multiply-adds per
// term and no reduction until the end, against a Shoup product with its own quotient per term.
struct Dot3 {
    u64 s0, s1, s2;
    u32 c;
};
__device__ __forceinline__ void dot3_clear(Dot3 &d) {
    d.s0 = d.s1 = d.s2 = 0;
    d.c = 0;
}
__device__ __forceinline__ void dot3_add(Dot3 &d, const u64 v, const u64 h) {
    const u32 vl = (u32)v, vh = (u32)(v >> 32), hl = (u32)h, hh = (u32)(h >> 32);
    const u64 p = (u64)vl * hl;
    d.s0 += p;
    d.c += d.s0 < p ? 1u : 0u;
    d.s1 += (u64)vl * hh;
    d.s1 += (u64)vh * hl;
    d.s2 += (u64)vh * hh;
}
// the sum as a 128-bit value (below 8 * 2^(60 + k) for constants below 2^k)
__device__ __forceinline__ u128_t dot3_value(const Dot3 &d) {
    u128_t t;
    const u64 mid = d.s1 << 32;
    t.lo = d.s0 + mid;
    t.hi = d.s2 + d.c + (d.s1 >> 32) + (t.lo < mid ? 1ull : 0ull);
    return t;
}
// ... reduced to [0, q): the high word (below 2^(k-1)) is folded with 2^64 mod q, which leaves a value below
// 2^(2k-1) + 2^64 < 6 * 2^(2k) for k >= 31, then one Barrett step
__device__ __forceinline__ u64 dot3_reduce(const Dot3 &d, const ModQ &m) {
    const u128_t t = dot3_value(d);
    u128_t u = mul64wide(t.hi, m.r64);
    const u64 lo = u.lo + t.lo;
    u.hi += lo < t.lo ? 1ull : 0ull;
    u.lo = lo;
    return barrett128(u, m);
}
__device__ __forceinline__ u64 addmod(u64 a, u64 b, u64 q) {
    u64 s = a + b;
    return s >= q ? s - q : s;
}
__device__ __forceinline__ u64 submod(u64 a, u64 b, u64 q) { return a >= b ? a - b : a + q - b; }

// ---- the same reductions for a modulus that is uniform over the wavefront (the prime of a workgroup's limb) ----------
// A 64-bit subtraction is a borrow chain of two instructions with a wait state between them on gfx950, an addition is one
// instruction: a value is reduced by ADDING 2^64 - m, kept in scalar registers where the compiler cannot see through it
// and turn the sum back into a subtraction, and selecting.  Same values as the forms above.
__device__ __forceinline__ u64 neg_uniform(u64 m) {
    u64 n = 0 - m;
    asm("" : "+s"(n));
    return n;
}
// u >= m ? u - m : u
__device__ __forceinline__ u64 cond_sub_u(u64 u, const u64 m) {
    u64 t = u + neg_uniform(m);
    asm("" : "+v"(t));
    return u >= m ? t : u;
}
__device__ __forceinline__ u64 mul_shoup_lazy_u(u64 x, u64 w, u64 ws, u64 q) {
    return x * w + __umul64hi(x, ws) * neg_uniform(q);
}
__device__ __forceinline__ u64 mul_shoup_u(u64 x, u64 w, u64 ws, u64 q) {
    return cond_sub_u(mul_shoup_lazy_u(x, w, ws, q), q);
}
__device__ __forceinline__ u64 barrett128_u(u128_t t, const ModQ &m) {
    const u32 k = m.k;
    const u64 t1 = (t.hi << (65 - k)) | (t.lo >> (k - 1));
    const u128_t p = mul64wide(t1, m.mu);
    const u64 qhat = (p.hi << (63 - k)) | (p.lo >> (k + 1));
    const u64 q = m.q;
    const u64 r = t.lo + qhat * neg_uniform(q);
    return cond_sub_u(cond_sub_u(cond_sub_u(r, 4 * q), 2 * q), q);
}
__device__ __forceinline__ u64 barrett_tight_u(u128_t t, const ModQ &m) {
    const u32 k = m.k;
    const u64 t1 = (t.hi << (66 - k)) | (t.lo >> (k - 2));
    const u64 qhat = __umul64hi(t1, m.mu3) >> (k - 59);
    return cond_sub_u(t.lo + qhat * neg_uniform(m.q), m.q);
}
__device__ __forceinline__ u64 barrett3_u(u128_t t, const ModQ &m) {
    return m.mu3 != 0 ? barrett_tight_u(t, m) : barrett128_u(t, m);
}
__device__ __forceinline__ u64 mulmod_u(u64 a, u64 b, const ModQ &m) { return barrett3_u(mul64wide(a, b), m); }
__device__ __forceinline__ u64 addmod_u(u64 a, u64 b, u64 q) { return cond_sub_u(a + b, q); }
__device__ __forceinline__ u64 negmod(u64 a, u64 q) { return a ? q - a : 0; }

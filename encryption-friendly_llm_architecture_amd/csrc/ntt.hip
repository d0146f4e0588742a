// Batched negacyclic NTT / INTT over RNS primes < 2^61 for gfx950.
//
// Forward: merged-twiddle Cooley-Tukey, natural order in, bit-reversed order out
//   out[k] = sum_j a[j] psi^{(2 bitrev(k)+1) j};  inverse: Gentleman-Sande with the 1/N factor.
// Twiddle table per prime: tw[i] = (psi^bitrev(i), floor(that * 2^64 / q)) as one 16-byte entry.
//
// N = 2^16 does not fit a CU's LDS (512 KiB per limb), so a transform is two launches over the
// 256 x 256 view  index = r*256 + c:
//   forward pass 1: stages 0..7  act down columns  (butterfly distance >= 256)
//   forward pass 2: stages 8..15 act inside rows   (distance <= 128)
// and mirrored for the inverse.  Each workgroup (256 threads = 4 wavefronts) owns a 16-column
// (or 16-row) slab; a thread keeps 16 residues in registers, runs a radix-16 block (4 stages)
// on them, swaps through LDS once and runs the second radix-16 block.  All global accesses
// are 128-byte row segments shared by 16 adjacent lanes.
//
// Other sizes (2^6 .. 2^15, used by the small-parameter tests) run a plain LDS kernel with the
// same butterfly network, so residues are identical for every N.
#include <algorithm>
#include <cstring>

#include "hemm_internal.hpp"

namespace {
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
// Column passes address a limb through a buffer resource: the limb's base sits in scalar registers, the slab row
// (a step of 2 KiB or 32 KiB) goes into the scalar offset of each access and a thread supplies one 32-bit byte offset
// for all of its 16 accesses -- with 64-bit addresses in vector registers every access costs an add with carry.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t limb_rsrc(const void *p) {
    return __builtin_amdgcn_make_buffer_rsrc((void *)p, 0, -1, 0x00020000);   // raw, no range limit, 32-bit format
}
template <class E>
__device__ __forceinline__ E buf_load(const __amdgpu_buffer_rsrc_t r, const u32 voff, const u32 soff) {
    const u32x2 w = __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 0);
    const u64 u = ((u64)w.y << 32) | w.x;
    E v;
    __builtin_memcpy(&v, &u, 8);
    return v;
}
template <class E>
__device__ __forceinline__ void buf_store(const __amdgpu_buffer_rsrc_t r, const u32 voff, const u32 soff, const E v) {
    u64 u;
    __builtin_memcpy(&u, &v, 8);
    u32x2 w;
    w.x = (u32)u;
    w.y = (u32)(u >> 32);
    __builtin_amdgcn_raw_buffer_store_b64(w, r, voff, soff, 0);
}

struct __align__(16) Tw {
    u64 w, ws;
};

// Lazy butterflies (q < 2^61, so 8q < 2^64): forward values stay in [0, 8q), inverse values in [0, 4q); q4 = 4q.
// u -= 4q when u >= 4q, written as an addition of -4q and a select: no borrow chain
__device__ __forceinline__ u64 csub(u64 u, const u64 m, const u64 neg_m) {
    u64 t = u + neg_m;
    asm("" : "+v"(t));          // keeps the compiler from turning this back into a subtraction of a selected 0 / m
    return u >= m ? t : u;
}
// 2^64 - m as a value the compiler cannot see through (it would turn x + (2^64 - m) back into a subtraction)
__device__ __forceinline__ u64 opaque_neg(u64 m) {
    u64 n = 0 - m;
    asm("" : "+s"(n));
    return n;
}
__device__ __forceinline__ void ct_bfly(u64 &x, u64 &y, const Tw tw, const u64 q, const u64 q4, const u64 nq4) {
    const u64 u = csub(x, q4, nq4);                        // < 4q
    const u64 v = mul_shoup_lazy4(y, tw.w, tw.ws, q);      // < 4q
    x = u + v;
    y = u - v + q4;
}
__device__ __forceinline__ void gs_bfly(u64 &x, u64 &y, const Tw tw, const u64 q, const u64 q4, const u64 nq4) {
    const u64 u = x, v = y;                                // < 4q each
    x = csub(u + v, q4, nq4);
    y = mul_shoup_lazy4(u - v + q4, tw.w, tw.ws, q);
}

// ------------------------------------------------------------------------------------------
// generic LDS kernel: tile [R rows][CW cols], global index = r*rowstride + c0 + cc
// ------------------------------------------------------------------------------------------
struct GenericPass {
    int logN;
    int R, CW;          // tile shape (powers of two)
    int rowstride;      // distance between tile rows in the limb
    int s_begin, s_end; // forward: stages s_begin..s_end-1 ascending; inverse: descending
    int tiles_per_limb;
    int first, last;    // first / last pass of the transform
};

template <bool INV>
__global__ __launch_bounds__(256) void ntt_generic_kernel(u64 *__restrict__ data, const Tw *__restrict__ tw_all,
                                                          const ModQ *__restrict__ modq,
                                                          const u64 *__restrict__ ninv, const u64 *__restrict__ ninv_s,
                                                          LimbList ll, LimbList sl, int n_limbs, size_t poly_stride,
                                                          GenericPass gp) {
    extern __shared__ u64 lds[];
    const int N = 1 << gp.logN;
    const int limb = blockIdx.y % n_limbs, poly = blockIdx.y / n_limbs;
    const int prime = ll.idx[limb];
    const Tw *tw = tw_all + (size_t)prime * N;
    const u64 q = modq[prime].q, q2 = 2 * q, q4 = 4 * q, nq4 = opaque_neg(q4);
    u64 *base = data + (size_t)poly * poly_stride + (size_t)sl.idx[limb] * N;
    const int tile = blockIdx.x;
    // tile origin: strided pass tiles walk the columns; contiguous pass tiles walk the limb
    const int c0 = (gp.rowstride == 1) ? tile * gp.R * gp.CW : tile * gp.CW;
    const int elems = gp.R * gp.CW;
    for (int e = threadIdx.x; e < elems; e += blockDim.x) {
        int r = e / gp.CW, cc = e % gp.CW;
        lds[e] = base[(size_t)r * gp.rowstride + c0 + cc];
    }
    __syncthreads();
    const int half = elems / 2;
    if (!INV) {
        for (int s = gp.s_begin; s < gp.s_end; s++) {
            const int t = N >> (s + 1);
            const int tr = t / gp.rowstride;  // row distance inside the tile
            for (int b = threadIdx.x; b < half; b += blockDim.x) {
                int cc = b % gp.CW, rb = b / gp.CW;
                int r = (rb / tr) * 2 * tr + rb % tr;
                int i = r * gp.CW + cc, j = i + tr * gp.CW;
                int gidx = r * gp.rowstride + c0 + cc;
                Tw w = tw[(1 << s) + (gidx / (2 * t))];
                u64 x = lds[i], y = lds[j];
                ct_bfly(x, y, w, q, q4, nq4);
                lds[i] = x;
                lds[j] = y;
            }
            __syncthreads();
        }
    } else {
        for (int s = gp.s_begin - 1; s >= gp.s_end; s--) {
            const int t = N >> (s + 1);
            const int tr = t / gp.rowstride;
            for (int b = threadIdx.x; b < half; b += blockDim.x) {
                int cc = b % gp.CW, rb = b / gp.CW;
                int r = (rb / tr) * 2 * tr + rb % tr;
                int i = r * gp.CW + cc, j = i + tr * gp.CW;
                int gidx = r * gp.rowstride + c0 + cc;
                Tw w = tw[(1 << s) + (gidx / (2 * t))];
                u64 x = lds[i], y = lds[j];
                gs_bfly(x, y, w, q, q4, nq4);
                lds[i] = x;
                lds[j] = y;
            }
            __syncthreads();
        }
    }
    const u64 ni = ninv[prime], nis = ninv_s[prime];
    for (int e = threadIdx.x; e < elems; e += blockDim.x) {
        int r = e / gp.CW, cc = e % gp.CW;
        u64 v = lds[e];
        if (gp.last) {
            if (INV) {
                v = mul_shoup_lazy(v, ni, nis, q);
            } else {
                if (v >= q4) v -= q4;
                if (v >= q2) v -= q2;
            }
            if (v >= q) v -= q;
        }
        base[(size_t)r * gp.rowstride + c0 + cc] = v;
    }
}

// ------------------------------------------------------------------------------------------
// N = 2^16 kernels
// ------------------------------------------------------------------------------------------
// Two arithmetic back ends share the kernels below.
//
// IntField: 64-bit Shoup butterflies with values kept in [0, 4q) (Harvey), for primes up to 2^61.
//
// FpField: primes below 2^44 in double precision.  gfx950 issues one FP64 FMA per lane per clock but
// has to assemble every 64-bit integer product from 32-bit pieces, so for residues that fit a double
// exactly the floating-point butterfly is about a third of the instructions.  A product y*w mod q is
//     c = rint(y * (w/q));  h = fl(y*w);  l = fma(y, w, -h)  [exact low part];  r = fma(-c, q, h) + l
// Both h - c*q and the final sum are integers far below 2^53, so r is an exact residue of y*w, whatever c is.  The
// quotient w/q is formed as fl(w * fl(1/q)): y * (w/q) is then off by at most |y| * 1.5 * 2^-52, so
// |r| <= (0.5 + |y| * 1.5 * 2^-52) q -- 0.57 q for |y| < 2^47.5, 0.8 q for |y| < 2^49.7.  Values stay signed and
// unreduced through the forward stages (growth 0.57 q per stage: below 11 q < 2^48 after all 16); the inverse
// stages double the sums, so a radix-16 block first reduces its inputs.
// The last pass maps to [0, q), which makes the stored result identical to the integer path's.
// Between the two launches of one transform the buffer holds the raw doubles.
#pragma clang fp contract(off)

// LAZY16 (primes below 2^60, so 16q < 2^64; forward transforms only): forward values stay in [0, 16q) and only every
// other stage corrects its first operand -- by 8q, which takes values below 16q to below 8q; the stage after it adds up
// to 4q twice without a correction.  One conditional subtraction per two butterflies instead of one per butterfly.
template <bool LAZY16>
struct IntFieldT {
    typedef u64 E;
    typedef Tw W;
    u64 q, q2, q4, nq8, nq4, nq2, nq1, ni, nis;
    __device__ __forceinline__ IntFieldT(const ModQ *modq, const u64 *ninv, const u64 *ninv_s, const double *, int prime) {
        q = modq[prime].q;
        q2 = 2 * q;
        q4 = 4 * q;
        nq8 = opaque_neg(2 * q4);
        nq4 = opaque_neg(q4);
        nq2 = opaque_neg(q2);
        nq1 = opaque_neg(q);
        ni = ninv[prime];
        nis = ninv_s[prime];
    }
    __device__ __forceinline__ E from_canonical(u64 v) const { return v; }
    __device__ __forceinline__ E from_dot(const Dot3 &d, const ModQ &m) const { return dot3_reduce(d, m); }
    // odd: the stage's index within its radix-16 block is odd
    __device__ __forceinline__ void ct(E &x, E &y, const W tw, const bool odd) const {
        if (!LAZY16) {
            ct_bfly(x, y, tw, q, q4, nq4);
            return;
        }
        const u64 u = odd ? x : csub(x, 2 * q4, nq8);   // < 12q on odd stages, < 8q on even ones
        const u64 v = mul_shoup_lazy4(y, tw.w, tw.ws, q);              // < 4q
        x = u + v;
        y = u - v + q4;
    }
    __device__ __forceinline__ void gs(E &x, E &y, const W tw) const { gs_bfly(x, y, tw, q, q4, nq4); }
    __device__ __forceinline__ void after_inverse_block(E (&)[16]) const {}
    __device__ __forceinline__ u64 to_canonical(E v) const {   // v < 8q (16q with LAZY16)
        if (LAZY16) v = csub(v, 2 * q4, nq8);
        return csub(csub(csub(v, q4, nq4), q2, nq2), q, nq1);
    }
    __device__ __forceinline__ u64 scale_to_canonical(E v) const {
        return csub(mul_shoup_lazy(v, ni, nis, q), q, nq1);
    }
    // (y - v) * cst mod q for a transformed value v and a canonical minuend y
    __device__ __forceinline__ u64 sub_scale(E v, u64 y, const Tw cst) const {
        const u64 c = to_canonical(v);
        const u64 d = y >= c ? y - c : y + q - c;
        return csub(mul_shoup_lazy(d, cst.w, cst.ws, q), q, nq1);
    }
};

typedef IntFieldT<false> IntField;


struct FpField {
    typedef double E;
    typedef double W;   // the twiddle as a double; its quotient w / q is formed on the fly as w * (1 / q)
    double q, qinv, ni, niinv;
    __device__ __forceinline__ FpField(const ModQ *, const u64 *, const u64 *, const double *fp, int prime) {
        q = fp[4 * prime];
        qinv = fp[4 * prime + 1];
        ni = fp[4 * prime + 2];
        niinv = fp[4 * prime + 3];
    }
    __device__ __forceinline__ E mulmod(E y, E w, E winv) const {
        const double c = __builtin_rint(y * winv);
        const double h = y * w;
        const double l = __builtin_fma(y, w, -h);
        return __builtin_fma(-c, q, h) + l;
    }
    __device__ __forceinline__ E reduce(E x) const { return __builtin_fma(-__builtin_rint(x * qinv), q, x); }
    __device__ __forceinline__ E from_canonical(u64 v) const {
        return __longlong_as_double((long long)(v | 0x4330000000000000ull)) - 4503599627370496.0;
    }
    // A lazy dot product (three accumulators of weights 1, 2^32, 2^64 and a carry count of weight 2^64) as a residue of
    // magnitude below q: regrouped into pieces of weights 1, 2^32, 2^64 below 2^32, 2^33 and 2^45 (constants below
    // 2^44, residues below 2^60, 8 terms), each exact in a double; the two upper ones are multiplied by 2^32 and 2^64
    // mod q.  No integer reduction and no conversion from canonical form.
    __device__ __forceinline__ E from_dot(const Dot3 &d, const ModQ &) const {
        const u64 p1 = (d.s0 >> 32) + (d.s1 & 0xffffffffull), p2 = (d.s1 >> 32) + d.s2 + d.c;
        const double r32 = reduce(4294967296.0), r64 = reduce(18446744073709551616.0);
        const double a = (double)(u32)d.s0 + mulmod(from_canonical(p1), r32, r32 * qinv) +
                         mulmod(from_canonical(p2), r64, r64 * qinv);
        return reduce(a);
    }
    __device__ __forceinline__ void ct(E &x, E &y, const W tw, const bool) const {
        const double v = mulmod(y, tw, tw * qinv);
        const double u = x;
        x = u + v;
        y = u - v;
    }
    __device__ __forceinline__ void gs(E &x, E &y, const W tw) const {
        const double u = x, v = y;
        x = u + v;
        y = mulmod(u - v, tw, tw * qinv);
    }
    // A Gentleman-Sande block of four stages doubles the sums: from inputs bounded by B its outputs are bounded by
    // 16 B (element 0), 8 r (element 1), 4 r, 4 r, 2 r x 4, r x 8 with r the bound of a product, and the largest
    // value it multiplies is 16 B.  With only elements 0 and 1 reduced after each block every block starts from
    // B <= 4 r: r <= 0.8 q gives B <= 3.2 q and 16 B <= 51 q < 2^49.7 (q < 2^44), for which r <= 0.8 q holds again;
    // products of values below 2^50 are still exact.
    __device__ __forceinline__ void after_inverse_block(E (&x)[16]) const {
        x[0] = reduce(x[0]);
        x[1] = reduce(x[1]);
    }
    __device__ __forceinline__ u64 centred_to_canonical(E r) const {
        r += r < 0.0 ? q : 0.0;
        return (u64)__double_as_longlong(r + 4503599627370496.0) & 0x000fffffffffffffull;
    }
    __device__ __forceinline__ u64 to_canonical(E v) const { return centred_to_canonical(reduce(v)); }
    __device__ __forceinline__ u64 scale_to_canonical(E v) const { return centred_to_canonical(mulmod(v, ni, niinv)); }
    __device__ __forceinline__ u64 sub_scale(E v, u64 y, const Tw cst) const {
        const double w = (double)cst.w;
        return centred_to_canonical(mulmod(from_canonical(y) - v, w, w * qinv));
    }
};

// radix-16 block of 4 Cooley-Tukey stages on registers; stage s, group g uses twiddle
// (X << s) + g.
template <class F>
__device__ __forceinline__ void radix16_fwd(const F &f, typename F::E (&x)[16], const typename F::W *__restrict__ tw,
                                            const u32 X) {
#pragma unroll
    for (int s = 0; s < 4; s++) {
        const int d = 8 >> s;
#pragma unroll
        for (int g = 0; g < (1 << s); g++) {
            const typename F::W w = tw[(X << s) + g];
#pragma unroll
            for (int j = 0; j < d; j++) f.ct(x[g * 2 * d + j], x[g * 2 * d + j + d], w, (s & 1) != 0);
        }
    }
}
// radix-16 block of 4 Gentleman-Sande stages; stage s (distance 1<<s), group g uses twiddle
// (X << (3-s)) + g.
template <class F>
__device__ __forceinline__ void radix16_inv(const F &f, typename F::E (&x)[16], const typename F::W *__restrict__ tw,
                                            const u32 X) {
#pragma unroll
    for (int s = 0; s < 4; s++) {
        const int d = 1 << s;
#pragma unroll
        for (int g = 0; g < (8 >> s); g++) {
            const typename F::W w = tw[(X << (3 - s)) + g];
#pragma unroll
            for (int j = 0; j < d; j++) f.gs(x[g * 2 * d + j], x[g * 2 * d + j + d], w);
        }
    }
}

// The inner radix-16 block of a row pass (X = 16 (256 + r) + c: a different X for every thread) reads its 15 twiddles
// from a table laid out for it: entry ((r * 15 + slot) * 16 + c), slot = 2^l - 1 + g for twiddle (X << l) + g, so that
// the 16 threads of a row read 16 consecutive entries per (l, g) -- from the stage-ordered table they would read 16
// entries 2^l apart, up to 64 cache lines per load instruction of a wavefront instead of 8.
template <class F>
__device__ __forceinline__ void radix16_fwd_rows(const F &f, typename F::E (&x)[16], const typename F::W *__restrict__ rt) {
#pragma unroll
    for (int s = 0; s < 4; s++) {
        const int d = 8 >> s;
#pragma unroll
        for (int g = 0; g < (1 << s); g++) {
            const typename F::W w = rt[((1 << s) - 1 + g) * 16];
#pragma unroll
            for (int j = 0; j < d; j++) f.ct(x[g * 2 * d + j], x[g * 2 * d + j + d], w, (s & 1) != 0);
        }
    }
}
template <class F>
__device__ __forceinline__ void radix16_inv_rows(const F &f, typename F::E (&x)[16], const typename F::W *__restrict__ rt) {
#pragma unroll
    for (int s = 0; s < 4; s++) {
        const int d = 1 << s;
#pragma unroll
        for (int g = 0; g < (8 >> s); g++) {
            const typename F::W w = rt[((8 >> s) - 1 + g) * 16];
#pragma unroll
            for (int j = 0; j < d; j++) f.gs(x[g * 2 * d + j], x[g * 2 * d + j + d], w);
        }
    }
}

#define ROWPAD 272  // 256 residues of a row + one pad word per 16, so a 16-lane column read
                    // (stride 17 words) hits 16 distinct bank pairs
__device__ __forceinline__ int padc(int c) { return c + (c >> 4); }

__device__ __forceinline__ int swz_row(int r) { return r ^ ((r >> 4) & 1); }

// forward pass 1 / inverse pass 2 work on a 256-row x 16-column slab.
template <bool INV, class F>
__device__ __forceinline__ void cols_body(const __amdgpu_buffer_rsrc_t limb, const u32 col, const Tw *__restrict__ tw_int,
                                          const F f, u64 *lds_raw) {
    typedef typename F::E E;
    const typename F::W *tw = (const typename F::W *)tw_int;
    E *lds = (E *)lds_raw;
    const int cc = threadIdx.x & 15, rh = threadIdx.x >> 4;
    // byte offsets of (row rh, col) and (row 16 rh, col); rows 16 k resp. k further on go into the scalar offset
    const u32 v_outer = (col + ((u32)rh << 8)) * 8u, v_inner = (col + ((u32)rh << 12)) * 8u;
    E x[16];
    if (!INV) {
#pragma unroll
        for (int k = 0; k < 16; k++) x[k] = f.from_canonical(buf_load<u64>(limb, v_outer, (u32)k << 15));
        radix16_fwd(f, x, tw, 1u);
        // row r of the slab is kept at row r ^ (bit 4 of r): the rows 16 apart that one wavefront reads together
        // after the exchange then alternate between the two halves of the 64 LDS banks instead of sharing 32 of them
#pragma unroll
        for (int k = 0; k < 16; k++) lds[swz_row(rh + 16 * k) * 16 + cc] = x[k];
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 16; k++) x[k] = lds[swz_row(16 * rh + k) * 16 + cc];
        radix16_fwd(f, x, tw, 16u + rh);
#pragma unroll
        for (int k = 0; k < 16; k++) buf_store<E>(limb, v_inner, (u32)k << 11, x[k]);
    } else {
#pragma unroll
        for (int k = 0; k < 16; k++) x[k] = buf_load<E>(limb, v_inner, (u32)k << 11);
        radix16_inv(f, x, tw, 16u + rh);
        f.after_inverse_block(x);
#pragma unroll
        for (int k = 0; k < 16; k++) lds[(16 * rh + k) * 16 + cc] = x[k];
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 16; k++) x[k] = lds[(rh + 16 * k) * 16 + cc];
        radix16_inv(f, x, tw, 1u);
#pragma unroll
        for (int k = 0; k < 16; k++) buf_store<u64>(limb, v_outer, (u32)k << 15, f.scale_to_canonical(x[k]));
    }
}

template <bool INV>
__global__ __launch_bounds__(256) void ntt16_cols_kernel(u64 *__restrict__ data, const Tw *__restrict__ tw_all,
                                                         const ModQ *__restrict__ modq,
                                                         const u64 *__restrict__ ninv, const u64 *__restrict__ ninv_s,
                                                         const double *__restrict__ fp, LimbList ll, LimbList sl,
                                                         int n_limbs, size_t poly_stride, const Tw *__restrict__ final_scale) {
    __shared__ u64 lds[256 * 16];
    const int limb = blockIdx.y % n_limbs, poly = blockIdx.y / n_limbs;
    const int prime = ll.idx[limb];
    const Tw *tw = tw_all + ((size_t)prime << 16);
    const __amdgpu_buffer_rsrc_t base = limb_rsrc(
        data + (size_t)poly * poly_stride + ((size_t)__builtin_amdgcn_readfirstlane((int)sl.idx[limb]) << 16));
    const u32 col = blockIdx.x * 16 + (threadIdx.x & 15);
    // final_scale (inverse transforms only): limb i ends with the constant final_scale[i] in place of 1/N -- a basis
    // conversion folds its (S/q_i)^-1 factor in here (the caller supplies (1/N)(S/q_i)^-1), at no cost
    if (fp[4 * prime] != 0.0) {
        FpField f(modq, ninv, ninv_s, fp, prime);
        if (INV && final_scale != nullptr) {
            f.ni = (double)final_scale[limb].w;
            f.niinv = f.ni * f.qinv;
        }
        cols_body<INV>(base, col, tw, f, lds);
    } else if (INV || (modq[prime].q >> 60) != 0) {
        IntField f(modq, ninv, ninv_s, fp, prime);
        if (INV && final_scale != nullptr) {
            f.ni = final_scale[limb].w;
            f.nis = final_scale[limb].ws;
        }
        cols_body<INV>(base, col, tw, f, lds);
    } else {
        cols_body<INV>(base, col, tw, IntFieldT<true>(modq, ninv, ninv_s, fp, prime), lds);
    }
}

// Forward pass 1 over a slab whose input is a basis conversion computed on the fly: the thread's 16 coefficients of
// the target limb are sum_i v_i * hat_i mod q over the NS source limbs of the limb's digit (sources pre-scaled, the
// same lazy sums and reductions as the stand-alone conversion kernels, so the residues are the same).  The workgroups
// of the target limbs that share a (polynomial, slab) pair have consecutive blockIdx.y and the same blockIdx.x, so
// they sit on one XCD at about the same time and all but the first find the source slabs in its L2.
template <int NS, class F>
__device__ __forceinline__ void cols_converted_body(const __amdgpu_buffer_rsrc_t limb, const u32 col,
                                                    const Tw *__restrict__ tw_int, const F f, u64 *lds_raw,
                                                    const __amdgpu_buffer_rsrc_t src, const u32 voff,
                                                    const u32 (&so)[NS], const u64 (&h)[NS], const int n_src,
                                                    const ModQ m) {
    typedef typename F::E E;
    const typename F::W *tw = (const typename F::W *)tw_int;
    E *lds = (E *)lds_raw;
    const int cc = threadIdx.x & 15, rh = threadIdx.x >> 4;
    E x[16];
    // eight coefficients at a time (three accumulators each), source by source, so that the eight loads of one source
    // limb are in flight together
#pragma unroll
    for (int half = 0; half < 2; half++) {
        Dot3 d[8];
#pragma unroll
        for (int k = 0; k < 8; k++) dot3_clear(d[k]);
#pragma unroll
        for (int i = 0; i < NS; i++) {
            if (i < n_src) {
                u64 v[8];
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    // row rh + 16 (8 half + k) of the slab: the row step of 32 KiB goes into the scalar offset
                    const u32x2 w = __builtin_amdgcn_raw_buffer_load_b64(src, voff, so[i] + ((u32)(8 * half + k) << 15), 0);
                    v[k] = ((u64)w.y << 32) | w.x;
                }
#pragma unroll
                for (int k = 0; k < 8; k++) dot3_add(d[k], v[k], h[i]);
            }
        }
#pragma unroll
        for (int k = 0; k < 8; k++) x[8 * half + k] = f.from_dot(d[k], m);
    }
    radix16_fwd(f, x, tw, 1u);
#pragma unroll
    for (int k = 0; k < 16; k++) lds[swz_row(rh + 16 * k) * 16 + cc] = x[k];
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; k++) x[k] = lds[swz_row(16 * rh + k) * 16 + cc];
    radix16_fwd(f, x, tw, 16u + rh);
    const u32 v_inner = (col + ((u32)rh << 12)) * 8u;   // (row 16 rh, col); row k further on in the scalar offset
#pragma unroll
    for (int k = 0; k < 16; k++) buf_store<E>(limb, v_inner, (u32)k << 11, x[k]);
}

// Register budget of three waves per SIMD (168): left alone the compiler takes 170 - 176 registers, which leaves two
// waves (measured 15 % slower); four waves (128 registers) only with about 86 spilled ones (18 % slower).
template <int NS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void ntt16_cols_converted_kernel(
    u64 *__restrict__ data, const Tw *__restrict__ tw_all, const ModQ *__restrict__ modq, const u64 *__restrict__ ninv,
    const u64 *__restrict__ ninv_s, const double *__restrict__ fp, LimbList ll, LimbList sl, int n_limbs,
    size_t poly_stride, ConvSources cs) {
    __shared__ u64 lds[256 * 16];
    const int per_poly = n_limbs + cs.n_copy;
    const int limb = blockIdx.y % per_poly, poly = blockIdx.y / per_poly;
    const size_t col = blockIdx.x * 16 + (threadIdx.x & 15);
    if (limb >= n_limbs) {   // a limb that is only copied into its slot
        const u64 *from = cs.copy_src + (size_t)poly * cs.copy_src_stride +
                          ((size_t)cs.copy_src_slot[limb - n_limbs] << 16) + col;
        u64 *base = data + (size_t)poly * poly_stride + ((size_t)cs.copy_dst_slot[limb - n_limbs] << 16) + col;
        const int rh = threadIdx.x >> 4;
        u64 t[16];
        if (cs.copy_galois != 0) {   // the copy of the source's automorphism
            const u64 *fl = from - col;
#pragma unroll
            for (int k = 0; k < 16; k++)
                t[k] = fl[galois_index(((u32)(rh + 16 * k) << 8) + (u32)col, cs.copy_galois, 16)];
        } else {
#pragma unroll
            for (int k = 0; k < 16; k++) t[k] = from[(size_t)(rh + 16 * k) << 8];
        }
#pragma unroll
        for (int k = 0; k < 16; k++) base[(size_t)(rh + 16 * k) << 8] = t[k];
        return;
    }
    const __amdgpu_buffer_rsrc_t base = limb_rsrc(
        data + (size_t)poly * poly_stride + ((size_t)__builtin_amdgcn_readfirstlane((int)sl.idx[limb]) << 16));
    const int prime = ll.idx[limb];
    const Tw *tw = tw_all + ((size_t)prime << 16);
    const int dg = __builtin_amdgcn_readfirstlane((int)cs.digit_of[limb]), n_src = cs.d[dg].n_src;
    // The sources are read through a buffer resource: base (the polynomial's source limbs; far below 4 GiB), source slot
    // and slab row sit in scalar registers, a thread supplies one 32-bit offset for all of its 16 n_src loads.
    const __amdgpu_buffer_rsrc_t src = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(cs.d[dg].src + (size_t)poly * cs.d[dg].src_poly_stride), 0, -1, 0x00020000);
    const u32 voff = (u32)(col + ((threadIdx.x >> 4) << 8)) * 8u;
    const Cst *hat = cs.d[dg].hat + prime;
    const ModQ m = modq[prime];
    u32 so[NS];
    u64 h[NS];
#pragma unroll
    for (int i = 0; i < NS; i++) {
        const int ii = i < n_src ? i : 0;
        so[i] = __builtin_amdgcn_readfirstlane((u32)cs.d[dg].src_slot[ii]) << 19;
        h[i] = hat[(size_t)ii * cs.hat_ld].w;
    }
    if (fp[4 * prime] != 0.0)
        cols_converted_body<NS>(base, (u32)col, tw, FpField(modq, ninv, ninv_s, fp, prime), lds, src, voff, so, h, n_src, m);
    else if ((m.q >> 60) != 0)
        cols_converted_body<NS>(base, (u32)col, tw, IntField(modq, ninv, ninv_s, fp, prime), lds, src, voff, so, h, n_src, m);
    else
        cols_converted_body<NS>(base, (u32)col, tw, IntFieldT<true>(modq, ninv, ninv_s, fp, prime), lds, src, voff, so, h, n_src, m);
}

// ------------------------------------------------------------------------------------------
// Column-slab kernel of a ModDown (or any conversion of a few source limbs): for one (polynomial, 16-column slab) a
// workgroup runs the second pass of the inverse transform of every source limb, keeps the canonical coefficients on
// chip -- the last four sources in registers, one more in LDS -- and then, target limb by target limb, takes the
// basis conversion as lazy dot products and runs the first pass of the forward transform.  The inverse result is
// never written and the sources are never read back: the three steps are local to the slab, only the row passes on
// either side need the other half of the 256 x 256 view.  Arithmetic, order of operations and stored values are those
// of ntt16_cols_kernel<true> followed by ntt16_cols_converted_kernel.
// 128 registers of sources per thread leave room for two waves per SIMD; LDS: 32 KiB exchange + 32 KiB source.
// ------------------------------------------------------------------------------------------
#define SLAB_REG_SOURCES 4
struct SlabSources {
    const u64 *src;            // first-pass output of the inverse transform (raw field values), [n_polys][.][N]
    size_t src_poly_stride;
    const Cst *hat;            // [n_src][hat_ld]  (S/q_i) mod prime, indexed by prime
    const Tw *final_scale;     // [n_src]  (1/N)(S/q_i)^-1 mod q_i
    int hat_ld, n_src, n_dst;
    uint8_t src_slot[SLAB_REG_SOURCES + 1], src_prime[SLAB_REG_SOURCES + 1];
    uint8_t dst_slot[HEMM_MAX_PRIMES], dst_prime[HEMM_MAX_PRIMES];
};

template <class F>
__device__ __forceinline__ void slab_inverse(const __amdgpu_buffer_rsrc_t limb, const u32 v_inner,
                                             const Tw *__restrict__ tw_int, const F f, u64 *lds_raw, u64 (&r)[16]) {
    typedef typename F::E E;
    const typename F::W *tw = (const typename F::W *)tw_int;
    E *lds = (E *)lds_raw;
    const int cc = threadIdx.x & 15, rh = threadIdx.x >> 4;
    E x[16];
#pragma unroll
    for (int k = 0; k < 16; k++) x[k] = buf_load<E>(limb, v_inner, (u32)k << 11);
    radix16_inv(f, x, tw, 16u + rh);
    f.after_inverse_block(x);
    __syncthreads();   // the previous exchange has been read by every wave
#pragma unroll
    for (int k = 0; k < 16; k++) lds[(16 * rh + k) * 16 + cc] = x[k];
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; k++) x[k] = lds[(rh + 16 * k) * 16 + cc];
    radix16_inv(f, x, tw, 1u);
#pragma unroll
    for (int k = 0; k < 16; k++) r[k] = f.scale_to_canonical(x[k]);
}

template <int NREG, bool LDS, class F>
__device__ __forceinline__ void slab_forward(const __amdgpu_buffer_rsrc_t limb, const u32 v_inner,
                                             const Tw *__restrict__ tw_int, const F f, u64 *lds_raw,
                                             const u64 *__restrict__ lsrc, const u64 hl,
                                             const u64 (&c)[SLAB_REG_SOURCES][16], const u64 (&h)[SLAB_REG_SOURCES],
                                             const ModQ m) {
    typedef typename F::E E;
    const typename F::W *tw = (const typename F::W *)tw_int;
    E *lds = (E *)lds_raw;
    const int cc = threadIdx.x & 15, rh = threadIdx.x >> 4;
    E x[16];
#pragma unroll
    for (int k = 0; k < 16; k++) {
        Dot3 d;
        dot3_clear(d);
        if (LDS) dot3_add(d, lsrc[k * 256 + threadIdx.x], hl);
#pragma unroll
        for (int j = SLAB_REG_SOURCES - NREG; j < SLAB_REG_SOURCES; j++) dot3_add(d, c[j][k], h[j]);
        x[k] = f.from_dot(d, m);
    }
    radix16_fwd(f, x, tw, 1u);
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; k++) lds[swz_row(rh + 16 * k) * 16 + cc] = x[k];
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; k++) x[k] = lds[swz_row(16 * rh + k) * 16 + cc];
    radix16_fwd(f, x, tw, 16u + rh);
#pragma unroll
    for (int k = 0; k < 16; k++) buf_store<E>(limb, v_inner, (u32)k << 11, x[k]);
}

template <int NREG, bool LDS>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void ntt16_slab_convert_kernel(
    u64 *__restrict__ data, const size_t poly_stride, const Tw *__restrict__ tw_all, const Tw *__restrict__ itw_all,
    const ModQ *__restrict__ modq, const u64 *__restrict__ ninv, const u64 *__restrict__ ninv_s,
    const double *__restrict__ fp, const SlabSources ss) {
    __shared__ u64 lds[256 * 16];
    __shared__ u64 lsrc[256 * 16];
    const int poly = blockIdx.y;
    const u32 col = blockIdx.x * 16 + (threadIdx.x & 15);
    const u32 v_inner = (col + ((u32)(threadIdx.x >> 4) << 12)) * 8u;   // (row 16 rh, col); row k further: scalar offset
    constexpr int n_lds = LDS ? 1 : 0, n_src = NREG + n_lds, first_reg = SLAB_REG_SOURCES - NREG;
    u64 c[SLAB_REG_SOURCES][16];
#pragma unroll
    for (int j = 0; j < SLAB_REG_SOURCES; j++)
#pragma unroll
        for (int k = 0; k < 16; k++) c[j][k] = 0;
    // source i < n_lds goes to LDS, the others shift through the register sets: the last source ends in c[3]
#pragma unroll 1
    for (int i = 0; i < n_src; i++) {
        const int prime = __builtin_amdgcn_readfirstlane((int)ss.src_prime[i]);
        const __amdgpu_buffer_rsrc_t limb = limb_rsrc(
            ss.src + (size_t)poly * ss.src_poly_stride + ((size_t)__builtin_amdgcn_readfirstlane((int)ss.src_slot[i]) << 16));
        const Tw *tw = itw_all + ((size_t)prime << 16);
        const Tw fs = ss.final_scale[i];
        if (i >= n_lds) {
#pragma unroll
            for (int k = 0; k < 16; k++) {
                c[0][k] = c[1][k];
                c[1][k] = c[2][k];
                c[2][k] = c[3][k];
            }
        }
        if (fp[4 * prime] != 0.0) {
            FpField f(modq, ninv, ninv_s, fp, prime);
            f.ni = (double)fs.w;
            f.niinv = f.ni * f.qinv;
            slab_inverse(limb, v_inner, tw, f, lds, c[3]);
        } else {
            IntField f(modq, ninv, ninv_s, fp, prime);
            f.ni = fs.w;
            f.nis = fs.ws;
            slab_inverse(limb, v_inner, tw, f, lds, c[3]);
        }
        if (i < n_lds) {
#pragma unroll
            for (int k = 0; k < 16; k++) lsrc[k * 256 + threadIdx.x] = c[3][k];
        }
    }
#pragma unroll 1
    for (int t = 0; t < ss.n_dst; t++) {
        const int prime = __builtin_amdgcn_readfirstlane((int)ss.dst_prime[t]);
        const __amdgpu_buffer_rsrc_t limb = limb_rsrc(
            data + (size_t)poly * poly_stride + ((size_t)__builtin_amdgcn_readfirstlane((int)ss.dst_slot[t]) << 16));
        const Tw *tw = tw_all + ((size_t)prime << 16);
        const ModQ m = modq[prime];
        const Cst *hat = ss.hat + prime;
        u64 h[SLAB_REG_SOURCES];
#pragma unroll
        for (int j = 0; j < SLAB_REG_SOURCES; j++) {
            const int i = n_lds + j - first_reg;
            h[j] = j >= first_reg ? hat[(size_t)i * ss.hat_ld].w : 0;
        }
        const u64 hl = LDS ? hat[0].w : 0;
        if (fp[4 * prime] != 0.0)
            slab_forward<NREG, LDS>(limb, v_inner, tw, FpField(modq, ninv, ninv_s, fp, prime), lds, lsrc, hl, c, h, m);
        else
            slab_forward<NREG, LDS>(limb, v_inner, tw, IntFieldT<true>(modq, ninv, ninv_s, fp, prime), lds, lsrc, hl, c, h, m);
    }
}

// A row's 16 threads sit in one wavefront (thread = row * 16 + column group), so the LDS exchanges of
// the row kernel never cross a wavefront: ordering them needs no workgroup barrier, only a fence that
// keeps the compiler from moving LDS accesses across it.
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Optional tail of a forward transform: instead of storing the transformed residues v in place, store
// (minuend - v) * cst[limb] to `out` -- the last step of ModDown / rescale, folded into the pass that
// already holds v in registers (saves one read and one write of every limb and a launch).
struct NttEpilogue {
    const u64 *minuend;
    u64 *out;
    const Tw *cst;  // per limb: constant and Shoup quotient
    size_t minuend_stride, out_stride;
    u32 galois;     // inverse transforms that read their input elsewhere: != 0 reads it through this automorphism
};
// An inverse transform may read its input elsewhere (same slot numbering, own polynomial stride) and leave the
// result in `data`: the first pass then loads from `minuend` (stride `minuend_stride`) instead of `data`.

// forward pass 2 / inverse pass 1 work on 16 whole rows (16 x 256 contiguous residues).
// GAL (inverse only): ld is the base of the source limb and residue k of the input is ld[galois_index(k)] -- an aligned
// group of 16 residues stays an aligned group under the automorphism, so the loads touch the same number of lines
template <bool INV, bool EPI, bool GAL, class F>
__device__ __forceinline__ void rows_body(u64 *__restrict__ row, const Tw *__restrict__ tw_int,
                                          const Tw *__restrict__ rtw_int, const F f, u64 *lds_raw, const u32 r, const u64 q,
                                          const u64 *__restrict__ mn, u64 *__restrict__ o, const Tw cst,
                                          const u64 *__restrict__ ld, const u32 gal = 0) {
    typedef typename F::E E;
    const typename F::W *tw = (const typename F::W *)tw_int;
    const int c = threadIdx.x & 15, rr = threadIdx.x >> 4;
    const typename F::W *rt = (const typename F::W *)rtw_int + (r * 15u * 16u + (u32)c);
    E *l = (E *)lds_raw + rr * ROWPAD;
    u64 *lc = lds_raw + rr * ROWPAD;
    E *mem = (E *)row;
    E x[16];
    if (!INV) {
#pragma unroll
        for (int k = 0; k < 16; k++) x[k] = mem[c + 16 * k];
        radix16_fwd(f, x, tw, 256u + r);
#pragma unroll
        for (int k = 0; k < 16; k++) l[padc(c + 16 * k)] = x[k];
        wave_sync();
#pragma unroll
        for (int k = 0; k < 16; k++) x[k] = l[padc(16 * c + k)];
        // the minuend of the fused tail is fetched under the second radix-16 block instead of after it
        u64 mv[EPI ? 16 : 1];
        if (EPI) {
#pragma unroll
            for (int k = 0; k < 16; k++) mv[k] = __builtin_nontemporal_load(mn + c + 16 * k);
        }
        radix16_fwd_rows(f, x, rt);
        wave_sync();
#pragma unroll
        for (int k = 0; k < 16; k++) l[padc(16 * c + k)] = x[k];
        wave_sync();
        if (EPI) {
#pragma unroll
            for (int k = 0; k < 16; k++) o[c + 16 * k] = f.sub_scale(l[padc(c + 16 * k)], mv[k], cst);
        } else {
#pragma unroll
            for (int k = 0; k < 16; k++) row[c + 16 * k] = f.to_canonical(l[padc(c + 16 * k)]);
        }
    } else {
        if (GAL) {
#pragma unroll
            for (int k = 0; k < 16; k++) lc[padc(c + 16 * k)] = ld[galois_index((r << 8) + (u32)(c + 16 * k), gal, 16)];
        } else {
#pragma unroll
            for (int k = 0; k < 16; k++) lc[padc(c + 16 * k)] = ld[c + 16 * k];
        }
        wave_sync();
#pragma unroll
        for (int k = 0; k < 16; k++) x[k] = f.from_canonical(lc[padc(16 * c + k)]);
        radix16_inv_rows(f, x, rt);
        f.after_inverse_block(x);
        wave_sync();
#pragma unroll
        for (int k = 0; k < 16; k++) l[padc(16 * c + k)] = x[k];
        wave_sync();
#pragma unroll
        for (int k = 0; k < 16; k++) x[k] = l[padc(c + 16 * k)];
        radix16_inv(f, x, tw, 256u + r);
        f.after_inverse_block(x);
#pragma unroll
        for (int k = 0; k < 16; k++) mem[c + 16 * k] = x[k];
    }
}

template <bool INV, bool EPI, bool GAL = false>
__global__ __launch_bounds__(256) void ntt16_rows_kernel(u64 *__restrict__ data, const Tw *__restrict__ tw_all,
                                                         const Tw *__restrict__ rtw_all,
                                                         const ModQ *__restrict__ modq, const double *__restrict__ fp,
                                                         LimbList ll, LimbList sl, int n_limbs, size_t poly_stride,
                                                         NttEpilogue ep) {
    __shared__ u64 lds[16 * ROWPAD];
    // The second radix-16 block of a row pass walks 1/16 of the prime's twiddle table per 16-row slab (as
    // many bytes as the slab's data), identical for every polynomial of the batch.  Workgroups are dealt
    // round-robin to the 8 XCDs, so the polynomials of one (limb, slab) pair are placed back to back on
    // one XCD and share those twiddles through its L2 instead of fetching them from HBM once each.
    const u32 n_polys = gridDim.x / (16u * (u32)n_limbs);
    const u32 xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3;
    const u32 poly = slot % n_polys, group = (slot / n_polys) * 8u + xcd;
    const int limb = (int)(group >> 4);
    const u32 slab = group & 15u;
    const int prime = ll.idx[limb];
    const Tw *tw = tw_all + ((size_t)prime << 16), *rtw = rtw_all + ((size_t)prime << 16);
    const u32 r = slab * 16 + (threadIdx.x >> 4);  // global row
    u64 *row = data + (size_t)poly * poly_stride + ((size_t)sl.idx[limb] << 16) + ((size_t)r << 8);
    const u64 *mn = nullptr;
    u64 *o = nullptr;
    Tw cst{0, 0};
    if (EPI) {
        const size_t off = ((size_t)limb << 16) + ((size_t)r << 8);
        mn = ep.minuend + (size_t)poly * ep.minuend_stride + off;
        o = ep.out + (size_t)poly * ep.out_stride + off;
        cst = ep.cst[limb];
    }
    const u64 q = modq[prime].q;
    const u64 *ld = row;
    if (INV && ep.minuend != nullptr)
        ld = ep.minuend + (size_t)poly * ep.minuend_stride + ((size_t)sl.idx[limb] << 16) + (GAL ? 0 : (size_t)r << 8);
    const u32 gal = GAL ? ep.galois : 0u;
    if (fp[4 * prime] != 0.0)
        rows_body<INV, EPI, GAL>(row, tw, rtw, FpField(modq, nullptr, nullptr, fp, prime), lds, r, q, mn, o, cst, ld, gal);
    else if (INV || (q >> 60) != 0)
        rows_body<INV, EPI, GAL>(row, tw, rtw, IntField(modq, nullptr, nullptr, fp, prime), lds, r, q, mn, o, cst, ld, gal);
    else
        rows_body<INV, EPI, GAL>(row, tw, rtw, IntFieldT<true>(modq, nullptr, nullptr, fp, prime), lds, r, q, mn, o, cst, ld,
                                 gal);
}

}  // namespace

// Forward transform of data[n_polys][n_limbs][N] (limb j = chain prime j) whose result is consumed as
// out = (minuend - NTT(data)) * cst[j]; returns false when this ring size has no fused tail (the caller
// then runs the transform and the subtraction separately).
// A transform is two launches, and the second reads what the first wrote.  On a large batch the first launch has
// pushed its early output out of the 256 MB memory-side cache by the time the second one starts, so batches are cut
// into runs of whole polynomials of about this many limbs (0.5 MiB each) and the two launches alternate run by run.
// Measured on 32 x 24 limbs, one stream: forward transforms are fastest at 192 limbs per run (60-bit primes 0.52 ->
// 0.43 ms, primes below 2^44 0.41 -> 0.36 ms), inverse ones at 384 (0.48 -> 0.44 ms, 0.37 -> 0.34 ms).  A plain batch
// of several runs (launch_ntt_slots) deals them out over two streams, the caller's and the context's second one:
// a launch of one run fills the part-empty last round of workgroups of the other's.  Same box, runs of 192 limbs in
// both directions: forward 0.378 -> 0.350 ms (60-bit) and 0.309 -> 0.278 ms (42-bit), inverse 0.390 -> 0.383 and
// 0.285 -> 0.278 ms; runs of 96, 128 or 256 limbs on two streams are 1 - 8 % slower than that.
static int polys_per_run(int n_limbs, int n_polys, bool inverse, bool two_streams = false) {
    // batches of up to 448 limbs (224 MiB: what one chain of the matrix products transforms at once, whose input a
    // producer has just written) are fastest as one run: 480 us for the ModDown of 64 polynomials against 497 us cut
    if (n_limbs * n_polys <= 448) return n_polys;
    const int limbs = inverse && !two_streams ? 384 : 192;
    int p = limbs / n_limbs;
    if (p < 1) p = 1;
    return p < n_polys ? p : n_polys;
}

bool launch_ntt_sub_scale(const hemm_context *c, u64 *data, int n_limbs, int n_polys, const u64 *minuend,
                          size_t minuend_stride, u64 *out, size_t out_stride, const void *cst_dev, hipStream_t s) {
    if (c->logN != 16) return false;
    account(c, TR_NTT, (size_t)3 * n_limbs * n_polys * c->N * 8, 2);   // limbs in, minuend in, result out
    LimbList ll, sl;
    for (int j = 0; j < HEMM_MAX_PRIMES; j++) ll.idx[j] = sl.idx[j] = (uint8_t)j;
    const Tw *tw = (const Tw *)c->d_w;
    const dim3 block(256);
    const size_t poly_stride = (size_t)n_limbs << 16;
    const int run = polys_per_run(n_limbs, n_polys, false);
    for (int p0 = 0; p0 < n_polys; p0 += run) {
        const int np = n_polys - p0 < run ? n_polys - p0 : run;
        u64 *d = data + (size_t)p0 * poly_stride;
        NttEpilogue ep{minuend + (size_t)p0 * minuend_stride, out + (size_t)p0 * out_stride, (const Tw *)cst_dev,
                       minuend_stride, out_stride};
        hipLaunchKernelGGL(ntt16_cols_kernel<false>, dim3(16, n_limbs * np), block, 0, s, d, tw, c->d_modq, c->d_ninv,
                           c->d_ninv_s, c->d_fp, ll, sl, n_limbs, poly_stride, (const Tw *)nullptr);
        hipLaunchKernelGGL((ntt16_rows_kernel<false, true>), dim3(16 * n_limbs * np), block, 0, s, d, tw, (const Tw *)c->d_rw,
                           c->d_modq, c->d_fp, ll, sl, n_limbs, poly_stride, ep);
    }
    return true;
}

bool launch_ntt_converted(const hemm_context *c, const ConvSources &cs, u64 *data, const LimbList &ll, const LimbList &sl,
                          int n_limbs, int n_polys, size_t poly_stride, hipStream_t s, const u64 *ep_minuend,
                          size_t ep_minuend_stride, u64 *ep_out, size_t ep_out_stride, const void *ep_cst_dev) {
    if (c->logN != 16) return false;
    if (n_limbs > HEMM_MAX_PRIMES || cs.n_copy < 0 || cs.n_copy > HEMM_MAX_PRIMES)
        throw std::invalid_argument("too many limbs in one converted transform");
    int widest = 0;
    for (int l = 0; l < n_limbs; l++) {
        if (cs.digit_of[l] >= CONV_MAX_DIGITS) throw std::invalid_argument("conversion digit out of range");
        widest = std::max(widest, cs.d[cs.digit_of[l]].n_src);
    }
    if (widest < 1 || widest > CONV_MAX_SOURCES) return false;
    if (n_limbs <= 0 || n_polys <= 0) return true;
    const bool tail = ep_out != nullptr;
    // sources of every digit in use once, limbs out (through the tail: minuend in, result out)
    size_t src_limbs = 0;
    bool seen[CONV_MAX_DIGITS] = {false, false, false, false};
    for (int l = 0; l < n_limbs; l++)
        if (!seen[cs.digit_of[l]]) {
            seen[cs.digit_of[l]] = true;
            src_limbs += (size_t)cs.d[cs.digit_of[l]].n_src;
        }
    if ((size_t)(n_limbs + cs.n_copy) * (size_t)n_polys > 65535)
        return false;   // more workgroup rows than one launch holds: the caller converts and transforms separately
    account(c, TR_BCONV, (src_limbs + 2 * (size_t)cs.n_copy) * n_polys * c->N * 8, 0);
    account(c, TR_NTT, (size_t)(tail ? 2 : 1) * n_limbs * n_polys * c->N * 8, 2);
    const Tw *tw = (const Tw *)c->d_w;
    const dim3 block(256), grid(16, (n_limbs + cs.n_copy) * n_polys);
#define CONV_CASE(K)                                                                                                    \
    hipLaunchKernelGGL(ntt16_cols_converted_kernel<K>, grid, block, 0, s, data, tw, c->d_modq, c->d_ninv, c->d_ninv_s, \
                       c->d_fp, ll, sl, n_limbs, poly_stride, cs)
    if (widest <= 2)
        CONV_CASE(2);
    else if (widest <= 5)
        CONV_CASE(5);
    else
        CONV_CASE(8);
#undef CONV_CASE
    if (tail) {
        NttEpilogue ep{ep_minuend, ep_out, (const Tw *)ep_cst_dev, ep_minuend_stride, ep_out_stride};
        hipLaunchKernelGGL((ntt16_rows_kernel<false, true>), dim3(16 * n_limbs * n_polys), block, 0, s, data, tw,
                           (const Tw *)c->d_rw, c->d_modq, c->d_fp, ll, sl, n_limbs, poly_stride, ep);
    } else {
        hipLaunchKernelGGL((ntt16_rows_kernel<false, false>), dim3(16 * n_limbs * n_polys), block, 0, s, data, tw,
                           (const Tw *)c->d_rw, c->d_modq, c->d_fp, ll, sl, n_limbs, poly_stride, NttEpilogue{});
    }
    return true;
}

// out[p][j] = (y[p][j] - conversion of the n_src listed limbs of y[p] to prime j) * cst[j] for j < nq_out, in three
// launches: first pass of the inverse transform of the listed limbs (in place), the column-slab kernel (second inverse
// pass, conversion, first forward pass into conv), second forward pass with the fused tail.  Same residues as the
// four-launch chain.  false when the shape has no such form (nothing was launched).
bool launch_moddown_slab(const hemm_context *c, u64 *y, size_t y_stride, const uint8_t *src_slot, const uint8_t *src_prime,
                         int n_src, const void *final_scale_dev, const void *hat_dev, int hat_ld, u64 *conv, int nq_out,
                         int n_polys, u64 *out, size_t out_stride, const void *cst_dev, hipStream_t s) {
    if (c->logN != 16 || n_src < 4 || n_src > 5 || nq_out < 1 || nq_out > HEMM_MAX_PRIMES) return false;
    if (n_polys <= 0) return true;
    SlabSources ss;
    memset(&ss, 0, sizeof(ss));
    LimbList sp, ssl, cl, ident;
    memset(&sp, 0, sizeof(sp));
    memset(&ssl, 0, sizeof(ssl));
    for (int j = 0; j < HEMM_MAX_PRIMES; j++) cl.idx[j] = ident.idx[j] = (uint8_t)j;
    for (int i = 0; i < n_src; i++) {
        ss.src_slot[i] = ssl.idx[i] = src_slot[i];
        ss.src_prime[i] = sp.idx[i] = src_prime[i];
    }
    for (int j = 0; j < nq_out; j++) {
        ss.dst_slot[j] = (uint8_t)j;
        ss.dst_prime[j] = (uint8_t)j;
    }
    ss.hat = (const Cst *)hat_dev;
    ss.final_scale = (const Tw *)final_scale_dev;
    ss.hat_ld = hat_ld;
    ss.n_src = n_src;
    ss.n_dst = nq_out;
    ss.src_poly_stride = y_stride;
    // same algorithmic bytes as the separate launches: the dropped limbs in and out of the inverse transform, the
    // conversion's sources, the minuend in and the result out of the forward transform
    account(c, TR_NTT, (size_t)2 * n_src * n_polys * c->N * 8, 1);
    account(c, TR_BCONV, (size_t)n_src * n_polys * c->N * 8, 1);
    account(c, TR_NTT, (size_t)2 * nq_out * n_polys * c->N * 8, 1);
    const dim3 block(256);
    const size_t conv_stride = (size_t)nq_out << 16;
    const int widest = n_src > nq_out ? n_src : nq_out;
    int run = 448 / widest;
    if (run < 1) run = 1;
    for (int p0 = 0; p0 < n_polys; p0 += run) {
        const int np = n_polys - p0 < run ? n_polys - p0 : run;
        u64 *yp = y + (size_t)p0 * y_stride;
        u64 *cp = conv + (size_t)p0 * conv_stride;
        ss.src = yp;
        hipLaunchKernelGGL((ntt16_rows_kernel<true, false>), dim3(16 * n_src * np), block, 0, s, yp, (const Tw *)c->d_iw,
                           (const Tw *)c->d_irw, c->d_modq, c->d_fp, sp, ssl, n_src, y_stride, NttEpilogue{});
#define SLAB_CASE(NREG, LDS)                                                                                             \
    hipLaunchKernelGGL((ntt16_slab_convert_kernel<NREG, LDS>), dim3(16, np), block, 0, s, cp, conv_stride,             \
                       (const Tw *)c->d_w, (const Tw *)c->d_iw, c->d_modq, c->d_ninv, c->d_ninv_s, c->d_fp, ss)
        if (n_src == 5)
            SLAB_CASE(4, true);
        else
            SLAB_CASE(4, false);
#undef SLAB_CASE
        NttEpilogue ep{yp, out + (size_t)p0 * out_stride, (const Tw *)cst_dev, y_stride, out_stride};
        hipLaunchKernelGGL((ntt16_rows_kernel<false, true>), dim3(16 * nq_out * np), block, 0, s, cp, (const Tw *)c->d_w,
                           (const Tw *)c->d_rw, c->d_modq, c->d_fp, cl, ident, nq_out, conv_stride, ep);
    }
    return true;
}

bool launch_intt_from(const hemm_context *c, const u64 *src, size_t src_poly_stride, u64 *data, const LimbList &ll,
                      const LimbList &sl, int n_limbs, int n_polys, size_t poly_stride, hipStream_t s,
                      const void *final_scale, u32 galois) {
    if (c->logN != 16) {
        if (galois != 0) throw std::invalid_argument("a transform reads through an automorphism at N = 2^16 only");
        return false;
    }
    if (n_limbs <= 0 || n_polys <= 0) return true;
    account(c, TR_NTT, (size_t)2 * n_limbs * n_polys * c->N * 8, 2);
    const Tw *tw = (const Tw *)c->d_iw;
    const dim3 block(256);
    const int run = polys_per_run(n_limbs, n_polys, true);
    for (int p0 = 0; p0 < n_polys; p0 += run) {
        const int np = n_polys - p0 < run ? n_polys - p0 : run;
        const int lanes = n_limbs * np;
        u64 *d = data + (size_t)p0 * poly_stride;
        NttEpilogue from{};
        from.minuend = src + (size_t)p0 * src_poly_stride;
        from.minuend_stride = src_poly_stride;
        from.galois = galois;
        if (galois != 0)
            hipLaunchKernelGGL((ntt16_rows_kernel<true, false, true>), dim3(16 * lanes), block, 0, s, d, tw,
                               (const Tw *)c->d_irw, c->d_modq, c->d_fp, ll, sl, n_limbs, poly_stride, from);
        else
            hipLaunchKernelGGL((ntt16_rows_kernel<true, false>), dim3(16 * lanes), block, 0, s, d, tw,
                               (const Tw *)c->d_irw, c->d_modq, c->d_fp, ll, sl, n_limbs, poly_stride, from);
        hipLaunchKernelGGL(ntt16_cols_kernel<true>, dim3(16, lanes), block, 0, s, d, tw, c->d_modq, c->d_ninv,
                           c->d_ninv_s, c->d_fp, ll, sl, n_limbs, poly_stride, (const Tw *)final_scale);
    }
    return true;
}

void launch_ntt_slots(const hemm_context *c, u64 *data, const LimbList &ll, const LimbList &sl, int n_limbs,
                      int n_polys, size_t poly_stride, bool inverse, hipStream_t s, const void *final_scale) {
    if (n_limbs <= 0 || n_polys <= 0) return;
    if (final_scale != nullptr && (!inverse || c->logN != 16))
        throw std::invalid_argument("a final constant is taken by the inverse transform of N = 2^16 only");
    account(c, TR_NTT, (size_t)2 * n_limbs * n_polys * c->N * 8, c->logN > 12 ? 2 : 1);
    const Tw *tw = (const Tw *)(inverse ? c->d_iw : c->d_w);
    const int lanes = n_limbs * n_polys;
    if (c->logN == 16) {
        const dim3 block(256);
        const int run = polys_per_run(n_limbs, n_polys, inverse, true);
        // several runs: the odd ones on the context's second stream, which starts after what the caller's stream holds
        // so far and is waited for before the call returns to it
        const bool two = run < n_polys;
        const hipStream_t own = s;
        if (two && c->aux == nullptr) {
            hemm_context *m = const_cast<hemm_context *>(c);
            HEMM_HIP(hipStreamCreateWithFlags(&m->aux, hipStreamNonBlocking));
            HEMM_HIP(hipEventCreateWithFlags(&m->aux_fork, hipEventDisableTiming));
            HEMM_HIP(hipEventCreateWithFlags(&m->aux_join, hipEventDisableTiming));
        }
        if (two) {
            HEMM_HIP(hipEventRecord(c->aux_fork, own));
            HEMM_HIP(hipStreamWaitEvent(c->aux, c->aux_fork, 0));
        }
        int run_index = 0;
        for (int p0 = 0; p0 < n_polys; p0 += run, run_index++) {
            const int np = n_polys - p0 < run ? n_polys - p0 : run;
            const int ln = n_limbs * np;
            u64 *d = data + (size_t)p0 * poly_stride;
            s = two && (run_index & 1) ? c->aux : own;
            if (!inverse) {
                hipLaunchKernelGGL(ntt16_cols_kernel<false>, dim3(16, ln), block, 0, s, d, tw, c->d_modq, c->d_ninv,
                                   c->d_ninv_s, c->d_fp, ll, sl, n_limbs, poly_stride, (const Tw *)nullptr);
                hipLaunchKernelGGL((ntt16_rows_kernel<false, false>), dim3(16 * ln), block, 0, s, d, tw,
                                   (const Tw *)c->d_rw, c->d_modq, c->d_fp, ll, sl, n_limbs, poly_stride, NttEpilogue{});
            } else {
                hipLaunchKernelGGL((ntt16_rows_kernel<true, false>), dim3(16 * ln), block, 0, s, d, tw,
                                   (const Tw *)c->d_irw, c->d_modq, c->d_fp, ll, sl, n_limbs, poly_stride, NttEpilogue{});
                hipLaunchKernelGGL(ntt16_cols_kernel<true>, dim3(16, ln), block, 0, s, d, tw, c->d_modq, c->d_ninv,
                                   c->d_ninv_s, c->d_fp, ll, sl, n_limbs, poly_stride, (const Tw *)final_scale);
            }
        }
        if (two) {
            HEMM_HIP(hipEventRecord(c->aux_join, c->aux));
            HEMM_HIP(hipStreamWaitEvent(own, c->aux_join, 0));
        }
        return;
    }
    // generic path
    const int logN = c->logN, N = c->N;
    GenericPass A{}, B{};
    int n_pass;
    if (logN <= 12) {
        n_pass = 1;
        B.logN = logN; B.R = N; B.CW = 1; B.rowstride = 1; B.s_begin = 0; B.s_end = logN;
        B.tiles_per_limb = 1;
    } else {
        n_pass = 2;
        const int sA = logN - 8;                 // strided stages
        A.logN = logN; A.R = 1 << sA; A.CW = (4096 >> sA) > 256 ? 256 : (4096 >> sA);
        A.rowstride = 256; A.s_begin = 0; A.s_end = sA; A.tiles_per_limb = 256 / A.CW;
        B.logN = logN; B.R = 4096; B.CW = 1; B.rowstride = 1; B.s_begin = sA; B.s_end = logN;
        B.tiles_per_limb = N / 4096;
    }
    auto run = [&](GenericPass gp, bool first, bool last) {
        gp.first = first; gp.last = last;
        dim3 grid(gp.tiles_per_limb, lanes), block(256);
        size_t sh = (size_t)gp.R * gp.CW * sizeof(u64);
        if (!inverse)
            hipLaunchKernelGGL(ntt_generic_kernel<false>, grid, block, sh, s, data, tw, c->d_modq, c->d_ninv,
                               c->d_ninv_s, ll, sl, n_limbs, poly_stride, gp);
        else {
            std::swap(gp.s_begin, gp.s_end);     // inverse walks stages downwards
            hipLaunchKernelGGL(ntt_generic_kernel<true>, grid, block, sh, s, data, tw, c->d_modq, c->d_ninv,
                               c->d_ninv_s, ll, sl, n_limbs, poly_stride, gp);
        }
    };
    if (n_pass == 1) {
        run(B, true, true);
    } else if (!inverse) {
        run(A, true, false);
        run(B, false, true);
    } else {
        run(B, true, false);
        run(A, false, true);
    }
}

void launch_ntt(const hemm_context *c, u64 *data, const LimbList &ll, int n_limbs, int n_polys,
                size_t poly_stride, bool inverse, hipStream_t s) {
    LimbList sl;
    for (int j = 0; j < HEMM_MAX_PRIMES; j++) sl.idx[j] = (uint8_t)j;
    launch_ntt_slots(c, data, ll, sl, n_limbs, n_polys, poly_stride, inverse, s);
}

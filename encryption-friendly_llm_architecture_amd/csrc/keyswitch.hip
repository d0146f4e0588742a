// Hybrid key switching (ModUp -> evaluation-key inner product -> ModDown) and rescale.
//
//   ModUp    : per digit d, coefficient-form fast basis conversion of the digit's limbs to every
//              other active limb (chain + special), then NTT of the converted limbs.
//   inner    : acc[pol][j] = sum_d ext_d[j] * evk[d][pol][prime(j)]   (128-bit lazy sum, one
//              Barrett step per output residue).  Reads the key exactly once: this is the
//              HBM-bound part, 2*beta*(nq+K) limbs of key per switch.
//   ModDown  : INTT of the special limbs, basis conversion P -> Q, NTT, (acc - conv) * P^-1.
//   rescale  : INTT of the last limb, reduce into every remaining prime, NTT, (c - t) * q_l^-1.
// Basis conversion is the float-free form  y_j = sum_i [x_i * (S/q_i)^-1]_{q_i} * (S/q_i) mod q_j.
#include <cstring>

#include "hemm_internal.hpp"
#include "hoisted.h"


namespace {

struct BConvArgs {
    const u64 *src;        // coefficient form
    u64 *dst;              // coefficient form
    size_t src_poly_stride, dst_poly_stride;
    const Cst *inv;        // [n_src]  (S/q_i)^-1 mod q_i
    const Cst *hat;        // [n_src][hat_ld]  (S/q_i) mod prime, indexed by prime
    int n_src, n_dst, hat_ld, logN;
    int pre_scaled;        // the source residues already carry their (S/q_i)^-1 factor (folded into the inverse transform)
    int split;             // register kernels: the target limbs are dealt to this many workgroups per coefficient block
                           // (blockIdx.y = polynomial * split + part); 0 counts as 1
    uint8_t src_slot[32], src_prime[32];
    uint8_t dst_slot[HEMM_MAX_PRIMES], dst_prime[HEMM_MAX_PRIMES];
};

// One thread owns one coefficient: the n_src scaled residues stay in LDS columns private to the
// thread, then every target limb is a short Shoup multiply-accumulate chain.
__global__ __launch_bounds__(256) void bconv_kernel(BConvArgs a, const ModQ *__restrict__ modq) {
    extern __shared__ u64 v[];  // [n_src][256]
    const int poly = blockIdx.y;
    const size_t n = (size_t)blockIdx.x * 256 + threadIdx.x;
    const u64 *src = a.src + poly * a.src_poly_stride;
    u64 *dst = a.dst + poly * a.dst_poly_stride;
    for (int i = 0; i < a.n_src; i++) {
        const u64 q = modq[a.src_prime[i]].q;
        const Cst c = a.inv[i];
        const u64 x = src[((size_t)a.src_slot[i] << a.logN) + n];
        v[i * 256 + threadIdx.x] = a.pre_scaled ? x : mul_shoup(x, c.w, c.ws, q);
    }
    for (int j = 0; j < a.n_dst; j++) {
        const int pj = a.dst_prime[j];
        const u64 q = modq[pj].q;
        u64 acc = 0;
        for (int i = 0; i < a.n_src; i++) {
            const Cst c = a.hat[i * a.hat_ld + pj];
            acc = addmod(acc, mul_shoup(v[i * 256 + threadIdx.x], c.w, c.ws, q), q);
        }
        dst[((size_t)a.dst_slot[j] << a.logN) + n] = acc;
    }
}

// Register form of the same conversion for up to 8 source limbs and primes below 2^60: a thread owns two adjacent
// coefficients (16-byte accesses), keeps the scaled source residues in registers and takes every target residue as a
// lazy dot product (four 32-bit multiply-adds per term) with one reduction at the end.
template <int NS>
__global__ __launch_bounds__(256) void bconv_reg_kernel(BConvArgs a, const ModQ *__restrict__ modq) {
    const int S = a.split > 1 ? a.split : 1;
    const int poly = blockIdx.y / S, part = blockIdx.y % S;
    const int per = (a.n_dst + S - 1) / S, j_lo = part * per, j_hi = min(a.n_dst, j_lo + per);
    const size_t n = ((size_t)blockIdx.x * 256 + threadIdx.x) * 2;
    const u64 *src = a.src + poly * a.src_poly_stride;
    u64 *dst = a.dst + poly * a.dst_poly_stride;
    u64 v0[NS], v1[NS];
#pragma unroll
    for (int i = 0; i < NS; i++) {
        const u64 q = modq[a.src_prime[i]].q;
        const Cst c = a.inv[i];
        const ulonglong2 x = *(const ulonglong2 *)(src + ((size_t)a.src_slot[i] << a.logN) + n);
        v0[i] = a.pre_scaled ? x.x : mul_shoup(x.x, c.w, c.ws, q);
        v1[i] = a.pre_scaled ? x.y : mul_shoup(x.y, c.w, c.ws, q);
    }
    for (int j = j_lo; j < j_hi; j++) {
        const int pj = a.dst_prime[j];
        const ModQ m = modq[pj];
        Dot3 d0, d1;
        dot3_clear(d0);
        dot3_clear(d1);
#pragma unroll
        for (int i = 0; i < NS; i++) {
            const u64 h = a.hat[i * a.hat_ld + pj].w;
            dot3_add(d0, v0[i], h);
            dot3_add(d1, v1[i], h);
        }
        *(ulonglong2 *)(dst + ((size_t)a.dst_slot[j] << a.logN) + n) = make_ulonglong2(dot3_reduce(d0, m), dot3_reduce(d1, m));
    }
}

// All digits of a ModUp in one launch (blockIdx.z = digit): the conversion of every digit to the limbs it does not
// own, plus the copy of its own limbs (already in NTT form in `own`) into its slice of the extended polynomial.
#define BCONV_MAX_DIGITS 4
struct BConvDigits {
    BConvArgs d[BCONV_MAX_DIGITS];  // d[0].split applies to every digit
    const u64 *own;        // [n_polys][.][N] NTT form, polynomial stride own_stride
    size_t own_stride;
    uint8_t own_lo[BCONV_MAX_DIGITS], own_hi[BCONV_MAX_DIGITS];
};
template <int NS>
__global__ __launch_bounds__(256) void bconv_digits_kernel(BConvDigits g, const ModQ *__restrict__ modq) {
    const BConvArgs &a = g.d[blockIdx.z];
    const int S = g.d[0].split > 1 ? g.d[0].split : 1;
    const int poly = blockIdx.y / S, part = blockIdx.y % S;
    const int per = (a.n_dst + S - 1) / S, j_lo = part * per, j_hi = min(a.n_dst, j_lo + per);
    const size_t n = ((size_t)blockIdx.x * 256 + threadIdx.x) * 2;
    const u64 *src = a.src + poly * a.src_poly_stride;
    u64 *dst = a.dst + poly * a.dst_poly_stride;
    u64 v0[NS], v1[NS];
#pragma unroll
    for (int i = 0; i < NS; i++) {
        v0[i] = v1[i] = 0;
        if (i < a.n_src) {
            const u64 q = modq[a.src_prime[i]].q;
            const Cst c = a.inv[i];
            const ulonglong2 x = *(const ulonglong2 *)(src + ((size_t)a.src_slot[i] << a.logN) + n);
            v0[i] = a.pre_scaled ? x.x : mul_shoup(x.x, c.w, c.ws, q);
            v1[i] = a.pre_scaled ? x.y : mul_shoup(x.y, c.w, c.ws, q);
        }
    }
    for (int j = j_lo; j < j_hi; j++) {
        const int pj = a.dst_prime[j];
        const ModQ m = modq[pj];
        Dot3 d0, d1;
        dot3_clear(d0);
        dot3_clear(d1);
#pragma unroll
        for (int i = 0; i < NS; i++) {
            if (i < a.n_src) {
                const u64 h = a.hat[i * a.hat_ld + pj].w;
                dot3_add(d0, v0[i], h);
                dot3_add(d1, v1[i], h);
            }
        }
        *(ulonglong2 *)(dst + ((size_t)a.dst_slot[j] << a.logN) + n) = make_ulonglong2(dot3_reduce(d0, m), dot3_reduce(d1, m));
    }
    const u64 *own = g.own + poly * g.own_stride;
    for (int j = g.own_lo[blockIdx.z] + part; j < g.own_hi[blockIdx.z]; j += S)
        *(ulonglong2 *)(dst + ((size_t)j << a.logN) + n) = *(const ulonglong2 *)(own + ((size_t)j << a.logN) + n);
}

// grid = (N / 256, n_polys) coefficients x polynomials
// A conversion over few polynomials has too few coefficient blocks to fill the GPU (N / 512 workgroups per polynomial
// and digit, each thread walking every target limb in turn): its target limbs are then dealt to `split` workgroups.
static int bconv_split(int N, int n_units, int n_dst) {
    const int blocks = (N / 512) * n_units;
    int S = (1536 + blocks - 1) / blocks;
    if (S > 8) S = 8;
    if (S > n_dst) S = n_dst;
    return S < 1 ? 1 : S;
}

// the lazy dot products of the register kernels hold 8 terms of 60 x 60 bits
static bool lazy_dot_ok(const hemm_context *c) {
    for (u64 q : c->primes)
        if ((q >> 60) != 0) return false;
    return true;
}

void launch_bconv(const hemm_context *c, const BConvArgs &a_in, const ModQ *modq, int N, int n_polys, hipStream_t s) {
    BConvArgs a = a_in;
    account(c, TR_BCONV, (size_t)(a.n_src + a.n_dst) * n_polys * N * 8);
    const bool reg = a.n_src <= 8 && N >= 512 && lazy_dot_ok(c);
    a.split = reg ? bconv_split(N, n_polys, a.n_dst) : 1;
    dim3 block(256), wide(N / 256, n_polys), pair(N / 512, n_polys * a.split);
    switch (reg ? a.n_src : 0) {
#define BCONV_CASE(K) case K: hipLaunchKernelGGL(bconv_reg_kernel<K>, pair, block, 0, s, a, modq); break;
        BCONV_CASE(1) BCONV_CASE(2) BCONV_CASE(3) BCONV_CASE(4) BCONV_CASE(5) BCONV_CASE(6) BCONV_CASE(7) BCONV_CASE(8)
#undef BCONV_CASE
        default: hipLaunchKernelGGL(bconv_kernel, wide, block, (size_t)a.n_src * 256 * 8, s, a, modq);
    }
}

struct DigitMap {
    uint8_t digit_of[HEMM_MAX_PRIMES];  // for limb j < nq: owning digit; 255 for special limbs
};

// acc[pol][j][n] = sum_d x_d[j][n] * evk[d][pol][prime(j)][n],  x_d = in[j] when limb j belongs to
// digit d (its residues were never converted), ext[d][j] otherwise.
__global__ __launch_bounds__(256) void inner_product_kernel(const u64 *__restrict__ in, const u64 *__restrict__ ext,
                                                            const u64 *__restrict__ evk, u64 *__restrict__ acc,
                                                            const ModQ *__restrict__ modq, LimbList ll, DigitMap dm,
                                                            int beta, int n_ext, int n_full, int logN) {
    const int j = blockIdx.y;
    const int prime = ll.idx[j];
    const ModQ m = modq[prime];
    const size_t n = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t N = (size_t)1 << logN;
    u128_t sb = {0, 0}, sa = {0, 0};
    for (int d = 0; d < beta; d++) {
        const u64 x = (dm.digit_of[j] == d) ? in[(size_t)j * N + n] : ext[((size_t)d * n_ext + j) * N + n];
        const u64 kb = evk[(((size_t)d * 2 + 0) * n_full + prime) * N + n];
        const u64 ka = evk[(((size_t)d * 2 + 1) * n_full + prime) * N + n];
        add128(sb, mul64wide(x, kb));
        add128(sa, mul64wide(x, ka));
    }
    acc[(size_t)j * N + n] = barrett128(sb, m);
    acc[((size_t)n_ext + j) * N + n] = barrett128(sa, m);
}

// out[p][j] = (a[p][j] - t[p][j]) * cst[j]  (+ add[p][j] when add != nullptr)
__global__ __launch_bounds__(256) void sub_scale_kernel(const u64 *__restrict__ a, size_t a_stride,
                                                        const u64 *__restrict__ t, size_t t_stride,
                                                        const u64 *__restrict__ add, size_t add_stride,
                                                        int add_polys, u64 *__restrict__ out, size_t out_stride,
                                                        const ModQ *__restrict__ modq, CstList cl, int n_limbs,
                                                        int logN) {
    const int limb = blockIdx.y % n_limbs, poly = blockIdx.y / n_limbs;
    const u64 q = modq[limb].q;
    const size_t e = ((size_t)limb << logN) + (size_t)blockIdx.x * 256 + threadIdx.x;
    u64 r = mul_shoup(submod(a[poly * a_stride + e], t[poly * t_stride + e], q), cl.c[limb].w, cl.c[limb].ws, q);
    if (add != nullptr && poly < add_polys) r = addmod(r, add[poly * add_stride + e], q);
    out[poly * out_stride + e] = r;
}

// t[p][j][n] = last[p][n] mod q_j
__global__ __launch_bounds__(256) void spread_kernel(const u64 *__restrict__ last, u64 *__restrict__ t,
                                                     size_t t_stride, const ModQ *__restrict__ modq, int n_limbs,
                                                     int logN) {
    const int limb = blockIdx.y % n_limbs, poly = blockIdx.y / n_limbs;
    const size_t n = (size_t)blockIdx.x * 256 + threadIdx.x;
    const u64 x = last[((size_t)poly << logN) + n];
    t[poly * t_stride + ((size_t)limb << logN) + n] = reduce64(x, modq[limb]);
}

u64 shoup_h(u64 w, u64 q) { return (u64)((((unsigned __int128)w) << 64) / q); }

// Hoisted rotations, several per output, combined with masks in the extended basis:
//   y[o][pol][j][n] = sum_{t in group o} mask_t[j][n] * ( sum_d ext_t[d][j][pi_t(n)] * evk_t[d][pol][j][n]
//                                                         + [pol = 0, j < nq] (P mod q_j) * b_t[j][pi_t(n)] )
// The automorphism is an index map on the reads (aligned 2^m-blocks map to aligned 2^m-blocks in the
// bit-reversed order, so a wavefront still reads whole 512-byte runs); the key is streamed once.
// MODE 1: the launch covers only limbs of primes below 2^44 (double-precision path); MODE 2: only the others
// (integer path); MODE 0: any limb, path chosen per workgroup.  jmap lists the n_j limbs of the launch.  The integer
// path keeps 128-bit accumulators and needs more registers, so on large launches the double-precision limbs get a
// kernel of their own and run at a higher occupancy; small launches stay whole (two part-filled launches cost more).
template <int MODE, bool COMPACT>
__device__ __forceinline__ void hoisted_terms_body(const RotTermDev *__restrict__ terms,
                                                   const u32 *__restrict__ group_off, u64 *__restrict__ y,
                                                   const ModQ *__restrict__ modq, const double *__restrict__ fp,
                                                   const LimbList &ll, const CstList &pmod, int nq, int E, int beta,
                                                   int n_full, int logN, int b_premultiplied, int n_out,
                                                   const LimbList &jmap, int n_j, const u32 *__restrict__ koff) {
    // A thread owns the residue pair (n, n+1): the automorphism maps an aligned pair to an aligned pair
    // (possibly swapped), so every access is a 16-byte load or store.
    // Work is dealt out by SOURCE chunk.  The automorphism maps aligned 512-coefficient chunks onto aligned
    // chunks, so output chunk c of output o gathers from exactly one source chunk s = pi_o(c).  Workgroups go
    // round-robin over the 8 XCDs (each with its own L2); XCD x takes the source chunks s = x (mod 8), and for
    // one (limb, s) all outputs run back to back.  Every XCD then only ever reads its own eighth of the
    // rotation sources and fetches it once, instead of each L2 pulling in all of them.
    const int cbits = logN - 9;
    const u32 chunks = 1u << cbits;
    u32 o, j, chunk;
    if (chunks >= 8) {
        const u32 xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3, per = chunks >> 3;
        o = slot % (u32)n_out;
        // Limbs of 60-bit primes are bound by integer arithmetic, limbs below 2^44 (double precision) by memory:
        // the limb index runs faster than the chunk index so that both kinds are resident together and the two
        // limits overlap instead of alternating.
        const u32 rest = slot / (u32)n_out;
        const u32 s = (rest / (u32)n_j) * 8u + xcd;
        j = jmap.idx[rest % (u32)n_j];
        (void)per;
        // output chunk whose gather lands in source chunk s: the low cbits+1 bits of the exponent 2 br(i) + 1
        // are fixed by the chunk; multiply them by g^-1 (mod 2^(cbits+1))
        u32 g = terms[group_off[o]].galois;
        if (g == 0) g = 1;
        u32 ginv = g;                      // g * g = 1 (mod 8); two Newton steps give 12 bits
        ginv *= 2u - g * ginv;
        ginv *= 2u - g * ginv;
        const u32 msk = (2u << cbits) - 1u;
        const u32 es = 2u * (__brev(s) >> (32 - cbits)) + 1u;
        const u32 eo = (es * ginv) & msk;
        chunk = __brev(eo >> 1) >> (32 - cbits);
    } else {
        o = blockIdx.x % (u32)n_out;
        const u32 rest = blockIdx.x / (u32)n_out;
        chunk = rest % chunks;
        j = jmap.idx[rest / chunks];
    }
    // output, limb and chunk are the same for the whole workgroup; the byte tables above are read with vector loads,
    // so say it: everything derived from them (the bases of all streams) then lives in scalar registers
    o = __builtin_amdgcn_readfirstlane(o);
    j = __builtin_amdgcn_readfirstlane(j);
    chunk = __builtin_amdgcn_readfirstlane(chunk);
    const int prime = __builtin_amdgcn_readfirstlane((int)ll.idx[j]);
    const u32 n = (chunk * 256 + threadIdx.x) * 2;
    const double fq = fp[4 * prime];
    const size_t N = (size_t)1 << logN;
    u64 rb[2], ra[2];
    if (MODE == 1 || (MODE == 0 && fq != 0.0 && beta <= 6)) {
        const FpMod f{fq, fp[4 * prime + 1]};
        double fb[2], fa[2];
        hoisted_pair_fp<COMPACT>(terms, group_off, koff, f, j < nq ? (double)pmod.c[j].w : 0.0, j, o, prime, n, nq, E,
                                 beta, n_full, logN, b_premultiplied, fb, fa);
        rb[0] = f.canonical(fb[0]);
        rb[1] = f.canonical(fb[1]);
        ra[0] = f.canonical(fa[0]);
        ra[1] = f.canonical(fa[1]);
    } else {
        hoisted_pair_int<COMPACT>(terms, group_off, koff, modq[prime], pmod, j, o, prime, n, nq, E, beta, n_full, logN,
                                  b_premultiplied, rb, ra);
    }
    stream_store2(y + (((size_t)o * 2 + 0) * E + j) * N + n, rb[0], rb[1]);
    stream_store2(y + (((size_t)o * 2 + 1) * E + j) * N + n, ra[0], ra[1]);
}

// Term lists of up to HOISTED_ARG_TERMS terms and outputs travel in the kernel arguments (no staging copy before
// the launch); longer lists are read from device memory.
static_assert(sizeof(RotTermDev) == 80, "the C ABI builds these records on the host");
#define HOISTED_ARG_TERMS 32
struct HoistedArgs {
    RotTermDev t[HOISTED_ARG_TERMS];
    u32 off[HOISTED_ARG_TERMS + 1];
};
// Register budget for five waves per SIMD (96 registers): the double-precision form needs 72 (74 on compact keys) and
// the integer form 93 - 96; the mixed form would take 109 and run at four waves, capped it spills two or three registers
// and gains a wave.  COMPACT: the key layout of the launch (hoisted.h, key_limb).
#define HOISTED_KERNEL __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(5))) void
template <int MODE, bool COMPACT>
HOISTED_KERNEL hoisted_terms_kernel(const HoistedArgs args, u64 *__restrict__ y, const ModQ *__restrict__ modq,
                                    const double *__restrict__ fp, LimbList ll, CstList pmod, int nq, int E, int beta,
                                    int n_full, int logN, int b_premultiplied, int n_out, LimbList jmap, int n_j,
                                    const u32 *__restrict__ koff) {
    hoisted_terms_body<MODE, COMPACT>(args.t, args.off, y, modq, fp, ll, pmod, nq, E, beta, n_full, logN,
                                      b_premultiplied, n_out, jmap, n_j, koff);
}
template <int MODE, bool COMPACT>
HOISTED_KERNEL hoisted_terms_list_kernel(const RotTermDev *__restrict__ terms, const u32 *__restrict__ group_off,
                                         u64 *__restrict__ y, const ModQ *__restrict__ modq,
                                         const double *__restrict__ fp, LimbList ll, CstList pmod, int nq, int E,
                                         int beta, int n_full, int logN, int b_premultiplied, int n_out, LimbList jmap,
                                         int n_j, const u32 *__restrict__ koff) {
    hoisted_terms_body<MODE, COMPACT>(terms, group_off, y, modq, fp, ll, pmod, nq, E, beta, n_full, logN,
                                      b_premultiplied, n_out, jmap, n_j, koff);
}
#undef HOISTED_KERNEL

struct LinTermDev {
    const u64 *ct;    // [n_polys][.][N]
    const u64 *mask;  // [nq][N] or nullptr (factor 1)
    u64 stride;       // polynomial stride of ct
    u64 galois;       // 0: mask used as is; else the mask is read through the automorphism X -> X^galois
};
// out[o][p][j] = sum_{t in group o} mask_t[j] * ct_t[p][j], p < n_polys (<= 3).  A thread owns the residue pair
// (n, n+1) of one limb for every polynomial (16-byte accesses; under an automorphism an aligned pair stays an
// aligned pair, possibly swapped), so each mask residue is read once; integer products are summed as 128-bit
// values and reduced every 4 terms.
template <int n_polys>
__device__ __forceinline__ void masked_sum_body(const LinTermDev *__restrict__ terms, const u32 *__restrict__ group_off,
                                                u64 *__restrict__ out, const ModQ *__restrict__ modq,
                                                const double *__restrict__ fp, int nq, int logN, int n_out) {
    // Workgroups go round-robin over the 8 XCDs, each with its own L2.  The outputs of one launch mostly
    // sum the same ciphertexts under different masks, so all outputs of a (limb, 512-coefficient) tile are
    // placed back to back on one XCD: the ciphertext tile is fetched from HBM once instead of once per output.
    const u32 tiles = (u32)nq << (logN - 9);
    u32 o, tile;
    if ((tiles & 7u) == 0) {
        const u32 xcd = blockIdx.x & 7u, slot = blockIdx.x >> 3;
        o = slot % (u32)n_out;
        tile = (slot / (u32)n_out) * 8u + xcd;
    } else {
        o = blockIdx.x % (u32)n_out;
        tile = blockIdx.x / (u32)n_out;
    }
    const int j = (int)(tile >> (logN - 9));
    const ModQ m = modq[j];
    const size_t N = (size_t)1 << logN;
    const u32 n = ((tile & ((1u << (logN - 9)) - 1)) * 256 + threadIdx.x) * 2;
    const size_t e = (size_t)j * N + n;
    const double fq = fp[4 * j];
    // mask residues of the pair (n, n+1), read through the term's automorphism if it has one
    auto load_mask = [&](const LinTermDev &T) -> ulonglong2 {
        if (T.galois == 0) return stream_load2(T.mask + e);
        const u32 np = galois_index(n, (u32)T.galois, logN);
        ulonglong2 v = *(const ulonglong2 *)(T.mask + (size_t)j * N + (np & ~1u));
        if (np & 1u) {
            const u64 tmp = v.x;
            v.x = v.y;
            v.y = tmp;
        }
        return v;
    };
    if (fq != 0.0) {
        // primes below 2^44: exact double-precision products (6 FP64 operations each)
        const FpMod f{fq, fp[4 * j + 1]};
        double facc[n_polys][2];
#pragma unroll
        for (int p = 0; p < n_polys; p++) facc[p][0] = facc[p][1] = 0.0;
        int since = 0;
        for (u32 t = group_off[o]; t < group_off[o + 1]; t++) {
            const LinTermDev T = terms[t];
            if (T.mask != nullptr) {
                const ulonglong2 mk = load_mask(T);
                const double dm0 = u64_to_double(mk.x), dm1 = u64_to_double(mk.y);
#pragma unroll
                for (int p = 0; p < n_polys; p++) {
                    const ulonglong2 cv = *(const ulonglong2 *)(T.ct + p * T.stride + e);
                    facc[p][0] += f.mul(u64_to_double(cv.x), dm0);
                    facc[p][1] += f.mul(u64_to_double(cv.y), dm1);
                }
            } else {
#pragma unroll
                for (int p = 0; p < n_polys; p++) {
                    const ulonglong2 cv = *(const ulonglong2 *)(T.ct + p * T.stride + e);
                    facc[p][0] += u64_to_double(cv.x);
                    facc[p][1] += u64_to_double(cv.y);
                }
            }
            if (++since == 64) {  // a term adds at most q: keep the running sums far below 2^52
#pragma unroll
                for (int p = 0; p < n_polys; p++) {
                    facc[p][0] = f.reduce(facc[p][0]);
                    facc[p][1] = f.reduce(facc[p][1]);
                }
                since = 0;
            }
        }
#pragma unroll
        for (int p = 0; p < n_polys; p++)
            stream_store2(out + ((size_t)o * n_polys + p) * nq * N + e, f.canonical(facc[p][0]), f.canonical(facc[p][1]));
        return;
    }
    u64 acc[n_polys][2];
    u128_t lazy[n_polys][2];
#pragma unroll
    for (int p = 0; p < n_polys; p++)
        for (int h = 0; h < 2; h++) {
            acc[p][h] = 0;
            lazy[p][h].lo = lazy[p][h].hi = 0;
        }
    int pending = 0;
    for (u32 t = group_off[o]; t < group_off[o + 1]; t++) {
        const LinTermDev T = terms[t];
        if (T.mask != nullptr) {
            const ulonglong2 mk = load_mask(T);
#pragma unroll
            for (int p = 0; p < n_polys; p++) {
                const ulonglong2 cv = *(const ulonglong2 *)(T.ct + p * T.stride + e);
                add128(lazy[p][0], mul64wide(cv.x, mk.x));
                add128(lazy[p][1], mul64wide(cv.y, mk.y));
            }
            if (++pending == 4) {
#pragma unroll
                for (int p = 0; p < n_polys; p++)
                    for (int h = 0; h < 2; h++) {
                        acc[p][h] = addmod(acc[p][h], barrett128(lazy[p][h], m), m.q);
                        lazy[p][h].lo = lazy[p][h].hi = 0;
                    }
                pending = 0;
            }
        } else {
#pragma unroll
            for (int p = 0; p < n_polys; p++) {
                const ulonglong2 cv = *(const ulonglong2 *)(T.ct + p * T.stride + e);
                acc[p][0] = addmod(acc[p][0], cv.x, m.q);
                acc[p][1] = addmod(acc[p][1], cv.y, m.q);
            }
        }
    }
#pragma unroll
    for (int p = 0; p < n_polys; p++) {
        if (pending) {
            acc[p][0] = addmod(acc[p][0], barrett128(lazy[p][0], m), m.q);
            acc[p][1] = addmod(acc[p][1], barrett128(lazy[p][1], m), m.q);
        }
        stream_store2(out + ((size_t)o * n_polys + p) * nq * N + e, acc[p][0], acc[p][1]);
    }
}

// Short term lists (the usual case: a handful of masked terms per output) travel in the kernel arguments, which
// saves the staging copy in front of the launch; longer lists are read from device memory.
#define MASKED_ARG_TERMS 32
struct MaskedArgs {
    LinTermDev t[MASKED_ARG_TERMS];
    u32 off[MASKED_ARG_TERMS + 1];
};
template <int n_polys>
__global__ __launch_bounds__(256) void masked_sum_kernel(const MaskedArgs args, u64 *__restrict__ out,
                                                         const ModQ *__restrict__ modq, const double *__restrict__ fp,
                                                         int nq, int logN, int n_out) {
    masked_sum_body<n_polys>(args.t, args.off, out, modq, fp, nq, logN, n_out);
}
template <int n_polys>
__global__ __launch_bounds__(256) void masked_sum_list_kernel(const LinTermDev *__restrict__ terms,
                                                              const u32 *__restrict__ group_off, u64 *__restrict__ out,
                                                              const ModQ *__restrict__ modq, const double *__restrict__ fp,
                                                              int nq, int logN, int n_out) {
    masked_sum_body<n_polys>(terms, group_off, out, modq, fp, nq, logN, n_out);
}

// acc3 (+)= sum_{g < G} (b1 b2, a1 b2 + a2 b1, a1 a2) of t1[g], t2[g], each [2][nq][N]
__global__ __launch_bounds__(256) void tensor_batch_kernel(const u64 *__restrict__ t1, const u64 *__restrict__ t2,
                                                           int G, u64 *__restrict__ acc3, size_t acc_stride,
                                                           int accumulate, const ModQ *__restrict__ modq, int nq,
                                                           int logN) {
    const int j = blockIdx.y;
    const ModQ m = modq[j];
    const size_t N = (size_t)1 << logN, P = (size_t)nq * N;
    const size_t e = (size_t)j * N + (size_t)blockIdx.x * 256 + threadIdx.x;
    u64 d0 = 0, d1 = 0, d2 = 0;
    if (accumulate) {
        d0 = acc3[e];
        d1 = acc3[acc_stride + e];
        d2 = acc3[2 * acc_stride + e];
    }
    for (int g = 0; g < G; g++) {
        const u64 b1 = t1[(size_t)g * 2 * P + e], a1 = t1[(size_t)g * 2 * P + P + e];
        const u64 b2 = t2[(size_t)g * 2 * P + e], a2 = t2[(size_t)g * 2 * P + P + e];
        d0 = addmod(d0, mulmod(b1, b2, m), m.q);
        u128_t t = mul64wide(a1, b2);
        add128(t, mul64wide(a2, b1));
        d1 = addmod(d1, barrett128(t, m), m.q);
        d2 = addmod(d2, mulmod(a1, a2, m), m.q);
    }
    acc3[e] = d0;
    acc3[acc_stride + e] = d1;
    acc3[2 * acc_stride + e] = d2;
}

// The same for up to TENSOR_MAX_GROUPS accumulators in one launch (blockIdx.z = group): the giant-step groups of a
// chain of shifts are a few such sums of at most g pairs each, and one launch over all of them fills the GPU where
// a launch per group is a single part-filled round of workgroups.  A thread owns the residue pair (n, n+1).
struct TensorGroups {
    const u64 *t1[TENSOR_MAX_GROUPS], *t2[TENSOR_MAX_GROUPS];
    u64 *acc[TENSOR_MAX_GROUPS];
    int n_pairs[TENSOR_MAX_GROUPS], accumulate[TENSOR_MAX_GROUPS];
};
__global__ __launch_bounds__(256) void tensor_groups_kernel(TensorGroups gr, size_t acc_stride,
                                                            const ModQ *__restrict__ modq, int nq, int logN) {
    const int j = blockIdx.y, z = blockIdx.z;
    const ModQ m = modq[j];
    const size_t N = (size_t)1 << logN, P = (size_t)nq * N;
    const size_t e = (size_t)j * N + ((size_t)blockIdx.x * 256 + threadIdx.x) * 2;
    const u64 *__restrict__ t1 = gr.t1[z], *__restrict__ t2 = gr.t2[z];
    u64 *__restrict__ acc3 = gr.acc[z];
    const int G = gr.n_pairs[z];
    ulonglong2 d0 = make_ulonglong2(0, 0), d1 = d0, d2 = d0;
    if (gr.accumulate[z]) {
        d0 = *(const ulonglong2 *)(acc3 + e);
        d1 = *(const ulonglong2 *)(acc3 + acc_stride + e);
        d2 = *(const ulonglong2 *)(acc3 + 2 * acc_stride + e);
    }
    for (int g = 0; g < G; g++) {
        const ulonglong2 b1 = stream_load2(t1 + (size_t)g * 2 * P + e), a1 = stream_load2(t1 + (size_t)g * 2 * P + P + e);
        const ulonglong2 b2 = *(const ulonglong2 *)(t2 + (size_t)g * 2 * P + e);
        const ulonglong2 a2 = *(const ulonglong2 *)(t2 + (size_t)g * 2 * P + P + e);
        d0.x = addmod(d0.x, mulmod(b1.x, b2.x, m), m.q);
        d0.y = addmod(d0.y, mulmod(b1.y, b2.y, m), m.q);
        u128_t t = mul64wide(a1.x, b2.x);
        add128(t, mul64wide(a2.x, b1.x));
        d1.x = addmod(d1.x, barrett128(t, m), m.q);
        t = mul64wide(a1.y, b2.y);
        add128(t, mul64wide(a2.y, b1.y));
        d1.y = addmod(d1.y, barrett128(t, m), m.q);
        d2.x = addmod(d2.x, mulmod(a1.x, a2.x, m), m.q);
        d2.y = addmod(d2.y, mulmod(a1.y, a2.y, m), m.q);
    }
    *(ulonglong2 *)(acc3 + e) = d0;
    *(ulonglong2 *)(acc3 + acc_stride + e) = d1;
    *(ulonglong2 *)(acc3 + 2 * acc_stride + e) = d2;
}

}  // namespace

// ---- tables -----------------------------------------------------------------------------------
// For every active chain length nq and digit d: inv[i] and hat[i][prime] of the digit's limbs;
// for ModDown: the same for the special basis.  Laid out in one device array of (w, ws) pairs.
struct KsTables {
    std::vector<Cst> host;
    Cst *dev = nullptr;
    std::vector<std::vector<size_t>> inv_off, hat_off;  // [nq][d]
    size_t p_inv_off = 0, p_hat_off = 0;
    std::vector<Cst> pinv;                               // P^-1 mod q_j
    std::vector<std::vector<Cst>> qlinv;                 // [l][j<l]  q_l^-1 mod q_j
    // merged ModDown + rescale: basis {q_{nq-1}} U P dropped at once
    std::vector<size_t> drop_inv_off, drop_hat_off;      // [nq]
    std::vector<std::vector<Cst>> dropinv;               // [nq][j<nq-1]  (P q_{nq-1})^-1 mod q_j
    size_t pinv_off = 0;                                 // device copies of pinv / dropinv[nq] / qlinv[l]
    std::vector<size_t> dropinv_off, qlinv_off;
    // (1/N) (S/q_i)^-1 mod q_i in source order: the constant an inverse transform of N = 2^16 ends with when a basis
    // conversion follows it.  modup: per chain length nq, limbs 0 .. nq-1 (each limb in its own digit's basis).
    size_t p_invn_off = 0;
    std::vector<size_t> drop_invn_off, modup_invn_off;   // [nq]
    size_t ones_off = 0;                                 // the constant 1 for every prime (a one-source conversion
                                                         // with it is a plain reduction into the target prime)
};

static KsTables *g_tables_of(const hemm_context *c);

static void build_tables(const hemm_context *c, KsTables &t) {
    const int nQ = c->nQ, K = c->nP, T = nQ + K, alpha = c->alpha;
    auto push_basis = [&](const std::vector<int> &src, size_t &inv_off, size_t &hat_off) {
        inv_off = t.host.size();
        for (size_t i = 0; i < src.size(); i++) {
            u64 qi = c->primes[src[i]], prod = 1;
            for (size_t k = 0; k < src.size(); k++)
                if (k != i) prod = h_mulmod(prod, c->primes[src[k]] % qi, qi);
            u64 inv = h_invmod(prod, qi);
            t.host.push_back(Cst{inv, shoup_h(inv, qi)});
        }
        hat_off = t.host.size();
        for (size_t i = 0; i < src.size(); i++)
            for (int pj = 0; pj < T; pj++) {
                u64 tq = c->primes[pj], prod = 1;
                for (size_t k = 0; k < src.size(); k++)
                    if (k != i) prod = h_mulmod(prod, c->primes[src[k]] % tq, tq);
                t.host.push_back(Cst{prod, shoup_h(prod, tq)});
            }
    };
    t.inv_off.assign(nQ + 1, {});
    t.hat_off.assign(nQ + 1, {});
    for (int nq = 1; nq <= nQ; nq++) {
        int beta = (nq + alpha - 1) / alpha;
        t.inv_off[nq].resize(beta);
        t.hat_off[nq].resize(beta);
        for (int d = 0; d < beta; d++) {
            std::vector<int> src;
            for (int j = d * alpha; j < std::min(nq, (d + 1) * alpha); j++) src.push_back(j);
            push_basis(src, t.inv_off[nq][d], t.hat_off[nq][d]);
        }
    }
    if (K > 0) {
        std::vector<int> src;
        for (int k = 0; k < K; k++) src.push_back(nQ + k);
        push_basis(src, t.p_inv_off, t.p_hat_off);
    }
    t.pinv.resize(nQ);
    for (int j = 0; j < nQ; j++) {
        u64 q = c->primes[j], P = 1;
        for (int k = 0; k < K; k++) P = h_mulmod(P, c->primes[nQ + k] % q, q);
        u64 inv = h_invmod(P, q);
        t.pinv[j] = Cst{inv, shoup_h(inv, q)};
    }
    t.qlinv.assign(nQ, {});
    for (int l = 1; l < nQ; l++)
        for (int j = 0; j < l; j++) {
            u64 q = c->primes[j];
            u64 inv = h_invmod(c->primes[l] % q, q);
            t.qlinv[l].push_back(Cst{inv, shoup_h(inv, q)});
        }
    t.drop_inv_off.assign(nQ + 1, 0);
    t.drop_hat_off.assign(nQ + 1, 0);
    t.dropinv.assign(nQ + 1, {});
    if (K > 0)
        for (int nq = 2; nq <= nQ; nq++) {
            std::vector<int> src;
            src.push_back(nq - 1);
            for (int k = 0; k < K; k++) src.push_back(nQ + k);
            push_basis(src, t.drop_inv_off[nq], t.drop_hat_off[nq]);
            for (int j = 0; j < nq - 1; j++) {
                u64 q = c->primes[j], prod = c->primes[nq - 1] % q;
                for (int k = 0; k < K; k++) prod = h_mulmod(prod, c->primes[nQ + k] % q, q);
                u64 inv = h_invmod(prod, q);
                t.dropinv[nq].push_back(Cst{inv, shoup_h(inv, q)});
            }
        }
    t.pinv_off = t.host.size();
    for (auto &x : t.pinv) t.host.push_back(x);
    t.dropinv_off.assign(nQ + 1, 0);
    for (int nq = 0; nq <= nQ; nq++) {
        t.dropinv_off[nq] = t.host.size();
        for (auto &x : t.dropinv[nq]) t.host.push_back(x);
    }
    t.qlinv_off.assign(nQ, 0);
    for (int l = 0; l < nQ; l++) {
        t.qlinv_off[l] = t.host.size();
        for (auto &x : t.qlinv[l]) t.host.push_back(x);
    }
    // inverse-transform constants with 1/N folded in, read back from the inv entries built above
    auto invn = [&](size_t inv_off, const std::vector<int> &src) {
        const size_t off = t.host.size();
        for (size_t i = 0; i < src.size(); i++) {
            const u64 q = c->primes[src[i]];
            const u64 v = h_mulmod(t.host[inv_off + i].w, h_invmod((u64)c->N % q, q), q);
            t.host.push_back(Cst{v, shoup_h(v, q)});
        }
        return off;
    };
    if (K > 0) {
        std::vector<int> src;
        for (int k = 0; k < K; k++) src.push_back(nQ + k);
        t.p_invn_off = invn(t.p_inv_off, src);
    }
    t.drop_invn_off.assign(nQ + 1, 0);
    if (K > 0)
        for (int nq = 2; nq <= nQ; nq++) {
            std::vector<int> src;
            src.push_back(nq - 1);
            for (int k = 0; k < K; k++) src.push_back(nQ + k);
            t.drop_invn_off[nq] = invn(t.drop_inv_off[nq], src);
        }
    t.modup_invn_off.assign(nQ + 1, 0);
    for (int nq = 1; nq <= nQ; nq++) {
        const int beta = (nq + alpha - 1) / alpha;
        t.modup_invn_off[nq] = t.host.size();
        for (int d = 0; d < beta; d++) {
            std::vector<int> src;
            for (int j = d * alpha; j < std::min(nq, (d + 1) * alpha); j++) src.push_back(j);
            invn(t.inv_off[nq][d], src);
        }
    }
    t.ones_off = t.host.size();
    for (int pj = 0; pj < T; pj++) t.host.push_back(Cst{1, 0});
    HEMM_HIP(hipMalloc((void **)&t.dev, t.host.size() * sizeof(Cst)));
    HEMM_HIP(hipMemcpy(t.dev, t.host.data(), t.host.size() * sizeof(Cst), hipMemcpyHostToDevice));
}

// tables live beside the context (created on first use, destroyed with it)
#include <map>
#include <mutex>
// The registry is never destroyed: contexts can be released from static destructors of other translation
// units (a cached mask holding the last reference), which may run after this file's statics would be gone.
struct KsRegistry {
    std::map<const hemm_context *, KsTables *> tabs;
    std::mutex mu;
};
static KsRegistry &ks_registry() {
    static KsRegistry *r = new KsRegistry();
    return *r;
}
static KsTables *g_tables_of(const hemm_context *c) {
    KsRegistry &r = ks_registry();
    std::lock_guard<std::mutex> lk(r.mu);
    auto it = r.tabs.find(c);
    if (it != r.tabs.end()) return it->second;
    KsTables *t = new KsTables();
    build_tables(c, *t);
    r.tabs[c] = t;
    return t;
}
void hemm_keyswitch_tables_free(const hemm_context *c) {
    KsRegistry &r = ks_registry();
    std::lock_guard<std::mutex> lk(r.mu);
    auto it = r.tabs.find(c);
    if (it == r.tabs.end()) return;
    (void)hipFree(it->second->dev);
    delete it->second;
    r.tabs.erase(it);
}

// scratch (u64 words) needed by key switching / rescale at full width
size_t hemm_scratch_words(const hemm_context *c) {
    const size_t N = c->N, T = c->nQ + c->nP;
    return ((size_t)c->dnum + 7) * T * N;
}
u64 *hemm_scratch(hemm_context *c) {
    if (!c->d_scratch) {
        c->scratch_bytes = hemm_scratch_words(c) * sizeof(u64);
        HEMM_HIP(hipMalloc((void **)&c->d_scratch, c->scratch_bytes));
    }
    return c->d_scratch;
}

// ---- ModUp ------------------------------------------------------------------------------------
// in: [nq][N] NTT form.  ext: [beta][nq+K][N]; limbs owned by digit d are NOT written in ext[d]
// unless fill_own is set (they equal `in`).  coef: scratch [nq][N].
void launch_modup(hemm_context *c, const u64 *in, int nq, u64 *ext, u64 *coef, bool fill_own, hipStream_t s) {
    KsTables *t = g_tables_of(c);
    const int K = c->nP, E = nq + K, alpha = c->alpha, beta = (nq + alpha - 1) / alpha;
    const size_t N = c->N;
    HEMM_HIP(hipMemcpyAsync(coef, in, (size_t)nq * N * 8, hipMemcpyDeviceToDevice, s));
    account(c, TR_POINTWISE, (size_t)2 * nq * N * 8);
    launch_ntt(c, coef, limbs_default(c, nq, 0), nq, 1, (size_t)nq * N, true, s);
    for (int d = 0; d < beta; d++) {
        const int lo = d * alpha, hi = std::min(nq, lo + alpha);
        BConvArgs a;
        memset(&a, 0, sizeof(a));
        a.src = coef;
        a.dst = ext + (size_t)d * E * N;
        a.inv = t->dev + t->inv_off[nq][d];
        a.hat = t->dev + t->hat_off[nq][d];
        a.n_src = hi - lo;
        a.hat_ld = c->nQ + c->nP;
        a.logN = c->logN;
        if (a.n_src > 32) throw std::invalid_argument("digit wider than 32 limbs");
        LimbList pl, sl;
        memset(&pl, 0, sizeof(pl));
        memset(&sl, 0, sizeof(sl));
        for (int i = 0; i < a.n_src; i++) {
            a.src_slot[i] = (uint8_t)(lo + i);
            a.src_prime[i] = (uint8_t)(lo + i);
        }
        int nd = 0;
        for (int j = 0; j < E; j++) {
            if (j >= lo && j < hi) continue;
            a.dst_slot[nd] = (uint8_t)j;
            a.dst_prime[nd] = (uint8_t)(j < nq ? j : c->nQ + (j - nq));
            pl.idx[nd] = a.dst_prime[nd];
            sl.idx[nd] = (uint8_t)j;
            nd++;
        }
        a.n_dst = nd;
        if (nd > 0) {
            launch_bconv(c, a, c->d_modq, (int)N, 1, s);
            launch_ntt_slots(c, a.dst, pl, sl, nd, 1, (size_t)E * N, false, s);
        }
        if (fill_own)
            HEMM_HIP(hipMemcpyAsync(a.dst + (size_t)lo * N, in + (size_t)lo * N, (size_t)(hi - lo) * N * 8,
                                    hipMemcpyDeviceToDevice, s));
    }
}

// acc: [2][nq+K][N]
void launch_inner_product(hemm_context *c, const u64 *in, const u64 *ext, const u64 *evk, int nq, u64 *acc,
                          hipStream_t s) {
    const int K = c->nP, E = nq + K, alpha = c->alpha, beta = (nq + alpha - 1) / alpha;
    DigitMap dm;
    memset(&dm, 255, sizeof(dm));
    if (in != nullptr)
        for (int j = 0; j < nq; j++) dm.digit_of[j] = (uint8_t)(j / alpha);
    dim3 grid(c->N / 256, E), block(256);
    account(c, TR_KEYPROD, (size_t)(3 * beta * E + 2 * E) * c->N * 8);
    hipLaunchKernelGGL(inner_product_kernel, grid, block, 0, s, in, ext, evk, acc, c->d_modq,
                       limbs_default(c, nq, 1), dm, beta, E, c->nQ + c->nP, c->logN);
}

// acc: [n_polys][nq+K][N] NTT (special limbs are overwritten with their coefficient form).
// out[p] = ModDown(acc[p]) (+ add[p] for p < add_polys).  conv: scratch [n_polys][nq][N].
void launch_moddown(hemm_context *c, u64 *acc, int nq, int n_polys, u64 *out, size_t out_stride, const u64 *add,
                    size_t add_stride, int add_polys, u64 *conv, hipStream_t s) {
    KsTables *t = g_tables_of(c);
    const int K = c->nP, E = nq + K;
    const size_t N = c->N;
    LimbList pl;
    memset(&pl, 0, sizeof(pl));
    for (int k = 0; k < K; k++) pl.idx[k] = (uint8_t)(c->nQ + k);
    launch_ntt(c, acc + (size_t)nq * N, pl, K, n_polys, (size_t)E * N, true, s);
    BConvArgs a;
    memset(&a, 0, sizeof(a));
    a.src = acc;
    a.src_poly_stride = (size_t)E * N;
    a.dst = conv;
    a.dst_poly_stride = (size_t)nq * N;
    a.inv = t->dev + t->p_inv_off;
    a.hat = t->dev + t->p_hat_off;
    a.n_src = K;
    a.n_dst = nq;
    a.hat_ld = c->nQ + c->nP;
    a.logN = c->logN;
    if (K > 32) throw std::invalid_argument("more than 32 special primes");
    for (int k = 0; k < K; k++) {
        a.src_slot[k] = (uint8_t)(nq + k);
        a.src_prime[k] = (uint8_t)(c->nQ + k);
    }
    for (int j = 0; j < nq; j++) {
        a.dst_slot[j] = (uint8_t)j;
        a.dst_prime[j] = (uint8_t)j;
    }
    launch_bconv(c, a, c->d_modq, (int)N, n_polys, s);
    const dim3 block(256);
    launch_ntt(c, conv, limbs_default(c, nq, 0), nq, n_polys, (size_t)nq * N, false, s);
    CstList cl;
    for (int j = 0; j < nq; j++) cl.c[j] = t->pinv[j];
    dim3 g2(N / 256, nq * n_polys);
    account(c, TR_POINTWISE, (size_t)(3 * n_polys + add_polys) * nq * N * 8);
    hipLaunchKernelGGL(sub_scale_kernel, g2, block, 0, s, acc, (size_t)E * N, conv, (size_t)nq * N, add, add_stride,
                       add_polys, out, out_stride, c->d_modq, cl, nq, c->logN);
}

// Full key switch of `in` ([nq][N], NTT) with `evk` ([dnum][2][nQ+K][N]):
// out[0] = ks_b (+ add_b), out[1] = ks_a; out poly stride out_stride.
void launch_keyswitch(hemm_context *c, const u64 *in, const u64 *evk, int nq, u64 *out, size_t out_stride,
                      const u64 *add_b, hipStream_t s, u32 galois, bool b_rotates, const u64 *add_a) {
    if (c->nP < 1) throw std::invalid_argument("key switching needs special primes");
    const int K = c->nP, E = nq + K, beta = (nq + c->alpha - 1) / c->alpha;
    const size_t N = c->N;
    u64 *sc = hemm_scratch(c);
    u64 *coef = sc;                              // [nq][N]   (reused as conv[2][nq] needs 2*nq)
    u64 *ext = coef + (size_t)2 * (c->nQ) * N;   // [beta][E][N]
    u64 *acc = ext + (size_t)beta * E * N;       // [2][E][N]
    launch_modup_batch(c, in, (size_t)nq * N, nq, 1, ext, coef, s, galois);   // same arithmetic as launch_modup
    if (b_rotates && (galois == 0 || N < 512)) throw std::invalid_argument("add_b rotates only with the key switch's input");
    if (add_a != nullptr && (N < 512 || add_b == nullptr || b_rotates))
        throw std::invalid_argument("an addend for the second polynomial needs N >= 512 and one for the first");
    if (N >= 512) {
        // the key product as a hoisted sum of one term under the identity automorphism: P * add_b joins the sum in
        // the extended basis, so the ModDown needs no addend and ends in the forward transform's fused tail
        // (identical residues: every step is exact modular arithmetic in the same order)
        RotTermDev term[2];
        memset(term, 0, sizeof(term));
        term[0].ext = ext;
        term[0].b = add_b;
        term[0].evk = evk;
        term[0].galois = 1;
        term[0].pt_galois = 1;
        if (galois != 0 && b_rotates) {   // ext holds the rotated digits already: only add_b goes through the automorphism
            term[0].galois = galois;
            term[0].flags = ROT_TERM_EXT_ROTATED;
        }
        int n_terms = 1;
        if (add_a != nullptr) {   // (add_b, add_a) as a term without a key: P times both joins the sum on the chain limbs
            term[0].b = nullptr;
            term[1].ext = add_a;
            term[1].b = add_b;
            term[1].galois = 1;
            term[1].pt_galois = 1;
            n_terms = 2;
        }
        const u32 off[2] = {0, (u32)n_terms};
        launch_hoisted_terms_args(c, term, n_terms, off, 1, nq, acc, false, s);
        launch_moddown_batch(c, acc, nq, 2, 0, out, out_stride, coef, s);
        return;
    }
    launch_inner_product(c, in, ext, evk, nq, acc, s);
    launch_moddown(c, acc, nq, 2, out, out_stride, add_b, 0, add_b ? 1 : 0, coef, s);
}

// in: [n_polys][nq][N] -> out: [n_polys][nq-1][N]; sc: scratch of n_polys * nq * N words, fully written before it
// is read
static void rescale_with(hemm_context *c, KsTables *t, u64 *sc, const u64 *in, size_t in_stride, u64 *out,
                         size_t out_stride, int nq, int n_polys, hipStream_t s) {
    const size_t N = c->N;
    u64 *last = sc;                               // [n_polys][N]
    u64 *tt = sc + (size_t)n_polys * N;           // [n_polys][nq-1][N]
    LimbList pl, ident;
    memset(&pl, 0, sizeof(pl));
    pl.idx[0] = (uint8_t)(nq - 1);
    for (int j = 0; j < HEMM_MAX_PRIMES; j++) ident.idx[j] = (uint8_t)j;
    if (!launch_intt_from(c, in + (size_t)(nq - 1) * N, in_stride, last, pl, ident, 1, n_polys, N, s)) {
        for (int p = 0; p < n_polys; p++)
            HEMM_HIP(hipMemcpyAsync(last + (size_t)p * N, in + p * in_stride + (size_t)(nq - 1) * N, N * 8,
                                    hipMemcpyDeviceToDevice, s));
        launch_ntt(c, last, pl, 1, n_polys, N, true, s);
    }
    if (c->logN == 16 && lazy_dot_ok(c)) {
        // the reduction of the last limb's coefficients into every remaining prime is a one-source conversion with
        // the constant 1: computed inside the first pass of the forward transform
        ConvSources cs;
        memset(&cs, 0, sizeof(cs));
        cs.d[0].src = last;
        cs.d[0].hat = t->dev + t->ones_off;
        cs.d[0].src_poly_stride = N;
        cs.d[0].n_src = 1;
        cs.hat_ld = c->nQ + c->nP;
        if (launch_ntt_converted(c, cs, tt, limbs_default(c, nq - 1, 0), ident, nq - 1, n_polys, (size_t)(nq - 1) * N, s,
                                 in, in_stride, out, out_stride, t->dev + t->qlinv_off[nq - 1]))
            return;
    }
    dim3 grid(N / 256, (nq - 1) * n_polys), block(256);
    account(c, TR_POINTWISE, (size_t)n_polys * nq * N * 8);
    hipLaunchKernelGGL(spread_kernel, grid, block, 0, s, last, tt, (size_t)(nq - 1) * N, c->d_modq, nq - 1, c->logN);
    if (launch_ntt_sub_scale(c, tt, nq - 1, n_polys, in, in_stride, out, out_stride, t->dev + t->qlinv_off[nq - 1], s))
        return;
    launch_ntt(c, tt, limbs_default(c, nq - 1, 0), nq - 1, n_polys, (size_t)(nq - 1) * N, false, s);
    CstList cl;
    for (int j = 0; j < nq - 1; j++) cl.c[j] = t->qlinv[nq - 1][j];
    account(c, TR_POINTWISE, (size_t)3 * n_polys * (nq - 1) * N * 8);
    hipLaunchKernelGGL(sub_scale_kernel, grid, block, 0, s, in, in_stride, tt, (size_t)(nq - 1) * N,
                       (const u64 *)nullptr, (size_t)0, 0, out, out_stride, c->d_modq, cl, nq - 1, c->logN);
}

void launch_rescale(hemm_context *c, const u64 *in, size_t in_stride, u64 *out, size_t out_stride, int nq,
                    int n_polys, hipStream_t s) {
    if (nq < 2) throw std::invalid_argument("rescale needs at least two limbs");
    rescale_with(c, g_tables_of(c), hemm_scratch(c), in, in_stride, out, out_stride, nq, n_polys, s);
}

// ---- rescale for callers that cannot allocate ----------------------------------------------------
// The scratch of the call below lives in the library's own device image: 32 limbs of N = 2^16 (16 MiB) per GPU the
// library runs on, held until the process ends.  Host code never passes the array's name to a kernel or a copy: the
// name is only a handle for hipGetSymbolAddress, which yields the array's address on the device that is current,
// and each device has its own.
#include "../../include/hemm.h"   // HEMM_STATIC_SCRATCH_WORDS: the limit callers size against is the array's size
#define HEMM_MAX_DEVICES 64
static __device__ __align__(256) u64 scratch[HEMM_STATIC_SCRATCH_WORDS];
static u64 *g_static_scratch[HEMM_MAX_DEVICES];   // per device, filled by hemm_static_setup

size_t hemm_static_scratch_words() { return HEMM_STATIC_SCRATCH_WORDS; }

// Set-up for launch_rescale_static, run by hemm_context_create with the context's device current: resolves the
// device address of the scratch array on that device (once per device) and builds the context's constant tables,
// so that the call itself has nothing left to allocate.
static std::mutex &static_setup_mutex() {
    static std::mutex *mu = new std::mutex();
    return *mu;
}
void hemm_static_setup(hemm_context *c) {
    std::lock_guard<std::mutex> lk(static_setup_mutex());
    if (c->device < 0 || c->device >= HEMM_MAX_DEVICES) throw std::invalid_argument("device index out of range");
    if (g_static_scratch[c->device] == nullptr) {
        u64 *ptr = nullptr;
        HEMM_HIP(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
        if (ptr == nullptr) throw std::runtime_error("hipGetSymbolAddress returned no address for the scratch array");
        g_static_scratch[c->device] = ptr;
    }
    (void)g_tables_of(c);
}

void launch_rescale_static(hemm_context *c, const u64 *in, size_t in_stride, u64 *out, size_t out_stride, int nq,
                           int n_polys, hipStream_t s) {
    if (nq < 2) throw std::invalid_argument("rescale needs at least two limbs");
    if (n_polys < 1 || (size_t)n_polys * (size_t)nq * (size_t)c->N > HEMM_STATIC_SCRATCH_WORDS)
        throw std::invalid_argument("n_polys * nq * N exceeds the static scratch of " +
                                    std::to_string((size_t)HEMM_STATIC_SCRATCH_WORDS) + " words (HEMM_STATIC_SCRATCH_WORDS)");
    int dev = -1;
    HEMM_HIP(hipGetDevice(&dev));
    if (dev != c->device) throw std::invalid_argument("the context belongs to another device than the current one");
    KsTables *t = nullptr;
    {
        KsRegistry &r = ks_registry();
        std::lock_guard<std::mutex> lk(r.mu);
        auto it = r.tabs.find(c);
        if (it != r.tabs.end()) t = it->second;
    }
    if (dev < 0 || dev >= HEMM_MAX_DEVICES) throw std::invalid_argument("device index out of range");
    u64 *sc = nullptr;
    {
        std::lock_guard<std::mutex> lk(static_setup_mutex());
        sc = g_static_scratch[dev];
    }
    if (t == nullptr || sc == nullptr) throw std::runtime_error("context was not set up by hemm_context_create");
    rescale_with(c, t, sc, in, in_stride, out, out_stride, nq, n_polys, s);
}

// ---- compact evaluation keys -----------------------------------------------------------------------
// out: the compact layout the hoisted kernels read (hoisted.h, key_limb) of a plain key [dnum][2][n_full][N]
__global__ __launch_bounds__(256) void key_compact_kernel(const u64 *__restrict__ evk, char *__restrict__ out,
                                                          const u32 *__restrict__ koff, const double *__restrict__ fp,
                                                          int n_full, int logN) {
    const size_t N = (size_t)1 << logN;
    const int prime = blockIdx.y % n_full, slice = blockIdx.y / n_full;   // slice = digit * 2 + polynomial
    const size_t n = ((size_t)blockIdx.x * 256 + threadIdx.x) * 2;
    const ulonglong2 v = *(const ulonglong2 *)(evk + ((size_t)slice * n_full + prime) * N + n);
    char *limb = out + ((size_t)slice * koff[n_full] + koff[prime]) * (2 * N);
    if (fp[4 * prime] != 0.0) {
        u32 *pair = (u32 *)(limb + n * 6);
        pair[0] = (u32)v.x;
        pair[1] = (u32)v.y;
        pair[2] = (u32)(v.x >> 32) | ((u32)(v.y >> 32) << 16);
    } else {
        *(ulonglong2 *)(limb + n * 8) = v;
    }
}
// the inverse: the plain key [dnum][2][n_full][N] of a compact one (lossless: 6 bytes hold any residue below 2^48)
__global__ __launch_bounds__(256) void key_expand_kernel(const char *__restrict__ in, u64 *__restrict__ evk,
                                                         const u32 *__restrict__ koff, const double *__restrict__ fp,
                                                         int n_full, int logN) {
    const size_t N = (size_t)1 << logN;
    const int prime = blockIdx.y % n_full, slice = blockIdx.y / n_full;
    const size_t n = ((size_t)blockIdx.x * 256 + threadIdx.x) * 2;
    const char *limb = in + ((size_t)slice * koff[n_full] + koff[prime]) * (2 * N);
    ulonglong2 v;
    if (fp[4 * prime] != 0.0) {
        const u32 *pair = (const u32 *)(limb + n * 6);
        const u32 hi = pair[2];
        v.x = ((u64)(hi & 0xffffu) << 32) | pair[0];
        v.y = ((u64)(hi >> 16) << 32) | pair[1];
    } else {
        v = *(const ulonglong2 *)(limb + n * 8);
    }
    *(ulonglong2 *)(evk + ((size_t)slice * n_full + prime) * N + n) = v;
}
size_t key_compact_words(const hemm_context *c) {
    return (size_t)c->dnum * 2 * c->key_off[c->nQ + c->nP] * (2 * (size_t)c->N) / 8;
}
void launch_key_compact(const hemm_context *c, const u64 *evk, u64 *out, hipStream_t s) {
    if (c->N < 512) throw std::invalid_argument("compact keys need N >= 512");
    const int n_full = c->nQ + c->nP;
    account(c, TR_POINTWISE, (size_t)c->dnum * 2 * n_full * c->N * 8 + key_compact_words(c) * 8);
    hipLaunchKernelGGL(key_compact_kernel, dim3(c->N / 512, c->dnum * 2 * n_full), dim3(256), 0, s, evk, (char *)out,
                       c->d_key_off, c->d_fp, n_full, c->logN);
}

void launch_key_expand(const hemm_context *c, const u64 *compact, u64 *evk, hipStream_t s) {
    if (c->N < 512) throw std::invalid_argument("compact keys need N >= 512");
    const int n_full = c->nQ + c->nP;
    account(c, TR_POINTWISE, (size_t)c->dnum * 2 * n_full * c->N * 8 + key_compact_words(c) * 8);
    hipLaunchKernelGGL(key_expand_kernel, dim3(c->N / 512, c->dnum * 2 * n_full), dim3(256), 0, s, (const char *)compact, evk,
                       c->d_key_off, c->d_fp, n_full, c->logN);
}

// ---- batched / hoisted forms ---------------------------------------------------------------------
// in: [n_in][.][N] (polynomial stride in_stride, first nq limbs used) -> ext [n_in][beta][nq+K][N], own
// limbs of every digit filled.  coef: workspace [n_in][nq][N].
// The form of launch_modup_batch in which the conversions of all digits and the copies of their own limbs are one
// launch (the first pass of the forward transform) is the one that can read its input through an automorphism.
bool modup_through_automorphism_ok(const hemm_context *c, int nq) {
    const int K = c->nP, E = nq + K, alpha = c->alpha, beta = (nq + alpha - 1) / alpha;
    return c->logN == 16 && alpha <= 8 && alpha <= CONV_MAX_SOURCES && beta <= BCONV_MAX_DIGITS &&
           beta <= CONV_MAX_DIGITS && beta * E <= 255 && beta * E - nq <= HEMM_MAX_PRIMES && lazy_dot_ok(c);
}

void launch_modup_batch(hemm_context *c, const u64 *in, size_t in_stride, int nq, int n_in, u64 *ext, u64 *coef,
                        hipStream_t s, u32 galois) {
    KsTables *t = g_tables_of(c);
    const int K = c->nP, E = nq + K, alpha = c->alpha, beta = (nq + alpha - 1) / alpha;
    const size_t N = c->N;
    if (alpha > 32) throw std::invalid_argument("digit wider than 32 limbs");
    const LimbList chain = limbs_default(c, nq, 0);
    LimbList ident;
    for (int j = 0; j < HEMM_MAX_PRIMES; j++) ident.idx[j] = (uint8_t)j;
    const bool fold = c->logN == 16;
    if (galois != 0 && !modup_through_automorphism_ok(c, nq))
        throw std::invalid_argument("this ModUp shape has no form that reads its input through an automorphism");
    if (!launch_intt_from(c, in, in_stride, coef, chain, ident, nq, n_in, (size_t)nq * N, s,
                          fold ? t->dev + t->modup_invn_off[nq] : nullptr, galois)) {
        HEMM_HIP(hipMemcpy2DAsync(coef, (size_t)nq * N * 8, in, in_stride * 8, (size_t)nq * N * 8, n_in,
                                  hipMemcpyDeviceToDevice, s));
        launch_ntt(c, coef, chain, nq, n_in, (size_t)nq * N, true, s);
    }
    // One conversion launch and one forward transform for all digits when the ring size allows: the converted
    // limbs of every digit are addressed as slots d*E + j of one extended polynomial per input.
    const bool joint = c->N >= 512 && alpha <= 8 && beta <= BCONV_MAX_DIGITS && beta * E <= 255 &&
                       beta * E - nq <= HEMM_MAX_PRIMES && lazy_dot_ok(c);
    BConvDigits g;
    memset(&g, 0, sizeof(g));
    g.own = in;
    g.own_stride = in_stride;
    LimbList jp, js;
    memset(&jp, 0, sizeof(jp));
    memset(&js, 0, sizeof(js));
    int n_joint = 0;
    for (int d = 0; d < beta; d++) {
        const int lo = d * alpha, hi = std::min(nq, lo + alpha);
        BConvArgs a;
        memset(&a, 0, sizeof(a));
        a.src = coef;
        a.src_poly_stride = (size_t)nq * N;
        a.dst = ext + (size_t)d * E * N;
        a.dst_poly_stride = (size_t)beta * E * N;
        a.inv = t->dev + t->inv_off[nq][d];
        a.hat = t->dev + t->hat_off[nq][d];
        a.n_src = hi - lo;
        a.hat_ld = c->nQ + c->nP;
        a.logN = c->logN;
        a.pre_scaled = fold ? 1 : 0;
        LimbList pl, sl;
        memset(&pl, 0, sizeof(pl));
        memset(&sl, 0, sizeof(sl));
        for (int i = 0; i < a.n_src; i++) {
            a.src_slot[i] = (uint8_t)(lo + i);
            a.src_prime[i] = (uint8_t)(lo + i);
        }
        int nd = 0;
        for (int j = 0; j < E; j++) {
            if (j >= lo && j < hi) continue;
            a.dst_slot[nd] = (uint8_t)j;
            a.dst_prime[nd] = (uint8_t)(j < nq ? j : c->nQ + (j - nq));
            pl.idx[nd] = a.dst_prime[nd];
            sl.idx[nd] = (uint8_t)j;
            if (joint) {
                jp.idx[n_joint] = a.dst_prime[nd];
                js.idx[n_joint] = (uint8_t)(d * E + j);
                n_joint++;
            }
            nd++;
        }
        a.n_dst = nd;
        if (joint) {
            g.d[d] = a;
            g.own_lo[d] = (uint8_t)lo;
            g.own_hi[d] = (uint8_t)hi;
            continue;
        }
        if (nd > 0) {
            launch_bconv(c, a, c->d_modq, (int)N, n_in, s);
            launch_ntt_slots(c, a.dst, pl, sl, nd, n_in, (size_t)beta * E * N, false, s);
        }
        HEMM_HIP(hipMemcpy2DAsync(a.dst + (size_t)lo * N, (size_t)beta * E * N * 8, in + (size_t)lo * N, in_stride * 8,
                                  (size_t)(hi - lo) * N * 8, n_in, hipMemcpyDeviceToDevice, s));
    }
    if (!joint) return;
    if (fold) {
        // the conversions of all digits inside the first pass of the forward transform; the same launch copies every
        // digit's own limbs into its slice
        ConvSources cs;
        memset(&cs, 0, sizeof(cs));
        cs.hat_ld = c->nQ + c->nP;
        int l = 0;
        for (int d = 0; d < beta; d++) {
            cs.d[d].src = g.d[d].src;
            cs.d[d].hat = g.d[d].hat;
            cs.d[d].src_poly_stride = g.d[d].src_poly_stride;
            cs.d[d].n_src = g.d[d].n_src;
            for (int i = 0; i < g.d[d].n_src; i++) cs.d[d].src_slot[i] = g.d[d].src_slot[i];
            for (int j = 0; j < g.d[d].n_dst; j++) cs.digit_of[l++] = (uint8_t)d;
        }
        cs.copy_src = in;
        cs.copy_src_stride = in_stride;
        cs.n_copy = nq;
        cs.copy_galois = galois;
        for (int j = 0; j < nq; j++) {
            cs.copy_src_slot[j] = (uint8_t)j;
            cs.copy_dst_slot[j] = (uint8_t)((j / alpha) * E + j);
        }
        if (launch_ntt_converted(c, cs, ext, jp, js, n_joint, n_in, (size_t)beta * E * N, s)) return;
    }
    if (galois != 0) throw std::invalid_argument("this ModUp shape has no form that reads through an automorphism");
    g.d[0].split = bconv_split((int)N, n_in * beta, E - alpha);
    const dim3 grid((unsigned)(N / 512), n_in * g.d[0].split, beta), block(256);
    const int widest = std::min(nq, alpha);
    account(c, TR_BCONV, (size_t)n_in * (beta * E + nq) * N * 8);   // every digit's sources and its whole slice
    if (widest <= 2)
        hipLaunchKernelGGL(bconv_digits_kernel<2>, grid, block, 0, s, g, c->d_modq);
    else if (widest <= 5)
        hipLaunchKernelGGL(bconv_digits_kernel<5>, grid, block, 0, s, g, c->d_modq);
    else
        hipLaunchKernelGGL(bconv_digits_kernel<8>, grid, block, 0, s, g, c->d_modq);
    launch_ntt_slots(c, ext, jp, js, n_joint, n_in, (size_t)beta * E * N, false, s);
}


// Algorithmic bytes of one hoisted sum: every distinct source once (its extended digits and, where present, its b),
// every term's key once, full masks and plaintext factors once per distinct pointer (run tables by their own size),
// every output once.
static size_t hoisted_bytes(const hemm_context *c, const RotTermDev *t, int n_terms, int n_out, int nq) {
    const size_t limb = (size_t)c->N * 8;
    const int E = nq + c->nP, beta = (nq + c->alpha - 1) / c->alpha;
    std::vector<const u64 *> seen;
    auto first = [&](const u64 *p) {
        if (p == nullptr) return false;
        for (const u64 *q : seen)
            if (q == p) return false;
        seen.push_back(p);
        return true;
    };
    size_t bytes = (size_t)n_out * 2 * E * limb;
    // key bytes of the launch's limbs per (digit, polynomial): 6 bytes per residue of a prime below 2^44 in a compact key
    size_t compact_slice = 0;
    for (int j = 0; j < E; j++) {
        const int prime = j < nq ? j : c->nQ + (j - nq);
        compact_slice += (size_t)c->N * ((c->primes[prime] >> 44) == 0 ? 6 : 8);
    }
    for (int i = 0; i < n_terms; i++) {
        if (t[i].evk == nullptr) {   // no key: the two polynomials on the chain limbs
            if (first(t[i].ext)) bytes += (size_t)nq * limb;
        } else {
            bytes += (size_t)2 * beta * ((t[i].flags & ROT_TERM_COMPACT_KEY) ? compact_slice : (size_t)E * limb);   // the key
            if (first(t[i].ext)) bytes += (size_t)beta * E * limb;
        }
        if (first(t[i].b)) bytes += (size_t)nq * limb;
        if (first(t[i].ext2)) bytes += (size_t)beta * E * limb;
        if (first(t[i].b2)) bytes += (size_t)nq * limb;
        const size_t mask_bytes = t[i].mask_shift ? (size_t)E * 2 * (limb >> t[i].mask_shift) : (size_t)E * limb;
        if (first(t[i].mask)) bytes += mask_bytes;
        if (first(t[i].mask2)) bytes += mask_bytes;
        if (first(t[i].pt)) bytes += (size_t)E * limb;
    }
    return bytes;
}

// terms / group_off are DEVICE arrays (n_out + 1 offsets); y: [n_out][2][nq+K][N]
// P mod q_j (and Shoup quotient) for the chain limbs j < nq
static CstList p_mod_chain(const hemm_context *c, int nq) {
    CstList pm;
    memset(&pm, 0, sizeof(pm));
    for (int j = 0; j < nq; j++) {
        u64 q = c->primes[j], P = 1;
        for (int k = 0; k < c->nP; k++) P = h_mulmod(P, c->primes[c->nQ + k] % q, q);
        pm.c[j] = Cst{P, shoup_h(P, q)};
    }
    return pm;
}

// Limbs of the extended basis handled in double precision (primes below 2^44, at most 6 digits) and the others;
// true when the launch is large enough (in workgroups) for one kernel per kind to pay.
static bool split_limbs(const hemm_context *c, int nq, int beta, int n_out, LimbList &fpl, int &n_fp, LimbList &il,
                        int &n_int, LimbList &all) {
    const LimbList ll = limbs_default(c, nq, 1);
    const int E = nq + c->nP;
    memset(&fpl, 0, sizeof(fpl));
    memset(&il, 0, sizeof(il));
    n_fp = n_int = 0;
    for (int j = 0; j < HEMM_MAX_PRIMES; j++) all.idx[j] = (uint8_t)j;
    for (int j = 0; j < E; j++) {
        if (c->primes[ll.idx[j]] < (1ull << 44) && beta <= 6)
            fpl.idx[n_fp++] = (uint8_t)j;
        else
            il.idx[n_int++] = (uint8_t)j;
    }
    return n_fp > 0 && n_int > 0 && (size_t)n_out * E * (c->N / 512) >= 16384;
}

void launch_hoisted_terms(hemm_context *c, const void *terms_dev, const u32 *group_off_dev, int n_out, int nq, u64 *y,
                          bool b_premultiplied, hipStream_t s, const void *terms_host, int n_terms, bool compact) {
    const int K = c->nP, E = nq + K, beta = (nq + c->alpha - 1) / c->alpha;
    if (terms_host != nullptr) account(c, TR_KEYPROD, hoisted_bytes(c, (const RotTermDev *)terms_host, n_terms, n_out, nq));
    const CstList pm = p_mod_chain(c, nq);
    if (c->N < 512) throw std::invalid_argument("hoisted terms need N >= 512");
    // with more than 6 digits the limbs of primes below 2^44 go through the integer path, which reads whole words
    if (compact && beta > 6) throw std::invalid_argument("compact keys need at most 6 digits");
    // the kernels address a key by 32-bit byte offsets
    if ((size_t)c->dnum * 2 * (c->nQ + c->nP) * c->N * 8 >= ((size_t)1 << 32))
        throw std::invalid_argument("hoisted terms need keys below 4 GiB");
    LimbList fpl, il, all;
    int n_fp, n_int;
    const bool split = split_limbs(c, nq, beta, n_out, fpl, n_fp, il, n_int, all);
    const dim3 block(256);
    const size_t per_limb = (size_t)n_out * (c->N / 512);
    const LimbList ll = limbs_default(c, nq, 1);
    const RotTermDev *td = (const RotTermDev *)terms_dev;
    const int n_full = c->nQ + c->nP, pre = b_premultiplied ? 1 : 0;
#define HOISTED_LIST(MODE, COMPACT, GRID, JM, NJ)                                                                  \
    hipLaunchKernelGGL((hoisted_terms_list_kernel<MODE, COMPACT>), dim3((unsigned)(GRID)), block, 0, s, td,        \
                       group_off_dev, y, c->d_modq, c->d_fp, ll, pm, nq, E, beta, n_full, c->logN, pre, n_out, JM, \
                       NJ, c->d_key_off)
    if (!split) {
        if (compact)
            HOISTED_LIST(0, true, per_limb * E, all, E);
        else
            HOISTED_LIST(0, false, per_limb * E, all, E);
        return;
    }
    if (compact) {
        HOISTED_LIST(1, true, per_limb * n_fp, fpl, n_fp);
        HOISTED_LIST(2, true, per_limb * n_int, il, n_int);
    } else {
        HOISTED_LIST(1, false, per_limb * n_fp, fpl, n_fp);
        HOISTED_LIST(2, false, per_limb * n_int, il, n_int);
    }
#undef HOISTED_LIST
}
// the same with the term list (host memory, already merged: n_terms <= HOISTED_ARG_TERMS, n_out <= HOISTED_ARG_TERMS)
// passed in the kernel arguments
int hoisted_arg_capacity() { return HOISTED_ARG_TERMS; }
void launch_hoisted_terms_args(hemm_context *c, const void *terms_host, int n_terms, const u32 *group_off_host, int n_out,
                               int nq, u64 *y, bool b_premultiplied, hipStream_t s) {
    const int K = c->nP, E = nq + K, beta = (nq + c->alpha - 1) / c->alpha;
    const CstList pm = p_mod_chain(c, nq);
    if (c->N < 512) throw std::invalid_argument("hoisted terms need N >= 512");
    if (n_terms > HOISTED_ARG_TERMS || n_out > HOISTED_ARG_TERMS)
        throw std::invalid_argument("term list too long for the argument path");
    account(c, TR_KEYPROD, hoisted_bytes(c, (const RotTermDev *)terms_host, n_terms, n_out, nq));
    HoistedArgs a;
    memset(&a, 0, sizeof(a));
    memcpy(a.t, terms_host, (size_t)n_terms * sizeof(RotTermDev));
    memcpy(a.off, group_off_host, (size_t)(n_out + 1) * sizeof(u32));
    LimbList fpl, il, all;
    int n_fp, n_int;
    const bool split = split_limbs(c, nq, beta, n_out, fpl, n_fp, il, n_int, all);
    const dim3 block(256);
    const size_t per_limb = (size_t)n_out * (c->N / 512);
    const LimbList ll = limbs_default(c, nq, 1);
    const int n_full = c->nQ + c->nP, pre = b_premultiplied ? 1 : 0;
    const bool compact = n_terms > 0 && (((const RotTermDev *)terms_host)[0].flags & ROT_TERM_COMPACT_KEY) != 0;
    if (compact && beta > 6) throw std::invalid_argument("compact keys need at most 6 digits");
    if ((size_t)c->dnum * 2 * (c->nQ + c->nP) * c->N * 8 >= ((size_t)1 << 32))
        throw std::invalid_argument("hoisted terms need keys below 4 GiB");
#define HOISTED_ARGS(MODE, COMPACT, GRID, JM, NJ)                                                                  \
    hipLaunchKernelGGL((hoisted_terms_kernel<MODE, COMPACT>), dim3((unsigned)(GRID)), block, 0, s, a, y, c->d_modq, \
                       c->d_fp, ll, pm, nq, E, beta, n_full, c->logN, pre, n_out, JM, NJ, c->d_key_off)
    if (!split) {
        if (compact)
            HOISTED_ARGS(0, true, per_limb * E, all, E);
        else
            HOISTED_ARGS(0, false, per_limb * E, all, E);
        return;
    }
    if (compact) {
        HOISTED_ARGS(1, true, per_limb * n_fp, fpl, n_fp);
        HOISTED_ARGS(2, true, per_limb * n_int, il, n_int);
    } else {
        HOISTED_ARGS(1, false, per_limb * n_fp, fpl, n_fp);
        HOISTED_ARGS(2, false, per_limb * n_int, il, n_int);
    }
#undef HOISTED_ARGS
}

// y: [n_polys][nq+K][N] NTT (dropped limbs are clobbered).  drop_last = 0: out[p] = y[p] / P over nq limbs;
// drop_last = 1: out[p] = y[p] / (P q_{nq-1}) over nq-1 limbs (ModDown and rescale in one conversion).
// conv: workspace [n_polys][nq_out][N].
void launch_moddown_batch(hemm_context *c, u64 *y, int nq, int n_polys, int drop_last, u64 *out, size_t out_stride,
                          u64 *conv, hipStream_t s, bool slab) {
    KsTables *t = g_tables_of(c);
    const int K = c->nP, E = nq + K, nq_out = drop_last ? nq - 1 : nq;
    const size_t N = c->N;
    if (drop_last && nq < 2) throw std::invalid_argument("merged rescale needs at least two limbs");
    BConvArgs a;
    memset(&a, 0, sizeof(a));
    LimbList pl, sl;
    memset(&pl, 0, sizeof(pl));
    memset(&sl, 0, sizeof(sl));
    int ns = 0;
    if (drop_last) {
        a.src_slot[ns] = (uint8_t)(nq - 1);
        a.src_prime[ns] = (uint8_t)(nq - 1);
        ns++;
    }
    for (int k = 0; k < K; k++) {
        a.src_slot[ns] = (uint8_t)(nq + k);
        a.src_prime[ns] = (uint8_t)(c->nQ + k);
        ns++;
    }
    if (ns > 32) throw std::invalid_argument("more than 32 limbs dropped");
    for (int i = 0; i < ns; i++) {
        pl.idx[i] = a.src_prime[i];
        sl.idx[i] = a.src_slot[i];
    }
    const bool fold = c->logN == 16;   // the inverse transform ends with (1/N)(S/q_i)^-1: no scaling pass in the conversion
    // the three-launch form with one column-slab kernel in the middle, only on request: it moves a fifth less data but
    // runs at two waves per SIMD and is slower on every batch size measured
    if (slab && !(fold && lazy_dot_ok(c))) throw std::invalid_argument("the column-slab ModDown needs N = 2^16 and primes below 2^60");
    if (slab) {
        if (!launch_moddown_slab(c, y, (size_t)E * N, a.src_slot, a.src_prime, ns,
                            t->dev + (drop_last ? t->drop_invn_off[nq] : t->p_invn_off),
                            t->dev + (drop_last ? t->drop_hat_off[nq] : t->p_hat_off), c->nQ + c->nP, conv, nq_out, n_polys,
                            out, out_stride, t->dev + (drop_last ? t->dropinv_off[nq] : t->pinv_off), s))
            throw std::invalid_argument("the column-slab ModDown takes 4 or 5 dropped limbs");
        return;
    }
    launch_ntt_slots(c, y, pl, sl, ns, n_polys, (size_t)E * N, true, s,
                     fold ? t->dev + (drop_last ? t->drop_invn_off[nq] : t->p_invn_off) : nullptr);
    a.pre_scaled = fold ? 1 : 0;
    a.src = y;
    a.src_poly_stride = (size_t)E * N;
    a.dst = conv;
    a.dst_poly_stride = (size_t)nq_out * N;
    a.inv = t->dev + (drop_last ? t->drop_inv_off[nq] : t->p_inv_off);
    a.hat = t->dev + (drop_last ? t->drop_hat_off[nq] : t->p_hat_off);
    a.n_src = ns;
    a.n_dst = nq_out;
    a.hat_ld = c->nQ + c->nP;
    a.logN = c->logN;
    for (int j = 0; j < nq_out; j++) {
        a.dst_slot[j] = (uint8_t)j;
        a.dst_prime[j] = (uint8_t)j;
    }
    const dim3 block(256);
    const Cst *cst_dev = t->dev + (drop_last ? t->dropinv_off[nq] : t->pinv_off);
    if (fold && ns <= CONV_MAX_SOURCES && lazy_dot_ok(c)) {
        // the conversion is computed inside the first pass of the forward transform: no conversion launch, and the
        // converted limbs are neither written in coefficient form nor read back
        ConvSources cs;
        memset(&cs, 0, sizeof(cs));
        cs.d[0].src = y;
        cs.d[0].hat = a.hat;
        cs.d[0].src_poly_stride = a.src_poly_stride;
        cs.d[0].n_src = ns;
        for (int i = 0; i < ns; i++) cs.d[0].src_slot[i] = a.src_slot[i];
        cs.hat_ld = a.hat_ld;
        LimbList cl = limbs_default(c, nq_out, 0), ident;
        for (int j = 0; j < HEMM_MAX_PRIMES; j++) ident.idx[j] = (uint8_t)j;
        if (launch_ntt_converted(c, cs, conv, cl, ident, nq_out, n_polys, (size_t)nq_out * N, s, y, (size_t)E * N, out,
                                 out_stride, cst_dev))
            return;
    }
    launch_bconv(c, a, c->d_modq, (int)N, n_polys, s);
    if (launch_ntt_sub_scale(c, conv, nq_out, n_polys, y, (size_t)E * N, out, out_stride, cst_dev, s)) return;
    launch_ntt(c, conv, limbs_default(c, nq_out, 0), nq_out, n_polys, (size_t)nq_out * N, false, s);
    CstList cl;
    for (int j = 0; j < nq_out; j++) cl.c[j] = drop_last ? t->dropinv[nq][j] : t->pinv[j];
    dim3 g2(N / 256, nq_out * n_polys);
    account(c, TR_POINTWISE, (size_t)3 * n_polys * nq_out * N * 8);
    hipLaunchKernelGGL(sub_scale_kernel, g2, block, 0, s, y, (size_t)E * N, conv, (size_t)nq_out * N,
                       (const u64 *)nullptr, (size_t)0, 0, out, out_stride, c->d_modq, cl, nq_out, c->logN);
}


// Algorithmic bytes of a masked sum: distinct ciphertexts and masks once, outputs once.
static size_t masked_bytes(const hemm_context *c, const LinTermDev *t, int n_terms, int n_out, int nq, int n_polys) {
    const size_t limb = (size_t)c->N * 8;
    std::vector<const u64 *> seen;
    auto first = [&](const u64 *p) {
        if (p == nullptr) return false;
        for (const u64 *q : seen)
            if (q == p) return false;
        seen.push_back(p);
        return true;
    };
    size_t bytes = (size_t)n_out * n_polys * nq * limb;
    for (int i = 0; i < n_terms; i++) {
        if (first(t[i].ct)) bytes += (size_t)n_polys * nq * limb;
        if (first(t[i].mask)) bytes += (size_t)nq * limb;
    }
    return bytes;
}

void launch_masked_sum(hemm_context *c, const void *terms_dev, const u32 *group_off_dev, int n_out, int nq, int n_polys,
                       u64 *out, hipStream_t s, const void *terms_host, int n_terms) {
    if (n_polys > 3) throw std::invalid_argument("masked sums take at most 3 polynomials");
    if (terms_host != nullptr) account(c, TR_MASKED, masked_bytes(c, (const LinTermDev *)terms_host, n_terms, n_out, nq, n_polys));
    if (c->N < 512) throw std::invalid_argument("masked sums need N >= 512");
    dim3 grid((unsigned)(c->N / 512) * nq * n_out), block(256);
    const LinTermDev *td = (const LinTermDev *)terms_dev;
    if (n_polys == 1)
        hipLaunchKernelGGL(masked_sum_list_kernel<1>, grid, block, 0, s, td, group_off_dev, out, c->d_modq, c->d_fp, nq,
                           c->logN, n_out);
    else if (n_polys == 2)
        hipLaunchKernelGGL(masked_sum_list_kernel<2>, grid, block, 0, s, td, group_off_dev, out, c->d_modq, c->d_fp, nq,
                           c->logN, n_out);
    else
        hipLaunchKernelGGL(masked_sum_list_kernel<3>, grid, block, 0, s, td, group_off_dev, out, c->d_modq, c->d_fp, nq,
                           c->logN, n_out);
}
// table[run] = (value, floor(value * 2^64 / q)) of each run of a mask over the extended basis; *differs is set when
// some run is not constant
__global__ __launch_bounds__(256) void compact_mask_kernel(const u64 *__restrict__ mask, u64 *__restrict__ table,
                                                           size_t total, int shift, int logN,
                                                           const ModQ *__restrict__ modq, LimbList ll,
                                                           u32 *__restrict__ differs) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;        // limb * N + position
    if (i >= total) return;
    const size_t run = i >> shift;
    const u64 v = mask[i], first = mask[run << shift];
    if ((i & (((size_t)1 << shift) - 1)) == 0) {
        const u64 q = modq[ll.idx[i >> logN]].q;
        u64 rem = v, ws = 0;                                         // long division of v * 2^64 by q (v < q < 2^61)
        for (int b = 0; b < 64; b++) {
            rem <<= 1;
            ws <<= 1;
            if (rem >= q) {
                rem -= q;
                ws |= 1;
            }
        }
        table[2 * run] = v;
        table[2 * run + 1] = ws;
    }
    if (v != first) atomicOr(differs, 1u);
}
bool launch_compact_mask(hemm_context *c, const u64 *mask, int n_limbs, int shift, u64 *table, hipStream_t s) {
    if (n_limbs <= c->nP) throw std::invalid_argument("run tables are built for masks over the extended basis");
    u32 *flag = nullptr, h = 0;
    HEMM_HIP(hipMalloc((void **)&flag, sizeof(u32)));
    HEMM_HIP(hipMemcpyAsync(flag, &h, sizeof(u32), hipMemcpyHostToDevice, s));
    const size_t total = (size_t)n_limbs * c->N;
    hipLaunchKernelGGL(compact_mask_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, mask, table, total,
                       shift, c->logN, c->d_modq, limbs_default(c, n_limbs - c->nP, 1), flag);
    HEMM_HIP(hipMemcpyAsync(&h, flag, sizeof(u32), hipMemcpyDeviceToHost, s));
    HEMM_HIP(hipStreamSynchronize(s));
    HEMM_HIP(hipFree(flag));
    return h == 0;
}
// sum of `parts` consecutive partial results per output over the extended basis, residue pairs, canonical in and out
__global__ __launch_bounds__(256) void sum_parts_kernel(const u64 *__restrict__ part, int parts, u64 *__restrict__ y,
                                                        const ModQ *__restrict__ modq, LimbList ll, int E, int logN,
                                                        size_t pairs) {
    const size_t N = (size_t)1 << logN, poly_limbs = (size_t)2 * E;
    const size_t pair = (size_t)blockIdx.x * 256 + threadIdx.x;     // over [n_out][2][E][N/2]
    if (pair >= pairs) return;
    const size_t limb = (pair * 2) >> logN;                         // (o * 2 + p) * E + j
    const size_t o = limb / poly_limbs, within = limb % poly_limbs;
    const u64 q = modq[ll.idx[within % E]].q;
    const size_t e = within * N + ((pair * 2) & (N - 1));
    u64 a0 = 0, a1 = 0;
    for (int k = 0; k < parts; k++) {
        const ulonglong2 v = stream_load2(part + ((o * parts + k) * poly_limbs) * N + e);
        a0 = addmod(a0, v.x, q);
        a1 = addmod(a1, v.y, q);
    }
    stream_store2(y + (o * poly_limbs) * N + e, a0, a1);
}
void launch_sum_parts(hemm_context *c, const u64 *part, int parts, int n_out, int nq, u64 *y, hipStream_t s) {
    const int E = nq + c->nP;
    const size_t pairs = (size_t)n_out * 2 * E * (c->N / 2);
    account(c, TR_KEYPROD, (size_t)(parts + 1) * n_out * 2 * (nq + c->nP) * c->N * 8);
    hipLaunchKernelGGL(sum_parts_kernel, dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, s, part, parts, y, c->d_modq,
                       limbs_default(c, nq, 1), E, c->logN, pairs);
}
// the same with the term list in host memory (n_terms, n_out <= masked_arg_capacity()), passed in the kernel arguments
int masked_arg_capacity() { return MASKED_ARG_TERMS; }
void launch_masked_sum_args(hemm_context *c, const void *terms_host, int n_terms, const u32 *group_off_host, int n_out,
                            int nq, int n_polys, u64 *out, hipStream_t s) {
    if (n_polys > 3) throw std::invalid_argument("masked sums take at most 3 polynomials");
    if (c->N < 512) throw std::invalid_argument("masked sums need N >= 512");
    if (n_terms > MASKED_ARG_TERMS || n_out > MASKED_ARG_TERMS)
        throw std::invalid_argument("term list too long for the argument path");
    account(c, TR_MASKED, masked_bytes(c, (const LinTermDev *)terms_host, n_terms, n_out, nq, n_polys));
    MaskedArgs a;
    memset(&a, 0, sizeof(a));
    memcpy(a.t, terms_host, (size_t)n_terms * sizeof(LinTermDev));
    memcpy(a.off, group_off_host, (size_t)(n_out + 1) * sizeof(u32));
    dim3 grid((unsigned)(c->N / 512) * nq * n_out), block(256);
    if (n_polys == 1)
        hipLaunchKernelGGL(masked_sum_kernel<1>, grid, block, 0, s, a, out, c->d_modq, c->d_fp, nq, c->logN, n_out);
    else if (n_polys == 2)
        hipLaunchKernelGGL(masked_sum_kernel<2>, grid, block, 0, s, a, out, c->d_modq, c->d_fp, nq, c->logN, n_out);
    else
        hipLaunchKernelGGL(masked_sum_kernel<3>, grid, block, 0, s, a, out, c->d_modq, c->d_fp, nq, c->logN, n_out);
}

int tensor_max_groups() { return TENSOR_MAX_GROUPS; }
void launch_tensor_groups(hemm_context *c, const TensorGroupHost *g, int n_groups, int nq, size_t acc_stride,
                          hipStream_t s) {
    if (n_groups < 1 || n_groups > TENSOR_MAX_GROUPS) throw std::invalid_argument("between 1 and 8 groups per launch");
    if (c->N < 512) throw std::invalid_argument("grouped tensor sums need N >= 512");
    TensorGroups gr;
    memset(&gr, 0, sizeof(gr));
    size_t bytes = 0;
    for (int i = 0; i < n_groups; i++) {
        gr.t1[i] = g[i].t1;
        gr.t2[i] = g[i].t2;
        gr.acc[i] = g[i].acc;
        gr.n_pairs[i] = g[i].n_pairs;
        gr.accumulate[i] = g[i].accumulate ? 1 : 0;
        bytes += (size_t)(4 * g[i].n_pairs + (g[i].accumulate ? 6 : 3)) * nq * c->N * 8;
    }
    account(c, TR_TENSOR, bytes);
    hipLaunchKernelGGL(tensor_groups_kernel, dim3(c->N / 512, nq, n_groups), dim3(256), 0, s, gr, acc_stride, c->d_modq,
                       nq, c->logN);
}
void launch_tensor_batch(hemm_context *c, const u64 *t1, const u64 *t2, int G, int nq, u64 *acc3, size_t acc_stride,
                         bool accumulate, hipStream_t s) {
    dim3 grid(c->N / 256, nq), block(256);
    account(c, TR_TENSOR, (size_t)(4 * G + (accumulate ? 6 : 3)) * nq * c->N * 8);
    hipLaunchKernelGGL(tensor_batch_kernel, grid, block, 0, s, t1, t2, G, acc3, acc_stride, accumulate ? 1 : 0, c->d_modq,
                       nq, c->logN);
}

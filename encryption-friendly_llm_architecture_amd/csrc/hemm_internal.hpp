// Internal host-side declarations shared by the C-ABI translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <stdexcept>
#include <string>
#include <vector>

#include "modarith.h"

#define HEMM_MAX_PRIMES 64

// Which prime each limb of an operand uses.  Limb j of an operand whose chain part has `nq`
// active limbs uses prime j when j < nq, and special prime nQ + (j - nq) otherwise; explicit
// lists cover everything else (digit subsets, benchmark batches).
struct LimbList {
    uint8_t idx[HEMM_MAX_PRIMES];
};

struct hemm_context {
    int device;
    int logN, N, nQ, nP, dnum, alpha;
    std::vector<u64> primes;        // nQ chain primes, then nP special primes
    std::vector<u64> psi;           // primitive 2N-th roots
    std::vector<ModQ> modq;         // host copy
    // device tables, all [prime][N] unless noted
    u64 *d_w, *d_iw;                // (psi^bitrev(i), Shoup quotient), forward and inverse transform
    u64 *d_rw, *d_irw;              // N = 2^16: the twiddles of the row passes' inner radix-16 blocks in the order their
                                    // threads read them, entry (r * 15 + 2^l - 1 + g) * 16 + c = entry
                                    // ((16 (256 + r) + c) << l) + g of d_w / d_iw (nullptr for other ring sizes)
    u64 *d_ninv, *d_ninv_s;         // [prime]
    ModQ *d_modq;                   // [prime]
    double *d_fp;                   // [prime][4]: q, 1/q, 1/N mod q, that / q as doubles; q = 0 marks a prime of
                                    // 44 bits or more, which only the integer code paths handle
    u64 *d_imag, *d_imag_s;         // [prime] psi^(N/2) and Shoup quotient
    // scratch owned by the context (single stream use)
    u64 *d_scratch;
    size_t scratch_bytes;
    // staging for the term lists of batched calls: one region per stream that has staged a list (a region has one
    // user at a time: the copy into it and the kernel that reads it are ordered on that stream)
    std::vector<std::pair<hipStream_t, void *>> d_desc;
    hipStream_t stream = nullptr;   // what a null stream argument of an entry point means for this context
    // a second stream (non-blocking, default priority) for the runs of a large transform batch: the odd runs go there,
    // forked from and joined back into the caller's stream with the two events inside the same call.  Made on first
    // use: a process has few hardware queues, and a stream that is never used would still share one with a busy stream
    hipStream_t aux = nullptr;
    hipEvent_t aux_fork = nullptr, aux_join = nullptr;
    // compact evaluation keys: offset of every prime's limb inside a (digit, polynomial) slice and, last entry, the
    // slice size, in units of 2N bytes (a prime below 2^44 takes 6 bytes per residue = 3 units, any other 4)
    std::vector<u32> key_off;
    u32 *d_key_off;
    // Algorithmic bytes of everything launched on this context since the last reset, by kind of work: for each
    // launch the operands it has to read once plus the results it has to write once (what a launch of that kind
    // cannot avoid moving), counted on the host when the launch is queued.  A 2^16-point transform counts one
    // read and one write of every limb although it runs as two launches.
    unsigned long long traffic[8], launches[8];
};
enum { TR_NTT = 0, TR_KEYPROD, TR_BCONV, TR_TENSOR, TR_MASKED, TR_POINTWISE, TR_KINDS };
inline void account(const hemm_context *c, int kind, size_t bytes, int n_launches = 1) {
    hemm_context *m = const_cast<hemm_context *>(c);
    m->traffic[kind] += bytes;
    m->launches[kind] += (unsigned long long)n_launches;
}

// a constant and its Shoup quotient floor(w * 2^64 / q)
struct __align__(16) Cst {
    u64 w, ws;
};

// NTT-domain index of the automorphism X -> X^g: out[k] = in[galois_index(k)]
__device__ __forceinline__ u32 galois_index(u32 k, u32 g, int logN) {
    const u32 br = __brev(k) >> (32 - logN);
    const u32 e = ((2 * br + 1) * g) & ((2u << logN) - 1);
    return __brev(e >> 1) >> (32 - logN);
}

void hemm_set_error(const std::string &msg);

#define HEMM_HIP(call)                                                                       \
    do {                                                                                     \
        hipError_t e_ = (call);                                                              \
        if (e_ != hipSuccess)                                                                \
            throw std::runtime_error(std::string(#call) + ": " + hipGetErrorString(e_));     \
    } while (0)

// host modular helpers (context set-up only)
u64 h_mulmod(u64 a, u64 b, u64 q);
u64 h_powmod(u64 a, u64 e, u64 q);
u64 h_invmod(u64 a, u64 q);

LimbList limbs_default(const hemm_context *c, int nq, int with_p);

// kernel launchers (defined in the .hip files)
// final_scale (device, one (constant, Shoup quotient) pair per limb of the launch, or nullptr): an inverse transform
// of N = 2^16 ends with that constant in place of 1/N
void launch_ntt_slots(const hemm_context *c, u64 *data, const LimbList &ll, const LimbList &sl, int n_limbs,
                      int n_polys, size_t poly_stride, bool inverse, hipStream_t s, const void *final_scale = nullptr);
bool launch_ntt_sub_scale(const hemm_context *c, u64 *data, int n_limbs, int n_polys, const u64 *minuend,
                          size_t minuend_stride, u64 *out, size_t out_stride, const void *cst_dev, hipStream_t s);
// A forward transform of N = 2^16 whose input is a fast basis conversion: limb l of the launch is the conversion of
// the coefficient-form sources of digit digit_of[l] (already carrying their (S/q_i)^-1 factors) to prime ll[l],
// computed while the first pass loads its slab instead of being written by a conversion launch and read back.
#define CONV_MAX_DIGITS 4
#define CONV_MAX_SOURCES 8
struct ConvSources {
    struct Digit {
        const u64 *src;             // coefficient form, [n_polys][.][N]
        const Cst *hat;             // [n_src][hat_ld]  (S/q_i) mod prime, indexed by prime
        size_t src_poly_stride;
        int n_src;
        uint8_t src_slot[CONV_MAX_SOURCES];
    } d[CONV_MAX_DIGITS];
    int hat_ld;
    uint8_t digit_of[HEMM_MAX_PRIMES];
    // n_copy further limbs of the launch are plain copies (first pass only, no transform): slot copy_src_slot[i] of
    // copy_src (NTT form, polynomial stride copy_src_stride) to slot copy_dst_slot[i] of data
    const u64 *copy_src;
    size_t copy_src_stride;
    int n_copy;
    u32 copy_galois;            // != 0: the copies read their source through this automorphism (N = 2^16)
    uint8_t copy_src_slot[HEMM_MAX_PRIMES], copy_dst_slot[HEMM_MAX_PRIMES];
};
// data: [n_polys][.][N] (polynomial stride poly_stride), limb l written to slot sl[l].  With ep_* set the second pass
// ends with out = (minuend - transform) * cst[l] (slots of minuend / out = l) and data is only a workspace.
// false when the ring size or the source counts have no such form (nothing was launched).
bool launch_ntt_converted(const hemm_context *c, const ConvSources &cs, u64 *data, const LimbList &ll, const LimbList &sl,
                          int n_limbs, int n_polys, size_t poly_stride, hipStream_t s, const u64 *ep_minuend = nullptr,
                          size_t ep_minuend_stride = 0, u64 *ep_out = nullptr, size_t ep_out_stride = 0,
                          const void *ep_cst_dev = nullptr);
// out[p][j] = (y[p][j] - conversion of the n_src listed limbs of y[p] to prime j) * cst[j], j < nq_out, as inverse row
// pass (in place on the listed limbs), one column-slab kernel (second inverse pass, conversion as lazy dot products, first
// forward pass into conv[n_polys][nq_out][N]) and forward row pass with the fused tail.  final_scale / hat / cst: device
// tables in source order, [n_src][hat_ld] by prime, by target limb.  false when the shape has no such form.
bool launch_moddown_slab(const hemm_context *c, u64 *y, size_t y_stride, const uint8_t *src_slot, const uint8_t *src_prime,
                         int n_src, const void *final_scale_dev, const void *hat_dev, int hat_ld, u64 *conv, int nq_out,
                         int n_polys, u64 *out, size_t out_stride, const void *cst_dev, hipStream_t s);
// inverse transform reading src (same slot numbering as data, polynomial stride src_poly_stride) and leaving the
// coefficients in data; false when this ring size has no out-of-place form (the caller copies, then transforms)
// galois != 0: src is read through that automorphism (the transform of the rotated polynomial, without a launch
// that rotates it first)
bool launch_intt_from(const hemm_context *c, const u64 *src, size_t src_poly_stride, u64 *data, const LimbList &ll,
                      const LimbList &sl, int n_limbs, int n_polys, size_t poly_stride, hipStream_t s,
                      const void *final_scale = nullptr, u32 galois = 0);
void launch_ntt(const hemm_context *c, u64 *data, const LimbList &ll, int n_limbs, int n_polys,
                size_t poly_stride, bool inverse, hipStream_t s);
void launch_binary(const hemm_context *c, int op, const u64 *a, size_t a_stride, const u64 *b, size_t b_stride,
                   u64 *out, size_t out_stride, const LimbList &ll, int n_limbs, int n_polys, hipStream_t s);
void launch_mul_scalar(const hemm_context *c, const u64 *a, size_t a_stride, const u64 *scalars, u64 *out,
                       size_t out_stride, const LimbList &ll, int n_limbs, int n_polys, hipStream_t s);
void launch_add_scalar(const hemm_context *c, const u64 *a, const u64 *re, const u64 *im, u64 *out, const LimbList &ll,
                       int n_limbs, hipStream_t s);
void launch_encode(const hemm_context *c, double *slots, double scale, const LimbList &ll, int n_limbs, int n_msgs, u64 *out,
                   hipStream_t s);
void launch_decode(const hemm_context *c, const u64 *pt, int n_limbs, double scale, u64 *work, double *slots, hipStream_t s);
void hemm_embedding_tables_free(const hemm_context *c);
void launch_zero(const hemm_context *c, u64 *out, size_t words, hipStream_t s);
void launch_mul_imag(const hemm_context *c, const u64 *a, size_t a_stride, u64 *out, size_t out_stride,
                     const LimbList &ll, int n_limbs, int n_polys, hipStream_t s);
void launch_tensor(const hemm_context *c, const u64 *c1, size_t s1, const u64 *c2, size_t s2, u64 *out,
                   size_t out_stride, int nq, bool accumulate, hipStream_t s);
void launch_galois(const hemm_context *c, const u64 *a, size_t a_stride, u64 *out, size_t out_stride, u64 g,
                   int n_limbs, int n_polys, hipStream_t s);
void launch_sample_uniform(const hemm_context *c, const u64 *stream_keys, const LimbList &ll, int n_limbs, u64 *out,
                           hipStream_t s);
void launch_sample_error(const hemm_context *c, u64 stream_key, const LimbList &ll, int n_limbs, u64 *out, hipStream_t s);
size_t hemm_scratch_words(const hemm_context *c);
u64 *hemm_scratch(hemm_context *c);
void launch_modup(hemm_context *c, const u64 *in, int nq, u64 *ext, u64 *coef, bool fill_own, hipStream_t s);
void launch_inner_product(hemm_context *c, const u64 *in, const u64 *ext, const u64 *evk, int nq, u64 *acc,
                          hipStream_t s);
void launch_moddown(hemm_context *c, u64 *acc, int nq, int n_polys, u64 *out, size_t out_stride, const u64 *add,
                    size_t add_stride, int add_polys, u64 *conv, hipStream_t s);
// galois != 0 (N = 2^16): the key switch of the automorphism of `in`, which is read through it where the ModUp reads
// it; b_rotates: add_b is read through the same automorphism where the key product adds it; add_a (N >= 512, with
// add_b): out[1] = ks_a + add_a as well, both addends entering the sum in the extended basis
void launch_keyswitch(hemm_context *c, const u64 *in, const u64 *evk, int nq, u64 *out, size_t out_stride,
                      const u64 *add_b, hipStream_t s, u32 galois = 0, bool b_rotates = false,
                      const u64 *add_a = nullptr);
void launch_rescale(hemm_context *c, const u64 *in, size_t in_stride, u64 *out, size_t out_stride, int nq,
                    int n_polys, hipStream_t s);
void launch_modup_batch(hemm_context *c, const u64 *in, size_t in_stride, int nq, int n_in, u64 *ext, u64 *coef,
                        hipStream_t s, u32 galois = 0);
// whether launch_modup_batch at this level takes a non-zero `galois` (its input read through that automorphism)
bool modup_through_automorphism_ok(const hemm_context *c, int nq);
// terms_host / n_terms: the host copy of the list (only read for the byte accounting; may be nullptr)
// compact: every term's key is in the compact layout (all terms of a launch use the same layout)
void launch_hoisted_terms(hemm_context *c, const void *terms_dev, const u32 *group_off_dev, int n_out, int nq, u64 *y,
                          bool b_premultiplied, hipStream_t s, const void *terms_host = nullptr, int n_terms = 0,
                          bool compact = false);
int hoisted_arg_capacity();
void launch_hoisted_terms_args(hemm_context *c, const void *terms_host, int n_terms, const u32 *group_off_host, int n_out,
                               int nq, u64 *y, bool b_premultiplied, hipStream_t s);
void launch_moddown_batch(hemm_context *c, u64 *y, int nq, int n_polys, int drop_last, u64 *out, size_t out_stride,
                          u64 *conv, hipStream_t s, bool slab = false);
void launch_masked_sum(hemm_context *c, const void *terms_dev, const u32 *group_off_dev, int n_out, int nq, int n_polys,
                       u64 *out, hipStream_t s, const void *terms_host = nullptr, int n_terms = 0);
// y[o][p][j] = sum_{q < parts} part[o * parts + q][p][j] over the extended basis, y / part: [.][2][nq+K][N]
void launch_sum_parts(hemm_context *c, const u64 *part, int parts, int n_out, int nq, u64 *y, hipStream_t s);
size_t key_compact_words(const hemm_context *c);
void launch_key_compact(const hemm_context *c, const u64 *evk, u64 *out, hipStream_t s);
void launch_key_expand(const hemm_context *c, const u64 *compact, u64 *evk, hipStream_t s);
int masked_arg_capacity();
// table[j][r] = mask[j][r << shift]; true when every aligned run of 2^shift residues of the mask is constant
bool launch_compact_mask(hemm_context *c, const u64 *mask, int n_limbs, int shift, u64 *table, hipStream_t s);
void launch_masked_sum_args(hemm_context *c, const void *terms_host, int n_terms, const u32 *group_off_host, int n_out,
                            int nq, int n_polys, u64 *out, hipStream_t s);
// several tensor sums in one launch: acc[i] (+)= sum over n_pairs[i] pairs of t1[i], t2[i] (distinct accumulators)
#define TENSOR_MAX_GROUPS 8
struct TensorGroupHost {
    const u64 *t1, *t2;
    u64 *acc;
    int n_pairs;
    bool accumulate;
};
int tensor_max_groups();
void launch_tensor_groups(hemm_context *c, const TensorGroupHost *g, int n_groups, int nq, size_t acc_stride,
                          hipStream_t s);
void launch_tensor_batch(hemm_context *c, const u64 *t1, const u64 *t2, int G, int nq, u64 *acc3, size_t acc_stride,
                         bool accumulate, hipStream_t s);

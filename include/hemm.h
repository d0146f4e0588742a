/* C ABI of the MI355X RNS-CKKS kernels under HEMMer's homomorphic matrix multiplication.
 *
 * The reference reaches its ring arithmetic through the C++ classes of the closed HEaaN
 * library (ciphertext/external/include/HEaaN/HomEvaluator.hpp:30-616, Context.hpp:39-206);
 * there is no FFI layer.  Each entry point below names the HEaaN call whose device work it
 * replaces.  All data pointers are DEVICE pointers to uint64 residues laid out
 * [poly][limb][N] (the layout the reference's own NCCL calls rely on,
 * ciphertext/src/HEMMer.cpp:2625-2635); limb j of an operand with `nq` active chain limbs
 * uses chain prime j for j < nq and special prime (j - nq) after that.  `stream` is a
 * hipStream_t (NULL = default stream); calls are asynchronous on it.
 *
 * A context owns one device scratch region.  hemm_modup, hemm_moddown, hemm_keyswitch,
 * hemm_rotate, hemm_relinearize and hemm_rescale work in it, so two such calls queued on
 * DIFFERENT streams of one context race unless the caller orders them with events.  Calls that
 * take a `workspace` argument use only that memory; the batched calls (hemm_hoisted_*,
 * hemm_masked_sum_batch) copy term lists longer than 32 through a staging region of their own
 * per stream (up to 8 streams per context), so they may run side by side on two streams.
 *
 * Return value: 0 = ok, 1 = invalid argument, 2 = HIP/runtime failure; the text is in
 * hemm_last_error().
 */
#ifndef HEMM_H
#define HEMM_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct hemm_context hemm_context;

const char *hemm_last_error(void);

/* HEaaN::makeContext (Context.hpp:39,88): ring degree 2^log_n, n_q chain primes followed by
 * n_p special (key-switching) primes, all in [2^31, 2^61) and = 1 mod 2^(log_n+1); dnum = number of
 * key-switching digits.  Twiddle tables are built on the current device. */
int hemm_context_create(uint32_t log_n, uint32_t n_q, uint32_t n_p, const uint64_t *primes,
                        uint32_t dnum, hemm_context **out);
void hemm_context_destroy(hemm_context *ctx);
/* The stream that a null `stream` argument of the entry points below stands for on this context: the legacy default
 * stream until another one is named here.  For callers that record the library's launches into a HIP graph (stream
 * capture cannot use the legacy default stream) or keep the library off the default stream altogether.  The context's
 * scratch and staging regions have one user at a time: calls on different streams of one context must not overlap. */
int hemm_context_set_stream(hemm_context *ctx, void *stream);
void *hemm_context_stream(const hemm_context *ctx);
/* primitive 2N-th root of unity used for prime `idx` (smallest g^((q-1)/2N) of order 2N) */
uint64_t hemm_context_psi(const hemm_context *ctx, uint32_t idx);

/* Largest `count` primes below 2^bits congruent to 1 mod 2^(log_n+1), descending
 * (HEaaN::getPrimeList, Context.hpp:201, is a fixed preset; this build takes explicit lists). */
int hemm_primes_below(uint32_t bits, uint32_t log_n, uint32_t count, uint64_t *out);

/* HIP-event stopwatch on `stream` (the reference times with cudaDeviceSynchronize + std::chrono,
 * ciphertext/src/TransformerBlock.cpp:101-112).  stop() waits for the stream and returns ms. */
int hemm_timer_create(void **timer);
int hemm_timer_start(void *timer, void *stream);
int hemm_timer_stop(void *timer, void *stream, float *ms);
void hemm_timer_destroy(void *timer);

/* Samplers behind KeyGenerator / Encryptor (HEaaN keeps them internal: KeyGenerator.hpp:31-95, Encryptor.hpp:32-49).
 * Counter-based: value i of a stream is a function of (stream key, i) only.
 *   hemm_sample_uniform: out[j][i] uniform in [0, q_{prime_idx[j]}) from stream_keys[j] (masked rejection);
 *   hemm_sample_error:   out[j][i] = e_i mod q_{prime_idx[j]}, e centred binomial (21 bit pairs) from stream_key.
 * Both write coefficient-order values [n_limbs][N]; the error is a coefficient vector (transform it with hemm_ntt),
 * the uniform values are used directly as NTT-form residues. */
int hemm_sample_uniform(hemm_context *ctx, const uint64_t *stream_keys, const uint32_t *prime_idx, uint32_t n_limbs,
                        uint64_t *out, void *stream);
int hemm_sample_error(hemm_context *ctx, uint64_t stream_key, const uint32_t *prime_idx, uint32_t n_limbs, uint64_t *out,
                      void *stream);

/* Batched negacyclic NTT (inverse = 0: natural -> bit-reversed order) or INTT (inverse = 1,
 * including 1/N) in place over data[n_polys][n_limbs][N]; limb j uses prime prime_idx[j]
 * (host array).  Every NTT-form operand of HomEvaluator goes through this.  At N = 2^16 a batch of more than 448
 * limbs is cut into runs of 192 limbs that alternate between `stream` and a second stream of the context; the second
 * stream starts after what `stream` holds so far and `stream` waits for it before the call's work counts as done, so
 * the call stays ordered on `stream` like any other. */
int hemm_ntt(hemm_context *ctx, uint64_t *data, const uint32_t *prime_idx, uint32_t n_limbs,
             uint32_t n_polys, int inverse, void *stream);

/* ---- streaming residue kernels -------------------------------------------------------------
 * Operands are [n_polys][n_limbs][N] with their own polynomial stride (in uint64 words), so a
 * higher-level operand can be read at a lower level ("levels auto-adjust to the lower operand",
 * HomEvaluator.hpp:128-129); stride 0 broadcasts one polynomial (a plaintext).  n_limbs =
 * nq + (with_p ? n_p : 0).  `out` may alias an input element-for-element. */
enum { HEMM_ADD = 0, HEMM_SUB = 1, HEMM_MUL = 2, HEMM_NEG = 3, HEMM_MAC = 4 };
/* HomEvaluator::add :144 / sub :223 / negate :67 / multWithoutRescale(ct, pt) :491 (HEMM_MUL with
 * b_stride = 0) / multiply-accumulate for the diagonal accumulation of matmul :600 */
int hemm_pointwise(hemm_context *ctx, int op, const uint64_t *a, size_t a_stride, const uint64_t *b,
                   size_t b_stride, uint64_t *out, size_t out_stride, uint32_t nq, int with_p,
                   uint32_t n_polys, void *stream);
/* HomEvaluator::multInteger :347 / constant multiply :276,:478: residue-wise product with one
 * host-side scalar per limb (scalars[j] is reduced modulo limb j's prime). */
int hemm_mul_scalar(hemm_context *ctx, const uint64_t *a, size_t a_stride, const uint64_t *scalars,
                    uint64_t *out, size_t out_stride, uint32_t nq, int with_p, uint32_t n_polys,
                    void *stream);
/* EnDecoder::encode (EnDecoder.hpp:51): n_msgs messages of N/2 complex slots each (device memory, interleaved
 * re, im doubles, [n_msgs][N/2][2]; CLOBBERED) -> plaintexts out [n_msgs][nq (+ n_p)][N] in NTT form, coefficient
 * i = round(scale * c_i) for the inverse canonical embedding c of the slots on the orbit zeta^(5^j).  Double precision
 * with one IEEE operation per step in a fixed order: the same bits as a host loop over the same butterflies. */
int hemm_encode(hemm_context *ctx, double *slots, double scale, uint32_t nq, int with_p, uint32_t n_msgs, uint64_t *out,
                void *stream);
/* EnDecoder::decode (EnDecoder.hpp:66): plaintext pt [>= n_limbs][N] (NTT form, limbs of chain primes 0 .. n_limbs-1,
 * n_limbs = 1 or 2: the centred value is recovered from that many limbs) -> slots [N/2][2] doubles on the device;
 * workspace: n_limbs * N words. */
int hemm_decode(hemm_context *ctx, const uint64_t *pt, uint32_t n_limbs, double scale, uint64_t *workspace, double *slots,
                void *stream);
/* HomEvaluator::add(Ciphertext, Complex) :159 / sub :207 without a plaintext: out[j][k] = a[j][k] + re[j] +- im[j] I_j,
 * the NTT form of the constant polynomial re + im X^(N/2) (a complex constant in every slot; I_j = psi_j^(N/2), the
 * sign flips on the upper half of the bit-reversed index range).  One polynomial [nq (+ n_p)][N]; re / im hold one
 * residue per limb on the host, im may be NULL.  N >= 512. */
int hemm_add_scalar(hemm_context *ctx, const uint64_t *a, const uint64_t *re, const uint64_t *im, uint64_t *out,
                    uint32_t nq, int with_p, void *stream);
/* HomEvaluator::multImagUnit :330: multiply by the monomial X^(N/2) in NTT form. */
/* out[0 .. words) = 0 by a kernel (an even number of words, 16-byte aligned): the clearing step of an accumulation,
 * safe to record into a HIP graph where a memset node is not.  No counterpart in HEaaN. */
int hemm_zero(hemm_context *ctx, uint64_t *out, size_t words, void *stream);
int hemm_mul_imag_unit(hemm_context *ctx, const uint64_t *a, size_t a_stride, uint64_t *out,
                       size_t out_stride, uint32_t nq, uint32_t n_polys, void *stream);
/* HomEvaluator::tensor :518: (b1,a1) x (b2,a2) -> (b1 b2, a1 b2 + a2 b1, a1 a2); accumulate != 0
 * adds into `out` (the running 3-polynomial sum of the CCMM loop, MatrixUtils.cpp:1434-1439). */
int hemm_tensor(hemm_context *ctx, const uint64_t *ct1, size_t stride1, const uint64_t *ct2,
                size_t stride2, uint64_t *out, size_t out_stride, uint32_t nq, int accumulate,
                void *stream);
/* Galois automorphism X -> X^galois on NTT-form limbs (the keyless half of leftRotate :370-403 and
 * conjugate :465; all of leftRotate(Plaintext) :376).  `out` must not alias `a`. */
int hemm_automorphism(hemm_context *ctx, const uint64_t *a, size_t a_stride, uint64_t *out,
                      size_t out_stride, uint64_t galois, uint32_t n_limbs, uint32_t n_polys,
                      void *stream);

/* ---- hybrid key switching (inside leftRotate/rightRotate :383-403, conjugate :465, relinearize
 * :524).  Evaluation key layout: [dnum][2 (b, a)][n_q + n_p][N], NTT form.  The stages are exposed
 * one by one so each can be checked against the CPU oracle; hemm_keyswitch chains them. ---- */
/* in [nq][N] -> ext [beta][nq + n_p][N], beta = ceil(nq / alpha), alpha = ceil(n_q / dnum) */
int hemm_modup(hemm_context *ctx, const uint64_t *in, uint32_t nq, uint64_t *ext, void *stream);
/* ext [beta][nq + n_p][N], evk -> acc [2][nq + n_p][N] */
int hemm_inner_product(hemm_context *ctx, const uint64_t *ext, const uint64_t *evk, uint32_t nq,
                       uint64_t *acc, void *stream);
/* acc [n_polys][nq + n_p][N] (clobbered) -> out [n_polys][nq][N] = acc / P */
int hemm_moddown(hemm_context *ctx, uint64_t *acc, uint32_t nq, uint32_t n_polys, uint64_t *out,
                 size_t out_stride, void *stream);
/* in [nq][N], evk -> out[0] = ks_b (+ add_b[nq][N] when not NULL), out[1] = ks_a */
int hemm_keyswitch(hemm_context *ctx, const uint64_t *in, const uint64_t *evk, uint32_t nq,
                   uint64_t *out, size_t out_stride, const uint64_t *add_b, void *stream);
/* HomEvaluator::leftRotate(ct) :383 / conjugate :465: automorphism of (b, a) + key switch of a. */
int hemm_rotate(hemm_context *ctx, const uint64_t *ct, size_t ct_stride, const uint64_t *evk,
                uint64_t galois, uint32_t nq, uint64_t *out, size_t out_stride, void *stream);
/* HomEvaluator::relinearize :524: (d0, d1, d2) -> (d0 + ks_b(d2), d1 + ks_a(d2)) */
int hemm_relinearize(hemm_context *ctx, const uint64_t *ct3, size_t ct_stride, const uint64_t *evk,
                     uint32_t nq, uint64_t *out, size_t out_stride, void *stream);
/* ---- batched / hoisted forms: what one GPU-sized launch does where the reference issues one
 * evaluator call per rotation.  They have no single counterpart in HomEvaluator; each replaces a
 * run of leftRotate / multWithoutRescale / add / rescale calls of the matmul loops
 * (MatrixUtils.cpp:800-845, 1413-1433). ---- */
/* ModUp of n_in polynomials at once: in [n_in][.][N] (stride in_stride, nq limbs used) ->
 * ext [n_in][beta][nq+n_p][N]; workspace >= n_in*nq*N words. */
int hemm_modup_batch(hemm_context *ctx, const uint64_t *in, size_t in_stride, uint32_t nq, uint32_t n_in,
                     uint64_t *ext, uint64_t *workspace, void *stream);
/* One hoisted rotation term: automorphism `galois` applied to an already extended source (ext, b),
 * inner product with evk, optional plaintext mask over the extended basis (NULL = 1). */
typedef struct {
    const uint64_t *ext;  /* [beta][nq+n_p][N] */
    const uint64_t *b;    /* [nq][N], or NULL: the term contributes only the key product (used for the
                           * degree-2 component of a tensor product, with a key for the rotated s^2) */
    const uint64_t *evk;  /* [dnum][2][n_q+n_p][N], or NULL: a term that needs no key switch, mask * pt * P * (b, a) on the
                           * chain limbs with the a-polynomial [nq][N] in `ext` (always as it is, also where b is
                           * premultiplied; b may be NULL; galois = 1; of its mask only the nq chain limbs are read): the
                           * unrotated part of a masked sum joins its rotated parts before their common ModDown */
    const uint64_t *mask; /* [nq+n_p][N] or NULL; with mask_shift = s > 0 a run table [nq+n_p][N >> s][2] */
    uint32_t galois;
    uint32_t mask_shift;  /* 0: full mask.  s >= 1: the mask is constant over aligned runs of 2^s coefficients
                           * (the NTT form of a slot pattern with period 2^(logN-1-s)) and `mask` holds one value
                           * per run, as written by hemm_compact_mask */
    const uint64_t *pt;   /* [nq+n_p][N] or NULL: a second plaintext factor over the extended basis, read through
                           * the automorphism pt_galois (the rotated weight of a plaintext-ciphertext product) */
    uint32_t pt_galois;   /* odd, < 2N; 1 = as stored */
    uint32_t flags;       /* 0, or HEMM_ROT_COMPACT_KEY: evk is the compact form written by hemm_key_compact */
} hemm_rot_term;
#define HEMM_ROT_COMPACT_KEY 1u
/* Compact form of an evaluation key for the hoisted sums (hemm_hoisted_terms / hemm_hoisted_moddown), which read a key
 * once per launch and move little else: residues of primes below 2^44 take 6 bytes instead of 8 (per digit and
 * polynomial the limbs back to back; such a limb as N/2 records of 12 bytes, one per residue pair: two 32-bit low
 * words, then the two 16-bit high halves in one word; any other limb as N words).  Needs N >= 512 and at most 6
 * digits per key switch.  All terms of one call use the same layout.  out: hemm_key_compact_words(ctx) words.  The
 * plain key is what every other call takes.
 * No counterpart in HEaaN's interface (its key storage is not exposed). */
size_t hemm_key_compact_words(const hemm_context *ctx);
int hemm_key_compact(hemm_context *ctx, const uint64_t *evk, uint64_t *out, void *stream);
/* the plain key [dnum][2][n_q+n_p][N] back from its compact form (lossless), for holders that keep only the latter */
int hemm_key_expand(hemm_context *ctx, const uint64_t *compact, uint64_t *evk, void *stream);
/* Algorithmic bytes of everything queued on this context since the last reset, by kind of work (for each launch: the
 * operands it must read once plus the results it must write once; a two-launch 2^16-point transform counts one read
 * and one write per limb), and the number of launches; counted on the host, costs nothing on the device.  Kinds:
 * 0 transforms, 1 key products (inner products, hoisted sums), 2 basis conversions, 3 tensor products and their
 * accumulation, 4 masked sums, 5 other pointwise work and copies; entries 6, 7 are 0.  Either array may be NULL.
 * No counterpart in HEaaN's interface: it is the per-kernel byte breakdown a roofline report needs. */
#define HEMM_TRAFFIC_KINDS 8
int hemm_traffic(hemm_context *ctx, uint64_t *bytes, uint64_t *launches, int reset);
/* sizeof(hemm_rot_term) and sizeof(hemm_lin_term) as this library was built: a binding checks its own record layouts
 * against them before it passes term lists. */
void hemm_abi_sizes(uint32_t *rot_term_bytes, uint32_t *lin_term_bytes);
/* y[o] = sum of the n_parts consecutive partial sums parts[o * n_parts .. ) of hemm_hoisted_terms, limb-wise over the
 * extended basis; y: [n_out][2][nq+n_p][N], parts: [n_out * n_parts][2][nq+n_p][N].  A sum with one output and many
 * terms is split over several partial outputs (more workgroups, more keys in flight) and added up here before its
 * single ModDown.  No counterpart in HEaaN's interface. */
int hemm_sum_parts(hemm_context *ctx, const uint64_t *parts, uint32_t n_parts, uint32_t n_out, uint32_t nq, uint64_t *y,
                   void *stream);
/* Run table of a mask over the extended basis (n_limbs = nq + n_p) that is constant over aligned runs of 2^shift
 * coefficients: table[j][r] = { v = mask[j][r << shift], floor(v * 2^64 / prime_j) } (2 * n_limbs * (N >> shift)
 * words; the second word lets the 60-bit limbs multiply by v as by a constant); *is_constant = 0 (and the table is
 * not to be used) when some run of the mask is not constant.  Synchronises the stream.  No counterpart in HEaaN's interface: it removes the mask traffic of hoisted sums whose
 * masks select columns of a power-of-two period. */
int hemm_compact_mask(hemm_context *ctx, const uint64_t *mask, uint32_t n_limbs, uint32_t shift, uint64_t *table,
                      int *is_constant, void *stream);
/* y[o] = sum over terms[group_offsets[o] .. group_offsets[o+1]) of
 *        mask * pt_galois(pt) * ( <galois(ext), evk> + P * galois(b) )   in the extended basis (absent factors
 *        are 1), y: [n_out][2][nq+n_p][N].
 * terms / group_offsets are host arrays.  b_premultiplied != 0: every term's b already holds P*b
 * (hemm_mul_scalar with P mod q_j once per source instead of once per term). */
int hemm_hoisted_terms(hemm_context *ctx, const hemm_rot_term *terms, const uint32_t *group_offsets,
                       uint32_t n_out, uint32_t nq, uint64_t *y, int b_premultiplied, void *stream);
/* hemm_hoisted_terms followed by hemm_moddown_batch on all n_out outputs (one term upload, one call).
 * y_workspace: [n_out][2][nq+K][N] receives the sums and is clobbered; out: [n_out][2][nq_out][N] with
 * polynomial stride out_stride; workspace: [n_out][2][nq_out][N].  No counterpart in HEaaN's interface: it is
 * the key-switch tail of HomEvaluator::leftRotate / multWithoutRescale + rescale for a batch of outputs. */
int hemm_hoisted_moddown(hemm_context *ctx, const hemm_rot_term *terms, const uint32_t *group_offsets,
                         uint32_t n_out, uint32_t nq, int b_premultiplied, int drop_last, uint64_t *y_workspace,
                         uint64_t *out, size_t out_stride, uint64_t *workspace, void *stream);

/* y [n_polys][nq+n_p][N] (clobbered) -> out [n_polys][nq - drop_last][N]: division by P (drop_last = 0)
 * or by P*q_{nq-1} (drop_last = 1, ModDown and rescale in one basis conversion);
 * workspace >= n_polys*(nq-drop_last)*N words.
 * drop_last | HEMM_MODDOWN_COLUMN_SLAB (N = 2^16, 4 or 5 dropped limbs, primes below 2^60) runs the same arithmetic
 * in three launches instead of four: the second pass of the inverse transform, the basis conversion and the first
 * pass of the forward transform in one kernel per 16-column slab, so the dropped limbs are not written in
 * coefficient form and read back (identical residues; a fifth less memory traffic, but slower where measured, so
 * nothing in the library selects it by itself). */
#define HEMM_MODDOWN_COLUMN_SLAB 2
int hemm_moddown_batch(hemm_context *ctx, uint64_t *y, uint32_t nq, uint32_t n_polys, int drop_last,
                       uint64_t *out, size_t out_stride, uint64_t *workspace, void *stream);
typedef struct {
    const uint64_t *ct;   /* [n_polys][.][N] */
    const uint64_t *mask; /* [nq][N] or NULL */
    uint64_t stride;      /* polynomial stride of ct in words */
    uint64_t galois;      /* 0, or the mask is read through X -> X^galois (a rotated plaintext:
                             leftRotate(Plaintext), HomEvaluator.hpp:376, without materialising it) */
} hemm_lin_term;
/* out[o][p] = sum over the terms of group o of mask * ct[p]; out: [n_out][n_polys][nq][N] */
int hemm_masked_sum_batch(hemm_context *ctx, const hemm_lin_term *terms, const uint32_t *group_offsets,
                          uint32_t n_out, uint32_t nq, uint32_t n_polys, uint64_t *out, void *stream);
/* acc3 [3][nq][N] (+)= sum_g tensor(t1[g], t2[g]); t1, t2: [n_pairs][2][nq][N] */
int hemm_tensor_batch(hemm_context *ctx, const uint64_t *t1, const uint64_t *t2, uint32_t n_pairs, uint32_t nq,
                      uint64_t *acc3, int accumulate, void *stream);
/* the same with the three polynomials of the accumulator acc_stride words apart (several accumulators can then be
 * kept polynomial-major, [3][count][nq][N], so that one hemm_modup_batch covers a polynomial of all of them) */
int hemm_tensor_batch_strided(hemm_context *ctx, const uint64_t *t1, const uint64_t *t2, uint32_t n_pairs, uint32_t nq,
                              uint64_t *acc3, size_t acc_stride, int accumulate, void *stream);
/* several such sums in one launch (at most 8; N >= 512): group i adds the n_pairs tensor products of t1[k], t2[k],
 * k < n_pairs, to its own accumulator acc3 (or stores them when accumulate is 0).  The accumulators of one call must
 * not overlap.  One launch over the giant-step groups of a chain of shifts fills the GPU where a launch per group
 * does not.  No counterpart in HEaaN's interface (HomEvaluator::tensor :518 takes one pair). */
typedef struct {
    const uint64_t *t1, *t2; /* [n_pairs][2][nq][N] each */
    uint64_t *acc3;          /* three polynomials acc_stride words apart */
    uint32_t n_pairs;
    uint32_t accumulate;     /* 0 or 1 */
} hemm_tensor_group;
int hemm_tensor_batch_groups(hemm_context *ctx, const hemm_tensor_group *groups, uint32_t n_groups, uint32_t nq,
                             size_t acc_stride, void *stream);

/* HomEvaluator::rescale :540: [n_polys][nq][N] -> [n_polys][nq-1][N], (c_i - [c_last]_{q_i}) / q_last.
 * With more than one polynomial, in_stride >= nq * N and out_stride >= (nq - 1) * N; out may not overlap in, except
 * out == in with equal strides (each result then takes the place of its own input); anything else is refused. */
int hemm_rescale(hemm_context *ctx, const uint64_t *in, size_t in_stride, uint64_t *out,
                 size_t out_stride, uint32_t nq, uint32_t n_polys, void *stream);


/* hemm_rescale for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments, same kernels and same
 * result as hemm_rescale, but its scratch (n_polys * nq * N words) is a fixed array inside the library's device image
 * instead of the context's lazily allocated buffer, and the constant tables it reads were built by
 * hemm_context_create: the call itself makes no hipMalloc / hipFree.  Limit: n_polys * nq * N <=
 * HEMM_STATIC_SCRATCH_WORDS (16 MiB: a two-polynomial ciphertext of up to 16 limbs at N = 2^16), larger inputs are
 * rejected with return value 1.  The array is held once per GPU until the process ends and is shared by every call
 * on that GPU: calls that overlap on one GPU (two streams, two contexts) race.  Nothing in it has to start at zero;
 * every word a call reads was written by that call.  The context's device must be the current one. */
#define HEMM_STATIC_SCRATCH_WORDS (32u << 16)
int hemm_rescale_static(hemm_context *ctx, const uint64_t *in, size_t in_stride, uint64_t *out,
                        size_t out_stride, uint32_t nq, uint32_t n_polys, void *stream);

#ifdef __cplusplus
}
#endif
#endif

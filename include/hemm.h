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
 * n_p special (key-switching) primes, all < 2^61 and = 1 mod 2^(log_n+1); dnum = number of
 * key-switching digits.  Twiddle tables are built on the current device. */
int hemm_context_create(uint32_t log_n, uint32_t n_q, uint32_t n_p, const uint64_t *primes,
                        uint32_t dnum, hemm_context **out);
void hemm_context_destroy(hemm_context *ctx);
/* primitive 2N-th root of unity used for prime `idx` (smallest g^((q-1)/2N) of order 2N) */
uint64_t hemm_context_psi(const hemm_context *ctx, uint32_t idx);

/* Largest `count` primes below 2^bits congruent to 1 mod 2^(log_n+1), descending
 * (HEaaN::getPrimeList, Context.hpp:201, is a fixed preset; this build takes explicit lists). */
int hemm_primes_below(uint32_t bits, uint32_t log_n, uint32_t count, uint64_t *out);

/* Batched negacyclic NTT (inverse = 0: natural -> bit-reversed order) or INTT (inverse = 1,
 * including 1/N) in place over data[n_polys][n_limbs][N]; limb j uses prime prime_idx[j]
 * (host array).  Every NTT-form operand of HomEvaluator goes through this. */
int hemm_ntt(hemm_context *ctx, uint64_t *data, const uint32_t *prime_idx, uint32_t n_limbs,
             uint32_t n_polys, int inverse, void *stream);

#ifdef __cplusplus
}
#endif
#endif

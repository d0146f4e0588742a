// extern "C" boundary (declared in include/hemm.h).
#include <cstring>

#include "../../include/hemm.h"
#include "hemm_internal.hpp"

hemm_context *hemm_context_build(int logN, int nQ, int nP, const u64 *primes, int dnum);
void hemm_context_free(hemm_context *c);
void hemm_primes_below_impl(int bits, int logN, int count, u64 *out);

static thread_local std::string g_err;
void hemm_set_error(const std::string &m) { g_err = m; }

#define HEMM_TRY try {
#define HEMM_CATCH                                \
    }                                             \
    catch (const std::invalid_argument &e) {      \
        g_err = e.what();                         \
        return 1;                                 \
    }                                             \
    catch (const std::exception &e) {             \
        g_err = e.what();                         \
        return 2;                                 \
    }                                             \
    return 0;

static void need(bool ok, const char *msg) {
    if (!ok) throw std::invalid_argument(msg);
}
static void check_launch() { HEMM_HIP(hipGetLastError()); }

extern "C" {

const char *hemm_last_error(void) { return g_err.c_str(); }

int hemm_context_create(uint32_t log_n, uint32_t n_q, uint32_t n_p, const uint64_t *primes, uint32_t dnum,
                        hemm_context **out) {
    HEMM_TRY
    need(out && primes, "null argument");
    *out = hemm_context_build((int)log_n, (int)n_q, (int)n_p, (const u64 *)primes, (int)dnum);
    HEMM_CATCH
}
void hemm_context_destroy(hemm_context *ctx) { hemm_context_free(ctx); }
uint64_t hemm_context_psi(const hemm_context *ctx, uint32_t idx) { return ctx->psi.at(idx); }

int hemm_primes_below(uint32_t bits, uint32_t log_n, uint32_t count, uint64_t *out) {
    HEMM_TRY
    need(out && bits >= 21 && bits <= 61 && log_n >= 1 && log_n + 2 <= bits, "bad arguments");
    hemm_primes_below_impl((int)bits, (int)log_n, (int)count, (u64 *)out);
    HEMM_CATCH
}

int hemm_ntt(hemm_context *ctx, uint64_t *data, const uint32_t *prime_idx, uint32_t n_limbs, uint32_t n_polys,
             int inverse, void *stream) {
    HEMM_TRY
    need(ctx && data && prime_idx, "null argument");
    need(n_limbs >= 1 && n_limbs <= HEMM_MAX_PRIMES, "n_limbs out of range");
    LimbList ll;
    memset(&ll, 0, sizeof(ll));
    for (uint32_t j = 0; j < n_limbs; j++) {
        need(prime_idx[j] < (uint32_t)(ctx->nQ + ctx->nP), "prime index out of range");
        ll.idx[j] = (uint8_t)prime_idx[j];
    }
    launch_ntt(ctx, (u64 *)data, ll, (int)n_limbs, (int)n_polys, (size_t)n_limbs * ctx->N, inverse != 0,
               (hipStream_t)stream);
    check_launch();
    HEMM_CATCH
}

}  // extern "C"

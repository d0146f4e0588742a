// Internal host-side declarations shared by the C-ABI translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <stdexcept>
#include <string>
#include <vector>

#include "modarith.cuh"

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
    u64 *d_w, *d_ws;                // psi^bitrev(i) and Shoup quotients (forward)
    u64 *d_iw, *d_iws;              // inverse-transform twiddles
    u64 *d_ninv, *d_ninv_s;         // [prime]
    ModQ *d_modq;                   // [prime]
    u64 *d_imag, *d_imag_s;         // [prime] psi^(N/2) and Shoup quotient
    // scratch owned by the context (single stream use)
    u64 *d_scratch;
    size_t scratch_bytes;
};

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
void launch_ntt(const hemm_context *c, u64 *data, const LimbList &ll, int n_limbs, int n_polys,
                size_t poly_stride, bool inverse, hipStream_t s);

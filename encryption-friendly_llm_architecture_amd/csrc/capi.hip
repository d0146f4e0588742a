// extern "C" boundary (declared in include/hemm.h).
#include <cstring>
#include <vector>

#include "../../include/hemm.h"
#include "hemm_internal.hpp"

hemm_context *hemm_context_build(int logN, int nQ, int nP, const u64 *primes, int dnum);
void hemm_context_free(hemm_context *c);
void hemm_primes_below_impl(int bits, int logN, int count, u64 *out);
void hemm_keyswitch_tables_free(const hemm_context *c);
void hemm_static_setup(hemm_context *c);
size_t hemm_static_scratch_words();
void launch_rescale_static(hemm_context *c, const u64 *in, size_t in_stride, u64 *out, size_t out_stride, int nq,
                           int n_polys, hipStream_t s);

static thread_local std::string g_err;
void hemm_set_error(const std::string &m) { g_err = m; }

// A null stream argument means the context's stream (the legacy default stream unless hemm_context_set_stream named
// another one -- stream capture cannot use the legacy default stream).
static inline hipStream_t on_stream(const hemm_context *ctx, void *stream) {
    return stream != nullptr ? (hipStream_t)stream : ctx->stream;
}

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
    hemm_context *c = hemm_context_build((int)log_n, (int)n_q, (int)n_p, (const u64 *)primes, (int)dnum);
    try {
        hemm_static_setup(c);   // constant tables and the address of the static scratch: hemm_rescale_static allocates nothing
    } catch (...) {
        hemm_keyswitch_tables_free(c);
        hemm_embedding_tables_free(c);
        hemm_context_free(c);
        throw;
    }
    *out = c;
    HEMM_CATCH
}
void hemm_context_destroy(hemm_context *ctx) {
    if (ctx) {
        hemm_keyswitch_tables_free(ctx);
        hemm_embedding_tables_free(ctx);
    }
    hemm_context_free(ctx);
}
uint64_t hemm_context_psi(const hemm_context *ctx, uint32_t idx) { return ctx->psi.at(idx); }

struct hemm_timer {
    hipEvent_t a, b;
};
int hemm_timer_create(void **timer) {
    HEMM_TRY
    need(timer, "null argument");
    hemm_timer *t = new hemm_timer();
    HEMM_HIP(hipEventCreate(&t->a));
    HEMM_HIP(hipEventCreate(&t->b));
    *timer = t;
    HEMM_CATCH
}
int hemm_timer_start(void *timer, void *stream) {
    HEMM_TRY
    need(timer, "null argument");
    HEMM_HIP(hipEventRecord(((hemm_timer *)timer)->a, (hipStream_t)stream));
    HEMM_CATCH
}
int hemm_timer_stop(void *timer, void *stream, float *ms) {
    HEMM_TRY
    need(timer && ms, "null argument");
    hemm_timer *t = (hemm_timer *)timer;
    HEMM_HIP(hipEventRecord(t->b, (hipStream_t)stream));
    HEMM_HIP(hipEventSynchronize(t->b));
    HEMM_HIP(hipEventElapsedTime(ms, t->a, t->b));
    HEMM_CATCH
}
void hemm_timer_destroy(void *timer) {
    if (!timer) return;
    hemm_timer *t = (hemm_timer *)timer;
    (void)hipEventDestroy(t->a);
    (void)hipEventDestroy(t->b);
    delete t;
}

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
               on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

static LimbList explicit_limbs(hemm_context *ctx, const uint32_t *prime_idx, uint32_t n_limbs) {
    need(ctx && prime_idx, "null argument");
    need(ctx->logN >= 9, "residue kernels need log_n >= 9");
    need(n_limbs >= 1 && n_limbs <= HEMM_MAX_PRIMES, "n_limbs out of range");
    LimbList ll;
    memset(&ll, 0, sizeof(ll));
    for (uint32_t j = 0; j < n_limbs; j++) {
        need(prime_idx[j] < (uint32_t)(ctx->nQ + ctx->nP), "prime index out of range");
        ll.idx[j] = (uint8_t)prime_idx[j];
    }
    return ll;
}

int hemm_sample_uniform(hemm_context *ctx, const uint64_t *stream_keys, const uint32_t *prime_idx, uint32_t n_limbs,
                        uint64_t *out, void *stream) {
    HEMM_TRY
    const LimbList ll = explicit_limbs(ctx, prime_idx, n_limbs);
    need(stream_keys && out, "null operand");
    launch_sample_uniform(ctx, (const u64 *)stream_keys, ll, (int)n_limbs, (u64 *)out, on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_sample_error(hemm_context *ctx, uint64_t stream_key, const uint32_t *prime_idx, uint32_t n_limbs, uint64_t *out,
                      void *stream) {
    HEMM_TRY
    const LimbList ll = explicit_limbs(ctx, prime_idx, n_limbs);
    need(out, "null operand");
    launch_sample_error(ctx, (u64)stream_key, ll, (int)n_limbs, (u64 *)out, on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

static LimbList chain_limbs(hemm_context *ctx, uint32_t nq, int with_p, int *n_limbs) {
    need(ctx, "null context");
    need(ctx->logN >= 9, "residue kernels need log_n >= 9");
    need(nq >= 1 && nq <= (uint32_t)ctx->nQ, "nq out of range");
    *n_limbs = (int)nq + (with_p ? ctx->nP : 0);
    return limbs_default(ctx, (int)nq, with_p);
}

int hemm_pointwise(hemm_context *ctx, int op, const uint64_t *a, size_t a_stride, const uint64_t *b, size_t b_stride,
                   uint64_t *out, size_t out_stride, uint32_t nq, int with_p, uint32_t n_polys, void *stream) {
    HEMM_TRY
    int nl;
    LimbList ll = chain_limbs(ctx, nq, with_p, &nl);
    need(a && out && (b || op == HEMM_NEG), "null operand");
    need(op >= 0 && op <= 4, "unknown op");
    launch_binary(ctx, op, (const u64 *)a, a_stride, (const u64 *)b, b_stride, (u64 *)out, out_stride, ll, nl,
                  (int)n_polys, on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_mul_scalar(hemm_context *ctx, const uint64_t *a, size_t a_stride, const uint64_t *scalars, uint64_t *out,
                    size_t out_stride, uint32_t nq, int with_p, uint32_t n_polys, void *stream) {
    HEMM_TRY
    int nl;
    LimbList ll = chain_limbs(ctx, nq, with_p, &nl);
    need(a && out && scalars, "null operand");
    launch_mul_scalar(ctx, (const u64 *)a, a_stride, (const u64 *)scalars, (u64 *)out, out_stride, ll, nl,
                      (int)n_polys, on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_encode(hemm_context *ctx, double *slots, double scale, uint32_t nq, int with_p, uint32_t n_msgs, uint64_t *out,
                void *stream) {
    HEMM_TRY
    int nl;
    LimbList ll = chain_limbs(ctx, nq, with_p, &nl);
    need(slots && out && n_msgs >= 1, "null operand");
    need(scale > 0, "scale must be positive");
    launch_encode(ctx, slots, scale, ll, nl, (int)n_msgs, (u64 *)out, on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_decode(hemm_context *ctx, const uint64_t *pt, uint32_t n_limbs, double scale, uint64_t *workspace, double *slots,
                void *stream) {
    HEMM_TRY
    need(pt && workspace && slots, "null operand");
    need(n_limbs >= 1 && n_limbs <= 2 && (int)n_limbs <= ctx->nQ, "decode reads one or two limbs");
    need(scale > 0, "scale must be positive");
    launch_decode(ctx, (const u64 *)pt, (int)n_limbs, scale, (u64 *)workspace, slots, on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_add_scalar(hemm_context *ctx, const uint64_t *a, const uint64_t *re, const uint64_t *im, uint64_t *out,
                    uint32_t nq, int with_p, void *stream) {
    HEMM_TRY
    int nl;
    LimbList ll = chain_limbs(ctx, nq, with_p, &nl);
    need(a && out && re, "null operand");
    need(ctx->N >= 512, "needs N >= 512");
    launch_add_scalar(ctx, (const u64 *)a, (const u64 *)re, (const u64 *)im, (u64 *)out, ll, nl, on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_zero(hemm_context *ctx, uint64_t *out, size_t words, void *stream) {
    HEMM_TRY
    need(ctx && out, "null operand");
    need((words & 1) == 0 && ((uintptr_t)out & 15) == 0, "an even number of words at a 16-byte boundary is needed");
    if (words) launch_zero(ctx, (u64 *)out, words, on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_mul_imag_unit(hemm_context *ctx, const uint64_t *a, size_t a_stride, uint64_t *out, size_t out_stride,
                       uint32_t nq, uint32_t n_polys, void *stream) {
    HEMM_TRY
    int nl;
    LimbList ll = chain_limbs(ctx, nq, 0, &nl);
    need(a && out, "null operand");
    launch_mul_imag(ctx, (const u64 *)a, a_stride, (u64 *)out, out_stride, ll, nl, (int)n_polys, on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_tensor(hemm_context *ctx, const uint64_t *ct1, size_t stride1, const uint64_t *ct2, size_t stride2,
                uint64_t *out, size_t out_stride, uint32_t nq, int accumulate, void *stream) {
    HEMM_TRY
    int nl;
    chain_limbs(ctx, nq, 0, &nl);
    need(ct1 && ct2 && out, "null operand");
    launch_tensor(ctx, (const u64 *)ct1, stride1, (const u64 *)ct2, stride2, (u64 *)out, out_stride, (int)nq,
                  accumulate != 0, on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_automorphism(hemm_context *ctx, const uint64_t *a, size_t a_stride, uint64_t *out, size_t out_stride,
                      uint64_t galois, uint32_t n_limbs, uint32_t n_polys, void *stream) {
    HEMM_TRY
    need(ctx && a && out, "null operand");
    need(ctx->logN >= 9, "residue kernels need log_n >= 9");
    need(a != out, "automorphism cannot run in place");
    need((galois & 1) && galois < 2 * (uint64_t)ctx->N, "galois element must be odd and < 2N");
    launch_galois(ctx, (const u64 *)a, a_stride, (u64 *)out, out_stride, galois, (int)n_limbs, (int)n_polys,
                  on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_modup(hemm_context *ctx, const uint64_t *in, uint32_t nq, uint64_t *ext, void *stream) {
    HEMM_TRY
    int nl;
    chain_limbs(ctx, nq, 1, &nl);
    need(in && ext, "null operand");
    need(ctx->nP >= 1, "key switching needs special primes");
    launch_modup(ctx, (const u64 *)in, (int)nq, (u64 *)ext, hemm_scratch(ctx), true, on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_inner_product(hemm_context *ctx, const uint64_t *ext, const uint64_t *evk, uint32_t nq, uint64_t *acc,
                       void *stream) {
    HEMM_TRY
    int nl;
    chain_limbs(ctx, nq, 1, &nl);
    need(ext && evk && acc, "null operand");
    launch_inner_product(ctx, nullptr, (const u64 *)ext, (const u64 *)evk, (int)nq, (u64 *)acc, on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_moddown(hemm_context *ctx, uint64_t *acc, uint32_t nq, uint32_t n_polys, uint64_t *out, size_t out_stride,
                 void *stream) {
    HEMM_TRY
    int nl;
    chain_limbs(ctx, nq, 1, &nl);
    need(acc && out, "null operand");
    need(ctx->nP >= 1, "key switching needs special primes");
    need(n_polys >= 1 && n_polys <= 2, "n_polys must be 1 or 2");
    launch_moddown(ctx, (u64 *)acc, (int)nq, (int)n_polys, (u64 *)out, out_stride, nullptr, 0, 0, hemm_scratch(ctx),
                   on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_keyswitch(hemm_context *ctx, const uint64_t *in, const uint64_t *evk, uint32_t nq, uint64_t *out,
                   size_t out_stride, const uint64_t *add_b, void *stream) {
    HEMM_TRY
    int nl;
    chain_limbs(ctx, nq, 1, &nl);
    need(in && evk && out, "null operand");
    launch_keyswitch(ctx, (const u64 *)in, (const u64 *)evk, (int)nq, (u64 *)out, out_stride, (const u64 *)add_b,
                     on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_rotate(hemm_context *ctx, const uint64_t *ct, size_t ct_stride, const uint64_t *evk, uint64_t galois,
                uint32_t nq, uint64_t *out, size_t out_stride, void *stream) {
    HEMM_TRY
    int nl;
    chain_limbs(ctx, nq, 1, &nl);
    need(ct && evk && out, "null operand");
    need((galois & 1) && galois < 2 * (uint64_t)ctx->N, "galois element must be odd and < 2N");
    const size_t N = ctx->N;
    u64 *rot = hemm_scratch(ctx) + hemm_scratch_words(ctx) - (size_t)2 * ctx->nQ * N;  // [2][nq][N]
    const hipStream_t s = on_stream(ctx, stream);
    if (modup_through_automorphism_ok(ctx, (int)nq)) {
        // No launch that rotates: the ModUp reads the second polynomial through the automorphism (first inverse pass
        // and the copies of the digits' own limbs) and the key product reads the first one through it -- the same
        // residues as rotating both first.
        launch_keyswitch(ctx, (const u64 *)ct + ct_stride, (const u64 *)evk, (int)nq, (u64 *)out, out_stride,
                         (const u64 *)ct, s, (u32)galois, true);
    } else {
        launch_galois(ctx, (const u64 *)ct, ct_stride, rot, (size_t)nq * N, galois, (int)nq, 2, s);
        launch_keyswitch(ctx, rot + (size_t)nq * N, (const u64 *)evk, (int)nq, (u64 *)out, out_stride, rot, s);
    }
    check_launch();
    HEMM_CATCH
}

int hemm_relinearize(hemm_context *ctx, const uint64_t *ct3, size_t ct_stride, const uint64_t *evk, uint32_t nq,
                     uint64_t *out, size_t out_stride, void *stream) {
    HEMM_TRY
    int nl;
    LimbList ll = chain_limbs(ctx, nq, 0, &nl);
    need(ct3 && evk && out, "null operand");
    const size_t N = ctx->N;
    if (N >= 512) {
        // (d0, d1) joins the key product of d2 in the extended basis as a term without a key: the ModDown leaves the
        // finished pair, no addition launch (P d + x divided by P is d + x / P exactly)
        launch_keyswitch(ctx, (const u64 *)ct3 + 2 * ct_stride, (const u64 *)evk, (int)nq, (u64 *)out, out_stride,
                         (const u64 *)ct3, on_stream(ctx, stream), 0, false, (const u64 *)ct3 + ct_stride);
        check_launch();
        return 0;
    }
    u64 *tmp = hemm_scratch(ctx) + hemm_scratch_words(ctx) - (size_t)2 * ctx->nQ * N;  // [2][nq][N]
    launch_keyswitch(ctx, (const u64 *)ct3 + 2 * ct_stride, (const u64 *)evk, (int)nq, tmp, (size_t)nq * N, nullptr,
                     on_stream(ctx, stream));
    launch_binary(ctx, HEMM_ADD, (const u64 *)ct3, ct_stride, tmp, (size_t)nq * N, (u64 *)out, out_stride, ll, nl, 2,
                  on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

// descriptor staging: one device region per stream, reused by every call on it (copies and kernels are ordered on the
// stream)
static void *upload_desc(hemm_context *ctx, const void *a, size_t na, const void *b, size_t nb, void **second,
                         hipStream_t s) {
    const size_t cap = 4u << 20;
    void *region = nullptr;
    for (auto &kv : ctx->d_desc)
        if (kv.first == s) region = kv.second;
    if (region == nullptr) {
        if (ctx->d_desc.size() >= 8) throw std::invalid_argument("term lists were staged on more than 8 streams of one context");
        HEMM_HIP(hipMalloc(&region, cap));
        ctx->d_desc.emplace_back(s, region);
    }
    const size_t off_b = (na + 255) & ~(size_t)255;
    if (off_b + nb > cap) throw std::invalid_argument("too many terms in one batched call");
    // the list is copied from pageable host memory that is gone when the call returns: nothing a graph could replay
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (s != nullptr && hipStreamIsCapturing(s, &capturing) == hipSuccess && capturing != hipStreamCaptureStatusNone)
        throw std::invalid_argument("a term list too long for the kernel arguments cannot be recorded into a graph");
    // both lists in one copy (pageable source: the runtime has read it when the call returns)
    std::vector<char> both(off_b + nb);
    memcpy(both.data(), a, na);
    memcpy(both.data() + off_b, b, nb);
    HEMM_HIP(hipMemcpyAsync(region, both.data(), both.size(), hipMemcpyHostToDevice, s));
    *second = (char *)region + off_b;
    return region;
}

int hemm_modup_batch(hemm_context *ctx, const uint64_t *in, size_t in_stride, uint32_t nq, uint32_t n_in,
                     uint64_t *ext, uint64_t *workspace, void *stream) {
    HEMM_TRY
    int nl;
    chain_limbs(ctx, nq, 1, &nl);
    need(in && ext && workspace && n_in >= 1, "null operand");
    need(ctx->nP >= 1, "key switching needs special primes");
    launch_modup_batch(ctx, (const u64 *)in, in_stride, (int)nq, (int)n_in, (u64 *)ext, (u64 *)workspace,
                       on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

// Validates a list of rotation terms, merges consecutive masked terms of a group that use the same key and
// Galois element into one two-source term (the kernels then stream that key once for both), and uploads
// the device descriptors.
struct RotDev {
    const u64 *ext, *b, *evk, *mask;
    u32 galois, mask_shift;
    const u64 *ext2, *b2, *mask2;
    const u64 *pt;
    u32 pt_galois, flags;
};
static_assert(sizeof(RotDev) == 80, "RotDev must match the kernels' RotTermDev");
static void build_rot_terms(hemm_context *ctx, const hemm_rot_term *terms, const uint32_t *group_offsets, uint32_t n_out,
                            std::vector<RotDev> &d, std::vector<uint32_t> &off) {
    const uint32_t n_terms = group_offsets[n_out];
    d.clear();
    off.assign(1, 0);
    d.reserve(n_terms);
    for (uint32_t o = 0; o < n_out; o++) {
        need(group_offsets[o + 1] >= group_offsets[o], "group offsets must not decrease");
        for (uint32_t t = group_offsets[o]; t < group_offsets[o + 1]; t++) {
            need(terms[t].ext != nullptr, "null pointer in a rotation term");
            // a term without a key: mask * pt * P * (b, a), the a-polynomial in `ext`; it rotates nothing
            need(terms[t].evk != nullptr || terms[t].galois == 1, "a term without a key takes the identity automorphism");
            need((terms[t].galois & 1) && terms[t].galois < 2 * (uint64_t)ctx->N, "galois element must be odd and < 2N");
            need(terms[t].mask_shift == 0 || (terms[t].mask && (int)terms[t].mask_shift < ctx->logN),
                 "mask_shift needs a run table and must be below log N");
            need(terms[t].pt == nullptr || ((terms[t].pt_galois & 1) && terms[t].pt_galois < 2 * (uint64_t)ctx->N),
                 "pt_galois must be odd and < 2N");
            need((terms[t].flags & ~(uint32_t)HEMM_ROT_COMPACT_KEY) == 0, "unknown flag in a rotation term");
            RotDev cur{(const u64 *)terms[t].ext, (const u64 *)terms[t].b, (const u64 *)terms[t].evk,
                       (const u64 *)terms[t].mask, (u32)terms[t].galois, terms[t].mask ? (u32)terms[t].mask_shift : 0u,
                       nullptr, nullptr, nullptr, (const u64 *)terms[t].pt, terms[t].pt ? (u32)terms[t].pt_galois : 1u,
                       (u32)terms[t].flags};
            if (t + 1 < group_offsets[o + 1] && terms[t].evk && terms[t].mask && terms[t + 1].mask && terms[t].b && terms[t + 1].ext && terms[t + 1].b &&
                terms[t + 1].evk == terms[t].evk && terms[t + 1].galois == terms[t].galois &&
                terms[t + 1].mask_shift == terms[t].mask_shift && terms[t + 1].pt == terms[t].pt &&
                (terms[t].pt == nullptr || terms[t + 1].pt_galois == terms[t].pt_galois)) {
                cur.ext2 = (const u64 *)terms[t + 1].ext;
                cur.b2 = (const u64 *)terms[t + 1].b;
                cur.mask2 = (const u64 *)terms[t + 1].mask;
                t++;
            }
            d.push_back(cur);
        }
        off.push_back((uint32_t)d.size());
    }
    // the key layout is a property of the launch: terms without a key follow the others
    u32 layout = 0;
    for (const RotDev &t : d)
        if (t.evk != nullptr) {
            layout = t.flags;
            break;
        }
    for (RotDev &t : d)
        if (t.evk == nullptr) t.flags = layout;
}
// hoisted sums of a validated, merged term list: short lists travel in the kernel arguments, long ones through the
// staging region
static void run_hoisted_terms(hemm_context *ctx, const hemm_rot_term *terms, const uint32_t *group_offsets, uint32_t n_out,
                              uint32_t nq, u64 *y, bool b_premultiplied, hipStream_t stream) {
    std::vector<RotDev> d;
    std::vector<uint32_t> off;
    build_rot_terms(ctx, terms, group_offsets, n_out, d, off);
    for (const RotDev &t : d)
        need(t.flags == d[0].flags, "all terms of a hoisted sum must use the same key layout");
    if ((int)d.size() <= hoisted_arg_capacity() && (int)n_out <= hoisted_arg_capacity()) {
        launch_hoisted_terms_args(ctx, d.data(), (int)d.size(), off.data(), (int)n_out, (int)nq, y, b_premultiplied, stream);
        return;
    }
    void *off_dev = nullptr;
    void *terms_dev = upload_desc(ctx, d.data(), d.size() * sizeof(RotDev), off.data(), (n_out + 1) * sizeof(uint32_t),
                                  &off_dev, stream);
    launch_hoisted_terms(ctx, terms_dev, (const u32 *)off_dev, (int)n_out, (int)nq, y, b_premultiplied, stream, d.data(),
                         (int)d.size(), !d.empty() && (d[0].flags & HEMM_ROT_COMPACT_KEY) != 0);
}

size_t hemm_key_compact_words(const hemm_context *ctx) { return ctx ? key_compact_words(ctx) : 0; }
int hemm_key_compact(hemm_context *ctx, const uint64_t *evk, uint64_t *out, void *stream) {
    HEMM_TRY
    need(ctx && evk && out, "null operand");
    launch_key_compact(ctx, (const u64 *)evk, (u64 *)out, on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_key_expand(hemm_context *ctx, const uint64_t *compact, uint64_t *evk, void *stream) {
    HEMM_TRY
    need(ctx && compact && evk, "null operand");
    launch_key_expand(ctx, (const u64 *)compact, (u64 *)evk, on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_hoisted_terms(hemm_context *ctx, const hemm_rot_term *terms, const uint32_t *group_offsets, uint32_t n_out,
                       uint32_t nq, uint64_t *y, int b_premultiplied, void *stream) {
    HEMM_TRY
    int nl;
    chain_limbs(ctx, nq, 1, &nl);
    need(terms && group_offsets && y && n_out >= 1, "null operand");
    need(ctx->nP >= 1, "key switching needs special primes");
    run_hoisted_terms(ctx, terms, group_offsets, n_out, nq, (u64 *)y, b_premultiplied != 0, on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_hoisted_moddown(hemm_context *ctx, const hemm_rot_term *terms, const uint32_t *group_offsets, uint32_t n_out,
                         uint32_t nq, int b_premultiplied, int drop_last, uint64_t *y_workspace, uint64_t *out,
                         size_t out_stride, uint64_t *workspace, void *stream) {
    HEMM_TRY
    int nl;
    chain_limbs(ctx, nq, 1, &nl);
    need(terms && group_offsets && y_workspace && out && workspace && n_out >= 1, "null operand");
    need(ctx->nP >= 1, "key switching needs special primes");
    run_hoisted_terms(ctx, terms, group_offsets, n_out, nq, (u64 *)y_workspace, b_premultiplied != 0, on_stream(ctx, stream));
    launch_moddown_batch(ctx, (u64 *)y_workspace, (int)nq, (int)(2 * n_out), drop_last != 0, (u64 *)out, out_stride,
                         (u64 *)workspace, on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_moddown_batch(hemm_context *ctx, uint64_t *y, uint32_t nq, uint32_t n_polys, int drop_last, uint64_t *out,
                       size_t out_stride, uint64_t *workspace, void *stream) {
    HEMM_TRY
    int nl;
    chain_limbs(ctx, nq, 1, &nl);
    need(y && out && workspace && n_polys >= 1, "null operand");
    need(ctx->nP >= 1, "key switching needs special primes");
    need((drop_last & ~(1 | HEMM_MODDOWN_COLUMN_SLAB)) == 0, "unknown ModDown flag");
    launch_moddown_batch(ctx, (u64 *)y, (int)nq, (int)n_polys, (drop_last & 1) != 0, (u64 *)out, out_stride,
                         (u64 *)workspace, on_stream(ctx, stream), (drop_last & HEMM_MODDOWN_COLUMN_SLAB) != 0);
    check_launch();
    HEMM_CATCH
}

int hemm_masked_sum_batch(hemm_context *ctx, const hemm_lin_term *terms, const uint32_t *group_offsets, uint32_t n_out,
                          uint32_t nq, uint32_t n_polys, uint64_t *out, void *stream) {
    HEMM_TRY
    int nl;
    chain_limbs(ctx, nq, 0, &nl);
    need(terms && group_offsets && out && n_out >= 1 && n_polys >= 1, "null operand");
    const uint32_t n_terms = group_offsets[n_out];
    for (uint32_t t = 0; t < n_terms; t++) {
        need(terms[t].ct != nullptr, "null pointer in a term");
        need(terms[t].galois == 0 || ((terms[t].galois & 1) && terms[t].galois < 2 * (uint64_t)ctx->N),
             "galois element must be odd and < 2N");
    }
    static_assert(sizeof(hemm_lin_term) == 32, "the kernels read these records as they are");
    if ((int)n_terms <= masked_arg_capacity() && (int)n_out <= masked_arg_capacity()) {
        launch_masked_sum_args(ctx, terms, (int)n_terms, group_offsets, (int)n_out, (int)nq, (int)n_polys, (u64 *)out,
                               on_stream(ctx, stream));
        check_launch();
        return 0;
    }
    void *off_dev = nullptr;
    void *terms_dev = upload_desc(ctx, terms, n_terms * sizeof(hemm_lin_term), group_offsets,
                                  (n_out + 1) * sizeof(uint32_t), &off_dev, on_stream(ctx, stream));
    launch_masked_sum(ctx, terms_dev, (const u32 *)off_dev, (int)n_out, (int)nq, (int)n_polys, (u64 *)out,
                      on_stream(ctx, stream), terms, (int)n_terms);
    check_launch();
    HEMM_CATCH
}

int hemm_context_set_stream(hemm_context *ctx, void *stream) {
    HEMM_TRY
    need(ctx != nullptr, "null context");
    ctx->stream = (hipStream_t)stream;
    HEMM_CATCH
}
void *hemm_context_stream(const hemm_context *ctx) { return ctx ? (void *)ctx->stream : nullptr; }

int hemm_traffic(hemm_context *ctx, uint64_t *bytes, uint64_t *launches, int reset) {
    HEMM_TRY
    need(ctx != nullptr, "null context");
    for (int k = 0; k < HEMM_TRAFFIC_KINDS; k++) {
        if (bytes) bytes[k] = k < TR_KINDS ? ctx->traffic[k] : 0;
        if (launches) launches[k] = k < TR_KINDS ? ctx->launches[k] : 0;
    }
    if (reset) {
        memset(ctx->traffic, 0, sizeof(ctx->traffic));
        memset(ctx->launches, 0, sizeof(ctx->launches));
    }
    HEMM_CATCH
}

void hemm_abi_sizes(uint32_t *rot_term_bytes, uint32_t *lin_term_bytes) {
    if (rot_term_bytes) *rot_term_bytes = (uint32_t)sizeof(hemm_rot_term);
    if (lin_term_bytes) *lin_term_bytes = (uint32_t)sizeof(hemm_lin_term);
}

int hemm_sum_parts(hemm_context *ctx, const uint64_t *parts, uint32_t n_parts, uint32_t n_out, uint32_t nq, uint64_t *y,
                   void *stream) {
    HEMM_TRY
    int nl;
    chain_limbs(ctx, nq, 1, &nl);
    need(parts && y && n_parts >= 1 && n_out >= 1, "null operand");
    need(ctx->N >= 2, "ring too small");
    launch_sum_parts(ctx, (const u64 *)parts, (int)n_parts, (int)n_out, (int)nq, (u64 *)y, on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_compact_mask(hemm_context *ctx, const uint64_t *mask, uint32_t n_limbs, uint32_t shift, uint64_t *table,
                      int *is_constant, void *stream) {
    HEMM_TRY
    need(mask && table && is_constant, "null operand");
    need((int)n_limbs > ctx->nP && shift >= 1 && (int)shift < ctx->logN,
         "the mask must cover the extended basis and shift must be in [1, log N)");
    *is_constant = launch_compact_mask(ctx, (const u64 *)mask, (int)n_limbs, (int)shift, (u64 *)table, on_stream(ctx, stream)) ? 1 : 0;
    check_launch();
    HEMM_CATCH
}

int hemm_tensor_batch(hemm_context *ctx, const uint64_t *t1, const uint64_t *t2, uint32_t n_pairs, uint32_t nq,
                      uint64_t *acc3, int accumulate, void *stream) {
    return hemm_tensor_batch_strided(ctx, t1, t2, n_pairs, nq, acc3, (size_t)nq * (size_t)ctx->N, accumulate, stream);
}
int hemm_tensor_batch_strided(hemm_context *ctx, const uint64_t *t1, const uint64_t *t2, uint32_t n_pairs, uint32_t nq,
                              uint64_t *acc3, size_t acc_stride, int accumulate, void *stream) {
    HEMM_TRY
    int nl;
    chain_limbs(ctx, nq, 0, &nl);
    need(t1 && t2 && acc3 && n_pairs >= 1, "null operand");
    need(acc_stride >= (size_t)nq * (size_t)ctx->N, "accumulator stride below one polynomial");
    launch_tensor_batch(ctx, (const u64 *)t1, (const u64 *)t2, (int)n_pairs, (int)nq, (u64 *)acc3, acc_stride,
                        accumulate != 0, on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_tensor_batch_groups(hemm_context *ctx, const hemm_tensor_group *groups, uint32_t n_groups, uint32_t nq,
                             size_t acc_stride, void *stream) {
    HEMM_TRY
    int nl;
    chain_limbs(ctx, nq, 0, &nl);
    need(groups != nullptr && n_groups >= 1 && (int)n_groups <= tensor_max_groups(), "between 1 and 8 groups per call");
    need(acc_stride >= (size_t)nq * (size_t)ctx->N, "accumulator stride below one polynomial");
    std::vector<TensorGroupHost> g(n_groups);
    const size_t poly = (size_t)nq * (size_t)ctx->N;
    for (uint32_t i = 0; i < n_groups; i++) {
        need(groups[i].t1 && groups[i].t2 && groups[i].acc3 && groups[i].n_pairs >= 1, "null operand");
        need(groups[i].accumulate <= 1, "accumulate is 0 or 1");
        // polynomial p of accumulator i covers [acc3 + p * stride, + poly): no two of one call may overlap
        for (uint32_t k = 0; k < i; k++)
            for (int p = 0; p < 3; p++)
                for (int r = 0; r < 3; r++) {
                    const uint64_t *a = groups[i].acc3 + p * acc_stride, *b = groups[k].acc3 + r * acc_stride;
                    need(a + poly <= b || b + poly <= a, "accumulators of one call overlap");
                }
        g[i] = TensorGroupHost{(const u64 *)groups[i].t1, (const u64 *)groups[i].t2, (u64 *)groups[i].acc3,
                               (int)groups[i].n_pairs, groups[i].accumulate != 0};
    }
    launch_tensor_groups(ctx, g.data(), (int)n_groups, (int)nq, acc_stride, on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

// Strides of a batch must hold a whole polynomial, and the output may only share memory with the input when both lay
// their polynomials out alike (out == in, equal strides: polynomial p of the result then overwrites the first nq - 1
// limbs of polynomial p of the input, which the call has read by then); any other overlap would let one polynomial's
// result land in another's unread input.
static void check_rescale_layout(const hemm_context *ctx, const uint64_t *in, size_t in_stride, const uint64_t *out,
                                 size_t out_stride, uint32_t nq, uint32_t n_polys) {
    const size_t N = ctx->N, in_words = (size_t)nq * N, out_words = (size_t)(nq - 1) * N;
    if (n_polys > 1) {
        need(in_stride >= in_words, "in_stride is shorter than a polynomial of nq limbs");
        need(out_stride >= out_words, "out_stride is shorter than a polynomial of nq - 1 limbs");
    }
    const uint64_t *in_end = in + (size_t)(n_polys - 1) * in_stride + in_words;
    const uint64_t *out_end = out + (size_t)(n_polys - 1) * out_stride + out_words;
    const bool overlap = out < in_end && in < out_end;
    need(!overlap || (out == in && (n_polys == 1 || out_stride == in_stride)),
         "out overlaps in (only out == in with equal strides is allowed)");
}

int hemm_rescale(hemm_context *ctx, const uint64_t *in, size_t in_stride, uint64_t *out, size_t out_stride,
                 uint32_t nq, uint32_t n_polys, void *stream) {
    HEMM_TRY
    int nl;
    chain_limbs(ctx, nq, 0, &nl);
    need(in && out, "null operand");
    need(nq >= 2, "rescale needs at least two limbs");
    need(n_polys >= 1 && (size_t)n_polys * nq * ctx->N <= hemm_scratch_words(ctx),
         "n_polys * nq limbs must fit the context's scratch ((dnum + 7) * (nQ + nP) limbs)");
    check_rescale_layout(ctx, in, in_stride, out, out_stride, nq, n_polys);
    launch_rescale(ctx, (const u64 *)in, in_stride, (u64 *)out, out_stride, (int)nq, (int)n_polys,
                   on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

int hemm_rescale_static(hemm_context *ctx, const uint64_t *in, size_t in_stride, uint64_t *out, size_t out_stride,
                        uint32_t nq, uint32_t n_polys, void *stream) {
    HEMM_TRY
    need(ctx && in && out, "null operand");
    need(ctx->logN >= 9, "residue kernels need log_n >= 9");
    need(nq >= 2 && nq <= (uint32_t)ctx->nQ, "nq must be in [2, n_q]");
    need(n_polys >= 1 && (size_t)n_polys * nq * ctx->N <= hemm_static_scratch_words(),
         "n_polys * nq * N must not exceed HEMM_STATIC_SCRATCH_WORDS");
    check_rescale_layout(ctx, in, in_stride, out, out_stride, nq, n_polys);
    launch_rescale_static(ctx, (const u64 *)in, in_stride, (u64 *)out, out_stride, (int)nq, (int)n_polys,
                          on_stream(ctx, stream));
    check_launch();
    HEMM_CATCH
}

}  // extern "C"

static_assert(HEMM_STATIC_SCRATCH_WORDS == ((size_t)32 << 16), "hemm.h documents 32 limbs of N = 2^16");

// extern "C" facade over HELLM::HEMMer (declared in include/hellm.h).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>

#include "../../../include/hellm.h"
#include "HELLM/HEMMer.hpp"
#include "HELLM/PolyEval.hpp"
#include "context_content.hpp"

void hemm_set_error(const std::string &msg);

using namespace HELLM;

struct hellm_hemmer {
    HEMMer *m;
};
struct hellm_ct {
    CtxtTensor t;
};
struct hellm_pt {
    PtxtTensor t;
};
struct hellm_ctvec {
    std::vector<Ciphertext> v;
};

#define FACADE_TRY try {
#define FACADE_CATCH                           \
    }                                          \
    catch (const std::invalid_argument &e) {   \
        hemm_set_error(e.what());              \
        return 1;                              \
    }                                          \
    catch (const std::exception &e) {          \
        hemm_set_error(e.what());              \
        return 2;                              \
    }                                          \
    return 0;

static Matrix mat(const double *p, uint32_t rows, uint32_t cols) {
    if (!p) throw std::invalid_argument("null matrix");
    Matrix m(rows, cols);
    memcpy(m.v.data(), p, sizeof(double) * m.v.size());
    return m;
}
static void need(bool ok, const char *msg) {
    if (!ok) throw std::invalid_argument(msg);
}

extern "C" {

int hellm_hemmer_create(uint32_t log_n, uint32_t n_q, uint32_t n_p, const uint64_t *primes, uint32_t dnum,
                        uint32_t log_scale, uint32_t min_boot, uint64_t seed, hellm_hemmer **out) {
    FACADE_TRY
    need(primes && out, "null argument");
    HEaaN::setSeed(seed);
    std::vector<u64> q(primes, primes + n_q), p(primes + n_q, primes + n_q + n_p);
    Context c = makeContextCustom(log_n, q, p, dnum, log_scale);
    *out = new hellm_hemmer{new HEMMer(c, min_boot)};
    FACADE_CATCH
}
int hellm_hemmer_create_preset(uint64_t seed, hellm_hemmer **out) {
    FACADE_TRY
    need(out, "null argument");
    HEaaN::setSeed(seed);
    *out = new hellm_hemmer{new HEMMer(0, ParameterPreset::FGb)};
    FACADE_CATCH
}
void hellm_hemmer_destroy(hellm_hemmer *h) {
    if (!h) return;
    delete h->m;
    delete h;
}
int hellm_hemmer_info(hellm_hemmer *h, uint32_t *log_n, uint32_t *n_q, uint32_t *n_p, uint32_t *dnum, uint32_t *dim,
                      uint64_t *primes) {
    FACADE_TRY
    need(h, "null argument");
    const Context &c = h->m->getContext();
    if (log_n) *log_n = (uint32_t)c->logN;
    if (n_q) *n_q = (uint32_t)c->nQ;
    if (n_p) *n_p = (uint32_t)c->nP;
    if (dnum) *dnum = (uint32_t)c->dnum;
    if (dim) *dim = (uint32_t)h->m->dim();
    if (primes) {
        auto l = getPrimeList(c);
        memcpy(primes, l.data(), l.size() * 8);
    }
    FACADE_CATCH
}
int hellm_secret_coeffs(hellm_hemmer *h, int32_t *out) {
    FACADE_TRY
    need(h && out, "null argument");
    const auto &v = h->m->getsk().getCoefficients();
    for (size_t i = 0; i < v.size(); i++) out[i] = v[i];
    FACADE_CATCH
}
int hellm_export_key(hellm_hemmer *h, uint64_t galois, uint64_t *out) {
    FACADE_TRY
    need(h && out, "null argument");
    const Context &c = h->m->getContext();
    const size_t words = c->dnum * 2 * (c->nQ + c->nP) * c->N;
    // the key pack is reachable through the evaluator's relinearize / rotate only; export via a friend path
    const u64 *src = galois == 0 ? h->m->keyPack().multKey() : h->m->keyPack().galoisKey(galois);
    if (hipMemcpy(out, src, words * 8, hipMemcpyDeviceToHost) != hipSuccess) throw RuntimeException("hipMemcpy failed");
    FACADE_CATCH
}
int hellm_ensure_rotation_keys(hellm_hemmer *h, const uint64_t *rots, uint32_t count) {
    FACADE_TRY
    need(h && rots, "null argument");
    h->m->ensureRotationKeys(std::vector<u64>(rots, rots + count));
    FACADE_CATCH
}
int hellm_set_schedule(hellm_hemmer *h, int fused, uint32_t batch) {
    FACADE_TRY
    need(h && batch >= 1, "bad argument");
    h->m->setFused(fused != 0, batch);
    FACADE_CATCH
}
int hellm_assume_single_tile(hellm_hemmer *h, int on) {
    FACADE_TRY
    need(h != nullptr, "null argument");
    h->m->assumeSingleTile(on != 0);
    FACADE_CATCH
}
int hellm_sync(void) {
    FACADE_TRY
    CudaTools::cudaDeviceSynchronize();
    FACADE_CATCH
}

int hellm_key_bytes(hellm_hemmer *h, uint64_t *plain, uint64_t *compact, uint64_t *pool) {
    FACADE_TRY
    need(h, "null argument");
    const auto kb = h->m->keyPack().keyBytes();
    if (plain) *plain = kb.first;
    if (compact) *compact = kb.second;
    if (pool) *pool = h->m->getContext()->pool_bytes;
    FACADE_CATCH
}
int hellm_phase_trace(hellm_hemmer *h, int on) {
    FACADE_TRY
    need(h, "null argument");
    auto &c = *h->m->getContext();
    c.traceClear();
    c.trace_on = on != 0;
    FACADE_CATCH
}
int hellm_phase_report(hellm_hemmer *h, char *text, size_t capacity) {
    FACADE_TRY
    need(h && text && capacity > 0, "null argument");
    auto &c = *h->m->getContext();
    if (hipDeviceSynchronize() != hipSuccess) throw RuntimeException("hipDeviceSynchronize failed");
    std::string out;
    for (size_t i = 1; i < c.trace_marks.size(); i++) {
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, c.trace_marks[i - 1].second, c.trace_marks[i].second) != hipSuccess)
            throw RuntimeException("hipEventElapsedTime failed");
        out += c.trace_marks[i].first + "\t" + std::to_string(ms) + "\n";
    }
    need(out.size() + 1 <= capacity, "report does not fit the buffer");
    memcpy(text, out.c_str(), out.size() + 1);
    c.traceClear();
    FACADE_CATCH
}
// ---- a sequence of calls recorded once and replayed (HIP graph) ----------------------------------------------------
struct hellm_graph {
    HEaaN::Context ctx;
    hipStream_t stream = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    std::vector<std::pair<size_t, HEaaN::u64 *>> owned;   // intermediates of the recorded calls
    size_t nodes = 0;
};
namespace {
void hipck(hipError_t e, const char *what) {
    if (e != hipSuccess) throw RuntimeException(std::string(what) + ": " + hipGetErrorString(e));
}
thread_local hellm_graph *g_recording = nullptr;
}  // namespace
int hellm_graph_begin(hellm_hemmer *h) {
    FACADE_TRY
    need(h, "null argument");
    if (g_recording) throw RuntimeException("a recording is already open on this thread");
    HEaaN::Context c = h->m->getContext();
    if (c->side_open || c->capture_open || c->stream() != nullptr)
        throw RuntimeException("the context is busy with another stream");
    auto *g = new hellm_graph();
    g->ctx = c;
    try {
        hipck(hipDeviceSynchronize(), "hipDeviceSynchronize");
        hipck(hipStreamCreateWithFlags(&g->stream, hipStreamNonBlocking), "hipStreamCreateWithFlags");
        if (hemm_context_set_stream(c->dev, g->stream) != 0) throw RuntimeException(hemm_last_error());
        hipck(hipStreamBeginCapture(g->stream, hipStreamCaptureModeRelaxed), "hipStreamBeginCapture");
    } catch (...) {
        (void)hemm_context_set_stream(c->dev, nullptr);
        if (g->stream) (void)hipStreamDestroy(g->stream);
        delete g;
        throw;
    }
    c->capture_open = true;
    g_recording = g;
    FACADE_CATCH
}
int hellm_graph_end(hellm_hemmer *h, hellm_graph **out) {
    FACADE_TRY
    need(h && out, "null argument");
    hellm_graph *g = g_recording;
    if (!g || g->ctx != h->m->getContext()) throw RuntimeException("no recording is open on this context");
    g_recording = nullptr;
    HEaaN::Context c = g->ctx;
    const hipError_t e = hipStreamEndCapture(g->stream, &g->graph);
    (void)hemm_context_set_stream(c->dev, nullptr);
    {
        std::lock_guard<std::mutex> lk(c->mu);
        c->capture_open = false;
        g->owned.swap(c->captured);
    }
    auto drop = [&]() {
        std::lock_guard<std::mutex> lk(c->mu);
        for (auto &kv : g->owned) c->pool.emplace(kv.first, kv.second);
        if (g->graph) (void)hipGraphDestroy(g->graph);
        (void)hipStreamDestroy(g->stream);
        delete g;
    };
    if (e != hipSuccess) {
        drop();
        throw RuntimeException(std::string("hipStreamEndCapture: ") + hipGetErrorString(e));
    }
    if (hipGraphGetNodes(g->graph, nullptr, &g->nodes) != hipSuccess) g->nodes = 0;
    const hipError_t ei = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
    if (ei != hipSuccess) {
        drop();
        throw RuntimeException(std::string("hipGraphInstantiate: ") + hipGetErrorString(ei));
    }
    *out = g;
    FACADE_CATCH
}
int hellm_graph_launch(hellm_graph *g) {
    FACADE_TRY
    need(g && g->exec, "null argument");
    hipck(hipGraphLaunch(g->exec, g->stream), "hipGraphLaunch");
    FACADE_CATCH
}
int hellm_graph_sync(hellm_graph *g) {
    FACADE_TRY
    need(g, "null argument");
    hipck(hipStreamSynchronize(g->stream), "hipStreamSynchronize");
    FACADE_CATCH
}
int hellm_graph_nodes(const hellm_graph *g, uint64_t *out) {
    FACADE_TRY
    need(g && out, "null argument");
    *out = g->nodes;
    FACADE_CATCH
}
void hellm_graph_destroy(hellm_graph *g) {
    if (!g) return;
    (void)hipStreamSynchronize(g->stream);
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    (void)hipStreamDestroy(g->stream);
    {
        std::lock_guard<std::mutex> lk(g->ctx->mu);
        for (auto &kv : g->owned) g->ctx->pool.emplace(kv.first, kv.second);
    }
    delete g;
}

int hellm_traffic(hellm_hemmer *h, uint64_t *bytes, uint64_t *launches, int reset) {
    FACADE_TRY
    need(h, "null argument");
    if (hemm_traffic(h->m->getContext()->dev, bytes, launches, reset) != 0) throw RuntimeException(hemm_last_error());
    FACADE_CATCH
}

int hellm_encrypt(hellm_hemmer *h, const double *m, uint32_t rows, uint32_t cols, hellm_ct **out) {
    FACADE_TRY
    need(h && out, "null argument");
    *out = new hellm_ct{h->m->encrypt(mat(m, rows, cols))};
    FACADE_CATCH
}
int hellm_encrypt2(hellm_hemmer *h, const double *a, const double *b, uint32_t rows, uint32_t cols, hellm_ct **out) {
    FACADE_TRY
    need(h && out, "null argument");
    *out = new hellm_ct{h->m->encrypt2(mat(a, rows, cols), mat(b, rows, cols))};
    FACADE_CATCH
}
int hellm_encode(hellm_hemmer *h, const double *m, uint32_t rows, uint32_t cols, uint32_t level, hellm_pt **out) {
    FACADE_TRY
    need(h && out, "null argument");
    *out = new hellm_pt{h->m->encode(mat(m, rows, cols), level)};
    FACADE_CATCH
}
int hellm_encode2(hellm_hemmer *h, const double *a, const double *b, uint32_t rows, uint32_t cols, uint32_t level,
                  hellm_pt **out) {
    FACADE_TRY
    need(h && out, "null argument");
    *out = new hellm_pt{h->m->encode2(mat(a, rows, cols), mat(b, rows, cols), level)};
    FACADE_CATCH
}
int hellm_encode_diagonal_to_row4(hellm_hemmer *h, const double *w1, const double *w2, const double *w3,
                                  const double *w4, uint32_t rows, uint32_t cols, uint32_t level, hellm_pt **out) {
    FACADE_TRY
    need(h && out, "null argument");
    *out = new hellm_pt{h->m->encodeDiagonalToRow4(mat(w1, rows, cols), mat(w2, rows, cols), mat(w3, rows, cols),
                                                   mat(w4, rows, cols), level)};
    FACADE_CATCH
}
int hellm_reduce_row_sum_with_scaled_mask(hellm_hemmer *h, hellm_ct *a, const double *mask_left, const double *mask_right,
                                          uint32_t rows, uint32_t cols) {
    FACADE_TRY
    need(h && a && mask_left && mask_right, "null argument");
    h->m->reduceRowSumWithScaledMask(a->t, h->m->message2(mat(mask_left, rows, cols), mat(mask_right, rows, cols)));
    FACADE_CATCH
}
int hellm_one_mat_rot_sum_inplace(hellm_hemmer *h, hellm_ct *a, hellm_ct *b) {
    FACADE_TRY
    need(h && a && b, "null argument");
    h->m->oneMatRotSumInplace(a->t, b->t);
    FACADE_CATCH
}
int hellm_mask_right_left(hellm_hemmer *h, const hellm_ct *a, hellm_ct **out_left, hellm_ct **out_right) {
    FACADE_TRY
    need(h && a && out_left && out_right, "null argument");
    hellm_ct *l = new hellm_ct{a->t}, *r = new hellm_ct{a->t};
    h->m->maskRightLeft(a->t, l->t, r->t);
    *out_left = l;
    *out_right = r;
    FACADE_CATCH
}
int hellm_mask_first_col_inplace(hellm_hemmer *h, hellm_ct *a) {
    FACADE_TRY
    need(h && a, "null argument");
    h->m->maskFirstColInplace(a->t);
    FACADE_CATCH
}
int hellm_row_moments(hellm_hemmer *h, const hellm_ct *const *tiles, uint32_t count, double inv_count, hellm_ct **mean,
                      hellm_ct **mean_square) {
    FACADE_TRY
    need(h && tiles && count >= 1 && mean && mean_square, "null argument");
    std::vector<HELLM::CtxtTensor> v;
    for (uint32_t i = 0; i < count; i++) {
        need(tiles[i] != nullptr, "null tile");
        v.push_back(tiles[i]->t);
    }
    hellm_ct *m = new hellm_ct{v[0]}, *sq = new hellm_ct{v[0]};
    h->m->rowMoments(v, inv_count, m->t, sq->t);
    *mean = m;
    *mean_square = sq;
    FACADE_CATCH
}
int hellm_encode_weight_grid(hellm_hemmer *h, const double *tiles, uint32_t height, uint32_t width, uint32_t rows,
                             uint32_t cols, const char *save_path) {
    FACADE_TRY
    need(h && tiles && save_path, "null argument");
    std::vector<std::vector<Matrix>> grid(height);
    for (uint32_t i = 0; i < height; i++)
        for (uint32_t j = 0; j < width; j++)
            grid[i].push_back(mat(tiles + ((size_t)i * width + j) * rows * cols, rows, cols));
    h->m->encodeWeight(grid, save_path);
    FACADE_CATCH
}
int hellm_encode_weight_list(hellm_hemmer *h, const double *tiles, uint32_t count, uint32_t rows, uint32_t cols,
                             const char *save_path) {
    FACADE_TRY
    need(h && tiles && save_path, "null argument");
    std::vector<Matrix> v;
    for (uint32_t i = 0; i < count; i++) v.push_back(mat(tiles + (size_t)i * rows * cols, rows, cols));
    h->m->encodeWeight(v, save_path);
    FACADE_CATCH
}
int hellm_get_weight(hellm_hemmer *h, const char *file, uint32_t level, hellm_pt **out) {
    FACADE_TRY
    need(h && file && out, "null argument");
    *out = new hellm_pt{h->m->getWeight(file, level)};
    FACADE_CATCH
}
int hellm_ct_save(hellm_hemmer *h, const hellm_ct *ct, const char *file) {
    FACADE_TRY
    need(h && ct && file, "null argument");
    h->m->saveCtxtTensor(ct->t, file);
    FACADE_CATCH
}
int hellm_ct_load(hellm_hemmer *h, const char *file, hellm_ct **out) {
    FACADE_TRY
    need(h && file && out, "null argument");
    *out = new hellm_ct{h->m->loadCtxtTensor(file)};
    FACADE_CATCH
}
int hellm_decrypt(hellm_hemmer *h, const hellm_ct *ct, double *out) {
    FACADE_TRY
    need(h && ct && out, "null argument");
    Matrix m = h->m->decrypt(ct->t);
    memcpy(out, m.v.data(), m.v.size() * sizeof(double));
    FACADE_CATCH
}
int hellm_decrypt2(hellm_hemmer *h, const hellm_ct *ct, double *out) {
    FACADE_TRY
    need(h && ct && out, "null argument");
    auto ms = h->m->decrypt2(ct->t);
    memcpy(out, ms[0].v.data(), ms[0].v.size() * sizeof(double));
    memcpy(out + ms[0].v.size(), ms[1].v.data(), ms[1].v.size() * sizeof(double));
    FACADE_CATCH
}
int hellm_decrypt_slots(hellm_hemmer *h, const hellm_ct *ct, double *re_im) {
    FACADE_TRY
    need(h && ct && re_im, "null argument");
    Message msg(getLogFullSlots(h->m->getContext()));
    h->m->getDec().decrypt(ct->t.get(), h->m->getsk(), msg);
    for (u64 i = 0; i < msg.getSize(); i++) {
        re_im[2 * i] = msg[i].real();
        re_im[2 * i + 1] = msg[i].imag();
    }
    FACADE_CATCH
}

int hellm_ct_info(const hellm_ct *ct, uint32_t *num_poly, uint32_t *level, uint32_t *rc, uint32_t *rows,
                  uint32_t *cols, uint32_t *bw) {
    FACADE_TRY
    need(ct, "null argument");
    if (num_poly) *num_poly = (uint32_t)ct->t.get().getNumPoly();
    if (level) *level = (uint32_t)ct->t.get().getLevel();
    if (rc) *rc = (uint32_t)ct->t.get().getRescaleCounter();
    if (rows) *rows = (uint32_t)ct->t.getHeight();
    if (cols) *cols = (uint32_t)ct->t.getWidth();
    if (bw) *bw = (uint32_t)ct->t.getBlockWidth();
    FACADE_CATCH
}
int hellm_ct_download(const hellm_ct *ct, uint64_t *out) {
    FACADE_TRY
    need(ct && out, "null argument");
    const Ciphertext &c = ct->t.get();
    if (hipMemcpy(out, c.buf_.data(), c.buf_.words() * 8, hipMemcpyDeviceToHost) != hipSuccess)
        throw RuntimeException("hipMemcpy failed");
    FACADE_CATCH
}
int hellm_ct_upload(hellm_hemmer *h, const uint64_t *residues, uint32_t num_poly, uint32_t level, uint32_t rc,
                    uint32_t rows, uint32_t cols, uint32_t bw, hellm_ct **out) {
    FACADE_TRY
    need(h && residues && out, "null argument");
    const Context &c = h->m->getContext();
    need(num_poly >= 1 && num_poly <= 3 && level < c->nQ, "bad ciphertext shape");
    Ciphertext ct(c);
    ct.allocate(num_poly, level, rc);
    if (hipMemcpy(ct.buf_.data(), residues, ct.buf_.words() * 8, hipMemcpyHostToDevice) != hipSuccess)
        throw RuntimeException("hipMemcpy failed");
    *out = new hellm_ct{CtxtTensor(TileTensorShape(rows, cols, bw), ct)};
    FACADE_CATCH
}
int hellm_ct_clone(const hellm_ct *ct, hellm_ct **out) {
    FACADE_TRY
    need(ct && out, "null argument");
    *out = new hellm_ct{ct->t};
    FACADE_CATCH
}
int hellm_ct_assign(hellm_hemmer *h, hellm_ct *dst, const hellm_ct *src) {
    FACADE_TRY
    need(h && dst && src, "null argument");
    HEaaN::Ciphertext &d = dst->t.get();
    const HEaaN::Ciphertext &s = src->t.get();
    if (d.getNumPoly() != s.getNumPoly() || d.getLevel() != s.getLevel() || d.getRescaleCounter() != s.getRescaleCounter() ||
        d.buf_.words() != s.buf_.words())
        throw std::invalid_argument("[assign] the two ciphertexts differ in polynomials, level or pending rescales");
    if (d.buf_.data() != s.buf_.data() &&
        hipMemcpyAsync(d.buf_.data(), s.buf_.data(), s.buf_.words() * 8, hipMemcpyDeviceToDevice, h->m->getContext()->stream()) !=
            hipSuccess)
        throw RuntimeException("hipMemcpyAsync failed");
    d.occupied_ = std::max(d.occupied_, s.occupied_);   // never claims more empty slots than either had
    FACADE_CATCH
}
void hellm_ct_destroy(hellm_ct *ct) { delete ct; }
void hellm_pt_destroy(hellm_pt *pt) { delete pt; }
int hellm_pt_download(const hellm_pt *pt, uint32_t *level, uint64_t *out) {
    FACADE_TRY
    need(pt, "null argument");
    if (level) *level = (uint32_t)pt->t.getLevel();
    if (out && hipMemcpy(out, pt->t.get().buf_.data(), pt->t.get().buf_.words() * 8, hipMemcpyDeviceToHost) != hipSuccess)
        throw RuntimeException("hipMemcpy failed");
    FACADE_CATCH
}
void hellm_ctvec_destroy(hellm_ctvec *v) { delete v; }
int hellm_ctvec_size(const hellm_ctvec *v, uint32_t *out) {
    FACADE_TRY
    need(v && out, "null argument");
    *out = (uint32_t)v->v.size();
    FACADE_CATCH
}
int hellm_ctvec_get(const hellm_ctvec *v, uint32_t i, uint32_t rows, uint32_t cols, uint32_t bw, hellm_ct **out) {
    FACADE_TRY
    need(v && out && i < v->v.size(), "bad argument");
    *out = new hellm_ct{CtxtTensor(TileTensorShape(rows, cols, bw), v->v[i])};
    FACADE_CATCH
}

#define UNARY_EVAL(name, expr)                                        \
    int name(hellm_hemmer *h, const hellm_ct *a, hellm_ct **out) {    \
        FACADE_TRY                                                    \
        need(h && a && out, "null argument");                         \
        hellm_ct *r = new hellm_ct{a->t};                             \
        try {                                                         \
            expr;                                                     \
        } catch (...) {                                               \
            delete r;                                                 \
            throw;                                                    \
        }                                                             \
        *out = r;                                                     \
        FACADE_CATCH                                                  \
    }

int hellm_left_rotate(hellm_hemmer *h, const hellm_ct *a, uint64_t rot, hellm_ct **out) {
    FACADE_TRY
    need(h && a && out, "null argument");
    h->m->ensureRotationKeys({rot});
    hellm_ct *r = new hellm_ct{a->t};
    h->m->getEval().leftRotate(a->t.get(), rot, r->t.get());
    *out = r;
    FACADE_CATCH
}
UNARY_EVAL(hellm_conjugate, h->m->getEval().conjugate(a->t.get(), r->t.get()))
UNARY_EVAL(hellm_mult_imag_unit, h->m->getEval().multImagUnit(a->t.get(), r->t.get()))
UNARY_EVAL(hellm_diagonal_to_column, r->t = h->m->diagonalToColumn(a->t))
UNARY_EVAL(hellm_diagonal_to_row, r->t = h->m->diagonalToRow(a->t))

int hellm_mult(hellm_hemmer *h, const hellm_ct *a, const hellm_ct *b, hellm_ct **out) {
    FACADE_TRY
    need(h && a && b && out, "null argument");
    hellm_ct *r = new hellm_ct{a->t};
    h->m->getEval().mult(a->t.get(), b->t.get(), r->t.get());
    *out = r;
    FACADE_CATCH
}
int hellm_mult_const(hellm_hemmer *h, const hellm_ct *a, double re, double im, hellm_ct **out) {
    FACADE_TRY
    need(h && a && out, "null argument");
    hellm_ct *r = new hellm_ct{a->t};
    h->m->getEval().mult(a->t.get(), HEaaN::Complex(re, im), r->t.get());
    *out = r;
    FACADE_CATCH
}
int hellm_add_const(hellm_hemmer *h, const hellm_ct *a, double re, double im, hellm_ct **out) {
    FACADE_TRY
    need(h && a && out, "null argument");
    hellm_ct *r = new hellm_ct{a->t};
    h->m->getEval().add(a->t.get(), HEaaN::Complex(re, im), r->t.get());
    *out = r;
    FACADE_CATCH
}
int hellm_add(hellm_hemmer *h, const hellm_ct *a, const hellm_ct *b, hellm_ct **out) {
    FACADE_TRY
    need(h && a && b && out, "null argument");
    hellm_ct *r = new hellm_ct{a->t};
    h->m->getEval().add(a->t.get(), b->t.get(), r->t.get());
    *out = r;
    FACADE_CATCH
}
int hellm_level_down(hellm_hemmer *h, const hellm_ct *a, uint32_t target, hellm_ct **out) {
    FACADE_TRY
    need(h && a && out, "null argument");
    hellm_ct *r = new hellm_ct{a->t};
    h->m->getEval().levelDown(a->t.get(), target, r->t.get());
    *out = r;
    FACADE_CATCH
}

int hellm_exp_iter(hellm_hemmer *h, const hellm_ct *a, int num_iter, hellm_ct **out) {
    FACADE_TRY
    need(h && a && out && num_iter >= 0, "bad argument");
    hellm_ct *r = new hellm_ct{a->t};
    HELLM::Exp::exp_iter(h->m->getEval(), h->m->getBtp(), a->t.get(), r->t.get(), num_iter);
    *out = r;
    FACADE_CATCH
}
int hellm_exp_iter_parallel(hellm_hemmer *h, hellm_ct **cts, uint32_t n, int num_iter) {
    FACADE_TRY
    need(h && cts && num_iter >= 0, "bad argument");
    std::vector<HELLM::CtxtTensor> op;
    op.reserve(n);
    for (uint32_t i = 0; i < n; i++) {
        need(cts[i] != nullptr, "null ciphertext");
        op.push_back(cts[i]->t);
    }
    HELLM::Exp::exp_iter_Parallel(h->m->getEval(), h->m->getBtp(), op, num_iter);
    for (uint32_t i = 0; i < n; i++) cts[i]->t = op[i];
    FACADE_CATCH
}
int hellm_eval_odd_polynomial(hellm_hemmer *h, const hellm_ct *a, const double *coeffs, uint32_t n_coeffs, int k, int l,
                              hellm_ct **out) {
    FACADE_TRY
    need(h && a && coeffs && out, "null argument");
    hellm_ct *r = new hellm_ct{a->t};
    HEaaN::Ciphertext x(a->t.get());
    HELLM::ReLU::evalOddPolynomial(h->m->getEval(), x, r->t.get(), std::vector<double>(coeffs, coeffs + n_coeffs), k, l);
    *out = r;
    FACADE_CATCH
}
int hellm_eval_chebyshev(hellm_hemmer *h, const hellm_ct *a, const double *coeffs, uint32_t n_coeffs, uint32_t baby_steps,
                         double multiplier, hellm_ct **out) {
    FACADE_TRY
    need(h && a && coeffs && out, "null argument");
    hellm_ct *r = new hellm_ct{a->t};
    r->t.get() = HEaaN::Math::evaluateChebyshevExpansion(
        h->m->getEval(), h->m->getBtp(), a->t.get(),
        HEaaN::Math::ChebyshevCoefficients(std::vector<HEaaN::Real>(coeffs, coeffs + n_coeffs), baby_steps), multiplier);
    *out = r;
    FACADE_CATCH
}

int hellm_linear_transform(hellm_hemmer *h, const hellm_ct *a, double left, double right, hellm_ct **out) {
    FACADE_TRY
    need(h && a && out, "null argument");
    hellm_ct *r = new hellm_ct{a->t};
    r->t.get() = HEaaN::Math::linearTransform(h->m->getEval(), h->m->getBtp(), a->t.get(),
                                              HEaaN::Math::InputInterval(left, right));
    *out = r;
    FACADE_CATCH
}

int hellm_transpose_inplace(hellm_hemmer *h, hellm_ct *a, uint32_t T) {
    FACADE_TRY
    need(h && a, "null argument");
    h->m->transposeInplace(a->t, T);
    FACADE_CATCH
}
int hellm_complex_packing_inplace(hellm_hemmer *h, hellm_ct *a) {
    FACADE_TRY
    need(h && a, "null argument");
    h->m->complexPackingInplace(a->t);
    FACADE_CATCH
}
int hellm_complex_packing_row_inplace(hellm_hemmer *h, hellm_ct *a) {
    FACADE_TRY
    need(h && a, "null argument");
    h->m->complexPackingRowInplace(a->t);
    FACADE_CATCH
}
int hellm_transpose_complex_packing_inplace(hellm_hemmer *h, hellm_ct *a, uint32_t T) {
    FACADE_TRY
    need(h && a, "null argument");
    h->m->transposeComplexPackingInplace(a->t, T);
    FACADE_CATCH
}
int hellm_split_in_two(hellm_hemmer *h, hellm_ct *a, hellm_ct **o1, hellm_ct **o2) {
    FACADE_TRY
    need(h && a && o1 && o2, "null argument");
    hellm_ct *r1 = new hellm_ct{a->t}, *r2 = new hellm_ct{a->t};
    h->m->splitInTwo(a->t, r1->t, r2->t);
    *o1 = r1;
    *o2 = r2;
    FACADE_CATCH
}

#define BINARY_MM(name, BT, call)                                                                   \
    int name(hellm_hemmer *h, const hellm_ct *a, const BT *b, uint32_t T, hellm_ct **out) {          \
        FACADE_TRY                                                                                   \
        need(h && a && b && out, "null argument");                                                   \
        *out = new hellm_ct{h->m->call(a->t, b->t, T)};                                              \
        FACADE_CATCH                                                                                 \
    }
BINARY_MM(hellm_single_cc_matmul, hellm_ct, singleCCMatMul)
BINARY_MM(hellm_single_matmul, hellm_pt, singleMatMul)
BINARY_MM(hellm_packed_matmul, hellm_ct, packedMatMul)

#define UNARY_MM(name, call)                                                      \
    int name(hellm_hemmer *h, const hellm_ct *a, uint32_t T, hellm_ct **out) {    \
        FACADE_TRY                                                                \
        need(h && a && out, "null argument");                                     \
        *out = new hellm_ct{h->m->call(a->t, T)};                                 \
        FACADE_CATCH                                                              \
    }
UNARY_MM(hellm_packed_matmul_pre, packedMatMulPre)
UNARY_MM(hellm_packed_matmul_pre_rev, packedMatMulPreRev)
UNARY_MM(hellm_matmul_pre_rev, matMulPreRev)

int hellm_packed_matmul_pre_rot(hellm_hemmer *h, const hellm_ct *a, uint32_t T, hellm_ctvec **out) {
    FACADE_TRY
    need(h && a && out, "null argument");
    hellm_ctvec *v = new hellm_ctvec();
    try {
        h->m->packedMatMulPreRot(a->t, v->v, T);
    } catch (...) {
        delete v;
        throw;
    }
    *out = v;
    FACADE_CATCH
}
int hellm_matmul_pre(hellm_hemmer *h, const hellm_ct *a, uint32_t T, hellm_ctvec **out) {
    FACADE_TRY
    need(h && a && out, "null argument");
    hellm_ctvec *v = new hellm_ctvec();
    try {
        h->m->matMulPre(a->t, v->v, T);
    } catch (...) {
        delete v;
        throw;
    }
    *out = v;
    FACADE_CATCH
}
int hellm_packed_matmul_cc_reuse(hellm_hemmer *h, const hellm_ctvec *tmp, const hellm_ct *b, uint32_t T,
                                 hellm_ct **out) {
    FACADE_TRY
    need(h && tmp && b && out, "null argument");
    *out = new hellm_ct{h->m->packedMatMulCCReuse(tmp->v, b->t, T)};
    FACADE_CATCH
}
int hellm_matmul_reuse(hellm_hemmer *h, const hellm_ctvec *tmp, const hellm_pt *b, uint32_t T, hellm_ct **out) {
    FACADE_TRY
    need(h && tmp && b && out, "null argument");
    *out = new hellm_ct{h->m->matMulReUse(tmp->v, b->t, T)};
    FACADE_CATCH
}
int hellm_matmul_cc_reuse(hellm_hemmer *h, const hellm_ctvec *tmp, const hellm_ct *b, uint32_t T, hellm_ct **out) {
    FACADE_TRY
    need(h && tmp && b && out, "null argument");
    *out = new hellm_ct{h->m->matMulCCReUse(tmp->v, b->t, T)};
    FACADE_CATCH
}
int hellm_repack_cc(hellm_hemmer *h, hellm_ct *a, hellm_ct **out) {
    FACADE_TRY
    need(h && a && out, "null argument");
    *out = new hellm_ct{h->m->repackCC(a->t)};
    FACADE_CATCH
}
int hellm_complex_packing(hellm_hemmer *h, const hellm_ct *a, const hellm_ct *b, hellm_ct **out) {
    FACADE_TRY
    need(h && a && b && out, "null argument");
    *out = new hellm_ct{h->m->complexPacking(a->t, b->t)};
    FACADE_CATCH
}
int hellm_complex_packing_rev(hellm_hemmer *h, const hellm_ct *a, const hellm_ct *b, hellm_ct **out) {
    FACADE_TRY
    need(h && a && b && out, "null argument");
    *out = new hellm_ct{h->m->complexPackingRev(a->t, b->t)};
    FACADE_CATCH
}
int hellm_complex_packing_pt(hellm_hemmer *h, const hellm_pt *a, const hellm_pt *b, hellm_pt **out) {
    FACADE_TRY
    need(h && a && b && out, "null argument");
    *out = new hellm_pt{h->m->complexPacking(a->t, b->t)};
    FACADE_CATCH
}
int hellm_repack_not_bts(hellm_hemmer *h, hellm_ct *a, hellm_ct *b, hellm_ct **out) {
    FACADE_TRY
    need(h && a && b && out, "null argument");
    *out = new hellm_ct{h->m->repack_notBTS(a->t, b->t)};
    FACADE_CATCH
}
int hellm_repack_lora_opti(hellm_hemmer *h, hellm_ct *a, hellm_ct *b, hellm_ct **out) {
    FACADE_TRY
    need(h && a && b && out, "null argument");
    *out = new hellm_ct{h->m->repack_loraOpti(a->t, b->t)};
    FACADE_CATCH
}
int hellm_matmul_high_low(hellm_hemmer *h, const hellm_ct *a, const hellm_ct *b, uint32_t in_col_block,
                          uint32_t target_level, hellm_ct **out) {
    FACADE_TRY
    need(h && a && b && out, "null argument");
    *out = new hellm_ct{h->m->matMulHighLow(a->t, b->t, in_col_block, target_level)};
    FACADE_CATCH
}
int hellm_matmul_low_high(hellm_hemmer *h, const hellm_ct *a, const hellm_ct *b, uint32_t in_row_block,
                          uint32_t target_level, hellm_ct **out) {
    FACADE_TRY
    need(h && a && b && out, "null argument");
    *out = new hellm_ct{h->m->matMulLowHigh(a->t, b->t, in_row_block, target_level)};
    FACADE_CATCH
}
int hellm_matmul_low_low(hellm_hemmer *h, const hellm_ct *a, const hellm_ct *b, uint32_t in_col_block,
                         uint32_t in_row_block, uint32_t target_level, hellm_ct **out) {
    FACADE_TRY
    need(h && a && b && out, "null argument");
    *out = new hellm_ct{h->m->matMulLowLow(a->t, b->t, in_col_block, in_row_block, target_level)};
    FACADE_CATCH
}
// which: 0 repackToOneCol, 1 repackToMultiCol, 2 repackToOneRow, 3 repackToMultiRow, 4 getLowColBlock, 5 getLowRowBlock
int hellm_low_rank_block(hellm_hemmer *h, const hellm_ct *a, uint32_t which, uint32_t block, hellm_ct **out) {
    FACADE_TRY
    need(h && a && out, "null argument");
    need(which < 6, "which must be 0..5");
    const HELLM::HEMMer &m = *h->m;
    *out = new hellm_ct{which == 0   ? m.repackToOneCol(a->t, block)
                        : which == 1 ? m.repackToMultiCol(a->t, block)
                        : which == 2 ? m.repackToOneRow(a->t, block)
                        : which == 3 ? m.repackToMultiRow(a->t, block)
                        : which == 4 ? m.getLowColBlock(a->t, block)
                                     : m.getLowRowBlock(a->t, block)};
    FACADE_CATCH
}
// up = 0: loraRank2Down(cts[0..count), weight) -> out[0..2); up = 1: loraRank2Up(cts[0..2), weight, n_out) -> out[0..n_out)
int hellm_lora_rank2(hellm_hemmer *h, int up, const hellm_ct *const *cts, uint32_t count, const hellm_ct *weight,
                     uint32_t n_out, uint32_t weight_level, hellm_ct **out) {
    FACADE_TRY
    need(h && cts && weight && out && count >= 1, "null argument");
    std::vector<HELLM::CtxtTensor> v;
    for (uint32_t i = 0; i < count; i++) {
        need(cts[i] != nullptr, "null ciphertext");
        v.push_back(cts[i]->t);
    }
    std::vector<HELLM::CtxtTensor> r =
        up ? h->m->loraRank2Up(v, weight->t, n_out, weight_level) : h->m->loraRank2Down(v, weight->t, weight_level);
    for (size_t i = 0; i < r.size(); i++) out[i] = new hellm_ct{r[i]};
    FACADE_CATCH
}

}  // extern "C"

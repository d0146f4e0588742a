// Implementation of the HEaaN-compatible host surface (host/HEaaN/HEaaN.hpp): object lifetime,
// level / scale bookkeeping, host-side encoding and sampling; every ring operation is a C-ABI call.
#include <algorithm>
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstring>
#include <fstream>
#include <mutex>

#include "../../../include/hemm.h"
#include "HEaaN/HEaaN.hpp"
#include "context_content.hpp"

namespace HEaaN {

namespace {

void ck(int rc) {
    if (rc == 0) return;
    std::string m = hemm_last_error();
    if (rc == 1) throw std::invalid_argument(m);
    throw RuntimeException(m);
}
void hip_ck(hipError_t e, const char *what) {
    if (e != hipSuccess) throw RuntimeException(std::string(what) + ": " + hipGetErrorString(e));
}

typedef unsigned __int128 u128;
u64 mulmod(u64 a, u64 b, u64 q) { return (u64)((u128)a * b % q); }
u64 powmod(u64 a, u64 e, u64 q) {
    u64 r = 1 % q;
    a %= q;
    while (e) {
        if (e & 1) r = mulmod(r, a, q);
        a = mulmod(a, a, q);
        e >>= 1;
    }
    return r;
}
u64 invmod(u64 a, u64 q) { return powmod(a % q, q - 2, q); }
bool is_prime(u64 n) {
    static const u64 bases[] = {2, 3, 5, 7, 11, 13, 17, 19, 23, 29, 31, 37};
    if (n < 2) return false;
    for (u64 p : bases)
        if (n % p == 0) return n == p;
    u64 d = n - 1;
    int s = 0;
    while (!(d & 1)) {
        d >>= 1;
        s++;
    }
    for (u64 a : bases) {
        u64 x = powmod(a, d, n);
        if (x == 1 || x == n - 1) continue;
        bool comp = true;
        for (int i = 1; i < s && comp; i++) {
            x = mulmod(x, x, n);
            if (x == n - 1) comp = false;
        }
        if (comp) return false;
    }
    return true;
}

// counter-based generator: splitmix64 finaliser over (stream key + counter * golden gamma)
u64 sm64(u64 x) {
    x += 0x9E3779B97F4A7C15ull;
    u64 z = x;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
u64 stream_key(u64 seed, u64 tag, u64 a, u64 b) { return sm64(sm64(sm64(seed + tag) + a) + b); }
u64 draw(u64 key, u64 ctr) { return sm64(key + ctr * 0x9E3779B97F4A7C15ull); }
enum { TAG_SK = 1, TAG_EVK_A = 2, TAG_EVK_E = 3, TAG_ENC_A = 4, TAG_ENC_E = 5 };

u64 g_seed = 0x5eed;
u64 g_enc_counter = 0;

}  // namespace

void setSeed(u64 seed) {
    g_seed = seed;
    g_enc_counter = 0;
}

Device getDefaultDevice() { return Device{DeviceType::CPU, 0}; }
Device getCurrentCudaDevice() {
    int d = 0;
    (void)hipGetDevice(&d);
    return Device{DeviceType::GPU, d};
}
void setCurrentCudaDevice(int id) { hip_ck(hipSetDevice(id), "hipSetDevice"); }
void CudaTools::cudaDeviceSynchronize() { hip_ck(hipDeviceSynchronize(), "hipDeviceSynchronize"); }
void CudaTools::cudaSetDevice(int id) { hip_ck(hipSetDevice(id), "hipSetDevice"); }

Context makeContextCustom(u64 log_degree, const std::vector<u64> &chain, const std::vector<u64> &special, u64 dnum,
                          u64 log_scale) {
    auto c = std::make_shared<ContextContent>();
    std::vector<u64> all(chain);
    all.insert(all.end(), special.begin(), special.end());
    ck(hemm_context_create((uint32_t)log_degree, (uint32_t)chain.size(), (uint32_t)special.size(), all.data(),
                           (uint32_t)dnum, &c->dev));
    c->logN = log_degree;
    c->N = u64(1) << log_degree;
    c->nQ = chain.size();
    c->nP = special.size();
    c->dnum = dnum;
    c->alpha = (c->nQ + dnum - 1) / dnum;
    c->log_scale = log_scale;
    c->q = chain;
    c->p = special;
    c->delta.assign(c->nQ, 0.0);
    c->delta[c->nQ - 1] = std::ldexp(1.0, (int)log_scale);
    for (size_t l = c->nQ - 1; l >= 1; l--) c->delta[l - 1] = c->delta[l] * c->delta[l] / (double)c->q[l];
    const u64 n = c->N / 2, M = 2 * c->N;
    c->rot_group.resize(n);
    u64 g = 1;
    for (u64 j = 0; j < n; j++) {
        c->rot_group[j] = g;
        g = g * 5 % M;
    }
    c->ksi_re.resize(M + 1);
    c->ksi_im.resize(M + 1);
    // separate loops: a cos / sin pair on one value may be merged into one sincos call, which rounds differently
    for (u64 k = 0; k <= M; k++) c->ksi_re[k] = cos(2.0 * M_PI * (double)k / (double)M);
    for (u64 k = 0; k <= M; k++) c->ksi_im[k] = sin(2.0 * M_PI * (double)k / (double)M);
    return c;
}

static u64 nearest_prime(double target, u64 log_degree, const std::vector<u64> &skip) {
    const u64 m = u64(2) << log_degree;
    const u64 t = (u64)target;
    const u64 base = t - (t % m) + 1;
    auto used = [&](u64 x) {
        for (u64 s : skip)
            if (s == x) return true;
        return false;
    };
    for (u64 k = 0;; k++) {
        u64 lo = base - k * m, hi = base + (k + 1) * m;
        double dlo = std::fabs((double)lo - target), dhi = std::fabs((double)hi - target);
        u64 first = (dlo < dhi || (dlo == dhi && lo < hi)) ? lo : hi, second = (first == lo) ? hi : lo;
        if (k == 0) {
            // candidates base and base + m
            if (!used(first) && is_prime(first)) return first;
            if (!used(second) && is_prime(second)) return second;
        } else {
            if (!used(first) && is_prime(first)) return first;
            if (!used(second) && is_prime(second)) return second;
        }
    }
}

Context makeContextGenerated(u64 log_degree, u64 n_chain, u64 n_special, u64 dnum, u64 base_bits, u64 scale_bits,
                             u64 special_bits) {
    std::vector<u64> q(n_chain), p(n_special), used;
    ck(hemm_primes_below((uint32_t)base_bits, (uint32_t)log_degree, 1, &q[0]));
    used.push_back(q[0]);
    double delta = std::ldexp(1.0, (int)scale_bits);
    const double s = delta;
    for (size_t l = n_chain - 1; l >= 1; l--) {
        double target = delta * delta / s;
        q[l] = nearest_prime(target, log_degree, used);
        used.push_back(q[l]);
        delta = delta * delta / (double)q[l];
    }
    // special primes: largest below 2^special_bits not already used
    std::vector<u64> cand(n_special + n_chain + 1);
    ck(hemm_primes_below((uint32_t)special_bits, (uint32_t)log_degree, (uint32_t)cand.size(), cand.data()));
    size_t k = 0;
    for (u64 c : cand) {
        bool u = false;
        for (u64 x : used) u |= (x == c);
        if (!u && k < n_special) p[k++] = c;
    }
    return makeContextCustom(log_degree, q, p, dnum, scale_bits);
}

Context makeContext(ParameterPreset preset, const std::vector<int> &device_ids) {
    if (!device_ids.empty()) setCurrentCudaDevice(device_ids[0]);
    if (preset != ParameterPreset::FGb) throw RuntimeException("only the FGb-sized preset is built in");
    return makeContextGenerated(16, 13, 4, 3, 60, 42, 60);
}

u64 getLogFullSlots(const Context &c) { return c->logN - 1; }
u64 getDegree(const Context &c) { return c->N; }
u64 getEncryptionLevel(const Context &c) { return c->nQ - 1; }
std::vector<u64> getPrimeList(const Context &c) {
    std::vector<u64> r(c->q);
    r.insert(r.end(), c->p.begin(), c->p.end());
    return r;
}
std::vector<Real> getDefaultScaleFactorList(const Context &c) { return c->delta; }
hemm_context *getDeviceContext(const Context &c) { return c->dev; }

// ---- device buffer -----------------------------------------------------------------------------
DeviceBuffer::DeviceBuffer(const Context &c, size_t words) { resize(c, words); }
DeviceBuffer::DeviceBuffer(const DeviceBuffer &o) { *this = o; }
DeviceBuffer::DeviceBuffer(DeviceBuffer &&o) noexcept { *this = std::move(o); }
DeviceBuffer &DeviceBuffer::operator=(const DeviceBuffer &o) {
    if (this == &o) return *this;
    if (o.ptr_ == nullptr) {
        release();
        return *this;
    }
    resize(o.ctx_, o.words_);
    hip_ck(hipMemcpyAsync(ptr_, o.ptr_, words_ * 8, hipMemcpyDeviceToDevice, ctx_->stream()), "hipMemcpyAsync");
    return *this;
}
DeviceBuffer &DeviceBuffer::operator=(DeviceBuffer &&o) noexcept {
    if (this == &o) return *this;
    release();
    ctx_ = std::move(o.ctx_);
    ptr_ = o.ptr_;
    words_ = o.words_;
    cap_ = o.cap_;
    o.ptr_ = nullptr;
    o.words_ = o.cap_ = 0;
    return *this;
}
DeviceBuffer::~DeviceBuffer() { release(); }
void DeviceBuffer::release() {
    if (ptr_ && ctx_) ctx_->release(ptr_, cap_);
    ptr_ = nullptr;
    words_ = cap_ = 0;
    ctx_.reset();
}
void DeviceBuffer::resize(const Context &c, size_t words) {
    if (ptr_ && cap_ == words && ctx_ == c) {
        words_ = words;
        return;
    }
    release();
    ctx_ = c;
    ptr_ = c->alloc(words);
    words_ = cap_ = words;
}

// ---- value types -------------------------------------------------------------------------------
void Message::save(const std::string &path) const {
    std::ofstream f(path, std::ios::binary);
    if (!f) throw RuntimeException("cannot open " + path);
    f.write((const char *)&log_slots_, 8);
    f.write((const char *)v_.data(), (std::streamsize)(v_.size() * sizeof(Complex)));
}
void Message::load(const std::string &path) {
    std::ifstream f(path, std::ios::binary);
    if (!f) throw RuntimeException("cannot open " + path);
    f.read((char *)&log_slots_, 8);
    if (log_slots_ > 20) throw RuntimeException("bad message file " + path);
    v_.resize(size_t(1) << log_slots_);
    f.read((char *)v_.data(), (std::streamsize)(v_.size() * sizeof(Complex)));
}

void Plaintext::allocate(u64 level, u64 rc) {
    level_ = level;
    rescale_counter_ = rc;
    occupied_ = ~u64(0);
    log_slots_ = ctx_->logN - 1;
    buf_.resize(ctx_, (level + 1) * ctx_->N);
    compact_shift_ = 0;
    compact_ = DeviceBuffer();
    if (hash_state_ == 1) hash_state_ = 0;
}
bool Plaintext::makeCompact() {
    if (compact_shift_ != 0) return true;
    const u64 N = ctx_->N, limbs = buf_.words() / N;
    if (limbs != level_ + 1 + ctx_->nP || ctx_->logN < 10) return false;   // masks over the extended basis only
    // slot patterns of period 2^6 .. 2^8 give runs of 2^(logN-7) .. 2^(logN-9) residues: longest runs first
    for (u32 shift = (u32)ctx_->logN - 7; shift >= (u32)ctx_->logN - 9; shift--) {
        DeviceBuffer t(ctx_, 2 * limbs * (N >> shift));   // (value, Shoup companion) per run
        int ok = 0;
        ck(hemm_compact_mask(ctx_->dev, buf_.data(), (uint32_t)limbs, shift, t.data(), &ok, nullptr));
        if (ok) {
            compact_ = std::move(t);
            compact_shift_ = shift;
            return true;
        }
    }
    return false;
}
void Plaintext::setLevel(u64 level) {
    if (level > level_) throw RuntimeException("Plaintext::setLevel can only lower the level");
    if (level == level_) return;
    compact_shift_ = 0;
    compact_ = DeviceBuffer();
    if (hash_state_ == 1) hash_state_ = 0;
    DeviceBuffer nb(ctx_, (level + 1) * ctx_->N);
    hip_ck(hipMemcpyAsync(nb.data(), buf_.data(), (level + 1) * ctx_->N * 8, hipMemcpyDeviceToDevice, ctx_->stream()),
           "hipMemcpyAsync");
    buf_ = std::move(nb);
    level_ = level;
}

void Ciphertext::allocate(u64 num_poly, u64 level, u64 rc) {
    num_poly_ = num_poly;
    level_ = level;
    rescale_counter_ = rc;
    log_slots_ = ctx_->logN - 1;
    occupied_ = ~u64(0);
    buf_.resize(ctx_, num_poly * (level + 1) * ctx_->N);
}
size_t Ciphertext::polyStride() const { return (size_t)(level_ + 1) * ctx_->N; }
u64 *Ciphertext::getPolyData(u64 i, u64 level) const {
    if (i >= num_poly_) throw RuntimeException("polynomial index out of range");
    occupied_ = ~u64(0);   // the caller may write through the pointer
    return buf_.data() + i * polyStride() + level * ctx_->N;
}
void Ciphertext::save(const std::string &path) const {
    std::ofstream f(path, std::ios::binary);
    if (!f) throw RuntimeException("cannot open " + path);
    u64 hdr[4] = {num_poly_, level_, rescale_counter_, ctx_->N};
    f.write((const char *)hdr, sizeof(hdr));
    std::vector<u64> h(buf_.words());
    hip_ck(hipMemcpy(h.data(), buf_.data(), h.size() * 8, hipMemcpyDeviceToHost), "hipMemcpy");
    f.write((const char *)h.data(), (std::streamsize)(h.size() * 8));
}
void Ciphertext::load(const std::string &path) {
    std::ifstream f(path, std::ios::binary);
    if (!f) throw RuntimeException("cannot open " + path);
    u64 hdr[4];
    f.read((char *)hdr, sizeof(hdr));
    if (hdr[3] != ctx_->N || hdr[1] >= ctx_->nQ || hdr[0] < 1 || hdr[0] > 3)
        throw RuntimeException("ciphertext file does not match the context: " + path);
    allocate(hdr[0], hdr[1], hdr[2]);
    std::vector<u64> h(buf_.words());
    f.read((char *)h.data(), (std::streamsize)(h.size() * 8));
    hip_ck(hipMemcpy(buf_.data(), h.data(), h.size() * 8, hipMemcpyHostToDevice), "hipMemcpy");
}

// ---- small helpers over the C ABI ---------------------------------------------------------------
namespace {

// signed coefficient vector -> residues for primes [first, first+count) of the context, uploaded
// and transformed to NTT form in `dst` ([count][N]).
void lift_and_ntt(const Context &c, const std::vector<i64> &coeffs, const std::vector<uint32_t> &primes, u64 *dst) {
    const size_t N = c->N;
    std::vector<u64> h(primes.size() * N);
    for (size_t j = 0; j < primes.size(); j++) {
        const u64 q = c->prime(primes[j]);
        u64 *o = h.data() + j * N;
        for (size_t i = 0; i < N; i++) {
            i64 v = coeffs[i];
            if (v >= 0)
                o[i] = (u64)v % q;
            else {
                u64 r = (u64)(-v) % q;
                o[i] = r ? q - r : 0;
            }
        }
    }
    hip_ck(hipMemcpy(dst, h.data(), h.size() * 8, hipMemcpyHostToDevice), "hipMemcpy");
    ck(hemm_ntt(c->dev, dst, primes.data(), (uint32_t)primes.size(), 1, 0, nullptr));
}

std::vector<uint32_t> all_primes(const Context &c) {
    std::vector<uint32_t> r(c->nQ + c->nP);
    for (size_t i = 0; i < r.size(); i++) r[i] = (uint32_t)i;
    return r;
}
std::vector<uint32_t> chain_primes(u64 count) {
    std::vector<uint32_t> r(count);
    for (size_t i = 0; i < count; i++) r[i] = (uint32_t)i;
    return r;
}

u64 galois_of_rotation(const Context &c, u64 rot) { return powmod(5, rot % (c->N / 2), 2 * c->N); }

}  // namespace

// ---- keys ----------------------------------------------------------------------------------------
SecretKey::SecretKey(const Context &c) : ctx_(c), coeffs_(c->N, 0) {
    const u64 key = stream_key(g_seed, TAG_SK, 0, 0);
    const int hw = (int)std::min<u64>(192, c->N / 2);
    int placed = 0;
    for (u64 ctr = 0; placed < hw; ctr++) {
        u64 x = draw(key, ctr);
        size_t pos = (size_t)(x & (c->N - 1));
        if (coeffs_[pos]) continue;
        coeffs_[pos] = (x >> 63) ? -1 : 1;
        placed++;
    }
    upload();
}
SecretKey::SecretKey(const Context &c, const int *coefficients) : ctx_(c), coeffs_(coefficients, coefficients + c->N) {
    upload();
}
SecretKey::SecretKey(const Context &c, const std::string &path) : ctx_(c), coeffs_(c->N, 0) {
    std::ifstream f(path, std::ios::binary);
    if (!f) throw RuntimeException("cannot open " + path);
    u64 n = 0;
    f.read((char *)&n, 8);
    if (n != c->N) throw RuntimeException("secret key file does not match the context");
    f.read((char *)coeffs_.data(), (std::streamsize)(n * sizeof(int)));
    upload();
}
void SecretKey::save(const std::string &path) const {
    std::ofstream f(path, std::ios::binary);
    if (!f) throw RuntimeException("cannot open " + path);
    u64 n = coeffs_.size();
    f.write((const char *)&n, 8);
    f.write((const char *)coeffs_.data(), (std::streamsize)(n * sizeof(int)));
}
void SecretKey::upload() {
    const size_t T = ctx_->nQ + ctx_->nP;
    ntt_.resize(ctx_, T * ctx_->N);
    std::vector<i64> v(coeffs_.begin(), coeffs_.end());
    lift_and_ntt(ctx_, v, all_primes(ctx_), ntt_.data());
}

const u64 *KeyPack::multKey() const {
    if (!hasMultKey()) throw RuntimeException("multiplication key has not been generated");
    return mult_.data();
}
const u64 *KeyPack::plainOrRebuilt(int kind, u64 g) const {
    auto &plain = kind == 1 ? galois_ : galois_sq_;
    auto it = plain.find(g);
    if (it != plain.end()) return it->second.data();
    auto ct = compact_.find({kind, g});
    if (ct == compact_.end())
        throw RuntimeException(std::string(kind == 1 ? "no key" : "no square key") + " for Galois element " + std::to_string(g));
    // rebuilt plain forms are few at a time: a chain of single rotations uses a handful of steps over and over
    const size_t keep = 4;
    while (rebuilt_.size() >= keep) {
        (rebuilt_.front().first == 1 ? galois_ : galois_sq_).erase(rebuilt_.front().second);
        rebuilt_.erase(rebuilt_.begin());
    }
    DeviceBuffer b(ctx_, ctx_->dnum * 2 * (ctx_->nQ + ctx_->nP) * ctx_->N);
    ck(hemm_key_expand(ctx_->dev, ct->second.data(), b.data(), nullptr));
    rebuilt_.emplace_back(kind, g);
    return plain.emplace(g, std::move(b)).first->second.data();
}
const u64 *KeyPack::galoisKey(u64 g) const { return plainOrRebuilt(1, g); }
const u64 *KeyPack::galoisSquareKey(u64 g) const { return plainOrRebuilt(2, g); }
const u64 *KeyPack::compactKey(int kind, u64 g) const {
    const auto id = std::make_pair(kind, kind == 0 ? u64(0) : g);
    auto it = compact_.find(id);
    if (it == compact_.end()) {
        const u64 *plain = kind == 0 ? multKey() : kind == 1 ? galoisKey(g) : galoisSquareKey(g);
        DeviceBuffer c(ctx_, hemm_key_compact_words(ctx_->dev));
        ck(hemm_key_compact(ctx_->dev, plain, c.data(), nullptr));
        // made once per key, on the context's stream: finished before the caller queues its sum on whichever stream (the
        // side stream does not wait for later work of that one)
        hip_ck(hipStreamSynchronize(ctx_->stream()), "hipStreamSynchronize");
        it = compact_.emplace(id, std::move(c)).first;
        if (kind != 0) {   // the plain form goes back to the pool (the next key generated takes its place)
            (kind == 1 ? galois_ : galois_sq_).erase(g);
            for (size_t i = 0; i < rebuilt_.size(); i++)
                if (rebuilt_[i] == std::make_pair(kind, g)) {
                    rebuilt_.erase(rebuilt_.begin() + (long)i);
                    break;
                }
        }
    }
    return it->second.data();
}
bool KeyPack::compactible() const { return ctx_->dnum <= 6 && ctx_->N >= 512; }
std::pair<u64, u64> KeyPack::keyBytes() const {
    u64 plain = mult_.words() * 8, compact = 0;
    for (auto &kv : galois_) plain += kv.second.words() * 8;
    for (auto &kv : galois_sq_) plain += kv.second.words() * 8;
    for (auto &kv : compact_) compact += kv.second.words() * 8;
    return {plain, compact};
}
void KeyPack::save(const std::string &dir) const {
    const size_t words = ctx_->dnum * 2 * (ctx_->nQ + ctx_->nP) * ctx_->N;
    std::vector<u64> h(words);
    auto dump = [&](const std::string &name, const DeviceBuffer &b) {
        hip_ck(hipMemcpy(h.data(), b.data(), words * 8, hipMemcpyDeviceToHost), "hipMemcpy");
        std::ofstream f(dir + "/" + name, std::ios::binary);
        if (!f) throw RuntimeException("cannot open " + dir + "/" + name);
        f.write((const char *)h.data(), (std::streamsize)(words * 8));
    };
    std::ofstream idx(dir + "/KeyPack.idx");
    if (hasMultKey()) {
        dump("MultKey.bin", mult_);
        idx << "mult\n";
    }
    // every key, whichever form it is held in (a plain form that was given up is rebuilt for the dump)
    std::vector<u64> gal, sq;
    for (auto &kv : galois_) gal.push_back(kv.first);
    for (auto &kv : galois_sq_) sq.push_back(kv.first);
    for (auto &kv : compact_) {
        if (kv.first.first == 1 && !galois_.count(kv.first.second)) gal.push_back(kv.first.second);
        if (kv.first.first == 2 && !galois_sq_.count(kv.first.second)) sq.push_back(kv.first.second);
    }
    std::sort(gal.begin(), gal.end());
    std::sort(sq.begin(), sq.end());
    auto dump_ptr = [&](const std::string &name, const u64 *src) {
        hip_ck(hipMemcpy(h.data(), src, words * 8, hipMemcpyDeviceToHost), "hipMemcpy");
        std::ofstream f(dir + "/" + name, std::ios::binary);
        if (!f) throw RuntimeException("cannot open " + dir + "/" + name);
        f.write((const char *)h.data(), (std::streamsize)(words * 8));
    };
    for (u64 g : gal) {
        dump_ptr("GaloisKey_" + std::to_string(g) + ".bin", galoisKey(g));
        idx << g << "\n";
    }
    for (u64 g : sq) {
        dump_ptr("GaloisSquareKey_" + std::to_string(g) + ".bin", galoisSquareKey(g));
        idx << "sq" << g << "\n";
    }
}
KeyPack::KeyPack(const Context &c, const std::string &dir) : ctx_(c) {
    const size_t words = c->dnum * 2 * (c->nQ + c->nP) * c->N;
    std::vector<u64> h(words);
    std::ifstream idx(dir + "/KeyPack.idx");
    if (!idx) throw RuntimeException("cannot open " + dir + "/KeyPack.idx");
    std::string line;
    auto slurp = [&](const std::string &name, DeviceBuffer &b) {
        std::ifstream f(dir + "/" + name, std::ios::binary);
        if (!f) throw RuntimeException("cannot open " + dir + "/" + name);
        f.read((char *)h.data(), (std::streamsize)(words * 8));
        b.resize(c, words);
        hip_ck(hipMemcpy(b.data(), h.data(), words * 8, hipMemcpyHostToDevice), "hipMemcpy");
    };
    while (std::getline(idx, line)) {
        if (line == "mult")
            slurp("MultKey.bin", mult_);
        else if (line.rfind("sq", 0) == 0) {
            u64 g = std::stoull(line.substr(2));
            slurp("GaloisSquareKey_" + line.substr(2) + ".bin", galois_sq_[g]);
        } else if (!line.empty()) {
            u64 g = std::stoull(line);
            slurp("GaloisKey_" + line + ".bin", galois_[g]);
        }
    }
}

// evk[d] = (b_d, a_d) over all nQ+nP primes, NTT form:
//   a_d uniform, b_d = -a_d*s + e_d (+ [P mod q_i] * s_from on the limbs of digit d)
void KeyGenerator::genSwitchKey(u64 key_id, const u64 *s_from, DeviceBuffer &out) const {
    const Context &c = ctx_;
    const size_t N = c->N, T = c->nQ + c->nP;
    out.resize(c, c->dnum * 2 * T * N);
    DeviceBuffer e(c, T * N), tmp(c, T * N);
    const auto primes = all_primes(c);
    std::vector<u64> keys(T);
    for (u64 d = 0; d < c->dnum; d++) {
        u64 *b = out.data() + (d * 2 + 0) * T * N, *a = out.data() + (d * 2 + 1) * T * N;
        // error and uniform part are sampled on the device (same counter-based streams as the host samplers)
        ck(hemm_sample_error(c->dev, stream_key(g_seed, TAG_EVK_E, key_id, d), primes.data(), (uint32_t)T, e.data(), nullptr));
        ck(hemm_ntt(c->dev, e.data(), primes.data(), (uint32_t)T, 1, 0, nullptr));
        for (size_t i = 0; i < T; i++) keys[i] = stream_key(g_seed, TAG_EVK_A, key_id, d * T + i);
        ck(hemm_sample_uniform(c->dev, keys.data(), primes.data(), (uint32_t)T, a, nullptr));
        // tmp = a*s ; b = e - tmp     (all T limbs: chain then special, i.e. nq = nQ with_p = 1)
        ck(hemm_pointwise(c->dev, HEMM_MUL, a, 0, sk_.ntt(), 0, tmp.data(), 0, (uint32_t)c->nQ, 1, 1, nullptr));
        ck(hemm_pointwise(c->dev, HEMM_SUB, e.data(), 0, tmp.data(), 0, b, 0, (uint32_t)c->nQ, 1, 1, nullptr));
        // b += [P mod q_i] * s_from on the digit's limbs
        const size_t lo = d * c->alpha, hi = std::min<size_t>(c->nQ, lo + c->alpha);
        if (lo < hi) {
            std::vector<u64> sc(c->nQ, 0);
            for (size_t i = lo; i < hi; i++) {
                u64 P = 1;
                for (u64 p : c->p) P = mulmod(P, p % c->q[i], c->q[i]);
                sc[i] = P;
            }
            ck(hemm_mul_scalar(c->dev, s_from, 0, sc.data(), tmp.data(), 0, (uint32_t)c->nQ, 0, 1, nullptr));
            ck(hemm_pointwise(c->dev, HEMM_ADD, b, 0, tmp.data(), 0, b, 0, (uint32_t)c->nQ, 0, 1, nullptr));
        }
    }
}
void KeyGenerator::genMultKey() const {
    const size_t T = ctx_->nQ + ctx_->nP;
    DeviceBuffer s2(ctx_, T * ctx_->N);
    ck(hemm_pointwise(ctx_->dev, HEMM_MUL, sk_.ntt(), 0, sk_.ntt(), 0, s2.data(), 0, (uint32_t)ctx_->nQ, 1, 1, nullptr));
    genSwitchKey(0, s2.data(), pack_.mult_);
    pack_.compact_.erase(std::make_pair(0, u64(0)));   // a compact form of an earlier multiplication key is stale
}
static void gen_galois(const KeyGenerator &, const Context &c, const SecretKey &sk, u64 g, DeviceBuffer &sg) {
    const size_t T = c->nQ + c->nP;
    sg.resize(c, T * c->N);
    ck(hemm_automorphism(c->dev, sk.ntt(), 0, sg.data(), 0, g, (uint32_t)T, 1, nullptr));
}
void KeyGenerator::genConjKey() const {
    const u64 g = 2 * ctx_->N - 1;
    if (pack_.hasGaloisKey(g)) return;
    DeviceBuffer sg;
    gen_galois(*this, ctx_, sk_, g, sg);
    genSwitchKey(g, sg.data(), pack_.galois_[g]);
}
void KeyGenerator::genLeftRotKey(u64 rot) const {
    const u64 slots = ctx_->N / 2;
    rot %= slots;
    if (rot == 0) return;
    const u64 g = galois_of_rotation(ctx_, rot);
    if (pack_.hasGaloisKey(g)) return;
    DeviceBuffer sg;
    gen_galois(*this, ctx_, sk_, g, sg);
    genSwitchKey(g, sg.data(), pack_.galois_[g]);
    if (pack_.compact_on_generate_ && pack_.compactible()) (void)pack_.compactKey(1, g);
}
void KeyGenerator::genGaloisKey(u64 g) const {
    if (g % 2 == 0 || g >= 2 * ctx_->N) throw RuntimeException("a Galois element is odd and below 2N");
    if (g == 1 || pack_.hasGaloisKey(g)) return;
    DeviceBuffer sg;
    gen_galois(*this, ctx_, sk_, g, sg);
    genSwitchKey(g, sg.data(), pack_.galois_[g]);
    if (pack_.compact_on_generate_ && pack_.compactible()) (void)pack_.compactKey(1, g);
}
void KeyGenerator::genLeftRotSquareKey(u64 rot) const {
    const u64 slots = ctx_->N / 2;
    rot %= slots;
    genGaloisSquareKey(rot == 0 ? 1 : galois_of_rotation(ctx_, rot));
}
// key id of a square key: the Galois element with bit 40 set (Galois elements are below 2N <= 2^18)
void KeyGenerator::genGaloisSquareKey(u64 g) const {
    if (g % 2 == 0 || g >= 2 * ctx_->N) throw RuntimeException("a Galois element is odd and below 2N");
    if (pack_.hasGaloisSquareKey(g)) return;
    const size_t T = ctx_->nQ + ctx_->nP;
    DeviceBuffer s2(ctx_, T * ctx_->N), sg(ctx_, T * ctx_->N);
    ck(hemm_pointwise(ctx_->dev, HEMM_MUL, sk_.ntt(), 0, sk_.ntt(), 0, s2.data(), 0, (uint32_t)ctx_->nQ, 1, 1, nullptr));
    ck(hemm_automorphism(ctx_->dev, s2.data(), 0, sg.data(), 0, g, (uint32_t)T, 1, nullptr));
    genSwitchKey((u64(1) << 40) | g, sg.data(), pack_.galois_sq_[g]);
    if (pack_.compact_on_generate_ && pack_.compactible()) (void)pack_.compactKey(2, g);
}
void KeyGenerator::genRightRotKey(u64 rot) const {
    const u64 slots = ctx_->N / 2;
    genLeftRotKey((slots - rot % slots) % slots);
}
void KeyGenerator::genRotKeyBundle() const {
    for (u64 r = 1; r < ctx_->N / 2; r <<= 1) {
        genLeftRotKey(r);
        genRightRotKey(r);
    }
}
void KeyGenerator::genCommonKeys() const {
    genMultKey();
    genConjKey();
    genRotKeyBundle();
}

// ---- encode / decode -------------------------------------------------------------------------------
namespace {
void bitrev_perm(std::vector<double> &re, std::vector<double> &im) {
    const size_t n = re.size();
    for (size_t i = 1, j = 0; i < n; i++) {
        size_t bit = n >> 1;
        for (; j >= bit; bit >>= 1) j -= bit;
        j += bit;
        if (i < j) {
            std::swap(re[i], re[j]);
            std::swap(im[i], im[j]);
        }
    }
}
}  // namespace

static Plaintext encode_impl(const Context &c, const Message &msg, u64 level, u64 rescale_counter, bool extended,
                             double scale_override = 0) {
    if (level >= c->nQ) throw RuntimeException("encode: level above the encryption level");
    if (rescale_counter != 0) throw RuntimeException("encode: only rescale counter 0 is supported");
    const size_t n = c->N / 2, M = 2 * c->N;
    if (msg.getSize() != n) throw RuntimeException("encode: message must fill all N/2 slots");
    if (c->N >= 512) {
        // on the device: the same butterflies in the same order (one IEEE operation per step), so the same residues
        // as the host loop below
        static_assert(sizeof(Complex) == 16, "a message is an array of (re, im) doubles");
        const double scale = scale_override != 0 ? scale_override : c->delta[level];
        Plaintext pt(c);
        pt.allocate(level, 0);
        const size_t limbs = level + 1 + (extended ? c->nP : 0);
        if (extended) pt.buf_.resize(c, limbs * c->N);
        DeviceBuffer z(c, c->N);
        hip_ck(hipMemcpy(z.data(), &msg[0], n * sizeof(Complex), hipMemcpyHostToDevice), "hipMemcpy");
        ck(hemm_encode(c->dev, (double *)z.data(), scale, (uint32_t)level + 1, extended ? 1 : 0, 1, pt.buf_.data(), nullptr));
        size_t occupied = n;
        while (occupied > 0 && msg[occupied - 1] == Complex(0, 0)) occupied--;
        pt.occupied_ = occupied;
        if (scale_override != 0) pt.scale_ = scale_override;
        return pt;
    }
    std::vector<double> re(n), im(n);
    for (size_t i = 0; i < n; i++) {
        re[i] = msg[i].real();
        im[i] = msg[i].imag();
    }
    // inverse of the canonical embedding on the orbit zeta^{5^j}
    for (size_t len = n; len >= 2; len >>= 1) {
        const size_t lenh = len >> 1, lenq = len << 2, gap = M / lenq;
        for (size_t i = 0; i < n; i += len)
            for (size_t j = 0; j < lenh; j++) {
                const size_t idx = (lenq - (c->rot_group[j] % lenq)) * gap;
                const double ur = re[i + j] + re[i + j + lenh], ui = im[i + j] + im[i + j + lenh];
                const double vr = re[i + j] - re[i + j + lenh], vi = im[i + j] - im[i + j + lenh];
                const double kr = c->ksi_re[idx], ki = c->ksi_im[idx];
                re[i + j] = ur;
                im[i + j] = ui;
                re[i + j + lenh] = vr * kr - vi * ki;
                im[i + j + lenh] = vr * ki + vi * kr;
            }
    }
    bitrev_perm(re, im);
    const double scale = scale_override != 0 ? scale_override : c->delta[level];
    std::vector<i64> coeffs(c->N);
    for (size_t i = 0; i < n; i++) {
        coeffs[i] = (i64)llround(re[i] / (double)n * scale);
        coeffs[i + n] = (i64)llround(im[i] / (double)n * scale);
    }
    Plaintext pt(c);
    pt.allocate(level, 0);
    std::vector<uint32_t> primes = chain_primes(level + 1);
    if (extended) {
        for (u64 k = 0; k < c->nP; k++) primes.push_back((uint32_t)(c->nQ + k));
        pt.buf_.resize(c, primes.size() * c->N);
    }
    lift_and_ntt(c, coeffs, primes, pt.buf_.data());
    size_t occupied = n;
    while (occupied > 0 && msg[occupied - 1] == Complex(0, 0)) occupied--;
    pt.occupied_ = occupied;
    if (scale_override != 0) pt.scale_ = scale_override;
    return pt;
}
Plaintext EnDecoder::encode(const Message &msg, u64 level, u64 rescale_counter) const {
    return encode_impl(ctx_, msg, level, rescale_counter, false);
}
Plaintext EnDecoder::encodeExtended(const Message &msg, u64 level) const {
    return encode_impl(ctx_, msg, level, 0, true);
}
Plaintext EnDecoder::encodeExtended(const Message &msg, u64 level, Real scale) const {
    return encode_impl(ctx_, msg, level, 0, true, (double)scale);
}
Plaintext EnDecoder::encode(const Message &msg) const { return encode(msg, getEncryptionLevel(ctx_)); }

Message EnDecoder::decode(const Plaintext &pt) const {
    const Context &c = ctx_;
    const size_t N = c->N, n = N / 2, M = 2 * N;
    const u64 two = pt.level_ >= 1 ? 1 : 0;
    if (N >= 512) {
        double scale = pt.scale_;
        if (scale == 0) {
            scale = c->delta[pt.level_];
            for (u64 k = 0; k < pt.rescale_counter_; k++) scale *= c->delta[pt.level_];
        }
        DeviceBuffer work(c, (two + 1) * N), z(c, N);
        ck(hemm_decode(c->dev, pt.buf_.data(), (uint32_t)(two + 1), scale, work.data(), (double *)z.data(), nullptr));
        Message m(c->logN - 1);
        hip_ck(hipMemcpy(&m[0], z.data(), n * sizeof(Complex), hipMemcpyDeviceToHost), "hipMemcpy");
        return m;
    }
    DeviceBuffer tmp(c, (two + 1) * N);
    hip_ck(hipMemcpyAsync(tmp.data(), pt.buf_.data(), (two + 1) * N * 8, hipMemcpyDeviceToDevice, c->stream()), "memcpy");
    ck(hemm_ntt(c->dev, tmp.data(), chain_primes(two + 1).data(), (uint32_t)(two + 1), 1, 1, nullptr));
    std::vector<u64> h((two + 1) * N);
    hip_ck(hipMemcpy(h.data(), tmp.data(), h.size() * 8, hipMemcpyDeviceToHost), "hipMemcpy");
    double scale = pt.scale_;
    if (scale == 0) {
        scale = c->delta[pt.level_];
        for (u64 k = 0; k < pt.rescale_counter_; k++) scale *= c->delta[pt.level_];
    }
    std::vector<double> co(N);
    const u64 q0 = c->q[0];
    if (!two) {
        for (size_t i = 0; i < N; i++) {
            u64 v = h[i];
            co[i] = (v > q0 / 2 ? -(double)(q0 - v) : (double)v) / scale;
        }
    } else {
        const u64 q1 = c->q[1], q0inv = invmod(q0 % q1, q1);
        const u128 Q = (u128)q0 * q1;
        for (size_t i = 0; i < N; i++) {
            const u64 l0 = h[i], l1 = h[N + i];
            const u64 a = l1 % q1, b = l0 % q1;
            const u64 d = a >= b ? a - b : a + q1 - b;
            const u64 k = mulmod(d, q0inv, q1);
            const u128 x = (u128)l0 + (u128)q0 * k;
            double v;
            if (x > Q / 2) {
                u128 y = Q - x;
                v = -((double)(u64)(y >> 64) * 18446744073709551616.0 + (double)(u64)y);
            } else
                v = (double)(u64)(x >> 64) * 18446744073709551616.0 + (double)(u64)x;
            co[i] = v / scale;
        }
    }
    std::vector<double> re(n), im(n);
    for (size_t i = 0; i < n; i++) {
        re[i] = co[i];
        im[i] = co[i + n];
    }
    bitrev_perm(re, im);
    for (size_t len = 2; len <= n; len <<= 1) {
        const size_t lenh = len >> 1, lenq = len << 2, gap = M / lenq;
        for (size_t i = 0; i < n; i += len)
            for (size_t j = 0; j < lenh; j++) {
                const size_t idx = (c->rot_group[j] % lenq) * gap;
                const double kr = c->ksi_re[idx], ki = c->ksi_im[idx];
                const double xr = re[i + j + lenh], xi = im[i + j + lenh];
                const double vr = xr * kr - xi * ki, vi = xr * ki + xi * kr;
                const double ur = re[i + j], ui = im[i + j];
                re[i + j] = ur + vr;
                im[i + j] = ui + vi;
                re[i + j + lenh] = ur - vr;
                im[i + j + lenh] = ui - vi;
            }
    }
    Message m(c->logN - 1);
    for (size_t i = 0; i < n; i++) m[i] = Complex(re[i], im[i]);
    return m;
}

// ---- encrypt / decrypt -------------------------------------------------------------------------------
void Encryptor::encrypt(const Plaintext &pt, const SecretKey &sk, Ciphertext &ct) const {
    const Context &c = ctx_;
    const size_t N = c->N, nq = pt.level_ + 1;
    const u64 enc_id = g_enc_counter++;
    Ciphertext out(c);
    out.allocate(2, pt.level_, pt.rescale_counter_);
    u64 *b = out.buf_.data(), *a = b + nq * N;
    const auto primes = chain_primes(nq);
    std::vector<u64> keys(nq);
    for (size_t i = 0; i < nq; i++) keys[i] = stream_key(g_seed + enc_id, TAG_ENC_A, i, 0);
    ck(hemm_sample_uniform(c->dev, keys.data(), primes.data(), (uint32_t)nq, a, nullptr));
    DeviceBuffer e(c, nq * N), tmp(c, nq * N);
    ck(hemm_sample_error(c->dev, stream_key(g_seed + enc_id, TAG_ENC_E, 0, 0), primes.data(), (uint32_t)nq, e.data(), nullptr));
    ck(hemm_ntt(c->dev, e.data(), primes.data(), (uint32_t)nq, 1, 0, nullptr));
    ck(hemm_pointwise(c->dev, HEMM_MUL, a, 0, sk.ntt(), 0, tmp.data(), 0, (uint32_t)nq, 0, 1, nullptr));
    ck(hemm_pointwise(c->dev, HEMM_SUB, e.data(), 0, tmp.data(), 0, b, 0, (uint32_t)nq, 0, 1, nullptr));
    ck(hemm_pointwise(c->dev, HEMM_ADD, b, 0, pt.buf_.data(), 0, b, 0, (uint32_t)nq, 0, 1, nullptr));
    out.occupied_ = pt.occupied_;
    ct = std::move(out);
}
void Encryptor::encrypt(const Message &msg, const SecretKey &sk, Ciphertext &ct) const {
    EnDecoder ed(ctx_);
    encrypt(ed.encode(msg), sk, ct);
}
void Decryptor::decrypt(const Ciphertext &ct, const SecretKey &sk, Plaintext &pt) const {
    const Context &c = ctx_;
    const size_t N = c->N;
    const u64 lvl = std::min<u64>(ct.level_, 1);
    const uint32_t nq = (uint32_t)lvl + 1;
    Plaintext out(c);
    out.allocate(lvl, 0);
    DeviceBuffer tmp(c, nq * N);
    u64 *m = out.buf_.data();
    ck(hemm_pointwise(c->dev, HEMM_MUL, ct.buf_.data() + ct.polyStride(), 0, sk.ntt(), 0, tmp.data(), 0, nq, 0, 1, nullptr));
    ck(hemm_pointwise(c->dev, HEMM_ADD, ct.buf_.data(), 0, tmp.data(), 0, m, 0, nq, 0, 1, nullptr));
    if (ct.num_poly_ == 3) {
        ck(hemm_pointwise(c->dev, HEMM_MUL, sk.ntt(), 0, sk.ntt(), 0, tmp.data(), 0, nq, 0, 1, nullptr));
        ck(hemm_pointwise(c->dev, HEMM_MAC, ct.buf_.data() + 2 * ct.polyStride(), 0, tmp.data(), 0, m, 0, nq, 0, 1, nullptr));
    }
    out.level_ = lvl;
    out.rescale_counter_ = ct.rescale_counter_;
    // only the low limbs are kept, but the values still carry the scale of the source level
    Real sc = c->delta[ct.level_];
    for (u64 k = 0; k < ct.rescale_counter_; k++) sc *= c->delta[ct.level_];
    out.scale_ = sc;
    pt = std::move(out);
}
void Decryptor::decrypt(const Ciphertext &ct, const SecretKey &sk, Message &msg) const {
    Plaintext pt(ctx_);
    decrypt(ct, sk, pt);
    msg = EnDecoder(ctx_).decode(pt);
}

}  // namespace HEaaN

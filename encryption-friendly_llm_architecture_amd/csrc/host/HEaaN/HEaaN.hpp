// HEaaN-compatible C++ surface over the MI355X kernels (C ABI in include/hemm.h).
//
// HEMMer's matrix multiplication (ciphertext/src/MatrixUtils.cpp, ciphertext/src/HEMMer.cpp of the
// reference) is written against the public classes of the closed HEaaN library
// (ciphertext/external/include/HEaaN/*.hpp).  This header re-declares, in this build's own words,
// the subset of that surface the matrix-multiplication path calls, with the same names, argument
// order and error behaviour, so code written for that path compiles against it unchanged.  Every
// ring operation is a call through the C ABI into hand-written gfx950 kernels; nothing falls back to
// the CPU.  Encoding's embedding FFT and the key/encryption samplers run on the host (set-up work);
// their NTTs and products run on the device.
//
// Semantics kept from the HEaaN headers: ciphertext = (b, a) decrypting as b + a*s
// (EncryptionType.hpp:37-38); left rotation maps (m0, m1, ...) to (m_r, m_{r+1}, ...)
// (HomEvaluator.hpp:369); tensor output order (b1b2, a1b2+a2b1, a1a2) (:510-514); rescale maps
// level l to l-1 dividing by q_l (:536-538); binary ops drop to the lower operand's level
// (:128-129); every level has one fixed scale factor (Context.hpp:196-201), here
// Delta_L = 2^log_scale and Delta_{l-1} = Delta_l^2 / q_l.
#pragma once
#include <complex>
#include <cstdint>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

struct hemm_context;

namespace HEaaN {

using u64 = uint64_t;
using i64 = int64_t;
using u32 = uint32_t;
using Real = double;
using Complex = std::complex<double>;

class RuntimeException : public std::runtime_error {
public:
    explicit RuntimeException(const std::string &m) : std::runtime_error(m) {}
};

enum class DeviceType { CPU, GPU };
struct Device {
    DeviceType type = DeviceType::CPU;
    int id = 0;
};
Device getDefaultDevice();
Device getCurrentCudaDevice();
void setCurrentCudaDevice(int id);
struct CudaTools {
    static void cudaDeviceSynchronize();
    static void cudaSetDevice(int id);
};

// FGb is the preset HEMMer always asks for (HEMMer.hpp:36).  The closed library's prime list is
// not available, so FGb here means: N = 2^16, 13 chain primes (60-bit base + 12 of ~2^42), 4 special
// 60-bit primes, dnum = 3, scale 2^42.  Custom sets go through makeContextCustom.
enum class ParameterPreset { FGb, CUSTOM };

struct ContextContent;
using Context = std::shared_ptr<ContextContent>;

Context makeContext(ParameterPreset preset = ParameterPreset::FGb, const std::vector<int> &device_ids = {});
Context makeContextCustom(u64 log_degree, const std::vector<u64> &chain_primes,
                          const std::vector<u64> &special_primes, u64 dnum, u64 log_scale = 42);
// chain chosen top-down so every level's scale stays next to 2^scale_bits
Context makeContextGenerated(u64 log_degree, u64 n_chain, u64 n_special, u64 dnum, u64 base_bits = 60,
                             u64 scale_bits = 42, u64 special_bits = 60);

u64 getLogFullSlots(const Context &c);
u64 getDegree(const Context &c);
u64 getEncryptionLevel(const Context &c);
std::vector<u64> getPrimeList(const Context &c);
std::vector<Real> getDefaultScaleFactorList(const Context &c);
hemm_context *getDeviceContext(const Context &c);
void setSeed(u64 seed);  // seeds the key / encryption samplers

// ---- device memory ---------------------------------------------------------------------------
class DeviceBuffer {
public:
    DeviceBuffer() = default;
    DeviceBuffer(const Context &c, size_t words);
    DeviceBuffer(const DeviceBuffer &o);
    DeviceBuffer(DeviceBuffer &&o) noexcept;
    DeviceBuffer &operator=(const DeviceBuffer &o);
    DeviceBuffer &operator=(DeviceBuffer &&o) noexcept;
    ~DeviceBuffer();
    u64 *data() const { return ptr_; }
    size_t words() const { return words_; }
    void resize(const Context &c, size_t words);  // contents undefined afterwards
    void release();

private:
    Context ctx_;
    u64 *ptr_ = nullptr;
    size_t words_ = 0, cap_ = 0;
};

// ---- value types -----------------------------------------------------------------------------
class Message {
public:
    Message() = default;
    explicit Message(u64 log_slots) : log_slots_(log_slots), v_(size_t(1) << log_slots) {}
    Message(u64 log_slots, Complex init) : log_slots_(log_slots), v_(size_t(1) << log_slots, init) {}
    Complex &operator[](u64 i) { return v_[i]; }
    const Complex &operator[](u64 i) const { return v_[i]; }
    auto begin() { return v_.begin(); }
    auto end() { return v_.end(); }
    auto begin() const { return v_.begin(); }
    auto end() const { return v_.end(); }
    u64 getSize() const { return v_.size(); }
    u64 getLogSlots() const { return log_slots_; }
    void to(const Device &) {}  // messages live on the host; encode uploads
    void save(const std::string &path) const;
    void load(const std::string &path);

private:
    u64 log_slots_ = 0;
    std::vector<Complex> v_;
};

class Plaintext {
public:
    explicit Plaintext(const Context &c) : ctx_(c) {}
    u64 getLevel() const { return level_; }
    void setLevel(u64 level);  // only lowering: keeps the first level+1 limbs
    u64 getLogSlots() const { return log_slots_; }
    u64 getRescaleCounter() const { return rescale_counter_; }
    void to(const Device &) {}
    u64 *getMxData() const {
        hash_state_ = 2;   // a writable pointer is out: the content can change behind this object's back
        return buf_.data();
    }
    const Context &getContext() const { return ctx_; }
    // internal
    void allocate(u64 level, u64 rescale_counter);
    Context ctx_;
    DeviceBuffer buf_;  // [level+1][N], NTT form
    u64 level_ = 0, log_slots_ = 0, rescale_counter_ = 0;
    Real scale_ = 0;    // scale of the encoded values; 0 = the fixed scale of (level, rescale counter)
    u64 occupied_ = ~u64(0);   // slots at and beyond this index were encoded as exact zeros (all ones: unknown)
    // Run table of a mask whose residues are constant over aligned runs of 2^compact_shift_ coefficients (the NTT
    // form of a slot pattern with a power-of-two period): [limbs][N >> shift].  Filled by makeCompact() on masks
    // that are cached and never written again; allocate() and setLevel() drop it.
    DeviceBuffer compact_;
    u32 compact_shift_ = 0;
    bool makeCompact();        // true when a table was found
    // Hash of the residues, kept by callers that cache work per plaintext content (the weight preparation of the
    // plaintext x ciphertext product): 0 = not computed, 1 = content_hash_ is valid (every evaluator operation writes
    // a plaintext through allocate(), which resets this), 2 = never valid (see getMxData()).
    mutable u64 content_hash_ = 0, content_hash2_ = 0;   // two independent 64-bit digests: a 128-bit key
    mutable int hash_state_ = 0;
};

class Ciphertext {
public:
    explicit Ciphertext(const Context &c) : ctx_(c) {}
    u64 getLevel() const { return level_; }
    u64 getLogSlots() const { return log_slots_; }
    u64 getNumPoly() const { return num_poly_; }
    u64 getRescaleCounter() const { return rescale_counter_; }
    // device pointer to polynomial i; limbs [0, level] are contiguous (what the reference hands to
    // ncclAllReduce, HEMMer.cpp:2629-2632)
    u64 *getPolyData(u64 i, u64 level = 0) const;
    Device getDevice() const { return Device{DeviceType::GPU, 0}; }
    void to(const Device &) {}
    void save(const std::string &path) const;
    void load(const std::string &path);
    const Context &getContext() const { return ctx_; }
    // internal
    void allocate(u64 num_poly, u64 level, u64 rescale_counter);
    size_t polyStride() const;
    Context ctx_;
    DeviceBuffer buf_;  // [num_poly][level+1][N], NTT form
    u64 level_ = 0, log_slots_ = 0, num_poly_ = 0, rescale_counter_ = 0;
    // Slots at and beyond this index are known to hold zero (up to noise); all ones = nothing known.  Set by
    // Encryptor::encrypt from the plaintext, carried through the slot-wise operations of HomEvaluator (add, products,
    // rescale, levelDown, conjugation ...), forgotten by everything else: rotations, allocate(), load(), and
    // getPolyData(), which hands out a writable pointer.  Products use it to tell a single tile from stacked tiles.
    mutable u64 occupied_ = ~u64(0);
    u64 occupiedSlots() const { return occupied_; }
};

class SecretKey {
public:
    explicit SecretKey(const Context &c);                 // seeded ternary, Hamming weight 192
    SecretKey(const Context &c, const int *coefficients); // caller-given coefficients in {-1,0,1}
    SecretKey(const Context &c, const std::string &path);
    void save(const std::string &path) const;
    void to(const Device &) {}
    const std::vector<int> &getCoefficients() const { return coeffs_; }
    const u64 *ntt() const { return ntt_.data(); }  // [nQ+nP][N]
    const Context &getContext() const { return ctx_; }

private:
    void upload();
    Context ctx_;
    std::vector<int> coeffs_;
    DeviceBuffer ntt_;
};

// Evaluation keys resident in HBM: [dnum][2][nQ+nP][N] each.
class KeyPack {
public:
    explicit KeyPack(const Context &c) : ctx_(c) {}
    KeyPack(const Context &c, const std::string &dir);
    void save(const std::string &dir) const;
    void to(const Device &) {}
    bool hasMultKey() const { return mult_.words() != 0; }
    bool hasGaloisKey(u64 galois) const { return galois_.count(galois) != 0 || compact_.count({1, galois}) != 0; }
    const u64 *multKey() const;
    const u64 *galoisKey(u64 galois) const;
    // key switching rho_g(s)^2 -> s: rotates the degree-2 component of an un-relinearised product directly
    bool hasGaloisSquareKey(u64 galois) const { return galois_sq_.count(galois) != 0 || compact_.count({2, galois}) != 0; }
    const u64 *galoisSquareKey(u64 galois) const;
    const Context &getContext() const { return ctx_; }
    // The compact form of a key for the hoisted sums (hemm_key_compact: 6 bytes per residue of a prime below 2^44),
    // made on first request.  kind: 0 multiplication key, 1 key of X -> X^galois, 2 its square key.
    // A Galois or square key that has a compact form gives up its plain form (the sums read only the compact one, and
    // there are hundreds of such keys); galoisKey / galoisSquareKey rebuild the plain form on request
    // (hemm_key_expand, lossless) and keep the few most recent ones.  The multiplication key keeps both forms.
    const u64 *compactKey(int kind, u64 galois) const;
    // device bytes held by the keys: plain forms, compact forms
    std::pair<u64, u64> keyBytes() const;
    // internal
    Context ctx_;
    DeviceBuffer mult_;
    mutable std::map<u64, DeviceBuffer> galois_, galois_sq_;
    mutable std::map<std::pair<int, u64>, DeviceBuffer> compact_;
    mutable std::vector<std::pair<int, u64>> rebuilt_;   // plain forms rebuilt from compact ones, oldest first
    // set by a holder whose work goes through the hoisted sums: KeyGenerator then compacts a Galois or square key as
    // soon as it is generated, so that at most one plain form exists at a time while hundreds of keys are derived
    bool compact_on_generate_ = false;
    bool compactible() const;   // the hoisted kernels take compact keys for this context (N >= 512, at most 6 digits)

private:
    const u64 *plainOrRebuilt(int kind, u64 galois) const;
};

class KeyGenerator {
public:
    KeyGenerator(const Context &c, const SecretKey &sk, KeyPack &pack) : ctx_(c), sk_(sk), pack_(pack) {}
    void genEncKey() const {}  // encryption here is secret-key (Encryptor::encrypt(pt, sk, ct))
    void genMultKey() const;
    void genConjKey() const;
    void genLeftRotKey(u64 rot) const;
    void genRightRotKey(u64 rot) const;
    void genLeftRotSquareKey(u64 rot) const;   // KeyPack::galoisSquareKey of a left rotation (not in HEaaN)
    // keys by Galois element (not in HEaaN): of X -> X^g for any odd g, e.g. a rotation followed by the conjugation
    void genGaloisKey(u64 galois) const;
    void genGaloisSquareKey(u64 galois) const;
    void genRotKeyBundle() const;   // every power-of-two left and right rotation
    void genCommonKeys() const;     // mult + conj + power-of-two rotations
    void genRotKeysForBootstrap(u64) const {}  // bootstrapping is outside this build

private:
    void genSwitchKey(u64 key_id, const u64 *s_from, DeviceBuffer &out) const;
    Context ctx_;
    const SecretKey &sk_;
    KeyPack &pack_;
};

class EnDecoder {
public:
    explicit EnDecoder(const Context &c) : ctx_(c) {}
    Plaintext encode(const Message &msg, u64 level, u64 rescale_counter = 0) const;
    Plaintext encode(const Message &msg) const;
    Message decode(const Plaintext &pt) const;
    // plaintext over the extended basis (limbs q_0..q_level then the special primes), for masks that
    // are applied before ModDown
    Plaintext encodeExtended(const Message &msg, u64 level) const;
    // the same with the values scaled by `scale` instead of the level's fixed scale
    Plaintext encodeExtended(const Message &msg, u64 level, Real scale) const;

private:
    Context ctx_;
};

class Encryptor {
public:
    explicit Encryptor(const Context &c) : ctx_(c) {}
    void encrypt(const Plaintext &pt, const SecretKey &sk, Ciphertext &ct) const;
    void encrypt(const Message &msg, const SecretKey &sk, Ciphertext &ct) const;

private:
    Context ctx_;
};

class Decryptor {
public:
    explicit Decryptor(const Context &c) : ctx_(c) {}
    void decrypt(const Ciphertext &ct, const SecretKey &sk, Message &msg) const;
    void decrypt(const Ciphertext &ct, const SecretKey &sk, Plaintext &pt) const;

private:
    Context ctx_;
};

class HomEvaluator {
public:
    HomEvaluator(const Context &c, const KeyPack &pack) : ctx_(c), pack_(pack) {}
    const Context &getContext() const { return ctx_; }
    const KeyPack &getKeyPack() const { return pack_; }

    void negate(const Ciphertext &a, Ciphertext &out) const;
    void add(const Ciphertext &a, const Ciphertext &b, Ciphertext &out) const;
    void add(const Ciphertext &a, const Plaintext &b, Ciphertext &out) const;
    void add(const Ciphertext &a, const Message &b, Ciphertext &out) const;
    void add(const Ciphertext &a, const Complex &c, Ciphertext &out) const;
    void add(const Plaintext &a, const Plaintext &b, Plaintext &out) const;
    void sub(const Ciphertext &a, const Ciphertext &b, Ciphertext &out) const;
    void sub(const Ciphertext &a, const Message &b, Ciphertext &out) const;

    void mult(const Ciphertext &a, const Ciphertext &b, Ciphertext &out) const;
    // out[i] = mult(*a[i], *b[i]) for products that do not depend on one another -- the same residues as the calls one
    // by one, through shared launches when the operands sit at one level: the tensor products, ONE ModUp of all the
    // third polynomials, ONE sum with the multiplication key, ONE ModDown and ONE rescale.  (No counterpart in HEaaN's
    // interface: the polynomial evaluators issue the independent products of a step together.)
    void multBatch(const std::vector<const Ciphertext *> &a, const std::vector<const Ciphertext *> &b,
                   std::vector<Ciphertext> &out) const;
    // out[i] = rescale(multWithoutRescale(a, csts[i])) for real constants, the products through ONE rescale (same
    // residues as the calls one by one; a is rescaled, two polynomials, above level 0)
    void multRealBatch(const Ciphertext &a, const std::vector<Real> &csts, std::vector<Ciphertext> &out) const;
    void mult(const Ciphertext &a, const Plaintext &b, Ciphertext &out) const;
    void mult(const Ciphertext &a, const Message &b, Ciphertext &out) const;
    void mult(const Ciphertext &a, const Complex &c, Ciphertext &out) const;
    void mult(const Plaintext &a, const Complex &c, Plaintext &out) const;
    void mult(const Plaintext &a, const Plaintext &b, Plaintext &out) const;
    void multWithoutRescale(const Ciphertext &a, const Plaintext &b, Ciphertext &out) const;
    void multWithoutRescale(const Ciphertext &a, const Complex &c, Ciphertext &out) const;
    void multImagUnit(const Ciphertext &a, Ciphertext &out) const;
    void multInteger(const Ciphertext &a, i64 v, Ciphertext &out) const;
    void square(const Ciphertext &a, Ciphertext &out) const;

    void tensor(const Ciphertext &a, const Ciphertext &b, Ciphertext &out) const;
    void relinearize(const Ciphertext &a, Ciphertext &out) const;
    void rescale(Ciphertext &a) const;
    void rescale(Plaintext &a) const;
    void levelDown(const Ciphertext &a, u64 target_level, Ciphertext &out) const;
    void levelDownOne(const Ciphertext &a, Ciphertext &out) const;

    void leftRotate(const Message &a, u64 rot, Message &out) const;
    void rightRotate(const Message &a, u64 rot, Message &out) const;
    void leftRotate(const Plaintext &a, u64 rot, Plaintext &out) const;
    void rightRotate(const Plaintext &a, u64 rot, Plaintext &out) const;
    void leftRotate(const Ciphertext &a, u64 rot, Ciphertext &out) const;
    void rightRotate(const Ciphertext &a, u64 rot, Ciphertext &out) const;
    void leftRotateReduce(const Ciphertext &a, u64 idx_interval, u64 num_summation, Ciphertext &out) const;
    void conjugate(const Ciphertext &a, Ciphertext &out) const;

    // out = rescale( sum_k cts[k] * leftRotate(pt, k * slots / cts.size()) )  -- the diagonal-packing
    // accumulation behind HEMMer::matMulReUse (MatrixUtils.cpp:1636)
    void matmul(const std::vector<Ciphertext> &cts, const Plaintext &pt, Ciphertext &out) const;
    // the same with the plaintext rotated by k * step slots for term k (step = 0: slots / cts.size())
    void matmul(const std::vector<Ciphertext> &cts, const Plaintext &pt, Ciphertext &out, u64 step) const;
    void modReduct(Ciphertext &) const {}  // residues here are always kept in [0, q)

    // extension used by the fused assemble step: out = a*ma + b*mb (no rescale)
    void maskedSum(const Ciphertext &a, const Plaintext &ma, const Ciphertext &b, const Plaintext &mb,
                   Ciphertext &out) const;
    void tensorAccumulate(const Ciphertext &a, const Ciphertext &b, Ciphertext &acc, bool first) const;

private:
    void applyGalois(const Ciphertext &a, u64 galois, Ciphertext &out) const;
    Context ctx_;
    const KeyPack &pack_;
};

// Bootstrapping is outside this build; the class only supplies the level constant the matrix
// multiplications compare against (MatrixUtils.cpp:1111-1115,1320-1324).
class Bootstrapper {
public:
    explicit Bootstrapper(const HomEvaluator &, u64 min_level = 3) : min_level_(min_level) {}
    u64 getMinLevelForBootstrap() const { return min_level_; }
    void bootstrap(const Ciphertext &, Ciphertext &) const;
    void bootstrap(const Ciphertext &, Ciphertext &, Ciphertext &) const;   // complex input -> real and imaginary part
    void bootstrapExtended(const Ciphertext &, Ciphertext &) const;
    void bootstrapExtended(const Ciphertext &, Ciphertext &, Ciphertext &) const;

private:
    u64 min_level_;
};

}  // namespace HEaaN

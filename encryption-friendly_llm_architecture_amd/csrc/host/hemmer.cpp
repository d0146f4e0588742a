// HEMMer facade (reference: ciphertext/src/HEMMer.cpp, codec :232-416,:579-638, packing :764-831,
// matmul entry points :833-880,:964-1124, transpose :1166-1172, masks :2336-2400).
#include <cmath>

#include <fstream>

#include "HELLM/HEMMer.hpp"

namespace HELLM {

static MatrixTransformer matrix_transformer;
void cleanUpMatrixTransformer() { matrix_transformer.cleanUp(); }

namespace {
enum { MASK_COL_EVEN = 0, MASK_ROW_EVEN = 1, MASK_LEFT_HALF = 2, MASK_MATMUL = 3, MASK_MATMUL_HALF = 4 };

i64 tileDim(u64 log_slots) {
    if (log_slots < 3 || (log_slots & 1) == 0)
        throw RuntimeException("HEMMer needs 2 * n * n slots: the number of slots must be an odd power of two");
    return i64(1) << ((log_slots - 1) / 2);
}
i64 pow2ceil(i64 v) {
    i64 p = 1;
    while (p < v) p <<= 1;
    return p;
}
}  // namespace

HEMMer HEMMer::genHEMMer(int device_id, ParameterPreset preset, const bool) { return HEMMer(device_id, preset); }

HEMMer::HEMMer(int device_id, ParameterPreset preset)
    : device_id_(device_id), context_(makeContext(preset, {device_id})), log_slots_(getLogFullSlots(context_)),
      dim_(tileDim(log_slots_)), sk_(context_), enc_(context_), dec_(context_), endec_(context_), pack_(context_),
      eval_(context_, pack_), btp_(eval_, 3) {
    init();
}
HEMMer::HEMMer(const Context &context, u64 min_bootstrap_level)
    : context_(context), log_slots_(getLogFullSlots(context_)), dim_(tileDim(log_slots_)), sk_(context_),
      enc_(context_), dec_(context_), endec_(context_), pack_(context_), eval_(context_, pack_),
      btp_(eval_, min_bootstrap_level) {
    init();
}
HEMMer::HEMMer(const std::string &key_path, int device_id, ParameterPreset preset)
    : device_id_(device_id), context_(makeContext(preset, {device_id})), log_slots_(getLogFullSlots(context_)),
      dim_(tileDim(log_slots_)), sk_(context_, key_path + "/SecretKey.bin"), enc_(context_), dec_(context_),
      endec_(context_), pack_(context_, key_path), eval_(context_, pack_), btp_(eval_, 3) {
    init();
}
HEMMer::~HEMMer() = default;

void HEMMer::init() {
    pack_.compact_on_generate_ = fused_;
    KeyGenerator keygen(context_, sk_, pack_);
    if (!pack_.hasMultKey()) keygen.genMultKey();
    keygen.genConjKey();
    const i64 n = dim_;
    Matrix even(n, n), tr_even(n, n), ones(n, n, 1.0), zeros(n, n, 0.0);
    for (i64 r = 0; r < n; r++)
        for (i64 c = 0; c < n; c++) {
            even.at(r, c) = (c % 2 == 0) ? 1.0 : 0.0;
            tr_even.at(r, c) = (r % 2 == 0) ? 1.0 : 0.0;
        }
    col_mask_even_ = message2(even, even);
    row_mask_even_ = message2(tr_even, tr_even);
    mask_left_half_ = message2(ones, zeros);
    mask_matmul_ = message2(ones, zeros);
    mask_matmul_half_ = message2(Matrix(n, n, 0.5), zeros);
}

void HEMMer::save(const std::string &keys_path) {
    sk_.save(keys_path + "/SecretKey.bin");
    pack_.save(keys_path);
}

const Plaintext &HEMMer::cachedMask(int id, u64 level) const {
    auto key = std::make_pair(id, level);
    auto it = mask_cache_.find(key);
    if (it != mask_cache_.end()) return it->second;
    const Message *m = id == MASK_COL_EVEN ? &col_mask_even_
                       : id == MASK_ROW_EVEN ? &row_mask_even_
                       : id == MASK_LEFT_HALF ? &mask_left_half_
                       : id == MASK_MATMUL_HALF ? &mask_matmul_half_
                                                : &mask_matmul_;
    return mask_cache_.emplace(key, endec_.encode(*m, level)).first->second;
}

namespace {
enum { SEL_FIRST_COL = 100, SEL_LAST_COL, SEL_LEFT_COLS, SEL_RIGHT_COLS, SEL_FIRST_ROW, SEL_FIRST_COL_LEFT_TILE };
}
const Plaintext &HEMMer::selectorMask(int which, u64 level) const {
    auto key = std::make_pair(which, level);
    auto it = mask_cache_.find(key);
    if (it != mask_cache_.end()) return it->second;
    const i64 n = dim_;
    Matrix m(n, n, 0.0), zero(n, n, 0.0);
    for (i64 r = 0; r < n; r++)
        for (i64 c = 0; c < n; c++) {
            bool on = false;
            switch (which) {
                case SEL_FIRST_COL:
                case SEL_FIRST_COL_LEFT_TILE: on = c == 0; break;
                case SEL_LAST_COL: on = c == n - 1; break;
                case SEL_LEFT_COLS: on = c < n / 2; break;
                case SEL_RIGHT_COLS: on = c >= n / 2; break;
                case SEL_FIRST_ROW: on = r == 0; break;
                default: throw std::invalid_argument("[selectorMask] unknown mask");
            }
            if (on) m.at(r, c) = 1.0;
        }
    const Message msg = which == SEL_FIRST_COL_LEFT_TILE ? message2(m, zero) : message2(m, m);
    return mask_cache_.emplace(key, endec_.encode(msg, level)).first->second;
}

void HEMMer::ensureRotationKeys(const std::vector<u64> &rots) const {
    const u64 slots = u64(1) << log_slots_;
    KeyGenerator keygen(context_, sk_, pack_);
    for (u64 r : rots) {
        r %= slots;
        if (r == 0 || have_rot_.count(r)) continue;
        keygen.genLeftRotKey(r);
        have_rot_.insert(r);
    }
}

// rotations issued by a diagonal transform of `kind` on tiles in rows of `width` slots
std::vector<u64> HEMMer::transformRotations(MaskKind kind, i64 width) const {
    const u64 slots = u64(1) << log_slots_;
    const i64 n = dim_;
    if (fused_ && kind != MaskKind::Diagonal)   // the batched products may take the two-stage form
        ensureRotationKeys(MatrixTransformer::twoStageRotations(kind, TileTensorShape(n, n, width), log_slots_));
    std::vector<u64> r;
    auto left = [&](i64 v) { r.push_back((u64)(((v % (i64)slots) + (i64)slots) % (i64)slots)); };
    if (kind == MaskKind::Diagonal) {
        const i64 count = 2 * n - 1, bs = (i64)std::ceil(std::sqrt((double)count)),
                  gs = (i64)std::ceil((double)count / (double)bs), step = width - 1;
        left(-(n - 1) * step);
        left(step);
        for (i64 i = 1; i < gs; i++) left(i * bs * step);
        return r;
    }
    const bool packed = kind == MaskKind::PackedHorizontal || kind == MaskKind::PackedVertical;
    const bool vertical = kind == MaskKind::Vertical || kind == MaskKind::PackedVertical;
    const i64 cell = packed ? 2 : 1, units = n / cell, step = cell * (vertical ? width : 1);
    const i64 bs = (i64)std::ceil(std::sqrt((double)(2 * units - 1))),
              gs = (i64)std::ceil((double)(units - 1) / (double)bs);
    for (i64 j = 0; j < (fused_ ? bs : 1); j++) left((j + 1) * step);   // hoisted baby steps are direct rotations
    for (i64 i = 0; i < gs; i++) {
        left(-(units - i * bs) * step);
        if (i > 0) left(i * bs * step);
    }
    return r;
}

// ---- codec ---------------------------------------------------------------------------------------------
Message HEMMer::message2(const Matrix &a, const Matrix &b) const {
    if (a.rows != b.rows || a.cols != b.cols) throw RuntimeException("message2: shapes differ");
    Message msg(log_slots_, 0);
    if ((u64)(2 * a.rows * a.cols) > msg.getSize()) throw RuntimeException("message2: matrices do not fit");
    for (i64 r = 0; r < a.rows; r++)
        for (i64 c = 0; c < a.cols; c++) {
            msg[(u64)(r * 2 * a.cols + c)] = a.at(r, c);
            msg[(u64)(r * 2 * a.cols + a.cols + c)] = b.at(r, c);
        }
    return msg;
}
PtxtTensor HEMMer::encode(const Matrix &data, u64 level) const {
    Message msg(log_slots_, 0);
    if (data.v.size() > msg.getSize()) throw RuntimeException("encode: matrix does not fit");
    for (size_t i = 0; i < data.v.size(); i++) msg[i] = data.v[i];
    if (level == 0) level = getEncryptionLevel(context_);
    return PtxtTensor(data.rows, data.cols, endec_.encode(msg, level));
}
PtxtTensor HEMMer::encode2(const Matrix &a, const Matrix &b, u64 level) const {
    Message msg = message2(a, b);
    if (level == 0) level = getEncryptionLevel(context_);
    return PtxtTensor(a.rows, a.cols, endec_.encode(msg, level), a.cols * 2);
}
// weight layout of the hoisted plaintext product: 0.5 (W1 - i W3) | 0.5 (W2 - i W4), column j of each
// half rolled up by j (the tau layout)
Message HEMMer::msgDiagonalToRow4(const Matrix &w1, const Matrix &w2, const Matrix &w3, const Matrix &w4) const {
    const i64 h = w1.rows, w = w1.cols;
    Message msg(log_slots_, 0);
    if ((u64)(2 * h * w) > msg.getSize()) throw RuntimeException("msgDiagonalToRow4: matrices do not fit");
    for (i64 r = 0; r < h; r++)
        for (i64 c = 0; c < w; c++) {
            const i64 src = (r + c) % h;
            msg[(u64)(r * 2 * w + c)] = Complex(0.5 * w1.at(src, c), -0.5 * w3.at(src, c));
            msg[(u64)(r * 2 * w + w + c)] = Complex(0.5 * w2.at(src, c), -0.5 * w4.at(src, c));
        }
    return msg;
}
PtxtTensor HEMMer::encodeDiagonalToRow4(const Matrix &w1, const Matrix &w2, const Matrix &w3, const Matrix &w4,
                                        u64 level) const {
    Message msg = msgDiagonalToRow4(w1, w2, w3, w4);
    if (level == 0) level = getEncryptionLevel(context_);
    return PtxtTensor(w1.rows, w1.cols, endec_.encode(msg, level), w1.cols * 2);
}
// ---- rotate-and-sum reductions -----------------------------------------------------------------------
namespace {
std::vector<u64> logSteps(u64 bound, u64 slots) {
    std::vector<u64> r;
    for (u64 i = 1; i < bound; i <<= 1) {
        r.push_back(i);
        r.push_back(slots - i);
    }
    return r;
}
}  // namespace

void HEMMer::reduceRowSumWithScaledMask(CtxtTensor &tensor, const Message &mask) const {
    const u64 w = (u64)tensor.getBlockWidth(), slots = u64(1) << log_slots_;
    if (fused_ && (w & (w - 1)) == 0) {   // the same sums, each as hoisted sums of its rotations
        ensureRotationKeys(rotateSumRotations(1, w, log_slots_));
        ensureRotationKeys(rotateSumRotations(-1, w, log_slots_));
        rotateSumFused(eval_, {{&tensor.get(), 1, &tensor.get()}}, w);
        eval_.mult(tensor.get(), mask, tensor.get());
        rotateSumFused(eval_, {{&tensor.get(), -1, &tensor.get()}}, w);
        return;
    }
    ensureRotationKeys(logSteps(w, slots));
    Ciphertext tmp(context_);
    for (u64 i = 1; i < w; i <<= 1) {
        eval_.leftRotate(tensor.get(), i, tmp);
        eval_.add(tensor.get(), tmp, tensor.get());
    }
    eval_.mult(tensor.get(), mask, tensor.get());
    for (u64 i = 1; i < w; i <<= 1) {
        eval_.rightRotate(tensor.get(), i, tmp);
        eval_.add(tensor.get(), tmp, tensor.get());
    }
}

void HEMMer::oneMatRotSumInplace(CtxtTensor &a, CtxtTensor &b) const {
    const u64 n = (u64)dim_, slots = u64(1) << log_slots_;
    if (fused_ && n >= 4 && (n & (n - 1)) == 0 && a.getLevel() == b.getLevel()) {
        // both tensors through the same launch chains: a to the left and b to the right, then the other way round
        for (i64 unit : {i64(1), i64(-1)}) {
            ensureRotationKeys(rotateSumRotations(unit, n / 2, log_slots_));
            ensureRotationKeys(rotateSumRotations(unit, n, log_slots_));
        }
        rotateSumFused(eval_, {{&a.get(), 1, &a.get()}, {&b.get(), -1, &b.get()}}, n / 2);
        eval_.mult(a.get(), selectorMask(SEL_FIRST_COL, a.getLevel()), a.get());
        eval_.mult(b.get(), selectorMask(SEL_LAST_COL, b.getLevel()), b.get());
        rotateSumFused(eval_, {{&a.get(), -1, &a.get()}, {&b.get(), 1, &b.get()}}, n);
        return;
    }
    ensureRotationKeys(logSteps(n, slots));
    Ciphertext tmp(context_);
    for (u64 rot = 1; rot < n / 2; rot <<= 1) {
        eval_.leftRotate(a.get(), rot, tmp);
        eval_.add(a.get(), tmp, a.get());
        eval_.rightRotate(b.get(), rot, tmp);
        eval_.add(b.get(), tmp, b.get());
    }
    eval_.mult(a.get(), selectorMask(SEL_FIRST_COL, a.getLevel()), a.get());
    eval_.mult(b.get(), selectorMask(SEL_LAST_COL, b.getLevel()), b.get());
    for (u64 rot = 1; rot < n; rot <<= 1) {
        eval_.rightRotate(a.get(), rot, tmp);
        eval_.add(a.get(), tmp, a.get());
        eval_.leftRotate(b.get(), rot, tmp);
        eval_.add(b.get(), tmp, b.get());
    }
}

void HEMMer::maskRightLeft(const CtxtTensor &tensor, CtxtTensor &out_left, CtxtTensor &out_right) const {
    eval_.mult(tensor.get(), selectorMask(SEL_LEFT_COLS, tensor.getLevel()), out_left.get());
    eval_.mult(tensor.get(), selectorMask(SEL_RIGHT_COLS, tensor.getLevel()), out_right.get());
}

void HEMMer::maskFirstColInplace(CtxtTensor &tensor) const {
    eval_.mult(tensor.get(), selectorMask(SEL_FIRST_COL, tensor.getLevel()), tensor.get());
}

void HEMMer::rowMoments(const std::vector<CtxtTensor> &tiles, Real inv_count, CtxtTensor &mean,
                        CtxtTensor &mean_square) const {
    if (tiles.empty()) throw std::invalid_argument("[rowMoments] no tiles");
    Ciphertext tmp(context_);
    mean.get() = tiles[0].get();
    eval_.tensor(tiles[0].get(), tiles[0].get(), mean_square.get());
    for (size_t i = 1; i < tiles.size(); i++) {
        eval_.tensor(tiles[i].get(), tiles[i].get(), tmp);
        eval_.add(mean_square.get(), tmp, mean_square.get());
        eval_.add(mean.get(), tiles[i].get(), mean.get());
    }
    eval_.relinearize(mean_square.get(), mean_square.get());
    eval_.rescale(mean_square.get());
    // both halves of the pair layout are summed together (one token row spans the whole block width)
    Matrix scaled(dim_, dim_, 0.0), zero(dim_, dim_, 0.0);
    for (i64 r = 0; r < dim_; r++) scaled.at(r, 0) = inv_count;
    const Message mask = message2(scaled, zero);
    reduceRowSumWithScaledMask(mean_square, mask);
    reduceRowSumWithScaledMask(mean, mask);
}

void HEMMer::encodeWeight(const std::vector<std::vector<Matrix>> &grid, const std::string &save_path) const {
    const size_t height = grid.size();
    if (height == 0) throw std::invalid_argument("[encodeWeight] empty weight");
    const size_t width = grid[0].size();
    for (const auto &row : grid)
        if (row.size() != width) throw std::invalid_argument("[encodeWeight] ragged tile grid");
    for (size_t i = 0; i < height / 4; i++)
        for (size_t j = 0; j < width; j++)
            msgDiagonalToRow4(grid[4 * i][j], grid[4 * i + 1][j], grid[4 * i + 2][j], grid[4 * i + 3][j])
                .save(save_path + std::to_string(i) + "_" + std::to_string(j) + ".msg");
    if (height % 4 > 0) {
        if (height < 2) throw std::invalid_argument("[encodeWeight] a trailing group needs two tile rows");
        const Matrix zero(dim_, dim_, 0.0);
        for (size_t j = 0; j < width; j++)
            msgDiagonalToRow4(grid[height - 2][j], grid[height - 1][j], zero, zero)
                .save(save_path + std::to_string(height / 4) + "_" + std::to_string(j) + ".msg");
    }
}
void HEMMer::encodeWeight(const std::vector<Matrix> &tiles, const std::string &save_path) const {
    for (size_t i = 0; i < tiles.size() / 2; i++)
        message2(tiles[2 * i], tiles[2 * i + 1]).save(save_path + std::to_string(i) + ".msg");
}
PtxtTensor HEMMer::getWeight(const std::string &file, u64 level) const {
    Message msg(log_slots_);
    msg.load(file);
    if (msg.getLogSlots() != log_slots_) throw RuntimeException("weight file does not match the slot count: " + file);
    return PtxtTensor(dim_, dim_, endec_.encode(msg, level), 2 * dim_);
}
void HEMMer::saveCtxtTensor(const CtxtTensor &t, const std::string &file) const {
    t.get().save(file);
    std::ofstream f(file + ".shape", std::ios::binary);
    if (!f) throw RuntimeException("cannot open " + file + ".shape");
    const i64 shape[3] = {t.getHeight(), t.getWidth(), t.getBlockWidth()};
    f.write((const char *)shape, sizeof(shape));
}
CtxtTensor HEMMer::loadCtxtTensor(const std::string &file) const {
    std::ifstream f(file + ".shape", std::ios::binary);
    if (!f) throw RuntimeException("cannot open " + file + ".shape");
    i64 shape[3];
    f.read((char *)shape, sizeof(shape));
    CtxtTensor t(context_, shape[0], shape[1], shape[2]);
    t.get().load(file);
    return t;
}

CtxtTensor HEMMer::encrypt(const Matrix &data) const {
    PtxtTensor p = encode(data);
    CtxtTensor ret(context_, p.getShape());
    enc_.encrypt(p.get(), sk_, ret.get());
    return ret;
}
CtxtTensor HEMMer::encrypt2(const Matrix &a, const Matrix &b) const {
    PtxtTensor p = encode2(a, b);
    CtxtTensor ret(context_, p.getShape());
    enc_.encrypt(p.get(), sk_, ret.get());
    return ret;
}
Matrix HEMMer::decrypt(const CtxtTensor &t) const {
    Message msg(log_slots_);
    dec_.decrypt(t.get(), sk_, msg);
    Matrix m(t.getHeight(), t.getWidth());
    for (size_t i = 0; i < m.v.size(); i++) m.v[i] = msg[i].real();
    return m;
}
std::vector<Matrix> HEMMer::decrypt2(const CtxtTensor &t) const {
    Message msg(log_slots_);
    dec_.decrypt(t.get(), sk_, msg);
    const i64 h = t.getHeight(), w = t.getWidth();
    std::vector<Matrix> out(2, Matrix(h, w));
    for (i64 r = 0; r < h; r++)
        for (i64 c = 0; c < w; c++) {
            out[0].at(r, c) = msg[(u64)(r * 2 * w + c)].real();
            out[1].at(r, c) = msg[(u64)(r * 2 * w + w + c)].real();
        }
    return out;
}

// ---- packing ---------------------------------------------------------------------------------------------
void HEMMer::transposeInplace(CtxtTensor &t, u64 target_level) const {
    if (fused_ && t.getHeight() == t.getWidth() && t.getHeight() == dim_) {
        // batched: the 2n - 1 diagonals through the same launch chain as sigma / tau (hoisted baby steps, one masked-sum
        // launch, giant steps summed before one ModDown)
        const u64 slots = u64(1) << log_slots_;
        const i64 n = dim_, step = t.getBlockWidth() - 1;
        const i64 bs = (i64)std::ceil(std::sqrt((double)(2 * n - 1))), gs = (i64)std::ceil((double)(n - 1) / (double)bs);
        std::vector<u64> r;
        auto left = [&](i64 v) { r.push_back((u64)(((v % (i64)slots) + (i64)slots) % (i64)slots)); };
        for (i64 j = 0; j < bs; j++) left((j + 1) * step);
        for (i64 i = 0; i < gs; i++) {
            left(-(n - i * bs) * step);
            if (i > 0) left(i * bs * step);
        }
        ensureRotationKeys(r);
        if (target_level > 0) eval_.levelDown(t.get(), 1 + target_level, t.get());
        const TileTensorShape shape(t.getWidth(), t.getHeight(), t.getBlockWidth());
        Ciphertext out = matrix_transformer.diagonalTransformFused(eval_, t.get(), MaskKind::DiagonalSigned, shape);
        t = CtxtTensor(shape, out);
        return;
    }
    ensureRotationKeys(transformRotations(MaskKind::Diagonal, t.getBlockWidth()));
    if (target_level > 0) eval_.levelDown(t.get(), 1 + target_level, t.get());
    t = matrix_transformer.transpose(eval_, t);
}

// adjacent columns (2c, 2c+1) -> a + i b, written to both slots of the pair
void HEMMer::complexPackingInplace(CtxtTensor &t) const {
    const u64 slots = u64(1) << log_slots_;
    ensureRotationKeys({1, slots - 1});
    Ciphertext odd(context_), even(context_), fus(context_);
    const Plaintext &m = cachedMask(MASK_COL_EVEN, t.getLevel());
    eval_.mult(t.get(), m, even);
    eval_.leftRotate(t.get(), 1, odd);
    eval_.multImagUnit(odd, odd);
    eval_.mult(odd, m, odd);
    eval_.add(odd, even, fus);
    eval_.rightRotate(fus, 1, t.get());
    eval_.add(t.get(), fus, t.get());
}
void HEMMer::transposeComplexPackingInplace(CtxtTensor &t, u64 target_level) const {
    const u64 slots = u64(1) << log_slots_;
    ensureRotationKeys({1, slots - 1});
    Ciphertext odd(context_), even(context_), fus(context_);
    const Plaintext &m = cachedMask(MASK_COL_EVEN, t.getLevel());
    eval_.mult(t.get(), m, even);
    eval_.leftRotate(t.get(), 1, odd);
    eval_.multImagUnit(odd, odd);
    eval_.negate(odd, odd);
    eval_.mult(odd, m, odd);
    eval_.add(odd, even, fus);
    eval_.rightRotate(fus, 1, t.get());
    eval_.add(t.get(), fus, t.get());
    if (target_level > 0) eval_.levelDown(t.get(), 1 + target_level, t.get());
    transposeInplace(t);
}
// adjacent rows (2k, 2k+1) -> a - i b, written to both rows of the pair
void HEMMer::complexPackingRowInplace(CtxtTensor &t) const {
    const u64 slots = u64(1) << log_slots_, w = (u64)t.getBlockWidth();
    ensureRotationKeys({w, slots - w});
    Ciphertext odd(context_), even(context_), fus(context_);
    // even rows of rows `w` slots wide: the reference's mask is laid out for the pair layout (w = 2 n); other widths
    // get their own pattern
    const Plaintext *mp;
    if (w == (u64)(2 * dim_)) {
        mp = &cachedMask(MASK_ROW_EVEN, t.getLevel());
    } else {
        const auto key = std::make_pair(1000 + (int)w, t.getLevel());
        auto it = mask_cache_.find(key);
        if (it == mask_cache_.end()) {
            Message msg(log_slots_, 0);
            for (u64 j = 0; j < slots; j++)
                if ((j / w) % 2 == 0) msg[j] = 1;
            it = mask_cache_.emplace(key, endec_.encode(msg, t.getLevel())).first;
        }
        mp = &it->second;
    }
    const Plaintext &m = *mp;
    eval_.mult(t.get(), m, even);
    eval_.leftRotate(t.get(), w, odd);
    eval_.multImagUnit(odd, odd);
    eval_.negate(odd, odd);
    eval_.mult(odd, m, odd);
    eval_.add(even, odd, fus);
    eval_.rightRotate(fus, w, t.get());
    eval_.add(t.get(), fus, t.get());
}
void HEMMer::splitInTwo(CtxtTensor &t, CtxtTensor &t1, CtxtTensor &t2) const {
    const u64 slots = u64(1) << log_slots_, width = (u64)t.getWidth();
    ensureRotationKeys({width, slots - width});
    Ciphertext tmp(context_), low(context_);
    eval_.mult(t.get(), cachedMask(MASK_LEFT_HALF, t.getLevel()), tmp);
    eval_.levelDown(t.get(), tmp.getLevel(), low);
    eval_.sub(low, tmp, t2.get());
    eval_.rightRotate(tmp, width, t1.get());
    eval_.add(t1.get(), tmp, t1.get());
    eval_.leftRotate(t2.get(), width, tmp);
    eval_.add(t2.get(), tmp, t2.get());
}

// ---- products ---------------------------------------------------------------------------------------------
CtxtTensor HEMMer::diagonalToColumn(const CtxtTensor &a) const {
    ensureRotationKeys(transformRotations(MaskKind::Horizontal, a.getBlockWidth()));
    if (fused_) {   // one stage (the level contract: in at l, out at l - 1) through the batched launches
        CtxtTensor res(a);
        res.get() = matrix_transformer.diagonalTransformFused(eval_, a.get(), MaskKind::Horizontal, a.getShape());
        return res;
    }
    return matrix_transformer.diagonalToColumn(eval_, a);
}
CtxtTensor HEMMer::diagonalToRow(const CtxtTensor &b) const {
    ensureRotationKeys(transformRotations(MaskKind::Vertical, b.getBlockWidth()));
    if (fused_) {
        CtxtTensor res(b);
        res.get() = matrix_transformer.diagonalTransformFused(eval_, b.get(), MaskKind::Vertical, b.getShape());
        return res;
    }
    return matrix_transformer.diagonalToRow(eval_, b);
}
CtxtTensor HEMMer::singleCCMatMul(const CtxtTensor &a, const CtxtTensor &b, u64 T) const {
    const u64 slots = u64(1) << log_slots_;
    const i64 w = a.getBlockWidth(), n = pow2ceil(a.getWidth());
    ensureRotationKeys(transformRotations(MaskKind::Horizontal, w));
    ensureRotationKeys(transformRotations(MaskKind::Vertical, w));
    if (fused_) {
        // One tile block and nothing else in the slot vector: promised by the caller, or known because the operand
        // comes from Encryptor::encrypt through slot-wise operations only (Ciphertext::occupiedSlots).  Only B has to
        // be such a tile: its row shifts become exact rotations once tau(B) is copied into every block, and each
        // slot of the sum over the shifts of sigma(A) then holds what it should whatever A carries in its other
        // blocks (column shifts stay inside a row; the rotations of the baby-step / giant-step split cancel slot by
        // slot).  What A carries there shows up in the other blocks of the result, so the result is known to be a
        // single tile only when A is one as well.
        const u64 block = (u64)(n * w);
        const bool a_single = single_tile_ || a.get().occupiedSlots() <= block;
        const bool single = single_tile_ || b.get().occupiedSlots() <= block;
        const u64 unknown = ~u64(0);
        // A single tile with a level to spare goes through the complex-packed product: adjacent columns of A and
        // adjacent rows of B are fused into complex slots (one level), the product then needs n / 2 column shifts
        // (each a key product and a ModDown) instead of n, and x + conj(x) returns the real product.
        if (block <= slots && slots % block == 0 && n >= 4 && a.getHeight() == n && a.getWidth() == n &&
            b.getHeight() == n && b.getWidth() == n &&
            std::min(a.getLevel(), b.getLevel()) >= T + 3 && a.get().getRescaleCounter() == 0 &&
            b.get().getRescaleCounter() == 0) {
            // both packings through one launch chain, at level T+5 (the transforms start from T+4)
            ensureRotationKeys({1, slots - 1, (u64)w, slots - (u64)w});
            ensureRotationKeys(transformRotations(MaskKind::PackedHorizontal, w));
            ensureRotationKeys(transformRotations(MaskKind::PackedVertical, w));
            // three levels above the target with exact row rotations: B's packing and first tau stage are one composite
            // map (MatrixTransformer::packingStageOne), with rotations of its own
            // operands with a level less than a separate packing needs (A below T+5 or B below T+4) and exact row
            // rotations: the packing and the first transform stage are one composite map, with rotations of its own
            // (with masked row shifts both operands end at T+2: composite maps when the lower one is at T+4)
            const bool exact_rows = block == slots || (single && block < slots);
            const bool separate = a.getLevel() >= T + 5 && b.getLevel() >= T + 4;
            if (n >= 8 && ((exact_rows && !separate) || (!exact_rows && std::min(a.getLevel(), b.getLevel()) == T + 4))) {
                ensureRotationKeys(MatrixTransformer::packingStageOneRotations(MaskKind::PackedVertical,
                                                                               TileTensorShape(n, n, w), log_slots_));
                if (a.getLevel() >= T + 4)
                    ensureRotationKeys(MatrixTransformer::packingStageOneRotations(MaskKind::PackedHorizontal,
                                                                                   TileTensorShape(n, n, w), log_slots_));
            }
            std::vector<u64> sq;
            // stacked tiles / unknown content keep their per-block products: the packed cells then shift through
            // masked pairs (no baby-step / giant-step split, which needs exact row rotations)
            const bool spread = single && block < slots;
            ensureRotationKeys(fusedCcmmRotations(TileTensorShape(n, n, w), log_slots_, sq, true, spread));
            KeyGenerator kg(context_, sk_, pack_);
            for (u64 r : sq) kg.genLeftRotSquareKey(r);
            // x + conj(x) inside the product: its giant-step sum (exact row rotations: the block fills the slot vector
            // or is spread over it) takes every term a second time under the Galois element times 2N - 1
            if (block == slots || spread) {
                const u64 two_n = 4 * slots, cj = two_n - 1;   // 2N with N = 2 * slots
                auto galois = [&](u64 r) {   // 5^r mod 2N
                    u64 g = 1, b = 5 % two_n;
                    for (r %= slots; r; r >>= 1, b = b * b % two_n)
                        if (r & 1) g = g * b % two_n;
                    return g;
                };
                kg.genConjKey();
                kg.genGaloisSquareKey(cj);
                for (u64 r : sq) {
                    const u64 gc = (galois(r) * cj) % two_n;
                    kg.genGaloisKey(gc);
                    kg.genGaloisSquareKey(gc);
                }
            }
            CtxtTensor res = multMatMatComplexPackedFused(eval_, btp_, a, b, T, matrix_transformer, batch_, spread, true);
            if (spread) res.get().occupied_ = a_single ? block : unknown;
            return res;
        }
        std::vector<u64> square_rots;
        ensureRotationKeys(fusedCcmmRotations(TileTensorShape(n, n, w), log_slots_, square_rots, false, single));
        KeyGenerator keygen(context_, sk_, pack_);
        for (u64 r : square_rots) keygen.genLeftRotSquareKey(r);
        CtxtTensor res = multMatMatFused(eval_, btp_, a, b, T, matrix_transformer, batch_, single);
        if (!a_single) res.get().occupied_ = unknown;
        return res;
    }
    ensureRotationKeys({1, (u64)w, slots - (u64)n, slots - (u64)((n * w) % (i64)slots)});
    return multMatMat(eval_, btp_, a, b, T, matrix_transformer);
}
CtxtTensor HEMMer::singleMatMul(const CtxtTensor &a, const PtxtTensor &b, u64 T) const {
    const u64 slots = u64(1) << log_slots_;
    const i64 w = a.getBlockWidth(), n = pow2ceil(a.getWidth());
    ensureRotationKeys(transformRotations(MaskKind::Horizontal, w));
    if (fused_) {
        ensureRotationKeys(fusedRotations(TileTensorShape(n, n, w), log_slots_, false, false));
        CtxtTensor res(context_, a.getHeight(), b.getWidth(), w);
        if (multMatMatPlainFused(eval_, btp_, a, b, T, matrix_transformer, batch_, res)) return res;
    }
    ensureRotationKeys({1, slots - (u64)n});
    return multMatMat(eval_, btp_, a, b, T, matrix_transformer);
}
CtxtTensor HEMMer::packedMatMul(const CtxtTensor &a, const CtxtTensor &b, u64 T) const {
    const u64 slots = u64(1) << log_slots_;
    const i64 w = a.getBlockWidth(), n = pow2ceil(a.getWidth());
    ensureRotationKeys(transformRotations(MaskKind::PackedHorizontal, w));
    ensureRotationKeys(transformRotations(MaskKind::PackedVertical, w));
    // a single tile in part of the slots is taken only on the caller's promise (assumeSingleTile): the packing that
    // produced the operands rotates, which forgets what the evaluator knew about empty slots
    const bool spread = single_tile_ && (u64)(n * w) < slots && slots % (u64)(n * w) == 0;
    if (fused_ && ((u64)(n * w) == slots || spread)) {
        std::vector<u64> square_rots;
        ensureRotationKeys(fusedCcmmRotations(TileTensorShape(n, n, w), log_slots_, square_rots, true, spread));
        KeyGenerator keygen(context_, sk_, pack_);
        for (u64 r : square_rots) keygen.genLeftRotSquareKey(r);
        return multPackedMatMatFused(eval_, btp_, a, b, T, matrix_transformer, batch_, spread);
    }
    ensureRotationKeys({2, (u64)(2 * w), slots - (u64)n});
    return multPackedMatMat(eval_, btp_, a, b, T, matrix_transformer);
}
CtxtTensor HEMMer::packedMatMulPre(const CtxtTensor &a, u64 T) const {
    ensureRotationKeys(transformRotations(MaskKind::PackedHorizontal, a.getBlockWidth()));
    if (fused_ && a.getLevel() >= T + 3) {   // sigma through the batched launches (two stages with a level to spare)
        CtxtTensor res(a);
        res.get() = matrix_transformer.lowerAndTransformFused(eval_, a.get(), MaskKind::PackedHorizontal, a.getShape(), T + 2);
        return res;
    }
    return multPackedMatMatPre(eval_, a, T, matrix_transformer);
}
void HEMMer::packedMatMulPreRot(const CtxtTensor &a, std::vector<Ciphertext> &tmp, u64 T) const {
    const u64 slots = u64(1) << log_slots_;
    if (fused_ && a.getLevel() == T + 2 && a.get().getRescaleCounter() == 0) {
        std::vector<u64> rots{slots - (u64)a.getHeight()};
        for (i64 i = 1; i < a.getHeight() / 2; i++) rots.push_back((u64)(2 * i));
        ensureRotationKeys(rots);
        multPackedMatMatPreRotFused(eval_, a, tmp, T, matrix_transformer, batch_);
        return;
    }
    ensureRotationKeys({2, slots - (u64)a.getHeight()});
    multPackedMatMatPreRot(eval_, a, tmp, T, matrix_transformer);
}
CtxtTensor HEMMer::packedMatMulPreRev(const CtxtTensor &b, u64 T) const {
    ensureRotationKeys(transformRotations(MaskKind::PackedVertical, b.getBlockWidth()));
    if (fused_ && b.getLevel() >= T + 2) {   // tau through the batched launches (two stages with a level to spare)
        CtxtTensor res(b);
        res.setShape(pow2ceil(b.getHeight()), b.getWidth());
        res.get() = matrix_transformer.lowerAndTransformFused(eval_, b.get(), MaskKind::PackedVertical, res.getShape(), T + 1);
        return res;
    }
    return multPackedMatMatPreRev(eval_, b, T, matrix_transformer);
}
CtxtTensor HEMMer::packedMatMulCCReuse(const std::vector<Ciphertext> &tmp, const CtxtTensor &b, u64 T) const {
    if (fused_ && tmp.size() > 1) {
        const u64 step = (u64)(2 * b.getBlockWidth());
        std::vector<u64> rots;
        for (size_t k = 1; k < tmp.size(); k++) rots.push_back((k * step) % (u64(1) << log_slots_));
        ensureRotationKeys(rots);
        return multMatMatCCReUseFused(eval_, tmp, b, step, true, batch_);
    }
    ensureRotationKeys({(u64)(2 * b.getBlockWidth())});
    return multPackedMatMatCCReuse(eval_, tmp, b, T, matrix_transformer);
}
void HEMMer::matMulPre(const CtxtTensor &a, std::vector<Ciphertext> &tmp, u64 T) const {
    const u64 slots = u64(1) << log_slots_;
    ensureRotationKeys(transformRotations(MaskKind::Horizontal, a.getBlockWidth()));
    if (fused_) {
        ensureRotationKeys(fusedRotations(a.getShape(), log_slots_, false, false));
        multMatMatPreFused(eval_, a, tmp, T, matrix_transformer, batch_);
        return;
    }
    ensureRotationKeys({1, slots - (u64)a.getHeight()});
    multMatMatPre(eval_, a, tmp, T, matrix_transformer);
}
CtxtTensor HEMMer::matMulReUse(const std::vector<Ciphertext> &tmp, const PtxtTensor &b, u64 T) const {
    return multMatMatReUse(eval_, tmp, b, T, matrix_transformer);
}
CtxtTensor HEMMer::matMulPreRev(const CtxtTensor &b, u64 T) const {
    ensureRotationKeys(transformRotations(MaskKind::Vertical, b.getBlockWidth()));
    if (fused_ && b.getLevel() >= T + 2) {
        CtxtTensor res(b);
        res.get() = matrix_transformer.lowerAndTransformFused(eval_, b.get(), MaskKind::Vertical, b.getShape(), T + 1);
        return res;
    }
    return multMatMatPreRev(eval_, b, T, matrix_transformer);
}
CtxtTensor HEMMer::matMulCCReUse(const std::vector<Ciphertext> &tmp, const CtxtTensor &b, u64 T) const {
    if (fused_ && tmp.size() > 1) {
        const u64 step = (u64)b.getBlockWidth();
        std::vector<u64> rots;
        for (size_t k = 1; k < tmp.size(); k++) rots.push_back((k * step) % (u64(1) << log_slots_));
        ensureRotationKeys(rots);
        return multMatMatCCReUseFused(eval_, tmp, b, step, false, batch_);
    }
    ensureRotationKeys({(u64)b.getBlockWidth()});
    return multMatMatCCReUse(eval_, tmp, b, T, matrix_transformer);
}

// ---- LoRA low-rank path --------------------------------------------------------------------------------------
std::vector<u64> HEMMer::transformRotations(MaskKind kind, const TileTensorShape &shape) const {
    const u64 slots = u64(1) << log_slots_;
    if (fused_ && shape.getNumRows() == shape.getNumCols())   // the batched products may take the two-stage form
        ensureRotationKeys(MatrixTransformer::twoStageRotations(kind, shape, log_slots_));
    const bool vertical = kind == MaskKind::Vertical;
    const i64 rows = shape.getNumRows(), cols = shape.getNumCols(), step = vertical ? shape.getBlockWidth() : 1;
    const i64 units = vertical ? rows : cols, sub = std::min(rows, cols);
    const i64 bs = (i64)std::ceil(std::sqrt((double)(2 * sub - 1))), gs = (i64)std::ceil((double)(sub - 1) / (double)bs);
    std::vector<u64> r;
    auto left = [&](i64 v) { r.push_back((u64)(((v % (i64)slots) + (i64)slots) % (i64)slots)); };
    for (i64 j = 0; j < (fused_ ? bs : 1); j++) left((j + 1) * step);   // hoisted baby steps are direct rotations
    for (i64 i = 0; i < gs; i++) {
        left(-(units - i * bs) * step);
        if (i > 0) left(i * bs * step);
    }
    return r;
}
void HEMMer::ensureLogStepKeys(i64 first, i64 bound, i64 unit) const {
    const u64 slots = u64(1) << log_slots_;
    std::vector<u64> r;
    for (i64 i = first; i < bound; i <<= 1) {
        const u64 v = (u64)(i * unit) % slots;
        r.push_back(v);
        r.push_back((slots - v) % slots);
    }
    ensureRotationKeys(r);
}
CtxtTensor HEMMer::matMulHighLow(const CtxtTensor &a, const CtxtTensor &b, u64 in_col_block, u64 T) const {
    const u64 slots = u64(1) << log_slots_;
    const i64 w = b.getBlockWidth();
    ensureRotationKeys(transformRotations(MaskKind::Horizontal, a.getShape()));
    ensureRotationKeys(transformRotations(MaskKind::Vertical, TileTensorShape(b.getHeight(), LOW_DIM, w)));
    ensureLogStepKeys(LOW_DIM, w / 2, 1);
    ensureLogStepKeys(LOW_DIM, w / 2, w);
    ensureRotationKeys({1, (u64)w, slots - (u64)(w / 2), (slots - (u64)(a.getHeight() * w) % slots) % slots});
    return multMatMatHighLow(eval_, a, b, in_col_block, T, matrix_transformer, LOW_DIM, fused_);
}
CtxtTensor HEMMer::matMulLowHigh(const CtxtTensor &a, const CtxtTensor &b, u64 in_row_block, u64 T) const {
    const u64 slots = u64(1) << log_slots_;
    const i64 w = a.getBlockWidth();
    ensureRotationKeys(transformRotations(MaskKind::Horizontal, a.getShape()));
    ensureRotationKeys(transformRotations(MaskKind::Vertical, b.getShape()));
    ensureLogStepKeys(LOW_DIM, w / 2, w);
    ensureRotationKeys({1, (u64)w, slots - (u64)(w / 2), (slots - (u64)(a.getHeight() * w) % slots) % slots});
    return multMatMatLowHigh(eval_, a, b, in_row_block, T, matrix_transformer, LOW_DIM, fused_);
}
CtxtTensor HEMMer::matMulLowLow(const CtxtTensor &a, const CtxtTensor &b, u64 in_col_block, u64 in_row_block,
                                u64 T) const {
    const u64 slots = u64(1) << log_slots_;
    const i64 w = a.getBlockWidth();
    ensureRotationKeys(transformRotations(MaskKind::Horizontal, TileTensorShape(a.getHeight(), LOW_DIM, w)));
    ensureRotationKeys(transformRotations(MaskKind::Vertical, TileTensorShape(LOW_DIM, b.getWidth(), w)));
    ensureLogStepKeys(LOW_DIM, w / 2, 1);
    ensureLogStepKeys(LOW_DIM, w / 2, w);
    ensureRotationKeys({1, (u64)w, slots - (u64)(w / 2), (slots - (u64)(a.getHeight() * w) % slots) % slots});
    return multMatMatLowLow(eval_, a, b, in_col_block, in_row_block, T, matrix_transformer, LOW_DIM, fused_);
}

namespace {
// ones on columns [block * low, (block + 1) * low) of the first tile (or of every tile of width `cols`) in `rows` rows
Message lowColBlockMask(u64 log_slots, u64 rows, u64 cols, u64 w, u64 block, u64 low, bool every_tile) {
    Message m(log_slots, 0);
    for (u64 i = 0; i < rows; i++)
        for (u64 k = 0; k < (every_tile ? w : 1); k += cols)
            for (u64 j = block * low; j < (block + 1) * low; j++) m[i * w + k + j] = 1;
    return m;
}
// ones on rows [block * low, (block + 1) * low), columns [0, width)
Message lowRowBlockMask(u64 log_slots, u64 w, u64 block, u64 low, u64 width) {
    Message m(log_slots, 0);
    for (u64 i = block * low; i < (block + 1) * low; i++)
        for (u64 j = 0; j < width; j++) m[i * w + j] = 1;
    return m;
}
}  // namespace

CtxtTensor HEMMer::repackToOneCol(const CtxtTensor &t, u64 out_col_block) const {
    const u64 rows = (u64)t.getHeight(), cols = (u64)t.getWidth(), w = (u64)t.getBlockWidth();
    ensureLogStepKeys(LOW_DIM, (i64)w, 1);
    ensureLogStepKeys((i64)cols, (i64)cols + 1, 1);
    Ciphertext tmp(context_);
    CtxtTensor ret{t};
    u64 pos = out_col_block;
    for (u64 i = LOW_DIM; i < w; i <<= 1) {
        if (pos % 2 == 0)
            eval_.leftRotate(ret.get(), i, tmp);
        else
            eval_.rightRotate(ret.get(), i, tmp);
        eval_.add(ret.get(), tmp, ret.get());
        pos /= 2;
    }
    eval_.mult(ret.get(), lowColBlockMask(log_slots_, rows, cols, w, out_col_block, LOW_DIM, false), ret.get());
    for (u64 i = cols; i < w; i <<= 1) {   // copy to the other tiles of the row
        eval_.rightRotate(ret.get(), cols, tmp);
        eval_.add(ret.get(), tmp, ret.get());
    }
    return ret;
}
CtxtTensor HEMMer::repackToMultiCol(const CtxtTensor &t, u64 out_col_block) const {
    const u64 rows = (u64)t.getHeight(), cols = (u64)t.getWidth(), w = (u64)t.getBlockWidth();
    ensureLogStepKeys(LOW_DIM, (i64)(w / 2), 1);
    Ciphertext tmp(context_);
    CtxtTensor ret{t};
    u64 pos = out_col_block;
    for (u64 i = LOW_DIM; i < w / 2; i <<= 1) {
        if (pos % 2 == 0)
            eval_.leftRotate(ret.get(), i, tmp);
        else
            eval_.rightRotate(ret.get(), i, tmp);
        eval_.add(ret.get(), tmp, ret.get());
        pos /= 2;
    }
    eval_.mult(ret.get(), lowColBlockMask(log_slots_, rows, cols, w, out_col_block, LOW_DIM, true), ret.get());
    return ret;
}
CtxtTensor HEMMer::repackToOneRow(const CtxtTensor &t, u64 out_row_block) const {
    const u64 rows = (u64)t.getHeight(), cols = (u64)t.getWidth(), w = (u64)t.getBlockWidth();
    ensureLogStepKeys(LOW_DIM, (i64)rows, (i64)w);
    ensureLogStepKeys((i64)cols, (i64)cols + 1, 1);
    Ciphertext tmp(context_);
    CtxtTensor ret{t};
    u64 pos = out_row_block;
    for (u64 i = LOW_DIM; i < rows; i <<= 1) {
        if (pos % 2 == 0)
            eval_.leftRotate(ret.get(), i * w, tmp);
        else
            eval_.rightRotate(ret.get(), i * w, tmp);
        eval_.add(ret.get(), tmp, ret.get());
        pos /= 2;
    }
    for (u64 i = cols; i < w; i <<= 1) {   // sum the tiles of the row
        eval_.leftRotate(ret.get(), cols, tmp);
        eval_.add(ret.get(), tmp, ret.get());
    }
    eval_.mult(ret.get(), lowRowBlockMask(log_slots_, w, out_row_block, LOW_DIM, cols), ret.get());
    for (u64 i = cols; i < w; i += cols) {   // copy to the other tiles
        eval_.rightRotate(ret.get(), cols, tmp);
        eval_.add(ret.get(), tmp, ret.get());
    }
    return ret;
}
CtxtTensor HEMMer::repackToMultiRow(const CtxtTensor &t, u64 out_row_block) const {
    const u64 rows = (u64)t.getHeight(), w = (u64)t.getBlockWidth();
    ensureLogStepKeys(LOW_DIM, (i64)rows, (i64)w);
    Ciphertext tmp(context_);
    CtxtTensor ret{t};
    u64 pos = out_row_block;
    for (u64 i = LOW_DIM; i < rows; i <<= 1) {
        if (pos % 2 == 0)
            eval_.leftRotate(ret.get(), i * w, tmp);
        else
            eval_.rightRotate(ret.get(), i * w, tmp);
        eval_.add(ret.get(), tmp, ret.get());
        pos /= 2;
    }
    eval_.mult(ret.get(), lowRowBlockMask(log_slots_, w, out_row_block, LOW_DIM, w), ret.get());
    return ret;
}
CtxtTensor HEMMer::getLowColBlock(const CtxtTensor &t, u64 col_block) const {
    CtxtTensor res{t};
    eval_.mult(t.get(),
               lowColBlockMask(log_slots_, (u64)t.getHeight(), (u64)t.getWidth(), (u64)t.getBlockWidth(), col_block,
                               LOW_DIM, true),
               res.get());
    return res;
}
CtxtTensor HEMMer::getLowRowBlock(const CtxtTensor &t, u64 row_block) const {
    CtxtTensor res{t};
    eval_.mult(t.get(), lowRowBlockMask(log_slots_, (u64)t.getBlockWidth(), row_block, LOW_DIM, (u64)t.getBlockWidth()),
               res.get());
    return res;
}
CtxtTensor HEMMer::repack_loraOpti(CtxtTensor &t1, CtxtTensor &t2) const {
    const u64 slots = u64(1) << log_slots_, n = (u64)dim_;
    ensureRotationKeys({n, slots - n});
    CtxtTensor out(t1), tmp(t2);
    if (t1.get().getRescaleCounter() > 0) eval_.rescale(t1.get());
    if (t2.get().getRescaleCounter() > 0) eval_.rescale(t2.get());
    eval_.conjugate(t1.get(), out.get());
    eval_.add(t1.get(), out.get(), out.get());
    eval_.conjugate(t2.get(), tmp.get());
    eval_.add(t2.get(), tmp.get(), tmp.get());
    eval_.multImagUnit(tmp.get(), tmp.get());
    eval_.add(out.get(), tmp.get(), out.get());
    eval_.leftRotate(out.get(), n, tmp.get());
    eval_.add(out.get(), tmp.get(), out.get());
    CtxtTensor conj(out);
    eval_.conjugate(out.get(), conj.get());
    eval_.add(out.get(), conj.get(), out.get());
    eval_.sub(conj.get(), tmp.get(), tmp.get());
    eval_.multImagUnit(tmp.get(), tmp.get());
    const Plaintext &m = cachedMask(MASK_MATMUL_HALF, out.getLevel());
    eval_.mult(tmp.get(), m, tmp.get());
    eval_.mult(out.get(), m, out.get());
    eval_.rightRotate(tmp.get(), n, tmp.get());
    addInplace(out, tmp);
    return out;
}

// ---- rank-2 LoRA through element-wise products ---------------------------------------------------------------
void HEMMer::maskFirstRowInplace(CtxtTensor &tensor) const {
    eval_.mult(tensor.get(), selectorMask(SEL_FIRST_ROW, tensor.getLevel()), tensor.get());
}
void HEMMer::maskFirstColOnlyInplace(CtxtTensor &tensor) const {
    eval_.mult(tensor.get(), selectorMask(SEL_FIRST_COL_LEFT_TILE, tensor.getLevel()), tensor.get());
}
// rows 2i and 2i+1 of the weight tile, each moved to row 0, masked and copied to every row
std::vector<std::vector<CtxtTensor>> HEMMer::splitWeightRows(const CtxtTensor &weight, u64 count) const {
    const u64 w = (u64)weight.getBlockWidth(), n = (u64)dim_;
    std::vector<u64> rots{w};
    for (u64 i = 1; i < count; i++) rots.push_back(i * 2 * w);
    ensureRotationKeys(rots);
    if (!(fused_ && (n & (n - 1)) == 0)) ensureLogStepKeys(1, (i64)n, (i64)w);
    std::vector<std::vector<CtxtTensor>> out;
    CtxtTensor tmp{weight};
    for (u64 i = 0; i < count; i++) {
        if (i > 0) eval_.leftRotate(weight.get(), i * 2 * w, tmp.get());
        std::vector<CtxtTensor> pair{tmp, tmp};
        maskFirstRowInplace(pair[0]);
        eval_.leftRotate(pair[1].get(), w, pair[1].get());
        maskFirstRowInplace(pair[1]);
        out.push_back(std::move(pair));
    }
    if (fused_ && (n & (n - 1)) == 0) {   // row 0 copied to every row: all 2 * count tensors through the same launch chains
        ensureRotationKeys(rotateSumRotations(-(i64)w, n, log_slots_));
        std::vector<RotateSumJob> jobs;
        for (auto &pair : out)
            for (auto &x : pair) jobs.push_back({&x.get(), -(i64)w, &x.get()});
        rotateSumFused(eval_, jobs, n);
        return out;
    }
    Ciphertext t(context_);
    for (auto &pair : out)
        for (auto &x : pair)
            for (u64 rot = 1; rot < n; rot <<= 1) {
                eval_.rightRotate(x.get(), rot * w, t);
                eval_.add(x.get(), t, x.get());
            }
    return out;
}
std::vector<CtxtTensor> HEMMer::loraRank2Down(const std::vector<CtxtTensor> &cur, const CtxtTensor &lora_wa,
                                              u64 weight_level) const {
    if (cur.empty()) throw std::invalid_argument("[loraRank2Down] no activation tiles");
    const u64 w = (u64)lora_wa.getBlockWidth();
    CtxtTensor wa{lora_wa};
    eval_.levelDown(wa.get(), weight_level, wa.get());
    auto weights = splitWeightRows(wa, cur.size());
    if (!(fused_ && (w & (w - 1)) == 0)) ensureLogStepKeys(1, (i64)w, 1);
    std::vector<CtxtTensor> out;
    Ciphertext t(context_);
    for (u64 j = 0; j < 2; j++) {
        CtxtTensor acc{wa};
        eval_.mult(cur[0].get(), weights[0][j].get(), acc.get());
        for (size_t i = 1; i < cur.size(); i++) {
            eval_.mult(cur[i].get(), weights[i][j].get(), t);
            eval_.add(acc.get(), t, acc.get());
        }
        if (fused_ && (w & (w - 1)) == 0) {
            ensureRotationKeys(rotateSumRotations(1, w, log_slots_));
            rotateSumFused(eval_, {{&acc.get(), 1, &acc.get()}}, w);
        } else {
            for (u64 rot = 1; rot < w; rot <<= 1) {
                eval_.leftRotate(acc.get(), rot, t);
                eval_.add(acc.get(), t, acc.get());
            }
        }
        maskFirstColOnlyInplace(acc);
        out.push_back(std::move(acc));
    }
    return out;
}
std::vector<CtxtTensor> HEMMer::loraRank2Up(const std::vector<CtxtTensor> &xa_in, const CtxtTensor &lora_wb, u64 n_out,
                                            u64 weight_level) const {
    if (xa_in.size() != 2) throw std::invalid_argument("[loraRank2Up] two column ciphertexts are needed");
    const u64 w = (u64)lora_wb.getBlockWidth();
    CtxtTensor wb{lora_wb};
    eval_.levelDown(wb.get(), weight_level, wb.get());
    auto weights = splitWeightRows(wb, n_out);
    if (!(fused_ && (w & (w - 1)) == 0)) ensureLogStepKeys(1, (i64)w, 1);
    std::vector<CtxtTensor> xa{xa_in};
    Ciphertext t(context_);
    if (fused_ && (w & (w - 1)) == 0 && xa[0].getLevel() == xa[1].getLevel() &&
        xa[0].get().getRescaleCounter() == xa[1].get().getRescaleCounter()) {
        ensureRotationKeys(rotateSumRotations(-1, w, log_slots_));
        rotateSumFused(eval_, {{&xa[0].get(), -1, &xa[0].get()}, {&xa[1].get(), -1, &xa[1].get()}}, w);
    } else {
        for (auto &x : xa)
            for (u64 rot = 1; rot < w; rot <<= 1) {
                eval_.rightRotate(x.get(), rot, t);
                eval_.add(x.get(), t, x.get());
            }
    }
    std::vector<CtxtTensor> out;
    for (u64 i = 0; i < n_out; i++) {
        CtxtTensor y{wb};
        eval_.mult(xa[0].get(), weights[i][0].get(), y.get());
        eval_.mult(xa[1].get(), weights[i][1].get(), t);
        eval_.add(y.get(), t, y.get());
        out.push_back(std::move(y));
    }
    return out;
}

// x + conj(x) = 2 Re(x)
CtxtTensor HEMMer::repackCC(CtxtTensor &t) const {
    CtxtTensor out(t);
    eval_.conjugate(t.get(), out.get());
    eval_.add(t.get(), out.get(), out.get());
    return out;
}
PtxtTensor HEMMer::complexPacking(const PtxtTensor &a, const PtxtTensor &b) const {
    // 0.5 a - 0.5 i b on the decoded values
    Message ma = endec_.decode(a.get()), mb = endec_.decode(b.get());
    for (u64 i = 0; i < ma.getSize(); i++) ma[i] = 0.5 * ma[i] - Complex(0, 0.5) * mb[i];
    return PtxtTensor(a.getShape(), endec_.encode(ma, std::min(a.getLevel(), b.getLevel())));
}
CtxtTensor HEMMer::complexPacking(const CtxtTensor &a, const CtxtTensor &b) const {
    CtxtTensor res(b);
    eval_.multImagUnit(b.get(), res.get());
    eval_.add(a.get(), res.get(), res.get());
    return res;
}
CtxtTensor HEMMer::complexPackingRev(const CtxtTensor &a, const CtxtTensor &b) const {
    CtxtTensor res(b);
    eval_.multImagUnit(b.get(), res.get());
    eval_.sub(a.get(), res.get(), res.get());
    return res;
}
CtxtTensor HEMMer::repack_notBTS(CtxtTensor &t1, CtxtTensor &t2) const {
    const u64 slots = u64(1) << log_slots_, n = (u64)dim_;
    ensureRotationKeys({n, slots - n});
    CtxtTensor out(t1), tmp(t2);
    if (t1.get().getRescaleCounter() > 0) eval_.rescale(t1.get());
    if (t2.get().getRescaleCounter() > 0) eval_.rescale(t2.get());
    eval_.conjugate(t1.get(), out.get());
    eval_.add(t1.get(), out.get(), out.get());
    eval_.conjugate(t2.get(), tmp.get());
    eval_.add(t2.get(), tmp.get(), tmp.get());
    eval_.multImagUnit(tmp.get(), tmp.get());
    eval_.add(out.get(), tmp.get(), out.get());
    eval_.leftRotate(out.get(), n, tmp.get());
    eval_.add(out.get(), tmp.get(), out.get());
    const Plaintext &m = cachedMask(MASK_MATMUL, out.getLevel());
    eval_.mult(tmp.get(), m, tmp.get());
    eval_.mult(out.get(), m, out.get());
    eval_.rightRotate(tmp.get(), n, tmp.get());
    addInplace(out, tmp);
    return out;
}
CtxtTensor HEMMer::repack(CtxtTensor &t1, CtxtTensor &) const {
    Ciphertext dummy(context_);
    btp_.bootstrapExtended(t1.get(), dummy);  // throws: bootstrapping is outside this build
    return t1;
}

}  // namespace HELLM

// HEMMer: owns the context, keys and evaluator and exposes the matrix-multiplication entry points
// (reference: ciphertext/include/HELLM/HEMMer.hpp:33-351, matmul / packing / codec part).
// Where the reference takes torch::Tensor, this build takes a plain row-major Matrix of doubles:
// tensors are only a container on that path (HEMMer.cpp:232-275 copy them straight into a Message).
//
// Tile side n is fixed by the ring: n * n * 2 = N / 2 slots (n = 128 for N = 2^16, the reference's
// ModelArgs::HEAD_DIM).  "Single" layout: one n x n tile in rows of n slots (lower half of the slot
// vector).  "Pair" layout: two tiles side by side in rows of 2n slots (all slots).
#pragma once
#include <map>
#include <set>
#include <string>
#include <vector>

#include "HELLM/MatrixUtils.hpp"

namespace HELLM {

struct Matrix {
    i64 rows = 0, cols = 0;
    std::vector<double> v;  // row-major
    Matrix() = default;
    Matrix(i64 r, i64 c, double fill = 0.0) : rows(r), cols(c), v((size_t)(r * c), fill) {}
    double &at(i64 r, i64 c) { return v[(size_t)(r * cols + c)]; }
    double at(i64 r, i64 c) const { return v[(size_t)(r * cols + c)]; }
};

void cleanUpMatrixTransformer();

class HEMMer final {
public:
    static HEMMer genHEMMer(int device_id = 0, ParameterPreset preset = ParameterPreset::FGb,
                            const bool is_multi_gpu = false);
    explicit HEMMer(int device_id = 0, ParameterPreset preset = ParameterPreset::FGb);
    // any context (small rings for tests); min_bootstrap_level feeds the level checks
    HEMMer(const Context &context, u64 min_bootstrap_level);
    HEMMer(const std::string &key_path, int device_id = 0, ParameterPreset preset = ParameterPreset::FGb);
    ~HEMMer();
    HEMMer(const HEMMer &) = delete;

    const Context &getContext() const { return context_; }
    const HomEvaluator &getEval() const { return eval_; }
    const Bootstrapper &getBtp() const { return btp_; }
    const EnDecoder &getEnDec() const { return endec_; }
    const Decryptor &getDec() const { return dec_; }
    const SecretKey &getsk() const { return sk_; }
    i64 dim() const { return dim_; }
    const KeyPack &keyPack() const { return pack_; }
    // sigma / tau on their own (MatrixTransformer::diagonalToColumn / diagonalToRow with this HEMMer's keys)
    CtxtTensor diagonalToColumn(const CtxtTensor &a) const;
    CtxtTensor diagonalToRow(const CtxtTensor &b) const;

    void save(const std::string &keys_path);

    Message message2(const Matrix &a, const Matrix &b) const;
    PtxtTensor encode(const Matrix &data, u64 level = 0) const;
    PtxtTensor encode2(const Matrix &a, const Matrix &b, u64 level = 0) const;
    Message msgDiagonalToRow4(const Matrix &w1, const Matrix &w2, const Matrix &w3, const Matrix &w4) const;
    // Rotate-and-sum reductions on the pair layout (reference src/HEMMer.cpp):
    //   reduceRowSumWithScaledMask :2512-2530  sum every tile row over the block width (log-step left rotations),
    //                                          multiply by `mask`, spread the kept values back over the row
    //                                          (log-step right rotations);
    //   oneMatRotSumInplace :882-919           row sums of a over half a row into column 0 / of b into the last
    //                                          column, masked and spread over the whole row;
    //   maskRightLeft :1245-1249, maskFirstColInplace :1251-1253;
    //   rowMoments                             the first half of LayerNorm :1699-1760: over a list of tiles,
    //                                          mean and mean of squares of every token row (scaled by `inv_count`
    //                                          in column 0, then spread over the row), one level each.
    void reduceRowSumWithScaledMask(CtxtTensor &tensor, const Message &mask) const;
    void oneMatRotSumInplace(CtxtTensor &tensor_a, CtxtTensor &tensor_b) const;
    void maskRightLeft(const CtxtTensor &tensor, CtxtTensor &out_left, CtxtTensor &out_right) const;
    void maskFirstColInplace(CtxtTensor &tensor) const;
    void rowMoments(const std::vector<CtxtTensor> &tiles, Real inv_count, CtxtTensor &mean, CtxtTensor &mean_square) const;

    // Weight store (reference HEMMer::encodeWeight, src/HEMMer.cpp:437-482, and TransformerBlock::getWeight,
    // src/TransformerBlock.cpp:11009-11031).  A weight given as a height x width grid of tiles is written as
    //   <save_path><i>_<j>.msg = msgDiagonalToRow4(tile[4i][j], tile[4i+1][j], tile[4i+2][j], tile[4i+3][j])
    // (the last group takes tiles height-2, height-1 and two zero tiles when height is not a multiple of 4);
    // a list of tiles is written pairwise as <save_path><i>.msg = message2(tile[2i], tile[2i+1]).
    // File format (this build's own; HEaaN's is closed): u64 log_slots, then 2^log_slots complex128 values.
    void encodeWeight(const std::vector<std::vector<Matrix>> &grid, const std::string &save_path) const;
    void encodeWeight(const std::vector<Matrix> &tiles, const std::string &save_path) const;
    // reads one .msg file and encodes it at `level` as a pair-layout plaintext tile
    PtxtTensor getWeight(const std::string &file, u64 level) const;
    // ciphertext store: u64 {polynomials, level, rescale counter, N, rows, cols, block width}, then the residues
    void saveCtxtTensor(const CtxtTensor &t, const std::string &file) const;
    CtxtTensor loadCtxtTensor(const std::string &file) const;
    PtxtTensor encodeDiagonalToRow4(const Matrix &w1, const Matrix &w2, const Matrix &w3, const Matrix &w4,
                                    u64 level = 0) const;
    CtxtTensor encrypt(const Matrix &data) const;
    CtxtTensor encrypt2(const Matrix &a, const Matrix &b) const;
    Matrix decrypt(const CtxtTensor &t) const;
    std::vector<Matrix> decrypt2(const CtxtTensor &t) const;

    template <class T>
    void addInplace(CtxtTensor &a, const HETensor<T> &b) const {
        eval_.add(a.get(), b.get(), a.get());
    }
    template <class T>
    void hadamardMultInplace(CtxtTensor &a, const HETensor<T> &b) const {
        eval_.mult(a.get(), b.get(), a.get());
    }

    void transposeInplace(CtxtTensor &t, u64 target_level = 0) const;
    void complexPackingInplace(CtxtTensor &t) const;
    void complexPackingRowInplace(CtxtTensor &t) const;
    void transposeComplexPackingInplace(CtxtTensor &t, u64 target_level = 0) const;
    void splitInTwo(CtxtTensor &t, CtxtTensor &t1, CtxtTensor &t2) const;

    CtxtTensor packedMatMul(const CtxtTensor &a, const CtxtTensor &b, u64 target_level = 4) const;
    CtxtTensor packedMatMulPre(const CtxtTensor &a, u64 target_level = 4) const;
    void packedMatMulPreRot(const CtxtTensor &a, std::vector<Ciphertext> &tmp, u64 target_level = 4) const;
    CtxtTensor packedMatMulPreRev(const CtxtTensor &b, u64 target_level = 4) const;
    CtxtTensor packedMatMulCCReuse(const std::vector<Ciphertext> &tmp, const CtxtTensor &b,
                                   u64 target_level = 4) const;
    CtxtTensor singleMatMul(const CtxtTensor &a, const PtxtTensor &b, u64 target_level = 4) const;
    CtxtTensor singleCCMatMul(const CtxtTensor &a, const CtxtTensor &b, u64 target_level = 4) const;

    CtxtTensor repackCC(CtxtTensor &t) const;
    PtxtTensor complexPacking(const PtxtTensor &a, const PtxtTensor &b) const;
    CtxtTensor complexPacking(const CtxtTensor &a, const CtxtTensor &b) const;
    CtxtTensor complexPackingRev(const CtxtTensor &a, const CtxtTensor &b) const;
    CtxtTensor repack(CtxtTensor &t1, CtxtTensor &t2) const;         // needs bootstrapping: throws
    CtxtTensor repack_notBTS(CtxtTensor &t1, CtxtTensor &t2) const;

    void matMulPre(const CtxtTensor &a, std::vector<Ciphertext> &tmp, u64 target_level = 4) const;
    CtxtTensor matMulReUse(const std::vector<Ciphertext> &tmp, const PtxtTensor &b, u64 target_level = 4) const;
    CtxtTensor matMulPreRev(const CtxtTensor &b, u64 target_level = 4) const;
    CtxtTensor matMulCCReUse(const std::vector<Ciphertext> &tmp, const CtxtTensor &b, u64 target_level = 4) const;

    // LoRA low-rank path (reference src/HEMMer.cpp:2111-2332, 1055-1091; products in MatrixUtils.cpp:1681-1996).
    // A rank-`LOW_DIM` factor occupies LOW_DIM columns (or rows) of a tile, at column (row) block `block`:
    //   getLowColBlock / getLowRowBlock   keep that block of every tile;
    //   matMulHighLow(a, b, in_col_block) partial sums of A x B_low spread over the column blocks;
    //   matMulLowHigh(a, b, in_row_block) A_low x B, partial sums spread over the row blocks;
    //   matMulLowLow(a, b, col, row)      (rows x LOW_DIM) x (LOW_DIM x cols), complete product;
    //   repackToOneCol / OneRow           sum the partial sums of all blocks (both tiles of the pair layout
    //                                     included) into block `out_block`, copied to every tile;
    //   repackToMultiCol / MultiRow       the same per tile, without the copy.
    CtxtTensor matMulHighLow(const CtxtTensor &a, const CtxtTensor &b, u64 in_col_block, u64 target_level) const;
    CtxtTensor matMulLowHigh(const CtxtTensor &a, const CtxtTensor &b, u64 in_row_block, u64 target_level) const;
    CtxtTensor matMulLowLow(const CtxtTensor &a, const CtxtTensor &b, u64 in_col_block, u64 in_row_block,
                            u64 target_level = 4) const;
    CtxtTensor repackToOneCol(const CtxtTensor &t, u64 out_col_block) const;
    CtxtTensor repackToMultiCol(const CtxtTensor &t, u64 out_col_block) const;
    CtxtTensor repackToOneRow(const CtxtTensor &t, u64 out_row_block) const;
    CtxtTensor repackToMultiRow(const CtxtTensor &t, u64 out_row_block) const;
    CtxtTensor getLowColBlock(const CtxtTensor &t, u64 col_block) const;
    CtxtTensor getLowRowBlock(const CtxtTensor &t, u64 row_block) const;
    // repack of two un-rescaled product halves used by the LoRA path (src/HEMMer.cpp:1055-1091)
    CtxtTensor repack_loraOpti(CtxtTensor &t1, CtxtTensor &t2) const;

    // Rank-2 LoRA through element-wise products, the form the reference's layers run
    // (src/TransformerBlock.cpp:2199-2365).  Row 2i+j of the weight tile `lora_wa` holds column j of A for the i-th
    // pair of activation tiles, row 2i+j of `lora_wb` row j of B for the i-th pair of output tiles.
    //   loraRank2Down: X a_0 and X a_1, each in column 0 of the left tile (two ciphertexts);
    //   loraRank2Up:   (X A) B as n_out pair-layout ciphertexts.
    // The weights are first brought to `weight_level` (9 and 6 in the reference).
    std::vector<CtxtTensor> loraRank2Down(const std::vector<CtxtTensor> &cur, const CtxtTensor &lora_wa,
                                          u64 weight_level = 9) const;
    std::vector<CtxtTensor> loraRank2Up(const std::vector<CtxtTensor> &xa, const CtxtTensor &lora_wb, u64 n_out,
                                        u64 weight_level = 6) const;
    void maskFirstRowInplace(CtxtTensor &tensor) const;       // src/HEMMer.cpp:1259-1261
    void maskFirstColOnlyInplace(CtxtTensor &tensor) const;   // src/HEMMer.cpp:1255-1257 (left tile only)

    // Schedule of singleCCMatMul / packedMatMul / matMulPre: batched launches with hoisted rotations
    // (default) or one evaluator call per step in the reference's order.  `batch` = shifts per launch.
    void setFused(bool on, u64 batch = 16) {
        fused_ = on;
        batch_ = batch;
        // the batched schedules read rotation keys through the hoisted sums only: keys derived from now on are kept in
        // the compact form (KeyPack::compactKey), one plain form at a time while they are generated
        pack_.compact_on_generate_ = on;
    }
    bool fused() const { return fused_; }
    // Promise that the operands of singleCCMatMul hold a single tile block (as HEMMer::encrypt produces) and nothing
    // in the rest of the slot vector; see multMatMatFused.  Off by default.  Without the promise the same route is
    // taken when it is known from the operands themselves: Encryptor::encrypt records how many slots of the
    // plaintext were non-zero and the slot-wise evaluator operations carry that along (Ciphertext::occupiedSlots).
    void assumeSingleTile(bool on) { single_tile_ = on; }

    // generate (once) the direct rotation keys a routine needs; rotations are left shifts in slots
    void ensureRotationKeys(const std::vector<u64> &left_rotations) const;
    size_t rotationKeyCount() const { return have_rot_.size(); }

private:
    void init();
    const Plaintext &cachedMask(int id, u64 level) const;
    // the 0/1 masks of the reductions and the rank-2 LoRA path (column 0, column n-1, left / right half of the columns,
    // row 0; on both tiles of the pair layout or on the left one only), encoded once per level
    const Plaintext &selectorMask(int which, u64 level) const;
    std::vector<u64> transformRotations(MaskKind kind, i64 width) const;
    // the same for a (possibly rectangular) sigma / tau shape under the current schedule
    std::vector<u64> transformRotations(MaskKind kind, const TileTensorShape &shape) const;
    void ensureLogStepKeys(i64 first, i64 bound, i64 unit) const;
    std::vector<std::vector<CtxtTensor>> splitWeightRows(const CtxtTensor &weight, u64 count) const;   // +-i*unit for i = first, 2 first, ... < bound

    int device_id_ = 0;
    Context context_;
    u64 log_slots_;
    i64 dim_;
    SecretKey sk_;
    Encryptor enc_;
    Decryptor dec_;
    EnDecoder endec_;
    mutable KeyPack pack_;
    HomEvaluator eval_;
    Bootstrapper btp_;
    Message col_mask_even_, row_mask_even_, mask_left_half_, mask_matmul_, mask_matmul_half_;
    mutable std::map<std::pair<int, u64>, Plaintext> mask_cache_;
    mutable std::set<u64> have_rot_;
    bool fused_ = true, single_tile_ = false;
    u64 batch_ = 16;
};

}  // namespace HELLM

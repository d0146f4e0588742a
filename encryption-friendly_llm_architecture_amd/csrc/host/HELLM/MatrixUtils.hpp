// Homomorphic matrix products on packed tiles: the sigma/tau diagonal transforms, transpose, and the
// ciphertext x ciphertext / plaintext x ciphertext multiplications built on them.
// Mirrors the call surface of the reference's ciphertext/include/HELLM/MatrixUtils.hpp:130-215
// (free functions taking the evaluator, the operands, the target level and the transformer) and the
// MatrixTransformer methods of ciphertext/src/MatrixUtils.cpp:584-1098.
//
// Slot layout: value (r, c) of a tile lives in slot r * block_width + c; tiles repeat over the whole
// slot vector, and every mask below is tiled the same way, so one ciphertext may carry several tiles.
//
// Differences from the reference that do not change the decrypted result: transform masks are
// encoded once per (kind, shape, level) and stay resident in HBM in NTT form instead of being
// re-encoded from a Message on every multiplication, and a transform sums its masked rotations
// before a single rescale instead of rescaling each term.
#pragma once
#include <map>
#include <vector>

#include "HELLM/HETensor.hpp"

namespace HELLM {

// DiagonalSigned: the transpose's diagonals grouped the way sigma / tau group theirs (positive and negative diagonals in
// separate giant-step groups), which is what the batched transform walks; Diagonal keeps the reference's grouping.
enum class MaskKind {
    Horizontal, Vertical, PackedHorizontal, PackedVertical, Diagonal, DiagonalSigned,
    // the complex packing followed by the packed transform as ONE linear map (one level instead of two): diagonal r of
    // the composite collects mask_d (.) rho^(2 d unit)(M_e) over 2 d + e = r, e in {0, +1, -1} the packing's three terms
    PackingHorizontal, PackingVertical
};
// The complex packing as a linear map on the slots, out = Z x + M_+ rho^(step)(x) + M_- rho^(-step)(x) (step 1 for
// columns, the block width for rows): part 0 = Z, 1 = M_+, 2 = M_-.
Message packingMaskMessage(bool by_rows, i64 block_width, u64 log_slots, int part);

// 0/1 (or 0.5) slot pattern of diagonal `idx` for a transform kind, before any pre-rotation.
// Horizontal (sigma): rows r with r mod n == idx take columns [0, n - idx); negative idx = the wrapped
// part.  Vertical (tau): the same with rows and columns swapped.  Packed kinds work on 2 x 2 cells.
// Diagonal (transpose): output positions (r, c) with r - c == idx.
Message transformMaskMessage(MaskKind kind, const TileTensorShape &shape, u64 log_slots, i64 idx);
// Slot pattern of the two-stage transforms: stage 1 selects the rows (sigma) / columns (tau) whose cell index is r
// mod b, stage 2 those whose cell index div b is r; part 0: all of them, 1: the positions that do not wrap under the
// stage's rotation (r cells, or r b cells), 2: those that do.  b = twoStageSplit(cells per side).
Message twoStageMaskMessage(MaskKind kind, const TileTensorShape &shape, u64 log_slots, int stage, i64 r, int part);
i64 twoStageSplit(i64 units);   // the smallest power of two b with b * b >= units

class MatrixTransformer {
public:
    // mask `idx` of `kind`, pre-rotated for its baby-step/giant-step group and encoded at `level`
    const Plaintext &transformMask(const HomEvaluator &eval, MaskKind kind, const TileTensorShape &shape, u64 level,
                                   i64 idx);
    // assemble masks of a cyclic shift by i inside each tile row (columns) / tile column (rows):
    // [2i] selects the wrapped part, [2i+1] its complement; encoded at `level`
    std::vector<Plaintext> &getColMask(const HomEvaluator &eval, const TileTensorShape &shape, u64 level);
    std::vector<Plaintext> &getRowMask(const HomEvaluator &eval, const TileTensorShape &shape, u64 level);

    template <class T>
    HETensor<T> transpose(const HomEvaluator &eval, const HETensor<T> &op);
    // sigma(A)[i, j] = A[i, (i + j) mod n]
    template <class T>
    HETensor<T> diagonalToColumn(const HomEvaluator &eval, const HETensor<T> &op);
    // tau(B)[i, j] = B[(i + j) mod n, j]
    template <class T>
    HETensor<T> diagonalToRow(const HomEvaluator &eval, const HETensor<T> &op);
    CtxtTensor packedDiagonalToColumn(const HomEvaluator &eval, const CtxtTensor &op);
    CtxtTensor packedDiagonalToRow(const HomEvaluator &eval, const CtxtTensor &op);

    // The same transforms and assemble masks for the batched launches: masks over the extended basis
    // (chain limbs + special primes) so they can be applied before ModDown.
    // first_block_only: the masks are additionally zero outside the first tile block (rows >= shape rows), which
    // clears whatever the operand carries there
    std::vector<Plaintext> &getColMaskExt(const HomEvaluator &eval, const TileTensorShape &shape, u64 level,
                                          bool first_block_only = false);
    // ones on the first tile block, zero elsewhere (ordinary plaintext at `level`)
    const Plaintext &firstBlockMask(const HomEvaluator &eval, const TileTensorShape &shape, u64 level);
    std::vector<Plaintext> &getRowMaskExt(const HomEvaluator &eval, const TileTensorShape &shape, u64 level);
    // sigma / tau / packed variants with hoisted baby steps (one ModUp, all baby rotations in one launch
    // chain) and all giant-step rotations batched and summed in the extended basis
    Ciphertext diagonalTransformFused(const HomEvaluator &eval, const Ciphertext &in, MaskKind kind,
                                      const TileTensorShape &shape);

    // the same for n_jobs operands at one level through shared launches: in [job][2][level+1][N] -> out
    // [job][2][level][N] (one level lower, rescaled)
    void diagonalTransformBatch(const HomEvaluator &eval, const u64 *in, size_t n_jobs, u64 level, const MaskKind *kinds,
                                const TileTensorShape *shapes, u64 *out);

    // Two-stage form of the same sigma / tau (square tiles): row i is rotated by i mod b in the first stage and by
    // b (i div b) in the second (b ~ sqrt(n)), each stage one mask level: in [job][2][level+1][N] -> out
    // [job][2][level-1][N], TWO levels lower.  2 (b + n/b) keyed rotations with 2 (b + n/b) masks per operand
    // instead of b + 2 n/b rotations with 2 n - 1 masks, and every stage is a single output of the hoisted launch
    // (one ModDown per stage).  Used by the batched products when the operands have a level to spare.
    // scale_levels (optional, one per job): the level whose fixed scale job q's input carries -- an operand truncated to
    // `level` from a higher one; the masks of the first stage are then encoded at Delta_(level-1) q_level /
    // Delta_(scale level), which lands the result on the fixed scale of level - 1 without a levelDown in front.
    // first_stage = 2: only the second stage; `in` is then what a first stage from `level` left at level - 1.
    void diagonalTransformTwoStage(const HomEvaluator &eval, const u64 *in, size_t n_jobs, u64 level, const MaskKind *kinds,
                                   const TileTensorShape *shapes, u64 *out, const u64 *scale_levels = nullptr,
                                   int first_stage = 1);
    // The complex packing (by rows for PackedVertical, by columns for PackedHorizontal) and the FIRST stage of the
    // two-stage transform of `kind` as one linear map on the slots -- one hoisted sum, one mask level: the term that
    // rotates by a slots carries sum over (stage rotation r, packing shift e) with r + e = a of
    // stage mask_r (.) rho^r(packing mask_e).  in [2][level+1][N] (not packed yet) -> out [2][level][N], which the
    // second stage takes to level - 1: packing and transform in two levels, for an operand with one level less than
    // packing, stage 1 and stage 2 need on their own.
    // n_jobs operands through the same launch chain, in [job][2][level+1][N] -> out [job][2][level][N].
    // scale_levels (optional, one per job; 0: `level`): the level whose fixed scale the job's input carries when it was
    // only truncated to `level`.
    void packingStageOne(const HomEvaluator &eval, const u64 *in, size_t n_jobs, u64 level, const MaskKind *kinds,
                         const TileTensorShape *shapes, u64 *out, const u64 *scale_levels = nullptr);
    // left rotations (in slots) packingStageOne uses
    static std::vector<u64> packingStageOneRotations(MaskKind kind, const TileTensorShape &shape, u64 log_slots);
    // Brings `in` down to the level a transform ending at `end_level` starts from and runs it with the batched
    // launches: two stages from end_level + 2 when the operand is that high and the tile is square, otherwise one
    // stage from end_level + 1.
    Ciphertext lowerAndTransformFused(const HomEvaluator &eval, const Ciphertext &in, MaskKind kind,
                                      const TileTensorShape &shape, u64 end_level);
    // left rotations (in slots) the two-stage transform of `kind` uses on tiles in rows of `width` slots
    static std::vector<u64> twoStageRotations(MaskKind kind, const TileTensorShape &shape, u64 log_slots);

    void cleanUp();
    size_t cachedMasks() const;
    // The caches hold masks of ONE parameter set (ring size, chain and special primes, scale factors): contexts over the
    // same set share them; the first call with a context over another set empties them.  Every cached lookup starts here.
    void useChainOf(const Context &c);

private:
    struct Key {
        int kind;
        TileTensorShape shape;
        u64 level;
        i64 idx;
        bool operator<(const Key &o) const {
            return std::tie(kind, shape, level, idx) < std::tie(o.kind, o.shape, o.level, o.idx);
        }
    };
    Ciphertext diagonalTransform(const HomEvaluator &eval, const Ciphertext &in, MaskKind kind,
                                 const TileTensorShape &shape);
    std::vector<u64> chain_;   // N, nQ, the primes and the bit patterns of the scale factors the caches belong to
    Context last_context_;     // the context of the last lookup (held, so that its address cannot be taken by another)
    std::map<Key, Plaintext> masks_;
    std::map<std::pair<TileTensorShape, u64>, std::vector<Plaintext>> col_masks_, row_masks_;
    std::map<std::pair<TileTensorShape, u64>, std::vector<Plaintext>> col_masks_ext_, row_masks_ext_, col_masks_ext_first_;
    std::map<std::pair<TileTensorShape, u64>, Plaintext> first_block_masks_;

public:
    // tau(B) of a plaintext weight over the extended basis, kept per weight: the key is a hash of the weight's
    // residues, so a weight whose content changes is prepared again.  layout: 0 = not usable by the batched product,
    // 1 = equal tile blocks, 2 = only the first block is non-zero.
    struct WeightTau {
        Plaintext tau;
        int layout;
    };
    // complexPackingInplace (rows[q] false: adjacent columns -> a + i b) / complexPackingRowInplace (true: adjacent
    // rows of rows `w` slots wide -> a - i b) of n_jobs ciphertexts at `level` through one launch chain: both
    // rotations of every job from one ModUp, masks applied in the extended basis, ModDown merged with the rescale.
    // in: [job][2][level+1][N], out: [job][2][level][N].
    // scale_levels (optional): job q is a truncated ciphertext that still carries the fixed scale of level
    // scale_levels[q] >= level; its masks absorb the change of scale (no levelDown in front)
    void complexPackingBatch(const HomEvaluator &eval, const u64 *in, size_t n_jobs, u64 level, const bool *rows, i64 w,
                             u64 *out, const u64 *scale_levels = nullptr);
    // (rows, w, level, part 0 = Z / 1 = +step / 2 = -step, level of the input's scale)
    std::map<std::tuple<int, i64, u64, int, u64>, Plaintext> pack_masks_;
    std::map<std::tuple<u64, u64, TileTensorShape, u64>, WeightTau> weight_tau_;
    std::vector<std::tuple<u64, u64, TileTensorShape, u64>> weight_tau_order_;

private:
    // (kind, shape, level, (scale level * 4 + stage) * 4096 + r * 4 + part) -> mask of the two-stage transforms; part 0 is
    // an ordinary plaintext (the unrotated rows), parts 1 / 2 (main / wrapped columns) are over the extended basis; masks
    // that absorb a change of scale (scale level != 0) are all over the extended basis
    std::map<Key, Plaintext> two_stage_masks_;
    // (kind, shape, level, 0) -> (left rotation in slots, mask over the extended basis) of packingStageOne
    std::map<Key, std::vector<std::pair<u64, Plaintext>>> packing_stage_one_masks_;
    const Plaintext &twoStageMask(const HomEvaluator &eval, MaskKind kind, const TileTensorShape &shape, u64 level,
                                  int stage, i64 r, int part, u64 from = 0);
};

// A x B for two encrypted tiles (HEMMer::singleCCMatMul); output level = target_level.
template <class T>
CtxtTensor multMatMat(const HomEvaluator &eval, const Bootstrapper &btp, const CtxtTensor &op1,
                      const HETensor<T> &op2, u64 target_level, MatrixTransformer &transformer);
// two products per call on complex-packed operands (HEMMer::packedMatMul)
CtxtTensor multPackedMatMat(const HomEvaluator &eval, const Bootstrapper &btp, const CtxtTensor &op1,
                            const CtxtTensor &op2, u64 target_level, MatrixTransformer &transformer);
CtxtTensor multPackedMatMatPre(const HomEvaluator &eval, const CtxtTensor &a, u64 target_level,
                               MatrixTransformer &transformer);
void multPackedMatMatPreRot(const HomEvaluator &eval, const CtxtTensor &a, std::vector<Ciphertext> &tmp,
                            u64 target_level, MatrixTransformer &transformer);
CtxtTensor multPackedMatMatPreRev(const HomEvaluator &eval, const CtxtTensor &b, u64 target_level,
                                  MatrixTransformer &transformer);
CtxtTensor multPackedMatMatCCReuse(const HomEvaluator &eval, const std::vector<Ciphertext> &tmp, const CtxtTensor &b,
                                   u64 target_level, MatrixTransformer &transformer);
// hoisted form: all column shifts of sigma(A) once, then one accumulation per weight tile
void multMatMatPre(const HomEvaluator &eval, const CtxtTensor &a, std::vector<Ciphertext> &tmp, u64 target_level,
                   MatrixTransformer &transformer);
CtxtTensor multMatMatReUse(const HomEvaluator &eval, const std::vector<Ciphertext> &tmp, const PtxtTensor &b,
                           u64 target_level, MatrixTransformer &transformer);
CtxtTensor multMatMatPreRev(const HomEvaluator &eval, const CtxtTensor &b, u64 target_level,
                            MatrixTransformer &transformer);
CtxtTensor multMatMatCCReUse(const HomEvaluator &eval, const std::vector<Ciphertext> &tmp, const CtxtTensor &b,
                             u64 target_level, MatrixTransformer &transformer);

// LoRA low-rank products: one operand uses only `low_dim` columns (HighLow), rows (LowHigh) or both one thin
// operand each (LowLow), sitting at the given column / row block of every tile.  `fused` runs the sigma / tau
// transforms through the batched launches; the few remaining operations are ordinary evaluator calls.
constexpr i64 LOW_DIM = 2;   // LoRA rank (reference ModelArgs.hpp:67)
CtxtTensor multMatMatHighLow(const HomEvaluator &eval, const CtxtTensor &op1, const CtxtTensor &op2, u64 in_col_block,
                             u64 target_level, MatrixTransformer &transformer, i64 low_dim = LOW_DIM,
                             bool fused = false);
CtxtTensor multMatMatLowHigh(const HomEvaluator &eval, const CtxtTensor &op1, const CtxtTensor &op2, u64 in_row_block,
                             u64 target_level, MatrixTransformer &transformer, i64 low_dim = LOW_DIM,
                             bool fused = false);
CtxtTensor multMatMatLowLow(const HomEvaluator &eval, const CtxtTensor &op1, const CtxtTensor &op2, u64 in_col_block,
                            u64 in_row_block, u64 target_level, MatrixTransformer &transformer, i64 low_dim = LOW_DIM,
                            bool fused = false);

// Batched schedules of the same products (same decrypted results, far fewer and larger launches):
// every column / row shift of the main loop is a direct hoisted rotation of sigma(A) / tau(B) (one ModUp
// per operand), the two masked halves of a shift are combined before one merged ModDown + rescale, and
// `batch` shifts are processed per launch.
// single_tile: the caller promises that both operands hold one tile block and nothing else (what HEMMer::encrypt
// produces).  tau(B) is then copied into every block of the slot vector, which turns its row shifts into exact
// rotations and opens the baby-step / giant-step route also for a matrix that fills only part of the slots.  With
// operands that carry further tiles the result would mix them, so the default is off; HEMMer::singleCCMatMul sets
// it when Ciphertext::occupiedSlots() of both operands shows it to be true.
CtxtTensor multMatMatFused(const HomEvaluator &eval, const Bootstrapper &btp, const CtxtTensor &op1,
                           const CtxtTensor &op2, u64 target_level, MatrixTransformer &transformer, u64 batch = 16,
                           bool single_tile = false);
// single_tile: the operands hold one tile block and nothing else (as for multMatMatFused)
CtxtTensor multPackedMatMatFused(const HomEvaluator &eval, const Bootstrapper &btp, const CtxtTensor &op1,
                                 const CtxtTensor &op2, u64 target_level, MatrixTransformer &transformer,
                                 u64 batch = 16, bool single_tile = false);
void multMatMatPreFused(const HomEvaluator &eval, const CtxtTensor &a, std::vector<Ciphertext> &tmp, u64 target_level,
                        MatrixTransformer &transformer, u64 batch = 16, bool first_block_only = false);
// plaintext x ciphertext product through the hoisted column shifts (see matrix_utils_fused.cpp for the layouts it takes)
bool multMatMatPlainFused(const HomEvaluator &eval, const Bootstrapper &btp, const CtxtTensor &op1, const PtxtTensor &op2,
                          u64 target_level, MatrixTransformer &transformer, u64 batch, CtxtTensor &res);
// the n/2 column shifts (by two columns each) of a packed sigma(A) at level T+2, as ciphertexts at level T+1
// (multPackedMatMatPreRot through the hoisted launches)
void multPackedMatMatPreRotFused(const HomEvaluator &eval, const CtxtTensor &a, std::vector<Ciphertext> &tmp, u64 target_level,
                                 MatrixTransformer &transformer, u64 batch = 16);
// pa = complexPackingInplace(a) (adjacent columns), pb = complexPackingRowInplace(b) (adjacent rows of width w), through
// MatrixTransformer::complexPackingBatch at min(level of a, level of b, pack_level): operands above it are lowered first
void complexPackingPair(const HomEvaluator &eval, MatrixTransformer &transformer, const Ciphertext &a, const Ciphertext &b,
                        i64 w, Ciphertext &pa, Ciphertext &pb, u64 pack_level = ~u64(0));
// complexPackingPair at min(levels, target_level + 5) followed by multPackedMatMatFused, the packed pair passed on in
// place: the complex product of two plain n x n tiles (its real part, x + conj(x), is A B); needs level >= T+3.
// add_conj: returns x + conj(x) itself; where the schedule ends in a giant-step sum the conjugated terms join that sum
// (keys of every giant rotation's Galois element times 2N - 1, plain and square, and the square key of 2N - 1:
// KeyGenerator::genGaloisKey / genGaloisSquareKey), otherwise the result is conjugated and added.
CtxtTensor multMatMatComplexPackedFused(const HomEvaluator &eval, const Bootstrapper &btp, const CtxtTensor &a,
                                        const CtxtTensor &b, u64 target_level, MatrixTransformer &transformer,
                                        u64 batch = 16, bool single_tile = false, bool add_conj = false);
// sum_k tmp[k] (x) rho^(k step)(b), relinearised (and rescaled when rescale_after): the ciphertext x ciphertext re-use
// forms (multMatMatCCReUse: step = block width; multPackedMatMatCCReuse: step = 2 block widths, rescale) with all
// rotations of b taken from ONE ModUp through direct keys, in batches of hoisted sums
CtxtTensor multMatMatCCReUseFused(const HomEvaluator &eval, const std::vector<Ciphertext> &tmp, const CtxtTensor &b,
                                  u64 step, bool rescale_after, u64 batch = 16);
// left rotations (in slots) whose direct keys the batched schedules use
// Rotate-and-sum as hoisted sums.  The reference adds log2(count) rotations one after the other (x += rot(x, 2^k unit));
// the same sum, out = sum_{i < count} leftRotate(in, i * unit) (unit < 0: to the right; count a power of two), is taken
// here in at most two stages -- i = i0 + b i1 -- each ONE ModUp, ONE sum of the stage's rotations (its unrotated input a
// term without a key) and ONE ModDown, for all jobs of the call together.  The jobs share level and count; `in` may be
// `out`.
struct RotateSumJob {
    const Ciphertext *in;
    i64 unit;
    Ciphertext *out;
};
void rotateSumFused(const HomEvaluator &eval, const std::vector<RotateSumJob> &jobs, u64 count);
// left rotation amounts whose keys rotateSumFused needs for (unit, count)
std::vector<u64> rotateSumRotations(i64 unit, u64 count, u64 log_slots);

std::vector<u64> fusedRotations(const TileTensorShape &shape, u64 log_slots, bool packed, bool need_rows);
// the same for multMatMatFused; square_rots receives the giant steps that also need KeyPack::galoisSquareKey
std::vector<u64> fusedCcmmRotations(const TileTensorShape &shape, u64 log_slots, std::vector<u64> &square_rots,
                                    bool packed = false, bool single_tile = false);

}  // namespace HELLM

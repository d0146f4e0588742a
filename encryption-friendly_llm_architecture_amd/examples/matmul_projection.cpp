// A caller of the matrix-multiplication path written the way the reference's micro-benchmark drives HELLM::HEMMer
// (ciphertext/examples/bert-matmul.cpp:159-208: complexPacking of two activation tiles, matMulPre once, matMulReUse
// per weight tile group with addInplace accumulation; :292-338: singleCCMatMul-style products), compiled as plain
// C++ against this build's headers and linked with libhemm.so only.  Differences from the reference's source:
// matrices are HELLM::Matrix (row-major doubles) where the reference passes torch::Tensor, genHEMMer takes no MPI
// rank, and the final repack uses repackCC (x + conj x) because HEMMer::repack needs bootstrapping.
//
//   g++ -std=c++17 matmul_projection.cpp -I ../csrc/host -I ../../include -L .. -lhemm
//
// Prints the max-abs errors against float64 products and exits 0 when all are within 2^-12.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "HELLM/HEMMer.hpp"

using namespace HELLM;

namespace {

Matrix randomMatrix(std::mt19937_64 &gen, i64 n, double sigma) {
    std::normal_distribution<double> d(0.0, sigma);
    Matrix m(n, n);
    for (auto &x : m.v) x = d(gen);
    return m;
}
Matrix matmul(const Matrix &a, const Matrix &b) {
    Matrix c(a.rows, b.cols);
    for (i64 i = 0; i < a.rows; i++)
        for (i64 k = 0; k < a.cols; k++) {
            const double x = a.at(i, k);
            for (i64 j = 0; j < b.cols; j++) c.at(i, j) += x * b.at(k, j);
        }
    return c;
}
double maxAbsDiff(const Matrix &a, const Matrix &b) {
    double e = 0;
    for (size_t i = 0; i < a.v.size(); i++) e = std::fmax(e, std::fabs(a.v[i] - b.v[i]));
    return e;
}

}  // namespace

int main() {
    HEaaN::setSeed(3);
    HEMMer hemmer = HEMMer::genHEMMer();
    const i64 n = hemmer.dim();
    std::mt19937_64 gen(11);
    const u64 target_level = 4;
    const int n_in = 4, n_out = 2;     // activation tiles of one token block, output tile columns
    std::vector<Matrix> x, want(n_out, Matrix(n, n));
    std::vector<std::vector<Matrix>> w(n_in, std::vector<Matrix>());
    for (int i = 0; i < n_in; i++) x.push_back(randomMatrix(gen, n, 0.1));
    for (int i = 0; i < n_in; i++)
        for (int j = 0; j < n_out; j++) w[i].push_back(randomMatrix(gen, n, 0.02));
    for (int j = 0; j < n_out; j++)
        for (int i = 0; i < n_in; i++) {
            const Matrix p = matmul(x[i], w[i][j]);
            for (size_t k = 0; k < p.v.size(); k++) want[j].v[k] += p.v[k];
        }

    // PCMM as in bert-matmul.cpp:159-208: two activation tiles per complex-packed ciphertext (each tile copied into
    // both halves of the pair layout), the column shifts of sigma(X) computed once and reused for every weight
    CtxtTensor acc = hemmer.encrypt2(x[0], x[0]);
    for (int i = 0; i < n_in / 2; i++) {
        auto packed_x = hemmer.complexPacking(hemmer.encrypt2(x[2 * i], x[2 * i]),
                                              hemmer.encrypt2(x[2 * i + 1], x[2 * i + 1]));
        std::vector<HEaaN::Ciphertext> tmp;
        hemmer.matMulPre(packed_x, tmp, target_level);
        // msgDiagonalToRow4(W1, W2, W3, W4): result columns X0 W1 + X1 W3 | X0 W2 + X1 W4
        auto ptxt_weight = hemmer.encodeDiagonalToRow4(w[2 * i][0], w[2 * i][1], w[2 * i + 1][0], w[2 * i + 1][1],
                                                       target_level + 1);
        if (i == 0) {
            acc = hemmer.matMulReUse(tmp, ptxt_weight, target_level);
        } else {
            hemmer.addInplace(acc, hemmer.matMulReUse(tmp, ptxt_weight, target_level));
        }
    }
    const std::vector<Matrix> got = hemmer.decrypt2(hemmer.repackCC(acc));
    const double e_pcmm = std::fmax(maxAbsDiff(got[0], want[0]), maxAbsDiff(got[1], want[1]));

    // CCMM: one encrypted tile times another (HEMMer::singleCCMatMul), and its plaintext-weight counterpart
    const Matrix a = randomMatrix(gen, n, 0.5), b = randomMatrix(gen, n, 0.5);
    const Matrix ab = matmul(a, b);
    const CtxtTensor ca = hemmer.encrypt(a), cb = hemmer.encrypt(b);
    const double e_ccmm = maxAbsDiff(hemmer.decrypt(hemmer.singleCCMatMul(ca, cb, target_level)), ab);
    const double e_single = maxAbsDiff(hemmer.decrypt(hemmer.singleMatMul(ca, hemmer.encode(b), target_level)), ab);

    std::printf("pcmm_pre_reuse_max_abs_err %.3e\nccmm_max_abs_err %.3e\npcmm_single_max_abs_err %.3e\n", e_pcmm, e_ccmm,
                e_single);
    const double tol = std::ldexp(1.0, -12);
    const bool ok = e_pcmm < tol && e_ccmm < tol && e_single < tol;
    std::printf(ok ? "OK\n" : "FAILED\n");
    HELLM::cleanUpMatrixTransformer();
    return ok ? 0 : 1;
}

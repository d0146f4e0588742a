// Shape tag + ciphertext/plaintext payload, as HEMMer passes matrices around
// (reference: ciphertext/include/HELLM/HETensor.hpp:16-86).  A tile of `rows x cols` values sits
// row-major in rows of `block_width` slots; block_width is the power of two >= cols unless given.
#pragma once
#include <tuple>
#include <utility>

#include "HEaaN/HEaaN.hpp"

namespace HELLM {

using namespace HEaaN;

class TileTensorShape {
public:
    TileTensorShape() = default;
    TileTensorShape(i64 rows, i64 cols) : rows_(rows), cols_(cols), block_width_(nextPow2(cols)) {}
    TileTensorShape(i64 rows, i64 cols, i64 block_width) : rows_(rows), cols_(cols), block_width_(block_width) {}
    i64 getNumRows() const { return rows_; }
    i64 getNumCols() const { return cols_; }
    i64 getBlockWidth() const { return block_width_; }
    void setNumRows(i64 r) { rows_ = r; }
    void setNumCols(i64 c) { cols_ = c; }
    bool operator==(const TileTensorShape &o) const {
        return rows_ == o.rows_ && cols_ == o.cols_ && block_width_ == o.block_width_;
    }
    bool operator<(const TileTensorShape &o) const {
        return std::tie(rows_, cols_, block_width_) < std::tie(o.rows_, o.cols_, o.block_width_);
    }

private:
    static i64 nextPow2(i64 v) {
        i64 p = 1;
        while (p < v) p <<= 1;
        return p;
    }
    i64 rows_ = 0, cols_ = 0, block_width_ = 0;
};

template <class T>
class HETensor {
public:
    HETensor(const Context &c, i64 rows, i64 cols) : shape_(rows, cols), data_(c) {}
    HETensor(const Context &c, i64 rows, i64 cols, i64 block_width) : shape_(rows, cols, block_width), data_(c) {}
    HETensor(const Context &c, const TileTensorShape &s) : shape_(s), data_(c) {}
    HETensor(i64 rows, i64 cols, const T &d) : shape_(rows, cols), data_(d) {}
    HETensor(i64 rows, i64 cols, const T &d, i64 block_width) : shape_(rows, cols, block_width), data_(d) {}
    HETensor(const TileTensorShape &s, const T &d) : shape_(s), data_(d) {}

    T &get() { return data_; }
    const T &get() const { return data_; }
    const TileTensorShape &getShape() const { return shape_; }
    i64 getHeight() const { return shape_.getNumRows(); }
    i64 getWidth() const { return shape_.getNumCols(); }
    i64 getBlockWidth() const { return shape_.getBlockWidth(); }
    u64 getLevel() const { return data_.getLevel(); }
    u64 getLogSlots() const { return data_.getLogSlots(); }
    void setShape(i64 rows, i64 cols) {
        shape_.setNumRows(rows);
        shape_.setNumCols(cols);
    }

private:
    TileTensorShape shape_;
    T data_;
};

using CtxtTensor = HETensor<Ciphertext>;
using PtxtTensor = HETensor<Plaintext>;

}  // namespace HELLM

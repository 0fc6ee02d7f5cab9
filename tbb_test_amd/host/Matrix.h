// Matrix<T, PAD>: padded row-major host matrix, the benchmark's host-side tensor type.
//
// Layout contract (what the device upload and the reduce rely on; reference Matrix.h:29-30,
// 100-121,148): element (i, j) lives at data_[i * ld() + j] with ld() = ncols() + PAD, and the
// allocation holds (nrows + PAD) * (ncols + PAD) elements starting on a 4 KiB boundary, so the
// PAD tail columns of every row are addressable (the all-reduce runs over whole padded rows).
// Unlike the reference this class tracks ownership: a matrix wrapped around foreign memory
// (pointer / aligned_vector constructors) never frees it.
#ifndef MATRIX_H
#define MATRIX_H

#include <algorithm>
#include <cassert>
#include <cmath>
#include <cstdlib>
#include <iomanip>
#include <iostream>
#include <new>
#include <string>
#include <utility>
#include <vector>

#include "Rand.h"

template <typename T, int PAD = 0>
class Matrix {
 public:
  // nrows x ncols, contents unspecified
  Matrix(const int nrows, const int ncols, const std::string name = "")
      : data_(nullptr), nrows_(nrows), ncols_(ncols), name_(name), owned_(true) {
    allocate();
  }

  // view over caller-owned storage with the same padded layout
  Matrix(const int nrows, const int ncols, T* ptr, const std::string name = "")
      : data_(ptr), nrows_(nrows), ncols_(ncols), name_(name), owned_(false) {
    assert(nrows_ > 0 && ncols_ > 0);
  }

  // shape = {nrows, ncols}; filled with `low`, then uniformly in [low, high] when high > low
  explicit Matrix(const std::vector<int> shape, const T low = T(0), const T high = T(0),
                  bool duplicates = true, const std::string name = "")
      : data_(nullptr), nrows_(shape.at(0)), ncols_(shape.at(1)), name_(name), owned_(true) {
    assert(shape.size() == 2);
    allocate();
    for (int i = 0; i < nrows_; ++i) std::fill_n(rawData(i, 0), ncols_, low);
    if (low < high) randFill(low, high, duplicates);
  }

  Matrix(const Matrix&) = delete;
  Matrix& operator=(const Matrix&) = delete;
  Matrix(Matrix&& o) noexcept
      : data_(o.data_), nrows_(o.nrows_), ncols_(o.ncols_), name_(std::move(o.name_)),
        owned_(o.owned_) {
    o.data_ = nullptr;
    o.owned_ = false;
  }

  ~Matrix() { release(); }

  // new random contents in [low, high], or zeros (padding included) when the range is empty
  void newInput(const T low = T(0), const T high = T(0), bool duplicates = true) {
    if (low < high) {
      randFill(low, high, duplicates);
    } else {
      std::fill_n(data_, allocatedElems(), T(0));
    }
  }

  T& operator()(int row, int col) {
    assert(row >= 0 && row < nrows_ && col >= 0 && col < ncols_);
    return data_[offset(row, col)];
  }
  const T& operator()(int row, int col) const {
    assert(row >= 0 && row < nrows_ && col >= 0 && col < ncols_);
    return data_[offset(row, col)];
  }

  T* rawData() { return data_; }
  const T* rawData() const { return data_; }
  T* rawData(int row, int col) { return data_ + offset(row, col); }
  const T* rawData(int row, int col) const { return data_ + offset(row, col); }

  // logical element count (padding excluded)
  const std::size_t size() const { return (std::size_t)nrows_ * ncols_; }
  // elements actually allocated, padding rows and columns included
  std::size_t allocatedElems() const { return ((std::size_t)nrows_ + PAD) * ((std::size_t)ncols_ + PAD); }

  void realloc(int nrows, int ncols) {
    release();
    nrows_ = nrows;
    ncols_ = ncols;
    owned_ = true;
    allocate();
  }
  void realloc(const std::vector<int>& shape) { realloc(shape.at(0), shape.at(1)); }

  // re-point at a flat vector (dense, so only meaningful for PAD == 0); does not take ownership
  void assign(aligned_vector<T>& other, int nrows, int ncols) {
    assert((std::size_t)nrows * ncols == other.size());
    release();
    nrows_ = nrows;
    ncols_ = ncols;
    data_ = other.data();
    owned_ = false;
  }

  const std::vector<int> shape() const { return {nrows_, ncols_}; }
  const std::string name() const { return name_; }
  const int nrows() const { return nrows_; }
  const int ncols() const { return ncols_; }
  int ld() const { return ncols_ + PAD; }

  // element-wise comparison of the logical contents with relative tolerance 1e-6
  bool operator==(const Matrix& other) const {
    if (nrows_ != other.nrows_ || ncols_ != other.ncols_) return false;
    const double rtol = 1e-6;
    for (int i = 0; i < nrows_; ++i) {
      for (int j = 0; j < ncols_; ++j) {
        double a = (double)(*this)(i, j), b = (double)other(i, j);
        if (std::abs(a - b) > rtol * std::abs(b)) {
          std::cout << "(" << i << "," << j << ") " << a << " vs " << b << "\n";
          return false;
        }
      }
    }
    return true;
  }

  // uniform fill, one row at a time so the padding never consumes random numbers
  void randFill(T low, T high, bool duplicates = true) {
    for (int i = 0; i < nrows_; ++i) ::randFill(rawData(i, 0), (std::size_t)ncols_, low, high, duplicates);
  }

  T* data_;

 protected:
  std::size_t offset(int row, int col) const { return (std::size_t)row * (ncols_ + PAD) + col; }

  void allocate() {
    assert(nrows_ > 0 && ncols_ > 0);
    void* p = nullptr;
    if (posix_memalign(&p, 4096, sizeof(T) * allocatedElems()) != 0 || !p) throw std::bad_alloc();
    data_ = static_cast<T*>(p);
  }
  void release() {
    if (owned_ && data_) std::free(data_);
    data_ = nullptr;
  }

  int nrows_;
  int ncols_;
  std::string name_;
  bool owned_;
};

inline const std::vector<int> shape(int nrows, int ncols) { return {nrows, ncols}; }

template <typename T, int PAD>
T sum(const Matrix<T, PAD>& m) {
  T total = T(0);
  for (int i = 0; i < m.nrows(); ++i)
    for (int j = 0; j < m.ncols(); ++j) total += m(i, j);
  return total;
}

template <typename T, int PAD>
std::ostream& operator<<(std::ostream& os, const Matrix<T, PAD>& m) {
  os << "Matrix " << m.name() << ": " << m.nrows() << " x " << m.ncols() << "\n";
  for (int i = 0; i < m.nrows(); ++i) {
    for (int j = 0; j < m.ncols(); ++j) os << std::setprecision(9) << m(i, j) << " ";
    os << "\n";
  }
  return os;
}

#endif

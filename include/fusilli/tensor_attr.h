// Context and TensorAttr: a tensor is logical dims in the op's fixed logical
// order plus element strides that define the physical layout.
//
// Behavioural mirror of the reference's attributes/tensor_attributes.h:159-809
// and graph/context.h:24-61: same setters/getters, the same validation order,
// codes and messages, the same layout helpers (stride orders, stride
// generation, broadcast shape, logical<->physical permutations).
#ifndef FUSILLI_TENSOR_ATTR_H
#define FUSILLI_TENSOR_ATTR_H

#include <algorithm>
#include <cstdint>
#include <initializer_list>
#include <memory>
#include <numeric>
#include <optional>
#include <ranges>
#include <span>
#include <string>
#include <variant>
#include <vector>

#include "errors.h"
#include "types.h"

namespace fusilli {

// Graph-wide defaults (graph/context.h:24-61).
class Context {
public:
  Context &setIntermediateDataType(DataType t) {
    intermediate_ = t;
    return *this;
  }
  Context &setIODataType(DataType t) {
    io_ = t;
    return *this;
  }
  Context &setComputeDataType(DataType t) {
    compute_ = t;
    return *this;
  }
  Context &setName(const std::string &n) {
    name_ = n;
    return *this;
  }
  DataType getIODataType() const { return io_; }
  DataType getIntermediateDataType() const { return intermediate_; }
  DataType getComputeDataType() const { return compute_; }
  const std::string &getName() const { return name_; }

private:
  DataType compute_ = DataType::NotSet;
  DataType intermediate_ = DataType::NotSet;
  DataType io_ = DataType::NotSet;
  std::string name_;
};

template <typename R>
concept Int64Range = std::ranges::forward_range<R> &&
                     std::is_same_v<std::ranges::range_value_t<R>, int64_t>;

// ---- layout helpers ---------------------------------------------------------
// A stride order ranks dims from fastest (0) to slowest changing.

// Row-major: last dim fastest.  4-D: {3, 2, 1, 0}.
inline std::vector<size_t> getContiguousStrideOrder(size_t rank) {
  std::vector<size_t> order(rank);
  for (size_t i = 0; i < rank; ++i)
    order[i] = rank - 1 - i;
  return order;
}

// Channels-last: dim 1 fastest, then the spatial dims right to left, dim 0
// slowest.  4-D: {3, 0, 2, 1}.
inline std::vector<size_t> getChannelsLastStrideOrder(size_t rank) {
  assert(rank >= 3 && "channels-last needs at least 3 dims");
  std::vector<size_t> order(rank);
  order[1] = 0;
  size_t next = 1;
  for (size_t i = rank - 1; i >= 2; --i)
    order[i] = next++;
  order[0] = next;
  return order;
}

// The stride order that `stride` itself follows, extended with slower dims if
// `outRank` is larger.  {10, 30, 20} -> {0, 2, 1}.
inline std::vector<size_t>
generateStrideOrderPreservingFormat(const std::vector<int64_t> stride,
                                    size_t outRank) {
  std::vector<size_t> byStride(stride.size());
  std::iota(byStride.begin(), byStride.end(), size_t{0});
  std::sort(byStride.begin(), byStride.end(),
            [&](size_t a, size_t b) { return stride[a] < stride[b]; });
  std::vector<size_t> order(stride.size());
  for (size_t rank = 0; rank < byStride.size(); ++rank)
    order[byStride[rank]] = rank;
  for (size_t i = order.size(); i < outRank; ++i)
    order.push_back(i);
  return order;
}

// Dense strides for `dim` laid out in `order`.
inline std::vector<int64_t>
generateStrideFromDim(const std::vector<int64_t> &dim,
                      const std::vector<size_t> &order) {
  const size_t rank = dim.size();
  std::vector<size_t> dimAtRank(rank);
  for (size_t i = 0; i < rank; ++i)
    dimAtRank[order[i]] = i;
  std::vector<int64_t> stride(rank);
  int64_t running = 1;
  for (size_t r = 0; r < rank; ++r) {
    stride[dimAtRank[r]] = running;
    running *= dim[dimAtRank[r]];
  }
  return stride;
}

// Strides from a layout name: "NHC"/"NHWC"/"NDHWC" are channels-last,
// "N"/"NC"/"NCH"/"NCHW"/"NCDHW" contiguous.
inline ErrorOr<std::vector<int64_t>>
generateStrideFromLayout(const std::vector<int64_t> &dims,
                         const std::string &layout) {
  FUSILLI_RETURN_ERROR_IF(
      dims.size() != layout.size(), ErrorCode::InvalidArgument,
      "Invalid input dimensions and layout: they must have the same rank");
  for (const char *cl : {"NHC", "NHWC", "NDHWC"})
    if (layout == cl)
      return ok(
          generateStrideFromDim(dims, getChannelsLastStrideOrder(dims.size())));
  for (const char *ct : {"N", "NC", "NCH", "NCHW", "NCDHW"})
    if (layout == ct)
      return ok(
          generateStrideFromDim(dims, getContiguousStrideOrder(dims.size())));
  return error(ErrorCode::InvalidArgument, "Invalid layout string: " + layout);
}

inline std::vector<int64_t> getPreserveContiguousPermuteOrder(size_t rank) {
  std::vector<int64_t> p(rank);
  std::iota(p.begin(), p.end(), int64_t{0});
  return p;
}

// NHWC -> NCHW as a permutation of physical axes: {0, 3, 1, 2} for rank 4.
inline std::vector<int64_t>
getChannelsLastToContiguousPermuteOrder(size_t rank) {
  assert(rank >= 3);
  std::vector<int64_t> p(rank);
  p[0] = 0;
  p[1] = static_cast<int64_t>(rank) - 1;
  for (size_t i = 2; i < rank; ++i)
    p[i] = static_cast<int64_t>(i) - 1;
  return p;
}

// NCHW -> NHWC: {0, 2, 3, 1} for rank 4.
inline std::vector<int64_t>
getContiguousToChannelsLastPermuteOrder(size_t rank) {
  assert(rank >= 3);
  std::vector<int64_t> p(rank);
  p[0] = 0;
  for (size_t i = 1; i + 1 < rank; ++i)
    p[i] = static_cast<int64_t>(i) + 1;
  p[rank - 1] = 1;
  return p;
}

inline std::vector<int64_t>
inversePermutation(const std::vector<int64_t> &perm) {
  std::vector<int64_t> inv(perm.size());
  for (size_t i = 0; i < perm.size(); ++i)
    inv[static_cast<size_t>(perm[i])] = static_cast<int64_t>(i);
  return inv;
}

// PyTorch-style (right-aligned) broadcast of a set of shapes; empty shapes
// are ignored.
inline ErrorOr<std::vector<int64_t>>
computeBroadcastShape(const std::vector<std::vector<int64_t>> &shapes) {
  size_t rank = 0;
  bool any = false;
  for (const auto &s : shapes)
    if (!s.empty()) {
      any = true;
      rank = std::max(rank, s.size());
    }
  FUSILLI_RETURN_ERROR_IF(!any, ErrorCode::InvalidAttribute,
                          "All input shapes are empty");
  std::vector<int64_t> out(rank, 1);
  for (const auto &s : shapes) {
    for (size_t back = 0; back < s.size(); ++back) {
      int64_t &o = out[rank - 1 - back];
      const int64_t d = s[s.size() - 1 - back];
      if (o == 1)
        o = d;
      FUSILLI_RETURN_ERROR_IF(d != 1 && o != d, ErrorCode::InvalidAttribute,
                              "Cannot broadcast two non unit dimensions");
    }
  }
  return ok(std::move(out));
}

// ---- TensorAttr -------------------------------------------------------------
class TensorAttr {
public:
  using scalar_t = std::variant<int64_t, int32_t, float, double>;

  TensorAttr() = default;

  // Scalar constants: dim = stride = {1}; never part of a variant pack.
  explicit TensorAttr(float v) { makeScalar(v, DataType::Float); }
  explicit TensorAttr(double v) { makeScalar(v, DataType::Double); }
  explicit TensorAttr(int32_t v) { makeScalar(v, DataType::Int32); }
  explicit TensorAttr(int64_t v) { makeScalar(v, DataType::Int64); }

  ErrorObject validate() const {
    FUSILLI_LOG_LABEL_ENDL("INFO: Validating tensor '" << name_ << "'");
    const std::string who = "Tensor '" + name_ + "'";
    FUSILLI_RETURN_ERROR_IF(dim_.empty(), ErrorCode::AttributeNotSet,
                            who + " dims not set");
    FUSILLI_RETURN_ERROR_IF(stride_.empty(), ErrorCode::AttributeNotSet,
                            who + " strides not set");
    FUSILLI_RETURN_ERROR_IF(
        dim_.size() != stride_.size(), ErrorCode::InvalidAttribute,
        who + " uses dim and stride of different dimensionality");
    for (size_t idx : dynamicDims_) {
      FUSILLI_RETURN_ERROR_IF(
          idx >= dim_.size(), ErrorCode::InvalidAttribute,
          who + " has dynamic dim index " + std::to_string(idx) +
              " out of range for rank " + std::to_string(dim_.size()));
      FUSILLI_RETURN_ERROR_IF(
          stride_[idx] == 0, ErrorCode::InvalidAttribute,
          who + " has dynamic dim at index " + std::to_string(idx) +
              " with stride 0 (broadcast stride), which is not supported");
      FUSILLI_RETURN_ERROR_IF(
          dim_[idx] == 1, ErrorCode::InvalidAttribute,
          who + " has dynamic dim at index " + std::to_string(idx) +
              " with representative size 1, which is not supported");
    }
    FUSILLI_RETURN_ERROR_IF(
        hasBroadcastDims() && hasDynamicDims(), ErrorCode::InvalidAttribute,
        who + " has dynamic dimensions on a tensor with broadcast strides, "
              "which is not supported");
    FUSILLI_RETURN_ERROR_IF(
        !hasValidPhysicalRepresentation(), ErrorCode::InvalidAttribute,
        who + " has invalid physical representation. It must be a valid "
              "permutation of the logical dimensions");
    FUSILLI_RETURN_ERROR_IF(dataType_ == DataType::NotSet,
                            ErrorCode::AttributeNotSet,
                            who + " data type not set");
    FUSILLI_RETURN_ERROR_IF(
        isVirtual_ && isScalar_, ErrorCode::InvalidAttribute,
        who + " cannot be both virtual (intermediate) and a scalar constant");
    FUSILLI_RETURN_ERROR_IF(
        scalarValue_.has_value() && !isScalar_, ErrorCode::InvalidAttribute,
        who + " has a scalar value set but is not marked as a scalar");
    FUSILLI_RETURN_ERROR_IF(
        !scalarValue_.has_value() && isScalar_, ErrorCode::InvalidAttribute,
        who + " is marked as a scalar but does not have a scalar value set");
    return ok();
  }

  // Unset dtype <- intermediate dtype if virtual, else the I/O dtype.
  TensorAttr &fillFromContext(const Context &ctx) {
    if (dataType_ == DataType::NotSet)
      dataType_ = isVirtual_ ? ctx.getIntermediateDataType()
                             : ctx.getIODataType();
    return *this;
  }

  // Setters.
  TensorAttr &setName(const std::string &n) {
    name_ = n;
    return *this;
  }
  TensorAttr &setDataType(DataType t) {
    dataType_ = t;
    return *this;
  }
  TensorAttr &setDim(const std::vector<int64_t> &d) {
    dim_ = d;
    return *this;
  }
  template <Int64Range R> TensorAttr &setDim(R &&d) {
    dim_.assign(d.begin(), d.end());
    return *this;
  }
  TensorAttr &setStride(const std::vector<int64_t> &s) {
    stride_ = s;
    return *this;
  }
  template <Int64Range R> TensorAttr &setStride(R &&s) {
    stride_.assign(s.begin(), s.end());
    return *this;
  }
  TensorAttr &setDynamicDim(size_t index) {
    dynamicDims_.push_back(index);
    normaliseDynamicDims();
    return *this;
  }
  TensorAttr &setDynamicDims(std::span<const size_t> indices) {
    dynamicDims_.assign(indices.begin(), indices.end());
    normaliseDynamicDims();
    return *this;
  }
  TensorAttr &setDynamicDims(std::initializer_list<size_t> indices) {
    return setDynamicDims(std::span<const size_t>(indices.begin(), indices.size()));
  }
  TensorAttr &clearDynamicDims() {
    dynamicDims_.clear();
    return *this;
  }
  TensorAttr &setIsVirtual(bool v) {
    isVirtual_ = v;
    return *this;
  }
  TensorAttr &setOutput(bool isOutput) { return setIsVirtual(!isOutput); }
  TensorAttr &setIsScalar(bool v) {
    isScalar_ = v;
    return *this;
  }

  // Getters.
  const std::string &getName() const { return name_; }
  DataType getDataType() const { return dataType_; }
  const std::vector<int64_t> &getDim() const { return dim_; }
  const std::vector<int64_t> &getStride() const { return stride_; }
  bool isDynamicDim(size_t i) const {
    return std::binary_search(dynamicDims_.begin(), dynamicDims_.end(), i);
  }
  bool hasDynamicDims() const { return !dynamicDims_.empty(); }
  const std::vector<size_t> &getDynamicDims() const { return dynamicDims_; }
  int64_t getVolume() const {
    return std::accumulate(dim_.begin(), dim_.end(), int64_t{1},
                           std::multiplies<int64_t>());
  }
  bool isVirtual() const { return isVirtual_; }
  bool isScalar() const { return isScalar_; }
  std::optional<scalar_t> getScalarValue() const { return scalarValue_; }

  bool isContiguous() const {
    return stride_ ==
           generateStrideFromDim(dim_, getContiguousStrideOrder(dim_.size()));
  }
  bool isChannelsLast() const {
    return stride_ ==
           generateStrideFromDim(dim_, getChannelsLastStrideOrder(dim_.size()));
  }

  bool hasBroadcastDims() const {
    for (size_t i = 0; i < dim_.size() && i < stride_.size(); ++i)
      if (dim_[i] > 1 && stride_[i] == 0)
        return true;
    return false;
  }

  // Dims with broadcast dims (stride 0) collapsed to 1.
  std::vector<int64_t> getUnexpandedDim() const {
    std::vector<int64_t> d = dim_;
    for (size_t i = 0; i < d.size() && i < stride_.size(); ++i)
      if (d[i] > 1 && stride_[i] == 0)
        d[i] = 1;
    return d;
  }

  // Strides must describe a dense permutation of the dims: sorted by stride,
  // each stride equals the product of the faster dims.  Unit dims and
  // broadcast dims (stride 0) are free.
  bool hasValidPhysicalRepresentation() const {
    if (dim_.size() != stride_.size())
      return false;
    std::vector<std::pair<int64_t, int64_t>> byStride;
    for (size_t i = 0; i < dim_.size(); ++i) {
      if (stride_[i] < 0)
        return false;
      byStride.emplace_back(stride_[i], dim_[i]);
    }
    std::stable_sort(byStride.begin(), byStride.end(),
                     [](const auto &a, const auto &b) { return a.first < b.first; });
    int64_t expect = 1;
    for (const auto &[s, d] : byStride) {
      if (d == 1 || s == 0)
        continue;
      if (s != expect)
        return false;
      expect = s * d;
    }
    return true;
  }

  // perm[i] = logical dim found at physical position i.  Only dims that are
  // neither unit nor broadcast move; the rest keep their index.
  std::vector<int64_t> getLogicalToPhysicalPermuteOrder() const {
    const size_t rank = dim_.size();
    std::vector<int64_t> perm(rank);
    std::iota(perm.begin(), perm.end(), int64_t{0});
    std::vector<size_t> movable;
    for (size_t i = 0; i < rank; ++i)
      if (dim_[i] != 1 && stride_[i] != 0)
        movable.push_back(i);
    std::vector<size_t> slowestFirst = movable;
    std::stable_sort(slowestFirst.begin(), slowestFirst.end(),
                     [&](size_t a, size_t b) { return stride_[a] > stride_[b]; });
    for (size_t i = 0; i < movable.size(); ++i)
      perm[movable[i]] = static_cast<int64_t>(slowestFirst[i]);
    return perm;
  }

  std::vector<int64_t> getPhysicalToLogicalPermuteOrder() const {
    return inversePermutation(getLogicalToPhysicalPermuteOrder());
  }

  // Shape of the buffer that backs this tensor (broadcast dims occupy 1).
  std::vector<int64_t> getPhysicalDim() const {
    assert(hasValidPhysicalRepresentation());
    const auto perm = getLogicalToPhysicalPermuteOrder();
    std::vector<int64_t> phys(dim_.size());
    for (size_t i = 0; i < dim_.size(); ++i) {
      const size_t src = static_cast<size_t>(perm[i]);
      phys[i] = (dim_[src] > 1 && stride_[src] == 0) ? 1 : dim_[src];
    }
    return phys;
  }

private:
  template <typename V> void makeScalar(V v, DataType t) {
    scalarValue_ = v;
    isScalar_ = true;
    dim_ = stride_ = {1};
    dataType_ = t;
  }
  void normaliseDynamicDims() {
    std::sort(dynamicDims_.begin(), dynamicDims_.end());
    dynamicDims_.erase(std::unique(dynamicDims_.begin(), dynamicDims_.end()),
                       dynamicDims_.end());
  }

  std::string name_;
  DataType dataType_ = DataType::NotSet;
  std::vector<int64_t> dim_;
  std::vector<int64_t> stride_;
  std::vector<size_t> dynamicDims_;
  bool isVirtual_ = false;
  bool isScalar_ = false;
  std::optional<scalar_t> scalarValue_;
};

struct TensorAttrSortByName {
  bool operator()(const std::shared_ptr<TensorAttr> &a,
                  const std::shared_ptr<TensorAttr> &b) const {
    return a->getName() < b->getName();
  }
};

// Scalar constant as a double (the value planners inline into kernels).
inline double scalarAsDouble(const TensorAttr &t) {
  const auto v = t.getScalarValue();
  if (!v)
    return 0.0;
  return std::visit([](auto x) { return static_cast<double>(x); }, *v);
}

} // namespace fusilli

#endif // FUSILLI_TENSOR_ATTR_H

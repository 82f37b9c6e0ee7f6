// Stride algebra of the reference's tensors (adrastea_models/src/tensor.rs:25-150) for C++ callers
// of the C ABI.  Strides are in elements; dims are outermost first.  Violations throw
// std::invalid_argument where the reference assert!-panics.
#pragma once

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <utility>
#include <vector>

namespace adrastea {

struct TensorLayout {
  std::vector<size_t> dims, strides;

  TensorLayout(std::vector<size_t> d, std::vector<size_t> s) : dims(std::move(d)), strides(std::move(s)) {
    // tensor.rs:32-39
    if (dims.size() != strides.size() || dims.empty()) throw std::invalid_argument("dims/strides mismatch");
    for (size_t x : dims) if (x == 0) throw std::invalid_argument("zero-sized dimension");
    for (size_t x : strides) if (x == 0) throw std::invalid_argument("zero stride");
  }

  static TensorLayout row_major(const std::vector<size_t>& dims) {  // tensor.rs:41-50
    std::vector<size_t> st(dims.size());
    size_t s = 1;
    for (size_t i = dims.size(); i-- > 0;) { st[i] = s; s *= dims[i]; }
    return TensorLayout(dims, st);
  }
  static TensorLayout column_major(const std::vector<size_t>& dims) {  // tensor.rs:52-60
    TensorLayout r = row_major(dims);
    std::swap(r.strides[dims.size() - 2], r.strides[dims.size() - 1]);
    return r;
  }
  size_t largest_address() const {  // tensor.rs:62-68
    size_t a = 0;
    for (size_t i = 0; i < dims.size(); i++) a += (dims[i] - 1) * strides[i];
    return a;
  }
  TensorLayout permute(const std::vector<size_t>& order) const {  // tensor.rs:70-79
    if (order.size() != dims.size()) throw std::invalid_argument("permute: one index per dimension");
    std::vector<size_t> d, s;
    for (size_t i : order) { d.push_back(dims.at(i)); s.push_back(strides.at(i)); }
    return TensorLayout(d, s);
  }
  // "poor man's .view()": keeps only the volume, fresh contiguous strides (tensor.rs:82-105)
  TensorLayout shape_cast(const std::vector<long>& nd) const {
    size_t vol = 1;
    for (size_t x : dims) vol *= x;
    size_t known = 1;
    int neg = 0;
    for (long x : nd) { if (x < 0) neg++; else known *= (size_t)x; }
    if (neg > 1) throw std::invalid_argument("shape_cast: at most one inferred dimension");
    std::vector<size_t> out;
    size_t prod = 1;
    for (long x : nd) { size_t v = x < 0 ? vol / known : (size_t)x; out.push_back(v); prod *= v; }
    if (prod != vol) throw std::invalid_argument("shape_cast must preserve the volume");
    return row_major(out);
  }
  size_t size(long dim) const { return dims.at(dim < 0 ? dims.size() + dim : (size_t)dim); }      // :107-113
  size_t stride(long dim) const { return strides.at(dim < 0 ? strides.size() + dim : (size_t)dim); }  // :115-121
  std::pair<size_t, TensorLayout> skip(const std::vector<long>& sizes) const {  // tensor.rs:123-136
    size_t off = 0;
    std::vector<size_t> d, s;
    for (size_t i = 0; i < sizes.size() && i < dims.size(); i++) {
      long sz = sizes[i] == -1 ? (long)dims[i] : sizes[i];
      if (sz < 0 || (size_t)sz > dims[i]) throw std::invalid_argument("skip size out of range");
      off += strides[i] * (size_t)sz;
      d.push_back(dims[i] - (size_t)sz);
      s.push_back(strides[i]);
    }
    return {off, TensorLayout(d, s)};
  }
  TensorLayout take(const std::vector<long>& sizes) const {  // tensor.rs:138-149
    std::vector<size_t> d, s;
    for (size_t i = 0; i < sizes.size() && i < dims.size(); i++) {
      long sz = sizes[i] == -1 ? (long)dims[i] : sizes[i];
      if (sz < 0 || (size_t)sz > dims[i]) throw std::invalid_argument("take size out of range");
      d.push_back((size_t)sz);
      s.push_back(strides[i]);
    }
    return TensorLayout(d, s);
  }
  bool operator==(const TensorLayout& o) const { return dims == o.dims && strides == o.strides; }
  bool operator<(const TensorLayout& o) const { return dims != o.dims ? dims < o.dims : strides < o.strides; }
};

// A layout over device memory the caller owns (fp16 as raw uint16_t bit patterns).
template <typename T>
struct TensorView {
  T* ptr;
  TensorLayout layout;
  TensorView(T* p, TensorLayout l) : ptr(p), layout(std::move(l)) {}
  size_t size(long d) const { return layout.size(d); }
  size_t stride(long d) const { return layout.stride(d); }
  TensorView permute(const std::vector<size_t>& o) const { return TensorView(ptr, layout.permute(o)); }
  TensorView shape_cast(const std::vector<long>& d) const { return TensorView(ptr, layout.shape_cast(d)); }
  TensorView skip(const std::vector<long>& s) const { auto r = layout.skip(s); return TensorView(ptr + r.first, r.second); }
  TensorView take(const std::vector<long>& s) const { return TensorView(ptr, layout.take(s)); }
};

}  // namespace adrastea

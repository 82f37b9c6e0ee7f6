// C++ host side of the matmul interface, mirroring adrastea_models/src/kernels.rs:81-167
// (option types), :206-213 (the two trait methods), :753-890 (lowering to the 22-scalar tuple)
// and :231-359 (MatmulTracer).  GpuKernels launches through the C ABI of
// include/adrastea_kernels.h; shape mismatches throw std::logic_error where the reference
// assert_eq!-panics, launcher errors throw AdrasteaError where it returns anyhow::Error.
#pragma once

#include <mutex>
#include <set>
#include <stdexcept>
#include <string>
#include <tuple>

#include "../../include/adrastea_kernels.h"
#include "tensor.hpp"

namespace adrastea {

using f16 = uint16_t;  // raw fp16 bits

struct AdrasteaError : std::runtime_error {
  int code;
  AdrasteaError(int c, const std::string& what) : std::runtime_error(what + ": " + adr_strerror(c)), code(c) {}
};

enum class MatmulMask : uint32_t { None = 0, Causal = 1 };

struct MatmulLoad {
  uint32_t op = ADR_LOAD_IDENTITY;
  float scale = 1.0f;
  static MatmulLoad Identity() { return {}; }
  static MatmulLoad Scale(float s) { return {ADR_LOAD_SCALE, s}; }
  uint32_t lower() const { return op; }
};

struct MatmulStore {
  uint32_t op = ADR_STORE_IDENTITY;
  float beta = 0.0f, scale = 1.0f;
  const f16* bias = nullptr;  // length-N vector indexed by output column
  static MatmulStore Identity() { return {}; }
  static MatmulStore GeluBias(const f16* b) { return {ADR_STORE_GELU_BIAS, 0, 1, b}; }
  static MatmulStore QuickGeluBias(const f16* b) { return {ADR_STORE_QUICK_GELU_BIAS, 0, 1, b}; }
  static MatmulStore BetaGeluBias(float beta, const f16* b) { return {ADR_STORE_BETA_GELU_BIAS, beta, 1, b}; }
  static MatmulStore BetaBias(float beta, const f16* b) { return {ADR_STORE_BETA_BIAS, beta, 1, b}; }
  static MatmulStore Scale(float s) { return {ADR_STORE_SCALE, 0, s, nullptr}; }
  static MatmulStore Add() { return {ADR_STORE_ADD, 0, 1, nullptr}; }
  uint32_t lower() const { return op; }
};

struct MatmulOptions {
  MatmulLoad load_;
  MatmulStore store_;
  MatmulMask mask_ = MatmulMask::None;
  static MatmulOptions make() { return {}; }
  MatmulOptions load(MatmulLoad l) const { MatmulOptions o = *this; o.load_ = l; return o; }
  MatmulOptions store(MatmulStore s) const { MatmulOptions o = *this; o.store_ = s; return o; }
  MatmulOptions mask(MatmulMask m) const { MatmulOptions o = *this; o.mask_ = m; return o; }
};

struct LoweredMatmul {
  int32_t batches, m, k, n;
  int32_t so[3], sl[3], sr[3];  // (x, y, z) strides of output, left, right
  float beta, scale;
  uint32_t store, load, mask;
};

inline LoweredMatmul lower_matmul(const TensorLayout& out, const TensorLayout& left, const TensorLayout& right,
                                  const MatmulOptions& o) {
  if (left.size(-1) != right.size(-2)) throw std::logic_error("K mismatch");   // kernels.rs:825
  if (out.size(-2) != left.size(-2)) throw std::logic_error("M mismatch");     // kernels.rs:826
  if (out.size(-1) != right.size(-1)) throw std::logic_error("N mismatch");    // kernels.rs:827
  LoweredMatmul r{};
  float scale = o.load_.op == ADR_LOAD_SCALE ? o.load_.scale : 1.0f;
  if (o.store_.op == ADR_STORE_SCALE) scale *= o.store_.scale;  // ONE float for both (:837-843)
  r.scale = scale;
  r.beta = (o.store_.op == ADR_STORE_BETA_GELU_BIAS || o.store_.op == ADR_STORE_BETA_BIAS) ? o.store_.beta : 0.0f;
  r.batches = out.dims.size() > 2 ? (int32_t)out.size(-3) : 1;
  r.m = (int32_t)left.size(-2); r.k = (int32_t)left.size(-1); r.n = (int32_t)right.size(-1);
  auto xyz = [](const TensorLayout& l, int32_t* s) {
    s[0] = (int32_t)l.stride(-1); s[1] = (int32_t)l.stride(-2);
    s[2] = l.dims.size() > 2 ? (int32_t)l.stride(-3) : 0;  // rank-2 operands broadcast (:868-880)
  };
  xyz(out, r.so); xyz(left, r.sl); xyz(right, r.sr);
  r.store = o.store_.lower(); r.load = o.load_.lower(); r.mask = (uint32_t)o.mask_;
  return r;
}

struct CommonKernels {
  virtual ~CommonKernels() = default;
  virtual void matmul_f16(TensorView<f16>& output, const TensorView<const f16>& left,
                          const TensorView<const f16>& right, const MatmulOptions& options) = 0;
  virtual void matmul_f16_slow(TensorView<f16>& output, const TensorView<const f16>& left,
                               const TensorView<const f16>& right, const MatmulOptions& options) = 0;
  virtual void softmax_rows_inplace(TensorView<f16>& output, float temperature) = 0;
  // Not in the reference's trait: the three calls of llama.rs:541-554 (QK^T with Scale and the
  // mask, softmax_rows_inplace, P.V) as one launch.  query/output: [heads, m, d] views, key/value:
  // [heads, n, d] views (rank 2 = one head).
  virtual void attention_f16(TensorView<f16>& output, const TensorView<const f16>& query,
                             const TensorView<const f16>& key, const TensorView<const f16>& value,
                             float scale, float temperature, MatmulMask mask) = 0;
  virtual void error_stats_f16(TensorView<float>& output, const TensorView<const f16>& lhs,
                               const TensorView<const f16>& rhs) = 0;
  virtual void error_stats_f32(TensorView<float>& output, const TensorView<const float>& lhs,
                               const TensorView<const float>& rhs) = 0;
};

// TensorGpuDescriptor::from (kernels.rs:38-55): dims and strides reversed, innermost first.
template <typename T>
inline adr_tensor_desc descriptor(const TensorView<T>& v) {
  adr_tensor_desc d{};
  d.ptr = (void*)v.ptr;
  d.dims = (uint32_t)v.layout.dims.size();
  for (size_t i = 0; i < v.layout.dims.size(); i++) {
    d.shape[i] = (uint32_t)v.layout.dims[v.layout.dims.size() - 1 - i];
    d.strides[i] = (uint32_t)v.layout.strides[v.layout.dims.size() - 1 - i];
  }
  return d;
}

class GpuKernels : public CommonKernels {
 public:
  // `workspace`: optional device buffer (16-byte aligned) the caller owns for as long as this
  // object lives; with it, products with few output tiles and a long K are split over K
  // (adr_matmul_f16_ws).  Calls on one object must not overlap in time when it is set.
  explicit GpuKernels(adr_stream_t stream = nullptr, void* workspace = nullptr, int64_t workspace_bytes = 0)
      : stream_(stream), workspace_(workspace), workspace_bytes_(workspace ? workspace_bytes : 0) {}
  void matmul_f16(TensorView<f16>& o, const TensorView<const f16>& l, const TensorView<const f16>& r,
                  const MatmulOptions& opt) override {
    if (workspace_bytes_ <= 0) return run(adr_matmul_f16, "matmul_f16", o, l, r, opt);
    LoweredMatmul w = lower_matmul(o.layout, l.layout, r.layout, opt);
    int rc = adr_matmul_f16_ws(stream_, o.ptr, l.ptr, r.ptr, w.batches, w.m, w.k, w.n, w.so[0], w.so[1], w.so[2],
                               w.sl[0], w.sl[1], w.sl[2], w.sr[0], w.sr[1], w.sr[2], opt.store_.bias, w.beta,
                               w.scale, w.store, w.load, w.mask, workspace_, workspace_bytes_);
    if (rc) throw AdrasteaError(rc, "matmul_f16");
  }
  void matmul_f16_slow(TensorView<f16>& o, const TensorView<const f16>& l, const TensorView<const f16>& r,
                       const MatmulOptions& opt) override { run(adr_matmul_f16_slow, "matmul_f16_slow", o, l, r, opt); }
  // kernels.rs:892-915: rows = size(-2), heads = size(-3) (1 for rank 2), width = size(-1); like
  // the reference's kernel, the view is taken to be contiguous.
  void softmax_rows_inplace(TensorView<f16>& o, float temperature) override {
    if (!(o.layout == TensorLayout::row_major(o.layout.dims))) throw std::logic_error("softmax_rows: contiguous view");
    const int32_t heads = o.layout.dims.size() > 2 ? (int32_t)o.size(-3) : 1;
    int rc = adr_softmax_rows(stream_, o.ptr, o.ptr, heads, (int32_t)o.size(-2), (int32_t)o.size(-1), temperature);
    if (rc) throw AdrasteaError(rc, "softmax_rows_inplace");
  }
  void attention_f16(TensorView<f16>& o, const TensorView<const f16>& q, const TensorView<const f16>& k,
                     const TensorView<const f16>& v, float scale, float temperature, MatmulMask mask) override {
    const size_t rank = q.layout.dims.size();
    if ((rank != 2 && rank != 3) || o.layout.dims.size() != rank || k.layout.dims.size() != rank ||
        v.layout.dims.size() != rank)
      throw std::logic_error("attention_f16: rank 2 or 3 views");
    const int32_t heads = rank == 3 ? (int32_t)q.size(-3) : 1;
    const int32_t m = (int32_t)q.size(-2), d = (int32_t)q.size(-1), n = (int32_t)k.size(-2);
    if ((int32_t)k.size(-1) != d || (int32_t)v.size(-1) != d || (int32_t)v.size(-2) != n ||
        (int32_t)o.size(-2) != m || (int32_t)o.size(-1) != d ||
        (rank == 3 && ((int32_t)o.size(-3) != heads || (int32_t)k.size(-3) != heads || (int32_t)v.size(-3) != heads)))
      throw std::logic_error("attention_f16: shape mismatch");
    auto z = [&](const TensorLayout& l) { return rank == 3 ? (int32_t)l.stride(-3) : 0; };
    int rc = adr_attention_f16(stream_, o.ptr, q.ptr, k.ptr, v.ptr, heads, m, n, d,
                               (int32_t)o.layout.stride(-1), (int32_t)o.layout.stride(-2), z(o.layout),
                               (int32_t)q.layout.stride(-1), (int32_t)q.layout.stride(-2), z(q.layout),
                               (int32_t)k.layout.stride(-1), (int32_t)k.layout.stride(-2), z(k.layout),
                               (int32_t)v.layout.stride(-1), (int32_t)v.layout.stride(-2), z(v.layout),
                               scale, temperature, (uint32_t)mask);
    if (rc) throw AdrasteaError(rc, "attention_f16");
  }
  // kernels.rs:717-751: both operands flattened with shape_cast(&[-1]); equal lengths
  void error_stats_f16(TensorView<float>& out, const TensorView<const f16>& l, const TensorView<const f16>& r) override {
    auto lf = l.shape_cast({-1}), rf = r.shape_cast({-1});
    if (lf.size(-1) != rf.size(-1)) throw std::logic_error("error_stats: length mismatch");
    int rc = adr_error_stats_f16(stream_, descriptor(out), descriptor(lf), descriptor(rf));
    if (rc) throw AdrasteaError(rc, "error_stats_f16");
  }
  void error_stats_f32(TensorView<float>& out, const TensorView<const float>& l, const TensorView<const float>& r) override {
    auto lf = l.shape_cast({-1}), rf = r.shape_cast({-1});
    if (lf.size(-1) != rf.size(-1)) throw std::logic_error("error_stats: length mismatch");
    int rc = adr_error_stats_f32(stream_, descriptor(out), descriptor(lf), descriptor(rf));
    if (rc) throw AdrasteaError(rc, "error_stats_f32");
  }
  std::string plan(const TensorLayout& o, const TensorLayout& l, const TensorLayout& r, const MatmulOptions& opt) const {
    LoweredMatmul w = lower_matmul(o, l, r, opt);
    char name[64];
    int rc = adr_matmul_f16_plan(name, sizeof name, w.batches, w.m, w.k, w.n, w.so[0], w.so[1], w.so[2], w.sl[0],
                                 w.sl[1], w.sl[2], w.sr[0], w.sr[1], w.sr[2], w.store, w.load, w.mask);
    if (rc) throw AdrasteaError(rc, "matmul_f16_plan");
    return name;
  }

 private:
  template <typename F>
  void run(F fn, const char* what, TensorView<f16>& o, const TensorView<const f16>& l,
           const TensorView<const f16>& r, const MatmulOptions& opt) {
    LoweredMatmul w = lower_matmul(o.layout, l.layout, r.layout, opt);
    int rc = fn(stream_, o.ptr, l.ptr, r.ptr, w.batches, w.m, w.k, w.n, w.so[0], w.so[1], w.so[2], w.sl[0], w.sl[1],
                w.sl[2], w.sr[0], w.sr[1], w.sr[2], opt.store_.bias, w.beta, w.scale, w.store, w.load, w.mask);
    if (rc) throw AdrasteaError(rc, what);
  }
  adr_stream_t stream_;
  void* workspace_;
  int64_t workspace_bytes_;
};

// Records the set of (left, right, output) layouts seen, then forwards (kernels.rs:231-359).
class MatmulTracer : public CommonKernels {
 public:
  explicit MatmulTracer(CommonKernels& inner) : inner_(inner) {}
  void clear() { std::lock_guard<std::mutex> g(mu_); shapes_.clear(); }
  std::set<std::tuple<TensorLayout, TensorLayout, TensorLayout>> shapes() { std::lock_guard<std::mutex> g(mu_); return shapes_; }
  void matmul_f16(TensorView<f16>& o, const TensorView<const f16>& l, const TensorView<const f16>& r,
                  const MatmulOptions& opt) override { rec(o, l, r); inner_.matmul_f16(o, l, r, opt); }
  void matmul_f16_slow(TensorView<f16>& o, const TensorView<const f16>& l, const TensorView<const f16>& r,
                       const MatmulOptions& opt) override { rec(o, l, r); inner_.matmul_f16_slow(o, l, r, opt); }
  void softmax_rows_inplace(TensorView<f16>& o, float t) override { inner_.softmax_rows_inplace(o, t); }
  void attention_f16(TensorView<f16>& o, const TensorView<const f16>& q, const TensorView<const f16>& k,
                     const TensorView<const f16>& v, float scale, float t, MatmulMask mask) override {
    inner_.attention_f16(o, q, k, v, scale, t, mask);
  }
  void error_stats_f16(TensorView<float>& out, const TensorView<const f16>& l, const TensorView<const f16>& r) override { inner_.error_stats_f16(out, l, r); }
  void error_stats_f32(TensorView<float>& out, const TensorView<const float>& l, const TensorView<const float>& r) override { inner_.error_stats_f32(out, l, r); }

 private:
  void rec(const TensorView<f16>& o, const TensorView<const f16>& l, const TensorView<const f16>& r) {
    std::lock_guard<std::mutex> g(mu_);
    shapes_.insert(std::make_tuple(l.layout, r.layout, o.layout));
  }
  CommonKernels& inner_;
  std::mutex mu_;
  std::set<std::tuple<TensorLayout, TensorLayout, TensorLayout>> shapes_;
};

}  // namespace adrastea

// wkf_tensor.hpp -- a typed host facade over the C ABI of wkf_tensor.h, header-only, C++17.
//
// The reference's public type is `Tensor<const R: usize, D: DataType>` (src/tensor.rs:418-644, re-exported by
// src/lib.rs:1-11): the rank and the element type are part of the type, so a reduce yields `Tensor<R - 1, D>`, a
// `broadcast` names its output rank, `mat_mul` only exists for rank 2 and a mismatch is a compile error.  This header
// is that surface for a C++ host: `wkf::Tensor<R, D>` with the same method names, the same operator set
// (tensor-with-literal on both sides, tensor-with-tensor, unary minus) and the same laziness -- every call only records
// a node through one C entry point; `as_slice()` materialises and downloads.  Where the reference panics this throws
// `wkf::Error` carrying the status code and the text of wkf_last_error().
//
// It adds nothing to the C ABI and holds no state of its own beyond the handles.
#ifndef WKF_TENSOR_HPP
#define WKF_TENSOR_HPP

#include <array>
#include <cstdint>
#include <cstring>
#include <initializer_list>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "wkf_tensor.h"

namespace wkf {

// A failed call: the reference's panics and `Result::Err`s (src/tensor.rs:551-554) as one exception type.
struct Error : std::runtime_error {
  int code;
  Error(int c, const std::string& what) : std::runtime_error(what), code(c) {}
};
inline void check(int rc) {
  if (rc != WKF_OK) throw Error(rc, wkf_last_error());
}

// `DataType` (src/tensor.rs:20-67): the element types a tensor can hold.  F16 values cross this boundary as their
// 16 bits (`Half`); `Half::from_float` / `to_float` convert with round-to-nearest-even.
struct Half {
  uint16_t bits;
  static Half from_float(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    x &= 0x7fffffffu;
    if (x >= 0x7f800000u) return Half{uint16_t(sign | 0x7c00u | (x > 0x7f800000u ? 0x200u : 0u))};  // inf, NaN
    if (x >= 0x477ff000u) return Half{uint16_t(sign | 0x7c00u)};                                    // rounds to inf
    if (x < 0x33000001u) return Half{uint16_t(sign)};                                               // rounds to zero
    int e = int(x >> 23) - 127;
    uint32_t m = (x & 0x7fffffu) | 0x800000u;  // 24-bit significand
    int shift = 13;                             // bits dropped for a normal result
    if (e < -14) {                              // subnormal result
      shift += -14 - e;
      e = -15;
    }
    const uint32_t kept = m >> shift, rest = m & ((1u << shift) - 1u), halfway = 1u << (shift - 1);
    uint32_t h = (uint32_t(e + 15) << 10) + (kept - (e == -15 ? 0u : 0x400u));
    if (rest > halfway || (rest == halfway && (kept & 1u))) h++;  // a carry into the exponent is the right result
    return Half{uint16_t(sign | h)};
  }
  float to_float() const {
    const uint32_t sign = uint32_t(bits & 0x8000u) << 16, e = (bits >> 10) & 31u, m = bits & 0x3ffu;
    uint32_t x;
    if (e == 31u) x = sign | 0x7f800000u | (m << 13);
    else if (e != 0u) x = sign | ((e + 112u) << 23) | (m << 13);
    else if (m == 0u) x = sign;
    else {
      int s = 0;
      uint32_t mm = m;
      while (!(mm & 0x400u)) { mm <<= 1; s++; }
      x = sign | (uint32_t(113 - s) << 23) | ((mm & 0x3ffu) << 13);
    }
    float f;
    std::memcpy(&f, &x, 4);
    return f;
  }
};
struct F32 {
  using host_type = float;
  static constexpr int id = WKF_F32;
  static float to_float(float v) { return v; }
  static float from_float(float v) { return v; }
};
struct F16 {
  using host_type = Half;
  static constexpr int id = WKF_F16;
  static float to_float(Half v) { return v.to_float(); }
  static Half from_float(float v) { return Half::from_float(v); }
};

// `Device` (src/device.rs:9-48).  Copies share the device; it is released with the last copy (and, inside the
// library, only once the last buffer on it is gone).
class Device {
 public:
  // Device::new, src/device.rs:14-32: the GPU with this ordinal.
  static Device create(int ordinal = 0) {
    wkf_device* d = nullptr;
    check(wkf_device_create(ordinal, &d));
    return Device(d);
  }
  // A device with no GPU behind it: every kernel is planned and compiled, nothing runs, and reading a computed
  // tensor back fails with WKF_ERR_NO_DEVICE.
  static Device planner() {
    wkf_device* d = nullptr;
    check(wkf_device_create_planner(&d));
    return Device(d);
  }
  wkf_device* handle() const { return h_.get(); }
  void sync() const { check(wkf_device_sync(h_.get())); }
  void set_fusion(int mode) const { check(wkf_device_set_fusion(h_.get(), mode)); }
  void set_reference_compat(bool on) const { check(wkf_device_set_reference_compat(h_.get(), on ? 1 : 0)); }
  wkf_props props() const {
    wkf_props p;
    check(wkf_device_props(h_.get(), &p));
    return p;
  }

 private:
  explicit Device(wkf_device* d) : h_(d, [](wkf_device* p) { wkf_device_destroy(p); }) {}
  std::shared_ptr<wkf_device> h_;
};

// One launched kernel of the last materialisation: `QueryResults` of src/query.rs:9-48.
struct KernelInfo {
  uint64_t elapsed_ns;
  std::string kind, signature, detail;
};

// A half-open index range per dimension: the reference's `Range<usize>` (`0..2`).
using Range = std::pair<size_t, size_t>;

template <int R, class D>
class TensorSlice;

// `Tensor<const R: usize, D: DataType>`, src/tensor.rs:418-644.
template <int R, class D = F32>
class Tensor {
  static_assert(R >= 0, "rank");

 public:
  using element = typename D::host_type;
  static constexpr int rank_v = R;

  // Tensor::new, src/tensor.rs:518-531: row-major data of the given shape (the nested-array forms of `IntoTensor`,
  // :646-760, become shape + flat data).
  Tensor(const Device& dev, const std::array<size_t, size_t(R)>& shape, const element* data) {
    check(wkf_tensor_new(dev.handle(), D::id, R, shape.data(), data, &h_));
  }
  Tensor(const Device& dev, const std::array<size_t, size_t(R)>& shape, const std::vector<element>& data) {
    size_t n = 1;
    for (size_t d : shape) n *= d;
    if (data.size() != n) throw Error(WKF_ERR_INVALID_ARG, "Tensor: the data does not fill the shape");
    check(wkf_tensor_new(dev.handle(), D::id, R, shape.data(), data.data(), &h_));
  }
  // from f32 literals, converted to the element type (what the reference's tests write)
  static Tensor from_floats(const Device& dev, const std::array<size_t, size_t(R)>& shape, std::initializer_list<float> values) {
    std::vector<element> v;
    v.reserve(values.size());
    for (float f : values) v.push_back(D::from_float(f));
    return Tensor(dev, shape, v);
  }
  // The nested-array forms of `IntoTensor` (src/tensor.rs:646-760): `Tensor::new(&device, &[[1., 2.], [3., 4.]])` is
  // `Tensor<2>::from(dev, {{1, 2}, {3, 4}})`; every row (and every matrix of a rank-3 literal) must have the same length.
  static Tensor from(const Device& dev, std::initializer_list<float> v) {
    static_assert(R == 1, "a flat list is a rank-1 tensor");
    return from_floats(dev, {v.size()}, v);
  }
  static Tensor from(const Device& dev, std::initializer_list<std::initializer_list<float>> rows) {
    static_assert(R == 2, "a list of lists is a rank-2 tensor");
    const size_t cols = rows.size() ? rows.begin()->size() : 0;
    std::vector<element> flat;
    for (const auto& r : rows) {
      if (r.size() != cols) throw Error(WKF_ERR_INVALID_ARG, "Tensor::from: rows of different lengths");
      for (float f : r) flat.push_back(D::from_float(f));
    }
    return Tensor(dev, {rows.size(), cols}, flat);
  }
  static Tensor from(const Device& dev, std::initializer_list<std::initializer_list<std::initializer_list<float>>> mats) {
    static_assert(R == 3, "a list of lists of lists is a rank-3 tensor");
    const size_t rows = mats.size() ? mats.begin()->size() : 0;
    const size_t cols = rows ? mats.begin()->begin()->size() : 0;
    std::vector<element> flat;
    for (const auto& m : mats) {
      if (m.size() != rows) throw Error(WKF_ERR_INVALID_ARG, "Tensor::from: matrices of different heights");
      for (const auto& r : m) {
        if (r.size() != cols) throw Error(WKF_ERR_INVALID_ARG, "Tensor::from: rows of different lengths");
        for (float f : r) flat.push_back(D::from_float(f));
      }
    }
    return Tensor(dev, {mats.size(), rows, cols}, flat);
  }
  // arange / arange_step, src/composite/arange.rs:4-12 (rank 1)
  static Tensor arange(const Device& dev, float start, float end, float step = 1.0f) {
    static_assert(R == 1, "arange builds a rank-1 tensor");
    wkf_tensor* o = nullptr;
    check(wkf_tensor_arange(dev.handle(), D::id, start, end, step, &o));
    return Tensor(o);
  }

  Tensor(const Tensor& o) { check(wkf_tensor_clone(o.h_, &h_)); }  // Clone: another handle on the same node
  Tensor(Tensor&& o) noexcept : h_(o.h_) { o.h_ = nullptr; }
  Tensor& operator=(Tensor o) noexcept {
    std::swap(h_, o.h_);
    return *this;
  }
  ~Tensor() {
    if (h_) wkf_tensor_free(h_);
  }

  // shape / rank / datatype, src/tensor.rs:629-640
  std::array<size_t, size_t(R)> shape() const {
    std::array<size_t, size_t(R)> s{};
    if (wkf_tensor_rank(h_) != R) throw Error(WKF_ERR_INVALID_ARG, "Tensor: the handle's rank differs from the type's");
    check(wkf_tensor_shape(h_, s.data()));
    return s;
  }
  static constexpr size_t rank() { return size_t(R); }
  static constexpr int datatype() { return D::id; }

  // ---- tensor with literal, src/element_wise.rs:197-675 ----
  friend Tensor operator+(const Tensor& t, float c) { return t.scalar(WKF_OP_ADD_CONST, c); }
  friend Tensor operator+(float c, const Tensor& t) { return t.scalar(WKF_OP_ADD_CONST, c); }
  friend Tensor operator-(const Tensor& t, float c) { return t.scalar(WKF_OP_SUB_CONST, c); }
  friend Tensor operator-(float c, const Tensor& t) { return t.scalar(WKF_OP_CONST_SUB, c); }
  friend Tensor operator*(const Tensor& t, float c) { return t.scalar(WKF_OP_MUL_CONST, c); }
  friend Tensor operator*(float c, const Tensor& t) { return t.scalar(WKF_OP_MUL_CONST, c); }
  friend Tensor operator/(const Tensor& t, float c) { return t.scalar(WKF_OP_DIV_CONST, c); }
  friend Tensor operator/(float c, const Tensor& t) { return t.scalar(WKF_OP_CONST_DIV, c); }
  // ---- unary, src/element_wise.rs:678-1380 ----
  Tensor exp() const { return unary(WKF_OP_EXP); }
  Tensor exp2() const { return unary(WKF_OP_EXP2); }
  Tensor log() const { return unary(WKF_OP_LOG); }
  Tensor log2() const { return unary(WKF_OP_LOG2); }
  Tensor sqr() const { return unary(WKF_OP_SQR); }
  Tensor sqrt() const { return unary(WKF_OP_SQRT); }
  Tensor sin() const { return unary(WKF_OP_SIN); }
  Tensor cos() const { return unary(WKF_OP_COS); }
  Tensor tan() const { return unary(WKF_OP_TAN); }
  Tensor asin() const { return unary(WKF_OP_ASIN); }
  Tensor acos() const { return unary(WKF_OP_ACOS); }
  Tensor atan() const { return unary(WKF_OP_ATAN); }
  Tensor sinh() const { return unary(WKF_OP_SINH); }
  Tensor cosh() const { return unary(WKF_OP_COSH); }
  Tensor tanh() const { return unary(WKF_OP_TANH); }
  Tensor asinh() const { return unary(WKF_OP_ASINH); }
  Tensor acosh() const { return unary(WKF_OP_ACOSH); }
  Tensor atanh() const { return unary(WKF_OP_ATANH); }
  Tensor abs() const { return unary(WKF_OP_ABS); }
  Tensor operator-() const { return unary(WKF_OP_NEG); }
  // cast, src/element_wise.rs:1408-1471
  template <class D2>
  Tensor<R, D2> cast() const {
    wkf_tensor* o = nullptr;
    check(wkf_tensor_cast(h_, D2::id, &o));
    return Tensor<R, D2>::adopt(o);
  }
  // ---- tensor with tensor, src/pair_wise.rs:205-528: equal rank and element type by construction ----
  friend Tensor operator+(const Tensor& a, const Tensor& b) { return a.binary(b, WKF_OP_ADD); }
  friend Tensor operator-(const Tensor& a, const Tensor& b) { return a.binary(b, WKF_OP_SUB); }
  friend Tensor operator*(const Tensor& a, const Tensor& b) { return a.binary(b, WKF_OP_MUL); }
  friend Tensor operator/(const Tensor& a, const Tensor& b) { return a.binary(b, WKF_OP_DIV); }
  Tensor pow(const Tensor& other) const { return binary(other, WKF_OP_POW); }
  // ---- reductions along one axis, src/reduce.rs:433-815: the result has one dimension fewer ----
  Tensor<R - 1, D> sum(size_t dim) const { return reduce(WKF_REDUCE_SUM, dim); }
  Tensor<R - 1, D> max(size_t dim) const { return reduce(WKF_REDUCE_MAX, dim); }
  Tensor<R - 1, D> min(size_t dim) const { return reduce(WKF_REDUCE_MIN, dim); }
  Tensor<R - 1, D> product(size_t dim) const { return reduce(WKF_REDUCE_PRODUCT, dim); }
  // mat_mul, src/matmul.rs:25-29 (rank 2 there; equal ranks above 2 multiply matrix by matrix over the leading
  // dimensions)
  Tensor mat_mul(const Tensor& other) const {
    static_assert(R >= 2, "mat_mul needs matrices");
    wkf_tensor* o = nullptr;
    check(wkf_tensor_mat_mul(h_, other.h_, &o));
    return Tensor(o);
  }
  // ---- views, src/map_layout.rs:41-99, src/composite/narrow.rs ----
  Tensor slice(const std::array<Range, size_t(R)>& ranges) const {
    size_t b[R > 0 ? R : 1], e[R > 0 ? R : 1];
    for (int i = 0; i < R; i++) {
      b[i] = ranges[size_t(i)].first;
      e[i] = ranges[size_t(i)].second;
    }
    wkf_tensor* o = nullptr;
    check(wkf_tensor_slice(h_, b, e, &o));
    return Tensor(o);
  }
  Tensor transpose(size_t first_axis, size_t second_axis) const {
    wkf_tensor* o = nullptr;
    check(wkf_tensor_transpose(h_, first_axis, second_axis, &o));
    return Tensor(o);
  }
  template <int R2>
  Tensor<R2, D> broadcast(const std::array<size_t, size_t(R2)>& out_shape) const {
    static_assert(R2 == R + 1, "broadcast adds one leading dimension (src/map_layout.rs:69-77)");
    wkf_tensor* o = nullptr;
    check(wkf_tensor_broadcast(h_, R2, out_shape.data(), &o));
    return Tensor<R2, D>::adopt(o);
  }
  Tensor narrow(size_t axis, size_t start, size_t length) const {
    wkf_tensor* o = nullptr;
    check(wkf_tensor_narrow(h_, axis, start, length, &o));
    return Tensor(o);
  }
  // ---- copies, src/resize.rs:121-145, src/slice_assign.rs:76-80, src/composite/cat.rs ----
  Tensor resize(const std::array<size_t, size_t(R)>& new_shape) const {
    wkf_tensor* o = nullptr;
    check(wkf_tensor_resize(h_, new_shape.data(), &o));
    return Tensor(o);
  }
  template <int R2>
  Tensor<R2, D> reshape(const std::array<size_t, size_t(R2)>& new_shape) const {
    wkf_tensor* o = nullptr;
    check(wkf_tensor_reshape(h_, R2, new_shape.data(), &o));
    return Tensor<R2, D>::adopt(o);
  }
  Tensor<R + 1, D> unsqueeze(size_t axis) const {
    wkf_tensor* o = nullptr;
    check(wkf_tensor_unsqueeze(h_, axis, &o));
    return Tensor<R + 1, D>::adopt(o);
  }
  Tensor slice_assign(const std::array<Range, size_t(R)>& ranges, const Tensor& value) const {
    size_t b[R > 0 ? R : 1], e[R > 0 ? R : 1];
    for (int i = 0; i < R; i++) {
      b[i] = ranges[size_t(i)].first;
      e[i] = ranges[size_t(i)].second;
    }
    wkf_tensor* o = nullptr;
    check(wkf_tensor_slice_assign(h_, b, e, value.h_, &o));
    return Tensor(o);
  }
  static Tensor cat(const std::vector<Tensor>& tensors, size_t dim) {
    std::vector<const wkf_tensor*> hs;
    for (const Tensor& t : tensors) hs.push_back(t.h_);
    wkf_tensor* o = nullptr;
    check(wkf_tensor_cat(hs.data(), int(hs.size()), dim, &o));
    return Tensor(o);
  }
  // ---- composites, src/composite/*.rs ----
  Tensor silu() const {
    wkf_tensor* o = nullptr;
    check(wkf_tensor_silu(h_, &o));
    return Tensor(o);
  }
  Tensor layer_norm(const Tensor<1, D>& weight, float eps) const {
    static_assert(R == 2, "layer_norm is defined on [rows, hidden] (src/composite/rms_norm.rs:7-8)");
    wkf_tensor* o = nullptr;
    check(wkf_tensor_layer_norm(h_, weight.handle(), eps, &o));
    return Tensor(o);
  }
  Tensor rope(const Tensor<2, D>& cos, const Tensor<2, D>& sin) const {
    static_assert(R == 3, "rope is defined on [heads, sequence, embed] (src/composite/rope.rs:12-13)");
    wkf_tensor* o = nullptr;
    check(wkf_tensor_rope(h_, cos.handle(), sin.handle(), &o));
    return Tensor(o);
  }
  Tensor softmax() const {
    static_assert(R == 1, "softmax is defined on rank 1 (src/composite/softmax.rs:3-4); softmax_last_dim takes any rank");
    wkf_tensor* o = nullptr;
    check(wkf_tensor_softmax(h_, &o));
    return Tensor(o);
  }
  Tensor softmax_last_dim() const {
    wkf_tensor* o = nullptr;
    check(wkf_tensor_softmax_last_dim(h_, &o));
    return Tensor(o);
  }
  // ---- running the graph ----
  void materialize() const { check(wkf_tensor_materialize(h_)); }
  // as_slice, src/tensor.rs:551-554 (blocking: there is no executor to await on)
  TensorSlice<R, D> as_slice() const;
  // all_timing_information, src/tensor.rs:556-558
  std::vector<KernelInfo> all_timing_information() const {
    std::vector<KernelInfo> out;
    const int n = wkf_tensor_kernel_count(h_);
    for (int i = 0; i < n; i++) {
      char kind[64], sig[4096], detail[1024];
      uint64_t ns = 0;
      check(wkf_tensor_kernel_info(h_, i, &ns, kind, sizeof kind, sig, sizeof sig, detail, sizeof detail));
      out.push_back({ns, kind, sig, detail});
    }
    return out;
  }
  // graphvis, src/tensor.rs:641-643: the lazy graph as DOT text
  std::string graphvis() const {
    size_t needed = 0;
    check(wkf_tensor_graphvis(h_, nullptr, 0, &needed));
    std::string s(needed, '\0');
    check(wkf_tensor_graphvis(h_, &s[0], s.size(), &needed));
    s.resize(std::strlen(s.c_str()));
    return s;
  }

  wkf_tensor* handle() const { return h_; }
  // takes ownership of a handle whose rank and element type the caller vouches for (checked)
  static Tensor adopt(wkf_tensor* h) {
    if (wkf_tensor_rank(h) != R || wkf_tensor_dtype(h) != D::id) {
      wkf_tensor_free(h);
      throw Error(WKF_ERR_INVALID_ARG, "Tensor: the handle's rank or element type differs from the type's");
    }
    return Tensor(h);
  }

 private:
  explicit Tensor(wkf_tensor* h) : h_(h) {}
  Tensor scalar(int op, float c) const {
    wkf_tensor* o = nullptr;
    check(wkf_tensor_scalar_op(h_, op, c, &o));
    return Tensor(o);
  }
  Tensor unary(int op) const {
    wkf_tensor* o = nullptr;
    check(wkf_tensor_unary_op(h_, op, &o));
    return Tensor(o);
  }
  Tensor binary(const Tensor& b, int op) const {
    wkf_tensor* o = nullptr;
    check(wkf_tensor_binary_op(h_, b.h_, op, &o));
    return Tensor(o);
  }
  Tensor<R - 1, D> reduce(int op, size_t dim) const {
    static_assert(R >= 1, "a rank-0 tensor has no axis to reduce");
    wkf_tensor* o = nullptr;
    check(wkf_tensor_reduce(h_, op, dim, &o));
    return Tensor<R - 1, D>::adopt(o);
  }
  wkf_tensor* h_ = nullptr;
  template <int, class>
  friend class Tensor;
};

// `TensorSlice<R, D>`, src/tensor.rs:762-870: the downloaded buffer plus the layout that indexes it.
template <int R, class D>
class TensorSlice {
 public:
  using element = typename D::host_type;
  explicit TensorSlice(wkf_slice* s) : s_(s, [](wkf_slice* p) { wkf_slice_free(p); }) {
    if (wkf_slice_rank(s) != R || wkf_slice_dtype(s) != D::id) throw Error(WKF_ERR_INVALID_ARG, "TensorSlice: rank or element type mismatch");
    check(wkf_slice_layout(s, &offset_, shape_.data(), strides_.data()));
  }
  const std::array<size_t, size_t(R)>& shape() const { return shape_; }
  // TensorSlice::get, :827-846: the element, or nothing when an index is out of range
  bool get(const std::array<size_t, size_t(R)>& index, float* out) const { return wkf_slice_get(s_.get(), index.data(), out) == WKF_OK; }
  // Index<[usize; R]>, :848-857
  float operator[](const std::array<size_t, size_t(R)>& index) const {
    float v = 0;
    if (!get(index, &v)) throw Error(WKF_ERR_INVALID_ARG, "TensorSlice: index out of range");
    return v;
  }
  // every element in row-major order, widened to f32
  std::vector<float> to_floats() const {
    size_t bytes = 0;
    const element* base = static_cast<const element*>(wkf_slice_data(s_.get(), &bytes));
    size_t n = 1;
    for (size_t d : shape_) n *= d;
    std::vector<float> out(n);
    std::array<size_t, size_t(R)> idx{};
    for (size_t k = 0; k < n; k++) {
      size_t at = offset_;
      for (int d = 0; d < R; d++) at += idx[size_t(d)] * strides_[size_t(d)];
      out[k] = D::to_float(base[at]);
      for (int d = R - 1; d >= 0; d--) {
        if (++idx[size_t(d)] < shape_[size_t(d)]) break;
        idx[size_t(d)] = 0;
      }
    }
    return out;
  }

 private:
  std::shared_ptr<wkf_slice> s_;
  size_t offset_ = 0;
  std::array<size_t, size_t(R)> shape_{}, strides_{};
};

template <int R, class D>
TensorSlice<R, D> Tensor<R, D>::as_slice() const {
  wkf_slice* s = nullptr;
  check(wkf_tensor_as_slice(h_, &s));
  return TensorSlice<R, D>(s);
}

}  // namespace wkf
#endif

// Level 1 of the C ABI (include/wkf_tensor.h): the lazy Tensor API of the
// reference behind C handles, plus the composites, which are built from the
// primitive ops exactly as the reference builds them (src/composite/*.rs).
#include "wkf_tensor.h"

#include <cmath>
#include <cstring>
#include <mutex>
#include <sstream>
#include <unordered_map>

#include "graph.h"

using namespace wkf;

// hip_ffi.cpp owns the thread-local error string; this hook lets the upper layers set it.
void wkf_set_last_error_(const char* msg);
void wkf_add_destroy_hook_(void (*fn)(wkf_device*));

struct wkf_tensor {
  wkf_device* dev;
  NodeP node;
  std::vector<LaunchRecord> launches;  // of the last materialize
};

struct wkf_slice {
  std::vector<unsigned char> bytes;
  Layout layout;
  DType dtype;
};

namespace wkf {
// signature -> generated source, for inspection (filled by Resolver::kernel)
std::mutex g_source_mu;
std::unordered_map<std::string, std::string> g_sources;

// f32 -> f16 bits, round to nearest even, overflow to infinity (what half::f16::from_f32 does).
uint16_t f32_to_f16_bits(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t exp = (x >> 23) & 0xff;
  uint32_t man = x & 0x7fffffu;
  if (exp == 0xff) return uint16_t(sign | 0x7c00u | (man ? 0x200u | (man >> 13) : 0));
  int e = int(exp) - 127 + 15;
  if (e >= 31) return uint16_t(sign | 0x7c00u);
  if (e <= 0) {
    if (e < -10) return uint16_t(sign);
    man |= 0x800000u;
    int shift = 14 - e;
    uint32_t half = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1);
    uint32_t mid = 1u << (shift - 1);
    if (rem > mid || (rem == mid && (half & 1))) half++;
    return uint16_t(sign | half);
  }
  uint32_t half = (uint32_t(e) << 10) | (man >> 13);
  uint32_t rem = man & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (half & 1))) half++;
  return uint16_t(sign | half);
}

float f16_bits_to_f32(uint16_t h) {
  uint32_t sign = uint32_t(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1f;
  uint32_t man = h & 0x3ffu;
  uint32_t x;
  if (exp == 0) {
    if (man == 0) x = sign;
    else {
      int e = -1;
      do {
        e++;
        man <<= 1;
      } while (!(man & 0x400u));
      x = sign | uint32_t(127 - 15 - e) << 23 | (man & 0x3ffu) << 13;
    }
  } else if (exp == 31) x = sign | 0x7f800000u | man << 13;
  else x = sign | (exp - 15 + 127) << 23 | man << 13;
  float f;
  memcpy(&f, &x, 4);
  return f;
}
}  // namespace wkf

namespace {

std::mutex g_settings_mu;
std::unordered_map<wkf_device*, Settings> g_settings;

void forget_device(wkf_device* dev) {
  std::lock_guard<std::mutex> lock(g_settings_mu);
  g_settings.erase(dev);
}

Settings settings_for(wkf_device* dev) {
  static const bool hooked = (wkf_add_destroy_hook_(&forget_device), true);
  (void)hooked;
  std::lock_guard<std::mutex> lock(g_settings_mu);
  auto it = g_settings.find(dev);
  if (it == g_settings.end()) {
    // tuning knobs read once per device
    Settings st;
    if (const char* u = getenv("WKF_MAP_UNROLL")) {
      int v = atoi(u);
      if (v == 1 || v == 2 || v == 4 || v == 8) st.map_unroll = v;
    }
    if (const char* nt = getenv("WKF_NONTEMPORAL_BYTES")) st.nontemporal_bytes = size_t(atoll(nt));
    if (const char* t = getenv("WKF_REDUCE_THREADS")) {
      int v = atoi(t);
      if (v >= 1 && v <= 1024 && (v & (v - 1)) == 0) st.reduce_threads = v;
    }
    if (const char* t = getenv("WKF_ROW_THREADS")) {
      int v = atoi(t);
      if (v >= 1 && v <= 1024 && (v & (v - 1)) == 0) st.row_threads = v;
    }
    if (const char* u = getenv("WKF_GEMM_T128")) st.gemm_t128 = atoi(u) != 0;
    if (const char* u = getenv("WKF_GEMM_SHORTK")) st.gemm_shortk = atoi(u) != 0;
    if (const char* u = getenv("WKF_GEMM_STREAM")) st.gemm_stream = atoi(u) != 0;
    if (const char* u = getenv("WKF_MAP_TILE_VEC")) st.map_tile_vec = atoi(u) != 0;
    if (const char* u = getenv("WKF_GEMM_TAIL")) st.gemm_tail = atoi(u) != 0;
    if (const char* u = getenv("WKF_GEMM_DMA")) st.gemm_dma = atoi(u) != 0;
    if (const char* u = getenv("WKF_GEMM_FLEX")) st.gemm_flex = !(u[0] == '0' && u[1] == 0);
    if (const char* u = getenv("WKF_MATH_F32")) st.math_f32 = atoi(u) != 0;
    if (const char* u = getenv("WKF_MAP_TILE_128")) st.map_tile_128 = atoi(u) != 0;
    if (const char* u = getenv("WKF_MAP_TABLE_MIN")) st.map_table_min = size_t(std::max(0ll, atoll(u)));
    if (const char* u = getenv("WKF_ROW_SPLIT")) st.row_split = atoi(u) != 0;
    if (const char* u = getenv("WKF_ROW_TEAM")) st.row_team = atoi(u) != 0;
    if (const char* u = getenv("WKF_ROW_STREAM_VECTORS")) {
      int v = atoi(u);
      if (v >= 1 && v <= 8) st.row_stream_vectors = v;
    }
    if (const char* u = getenv("WKF_ROW_STREAM_MIN_ROWS")) st.row_stream_min_rows = size_t(std::max(1ll, atoll(u)));
    if (const char* u = getenv("WKF_SKINNY_TR_ROWS")) {
      int v = atoi(u);
      if (v >= 1 && v <= 33) st.skinny_tr_rows = v;
    }
    if (const char* u = getenv("WKF_SKINNY_BLOCKS")) {
      int v = atoi(u);
      if (v >= 1 && v <= 65536) st.skinny_blocks = v;
    }
    if (const char* u = getenv("WKF_REDUCE_UNROLL")) {
      int v = atoi(u);
      if (v == 1 || v == 2 || v == 4 || v == 8) st.reduce_unroll = v;
    }
    it = g_settings.emplace(dev, st).first;
  }
  return it->second;
}

// Runs `f`, mapping exceptions to status codes + wkf_last_error().
template <typename F>
int guarded(F&& f) {
  try {
    f();
    return WKF_OK;
  } catch (const Error& e) {
    wkf_set_last_error_(e.what());
    return e.code;
  } catch (const std::bad_alloc&) {
    wkf_set_last_error_("host allocation failed");
    return WKF_ERR_OOM;
  } catch (const std::exception& e) {
    wkf_set_last_error_(e.what());
    return WKF_ERR_INVALID_ARG;
  } catch (...) {
    wkf_set_last_error_("unknown exception");
    return WKF_ERR_INVALID_ARG;
  }
}

wkf_tensor* wrap(wkf_device* dev, NodeP n) {
  wkf_tensor* t = new wkf_tensor();
  t->dev = dev;
  t->node = std::move(n);
  return t;
}

void need(const void* p, const char* what) {
  if (!p) invalid(std::string(what) + ": null argument");
}

NodeP make(NodeKind k, DType dt, std::vector<size_t> shape) {
  NodeP n = std::make_shared<Node>();
  n->kind = k;
  n->dtype = dt;
  n->shape = std::move(shape);
  return n;
}

// ---- node constructors (LazyTensorData::*, src/tensor.rs:179-284) -----------

NodeP n_element_wise(const NodeP& in, Op op, float c, DType out_dt) {
  NodeP n = make(NodeKind::ElementWise, out_dt, in->shape);
  n->a = in;
  n->op = op;
  n->constant = c;
  return n;
}
NodeP n_unary(const NodeP& in, Op op) { return n_element_wise(in, op, 0.f, in->dtype); }
NodeP n_scalar(const NodeP& in, Op op, float c) { return n_element_wise(in, op, c, in->dtype); }
NodeP n_cast(const NodeP& in, DType dt) { return in->dtype == dt ? in : n_element_wise(in, Op::Cast, 0.f, dt); }

NodeP n_pair_wise(const NodeP& a, const NodeP& b, Op op) {
  if (a->dtype != b->dtype) invalid("pair-wise op: operand dtypes differ");
  if (a->shape != b->shape) invalid("pair-wise op: operand shapes differ");  // src/pair_wise.rs:92
  NodeP n = make(NodeKind::PairWise, a->dtype, a->shape);
  n->a = a;
  n->b = b;
  n->op = op;
  return n;
}

NodeP n_reduce(const NodeP& in, ReduceOp rop, size_t axis) {
  if (axis >= in->shape.size()) invalid("reduce: axis out of range");
  std::vector<size_t> shape;
  for (size_t d = 0; d < in->shape.size(); d++)
    if (d != axis) shape.push_back(in->shape[d]);  // src/tensor.rs:221-242
  NodeP n = make(NodeKind::Reduce, in->dtype, shape);
  n->a = in;
  n->rop = rop;
  n->axis = axis;
  return n;
}

NodeP n_slice(const NodeP& in, const std::vector<std::pair<size_t, size_t>>& ranges) {
  if (ranges.size() != in->shape.size()) invalid("slice: one range per dimension is required");
  std::vector<size_t> shape;
  for (size_t d = 0; d < ranges.size(); d++) {
    if (ranges[d].first > ranges[d].second || ranges[d].second > in->shape[d]) invalid("slice: range outside the tensor");
    shape.push_back(ranges[d].second - ranges[d].first);
  }
  NodeP n = make(NodeKind::MapLayout, in->dtype, shape);
  n->a = in;
  n->map_kind = MapKind::Slice;
  n->ranges = ranges;
  return n;
}

NodeP n_narrow(const NodeP& in, size_t axis, size_t start, size_t length) {
  if (axis >= in->shape.size()) invalid("narrow: axis out of range");                        // src/composite/narrow.rs:7
  if (start + length > in->shape[axis]) invalid("narrow: start + length exceeds the axis");  // :6
  std::vector<std::pair<size_t, size_t>> r;
  for (size_t d = 0; d < in->shape.size(); d++)
    r.push_back(d == axis ? std::make_pair(start, start + length) : std::make_pair(size_t(0), in->shape[d]));
  return n_slice(in, r);
}

NodeP n_transpose(const NodeP& in, size_t a0, size_t a1) {
  if (a0 >= in->shape.size() || a1 >= in->shape.size()) invalid("transpose: axis out of range");
  std::vector<size_t> shape = in->shape;
  std::swap(shape[a0], shape[a1]);
  NodeP n = make(NodeKind::MapLayout, in->dtype, shape);
  n->a = in;
  n->map_kind = MapKind::Transpose;
  n->axis0 = a0;
  n->axis1 = a1;
  return n;
}

// Insert one broadcast (stride 0) dimension of size `size` at position `axis`.
NodeP n_broadcast_at(const NodeP& in, size_t axis, size_t size) {
  if (axis > in->shape.size()) invalid("broadcast: axis out of range");
  std::vector<size_t> shape = in->shape;
  shape.insert(shape.begin() + axis, size);
  NodeP n = make(NodeKind::MapLayout, in->dtype, shape);
  n->a = in;
  n->map_kind = MapKind::Broadcast;
  n->axis0 = axis;
  n->new_shape = shape;
  return n;
}

// Tensor::broadcast, src/map_layout.rs:69-98: the new dimension goes where the
// shapes first differ (after the last dimension if they never do).
NodeP n_broadcast(const NodeP& in, const std::vector<size_t>& out_shape) {
  const std::vector<size_t>& s = in->shape;
  if (out_shape.size() != s.size() + 1) invalid("broadcast: the output rank must be the input rank + 1");
  size_t new_dim = 0;
  while (new_dim < s.size() && s[new_dim] == out_shape[new_dim]) new_dim++;
  for (size_t i = new_dim; i < s.size(); i++)
    if (s[i] != out_shape[i + 1]) invalid("broadcast: shapes do not line up");  // :78-79
  return n_broadcast_at(in, new_dim, out_shape[new_dim]);
}

NodeP n_resize(const NodeP& in, const std::vector<size_t>& new_shape) {
  if (new_shape.size() != in->shape.size()) invalid("resize: rank must not change");
  NodeP n = make(NodeKind::Resize, in->dtype, new_shape);
  n->a = in;
  n->new_shape = new_shape;
  n->fill_shape = in->shape;  // src/resize.rs:121-129
  return n;
}

NodeP n_reshape(const NodeP& in, const std::vector<size_t>& new_shape) {
  size_t a = 1, b = 1;
  for (size_t d : in->shape) a *= d;
  for (size_t d : new_shape) b *= d;
  if (a != b) invalid("reshape: element counts differ");  // src/resize.rs:132-135
  NodeP n = make(NodeKind::Resize, in->dtype, new_shape);
  n->a = in;
  n->new_shape = new_shape;
  n->fill_shape = new_shape;  // :137-143
  return n;
}

NodeP n_slice_assign(const NodeP& target, const std::vector<std::pair<size_t, size_t>>& ranges, const NodeP& value) {
  if (target->dtype != value->dtype) invalid("slice_assign: dtypes differ");
  if (ranges.size() != target->shape.size() || value->shape.size() != target->shape.size())
    invalid("slice_assign: rank mismatch");
  for (size_t d = 0; d < ranges.size(); d++) {
    if (ranges[d].first > ranges[d].second || ranges[d].second > target->shape[d])
      invalid("slice_assign: range outside the tensor");
    if (ranges[d].second - ranges[d].first != value->shape[d])
      invalid("slice_assign: the value's shape does not match the slice");  // src/slice_assign.rs:69
  }
  NodeP n = make(NodeKind::SliceAssign, target->dtype, target->shape);
  n->a = target;
  n->b = value;
  n->ranges = ranges;
  return n;
}

// Tensor::cat, src/composite/cat.rs:3-41: resize the first piece to the total
// shape, then slice_assign every other piece behind it.
NodeP n_cat(const std::vector<NodeP>& v, size_t dim) {
  if (v.empty()) invalid("cat: no tensors");
  const size_t R = v[0]->shape.size();
  if (dim >= R) {
    // The reference returns a wrongly shaped result here (its rope calls cat(.., 2)
    // on rank-2 tables, src/composite/rope.rs:3,16-17); an out-of-range dim is rejected.
    invalid("cat: dim out of range");
  }
  std::vector<size_t> shape = v[0]->shape;
  shape[dim] = 0;
  for (const NodeP& t : v) {
    if (t->shape.size() != R || t->dtype != v[0]->dtype) invalid("cat: rank or dtype mismatch");
    for (size_t i = 0; i < R; i++) {
      if (i == dim) shape[i] += t->shape[i];
      else if (shape[i] != t->shape[i]) invalid("cat: shapes differ outside the cat dimension");
    }
  }
  NodeP larger = n_resize(v[0], shape);
  size_t index = v[0]->shape[dim];
  for (size_t k = 1; k < v.size(); k++) {
    size_t len = v[k]->shape[dim];
    std::vector<std::pair<size_t, size_t>> r;
    for (size_t i = 0; i < R; i++) r.push_back(i == dim ? std::make_pair(index, index + len) : std::make_pair(size_t(0), shape[i]));
    larger = n_slice_assign(larger, r, v[k]);
    index += len;
  }
  return larger;
}

NodeP n_mat_mul(const NodeP& a, const NodeP& b) {
  const size_t R = a->shape.size();
  if (R < 2 || b->shape.size() != R) invalid("mat_mul: operands must have the same rank, 2 or (for a batch) more");
  if (a->dtype != b->dtype) invalid("mat_mul: operand dtypes differ");
  if (a->shape[R - 1] != b->shape[R - 2]) invalid("mat_mul: inner dimensions differ");  // src/matmul.rs:194
  std::vector<size_t> shape(a->shape.begin(), a->shape.end() - 2);
  for (size_t d = 0; d + 2 < R; d++)
    if (a->shape[d] != b->shape[d]) invalid("mat_mul: batch dimensions differ");
  shape.push_back(a->shape[R - 2]);
  shape.push_back(b->shape[R - 1]);
  NodeP n = make(NodeKind::MatMul, a->dtype, shape);
  n->a = a;
  n->b = b;
  return n;
}

// silu(x) = x / (1 + exp(-x)), src/composite/silu.rs:4-7
NodeP n_silu(const NodeP& x) {
  return n_pair_wise(x, n_scalar(n_unary(n_unary(x, Op::Neg), Op::Exp), Op::AddC, 1.f), Op::Div);
}

// `layer_norm` = RMSNorm computed in f32, src/composite/rms_norm.rs:8-15.
NodeP n_layer_norm(const NodeP& x, const NodeP& weight, float eps, bool as_written) {
  if (x->shape.size() != 2 || weight->shape.size() != 1) invalid("layer_norm: expects a rank-2 tensor and a rank-1 weight");
  if (weight->shape[0] != x->shape[1]) invalid("layer_norm: the weight length must equal the last dimension");
  if (weight->dtype != x->dtype) invalid("layer_norm: dtype mismatch");
  const size_t hidden = x->shape[1];
  NodeP f32_self = n_cast(x, DType::F32);
  NodeP norm_x = n_scalar(n_reduce(n_unary(f32_self, Op::Sqr), ReduceOp::Sum, 1), Op::DivC, float(hidden));
  NodeP rms = n_unary(n_scalar(norm_x, Op::AddC, eps), Op::Sqrt);
  // The reference spells these two broadcasts with Tensor::broadcast, which picks
  // the wrong dimension for the weight when rows == hidden (src/map_layout.rs:69-75);
  // the dimensions are named here.
  // the dimensions are named here.  `as_written` (wkf_device_set_reference_compat) takes Tensor::broadcast for
  // both, as the reference's text does: on a square input the weight is then indexed by row.
  if (as_written) {
    NodeP x_normed = n_pair_wise(f32_self, n_broadcast(rms, x->shape), Op::Div);
    return n_pair_wise(n_cast(x_normed, x->dtype), n_broadcast(weight, x->shape), Op::Mul);
  }
  NodeP x_normed = n_pair_wise(f32_self, n_broadcast_at(rms, 1, hidden), Op::Div);
  return n_pair_wise(n_cast(x_normed, x->dtype), n_broadcast_at(weight, 0, x->shape[0]), Op::Mul);
}

// rotate_half, src/composite/rope.rs:5-10
NodeP n_rotate_half(const NodeP& xs) {
  const size_t last = xs->shape.size() - 1;
  const size_t d = xs->shape[last];
  NodeP x1 = n_narrow(xs, last, 0, d / 2);
  NodeP x2 = n_narrow(xs, last, d / 2, d - d / 2);
  return n_cat({n_unary(x2, Op::Neg), x1}, last);
}

// Tensor<3>::rope, src/composite/rope.rs:12-22.  The reference duplicates the
// half-width tables with cat(.., 2) on rank-2 tensors, which cannot work as
// written; the tables are duplicated along their last dimension here, and
// full-width tables are taken as they are.
NodeP n_rope(const NodeP& x, NodeP cos, NodeP sin) {
  if (x->shape.size() != 3 || cos->shape.size() != 2 || sin->shape.size() != 2) invalid("rope: expects [heads, seq, dim] and rank-2 tables");
  if (cos->shape != sin->shape || cos->dtype != x->dtype || sin->dtype != x->dtype) invalid("rope: table shape / dtype mismatch");
  const size_t seq = x->shape[1], dim = x->shape[2];
  if (cos->shape[1] * 2 == dim) {
    cos = n_cat({cos, cos}, 1);
    sin = n_cat({sin, sin}, 1);
  } else if (cos->shape[1] != dim) {
    invalid("rope: the tables must be dim/2 or dim wide");
  }
  if (cos->shape[0] < seq) invalid("rope: the tables are shorter than the sequence");
  cos = n_narrow(cos, 0, 0, seq);
  sin = n_narrow(sin, 0, 0, seq);
  NodeP rotated = n_rotate_half(x);
  return n_pair_wise(n_pair_wise(x, n_broadcast_at(cos, 0, x->shape[0]), Op::Mul),
                     n_pair_wise(rotated, n_broadcast_at(sin, 0, x->shape[0]), Op::Mul), Op::Add);
}

// Tensor<1>::softmax, src/composite/softmax.rs:4-10
NodeP n_softmax(const NodeP& x) {
  if (x->shape.size() != 1) invalid("softmax: rank 1 only (use softmax_last_dim)");
  NodeP e = n_unary(x, Op::Exp);
  return n_pair_wise(e, n_broadcast_at(n_reduce(e, ReduceOp::Sum, 0), 0, x->shape[0]), Op::Div);
}

NodeP n_softmax_last_dim(const NodeP& x) {
  if (x->shape.empty()) invalid("softmax_last_dim: rank 0");
  const size_t last = x->shape.size() - 1, n = x->shape[last];
  NodeP m = n_broadcast_at(n_reduce(x, ReduceOp::Max, last), last, n);
  NodeP e = n_unary(n_pair_wise(x, m, Op::Sub), Op::Exp);
  NodeP s = n_broadcast_at(n_reduce(e, ReduceOp::Sum, last), last, n);
  return n_pair_wise(e, s, Op::Div);
}

std::vector<std::pair<size_t, size_t>> ranges_of(const wkf_tensor* t, const size_t* starts, const size_t* ends) {
  std::vector<std::pair<size_t, size_t>> r;
  for (size_t d = 0; d < t->node->shape.size(); d++) r.push_back({starts[d], ends[d]});
  return r;
}

DType dtype_of(int d) {
  if (d != WKF_F32 && d != WKF_F16) invalid("unknown dtype");
  return DType(d);
}

}  // namespace

extern "C" {

int wkf_device_set_fusion(wkf_device* dev, int mode) {
  return guarded([&] {
    need(dev, "wkf_device_set_fusion");
    if (mode != WKF_FUSION_REFERENCE && mode != WKF_FUSION_TREE) invalid("unknown fusion mode");
    settings_for(dev);  // creates the entry (and reads the tuning knobs) on first use
    std::lock_guard<std::mutex> lock(g_settings_mu);
    g_settings[dev].fusion = FusionMode(mode);
  });
}

int wkf_device_get_fusion(wkf_device* dev) { return int(settings_for(dev).fusion); }

int wkf_device_set_timing(wkf_device* dev, int enabled) {
  return guarded([&] {
    need(dev, "wkf_device_set_timing");
    settings_for(dev);  // creates the entry (and reads the tuning knobs) on first use
    std::lock_guard<std::mutex> lock(g_settings_mu);
    g_settings[dev].timing = enabled != 0;
  });
}

int wkf_device_set_row_teams(wkf_device* dev, int enabled, uint32_t spin_polls) {
  return guarded([&] {
    need(dev, "wkf_device_set_row_teams");
    settings_for(dev);
    std::lock_guard<std::mutex> lock(g_settings_mu);
    g_settings[dev].row_team = enabled != 0;
    g_settings[dev].row_team_spin = (spin_polls & 0x7fffffffu) == 0 ? Settings().row_team_spin : (spin_polls & 0x7fffffffu);
    g_settings[dev].row_team_test_mute = (spin_polls >> 31) != 0;
  });
}

int wkf_device_set_reference_compat(wkf_device* dev, int enabled) {
  return guarded([&] {
    need(dev, "wkf_device_set_reference_compat");
    settings_for(dev);
    std::lock_guard<std::mutex> lock(g_settings_mu);
    g_settings[dev].reference_compat = enabled != 0;
  });
}

int wkf_device_set_map_table(wkf_device* dev, uint64_t min_elements) {
  return guarded([&] {
    need(dev, "wkf_device_set_map_table");
    settings_for(dev);
    std::lock_guard<std::mutex> lock(g_settings_mu);
    g_settings[dev].map_table_min = size_t(min_elements);
  });
}

int wkf_device_row_team_fallbacks(wkf_device* dev, uint64_t* out) {
  return guarded([&] {
    need(dev, "wkf_device_row_team_fallbacks");
    need(out, "wkf_device_row_team_fallbacks");
    *out = team_fallbacks(dev);
  });
}

int wkf_device_set_exact_math(wkf_device* dev, int exact) {
  return guarded([&] {
    need(dev, "wkf_device_set_exact_math");
    settings_for(dev);
    std::lock_guard<std::mutex> lock(g_settings_mu);
    g_settings[dev].exact_math = exact != 0;
  });
}

int wkf_tensor_new(wkf_device* dev, int dtype, int rank, const size_t* shape, const void* data, wkf_tensor** out) {
  return guarded([&] {
    need(dev, "wkf_tensor_new");
    need(out, "wkf_tensor_new");
    if (rank < 0 || (rank > 0 && !shape)) invalid("wkf_tensor_new: bad rank / shape");
    DType dt = dtype_of(dtype);
    std::vector<size_t> sh(shape, shape + rank);
    NodeP n = make(NodeKind::Tensor, dt, sh);
    n->data.device = dev;
    n->data.layout = Layout::contiguous(sh);
    n->data.dtype = dt;
    size_t bytes = n->data.layout.numel() * dtype_size(dt);
    if (bytes && !data) invalid("wkf_tensor_new: null data");
    wkf_buffer* b = nullptr;
    int rc = wkf_buffer_alloc(dev, std::max<size_t>(4, (bytes + 3) & ~size_t(3)), 0, &b);
    if (rc != WKF_OK) throw Error(rc, wkf_last_error());
    n->data.buffer = BufRef(b);
    rc = wkf_buffer_upload(b, 0, data, bytes);
    if (rc != WKF_OK) throw Error(rc, wkf_last_error());
    *out = wrap(dev, n);
  });
}

int wkf_tensor_clone(const wkf_tensor* t, wkf_tensor** out) {
  return guarded([&] {
    need(t, "wkf_tensor_clone");
    need(out, "wkf_tensor_clone");
    *out = wrap(t->dev, t->node);
  });
}

void wkf_tensor_free(wkf_tensor* t) {
  if (!t) return;
  for (LaunchRecord& r : t->launches)
    if (r.timer) wkf_timer_destroy(r.timer);
  delete t;
}

int wkf_tensor_rank(const wkf_tensor* t) { return t ? int(t->node->shape.size()) : -1; }
int wkf_tensor_shape(const wkf_tensor* t, size_t* out) {
  return guarded([&] {
    need(t, "wkf_tensor_shape");
    for (size_t d = 0; d < t->node->shape.size(); d++) out[d] = t->node->shape[d];
  });
}
int wkf_tensor_dtype(const wkf_tensor* t) { return t ? int(t->node->dtype) : -1; }

int wkf_tensor_scalar_op(const wkf_tensor* t, int op, float c, wkf_tensor** out) {
  return guarded([&] {
    need(t, "wkf_tensor_scalar_op");
    need(out, "wkf_tensor_scalar_op");
    if (!is_const_op(Op(op))) invalid("wkf_tensor_scalar_op: not a tensor-with-literal op");
    *out = wrap(t->dev, n_scalar(t->node, Op(op), c));
  });
}

int wkf_tensor_unary_op(const wkf_tensor* t, int op, wkf_tensor** out) {
  return guarded([&] {
    need(t, "wkf_tensor_unary_op");
    need(out, "wkf_tensor_unary_op");
    if (!is_unary_op(Op(op))) invalid("wkf_tensor_unary_op: not a unary op");
    *out = wrap(t->dev, n_unary(t->node, Op(op)));
  });
}

int wkf_tensor_cast(const wkf_tensor* t, int dtype, wkf_tensor** out) {
  return guarded([&] {
    need(t, "wkf_tensor_cast");
    need(out, "wkf_tensor_cast");
    *out = wrap(t->dev, n_cast(t->node, dtype_of(dtype)));
  });
}

int wkf_tensor_binary_op(const wkf_tensor* a, const wkf_tensor* b, int op, wkf_tensor** out) {
  return guarded([&] {
    need(a, "wkf_tensor_binary_op");
    need(b, "wkf_tensor_binary_op");
    need(out, "wkf_tensor_binary_op");
    if (a->dev != b->dev) invalid("pair-wise op: tensors live on different devices");
    if (!is_binary_op(Op(op))) invalid("wkf_tensor_binary_op: not a pair-wise op");
    *out = wrap(a->dev, n_pair_wise(a->node, b->node, Op(op)));
  });
}

int wkf_tensor_reduce(const wkf_tensor* t, int reduce_op, size_t axis, wkf_tensor** out) {
  return guarded([&] {
    need(t, "wkf_tensor_reduce");
    need(out, "wkf_tensor_reduce");
    if (reduce_op < 0 || reduce_op > 3) invalid("wkf_tensor_reduce: unknown reduction");
    *out = wrap(t->dev, n_reduce(t->node, ReduceOp(reduce_op), axis));
  });
}

int wkf_tensor_reduce_into(const wkf_tensor* t, int reduce_op, size_t axis, wkf_tensor* out) {
  return guarded([&] {
    need(t, "wkf_tensor_reduce_into");
    need(out, "wkf_tensor_reduce_into");
    if (reduce_op < 0 || reduce_op > 3) invalid("wkf_tensor_reduce_into: unknown reduction");
    if (t->dev != out->dev) invalid("wkf_tensor_reduce_into: tensors live on different devices");
    // both tensors hold data already (leaves): nothing below them needs a kernel or a buffer
    if (t->node->kind != NodeKind::Tensor || out->node->kind != NodeKind::Tensor)
      invalid("wkf_tensor_reduce_into: the input and the output must be tensors that hold data (wkf_tensor_new), not lazy expressions");
    if (!t->node->data.layout.is_contiguous() || !out->node->data.layout.is_contiguous())
      invalid("wkf_tensor_reduce_into: the input and the output must be dense");
    NodeP rn = n_reduce(t->node, ReduceOp(reduce_op), axis);  // checks the axis; shape and dtype of the result
    if (out->node->shape != rn->shape || out->node->dtype != rn->dtype)
      invalid("wkf_tensor_reduce_into: the output must have the input's shape without the reduced axis, and its dtype");
    if (wkf_buffer_ptr(out->node->data.buffer.get()) == wkf_buffer_ptr(t->node->data.buffer.get()))
      invalid("wkf_tensor_reduce_into: the output shares the input's buffer");
    Resolver::NoAlloc na;
    na.out = out->node->data;
    Resolver res(t->dev, settings_for(t->dev), nullptr);
    res.set_noalloc(&na);
    TensorData got = res.resolve_root(rn);
    if (got.buffer.get() != na.out.buffer.get())
      throw Error(WKF_ERR_UNSUPPORTED, "wkf_tensor_reduce_into: the result was not written to the output tensor");
  });
}

int wkf_tensor_mat_mul(const wkf_tensor* a, const wkf_tensor* b, wkf_tensor** out) {
  return guarded([&] {
    need(a, "wkf_tensor_mat_mul");
    need(b, "wkf_tensor_mat_mul");
    need(out, "wkf_tensor_mat_mul");
    if (a->dev != b->dev) invalid("mat_mul: tensors live on different devices");
    *out = wrap(a->dev, n_mat_mul(a->node, b->node));
  });
}

int wkf_tensor_slice(const wkf_tensor* t, const size_t* starts, const size_t* ends, wkf_tensor** out) {
  return guarded([&] {
    need(t, "wkf_tensor_slice");
    need(out, "wkf_tensor_slice");
    *out = wrap(t->dev, n_slice(t->node, ranges_of(t, starts, ends)));
  });
}

int wkf_tensor_transpose(const wkf_tensor* t, size_t a0, size_t a1, wkf_tensor** out) {
  return guarded([&] {
    need(t, "wkf_tensor_transpose");
    need(out, "wkf_tensor_transpose");
    *out = wrap(t->dev, n_transpose(t->node, a0, a1));
  });
}

int wkf_tensor_broadcast(const wkf_tensor* t, int out_rank, const size_t* out_shape, wkf_tensor** out) {
  return guarded([&] {
    need(t, "wkf_tensor_broadcast");
    need(out, "wkf_tensor_broadcast");
    if (out_rank < 1) invalid("broadcast: bad rank");
    *out = wrap(t->dev, n_broadcast(t->node, std::vector<size_t>(out_shape, out_shape + out_rank)));
  });
}

int wkf_tensor_narrow(const wkf_tensor* t, size_t axis, size_t start, size_t length, wkf_tensor** out) {
  return guarded([&] {
    need(t, "wkf_tensor_narrow");
    need(out, "wkf_tensor_narrow");
    *out = wrap(t->dev, n_narrow(t->node, axis, start, length));
  });
}

int wkf_tensor_resize(const wkf_tensor* t, const size_t* new_shape, wkf_tensor** out) {
  return guarded([&] {
    need(t, "wkf_tensor_resize");
    need(out, "wkf_tensor_resize");
    *out = wrap(t->dev, n_resize(t->node, std::vector<size_t>(new_shape, new_shape + t->node->shape.size())));
  });
}

int wkf_tensor_reshape(const wkf_tensor* t, int new_rank, const size_t* new_shape, wkf_tensor** out) {
  return guarded([&] {
    need(t, "wkf_tensor_reshape");
    need(out, "wkf_tensor_reshape");
    if (new_rank < 0) invalid("reshape: bad rank");
    *out = wrap(t->dev, n_reshape(t->node, std::vector<size_t>(new_shape, new_shape + new_rank)));
  });
}

int wkf_tensor_unsqueeze(const wkf_tensor* t, size_t axis, wkf_tensor** out) {
  return guarded([&] {
    need(t, "wkf_tensor_unsqueeze");
    need(out, "wkf_tensor_unsqueeze");
    // src/composite/unsqueeze.rs:3-16 asserts axis < rank; appending a trailing axis is allowed too.
    if (axis > t->node->shape.size()) invalid("unsqueeze: axis out of range");
    std::vector<size_t> shape = t->node->shape;
    shape.insert(shape.begin() + axis, 1);
    *out = wrap(t->dev, n_reshape(t->node, shape));
  });
}

int wkf_tensor_slice_assign(const wkf_tensor* t, const size_t* starts, const size_t* ends, const wkf_tensor* value,
                            wkf_tensor** out) {
  return guarded([&] {
    need(t, "wkf_tensor_slice_assign");
    need(value, "wkf_tensor_slice_assign");
    need(out, "wkf_tensor_slice_assign");
    *out = wrap(t->dev, n_slice_assign(t->node, ranges_of(t, starts, ends), value->node));
  });
}

int wkf_tensor_cat(const wkf_tensor* const* tensors, int count, size_t dim, wkf_tensor** out) {
  return guarded([&] {
    need(tensors, "wkf_tensor_cat");
    need(out, "wkf_tensor_cat");
    if (count < 1) invalid("cat: no tensors");
    std::vector<NodeP> v;
    for (int i = 0; i < count; i++) {
      need(tensors[i], "wkf_tensor_cat");
      v.push_back(tensors[i]->node);
    }
    *out = wrap(tensors[0]->dev, n_cat(v, dim));
  });
}

int wkf_tensor_silu(const wkf_tensor* t, wkf_tensor** out) {
  return guarded([&] {
    need(t, "wkf_tensor_silu");
    need(out, "wkf_tensor_silu");
    *out = wrap(t->dev, n_silu(t->node));
  });
}

int wkf_tensor_layer_norm(const wkf_tensor* t, const wkf_tensor* weight, float eps, wkf_tensor** out) {
  return guarded([&] {
    need(t, "wkf_tensor_layer_norm");
    need(weight, "wkf_tensor_layer_norm");
    need(out, "wkf_tensor_layer_norm");
    *out = wrap(t->dev, n_layer_norm(t->node, weight->node, eps, settings_for(t->dev).reference_compat));
  });
}

int wkf_tensor_rope(const wkf_tensor* t, const wkf_tensor* cos, const wkf_tensor* sin, wkf_tensor** out) {
  return guarded([&] {
    need(t, "wkf_tensor_rope");
    need(cos, "wkf_tensor_rope");
    need(sin, "wkf_tensor_rope");
    need(out, "wkf_tensor_rope");
    *out = wrap(t->dev, n_rope(t->node, cos->node, sin->node));
  });
}

int wkf_tensor_softmax(const wkf_tensor* t, wkf_tensor** out) {
  return guarded([&] {
    need(t, "wkf_tensor_softmax");
    need(out, "wkf_tensor_softmax");
    *out = wrap(t->dev, n_softmax(t->node));
  });
}

int wkf_tensor_softmax_last_dim(const wkf_tensor* t, wkf_tensor** out) {
  return guarded([&] {
    need(t, "wkf_tensor_softmax_last_dim");
    need(out, "wkf_tensor_softmax_last_dim");
    *out = wrap(t->dev, n_softmax_last_dim(t->node));
  });
}

int wkf_tensor_arange(wkf_device* dev, int dtype, float start, float end, float step, wkf_tensor** out) {
  return guarded([&] {
    need(dev, "wkf_tensor_arange");
    need(out, "wkf_tensor_arange");
    DType dt = dtype_of(dtype);
    if (step == 0.f || std::isnan(step)) invalid("arange: step must be non-zero");
    // The running value is kept in the tensor dtype, as the reference's `current += step` is.
    auto rnd = [&](float v) { return dt == DType::F16 ? f16_bits_to_f32(f32_to_f16_bits(v)) : v; };
    std::vector<float> vals;
    float cur = rnd(start);
    const float e = rnd(end), st = rnd(step);
    if (st >= 0.f) {
      while (cur < e) {
        vals.push_back(cur);
        float next = rnd(cur + st);
        if (next == cur) invalid("arange: step too small for the dtype");
        cur = next;
      }
    } else {
      while (cur > e) {
        vals.push_back(cur);
        float next = rnd(cur + st);
        if (next == cur) invalid("arange: step too small for the dtype");
        cur = next;
      }
    }
    size_t shape = vals.size();
    int rc;
    if (dt == DType::F32) rc = wkf_tensor_new(dev, dtype, 1, &shape, vals.data(), out);
    else {
      std::vector<uint16_t> h(vals.size());
      for (size_t i = 0; i < vals.size(); i++) h[i] = f32_to_f16_bits(vals[i]);
      rc = wkf_tensor_new(dev, dtype, 1, &shape, h.data(), out);
    }
    if (rc != WKF_OK) throw Error(rc, wkf_last_error());
  });
}

// `st`: the settings to resolve under (null: the device's); `*team` tells whether a team row kernel was launched
static TensorData materialize(wkf_tensor* t, const Settings* st = nullptr, bool* team = nullptr) {
  for (LaunchRecord& r : t->launches)
    if (r.timer) wkf_timer_destroy(r.timer);
  t->launches.clear();
  Resolver res(t->dev, st ? *st : settings_for(t->dev), &t->launches);
  TensorData td = res.resolve_root(t->node);
  if (team) *team = res.team_launched();
  return td;
}

// The settings of `dev` with team row kernels off: what a read-back resolves under, a second time, when a team
// kernel of its first pass gave up waiting.  The graph is still lazy and its leaves are never written in place,
// so the second pass computes the same tensor from the same inputs, one launch per stage or a block per row.
static Settings without_teams(wkf_device* dev) {
  Settings st = settings_for(dev);
  st.row_team = false;
  return st;
}

int wkf_tensor_materialize(wkf_tensor* t) {
  return guarded([&] {
    need(t, "wkf_tensor_materialize");
    materialize(t);
  });
}

static std::vector<TensorData> materialize_many(wkf_tensor** ts, int n, const char* who, const Settings* st = nullptr, bool* team = nullptr) {
  need(ts, who);
  if (n <= 0) invalid(std::string(who) + ": no tensors");
  std::vector<NodeP> roots;
  for (int i = 0; i < n; i++) {
    need(ts[i], who);
    if (ts[i]->dev != ts[0]->dev) invalid(std::string(who) + ": tensors of different devices");
    for (LaunchRecord& r : ts[i]->launches)
      if (r.timer) wkf_timer_destroy(r.timer);
    ts[i]->launches.clear();
    roots.push_back(ts[i]->node);
  }
  // every launch of the joint pass is recorded on the first tensor
  Resolver res(ts[0]->dev, st ? *st : settings_for(ts[0]->dev), &ts[0]->launches);
  std::vector<TensorData> tds = res.resolve_roots(roots);
  if (team) *team = res.team_launched();
  return tds;
}

int wkf_tensor_materialize_many(wkf_tensor** ts, int n) {
  return guarded([&] { materialize_many(ts, n, "wkf_tensor_materialize_many"); });
}

int wkf_tensor_kernel_count(const wkf_tensor* t) { return t ? int(t->launches.size()) : -1; }

static void copy_str(const std::string& s, char* out, size_t cap) {
  if (!out || !cap) return;
  size_t n = std::min(cap - 1, s.size());
  memcpy(out, s.data(), n);
  out[n] = 0;
}

int wkf_tensor_kernel_info(const wkf_tensor* t, int i, uint64_t* elapsed_ns, char* kind, size_t kind_cap,
                           char* signature, size_t signature_cap, char* detail, size_t detail_cap) {
  return guarded([&] {
    need(t, "wkf_tensor_kernel_info");
    if (i < 0 || size_t(i) >= t->launches.size()) invalid("wkf_tensor_kernel_info: index out of range");
    const LaunchRecord& r = t->launches[i];
    if (elapsed_ns) {
      *elapsed_ns = 0;
      if (r.timer) {
        int rc = wkf_timer_elapsed_ns(r.timer, elapsed_ns);
        if (rc != WKF_OK) throw Error(rc, wkf_last_error());
      }
    }
    copy_str(r.kind, kind, kind_cap);
    copy_str(r.signature, signature, signature_cap);
    copy_str(r.detail, detail, detail_cap);
  });
}

int wkf_kernel_source(const char* signature, char* out, size_t cap, size_t* needed) {
  return guarded([&] {
    need(signature, "wkf_kernel_source");
    std::lock_guard<std::mutex> lock(g_source_mu);
    auto it = g_sources.find(signature);
    if (it == g_sources.end()) invalid("wkf_kernel_source: no kernel with this signature was generated by this process");
    if (needed) *needed = it->second.size() + 1;
    copy_str(it->second, out, cap);
  });
}

extern "C++" {
namespace {
// DOT text of the lazy graph below `root` in the reference's format (src/compute_graph/visualize.rs:13-271):
// one node per graph node, labelled `<name> ([shape] dtype) #<id>`, edges from inputs to their consumer, a
// node reached twice emitted once.  Every layout op is called "slice" there (visualize.rs:196).
std::string graph_dot(const NodeP& root) {
  std::ostringstream o;
  o << "digraph \"ComputeGraph\" {\n";
  std::map<const Node*, std::string> ids;
  std::function<std::string(const NodeP&)> visit = [&](const NodeP& n) -> std::string {
    auto it = ids.find(n.get());
    if (it != ids.end()) return it->second;
    std::vector<std::string> inputs;
    if (n->kind != NodeKind::Tensor) {
      if (n->a) inputs.push_back(visit(n->a));
      if (n->b) inputs.push_back(visit(n->b));
    }
    const char* name = "tensor";
    switch (n->kind) {
      case NodeKind::Tensor: name = "tensor"; break;
      case NodeKind::ElementWise:
      case NodeKind::PairWise: name = op_name(n->op); break;
      case NodeKind::Reduce: name = reduce_name(n->rop); break;
      case NodeKind::MatMul: name = "matmul"; break;
      case NodeKind::MapLayout: name = "slice"; break;
      case NodeKind::Resize: name = "resize"; break;
      case NodeKind::SliceAssign: name = "slice_assign"; break;
    }
    std::ostringstream id;
    id << '"' << name << " ([";
    for (size_t d = 0; d < n->shape.size(); d++) id << (d ? ", " : "") << n->shape[d];
    id << "] " << dtype_name(n->dtype) << ") #" << ids.size() << '"';
    ids[n.get()] = id.str();
    o << "  " << id.str() << ";\n";
    for (const std::string& in : inputs) o << "  " << in << " -> " << id.str() << ";\n";
    return id.str();
  };
  visit(root);
  o << "}\n";
  return o.str();
}
}  // namespace
}  // extern "C++"

static std::unique_ptr<wkf_slice> download_slice(const TensorData& td) {
  std::unique_ptr<wkf_slice> s(new wkf_slice());
  s->layout = td.layout;
  s->dtype = td.dtype;
  s->bytes.resize(wkf_buffer_size(td.buffer.get()));
  int rc = wkf_buffer_download(td.buffer.get(), 0, s->bytes.data(), s->bytes.size());
  if (rc != WKF_OK) throw Error(rc, wkf_last_error());
  return s;
}

int wkf_tensor_as_slice_many(wkf_tensor** ts, int n, wkf_slice** out) {
  return guarded([&] {
    need(out, "wkf_tensor_as_slice_many");
    need(ts, "wkf_tensor_as_slice_many");
    if (n > 0 && ts[0]) team_begin(ts[0]->dev);
    std::vector<std::unique_ptr<wkf_slice>> slices;
    bool team = false;
    std::vector<TensorData> tds = materialize_many(ts, n, "wkf_tensor_as_slice_many", nullptr, &team);
    for (const TensorData& td : tds) slices.push_back(download_slice(td));
    if (team && team_gave_up(ts[0]->dev)) {  // every tensor of the call is on that device
      slices.clear();
      tds.clear();
      const Settings st = without_teams(ts[0]->dev);
      tds = materialize_many(ts, n, "wkf_tensor_as_slice_many", &st);
      for (const TensorData& td : tds) slices.push_back(download_slice(td));
    }
    for (int i = 0; i < n; i++) out[i] = slices[size_t(i)].release();
  });
}

int wkf_tensor_graphvis(const wkf_tensor* t, char* out, size_t cap, size_t* needed) {
  return guarded([&] {
    need(t, "wkf_tensor_graphvis");
    const std::string dot = graph_dot(t->node);
    if (needed) *needed = dot.size() + 1;
    copy_str(dot, out, cap);
  });
}

int wkf_tensor_as_slice(wkf_tensor* t, wkf_slice** out) {
  return guarded([&] {
    need(t, "wkf_tensor_as_slice");
    need(out, "wkf_tensor_as_slice");
    team_begin(t->dev);
    bool team = false;
    TensorData td = materialize(t, nullptr, &team);
    std::unique_ptr<wkf_slice> s = download_slice(td);
    if (team && team_gave_up(t->dev)) {
      s.reset();
      td = TensorData();
      const Settings st = without_teams(t->dev);
      td = materialize(t, &st);
      s = download_slice(td);
    }
    *out = s.release();
  });
}

void wkf_slice_free(wkf_slice* s) { delete s; }
extern "C++" {
namespace {
Layout layout_from(int rank, size_t offset, const size_t* shape, const size_t* strides, const char* who) {
  if (rank < 0 || (rank > 0 && (!shape || !strides))) invalid(std::string(who) + ": bad rank / shape / strides");
  Layout l;
  l.offset = offset;
  l.shape.assign(shape, shape + rank);
  l.strides.assign(strides, strides + rank);
  return l;
}
}  // namespace
}  // extern "C++"

int wkf_layout_contiguous(int rank, const size_t* shape, size_t* strides_out) {
  return guarded([&] {
    if (rank < 0 || (rank > 0 && (!shape || !strides_out))) invalid("wkf_layout_contiguous: bad rank / shape");
    const auto st = Layout::contiguous_strides(std::vector<size_t>(shape, shape + rank));
    for (int d = 0; d < rank; d++) strides_out[d] = st[d];
  });
}

int wkf_layout_is_contiguous(int rank, size_t offset, const size_t* shape, const size_t* strides, int* out) {
  return guarded([&] {
    need(out, "wkf_layout_is_contiguous");
    *out = layout_from(rank, offset, shape, strides, "wkf_layout_is_contiguous").is_contiguous() ? 1 : 0;
  });
}

int wkf_layout_slice(int rank, size_t offset, const size_t* shape, const size_t* strides, const size_t* begin,
                     const size_t* end, size_t* offset_out, size_t* shape_out) {
  return guarded([&] {
    const Layout l = layout_from(rank, offset, shape, strides, "wkf_layout_slice");
    if (rank > 0 && (!begin || !end || !shape_out)) invalid("wkf_layout_slice: missing ranges / output");
    need(offset_out, "wkf_layout_slice");
    std::vector<std::pair<size_t, size_t>> ranges;
    for (int d = 0; d < rank; d++) {
      if (end[d] < begin[d] || end[d] > l.shape[d]) invalid("wkf_layout_slice: range outside the shape");
      ranges.emplace_back(begin[d], end[d]);
    }
    const Layout r = l.slice(ranges);
    *offset_out = r.offset;
    for (int d = 0; d < rank; d++) shape_out[d] = r.shape[d];
  });
}

int wkf_slice_rank(const wkf_slice* s) { return s ? int(s->layout.rank()) : -1; }
int wkf_slice_dtype(const wkf_slice* s) { return s ? int(s->dtype) : -1; }

int wkf_slice_layout(const wkf_slice* s, size_t* offset, size_t* shape, size_t* strides) {
  return guarded([&] {
    need(s, "wkf_slice_layout");
    if (offset) *offset = s->layout.offset;
    for (size_t d = 0; d < s->layout.rank(); d++) {
      if (shape) shape[d] = s->layout.shape[d];
      if (strides) strides[d] = s->layout.strides[d];
    }
  });
}

const void* wkf_slice_data(const wkf_slice* s, size_t* bytes) {
  if (!s) return nullptr;
  if (bytes) *bytes = s->bytes.size();
  return s->bytes.data();
}

int wkf_slice_get(const wkf_slice* s, const size_t* index, float* out) {
  return guarded([&] {
    need(s, "wkf_slice_get");
    need(out, "wkf_slice_get");
    size_t at = s->layout.offset;
    for (size_t d = 0; d < s->layout.rank(); d++) {
      if (index[d] >= s->layout.shape[d]) invalid("index out of range");
      at += index[d] * s->layout.strides[d];
    }
    if ((at + 1) * dtype_size(s->dtype) > s->bytes.size()) invalid("index outside the buffer");
    if (s->dtype == DType::F32) memcpy(out, s->bytes.data() + at * 4, 4);
    else {
      uint16_t h;
      memcpy(&h, s->bytes.data() + at * 2, 2);
      *out = f16_bits_to_f32(h);
    }
  });
}

}  // extern "C"

#include "graph.h"

#include <algorithm>
#include <functional>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <set>
#include <unordered_map>
#include <sstream>

namespace wkf {

namespace {

void check(int rc) {
  if (rc != WKF_OK) throw Error(rc, wkf_last_error());
}

uint32_t to_u32(size_t v, const char* what) {
  if (v > 0xffffffffull) throw Error(WKF_ERR_UNSUPPORTED, std::string(what) + " does not fit 32-bit indexing");
  return uint32_t(v);
}

int pow2_ceil(size_t v) {
  int p = 1;
  while (size_t(p) < v) p <<= 1;
  return p;
}

Space coalesce(const std::vector<size_t>& shape, const std::vector<std::vector<size_t>>& strides) {
  Space s;
  s.strides.resize(strides.size());
  for (size_t d = 0; d < shape.size(); d++) {
    if (shape[d] == 1) continue;
    bool merged = false;
    if (!s.shape.empty()) {
      bool ok = true;
      for (size_t k = 0; k < strides.size(); k++) ok &= s.strides[k].back() == shape[d] * strides[k][d];
      if (ok) {
        s.shape.back() *= shape[d];
        for (size_t k = 0; k < strides.size(); k++) s.strides[k].back() = strides[k][d];
        merged = true;
      }
    }
    if (!merged) {
      s.shape.push_back(shape[d]);
      for (size_t k = 0; k < strides.size(); k++) s.strides[k].push_back(strides[k][d]);
    }
  }
  return s;
}

std::string dims(const std::vector<size_t>& v) {
  std::ostringstream o;
  o << '[';
  for (size_t i = 0; i < v.size(); i++) o << (i ? "," : "") << v[i];
  o << ']';
  return o.str();
}

void* element_ptr(const TensorData& td) { return wkf_buffer_ptr(td.buffer.get()); }

}  // namespace

// ---------------------------------------------------------------------------

int Resolver::ExprBuilder::load(const TensorData& td) {
  for (size_t k = 0; k < operands.size(); k++) {
    if (operands[k].buffer.get() == td.buffer.get() && operands[k].dtype == td.dtype && operands[k].layout == td.layout)
      return operand_value[k];
  }
  operands.push_back(td);
  Instr in;
  in.op = Op::Load;
  in.dtype = td.dtype;
  in.operand = int(operands.size()) - 1;
  prog.ins.push_back(in);
  operand_value.push_back(int(prog.ins.size()) - 1);
  return operand_value.back();
}

int Resolver::ExprBuilder::emit(Op op, int a, int b, DType dt, bool has_const, float c) {
  Instr in;
  in.op = op;
  in.a = a;
  in.b = b;
  in.dtype = dt;
  if (has_const) {
    in.cslot = int(prog.consts.size());
    prog.consts.push_back(c);
  }
  prog.ins.push_back(in);
  return int(prog.ins.size()) - 1;
}

int Resolver::build(ExprBuilder& eb, const NodeP& n, int pairwise_budget) {
  auto it = eb.memo.find(n.get());
  if (it != eb.memo.end()) return it->second;
  int v;
  // Keep kernels within a sane register / argument budget: past it, a sub-tree is materialised.
  const bool room = eb.prog.ins.size() < 48 && eb.operands.size() < 7;
  NodeP piece;
  if (eb.split && !eb.inside_piece && (n->kind == NodeKind::SliceAssign || n->kind == NodeKind::MapLayout))
    piece = slice_through(n, eb.split->axis, eb.split->start, eb.split->end);
  if (piece) {
    // cat([A, B]) (possibly under broadcasts) restricted to this piece's range IS A or B
    const bool was = eb.inside_piece;
    eb.inside_piece = true;  // operands below are already piece-shaped
    v = build(eb, piece, pairwise_budget);
    eb.inside_piece = was;
  } else if (n->kind == NodeKind::ElementWise) {
    int a = build(eb, n->a, pairwise_budget);
    v = eb.emit(n->op, a, -1, n->dtype, is_const_op(n->op), n->constant);
  } else if (n->kind == NodeKind::PairWise && pairwise_budget > 0 && room) {
    int a = build(eb, n->a, pairwise_budget - 1);
    int b = build(eb, n->b, pairwise_budget - 1);
    v = eb.emit(n->op, a, b, n->dtype, false, 0.f);
  } else {
    TensorData td = resolve(n);
    if (eb.split && n->kind != NodeKind::Tensor) materialized_[n.get()] = td;  // the other piece's pass reuses it
    if (eb.split && !eb.inside_piece) {
      std::vector<std::pair<size_t, size_t>> r;
      for (size_t d = 0; d < td.layout.rank(); d++)
        r.push_back(d == eb.split->axis ? std::make_pair(eb.split->start, eb.split->end) : std::make_pair(size_t(0), td.layout.shape[d]));
      td.layout = td.layout.slice(r);
    }
    v = eb.load(td);
  }
  eb.memo[n.get()] = v;
  return v;
}

namespace {
// cat([A, B], axis) as Tensor::cat builds it (src/composite/cat.rs:3-41): slice_assign(resize(A, total), [len(A), total) on axis, B).
bool match_cat2(const Node* n, NodeP* a, NodeP* b, size_t* axis) {
  if (n->kind != NodeKind::SliceAssign || n->a->kind != NodeKind::Resize) return false;
  const Node* rz = n->a.get();
  const std::vector<size_t>& total = n->shape;
  const std::vector<size_t>& sa = rz->a->shape;
  const std::vector<size_t>& sb = n->b->shape;
  if (rz->new_shape != total || rz->fill_shape != sa || sa.size() != total.size() || sb.size() != total.size()) return false;
  int ax = -1;
  for (size_t d = 0; d < total.size(); d++) {
    if (sa[d] == total[d] && sb[d] == total[d] && n->ranges[d] == std::make_pair(size_t(0), total[d])) continue;
    if (ax >= 0) return false;
    if (sa[d] + sb[d] != total[d] || n->ranges[d] != std::make_pair(sa[d], total[d])) return false;
    ax = int(d);
  }
  if (ax < 0) return false;
  *a = rz->a;
  *b = n->b;
  *axis = size_t(ax);
  return true;
}

const Node* find_cat2(const Node* n, int depth = 0) {
  if (depth > 64) return nullptr;
  NodeP a, b;
  size_t axis;
  if (match_cat2(n, &a, &b, &axis)) return n;
  if (n->kind == NodeKind::ElementWise) return find_cat2(n->a.get(), depth + 1);
  if (n->kind == NodeKind::PairWise) {
    if (const Node* f = find_cat2(n->a.get(), depth + 1)) return f;
    return find_cat2(n->b.get(), depth + 1);
  }
  return nullptr;
}
}  // namespace

// The node that computes `n` restricted to [start, end) along `axis` without computing the rest of `n`,
// or null when there is no such shortcut: a two-piece cat cut exactly at its seam is one of its pieces,
// and a broadcast of such a cat is the broadcast of the piece.
NodeP Resolver::slice_through(const NodeP& n, size_t axis, size_t start, size_t end) {
  auto key = std::make_tuple(n.get(), axis, start, end);
  auto it = sliced_.find(key);
  if (it != sliced_.end()) return it->second;
  NodeP result;
  NodeP a, b;
  size_t cat_axis = 0;
  if (match_cat2(n.get(), &a, &b, &cat_axis)) {
    if (cat_axis == axis) {
      const size_t mid = a->shape[axis];
      if (start == 0 && end == mid) result = a;
      else if (start == mid && end == n->shape[axis]) result = b;
    }
  } else if (n->kind == NodeKind::MapLayout && n->map_kind == MapKind::Broadcast && axis != n->axis0) {
    NodeP inner = slice_through(n->a, axis > n->axis0 ? axis - 1 : axis, start, end);
    if (inner) {
      auto m = std::make_shared<Node>(*n);
      m->a = inner;
      m->shape[axis] = end - start;
      m->new_shape = m->shape;
      result = m;
    }
  }
  else if (n->kind == NodeKind::MapLayout && n->map_kind == MapKind::Slice && axis < n->ranges.size() &&
           n->ranges[axis] == std::make_pair(size_t(0), n->a->shape[axis])) {
    // a slice that leaves `axis` whole (narrow on another dimension)
    NodeP inner = slice_through(n->a, axis, start, end);
    if (inner) {
      auto m = std::make_shared<Node>(*n);
      m->a = inner;
      m->ranges[axis] = std::make_pair(size_t(0), end - start);
      m->shape[axis] = end - start;
      result = m;
    }
  } else if (n->kind == NodeKind::MapLayout && n->map_kind == MapKind::Transpose) {
    const size_t inner_axis = axis == n->axis0 ? n->axis1 : axis == n->axis1 ? n->axis0 : axis;
    NodeP inner = slice_through(n->a, inner_axis, start, end);
    if (inner) {
      auto m = std::make_shared<Node>(*n);
      m->a = inner;
      m->shape[axis] = end - start;
      result = m;
    }
  }
  sliced_[key] = result;  // keeps the temporary node alive for the whole resolve (maps are keyed by address)
  return result;
}

}  // namespace wkf
// hip_ffi.cpp: the device's static scratch array as a buffer handle (a new reference) and its size
wkf_buffer* wkf_scratch_(wkf_device* dev, size_t* bytes);
// hip_ffi.cpp: `fn` is called when a device is about to be destroyed, to drop state (and buffers) kept for it
void wkf_add_destroy_hook_(void (*fn)(wkf_device*));
// hip_ffi.cpp: wkf_device_destroy has been called and only live buffers keep the device
bool wkf_device_closing_(wkf_device* dev);
namespace wkf {

namespace {
// One 8-byte word per device for team row kernels (the lanes that gave up waiting), allocated at the first such
// launch and kept until the device is destroyed; `pending` = a team kernel ran since the word was last read.
struct TeamWord {
  BufRef buf;
  bool pending = false;
  uint64_t fallbacks = 0;
};
std::mutex g_team_mu;
std::unordered_map<wkf_device*, TeamWord> g_team;
void team_forget(wkf_device* dev) {
  TeamWord w;
  {
    std::lock_guard<std::mutex> lock(g_team_mu);
    auto it = g_team.find(dev);
    if (it == g_team.end()) return;
    w = std::move(it->second);
    g_team.erase(it);
  }
}  // the buffer is released here, outside the lock
void* team_word(wkf_device* dev) {
  static const bool hooked = (wkf_add_destroy_hook_(&team_forget), true);
  (void)hooked;
  std::lock_guard<std::mutex> lock(g_team_mu);
  TeamWord& w = g_team[dev];
  if (!w.buf) {
    wkf_buffer* b = nullptr;
    check(wkf_buffer_alloc(dev, 8, 1, &b));
    w.buf = BufRef(b);
  }
  w.pending = true;
  return wkf_buffer_ptr(w.buf.get());
}
// the word of `dev` when team kernels ran since it was last read (and marks it read), else nothing
BufRef team_take_pending(wkf_device* dev) {
  std::lock_guard<std::mutex> lock(g_team_mu);
  auto it = g_team.find(dev);
  if (it == g_team.end() || !it->second.pending) return BufRef();
  it->second.pending = false;
  return it->second.buf;
}
}  // namespace

void team_begin(wkf_device* dev) {
  BufRef buf = team_take_pending(dev);
  if (!buf || wkf_device_is_planner(dev)) return;
  const unsigned long long zero = 0;  // in stream order: after the launches that may still count, before the ones to come
  check(wkf_buffer_upload(buf.get(), 0, &zero, sizeof zero));
}

bool team_gave_up(wkf_device* dev) {
  BufRef buf = team_take_pending(dev);
  if (!buf || wkf_device_is_planner(dev)) return false;
  unsigned long long n = 0;
  check(wkf_buffer_download(buf.get(), 0, &n, sizeof n));
  if (n == 0) return false;
  const unsigned long long zero = 0;
  check(wkf_buffer_upload(buf.get(), 0, &zero, sizeof zero));
  std::lock_guard<std::mutex> lock(g_team_mu);
  g_team[dev].fallbacks++;
  return true;
}

uint64_t team_fallbacks(wkf_device* dev) {
  std::lock_guard<std::mutex> lock(g_team_mu);
  auto it = g_team.find(dev);
  return it == g_team.end() ? 0 : it->second.fallbacks;
}

namespace {
// Lookup tables of map programs over f16 (try_map_table): per device the 65536 bit patterns as an input tensor and
// the most recently used tables, keyed by program, math policy and constants.
struct MapTables {
  BufRef patterns;
  std::vector<std::pair<std::string, BufRef>> tables;  // most recently used last
};
constexpr size_t kMaxMapTables = 32;  // 128 KiB each
std::mutex g_tables_mu;
std::unordered_map<wkf_device*, MapTables> g_tables;
void tables_forget(wkf_device* dev) {
  MapTables t;
  {
    std::lock_guard<std::mutex> lock(g_tables_mu);
    auto it = g_tables.find(dev);
    if (it == g_tables.end()) return;
    t = std::move(it->second);
    g_tables.erase(it);
  }
}  // the buffers are released here, outside the lock
}  // namespace

BufRef Resolver::map_table_for(const Program& prog) {
  const MathPolicy policy = st_.exact_math ? MathPolicy::Exact : st_.math_f32 ? MathPolicy::Folded : MathPolicy::Stored;
  std::string key = prog.signature() + "|m" + std::to_string(int(policy)) + "|";
  for (float c : prog.consts) {
    char buf[16];
    snprintf(buf, sizeof buf, "%08x,", __builtin_bit_cast(unsigned, c));
    key += buf;
  }
  static const bool hooked = (wkf_add_destroy_hook_(&tables_forget), true);
  (void)hooked;
  BufRef patterns, table;
  {
    std::lock_guard<std::mutex> lock(g_tables_mu);
    MapTables& mt = g_tables[dev_];
    patterns = mt.patterns;
    for (size_t i = 0; i < mt.tables.size(); i++)
      if (mt.tables[i].first == key) {
        table = mt.tables[i].second;
        std::rotate(mt.tables.begin() + long(i), mt.tables.begin() + long(i) + 1, mt.tables.end());
        break;
      }
  }
  if (!table) {
    if (!patterns) {
      wkf_buffer* b = nullptr;
      check(wkf_buffer_alloc(dev_, 65536 * 2, 0, &b));
      patterns = BufRef(b);
      std::vector<uint16_t> all(65536);
      for (size_t i = 0; i < all.size(); i++) all[i] = uint16_t(i);
      check(wkf_buffer_upload(b, 0, all.data(), all.size() * 2));
    }
    TensorData tin;
    tin.device = dev_;
    tin.buffer = patterns;
    tin.layout = Layout::contiguous({65536});
    tin.dtype = DType::F16;
    TensorData tout = alloc({65536}, DType::F16, false);
    launch_map(prog, {tin}, tout, false);  // the ordinary kernel (65536 elements are below any threshold), same policy
    table = tout.buffer;
    std::lock_guard<std::mutex> lock(g_tables_mu);
    MapTables& mt = g_tables[dev_];
    if (!mt.patterns) mt.patterns = patterns;
    if (mt.tables.size() >= kMaxMapTables) mt.tables.erase(mt.tables.begin());
    mt.tables.push_back({key, table});
  }
  return table;
}

BufRef Resolver::cut_table(Program& prog, const std::vector<TensorData>& in, size_t numel, std::string* what) {
  if (st_.fusion != FusionMode::Tree || st_.map_table_min == 0 || numel < std::max<size_t>(st_.map_table_min, 1u << 17) || noalloc_ ||
      wkf_device_closing_(dev_))
    return BufRef();
  const int n = int(prog.ins.size());
  // the one operand a value depends on (-1: none yet, -2: several)
  std::vector<int> leaf(size_t(n), -1);
  auto join = [](int x, int y) { return x == -1 ? y : y == -1 ? x : x == y ? x : -2; };
  for (int i = 0; i < n; i++) {
    const Instr& q = prog.ins[size_t(i)];
    if (q.op == Op::Lookup) return BufRef();
    if (q.op == Op::Load) leaf[size_t(i)] = q.operand;
    else leaf[size_t(i)] = join(q.a >= 0 ? leaf[size_t(q.a)] : -1, q.b >= 0 ? leaf[size_t(q.b)] : -1);
  }
  // the instructions a value is computed from, itself included
  auto cone_of = [&](int f) {
    std::vector<bool> inc(size_t(n), false);
    inc[size_t(f)] = true;
    for (int i = f; i >= 0; i--)
      if (inc[size_t(i)]) {
        if (prog.ins[size_t(i)].a >= 0) inc[size_t(prog.ins[size_t(i)].a)] = true;
        if (prog.ins[size_t(i)].b >= 0) inc[size_t(prog.ins[size_t(i)].b)] = true;
      }
    return inc;
  };
  // the program that computes value f from its one operand (operand 0 there)
  auto sub_program = [&](int f) {
    const std::vector<bool> inc = cone_of(f);
    Program sub;
    std::vector<int> id(size_t(n), -1);
    for (int i = 0; i <= f; i++) {
      if (!inc[size_t(i)]) continue;
      Instr q = prog.ins[size_t(i)];
      if (q.op == Op::Load) q.operand = 0;
      if (q.a >= 0) q.a = id[size_t(q.a)];
      if (q.b >= 0) q.b = id[size_t(q.b)];
      if (q.cslot >= 0) {
        sub.consts.push_back(prog.consts[size_t(q.cslot)]);
        q.cslot = int(sub.consts.size()) - 1;
      }
      id[size_t(i)] = int(sub.ins.size());
      sub.ins.push_back(q);
    }
    sub.result = id[size_t(f)];
    sub.result_feeds = f != prog.result;
    return sub;
  };
  int best = -1, best_cost = 0;
  for (int f = 0; f < n; f++) {
    const Instr& q = prog.ins[size_t(f)];
    if (q.op == Op::Load || leaf[size_t(f)] < 0 || q.dtype != DType::F16 || in[size_t(leaf[size_t(f)])].dtype != DType::F16) continue;
    // (any f16 value of one operand qualifies; the one that takes the most work with it wins, the later of equals: where
    // other operands come in, where the result is stored, or where a cast leaves f16)
    const Program sub = sub_program(f);
    const int cost = program_cost(sub) + (sub.result_feeds && is_unary_op(q.op) ? 7 : 0);
    if (cost >= best_cost) {
      best = f;
      best_cost = cost;
    }
  }
  if (best < 0 || best_cost < 8) return BufRef();   // one interior transcendental is worth the lookup; a few cheap ops are not
  const Program sub = sub_program(best);
  BufRef table = map_table_for(sub);
  // the value becomes a lookup on its operand's load; what only it needed goes away
  const std::vector<bool> inc = cone_of(best);
  int load = -1;
  for (int i = 0; i < best && load < 0; i++)
    if (inc[size_t(i)] && prog.ins[size_t(i)].op == Op::Load) load = i;
  Instr lk;
  lk.op = Op::Lookup;
  lk.a = load;
  lk.dtype = DType::F16;
  prog.ins[size_t(best)] = lk;
  std::vector<bool> live(size_t(n), false);
  live[size_t(prog.result)] = true;
  for (int i = n - 1; i >= 0; i--)
    if (live[size_t(i)]) {
      if (prog.ins[size_t(i)].a >= 0) live[size_t(prog.ins[size_t(i)].a)] = true;
      if (prog.ins[size_t(i)].b >= 0) live[size_t(prog.ins[size_t(i)].b)] = true;
    }
  Program cut;
  cut.consts = prog.consts;   // slots keep their numbers (a slot nothing reads any more costs four bytes of arguments)
  std::vector<int> id(size_t(n), -1);
  for (int i = 0; i < n; i++) {
    if (!live[size_t(i)]) continue;
    Instr q = prog.ins[size_t(i)];
    if (q.a >= 0) q.a = id[size_t(q.a)];
    if (q.b >= 0) q.b = id[size_t(q.b)];
    id[size_t(i)] = int(cut.ins.size());
    cut.ins.push_back(q);
  }
  cut.result = id[size_t(prog.result)];
  cut.result_feeds = prog.result_feeds;
  prog = cut;
  if (what) *what = sub.signature();
  return table;
}

bool Resolver::try_map_table(const Program& prog, const std::vector<TensorData>& in, const TensorData& out, bool in_place) {
  const size_t numel = out.layout.numel();
  if (st_.fusion != FusionMode::Tree || st_.map_table_min == 0 || numel < std::max<size_t>(st_.map_table_min, 1u << 17) || noalloc_) return false;
  if (in.size() != 1 || in[0].dtype != DType::F16 || out.dtype != DType::F16 || prog.result_dtype() != DType::F16) return false;
  // both dense in the same order (any permutation of dimensions, as long as input and output share it), 16-byte aligned
  if (in[0].layout.strides != out.layout.strides || in[0].layout.offset % 8 || out.layout.offset % 8) return false;
  {
    std::vector<std::pair<size_t, size_t>> dims_by_stride;
    for (size_t d = 0; d < out.layout.shape.size(); d++)
      if (out.layout.shape[d] != 1) dims_by_stride.push_back({out.layout.strides[d], out.layout.shape[d]});
    std::sort(dims_by_stride.begin(), dims_by_stride.end());
    size_t expect = 1;
    for (const auto& ds : dims_by_stride) {
      if (ds.first != expect) return false;
      expect *= ds.second;
    }
  }
  if (numel / 8 > 0xffffffffull || program_cost(prog) < 12 || wkf_device_closing_(dev_)) return false;
  if ((in[0].layout.offset + numel) * 2 > wkf_buffer_size(in[0].buffer.get()) + 3 || (out.layout.offset + numel) * 2 > wkf_buffer_size(out.buffer.get()) + 3)
    invalid("map kernel: a layout reaches past the end of its buffer");

  BufRef table = map_table_for(prog);

  const std::string sig = map_table_signature();
  wkf_kernel* k = kernel(sig, [&] { return map_table_source(); });
  struct {
    const void* in;
    void* out;
    const void* table;
    uint32_t nvec, ntail;
  } args = {static_cast<const char*>(element_ptr(in[0])) + in[0].layout.offset * 2, static_cast<char*>(element_ptr(out)) + out.layout.offset * 2,
            wkf_buffer_ptr(table.get()), uint32_t(numel / 8), uint32_t(numel % 8)};
  std::vector<unsigned char> bytes(sizeof(args));
  memcpy(bytes.data(), &args, sizeof(args));
  wkf_props props;
  check(wkf_device_props(dev_, &props));
  LaunchRecord r;
  r.kind = "map";
  r.signature = sig;
  r.in_place = in_place;
  r.grid[0] = to_u32(std::min<size_t>(size_t(std::max(1, props.compute_units)), (numel / 8 + kMapTableBlock - 1) / kMapTableBlock), "grid");
  r.block[0] = kMapTableBlock;
  std::ostringstream d;
  d << "shape=[" << numel << "] table lookup: 65536 values of " << prog.signature() << (in_place ? " in_place" : "");
  r.detail = d.str();
  record(std::move(r), k, bytes);
  return true;
}

TensorData Resolver::alloc(const std::vector<size_t>& shape, DType dt, bool zero, bool result) {
  TensorData td;
  td.device = dev_;
  td.layout = Layout::contiguous(shape);
  td.dtype = dt;
  wkf_buffer* b = nullptr;
  // padded_tensor_size, src/tensor.rs:775-783: a multiple of 4 bytes, at least 4.
  size_t bytes = std::max<size_t>(4, (td.layout.numel() * dtype_size(dt) + 3) & ~size_t(3));
  if (noalloc_) {
    // nothing is allocated: the result is the caller's tensor, a temporary is the device's static scratch array
    if (zero) throw Error(WKF_ERR_UNSUPPORTED, "allocation-free call: the graph needs a zero-filled buffer");
    if (result) {
      // the launch that finishes the reduction writes the caller's tensor: bound to it by role, not by a shape that
      // a temporary might share
      if (noalloc_->out_taken || shape != noalloc_->out.layout.shape || dt != noalloc_->out.dtype)
        throw Error(WKF_ERR_UNSUPPORTED, "allocation-free call: the result does not fit the output tensor");
      noalloc_->out_taken = true;
      return noalloc_->out;
    }
    size_t cap = 0;
    wkf_buffer* sb = wkf_scratch_(dev_, &cap);
    if (!sb) throw Error(WKF_ERR_HIP, "allocation-free call: the device has no scratch array");
    td.buffer = BufRef(sb);
    if (noalloc_->scratch_taken) throw Error(WKF_ERR_UNSUPPORTED, "allocation-free call: the graph needs more than one temporary");
    if (bytes > cap)
      throw Error(WKF_ERR_INVALID_ARG, "allocation-free call: the reduction needs " + std::to_string(bytes) +
                                           " bytes of partial results, the static scratch array holds " + std::to_string(cap));
    noalloc_->scratch_taken = true;
    return td;
  }
  check(wkf_buffer_alloc(dev_, bytes, zero ? 1 : 0, &b));
  td.buffer = BufRef(b);
  return td;
}

extern std::mutex g_source_mu;
extern std::unordered_map<std::string, std::string> g_sources;

// Every kernel gets its own entry-point name, "wkf_<kind>_<hash of the signature>", so that
// profilers list fused kernels separately.
static std::string entry_name(const std::string& sig) {
  uint64_t h = 1469598103934665603ull;
  for (unsigned char c : sig) {
    h ^= c;
    h *= 1099511628211ull;
  }
  char buf[80];
  std::string kind = sig.substr(0, sig.find('|'));
  snprintf(buf, sizeof(buf), "wkf_%s_%08x", kind.c_str(), unsigned(h ^ (h >> 32)));
  return buf;
}

wkf_kernel* Resolver::kernel(const std::string& sig, const std::function<std::string()>& make_body) {
  wkf_kernel* cached = nullptr;
  check(wkf_module_find(dev_, sig.c_str(), &cached));
  if (cached) return cached;  // the hot path: no source text is built
  if (noalloc_)
    throw Error(WKF_ERR_INVALID_ARG, "allocation-free call: kernel '" + sig + "' is not loaded on this device (loading a code object "
                "allocates); run wkf_tensor_reduce + wkf_tensor_materialize once on a tensor of this shape and dtype first");
  const std::string entry = entry_name(sig);
  const std::string src = "#define WKF_ENTRY " + entry + "\n" + make_body();
  {
    std::lock_guard<std::mutex> lock(g_source_mu);
    g_sources.emplace(sig, src);
  }
  if (const char* dir = getenv("WKF_DUMP_SOURCES")) {
    // every kernel's text as it goes to the compiler, "<dir>/<entry>.hip" (signature in the first line)
    if (FILE* f = fopen((std::string(dir) + "/" + entry + ".hip").c_str(), "w")) {
      fprintf(f, "// %s\n%s", sig.c_str(), src.c_str());
      fclose(f);
    }
  }
  wkf_kernel* k = nullptr;
  check(wkf_module_get(dev_, sig.c_str(), src.c_str(), entry.c_str(), &k));
  return k;
}

void Resolver::record(LaunchRecord&& r, wkf_kernel* k, const std::vector<unsigned char>& args) {
  if (st_.timing && !noalloc_) check(wkf_timer_create(dev_, &r.timer));
  int rc = wkf_launch(dev_, k, r.grid, r.block, 0, args.data(), args.size(), r.timer);
  if (rc != WKF_OK) {
    if (r.timer) wkf_timer_destroy(r.timer);
    throw Error(rc, wkf_last_error());
  }
  if (log_) log_->push_back(std::move(r));
  else if (r.timer) wkf_timer_destroy(r.timer);
}

TensorData Resolver::resolve(const NodeP& n) {
  auto it = materialized_.find(n.get());
  if (it != materialized_.end()) return it->second;
  TensorData out = resolve_uncached(n);
  if (shared_.count(n.get()) && n->kind != NodeKind::Tensor) materialized_[n.get()] = out;
  return out;
}

TensorData Resolver::resolve_uncached(const NodeP& n) {
  switch (n->kind) {
    case NodeKind::Tensor:
      return n->data;  // a clone: the graph keeps its own reference, so a leaf is never "owned" (src/compute_graph/resolve.rs:246-248)
    case NodeKind::ElementWise: {
      // collect_element_wise_ops, src/compute_graph/resolve.rs:49-61
      std::vector<const Node*> chain;
      const Node* cur = n.get();
      NodeP base;
      while (cur->kind == NodeKind::ElementWise) {
        chain.push_back(cur);
        base = cur->a;
        cur = cur->a.get();
      }
      if (base->kind == NodeKind::Reduce && !materialized_.count(base.get()))
        return run_reduce(base, chain);  // post-fusion into the reduce, src/compute_graph/resolve.rs:72-74
      return run_map(n);
    }
    case NodeKind::PairWise: return run_map(n);
    case NodeKind::Reduce: return run_reduce(n, {});
    case NodeKind::MatMul: return run_matmul(n);
    case NodeKind::MapLayout: return run_map_layout(n);
    case NodeKind::Resize: return run_resize(n);
    case NodeKind::SliceAssign: return run_slice_assign(n);
  }
  invalid("resolve: unknown node kind");
}

// A node consumed by several nodes of the graph under `root` is computed once per
// resolve and shared.  (The reference recomputes it per use, src/tensor.rs:286-288;
// the values are identical, and because the shared copy holds a reference the
// buffer is never reused in place.)
TensorData Resolver::resolve_root(const NodeP& root) {
  std::map<const Node*, int> uses;
  std::set<const Node*>& shared = shared_;
  shared.clear();
  materialized_.clear();
  sliced_.clear();
  // An element-wise or pair-wise node is inlined into every kernel that uses it,
  // so its second use is also a second use of its inputs: the walk goes through
  // it twice.  Any other node is cut off at its second use.
  std::function<void(const NodeP&)> walk = [&](const NodeP& n) {
    if (!n) return;
    const int seen = ++uses[n.get()];
    if (seen > 2) return;
    if (seen == 2) {
      shared.insert(n.get());
      if (n->kind != NodeKind::ElementWise && n->kind != NodeKind::PairWise) return;
    }
    walk(n->a);
    walk(n->b);
  };
  // Under the reference rules nothing is shared: a node used twice is computed twice.
  if (st_.fusion == FusionMode::Tree) walk(root);
  shared.erase(root.get());
  TensorData out = resolve(root);
  materialized_.clear();
  sliced_.clear();
  return out;
}

// Several roots in one pass: what they share is computed once, and reductions over the last axis of
// the same rows run as one kernel.  (The reference materialises one tensor per call.)
std::vector<TensorData> Resolver::resolve_roots(const std::vector<NodeP>& roots) {
  std::map<const Node*, int> uses;
  shared_.clear();
  materialized_.clear();
  sliced_.clear();
  std::function<void(const NodeP&)> walk = [&](const NodeP& n) {
    if (!n) return;
    const int seen = ++uses[n.get()];
    if (seen > 2) return;
    if (seen == 2) {
      shared_.insert(n.get());
      if (n->kind != NodeKind::ElementWise && n->kind != NodeKind::PairWise) return;
    }
    walk(n->a);
    walk(n->b);
  };
  if (st_.fusion == FusionMode::Tree) {
    for (const NodeP& r : roots) walk(r);
    // group the roots that are [a chain above] a reduce over the last axis by the shape they reduce
    std::map<std::vector<size_t>, std::vector<ReduceRoot>> groups;
    for (const NodeP& r : roots) {
      if (materialized_.count(r.get())) continue;
      ReduceRoot m;
      m.root = r.get();
      const Node* cur = r.get();
      while (cur->kind == NodeKind::ElementWise) {
        m.chain.push_back(cur);
        cur = cur->a.get();
      }
      if (cur->kind != NodeKind::Reduce || cur->a->shape.empty() || cur->axis != cur->a->shape.size() - 1) continue;
      bool inner_shared = shared_.count(cur) > 0;
      for (size_t i = 1; i < m.chain.size(); i++) inner_shared |= shared_.count(m.chain[i]) > 0;
      if (inner_shared) continue;  // something else needs the reduce's own value
      m.reduce = cur;
      bool dup = false;
      for (const ReduceRoot& o : groups[cur->a->shape]) dup |= o.root == m.root;
      if (!dup) groups[cur->a->shape].push_back(m);
    }
    for (auto& g : groups) {
      std::vector<TensorData> outs;
      if (try_parallel_reduces(g.second, &outs))
        for (size_t i = 0; i < g.second.size(); i++) materialized_[g.second[i].root] = outs[i];
    }
  }
  std::vector<TensorData> out;
  for (const NodeP& r : roots) {
    TensorData td = resolve(r);
    materialized_[r.get()] = td;  // a root listed twice, or used below another root, is computed once
    out.push_back(td);
  }
  materialized_.clear();
  sliced_.clear();
  return out;
}

// ---- row kernels -----------------------------------------------------------------------------

namespace {
constexpr int kScalarBase = 1000;  // placeholder operand index of "scalar of stage s" until the operand count is known

// A broadcast along the last axis of [an element-wise chain over] a reduce over the last axis of a
// tensor of the same rows: returns that reduce node (and the chain, outermost first), else null.
const Node* row_scalar_source(const Node* n, const std::vector<size_t>& shape, std::vector<const Node*>* chain) {
  if (n->kind != NodeKind::MapLayout || n->map_kind != MapKind::Broadcast) return nullptr;
  if (shape.empty() || n->axis0 != shape.size() - 1 || n->shape != shape) return nullptr;
  const Node* cur = n->a.get();
  while (cur->kind == NodeKind::ElementWise) {
    if (chain) chain->push_back(cur);
    cur = cur->a.get();
  }
  if (cur->kind != NodeKind::Reduce || cur->axis != shape.size() - 1 || cur->a->shape != shape) return nullptr;
  return cur;
}

bool has_row_pattern(const Node* n, const std::vector<size_t>& shape, int depth = 0) {
  if (depth > 64) return false;
  if (row_scalar_source(n, shape, nullptr)) return true;
  if (n->kind == NodeKind::ElementWise) return has_row_pattern(n->a.get(), shape, depth + 1);
  if (n->kind == NodeKind::PairWise) return has_row_pattern(n->a.get(), shape, depth + 1) || has_row_pattern(n->b.get(), shape, depth + 1);
  return false;
}
}  // namespace

struct Resolver::RowBuild {
  std::vector<size_t> shape;
  std::vector<TensorData> operands;
  std::vector<RowStage> stages;
  std::map<const Node*, int> stage_of;  // reduce node -> stage
  bool ok = true;
};

int Resolver::row_build(RowBuild& rb, Program& prog, std::map<const Node*, int>& memo, std::map<int, int>& loads, const NodeP& n) {
  auto it = memo.find(n.get());
  if (it != memo.end()) return it->second;
  auto load = [&](int operand, DType dt) {
    auto l = loads.find(operand);
    if (l != loads.end()) return l->second;
    Instr in;
    in.op = Op::Load;
    in.dtype = dt;
    in.operand = operand;
    prog.ins.push_back(in);
    return loads[operand] = int(prog.ins.size()) - 1;
  };
  int v = -1;
  std::vector<const Node*> chain;
  if (const Node* red = row_scalar_source(n.get(), rb.shape, &chain)) {
    int stage;
    auto st = rb.stage_of.find(red);
    if (st != rb.stage_of.end()) stage = st->second;
    else {
      // the stage's own expression first (it may create earlier stages), then the stage
      RowStage rs;
      rs.rop = red->rop;
      std::map<const Node*, int> pmemo;
      std::map<int, int> ploads;
      rs.pre.result = row_build(rb, rs.pre, pmemo, ploads, red->a);
      if (!rb.ok) return 0;
      Instr ld;
      ld.op = Op::Load;
      ld.dtype = rs.pre.result_dtype();
      ld.operand = 0;
      rs.post.ins.push_back(ld);
      rs.post.result = 0;
      rb.stages.push_back(rs);
      stage = int(rb.stages.size()) - 1;
      rb.stage_of[red] = stage;
    }
    // the chain between the reduce and the broadcast is applied per element here (one scalar op per
    // lane and row element costs nothing next to the loads and keeps one code path)
    v = load(kScalarBase + stage, rb.stages[stage].post.result_dtype());
    for (size_t i = chain.size(); i-- > 0;) {
      const Node* c = chain[i];
      if (c->op == Op::Sin || c->op == Op::Cos) rb.ok = false;
      Instr in;
      in.op = c->op;
      in.a = v;
      in.dtype = c->dtype;
      if (is_const_op(c->op)) {
        in.cslot = int(prog.consts.size());
        prog.consts.push_back(c->constant);
      }
      prog.ins.push_back(in);
      v = int(prog.ins.size()) - 1;
    }
  } else if (n->kind == NodeKind::ElementWise) {
    if (n->op == Op::Sin || n->op == Op::Cos) rb.ok = false;  // would need the far-argument redo path
    int a = row_build(rb, prog, memo, loads, n->a);
    Instr in;
    in.op = n->op;
    in.a = a;
    in.dtype = n->dtype;
    if (is_const_op(n->op)) {
      in.cslot = int(prog.consts.size());
      prog.consts.push_back(n->constant);
    }
    prog.ins.push_back(in);
    v = int(prog.ins.size()) - 1;
  } else if (n->kind == NodeKind::PairWise && prog.ins.size() < 48) {
    int a = row_build(rb, prog, memo, loads, n->a);
    int b = row_build(rb, prog, memo, loads, n->b);
    Instr in;
    in.op = n->op;
    in.a = a;
    in.b = b;
    in.dtype = n->dtype;
    prog.ins.push_back(in);
    v = int(prog.ins.size()) - 1;
  } else {
    TensorData td = resolve(n);
    if (td.layout.shape != rb.shape) {
      rb.ok = false;
      return 0;
    }
    int k = -1;
    for (size_t i = 0; i < rb.operands.size(); i++)
      if (rb.operands[i].buffer.get() == td.buffer.get() && rb.operands[i].dtype == td.dtype && rb.operands[i].layout == td.layout) k = int(i);
    if (k < 0) {
      rb.operands.push_back(td);
      k = int(rb.operands.size()) - 1;
    }
    v = load(k, td.dtype);
  }
  memo[n.get()] = v;
  return v;
}

bool Resolver::try_row_kernel(const NodeP& root, TensorData* result) {
  if (st_.fusion != FusionMode::Tree || root->shape.empty()) return false;
  if (!has_row_pattern(root.get(), root->shape)) return false;
  RowBuild rb;
  rb.shape = root->shape;
  Program final;
  std::map<const Node*, int> memo;
  std::map<int, int> loads;
  final.result = row_build(rb, final, memo, loads, root);
  if (!rb.ok || rb.stages.empty() || rb.operands.empty() || rb.operands.size() > 4 || rb.stages.size() > 4) return false;
  std::vector<TensorData> outs;
  if (!launch_row(rb, &final, &outs)) return false;
  *result = outs[0];
  return true;
}

// Several reductions over the last axis of the same rows (row max and row sum(exp(x - 1)) of one matrix)
// in ONE pass: a row kernel whose stages are the reductions and which stores one scalar per stage and row
// instead of a mapped row.  The reference lists this as to-do (README.md:20) and runs one kernel each.
bool Resolver::try_parallel_reduces(const std::vector<ReduceRoot>& members, std::vector<TensorData>* outs) {
  if (st_.fusion != FusionMode::Tree || members.size() < 2 || members.size() > 4) return false;
  RowBuild rb;
  rb.shape = members[0].reduce->a->shape;
  if (rb.shape.empty()) return false;
  for (const ReduceRoot& m : members) {
    if (m.reduce->a->shape != rb.shape || m.reduce->axis != rb.shape.size() - 1) return false;
    RowStage rs;
    rs.rop = m.reduce->rop;
    std::map<const Node*, int> pmemo;
    std::map<int, int> ploads;
    rs.pre.result = row_build(rb, rs.pre, pmemo, ploads, m.reduce->a);
    if (!rb.ok) return false;
    for (const Instr& in : rs.pre.ins)
      if (in.op == Op::Load && in.operand >= kScalarBase) return false;  // depends on another reduction of the rows
    Instr ld;
    ld.op = Op::Load;
    ld.dtype = rs.pre.result_dtype();
    ld.operand = 0;
    rs.post.ins.push_back(ld);
    int cur = 0;
    for (size_t i = m.chain.size(); i-- > 0;) {  // the chain above the reduce, innermost first
      const Node* c = m.chain[i];
      if (c->op == Op::Sin || c->op == Op::Cos) return false;  // would need the far-argument redo path
      Instr in;
      in.op = c->op;
      in.a = cur;
      in.dtype = c->dtype;
      if (is_const_op(c->op)) {
        in.cslot = int(rs.post.consts.size());
        rs.post.consts.push_back(c->constant);
      }
      rs.post.ins.push_back(in);
      cur = int(rs.post.ins.size()) - 1;
    }
    rs.post.result = cur;
    rb.stages.push_back(rs);
  }
  if (rb.stages.size() != members.size() || rb.operands.empty() || rb.operands.size() > 4) return false;
  return launch_row(rb, nullptr, outs);
}

// Plans and launches a row kernel: with `final`, one output of the rows' shape (softmax, RMSNorm);
// without, one output per stage holding that stage's scalar of every row (parallel reductions).
bool Resolver::launch_row(RowBuild& rb, const Program* final_in, std::vector<TensorData>* outs) {
  const bool scalars = final_in == nullptr;
  Program final;
  if (final_in) final = *final_in;
  const size_t R = rb.shape.size(), axis = R - 1, n = rb.shape[axis];
  const size_t K = rb.operands.size(), S = rb.stages.size();
  const size_t NOUT = scalars ? S : 1;

  RowSpec spec;
  size_t max_elem = scalars ? 2 : dtype_size(final.result_dtype());
  for (const TensorData& td : rb.operands) max_elem = std::max(max_elem, dtype_size(td.dtype));
  const int Vmax = int(16 / max_elem);
  if (n == 0) return false;
  std::vector<size_t> out_shape(rb.shape.begin(), rb.shape.end() - 1);
  std::vector<std::vector<size_t>> ostr;
  for (const TensorData& td : rb.operands) ostr.push_back(std::vector<size_t>(td.layout.strides.begin(), td.layout.strides.end() - 1));
  // outputs are fresh contiguous tensors: rows of the full shape, or one scalar per row
  std::vector<size_t> full_strides = Layout::contiguous_strides(rb.shape);
  for (size_t q = 0; q < NOUT; q++)
    ostr.push_back(scalars ? Layout::contiguous_strides(out_shape) : std::vector<size_t>(full_strides.begin(), full_strides.end() - 1));
  Space sp = coalesce(out_shape, ostr);
  const size_t Ro = sp.shape.size();
  if (Ro > 3) return false;
  for (size_t k = 0; k < K; k++) {
    const TensorData& td = rb.operands[k];
    if (td.layout.strides[axis] > 1) return false;
    if (td.layout.extent() > 0xffffffffull) return false;
    spec.in.push_back({td.dtype, int(td.layout.strides[axis])});
  }
  // The widest vector (16 bytes down to one element) that divides the row and on which every row of every
  // operand, and of the output when it has full rows, starts aligned
  auto aligned = [&](int v) {
    if (n % size_t(v)) return false;
    for (size_t k = 0; k < K + (scalars ? 0 : NOUT); k++) {
      if (k < K && rb.operands[k].layout.strides[axis] != 1) continue;
      if (k < K && rb.operands[k].layout.offset % size_t(v)) return false;
      for (size_t d = 0; d < Ro; d++)
        if (sp.strides[k][d] % size_t(v)) return false;
    }
    return true;
  };
  int V = Vmax;
  while (V > 1 && !aligned(V)) V /= 2;
  const size_t nvec = n / V;
  // a lane holds at most 16 vectors of each operand; narrower vectors may be more (the same registers), for
  // rows that no number of lanes covers otherwise
  const size_t max_nv = size_t(16 * (Vmax / V));
  // Lanes per row, measured on MI355X: two 16-byte vectors per lane up to 256 lanes (softmax over 2048
  // floats: 169 us with 256 lanes, 173 with 64; RMSNorm over 4096: 15.9 us with 256, 17.2 with 128), more
  // lanes only when a lane would otherwise hold more than 16 vectors.  An f16 row of up to 256 vectors stays in ONE wave
  // (four vectors per lane, no fold through the LDS and no barrier: f16 softmax over 2048: 87.1 us with 128 lanes, 83.8
  // with 64; f32 rows of 1024 lose 2 % that way and keep 128 lanes).
  const int T_wide = [&] {
    int t = std::min(256, pow2_ceil((nvec + 1) / 2));
    if (nvec <= 256 && Vmax == 8) t = std::min(t, 64);
    // stored reductions only (no result rows): four vectors per lane up to 512 lanes (row max + row sum(exp(x - 1)) of
    // f32 [8192,8192] in one pass: 42.5 us with 256 lanes, 41.1 with 512, 45.0 with 1024)
    while (scalars && t < 512 && nvec > size_t(t) * 4) t *= 2;
    while (t < 1024 && nvec > size_t(t) * 16) t *= 2;
    return t;
  }();
  int T = T_wide;
  while (T > 1 && nvec % size_t(T)) T /= 2;  // first choice: the row splits evenly over the lanes
  if (st_.row_threads > 0 && size_t(st_.row_threads) <= nvec) T = st_.row_threads;
  bool ragged = false;
  if (nvec % T || nvec / T > 16 || (nvec / T) * V * K > 128) {
    // otherwise the widest layout, with the lanes past the end of the row masked in their last vector
    T = T_wide;
    ragged = true;
  }
  size_t NV = (nvec + T - 1) / T;
  size_t nrows = 1;
  for (size_t d : out_shape) nrows *= d;
  if (nrows > 0xffffffffull) return false;
  bool streamed = false, split = false, team = false;
  size_t parts = 1, chunk = 0, teams = 0;
  if (NV > max_nv || NV * V * K > 128) {
    // The row does not fit the registers of a block.  With enough rows to occupy the chip, one block per row
    // streams its row once per stage and once more for the result, in ONE launch; the passes after the first
    // find the row in the caches when it fits them.  With only a few rows a block per row would leave most
    // compute units idle: every row is then cut into parts with a block each and every stage becomes a launch
    // of its own, which leaves its parts' values to the next (softmax: two launches).  Reductions that are
    // stored (no result rows) are folded across the whole grid by the caller instead.
    if (nvec < 1024) return false;
    // First choice: the row in the registers of a team of blocks (one launch, one read).  Eight 16-byte vectors
    // per lane over all operands, 256 lanes per block, at most 256 parts.  The launch bounds of the kernel
    // guarantee four resident blocks per compute unit, and the grid never asks for more than that, because
    // the blocks of a team wait for each other.
    size_t kfull = 0;
    for (size_t k = 0; k < K; k++) kfull += rb.operands[k].layout.strides[axis] == 1 ? 1 : 0;
    const size_t team_nv = std::max<size_t>(1, 8 / std::max<size_t>(1, kfull));
    const size_t team_lanes = 256;
    const size_t team_parts = (nvec + team_lanes * team_nv - 1) / (team_lanes * team_nv);
    wkf_props props;
    check(wkf_device_props(dev_, &props));
    const size_t resident = size_t(std::max(1, props.compute_units)) * 4;
    // (a device that is only kept by its live buffers gets no new per-device state: the word team kernels count in)
    if (st_.row_team && !scalars && !noalloc_ && kfull >= 1 && team_parts >= 2 && team_parts <= 256 && team_parts <= resident &&
        !wkf_device_closing_(dev_)) {
      team = true;
      ragged = false;
      T = int(team_lanes);
      NV = team_nv;
      parts = team_parts;
      teams = std::min(nrows, resident / team_parts);
      teams = (nrows + (nrows + teams - 1) / teams - 1) / ((nrows + teams - 1) / teams);  // as many rounds, evenly filled
    } else {
    streamed = true;
    ragged = false;
    NV = std::max<size_t>(1, std::min<size_t>(4, 8 / std::max<size_t>(1, K)));  // vectors in flight per lane and operand
    if (st_.row_stream_vectors > 0) NV = size_t(st_.row_stream_vectors);
    if (nrows >= st_.row_stream_min_rows) {
      T = 1024;
    } else {
      if (scalars || !st_.row_split) return false;
      split = true;
      T = 256;
      // about eight blocks per compute unit, every part a whole number of steps of the block, at most one part per lane
      const size_t step = size_t(T) * NV;
      const size_t want = std::min<size_t>(size_t(T), std::max<size_t>(1, 2048 / nrows));
      chunk = ((nvec + want - 1) / want + step - 1) / step * step;
      parts = (nvec + chunk - 1) / chunk;
    }
    }
  }

  // operand numbering: full operands 0..K-1, then the scalars
  auto renumber = [&](Program& p) {
    for (Instr& in : p.ins)
      if (in.op == Op::Load && in.operand >= kScalarBase) in.operand = int(K) + (in.operand - kScalarBase);
  };
  for (RowStage& st : rb.stages) renumber(st.pre);
  renumber(final);
  spec.outer_rank = int(Ro);
  spec.vec = V;
  spec.threads_per_row = T;
  spec.block = std::max(256, T);
  spec.vectors_per_lane = int(NV);
  spec.ragged = ragged;
  spec.streamed = streamed;
  spec.team = team;
  spec.team_mute = team && st_.row_team_test_mute;
  spec.stages = rb.stages;
  if ((streamed || team) && rb.stages.size() >= 2) {
    // softmax's pair of stages, max(x) then sum(exp(x - max)), is folded in one pass over a streamed row
    const RowStage& s0 = rb.stages[0];
    const RowStage& s1 = rb.stages[1];
    auto is_load = [](const Instr& in, int operand) { return in.op == Op::Load && in.operand == operand; };
    const bool max_of_x = s0.rop == ReduceOp::Max && s0.pre.ins.size() == 1 && is_load(s0.pre.ins[0], 0) && s0.post.ins.size() == 1;
    bool sum_exp = s1.rop == ReduceOp::Sum && s1.pre.ins.size() == 4 && s1.post.ins.size() == 1 && s1.pre.result == 3 &&
                   s1.pre.ins[2].op == Op::Sub && s1.pre.ins[3].op == Op::Exp && s1.pre.ins[3].a == 2;
    if (sum_exp) {
      const Instr& x = s1.pre.ins[s1.pre.ins[2].a];
      const Instr& m = s1.pre.ins[s1.pre.ins[2].b];
      sum_exp = is_load(x, 0) && is_load(m, int(K));
    }
    spec.online_max_sum = max_of_x && sum_exp;
  }
  spec.final = final;
  spec.store_scalars = scalars;
  spec.out_dtype = scalars ? DType::F32 : final.result_dtype();
  spec.exact_math = st_.exact_math;

  outs->clear();
  for (size_t q = 0; q < NOUT; q++)
    outs->push_back(scalars ? alloc(out_shape, rb.stages[q].post.result_dtype(), false) : alloc(rb.shape, final.result_dtype(), false));
  if (nrows == 0) return true;

  RowArgs args;
  args.nrows = uint32_t(nrows);
  args.nvec = uint32_t(nvec);
  for (size_t d = 0; d < Ro; d++) args.oshape.push_back(to_u32(sp.shape[d], "shape"));
  for (size_t k = 0; k < K + NOUT; k++) {
    const TensorData& td = k < K ? rb.operands[k] : (*outs)[k - K];
    args.ptrs.push_back(element_ptr(td));
    args.offsets.push_back(to_u32(td.layout.offset, "offset"));
    std::vector<uint32_t> st;
    for (size_t d = 0; d < Ro; d++) st.push_back(to_u32(sp.strides[k][d], "stride"));
    args.ostrides.push_back(st);
  }
  for (const RowStage& st : rb.stages) {
    args.consts.insert(args.consts.end(), st.pre.consts.begin(), st.pre.consts.end());
    args.consts.insert(args.consts.end(), st.post.consts.begin(), st.post.consts.end());
  }
  args.consts.insert(args.consts.end(), final.consts.begin(), final.consts.end());

  std::ostringstream d;
  d << "rows=" << nrows << " n=" << n << " vec=" << V << " threads_per_row=" << T << " vectors_per_lane=" << NV << " stages="
    << rb.stages.size() << " operands=" << K + NOUT;
  if (scalars) d << " reductions=" << S;
  if (ragged) d << " ragged";
  if (streamed) d << (spec.online_max_sum ? " streamed (max and sum in one pass)" : " streamed");
  const size_t rpb = size_t(spec.block / T);
  if (team) {
    // zero-filled slots [stages][rows][parts] of 64 bits; the device's give-up count as the last pointer
    TensorData slots = alloc({S * nrows * parts * 2}, DType::F32, true);
    args.ptrs.push_back(element_ptr(slots));
    args.ptrs.push_back(team_word(dev_));
    args.parts = to_u32(parts, "parts");
    args.spin = st_.row_team_spin;
    team_launched_ = true;
    std::string sig = row_signature(spec);
    wkf_kernel* k = kernel(sig, [&] { return row_source(spec); });
    LaunchRecord r;
    r.kind = "row";
    r.signature = sig;
    r.grid[0] = to_u32(teams * parts, "grid");
    r.block[0] = 256;
    d << (spec.online_max_sum ? ", max and sum in one exchange" : "") << ", rows in the registers of teams of " << parts << " blocks, " << teams << " teams";
    r.detail = d.str();
    record(std::move(r), k, row_pack_args(spec, args));
    return true;
  }
  if (!split) {
    std::string sig = row_signature(spec);
    wkf_kernel* k = kernel(sig, [&] { return row_source(spec); });
    LaunchRecord r;
    r.kind = "row";
    r.signature = sig;
    r.grid[0] = to_u32((nrows + rpb - 1) / rpb, "grid");
    r.block[0] = uint32_t(spec.block);
    r.detail = d.str();
    record(std::move(r), k, row_pack_args(spec, args));
    return true;
  }
  // split rows: one launch per stage (an online pair counts as one), then the launch that writes the rows
  TensorData part_values = alloc({S, nrows, parts}, DType::F32, false);
  args.ptrs.push_back(element_ptr(part_values));
  args.parts = to_u32(parts, "parts");
  args.chunk = to_u32(chunk, "chunk");
  spec.split = true;
  std::vector<int> phases;
  for (size_t p = 0; p <= S; p++)
    if (!(spec.online_max_sum && p == 1)) phases.push_back(int(p));
  for (size_t i = 0; i < phases.size(); i++) {
    spec.split_phase = phases[i];
    std::string sig = row_signature(spec);
    wkf_kernel* k = kernel(sig, [&] { return row_source(spec); });
    LaunchRecord r;
    r.kind = "row";
    r.signature = sig;
    r.grid[0] = to_u32(nrows * parts, "grid");
    r.block[0] = uint32_t(spec.block);
    std::ostringstream dd;
    dd << d.str() << ", rows split in " << parts << " parts of " << chunk << " vectors: launch " << i + 1 << " of " << phases.size();
    r.detail = dd.str();
    record(std::move(r), k, row_pack_args(spec, args));
  }
  return true;
}

TensorData Resolver::run_map(const NodeP& root) {
  {
    TensorData fused;
    if (try_row_kernel(root, &fused)) return fused;
  }
  // A consumer of cat([A, B]) runs once per piece and writes straight into its part of the result,
  // instead of copying the pieces together first and reading the copy back (rope's rotate_half).
  if (st_.fusion == FusionMode::Tree && root->kind != NodeKind::SliceAssign) {
    if (const Node* cat = find_cat2(root.get())) {
      NodeP pa, pb;
      size_t axis = 0;
      match_cat2(cat, &pa, &pb, &axis);
      const size_t mid = pa->shape[axis], total = cat->shape[axis];
      TensorData out;
      CatPiece piece[2];
      ExprBuilder eb[2];
      TensorData view[2];
      for (int part = 0; part < 2; part++) {
        piece[part].axis = axis;
        piece[part].start = part == 0 ? 0 : mid;
        piece[part].end = part == 0 ? mid : total;
        eb[part].split = &piece[part];
        eb[part].prog.result = build(eb[part], root, pairwise_budget_for_map());
        if (part == 0) out = alloc(root->shape, eb[part].prog.result_dtype(), false);
        std::vector<std::pair<size_t, size_t>> r;
        for (size_t d = 0; d < root->shape.size(); d++)
          r.push_back(d == axis ? std::make_pair(piece[part].start, piece[part].end) : std::make_pair(size_t(0), root->shape[d]));
        view[part] = out;
        view[part].layout = out.layout.slice(r);
      }
      if (mid == total - mid && mid > 0) {
        // Pieces of one shape (rope's two halves): ONE kernel with two stores; the operands the pieces
        // share (x1, x2, cos, sin) are loaded once.
        std::vector<TensorData> operands = eb[0].operands;
        Program second = eb[1].prog;
        for (Instr& in : second.ins) {
          if (in.op != Op::Load) continue;
          const TensorData& td = eb[1].operands[size_t(in.operand)];
          size_t k = 0;
          for (; k < operands.size(); k++)
            if (operands[k].buffer.get() == td.buffer.get() && operands[k].dtype == td.dtype && operands[k].layout == td.layout) break;
          if (k == operands.size()) operands.push_back(td);
          in.operand = int(k);
        }
        if (operands.size() <= 8) {
          launch_map(eb[0].prog, operands, view[0], false, {second}, {view[1]});
          return out;
        }
      }
      for (int part = 0; part < 2; part++)
        if (piece[part].end > piece[part].start) launch_map(eb[part].prog, eb[part].operands, view[part], false);
      return out;
    }
  }
  ExprBuilder eb;
  int v = build(eb, root, pairwise_budget_for_map());
  eb.prog.result = v;
  const DType out_dt = eb.prog.result_dtype();
  // In-place rule: src/element_wise.rs:98 and src/pair_wise.rs:95-107 -- the first
  // operand of the output dtype that nobody else references and that has no
  // stride-0 overlap is overwritten; otherwise a fresh contiguous tensor.
  int reuse = -1;
  for (size_t k = 0; k < eb.operands.size(); k++) {
    const TensorData& td = eb.operands[k];
    if (td.dtype == out_dt && td.owned() && !td.layout.allocation_overlaps()) {
      reuse = int(k);
      break;
    }
  }
  TensorData out = reuse >= 0 ? eb.operands[reuse] : alloc(root->shape, out_dt, false);
  launch_map(eb.prog, eb.operands, out, reuse >= 0);
  return out;
}

void Resolver::launch_map(const Program& prog, const std::vector<TensorData>& in, const TensorData& out, bool in_place,
                          const std::vector<Program>& more_prog, const std::vector<TensorData>& more_out) {
  const std::vector<size_t>& shape = out.layout.shape;
  for (const TensorData& td : more_out)
    if (td.layout.shape != shape) invalid("map kernel: outputs of different shapes");
  for (const TensorData& td : in)
    if (td.layout.shape != shape)
      invalid("operand shapes differ: " + dims(td.layout.shape) + " vs " + dims(shape));  // src/pair_wise.rs:92
  size_t numel = out.layout.numel();
  if (numel == 0) return;
  if (more_out.empty() && try_map_table(prog, in, out, in_place)) return;

  // The order in which a map visits its elements is free: walk the dimensions in the order of the
  // OUTPUT's strides (largest first), so that a transposed output written in place is still one
  // linear sweep and stores are always as coalesced as the layout allows.
  std::vector<size_t> order;
  {
    // dimensions of size 1 stay where they are (their strides mean nothing); the others are sorted
    std::vector<size_t> real;
    for (size_t d = 0; d < shape.size(); d++)
      if (shape[d] != 1) real.push_back(d);
    std::stable_sort(real.begin(), real.end(), [&](size_t x, size_t y) { return out.layout.strides[x] > out.layout.strides[y]; });
    size_t next = 0;
    for (size_t d = 0; d < shape.size(); d++) order.push_back(shape[d] == 1 ? d : real[next++]);
  }
  std::vector<size_t> pshape;
  for (size_t d : order) pshape.push_back(shape[d]);
  std::vector<std::vector<size_t>> strides;
  const size_t N = in.size() + 1 + more_out.size();
  auto td_of = [&](size_t k) -> const TensorData& { return k < in.size() ? in[k] : k == in.size() ? out : more_out[k - in.size() - 1]; };
  for (size_t k = 0; k < N; k++) {
    const std::vector<size_t>& st = td_of(k).layout.strides;
    std::vector<size_t> ps;
    for (size_t d : order) ps.push_back(st[d]);
    strides.push_back(ps);
  }
  Space sp = coalesce(pshape, strides);
  if (sp.shape.empty()) {
    sp.shape.push_back(1);
    for (auto& s : sp.strides) s.push_back(1);
  }
  const size_t R = sp.shape.size();
  if (R > size_t(kMaxRank)) throw Error(WKF_ERR_UNSUPPORTED, "map kernel: more than 6 non-mergeable dimensions");
  // Vector width: 16 bytes of the widest element type, shrunk until every operand
  // is either unit-stride and aligned or a broadcast along the inner dimension.
  size_t max_elem = 2;
  for (size_t k = 0; k < N; k++) max_elem = std::max(max_elem, dtype_size(td_of(k).dtype));
  int vec = int(16 / max_elem);
  auto vec_ok = [&](int V) {
    if (sp.shape[R - 1] % V) return false;
    for (size_t k = 0; k < N; k++) {
      size_t inner = sp.strides[k][R - 1];
      if (inner > 1) return false;
      if (inner == 0) {
        if (k >= in.size()) return false;
        continue;
      }
      if (td_of(k).layout.offset % V) return false;
      for (size_t d = 0; d + 1 < R; d++)
        if (sp.strides[k][d] % V) return false;
    }
    return true;
  };
  while (vec > 1 && !vec_ok(vec)) vec /= 2;

  MapSpec spec;
  spec.rank = int(R);
  spec.vec = vec;
  spec.prog = prog;
  spec.math = st_.exact_math ? MathPolicy::Exact : st_.math_f32 ? MathPolicy::Folded : MathPolicy::Stored;
  // Inputs that run along another dimension than the output (a transposed operand): tiled kernel.
  spec.more_prog = more_prog;
  if (vec == 1 && R >= 2 && numel >= (size_t(1) << 16) && sp.strides[N - 1][R - 1] == 1 && sp.shape[R - 1] >= 16 &&
      st_.fusion != FusionMode::Reference && more_out.empty()) {
    int ta = -1;
    for (size_t k = 0; k + 1 < N && ta < 0; k++) {
      if (sp.strides[k][R - 1] <= 1) continue;
      for (size_t dd = 0; dd + 1 < R; dd++)
        if (sp.strides[k][dd] == 1 && sp.shape[dd] >= 16) ta = int(dd);
    }
    if (ta >= 0) {
      size_t ncrossed = 0;
      for (size_t k = 0; k + 1 < N; k++) {
        const bool x = sp.strides[k][R - 1] > 1 && sp.strides[k][ta] != 0 && sp.strides[k][ta] < sp.strides[k][R - 1];
        spec.crossed.push_back(x);
        ncrossed += x;
      }
      if (ncrossed >= 1 && ncrossed <= 3) spec.tile_dim = ta;
    }
  }
  if (spec.tile_dim >= 0) {
    launch_map_tiled(spec, sp, in, out, in_place);
    return;
  }
  const size_t nwork = numel / vec;
  spec.unroll = nwork >= (1u << 20) ? st_.map_unroll : nwork >= (1u << 16) ? 2 : 1;
  // A costly value that depends on one f16 operand only (silu(a) inside silu(a) * (b + bias), the whole chain over a
  // strided view) is a function of 16 bits: the kernel looks it up in a table held in the LDS instead of computing it.
  std::string tabled;
  BufRef table;
  if (more_out.empty()) table = cut_table(spec.prog, in, numel, &tabled);
  if (table) {
    spec.table = true;
    spec.unroll = 1;
  }
  size_t bytes = 0;
  std::vector<size_t> cstrides = Layout::contiguous_strides(sp.shape);
  for (size_t k = 0; k < N; k++) {
    MapOperandSpec os;
    os.dtype = td_of(k).dtype;
    os.linear = sp.strides[k] == cstrides;
    os.inner_stride = vec > 1 ? int(sp.strides[k][R - 1]) : -1;
    if (os.linear) os.inner_stride = vec > 1 ? 1 : -1;
    if (k < in.size()) spec.in.push_back(os);
    else if (k == in.size()) spec.out = os;
    else spec.more_out.push_back(os);
    bytes += os.linear ? numel * dtype_size(os.dtype) : 0;
  }
  spec.nontemporal = bytes >= st_.nontemporal_bytes;

  MapArgs args;
  // (a block computes the index of its first work item plus up to 16384: that sum stays below 2^32 as well)
  if (nwork > 0xffffffffull - (size_t(1) << 16)) throw Error(WKF_ERR_UNSUPPORTED, "map kernel: more than 2^32 - 2^16 work items");
  args.nwork = to_u32(nwork, "tensor size");
  for (size_t d = 0; d < R; d++) args.shape.push_back(to_u32(d == R - 1 ? sp.shape[d] / vec : sp.shape[d], "shape"));
  for (size_t k = 0; k < N; k++) {
    const TensorData& td = td_of(k);
    to_u32(td.layout.extent(), "tensor extent");
    if (td.layout.extent() * dtype_size(td.dtype) > wkf_buffer_size(td.buffer.get()) + 3)
      invalid("map kernel: a layout reaches past the end of its buffer");
    args.ptrs.push_back(element_ptr(td));
    args.offsets.push_back(to_u32(td.layout.offset, "offset"));
    std::vector<uint32_t> st;
    for (size_t d = 0; d < R; d++) st.push_back(to_u32(sp.strides[k][d], "stride"));
    args.strides.push_back(st);
  }
  args.consts = prog.consts;
  for (const Program& p : more_prog) args.consts.insert(args.consts.end(), p.consts.begin(), p.consts.end());
  if (table) args.table = wkf_buffer_ptr(table.get());

  std::string sig = map_signature(spec);
  wkf_kernel* k = kernel(sig, [&] { return map_source(spec); });
  LaunchRecord r;
  r.kind = "map";
  r.signature = sig;
  r.in_place = in_place;
  size_t per_block = size_t(table ? kMapTableBlock : kMapBlock) * spec.unroll;
  r.grid[0] = to_u32((nwork + per_block - 1) / per_block, "grid");
  r.block[0] = table ? kMapTableBlock : kMapBlock;
  if (table) {
    // one workgroup per compute unit keeps the table and walks the chunks
    wkf_props props;
    check(wkf_device_props(dev_, &props));
    r.grid[0] = std::min(r.grid[0], uint32_t(std::max(1, props.compute_units)));
  }
  std::ostringstream d;
  d << "shape=" << dims(sp.shape) << " vec=" << vec << " unroll=" << spec.unroll << " operands=" << N
    << (in_place ? " in_place" : "");
  if (table) d << " table lookup: 65536 values of " << tabled;
  if (!more_out.empty()) d << " outputs=" << 1 + more_out.size();
  r.detail = d.str();
  record(std::move(r), k, map_pack_args(spec, args));
}

void Resolver::launch_map_tiled(MapSpec& spec, const Space& sp, const std::vector<TensorData>& in, const TensorData& out,
                                bool in_place) {
  const size_t R = sp.shape.size(), N = in.size() + 1, ta = size_t(spec.tile_dim);
  auto td_of = [&](size_t k) -> const TensorData& { return k < in.size() ? in[k] : out; };
  spec.unroll = 1;
  spec.nontemporal = false;
  // four elements per access when every operand allows it: unit stride along its own dimension of the tile (or, for an
  // input that does not cross, none along the last one), everything else a multiple of four elements
  bool vec4 = st_.map_tile_vec && sp.shape[ta] % 4 == 0 && sp.shape[R - 1] % 4 == 0;
  for (size_t k = 0; k < N && vec4; k++) {
    const bool crossed = k < in.size() && spec.crossed[k];
    const size_t own = crossed ? ta : R - 1;
    const size_t s_own = sp.strides[k][own];
    if (!crossed && k < in.size() && s_own == 0) continue;  // one value per tile row: a scalar load, nothing to align
    if (s_own != 1) vec4 = false;
    for (size_t d = 0; d < R; d++)
      if (d != own && sp.strides[k][d] % 4) vec4 = false;
    if (td_of(k).layout.offset % 4) vec4 = false;
  }
  spec.tile_vec = vec4 ? 4 : 1;
  {
    size_t bytes = 0;
    for (size_t k = 0; k < N; k++) bytes += out.layout.numel() * dtype_size(td_of(k).dtype);
    spec.nontemporal = vec4 && bytes >= st_.nontemporal_bytes;
  }
  for (size_t k = 0; k < N; k++) {
    MapOperandSpec os;
    os.dtype = td_of(k).dtype;
    os.linear = false;
    os.inner_stride = vec4 && k < in.size() && !spec.crossed[k] ? int(sp.strides[k][R - 1]) : -1;
    if (k < in.size()) spec.in.push_back(os);
    else spec.out = os;
  }
  MapArgs args;
  args.nwork = to_u32(out.layout.numel(), "tensor size");
  for (size_t d = 0; d < R; d++) args.shape.push_back(to_u32(sp.shape[d], "shape"));
  for (size_t k = 0; k < N; k++) {
    const TensorData& td = td_of(k);
    to_u32(td.layout.extent(), "tensor extent");
    if (td.layout.extent() * dtype_size(td.dtype) > wkf_buffer_size(td.buffer.get()) + 3)
      invalid("map kernel: a layout reaches past the end of its buffer");
    args.ptrs.push_back(element_ptr(td));
    args.offsets.push_back(to_u32(td.layout.offset, "offset"));
    std::vector<uint32_t> st;
    for (size_t d = 0; d < R; d++) st.push_back(to_u32(sp.strides[k][d], "stride"));
    args.strides.push_back(st);
  }
  args.consts = spec.prog.consts;
  // Tiles of 128 x 128 where four-element accesses are possible, both extents reach 128, there are tiles enough for the
  // chip twice over, and the crossed inputs' tiles leave room for two workgroups per compute unit: a row of such a tile
  // is 512 consecutive bytes of f32 instead of 256 (a transposing copy of f32 [8192,8192]: 5.0 -> 5.5 TB/s).
  if (vec4 && st_.map_tile_128 && sp.shape[ta] >= 128 && sp.shape[R - 1] >= 128) {
    size_t lds = 0, tiles = ((sp.shape[ta] + 127) / 128) * ((sp.shape[R - 1] + 127) / 128);
    for (size_t k = 0; k < in.size(); k++)
      if (spec.crossed[k]) lds += 128 * (128 + (dtype_size(in[k].dtype) == 2 ? 2 : 1)) * dtype_size(in[k].dtype);
    for (size_t d = 0; d + 1 < R; d++)
      if (d != ta) tiles *= sp.shape[d];
    wkf_props props;
    check(wkf_device_props(dev_, &props));
    if (lds <= 80 * 1024 && tiles >= 2 * size_t(std::max(1, props.compute_units))) spec.tile_size = 128;
  }
  const size_t kTile = size_t(spec.tile_size);
  size_t blocks = ((sp.shape[ta] + kTile - 1) / kTile) * ((sp.shape[R - 1] + kTile - 1) / kTile);
  for (size_t d = 0; d + 1 < R; d++)
    if (d != ta) blocks *= sp.shape[d];
  std::string sig = map_signature(spec);
  wkf_kernel* k = kernel(sig, [&] { return map_source(spec); });
  LaunchRecord r;
  r.kind = "map";
  r.signature = sig;
  r.grid[0] = to_u32(blocks, "grid");
  r.block[0] = kMapBlock;
  std::ostringstream d;
  d << "shape=" << dims(sp.shape) << " tiled dim=" << ta << " operands=" << N << (vec4 ? " vec=4" : "") << (spec.tile_size != 64 ? " tile=128" : "")
    << (in_place ? " in_place" : "");
  r.detail = d.str();
  r.in_place = in_place;
  record(std::move(r), k, map_pack_args(spec, args));
}

TensorData Resolver::make_contiguous(const TensorData& td) {
  if (td.layout.is_contiguous()) return td;
  TensorData out = alloc(td.layout.shape, td.dtype, false);
  Program p;
  Instr in;
  in.op = Op::Load;
  in.dtype = td.dtype;
  in.operand = 0;
  p.ins.push_back(in);
  p.result = 0;
  launch_map(p, {td}, out, false);
  return out;
}

TensorData Resolver::run_reduce(const NodeP& rn, const std::vector<const Node*>& post_chain) {
  ExprBuilder eb;
  int v = build(eb, rn->a, pairwise_budget_for_reduce());
  eb.prog.result = v;
  const DType pre_dt = eb.prog.result_dtype();
  // post: the chain above the reduce, innermost first (src/compute_graph/resolve.rs:164-196)
  Program post;
  {
    Instr ld;
    ld.op = Op::Load;
    ld.dtype = pre_dt;
    ld.operand = 0;
    post.ins.push_back(ld);
    int cur = 0;
    for (size_t i = post_chain.size(); i-- > 0;) {
      const Node* c = post_chain[i];
      Instr in;
      in.op = c->op;
      in.a = cur;
      in.dtype = c->dtype;
      if (is_const_op(c->op)) {
        in.cslot = int(post.consts.size());
        post.consts.push_back(c->constant);
      }
      post.ins.push_back(in);
      cur = int(post.ins.size()) - 1;
    }
    post.result = cur;
  }
  const std::vector<size_t>& shape = rn->a->shape;
  const size_t axis = rn->axis;
  if (axis >= shape.size()) invalid("reduce: axis out of range");
  for (const TensorData& td : eb.operands)
    if (td.layout.shape != shape) invalid("reduce: operand shapes differ");

  ReduceJob job;
  job.pre = eb.prog;
  job.operands = eb.operands;
  job.axis = axis;
  job.rop = rn->rop;
  job.post = post;
  job.fold_dtype = pre_dt;

  // Few outputs over a long axis leave most of the chip idle: fold S slices of the axis side by side
  // into f32 partials, then fold the partials.  (The reference always uses one workgroup per output,
  // src/reduce.rs:316-346.)
  const size_t n = shape[axis];
  size_t nrows = 1;
  for (size_t d = 0; d < shape.size(); d++)
    if (d != axis) nrows *= shape[d];
  const size_t S = st_.fusion == FusionMode::Reference ? 1 : reduce_split(job, nrows, n);
  if (S <= 1) return launch_reduce(job);

  // The slice index goes where the axis was when the axis is the unit-stride one (rows and slices then
  // merge into one dimension), in front otherwise (the lanes stay on the unit-stride outputs).
  bool row = true;
  for (const TensorData& td : job.operands) row &= td.layout.strides[axis] <= 1;
  const size_t pos = row ? axis : 0;
  ReduceJob first = job;
  first.raw = true;
  first.axis = axis + 1;
  for (TensorData& td : first.operands) {
    Layout l;
    l.offset = td.layout.offset;
    for (size_t d = 0; d < shape.size(); d++) {
      if (d == pos) {
        l.shape.push_back(S);
        l.strides.push_back(td.layout.strides[axis] * (n / S));
      }
      l.shape.push_back(d == axis ? n / S : shape[d]);
      l.strides.push_back(td.layout.strides[d]);
    }
    td.layout = l;
  }
  if (reduce_outer_rank(first) > 3) return launch_reduce(job);
  TensorData partial = launch_reduce(first);

  ReduceJob second;
  {
    Instr ld;
    ld.op = Op::Load;
    ld.dtype = DType::F32;
    ld.operand = 0;
    second.pre.ins.push_back(ld);
    second.pre.result = 0;
  }
  second.operands = {partial};
  second.axis = pos;
  second.rop = rn->rop;
  second.post = post;
  second.fold_dtype = pre_dt;
  return launch_reduce(second);
}

size_t Resolver::reduce_outer_rank(const ReduceJob& job) {
  const std::vector<size_t>& shape = job.operands[0].layout.shape;
  std::vector<size_t> out_shape;
  std::vector<std::vector<size_t>> ostr(job.operands.size() + 1);
  for (size_t d = 0; d < shape.size(); d++) {
    if (d == job.axis) continue;
    out_shape.push_back(shape[d]);
    for (size_t k = 0; k < job.operands.size(); k++) ostr[k].push_back(job.operands[k].layout.strides[d]);
  }
  ostr.back() = Layout::contiguous_strides(out_shape);
  return coalesce(out_shape, ostr).shape.size();
}

size_t Resolver::reduce_split(const ReduceJob& job, size_t nrows, size_t n) {
  if (nrows == 0 || n < 4096) return 1;
  bool row = true;
  for (const TensorData& td : job.operands) row &= td.layout.strides[job.axis] <= 1;
  wkf_props props;
  check(wkf_device_props(dev_, &props));
  const size_t cus = size_t(std::max(1, props.compute_units));
  size_t S = 1;
  if (row) {
    // one block of 1024 lanes per row: split until there are about four blocks per compute unit,
    // keeping at least 8192 elements per slice
    while (nrows * S < 4 * cus && n / (2 * S) >= 8192 && n % (2 * S) == 0) S *= 2;
  } else {
    // one block of 16 waves per 256 (at best) neighbouring outputs: keep at least 128 axis steps per slice
    const size_t blocks = (nrows + 255) / 256;
    while (blocks * S < 8 * cus && n / (2 * S) >= 128 && n % (2 * S) == 0) S *= 2;
  }
  return S;
}

TensorData Resolver::launch_reduce(const ReduceJob& job) {
  const std::vector<TensorData>& ops = job.operands;
  const std::vector<size_t>& shape = ops[0].layout.shape;
  const size_t axis = job.axis;
  const DType pre_dt = job.pre.result_dtype();
  const DType out_dt = job.raw ? DType::F32 : job.post.result_dtype();
  std::vector<size_t> out_shape;
  for (size_t d = 0; d < shape.size(); d++)
    if (d != axis) out_shape.push_back(shape[d]);
  // (raw partial sums are a temporary; anything else a reduce launch stores is the value of its reduce node)
  TensorData out = alloc(out_shape, out_dt, false, !job.raw);
  const size_t nrows = out.layout.numel();
  const size_t n = shape[axis];
  if (nrows == 0) return out;

  const size_t N = ops.size();
  std::vector<std::vector<size_t>> ostr;
  for (const TensorData& td : ops) {
    std::vector<size_t> s;
    for (size_t d = 0; d < shape.size(); d++)
      if (d != axis) s.push_back(td.layout.strides[d]);
    ostr.push_back(s);
  }
  ostr.push_back(out.layout.strides);
  Space sp = coalesce(out_shape, ostr);
  const size_t Ro = sp.shape.size();
  if (Ro > 3) {
    // The reduce kernels decode at most three outer dimensions (the reference's takes any rank, src/reduce.rs:83-281):
    // a view whose outer dimensions do not merge that far is copied into a dense buffer first (one map pass, any
    // rank up to the map kernel's), after which the dimensions on either side of the axis merge into one each.
    bool dense = true;
    for (const TensorData& td : ops) dense &= td.layout.is_contiguous();
    if (dense) throw Error(WKF_ERR_UNSUPPORTED, "reduce kernel: more than 3 non-mergeable outer dimensions");
    ReduceJob copy = job;
    for (TensorData& td : copy.operands) td = make_contiguous(td);
    return launch_reduce(copy);
  }

  ReduceSpec spec;
  spec.outer_rank = int(Ro);
  spec.rop = job.rop;
  spec.out_dtype = out_dt;
  spec.pre = job.pre;
  spec.post = job.post;
  spec.raw_out = job.raw;
  spec.fold_dtype = job.fold_dtype;
  spec.math_pre = st_.exact_math ? MathPolicy::Exact : MathPolicy::Folded;
  spec.math_post = st_.exact_math ? MathPolicy::Exact : MathPolicy::Stored;
  spec.vec = 1;
  spec.threads_per_row = 1;
  spec.block = 256;
  spec.unroll = 1;
  spec.waves = 1;
  bool row = true;
  for (const TensorData& td : ops) row &= (n <= 1 || td.layout.strides[axis] <= 1);
  spec.shape = row ? ReduceShape::Row : ReduceShape::Col;

  size_t max_elem = 2;
  for (const TensorData& td : ops) max_elem = std::max(max_elem, dtype_size(td.dtype));
  max_elem = std::max(max_elem, dtype_size(out_dt));

  LaunchRecord r;
  std::ostringstream d;
  if (row) {
    int vec = int(16 / max_elem);
    auto vec_ok = [&](int V) {
      if (n % V) return false;
      for (size_t k = 0; k < N; k++) {
        const TensorData& td = ops[k];
        if (td.layout.strides[axis] == 0) continue;
        if (td.layout.offset % V) return false;
        for (size_t dd = 0; dd < Ro; dd++)
          if (sp.strides[k][dd] % V) return false;
      }
      return true;
    };
    while (vec > 1 && !vec_ok(vec)) vec /= 2;
    spec.vec = vec;
    const size_t nvec = n / vec;
    // Lanes per row, measured on MI355X: long rows want many lanes with few loads each (two 16-byte loads
    // per lane, at most 512 lanes: 8192 floats per row run at 6.85 TB/s with 512 lanes, 6.55 with 256, 5.9
    // with 1024), short rows want few lanes (the fold across lanes costs more than the loads).  More lanes
    // per row when there are too few rows to fill the chip.
    const size_t per_lane_target = nvec >= 256 ? 2 : nvec >= 64 ? 4 : 8;
    int T = std::min(512, pow2_ceil((nvec + per_lane_target - 1) / per_lane_target));
    wkf_props props;
    check(wkf_device_props(dev_, &props));
    const size_t want_threads = size_t(props.compute_units) * 1024;
    while (T < 1024 && size_t(T) * 2 <= nvec && nrows * T < want_threads) T *= 2;
    if (st_.reduce_threads > 0 && size_t(st_.reduce_threads) <= std::max<size_t>(1, nvec)) T = st_.reduce_threads;
    spec.threads_per_row = T;
    spec.block = std::max(256, T);
    size_t per_lane = (nvec + T - 1) / T;
    spec.unroll = per_lane >= 4 ? 4 : per_lane >= 2 ? 2 : 1;
    if (st_.reduce_unroll > 0 && size_t(st_.reduce_unroll) <= per_lane) spec.unroll = st_.reduce_unroll;
    for (const TensorData& td : ops) spec.in.push_back({td.dtype, (n <= 1 || td.layout.strides[axis] == 0) ? 0 : 1, -1});
    size_t rpb = size_t(spec.block / T);
    r.grid[0] = to_u32((nrows + rpb - 1) / rpb, "grid");
    r.block[0] = uint32_t(spec.block);
    r.kind = "red_row";
    d << "rows=" << nrows << " n=" << n << " vec=" << vec << " threads_per_row=" << T << " unroll=" << spec.unroll;
  } else {
    // Lanes sit on the last outer dim; V neighbouring outputs per lane when every operand is
    // unit-stride (or a broadcast) and 16-byte aligned there.
    const size_t lanes_dim = Ro ? sp.shape[Ro - 1] : 1;
    int vec = Ro ? int(16 / max_elem) : 1;
    auto vec_ok = [&](int V) {
      if (lanes_dim % V) return false;
      for (size_t k = 0; k <= N; k++) {
        const TensorData& td = k < N ? ops[k] : out;
        const size_t inner = sp.strides[k][Ro - 1];
        if (inner > 1) return false;
        if (inner == 0) {
          if (k == N) return false;
          continue;
        }
        if (td.layout.offset % V) return false;
        for (size_t dd = 0; dd + 1 < Ro; dd++)
          if (sp.strides[k][dd] % V) return false;
        if (k < N && td.layout.strides[axis] % V) return false;
      }
      return true;
    };
    while (vec > 1 && !vec_ok(vec)) vec /= 2;
    spec.vec = vec;
    spec.waves = n >= 64 ? 16 : n >= 8 ? 4 : 1;
    const size_t steps = (n + spec.waves - 1) / spec.waves;
    spec.unroll = steps >= 4 ? 4 : steps >= 2 ? 2 : 1;
    for (size_t k = 0; k < N; k++) spec.in.push_back({ops[k].dtype, -1, vec > 1 ? int(sp.strides[k][Ro - 1]) : -1});
    const size_t per_block = size_t(64) * vec;
    const size_t rest = nrows / lanes_dim;
    r.grid[0] = to_u32(((lanes_dim + per_block - 1) / per_block) * rest, "grid");
    r.block[0] = uint32_t(64 * spec.waves);
    r.kind = "red_col";
    d << "outputs=" << nrows << " n=" << n << " vec=" << vec << " waves=" << spec.waves << " unroll=" << spec.unroll;
  }
  if (job.raw) d << " partial";

  ReduceArgs args;
  args.nrows = to_u32(nrows, "output size");
  args.n = to_u32(n, "axis length");
  for (size_t dd = 0; dd < Ro; dd++) args.oshape.push_back(to_u32(sp.shape[dd], "shape"));
  for (size_t k = 0; k <= N; k++) {
    const TensorData& td = k < N ? ops[k] : out;
    to_u32(td.layout.extent(), "tensor extent");
    args.ptrs.push_back(element_ptr(td));
    args.offsets.push_back(to_u32(td.layout.offset, "offset"));
    std::vector<uint32_t> st;
    for (size_t dd = 0; dd < Ro; dd++) st.push_back(to_u32(sp.strides[k][dd], "stride"));
    args.ostrides.push_back(st);
    if (k < N) args.astrides.push_back(to_u32(td.layout.strides[axis], "stride"));
  }
  args.consts = job.pre.consts;
  if (!job.raw) args.consts.insert(args.consts.end(), job.post.consts.begin(), job.post.consts.end());

  std::string sig = reduce_signature(spec);
  wkf_kernel* k = kernel(sig, [&] { return reduce_source(spec); });
  r.signature = sig;
  r.detail = d.str();
  record(std::move(r), k, reduce_pack_args(spec, args));
  (void)pre_dt;
  return out;
}

TensorData Resolver::run_map_layout(const NodeP& n) {
  // MapLayoutOperation::run, src/map_layout.rs:26-39: a view on the same buffer.
  TensorData in = resolve(n->a);
  TensorData out = in;
  const Layout& l = in.layout;
  switch (n->map_kind) {
    case MapKind::Slice: out.layout = l.slice(n->ranges); break;
    case MapKind::Transpose:
      std::swap(out.layout.shape[n->axis0], out.layout.shape[n->axis1]);
      std::swap(out.layout.strides[n->axis0], out.layout.strides[n->axis1]);
      break;
    case MapKind::Broadcast: {
      // one stride-0 dimension inserted at axis0, src/map_layout.rs:69-98
      Layout b;
      b.offset = l.offset;
      b.shape = n->new_shape;
      for (size_t i = 0; i <= l.rank(); i++) {
        if (i == n->axis0) b.strides.push_back(0);
        if (i < l.rank()) b.strides.push_back(l.strides[i]);
      }
      out.layout = b;
      break;
    }
  }
  return out;
}

TensorData Resolver::run_resize(const NodeP& n) {
  const std::vector<size_t>& in_shape = n->a->shape;
  const bool is_reshape = n->fill_shape == n->new_shape && in_shape != n->new_shape;
  ExprBuilder eb;
  if (st_.fusion == FusionMode::Tree) {
    eb.prog.result = build(eb, n->a, pairwise_budget_for_map());
  } else {
    eb.prog.result = eb.load(resolve(n->a));
  }
  const DType dt = eb.prog.result_dtype();
  if (is_reshape && st_.fusion == FusionMode::Tree && eb.prog.ins.size() == 1 && eb.prog.ins[0].op == Op::Load &&
      eb.operands[0].layout.strides == Layout::contiguous_strides(eb.operands[0].layout.shape)) {
    // Reshaping a tensor that already lies dense in memory is a new layout on the same buffer.  (The reference
    // always copies, src/resize.rs:131-144; the values are the same and the shared buffer is never written in place.)
    TensorData view = eb.operands[0];
    const size_t offset = view.layout.offset;
    view.layout = Layout::contiguous(n->new_shape);
    view.layout.offset = offset;
    return view;
  }
  if (is_reshape || in_shape == n->new_shape) {
    // reshape (src/resize.rs:131-144): a dense copy in the input's own index order;
    // the contiguous result is then read with the new shape.
    TensorData out = alloc(in_shape, dt, false);
    launch_map(eb.prog, eb.operands, out, false);
    out.layout = Layout::contiguous(n->new_shape);
    return out;
  }
  // resize (src/resize.rs:121-129): the input lands in the [0, in_shape) corner of a
  // zero-filled tensor of the new shape (wgpu zero-initialises, hipMalloc does not).
  // Where the new shape is smaller than the input the copy is cropped.
  if (in_shape.size() != n->new_shape.size()) invalid("resize: rank must not change");
  std::vector<std::pair<size_t, size_t>> corner;
  bool pad = false;
  for (size_t d = 0; d < in_shape.size(); d++) {
    corner.push_back({0, std::min(in_shape[d], n->new_shape[d])});
    pad |= n->new_shape[d] > in_shape[d];
  }
  TensorData out = alloc(n->new_shape, dt, pad);
  TensorData view = out;
  view.layout = out.layout.slice(corner);
  std::vector<TensorData> ops = eb.operands;
  for (TensorData& td : ops) td.layout = td.layout.slice(corner);
  launch_map(eb.prog, ops, view, false);
  return out;
}

namespace {
// cat([p0, ..., pk], axis) as Tensor::cat builds it (src/composite/cat.rs:3-41): resize(p0) to the total shape,
// then one slice_assign per further piece, each filling the next range of `axis`.  Returns the pieces in
// order when `n` is exactly that and the pieces tile the axis without gaps.
bool match_cat_chain(const Node* n, std::vector<NodeP>* pieces, size_t* axis) {
  std::vector<std::pair<size_t, NodeP>> assigned;  // (start on the axis, piece), outermost first
  int ax = -1;
  const Node* cur = n;
  const std::vector<size_t>& total = n->shape;
  while (cur->kind == NodeKind::SliceAssign) {
    if (cur->shape != total || cur->ranges.size() != total.size() || cur->b->shape.size() != total.size()) return false;
    int this_ax = -1;
    for (size_t d = 0; d < total.size(); d++) {
      const bool whole = cur->ranges[d] == std::make_pair(size_t(0), total[d]) && cur->b->shape[d] == total[d];
      if (whole) continue;
      if (this_ax >= 0) return false;
      this_ax = int(d);
    }
    if (this_ax < 0) return false;  // overwrites everything: not a cat
    if (ax >= 0 && ax != this_ax) return false;
    ax = this_ax;
    if (cur->ranges[ax].second - cur->ranges[ax].first != cur->b->shape[ax]) return false;
    assigned.push_back({cur->ranges[ax].first, cur->b});
    cur = cur->a.get();
  }
  if (cur->kind != NodeKind::Resize || ax < 0 || cur->new_shape != total || cur->fill_shape != cur->a->shape ||
      cur->a->shape.size() != total.size())
    return false;
  for (size_t d = 0; d < total.size(); d++)
    if (int(d) != ax && cur->a->shape[d] != total[d]) return false;
  pieces->clear();
  pieces->push_back(cur->a);
  size_t at = cur->a->shape[ax];
  for (size_t i = assigned.size(); i-- > 0;) {
    if (assigned[i].first != at) return false;
    pieces->push_back(assigned[i].second);
    at += assigned[i].second->shape[ax];
  }
  if (at != total[ax]) return false;
  *axis = size_t(ax);
  return true;
}
}  // namespace

TensorData Resolver::run_slice_assign(const NodeP& n) {
  if (st_.fusion == FusionMode::Tree) {
    // A whole cat: every piece is written once, straight into its range of a fresh buffer -- no zero fill of
    // the padded tensor and no read-back (the reference pads, copies and then assigns piece by piece).
    std::vector<NodeP> pieces;
    size_t axis = 0;
    if (match_cat_chain(n.get(), &pieces, &axis)) {
      TensorData out = alloc(n->shape, n->dtype, false);
      size_t at = 0;
      for (const NodeP& piece : pieces) {
        const size_t len = piece->shape[axis];
        if (len > 0) {
          ExprBuilder eb;
          eb.prog.result = build(eb, piece, pairwise_budget_for_map());
          if (eb.prog.result_dtype() != n->dtype) invalid("cat: dtype mismatch");
          std::vector<std::pair<size_t, size_t>> r;
          for (size_t d = 0; d < n->shape.size(); d++)
            r.push_back(d == axis ? std::make_pair(at, at + len) : std::make_pair(size_t(0), n->shape[d]));
          TensorData view = out;
          view.layout = out.layout.slice(r);
          launch_map(eb.prog, eb.operands, view, false);
        }
        at += len;
      }
      return out;
    }
  }
  TensorData target = resolve(n->a);
  if (!target.owned() || target.layout.allocation_overlaps()) {
    // The reference writes into the target's buffer whoever else holds it
    // (src/slice_assign.rs:68-72), which can change a tensor the caller still
    // uses.  A shared target is copied first.
    TensorData copy = alloc(target.layout.shape, target.dtype, false);
    Program p;
    Instr ld;
    ld.op = Op::Load;
    ld.dtype = target.dtype;
    ld.operand = 0;
    p.ins.push_back(ld);
    p.result = 0;
    launch_map(p, {target}, copy, false);
    target = copy;
  }
  ExprBuilder eb;
  if (st_.fusion == FusionMode::Tree) eb.prog.result = build(eb, n->b, pairwise_budget_for_map());
  else eb.prog.result = eb.load(resolve(n->b));
  if (eb.prog.result_dtype() != target.dtype) invalid("slice_assign: dtype mismatch");
  TensorData view = target;
  view.layout = target.layout.slice(n->ranges);
  if (view.layout.shape != n->b->shape)
    invalid("slice_assign: value shape " + dims(n->b->shape) + " does not match the slice " + dims(view.layout.shape));  // src/slice_assign.rs:69
  launch_map(eb.prog, eb.operands, view, true);
  return target;
}

}  // namespace wkf

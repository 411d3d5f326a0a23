// Device-agnostic host types shared by the lazy graph, the fusion pass and the
// kernel generator: data types, op codes, layouts, tensor data, graph nodes and
// the fused-expression program.  Citations name files of the reference crate.
#pragma once

#include <cstddef>
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "wkf_hip.h"

namespace wkf {

// DataTypeEnum, src/tensor.rs:69-88.
enum class DType : int { F32 = 0, F16 = 1 };
inline size_t dtype_size(DType d) { return d == DType::F32 ? 4 : 2; }
inline const char* dtype_name(DType d) { return d == DType::F32 ? "f32" : "f16"; }

// One code per element-wise / pair-wise function of the reference
// (src/element_wise.rs:197-1471, src/pair_wise.rs:205-528).  The numeric values
// are part of the C ABI (include/wkf_tensor.h).
enum class Op : int {
  AddC = 0, SubC, RSubC, MulC, DivC, RDivC,                          // tensor (op) f32 literal
  Exp = 16, Exp2, Log, Log2, Sqr, Sqrt, Sin, Cos, Tan, Asin, Acos,   // unary
  Atan, Sinh, Cosh, Tanh, Asinh, Acosh, Atanh, Abs, Neg,
  Cast = 48,                                                         // to the instruction's dtype
  Add = 64, Sub, Mul, Div, Pow,                                      // pair-wise
  Load = 96,                                                         // read operand #operand
  Lookup = 97,                                                       // f16 only: the value the kernel's table holds for the bit pattern of `a` (planner-made, never part of a graph)
};
inline bool is_const_op(Op o) { return int(o) >= 0 && int(o) <= int(Op::RDivC); }
inline bool is_unary_op(Op o) { return int(o) >= int(Op::Exp) && int(o) <= int(Op::Neg); }
inline bool is_binary_op(Op o) { return int(o) >= int(Op::Add) && int(o) <= int(Op::Pow); }
const char* op_name(Op o);

// src/reduce.rs:433-815.
enum class ReduceOp : int { Sum = 0, Max = 1, Min = 2, Product = 3 };
const char* reduce_name(ReduceOp r);

struct Error : std::runtime_error {
  int code;
  Error(int c, const std::string& m) : std::runtime_error(m), code(c) {}
};
[[noreturn]] inline void invalid(const std::string& m) { throw Error(WKF_ERR_INVALID_ARG, m); }

// Layout in ELEMENT units, src/layout.rs:33-94.
struct Layout {
  size_t offset = 0;
  std::vector<size_t> shape;
  std::vector<size_t> strides;

  static Layout contiguous(const std::vector<size_t>& shape);
  static std::vector<size_t> contiguous_strides(const std::vector<size_t>& shape);
  size_t rank() const { return shape.size(); }
  size_t numel() const;
  bool is_contiguous() const;          // offset == 0 && row-major strides, src/layout.rs:58-60
  bool allocation_overlaps() const;    // any stride 0, src/layout.rs:87-89
  Layout slice(const std::vector<std::pair<size_t, size_t>>& ranges) const;  // src/layout.rs:62-71
  // Largest element index touched + 1 (0 for an empty layout).
  size_t extent() const;
  bool operator==(const Layout& o) const { return offset == o.offset && shape == o.shape && strides == o.strides; }
};

// Intrusive reference to a level-0 buffer.
class BufRef {
 public:
  BufRef() = default;
  explicit BufRef(wkf_buffer* adopt) : b_(adopt) {}
  BufRef(const BufRef& o) : b_(o.b_) { wkf_buffer_retain(b_); }
  BufRef(BufRef&& o) noexcept : b_(o.b_) { o.b_ = nullptr; }
  BufRef& operator=(BufRef o) { std::swap(b_, o.b_); return *this; }
  ~BufRef() { wkf_buffer_release(b_); }
  wkf_buffer* get() const { return b_; }
  explicit operator bool() const { return b_ != nullptr; }
  void reset() { wkf_buffer_release(b_); b_ = nullptr; }
 private:
  wkf_buffer* b_ = nullptr;
};

// TensorData, src/tensor.rs:301-416: ref-counted device buffer + layout + dtype.
struct TensorData {
  wkf_device* device = nullptr;
  BufRef buffer;
  Layout layout;
  DType dtype = DType::F32;
  bool owned() const { return wkf_buffer_refcount(buffer.get()) == 1; }  // src/tensor.rs:413-415
};

// ---- the lazy graph ------------------------------------------------------
// The reference keeps eight node tables keyed by typed ids inside a shared,
// mergeable graph object (src/compute_graph/mod.rs:20-276).  Here a node owns
// its parents through shared pointers, so there is nothing to merge when two
// tensors meet and a node dies with its last handle.
enum class NodeKind { Tensor, ElementWise, PairWise, Reduce, MatMul, MapLayout, Resize, SliceAssign };

struct Node;
using NodeP = std::shared_ptr<Node>;

enum class MapKind { Slice, Transpose, Broadcast };

struct Node {
  NodeKind kind;
  DType dtype;                     // dtype of this node's value
  std::vector<size_t> shape;       // static shape (TensorInfo, src/tensor.rs:90-150)
  NodeP a, b;                      // inputs (b: second operand / slice_assign value)
  Op op = Op::Load;                // ElementWise / PairWise
  float constant = 0.f;            // ElementWise with a literal
  ReduceOp rop = ReduceOp::Sum;    // Reduce
  size_t axis = 0;                 // Reduce
  MapKind map_kind = MapKind::Slice;              // MapLayout
  std::vector<std::pair<size_t, size_t>> ranges;  // MapLayout::Slice, SliceAssign
  size_t axis0 = 0, axis1 = 0;                    // MapLayout::Transpose; Broadcast: axis0 = inserted dim
  std::vector<size_t> new_shape, fill_shape;      // Resize (src/resize.rs:12-26); Broadcast: new_shape
  TensorData data;                                // Tensor leaf
};

// ---- fused expression program ---------------------------------------------
// What the reference passes around as lists of WGSL snippets
// (ElementWiseFunction, src/element_wise.rs:167-195) is kept as a small SSA
// program: every instruction yields one value of its own dtype, rounded to
// that dtype before the next instruction sees it (src/kernel.rs:540-553).
struct Instr {
  Op op;
  int a = -1, b = -1;   // value ids of the inputs
  DType dtype;          // dtype of the result
  int operand = -1;     // Load: which kernel operand
  int cslot = -1;       // const ops: index into the constant array
};

struct Program {
  std::vector<Instr> ins;
  std::vector<float> consts;
  int result = -1;
  // The result is read by further arithmetic outside this program (the program fills a lookup table for a value that
  // the kernel it was cut from computes in its interior): its last op is evaluated the way an interior op is.
  bool result_feeds = false;
  DType result_dtype() const { return ins[result].dtype; }
  // Text that identifies the program's structure (constants excluded: they are kernel arguments).
  std::string signature() const;
};

enum class FusionMode : int {
  Reference = 0,  // exactly the rules of src/compute_graph/resolve.rs:49-196
  Tree = 1,       // + pair-wise trees and copies fuse (README.md:19-21 of the reference lists these as to-do)
};

}  // namespace wkf

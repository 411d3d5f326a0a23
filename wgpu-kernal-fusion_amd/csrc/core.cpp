#include "core.h"

#include <sstream>

namespace wkf {

const char* op_name(Op o) {
  switch (o) {
    case Op::AddC: return "add_const";
    case Op::SubC: return "subtract_const";
    case Op::RSubC: return "const_subtract";
    case Op::MulC: return "multiply_const";
    case Op::DivC: return "divide_const";
    case Op::RDivC: return "const_divide";
    case Op::Exp: return "exp";
    case Op::Exp2: return "exp2";
    case Op::Log: return "log";
    case Op::Log2: return "log2";
    case Op::Sqr: return "sqr";
    case Op::Sqrt: return "sqrt";
    case Op::Sin: return "sin";
    case Op::Cos: return "cos";
    case Op::Tan: return "tan";
    case Op::Asin: return "asin";
    case Op::Acos: return "acos";
    case Op::Atan: return "atan";
    case Op::Sinh: return "sinh";
    case Op::Cosh: return "cosh";
    case Op::Tanh: return "tanh";
    case Op::Asinh: return "asinh";
    case Op::Acosh: return "acosh";
    case Op::Atanh: return "atanh";
    case Op::Abs: return "abs";
    case Op::Neg: return "neg";
    case Op::Cast: return "cast";
    case Op::Add: return "add";
    case Op::Sub: return "sub";
    case Op::Mul: return "mul";
    case Op::Div: return "div";
    case Op::Pow: return "pow";
    case Op::Load: return "load";
    case Op::Lookup: return "lookup";
  }
  return "?";
}

const char* reduce_name(ReduceOp r) {
  switch (r) {
    case ReduceOp::Sum: return "sum";
    case ReduceOp::Max: return "max";
    case ReduceOp::Min: return "min";
    case ReduceOp::Product: return "product";
  }
  return "?";
}

std::vector<size_t> Layout::contiguous_strides(const std::vector<size_t>& shape) {
  std::vector<size_t> s(shape.size());
  size_t acc = 1;
  for (size_t i = shape.size(); i-- > 0;) {
    s[i] = acc;
    acc *= shape[i];
  }
  return s;
}

Layout Layout::contiguous(const std::vector<size_t>& shape) {
  Layout l;
  l.offset = 0;
  l.shape = shape;
  l.strides = contiguous_strides(shape);
  return l;
}

size_t Layout::numel() const {
  size_t n = 1;
  for (size_t d : shape) n *= d;
  return n;
}

bool Layout::is_contiguous() const { return offset == 0 && strides == contiguous_strides(shape); }

bool Layout::allocation_overlaps() const {
  for (size_t s : strides)
    if (s == 0) return true;
  return false;
}

Layout Layout::slice(const std::vector<std::pair<size_t, size_t>>& ranges) const {
  if (ranges.size() != shape.size()) invalid("slice: one range per dimension is required");
  Layout l;
  l.offset = offset;
  l.strides = strides;
  l.shape.resize(shape.size());
  for (size_t i = 0; i < ranges.size(); i++) {
    if (ranges[i].first > ranges[i].second) invalid("slice: range start is past its end");
    l.offset += strides[i] * ranges[i].first;
    l.shape[i] = ranges[i].second - ranges[i].first;
  }
  return l;
}

size_t Layout::extent() const {
  if (numel() == 0) return 0;
  size_t last = offset;
  for (size_t i = 0; i < shape.size(); i++) last += (shape[i] - 1) * strides[i];
  return last + 1;
}

std::string Program::signature() const {
  std::ostringstream s;
  for (size_t i = 0; i < ins.size(); i++) {
    const Instr& in = ins[i];
    if (i) s << ';';
    s << op_name(in.op) << ':' << dtype_name(in.dtype);
    if (in.op == Op::Load) s << "@" << in.operand;
    else {
      s << '(' << in.a;
      if (in.b >= 0) s << ',' << in.b;
      if (in.cslot >= 0) s << ",c" << in.cslot;
      s << ')';
    }
  }
  s << "->" << result;
  if (result_feeds) s << "!";
  return s.str();
}

}  // namespace wkf

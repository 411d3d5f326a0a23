#include "codegen.h"

#include <cstring>
#include <sstream>

namespace wkf {
namespace {

const char* ctype(DType d) { return d == DType::F32 ? "float" : "_Float16"; }

std::string vtype(DType d, int v) {
  if (v == 1) return ctype(d);
  return std::string(d == DType::F32 ? "wkf_f32x" : "wkf_f16x") + std::to_string(v);
}

// Shared by every generated translation unit.
const char* const kPrelude =
#include "kernels/prelude.hip.inc"
    ;

// exp / sin / cos with f64 Taylor cores; appended only to kernels that use them.
const char* const kMath =
#include "kernels/math.hip.inc"
    ;

// True when instruction i of p is evaluated with an f64 core under `policy`.
bool exact_op(const Program& p, size_t i, MathPolicy policy) {
  if (policy == MathPolicy::Exact) return true;
  if (policy == MathPolicy::Folded) return false;
  for (size_t j = i + 1; j < p.ins.size(); j++)
    if (p.ins[j].a == int(i) || p.ins[j].b == int(i)) return true;  // interior: something reads it
  return p.result_feeds && int(i) == p.result;                       // ... or something outside the program does
}

bool has_core(Op o) { return o == Op::Exp || o == Op::Sin || o == Op::Cos || o == Op::Tanh; }

// Needs the f64 cores of kernels/math.hip.inc.
bool uses_math(const Program& p, MathPolicy policy) {
  for (size_t i = 0; i < p.ins.size(); i++)
    if (has_core(p.ins[i].op) && exact_op(p, i, policy)) return true;
  return false;
}

// An exact transcendental op with an f16 result outside exact-math mode: the f32 library settles the f16 rounding
// for all but a few arguments in a thousand, and only those go through f64 (wkf_h_via_f32 below).
bool h_via_f32(const Program& p, size_t i, MathPolicy policy) {
  return p.ins[i].dtype == DType::F16 && policy != MathPolicy::Exact && exact_op(p, i, policy);
}

// Uses the branch-free sin / cos core, i.e. needs the `far` flag and a far variant.
bool uses_trig(const Program& p, MathPolicy policy) {
  for (size_t i = 0; i < p.ins.size(); i++)
    if ((p.ins[i].op == Op::Sin || p.ins[i].op == Op::Cos) && exact_op(p, i, policy) && !h_via_f32(p, i, policy)) return true;
  return false;
}

// An exact transcendental op with an f16 result is evaluated in f64 and rounded to f16 ONCE.  The
// compiler's f64 -> f16 conversion is a long integer sequence, so the common case goes f64 -> f32 -> f16
// and only a value whose f32 rounding lies within an f32 ulp of an f16 rounding boundary (where the two
// roundings could differ from one) takes the direct conversion.
const char* const kRoundH =
    "static __device__ __forceinline__ _Float16 wkf_round_h(double d) {\n"
    "  const float y = (float)d;\n"
    "  const _Float16 lo = (_Float16)(y * 0x1.fffffep-1f), hi = (_Float16)(y * 0x1.000002p+0f);\n"
    "  if (__builtin_expect(lo == hi, 1)) return lo;\n"
    "  return (_Float16)d;\n"
    "}\n"
    // An f16 result that feeds further arithmetic must be the correctly rounded one.  The f32 library's value y is
    // within a few f32 ulps of the true one; y (1 -+ 2^-20) brackets it with room to spare (16 ulps), and when both
    // ends round to the same f16 value that value is the answer.  Otherwise (about two arguments in a thousand) the
    // f64 routine decides.  Conversions are compared, not bits, so zeros, subnormals, infinities and NaN need no case.
    "template <typename F> static __device__ __forceinline__ _Float16 wkf_h_via_f32(float y, F exact) {\n"
    "  const _Float16 lo = (_Float16)(y * 0x1.ffffe0p-1f), hi = (_Float16)(y * 0x1.000010p+0f);\n"
    "  if (__builtin_expect(lo == hi, 1)) return lo;\n"
    "  return exact();\n"
    "}\n";

bool is_transcendental(Op o) {
  switch (o) {
    case Op::Load: case Op::AddC: case Op::SubC: case Op::RSubC: case Op::MulC: case Op::DivC: case Op::RDivC: case Op::Sqr:
    case Op::Neg: case Op::Abs: case Op::Cast: case Op::Add: case Op::Sub: case Op::Mul: case Op::Div: case Op::Sqrt: case Op::Lookup:
      return false;
    default:
      return true;
  }
}

bool uses_round_h(const Program& p, MathPolicy policy) {
  for (size_t i = 0; i < p.ins.size(); i++)
    if (p.ins[i].dtype == DType::F16 && is_transcendental(p.ins[i].op) && exact_op(p, i, policy)) return true;
  return false;
}

const char* lib_fn(Op o) {
  switch (o) {
    case Op::Exp: return "exp";
    case Op::Exp2: return "exp2";
    case Op::Log: return "log";
    case Op::Log2: return "log2";
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
    default: return nullptr;
  }
}

// f32 -> f32 call text of a unary math op on the f32 expression `a`.
// `wide`: the destination is f16, so an exact op yields its f64 value (rounded once by the caller's cast).
std::string math_call(Op o, const std::string& a, bool exact, bool far_variant, bool wide = false) {
  const std::string f = lib_fn(o);
  if (o == Op::Sqrt || !exact) return f + "f(" + a + ")";  // sqrtf is correctly rounded already
  const char* d = wide ? "_d" : "";
  if (o == Op::Exp) return std::string("wkf_exp") + d + "(" + a + ")";
  if (o == Op::Tanh) return std::string("wkf_tanh") + d + "(" + a + ")";
  if (o == Op::Sin || o == Op::Cos) return "wkf_" + f + (far_variant ? std::string("_far") + d + "(" + a + ")" : std::string(d) + "(" + a + ", far)");
  return (wide ? "" : "(float)") + f + "((double)(" + a + "))";  // the library's f64 routine, rounded once
}

// Emits `static __device__ RT name(T0 x0, ..., const float* c[, bool& far])`: one
// statement per fused op, each result held in a variable of the op's own dtype so
// that it is rounded before the next op reads it (src/kernel.rs:540-553 gives
// every fused function a typed signature for the same effect).
// A program with sin / cos gets two functions: `name`, whose branch-free trig sets
// `far` when an argument is outside its exact range, and `name_far`, which goes
// through the library's f64 sin / cos and is called to redo the work when `far`.
void emit_program_variant(std::ostringstream& o, const Program& p, const std::string& name,
                          const std::vector<DType>& operand_types, MathPolicy policy, bool far_variant) {
  const bool trig = uses_trig(p, policy);
  o << "static __device__ " << (far_variant ? "__attribute__((noinline)) " : "__forceinline__ ") << ctype(p.result_dtype())
    << " " << name << (far_variant ? "_far" : "") << "(";
  for (size_t i = 0; i < operand_types.size(); i++) o << ctype(operand_types[i]) << " x" << i << ", ";
  if (far_variant) {
    // constants by value: handing a pointer into the kernel-argument block to a function that is not
    // inlined makes the compiler copy the whole block to scratch memory and use it from there
    o << "int";
    for (size_t i = 0; i < p.consts.size(); i++) o << ", float k" << i;
    o << ") {\n";
  } else {
    o << "const float* c" << (trig ? ", bool& far" : "") << ") {\n";
  }
  for (size_t i = 0; i < p.ins.size(); i++) {
    const Instr& in = p.ins[i];
    const bool h = in.dtype == DType::F16;
    const char* t = ctype(in.dtype);
    std::string a = "v" + std::to_string(in.a), b = "v" + std::to_string(in.b);
    const std::string kref = far_variant ? "k" + std::to_string(in.cslot) : "c[" + std::to_string(in.cslot) + "]";
    std::string k = h ? "(_Float16)" + kref : kref;
    o << "  const " << t << " v" << i << " = ";
    switch (in.op) {
      case Op::Load: o << "x" << in.operand; break;
      case Op::Lookup: o << "wkf_lookup(" << a << ")"; break;
      case Op::AddC: o << a << " + " << k; break;
      case Op::SubC: o << a << " - " << k; break;
      case Op::RSubC: o << k << " - " << a; break;
      case Op::MulC: o << a << " * " << k; break;
      case Op::DivC: o << a << " / " << k; break;
      case Op::RDivC: o << k << " / " << a; break;
      case Op::Sqr: o << a << " * " << a; break;
      case Op::Neg: o << "-" << a; break;
      case Op::Abs:
        if (h) o << "(_Float16)__builtin_fabsf((float)" << a << ")";
        else o << "__builtin_fabsf(" << a << ")";
        break;
      case Op::Cast: o << "(" << t << ")" << a; break;
      case Op::Add: o << a << " + " << b; break;
      case Op::Sub: o << a << " - " << b; break;
      case Op::Mul: o << a << " * " << b; break;
      case Op::Div: o << a << " / " << b; break;
      case Op::Pow: {
        const bool exact = exact_op(p, i, policy);
        std::string call = exact ? std::string(h ? "" : "(float)") + "pow((double)" + a + ", (double)" + b + ")"
                                 : (h ? "powf((float)" + a + ", (float)" + b + ")" : "powf(" + a + ", " + b + ")");
        if (h && exact) o << "wkf_round_h(" << call << ")";
        else o << (h ? "(_Float16)" : "") << call;
        break;
      }
      default: {
        const bool exact = exact_op(p, i, policy);
        if (h && exact && in.op == Op::Exp && policy != MathPolicy::Exact) {
          // an interior exp on f16: correctly rounded through the f32 library with a rare f64 fallback
          o << "wkf_exp_h((float)" << a << ")";
          break;
        }
        if (h && !exact && in.op == Op::Exp) {
          // f16 result: 2^(x log2 e) on the hardware unit (relative error about 2^-21 for any f16 argument,
          // a thousand times finer than the f16 grid); the f32 library's exp would cost more than the loads.
          o << "(_Float16)__builtin_amdgcn_exp2f((float)" << a << " * 0x1.715476p+0f)";
          break;
        }
        if (h && exact && policy != MathPolicy::Exact && (in.op == Op::Sin || in.op == Op::Cos)) {
          // an interior sin / cos on f16: f64 reduction, f32 core, and the f64 core where that cannot decide
          o << (in.op == Op::Sin ? "wkf_sin_h" : "wkf_cos_h") << "((float)" << a << ")";
          break;
        }
        if (h && exact && policy != MathPolicy::Exact && in.op != Op::Sqrt) {
          // an interior transcendental on f16: the f32 library, and the library's f64 routine where that cannot decide
          const std::string f = lib_fn(in.op);
          o << "wkf_h_via_f32(" << f << "f((float)" << a << "), [&] { return wkf_round_h(" << f << "((double)" << a << ")); })";
          break;
        }
        std::string call = math_call(in.op, h ? "(float)" + a : a, exact, far_variant, h);
        // (sqrtf of an f16 value is the correctly rounded f32 root, and 24 bits are enough for the second rounding to f16
        // to be harmless: no f64 step, whatever reads the value)
        if (h && exact && in.op != Op::Sqrt) o << "wkf_round_h(" << call << ")";
        else o << (h ? "(_Float16)" : "") << call;
      }
    }
    o << ";\n";
  }
  o << "  return v" << p.result << ";\n}\n";
}

// The constant argument(s) of a call to an emitted program: the pointer `base + off` for the ordinary
// variant, a dummy int followed by the values themselves for the far variant.
std::string const_args(const Program& p, const std::string& base, int off, bool far_variant) {
  if (!far_variant) return off ? base + " + " + std::to_string(off) : base;
  std::string r = "0";
  for (size_t i = 0; i < p.consts.size(); i++) r += ", " + base + "[" + std::to_string(off + int(i)) + "]";
  return r;
}

void emit_program(std::ostringstream& o, const Program& p, const std::string& name,
                  const std::vector<DType>& operand_types, MathPolicy policy) {
  emit_program_variant(o, p, name, operand_types, policy, false);
  if (uses_trig(p, policy)) emit_program_variant(o, p, name, operand_types, policy, true);
}

void put32(std::vector<unsigned char>& b, uint32_t v) {
  unsigned char t[4];
  memcpy(t, &v, 4);
  b.insert(b.end(), t, t + 4);
}
void putf(std::vector<unsigned char>& b, float v) {
  unsigned char t[4];
  memcpy(t, &v, 4);
  b.insert(b.end(), t, t + 4);
}
void putp(std::vector<unsigned char>& b, const void* v) {
  unsigned char t[8];
  memcpy(t, &v, 8);
  b.insert(b.end(), t, t + 8);
}
void pad8(std::vector<unsigned char>& b) {
  while (b.size() % 8) b.push_back(0);
}

}  // namespace

// ===========================================================================
// map kernels
// ===========================================================================

std::string map_signature(const MapSpec& s) {
  std::ostringstream o;
  o << "map|gfx950|r" << s.rank << "|v" << s.vec << "|u" << s.unroll << (s.nontemporal ? "|nt" : "|ca") << "|in:";
  for (const auto& i : s.in) o << dtype_name(i.dtype) << (i.linear ? 'L' : 'S') << i.inner_stride << ',';
  o << "|out:" << dtype_name(s.out.dtype) << (s.out.linear ? 'L' : 'S') << s.out.inner_stride;
  o << "|m" << int(s.math) << "|" << s.prog.signature();
  if (s.table) o << "|table";
  for (size_t j = 0; j < s.more_out.size(); j++)
    o << "|out+:" << dtype_name(s.more_out[j].dtype) << (s.more_out[j].linear ? 'L' : 'S') << s.more_out[j].inner_stride << "|"
      << s.more_prog[j].signature();
  if (s.tile_dim >= 0) {
    o << "|tile" << s.tile_dim << ':';
    for (size_t k = 0; k < s.in.size(); k++) o << (s.crossed[k] ? 'x' : '-');
    if (s.tile_vec > 1) o << "|tv" << s.tile_vec;
    if (s.tile_size != 64) o << "|ts" << s.tile_size;
  }
  return o.str();
}

namespace {
// out = expr(inputs) where some inputs run along `tile_dim` and the output along the last dimension.
// The same with four elements per global access.  A thread is lane q = t % 16 of row r = t / 16: sixteen lanes cover the
// 64 elements of a tile row along the operand's unit-stride dimension, a pass covers 16 rows, four passes the tile.
// The LDS tile is [b][a] with an odd pitch in 4-byte words, so the four scalar writes of a vector read along a and
// the four scalar reads of a vector written along b are both free of bank conflicts.
std::string map_tiled_vec_source(const MapSpec& s) {
  const int N = int(s.in.size()) + 1;
  const int R = s.rank, TA = s.tile_dim, TB = s.rank - 1;
  const int NC = s.prog.consts.empty() ? 1 : int(s.prog.consts.size());
  // T x T tile; LQ lanes of four elements cover a tile row, the block's 256 lanes RP rows a pass, NP passes the tile
  const int T = s.tile_size, LQ = T / 4, RP = kMapBlock / LQ, NP = T / RP;
  std::ostringstream o;
  o << kPrelude;
  if (uses_math(s.prog, s.math)) o << kMath;
  if (uses_round_h(s.prog, s.math)) o << kRoundH;
  o << "struct Args { void* p[" << N << "]; u32 nwork; u32 shape[" << R << "]; u32 off[" << N << "]; u32 stride[" << N
    << "][" << R << "]; float c[" << NC << "]; };\n";
  std::vector<DType> types;
  for (const auto& i : s.in) types.push_back(i.dtype);
  emit_program(o, s.prog, "wkf_expr", types, s.math);
  const bool trig = uses_trig(s.prog, s.math);
  auto dt = [&](int k) { return k < N - 1 ? s.in[k].dtype : s.out.dtype; };
  auto ptr = [&](int k) {
    return std::string("((") + (k < N - 1 ? "const " : "") + ctype(dt(k)) + "*)a.p[" + std::to_string(k) + "])";
  };
  o << "extern \"C\" __global__ void __launch_bounds__(" << kMapBlock << ") WKF_ENTRY(const Args a) {\n";
  for (int k = 0; k < N - 1; k++)
    if (s.crossed[k])
      o << "  __shared__ " << ctype(dt(k)) << " tile" << k << "[" << T << "][" << T + (dtype_size(dt(k)) == 2 ? 2 : 1) << "];\n";
  o << "  const u32 q = threadIdx.x & " << LQ - 1 << "u, r = threadIdx.x / " << LQ << "u;\n";
  o << "  const u32 A = a.shape[" << TA << "], B = a.shape[" << TB << "];\n";
  o << "  const u32 tiles_a = (A + " << T - 1 << "u) / " << T << "u, tiles_b = (B + " << T - 1 << "u) / " << T << "u;\n";
  // Tiles are walked along b, each row of tiles starting one tile further on (a diagonal order): workgroups that run
  // at the same time then touch rows of the crossed operands whose distance is not a fixed multiple of 64 rows
  // (measured on an f32 [8192,8192] transposing copy: 3959 -> 4582 GB/s, with the non-temporal bits 5082).
  o << "  u32 rem = blockIdx.x;\n";
  o << "  const u32 tb_ = rem % tiles_b; rem /= tiles_b;\n";
  o << "  const u32 ta_ = rem % tiles_a; rem /= tiles_a;\n";
  o << "  const u32 b0 = ((tb_ + ta_) % tiles_b) * " << T << "u, a0 = ta_ * " << T << "u;\n";
  std::vector<int> others;
  for (int d = R - 2; d >= 0; d--)
    if (d != TA) others.push_back(d);
  for (size_t i = 0; i < others.size(); i++) {
    const int d = others[i];
    if (i + 1 < others.size()) o << "  const u32 i" << d << " = rem % a.shape[" << d << "]; rem /= a.shape[" << d << "];\n";
    else o << "  const u32 i" << d << " = rem;\n";
  }
  for (int k = 0; k < N; k++) {
    o << "  const u32 base" << k << " = a.off[" << k << "]";
    for (int d : others) o << " + i" << d << " * a.stride[" << k << "][" << d << "]";
    o << ";\n";
  }
  // phase 1: crossed inputs, a vector along tile_dim per lane (indices clamped: every load is unconditional; A and B
  // are multiples of 4, so a vector lies inside or outside as a whole)
  for (int k = 0; k < N - 1; k++) {
    if (!s.crossed[k]) continue;
    std::string vt = vtype(dt(k), 4);
    o << "  {\n    " << vt << " v[" << NP << "];\n";
    o << "    const u32 aa = min(a0 + q * 4u, A - 4u);\n";
    o << "#pragma unroll\n    for (int j = 0; j < " << NP << "; j++) {\n";
    o << "      const u32 bb = min(b0 + r + " << RP << "u * j, B - 1u);\n";
    o << "      v[j] = " << (s.nontemporal ? "__builtin_nontemporal_load(" : "*(") << "(const " << vt << "*)(" << ptr(k) << " + (base" << k
      << " + aa + bb * a.stride[" << k << "][" << TB << "])));\n    }\n";
    o << "#pragma unroll\n    for (int j = 0; j < " << NP << "; j++)\n#pragma unroll\n      for (int e = 0; e < 4; e++) tile" << k
      << "[r + " << RP << "u * j][q * 4u + e] = v[j][e];\n  }\n";
  }
  o << "  __syncthreads();\n";
  // phase 2: a vector along the last dim per lane
  o << "  const u32 bb = min(b0 + q * 4u, B - 4u);\n";
  o << "  const bool b_live = b0 + q * 4u < B;\n";
  std::string ovt = vtype(s.out.dtype, 4);
  o << "#pragma unroll\n  for (int j = 0; j < " << NP << "; j++) {\n";
  o << "    const u32 al = r + " << RP << "u * j, aa = a0 + al, ac = min(aa, A - 1u);\n";
  for (int k = 0; k < N - 1; k++) {
    if (s.crossed[k]) continue;
    if (s.in[k].inner_stride == 1)
      o << "    const " << vtype(dt(k), 4) << " s" << k << " = " << (s.nontemporal ? "__builtin_nontemporal_load(" : "*(") << "(const " << vtype(dt(k), 4)
        << "*)(" << ptr(k) << " + (base" << k << " + ac * a.stride[" << k << "][" << TA << "] + bb)));\n";
    else
      o << "    const " << ctype(dt(k)) << " s" << k << " = " << ptr(k) << "[base" << k << " + ac * a.stride[" << k << "][" << TA << "]];\n";
  }
  o << "    " << ovt << " ov;\n";
  for (int e = 0; e < 4; e++) {
    std::ostringstream call;
    for (int k = 0; k < N - 1; k++) {
      if (s.crossed[k]) call << "tile" << k << "[q * 4u + " << e << "][al], ";
      else if (s.in[k].inner_stride == 1) call << "s" << k << "[" << e << "], ";
      else call << "s" << k << ", ";
    }
    o << "    {\n";
    if (trig) o << "      bool far = false;\n";
    o << "      " << ctype(s.out.dtype) << " v = wkf_expr(" << call.str() << "a.c" << (trig ? ", far" : "") << ");\n";
    if (trig) o << "      if (__builtin_expect(far, 0)) v = wkf_expr_far(" << call.str() << const_args(s.prog, "a.c", 0, true) << ");\n";
    o << "      ov[" << e << "] = v;\n    }\n";
  }
  o << "    if (b_live && aa < A) ";
  if (s.nontemporal) o << "__builtin_nontemporal_store(ov, (" << ovt << "*)(" << ptr(N - 1) << " + (base" << N - 1 << " + aa * a.stride[" << N - 1 << "][" << TA << "] + bb)));\n";
  else o << "*(" << ovt << "*)(" << ptr(N - 1) << " + (base" << N - 1 << " + aa * a.stride[" << N - 1 << "][" << TA << "] + bb)) = ov;\n";
  o << "  }\n}\n";
  return o.str();
}

std::string map_tiled_source(const MapSpec& s) {
  if (s.tile_vec == 4) return map_tiled_vec_source(s);
  const int N = int(s.in.size()) + 1;
  const int R = s.rank, TA = s.tile_dim, TB = s.rank - 1;
  const int NC = s.prog.consts.empty() ? 1 : int(s.prog.consts.size());
  const int PER = kMapTile * kMapTile / kMapBlock;  // tile rows per thread
  std::ostringstream o;
  o << kPrelude;
  if (uses_math(s.prog, s.math)) o << kMath;
  if (uses_round_h(s.prog, s.math)) o << kRoundH;
  o << "struct Args { void* p[" << N << "]; u32 nwork; u32 shape[" << R << "]; u32 off[" << N << "]; u32 stride[" << N
    << "][" << R << "]; float c[" << NC << "]; };\n";
  std::vector<DType> types;
  for (const auto& i : s.in) types.push_back(i.dtype);
  emit_program(o, s.prog, "wkf_expr", types, s.math);
  const bool trig = uses_trig(s.prog, s.math);
  auto dt = [&](int k) { return k < N - 1 ? s.in[k].dtype : s.out.dtype; };
  auto ptr = [&](int k) {
    return std::string("((") + (k < N - 1 ? "const " : "") + ctype(dt(k)) + "*)a.p[" + std::to_string(k) + "])";
  };
  o << "extern \"C\" __global__ void __launch_bounds__(" << kMapBlock << ") WKF_ENTRY(const Args a) {\n";
  for (int k = 0; k < N - 1; k++)
    if (s.crossed[k])  // the padding keeps both the row-wise writes and the column-wise reads free of bank conflicts
      o << "  __shared__ " << ctype(dt(k)) << " tile" << k << "[" << kMapTile << "][" << kMapTile + (dtype_size(dt(k)) == 2 ? 2 : 1) << "];\n";
  o << "  const u32 tx = threadIdx.x & 63u, ty = threadIdx.x >> 6;\n";
  o << "  const u32 A = a.shape[" << TA << "], B = a.shape[" << TB << "];\n";
  o << "  const u32 tiles_a = (A + 63u) / 64u, tiles_b = (B + 63u) / 64u;\n";
  // Tiles are walked along b, each row of tiles starting one tile further on (a diagonal order): workgroups that run
  // at the same time then touch rows of the crossed operands whose distance is not a fixed multiple of 64 rows
  // (measured on an f32 [8192,8192] transposing copy: 3959 -> 4582 GB/s, with the non-temporal bits 5082).
  o << "  u32 rem = blockIdx.x;\n";
  o << "  const u32 tb_ = rem % tiles_b; rem /= tiles_b;\n";
  o << "  const u32 ta_ = rem % tiles_a; rem /= tiles_a;\n";
  o << "  const u32 b0 = ((tb_ + ta_) % tiles_b) * 64u, a0 = ta_ * 64u;\n";
  std::vector<int> others;
  for (int d = R - 2; d >= 0; d--)
    if (d != TA) others.push_back(d);
  for (size_t i = 0; i < others.size(); i++) {
    const int d = others[i];
    if (i + 1 < others.size()) o << "  const u32 i" << d << " = rem % a.shape[" << d << "]; rem /= a.shape[" << d << "];\n";
    else o << "  const u32 i" << d << " = rem;\n";
  }
  for (int k = 0; k < N; k++) {
    o << "  const u32 base" << k << " = a.off[" << k << "]";
    for (int d : others) o << " + i" << d << " * a.stride[" << k << "][" << d << "]";
    o << ";\n";
  }
  // phase 1: crossed inputs, lanes along tile_dim (indices clamped so that every load is unconditional)
  for (int k = 0; k < N - 1; k++) {
    if (!s.crossed[k]) continue;
    o << "  {\n    " << ctype(dt(k)) << " r[" << PER << "];\n";
    o << "    const u32 aa = min(a0 + tx, A - 1u);\n";
    o << "#pragma unroll\n    for (int j = 0; j < " << PER << "; j++) {\n";
    o << "      const u32 bb = min(b0 + ty * " << PER << "u + j, B - 1u);\n";
    o << "      r[j] = " << ptr(k) << "[base" << k << " + aa * a.stride[" << k << "][" << TA << "] + bb * a.stride[" << k << "]["
      << TB << "]];\n    }\n";
    o << "#pragma unroll\n    for (int j = 0; j < " << PER << "; j++) tile" << k << "[ty * " << PER << "u + j][tx] = r[j];\n  }\n";
  }
  o << "  __syncthreads();\n";
  // phase 2: lanes along the last dim
  o << "  const u32 bb = min(b0 + tx, B - 1u);\n";
  o << "  const bool b_live = b0 + tx < B;\n";
  for (int k = 0; k < N - 1; k++) {
    if (s.crossed[k]) continue;
    o << "  " << ctype(dt(k)) << " s" << k << "[" << PER << "];\n";
    o << "#pragma unroll\n  for (int j = 0; j < " << PER << "; j++) {\n";
    o << "    const u32 aa = min(a0 + ty * " << PER << "u + j, A - 1u);\n";
    o << "    s" << k << "[j] = " << ptr(k) << "[base" << k << " + aa * a.stride[" << k << "][" << TA << "] + bb * a.stride[" << k
      << "][" << TB << "]];\n  }\n";
  }
  o << "#pragma unroll\n  for (int j = 0; j < " << PER << "; j++) {\n";
  o << "    const u32 aa = a0 + ty * " << PER << "u + j;\n";
  std::ostringstream call;
  for (int k = 0; k < N - 1; k++) {
    if (s.crossed[k]) call << "tile" << k << "[tx][ty * " << PER << "u + j], ";
    else call << "s" << k << "[j], ";
  }
  if (trig) o << "    bool far = false;\n";
  o << "    " << ctype(s.out.dtype) << " v = wkf_expr(" << call.str() << "a.c" << (trig ? ", far" : "") << ");\n";
  if (trig) o << "    if (__builtin_expect(far, 0)) v = wkf_expr_far(" << call.str() << const_args(s.prog, "a.c", 0, true) << ");\n";
  o << "    if (b_live && aa < A) " << ptr(N - 1) << "[base" << N - 1 << " + aa * a.stride[" << N - 1 << "][" << TA
    << "] + bb * a.stride[" << N - 1 << "][" << TB << "]] = v;\n";
  o << "  }\n}\n";
  return o.str();
}
}  // namespace

std::string map_source(const MapSpec& s) {
  if (s.tile_dim >= 0) return map_tiled_source(s);
  const int NI = int(s.in.size());
  const int NO = 1 + int(s.more_out.size());
  const int N = NI + NO;  // operands: inputs, then outputs
  const int R = s.rank, V = s.vec, U = s.unroll;
  std::vector<const Program*> progs = {&s.prog};
  std::vector<const MapOperandSpec*> outs = {&s.out};
  for (int j = 1; j < NO; j++) {
    progs.push_back(&s.more_prog[j - 1]);
    outs.push_back(&s.more_out[j - 1]);
  }
  std::vector<int> coff;  // where each program's constants start in the argument block
  int NC = 0;
  for (const Program* p : progs) {
    coff.push_back(NC);
    NC += int(p->consts.size());
  }
  NC = std::max(1, NC);
  std::ostringstream o;
  o << kPrelude;
  bool any_math = false, any_trig = false;
  std::vector<bool> trig;
  for (const Program* p : progs) {
    any_math |= uses_math(*p, s.math);
    trig.push_back(uses_trig(*p, s.math));
    any_trig |= trig.back();
  }
  if (any_math) o << kMath;
  {
    bool any_round_h = false;
    for (const Program* p : progs) any_round_h |= uses_round_h(*p, s.math);
    if (any_round_h) o << kRoundH;
  }
  o << "struct Args { void* p[" << N << "]; u32 nwork; u32 shape[" << R << "]; u32 off[" << N << "]; u32 stride[" << N
    << "][" << R << "]; float c[" << NC << "];" << (s.table ? " const unsigned short* table;" : "") << " };\n";
  // threads per block; a kernel with a table runs 1024 lanes per compute unit around its 128 KiB of LDS
  const int B = s.table ? kMapTableBlock : kMapBlock;
  if (s.table)
    o << "__shared__ __attribute__((aligned(16))) unsigned short wkf_lut[65536];\n"
         "static __device__ __forceinline__ _Float16 wkf_lookup(_Float16 x) {\n"
         "  return __builtin_bit_cast(_Float16, wkf_lut[__builtin_bit_cast(unsigned short, x)]);\n}\n";
  std::vector<DType> types;
  for (const auto& i : s.in) types.push_back(i.dtype);
  auto fn = [&](int q) { return q == 0 ? std::string("wkf_expr") : "wkf_expr" + std::to_string(q); };
  for (int q = 0; q < NO; q++) emit_program(o, *progs[q], fn(q), types, s.math);

  bool need_unravel = false;
  for (const auto& i : s.in) need_unravel |= !i.linear;
  for (const MapOperandSpec* op : outs) need_unravel |= !op->linear;

  auto operand = [&](int k) -> const MapOperandSpec& { return k < NI ? s.in[k] : *outs[k - NI]; };
  auto index_expr = [&](int k, int j) {
    const MapOperandSpec& op = operand(k);
    std::ostringstream e;
    std::string w = "w" + std::to_string(j);
    if (op.linear) {
      e << "a.off[" << k << "] + " << w << " * " << V << "u";
      return e.str();
    }
    e << "a.off[" << k << "]";
    for (int d = 0; d < R - 1; d++) e << " + i" << d << "_" << j << " * a.stride[" << k << "][" << d << "]";
    if (op.inner_stride == 1) e << " + i" << R - 1 << "_" << j << " * " << V << "u";
    else if (op.inner_stride < 0) e << " + i" << R - 1 << "_" << j << " * a.stride[" << k << "][" << R - 1 << "]";
    return e.str();
  };
  // A vector operand whose inner stride is 0 is one scalar broadcast to every lane of the work item.
  auto is_vec_load = [&](int k) { return V > 1 && (operand(k).linear || operand(k).inner_stride == 1); };

  auto emit_index = [&](int j, const char* ind) {
    o << ind << "const u32 w" << j << " = w_first + " << j * B << "u;\n";
    if (need_unravel) {
      o << ind << "u32 rem" << j << " = w" << j << ";\n";
      for (int d = R - 1; d > 0; d--) {
        o << ind << "const u32 i" << d << "_" << j << " = rem" << j << " % a.shape[" << d << "]; rem" << j
          << " /= a.shape[" << d << "];\n";
      }
      o << ind << "const u32 i0_" << j << " = rem" << j << ";\n";
    }
  };
  auto emit_loads = [&](int j, const char* ind) {
    for (int k = 0; k < NI; k++) {
      const MapOperandSpec& op = s.in[k];
      std::string ptr = std::string("((const ") + ctype(op.dtype) + "*)a.p[" + std::to_string(k) + "])";
      if (is_vec_load(k)) {
        std::string vt = vtype(op.dtype, V);
        o << ind << "const " << vt << " r" << k << "_" << j << " = ";
        if (s.nontemporal && op.linear)
          o << "__builtin_nontemporal_load((const " << vt << "*)(" << ptr << " + (" << index_expr(k, j) << ")));\n";
        else
          o << "*(const " << vt << "*)(" << ptr << " + (" << index_expr(k, j) << "));\n";
      } else {
        o << ind << "const " << ctype(op.dtype) << " r" << k << "_" << j << " = " << ptr << "[" << index_expr(k, j)
          << "];\n";
      }
    }
  };
  // value name of output q, work item j
  auto oname = [&](int q, int j) { return "o" + std::to_string(j) + (q ? "_" + std::to_string(q) : ""); };
  auto emit_compute = [&](int j, const char* ind, bool far_variant) {
    for (int q = 0; q < NO; q++) {
      if (far_variant && !trig[q]) continue;
      for (int e = 0; e < V; e++) {
        o << ind << oname(q, j);
        if (V > 1) o << "[" << e << "]";
        o << " = " << fn(q) << (far_variant ? "_far" : "") << "(";
        for (int k = 0; k < NI; k++) {
          o << "r" << k << "_" << j;
          if (is_vec_load(k)) o << "[" << e << "]";
          o << ", ";
        }
        o << const_args(*progs[q], "a.c", coff[q], far_variant) << (trig[q] && !far_variant ? ", far" : "") << ");\n";
      }
    }
  };
  auto emit_store = [&](int j, const char* ind) {
    for (int q = 0; q < NO; q++) {
      const MapOperandSpec& op = *outs[q];
      const std::string ot = vtype(op.dtype, V);
      const std::string optr = std::string("((") + ctype(op.dtype) + "*)a.p[" + std::to_string(NI + q) + "])";
      if (V > 1) {
        if (s.nontemporal && op.linear)
          o << ind << "__builtin_nontemporal_store(" << oname(q, j) << ", (" << ot << "*)(" << optr << " + (" << index_expr(NI + q, j)
            << ")));\n";
        else
          o << ind << "*(" << ot << "*)(" << optr << " + (" << index_expr(NI + q, j) << ")) = " << oname(q, j) << ";\n";
      } else {
        o << ind << optr << "[" << index_expr(NI + q, j) << "] = " << oname(q, j) << ";\n";
      }
    }
  };
  // loads -> fused expression on every element -> (rarely) redo through the far variant -> stores
  auto emit_batch = [&](int j0, int j1, const std::string& ind) {
    for (int j = j0; j < j1; j++) emit_loads(j, ind.c_str());
    for (int j = j0; j < j1; j++)
      for (int q = 0; q < NO; q++) o << ind << vtype(outs[q]->dtype, V) << " " << oname(q, j) << ";\n";
    if (any_trig) o << ind << "bool far = false;\n";
    for (int j = j0; j < j1; j++) emit_compute(j, ind.c_str(), false);
    if (any_trig) {
      o << ind << "if (__builtin_expect(far, 0)) {\n";
      for (int j = j0; j < j1; j++) emit_compute(j, (ind + "  ").c_str(), true);
      o << ind << "}\n";
    }
    for (int j = j0; j < j1; j++) emit_store(j, ind.c_str());
  };

  o << "extern \"C\" __global__ void __launch_bounds__(" << B << ") WKF_ENTRY(const Args a) {\n";
  if (s.table) {
    // the table goes to the LDS once; the block then walks chunks blockIdx.x, blockIdx.x + gridDim.x, ...
    o << "  typedef u32 wkf_u4 __attribute__((ext_vector_type(4)));\n"
         "#pragma unroll\n"
         "  for (int i = 0; i < " << 65536 * 2 / 16 / B << "; i++) ((wkf_u4*)wkf_lut)[threadIdx.x + i * " << B << "u] = ((const wkf_u4*)a.table)[threadIdx.x + i * " << B << "u];\n"
         "  __syncthreads();\n";
    o << "  const u32 nchunk = a.nwork / " << B * U << "u + (a.nwork % " << B * U << "u != 0u);\n";
    o << "  for (u32 chunk = blockIdx.x; chunk < nchunk; chunk += gridDim.x) {\n";
    o << "  const u32 w_block = chunk * " << B * U << "u;\n";
  } else {
    o << "  const u32 w_block = blockIdx.x * " << B * U << "u;\n";
  }
  o << "  const u32 w_first = w_block + threadIdx.x;\n";
  if (s.table) o << "  if (a.nwork - w_block >= " << B * U << "u) {\n";
  else o << "  if (w_block + " << B * U << "u <= a.nwork) {\n";
  // Full block: every load is issued before the first use so that U independent
  // 16-byte requests per operand are in flight per lane.
  for (int j = 0; j < U; j++) emit_index(j, "    ");
  emit_batch(0, U, "    ");
  o << "  } else {\n";
  for (int j = 0; j < U; j++) {
    o << "    {\n";
    emit_index(j, "      ");
    o << "      if (w" << j << " < a.nwork) {\n";
    emit_batch(j, j + 1, "        ");
    o << "      }\n    }\n";
  }
  o << "  }\n";
  if (s.table) o << "  }\n";
  o << "}\n";
  return o.str();
}

std::string map_table_signature() { return "maptable|gfx950|f16|b1024|u1"; }

std::string map_table_source() {
  std::ostringstream o;
  o << kPrelude;
  // One 16-byte vector per lane and round: 16 KiB in flight per compute unit is what a grid that stays on the chip
  // streams fastest with (a plain copy of this shape: 42.8 us for 2 x 128 MiB with one vector, 46.7 with four)
  o << R"WKF(
typedef unsigned short u16;
typedef u32 wkf_u4 __attribute__((ext_vector_type(4)));
struct Args { const u16* in; u16* out; const u16* table; u32 nvec; u32 ntail; };
extern "C" __global__ void __launch_bounds__(1024) WKF_ENTRY(const Args a) {
  __shared__ __attribute__((aligned(16))) u16 lut[65536];
  const u32 t = threadIdx.x;
  const wkf_u4* const in = (const wkf_u4*)a.in;
  wkf_u4* const out = (wkf_u4*)a.out;
  const u32 step = gridDim.x * 1024u;
  u32 w = blockIdx.x * 1024u + t;
  // the first vector of the data is asked for before the table, so that it travels while the table is copied
  wkf_u4 v = w < a.nvec ? __builtin_nontemporal_load(in + w) : (wkf_u4)(0u);
#pragma unroll
  for (int i = 0; i < 8; i++) ((wkf_u4*)lut)[t + i * 1024u] = ((const wkf_u4*)a.table)[t + i * 1024u];
  __syncthreads();
  if (blockIdx.x == 0 && t < a.ntail) a.out[size_t(a.nvec) * 8u + t] = lut[a.in[size_t(a.nvec) * 8u + t]];
  while (w < a.nvec) {
    wkf_u4 r;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const u32 d = v[e];
      r[e] = u32(lut[d & 0xffffu]) | (u32(lut[d >> 16]) << 16);
    }
    const u32 w_now = w;
    w += step;
    // the next round's load goes out before this round's store
    v = w < a.nvec ? __builtin_nontemporal_load(in + w) : (wkf_u4)(0u);
    __builtin_nontemporal_store(r, out + w_now);
  }
}
)WKF";
  return o.str();
}

int program_cost(const Program& p) {
  int cost = 0;
  for (size_t i = 0; i < p.ins.size(); i++) {
    const Op op = p.ins[i].op;
    const bool interior = int(i) != p.result;
    switch (op) {
      case Op::Load: break;
      case Op::DivC: case Op::RDivC: case Op::Div: cost += 3; break;
      case Op::Sqrt: cost += 2; break;
      case Op::Pow: cost += 10; break;
      case Op::Sqr: case Op::Abs: case Op::Neg: cost += 1; break;
      default: cost += is_unary_op(op) ? (interior ? 10 : 3) : 1; break;
    }
  }
  return cost;
}

std::vector<unsigned char> map_pack_args(const MapSpec& s, const MapArgs& a) {
  const size_t N = s.in.size() + 1 + s.more_out.size();
  const size_t R = size_t(s.rank);
  if (a.ptrs.size() != N || a.shape.size() != R || a.offsets.size() != N || a.strides.size() != N)
    throw Error(WKF_ERR_INVALID_ARG, "map_pack_args: argument arity does not match the kernel");
  std::vector<unsigned char> b;
  for (void* p : a.ptrs) putp(b, p);
  put32(b, a.nwork);
  for (uint32_t v : a.shape) put32(b, v);
  for (uint32_t v : a.offsets) put32(b, v);
  for (const auto& st : a.strides) {
    if (st.size() != R) throw Error(WKF_ERR_INVALID_ARG, "map_pack_args: stride rank mismatch");
    for (uint32_t v : st) put32(b, v);
  }
  size_t nc = s.prog.consts.size();
  for (const Program& p : s.more_prog) nc += p.consts.size();
  nc = std::max<size_t>(1, nc);
  for (size_t i = 0; i < nc; i++) putf(b, i < a.consts.size() ? a.consts[i] : 0.f);
  pad8(b);
  if (s.table) {
    if (!a.table) throw Error(WKF_ERR_INVALID_ARG, "map_pack_args: the kernel takes a table");
    putp(b, const_cast<void*>(a.table));
  }
  return b;
}

// ===========================================================================
// reduce kernels
// ===========================================================================

namespace {
const char* fold_macro(ReduceOp r) {
  // The reference always calls the combine as f(new_value, merged), src/reduce.rs:183,204,254.
  switch (r) {
    case ReduceOp::Sum: return "#define WKF_FOLD(v, acc) ((v) + (acc))\n#define WKF_SEED 0.0f\n";
    case ReduceOp::Max: return "#define WKF_FOLD(v, acc) fmaxf((v), (acc))\n#define WKF_SEED (-3.40282e+38f)\n";
    case ReduceOp::Min: return "#define WKF_FOLD(v, acc) fminf((v), (acc))\n#define WKF_SEED (3.40282e+38f)\n";
    case ReduceOp::Product: return "#define WKF_FOLD(v, acc) ((v) * (acc))\n#define WKF_SEED 1.0f\n";
  }
  return "";
}
const char* const kReduceHelpers =
#include "kernels/reduce_helpers.hip.inc"
    ;
}  // namespace

std::string reduce_signature(const ReduceSpec& s) {
  std::ostringstream o;
  o << (s.shape == ReduceShape::Row ? "red_row" : "red_col") << "|gfx950|" << reduce_name(s.rop) << "|or" << s.outer_rank
    << "|v" << s.vec << "|t" << s.threads_per_row << "|b" << s.block << "|u" << s.unroll << "|w" << s.waves << "|in:";
  for (const auto& i : s.in) o << dtype_name(i.dtype) << 'a' << i.axis_stride << 'i' << i.inner_stride << ',';
  o << "|out:" << dtype_name(s.out_dtype) << "|m" << int(s.math_pre) << int(s.math_post) << "|pre:" << s.pre.signature();
  if (s.raw_out) o << "|raw";
  else o << "|fold:" << dtype_name(s.fold_dtype) << "|post:" << s.post.signature();
  return o.str();
}

std::string reduce_source(const ReduceSpec& s) {
  const int N = int(s.in.size());
  const int Ro = s.outer_rank;
  const int NCpre = int(s.pre.consts.size());
  const int NC = std::max(1, NCpre + int(s.post.consts.size()));
  const DType pre_dt = s.pre.result_dtype();
  const bool raw = s.raw_out;
  std::ostringstream o;
  o << kPrelude;
  if (uses_math(s.pre, s.math_pre) || (!raw && uses_math(s.post, s.math_post))) o << kMath;
  if (uses_round_h(s.pre, s.math_pre) || (!raw && uses_round_h(s.post, s.math_post))) o << kRoundH;
  o << fold_macro(s.rop);
  o << kReduceHelpers;
  o << "struct Args { void* p[" << N + 1 << "]; u32 nrows; u32 n; u32 nvec; u32 oshape[" << std::max(1, Ro)
    << "]; u32 off[" << N + 1 << "]; u32 ostride[" << N + 1 << "][" << std::max(1, Ro) << "]; u32 astride["
    << std::max(1, N) << "]; float c[" << NC << "]; };\n";
  std::vector<DType> types;
  for (const auto& i : s.in) types.push_back(i.dtype);
  emit_program(o, s.pre, "wkf_pre", types, s.math_pre);
  if (!raw) emit_program(o, s.post, "wkf_post", {s.fold_dtype}, s.math_post);

  auto unravel = [&](const char* row, const char* ind) {
    // i_d = index along outer dim d of output element `row`
    if (Ro == 0) return;
    o << ind << "u32 rem = " << row << ";\n";
    for (int d = Ro - 1; d > 0; d--)
      o << ind << "const u32 i" << d << " = rem % a.oshape[" << d << "]; rem /= a.oshape[" << d << "];\n";
    o << ind << "const u32 i0 = rem;\n";
  };
  auto base_expr = [&](int k) {
    std::ostringstream e;
    e << "a.off[" << k << "]";
    for (int d = 0; d < Ro; d++) e << " + i" << d << " * a.ostride[" << k << "][" << d << "]";
    return e.str();
  };
  auto ptr = [&](int k) { return std::string("((const ") + ctype(s.in[k].dtype) + "*)a.p[" + std::to_string(k) + "])"; };
  // the folded value is rounded to the tensor dtype, then `post` runs in that dtype
  // A post chain with sin / cos runs once per output, so it simply takes the far variant.
  auto store_value = [&](const std::string& acc) {
    if (raw) return acc;
    const bool post_far = uses_trig(s.post, s.math_post);
    return std::string(post_far ? "wkf_post_far((" : "wkf_post((") + ctype(s.fold_dtype) + ")" + acc + ", " +
           const_args(s.post, "a.c", NCpre, post_far) + ")";
  };
  std::string out_ptr = std::string("((") + ctype(raw ? DType::F32 : s.out_dtype) + "*)a.p[" + std::to_string(N) + "])";

  if (s.shape == ReduceShape::Row) {
    const int T = s.threads_per_row, V = s.vec, U = s.unroll, B = s.block;
    const int RPB = B / T;
    o << "extern \"C\" __global__ void __launch_bounds__(" << B << ") WKF_ENTRY(const Args a) {\n";
    if (T > 64) o << "  __shared__ float wkf_partial[" << B / 64 << "];\n";
    o << "  const u32 t = threadIdx.x % " << T << "u;\n";
    o << "  const u32 row_raw = blockIdx.x * " << RPB << "u + threadIdx.x / " << T << "u;\n";
    o << "  const bool live = row_raw < a.nrows;\n";
    o << "  const u32 row = live ? row_raw : 0u;\n";  // dead lanes redo row 0 so every lane reaches the barriers
    unravel("row", "  ");
    for (int k = 0; k < N; k++) {
      o << "  const " << ctype(s.in[k].dtype) << "* q" << k << " = " << ptr(k) << " + (" << base_expr(k) << ");\n";
      if (s.in[k].axis_stride == 0) o << "  const " << ctype(s.in[k].dtype) << " s" << k << " = q" << k << "[0];\n";
    }
    o << "  float acc = WKF_SEED;\n";
    auto emit_loads = [&](int j, const char* ind) {
      for (int k = 0; k < N; k++) {
        if (s.in[k].axis_stride == 0) continue;
        std::string vt = vtype(s.in[k].dtype, V);
        o << ind << "const " << vt << " r" << k << "_" << j << " = ";
        if (V > 1) o << "__builtin_nontemporal_load((const " << vt << "*)(q" << k << " + (k + " << j * T << "u) * " << V << "u));\n";
        else o << "q" << k << "[k + " << j * T << "u];\n";
      }
    };
    const bool trig = uses_trig(s.pre, s.math_pre);
    auto emit_values = [&](int j, const char* ind, bool far_variant) {
      for (int e = 0; e < V; e++) {
        o << ind << "t" << j << "_" << e << " = wkf_pre" << (far_variant ? "_far" : "") << "(";
        for (int k = 0; k < N; k++) {
          if (s.in[k].axis_stride == 0) o << "s" << k;
          else {
            o << "r" << k << "_" << j;
            if (V > 1) o << "[" << e << "]";
          }
          o << ", ";
        }
        o << const_args(s.pre, "a.c", 0, far_variant) << (trig && !far_variant ? ", far" : "") << ");\n";
      }
    };
    // loads -> pre on every element -> (rarely) redo through the far variant -> fold
    auto emit_iteration = [&](int j1, const std::string& ind) {
      for (int j = 0; j < j1; j++) emit_loads(j, ind.c_str());
      for (int j = 0; j < j1; j++)
        for (int e = 0; e < V; e++) o << ind << ctype(pre_dt) << " t" << j << "_" << e << ";\n";
      if (trig) o << ind << "bool far = false;\n";
      for (int j = 0; j < j1; j++) emit_values(j, ind.c_str(), false);
      if (trig) {
        o << ind << "if (__builtin_expect(far, 0)) {\n";
        for (int j = 0; j < j1; j++) emit_values(j, (ind + "  ").c_str(), true);
        o << ind << "}\n";
      }
      for (int j = 0; j < j1; j++)
        for (int e = 0; e < V; e++) o << ind << "acc = WKF_FOLD((float)t" << j << "_" << e << ", acc);\n";
    };
    o << "  u32 k = t;\n";
    if (U > 1) {
      o << "  for (; k + " << (U - 1) * T << "u < a.nvec; k += " << U * T << "u) {\n";
      emit_iteration(U, "    ");
      o << "  }\n";
    }
    o << "  for (; k < a.nvec; k += " << T << "u) {\n";
    emit_iteration(1, "    ");
    o << "  }\n";
    if (T > 1) o << "  acc = wkf_lanes_fold<" << std::min(T, 64) << ">(acc);\n";
    if (T > 64) {
      const int WPR = T / 64;  // waves per row
      o << "  if ((threadIdx.x & 63u) == 0u) wkf_partial[threadIdx.x >> 6] = acc;\n";
      o << "  __syncthreads();\n";
      o << "  const u32 first_wave = (threadIdx.x / " << T << "u) * " << WPR << "u;\n";
      o << "  acc = wkf_partial[first_wave];\n";
      o << "  for (u32 w = 1; w < " << WPR << "u; w++) acc = WKF_FOLD(wkf_partial[first_wave + w], acc);\n";
    }
    o << "  if (live && t == 0u) " << out_ptr << "[" << base_expr(N) << "] = " << store_value("acc") << ";\n";
    o << "}\n";
  } else {
    // Each lane owns V neighbouring outputs of the LAST outer dim (one 16-byte load per axis step when
    // V > 1); the W waves of the block walk the axis W steps apart, U steps in flight per wave.
    const int W = s.waves, V = s.vec, U = s.unroll;
    o << "extern \"C\" __global__ void __launch_bounds__(" << 64 * W << ") WKF_ENTRY(const Args a) {\n";
    if (W > 1) o << "  __shared__ float wkf_partial[" << W << "][" << V << "][64];\n";
    o << "  const u32 lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;\n";
    if (Ro == 0) {
      o << "  const bool live = lane == 0u && blockIdx.x == 0u;\n";
    } else {
      o << "  const u32 ntile = (a.oshape[" << Ro - 1 << "] + " << 64 * V - 1 << "u) / " << 64 * V << "u;\n";
      o << "  const u32 col = ((blockIdx.x % ntile) * 64u + lane) * " << V << "u;\n";
      o << "  const bool live = col < a.oshape[" << Ro - 1 << "];\n";
      o << "  const u32 i" << Ro - 1 << " = live ? col : 0u;\n";
      if (Ro > 1) {
        o << "  u32 rem = blockIdx.x / ntile;\n";
        for (int d = Ro - 2; d > 0; d--)
          o << "  const u32 i" << d << " = rem % a.oshape[" << d << "]; rem /= a.oshape[" << d << "];\n";
        o << "  const u32 i0 = rem;\n";
      }
    }
    for (int k = 0; k < N; k++)
      o << "  const " << ctype(s.in[k].dtype) << "* q" << k << " = " << ptr(k) << " + (" << base_expr(k) << ");\n";
    o << "  float acc[" << V << "];\n";
    o << "  for (int e = 0; e < " << V << "; e++) acc[e] = WKF_SEED;\n";
    const bool trig = uses_trig(s.pre, s.math_pre);
    auto wide = [&](int k) { return V > 1 && s.in[k].inner_stride == 1; };
    auto emit_step = [&](int j1, const std::string& ind) {
      for (int j = 0; j < j1; j++)
        for (int k = 0; k < N; k++) {
          std::string vt = wide(k) ? vtype(s.in[k].dtype, V) : ctype(s.in[k].dtype);
          std::string at = "q" + std::to_string(k) + " + (k + " + std::to_string(j * W) + "u) * a.astride[" + std::to_string(k) + "]";
          o << ind << "const " << vt << " r" << k << "_" << j << " = ";
          if (wide(k)) o << "__builtin_nontemporal_load((const " << vt << "*)(" << at << "));\n";
          else o << "*(" << at << ");\n";
        }
      for (int j = 0; j < j1; j++)
        for (int e = 0; e < V; e++) o << ind << ctype(pre_dt) << " t" << j << "_" << e << ";\n";
      if (trig) o << ind << "bool far = false;\n";
      auto values = [&](bool far_variant, const std::string& ind2) {
        for (int j = 0; j < j1; j++)
          for (int e = 0; e < V; e++) {
            o << ind2 << "t" << j << "_" << e << " = wkf_pre" << (far_variant ? "_far" : "") << "(";
            for (int k = 0; k < N; k++) {
              o << "r" << k << "_" << j;
              if (wide(k)) o << "[" << e << "]";
              o << ", ";
            }
            o << const_args(s.pre, "a.c", 0, far_variant) << (trig && !far_variant ? ", far" : "") << ");\n";
          }
      };
      values(false, ind);
      if (trig) {
        o << ind << "if (__builtin_expect(far, 0)) {\n";
        values(true, ind + "  ");
        o << ind << "}\n";
      }
      for (int j = 0; j < j1; j++)
        for (int e = 0; e < V; e++) o << ind << "acc[" << e << "] = WKF_FOLD((float)t" << j << "_" << e << ", acc[" << e << "]);\n";
    };
    o << "  u32 k = wave;\n";
    if (U > 1) {
      o << "  for (; k + " << (U - 1) * W << "u < a.n; k += " << U * W << "u) {\n";
      emit_step(U, "    ");
      o << "  }\n";
    }
    o << "  for (; k < a.n; k += " << W << "u) {\n";
    emit_step(1, "    ");
    o << "  }\n";
    auto emit_store = [&](const std::string& ind) {
      if (V == 1) {
        o << ind << "if (live) " << out_ptr << "[" << base_expr(N) << "] = " << store_value("acc[0]") << ";\n";
        return;
      }
      const DType odt = raw ? DType::F32 : s.out_dtype;
      o << ind << "if (live) {\n";
      o << ind << "  " << vtype(odt, V) << " ov;\n";
      for (int e = 0; e < V; e++) o << ind << "  ov[" << e << "] = " << store_value("acc[" + std::to_string(e) + "]") << ";\n";
      o << ind << "  *(" << vtype(odt, V) << "*)(" << out_ptr << " + (" << base_expr(N) << ")) = ov;\n";
      o << ind << "}\n";
    };
    if (W > 1) {
      o << "  for (int e = 0; e < " << V << "; e++) wkf_partial[wave][e][lane] = acc[e];\n  __syncthreads();\n";
      o << "  if (wave == 0u) {\n";
      o << "    for (u32 w = 1; w < " << W << "u; w++)\n";
      o << "      for (int e = 0; e < " << V << "; e++) acc[e] = WKF_FOLD(wkf_partial[w][e][lane], acc[e]);\n";
      emit_store("    ");
      o << "  }\n";
    } else {
      emit_store("  ");
    }
    o << "}\n";
  }
  return o.str();
}

std::vector<unsigned char> reduce_pack_args(const ReduceSpec& s, const ReduceArgs& a) {
  const size_t N = s.in.size();
  const size_t Ro = size_t(s.outer_rank);
  if (a.ptrs.size() != N + 1 || a.oshape.size() != Ro || a.offsets.size() != N + 1 || a.ostrides.size() != N + 1 ||
      a.astrides.size() != N)
    throw Error(WKF_ERR_INVALID_ARG, "reduce_pack_args: argument arity does not match the kernel");
  std::vector<unsigned char> b;
  for (void* p : a.ptrs) putp(b, p);
  put32(b, a.nrows);
  put32(b, a.n);
  put32(b, s.shape == ReduceShape::Row ? a.n / uint32_t(s.vec) : a.n);
  for (size_t d = 0; d < std::max<size_t>(1, Ro); d++) put32(b, d < Ro ? a.oshape[d] : 1);
  for (uint32_t v : a.offsets) put32(b, v);
  for (const auto& st : a.ostrides) {
    if (st.size() != Ro) throw Error(WKF_ERR_INVALID_ARG, "reduce_pack_args: stride rank mismatch");
    for (size_t d = 0; d < std::max<size_t>(1, Ro); d++) put32(b, d < Ro ? st[d] : 0);
  }
  for (size_t k = 0; k < std::max<size_t>(1, N); k++) put32(b, k < N ? a.astrides[k] : 0);
  size_t nc = std::max<size_t>(1, s.pre.consts.size() + s.post.consts.size());
  for (size_t i = 0; i < nc; i++) putf(b, i < a.consts.size() ? a.consts[i] : 0.f);
  pad8(b);
  return b;
}

}  // namespace wkf

// ===========================================================================
// row kernels
// ===========================================================================
namespace wkf {
namespace {
const char* const kRowHelpers =
#include "kernels/row_helpers.hip.inc"
    ;
const char* fold_text(ReduceOp r) {
  switch (r) {
    case ReduceOp::Sum: return "v + a";
    case ReduceOp::Max: return "fmaxf(v, a)";
    case ReduceOp::Min: return "fminf(v, a)";
    case ReduceOp::Product: return "v * a";
  }
  return "";
}
const char* seed_text(ReduceOp r) {
  switch (r) {
    case ReduceOp::Sum: return "0.0f";
    case ReduceOp::Max: return "-3.40282e+38f";
    case ReduceOp::Min: return "3.40282e+38f";
    case ReduceOp::Product: return "1.0f";
  }
  return "";
}
}  // namespace

std::string row_signature(const RowSpec& s) {
  std::ostringstream o;
  o << "row|gfx950|or" << s.outer_rank << "|v" << s.vec << "|t" << s.threads_per_row << "|b" << s.block << "|nv"
    << s.vectors_per_lane << "|x" << int(s.exact_math) << "|in:";
  for (const auto& i : s.in) o << dtype_name(i.dtype) << 'a' << i.axis_stride << ',';
  o << "|out:" << dtype_name(s.out_dtype);
  for (const auto& st : s.stages) o << "|" << reduce_name(st.rop) << "{" << st.pre.signature() << "}{" << st.post.signature() << "}";
  if (s.store_scalars) o << "|scalars";
  else o << "|final{" << s.final.signature() << "}";
  if (s.ragged) o << "|ragged";
  if (s.streamed) o << "|streamed";
  if (s.online_max_sum) o << "|online";
  if (s.split) o << "|split" << s.split_phase;
  if (s.team) o << "|team";
  if (s.team && s.team_mute) o << "|mute";
  return o.str();
}

std::string row_source(const RowSpec& s) {
  const int K = int(s.in.size()), S = int(s.stages.size());
  const int Ro = s.outer_rank, T = s.threads_per_row, V = s.vec, NV = s.vectors_per_lane, B = s.block;
  const int RPB = B / T;
  const MathPolicy fold_policy = s.exact_math ? MathPolicy::Exact : MathPolicy::Folded;
  // Everything a row kernel stores is combined with a fold result, so it is in the reduction
  // tolerance class (1e-5 relative) as a whole: the f32 library is used throughout.
  // A stored reduction (no `final`) finishes like any reduce kernel does.
  const MathPolicy store_policy = s.store_scalars ? (s.exact_math ? MathPolicy::Exact : MathPolicy::Stored) : fold_policy;
  const int NOUT = s.store_scalars ? int(s.stages.size()) : 1;
  int nc = 0;
  std::vector<int> pre_off, post_off;
  for (const auto& st : s.stages) {
    pre_off.push_back(nc);
    nc += int(st.pre.consts.size());
    post_off.push_back(nc);
    nc += int(st.post.consts.size());
  }
  const int final_off = nc;
  if (!s.store_scalars) nc += int(s.final.consts.size());
  std::ostringstream o;
  o << kPrelude;
  bool math = !s.store_scalars && uses_math(s.final, store_policy);
  for (const auto& st : s.stages) math |= uses_math(st.pre, fold_policy) || uses_math(st.post, store_policy);
  if (math) o << kMath;
  {
    bool round_h = !s.store_scalars && uses_round_h(s.final, store_policy);
    for (const auto& st : s.stages) round_h |= uses_round_h(st.pre, fold_policy) || uses_round_h(st.post, store_policy);
    if (round_h) o << kRoundH;
  }
  o << kRowHelpers;
  o << "struct Args { void* p[" << K + NOUT + (s.split ? 1 : 0) + (s.team ? 2 : 0) << "]; u32 nrows; " << (s.ragged || s.streamed || s.team ? "u32 nvec; " : "")
    << (s.split ? "u32 parts; u32 chunk; " : "") << (s.team ? "u32 parts; u32 spin; " : "")
    << "u32 oshape[" << std::max(1, Ro) << "]; u32 off[" << K + NOUT
    << "]; u32 ostride[" << K + NOUT << "][" << std::max(1, Ro) << "]; float c[" << std::max(1, nc) << "]; };\n";
  // operand types as every program sees them: the K full operands, then one scalar per earlier stage
  std::vector<DType> types;
  for (const auto& i : s.in) types.push_back(i.dtype);
  for (int k = 0; k < S; k++) {
    std::vector<DType> tk = types;
    emit_program(o, s.stages[k].pre, "wkf_pre" + std::to_string(k), tk, fold_policy);
    emit_program(o, s.stages[k].post, "wkf_post" + std::to_string(k), {s.stages[k].pre.result_dtype()}, store_policy);
    types.push_back(s.stages[k].post.result_dtype());
  }
  if (!s.store_scalars) emit_program(o, s.final, "wkf_final", types, store_policy);

  if (s.team) {
    // ---- rows longer than the registers of a block, held in the registers of a TEAM of blocks ----
    // Block b works on part b % parts of rows b / parts, b / parts + teams, ...: its share of the row (NV vectors
    // per lane and operand) comes into registers once and stays there.  Every stage is folded inside the block,
    // lane 192 puts the block's value into slot [stage][row][part] (64 bits: the value and a "written" mark, one
    // atomic store), the lanes of wave 3 read the slots of all parts, waiting until each is written, fold them and
    // hand the row's value to the other waves through the LDS.  The NEXT row's loads are issued before this row
    // is folded and travel meanwhile (memory operations of a wave return in order, so wave 3 sees a slot only
    // after its own share of those loads has landed; a wave that held no data would see it sooner, but a quarter
    // fewer registers per round cost more than that wait: 155 us against 117 for softmax over [256, 262144]).
    // All blocks of a team are resident together: blocks start in the order of their index, a team's blocks are
    // neighbours, and the host sizes the grid for four blocks per compute unit, which the launch bounds
    // guarantee; even a chip that held fewer would hold whole teams first, and those run to their end without
    // anyone else.  So the wait ends; it is bounded all the same (a.spin polls per lane over the whole kernel),
    // and a lane that gives up counts itself in *gave_up, which the host reads before it hands any result out.
    // A slot is written once and never reused.  Softmax's max / sum pair crosses in one exchange: the sums
    // travel relative to their part's maximum and are rescaled to the row's.  (Starting every other team half a
    // row late, so that one half moves data while the other waits, only added the delay: 117 -> 122-126 us.)
    const int TD = 256;  // data lanes
    const int XL = 192;  // first lane of the wave that also talks to the other blocks
    const int NW = TD / 64;
    if (T != TD || B != 256 || s.store_scalars || S < 1) throw Error(WKF_ERR_INVALID_ARG, "row_source: team kernels are blocks of 256 lanes with a result row");
    o << "typedef unsigned long long u64;\n";
    o << "static __device__ __forceinline__ void wkf_team_put(u64* slot, float v) {\n"
         "  __hip_atomic_store(slot, 0x100000000ull | (u64)__builtin_bit_cast(u32, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);\n}\n";
    // two slots a poll (the loads travel together); a stage with one value passes its slot twice
    o << "static __device__ __forceinline__ void wkf_team_get(u64* slot_a, u64* slot_b, float& va, float& vb, u32& polls_left, u64* gave_up) {\n"
         "  for (;;) {\n"
         "    const u64 wa = __hip_atomic_load(slot_a, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);\n"
         "    const u64 wb = __hip_atomic_load(slot_b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);\n"
         "    va = __builtin_bit_cast(float, (u32)wa);\n"
         "    vb = __builtin_bit_cast(float, (u32)wb);\n"
         "    if ((wa >> 32) != 0ull && (wb >> 32) != 0ull) return;\n"
         "    if (polls_left == 0u) {\n"
         "      __hip_atomic_fetch_add(gave_up, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);\n"
         "      return;\n"
         "    }\n"
         "    polls_left--;\n"
         "    __builtin_amdgcn_s_sleep(2);\n"
         "  }\n}\n";
    // every sync point of a row has LDS words of its own: a word is written again only one row later, with at
    // least one barrier between any wave's read of it and that write
    int nsync = 0;
    for (int k = 0; k < S; k++) nsync += 2;
    o << "extern \"C\" __global__ void __launch_bounds__(256, 4) WKF_ENTRY(const Args a) {\n";
    o << "  __shared__ float wkf_lds[" << nsync << "][4];\n";
    o << "  const u32 t = threadIdx.x;\n";
    o << "  const bool data_wave = __builtin_amdgcn_readfirstlane(threadIdx.x) < " << TD << "u;  // uniform over the wave\n";
    o << "  const bool talk_wave = __builtin_amdgcn_readfirstlane(threadIdx.x) >= " << XL << "u;\n";
    o << "  const u32 part = blockIdx.x % a.parts;\n";
    o << "  const u32 teams = gridDim.x / a.parts;\n";
    o << "  u64* const slots = (u64*)a.p[" << K + 1 << "];\n";
    o << "  u64* const gave_up = (u64*)a.p[" << K + 2 << "];\n";
    o << "  u32 polls_left = a.spin;\n";
    // a variant of its own for the host-side test of the give-up path: part 0 never writes its slots
    const std::string may_put = s.team_mute ? " && part != 0u" : "";
    for (int k = 0; k < S; k++) {
      const bool online = s.online_max_sum && k < 2;
      o << "  auto fold" << k << " = [](float v, float a) { return " << fold_text(online ? (k == 0 ? ReduceOp::Max : ReduceOp::Sum) : s.stages[k].rop)
        << "; };\n";
    }
    auto stage_rop = [&](int k) { return s.online_max_sum && k < 2 ? (k == 0 ? ReduceOp::Max : ReduceOp::Sum) : s.stages[k].rop; };
    // the element offset of operand k's row `row`, through index variables with the suffix `sfx`
    auto emit_indices = [&](const char* ind, const char* row, const char* sfx) {
      if (Ro > 0) {
        o << ind << "u32 rem" << sfx << " = " << row << ";\n";
        for (int d = Ro - 1; d > 0; d--)
          o << ind << "const u32 i" << d << sfx << " = rem" << sfx << " % a.oshape[" << d << "]; rem" << sfx << " /= a.oshape[" << d << "];\n";
        o << ind << "const u32 i0" << sfx << " = rem" << sfx << ";\n";
      }
    };
    auto base_expr = [&](int k, const char* sfx) {
      std::ostringstream e;
      e << "a.off[" << k << "]";
      for (int d = 0; d < Ro; d++) e << " + i" << d << sfx << " * a.ostride[" << k << "][" << d << "]";
      return e.str();
    };
    // The loads of one row into the variables <x|s><dst>k_j.  They are buffer loads without a branch around them, so
    // that the compiler can count the loads in flight and wait for exactly those it needs (after a load under
    // `if` it waits for all of them): the resource ends where the row ends, or has no extent at all when there is
    // no such row or the wave holds no data (`has`), and a load past its end returns zeros without touching memory.
    auto buffer_load = [&](DType dt, int lanes, const std::string& rsrc, const std::string& off) {
      const size_t bytes = dtype_size(dt) * size_t(lanes);
      const char* fn = bytes == 16 ? "b128" : bytes == 8 ? "b64" : bytes == 4 ? "b32" : "b16";
      return "__builtin_bit_cast(" + vtype(dt, lanes) + ", __builtin_amdgcn_raw_buffer_load_" + fn + "(" + rsrc + ", " + off + ", 0, 2))";
    };
    auto emit_loads = [&](const char* ind, const char* row, const char* sfx, const char* dst, const char* has) {
      emit_indices(ind, row, sfx);
      for (int k = 0; k < K; k++) {
        const char* ct = ctype(s.in[k].dtype);
        const size_t es = dtype_size(s.in[k].dtype);
        const bool scalar = s.in[k].axis_stride == 0;
        o << ind << "const __amdgpu_buffer_rsrc_t rs" << k << sfx << " = __builtin_amdgcn_make_buffer_rsrc((void*)(((const " << ct << "*)a.p[" << k
          << "]) + (" << base_expr(k, sfx) << ")), 0, " << has << " ? " << (scalar ? std::to_string(es) + "u" : "a.nvec * " + std::to_string(es * size_t(V)) + "u")
          << " : 0u, 0x00020000);\n";
        if (scalar) {
          o << ind << "s" << dst << k << " = " << buffer_load(s.in[k].dtype, 1, "rs" + std::to_string(k) + sfx, "0u") << ";\n";
        } else {
          for (int j = 0; j < NV; j++)
            o << ind << "x" << dst << k << "_" << j << " = "
              << buffer_load(s.in[k].dtype, V, "rs" + std::to_string(k) + sfx, "j" + std::to_string(j) + " * " + std::to_string(es * size_t(V)) + "u") << ";\n";
        }
      }
    };
    auto declare = [&](const char* ind, const char* dst) {
      for (int k = 0; k < K; k++) {
        if (s.in[k].axis_stride == 0) o << ind << ctype(s.in[k].dtype) << " s" << dst << k << ";\n";
        else
          for (int j = 0; j < NV; j++) o << ind << vtype(s.in[k].dtype, V) << " x" << dst << k << "_" << j << ";\n";
      }
    };
    for (int j = 0; j < NV; j++)
      o << "  const u32 j" << j << " = (part * " << NV << "u + " << j << "u) * " << TD << "u + t; const bool ok" << j << " = data_wave && j" << j << " < a.nvec;\n";
    o << "  const u32 row0 = blockIdx.x / a.parts;\n";
    // Two register sets take turns: the loop body is written out once per set with the roles swapped (this row, the
    // next), so that no set is ever copied into the other; a copy would have to wait for the loads it copies.
    // (Three sets, loads two rows ahead and a wave 3 that holds no data and sees the slots at once, were much
    // slower: 191 us for softmax over [256, 262144] against 118.)
    const int NSET = 2;
    const char* const set_name[2] = {"a", "b"};
    for (int q = 0; q < NSET; q++) declare("  ", set_name[q]);
    o << "  {\n";
    emit_loads("    ", "min(row0, a.nrows - 1u)", "f", set_name[0], "(data_wave && row0 < a.nrows)");
    o << "  }\n";
    o << "  u32 row = row0;\n";
    o << "  for (;;) {\n";
    for (int turn = 0; turn < NSET; turn++) {
    const std::string cur = set_name[turn % NSET], far = set_name[(turn + NSET - 1) % NSET];
    o << "  {  // this row in set " << cur << ", loads into set " << far << "\n";
    o << "  {\n";
    emit_loads("    ", "min(row + teams, a.nrows - 1u)", "n", far.c_str(), "(data_wave && row + teams < a.nrows)");
    o << "  }\n";
    emit_indices("  ", "row", "");
    auto call_args = [&](int j, int e, int nscalars) {
      std::ostringstream c;
      for (int k = 0; k < K; k++) {
        if (s.in[k].axis_stride == 0) c << "s" << cur << k;
        else {
          c << "x" << cur << k << "_" << j;
          if (V > 1) c << "[" << e << "]";
        }
        c << ", ";
      }
      for (int q = 0; q < nscalars; q++) c << "r" << q << ", ";
      return c.str();
    };
    int sync = 0;
    // acc<k> over this lane's vectors, then over the block's data waves; every wave gets the value
    auto own_fold = [&](int k, const char* ind) {
      // (no branch: a vector past the end of the row came back as zeros and folds as the seed)
      const char* seed = seed_text(stage_rop(k));
      for (int j = 0; j < NV; j++)
        for (int e = 0; e < V; e++)
          o << ind << "acc" << k << " = fold" << k << "(ok" << j << " ? (float)wkf_pre" << k << "(" << call_args(j, e, k) << "a.c + " << pre_off[k] << ") : "
            << seed << ", acc" << k << ");\n";
      o << ind << "acc" << k << " = wkf_lanes_fold_with<64>(acc" << k << ", fold" << k << ");\n";
      o << ind << "if (data_wave && (t & 63u) == 0u) wkf_lds[" << sync << "][t >> 6] = acc" << k << ";\n";
      o << ind << "__syncthreads();\n";
      o << ind << "acc" << k << " = fold" << k << "(wkf_lds[" << sync << "][0], fold" << k << "(wkf_lds[" << sync << "][1], wkf_lds[" << sync << "][2]));\n";
      if (NW == 4) o << ind << "acc" << k << " = fold" << k << "(wkf_lds[" << sync << "][3], acc" << k << ");\n";
      sync++;
    };
    auto slot = [&](int k, const char* who) { return "slots + ((" + std::to_string(k) + "u * a.nrows + row) * a.parts + " + who + ")"; };
    auto post = [&](int k) {
      o << "  const " << ctype(s.stages[k].post.result_dtype()) << " r" << k << " = wkf_post" << k << "((" << ctype(s.stages[k].pre.result_dtype())
        << ")acc" << k << ", a.c + " << post_off[k] << ");\n";
    };
    for (int k = 0; k < S; k++) {
      if (s.online_max_sum && k == 0) {
        o << "  float acc0 = " << seed_text(ReduceOp::Max) << ", acc1 = " << seed_text(ReduceOp::Sum) << ";\n";
        own_fold(0, "  ");
        o << "  {\n    const " << ctype(s.stages[0].post.result_dtype()) << " r0 = wkf_post0((" << ctype(s.stages[0].pre.result_dtype())
          << ")acc0, a.c + " << post_off[0] << ");  // this part's maximum\n";
        own_fold(1, "    ");
        o << "  }\n";
        o << "  if (talk_wave) {\n";
        o << "    if (t == " << XL << "u" << may_put << ") {\n      wkf_team_put(" << slot(0, "part") << ", acc0);\n      wkf_team_put(" << slot(1, "part") << ", acc1);\n    }\n";
        o << "    float row_max = " << seed_text(ReduceOp::Max) << ", row_sum = 0.0f;\n";
        o << "    for (u32 p = t - " << XL << "u; p < a.parts; p += 64u) {\n";
        o << "      float part_max, part_sum;\n";
        o << "      wkf_team_get(" << slot(0, "p") << ", " << slot(1, "p") << ", part_max, part_sum, polls_left, gave_up);\n";
        o << "      const float m = fmaxf(part_max, row_max);\n";
        o << "      row_sum = row_sum * expf(row_max - m) + part_sum * expf(part_max - m);\n";
        o << "      row_max = m;\n";
        o << "    }\n";
        o << "    const float lane_max = row_max;\n";
        o << "    row_max = wkf_lanes_fold_with<64>(row_max, fold0);\n";
        o << "    row_sum = wkf_lanes_fold_with<64>(row_sum * expf(lane_max - row_max), fold1);\n";
        o << "    if (t == " << XL << "u) {\n      wkf_lds[" << sync << "][0] = row_max;\n      wkf_lds[" << sync << "][1] = row_sum;\n    }\n";
        o << "  }\n";
        o << "  __syncthreads();\n";
        o << "  acc0 = wkf_lds[" << sync << "][0];\n  acc1 = wkf_lds[" << sync << "][1];\n";
        sync++;
        post(0);
        post(1);
        k = 1;
        continue;
      }
      o << "  float acc" << k << " = " << seed_text(s.stages[k].rop) << ";\n";
      own_fold(k, "  ");
      o << "  if (talk_wave) {\n";
      o << "    if (t == " << XL << "u" << may_put << ") wkf_team_put(" << slot(k, "part") << ", acc" << k << ");\n";
      o << "    float v = " << seed_text(s.stages[k].rop) << ";\n";
      o << "    for (u32 p = t - " << XL << "u; p < a.parts; p += 64u) {\n";
      o << "      float pa, pb;\n";
      o << "      wkf_team_get(" << slot(k, "p") << ", " << slot(k, "p") << ", pa, pb, polls_left, gave_up);\n";
      o << "      v = fold" << k << "(pa, v);\n";
      o << "    }\n";
      o << "    v = wkf_lanes_fold_with<64>(v, fold" << k << ");\n";
      o << "    if (t == " << XL << "u) wkf_lds[" << sync << "][0] = v;\n";
      o << "  }\n";
      o << "  __syncthreads();\n";
      o << "  acc" << k << " = wkf_lds[" << sync << "][0];\n";
      sync++;
      post(k);
    }
    const char* ot = ctype(s.out_dtype);
    std::string ovt = vtype(s.out_dtype, V);
    o << "  " << ot << "* qo = ((" << ot << "*)a.p[" << K << "]) + (" << base_expr(K, "") << ");\n";
    for (int j = 0; j < NV; j++) {
      o << "  if (ok" << j << ") {\n    " << ovt << " ov;\n";
      for (int e = 0; e < V; e++) {
        o << "    ov";
        if (V > 1) o << "[" << e << "]";
        o << " = wkf_final(" << call_args(j, e, S) << "a.c + " << final_off << ");\n";
      }
      o << "    __builtin_nontemporal_store(ov, (" << ovt << "*)(qo + j" << j << " * " << V << "u));\n  }\n";
    }
    o << "  }\n";
    o << "  row += teams;\n  if (row >= a.nrows) break;\n";
    }
    o << "  }\n}\n";
    return o.str();
  }
  o << "extern \"C\" __global__ void __launch_bounds__(" << B << ") WKF_ENTRY(const Args a) {\n";
  if (T > 64) o << "  __shared__ float wkf_partial[" << std::max(1, S) << "][" << B / 64 << "];\n";
  o << "  const u32 t = threadIdx.x % " << T << "u;\n";
  if (s.split) o << "  const u32 part = blockIdx.x % a.parts;\n  const u32 row_raw = blockIdx.x / a.parts;\n";
  else o << "  const u32 row_raw = blockIdx.x * " << RPB << "u + threadIdx.x / " << T << "u;\n";
  o << "  const bool live = row_raw < a.nrows;\n";
  o << "  const u32 row = live ? row_raw : 0u;\n";
  if (s.ragged) o << "  const bool last_ok = t + " << (NV - 1) * T << "u < a.nvec;  // this lane's last vector lies inside the row\n";
  if (Ro > 0) {
    o << "  u32 rem = row;\n";
    for (int d = Ro - 1; d > 0; d--) o << "  const u32 i" << d << " = rem % a.oshape[" << d << "]; rem /= a.oshape[" << d << "];\n";
    o << "  const u32 i0 = rem;\n";
  }
  auto base_expr = [&](int k) {
    std::ostringstream e;
    e << "a.off[" << k << "]";
    for (int d = 0; d < Ro; d++) e << " + i" << d << " * a.ostride[" << k << "][" << d << "]";
    return e.str();
  };
  if (s.streamed) {
    // ---- rows longer than the registers of a block: one pass over the row per stage, one more for the result ----
    const int U = NV;
    for (int k = 0; k < K; k++) {
      const char* ct = ctype(s.in[k].dtype);
      o << "  const " << ct << "* q" << k << " = ((const " << ct << "*)a.p[" << k << "]) + (" << base_expr(k) << ");\n";
      if (s.in[k].axis_stride == 0) o << "  const " << ct << " s" << k << " = q" << k << "[0];\n";
    }
    auto sargs = [&](int u, int e, int nscalars) {
      std::ostringstream c;
      for (int k = 0; k < K; k++) {
        if (s.in[k].axis_stride == 0) c << "s" << k;
        else {
          c << "x" << k << "_" << u;
          if (V > 1) c << "[" << e << "]";
        }
        c << ", ";
      }
      for (int q = 0; q < nscalars; q++) c << "r" << q << ", ";
      return c.str();
    };
    // A split kernel walks its part of the row, [part * chunk, (part + 1) * chunk); an unsplit one all of it.
    if (s.split) o << "  const u32 lo = part * a.chunk;\n  const u32 hi = min(a.nvec, lo + a.chunk);\n";
    else o << "  const u32 lo = 0u;\n  const u32 hi = a.nvec;\n";
    const std::string loop = "  for (u32 base = lo; base < hi; base += " + std::to_string(T * U) + "u) {\n";
    // `last`: the final pass streams (nothing reads the row again); earlier passes leave it in the caches
    auto emit_loads = [&](bool last) {
      for (int u = 0; u < U; u++) o << "    const u32 j" << u << " = base + t + " << u * T << "u; const bool ok" << u << " = j" << u << " < hi;\n";
      for (int k = 0; k < K; k++) {
        if (s.in[k].axis_stride == 0) continue;
        std::string vt = vtype(s.in[k].dtype, V);
        for (int u = 0; u < U; u++) {
          o << "    const " << vt << " x" << k << "_" << u << " = !ok" << u << " ? (" << vt << ")(0) : ";
          if (last) o << "__builtin_nontemporal_load((const " << vt << "*)(q" << k << " + j" << u << " * " << V << "u));\n";
          else o << "*(const " << vt << "*)(q" << k << " + j" << u << " * " << V << "u);\n";
        }
      }
    };
    const bool last_is_stage = s.store_scalars;
    auto block_fold = [&](int k) {  // acc<k> of every lane -> the row's value in every lane
      o << "  acc" << k << " = wkf_lanes_fold_with<64>(acc" << k << ", fold" << k << ");\n";
      if (T > 64) {
        o << "  if ((threadIdx.x & 63u) == 0u) wkf_partial[" << k << "][threadIdx.x >> 6] = acc" << k << ";\n";
        o << "  __syncthreads();\n";
        o << "  acc" << k << " = wkf_partial[" << k << "][0];\n";
        o << "  for (u32 w = 1; w < " << T / 64 << "u; w++) acc" << k << " = fold" << k << "(wkf_partial[" << k << "][w], acc" << k << ");\n";
      }
    };
    auto emit_post = [&](int k) {
      o << "  const " << ctype(s.stages[k].post.result_dtype()) << " r" << k << " = wkf_post" << k << "((" << ctype(s.stages[k].pre.result_dtype())
        << ")acc" << k << ", a.c + " << post_off[k] << ");\n";
    };
    for (int k = 0; k < S; k++) {
      const bool online = s.online_max_sum && k < 2;
      o << "  float acc" << k << " = " << seed_text(online ? (k == 0 ? ReduceOp::Max : ReduceOp::Sum) : s.stages[k].rop) << ";\n";
      o << "  auto fold" << k << " = [](float v, float a) { return " << fold_text(online ? (k == 0 ? ReduceOp::Max : ReduceOp::Sum) : s.stages[k].rop)
        << "; };\n";
    }
    // Split rows: stage k of part q of a row leaves its folded value in wp[(k * nrows + row) * parts + q]; the
    // kernels after it fold a row's `parts` values (one per lane) before they start.  The sums of an online pair
    // are relative to their own part's maximum and are rescaled to the row's when they are combined.
    const int first = s.split ? s.split_phase : 0;  // the first stage this kernel folds itself
    if (s.split) {
      o << "  float* const wp = (float*)a.p[" << K + NOUT << "];\n";
      auto part_at = [&](int k) { return "wp[(" + std::to_string(k) + "u * a.nrows + row) * a.parts + t]"; };
      for (int k = 0; k < first; k++) {
        if (s.online_max_sum && k == 0) {
          o << "  const float part_max = t < a.parts ? " << part_at(0) << " : acc0;\n  acc0 = part_max;\n";
          block_fold(0);
          o << "  if (t < a.parts) acc1 = " << part_at(1) << " * expf(part_max - acc0);\n";
          block_fold(1);
          emit_post(0);
          emit_post(1);
          k = 1;
          continue;
        }
        o << "  if (t < a.parts) acc" << k << " = " << part_at(k) << ";\n";
        block_fold(k);
        emit_post(k);
      }
    }
    auto leave_parts = [&](int k0, int k1) {  // a split kernel ends here: lane 0 stores what this part folded
      o << "  if (t == 0u) {\n";
      for (int k = k0; k <= k1; k++) o << "    wp[(" << k << "u * a.nrows + row) * a.parts + part] = acc" << k << ";\n";
      o << "  }\n}\n";
    };
    if (s.online_max_sum && first == 0) {
      // stages 0 and 1 in one pass: every lane keeps a running maximum m and the sum of exp(x - m) over what it
      // has seen; when m grows the sum is rescaled by exp(old m - new m).  Lanes are combined the same way.
      const char* mt = ctype(s.stages[0].post.result_dtype());
      o << loop;
      emit_loads(last_is_stage && S == 2);
      for (int u = 0; u < U; u++) {
        o << "    if (ok" << u << ") {\n";
        o << "      float cm = acc0;\n";
        for (int e = 0; e < V; e++) o << "      cm = fmaxf((float)wkf_pre0(" << sargs(u, e, 0) << "a.c + " << pre_off[0] << "), cm);\n";
        o << "      if (cm > acc0) {  // rare after the first steps of a row: exp(0) = 1 would change nothing\n        acc1 *= expf(acc0 - cm);\n        acc0 = cm;\n      }\n";
        o << "      const " << mt << " r0 = wkf_post0((" << ctype(s.stages[0].pre.result_dtype()) << ")cm, a.c + " << post_off[0] << ");\n";
        for (int e = 0; e < V; e++) o << "      acc1 += (float)wkf_pre1(" << sargs(u, e, 1) << "a.c + " << pre_off[1] << ");\n";
        o << "    }\n";
      }
      o << "  }\n";
      o << "  const float lane_max = acc0;\n";
      block_fold(0);
      o << "  acc1 *= expf(lane_max - acc0);\n";
      block_fold(1);
      if (s.split) {
        leave_parts(0, 1);
        return o.str();
      }
      emit_post(0);
      emit_post(1);
    }
    for (int k = std::max(first, s.online_max_sum ? 2 : 0); k < S; k++) {
      o << loop;
      emit_loads(last_is_stage && k == S - 1);
      for (int u = 0; u < U; u++) {
        o << "    if (ok" << u << ") {\n";
        for (int e = 0; e < V; e++)
          o << "      acc" << k << " = fold" << k << "((float)wkf_pre" << k << "(" << sargs(u, e, k) << "a.c + " << pre_off[k] << "), acc" << k << ");\n";
        o << "    }\n";
      }
      o << "  }\n";
      block_fold(k);
      if (s.split) {
        leave_parts(k, k);
        return o.str();
      }
      emit_post(k);
    }
    if (s.store_scalars) {
      o << "  if (live && t == 0u) {\n";
      for (int k = 0; k < S; k++) {
        const char* st = ctype(s.stages[k].post.result_dtype());
        o << "    ((" << st << "*)a.p[" << K + k << "])[" << base_expr(K + k) << "] = r" << k << ";\n";
      }
      o << "  }\n}\n";
      return o.str();
    }
    const char* sot = ctype(s.out_dtype);
    std::string ovt = vtype(s.out_dtype, V);
    o << "  " << sot << "* qo = ((" << sot << "*)a.p[" << K << "]) + (" << base_expr(K) << ");\n";
    o << loop;
    emit_loads(true);
    for (int u = 0; u < U; u++) {
      o << "    if (live && ok" << u << ") {\n      " << ovt << " ov;\n";
      for (int e = 0; e < V; e++) {
        o << "      ov";
        if (V > 1) o << "[" << e << "]";
        o << " = wkf_final(" << sargs(u, e, S) << "a.c + " << final_off << ");\n";
      }
      o << "      __builtin_nontemporal_store(ov, (" << ovt << "*)(qo + j" << u << " * " << V << "u));\n    }\n";
    }
    o << "  }\n}\n";
    return o.str();
  }
  // the row of every operand comes into registers once
  for (int k = 0; k < K; k++) {
    const char* ct = ctype(s.in[k].dtype);
    o << "  const " << ct << "* q" << k << " = ((const " << ct << "*)a.p[" << k << "]) + (" << base_expr(k) << ");\n";
    if (s.in[k].axis_stride == 0) {
      o << "  const " << ct << " s" << k << " = q" << k << "[0];\n";
    } else {
      std::string vt = vtype(s.in[k].dtype, V);
      for (int j = 0; j < NV; j++) {
        o << "  const " << vt << " x" << k << "_" << j << " = ";
        if (s.ragged && j == NV - 1) o << "!last_ok ? (" << vt << ")(0) : ";
        o << "__builtin_nontemporal_load((const " << vt << "*)(q" << k << " + (t + " << j * T << "u) * " << V << "u));\n";
      }
    }
  }
  auto call_args = [&](int j, int e, int nscalars) {
    std::ostringstream c;
    for (int k = 0; k < K; k++) {
      if (s.in[k].axis_stride == 0) c << "s" << k;
      else {
        c << "x" << k << "_" << j;
        if (V > 1) c << "[" << e << "]";
      }
      c << ", ";
    }
    for (int q = 0; q < nscalars; q++) c << "r" << q << ", ";
    return c.str();
  };
  for (int k = 0; k < S; k++) {
    const RowStage& st = s.stages[k];
    o << "  float acc" << k << " = " << seed_text(st.rop) << ";\n";
    o << "  auto fold" << k << " = [](float v, float a) { return " << fold_text(st.rop) << "; };\n";
    for (int j = 0; j < NV; j++) {
      const bool guard = s.ragged && j == NV - 1;
      if (guard) o << "  if (last_ok) {\n";
      for (int e = 0; e < V; e++)
        o << "  acc" << k << " = fold" << k << "((float)wkf_pre" << k << "(" << call_args(j, e, k) << "a.c + " << pre_off[k] << "), acc"
          << k << ");\n";
      if (guard) o << "  }\n";
    }
    if (T > 1) o << "  acc" << k << " = wkf_lanes_fold_with<" << std::min(T, 64) << ">(acc" << k << ", fold" << k << ");\n";
    if (T > 64) {
      const int WPR = T / 64;
      o << "  if ((threadIdx.x & 63u) == 0u) wkf_partial[" << k << "][threadIdx.x >> 6] = acc" << k << ";\n";
      o << "  __syncthreads();\n";
      o << "  {\n    const u32 first_wave = (threadIdx.x / " << T << "u) * " << WPR << "u;\n";
      o << "    acc" << k << " = wkf_partial[" << k << "][first_wave];\n";
      o << "    for (u32 w = 1; w < " << WPR << "u; w++) acc" << k << " = fold" << k << "(wkf_partial[" << k << "][first_wave + w], acc" << k
        << ");\n  }\n";
    }
    o << "  const " << ctype(st.post.result_dtype()) << " r" << k << " = wkf_post" << k << "((" << ctype(st.pre.result_dtype()) << ")acc" << k
      << ", a.c + " << post_off[k] << ");\n";
  }
  if (s.store_scalars) {
    o << "  if (live && t == 0u) {\n";
    for (int k = 0; k < S; k++) {
      const char* st = ctype(s.stages[k].post.result_dtype());
      o << "    ((" << st << "*)a.p[" << K + k << "])[" << base_expr(K + k) << "] = r" << k << ";\n";
    }
    o << "  }\n}\n";
    return o.str();
  }
  const char* ot = ctype(s.out_dtype);
  o << "  if (live) {\n";
  o << "    " << ot << "* qo = ((" << ot << "*)a.p[" << K << "]) + (" << base_expr(K) << ");\n";
  for (int j = 0; j < NV; j++) {
    std::string vt = vtype(s.out_dtype, V);
    o << "    " << vt << " o" << j << ";\n";
    for (int e = 0; e < V; e++) {
      o << "    o" << j;
      if (V > 1) o << "[" << e << "]";
      o << " = wkf_final(" << call_args(j, e, S) << "a.c + " << final_off << ");\n";
    }
    o << "    " << (s.ragged && j == NV - 1 ? "if (last_ok) " : "") << "__builtin_nontemporal_store(o" << j << ", (" << vt << "*)(qo + (t + " << j * T
      << "u) * " << V << "u));\n";
  }
  o << "  }\n}\n";
  return o.str();
}

std::vector<unsigned char> row_pack_args(const RowSpec& s, const RowArgs& a) {
  const size_t K = s.in.size(), Ro = size_t(s.outer_rank);
  const size_t NP = K + (s.store_scalars ? s.stages.size() : 1);
  if (a.ptrs.size() != NP + (s.split ? 1 : 0) + (s.team ? 2 : 0) || a.oshape.size() != Ro || a.offsets.size() != NP || a.ostrides.size() != NP)
    throw Error(WKF_ERR_INVALID_ARG, "row_pack_args: argument arity does not match the kernel");
  std::vector<unsigned char> b;
  for (void* p : a.ptrs) putp(b, p);
  put32(b, a.nrows);
  if (s.ragged || s.streamed || s.team) put32(b, a.nvec);
  if (s.split) {
    put32(b, a.parts);
    put32(b, a.chunk);
  }
  if (s.team) {
    put32(b, a.parts);
    put32(b, a.spin);
  }
  for (size_t d = 0; d < std::max<size_t>(1, Ro); d++) put32(b, d < Ro ? a.oshape[d] : 1);
  for (uint32_t v : a.offsets) put32(b, v);
  for (const auto& st : a.ostrides) {
    if (st.size() != Ro) throw Error(WKF_ERR_INVALID_ARG, "row_pack_args: stride rank mismatch");
    for (size_t d = 0; d < std::max<size_t>(1, Ro); d++) put32(b, d < Ro ? st[d] : 0);
  }
  size_t nc = s.store_scalars ? 0 : s.final.consts.size();
  for (const auto& st : s.stages) nc += st.pre.consts.size() + st.post.consts.size();
  nc = std::max<size_t>(1, nc);
  for (size_t i = 0; i < nc; i++) putf(b, i < a.consts.size() ? a.consts[i] : 0.f);
  pad8(b);
  return b;
}

}  // namespace wkf

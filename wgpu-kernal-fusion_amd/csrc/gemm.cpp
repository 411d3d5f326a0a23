// mat_mul: UntypedMatMul::run_with_query of the reference (src/matmul.rs:157-205).
#include <cstring>
#include <sstream>

#include "graph.h"

namespace wkf {

namespace {
const char* const kGemmF16 =
#include "kernels/gemm_f16.hip.inc"
    ;
const char* const kGemmF32 =
#include "kernels/gemm_f32.hip.inc"
    ;
const char* const kGemmGeneric =
#include "kernels/gemm_generic.hip.inc"
    ;
}  // namespace

GemmKind gemm_pick(DType dt, size_t m, size_t n, size_t k) {
  if (m == 0 || n == 0 || k == 0) return GemmKind::Generic;
  const bool whole = m % 256 == 0 && n % 256 == 0;
  if (dt == DType::F16 && whole && k % 64 == 0) return GemmKind::MfmaF16;
  if (dt == DType::F32 && whole && k % 32 == 0) return GemmKind::MfmaF32;
  // ragged shapes keep the MFMA kernels as long as every row of A and B starts on a 16-byte boundary
  // and the problem is worth a 256 x 256 tile; tiny or unaligned ones take the generic kernel
  const size_t chunk = dt == DType::F16 ? 8 : 4;
  if (k % chunk == 0 && n % chunk == 0 && m >= 16 && n >= 16 && m * n * k >= (size_t(1) << 18))
    return dt == DType::F16 ? GemmKind::MfmaF16Edge : GemmKind::MfmaF32Edge;
  return GemmKind::Generic;
}

std::string gemm_signature(GemmKind kind, DType dt) {
  switch (kind) {
    case GemmKind::MfmaF16: return "gemm|gfx950|f16|mfma32x32x16|256x256x64|w2x2";
    case GemmKind::MfmaF32: return "gemm|gfx950|f32|mfma32x32x2|256x256x32|w2x2";
    case GemmKind::MfmaF16Edge: return "gemm|gfx950|f16|mfma32x32x16|256x256x64|w2x2|edge";
    case GemmKind::MfmaF32Edge: return "gemm|gfx950|f32|mfma32x32x2|256x256x32|w2x2|edge";
    case GemmKind::Generic: return std::string("gemm|gfx950|") + dtype_name(dt) + "|generic|64x64x16";
  }
  return "";
}

std::string gemm_source(GemmKind kind, DType dt) {
  switch (kind) {
    case GemmKind::MfmaF16: return kGemmF16;
    case GemmKind::MfmaF32: return kGemmF32;
    case GemmKind::MfmaF16Edge: return std::string("#define WKF_EDGE 1\n") + kGemmF16;
    case GemmKind::MfmaF32Edge: return std::string("#define WKF_EDGE 1\n") + kGemmF32;
    case GemmKind::Generic:
      return std::string("#define WKF_T ") + (dt == DType::F32 ? "float" : "_Float16") + "\n" + kGemmGeneric;
  }
  return "";
}

TensorData Resolver::run_matmul(const NodeP& n) {
  // no fusion on either side (src/compute_graph/resolve.rs:138-154)
  TensorData a = resolve(n->a);
  TensorData b = resolve(n->b);
  if (a.layout.rank() != 2 || b.layout.rank() != 2) invalid("mat_mul: both operands must have rank 2");
  if (a.dtype != b.dtype) invalid("mat_mul: operand dtypes differ");
  const size_t M = a.layout.shape[0], K = a.layout.shape[1], N = b.layout.shape[1];
  if (b.layout.shape[0] != K) invalid("mat_mul: inner dimensions differ");  // src/matmul.rs:194
  // The reference kernel ignores strides and offsets (src/matmul.rs:96-103), which is only
  // right for contiguous operands; a view is copied into a dense buffer first.
  a = make_contiguous(a);
  b = make_contiguous(b);
  TensorData out = alloc({M, N}, a.dtype, false);
  if (M == 0 || N == 0) return out;
  if (M > 0xffffffffull || N > 0xffffffffull || K > 0xffffffffull) throw Error(WKF_ERR_UNSUPPORTED, "mat_mul: dimension does not fit 32 bits");

  const GemmKind kind = gemm_pick(a.dtype, M, N, K);
  std::string sig = gemm_signature(kind, a.dtype);
  wkf_kernel* k = kernel(sig, [&] { return gemm_source(kind, a.dtype); });

  struct {
    const void* a;
    const void* b;
    void* c;
    uint32_t m, n, k, pad;
  } args = {wkf_buffer_ptr(a.buffer.get()), wkf_buffer_ptr(b.buffer.get()), wkf_buffer_ptr(out.buffer.get()),
            uint32_t(M), uint32_t(N), uint32_t(K), 0};
  std::vector<unsigned char> bytes(sizeof(args));
  memcpy(bytes.data(), &args, sizeof(args));

  LaunchRecord r;
  r.kind = "gemm";
  r.signature = sig;
  r.block[0] = 256;
  if (kind == GemmKind::Generic) {
    r.grid[0] = uint32_t((N + 63) / 64);
    r.grid[1] = uint32_t((M + 63) / 64);
    if (r.grid[1] > 65535) throw Error(WKF_ERR_UNSUPPORTED, "mat_mul: too many rows for the generic kernel");
  } else {
    const size_t tiles = ((M + 255) / 256) * ((N + 255) / 256);
    if (tiles > 0x7fffffffull) throw Error(WKF_ERR_UNSUPPORTED, "mat_mul: too many tiles");
    r.grid[0] = uint32_t(tiles);
  }
  std::ostringstream d;
  d << "m=" << M << " n=" << N << " k=" << K << (kind == GemmKind::Generic ? " generic" : " mfma 256x256 tiles");
  if (kind == GemmKind::MfmaF16Edge || kind == GemmKind::MfmaF32Edge) d << " edge";
  r.detail = d.str();
  record(std::move(r), k, bytes);
  return out;
}

}  // namespace wkf

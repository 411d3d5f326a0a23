// mat_mul: UntypedMatMul::run_with_query of the reference (src/matmul.rs:157-205).
#include <algorithm>
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
const char* const kGemmSkinny =
#include "kernels/gemm_skinny.hip.inc"
    ;
const char* const kGemmSkinnyNarrow =
#include "kernels/gemm_skinny_narrow.hip.inc"
    ;
const char* const kGemmSkinnyBt =
#include "kernels/gemm_skinny_bt.hip.inc"
    ;
const char* const kGemmSkinnyBtBlock =
#include "kernels/gemm_skinny_bt_block.hip.inc"
    ;
const char* const kGemmSkinnyBtValu =
#include "kernels/gemm_skinny_bt_valu.hip.inc"
    ;
const char* const kGemmSkinnyTr =
#include "kernels/gemm_skinny_tr.hip.inc"
    ;
const char* const kGemmF16T128 =
#include "kernels/gemm_f16_t128.hip.inc"
    ;
const char* const kGemmF16Dma =
#include "kernels/gemm_f16_dma.hip.inc"
    ;
const char* const kGemmF16Flex =
#include "kernels/gemm_f16_flex.hip.inc"
    ;
const char* const kGemmF16Stream =
#include "kernels/gemm_f16_stream.hip.inc"
    ;
const char* const kGemmF16Tail =
#include "kernels/gemm_f16_tail.hip.inc"
    ;
const char* const kGemmF32Tail =
#include "kernels/gemm_f32_tail.hip.inc"
    ;
const char* const kGemmF16ShortK =
#include "kernels/gemm_f16_shortk.hip.inc"
    ;
// most rows of A the lane-per-column bandwidth kernel takes (accumulators: rows x 8 per lane for f16, rows x 4 for f32;
// f32 has no MFMA decode kernel for a row-major B, and a 256-row MFMA tile for 32 rows of f32 is 3 times slower still)
constexpr size_t kSkinnyRowsF16 = 16, kSkinnyRowsF32 = 32;
}  // namespace

GemmKind gemm_pick(DType dt, size_t m, size_t n, size_t k, bool b_transposed) {
  if (m == 0 || n == 0 || k == 0) return GemmKind::Generic;
  const bool whole = m % 256 == 0 && n % 256 == 0;
  // (the full-tile f16 kernel addresses a tile's rows with 32-bit byte offsets from the tile origin)
  if (dt == DType::F16 && whole && k % 64 == 0 && k <= (size_t(1) << 21) && n <= (size_t(1) << 22)) return GemmKind::MfmaF16;
  if (dt == DType::F32 && whole && k % 32 == 0) return GemmKind::MfmaF32;
  // ragged shapes keep the MFMA kernels as long as every row of A and B starts on a 16-byte boundary
  // and the problem is worth a 256 x 256 tile; tiny or unaligned ones take the generic kernel
  const size_t chunk = dt == DType::F16 ? 8 : 4;
  if (k % chunk == 0 && (b_transposed || n % chunk == 0) && m >= 16 && n >= 16 && m * n * k >= (size_t(1) << 18))
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

// Chooses the tile of the flexible f16 kernel for [M x K] x [K x N] on `cus` compute units: 32-row and 32-column blocks
// per wave (the tile is 64 ni x 64 nj), LDS stages and K slices, by a cost model fitted to a sweep on MI355X
// (21 shapes [64..1024] x {4096, 11008} x {4096, 11008}, 14 configurations; mean error 8 %).  A step of a lone
// workgroup on a compute unit takes `step_us`; two workgroups that share a compute unit (128 x 128 tiles in two
// stages) take 0.79 of running one after the other; every further round costs 7.5 us, the fold of K slices 8.5 us.
struct FlexChoice { int ni, nj, ns; size_t slices; };
static double flex_model_us(const FlexChoice& c, size_t M, size_t N, size_t K, size_t batch, size_t cus) {
  static const double step_us[3][5] = {{0, 0, 0, 0, 0}, {0, 0, 0.281, 0.414, 0.566}, {0, 0, 0.427, 0.635, 0.737}};
  const size_t tiles = ((M + 64 * c.ni - 1) / (64 * c.ni)) * ((N + 64 * c.nj - 1) / (64 * c.nj)) * batch;
  size_t kc = ((K + c.slices - 1) / c.slices + 63) / 64 * 64;
  const size_t S = (K + kc - 1) / kc, steps = kc / 64;
  const size_t per_cu = 160 / (size_t(c.ns) * 8 * (c.ni + c.nj)) >= 2 ? 2 : 1;
  const size_t load = (tiles * S + cus - 1) / cus;  // workgroups per compute unit
  const double s = step_us[c.ni][c.nj] * (c.ns == 2 ? 1.6 : 1.0);
  double t = 3.4;
  if (per_cu == 1) t += double(load) * steps * s + double(load - 1) * 7.5;
  else {
    const size_t rounds = (load + 1) / 2;
    t += double(load / 2) * steps * s * 2 * 0.79 + double(load % 2) * steps * s + double(rounds - 1) * 7.5;
  }
  if (S > 1) t += 8.5;
  return t;
}
static void pick_flex(size_t M, size_t N, size_t K, size_t batch, size_t cus, int* ni, int* nj, int* ns, size_t* slices) {
  static const FlexChoice candidates[] = {{2, 3, 4, 1}, {2, 3, 4, 3}, {2, 3, 3, 2}, {2, 2, 2, 1}, {2, 2, 2, 2}, {2, 2, 2, 4}, {1, 3, 4, 1}, {1, 3, 4, 2},
                                          {1, 3, 4, 4}, {1, 4, 4, 1}, {1, 2, 5, 2}, {1, 2, 5, 4}};
  *ni = 0;
  double best = 1e30;
  for (const FlexChoice& c : candidates) {
    if (batch > 1 && c.slices > 1) continue;
    if (c.slices > 1 && (K / c.slices < 512 || c.slices * M * N * 4 > (M * K + K * N) * 2)) continue;  // partial sums stay below the operands' bytes
    const double t = flex_model_us(c, M, N, K, batch, cus);
    if (t < best) {
      best = t;
      *ni = c.ni;
      *nj = c.nj;
      *ns = c.ns;
      *slices = c.slices;
    }
  }
}

TensorData Resolver::run_matmul(const NodeP& n) {
  // no fusion on either side (src/compute_graph/resolve.rs:138-154)
  TensorData a = resolve(n->a);
  TensorData b = resolve(n->b);
  const size_t R = a.layout.rank();
  if (R < 2 || b.layout.rank() != R) invalid("mat_mul: operands must have the same rank, 2 or (for a batch) more");
  if (a.dtype != b.dtype) invalid("mat_mul: operand dtypes differ");
  // leading dimensions are a batch of independent products (no counterpart in the reference, whose mat_mul is rank 2)
  size_t batch = 1;
  std::vector<size_t> out_shape;
  for (size_t d = 0; d + 2 < R; d++) {
    if (a.layout.shape[d] != b.layout.shape[d]) invalid("mat_mul: batch dimensions differ");
    batch *= a.layout.shape[d];
    out_shape.push_back(a.layout.shape[d]);
  }
  const size_t M = a.layout.shape[R - 2], N = b.layout.shape[R - 1];
  size_t K = a.layout.shape[R - 1];
  if (b.layout.shape[R - 2] != K) invalid("mat_mul: inner dimensions differ");  // src/matmul.rs:194
  out_shape.push_back(M);
  out_shape.push_back(N);
  // The reference kernel ignores strides and offsets (src/matmul.rs:96-103), which is only
  // right for contiguous operands; a view is copied into a dense buffer first.
  a = make_contiguous(a);
  // ... except B = transpose(W) of a dense W[N][K] (x * W^T, the linear-layer form; q * k^T per head in a
  // batch): the MFMA kernels read it as it lies (k contiguous), when its rows are 16-byte aligned and the
  // problem is worth a tile.
  bool b_is_t = st_.fusion == FusionMode::Tree && K > 1 && N > 1;
  if (b_is_t) {
    Layout w = b.layout;  // the last two dimensions swapped back: dense exactly when b is such a transpose
    std::swap(w.shape[R - 2], w.shape[R - 1]);
    std::swap(w.strides[R - 2], w.strides[R - 1]);
    b_is_t = w.is_contiguous();
  }
  const size_t V = a.dtype == DType::F16 ? 8 : 4;
  if (st_.fusion == FusionMode::Tree && K % V != 0 && M * N * K >= (size_t(1) << 24)) {
    // Rows of A (and of a transposed B) that do not start on 16 bytes because K is odd, say: zero-padded copies up to
    // the next multiple of the vector keep a large product on the MFMA kernels; the zeros add nothing to the sums.
    const size_t Kp = (K + V - 1) / V * V;
    auto pad_dim = [&](const TensorData& t, size_t dim) {  // t dense; returns a dense copy with `dim` grown to Kp
      std::vector<size_t> shape = t.layout.shape;
      shape[dim] = Kp;
      TensorData out = alloc(shape, t.dtype, true);
      std::vector<std::pair<size_t, size_t>> corner;
      for (size_t d = 0; d < shape.size(); d++) corner.push_back({0, t.layout.shape[d]});
      TensorData view = out;
      view.layout = out.layout.slice(corner);
      Program p;
      Instr in;
      in.op = Op::Load;
      in.dtype = t.dtype;
      in.operand = 0;
      p.ins.push_back(in);
      p.result = 0;
      launch_map(p, {t}, view, false);
      return out;
    };
    a = pad_dim(a, R - 1);
    if (b_is_t) {
      TensorData w = b;  // the dense [..., N, K] behind the transposed view
      std::swap(w.layout.shape[R - 2], w.layout.shape[R - 1]);
      std::swap(w.layout.strides[R - 2], w.layout.strides[R - 1]);
      b = pad_dim(w, R - 1);
      std::swap(b.layout.shape[R - 2], b.layout.shape[R - 1]);
      std::swap(b.layout.strides[R - 2], b.layout.strides[R - 1]);
    } else {
      b = pad_dim(make_contiguous(b), R - 2);
    }
    K = Kp;
  }
  const bool decode_bt = M >= 1 && M <= 32 && K % V == 0 && N * K >= (size_t(1) << 16);  // what the M <= 32 kernel for B^T takes
  if (!b_is_t && st_.fusion == FusionMode::Tree && N % V != 0 && M * N * K >= (size_t(1) << 24) &&
      (decode_bt || gemm_pick(a.dtype, M, N, K, true) != GemmKind::Generic)) {
    // Rows of B that do not start on 16 bytes (N odd, say) would leave a large product to the generic kernel:
    // a transposed copy of B (k contiguous, rows aligned because K is) costs one pass over B and keeps it on MFMA.
    TensorData view = b;
    std::swap(view.layout.shape[R - 2], view.layout.shape[R - 1]);
    std::swap(view.layout.strides[R - 2], view.layout.strides[R - 1]);
    b = make_contiguous(view);  // dense [..., N, K]
    std::swap(b.layout.shape[R - 2], b.layout.shape[R - 1]);
    std::swap(b.layout.strides[R - 2], b.layout.strides[R - 1]);  // seen as [..., K, N] again: the transpose of a dense matrix
    b_is_t = true;
  }
  // ... and with up to 32 rows of A (decode) W is streamed once, straight into MFMA operands
  const bool skinny_bt = b_is_t && decode_bt;
  bool bt = false;
  if (skinny_bt) {
    // handled below
  } else if (b_is_t && gemm_pick(a.dtype, M, N, K, true) != GemmKind::Generic) {
    bt = true;
  } else {
    b = make_contiguous(b);
  }
  if (M == 0 || N == 0 || batch == 0) return alloc(out_shape, a.dtype, false);
  if (batch > 65535) throw Error(WKF_ERR_UNSUPPORTED, "mat_mul: more than 65535 matrices in a batch");
  if (M > 0xffffffffull || N > 0xffffffffull || K > 0xffffffffull) throw Error(WKF_ERR_UNSUPPORTED, "mat_mul: dimension does not fit 32 bits");
  auto slices_shape = [&](size_t slices) {  // partial sums: [slice][batch...][M][N]
    std::vector<size_t> sh = {slices};
    sh.insert(sh.end(), out_shape.begin(), out_shape.end());
    return sh;
  };
  auto fold_slices = [&](const TensorData& part) {
    // adds the f32 partial sums of the K slices ([S][batch...][M][N]) and rounds to the tensor dtype
    ReduceJob fold;
    Instr ld;
    ld.op = Op::Load;
    ld.dtype = DType::F32;
    ld.operand = 0;
    fold.pre.ins.push_back(ld);
    fold.pre.result = 0;
    ld.dtype = a.dtype;
    fold.post.ins.push_back(ld);
    fold.post.result = 0;
    fold.operands = {part};
    fold.axis = 0;
    fold.rop = ReduceOp::Sum;
    fold.fold_dtype = a.dtype;
    return launch_reduce(fold);
  };
  if (skinny_bt) {
    const size_t kblock = 128 / dtype_size(a.dtype);  // 128 bytes of every row per step
    const bool valu_rows = a.dtype == DType::F32 ? M <= 16 : M <= 4;
    wkf_props bprops;
    if (wkf_device_props(dev_, &bprops) != WKF_OK) throw Error(WKF_ERR_HIP, wkf_last_error());
    if (!valu_rows && M <= 16 && (N + 31) / 32 * batch >= size_t(std::max(1, bprops.compute_units)) && K >= 8 * kblock) {
      // Enough groups of 32 rows of W to give every compute unit a block: the eight waves of a block share K among
      // themselves and add up through the LDS, so there are no partial sums in memory and no second launch
      // ([M x 4096] x W[11008 x 4096]^T f16, M = 8: 22.4 + 4.0 us -> 25.0 us, M = 16: 27.9 + 4.0 -> 27.2; at M = 32 the
      // short walks of K cost more than the second launch)
      size_t chunk = (K + 7) / 8;
      chunk = (chunk + kblock - 1) / kblock * kblock;
      TensorData out = alloc(out_shape, a.dtype, false);
      const std::string sig = std::string("gemm|gfx950|") + dtype_name(a.dtype) + "|skinny_bt|mfma32x32|block8";
      wkf_kernel* k = kernel(sig, [&] { return std::string("#define WKF_H ") + (a.dtype == DType::F16 ? "1" : "0") + "\n" + kGemmSkinnyBtBlock; });
      struct {
        const void* a;
        const void* w;
        void* c;
        uint32_t m, n, k, chunk;
      } bargs = {wkf_buffer_ptr(a.buffer.get()), wkf_buffer_ptr(b.buffer.get()), wkf_buffer_ptr(out.buffer.get()),
                 uint32_t(M), uint32_t(N), uint32_t(K), uint32_t(chunk)};
      std::vector<unsigned char> bbytes(sizeof(bargs));
      memcpy(bbytes.data(), &bargs, sizeof(bargs));
      LaunchRecord r;
      r.kind = "gemm";
      r.signature = sig;
      r.block[0] = 512;
      r.grid[0] = uint32_t((N + 31) / 32);
      r.grid[2] = uint32_t(batch);
      std::ostringstream d;
      d << "m=" << M << " n=" << N << " k=" << K << " skinny B^T, K over the 8 waves of a block";
      if (batch > 1) d << " batch=" << batch;
      r.detail = d.str();
      record(std::move(r), k, bbytes);
      return out;
    }
    const size_t gridx = (N + 127) / 128;
    // workgroups to aim for, from a sweep on MI355X ([M x 4096] x W[11008 x 4096]^T and W[4096 x 4096]^T): more slices
    // fill the chip, fewer keep the f32 partial sums (written and read once more by the fold) small as M grows
    // up to 16 rows of f32: the vector ALUs keep up with the memory where the f32 matrix instruction (on 32 padded
    // rows) does not; the block keeps its slice of A in the LDS, which bounds the slice
    // ([M x 4096] x W[11008 x 4096]^T, kernel + fold: M = 1 54 -> 34 us, M = 8 58 -> 43, M = 16 71 -> 61; [16 x 11008] x W[4096 x 11008]^T 65 -> 44)
    const bool valu = a.dtype == DType::F32 ? M <= 16 : M <= 4;
    const size_t want = st_.skinny_blocks > 0 ? size_t(st_.skinny_blocks) : (M >= 16 ? 512 : 1024);
    size_t S = (want + gridx * batch - 1) / (gridx * batch);
    S = std::min(S, std::max<size_t>(1, K * dtype_size(a.dtype) / (8 * M)));  // partial sums stay under half of W's bytes
    S = std::min(S, std::max<size_t>(1, K / (2 * kblock)));
    if (valu) {
      // the block's slice of A lives in static LDS, [M][chunk_max] with chunk_max a power of two: at most 2048
      // elements of each row and at most 64 KiB in all, so that several blocks share a compute unit
      size_t lim = 2048;
      while (lim > 256 && M * lim * dtype_size(a.dtype) > 65536) lim /= 2;
      S = std::max(S, (K + lim - 1) / lim);
    }
    size_t chunk = (K + S - 1) / S;
    chunk = (chunk + kblock - 1) / kblock * kblock;
    S = (K + chunk - 1) / chunk;
    if (S > 65535) throw Error(WKF_ERR_UNSUPPORTED, "mat_mul: too many K slices");
    // Rows of A that fit the LDS whole: no slices and no second launch
    // ([1 x 4096] x W[11008 x 4096]^T f16: 16.8 + 3.9 us in two launches -> 14.6 us in one; f32: 31.9 + 4.0 -> 29.6)
    const size_t vlen = 16 / dtype_size(a.dtype);
    const size_t k_lds = (K + 256 * vlen - 1) / (256 * vlen) * (256 * vlen);
    const bool whole_k = valu && M * k_lds * dtype_size(a.dtype) <= 65536;
    // (a whole wave walks one row of W, 1 KiB a load, unless a row is shorter than that: measured on
    // [1 x 4096] x W[11008 x 4096]^T with 1, 2, 4, 8 rows a wave, f16 14.6, 18.5, 15.7, 20.2 us, f32 29.6, 30.3, 38.4, 33.9 us)
    size_t rows_per_wave = 1;
    while (rows_per_wave < 8 && K * dtype_size(a.dtype) * rows_per_wave < 1024) rows_per_wave *= 2;
    if (whole_k) {
      S = 1;
      chunk = K;
    }
    TensorData part = whole_k ? TensorData() : alloc(slices_shape(S), DType::F32, false);
    TensorData out_whole = whole_k ? alloc(out_shape, a.dtype, false) : TensorData();
    size_t chunk_max = 256;
    while (chunk_max < chunk) chunk_max *= 2;
    if (whole_k) chunk_max = k_lds;
    const std::string sig = valu ? std::string("gemm|gfx950|") + dtype_name(a.dtype) + "|skinny_bt|valu|m" + std::to_string(M) + "|c" + std::to_string(chunk_max) +
                                       (whole_k ? "|r" + std::to_string(rows_per_wave) : std::string())
                                 : std::string("gemm|gfx950|") + dtype_name(a.dtype) + "|skinny_bt|mfma32x32";
    wkf_kernel* k = kernel(sig, [&] {
      if (valu)
        return std::string("#define WKF_H ") + (a.dtype == DType::F16 ? "1" : "0") + "\n#define WKF_M " + std::to_string(M) + "\n#define WKF_CHUNK_MAX " +
               std::to_string(chunk_max) + "\n#define WKF_WHOLE_K " + (whole_k ? "1" : "0") + "\n#define WKF_R " + std::to_string(rows_per_wave) + "\n" +
               kGemmSkinnyBtValu;
      return std::string("#define WKF_H ") + (a.dtype == DType::F16 ? "1" : "0") + "\n" + kGemmSkinnyBt;
    });
    struct {
      const void* a;
      const void* w;
      void* part;
      uint32_t m, n, k, chunk;
    } sargs = {wkf_buffer_ptr(a.buffer.get()), wkf_buffer_ptr(b.buffer.get()), whole_k ? nullptr : wkf_buffer_ptr(part.buffer.get()),
               uint32_t(M), uint32_t(N), uint32_t(K), uint32_t(chunk)};
    std::vector<unsigned char> sbytes(sizeof(sargs));
    memcpy(sbytes.data(), &sargs, sizeof(sargs));
    if (valu) {
      struct {
        const void* a;
        const void* w;
        void* part;
        void* c;
        uint32_t m, n, k, chunk;
      } vargs = {sargs.a, sargs.w, sargs.part, whole_k ? wkf_buffer_ptr(out_whole.buffer.get()) : nullptr, sargs.m, sargs.n, sargs.k, sargs.chunk};
      sbytes.resize(sizeof(vargs));
      memcpy(sbytes.data(), &vargs, sizeof(vargs));
    }
    LaunchRecord r;
    r.kind = "gemm";
    r.signature = sig;
    r.block[0] = 256;
    r.grid[0] = uint32_t(whole_k ? (N + 4 * rows_per_wave - 1) / (4 * rows_per_wave) : gridx);
    r.grid[1] = uint32_t(S);
    r.grid[2] = uint32_t(batch);
    std::ostringstream d;
    d << "m=" << M << " n=" << N << " k=" << K << " skinny B^T" << (valu ? " valu" : "");
    if (whole_k) d << " whole K, " << rows_per_wave << " rows a wave";
    else d << " slices=" << S;
    if (batch > 1) d << " batch=" << batch;
    r.detail = d.str();
    record(std::move(r), k, sbytes);
    if (whole_k) return out_whole;
    return fold_slices(part);
  }
  // Up to 32 rows of A against a row-major f16 B: B is streamed once through wave-private LDS tiles and read back
  // k-contiguous by LDS transpose reads into MFMA operands (beyond a few rows the lane-per-column kernel below is
  // bound by its scalar multiply-adds, not by memory).
  // (measured on MI355X, [M x 4096] x [4096 x 11008] f16: M = 1 27 us on the lane-per-column kernel against 31 here,
  // M = 4 37 against 33, M = 8 44 against 34, M = 16 71 against 35)
  const size_t tr_min_rows = st_.skinny_tr_rows > 0 ? size_t(st_.skinny_tr_rows) : 4;
  if (st_.fusion == FusionMode::Tree && !bt && a.dtype == DType::F16 && M >= tr_min_rows && M <= 32 && N % 8 == 0 && K % 8 == 0 &&
      N * K >= (size_t(1) << 16)) {
    const size_t gridx = (N + 255) / 256;
    const size_t want = st_.skinny_blocks > 0 ? size_t(st_.skinny_blocks) : (M >= 16 ? 512 : 1024);
    size_t S = (want + gridx * batch - 1) / (gridx * batch);
    S = std::min(S, std::max<size_t>(1, K * 2 / (8 * M)));  // partial sums stay under half of B's bytes
    S = std::min(S, std::max<size_t>(1, K / 64));
    size_t chunk = (K + S - 1) / S;
    chunk = (chunk + 31) / 32 * 32;
    S = (K + chunk - 1) / chunk;
    if (S > 65535) throw Error(WKF_ERR_UNSUPPORTED, "mat_mul: too many K slices");
    TensorData part = alloc(slices_shape(S), DType::F32, false);
    const std::string sig = "gemm|gfx950|f16|skinny_tr|mfma32x32x16";
    wkf_kernel* k = kernel(sig, [&] { return std::string(kGemmSkinnyTr); });
    struct {
      const void* a;
      const void* b;
      void* part;
      uint32_t m, n, k, chunk;
    } sargs = {wkf_buffer_ptr(a.buffer.get()), wkf_buffer_ptr(b.buffer.get()), wkf_buffer_ptr(part.buffer.get()),
               uint32_t(M), uint32_t(N), uint32_t(K), uint32_t(chunk)};
    std::vector<unsigned char> sbytes(sizeof(sargs));
    memcpy(sbytes.data(), &sargs, sizeof(sargs));
    LaunchRecord r;
    r.kind = "gemm";
    r.signature = sig;
    r.block[0] = 256;
    r.grid[0] = uint32_t(gridx);
    r.grid[1] = uint32_t(S);
    r.grid[2] = uint32_t(batch);
    std::ostringstream d;
    d << "m=" << M << " n=" << N << " k=" << K << " skinny mfma slices=" << S;
    if (batch > 1) d << " batch=" << batch;
    r.detail = d.str();
    record(std::move(r), k, sbytes);
    return fold_slices(part);
  }
  // A handful of rows (decode): reading B once is all the work -> the bandwidth kernel, K cut into slices
  // across the grid, then one reduce launch that adds the slices and rounds to the tensor dtype.
  if (st_.fusion == FusionMode::Tree && !bt && M <= (a.dtype == DType::F16 ? kSkinnyRowsF16 : kSkinnyRowsF32) && N % V == 0 && K >= 16 && N * K >= (size_t(1) << 16)) {
    const size_t esize = dtype_size(a.dtype);
    // A narrow B (rows of at most 2 KiB, p . v at decode time) would leave most lanes of the lane-per-column kernel
    // without columns: its lanes cover a few consecutive rows of B each instead
    // ([32,1,2048] x [32,2048,128] f16: 11.5 -> 3 us before the fold)
    const bool narrow = M <= 4 && N / V <= 128 && K >= 64;
    size_t lanes_per_row = 1;
    while (lanes_per_row < N / V) lanes_per_row *= 2;
    const size_t colblocks = narrow ? 1 : (N + 256 * V - 1) / (256 * V);
    const size_t want = st_.skinny_blocks > 0 ? size_t(st_.skinny_blocks) : 1024;
    size_t S = (want + colblocks * batch - 1) / (colblocks * batch);
    S = std::min(S, std::max<size_t>(1, K * esize / (8 * M)));  // partial sums stay under half of B's bytes
    S = std::min(S, K / (narrow ? 64 : 16));
    S = std::max<size_t>(S, 1);
    size_t chunk = (K + S - 1) / S;
    chunk = (chunk + 3) & ~size_t(3);
    S = (K + chunk - 1) / chunk;
    if (S > 65535) throw Error(WKF_ERR_UNSUPPORTED, "mat_mul: too many K slices");
    TensorData part = alloc(slices_shape(S), DType::F32, false);
    std::ostringstream sg;
    sg << "gemm|gfx950|" << dtype_name(a.dtype) << "|skinny|m" << M << "|v" << V;
    if (narrow) sg << "|narrow" << lanes_per_row;
    const std::string sig = sg.str();
    wkf_kernel* k = kernel(sig, [&] {
      std::ostringstream src;
      src << "#define WKF_T " << (a.dtype == DType::F32 ? "float" : "_Float16") << "\n#define WKF_V " << V << "\n#define WKF_M " << M << "\n";
      if (narrow) src << "#define WKF_LR " << lanes_per_row << "\n" << kGemmSkinnyNarrow;
      else src << kGemmSkinny;
      return src.str();
    });
    struct {
      const void* a;
      const void* b;
      void* part;
      uint32_t m, n, k, chunk;
    } sargs = {wkf_buffer_ptr(a.buffer.get()), wkf_buffer_ptr(b.buffer.get()), wkf_buffer_ptr(part.buffer.get()),
               uint32_t(M), uint32_t(N), uint32_t(K), uint32_t(chunk)};
    std::vector<unsigned char> sbytes(sizeof(sargs));
    memcpy(sbytes.data(), &sargs, sizeof(sargs));
    LaunchRecord r;
    r.kind = "gemm";
    r.signature = sig;
    r.block[0] = 256;
    r.grid[0] = uint32_t(colblocks);
    r.grid[1] = uint32_t(S);
    r.grid[2] = uint32_t(batch);
    std::ostringstream d;
    d << "m=" << M << " n=" << N << " k=" << K << " skinny" << (narrow ? " narrow" : "") << " slices=" << S;
    if (batch > 1) d << " batch=" << batch;
    r.detail = d.str();
    record(std::move(r), k, sbytes);

    return fold_slices(part);
  }

  const GemmKind kind = gemm_pick(a.dtype, M, N, K, bt);
  const bool mfma = kind != GemmKind::Generic;
  // A few tiles over a long K leave most compute units idle: cut K into slices across blockIdx.y
  // (f32 partial sums per slice, then one reduce launch), as long as the partial sums stay below
  // the bytes of A and B.
  size_t slices = 1, kchunk = 0;
  wkf_props props;
  if (wkf_device_props(dev_, &props) != WKF_OK) throw Error(WKF_ERR_HIP, wkf_last_error());
  const size_t cus = size_t(std::max(1, props.compute_units));
  // f16 products whose 256 x 256 tiles would fill at most half of the chip take 128 x 128 tiles, two workgroups per
  // compute unit ([512 x 4096] x [4096 x 11008]: 68 us against 109; with 172 of the large tiles, [1024 x ...], the large
  // tile is the faster one again: 97 us against 114)
  const size_t tiles256 = ((M + 255) / 256) * ((N + 255) / 256);
  // ... and so do products that would waste half of every large tile (128 columns of attention values, say)
  const size_t pad256 = ((M + 255) / 256 * 256) * ((N + 255) / 256 * 256), pad128 = ((M + 127) / 128 * 128) * ((N + 127) / 128 * 128);
  // ... but not a single product over a long K with 48 large tiles or more: cut into K slices those fill the chip, and
  // over a long K the large tile's lower LDS traffic per flop outweighs the partial sums ([1280 x 11008] x [11008 x 4096]:
  // 121 us in 3 slices against 174 on the small tile; at K = 4096 the small tile still wins: 54 against 61 for [1024 x ...])
  const bool long_k_in_slices = batch == 1 && K >= 8192 && tiles256 >= 48;
  // (its loads take 32-bit byte offsets into a matrix: each operand matrix stays under 2 GiB)
  const bool t128 = mfma && a.dtype == DType::F16 && st_.fusion == FusionMode::Tree && st_.gemm_t128 &&
                    ((tiles256 * batch * 2 <= cus && !long_k_in_slices) || pad128 * 20 <= pad256 * 11) && M * K < (size_t(1) << 30) && K * N < (size_t(1) << 30);
  // Tiles of 64 NI x 64 NJ with the operands loaded straight into the LDS (kernels/gemm_f16_flex.hip.inc), for products
  // that the 256 x 256 tile would spread badly over the chip.  WKF_GEMM_FLEX="ni,nj,stages,slices" forces a shape.
  // (rows of C 16-byte aligned, N % 8 == 0: the kernel stores whole 16-byte vectors)
  if (mfma && a.dtype == DType::F16 && st_.fusion == FusionMode::Tree && K % 64 == 0 && N % 8 == 0 && M * K < (size_t(1) << 30) &&
      K * N < (size_t(1) << 30)) {
    int ni = 0, nj = 0, ns = 0;
    size_t S = 1;
    bool forced = false;
    if (const char* f = getenv("WKF_GEMM_FLEX")) {
      unsigned long long sl = 1;
      forced = sscanf(f, "%d,%d,%d,%llu", &ni, &nj, &ns, &sl) == 4 && ni >= 1 && ni <= 2 && nj >= 2 && nj <= 4 && ns >= 2 &&
               size_t(ns) * 8 * (ni + nj) <= 160 && sl >= 1;
      S = size_t(sl);
      if (!forced) ni = 0;
    }
    // where the 128 x 128 tile would be taken (a few hundred rows against a wide weight, small batches), except one
    // column of tiles over a long K against a small B, which keeps that kernel's rotated walk over K
    const bool one_column = N <= 128 && K >= 512 && K * N * dtype_size(a.dtype) <= (size_t(1) << 20);
    if (!forced && st_.gemm_flex && t128 && !one_column) {
      S = 1;
      pick_flex(M, N, K, batch, cus, &ni, &nj, &ns, &S);
    }
    if (ni > 0 && batch > 1) S = 1;
    size_t kc = 0;
    if (ni > 0 && S > 1) {
      kc = ((K + S - 1) / S + 63) / 64 * 64;
      S = (K + kc - 1) / kc;
    }
    if (ni > 0) {
      const bool sp = S > 1;
      const size_t bm = 64 * size_t(ni), bn = 64 * size_t(nj);
      const size_t ftiles = ((M + bm - 1) / bm) * ((N + bn - 1) / bn);
      if (ftiles > 0x7fffffffull || S > 65535) throw Error(WKF_ERR_UNSUPPORTED, "mat_mul: too many tiles");
      TensorData fout = sp ? alloc(slices_shape(S), DType::F32, false) : alloc(out_shape, a.dtype, false);
      std::string fsig = "gemm|gfx950|f16|mfma32x32x16|" + std::to_string(bm) + "x" + std::to_string(bn) + "x64|w2x2|direct to LDS|stages" + std::to_string(ns);
      if (sp) fsig += "|splitk";
      if (bt) fsig += "|bt";
      wkf_kernel* fk = kernel(fsig, [&] {
        return "#define WKF_NI " + std::to_string(ni) + "\n#define WKF_NJ " + std::to_string(nj) + "\n#define WKF_NS " + std::to_string(ns) + "\n" +
               (sp ? "#define WKF_SPLITK 1\n" : "") + (bt ? "#define WKF_BT 1\n" : "") + kGemmF16Flex;
      });
      struct {
        const void* a;
        const void* b;
        void* c;
        uint32_t m, n, k, kchunk;
      } fargs = {wkf_buffer_ptr(a.buffer.get()), wkf_buffer_ptr(b.buffer.get()), wkf_buffer_ptr(fout.buffer.get()),
                 uint32_t(M), uint32_t(N), uint32_t(K), uint32_t(kc)};
      std::vector<unsigned char> fbytes(sizeof(fargs));
      memcpy(fbytes.data(), &fargs, sizeof(fargs));
      LaunchRecord r;
      r.kind = "gemm";
      r.signature = fsig;
      r.block[0] = 256;
      r.grid[0] = uint32_t(ftiles);
      r.grid[1] = uint32_t(S);
      r.grid[2] = uint32_t(batch);
      std::ostringstream d;
      d << "m=" << M << " n=" << N << " k=" << K << " mfma " << bm << "x" << bn << " tiles" << (bt ? " B^T" : "") << ", operands loaded straight into the LDS, "
        << ns << " stages";
      if (sp) d << " slices=" << S;
      if (batch > 1) d << " batch=" << batch;
      r.detail = d.str();
      record(std::move(r), fk, fbytes);
      return sp ? fold_slices(fout) : fout;
    }
  }
  const size_t tile = t128 ? 128 : 256;
  const size_t tiles = ((M + tile - 1) / tile) * ((N + tile - 1) / tile);
  const size_t slots = t128 ? 2 * cus : cus;  // workgroups the chip holds at once
  if (mfma && batch == 1 && st_.fusion == FusionMode::Tree) {
    const size_t bk = a.dtype == DType::F16 ? 64 : 32;
    if (tiles * 2 <= slots && K >= 1024) {
      size_t S = std::min(std::max<size_t>(1, slots / tiles), K / 512);  // rounded down: one workgroup more than the chip holds costs a second round
      while (S > 1 && S * M * N * 4 > (M * K + K * N) * dtype_size(a.dtype)) S--;
      if (S > 1) {
        kchunk = (K + S - 1) / S;
        kchunk = (kchunk + bk - 1) / bk * bk;
        slices = (K + kchunk - 1) / kchunk;
      }
    }
  }
  const bool split = slices > 1;
  // Full tiles (f16 also ragged ones) that do not fill a whole number of rounds on the chip (the [2048 x 4096] x [4096 x 11008] MLP
  // product: 344 tiles on 256 compute units): the tiles of the last, partly filled round are computed as two halves
  // of 128 rows each by twice as many workgroups, so that round fills twice as many compute units and takes about
  // half as long (kernels/gemm_f16_tail.hip.inc, kernels/gemm_f32_tail.hip.inc).
  size_t ntail = 0, nmain = 0;
  const bool tail_ragged = kind == GemmKind::MfmaF16Edge && K <= (size_t(1) << 21) && N <= (size_t(1) << 22) && N % 8 == 0;
  // full f16 tiles whose offsets inside a tile fit 32 bits: the operands go from memory straight into the LDS
  // (kernels/gemm_f16_dma.hip.inc; B as it lies or transposed, single products and batches, whole and half tiles)
  const bool dma_ok = kind == GemmKind::MfmaF16 && !t128 && !split && st_.fusion == FusionMode::Tree && st_.gemm_dma &&
                      K <= (size_t(1) << 21) && N <= (size_t(1) << 22);
  if ((kind == GemmKind::MfmaF16 || kind == GemmKind::MfmaF32 || tail_ragged) && (!bt || dma_ok) && !t128 && !split && batch == 1 &&
      st_.fusion == FusionMode::Tree && st_.gemm_tail) {
    nmain = tiles / cus * cus;
    ntail = tiles - nmain;
    if (nmain == 0 || ntail * 2 > cus) ntail = 0;
  }
  const bool tail = ntail > 0;
  // Many full tiles over K = 64 or 128 (attention scores, a low-rank update): what bounds them is the stores of C.  One
  // workgroup per compute unit walks the tiles of the whole batch with the next tile's operands in flight under the
  // current tile's MFMAs and stores (kernels/gemm_f16_shortk.hip.inc).
  const bool many_tiles = kind == GemmKind::MfmaF16 && !t128 && !split && !tail && st_.fusion == FusionMode::Tree && tiles * batch >= 4 * cus &&
                          cus % 8 == 0 && tiles * batch <= 0xffffffffull;
  // ... and over K = 128 to 256 the stores of a tile are issued under the MFMAs of the next (kernels/gemm_f16_stream.hip.inc)
  // (its buffer resources cover one whole tensor of the batch each: 32-bit byte offsets)
  const bool stream = many_tiles && st_.gemm_stream && (K == 128 || K == 192 || K == 256) && batch * M * K < (size_t(1) << 30) &&
                      batch * K * N < (size_t(1) << 30) && batch * M * N < (size_t(1) << 30);
  const bool shortk = many_tiles && !stream && st_.gemm_shortk && (K == 64 || K == 128);
  // one column of 128-wide tiles over a long K, B small enough to stay in L2: the workgroups share no rows of A and
  // start their walk over K at different tiles (kernels/gemm_f16_t128.hip.inc, WKF_ROTK)
  const bool dma = dma_ok && !shortk && !stream;
  if (dma && !tail) nmain = tiles;
  const bool rotk = t128 && !split && N <= 128 && K >= 512 && K * N * dtype_size(a.dtype) <= (size_t(1) << 20);
  TensorData out = split ? alloc(slices_shape(slices), DType::F32, false) : alloc(out_shape, a.dtype, false);
  std::string sig = t128 ? std::string("gemm|gfx950|f16|mfma32x32x16|128x128x64|w2x2|edge") : gemm_signature(kind, a.dtype);
  // ragged f16 shapes (and K slices) on the large tile: buffer loads that read zeros past the edges, unless an offset
  // inside a tile could pass 32 bits or rows of C do not start 16-byte aligned; those keep 64-bit pointers
  const bool f16_large = !t128 && (kind == GemmKind::MfmaF16 || kind == GemmKind::MfmaF16Edge);
  const bool ragged16 = f16_large && (split || kind == GemmKind::MfmaF16Edge);
  const bool edge_ptr = ragged16 && !(K <= (size_t(1) << 21) && N <= (size_t(1) << 22) && N % 8 == 0);
  if (split) sig += sig.find("|edge") == std::string::npos ? "|edge|splitk" : "|splitk";
  if (edge_ptr) sig += "|ptr";
  if (bt) sig += "|bt";
  if (rotk) sig += "|rotk";
  if (shortk) sig += K == 64 ? "|whole K in LDS|nt1" : "|whole K in LDS|nt2";
  if (stream) sig += "|stores under the next tile|nk" + std::to_string(K / 64);
  if (tail && !dma) sig += "|last round in half tiles";  // (a ragged shape keeps "|edge" in front of it)
  if (dma) sig += "|direct to LDS";  // one binary for whole tiles and for a last round in half tiles
  wkf_kernel* k = kernel(sig, [&] {
    if (dma) return std::string(bt ? "#define WKF_BT 1\n" : "") + kGemmF16Dma;
    if (tail && kind == GemmKind::MfmaF32) return std::string(kGemmF32Tail);
    if (tail) return std::string(tail_ragged ? "#define WKF_EDGEBUF 1\n" : "") + kGemmF16Tail;
    std::string src = bt ? "#define WKF_BT 1\n" : "";
    if (t128) return src + (split ? "#define WKF_SPLITK 1\n" : "") + (rotk ? "#define WKF_ROTK 1\n" : "") + kGemmF16T128;
    if (shortk) return src + (K == 64 ? "#define WKF_NT 1\n" : "#define WKF_NT 2\n") + kGemmF16ShortK;
    if (stream) return src + "#define WKF_NK " + std::to_string(K / 64) + "\n" + kGemmF16Stream;
    if (ragged16) return src + (split ? "#define WKF_SPLITK 1\n" : "") + (edge_ptr ? "#define WKF_EDGE 1\n" : "#define WKF_EDGEBUF 1\n") + kGemmF16;
    if (!split) return src + gemm_source(kind, a.dtype);
    const GemmKind base = a.dtype == DType::F16 ? GemmKind::MfmaF16Edge : GemmKind::MfmaF32Edge;
    return src + "#define WKF_SPLITK 1\n" + gemm_source(base, a.dtype);
  });

  struct {
    const void* a;
    const void* b;
    void* c;
    uint32_t m, n, k, kchunk;
  } args = {wkf_buffer_ptr(a.buffer.get()), wkf_buffer_ptr(b.buffer.get()), wkf_buffer_ptr(out.buffer.get()),
            uint32_t(M), uint32_t(N), uint32_t(K), uint32_t(kchunk)};
  if (shortk || stream) args.kchunk = uint32_t(batch);  // the kernel walks the tiles of every matrix itself
  std::vector<unsigned char> bytes(sizeof(args));
  memcpy(bytes.data(), &args, sizeof(args));
  if (tail || dma) {
    const uint32_t extra[2] = {uint32_t(nmain), uint32_t(ntail)};
    const size_t at = bytes.size();
    bytes.resize(at + sizeof(extra));
    memcpy(bytes.data() + at, extra, sizeof(extra));
  }

  LaunchRecord r;
  r.kind = "gemm";
  r.signature = sig;
  r.block[0] = 256;
  if (kind == GemmKind::Generic) {
    r.grid[0] = uint32_t((N + 63) / 64);
    r.grid[1] = uint32_t((M + 63) / 64);
    if (r.grid[1] > 65535) throw Error(WKF_ERR_UNSUPPORTED, "mat_mul: too many rows for the generic kernel");
  } else {
    if (tiles > 0x7fffffffull) throw Error(WKF_ERR_UNSUPPORTED, "mat_mul: too many tiles");
    r.grid[0] = uint32_t((shortk || stream) ? cus : (tail || dma) ? nmain + 2 * ntail : tiles);
    r.grid[1] = uint32_t(slices);
  }
  r.grid[2] = uint32_t((shortk || stream) ? 1 : batch);
  std::ostringstream d;
  d << "m=" << M << " n=" << N << " k=" << K << (kind == GemmKind::Generic ? " generic" : t128 ? " mfma 128x128 tiles" : " mfma 256x256 tiles");
  if (!t128 && (kind == GemmKind::MfmaF16Edge || kind == GemmKind::MfmaF32Edge)) d << " edge";
  if (bt) d << " B^T";
  if (rotk) d << " K start rotated";
  if (shortk) d << ", whole K in LDS, one workgroup per compute unit walks the tiles";
  if (dma) d << ", operands loaded straight into the LDS";
  if (stream) d << ", one workgroup per compute unit walks the tiles, a tile's stores under the next tile's MFMAs";
  if (split) d << " slices=" << slices;
  if (tail) d << ", last round: " << ntail << " tiles as " << 2 * ntail << " halves of 128 rows";
  if (batch > 1) d << " batch=" << batch;
  r.detail = d.str();
  record(std::move(r), k, bytes);
  if (split) {
    return fold_slices(out);
  }
  return out;
}

}  // namespace wkf

// Kernel generator: turns a fused-kernel description into HIP source for gfx950
// plus the signature the code-object cache is keyed by.  It replaces the WGSL
// assembler of the reference (GenericKernel, src/kernel.rs:19-496, and
// VisitTiledKernel, src/visit_tiled.rs:10-194).  Shapes, strides, offsets and
// literal constants are kernel ARGUMENTS, so one binary serves every tensor size
// and every constant value of the same fused structure.
#pragma once

#include <string>
#include <vector>

#include "core.h"

namespace wkf {

// ---- map kernels: out[i] = expr(in_0[i], ..., in_{n-1}[i]) -----------------
// Covers the reference's element-wise, pair-wise, resize and slice_assign
// kernels (K1, K2, K5, K6: src/visit_tiled.rs:80-144, src/resize.rs:43-88,
// src/slice_assign.rs:49-66).
struct MapOperandSpec {
  DType dtype;
  bool linear;       // index = offset + work_item * V (contiguous over the iteration space)
  int inner_stride;  // vector mode: 0 or 1 (compile-time); scalar mode: -1 = run-time value
};

// Which implementation a transcendental op gets.
//  Stored: the kernel's values are stored as they are.  An op whose value feeds
//          another op ("interior") is evaluated with an f64 core and rounded
//          once, so it matches the correctly rounded f32 value and later ops
//          cannot amplify an error; the LAST op of the chain may be off by the
//          f32 library's <= 1-2 ulp, which nothing amplifies.
//  Folded: the values only feed a sum / product / max / min (tolerance class
//          1e-5 relative): every op uses the f32 library.
//  Exact:  every op is evaluated with an f64 core.
enum class MathPolicy : int { Stored = 0, Folded = 1, Exact = 2 };

struct MapSpec {
  // Tiled variant (tile_dim >= 0): some inputs ("crossed") are unit-stride along dimension `tile_dim`
  // while the output is unit-stride along the last one, e.g. out = transpose(x) + y.  A block moves a
  // 64 x 64 tile of (tile_dim, last dim): crossed inputs are read along tile_dim into LDS and read back
  // along the last dim, so global loads and stores are both coalesced.  vec is 1.
  int tile_dim = -1;
  // tile_vec == 4: every operand is read and written four elements at a time along its unit-stride dimension (both
  // tile extents are multiples of 4, every other stride and every offset too); non-crossed inputs then have
  // inner_stride 1 (a vector per lane) or 0 (one value per tile row)
  int tile_vec = 1;
  // edge of the square tile: 64, or 128 with tile_vec == 4 when the operands are large and the tiles of the crossed
  // inputs leave room for two workgroups per compute unit (longer runs of consecutive bytes per row of a tile)
  int tile_size = 64;
  std::vector<bool> crossed;         // per input; used when tile_dim >= 0
  int rank;                          // rank of the coalesced iteration space (1..kMaxRank)
  int vec;                           // elements per work item: 1, 2, 4 or 8
  int unroll;                        // work items per thread
  bool nontemporal;                  // streaming loads/stores bypass cache allocation
  std::vector<MapOperandSpec> in;    // inputs
  MapOperandSpec out;
  Program prog;
  // Further outputs computed from the same inputs over the same iteration space (one more store each;
  // shared loads and shared sub-expressions are done once).  Not with tile_dim.
  std::vector<MapOperandSpec> more_out;
  std::vector<Program> more_prog;
  MathPolicy math = MathPolicy::Stored;
  // The program holds Op::Lookup instructions: the kernel takes a table of 65536 f16 values as one more argument, copies
  // it into the LDS of 1024-lane workgroups that stay on their compute unit, and these walk the work items (unroll is 1).
  bool table = false;
};
constexpr int kMaxRank = 6;
constexpr int kMapBlock = 256;
constexpr int kMapTile = 64;

std::string map_signature(const MapSpec& s);
std::string map_source(const MapSpec& s);
// out[i] = table[in[i]] over dense f16 data: any map whose only operand is one f16 tensor, with an f16 result, is a
// function of 16 bits.  The table (65536 f16 values, 128 KiB, built once per program and constants by the map kernel
// itself run over every bit pattern) is copied into the LDS of one 1024-lane workgroup per compute unit, which then
// streams the data with 16-byte loads and stores and eight LDS reads per vector.  One binary serves every program.
// Arguments: {const void* in; void* out; const void* table; u32 nvec (16-byte vectors); u32 ntail (elements after them)}.
constexpr int kMapTableBlock = 1024;
std::string map_table_signature();
std::string map_table_source();
// what a program costs per element in units of a plain arithmetic op (an estimate: a transcendental function whose value
// feeds further arithmetic takes a correctly rounded core, about ten; the last one before the store about three)
int program_cost(const Program& p);
// Size in bytes of the argument block and the packer that fills it.
struct MapArgs {
  std::vector<void*> ptrs;               // inputs..., out, further outputs...
  uint32_t nwork;                        // number of work items (vectors)
  std::vector<uint32_t> shape;           // coalesced shape; the last entry is in work items
  std::vector<uint32_t> offsets;         // per operand, elements
  std::vector<std::vector<uint32_t>> strides;  // per operand, per dim, elements
  std::vector<float> consts;             // of prog, then of every further program
  const void* table = nullptr;           // MapSpec::table: 65536 f16 values on the device
};
std::vector<unsigned char> map_pack_args(const MapSpec& s, const MapArgs& a);

// ---- reduce kernels -----------------------------------------------------------
// K3 of the reference (src/reduce.rs:83-281) re-designed: `Row` puts T
// consecutive lanes on one output element and walks the axis with coalesced
// vector loads; `Col` puts the 64 lanes of a wave on 64 neighbouring outputs and
// walks the axis in the waves of the block.
enum class ReduceShape { Row, Col };

struct ReduceOperandSpec {
  DType dtype;
  int axis_stride;        // Row: 0 or 1 (compile time).  Col: -1 = run-time value
  int inner_stride = -1;  // Col with vec > 1: stride along the lanes' dimension, 0 or 1 (compile time)
};

struct ReduceSpec {
  ReduceShape shape;
  int outer_rank;                 // 0..3 dims of the output iteration space (coalesced)
  int vec;                        // Row: elements per load along the axis.  Col: neighbouring outputs per lane
  int threads_per_row;            // Row: T (power of two, 1..1024)
  int block;                      // threads per block
  int unroll;                     // independent loads in flight per operand
  int waves;                      // Col: waves per block walking the axis
  ReduceOp rop;
  std::vector<ReduceOperandSpec> in;
  DType out_dtype;
  Program pre;                    // value fed to the fold (one per axis element)
  Program post;                   // applied once to the folded value; one Load of operand 0 = the folded value
  MathPolicy math_pre = MathPolicy::Folded;
  MathPolicy math_post = MathPolicy::Stored;
  // A long axis with few outputs is folded in two launches: the first folds S slices of the axis and
  // stores the f32 accumulators as they are (`raw_out`, no rounding, no post), the second folds those
  // and finishes as a one-launch reduce would: round to `fold_dtype`, then `post`.
  bool raw_out = false;
  DType fold_dtype = DType::F32;  // dtype the folded value is rounded to before `post` (the reduced tensor's)
};

std::string reduce_signature(const ReduceSpec& s);
std::string reduce_source(const ReduceSpec& s);
struct ReduceArgs {
  std::vector<void*> ptrs;                        // inputs..., out
  uint32_t nrows;                                 // number of outputs
  uint32_t n;                                     // axis length (elements)
  std::vector<uint32_t> oshape;                   // outer shape
  std::vector<uint32_t> offsets;                  // per operand incl. out
  std::vector<std::vector<uint32_t>> ostrides;    // per operand incl. out, per outer dim
  std::vector<uint32_t> astrides;                 // per input
  std::vector<float> consts;                      // pre consts then post consts
};
std::vector<unsigned char> reduce_pack_args(const ReduceSpec& s, const ReduceArgs& a);

// ---- row kernels: reductions over the last axis whose results are used again on the same rows ----
// softmax (max -> sum(exp(x - max)) -> exp(x - max) / sum) and RMSNorm (sum(x^2) -> x / rms * w) read
// each row once: T lanes hold the row of every operand in registers, each `stage` folds an
// expression over the row into one scalar per row (which later stages and the final expression may
// use), and the final expression is stored.  No counterpart in the reference, which runs one kernel
// per reduce and per pair-wise op (src/compute_graph/resolve.rs:96-196); the values are the same.
struct RowStage {
  ReduceOp rop;
  Program pre;    // operands: full operands 0..K-1, then the scalars of earlier stages K..K+s-1
  Program post;   // one Load (operand 0 = the folded value)
};

struct RowSpec {
  int outer_rank;                       // dims of the row index space (coalesced), 0..3
  int vec;                              // elements per 16-byte load
  int threads_per_row;                  // T
  int block;                            // threads per block
  int vectors_per_lane;                 // NV: row length = NV * T * vec exactly, unless `ragged`
  // ragged: the row holds `nvec` vectors (a launch argument) with (NV - 1) * T < nvec <= NV * T; lanes whose last
  // vector lies past the end of the row neither load, fold nor store it
  bool ragged = false;
  // streamed: the row is longer than a block's registers hold.  One block of T lanes per row walks the row's `nvec`
  // vectors (a launch argument) once per stage and once more for the final expression, `vectors_per_lane` vectors
  // of every operand in flight per lane; the passes after the first find the row in the caches when it fits them.
  bool streamed = false;
  // streamed rows whose first two stages are max(x) and sum(exp(x - max)) (softmax): both are folded in ONE pass
  // with a running maximum (the running sum is rescaled by exp(old max - new max) whenever the maximum grows), so
  // the row is read twice in all instead of three times
  bool online_max_sum = false;
  // split (streamed rows only, with a `final`): too few rows to occupy the chip with a block each.  Every row is cut
  // into `parts` parts (a launch argument) of `chunk` vectors, one block of T lanes per part, and the stages become
  // kernels of their own: kernel `split_phase` = k < stages folds stage k over its part and leaves the value in a
  // buffer of [stages][rows][parts] floats (the extra, last pointer argument); kernel `split_phase` = stages writes
  // the result.  Each first folds the parts of the stages before it.  An online pair is one kernel (phase 0).
  bool split = false;
  int split_phase = 0;
  // team (rows with a `final`, 256 lanes): the row is longer than a block's registers hold but fits those of `parts`
  // blocks (a launch argument) with `vectors_per_lane` vectors per lane each.  One launch, the row is read once:
  // the blocks of a row exchange their folded values through 64-bit slots [stages][rows][parts] (second to last
  // pointer argument, zero-filled by the caller) and wait for each other, which needs every block of the grid
  // resident: the grid is teams * parts blocks with at most four blocks per compute unit, and a team walks rows
  // team, team + teams, ...  The last pointer argument counts the lanes that gave up waiting (see `spin`).
  bool team = false;
  bool team_mute = false;               // a variant for host-side tests of the give-up path: part 0 of every row never writes its slots
  std::vector<ReduceOperandSpec> in;    // axis_stride 1 (row in registers) or 0 (one scalar per row)
  std::vector<RowStage> stages;
  Program final;                        // same operand numbering as a stage's pre
  DType out_dtype;
  bool exact_math = false;
  // Parallel reductions: no `final`; output q (one per stage) holds post_q(fold_q) of every row.
  bool store_scalars = false;
};

std::string row_signature(const RowSpec& s);
std::string row_source(const RowSpec& s);
struct RowArgs {
  std::vector<void*> ptrs;                        // inputs..., out (store_scalars: one out per stage)[, the parts of a split row][, slots, give-up count of a team]
  uint32_t nrows;
  uint32_t nvec = 0;                              // ragged and streamed kernels only: vectors per row
  uint32_t parts = 0, chunk = 0;                  // split kernels: parts per row, vectors per part; team kernels: parts
  uint32_t spin = 0;                              // team kernels: polls a lane may spend waiting over the whole kernel
  std::vector<uint32_t> oshape;
  std::vector<uint32_t> offsets;                  // per operand incl. outputs
  std::vector<std::vector<uint32_t>> ostrides;    // per operand incl. outputs, per outer dim
  std::vector<float> consts;                      // stage 0 pre, stage 0 post, stage 1 pre, ..., final
};
std::vector<unsigned char> row_pack_args(const RowSpec& s, const RowArgs& a);

// ---- GEMM ----------------------------------------------------------------------
// K4 of the reference (src/matmul.rs:56-155) re-designed for MFMA: hand-written
// kernels (kernels/gemm_*.hip.inc), chosen by dtype and by whether the shape is
// a multiple of the 256 x 256 x BK tile.
// The *Edge kinds are the same kernels compiled with edge handling for shapes that are not multiples of
// the tile (rows of A and B still have to start 16-byte aligned).
enum class GemmKind { MfmaF16, MfmaF32, MfmaF16Edge, MfmaF32Edge, Generic };
GemmKind gemm_pick(DType dt, size_t m, size_t n, size_t k, bool b_transposed = false);
std::string gemm_signature(GemmKind kind, DType dt);
std::string gemm_source(GemmKind kind, DType dt);

}  // namespace wkf

// The executor of the lazy graph: walks a node, applies the fusion rules and
// plans + launches one generated kernel per fused group.  Restates
// ComputeGraphInner::resolve and its helpers (src/compute_graph/resolve.rs:16-248)
// and the run_with_query methods of the reference's kernel objects.
#pragma once

#include <functional>
#include <map>
#include <set>
#include <string>
#include <tuple>
#include <vector>

#include "codegen.h"
#include "core.h"

namespace wkf {

// One kernel launch of a resolve; the analogue of a PerformanceQueries entry in
// the reference's timing map (src/compute_graph/mod.rs:275).
struct LaunchRecord {
  std::string kind;        // map | red_row | red_col | gemm
  std::string signature;   // cache key of the kernel
  std::string detail;      // human-readable launch geometry
  wkf_timer* timer = nullptr;
  uint32_t grid[3] = {1, 1, 1};
  uint32_t block[3] = {1, 1, 1};
  bool in_place = false;
};

struct Settings {
  FusionMode fusion = FusionMode::Tree;
  bool timing = true;             // record a hipEvent pair around every launch
  int map_unroll = 4;             // work items per thread in large map kernels (WKF_MAP_UNROLL overrides: 1, 2, 4, 8)
  bool reference_compat = false;  // composites keep the reference's text where it differs in value from what it means: layer_norm's weight through Tensor::broadcast (indexed by row on square inputs)
  bool exact_math = false;        // every transcendental through an f64 core (MathPolicy::Exact)
  bool map_tile_128 = true;       // transposing map kernels may take 128 x 128 tiles (WKF_MAP_TILE_128=0: always 64 x 64)
  bool math_f32 = false;          // measurement only (WKF_MATH_F32=1): map kernels take the f32 library for every transcendental, outside the 2-ulp bound of fused chains; shows what the f64 cores cost
  size_t nontemporal_bytes = size_t(32) << 20;  // map kernels moving at least this much use streaming loads/stores
  int reduce_threads = 0;         // lanes per row in row reduces; 0 = chosen from the shape (WKF_REDUCE_THREADS overrides)
  int row_threads = 0;            // lanes per row in row kernels; 0 = chosen from the shape (WKF_ROW_THREADS overrides)
  size_t map_table_min = size_t(1) << 25;  // fewest elements for which a costly map over ONE dense f16 tensor (f16 result) runs as a table lookup; 0 = never (WKF_MAP_TABLE_MIN)
  bool map_tile_vec = true;       // transposing map kernels move four elements per access where the layouts allow it (WKF_MAP_TILE_VEC=0: one)
  bool gemm_shortk = true;        // many full f16 tiles over K = 64 or 128: one workgroup per compute unit walks them (WKF_GEMM_SHORTK=0 turns it off)
  bool gemm_stream = true;        // many full f16 tiles over K = 128 to 256: one workgroup per compute unit walks them and a tile's stores leave under the next tile's MFMAs (WKF_GEMM_STREAM=0 turns it off)
  bool gemm_t128 = true;          // 128 x 128 tiles for f16 products that do not fill the chip with 256 x 256 ones (WKF_GEMM_T128=0 turns it off)
  bool gemm_dma = true;           // full f16 256 x 256 tiles load their operands from memory straight into the LDS (WKF_GEMM_DMA=0: through registers)
  bool gemm_flex = true;          // f16 products that the 256 x 256 tile spreads badly over the chip take tiles of 64 NI x 64 NJ chosen per shape (WKF_GEMM_FLEX=0 turns it off; "ni,nj,stages,slices" forces one)
  bool gemm_tail = true;          // a partly filled last round of f16 tiles runs as half tiles (WKF_GEMM_TAIL=0 turns it off)
  int skinny_tr_rows = 0;         // fewest rows of A for the MFMA decode kernel on row-major B; 0 = chosen (WKF_SKINNY_TR_ROWS overrides)
  int skinny_blocks = 0;          // workgroups the decode-sized mat_mul kernels aim for; 0 = chosen (WKF_SKINNY_BLOCKS overrides)
  int reduce_unroll = 0;          // loads in flight per lane in row reduces; 0 = chosen (WKF_REDUCE_UNROLL overrides)
  bool row_split = true;             // rows too long for a block's registers and too few to stream with a block each: one launch per stage over parts of rows (WKF_ROW_SPLIT=0: fold each reduction across the grid instead)
  bool row_team = true;              // rows too long for a block's registers that fit those of up to 256 blocks: one launch, the row read once, the blocks of a row exchange their folds and wait for each other (WKF_ROW_TEAM=0 turns it off)
  uint32_t row_team_spin = 1u << 20; // polls a lane of such a kernel may spend waiting before it gives up (the read-back then computes the tensor again without teams)
  bool row_team_test_mute = false;   // tests of that path: a kernel variant in which part 0 of every row stays silent
  int row_stream_vectors = 0;        // vectors per lane and operand in flight in the kernels that stream rows longer than a block's registers; 0 = chosen (WKF_ROW_STREAM_VECTORS)
  size_t row_stream_min_rows = 256;  // fewest rows for the one-launch kernel that streams rows longer than a block's registers (WKF_ROW_STREAM_MIN_ROWS)
};

// The iteration space of one kernel seen by all of its operands at once:
// `shape` plus one stride vector per operand.  Dimensions of size 1 are dropped
// and neighbouring dimensions are merged when every operand walks them as one.
struct Space {
  std::vector<size_t> shape;
  std::vector<std::vector<size_t>> strides;  // [operand][dim]
};

// Team row kernels count the lanes that gave up waiting for another block in one word per device.
// team_begin: before a read-back starts its launches; clears a count left by launches nobody read back.
// team_gave_up: after the read-back's download has synchronised the stream and only when its own launches
// included a team kernel; true (and the count cleared) when a lane gave up, so that the caller computes the
// tensor again without teams instead of handing that result out.
void team_begin(wkf_device* dev);
bool team_gave_up(wkf_device* dev);
// read-backs that were computed a second time for that reason, per device (tests)
uint64_t team_fallbacks(wkf_device* dev);

class Resolver {
 public:
  Resolver(wkf_device* dev, const Settings& st, std::vector<LaunchRecord>* log) : dev_(dev), st_(st), log_(log) {}
  // Entry point: materialise `root` (ComputeGraph::resolve, src/compute_graph/mod.rs:241-248).
  TensorData resolve_root(const NodeP& root);
  // Several tensors in one pass (shared sub-graphs once, sibling row reductions in one kernel).
  std::vector<TensorData> resolve_roots(const std::vector<NodeP>& roots);
  // Allocation-free mode (wkf_tensor_reduce_into): the result goes into `out`, a temporary comes from the
  // device's static scratch array (at most one, at most its size), and a kernel that this device has not loaded
  // yet is an error instead of a compilation; no launch is timed.  Anything else the graph would allocate fails.
  struct NoAlloc {
    TensorData out;
    bool out_taken = false, scratch_taken = false;
  };
  void set_noalloc(NoAlloc* na) { noalloc_ = na; }
  // whether any launch of this resolver was a team row kernel (whose result needs team_gave_up before it leaves)
  bool team_launched() const { return team_launched_; }

 private:
  TensorData resolve(const NodeP& n);
  TensorData resolve_uncached(const NodeP& n);
  // When a map kernel consumes cat([A, B], axis), the expression is built once per piece: every cat cut
  // at that seam (also below broadcasts) stands for its A (or B) and every other operand is sliced to the
  // piece's range.  Pieces of one shape then share ONE kernel with two stores.
  struct CatPiece {
    size_t axis = 0, start = 0, end = 0;
  };
  NodeP slice_through(const NodeP& n, size_t axis, size_t start, size_t end);
  struct ExprBuilder {
    const CatPiece* split = nullptr;
    bool inside_piece = false;
    Program prog;
    std::vector<TensorData> operands;
    std::map<const Node*, int> memo;
    std::vector<int> operand_value;  // value id of the Load of operand k
    int load(const TensorData& td);
    int emit(Op op, int a, int b, DType dt, bool has_const, float c);
  };

  int build(ExprBuilder& eb, const NodeP& n, int pairwise_budget);
  int pairwise_budget_for_map() const { return st_.fusion == FusionMode::Tree ? 1 << 20 : 1; }
  int pairwise_budget_for_reduce() const { return st_.fusion == FusionMode::Tree ? 1 << 20 : 0; }

  TensorData run_map(const NodeP& root);
  // Row kernels (codegen.h, RowSpec): tried first for a map whose operands include last-axis
  // reductions of the same rows broadcast back along that axis.  Returns false when the pattern
  // or the layouts do not fit; the caller then takes the ordinary path.
  struct RowBuild;
  bool try_row_kernel(const NodeP& root, TensorData* out);
  struct ReduceRoot {
    const Node* root = nullptr;         // [chain above] reduce
    const Node* reduce = nullptr;
    std::vector<const Node*> chain;     // element-wise nodes above the reduce, outermost first
  };
  bool try_parallel_reduces(const std::vector<ReduceRoot>& members, std::vector<TensorData>* outs);
  bool launch_row(RowBuild& rb, const Program* final, std::vector<TensorData>* outs);
  int row_build(RowBuild& rb, Program& prog, std::map<const Node*, int>& memo, std::map<int, int>& loads, const NodeP& n);
  TensorData run_reduce(const NodeP& reduce, const std::vector<const Node*>& post_chain);
  // One reduce launch: fold `pre(operands)` over `axis`, then (unless `raw`) round to `fold_dtype` and apply `post`.
  struct ReduceJob {
    Program pre, post;
    std::vector<TensorData> operands;  // all of one shape
    size_t axis = 0;
    ReduceOp rop = ReduceOp::Sum;
    DType fold_dtype = DType::F32;
    bool raw = false;                  // store the f32 accumulators (first launch of a split reduce)
  };
  TensorData launch_reduce(const ReduceJob& job);
  // Number of axis slices a reduce is split into (1 = one launch).
  size_t reduce_split(const ReduceJob& job, size_t nrows, size_t n);
  // Rank of the job's output iteration space after merging dimensions (the kernels take up to 3).
  size_t reduce_outer_rank(const ReduceJob& job);
  TensorData run_matmul(const NodeP& n);
  TensorData run_map_layout(const NodeP& n);
  TensorData run_resize(const NodeP& n);
  TensorData run_slice_assign(const NodeP& n);

  // out[i] = prog(operands[i]) over out.layout.shape; every operand layout has that shape.
  // `more_prog[j]` (over the same operands) is stored to `more_out[j]` by the same kernel.
  void launch_map(const Program& prog, const std::vector<TensorData>& in, const TensorData& out, bool in_place,
                  const std::vector<Program>& more_prog = {}, const std::vector<TensorData>& more_out = {});
  // A map over one dense f16 tensor with an f16 result is a function of 16 bits: from map_table_min elements on, and
  // when the program costs enough to make the kernel compute-bound, its 65536 values are computed once (by the ordinary
  // kernel, over every bit pattern; kept per device, program and constants) and the data is streamed through a
  // lookup in the LDS.  Bit-identical to the ordinary kernel by construction.  False: not applicable, nothing launched.
  bool try_map_table(const Program& prog, const std::vector<TensorData>& in, const TensorData& out, bool in_place);
  // the table of `prog` (one f16 operand, f16 result) over all 65536 bit patterns, from the device's cache or built now
  BufRef map_table_for(const Program& prog);
  // Replaces the costliest value of `prog` that depends on one f16 operand only by a table lookup (Op::Lookup) and returns
  // the table, or nothing when no value is worth it
  BufRef cut_table(Program& prog, const std::vector<TensorData>& in, size_t numel, std::string* what);
  void launch_map_tiled(MapSpec& spec, const Space& sp, const std::vector<TensorData>& in, const TensorData& out, bool in_place);
  // `result`: the buffer receives the value of a reduce node (allocation-free mode: the caller's output tensor)
  TensorData alloc(const std::vector<size_t>& shape, DType dt, bool zero, bool result = false);
  TensorData make_contiguous(const TensorData& td);
  void record(LaunchRecord&& r, wkf_kernel* k, const std::vector<unsigned char>& args);
  wkf_kernel* kernel(const std::string& sig, const std::function<std::string()>& make_body);

  wkf_device* dev_;
  NoAlloc* noalloc_ = nullptr;
  bool team_launched_ = false;
  Settings st_;
  std::vector<LaunchRecord>* log_;
  std::set<const Node*> shared_;
  std::map<const Node*, TensorData> materialized_;  // nodes with several consumers, computed once per resolve
  std::map<std::tuple<const Node*, size_t, size_t, size_t>, NodeP> sliced_;  // slice_through results (and owners of its temporary nodes)
};

}  // namespace wkf

/*
 * wkf_tensor.h -- level 1 of the C ABI: the lazy Tensor API of the reference
 * crate (`Tensor<const R, D>`, re-exported by src/lib.rs:1-11) behind opaque C
 * handles.  A Rust `Tensor<R, D>` facade binds these one-to-one through an
 * `extern "C"` block; ranks and dtypes are checked at run time where
 * the Rust types check them at compile time.
 *
 * Every op only records a node (src/tensor.rs:179-284); nothing touches the GPU
 * until wkf_tensor_materialize / wkf_tensor_as_slice.  Where the reference
 * panics (shape mismatch, bad axis ...) these return WKF_ERR_INVALID_ARG and
 * leave the message in wkf_last_error().
 *
 * Threads: graph nodes are immutable and a materialisation keeps its state to itself, so different handles
 * (also of graphs that share nodes) may be used from different threads at once; the device layer serialises
 * what reaches the stream.  One handle is for one thread at a time (a materialisation rewrites its launch list).
 *
 * Paths in comments are relative to the reference checkout.
 */
#ifndef WKF_TENSOR_H
#define WKF_TENSOR_H

#include "wkf_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct wkf_tensor wkf_tensor;
typedef struct wkf_slice wkf_slice;

/* DataTypeEnum, src/tensor.rs:69-88 */
enum { WKF_F32 = 0, WKF_F16 = 1 };

/* Element-wise functions.  tensor-with-literal: src/element_wise.rs:197-675. */
enum {
  WKF_OP_ADD_CONST = 0, /* t + c, c + t   :197-271 */
  WKF_OP_SUB_CONST = 1, /* t - c          :445-458 */
  WKF_OP_CONST_SUB = 2, /* c - t          :485-498 */
  WKF_OP_MUL_CONST = 3, /* t * c, c * t   :525-571 */
  WKF_OP_DIV_CONST = 4, /* t / c          :598-611 */
  WKF_OP_CONST_DIV = 5, /* c / t          :638-651 */
  /* unary: src/element_wise.rs:678-1380 */
  WKF_OP_EXP = 16, WKF_OP_EXP2, WKF_OP_LOG, WKF_OP_LOG2, WKF_OP_SQR, WKF_OP_SQRT, WKF_OP_SIN, WKF_OP_COS,
  WKF_OP_TAN, WKF_OP_ASIN, WKF_OP_ACOS, WKF_OP_ATAN, WKF_OP_SINH, WKF_OP_COSH, WKF_OP_TANH, WKF_OP_ASINH,
  WKF_OP_ACOSH, WKF_OP_ATANH, WKF_OP_ABS, WKF_OP_NEG,
  /* pair-wise: src/pair_wise.rs:205-528 */
  WKF_OP_ADD = 64, WKF_OP_SUB, WKF_OP_MUL, WKF_OP_DIV, WKF_OP_POW
};

/* src/reduce.rs:433-815 */
enum { WKF_REDUCE_SUM = 0, WKF_REDUCE_MAX = 1, WKF_REDUCE_MIN = 2, WKF_REDUCE_PRODUCT = 3 };

/* Which fusion rules the executor applies on this device.
 * WKF_FUSION_REFERENCE: exactly src/compute_graph/resolve.rs:49-196 (element-wise
 *   chains fuse into one kernel, into the two operands and the result of ONE
 *   pair-wise op, and before/after a reduce; nothing else fuses; a node used
 *   twice is computed twice).
 * WKF_FUSION_TREE (default): additionally whole pair-wise trees, and the copies
 *   of resize / slice_assign, fuse with the element-wise work around them, and a
 *   node used twice is computed once.  Every op is still rounded on its own, so
 *   results are identical to the reference rules. */
enum { WKF_FUSION_REFERENCE = 0, WKF_FUSION_TREE = 1 };
int wkf_device_set_fusion(wkf_device* dev, int mode);
int wkf_device_get_fusion(wkf_device* dev);

/* Accuracy of exp / sin / cos and the other transcendental ops (no reference
 * counterpart: the reference leaves them to the WGSL driver, which only bounds
 * them, e.g. exp to 3 + 2|x| ulp).
 * Default (0): an op whose value feeds further arithmetic of the same kernel is
 *   evaluated in f64 and rounded once (it equals the correctly rounded f32 value,
 *   so later ops cannot amplify an error); the last op before a store uses the
 *   f32 library (<= 1-2 ulp); values that only feed a reduction use the f32 library.
 * exact != 0: every transcendental op is evaluated in f64 and rounded once. */
int wkf_device_set_exact_math(wkf_device* dev, int exact);

/* Rows longer than one workgroup's registers (no reference counterpart: the reference's reduce takes a row of any
 * length in one workgroup, src/reduce.rs:340-350, and its composites read such a row once per stage).  Here a row
 * that fits the registers of up to 256 workgroups is computed in ONE launch that reads it once: the workgroups of
 * a row exchange their folded values through memory and wait for each other (all of them are resident: the grid
 * never exceeds what the kernel's registers and the chip's compute units hold).  The wait is bounded: a lane polls
 * at most `spin_polls` times over the whole kernel (low 31 bits; 0 = the default, 2^20) and then gives up, which
 * the kernel counts.  wkf_tensor_as_slice / _as_slice_many read that count after their download whenever their own
 * launches included such a kernel; when it is not zero they compute the tensor a second time with teams off
 * (one launch per stage, or one workgroup streaming each row) and hand out that result, so a GPU shared with
 * other work costs time, never a wrong or refused result.  The top bit of `spin_polls` selects a kernel variant
 * for tests of that path, in which one workgroup per row never publishes its value.  enabled = 0 turns teams off.
 * wkf_device_row_team_fallbacks: how many read-backs of this device were computed a second time. */
int wkf_device_set_row_teams(wkf_device* dev, int enabled, uint32_t spin_polls);
int wkf_device_row_team_fallbacks(wkf_device* dev, uint64_t* out);

/* Where a composite of the reference differs IN VALUE from what it means, this library computes what it means; with
 * `enabled` != 0 tensors built afterwards on this device follow the reference's text instead.  One case today:
 * layer_norm (src/composite/rms_norm.rs:13-14) broadcasts its weight with Tensor::broadcast, which puts the new
 * dimension where the shapes first differ (src/map_layout.rs:69-77); for a square input (rows == hidden) that is
 * position 1, so the weight is indexed by ROW.  Off by default (RMSNorm as meant: the weight along the last dimension). */
int wkf_device_set_reference_compat(wkf_device* dev, int enabled);

/* Maps over f16 as table lookups (no reference counterpart).  An element-wise kernel whose only operand is ONE dense
 * f16 tensor and whose result is f16 computes a function of 16 bits.  When the fused chain is costly enough to
 * make the kernel compute-bound (a transcendental function whose value feeds further arithmetic, say) and the
 * tensor has at least `min_elements` elements (default 2^25, where the lookup is about a fifth faster; below 2^24 it does not pay; 0 = never), the 65536 values are computed once by
 * the ordinary kernel over every bit pattern (kept per device, program and constants, the 32 most recent) and the
 * data is streamed through a lookup in the LDS: the same bits as the ordinary kernel, at memory speed. */
int wkf_device_set_map_table(wkf_device* dev, uint64_t min_elements);

/* Per-kernel GPU timestamps (PerformanceQueries, src/query.rs:50-126: the reference
 * attaches one to every kernel).  On by default; a caller that only wants results can
 * switch the hipEvent pair per launch off. */
int wkf_device_set_timing(wkf_device* dev, int enabled);

/* Tensor::new, src/tensor.rs:518-531 (+ IntoTensor :441-515): uploads `data`
 * (row-major, numel * sizeof(dtype) bytes) into a new leaf tensor. */
int wkf_tensor_new(wkf_device* dev, int dtype, int rank, const size_t* shape, const void* data, wkf_tensor** out);
/* Clone of a handle (Tensor: Clone, src/tensor.rs:435-442): same node. */
int wkf_tensor_clone(const wkf_tensor* t, wkf_tensor** out);
void wkf_tensor_free(wkf_tensor* t);
int wkf_tensor_rank(const wkf_tensor* t);                 /* Tensor::rank, src/tensor.rs:634-636 */
int wkf_tensor_shape(const wkf_tensor* t, size_t* out);   /* Tensor::shape, :630-632 */
int wkf_tensor_dtype(const wkf_tensor* t);                /* Tensor::datatype, :638-640 */

/* t (op) c with an f32 literal; op is one of WKF_OP_*_CONST / WKF_OP_CONST_*. */
int wkf_tensor_scalar_op(const wkf_tensor* t, int op, float c, wkf_tensor** out);
/* exp ... neg */
int wkf_tensor_unary_op(const wkf_tensor* t, int op, wkf_tensor** out);
/* Tensor::cast, src/element_wise.rs:1408-1471 (T -> T records no node). */
int wkf_tensor_cast(const wkf_tensor* t, int dtype, wkf_tensor** out);
/* add sub mul div pow; shapes and dtypes must be equal (src/pair_wise.rs:92). */
int wkf_tensor_binary_op(const wkf_tensor* a, const wkf_tensor* b, int op, wkf_tensor** out);
/* Sum::sum / Max::max / Min::min / Product::product over `axis`; rank drops by one. */
int wkf_tensor_reduce(const wkf_tensor* t, int reduce_op, size_t axis, wkf_tensor** out);
/* wkf_tensor_reduce + wkf_tensor_materialize for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc); it has no counterpart in the reference.  `t` and
 * `out` are dense tensors that hold data already (wkf_tensor_new), `out` with t's shape minus `axis` and t's dtype;
 * the result is written into out's buffer with the same kernels, launches and bits as the allocating path.  The
 * call allocates nothing on the device: no hipMalloc / hipFree, no code-object load, no event.  A reduction that is
 * folded in two launches (few outputs over a long axis) keeps its f32 partial results in a file-scope device array
 * of 1 MiB that every GPU the library runs on holds until the process ends; a reduction whose partial results need
 * more is refused with WKF_ERR_INVALID_ARG.  The kernels must be loaded already: run the allocating path once on
 * tensors of the same shape and dtype (else WKF_ERR_INVALID_ARG names the missing kernel).  Nothing in the array has
 * to start at zero (the first launch overwrites every partial result the second reads), and it keeps the last
 * call's contents.  All calls on one device share the array: calls that overlap on one device race. */
int wkf_tensor_reduce_into(const wkf_tensor* t, int reduce_op, size_t axis, wkf_tensor* out);
/* Tensor::mat_mul, src/matmul.rs:25-29: rank 2, same dtype, [M,K] x [K,N].  Beyond the reference (whose mat_mul
 * is rank 2 only): operands of equal rank > 2 are a batch, [..., M, K] x [..., K, N] -> [..., M, N] with equal
 * leading dimensions (at most 65535 matrices), one launch for all of them. */
int wkf_tensor_mat_mul(const wkf_tensor* a, const wkf_tensor* b, wkf_tensor** out);

/* Zero-copy views, src/map_layout.rs:42-98. */
int wkf_tensor_slice(const wkf_tensor* t, const size_t* starts, const size_t* ends, wkf_tensor** out);
int wkf_tensor_transpose(const wkf_tensor* t, size_t first_axis, size_t second_axis, wkf_tensor** out);
int wkf_tensor_broadcast(const wkf_tensor* t, int out_rank, const size_t* out_shape, wkf_tensor** out);
/* src/composite/narrow.rs:3-16 */
int wkf_tensor_narrow(const wkf_tensor* t, size_t axis, size_t start, size_t length, wkf_tensor** out);

/* Copies, src/resize.rs:121-145, src/composite/unsqueeze.rs:3-53. */
int wkf_tensor_resize(const wkf_tensor* t, const size_t* new_shape, wkf_tensor** out);
int wkf_tensor_reshape(const wkf_tensor* t, int new_rank, const size_t* new_shape, wkf_tensor** out);
int wkf_tensor_unsqueeze(const wkf_tensor* t, size_t axis, wkf_tensor** out);
/* src/slice_assign.rs:76-80 */
int wkf_tensor_slice_assign(const wkf_tensor* t, const size_t* starts, const size_t* ends, const wkf_tensor* value,
                            wkf_tensor** out);
/* Tensor::cat, src/composite/cat.rs:3-41 */
int wkf_tensor_cat(const wkf_tensor* const* tensors, int count, size_t dim, wkf_tensor** out);

/* Composites, src/composite/{silu,rms_norm,rope,softmax,arange}.rs */
int wkf_tensor_silu(const wkf_tensor* t, wkf_tensor** out);
/* `layer_norm` of the reference is RMSNorm: (x / sqrt(mean(x^2) + eps)) * weight, computed in f32. */
int wkf_tensor_layer_norm(const wkf_tensor* t, const wkf_tensor* weight, float eps, wkf_tensor** out);
/* rope: t [heads, seq, dim]; cos/sin [max_seq, dim/2] (duplicated on the last dim) or [max_seq, dim]. */
int wkf_tensor_rope(const wkf_tensor* t, const wkf_tensor* cos, const wkf_tensor* sin, wkf_tensor** out);
/* rank-1 softmax exactly as src/composite/softmax.rs:4-10 (no max subtraction). */
int wkf_tensor_softmax(const wkf_tensor* t, wkf_tensor** out);
/* Max-subtracted softmax over the last dim of any rank, built from the same
 * primitives (max, sub, exp, sum, div); not in the reference. */
int wkf_tensor_softmax_last_dim(const wkf_tensor* t, wkf_tensor** out);
/* arange / arange_step, src/composite/arange.rs:4-23 (host loop + upload). */
int wkf_tensor_arange(wkf_device* dev, int dtype, float start, float end, float step, wkf_tensor** out);

/* LazyTensorData::materialize, src/tensor.rs:286-288: run the graph under `t`.
 * The result stays on the device; kernels are timed with a hipEvent pair each. */
int wkf_tensor_materialize(wkf_tensor* t);
/* wkf_tensor_materialize / wkf_tensor_as_slice for several tensors of one device in ONE pass over their
 * joint graph: what they share is computed once, and reductions over the last axis of the same rows (row
 * max and row sum(exp(x - 1)) of one matrix) run as one kernel that reads the rows once -- the "parallel
 * reduces" the reference lists as to-do (README.md:20; its resolve, src/compute_graph/mod.rs:241-248,
 * takes one key per call).  Every launch of the pass is recorded on ts[0] (wkf_tensor_kernel_info).
 * as_slice_many writes n slices into out[0..n), each to be released with wkf_slice_free. */
int wkf_tensor_materialize_many(wkf_tensor** ts, int n);
int wkf_tensor_as_slice_many(wkf_tensor** ts, int n, wkf_slice** out);
/* Tensor::all_timing_information, src/tensor.rs:556-558: number of kernels the
 * last materialize launched, and for kernel `i` its elapsed time, kind and
 * cache signature. */
int wkf_tensor_kernel_count(const wkf_tensor* t);
int wkf_tensor_kernel_info(const wkf_tensor* t, int i, uint64_t* elapsed_ns, char* kind, size_t kind_cap,
                           char* signature, size_t signature_cap, char* detail, size_t detail_cap);
/* Tensor::graphvis, src/tensor.rs:641-643 -> src/compute_graph/visualize.rs:13-271: the lazy graph below `t`
 * as Graphviz DOT text (`digraph "ComputeGraph"`), one node per graph node labelled
 * `<name> ([shape] dtype) #<id>` and one edge per input, in the reference's format.  Writes at most `cap`
 * bytes (NUL-terminated) and the full length + 1 into *needed.  Materialising does not change the graph
 * (nor does it in the reference: ComputeGraph::resolve keeps every node, src/compute_graph/mod.rs:241-248). */
int wkf_tensor_graphvis(const wkf_tensor* t, char* out, size_t cap, size_t* needed);
/* The generated HIP source of a kernel signature seen by this process (for inspection and tests). */
int wkf_kernel_source(const char* signature, char* out, size_t cap, size_t* needed);

/* Layout, src/layout.rs:33-94: the view algebra in elements (offset, shape[rank], strides[rank]) as plain host
 * functions; nothing here touches a device.
 * wkf_layout_contiguous  = Layout::contiguous (:41-48): writes the row-major strides of `shape`.
 * wkf_layout_is_contiguous = Layout::is_contiguous (:58-60): *out = 1 when offset == 0 and the strides are the
 *   row-major ones of the shape, else 0 (so a slice of one element out of a [2,3] tensor is NOT contiguous).
 * wkf_layout_slice       = Layout::slice (:62-71) with ranges [begin[d], end[d]): the new offset and shape; the
 *   strides stay as they are.  end < begin or end > shape is WKF_ERR_INVALID_ARG (the reference's Range::len
 *   would give 0 for the former and it never checks the latter; a layout that points outside its buffer is
 *   refused here instead of at the kernel). */
int wkf_layout_contiguous(int rank, const size_t* shape, size_t* strides_out);
int wkf_layout_is_contiguous(int rank, size_t offset, const size_t* shape, const size_t* strides, int* out);
int wkf_layout_slice(int rank, size_t offset, const size_t* shape, const size_t* strides, const size_t* begin,
                     const size_t* end, size_t* offset_out, size_t* shape_out);

/* Tensor::as_slice, src/tensor.rs:533-554: materialise, download the WHOLE
 * buffer, and keep the layout so that strided views are decoded on the host
 * (TensorSlice, src/tensor.rs:669-855). */
int wkf_tensor_as_slice(wkf_tensor* t, wkf_slice** out);
void wkf_slice_free(wkf_slice* s);
int wkf_slice_rank(const wkf_slice* s);
int wkf_slice_dtype(const wkf_slice* s);
/* layout: offset, shape[rank], strides[rank], all in elements */
int wkf_slice_layout(const wkf_slice* s, size_t* offset, size_t* shape, size_t* strides);
/* Pointer to element 0 of the downloaded buffer and its size in bytes. */
const void* wkf_slice_data(const wkf_slice* s, size_t* bytes);
/* TensorSlice::get, src/tensor.rs:827-846: 0 and the element widened to f32, or
 * WKF_ERR_INVALID_ARG when an index is out of range. */
int wkf_slice_get(const wkf_slice* s, const size_t* index, float* out);

#ifdef __cplusplus
}
#endif
#endif

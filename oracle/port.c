/*
 * CPU port of the reference's kernel decomposition for the benchmark
 * configurations.  TEST / BASELINE INFRASTRUCTURE ONLY: it is the `cpu_baseline`
 * leg of bench.py (kind "port") and is itself checked against oracle/oracle.py
 * in tests/test_port.py.  The product never links or calls it.
 *
 * The reference cannot run on a CPU here (Rust + a git-pinned wgpu + a Vulkan
 * ICD, none of which exist on the box), so this file restates, in f32 with the
 * host libm and OpenMP over all cores, the SAME number of passes over memory the
 * reference's executor would launch (src/compute_graph/resolve.rs:49-196):
 *   config 1  exp(sin(x*2+1))          1 element-wise kernel   (element_wise.rs:89-164)
 *   config 2  row max ; row sum(exp(x-1))   1 reduce kernel each (reduce.rs:283-386)
 *   config 3  silu(a) * (b + bias)     3 pair-wise kernels      (pair_wise.rs:86-177)
 *   config 4  RMSNorm = 1 reduce + 2 pair-wise (composite/rms_norm.rs:8-15);
 *             RoPE and softmax as their primitive sequences
 *   config 5  GEMM: a blocked f32 loop (f16 inputs widened by the caller)
 */
#include <math.h>
#include <stddef.h>
#include <string.h>

#define MAX_SEED (-3.40282e+38f) /* src/reduce.rs:640 */

int port_threads(void);

#ifdef _OPENMP
#include <omp.h>
int port_threads(void) { return omp_get_max_threads(); }
#else
int port_threads(void) { return 1; }
#endif

/* config 1: multiply_const, add_const, sin, exp fused into one pass */
void port_c1(const float* x, float* y, size_t n) {
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; i++) {
    float v = x[i] * 2.0f;
    v = v + 1.0f;
    v = sinf(v);
    y[i] = expf(v);
  }
}

/* config 2a: max over axis 1 */
void port_row_max(const float* x, float* out, size_t rows, size_t cols) {
#pragma omp parallel for schedule(static)
  for (size_t r = 0; r < rows; r++) {
    float m = MAX_SEED;
    const float* p = x + r * cols;
    for (size_t c = 0; c < cols; c++) m = fmaxf(p[c], m);
    out[r] = m;
  }
}

/* config 2b: sum over axis 1 with the fused prologue [subtract_const 1, exp] */
void port_row_sum_exp_sub(const float* x, float* out, size_t rows, size_t cols, float c0) {
#pragma omp parallel for schedule(static)
  for (size_t r = 0; r < rows; r++) {
    float s = 0.0f;
    const float* p = x + r * cols;
    for (size_t c = 0; c < cols; c++) s = expf(p[c] - c0) + s;
    out[r] = s;
  }
}

/* config 3, as the reference runs it: (1) t1 = a / (1 + exp(-a)); (2) t2 = b + bias (strided);
 * (3) t1 = t1 * t2 in place.  outer = 32*1024 rows, inner = 4096. */
void port_c3(const float* a, const float* b, const float* bias, float* t1, float* t2, size_t outer, size_t inner) {
  const size_t n = outer * inner;
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; i++) {
    float e = expf(-a[i]);
    t1[i] = a[i] / (1.0f + e);
  }
#pragma omp parallel for schedule(static)
  for (size_t r = 0; r < outer; r++)
    for (size_t c = 0; c < inner; c++) t2[r * inner + c] = b[r * inner + c] + bias[c];
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; i++) t1[i] = t1[i] * t2[i];
}

/* config 4 RMSNorm: reduce(pre sqr; post /H, +eps, sqrt) -> [rows]; x / rms (strided); * weight (strided) */
void port_rmsnorm(const float* x, const float* w, float eps, float* rms, float* out, size_t rows, size_t hidden) {
#pragma omp parallel for schedule(static)
  for (size_t r = 0; r < rows; r++) {
    float s = 0.0f;
    for (size_t c = 0; c < hidden; c++) s = x[r * hidden + c] * x[r * hidden + c] + s;
    rms[r] = sqrtf(s / (float)hidden + eps);
  }
#pragma omp parallel for schedule(static)
  for (size_t r = 0; r < rows; r++)
    for (size_t c = 0; c < hidden; c++) out[r * hidden + c] = x[r * hidden + c] / rms[r];
#pragma omp parallel for schedule(static)
  for (size_t r = 0; r < rows; r++)
    for (size_t c = 0; c < hidden; c++) out[r * hidden + c] = out[r * hidden + c] * w[c];
}

/* config 4 RoPE (non-interleaved): rot = cat(-x2, x1) materialised, then x*cos + rot*sin.
 * x [heads, seq, dim], cos/sin [seq, dim] (already full width). */
void port_rope(const float* x, const float* cs, const float* sn, float* rot, float* out, size_t heads, size_t seq, size_t dim) {
  const size_t half = dim / 2, rows = heads * seq;
#pragma omp parallel for schedule(static)
  for (size_t r = 0; r < rows; r++) {
    for (size_t c = 0; c < half; c++) rot[r * dim + c] = -x[r * dim + half + c];
    for (size_t c = 0; c < half; c++) rot[r * dim + half + c] = x[r * dim + c];
  }
#pragma omp parallel for schedule(static)
  for (size_t r = 0; r < rows; r++) {
    const size_t pos = r % seq;
    for (size_t c = 0; c < dim; c++) {
      float p = x[r * dim + c] * cs[pos * dim + c];
      float q = rot[r * dim + c] * sn[pos * dim + c];
      out[r * dim + c] = p + q;
    }
  }
}

/* config 4 softmax over the last dim from the primitives: max; sum(exp(x - max)); exp(x - max) / sum */
void port_softmax_rows(const float* x, float* mx, float* sm, float* out, size_t rows, size_t cols) {
  port_row_max(x, mx, rows, cols);
#pragma omp parallel for schedule(static)
  for (size_t r = 0; r < rows; r++) {
    float s = 0.0f;
    for (size_t c = 0; c < cols; c++) s = expf(x[r * cols + c] - mx[r]) + s;
    sm[r] = s;
  }
#pragma omp parallel for schedule(static)
  for (size_t r = 0; r < rows; r++)
    for (size_t c = 0; c < cols; c++) out[r * cols + c] = expf(x[r * cols + c] - mx[r]) / sm[r];
}

/* config 5: C = A B, f32, blocked; not a BLAS call */
void port_gemm_f32(const float* a, const float* b, float* c, size_t m, size_t n, size_t k) {
  enum { TM = 64, TN = 256, TK = 64 };
#pragma omp parallel for collapse(2) schedule(static)
  for (size_t i0 = 0; i0 < m; i0 += TM)
    for (size_t j0 = 0; j0 < n; j0 += TN) {
      const size_t i1 = i0 + TM < m ? i0 + TM : m, j1 = j0 + TN < n ? j0 + TN : n;
      for (size_t i = i0; i < i1; i++) memset(c + i * n + j0, 0, (j1 - j0) * sizeof(float));
      for (size_t k0 = 0; k0 < k; k0 += TK) {
        const size_t k1 = k0 + TK < k ? k0 + TK : k;
        for (size_t i = i0; i < i1; i++)
          for (size_t kk = k0; kk < k1; kk++) {
            const float av = a[i * k + kk];
            const float* bp = b + kk * n;
            float* cp = c + i * n;
            for (size_t j = j0; j < j1; j++) cp[j] += av * bp[j];
          }
      }
    }
}

"""The typed C++ facade (include/wkf_tensor.hpp: `wkf::Tensor<R, D>`, the shape of the reference's
`Tensor<const R, D>`, src/tensor.rs:418-644) compiled with the host compiler and linked against the library.

Without a GPU the program runs on the plan-only device: it checks the compile-time ranks and element types of every
method's result, the f16 conversions of the header, the plans (which kernels a graph becomes) and the error path.
On a GPU the same program computes the expressions of the reference's own tests (literal inputs and expected values as
in src/element_wise.rs:1473-1530, src/reduce.rs:817-1000, src/matmul.rs:207-318, src/map_layout.rs:101-260,
src/composite/*.rs) and compares."""
import os
import shutil
import subprocess
import textwrap

import pytest

from helpers import ROOT

PROGRAM = textwrap.dedent(r"""
    #include <cmath>
    #include <cstdio>
    #include <type_traits>
    #include "wkf_tensor.hpp"

    using wkf::Device; using wkf::Tensor; using wkf::F32; using wkf::F16; using wkf::Half; using wkf::Range;

    static int failures = 0, checks = 0;
    static void expect(bool ok, const char* what) { checks++; if (!ok) { failures++; std::printf("FAIL %s\n", what); } }
    static bool close(const std::vector<float>& got, std::initializer_list<float> want, float tol) {
      if (got.size() != want.size()) return false;
      size_t i = 0;
      for (float w : want) { if (!(std::fabs(got[i] - w) <= tol * (1.0f + std::fabs(w)))) { std::printf("  [%zu] got %g want %g\n", i, got[i], w); return false; } i++; }
      return true;
    }

    // On a GPU: read the tensor back and compare.  On the plan-only device: plan and compile its kernels, nothing to compare.
    static bool on_gpu = false;
    template <class T> static void verify(const T& t, std::initializer_list<float> want, float tol, const char* what) {
      if (!on_gpu) { t.materialize(); expect(true, what); return; }
      expect(close(t.as_slice().to_floats(), want, tol), what);
    }

    // ranks and element types are part of the type: these hold at compile time
    template <class T, int R, class D> constexpr bool is_tensor = std::is_same<T, Tensor<R, D>>::value;

    int main(int argc, char** argv) {
      const bool gpu = argc > 1 && std::string(argv[1]) == "gpu";
      on_gpu = gpu;
      try {
        Device dev = gpu ? Device::create(0) : Device::planner();
        auto x = Tensor<2, F32>::from_floats(dev, {3, 2}, {1, 2, 3, 4, 5, 6});
        static_assert(is_tensor<decltype(x + 1.0f), 2, F32>, "t + c");
        static_assert(is_tensor<decltype(1.0f - x), 2, F32>, "c - t");
        static_assert(is_tensor<decltype(-x), 2, F32>, "-t");
        static_assert(is_tensor<decltype(x.sum(0)), 1, F32>, "a reduce drops one dimension");
        static_assert(is_tensor<decltype(x.sum(0).max(0)), 0, F32>, "down to rank 0");
        static_assert(is_tensor<decltype(x.cast<F16>()), 2, F16>, "cast changes the element type");
        static_assert(is_tensor<decltype(x.unsqueeze(0)), 3, F32>, "unsqueeze adds a dimension");
        static_assert(is_tensor<decltype(x.reshape<1>({6})), 1, F32>, "reshape names its rank");
        static_assert(is_tensor<decltype(x.sum(1).broadcast<2>({3, 2})), 2, F32>, "broadcast names its rank");
        static_assert(is_tensor<decltype(x.mat_mul(x.transpose(0, 1))), 2, F32>, "mat_mul keeps the rank");
        static_assert(is_tensor<decltype(x * x + x), 2, F32>, "tensor with tensor");

        // f16 conversions of the header: every bit pattern survives the round trip, ties go to even
        bool round_trip = true;
        for (unsigned b = 0; b < 65536; b++) {
          const Half h{uint16_t(b)};
          const bool nan = ((b >> 10) & 31u) == 31u && (b & 0x3ffu) != 0;
          if (!nan && Half::from_float(h.to_float()).bits != b) round_trip = false;
        }
        expect(round_trip, "f16 round trip");
        expect(Half::from_float(1.0f + 0x1p-11f).bits == 0x3c00 && Half::from_float(1.0f + 0x1.8p-10f).bits == 0x3c02, "ties to even");
        expect(Half::from_float(65520.0f).bits == 0x7c00 && Half::from_float(65519.0f).bits == 0x7bff, "overflow boundary");
        expect(Half::from_float(0x1p-25f).bits == 0 && Half::from_float(0x1.000002p-25f).bits == 1, "underflow boundary");

        // the nested-literal constructors build the same tensors as shape + flat data
        {
          auto n2 = Tensor<2, F32>::from(dev, {{1, 2}, {3, 4}, {5, 6}});
          auto n3 = Tensor<3, F16>::from(dev, {{{1, 2, 3}}, {{4, 5, 6}}});
          auto n1 = Tensor<1, F32>::from(dev, {7, 8, 9});
          expect(n2.shape()[0] == 3 && n2.shape()[1] == 2 && n3.shape()[0] == 2 && n3.shape()[1] == 1 && n3.shape()[2] == 3 && n1.shape()[0] == 3, "nested literals: shapes");
          expect(n2.as_slice()[{2, 0}] == 5.0f && n3.as_slice()[{1, 0, 2}] == 6.0f && n1.as_slice()[{1}] == 8.0f, "nested literals: values");
          bool ragged = false;
          try { Tensor<2, F32>::from(dev, {{1, 2}, {3}}); } catch (const wkf::Error& e) { ragged = e.code == WKF_ERR_INVALID_ARG; }
          expect(ragged, "ragged literal throws");
        }

        // shapes travel with the graph
        auto s = ((x * 2.0f) + 1.0f).sum(1);
        expect(s.shape()[0] == 3, "shape of a reduce");
        expect(x.graphvis().find("digraph") != std::string::npos, "graphvis");
        s.materialize();
        auto info = s.all_timing_information();
        expect(info.size() == 1 && info[0].kind == "red_row" && info[0].signature.find("multiply_const") != std::string::npos,
               "(x * 2 + 1).sum(1) is one reduce kernel with the chain fused in");
        // the reference panics on a bad axis; here an exception with the message
        bool threw = false;
        try { x.sum(5); } catch (const wkf::Error& e) { threw = e.code == WKF_ERR_INVALID_ARG && std::string(e.what()).size() > 0; }
        expect(threw, "bad axis throws");
        threw = false;
        try { x.mat_mul(x); } catch (const wkf::Error& e) { threw = e.code == WKF_ERR_INVALID_ARG; }
        expect(threw, "[3,2] x [3,2] throws");

        if (!gpu) {
          bool refused = false;
          try { s.as_slice(); } catch (const wkf::Error& e) { refused = e.code == WKF_ERR_NO_DEVICE; }
          expect(refused, "no GPU: reading a computed tensor is refused");
          auto leaf = x.as_slice();   // a leaf is host data on this device
          expect(leaf[{2, 1}] == 6.0f, "leaf read-back");
        }
        {
          // element-wise with literals and unary ops (src/element_wise.rs tests: [[1,2],[3,4],[5,6]])
          verify((x + 1.0f), {2, 3, 4, 5, 6, 7}, 0, "x + 1");
          verify((1.0f - x), {0, -1, -2, -3, -4, -5}, 0, "1 - x");
          verify((x / 2.0f), {0.5f, 1, 1.5f, 2, 2.5f, 3}, 0, "x / 2");
          verify((2.0f / x), {2, 1, 2.0f / 3, 0.5f, 0.4f, 1.0f / 3}, 1e-6f, "2 / x");
          verify((-x).abs().sqrt(), {1, std::sqrt(2.0f), std::sqrt(3.0f), 2, std::sqrt(5.0f), std::sqrt(6.0f)}, 1e-6f, "sqrt(abs(-x))");
          verify(((x * 2.0f) + 1.0f).sin().exp(),
                 {std::exp(std::sin(3.0f)), std::exp(std::sin(5.0f)), std::exp(std::sin(7.0f)), std::exp(std::sin(9.0f)), std::exp(std::sin(11.0f)), std::exp(std::sin(13.0f))}, 1e-6f, "exp(sin(2x+1))");
          // tensor with tensor
          verify((x * x - x), {0, 2, 6, 12, 20, 30}, 0, "x*x - x");
          verify(x.pow(x), {1, 4, 27, 256, 3125, 46656}, 1e-5f, "x^x");
          // reductions (src/reduce.rs tests)
          verify(x.sum(0), {9, 12}, 0, "sum(0)");
          verify(x.sum(1), {3, 7, 11}, 0, "sum(1)");
          verify(x.max(1), {2, 4, 6}, 0, "max(1)");
          verify(x.min(0), {1, 2}, 0, "min(0)");
          verify(x.product(1), {2, 12, 30}, 0, "product(1)");
          verify(s, {8, 16, 24}, 0, "(2x+1).sum(1)");
          verify(x.sum(0).sum(0), {21}, 0, "rank 0");
          // mat_mul (src/matmul.rs:268-318 compares with the textbook product)
          auto a = Tensor<2, F32>::from_floats(dev, {2, 3}, {1, 2, 3, 4, 5, 6});
          verify(a.mat_mul(x), {22, 28, 49, 64}, 0, "[2,3] x [3,2]");
          verify(x.mat_mul(x.transpose(0, 1)), {5, 11, 17, 11, 25, 39, 17, 39, 61}, 0, "x x^T");
          // views and copies (src/map_layout.rs, src/resize.rs, src/slice_assign.rs tests)
          verify(x.slice({Range{0, 2}, Range{0, 1}}), {1, 3}, 0, "slice");
          verify(x.transpose(0, 1), {1, 3, 5, 2, 4, 6}, 0, "transpose");
          verify(x.sum(1).broadcast<2>({2, 3}), {3, 7, 11, 3, 7, 11}, 0, "broadcast");
          verify(x.narrow(0, 1, 2), {3, 4, 5, 6}, 0, "narrow");
          verify(x.resize({2, 3}), {1, 2, 0, 3, 4, 0}, 0, "resize crops and zero-fills");
          verify(x.reshape<1>({6}), {1, 2, 3, 4, 5, 6}, 0, "reshape");
          auto v = Tensor<2, F32>::from_floats(dev, {1, 2}, {9, 8});
          verify(x.slice_assign({Range{1, 2}, Range{0, 2}}, v), {1, 2, 9, 8, 5, 6}, 0, "slice_assign");
          verify(Tensor<2, F32>::cat({x, v}, 0), {1, 2, 3, 4, 5, 6, 9, 8}, 0, "cat");
          verify(Tensor<1, F32>::arange(dev, 0, 5), {0, 1, 2, 3, 4}, 0, "arange");
          // composites
          auto sig = [](float t) { return t / (1.0f + std::exp(-t)); };
          verify(x.silu(), {sig(1), sig(2), sig(3), sig(4), sig(5), sig(6)}, 1e-6f, "silu");
          auto w = Tensor<1, F32>::from_floats(dev, {2}, {1, 2});
          {
                    const float rows[3][2] = {{1, 2}, {3, 4}, {5, 6}};
            bool ok = true;
            auto ln = x.layer_norm(w, 1e-5f);
            ln.materialize();
            auto got = gpu ? ln.as_slice().to_floats() : std::vector<float>(6, 0.0f);
            for (int r = 0; r < 3 && gpu; r++) {
              const float ms = (rows[r][0] * rows[r][0] + rows[r][1] * rows[r][1]) / 2.0f, inv = 1.0f / std::sqrt(ms + 1e-5f);
              for (int c = 0; c < 2; c++) ok = ok && std::fabs(got[size_t(r * 2 + c)] - rows[r][c] * inv * float(c + 1)) < 1e-5f;
            }
            expect(ok, "layer_norm");
          }
          {
            const float e1 = std::exp(1.0f), e2 = std::exp(2.0f), e3 = std::exp(3.0f), z = e1 + e2 + e3;
            verify(Tensor<1, F32>::from_floats(dev, {3}, {1, 2, 3}).softmax(), {e1 / z, e2 / z, e3 / z}, 1e-6f, "softmax");
            const float lo = 1.0f / (1.0f + std::exp(1.0f)), hi = 1.0f / (1.0f + std::exp(-1.0f));   // every row is (t, t + 1)
            verify(x.softmax_last_dim(), {lo, hi, lo, hi, lo, hi}, 1e-6f, "softmax_last_dim");
          }
          // f16 end to end
          auto h = x.cast<F16>();
          verify(((h * 2.0f) + 1.0f), {3, 5, 7, 9, 11, 13}, 0, "f16 chain");
          verify(h.sum(1).cast<F32>(), {3, 7, 11}, 0, "f16 reduce, cast back");
          expect(x.sum(1).all_timing_information().empty(), "nothing launched before a read-back");
        }
      } catch (const wkf::Error& e) {
        std::printf("FAIL exception %d: %s\n", e.code, e.what());
        return 1;
      }
      std::printf("%s %d checks %d failures\n", failures ? "FAILED" : "OK", checks, failures);
      return failures ? 1 : 0;
    }
""")


def build(tmp_path):
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("no g++ on this machine")
    libdir = os.path.join(ROOT, "wgpu-kernal-fusion_amd")
    if not os.path.exists(os.path.join(libdir, "libwkf_hip.so")):
        pytest.fail("wgpu-kernal-fusion_amd/libwkf_hip.so is not built (bash wgpu-kernal-fusion_amd/build.sh)")
    src = tmp_path / "facade.cpp"
    src.write_text(PROGRAM)
    exe = tmp_path / "facade"
    cmd = [gxx, "-std=c++17", "-O1", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe),
           "-L", libdir, "-lwkf_hip", f"-Wl,-rpath,{libdir}"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    return exe


def test_cpp_facade_compiles_and_plans(tmp_path):
    exe = build(tmp_path)
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and r.stdout.strip().splitlines()[-1].startswith("OK "), r.stdout + r.stderr


@pytest.mark.gpu
def test_cpp_facade_computes_the_reference_examples(tmp_path):
    exe = build(tmp_path)
    if os.environ.get("WKF_TEST_PLAN_ONLY") == "1":
        r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)  # compiles the kernels into the cache
        assert r.returncode == 0, r.stdout + r.stderr
        pytest.skip("planned and compiled without a GPU; nothing was computed")
    r = subprocess.run([str(exe), "gpu"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and r.stdout.strip().splitlines()[-1].startswith("OK "), r.stdout + r.stderr

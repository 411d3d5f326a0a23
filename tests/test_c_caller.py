"""The C ABI used from plain C: the headers compile as C99 and a small C program linked against the
library builds a lazy expression, has it planned on a device without a GPU, and reads the plan back.
(No compute: that needs a GPU and is covered by the GPU parity tests through the same entry points.)"""
import os
import shutil
import subprocess
import textwrap

import pytest

from helpers import ROOT

PROGRAM = textwrap.dedent(r"""
    #include <stdio.h>
    #include <string.h>
    #include "wkf_hip.h"
    #include "wkf_tensor.h"

    #define CHECK(call) do { int rc_ = (call); if (rc_ != WKF_OK) { printf("FAIL %s -> %d: %s\n", #call, rc_, wkf_last_error()); return 1; } } while (0)

    int main(void) {
      wkf_device* dev = NULL;
      CHECK(wkf_device_create_planner(&dev));
      wkf_props props;
      CHECK(wkf_device_props(dev, &props));
      float data[6] = {1, 2, 3, 4, 5, 6};
      size_t shape[2] = {3, 2};
      wkf_tensor *x = NULL, *y = NULL, *z = NULL, *s = NULL;
      CHECK(wkf_tensor_new(dev, WKF_F32, 2, shape, data, &x));
      CHECK(wkf_tensor_scalar_op(x, WKF_OP_MUL_CONST, 2.0f, &y));          /* (x * 2 + 1).sum(1): one fused reduce kernel */
      CHECK(wkf_tensor_scalar_op(y, WKF_OP_ADD_CONST, 1.0f, &z));
      CHECK(wkf_tensor_reduce(z, WKF_REDUCE_SUM, 1, &s));
      size_t out_shape[4];
      if (wkf_tensor_rank(s) != 1) { printf("FAIL rank\n"); return 1; }
      CHECK(wkf_tensor_shape(s, out_shape));
      CHECK(wkf_tensor_materialize(s));
      char kind[32], sig[512], detail[256];
      uint64_t ns = 0;
      int n = wkf_tensor_kernel_count(s);
      CHECK(wkf_tensor_kernel_info(s, 0, &ns, kind, sizeof kind, sig, sizeof sig, detail, sizeof detail));
      printf("arch=%s wave=%d rows=%zu kernels=%d kind=%s pre=%d\n", props.arch, props.wave_size, out_shape[0], n, kind,
             strstr(sig, "multiply_const") && strstr(sig, "add_const"));
      wkf_slice* sl = NULL;
      int rc = wkf_tensor_as_slice(s, &sl);                                   /* no GPU: refused with a status code */
      printf("as_slice=%d\n", rc);
      wkf_slice* leaf = NULL;
      CHECK(wkf_tensor_as_slice(x, &leaf));                                  /* a leaf is host data on this device */
      size_t idx[2] = {2, 1};
      float v = 0;
      CHECK(wkf_slice_get(leaf, idx, &v));
      printf("leaf[2][1]=%g\n", v);
      wkf_tensor* bad = NULL;
      printf("axis_error=%d\n", wkf_tensor_reduce(x, WKF_REDUCE_SUM, 5, &bad));
      wkf_slice_free(leaf);
      wkf_tensor_free(s); wkf_tensor_free(z); wkf_tensor_free(y); wkf_tensor_free(x);
      wkf_device_destroy(dev);
      return 0;
    }
""")


@pytest.mark.skipif(shutil.which("gcc") is None, reason="no C compiler")
def test_headers_are_c99_and_a_c_program_drives_the_abi(wkf, tmp_path):
    inc = os.path.join(ROOT, "include")
    for header in ("wkf_hip.h", "wkf_tensor.h"):
        subprocess.check_call(["gcc", "-std=c99", "-fsyntax-only", "-Wall", "-Wextra", "-pedantic", "-x", "c", "-I", inc,
                               os.path.join(inc, header)])
    src = tmp_path / "caller.c"
    src.write_text(PROGRAM)
    exe = tmp_path / "caller"
    libdir = os.path.dirname(wkf.LIB_PATH)
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-I", inc, str(src), "-o", str(exe), "-L", libdir, "-lwkf_hip",
                           "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib"])
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    lines = out.stdout.strip().splitlines()
    assert lines[0] == "arch=gfx950 wave=64 rows=3 kernels=1 kind=red_row pre=1"
    assert lines[1] == "as_slice=5"      # WKF_ERR_NO_DEVICE
    assert lines[2] == "leaf[2][1]=6"
    assert lines[3] == "axis_error=3"    # WKF_ERR_INVALID_ARG

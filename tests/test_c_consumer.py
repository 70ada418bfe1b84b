"""The boundary as a C program sees it: `include/mlu_op.h` and `include/mlu_op_ext.h` compile as
strict C99 and as C++17, and a C program linked against the shared library walks the reference's
call sequence (handle, descriptors, workspace query, operator) with a handle that has no device:
every check runs, and the operator stops with EXECUTION_FAILED where it would launch."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")
LIBDIR = os.path.join(ROOT, "mlu-ops_amd", "lib")

PROGRAM = r"""
#include <stdio.h>
#include <string.h>
#include "mlu_op.h"
#include "mlu_op_ext.h"

#define EXPECT(call, want)                                                       \
  do {                                                                           \
    mluOpStatus_t s_ = (call);                                                   \
    if (s_ != (want)) {                                                          \
      printf("line %d: %s gave %s\n", __LINE__, #call, mluOpGetErrorString(s_)); \
      return 1;                                                                  \
    }                                                                            \
  } while (0)

static int tensor(mluOpTensorDescriptor_t *d, mluOpDataType_t t, int n, const int *dims) {
  if (mluOpCreateTensorDescriptor(d) != MLUOP_STATUS_SUCCESS) return 1;
  return mluOpSetTensorDescriptor(*d, MLUOP_LAYOUT_ARRAY, t, n, dims) != MLUOP_STATUS_SUCCESS;
}

int main(void) {
  int major = -1, minor = -1, patch = -1;
  size_t bytes = 0, ws = 0;
  mluOpHandle_t handle = NULL;
  mluOpQueue_t queue = (mluOpQueue_t)0x1;
  mluOpSparseConvolutionDescriptor_t conv = NULL;
  mluOpTensorDescriptor_t indices, pairs, out_indices, num;
  const int L = 1000, K = 27;
  const int d_indices[2] = {1000, 4}, d_pairs[3] = {27, 2, 1000}, d_num[1] = {27};
  const int pad[3] = {1, 1, 1}, one[3] = {1, 1, 1}, space[3] = {16, 32, 32}, filter[3] = {3, 3, 3};
  int num_act_out = -1;
  char fake[64];

  mluOpGetLibVersion(&major, &minor, &patch);
  if (major < 0 || minor < 0 || patch < 0) return 2;
  EXPECT(mluOpGetSizeOfDataType(MLUOP_DTYPE_HALF, &bytes), MLUOP_STATUS_SUCCESS);
  if (bytes != 2) return 3;
  if (strlen(mluOpGetErrorString(MLUOP_STATUS_BAD_PARAM)) == 0) return 4;

  EXPECT(mluOpCreate(&handle), MLUOP_STATUS_SUCCESS);
  EXPECT(mluOpGetQueue(handle, &queue), MLUOP_STATUS_SUCCESS);
  if (queue != NULL) return 5;

  EXPECT(mluOpCreateSparseConvolutionDescriptor(&conv), MLUOP_STATUS_SUCCESS);
  EXPECT(mluOpSetSparseConvolutionDescriptor(conv, 5, 1, pad, one, one, space, filter, space, 1, 0, 0),
         MLUOP_STATUS_SUCCESS);
  EXPECT(mluOpSetSparseConvolutionDescriptor(conv, 4, 1, pad, one, one, space, filter, space, 1, 0, 0),
         MLUOP_STATUS_BAD_PARAM);
  if (tensor(&indices, MLUOP_DTYPE_INT32, 2, d_indices) || tensor(&pairs, MLUOP_DTYPE_INT32, 3, d_pairs) ||
      tensor(&out_indices, MLUOP_DTYPE_INT32, 2, d_indices) || tensor(&num, MLUOP_DTYPE_INT32, 1, d_num))
    return 6;
  if (mluOpGetTensorElementNum(pairs) != (size_t)K * 2 * L) return 7;

  EXPECT(mluOpGetIndicePairsWorkspaceSize(handle, conv, indices, pairs, out_indices, num, &ws),
         MLUOP_STATUS_SUCCESS);
  if (ws == 0) return 8;
  EXPECT(mluOpGetIndicePairsWorkspaceSize(handle, conv, indices, pairs, out_indices, num, NULL),
         MLUOP_STATUS_BAD_PARAM);
  /* NULL data pointer: refused by the checks before anything would launch */
  EXPECT(mluOpGetIndicePairs(handle, conv, indices, NULL, fake, ws, pairs, fake, out_indices, fake, num, fake),
         MLUOP_STATUS_BAD_PARAM);
  /* all checks pass; this handle has no device, so the launch point reports it */
  EXPECT(mluOpGetIndicePairs(handle, conv, indices, fake, fake, ws, pairs, fake, out_indices, fake, num, fake),
         MLUOP_STATUS_EXECUTION_FAILED);
  EXPECT(mluOpGetSparseConvolutionNumActOut(conv, &num_act_out), MLUOP_STATUS_SUCCESS);

  EXPECT(mluOpExtSetSparseConvExtendedModes(handle, 1), MLUOP_STATUS_SUCCESS);
  EXPECT(mluOpExtSetDistinctPairsPromise(handle, 1), MLUOP_STATUS_SUCCESS);
  EXPECT(mluOpExtGetRowMapSize(pairs, L, &bytes), MLUOP_STATUS_SUCCESS);
  if (bytes < (size_t)K * L * 4) return 9;
  EXPECT(mluOpExtUseRowMap(handle, fake), MLUOP_STATUS_BAD_PARAM);
  EXPECT(mluOpExtForgetRowMap(handle, NULL), MLUOP_STATUS_SUCCESS);

  EXPECT(mluOpDestroyTensorDescriptor(indices), MLUOP_STATUS_SUCCESS);
  EXPECT(mluOpDestroyTensorDescriptor(pairs), MLUOP_STATUS_SUCCESS);
  EXPECT(mluOpDestroyTensorDescriptor(out_indices), MLUOP_STATUS_SUCCESS);
  EXPECT(mluOpDestroyTensorDescriptor(num), MLUOP_STATUS_SUCCESS);
  EXPECT(mluOpDestroySparseConvolutionDescriptor(conv), MLUOP_STATUS_SUCCESS);
  EXPECT(mluOpDestroy(handle), MLUOP_STATUS_SUCCESS);
  printf("boundary ok %d.%d.%d workspace %lu\n", major, minor, patch, (unsigned long)ws);
  return 0;
}
"""


def run(cmd, **kw):
    return subprocess.run(cmd, capture_output=True, text=True, timeout=120, **kw)


@pytest.mark.skipif(shutil.which("gcc") is None, reason="no C compiler")
def test_headers_are_strict_c99_and_cxx17(tmp_path):
    src = tmp_path / "headers.c"
    src.write_text('#include "mlu_op.h"\n#include "mlu_op_ext.h"\nint main(void) { return 0; }\n')
    r = run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I", INCLUDE, str(src)])
    assert r.returncode == 0, r.stderr
    r = run(["g++", "-std=c++17", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-x", "c++",
             "-I", INCLUDE, str(src)])
    assert r.returncode == 0, r.stderr


@pytest.mark.skipif(shutil.which("gcc") is None, reason="no C compiler")
def test_c_program_walks_the_call_sequence(tmp_path):
    lib = os.environ.get("MLUOP_LIBRARY") or os.path.join(LIBDIR, "libmluops.so")
    if not os.path.exists(lib):
        pytest.fail("%s is not built" % lib)
    src, exe = tmp_path / "consumer.c", tmp_path / "consumer"
    src.write_text(PROGRAM)
    r = run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-I", INCLUDE, str(src), "-o", str(exe),
             lib, "-Wl,-rpath," + os.path.dirname(lib), "-Wl,--allow-shlib-undefined"])
    assert r.returncode == 0, r.stderr
    env = dict(os.environ, MLUOP_HOST_ONLY_HANDLE="1")
    r = run([str(exe)], env=env)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)
    assert r.stdout.startswith("boundary ok"), r.stdout

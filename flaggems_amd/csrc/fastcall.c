/* Low-overhead Python binding of the decode-critical C-ABI entry points (CPython C API, no PyTorch).
 *
 * ctypes converts every argument of a call through its foreign-function machinery: for the 21 arguments of
 * fg_block_fp8_gemm that is 2-3 us per call, as long as a decode-sized kernel runs.  The reference has the same
 * concern and answers it with a leaner C++ wrapper (cpp/lib/fp8_matmul_direct.cpp:25-180, motivation at :62-63).
 * Here the Python host passes the address of the C function (taken once from the loaded shared library) followed
 * by its arguments as Python ints / floats / None, and this module calls it: METH_FASTCALL, one PyLong conversion
 * per argument, no allocation.
 *
 * Built by flaggems_amd/build.py with the host compiler next to libflaggems_amd.so; it links nothing of the library
 * (the function pointers come in as arguments), so it loads on a host without a GPU as well.
 */
#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <stdint.h>

/* Python int (or None = 0) -> 64-bit value; pointers and sizes arrive as non-negative ints */
static int as_u64(PyObject* o, uint64_t* out) {
  if (o == Py_None) { *out = 0; return 0; }
  unsigned long long v = PyLong_AsUnsignedLongLongMask(o);
  if (v == (unsigned long long)-1 && PyErr_Occurred()) return -1;
  *out = (uint64_t)v;
  return 0;
}
static int as_i64(PyObject* o, int64_t* out) {
  long long v = PyLong_AsLongLong(o);
  if (v == -1 && PyErr_Occurred()) return -1;
  *out = (int64_t)v;
  return 0;
}
static int as_f32(PyObject* o, float* out) {
  double v = PyFloat_AsDouble(o);
  if (v == -1.0 && PyErr_Occurred()) return -1;
  *out = (float)v;
  return 0;
}

#define NEED(n)                                                                                    \
  if (nargs != (n)) {                                                                              \
    PyErr_Format(PyExc_TypeError, "%s: expected %d arguments, got %zd", __func__, (n), nargs);    \
    return NULL;                                                                                   \
  }
#define PTR(i, name) uint64_t name; if (as_u64(args[i], &name)) return NULL
#define I64(i, name) int64_t name; if (as_i64(args[i], &name)) return NULL
#define F32(i, name) float name; if (as_f32(args[i], &name)) return NULL

/* fg_block_fp8_gemm / fg_block_fp8_gemm_pow2_scales (include/flaggems_amd.h): fn, then the 21 arguments */
typedef int (*block_gemm_fn)(const void*, int64_t, const void*, int64_t, const float*, int64_t, int64_t, const float*, int64_t,
                             int64_t, void*, int64_t, int, int64_t, int64_t, int64_t, int64_t, int64_t, void*, size_t, void*);
static PyObject* block_fp8_gemm(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
  (void)self;
  NEED(22);
  PTR(0, fn); PTR(1, A); I64(2, lda); PTR(3, B); I64(4, ldb); PTR(5, As); I64(6, as_rs); I64(7, as_cs);
  PTR(8, Bs); I64(9, bs_rs); I64(10, bs_cs); PTR(11, C); I64(12, ldc); I64(13, c_dtype);
  I64(14, M); I64(15, N); I64(16, K); I64(17, bn); I64(18, bk); PTR(19, ws); PTR(20, ws_bytes); PTR(21, stream);
  const int rc = ((block_gemm_fn)(uintptr_t)fn)((const void*)(uintptr_t)A, lda, (const void*)(uintptr_t)B, ldb,
                                                (const float*)(uintptr_t)As, as_rs, as_cs, (const float*)(uintptr_t)Bs, bs_rs, bs_cs,
                                                (void*)(uintptr_t)C, ldc, (int)c_dtype, M, N, K, bn, bk,
                                                (void*)(uintptr_t)ws, (size_t)ws_bytes, (void*)(uintptr_t)stream);
  return PyLong_FromLong(rc);
}

/* fg_group_quant_fp8: fn, then the 20 arguments */
typedef int (*group_quant_fn)(const void*, int, int64_t, int64_t, int64_t, void*, int, int64_t, float*, int64_t, int64_t, int64_t,
                              float, float, float, float, int, int, int, void*);
static PyObject* group_quant_fp8(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
  (void)self;
  NEED(21);
  PTR(0, fn); PTR(1, x); I64(2, x_dtype); I64(3, rows); I64(4, cols); I64(5, x_rs); PTR(6, q); I64(7, q_dtype); I64(8, q_rs);
  PTR(9, s); I64(10, s_rs); I64(11, s_cs); I64(12, group); F32(13, floor_); F32(14, fmin_); F32(15, fmax_); F32(16, inv);
  I64(17, scale_rule); I64(18, quot_rule); I64(19, pow2_rule); PTR(20, stream);
  const int rc = ((group_quant_fn)(uintptr_t)fn)((const void*)(uintptr_t)x, (int)x_dtype, rows, cols, x_rs, (void*)(uintptr_t)q,
                                                 (int)q_dtype, q_rs, (float*)(uintptr_t)s, s_rs, s_cs, group, floor_, fmin_, fmax_,
                                                 inv, (int)scale_rule, (int)quot_rule, (int)pow2_rule, (void*)(uintptr_t)stream);
  return PyLong_FromLong(rc);
}

/* fg_scaled_fp8_gemm / fg_scaled_int8_gemm: fn, then the 19 arguments */
typedef int (*scaled_gemm_fn)(const void*, int64_t, const void*, int64_t, const float*, int, const float*, int, const void*, int,
                              void*, int64_t, int, int64_t, int64_t, int64_t, void*, size_t, void*);
static PyObject* scaled_gemm(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
  (void)self;
  NEED(20);
  PTR(0, fn); PTR(1, A); I64(2, lda); PTR(3, B); I64(4, ldb); PTR(5, sa); I64(6, sa_per_row); PTR(7, sb); I64(8, sb_per_col);
  PTR(9, bias); I64(10, bias_dtype); PTR(11, C); I64(12, ldc); I64(13, c_dtype); I64(14, M); I64(15, N); I64(16, K);
  PTR(17, ws); PTR(18, ws_bytes); PTR(19, stream);
  const int rc = ((scaled_gemm_fn)(uintptr_t)fn)((const void*)(uintptr_t)A, lda, (const void*)(uintptr_t)B, ldb,
                                                 (const float*)(uintptr_t)sa, (int)sa_per_row, (const float*)(uintptr_t)sb,
                                                 (int)sb_per_col, (const void*)(uintptr_t)bias, (int)bias_dtype, (void*)(uintptr_t)C,
                                                 ldc, (int)c_dtype, M, N, K, (void*)(uintptr_t)ws, (size_t)ws_bytes,
                                                 (void*)(uintptr_t)stream);
  return PyLong_FromLong(rc);
}

static PyMethodDef methods[] = {
    {"block_fp8_gemm", (PyCFunction)(void (*)(void))block_fp8_gemm, METH_FASTCALL,
     "block_fp8_gemm(fn_address, *the 21 arguments of fg_block_fp8_gemm) -> status"},
    {"group_quant_fp8", (PyCFunction)(void (*)(void))group_quant_fp8, METH_FASTCALL,
     "group_quant_fp8(fn_address, *the 20 arguments of fg_group_quant_fp8) -> status"},
    {"scaled_gemm", (PyCFunction)(void (*)(void))scaled_gemm, METH_FASTCALL,
     "scaled_gemm(fn_address, *the 19 arguments of fg_scaled_fp8_gemm / fg_scaled_int8_gemm) -> status"},
    {NULL, NULL, 0, NULL}};

static struct PyModuleDef module = {PyModuleDef_HEAD_INIT, "_fg_fastcall",
                                    "argument marshalling for the decode-critical flaggems_amd C-ABI calls", -1, methods,
                                    NULL, NULL, NULL, NULL};

PyMODINIT_FUNC PyInit__fg_fastcall(void) { return PyModule_Create(&module); }

/* CPython binding of the two GEMM entry points of libfp8bs.so (include/fp8bs.h), for callers that issue many
 * small calls from Python: ctypes spends ~1.2 us marshalling the 13 arguments of fp8bs_gemm_ex, this module
 * ~0.15 us.  Pointers and the stream arrive as Python ints (tensor.data_ptr(), the raw hipStream_t) or None;
 * the status code is returned as an int.  Nothing else lives here: checks, planning and launches are the
 * library's.  Built by build.py with the host compiler; when the module is missing the package binds the same
 * functions through ctypes (the library itself has no substitute).
 * Stands where the reference has its pybind11 module built by load_inline
 * (1-amd-fp8-mm/amd-fp8-mm-submission.py:582-592). */
#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <stdint.h>

#include "fp8bs.h"

/* a Python int (address) or None -> pointer; -1 with an exception set on anything else */
static int as_pointer(PyObject* o, void** out) {
    if (o == Py_None) { *out = NULL; return 0; }
    void* p = PyLong_AsVoidPtr(o);
    if (p == NULL && PyErr_Occurred()) return -1;
    *out = p;
    return 0;
}

static int as_int(PyObject* o, int* out) {
    long v = PyLong_AsLong(o);
    if (v == -1 && PyErr_Occurred()) return -1;
    if (v < INT32_MIN || v > INT32_MAX) { PyErr_SetString(PyExc_OverflowError, "argument does not fit a C int"); return -1; }
    *out = (int)v;
    return 0;
}

/* gemm_ex(a, b, a_scale, b_scale, c, ws, ws_bytes, m, n, k, variant, split_k, stream) -> status */
static PyObject* py_gemm_ex(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
    (void)self;
    if (nargs != 13) { PyErr_SetString(PyExc_TypeError, "gemm_ex takes 13 arguments"); return NULL; }
    void* p[6]; void* stream; int v[5];
    for (int i = 0; i < 6; i++) if (as_pointer(args[i], &p[i]) < 0) return NULL;
    size_t ws_bytes = PyLong_AsSize_t(args[6]);
    if (ws_bytes == (size_t)-1 && PyErr_Occurred()) return NULL;
    for (int i = 0; i < 5; i++) if (as_int(args[7 + i], &v[i]) < 0) return NULL;
    if (as_pointer(args[12], &stream) < 0) return NULL;
    int st = fp8bs_gemm_ex(p[0], p[1], (const float*)p[2], (const float*)p[3], p[4], p[5], ws_bytes, v[0], v[1], v[2], v[3], v[4], stream);
    return PyLong_FromLong(st);
}

/* gemm_grouped_ex(a, b, a_scale, b_scale, c, row_offsets, num_experts, total_rows, n, k, variant, stream) -> status */
static PyObject* py_gemm_grouped_ex(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
    (void)self;
    if (nargs != 12) { PyErr_SetString(PyExc_TypeError, "gemm_grouped_ex takes 12 arguments"); return NULL; }
    void* p[6]; void* stream; int v[5];
    for (int i = 0; i < 6; i++) if (as_pointer(args[i], &p[i]) < 0) return NULL;
    for (int i = 0; i < 5; i++) if (as_int(args[6 + i], &v[i]) < 0) return NULL;
    if (as_pointer(args[11], &stream) < 0) return NULL;
    int st = fp8bs_gemm_grouped_ex(p[0], p[1], (const float*)p[2], (const float*)p[3], p[4], (const int32_t*)p[5], v[0], v[1], v[2], v[3], v[4], stream);
    return PyLong_FromLong(st);
}

static PyMethodDef methods[] = {
    {"gemm_ex", (PyCFunction)(void (*)(void))py_gemm_ex, METH_FASTCALL, "fp8bs_gemm_ex with addresses as ints; returns the status code"},
    {"gemm_grouped_ex", (PyCFunction)(void (*)(void))py_gemm_grouped_ex, METH_FASTCALL, "fp8bs_gemm_grouped_ex with addresses as ints; returns the status code"},
    {NULL, NULL, 0, NULL},
};

static struct PyModuleDef module = {PyModuleDef_HEAD_INIT, "_fp8bs_pycall", "fast calls into libfp8bs.so", -1, methods, NULL, NULL, NULL, NULL};

PyMODINIT_FUNC PyInit__fp8bs_pycall(void) { return PyModule_Create(&module); }

/* Direct calls of the C ABI for the operations a network step issues by the thousand.
 *
 * ctypes converts every argument through its type table on every call (0.8-0.9 us for the five to
 * eight arguments of an elementwise or matrix-vector entry point); a METH_FASTCALL method that
 * reads Python ints and floats itself costs a tenth of that. The module knows nothing about the
 * library: Calls(addresses) takes the addresses of the entry points (name -> integer, as ctypes
 * hands them out), so it serves whichever library the binding loaded. Each method returns the
 * entry point's int status; the GIL is released around the call, as ctypes does.
 *
 * Device addresses arrive as Python ints (or None for NULL), sizes as ints, scalars as floats or
 * ints; a float32 scalar is the C cast of the Python float, which is what ctypes' c_float does.
 */
#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <stddef.h>
#include <stdint.h>

typedef int (*binary_fn)(int, const float*, const float*, float*, size_t);
typedef int (*mult_add_tt_fn)(const float*, const float*, float*, size_t);
typedef int (*scalar_fn)(int, float, const float*, float*, size_t);
typedef int (*unary_fn)(int, const float*, float*, size_t);
typedef int (*deriv_fn)(int, const float*, const float*, float*, size_t);
typedef int (*clip_fn)(const float*, float, float, float*, size_t);
typedef int (*mv_fn)(int, const float*, const float*, float*, int64_t, int64_t, int, int);
typedef int (*fill_fn)(float*, float, size_t);
typedef int (*gemm_fn)(int, int, int64_t, int64_t, int64_t, float, const float*, int64_t, const float*, int64_t,
                       float, float*, int64_t);
typedef int (*d2d_fn)(void*, const void*, size_t);
typedef int (*sum_fn)(const float*, float*, int64_t, int64_t, int);

typedef struct {
    PyObject_HEAD
    binary_fn binary;
    mult_add_tt_fn mult_add_tt;
    scalar_fn scalar;
    unary_fn unary;
    deriv_fn deriv;
    clip_fn clip;
    mv_fn mv;
    fill_fn fill;
    gemm_fn gemm;
    d2d_fn d2d;
    sum_fn sum;
} Calls;

static int as_ptr(PyObject* o, void** p) {
    if (o == Py_None) {
        *p = NULL;
        return 0;
    }
    unsigned long long v = PyLong_AsUnsignedLongLong(o);
    if (v == (unsigned long long)-1 && PyErr_Occurred()) return -1;
    *p = (void*)(uintptr_t)v;
    return 0;
}

static int as_i64(PyObject* o, long long* v) {
    *v = PyLong_AsLongLong(o);
    return (*v == -1 && PyErr_Occurred()) ? -1 : 0;
}

static int as_size(PyObject* o, size_t* v) {
    long long s = PyLong_AsLongLong(o);
    if (s == -1 && PyErr_Occurred()) return -1;
    if (s < 0) {
        PyErr_SetString(PyExc_ValueError, "negative element count");
        return -1;
    }
    *v = (size_t)s;
    return 0;
}

static int as_int(PyObject* o, int* v) {
    long s = PyLong_AsLong(o);
    if (s == -1 && PyErr_Occurred()) return -1;
    *v = (int)s;
    return 0;
}

static int as_f32(PyObject* o, float* v) {
    double d = PyFloat_AsDouble(o);
    if (d == -1.0 && PyErr_Occurred()) return -1;
    *v = (float)d;
    return 0;
}

#define REQUIRE(count, fn, name)                                                                   \
    if (nargs != (count)) {                                                                        \
        PyErr_Format(PyExc_TypeError, name " takes %d arguments (%zd given)", (count), nargs);     \
        return NULL;                                                                               \
    }                                                                                              \
    if (!self->fn) {                                                                               \
        PyErr_SetString(PyExc_RuntimeError, name ": the library does not have this entry point");  \
        return NULL;                                                                               \
    }

#define CALL(expr)                     \
    int st;                            \
    Py_BEGIN_ALLOW_THREADS st = (expr); \
    Py_END_ALLOW_THREADS return PyLong_FromLong(st);

static PyObject* calls_binary(Calls* self, PyObject* const* args, Py_ssize_t nargs) {
    REQUIRE(5, binary, "binary")
    int op; void *a, *b, *out; size_t n;
    if (as_int(args[0], &op) || as_ptr(args[1], &a) || as_ptr(args[2], &b) || as_ptr(args[3], &out) ||
        as_size(args[4], &n)) return NULL;
    CALL(self->binary(op, a, b, out, n))
}

static PyObject* calls_mult_add_tt(Calls* self, PyObject* const* args, Py_ssize_t nargs) {
    REQUIRE(4, mult_add_tt, "mult_add_tt")
    void *a, *b, *out; size_t n;
    if (as_ptr(args[0], &a) || as_ptr(args[1], &b) || as_ptr(args[2], &out) || as_size(args[3], &n)) return NULL;
    CALL(self->mult_add_tt(a, b, out, n))
}

static PyObject* calls_scalar(Calls* self, PyObject* const* args, Py_ssize_t nargs) {
    REQUIRE(5, scalar, "scalar")
    int op; float s; void *t, *out; size_t n;
    if (as_int(args[0], &op) || as_f32(args[1], &s) || as_ptr(args[2], &t) || as_ptr(args[3], &out) ||
        as_size(args[4], &n)) return NULL;
    CALL(self->scalar(op, s, t, out, n))
}

static PyObject* calls_unary(Calls* self, PyObject* const* args, Py_ssize_t nargs) {
    REQUIRE(4, unary, "unary")
    int op; void *x, *y; size_t n;
    if (as_int(args[0], &op) || as_ptr(args[1], &x) || as_ptr(args[2], &y) || as_size(args[3], &n)) return NULL;
    CALL(self->unary(op, x, y, n))
}

static PyObject* calls_deriv(Calls* self, PyObject* const* args, Py_ssize_t nargs) {
    REQUIRE(5, deriv, "deriv")
    int op; void *y, *dy, *dx; size_t n;
    if (as_int(args[0], &op) || as_ptr(args[1], &y) || as_ptr(args[2], &dy) || as_ptr(args[3], &dx) ||
        as_size(args[4], &n)) return NULL;
    CALL(self->deriv(op, y, dy, dx, n))
}

static PyObject* calls_clip(Calls* self, PyObject* const* args, Py_ssize_t nargs) {
    REQUIRE(5, clip, "clip")
    void *a, *out; float lo, hi; size_t n;
    if (as_ptr(args[0], &a) || as_f32(args[1], &lo) || as_f32(args[2], &hi) || as_ptr(args[3], &out) ||
        as_size(args[4], &n)) return NULL;
    CALL(self->clip(a, lo, hi, out, n))
}

static PyObject* calls_mv(Calls* self, PyObject* const* args, Py_ssize_t nargs) {
    REQUIRE(8, mv, "mv")
    int op, col, acc; void *m, *v, *out; long long M, N;
    if (as_int(args[0], &op) || as_ptr(args[1], &m) || as_ptr(args[2], &v) || as_ptr(args[3], &out) ||
        as_i64(args[4], &M) || as_i64(args[5], &N) || as_int(args[6], &col) || as_int(args[7], &acc)) return NULL;
    CALL(self->mv(op, m, v, out, M, N, col, acc))
}

static PyObject* calls_fill(Calls* self, PyObject* const* args, Py_ssize_t nargs) {
    REQUIRE(3, fill, "fill")
    void* mem; float val; size_t n;
    if (as_ptr(args[0], &mem) || as_f32(args[1], &val) || as_size(args[2], &n)) return NULL;
    CALL(self->fill(mem, val, n))
}

static PyObject* calls_gemm(Calls* self, PyObject* const* args, Py_ssize_t nargs) {
    REQUIRE(13, gemm, "gemm")
    int ta, tb; long long M, N, K, lda, ldb, ldc; float alpha, beta; void *A, *B, *C;
    if (as_int(args[0], &ta) || as_int(args[1], &tb) || as_i64(args[2], &M) || as_i64(args[3], &N) ||
        as_i64(args[4], &K) || as_f32(args[5], &alpha) || as_ptr(args[6], &A) || as_i64(args[7], &lda) ||
        as_ptr(args[8], &B) || as_i64(args[9], &ldb) || as_f32(args[10], &beta) || as_ptr(args[11], &C) ||
        as_i64(args[12], &ldc)) return NULL;
    CALL(self->gemm(ta, tb, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc))
}

static PyObject* calls_d2d(Calls* self, PyObject* const* args, Py_ssize_t nargs) {
    REQUIRE(3, d2d, "d2d")
    void *dst, *src; size_t nbytes;
    if (as_ptr(args[0], &dst) || as_ptr(args[1], &src) || as_size(args[2], &nbytes)) return NULL;
    CALL(self->d2d(dst, src, nbytes))
}

static PyObject* calls_sum(Calls* self, PyObject* const* args, Py_ssize_t nargs) {
    REQUIRE(5, sum, "sum")
    void *a, *out; long long M, N; int axis;
    if (as_ptr(args[0], &a) || as_ptr(args[1], &out) || as_i64(args[2], &M) || as_i64(args[3], &N) ||
        as_int(args[4], &axis)) return NULL;
    CALL(self->sum(a, out, M, N, axis))
}

static int lookup(PyObject* table, const char* name, void** out) {
    PyObject* v = PyMapping_GetItemString(table, name);
    *out = NULL;
    if (!v) {
        PyErr_Clear();      /* a library without this entry point: the method raises when it is called */
        return 0;
    }
    int bad = as_ptr(v, out);
    Py_DECREF(v);
    return bad;
}

static int calls_init(Calls* self, PyObject* args, PyObject* kwds) {
    PyObject* table;
    if (!PyArg_ParseTuple(args, "O", &table)) return -1;
    (void)kwds;
    if (lookup(table, "bship_binary_f32", (void**)&self->binary) ||
        lookup(table, "bship_mult_add_tt_f32", (void**)&self->mult_add_tt) ||
        lookup(table, "bship_scalar_f32", (void**)&self->scalar) ||
        lookup(table, "bship_unary_f32", (void**)&self->unary) ||
        lookup(table, "bship_deriv_f32", (void**)&self->deriv) ||
        lookup(table, "bship_clip_f32", (void**)&self->clip) ||
        lookup(table, "bship_mv_f32", (void**)&self->mv) ||
        lookup(table, "bship_fill_f32", (void**)&self->fill) ||
        lookup(table, "bship_gemm_f32", (void**)&self->gemm) ||
        lookup(table, "bship_d2d", (void**)&self->d2d) ||
        lookup(table, "bship_sum_f32", (void**)&self->sum))
        return -1;
    return 0;
}

static PyMethodDef calls_methods[] = {
    {"binary", (PyCFunction)(void (*)(void))calls_binary, METH_FASTCALL, "bship_binary_f32(op, a, b, out, n)"},
    {"mult_add_tt", (PyCFunction)(void (*)(void))calls_mult_add_tt, METH_FASTCALL, "bship_mult_add_tt_f32(a, b, out, n)"},
    {"scalar", (PyCFunction)(void (*)(void))calls_scalar, METH_FASTCALL, "bship_scalar_f32(op, s, t, out, n)"},
    {"unary", (PyCFunction)(void (*)(void))calls_unary, METH_FASTCALL, "bship_unary_f32(op, x, y, n)"},
    {"deriv", (PyCFunction)(void (*)(void))calls_deriv, METH_FASTCALL, "bship_deriv_f32(op, y, dy, dx, n)"},
    {"clip", (PyCFunction)(void (*)(void))calls_clip, METH_FASTCALL, "bship_clip_f32(a, lo, hi, out, n)"},
    {"mv", (PyCFunction)(void (*)(void))calls_mv, METH_FASTCALL, "bship_mv_f32(op, m, v, out, M, N, v_is_col, accumulate)"},
    {"fill", (PyCFunction)(void (*)(void))calls_fill, METH_FASTCALL, "bship_fill_f32(mem, val, n)"},
    {"gemm", (PyCFunction)(void (*)(void))calls_gemm, METH_FASTCALL,
     "bship_gemm_f32(transa, transb, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc)"},
    {"d2d", (PyCFunction)(void (*)(void))calls_d2d, METH_FASTCALL, "bship_d2d(dst, src, nbytes)"},
    {"sum", (PyCFunction)(void (*)(void))calls_sum, METH_FASTCALL, "bship_sum_f32(a, out, M, N, axis)"},
    {NULL, NULL, 0, NULL}};

static PyTypeObject CallsType = {
    PyVarObject_HEAD_INIT(NULL, 0).tp_name = "brainstorm_amd._fastcall.Calls",
    .tp_basicsize = sizeof(Calls),
    .tp_flags = Py_TPFLAGS_DEFAULT,
    .tp_doc = "Calls(addresses): direct calls of the C ABI entry points whose addresses the mapping gives.",
    .tp_methods = calls_methods,
    .tp_init = (initproc)calls_init,
    .tp_new = PyType_GenericNew,
};

static PyModuleDef fastcall_module = {PyModuleDef_HEAD_INIT, "_fastcall",
                                      "Direct calls of libbship's hottest entry points.", -1, NULL};

PyMODINIT_FUNC PyInit__fastcall(void) {
    if (PyType_Ready(&CallsType) < 0) return NULL;
    PyObject* m = PyModule_Create(&fastcall_module);
    if (!m) return NULL;
    Py_INCREF(&CallsType);
    if (PyModule_AddObject(m, "Calls", (PyObject*)&CallsType) < 0) {
        Py_DECREF(&CallsType);
        Py_DECREF(m);
        return NULL;
    }
    return m;
}

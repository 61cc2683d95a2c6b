/* CPython fast path into the GEMM dispatcher: flextrain_amd._dispatch_fast.
 *
 * Same call contract as the reference's `_dispatch_pyext.matmul_fast`
 * (helpers/matmul_dispatcher/src/dispatch_pyext.cpp:37-140): 24 positional arguments, all plain
 * Python ints / floats, in the order
 *     ctx, stream, M, N, K, A, lda, trans_a, B, ldb, trans_b, C, ldc, D, ldd,
 *     workspace, workspace_bytes, a_dt, b_dt, c_dt, d_dt, compute_dt, alpha, beta
 * TypeError on any other argument count, ValueError for a null context, RuntimeError when
 * dispatch_matmul reports failure, None otherwise.
 *
 * The module does not link against libflexhip.so: Python loads that library once (ctypes) and hands
 * this module the address of its `dispatch_matmul` through bind(), so both paths share one copy of
 * the library and its per-context caches.  Plain C, no dependency beyond the CPython headers. */
#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <limits.h>
#include <stddef.h>
#include <stdint.h>

typedef int (*dispatch_fn)(void* ctx, intptr_t stream, int M, int N, int K, intptr_t A, int lda, intptr_t B,
                           int ldb, intptr_t C, int ldc, intptr_t D, int ldd, intptr_t ws, size_t ws_bytes,
                           int a_dt, int b_dt, int c_dt, int d_dt, int compute_dt, float alpha, float beta,
                           int trans_a, int trans_b);

static dispatch_fn g_dispatch = NULL;

/* argument kinds, in call order */
enum { AS_PTR, AS_INT, AS_SIZE, AS_REAL };
static const unsigned char kKinds[24] = {
    AS_PTR, AS_PTR,                     /* ctx, stream */
    AS_INT, AS_INT, AS_INT,             /* M, N, K */
    AS_PTR, AS_INT, AS_INT,             /* A, lda, trans_a */
    AS_PTR, AS_INT, AS_INT,             /* B, ldb, trans_b */
    AS_PTR, AS_INT,                     /* C, ldc */
    AS_PTR, AS_INT,                     /* D, ldd */
    AS_PTR, AS_SIZE,                    /* workspace, bytes */
    AS_INT, AS_INT, AS_INT, AS_INT, AS_INT, /* dtypes */
    AS_REAL, AS_REAL};                  /* alpha, beta */

static PyObject* fast_bind(PyObject* self, PyObject* arg) {
    (void)self;
    void* p = PyLong_AsVoidPtr(arg);
    if (p == NULL && PyErr_Occurred()) return NULL;
    g_dispatch = (dispatch_fn)p;
    Py_RETURN_NONE;
}

static PyObject* fast_matmul(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
    (void)self;
    if (nargs != 24) {
        PyErr_Format(PyExc_TypeError, "matmul_fast takes exactly 24 positional arguments (%zd given)", nargs);
        return NULL;
    }
    if (g_dispatch == NULL) {
        PyErr_SetString(PyExc_RuntimeError, "matmul_fast: not bound to a dispatcher library (call bind first)");
        return NULL;
    }
    intptr_t p[24];
    double r[2] = {0.0, 0.0};
    for (int i = 0; i < 24; ++i) {
        /* stop at the first argument that does not convert: no C-API call may follow a set exception */
        switch (kKinds[i]) {
            case AS_PTR:
                p[i] = (intptr_t)PyLong_AsVoidPtr(args[i]);
                if (p[i] == 0 && PyErr_Occurred()) return NULL;
                break;
            case AS_INT: {
                const long v = PyLong_AsLong(args[i]);
                if (v == -1 && PyErr_Occurred()) return NULL;
                if (v < INT_MIN || v > INT_MAX) {       /* the dispatcher takes C ints: never truncate silently */
                    PyErr_Format(PyExc_OverflowError, "matmul_fast: argument %d (%ld) does not fit a C int", i, v);
                    return NULL;
                }
                p[i] = (intptr_t)v;
                break;
            }
            case AS_SIZE: {
                const size_t v = PyLong_AsSize_t(args[i]);
                if (v == (size_t)-1 && PyErr_Occurred()) return NULL;
                p[i] = (intptr_t)v;
                break;
            }
            default:
                r[i - 22] = PyFloat_AsDouble(args[i]);
                if (r[i - 22] == -1.0 && PyErr_Occurred()) return NULL;
                p[i] = 0;
                break;
        }
    }
    if (p[0] == 0) {
        PyErr_SetString(PyExc_ValueError, "matmul_fast: the dispatcher context is null");
        return NULL;
    }
    const int rc = g_dispatch((void*)p[0], p[1], (int)p[2], (int)p[3], (int)p[4], p[5], (int)p[6], p[8], (int)p[9],
                              p[11], (int)p[12], p[13], (int)p[14], p[15], (size_t)p[16], (int)p[17], (int)p[18],
                              (int)p[19], (int)p[20], (int)p[21], (float)r[0], (float)r[1], (int)p[7], (int)p[10]);
    if (rc != 0) {
        PyErr_Format(PyExc_RuntimeError, "matmul_fast: dispatch_matmul failed (rc=%d)", rc);
        return NULL;
    }
    Py_RETURN_NONE;
}

static PyMethodDef kMethods[] = {
    {"bind", (PyCFunction)fast_bind, METH_O, "bind(address of dispatch_matmul in the loaded library)"},
    {"matmul_fast", (PyCFunction)(void (*)(void))fast_matmul, METH_FASTCALL,
     "matmul_fast(ctx, stream, M, N, K, A, lda, trans_a, B, ldb, trans_b, C, ldc, D, ldd, ws, ws_bytes, "
     "a_dt, b_dt, c_dt, d_dt, compute_dt, alpha, beta) -> None"},
    {NULL, NULL, 0, NULL}};

static struct PyModuleDef kModule = {PyModuleDef_HEAD_INIT, "_dispatch_fast",
                                     "Fast-call entry into the GEMM dispatcher of libflexhip.so.", -1, kMethods,
                                     NULL, NULL, NULL, NULL};

PyMODINIT_FUNC PyInit__dispatch_fast(void) { return PyModule_Create(&kModule); }

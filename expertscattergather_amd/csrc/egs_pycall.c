/* CPython module `_egs_pycall`: the four launcher-level entry points of include/egs_hip.h callable from Python with
 * plain integers, without the per-argument conversion cost of ctypes (about 0.25 us per argument; a launcher call has
 * 14 to 23 of them and a forward + backward step at the reference's default shape takes ~50 us on the GPU).
 *
 * Nothing but argument passing happens here: every function takes integers (device pointers as integers, 0 for a null
 * pointer; the six sizes of egs_dims spelled out), calls the C entry point of the same name in libegs_hip.so with the
 * GIL released, and returns its status code.  The Python side (hip_kernels.py) uses this module when it is built and
 * ctypes otherwise; both reach the same library.
 *
 * Reference counterparts of the entry points: egs/triton_kernels.py:367-392 (gather forward), :400-441 (gather
 * backward), :449-474 (scatter forward), :483-525 (scatter backward).
 */
#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <stdint.h>
#include "egs_hip.h"

/* converts `n` positional integers; returns 0 on success, -1 with an exception set */
static int ints(PyObject *const *args, Py_ssize_t nargs, Py_ssize_t n, const char *name, uint64_t *out)
{
    if (nargs != n) {
        PyErr_Format(PyExc_TypeError, "%s takes %zd integers, got %zd", name, n, nargs);
        return -1;
    }
    for (Py_ssize_t i = 0; i < n; ++i) {
        PyObject *o = args[i];
        if (!PyLong_Check(o)) {
            PyErr_Format(PyExc_TypeError, "%s: argument %zd is not an integer", name, i);
            return -1;
        }
        /* sizes and strides may be negative only by mistake: pass them through as two's complement, the library validates */
        uint64_t v = (uint64_t)PyLong_AsUnsignedLongLongMask(o);
        if (v == (uint64_t)-1 && PyErr_Occurred()) return -1;
        out[i] = v;
    }
    return 0;
}

static egs_dims dims_of(const uint64_t *a)
{
    egs_dims d;
    d.B = (int32_t)a[0]; d.T = (int32_t)a[1]; d.E = (int32_t)a[2];
    d.K = (int32_t)a[3]; d.I = (int32_t)a[4]; d.J = (int32_t)a[5];
    return d;
}

#define PTR(x) ((void *)(uintptr_t)(x))

/* gather_forward(X, W, Ind, Y, table, table_bytes, B, T, E, K, I, J, ldx_b, ldx_t, dtype, ind_dtype, stream) */
static PyObject *py_gather_forward(PyObject *self, PyObject *const *args, Py_ssize_t nargs)
{
    uint64_t a[17];
    if (ints(args, nargs, 17, "gather_forward", a)) return NULL;
    const egs_dims d = dims_of(a + 6);
    int rc;
    Py_BEGIN_ALLOW_THREADS
    rc = egs_expert_gather_forward_table(PTR(a[0]), PTR(a[1]), PTR(a[2]), PTR(a[3]), PTR(a[4]), (size_t)a[5], &d,
                                         (int64_t)a[12], (int64_t)a[13], (int)a[14], (int)a[15], PTR(a[16]));
    Py_END_ALLOW_THREADS
    return PyLong_FromLong(rc);
}

/* scatter_forward(Y, W, Ind, table, table_bytes, Out, workspace, workspace_bytes, B, T, E, K, I, J, dtype, ind_dtype, mode, stream) */
static PyObject *py_scatter_forward(PyObject *self, PyObject *const *args, Py_ssize_t nargs)
{
    uint64_t a[18];
    if (ints(args, nargs, 18, "scatter_forward", a)) return NULL;
    const egs_dims d = dims_of(a + 8);
    int rc;
    Py_BEGIN_ALLOW_THREADS
    rc = egs_expert_scatter_forward_table(PTR(a[0]), PTR(a[1]), PTR(a[2]), PTR(a[3]), (size_t)a[4], PTR(a[5]), PTR(a[6]),
                                          (size_t)a[7], &d, (int)a[14], (int)a[15], (int)a[16], PTR(a[17]));
    Py_END_ALLOW_THREADS
    return PyLong_FromLong(rc);
}

/* gather_backward(X, W, Ind, table, table_bytes, grad_Y, grad_X, grad_W, workspace, workspace_bytes, B, T, E, K, I, J,
 *                 ldx_b, ldx_t, dtype, ind_dtype, mode, stream) */
static PyObject *py_gather_backward(PyObject *self, PyObject *const *args, Py_ssize_t nargs)
{
    uint64_t a[22];
    if (ints(args, nargs, 22, "gather_backward", a)) return NULL;
    const egs_dims d = dims_of(a + 10);
    int rc;
    Py_BEGIN_ALLOW_THREADS
    rc = egs_expert_gather_backward_table(PTR(a[0]), PTR(a[1]), PTR(a[2]), PTR(a[3]), (size_t)a[4], PTR(a[5]), PTR(a[6]),
                                          PTR(a[7]), PTR(a[8]), (size_t)a[9], &d, (int64_t)a[16], (int64_t)a[17],
                                          (int)a[18], (int)a[19], (int)a[20], PTR(a[21]));
    Py_END_ALLOW_THREADS
    return PyLong_FromLong(rc);
}

/* scatter_backward(Y, W, Ind, grad_Out, grad_Y, grad_W, workspace, workspace_bytes, B, T, E, K, I, J, ldg_b, ldg_t,
 *                  dtype, ind_dtype, stream) */
static PyObject *py_scatter_backward(PyObject *self, PyObject *const *args, Py_ssize_t nargs)
{
    uint64_t a[19];
    if (ints(args, nargs, 19, "scatter_backward", a)) return NULL;
    const egs_dims d = dims_of(a + 8);
    int rc;
    Py_BEGIN_ALLOW_THREADS
    rc = egs_expert_scatter_backward(PTR(a[0]), PTR(a[1]), PTR(a[2]), PTR(a[3]), PTR(a[4]), PTR(a[5]), PTR(a[6]),
                                     (size_t)a[7], &d, (int64_t)a[14], (int64_t)a[15], (int)a[16], (int)a[17], PTR(a[18]));
    Py_END_ALLOW_THREADS
    return PyLong_FromLong(rc);
}

static PyObject *py_abi_version(PyObject *self, PyObject *noargs)
{
    return PyLong_FromLong(egs_abi_version());
}

static PyMethodDef methods[] = {
    {"gather_forward", (PyCFunction)(void (*)(void))py_gather_forward, METH_FASTCALL, "egs_expert_gather_forward_table"},
    {"scatter_forward", (PyCFunction)(void (*)(void))py_scatter_forward, METH_FASTCALL, "egs_expert_scatter_forward_table"},
    {"gather_backward", (PyCFunction)(void (*)(void))py_gather_backward, METH_FASTCALL, "egs_expert_gather_backward_table"},
    {"scatter_backward", (PyCFunction)(void (*)(void))py_scatter_backward, METH_FASTCALL, "egs_expert_scatter_backward"},
    {"abi_version", py_abi_version, METH_NOARGS, "egs_abi_version"},
    {NULL, NULL, 0, NULL},
};

static struct PyModuleDef module = {PyModuleDef_HEAD_INIT, "_egs_pycall", "integer-argument launchers of libegs_hip.so", -1, methods};

PyMODINIT_FUNC PyInit__egs_pycall(void)
{
    return PyModule_Create(&module);
}

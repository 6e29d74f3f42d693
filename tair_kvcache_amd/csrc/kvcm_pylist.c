/* kvcm_pylist.c -- CPython extension `tair_kvcache_amd._kvcm_pylist`: Python lists of ints -> packed int32.
 *
 * The reference's operators receive their indices as Python lists (List[int] of B*T token slots, or the nested
 * List[List[int]] that generate_blocks_idx returns: kv_cache_manager/py_connector/vllm/v1_connector.py:308-320,
 * kv_cache_manager/py_connector/kernel/batch_gather_scatter_helper.py:101-121). Turning 2048 of them into something a
 * C function can read costs 12 us through array('i', list), 40 us row by row for the nested form and 100 us through
 * torch.tensor -- under the interpreter lock that the connector's 32 worker threads share, which makes it the one part
 * of a transfer task that does not overlap with anything. One C loop over the list objects takes 3 us.
 *
 * Host code only; no device work. Built with gcc by tair_kvcache_amd/build.py.
 */
#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <stdint.h>

static int is_seq(PyObject *o) { return PyList_Check(o) || PyTuple_Check(o); }

/* the items of one flat list or tuple -> dst; returns 0, or -1 with an exception set */
static int pack_flat(PyObject *seq, int32_t *dst) {
    const Py_ssize_t n = PySequence_Fast_GET_SIZE(seq);
    PyObject **items = PySequence_Fast_ITEMS(seq);
    for (Py_ssize_t i = 0; i < n; ++i) {
        PyObject *it = items[i];
        long v;
        if (PyLong_CheckExact(it)) {
            int overflow = 0;
            v = PyLong_AsLongAndOverflow(it, &overflow);
            if (overflow) {
                PyErr_SetString(PyExc_OverflowError, "index does not fit 32 bits");
                return -1;
            }
        } else {
            if (PyFloat_Check(it) || !PyIndex_Check(it)) {
                PyErr_Format(PyExc_TypeError, "index lists hold integers, not %.100s", Py_TYPE(it)->tp_name);
                return -1;
            }
            v = PyLong_AsLong(it); /* an int subclass, a NumPy integer: through __index__ */
            if (v == -1 && PyErr_Occurred()) {
                return -1;
            }
        }
        if (v < INT32_MIN || v > INT32_MAX) {
            PyErr_SetString(PyExc_OverflowError, "index does not fit 32 bits");
            return -1;
        }
        dst[i] = (int32_t)v;
    }
    return 0;
}

/* pack_i32(seq) -> bytes of native int32: seq is a list or tuple of ints, or a list or tuple of such lists or tuples
 * (rows are concatenated). TypeError for anything else, OverflowError for a value beyond 32 bits. */
static PyObject *pack_i32(PyObject *self, PyObject *seq) {
    (void)self;
    if (!is_seq(seq)) {
        PyErr_SetString(PyExc_TypeError, "pack_i32 takes a list or tuple");
        return NULL;
    }
    const Py_ssize_t n_outer = PySequence_Fast_GET_SIZE(seq);
    PyObject **outer = PySequence_Fast_ITEMS(seq);
    const int nested = n_outer > 0 && is_seq(outer[0]);
    Py_ssize_t total = n_outer;
    if (nested) {
        total = 0;
        for (Py_ssize_t r = 0; r < n_outer; ++r) {
            if (!is_seq(outer[r])) {
                PyErr_SetString(PyExc_TypeError, "a nested index list holds lists or tuples only");
                return NULL;
            }
            total += PySequence_Fast_GET_SIZE(outer[r]);
        }
    }
    if (total > PY_SSIZE_T_MAX / 4) {
        PyErr_SetString(PyExc_OverflowError, "index list too long");
        return NULL;
    }
    PyObject *out = PyBytes_FromStringAndSize(NULL, total * 4);
    if (!out) {
        return NULL;
    }
    int32_t *dst = (int32_t *)PyBytes_AS_STRING(out);
    int rc = 0;
    if (nested) {
        for (Py_ssize_t r = 0; r < n_outer && rc == 0; ++r) {
            rc = pack_flat(outer[r], dst);
            dst += PySequence_Fast_GET_SIZE(outer[r]);
        }
    } else {
        rc = pack_flat(seq, dst);
    }
    if (rc != 0) {
        Py_DECREF(out);
        return NULL;
    }
    return out;
}

static PyMethodDef methods[] = {
    {"pack_i32", pack_i32, METH_O, "list or tuple of ints (or of lists of ints) -> bytes of native int32"},
    {NULL, NULL, 0, NULL}};

static struct PyModuleDef module = {PyModuleDef_HEAD_INIT, "_kvcm_pylist", "index lists -> packed int32", -1, methods,
                                    NULL, NULL, NULL, NULL};

PyMODINIT_FUNC PyInit__kvcm_pylist(void) { return PyModule_Create(&module); }

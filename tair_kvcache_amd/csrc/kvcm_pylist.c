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

/* one item of an index list -> *out; returns 0, or -1 with an exception set */
static int item_i32(PyObject *it, int32_t *out) {
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
    *out = (int32_t)v;
    return 0;
}

/* the items of one flat list or tuple -> dst; returns 0, or -1 with an exception set */
static int pack_flat(PyObject *seq, int32_t *dst) {
    const Py_ssize_t n = PySequence_Fast_GET_SIZE(seq);
    PyObject **items = PySequence_Fast_ITEMS(seq);
    for (Py_ssize_t i = 0; i < n; ++i) {
        if (item_i32(items[i], dst + i) != 0) {
            return -1;
        }
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

/* blocks_idx(manager_block_idxes, local_block_ids, manager_block_size, local_block_size) -> bytes of native int32
 * [len(manager_block_idxes)][manager_block_size]: the token slots of the manager blocks,
 *   out[b][i] = local_block_ids[tok / local_block_size] * local_block_size + tok % local_block_size,
 *   tok = manager_block_idxes[b] * manager_block_size + i
 * -- TairKvCacheConnector.generate_blocks_idx (kv_cache_manager/py_connector/vllm/v1_connector.py:308-320) as one C
 * loop instead of a Python double loop (258 us for 128 blocks of 16 tokens there, 2 us here; 1 ms and 5 us for
 * blocks of 64 tokens over engine blocks of 16). Returns None when a
 * manager block reaches beyond local_block_ids (the reference asserts; the caller raises). Both lists are lists or
 * tuples of ints. */
static PyObject *blocks_idx(PyObject *self, PyObject *args) {
    (void)self;
    PyObject *mgr, *local;
    long long t_mgr, t_eng;
    if (!PyArg_ParseTuple(args, "OOLL", &mgr, &local, &t_mgr, &t_eng)) {
        return NULL;
    }
    if (!is_seq(mgr) || !is_seq(local)) {
        PyErr_SetString(PyExc_TypeError, "blocks_idx takes lists or tuples of ints");
        return NULL;
    }
    if (t_mgr <= 0 || t_eng <= 0 || t_mgr > INT32_MAX || t_eng > INT32_MAX) {
        PyErr_SetString(PyExc_ValueError, "block sizes must be positive");
        return NULL;
    }
    const Py_ssize_t B = PySequence_Fast_GET_SIZE(mgr), n_local = PySequence_Fast_GET_SIZE(local);
    if (B > PY_SSIZE_T_MAX / 4 / (Py_ssize_t)t_mgr) {
        PyErr_SetString(PyExc_OverflowError, "index too long");
        return NULL;
    }
    PyObject *out = PyBytes_FromStringAndSize(NULL, B * (Py_ssize_t)t_mgr * 4);
    if (!out) {
        return NULL;
    }
    PyObject **m_items = PySequence_Fast_ITEMS(mgr), **l_items = PySequence_Fast_ITEMS(local);
    int32_t *dst = (int32_t *)PyBytes_AS_STRING(out);
    /* only the entries of local_block_ids that a manager block touches are read: a request's block list is
     * thousands of entries long, a task touches 128 */
    for (Py_ssize_t b = 0; b < B; ++b) {
        int32_t mb;
        if (item_i32(m_items[b], &mb) != 0) {
            Py_DECREF(out);
            return NULL;
        }
        long long tok = (long long)mb * t_mgr;
        const long long end = tok + t_mgr;
        if (tok < 0 || (end - 1) / t_eng >= n_local) { /* beyond the request's block list */
            Py_DECREF(out);
            Py_RETURN_NONE;
        }
        while (tok < end) {
            const long long blk = tok / t_eng, within = tok % t_eng;
            long long n = t_eng - within;
            if (n > end - tok) {
                n = end - tok;
            }
            int32_t lb;
            if (item_i32(l_items[blk], &lb) != 0) {
                Py_DECREF(out);
                return NULL;
            }
            const long long slot = (long long)lb * t_eng + within;
            if (slot < INT32_MIN || slot + n - 1 > INT32_MAX) {
                Py_DECREF(out);
                PyErr_SetString(PyExc_OverflowError, "token slot does not fit 32 bits");
                return NULL;
            }
            for (long long i = 0; i < n; ++i) {
                *dst++ = (int32_t)(slot + i);
            }
            tok += n;
        }
    }
    return out;
}

static PyMethodDef methods[] = {
    {"blocks_idx", blocks_idx, METH_VARARGS,
     "(manager_block_idxes, local_block_ids, manager_block_size, local_block_size) -> bytes of int32 token slots, or None"},
    {"pack_i32", pack_i32, METH_O, "list or tuple of ints (or of lists of ints) -> bytes of native int32"},
    {NULL, NULL, 0, NULL}};

static struct PyModuleDef module = {PyModuleDef_HEAD_INIT, "_kvcm_pylist", "index lists -> packed int32", -1, methods,
                                    NULL, NULL, NULL, NULL};

PyMODINIT_FUNC PyInit__kvcm_pylist(void) { return PyModule_Create(&module); }

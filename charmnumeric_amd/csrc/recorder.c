/* The recording hot path of the frontend as a CPython extension (module `_cnrec`).
 *
 * `Handle` is the C base type of the frontend's Array and ArrayView classes: it holds their fields
 * as C struct members (visible from Python under the names array.py uses) and implements the four
 * things a loop over array statements spends its time in -- indexing (`u[1:-1, :-2]`), the binary
 * operators, slice assignment and the deletion record of a dying array -- for the common forms:
 * keys made of integers and slices, operands that are two arrays of one element type and shape or
 * an array and a plain Python number. Everything else (ellipsis, broadcasting one-element arrays,
 * mixed element types, host data, every error message) is handed to the Python implementation in
 * array.py, which stays the definition of the behaviour: with `set_fast(0)` every call goes there,
 * and the statement logs of both routes are compared byte for byte in the tests.
 *
 * Upstream's counterpart is the operator and slicing code of charmnumeric/charmnumeric.py:272-343
 * and :394-489 together with charmtyles' recording calls behind it.
 *
 * Record layouts (little endian, include/cnexec.h):
 *   head    6 x i32   kind, name, opcode, dtype, n_operands, aux
 *   shape   4 x i32   ndims, extent[3] (unused = 0)
 *   ref    15 x i32   1, name, base_ndims, dtype, broadcast, has_region, start[3], stop[3], step[3]
 *   scalar  i32 0, i32 0, f64 value
 *   region 10 x i32   ndims, start[3], stop[3], step[3]
 *   delete  2 x i32   5, name
 */
#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <structmember.h>
#include <stdint.h>
#include <string.h>

enum { KIND_OP = 2, KIND_SET = 3, KIND_DELETE = 5 };
enum { REF_BYTES = 60, SCALAR_BYTES = 16, HEAD_BYTES = 24, SHAPE_BYTES = 16, REGION_BYTES = 40 };

typedef struct {
    PyObject_HEAD
    PyObject* shape;     /* tuple of ints */
    PyObject* dtype;     /* numpy dtype */
    PyObject* rb;        /* cached operand bytes, or NULL */
    PyObject* base;      /* views: the array they look into; arrays: NULL */
    PyObject* region;    /* views: (start, stop, step), each a tuple of ints, in base coordinates */
    PyObject* all_ones;  /* arrays: truthy while every element is known to be 1 */
    long long n;         /* elements */
    int ndims, wire, name, gen;
} Handle;

static PyTypeObject HandleType;

/* set by setup() */
static PyObject* g_state;          /* lazy._state */
static PyTypeObject* g_array_type; /* array.Array */
static PyTypeObject* g_view_type;  /* array.ArrayView */
static PyObject *g_py_getitem, *g_py_setitem, *g_py_binary, *g_flush_if_due;
static int g_op[4];                /* opcodes of + - * / */
static int g_fast = 1;
static PyObject *s_pending, *s_next_name, *s_generation, *s_flush_at, *s_in_expression;

static int is_handle(PyObject* o) { return PyObject_TypeCheck(o, &HandleType); }
static int is_view(const Handle* h) { return h->base != NULL && h->base != Py_None; }

/* ---- small helpers ---- */

static int ints_of(PyObject* tuple, int nd, int* out) {
    if (tuple == NULL || !PyTuple_CheckExact(tuple) || PyTuple_GET_SIZE(tuple) != nd)
        return -1;
    for (int d = 0; d < nd; ++d) {
        long v = PyLong_AsLong(PyTuple_GET_ITEM(tuple, d));
        if (v == -1 && PyErr_Occurred()) {
            PyErr_Clear();
            return -1;
        }
        if (v < INT32_MIN || v > INT32_MAX)
            return -1;
        out[d] = (int)v;
    }
    return 0;
}

static PyObject* tuple_of(int nd, const int* v) {
    PyObject* t = PyTuple_New(nd);
    if (t == NULL)
        return NULL;
    for (int d = 0; d < nd; ++d) {
        PyObject* x = PyLong_FromLong(v[d]);
        if (x == NULL) {
            Py_DECREF(t);
            return NULL;
        }
        PyTuple_SET_ITEM(t, d, x);
    }
    return t;
}

static void put_i32(char* p, int32_t v) { memcpy(p, &v, 4); }

static long long state_int(PyObject* attr, int* ok) {
    PyObject* v = PyObject_GetAttr(g_state, attr);
    if (v == NULL) {
        *ok = 0;
        return 0;
    }
    long long x = PyLong_AsLongLong(v);
    Py_DECREF(v);
    if (x == -1 && PyErr_Occurred()) {
        *ok = 0;
        return 0;
    }
    return x;
}

/* Appends one record to the log. `expression`: 1 an elementwise operation, 0 an assignment (both
 * flush first when an automatic flush is due), -1 a deletion (never flushes). Steals `record`. */
static int log_append(PyObject* record, int expression) {
    if (record == NULL)
        return -1;
    PyObject* pending = PyObject_GetAttr(g_state, s_pending);
    if (pending == NULL || !PyList_CheckExact(pending)) {
        Py_XDECREF(pending);
        Py_DECREF(record);
        if (!PyErr_Occurred())
            PyErr_SetString(PyExc_RuntimeError, "the statement log is not a list");
        return -1;
    }
    if (expression >= 0) {
        int ok = 1;
        const long long flush_at = state_int(s_flush_at, &ok);
        if (!ok) {
            Py_DECREF(pending);
            Py_DECREF(record);
            return -1;
        }
        if ((long long)PyList_GET_SIZE(pending) >= flush_at) {
            PyObject* r = PyObject_CallNoArgs(g_flush_if_due);
            Py_DECREF(pending);
            if (r == NULL) {
                Py_DECREF(record);
                return -1;
            }
            Py_DECREF(r);
            pending = PyObject_GetAttr(g_state, s_pending);   /* a flush starts a new list */
            if (pending == NULL || !PyList_CheckExact(pending)) {
                Py_XDECREF(pending);
                Py_DECREF(record);
                return -1;
            }
        }
        if (PyObject_SetAttr(g_state, s_in_expression, expression ? Py_True : Py_False) < 0) {
            Py_DECREF(pending);
            Py_DECREF(record);
            return -1;
        }
    }
    const int rc = PyList_Append(pending, record);
    Py_DECREF(pending);
    Py_DECREF(record);
    return rc;
}

/* The 60 bytes that name `h` as an operand (cached on the object). New reference, or NULL with
 * *fallback set when the object is not in a state this code handles. */
static PyObject* operand_bytes(Handle* h, int* fallback) {
    if (h->rb != NULL && h->rb != Py_None && PyBytes_CheckExact(h->rb) && PyBytes_GET_SIZE(h->rb) == REF_BYTES) {
        Py_INCREF(h->rb);
        return h->rb;
    }
    int32_t f[15] = {1, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    if (is_view(h)) {
        if (!is_handle(h->base)) {
            *fallback = 1;
            return NULL;
        }
        Handle* b = (Handle*)h->base;
        const int nd = b->ndims;
        int bs[3], r[3][3];
        if (nd < 1 || nd > 3 || h->region == NULL || !PyTuple_CheckExact(h->region) ||
            PyTuple_GET_SIZE(h->region) != 3 || ints_of(b->shape, nd, bs) < 0) {
            *fallback = 1;
            return NULL;
        }
        for (int k = 0; k < 3; ++k)
            if (ints_of(PyTuple_GET_ITEM(h->region, k), nd, r[k]) < 0) {
                *fallback = 1;
                return NULL;
            }
        int whole = h->n == b->n;
        for (int d = 0; d < nd && whole; ++d)
            whole = r[0][d] == 0 && r[1][d] == bs[d] && r[2][d] == 1;
        f[1] = b->name;
        f[2] = nd;
        f[3] = h->wire;
        if (!whole) {
            f[5] = 1;
            for (int d = 0; d < nd; ++d) {
                f[6 + d] = r[0][d];
                f[9 + d] = r[1][d];
                f[12 + d] = r[2][d];
            }
        }
    } else {
        f[1] = h->name;
        f[2] = h->ndims;
        f[3] = h->wire;
    }
    PyObject* out = PyBytes_FromStringAndSize((const char*)f, REF_BYTES);
    if (out == NULL)
        return NULL;
    Py_INCREF(out);
    Py_XSETREF(h->rb, out);
    return out;
}

/* A plain Python float or int as the 16 bytes of a literal operand. */
static int scalar_bytes(PyObject* v, char* dst) {
    double x;
    if (PyFloat_CheckExact(v))
        x = PyFloat_AS_DOUBLE(v);
    else if (PyLong_CheckExact(v)) {
        x = PyLong_AsDouble(v);
        if (x == -1.0 && PyErr_Occurred()) {
            PyErr_Clear();
            return -1;
        }
    } else
        return -1;
    put_i32(dst, 0);
    put_i32(dst + 4, 0);
    memcpy(dst + 8, &x, 8);
    return 0;
}

/* ---- keys ---- */

/* (start, stop, step) of `key` on an object of `shape`, for keys of integers and slices with
 * positive steps that name at most nd dimensions. 0 on success, 1 when Python should take over. */
static int parse_key(PyObject* key, int nd, const int* shape, int* start, int* stop, int* step) {
    PyObject* single[1] = {key};
    PyObject** items = single;
    Py_ssize_t count = 1;
    if (PyTuple_CheckExact(key)) {
        count = PyTuple_GET_SIZE(key);
        items = &PyTuple_GET_ITEM(key, 0);
    }
    if (count > nd)
        return 1;
    for (int d = 0; d < nd; ++d) {
        start[d] = 0;
        stop[d] = shape[d];
        step[d] = 1;
    }
    for (Py_ssize_t d = 0; d < count; ++d) {
        PyObject* item = items[d];
        if (PyLong_CheckExact(item)) {
            long v = PyLong_AsLong(item);
            if (v == -1 && PyErr_Occurred()) {
                PyErr_Clear();
                return 1;
            }
            if (v < 0)
                v += shape[d];
            if (v < 0 || v >= shape[d])
                return 1;
            start[d] = (int)v;
            stop[d] = (int)v + 1;
        } else if (PySlice_Check(item)) {
            Py_ssize_t s, e, st;
            if (PySlice_Unpack(item, &s, &e, &st) < 0) {
                PyErr_Clear();
                return 1;
            }
            if (st <= 0)
                return 1;
            PySlice_AdjustIndices(shape[d], &s, &e, st);
            if (st > INT32_MAX)
                return 1;
            start[d] = (int)s;
            stop[d] = (int)e;
            step[d] = (int)st;
        } else
            return 1;
    }
    return 0;
}

/* `inner` (relative to the view `h`, or to the array `h`) in the base array's coordinates, and the
 * extents it selects. 0 on success, 1 for Python (empty selections, malformed objects). */
static int compose(Handle* h, int nd, int* start, int* stop, int* step, int* extent, long long* elems) {
    if (is_view(h)) {
        int o[3][3];
        if (h->region == NULL || !PyTuple_CheckExact(h->region) || PyTuple_GET_SIZE(h->region) != 3)
            return 1;
        for (int k = 0; k < 3; ++k)
            if (ints_of(PyTuple_GET_ITEM(h->region, k), nd, o[k]) < 0)
                return 1;
        int unit = 1;
        for (int d = 0; d < nd; ++d)
            unit = unit && step[d] == 1 && o[2][d] == 1;
        for (int d = 0; d < nd; ++d) {
            if (unit) {
                start[d] += o[0][d];
                stop[d] += o[0][d];
            } else {
                const long long cnt = stop[d] > start[d] ? ((long long)stop[d] - start[d] + step[d] - 1) / step[d] : 0;
                const long long first = (long long)o[0][d] + (long long)start[d] * o[2][d];
                const long long st = (long long)o[2][d] * step[d];
                const long long last = cnt ? first + (cnt - 1) * st + 1 : first;
                if (st > INT32_MAX || last > INT32_MAX)
                    return 1;
                start[d] = (int)first;
                step[d] = (int)st;
                stop[d] = (int)last;
            }
        }
    }
    long long n = 1;
    for (int d = 0; d < nd; ++d) {
        const long long cnt = stop[d] > start[d] ? ((long long)stop[d] - start[d] + step[d] - 1) / step[d] : 0;
        if (cnt <= 0)
            return 1;
        extent[d] = (int)cnt;
        n *= cnt;
    }
    *elems = n;
    return 0;
}

static PyObject* region_tuple(int nd, const int* start, const int* stop, const int* step) {
    PyObject *a = tuple_of(nd, start), *b = tuple_of(nd, stop), *c = tuple_of(nd, step);
    PyObject* out = (a && b && c) ? PyTuple_Pack(3, a, b, c) : NULL;
    Py_XDECREF(a);
    Py_XDECREF(b);
    Py_XDECREF(c);
    return out;
}

/* ---- indexing ---- */

static PyObject* handle_subscript(PyObject* self, PyObject* key) {
    Handle* h = (Handle*)self;
    const int nd = h->ndims;
    int shape[3], start[3], stop[3], step[3], extent[3];
    long long elems = 0;
    if (!g_fast || g_view_type == NULL || nd < 1 || nd > 3 || ints_of(h->shape, nd, shape) < 0 ||
        parse_key(key, nd, shape, start, stop, step) || compose(h, nd, start, stop, step, extent, &elems))
        return PyObject_CallFunctionObjArgs(g_py_getitem, self, key, NULL);
    Handle* base = is_view(h) ? (Handle*)h->base : h;
    Handle* v = (Handle*)g_view_type->tp_alloc(g_view_type, 0);
    if (v == NULL)
        return NULL;
    v->region = region_tuple(nd, start, stop, step);
    v->shape = tuple_of(nd, extent);
    if (v->region == NULL || v->shape == NULL) {
        Py_DECREF(v);
        return NULL;
    }
    Py_INCREF(base);
    v->base = (PyObject*)base;
    Py_XINCREF(base->dtype);
    v->dtype = base->dtype;
    v->ndims = base->ndims;
    v->wire = base->wire;
    v->n = elems;
    return (PyObject*)v;
}

/* ---- assignment into a slice ---- */

static int handle_ass_subscript(PyObject* self, PyObject* key, PyObject* value) {
    if (value == NULL) {
        PyErr_SetString(PyExc_TypeError, "charmnumeric arrays do not support item deletion");
        return -1;
    }
    Handle* h = (Handle*)self;
    const int nd = h->ndims;
    int shape[3], start[3], stop[3], step[3], extent[3];
    long long elems = 0;
    char operand[REF_BYTES];
    Py_ssize_t operand_len = 0;
    int fallback = !g_fast || nd < 1 || nd > 3 || ints_of(h->shape, nd, shape) < 0 ||
                   parse_key(key, nd, shape, start, stop, step) || compose(h, nd, start, stop, step, extent, &elems);
    Handle* base = is_view(h) ? (Handle*)h->base : h;
    if (!fallback && !is_handle((PyObject*)base))
        fallback = 1;
    if (!fallback) {
        if (is_handle(value)) {
            Handle* r = (Handle*)value;
            int rs[3];
            if (r->wire != base->wire || r->ndims != nd || ints_of(r->shape, nd, rs) < 0)
                fallback = 1;
            for (int d = 0; d < nd && !fallback; ++d)
                fallback = rs[d] != extent[d];
            if (!fallback) {
                PyObject* rb = operand_bytes(r, &fallback);
                if (rb == NULL && !fallback)
                    return -1;
                if (rb != NULL) {
                    memcpy(operand, PyBytes_AS_STRING(rb), REF_BYTES);
                    operand_len = REF_BYTES;
                    Py_DECREF(rb);
                }
            }
        } else if (scalar_bytes(value, operand) == 0)
            operand_len = SCALAR_BYTES;
        else
            fallback = 1;
    }
    if (fallback) {
        PyObject* r = PyObject_CallFunctionObjArgs(g_py_setitem, self, key, value, NULL);
        if (r == NULL)
            return -1;
        Py_DECREF(r);
        return 0;
    }
    Py_INCREF(Py_False);
    Py_XSETREF(base->all_ones, Py_False);
    PyObject* rec = PyBytes_FromStringAndSize(NULL, HEAD_BYTES + SHAPE_BYTES + REGION_BYTES + operand_len);
    if (rec == NULL)
        return -1;
    char* p = PyBytes_AS_STRING(rec);
    const int32_t head[6] = {KIND_SET, base->name, 0, base->wire, 1, nd};
    memcpy(p, head, HEAD_BYTES);
    p += HEAD_BYTES;
    int32_t sh[4] = {nd, 0, 0, 0}, rg[10] = {nd, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    for (int d = 0; d < nd; ++d) {
        sh[1 + d] = extent[d];
        rg[1 + d] = start[d];
        rg[4 + d] = stop[d];
        rg[7 + d] = step[d];
    }
    memcpy(p, sh, SHAPE_BYTES);
    p += SHAPE_BYTES;
    memcpy(p, rg, REGION_BYTES);
    p += REGION_BYTES;
    memcpy(p, operand, (size_t)operand_len);
    return log_append(rec, 0);
}

/* ---- binary operators ---- */

static PyObject* binary(int which, PyObject* a, PyObject* b) {
    const int la = is_handle(a), lb = is_handle(b);
    Handle* like = NULL;
    char oa[REF_BYTES], ob[REF_BYTES];
    Py_ssize_t na = 0, nb = 0;
    int fallback = !g_fast || g_array_type == NULL;
    if (!fallback && la && lb) {
        Handle *x = (Handle*)a, *y = (Handle*)b;
        int xs[3], ys[3];
        if (x->wire != y->wire || x->ndims != y->ndims || x->n <= 1 || y->n <= 1 || x->ndims < 1 || x->ndims > 3 ||
            ints_of(x->shape, x->ndims, xs) < 0 || ints_of(y->shape, y->ndims, ys) < 0)
            fallback = 1;
        for (int d = 0; !fallback && d < x->ndims; ++d)
            fallback = xs[d] != ys[d];
        like = x;
    } else if (!fallback && la) {
        like = (Handle*)a;
        fallback = scalar_bytes(b, ob) != 0;
        nb = SCALAR_BYTES;
    } else if (!fallback && lb) {
        like = (Handle*)b;
        fallback = scalar_bytes(a, oa) != 0;
        na = SCALAR_BYTES;
    } else
        fallback = 1;
    int ls[3];
    if (!fallback && (like->ndims < 1 || like->ndims > 3 || ints_of(like->shape, like->ndims, ls) < 0))
        fallback = 1;
    if (!fallback && la) {
        PyObject* rb = operand_bytes((Handle*)a, &fallback);
        if (rb == NULL && !fallback)
            return NULL;
        if (rb != NULL) {
            memcpy(oa, PyBytes_AS_STRING(rb), REF_BYTES);
            na = REF_BYTES;
            Py_DECREF(rb);
        }
    }
    if (!fallback && lb) {
        PyObject* rb = operand_bytes((Handle*)b, &fallback);
        if (rb == NULL && !fallback)
            return NULL;
        if (rb != NULL) {
            memcpy(ob, PyBytes_AS_STRING(rb), REF_BYTES);
            nb = REF_BYTES;
            Py_DECREF(rb);
        }
    }
    if (fallback) {
        if (!la && !lb)
            Py_RETURN_NOTIMPLEMENTED;
        PyObject* op = PyLong_FromLong(g_op[which]);
        if (op == NULL)
            return NULL;
        PyObject* r = PyObject_CallFunctionObjArgs(g_py_binary, op, a, b, NULL);
        Py_DECREF(op);
        return r;
    }
    int ok = 1;
    const long long name = state_int(s_next_name, &ok), gen = state_int(s_generation, &ok);
    if (!ok)
        return NULL;
    PyObject* next = PyLong_FromLongLong(name + 1);
    if (next == NULL || PyObject_SetAttr(g_state, s_next_name, next) < 0) {
        Py_XDECREF(next);
        return NULL;
    }
    Py_DECREF(next);
    Handle* out = (Handle*)g_array_type->tp_alloc(g_array_type, 0);
    if (out == NULL)
        return NULL;
    Py_XINCREF(like->shape);
    out->shape = like->shape;
    Py_XINCREF(like->dtype);
    out->dtype = like->dtype;
    out->ndims = like->ndims;
    out->wire = like->wire;
    out->n = like->n;
    out->name = (int)name;
    out->gen = (int)gen;
    PyObject* rec = PyBytes_FromStringAndSize(NULL, HEAD_BYTES + SHAPE_BYTES + na + nb);
    if (rec == NULL) {
        out->name = 0;                      /* never recorded: nothing to delete */
        Py_DECREF(out);
        return NULL;
    }
    char* p = PyBytes_AS_STRING(rec);
    const int32_t head[6] = {KIND_OP, (int32_t)name, g_op[which], like->wire, 2, 0};
    memcpy(p, head, HEAD_BYTES);
    p += HEAD_BYTES;
    int32_t sh[4] = {like->ndims, 0, 0, 0};
    for (int d = 0; d < like->ndims; ++d)
        sh[1 + d] = ls[d];
    memcpy(p, sh, SHAPE_BYTES);
    p += SHAPE_BYTES;
    memcpy(p, oa, (size_t)na);
    p += na;
    memcpy(p, ob, (size_t)nb);
    if (log_append(rec, 1) < 0) {
        out->name = 0;                      /* never recorded: nothing to delete */
        Py_DECREF(out);
        return NULL;
    }
    return (PyObject*)out;
}

static PyObject* handle_add(PyObject* a, PyObject* b) { return binary(0, a, b); }
static PyObject* handle_sub(PyObject* a, PyObject* b) { return binary(1, a, b); }
static PyObject* handle_mul(PyObject* a, PyObject* b) { return binary(2, a, b); }
static PyObject* handle_div(PyObject* a, PyObject* b) { return binary(3, a, b); }
static PyObject* handle_neg(PyObject* a) {
    /* upstream spells negation as multiplication by -1 (charmnumeric.py:427-434) */
    PyObject* minus_one = PyLong_FromLong(-1);
    if (minus_one == NULL)
        return NULL;
    PyObject* r = binary(2, a, minus_one);
    Py_DECREF(minus_one);
    return r;
}

/* ---- life cycle ---- */

static PyObject* handle_new(PyTypeObject* type, PyObject* args, PyObject* kwds) {
    (void)args;
    (void)kwds;
    return type->tp_alloc(type, 0);      /* all fields zero; __init__ of the subclass fills them */
}

/* An array that dies leaves a deletion record (a handle from before the last reset() names nothing
 * any more). Never flushes: it may run at any point, even while the interpreter shuts down. */
static void handle_finalize(PyObject* self) {
    Handle* h = (Handle*)self;
    if (is_view(h) || h->name <= 0 || g_state == NULL)
        return;
    PyObject *et, *ev, *tb;
    PyErr_Fetch(&et, &ev, &tb);
    int ok = 1;
    const long long gen = state_int(s_generation, &ok);
    if (ok && gen == h->gen) {
        const int32_t rec[2] = {KIND_DELETE, h->name};
        log_append(PyBytes_FromStringAndSize((const char*)rec, 8), -1);
    }
    PyErr_Clear();
    PyErr_Restore(et, ev, tb);
}

static int handle_traverse(PyObject* self, visitproc visit, void* arg) {
    Handle* h = (Handle*)self;
    Py_VISIT(h->shape);
    Py_VISIT(h->dtype);
    Py_VISIT(h->rb);
    Py_VISIT(h->base);
    Py_VISIT(h->region);
    Py_VISIT(h->all_ones);
    return 0;
}

static int handle_clear(PyObject* self) {
    Handle* h = (Handle*)self;
    Py_CLEAR(h->shape);
    Py_CLEAR(h->dtype);
    Py_CLEAR(h->rb);
    Py_CLEAR(h->base);
    Py_CLEAR(h->region);
    Py_CLEAR(h->all_ones);
    return 0;
}

static void handle_dealloc(PyObject* self) {
    if (PyObject_CallFinalizerFromDealloc(self) < 0)
        return;                                /* resurrected */
    PyObject_GC_UnTrack(self);
    handle_clear(self);
    Py_TYPE(self)->tp_free(self);
}

static PyMemberDef handle_members[] = {
    {"shape", T_OBJECT, offsetof(Handle, shape), 0, "extents"},
    {"dtype", T_OBJECT, offsetof(Handle, dtype), 0, "numpy element type"},
    {"_rb", T_OBJECT, offsetof(Handle, rb), 0, "cached operand bytes"},
    {"base", T_OBJECT, offsetof(Handle, base), 0, "views: the array looked into"},
    {"region", T_OBJECT, offsetof(Handle, region), 0, "views: (start, stop, step) in base coordinates"},
    {"_all_ones", T_OBJECT, offsetof(Handle, all_ones), 0, "arrays: every element known to be 1"},
    {"_n", T_LONGLONG, offsetof(Handle, n), 0, "elements"},
    {"ndims", T_INT, offsetof(Handle, ndims), 0, "rank"},
    {"_wire", T_INT, offsetof(Handle, wire), 0, "element type number of the executor"},
    {"name", T_INT, offsetof(Handle, name), 0, "arrays: name in the executor"},
    {"_gen", T_INT, offsetof(Handle, gen), 0, "arrays: reset() generation of the name"},
    {NULL, 0, 0, 0, NULL}};

static PyNumberMethods handle_number = {
    .nb_add = handle_add,
    .nb_subtract = handle_sub,
    .nb_multiply = handle_mul,
    .nb_true_divide = handle_div,
    .nb_negative = handle_neg,
};

static PyMappingMethods handle_mapping = {
    .mp_subscript = handle_subscript,
    .mp_ass_subscript = handle_ass_subscript,
};

static PyTypeObject HandleType = {
    PyVarObject_HEAD_INIT(NULL, 0).tp_name = "charmnumeric_amd._cnrec.Handle",
    .tp_basicsize = sizeof(Handle),
    .tp_flags = Py_TPFLAGS_DEFAULT | Py_TPFLAGS_BASETYPE | Py_TPFLAGS_HAVE_GC,
    .tp_doc = "C base of Array and ArrayView: fields and the recording fast paths",
    .tp_new = handle_new,
    .tp_dealloc = handle_dealloc,
    .tp_finalize = handle_finalize,
    .tp_traverse = handle_traverse,
    .tp_clear = handle_clear,
    .tp_members = handle_members,
    .tp_as_number = &handle_number,
    .tp_as_mapping = &handle_mapping,
};

/* ---- module ---- */

static PyObject* mod_setup(PyObject* self, PyObject* args) {
    (void)self;
    PyObject *state, *array_type, *view_type, *getitem, *setitem, *binop, *flush;
    int add, sub, mul, div;
    if (!PyArg_ParseTuple(args, "OOOOOOO(iiii)", &state, &array_type, &view_type, &getitem, &setitem, &binop, &flush,
                          &add, &sub, &mul, &div))
        return NULL;
    if (!PyType_Check(array_type) || !PyType_Check(view_type) ||
        !PyType_IsSubtype((PyTypeObject*)array_type, &HandleType) ||
        !PyType_IsSubtype((PyTypeObject*)view_type, &HandleType)) {
        PyErr_SetString(PyExc_TypeError, "Array and ArrayView must derive from Handle");
        return NULL;
    }
    Py_INCREF(state);
    Py_XSETREF(g_state, state);
    Py_INCREF(array_type);
    Py_XDECREF((PyObject*)g_array_type);
    g_array_type = (PyTypeObject*)array_type;
    Py_INCREF(view_type);
    Py_XDECREF((PyObject*)g_view_type);
    g_view_type = (PyTypeObject*)view_type;
    Py_INCREF(getitem);
    Py_XSETREF(g_py_getitem, getitem);
    Py_INCREF(setitem);
    Py_XSETREF(g_py_setitem, setitem);
    Py_INCREF(binop);
    Py_XSETREF(g_py_binary, binop);
    Py_INCREF(flush);
    Py_XSETREF(g_flush_if_due, flush);
    g_op[0] = add;
    g_op[1] = sub;
    g_op[2] = mul;
    g_op[3] = div;
    Py_RETURN_NONE;
}

static PyObject* mod_set_fast(PyObject* self, PyObject* arg) {
    (void)self;
    const int v = PyObject_IsTrue(arg);
    if (v < 0)
        return NULL;
    const int before = g_fast;
    g_fast = v;
    return PyBool_FromLong(before);
}

static PyMethodDef mod_methods[] = {
    {"setup", mod_setup, METH_VARARGS,
     "setup(state, Array, ArrayView, getitem, setitem, binary, flush_if_due, (add, sub, mul, div))"},
    {"set_fast", mod_set_fast, METH_O, "set_fast(on) -> previous setting; off: every call takes the Python route"},
    {NULL, NULL, 0, NULL}};

static struct PyModuleDef mod_def = {PyModuleDef_HEAD_INIT, "_cnrec", "recording hot path of the frontend", -1,
                                     mod_methods, NULL, NULL, NULL, NULL};

PyMODINIT_FUNC PyInit__cnrec(void) {
    if (PyType_Ready(&HandleType) < 0)
        return NULL;
    PyObject* m = PyModule_Create(&mod_def);
    if (m == NULL)
        return NULL;
    s_pending = PyUnicode_InternFromString("pending");
    s_next_name = PyUnicode_InternFromString("next_name");
    s_generation = PyUnicode_InternFromString("generation");
    s_flush_at = PyUnicode_InternFromString("flush_at");
    s_in_expression = PyUnicode_InternFromString("in_expression");
    Py_INCREF(&HandleType);
    if (PyModule_AddObject(m, "Handle", (PyObject*)&HandleType) < 0) {
        Py_DECREF(&HandleType);
        Py_DECREF(m);
        return NULL;
    }
    return m;
}

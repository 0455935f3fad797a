/* Host-side replay of a repeated single statement, as a CPython extension.
 *
 * A statement `out[:] = expr` that the backend has run before costs, in Python,
 * one walk over the op-tree (the key of the launch cache), a dictionary lookup
 * and one call through ctypes per recorded launch.  This module does the same
 * three steps in C: `Replayer.replay(out, value)` walks the tree, builds the very
 * key `NervanaHIPBase._launch_key` builds, looks it up in the backend's launch
 * cache and calls `nh_launch_prepared` (include/neonhip.h) on the entry's launch
 * records.  Anything it does not recognise -- a key that is not in the cache, an
 * entry without prepared records, numbers that differ from the recorded ones, an
 * operand type it does not know -- is answered with 0 and the caller takes the
 * general Python path; nothing is decided here that the Python path would decide
 * differently.  The role of the reference's per-call argument derivation that its
 * own comment wants cached (neon/backends/float_ew.py:640-641).
 *
 * No GPU headers: the launch function is handed over as an address at set-up.
 */
#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <structmember.h>
#include <stdint.h>

typedef int (*launch_fn)(const void*);

static PyObject *s_geom, *s_op, *s_axis, *s_idx, *s_fast, *s_bar, *s_assign;

/* ---- Records: the launch records and numbers of one cache entry --------------------- */
typedef struct {
    PyObject_HEAD
    Py_ssize_t nrec, nraw;
    const void** recs;
    double* raw;
    PyObject* keep;          /* whatever owns the memory the records point into */
    PyObject* coop;          /* NULL, or a tuple of (key, plan): plans whose workgroups wait for one another,
                              * to be entered into the replayer's table of plans to check after each replay */
} Records;

/* (both types take part in cycle collection: backend -> replayer -> launch cache -> entry ->
 * records / temporaries -> tensors -> backend is a cycle the collector has to see through) */
static int Records_traverse(Records* self, visitproc visit, void* arg) {
    Py_VISIT(self->keep);
    Py_VISIT(self->coop);
    return 0;
}

static int Records_clear(Records* self) {
    Py_CLEAR(self->keep);
    Py_CLEAR(self->coop);
    return 0;
}

static void Records_dealloc(Records* self) {
    PyObject_GC_UnTrack(self);
    PyMem_Free((void*)self->recs);
    PyMem_Free(self->raw);
    Py_XDECREF(self->keep);
    Py_XDECREF(self->coop);
    Py_TYPE(self)->tp_free((PyObject*)self);
}

static int fill_raw(Records* self, PyObject* seq) {
    PyObject* fast = PySequence_Fast(seq, "numbers must be a sequence");
    if (!fast) return -1;
    Py_ssize_t n = PySequence_Fast_GET_SIZE(fast);
    double* raw = (double*)PyMem_Malloc((n ? n : 1) * sizeof(double));
    if (!raw) { Py_DECREF(fast); PyErr_NoMemory(); return -1; }
    for (Py_ssize_t i = 0; i < n; ++i) {
        raw[i] = PyFloat_AsDouble(PySequence_Fast_GET_ITEM(fast, i));
        if (raw[i] == -1.0 && PyErr_Occurred()) { PyMem_Free(raw); Py_DECREF(fast); return -1; }
    }
    Py_DECREF(fast);
    PyMem_Free(self->raw);
    self->raw = raw;
    self->nraw = n;
    return 0;
}

static PyObject* Records_new(PyTypeObject* type, PyObject* args, PyObject* kw) {
    PyObject *addresses, *numbers, *keep, *coop = NULL;
    if (!PyArg_ParseTuple(args, "OOO|O:Records", &addresses, &numbers, &keep, &coop)) return NULL;
    if (coop == Py_None) coop = NULL;
    if (coop) {
        int ok = PyTuple_Check(coop);
        for (Py_ssize_t i = 0; ok && i < PyTuple_GET_SIZE(coop); ++i) {
            PyObject* item = PyTuple_GET_ITEM(coop, i);
            ok = PyTuple_Check(item) && PyTuple_GET_SIZE(item) == 2;
        }
        if (!ok) { PyErr_SetString(PyExc_TypeError, "coop must be a tuple of (key, plan) pairs"); return NULL; }
    }
    PyObject* fast = PySequence_Fast(addresses, "addresses must be a sequence");
    if (!fast) return NULL;
    Records* self = (Records*)type->tp_alloc(type, 0);
    if (!self) { Py_DECREF(fast); return NULL; }
    self->nrec = PySequence_Fast_GET_SIZE(fast);
    self->recs = (const void**)PyMem_Malloc((self->nrec ? self->nrec : 1) * sizeof(void*));
    if (!self->recs) { Py_DECREF(fast); Py_DECREF(self); return PyErr_NoMemory(); }
    for (Py_ssize_t i = 0; i < self->nrec; ++i) {
        self->recs[i] = PyLong_AsVoidPtr(PySequence_Fast_GET_ITEM(fast, i));
        if (!self->recs[i]) {
            if (!PyErr_Occurred()) PyErr_SetString(PyExc_ValueError, "null launch record");
            Py_DECREF(fast); Py_DECREF(self); return NULL;
        }
    }
    Py_DECREF(fast);
    if (fill_raw(self, numbers) < 0) { Py_DECREF(self); return NULL; }
    Py_INCREF(keep);
    self->keep = keep;
    Py_XINCREF(coop);
    self->coop = coop;
    return (PyObject*)self;
}

static PyObject* Records_set_numbers(Records* self, PyObject* numbers) {
    if (fill_raw(self, numbers) < 0) return NULL;
    Py_RETURN_NONE;
}

static PyMethodDef Records_methods[] = {
    {"set_numbers", (PyCFunction)Records_set_numbers, METH_O,
     "the numbers the records' argument buffers now hold"},
    {NULL, NULL, 0, NULL}};

static PyMemberDef Records_members[] = {
    {"launches", T_PYSSIZET, offsetof(Records, nrec), READONLY, "number of launch records"},
    {NULL, 0, 0, 0, NULL}};

static PyTypeObject RecordsType = {
    PyVarObject_HEAD_INIT(NULL, 0)
    .tp_name = "neon_amd._fastpath.Records",
    .tp_basicsize = sizeof(Records),
    .tp_dealloc = (destructor)Records_dealloc,
    .tp_flags = Py_TPFLAGS_DEFAULT | Py_TPFLAGS_HAVE_GC,
    .tp_traverse = (traverseproc)Records_traverse,
    .tp_clear = (inquiry)Records_clear,
    .tp_doc = "Records(addresses, numbers, keep[, coop]): launch records of one statement",
    .tp_methods = Records_methods,
    .tp_members = Records_members,
    .tp_new = Records_new,
};

/* ---- the walk ------------------------------------------------------------------------- */
#define MAX_PARTS 512
#define MAX_RAW 128

typedef struct {
    PyObject* parts[MAX_PARTS];   /* owned references */
    Py_ssize_t nparts;
    double raw[MAX_RAW];
    Py_ssize_t nraw;
    PyTypeObject* tensor_cls;
    int depth;
} Walk;

/* 0 = ok, -1 = not replayable here (a Python error may be set; the caller clears it) */
static int push(Walk* w, PyObject* owned) {
    if (!owned) return -1;
    if (w->nparts >= MAX_PARTS) { Py_DECREF(owned); return -1; }
    w->parts[w->nparts++] = owned;
    return 0;
}

static int push_number(Walk* w, double v) {
    if (v == -1.0 && PyErr_Occurred()) return -1;
    if (w->nraw >= MAX_RAW) return -1;
    w->raw[w->nraw++] = v;
    Py_INCREF(Py_None);
    return push(w, Py_None);
}

static int walk_node(Walk* w, PyObject* d, PyObject* left, PyObject* right);

static int walk_operand(Walk* w, PyObject* x) {
    PyTypeObject* t = Py_TYPE(x);
    if (t == w->tensor_cls) return push(w, PyObject_GetAttr(x, s_geom));
    if (t == &PyFloat_Type) return push_number(w, PyFloat_AS_DOUBLE(x));
    if (t == &PyLong_Type) return push_number(w, PyLong_AsDouble(x));
    if (x == Py_None) return 0;
    if (PyTuple_Check(x)) {
        if (PyTuple_GET_SIZE(x) != 3) return -1;
        return walk_node(w, PyTuple_GET_ITEM(x, 0), PyTuple_GET_ITEM(x, 1), PyTuple_GET_ITEM(x, 2));
    }
    if (PyFloat_Check(x)) return push_number(w, PyFloat_AsDouble(x));
    if (PyLong_Check(x)) return push_number(w, PyLong_AsDouble(x));
    return -1;
}

static int walk_node(Walk* w, PyObject* d, PyObject* left, PyObject* right) {
    if (!PyDict_Check(d) || ++w->depth > 200) return -1;
    if (walk_operand(w, left) < 0 || walk_operand(w, right) < 0) return -1;
    w->depth--;
    PyObject* op = PyDict_GetItemWithError(d, s_op);             /* borrowed */
    if (!op || !PyUnicode_Check(op)) return -1;
    PyObject* axis = PyDict_GetItemWithError(d, s_axis);         /* borrowed */
    if (axis) {
        if (PyUnicode_CompareWithASCIIString(op, "onehot") == 0) {
            PyObject* idx = PyDict_GetItemWithError(d, s_idx);
            if (!idx) return -1;
            PyObject* g = PyObject_GetAttr(idx, s_geom);
            if (!g) return -1;
            PyObject* part = PyTuple_Pack(3, op, axis, g);
            Py_DECREF(g);
            return push(w, part);
        }
        return push(w, PyTuple_Pack(2, op, axis));
    }
    if (PyErr_Occurred()) return -1;
    if (PyUnicode_CompareWithASCIIString(op, "rand") == 0) return -1;     /* random trees are never replayed */
    Py_INCREF(op);
    return push(w, op);
}

/* ---- Replayer: one per backend instance ----------------------------------------------- */
typedef struct {
    PyObject_HEAD
    PyObject* cache;              /* the backend's launch cache (dict) */
    PyTypeObject* tensor_cls;
    launch_fn launch;
    PyObject* pending;            /* NULL, or the backend's dict of cooperative plans launched since it last
                                   * looked at their status words */
    long long replayed, launches;
} Replayer;

static int Replayer_traverse(Replayer* self, visitproc visit, void* arg) {
    Py_VISIT(self->cache);
    Py_VISIT((PyObject*)self->tensor_cls);
    Py_VISIT(self->pending);
    return 0;
}

static int Replayer_clear(Replayer* self) {
    Py_CLEAR(self->cache);
    Py_CLEAR(self->tensor_cls);
    Py_CLEAR(self->pending);
    return 0;
}

static void Replayer_dealloc(Replayer* self) {
    PyObject_GC_UnTrack(self);
    Py_XDECREF(self->cache);
    Py_XDECREF((PyObject*)self->tensor_cls);
    Py_XDECREF(self->pending);
    Py_TYPE(self)->tp_free((PyObject*)self);
}

static PyObject* Replayer_new(PyTypeObject* type, PyObject* args, PyObject* kw) {
    PyObject *cache, *cls, *fn, *pending = NULL;
    if (!PyArg_ParseTuple(args, "O!O!O|O!:Replayer", &PyDict_Type, &cache, &PyType_Type, &cls, &fn,
                          &PyDict_Type, &pending)) return NULL;
    void* p = PyLong_AsVoidPtr(fn);
    if (!p) {
        if (!PyErr_Occurred()) PyErr_SetString(PyExc_ValueError, "null launch function");
        return NULL;
    }
    Replayer* self = (Replayer*)type->tp_alloc(type, 0);
    if (!self) return NULL;
    Py_INCREF(cache);
    Py_INCREF(cls);
    self->cache = cache;
    self->tensor_cls = (PyTypeObject*)cls;
    self->launch = (launch_fn)p;
    Py_XINCREF(pending);
    self->pending = pending;
    return (PyObject*)self;
}

/* key(out, value) -> (key tuple, list of numbers): what replay() looks up; for tests */
static PyObject* build_key(Walk* w) {
    Py_INCREF(s_bar);
    if (push(w, s_bar) < 0) return NULL;
    PyObject* key = PyTuple_New(w->nparts);
    if (!key) return NULL;
    for (Py_ssize_t i = 0; i < w->nparts; ++i) PyTuple_SET_ITEM(key, i, w->parts[i]);   /* steals */
    w->nparts = 0;
    return key;
}

static void walk_release(Walk* w) {
    for (Py_ssize_t i = 0; i < w->nparts; ++i) Py_DECREF(w->parts[i]);
    w->nparts = 0;
}

static int walk_statement(Replayer* self, Walk* w, PyObject* out, PyObject* value) {
    w->nparts = w->nraw = 0;
    w->depth = 0;
    w->tensor_cls = self->tensor_cls;
    if (walk_operand(w, out) < 0 || walk_operand(w, value) < 0) return -1;
    Py_INCREF(s_assign);
    return push(w, s_assign);
}

static PyObject* Replayer_key(Replayer* self, PyObject* args) {
    PyObject *out, *value;
    if (!PyArg_ParseTuple(args, "OO:key", &out, &value)) return NULL;
    Walk w;
    if (walk_statement(self, &w, out, value) < 0) {
        walk_release(&w);
        if (!PyErr_Occurred()) PyErr_SetString(PyExc_TypeError, "not replayable");
        return NULL;
    }
    PyObject* key = build_key(&w);
    if (!key) { walk_release(&w); return NULL; }
    PyObject* nums = PyList_New(w.nraw);
    if (!nums) { Py_DECREF(key); return NULL; }
    for (Py_ssize_t i = 0; i < w.nraw; ++i) {
        PyObject* f = PyFloat_FromDouble(w.raw[i]);
        if (!f) { Py_DECREF(key); Py_DECREF(nums); return NULL; }
        PyList_SET_ITEM(nums, i, f);
    }
    PyObject* r = PyTuple_Pack(2, key, nums);
    Py_DECREF(key);
    Py_DECREF(nums);
    return r;
}

/* key_group(trees) -> (key tuple, list of numbers) of a GROUP of assign trees (each a 3-tuple
 * (op dict, target, value)): the key NervanaHIPBase._launch_key builds for the group.  Raises
 * TypeError when a tree is not replayable. */
static PyObject* Replayer_key_group(Replayer* self, PyObject* trees) {
    PyObject* fast = PySequence_Fast(trees, "key_group takes a sequence of assign trees");
    if (!fast) return NULL;
    Walk w;
    w.nparts = w.nraw = 0;
    w.depth = 0;
    w.tensor_cls = self->tensor_cls;
    Py_ssize_t n = PySequence_Fast_GET_SIZE(fast);
    for (Py_ssize_t k = 0; k < n; ++k) {
        PyObject* tree = PySequence_Fast_GET_ITEM(fast, k);
        int ok = PyTuple_Check(tree) && PyTuple_GET_SIZE(tree) == 3 &&
                 walk_node(&w, PyTuple_GET_ITEM(tree, 0), PyTuple_GET_ITEM(tree, 1), PyTuple_GET_ITEM(tree, 2)) == 0;
        if (ok) {
            Py_INCREF(s_bar);
            ok = push(&w, s_bar) == 0;
        }
        if (!ok) {
            walk_release(&w);
            Py_DECREF(fast);
            if (!PyErr_Occurred()) PyErr_SetString(PyExc_TypeError, "not replayable");
            return NULL;
        }
    }
    Py_DECREF(fast);
    PyObject* key = PyTuple_New(w.nparts);
    if (!key) { walk_release(&w); return NULL; }
    for (Py_ssize_t i = 0; i < w.nparts; ++i) PyTuple_SET_ITEM(key, i, w.parts[i]);   /* steals */
    w.nparts = 0;
    PyObject* nums = PyList_New(w.nraw);
    if (!nums) { Py_DECREF(key); return NULL; }
    for (Py_ssize_t i = 0; i < w.nraw; ++i) {
        PyObject* f = PyFloat_FromDouble(w.raw[i]);
        if (!f) { Py_DECREF(key); Py_DECREF(nums); return NULL; }
        PyList_SET_ITEM(nums, i, f);
    }
    PyObject* r = PyTuple_Pack(2, key, nums);
    Py_DECREF(key);
    Py_DECREF(nums);
    return r;
}

/* replay(out, value) -> 1: the statement's recorded launches were issued; 0: not handled here;
 * a negative number: minus the error code nh_launch_prepared returned (launches may be partly
 * issued; the recording has been dropped from the cache) */
static PyObject* Replayer_replay(Replayer* self, PyObject* const* args, Py_ssize_t nargs) {
    if (nargs != 2) { PyErr_SetString(PyExc_TypeError, "replay(out, value)"); return NULL; }
    Walk w;
    long result = 0;
    if (walk_statement(self, &w, args[0], args[1]) < 0) goto unhandled;
    {
        PyObject* key = build_key(&w);
        if (!key) goto unhandled;
        PyObject* entry = self->cache ? PyDict_GetItemWithError(self->cache, key) : NULL;      /* borrowed */
        if (!entry) { Py_DECREF(key); goto unhandled; }
        PyObject* recs = PyObject_GetAttr(entry, s_fast);
        if (!recs) { Py_DECREF(key); goto unhandled; }
        if (Py_TYPE(recs) == &RecordsType) {
            Records* r = (Records*)recs;
            int same = r->nraw == w.nraw;
            for (Py_ssize_t i = 0; same && i < w.nraw; ++i) same = r->raw[i] == w.raw[i];
            if (same && r->coop && !self->pending) same = 0;       /* nowhere to note the plans: not handled here */
            if (same) {
                result = 1;
                for (Py_ssize_t i = 0; i < r->nrec; ++i) {
                    int rc = self->launch(r->recs[i]);
                    if (rc) { result = -(long)rc; break; }
                }
                if (result == 1 && r->coop) {
                    for (Py_ssize_t i = 0; i < PyTuple_GET_SIZE(r->coop); ++i) {
                        PyObject* item = PyTuple_GET_ITEM(r->coop, i);
                        if (PyDict_SetItem(self->pending, PyTuple_GET_ITEM(item, 0), PyTuple_GET_ITEM(item, 1)) < 0) {
                            Py_DECREF(recs);
                            Py_DECREF(key);
                            return NULL;
                        }
                    }
                }
                if (result == 1) {
                    self->replayed += 1;
                    self->launches += r->nrec;
                } else if (PyDict_DelItem(self->cache, key) < 0) {
                    /* a recording whose launch failed is not offered again (the caller raises) */
                    PyErr_Clear();
                }
            }
        }
        Py_DECREF(recs);
        Py_DECREF(key);
        return PyLong_FromLong(result);
    }
unhandled:
    walk_release(&w);
    PyErr_Clear();
    return PyLong_FromLong(0);
}

static PyMemberDef Replayer_members[] = {
    {"replayed", T_LONGLONG, offsetof(Replayer, replayed), 0, "statements replayed here"},
    {"launches", T_LONGLONG, offsetof(Replayer, launches), 0, "launches issued here"},
    {NULL, 0, 0, 0, NULL}};

static PyMethodDef Replayer_methods[] = {
    {"replay", (PyCFunction)(void (*)(void))Replayer_replay, METH_FASTCALL,
     "replay(out, value) -> 1 issued, 0 not handled, < 0 minus the launch error code"},
    {"key", (PyCFunction)Replayer_key, METH_VARARGS, "key(out, value) -> (cache key, numbers)"},
    {"key_group", (PyCFunction)Replayer_key_group, METH_O,
     "key_group(assign trees) -> (cache key of the statement group, numbers)"},
    {NULL, NULL, 0, NULL}};

static PyTypeObject ReplayerType = {
    PyVarObject_HEAD_INIT(NULL, 0)
    .tp_name = "neon_amd._fastpath.Replayer",
    .tp_basicsize = sizeof(Replayer),
    .tp_dealloc = (destructor)Replayer_dealloc,
    .tp_flags = Py_TPFLAGS_DEFAULT | Py_TPFLAGS_HAVE_GC,
    .tp_traverse = (traverseproc)Replayer_traverse,
    .tp_clear = (inquiry)Replayer_clear,
    .tp_doc = "Replayer(launch_cache, tensor_class, address of nh_launch_prepared[, pending cooperative plans])",
    .tp_methods = Replayer_methods,
    .tp_members = Replayer_members,
    .tp_new = Replayer_new,
};

/* ---- elementwise node construction for the package's own API copy ---------------------- */
/* OpTreeNode.build(op, a, b) for an elementwise op without keyword arguments, as
 * neon_amd/backends/backend.py does it in Python (shape = per-axis maximum of the operand
 * shapes; numbers are 1x1, a missing operand 0x0, 1-d shapes padded to 2-d).  Anything it
 * is not sure about -- an op outside the set, an operand of an unknown type, a shape that is
 * not one or two integers -- is answered with None and Python takes over. */
static PyObject *b_node_cls, *b_tensor_cls, *b_ew_ops, *b_red_ops, *s_shape, *t_scalar, *t_none;

static PyObject* builder_configure(PyObject* self, PyObject* args) {
    PyObject *node_cls, *tensor_cls, *ops, *red_ops = NULL;
    if (!PyArg_ParseTuple(args, "O!O!O|O:configure_builder", &PyType_Type, &node_cls, &PyType_Type, &tensor_cls, &ops,
                          &red_ops))
        return NULL;
    if (!PyType_IsSubtype((PyTypeObject*)node_cls, &PyTuple_Type)) {
        PyErr_SetString(PyExc_TypeError, "the node class must derive from tuple");
        return NULL;
    }
    PyObject* frozen = PyFrozenSet_New(ops);
    if (!frozen) return NULL;
    PyObject* frozen_red = PyFrozenSet_New(red_ops);      /* (NULL: the empty set) */
    if (!frozen_red) { Py_DECREF(frozen); return NULL; }
    Py_INCREF(node_cls); Py_XSETREF(b_node_cls, node_cls);
    Py_INCREF(tensor_cls); Py_XSETREF(b_tensor_cls, tensor_cls);
    Py_XSETREF(b_ew_ops, frozen);
    Py_XSETREF(b_red_ops, frozen_red);
    Py_RETURN_NONE;
}

/* 1 = ok (rows, cols set; *keep = the operand's own 2-tuple when it has one, borrowed),
 * 0 = let Python decide, -1 = error */
static int operand_shape(PyObject* x, Py_ssize_t* rows, Py_ssize_t* cols, PyObject** keep) {
    *keep = NULL;
    if (x == Py_None) { *rows = *cols = 0; *keep = t_none; return 1; }
    if (PyFloat_Check(x) || PyLong_Check(x)) { *rows = *cols = 1; *keep = t_scalar; return 1; }
    PyObject* shp;
    if (PyObject_TypeCheck(x, (PyTypeObject*)b_node_cls)) {
        PyObject* d = PyTuple_GET_SIZE(x) == 3 ? PyTuple_GET_ITEM(x, 0) : NULL;
        if (!d || !PyDict_Check(d)) return 0;
        shp = PyDict_GetItemWithError(d, s_shape);       /* borrowed */
        if (!shp) return PyErr_Occurred() ? -1 : 0;
        Py_INCREF(shp);
    } else if (PyObject_TypeCheck(x, (PyTypeObject*)b_tensor_cls)) {
        shp = PyObject_GetAttr(x, s_shape);
        if (!shp) return -1;
    } else {
        return 0;
    }
    int ok = 0;
    if (PyTuple_Check(shp)) {
        Py_ssize_t n = PyTuple_GET_SIZE(shp);
        if ((n == 1 || n == 2) && PyLong_Check(PyTuple_GET_ITEM(shp, 0)) && (n == 1 || PyLong_Check(PyTuple_GET_ITEM(shp, 1)))) {
            *rows = PyLong_AsSsize_t(PyTuple_GET_ITEM(shp, 0));
            *cols = n == 2 ? PyLong_AsSsize_t(PyTuple_GET_ITEM(shp, 1)) : 1;
            ok = !((*rows == -1 || *cols == -1) && PyErr_Occurred());
            if (!ok) PyErr_Clear();
            /* (the tuple stays alive through its owner, the operand, for as long as we use it) */
            if (ok && n == 2) *keep = shp;
        }
    }
    Py_DECREF(shp);
    return ok;
}

static PyObject* builder_ew_node(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
    if (nargs != 3) { PyErr_SetString(PyExc_TypeError, "ew_node(op, a, b)"); return NULL; }
    if (!b_node_cls) Py_RETURN_NONE;
    int known = PySet_Contains(b_ew_ops, args[0]);
    if (known < 0) return NULL;
    if (!known) Py_RETURN_NONE;
    Py_ssize_t ra, ca, rb, cb;
    PyObject *ka, *kb;
    int ok = operand_shape(args[1], &ra, &ca, &ka);
    if (ok > 0) ok = operand_shape(args[2], &rb, &cb, &kb);
    if (ok < 0) return NULL;
    if (!ok) Py_RETURN_NONE;
    PyObject* shape;
    if (ra == rb && ca == cb && ka) { shape = ka; Py_INCREF(shape); }
    else if (ra >= rb && ca >= cb && ka) { shape = ka; Py_INCREF(shape); }
    else if (rb >= ra && cb >= ca && kb) { shape = kb; Py_INCREF(shape); }
    else shape = Py_BuildValue("(nn)", ra > rb ? ra : rb, ca > cb ? ca : cb);
    if (!shape) return NULL;
    PyObject* d = PyDict_New();
    if (!d || PyDict_SetItem(d, s_op, args[0]) < 0 || PyDict_SetItem(d, s_shape, shape) < 0) {
        Py_XDECREF(d); Py_DECREF(shape); return NULL;
    }
    Py_DECREF(shape);
    PyTypeObject* cls = (PyTypeObject*)b_node_cls;
    PyObject* node = cls->tp_alloc(cls, 3);
    if (!node) { Py_DECREF(d); return NULL; }
    PyTuple_SET_ITEM(node, 0, d);
    Py_INCREF(args[1]); PyTuple_SET_ITEM(node, 1, args[1]);
    Py_INCREF(args[2]); PyTuple_SET_ITEM(node, 2, args[2]);
    return node;
}

/* OpTreeNode.build(op, a, None, axis=axis) for a reduction along axis 0 or 1 of a two-dimensional operand:
 * {"op", "shape", "axis"} with the operand's shape, that axis set to 1.  None: Python builds it. */
static PyObject* builder_red_node(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
    if (nargs != 3) { PyErr_SetString(PyExc_TypeError, "red_node(op, a, axis)"); return NULL; }
    if (!b_node_cls || !b_red_ops || !PyLong_CheckExact(args[2])) Py_RETURN_NONE;
    int known = PySet_Contains(b_red_ops, args[0]);
    if (known < 0) return NULL;
    if (!known) Py_RETURN_NONE;
    const long axis = PyLong_AsLong(args[2]);
    if (axis == -1 && PyErr_Occurred()) { PyErr_Clear(); Py_RETURN_NONE; }
    if (axis != 0 && axis != 1) Py_RETURN_NONE;
    Py_ssize_t ra, ca;
    PyObject* ka;
    if (args[1] == Py_None || PyFloat_Check(args[1]) || PyLong_Check(args[1])) Py_RETURN_NONE;
    int ok = operand_shape(args[1], &ra, &ca, &ka);
    if (ok < 0) return NULL;
    if (!ok) Py_RETURN_NONE;
    PyObject* shape = axis == 0 ? Py_BuildValue("(in)", 1, ca) : Py_BuildValue("(ni)", ra, 1);
    if (!shape) return NULL;
    PyObject* d = PyDict_New();
    if (!d || PyDict_SetItem(d, s_op, args[0]) < 0 || PyDict_SetItem(d, s_shape, shape) < 0 ||
        PyDict_SetItem(d, s_axis, args[2]) < 0) {
        Py_XDECREF(d); Py_DECREF(shape); return NULL;
    }
    Py_DECREF(shape);
    PyTypeObject* cls = (PyTypeObject*)b_node_cls;
    PyObject* node = cls->tp_alloc(cls, 3);
    if (!node) { Py_DECREF(d); return NULL; }
    PyTuple_SET_ITEM(node, 0, d);
    Py_INCREF(args[1]); PyTuple_SET_ITEM(node, 1, args[1]);
    Py_INCREF(Py_None); PyTuple_SET_ITEM(node, 2, Py_None);
    return node;
}

static PyMethodDef module_methods[] = {
    {"configure_builder", builder_configure, METH_VARARGS,
     "configure_builder(node class, tensor class, elementwise op names[, reduction op names])"},
    {"red_node", (PyCFunction)(void (*)(void))builder_red_node, METH_FASTCALL,
     "red_node(op, a, axis) -> node, or None when Python has to build it"},
    {"ew_node", (PyCFunction)(void (*)(void))builder_ew_node, METH_FASTCALL,
     "ew_node(op, a, b) -> node, or None when Python has to build it"},
    {NULL, NULL, 0, NULL}};

static struct PyModuleDef moduledef = {
    PyModuleDef_HEAD_INIT, "_fastpath", "C replay of repeated op-tree statements", -1, module_methods, NULL, NULL, NULL, NULL};

PyMODINIT_FUNC PyInit__fastpath(void) {
    if (PyType_Ready(&RecordsType) < 0 || PyType_Ready(&ReplayerType) < 0) return NULL;
    PyObject* m = PyModule_Create(&moduledef);
    if (!m) return NULL;
    s_geom = PyUnicode_InternFromString("_geom");
    s_op = PyUnicode_InternFromString("op");
    s_axis = PyUnicode_InternFromString("axis");
    s_idx = PyUnicode_InternFromString("idx");
    s_fast = PyUnicode_InternFromString("fast");
    s_bar = PyUnicode_InternFromString("|");
    s_assign = PyUnicode_InternFromString("assign");
    s_shape = PyUnicode_InternFromString("shape");
    t_scalar = Py_BuildValue("(ii)", 1, 1);
    t_none = Py_BuildValue("(ii)", 0, 0);
    if (!s_geom || !s_op || !s_axis || !s_idx || !s_fast || !s_bar || !s_assign || !s_shape || !t_scalar || !t_none)
        return NULL;
    Py_INCREF(&RecordsType);
    Py_INCREF(&ReplayerType);
    if (PyModule_AddObject(m, "Records", (PyObject*)&RecordsType) < 0) return NULL;
    if (PyModule_AddObject(m, "Replayer", (PyObject*)&ReplayerType) < 0) return NULL;
    return m;
}

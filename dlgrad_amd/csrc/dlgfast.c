/*
 * _dlgfast -- a compiled binding for the three calls the hip runtime makes per op.
 *
 * dlgrad binds its C kernels through cffi (dlgrad/runtime/cpu.py:49, :69-78), and per op it
 * makes three foreign calls: allocate the output (cpu.py:82-107), call the kernel
 * (cpu.py:289) and, later, the ffi.gc finaliser that frees it (cpu.py:102).  Through ctypes
 * (or cffi's ABI mode) each of those costs 1-3 microseconds of argument conversion, which on a
 * GPU -- where a kernel for a small tensor runs for about as long -- decides the speed of an
 * eager step.  This module is what cffi's API mode would generate for those three functions,
 * written by hand against the CPython C API: it calls dlg_hip_alloc, dlg_hip_free and
 * dlg_hip_launch of include/dlgrad_hip.h through function pointers taken from the already
 * loaded libdlgrad_hip.so (bind()), so it links against nothing and contains no device logic.
 *
 *   DevPtr(addr, nbytes, base=None)   an address in device memory.  With no base it owns the
 *                                     block: dlg_hip_free(addr) runs when the object dies.
 *                                     ptr + n is a view n floats further on that keeps its
 *                                     base alive (the slices of dlgrad/tensor.py:816-821).
 *   alloc(nbytes) -> DevPtr           dlg_hip_alloc; MemoryError on failure
 *   launch(handle, gx, gy, gz, bx, by, bz, args)          dlg_hip_launch, shared_bytes = 0
 *   launch_out(handle, gx, gy, gz, bx, by, bz, args, offset, nbytes) -> DevPtr
 *                                     allocates nbytes, writes the address into a copy of the
 *                                     argument block at `offset`, launches: the output
 *                                     allocation and the kernel call of one op in one call
 *   bind(alloc, free, launch, last_error)                 the four function addresses
 *
 * Everything else (init, transfers, compile, graphs, events) stays on the ordinary binding
 * in dlgrad_amd/ffi.py; the runtime falls back to that binding for these three calls too when
 * this module has not been built.
 */
#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include "structmember.h"

typedef int (*alloc_fn)(size_t, void **);
typedef int (*free_fn)(void *);
typedef int (*launch_fn)(uint64_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t,
                         const void *, size_t);
typedef const char *(*error_fn)(void);

static alloc_fn p_alloc;
static free_fn p_free;
static launch_fn p_launch;
static error_fn p_error;
static unsigned long long n_launches;          /* launches issued through this module */

typedef struct {
    PyObject_HEAD
    unsigned long long addr;
    unsigned long long nbytes;
    PyObject *base;                             /* NULL: this object owns the block */
    PyObject *weakrefs;
} DevPtr;

static PyTypeObject DevPtr_Type;

static PyObject *devptr_make(unsigned long long addr, unsigned long long nbytes, PyObject *base) {
    DevPtr *p = PyObject_New(DevPtr, &DevPtr_Type);
    if (!p) return NULL;
    p->addr = addr;
    p->nbytes = nbytes;
    Py_XINCREF(base);
    p->base = base;
    p->weakrefs = NULL;
    return (PyObject *)p;
}

static PyObject *devptr_new(PyTypeObject *type, PyObject *args, PyObject *kw) {
    static char *names[] = {"addr", "nbytes", "base", NULL};
    unsigned long long addr, nbytes;
    PyObject *base = Py_None;
    if (!PyArg_ParseTupleAndKeywords(args, kw, "KK|O", names, &addr, &nbytes, &base)) return NULL;
    return devptr_make(addr, nbytes, base == Py_None ? NULL : base);
}

static void devptr_dealloc(DevPtr *p) {
    if (p->weakrefs) PyObject_ClearWeakRefs((PyObject *)p);
    if (p->base) {
        Py_DECREF(p->base);
    } else if (p->addr && p_free) {
        (void)p_free((void *)(uintptr_t)p->addr);       /* a no-op once the library has shut down */
    }
    PyObject_Free(p);
}

static PyObject *devptr_add(PyObject *a, PyObject *b) {
    if (Py_TYPE(a) != &DevPtr_Type || !PyLong_Check(b)) Py_RETURN_NOTIMPLEMENTED;
    DevPtr *p = (DevPtr *)a;
    long long n = PyLong_AsLongLong(b);
    if (n == -1 && PyErr_Occurred()) return NULL;
    if (n < 0 || (unsigned long long)n * 4ull > p->nbytes) {
        PyErr_Format(PyExc_IndexError, "offset %lld elements outside a %llu-byte block", n, p->nbytes);
        return NULL;
    }
    unsigned long long off = 4ull * (unsigned long long)n;
    return devptr_make(p->addr + off, p->nbytes - off, p->base ? p->base : a);
}

static PyObject *devptr_repr(DevPtr *p) {
    char buf[96];
    snprintf(buf, sizeof buf, "DevicePtr(0x%llx, %llu B%s)", p->addr, p->nbytes, p->base ? ", view" : "");
    return PyUnicode_FromString(buf);
}

static PyObject *devptr_get_base(DevPtr *p, void *unused) {
    PyObject *b = p->base ? p->base : Py_None;
    Py_INCREF(b);
    return b;
}

static PyMemberDef devptr_members[] = {
    {"addr", T_ULONGLONG, offsetof(DevPtr, addr), READONLY, "device address"},
    {"nbytes", T_ULONGLONG, offsetof(DevPtr, nbytes), READONLY, "bytes from addr to the end of the block"},
    {NULL}
};
static PyGetSetDef devptr_getset[] = {
    {"base", (getter)devptr_get_base, NULL, "the owning pointer of a view, or None", NULL},
    {NULL}
};
static PyNumberMethods devptr_number = {.nb_add = devptr_add};

static PyTypeObject DevPtr_Type = {
    PyVarObject_HEAD_INIT(NULL, 0)
    .tp_name = "dlgrad_amd._dlgfast.DevPtr",
    .tp_basicsize = sizeof(DevPtr),
    .tp_dealloc = (destructor)devptr_dealloc,
    .tp_repr = (reprfunc)devptr_repr,
    .tp_as_number = &devptr_number,
    .tp_flags = Py_TPFLAGS_DEFAULT,
    .tp_doc = "An address in device memory; owns its block unless it has a base.",
    .tp_weaklistoffset = offsetof(DevPtr, weakrefs),
    .tp_members = devptr_members,
    .tp_getset = devptr_getset,
    .tp_new = devptr_new,
};

static PyObject *raise_last(PyObject *exc, int rc) {
    const char *msg = p_error ? p_error() : "";
    PyErr_Format(exc, "%s [rc=%d]", msg ? msg : "", rc);
    return NULL;
}

static int need_bound(void) {
    if (p_alloc && p_free && p_launch) return 1;
    PyErr_SetString(PyExc_RuntimeError, "_dlgfast.bind() has not been called");
    return 0;
}

static PyObject *fast_bind(PyObject *self, PyObject *args) {
    unsigned long long a, f, l, e;
    if (!PyArg_ParseTuple(args, "KKKK", &a, &f, &l, &e)) return NULL;
    p_alloc = (alloc_fn)(uintptr_t)a;
    p_free = (free_fn)(uintptr_t)f;
    p_launch = (launch_fn)(uintptr_t)l;
    p_error = (error_fn)(uintptr_t)e;
    Py_RETURN_NONE;
}

static PyObject *fast_alloc(PyObject *self, PyObject *arg) {
    if (!need_bound()) return NULL;
    unsigned long long nbytes = PyLong_AsUnsignedLongLong(arg);
    if (nbytes == (unsigned long long)-1 && PyErr_Occurred()) return NULL;
    void *p = NULL;
    int rc = p_alloc((size_t)nbytes, &p);
    if (rc != 0) return raise_last(rc == -9 ? PyExc_RuntimeError : PyExc_MemoryError, rc);   /* -9: refused inside a capture */
    return devptr_make((unsigned long long)(uintptr_t)p, nbytes, NULL);
}

/* handle, gx, gy, gz, bx, by, bz from args[0..6]; 0 on failure with an exception set */
static int parse_geometry(PyObject *const *args, uint64_t *handle, uint32_t g[6]) {
    unsigned long long h = PyLong_AsUnsignedLongLong(args[0]);
    if (h == (unsigned long long)-1 && PyErr_Occurred()) return 0;
    *handle = h;
    for (int i = 0; i < 6; ++i) {
        unsigned long v = PyLong_AsUnsignedLong(args[1 + i]);
        if (v == (unsigned long)-1 && PyErr_Occurred()) return 0;
        if (v > 0xFFFFFFFFul) {
            PyErr_SetString(PyExc_OverflowError, "grid or block extent beyond 32 bits");
            return 0;
        }
        g[i] = (uint32_t)v;
    }
    return 1;
}

static PyObject *fast_launch(PyObject *self, PyObject *const *args, Py_ssize_t nargs) {
    if (!need_bound()) return NULL;
    if (nargs != 8) {
        PyErr_SetString(PyExc_TypeError, "launch(handle, gx, gy, gz, bx, by, bz, args)");
        return NULL;
    }
    uint64_t handle;
    uint32_t g[6];
    if (!parse_geometry(args, &handle, g)) return NULL;
    char *buf;
    Py_ssize_t size;
    if (PyBytes_AsStringAndSize(args[7], &buf, &size) < 0) return NULL;
    int rc = p_launch(handle, g[0], g[1], g[2], g[3], g[4], g[5], 0, buf, (size_t)size);
    if (rc != 0) return raise_last(PyExc_RuntimeError, rc);
    ++n_launches;
    Py_RETURN_NONE;
}

#define MAX_ARGS_BYTES 512

static PyObject *fast_launch_out(PyObject *self, PyObject *const *args, Py_ssize_t nargs) {
    if (!need_bound()) return NULL;
    if (nargs != 10) {
        PyErr_SetString(PyExc_TypeError, "launch_out(handle, gx, gy, gz, bx, by, bz, args, offset, nbytes)");
        return NULL;
    }
    uint64_t handle;
    uint32_t g[6];
    if (!parse_geometry(args, &handle, g)) return NULL;
    char *buf;
    Py_ssize_t size;
    if (PyBytes_AsStringAndSize(args[7], &buf, &size) < 0) return NULL;
    Py_ssize_t offset = PyLong_AsSsize_t(args[8]);
    if (offset == -1 && PyErr_Occurred()) return NULL;
    unsigned long long nbytes = PyLong_AsUnsignedLongLong(args[9]);
    if (nbytes == (unsigned long long)-1 && PyErr_Occurred()) return NULL;
    if (size > MAX_ARGS_BYTES || offset < 0 || offset + 8 > size || (offset & 7)) {
        PyErr_SetString(PyExc_ValueError, "launch_out: argument block too large, or the output slot is not inside it");
        return NULL;
    }
    void *p = NULL;
    int rc = p_alloc((size_t)nbytes, &p);
    if (rc != 0) return raise_last(rc == -9 ? PyExc_RuntimeError : PyExc_MemoryError, rc);   /* -9: refused inside a capture */
    PyObject *out = devptr_make((unsigned long long)(uintptr_t)p, nbytes, NULL);
    if (!out) {
        (void)p_free(p);
        return NULL;
    }
    char local[MAX_ARGS_BYTES] __attribute__((aligned(16)));
    memcpy(local, buf, (size_t)size);
    memcpy(local + offset, &p, sizeof p);
    rc = p_launch(handle, g[0], g[1], g[2], g[3], g[4], g[5], 0, local, (size_t)size);
    if (rc != 0) {
        Py_DECREF(out);                                  /* gives the block back */
        return raise_last(PyExc_RuntimeError, rc);
    }
    ++n_launches;
    return out;
}

static PyObject *fast_launches(PyObject *self, PyObject *unused) {
    return PyLong_FromUnsignedLongLong(n_launches);
}

static PyMethodDef methods[] = {
    {"bind", fast_bind, METH_VARARGS, "bind(alloc, free, launch, last_error): addresses of the four library functions"},
    {"alloc", fast_alloc, METH_O, "alloc(nbytes) -> DevPtr"},
    {"launch", (PyCFunction)(void (*)(void))fast_launch, METH_FASTCALL, "launch(handle, gx, gy, gz, bx, by, bz, args)"},
    {"launch_out", (PyCFunction)(void (*)(void))fast_launch_out, METH_FASTCALL,
     "launch_out(handle, gx, gy, gz, bx, by, bz, args, offset, nbytes) -> DevPtr of the freshly allocated output"},
    {"launches", fast_launches, METH_NOARGS, "launches issued through this module"},
    {NULL, NULL, 0, NULL}
};

static struct PyModuleDef moduledef = {PyModuleDef_HEAD_INIT, "_dlgfast", "compiled binding of alloc / free / launch", -1, methods};

PyMODINIT_FUNC PyInit__dlgfast(void) {
    if (PyType_Ready(&DevPtr_Type) < 0) return NULL;
    PyObject *m = PyModule_Create(&moduledef);
    if (!m) return NULL;
    Py_INCREF(&DevPtr_Type);
    if (PyModule_AddObject(m, "DevPtr", (PyObject *)&DevPtr_Type) < 0) {
        Py_DECREF(&DevPtr_Type);
        Py_DECREF(m);
        return NULL;
    }
    return m;
}

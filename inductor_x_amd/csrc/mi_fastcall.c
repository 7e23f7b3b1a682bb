/* CPython entry to mi_launch_packed with no per-call marshalling objects.
 *
 * The launcher's C ABI (include/mi355_launcher.h) is what any host language binds; from Python the
 * generic binding is ctypes (inductor_x_amd/launcher.py), which builds a dozen argument objects per
 * call.  This module is the same call made through the vectorcall convention: the kernel handle,
 * the launch shape, the raw stream and the packed argument segment go straight to
 * mi_launch_packed, whose address the launcher module hands over once with bind().  It stands
 * where the reference's generated launcher closure calls the Triton binary
 * (reference inductor_x/npu_triton_heuristics.py:239-253).
 */
#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <stdint.h>

typedef int (*launch_packed_fn)(void*, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t,
                                void*, const void*, size_t);
static launch_packed_fn g_launch = NULL;

static PyObject* fast_bind(PyObject* self, PyObject* addr) {
  (void)self;
  void* p = PyLong_AsVoidPtr(addr);
  if (p == NULL && PyErr_Occurred()) return NULL;
  g_launch = (launch_packed_fn)p;
  Py_RETURN_NONE;
}

/* launch(function, gx, gy, gz, bx, by, bz, lds_bytes, stream, segment: bytes) -> int (hipError_t) */
static PyObject* fast_launch(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
  (void)self;
  if (nargs != 10) {
    PyErr_SetString(PyExc_TypeError, "launch() takes 10 positional arguments");
    return NULL;
  }
  if (g_launch == NULL) {
    PyErr_SetString(PyExc_RuntimeError, "launch() before bind()");
    return NULL;
  }
  void* fn = PyLong_AsVoidPtr(args[0]);
  if (fn == NULL && PyErr_Occurred()) return NULL;
  uint32_t dims[7];
  for (int i = 0; i < 7; ++i) {
    unsigned long v = PyLong_AsUnsignedLong(args[1 + i]);
    if (v == (unsigned long)-1 && PyErr_Occurred()) return NULL;
    if (v > 0xffffffffUL) {
      PyErr_SetString(PyExc_OverflowError, "launch dimension does not fit 32 bits");
      return NULL;
    }
    dims[i] = (uint32_t)v;
  }
  void* stream = PyLong_AsVoidPtr(args[8]);
  if (stream == NULL && PyErr_Occurred()) return NULL;
  char* seg = NULL;
  Py_ssize_t len = 0;
  if (PyBytes_AsStringAndSize(args[9], &seg, &len) < 0) return NULL;
  int err = g_launch(fn, dims[0], dims[1], dims[2], dims[3], dims[4], dims[5], dims[6], stream, seg, (size_t)len);
  return PyLong_FromLong(err);
}

static PyMethodDef methods[] = {
    {"bind", (PyCFunction)fast_bind, METH_O, "bind(address of mi_launch_packed)"},
    {"launch", (PyCFunction)(void (*)(void))fast_launch, METH_FASTCALL,
     "launch(function, gx, gy, gz, bx, by, bz, lds_bytes, stream, segment) -> hipError_t"},
    {NULL, NULL, 0, NULL},
};

static struct PyModuleDef module = {PyModuleDef_HEAD_INIT, "_mi_fastcall", NULL, -1, methods, NULL, NULL, NULL, NULL};

PyMODINIT_FUNC PyInit__mi_fastcall(void) { return PyModule_Create(&module); }

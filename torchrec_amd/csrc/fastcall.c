/* Minimal CPython module in front of the C ABI's hot entry point.
 *
 * The serving call of a collection ends in one tra_tbe_forward_lengths(...) with fifteen scalar
 * arguments.  Through ctypes their conversion costs about as much as the checks of the entry
 * point itself; here they are read straight from the argument vector (METH_FASTCALL) and the
 * same C function is called through a pointer that Python hands over once (bind), so this
 * module links against nothing but libpython.  It adds no behaviour: same symbol, same
 * arguments, same return code as declared in include/torchrec_amd.h.
 */
#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <stdint.h>

typedef int (*forward_lengths_fn)(void* tbe, const void* weights, const void* indices, const void* lengths,
                                  int32_t idx_is_i64, const float* per_sample_weights, int32_t batch_size,
                                  int32_t num_keys, int64_t num_indices, int32_t pooling_mode, int32_t out_dtype,
                                  void* out, int64_t out_stride, void* workspace, void* stream);

static forward_lengths_fn g_forward_lengths = NULL;

/* An address or integer argument: a Python int, or None for a null pointer. */
static inline int as_u64(PyObject* o, uint64_t* v) {
  if (o == Py_None) {
    *v = 0;
    return 0;
  }
  *v = PyLong_AsUnsignedLongLongMask(o);
  return (*v == (uint64_t)-1 && PyErr_Occurred()) ? -1 : 0;
}

static PyObject* bind(PyObject* self, PyObject* arg) {
  uint64_t p;
  (void)self;
  if (as_u64(arg, &p) != 0) return NULL;
  g_forward_lengths = (forward_lengths_fn)(uintptr_t)p;
  Py_RETURN_NONE;
}

/* forward_lengths(plan, weights, indices, lengths, idx_is_i64, per_sample_weights, batch_size, num_keys,
 *                 num_indices, pooling_mode, out_dtype, out, out_stride, workspace, stream) -> int */
static PyObject* forward_lengths(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
  uint64_t v[15];
  (void)self;
  if (nargs != 15) {
    PyErr_SetString(PyExc_TypeError, "forward_lengths takes 15 arguments");
    return NULL;
  }
  if (g_forward_lengths == NULL) {
    PyErr_SetString(PyExc_RuntimeError, "forward_lengths: bind() has not been called");
    return NULL;
  }
  for (int i = 0; i < 15; ++i)
    if (as_u64(args[i], &v[i]) != 0) return NULL;
  const int rc = g_forward_lengths((void*)(uintptr_t)v[0], (const void*)(uintptr_t)v[1], (const void*)(uintptr_t)v[2],
                                   (const void*)(uintptr_t)v[3], (int32_t)v[4], (const float*)(uintptr_t)v[5],
                                   (int32_t)v[6], (int32_t)v[7], (int64_t)v[8], (int32_t)v[9], (int32_t)v[10],
                                   (void*)(uintptr_t)v[11], (int64_t)v[12], (void*)(uintptr_t)v[13],
                                   (void*)(uintptr_t)v[14]);
  return PyLong_FromLong(rc);
}

static PyMethodDef methods[] = {
    {"bind", bind, METH_O, "bind(address of tra_tbe_forward_lengths)"},
    {"forward_lengths", (PyCFunction)(void (*)(void))forward_lengths, METH_FASTCALL,
     "tra_tbe_forward_lengths(...) with integer arguments; returns its return code"},
    {NULL, NULL, 0, NULL}};

static struct PyModuleDef module = {PyModuleDef_HEAD_INIT, "_fastcall", NULL, -1, methods, NULL, NULL, NULL, NULL};

PyMODINIT_FUNC PyInit__fastcall(void) { return PyModule_Create(&module); }

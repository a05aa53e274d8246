/* _kvc_fast: CPython entry to the two per-layer plan calls of libkvcache.
 *
 * A forward pass calls the K/V write once per layer; at decode sizes the launch
 * is host-bound, so what the binding adds per call is what a serving loop feels.
 * ctypes converts and type-checks every argument through Python objects (about
 * 0.8 us for nine arguments); these METH_FASTCALL wrappers read the integers
 * straight off the argument vector. They add nothing to the C ABI: each one
 * forwards to the entry point of the same name in include/kvcache.h.
 * Pointers travel as Python ints (tensor.data_ptr(), the plan handle, the raw
 * stream); None stands for NULL.
 */
#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <stdint.h>

#include "kvcache.h"

static int as_ptr(PyObject* o, void** out) {
  if (o == Py_None) {
    *out = NULL;
    return 0;
  }
  *out = PyLong_AsVoidPtr(o);
  return (*out == NULL && PyErr_Occurred()) ? -1 : 0;
}

static int as_i64(PyObject* o, int64_t* out) {
  *out = (int64_t)PyLong_AsLongLong(o);
  return (*out == -1 && PyErr_Occurred()) ? -1 : 0;
}

/* write_plan_append(plan, key, value, key_token_stride, value_token_stride,
 *                   paged_kv_cache, page_stride, num_pages, stream) -> int */
static PyObject* fast_write_plan_append(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
  void *plan, *key, *value, *cache, *stream;
  int64_t ks, vs, page_stride, num_pages;
  (void)self;
  if (nargs != 9) {
    PyErr_SetString(PyExc_TypeError, "write_plan_append takes 9 arguments");
    return NULL;
  }
  if (as_ptr(args[0], &plan) || as_ptr(args[1], &key) || as_ptr(args[2], &value) ||
      as_i64(args[3], &ks) || as_i64(args[4], &vs) || as_ptr(args[5], &cache) ||
      as_i64(args[6], &page_stride) || as_i64(args[7], &num_pages) || as_ptr(args[8], &stream))
    return NULL;
  return PyLong_FromLong(kvc_write_plan_append((const kvc_write_plan*)plan, key, value, ks, vs, cache,
                                               page_stride, num_pages, stream));
}

/* rotary_plan_run(plan, query, key, value, q_token_stride, k_token_stride, v_token_stride,
 *                 query_out, key_out, paged_kv_cache, page_stride, num_pages, stream) -> int */
static PyObject* fast_rotary_plan_run(PyObject* self, PyObject* const* args, Py_ssize_t nargs) {
  void *plan, *q, *k, *v, *qo, *ko, *cache, *stream;
  int64_t qs, ks, vs, page_stride, num_pages;
  (void)self;
  if (nargs != 13) {
    PyErr_SetString(PyExc_TypeError, "rotary_plan_run takes 13 arguments");
    return NULL;
  }
  if (as_ptr(args[0], &plan) || as_ptr(args[1], &q) || as_ptr(args[2], &k) || as_ptr(args[3], &v) ||
      as_i64(args[4], &qs) || as_i64(args[5], &ks) || as_i64(args[6], &vs) || as_ptr(args[7], &qo) ||
      as_ptr(args[8], &ko) || as_ptr(args[9], &cache) || as_i64(args[10], &page_stride) ||
      as_i64(args[11], &num_pages) || as_ptr(args[12], &stream))
    return NULL;
  return PyLong_FromLong(kvc_rotary_plan_run((const kvc_rotary_plan*)plan, q, k, v, qs, ks, vs, qo, ko,
                                             cache, page_stride, num_pages, stream));
}

static PyMethodDef methods[] = {
    {"write_plan_append", (PyCFunction)(void (*)(void))fast_write_plan_append, METH_FASTCALL,
     "kvc_write_plan_append with integer arguments; returns the kvc_status."},
    {"rotary_plan_run", (PyCFunction)(void (*)(void))fast_rotary_plan_run, METH_FASTCALL,
     "kvc_rotary_plan_run with integer arguments; returns the kvc_status."},
    {NULL, NULL, 0, NULL}};

static struct PyModuleDef module = {PyModuleDef_HEAD_INIT, "_kvc_fast",
                                    "Low-overhead calls into libkvcache's per-layer plan entry points.",
                                    -1, methods, NULL, NULL, NULL, NULL};

PyMODINIT_FUNC PyInit__kvc_fast(void) {
  PyObject* m = PyModule_Create(&module);
  if (m && PyModule_AddIntConstant(m, "abi_version", KVC_ABI_VERSION) < 0) {
    Py_DECREF(m);
    return NULL;
  }
  return m;
}

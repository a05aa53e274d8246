/* _kvc_fast: CPython entry to the two per-layer plan calls of libkvcache.
 *
 * A forward pass calls the K/V write once per layer; at decode sizes the launch
 * is host-bound, so what the binding adds per call is what a serving loop feels.
 * ctypes converts and type-checks every argument through Python objects (about
 * 0.8 us for nine arguments) and the layout checks of three or five tensors cost
 * another microsecond of attribute reads in Python. Here the tensors are
 * unpacked in C++ (pointer, strides, sizes, dtype and device are plain member
 * reads) and the integers are read straight off the argument vector.
 *
 * The wrappers add nothing to the C ABI: each forwards to the entry point of
 * the same name in include/kvcache.h. They only accept the layouts the common
 * case produces and return NOT_FAST (1) for anything else, so that the Python
 * caller can run its own checks, which name what is wrong or handle the rare
 * layout; a negative return is the kvc_status of the library call.
 */
#include <torch/csrc/autograd/python_variable.h>

#include <ATen/core/Tensor.h>

#include <cstdint>

#include "kvcache.h"

namespace {

constexpr long NOT_FAST = 1;

bool as_ptr(PyObject* o, void** out) {
  if (o == Py_None) {
    *out = nullptr;
    return true;
  }
  *out = PyLong_AsVoidPtr(o);
  return !(*out == nullptr && PyErr_Occurred());
}

bool as_i64(PyObject* o, int64_t* out) {
  *out = (int64_t)PyLong_AsLongLong(o);
  return !(*out == -1 && PyErr_Occurred());
}

// Token-major rows, dense inside a token: [n, width] or [n, heads, dim] with
// heads * dim == width. Returns the token stride in elements, or -1.
int64_t row_stride(const at::Tensor& t, int64_t n, int64_t width, int dtype, int device) {
  if ((int)t.scalar_type() != dtype || !t.is_cuda() || t.device().index() != device) return -1;
  const auto sizes = t.sizes();
  const auto strides = t.strides();
  if (sizes.size() == 2) {
    if (sizes[0] != n || sizes[1] != width || strides[1] != 1) return -1;
  } else if (sizes.size() == 3) {
    if (sizes[0] != n || sizes[1] * sizes[2] != width || strides[2] != 1 ||
        (sizes[1] > 1 && strides[1] != sizes[2]))
      return -1;
  } else {
    return -1;
  }
  if (n > 1 && strides[0] < width) return -1;
  return n > 1 ? strides[0] : width;
}

// One layer of the pool, [num_pages, 2, page_size, H, D] with contiguous pages.
// Returns the page stride in elements, or -1.
int64_t page_stride(const at::Tensor& c, int64_t page_size, int64_t heads, int64_t dim, int dtype,
                    int device, int64_t* num_pages) {
  if ((int)c.scalar_type() != dtype || !c.is_cuda() || c.device().index() != device) return -1;
  const auto sizes = c.sizes();
  const auto strides = c.strides();
  if (sizes.size() != 5 || sizes[1] != 2 || sizes[2] != page_size || sizes[3] != heads || sizes[4] != dim)
    return -1;
  const int64_t row = heads * dim;
  if (strides[4] != 1 || strides[3] != dim || strides[2] != row || strides[1] != page_size * row) return -1;
  *num_pages = sizes[0];
  if (sizes[0] < 1) return -1;
  if (sizes[0] > 1 && strides[0] < 2 * page_size * row) return -1;  // overlapping pages
  return sizes[0] > 1 ? strides[0] : 2 * page_size * row;
}

const at::Tensor* tensor_of(PyObject* o) {
  return THPVariable_Check(o) ? &THPVariable_Unpack(o) : nullptr;
}

/* write_plan_append(plan, nnz, heads, dim, page_size, dtype, device, key, value, cache, stream) */
PyObject* fast_write_plan_append(PyObject*, PyObject* const* args, Py_ssize_t nargs) {
  void *plan, *stream;
  int64_t nnz, heads, dim, page_size, dtype, device;
  if (nargs != 11) {
    PyErr_SetString(PyExc_TypeError, "write_plan_append takes 11 arguments");
    return nullptr;
  }
  if (!as_ptr(args[0], &plan) || !as_i64(args[1], &nnz) || !as_i64(args[2], &heads) ||
      !as_i64(args[3], &dim) || !as_i64(args[4], &page_size) || !as_i64(args[5], &dtype) ||
      !as_i64(args[6], &device) || !as_ptr(args[10], &stream))
    return nullptr;
  const at::Tensor* k = tensor_of(args[7]);
  const at::Tensor* v = tensor_of(args[8]);
  const at::Tensor* c = tensor_of(args[9]);
  if (!k || !v || !c) return PyLong_FromLong(NOT_FAST);
  const int64_t row = heads * dim;
  const int64_t ks = row_stride(*k, nnz, row, (int)dtype, (int)device);
  const int64_t vs = row_stride(*v, nnz, row, (int)dtype, (int)device);
  int64_t num_pages = 0;
  const int64_t ps = page_stride(*c, page_size, heads, dim, (int)dtype, (int)device, &num_pages);
  if (ks < 0 || vs < 0 || ps < 0) return PyLong_FromLong(NOT_FAST);
  return PyLong_FromLong(kvc_write_plan_append((const kvc_write_plan*)plan, k->data_ptr(), v->data_ptr(),
                                               ks, vs, c->data_ptr(), ps, num_pages, stream));
}

/* rotary_plan_run(plan, nnz, q_heads, heads, dim, page_size, dtype, device,
 *                 query, key, value, query_out, key_out | None, cache, stream) */
PyObject* fast_rotary_plan_run(PyObject*, PyObject* const* args, Py_ssize_t nargs) {
  void *plan, *stream;
  int64_t nnz, q_heads, heads, dim, page_size, dtype, device;
  if (nargs != 15) {
    PyErr_SetString(PyExc_TypeError, "rotary_plan_run takes 15 arguments");
    return nullptr;
  }
  if (!as_ptr(args[0], &plan) || !as_i64(args[1], &nnz) || !as_i64(args[2], &q_heads) ||
      !as_i64(args[3], &heads) || !as_i64(args[4], &dim) || !as_i64(args[5], &page_size) ||
      !as_i64(args[6], &dtype) || !as_i64(args[7], &device) || !as_ptr(args[14], &stream))
    return nullptr;
  const at::Tensor* q = tensor_of(args[8]);
  const at::Tensor* k = tensor_of(args[9]);
  const at::Tensor* v = tensor_of(args[10]);
  const at::Tensor* qo = tensor_of(args[11]);
  const at::Tensor* ko = args[12] == Py_None ? nullptr : tensor_of(args[12]);
  const at::Tensor* c = tensor_of(args[13]);
  if (!q || !k || !v || !qo || !c || (args[12] != Py_None && !ko)) return PyLong_FromLong(NOT_FAST);
  const int64_t q_row = q_heads * dim, kv_row = heads * dim;
  const int dt = (int)dtype, dev = (int)device;
  const int64_t qs = row_stride(*q, nnz, q_row, dt, dev);
  const int64_t ks = row_stride(*k, nnz, kv_row, dt, dev);
  const int64_t vs = row_stride(*v, nnz, kv_row, dt, dev);
  // outputs are written with dense rows
  if (qs < 0 || ks < 0 || vs < 0 || row_stride(*qo, nnz, q_row, dt, dev) != q_row ||
      (ko && row_stride(*ko, nnz, kv_row, dt, dev) != kv_row))
    return PyLong_FromLong(NOT_FAST);
  int64_t num_pages = 0;
  const int64_t ps = page_stride(*c, page_size, heads, dim, dt, dev, &num_pages);
  if (ps < 0) return PyLong_FromLong(NOT_FAST);
  return PyLong_FromLong(kvc_rotary_plan_run((const kvc_rotary_plan*)plan, q->data_ptr(), k->data_ptr(),
                                             v->data_ptr(), qs, ks, vs, qo->data_ptr(),
                                             ko ? ko->data_ptr() : nullptr, c->data_ptr(), ps, num_pages,
                                             stream));
}

/* scalar_type_code(tensor) -> the integer the two calls above compare dtypes with */
PyObject* scalar_type_code(PyObject*, PyObject* o) {
  const at::Tensor* t = tensor_of(o);
  if (!t) {
    PyErr_SetString(PyExc_TypeError, "scalar_type_code takes a tensor");
    return nullptr;
  }
  return PyLong_FromLong((long)t->scalar_type());
}

PyMethodDef methods[] = {
    {"write_plan_append", (PyCFunction)(void (*)(void))fast_write_plan_append, METH_FASTCALL,
     "kvc_write_plan_append on (key, value, cache) tensors; 0, 1 = not the fast layout, or a negative kvc_status."},
    {"rotary_plan_run", (PyCFunction)(void (*)(void))fast_rotary_plan_run, METH_FASTCALL,
     "kvc_rotary_plan_run on tensors; 0, 1 = not the fast layout, or a negative kvc_status."},
    {"scalar_type_code", (PyCFunction)scalar_type_code, METH_O, "Integer code of a tensor's dtype."},
    {nullptr, nullptr, 0, nullptr}};

PyModuleDef module = {PyModuleDef_HEAD_INIT, "_kvc_fast",
                      "Low-overhead calls into libkvcache's per-layer plan entry points.", -1, methods,
                      nullptr, nullptr, nullptr, nullptr};

}  // namespace

PyMODINIT_FUNC PyInit__kvc_fast(void) {
  PyObject* m = PyModule_Create(&module);
  if (m && (PyModule_AddIntConstant(m, "abi_version", KVC_ABI_VERSION) < 0 ||
            PyModule_AddIntConstant(m, "NOT_FAST", NOT_FAST) < 0)) {
    Py_DECREF(m);
    return nullptr;
  }
  return m;
}

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
 * The same holds for the drop-in per-layer calls (`append_paged`,
 * `reshape_and_cache`, `rotary_pos_emb`, `rotary_append_paged`): up to twelve
 * tensors checked here instead of in Python.
 *
 * The wrappers add nothing to the C ABI: each forwards to the entry point of
 * the same name in include/kvcache.h. They only accept the layouts the common
 * case produces and return NOT_FAST (1) for anything else, so that the Python
 * caller can run its own checks, which name what is wrong or handle the rare
 * layout; a negative return is the kvc_status of the library call.
 */
#include <torch/csrc/autograd/python_variable.h>

#include <ATen/core/Tensor.h>

#include <hip/hip_runtime_api.h>

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

// rows as above, but the tensor may hold more rows than are written
int64_t row_stride_at_least(const at::Tensor& t, int64_t n, int64_t width, int dtype, int device) {
  if (t.dim() < 1 || t.sizes()[0] < n) return -1;
  if (t.sizes()[0] == n) return row_stride(t, n, width, dtype, device);
  const int64_t st = row_stride(t, t.sizes()[0], width, dtype, device);
  return st < 0 ? -1 : (n > 1 ? st : width);
}

// dense 1-D index array of the given integer type on the device
bool index_array(const at::Tensor& t, int device, at::ScalarType type) {
  if (!t.is_cuda() || t.device().index() != device || t.dim() != 1 || t.scalar_type() != type) return false;
  return t.sizes()[0] <= 1 || t.strides()[0] == 1;
}

// the launch goes to the current device: anything else is left to the caller's slow path
bool on_current_device(int device) {
  int cur = -1;
  return hipGetDevice(&cur) == hipSuccess && cur == device;
}

/* append_paged(key, value, batch_indices, positions, cache, kv_indices, kv_indptr,
 *              kv_last_page_len, device, stream): kvc_append_paged_kv_cache on tensors */
PyObject* fast_append_paged(PyObject*, PyObject* const* args, Py_ssize_t nargs) {
  if (nargs != 10) {
    PyErr_SetString(PyExc_TypeError, "append_paged takes 10 arguments");
    return nullptr;
  }
  int64_t device;
  void* stream;
  if (!as_i64(args[8], &device) || !as_ptr(args[9], &stream)) return nullptr;
  const at::Tensor* t[8];
  for (int i = 0; i < 8; ++i)
    if (!(t[i] = tensor_of(args[i]))) return PyLong_FromLong(NOT_FAST);
  const at::Tensor &k = *t[0], &v = *t[1], &bi = *t[2], &pos = *t[3], &c = *t[4], &ind = *t[5],
                   &ptr = *t[6], &last = *t[7];
  const int dev = (int)device;
  if (!on_current_device(dev)) return PyLong_FromLong(NOT_FAST);
  if (!index_array(bi, dev, at::kInt) || !index_array(pos, dev, at::kInt) || !index_array(ind, dev, at::kInt) ||
      !index_array(ptr, dev, at::kInt) || !index_array(last, dev, at::kInt))
    return PyLong_FromLong(NOT_FAST);
  const int64_t nnz = bi.sizes()[0];
  if (pos.sizes()[0] != nnz || ptr.sizes()[0] < 1 || c.dim() != 5) return PyLong_FromLong(NOT_FAST);
  const auto cs = c.sizes();
  const int64_t page_size = cs[2], heads = cs[3], dim = cs[4], row = heads * dim;
  const int dtype = (int)c.scalar_type();
  int64_t num_pages = 0;
  const int64_t ps = page_stride(c, page_size, heads, dim, dtype, dev, &num_pages);
  const int64_t ks = row_stride_at_least(k, nnz, row, dtype, dev);
  const int64_t vs = row_stride_at_least(v, nnz, row, dtype, dev);
  if (ps < 0 || ks < 0 || vs < 0 || nnz == 0 || row == 0) return PyLong_FromLong(NOT_FAST);
  return PyLong_FromLong(kvc_append_paged_kv_cache(
      k.data_ptr(), v.data_ptr(), (const int32_t*)bi.data_ptr(), (const int32_t*)pos.data_ptr(),
      c.data_ptr(), (const int32_t*)ind.data_ptr(), (const int32_t*)ptr.data_ptr(),
      (const int32_t*)last.data_ptr(), nnz, ptr.sizes()[0] - 1, ind.sizes()[0], heads, dim, page_size,
      ks, vs, ps, num_pages, (int)c.element_size(), stream));
}

/* reshape_and_cache(key, value, cache, slot_mapping, device, stream): kvc_reshape_and_cache
 * on one layer of the interleaved pool, [num_blocks, 2, block_size, H, D] */
PyObject* fast_reshape_and_cache(PyObject*, PyObject* const* args, Py_ssize_t nargs) {
  if (nargs != 6) {
    PyErr_SetString(PyExc_TypeError, "reshape_and_cache takes 6 arguments");
    return nullptr;
  }
  int64_t device;
  void* stream;
  if (!as_i64(args[4], &device) || !as_ptr(args[5], &stream)) return nullptr;
  const at::Tensor* k = tensor_of(args[0]);
  const at::Tensor* v = tensor_of(args[1]);
  const at::Tensor* c = tensor_of(args[2]);
  const at::Tensor* sl = tensor_of(args[3]);
  if (!k || !v || !c || !sl) return PyLong_FromLong(NOT_FAST);
  const int dev = (int)device;
  if (!on_current_device(dev) || c->dim() != 5) return PyLong_FromLong(NOT_FAST);
  const int slot_bytes = sl->scalar_type() == at::kLong ? 8 : 4;
  if (!index_array(*sl, dev, slot_bytes == 8 ? at::kLong : at::kInt)) return PyLong_FromLong(NOT_FAST);
  const int64_t n = sl->sizes()[0];
  const auto cs = c->sizes();
  const int64_t bs = cs[2], heads = cs[3], dim = cs[4], row = heads * dim;
  const int dtype = (int)c->scalar_type();
  int64_t num_blocks = 0;
  const int64_t stride = page_stride(*c, bs, heads, dim, dtype, dev, &num_blocks);
  const int64_t ks = row_stride(*k, n, row, dtype, dev);
  const int64_t vs = row_stride(*v, n, row, dtype, dev);
  if (stride < 0 || ks < 0 || vs < 0 || n == 0 || row == 0) return PyLong_FromLong(NOT_FAST);
  char* kc = (char*)c->data_ptr();
  return PyLong_FromLong(kvc_reshape_and_cache(k->data_ptr(), v->data_ptr(), kc,
                                               kc + bs * row * (int64_t)c->element_size(), sl->data_ptr(),
                                               slot_bytes, n, row, ks, vs, bs, stride, row, num_blocks,
                                               (int)c->element_size(), stream));
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

// [n, width] or [n, heads, dim] rows, dense inside a token: width and token stride, or false
bool token_rows(const at::Tensor& t, int64_t n, at::ScalarType type, int device, int64_t* width,
                int64_t* stride) {
  if (t.scalar_type() != type || (t.dim() != 2 && t.dim() != 3) || t.sizes()[0] != n) return false;
  *width = t.dim() == 2 ? t.sizes()[1] : t.sizes()[1] * t.sizes()[2];
  *stride = row_stride(t, n, *width, (int)type, device);
  return *stride >= 0;
}

int kvc_dtype_of(at::ScalarType t) {
  return t == at::kBFloat16 ? KVC_DTYPE_BF16 : t == at::kHalf ? KVC_DTYPE_F16 : t == at::kFloat ? KVC_DTYPE_F32 : -1;
}

// cos/sin table [max_position, 2 * rotary_dim], contiguous
bool cos_sin_table(const at::Tensor& cs, at::ScalarType type, int device) {
  return cs.is_cuda() && cs.device().index() == device && cs.scalar_type() == type && cs.dim() == 2 &&
         cs.sizes()[1] % 2 == 0 && cs.strides()[1] == 1 && (cs.sizes()[0] <= 1 || cs.strides()[0] == cs.sizes()[1]);
}

/* rotary_pos_emb(query, key, positions, cos_sin_cache, head_dim, query_out, key_out, device, stream):
 * kvc_rotary_pos_emb on tensors; the outputs are dense [n, width] buffers of the caller */
PyObject* fast_rotary_pos_emb(PyObject*, PyObject* const* args, Py_ssize_t nargs) {
  if (nargs != 9) {
    PyErr_SetString(PyExc_TypeError, "rotary_pos_emb takes 9 arguments");
    return nullptr;
  }
  int64_t head_dim, device;
  void* stream;
  if (!as_i64(args[4], &head_dim) || !as_i64(args[7], &device) || !as_ptr(args[8], &stream)) return nullptr;
  const at::Tensor* q = tensor_of(args[0]);
  const at::Tensor* k = tensor_of(args[1]);
  const at::Tensor* pos = tensor_of(args[2]);
  const at::Tensor* cs = tensor_of(args[3]);
  const at::Tensor* qo = tensor_of(args[5]);
  const at::Tensor* ko = tensor_of(args[6]);
  if (!q || !k || !pos || !cs || !qo || !ko || head_dim <= 0) return PyLong_FromLong(NOT_FAST);
  const int dev = (int)device;
  const at::ScalarType type = q->scalar_type();
  const int kd = kvc_dtype_of(type);
  if (kd < 0 || !on_current_device(dev) || !cos_sin_table(*cs, type, dev)) return PyLong_FromLong(NOT_FAST);
  const bool pos64 = pos->scalar_type() == at::kLong;
  if (!index_array(*pos, dev, pos64 ? at::kLong : at::kInt)) return PyLong_FromLong(NOT_FAST);
  const int64_t n = pos->sizes()[0];
  int64_t qw, qs, kw, ks, ow, os;
  if (n == 0 || !token_rows(*q, n, type, dev, &qw, &qs) || !token_rows(*k, n, type, dev, &kw, &ks) ||
      qw % head_dim || kw % head_dim)
    return PyLong_FromLong(NOT_FAST);
  if (!token_rows(*qo, n, type, dev, &ow, &os) || ow != qw || os != qw) return PyLong_FromLong(NOT_FAST);
  if (!token_rows(*ko, n, type, dev, &ow, &os) || ow != kw || os != kw) return PyLong_FromLong(NOT_FAST);
  return PyLong_FromLong(kvc_rotary_pos_emb(q->data_ptr(), k->data_ptr(), pos->data_ptr(), pos64 ? 8 : 4,
                                            cs->data_ptr(), cs->sizes()[0], n, qw / head_dim, kw / head_dim,
                                            head_dim, cs->sizes()[1] / 2, qs, ks, qo->data_ptr(),
                                            ko->data_ptr(), qw, kw, kd, stream));
}

/* rotary_append_paged(query, key, value, batch_indices, positions, cos_sin_cache, head_dim, cache,
 *                     kv_indices, kv_indptr, kv_last_page_len, query_out, key_out | None, device, stream):
 * kvc_rotary_pos_emb_and_append_paged on tensors */
PyObject* fast_rotary_append_paged(PyObject*, PyObject* const* args, Py_ssize_t nargs) {
  if (nargs != 15) {
    PyErr_SetString(PyExc_TypeError, "rotary_append_paged takes 15 arguments");
    return nullptr;
  }
  int64_t head_dim, device;
  void* stream;
  if (!as_i64(args[6], &head_dim) || !as_i64(args[13], &device) || !as_ptr(args[14], &stream)) return nullptr;
  const at::Tensor* q = tensor_of(args[0]);
  const at::Tensor* k = tensor_of(args[1]);
  const at::Tensor* v = tensor_of(args[2]);
  const at::Tensor* bi = tensor_of(args[3]);
  const at::Tensor* pos = tensor_of(args[4]);
  const at::Tensor* cs = tensor_of(args[5]);
  const at::Tensor* c = tensor_of(args[7]);
  const at::Tensor* ind = tensor_of(args[8]);
  const at::Tensor* ptr = tensor_of(args[9]);
  const at::Tensor* last = tensor_of(args[10]);
  const at::Tensor* qo = tensor_of(args[11]);
  const at::Tensor* ko = args[12] == Py_None ? nullptr : tensor_of(args[12]);
  if (!q || !k || !v || !bi || !pos || !cs || !c || !ind || !ptr || !last || !qo ||
      (args[12] != Py_None && !ko) || head_dim <= 0)
    return PyLong_FromLong(NOT_FAST);
  const int dev = (int)device;
  const at::ScalarType type = q->scalar_type();
  const int kd = kvc_dtype_of(type);
  if (kd < 0 || !on_current_device(dev) || !cos_sin_table(*cs, type, dev)) return PyLong_FromLong(NOT_FAST);
  if (!index_array(*bi, dev, at::kInt) || !index_array(*pos, dev, at::kInt) || !index_array(*ind, dev, at::kInt) ||
      !index_array(*ptr, dev, at::kInt) || !index_array(*last, dev, at::kInt) || ptr->sizes()[0] < 1)
    return PyLong_FromLong(NOT_FAST);
  const int64_t n = pos->sizes()[0];
  if (n == 0 || bi->sizes()[0] != n || c->dim() != 5 || c->sizes()[4] != head_dim) return PyLong_FromLong(NOT_FAST);
  const int64_t page_size = c->sizes()[2], heads = c->sizes()[3], row = heads * head_dim;
  int64_t num_pages = 0;
  const int64_t ps = page_stride(*c, page_size, heads, head_dim, (int)type, dev, &num_pages);
  int64_t qw, qs, kw, ks, vw, vs, ow, os;
  if (ps < 0 || !token_rows(*q, n, type, dev, &qw, &qs) || !token_rows(*k, n, type, dev, &kw, &ks) ||
      !token_rows(*v, n, type, dev, &vw, &vs) || qw % head_dim || kw != row || vw != row)
    return PyLong_FromLong(NOT_FAST);
  if (!token_rows(*qo, n, type, dev, &ow, &os) || ow != qw || os != qw) return PyLong_FromLong(NOT_FAST);
  if (ko && (!token_rows(*ko, n, type, dev, &ow, &os) || ow != kw || os != kw)) return PyLong_FromLong(NOT_FAST);
  return PyLong_FromLong(kvc_rotary_pos_emb_and_append_paged(
      q->data_ptr(), k->data_ptr(), v->data_ptr(), (const int32_t*)bi->data_ptr(),
      (const int32_t*)pos->data_ptr(), cs->data_ptr(), cs->sizes()[0], n, qw / head_dim, heads, head_dim,
      cs->sizes()[1] / 2, qs, ks, vs, qo->data_ptr(), ko ? ko->data_ptr() : nullptr, qw, row, c->data_ptr(),
      (const int32_t*)ind->data_ptr(), (const int32_t*)ptr->data_ptr(), ptr->sizes()[0] - 1,
      ind->sizes()[0], page_size, ps, num_pages, kd, stream));
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
    {"append_paged", (PyCFunction)(void (*)(void))fast_append_paged, METH_FASTCALL,
     "kvc_append_paged_kv_cache on tensors; 0, 1 = not the fast layout, or a negative kvc_status."},
    {"reshape_and_cache", (PyCFunction)(void (*)(void))fast_reshape_and_cache, METH_FASTCALL,
     "kvc_reshape_and_cache on tensors; 0, 1 = not the fast layout, or a negative kvc_status."},
    {"rotary_pos_emb", (PyCFunction)(void (*)(void))fast_rotary_pos_emb, METH_FASTCALL,
     "kvc_rotary_pos_emb on tensors; 0, 1 = not the fast layout, or a negative kvc_status."},
    {"rotary_append_paged", (PyCFunction)(void (*)(void))fast_rotary_append_paged, METH_FASTCALL,
     "kvc_rotary_pos_emb_and_append_paged on tensors; 0, 1 = not the fast layout, or a negative kvc_status."},
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

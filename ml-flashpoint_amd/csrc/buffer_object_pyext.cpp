// CPython extension module `buffer_object_ext`: the Python face of the C-ABI buffer object.
//
// It exposes the same class the reference's pybind11 module does
// (src/ml_flashpoint/checkpoint_object_manager/buffer_object/bindings.cpp:27-100):
//   BufferObject(object_id, capacity, overwrite=False)   create + map read-write
//   BufferObject(object_id)                              map an existing file read-only
//   close(truncate_size=None), resize(new_capacity), get_id(), get_capacity(), get_data_ptr(),
//   properties `closed`, `is_readonly`, and the buffer protocol (1-D uint8 view of the mapping).
// Written against the plain CPython C API; all file/mmap work is delegated to include/mlf_buffer.h and
// runs with the GIL released.  Failures surface as RuntimeError carrying the C-ABI's message.
#define PY_SSIZE_T_CLEAN
#include <Python.h>

#include "mlf_buffer.h"

namespace {

struct PyBufferObject {
  PyObject_HEAD
  mlf_buffer* handle;
};

PyObject* raise_last(void) {
  PyErr_SetString(PyExc_RuntimeError, mlf_buffer_last_error());
  return nullptr;
}

int bo_init(PyObject* self_, PyObject* args, PyObject* kwargs) {
  auto* self = reinterpret_cast<PyBufferObject*>(self_);
  static const char* kwlist[] = {"object_id", "capacity", "overwrite", nullptr};
  const char* object_id = nullptr;
  PyObject* capacity = Py_None;
  int overwrite = 0;
  if (!PyArg_ParseTupleAndKeywords(args, kwargs, "s|Op", const_cast<char**>(kwlist), &object_id, &capacity,
                                   &overwrite))
    return -1;
  if (self->handle) {  // __init__ called twice: drop the previous mapping
    mlf_buffer_destroy(self->handle);
    self->handle = nullptr;
  }
  mlf_buffer* h = nullptr;
  int rc;
  if (capacity == Py_None) {
    Py_BEGIN_ALLOW_THREADS
    rc = mlf_buffer_open_readonly(object_id, &h);
    Py_END_ALLOW_THREADS
  } else {
    size_t cap = PyLong_AsSize_t(capacity);
    if (cap == (size_t)-1 && PyErr_Occurred()) return -1;
    Py_BEGIN_ALLOW_THREADS
    rc = mlf_buffer_create(object_id, cap, overwrite, &h);
    Py_END_ALLOW_THREADS
  }
  if (rc != MLF_OK) {
    raise_last();
    return -1;
  }
  self->handle = h;
  return 0;
}

void bo_dealloc(PyObject* self_) {
  auto* self = reinterpret_cast<PyBufferObject*>(self_);
  if (self->handle) {
    mlf_buffer* h = self->handle;
    self->handle = nullptr;
    Py_BEGIN_ALLOW_THREADS
    mlf_buffer_destroy(h);
    Py_END_ALLOW_THREADS
  }
  Py_TYPE(self_)->tp_free(self_);
}

PyObject* bo_close(PyObject* self_, PyObject* args, PyObject* kwargs) {
  auto* self = reinterpret_cast<PyBufferObject*>(self_);
  static const char* kwlist[] = {"truncate_size", nullptr};
  PyObject* truncate = Py_None;
  if (!PyArg_ParseTupleAndKeywords(args, kwargs, "|O", const_cast<char**>(kwlist), &truncate)) return nullptr;
  int has_truncate = truncate != Py_None;
  size_t size = 0;
  if (has_truncate) {
    size = PyLong_AsSize_t(truncate);
    if (size == (size_t)-1 && PyErr_Occurred()) return nullptr;
  }
  if (self->handle) {
    // close never raises: a failed cleanup step is reported on stderr only, the object ends up closed.
    int rc;
    Py_BEGIN_ALLOW_THREADS
    rc = mlf_buffer_close(self->handle, has_truncate, size);
    Py_END_ALLOW_THREADS
    if (rc != MLF_OK)
      PySys_WriteStderr("BufferObject.close('%s'): %s\n", mlf_buffer_id(self->handle), mlf_buffer_last_error());
  }
  Py_RETURN_NONE;
}

PyObject* bo_resize(PyObject* self_, PyObject* args, PyObject* kwargs) {
  auto* self = reinterpret_cast<PyBufferObject*>(self_);
  static const char* kwlist[] = {"new_capacity", nullptr};
  PyObject* cap_obj = nullptr;
  if (!PyArg_ParseTupleAndKeywords(args, kwargs, "O", const_cast<char**>(kwlist), &cap_obj)) return nullptr;
  size_t cap = PyLong_AsSize_t(cap_obj);
  if (cap == (size_t)-1 && PyErr_Occurred()) return nullptr;
  int rc;
  Py_BEGIN_ALLOW_THREADS
  rc = mlf_buffer_resize(self->handle, cap);
  Py_END_ALLOW_THREADS
  if (rc != MLF_OK) return raise_last();
  Py_RETURN_NONE;
}

PyObject* bo_reserve(PyObject* self_, PyObject* args, PyObject* kwargs) {
  auto* self = reinterpret_cast<PyBufferObject*>(self_);
  static const char* kwlist[] = {"offset", "nbytes", nullptr};
  PyObject *off_obj = nullptr, *len_obj = nullptr;
  if (!PyArg_ParseTupleAndKeywords(args, kwargs, "OO", const_cast<char**>(kwlist), &off_obj, &len_obj)) return nullptr;
  size_t off = PyLong_AsSize_t(off_obj);
  if (off == (size_t)-1 && PyErr_Occurred()) return nullptr;
  size_t len = PyLong_AsSize_t(len_obj);
  if (len == (size_t)-1 && PyErr_Occurred()) return nullptr;
  int rc;
  Py_BEGIN_ALLOW_THREADS
  rc = mlf_buffer_reserve(self->handle, off, len);
  Py_END_ALLOW_THREADS
  if (rc != MLF_OK) return raise_last();
  Py_RETURN_NONE;
}

PyObject* bo_prefault(PyObject* self_, PyObject* args, PyObject* kwargs) {
  auto* self = reinterpret_cast<PyBufferObject*>(self_);
  static const char* kwlist[] = {"offset", "nbytes", "threads", nullptr};
  PyObject *off_obj = nullptr, *len_obj = nullptr;
  int threads = 4;
  if (!PyArg_ParseTupleAndKeywords(args, kwargs, "OO|i", const_cast<char**>(kwlist), &off_obj, &len_obj, &threads)) return nullptr;
  size_t off = PyLong_AsSize_t(off_obj);
  if (off == (size_t)-1 && PyErr_Occurred()) return nullptr;
  size_t len = PyLong_AsSize_t(len_obj);
  if (len == (size_t)-1 && PyErr_Occurred()) return nullptr;
  int rc;
  Py_BEGIN_ALLOW_THREADS
  rc = mlf_buffer_prefault(self->handle, off, len, threads);
  Py_END_ALLOW_THREADS
  if (rc != MLF_OK) return raise_last();
  Py_RETURN_NONE;
}

PyObject* bo_get_id(PyObject* self_, PyObject*) {
  auto* self = reinterpret_cast<PyBufferObject*>(self_);
  return PyUnicode_FromString(mlf_buffer_id(self->handle));
}

PyObject* bo_get_capacity(PyObject* self_, PyObject*) {
  auto* self = reinterpret_cast<PyBufferObject*>(self_);
  return PyLong_FromSize_t(mlf_buffer_capacity(self->handle));
}

PyObject* bo_get_data_ptr(PyObject* self_, PyObject*) {
  auto* self = reinterpret_cast<PyBufferObject*>(self_);
  if (mlf_buffer_is_closed(self->handle)) {
    PyErr_SetString(PyExc_RuntimeError, "Buffer is closed: cannot access data pointer.");
    return nullptr;
  }
  return PyLong_FromVoidPtr(mlf_buffer_data_ptr(self->handle));
}

PyObject* bo_fileno(PyObject* self_, PyObject*) {
  auto* self = reinterpret_cast<PyBufferObject*>(self_);
  if (mlf_buffer_is_closed(self->handle)) {
    PyErr_SetString(PyExc_RuntimeError, "Buffer is closed: no file descriptor.");
    return nullptr;
  }
  return PyLong_FromLong(mlf_buffer_fd(self->handle));
}

PyObject* bo_closed(PyObject* self_, void*) {
  auto* self = reinterpret_cast<PyBufferObject*>(self_);
  return PyBool_FromLong(mlf_buffer_is_closed(self->handle));
}

PyObject* bo_is_readonly(PyObject* self_, void*) {
  auto* self = reinterpret_cast<PyBufferObject*>(self_);
  return PyBool_FromLong(mlf_buffer_is_readonly(self->handle));
}

int bo_getbuffer(PyObject* self_, Py_buffer* view, int flags) {
  auto* self = reinterpret_cast<PyBufferObject*>(self_);
  if (mlf_buffer_is_closed(self->handle)) {
    // BufferError whose __cause__ is the RuntimeError that names the reason.
    PyObject* cause = PyObject_CallFunction(PyExc_RuntimeError, "s", "Cannot create buffer view on a closed BufferObject");
    PyObject* err = PyObject_CallFunction(PyExc_BufferError, "s", "Cannot create buffer view on a closed BufferObject");
    if (cause && err) {
      PyException_SetCause(err, cause);  // steals `cause`
      PyErr_SetObject(PyExc_BufferError, err);
    } else {
      Py_XDECREF(cause);
    }
    Py_XDECREF(err);
    view->obj = nullptr;
    return -1;
  }
  return PyBuffer_FillInfo(view, self_, mlf_buffer_data_ptr(self->handle), (Py_ssize_t)mlf_buffer_capacity(self->handle),
                           mlf_buffer_is_readonly(self->handle), flags);
}

PyMethodDef bo_methods[] = {
    {"close", (PyCFunction)(void (*)(void))bo_close, METH_VARARGS | METH_KEYWORDS, "Closes the buffer object."},
    {"resize", (PyCFunction)(void (*)(void))bo_resize, METH_VARARGS | METH_KEYWORDS, "Resizes the buffer object."},
    {"reserve", (PyCFunction)(void (*)(void))bo_reserve, METH_VARARGS | METH_KEYWORDS,
     "Allocates the pages of a byte range of the file now instead of at first touch."},
    {"prefault", (PyCFunction)(void (*)(void))bo_prefault, METH_VARARGS | METH_KEYWORDS,
     "Allocates the pages of a byte range and maps them writable, so that the first stores take no page fault."},
    {"get_id", bo_get_id, METH_NOARGS, "Gets the buffer object id."},
    {"get_capacity", bo_get_capacity, METH_NOARGS, "Gets the buffer object capacity."},
    {"get_data_ptr", bo_get_data_ptr, METH_NOARGS, "Returns the raw memory address of the buffer as an integer."},
    {"fileno", bo_fileno, METH_NOARGS, "Returns the descriptor of the mapped file (owned by the buffer object)."},
    {nullptr, nullptr, 0, nullptr}};

PyGetSetDef bo_getset[] = {{"closed", bo_closed, nullptr, "True once closed.", nullptr},
                           {"is_readonly", bo_is_readonly, nullptr, "True for read-only mappings.", nullptr},
                           {nullptr, nullptr, nullptr, nullptr, nullptr}};

PyBufferProcs bo_as_buffer = {bo_getbuffer, nullptr};

PyTypeObject BufferObjectType = {PyVarObject_HEAD_INIT(nullptr, 0)};

PyModuleDef module_def = {PyModuleDef_HEAD_INIT, "buffer_object_ext", "File-backed shared-memory buffer object", -1,
                          nullptr,               nullptr,             nullptr,                                   nullptr,
                          nullptr};

}  // namespace

PyMODINIT_FUNC PyInit_buffer_object_ext(void) {
  BufferObjectType.tp_name = "buffer_object_ext.BufferObject";
  BufferObjectType.tp_basicsize = sizeof(PyBufferObject);
  BufferObjectType.tp_flags = Py_TPFLAGS_DEFAULT;
  BufferObjectType.tp_doc = "mmap-ed file buffer (create read-write, or open read-only)";
  BufferObjectType.tp_new = PyType_GenericNew;
  BufferObjectType.tp_init = bo_init;
  BufferObjectType.tp_dealloc = bo_dealloc;
  BufferObjectType.tp_methods = bo_methods;
  BufferObjectType.tp_getset = bo_getset;
  BufferObjectType.tp_as_buffer = &bo_as_buffer;
  if (PyType_Ready(&BufferObjectType) < 0) return nullptr;
  PyObject* m = PyModule_Create(&module_def);
  if (!m) return nullptr;
  Py_INCREF(&BufferObjectType);
  if (PyModule_AddObject(m, "BufferObject", reinterpret_cast<PyObject*>(&BufferObjectType)) < 0) {
    Py_DECREF(&BufferObjectType);
    Py_DECREF(m);
    return nullptr;
  }
  return m;
}

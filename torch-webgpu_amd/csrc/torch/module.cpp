// Python module torch_webgpu._C.  Loading the shared object runs the static
// registrars (guard, allocator, operator kernels), as in the reference
// (csrc/bindings.cpp:46-58, whose module has an empty method table).  A few
// runtime helpers are exposed for the torch.webgpu device module.
#include <Python.h>

#include "twg.h"

namespace {

PyObject *raise_twg(int rc) {
  PyErr_Format(PyExc_RuntimeError, "torch_webgpu: %s (code %d)", twg_error_string(rc), rc);
  return nullptr;
}

PyObject *py_init(PyObject *, PyObject *) {
  int rc = twg_init();
  if (rc) return raise_twg(rc);
  Py_RETURN_NONE;
}

PyObject *py_is_initialized(PyObject *, PyObject *) { return PyBool_FromLong(twg_is_initialized()); }

PyObject *py_synchronize(PyObject *, PyObject *) {
  int rc;
  Py_BEGIN_ALLOW_THREADS rc = twg_stream_sync(nullptr);
  Py_END_ALLOW_THREADS if (rc) return raise_twg(rc);
  Py_RETURN_NONE;
}

PyObject *py_empty_cache(PyObject *, PyObject *) {
  int rc = twg_empty_cache();
  if (rc) return raise_twg(rc);
  Py_RETURN_NONE;
}

PyObject *py_memory_stats(PyObject *, PyObject *) {
  twg_mem_stats_t st;
  int rc = twg_mem_stats(&st);
  if (rc) return raise_twg(rc);
  return Py_BuildValue("{s:L,s:L,s:L,s:L,s:L}", "bytes_in_use", (long long)st.bytes_in_use,
                       "bytes_cached", (long long)st.bytes_cached, "n_device_mallocs",
                       (long long)st.n_device_mallocs, "n_cache_hits", (long long)st.n_cache_hits,
                       "n_allocs", (long long)st.n_allocs);
}

PyObject *py_device_info(PyObject *, PyObject *) {
  char name[256];
  int32_t cus = 0;
  int64_t mem = 0;
  int rc = twg_device_info(name, sizeof(name), &cus, &mem);
  if (rc) return raise_twg(rc);
  return Py_BuildValue("{s:s,s:i,s:L}", "name", name, "compute_units", (int)cus, "total_memory",
                       (long long)mem);
}

PyMethodDef methods[] = {
    {"_init", py_init, METH_NOARGS, "Bind the GPU and create the stream."},
    {"_is_initialized", py_is_initialized, METH_NOARGS, "True once the GPU is bound."},
    {"_synchronize", py_synchronize, METH_NOARGS, "Wait for all queued work."},
    {"_empty_cache", py_empty_cache, METH_NOARGS, "Return cached device blocks to the driver."},
    {"_memory_stats", py_memory_stats, METH_NOARGS, "Allocator counters."},
    {"_device_info", py_device_info, METH_NOARGS, "Name, compute units and memory of the GPU."},
    {nullptr, nullptr, 0, nullptr}};

struct PyModuleDef module_def = {PyModuleDef_HEAD_INIT, "torch_webgpu._C",
                                 "MI355X kernels behind the webgpu PrivateUse1 backend", -1, methods};

}  // namespace

PyMODINIT_FUNC PyInit__C(void) { return PyModule_Create(&module_def); }

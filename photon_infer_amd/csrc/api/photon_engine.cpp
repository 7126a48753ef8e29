// C entry points of the engine for C / C++ programs: an interpreter hosted in the calling
// process drives the package's own ContinuousBatchEngine (see photon_engine.h).
#include "photon_engine.h"

#include <Python.h>
#include <dlfcn.h>

#include <mutex>
#include <string>

namespace {

thread_local std::string g_error;
std::once_flag g_started;
bool g_we_started = false;

// the folder that holds the package: this library lies in <root>/photon_infer_amd/csrc/_build/
std::string package_root() {
  Dl_info info;
  if (!dladdr(reinterpret_cast<const void*>(&package_root), &info) || !info.dli_fname) return ".";
  std::string p(info.dli_fname);
  for (int up = 0; up < 4; ++up) {
    const size_t cut = p.find_last_of('/');
    if (cut == std::string::npos) return ".";
    p.erase(cut);
  }
  return p.empty() ? "/" : p;
}

void start_interpreter() {
  if (!Py_IsInitialized()) {
    Py_InitializeEx(0);          // no signal handlers: the host program keeps its own
    g_we_started = true;
  }
  PyGILState_STATE gil = PyGILState_Ensure();
  PyObject* sys_path = PySys_GetObject("path");   // borrowed
  const char* env_root = getenv("PHOTON_INFER_AMD_ROOT");
  PyObject* root = PyUnicode_FromString(env_root ? env_root : package_root().c_str());
  if (sys_path && root) PyList_Insert(sys_path, 0, root);
  Py_XDECREF(root);
  PyGILState_Release(gil);
  if (g_we_started) PyEval_SaveThread();   // every later call takes the lock through PyGILState_Ensure
}

// The pending Python exception as text, cleared.
std::string take_error() {
  PyObject *type = nullptr, *value = nullptr, *trace = nullptr;
  PyErr_Fetch(&type, &value, &trace);
  PyErr_NormalizeException(&type, &value, &trace);
  std::string text = "unknown error";
  if (value) {
    PyObject* s = PyObject_Str(value);
    if (s) {
      const char* c = PyUnicode_AsUTF8(s);
      if (c) text = c;
      Py_DECREF(s);
    }
    if (type) {
      PyObject* n = PyObject_GetAttrString(type, "__name__");
      if (n) {
        const char* c = PyUnicode_AsUTF8(n);
        if (c) text = std::string(c) + ": " + text;
        Py_DECREF(n);
      }
    }
  }
  Py_XDECREF(type); Py_XDECREF(value); Py_XDECREF(trace);
  PyErr_Clear();
  return text;
}

struct Gil {
  PyGILState_STATE s;
  Gil() : s(PyGILState_Ensure()) {}
  ~Gil() { PyGILState_Release(s); }
};

void set_item(PyObject* dict, const char* key, PyObject* value) {   // steals value
  if (value) {
    PyDict_SetItemString(dict, key, value);
    Py_DECREF(value);
  }
}

}  // namespace

struct pi_engine {
  PyObject* engine;   // photon_infer_amd.ContinuousBatchEngine
};

extern "C" {

const char* pi_engine_last_error(void) { return g_error.c_str(); }

pi_engine* pi_engine_create(const char* model_dir, const pi_engine_options* o) {
  if (!model_dir) { g_error = "pi_engine_create: no model folder given"; return nullptr; }
  std::call_once(g_started, start_interpreter);
  Gil gil;
  PyObject* pkg = PyImport_ImportModule("photon_infer_amd");
  if (!pkg) { g_error = take_error(); return nullptr; }
  PyObject* cls = PyObject_GetAttrString(pkg, "ContinuousBatchEngine");
  Py_DECREF(pkg);
  if (!cls) { g_error = take_error(); return nullptr; }
  PyObject* args = Py_BuildValue("(s)", model_dir);
  PyObject* kw = PyDict_New();
  if (o) {
    if (o->dtype && *o->dtype) set_item(kw, "dtype", PyUnicode_FromString(o->dtype));
    if (o->block_size > 0) set_item(kw, "block_size", PyLong_FromLong(o->block_size));
    if (o->num_blocks > 0) set_item(kw, "num_blocks", PyLong_FromLong(o->num_blocks));
    if (o->max_batch > 0) set_item(kw, "max_batch", PyLong_FromLong(o->max_batch));
    if (o->max_step_tokens > 0) set_item(kw, "max_step_tokens", PyLong_FromLong(o->max_step_tokens));
    if (o->chunk_size > 0) set_item(kw, "chunk_size", PyLong_FromLong(o->chunk_size));
    if (o->max_model_len > 0) set_item(kw, "max_model_len", PyLong_FromLong(o->max_model_len));
  }
  PyObject* eng = (args && kw) ? PyObject_Call(cls, args, kw) : nullptr;
  Py_XDECREF(args); Py_XDECREF(kw); Py_DECREF(cls);
  if (!eng) { g_error = take_error(); return nullptr; }
  return new pi_engine{eng};
}

void pi_engine_destroy(pi_engine* e) {
  if (!e) return;
  {
    Gil gil;
    Py_XDECREF(e->engine);
  }
  delete e;
}

long pi_engine_add_request(pi_engine* e, const int* tokens, int n, int max_new_tokens, float temperature, long seed,
                           int ignore_eos) {
  if (!e || (n > 0 && !tokens) || n < 0) { g_error = "pi_engine_add_request: bad arguments"; return -1; }
  Gil gil;
  PyObject* list = PyList_New(n);
  for (int i = 0; list && i < n; ++i) PyList_SET_ITEM(list, i, PyLong_FromLong(tokens[i]));
  PyObject* seed_obj = seed >= 0 ? PyLong_FromLong(seed) : (Py_INCREF(Py_None), Py_None);
  PyObject* r = list ? PyObject_CallMethod(e->engine, "add_request", "OidOO", list, max_new_tokens, (double)temperature,
                                           seed_obj, ignore_eos ? Py_True : Py_False)
                     : nullptr;
  Py_XDECREF(list); Py_XDECREF(seed_obj);
  if (!r) { g_error = take_error(); return -1; }
  const long id = PyLong_AsLong(r);
  Py_DECREF(r);
  if (id < 0 && PyErr_Occurred()) { g_error = take_error(); return -1; }
  return id;
}

int pi_engine_step(pi_engine* e) {
  if (!e) { g_error = "pi_engine_step: no engine"; return -1; }
  Gil gil;
  PyObject* r = PyObject_CallMethod(e->engine, "step", nullptr);
  if (!r) { g_error = take_error(); return -1; }
  const Py_ssize_t n = PySequence_Size(r);
  Py_DECREF(r);
  if (n < 0) { g_error = take_error(); return -1; }
  return (int)n;
}

int pi_engine_has_work(pi_engine* e) {
  if (!e) { g_error = "pi_engine_has_work: no engine"; return -1; }
  Gil gil;
  PyObject* r = PyObject_CallMethod(e->engine, "has_work", nullptr);
  if (!r) { g_error = take_error(); return -1; }
  const int v = PyObject_IsTrue(r);
  Py_DECREF(r);
  return v;
}

int pi_engine_run_until_complete(pi_engine* e) {
  if (!e) { g_error = "pi_engine_run_until_complete: no engine"; return -1; }
  Gil gil;
  PyObject* r = PyObject_CallMethod(e->engine, "run_until_complete", nullptr);
  if (!r) { g_error = take_error(); return -1; }
  Py_DECREF(r);
  return 0;
}

int pi_engine_result(pi_engine* e, long id, int* out, int capacity) {
  if (!e) { g_error = "pi_engine_result: no engine"; return -1; }
  Gil gil;
  PyObject* r = PyObject_CallMethod(e->engine, "get_result", "l", id);
  if (!r) { g_error = take_error(); return -1; }
  const Py_ssize_t n = PySequence_Size(r);
  for (Py_ssize_t i = 0; out && i < n && i < capacity; ++i) {
    PyObject* item = PySequence_GetItem(r, i);
    out[i] = item ? (int)PyLong_AsLong(item) : -1;
    Py_XDECREF(item);
  }
  Py_DECREF(r);
  if (n < 0 || PyErr_Occurred()) { g_error = take_error(); return -1; }
  return (int)n;
}

int pi_engine_finished(pi_engine* e, long id) {
  if (!e) { g_error = "pi_engine_finished: no engine"; return -1; }
  Gil gil;
  PyObject* req = PyObject_CallMethod(e->engine, "get_request", "l", id);
  if (!req) { g_error = take_error(); return -1; }
  if (req == Py_None) { Py_DECREF(req); g_error = "no request with this id"; return -1; }
  PyObject* r = PyObject_CallMethod(req, "is_finished", nullptr);
  Py_DECREF(req);
  if (!r) { g_error = take_error(); return -1; }
  const int v = PyObject_IsTrue(r);
  Py_DECREF(r);
  return v;
}

}  // extern "C"

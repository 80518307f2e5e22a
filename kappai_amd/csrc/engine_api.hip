// The C API of the engine (engine_api.h): a shell over kappai_amd.engine.capi.Session.
//
// No GPU code and no engine logic: every function takes the interpreter's lock, calls one method
// of the session with plain numbers (sizes, ids, addresses of the caller's buffers) and turns
// an exception into an error code and a message.  When the process has no interpreter yet, the
// first kappai_engine_create starts one and puts the package's folder on its path (the folder
// two levels above the one this library was loaded from).
#include "engine_api.h"

#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <dlfcn.h>
#include <limits.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <string>
#include <vector>

struct kappai_engine {
  PyObject* session;
};

namespace {

thread_local char g_error[512];

void set_error(const char* what) { snprintf(g_error, sizeof g_error, "%s", what); }

// the current Python exception as text (and cleared)
void error_from_python(const char* where) {
  PyObject *type = nullptr, *value = nullptr, *trace = nullptr;
  PyErr_Fetch(&type, &value, &trace);
  PyErr_NormalizeException(&type, &value, &trace);
  std::string text = where;
  text += ": ";
  if (type != nullptr) {
    PyObject* name = PyObject_GetAttrString(type, "__name__");
    if (name != nullptr) {
      const char* s = PyUnicode_AsUTF8(name);
      if (s != nullptr) text += s;
      Py_DECREF(name);
    }
  }
  if (value != nullptr) {
    PyObject* str = PyObject_Str(value);
    if (str != nullptr) {
      const char* s = PyUnicode_AsUTF8(str);
      if (s != nullptr) {
        text += ": ";
        text += s;
      }
      Py_DECREF(str);
    }
  }
  PyErr_Clear();
  Py_XDECREF(type);
  Py_XDECREF(value);
  Py_XDECREF(trace);
  set_error(text.c_str());
}

// The folder that holds the package: <root>/kappai_amd/csrc/_build/engine_api.so -> <root>,
// unless KAPPAI_AMD_ROOT names it.
std::string package_root() {
  const char* env = getenv("KAPPAI_AMD_ROOT");
  if (env != nullptr && env[0] != 0) return env;
  Dl_info info;
  if (dladdr((const void*)&package_root, &info) == 0 || info.dli_fname == nullptr) return "";
  char resolved[4096];
  if (realpath(info.dli_fname, resolved) == nullptr) return "";
  std::string path = resolved;
  for (int up = 0; up < 4; ++up) {
    const size_t slash = path.find_last_of('/');
    if (slash == std::string::npos) return "";
    path.erase(slash);
  }
  return path;
}

// Starts an interpreter if the process has none.  After this, every entry takes the lock with
// PyGILState_Ensure whoever owns the interpreter.
bool interpreter_ready() {
  static std::mutex starting;        // two first calls at once start one interpreter
  std::lock_guard<std::mutex> guard(starting);
  if (Py_IsInitialized()) return true;
  Py_InitializeEx(0);
  if (!Py_IsInitialized()) {
    set_error("kappai_engine: the Python interpreter could not be started");
    return false;
  }
  PyEval_SaveThread();               // release the lock the start-up left us holding
  return true;
}

struct Locked {                      // the interpreter's lock for the length of a call
  PyGILState_STATE state;
  Locked() : state(PyGILState_Ensure()) {}
  ~Locked() { PyGILState_Release(state); }
};

bool put_root_on_path() {
  const std::string root = package_root();
  if (root.empty()) return true;
  PyObject* sys_path = PySys_GetObject("path");       // borrowed
  if (sys_path == nullptr) return true;
  PyObject* entry = PyUnicode_FromString(root.c_str());
  if (entry == nullptr) return false;
  const int has = PySequence_Contains(sys_path, entry);
  if (has == 0) PyList_Insert(sys_path, 0, entry);
  Py_DECREF(entry);
  return true;
}

// session.<method>(*args) -> long, or -1 with the error set.  `format` as Py_BuildValue takes it.
long call_long(kappai_engine* engine, const char* method, const char* format, ...) {
  if (engine == nullptr || engine->session == nullptr) {
    set_error("kappai_engine: no engine");
    return -1;
  }
  va_list va;
  va_start(va, format);
  PyObject* args = Py_VaBuildValue(format, va);
  va_end(va);
  if (args == nullptr) {
    error_from_python(method);
    return -1;
  }
  PyObject* fn = PyObject_GetAttrString(engine->session, method);
  PyObject* result = fn ? PyObject_CallObject(fn, args) : nullptr;
  Py_XDECREF(fn);
  Py_DECREF(args);
  if (result == nullptr) {
    error_from_python(method);
    return -1;
  }
  const long value = result == Py_None ? 0 : PyLong_AsLong(result);
  Py_DECREF(result);
  if (value == -1 && PyErr_Occurred()) {
    error_from_python(method);
    return -1;
  }
  return value;
}

// An engine that kappai_engine_create returned, in a process whose interpreter still runs (the
// lock must not be asked for without one).
bool engine_ok(const kappai_engine* engine) {
  if (engine == nullptr || engine->session == nullptr || !Py_IsInitialized()) {
    set_error("kappai_engine: no engine");
    return false;
  }
  return true;
}

bool sampling_ok(const kappai_sampling* s) {
  if (s == nullptr) {
    set_error("kappai_engine: no sampling options");
    return false;
  }
  return true;
}

}  // namespace

extern "C" const char* kappai_engine_error(void) { return g_error; }

extern "C" void kappai_engine_config_default(kappai_engine_config* c) {
  if (c != nullptr) memset(c, 0, sizeof *c);
}

extern "C" void kappai_sampling_default(kappai_sampling* s) {
  if (s == nullptr) return;
  s->temperature = 0.80f;
  s->top_k = 40;
  s->top_p = 0.90f;
  s->min_p = 0.10f;
  s->repeat_penalty = 1.0f;
  s->repeat_last_n = 64;
  s->seed = 0;
  s->n_predict = -1;
}

extern "C" void kappai_sampling_greedy(kappai_sampling* s, int n_predict) {
  if (s == nullptr) return;
  kappai_sampling_default(s);
  s->temperature = 0.0f;
  s->top_k = 0;
  s->top_p = 1.0f;
  s->min_p = 0.0f;
  s->n_predict = n_predict;
}

extern "C" kappai_engine* kappai_engine_create(const kappai_engine_config* c) {
  g_error[0] = 0;
  if (c == nullptr || c->model == nullptr || c->model[0] == 0) {
    set_error("kappai_engine_create: the configuration names no model folder");
    return nullptr;
  }
  if (!interpreter_ready()) return nullptr;
  Locked lock;
  if (!put_root_on_path()) {
    error_from_python("kappai_engine_create");
    return nullptr;
  }
  PyObject* module = PyImport_ImportModule("kappai_amd.engine.capi");
  if (module == nullptr) {
    error_from_python("kappai_engine_create: import kappai_amd.engine.capi");
    return nullptr;
  }
  PyObject* options = Py_BuildValue(
      "{s:s,s:s,s:i,s:i,s:i,s:i,s:i,s:i,s:i}", "model", c->model, "dtype",
      (c->dtype != nullptr && c->dtype[0]) ? c->dtype : "bfloat16", "device", c->device,
      "ctx_size", c->ctx_size, "page_size", c->page_size, "num_pages", c->num_pages, "max_batch",
      c->max_batch, "token_budget", c->token_budget, "chunk", c->chunk);
  if (options != nullptr && c->decode_graphs != 0) {
    PyObject* flag = PyBool_FromLong(c->decode_graphs > 0);
    PyDict_SetItemString(options, "decode_graphs", flag);
    Py_DECREF(flag);
  }
  PyObject* session = options ? PyObject_CallMethod(module, "create", "O", options) : nullptr;
  Py_XDECREF(options);
  Py_DECREF(module);
  if (session == nullptr) {
    error_from_python("kappai_engine_create");
    return nullptr;
  }
  kappai_engine* engine = new kappai_engine{session};
  return engine;
}

extern "C" void kappai_engine_destroy(kappai_engine* engine) {
  if (engine == nullptr) return;
  if (engine->session != nullptr && Py_IsInitialized()) {
    Locked lock;
    PyObject* r = PyObject_CallMethod(engine->session, "close", nullptr);
    if (r == nullptr) PyErr_Clear();
    Py_XDECREF(r);
    Py_DECREF(engine->session);
  }
  delete engine;
}

extern "C" int kappai_engine_add_request(kappai_engine* engine, const int* ids, int n,
                                         const kappai_sampling* s) {
  g_error[0] = 0;
  if (!sampling_ok(s)) return -1;
  if (ids == nullptr || n < 1) {
    set_error("kappai_engine_add_request: a prompt needs at least one token");
    return -1;
  }
  if (!engine_ok(engine)) return -1;
  Locked lock;
  return (int)call_long(engine, "add_request", "(KififffiKi)", (unsigned long long)(uintptr_t)ids,
                        n, (double)s->temperature, s->top_k, (double)s->top_p, (double)s->min_p,
                        (double)s->repeat_penalty, s->repeat_last_n,
                        (unsigned long long)s->seed, s->n_predict);
}

extern "C" int kappai_engine_abort(kappai_engine* engine, int request_id) {
  g_error[0] = 0;
  if (!engine_ok(engine)) return -1;
  Locked lock;
  return (int)call_long(engine, "abort", "(i)", request_id);
}

extern "C" int kappai_engine_has_work(kappai_engine* engine) {
  g_error[0] = 0;
  if (!engine_ok(engine)) return -1;
  Locked lock;
  return (int)call_long(engine, "has_work", "()");
}

extern "C" int kappai_engine_step(kappai_engine* engine, kappai_step_output* outputs,
                                  int capacity) {
  g_error[0] = 0;
  if (capacity < 0 || (capacity > 0 && outputs == nullptr)) {
    set_error("kappai_engine_step: no place for the outputs");
    return -1;
  }
  if (!engine_ok(engine)) return -1;
  Locked lock;
  return (int)call_long(engine, "step", "(Ki)", (unsigned long long)(uintptr_t)outputs, capacity);
}

extern "C" int kappai_engine_output(kappai_engine* engine, int request_id, int* tokens,
                                    int capacity) {
  g_error[0] = 0;
  if (!engine_ok(engine)) return -1;
  Locked lock;
  return (int)call_long(engine, "output", "(iKi)", request_id,
                        (unsigned long long)(uintptr_t)tokens, tokens ? capacity : 0);
}

extern "C" int kappai_engine_release(kappai_engine* engine, int request_id) {
  g_error[0] = 0;
  if (!engine_ok(engine)) return -1;
  Locked lock;
  return (int)call_long(engine, "release", "(i)", request_id);
}

extern "C" int kappai_engine_generate(kappai_engine* engine, const int* ids, int n,
                                      const kappai_sampling* s, int* tokens, int capacity) {
  g_error[0] = 0;
  if (!sampling_ok(s)) return -1;
  if (ids == nullptr || n < 1) {
    set_error("kappai_engine_generate: a prompt needs at least one token");
    return -1;
  }
  if (!engine_ok(engine)) return -1;
  Locked lock;
  return (int)call_long(engine, "generate", "(KififffiKiKi)", (unsigned long long)(uintptr_t)ids,
                        n, (double)s->temperature, s->top_k, (double)s->top_p, (double)s->min_p,
                        (double)s->repeat_penalty, s->repeat_last_n,
                        (unsigned long long)s->seed, s->n_predict,
                        (unsigned long long)(uintptr_t)tokens, tokens ? capacity : 0);
}

extern "C" int kappai_engine_forward(kappai_engine* engine, const kappai_forward_entry* entries,
                                     int n_entries, float* logits, size_t capacity_floats) {
  g_error[0] = 0;
  if (entries == nullptr || n_entries < 1) {
    set_error("kappai_engine_forward: a step needs at least one entry");
    return -1;
  }
  // the entries' tables side by side, as the host reads them
  std::vector<int> ids(n_entries), counts(n_entries), want_counts(n_entries), tokens, want;
  for (int i = 0; i < n_entries; ++i) {
    const kappai_forward_entry& e = entries[i];
    if (e.n_tokens < 1 || e.tokens == nullptr || e.n_want < 0 || (e.n_want > 0 && e.want == nullptr)) {
      set_error("kappai_engine_forward: an entry brings no tokens, or wants rows it does not name");
      return -1;
    }
    ids[i] = e.request_id;
    counts[i] = e.n_tokens;
    want_counts[i] = e.n_want;
    tokens.insert(tokens.end(), e.tokens, e.tokens + e.n_tokens);
    want.insert(want.end(), e.want, e.want + e.n_want);
  }
  if (want.empty()) want.push_back(0);            // (an address to hand over; its count is 0)
  if (!engine_ok(engine)) return -1;
  Locked lock;
  return (int)call_long(engine, "forward", "(iKKKKKKK)", n_entries,
                        (unsigned long long)(uintptr_t)ids.data(),
                        (unsigned long long)(uintptr_t)counts.data(),
                        (unsigned long long)(uintptr_t)tokens.data(),
                        (unsigned long long)(uintptr_t)want_counts.data(),
                        (unsigned long long)(uintptr_t)want.data(),
                        (unsigned long long)(uintptr_t)logits,
                        (unsigned long long)capacity_floats);
}

extern "C" int kappai_engine_end(kappai_engine* engine, int request_id) {
  g_error[0] = 0;
  if (!engine_ok(engine)) return -1;
  Locked lock;
  return (int)call_long(engine, "end", "(i)", request_id);
}

extern "C" int kappai_engine_get_stats(kappai_engine* engine, kappai_engine_stats* stats) {
  g_error[0] = 0;
  if (stats == nullptr) {
    set_error("kappai_engine_get_stats: no place for the numbers");
    return -1;
  }
  if (!engine_ok(engine)) return -1;
  Locked lock;
  const long n = call_long(engine, "stats", "(Ki)", (unsigned long long)(uintptr_t)stats,
                           (int)(sizeof *stats / sizeof(double)));
  return n < 0 ? -1 : 0;
}

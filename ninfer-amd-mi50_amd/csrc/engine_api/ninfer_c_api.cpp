// The engine's C interface over an interpreter inside the calling process: every function
// takes the interpreter's lock, calls its namesake in ninfer_amd.api.c_bridge with plain
// integers (pointers travel as integers; the bridge reads and writes the caller's memory
// through ctypes) and turns a Python exception into a negative return code and a message.
// Reference: src/api/ninfer_c_api.cpp:54-260 (the same functions over its C++ engine).
#include "ninfer_c_api.h"

#include <Python.h>
#include <dlfcn.h>

#include <cstdarg>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>

struct ninfer_engine {
  PyObject* obj;   // ninfer_amd.Ninfer
};
struct ninfer_session {
  PyObject* obj;   // ninfer_amd.api.ninfer.Session
  ninfer_engine* engine;
};

namespace {

thread_local std::string last_error;
PyObject* bridge = nullptr;   // the module ninfer_amd.api.c_bridge
std::once_flag started;
bool start_failed = false;
std::string start_error;

// Where ninfer_amd.py makes the package importable: NINFER_AMD_ROOT of the environment, else
// the folder this library was built from, else four folders above the library's file
// (<root>/<package>/csrc/_build/lib*.so).
std::string repo_root() {
  if (const char* env = getenv("NINFER_AMD_ROOT")) return env;
#ifdef NINFER_AMD_ROOT
  return NINFER_AMD_ROOT;
#endif
  Dl_info info;
  if (!dladdr((void*)&repo_root, &info) || !info.dli_fname) return ".";
  std::string p = info.dli_fname;
  for (int up = 0; up < 4; ++up) {
    const size_t cut = p.find_last_of('/');
    if (cut == std::string::npos) return ".";
    p.resize(cut);
  }
  return p;
}

std::string fetch_exception() {
  PyObject *type = nullptr, *value = nullptr, *trace = nullptr;
  PyErr_Fetch(&type, &value, &trace);
  PyErr_NormalizeException(&type, &value, &trace);
  std::string text = "unknown Python error";
  if (value) {
    if (PyObject* s = PyObject_Str(value)) {
      if (const char* c = PyUnicode_AsUTF8(s)) text = c;
      Py_DECREF(s);
    }
    if (type) {
      if (PyObject* n = PyObject_GetAttrString(type, "__name__")) {
        if (const char* c = PyUnicode_AsUTF8(n)) text = std::string(c) + ": " + text;
        Py_DECREF(n);
      }
    }
  }
  PyErr_Clear();
  Py_XDECREF(type);
  Py_XDECREF(value);
  Py_XDECREF(trace);
  return text;
}

// Starts the interpreter if the process has none, and imports the bridge. Afterwards no
// thread holds the interpreter's lock on account of this library.
void start() {
  const bool own = !Py_IsInitialized();
  if (own) Py_InitializeEx(0);   // no signal handlers: the host program keeps its own
  PyGILState_STATE g = PyGILState_Ensure();
  const std::string root = repo_root();
  PyObject* sys_path = PySys_GetObject("path");   // borrowed
  PyObject* entry = PyUnicode_FromString(root.c_str());
  if (sys_path && entry && !PySequence_Contains(sys_path, entry)) PyList_Insert(sys_path, 0, entry);
  Py_XDECREF(entry);
  bridge = PyImport_ImportModule("ninfer_amd.api.c_bridge");
  if (!bridge) {
    start_failed = true;
    start_error = "cannot import ninfer_amd.api.c_bridge from " + root + ": " + fetch_exception();
  }
  PyGILState_Release(g);
  if (own) PyEval_SaveThread();   // the starting thread gives the lock up for good
}

struct Lock {
  PyGILState_STATE g;
  Lock() : g(PyGILState_Ensure()) {}
  ~Lock() { PyGILState_Release(g); }
};

bool ready() {
  std::call_once(started, start);
  if (start_failed) last_error = start_error;
  return !start_failed;
}

// bridge.<name>(*args) -> new reference, or null with last_error set. `fmt` as Py_BuildValue.
PyObject* call(const char* name, const char* fmt, ...) {
  PyObject* fn = PyObject_GetAttrString(bridge, name);
  if (!fn) {
    last_error = fetch_exception();
    return nullptr;
  }
  va_list va;
  va_start(va, fmt);
  PyObject* args = Py_VaBuildValue(fmt, va);
  va_end(va);
  PyObject* out = nullptr;
  if (args) {
    out = PyObject_CallObject(fn, args);
    Py_DECREF(args);
  }
  Py_DECREF(fn);
  if (!out) last_error = fetch_exception();
  return out;
}

long long as_number(PyObject* o, long long on_error) {
  if (!o) return on_error;
  const long long v = PyLong_AsLongLong(o);
  Py_DECREF(o);
  if (v == -1 && PyErr_Occurred()) {
    last_error = fetch_exception();
    return on_error;
  }
  return v;
}

long long engine_number(ninfer_engine_t* e, const char* what) {
  if (!e) return -1;
  Lock lock;
  return as_number(call("engine_number", "(Os)", e->obj, what), -1);
}

// the sessions' Python objects as a list (a new reference), or null with last_error set
PyObject* session_list(ninfer_session_t** sessions, int n, const char* who) {
  PyObject* list = PyList_New(n);
  if (!list) {
    last_error = fetch_exception();
    return nullptr;
  }
  for (int i = 0; i < n; ++i) {
    if (!sessions[i]) {
      Py_DECREF(list);
      last_error = std::string(who) + ": null session";
      return nullptr;
    }
    Py_INCREF(sessions[i]->obj);
    PyList_SET_ITEM(list, i, sessions[i]->obj);
  }
  return list;
}

}  // namespace

extern "C" {

const char* ninfer_last_error(void) { return last_error.c_str(); }

int ninfer_load(const char* model_dir, const ninfer_options_t* o, ninfer_engine_t** out_engine) {
  if (!model_dir || !out_engine) {
    last_error = "ninfer_load: null argument";
    return -1;
  }
  if (!ready()) return -1;
  Lock lock;
  PyObject* eng = call("load", "(siiiizz)", model_dir, o ? o->max_context : 0, o ? o->prefill_chunk : 0,
                       o ? o->num_sequences : 0, o ? o->gpu_count : 0, o ? o->quant : nullptr,
                       o ? o->parallel : nullptr);
  if (!eng) return -1;
  *out_engine = new ninfer_engine{eng};
  return 0;
}

void ninfer_engine_free(ninfer_engine_t* engine) {
  if (!engine) return;
  {
    Lock lock;
    Py_XDECREF(call("close", "(O)", engine->obj));
    Py_DECREF(engine->obj);
  }
  delete engine;
}

int ninfer_vocab_size(ninfer_engine_t* e) { return (int)engine_number(e, "vocab"); }
int ninfer_max_context(ninfer_engine_t* e) { return (int)engine_number(e, "max_context"); }
int ninfer_num_sequences(ninfer_engine_t* e) { return (int)engine_number(e, "num_sequences"); }
int ninfer_device_count(ninfer_engine_t* e) { return (int)engine_number(e, "devices"); }
long long ninfer_kv_bytes_per_token(ninfer_engine_t* e) { return engine_number(e, "kv_bytes_per_token"); }
long long ninfer_kv_total_bytes(ninfer_engine_t* e) { return engine_number(e, "kv_total_bytes"); }
long long ninfer_kv_seq_stride_elems(ninfer_engine_t* e) { return e ? 0 : -1; }

long long ninfer_kv_pages_total(ninfer_engine_t* e) { return engine_number(e, "pages_total"); }
long long ninfer_kv_pages_free(ninfer_engine_t* e) { return engine_number(e, "pages_free"); }
long long ninfer_kv_pages_reused(ninfer_engine_t* e) { return engine_number(e, "pages_reused"); }

int ninfer_tensor_read(ninfer_engine_t* engine, const char* name, long long offset, long long count,
                       float* out) {
  if (!engine || !name || !out || count < 0) {
    last_error = "ninfer_tensor_read: null argument or negative count";
    return -1;
  }
  Lock lock;
  return (int)as_number(call("tensor_read", "(OsLLK)", engine->obj, name, offset, count,
                             (unsigned long long)(uintptr_t)out), -1);
}

int ninfer_tokenize(ninfer_engine_t*, const char*, long long*, int) {
  last_error = "ninfer_tokenize: this engine has no tokenizer (token ids in, token ids out)";
  return -1;
}
int ninfer_detokenize(ninfer_engine_t*, const long long*, int, char*, int) {
  last_error = "ninfer_detokenize: this engine has no tokenizer (token ids in, token ids out)";
  return -1;
}

ninfer_session_t* ninfer_session_create(ninfer_engine_t* engine) {
  if (!engine) return nullptr;
  Lock lock;
  PyObject* s = call("session", "(O)", engine->obj);
  return s ? new ninfer_session{s, engine} : nullptr;
}

void ninfer_session_free(ninfer_session_t* session) {
  if (!session) return;
  {
    Lock lock;
    Py_XDECREF(call("session_close", "(O)", session->obj));
    Py_DECREF(session->obj);
  }
  delete session;
}

void ninfer_session_reset(ninfer_session_t* session) {
  if (!session) return;
  Lock lock;
  Py_XDECREF(call("session_reset", "(O)", session->obj));
}

int ninfer_session_slot(ninfer_session_t* s) {
  if (!s) return -1;
  Lock lock;
  return (int)as_number(call("session_number", "(Os)", s->obj, "slot"), -1);
}
int ninfer_session_length(ninfer_session_t* s) {
  if (!s) return -1;
  Lock lock;
  return (int)as_number(call("session_number", "(Os)", s->obj, "length"), -1);
}

int ninfer_prefill(ninfer_session_t* s, const long long* tokens, int count, float* out_logits, int capacity) {
  if (!s || !tokens || count <= 0 || !out_logits) {
    last_error = "ninfer_prefill: null argument or no tokens";
    return -1;
  }
  Lock lock;
  return (int)as_number(call("prefill", "(OKiKi)", s->obj, (unsigned long long)(uintptr_t)tokens, count,
                             (unsigned long long)(uintptr_t)out_logits, capacity), -1);
}

int ninfer_decode(ninfer_session_t* s, long long token, float* out_logits, int capacity) {
  if (!s || !out_logits) {
    last_error = "ninfer_decode: null argument";
    return -1;
  }
  Lock lock;
  return (int)as_number(call("decode", "(OLKi)", s->obj, token, (unsigned long long)(uintptr_t)out_logits,
                             capacity), -1);
}

int ninfer_decode_batch(ninfer_engine_t* engine, ninfer_session_t** sessions, const long long* tokens, int n,
                        float* out_logits, int capacity) {
  if (!engine || !sessions || !tokens || n <= 0 || !out_logits) {
    last_error = "ninfer_decode_batch: null argument or no sessions";
    return -1;
  }
  Lock lock;
  PyObject* list = session_list(sessions, n, "ninfer_decode_batch");
  if (!list) return -1;
  const int rc = (int)as_number(call("decode_batch", "(OOKKi)", engine->obj, list,
                                     (unsigned long long)(uintptr_t)tokens,
                                     (unsigned long long)(uintptr_t)out_logits, capacity), -1);
  Py_DECREF(list);
  return rc;
}

int ninfer_step(ninfer_engine_t* engine, ninfer_session_t** sessions, const int* q_len, int n_sessions,
                const long long* tokens, const int* logit_rows, int n_rows, float* out_logits,
                int capacity) {
  if (!engine || !sessions || !q_len || !tokens || n_sessions <= 0 || n_rows < 0 ||
      (n_rows > 0 && (!logit_rows || !out_logits))) {
    last_error = "ninfer_step: null argument or no sessions";
    return -1;
  }
  Lock lock;
  PyObject* list = session_list(sessions, n_sessions, "ninfer_step");
  if (!list) return -1;
  const int rc = (int)as_number(call("step", "(OOKKKiKi)", engine->obj, list,
                                     (unsigned long long)(uintptr_t)q_len,
                                     (unsigned long long)(uintptr_t)tokens,
                                     (unsigned long long)(uintptr_t)logit_rows, n_rows,
                                     (unsigned long long)(uintptr_t)out_logits, capacity), -1);
  Py_DECREF(list);
  return rc;
}

long long ninfer_request_add(ninfer_engine_t* engine, const long long* prompt, int count, int max_new_tokens,
                             float temperature, int top_k, float top_p, float repetition_penalty,
                             unsigned long long seed, const long long* stop_ids, int n_stop) {
  if (!engine || !prompt || count <= 0 || n_stop < 0 || (n_stop > 0 && !stop_ids)) {
    last_error = "ninfer_request_add: null argument or no prompt";
    return -1;
  }
  Lock lock;
  return as_number(call("request_add", "(OKiififfKKi)", engine->obj, (unsigned long long)(uintptr_t)prompt,
                        count, max_new_tokens, (double)temperature, top_k, (double)top_p,
                        (double)repetition_penalty, seed, (unsigned long long)(uintptr_t)stop_ids, n_stop),
                   -1);
}

int ninfer_run_step(ninfer_engine_t* engine) {
  if (!engine) return -1;
  Lock lock;
  return (int)as_number(call("run_step", "(O)", engine->obj), -1);
}

int ninfer_request_take(ninfer_engine_t* engine, long long id, long long* out_tokens, int capacity) {
  if (!engine || (capacity > 0 && !out_tokens) || capacity < 0) {
    last_error = "ninfer_request_take: null argument";
    return -1;
  }
  Lock lock;
  return (int)as_number(call("request_take", "(OLKi)", engine->obj, id,
                             (unsigned long long)(uintptr_t)out_tokens, capacity), -1);
}

long long ninfer_sample(ninfer_engine_t* engine, const float* logits, float temperature, int top_k, float top_p,
                        float repetition_penalty, unsigned long long seed) {
  if (!engine || !logits) {
    last_error = "ninfer_sample: null argument";
    return -1;
  }
  Lock lock;
  return as_number(call("sample", "(OKfiffK)", engine->obj, (unsigned long long)(uintptr_t)logits,
                        (double)temperature, top_k, (double)top_p, (double)repetition_penalty, seed), -1);
}

}  // extern "C"

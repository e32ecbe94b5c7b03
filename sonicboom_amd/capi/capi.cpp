// Implementation of sonicboom_amd.h: every call takes the interpreter lock, calls
// sonicboom_amd.capi.bridge.call(name, args...) and unpacks (status, result).  The package
// composes the model from parts and launches the HIP kernels; this file only carries handles,
// buffers and errors across the C boundary.  No exception crosses it: Python's are turned into
// statuses by the bridge, and anything this file itself meets becomes BOOM_ERR_INTERNAL.
#include "sonicboom_amd.h"

#include <Python.h>
#include <dlfcn.h>

#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_set>
#include <vector>

struct boom_error { std::string message; };
struct boom_llm_model { PyObject *obj; };
// A session's Python object holds its model: the session outlives boom_llm_model_free of the
// handle it was made from (/root/reference/capi/src/capi.cpp:2320-2350 keeps the model alive
// the same way).
struct boom_llm_session { PyObject *obj; };

namespace {

// The handles that are alive.  A handle is looked up here before it is touched, so a freed or
// made-up pointer is refused without being read (/root/reference/capi/src/capi.cpp:198-208).
std::mutex g_handles_lock;
std::unordered_set<const void *> g_models, g_sessions;

bool known(const std::unordered_set<const void *> &set, const void *h) {
  std::lock_guard<std::mutex> hold(g_handles_lock);
  return h && set.count(h) != 0;
}
void remember(std::unordered_set<const void *> &set, const void *h) {
  std::lock_guard<std::mutex> hold(g_handles_lock);
  set.insert(h);
}
bool forget(std::unordered_set<const void *> &set, const void *h) {
  std::lock_guard<std::mutex> hold(g_handles_lock);
  return h && set.erase(h) != 0;
}

boom_status fail(boom_error **slot, boom_status st, const std::string &msg) {
  if (slot) {
    delete *slot;                       // a handle from an earlier call is released first
    *slot = new (std::nothrow) boom_error{msg};
  }
  return st;
}

std::string package_root() {
  // <root>/sonicboom_amd/capi/_build/libsonicboom_amd.so  ->  <root>
  if (const char *env = std::getenv("SONICBOOM_AMD_ROOT")) return env;
  Dl_info info;
  if (!dladdr(reinterpret_cast<void *>(&boom_build_info), &info) || !info.dli_fname) return ".";
  std::string p = info.dli_fname;
  for (int up = 0; up < 4; ++up) {
    const size_t cut = p.find_last_of('/');
    if (cut == std::string::npos) return ".";
    p.erase(cut);
  }
  return p.empty() ? "/" : p;
}

std::once_flag g_once;
PyObject *g_call = nullptr;             // sonicboom_amd.capi.bridge.call
std::string g_init_error;

// Holds the interpreter lock for a scope.  A program without an interpreter gets one at the
// first call; its main thread then gives the lock up so that any thread may call in.
class Gil {
 public:
  Gil() {
    std::call_once(g_once, [] {
      if (!Py_IsInitialized()) {
#ifdef SB_LIBPYTHON
        // extension modules look the interpreter's symbols up globally; a program that loaded
        // this library privately (dlopen without RTLD_GLOBAL) would leave them unresolved
        dlopen(SB_LIBPYTHON, RTLD_NOW | RTLD_GLOBAL);
#endif
        Py_InitializeEx(0);
        PyEval_SaveThread();
      }
    });
    state_ = PyGILState_Ensure();
    if (!g_call && g_init_error.empty()) import_bridge();
  }
  ~Gil() { PyGILState_Release(state_); }

 private:
  static void import_bridge() {
    const std::string root = package_root();
    PyObject *sys_path = PySys_GetObject("path");       // borrowed
    PyObject *root_str = PyUnicode_FromString(root.c_str());
    if (sys_path && root_str && !PySequence_Contains(sys_path, root_str)) PyList_Insert(sys_path, 0, root_str);
    Py_XDECREF(root_str);
    PyObject *mod = PyImport_ImportModule("sonicboom_amd.capi.bridge");
    if (mod) {
      g_call = PyObject_GetAttrString(mod, "call");
      Py_DECREF(mod);
    }
    if (!g_call) {
      PyObject *type = nullptr, *value = nullptr, *tb = nullptr;
      PyErr_Fetch(&type, &value, &tb);
      PyObject *text = value ? PyObject_Str(value) : nullptr;
      const char *c = text ? PyUnicode_AsUTF8(text) : nullptr;
      g_init_error = std::string("cannot import sonicboom_amd.capi.bridge from ") + root + ": " + (c ? c : "?");
      Py_XDECREF(text); Py_XDECREF(type); Py_XDECREF(value); Py_XDECREF(tb);
      PyErr_Clear();
    }
  }
  PyGILState_STATE state_;
};

// Calls bridge.call(name, *args) (steals args).  On success *result holds a new reference.
boom_status bridge(const char *name, PyObject *args, PyObject **result, boom_error **err) {
  if (result) *result = nullptr;
  if (!g_call) {
    Py_XDECREF(args);
    return fail(err, BOOM_ERR_RUNTIME, g_init_error.empty() ? "the Python side is not available" : g_init_error);
  }
  if (!args) {
    PyErr_Clear();
    return fail(err, BOOM_ERR_INTERNAL, std::string(name) + ": could not build the arguments");
  }
  const Py_ssize_t n = PyTuple_Size(args);
  PyObject *full = PyTuple_New(n + 1);
  PyTuple_SetItem(full, 0, PyUnicode_FromString(name));
  for (Py_ssize_t i = 0; i < n; ++i) {
    PyObject *it = PyTuple_GetItem(args, i);
    Py_INCREF(it);
    PyTuple_SetItem(full, i + 1, it);
  }
  Py_DECREF(args);
  PyObject *ret = PyObject_CallObject(g_call, full);
  Py_DECREF(full);
  if (!ret || !PyTuple_Check(ret) || PyTuple_Size(ret) != 2) {
    PyErr_Clear();
    Py_XDECREF(ret);
    return fail(err, BOOM_ERR_INTERNAL, std::string(name) + ": the bridge did not answer");
  }
  const long st = PyLong_AsLong(PyTuple_GetItem(ret, 0));
  PyObject *val = PyTuple_GetItem(ret, 1);
  if (st != 0) {
    const char *c = PyUnicode_Check(val) ? PyUnicode_AsUTF8(val) : nullptr;
    const std::string msg = c ? c : "unknown failure";
    Py_DECREF(ret);
    PyErr_Clear();
    return fail(err, static_cast<boom_status>(st), msg);
  }
  if (result) {
    Py_INCREF(val);
    *result = val;
  }
  Py_DECREF(ret);
  return BOOM_OK;
}

const char *dtype_of(const boom_llm_load_options *o) {
  return (o && o->struct_size >= offsetof(boom_llm_load_options, dtype) + sizeof(o->dtype) && o->dtype) ? o->dtype
                                                                                                       : "bfloat16";
}
int device_of(const boom_llm_load_options *o) {
  return (o && o->struct_size >= offsetof(boom_llm_load_options, device) + sizeof(o->device)) ? o->device : 0;
}
bool live(const boom_llm_model *m) { return known(g_models, m); }
bool live(const boom_llm_session *s) { return known(g_sessions, s); }

boom_status wrap_model(PyObject *obj, boom_llm_model **out, boom_error **err) {
  boom_llm_model *m = new (std::nothrow) boom_llm_model{obj};
  if (!m) {
    Py_DECREF(obj);
    return fail(err, BOOM_ERR_INTERNAL, "out of memory");
  }
  remember(g_models, m);
  *out = m;
  return BOOM_OK;
}

}  // namespace

extern "C" {

boom_status boom_llm_model_load(const char *folder, const boom_llm_load_options *options,
                                boom_llm_model **model_out, boom_error **err_out) {
  if (!folder || !model_out) return fail(err_out, BOOM_ERR_INTERNAL, "boom_llm_model_load: NULL argument");
  *model_out = nullptr;
  Gil gil;
  PyObject *obj = nullptr;
  const boom_status st = bridge("model_load", Py_BuildValue("(ssi)", folder, dtype_of(options), device_of(options)),
                                &obj, err_out);
  return st != BOOM_OK ? st : wrap_model(obj, model_out, err_out);
}

boom_status boom_llm_model_random(const char *config_json_path, uint64_t seed, const boom_llm_load_options *options,
                                  boom_llm_model **model_out, boom_error **err_out) {
  if (!config_json_path || !model_out)
    return fail(err_out, BOOM_ERR_INTERNAL, "boom_llm_model_random: NULL argument");
  *model_out = nullptr;
  Gil gil;
  PyObject *obj = nullptr;
  const boom_status st =
      bridge("model_random",
             Py_BuildValue("(sKsi)", config_json_path, (unsigned long long)seed, dtype_of(options), device_of(options)),
             &obj, err_out);
  return st != BOOM_OK ? st : wrap_model(obj, model_out, err_out);
}

void boom_llm_model_free(boom_llm_model *model) {
  if (!forget(g_models, model)) return;      // NULL, made up, or freed before
  Gil gil;
  Py_DECREF(model->obj);
  delete model;
}

boom_status boom_llm_model_arch(const boom_llm_model *model, char *out, size_t cap, size_t *len_out,
                                boom_error **err_out) {
  if (!live(model) || !len_out) return fail(err_out, BOOM_ERR_INTERNAL, "boom_llm_model_arch: bad argument");
  Gil gil;
  PyObject *res = nullptr;
  const boom_status st = bridge("model_arch", Py_BuildValue("(O)", model->obj), &res, err_out);
  if (st != BOOM_OK) return st;
  Py_ssize_t n = 0;
  const char *c = PyUnicode_AsUTF8AndSize(res, &n);
  *len_out = size_t(n) + 1;              // with the NUL
  boom_status rc = BOOM_OK;
  if (!c) rc = fail(err_out, BOOM_ERR_INTERNAL, "boom_llm_model_arch: not a string");
  else if (!out || cap < size_t(n) + 1) rc = fail(err_out, BOOM_ERR_BINDING, "boom_llm_model_arch: buffer too small");
  else std::memcpy(out, c, size_t(n) + 1);
  Py_DECREF(res);
  return rc;
}

boom_status boom_llm_model_eos(const boom_llm_model *model, boom_token *out, size_t cap, size_t *n_out,
                               boom_error **err_out) {
  if (!live(model) || !n_out) return fail(err_out, BOOM_ERR_INTERNAL, "boom_llm_model_eos: bad argument");
  Gil gil;
  PyObject *res = nullptr;
  const boom_status st = bridge("model_eos", Py_BuildValue("(O)", model->obj), &res, err_out);
  if (st != BOOM_OK) return st;
  const Py_ssize_t n = PyList_Size(res);
  *n_out = size_t(n < 0 ? 0 : n);
  boom_status rc = BOOM_OK;
  if (n > 0 && (!out || cap < size_t(n))) rc = fail(err_out, BOOM_ERR_BINDING, "boom_llm_model_eos: buffer too small");
  else
    for (Py_ssize_t i = 0; i < n; ++i) out[i] = (boom_token)PyLong_AsLong(PyList_GetItem(res, i));
  Py_DECREF(res);
  return rc;
}

boom_status boom_llm_model_vocab(const boom_llm_model *model, uint32_t *vocab_out, boom_error **err_out) {
  if (!live(model) || !vocab_out) return fail(err_out, BOOM_ERR_INTERNAL, "boom_llm_model_vocab: bad argument");
  Gil gil;
  PyObject *res = nullptr;
  const boom_status st = bridge("model_vocab", Py_BuildValue("(O)", model->obj), &res, err_out);
  if (st != BOOM_OK) return st;
  *vocab_out = (uint32_t)PyLong_AsUnsignedLong(res);
  Py_DECREF(res);
  return BOOM_OK;
}

boom_status boom_llm_session_new(boom_llm_model *model, uint64_t max_tokens, boom_llm_session **session_out,
                                 boom_error **err_out) {
  if (!live(model) || !session_out) return fail(err_out, BOOM_ERR_INTERNAL, "boom_llm_session_new: bad argument");
  *session_out = nullptr;
  Gil gil;
  PyObject *obj = nullptr;
  const boom_status st =
      bridge("session_new", Py_BuildValue("(OK)", model->obj, (unsigned long long)max_tokens), &obj, err_out);
  if (st != BOOM_OK) return st;
  boom_llm_session *s = new (std::nothrow) boom_llm_session{obj};
  if (!s) {
    Py_DECREF(obj);
    return fail(err_out, BOOM_ERR_INTERNAL, "out of memory");
  }
  remember(g_sessions, s);
  *session_out = s;
  return BOOM_OK;
}

void boom_llm_session_free(boom_llm_session *session) {
  if (!forget(g_sessions, session)) return;
  Gil gil;
  Py_DECREF(session->obj);
  delete session;
}

boom_status boom_llm_slot_alloc(boom_llm_session *session, int32_t *slot_out, boom_error **err_out) {
  if (!live(session) || !slot_out) return fail(err_out, BOOM_ERR_INTERNAL, "boom_llm_slot_alloc: bad argument");
  Gil gil;
  PyObject *res = nullptr;
  const boom_status st = bridge("slot_alloc", Py_BuildValue("(O)", session->obj), &res, err_out);
  if (st != BOOM_OK) return st;
  *slot_out = (int32_t)PyLong_AsLong(res);
  Py_DECREF(res);
  return BOOM_OK;
}

boom_status boom_llm_slot_free(boom_llm_session *session, int32_t slot, boom_error **err_out) {
  if (!live(session)) return fail(err_out, BOOM_ERR_INTERNAL, "boom_llm_slot_free: bad argument");
  Gil gil;
  return bridge("slot_free", Py_BuildValue("(Oi)", session->obj, (int)slot), nullptr, err_out);
}

boom_status boom_llm_step(boom_llm_session *session, const boom_llm_step_entry *entries, size_t n_entries,
                          float *logits_out, size_t cap, size_t *n_out, boom_error **err_out) {
  if (!live(session) || (!entries && n_entries) || !n_out)
    return fail(err_out, BOOM_ERR_INTERNAL, "boom_llm_step: bad argument");
  Gil gil;
  uint32_t vocab = 0;
  {
    PyObject *res = nullptr;
    const boom_status st = bridge("session_vocab", Py_BuildValue("(O)", session->obj), &res, err_out);
    if (st != BOOM_OK) return st;
    vocab = (uint32_t)PyLong_AsUnsignedLong(res);
    Py_DECREF(res);
  }
  size_t wanted = 0;
  for (size_t i = 0; i < n_entries; ++i) {
    if ((!entries[i].tokens && entries[i].n_tokens) || (!entries[i].want && entries[i].n_want))
      return fail(err_out, BOOM_ERR_INTERNAL, "boom_llm_step: an entry holds a NULL array");
    wanted += entries[i].n_want;
  }
  *n_out = wanted * vocab;
  if (*n_out > cap || (*n_out && !logits_out))
    return fail(err_out, BOOM_ERR_BINDING, "boom_llm_step: the logits buffer is too small; nothing ran");
  PyObject *list = PyList_New((Py_ssize_t)n_entries);
  for (size_t i = 0; list && i < n_entries; ++i) {
    const boom_llm_step_entry &e = entries[i];
    PyObject *toks = PyList_New((Py_ssize_t)e.n_tokens), *want = PyList_New((Py_ssize_t)e.n_want);
    for (size_t j = 0; j < e.n_tokens; ++j) PyList_SetItem(toks, (Py_ssize_t)j, PyLong_FromLong(e.tokens[j]));
    for (size_t j = 0; j < e.n_want; ++j) PyList_SetItem(want, (Py_ssize_t)j, PyLong_FromUnsignedLong(e.want[j]));
    PyList_SetItem(list, (Py_ssize_t)i, Py_BuildValue("(iNN)", (int)e.slot, toks, want));
  }
  PyObject *res = nullptr;
  const boom_status st =
      bridge("step", Py_BuildValue("(ONK)", session->obj, list, (unsigned long long)(uintptr_t)logits_out), &res,
             err_out);
  Py_XDECREF(res);
  return st;
}

boom_status boom_llm_generate(boom_llm_session *session, const boom_token *const *prompts, const size_t *prompt_lens,
                              size_t n_prompts, const boom_llm_sampling *sampling, const boom_token *stop,
                              size_t n_stop, boom_llm_batch_token_cb cb, void *user, boom_token *out, uint32_t *n_out,
                              boom_error **err_out) {
  if (!live(session) || !sampling || (n_prompts && (!prompts || !prompt_lens || !n_out)) || (!stop && n_stop))
    return fail(err_out, BOOM_ERR_INTERNAL, "boom_llm_generate: bad argument");
  boom_llm_sampling sp;
  std::memset(&sp, 0, sizeof sp);
  std::memcpy(&sp, sampling, sampling->struct_size < sizeof sp ? sampling->struct_size : sizeof sp);
  // A struct too short to hold repeat_last_n gets the default window of 64; a 0 the caller wrote
  // is an empty window and switches every penalty off (/root/reference/capi/src/capi.cpp:2651-2653).
  if (sampling->struct_size < offsetof(boom_llm_sampling, repeat_last_n) + sizeof(sp.repeat_last_n))
    sp.repeat_last_n = 64;
  if (sampling->struct_size < offsetof(boom_llm_sampling, max_tokens) + sizeof(sp.max_tokens))
    return fail(err_out, BOOM_ERR_BINDING, "boom_llm_generate: sampling.struct_size does not reach max_tokens");
  if (sp.temperature < 0.f) return fail(err_out, BOOM_ERR_BINDING, "boom_llm_generate: temperature must be >= 0");
  if (sp.top_p < 0.f || sp.top_p > 1.f) return fail(err_out, BOOM_ERR_BINDING, "boom_llm_generate: top_p not in [0, 1]");
  if (n_prompts && sp.max_tokens && !out) return fail(err_out, BOOM_ERR_INTERNAL, "boom_llm_generate: no output buffer");
  Gil gil;
  PyObject *plist = PyList_New((Py_ssize_t)n_prompts);
  for (size_t i = 0; plist && i < n_prompts; ++i) {
    PyObject *toks = PyList_New((Py_ssize_t)prompt_lens[i]);
    for (size_t j = 0; j < prompt_lens[i]; ++j) PyList_SetItem(toks, (Py_ssize_t)j, PyLong_FromLong(prompts[i][j]));
    PyList_SetItem(plist, (Py_ssize_t)i, toks);
  }
  PyObject *opts = Py_BuildValue(
      "{s:f,s:f,s:I,s:K,s:I,s:f,s:f,s:I,s:f,s:f}", "temperature", sp.temperature, "top_p",
      (sp.top_p == 0.f ? 1.f : sp.top_p), "top_k", sp.top_k, "seed", (unsigned long long)sp.seed, "max_tokens",
      sp.max_tokens, "min_p", sp.min_p, "repeat_penalty", (sp.repeat_penalty == 0.f ? 1.f : sp.repeat_penalty),
      "repeat_last_n", sp.repeat_last_n, "presence_penalty", sp.presence_penalty,
      "frequency_penalty", sp.frequency_penalty);
  PyObject *stops;
  if (stop) {
    stops = PyList_New((Py_ssize_t)n_stop);
    for (size_t i = 0; i < n_stop; ++i) PyList_SetItem(stops, (Py_ssize_t)i, PyLong_FromLong(stop[i]));
  } else {
    stops = Py_None;
    Py_INCREF(stops);
  }
  PyObject *res = nullptr;
  const boom_status st =
      bridge("generate",
             Py_BuildValue("(ONNNKKKK)", session->obj, plist, opts, stops, (unsigned long long)(uintptr_t)cb,
                           (unsigned long long)(uintptr_t)user, (unsigned long long)(uintptr_t)out,
                           (unsigned long long)(uintptr_t)n_out),
             &res, err_out);
  Py_XDECREF(res);
  return st;
}

boom_status boom_llm_session_keep(boom_llm_session *session, int keep, boom_error **err_out) {
  if (!live(session)) return fail(err_out, BOOM_ERR_INTERNAL, "boom_llm_session_keep: bad argument");
  Gil gil;
  return bridge("session_keep", Py_BuildValue("(Oi)", session->obj, keep ? 1 : 0), nullptr, err_out);
}

boom_status boom_llm_session_reused(boom_llm_session *session, uint64_t *out, size_t cap, size_t *n_out,
                                    boom_error **err_out) {
  if (!live(session) || !n_out || (!out && cap))
    return fail(err_out, BOOM_ERR_INTERNAL, "boom_llm_session_reused: bad argument");
  Gil gil;
  PyObject *res = nullptr;
  const boom_status st =
      bridge("session_reused",
             Py_BuildValue("(OKK)", session->obj, (unsigned long long)(uintptr_t)out, (unsigned long long)cap), &res,
             err_out);
  if (st != BOOM_OK) return st;
  *n_out = (size_t)PyLong_AsUnsignedLongLong(res);
  Py_DECREF(res);
  if (*n_out > cap) return fail(err_out, BOOM_ERR_BINDING, "boom_llm_session_reused: the buffer is too small");
  return BOOM_OK;
}

const char *boom_error_message(const boom_error *err) { return err ? err->message.c_str() : ""; }
void boom_error_free(boom_error *err) { delete err; }

const char *boom_build_info(void) {
  static std::string info;
  Gil gil;
  PyObject *res = nullptr;
  if (bridge("build_info", PyTuple_New(0), &res, nullptr) == BOOM_OK && res) {
    const char *c = PyUnicode_AsUTF8(res);
    info = c ? c : "{}";
    Py_DECREF(res);
  } else if (info.empty()) {
    info = "{\"package\": \"sonicboom_amd\", \"python\": \"unavailable\"}";
  }
  return info.c_str();
}

}  // extern "C"

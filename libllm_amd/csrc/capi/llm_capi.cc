// The C API over the Python package: handles hold Python objects, arguments travel as JSON text,
// and every call takes the interpreter's lock for its duration.  See llm.h.
#include "llm.h"

#include <Python.h>
#include <dlfcn.h>

#include <sys/stat.h>

#include <cstring>
#include <string>

#ifndef LIBLLM_AMD_ROOT
#define LIBLLM_AMD_ROOT ""
#endif

struct llm_json_impl_t {
  std::string text = "{}";
};
struct llm_model_impl_t {
  PyObject *model = nullptr;
};
struct llm_completion_impl_t {
  PyObject *chunks = nullptr;
};

namespace {

thread_local std::string g_error;
PyObject *g_capi = nullptr;      // the module libllm_amd.capi
bool g_started_here = false;

int32_t fail(int32_t code, const std::string &msg) {
  g_error = msg;
  return code;
}

// The pending Python exception as text (and cleared).
std::string take_python_error() {
  PyObject *type = nullptr, *value = nullptr, *trace = nullptr;
  PyErr_Fetch(&type, &value, &trace);
  PyErr_NormalizeException(&type, &value, &trace);
  std::string msg = "unknown error";
  if (value != nullptr) {
    PyObject *s = PyObject_Str(value);
    if (s != nullptr) {
      const char *c = PyUnicode_AsUTF8(s);
      if (c != nullptr) msg = c;
      Py_DECREF(s);
    }
  }
  if (type != nullptr) {
    PyObject *n = PyObject_GetAttrString(type, "__name__");
    if (n != nullptr) {
      const char *c = PyUnicode_AsUTF8(n);
      if (c != nullptr) msg = std::string(c) + ": " + msg;
      Py_DECREF(n);
    }
  }
  Py_XDECREF(type);
  Py_XDECREF(value);
  Py_XDECREF(trace);
  PyErr_Clear();
  return msg;
}

bool holds_package(const std::string &root) {
  struct stat st;
  return !root.empty() && stat((root + "/libllm_amd/__init__.py").c_str(), &st) == 0;
}

// The folder that holds the package: this library lies in <root>/libllm_amd/_lib/; if it was
// built elsewhere, the folder known when it was compiled.
std::string package_root() {
  Dl_info info;
  if (dladdr(reinterpret_cast<void *>(&llm_init), &info) != 0 && info.dli_fname != nullptr) {
    std::string path = info.dli_fname;
    for (int up = 0; up < 3 && !path.empty(); ++up) {
      const size_t slash = path.find_last_of('/');
      path = slash == std::string::npos ? "" : path.substr(0, slash);
    }
    if (holds_package(path)) return path;
  }
  return holds_package(LIBLLM_AMD_ROOT) ? LIBLLM_AMD_ROOT : "";
}

struct Gil {
  PyGILState_STATE state;
  Gil() : state(PyGILState_Ensure()) {}
  ~Gil() { PyGILState_Release(state); }
};

bool ensure_module() {
  if (g_capi != nullptr) return true;
  const std::string root = package_root();
  if (!root.empty()) {
    PyObject *sys_path = PySys_GetObject("path");       // borrowed
    PyObject *entry = PyUnicode_FromString(root.c_str());
    if (sys_path != nullptr && entry != nullptr && PySequence_Contains(sys_path, entry) == 0)
      PyList_Insert(sys_path, 0, entry);
    Py_XDECREF(entry);
  }
  g_capi = PyImport_ImportModule("libllm_amd.capi");
  if (g_capi == nullptr) {
    g_error = "cannot import libllm_amd.capi: " + take_python_error();
    return false;
  }
  return true;
}

// Calls libllm_amd.capi.<name>(args...) ; a new reference or nullptr with g_error set.
PyObject *call(const char *name, PyObject *args) {
  if (!ensure_module()) {
    Py_XDECREF(args);
    return nullptr;
  }
  PyObject *fn = PyObject_GetAttrString(g_capi, name);
  PyObject *out = (fn != nullptr && args != nullptr) ? PyObject_CallObject(fn, args) : nullptr;
  Py_XDECREF(fn);
  Py_XDECREF(args);
  if (out == nullptr) g_error = take_python_error();
  return out;
}

}  // namespace

extern "C" {

void llm_init(void) {
  if (!Py_IsInitialized()) {
    Py_InitializeEx(0);
    g_started_here = true;
    PyEval_SaveThread();          // calls take the lock themselves
  }
}

const char *llm_get_last_error_message(void) { return g_error.c_str(); }

int32_t llm_json_init(llm_json_t *j) {
  if (j == nullptr) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: j");
  *j = new llm_json_impl_t();
  return 0;
}

int32_t llm_json_destroy(llm_json_t *j) {
  if (j == nullptr) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: j");
  delete *j;
  *j = nullptr;
  return 0;
}

int32_t llm_json_parse(llm_json_t *j, const char *json_str) {
  if (j == nullptr || *j == nullptr) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: j");
  if (json_str == nullptr) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: json_str");
  if (!Py_IsInitialized()) return fail(LLM_ERROR_ABORTED, "llm_init() was not called");
  Gil gil;
  PyObject *out = call("parse", Py_BuildValue("(s)", json_str));
  if (out == nullptr) return LLM_ERROR_ABORTED;
  const char *c = PyUnicode_AsUTF8(out);
  if (c != nullptr) (*j)->text = c;
  Py_DECREF(out);
  return 0;
}

int32_t llm_json_dump(llm_json_t *j, char *buf, int64_t buf_size) {
  if (j == nullptr || *j == nullptr) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: j");
  if (buf == nullptr || buf_size <= 0) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: buf");
  const std::string &text = (*j)->text;
  if ((int64_t)text.size() + 1 > buf_size) return fail(LLM_ERROR_INSUFFICIENT_BUFFER, "insufficient buffer");
  std::memcpy(buf, text.c_str(), text.size() + 1);
  return 0;
}

int32_t llm_model_init(llm_model_t *m) {
  if (m == nullptr) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: m");
  *m = new llm_model_impl_t();
  return 0;
}

int32_t llm_model_destroy(llm_model_t *m) {
  if (m == nullptr) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: m");
  if (*m != nullptr && (*m)->model != nullptr && Py_IsInitialized()) {
    Gil gil;
    Py_DECREF((*m)->model);
  }
  delete *m;
  *m = nullptr;
  return 0;
}

int32_t llm_model_load(llm_model_t *m, llm_json_t *kwargs) {
  if (m == nullptr || *m == nullptr) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: m");
  if (kwargs == nullptr || *kwargs == nullptr) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: kwargs");
  if (!Py_IsInitialized()) return fail(LLM_ERROR_ABORTED, "llm_init() was not called");
  Gil gil;
  PyObject *model = call("load", Py_BuildValue("(s)", (*kwargs)->text.c_str()));
  if (model == nullptr) return LLM_ERROR_ABORTED;
  Py_XDECREF((*m)->model);
  (*m)->model = model;
  return 0;
}

int32_t llm_model_get_info(llm_model_t *m, llm_json_t *info) {
  if (m == nullptr || *m == nullptr || (*m)->model == nullptr)
    return fail(LLM_ERROR_INVALID_ARG, "invalid argument: m");
  if (info == nullptr || *info == nullptr) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: info");
  Gil gil;
  PyObject *out = call("info", Py_BuildValue("(O)", (*m)->model));
  if (out == nullptr) return LLM_ERROR_ABORTED;
  const char *c = PyUnicode_AsUTF8(out);
  if (c != nullptr) (*info)->text = c;
  Py_DECREF(out);
  return 0;
}

int32_t llm_model_complete(llm_model_t *m, llm_json_t *kwargs, llm_completion_t *comp) {
  if (m == nullptr || *m == nullptr || (*m)->model == nullptr)
    return fail(LLM_ERROR_INVALID_ARG, "invalid argument: m");
  if (kwargs == nullptr || *kwargs == nullptr) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: kwargs");
  if (comp == nullptr || *comp == nullptr) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: comp");
  Gil gil;
  PyObject *chunks = call("complete", Py_BuildValue("(Os)", (*m)->model, (*kwargs)->text.c_str()));
  if (chunks == nullptr) return LLM_ERROR_ABORTED;
  Py_XDECREF((*comp)->chunks);
  (*comp)->chunks = chunks;
  return 0;
}

int32_t llm_model_generate(llm_model_t *m, llm_json_t *kwargs, llm_json_t *result) {
  if (m == nullptr || *m == nullptr || (*m)->model == nullptr)
    return fail(LLM_ERROR_INVALID_ARG, "invalid argument: m");
  if (kwargs == nullptr || *kwargs == nullptr) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: kwargs");
  if (result == nullptr || *result == nullptr) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: result");
  Gil gil;
  PyObject *out = call("generate", Py_BuildValue("(Os)", (*m)->model, (*kwargs)->text.c_str()));
  if (out == nullptr) return LLM_ERROR_ABORTED;
  const char *c = PyUnicode_AsUTF8(out);
  if (c != nullptr) (*result)->text = c;
  Py_DECREF(out);
  return 0;
}

int32_t llm_model_step(llm_model_t *m, llm_json_t *kwargs, float *logits, int64_t capacity, int64_t *n_rows) {
  if (m == nullptr || *m == nullptr || (*m)->model == nullptr)
    return fail(LLM_ERROR_INVALID_ARG, "invalid argument: m");
  if (kwargs == nullptr || *kwargs == nullptr) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: kwargs");
  if (n_rows == nullptr) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: n_rows");
  if (capacity < 0 || (capacity > 0 && logits == nullptr)) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: logits");
  Gil gil;
  PyObject *out = call("step", Py_BuildValue("(OsKL)", (*m)->model, (*kwargs)->text.c_str(),
                                             (unsigned long long)(uintptr_t)logits, (long long)capacity));
  if (out == nullptr) return LLM_ERROR_ABORTED;
  const long long rows = PyLong_AsLongLong(out);
  Py_DECREF(out);
  if (rows < 0) {
    *n_rows = -rows;
    return fail(LLM_ERROR_INSUFFICIENT_BUFFER, "insufficient buffer for the logits");
  }
  *n_rows = rows;
  return 0;
}

int32_t llm_completion_init(llm_completion_t *c) {
  if (c == nullptr) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: c");
  *c = new llm_completion_impl_t();
  return 0;
}

int32_t llm_completion_destroy(llm_completion_t *c) {
  if (c == nullptr) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: c");
  if (*c != nullptr && (*c)->chunks != nullptr && Py_IsInitialized()) {
    Gil gil;
    Py_DECREF((*c)->chunks);
  }
  delete *c;
  *c = nullptr;
  return 0;
}

int32_t llm_completion_get_next_chunk(llm_completion_t *c, llm_json_t *chunk) {
  if (c == nullptr || *c == nullptr || (*c)->chunks == nullptr)
    return fail(LLM_ERROR_INVALID_ARG, "invalid argument: c");
  if (chunk == nullptr || *chunk == nullptr) return fail(LLM_ERROR_INVALID_ARG, "invalid argument: chunk");
  Gil gil;
  PyObject *out = call("next_chunk", Py_BuildValue("(O)", (*c)->chunks));
  if (out == nullptr) return LLM_ERROR_ABORTED;
  if (out == Py_None) {
    Py_DECREF(out);
    return fail(LLM_ERROR_EOF, "the completion has ended");
  }
  const char *text = PyUnicode_AsUTF8(out);
  if (text != nullptr) (*chunk)->text = text;
  Py_DECREF(out);
  return 0;
}

}  // extern "C"

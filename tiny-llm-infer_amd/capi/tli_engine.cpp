// The C ABI of the engine (tli_engine.h): an embedded Python interpreter that drives
// tiny_llm_infer_amd.engine.c_api, which holds the few lines that build an engine from a
// plain dictionary and hand results back as lists.  No model code lives here.
#include "tli_engine.h"

#include <Python.h>
#include <dlfcn.h>
#include <limits.h>
#include <stdlib.h>

#include <string>
#include <vector>

struct tli_engine {
    PyObject* engine = nullptr;                       // the LLMEngine
    std::vector<uint64_t> ids;                        // results of the last step
    std::vector<std::vector<int32_t>> tokens;
};

static thread_local std::string g_error;

extern "C" const char* tli_engine_last_error(void) { return g_error.c_str(); }

static int fail(const std::string& what) {
    g_error = what;
    return 1;
}

// the pending Python exception as text
static int fail_from_python(const char* what) {
    PyObject *type = nullptr, *value = nullptr, *trace = nullptr;
    PyErr_Fetch(&type, &value, &trace);
    PyErr_NormalizeException(&type, &value, &trace);
    std::string text = what;
    if (value) {
        PyObject* s = PyObject_Str(value);
        const char* c = s ? PyUnicode_AsUTF8(s) : nullptr;
        if (c) text += std::string(": ") + c;
        Py_XDECREF(s);
    }
    PyErr_Clear();
    Py_XDECREF(type);
    Py_XDECREF(value);
    Py_XDECREF(trace);
    return fail(text);
}

struct Gil {
    PyGILState_STATE state;
    Gil() : state(PyGILState_Ensure()) {}
    ~Gil() { PyGILState_Release(state); }
};

// Starts the interpreter if this process has none, and puts the folder that holds the package
// (three levels above this library: <root>/tiny-llm-infer_amd/capi/libtli_engine.so) on sys.path.
static int ensure_python() {
    if (!Py_IsInitialized()) {
        Py_InitializeEx(0);
        PyEval_SaveThread();                          // from here on every entry takes the GIL itself
    }
    Gil gil;
    Dl_info info;
    if (!dladdr((const void*)&tli_engine_last_error, &info) || !info.dli_fname)
        return fail("cannot find the place of libtli_engine.so");
    char resolved[4096];
    std::string root = realpath(info.dli_fname, resolved) ? resolved : info.dli_fname;
    for (int up = 0; up < 3; ++up) {
        const size_t slash = root.find_last_of('/');
        if (slash == std::string::npos) return fail("libtli_engine.so is not inside the package tree");
        root.erase(slash);
    }
    PyObject* path = PySys_GetObject("path");         // borrowed
    PyObject* entry = PyUnicode_FromString(root.c_str());
    if (!path || !entry) return fail_from_python("sys.path");
    int have = PySequence_Contains(path, entry);
    if (have == 0) have = PyList_Insert(path, 0, entry) == 0 ? 1 : -1;
    Py_DECREF(entry);
    return have < 0 ? fail_from_python("sys.path") : 0;
}

static PyObject* helper(const char* name) {
    PyObject* module = PyImport_ImportModule("tiny_llm_infer_amd.engine.c_api");
    if (!module) return nullptr;
    PyObject* fn = PyObject_GetAttrString(module, name);
    Py_DECREF(module);
    return fn;
}

static void put(PyObject* dict, const char* key, PyObject* value) {   // steals value
    if (value) {
        PyDict_SetItemString(dict, key, value);
        Py_DECREF(value);
    }
}

extern "C" void tli_engine_default_config(tli_engine_config* c) {
    if (!c) return;
    *c = tli_engine_config{};
    c->dtype = "bfloat16";
    c->max_model_len = 2048;
    c->page_size = 16;
    c->max_num_seqs = 16;
    c->max_num_batched_tokens = 256;
    c->gpu_memory_utilization = 0.9f;
}

extern "C" void tli_engine_default_sampling(tli_sampling_params* s) {
    if (!s) return;
    *s = tli_sampling_params{};
    s->max_tokens = 64;
    s->top_p = 1.0f;
}

extern "C" int tli_engine_create(const tli_engine_config* c, tli_engine** out) {
    if (!c || !out) return fail("tli_engine_create: no configuration or no place for the engine");
    *out = nullptr;
    if ((c->model_dir != nullptr) == (c->config_json != nullptr))
        return fail("tli_engine_create: give model_dir, or config_json for random weights");
    if (ensure_python()) return 1;
    Gil gil;
    PyObject* fn = helper("create");
    if (!fn) return fail_from_python("tli_engine_create: cannot import the package");
    PyObject* d = PyDict_New();
    if (c->model_dir) put(d, "model_dir", PyUnicode_FromString(c->model_dir));
    if (c->config_json) put(d, "config_json", PyUnicode_FromString(c->config_json));
    put(d, "weights_seed", PyLong_FromUnsignedLongLong(c->weights_seed));
    put(d, "dtype", PyUnicode_FromString(c->dtype ? c->dtype : "bfloat16"));
    put(d, "max_model_len", PyLong_FromLong(c->max_model_len));
    put(d, "page_size", PyLong_FromLong(c->page_size));
    put(d, "num_kv_blocks", PyLong_FromLong(c->num_kv_blocks));
    put(d, "max_num_seqs", PyLong_FromLong(c->max_num_seqs));
    put(d, "max_num_batched_tokens", PyLong_FromLong(c->max_num_batched_tokens));
    put(d, "gpu_memory_utilization", PyFloat_FromDouble(c->gpu_memory_utilization));
    put(d, "enable_prefix_caching", PyBool_FromLong(c->enable_prefix_caching));
    PyObject* engine = PyObject_CallFunctionObjArgs(fn, d, nullptr);
    Py_DECREF(fn);
    Py_DECREF(d);
    if (!engine) return fail_from_python("tli_engine_create");
    tli_engine* e = new tli_engine;
    e->engine = engine;
    *out = e;
    return 0;
}

extern "C" void tli_engine_destroy(tli_engine* e) {
    if (!e) return;
    if (Py_IsInitialized()) {
        Gil gil;
        Py_XDECREF(e->engine);
    }
    delete e;
}

extern "C" int tli_engine_add_request(tli_engine* e, const int32_t* prompt, int n, const tli_sampling_params* s,
                                      uint64_t* request_id) {
    if (!e || !e->engine) return fail("tli_engine_add_request: no engine");
    if (n < 0 || (n > 0 && !prompt)) return fail("tli_engine_add_request: no prompt tokens");
    tli_sampling_params dflt;
    tli_engine_default_sampling(&dflt);
    if (!s) s = &dflt;
    Gil gil;
    PyObject* fn = helper("add_request");
    if (!fn) return fail_from_python("tli_engine_add_request");
    PyObject* tokens = PyList_New(n);
    for (int i = 0; i < n; ++i) PyList_SET_ITEM(tokens, i, PyLong_FromLong(prompt[i]));
    PyObject* d = PyDict_New();
    put(d, "max_tokens", PyLong_FromLong(s->max_tokens));
    put(d, "temperature", PyFloat_FromDouble(s->temperature));
    put(d, "top_p", PyFloat_FromDouble(s->top_p));
    put(d, "ignore_eos", PyBool_FromLong(s->ignore_eos));
    put(d, "seed", PyLong_FromUnsignedLongLong(s->seed));
    PyObject* id = PyObject_CallFunctionObjArgs(fn, e->engine, tokens, d, nullptr);
    Py_DECREF(fn);
    Py_DECREF(tokens);
    Py_DECREF(d);
    if (!id) return fail_from_python("tli_engine_add_request");
    if (request_id) *request_id = PyLong_AsUnsignedLongLong(id);
    Py_DECREF(id);
    return 0;
}

extern "C" int tli_engine_step(tli_engine* e, int* num_finished) {
    if (!e || !e->engine) return fail("tli_engine_step: no engine");
    Gil gil;
    PyObject* fn = helper("step");
    if (!fn) return fail_from_python("tli_engine_step");
    PyObject* done = PyObject_CallFunctionObjArgs(fn, e->engine, nullptr);     // [(request id, [tokens]), ...]
    Py_DECREF(fn);
    if (!done) return fail_from_python("tli_engine_step");
    e->ids.clear();
    e->tokens.clear();
    const Py_ssize_t count = PyList_Size(done);
    for (Py_ssize_t i = 0; i < count; ++i) {
        PyObject* pair = PyList_GetItem(done, i);                               // borrowed
        e->ids.push_back(PyLong_AsUnsignedLongLong(PyTuple_GetItem(pair, 0)));
        PyObject* toks = PyTuple_GetItem(pair, 1);
        std::vector<int32_t> v((size_t)PyList_Size(toks));
        for (size_t t = 0; t < v.size(); ++t) v[t] = (int32_t)PyLong_AsLong(PyList_GetItem(toks, (Py_ssize_t)t));
        e->tokens.push_back(std::move(v));
    }
    Py_DECREF(done);
    if (PyErr_Occurred()) return fail_from_python("tli_engine_step: results");
    if (num_finished) *num_finished = (int)e->ids.size();
    return 0;
}

extern "C" int tli_engine_result(tli_engine* e, int index, uint64_t* request_id, const int32_t** token_ids, int* n) {
    if (!e) return fail("tli_engine_result: no engine");
    if (index < 0 || (size_t)index >= e->ids.size())
        return fail("tli_engine_result: the last step finished " + std::to_string(e->ids.size()) + " requests");
    if (request_id) *request_id = e->ids[(size_t)index];
    if (token_ids) *token_ids = e->tokens[(size_t)index].data();
    if (n) *n = (int)e->tokens[(size_t)index].size();
    return 0;
}

static long long number(tli_engine* e, const char* name) {
    if (!e || !e->engine) return -1;
    Gil gil;
    PyObject* fn = helper(name);
    if (!fn) { fail_from_python(name); return -1; }
    PyObject* v = PyObject_CallFunctionObjArgs(fn, e->engine, nullptr);
    Py_DECREF(fn);
    if (!v) { fail_from_python(name); return -1; }
    const long long out = PyLong_AsLongLong(v);
    Py_DECREF(v);
    return out;
}

extern "C" int tli_engine_is_finished(tli_engine* e) { return number(e, "is_finished") != 0; }

extern "C" uint64_t tli_engine_total_generated_tokens(tli_engine* e) {
    const long long v = number(e, "total_generated_tokens");
    return v < 0 ? 0 : (uint64_t)v;
}

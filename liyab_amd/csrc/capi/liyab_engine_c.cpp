// The C library over the engine: forwards to `liyab_amd.capi` in a Python interpreter inside
// the process (see liyab_engine_c.h). Everything that touches Python holds the interpreter's lock.
#include "liyab_engine_c.h"

#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <dlfcn.h>

#include <mutex>
#include <string>

namespace {

thread_local std::string g_error;
std::mutex g_init_mutex;
bool g_started_here = false;   // this library started the interpreter (and released its lock afterwards)
PyObject* g_module = nullptr;  // liyab_amd.capi

liyab_status fail(liyab_status s, const std::string& msg) {
    g_error = msg;
    return s;
}

// The folder that holds the `liyab_amd` package: this library lives in <root>/liyab_amd/_lib/.
std::string tree_root() {
    Dl_info info;
    if (dladdr(reinterpret_cast<const void*>(&tree_root), &info) == 0 || info.dli_fname == nullptr) return "";
    std::string p(info.dli_fname);
    for (int up = 0; up < 3; ++up) {
        const size_t cut = p.find_last_of('/');
        if (cut == std::string::npos) return "";
        p.erase(cut);
    }
    return p;
}

// The pending Python exception as (status, "Type: message"); clears it.
liyab_status take_python_error(const char* what) {
    PyObject *type = nullptr, *value = nullptr, *trace = nullptr;
    PyErr_Fetch(&type, &value, &trace);
    PyErr_NormalizeException(&type, &value, &trace);
    std::string name = "error", text;
    if (type != nullptr) {
        if (PyObject* n = PyObject_GetAttrString(type, "__name__")) {
            if (const char* c = PyUnicode_AsUTF8(n)) name = c;
            Py_DECREF(n);
        }
    }
    if (value != nullptr) {
        if (PyObject* s = PyObject_Str(value)) {
            if (const char* c = PyUnicode_AsUTF8(s)) text = c;
            Py_DECREF(s);
        }
    }
    PyErr_Clear();
    Py_XDECREF(type);
    Py_XDECREF(value);
    Py_XDECREF(trace);
    liyab_status st = LIYAB_INTERNAL;
    if (name == "InvalidArgument") st = LIYAB_INVALID_ARGUMENT;
    else if (name == "InvalidModel") st = LIYAB_INVALID_MODEL;
    else if (name == "Unsupported") st = LIYAB_UNSUPPORTED;
    else if (name == "OutOfPages") st = LIYAB_OUT_OF_MEMORY;
    else if (name == "ContextFull") st = LIYAB_CONTEXT_FULL;
    else if (name == "Busy") st = LIYAB_BUSY;
    return fail(st, std::string(what) + ": " + name + ": " + text);
}

// Holds the interpreter's lock for a scope; starts the interpreter at first use.
class Python {
public:
    Python() {
        {
            std::lock_guard<std::mutex> lock(g_init_mutex);
            if (!Py_IsInitialized()) {
                Py_InitializeEx(0);  // no signal handlers: the host program keeps its own
                g_started_here = true;
                PyEval_SaveThread();  // give the lock up: every call takes it for itself below
            }
        }
        state_ = PyGILState_Ensure();
    }
    ~Python() { PyGILState_Release(state_); }
    Python(const Python&) = delete;
    Python& operator=(const Python&) = delete;

private:
    PyGILState_STATE state_;
};

// liyab_amd.capi, imported once (the caller holds the lock).
PyObject* module() {
    if (g_module != nullptr) return g_module;
    const std::string root = tree_root();
    if (!root.empty()) {
        PyObject* path = PySys_GetObject("path");  // borrowed
        PyObject* entry = PyUnicode_FromString(root.c_str());
        if (path != nullptr && entry != nullptr && PySequence_Contains(path, entry) == 0) PyList_Insert(path, 0, entry);
        Py_XDECREF(entry);
    }
    g_module = PyImport_ImportModule("liyab_amd.capi");
    return g_module;
}

}  // namespace

struct liyab_engine {
    PyObject* engine;  // liyab_amd.Engine
};

extern "C" {

const char* liyab_engine_last_error(void) { return g_error.c_str(); }

void liyab_engine_config_default(liyab_engine_config* c) {
    if (c == nullptr) return;
    c->model_path = nullptr;
    c->dtype = "bfloat16";
    c->context_length = 0;
    c->page_size = 16;
    c->num_pages = 0;
    c->max_sequences = 8;
    c->max_batched_tokens = 2048;
    c->prefill_chunk = 256;  // the reference's portion of a prompt (src/core/engine.cpp:2863-2864)
    c->batch_invariant = 0;
}

void liyab_sampling_params_default(liyab_sampling_params* p) {
    if (p == nullptr) return;
    // the reference's defaults (include/liyab/types.h:215-222)
    p->temperature = 0.8f;
    p->top_k = 40;
    p->top_p = 0.95f;
    p->seed = 0;
    p->max_tokens = 256;
}

liyab_status liyab_engine_create(const liyab_engine_config* config, liyab_engine** out_engine) {
    if (config == nullptr || out_engine == nullptr) return fail(LIYAB_INVALID_ARGUMENT, "engine_create: null argument");
    if (config->model_path == nullptr) return fail(LIYAB_INVALID_ARGUMENT, "engine_create: no model path");
    *out_engine = nullptr;
    Python py;
    PyObject* mod = module();
    if (mod == nullptr) return take_python_error("engine_create: importing liyab_amd.capi");
    PyObject* engine = PyObject_CallMethod(mod, "create", "ssiiiiiii", config->model_path,
                                           config->dtype != nullptr ? config->dtype : "bfloat16", config->context_length,
                                           config->page_size, config->num_pages, config->max_sequences,
                                           config->max_batched_tokens, config->prefill_chunk, config->batch_invariant);
    if (engine == nullptr) return take_python_error("engine_create");
    *out_engine = new liyab_engine{engine};
    return LIYAB_OK;
}

void liyab_engine_destroy(liyab_engine* engine) {
    if (engine == nullptr) return;
    {
        Python py;
        Py_XDECREF(engine->engine);
    }
    delete engine;
}

liyab_status liyab_engine_generate_tokens(liyab_engine* engine, const int32_t* tokens, size_t n_tokens,
                                          const liyab_sampling_params* params, liyab_token_callback callback, void* user_data,
                                          int32_t* out, size_t capacity, size_t* n_out, liyab_generation_stats* stats) {
    if (engine == nullptr || engine->engine == nullptr) return fail(LIYAB_INVALID_ARGUMENT, "generate_tokens: no engine");
    if (tokens == nullptr && n_tokens > 0) return fail(LIYAB_INVALID_ARGUMENT, "generate_tokens: null prompt");
    if (out == nullptr && capacity > 0) return fail(LIYAB_INVALID_ARGUMENT, "generate_tokens: null output with a capacity");
    liyab_sampling_params p;
    if (params != nullptr) p = *params;
    else liyab_sampling_params_default(&p);
    if (n_out != nullptr) *n_out = 0;
    Python py;
    PyObject* mod = module();
    if (mod == nullptr) return take_python_error("generate_tokens: importing liyab_amd.capi");
    // the prompt as bytes of int32; the callback and its argument as addresses (the module calls it through ctypes)
    PyObject* result = PyObject_CallMethod(
        mod, "generate", "Oy#fifKiKK", engine->engine, reinterpret_cast<const char*>(tokens),
        static_cast<Py_ssize_t>(n_tokens * sizeof(int32_t)), static_cast<double>(p.temperature), static_cast<int>(p.top_k),
        static_cast<double>(p.top_p), static_cast<unsigned long long>(p.seed), static_cast<int>(p.max_tokens),
        static_cast<unsigned long long>(reinterpret_cast<uintptr_t>(callback)),
        static_cast<unsigned long long>(reinterpret_cast<uintptr_t>(user_data)));
    if (result == nullptr) return take_python_error("generate_tokens");
    // (tokens as bytes of int32, prompt_tokens, prefill_ms, ttft_ms, decode_ms, tokens_per_second, kv_cache_bytes, preemptions, cancelled)
    const char* data = nullptr;
    Py_ssize_t size = 0;
    int prompt_tokens = 0, preemptions = 0, cancelled = 0;
    double prefill_ms = 0, ttft_ms = 0, decode_ms = 0, tps = 0;
    long long kv_bytes = 0;
    if (!PyArg_ParseTuple(result, "y#iddddLii", &data, &size, &prompt_tokens, &prefill_ms, &ttft_ms, &decode_ms, &tps, &kv_bytes,
                          &preemptions, &cancelled)) {
        Py_DECREF(result);
        return take_python_error("generate_tokens: reading the result");
    }
    const size_t n = static_cast<size_t>(size) / sizeof(int32_t);
    const int32_t* ids = reinterpret_cast<const int32_t*>(data);
    for (size_t i = 0; i < n && i < capacity; ++i) out[i] = ids[i];
    if (n_out != nullptr) *n_out = n;
    if (stats != nullptr) {
        stats->prompt_tokens = prompt_tokens;
        stats->generated_tokens = static_cast<int32_t>(n);
        stats->prefill_ms = prefill_ms;
        stats->ttft_ms = ttft_ms;
        stats->decode_ms = decode_ms;
        stats->tokens_per_second = tps;
        stats->kv_cache_bytes = kv_bytes;
        stats->preemptions = preemptions;
        stats->cancelled = cancelled;
    }
    Py_DECREF(result);
    return LIYAB_OK;
}

}  // extern "C"

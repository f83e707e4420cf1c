// The plain C interface of include/tuff_amd.h.
//
// Every entry point takes the interpreter lock, calls one function of the package's
// tuff_amd.capi module with integers (the handle, addresses of the caller's arrays, counts)
// and turns a Python exception into a negative return code plus a message for
// tuff_last_error().  The interpreter is the calling process's own if it has one; otherwise it
// is started at the first call, with the package's folder (found from this library's own
// path, or $TUFF_AMD_ROOT) on its module path.
#define PY_SSIZE_T_CLEAN
#include <Python.h>

#include <dlfcn.h>
#include <unistd.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>

#include "../../include/tuff_amd.h"

#define TUFF_API extern "C" __attribute__((visibility("default")))

struct tuff_engine {
    long long handle;   // key of the session in tuff_amd.capi
};

namespace {

thread_local std::string last_error;
std::mutex start_mutex;
bool started = false;          // bridge imported and checked
bool owns_interpreter = false;
PyThreadState* main_thread = nullptr;
PyObject* bridge = nullptr;    // module tuff_amd.capi

void set_error(const char* fmt, ...) {
    char buf[2048];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    last_error = buf;
}

// The pending Python exception as "Type: message"; clears it.
void take_python_error(const char* where) {
    PyObject *type = nullptr, *value = nullptr, *tb = nullptr;
    PyErr_Fetch(&type, &value, &tb);
    PyErr_NormalizeException(&type, &value, &tb);
    std::string msg = where;
    msg += ": ";
    if (type) {
        PyObject* name = PyObject_GetAttrString(type, "__name__");
        const char* s = name ? PyUnicode_AsUTF8(name) : nullptr;
        msg += s ? s : "error";
        Py_XDECREF(name);
    }
    if (value) {
        PyObject* str = PyObject_Str(value);
        const char* s = str ? PyUnicode_AsUTF8(str) : nullptr;
        if (s && *s) { msg += ": "; msg += s; }
        Py_XDECREF(str);
    }
    PyErr_Clear();
    Py_XDECREF(type); Py_XDECREF(value); Py_XDECREF(tb);
    last_error = msg;
}

// Folder that holds the tuff_amd package: $TUFF_AMD_ROOT, else the one this library was built
// into (<root>/tuff_amd/csrc/_lib/libtuff_amd.so).  Empty if neither holds the package.
std::string package_root() {
    auto holds = [](const std::string& root) {
        return !root.empty() && access((root + "/tuff_amd/__init__.py").c_str(), R_OK) == 0;
    };
    if (const char* env = getenv("TUFF_AMD_ROOT")) {
        if (holds(env)) return env;
    }
    Dl_info info;
    if (dladdr(reinterpret_cast<void*>(&package_root), &info) && info.dli_fname) {
        char resolved[4096];
        if (realpath(info.dli_fname, resolved)) {
            std::string p = resolved;
            for (int up = 0; up < 4; ++up) {
                size_t cut = p.rfind('/');
                if (cut == std::string::npos) return "";
                p.erase(cut);
            }
            if (holds(p)) return p;
        }
    }
    return "";
}

// Called with the interpreter lock held.
bool import_bridge() {
    std::string root = package_root();
    if (!root.empty()) {
        PyObject* path = PySys_GetObject("path");               // borrowed
        PyObject* entry = PyUnicode_FromString(root.c_str());
        if (path && entry && !PySequence_Contains(path, entry)) PyList_Insert(path, 0, entry);
        Py_XDECREF(entry);
    }
    bridge = PyImport_ImportModule("tuff_amd.capi");
    if (!bridge) {
        take_python_error("import tuff_amd.capi");
        if (root.empty()) last_error += " (the package was not found beside the library; set TUFF_AMD_ROOT)";
        return false;
    }
    PyObject* sizes = PyObject_CallMethod(bridge, "struct_sizes", nullptr);
    long a = 0, b = 0, c = 0;
    if (!sizes || !PyArg_ParseTuple(sizes, "lll", &a, &b, &c)) {
        take_python_error("tuff_amd.capi.struct_sizes");
        Py_XDECREF(sizes);
        return false;
    }
    Py_DECREF(sizes);
    if (a != (long)sizeof(tuff_sampling) || b != (long)sizeof(tuff_step_entry) || c != (long)sizeof(tuff_event)) {
        set_error("the header and tuff_amd/capi.py lay the structures out differently "
                  "(%zu/%zu/%zu bytes here, %ld/%ld/%ld there)",
                  sizeof(tuff_sampling), sizeof(tuff_step_entry), sizeof(tuff_event), a, b, c);
        return false;
    }
    return true;
}

// Takes the interpreter lock for one call; starts the interpreter and imports the bridge first
// if that has not happened yet.
class Call {
public:
    Call() {
        {
            std::lock_guard<std::mutex> lock(start_mutex);
            if (!Py_IsInitialized()) {
                Py_InitializeEx(0);                 // no signal handlers: the host program keeps its own
                owns_interpreter = true;
                main_thread = PyEval_SaveThread();  // give the lock up; every call takes it by itself
            }
        }
        gil_ = PyGILState_Ensure();
        last_error.clear();
        if (!started) started = import_bridge();    // under the interpreter lock, which orders it
        ok_ = started;
    }
    ~Call() { PyGILState_Release(gil_); }
    bool ok() const { return ok_; }

    // Calls tuff_amd.capi.<name>(*args built from fmt) and returns a new reference, or null with
    // last_error set.
    PyObject* call(const char* name, const char* fmt, ...) {
        PyObject* fn = PyObject_GetAttrString(bridge, name);
        if (!fn) { take_python_error(name); return nullptr; }
        va_list ap;
        va_start(ap, fmt);
        PyObject* args = Py_VaBuildValue(fmt, ap);
        va_end(ap);
        PyObject* res = nullptr;
        if (args) {
            res = PyObject_CallObject(fn, args);
            Py_DECREF(args);
        }
        Py_DECREF(fn);
        if (!res) take_python_error(name);
        return res;
    }

private:
    PyGILState_STATE gil_;
    bool ok_ = false;
};

int done(PyObject* res) {
    if (!res) return -1;
    Py_DECREF(res);
    return 0;
}

// The result as an int, or -1 with last_error set.
int as_int(PyObject* res) {
    if (!res) return -1;
    long v = PyLong_AsLong(res);
    Py_DECREF(res);
    if (v == -1 && PyErr_Occurred()) { take_python_error("result"); return -1; }
    return (int)v;
}

bool have(const void* p, const char* what) {
    if (p) return true;
    set_error("%s is null", what);
    return false;
}

}  // namespace

TUFF_API const char* tuff_last_error(void) { return last_error.c_str(); }

// The defaults of tuff_amd/sampling/params.py (the reference's, include/sampler.h:12-20), kept
// here so that asking for them does not start the interpreter.
TUFF_API void tuff_sampling_default(tuff_sampling* s) {
    if (!s) return;
    memset(s, 0, sizeof *s);
    s->temp = 0.0f;
    s->top_p = 1.0f;
    s->top_k = 0;
    s->min_p = 0.0f;
    s->repeat_penalty = 1.0f;
    s->repeat_last_n = 64;
    s->seed = 0;
    s->max_new_tokens = 128;
    s->ignore_eos = 0;
}

TUFF_API int tuff_model_write_random(const char* config_json, uint64_t seed, const char* out_dir,
                                     const char* stored_dtype) {
    if (!have(config_json, "config_json") || !have(out_dir, "out_dir") || !have(stored_dtype, "stored_dtype"))
        return -1;
    Call c;
    if (!c.ok()) return -1;
    return done(c.call("write_random", "(sKss)", config_json, (unsigned long long)seed, out_dir, stored_dtype));
}

TUFF_API int tuff_engine_open(tuff_engine** out, const char* model_dir, const char* dtype, int max_requests,
                              int ctx_size) {
    if (!have(out, "out") || !have(model_dir, "model_dir") || !have(dtype, "dtype")) return -1;
    *out = nullptr;
    Call c;
    if (!c.ok()) return -1;
    PyObject* r = c.call("open_engine", "(ssii)", model_dir, dtype, max_requests, ctx_size);
    if (!r) return -1;
    long long h = PyLong_AsLongLong(r);
    Py_DECREF(r);
    *out = new tuff_engine{h};
    return 0;
}

TUFF_API void tuff_engine_close(tuff_engine* eng) {
    if (!eng) return;
    {
        Call c;
        if (c.ok()) Py_XDECREF(c.call("close_engine", "(L)", eng->handle));
    }
    delete eng;
}

static int engine_info(const tuff_engine* eng, const char* what) {
    if (!have(eng, "eng")) return -2;
    Call c;
    if (!c.ok()) return -2;
    PyObject* r = c.call("info", "(Ls)", eng->handle, what);
    if (!r) return -2;
    return as_int(r);
}

TUFF_API int tuff_engine_vocab_size(const tuff_engine* eng) { return engine_info(eng, "vocab_size"); }
TUFF_API int tuff_engine_ctx_size(const tuff_engine* eng) { return engine_info(eng, "ctx_size"); }
TUFF_API int tuff_engine_eos_token(const tuff_engine* eng) { return engine_info(eng, "eos_token"); }

TUFF_API int tuff_request_begin(tuff_engine* eng, int64_t request) {
    if (!have(eng, "eng")) return -1;
    Call c;
    if (!c.ok()) return -1;
    return done(c.call("request_begin", "(LL)", eng->handle, (long long)request));
}

TUFF_API int tuff_request_end(tuff_engine* eng, int64_t request) {
    if (!have(eng, "eng")) return -1;
    Call c;
    if (!c.ok()) return -1;
    return done(c.call("request_end", "(LL)", eng->handle, (long long)request));
}

TUFF_API int tuff_request_length(const tuff_engine* eng, int64_t request) {
    if (!have(eng, "eng")) return -1;
    Call c;
    if (!c.ok()) return -1;
    return as_int(c.call("request_length", "(LL)", eng->handle, (long long)request));
}

TUFF_API int tuff_engine_step(tuff_engine* eng, const tuff_step_entry* entries, int n_entries, float* logits_out,
                              size_t rows_capacity) {
    if (!have(eng, "eng") || !have(entries, "entries")) return -1;
    Call c;
    if (!c.ok()) return -1;
    return done(c.call("engine_step", "(LKiKK)", eng->handle, (unsigned long long)(uintptr_t)entries, n_entries,
                       (unsigned long long)(uintptr_t)logits_out, (unsigned long long)rows_capacity));
}

TUFF_API int tuff_request_add(tuff_engine* eng, int64_t request, const int32_t* prompt, int n_prompt,
                              const tuff_sampling* s) {
    if (!have(eng, "eng") || !have(prompt, "prompt")) return -1;
    Call c;
    if (!c.ok()) return -1;
    return done(c.call("request_add", "(LLKiK)", eng->handle, (long long)request,
                       (unsigned long long)(uintptr_t)prompt, n_prompt, (unsigned long long)(uintptr_t)s));
}

TUFF_API int tuff_request_abort(tuff_engine* eng, int64_t request) {
    if (!have(eng, "eng")) return -1;
    Call c;
    if (!c.ok()) return -1;
    return done(c.call("request_abort", "(LL)", eng->handle, (long long)request));
}

TUFF_API int tuff_sched_step(tuff_engine* eng, tuff_event* events, int events_capacity, int* n_events) {
    if (!have(eng, "eng") || !have(n_events, "n_events")) return -1;
    if (events_capacity > 0 && !have(events, "events")) return -1;
    *n_events = 0;
    Call c;
    if (!c.ok()) return -1;
    PyObject* r = c.call("sched_step", "(LKi)", eng->handle, (unsigned long long)(uintptr_t)events, events_capacity);
    if (!r) return -1;
    int written = 0, left = 0;
    if (!PyArg_ParseTuple(r, "ii", &written, &left)) {
        take_python_error("sched_step");
        Py_DECREF(r);
        return -1;
    }
    Py_DECREF(r);
    *n_events = written;
    return left;
}

TUFF_API int tuff_generate(tuff_engine* eng, const int32_t* prompt, int n_prompt, const tuff_sampling* s,
                           int32_t* out, int out_capacity, int* n_out) {
    if (!have(eng, "eng") || !have(prompt, "prompt") || !have(n_out, "n_out")) return -1;
    if (out_capacity > 0 && !have(out, "out")) return -1;
    *n_out = 0;
    Call c;
    if (!c.ok()) return -1;
    int n = as_int(c.call("generate", "(LKiKKi)", eng->handle, (unsigned long long)(uintptr_t)prompt, n_prompt,
                          (unsigned long long)(uintptr_t)s, (unsigned long long)(uintptr_t)out, out_capacity));
    if (n < 0) return -1;
    *n_out = n;
    return 0;
}

TUFF_API void tuff_shutdown(void) {
    std::lock_guard<std::mutex> lock(start_mutex);
    if (!owns_interpreter || !Py_IsInitialized()) return;
    PyEval_RestoreThread(main_thread);
    Py_CLEAR(bridge);
    started = false;
    Py_FinalizeEx();
    owns_interpreter = false;
}

// The engine's C interface (tffinfer_engine.h) over the package's Python engine: an embedded
// interpreter, one module of plain functions (tffinfer_amd/capi_bridge.py), and copies between
// the caller's buffers and Python bytes.  No model code, cache or scheduling lives here.
#define _GNU_SOURCE
#define PY_SSIZE_T_CLEAN
#include <Python.h>
#include <dlfcn.h>
#include <libgen.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define TFF_ENGINE_BUILD
#include "tffinfer_engine.h"

struct tff_engine {
    PyObject* handle;      // capi_bridge.Handle
    int vocab;
};

static __thread char last_error[4096];
static PyObject* bridge;           // the module, once imported
static int started_here;           // this library started the interpreter (it is never finalised: what it has loaded holds GPU state until the process ends)

static void set_error(const char* what) {
    snprintf(last_error, sizeof last_error, "%s", what);
}

// The pending Python exception as "Type: message"; clears it.
static void take_python_error(const char* where) {
    PyObject *type = NULL, *value = NULL, *trace = NULL;
    PyErr_Fetch(&type, &value, &trace);
    PyErr_NormalizeException(&type, &value, &trace);
    const char* tname = type ? ((PyTypeObject*)type)->tp_name : "error";
    PyObject* text = value ? PyObject_Str(value) : NULL;
    const char* msg = text ? PyUnicode_AsUTF8(text) : NULL;
    snprintf(last_error, sizeof last_error, "%s: %s: %s", where, tname, msg ? msg : "(no message)");
    PyErr_Clear();
    Py_XDECREF(text);
    Py_XDECREF(type);
    Py_XDECREF(value);
    Py_XDECREF(trace);
}

// The folder that holds the package: this library lies in <root>/tffinfer_amd/lib/.
static int package_root(char* out, size_t n) {
    Dl_info info;
    if (!dladdr((void*)&package_root, &info) || !info.dli_fname) return -1;
    char* real = realpath(info.dli_fname, NULL);
    if (!real) return -1;
    char* d = dirname(real);            // .../tffinfer_amd/lib
    d = dirname(d);                     // .../tffinfer_amd
    d = dirname(d);                     // the root
    snprintf(out, n, "%s", d);
    free(real);
    return 0;
}

// Starts the interpreter if the process has none.  Returns with the interpreter's lock *not* held.
static int ensure_interpreter(void) {
    if (!Py_IsInitialized()) {
        Py_InitializeEx(0);             // no signal handlers: the host program keeps its own
        if (!Py_IsInitialized()) {
            set_error("the Python interpreter could not be started");
            return -1;
        }
        started_here = 1;
        PyEval_SaveThread();            // give up the lock; every call below takes it for itself
    }
    return 0;
}

// With the lock held: the bridge module, imported on first use.
static PyObject* get_bridge(void) {
    if (bridge) return bridge;
    PyObject* mod = PyImport_ImportModule("tffinfer_amd.capi_bridge");
    if (!mod) {
        // not on the interpreter's path: add the folder this library was built in
        PyErr_Clear();
        char root[2048];
        if (package_root(root, sizeof root) == 0) {
            PyObject* path = PySys_GetObject("path");     // borrowed
            PyObject* s = PyUnicode_FromString(root);
            if (path && s) PyList_Insert(path, 0, s);
            Py_XDECREF(s);
            mod = PyImport_ImportModule("tffinfer_amd.capi_bridge");
        }
    }
    if (!mod) {
        take_python_error("import tffinfer_amd.capi_bridge");
        return NULL;
    }
    bridge = mod;
    return bridge;
}

#define ENTER(fail)                                  \
    last_error[0] = 0;                               \
    if (ensure_interpreter() != 0) return fail;      \
    PyGILState_STATE gil_ = PyGILState_Ensure();     \
    PyObject* mod_ = get_bridge();                   \
    if (!mod_) {                                     \
        PyGILState_Release(gil_);                    \
        return fail;                                 \
    }
#define LEAVE(value)                                 \
    {                                                \
        PyGILState_Release(gil_);                    \
        return value;                                \
    }

static tff_engine* wrap(PyObject* handle, PyObject* mod) {
    tff_engine* e = (tff_engine*)calloc(1, sizeof *e);
    if (!e) {
        Py_DECREF(handle);
        set_error("out of memory");
        return NULL;
    }
    e->handle = handle;
    PyObject* v = PyObject_CallMethod(mod, "vocab_size", "O", handle);
    if (!v) {
        take_python_error("engine_create");
        Py_DECREF(handle);
        free(e);
        return NULL;
    }
    e->vocab = (int)PyLong_AsLong(v);
    Py_DECREF(v);
    return e;
}

TFF_ENGINE_API tff_engine* engine_create(const char* model_dir, const char* options_json) {
    if (!model_dir) {
        set_error("engine_create: no model folder");
        return NULL;
    }
    ENTER(NULL)
    PyObject* h = PyObject_CallMethod(mod_, "create", "ss", model_dir, options_json ? options_json : "");
    if (!h) {
        take_python_error("engine_create");
        LEAVE(NULL)
    }
    tff_engine* e = wrap(h, mod_);
    LEAVE(e)
}

TFF_ENGINE_API tff_engine* engine_create_random(const char* config_json_file, uint64_t seed, const char* options_json) {
    if (!config_json_file) {
        set_error("engine_create_random: no configuration file");
        return NULL;
    }
    ENTER(NULL)
    PyObject* h = PyObject_CallMethod(mod_, "create_random", "sKs", config_json_file, (unsigned long long)seed,
                                      options_json ? options_json : "");
    if (!h) {
        take_python_error("engine_create_random");
        LEAVE(NULL)
    }
    tff_engine* e = wrap(h, mod_);
    LEAVE(e)
}

TFF_ENGINE_API void engine_destroy(tff_engine* e) {
    if (!e) return;
    last_error[0] = 0;
    if (Py_IsInitialized()) {
        PyGILState_STATE g = PyGILState_Ensure();
        if (bridge) {
            PyObject* r = PyObject_CallMethod(bridge, "destroy", "O", e->handle);
            if (!r) take_python_error("engine_destroy");
            Py_XDECREF(r);
        }
        Py_DECREF(e->handle);
        PyGILState_Release(g);
    }
    free(e);
}

TFF_ENGINE_API int engine_vocab_size(tff_engine* e) {
    if (!e) {
        set_error("engine_vocab_size: no engine");
        return -1;
    }
    return e->vocab;
}

TFF_ENGINE_API int64_t engine_add_request(tff_engine* e, const int32_t* token_ids, int32_t n, const char* params_json) {
    if (!e || !token_ids || n <= 0) {
        set_error("engine_add_request: an engine and at least one token are needed");
        return -1;
    }
    ENTER(-1)
    PyObject* r = PyObject_CallMethod(mod_, "add_request", "Oy#s", e->handle, (const char*)token_ids,
                                      (Py_ssize_t)n * 4, params_json ? params_json : "");
    if (!r) {
        take_python_error("engine_add_request");
        LEAVE(-1)
    }
    const int64_t id = (int64_t)PyLong_AsLongLong(r);
    Py_DECREF(r);
    LEAVE(id)
}

TFF_ENGINE_API int engine_step(tff_engine* e, tff_step_event* events, int capacity) {
    if (!e || !events || capacity <= 0) {
        set_error("engine_step: an engine and room for at least one event are needed");
        return -1;
    }
    ENTER(-1)
    PyObject* r = PyObject_CallMethod(mod_, "step", "Oi", e->handle, capacity);
    if (!r) {
        take_python_error("engine_step");
        LEAVE(-1)
    }
    char* data = NULL;
    Py_ssize_t len = 0;
    if (PyBytes_AsStringAndSize(r, &data, &len) != 0 || len % (Py_ssize_t)sizeof(tff_step_event) != 0 ||
        len / (Py_ssize_t)sizeof(tff_step_event) > capacity) {
        PyErr_Clear();
        Py_DECREF(r);
        set_error("engine_step: malformed events");
        LEAVE(-1)
    }
    memcpy(events, data, (size_t)len);
    Py_DECREF(r);
    LEAVE((int)(len / (Py_ssize_t)sizeof(tff_step_event)))
}

static int call_int(tff_engine* e, const char* name, int with_id, int64_t id) {
    if (!e) {
        snprintf(last_error, sizeof last_error, "engine_%s: no engine", name);
        return -1;
    }
    ENTER(-1)
    PyObject* r = with_id ? PyObject_CallMethod(mod_, name, "OL", e->handle, (long long)id)
                          : PyObject_CallMethod(mod_, name, "O", e->handle);
    if (!r) {
        char where[64];
        snprintf(where, sizeof where, "engine_%s", name);
        take_python_error(where);
        LEAVE(-1)
    }
    const int v = (int)PyLong_AsLong(r);
    Py_DECREF(r);
    LEAVE(v)
}

TFF_ENGINE_API int engine_has_work(tff_engine* e) { return call_int(e, "has_work", 0, 0); }
TFF_ENGINE_API int engine_abort(tff_engine* e, int64_t request_id) { return call_int(e, "abort", 1, request_id); }
TFF_ENGINE_API int engine_end_raw(tff_engine* e, int64_t request_id) { return call_int(e, "end_raw", 1, request_id); }

TFF_ENGINE_API int engine_step_raw(tff_engine* e, const tff_raw_entry* entries, int n_entries, float* logits,
                                   int64_t capacity_floats) {
    if (!e || !entries || n_entries <= 0) {
        set_error("engine_step_raw: an engine and at least one entry are needed");
        return -1;
    }
    int64_t rows = 0;
    for (int i = 0; i < n_entries; ++i) {
        const tff_raw_entry* x = &entries[i];
        if (!x->tokens || x->n_tokens <= 0 || x->n_want < 0 || (x->n_want > 0 && !x->want)) {
            snprintf(last_error, sizeof last_error, "engine_step_raw: entry %d has no tokens or a bad list of places", i);
            return -1;
        }
        for (int j = 0; j < x->n_want; ++j)
            if (x->want[j] < 0 || x->want[j] >= x->n_tokens) {
                snprintf(last_error, sizeof last_error, "engine_step_raw: entry %d asks for place %d of %d tokens", i,
                         x->want[j], x->n_tokens);
                return -1;
            }
        rows += x->n_want;
    }
    if (rows * (int64_t)e->vocab > capacity_floats || (rows > 0 && !logits)) {
        snprintf(last_error, sizeof last_error, "engine_step_raw: %lld rows of %d logits do not fit %lld floats",
                 (long long)rows, e->vocab, (long long)capacity_floats);
        return -1;
    }
    ENTER(-1)
    PyObject *ids = PyList_New(n_entries), *toks = PyList_New(n_entries), *wants = PyList_New(n_entries);
    int ok = ids && toks && wants;
    for (int i = 0; ok && i < n_entries; ++i) {
        const tff_raw_entry* x = &entries[i];
        PyObject* a = PyLong_FromLongLong((long long)x->request_id);
        PyObject* b = PyBytes_FromStringAndSize((const char*)x->tokens, (Py_ssize_t)x->n_tokens * 4);
        PyObject* c = PyBytes_FromStringAndSize((const char*)x->want, (Py_ssize_t)x->n_want * 4);
        if (!a || !b || !c) {
            Py_XDECREF(a);
            Py_XDECREF(b);
            Py_XDECREF(c);
            ok = 0;
            break;
        }
        PyList_SET_ITEM(ids, i, a);        // steals the references
        PyList_SET_ITEM(toks, i, b);
        PyList_SET_ITEM(wants, i, c);
    }
    PyObject* r = ok ? PyObject_CallMethod(mod_, "step_raw", "OOOO", e->handle, ids, toks, wants) : NULL;
    Py_XDECREF(ids);
    Py_XDECREF(toks);
    Py_XDECREF(wants);
    if (!r) {
        if (PyErr_Occurred()) take_python_error("engine_step_raw");
        else set_error("engine_step_raw: out of memory");
        LEAVE(-1)
    }
    char* data = NULL;
    Py_ssize_t len = 0;
    if (PyBytes_AsStringAndSize(r, &data, &len) != 0 || len != (Py_ssize_t)(rows * e->vocab * 4)) {
        PyErr_Clear();
        Py_DECREF(r);
        set_error("engine_step_raw: the step returned another number of logits than asked for");
        LEAVE(-1)
    }
    if (len) memcpy(logits, data, (size_t)len);
    Py_DECREF(r);
    LEAVE((int)rows)
}

TFF_ENGINE_API const char* engine_last_error(void) { return last_error; }

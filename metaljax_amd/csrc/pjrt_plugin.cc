// PJRT C API plugin over this package's engine (`metaljax_amd.engine`): the
// `GetPjrtApi` entry point a JAX process loads, so that unmodified `jax.jit`
// programs reach the recognizer (the role of the reference's
// plugin/metal_pjrt.cc, GetPjrtApi at :1276).
//
// The plugin holds no device logic of its own.  Every PJRT object wraps a
// Python object of the engine, and the entry points the engine exports by name
// do the work (reference metal_pjrt.cc:547-563, :662-664, :990-1010, :1125,
// :1168):
//     compile_program(code, fmt, options)  -> executable (name, fingerprint,
//                                             num_outputs, num_params, out_types,
//                                             out_dims, donated_params)
//     execute(executable, [buffer])        -> [buffer]  (data, type_enum, dims, nbytes)
//     buffer_from_host(memoryview, type_enum, dims, byte_strides, offset)
//     to_host(buffer) -> bytes, buffer_pointer(buffer) -> int,
//     device_kind() -> str, stablehlo_version() -> [int]
// One client, one device (GPU 0), one memory space.  Everything is synchronous:
// an event is born ready (reference metal_pjrt.cc:160-164).  A Python exception
// becomes a PJRT_Error carrying the traceback text, code UNIMPLEMENTED if the
// exception's class name contains "Unsupported", else INTERNAL (reference
// metal_pjrt.cc:185-226).  Every entry point takes the GIL.
//
// Built against OpenXLA's xla/pjrt/c/pjrt_c_api.h (API 0.114); the build passes
// the directory that holds the header (`python -m metaljax_amd.build` looks for
// it in PJRT_C_API_INCLUDE and in the reference checkout's plugin/vendor).
#include <Python.h>

#include <atomic>
#include <cstring>
#include <map>
#include <mutex>
#include <string>
#include <utility>
#include <vector>

#include "pjrt_c_api.h"

namespace {

// ------------------------------------------------------------------ errors --
struct PluginError : PJRT_Error {
  PJRT_Error_Code code;
  std::string text;
};

void err_destroy(PJRT_Error* e) { delete static_cast<PluginError*>(e); }
void err_message(const PJRT_Error* e, const char** msg, size_t* n) {
  const auto* pe = static_cast<const PluginError*>(e);
  *msg = pe->text.data();
  *n = pe->text.size();
}
PJRT_Error_Code err_code(const PJRT_Error* e) { return static_cast<const PluginError*>(e)->code; }
void err_payloads(const PJRT_Error*, PJRT_Error_PayloadVisitor, void*) {}

const PJRT_Error_FunctionTable* err_table() {
  static const PJRT_Error_FunctionTable t = [] {
    PJRT_Error_FunctionTable v;
    memset(&v, 0, sizeof(v));
    v.struct_size = PJRT_Error_FunctionTable_STRUCT_SIZE;
    v.instance_size = sizeof(PluginError);
    v.destroy = err_destroy;
    v.message = err_message;
    v.get_code = err_code;
    v.for_each_payload = err_payloads;
    return v;
  }();
  return &t;
}

PJRT_Error* fail(PJRT_Error_Code code, std::string text) {
  auto* e = new PluginError;
  e->vtable = err_table();
  e->code = code;
  e->text = std::move(text);
  return e;
}

// The pending Python exception as a PJRT_Error (and cleared).
PJRT_Error* python_failure(const char* where) {
  PyObject *type = nullptr, *value = nullptr, *tb = nullptr;
  PyErr_Fetch(&type, &value, &tb);
  PyErr_NormalizeException(&type, &value, &tb);
  std::string cls = type ? reinterpret_cast<PyTypeObject*>(type)->tp_name : "Exception";
  std::string text;
  if (PyObject* mod = PyImport_ImportModule("traceback")) {
    PyObject* lines = PyObject_CallMethod(mod, "format_exception", "OOO", type ? type : Py_None,
                                          value ? value : Py_None, tb ? tb : Py_None);
    if (lines) {
      if (PyObject* sep = PyUnicode_FromString("")) {
        if (PyObject* joined = PyUnicode_Join(sep, lines)) {
          if (const char* s = PyUnicode_AsUTF8(joined)) text = s;
          Py_DECREF(joined);
        }
        Py_DECREF(sep);
      }
      Py_DECREF(lines);
    }
    Py_DECREF(mod);
  }
  PyErr_Clear();
  if (text.empty()) {
    text = cls;
    if (value) {
      if (PyObject* s = PyObject_Str(value)) {
        if (const char* c = PyUnicode_AsUTF8(s)) text += std::string(": ") + c;
        Py_DECREF(s);
      }
      PyErr_Clear();
    }
  }
  Py_XDECREF(type);
  Py_XDECREF(value);
  Py_XDECREF(tb);
  const bool unsupported = cls.find("Unsupported") != std::string::npos;
  return fail(unsupported ? PJRT_Error_Code_UNIMPLEMENTED : PJRT_Error_Code_INTERNAL,
              std::string(where) + ": " + text);
}

template <class Args>
PJRT_Error* not_implemented(Args*) {
  return fail(PJRT_Error_Code_UNIMPLEMENTED, "this plugin does not implement the entry point");
}

// A caller's argument struct may be older (smaller) than ours, never smaller
// than the fields that existed when the entry point was introduced; the size
// fields are checked where a call writes past the first members.
#define REQUIRE(cond, text)                                          \
  do {                                                               \
    if (!(cond)) return fail(PJRT_Error_Code_INVALID_ARGUMENT, text); \
  } while (0)

struct Gil {
  PyGILState_STATE s;
  Gil() : s(PyGILState_Ensure()) {}
  ~Gil() { PyGILState_Release(s); }
};

void ensure_python() {
  if (!Py_IsInitialized()) {
    Py_InitializeEx(0);
    PyEval_SaveThread();        // leave the GIL free: every entry point takes it
  }
}

}  // namespace

// ----------------------------------------------------------------- objects --
// (An event's state is read and written under its own mutex: a client may set
// an event it created on one thread while another asks whether it is ready.
// Callbacks run after the lock is released.)
struct PJRT_Event {
  std::mutex mu;
  bool ready = true;
  PJRT_Error_Code code = PJRT_Error_Code_OK;
  std::string text;
  std::vector<std::pair<PJRT_Event_OnReadyCallback, void*>> waiting;
};

struct PJRT_DeviceDescription {
  std::string kind, debug, text;
};

struct PJRT_Device {
  PJRT_Client* client = nullptr;
  PJRT_DeviceDescription description;
};

namespace {
struct MemorySpace : PJRT_Memory {
  PJRT_Client* client = nullptr;
  std::string kind = "device", debug = "qmm_hip device memory 0", text = "DEVICE_0";
  std::map<const void*, std::pair<void*, void (*)(void*)>> user;
  ~MemorySpace() {
    for (auto& kv : user)
      if (kv.second.second) kv.second.second(kv.second.first);
  }
};
void* mem_get_user(PJRT_Memory* m, const void* key) {
  auto& u = static_cast<MemorySpace*>(m)->user;
  auto it = u.find(key);
  return it == u.end() ? nullptr : it->second.first;
}
void mem_set_user(PJRT_Memory* m, const void* key, void* data, void (*dtor)(void*)) {
  auto& u = static_cast<MemorySpace*>(m)->user;
  auto it = u.find(key);
  if (it != u.end() && it->second.second) it->second.second(it->second.first);
  u[key] = {data, dtor};
}
const PJRT_Memory_FunctionTable* mem_table() {
  static const PJRT_Memory_FunctionTable t = [] {
    PJRT_Memory_FunctionTable v;
    memset(&v, 0, sizeof(v));
    v.struct_size = PJRT_Memory_FunctionTable_STRUCT_SIZE;
    v.instance_struct_size = PJRT_Memory_STRUCT_SIZE;
    v.get_user_data = mem_get_user;
    v.set_user_data = mem_set_user;
    return v;
  }();
  return &t;
}
}  // namespace

struct PJRT_Client {
  PyObject* engine = nullptr;
  PJRT_Device device;
  MemorySpace memory;
  PJRT_Device* devices[1];
  PJRT_Memory* memories[1];
  std::string platform = "qmm_hip", version = "metaljax_amd engine on gfx950";
};

namespace {
// What an executable and the loaded executables made from it share.
struct Program {
  std::atomic<int> refs{1};
  PyObject* ex = nullptr;
  std::string name, fingerprint, code;    // code: the module as it was handed to Compile
  size_t num_params = 0;
  std::vector<PJRT_Buffer_Type> out_types;
  std::vector<int64_t> out_dims;          // every output's dimensions, back to back
  std::vector<size_t> out_ranks;
  std::vector<int64_t> donated;           // parameters whose buffers the program consumes
  std::vector<const char*> out_kinds, param_kinds;
  std::vector<size_t> out_kind_sizes, param_kind_sizes;
};
void release(Program* p) {
  if (p && p->refs.fetch_sub(1) == 1) {
    Gil g;
    Py_CLEAR(p->ex);
    delete p;
  }
}
}  // namespace

struct PJRT_Executable {
  Program* program;
};

struct PJRT_LoadedExecutable {
  Program* program;
  PJRT_Client* client;
  bool deleted = false;
};

struct PJRT_Buffer {
  PJRT_Client* client = nullptr;
  PyObject* value = nullptr;               // the engine's buffer object
  PJRT_Buffer_Type type = PJRT_Buffer_Type_INVALID;
  std::vector<int64_t> dims, minor_to_major;
  size_t nbytes = 0;
  // touched by entry points that do not take the interpreter lock
  std::atomic<int> external_refs{0};
  std::atomic<bool> deleted{false};
};

struct PJRT_ExecuteContext {};

namespace {

// ------------------------------------------------------------------ helpers --
bool read_int_list(PyObject* seq, std::vector<int64_t>* out) {
  PyObject* fast = PySequence_Fast(seq, "expected a sequence of integers");
  if (!fast) return false;
  const Py_ssize_t n = PySequence_Fast_GET_SIZE(fast);
  for (Py_ssize_t i = 0; i < n; ++i) {
    const long long v = PyLong_AsLongLong(PySequence_Fast_GET_ITEM(fast, i));
    if (v == -1 && PyErr_Occurred()) {
      Py_DECREF(fast);
      return false;
    }
    out->push_back((int64_t)v);
  }
  Py_DECREF(fast);
  return true;
}

bool read_attr_ints(PyObject* obj, const char* name, std::vector<int64_t>* out) {
  PyObject* a = PyObject_GetAttrString(obj, name);
  if (!a) return false;
  const bool ok = read_int_list(a, out);
  Py_DECREF(a);
  return ok;
}

bool read_attr_size(PyObject* obj, const char* name, size_t* out) {
  PyObject* a = PyObject_GetAttrString(obj, name);
  if (!a) return false;
  const long long v = PyLong_AsLongLong(a);
  Py_DECREF(a);
  if (v == -1 && PyErr_Occurred()) return false;
  *out = (size_t)v;
  return true;
}

bool read_attr_text(PyObject* obj, const char* name, std::string* out) {
  PyObject* a = PyObject_GetAttrString(obj, name);
  if (!a) return false;
  PyObject* s = PyObject_Str(a);
  Py_DECREF(a);
  if (!s) return false;
  const char* c = PyUnicode_AsUTF8(s);
  if (c) *out = c;
  Py_DECREF(s);
  return c != nullptr;
}

PyObject* int_list(const int64_t* v, size_t n) {
  PyObject* l = PyList_New((Py_ssize_t)n);
  if (!l) return nullptr;
  for (size_t i = 0; i < n; ++i) PyList_SET_ITEM(l, (Py_ssize_t)i, PyLong_FromLongLong(v[i]));
  return l;
}

size_t type_bytes(PJRT_Buffer_Type t) {
  switch (t) {
    case PJRT_Buffer_Type_PRED: case PJRT_Buffer_Type_S8: case PJRT_Buffer_Type_U8: return 1;
    case PJRT_Buffer_Type_S16: case PJRT_Buffer_Type_U16: case PJRT_Buffer_Type_F16:
    case PJRT_Buffer_Type_BF16: return 2;
    case PJRT_Buffer_Type_S32: case PJRT_Buffer_Type_U32: case PJRT_Buffer_Type_F32: return 4;
    case PJRT_Buffer_Type_S64: case PJRT_Buffer_Type_U64: case PJRT_Buffer_Type_F64:
    case PJRT_Buffer_Type_C64: return 8;
    case PJRT_Buffer_Type_C128: return 16;
    default: return 0;
  }
}

// Wraps an engine buffer object (a new reference is taken).
PJRT_Buffer* wrap_buffer(PJRT_Client* client, PyObject* value) {
  auto* b = new PJRT_Buffer;
  b->client = client;
  size_t type = 0;
  if (!read_attr_size(value, "type_enum", &type) || !read_attr_ints(value, "dims", &b->dims) ||
      !read_attr_size(value, "nbytes", &b->nbytes)) {
    delete b;
    return nullptr;
  }
  b->type = (PJRT_Buffer_Type)type;
  for (size_t i = b->dims.size(); i-- > 0;) b->minor_to_major.push_back((int64_t)i);
  Py_INCREF(value);
  b->value = value;
  return b;
}

PJRT_Event* ready_event() { return new PJRT_Event; }

// ------------------------------------------------------------------- errors --
void ErrorDestroy(PJRT_Error_Destroy_Args* a) {
  if (a->error) a->error->vtable->destroy(a->error);
}
void ErrorMessage(PJRT_Error_Message_Args* a) {
  a->error->vtable->message(a->error, &a->message, &a->message_size);
}
PJRT_Error* ErrorGetCode(PJRT_Error_GetCode_Args* a) {
  a->code = a->error->vtable->get_code(a->error);
  return nullptr;
}
PJRT_Error* ErrorForEachPayload(PJRT_Error_ForEachPayload_Args* a) {
  a->error->vtable->for_each_payload(a->error, a->visitor, a->user_arg);
  return nullptr;
}

// ------------------------------------------------------------------- plugin --
PJRT_Error* PluginInitialize(PJRT_Plugin_Initialize_Args*) {
  ensure_python();
  return nullptr;
}

PJRT_Error* PluginAttributes(PJRT_Plugin_Attributes_Args* a) {
  // the StableHLO version the engine's reader understands, as the framework
  // asks for it before serialising a module
  static int64_t current[3] = {1, 0, 0}, minimum[3] = {0, 9, 0};
  static PJRT_NamedValue attrs[2];
  static std::once_flag once;
  // A thread that arrives holding the interpreter lock lets go of it while it
  // waits for the one that initialises (which needs that lock), and takes it back after.
  PyThreadState* released = Py_IsInitialized() && PyGILState_Check() ? PyEval_SaveThread() : nullptr;
  std::call_once(once, [] {                   // once, whichever thread asks first
    ensure_python();
    Gil g;
    if (PyObject* mod = PyImport_ImportModule("metaljax_amd.engine")) {
      if (PyObject* v = PyObject_CallMethod(mod, "stablehlo_version", nullptr)) {
        std::vector<int64_t> got;
        if (read_int_list(v, &got) && got.size() == 3)
          for (int i = 0; i < 3; ++i) current[i] = got[i];
        Py_DECREF(v);
      }
      Py_DECREF(mod);
    }
    PyErr_Clear();
    const char* names[2] = {"stablehlo_current_version", "stablehlo_minimum_version"};
    int64_t* values[2] = {current, minimum};
    for (int i = 0; i < 2; ++i) {
      memset(&attrs[i], 0, sizeof(attrs[i]));
      attrs[i].struct_size = PJRT_NamedValue_STRUCT_SIZE;
      attrs[i].name = names[i];
      attrs[i].name_size = strlen(names[i]);
      attrs[i].type = PJRT_NamedValue_kInt64List;
      attrs[i].int64_array_value = values[i];
      attrs[i].value_size = 3;
    }
  });
  if (released) PyEval_RestoreThread(released);
  a->attributes = attrs;
  a->num_attributes = 2;
  return nullptr;
}

// ------------------------------------------------------------------- events --
PJRT_Error* event_error(const PJRT_Event* e) {
  return e->code == PJRT_Error_Code_OK ? nullptr : fail(e->code, e->text);
}
PJRT_Error* EventDestroy(PJRT_Event_Destroy_Args* a) {
  delete a->event;
  return nullptr;
}
PJRT_Error* EventIsReady(PJRT_Event_IsReady_Args* a) {
  std::lock_guard<std::mutex> lock(a->event->mu);
  a->is_ready = a->event->ready;
  return nullptr;
}
PJRT_Error* EventError(PJRT_Event_Error_Args* a) {
  std::lock_guard<std::mutex> lock(a->event->mu);
  return event_error(a->event);
}
PJRT_Error* EventAwait(PJRT_Event_Await_Args* a) {
  // nothing runs behind the caller's back: an event that is not ready is one
  // the caller created and has not set
  std::lock_guard<std::mutex> lock(a->event->mu);
  REQUIRE(a->event->ready, "PJRT_Event_Await on an event nobody has set");
  return event_error(a->event);
}
PJRT_Error* EventOnReady(PJRT_Event_OnReady_Args* a) {
  PJRT_Error* now = nullptr;
  {
    std::lock_guard<std::mutex> lock(a->event->mu);
    if (!a->event->ready) {
      a->event->waiting.emplace_back(a->callback, a->user_arg);
      return nullptr;
    }
    now = event_error(a->event);
  }
  a->callback(now, a->user_arg);
  return nullptr;
}
PJRT_Error* EventCreate(PJRT_Event_Create_Args* a) {
  a->event = new PJRT_Event;
  a->event->ready = false;
  return nullptr;
}
PJRT_Error* EventSet(PJRT_Event_Set_Args* a) {
  PJRT_Event* e = a->event;
  std::vector<std::pair<PJRT_Event_OnReadyCallback, void*>> waiting;
  {
    std::lock_guard<std::mutex> lock(e->mu);
    REQUIRE(!e->ready, "PJRT_Event_Set on an event that is already set");
    e->code = a->error_code;
    if (a->error_message) e->text.assign(a->error_message, a->error_message_size);
    e->ready = true;
    waiting.swap(e->waiting);
  }
  for (auto& w : waiting) {
    PJRT_Error* err = nullptr;
    {
      std::lock_guard<std::mutex> lock(e->mu);
      err = event_error(e);
    }
    w.first(err, w.second);
  }
  return nullptr;
}

// ------------------------------------------------------------------- client --
PJRT_Error* ClientCreate(PJRT_Client_Create_Args* a) {
  ensure_python();
  Gil g;
  PyObject* engine = PyImport_ImportModule("metaljax_amd.engine");
  if (!engine) return python_failure("importing metaljax_amd.engine");
  auto* c = new PJRT_Client;
  c->engine = engine;
  c->device.client = c;
  c->memory.vtable = mem_table();
  c->memory.client = c;
  c->devices[0] = &c->device;
  c->memories[0] = &c->memory;
  std::string kind = "gpu";
  if (PyObject* k = PyObject_CallMethod(engine, "device_kind", nullptr)) {
    if (const char* s = PyUnicode_AsUTF8(k)) kind = s;
    Py_DECREF(k);
  }
  PyErr_Clear();
  c->device.description.kind = kind;
  c->device.description.debug = "qmm_hip device 0 (" + kind + ")";
  c->device.description.text = "QmmHipDevice(id=0)";
  a->client = c;
  return nullptr;
}

PJRT_Error* ClientDestroy(PJRT_Client_Destroy_Args* a) {
  if (a->client) {
    Gil g;
    Py_CLEAR(a->client->engine);
    delete a->client;
  }
  return nullptr;
}
PJRT_Error* ClientPlatformName(PJRT_Client_PlatformName_Args* a) {
  a->platform_name = a->client->platform.data();
  a->platform_name_size = a->client->platform.size();
  return nullptr;
}
PJRT_Error* ClientProcessIndex(PJRT_Client_ProcessIndex_Args* a) {
  a->process_index = 0;
  return nullptr;
}
PJRT_Error* ClientPlatformVersion(PJRT_Client_PlatformVersion_Args* a) {
  a->platform_version = a->client->version.data();
  a->platform_version_size = a->client->version.size();
  return nullptr;
}
PJRT_Error* ClientDevices(PJRT_Client_Devices_Args* a) {
  a->devices = a->client->devices;
  a->num_devices = 1;
  return nullptr;
}
PJRT_Error* ClientAddressableDevices(PJRT_Client_AddressableDevices_Args* a) {
  a->addressable_devices = a->client->devices;
  a->num_addressable_devices = 1;
  return nullptr;
}
PJRT_Error* ClientLookupDevice(PJRT_Client_LookupDevice_Args* a) {
  REQUIRE(a->id == 0, "there is one device, id 0");
  a->device = &a->client->device;
  return nullptr;
}
PJRT_Error* ClientLookupAddressableDevice(PJRT_Client_LookupAddressableDevice_Args* a) {
  REQUIRE(a->local_hardware_id == 0, "there is one device, local hardware id 0");
  a->addressable_device = &a->client->device;
  return nullptr;
}
PJRT_Error* ClientAddressableMemories(PJRT_Client_AddressableMemories_Args* a) {
  a->addressable_memories = a->client->memories;
  a->num_addressable_memories = 1;
  return nullptr;
}
PJRT_Error* ClientDefaultDeviceAssignment(PJRT_Client_DefaultDeviceAssignment_Args* a) {
  REQUIRE(a->num_replicas == 1 && a->num_partitions == 1, "one replica on one partition: there is one device");
  REQUIRE(a->default_assignment_size >= 1, "default_assignment holds no entry");
  a->default_assignment[0] = 0;
  return nullptr;
}

PJRT_Error* ClientCompile(PJRT_Client_Compile_Args* a) {
  REQUIRE(a->program && a->program->code, "no program");
  Gil g;
  PyObject* code = PyBytes_FromStringAndSize(a->program->code, (Py_ssize_t)a->program->code_size);
  PyObject* fmt = PyUnicode_FromStringAndSize(a->program->format ? a->program->format : "mlir",
                                              a->program->format ? (Py_ssize_t)a->program->format_size : 4);
  PyObject* opts = a->compile_options && a->compile_options_size
                       ? PyBytes_FromStringAndSize(a->compile_options, (Py_ssize_t)a->compile_options_size)
                       : (Py_INCREF(Py_None), Py_None);
  PyObject* ex = nullptr;
  if (code && fmt && opts) ex = PyObject_CallMethod(a->client->engine, "compile_program", "OOO", code, fmt, opts);
  Py_XDECREF(code);
  Py_XDECREF(fmt);
  Py_XDECREF(opts);
  if (!ex) return python_failure("compile_program");
  auto* p = new Program;
  p->ex = ex;
  p->code.assign(a->program->code, a->program->code_size);
  std::vector<int64_t> types;
  size_t outputs = 0;
  bool ok = read_attr_text(ex, "name", &p->name) && read_attr_text(ex, "fingerprint", &p->fingerprint) &&
            read_attr_size(ex, "num_outputs", &outputs) && read_attr_size(ex, "num_params", &p->num_params) &&
            read_attr_ints(ex, "out_types", &types) && read_attr_ints(ex, "donated_params", &p->donated);
  if (ok) {
    PyObject* dims = PyObject_GetAttrString(ex, "out_dims");
    PyObject* fast = dims ? PySequence_Fast(dims, "out_dims: expected a sequence") : nullptr;
    ok = fast != nullptr;
    for (Py_ssize_t i = 0; ok && i < PySequence_Fast_GET_SIZE(fast); ++i) {
      std::vector<int64_t> one;
      ok = read_int_list(PySequence_Fast_GET_ITEM(fast, i), &one);
      p->out_ranks.push_back(one.size());
      p->out_dims.insert(p->out_dims.end(), one.begin(), one.end());
    }
    Py_XDECREF(fast);
    Py_XDECREF(dims);
  }
  if (ok && (types.size() != outputs || p->out_ranks.size() != outputs)) {
    PyErr_SetString(PyExc_ValueError, "out_types / out_dims do not match num_outputs");
    ok = false;
  }
  if (!ok) {
    PJRT_Error* e = python_failure("reading the compiled program");
    release(p);
    return e;
  }
  for (int64_t t : types) p->out_types.push_back((PJRT_Buffer_Type)t);
  static const char kind[] = "device";
  p->out_kinds.assign(outputs, kind);
  p->out_kind_sizes.assign(outputs, sizeof(kind) - 1);
  p->param_kinds.assign(p->num_params, kind);
  p->param_kind_sizes.assign(p->num_params, sizeof(kind) - 1);
  a->executable = new PJRT_LoadedExecutable{p, a->client};
  return nullptr;
}

PJRT_Error* ClientBufferFromHostBuffer(PJRT_Client_BufferFromHostBuffer_Args* a) {
  const size_t item = type_bytes(a->type);
  if (item == 0) return fail(PJRT_Error_Code_UNIMPLEMENTED, "BufferFromHostBuffer: unsupported element type");
  REQUIRE(a->num_byte_strides == 0 || a->num_byte_strides == a->num_dims, "byte_strides does not match dims");
  // bytes of the caller's array that the view covers
  size_t extent = item;
  bool empty = false;
  for (size_t i = 0; i < a->num_dims; ++i) {
    REQUIRE(a->dims[i] >= 0, "negative dimension");
    if (a->dims[i] == 0) empty = true;
  }
  if (empty) {
    extent = 0;
  } else if (a->num_byte_strides) {
    for (size_t i = 0; i < a->num_dims; ++i) {
      REQUIRE(a->byte_strides[i] >= 0, "negative byte stride");
      extent += (size_t)(a->dims[i] - 1) * (size_t)a->byte_strides[i];
    }
  } else {
    for (size_t i = 0; i < a->num_dims; ++i) extent *= (size_t)a->dims[i];
  }
  REQUIRE(extent == 0 || a->data, "no host data");
  Gil g;
  static char nothing = 0;
  PyObject* view = PyMemoryView_FromMemory(extent ? const_cast<char*>(static_cast<const char*>(a->data)) : &nothing,
                                           (Py_ssize_t)extent, PyBUF_READ);
  PyObject* dims = int_list(a->dims, a->num_dims);
  PyObject* strides = a->num_byte_strides ? int_list(a->byte_strides, a->num_byte_strides)
                                          : (Py_INCREF(Py_None), Py_None);
  PyObject* value = nullptr;
  if (view && dims && strides)
    value = PyObject_CallMethod(a->client->engine, "buffer_from_host", "OiOOi", view, (int)a->type, dims, strides, 0);
  Py_XDECREF(view);
  Py_XDECREF(dims);
  Py_XDECREF(strides);
  if (!value) return python_failure("buffer_from_host");
  PJRT_Buffer* b = wrap_buffer(a->client, value);
  Py_DECREF(value);
  if (!b) return python_failure("reading the new buffer");
  // the engine has copied the bytes: the caller's array is free at once
  a->done_with_host_buffer = ready_event();
  a->buffer = b;
  return nullptr;
}

// ------------------------------------------------------ device descriptions --
PJRT_Error* DescriptionId(PJRT_DeviceDescription_Id_Args* a) {
  a->id = 0;
  return nullptr;
}
PJRT_Error* DescriptionProcessIndex(PJRT_DeviceDescription_ProcessIndex_Args* a) {
  a->process_index = 0;
  return nullptr;
}
PJRT_Error* DescriptionAttributes(PJRT_DeviceDescription_Attributes_Args* a) {
  a->attributes = nullptr;
  a->num_attributes = 0;
  return nullptr;
}
PJRT_Error* DescriptionKind(PJRT_DeviceDescription_Kind_Args* a) {
  a->device_kind = a->device_description->kind.data();
  a->device_kind_size = a->device_description->kind.size();
  return nullptr;
}
PJRT_Error* DescriptionDebugString(PJRT_DeviceDescription_DebugString_Args* a) {
  a->debug_string = a->device_description->debug.data();
  a->debug_string_size = a->device_description->debug.size();
  return nullptr;
}
PJRT_Error* DescriptionToString(PJRT_DeviceDescription_ToString_Args* a) {
  a->to_string = a->device_description->text.data();
  a->to_string_size = a->device_description->text.size();
  return nullptr;
}

// ------------------------------------------------------------------ devices --
PJRT_Error* DeviceGetDescription(PJRT_Device_GetDescription_Args* a) {
  a->device_description = &a->device->description;
  return nullptr;
}
PJRT_Error* DeviceIsAddressable(PJRT_Device_IsAddressable_Args* a) {
  a->is_addressable = true;
  return nullptr;
}
PJRT_Error* DeviceLocalHardwareId(PJRT_Device_LocalHardwareId_Args* a) {
  a->local_hardware_id = 0;
  return nullptr;
}
PJRT_Error* DeviceAddressableMemories(PJRT_Device_AddressableMemories_Args* a) {
  a->memories = a->device->client->memories;
  a->num_memories = 1;
  return nullptr;
}
PJRT_Error* DeviceDefaultMemory(PJRT_Device_DefaultMemory_Args* a) {
  a->memory = &a->device->client->memory;
  return nullptr;
}
PJRT_Error* DeviceMemoryStats(PJRT_Device_MemoryStats_Args* a) {
  // the engine's buffers belong to torch's allocator; nothing is tracked here
  a->bytes_in_use = 0;
  a->peak_bytes_in_use_is_set = a->num_allocs_is_set = a->largest_alloc_size_is_set = false;
  a->bytes_limit_is_set = a->bytes_reserved_is_set = a->peak_bytes_reserved_is_set = false;
  a->bytes_reservable_limit_is_set = a->largest_free_block_bytes_is_set = false;
  a->pool_bytes_is_set = a->peak_pool_bytes_is_set = false;
  return nullptr;
}

void no_attributes_to_free(PJRT_Device_Attributes*) {}
PJRT_Error* DeviceGetAttributes(PJRT_Device_GetAttributes_Args* a) {
  a->attributes = nullptr;
  a->num_attributes = 0;
  a->device_attributes = nullptr;
  a->attributes_deleter = no_attributes_to_free;
  return nullptr;
}

// ----------------------------------------------------------------- memories --
PJRT_Error* MemoryId(PJRT_Memory_Id_Args* a) {
  a->id = 0;
  return nullptr;
}
PJRT_Error* MemoryKind(PJRT_Memory_Kind_Args* a) {
  auto* m = static_cast<MemorySpace*>(a->memory);
  a->kind = m->kind.data();
  a->kind_size = m->kind.size();
  return nullptr;
}
PJRT_Error* MemoryKindId(PJRT_Memory_Kind_Id_Args* a) {
  a->kind_id = 0;
  return nullptr;
}
PJRT_Error* MemoryDebugString(PJRT_Memory_DebugString_Args* a) {
  auto* m = static_cast<MemorySpace*>(a->memory);
  a->debug_string = m->debug.data();
  a->debug_string_size = m->debug.size();
  return nullptr;
}
PJRT_Error* MemoryToString(PJRT_Memory_ToString_Args* a) {
  auto* m = static_cast<MemorySpace*>(a->memory);
  a->to_string = m->text.data();
  a->to_string_size = m->text.size();
  return nullptr;
}
PJRT_Error* MemoryAddressableByDevices(PJRT_Memory_AddressableByDevices_Args* a) {
  auto* m = static_cast<MemorySpace*>(a->memory);
  a->devices = m->client->devices;
  a->num_devices = 1;
  return nullptr;
}

// -------------------------------------------------------------- executables --
PJRT_Error* ExecutableDestroy(PJRT_Executable_Destroy_Args* a) {
  if (a->executable) {
    release(a->executable->program);
    delete a->executable;
  }
  return nullptr;
}
PJRT_Error* ExecutableName(PJRT_Executable_Name_Args* a) {
  a->executable_name = a->executable->program->name.data();
  a->executable_name_size = a->executable->program->name.size();
  return nullptr;
}
PJRT_Error* ExecutableNumReplicas(PJRT_Executable_NumReplicas_Args* a) {
  a->num_replicas = 1;
  return nullptr;
}
PJRT_Error* ExecutableNumPartitions(PJRT_Executable_NumPartitions_Args* a) {
  a->num_partitions = 1;
  return nullptr;
}
PJRT_Error* ExecutableNumOutputs(PJRT_Executable_NumOutputs_Args* a) {
  a->num_outputs = a->executable->program->out_types.size();
  return nullptr;
}
PJRT_Error* ExecutableCodeSize(PJRT_Executable_SizeOfGeneratedCodeInBytes_Args* a) {
  a->size_in_bytes = 0;                     // interpreted: no generated code
  return nullptr;
}
PJRT_Error* ExecutableCostAnalysis(PJRT_Executable_GetCostAnalysis_Args* a) {
  a->num_properties = 0;
  a->properties = nullptr;
  return nullptr;
}
PJRT_Error* ExecutableOutputMemoryKinds(PJRT_Executable_OutputMemoryKinds_Args* a) {
  Program* p = a->executable->program;
  a->num_outputs = p->out_kinds.size();
  a->memory_kinds = p->out_kinds.data();
  a->memory_kind_sizes = p->out_kind_sizes.data();
  return nullptr;
}
PJRT_Error* ExecutableParameterMemoryKinds(PJRT_Executable_ParameterMemoryKinds_Args* a) {
  Program* p = a->executable->program;
  a->num_parameters = p->param_kinds.size();
  a->memory_kinds = p->param_kinds.data();
  a->memory_kind_sizes = p->param_kind_sizes.data();
  return nullptr;
}
PJRT_Error* ExecutableOutputElementTypes(PJRT_Executable_OutputElementTypes_Args* a) {
  Program* p = a->executable->program;
  a->output_types = p->out_types.data();
  a->num_output_types = p->out_types.size();
  return nullptr;
}
PJRT_Error* ExecutableOutputDimensions(PJRT_Executable_OutputDimensions_Args* a) {
  Program* p = a->executable->program;
  a->num_outputs = p->out_ranks.size();
  a->dims = p->out_dims.data();
  a->dim_sizes = p->out_ranks.data();
  return nullptr;
}
PJRT_Error* ExecutableFingerprint(PJRT_Executable_Fingerprint_Args* a) {
  a->executable_fingerprint = a->executable->program->fingerprint.data();
  a->executable_fingerprint_size = a->executable->program->fingerprint.size();
  return nullptr;
}

// The program an executable was made from: nothing is optimised, so it is the
// module the caller compiled, in the format it came in ("mlir").
PJRT_Error* ExecutableOptimizedProgram(PJRT_Executable_OptimizedProgram_Args* a) {
  REQUIRE(a->program, "no program to fill");
  static const char format[] = "mlir";
  const std::string& code = a->executable->program->code;
  a->program->format = format;
  a->program->format_size = sizeof(format) - 1;
  if (!a->program->code) {                    // a query for the size
    a->program->code_size = code.size();
    return nullptr;
  }
  REQUIRE(a->program->code_size >= code.size(), "the program buffer is too small");
  memcpy(a->program->code, code.data(), code.size());
  a->program->code_size = code.size();
  return nullptr;
}

PJRT_Error* LoadedLogicalIds(PJRT_LoadedExecutable_AddressableDeviceLogicalIds_Args* a) {
  static PJRT_LogicalDeviceIds ids[1] = {{0, 0}};   // replica 0, partition 0 on the one device
  a->addressable_device_logical_ids = ids;
  a->num_addressable_device_logical_ids = 1;
  return nullptr;
}

// One replica of one computation on device 0, as an xla.DeviceAssignmentProto written out by hand
// (reference metal_pjrt.cc:930-942 answers the same way): field 1 replica_count = 1, field 2
// computation_count = 1, field 3 one ComputationDevice whose field 1, the packed replica_device_ids,
// holds the single id 0.  The bytes are static, so there is nothing for the deleter to free.
void keep_assignment(PJRT_DeviceAssignmentSerialized*) {}

PJRT_Error* LoadedDeviceAssignment(PJRT_LoadedExecutable_GetDeviceAssignment_Args* a) {
  static const char proto[] = {
      (1 << 3) | 0, 1,            // replica_count: varint 1
      (2 << 3) | 0, 1,            // computation_count: varint 1
      (3 << 3) | 2, 3,            // computation_devices: a message of three bytes
      (1 << 3) | 2, 1, 0,         //   replica_device_ids, packed: one varint, 0
  };
  a->serialized_bytes = proto;
  a->serialized_bytes_size = sizeof(proto);
  a->serialized_device_assignment = nullptr;
  a->serialized_device_assignment_deleter = keep_assignment;
  return nullptr;
}

PJRT_Error* LoadedDestroy(PJRT_LoadedExecutable_Destroy_Args* a) {
  if (a->executable) {
    release(a->executable->program);
    delete a->executable;
  }
  return nullptr;
}
PJRT_Error* LoadedGetExecutable(PJRT_LoadedExecutable_GetExecutable_Args* a) {
  Program* p = a->loaded_executable->program;
  p->refs.fetch_add(1);
  a->executable = new PJRT_Executable{p};
  return nullptr;
}
PJRT_Error* LoadedAddressableDevices(PJRT_LoadedExecutable_AddressableDevices_Args* a) {
  a->addressable_devices = a->executable->client->devices;
  a->num_addressable_devices = 1;
  return nullptr;
}
PJRT_Error* LoadedDelete(PJRT_LoadedExecutable_Delete_Args* a) {
  a->executable->deleted = true;
  return nullptr;
}
PJRT_Error* LoadedIsDeleted(PJRT_LoadedExecutable_IsDeleted_Args* a) {
  a->is_deleted = a->executable->deleted;
  return nullptr;
}
PJRT_Error* LoadedFingerprint(PJRT_LoadedExecutable_Fingerprint_Args* a) {
  a->executable_fingerprint = a->executable->program->fingerprint.data();
  a->executable_fingerprint_size = a->executable->program->fingerprint.size();
  return nullptr;
}

PJRT_Error* LoadedExecute(PJRT_LoadedExecutable_Execute_Args* a) {
  PJRT_LoadedExecutable* le = a->executable;
  REQUIRE(!le->deleted, "the executable has been deleted");
  REQUIRE(a->num_devices == 1, "there is one device: one argument list");
  Program* p = le->program;
  REQUIRE(a->num_args == p->num_params, "wrong number of arguments");
  if (a->options) REQUIRE(a->options->num_send_ops == 0 && a->options->num_recv_ops == 0, "no send / recv callbacks");
  Gil g;
  PyObject* args = PyList_New((Py_ssize_t)a->num_args);
  if (!args) return python_failure("execute");
  for (size_t i = 0; i < a->num_args; ++i) {
    PJRT_Buffer* b = a->argument_lists[0][i];
    if (!b || b->deleted || !b->value) {
      Py_DECREF(args);
      return fail(PJRT_Error_Code_INVALID_ARGUMENT, "argument " + std::to_string(i) + " is a deleted buffer");
    }
    Py_INCREF(b->value);
    PyList_SET_ITEM(args, (Py_ssize_t)i, b->value);
  }
  PyObject* outs = PyObject_CallMethod(le->client->engine, "execute", "OO", p->ex, args);
  Py_DECREF(args);
  if (!outs) return python_failure("execute");
  PyObject* fast = PySequence_Fast(outs, "execute: expected a sequence of buffers");
  Py_DECREF(outs);
  if (!fast) return python_failure("execute");
  const size_t n = (size_t)PySequence_Fast_GET_SIZE(fast);
  if (n != p->out_types.size()) {
    Py_DECREF(fast);
    return fail(PJRT_Error_Code_INTERNAL, "execute returned " + std::to_string(n) + " outputs, the program has " +
                                              std::to_string(p->out_types.size()));
  }
  std::vector<PJRT_Buffer*> made;
  for (size_t i = 0; i < n; ++i) {
    PJRT_Buffer* b = wrap_buffer(le->client, PySequence_Fast_GET_ITEM(fast, (Py_ssize_t)i));
    if (!b) {
      PJRT_Error* e = python_failure("reading an output buffer");
      for (PJRT_Buffer* m : made) {
        Py_CLEAR(m->value);
        delete m;
      }
      Py_DECREF(fast);
      return e;
    }
    made.push_back(b);
  }
  Py_DECREF(fast);
  for (size_t i = 0; i < n; ++i) a->output_lists[0][i] = made[i];
  // A donated parameter's buffer is consumed by the call (reference
  // metal_pjrt.cc:1032-1036) unless the caller lists it as not donatable: its
  // value is dropped and the handle reports deleted.  (The engine writes fresh
  // outputs, so nothing aliases the dropped value.)
  for (int64_t d : p->donated) {
    if (d < 0 || (size_t)d >= a->num_args) continue;
    bool keep = false;
    // (a caller built against an older header passes a shorter options struct)
    if (a->options &&
        a->options->struct_size >= PJRT_STRUCT_SIZE(PJRT_ExecuteOptions, num_non_donatable_input_indices))
      for (size_t k = 0; k < a->options->num_non_donatable_input_indices; ++k)
        keep = keep || a->options->non_donatable_input_indices[k] == d;
    if (keep) continue;
    PJRT_Buffer* b = a->argument_lists[0][d];
    if (b->external_refs > 0) continue;     // someone outside still reads it
    Py_CLEAR(b->value);
    b->deleted = true;
  }
  if (a->device_complete_events) a->device_complete_events[0] = ready_event();
  return nullptr;
}

// ------------------------------------------------------------------ buffers --
PJRT_Error* BufferDestroy(PJRT_Buffer_Destroy_Args* a) {
  if (a->buffer) {
    Gil g;
    Py_CLEAR(a->buffer->value);
    delete a->buffer;
  }
  return nullptr;
}
PJRT_Error* BufferElementType(PJRT_Buffer_ElementType_Args* a) {
  a->type = a->buffer->type;
  return nullptr;
}
PJRT_Error* BufferDimensions(PJRT_Buffer_Dimensions_Args* a) {
  a->dims = a->buffer->dims.data();
  a->num_dims = a->buffer->dims.size();
  return nullptr;
}
PJRT_Error* BufferUnpaddedDimensions(PJRT_Buffer_UnpaddedDimensions_Args* a) {
  a->unpadded_dims = a->buffer->dims.data();
  a->num_dims = a->buffer->dims.size();
  return nullptr;
}
PJRT_Error* BufferDynamicDimensionIndices(PJRT_Buffer_DynamicDimensionIndices_Args* a) {
  a->dynamic_dim_indices = nullptr;
  a->num_dynamic_dims = 0;
  return nullptr;
}
PJRT_Error* BufferGetMemoryLayout(PJRT_Buffer_GetMemoryLayout_Args* a) {
  memset(&a->layout, 0, sizeof(a->layout));
  a->layout.struct_size = PJRT_Buffer_MemoryLayout_STRUCT_SIZE;
  a->layout.type = PJRT_Buffer_MemoryLayout_Type_Tiled;
  a->layout.tiled.struct_size = PJRT_Buffer_MemoryLayout_Tiled_STRUCT_SIZE;
  a->layout.tiled.minor_to_major = a->buffer->minor_to_major.data();
  a->layout.tiled.minor_to_major_size = a->buffer->minor_to_major.size();
  return nullptr;
}
PJRT_Error* BufferOnDeviceSize(PJRT_Buffer_OnDeviceSizeInBytes_Args* a) {
  a->on_device_size_in_bytes = a->buffer->nbytes;
  return nullptr;
}
PJRT_Error* BufferDevice(PJRT_Buffer_Device_Args* a) {
  a->device = &a->buffer->client->device;
  return nullptr;
}
PJRT_Error* BufferMemory(PJRT_Buffer_Memory_Args* a) {
  a->memory = &a->buffer->client->memory;
  return nullptr;
}
PJRT_Error* BufferDelete(PJRT_Buffer_Delete_Args* a) {
  Gil g;
  Py_CLEAR(a->buffer->value);
  a->buffer->deleted = true;
  return nullptr;
}
PJRT_Error* BufferIsDeleted(PJRT_Buffer_IsDeleted_Args* a) {
  a->is_deleted = a->buffer->deleted;
  return nullptr;
}
PJRT_Error* same_value(PJRT_Buffer* src, PJRT_Buffer** dst) {
  // one device, one memory, immutable values: a copy is another handle
  REQUIRE(!src->deleted && src->value, "the buffer has been deleted");
  Gil g;
  PJRT_Buffer* b = wrap_buffer(src->client, src->value);
  if (!b) return python_failure("copying a buffer");
  *dst = b;
  return nullptr;
}
PJRT_Error* BufferCopyToDevice(PJRT_Buffer_CopyToDevice_Args* a) { return same_value(a->buffer, &a->dst_buffer); }
PJRT_Error* BufferCopyToMemory(PJRT_Buffer_CopyToMemory_Args* a) { return same_value(a->buffer, &a->dst_buffer); }

PJRT_Error* BufferToHostBuffer(PJRT_Buffer_ToHostBuffer_Args* a) {
  PJRT_Buffer* b = a->src;
  REQUIRE(!b->deleted && b->value, "the buffer has been deleted");
  if (!a->dst) {                              // a query for the size
    a->dst_size = b->nbytes;
    return nullptr;
  }
  REQUIRE(a->dst_size >= b->nbytes, "dst is smaller than the buffer");
  Gil g;
  PyObject* bytes = PyObject_CallMethod(b->client->engine, "to_host", "O", b->value);
  if (!bytes) return python_failure("to_host");
  char* data = nullptr;
  Py_ssize_t n = 0;
  if (PyBytes_AsStringAndSize(bytes, &data, &n) != 0) {
    Py_DECREF(bytes);
    return python_failure("to_host");
  }
  if ((size_t)n != b->nbytes) {
    Py_DECREF(bytes);
    return fail(PJRT_Error_Code_INTERNAL, "to_host returned " + std::to_string(n) + " bytes for a buffer of " +
                                              std::to_string(b->nbytes));
  }
  memcpy(a->dst, data, (size_t)n);
  Py_DECREF(bytes);
  a->event = ready_event();
  return nullptr;
}
PJRT_Error* BufferIsOnCpu(PJRT_Buffer_IsOnCpu_Args* a) {
  a->is_on_cpu = false;
  return nullptr;
}
PJRT_Error* BufferReadyEvent(PJRT_Buffer_ReadyEvent_Args* a) {
  a->event = ready_event();
  return nullptr;
}
PJRT_Error* buffer_address(PJRT_Buffer* b, uintptr_t* out) {
  REQUIRE(!b->deleted && b->value, "the buffer has been deleted");
  Gil g;
  PyObject* p = PyObject_CallMethod(b->client->engine, "buffer_pointer", "O", b->value);
  if (!p) return python_failure("buffer_pointer");
  const unsigned long long v = PyLong_AsUnsignedLongLong(p);
  Py_DECREF(p);
  if (v == (unsigned long long)-1 && PyErr_Occurred()) return python_failure("buffer_pointer");
  *out = (uintptr_t)v;
  return nullptr;
}
PJRT_Error* BufferUnsafePointer(PJRT_Buffer_UnsafePointer_Args* a) {
  return buffer_address(a->buffer, &a->buffer_pointer);
}
PJRT_Error* BufferOpaquePointer(PJRT_Buffer_OpaqueDeviceMemoryDataPointer_Args* a) {
  uintptr_t v = 0;
  if (PJRT_Error* e = buffer_address(a->buffer, &v)) return e;
  a->device_memory_ptr = reinterpret_cast<void*>(v);
  return nullptr;
}
PJRT_Error* BufferIncreaseRefs(PJRT_Buffer_IncreaseExternalReferenceCount_Args* a) {
  ++a->buffer->external_refs;
  return nullptr;
}
PJRT_Error* BufferDecreaseRefs(PJRT_Buffer_DecreaseExternalReferenceCount_Args* a) {
  REQUIRE(a->buffer->external_refs > 0, "the external reference count is already zero");
  --a->buffer->external_refs;
  return nullptr;
}

PJRT_Error* ContextCreate(PJRT_ExecuteContext_Create_Args* a) {
  a->context = new PJRT_ExecuteContext;
  return nullptr;
}
PJRT_Error* ContextDestroy(PJRT_ExecuteContext_Destroy_Args* a) {
  delete a->context;
  return nullptr;
}

}  // namespace

namespace {
void fill_api(PJRT_Api& api) {
  memset(&api, 0, sizeof(api));
  api.struct_size = PJRT_Api_STRUCT_SIZE;
  api.pjrt_api_version.struct_size = PJRT_Api_Version_STRUCT_SIZE;
  api.pjrt_api_version.major_version = PJRT_API_MAJOR;
  api.pjrt_api_version.minor_version = PJRT_API_MINOR;

#define HAVE(entry, fn) api.entry = fn
#define LACK(entry) api.entry = not_implemented<entry##_Args>
  HAVE(PJRT_Error_Destroy, ErrorDestroy);
  HAVE(PJRT_Error_Message, ErrorMessage);
  HAVE(PJRT_Error_GetCode, ErrorGetCode);
  HAVE(PJRT_Error_ForEachPayload, ErrorForEachPayload);
  HAVE(PJRT_Plugin_Initialize, PluginInitialize);
  HAVE(PJRT_Plugin_Attributes, PluginAttributes);
  HAVE(PJRT_Event_Destroy, EventDestroy);
  HAVE(PJRT_Event_IsReady, EventIsReady);
  HAVE(PJRT_Event_Error, EventError);
  HAVE(PJRT_Event_Await, EventAwait);
  HAVE(PJRT_Event_OnReady, EventOnReady);
  HAVE(PJRT_Event_Create, EventCreate);
  HAVE(PJRT_Event_Set, EventSet);

  HAVE(PJRT_Client_Create, ClientCreate);
  HAVE(PJRT_Client_Destroy, ClientDestroy);
  HAVE(PJRT_Client_PlatformName, ClientPlatformName);
  HAVE(PJRT_Client_ProcessIndex, ClientProcessIndex);
  HAVE(PJRT_Client_PlatformVersion, ClientPlatformVersion);
  HAVE(PJRT_Client_Devices, ClientDevices);
  HAVE(PJRT_Client_AddressableDevices, ClientAddressableDevices);
  HAVE(PJRT_Client_LookupDevice, ClientLookupDevice);
  HAVE(PJRT_Client_LookupAddressableDevice, ClientLookupAddressableDevice);
  HAVE(PJRT_Client_AddressableMemories, ClientAddressableMemories);
  HAVE(PJRT_Client_Compile, ClientCompile);
  HAVE(PJRT_Client_DefaultDeviceAssignment, ClientDefaultDeviceAssignment);
  HAVE(PJRT_Client_BufferFromHostBuffer, ClientBufferFromHostBuffer);
  LACK(PJRT_Client_TopologyDescription);
  LACK(PJRT_Client_CreateViewOfDeviceBuffer);
  LACK(PJRT_Client_CreateBuffersForAsyncHostToDevice);
  LACK(PJRT_Client_DmaMap);
  LACK(PJRT_Client_DmaUnmap);
  LACK(PJRT_Client_CreateUninitializedBuffer);
  LACK(PJRT_Client_UpdateGlobalProcessInfo);
  LACK(PJRT_Client_CreateAliasBuffer);
  LACK(PJRT_Client_FulfillAliasBuffer);
  LACK(PJRT_Client_CreateErrorBuffer);
  LACK(PJRT_Client_Load);

  HAVE(PJRT_DeviceDescription_Id, DescriptionId);
  HAVE(PJRT_DeviceDescription_ProcessIndex, DescriptionProcessIndex);
  HAVE(PJRT_DeviceDescription_Attributes, DescriptionAttributes);
  HAVE(PJRT_DeviceDescription_Kind, DescriptionKind);
  HAVE(PJRT_DeviceDescription_DebugString, DescriptionDebugString);
  HAVE(PJRT_DeviceDescription_ToString, DescriptionToString);
  HAVE(PJRT_Device_GetDescription, DeviceGetDescription);
  HAVE(PJRT_Device_IsAddressable, DeviceIsAddressable);
  HAVE(PJRT_Device_LocalHardwareId, DeviceLocalHardwareId);
  HAVE(PJRT_Device_AddressableMemories, DeviceAddressableMemories);
  HAVE(PJRT_Device_DefaultMemory, DeviceDefaultMemory);
  HAVE(PJRT_Device_MemoryStats, DeviceMemoryStats);
  LACK(PJRT_Device_PoisonExecution);
  LACK(PJRT_Device_CreateAsyncTrackingEvent);
  LACK(PJRT_Device_ClearMemoryStats);
  HAVE(PJRT_Device_GetAttributes, DeviceGetAttributes);
  LACK(PJRT_AsyncTrackingEvent_Destroy);
  HAVE(PJRT_Memory_Id, MemoryId);
  HAVE(PJRT_Memory_Kind, MemoryKind);
  HAVE(PJRT_Memory_Kind_Id, MemoryKindId);
  HAVE(PJRT_Memory_DebugString, MemoryDebugString);
  HAVE(PJRT_Memory_ToString, MemoryToString);
  HAVE(PJRT_Memory_AddressableByDevices, MemoryAddressableByDevices);

  HAVE(PJRT_Executable_Destroy, ExecutableDestroy);
  HAVE(PJRT_Executable_Name, ExecutableName);
  HAVE(PJRT_Executable_NumReplicas, ExecutableNumReplicas);
  HAVE(PJRT_Executable_NumPartitions, ExecutableNumPartitions);
  HAVE(PJRT_Executable_NumOutputs, ExecutableNumOutputs);
  HAVE(PJRT_Executable_SizeOfGeneratedCodeInBytes, ExecutableCodeSize);
  HAVE(PJRT_Executable_GetCostAnalysis, ExecutableCostAnalysis);
  HAVE(PJRT_Executable_OutputMemoryKinds, ExecutableOutputMemoryKinds);
  HAVE(PJRT_Executable_ParameterMemoryKinds, ExecutableParameterMemoryKinds);
  HAVE(PJRT_Executable_OutputElementTypes, ExecutableOutputElementTypes);
  HAVE(PJRT_Executable_OutputDimensions, ExecutableOutputDimensions);
  HAVE(PJRT_Executable_Fingerprint, ExecutableFingerprint);
  HAVE(PJRT_Executable_OptimizedProgram, ExecutableOptimizedProgram);
  LACK(PJRT_Executable_Serialize);
  LACK(PJRT_Executable_GetCompiledMemoryStats);
  LACK(PJRT_Executable_GetCompileOptions);
  LACK(PJRT_Executable_DeserializeAndLoad);
  HAVE(PJRT_LoadedExecutable_Destroy, LoadedDestroy);
  HAVE(PJRT_LoadedExecutable_GetExecutable, LoadedGetExecutable);
  HAVE(PJRT_LoadedExecutable_AddressableDevices, LoadedAddressableDevices);
  HAVE(PJRT_LoadedExecutable_Delete, LoadedDelete);
  HAVE(PJRT_LoadedExecutable_IsDeleted, LoadedIsDeleted);
  HAVE(PJRT_LoadedExecutable_Execute, LoadedExecute);
  HAVE(PJRT_LoadedExecutable_Fingerprint, LoadedFingerprint);
  HAVE(PJRT_LoadedExecutable_GetDeviceAssignment, LoadedDeviceAssignment);
  HAVE(PJRT_LoadedExecutable_AddressableDeviceLogicalIds, LoadedLogicalIds);

  HAVE(PJRT_Buffer_Destroy, BufferDestroy);
  HAVE(PJRT_Buffer_ElementType, BufferElementType);
  HAVE(PJRT_Buffer_Dimensions, BufferDimensions);
  HAVE(PJRT_Buffer_UnpaddedDimensions, BufferUnpaddedDimensions);
  HAVE(PJRT_Buffer_DynamicDimensionIndices, BufferDynamicDimensionIndices);
  HAVE(PJRT_Buffer_GetMemoryLayout, BufferGetMemoryLayout);
  HAVE(PJRT_Buffer_OnDeviceSizeInBytes, BufferOnDeviceSize);
  HAVE(PJRT_Buffer_Device, BufferDevice);
  HAVE(PJRT_Buffer_Memory, BufferMemory);
  HAVE(PJRT_Buffer_Delete, BufferDelete);
  HAVE(PJRT_Buffer_IsDeleted, BufferIsDeleted);
  HAVE(PJRT_Buffer_CopyToDevice, BufferCopyToDevice);
  HAVE(PJRT_Buffer_CopyToMemory, BufferCopyToMemory);
  HAVE(PJRT_Buffer_ToHostBuffer, BufferToHostBuffer);
  HAVE(PJRT_Buffer_IsOnCpu, BufferIsOnCpu);
  HAVE(PJRT_Buffer_ReadyEvent, BufferReadyEvent);
  HAVE(PJRT_Buffer_UnsafePointer, BufferUnsafePointer);
  HAVE(PJRT_Buffer_IncreaseExternalReferenceCount, BufferIncreaseRefs);
  HAVE(PJRT_Buffer_DecreaseExternalReferenceCount, BufferDecreaseRefs);
  HAVE(PJRT_Buffer_OpaqueDeviceMemoryDataPointer, BufferOpaquePointer);
  LACK(PJRT_Buffer_CopyRawToHost);
  LACK(PJRT_Buffer_CopyRawToHostFuture);
  LACK(PJRT_Buffer_Bitcast);

  LACK(PJRT_CopyToDeviceStream_Destroy);
  LACK(PJRT_CopyToDeviceStream_AddChunk);
  LACK(PJRT_CopyToDeviceStream_TotalBytes);
  LACK(PJRT_CopyToDeviceStream_GranuleSize);
  LACK(PJRT_CopyToDeviceStream_CurrentBytes);
  LACK(PJRT_TopologyDescription_Create);
  LACK(PJRT_TopologyDescription_Destroy);
  LACK(PJRT_TopologyDescription_PlatformName);
  LACK(PJRT_TopologyDescription_PlatformVersion);
  LACK(PJRT_TopologyDescription_GetDeviceDescriptions);
  LACK(PJRT_TopologyDescription_Serialize);
  LACK(PJRT_TopologyDescription_Attributes);
  LACK(PJRT_TopologyDescription_Deserialize);
  LACK(PJRT_TopologyDescription_Fingerprint);
  LACK(PJRT_TopologyDescription_MakeCanonicalShapeForMemorySpace);
  LACK(PJRT_TopologyDescription_GetMemorySpaceKindIds);
  LACK(PJRT_AsyncHostToDeviceTransferManager_Destroy);
  LACK(PJRT_AsyncHostToDeviceTransferManager_TransferData);
  LACK(PJRT_AsyncHostToDeviceTransferManager_RetrieveBuffer);
  LACK(PJRT_AsyncHostToDeviceTransferManager_Device);
  LACK(PJRT_AsyncHostToDeviceTransferManager_BufferCount);
  LACK(PJRT_AsyncHostToDeviceTransferManager_BufferSize);
  LACK(PJRT_AsyncHostToDeviceTransferManager_SetBufferError);
  LACK(PJRT_AsyncHostToDeviceTransferManager_AddMetadata);
  LACK(PJRT_AsyncHostToDeviceTransferManager_TransferLiteral);
  LACK(PJRT_Buffer_DonateWithControlDependency);
  LACK(PJRT_Compile);
  HAVE(PJRT_ExecuteContext_Create, ContextCreate);
  HAVE(PJRT_ExecuteContext_Destroy, ContextDestroy);
#undef HAVE
#undef LACK
}
}  // namespace

extern "C" __attribute__((visibility("default"))) const PJRT_Api* GetPjrtApi() {
  static const PJRT_Api* const table = [] {   // filled once, whichever thread asks first
    static PJRT_Api api;
    fill_api(api);
    return &api;
  }();
  return table;
}

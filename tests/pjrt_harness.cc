// Test harness: drives a PJRT plugin through the PJRT C API the way a
// framework's client does (load the library, GetPjrtApi, initialise, create a
// client, compile a module, move buffers in, execute, move results out), behind
// a flat C interface that the Python tests call with ctypes.  jax is not
// installed where these tests run; this is the caller that stands in for it.
// Test infrastructure: nothing in the package uses it.
//
// Built by `python -m metaljax_amd.build` against the same pjrt_c_api.h as the
// plugin.  Handles are indices into tables kept here; every call returns 0 or
// the PJRT_Error_Code of the failure (negative: a failure of the harness
// itself) and leaves the message in `pjrt_harness_last_error()`.
#include <dlfcn.h>
#include <stdint.h>

#include <cstring>
#include <string>
#include <vector>

#include "pjrt_c_api.h"

namespace {

void* g_lib = nullptr;
const PJRT_Api* g_api = nullptr;
PJRT_Client* g_client = nullptr;
PJRT_Device* g_device = nullptr;
std::string g_error;
std::vector<PJRT_LoadedExecutable*> g_exes;
std::vector<PJRT_Buffer*> g_bufs;

int harness_failure(const std::string& text) {
  g_error = text;
  return -1;
}

// Takes the error (if any): message kept, error destroyed, code returned.
int taken(PJRT_Error* e) {
  if (!e) return 0;
  PJRT_Error_Message_Args m;
  memset(&m, 0, sizeof(m));
  m.struct_size = PJRT_Error_Message_Args_STRUCT_SIZE;
  m.error = e;
  g_api->PJRT_Error_Message(&m);
  g_error.assign(m.message, m.message_size);
  PJRT_Error_GetCode_Args c;
  memset(&c, 0, sizeof(c));
  c.struct_size = PJRT_Error_GetCode_Args_STRUCT_SIZE;
  c.error = e;
  PJRT_Error* e2 = g_api->PJRT_Error_GetCode(&c);
  const int code = e2 ? (int)PJRT_Error_Code_UNKNOWN : (int)c.code;
  PJRT_Error_Destroy_Args d;
  memset(&d, 0, sizeof(d));
  d.struct_size = PJRT_Error_Destroy_Args_STRUCT_SIZE;
  d.error = e;
  g_api->PJRT_Error_Destroy(&d);
  return code ? code : (int)PJRT_Error_Code_UNKNOWN;
}

// Waits for an event a call handed out and destroys it, as a client does.
int settle(PJRT_Event* ev) {
  if (!ev) return 0;
  PJRT_Event_Await_Args w;
  memset(&w, 0, sizeof(w));
  w.struct_size = PJRT_Event_Await_Args_STRUCT_SIZE;
  w.event = ev;
  const int rc = taken(g_api->PJRT_Event_Await(&w));
  PJRT_Event_Destroy_Args d;
  memset(&d, 0, sizeof(d));
  d.struct_size = PJRT_Event_Destroy_Args_STRUCT_SIZE;
  d.event = ev;
  taken(g_api->PJRT_Event_Destroy(&d));
  return rc;
}

void copy_text(const char* s, size_t n, char* out, int cap) {
  if (!out || cap <= 0) return;
  const size_t m = n < (size_t)cap - 1 ? n : (size_t)cap - 1;
  memcpy(out, s, m);
  out[m] = 0;
}

#define NEED_OPEN() \
  if (!g_api || !g_client) return harness_failure("no plugin is open")

}  // namespace

extern "C" {

const char* pjrt_harness_last_error() { return g_error.c_str(); }

int pjrt_harness_open(const char* path) {
  if (g_client) return harness_failure("a plugin is already open");
  g_lib = dlopen(path, RTLD_NOW | RTLD_LOCAL);
  if (!g_lib) return harness_failure(std::string("dlopen: ") + dlerror());
  typedef const PJRT_Api* (*GetApi)();
  GetApi get = reinterpret_cast<GetApi>(dlsym(g_lib, "GetPjrtApi"));
  if (!get) return harness_failure("the library exports no GetPjrtApi");
  g_api = get();
  if (!g_api) return harness_failure("GetPjrtApi returned null");
  if (g_api->pjrt_api_version.major_version != PJRT_API_MAJOR)
    return harness_failure("the plugin speaks another major version of the API");
  if (g_api->struct_size < PJRT_Api_STRUCT_SIZE) return harness_failure("the plugin's PJRT_Api is shorter than this header's");
  PJRT_Plugin_Initialize_Args init;
  memset(&init, 0, sizeof(init));
  init.struct_size = PJRT_Plugin_Initialize_Args_STRUCT_SIZE;
  if (int rc = taken(g_api->PJRT_Plugin_Initialize(&init))) return rc;
  PJRT_Client_Create_Args cc;
  memset(&cc, 0, sizeof(cc));
  cc.struct_size = PJRT_Client_Create_Args_STRUCT_SIZE;
  if (int rc = taken(g_api->PJRT_Client_Create(&cc))) return rc;
  g_client = cc.client;
  PJRT_Client_AddressableDevices_Args ad;
  memset(&ad, 0, sizeof(ad));
  ad.struct_size = PJRT_Client_AddressableDevices_Args_STRUCT_SIZE;
  ad.client = g_client;
  if (int rc = taken(g_api->PJRT_Client_AddressableDevices(&ad))) return rc;
  if (ad.num_addressable_devices < 1) return harness_failure("the client has no addressable device");
  g_device = ad.addressable_devices[0];
  return 0;
}

int pjrt_harness_close() {
  NEED_OPEN();
  for (PJRT_Buffer* b : g_bufs)
    if (b) {
      PJRT_Buffer_Destroy_Args d;
      memset(&d, 0, sizeof(d));
      d.struct_size = PJRT_Buffer_Destroy_Args_STRUCT_SIZE;
      d.buffer = b;
      taken(g_api->PJRT_Buffer_Destroy(&d));
    }
  g_bufs.clear();
  for (PJRT_LoadedExecutable* e : g_exes)
    if (e) {
      PJRT_LoadedExecutable_Destroy_Args d;
      memset(&d, 0, sizeof(d));
      d.struct_size = PJRT_LoadedExecutable_Destroy_Args_STRUCT_SIZE;
      d.executable = e;
      taken(g_api->PJRT_LoadedExecutable_Destroy(&d));
    }
  g_exes.clear();
  PJRT_Client_Destroy_Args d;
  memset(&d, 0, sizeof(d));
  d.struct_size = PJRT_Client_Destroy_Args_STRUCT_SIZE;
  d.client = g_client;
  const int rc = taken(g_api->PJRT_Client_Destroy(&d));
  g_client = nullptr;
  g_device = nullptr;
  return rc;             // the library stays loaded: it may hold the interpreter's state
}

// API version, platform name, device kind, number of devices and memories,
// the plugin's stablehlo_current_version attribute (three integers, or -1s).
int pjrt_harness_info(int* version, char* platform, int platform_cap, char* kind, int kind_cap, int* counts,
                      int64_t* stablehlo) {
  NEED_OPEN();
  version[0] = g_api->pjrt_api_version.major_version;
  version[1] = g_api->pjrt_api_version.minor_version;
  PJRT_Client_PlatformName_Args pn;
  memset(&pn, 0, sizeof(pn));
  pn.struct_size = PJRT_Client_PlatformName_Args_STRUCT_SIZE;
  pn.client = g_client;
  if (int rc = taken(g_api->PJRT_Client_PlatformName(&pn))) return rc;
  copy_text(pn.platform_name, pn.platform_name_size, platform, platform_cap);
  PJRT_Device_GetDescription_Args gd;
  memset(&gd, 0, sizeof(gd));
  gd.struct_size = PJRT_Device_GetDescription_Args_STRUCT_SIZE;
  gd.device = g_device;
  if (int rc = taken(g_api->PJRT_Device_GetDescription(&gd))) return rc;
  PJRT_DeviceDescription_Kind_Args dk;
  memset(&dk, 0, sizeof(dk));
  dk.struct_size = PJRT_DeviceDescription_Kind_Args_STRUCT_SIZE;
  dk.device_description = gd.device_description;
  if (int rc = taken(g_api->PJRT_DeviceDescription_Kind(&dk))) return rc;
  copy_text(dk.device_kind, dk.device_kind_size, kind, kind_cap);
  PJRT_Client_Devices_Args dv;
  memset(&dv, 0, sizeof(dv));
  dv.struct_size = PJRT_Client_Devices_Args_STRUCT_SIZE;
  dv.client = g_client;
  if (int rc = taken(g_api->PJRT_Client_Devices(&dv))) return rc;
  counts[0] = (int)dv.num_devices;
  PJRT_Client_AddressableMemories_Args am;
  memset(&am, 0, sizeof(am));
  am.struct_size = PJRT_Client_AddressableMemories_Args_STRUCT_SIZE;
  am.client = g_client;
  if (int rc = taken(g_api->PJRT_Client_AddressableMemories(&am))) return rc;
  counts[1] = (int)am.num_addressable_memories;
  stablehlo[0] = stablehlo[1] = stablehlo[2] = -1;
  PJRT_Plugin_Attributes_Args pa;
  memset(&pa, 0, sizeof(pa));
  pa.struct_size = PJRT_Plugin_Attributes_Args_STRUCT_SIZE;
  if (int rc = taken(g_api->PJRT_Plugin_Attributes(&pa))) return rc;
  for (size_t i = 0; i < pa.num_attributes; ++i) {
    const PJRT_NamedValue& v = pa.attributes[i];
    if (std::string(v.name, v.name_size) == "stablehlo_current_version" && v.type == PJRT_NamedValue_kInt64List &&
        v.value_size == 3)
      for (int j = 0; j < 3; ++j) stablehlo[j] = v.int64_array_value[j];
  }
  return 0;
}

int pjrt_harness_compile(const char* code, int64_t code_size, const char* format, int* handle) {
  NEED_OPEN();
  PJRT_Program prog;
  memset(&prog, 0, sizeof(prog));
  prog.struct_size = PJRT_Program_STRUCT_SIZE;
  prog.code = const_cast<char*>(code);
  prog.code_size = (size_t)code_size;
  prog.format = format;
  prog.format_size = strlen(format);
  PJRT_Client_Compile_Args c;
  memset(&c, 0, sizeof(c));
  c.struct_size = PJRT_Client_Compile_Args_STRUCT_SIZE;
  c.client = g_client;
  c.program = &prog;
  if (int rc = taken(g_api->PJRT_Client_Compile(&c))) return rc;
  g_exes.push_back(c.executable);
  *handle = (int)g_exes.size() - 1;
  return 0;
}

// counts: [num_outputs, num_replicas, num_partitions]; types[i], ranks[i] and
// the dimensions back to back in dims (at most `cap` outputs / 8*cap dims).
int pjrt_harness_executable_info(int handle, int* counts, int* types, int* ranks, int64_t* dims, int cap,
                                 char* name, int name_cap, char* fingerprint, int fingerprint_cap) {
  NEED_OPEN();
  if (handle < 0 || handle >= (int)g_exes.size() || !g_exes[handle]) return harness_failure("no such executable");
  PJRT_LoadedExecutable_GetExecutable_Args ge;
  memset(&ge, 0, sizeof(ge));
  ge.struct_size = PJRT_LoadedExecutable_GetExecutable_Args_STRUCT_SIZE;
  ge.loaded_executable = g_exes[handle];
  if (int rc = taken(g_api->PJRT_LoadedExecutable_GetExecutable(&ge))) return rc;
  PJRT_Executable* ex = ge.executable;
  int rc = 0;
  do {
    PJRT_Executable_NumOutputs_Args no;
    memset(&no, 0, sizeof(no));
    no.struct_size = PJRT_Executable_NumOutputs_Args_STRUCT_SIZE;
    no.executable = ex;
    if ((rc = taken(g_api->PJRT_Executable_NumOutputs(&no)))) break;
    counts[0] = (int)no.num_outputs;
    PJRT_Executable_NumReplicas_Args nr;
    memset(&nr, 0, sizeof(nr));
    nr.struct_size = PJRT_Executable_NumReplicas_Args_STRUCT_SIZE;
    nr.executable = ex;
    if ((rc = taken(g_api->PJRT_Executable_NumReplicas(&nr)))) break;
    counts[1] = (int)nr.num_replicas;
    PJRT_Executable_NumPartitions_Args np;
    memset(&np, 0, sizeof(np));
    np.struct_size = PJRT_Executable_NumPartitions_Args_STRUCT_SIZE;
    np.executable = ex;
    if ((rc = taken(g_api->PJRT_Executable_NumPartitions(&np)))) break;
    counts[2] = (int)np.num_partitions;
    PJRT_Executable_OutputElementTypes_Args ot;
    memset(&ot, 0, sizeof(ot));
    ot.struct_size = PJRT_Executable_OutputElementTypes_Args_STRUCT_SIZE;
    ot.executable = ex;
    if ((rc = taken(g_api->PJRT_Executable_OutputElementTypes(&ot)))) break;
    PJRT_Executable_OutputDimensions_Args od;
    memset(&od, 0, sizeof(od));
    od.struct_size = PJRT_Executable_OutputDimensions_Args_STRUCT_SIZE;
    od.executable = ex;
    if ((rc = taken(g_api->PJRT_Executable_OutputDimensions(&od)))) break;
    if (ot.num_output_types != no.num_outputs || od.num_outputs != no.num_outputs) {
      rc = harness_failure("output types / dimensions do not match the number of outputs");
      break;
    }
    size_t at = 0;
    for (size_t i = 0; i < no.num_outputs && (int)i < cap; ++i) {
      types[i] = (int)ot.output_types[i];
      ranks[i] = (int)od.dim_sizes[i];
      for (size_t j = 0; j < od.dim_sizes[i] && at < (size_t)cap * 8; ++j, ++at) dims[at] = od.dims[at];
    }
    PJRT_Executable_Name_Args en;
    memset(&en, 0, sizeof(en));
    en.struct_size = PJRT_Executable_Name_Args_STRUCT_SIZE;
    en.executable = ex;
    if ((rc = taken(g_api->PJRT_Executable_Name(&en)))) break;
    copy_text(en.executable_name, en.executable_name_size, name, name_cap);
    PJRT_Executable_Fingerprint_Args fp;
    memset(&fp, 0, sizeof(fp));
    fp.struct_size = PJRT_Executable_Fingerprint_Args_STRUCT_SIZE;
    fp.executable = ex;
    if ((rc = taken(g_api->PJRT_Executable_Fingerprint(&fp)))) break;
    copy_text(fp.executable_fingerprint, fp.executable_fingerprint_size, fingerprint, fingerprint_cap);
  } while (false);
  PJRT_Executable_Destroy_Args d;
  memset(&d, 0, sizeof(d));
  d.struct_size = PJRT_Executable_Destroy_Args_STRUCT_SIZE;
  d.executable = ex;
  g_api->PJRT_Executable_Destroy(&d);       // (keeps the message of a failure above)
  return rc;
}

// byte_strides may be null (dense row-major).
int pjrt_harness_buffer_from_host(const void* data, int type, const int64_t* dims, int num_dims,
                                  const int64_t* byte_strides, int* handle) {
  NEED_OPEN();
  PJRT_Client_BufferFromHostBuffer_Args a;
  memset(&a, 0, sizeof(a));
  a.struct_size = PJRT_Client_BufferFromHostBuffer_Args_STRUCT_SIZE;
  a.client = g_client;
  a.data = data;
  a.type = (PJRT_Buffer_Type)type;
  a.dims = dims;
  a.num_dims = (size_t)num_dims;
  a.byte_strides = byte_strides;
  a.num_byte_strides = byte_strides ? (size_t)num_dims : 0;
  a.host_buffer_semantics = PJRT_HostBufferSemantics_kImmutableOnlyDuringCall;
  a.device = g_device;
  if (int rc = taken(g_api->PJRT_Client_BufferFromHostBuffer(&a))) return rc;
  if (int rc = settle(a.done_with_host_buffer)) return rc;
  g_bufs.push_back(a.buffer);
  *handle = (int)g_bufs.size() - 1;
  return 0;
}

// info: [type, rank, nbytes, pointer, on_cpu, deleted]; dims: at most 8.
int pjrt_harness_buffer_info(int handle, int64_t* info, int64_t* dims) {
  NEED_OPEN();
  if (handle < 0 || handle >= (int)g_bufs.size() || !g_bufs[handle]) return harness_failure("no such buffer");
  PJRT_Buffer* b = g_bufs[handle];
  PJRT_Buffer_ElementType_Args et;
  memset(&et, 0, sizeof(et));
  et.struct_size = PJRT_Buffer_ElementType_Args_STRUCT_SIZE;
  et.buffer = b;
  if (int rc = taken(g_api->PJRT_Buffer_ElementType(&et))) return rc;
  info[0] = (int64_t)et.type;
  PJRT_Buffer_Dimensions_Args bd;
  memset(&bd, 0, sizeof(bd));
  bd.struct_size = PJRT_Buffer_Dimensions_Args_STRUCT_SIZE;
  bd.buffer = b;
  if (int rc = taken(g_api->PJRT_Buffer_Dimensions(&bd))) return rc;
  info[1] = (int64_t)bd.num_dims;
  for (size_t i = 0; i < bd.num_dims && i < 8; ++i) dims[i] = bd.dims[i];
  PJRT_Buffer_OnDeviceSizeInBytes_Args sz;
  memset(&sz, 0, sizeof(sz));
  sz.struct_size = PJRT_Buffer_OnDeviceSizeInBytes_Args_STRUCT_SIZE;
  sz.buffer = b;
  if (int rc = taken(g_api->PJRT_Buffer_OnDeviceSizeInBytes(&sz))) return rc;
  info[2] = (int64_t)sz.on_device_size_in_bytes;
  PJRT_Buffer_IsDeleted_Args del;
  memset(&del, 0, sizeof(del));
  del.struct_size = PJRT_Buffer_IsDeleted_Args_STRUCT_SIZE;
  del.buffer = b;
  if (int rc = taken(g_api->PJRT_Buffer_IsDeleted(&del))) return rc;
  info[5] = del.is_deleted ? 1 : 0;
  info[3] = 0;
  if (!del.is_deleted) {
    PJRT_Buffer_UnsafePointer_Args up;
    memset(&up, 0, sizeof(up));
    up.struct_size = PJRT_Buffer_UnsafePointer_Args_STRUCT_SIZE;
    up.buffer = b;
    if (int rc = taken(g_api->PJRT_Buffer_UnsafePointer(&up))) return rc;
    info[3] = (int64_t)up.buffer_pointer;
  }
  PJRT_Buffer_IsOnCpu_Args oc;
  memset(&oc, 0, sizeof(oc));
  oc.struct_size = PJRT_Buffer_IsOnCpu_Args_STRUCT_SIZE;
  oc.buffer = b;
  if (int rc = taken(g_api->PJRT_Buffer_IsOnCpu(&oc))) return rc;
  info[4] = oc.is_on_cpu ? 1 : 0;
  return 0;
}

// dst null: only the size is asked for (returned in *size).
int pjrt_harness_to_host(int handle, void* dst, int64_t* size) {
  NEED_OPEN();
  if (handle < 0 || handle >= (int)g_bufs.size() || !g_bufs[handle]) return harness_failure("no such buffer");
  PJRT_Buffer_ToHostBuffer_Args a;
  memset(&a, 0, sizeof(a));
  a.struct_size = PJRT_Buffer_ToHostBuffer_Args_STRUCT_SIZE;
  a.src = g_bufs[handle];
  a.dst = dst;
  a.dst_size = dst ? (size_t)*size : 0;
  if (int rc = taken(g_api->PJRT_Buffer_ToHostBuffer(&a))) return rc;
  if (!dst) {
    *size = (int64_t)a.dst_size;
    return 0;
  }
  return settle(a.event);
}

namespace {
int64_t g_keep[16];
int g_num_keep = 0;
}  // namespace

// Parameters the next execute lists as not donatable (at most 16).
int pjrt_harness_keep_inputs(const int64_t* indices, int n) {
  g_num_keep = n < 16 ? n : 16;
  for (int i = 0; i < g_num_keep; ++i) g_keep[i] = indices[i];
  return 0;
}

int pjrt_harness_execute(int exe, const int* args, int num_args, int* outs, int out_cap, int* num_outs) {
  NEED_OPEN();
  if (exe < 0 || exe >= (int)g_exes.size() || !g_exes[exe]) return harness_failure("no such executable");
  std::vector<PJRT_Buffer*> in((size_t)num_args);
  for (int i = 0; i < num_args; ++i) {
    if (args[i] < 0 || args[i] >= (int)g_bufs.size() || !g_bufs[args[i]]) return harness_failure("no such buffer");
    in[(size_t)i] = g_bufs[args[i]];
  }
  // how many outputs the caller has to make room for
  PJRT_LoadedExecutable_GetExecutable_Args ge;
  memset(&ge, 0, sizeof(ge));
  ge.struct_size = PJRT_LoadedExecutable_GetExecutable_Args_STRUCT_SIZE;
  ge.loaded_executable = g_exes[exe];
  if (int rc = taken(g_api->PJRT_LoadedExecutable_GetExecutable(&ge))) return rc;
  PJRT_Executable_NumOutputs_Args no;
  memset(&no, 0, sizeof(no));
  no.struct_size = PJRT_Executable_NumOutputs_Args_STRUCT_SIZE;
  no.executable = ge.executable;
  int rc = taken(g_api->PJRT_Executable_NumOutputs(&no));
  PJRT_Executable_Destroy_Args xd;
  memset(&xd, 0, sizeof(xd));
  xd.struct_size = PJRT_Executable_Destroy_Args_STRUCT_SIZE;
  xd.executable = ge.executable;
  g_api->PJRT_Executable_Destroy(&xd);
  if (rc) return rc;
  if ((int)no.num_outputs > out_cap) return harness_failure("more outputs than the caller has room for");
  std::vector<PJRT_Buffer*> out(no.num_outputs, nullptr);
  PJRT_Buffer* const* arg_lists[1] = {in.data()};
  PJRT_Buffer** out_lists[1] = {out.data()};
  PJRT_Event* done[1] = {nullptr};
  PJRT_ExecuteOptions opts;
  memset(&opts, 0, sizeof(opts));
  opts.struct_size = PJRT_ExecuteOptions_STRUCT_SIZE;
  opts.non_donatable_input_indices = g_keep;
  opts.num_non_donatable_input_indices = (size_t)g_num_keep;
  g_num_keep = 0;
  PJRT_LoadedExecutable_Execute_Args a;
  memset(&a, 0, sizeof(a));
  a.struct_size = PJRT_LoadedExecutable_Execute_Args_STRUCT_SIZE;
  a.executable = g_exes[exe];
  a.options = &opts;
  a.argument_lists = arg_lists;
  a.num_devices = 1;
  a.num_args = (size_t)num_args;
  a.output_lists = out_lists;
  a.device_complete_events = done;
  if ((rc = taken(g_api->PJRT_LoadedExecutable_Execute(&a)))) return rc;
  if ((rc = settle(done[0]))) return rc;
  for (size_t i = 0; i < out.size(); ++i) {
    g_bufs.push_back(out[i]);
    outs[i] = (int)g_bufs.size() - 1;
  }
  *num_outs = (int)out.size();
  return 0;
}

// Delete (the value is dropped, the handle stays valid and reports deleted).
int pjrt_harness_buffer_delete(int handle) {
  NEED_OPEN();
  if (handle < 0 || handle >= (int)g_bufs.size() || !g_bufs[handle]) return harness_failure("no such buffer");
  PJRT_Buffer_Delete_Args d;
  memset(&d, 0, sizeof(d));
  d.struct_size = PJRT_Buffer_Delete_Args_STRUCT_SIZE;
  d.buffer = g_bufs[handle];
  return taken(g_api->PJRT_Buffer_Delete(&d));
}

int pjrt_harness_buffer_destroy(int handle) {
  NEED_OPEN();
  if (handle < 0 || handle >= (int)g_bufs.size() || !g_bufs[handle]) return harness_failure("no such buffer");
  PJRT_Buffer_Destroy_Args d;
  memset(&d, 0, sizeof(d));
  d.struct_size = PJRT_Buffer_Destroy_Args_STRUCT_SIZE;
  d.buffer = g_bufs[handle];
  g_bufs[handle] = nullptr;
  return taken(g_api->PJRT_Buffer_Destroy(&d));
}

// An entry point the plugin leaves out: must answer UNIMPLEMENTED, not crash.
int pjrt_harness_topology() {
  NEED_OPEN();
  PJRT_Client_TopologyDescription_Args t;
  memset(&t, 0, sizeof(t));
  t.struct_size = PJRT_Client_TopologyDescription_Args_STRUCT_SIZE;
  t.client = g_client;
  return taken(g_api->PJRT_Client_TopologyDescription(&t));
}

namespace {
int g_called = 0;
int g_called_code = -1;
void on_ready(PJRT_Error* e, void* arg) {
  ++g_called;
  g_called_code = e ? taken(e) : 0;
  *static_cast<int*>(arg) += 1;
}
}  // namespace

// A scripted walk over the smaller entry points (events a caller creates and
// sets, buffer copies / layout / reference counts, memories and their user
// data, device assignment, look-ups).  0, or the number of the first step whose
// answer was not the expected one (the message says what the plugin answered).
#define STEP(n, cond)                 \
  do {                                \
    if (!(cond)) return (n);          \
  } while (0)
#define ARGS(T, v)                    \
  T v;                                \
  memset(&v, 0, sizeof(v));           \
  v.struct_size = T##_STRUCT_SIZE

int pjrt_harness_walk(int buffer, int exe) {
  NEED_OPEN();
  if (buffer < 0 || buffer >= (int)g_bufs.size() || !g_bufs[buffer]) return harness_failure("no such buffer");
  if (exe < 0 || exe >= (int)g_exes.size() || !g_exes[exe]) return harness_failure("no such executable");
  PJRT_Buffer* b = g_bufs[buffer];
  PJRT_LoadedExecutable* le = g_exes[exe];
  g_error.clear();
  // -- an event the caller creates: not ready, callback deferred, then set
  ARGS(PJRT_Event_Create_Args, ec);
  STEP(1, taken(g_api->PJRT_Event_Create(&ec)) == 0 && ec.event);
  ARGS(PJRT_Event_IsReady_Args, ir);
  ir.event = ec.event;
  STEP(2, taken(g_api->PJRT_Event_IsReady(&ir)) == 0 && !ir.is_ready);
  int hits = 0;
  g_called = 0;
  ARGS(PJRT_Event_OnReady_Args, orr);
  orr.event = ec.event;
  orr.callback = on_ready;
  orr.user_arg = &hits;
  STEP(3, taken(g_api->PJRT_Event_OnReady(&orr)) == 0 && hits == 0);
  ARGS(PJRT_Event_Await_Args, aw);
  aw.event = ec.event;
  STEP(4, taken(g_api->PJRT_Event_Await(&aw)) == (int)PJRT_Error_Code_INVALID_ARGUMENT);   // nobody has set it: no wait for ever
  ARGS(PJRT_Event_Set_Args, es);
  es.event = ec.event;
  es.error_code = PJRT_Error_Code_OK;
  STEP(5, taken(g_api->PJRT_Event_Set(&es)) == 0 && hits == 1 && g_called_code == 0);
  STEP(6, taken(g_api->PJRT_Event_IsReady(&ir)) == 0 && ir.is_ready);
  STEP(7, taken(g_api->PJRT_Event_Await(&aw)) == 0);
  STEP(8, taken(g_api->PJRT_Event_OnReady(&orr)) == 0 && hits == 2);       // already ready: called at once
  ARGS(PJRT_Event_Destroy_Args, ed);
  ed.event = ec.event;
  STEP(9, taken(g_api->PJRT_Event_Destroy(&ed)) == 0);
  // -- an event set with an error hands that error to whoever asks
  ARGS(PJRT_Event_Create_Args, ec2);
  STEP(10, taken(g_api->PJRT_Event_Create(&ec2)) == 0);
  ARGS(PJRT_Event_Set_Args, es2);
  es2.event = ec2.event;
  es2.error_code = PJRT_Error_Code_ABORTED;
  es2.error_message = "stopped by the caller";
  es2.error_message_size = strlen(es2.error_message);
  STEP(11, taken(g_api->PJRT_Event_Set(&es2)) == 0);
  ARGS(PJRT_Event_Error_Args, ee);
  ee.event = ec2.event;
  STEP(12, taken(g_api->PJRT_Event_Error(&ee)) == (int)PJRT_Error_Code_ABORTED && g_error == "stopped by the caller");
  ed.event = ec2.event;
  STEP(13, taken(g_api->PJRT_Event_Destroy(&ed)) == 0);
  // -- a buffer's own event is ready
  ARGS(PJRT_Buffer_ReadyEvent_Args, re);
  re.buffer = b;
  STEP(14, taken(g_api->PJRT_Buffer_ReadyEvent(&re)) == 0 && re.event);
  ir.event = re.event;
  STEP(15, taken(g_api->PJRT_Event_IsReady(&ir)) == 0 && ir.is_ready && settle(re.event) == 0);
  // -- layout: dense, minor to major = last dimension first
  ARGS(PJRT_Buffer_Dimensions_Args, bd);
  bd.buffer = b;
  STEP(16, taken(g_api->PJRT_Buffer_Dimensions(&bd)) == 0);
  ARGS(PJRT_Buffer_GetMemoryLayout_Args, ml);
  ml.buffer = b;
  STEP(17, taken(g_api->PJRT_Buffer_GetMemoryLayout(&ml)) == 0 && ml.layout.type == PJRT_Buffer_MemoryLayout_Type_Tiled &&
               ml.layout.tiled.minor_to_major_size == bd.num_dims && ml.layout.tiled.num_tiles == 0);
  for (size_t i = 0; i < bd.num_dims; ++i) STEP(18, ml.layout.tiled.minor_to_major[i] == (int64_t)(bd.num_dims - 1 - i));
  ARGS(PJRT_Buffer_UnpaddedDimensions_Args, ud);
  ud.buffer = b;
  STEP(19, taken(g_api->PJRT_Buffer_UnpaddedDimensions(&ud)) == 0 && ud.num_dims == bd.num_dims);
  ARGS(PJRT_Buffer_DynamicDimensionIndices_Args, dd);
  dd.buffer = b;
  STEP(20, taken(g_api->PJRT_Buffer_DynamicDimensionIndices(&dd)) == 0 && dd.num_dynamic_dims == 0);
  // -- a copy to the (only) device is another buffer with the same bytes
  ARGS(PJRT_Buffer_CopyToDevice_Args, cd);
  cd.buffer = b;
  cd.dst_device = g_device;
  STEP(21, taken(g_api->PJRT_Buffer_CopyToDevice(&cd)) == 0 && cd.dst_buffer && cd.dst_buffer != b);
  {
    ARGS(PJRT_Buffer_ToHostBuffer_Args, q1);
    q1.src = b;
    ARGS(PJRT_Buffer_ToHostBuffer_Args, q2);
    q2.src = cd.dst_buffer;
    STEP(22, taken(g_api->PJRT_Buffer_ToHostBuffer(&q1)) == 0 && taken(g_api->PJRT_Buffer_ToHostBuffer(&q2)) == 0 &&
                 q1.dst_size == q2.dst_size);
    std::vector<char> h1(q1.dst_size + 1), h2(q2.dst_size + 1);
    q1.dst = h1.data();
    q2.dst = h2.data();
    STEP(23, taken(g_api->PJRT_Buffer_ToHostBuffer(&q1)) == 0 && settle(q1.event) == 0 &&
                 taken(g_api->PJRT_Buffer_ToHostBuffer(&q2)) == 0 && settle(q2.event) == 0 && h1 == h2);
    q1.dst_size = q1.dst_size ? q1.dst_size - 1 : 0;              // too small a destination is refused
    if (q2.dst_size) STEP(24, taken(g_api->PJRT_Buffer_ToHostBuffer(&q1)) == (int)PJRT_Error_Code_INVALID_ARGUMENT);
  }
  ARGS(PJRT_Buffer_Destroy_Args, bdel);
  bdel.buffer = cd.dst_buffer;
  STEP(25, taken(g_api->PJRT_Buffer_Destroy(&bdel)) == 0);
  // -- external reference counts go up and down, never below zero
  ARGS(PJRT_Buffer_IncreaseExternalReferenceCount_Args, inc);
  inc.buffer = b;
  ARGS(PJRT_Buffer_DecreaseExternalReferenceCount_Args, dec);
  dec.buffer = b;
  STEP(26, taken(g_api->PJRT_Buffer_IncreaseExternalReferenceCount(&inc)) == 0 &&
               taken(g_api->PJRT_Buffer_DecreaseExternalReferenceCount(&dec)) == 0);
  STEP(27, taken(g_api->PJRT_Buffer_DecreaseExternalReferenceCount(&dec)) == (int)PJRT_Error_Code_INVALID_ARGUMENT);
  ARGS(PJRT_Buffer_OpaqueDeviceMemoryDataPointer_Args, op);
  op.buffer = b;
  ARGS(PJRT_Buffer_UnsafePointer_Args, up);
  up.buffer = b;
  STEP(28, taken(g_api->PJRT_Buffer_OpaqueDeviceMemoryDataPointer(&op)) == 0 && taken(g_api->PJRT_Buffer_UnsafePointer(&up)) == 0 &&
               (uintptr_t)op.device_memory_ptr == up.buffer_pointer && up.buffer_pointer != 0);
  // -- the buffer's memory is the device's default memory, kind "device", with user data
  ARGS(PJRT_Buffer_Memory_Args, bm);
  bm.buffer = b;
  STEP(29, taken(g_api->PJRT_Buffer_Memory(&bm)) == 0 && bm.memory && bm.memory->vtable);
  ARGS(PJRT_Device_DefaultMemory_Args, dm);
  dm.device = g_device;
  STEP(30, taken(g_api->PJRT_Device_DefaultMemory(&dm)) == 0 && dm.memory == bm.memory);
  ARGS(PJRT_Memory_Kind_Args, mk);
  mk.memory = bm.memory;
  STEP(31, taken(g_api->PJRT_Memory_Kind(&mk)) == 0 && std::string(mk.kind, mk.kind_size) == "device");
  static int key = 0, payload = 42;
  STEP(32, bm.memory->vtable->get_user_data(bm.memory, &key) == nullptr);
  bm.memory->vtable->set_user_data(bm.memory, &key, &payload, nullptr);
  STEP(33, bm.memory->vtable->get_user_data(bm.memory, &key) == &payload);
  ARGS(PJRT_Memory_AddressableByDevices_Args, mad);
  mad.memory = bm.memory;
  STEP(34, taken(g_api->PJRT_Memory_AddressableByDevices(&mad)) == 0 && mad.num_devices == 1 && mad.devices[0] == g_device);
  ARGS(PJRT_Buffer_Device_Args, bdev);
  bdev.buffer = b;
  STEP(35, taken(g_api->PJRT_Buffer_Device(&bdev)) == 0 && bdev.device == g_device);
  // -- look-ups and the default assignment of one replica on one partition
  ARGS(PJRT_Client_LookupDevice_Args, ld);
  ld.client = g_client;
  ld.id = 0;
  STEP(36, taken(g_api->PJRT_Client_LookupDevice(&ld)) == 0 && ld.device == g_device);
  ld.id = 1;
  STEP(37, taken(g_api->PJRT_Client_LookupDevice(&ld)) == (int)PJRT_Error_Code_INVALID_ARGUMENT);
  int assignment[2] = {-1, -1};
  ARGS(PJRT_Client_DefaultDeviceAssignment_Args, da);
  da.client = g_client;
  da.num_replicas = 1;
  da.num_partitions = 1;
  da.default_assignment_size = 1;
  da.default_assignment = assignment;
  STEP(38, taken(g_api->PJRT_Client_DefaultDeviceAssignment(&da)) == 0 && assignment[0] == 0);
  da.num_replicas = 2;
  da.default_assignment_size = 2;
  STEP(39, taken(g_api->PJRT_Client_DefaultDeviceAssignment(&da)) == (int)PJRT_Error_Code_INVALID_ARGUMENT);
  // -- the loaded executable: its device, its fingerprint, memory kinds, delete
  ARGS(PJRT_LoadedExecutable_AddressableDevices_Args, lad);
  lad.executable = le;
  STEP(40, taken(g_api->PJRT_LoadedExecutable_AddressableDevices(&lad)) == 0 && lad.num_addressable_devices == 1 &&
               lad.addressable_devices[0] == g_device);
  ARGS(PJRT_LoadedExecutable_GetExecutable_Args, ge);
  ge.loaded_executable = le;
  STEP(41, taken(g_api->PJRT_LoadedExecutable_GetExecutable(&ge)) == 0 && ge.executable);
  ARGS(PJRT_Executable_Fingerprint_Args, f1);
  f1.executable = ge.executable;
  ARGS(PJRT_LoadedExecutable_Fingerprint_Args, f2);
  f2.executable = le;
  STEP(42, taken(g_api->PJRT_Executable_Fingerprint(&f1)) == 0 && taken(g_api->PJRT_LoadedExecutable_Fingerprint(&f2)) == 0 &&
               std::string(f1.executable_fingerprint, f1.executable_fingerprint_size) ==
                   std::string(f2.executable_fingerprint, f2.executable_fingerprint_size));
  ARGS(PJRT_Executable_OutputMemoryKinds_Args, omk);
  omk.executable = ge.executable;
  STEP(43, taken(g_api->PJRT_Executable_OutputMemoryKinds(&omk)) == 0 && omk.num_outputs >= 1 &&
               std::string(omk.memory_kinds[0], omk.memory_kind_sizes[0]) == "device");
  ARGS(PJRT_Executable_GetCostAnalysis_Args, ca);
  ca.executable = ge.executable;
  STEP(44, taken(g_api->PJRT_Executable_GetCostAnalysis(&ca)) == 0 && ca.num_properties == 0);
  ARGS(PJRT_Executable_Serialize_Args, ser);
  ser.executable = ge.executable;
  STEP(45, taken(g_api->PJRT_Executable_Serialize(&ser)) == (int)PJRT_Error_Code_UNIMPLEMENTED);
  {   // the program comes back as it went in: size query first, then the bytes
    PJRT_Program prog;
    memset(&prog, 0, sizeof(prog));
    prog.struct_size = PJRT_Program_STRUCT_SIZE;
    ARGS(PJRT_Executable_OptimizedProgram_Args, opg);
    opg.executable = ge.executable;
    opg.program = &prog;
    STEP(50, taken(g_api->PJRT_Executable_OptimizedProgram(&opg)) == 0 && prog.code_size > 0 &&
                 std::string(prog.format, prog.format_size) == "mlir");
    std::vector<char> text(prog.code_size);
    prog.code = text.data();
    STEP(51, taken(g_api->PJRT_Executable_OptimizedProgram(&opg)) == 0 &&
                 std::string(text.data(), text.size()).find("func.func") != std::string::npos);
    ARGS(PJRT_LoadedExecutable_AddressableDeviceLogicalIds_Args, lids);
    lids.executable = le;
    STEP(52, taken(g_api->PJRT_LoadedExecutable_AddressableDeviceLogicalIds(&lids)) == 0 &&
                 lids.num_addressable_device_logical_ids == 1 && lids.addressable_device_logical_ids[0].replica == 0 &&
                 lids.addressable_device_logical_ids[0].partition == 0);
  }
  {   // the device assignment, decoded field by field: one replica of one computation, on device 0
    ARGS(PJRT_LoadedExecutable_GetDeviceAssignment_Args, da);
    da.executable = le;
    STEP(53, taken(g_api->PJRT_LoadedExecutable_GetDeviceAssignment(&da)) == 0 && da.serialized_bytes &&
                 da.serialized_device_assignment_deleter);
    const unsigned char* p = reinterpret_cast<const unsigned char*>(da.serialized_bytes);
    const unsigned char* end = p + da.serialized_bytes_size;
    long replicas = -1, computations = -1, devices = 0, first_id = -1;
    auto varint = [&](const unsigned char*& q, const unsigned char* lim) {
      unsigned long v = 0;
      for (int shift = 0; q < lim; shift += 7) {
        const unsigned char c = *q++;
        v |= (unsigned long)(c & 0x7F) << shift;
        if (!(c & 0x80)) break;
      }
      return (long)v;
    };
    bool well_formed = true;
    while (p < end && well_formed) {
      const long key = varint(p, end);
      if (key == ((1 << 3) | 0)) replicas = varint(p, end);
      else if (key == ((2 << 3) | 0)) computations = varint(p, end);
      else if (key == ((3 << 3) | 2)) {
        const long len = varint(p, end);
        const unsigned char* sub_end = p + len;
        well_formed = sub_end <= end;
        while (well_formed && p < sub_end) {
          const long sub = varint(p, sub_end);
          if (sub != ((1 << 3) | 2)) { well_formed = false; break; }
          const long n = varint(p, sub_end);
          const unsigned char* ids_end = p + n;
          well_formed = ids_end <= sub_end;
          while (well_formed && p < ids_end) {
            const long id = varint(p, ids_end);
            if (devices++ == 0) first_id = id;
          }
        }
      } else well_formed = false;
    }
    STEP(54, well_formed && replicas == 1 && computations == 1 && devices == 1 && first_id == 0);
    da.serialized_device_assignment_deleter(da.serialized_device_assignment);
  }
  ARGS(PJRT_Executable_Destroy_Args, xd);
  xd.executable = ge.executable;
  STEP(46, taken(g_api->PJRT_Executable_Destroy(&xd)) == 0);
  ARGS(PJRT_ExecuteContext_Create_Args, cc);
  STEP(47, taken(g_api->PJRT_ExecuteContext_Create(&cc)) == 0 && cc.context);
  ARGS(PJRT_ExecuteContext_Destroy_Args, cdx);
  cdx.context = cc.context;
  STEP(48, taken(g_api->PJRT_ExecuteContext_Destroy(&cdx)) == 0);
  ARGS(PJRT_Device_MemoryStats_Args, ms);
  ms.device = g_device;
  STEP(49, taken(g_api->PJRT_Device_MemoryStats(&ms)) == 0 && !ms.bytes_limit_is_set);
  g_error.clear();
  return 0;
}

// Marks the executable deleted (it stays a valid handle that refuses to run).
int pjrt_harness_executable_delete(int exe) {
  NEED_OPEN();
  if (exe < 0 || exe >= (int)g_exes.size() || !g_exes[exe]) return harness_failure("no such executable");
  ARGS(PJRT_LoadedExecutable_Delete_Args, d);
  d.executable = g_exes[exe];
  if (int rc = taken(g_api->PJRT_LoadedExecutable_Delete(&d))) return rc;
  ARGS(PJRT_LoadedExecutable_IsDeleted_Args, q);
  q.executable = g_exes[exe];
  if (int rc = taken(g_api->PJRT_LoadedExecutable_IsDeleted(&q))) return rc;
  return q.is_deleted ? 0 : harness_failure("still reported alive");
}

// How many members of PJRT_Api (function pointers) the plugin left null.
int pjrt_harness_null_entries() {
  if (!g_api) return harness_failure("no plugin is open");
  const size_t first = offsetof(PJRT_Api, PJRT_Error_Destroy);
  int nulls = 0;
  for (size_t off = first; off + sizeof(void*) <= PJRT_Api_STRUCT_SIZE && off + sizeof(void*) <= g_api->struct_size;
       off += sizeof(void*)) {
    void* p;
    memcpy(&p, reinterpret_cast<const char*>(g_api) + off, sizeof(p));
    if (!p) ++nulls;
  }
  return nulls;
}

}  // extern "C"

// Default binding of the device-operations table: libtcpxu_hip.so, found next to this library.
#include <dlfcn.h>

#include <string>

#include "plugin_internal.h"

namespace tcpx {
namespace {

tcpxDeviceOps g_hip_ops;
void* g_hip_lib = nullptr;

std::string own_directory() {
  Dl_info info;
  if (dladdr(reinterpret_cast<void*>(&default_device_ops), &info) && info.dli_fname) {
    std::string p(info.dli_fname);
    const size_t slash = p.rfind('/');
    if (slash != std::string::npos) return p.substr(0, slash + 1);
  }
  return "";
}

template <typename Fn>
bool bind(Fn* slot, const char* name) {
  *slot = reinterpret_cast<Fn>(dlsym(g_hip_lib, name));
  if (!*slot) WARN("libtcpxu_hip.so does not export %s", name);
  return *slot != nullptr;
}

}  // namespace

const tcpxDeviceOps* default_device_ops() {
  if (g_hip_lib) return &g_hip_ops;
  const std::string path = own_directory() + "libtcpxu_hip.so";
  g_hip_lib = dlopen(path.c_str(), RTLD_NOW | RTLD_GLOBAL);
  if (!g_hip_lib) g_hip_lib = dlopen("libtcpxu_hip.so", RTLD_NOW | RTLD_GLOBAL);
  if (!g_hip_lib) {
    WARN("cannot load the HIP layer %s: %s", path.c_str(), dlerror());
    return nullptr;
  }
  bool ok = true;
  ok &= bind(&g_hip_ops.device_count, "tcpxuDeviceCount");
  ok &= bind(&g_hip_ops.arena_create, "tcpxuArenaCreate");
  ok &= bind(&g_hip_ops.arena_destroy, "tcpxuArenaDestroy");
  ok &= bind(&g_hip_ops.mapped_alloc, "tcpxuMappedAlloc");
  ok &= bind(&g_hip_ops.mapped_free, "tcpxuMappedFree");
  ok &= bind(&g_hip_ops.device_alloc, "tcpxuDeviceAlloc");
  ok &= bind(&g_hip_ops.device_free, "tcpxuDeviceFree");
  ok &= bind(&g_hip_ops.copy_to_device, "tcpxuCopyToDevice");
  ok &= bind(&g_hip_ops.engine_create, "tcpxuEngineCreate");
  ok &= bind(&g_hip_ops.engine_start, "tcpxuEngineStart");
  ok &= bind(&g_hip_ops.engine_stop, "tcpxuEngineStop");
  ok &= bind(&g_hip_ops.engine_destroy, "tcpxuEngineDestroy");
  ok &= bind(&g_hip_ops.engine_submit, "tcpxuEngineSubmit");
  ok &= bind(&g_hip_ops.engine_submit_sized, "tcpxuEngineSubmitSized");
  ok &= bind(&g_hip_ops.last_error, "tcpxuLastError");
  ok &= bind(&g_hip_ops.visible_alloc, "tcpxuVisibleAlloc");
  ok &= bind(&g_hip_ops.visible_free, "tcpxuVisibleFree");
  ok &= bind(&g_hip_ops.visible_flush, "tcpxuVisibleFlush");
  if (!ok) {
    dlclose(g_hip_lib);
    g_hip_lib = nullptr;
    return nullptr;
  }
  return &g_hip_ops;
}

ncclResult_t device_result(int rc, const char* what) {
  if (rc == TCPXU_SUCCESS) return ncclSuccess;
  WARN("%s failed with %d: %s", what, rc, (g.ops && g.ops->last_error) ? g.ops->last_error() : "");
  // A failing device call maps to the "unhandled device error" code, as CUCHECK does
  // (src/misc/cuda_checks.h:38-49); other codes pass through with their ncclResult_t value.
  return static_cast<ncclResult_t>(rc);
}

}  // namespace tcpx

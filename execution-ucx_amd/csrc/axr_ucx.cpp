// The part of a real UCX backend that can be built and tested without UCX headers: find
// libucp at run time, resolve the entry points the tensor-bundle path would call, and say
// clearly what is missing.  The reference links UCX at build time and calls
//   ucp_init / ucp_worker_create            ucx_am_context.cpp:694-749
//   ucp_mem_map / ucp_mem_unmap             ucx_am_context.cpp:1128-1147 (register_ucx_memory)
//   ucp_am_send_nbx                         ucx_connection.cpp:353-374, 401-426
//   ucp_am_recv_data_nbx                    ucx_connection.cpp:376-399, 428-453
//   ucp_worker_progress                     ucx_am_context.cpp:218-296
// Their parameter structures (ucp_params_t, ucp_mem_map_params_t, ucp_request_param_t) come
// from ucp.h, which this build does not have: nothing here restates them, so nothing beyond
// ucp_get_version (three unsigned out-parameters) is ever called.
#include <dlfcn.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>

#include "axr_internal.h"

using namespace axr;

namespace {

const char* const kSymbols[AXR_UCX_SYMBOLS] = {"ucp_init_version", "ucp_worker_create", "ucp_mem_map",
                                               "ucp_am_send_nbx",  "ucp_am_recv_data_nbx", "ucp_worker_progress"};

struct UcxLibrary {
  std::mutex mu;
  bool probed = false;
  axr_ucx_probe_t result;
  void* handle = nullptr;
  void* entry[AXR_UCX_SYMBOLS] = {};
};
UcxLibrary& ucx_library() {
  static UcxLibrary lib;
  return lib;
}

void probe_locked(UcxLibrary& lib) {
  axr_ucx_probe_t& r = lib.result;
  std::memset(&r, 0, sizeof(r));
  const char* override_path = std::getenv("AXR_UCX_LIBRARY");
  const char* candidates[] = {override_path, "libucp.so.0", "libucp.so"};
  std::string tried;
  for (const char* name : candidates) {
    if (!name || !*name) continue;
    lib.handle = dlopen(name, RTLD_NOW | RTLD_LOCAL);
    if (lib.handle) {
      std::snprintf(r.library, sizeof(r.library), "%s", name);
      break;
    }
    const char* why = dlerror();
    tried += std::string(tried.empty() ? "" : "; ") + name + ": " + (why ? why : "not found");
    if (name == override_path) break;   // a library named explicitly is the only one tried
  }
  if (!lib.handle) {
    std::snprintf(r.message, sizeof(r.message), "no UCX library could be loaded (%s)", tried.c_str());
    return;
  }
  typedef void (*get_version_fn)(unsigned*, unsigned*, unsigned*);
  if (auto get_version = reinterpret_cast<get_version_fn>(dlsym(lib.handle, "ucp_get_version")))
    get_version(&r.version_major, &r.version_minor, &r.version_release);
  int found = 0;
  std::string missing;
  for (int i = 0; i < AXR_UCX_SYMBOLS; ++i) {
    lib.entry[i] = dlsym(lib.handle, kSymbols[i]);
    r.have_symbol[i] = lib.entry[i] ? 1 : 0;
    found += r.have_symbol[i];
    if (!lib.entry[i]) missing += std::string(missing.empty() ? "" : ", ") + kSymbols[i];
  }
  r.available = found == AXR_UCX_SYMBOLS ? 1 : 0;
  if (r.available)
    std::snprintf(r.message, sizeof(r.message), "%s loaded, UCX %u.%u.%u, every entry point present", r.library,
                  r.version_major, r.version_minor, r.version_release);
  else
    std::snprintf(r.message, sizeof(r.message), "%s loaded but lacks: %s", r.library, missing.c_str());
}

}  // namespace

extern "C" {

static int ucx_probe_body(axr_ucx_probe_t* out) {
  if (!out) return fail(AXR_ERR_INVALID, "axr_ucx_probe: null result");
  UcxLibrary& lib = ucx_library();
  std::lock_guard<std::mutex> lock(lib.mu);
  if (!lib.probed) {
    probe_locked(lib);
    lib.probed = true;
  }
  *out = lib.result;
  return AXR_OK;
}
int axr_ucx_probe(axr_ucx_probe_t* out) {
  return guarded([&] { return ucx_probe_body(out); });
}

const char* axr_ucx_symbol_name(int index) {
  return index >= 0 && index < AXR_UCX_SYMBOLS ? kSymbols[index] : "";
}

static int am_context_create_ucx_body(const char* name, axr_am_context_t** ctx) {
  (void)name;
  if (!ctx) return fail(AXR_ERR_INVALID, "axr_am_context_create_ucx: null result");
  *ctx = nullptr;
  axr_ucx_probe_t probe;
  int rc = ucx_probe_body(&probe);
  if (rc) return rc;
  if (!probe.available)
    return fail(AXR_ERR_UNSUPPORTED, std::string("axr_am_context_create_ucx: ") + probe.message +
                                         "; use axr_am_context_create (the in-process loopback context)");
  return fail(AXR_ERR_UNSUPPORTED,
              std::string("axr_am_context_create_ucx: ") + probe.message +
                  ", but this build was made without ucp.h: the parameter structures of ucp_init_version, "
                  "ucp_mem_map and ucp_am_send_nbx are not known to it, so no UCX call beyond ucp_get_version "
                  "is made; use axr_am_context_create (the in-process loopback context)");
}
int axr_am_context_create_ucx(const char* name, axr_am_context_t** ctx) {
  return guarded([&] { return am_context_create_ucx_body(name, ctx); });
}

}  // extern "C"

// ABI version and per-thread error text of libmesh_moe_hip.so.
#include <stdarg.h>

#include "common.h"

namespace mesh_moe {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

}  // namespace mesh_moe

extern "C" int mesh_moe_abi_version(void) { return MESH_MOE_ABI_VERSION; }

extern "C" const char* mesh_moe_last_error(void) { return mesh_moe::g_error; }

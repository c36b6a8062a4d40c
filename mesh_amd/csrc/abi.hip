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

// CRC-32C (Castagnoli, reflected polynomial 0x82f63b78), eight bytes per step
// from eight tables; host code, no GPU work.
namespace {

struct Crc32cTables {
  uint32_t t[8][256];
  Crc32cTables() {
    for (uint32_t i = 0; i < 256; ++i) {
      uint32_t c = i;
      for (int k = 0; k < 8; ++k) c = (c >> 1) ^ ((c & 1u) ? 0x82f63b78u : 0u);
      t[0][i] = c;
    }
    for (uint32_t i = 0; i < 256; ++i)
      for (int j = 1; j < 8; ++j)
        t[j][i] = (t[j - 1][i] >> 8) ^ t[0][t[j - 1][i] & 0xffu];
  }
};

}  // namespace

extern "C" uint32_t mesh_moe_crc32c(uint32_t crc, const void* data, size_t n) {
  static const Crc32cTables tables;
  const auto& t = tables.t;
  const uint8_t* p = static_cast<const uint8_t*>(data);
  uint32_t c = ~crc;
  while (n > 0 && (reinterpret_cast<uintptr_t>(p) & 7u) != 0) {
    c = (c >> 8) ^ t[0][(c ^ *p++) & 0xffu];
    --n;
  }
  for (; n >= 8; n -= 8, p += 8) {
    uint64_t w;
    memcpy(&w, p, 8);
    w ^= c;
    c = t[7][w & 0xff] ^ t[6][(w >> 8) & 0xff] ^ t[5][(w >> 16) & 0xff] ^
        t[4][(w >> 24) & 0xff] ^ t[3][(w >> 32) & 0xff] ^
        t[2][(w >> 40) & 0xff] ^ t[1][(w >> 48) & 0xff] ^ t[0][w >> 56];
  }
  for (; n > 0; --n) c = (c >> 8) ^ t[0][(c ^ *p++) & 0xffu];
  return ~c;
}

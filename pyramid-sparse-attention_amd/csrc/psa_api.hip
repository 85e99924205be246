// Library-level entry points: version, error string, pooled-buffer geometry.
#include <stdarg.h>

#include "psa_common.h"

static thread_local char g_err[512] = "";

void psa_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

int psa_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    psa_set_error("%s: %s", what, hipGetErrorString(e));
    return PSA_ERR_LAUNCH;
  }
  return PSA_OK;
}

extern "C" int psa_version(void) { return 100; }

extern "C" const char* psa_last_error(void) { return g_err; }

static int64_t npad_of(int L, int block_n) { return (int64_t)((L + block_n - 1) / block_n) * block_n; }

extern "C" int64_t psa_pool_elems(int B, int Hkv, int L, int D, int block_n) {
  if (B <= 0 || Hkv <= 0 || L <= 0 || D <= 0 || block_n <= 0) return 0;
  return (int64_t)B * Hkv * D * (npad_of(L, block_n) / 8) * 7;
}

extern "C" int64_t psa_pool_level_offset(int B, int Hkv, int L, int D, int block_n, int level) {
  if (B <= 0 || Hkv <= 0 || L <= 0 || D <= 0 || block_n <= 0) return -1;
  int64_t per = (int64_t)B * Hkv * D * (npad_of(L, block_n) / 8);  // elements of level 8
  switch (level) {
    case 2: return 0;
    case 4: return per * 4;
    case 8: return per * 6;
    default: return -1;
  }
}

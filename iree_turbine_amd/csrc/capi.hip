// Error plumbing and introspection entry points of the C ABI.
#include "common.hpp"
#include <string.h>

namespace mi355 {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* kernel, dim3 grid, dim3 block, size_t lds) {
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) return 0;
  set_error("%s: launch failed, grid=(%u,%u,%u) block=(%u,%u,%u) lds=%zu: %s", kernel, grid.x, grid.y, grid.z, block.x,
            block.y, block.z, lds, hipGetErrorString(e));
  return (int)e;
}

int gemm_variant_count();
const char* gemm_variant_name(int i);
int fa_variant_count();
const char* fa_variant_name(int i);
int decode_variant_count();
const char* decode_variant_name(int i);
int mxfp4_variant_count();
const char* mxfp4_variant_name(int i);
int mxfp8_variant_count();
const char* mxfp8_variant_name(int i);
int mxfp6_variant_count();
const char* mxfp6_variant_name(int i);

}  // namespace mi355

using namespace mi355;

extern "C" int mi355_abi_version(void) { return MI355_ABI_VERSION; }

// The timing-only ablations this library was built with (common.hpp), "" for the product build.
extern "C" const char* mi355_build_flags(void) {
  return ""
#if defined(MI355_ABLATE_NO_LOADS)
         " NO_LOADS"
#endif
#if defined(MI355_ABLATE_L1_LOADS)
         " L1_LOADS"
#endif
#if defined(MI355_ABLATE_NO_LOAD_WAITS)
         " NO_LOAD_WAITS"
#endif
#if defined(MI355_ABLATE_NO_BARRIERS)
         " NO_BARRIERS"
#endif
#if defined(MI355_ABLATE_PLAIN_LOAD_ORDER)
         " PLAIN_LOAD_ORDER"
#endif
#if defined(MI355_ABLATE_NO_SCALE_READS)
         " NO_SCALE_READS"
#endif
#if defined(MI355_ABLATE_NO_SCALE_LOADS)
         " NO_SCALE_LOADS"
#endif
#if defined(MI355_ABLATE_NO_A_LOADS)
         " NO_A_LOADS"
#endif
#if defined(MI355_ABLATE_NO_STORES)
         " NO_STORES"
#endif
#if defined(MI355_ABLATE_NO_EXP)
         " NO_EXP"
#endif
#if defined(MI355_ABLATE_NO_K_READS)
         " NO_K_READS"
#endif
#if defined(MI355_ABLATE_NO_V_READS)
         " NO_V_READS"
#endif
      ;
}
extern "C" const char* mi355_last_error(void) { return g_error; }

extern "C" int mi355_variant_count(const char* family) {
  if (!family) return 0;
  if (!strcmp(family, "gemm_f16_nt")) return gemm_variant_count();
  if (!strcmp(family, "flash_attn_fwd")) return fa_variant_count();
  if (!strcmp(family, "paged_decode")) return decode_variant_count();
  if (!strcmp(family, "mxfp4_gemm")) return mxfp4_variant_count();
  if (!strcmp(family, "mxfp8_gemm")) return mxfp8_variant_count();
  if (!strcmp(family, "mxfp6_gemm")) return mxfp6_variant_count();
  return 0;
}

extern "C" const char* mi355_variant_name(const char* family, int i) {
  if (!family) return nullptr;
  if (!strcmp(family, "gemm_f16_nt")) return gemm_variant_name(i);
  if (!strcmp(family, "flash_attn_fwd")) return fa_variant_name(i);
  if (!strcmp(family, "paged_decode")) return decode_variant_name(i);
  if (!strcmp(family, "mxfp4_gemm")) return mxfp4_variant_name(i);
  if (!strcmp(family, "mxfp8_gemm")) return mxfp8_variant_name(i);
  if (!strcmp(family, "mxfp6_gemm")) return mxfp6_variant_name(i);
  return nullptr;
}

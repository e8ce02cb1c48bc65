// Error state and version queries of libparoatten_hip.
#include "paro_common.hpp"

namespace paro {
static thread_local char g_err[512] = "";
void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}
}  // namespace paro

// 2: the measurement aids (paro_diag_*) left this library for one of their own; entry points were added
// (paro_rope_k_mean_permute_quant_fwd, paro_v_f16_pack, ...), no remaining signature changed
extern "C" int paro_abi_version(void) { return 2; }
extern "C" const char* paro_last_error(void) { return paro::g_err; }
extern "C" const char* paro_build_arch(void) { return "gfx950"; }

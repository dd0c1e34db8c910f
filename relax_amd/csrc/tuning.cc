// The test hooks of include/relax_amd_wq_testing.h: work-split overrides of the calling thread.
#include "tuning.h"

#include "../../include/relax_amd_wq_testing.h"

namespace wq {

Tuning& tuning() {
  static thread_local Tuning t;
  return t;
}

}  // namespace wq

extern "C" void wq_debug_set_gemm_config(int cfg) { wq::tuning().gemm_cfg = cfg; }
extern "C" void wq_debug_set_gemm_tail_split(int on) { wq::tuning().gemm_tail_split = on; }
extern "C" void wq_debug_set_gemv_config(int rows, int gpl) {
  wq::tuning().gemv_rows = rows;
  wq::tuning().gemv_gpl = gpl;
}
extern "C" void wq_debug_set_gemv_blocks_per_cu(int n) { wq::tuning().gemv_blocks_per_cu = n; }
extern "C" void wq_debug_set_skinny_config(int nw, int stages, int waves) {
  wq::tuning().skinny_nw = nw;
  wq::tuning().skinny_stages = stages;
  wq::tuning().skinny_waves = waves;
}
extern "C" void wq_debug_set_intb_gemv_k_split(int ways) { wq::tuning().intb_k_split = ways; }

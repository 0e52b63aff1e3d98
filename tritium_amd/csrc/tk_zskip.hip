// gfx950 decode kernel, 32x32x32 form, for launches in which some plane carries a zero-chunk map: the instantiations
// of tk_flow32_kernel (tk_flow.h, ZMAP) that fetch marked chunks from the plane's resident all-zero chunk instead of
// from memory. They live in a translation unit of their own so that the plain forms keep their code and their
// register budgets untouched (the 16x16x64 kernel decides at run time; there the look-up is scalar and free). Both
// operand orders (cfg.swap: weights first, the int8 contract's).
// Compiled with -ffp-contract=off like every kernel whose epilogue must round as the CPU does.

#include "tk_flow.h"

template <int P, int RT2, bool SWAP>
static hipError_t zmap_flow32_pr(hipStream_t s, const TkProblem &sg, const TkProblem *table, const int *wg_prob,
                                 const TkLaunchCfg &cfg) {
  const int threads = cfg.waves * 64;
  switch (cfg.ring) {
    case 2:
      if (table) return flow_launch_one(tk_flow32_kernel<P, RT2, 2, true, true, SWAP>, s, sg, table, wg_prob, cfg, threads);
      return flow_launch_one(tk_flow32_kernel<P, RT2, 2, false, true, SWAP>, s, sg, table, wg_prob, cfg, threads);
    case 3:
      if (table) return flow_launch_one(tk_flow32_kernel<P, RT2, 3, true, true, SWAP>, s, sg, table, wg_prob, cfg, threads);
      return flow_launch_one(tk_flow32_kernel<P, RT2, 3, false, true, SWAP>, s, sg, table, wg_prob, cfg, threads);
    case 4:
      if (table) return flow_launch_one(tk_flow32_kernel<P, RT2, 4, true, true, SWAP>, s, sg, table, wg_prob, cfg, threads);
      return flow_launch_one(tk_flow32_kernel<P, RT2, 4, false, true, SWAP>, s, sg, table, wg_prob, cfg, threads);
    default: return hipErrorInvalidValue;
  }
}

template <int P>
static hipError_t zmap_flow32_p(hipStream_t s, const TkProblem &sg, const TkProblem *table, const int *wg_prob,
                                const TkLaunchCfg &cfg) {
  switch (cfg.rt) {
    case 2: return cfg.swap ? zmap_flow32_pr<P, 1, true>(s, sg, table, wg_prob, cfg) : zmap_flow32_pr<P, 1, false>(s, sg, table, wg_prob, cfg);
    case 4: return cfg.swap ? zmap_flow32_pr<P, 2, true>(s, sg, table, wg_prob, cfg) : zmap_flow32_pr<P, 2, false>(s, sg, table, wg_prob, cfg);
    default: return hipErrorInvalidValue;
  }
}

hipError_t tk_launch_flow32_zmap(hipStream_t s, const TkProblem *single, const TkProblem *table, const int *wg_prob,
                                 const TkLaunchCfg &cfg) {
  if (!cfg.grid) return hipSuccess;
  if (!cfg.wide_mfma) return hipErrorInvalidValue;
  TkProblem dummy = {};
  const TkProblem &sg = single ? *single : dummy;
  switch (cfg.planes) {
    case 1: return zmap_flow32_p<1>(s, sg, table, wg_prob, cfg);
    case 2: return zmap_flow32_p<2>(s, sg, table, wg_prob, cfg);
    default: return hipErrorInvalidValue;
  }
}

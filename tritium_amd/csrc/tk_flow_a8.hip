// gfx950 decode kernel, both matrix-instruction forms, second operand order (tk_flow.h, SWAP): the instantiations that
// launches under the int8 contract take. Weights are the first operand of the matrix instruction and activations the second, so a lane
// finishes four consecutive output channels of one token and writes them with one store. A translation unit of its own:
// the first-order forms (float contract, single-launch form that builds its rows) keep their code and register budgets.
// Compiled with -ffp-contract=off like every kernel whose epilogue must round as the CPU does.

#include "tk_flow.h"

template <int P, int RT, int TW>
static hipError_t swapped_tw(hipStream_t s, const TkProblem &sg, const TkProblem *table, const int *wg_prob,
                             const TkLaunchCfg &cfg) {
  const int threads = cfg.waves * 64;
  switch (cfg.ring) {
    case 2:
      if (table) return flow_launch_one(tk_flow_kernel<P, RT, TW, 2, true, false, true>, s, sg, table, wg_prob, cfg, threads);
      return flow_launch_one(tk_flow_kernel<P, RT, TW, 2, false, false, true>, s, sg, table, wg_prob, cfg, threads);
    case 3:
      if (table) return flow_launch_one(tk_flow_kernel<P, RT, TW, 3, true, false, true>, s, sg, table, wg_prob, cfg, threads);
      return flow_launch_one(tk_flow_kernel<P, RT, TW, 3, false, false, true>, s, sg, table, wg_prob, cfg, threads);
    case 4:
      if (table) return flow_launch_one(tk_flow_kernel<P, RT, TW, 4, true, false, true>, s, sg, table, wg_prob, cfg, threads);
      return flow_launch_one(tk_flow_kernel<P, RT, TW, 4, false, false, true>, s, sg, table, wg_prob, cfg, threads);
    case 5:
      if (table) return flow_launch_one(tk_flow_kernel<P, RT, TW, 5, true, false, true>, s, sg, table, wg_prob, cfg, threads);
      return flow_launch_one(tk_flow_kernel<P, RT, TW, 5, false, false, true>, s, sg, table, wg_prob, cfg, threads);
    default: return hipErrorInvalidValue;
  }
}

template <int P, int RT>
static hipError_t swapped_pr(hipStream_t s, const TkProblem &sg, const TkProblem *table, const int *wg_prob,
                             const TkLaunchCfg &cfg) {
  constexpr int TW = ((RT >= 4 && P <= 2) || (RT == 2 && P == 1)) ? 2 : 1;  // runs per wave: as the first-order launcher
  if constexpr (P <= 2 && RT == 1) {
    if (cfg.tw == 2) return swapped_tw<P, RT, 2>(s, sg, table, wg_prob, cfg);
    return swapped_tw<P, RT, 1>(s, sg, table, wg_prob, cfg);
  } else {
    return swapped_tw<P, RT, TW>(s, sg, table, wg_prob, cfg);
  }
}

template <int P>
static hipError_t swapped_p(hipStream_t s, const TkProblem &sg, const TkProblem *table, const int *wg_prob,
                            const TkLaunchCfg &cfg) {
  switch (cfg.rt) {
    case 1: return swapped_pr<P, 1>(s, sg, table, wg_prob, cfg);
    case 2: return swapped_pr<P, 2>(s, sg, table, wg_prob, cfg);
    case 4: return swapped_pr<P, 4>(s, sg, table, wg_prob, cfg);
    default: return hipErrorInvalidValue;
  }
}

// 32x32x32 form, weights first
template <int P, int RT2>
static hipError_t swapped32_pr(hipStream_t s, const TkProblem &sg, const TkProblem *table, const int *wg_prob,
                               const TkLaunchCfg &cfg) {
  const int threads = cfg.waves * 64;
  switch (cfg.ring) {
    case 2:
      if (table) return flow_launch_one(tk_flow32_kernel<P, RT2, 2, true, false, true>, s, sg, table, wg_prob, cfg, threads);
      return flow_launch_one(tk_flow32_kernel<P, RT2, 2, false, false, true>, s, sg, table, wg_prob, cfg, threads);
    case 3:
      if (table) return flow_launch_one(tk_flow32_kernel<P, RT2, 3, true, false, true>, s, sg, table, wg_prob, cfg, threads);
      return flow_launch_one(tk_flow32_kernel<P, RT2, 3, false, false, true>, s, sg, table, wg_prob, cfg, threads);
    case 4:
      if (table) return flow_launch_one(tk_flow32_kernel<P, RT2, 4, true, false, true>, s, sg, table, wg_prob, cfg, threads);
      return flow_launch_one(tk_flow32_kernel<P, RT2, 4, false, false, true>, s, sg, table, wg_prob, cfg, threads);
    default: return hipErrorInvalidValue;
  }
}

template <int P>
static hipError_t swapped32_p(hipStream_t s, const TkProblem &sg, const TkProblem *table, const int *wg_prob,
                              const TkLaunchCfg &cfg) {
  switch (cfg.rt) {
    case 2: return swapped32_pr<P, 1>(s, sg, table, wg_prob, cfg);
    case 4: return swapped32_pr<P, 2>(s, sg, table, wg_prob, cfg);
    default: return hipErrorInvalidValue;
  }
}

hipError_t tk_launch_flow_swapped(hipStream_t s, const TkProblem *single, const TkProblem *table, const int *wg_prob,
                                  const TkLaunchCfg &cfg) {
  if (!cfg.grid) return hipSuccess;
  if (cfg.fused || cfg.base3 || (cfg.wide_mfma && cfg.zmap32)) return hipErrorInvalidValue;  // (maps + 32x32x32: tk_launch_flow32_zmap)
  TkProblem dummy = {};
  const TkProblem &sg = single ? *single : dummy;
  if (cfg.wide_mfma) {
    switch (cfg.planes) {
      case 1: return swapped32_p<1>(s, sg, table, wg_prob, cfg);
      case 2: return swapped32_p<2>(s, sg, table, wg_prob, cfg);
      default: return hipErrorInvalidValue;
    }
  }
  switch (cfg.planes) {
    case 1: return swapped_p<1>(s, sg, table, wg_prob, cfg);
    case 2: return swapped_p<2>(s, sg, table, wg_prob, cfg);
    case 3: return swapped_p<3>(s, sg, table, wg_prob, cfg);
    case 4: return swapped_p<4>(s, sg, table, wg_prob, cfg);
    default: return hipErrorInvalidValue;
  }
}

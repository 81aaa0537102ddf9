// One translation unit of a tile engine's kernels and launch sequences
// (tlce_host.h).  Compiled several times with different definitions:
//   TLCE_UNIT_ENGINE  the engine type, e.g. MfmaDirect4Engine<__bf16>
//   TLCE_UNIT_PART    0: everything of that engine in one unit (engines whose
//                        kernels compile quickly);
//                     1..5: one kernel family (forward statistics, logit-gradient
//                        panels without soft cap and bias, gradient contractions,
//                        KL panels, float32 logits panels), 7..9: the other
//                        logit-gradient variants (soft cap, bias, both),
//                        10, 11: the forward statistics and the logit-gradient
//                        panels over a head stored [h, v],
//                        12: the exponentiated-logits panel of the forward that
//                        leaves the gradients (with TLCE_UNIT_FUSED, which also adds
//                        that sequence to part 6: the bf16 direct engine only),
//                        6: the launch sequences over them.
#include "tlce_host.h"
#include "tlce_fused.h"

#ifndef TLCE_UNIT_ENGINE
#error "define TLCE_UNIT_ENGINE and TLCE_UNIT_PART (see turbo_dllm_amd/build.py)"
#endif

namespace tlce {

using UnitEngine = TLCE_UNIT_ENGINE;

#if TLCE_UNIT_PART == 0
TLCE_ENGINE_ENTRY_POINTS(template, UnitEngine)
#else
#if TLCE_UNIT_PART == 1
TLCE_LAUNCHERS_FORWARD(template, UnitEngine)
#else
TLCE_LAUNCHERS_FORWARD(extern template, UnitEngine)
#endif
#if TLCE_UNIT_PART == 2
TLCE_LAUNCHERS_GRAD_LOGITS(template, UnitEngine, false, false)
#else
TLCE_LAUNCHERS_GRAD_LOGITS(extern template, UnitEngine, false, false)
#endif
#if TLCE_UNIT_PART == 7
TLCE_LAUNCHERS_GRAD_LOGITS(template, UnitEngine, true, false)
#else
TLCE_LAUNCHERS_GRAD_LOGITS(extern template, UnitEngine, true, false)
#endif
#if TLCE_UNIT_PART == 8
TLCE_LAUNCHERS_GRAD_LOGITS(template, UnitEngine, false, true)
#else
TLCE_LAUNCHERS_GRAD_LOGITS(extern template, UnitEngine, false, true)
#endif
#if TLCE_UNIT_PART == 9
TLCE_LAUNCHERS_GRAD_LOGITS(template, UnitEngine, true, true)
#else
TLCE_LAUNCHERS_GRAD_LOGITS(extern template, UnitEngine, true, true)
#endif
#if TLCE_UNIT_PART == 3
TLCE_LAUNCHERS_GEMM(template, UnitEngine)
#else
TLCE_LAUNCHERS_GEMM(extern template, UnitEngine)
#endif
#if TLCE_UNIT_PART == 4
TLCE_LAUNCHERS_KL(template, UnitEngine)
#else
TLCE_LAUNCHERS_KL(extern template, UnitEngine)
#endif
#if TLCE_UNIT_PART == 5
TLCE_LAUNCHERS_LOGITS(template, UnitEngine)
#else
TLCE_LAUNCHERS_LOGITS(extern template, UnitEngine)
#endif
#if TLCE_UNIT_PART == 10
TLCE_LAUNCHERS_FORWARD_DIM_FIRST(template, UnitEngine)
#else
TLCE_LAUNCHERS_FORWARD_DIM_FIRST(extern template, UnitEngine)
#endif
#if TLCE_UNIT_PART == 11
TLCE_LAUNCHERS_GRAD_LOGITS_DIM_FIRST(template, UnitEngine)
#else
TLCE_LAUNCHERS_GRAD_LOGITS_DIM_FIRST(extern template, UnitEngine)
#endif
#ifdef TLCE_UNIT_FUSED   // the engine the forward that leaves the gradients is built for
#if TLCE_UNIT_PART == 12
TLCE_LAUNCHERS_EXP_PANEL(template, UnitEngine)
#else
TLCE_LAUNCHERS_EXP_PANEL(extern template, UnitEngine)
#endif
#endif
#if TLCE_UNIT_PART == 6
TLCE_ENGINE_ENTRY_POINTS(template, UnitEngine)
#ifdef TLCE_UNIT_FUSED
TLCE_FUSED_ENTRY_POINTS(template, UnitEngine)
#endif
#endif
#endif

}  // namespace tlce

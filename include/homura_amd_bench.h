/* Measurement and test-support entry points of libhomura_amd.so. They are not part of the drop-in
 * boundary (include/homura_amd.h): nothing here has a counterpart in the reference's FFI. */
#ifndef HOMURA_AMD_BENCH_H
#define HOMURA_AMD_BENCH_H

#include "homura_amd.h"

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default)

/* Phase trace of the latest whole-step decode launch: device-clock ticks (100 MHz) taken by workgroup
 * 0 at 11 points per layer (both workgroup barriers of the Q|K|V, attention, O, gate|up and down
 * phases; the end of the fold follows attention's second barrier) and one at the end of the kernel, then
 * a word that is 1 when the step found its workgroups dealt round-robin to the dies and used die-local
 * exchanges. The first call switches recording on and stores 0 in *n_out; later calls copy
 * layers * 11 + 2 entries of the step that ran last. */
int hm_model_whole_step_trace(hm_model *m, unsigned long long *h_out, int cap, int *n_out);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif

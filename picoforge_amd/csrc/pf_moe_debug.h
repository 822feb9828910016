/* Diagnostic entry points of libpicoforge_moe.so: for the library's tests and measuring programs, not part of the
 * boundary (include/pf_moe_hip.h), and nothing a forward loop calls. */
#pragma once
#include "../../include/pf_moe_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Tests: route every batch size through the general kernels (on != 0) instead of the specialised ones. */
void pf_hip_work_force_general(PfHipWork *work, int on);

/* Every later forward on this workspace enqueues only the first `count` of its dependent kernel groups (decode
 * path: its kernels; other paths: four groups; 0 = all; results are then incomplete).  A measuring program times
 * the chain cut after 1, 2, ... groups and takes differences. */
void pf_hip_work_limit_kernels(PfHipWork *work, int count);

/* A workspace created while PF_WORK_GUARD=1 is in the environment has 4096 bytes of a fixed pattern behind each
 * of its buffers.  Returns PF_HIP_OK with *damaged = the number of guards that no longer hold the pattern
 * (0 also for a workspace without guards) and *first = the index of the first such buffer, in the order of the
 * workspace's layout. */
int pf_hip_work_check_guards(PfHipWork *work, int *damaged, int *first);

#ifdef __cplusplus
}
#endif

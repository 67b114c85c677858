/* C ABI of liborion_policy.so: the scheduler's dispatch policy with no GPU
 * dependency.  It lets a CPU-only host replay the observation log of a run and
 * check the dispatch-decision sequence, and parse profile files the way the
 * scheduler does.
 *
 * Reference counterparts (eth-easl/orion):
 *   policy ........ Scheduler::busy_wait_profile, schedule_reef,
 *                   schedule_sequential (src/scheduler/scheduler_eval.cpp:93-487)
 *   profile files . populate_kernel_info (src/scheduler/scheduler_eval.cpp:498-526)
 * The reference has no replay entry point; its policy is only reachable through
 * schedule() on a live GPU.
 */
#ifndef ORION_POLICY_H_
#define ORION_POLICY_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Replays an observation log (text, format in orion_amd/csrc/policy/obslog.h)
 * through the policy.  On success returns 0 and stores a malloc'd decision log
 * in *decisions_out.  On a malformed log or a divergence returns 2 and stores
 * a malloc'd message in *error_out.  Free either with orion_policy_free.
 * sequential_fix != 0 selects the repaired time-slicing rule (the reference's
 * schedule_sequential, scheduler_eval.cpp:185-223, cannot dispatch once a
 * client is past its tenth iteration). */
int orion_policy_replay(const char* observations, int sequential_fix,
                        char** decisions_out, char** error_out);
/* The same replay; the decision log carries a line "P" before the decisions
 * of every logged poll, so that decisions can be read poll by poll beside the
 * observation log's P lines (one iteration of the loop at
 * scheduler_eval.cpp:277-302 each). */
int orion_policy_replay_by_poll(const char* observations, int sequential_fix,
                                char** decisions_out, char** error_out);
void orion_policy_free(char* p);

/* populate_kernel_info + the max-SM scan of setup (scheduler_eval.cpp:498-526,
 * :595-598): row count, max(SM_usage) starting from 0, and the sum of the fp32
 * durations accumulated in double.  Returns 0, or 2 with *error_out set. */
int orion_profile_stats(const char* path, int* rows, int* max_sm_used,
                        double* duration_sum, char** error_out);

/* One parsed row (0-based, header excluded).  Returns 0, 1 if out of range,
 * 2 if the file does not parse. */
int orion_profile_row(const char* path, int row, char* name, size_t name_cap,
                      int* profile, int* mem, int* sm_used, float* duration);

/* CU-mask slot for a best-effort record (no reference counterpart).  masks are
 * ascending CU counts, the last one the whole GPU.  -1 for records that are not
 * kernels (rec_class != 0).  With the high-priority client idle (hp_active ==
 * 0) the whole GPU, or the largest partial mask for a kernel whose profiled
 * duration alone exceeds the best-effort duration budget (long_kernel != 0);
 * with a request in flight the smallest mask holding sm_used, never the whole
 * GPU when a partial mask exists.  algo: 0 orion, 1 reef, 2 sequential (the
 * latter two always use the last slot). */
int orion_place_cu_slot(const int* masks, int n_masks, int rec_class,
                        int sm_used, int algo, int hp_active, int long_kernel);

#ifdef __cplusplus
}
#endif
#endif /* ORION_POLICY_H_ */

/* C ABI of scheduler_eval.so and of the control calls of libinttemp.so: the
 * drop-in boundary of the scheduling hot path.  Names, argument order and
 * meaning are those the reference's Python frontend binds through ctypes
 * (src/scheduler_frontend.py:13,60,72,78,85,91) and its client loops call
 * (benchmarking/benchmark_suite/train_imagenet.py:63-68,88).
 *
 * The reference passes Python bools as C ints and reads pointer results as
 * 32-bit ints (ctypes defaults); both work here because every bool parameter
 * is read from the low byte and the handle is never dereferenced.
 */
#ifndef ORION_SCHEDULER_H_
#define ORION_SCHEDULER_H_

#include <stdbool.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- scheduler_eval.so ------------------------------------------------- */

/* reference: sched_init, src/scheduler/scheduler_eval.cpp:491-495.
 * Returns an opaque token; all state is process-global. */
void* sched_init(void);

/* reference: setup, scheduler_eval.cpp:542-660.  The LAST client is the
 * high-priority one.  tids are the OS thread ids of the client threads; files
 * are profile CSVs (Name,Profile,Memory_footprint,SM_usage,Duration) with at
 * least num_kernels[i] rows.  Creates the streams (one spanning all CUs for
 * the high-priority client, one per CU-mask size for each best-effort client)
 * and starts routing the client threads' HIP calls through their queues.
 * Aborts with a message on an unreadable profile (the reference asserts).
 * Environment: ORION_BE_CU_MASKS (ascending CU counts, default
 * cus/8,cus/4,cus/2,cus), ORION_MAX_SMS (default: the device's CU count; the
 * reference hard-codes 80, scheduler_eval.cpp:20), ORION_RECORD_DIR (write
 * observations.log / decisions.log there), ORION_QUIET,
 * ORION_SEQUENTIAL_AS_WRITTEN, and the recorded policy options
 * ORION_CONFINE_LONG_BE, ORION_RESERVE_HP_CUS, ORION_ADMIT_OVERSIZED,
 * ORION_SLIDING_THROTTLE.
 * `models` decides one thing: with ORION_BE_RUN_AHEAD=1 only best-effort
 * clients named "gemm_bf16" or "triad_f32" queue records ahead of their
 * dispatch (see orion_client_deferred below). */
void setup(void* scheduler, int num_clients, int* tids, char** models,
           char** files, int* num_kernels, int* num_iters, bool* train,
           bool reef);

/* reference: setup_change, scheduler_eval.cpp:528-540: swap a client's profile
 * and kernel count (training clients after their first iteration). */
void setup_change(void* scheduler, int client_id, char* file, int num_kernels);

/* reference: schedule, scheduler_eval.cpp:663-670 -> busy_wait_profile
 * :238-487.  Blocks until every client has reached warmup_iters (warm-up) or
 * its iteration limit / has acknowledged a stop (measured run).  reef / seq
 * select the alternative policies; reef_depth is REEF's queue depth or, for
 * the Orion policy, the budget in ns of outstanding best-effort work.
 * Returns NULL.  After a call with warmup == false the client threads' HIP
 * calls pass straight through again. */
void* schedule(void* scheduler, int num_clients, bool profile_mode, int iter,
               bool warmup, int warmup_iters, bool reef, bool seq,
               int reef_depth, int hp_limit, int update_start);

/* reference: reset, scheduler_eval.cpp:672-675. */
void* reset(void* scheduler, int num_clients);

/* No reference counterpart: stream the scheduler created for a client (its
 * widest one), CU count in use, per-iteration wall times (ms) the scheduler
 * measured for a client (returns how many exist, copies at most cap), and
 * teardown of all scheduler state. */
void* orion_client_stream(int client);
int orion_sched_num_cus(void);
int orion_sched_iteration_ms(int client, float* out, int cap);
void orion_sched_teardown(void);

/* Profile capture (no reference counterpart; replaces the Nsight runs of
 * PROFILE.md:7-54).  orion_profile_begin routes the client thread `client_tid`
 * through the interception layer and opens the trace file; orion_profile_run
 * serves it alone, in order, timing every kernel with HIP events, until it has
 * completed `until_iteration` iterations (an iteration ends at block());
 * orion_profile_end stops routing and closes the trace.  Trace columns:
 * iteration,index,type,name,grid_x..z,block_x..z,dyn_lds,regs,static_lds,
 * duration_ns.  All return 0 on success. */
int orion_profile_begin(int client_tid, const char* trace_path);
int orion_profile_run(int until_iteration);
int orion_profile_end(void);

/* ---- libinttemp.so (LD_PRELOAD) ---------------------------------------- */

/* reference: block, src/cuda_capture/intercept_temp.cpp:124-130.  Called by a
 * client thread after submitting iteration `it`; returns when the scheduler
 * has seen all its kernels complete. */
void block(int it);

/* reference: stop, intercept_temp.cpp:132-141.  Non-zero once the scheduler
 * asked the calling client to stop (the high-priority client is done); the
 * call acknowledges it.  Returns int (the reference returns a C bool that its
 * caller reads as an int). */
int stop(void);

/* No reference counterpart (the reference patches PyTorch instead,
 * setup/orion-torch-changes.patch:779-803): tie the calling thread, or a
 * stream the calling client thread uses, to a client, so that work issued on
 * the client's behalf by other threads is routed to its queue. */
void orion_register_thread(int client);
void orion_register_stream(void* stream);
int orion_client_index(void);
/* The client a call naming `stream` from the calling thread would be queued
 * for; negative when the call would go straight to the runtime (reference
 * counterpart of the lookup: get_idx, src/cuda_capture/utils_interc.cpp:3-51). */
int orion_client_of_stream(void* stream);
/* With ORION_PIN_THREADS=1: the CPU the calling client or scheduler thread was
 * pinned to when it was first identified (reference: the sched_setaffinity of
 * get_idx, src/cuda_capture/utils_interc.cpp:36-49).  -1 when it is not pinned:
 * by default (threads are left to the kernel's placement, which measured
 * better on the hosts of these GPUs), with too few CPUs, or for a thread that
 * is no client.  The masks in force before are restored when the job ends. */
int orion_pinned_cpu(void);

/* No reference counterpart: while on, the calling thread's HIP calls bypass the
 * queues.  Client loops use it around model construction and library
 * auto-tuning, whose kernel count differs from run to run on ROCm and would
 * otherwise never match a profile's row count. */
void orion_thread_passthrough(int on);

/* No reference counterpart: how many records `client` has queued since the job
 * was set up, and how many of them it queued without waiting for their
 * dispatch.  The latter is zero unless ORION_BE_RUN_AHEAD=1 is set and setup()
 * was given "gemm_bf16" or "triad_f32" as the client's model name (clients made
 * of this library's own kernels; no other client is ever cleared for it): then
 * the best-effort client's kernel launches, device-to-device copies and fills
 * are queued with a deep copy of their arguments and the call returns at once
 * (hipSuccess, as every queued call of the reference returns:
 * intercept_temp.cpp:418-458), up to 64 records ahead of the scheduler.  By
 * default, and for every other client always, every record is handed over
 * synchronously, as in the reference (intercept_temp.cpp:404-416). */
unsigned long long orion_client_submitted(int client);
unsigned long long orion_client_deferred(int client);

/* No reference counterpart: with ORION_CALL_TIMING=1 in the environment, the
 * time the calling thread has spent so far inside the interposed kernel-launch
 * and hipMemcpyAsync entry points (from entry to return, the runtime's own
 * call included) and the number of such calls; both zero otherwise.  A client
 * loop uses the pair to split a request's submission time into time inside the
 * runtime and this library and time inside the framework. */
unsigned long long orion_thread_time_in_calls_ns(void);
unsigned long long orion_thread_calls(void);

/* No reference counterpart.  On glibc before 2.39 a thread's accesses to
 * thread-local variables of shared libraries (a framework makes dozens per
 * operator) take the dynamic loader's slow path for good once a library with
 * thread-local storage has been loaded or unloaded after the newest one the
 * thread has touched; a process that loads libraries lazily is in that state
 * from its first request on (measured on the ResNet-50 bs4 request: +0.25 to
 * +0.45 ms per request).  While a job runs the library keeps its client threads
 * out of that state by itself: it reloads a one-variable helper library
 * (liborion_tlsfresh.so, beside libinttemp.so) whenever the set of loaded
 * libraries has changed and has every client thread call into the fresh copy
 * once (ORION_TLS_REFRESH=0 switches that off).  orion_tls_fresh_check() does
 * the same for the calling thread on demand, for threads the library does not
 * schedule; orion_tls_fresh_stats() reports how many reloads and calls into a
 * fresh copy there have been. */
void orion_tls_fresh_check(void);
void orion_tls_fresh_stats(unsigned long long* reloads, unsigned long long* touches);

#ifdef __cplusplus
}
#endif
#endif /* ORION_SCHEDULER_H_ */

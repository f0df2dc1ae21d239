/* hpx_sched.h: C ABI of the task scheduler that sits on top of the codecs of hpx.h.
 *
 * It replaces the layer between the reference's Python module and its kernel
 * drivers: Task / TaskQueue / FinishQueue / ThreadManager (hp_cuda.h:28-148),
 * the four RunLoopOnceFor* batch builders (hp_cuda.cpp:163-772), the B <-> C
 * staging copies they issue, and init / end / submit_task / getResults
 * (hp_cuda.cpp:824-1066).  Signatures use plain pointers and sizes; the torch
 * extension csrc/hp_cuda_module.cpp (and torch-hipress-extension_amd/hp_cuda.py
 * over ctypes) puts the reference's torch-tensor interface
 * (hp_cuda.cpp:1073-1080) on top and keeps the tensors alive while a task is in
 * flight.
 *
 * What is kept: task ids, the grouping of one batch's tasks into multi-tensor
 * codec calls and their order (per algorithm, see hpx_sched.cpp), which
 * finished queue a task's name appears in, the fixed GradDrop transfer size
 * 4 + 8*ceil(N*(1-drop_ratio)) (hp_cuda.cpp:230), root tasks decoding every
 * gathered slot but their own rank's and then re-encoding.
 * What is different: one worker thread that sleeps on a condition variable
 * (the reference polls five queues every 500 us, one for TBQ); staging copies
 * run on a data stream ordered against the compute stream by events; a batch's
 * transfers and codec calls are cut into runs (1 MB of messages, then 2, 4 ...
 * 16 MB; GradDrop: one run) so that one run's transfer overlaps the next run's
 * kernels, all messages of a run in ONE kernel launch that reads or writes the
 * pinned host buffers directly (through a pinned bounce buffer when the caller's
 * host tensor is pageable) instead of one copy call per message; a name is
 * published once its own run's copy has landed rather than at fixed points of
 * the batch; HIP errors are counted and kept (hpx_sched_error) instead of ignored;
 * a task whose buffers are too small for its message is skipped and counted as
 * a failure (the reference overruns them), and its name is still published.
 */
#ifndef HPX_SCHED_H_
#define HPX_SCHED_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* hp_cuda.h:21-26 */
#define HPX_COMP_TASK 10
#define HPX_DECOMP_TASK 20
#define HPX_ROOT_DECOMP_COMP_TASK 30
#define HPX_POWERSGD_ENCODE1 40
#define HPX_POWERSGD_ENCODE2 50
#define HPX_POWERSGD_DECODE 60

/* One unit of work (the reference's Task, hp_cuda.h:28-51).  Device pointers:
 * tensor, residual, B, M, P, Q.  Host pointer: C.  All memory is the caller's
 * and must stay valid until the task's serial comes back from
 * hpx_sched_take_done. */
typedef struct hpx_task {
  const char* name;        /* copied */
  int32_t task_id;
  int32_t is_root;         /* 0 or 1; decoders add into `tensor` when 1 */
  float* tensor;           /* gradient */
  int64_t tensor_numel;
  float* residual;         /* NULL where the algorithm has none (TernGrad) */
  int64_t residual_numel;
  uint8_t* B;              /* device message buffer */
  int64_t B_bytes;
  uint8_t* C;              /* host message buffer; `size` slots of one message each for a root task */
  int64_t C_bytes;
  float* M;                /* PowerSGD: n x m */
  float* P;                /* n x r */
  float* Q;                /* m x r */
  int32_t n, m, r;
} hpx_task_t;

/* Replaces init (hp_cuda.cpp:824-874).  alg is "terngrad", "tbq", "graddrop" or
 * "powersgd"; parameters are (key, value) pairs with the reference's keys
 * (enable_random, bitwidth | threshold | drop_ratio, sample_rate |
 * matrix_approximation_rank) plus the optional key "seed", which fixes the RNG
 * seed of every TernGrad / GradDrop encode (the reference reads the clock).
 * Starts the worker thread on `device`.  Returns 0, or -3 for an unknown
 * algorithm (the reference prints and returns false), -2 for a HIP error.
 * Calling it again while running re-reads the parameters and keeps the thread,
 * as the reference does (hp_cuda.cpp:814). */
int hpx_sched_init(const char* alg, const char* const* keys, const double* values, int nparams,
                   int device, int rank, int size);

/* Replaces end (hp_cuda.cpp:883-890): finishes the queued tasks, stops and joins
 * the worker, frees streams and staging memory.  Finished names stay readable. */
int hpx_sched_end(void);

/* Replaces submit_task (three overloads, hp_cuda.cpp:936-1041).  Checks what the
 * reference checks (is_root in {0,1}; task id valid for the algorithm family;
 * worker running) and returns -3 with the reference's message in
 * hpx_sched_error() otherwise.  *serial receives a number that identifies the
 * task in hpx_sched_take_done. */
int hpx_sched_submit(const hpx_task_t* task, uint64_t* serial);

/* Replaces getResults (hp_cuda.cpp:1043-1066): pops names of finished tasks of
 * the queue that `task_id` maps to (10/40, 20/60, 30/50) into buf as consecutive
 * NUL-terminated strings, as many as fit in `cap` bytes, and returns how many
 * (names that do not fit stay queued).  -3 for an id that maps to no queue. */
int64_t hpx_sched_get_results(int task_id, char* buf, int64_t cap);

/* No counterpart in the reference (its callers poll getResults): waits until the
 * queue that `task_id` maps to is non-empty or timeout_ms has passed.  Returns 1
 * if it is non-empty, 0 on timeout, -3 for a bad id. */
int hpx_sched_wait(int task_id, int timeout_ms);

/* Serials of tasks the scheduler is done with (their buffers are no longer
 * touched): up to `cap`, returns how many.  The holder of the tensors drops its
 * references on these. */
int64_t hpx_sched_take_done(uint64_t* serials, int64_t cap);

/* Number of codec / HIP failures since init, and the text of the last one. */
int64_t hpx_sched_error_count(void);
const char* hpx_sched_error(void);

#ifdef __cplusplus
}
#endif
#endif /* HPX_SCHED_H_ */

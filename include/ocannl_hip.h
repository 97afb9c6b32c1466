/* ocannl_hip.h -- C ABI of the MI355X (gfx950) arrayjit backend for OCANNL.
 *
 * This is the surface an OCaml `Hip_backend : Backend_impl.Lowered_backend` binds through ctypes;
 * it replaces what the CUDA backend gets from the external `cudajit` package plus the CUDA
 * backend's own compile/link/launch code.  Every entry point cites the reference interface it
 * stands behind (paths relative to the OCANNL tree).
 *
 * Conventions
 *   - every function returns 0 on success or a negative OCANNL_HIP_E_* code; the message for the
 *     calling thread's last failure is ocannl_hip_last_error().  The OCaml stub maps
 *     E_USER -> Utils.User_error, E_INVALID -> Invalid_argument, the rest -> Failure
 *     (arrayjit/lib/cuda_backend.ml:1017-1035 uses exactly this split).
 *   - one FIFO stream per device (arrayjit/lib/backend_intf.ml:262-265); every call makes its
 *     device current first (cuda_backend.ml:56 `set_ctx`).
 *   - buffers are named by (pool_id, byte offset): Backend_intf.buffer_loc
 *     (arrayjit/lib/backend_intf.ml:7-16); the pool_id -> base table is private to the library
 *     (cuda_backend.ml:60-94).
 *   - host memory passed to from_host/to_host is caller-owned and must stay valid until the
 *     caller's next ocannl_hip_await on that device (arrayjit/lib/context.ml:338-343,389).
 *   - all calls come from one host thread at a time.
 */
#ifndef OCANNL_HIP_H
#define OCANNL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OCANNL_HIP_OK 0
#define OCANNL_HIP_E_USER (-1)     /* Utils.User_error: bad static index, unsupported precision ... */
#define OCANNL_HIP_E_INVALID (-2)  /* Invalid_argument: misuse of the interface, malformed IR      */
#define OCANNL_HIP_E_RUNTIME (-3)  /* Failure: HIP / hiprtc error                                  */

/* Size of the library's static device scratch array (see ocannl_hip_routine_run_static_scratch). */
#define OCANNL_HIP_STATIC_SCRATCH_BYTES (32ull << 20)

typedef struct ocannl_hip_device ocannl_hip_device;    /* (dev, runner) of one ordinal            */
typedef struct ocannl_hip_event ocannl_hip_event;      /* Lowered_backend.event                   */
typedef struct ocannl_hip_code ocannl_hip_code;        /* Lowered_backend.code / code_batch       */
typedef struct ocannl_hip_routine ocannl_hip_routine;  /* the linked launch closure (Task.t work) */

/* Backend_intf.buffer_loc for one tensor node (backend_intf.ml:7-18: ctx_buffers entries). */
typedef struct {
  int32_t node_id;
  int32_t pool_id;
  uint64_t offset;   /* bytes */
} ocannl_hip_node_loc;

/* Kparam description (Backend_intf.kparam_source, backend_intf.ml:41-57). */
typedef struct {
  int32_t kind;        /* 0 = Kparam_ptr, 1 = Static_idx, 2 = Merge_buffer */
  int32_t id;          /* node id or static symbol                       */
  int64_t size_bytes;  /* Kparam_ptr: padded node size; Static_idx: range or -1 */
} ocannl_hip_kparam;

/* One device kernel of a compiled routine, for measurement and debugging. */
typedef struct {
  int32_t kind;            /* 0 = generated pointwise/reduction kernel, 1 = fill, 2 = MFMA contraction */
  int32_t coop_lanes;      /* lanes cooperating on one output (generated reduction kernels)          */
  double flops;            /* algorithmic: 2 * product of all loop extents for a contraction         */
  double bytes;            /* algorithmic: distinct elements read once + written once, in bytes      */
  int64_t m, n, k, batch;  /* contraction shape after symbol classification (0 otherwise); contractions
                              sharing the launch count as batch entries, a chain of operand pairs into
                              one result as a longer k                                                 */
  char name[96];
  int32_t queue;           /* 0 = the device's main queue; 1 = its side queue: a contraction off the critical
                              path that runs beside the kernels that follow it (compile option side_queue=1|2;
                              without it every kernel reports 0) */
  int32_t reserved;
} ocannl_hip_kernel_info;

const char* ocannl_hip_last_error(void);

/* ---- devices: Backend_device_common (backend_intf.ml:206-266) ------------------------------- */
/* Cu.init + lazy per-device set-up (cuda_backend.ml:113-118,215-238). Idempotent. */
int ocannl_hip_init(void);
int ocannl_hip_num_devices(int* count);                                  /* num_devices, :258    */
int ocannl_hip_get_device(int ordinal, ocannl_hip_device** dev);         /* get_device, :257     */
int ocannl_hip_get_name(ocannl_hip_device* dev, char* buf, size_t cap);  /* Device.get_name, :204 */
int ocannl_hip_static_properties(char* buf, size_t cap);   /* static_properties sexp, :231; cuda_backend.ml:1092-1112 */
int ocannl_hip_get_used_memory(ocannl_hip_device* dev, uint64_t* bytes); /* get_used_memory, :239 */
int ocannl_hip_get_debug_info(ocannl_hip_device* dev, char* buf, size_t cap); /* get_debug_info, :244 */
/* get_global_debug_info (backend_intf.ml:242; the CUDA backend's reports its live streams,
   cuda_backend.ml:1088-1090): a sexp of process-wide counters -- live devices (one stream each), events,
   compiled codes, linked routines, routines compiled, hiprtc modules built, routines rebuilt without
   16-byte accesses for a context at element-aligned offsets, runs enqueued, pools and their bytes. */
int ocannl_hip_get_global_debug_info(char* buf, size_t cap);
int ocannl_hip_await(ocannl_hip_device* dev);                            /* await, :247          */
int ocannl_hip_is_idle(ocannl_hip_device* dev, int* idle);               /* is_idle, :254        */

/* ---- events (backend_intf.ml:221-251; cuda_backend.ml:108-111) ------------------------------- */
int ocannl_hip_all_work(ocannl_hip_device* dev, ocannl_hip_event** ev);  /* all_work             */
int ocannl_hip_sync(ocannl_hip_event* ev);                               /* sync                 */
int ocannl_hip_is_done(ocannl_hip_event* ev, int* done);                 /* is_done              */
int ocannl_hip_will_wait_for(ocannl_hip_device* dev, ocannl_hip_event* ev); /* will_wait_for     */
void ocannl_hip_event_free(ocannl_hip_event* ev);

/* ---- Slab_alloc (backend_intf.ml:22-37; cuda_backend.ml:60-94) ------------------------------- */
/* Allocating an existing pool_id frees the old slab first (merge-buffer regrowth, :71-76). */
int ocannl_hip_alloc_pool(ocannl_hip_device* dev, int pool_id, uint64_t size_in_bytes, uint64_t alignment);
int ocannl_hip_free_pool(ocannl_hip_device* dev, int pool_id);
int ocannl_hip_memset_zero(ocannl_hip_device* dev, int pool_id, uint64_t offset, uint64_t size_in_bytes);

/* ---- copies: No_buffer_retrieval_or_syncing (arrayjit/lib/backend_impl.ml:292-314) ----------- */
/* Asynchronous on the device stream (cuda_backend.ml:267-287). */
int ocannl_hip_from_host(ocannl_hip_device* dst, int pool_id, uint64_t offset, const void* src, uint64_t bytes);
int ocannl_hip_to_host(ocannl_hip_device* src, int pool_id, uint64_t offset, void* dst, uint64_t bytes);
/* Same-device or peer copy (cuda_backend.ml:289-314); dst_pool_id < 0 means "into the merge buffer of dst",
   which is (re)grown to `bytes` as pool 0 (cuda_backend.ml:130-134). */
int ocannl_hip_device_to_device(ocannl_hip_device* dst, int dst_pool_id, uint64_t dst_offset,
                                ocannl_hip_device* src, int src_pool_id, uint64_t src_offset, uint64_t bytes);

/* ---- compile / link / run (backend_impl.ml:347-367) ------------------------------------------ */
/* Lowered_backend.compile / compile_batch: `llir` is the serialised Low_level.optimized of one or
   more routines (name, static indices, node table, statement tree).  Splits each routine into
   kernels, maps large `+*` contractions to the MFMA kernels, generates HIP for the rest and
   compiles it with hiprtc for gfx950.  Needs no GPU. */
int ocannl_hip_compile(const char* llir, size_t len, ocannl_hip_code** code);
/* Same, with "key=value;..." options: mfma=0|1 (matrix-core kernels for contractions), coop=0|1
   (lanes sharing reductions; off = the summation order of the serial C code), rows=0|1 (fusing
   consecutive row-wise phases into one kernel), bf16_copies=0|1 (rounding an fp32 operand of a
   bf16 contraction once into scratch instead of in every kernel that reads it), serial=0|1 (a routine
   of tiny phases as one single-workgroup kernel), groups=0|1 (independent contractions of identical
   shapes share a launch), chains=0|1 (`c =+ a * b` statements into one result with identical operand
   shapes share a launch), parallel=0|1 (consecutive small phases that do not depend on one another
   run side by side in one launch), graphs=0|1 (a routine's
   kernels are captured into a HIP graph per combination of static-index values and replayed as one unit
   by ocannl_hip_routine_run; off by default), debug_log=0|1 (in-routine logging, see
   ocannl_hip_routine_log_id; the wire form then carries every Set's text), side_queue=0|1|2 (contractions
   whose results nothing needs for a while -- weight gradients -- run on a second queue of the device, beside
   the kernels that follow; 2: generated kernels of a few MB as well; off by default), epilogues=0|1 (`y := x + bias` and `z := relu(y)` right behind the
   contraction that produces x run in that contraction's epilogue), fused=0|1|2 (a short-K contraction whose only reader is the row-wise
   kernel that follows -- attention scores ahead of the soft-max chain -- runs on the matrix cores as that
   kernel's prologue, into LDS, instead of as a launch of its own; 2: also when its result is a context
   node that has to be stored anyway), proj=0|1 (a contraction over the row position whose operand such a
   kernel produces -- attention weights times V -- runs as that kernel's epilogue on the 32 rows the
   workgroup holds in LDS), row_waves=4|8|16 (waves per workgroup of those kernels), row_vec=0|1 (a lane
   takes runs of four neighbouring row positions; off), group_window=<n> (how many phases apart
   contractions may be and still share a launch), reuse=0|1 (a later sub-expression that spells out again what
   an earlier statement stored -- the reference's optimiser inlines a tensor into every reader at the
   assigned position, low_level.ml:496-552 -- reads the stored tensor instead; on), min_mfma_flops=<n>, large_models=0|1 (64-bit loop
   indices and offsets in generated kernels, the `large_models` setting of c_syntax.ml:111-112; a
   routine with a node of more than 2^31 - 1 elements gets them without asking). */
int ocannl_hip_compile_opts(const char* llir, size_t len, const char* options, ocannl_hip_code** code);
/* Drops the caller's reference.  Routines linked from the code keep what they need alive (the launch
   closure's context_lifetime, cuda_backend.ml:1046-1051), so code_free before routine_free is fine. */
void ocannl_hip_code_free(ocannl_hip_code* code);
int ocannl_hip_code_num_routines(ocannl_hip_code* code, int* n);
int ocannl_hip_code_routine_name(ocannl_hip_code* code, int index, char* buf, size_t cap);
/* The kparam list of routine `index` (c_syntax.ml:1046-1084): pass params=NULL to query the count. */
int ocannl_hip_code_kparams(ocannl_hip_code* code, int index, ocannl_hip_kparam* params, int cap, int* count);
/* Generated HIP source (the `.hip` dump under output_debug_files_in_build_directory). */
int ocannl_hip_code_source(ocannl_hip_code* code, char* buf, size_t cap, size_t* needed);
/* The gfx950 code object hiprtc built for routine `index` (its generated kernels; empty for a routine
   made of matrix-core launches and fills only): the `.ptx` dump of cuda_backend.ml:193-202 under
   output_debug_files_in_build_directory.  An ELF file: `llvm-objdump -d` prints its ISA.  Pass
   buf = NULL to query the size. */
int ocannl_hip_code_object(ocannl_hip_code* code, int index, char* buf, size_t cap, size_t* needed);
int ocannl_hip_code_num_kernels(ocannl_hip_code* code, int index, int* n);
int ocannl_hip_code_kernel_info(ocannl_hip_code* code, int index, int kernel, ocannl_hip_kernel_info* info);

/* Lowered_backend.link (backend_impl.ml:355; cuda_backend.ml:983-1066): loads the module on `dev`,
   resolves every Kparam_ptr through `locs` (the resulting context's ctx_buffers), allocates the
   routine-private scratch for `Local` nodes.  Missing nodes raise E_USER (cc_backend.ml:411-415).
   Offsets need only be aligned to the node's element size, as Backends.plan_pool_segments packs them
   (arrayjit/lib/backends.ml:22-51): when an operand of a matrix-core kernel sits at an offset that is
   not 16-byte aligned, the routine is linked in a second form, built on first need, in which
   generated kernels do that work element by element (slower; same results within tolerance). */
int ocannl_hip_link(ocannl_hip_device* dev, ocannl_hip_code* code, int index, const ocannl_hip_node_loc* locs,
                    int n_locs, ocannl_hip_routine** routine);
void ocannl_hip_routine_free(ocannl_hip_routine* routine);
/* lowered_bindings: the `int ref` behind a Static_idx (arrayjit/lib/indexing.ml:60-93). */
int ocannl_hip_routine_set_static(ocannl_hip_routine* routine, int symbol, int64_t value);
/* Task.run of the launch closure (cuda_backend.ml:991-1044): range-checks static indices
   (E_USER on failure, :1015-1030), binds the merge buffer for a routine that reads one (pool 0 as it
   is now, :1009-1011; E_USER when no transfer has filled it or it is smaller than the merge node),
   then enqueues the routine's kernels on the device stream. */
int ocannl_hip_routine_run(ocannl_hip_routine* routine);
/* No counterpart in the reference.  For callers that cannot allocate device memory (code under HIP
   graph capture, tight serving loops, harnesses that forbid hipMalloc): ocannl_hip_routine_run with
   the routine's scratch memory -- `Local` nodes, tensors the planner materialises, the split-K
   workspace of the MFMA kernels -- taken from a static device array of
   OCANNL_HIP_STATIC_SCRATCH_BYTES that belongs to the loaded library (one copy per GPU, held until
   the process ends) instead of the arena that link allocated.  Inputs and outputs are the context
   nodes the routine was linked against, as for routine_run.  Calls no hipMalloc / hipFree / event or
   other allocating routine; zero fills run as kernels, not memsets.  A routine whose scratch needs
   exceed the array is refused with E_USER.  Every call on a GPU shares that GPU's array, which keeps
   the previous call's contents (nothing in it needs to start at zero: every routine fills what it
   reads); calls that overlap on one GPU -- other than in order on the device's one stream -- race. */
int ocannl_hip_routine_run_static_scratch(ocannl_hip_routine* routine);
/* debug_log_from_routines (arrayjit/lib/utils.ml:591; c_syntax.ml:493-535; cuda_backend.ml:871-893,992-1041):
   a routine compiled with the option debug_log=1 prints, from the device, what every statement
   computes: `<log id>: # <statement>$` and `<log id>: lhs[offset]{=old} = new = expression{=values}$`
   (`$` stands for a newline, as in the CUDA backend), comments as `<log id>: COMMENT: text$`, in program
   order -- such a routine runs every top-level statement as ONE thread.  The lines go to the process's
   standard output when the device is next synchronised; this returns the id of the routine's latest
   run, the prefix by which the host picks its lines out (Utils.add_log_processor ~prefix). */
int ocannl_hip_routine_log_id(ocannl_hip_routine* routine, int* log_id);
/* Same, bracketing every kernel with HIP events on the device stream; synchronises and writes the
   per-kernel milliseconds (cap >= number of kernels).  For measurement only. */
int ocannl_hip_routine_run_timed(ocannl_hip_routine* routine, float* kernel_ms, int cap);

/* Measurement inside a timed region: also bracket kernel `kernel_index` of every following
   ocannl_hip_routine_run with HIP events on the device stream, without synchronising; may be called
   for several kernels, -1 clears the selection. */
int ocannl_hip_routine_profile_kernel(ocannl_hip_routine* routine, int kernel_index);
/* Synchronises, returns the summed duration and the number of bracketed launches since the last read. */
int ocannl_hip_routine_profile_read(ocannl_hip_routine* routine, double* total_ms, int64_t* launches);

#ifdef __cplusplus
}
#endif
#endif /* OCANNL_HIP_H */

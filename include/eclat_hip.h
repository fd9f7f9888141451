/* C ABI of libeclat_hip: the MI355X (gfx950) kernel backend for the eclat tensor compiler.
 *
 * These entry points are what a `crates/backend-hip` in the reference workspace binds to
 * implement the reference's backend traits; each group cites the trait methods it stands for
 * (paths relative to the reference repository).  All functions are thread-safe, return 0 on
 * success and a non-zero EH_ERR_* code otherwise; eh_last_error() then gives the message of the
 * calling thread's most recent failure.  Handles are opaque.  No function takes or returns a
 * framework tensor type: only plain pointers, sizes and NUL-terminated strings.
 *
 * Kernel ASTs travel as text, e.g.
 *   (program (kernel "E_4_0" (params ("buf0" (ptr f32 global) imm normal) ...) (grid ...) (tg ...)
 *     (range "ridx0" (const i64 0) (const i64 1) (const i64 4) (store (var "buf4") ... ) sequential)))
 * one s-expression per reference `AstNode` variant (src/ast/mod.rs:107-385).
 */
#ifndef ECLAT_HIP_H
#define ECLAT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define EH_OK 0
#define EH_ERR_INVALID 1   /* bad argument / handle */
#define EH_ERR_PARSE 2     /* malformed AST text or options */
#define EH_ERR_UNSUPPORTED 3
#define EH_ERR_COMPILE 4   /* hiprtc rejected generated or given source */
#define EH_ERR_DEVICE 5    /* HIP runtime error, or no device */
#define EH_ERR_SIZE 6      /* buffer size mismatch */

typedef struct eh_device eh_device;
typedef struct eh_buffer eh_buffer;
typedef struct eh_program eh_program;   /* one or more launches compiled from a Program AST */
typedef struct eh_graph eh_graph;       /* one execute of a program on fixed buffers, replayable */
typedef struct eh_plan eh_plan;         /* rendered sources + dispatch, no device involved */
typedef struct eh_event eh_event;
typedef struct eh_module eh_module;     /* one entry point of a loaded code object */

/* ---- library ---------------------------------------------------------------------------- */
int eh_version(void);                   /* 100 * major + minor */
const char* eh_last_error(void);        /* valid until the calling thread's next failing call */
void eh_free(void* p);                  /* releases memory handed out by eh_compile_source and eh_normalize_ast */

/* ---- BackendRegistry: kind/name/is_available/list_devices/create_device
 *      (src/backend/device.rs:83-131), Device::profile (src/backend/traits.rs:273-306) ------- */
typedef struct eh_device_props {
  char name[128];
  char arch[32];                        /* "gfx950" */
  int compute_units;
  int warp_size;                        /* 64 */
  int max_work_group_size;
  size_t local_memory_size;             /* LDS bytes per compute unit */
  size_t global_memory_size;
  int clock_khz;
  int memory_clock_khz;
  int memory_bus_bits;
  int l2_bytes;
} eh_device_props;

int eh_device_count(int* count);        /* 0 devices is not an error */
int eh_device_open(int index, eh_device** out);
int eh_device_close(eh_device* dev);    /* buffers and programs of the device must be gone */
int eh_device_get_props(eh_device* dev, eh_device_props* out);
int eh_device_sync(eh_device* dev);     /* waits for everything queued on the device's stream */
/* The device's stream (a hipStream_t), for callers that order their own work against the library's
 * or capture its launches into a graph of their own (eh_program_execute_static with sync == 0
 * between hipStreamBeginCapture and hipStreamEndCapture on this stream).  No counterpart in the
 * reference, whose devices own their queues (src/backend/traits.rs:273-306). */
int eh_device_stream(eh_device* dev, void** stream);

/* ---- Buffer: allocate (zero-filled), byte_len, write_from_host (size must match exactly),
 *      read_to_host, clone_buffer (src/backend/traits.rs:455-482;
 *      crates/backend-c/src/buffer.rs:84-131); BackendRegistry::allocate_buffer
 *      (src/backend/device.rs:132-134) -------------------------------------------------------- */
/* A new buffer reads as zeros.  The fill is put off until the contents are needed (a kernel that
 * reads the buffer or writes part of it, a copy out of it, eh_buffer_device_ptr) and dropped
 * when a full write from the host or a launch that writes every element comes first: an output
 * the executor allocates per kernel costs no fill.
 * Released buffers' memory is kept by the device (up to a quarter of its memory) and reused by
 * later allocations of the same size, so the executor's allocate-per-kernel pattern
 * (src/backend/executor.rs:313-332) costs no hipMalloc/hipFree after the first pass.
 * eh_device_trim gives the kept blocks back to the driver; *kept_bytes (may be NULL) receives
 * how much was kept before.  ECLAT_HIP_NO_POOL in the environment turns the reuse off. */
int eh_device_trim(eh_device* dev, size_t* kept_bytes);
int eh_buffer_alloc(eh_device* dev, size_t bytes, eh_buffer** out);
int eh_buffer_retain(eh_buffer* buf);
int eh_buffer_release(eh_buffer* buf);
int eh_buffer_bytes(eh_buffer* buf, size_t* bytes);
int eh_buffer_write(eh_buffer* buf, const void* src, size_t bytes);
int eh_buffer_read(eh_buffer* buf, void* dst, size_t bytes);
int eh_buffer_copy(eh_buffer* dst, eh_buffer* src);        /* device-to-device, same size */
int eh_buffer_device_ptr(eh_buffer* buf, void** ptr);

/* ---- Renderer: AST -> source + dispatch sizes, no device needed
 *      (src/backend/renderer.rs:20-35; KernelSourceRenderer and extract_kernel_config,
 *      src/backend/pipeline.rs:27-33, 344-410).  `options` is NULL or "key=value,..." with keys
 *      arch, fuse, vectorize, transpose, window, row_threads, row_elems, flat_block, flat_iters, gemm, gemm_bm,
 *      gemm_bn, gemm_bk, gemm_wm, gemm_wn, gemm_split_k, gemm_waves, gemm_setprio, gemm_fold, gemm_window, window_passes,
 *      gemm_epilogue, gemm_dma, gemm_mix, gemm_prefetch, gemm_transpose, gemm_merge_batch, nontemporal,
 *      normalize, allow_serial, reindex, rematerialize, merge_launches, merge_templates, gemm_tail, guard_branches, ranged_loads,
 *      lanes, lane_us.
 *      merge_launches (default 1): launches of a program that do not depend on each other go out as one launch;
 *      merge_templates (default 1): so do small MFMA contractions among themselves (a layer's input and weight
 *      gradient), each a part of the launch that uses the launch's LDS in turn; gemm_tail (default 1): a pooling
 *      reduce over a convolution's stored result is computed by the convolution's workgroups from LDS.
 *      lanes (default 1; 2 or more): launches of a program that do not depend on each other are spread
 *      over that many streams (lane 0 is the device's stream; a program's execute forks the side
 *      lanes off it and joins them back, so callers still see one stream); launches estimated
 *      above lane_us microseconds (default 100) stay on lane 0.
 *      A kernel that no schedule recognises, would run in a single work-item and loops more than
 *      2^17 times is refused with EH_ERR_UNSUPPORTED unless allow_serial=1 (loops whose bounds move
 *      with enclosing loops count by their extreme; bounds that cannot be bounded count as too many).
 *      A large kernel that is planned one work-item per outer iteration because its loop structure
 *      was not recognised carries ",degraded" in its schedule string and is logged once. ------- */
typedef struct eh_launch_info {
  const char* entry;                    /* kernel symbol */
  const char* source;                   /* HIP C translation unit */
  const char* schedule;                 /* e.g. "row(T=256,V=4,NV=4,reg,rows/block=1)" */
  unsigned grid[3];                     /* workgroups */
  unsigned block[3];                    /* work-items per workgroup */
  unsigned lds_bytes;                   /* dynamic LDS */
  int n_args;                           /* pointer parameters, see eh_plan_launch_arg */
  int n_kernels;                        /* lowered kernels covered by this launch */
  double algo_bytes;                    /* each distinct external buffer counted once */
  double flops;                         /* 2*M*N*K for contractions, else 0 */
  int lane;                             /* 0: the device's stream; 1..: a side stream beside it */
  int n_waits;                          /* launches on other lanes this one waits for */
  unsigned long long tune_key;          /* what options for this launch alone are filed under (see ECLAT_HIP_TUNE below) */
} eh_launch_info;

int eh_render_program(const char* ast_text, const char* options, eh_plan** out);
/* Tuned options.  When the environment variable ECLAT_HIP_TUNE names a file, eh_render_program and
 * eh_program_compile look the program up in it and take the options filed there, with `options` on
 * top: one line per program, "<key as 16 hex digits> <key=value,...>", '#' starts a comment, the
 * last line for a key counts.  The key is what eh_tune_key returns for the program's AST text (the
 * FNV-1a hash of its canonical text), or a launch's key (eh_launch_info.tune_key: the same hash of the
 * first lowered kernel the launch covers): options under a launch's key apply to that launch alone,
 * in whatever program it turns up; in an options string the same is written "@<key>:name=value".
 * A file that cannot be read is reported on stderr once and ignored.  The
 * measured schedule search (python -m harp_amd.tune --save <file>) writes such lines.  It stands
 * where the reference's optimiser picks its rewrites by a static cost
 * (src/opt/ast/optimizer/beam_search.rs:34-66): here the choice is measured once and filed. */
int eh_tune_key(const char* ast_text, unsigned long long* key);
/* The program (or kernel) with the rewrites of the reference's AST optimiser undone where they are
 * recognised -- what eh_render_program and eh_program_compile plan from.  That optimiser runs
 * before any backend sees a kernel (pipeline.optimize, src/backend/executor.rs:169-176,
 * src/backend/compile.rs:246-265): shifts for multiplications by powers of two
 * (src/opt/ast/rules/bit_ops.rs:19-83), tiled loops with remainder loops or guards and unrolled
 * loops (src/opt/ast/transforms.rs:238-361, 393-630).  The result computes what the input
 * computes, statement for statement.  *out_text is AST text, released with eh_free. */
int eh_normalize_ast(const char* ast_text, char** out_text);
/* The local work size Pipeline::compile_ast derives from a kernel's dispatch hints
 * (src/backend/pipeline.rs:160-192 with compute_compatible_local_size, :475-489): per dimension the
 * largest divisor of global[i] that is at most preferred[i], then, while the three multiply to more
 * than max_work_group, the largest dimension steps down to the next smaller divisor of its global
 * size.  Kernels that carry their own dispatch (grid x thread group in the AST) are launched with
 * it: global = grid * thread group, workgroups = global / local.  Kernel::execute_with_sizes
 * (src/backend/traits.rs:556-566), whose sizes are global, divides by this too. */
int eh_fit_local_size(const size_t global[3], const size_t preferred[3], size_t max_work_group, size_t local[3]);
int eh_plan_num_launches(eh_plan* plan, int* n);
int eh_plan_launch(eh_plan* plan, int launch, eh_launch_info* out);    /* strings live as long as the plan */
int eh_plan_launch_arg(eh_plan* plan, int launch, int arg, const char** buffer_name);
int eh_plan_launch_kernel(eh_plan* plan, int launch, int k, const char** kernel_name);
/* Whether the launch writes the buffer of parameter `arg` (0 no, 1 yes, 2: every element of it,
 * given a buffer of exactly the kernel's output size: such a buffer need not hold anything
 * before), and launch number `i` (of n_waits) on another lane that must have finished before
 * this one starts.  Launches are listed in the order
 * in which they are issued; every launch a launch depends on comes before it. */
int eh_plan_launch_arg_written(eh_plan* plan, int launch, int arg, int* written);
int eh_plan_launch_wait(eh_plan* plan, int launch, int i, int* waited_launch);
int eh_plan_num_buffers(eh_plan* plan, int* n);
int eh_plan_buffer(eh_plan* plan, int i, const char** name, const char** role, size_t* bytes, int* elided);
int eh_plan_release(eh_plan* plan);

/* ---- Compiler: source -> code object with hiprtc for `arch` (NULL = gfx950), no device needed
 *      (Compiler::compile, src/backend/traits.rs:592-607; crates/backend-c/src/compiler.rs:101-165).
 *      *blob is released with eh_free. ----------------------------------------------------------- */
int eh_compile_source(const char* source, const char* arch, void** blob, size_t* len);

/* ---- BackendRegistry::compile_ast + Kernel (src/backend/device.rs:136-160;
 *      src/backend/traits.rs:531-587): compile a Program AST for a device and run it.
 *      A program made of one kernel without a buffer table is the per-kernel drop-in:
 *      eh_program_execute_positional == Kernel::execute(inputs, outputs).  A program with a
 *      buffer table `(buffers ("name" dtype (shape ...) input|output|temp) ...)` is compiled
 *      as a whole: kernels are fused where possible and temps that never reach memory are
 *      reported as elided. ------------------------------------------------------------------------ */
int eh_program_compile(eh_device* dev, const char* ast_text, const char* options, eh_program** out);
int eh_program_release(eh_program* prog);
int eh_program_num_buffers(eh_program* prog, int* n);
int eh_program_buffer(eh_program* prog, int i, const char** name, const char** role, size_t* bytes, int* elided);
int eh_program_num_launches(eh_program* prog, int* n);
int eh_program_launch(eh_program* prog, int launch, eh_launch_info* out);
/* bufs[i] binds buffer i of the table eh_program_buffer reports: the caller's entries in their
 * order, then scratch temps the plan added (names starting with "eh_").  NULL is allowed for
 * elided buffers and for temps (the program then keeps its own), and bufs may stop anywhere
 * after the last input or output.  sync != 0 waits for completion (the reference's kernels are
 * synchronous); sync == 0 only queues the launches on the device's stream.
 * Different entries of the table must be different buffers (an output must not alias an input,
 * no in-place update): launches that do not depend on each other by buffer name may run in another
 * order than the kernels were written, or together.  This is checked: two entries bound to
 * overlapping device memory, at least one of which some launch writes, fail with EH_ERR_INVALID
 * before anything is queued (eh_program_execute, _static and _record alike); entries the program
 * only reads may share memory. */
int eh_program_execute(eh_program* prog, eh_buffer* const* bufs, int n_bufs, int sync);
int eh_program_execute_positional(eh_program* prog, eh_buffer* const* inputs, int n_inputs,
                                  eh_buffer* const* outputs, int n_outputs, int sync);
/* eh_program_execute for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * It calls no hipMalloc or hipFree: the scratch temps the plan appended to the buffer table (names
 * starting with "eh_": partial results of split reductions and split-K contractions, chunk totals
 * of scans) are placed, each at a 256-byte boundary, in one static block of device memory of
 * EH_STATIC_SCRATCH_BYTES that every device the library runs on holds until the process ends;
 * every other buffer that reaches memory (inputs, outputs and the caller's own temps) must be
 * given.  A program whose scratch temps do not fit fails with EH_ERR_SIZE and launches nothing.
 * All calls on one GPU share that GPU's block, whichever eh_device handle they come through, and
 * the block keeps the previous call's contents (no kernel relies on them: every scratch element is
 * written before it is read).  Calls that overlap on one GPU would race on it.  Calls through one
 * handle are ordered on that handle's stream; a call through another handle of the same GPU (its
 * own stream) is made to wait on the device for the launches of the call that used the block
 * before it, so calls made through this library do not overlap on the block, with sync == 0 too.
 * What the library cannot order is a launch sequence captured into a caller's graph: when a replay
 * runs, and beside what, is the caller's business (no wait is recorded under capture), so replays
 * of such graphs and other users of the block on that GPU must be serialised by the caller.
 * A given buffer that nothing has written yet and that the program does not overwrite whole gets
 * its zero fill queued first (no allocation); under stream capture that is an error instead,
 * since a recorded fill would run again on every replay: write or read such a buffer once before. */
#define EH_STATIC_SCRATCH_BYTES ((size_t)8 << 20)
int eh_program_execute_static(eh_program* prog, eh_buffer* const* bufs, int n_bufs, int sync);
/* The launches of one eh_program_execute(prog, bufs, n_bufs, .) captured as a HIP graph of kernel
 * nodes and replayed with one call: for callers that run the same program on the same buffers
 * many times (the training loop of examples/function_fitting/main.rs:60-120 runs one compiled
 * step per iteration).  The reference has no counterpart; results are those of eh_program_execute.
 * The graph holds references to the bound buffers, so they may be released while it lives; their
 * CONTENTS are read at replay time.  Replays are ordered on the device's stream like launches. */
int eh_program_record(eh_program* prog, eh_buffer* const* bufs, int n_bufs, eh_graph** out);
int eh_graph_replay(eh_graph* graph, int sync);
int eh_graph_release(eh_graph* graph);
/* Kernel::get_binary / BackendRegistry::compile_from_binary (src/backend/traits.rs:576-586,
 * src/backend/device.rs:161-170): the gfx950 code object of one launch. */
int eh_program_binary(eh_program* prog, int launch, const void** blob, size_t* len);

/* ---- Thin module layer: load a gfx950 code object (from eh_compile_source, eh_program_binary or
 *      the disk cache) and launch one entry point with buffer arguments.  This is
 *      BackendRegistry::compile_from_binary + Kernel::execute_with_sizes
 *      (src/backend/device.rs:161-170, src/backend/traits.rs:556-566); `grid` counts
 *      workgroups, `block` work-items per workgroup. -------------------------------------------- */
int eh_module_load(eh_device* dev, const void* blob, size_t len, const char* entry, eh_module** out);
int eh_module_launch(eh_module* mod, const unsigned grid[3], const unsigned block[3], unsigned lds_bytes,
                     eh_buffer* const* args, int n_args, int sync);
int eh_module_release(eh_module* mod);

/* ---- timing on the device's stream (HIP events) ------------------------------------------------ */
int eh_event_create(eh_device* dev, eh_event** out);
int eh_event_record(eh_event* ev);          /* on the device's stream */
int eh_event_sync(eh_event* ev);
int eh_event_elapsed_ms(eh_event* start, eh_event* stop, float* ms);
int eh_event_release(eh_event* ev);

#ifdef __cplusplus
}
#endif
#endif /* ECLAT_HIP_H */

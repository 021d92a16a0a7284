/*
 * acc_hip.h -- C ABI of libacchip, the MI355X (gfx950) runtime under an
 * Accelerate backend.  It is what a `Data.Array.Accelerate.HIP` module binds
 * with `foreign import ccall` in place of everything accelerate-cuda reaches
 * through the `cuda` package (Foreign.CUDA.Driver / Foreign.CUDA.Analysis) and
 * the external `nvcc`.
 *
 * Two layers:
 *
 *   A. driver layer   -- devices, memory, transfers, streams, events, modules,
 *                        run-time compilation with a content-hashed code-object
 *                        cache, occupancy, raw launches;
 *   B. skeleton layer -- instantiate one of the hand-written gfx950 skeleton
 *                        templates with the scalar fragments the code generator
 *                        produced (acc_skel_create), and run it with the
 *                        temporaries, launch shapes and multi-kernel protocols
 *                        it needs (acc_exec_*).  These are the roles of
 *                        the CUDA/CodeGen modules (templates) and of the skeleton
 *                        drivers in CUDA/Execute.hs:264-450.
 *
 * Conventions
 *   - plain C: pointers, sizes, fixed-width integers; no C++ or torch types;
 *   - every function returns an int status (ACC_OK == 0); the message of the
 *     last failure on the calling thread is acc_last_error(); nothing aborts.
 *     (The reference throws CUDAException, State.hs:86-88; out-of-memory is its
 *     one recoverable error, Array/Remote.hs:63-67 -> ACC_ERR_OOM here);
 *   - device pointers are uint64_t (Haskell does pointer arithmetic itself, as
 *     with advanceDevPtr / plusDevPtr);
 *   - acc_stream / acc_event / acc_module / acc_function are the HIP handles
 *     themselves (hipStream_t, ...); a NULL stream is the default stream;
 *   - the caller owns every handle it creates; the library owns the kernel
 *     cache and per-context scratch memory; destroy/free of NULL is a no-op;
 *   - thread safety: every entry point may be called from any thread; the
 *     device of the context is made current on entry.  One acc_skel may be
 *     executed from several threads, calls on the SAME stream are ordered.
 */
#ifndef ACC_HIP_H
#define ACC_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

/* ---- status codes -------------------------------------------------------- */
#define ACC_OK               0
#define ACC_ERR_INVALID      1   /* bad argument, shape mismatch, fold1 of empty array */
#define ACC_ERR_OOM          2   /* device allocation failed: caller may evict and retry */
#define ACC_ERR_COMPILE      3   /* run-time compilation failed: see acc_compile_log */
#define ACC_ERR_NOT_FOUND    4   /* no such kernel entry / device */
#define ACC_ERR_HIP          5   /* any other HIP runtime error */
#define ACC_ERR_UNSUPPORTED  6   /* valid Accelerate, not implemented by this backend */
#define ACC_ERR_IO           7   /* kernel cache file trouble (never fatal to a compile) */
#define ACC_ERR_STUCK        8   /* a kernel gave up a wait for another workgroup: see acc_context_sync */

typedef struct acc_context_s *acc_context;
typedef struct acc_skel_s    *acc_skel;
typedef void *acc_stream;     /* hipStream_t   */
typedef void *acc_event;      /* hipEvent_t    */
typedef void *acc_module;     /* hipModule_t   */
typedef void *acc_function;   /* hipFunction_t */
typedef uint64_t acc_devptr;

const char *acc_last_error(void);
const char *acc_version(void);

/* =========================================================================
 * A. driver layer
 * ========================================================================= */

/* CUDA.initialise / count / props: State.hs:127-132, Analysis/Device.hs:31-41 */
int acc_init(void);
int acc_device_count(int *count);

typedef struct acc_device_props {
  char     name[256];
  char     arch[64];               /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
  int32_t  compute_units;
  int32_t  wavefront_size;
  int32_t  max_threads_per_block;
  int32_t  clock_khz;
  int64_t  lds_per_block;          /* bytes a single workgroup may use */
  int64_t  lds_per_cu;
  int64_t  l2_bytes;
  int64_t  total_mem;
  int32_t  regs_per_block;
  int32_t  max_threads_per_cu;
} acc_device_props;
int acc_device_get_props(int device, acc_device_props *out);

/* Context.hs:55-71 (create), :99-111 (destroy).  HIP has one primary context
 * per device, so there is no push/pop (State.hs:84-92) and no cache config.  */
int acc_context_create(int device, acc_context *out);
int acc_context_destroy(acc_context ctx);
int acc_context_device(acc_context ctx, int *device);
int acc_context_sync(acc_context ctx);                 /* CUDA.sync */
/* Waits inside kernels (a scan tile for its predecessors' descriptors, the collecting workgroup of a fold for the
 * others' partial results, a lane of a permute for a lock) are bounded.  A wait that runs out ends the kernel
 * normally, with a wrong result, and leaves a mark that the next synchronising call on the context --
 * acc_context_sync, acc_stream_sync, acc_event_sync, acc_memcpy_d2h -- returns as ACC_ERR_STUCK, once: nothing
 * enqueued on the context since its last successful synchronisation is then to be trusted.  The reference has no
 * counterpart: its kernels do not wait for one another (a lock that never opens hangs it, IndexSpace.hs:285-303). */

/* Scratch memory the skeleton drivers keep per context (fold partials, scan descriptors, permute tables and locks,
 * Execute.hs:304-315,402-405 allocate theirs per use) is reused between calls and grows to the largest request.
 * acc_context_trim frees every block that is not in use (it waits for the device first) and reports the bytes
 * given back; acc_context_scratch_bytes says how much is held.  acc_memtable_malloc trims by itself before it
 * gives up. */
int acc_context_trim(acc_context ctx, size_t *freed_bytes);
int acc_context_scratch_bytes(acc_context ctx, size_t *bytes);
/* For tests of the failure path only: store `value` in the 32-bit word `word` of the per-target lock block that
 * the context's last locked permute used (ACC_ERR_NOT_FOUND if there is none, ACC_ERR_INVALID past its end).  A
 * lock left at 1 makes that permute's bounded wait run out. */
int acc_context_debug_poke_lock(acc_context ctx, size_t word, uint32_t value);

/* Tuning knobs, "name=value,name=value": overrides of the defaults the skeleton generator and the drivers work with
 * (tile shapes, thresholds between kernel forms), for measurement; the counterpart of the reference's
 * -fflags read once at start-up (Debug.hs:100-140).  The text is parsed once into an immutable table, and no
 * driver call ever reads the environment.  The process's table comes from ACC_HIP_TUNE in the environment when it
 * is first wanted; acc_tuning_set replaces it (NULL: read ACC_HIP_TUNE again, now).  A context takes the process's
 * table when it is created, acc_context_set_tuning gives it another (NULL: the process's); an instance works with
 * the table its context had when it was created, for as long as it lives.  acc_skel_preview and
 * acc_skel_compile_only, which have no context, use the process's table.                                     */
int acc_tuning_set(const char *text);
const char *acc_tuning_text(void);                  /* the process's table as text; valid until the thread's next call */
int acc_context_set_tuning(acc_context ctx, const char *text);

/* CUDA.mallocArray / free / getMemInfo: Array/Remote.hs:63-79,191 */
int acc_malloc(acc_context ctx, size_t bytes, acc_devptr *out);
int acc_free(acc_context ctx, acc_devptr p);
int acc_mem_info(acc_context ctx, size_t *free_bytes, size_t *total_bytes);

/* pinned host staging buffers for asynchronous transfers (the memory is the process's: it may be given back after
 * its context has been destroyed, with a NULL context) */
int acc_host_alloc(acc_context ctx, size_t bytes, void **out);
int acc_host_free(acc_context ctx, void *p);

/* pokeArray / peekArray / copyArray [Async], memsetAsync:
 * Array/Prim.hs:189-391, Execute.hs:405.  stream == NULL: default stream.
 * The non-async forms return after the copy has completed.                  */
int acc_memcpy_h2d(acc_context ctx, acc_devptr dst, const void *src, size_t bytes);
int acc_memcpy_d2h(acc_context ctx, void *dst, acc_devptr src, size_t bytes);
int acc_memcpy_d2d(acc_context ctx, acc_devptr dst, acc_devptr src, size_t bytes);
int acc_memcpy_h2d_async(acc_context ctx, acc_devptr dst, const void *src, size_t bytes, acc_stream s);
int acc_memcpy_d2h_async(acc_context ctx, void *dst, acc_devptr src, size_t bytes, acc_stream s);
int acc_memcpy_d2d_async(acc_context ctx, acc_devptr dst, acc_devptr src, size_t bytes, acc_stream s);
int acc_memset32_async(acc_context ctx, acc_devptr dst, uint32_t value, size_t count, acc_stream s);

/* Execute/Stream.hs:102,134 and Execute/Event.hs:70-127, Debug.hs:48-67.  A stream that is destroyed with nothing
 * pending on it, and an event that is destroyed while it waits for nothing, are kept by the context (up to 64 of
 * each) and handed out by the next create of their kind: the reservoir of Execute/Stream.hs:118-140 and the event
 * table of Execute/Event.hs:63-85.                                                                            */
int acc_stream_create(acc_context ctx, acc_stream *out);
int acc_stream_destroy(acc_context ctx, acc_stream s);
int acc_stream_sync(acc_context ctx, acc_stream s);
int acc_stream_wait_event(acc_context ctx, acc_stream s, acc_event e);
int acc_event_create(acc_context ctx, int enable_timing, acc_event *out);
int acc_event_destroy(acc_context ctx, acc_event e);
int acc_event_record(acc_context ctx, acc_event e, acc_stream s);
int acc_event_sync(acc_context ctx, acc_event e);
int acc_event_query(acc_context ctx, acc_event e, int *done);
int acc_event_elapsed_ms(acc_context ctx, acc_event start, acc_event stop, float *ms);

/* Run-time compilation with the kernel cache.  Replaces the nvcc subprocess
 * and the two-level cache: Compile.hs:543-594, Persistent.hs:77-137,218-228,
 * 305-378.  Key = SHA-256 of (library version, target, compiler version,
 * options, the device headers, the source text); look-up order is RAM table,
 * then <cache dir>/<target>/<key>.co (size- and hash-checked, rewritten if
 * damaged), then hiprtc.  Compilation needs no GPU.
 *
 *   target  "gfx950" style ISA name; NULL = the context's device (ctx may be
 *           NULL only when target is given)
 *   code    receives a pointer owned by the cache, valid until acc_cache_clear
 */
int acc_compile(acc_context ctx, const char *target, const char *source,
                const char *const *options, int n_options,
                const void **code, size_t *code_size);
const char *acc_compile_log(void);                       /* log of the last compile on this thread */
int acc_cache_set_dir(const char *dir);                  /* NULL/"" = memory only; default
                                                            $ACC_HIP_CACHE_DIR or ~/.accelerate/accelerate-hip-<ver>/cache */
const char *acc_cache_dir(void);
typedef struct acc_cache_stats { uint64_t ram_hits, disk_hits, compiles, disk_errors; } acc_cache_stats;
int acc_cache_get_stats(acc_cache_stats *out);
int acc_cache_clear(int also_disk);                      /* -fflush-cache of the reference's debug flags */

/* CUDA.loadData / getFun / unload / requires: Compile.hs:453-465,505,534 */
int acc_module_load(acc_context ctx, const void *code, size_t code_size, acc_module *out);
int acc_module_unload(acc_context ctx, acc_module m);
int acc_module_get_function(acc_context ctx, acc_module m, const char *entry, acc_function *out);
#define ACC_FUNC_NUM_REGS            0
#define ACC_FUNC_SHARED_SIZE_BYTES   1
#define ACC_FUNC_CONST_SIZE_BYTES    2
#define ACC_FUNC_LOCAL_SIZE_BYTES    3
#define ACC_FUNC_MAX_THREADS         4
int acc_function_attr(acc_context ctx, acc_function f, int which, int *value);

/* CUDA.optimalBlockSizeOf / Occupancy: Analysis/Launch.hs:42-102.  Resident
 * workgroups per compute unit for the given block size and dynamic LDS.      */
int acc_occupancy(acc_context ctx, acc_function f, int block, size_t dyn_lds, int *blocks_per_cu);

/* CUDA.launchKernel fn (grid,1,1) (cta,1,1) smem stream args: Execute.hs:975-978 */
int acc_launch(acc_context ctx, acc_function f, uint32_t grid, uint32_t block, uint32_t dyn_lds,
               acc_stream s, void **args);

/* Pure launch arithmetic of Analysis/Launch.hs, exposed for the host side
 * and for tests: blocks needed for `n` elements at `per_block` each, at most
 * `cus * blocks_per_cu`, at least 1 (split, :124-128; maxGrid, :51-55).      */
int64_t acc_launch_grid(int64_t n, int64_t per_block, int64_t cus, int64_t blocks_per_cu);

/* =========================================================================
 * B. skeleton layer
 * ========================================================================= */

#define ACC_MAX_RANK 8
#define ACC_MAX_COMP 16     /* components of a (flattened) tuple element: Accelerate's tuples have up to 15 */

/* A device-resident array as the kernels see it: extents outermost first
 * (row-major, innermost dimension last: CodeGen/Base.hs:193-202) and one
 * device pointer per tuple component, structure-of-arrays
 * (Array/Prim.hs:64-110; include/AccFFI.h:10-30 has the same shape/adata
 * split).  rank 0 is a Scalar (one element).                                */
typedef struct acc_array {
  int32_t    rank;
  int32_t    ncomp;
  int64_t    shape[ACC_MAX_RANK];
  acc_devptr ptr[ACC_MAX_COMP];
} acc_array;

/* signature of one free array variable of the scalar fragments (Gamma,
 * AST.hs:87-112).  Variable k becomes the kernel parameters
 *     const Int64 shIn<k>_<rank-1> ... shIn<k>_0,
 *     const T<ncomp-1>* arrIn<k>_<ncomp-1> ... const T0* arrIn<k>_0
 * exactly as CodeGen/Base.hs:69-89,348-383 names and orders them, and the
 * fragments index them as arrIn<k>_<c>[i] (CodeGen.hs:714-747).              */
typedef struct acc_env_sig {
  int32_t     rank;
  int32_t     ncomp;
  const char *type[ACC_MAX_COMP];   /* C type of each component, component 0 first */
} acc_env_sig;

/* skeleton kinds: one per entry of CodeGen.hs:91-136 that is built */
enum {
  ACC_SKEL_MAP        = 0,   /* entry "map"       Mapping.hs:39-78      */
  ACC_SKEL_GENERATE   = 1,   /* entry "generate"  IndexSpace.hs:47-83   */
  ACC_SKEL_TRANSFORM  = 2,   /* entry "transform" IndexSpace.hs:96-141 (backpermute too) */
  ACC_SKEL_FOLD       = 3,   /* foldAll / fold    Reduction.hs:56-65    */
  ACC_SKEL_FOLD1      = 4,   /* fold1All / fold1  Reduction.hs:67-75    */
  ACC_SKEL_FOLDSEG    = 5,   /* foldSeg           Reduction.hs:399-408  */
  ACC_SKEL_FOLD1SEG   = 6,   /* fold1Seg          Reduction.hs:410-418  */
  ACC_SKEL_SCANL      = 7,   /* PrefixSum.hs:51-66   */
  ACC_SKEL_SCANL1     = 8,   /* PrefixSum.hs:77-91   */
  ACC_SKEL_SCANLP     = 9,   /* scanl'  PrefixSum.hs:102-114 */
  ACC_SKEL_SCANR      = 10,
  ACC_SKEL_SCANR1     = 11,
  ACC_SKEL_SCANRP     = 12,  /* scanr' */
  ACC_SKEL_PERMUTE    = 13,  /* IndexSpace.hs:160-303 */
  ACC_SKEL_STENCIL    = 14,  /* Stencil.hs:55-114     */
  ACC_SKEL_STENCIL2   = 15,  /* Stencil.hs:118-237: two sources, result over the intersection of their extents */
  ACC_SKEL_KIND_COUNT = 16
};

/* how `combine` may be applied atomically by permute */
enum {
  ACC_COMBINE_GENERIC = 0,   /* compare-and-swap loop on the element's bits (4/8-byte elements) */
  ACC_COMBINE_ADD     = 1,   /* combine x y == x + y   -> hardware atomic add   */
  ACC_COMBINE_MIN     = 2,
  ACC_COMBINE_MAX     = 3,
  ACC_COMBINE_AND     = 4,
  ACC_COMBINE_OR      = 5,
  ACC_COMBINE_XOR     = 6
};

/* stencil boundary conditions: Stencil/Extra.hs:112-116 */
enum { ACC_BOUNDARY_CLAMP = 0, ACC_BOUNDARY_MIRROR = 1, ACC_BOUNDARY_WRAP = 2, ACC_BOUNDARY_CONSTANT = 3 };

/* flags */
#define ACC_FLAG_FOLD_RIGHT   1u  /* foldSeg: associate x0 (+) (x1 (+) (... (+) z)) instead of ((x0 (+) x1) ...) (+) z */
#define ACC_FLAG_FAST_MATH    2u  /* allow FMA contraction (default: off, every scalar op rounds as written) */
#define ACC_FLAG_TILED        8u  /* map family, out_rank >= 2: produce the result in square tiles of its two innermost
                                     dimensions instead of runs of the innermost one, for element functions that read
                                     their sources across rows (a transposing backpermute: IndexSpace.hs:96-141 reads
                                     one element of every source row per run); the results are the same.
                                     fold / fold1 along the innermost dimension (out_rank >= 1): the same statement
                                     about the element function -- where the ROW of the folded array moves by one, it
                                     reads neighbouring addresses (the fold of a transposed matrix, a matrix product
                                     written as a fold over replicated operands) -- and a lane then takes a row,
                                     neighbouring rows in neighbouring lanes, instead of a team of lanes along a row;
                                     the operands meet in index order as always.  (The element function of any fold
                                     with out_rank >= 1 may name `acc_row` and `acc_col`, the row of the folded array
                                     and the place within it: ix == acc_row * row length + acc_col.  Kernels that give
                                     a row to a lane know both without a division, and what depends on acc_row alone
                                     leaves the lane's loop.) */
#define ACC_FLAG_TILE_DIM(d)  ((uint32_t)(d) << 8)  /* with ACC_FLAG_TILED on a map of rank >= 3: the tiles' second dimension
                                     is the d-th above the innermost one (1, and what 0 means: the second innermost; 2: the
                                     third innermost, ...), for an element function that reads its sources along THAT
                                     dimension of the result -- a volume turned so that what was its innermost dimension
                                     becomes its outermost; 1 <= d < out_rank */
#define ACC_FLAG_GUARDED      4u  /* the instance may run under an acc_guard (see acc_guard_create): its kernels take the
                                     guard's address as one more, last, parameter and do nothing once the guard is down */

/* What the code generator hands over for one array operation: the pieces
 * CUTranslSkel / CUFun1 / CUFun2 / CUExp / CUDelayed carry across the
 * reference's Compile boundary (CodeGen/Base.hs:98-138), as HIP C++ text.
 * Fragments are EXPRESSIONS (GNU statement expressions ({ ...; v; }) allow
 * local bindings) over the names given below and the env parameters.        */
typedef struct acc_skel_desc {
  int32_t            kind;          /* ACC_SKEL_*                                           */
  uint32_t           flags;         /* ACC_FLAG_*                                           */
  int32_t            n_env;         /* free array variables In0 .. In<n_env-1>              */
  const acc_env_sig *env;
  const char        *elt_type;      /* C type of the result element, or "T<n-1>, ..., T0" for a
                                     * tuple: the generated code then declares
                                     *   struct acc_elt { T<n-1> a<n-1>; ...; T0 a0; };
                                     * fragments produce and take apart acc_elt values, and the
                                     * result array has one pointer per component (CodeGen/
                                     * Base.hs:344-357).  A stencil may produce tuples and
                                     * read them (stencil_in_type)                            */
  int32_t            elt_size;      /* sizeof(elt_type); 0 = derive from the type's name    */
  int32_t            out_rank;      /* map family, stencil: rank of the result (>= 0)       */
  const char        *preamble;      /* file-scope declarations for the fragments, or NULL   */
  const char        *get;           /* delayed input / element function over `ix` (Int64 linear
                                       index); map family: value of out[ix].  Not used by stencil. */
  const char        *combine;       /* over `x`, `y`: fold, foldSeg, scans, permute.  A permute
                                       whose combination is spelt as its first operand alone -- `x`, or
                                       `acc_elt{x.a<n-1>, ..., x.a0}` for a tuple: `permute const`, the
                                       scatter of a compaction or of a sorting pass -- stores the new
                                       values and reads and locks nothing; of several sources on one
                                       target one wins whole */
  const char        *seed;          /* NULL for the seedless kinds                           */
  const char        *permutation;   /* permute: linear target index of source `ix`, or
                                       ACC_IGNORE (-1) to drop the element                   */
  int32_t            combine_hint;  /* ACC_COMBINE_*: lets permute use hardware atomics      */
  /* stencil: taps t0 .. t<n-1> at offsets (dy, dx) from the focus (1-D: dy = 0; 3-D: see tap_dz),
   * `stencil_fn` is an expression over t0.. giving the result element       */
  int32_t            boundary;      /* ACC_BOUNDARY_*                                       */
  const char        *boundary_constant; /* ACC_BOUNDARY_CONSTANT: the value outside the source; of a
                                           source of tuples one value per component, "v<n-1>, ..., v0" */
  int32_t            n_taps;
  const int32_t     *tap_dy;
  const int32_t     *tap_dx;
  const char        *stencil_fn;
  const char        *stencil_in_type; /* element type of the source array; NULL = elt_type.  "T<n-1>, ..., T0" for a
                                         source of tuples (Stencil/Extra.hs:53-128 reads every component): the
                                         source acc_array then has one pointer per component, and a tap is a value of
                                         struct acc_in1_elt { T<n-1> a<n-1>; ...; T0 a0; } (t0.a1, t0.a0; the second
                                         source of a stencil2: acc_in2_elt, u0.a1, ...) */
  const char        *seg_type;      /* foldSeg: C type of the offsets (NULL = "Int32")       */
  /* stencil2 only: the second source, with taps u0 .. u<n-1>; `stencil_fn` is over t0.. and u0.. */
  int32_t            boundary2;
  const char        *boundary2_constant;
  int32_t            n_taps2;
  const int32_t     *tap2_dy;
  const int32_t     *tap2_dx;
  const char        *stencil_in2_type; /* NULL = elt_type */
  /* rank-3 stencils: the taps' offsets across planes (NULL = all in the focus' plane) */
  const int32_t     *tap_dz;
  const int32_t     *tap2_dz;
  /* stencils of any rank (Stencil.hs:55-114 serves every rank through cfromIndex, Base.hs:207-218): the taps'
   * offsets as n_taps rows of out_rank numbers, outermost dimension first.  Where given, tap_dz / tap_dy / tap_dx
   * are not read; required for out_rank > 3.  (Offsets of up to 2 planes and 4 rows and columns in up to three
   * dimensions run on strips of rows held in registers; anything else an element a thread, as the reference does.) */
  const int32_t     *tap_offsets;
  const int32_t     *tap2_offsets;
} acc_skel_desc;

/* Generate + compile (through the cache) + load one skeleton instance and
 * work out its launch shape.  The counterpart of build1/compile/link,
 * Compile.hs:444-459,484-566, which yields the AccKernel record AST.hs:51-59. */
int acc_skel_create(acc_context ctx, const acc_skel_desc *desc, acc_skel *out);
int acc_skel_destroy(acc_skel s);

/* The same with the compilation left to a pool of worker threads: the description is checked and the source
 * generated before the call returns (what is wrong with either is reported here), the instance's first variant is
 * compiled in the background, and whatever first needs the compiled kernel -- acc_exec_*, acc_skel_get_info,
 * acc_skel_wait -- waits for it and reports a compiler failure then, with acc_compile_log() set as if the caller
 * had compiled.  This is how the reference builds the kernels of a program: build1 forks one compilation per array
 * operation, no more at a time than the machine has processors (Compile.hs:484-538,620-660), and the executing thread
 * blocks where a kernel is first used (the lazy `link`, Compile.hs:444-459) -- so a program of several kernels is
 * ready after the slowest of them, not after their sum.  acc_skel_create is this call followed by acc_skel_wait.
 * acc_skel_poll says without waiting whether the compilation has ended (well or badly); acc_compile_threads the
 * size the pool may grow to: the machine's processors, at most 16 unless ACC_HIP_COMPILE_THREADS in the environment
 * says otherwise.  An instance may be destroyed while its compilation runs.                                      */
int acc_skel_create_async(acc_context ctx, const acc_skel_desc *desc, acc_skel *out);
int acc_skel_wait(acc_skel s);
/* Start compiling another variant of the instance in the background (numbering as for acc_skel_preview), for a
 * caller that knows ahead of a launch what its operands will look like -- unaligned, small, narrow; nothing happens
 * if the variant is ready or under way.  Without it a variant other than 0 is compiled by the first call that needs
 * it, which waits.                                                                                            */
int acc_skel_prefetch(acc_skel s, int variant);
int acc_skel_poll(acc_skel s, int *ready);
int acc_compile_threads(void);
/* Before the process exits: abandon the compilations that have not started (whoever waits for one gets
 * ACC_ERR_COMPILE), wait for the ones that run, end the workers.  exit() tears down the compiler's static data while
 * a worker may still be inside the compiler; a host that may exit with compilations under way calls this first (from
 * its own at-exit hook: the reference's forked compiler threads simply die with the Haskell main thread, and its
 * nvcc is a process of its own).  Instances created afterwards compile on the thread that first needs them.    */
int acc_compile_drain(void);

/* The generated translation unit (for -ddump-cc style debugging and tests).
 * variant 0 = aligned (128-bit accesses assumed legal), 1 = unaligned.      */
int acc_skel_source(acc_skel s, int variant, const char **source);
/* the same text straight from a description, without a context or a GPU; the
 * string stays valid until the calling thread's next call of this function.
 * A permute has further forms the driver chooses between by the number of
 * targets, at variant + 2 (tables under locks in LDS), + 4 (several LDS
 * windows of targets), + 6 (16-bit counts in LDS, integer addition); a scan
 * its small tiles and a segmented fold its longer staged chunk at + 2; a
 * segmented fold of a vector the forms that hand segments far longer than
 * the rest over to a second launch at + 4; a stencil half and a quarter of
 * the columns a lane at + 2 and + 4, and an element a thread (for arrays of
 * a few columns) at + 6; a map in tiles the map in runs at + 2                */
int acc_skel_preview(const acc_skel_desc *desc, int variant, const char **source, const char **entry);
/* compile only (no GPU needed): used by the build check */
int acc_skel_compile_only(const char *target, const acc_skel_desc *desc, size_t *code_size);

/* kernel record of the instance: AccKernel, AST.hs:51-59 */
typedef struct acc_skel_info {
  char    entry[64];
  int32_t block;              /* threads per workgroup          */
  int32_t blocks_per_cu;      /* occupancy of the main kernel   */
  int32_t num_regs;
  int32_t static_lds;
  int32_t elements_per_block; /* tile size                      */
} acc_skel_info;
int acc_skel_get_info(acc_skel s, acc_skel_info *out);

/* ---- skeleton drivers (Execute.hs:264-450) ----------------------------------
 * `env` points at n_env arrays in Gamma order.  All work is enqueued on
 * `stream` and the call returns without waiting.                             */

/* map / generate / transform: executeOp, Execute.hs:264-268.  out has the
 * desc's out_rank; one element is written per index of out.                 */
int acc_exec_map(acc_skel s, const acc_array *env, const acc_array *out, acc_stream stream);

/* fold / fold1: foldOp / fold1Op / foldCore / foldRec, Execute.hs:282-318.
 * in_shape has in_rank >= 1 extents of the delayed input; out has rank
 * in_rank-1.  fold1 of an empty innermost dimension is ACC_ERR_INVALID
 * ("empty array", Execute.hs:282-285).                                       */
int acc_exec_fold(acc_skel s, const acc_array *env, int32_t in_rank, const int64_t *in_shape,
                  const acc_array *out, acc_stream stream);

/* foldSeg / fold1Seg: foldSegOp, Execute.hs:320-324.  `n` elements in one row;
 * `offsets` is the manifest vector of nseg+1 segment starts (the front end
 * has already turned lengths into offsets, CUDA.hs:402); out has nseg
 * elements.                                                                  */
int acc_exec_foldseg(acc_skel s, const acc_array *env, int64_t n, const acc_array *offsets,
                     const acc_array *out, acc_stream stream);
/* The same for an input of any rank (foldSegOp (sh :. _) (Z :. sz) = executeOp (sh :. sz - 1), Execute.hs:323-324):
 * the descriptor segments the innermost dimension of EVERY outer row, segment s of a row being
 * [offsets[s], offsets[s+1]) within it (CodeGen/Reduction.hs:473-474,485-486); what a row holds beyond its last
 * segment is not read into any result.  in_rank must equal the desc's out_rank (0 and 1 both mean a vector);
 * out has the input's outer extents and exactly nseg elements a row (a vector may be longer).                  */
int acc_exec_foldseg_nd(acc_skel s, const acc_array *env, int32_t in_rank, const int64_t *in_shape,
                        const acc_array *offsets, const acc_array *out, acc_stream stream);

/* scans: scanOp / scan1Op / scan'Op / scanCore, Execute.hs:328-392.
 *   scanl, scanr    : out holds n+1 elements, `total` is ignored (may be NULL)
 *   scanl1, scanr1  : out holds n elements
 *   scanl', scanr'  : out holds n elements, total is a Scalar                */
int acc_exec_scan(acc_skel s, const acc_array *env, int64_t n, const acc_array *out,
                  const acc_array *total, acc_stream stream);

/* The same scan for callers that cannot allocate device memory: code under HIP graph capture, tight serving
 * loops, harnesses that forbid it.  It has no counterpart in the reference (whose scanCore allocates its block
 * sums on every call, Execute.hs:371-376).  The tile descriptors live in a file-scope array in device memory that
 * the library holds on every device it has a context on, until the process ends (about 1 MB); the call allocates
 * nothing, compiles nothing and loads nothing:
 *   - the input may span at most ACC_NOALLOC_MAX_TILES tiles of acc_skel_info.elements_per_block elements
 *     (32768 Int32 each: 2^28 elements); more is ACC_ERR_INVALID;
 *   - the variant that acc_exec_scan takes for such operands must have been loaded already, else ACC_ERR_INVALID.
 *     There are four: for operands aligned to 16 bytes or not, and for arrays of at most 12 MB (scanned in tiles
 *     an eighth the size) or more.  acc_skel_create loads the one for large aligned arrays, a first acc_exec_scan
 *     on operands of the same alignment and on the same side of 12 MB each of the others;
 *   - every call on a device shares that device's array: calls that overlap in time on one device, from any
 *     stream, thread or context, race.  Calls ordered on one stream are fine.  A call of more tiles than the device
 *     holds at once must not overlap ANY other scan of that size on the device either, acc_exec_scan's included:
 *     acc_exec_scan chains such scans across streams with events, which this entry point, possibly under capture,
 *     does not;
 *   - a call makes two launches: a small kernel that counts the launch's tag in the array's header, and the scan,
 *     which reads it there.  A graph that records the call therefore gets a fresh tag at every replay; were the tag
 *     an argument of the recorded launch, a replay would take the descriptors its predecessor left for its own.
 * Results are those of acc_exec_scan, bit for bit.                                                          */
#define ACC_NOALLOC_MAX_TILES 8192
int acc_exec_scan_noalloc(acc_skel s, const acc_array *env, int64_t n, const acc_array *out,
                          const acc_array *total, acc_stream stream);

/* permute: permuteOp, Execute.hs:396-408.  `n_src` source elements (linear);
 * out is first filled from `defaults` (same shape), then combined into.
 * defaults may alias out (then nothing is copied).                           */
int acc_exec_permute(acc_skel s, const acc_array *env, int64_t n_src, const acc_array *defaults,
                     const acc_array *out, acc_stream stream);

/* stencil: stencilOp, Execute.hs:413-425 (launched once, not twice).  `in` is
 * the manifest source, out has the same shape (any rank up to ACC_MAX_RANK).  */
int acc_exec_stencil(acc_skel s, const acc_array *env, const acc_array *in, const acc_array *out,
                     acc_stream stream);

/* stencil2: stencil2Op, Execute.hs:427-450.  Two manifest sources of the same
 * rank; out must be no larger than the intersection of their extents (that is
 * the result's shape, Stencil.hs:118-119).  Each source keeps its own boundary
 * condition, applied at its own edges.                                        */
int acc_exec_stencil2(acc_skel s, const acc_array *env, const acc_array *in1, const acc_array *in2,
                      const acc_array *out, acc_stream stream);

/* `iters` applications of the same stencil, ping-ponging between a and b on
 * the device with no host round trip (what `awhile` with a counter, or a
 * repeated run1, computes: Execute.hs:236-244, CUDA.hs:325-333).  The input is
 * a; *result_in_b tells where the last application wrote.                    */
int acc_exec_stencil_iterate(acc_skel s, const acc_array *env, const acc_array *a, const acc_array *b,
                             int32_t iters, acc_stream stream, int32_t *result_in_b);

/* awhile, Execute.hs:236-244, without a host round trip per iteration.  The reference evaluates the predicate, reads
 * its Scalar Bool back and decides on the host, every iteration.  Here a guard -- two words in device memory, `alive`
 * and `count` -- stands between the predicate and the body:
 *
 *     acc_guard_create; acc_stream_set_guard(stream, guard); acc_guard_reset         alive = 1, count = 0
 *     K times:   <the predicate's skeletons>; acc_guard_latch(pred);  <the body's skeletons>
 *     acc_guard_read -> alive, count;   repeat while alive
 *
 * acc_guard_latch takes the predicate's result, a rank-0 array of Bool (one byte), where it lies on the device:
 * alive becomes alive && pred, and count goes up by one if the loop is still alive, so that count is the number of
 * times the body has really run.  Every skeleton executed on a stream that has a guard set must have been created with
 * ACC_FLAG_GUARDED (else ACC_ERR_INVALID): its kernels load `alive` on entry and return at once when it is zero, and so
 * do the copies the drivers make (a permute's defaults).  The iterations enqueued past the end of the loop therefore
 * leave their result arrays untouched, and the value of the loop is what the count-th application of the body
 * produced (the initial value if count is 0).  The host reads the guard once per K iterations instead of once per
 * iteration.  A guard serves one loop at a time; acc_stream_set_guard(stream, NULL) takes it off the stream.     */
typedef struct acc_guard_s *acc_guard;
int acc_guard_create(acc_context ctx, acc_guard *out);
int acc_guard_destroy(acc_guard g);
int acc_guard_reset(acc_guard g, acc_stream stream);
int acc_guard_latch(acc_guard g, const acc_array *pred, acc_stream stream);
int acc_guard_read(acc_guard g, acc_stream stream, int32_t *alive, int64_t *count);   /* waits for the stream */
int acc_stream_set_guard(acc_context ctx, acc_stream stream, acc_guard g);

/* Time on the device of the kernels a thread launches through the skeleton drivers between the two calls: an event
 * before and one behind every launch, summed by acc_trace_stop, which waits for them (Debug.hs:41-76 `timed`, hooked
 * at Execute.hs:975-982; the reference prints one line per launch under -ddump-exec, which ACC_HIP_DEBUG=dump-exec
 * in the environment does here).  Per thread; the kernels run as usual.                                           */
int acc_trace_start(acc_context ctx);
int acc_trace_stop(acc_context ctx, int32_t *launches, double *gpu_ms);

/* =========================================================================
 * C. memory table
 * ========================================================================= */

/* The association between host arrays and their device copies, with reuse of
 * freed blocks and least-recently-used eviction when the device (or a budget)
 * is full: the roles of Array/Remote.hs:111-196 and of the LRU table it takes
 * from the `accelerate` base package (Data.Array.Accelerate.Array.Remote.LRU,
 * accelerate-1.0; not part of the reference tree).
 *
 *   key     identity of the host array (the reference uses the StableName of
 *           its ArrayData; the address of the host storage serves as well)
 *   host    the host storage of `bytes` bytes: evicted data is written there
 *           and read from there when the array is wanted again.  It must stay
 *           valid until acc_memtable_free(key)
 *   frozen  non-zero: the host copy is authoritative and already holds the
 *           data (a `use`d array): it is uploaded when first acquired and
 *           eviction drops the device copy without writing back.  Zero: the
 *           array is produced on the device; eviction writes it back first
 *
 * Device blocks are rounded up to ACC_MEMTABLE_GRANULE bytes (the reference's
 * remoteAllocationSize, Array/Remote.hs:80) and a freed block waits in a
 * nursery for the next array of the same rounded size.  When an allocation
 * does not fit, the nursery is returned to the device first; then arrays that
 * are neither acquired nor still in use by work recorded at their last release
 * are evicted, least recently used first.  ACC_ERR_OOM if that is not enough.  */
typedef struct acc_memtable_s *acc_memtable;
#define ACC_MEMTABLE_GRANULE 1024

/* budget_bytes: upper bound on device bytes held by the table (arrays +
 * nursery); 0 = bounded only by what the device gives (new, :103-106)        */
int acc_memtable_create(acc_context ctx, uint64_t budget_bytes, acc_memtable *out);
int acc_memtable_destroy(acc_memtable mt);          /* frees every managed block */

/* malloc, Array/Remote.hs:141-155.  *is_new = 0 when the key is already in the
 * table (nothing is allocated or uploaded again: an array `use`d twice is
 * uploaded once, Array/Prim.hs:177-192)                                       */
int acc_memtable_malloc(acc_memtable mt, uint64_t key, void *host, uint64_t bytes, int frozen, int *is_new);

/* withRemote, Array/Remote.hs:113-135, as a bracket the caller closes: acquire
 * returns the device pointer (allocating and uploading on `stream` first when
 * the array was evicted or never uploaded) and keeps the array resident until
 * the matching release; release names the stream the array was used on, and
 * the block is neither evicted nor handed to another array before the work
 * queued at that moment on every stream it was released on has completed.
 * An acquire on another stream while the upload is still in flight makes that
 * stream wait for the upload.  Ordering between the kernel that produces an
 * array and its consumers on other streams stays with the caller (events, as
 * Execute.hs:104-105 does with `after`).  Acquires nest.                      */
int acc_memtable_acquire(acc_memtable mt, uint64_t key, acc_stream stream, acc_devptr *out);
int acc_memtable_release(acc_memtable mt, uint64_t key, acc_stream stream);

/* free, Array/Remote.hs:160-170: the host array is gone.  The block goes to
 * the nursery once work recorded at the last release has completed.          */
int acc_memtable_free(acc_memtable mt, uint64_t key);

/* insertUnmanaged, Array/Remote.hs:177-189: device memory the table did not
 * allocate; it is never evicted, reused or freed by the table                */
int acc_memtable_insert_unmanaged(acc_memtable mt, uint64_t key, acc_devptr p, uint64_t bytes);

/* reclaim, Array/Remote.hs:195-196: return the nursery to the device         */
int acc_memtable_reclaim(acc_memtable mt);

typedef struct acc_memtable_stats {
  uint64_t resident_bytes;     /* device bytes under live keys (rounded sizes) */
  uint64_t nursery_bytes;
  uint64_t arrays, resident_arrays;
  uint64_t device_allocs;      /* hipMalloc calls */
  uint64_t nursery_hits;       /* allocations served from the nursery */
  uint64_t uploads, upload_bytes;
  uint64_t evictions, writebacks, writeback_bytes;
} acc_memtable_stats;
int acc_memtable_get_stats(acc_memtable mt, acc_memtable_stats *out);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif
#ifdef __cplusplus
}
#endif
#endif /* ACC_HIP_H */

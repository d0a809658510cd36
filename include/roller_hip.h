/* roller_hip.h -- C ABI of libroller_hip.so: JIT, load, launch and time the Roller fp32 GEMM on
 * one MI355X (gfx950).
 *
 * The reference (NaOHCC/mlir-roller) reaches its GPU through CuPy from Python; this library is
 * what a maintainer binds instead (ctypes, cgo, JNI ... -- plain pointers and sizes only).  Each
 * entry point names the reference call it replaces as file:line under /root/reference/.
 *
 * Conventions
 *   - every function returns an int status: 0 = success, > 0 = a hipError_t, < 0 = an RL_ERR_*
 *     code below.  rl_last_error() returns the text for the last failure on the calling thread.
 *   - handles are opaque pointers owned by the library; device memory is owned by whoever
 *     allocated it (rl_malloc'd memory is freed by rl_free and by nothing else).
 *   - one device per process (the reference pins one GPU through its environment, .env:5-6);
 *     calls are synchronous with respect to the host except rl_launch / rl_gemm_* / rl_event_record,
 *     which enqueue on the given stream (NULL = the default stream).
 *   - the library is thread-safe: every entry point selects the device of rl_init on the calling
 *     thread, plan creation and the cache directory are serialised, launches of plans may run
 *     concurrently with each other, and rl_gemm_plans_clear waits for running launch calls and for
 *     the device before it unloads anything.  rl_module_unload likewise drains the device first.
 *     Error text is thread-local.
 */
#ifndef ROLLER_HIP_H
#define ROLLER_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RL_OK 0
#define RL_ERR_INVALID_ARG (-1001) /* bad pointer, shape, stride, alignment or tile parameter */
#define RL_ERR_COMPILE (-1002)     /* hiprtc rejected the program; see the build log */
#define RL_ERR_IO (-1003)          /* code-object cache could not be read or written */
#define RL_ERR_NO_DEVICE (-1004)   /* no usable HIP device */

typedef void* rl_module;
typedef void* rl_function;
typedef void* rl_stream;
typedef void* rl_event;
typedef struct rl_gemm_plan rl_gemm_plan;

/* What the rTile policy needs to know about the device (mirrors the fields of TileDevice,
 * src/arch.py:9-37, that can be read from the runtime). */
typedef struct rl_device_props {
  char name[128];
  char arch[64];            /* e.g. "gfx950:sramecc+:xnack-" */
  int compute_units;        /* 256 on MI355X */
  int wavefront_size;       /* 64 */
  int lds_bytes_per_block;  /* largest LDS allocation one workgroup may opt into */
  int regs_per_block;
  int l2_bytes;
  int clock_khz;            /* peak engine clock */
  int mem_clock_khz;
  int mem_bus_bits;
  size_t total_mem_bytes;
} rl_device_props;

/* Tile configuration of the fp32 GEMM kernel template; one field per template parameter.
 * Replaces the (block_tile, thread_tile, rstep, pipeline_depth) tuple that the reference feeds
 * to GEMMBuilder.build_transform_pipeline (src/roller.py:93-99). */
typedef struct rl_gemm_config {
  int bm, bn;      /* block tile            <- hint.block_tile                       */
  int bk;          /* K step                <- hint.rstep                            */
  int wm, wn;      /* wave tile             <- 64 lanes x hint.thread_tile           */
  int mi;          /* 32: v_mfma_f32_32x32x2_f32, 16: v_mfma_f32_16x16x4_f32        */
  int stages;      /* pipeline depth 1..5   <- pipeline_depth: 1, 2, 2, 3, 4 LDS buffers;
                      3 adds a register stage, 4 and 5 need direct=1                 */
  int pad_a, pad_b;/* LDS row padding in floats (multiples of 4)                     */
  int vec;         /* 4: 128-bit global accesses, 1: dword accesses (any K, N, ld)   */
  int edge;        /* 1: ragged tiles predicated (any M, N, K), 2: M and N may be ragged,
                      bk|K required, 0: bm|M, bn|N, bk|K required                     */
  int swz;         /* bit0: XCD-contiguous tile order, bit1: panel walk              */
  int group;       /* panel height in tiles (reference: panel-width=8, roller.py:338)*/
  int accum;       /* 0: C = A*B, 1: C += A*B (linalg.matmul semantics, roller.py:62)*/
  int direct;      /* 1: global loads write LDS directly (no staging registers, swizzled
                      A rows); needs stages>=3, pad_a=pad_b=0, bk a power of 2, and with
                      vec=1 stages=3 and edge=1                                       */
  int trans_b;     /* 1: the second operand is Bt[N][ldb>=K], C = A*Bt^T (the [spatial, reduce]
                      layout of MatmulConfig.get_input_shapes, src/analyze.py:33-41); pad_b then
                      pads the K-contiguous rows of its LDS tile like pad_a                   */
  int streamk;     /* 0: one workgroup per tile of C, grid (ceil(N/bn), ceil(M/bm)) as at src/roller.py:536.
                      1..8: a fixed grid of that many workgroups per CU; each works one tile of every full
                      round of the grid and an equal share of the (tile, K step) units of the tiles left
                      over, and tiles whose K range is split are summed in K order through a workspace.  Stands in for what the reference gets from ranking tilings by rounds of
                      blocks (num_wave, src/analyze.py:164-166).  Needs stages=3                     */
} rl_gemm_config;

/* How a stream-K configuration splits one problem (rl_gemm_streamk_schedule). */
typedef struct rl_streamk_schedule {
  int grid;             /* workgroups launched */
  int k_steps;          /* K steps per tile */
  int tiles, tile_rows, tile_cols;
  long units;           /* tiles * k_steps; every workgroup gets units / grid of them, give or take one */
  size_t workspace_bytes, counter_bytes;
  int whole_tiles;      /* a multiple of grid: the first so many tiles (in walk order) are worked whole,
                           tile round * grid + g by workgroup g, after its share of the units of the rest */
} rl_streamk_schedule;

/* One run of K steps of one tile, as a workgroup of a stream-K launch works it. */
typedef struct rl_streamk_segment {
  int tile, tile_m, tile_n;  /* tile number in walk order (its arrival counter), tile row and column */
  int k_begin, k_end;        /* K steps [k_begin, k_end) of the tile */
  int pieces;                /* workgroups that share the tile (1: this segment is the whole tile) */
  int first_workgroup;       /* the one with the tile's first K steps; the pieces follow in workgroup order */
  int slot;                  /* workspace slot this piece is stored in, -1 if pieces == 1 */
} rl_streamk_segment;

/* ---- library / device ---------------------------------------------------------------------- */

/* Selects `device` and creates the HIP context.  Idempotent.  Replaces CuPy's implicit context
 * creation on first use (src/roller.py:532). */
int rl_init(int device);

/* Fills *out for the device chosen by rl_init.  Replaces the hard-coded device constants of
 * src/arch.py:41-61 with values read from the runtime. */
int rl_device_info(rl_device_props* out);

/* Text of the last error raised on this thread ("" if none).  Replaces the Python exceptions
 * that benchmark.py:55-58 catches per hint. */
const char* rl_last_error(void);

/* ---- JIT: hiprtc ---------------------------------------------------------------------------- */

/* Compiles HIP source text for gfx950.  On success *code / *code_size receive a malloc'd code
 * object.  *log (may be NULL) receives the malloc'd build log, also on failure.  Free both with
 * rl_free_host.  Replaces Lower.lower_module (src/roller.py:468-496): MLIR -> PTX. */
int rl_compile(const char* source, const char* name, const char* const* options, int n_options,
               void** code, size_t* code_size, char** log);
void rl_free_host(void* p);

/* Replace cp.cuda.Module().load / get_function / funcSetAttribute(MAX_DYNAMIC_SHARED_SIZE_BYTES)
 * (src/roller.py:504-510). */
int rl_module_load(const void* code, rl_module* out);
int rl_module_get_function(rl_module m, const char* name, rl_function* out);
int rl_module_unload(rl_module m);
/* Fails with RL_ERR_INVALID_ARG and text when the runtime grants less than `bytes` (the limit is
 * read back after the opt-in: function attribute where the runtime keeps one, otherwise the
 * device's per-workgroup LDS minus the function's static LDS). */
int rl_func_set_max_dynamic_lds(rl_function f, int bytes);

/* Launches f.  `args` holds n_args pointers, one per kernel parameter, each pointing at that
 * parameter's value.  Replaces cuda_func(grid, block, args, shared_mem=) (src/roller.py:545-550). */
int rl_launch(rl_function f, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by,
              unsigned bz, unsigned lds_bytes, rl_stream stream, void** args, int n_args);

/* ---- device memory: replaces cp.random.rand / cp.zeros / .data.ptr (src/roller.py:532-534) -- */
int rl_malloc(void** dptr, size_t bytes);
int rl_free(void* dptr);
int rl_memcpy_h2d(void* dst, const void* src, size_t bytes);
int rl_memcpy_d2h(void* dst, const void* src, size_t bytes);
int rl_memset(void* dptr, int byte_value, size_t bytes);

/* ---- streams and events: replace cp.cuda.Event / get_elapsed_time (src/roller.py:514-522,580) */
int rl_stream_create(rl_stream* out);
int rl_stream_destroy(rl_stream s);
int rl_event_create(rl_event* out);
int rl_event_record(rl_event e, rl_stream s);
int rl_event_sync(rl_event e);
int rl_event_elapsed_ms(rl_event start, rl_event stop, float* ms);
int rl_event_destroy(rl_event e);
int rl_sync(void);

/* ---- the GEMM path itself -------------------------------------------------------------------
 * The kernel template is part of the library.  A plan is one compiled instance of it:
 * Compiler(config, hint, pipeline_depth).compile() of src/roller.py:345-387. */

/* The HIP source of the kernel template (NUL-terminated, owned by the library). */
const char* rl_gemm_template_source(void);

/* Checks cfg against the template's constraints without compiling.  *lds_bytes (may be NULL)
 * receives the dynamic LDS size = buffers(stages) * (bm*(bk+pad_a) + bk*(bn+pad_b)) * 4
 * (bn*(bk+pad_b) for the second term when trans_b), the padded
 * counterpart of hint.smem_cost * pipeline_depth (src/roller.py:385); *threads (may be NULL)
 * receives 64 * (bm/wm) * (bn/wn). */
int rl_gemm_config_check(const rl_gemm_config* cfg, int* lds_bytes, int* threads);

/* Directory of the on-disk code-object cache (NULL or "" disables it).  Files are keyed by a hash
 * of template source, options and hiprtc version; each file is the code object plus a 16-byte
 * trailer with its checksum, and a file that fails the check, or that the driver refuses to load,
 * is recompiled in place.  The reference has no cache: it rebuilds every (shape, hint) from
 * scratch (src/roller.py:358-387). */
int rl_set_cache_dir(const char* path);

/* Compiles cfg without touching a device and stores the code object in the cache directory
 * (ahead-of-time warm-up; works on a machine that has no GPU).  *code_size (may be NULL) receives
 * the size of the code object, 16 bytes less than the cache file. */
int rl_gemm_precompile(const rl_gemm_config* cfg, size_t* code_size);

/* JIT-compiles (or fetches from the in-process / on-disk cache) and loads the kernel for cfg.
 * Plans are shared: creating the same cfg twice returns the same plan.  *compile_ms (may be NULL)
 * receives the time spent in hiprtc, 0 on a cache hit. */
int rl_gemm_plan_create(const rl_gemm_config* cfg, rl_gemm_plan** out, float* compile_ms);
int rl_gemm_plan_function(const rl_gemm_plan* plan, rl_function* out);
int rl_gemm_plan_lds_bytes(const rl_gemm_plan* plan);
/* Dynamic LDS bytes the runtime grants the plan's kernel, read back after the opt-in that the
 * reference does with funcSetAttribute(MAX_DYNAMIC_SHARED_SIZE_BYTES) (src/roller.py:508-510);
 * rl_gemm_plan_create fails with text when it is below rl_gemm_plan_lds_bytes. */
int rl_gemm_plan_lds_limit(const rl_gemm_plan* plan);
int rl_gemm_plan_threads(const rl_gemm_plan* plan);
/* What hiprtc printed when it compiled the plan's kernel ("" if nothing, or if the code object came
 * from the on-disk cache); owned by the library, valid while the plan is.  The counterpart of the IR
 * dumps of src/roller.py:480-495. */
const char* rl_gemm_plan_build_log(const rl_gemm_plan* plan);
/* Kernel resource usage read from the code object's metadata (-1 if unknown). */
int rl_gemm_plan_resources(const rl_gemm_plan* plan, int* vgprs, int* agprs, int* sgprs,
                           int* spilled, int* scratch_bytes);
/* Drops every plan and unloads its module.  Handles obtained earlier stay safe to pass in: the
 * plan entry points refuse them with RL_ERR_INVALID_ARG.  No counterpart in the reference, which
 * keeps every CuPy module alive until the process ends. */
int rl_gemm_plans_clear(void);

/* Enqueues C = A*B (or C += A*B when cfg.accum) for row-major fp32 device matrices
 * A[M,lda>=K], B[K,ldb>=N] (Bt[N,ldb>=K] when cfg.trans_b), C[M,ldc>=N].  Grid is (ceil(N/bn), ceil(M/bm)) as at
 * src/roller.py:536 (the reference floors; ragged tiles are predicated here when cfg.edge).
 * Rejects, with RL_ERR_INVALID_ARG and before anything is launched, shapes the plan was not built
 * for: vec=4 with K, N or a leading dimension not a multiple of 4 or a base pointer not 16-byte
 * aligned; edge=0 with a dimension that its tile does not divide; edge=2 with bk not dividing K.  M==0 or N==0 is a no-op;
 * K==0 writes zeros (or leaves C when accumulating). */
int rl_gemm_plan_launch(const rl_gemm_plan* plan, const float* A, const float* B, float* C,
                        int M, int N, int K, int lda, int ldb, int ldc, rl_stream stream);

/* Stream-K plans (cfg.streamk > 0) need a workspace: arrival counters (one unsigned per tile, zero
 * before a launch; the kernel leaves them at zero; the area is 256 KiB for up to 65536 tiles and
 * grows beyond) followed by two slots of bm*bn floats per workgroup.  rl_gemm_plan_launch takes it from the library, which keeps one per stream (allocated or
 * grown on first need, which synchronises that stream; launches on one stream run in order, and
 * launches on different streams use different workspaces).  rl_gemm_plan_launch_ws takes it from the
 * caller: `workspace` is device memory, 256-byte aligned, of at least rl_gemm_plan_workspace_bytes
 * bytes, whose first *counter_bytes bytes were zero before its first use -- and are zeroed again by
 * the caller before a launch whose *counter_bytes is larger than that of the launches the workspace
 * has served (only launches of more than 65536 tiles: their counters reach into what held the slots
 * of the others); launches that share a workspace must not overlap on the device.  For a plan without streamk both behave like
 * rl_gemm_plan_launch and the workspace is ignored (bytes = 0).  No counterpart in the reference
 * (src/roller.py:545-550 launches one block per tile). */
int rl_gemm_plan_workspace_bytes(const rl_gemm_plan* plan, int M, int N, int K, size_t* bytes, size_t* counter_bytes);
int rl_gemm_plan_launch_ws(const rl_gemm_plan* plan, const float* A, const float* B, float* C,
                           int M, int N, int K, int lda, int ldb, int ldc, void* workspace,
                           size_t workspace_bytes, rl_stream stream);

/* rl_gemm_plan_launch for callers that cannot allocate device memory: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  It calls no
 * hipMalloc / hipFree / allocating routine on any path: a stream-K plan takes its workspace from a
 * fixed array in device memory that is part of the library's own code object (256 KiB of arrival
 * counters + 64 MiB of slots; every GPU the library runs on holds it until the process ends), and a
 * launch that needs more -- more than 65536 tiles, or 2 * workgroups * bm * bn * 4 bytes beyond 64 MiB
 * -- is refused with RL_ERR_INVALID_ARG and text.  All calls on a GPU share that one array: calls that
 * overlap on the device (different streams) race; calls on one stream do not.  The kernels leave the
 * counters at zero, the slots keep the last call's pieces (every call overwrites what it reads).  For a
 * plan without streamk it is rl_gemm_plan_launch.  K == 0 writes zeros with a small fill kernel
 * (never a memset call, so the launch may sit in a captured graph). */
int rl_gemm_plan_launch_static(const rl_gemm_plan* plan, const float* A, const float* B, float* C,
                               int M, int N, int K, int lda, int ldb, int ldc, rl_stream stream);

/* The split of an M x N x K problem under a stream-K configuration on a device with `compute_units`
 * CUs, and the segments that workgroup `workgroup` works (at most `capacity` are written, *count
 * receives how many there are).  Host arithmetic only (no device needed): what the policy's cost
 * model and the tests read.  Replace the grid_size / num_wave fields of TileDict (src/analyze.py:150-166). */
int rl_gemm_streamk_schedule(const rl_gemm_config* cfg, int M, int N, int K, int compute_units,
                             rl_streamk_schedule* out);
int rl_gemm_streamk_segments(const rl_gemm_config* cfg, int M, int N, int K, int compute_units,
                             int workgroup, rl_streamk_segment* out, int capacity, int* count);

/* One call for hosts that do not keep plans: plan_create (cached) + plan_launch. */
int rl_gemm_f32(const rl_gemm_config* cfg, const float* A, const float* B, float* C, int M,
                int N, int K, int lda, int ldb, int ldc, rl_stream stream);

#ifdef __cplusplus
}
#endif
#endif /* ROLLER_HIP_H */

/*
 * libbfuse_rt -- C ABI of the MI355X fused-pair runtime.
 *
 * Plain C: pointers, ints and POD structs only.  Every function returns 0 on success and a
 * negative code on failure (bfuse_last_error() holds the text) unless stated otherwise.
 * The library is not re-entrant: like the reference harness it keeps one set of device
 * buffers and two streams in file-scope state (operation_cu.py:123-126).
 *
 * Citations are paths in the reference repository (jiny0ung97/bfuse-project).
 */
#ifndef BFUSE_RT_H
#define BFUSE_RT_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------------------------
 * Status
 * ---------------------------------------------------------------------------------------- */
enum {
    BFUSE_OK = 0,
    BFUSE_ERR_ARG = -1,      /* bad argument (null pointer, unknown name, shape mismatch) */
    BFUSE_ERR_HIP = -2,      /* a HIP runtime call failed; replaces CHECK_CUDA's exit(EXIT_FAILURE),
                                operation_cu.py:111-121 */
    BFUSE_ERR_STATE = -3,    /* called before bfuse_init / initialize_kernelN */
    BFUSE_ERR_SYNC = -4      /* a side of a fused kernel gave up waiting on its LDS barrier: the kernel ran to its
                                end, but that side carried on unsynchronised, so its output (and any timing of
                                the launch) is not to be trusted.  Reported by the first call that synchronises
                                after the launch: run_fuse, bfuse_synchronize, bfuse_download, bfuse_time,
                                bfuse_time_batched, bfuse_module_launch with us_out, bfuse_module_unload */
};
const char* bfuse_last_error(void);

/* Selects the device and creates the two streams the harness uses (S1, S2 of
 * operation_cu.py:126).  Fails if no HIP device is present: there is no CPU fallback. */
int bfuse_init(int device);
/* Waits for everything launched, frees the buffers of every side still initialized and unloads every code
 * object still loaded.  Calling it before bfuse_init (or twice) is harmless.  bfuse_init may be called again
 * afterwards; calling it for another device while a side still holds buffers is refused. */
int bfuse_shutdown(void);
/* name, CU count, LDS bytes per workgroup, wavefront size of the selected device */
int bfuse_device_info(char* name, size_t name_len, int* compute_units, int* lds_bytes, int* wave_size);
/* free and total device memory of the selected device in bytes (hipMemGetInfo); either may be NULL */
int bfuse_device_memory(size_t* free_bytes, size_t* total_bytes);

/* ------------------------------------------------------------------------------------------
 * Fusion index maps -- horizontal-fuser/src/Algorithms.cc.  Pure host arithmetic, usable
 * without a GPU.  The same code is compiled into the fused kernels.
 * ---------------------------------------------------------------------------------------- */
#define BFUSE_MAX_KERNELS 4
#define BFUSE_MAX_SEGMENTS 8

/* GridDim / BlockDim of one kernel -- horizontal-fuser/include/fuse/Contexts.h:13-26 */
typedef struct { int grid[3]; int block[3]; } bfuse_launch_dims;

typedef struct { int kern, off, width, base; } bfuse_slot;
typedef struct { int lo, hi, period, n_slot; bfuse_slot slot[BFUSE_MAX_KERNELS]; } bfuse_segment;
/* Block-fusion dispatch table: fused block `bid` in segment [lo,hi) belongs to the slot that
 * owns (bid-lo) % period; virt = base + ((bid-lo)/period)*width + ((bid-lo)%period - off). */
typedef struct {
    int n_kernels, n_seg;
    bfuse_segment seg[BFUSE_MAX_SEGMENTS];
    int fused_grid, fused_block;
    int threads[BFUSE_MAX_KERNELS];
} bfuse_block_plan;

typedef struct {
    int n_kernels;
    int thr_lo[BFUSE_MAX_KERNELS], thr_hi[BFUSE_MAX_KERNELS];
    int blocks[BFUSE_MAX_KERNELS];
    int fused_grid, fused_block;
} bfuse_thread_plan;

enum {
    BFUSE_PATTERN_ZIGZAG = 0,        /* coarseInterleaveWithoutSMPattern2, Algorithms.cc:528-739; p0 = M, p1 = N */
    BFUSE_PATTERN_PROPORTIONAL = 1,  /* coarseInterleaveWithoutSMPattern,  Algorithms.cc:319-526; p0 = MinOption */
    BFUSE_PATTERN_CHUNKED = 2,       /* coarseInterleavePattern,           Algorithms.cc:118-317; p0 = TotalSM */
    BFUSE_PATTERN_RANGES = 3         /* blockIdx ranges only (the tail branches, Algorithms.cc:661-685) */
};

/* hfusePattern, Algorithms.cc:19-116.  pad = 32 reproduces the reference, 64 is what the
 * gfx950 kernels use (one wavefront never holds threads of two operators). */
int bfuse_plan_threads(int n, const bfuse_launch_dims* kernels, int pad, bfuse_thread_plan* out);
int bfuse_plan_blocks(int pattern, int n, const bfuse_launch_dims* kernels, int p0, int p1,
                      bfuse_block_plan* out);
/* Return the kernel index owning the id (or -1 if none, or if plan is null) */
int bfuse_map_block(const bfuse_block_plan* plan, int bid, int* virt_block);
int bfuse_map_thread(const bfuse_thread_plan* plan, int bid, int tid, int* local_tid);
/* Evaluates bfuse_map_block for bid in [lo,hi) ON THE GPU with the device build of the map
 * (one thread per fused block) and copies the tables back. */
/* Placement probe: launches `workgroups` workgroups of `threads` threads that each record where
 * the hardware put them (XCD, shader engine, CU within the engine, SIMD) and when they started
 * (100 MHz wall-clock ticks), holding their slot for `hold` clock reads.  The counterpart of the
 * reference's `%smid` experiment (legacy/tests/block_scheduler_test/cuda/kernels.cu, the
 * "Block: %d | SM: %d" printf) -- on MI355X the answer decides which dispatch pattern works.
 * Output arrays have `workgroups` entries; any may be NULL. */
int bfuse_probe_placement(int workgroups, int threads, int hold, unsigned* xcc, unsigned* se, unsigned* cu, unsigned* simd,
                          unsigned long long* start_ticks);

/* Installs `plan` in a run-time-plan kernel (`<K1>_<K2>_fused_bfuse_rt`, kind 3): the same block
 * fusion, with the dispatch table as data instead of compiled in, so patterns and M:N ratios can
 * be swept without rebuilding (the reference's sweep edits Contexts.cc and rebuilds per ratio,
 * legacy/tests/single_bgemm_conv2d/auto.py:9-14).  The plan must map the fused block ids
 * one-to-one onto the blocks of the two sides; anything else is refused.  Afterwards the kernel
 * may be launched (mode BFUSE_MODE_BFUSE) with any 1-D grid from 1 to plan->fused_grid
 * workgroups: workgroup w handles fused blocks w, w + grid, ... (persistent workgroups, the
 * reference's legacy/tests/thread_pooling_test/temp.cu:576-612). */
int bfuse_set_plan(const void* func, const bfuse_block_plan* plan);

int bfuse_map_blocks_device(const bfuse_block_plan* plan, int lo, int hi, int* kernel_out, int* virt_out);

/* bfuse_map_blocks_device without any allocation.  No counterpart in the reference: it is for
 * callers that cannot allocate device memory where they call -- tight serving loops, harnesses that
 * forbid hipMalloc.  Same arguments and results; the two tables are staged in a fixed device array of
 * the library (2 x BFUSE_NOALLOC_MAX_IDS ints = 2 MiB per GPU, held until the process ends) whose
 * address is looked up in bfuse_init.  Like the allocating entry point it is synchronous: it launches
 * on the default stream and copies the tables into the caller's host arrays before it returns, so it
 * is not a call to make while a stream is being captured into a graph.  hi - lo above
 * BFUSE_NOALLOC_MAX_IDS is refused (BFUSE_ERR_ARG).  Calls on one GPU share that array: calls that
 * overlap on one GPU race. */
#define BFUSE_NOALLOC_MAX_IDS 262144
int bfuse_map_blocks_device_noalloc(const bfuse_block_plan* plan, int lo, int hi, int* kernel_out, int* virt_out);

/* Side barriers of horizontally fused and run-time-plan kernels (the replacement for the
 * reference's `bar.sync id, n`, horizontal-fuser/src/Matchers.cc:288-320) poll an LDS counter a
 * bounded number of times, then give up and report BFUSE_ERR_SYNC.  This sets the bound (polls,
 * default 4194304) for every kernel built into the same module as `func`. */
int bfuse_set_sync_spin_limit(const void* func, unsigned polls);

/* ------------------------------------------------------------------------------------------
 * Kernel registry -- the role of the reference's generated macro.h tables
 * (test-utils/test-suite-files/macro_h.py:79-198) and of kernels.yaml / {b,h}fuse_kernels.yaml
 * (horizontal-fuser/include/fuse/Utils.h:70-112).
 * ---------------------------------------------------------------------------------------- */
enum { BFUSE_KIND_SINGLE = 0, BFUSE_KIND_BFUSE = 1, BFUSE_KIND_HFUSE = 2, BFUSE_KIND_BFUSE_RT = 3 /* block fusion, plan set at run time */ };

typedef struct {
    char name[128];          /* KernelName; fused: <K1>_<K2>_fused_{bfuse,hfuse} (Contexts.cc:56-92) */
    const void* func;        /* launch handle: pass as `func` to run_kernelN / run_fuse */
    int kind;
    unsigned grid[3], block[3];
    int has_barriers;        /* KernelInfo.HasBarriers */
    int regs;                /* KernelInfo.Reg: VGPRs per lane from the code object (-1 without a GPU) */
    int lds_bytes;           /* static LDS of the kernel (-1 without a GPU) */
    int shape[3][4];         /* single kernels: I, F, O shapes, padded with 1s */
    int elem_bytes[3];
    char side[2][64];        /* fused kernels: the first two standalone kernels */
    int pattern, p0, p1;     /* bfuse kernels: dispatch pattern */
    int n_sides;             /* 1 for a standalone kernel; fused: how many kernels it runs (3 pointers each, in order) */
    char side_more[BFUSE_MAX_KERNELS - 2][64];   /* fused kernels of more than two: the third, fourth standalone kernel */
    int matrix_cores;        /* single kernels: 1 if the operator's inner loop is a stream of MFMAs (GEMMs, convolutions) */
} bfuse_kernel_info;

/* bfuse_kernel_count / bfuse_kernel_at enumerate every kernel except the library's self-test operators
 * (names starting with `selftest_`), which bfuse_kernel_find still finds by name. */
int bfuse_kernel_count(void);
int bfuse_kernel_at(int index, bfuse_kernel_info* out);
int bfuse_kernel_find(const char* name, bfuse_kernel_info* out);

/* Fused kernels built after the library.  The reference generates and compiles the fused kernels of a suite
 * when the suite is configured (scripts/configure_kernels.py:229-320 runs the fuser over every pair of the
 * user's config; CMakeLists_txt.py compiles the result into the suite's binary).  Here
 * `python -m bfuse_project_amd.build_pairs <suite dir>` writes the pairs of a configured suite that the library
 * holds no fused kernel for as instantiations over the registered operators' own types and compiles them into
 * one shared object per suite; bfuse_load_kernels adds its kernels to the registry (by name, like the built-in
 * ones).  Modules named in the environment variable BFUSE_KERNEL_MODULES (paths separated by ':') are loaded
 * before the first look at the registry, whatever the program.
 * bfuse_kernel_op_type: the C++ type of a standalone kernel's operator, spelled with every template argument
 * (NULL for unknown names and fused kernels) -- what such a module names its sides by.
 * bfuse_kernel_op_lds: the bytes of LDS that operator's body declares (-1 likewise), known without a device:
 * whether two operators fit one workgroup is decided from it before anything is compiled. */
int bfuse_load_kernels(const char* shared_object_path);
const char* bfuse_kernel_op_type(const char* name);
int bfuse_kernel_op_lds(const char* name);

/* ------------------------------------------------------------------------------------------
 * Harness functions -- test-utils/test-suite-files/operation_h.py:9-27.  Same names and
 * argument meaning.  Differences: data pointers are void* (bf16 sides), an int status is
 * returned instead of exit(), and `func` is the registry handle of a kernel with the
 * reference's three- / six-pointer ABI.  K / K1 / K2 (the reference's switch index into the
 * fusion sets) are accepted and ignored.
 * ---------------------------------------------------------------------------------------- */
typedef void (*bfuse_kernel3_fn)(const void*, const void*, void*);
typedef void (*bfuse_kernel6_fn)(const void*, const void*, void*, const void*, const void*, void*);

/* element sizes of side 1 / side 2 buffers (default 4 = float, as in the reference) */
int bfuse_set_elem_bytes(int side, int i_bytes, int f_bytes, int o_bytes);

/* device alloc of I/F/O for one side + stream create -- operation_cu.py:128-144 */
int initialize_kernel1(const int* I_shape, const int* F_shape, const int* O_shape);
int initialize_kernel2(const int* I_shape, const int* F_shape, const int* O_shape);
/* operation_cu.py:146-162 */
int finalize_kernel1(void);
int finalize_kernel2(void);
/* H2D of I,F; launch on the default stream; device sync; D2H of O -- operation_cu.py:164-201 */
int run_kernel1(const void* I, const void* F, void* O, const int* I_shape, const int* F_shape,
                const int* O_shape, bfuse_kernel3_fn func, const unsigned* gridDim,
                const unsigned* blockDim, size_t K);
int run_kernel2(const void* I, const void* F, void* O, const int* I_shape, const int* F_shape,
                const int* O_shape, bfuse_kernel3_fn func, const unsigned* gridDim,
                const unsigned* blockDim, size_t K);
/* both kernels, one per stream -- operation_cu.py:203-229 */
int run_parallel(const void* I1, const void* F1, void* O1, const void* I2, const void* F2, void* O2,
                 const int* I1_shape, const int* F1_shape, const int* O1_shape, const int* I2_shape,
                 const int* F2_shape, const int* O2_shape, bfuse_kernel3_fn func1, bfuse_kernel3_fn func2,
                 const unsigned* gridDim1, const unsigned* blockDim1, const unsigned* gridDim2,
                 const unsigned* blockDim2, size_t K1, size_t K2);
/* one fused kernel over both sides' buffers -- operation_cu.py:231-256 */
int run_fuse(const void* I1, const void* F1, void* O1, const void* I2, const void* F2, void* O2,
             const int* I1_shape, const int* F1_shape, const int* O1_shape, const int* I2_shape,
             const int* F2_shape, const int* O2_shape, bfuse_kernel6_fn func, const unsigned* gridDim,
             const unsigned* blockDim, size_t K1, size_t K2);

/* ------------------------------------------------------------------------------------------
 * Device-resident operation and GPU-side timing.  The reference copies H2D/D2H around every
 * launch but reports only the profiler's GPU-side kernel durations
 * (scripts/profile_test_suite.py:10-11,106-109; scripts/analyze_test_suite.py:103-161);
 * these entry points keep the operands in HBM and return those durations directly.
 * ---------------------------------------------------------------------------------------- */
int bfuse_upload(int side, const void* I, const void* F);   /* side 1 .. BFUSE_MAX_KERNELS */
int bfuse_zero_output(int side);
int bfuse_download(int side, void* O);
int bfuse_synchronize(void);

/* The same for a part of a tensor: operands and results of several GB (the reference's benchmark.yaml runs every
 * operator at batch 1024) need not pass through one host array.  `tensor`: 0 = I, 1 = F; offsets and sizes in
 * bytes.  No counterpart in the reference, whose harness copies whole tensors (operation_cu.py:74-118). */
int bfuse_upload_part(int side, int tensor, size_t offset, const void* src, size_t bytes);
int bfuse_download_part(int side, size_t offset, void* dst, size_t bytes);
/* Checksums of the side's output, computed on the device: the output is cut into chunks of `chunk_bytes`
 * (a multiple of 4 that divides it; at most 65535 chunks) and sums[2c], sums[2c+1] receive, mod 2^64, the sum
 * of chunk c's 32-bit words w[i] and the sum of w[i] * (i mod 65521 + 1).  Two runs wrote the same bytes iff
 * (up to collisions) their sums agree -- the comparison the reference makes on the host with check_matrix
 * (operation_cu.py:29-45), for outputs too large to copy back. */
int bfuse_checksum_output(int side, size_t chunk_bytes, unsigned long long* sums);
/* Fills tensor 0 (I) or 1 (F) of the side, on the device, with the values bfuse_fill_uniform(seed, n, lo, hi)
 * writes on the host (fp32 tensors) or their bfuse_f32_to_bf16 roundings (bf16 tensors): the reference's harness
 * fills host arrays with rand() and copies them (utils_cc.py:28-31); operands of several GB are written where
 * they are needed instead. */
int bfuse_fill_uniform_device(int side, int tensor, unsigned long long seed, float lo, float hi);

enum {
    BFUSE_MODE_KERNEL1 = 0,   /* the reference CLI's T = 0..4 (main_cc.py:22-36) */
    BFUSE_MODE_KERNEL2 = 1,
    BFUSE_MODE_PARALLEL = 2,  /* two streams */
    BFUSE_MODE_HFUSE = 3,
    BFUSE_MODE_BFUSE = 4,
    BFUSE_MODE_SERIAL = 5     /* kernel 1 then kernel 2 on one stream, no host sync in between */
};

/* One asynchronous launch of `mode` over the resident buffers (no copies, no sync).
 * func_a/grid_a/block_a: kernel 1 (modes 0,2,5) or the fused kernel (modes 3,4) or kernel 2 (mode 1);
 * func_b/...: kernel 2 (modes 2,5). */
int bfuse_launch(int mode, const void* func_a, const unsigned* grid_a, const unsigned* block_a,
                 const void* func_b, const unsigned* grid_b, const unsigned* block_b);

/* `warmup` untimed + `reps` timed launches of `mode`; GPU timestamps of each kernel's own
 * start and end.  us_total[r] = first kernel start -> last kernel end of repetition r;
 * us_a[r], us_b[r] = duration of each kernel (us_b only for modes 2 and 5; may be NULL).
 * In mode 2 the device is synchronised after every repetition, as the reference's run_parallel
 * does (operation_cu.py:199-228): two free-running streams would drift whole launches apart. */
int bfuse_time(int mode, const void* func_a, const unsigned* grid_a, const unsigned* block_a,
               const void* func_b, const unsigned* grid_b, const unsigned* block_b, int warmup, int reps,
               float* us_total, float* us_a, float* us_b);

/* Wall-clock throughput: `reps` launches of `mode` enqueued back to back between two stream
 * events; returns the mean microseconds per launch (includes dispatch gaps). */
int bfuse_time_batched(int mode, const void* func_a, const unsigned* grid_a, const unsigned* block_a,
                       const void* func_b, const unsigned* grid_b, const unsigned* block_b, int warmup,
                       int reps, float* us_per_launch);

/* The same measurement with the launches replayed from a HIP graph: `chain` repetitions of `mode` are captured
 * once (mode 5: the two kernels as a chain of dependent nodes; mode 2: as two independent nodes between a fork
 * and a join, repetition after repetition; modes 0, 1, 3, 4: one node per repetition), the graph is launched
 * once untimed and `reps` times between two stream events; returns the mean microseconds per repetition of
 * `mode`.  What it tells: how much of the back-to-back figure is the host's launch path -- the unfused pair as a
 * graph is the strongest form of the baseline the reference's run_kernel1 + run_kernel2 stand for
 * (operation_cu.py:128-197; the reference has no graph path).  Only kernel nodes are captured.  Under rocprofv3
 * (whose kernel tracing crashes on a graph launch on ROCm 7.2) the call is refused with BFUSE_ERR_STATE. */
int bfuse_time_graph(int mode, const void* func_a, const unsigned* grid_a, const unsigned* block_a,
                     const void* func_b, const unsigned* grid_b, const unsigned* block_b, int chain,
                     int reps, float* us_per_repetition);

/* ------------------------------------------------------------------------------------------
 * More than two kernels.  The reference's harness is two-sided (operation_h.py:9-27) while its
 * fuser takes a list of kernels of any length (horizontal-fuser/src/Algorithms.cc:23-35,540-566;
 * the fused kernel's parameters are the kernels' parameter lists one after the other,
 * Matchers.cc:523-602).  Sides 3 .. BFUSE_MAX_KERNELS are set up with the generic form of
 * initialize_kernelN / finalize_kernelN, and a launch list runs any registered kernels over any
 * sides: a standalone kernel over one side, a fused kernel over as many sides as it has kernels
 * (bfuse_kernel_info.n_sides), in the order of its pointers.
 * ---------------------------------------------------------------------------------------- */
int bfuse_initialize_side(int side, const int* I_shape, const int* F_shape, const int* O_shape);
int bfuse_finalize_side(int side);

typedef struct {
    const void* func;                 /* registry handle */
    unsigned grid[3], block[3];       /* must be the kernel's own launch shape (bfuse_kernel_info) */
    int n_sides;                      /* must equal the kernel's n_sides */
    int sides[BFUSE_MAX_KERNELS];     /* 1-based, distinct: which resident buffers each of its kernels runs over */
} bfuse_launch_desc;

/* The launches in order on the default stream, asynchronously (no copies, no host sync). */
int bfuse_launch_list(int n, const bfuse_launch_desc* launches);
/* `warmup` untimed rounds, then two measurements of `reps` rounds each (either output may be NULL):
 * us_each[j] = mean GPU-side duration of launch j (its own start and end timestamps);
 * *us_queued = wall clock per round with all rounds enqueued back to back. */
int bfuse_time_list(int n, const bfuse_launch_desc* launches, int warmup, int reps, float* us_each, float* us_queued);

/* ------------------------------------------------------------------------------------------
 * Kernels from a code object: what the horizontal-fuser front end emits (one fused HIP kernel
 * per fusion, compiled with `hipcc --genco`), or any kernel with the reference's three- /
 * six-pointer ABI (macro_h.py:182-198).  Launched over the same resident buffers as the
 * built-in kernels; the caller vouches for the launch shape (it comes from the
 * {b,h}fuse_kernels.yaml the front end wrote).
 * ---------------------------------------------------------------------------------------- */
int bfuse_module_load(const char* code_object_path, int* module_id);
int bfuse_module_unload(int module_id);
/* n_ptrs = 3: launch `kernel_name` over side `side`; n_ptrs = 6, 9, 12: over sides 1 .. n_ptrs / 3.
 * Asynchronous on the default stream; if us_out is not NULL the call synchronises and returns
 * the kernel's GPU-side duration in microseconds. */
int bfuse_module_launch(int module_id, const char* kernel_name, const unsigned* gridDim, const unsigned* blockDim,
                        int n_ptrs, int side, float* us_out);

/* ------------------------------------------------------------------------------------------
 * Seeded synthetic inputs (host side): splitmix64 counter stream -> U[lo,hi) or Box-Muller
 * N(mean,std).  Element i depends only on (seed, i).
 * ---------------------------------------------------------------------------------------- */
void bfuse_fill_uniform(unsigned long long seed, size_t n, float lo, float hi, float* out);
void bfuse_fill_normal(unsigned long long seed, size_t n, float mean, float std, float* out);
/* round-to-nearest-even conversions for bf16 buffers */
void bfuse_f32_to_bf16(size_t n, const float* in, unsigned short* out);
void bfuse_bf16_to_f32(size_t n, const unsigned short* in, float* out);

/* The reference's acceptance rule, check_matrix (test-utils/test-suite-files/utils_cc.py:52-85):
 * element wrong iff |o-a| > eps and (a == 0 or |o-a|/|a| > eps).  Returns the number of wrong
 * elements (NaN mismatches count as wrong). */
long bfuse_check_matrix(const float* O, const float* O_ans, size_t count, float eps);

#ifdef __cplusplus
}
#endif
#endif /* BFUSE_RT_H */

/* C ABI of the runtime layer that generated Tiramisu host code calls to reach the GPU.
 *
 * This is the drop-in boundary of the HIP back-end: plain pointers and sizes, no C++ or
 * framework types.  Each entry point names the reference interface it replaces
 * (src/tiramisu_cuda_wrappers.cpp of the reference tree).  Failure model of the
 * reference is kept: a failing HIP call prints "Error at <function>: <reason>" on
 * stderr and ends the process with status 1, so successful calls return 0.
 *
 * Stream model: every call works on the calling thread's *current stream*.  It starts as
 * HIP's per-thread default stream (the reference compiles with
 * --default-stream per-thread, tiramisu_codegen_cuda.cpp:1745) and can be replaced
 * with tiramisu_hip_set_stream() by callers that time or overlap work.
 */
#ifndef TIRAMISU_HIP_WRAPPERS_H
#define TIRAMISU_HIP_WRAPPERS_H

#include <stdbool.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- memory (replaces tiramisu_cuda_malloc / tiramisu_cuda_free,
 *      tiramisu_cuda_wrappers.cpp:55-68).  Freed blocks are kept for the next request of the
 *      same size (generated functions allocate and free their temporaries on every call), up to
 *      TIRAMISU_HIP_POOL_BYTES of idle memory (default 16 GiB, 0 = no pooling); tiramisu_hip_free
 *      waits for the calling thread's stream before it takes a block back. ---- */
void *tiramisu_hip_malloc(uint64_t size);
int tiramisu_hip_free(void *ptr);

/* ---- copies (replace tiramisu_cuda_memcpy_to_device / _to_host / _to_symbol,
 *      tiramisu_cuda_wrappers.cpp:34-53).  Issued with hipMemcpyAsync on the current
 *      stream and completed before returning, like the reference's cudaMemcpy. ---- */
int tiramisu_hip_memcpy_to_device(void *to, void *from, uint64_t size);
int tiramisu_hip_memcpy_to_host(void *to, void *from, uint64_t size);
int tiramisu_hip_memcpy_to_symbol(void *to, void *from, uint64_t size);
/* Device-to-device copy; the reference prints such copies as device-to-host
 * (tiramisu_codegen_cuda.cpp:1416-1419), which its runtime tolerates by accident. */
int tiramisu_hip_memcpy_device_to_device(void *to, void *from, uint64_t size);

/* ---- synchronisation (replaces tiramisu_cuda_stream_synchronize,
 *      tiramisu_cuda_wrappers.cpp:164-169); the argument is ignored ---- */
int32_t tiramisu_hip_stream_synchronize(int32_t dummy);

/* ---- GEMM library call (replaces tiramisu_cublas_sgemm / tiramisu_cublas_dgemm,
 *      tiramisu_cuda_wrappers.cpp:74-162).  Row-major C = alpha*op(A)*op(B) + beta*C,
 *      A is MxK, B is KxN after op().  A leading dimension of 0 means tightly packed
 *      (ldA = transposeA ? M : K, ldB = transposeB ? K : N, ldC = N); offsets are in
 *      elements.  Runs this library's own MFMA kernels; no BLAS library is involved. ---- */
int tiramisu_hip_sgemm(float *A, float *B, float *C, uint64_t M, uint64_t N, uint64_t K, float alpha,
                       float beta, uint64_t ldA, uint64_t ldB, uint64_t ldC, uint64_t offsetA,
                       uint64_t offsetB, uint64_t offsetC, bool transposeA, bool transposeB);
int tiramisu_hip_dgemm(double *A, double *B, double *C, uint64_t M, uint64_t N, uint64_t K, double alpha,
                       double beta, uint64_t ldA, uint64_t ldB, uint64_t ldC, uint64_t offsetA,
                       uint64_t offsetB, uint64_t offsetC, bool transposeA, bool transposeB);
/* tiramisu_hip_sgemm for callers that cannot allocate device memory (code under HIP graph capture,
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments,
 * same kernels, bit-identical results; the difference is where deep reductions (at most 128 tiles of
 * 64x64 and K >= 2048, whose K range is split over workgroups) keep their partial tiles and per-tile
 * counters: tiramisu_hip_sgemm takes them from a per-thread workspace that it allocates and grows with
 * hipMalloc, this entry point from a 4 MiB (+512 B of counters) array that lives in the library's code
 * object, one copy per GPU, held until the process ends.  It calls no hipMalloc / hipFree.  A problem
 * whose split needs more than the array holds (tiles x chunks x 16 KiB: e.g. 640 x 640 x 4096, 300
 * partial tiles) is refused: a message on stderr, return value 1, nothing launched -- the one case in
 * this library where a failure returns instead of ending the process.  All calls on one GPU share the
 * array: calls that overlap on one GPU (two streams, two threads) race; serialise them.  The counters
 * are cleared by a small kernel before every use.  Returns 0 on success. */
int tiramisu_hip_sgemm_static_scratch(float *A, float *B, float *C, uint64_t M, uint64_t N, uint64_t K, float alpha,
                                      float beta, uint64_t ldA, uint64_t ldB, uint64_t ldC, uint64_t offsetA,
                                      uint64_t offsetB, uint64_t offsetC, bool transposeA, bool transposeB);
/* Batch scope (no counterpart in the reference).  Between _begin and _end the calling thread's tiramisu_hip_sgemm
 * calls are gathered instead of launched; _end launches them in call order, runs of calls of one shape (sizes,
 * leading dimensions, transposition, alpha, beta) as ONE launch with a problem per blockIdx.z (up to 8 per launch).
 * The gathered calls must be independent of one another: generated code opens a scope around the GEMM call of a
 * statement that it runs for all iterations of a host loop tagged parallel.  Scopes do not nest (_begin inside a
 * scope and _end outside one return 1); tiramisu_hip_sgemm_static_scratch and tiramisu_hip_dgemm are not gathered. */
int tiramisu_hip_batch_begin(void);
int tiramisu_hip_batch_end(void);

/* The scratch block that deep reductions of tiramisu_hip_sgemm use on the calling thread's current stream (partial
 * tiles and per-tile counters), or NULL before the first such call: one block per (host thread, stream), so that
 * calls of one thread on two streams may overlap.  No counterpart in the reference; for tests and diagnostics. */
void *tiramisu_hip_sgemm_workspace(void);

/* ---- memory the library keeps between calls.  No counterpart in the reference, whose generated code allocates and
 *      frees everything on every call. ---- */
/* Scratch that a generated function keeps from one call to the next (the third plane of a time-tiled stencil, the
 * hand-over area of the windowed convolution): one block per requesting site (generated code passes the address of
 * a static of its own), host thread and stream, at least `bytes` large, allocated at the first request and handed
 * out again at every later one.  *fresh (may be NULL) is 1 when this call allocated the block -- its contents are
 * undefined then -- and 0 when it is the block of the call before. */
void *tiramisu_hip_kept_scratch(const void *site, uint64_t bytes, int32_t *fresh);
/* Waits for the device, then gives back to HIP everything the library holds without anyone using it: the kept
 * scratch of all generated functions, the workspaces of tiramisu_hip_sgemm, the idle blocks of the pool behind
 * tiramisu_hip_malloc.  Returns the number of bytes released.  The caller makes sure that no generated function and
 * no GEMM call is running; later calls allocate again what they need. */
uint64_t tiramisu_hip_release_cached_memory(void);
/* What tiramisu_hip_release_cached_memory would release now. */
uint64_t tiramisu_hip_cached_memory_bytes(void);

/* ---- code objects and launches.  The reference links nvcc-compiled kernel wrappers
 *      (_kernel_N_wrapper, tiramisu_codegen_cuda.cpp:1288-1318) into the program; here
 *      generated host code is plain C++ that embeds a gfx950 code object and launches
 *      its kernels through these three calls. ---- */
/* Load a code object image (an .hsaco file's bytes) on the current device. */
void *tiramisu_hip_module_load(const void *image, uint64_t size);
/* Look a kernel up by name; exits with status 1 if the module does not define it. */
void *tiramisu_hip_module_get_function(void *module, const char *kernel_name);
/* Device address of a global variable of the module (a __constant__ array holding a buffer tagged
 * tag_gpu_constant()); exits with status 1 if the module does not define it or it is smaller
 * than `bytes`.  Replaces the `<buffer>_get_symbol()` host function the reference emits into its
 * .cu file (src/tiramisu_codegen_cuda.cpp:817-823); its result is what
 * tiramisu_hip_memcpy_to_symbol() takes as destination. */
void *tiramisu_hip_module_get_global(void *module, const char *name, uint64_t bytes);
/* Launch on the current stream.  args[i] points to the i-th kernel argument. */
int tiramisu_hip_launch(void *function, const uint32_t grid[3], const uint32_t block[3],
                        uint32_t dynamic_lds_bytes, void **args);

/* ---- host loops tagged parallel around GPU work.  The reference lowers such a loop to a Halide
 *      parallel loop (ForType::Parallel, tiramisu_codegen_halide.cpp:2104-2145): its iterations
 *      run on pool threads, each on its own per-thread default stream, and the program
 *      synchronises that stream before the iteration ends
 *      (benchmarks/DNN/blocks/LSTM/gpu_lib/generator.cpp:99-100, :133-135).  Here generated host
 *      code hands the loop body to this call: body(i, closure) runs once for every i in
 *      [first, last] on up to four pool threads, each with a stream of its own as its current
 *      stream.  The caller's stream is synchronised before the first iteration starts and every
 *      pool thread's stream before the call returns, so work before, inside and after the loop
 *      is ordered as in the serial loop; iterations must be independent of one another.
 *      Called from inside a parallel iteration, or with a single iteration, it runs the body
 *      in the calling thread. ---- */
void tiramisu_hip_parallel_for(int32_t first, int32_t last, void (*body)(int32_t, void *), void *closure);

/* ---- stream and timing helpers for wrappers and benchmarks (the reference's
 *      benchmarks bracket device work with get_time() calls,
 *      benchmarks/linear_algebra/blas/level3/sgemm/gpu/generator3.cpp:66-69) ---- */
/* Make `stream` (a hipStream_t) the calling thread's current stream; NULL restores the
 * per-thread default stream.  Pooled memory follows the stream rule of tiramisu_hip_free: a block
 * must be freed by a thread whose current stream is the one its last use was issued on (or after
 * that stream has been synchronised); freeing it from a thread on another stream may hand the
 * block out again while that work still runs. */
int tiramisu_hip_set_stream(void *stream);
void *tiramisu_hip_get_stream(void);
/* A new stream that does not synchronise with the default stream (default priority), for callers that overlap
 * calls; destroy waits for the stream's work and, if it is the calling thread's current stream, restores the
 * per-thread default stream.  Scratch blocks that the runtime keeps per (thread, stream) stay allocated until
 * tiramisu_hip_release_cached_memory. */
void *tiramisu_hip_stream_create(void);
int tiramisu_hip_stream_destroy(void *stream);
void *tiramisu_hip_event_create(void);
int tiramisu_hip_event_record(void *event);              /* on the current stream */
float tiramisu_hip_event_elapsed_ms(void *start, void *stop); /* waits for `stop` */
int tiramisu_hip_event_destroy(void *event);
int tiramisu_hip_device_count(void);

/* ---- per-launch timing.  Between profile_start and profile_stop every tiramisu_hip_launch
 *      (and GEMM library call), from any thread, is bracketed by two events on its current
 *      stream; profile_stop waits for them and keeps one (kernel name, milliseconds) record
 *      per launch, readable until the next profile_start.  The reference has no counterpart:
 *      its benchmarks use nvprof (utils/run_gpu_bench.py). ---- */
int tiramisu_hip_profile_start(void);
int tiramisu_hip_profile_stop(void);                 /* returns the number of records */
const char *tiramisu_hip_profile_name(int record);
float tiramisu_hip_profile_ms(int record);

#ifdef __cplusplus
}
#endif
#endif

/*
 * dlgrad_hip.h -- C ABI of libdlgrad_hip.so, the device layer under dlgrad's
 * `device="hip"` runtime (one MI355X / gfx950, one process, one stream).
 *
 * The reference binds, through cffi, one tiny C library per generated kernel
 * plus four allocation helpers (dlgrad/runtime/cpu.py:52-78 builds and dlopens
 * them; dlgrad/codegen/cpu_kernel.py holds the sources).  On a GPU the kernels
 * are device code objects, so the functions a Python runtime binds are the ones
 * below: memory, transfers, "compile this kernel source", "launch this kernel
 * with these packed arguments", ordering and timing.  Each entry names the
 * reference interface it stands in for.
 *
 * Conventions: every function returns 0 on success and a negative value on
 * failure; dlg_hip_last_error() then returns a human-readable message for the
 * calling thread's most recent failure.  Device pointers cross the boundary as
 * void*.  Nothing here takes or returns C++ or framework types, and nothing
 * calls back into the host language.  All work is issued on one internal,
 * default-priority stream; calls are asynchronous with respect to the host
 * unless stated otherwise.
 *
 * Threads: the allocator, the kernel table and the graph table are guarded by a
 * mutex, so allocation, free, module load and launch may come from any thread.
 * The stream is shared: work is ordered as issued, and the "current arena" and
 * "capture in progress" states are per process, so a capture (graph_begin ..
 * graph_end) and everything issued during it must come from one thread while
 * no other thread issues work.  The reference is single-threaded throughout
 * (dlgrad/runtime/cpu.py holds no lock).
 */
#ifndef DLGRAD_HIP_H
#define DLGRAD_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct dlg_hip_props {
    char     name[128];        /* marketing name                                   */
    char     arch[64];         /* gcnArchName, e.g. "gfx950:sramecc+:xnack-"       */
    int32_t  compute_units;    /* multiProcessorCount                              */
    int32_t  wavefront_size;   /* 64 on CDNA                                       */
    int32_t  clock_khz;        /* peak engine clock                                */
    int32_t  mem_clock_khz;    /* peak memory clock                                */
    int32_t  mem_bus_bits;     /* memory bus width                                 */
    int32_t  lds_bytes;        /* LDS per workgroup                                */
    int32_t  l2_bytes;         /* L2 per XCD                                       */
    int32_t  reserved;
    uint64_t total_mem;        /* bytes of device memory                           */
} dlg_hip_props_t;

/* ---- lifetime ------------------------------------------------------------
 * Stands in for the import-time side effects of dlgrad/runtime/cpu.py:30-41
 * (compiler discovery; exits when none is found).  Here: selects the device,
 * creates the stream.  Fails (<0) when no HIP device is present. Idempotent. */
int dlg_hip_init(int device);
int dlg_hip_device_count(int *count);
int dlg_hip_props(dlg_hip_props_t *out);
int dlg_hip_shutdown(void);

/* ---- memory --------------------------------------------------------------
 * dlg_hip_alloc      <- uninitialized_memory(nbytes)  cpu_kernel.py:671-687, CPU.malloc cpu.py:82-107
 * dlg_hip_alloc_zero <- initialized_memory(num,size)  cpu_kernel.py:690-705, CPU.calloc cpu.py:110-134
 * dlg_hip_fill_f32   <- init_with_scalar(...)         cpu_kernel.py:708-727, CPU.init_with_scalar cpu.py:167-191
 * dlg_hip_free       <- free_ptr(ptr)                 cpu_kernel.py:730-740 (the ffi.gc finaliser)
 * Blocks come from a size-bucketed pool over hipMalloc; free returns the block
 * to the pool (safe without a sync because every user is on the one stream).
 * Blocks of 8 MiB and more start 0, 4, 8 or 12 KiB into their pool block, in
 * turn, so that equal offsets into two large operands fall on different DRAM
 * banks; such pointers stay 4 KiB aligned, and dlg_hip_free takes the
 * pointer that dlg_hip_alloc returned.
 * A NULL/failed allocation is an error return, which the Python side turns
 * into MemoryError exactly where the reference does (cpu.py:104,132,189).
 * While a capture is in progress (dlg_hip_graph_begin) an allocation that the
 * current arena cannot serve from its returned blocks is refused with -9 (the
 * Python side raises RuntimeError): hipMalloc, and the stream wait of its
 * retry, are never issued under stream capture.                              */
int dlg_hip_alloc(size_t nbytes, void **out);
int dlg_hip_alloc_zero(size_t nbytes, void **out);
int dlg_hip_fill_f32(void *dst, float value, size_t count);
int dlg_hip_free(void *ptr);
/* pool introspection / release of cached blocks back to the driver */
int dlg_hip_pool_stats(uint64_t *bytes_in_use, uint64_t *bytes_cached, uint64_t *n_device_allocs);
int dlg_hip_pool_trim(void);

/* ---- transfers (synchronous with respect to the host) ----------------------
 * dlg_hip_h2d <- ffi.from_buffer(numpy) in Tensor.__init__ tensor.py:103-115 and
 *                ffi.memmove in Tensor.copy_from tensor.py:131-138
 * dlg_hip_d2h <- ffi.buffer(ptr, n) in Tensor.numpy / tobytes tensor.py:125-164, buffer.py:67-84
 * dlg_hip_d2d <- pointer aliasing on the host (reshape/slice views need no copy;
 *                this exists for explicit clones)                             */
int dlg_hip_h2d(void *dst_dev, const void *src_host, size_t nbytes);
int dlg_hip_d2h(void *dst_host, const void *src_dev, size_t nbytes);
int dlg_hip_d2d(void *dst_dev, const void *src_dev, size_t nbytes);

/* ---- pinned staging (the data path of dlgrad/nn/datasets.py:9-39 and of the
 * per-step batch in examples/mnist_mlp.py, where the reference hands numpy memory
 * to the kernels directly).  dlg_hip_host_alloc returns page-locked host memory
 * the GPU reads by DMA; dlg_hip_h2d_async enqueues a copy from such memory on the
 * stream and returns at once: the source must stay unchanged until a later
 * dlg_hip_sync (or event) has passed.  Unlike dlg_hip_h2d it may be issued during
 * a capture: the graph then re-reads the same host buffer on every replay, so a
 * loop only refills that buffer between replays.                              */
int dlg_hip_host_alloc(size_t nbytes, void **out);
int dlg_hip_host_free(void *ptr);
int dlg_hip_h2d_async(void *dst_dev, const void *src_pinned, size_t nbytes);

/* ---- kernels ---------------------------------------------------------------
 * dlg_hip_compile <- CPU._build_shared_object(source, so_path) cpu.py:52-62
 *      (clang/gcc subprocess).  Here hiprtc compiles HIP source for the given
 *      options (the caller passes --offload-arch=gfx950 ...) in-process and
 *      returns the code object bytes, which the caller may cache on disk the way
 *      the reference caches .so files under ~/.cache/dlgrad (cpu.py:64-78).
 *      Needs no GPU.  On failure the compiler log is in dlg_hip_compile_log().
 * dlg_hip_module_load <- CPU._get_handle(so_path) = ffi.dlopen cpu.py:69-72
 *      plus getattr(lib, func_name) cpu.py:274-275: loads a code object and
 *      resolves one kernel; the handle stays valid until shutdown.
 * dlg_hip_launch <- the cffi call of the generated function, e.g.
 *      func(x.ptr, y.ptr, outptr, shape_c, x_stride_c, y_stride_c) cpu.py:289.
 *      `args` is the kernel's argument block laid out with natural C alignment
 *      (what struct.pack("@...") produces); it is copied at launch time.    */
int dlg_hip_compile(const char *source, const char *name,
                    const char *const *options, int n_options,
                    void **code, size_t *code_size);
int dlg_hip_code_free(void *code);
const char *dlg_hip_compile_log(void);
int dlg_hip_module_load(const void *code, size_t code_size,
                        const char *kernel_name, uint64_t *handle);
int dlg_hip_launch(uint64_t handle,
                   uint32_t grid_x, uint32_t grid_y, uint32_t grid_z,
                   uint32_t block_x, uint32_t block_y, uint32_t block_z,
                   uint32_t shared_bytes, const void *args, size_t args_size);
/* registers/LDS/spill figures of a loaded kernel (for occupancy reasoning) */
int dlg_hip_kernel_attrs(uint64_t handle, int32_t *num_regs, int32_t *lds_bytes,
                         int32_t *scratch_bytes, int32_t *max_threads);

/* ---- full reduction (sum or max of n floats into one) as one call ----------------------
 * dlg_hip_reduce_full <- CPU.sum / CPU.max with dim = -1 (dlgrad/runtime/cpu.py:604-650) calling
 *      the generated `reduce` loop (dlgrad/codegen/cpu_kernel.py:150-177).  On the GPU it is two
 *      launches of the caller's stage kernel (hip_kernel.reduce_full_kernel, argument block
 *      {x, out, u32 n, float divisor, u32 chunk}): blocks of 2048 vector items each write one
 *      partial result, then one block folds the partials, divides by `divisor` (1, or n for a
 *      mean) and writes out[0].  k_stage reads x with `vec` floats per access (1, or 4 for a
 *      16-byte aligned x); k_fold is the same generator with vec = 4.  `workspace` receives the
 *      partials: ceil(ceil(n / vec) / 2048) floats, 16-byte aligned, device memory; it may be NULL
 *      when that count is 1.  More than 65536 partials (n > 2048 * vec * 65536) is an error: fold
 *      in pieces.  Asynchronous on the library's stream; allocates nothing itself.
 *
 * dlg_hip_reduce_full_static has NO counterpart in the reference.  It is the same call for
 *      callers that cannot allocate device memory or hand one in: code under stream capture,
 *      tight serving loops, harnesses that forbid hipMalloc.  The partials go to a 256 KiB array
 *      that is part of the library's device code (DLG_HIP_STATIC_SCRATCH_BYTES; every GPU the
 *      library is initialised on holds it until the process ends), so the call allocates
 *      nothing and records no memset; the same limit of 65536 partials applies and larger
 *      inputs are refused with a message.  The array is shared by every call on that GPU and
 *      keeps the last call's partials (each call overwrites the part it reads, so nothing needs
 *      clearing).  Calls on the library's one stream are ordered; calls that overlap on one GPU
 *      by any other route would race on the array.                                          */
#define DLG_HIP_STATIC_SCRATCH_BYTES (65536 * 4)
int dlg_hip_reduce_full(uint64_t k_stage, uint64_t k_fold, const void *x, uint64_t n, uint32_t vec,
                        float divisor, void *out, void *workspace, size_t workspace_bytes);
int dlg_hip_reduce_full_static(uint64_t k_stage, uint64_t k_fold, const void *x, uint64_t n, uint32_t vec,
                               float divisor, void *out);

/* ---- arenas and captured graphs ------------------------------------------------
 * No counterpart in the reference, whose CPU kernels have no launch cost to remove; on a
 * GPU a char-GPT training step is ~900 tiny launches and is bound by issuing them.
 * An arena is a private pool: while it is current (dlg_hip_arena_set), dlg_hip_alloc draws
 * from it and blocks return to it, so a graph captured inside it may replay writes to those
 * addresses for as long as the arena lives.  dlg_hip_graph_begin/end bracket a capture of
 * the internal stream (kernel launches only: synchronous transfers and memset-backed
 * calls fail while capturing); dlg_hip_graph_launch replays it on the same stream.                                                                */
int dlg_hip_arena_create(uint64_t *arena);
int dlg_hip_arena_set(uint64_t arena);            /* 0 = the ordinary pool */
/* Tops the arena's returned blocks up, size class by size class, to the largest number of blocks
 * of that class that were ever in use at once: after it, a pass that repeats the allocations the
 * arena has seen finds every block without a device allocation, also while results of the earlier
 * pass are still held.  Called between the warm-up pass and the capture, because an allocation that
 * misses the arena during a capture is refused (dlg_hip_alloc).  Fails inside a capture.           */
int dlg_hip_arena_reserve(uint64_t arena);
int dlg_hip_arena_destroy(uint64_t arena);
int dlg_hip_graph_begin(void);
int dlg_hip_graph_end(uint64_t *graph, uint64_t *n_nodes);   /* graph == NULL abandons the capture */
int dlg_hip_graph_launch(uint64_t graph);
int dlg_hip_graph_destroy(uint64_t graph);

/* ---- ordering and timing -----------------------------------------------------
 * The CPU reference is synchronous, so it has no counterpart; the Metal runtime's
 * commit()/waitUntilCompleted() per op (dlgrad/runtime/metal.py:124-128) is the
 * closest.  Here the host only waits when it asks to.                        */
int dlg_hip_sync(void);
int dlg_hip_event_create(uint64_t *event);
int dlg_hip_event_record(uint64_t event);
int dlg_hip_event_sync(uint64_t event);
int dlg_hip_event_elapsed_ms(uint64_t start, uint64_t stop, float *ms);
int dlg_hip_event_destroy(uint64_t event);

/* ---- errors ------------------------------------------------------------------
 * Reference: Python exceptions only (RuntimeError on compile failure cpu.py:61-62,
 * MemoryError on NULL).  The message of the last failing call on this thread. */
const char *dlg_hip_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* DLGRAD_HIP_H */

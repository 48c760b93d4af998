/*
 * dxhip.h — C ABI of libdxhip, the MI355X (gfx950) kernel layer of the deepx
 * `op-mem-hip` executor.
 *
 * This is the host<->kernel seam of the executor.  In the reference it is the set
 * of `launch_*` C++ templates that executor/op-cuda declares in
 *   executor/op-cuda/src/deepx/tensorfunc/elementwise_miaobyte_basic.cuh:11-98
 *   executor/op-cuda/src/deepx/tensorfunc/elementwise_miaobyte_sqrt.cuh:14-51
 *   executor/op-cuda/src/deepx/tensorfunc/elementwise_miaobyte_sin.cuh:19-33
 *   executor/op-cuda/src/deepx/tensorfunc/elementwise_miaobyte_compare.cuh:15-116
 *   executor/op-cuda/src/deepx/tensorfunc/reduce_miaobyte.cuh:16-52
 *   executor/op-cuda/src/deepx/tensorfunc/changeshape_miaobyte.cuh:16-79
 *   executor/op-cuda/src/deepx/tensorfunc/init_miaobyte.cuh:18-47
 *   executor/op-cuda/src/deepx/tensorfunc/matmul_cublas.hpp:16-145
 *   executor/op-cuda/src/deepx/tensorfunc/tensorlife_miaobyte.hpp:16-68
 * and whose arithmetic is defined by executor/op-ompsimd (the parity oracle).
 *
 * Conventions
 *  - plain pointers and sizes, no C++ types; every entry point returns an int:
 *    0 = ok, >0 = a hipError_t value, <0 = one of the DXH_ERR_* codes below.
 *    Nothing throws across the boundary.  A hipError_t that a call returns is reported by that call only: it is
 *    taken off the runtime's "last error", so the next launch does not find it there and report it as its own.
 *  - all tensor pointers are DEVICE pointers to contiguous row-major storage
 *    (executor/deepxcore/src/deepx/shape.cpp:21-32); shape/axis arrays are HOST
 *    pointers and are consumed before the call returns.
 *  - `dtype` is the reference's Precision bit value
 *    (executor/deepxcore/src/deepx/dtype.hpp:120-146), so the executor passes
 *    `shape.dtype` through unchanged.
 *  - bool tensors are one byte per element holding 0 or 1.
 *  - fp16 / bf16 ops compute in fp32 and round once (RNE) to the storage type,
 *    the convention of executor/op-cuda/src/deepx/tensorfunc/cuda_math.cuh:243-251.
 *  - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Calls
 *    are asynchronous: they return after enqueueing, like the reference's launches.
 *  - element counts are 64-bit; no entry point but dxh_malloc and dxh_pool_alloc
 *    allocates device memory.  Those that need device scratch (reductions, matmul) take a
 *    caller-provided workspace, sized by the matching *_workspace_bytes query.
 */
#ifndef DXHIP_H
#define DXHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DXH_API __attribute__((visibility("default")))

/* Precision bit values, executor/deepxcore/src/deepx/dtype.hpp:120-146 */
enum dxh_dtype {
    DXH_F64  = 1 << 0,
    DXH_F32  = 1 << 1,
    DXH_F16  = 1 << 2,
    DXH_BF16 = 1 << 3,
    DXH_I64  = 1 << 8,
    DXH_I32  = 1 << 9,
    DXH_I16  = 1 << 10,
    DXH_I8   = 1 << 11,
    DXH_BOOL = 1 << 13
};

enum dxh_error {
    DXH_OK = 0,
    DXH_ERR_DTYPE = -1,      /* dtype not supported by this op */
    DXH_ERR_ARG = -2,        /* null pointer, negative size, bad axis ... */
    DXH_ERR_SHAPE = -3,      /* shapes inconsistent for this op */
    DXH_ERR_WORKSPACE = -4,  /* workspace missing or too small */
    DXH_ERR_ALIGN = -5,      /* pointer not aligned to its element size */
    DXH_ERR_TOO_LARGE = -6,  /* the input needs more scratch than the entry point's fixed buffer holds */
    DXH_ERR_NOT_READY = -7   /* first use on this device is under stream capture: call dxh_set_device first */
};

/* A scalar operand.  Floating dtypes read `f`, integer and bool dtypes read `i`.
 * The executor fills both from T(std::stof(text)), the reference's scalar rule
 * (executor/deepxcore/src/deepx/tf/tf.hpp:119-123). */
typedef struct dxh_scalar {
    double f;
    int64_t i;
} dxh_scalar;

#define DXH_MAX_DIMS 12 /* the reference instantiates DIM 1..12, reduce_miaobyte.cu:61-107 */

/* ---- runtime: replaces cudaMalloc/cudaFree/cudaMemcpy of
 * executor/op-cuda/src/deepx/tensorfunc/tensorlife_miaobyte.hpp:16-68 ---------- */
/* The number a caller was compiled against; dxh_version() returns the one the loaded library was
 * built with.  It changes whenever an existing entry point changes its arguments or meaning
 * (additions keep it): 100 = first layout; 200 = dxh_matmul takes `workspace, workspace_bytes`
 * before `stream`, DXH_TUNE_MATMUL_TILE ranges 0..15.  A caller checks for equality once, at
 * load, and refuses to go on otherwise (a stream passed where a workspace is expected would be
 * dereferenced as memory). */
#define DXH_ABI_VERSION 200
DXH_API int dxh_version(void);
DXH_API const char *dxh_error_string(int code);
/* Launch-heuristic knobs (process wide; results never depend on them, only speed).
 * No counterpart in the reference, whose launch shape is fixed (cuda.hpp:45-67). */
enum dxh_tune_knob {
    DXH_TUNE_NT_STORE_BYTES = 0,       /* a launch of an elementwise kernel or a fused run that stores more than this many bytes
                                        * uses non-temporal stores (default 32 MiB; 0 = always) */
    DXH_TUNE_REDUCE_TARGET_BLOCKS = 1, /* workgroups a reduction stage aims for before it stops splitting R */
    DXH_TUNE_REDUCE_COL_MIN_ROWS = 2,  /* strided-axis stage: fewest rows per lane when R is split */
    DXH_TUNE_REDUCE_COL_MAX_LANES = 3, /* strided-axis stage: widest column-lane count (16..256) */
    DXH_TUNE_REDUCE_ROW_LOADS = 5,     /* contiguous-axis stage: 16-byte loads per lane a row's lane group aims for */
    DXH_TUNE_MATMUL_TILE = 4,          /* matmul workgroup tile, 0 = chosen per shape; bf16/f16: 1 128x128, 2 128x64, 3 64x128,
                                          4 256x256, 5 64x64, 6 192x256; 7 / 8 / 9 / 10 = 256x256 / 192x256 / 128x64 / 256x256 with
                                          operands loaded straight into LDS in K steps of 32 / 32 / 64 / 64 (K a multiple of 64,
                                          else the register-staged twin 4 / 6 / 2 / 4 runs); 11 / 12 / 13 = 160x256 / 128x256 /
                                          256x128 of the same kind in K steps of 64, the first two with one wave per 64 columns (twins 6 / 6 / 4);
                                          14 / 15 = 128x128 / 128x256 of that kind with K cut in two halves that are added inside
                                          the launch (scratch from the workspace; twins 1 / 12);
                                          f32: 1 128x128, 2 128x64, 3 64x64, 4 128x128 with K step 16 */
    DXH_TUNE_MATMUL_SPLITK = 6,        /* slices along K of a float matmul: 0 = chosen per shape (few output tiles and a long
                                          K are cut so that every CU has work), 1 = never, n <= 1024 = n slices.  Slices are
                                          added in slice order, so results do not vary from run to run. */
    DXH_TUNE_NT_LOAD = 7,              /* non-temporal hint on the loads of elementwise / compare / reduce kernels:
                                          0 = by op class and tensor size, 1 = always, 2 = never */
    DXH_TUNE_SKINNY_PER_CU = 8,        /* matmul with at most 8 rows of A (streaming kernel): workgroups per CU that the
                                          cut of K aims for (default 1) */
    DXH_TUNE_SKINNY_MIN_ROWS = 9,      /* ... and the fewest rows of B per K slice (default 256, at least 8) */
    DXH_TUNE_SKINNY_HALF = 10,         /* 1 = that kernel also for bf16 / f16 (default 0: they stay on the matrix pipe,
                                          which is as fast or faster for them) */
    DXH_TUNE_REDUCE_FUSED_FINISH = 11, /* strided-axis reduction whose reduced axis is cut into slices: 1 (default) = the
                                          workgroup that finishes a tile last adds the slices, in a fixed order, inside the
                                          same launch, 0 = a second launch does (also the fallback when the library's
                                          completion counters are used up).  The two differ in the last bits of a
                                          floating-point sum or product (different, each fixed, order of addition). */
    DXH_TUNE_CHAIN_STATIC = 12         /* dxh_chain / dxh_chain_rows: 1 (default) = a run that spells one of the sequences the
                                          library holds a compiled kernel for takes that kernel, 0 = every run goes through
                                          the interpreting kernel.  Same bits either way. */
};
DXH_API int dxh_tune(int knob, int64_t value);
DXH_API int dxh_device_count(int *count);
DXH_API int dxh_set_device(int device);
DXH_API int dxh_device_name(char *buf, size_t buflen);
DXH_API int dxh_malloc(void **ptr, size_t bytes);
DXH_API int dxh_free(void *ptr);
/* No counterpart in the reference, which goes to the driver for every tensor (cudaMalloc / cudaFree,
 * executor/op-cuda/src/deepx/tensorfunc/tensorlife_miaobyte.hpp:20,31) while its front allocates the result of every op right
 * before the op (front/py/deepx/nn/functional/leaffunc.py:30-38): freed blocks are kept by size class (eight classes per doubling,
 * steps of at most 2 MiB) and handed out again, so that a `newtensor` / `deltensor` pair costs a few microseconds of host time
 * instead of hipMalloc + a hipFree that waits for the device.  One pool per device; all five calls act on the current device's.
 *  - dxh_pool_alloc: a block of at least `bytes` (0 bytes still gets a pointer of its own).  The block may have been freed
 *    while launches that use it were still running: the caller's FIRST use of it must be ordered after them.  A launch or copy
 *    on the NULL stream is (it waits for every blocking stream); a launch on another stream is only if that stream has waited
 *    for them.  When the driver is out of memory every kept block goes back to it before the call gives up.
 *  - dxh_pool_free: takes back a pointer from dxh_pool_alloc without waiting for the device; DXH_ERR_ARG for any other pointer
 *    (the same one twice included), which is left alone.  Never pass such a pointer to dxh_free.
 *  - dxh_pool_trim: gives kept blocks back to the driver, largest first, until at most `keep_bytes` stay (`released`, if not NULL,
 *    gets the bytes given back).  dxh_malloc does this by itself when the driver is out of memory.
 *  - dxh_pool_limit: the most bytes the pool keeps (default: half the device's memory, or DXH_POOL_MAX_MB from the environment when
 *    the pool is first used); a free beyond it releases larger kept blocks first, and the block itself if it alone is over the limit.
 *  - dxh_pool_stats: counts since the pool was made, and what it holds now. */
typedef struct dxh_pool_stats_t {
    uint64_t hits, misses;            /* allocations served from a kept block / by the driver */
    uint64_t kept, released;          /* frees that kept the block / blocks given back to the driver */
    uint64_t kept_bytes, kept_blocks; /* in the pool now */
    uint64_t live_bytes, live_blocks; /* handed out now, in class sizes */
} dxh_pool_stats_t;
DXH_API int dxh_pool_alloc(void **ptr, size_t bytes);
DXH_API int dxh_pool_free(void *ptr);
DXH_API int dxh_pool_trim(size_t keep_bytes, size_t *released);
DXH_API int dxh_pool_limit(size_t max_kept_bytes);
DXH_API int dxh_pool_stats(dxh_pool_stats_t *out);
DXH_API int dxh_memcpy_h2d(void *dst, const void *src, size_t bytes, void *stream);
DXH_API int dxh_memcpy_d2h(void *dst, const void *src, size_t bytes, void *stream);
DXH_API int dxh_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream);
DXH_API int dxh_stream_create(void **stream);
DXH_API int dxh_stream_destroy(void *stream);
DXH_API int dxh_stream_sync(void *stream);
DXH_API int dxh_device_sync(void);
/* hipEvent helpers so a harness can time on the stream the kernels run on. */
DXH_API int dxh_event_create(void **event);
DXH_API int dxh_event_destroy(void *event);
DXH_API int dxh_event_record(void *event, void *stream);
DXH_API int dxh_event_sync(void *event);
/* No counterpart in the reference, whose launches name no stream (executor/op-cuda/src/deepx/tensorfunc/elementwise_miaobyte_basic.cu:113: `add_kernel<<<numBlocks, blockSize>>>`):
 * work launched on `stream` after this call waits for what `event` recorded (hipStreamWaitEvent).  How a caller that spreads
 * independent ops over several streams orders the dependent ones without going through the default stream. */
DXH_API int dxh_stream_wait_event(void *stream, void *event);
DXH_API int dxh_event_elapsed_ms(void *start, void *stop, float *ms);

/* ---- sharing one allocation between processes on the same GPU (heap tensors).
 * The reference plans this for its heap-tensor store (cudaIpcGetMemHandle / cudaIpcOpenMemHandle,
 * executor/heapmem-cuda/README.md:36-40); its tree holds no IPC code yet.  `handle` is an opaque
 * DXH_IPC_HANDLE_BYTES buffer that may be sent to another process as bytes.  `ptr` must be the
 * start of a dxh_malloc allocation (keep shared allocations under 2 GiB); a pointer obtained with
 * dxh_ipc_open is released with dxh_ipc_close, never dxh_free. */
#define DXH_IPC_HANDLE_BYTES 64
DXH_API int dxh_ipc_export(const void *ptr, void *handle);
DXH_API int dxh_ipc_open(const void *handle, void **ptr);
DXH_API int dxh_ipc_close(void *ptr);

/* ---- HIP graphs: record the kernels a sequence of dxh_* calls launches on `stream` once, replay
 * them with one launch.  No counterpart in the reference (it launches op by op on the default
 * stream); used by the executor for datagrams that carry several deepxIR lines
 * (executor/deepxcore/src/client/udpserver.cpp:49-58 already splits them).  `stream` must be a
 * stream from dxh_stream_create, not NULL.  Between begin and end only kernel-launching dxh_* calls
 * and dxh_memcpy_d2d may run on it; no allocation, synchronisation or host copy.  end_capture
 * returns an executable graph (NULL with an error code if the capture was invalidated). */
DXH_API int dxh_graph_begin_capture(void *stream);
DXH_API int dxh_graph_end_capture(void *stream, void **graph_exec);
DXH_API int dxh_graph_launch(void *graph_exec, void *stream);
DXH_API int dxh_graph_destroy(void *graph_exec);
/* Recorded launches that finish a reduction or a K-cut matmul inside one launch own counters of
 * the library's device array for as long as their graph lives; dxh_graph_destroy (on a graph that
 * has finished running) and a failed capture give them back.  Reports how many are taken and how
 * many there are on the current device; with none left such launches are recorded in their
 * two-launch form, which gives the same bits more slowly. */
DXH_API int dxh_graph_counter_stats(int64_t *in_use, int64_t *capacity);

/* ---- elementwise, C[i] = A[i] op B[i]
 * launch_add/sub/mul/div  elementwise_miaobyte_basic.cuh:16-98
 * launch_max/min          elementwise_miaobyte_compare.cuh:15-44
 * launch_pow              elementwise_miaobyte_sqrt.cuh:22-28   (f32/f64 only)
 * arithmetic per executor/op-ompsimd/src/deepx/tensorfunc/elementwise_miaobyte.hpp:115-318,430-448,599-764
 * dtypes: f64 f32 f16 bf16 i64 i32 i16 i8.  Integer division by zero yields 0. */
DXH_API int dxh_add(int dtype, const void *a, const void *b, void *c, int64_t n, void *stream);
DXH_API int dxh_sub(int dtype, const void *a, const void *b, void *c, int64_t n, void *stream);
DXH_API int dxh_mul(int dtype, const void *a, const void *b, void *c, int64_t n, void *stream);
DXH_API int dxh_div(int dtype, const void *a, const void *b, void *c, int64_t n, void *stream);
DXH_API int dxh_max(int dtype, const void *a, const void *b, void *c, int64_t n, void *stream);
DXH_API int dxh_min(int dtype, const void *a, const void *b, void *c, int64_t n, void *stream);
DXH_API int dxh_pow(int dtype, const void *a, const void *b, void *c, int64_t n, void *stream);

/* ---- elementwise with a scalar operand
 * launch_addscalar ... launch_rdivscalar  elementwise_miaobyte_basic.cuh:24-98
 * launch_maxscalar/minscalar             elementwise_miaobyte_compare.cuh:22-44
 * launch_powscalar/rpowscalar            elementwise_miaobyte_sqrt.cuh:30-44 (f32/f64 only)
 * r*scalar forms compute scalar op A[i]. */
DXH_API int dxh_addscalar(int dtype, const void *a, dxh_scalar s, void *c, int64_t n, void *stream);
DXH_API int dxh_subscalar(int dtype, const void *a, dxh_scalar s, void *c, int64_t n, void *stream);
DXH_API int dxh_rsubscalar(int dtype, dxh_scalar s, const void *a, void *c, int64_t n, void *stream);
DXH_API int dxh_mulscalar(int dtype, const void *a, dxh_scalar s, void *c, int64_t n, void *stream);
DXH_API int dxh_divscalar(int dtype, const void *a, dxh_scalar s, void *c, int64_t n, void *stream);
DXH_API int dxh_rdivscalar(int dtype, dxh_scalar s, const void *a, void *c, int64_t n, void *stream);
DXH_API int dxh_maxscalar(int dtype, const void *a, dxh_scalar s, void *c, int64_t n, void *stream);
DXH_API int dxh_minscalar(int dtype, const void *a, dxh_scalar s, void *c, int64_t n, void *stream);
DXH_API int dxh_powscalar(int dtype, const void *a, dxh_scalar s, void *c, int64_t n, void *stream);
DXH_API int dxh_rpowscalar(int dtype, dxh_scalar s, const void *a, void *c, int64_t n, void *stream);

/* ---- unary
 * launch_sqrt/log/exp  elementwise_miaobyte_sqrt.cuh:14-20,46-51 (f64 f32 f16 bf16)
 * launch_sin/cos/tan   elementwise_miaobyte_sin.cuh:19-33        (tan: f64 f32)
 * launch_invert        elementwise_miaobyte_basic.cuh:94-98      (i64 i32 i16 i8: ~x, bool: !x) */
DXH_API int dxh_sqrt(int dtype, const void *a, void *c, int64_t n, void *stream);
DXH_API int dxh_exp(int dtype, const void *a, void *c, int64_t n, void *stream);
DXH_API int dxh_log(int dtype, const void *a, void *c, int64_t n, void *stream);
DXH_API int dxh_sin(int dtype, const void *a, void *c, int64_t n, void *stream);
DXH_API int dxh_cos(int dtype, const void *a, void *c, int64_t n, void *stream);
DXH_API int dxh_tan(int dtype, const void *a, void *c, int64_t n, void *stream);
DXH_API int dxh_invert(int dtype, const void *a, void *c, int64_t n, void *stream);

/* ---- a run of elementwise ops in one launch
 * No counterpart in the reference, which launches op by op; for a caller that holds several
 * instructions at once (a datagram of deepxIR lines, udpserver.cpp:49-58).  Op k of the run is one of
 * the float ops above over tensors of `n` elements of `dtype` (f64 f32 f16 bf16); its tensor
 * operands are inputs[ref] or, as DXH_CHAIN_RESULT + j, the result of op j < k of the same run; its
 * result is rounded to `dtype` and stored to `out` before a later op uses it, so every `out` holds
 * exactly what the separate calls would have stored.  Inputs are read before any result is written:
 * an `out` may be one of the inputs (in-place ops), but a later op that is to see such a result must
 * name it as DXH_CHAIN_RESULT + j.  An op other than the last may have out = NULL: its result then only
 * feeds later ops of the run (for a tensor that a later op of the run overwrites anyway).
 * All pointers 16-byte aligned and n a multiple of 16 / sizeof(dtype),
 * else DXH_ERR_ALIGN (use the separate calls then).  Scalar forms take `scalar` and `lhs`; unary
 * forms `lhs` only. */
enum dxh_chain_code {
    DXH_CHAIN_ADD = 0, DXH_CHAIN_SUB, DXH_CHAIN_MUL, DXH_CHAIN_DIV, DXH_CHAIN_MAX, DXH_CHAIN_MIN,      /* lhs op rhs */
    DXH_CHAIN_ADDSCALAR, DXH_CHAIN_SUBSCALAR, DXH_CHAIN_RSUBSCALAR, DXH_CHAIN_MULSCALAR,               /* lhs op scalar; R: scalar op lhs */
    DXH_CHAIN_DIVSCALAR, DXH_CHAIN_RDIVSCALAR, DXH_CHAIN_MAXSCALAR, DXH_CHAIN_MINSCALAR,
    DXH_CHAIN_SQRT, DXH_CHAIN_EXP, DXH_CHAIN_LOG,                                                      /* f(lhs) */
    DXH_CHAIN_SQUARE, DXH_CHAIN_COPY, DXH_CHAIN_ROWSUM,                                                /* dxh_chain_rows only */
    DXH_CHAIN_ROWMAX, DXH_CHAIN_ROWMIN                                                                 /* dxh_chain_rows only */
};
#define DXH_CHAIN_MAX_OPS 8
#define DXH_CHAIN_ROWS_MAX_OPS 16
#define DXH_CHAIN_MAX_INPUTS 8
#define DXH_CHAIN_RESULT 16
typedef struct dxh_chain_op {
    int32_t code;      /* enum dxh_chain_code */
    int32_t lhs, rhs;  /* operand references */
    dxh_scalar scalar;
    void *out;         /* NULL: not stored */
} dxh_chain_op;
DXH_API int dxh_chain(int dtype, const void *const *inputs, int n_inputs, const dxh_chain_op *ops, int n_ops, int64_t n, void *stream);

/* ---- the same over a [rows, cols] view, with row / column vectors and casts
 * No counterpart in the reference either.  The tensors of this run may differ in dtype (f32 f16 bf16)
 * and in extent: [rows, cols] (DXH_CHAIN_FULL), a row vector [1, cols] or a column vector [rows, 1].
 * Op k is one of the ops of dxh_chain, DXH_CHAIN_SQUARE (lhs * lhs: powscalar with exponent 2 of
 * elementwise_miaobyte_sqrt.cuh:30, whose correctly rounded value that is) or DXH_CHAIN_COPY
 * (lhs as it is: with another dtype the cast of launch_todtype, elementwise_miaobyte_basic.cuh:11-16,
 * with a vector operand and full extent launch_broadcastTo, changeshape_miaobyte.cuh:42-46).  It computes
 * in fp32 on its operands' values and rounds the result to its own `dtype` before that is stored or
 * used, which is what the separate calls do: every `out` holds their bits.  An op of full extent takes
 * operands of any extent (a vector counts for every row or column); an op on row or column vectors takes
 * vectors of its own kind only and stores `cols` or `rows` elements.  Operand references, in-place use
 * of [rows, cols] tensors and out = NULL as for dxh_chain; a vector input must not be an `out` of the
 * run (DXH_ERR_ARG: run the ops that update it in place on their own).  cols a multiple of 4 and
 * [rows, cols] / row-vector pointers aligned to 4 elements, else DXH_ERR_ALIGN.  Up to
 * DXH_CHAIN_ROWS_MAX_OPS ops.
 * DXH_CHAIN_ROWSUM (fp32 only) is launch_sum (reduce_miaobyte.cuh:16-21) over the last axis inside the
 * run: lhs of full extent, the result a column vector with the bits dxh_sum stores for the same rows
 * (the lanes share the rows as its kernel would and add in its order).  DXH_CHAIN_ROWMAX and
 * DXH_CHAIN_ROWMIN are launch_reducemax / launch_reducemin (reduce_miaobyte.cuh:30-52) the same way
 * (the order matters for them too: NaN and the sign of a zero follow it).  In a run that the library
 * holds a compiled kernel for (DXH_TUNE_CHAIN_STATIC) the three also take f16 / bf16 operands, and rows
 * of up to eight 16-byte vectors per lane of the separate kernel's lane group; the interpreting kernel
 * takes fp32 operands only.  That needs rows short enough
 * for one lane group: dxh_chain_rows_can_sum says whether a [rows, cols] view qualifies (1) or not (0),
 * and a run with a row sum over one that does not is refused with DXH_ERR_SHAPE, as is a run that needs
 * more LDS than a CU has.  A run whose LDS need exceeds 64 KiB raises the kernel's limit first: once
 * per device, in dxh_set_device or on such a run's first launch, which must not be one under stream
 * capture (DXH_ERR_NOT_READY then). */
enum dxh_chain_extent { DXH_CHAIN_FULL = 0, DXH_CHAIN_ROW = 1, DXH_CHAIN_COLUMN = 2 };
typedef struct dxh_chain_tensor {
    const void *data;
    int32_t dtype;     /* DXH_F32, DXH_F16 or DXH_BF16 */
    int32_t extent;    /* enum dxh_chain_extent */
} dxh_chain_tensor;
typedef struct dxh_chain_rows_op {
    int32_t code;      /* enum dxh_chain_code */
    int32_t lhs, rhs;  /* index into inputs, or DXH_CHAIN_RESULT + j */
    dxh_scalar scalar;
    void *out;         /* NULL: not stored */
    int32_t dtype;     /* of the result */
    int32_t extent;    /* of the result */
} dxh_chain_rows_op;
DXH_API int dxh_chain_rows_can_sum(int64_t rows, int64_t cols);
/* How many dxh_chain / dxh_chain_rows launches of this process took a compiled kernel and how many the
 * interpreting one (for tests and for a caller that wants to see which of its runs are known). */
DXH_API int dxh_chain_stats(int64_t *compiled, int64_t *interpreted);
DXH_API int dxh_chain_rows(const dxh_chain_tensor *inputs, int n_inputs, const dxh_chain_rows_op *ops, int n_ops, int64_t rows, int64_t cols, void *stream);
/* Every check of dxh_chain_rows and no launch: DXH_OK when the same call would be launched (a planner asks before it
 * commits a row reduction to a run; touches no device state). */
DXH_API int dxh_chain_rows_check(const dxh_chain_tensor *inputs, int n_inputs, const dxh_chain_rows_op *ops, int n_ops, int64_t rows, int64_t cols);

/* ---- cast: launch_todtype elementwise_miaobyte_basic.cuh:11-16.
 * C[i] = static_cast<dst>(A[i]) (float->int truncates toward zero, saturating at
 * the integer range; float->f16/bf16 rounds RNE).  Same dtype = device copy. */
DXH_API int dxh_todtype(int src_dtype, const void *a, int dst_dtype, void *c, int64_t n, void *stream);

/* ---- compare -> bool mask (one byte, 0/1)
 * launch_equal/notequal(+scalar) with epsilon  elementwise_miaobyte_compare.cuh:46-84
 * launch_less/greater(+scalar)                 elementwise_miaobyte_compare.cuh:86-108
 * epsilon semantics follow op-ompsimd (elementwise_miaobyte.hpp:767-886):
 *   equal:    eps==0 ? a==b : |a-b| <= eps        notequal: eps==0 ? a!=b : |a-b| > eps */
DXH_API int dxh_equal(int dtype, const void *a, const void *b, float epsilon, void *mask, int64_t n, void *stream);
DXH_API int dxh_notequal(int dtype, const void *a, const void *b, float epsilon, void *mask, int64_t n, void *stream);
DXH_API int dxh_equalscalar(int dtype, const void *a, dxh_scalar s, float epsilon, void *mask, int64_t n, void *stream);
DXH_API int dxh_notequalscalar(int dtype, const void *a, dxh_scalar s, float epsilon, void *mask, int64_t n, void *stream);
DXH_API int dxh_less(int dtype, const void *a, const void *b, void *mask, int64_t n, void *stream);
DXH_API int dxh_greater(int dtype, const void *a, const void *b, void *mask, int64_t n, void *stream);
DXH_API int dxh_lessscalar(int dtype, const void *a, dxh_scalar s, void *mask, int64_t n, void *stream);
DXH_API int dxh_greaterscalar(int dtype, const void *a, dxh_scalar s, void *mask, int64_t n, void *stream);

/* ---- switch: launch_switch elementwise_miaobyte_compare.cuh:110-116.
 * C[i] = tensors[cases[i]][i]; cases_dtype is DXH_I32 or DXH_BOOL (bool needs exactly
 * two tensors, elementwise_miaobyte.hpp:1001-1024).  `tensors` is a HOST array of
 * `ntensors` device pointers, 1 <= ntensors <= DXH_SWITCH_MAX; it is passed to the
 * kernel by value (no device-side pointer table, no allocation).  A case value
 * outside [0, ntensors) selects nothing and writes zero bits. */
#define DXH_SWITCH_MAX 8
DXH_API int dxh_switch(int dtype, const void *const *tensors, int ntensors, int cases_dtype,
                       const void *cases, void *c, int64_t n, void *stream);

/* ---- reduce: launch_sum/prod/reducemax/reducemin reduce_miaobyte.cuh:16-52.
 * `shape[ndim]` is the input shape; `dims[ndims]` the reduced axes (negative allowed;
 * normalised, sorted, de-duplicated as executor/deepxcore/src/deepx/shape_reduce.cpp:11-45;
 * ndims==0 reduces every axis).  The output holds prod(kept dims) elements; keepdims
 * only changes the caller's view of it (shape_reduce.cpp:47-74).  f16/bf16 accumulate
 * in fp32, f32 in fp32, f64 in f64, integers wrap in their own width.
 * `workspace` may be NULL when dxh_reduce_workspace_bytes reports 0. */
DXH_API int dxh_reduce_workspace_bytes(int dtype, const int32_t *shape, int ndim,
                                       const int32_t *dims, int ndims, size_t *bytes);
DXH_API int dxh_sum(int dtype, const void *in, const int32_t *shape, int ndim, const int32_t *dims,
                    int ndims, void *out, void *workspace, size_t workspace_bytes, void *stream);
DXH_API int dxh_prod(int dtype, const void *in, const int32_t *shape, int ndim, const int32_t *dims,
                     int ndims, void *out, void *workspace, size_t workspace_bytes, void *stream);
DXH_API int dxh_reducemax(int dtype, const void *in, const int32_t *shape, int ndim,
                          const int32_t *dims, int ndims, void *out, void *workspace,
                          size_t workspace_bytes, void *stream);
DXH_API int dxh_reducemin(int dtype, const void *in, const int32_t *shape, int ndim,
                          const int32_t *dims, int ndims, void *out, void *workspace,
                          size_t workspace_bytes, void *stream);

/* dxh_sum for callers that cannot allocate or pass a workspace: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.  Same arguments
 * and results (bit for bit) as dxh_sum; the partial results that dxh_sum keeps in `workspace` live in
 * a device array of DXH_SUM_NOALLOC_SCRATCH_BYTES inside the library instead (one copy per GPU, held
 * until the process ends), and the call allocates and frees nothing.  A reduction whose
 * dxh_reduce_workspace_bytes exceeds that size is refused with DXH_ERR_TOO_LARGE.  Every call on one
 * GPU shares the array: calls that overlap there (two streams, two threads) race.  The array's address
 * is looked up on the first call on a device or by dxh_set_device; a first call under stream capture
 * returns DXH_ERR_NOT_READY. */
#define DXH_SUM_NOALLOC_SCRATCH_BYTES (4u << 20)
DXH_API int dxh_sum_noalloc(int dtype, const void *in, const int32_t *shape, int ndim, const int32_t *dims,
                            int ndims, void *out, void *stream);

/* ---- changeshape: changeshape_miaobyte.cuh:16-79.  Pure data movement, bit-exact,
 * chosen by element size, so every dtype above (and bool) is accepted.
 * transpose:   out[o] = in[p], p[dim_order[i]] = o[i]  (changeshape_miaobyte.hpp:45-67)
 * concat:      `ins` HOST array of device pointers, `axis_sizes[i]` = shape of source i on
 *              `axis`; `out_shape` is the result shape             (:69-100)
 * broadcastTo: numpy trailing-aligned rules, shape_changeshape.cpp:59-104
 * indexselect: out[pre,idx...,post] = in[pre, index[idx...], post]; index_dtype I32|I64;
 *              out-of-range indices are clamped into [0, shape[axis]) rather than read
 *              out of bounds (the reference does not check, :155-178)
 * repeat:      out[i] = in[i / repeats]                             (:181-200) */
DXH_API int dxh_transpose(int dtype, const void *in, const int32_t *shape, int ndim,
                          const int32_t *dim_order, void *out, void *stream);
DXH_API int dxh_concat(int dtype, const void *const *ins, int nins, const int32_t *axis_sizes,
                       const int32_t *out_shape, int ndim, int axis, void *out, void *stream);
DXH_API int dxh_broadcastTo(int dtype, const void *in, const int32_t *in_shape, int in_ndim,
                            const int32_t *out_shape, int out_ndim, void *out, void *stream);
DXH_API int dxh_indexselect(int dtype, const void *in, const int32_t *in_shape, int in_ndim,
                            int index_dtype, const void *index, const int32_t *index_shape,
                            int index_ndim, int axis, void *out, void *stream);
DXH_API int dxh_repeat(int dtype, const void *in, const int32_t *shape, int ndim,
                       const int32_t *repeats, void *out, void *stream);

/* ---- init: launch_constant / launch_arange init_miaobyte.cuh:18-30.
 * arange: out[i] = start + i*step computed in the dtype's arithmetic
 * (executor/op-ompsimd/src/deepx/tensorfunc/init_miaobyte.hpp:59-70). */
DXH_API int dxh_constant(int dtype, void *out, int64_t n, dxh_scalar value, void *stream);
DXH_API int dxh_arange(int dtype, void *out, int64_t n, dxh_scalar start, dxh_scalar step, void *stream);
/* launch_uniform / launch_normal / launch_dropout init_miaobyte.cuh:32-47.
 * uniform: out[i] = T(U[low,high));  normal: out[i] = T(N(mean,stddev));  dropout: inout[i] = 0
 * where U[0,1) < p, other elements unchanged (no rescale, init_miaobyte.hpp:26-54).
 * The random streams are counter based (a hash of seed and element index), reproducible for a
 * given seed != 0; seed == 0 draws a fresh seed, as the reference does.  The reference's own
 * two executors use different generators (libstdc++ minstd vs curand), so the bit stream is
 * not part of the contract — only the distribution is. */
DXH_API int dxh_uniform(int dtype, void *out, int64_t n, dxh_scalar low, dxh_scalar high, uint32_t seed, void *stream);
DXH_API int dxh_normal(int dtype, void *out, int64_t n, dxh_scalar mean, dxh_scalar stddev, uint32_t seed, void *stream);
DXH_API int dxh_dropout(int dtype, void *inout, int64_t n, float p, uint32_t seed, void *stream);

/* ---- matmul: replaces cublasSgemm(StridedBatched) matmul_cublas.hpp:16-145 and
 * cblas_sgemm executor/op-ompsimd/src/deepx/tensorfunc/matmul_cblas.hpp:11-60.
 * C[b,m,n] = sum_k A[b,m,k] * B[b,k,n], row-major, alpha=1 beta=0, `batch` = product of
 * the leading dims.  f16/bf16: MFMA with fp32 accumulate, one RNE rounding of the
 * result; f32/f64 accumulate in their own type; integers wrap.  A float product with few
 * output tiles and a long K is cut along K (DXH_TUNE_MATMUL_SPLITK) into partial products that
 * are added in a fixed order, and one whose rows are not 16-byte aligned (odd K or N, unaligned
 * bases) runs on zero-padded copies of A and B: both live in `workspace`, device memory of the
 * caller of at least dxh_matmul_workspace_bytes(same arguments) bytes, 256-byte aligned, that
 * no other call in flight uses; the library allocates nothing.  `workspace` may be NULL when the
 * query reports 0 (most shapes); a workspace that is too small gives DXH_ERR_WORKSPACE.  The
 * query only looks at the alignment of a, b, c, never at what they point to.  Which kernels run
 * depends on the arguments and the tuning knobs alone, so a call recorded under stream capture
 * gives the bits of the eager call.  One exception: the cut of a bf16 / f16 product into two halves
 * of K that are added inside one launch (tiles 14 and 15) counts its halves in a device array of the library
 * (the one the strided-axis reductions use: a slice per stream, launches recorded under capture take
 * counters that are never handed out again); with more than 32 streams at once, or some 250 such
 * launches recorded, the same tile runs uncut and the last bits of the sums differ. */
DXH_API int dxh_matmul_workspace_bytes(int dtype, const void *a, const void *b, const void *c, int64_t batch,
                                       int64_t m, int64_t k, int64_t n, size_t *bytes);
DXH_API int dxh_matmul(int dtype, const void *a, const void *b, void *c, int64_t batch, int64_t m,
                       int64_t k, int64_t n, void *workspace, size_t workspace_bytes, void *stream);

/* ---- several products that share their left operand: C_j[m,n] = sum_k A[m,k] * B_j[k,n], j < count
 * No counterpart in the reference, which multiplies one product per instruction; for a caller that holds
 * several instructions at once and finds consecutive matmul lines on one A — the gate and up projections
 * of the front's gated MLP (front/py/deepx/nn/modules/mlp/gatedmlp.py:20-26), the q / k / v projections of
 * its attention.  Every C_j holds the bits dxh_matmul stores for the same pair.  bf16 / f16 products that
 * take one of the large tiles uncut go out as ONE launch over all pairs (the tiles of the second product
 * start as those of the first finish: one launch, one prologue, stores under the next K loops); anything
 * else runs as `count` ordinary products, one after another.  bs / cs: HOST arrays of `count` device
 * pointers, all C_j distinct.  Workspace as for dxh_matmul, sized by the query below. */
DXH_API int dxh_matmul_shared_a_workspace_bytes(int dtype, const void *a, const void *const *bs, void *const *cs, int count,
                                                int64_t m, int64_t k, int64_t n, size_t *bytes);
DXH_API int dxh_matmul_shared_a(int dtype, const void *a, const void *const *bs, void *const *cs, int count, int64_t m,
                                int64_t k, int64_t n, void *workspace, size_t workspace_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DXHIP_H */

/*
 * hipcx.h -- C ABI of the MI355X (gfx950) kernel library behind the ChainerX `hip` backend.
 *
 * One entry point per ChainerX kernel class on the inference hot path.  Each function performs
 * exactly the work of one `Backend::CallKernel<XxxKernel>(...)` in the reference and is what the
 * `HipXxxKernel::Call` override of the `hip` backend plugin forwards to.  Paths in the comments
 * are relative to the reference tree, `CX/` = `chainerx_cc/chainerx/`.
 *
 * Conventions
 *  - Arrays are described by `hipcx_array`: `data` is the device address of element (0,...,0),
 *    i.e. `raw_data + offset` (CX/backend_util.h:10-13); strides are in BYTES, signed, and may be
 *    0 (broadcast / keep-dims) or permuted (transposed views), as in CX/array.h.
 *  - dtype codes are the values of `chainerx::Dtype` (CX/dtype.h:19-29).
 *  - Scalars follow `chainerx::Scalar` (CX/scalar.h): a kind tag plus an int64 or a double.
 *  - Every call is asynchronous on `stream` (a `hipStream_t`, may be NULL for the default
 *    stream), like the CUDA backend (CX/cuda/elementwise.cuh:41-47).
 *  - Every entry point may be called from several host threads at once (CX/testing/threading.h:34-60 is how the
 *    reference tests that); state shared between calls is guarded inside the library.  The exceptions say so:
 *    hipcx_sum_static_scratch (one scratch array per device) and the profiling window (one per process).
 *  - Return value: 0 on success, otherwise a `hipcx_status` naming the ChainerX exception type
 *    (CX/error.h:48-95) the plugin must throw; `hipcx_last_error()` gives the message.
 *  - Kernels that need device scratch memory take `workspace`/`workspace_bytes`; the matching
 *    `*_workspace_size` function tells how much.  No kernel entry point allocates; device memory
 *    comes from the caller, who may get it from the pool below (hipcx_malloc).
 */
#ifndef HIPCX_H_
#define HIPCX_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HIPCX_MAX_NDIM 10 /* CX/constant.h:6 kMaxNdim */

typedef enum hipcx_dtype { /* CX/dtype.h:19-29 */
    HIPCX_BOOL = 1,
    HIPCX_INT8 = 2,
    HIPCX_INT16 = 3,
    HIPCX_INT32 = 4,
    HIPCX_INT64 = 5,
    HIPCX_UINT8 = 6,
    HIPCX_FLOAT16 = 7,
    HIPCX_FLOAT32 = 8,
    HIPCX_FLOAT64 = 9
} hipcx_dtype;

typedef enum hipcx_status { /* CX/error.h:48-95 */
    HIPCX_OK = 0,
    HIPCX_CHAINERX_ERROR = 1,
    HIPCX_DIMENSION_ERROR = 2,
    HIPCX_DTYPE_ERROR = 3,
    HIPCX_NOT_IMPLEMENTED_ERROR = 4,
    HIPCX_INDEX_ERROR = 5,
    HIPCX_BACKEND_ERROR = 6,
    HIPCX_DEVICE_ERROR = 7,
    HIPCX_OUT_OF_MEMORY_ERROR = 8 /* chainerx::cuda::OutOfMemoryError, CX/cuda/memory_pool.h:34-37 */
} hipcx_status;

typedef enum hipcx_scalar_kind { /* CX/dtype.h DtypeKind */
    HIPCX_KIND_BOOL = 0,
    HIPCX_KIND_INT = 1,
    HIPCX_KIND_FLOAT = 3
} hipcx_scalar_kind;

typedef enum hipcx_index_bounds_mode { /* CX/array_index.h:21-26 */
    HIPCX_BOUNDS_DEFAULT = 0,
    HIPCX_BOUNDS_RAISE = 1,
    HIPCX_BOUNDS_WRAP = 2,
    HIPCX_BOUNDS_CLIP = 3
} hipcx_index_bounds_mode;

typedef enum hipcx_avg_pool_pad_mode { /* CX/routines/pooling.h:13-16 */
    HIPCX_PAD_ZERO = 1,
    HIPCX_PAD_IGNORE = 2
} hipcx_avg_pool_pad_mode;

typedef struct hipcx_array {
    void* data;
    int32_t dtype;
    int32_t ndim;
    int64_t shape[HIPCX_MAX_NDIM];
    int64_t strides[HIPCX_MAX_NDIM];
} hipcx_array;

typedef struct hipcx_scalar {
    int32_t kind; /* hipcx_scalar_kind */
    int32_t reserved;
    int64_t i; /* value when kind is BOOL or INT */
    double f;  /* value when kind is FLOAT */
} hipcx_scalar;

/* ---- library ---- */
const char* hipcx_last_error(void); /* thread-local message of the last failing call */
int hipcx_version(void);
int hipcx_device_count(int* count);          /* Backend::GetDeviceCount, CX/backend.h:29 */
int hipcx_synchronize(int device_index);     /* Device::Synchronize, CX/device.h:71 */
int hipcx_device_name(int device_index, char* buf, size_t buf_len);

/* ---- device memory: chainerx::Device (CX/device.h:24-71) as the CUDA backend implements it (CX/cuda/cuda_device/memory.cc) ----
 * Allocation goes through a pool per device (role of chainerx::cuda::MemoryPool, CX/cuda/memory_pool.{h,cc}): 512-byte
 * allocation units, freed blocks are cached and reused, and when the driver reports out of memory the cached blocks are
 * released and the allocation is tried once more before HIPCX_OUT_OF_MEMORY_ERROR is returned (memory_pool.cc:236-243).
 *   hipcx_malloc            Device::Allocate, device.h:33 (0 bytes -> NULL, CX/native/native_device/memory.cc:14-19)
 *   hipcx_free              the deleter of an allocation (cuda_device/memory.cc:19-24): returns the block to the pool; a pointer
 *                           the pool does not hold is HIPCX_CHAINERX_ERROR (memory_pool.cc:262-264); after hipcx_pool_destroy
 *                           it does nothing (the pool took its memory with it), also when a new pool exists on the device by then
 *   hipcx_record_stream     no counterpart in the reference (it launches everything on one stream): announces that `ptr`, a block
 *                           in use, has work queued on `stream`, a stream other than the one it was allocated for
 *                           (hipcx_malloc: the null stream).  hipcx_free then keeps the block out of the free lists until the work
 *                           that stream holds at the time of the free has run.  Without the announcement a block must not be
 *                           freed before its last use on a foreign stream was waited for: a block goes back to the free list of
 *                           its own stream at once and the next allocation there may overwrite it
 *   hipcx_pool_free_unused  MemoryPool::FreeUnusedBlocks, memory_pool.cc:172-203
 *   hipcx_pool_destroy      ~MemoryPool (memory_pool.cc:160-170): waits for the device, then gives every block back to the driver
 *   hipcx_memcpy_from_host  Device::MemoryCopyFrom with a native source = MemoryCopyFromHostAsync (cuda_device/memory.cc:37-51): the
 *                           bytes are staged in pooled page-locked memory and copied asynchronously on `stream`; `src` may be
 *                           reused as soon as the call returns
 *   hipcx_memcpy_to_host    Device::MemoryCopyTo with a native destination (cuda_device/memory.cc:104-122): ordered behind the work
 *                           queued on `stream`, complete when the call returns
 *   hipcx_memcpy_device     MemoryCopyFrom / MemoryCopyTo between hip devices (cuda_device/memory.cc:84-91,110-113), asynchronous
 *   hipcx_from_host_memory  Device::FromHostMemory, device.h:64 = Allocate + MemoryCopyFromHostAsync (cuda_device/memory.cc:146-150);
 *                           TransferDataFrom / TransferDataTo (device.h:49-60) are hipcx_malloc + one of the copies above
 *   hipcx_check_device_pointer  the check of Device::MakeDataFromForeignPointer (cuda_device/memory.cc:53-75)
 * hipcx_malloc_on_stream has no counterpart either (the reference launches everything on one stream): a block allocated for
 * `stream` is, once freed, only handed to later allocations for the same stream, so work queued on different streams (e.g. by
 * different host threads) never shares a block that may still be in use; hipcx_malloc is the null stream's variant, and
 * hipcx_from_host_memory allocates for the stream it copies on.  hipcx_free needs no stream: a block remembers where it belongs.
 * Arenas have no counterpart in the reference: allocations made after hipcx_pool_set_arena(device, a) with a > 0 come from, and
 * return to, free lists of their own, so the addresses a HIP graph captured in arena a refers to are not handed to anybody else
 * until hipcx_pool_release_arena(device, a).  Arena 0 is the general one.  The setting is per device, not per thread. */
typedef struct hipcx_pool_stats_t {
    uint64_t in_use_bytes;       /* handed out, rounded sizes */
    uint64_t cached_bytes;       /* free blocks held for reuse */
    uint64_t in_use_blocks;
    uint64_t cached_blocks;
    uint64_t device_allocations; /* hipMalloc calls that succeeded so far */
    uint64_t retries;            /* allocations that only succeeded after the cache was released */
} hipcx_pool_stats_t;
int hipcx_malloc(int device, size_t bytes, void** ptr);
int hipcx_malloc_on_stream(int device, size_t bytes, void* stream, void** ptr);
int hipcx_free(int device, void* ptr);
int hipcx_record_stream(int device, void* ptr, void* stream);
int hipcx_pool_free_unused(int device);
int hipcx_pool_stats(int device, hipcx_pool_stats_t* stats);
int hipcx_pool_set_arena(int device, int arena);
int hipcx_pool_release_arena(int device, int arena);
int hipcx_pool_destroy(int device);
int hipcx_memcpy_from_host(int device, void* dst, const void* src, size_t bytes, void* stream);
int hipcx_memcpy_to_host(int device, void* dst, const void* src, size_t bytes, void* stream);
int hipcx_memcpy_device(int dst_device, void* dst, int src_device, const void* src, size_t bytes, void* stream);
int hipcx_from_host_memory(int device, const void* src, size_t bytes, void** out, void* stream);
int hipcx_check_device_pointer(int device, const void* ptr);

/* ---- elementwise arithmetic: CX/kernels/arithmetic.h ---- */
/* Inputs must already have out's dtype (the plugin applies AsType as CX/native/kernel_regist.h:55-56 does). */
int hipcx_add(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream);        /* AddKernel :11 */
int hipcx_add_as(const hipcx_array* x1, hipcx_scalar x2, const hipcx_array* out, void* stream);           /* AddASKernel :16 */
int hipcx_subtract(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream);   /* SubtractKernel :21 */
int hipcx_subtract_as(const hipcx_array* x1, hipcx_scalar x2, const hipcx_array* out, void* stream);      /* SubtractASKernel :26 */
int hipcx_multiply(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream);   /* MultiplyKernel :31 */
int hipcx_multiply_as(const hipcx_array* x1, hipcx_scalar x2, const hipcx_array* out, void* stream);      /* MultiplyASKernel :36 */
int hipcx_divide(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream);     /* DivideKernel :56 */
int hipcx_divide_as(const hipcx_array* x1, hipcx_scalar x2, const hipcx_array* out, void* stream);        /* DivideASKernel :61 */
int hipcx_divide_sa(hipcx_scalar x1, const hipcx_array* x2, const hipcx_array* out, void* stream);        /* DivideSAKernel :66 */

/* ---- elementwise math: CX/kernels/explog.h, hyperbolic.h, misc.h ---- */
int hipcx_exp(const hipcx_array* x, const hipcx_array* out, void* stream);   /* ExpKernel explog.h:15 */
int hipcx_log(const hipcx_array* x, const hipcx_array* out, void* stream);   /* LogKernel explog.h:30 */
int hipcx_tanh(const hipcx_array* x, const hipcx_array* out, void* stream);  /* TanhKernel hyperbolic.h:18 */
int hipcx_sqrt(const hipcx_array* x, const hipcx_array* out, void* stream);  /* SqrtKernel misc.h:14 */
/* out = x1 < x2 ? pos : neg   (ReLU is Maximum(x,0) = IfLessElse(x,0,0,x), CX/routines/misc.cc:210-216) */
int hipcx_if_less_else_assa(const hipcx_array* x1, hipcx_scalar x2, hipcx_scalar pos, const hipcx_array* neg,
                            const hipcx_array* out, void* stream);            /* IfLessElseASSAKernel misc.h:36 */
int hipcx_if_greater_else_assa(const hipcx_array* x1, hipcx_scalar x2, hipcx_scalar pos, const hipcx_array* neg,
                               const hipcx_array* out, void* stream);         /* IfGreaterElseASSAKernel misc.h:43 */
int hipcx_if_greater_else_aaaa(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* pos, const hipcx_array* neg,
                               const hipcx_array* out, void* stream);         /* IfGreaterElseAAAAKernel misc.h:48 */

/* ---- logic: CX/kernels/logic.h (inputs share one dtype, out is bool) ---- */
int hipcx_equal(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream);          /* EqualKernel :9 */
int hipcx_not_equal(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream);      /* NotEqualKernel :14 */
int hipcx_greater(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream);        /* GreaterKernel :19 */
int hipcx_greater_equal(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream);  /* GreaterEqualKernel :24 */

/* ---- creation: CX/kernels/creation.h, misc.h ---- */
int hipcx_copy(const hipcx_array* a, const hipcx_array* out, void* stream);                       /* CopyKernel creation.h:16 (dtype-casting) */
int hipcx_fill(const hipcx_array* out, hipcx_scalar value, void* stream);                         /* FillKernel misc.h:9 */
int hipcx_arange(hipcx_scalar start, hipcx_scalar step, const hipcx_array* out, void* stream);    /* ArangeKernel creation.h:11 */

/* ---- further elementwise kernels ----
 * hipcx_unary: out = f(x), x.dtype == out.dtype.  Float dtypes only (float16 as Float16(f(float(x))), CX/numeric.h:59-83) for
 *   ErfKernel explog.h:10, Expm1Kernel :20, Exp2Kernel :25, Log10Kernel :35, Log2Kernel :40, Log1pKernel :45,
 *   SinhKernel hyperbolic.h:8, CoshKernel :13, ArcsinhKernel :23, ArccoshKernel :28,
 *   SinKernel trigonometric.h:8, CosKernel :13, TanKernel :18, ArcsinKernel :23, ArccosKernel :28, ArctanKernel :33,
 *   CeilKernel rounding.h:8, FloorKernel :13;
 *   numeric dtypes for SquareKernel misc.h:19 (x*x), AbsKernel :24, SignKernel :29 (NaN passes; CX/numeric.h:33-57). */
enum hipcx_unary_op {
    HIPCX_UNARY_ERF = 1, HIPCX_UNARY_EXPM1, HIPCX_UNARY_EXP2, HIPCX_UNARY_LOG10, HIPCX_UNARY_LOG2, HIPCX_UNARY_LOG1P,
    HIPCX_UNARY_SINH, HIPCX_UNARY_COSH, HIPCX_UNARY_ARCSINH, HIPCX_UNARY_ARCCOSH,
    HIPCX_UNARY_SIN, HIPCX_UNARY_COS, HIPCX_UNARY_TAN, HIPCX_UNARY_ARCSIN, HIPCX_UNARY_ARCCOS, HIPCX_UNARY_ARCTAN,
    HIPCX_UNARY_CEIL, HIPCX_UNARY_FLOOR,
    HIPCX_UNARY_SQUARE, HIPCX_UNARY_ABS, HIPCX_UNARY_SIGN
};
int hipcx_unary(int op, const hipcx_array* x, const hipcx_array* out, void* stream);

/* bool out = p(x), any x dtype: LogicalNotKernel logic.h:29 (!x), IsNanKernel :59, IsInfKernel :64, IsFiniteKernel :69
 * (integers and bool are never NaN / Inf, CX/numeric.h:17-31). */
enum hipcx_predicate_op { HIPCX_PRED_LOGICAL_NOT = 1, HIPCX_PRED_ISNAN, HIPCX_PRED_ISINF, HIPCX_PRED_ISFINITE };
int hipcx_predicate(int op, const hipcx_array* x, const hipcx_array* out, void* stream);

/* bool out = x1 op x2 on the truth values, operands of one dtype: LogicalAndKernel logic.h:34, LogicalOrKernel :39,
 * LogicalXorKernel :44 (!x1 != !x2). */
enum hipcx_logical_op { HIPCX_LOGICAL_AND = 1, HIPCX_LOGICAL_OR, HIPCX_LOGICAL_XOR };
int hipcx_logical(int op, const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream);

/* PowerKernel arithmetic.h:71, PowerASKernel :76, PowerSAKernel :81: numeric dtypes; integers by repeated squaring with
 * wrap-around, negative integer exponents give 0 except for bases 1 and -1 (CX/numeric.h:85-135); floats through pow.
 * FmodKernel arithmetic.h:107 and Arctan2Kernel trigonometric.h:38: float dtypes. */
int hipcx_power(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream);
int hipcx_power_as(const hipcx_array* x1, hipcx_scalar x2, const hipcx_array* out, void* stream);
int hipcx_power_sa(hipcx_scalar x1, const hipcx_array* x2, const hipcx_array* out, void* stream);
int hipcx_fmod(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream);
int hipcx_arctan2(const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream);

/* Integer-flavoured binary kernels, operands and out of one dtype; _as takes x2 as a scalar, _sa takes x1 as a scalar:
 *   FloorDivideKernel arithmetic.h:41, FloorDivideASKernel :46, FloorDivideSAKernel :51 and ModAAKernel :86, ModASKernel :93,
 *   ModSAKernel :100 -- numeric dtypes; integers round towards -inf and give 0 for a zero divisor, float Mod by zero is NaN
 *   (native/native_device/arithmetic.cc:107-139, 260-295);
 *   BitwiseAndKernel binary.h:11, BitwiseAndASKernel :16, BitwiseOrKernel :21, BitwiseOrASKernel :26, BitwiseXorKernel :31,
 *   BitwiseXorASKernel :36 -- bool and integer dtypes;
 *   LeftShiftAAKernel binary.h:41, LeftShiftASKernel :46, LeftShiftSAKernel :51, RightShiftAAKernel :56, RightShiftASKernel :61,
 *   RightShiftSAKernel :66 -- integer dtypes, evaluated in the promoted type as `x1 << x2` is in C++; a count outside
 *   [0, width of the promoted type) is undefined in the reference and is masked to that width here. */
enum hipcx_binary_op {
    HIPCX_BINARY_FLOOR_DIVIDE = 1, HIPCX_BINARY_MOD, HIPCX_BINARY_BITWISE_AND, HIPCX_BINARY_BITWISE_OR, HIPCX_BINARY_BITWISE_XOR,
    HIPCX_BINARY_LEFT_SHIFT, HIPCX_BINARY_RIGHT_SHIFT
};
int hipcx_binary(int op, const hipcx_array* x1, const hipcx_array* x2, const hipcx_array* out, void* stream);
int hipcx_binary_as(int op, const hipcx_array* x1, hipcx_scalar x2, const hipcx_array* out, void* stream);
int hipcx_binary_sa(int op, hipcx_scalar x1, const hipcx_array* x2, const hipcx_array* out, void* stream);

/* WhereKernel indexing.h:22, WhereAASKernel :27, WhereASAKernel :32, WhereASSKernel :37: out = condition ? x : y with a bool
 * condition array and x / y of out's dtype, arrays or scalars (native/native_device/indexing.cc:194-283). */
int hipcx_where(const hipcx_array* condition, const hipcx_array* x, const hipcx_array* y, const hipcx_array* out, void* stream);
int hipcx_where_aas(const hipcx_array* condition, const hipcx_array* x, hipcx_scalar y, const hipcx_array* out, void* stream);
int hipcx_where_asa(const hipcx_array* condition, hipcx_scalar x, const hipcx_array* y, const hipcx_array* out, void* stream);
int hipcx_where_ass(const hipcx_array* condition, hipcx_scalar x, hipcx_scalar y, const hipcx_array* out, void* stream);

/* ---- reductions: CX/kernels/reduction.h:18, statistics.h:13, sorting.h:9 ----
 * `axis` is sorted, unique, non-negative (CX/kernels/reduction.h:11-18); `out` either drops the
 * reduced axes or keeps them with extent 1.  argmax writes int64 and reproduces the native
 * backend's tie/NaN rule bit for bit (CX/native/reduce.h:46-83 with the functor of
 * CX/native/native_device/reduction.cc:34-61). */
size_t hipcx_reduce_workspace_size(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out);
int hipcx_sum(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out, void* workspace, size_t workspace_bytes,
              void* stream);
int hipcx_amax(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out, void* workspace, size_t workspace_bytes,
               void* stream);
int hipcx_argmax(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out, void* workspace,
                 size_t workspace_bytes, void* stream);

/* AMinKernel statistics.h:20 (identity MaxOrInf, NaN-propagating, native/native_device/statistics.cc:52-73); ArgMinKernel
 * sorting.h:14 (same tie/NaN rule as argmax with the comparison mirrored, native/native_device/reduction.cc:65-92);
 * AllKernel / AnyKernel logic.h:49,54 over bool arrays (the routine casts other dtypes to bool first,
 * native/native_device/logic.cc NativeAllKernel / NativeAnyKernel).  Workspace as for hipcx_sum. */
int hipcx_amin(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out, void* workspace, size_t workspace_bytes,
               void* stream);
int hipcx_argmin(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out, void* workspace,
                 size_t workspace_bytes, void* stream);
int hipcx_all(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out, void* workspace, size_t workspace_bytes,
              void* stream);
int hipcx_any(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out, void* workspace, size_t workspace_bytes,
              void* stream);

/* hipcx_sum without a workspace argument.  No counterpart in the reference: it is for callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc) and so cannot provide the workspace
 * hipcx_sum asks for.  The partial results live in a static device array of HIPCX_STATIC_SCRATCH_BYTES inside the library (one
 * copy per device, held until the process ends); the call allocates and frees nothing.  Reductions whose
 * hipcx_reduce_workspace_size exceeds that are refused with HIPCX_CHAINERX_ERROR.  Results are bit-identical to hipcx_sum's.
 * Calls that overlap on one device share the array and race: issue them on one stream, or serialise them. */
#define HIPCX_STATIC_SCRATCH_BYTES (4u << 20)
int hipcx_sum_static_scratch(const hipcx_array* a, const int8_t* axis, int naxis, const hipcx_array* out, void* stream);

/* ---- linear algebra / connection: CX/kernels/linalg.h:15, connection.h:21 ---- */
/* out[M,N] = a[M,K] . b[K,N], all three of one dtype.  float16/32/64 run on the matrix pipes; fp16 accumulates in fp32.  The
 * integer dtypes and bool are multiplied as the native backend does (CX/native/native_device/dot.cc:130-134, 181-227: one
 * accumulator of the array dtype, i.e. sums modulo 2^bits; bool is "any of the conjunctions") by a plain tiled kernel -- the cuda
 * backend raises for them (CX/cuda/cuda_device/dot.cu:74-76). */
size_t hipcx_dot_workspace_size(const hipcx_array* a, const hipcx_array* b, const hipcx_array* out);
int hipcx_dot(const hipcx_array* a, const hipcx_array* b, const hipcx_array* out, void* workspace, size_t workspace_bytes,
              void* stream);
/* Output extent of a convolution/pooling window (CX/routines/connection.cc:37-49). Returns -1 if not positive. */
int64_t hipcx_conv_out_dim(int64_t in_dim, int64_t kernel_size, int64_t stride, int64_t pad, int cover_all);
/* Convolution forward (ConvKernel CX/kernels/connection.h:14-32), x[N,C,H,W] (any strides), w[K,C,kh,kw], optional b[K] (NULL = none),
 * out[N,K,OH,OW] with any strides.  Other ranks, like the native kernel (CX/native/native_device/conv.cc:57-89): x[N,C,d_1..d_n] with
 * w[K,C,k_1..k_n], `stride` and `pad` holding n values; n = 0 and 1 run the 2-D kernels over extents of one, n >= 3 a plain
 * one-thread-per-output kernel (a correctness path: float accumulation for float16, bias added after rounding, as the native backend).
 * Integer dtypes and bool, which the native backend's Im2Col + TensorDot accepts like any other, run that plain kernel at every
 * rank (sums modulo 2^bits, equal bit for bit).  The plugin and the Python mirror allocate out C-contiguous (NCHW memory), like the CUDA
 * backend (CX/cuda/cuda_conv.cc:311); the native backend's own result is an NCHW view of NHWC memory
 * (CX/native/native_device/conv.cc:78-84), which this entry also accepts as `out`. */
size_t hipcx_conv_workspace_size(const hipcx_array* x, const hipcx_array* w, const hipcx_array* out);
/* Which kernel family hipcx_conv runs for these arguments (no counterpart in the reference: for tests and benchmarks that must
 * know that a specialised kernel, not the general one, produced a result).  0: general implicit GEMM (any dtype / layout);
 * 1: float16 NCHW kernels with 128-wide tiles; 2: float16 7x7 / 2 stem kernel; 3: float16 1x1 / stride 1 kernel that loads its
 * operands straight into LDS and walks 256 x 128 tiles; -1: invalid arguments. */
int hipcx_conv_route(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const int64_t* stride, const int64_t* pad,
                     const hipcx_array* out);
int hipcx_conv(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const int64_t* stride, const int64_t* pad,
               int cover_all, const hipcx_array* out, void* workspace, size_t workspace_bytes, void* stream);

/* ---- Im2Col / Col2Im (CX/native/im2col.cc:82-149, col2im.cc:76-122) and ConvTransposeKernel (CX/kernels/connection.h:51-66) ----
 * Two spatial axes; arrays of any strides (multiples of the item size).
 * hipcx_im2col: col[N, C, kh, kw, oh, ow] (kernel and window extents are read from col's shape; oh / ow must be
 *   hipcx_conv_out_dim of x's) gathered from x[N, C, H, W]; positions in the padding hold pad_value.  Any dtype.
 * hipcx_col2im: out[N, C, H, W] = for every image position the sum of the col elements that cover it, added in ascending
 *   (r, s) order from zero with one rounding to the dtype per addition: bit-identical to the native backend's chain of in-place
 *   strided Add kernels on a zero-filled padded image, cropped.  Any dtype but bool.
 * hipcx_conv_transpose: x[N, C_in, H, W], w[C_in, C_out, kh, kw], optional b[C_out], out[N, C_out, OH, OW] with OH / OW any size
 *   consistent with x's (CX/routines/connection.cc:268-279); all of one floating point dtype.  Stride 1 runs as one forward
 *   convolution with flipped filters, a 1x1 unpadded filter as a 1x1 convolution scattered into zeros, everything else as the
 *   native composition (matrix product over the input channels, col2im, bias).  `workspace`: 256-byte aligned device memory of
 *   hipcx_conv_transpose_workspace_size bytes.  Other ranks (x[N, C_in, d_1..d_n], w[C_in, C_out, k_1..k_n], n values in `stride`
 *   and `pad`, as the native kernel takes them, CX/native/native_device/conv.cc:126-160) run a plain one-thread-per-output kernel
 *   that follows the native composition's order of operations (bit-identical to it); no workspace. */
int hipcx_im2col(const hipcx_array* x, const int64_t* stride, const int64_t* pad, int cover_all, hipcx_scalar pad_value,
                 const hipcx_array* col, void* stream);
int hipcx_col2im(const hipcx_array* col, const int64_t* stride, const int64_t* pad, const hipcx_array* out, void* stream);
size_t hipcx_conv_transpose_workspace_size(const hipcx_array* x, const hipcx_array* w, const int64_t* stride, const int64_t* pad,
                                           const hipcx_array* out);
int hipcx_conv_transpose(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const int64_t* stride, const int64_t* pad,
                         const hipcx_array* out, void* workspace, size_t workspace_bytes, void* stream);

/* Opt-in fused entry.  No single kernel of the reference corresponds to it: it is the composition
 *   ConvKernel -> FixedBatchNormKernel over the output channels (axis (0,2,3), CX/routines/normalization.cc:113-153)
 *   -> AddKernel with `residual` -> IfLessElseASSAKernel(x, 0, 0, x) (ReLU, CX/routines/misc.cc:210-216)
 * that Chainer's conv-bn-relu blocks issue as separate kernel calls; here the tail runs in the convolution's epilogue,
 * in float on the float accumulator, and `out` is written once.  gamma/beta/mean/var are all NULL (no batch norm) or
 * hold one value of out's dtype per output channel ([K] or [1,K,1,1]); `residual` may be NULL; `relu` is 0 or 1.
 * Layouts or dtypes the fused kernel does not take are served by the separate kernels run in place on `out`.
 * Workspace as for hipcx_conv. */
int hipcx_conv_bn_act(const hipcx_array* x, const hipcx_array* w, const hipcx_array* b, const int64_t* stride, const int64_t* pad,
                      int cover_all, const hipcx_array* gamma, const hipcx_array* beta, const hipcx_array* mean, const hipcx_array* var,
                      hipcx_scalar eps, const hipcx_array* residual, int relu, const hipcx_array* out, void* workspace,
                      size_t workspace_bytes, void* stream);

/* Opt-in fused entries for two routine chains.  No single kernel of the reference corresponds to either.
 *
 * hipcx_log_softmax: LogSoftmax along axis 1 of a 2-D array (CX/routines/reduction.cc:78-92: AMaxKernel, SubtractKernel,
 *   ExpKernel, SumKernel, LogKernel, AddKernel, SubtractKernel -- 5 reads and 3 writes of the array) as one read and one
 *   write when a row is at most 64 KiB, two reads and one write otherwise (then `workspace` must hold
 *   hipcx_log_softmax_workspace_size(x) bytes).  Same float operations as the chain (max with AMax's NaN rule, exp(x - max),
 *   sum, max + log(sum), x - that); only the order of the row sum differs.  x and out: same shape and float dtype, unit
 *   stride along axis 1, any non-negative row stride.
 * hipcx_lstm_cell: the Lstm routine (CX/routines/connection.cc:396-446) for equal batch sizes: gate k of unit j is column
 *   4j+k of x[B,4H]; a = tanh(g0), i, f, o = 1/(1+exp(-g)) (CX/routines/activation.cc:74-78); c_out = a*i + f*c;
 *   h_out = o*tanh(c_out).  Same operations in the same order as the ~25 separate kernels: bit-identical for float32/float64
 *   (float16 rounds once instead of after every kernel).  Errors as the routine raises them (DimensionError, DtypeError). */
/* hipcx_n_step_lstm: RnnKernel (CX/kernels/rnn.h:34-49) in LSTM mode, one direction, float32 -- what NStepLstm
 *   (CX/routines/n_step_rnn.cc:434-443) computes.  The reference hands this kernel only to its "cuda" backend (n_step_rnn.cc:210)
 *   and composes the routine elsewhere, so a hip plugin reaches it after that test is widened; until then it is opt-in.
 *   hx, cx, hy, cy: [n_layers, B, H]; ws / bs: n_layers * 8 matrices [H, in] / vectors [H] in cuDNN order (input, forget, cell,
 *   output for x, then for h; in = xs' columns for layer 0, H above); xs[t]: [B_t, in] with B_t <= B; ys[t]: [B_t, H].  State rows
 *   beyond a step's batch keep their values.  The eight matrices of a layer are packed once per call, every launch advances all
 *   layers by one step (a wavefront: n_steps + n_layers - 1 launches), the gates never reach memory.  Equal to the composition
 *   within float32 tolerance (the sums run in another order).  Other dtypes: HIPCX_NOT_IMPLEMENTED_ERROR (compose the routine).
 *   `workspace`: 256-byte aligned, hipcx_n_step_lstm_workspace_size bytes (packed weights, padded state, layer outputs). */
size_t hipcx_n_step_lstm_workspace_size(int n_layers, const hipcx_array* hx, const hipcx_array* const* xs, int n_steps);
int hipcx_n_step_lstm(int n_layers, const hipcx_array* hx, const hipcx_array* cx, const hipcx_array* const* ws, const hipcx_array* const* bs,
                      const hipcx_array* const* xs, int n_steps, const hipcx_array* hy, const hipcx_array* cy, const hipcx_array* const* ys,
                      void* workspace, size_t workspace_bytes, void* stream);
/* hipcx_n_step_rnn / hipcx_n_step_rnn_backward: RnnKernel and RnnBackwardKernel (CX/kernels/rnn.h:34-66) for float32, every mode
 *   NStepRnnImpl passes (CX/routines/n_step_rnn.cc:434-497): `mode` 0 GRU, 1 LSTM, 2 RNN (`activation` 0 tanh, 1 relu; ignored for
 *   the other modes), `bidirectional` 0 / 1.  D = directions, G = 3 / 4 / 1 gates.
 *   hx, hy (cx, cy: LSTM only, else NULL): [n_layers * D, B, H], index layer * D + direction.  ws / bs: for every layer-direction
 *   2 * G matrices [H, in] ([H, H] for the second G) / vectors [H] in the reference's (cuDNN's) order, in = xs' columns for layer 0
 *   and D * H above.  xs[t]: [B_t, in] with B_t <= B; ys[t]: [B_t, D * H] (unit stride along the last axis).  Rows of the state beyond
 *   B_t keep their values (OneDirectionalLoop, n_step_rnn.cc:133-175).
 *   `reserve`: NULL for inference; for training hipcx_n_step_rnn_reserve_size bytes (256-byte aligned) that the forward pass fills
 *   (gate activations, the states before each step, the lower layers' outputs: the role of RnnGradState) and the backward pass reads.
 *   `workspace`: 256-byte aligned, hipcx_n_step_rnn_workspace_size bytes (`training` 1 covers both passes).
 *   Backward (RnnBackwardKernel::Call's grad lists): dhy (dcy: LSTM, may be NULL = zeros), dys[t] [B_t, D * H] (an entry may be NULL =
 *   zeros) -> dhx (dcx), dws / dbs shaped and ordered like ws / bs (C-contiguous), dxs[t] [B_t, in].
 *   Equal to the routine composition / its autograd gradients to float32 tolerance (sums in another order).  One-direction LSTM
 *   inference runs hipcx_n_step_lstm. */
size_t hipcx_n_step_rnn_reserve_size(int n_layers, int bidirectional, int mode, const hipcx_array* hx, const hipcx_array* const* xs, int n_steps);
size_t hipcx_n_step_rnn_workspace_size(int n_layers, int bidirectional, int mode, int training, const hipcx_array* hx, const hipcx_array* const* xs,
                                       int n_steps);
int hipcx_n_step_rnn(int n_layers, int bidirectional, int mode, int activation, const hipcx_array* hx, const hipcx_array* cx,
                     const hipcx_array* const* ws, const hipcx_array* const* bs, const hipcx_array* const* xs, int n_steps, const hipcx_array* hy,
                     const hipcx_array* cy, const hipcx_array* const* ys, void* reserve, size_t reserve_bytes, void* workspace,
                     size_t workspace_bytes, void* stream);
int hipcx_n_step_rnn_backward(int n_layers, int bidirectional, int mode, int activation, const hipcx_array* hx, const hipcx_array* const* ws,
                              const hipcx_array* const* bs, const hipcx_array* const* xs, int n_steps, const hipcx_array* dhy,
                              const hipcx_array* dcy, const hipcx_array* const* dys, const void* reserve, size_t reserve_bytes,
                              const hipcx_array* dhx, const hipcx_array* dcx, const hipcx_array* const* dws, const hipcx_array* const* dbs,
                              const hipcx_array* const* dxs, void* workspace, size_t workspace_bytes, void* stream);
size_t hipcx_log_softmax_workspace_size(const hipcx_array* x);
int hipcx_log_softmax(const hipcx_array* x, const hipcx_array* out, void* workspace, size_t workspace_bytes, void* stream);
int hipcx_lstm_cell(const hipcx_array* c, const hipcx_array* x, const hipcx_array* h_out, const hipcx_array* c_out, void* stream);

/* Measurement aid (no counterpart in the reference): between start and stop every implicit-GEMM launch made by
 * hipcx_dot / hipcx_conv from the calling process is bracketed by a pair of HIP events on its stream.  stop waits for them
 * and returns the number of launches, the sum of their durations, and their algorithmic flops (2 per multiply-add) and
 * bytes (each operand once).  One profiling window per process at a time; launches from any thread are recorded into it. */
int hipcx_profile_start(void);
int hipcx_profile_stop(int64_t* launches, double* total_ms, double* flops, double* bytes);
/* The launches of the last closed profiling window one by one, in launch order: duration, algorithmic flops and bytes of the
 * first min(capacity, *count) of them; *count is the number recorded.  Valid until the next hipcx_profile_start. */
int hipcx_profile_records(int64_t capacity, double* ms, double* flops, double* bytes, int64_t* count);

/* ---- normalization: FixedBatchNormKernel CX/kernels/normalization.h:107 ----
 * gamma/beta/mean/var have the keep-dims reduced shape of x over `axis`
 * (CX/routines/normalization.cc:61-101). out has x's shape and dtype. */
int hipcx_fixed_batch_norm(const hipcx_array* x, const hipcx_array* gamma, const hipcx_array* beta, const hipcx_array* mean,
                           const hipcx_array* var, hipcx_scalar eps, const int8_t* axis, int naxis, const hipcx_array* out,
                           void* stream);

/* ---- ConvGradWeightKernel CX/kernels/connection.h:34-49 (2-D, C-contiguous NCHW x and gy in gw's float dtype) ----
 * gw[k, c, r, s] = sum over n, oh, ow of gy[n, k, oh, ow] * x[n, c, oh*stride - pad + r, ow*stride - pad + s]: the native
 * backend's TensorDot(gy, Im2Col(x)) (CX/native/native_device/conv.cc:91-124), equal to tolerance (float accumulation).
 * inf / NaN in x or gy give the reference's inf / NaN in the reference's filter taps: the route for filters larger than 1x1 at
 * stride 1 (float16 / float32), whose sum runs over zero-padded rows in which an x value also meets zeros of a padded gy, notes
 * the input channels that hold a non-finite value and sums their taps again over the reference's windows.
 * Other ranks (x[N, C, d_1..d_n], gy[N, K, o_1..o_n], gw[K, C, k_1..k_n], any strides) run a plain kernel, one thread per filter
 * element with the native Dot's order of fused multiply-adds (bit-identical to the composition); no workspace. */
size_t hipcx_conv_grad_weight_workspace_size(const hipcx_array* x, const hipcx_array* gy, const hipcx_array* gw, const int64_t* stride,
                                             const int64_t* pad, int cover_all);
int hipcx_conv_grad_weight(const hipcx_array* x, const hipcx_array* gy, const int64_t* stride, const int64_t* pad, int cover_all,
                           const hipcx_array* gw, void* workspace, size_t workspace_bytes, void* stream);

/* ---- linear algebra: SolveKernel, InverseKernel, CholeskyKernel CX/kernels/linalg.h:20-43 (float32 / float64, 2-D) ----
 * The native backend calls LAPACK gesv / getrf + getri / potrf (CX/native/native_device/linalg.cc:280-347, 560-600); these entries
 * agree with it to rounding (blocked factorisations, 32 columns at a time, spread over many workgroups).  `out` is C-contiguous;
 * a (and b) are cast to out's dtype.  `error_flag`: a device int32 the caller zeroes; a singular / not positive definite matrix
 * stores LAPACK's `info` (1-based position) there and the reference's ChainerxError is the caller's to raise.  Workspace:
 * hipcx_solve_workspace_size(a) bytes for solve and inverse. */
size_t hipcx_solve_workspace_size(const hipcx_array* a);
int hipcx_solve(const hipcx_array* a, const hipcx_array* b, const hipcx_array* out, void* workspace, size_t workspace_bytes,
                int32_t* error_flag, void* stream);
int hipcx_inverse(const hipcx_array* a, const hipcx_array* out, void* workspace, size_t workspace_bytes, int32_t* error_flag, void* stream);
int hipcx_cholesky(const hipcx_array* a, const hipcx_array* out, int32_t* error_flag, void* stream);

/* ---- SyevdKernel CX/kernels/linalg.h:45-48 (float32 / float64, a 2-D and square) ----
 * Eigenvalues w (ascending) and, when compute_v, eigenvectors v (as columns) of the symmetric matrix held in a's `uplo` triangle
 * ('U' / 'L', either case; the other triangle is never read), as LAPACK syevd gives them to the native backend
 * (CX/native/native_device/linalg.cc:602-660).  Jacobi rotations: eigenvalues agree with LAPACK's to rounding, eigenvectors
 * up to the sign of each column (and up to a rotation inside an eigenspace of a repeated eigenvalue).  Up to 64 rows a two-sided
 * cyclic Jacobi runs in one workgroup; beyond that the columns of A + |A|_F I are made orthogonal by the one-sided block sweeps
 * of hipcx_svd (the rotations' product holds the eigenvectors, the eigenvalues are their Rayleigh quotients with A), and the
 * call waits for the stream once for the norm and once per sweep to read whether anything was rotated.  On a stream that is being
 * captured into a graph it waits for nothing: the norm stays on the device and 30 sweeps are recorded, each launch gated on the
 * flag of the sweep before it (the same rotations, the same results bit for bit; a matrix that needs more than 30 sweeps would be
 * left short of convergence there, against 60 with the host in the loop).
 * w: [n], v: [n, n], any strides, a's dtype.  Workspace: hipcx_syevd_workspace_size(a) bytes.  n <= 4096. */
size_t hipcx_syevd_workspace_size(const hipcx_array* a);
int hipcx_syevd(const hipcx_array* a, const hipcx_array* w, const hipcx_array* v, char uplo, int compute_v, void* workspace,
                size_t workspace_bytes, void* stream);

/* ---- QrKernel CX/kernels/linalg.h:38-41, modes CX/routines/linalg.h:22-28 (float32 / float64; a 2-D [m, n], cast to r's dtype) ----
 * Householder QR with LAPACK geqrf's reflectors (beta = -sign(alpha) * norm) and orgqr's Q, as the native backend calls them
 * (CX/native/native_device/linalg.cc:349-430): values and signs agree with it to rounding.  k = min(m, n).  Matrices of about a
 * hundred rows and more run as one launch per column with the trailing columns spread over workgroups, smaller ones (and those
 * above 4096 rows) in one workgroup.
 *   HIPCX_QR_REDUCED : q [m, k], r [k, n] upper triangular          HIPCX_QR_COMPLETE : q [m, m], r [m, n]
 *   HIPCX_QR_R       : r [k, n] alone (q ignored)                   HIPCX_QR_RAW      : r [n, m] = the factored matrix in column-major
 * order (R and the reflector vectors), q ignored.  tau [k] receives the reflector scalars in every mode. */
enum hipcx_qr_mode { HIPCX_QR_REDUCED = 0, HIPCX_QR_COMPLETE = 1, HIPCX_QR_R = 2, HIPCX_QR_RAW = 3 };
size_t hipcx_qr_workspace_size(const hipcx_array* a);
int hipcx_qr(const hipcx_array* a, const hipcx_array* q, const hipcx_array* r, const hipcx_array* tau, int mode, void* workspace,
             size_t workspace_bytes, void* stream);

/* ---- SvdKernel CX/kernels/linalg.h:33-36 (float32 / float64; a 2-D [m, n]; k = min(m, n)) ----
 * a = u @ diag(s) @ vt with s descending, as LAPACK gesdd gives it to the native backend (CX/native/native_device/linalg.cc:432-503):
 * u [m, k] and vt [k, n], or, full_matrices, u [m, m] and vt [n, n]; without compute_uv only s [k] is written (u, vt ignored).
 * One-sided Jacobi rotations: singular values agree with LAPACK's to rounding; singular vectors up to a common
 * sign of u[:, i] and vt[i, :] (and a rotation inside the space of a repeated value; the columns that complete a full u / vt, or
 * that belong to zero singular values, are some orthonormal basis of the same space).  Up to k = 64 the sweeps run in one
 * workgroup; beyond that a sweep is k / 16 launches over blocks of 16 columns (a workgroup per pair of blocks, a wavefront per
 * column pair), and the call waits for the stream once per sweep to read whether anything was rotated -- except on a stream that
 * is being captured into a graph, where 30 sweeps are recorded, each launch gated on the flag of the sweep before it (same
 * rotations, same results; see hipcx_syevd).  max(m, n) <= 4096. */
size_t hipcx_svd_workspace_size(const hipcx_array* a);
int hipcx_svd(const hipcx_array* a, const hipcx_array* u, const hipcx_array* s, const hipcx_array* vt, int full_matrices, int compute_uv,
              void* workspace, size_t workspace_bytes, void* stream);

/* ---- training-mode normalization: BatchNormKernel CX/kernels/normalization.h:32-47, BatchNormGradKernel :49-61 ----
 * For x C-contiguous with ndim >= 2 and `axis` = every axis but 1 (anything else: HIPCX_NOT_IMPLEMENTED_ERROR, and the caller
 * runs the reference's routine composition, CX/routines/normalization.cc:155-250).  gamma / beta / running_* / mean_out /
 * inv_std_out / ggamma / gbeta hold one value per channel, shaped [C] or as the keep-dims reduction of x, in x's dtype.
 * hipcx_batch_norm writes out, the batch mean and 1 / sqrt(var + eps) (the state the gradient needs) and updates running_mean /
 * running_var in place (decay, and n / max(n - 1, 1) on the variance).  Both need hipcx_batch_norm_workspace_size bytes. */
size_t hipcx_batch_norm_workspace_size(const hipcx_array* x, const int8_t* axis, int naxis);
/* 1 when hipcx_batch_norm / hipcx_batch_norm_grad take this case (x, the axis set, and `nparams` per-channel arrays: gamma,
 * beta, running statistics, or gout's state), 0 when the caller has to run the routine composition.  Sets no error. */
int hipcx_batch_norm_supported(const hipcx_array* x, const int8_t* axis, int naxis, const hipcx_array* const* params, int nparams);
int hipcx_batch_norm(const hipcx_array* x, const hipcx_array* gamma, const hipcx_array* beta, const hipcx_array* running_mean,
                     const hipcx_array* running_var, hipcx_scalar eps, hipcx_scalar decay, const int8_t* axis, int naxis,
                     const hipcx_array* out, const hipcx_array* mean_out, const hipcx_array* inv_std_out, void* workspace,
                     size_t workspace_bytes, void* stream);
int hipcx_batch_norm_grad(const hipcx_array* x, const hipcx_array* gamma, const hipcx_array* gout, const hipcx_array* mean,
                          const hipcx_array* inv_std, const int8_t* axis, int naxis, const hipcx_array* gx, const hipcx_array* ggamma,
                          const hipcx_array* gbeta, void* workspace, size_t workspace_bytes, void* stream);

/* ---- pooling: CX/kernels/pooling.h:29,83 (NCHW logical layout, any strides; x[N,C,d_1..d_n] with n values per window parameter:
 * the dedicated kernels are the 2-D ones, n = 1 runs them over an extent of one, n >= 3 a plain one-thread-per-output kernel with
 * the native backend's arithmetic, CX/native/native_device/pool.cc:69-94,191-302) ---- */
int hipcx_max_pool(const hipcx_array* x, const int64_t* kernel_size, const int64_t* stride, const int64_t* pad, int cover_all,
                   const hipcx_array* out, void* stream);
int hipcx_average_pool(const hipcx_array* x, const int64_t* kernel_size, const int64_t* stride, const int64_t* pad, int pad_mode,
                       const hipcx_array* out, void* stream);

/* ---- pooling gradients: MaxPoolGradKernel CX/kernels/pooling.h:47-65, AveragePoolGradKernel CX/kernels/pooling.h:95-107 ----
 * x is the forward input the reference keeps in its grad state; gx has x's shape.  Results carry the bits of the native
 * backend's Im2Col / ArgMax / Col2Im composition (CX/native/native_device/pool.cc:97-143, 304-346): contributions are added in
 * kernel-offset order with one rounding per addition, and the window maximum is chosen by ArgMax's tie and NaN rule.
 * `workspace`: device memory of hipcx_max_pool_grad_workspace_size(gout) bytes (the ArgMax of every window, one int each).
 * The three entries take any number of spatial axes like the forward ones (n values per window parameter); other than two run
 * plain kernels with the same bits and need no workspace. */
size_t hipcx_max_pool_grad_workspace_size(const hipcx_array* gout);
int hipcx_max_pool_grad(const hipcx_array* x, const hipcx_array* gout, const int64_t* kernel_size, const int64_t* stride,
                        const int64_t* pad, int cover_all, const hipcx_array* gx, void* workspace, size_t workspace_bytes, void* stream);
/* MaxPoolGradGradKernel CX/kernels/pooling.h:66-76: ggout[window] = ggx at the ArgMax position of x in that window (a position in
 * the padding gives the lowest value, as the native Im2Col fills it); ggx has x's shape, ggout the pooled shape. */
int hipcx_max_pool_grad_grad(const hipcx_array* x, const hipcx_array* ggx, const int64_t* kernel_size, const int64_t* stride,
                             const int64_t* pad, int cover_all, const hipcx_array* ggout, void* stream);
int hipcx_average_pool_grad(const hipcx_array* gout, const int64_t* kernel_size, const int64_t* stride, const int64_t* pad, int pad_mode,
                            const hipcx_array* gx, void* stream);

/* ---- indexing: TakeKernel CX/kernels/indexing.h:17 ----
 * Out-of-range indices in the DEFAULT and RAISE modes (the native backend throws IndexError from the kernel call,
 * CX/native/native_device/indexing.cc:68-74):
 *   `error_flag` not NULL: a device int32 the caller zeroes before the call; the kernel stores 1 there when an index is out of
 *       range; the caller reads it back and throws (one host wait per call).
 *   `error_flag` NULL, mode DEFAULT (what the routine passes for mode=None): the kernel records {index, extent, axis} in a sticky
 *       per-device record and the next hipcx_synchronize / hipcx_memcpy_to_host on the device -- the calls that wait for the
 *       device, and the only way results reach the host (CX/cuda/cuda_device/memory.cc:94-122) -- returns HIPCX_INDEX_ERROR
 *       with the reference's message and clears the record.  The take call itself never waits and can be captured into a graph.
 *       (A wait on a stream that the faulty kernel is not ordered before may miss it; the next wait reports it.)
 *   `error_flag` NULL, mode RAISE: refused with HIPCX_CHAINERX_ERROR.
 * WRAP and CLIP never report.  No mode ever reads or writes out of bounds: a faulty index is treated as 0 after it was reported.
 * Nothing is written to `out` by a call that is refused. */
int hipcx_take(const hipcx_array* a, const hipcx_array* indices, int8_t axis, const hipcx_array* out, int mode, int32_t* error_flag,
               void* stream);

/* AddAtKernel indexing.h:12 -- out = a, then out[l..., indices[i...], r...] += b[l..., i..., r...] along `axis`, the indices
 * walked in C order so that repeated indices accumulate in the reference's order (native/native_device/indexing.cc:107-190);
 * bounds modes and error_flag as for hipcx_take.  a, b and out share a dtype. */
int hipcx_add_at(const hipcx_array* a, const hipcx_array* indices, int8_t axis, const hipcx_array* b, const hipcx_array* out, int mode,
                 int32_t* error_flag, void* stream);

/* Creation kernels (native/native_device/fill.cc): IdentityKernel creation.h:24, EyeKernel(k) :31, TriKernel(k) :50 fill a
 * C-contiguous 2-D out with the 0/1 pattern; LinspaceKernel :43 writes (start*(n-1-i) + stop*i)/(n-1) evaluated in double;
 * DiagflatKernel :38 places the 1-D v on the k-th diagonal of a zeroed square out. */
int hipcx_identity(const hipcx_array* out, void* stream);
int hipcx_eye(int64_t k, const hipcx_array* out, void* stream);
int hipcx_tri(int64_t k, const hipcx_array* out, void* stream);
int hipcx_linspace(double start, double stop, const hipcx_array* out, void* stream);
int hipcx_diagflat(const hipcx_array* v, int64_t k, const hipcx_array* out, void* stream);

/* CumsumKernel reduction.h:23 -- inclusive prefix sums along `axis`, added serially in index order as native::Scan does
 * (CX/native/reduce.h:98-113): float results carry the native backend's bits.  out: a's float dtype, int64 for bool and
 * integer inputs (CX/routines/reduction.cc:115-127); float16 accumulates in float and rounds every prefix. */
int hipcx_cumsum(const hipcx_array* a, int8_t axis, const hipcx_array* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HIPCX_H_ */

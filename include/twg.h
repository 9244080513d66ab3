/*
 * twg.h - C ABI of libtwg_hip.so, the gfx950 (MI355X) kernel library that sits
 * underneath the "webgpu" PrivateUse1 backend of torch_webgpu.
 *
 * The reference (jmaczan/torch-webgpu) has no FFI of its own: its op layer talks
 * to Google Dawn through C++ objects.  Every entry point below therefore cites the
 * reference C++ function whose work it takes over.  No torch and no HIP types
 * cross this line: plain pointers, sizes and POD structs only, so the same
 * library is driven from the torch extension (csrc/torch), from ctypes, or from
 * any other host language with a C FFI.
 *
 * Conventions
 *  - Every function returns 0 on success.  A positive value is a hipError_t, a
 *    negative value is one of the TWG_E_* codes; twg_error_string() decodes both.
 *  - Device pointers are real device addresses, already advanced by the tensor's
 *    storage offset (the reference instead passes whole buffers plus element
 *    offsets: csrc/ops/binary.h:101-103, csrc/ops/unary.h:82-83).
 *  - `stream` is a hipStream_t passed as an opaque pointer; NULL selects the
 *    library's own in-order stream (the stand-in for the reference's single Dawn
 *    queue, csrc/core/webgpu_context.cpp:44).  Launches are asynchronous.
 *  - Iteration geometry travels in twg_iter_t, the 64-bit widening of the
 *    reference's uniform `Params` blocks (csrc/ops/binary.h:108-124,
 *    csrc/ops/unary.h:88-101).  Dimension 0 is the fastest-moving one, which is
 *    the order at::TensorIterator presents.  Strides are in elements, may be 0
 *    (broadcast) and may be negative.  The elementwise entry points visit the
 *    dimensions by ascending output stride whatever order they come in (the result
 *    does not depend on it); for masked_select the order of the dimensions is the
 *    order of the output.
 */
#ifndef TWG_H_
#define TWG_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TWG_MAX_DIMS 8 /* csrc/ops/binary.h:105 (MAX_DIMS) */

/* negative (library) error codes */
#define TWG_E_INVALID_ARG (-1)   /* bad ndim / negative extent / numel mismatch / null pointer */
#define TWG_E_UNSUPPORTED (-2)   /* valid request this build has no kernel for */
#define TWG_E_SCRATCH_SMALL (-3) /* masked_select scratch buffer too small */
#define TWG_E_OVERLAP (-4)       /* reserved */
#define TWG_E_TOO_LARGE (-5)     /* more elements than an entry point with a fixed limit takes */
#define TWG_E_BUSY (-6)          /* twg_masked_select_f32_static: its array is in use on another stream */
#define TWG_E_WAIT_ABANDONED (-7) /* masked_select: a tile waited for a status word nobody published */

typedef struct ihipStream_t *twg_stream_t; /* == hipStream_t */
typedef struct ihipEvent_t *twg_event_t;   /* == hipEvent_t  */

/* Operand slots of twg_iter_t.stride */
#define TWG_OUT 0
#define TWG_A 1
#define TWG_B 2

typedef struct twg_iter {
  int32_t ndim;  /* 0..TWG_MAX_DIMS; 0 means a single element */
  int32_t reserved;
  int64_t numel; /* product of shape[0..ndim) */
  int64_t shape[TWG_MAX_DIMS];
  int64_t stride[3][TWG_MAX_DIMS]; /* [TWG_OUT|TWG_A|TWG_B][dim], elements */
} twg_iter_t;

/* Unary functor selector: the reference's UnaryOp enum (csrc/ops/unary.h:20-26)
 * with GeLU split into the formula the reference actually evaluates (tanh,
 * csrc/ops/unary.cpp:93-95) and the exact erf form ATen means by
 * approximate='none'. */
enum twg_unary_op {
  TWG_UNARY_COPY = 0,      /* csrc/ops/unary.cpp:88-89 */
  TWG_UNARY_RELU = 1,      /* csrc/ops/unary.cpp:90-92 */
  TWG_UNARY_GELU_ERF = 2,  /* aten gelu(approximate='none') */
  TWG_UNARY_GELU_TANH = 3, /* csrc/ops/unary.cpp:93-95 */
  TWG_UNARY_SILU = 4,      /* csrc/ops/unary.cpp:96-98 */
  TWG_UNARY_ABS = 5        /* |x|; a boxed CPU fallback in the reference, csrc/bindings.cpp:35 */
};

/* ---------------------------------------------------------------- runtime */

/* Bind device 0, create the library stream.  Idempotent, thread safe.  Replaces
 * the lazy Dawn instance/adapter/device/queue singleton
 * (csrc/core/webgpu_context.cpp:9-68); unlike it, failure is returned, never
 * exit(1). */
int twg_init(void);
/* 1 once twg_init has succeeded (python/torch_webgpu/webgpu/__init__.py:4-5). */
int twg_is_initialized(void);
const char *twg_error_string(int code);
/* Name, compute-unit count and memory of the bound device (diagnostics, bench). */
int twg_device_info(char *name, size_t name_cap, int32_t *compute_units,
                    int64_t *total_mem_bytes);
/* The library's in-order stream. */
twg_stream_t twg_default_stream(void);
int twg_stream_sync(twg_stream_t stream);
int twg_device_sync(void);

/* Event timing on a given stream (used by the benchmark for the roofline
 * figures; no reference counterpart: the reference has no timing code). */
int twg_event_create(twg_event_t *ev);
int twg_event_destroy(twg_event_t ev);
int twg_event_record(twg_event_t ev, twg_stream_t stream);
int twg_event_sync(twg_event_t ev);
int twg_event_elapsed_ms(float *ms, twg_event_t start, twg_event_t stop);

/* -------------------------------------------------------------- allocator */

/* Caching device allocator.  Replaces WebGPUAllocator::allocate /
 * WebGPUCachingHostDeleter (csrc/core/webgpu_allocator.cpp:10-29), which create
 * and destroy one Dawn buffer per tensor.  Blocks are rounded up (512 B below
 * 1 MiB, 2 MiB above), kept on per-size free lists when freed and handed out
 * again without touching hipMalloc.  A block belongs to the library's in-order
 * stream: freed, it is reusable at once, because every later launch on that
 * stream runs after the work that still uses it (the reference gets the same
 * from Dawn's single queue).  n == 0 yields *p == NULL and success
 * (csrc/core/webgpu_allocator.cpp:33-38). */
int twg_malloc(void **p, size_t n);
int twg_free(void *p);
/* Tell the allocator that the block containing p is used by work queued on
 * `stream`, a stream of the caller's (every entry point takes one).  When such a
 * block is freed it is neither reused nor released until that work has finished:
 * twg_free records an event on each recorded stream and the block waits for them
 * (bytes_pending in twg_mem_stats).  Without this call a block used on another
 * stream than the library's must not be freed before the caller has synchronised
 * that stream.  If the stream is being captured into a graph at the time of the
 * free, the block is held until twg_empty_cache.  No counterpart in the reference
 * (one queue).  NULL or the library's stream: nothing to do, returns 0. */
int twg_record_stream(const void *p, twg_stream_t stream);
/* Return every cached (unused) block to the driver; waits for the library's
 * stream and for the recorded streams of freed blocks first. */
int twg_empty_cache(void);

typedef struct twg_mem_stats {
  int64_t bytes_in_use;   /* handed out, rounded sizes */
  int64_t bytes_cached;   /* sitting on free lists */
  int64_t n_device_mallocs; /* hipMalloc calls so far */
  int64_t n_cache_hits;   /* twg_malloc calls served from a free list */
  int64_t n_allocs;       /* twg_malloc calls with n > 0 */
  int64_t bytes_pending;  /* freed, waiting for work on a recorded stream */
} twg_mem_stats_t;
int twg_mem_stats(twg_mem_stats_t *out);

/* ----------------------------------------------------------------- copies */

/* Host -> device.  Replaces queue.WriteBuffer in copy_ (csrc/ops/copy.cpp:74-92).
 * Pageable host memory is staged through a ring of pinned memory, in pieces sized
 * to the copy, so the CPU memcpy of piece k+1 overlaps the DMA of piece k; the host
 * range may be reused as soon as the call returns. */
int twg_memcpy_h2d(void *dst_dev, const void *src_host, size_t nbytes, twg_stream_t stream);
/* Device -> host, blocking: on return the bytes are in dst_host.  Replaces the
 * staging-buffer + MapAsync + WaitAny + memcpy sequence of cpu_copy_with_webgpu
 * (csrc/ops/copy.cpp:33-56). */
int twg_memcpy_d2h(void *dst_host, const void *src_dev, size_t nbytes, twg_stream_t stream);
/* Side effects of the two host copies worth knowing: destinations of 8 MiB and more get
 * madvise(MADV_HUGEPAGE) on their 2 MiB-aligned interior (a freshly allocated destination
 * otherwise faults 4 KiB at a time, 13 GB/s instead of 30-39; set TWG_NO_HUGEPAGE_HINT in
 * the environment to leave the caller's mapping alone), and copies of 8 MiB and more are
 * shared with three helper threads that the first such copy creates and that sleep
 * otherwise.  A process forked after twg_init must not use the library (the helper threads
 * and the locks do not come along). */
/* Device -> device, contiguous.  Replaces CopyBufferToBuffer in copy_
 * (csrc/ops/copy.cpp:95-122).  Ranges must not overlap.  Copies of 128 MiB and more
 * between 16-byte aligned addresses run the library's streaming copy kernel (1 GiB in
 * 0.32 ms against 0.41 ms for hipMemcpyAsync); smaller or misaligned ones go to
 * hipMemcpyAsync, which is as fast or faster there. */
int twg_memcpy_d2d(void *dst_dev, const void *src_dev, size_t nbytes, twg_stream_t stream);
/* Fill nbytes with a byte value (kernel, not hipMemset, so it is safe to record
 * into a HIP graph). */
int twg_fill_bytes(void *dst_dev, int value, size_t nbytes, twg_stream_t stream);

/* ------------------------------------------------------------ elementwise */

/* out = a + alpha * b in binary32, product and sum rounded separately.
 * Replaces binary_kernel<BinaryOp::Add> and its WGSL
 * (csrc/ops/binary.h:29-215, csrc/ops/binary.cpp:55-98), as reached from
 * add_out_webgpu (csrc/ops/arithmetic.cpp:24-43).  Full broadcasting and
 * arbitrary strides through `it`. */
int twg_add_f32(float *out, const float *a, const float *b, float alpha,
                const twg_iter_t *it, twg_stream_t stream);
/* out = a + alpha * s for a host scalar s.  The reference lets a CPU scalar
 * tensor into the iterator and then misreads its storage as a device buffer
 * (csrc/ops/arithmetic.cpp:37, csrc/ops/binary.h:95); here the scalar is passed
 * by value.  Uses it->stride[TWG_OUT] and it->stride[TWG_A]. */
int twg_add_scalar_f32(float *out, const float *a, float s, float alpha,
                       const twg_iter_t *it, twg_stream_t stream);
/* out = a * b.  Replaces binary_kernel<BinaryOp::Mul> (csrc/ops/binary.cpp:99-101),
 * whose registration the reference leaves commented out
 * (csrc/ops/arithmetic.cpp:45-63,396). */
int twg_mul_f32(float *out, const float *a, const float *b, const twg_iter_t *it,
                twg_stream_t stream);
int twg_mul_scalar_f32(float *out, const float *a, float s, const twg_iter_t *it,
                       twg_stream_t stream);
/* out = max(0, a + b).  Replaces binary_kernel<BinaryOp::FusedAddRelu>
 * (csrc/ops/binary.cpp:102-104, csrc/ops/webgpu_ops.cpp:26-44). */
int twg_add_relu_f32(float *out, const float *a, const float *b, const twg_iter_t *it,
                     twg_stream_t stream);

/* out = f(in), f from enum twg_unary_op.  Replaces unary_kernel<Op> and its WGSL
 * (csrc/ops/unary.h:30-181, csrc/ops/unary.cpp:49-98), as reached from relu/
 * gelu/silu(_out) (csrc/ops/activation_functions.cpp:27-114) and from the
 * strided device-to-device branch of copy_ (csrc/ops/copy.cpp:123-134).  Uses
 * it->stride[TWG_OUT] and it->stride[TWG_A]. */
int twg_unary_f32(int op, float *out, const float *in, const twg_iter_t *it,
                  twg_stream_t stream);
/* Strided gather/scatter copy for 1-, 2-, 4- and 8-byte elements (bool masks
 * are 1 byte).  Same role as TWG_UNARY_COPY for non-float dtypes, which the
 * reference rejects (csrc/ops/unary.h:34). */
int twg_copy_strided(void *out, const void *in, int32_t elem_size,
                     const twg_iter_t *it, twg_stream_t stream);

/* Element types twg_cast converts between (torch.bool is one byte holding 0 or 1). */
enum twg_dtype {
  TWG_DT_BOOL = 0,
  TWG_DT_U8 = 1,
  TWG_DT_I32 = 2,
  TWG_DT_I64 = 3,
  TWG_DT_F16 = 4,
  TWG_DT_BF16 = 5,
  TWG_DT_F32 = 6,
  TWG_DT_F64 = 7,
  TWG_DT_I8 = 8,
  TWG_DT_I16 = 9
};
/* out[i] = (out_dtype) in[i] with ATen's CPU conversion rules (anything -> bool is
 * x != 0, float -> integer truncates, narrowing floats round to nearest even), any
 * strides.  No counterpart in the reference, whose copy_ moves bytes of one dtype
 * (csrc/ops/copy.cpp:95-134) and whose strided copy is fp32 only (unary.h:34); it is
 * what keeps `mask.float()`, `x.to(torch.int64)` and copies between host and device
 * tensors of different dtypes off the CPU.  Direct pairs: everything <-> TWG_DT_F32,
 * {BOOL, U8, I8, I16, I32, F64} <-> TWG_DT_I64, F64 -> BOOL; any other pair returns
 * TWG_E_UNSUPPORTED and is composed exactly from two of these by the caller (through
 * I64 between integer types and between F64 and integers, through F32 otherwise). */
int twg_cast(void *out, int32_t out_dtype, const void *in, int32_t in_dtype,
             const twg_iter_t *it, twg_stream_t stream);

/* out[i] = (a[i] == b[i]) as a 0/1 byte, IEEE semantics (NaN != NaN, -0 == +0).
 * Replaces the boxed CPU fallback registered for eq.Tensor / eq.Tensor_out
 * (csrc/bindings.cpp:38-39). */
int twg_eq_f32(uint8_t *out, const float *a, const float *b, const twg_iter_t *it,
               twg_stream_t stream);
/* out[i] = (a[i] != s).  Replaces the fallback for ne.Scalar / ne.Scalar_out
 * (csrc/bindings.cpp:36-37). */
int twg_ne_scalar_f32(uint8_t *out, const float *a, float s, const twg_iter_t *it,
                      twg_stream_t stream);
/* out[i] = a[i] & b[i] on 0/1 bytes.  Replaces the fallback for
 * bitwise_and.Tensor / bitwise_and.Tensor_out (csrc/bindings.cpp:40-41) for bool
 * (and uint8/int8) tensors. */
int twg_and_u8(uint8_t *out, const uint8_t *a, const uint8_t *b, const twg_iter_t *it,
               twg_stream_t stream);

/* ---------------------------------------------------------- masked_select */

/* Bytes of device scratch twg_masked_select_f32 needs for `numel` elements. */
size_t twg_masked_select_scratch_bytes(int64_t numel);
/* Single-pass ordered stream compaction: writes src[i] for every i with
 * mask[i] != 0, in increasing logical index i, to out[0..K) and K to *d_count
 * (device memory).  `out` must hold it->numel floats.  Replaces the boxed CPU
 * fallback registered for masked_select (csrc/bindings.cpp:42).  `it` describes
 * the broadcast logical shape: stride[TWG_A] addresses src, stride[TWG_B]
 * addresses mask, stride[TWG_OUT] is ignored; dim 0 fastest, so logical index i
 * is the row-major index of the broadcast shape reversed.  Asynchronous: read
 * *d_count with twg_memcpy_d2h (or call twg_masked_select_count, below).
 * A source or mask that is not dense in logical order (or is off its alignment: four
 * elements for the source, 4 bytes for the mask) is first copied dense on the device, from
 * 2^16 elements on, into a block of the library's allocator (numel elements for the source,
 * numel bytes for the mask; returned to the allocator before the call returns, reusable once
 * the stream has passed it); if the allocator has no room, or the stream is being captured,
 * such operands are gathered element by element instead, 3-5 times slower.
 * The scratch must belong to this call alone until its kernels have finished: it holds a
 * ticket counter and one status word per tile.  No wait inside the kernels is unbounded:
 * if the scratch is shared by two launches in flight, or overwritten under a running one,
 * a tile that has polled for a predecessor's word about a second gives up, it and every
 * tile whose output position rests on it write nothing, *d_count receives -1 instead of a
 * count when the last tile is among them, and the second 32-bit word of the scratch is set
 * to 1 (the first is the ticket counter; both are cleared by every launch of more than one
 * tile).  All workgroups exit either way. */
int twg_masked_select_f32(float *out, int64_t *d_count, const float *src,
                          const uint8_t *mask, const twg_iter_t *it, void *scratch,
                          size_t scratch_bytes, twg_stream_t stream);

/* twg_masked_select_f32 for callers that cannot allocate device memory (code under HIP
 * graph capture, serving loops with a fixed memory plan, harnesses that forbid hipMalloc):
 * same kernels, same results, but the tickets and status words live in a device array
 * that is part of the library's code object (2 MiB + 384 B per GPU, held until the process
 * ends) instead of a caller-provided scratch buffer.  It has no counterpart in the
 * reference.  The call allocates nothing and frees nothing once the library is
 * initialised (call twg_init() first: initialisation itself creates the stream).
 * it->numel may be at most TWG_MS_STATIC_MAX_NUMEL; larger inputs return TWG_E_TOO_LARGE.
 * All calls on one GPU share the one array.  Calls on one stream are ordered; nothing is
 * cleared between them (each launch marks its status words with its own epoch and counts
 * its tiles from where the ticket counter stands; the array is cleared before the first
 * call, when the 2^20 epochs run out, after a launch that failed, and by every call from
 * the first one under graph capture on).  A call on another stream while the previous call's kernels are still
 * running is refused with TWG_E_BUSY (the library records an event behind every call and
 * queries it; the event is created by twg_init).  Under graph capture that check cannot be
 * made and is skipped: a capturing caller orders its own uses of the array. */
#define TWG_MS_STATIC_MAX_NUMEL (INT64_C(1) << 30)
int twg_masked_select_f32_static(float *out, int64_t *d_count, const float *src,
                                 const uint8_t *mask, const twg_iter_t *it,
                                 twg_stream_t stream);

/* Test hook, no counterpart in the reference: twg_masked_select_f32 with the ticket counter
 * started at first_ticket (0..255) instead of 0 and the look-back's polling limit set to
 * max_poll_rounds (0 = the library's own).  Tiles below first_ticket are then never
 * compacted or published, so with first_ticket >= 1 on an input of two or more tiles every
 * look-back runs into the limit by construction: the way to exercise the give-up path of the
 * bounded wait with every workgroup still exiting normally.  Expect *d_count == -1 and the
 * scratch's error word set; `out` is not written by the tiles that gave up. */
int twg_masked_select_f32_wait_probe(float *out, int64_t *d_count, const float *src,
                                     const uint8_t *mask, const twg_iter_t *it, void *scratch,
                                     size_t scratch_bytes, uint32_t first_ticket,
                                     uint32_t max_poll_rounds, twg_stream_t stream);

/* The same compaction for elements of `elem_size` = 1, 2, 4 or 8 bytes (moved without
 * being looked at, so any dtype of that size; the CPU fallback the reference registers,
 * csrc/bindings.cpp:42, takes every dtype), with K delivered to the host: *count_host
 * is valid when the call returns, while the writes to `out` are only ordered on `stream`
 * like any other launch (work queued afterwards sees them).  The kernel stores K into
 * pinned host memory the moment the last tile knows it and the host polls that word,
 * which saves the separate read-back of twg_masked_select_f32 + twg_memcpy_d2h (one
 * launch and one wait per call; returns TWG_E_WAIT_ABANDONED where twg_masked_select_f32
 * would have delivered -1).  This is what the masked_select registration calls:
 * it needs K to shape the result.  `out` and `src` must be aligned to elem_size; every
 * element size takes the kernels of twg_masked_select_f32, instantiated for it (dense
 * operands with `src` aligned to four elements, 16 bytes for 8-byte elements; anything
 * else is copied dense first, see twg_masked_select_f32).
 * scratch == NULL with scratch_bytes == 0 selects the array the library keeps for
 * twg_masked_select_f32_static, with that entry point's limit (TWG_E_TOO_LARGE beyond
 * TWG_MS_STATIC_MAX_NUMEL elements) and its rule for streams (TWG_E_BUSY); the launch that
 * clears a caller's scratch then falls away (13 -> 9 us per call up to 2^19 elements). */
int twg_masked_select_count(void *out, int64_t *count_host, const void *src,
                            int32_t elem_size, const uint8_t *mask, const twg_iter_t *it,
                            void *scratch, size_t scratch_bytes, twg_stream_t stream);

/* ------------------------------------------- compare / and for every dtype */

/* out[i] = (a[i] == b[i]) as a 0/1 byte for two operands of one dtype (enum
 * twg_dtype), ATen's CPU semantics, which are what the reference's fallback gives
 * (csrc/bindings.cpp:38-39): IEEE for floating types, exact for integers.
 * TWG_DT_F32 runs the kernel of twg_eq_f32. */
int twg_eq(uint8_t *out, const void *a, const void *b, int32_t dtype, const twg_iter_t *it,
           twg_stream_t stream);
/* out[i] = (a[i] != s) for an operand of `dtype` (csrc/bindings.cpp:36-37).  The scalar
 * comes twice: s_f is used for floating dtypes (rounded to the dtype first, as ATen
 * does), s_i for integral ones and bool. */
int twg_ne_scalar(uint8_t *out, const void *a, int32_t dtype, double s_f, int64_t s_i,
                  const twg_iter_t *it, twg_stream_t stream);
/* out[i] = |a[i]| for every dtype but bool (csrc/bindings.cpp:35), out of a's dtype.
 * TWG_DT_F32 runs twg_unary_f32(TWG_UNARY_ABS). */
int twg_abs(void *out, const void *a, int32_t dtype, const twg_iter_t *it, twg_stream_t stream);
/* out[i] = a[i] & b[i] on integers of elem_size = 1, 2, 4 or 8 bytes
 * (csrc/bindings.cpp:40-41). */
int twg_and(void *out, const void *a, const void *b, int32_t elem_size, const twg_iter_t *it,
            twg_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* TWG_H_ */

/*
 * tannic_hip.h — C ABI of the gfx950 (MI355X) device backend for Tannic.
 *
 * Every entry point takes plain C structs by pointer, sizes and a stream
 * handle by value, and returns an `int` status.  No HIP, C++ or torch type
 * appears in a signature.  The structs below restate, field for field, the
 * runtime structs of the reference so that a `tensor_t*` produced by its
 * front end can be handed over unchanged:
 *
 *   tannic_tensor_t   <-> tensor_t      include/tannic/runtime/tensor.h:64-73
 *   tannic_shape_t    <-> shape_t       include/tannic/runtime/tensor.h:50-55
 *   tannic_strides_t  <-> strides_t     include/tannic/runtime/tensor.h:57-62
 *   tannic_scalar_t   <-> scalar_t      include/tannic/runtime/tensor.h:45-48
 *   tannic_stream_t   <-> stream_t      include/tannic/runtime/streams.h:32-34
 *   tannic_device_t   <-> device_t      include/tannic/runtime/resources.h:50-52
 *   tannic_environment_t <-> environment_t  include/tannic/runtime/resources.h:54-60
 *   enum values       <-> types.h:29-44, status.h:26-32, tensor.h:39-43,
 *                         resources.h:35-43
 *
 * Conventions shared by all kernels entry points:
 *   - descriptors are borrowed for the duration of the call only;
 *   - `address` already includes the view offset; strides are in ELEMENTS and
 *     may be 0 (expanded dims) or permuted; boolean tensors are bit-packed,
 *     LSB first, (size+7)/8 bytes; complex tensors are interleaved (re,im);
 *   - the destination is pre-allocated by the caller on the same device, with
 *     the shape and the dtype of the call's result: descriptors that do not
 *     fit each other, or that have elements but a null address, are refused
 *     with TANNIC_ERROR before anything is launched (the reference's kernels
 *     take them on trust);
 *   - work is enqueued on `stream` and the call returns without waiting;
 *   - nothing is thrown across this boundary: the status says what happened
 *     and tannic_hip_last_error() holds a message for TANNIC_ERROR.
 */
#ifndef TANNIC_HIP_H
#define TANNIC_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TANNIC_DIMENSIONS 8

enum tannic_type {
    TANNIC_ANY = 0,
    TANNIC_BOOLEAN = 1,
    TANNIC_INT8 = 2,
    TANNIC_INT16 = 3,
    TANNIC_INT32 = 4,
    TANNIC_INT64 = 5,
    TANNIC_FLOAT16 = 6,
    TANNIC_BFLOAT16 = 7,
    TANNIC_FLOAT32 = 8,
    TANNIC_FLOAT64 = 9,
    TANNIC_COMPLEX64 = 10,
    TANNIC_COMPLEX128 = 11,
    TANNIC_UNKNOWN = 12,
    TANNIC_TYPES = 13
};

enum tannic_status {
    TANNIC_SUCCESS = 0,
    TANNIC_ERROR = 1,
    TANNIC_UNSUPPORTED_DTYPE = 2,
    TANNIC_NULL_ALLOCATOR = 3,
    TANNIC_INCOMPATIBLE_DEVICES = 4
};

enum tannic_layout {
    TANNIC_SINGLETON = 0,
    TANNIC_CONTIGUOUS = 1,
    TANNIC_STRIDED = 2
};

enum tannic_environment_kind {
    TANNIC_HOST = 0,
    TANNIC_DEVICE = 1
};

enum tannic_host_traits {
    TANNIC_PAGEABLE = 1,
    TANNIC_PINNED = 2
};

typedef struct tannic_host_t {
    enum tannic_host_traits traits;
} tannic_host_t;

typedef struct tannic_device_t {
    int id;
} tannic_device_t;

typedef struct tannic_environment_t {
    enum tannic_environment_kind kind;
    union {
        tannic_host_t host;
        tannic_device_t device;
    } resource;
} tannic_environment_t;

typedef struct tannic_scalar_t {
    const void* address; /* HOST memory holding one value of `dtype` */
    enum tannic_type dtype;
} tannic_scalar_t;

typedef struct tannic_shape_t {
    union {
        const size_t* address;
        size_t sizes[TANNIC_DIMENSIONS];
    };
} tannic_shape_t;

typedef struct tannic_strides_t {
    union {
        const int64_t* address;
        int64_t sizes[TANNIC_DIMENSIONS];
    };
} tannic_strides_t;

typedef struct tannic_tensor_t {
    void* address;
    uint8_t rank;
    tannic_shape_t shape;
    tannic_strides_t strides;
    enum tannic_type dtype;
    tannic_environment_t environment;
    size_t size;
    enum tannic_layout layout;
} tannic_tensor_t;

typedef struct tannic_stream_t {
    uintptr_t address; /* carries the hipStream_t */
} tannic_stream_t;

#ifdef __cplusplus
static_assert(sizeof(tannic_tensor_t) == 176, "tensor_t layout");
static_assert(offsetof(tannic_tensor_t, rank) == 8, "tensor_t layout");
static_assert(offsetof(tannic_tensor_t, shape) == 16, "tensor_t layout");
static_assert(offsetof(tannic_tensor_t, strides) == 80, "tensor_t layout");
static_assert(offsetof(tannic_tensor_t, dtype) == 144, "tensor_t layout");
static_assert(offsetof(tannic_tensor_t, environment) == 148, "tensor_t layout");
static_assert(offsetof(tannic_tensor_t, size) == 160, "tensor_t layout");
static_assert(offsetof(tannic_tensor_t, layout) == 168, "tensor_t layout");
static_assert(sizeof(tannic_scalar_t) == 16 && offsetof(tannic_scalar_t, dtype) == 8, "scalar_t layout");
static_assert(sizeof(tannic_environment_t) == 8 && offsetof(tannic_environment_t, resource) == 4, "environment_t layout");
static_assert(sizeof(tannic_stream_t) == 8, "stream_t layout");
#endif

/* ------------------------------------------------------------------ *
 * Library state
 * ------------------------------------------------------------------ */

/* Message of the most recent TANNIC_ERROR / failed runtime call on this thread
 * ("" if none).  The pointer stays valid until the next failing call. */
const char* tannic_hip_last_error(void);

/* Name of the GPU architecture the kernels were compiled for ("gfx950"). */
const char* tannic_hip_arch(void);

/* ------------------------------------------------------------------ *
 * Devices, memory, streams          replaces src/cuda/mem.cuh:10-18,
 *                                   src/cuda/streams.cuh:8-26
 * ------------------------------------------------------------------ */

/* cuda::getDeviceCount            src/cuda/mem.cu:9-13   (-1 on runtime failure) */
int tannic_hip_get_device_count(void);
/* cuda::setDevice                 src/cuda/mem.cu:15-17 */
int tannic_hip_set_device(int id);
/* cuda::allocate                  src/cuda/mem.cu:19-27  stream-ordered, NULL on failure */
void* tannic_hip_allocate(const tannic_device_t* device, size_t nbytes);
/* cuda::deallocate                src/cuda/mem.cu:29-36  always returns NULL */
void* tannic_hip_deallocate(const tannic_device_t* device, void* address);
/* cuda::copyFromHost              src/cuda/mem.cu:38-44 */
int tannic_hip_copy_from_host(const tannic_device_t* device, const void* host, void* dev, size_t nbytes);
/* cuda::copyDeviceToHost          src/cuda/mem.cu:46-52  (host memory is valid on return) */
int tannic_hip_copy_device_to_host(const tannic_device_t* device, const void* dev, void* host, size_t nbytes);
/* cuda::compareFromHost           src/cuda/mem.cu:54-65  1 equal, 0 different, -1 failure */
int tannic_hip_compare_from_host(const tannic_device_t* device, const void* host, const void* dev, size_t nbytes);
/* cuda::copy                      src/cuda/mem.cu:67-93  H2D / D2H / D2D chosen by the environments */
int tannic_hip_copy(const tannic_tensor_t* src, tannic_tensor_t* dst, size_t nbytes, tannic_stream_t stream);
/* cuda::Streams::pop / put        src/cuda/streams.cu:23-38, src/bindings.cpp:22-42 */
tannic_stream_t tannic_hip_pop_stream(const tannic_device_t* device);
void tannic_hip_put_stream(const tannic_device_t* device, tannic_stream_t stream);
/* Block the host until `stream` / the current device is idle (the reference
 * reaches these only through compareFromHost/allclose; exposed for harnesses). */
int tannic_hip_stream_synchronize(tannic_stream_t stream);
int tannic_hip_device_synchronize(void);

/* A sequence of backend calls recorded once and replayed as one HIP graph: for loops whose cost is issuing the
 * calls, not running them (a decoder layer is some sixty short kernels).  No counterpart in the reference, whose
 * front end evaluates every expression where it is written.
 *   graph_begin   starts recording on the stream the device's backend calls use; every call until graph_end is
 *                 recorded instead of run.  One recording may be open at a time.  Calls that wait for the stream
 *                 (copies to pageable host memory, allclose) cannot be recorded: they fail and graph_end reports it.
 *   graph_end     closes the recording and prepares it for launching.
 *   graph_launch  queues one replay on that stream, ordered with the eager calls around it.
 *   graph_destroy waits for the stream and releases the recording.
 * Memory: tensors allocated while recording are written by every replay, at the same addresses.  Their blocks, and the
 * kernels' scratch, belong to the recording until graph_destroy (released earlier, they are reused only inside that
 * recording), so a replay never writes memory that a tensor outside the recording has been given.  Tensors that
 * existed before graph_begin and are read or written by the recorded calls (inputs, weights) must stay allocated for
 * as long as the recording is launched; new input is copied into them before graph_launch. */
void* tannic_hip_graph_begin(const tannic_device_t* device);
int tannic_hip_graph_end(void* recording);
int tannic_hip_graph_launch(void* recording);
void tannic_hip_graph_destroy(void* recording);
/* What the library has done so far, for tests that check more than results (no reference twin): out[0] kernel-scratch
 * acquisitions, out[1] tensor allocations and releases through tannic_hip_allocate / tannic_hip_deallocate, out[2] the
 * number of workgroups that shared K in the last matrix product that shared it. */
void tannic_hip_counters(uint64_t out[3]);
/* The stream a recording captures: a caller that keeps a device's stream to itself checks that it is this one. */
tannic_stream_t tannic_hip_graph_stream(void* recording);

/* Timing events on a stream, for benchmark harnesses (no reference twin). */
void* tannic_hip_event_create(void);
void tannic_hip_event_destroy(void* event);
int tannic_hip_event_record(void* event, tannic_stream_t stream);
/* milliseconds between two recorded events; waits for `stop`; <0 on failure */
float tannic_hip_event_elapsed_ms(void* start, void* stop);

/* Rate probe of the matrix pipe, for benchmark harnesses (no reference twin): `blocks` workgroups of four wavefronts
 * issue nothing but MFMAs, `iterations` x 2^21 multiply-adds per wavefront, on operand values the caller supplies
 * (`operands`: 64 KiB of device memory, 16 x 256 vectors of 16 bytes, read once; `sink`: 1 KiB per block, written
 * once).  shape 0: v_mfma_f32_32x32x16, shape 1: v_mfma_f32_16x16x32, shape 2: v_mfma_f32_16x16x32 with every two
 * consecutive MFMAs on the same accumulator; dtype TANNIC_FLOAT16 or TANNIC_BFLOAT16.
 * What it sustains on given values is the ceiling of a product of such values on this device. */
int tannic_hip_probe_mfma(int shape, int dtype, const void* operands, void* sink, uint32_t blocks, uint32_t iterations, tannic_stream_t stream);

/* ------------------------------------------------------------------ *
 * Unary elementwise                 replaces src/cuda/ops.cuh:11-24
 *                                   (CPU semantics: src/cpu/ops-unary.cpp:202-370)
 * dst is written contiguously in logical order.
 * ------------------------------------------------------------------ */
int tannic_hip_neg(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_repack(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_log(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_exp(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_sqrt(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_rsqrt(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream, float eps);
int tannic_hip_abs(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_sin(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_cos(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_tan(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_sinh(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_cosh(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_tanh(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream);

/* ------------------------------------------------------------------ *
 * Broadcasting binary elementwise   replaces src/cuda/ops.cuh:25-28
 *                                   (CPU semantics: src/cpu/ops-binary.cpp:65-128,434-448)
 * ------------------------------------------------------------------ */
int tannic_hip_add(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_sub(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_mul(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_pow(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream);
/* cuda::scale                       src/cuda/ops.cuh:29 (CPU: src/cpu/ops-scale.cpp:59-122) */
int tannic_hip_scale(const tannic_tensor_t* src, const tannic_scalar_t* scalar, tannic_tensor_t* dst, tannic_stream_t stream);

/* ------------------------------------------------------------------ *
 * Comparisons -> bit-packed boolean.  The reference has a CPU kernel only
 * (src/cpu/cmps.cpp:85-202) and throwing device stubs (src/comparisons.cpp:18-29);
 * these are the device twins of cpu::eq..le.  Both operands must have one
 * dtype (UNSUPPORTED_DTYPE otherwise): cpu::eq..le read the second operand
 * as the first's type, past the end of a narrower one.
 * ------------------------------------------------------------------ */
int tannic_hip_eq(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_ne(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_gt(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_ge(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_lt(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_le(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream);

/* ------------------------------------------------------------------ *
 * Complex construction              replaces src/cuda/complex.cuh:11-12
 *                                   (CPU: src/cpu/complex.cpp:223-229)
 * ------------------------------------------------------------------ */
int tannic_hip_view_as_cartesian(const tannic_tensor_t* re, const tannic_tensor_t* im, tannic_tensor_t* dst, tannic_stream_t stream);
int tannic_hip_view_as_polar(const tannic_tensor_t* rho, const tannic_tensor_t* theta, tannic_tensor_t* dst, tannic_stream_t stream);

/* ------------------------------------------------------------------ *
 * Shape-changing copies     replaces src/cuda/{reps,concat,outer,triang}.cuh
 * ------------------------------------------------------------------ */
/* cuda::repeat(src, dst, axis, reps, stream): every index along `axis` repeated `reps` times in place
 * (dst[.., j*reps + r, ..] = src[.., j, ..]); src strided, dst contiguous (CPU: src/cpu/reps.cpp:18-99) */
int tannic_hip_repeat(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream, int axis, int reps);
/* cuda::concat(a, b, dst, stream, axis): dst = a followed by b along `axis`; same dtype and rank, other extents equal;
 * sources strided, dst contiguous (src/cuda/concat.cuh:11; CPU: src/cpu/concat.cpp:18-129) */
int tannic_hip_concat(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream, int axis);
/* cuda::outer(a, b, dst, stream): dst[i][j] = a[i] * b[j] for vectors a, b, in the type of the CPU path's pair table
 * (src/cuda/outer.cuh:11; CPU: src/cpu/outer.cpp:18-110).  Pairs whose table type differs from the dtype the front end
 * gives the destination (the larger dtype code) return UNSUPPORTED_DTYPE. */
int tannic_hip_outer(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream);
/* cuda::triu / cuda::tril: rank 2; keeps j >= i + k (upper) or j <= i + k (lower) with the sum formed in
 * unsigned 64-bit as the CPU path forms it (src/cpu/triang.cpp:8-22, 24-105); other ranks: UNSUPPORTED_DTYPE */
int tannic_hip_triu(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream, int k);
int tannic_hip_tril(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream, int k);

/* ------------------------------------------------------------------ *
 * Copies and checks                 replaces src/cuda/cpy.cuh:9, src/cuda/val.cuh:11
 * ------------------------------------------------------------------ */
/* cuda::cpy: strided -> strided, size-1 dims broadcast (CPU: src/cpu/cpy.cpp:18-80) */
int tannic_hip_cpy(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream);
/* cuda::allclose: 1 close, 0 not close, -1 unsupported dtype or operands of two dtypes (the
 * reference throws there, src/cuda/val.cu:82-89); waits for the stream (CPU: src/cpu/val.cpp:17-83) */
int tannic_hip_allclose(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_stream_t stream, double rtol, double atol);

/* ------------------------------------------------------------------ *
 * Axis reductions                   replaces src/cuda/argred.cuh:11-14
 *                                   (CPU: src/cpu/argred.cpp:183-347)
 * 16-bit sums/means accumulate in fp32 and round once.
 * ------------------------------------------------------------------ */
int tannic_hip_argsum(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream, uint8_t axis);
int tannic_hip_argmean(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream, uint8_t axis);
int tannic_hip_argmax(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream, uint8_t axis);
int tannic_hip_argmin(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream, uint8_t axis);
/* Value max / min over an axis.  No counterpart in the reference (it has only
 * argmax/argmin, include/tannic/reductions.hpp:101-193).  The largest resp.
 * smallest number of the slice, +0 counting as larger than -0 and NaNs as
 * absent; a slice in which nothing exceeds -inf (+inf, the integer limits)
 * yields its first element, i.e. src[argmax].  dst dtype = src dtype. */
int tannic_hip_max(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream, uint8_t axis);
int tannic_hip_min(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream, uint8_t axis);

/* ------------------------------------------------------------------ *
 * Matrix multiply                   replaces src/cuda/matmul.cuh:12
 *                                   (CPU: src/cpu/matmul.cpp:126-176,254)
 * f16xf16 and bf16xbf16 accumulate in fp32 on MFMA and round once.
 * Operand extents must fit the destination ([.., M, K] x [.., K, N] -> [.., M, N], batch extents 1 or the
 * destination's): TANNIC_ERROR otherwise (the reference takes M, N from the destination and K from `a` on trust).
 * The batch coordinate of an operand with fewer batch dims is multiplied by the stride of the dim it is looked up in;
 * the reference multiplies it by the stride at the left-aligned position (src/cpu/matmul.cpp:107-118).
 * ------------------------------------------------------------------ */
int tannic_hip_gemm(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream);

/* tannic_hip_gemm for callers that must not allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, checks and results as
 * tannic_hip_gemm, bit for bit; the kernels that share K between workgroups (few output tiles, long K) leave their
 * fp32 partial sums in a fixed array of TANNIC_GEMM_NOALLOC_SCRATCH_BYTES that is part of the library's device code
 * (each device the library runs on holds one copy until the process ends) instead of a block from the scratch cache.
 * A product whose partial sums need more returns TANNIC_ERROR with the sizes in tannic_hip_last_error(); such a caller
 * uses tannic_hip_gemm.  Nothing is allocated or freed by this call, on the device or through the runtime.  All calls
 * on one device share the one array: calls that may overlap on a device (different streams, different threads) race;
 * calls on one stream are ordered by it. */
#define TANNIC_GEMM_NOALLOC_SCRATCH_BYTES ((size_t)8 << 20)
int tannic_hip_gemm_noalloc(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream);

/* cuda::conv1d(x, w, y, stream, pad, stride): x[N,C,L], w[O,C,K], y[N,O,(L+2*pad-K)/stride+1]; ERROR on rank != 3 or
 * shape mismatch; same dtype for signal and kernel (src/cuda/conv.cuh:11; CPU: src/cpu/conv1d.cpp:17-125) */
int tannic_hip_conv1d(const tannic_tensor_t* x, const tannic_tensor_t* w, tannic_tensor_t* y, tannic_stream_t stream, size_t pad, size_t stride);
/* ------------------------------------------------------------------ *
 * Convolution                       replaces src/cuda/conv.cuh:12-13
 *                                   (CPU: src/cpu/conv2d.cpp:116-265)
 * NCHW signal, OIHW kernel, cross-correlation, zero padding.
 * ------------------------------------------------------------------ */
int tannic_hip_conv2d(const tannic_tensor_t* signal, const tannic_tensor_t* kernel, tannic_tensor_t* dst,
                      tannic_stream_t stream, const size_t pad[2], const size_t stride[2]);
int tannic_hip_conv2d_biased(const tannic_tensor_t* signal, const tannic_tensor_t* kernel, const tannic_tensor_t* bias,
                             tannic_tensor_t* dst, tannic_stream_t stream, const size_t pad[2], const size_t stride[2]);

/* ------------------------------------------------------------------ *
 * Operators with no counterpart in the reference.  A Tannic program
 * spells them today as chains of the operators above (there is no
 * division, no cast, no softmax in the headers under include/tannic); each is one
 * pass here.  16- and 32-bit types are evaluated in float, float64 in
 * double, and rounded once.
 * ------------------------------------------------------------------ */
/* dst = a / b, broadcasting like mul; the floating pairs of mul's table (src/cpu/ops-binary.cpp:286-360). */
int tannic_hip_div(const tannic_tensor_t* a, const tannic_tensor_t* b, tannic_tensor_t* dst, tannic_stream_t stream);
/* dst[i] = src[i] in dst's dtype, any two real types; dst contiguous with src's shape.  Float to integer truncates
 * toward zero, out-of-range values give the nearest end of the range, NaN gives 0. */
int tannic_hip_cast(const tannic_tensor_t* src, tannic_tensor_t* dst, tannic_stream_t stream);
/* dst = gate / (1 + exp(-gate)) * up, broadcasting like mul; one floating dtype for all three. */
int tannic_hip_swiglu(const tannic_tensor_t* gate, const tannic_tensor_t* up, tannic_tensor_t* dst, tannic_stream_t stream);
/* dst[.., i] = x[.., i] / sqrt(mean_i(x[.., i]^2) + eps) * gain[i] over the last axis; x, dst contiguous. */
int tannic_hip_rms_norm(const tannic_tensor_t* x, const tannic_tensor_t* gain, tannic_tensor_t* dst, tannic_stream_t stream, float eps);
/* softmax over the last axis of s = x * scale + mask; mask is NULL or a contiguous [Q, L] table for x [.., Q, L]. */
int tannic_hip_softmax(const tannic_tensor_t* x, const tannic_tensor_t* mask, tannic_tensor_t* dst, tannic_stream_t stream, float scale);
/* Rotary embedding of x [.., n, d] (any strides) by cos, sin [n, d/2]: the pair (x[2i], x[2i+1]) turns by the
 * angle of position n; dst contiguous. */
int tannic_hip_rope(const tannic_tensor_t* x, const tannic_tensor_t* cos, const tannic_tensor_t* sin, tannic_tensor_t* dst, tannic_stream_t stream);

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* TANNIC_HIP_H */

// The `cuda::` surface Tannic's front end dispatches to, implemented on the
// gfx950 C ABI (include/tannic_hip.h).
//
// The front end reaches its device backend through functions in namespace
// `cuda`, declared in headers it includes as "cuda/<name>.cuh"
// (src/operations.cpp:8, src/functions.cpp:11, src/transformations.cpp:13-17,
// src/convolutions.cpp:6, src/reductions.cpp:8, src/complex.cpp:8,
// src/tensor.cpp:11-12, src/resources.cpp:9, src/bindings.cpp:8-9, src/IO.cpp:14,
// src/comparisons.cpp:11, src/filter.cpp:7).  Putting this directory first on the
// include path and compiling adapter.cpp into the library makes a build with the
// `CUDA` macro use this backend; nothing in the front end changes.
//
// Every function forwards to one tannic_hip_* entry point.  The runtime structs
// are the front end's own (runtime/tensor.h etc.); their layout is asserted to
// equal the C ABI's in adapter.cpp.
#pragma once

#include <cstddef>
#include <cstdint>

#include "runtime/resources.h"
#include "runtime/status.h"
#include "runtime/streams.h"
#include "runtime/tensor.h"
#include "runtime/types.h"

// src/bindings.cpp:26,37 names the stream handle type of the CUDA runtime.  Here
// it is an opaque pointer that carries a hipStream_t; no CUDA header is involved.
typedef void* cudaStream_t;

namespace cuda {

using tannic::device_t;
using tannic::scalar_t;
using tannic::status;
using tannic::stream_t;
using tannic::tensor_t;

// ---- memory (src/cuda/mem.cuh:10-18) ---------------------------------------------
int getDeviceCount();
void setDevice(int id);
void* allocate(const device_t*, size_t nbytes);
void* deallocate(const device_t*, void* address);
void copyFromHost(const device_t*, const void* host, void* dev, size_t nbytes);
bool compareFromHost(const device_t*, const void* host, const void* dev, size_t nbytes);
void copyDeviceToHost(const device_t*, const void* dev, void* host, size_t nbytes);
status copy(const tensor_t* src, tensor_t* dst, size_t nbytes, stream_t stream);

// ---- stream pool (src/cuda/streams.cuh:8-26) ---------------------------------------
class Streams {
   public:
    static Streams& instance();
    cudaStream_t pop(int device);
    void put(int device, cudaStream_t stream);
    Streams(const Streams&) = delete;
    Streams& operator=(const Streams&) = delete;

   private:
    Streams() = default;
};

// ---- elementwise (src/cuda/ops.cuh:11-30) ----------------------------------------------
status repack(const tensor_t*, tensor_t*, stream_t);
status log(const tensor_t*, tensor_t*, stream_t);
status exp(const tensor_t*, tensor_t*, stream_t);
status sqrt(const tensor_t*, tensor_t*, stream_t);
status rsqrt(const tensor_t*, tensor_t*, stream_t, float eps);
status abs(const tensor_t*, tensor_t*, stream_t);
status sin(const tensor_t*, tensor_t*, stream_t);
status cos(const tensor_t*, tensor_t*, stream_t);
status tan(const tensor_t*, tensor_t*, stream_t);
status sinh(const tensor_t*, tensor_t*, stream_t);
status cosh(const tensor_t*, tensor_t*, stream_t);
status tanh(const tensor_t*, tensor_t*, stream_t);
status neg(const tensor_t*, tensor_t*, stream_t);
status add(const tensor_t*, const tensor_t*, tensor_t*, stream_t);
status sub(const tensor_t*, const tensor_t*, tensor_t*, stream_t);
status mul(const tensor_t*, const tensor_t*, tensor_t*, stream_t);
status pow(const tensor_t*, const tensor_t*, tensor_t*, stream_t);
status scale(const tensor_t*, const scalar_t*, tensor_t*, stream_t);

// ---- matmul, convolution, reductions, complex, copies, checks --------------------------
status gemm(const tensor_t* a, const tensor_t* b, tensor_t* dst, stream_t stream);                       // src/cuda/matmul.cuh:12
status conv1d(const tensor_t*, const tensor_t*, tensor_t*, stream_t, const size_t pad, const size_t stride);  // src/cuda/conv.cuh:11 (not built yet)
status conv2d(const tensor_t* signal, const tensor_t* kernel, tensor_t* dst, stream_t, const size_t pad[2], const size_t stride[2]);
status conv2d(const tensor_t* signal, const tensor_t* kernel, const tensor_t* bias, tensor_t* dst, stream_t, const size_t pad[2], const size_t stride[2]);
status argsum(const tensor_t*, tensor_t*, stream_t, uint8_t axis);                                       // src/cuda/argred.cuh:11-14
status argmean(const tensor_t*, tensor_t*, stream_t, uint8_t axis);
status argmax(const tensor_t*, tensor_t*, stream_t, uint8_t axis);
status argmin(const tensor_t*, tensor_t*, stream_t, uint8_t axis);
status view_as_cartesian(const tensor_t*, const tensor_t*, tensor_t*, stream_t);                         // src/cuda/complex.cuh:11-12
status view_as_polar(const tensor_t*, const tensor_t*, tensor_t*, stream_t);
status cpy(const tensor_t* src, tensor_t* dst, stream_t stream);                                         // src/cuda/cpy.cuh:9
bool allclose(const tensor_t*, const tensor_t*, stream_t, double rtol = 1e-5, double atol = 1e-8);       // src/cuda/val.cuh:11

// ---- declared by the front end, not built on this backend yet: UNSUPPORTED_DTYPE ---------
status outer(const tensor_t*, const tensor_t*, tensor_t*, stream_t);          // src/cuda/outer.cuh:11
status repeat(const tensor_t*, tensor_t*, int axis, int reps, stream_t);      // src/cuda/reps.cuh:11
status concat(const tensor_t*, const tensor_t*, tensor_t*, stream_t, int);    // src/cuda/concat.cuh:11
status triu(const tensor_t*, tensor_t*, stream_t, int k = 0);                 // src/cuda/triang.cuh:11-12
status tril(const tensor_t*, tensor_t*, stream_t, int k = 0);

}  // namespace cuda

// Device comparisons and value max/min: the front end defines throwing
// cuda::eq..le itself, unconditionally (src/comparisons.cpp:18-29), so the
// device twins cannot share those names.  A front end that wants them guards its
// stubs with `#ifndef CUDA` and forwards to these.
// Comparisons on the device.  The reference has no device kernels for them: src/comparisons.cpp:18-29 defines these six
// as throwing stubs even in a device build, so a front end that links this backend needs those stubs put under
// `#ifndef CUDA` (frontend.patch next to this header does that).
namespace cuda {
status eq(const tensor_t*, const tensor_t*, tensor_t*, stream_t);
status ne(const tensor_t*, const tensor_t*, tensor_t*, stream_t);
status gt(const tensor_t*, const tensor_t*, tensor_t*, stream_t);
status ge(const tensor_t*, const tensor_t*, tensor_t*, stream_t);
status lt(const tensor_t*, const tensor_t*, tensor_t*, stream_t);
status le(const tensor_t*, const tensor_t*, tensor_t*, stream_t);
}  // namespace cuda

// Operators the reference's front end does not have (tannic_hip_functions.hpp builds expression nodes on them).
namespace tannic_hip {
using tannic::status;
using tannic::stream_t;
using tannic::tensor_t;
status max(const tensor_t*, tensor_t*, stream_t, uint8_t axis);
status min(const tensor_t*, tensor_t*, stream_t, uint8_t axis);
status div(const tensor_t*, const tensor_t*, tensor_t*, stream_t);
status swiglu(const tensor_t* gate, const tensor_t* up, tensor_t*, stream_t);
status cast(const tensor_t*, tensor_t*, stream_t);
status rms_norm(const tensor_t* x, const tensor_t* gain, tensor_t*, stream_t, float eps);
status softmax(const tensor_t* x, const tensor_t* mask_or_null, tensor_t*, stream_t, float scale);
status rope(const tensor_t* x, const tensor_t* cos, const tensor_t* sin, tensor_t*, stream_t);

// A sequence of the front end's evaluations on one device recorded once and replayed as one HIP graph
// (tannic_hip_graph_begin / end / launch / destroy):
//     tannic_hip::Recording r(0);          // device 0's stream is recording
//     Tensor y = f(x);                     // every backend call is recorded, none runs
//     r.end();
//     r.launch();                          // y holds f(x); write new values into x's memory and launch again
// Tensors created between the constructor and end() keep their addresses and are rewritten by every launch; tensors that
// existed before must outlive the launches.  Calls that wait for the device (copies to the host, allclose) throw while
// the recording is open.  Throws std::runtime_error with the library's message when a step fails.
class Recording {
   public:
    explicit Recording(int device = 0);
    Recording(const Recording&) = delete;
    Recording& operator=(const Recording&) = delete;
    ~Recording();
    void end();
    void launch();

   private:
    void* handle_;
};
}  // namespace tannic_hip

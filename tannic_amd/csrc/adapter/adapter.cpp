// Definitions of the `cuda::` functions of tannic_hip_adapter.hpp: one forward
// each to the C ABI.  Error convention of the reference's CUDA backend: runtime
// failures in the void memory functions end the process (src/cuda/exc.cuh:8-16),
// kernels return a status, allclose throws on an unsupported dtype
// (src/cuda/val.cu:87).
#include "tannic_hip_adapter.hpp"

#include <cstdio>
#include <cstdlib>
#include <stdexcept>
#include <string>

#include "../../../include/tannic_hip.h"

using namespace tannic;

static_assert(sizeof(tensor_t) == sizeof(tannic_tensor_t) && offsetof(tensor_t, rank) == offsetof(tannic_tensor_t, rank) &&
              offsetof(tensor_t, shape) == offsetof(tannic_tensor_t, shape) && offsetof(tensor_t, strides) == offsetof(tannic_tensor_t, strides) &&
              offsetof(tensor_t, dtype) == offsetof(tannic_tensor_t, dtype) && offsetof(tensor_t, environment) == offsetof(tannic_tensor_t, environment) &&
              offsetof(tensor_t, size) == offsetof(tannic_tensor_t, size) && offsetof(tensor_t, layout) == offsetof(tannic_tensor_t, layout),
              "tensor_t layout differs from the C ABI");
static_assert(sizeof(scalar_t) == sizeof(tannic_scalar_t) && offsetof(scalar_t, dtype) == offsetof(tannic_scalar_t, dtype), "scalar_t layout");
static_assert(sizeof(stream_t) == sizeof(tannic_stream_t) && sizeof(device_t) == sizeof(tannic_device_t), "stream_t / device_t layout");
static_assert(static_cast<int>(TYPES) == TANNIC_TYPES && static_cast<int>(float16) == TANNIC_FLOAT16 && static_cast<int>(complex128) == TANNIC_COMPLEX128, "type enum");
static_assert(static_cast<int>(SUCCESS) == TANNIC_SUCCESS && static_cast<int>(INCOMPATIBLE_DEVICES) == TANNIC_INCOMPATIBLE_DEVICES, "status enum");
static_assert(static_cast<int>(SINGLETON) == TANNIC_SINGLETON && static_cast<int>(STRIDED) == TANNIC_STRIDED, "layout enum");
static_assert(static_cast<int>(DEVICE) == TANNIC_DEVICE && static_cast<int>(PINNED) == TANNIC_PINNED, "environment enums");

namespace {
inline const tannic_tensor_t* in(const tensor_t* t) { return reinterpret_cast<const tannic_tensor_t*>(t); }
inline tannic_tensor_t* out(tensor_t* t) { return reinterpret_cast<tannic_tensor_t*>(t); }
inline const tannic_device_t* dev(const device_t* d) { return reinterpret_cast<const tannic_device_t*>(d); }
inline tannic_stream_t st(stream_t s) { return tannic_stream_t{s.address}; }
inline status code(int rc) { return static_cast<status>(rc); }
[[noreturn]] void die(const char* what) {
    std::fprintf(stderr, "tannic HIP backend: %s failed: %s\n", what, tannic_hip_last_error());
    std::exit(EXIT_FAILURE);
}
}  // namespace

namespace cuda {

int getDeviceCount() {
    const int n = tannic_hip_get_device_count();
    if (n < 0) die("getDeviceCount");
    return n;
}
void setDevice(int id) { if (tannic_hip_set_device(id) != TANNIC_SUCCESS) die("setDevice"); }
void* allocate(const device_t* d, size_t nbytes) {
    void* p = tannic_hip_allocate(dev(d), nbytes);
    if (!p) die("allocate");
    return p;
}
void* deallocate(const device_t* d, void* address) { return tannic_hip_deallocate(dev(d), address); }
void copyFromHost(const device_t* d, const void* host, void* device, size_t nbytes) {
    if (tannic_hip_copy_from_host(dev(d), host, device, nbytes) != TANNIC_SUCCESS) die("copyFromHost");
}
bool compareFromHost(const device_t* d, const void* host, const void* device, size_t nbytes) {
    const int r = tannic_hip_compare_from_host(dev(d), host, device, nbytes);
    if (r < 0) die("compareFromHost");
    return r == 1;
}
void copyDeviceToHost(const device_t* d, const void* device, void* host, size_t nbytes) {
    if (tannic_hip_copy_device_to_host(dev(d), device, host, nbytes) != TANNIC_SUCCESS) die("copyDeviceToHost");
}
status copy(const tensor_t* src, tensor_t* dst, size_t nbytes, stream_t stream) {
    // Tensor::to(Host) hands over the HOST destination's union as a device id (src/tensor.cpp:114-123);
    // the C ABI's copy only looks at the environment kinds, so that slip is harmless here.
    return code(tannic_hip_copy(in(src), out(dst), nbytes, st(stream)));
}

Streams& Streams::instance() {
    static Streams s;
    return s;
}
cudaStream_t Streams::pop(int device) {
    tannic_device_t d{device};
    return reinterpret_cast<cudaStream_t>(tannic_hip_pop_stream(&d).address);
}
void Streams::put(int device, cudaStream_t stream) {
    tannic_device_t d{device};
    tannic_hip_put_stream(&d, tannic_stream_t{reinterpret_cast<uintptr_t>(stream)});
}

#define TH_UNARY(name) status name(const tensor_t* s, tensor_t* d, stream_t q) { return code(tannic_hip_##name(in(s), out(d), st(q))); }
#define TH_BINARY(name) status name(const tensor_t* a, const tensor_t* b, tensor_t* d, stream_t q) { return code(tannic_hip_##name(in(a), in(b), out(d), st(q))); }
#define TH_REDUCE(name) status name(const tensor_t* s, tensor_t* d, stream_t q, uint8_t axis) { return code(tannic_hip_##name(in(s), out(d), st(q), axis)); }
TH_UNARY(repack) TH_UNARY(log) TH_UNARY(exp) TH_UNARY(sqrt) TH_UNARY(abs) TH_UNARY(sin) TH_UNARY(cos) TH_UNARY(tan)
TH_UNARY(sinh) TH_UNARY(cosh) TH_UNARY(tanh) TH_UNARY(neg) TH_UNARY(cpy)
status rsqrt(const tensor_t* s, tensor_t* d, stream_t q, float eps) { return code(tannic_hip_rsqrt(in(s), out(d), st(q), eps)); }
TH_BINARY(add) TH_BINARY(sub) TH_BINARY(mul) TH_BINARY(pow) TH_BINARY(gemm) TH_BINARY(view_as_cartesian) TH_BINARY(view_as_polar)
status scale(const tensor_t* s, const scalar_t* k, tensor_t* d, stream_t q) {
    return code(tannic_hip_scale(in(s), reinterpret_cast<const tannic_scalar_t*>(k), out(d), st(q)));
}
TH_REDUCE(argsum) TH_REDUCE(argmean) TH_REDUCE(argmax) TH_REDUCE(argmin)
status conv2d(const tensor_t* x, const tensor_t* w, tensor_t* y, stream_t q, const size_t pad[2], const size_t stride[2]) {
    return code(tannic_hip_conv2d(in(x), in(w), out(y), st(q), pad, stride));
}
status conv2d(const tensor_t* x, const tensor_t* w, const tensor_t* b, tensor_t* y, stream_t q, const size_t pad[2], const size_t stride[2]) {
    return code(tannic_hip_conv2d_biased(in(x), in(w), in(b), out(y), st(q), pad, stride));
}
bool allclose(const tensor_t* a, const tensor_t* b, stream_t q, double rtol, double atol) {
    const int r = tannic_hip_allclose(in(a), in(b), st(q), rtol, atol);
    if (r < 0) {
        // the library's own words where it has said why (shapes differ, the stream is being recorded); the reference's otherwise
        const std::string why = tannic_hip_last_error();
        throw std::runtime_error(why.rfind("allclose", 0) == 0 ? why : "Unsupported dtype");
    }
    return r == 1;
}

status conv1d(const tensor_t* x, const tensor_t* w, tensor_t* y, stream_t q, const size_t pad, const size_t stride) {
    return static_cast<status>(tannic_hip_conv1d(in(x), in(w), out(y), st(q), pad, stride));
}
status outer(const tensor_t* a, const tensor_t* b, tensor_t* d, stream_t q) { return static_cast<status>(tannic_hip_outer(in(a), in(b), out(d), st(q))); }
status repeat(const tensor_t* s, tensor_t* d, int axis, int reps, stream_t q) { return static_cast<status>(tannic_hip_repeat(in(s), out(d), st(q), axis, reps)); }
status concat(const tensor_t* a, const tensor_t* b, tensor_t* d, stream_t q, int axis) { return static_cast<status>(tannic_hip_concat(in(a), in(b), out(d), st(q), axis)); }
status triu(const tensor_t* s, tensor_t* d, stream_t q, int k) { return static_cast<status>(tannic_hip_triu(in(s), out(d), st(q), k)); }
status tril(const tensor_t* s, tensor_t* d, stream_t q, int k) { return static_cast<status>(tannic_hip_tril(in(s), out(d), st(q), k)); }

#define TH_CMP(name) status name(const tensor_t* a, const tensor_t* b, tensor_t* d, stream_t q) { return code(tannic_hip_##name(in(a), in(b), out(d), st(q))); }
TH_CMP(eq) TH_CMP(ne) TH_CMP(gt) TH_CMP(ge) TH_CMP(lt) TH_CMP(le)

}  // namespace cuda

namespace tannic_hip {
status max(const tensor_t* s, tensor_t* d, stream_t q, uint8_t axis) { return code(tannic_hip_max(in(s), out(d), st(q), axis)); }
status min(const tensor_t* s, tensor_t* d, stream_t q, uint8_t axis) { return code(tannic_hip_min(in(s), out(d), st(q), axis)); }
status div(const tensor_t* a, const tensor_t* b, tensor_t* d, stream_t q) { return code(tannic_hip_div(in(a), in(b), out(d), st(q))); }
status swiglu(const tensor_t* a, const tensor_t* b, tensor_t* d, stream_t q) { return code(tannic_hip_swiglu(in(a), in(b), out(d), st(q))); }
status cast(const tensor_t* s, tensor_t* d, stream_t q) { return code(tannic_hip_cast(in(s), out(d), st(q))); }
status rms_norm(const tensor_t* x, const tensor_t* g, tensor_t* d, stream_t q, float eps) { return code(tannic_hip_rms_norm(in(x), in(g), out(d), st(q), eps)); }
status softmax(const tensor_t* x, const tensor_t* mask, tensor_t* d, stream_t q, float scale) {
    return code(tannic_hip_softmax(in(x), mask ? in(mask) : nullptr, out(d), st(q), scale));
}
status rope(const tensor_t* x, const tensor_t* c, const tensor_t* s, tensor_t* d, stream_t q) { return code(tannic_hip_rope(in(x), in(c), in(s), out(d), st(q))); }

Recording::Recording(int device) {
    tannic_device_t dvc{};
    dvc.id = device;
    handle_ = tannic_hip_graph_begin(&dvc);
    if (!handle_) throw std::runtime_error(std::string("Recording: ") + tannic_hip_last_error());
}
Recording::~Recording() { tannic_hip_graph_destroy(handle_); }
void Recording::end() {
    if (tannic_hip_graph_end(handle_) != TANNIC_SUCCESS) throw std::runtime_error(std::string("Recording::end: ") + tannic_hip_last_error());
}
void Recording::launch() {
    if (tannic_hip_graph_launch(handle_) != TANNIC_SUCCESS) throw std::runtime_error(std::string("Recording::launch: ") + tannic_hip_last_error());
}
}  // namespace tannic_hip

// Drop-in check: Tannic's own C++ front end (expression templates, Tensor,
// Device, Callback dispatch) driving this repository's HIP backend through the
// `cuda::` adapter.  Every expression is evaluated twice by the SAME front end —
// once on Host (the reference's CPU kernels) and once on Device (this backend)
// — and the two results are compared on the device with the front end's own
// allclose (rtol = atol = 0 where the operation is exact on both sides).
//
// This file is this repository's code; it is compiled against the reference's
// headers and linked with the reference's front-end sources where they are
// mounted (oracle/Makefile, target _ref/frontend_dropin).  The resulting binary
// lives under oracle/_ref/ and is run by tests/test_gpu_frontend.py.
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <functional>
#include <string>
#include <vector>

#include "tensor.hpp"
#include "comparisons.hpp"
#include "complex.hpp"
#include "convolutions.hpp"
#include "filter.hpp"
#include "functions.hpp"
#include "reductions.hpp"
#include "transformations.hpp"

using namespace tannic;

static uint64_t mix(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

// host tensor with seeded uniform values in [low, high)
static Tensor seeded(type dtype, Shape shape, uint64_t id, double low, double high) {
    Tensor t(dtype, shape);
    t.initialize();
    const size_t n = t.nelements();
    const uint64_t base = mix(0x100000001B3ull * 7 + id);
    for (size_t i = 0; i < n; ++i) {
        const double u = static_cast<double>(mix(base + i) >> 40) * (1.0 / 16777216.0);
        const double v = low + (high - low) * u;
        if (dtype == float32) reinterpret_cast<float*>(t.bytes())[i] = static_cast<float>(v);
        else if (dtype == float64) reinterpret_cast<double*>(t.bytes())[i] = v;
        else if (dtype == int32) reinterpret_cast<int32_t*>(t.bytes())[i] = static_cast<int32_t>(v);
    }
    return t;
}

struct Case {
    std::string name;
    double rtol, atol;
    std::function<Tensor(Environment)> run;   // evaluates the expression with operands placed in the environment
};

static Tensor place(Tensor const& host, Environment env) {
    if (std::holds_alternative<Host>(env)) return host;
    return host.to(env);
}

int main() {
    if (Devices::count() < 1) {
        std::printf("no device\n");
        return 2;
    }
    const Tensor X = seeded(float32, {8, 64, 32}, 1, -4, 4);
    const Tensor Z = seeded(float32, {1, 64, 1}, 2, -4, 4);
    const Tensor P = seeded(float32, {8, 64, 32}, 3, 0.25, 4);
    const Tensor A = seeded(float32, {96, 80}, 4, -1, 1);
    const Tensor B = seeded(float32, {80, 72}, 5, -1, 1);
    const Tensor Bt = seeded(float32, {72, 80}, 6, -1, 1);
    const Tensor Q = seeded(float32, {2, 3, 20, 16}, 7, -1, 1);
    const Tensor Kt = seeded(float32, {24, 16}, 8, -1, 1);
    const Tensor D = seeded(float64, {33, 47}, 9, -2, 2);
    const Tensor I = seeded(int32, {4, 9, 5}, 10, -50, 50);
    const Tensor J = seeded(int32, {1, 9, 1}, 11, -50, 50);
    const Tensor S = seeded(float32, {2, 6, 12, 12}, 12, -1, 1);
    const Tensor W = seeded(float32, {5, 6, 3, 3}, 13, -0.4, 0.4);
    const Tensor Bias = seeded(float32, {5}, 14, -1, 1);
    const Tensor Rho = seeded(float32, {6, 10}, 15, 0.5, 2);
    const Tensor Theta = seeded(float32, {6, 10}, 16, -3, 3);
    const Tensor V1 = seeded(float32, {40}, 17, -2, 2);
    const Tensor V2 = seeded(float64, {25}, 18, -2, 2);
    const Tensor Sig = seeded(float32, {2, 6, 50}, 19, -1, 1);
    const Tensor W1 = seeded(float32, {5, 6, 4}, 20, -0.4, 0.4);
    const Tensor Sq = seeded(float32, {12, 12}, 21, -1, 1);

    std::vector<Case> cases = {
        {"log(P)", 1e-5, 1e-8, [&](Environment e) { return Tensor(log(place(P, e))); }},
        {"exp(X)", 1e-5, 1e-8, [&](Environment e) { return Tensor(exp(place(X, e))); }},
        {"sqrt, rsqrt, tanh", 1e-5, 1e-7, [&](Environment e) { Tensor p = place(P, e); return Tensor(sqrt(p) + rsqrt(p, 1e-5f) + tanh(p)); }},
        {"sin*cos - abs", 1e-5, 1e-6, [&](Environment e) { Tensor x = place(X, e); return Tensor(sin(x) * cos(x) - abs(x)); }},
        {"broadcast chain: log(abs(X)+1)+Z*Z-exp(X)+3*X", 1e-5, 2e-4, [&](Environment e) {
             Tensor x = place(X, e), z = place(Z, e);
             Tensor one(float32, {1});
             one.initialize({1.0f}, e);
             return Tensor(log(abs(x) + one) + z * z - exp(x) + 3 * x);
         }},
        {"neg and scale", 0, 0, [&](Environment e) { Tensor x = place(X, e); return Tensor(-x * 0.5f); }},
        {"int32 broadcast add (widened by *1.0f for the comparison)", 0, 0, [&](Environment e) {
             Tensor one(float32, {1});
             one.initialize({1.0f}, e);
             return Tensor((place(I, e) + place(J, e)) * one);
         }},
        {"float64 mul", 0, 0, [&](Environment e) { Tensor d = place(D, e); return Tensor(d * d - d); }},
        {"matmul NN", 1e-5, 1e-5, [&](Environment e) { return Tensor(matmul(place(A, e), place(B, e))); }},
        {"matmul NT (transposed view)", 1e-5, 1e-5, [&](Environment e) { return Tensor(matmul(place(A, e), place(Bt, e).transpose())); }},
        {"matmul rank4 x rank2^T", 1e-5, 1e-5, [&](Environment e) { return Tensor(matmul(place(Q, e), place(Kt, e).transpose())); }},
        {"conv2d 3x3 s1 p1 + bias", 1e-5, 1e-5, [&](Environment e) { return Tensor(convolve2D(place(S, e), place(W, e), place(Bias, e), 1, 1)); }},
        {"conv2d 3x3 s2 p0", 1e-5, 1e-5, [&](Environment e) { return Tensor(convolve2D(place(S, e), place(W, e), 2, 0)); }},
        {"sum over last axis", 1e-5, 1e-5, [&](Environment e) { return Tensor(sum(place(X, e), -1, true)); }},
        {"mean of squares over axis 1", 1e-5, 1e-5, [&](Environment e) { Tensor x = place(X, e); return Tensor(mean(x * x, 1)); }},
        {"polar -> realify", 1e-5, 1e-6, [&](Environment e) { return Tensor(realify(polar(place(Rho, e), place(Theta, e)))); }},
        {"repeat heads (axis 1, 4 times)", 0, 0, [&](Environment e) { return Tensor(repeat(place(Q, e), 4, 1)); }},
        {"concatenate along axis 1", 0, 0, [&](Environment e) { Tensor a = place(A, e); return Tensor(concatenate(a, a * 2.0f, 1)); }},
        {"outer float32 x float64", 0, 0, [&](Environment e) { return Tensor(outer(place(V1, e), place(V2, e))); }},
        {"triangular lower, offset 1", 0, 0, [&](Environment e) { return Tensor(triangular(place(Sq, e), Position::Lower, 1)); }},
        {"conv1d k4 s2 p1", 1e-5, 1e-5, [&](Environment e) { return Tensor(convolve1D(place(Sig, e), place(W1, e), 2, 1)); }},
    };

    int failures = 0;
    for (auto& c : cases) {
        bool ok = false;
        std::string note;
        try {
            Tensor host = c.run(Host{});
            Tensor device = c.run(Device());
            if (host.shape() != device.shape() || host.dtype() != device.dtype()) {
                note = "shape or dtype differs";
            } else {
                ok = allclose(device, host.to(Device()), c.rtol, c.atol);
                if (!ok) note = "allclose failed";
            }
        } catch (std::exception const& ex) {
            note = std::string("exception: ") + ex.what();
        }
        std::printf("%-50s %s %s\n", c.name.c_str(), ok ? "ok" : "FAILED", note.c_str());
        std::fflush(stdout);
        failures += ok ? 0 : 1;
    }
    std::printf("%d of %zu cases failed\n", failures, cases.size());
    return failures ? 1 : 0;
}

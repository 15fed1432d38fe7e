// Drop-in check: Tannic's own C++ front end (expression templates, Tensor,
// Device, Callback dispatch) driving this repository's HIP backend through the
// `cuda::` adapter.  Every expression is evaluated twice by the SAME front end —
// once on Host (the reference's CPU kernels) and once on Device (this backend)
// — and the two results are compared on the device with the front end's own
// allclose (rtol = atol = 0 where the operation is exact on both sides).
// The operators this backend adds (tannic_hip_functions.hpp: div, cast, max, min, softmax, rms_norm, swiglu, rope) have
// no CPU twin: their device results are compared with plain loops written here.  Device comparisons and the copy of
// a device tensor to the host go through the front end as patched by csrc/adapter/frontend.patch.
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
#include "tannic_hip_functions.hpp"   // the operators this backend adds to the front end's surface
#include "tannic_hip_serialization.hpp"   // tensors in the reference's file layout, host or device

#include <cmath>

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

// host float32 tensor filled by f(flat index)
template <class F>
static Tensor computed(Shape shape, F&& f) {
    Tensor t(float32, shape);
    t.initialize();
    for (size_t i = 0; i < t.nelements(); ++i) reinterpret_cast<float*>(t.bytes())[i] = static_cast<float>(f(i));
    return t;
}
static const float* values(Tensor const& host) { return reinterpret_cast<const float*>(host.bytes()); }

int main(int argc, char** argv) {
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

    // ---- operators without a CPU twin: the device against loops in double -----------------------------------------------
    const Tensor G = seeded(float32, {32}, 22, 0.5, 1.5);
    const Tensor Mask = computed({64, 32}, [](size_t i) { return (i % 32) > (i / 32) % 32 ? -INFINITY : 0.0; });
    const Tensor Cs = computed({64, 16}, [](size_t i) { return std::cos(0.37 * (i / 16) / (1.0 + i % 16)); });
    const Tensor Sn = computed({64, 16}, [](size_t i) { return std::sin(0.37 * (i / 16) / (1.0 + i % 16)); });
    const float* x = values(X);
    const float* pv = values(P);
    const float* g = values(G);
    struct DeviceOnly {
        std::string name;
        double rtol, atol;
        std::function<Tensor()> device;      // evaluated on the device
        std::function<Tensor()> expected;    // host tensor computed here
    };
    auto rows = [&](auto&& per_row) {   // X as 512 rows of 32
        return computed({8, 64, 32}, [&, cache = std::vector<double>(32), row = size_t(-1)](size_t i) mutable {
            if (i / 32 != row) { row = i / 32; per_row(x + row * 32, row, cache.data()); }
            return cache[i % 32];
        });
    };
    std::vector<DeviceOnly> added = {
        {"div(X, P)", 1e-6, 0, [&] { return Tensor(div(X.to(Device()), P.to(Device()))); }, [&] { return computed({8, 64, 32}, [&](size_t i) { return x[i] / pv[i]; }); }},
        {"div broadcast: X / Z", 1e-6, 0, [&] { return Tensor(div(X.to(Device()), Z.to(Device()))); },
         [&] { return computed({8, 64, 32}, [&](size_t i) { return x[i] / values(Z)[(i / 32) % 64]; }); }},
        {"cast int32 -> float32", 0, 0, [&] { return Tensor(cast(I.to(Device()), float32)); },
         [&] { return computed({4, 9, 5}, [&](size_t i) { return reinterpret_cast<const int32_t*>(I.bytes())[i]; }); }},
        {"cast float32 -> int32 -> float32 (truncation)", 0, 0, [&] { return Tensor(cast(cast(X.to(Device()), int32), float32)); },
         [&] { return computed({8, 64, 32}, [&](size_t i) { return std::trunc(x[i]); }); }},
        {"max over the last axis, kept", 0, 0, [&] { return Tensor(max(X.to(Device()), -1, true)); },
         [&] { return computed({8, 64, 1}, [&](size_t r) { double m = x[r * 32]; for (int j = 1; j < 32; ++j) m = std::max<double>(m, x[r * 32 + j]); return m; }); }},
        {"min over axis 1", 0, 0, [&] { return Tensor(min(X.to(Device()), 1)); },
         [&] { return computed({8, 32}, [&](size_t o) { double m = INFINITY; for (int j = 0; j < 64; ++j) m = std::min<double>(m, x[(o / 32) * 2048 + j * 32 + o % 32]); return m; }); }},
        {"X / max(|X|) composed of the new nodes", 1e-6, 0, [&] { Tensor d = X.to(Device()); return Tensor(div(d, max(abs(d), -1, true))); },
         [&] { return rows([](const float* r, size_t, double* out) { double m = 0; for (int j = 0; j < 32; ++j) m = std::max<double>(m, std::fabs(r[j])); for (int j = 0; j < 32; ++j) out[j] = r[j] / m; }); }},
        {"rms_norm(X, G, 1e-5)", 2e-6, 1e-7, [&] { return Tensor(rms_norm(X.to(Device()), G.to(Device()), 1e-5f)); },
         [&] { return rows([&](const float* r, size_t, double* out) { double ms = 0; for (int j = 0; j < 32; ++j) ms += double(r[j]) * r[j]; ms = 1.0 / std::sqrt(ms / 32 + 1e-5f); for (int j = 0; j < 32; ++j) out[j] = r[j] * ms * g[j]; }); }},
        {"softmax(0.5 * X)", 2e-6, 1e-9, [&] { return Tensor(softmax(X.to(Device()), 0.5f)); },
         [&] { return rows([](const float* r, size_t, double* out) { double m = -INFINITY, sum = 0; for (int j = 0; j < 32; ++j) m = std::max<double>(m, 0.5 * r[j]); for (int j = 0; j < 32; ++j) sum += out[j] = std::exp(0.5 * r[j] - m); for (int j = 0; j < 32; ++j) out[j] /= sum; }); }},
        {"softmax(X + causal mask)", 2e-6, 1e-9, [&] { return Tensor(softmax(X.to(Device()), Mask.to(Device()))); },
         [&] { return rows([](const float* r, size_t row, double* out) { const int q = row % 64 % 32; double m = -INFINITY, sum = 0; for (int j = 0; j <= q; ++j) m = std::max<double>(m, r[j]); for (int j = 0; j < 32; ++j) sum += out[j] = j <= q ? std::exp(r[j] - m) : 0.0; for (int j = 0; j < 32; ++j) out[j] /= sum; }); }},
        {"swiglu(X, P)", 2e-6, 1e-7, [&] { return Tensor(swiglu(X.to(Device()), P.to(Device()))); }, [&] { return computed({8, 64, 32}, [&](size_t i) { return x[i] / (1.0 + std::exp(-double(x[i]))) * pv[i]; }); }},
        {"rope(X, cos, sin)", 2e-6, 1e-6, [&] { return Tensor(rope(X.to(Device()), Cs.to(Device()), Sn.to(Device()))); },
         [&] { return computed({8, 64, 32}, [&](size_t i) { const size_t n = (i / 32) % 64, pair = (i % 32) / 2; const double c = values(Cs)[n * 16 + pair], sn = values(Sn)[n * 16 + pair];
                                                         const double e = x[i - i % 2], o = x[i - i % 2 + 1]; return i % 2 == 0 ? e * c - o * sn : e * sn + o * c; }); }},
    };

    int failures = 0;
    for (auto& c : added) {
        bool ok = false;
        std::string note;
        try {
            Tensor device = c.device();
            Tensor expected = c.expected();
            if (device.shape() != expected.shape() || device.dtype() != expected.dtype()) note = "shape or dtype differs";
            else if (!(ok = allclose(device, expected.to(Device()), c.rtol, c.atol))) note = "allclose failed";
        } catch (std::exception const& ex) {
            note = std::string("exception: ") + ex.what();
        }
        std::printf("%-50s %s %s\n", c.name.c_str(), ok ? "ok" : "FAILED", note.c_str());
        std::fflush(stdout);
        failures += ok ? 0 : 1;
    }
    // the new nodes exist on the device only
    {
        bool threw = false;
        try { Tensor t = softmax(X); } catch (std::exception const&) { threw = true; }
        std::printf("%-50s %s\n", "softmax of a host tensor throws", threw ? "ok" : "FAILED");
        failures += threw ? 0 : 1;
    }
    // ---- a sequence of the front end's evaluations recorded once and replayed as a graph ------------------------------------
    {
        bool ok = false;
        std::string note;
        try {
            Tensor x = X.to(Device()), z = Z.to(Device()), a = A.to(Device()), b = B.to(Device());
            Tensor one(float32, {1});
            one.initialize({1.0f}, Device());
            auto chain = [&] { return Tensor(log(abs(x) + one) + z * z - exp(x) + 3 * x); };
            auto product = [&] { return Tensor(matmul(a, b) * 0.5f); };
            const Tensor want_chain = chain(), want_product = product();
            tannic_hip::Recording recording(0);
            Tensor got_chain = chain();          // temporaries of the expression are released while recording
            Tensor got_product = product();
            recording.end();
            ok = true;
            for (int replay = 0; replay < 3 && ok; ++replay) {
                recording.launch();
                ok = allclose(got_chain, want_chain, 0, 0) && allclose(got_product, want_product, 0, 0);
                if (!ok) note = "replay " + std::to_string(replay) + " differs from the eager evaluation";
                Tensor between = chain();        // eager work between replays takes and returns blocks of the same sizes
                ok = ok && allclose(between, want_chain, 0, 0);
            }
            // new input in the same memory: the replay sees it
            Tensor x2 = seeded(float32, {8, 64, 32}, 31, -4, 4).to(Device());
            x[indexing::Range{0, 8}] = x2;
            const Tensor want2 = chain();
            recording.launch();
            if (ok && !allclose(got_chain, want2, 0, 0)) { ok = false; note = "replay after new input differs"; }
            // a call that waits for the device is refused while recording, and the device works afterwards
            bool threw = false;
            {
                tannic_hip::Recording open(0);
                Tensor t = chain();
                try { (void)allclose(t, want2, 0, 0); } catch (std::exception const&) { threw = true; }
            }
            if (ok && !threw) { ok = false; note = "allclose while recording did not throw"; }
            if (ok && !allclose(chain(), want2, 0, 0)) { ok = false; note = "eager evaluation after an abandoned recording differs"; }
        } catch (std::exception const& ex) {
            ok = false;
            note = std::string("exception: ") + ex.what();
        }
        std::printf("%-50s %s %s\n", "expressions recorded once, replayed as a graph", ok ? "ok" : "FAILED", note.c_str());
        failures += ok ? 0 : 1;
    }
    // ---- comparisons on the device and the copy back to the host, through the (patched) front end ------------------------
    {
        const Tensor I2 = seeded(int32, {4, 9, 5}, 23, -50, 50);
        const Tensor X2 = seeded(float32, {8, 64, 32}, 24, -4, 4);
        struct Pair { const char* name; std::function<Tensor(Tensor const&, Tensor const&)> run; };
        const std::vector<Pair> comparisons = {
            {"==", [](Tensor const& a, Tensor const& b) { return Tensor(a == b); }}, {"!=", [](Tensor const& a, Tensor const& b) { return Tensor(a != b); }},
            {">", [](Tensor const& a, Tensor const& b) { return Tensor(a > b); }},   {">=", [](Tensor const& a, Tensor const& b) { return Tensor(a >= b); }},
            {"<", [](Tensor const& a, Tensor const& b) { return Tensor(a < b); }},   {"<=", [](Tensor const& a, Tensor const& b) { return Tensor(a <= b); }},
        };
        for (auto const& [left, right, what] : {std::tuple<Tensor const&, Tensor const&, const char*>{I, I2, "int32"}, {X, X2, "float32"}, {X, X, "float32 with itself"}}) {
            for (auto const& c : comparisons) {
                bool ok = false;
                std::string note;
                try {
                    Tensor host = c.run(left, right);
                    Tensor device = c.run(left.to(Device()), right.to(Device()));
                    Tensor back = device.to(Host{});              // device -> host through Tensor::to
                    ok = back.dtype() == boolean && back.shape() == host.shape() && std::memcmp(back.bytes(), host.bytes(), (host.nelements() + 7) / 8) == 0;
                    if (!ok) note = "bit masks differ";
                } catch (std::exception const& ex) {
                    note = std::string("exception: ") + ex.what();
                }
                std::printf("%-50s %s %s\n", (std::string("device ") + c.name + " on " + what + ", copied back with to(Host)").c_str(), ok ? "ok" : "FAILED", note.c_str());
                failures += ok ? 0 : 1;
            }
        }
        // a float tensor's round trip host -> device -> host
        Tensor back = X.to(Device()).to(Host{});
        const bool same = std::memcmp(back.bytes(), X.bytes(), X.nelements() * sizeof(float)) == 0;
        std::printf("%-50s %s\n", "host -> device -> host round trip", same ? "ok" : "FAILED");
        failures += same ? 0 : 1;
    }

    // ---- tensors in the reference's file layout (include/tannic/serialization.hpp:26-66), through tannic_hip_serialization.hpp ----
    {
        auto check = [&](const char* what, bool ok) {
            std::printf("%-50s %s\n", what, ok ? "ok" : "FAILED");
            failures += ok ? 0 : 1;
        };
        try {
            const std::vector<std::byte> image = hip::dumps(X);
            // Header 15 bytes, Metadata 18 bytes, three extents, the data
            const unsigned char head[] = {0x45, 0x52, 0x49, 0x43, 0x01, 0xCD, 0xAB};
            uint64_t announced = 0, data = 0;
            std::memcpy(&announced, image.data() + 7, 8);
            std::memcpy(&data, image.data() + 15 + 9, 8);
            check("file image: sizes and the header's fixed bytes", image.size() == 15 + 18 + 24 + X.nbytes() && std::memcmp(image.data(), head, 7) == 0 &&
                                                                       announced == image.size() - 15 && data == X.nbytes() &&
                                                                       static_cast<unsigned char>(image[15]) == 24 && static_cast<unsigned char>(image[15 + 17]) == 3);
            Tensor back = hip::loads(image);
            check("file image -> host tensor: the same bytes", back.dtype() == float32 && back.shape() == X.shape() && std::memcmp(back.bytes(), X.bytes(), X.nbytes()) == 0);
            Tensor on_device = hip::loads(image, Device());
            check("file image -> device tensor", allclose(on_device, X.to(Device()), 0, 0));
            const std::vector<std::byte> again = hip::dumps(on_device);
            check("device tensor -> file image: the same image", again == image);
            Tensor packed = Tensor(I.to(Device()) > seeded(int32, {4, 9, 5}, 23, -50, 50).to(Device()));   // booleans: bit-packed data
            Tensor packed_back = hip::loads(hip::dumps(packed));
            Tensor packed_host = packed.to(Host{});
            check("boolean tensor round trip (bit-packed)", packed_back.dtype() == boolean && packed_back.shape() == packed.shape() &&
                                                                std::memcmp(packed_back.bytes(), packed_host.bytes(), (packed.nelements() + 7) / 8) == 0);
            bool threw = false;
            try { std::vector<std::byte> cut(image.begin(), image.end() - 5); (void)hip::loads(cut); } catch (std::exception const&) { threw = true; }
            check("a truncated image is refused", threw);
            threw = false;
            try { std::vector<std::byte> bad = image; bad[0] = std::byte{0}; (void)hip::loads(bad); } catch (std::exception const&) { threw = true; }
            check("an image with another magic is refused", threw);
            threw = false;
            try { (void)hip::dumps(Tensor(transpose(X, 0, 2))); } catch (std::exception const&) { threw = true; }
            check("a transposed view is not written", threw);
            if (argc > 1) {
                // files shared with the Python reader and writer of the same layout
                const std::string dir = argv[1];
                hip::save(X.to(Device()) * 0.5f, dir + "/from_cpp.tannic");
                Tensor theirs = hip::load(dir + "/from_python.tannic", Device());
                Tensor expected = computed({2, 3, 4}, [](size_t i) { return 0.5 * i; });
                check("a file written by the Python writer, loaded onto the device", theirs.dtype() == float32 && theirs.shape() == expected.shape() && allclose(theirs, expected.to(Device()), 0, 0));
            }
        } catch (std::exception const& ex) {
            std::printf("%-50s FAILED exception: %s\n", "tensor files", ex.what());
            failures += 1;
        }
    }

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
    std::printf("%d of %zu cases failed\n", failures, cases.size() + added.size() + 21 + 8 + (argc > 1 ? 1 : 0));
    return failures ? 1 : 0;
}

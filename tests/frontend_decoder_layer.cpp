// One Llama-3 decoder layer written with Tannic's own C++ front end (Tensor, views, slices, expression templates,
// Callback dispatch) and evaluated by this repository's HIP backend through the `cuda::` adapter.
//
//     frontend_decoder_layer check               reduced size, float32: the layer evaluated by the front end on Host (the
//                                                reference's CPU kernels) and on Device, compared; the one-pass form
//                                                (tannic_hip_functions.hpp) against the composed form on the device;
//                                                a recording of the layer replayed and compared bit for bit
//     frontend_decoder_layer full [dir] [iters]  hidden 4096, 32/8 heads of 128, FFN 14336, 512 positions, bfloat16:
//                                                both forms eager and replayed as a recording, timed; with `dir` the
//                                                inputs, parameters and results are written there as raw little-endian
//                                                files for a caller that evaluates the same layer another way
//
// The expressions are the ones a Tannic program can write today: no division, no cast and no softmax exist in the
// front end, so the reciprocal of a sum is rsqrt(s) * rsqrt(s), the rotary embedding is the real-valued form on
// stride-2 slices (complex tensors are float32 / float64 only, include/tannic/complex.hpp:53-58) and the causal mask is
// a host-built table added to the scores.  The row maximum of the softmax is this backend's `max` node (the reference
// has argmax only); on Host, where that node does not exist, the softmax is evaluated without the shift.
//
// This file is this repository's code; oracle/Makefile compiles it against the reference's headers and links it with
// the reference's front-end sources where they are mounted (target _ref/frontend_decoder_layer).
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "tensor.hpp"
#include "comparisons.hpp"
#include "functions.hpp"
#include "reductions.hpp"
#include "transformations.hpp"
#include "views.hpp"
#include "tannic_hip_functions.hpp"

extern "C" int tannic_hip_device_synchronize(void);

using namespace tannic;

struct LayerShape {
    size_t hidden = 4096, heads = 32, kv_heads = 8, head_dim = 128, ffn = 14336, seq = 512;
    float eps = 1e-5f;
    double theta = 500000.0;
};

using Parameters = std::map<std::string, Tensor>;

// ---- seeded values ---------------------------------------------------------------------------------------------------
static uint64_t mix(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

static uint16_t to_bfloat16(float value) {   // round to nearest even
    uint32_t bits;
    std::memcpy(&bits, &value, 4);
    if ((bits & 0x7FFFFFFFu) > 0x7F800000u) return static_cast<uint16_t>((bits >> 16) | 0x40);
    bits += 0x7FFFu + ((bits >> 16) & 1u);
    return static_cast<uint16_t>(bits >> 16);
}

static void store(Tensor& t, size_t i, double value) {
    if (t.dtype() == float32) reinterpret_cast<float*>(t.bytes())[i] = static_cast<float>(value);
    else reinterpret_cast<uint16_t*>(t.bytes())[i] = to_bfloat16(static_cast<float>(value));
}

// host tensor of N(0, sigma) values (Box-Muller on a counter-based hash; both outputs of a pair are used)
static Tensor normal(type dtype, Shape shape, uint64_t id, double sigma) {
    Tensor t(dtype, shape);
    t.initialize();
    const size_t n = t.nelements();
    const uint64_t base = mix(0x100000001B3ull * 11 + id);
    for (size_t i = 0; i < n; i += 2) {
        const double u1 = (static_cast<double>(mix(base + i) >> 11) + 1.0) * (1.0 / 9007199254740993.0);
        const double u2 = static_cast<double>(mix(base + i + 1) >> 11) * (1.0 / 9007199254740992.0);
        const double radius = sigma * std::sqrt(-2.0 * std::log(u1)), angle = 6.283185307179586 * u2;
        store(t, i, radius * std::cos(angle));
        if (i + 1 < n) store(t, i + 1, radius * std::sin(angle));
    }
    return t;
}

template <class F>
static Tensor table(type dtype, Shape shape, F&& f) {
    Tensor t(dtype, shape);
    t.initialize();
    for (size_t i = 0; i < t.nelements(); ++i) store(t, i, f(i));
    return t;
}

static Parameters parameters(LayerShape const& s, type dtype, Environment env) {
    const size_t nq = s.heads * s.head_dim, nkv = s.kv_heads * s.head_dim;
    Parameters w;
    auto put = [&](const char* name, Tensor host) { w.emplace(name, std::holds_alternative<Host>(env) ? host : host.to(env)); };
    put("wq", normal(dtype, {nq, s.hidden}, 1, 0.02));
    put("wk", normal(dtype, {nkv, s.hidden}, 2, 0.02));
    put("wv", normal(dtype, {nkv, s.hidden}, 3, 0.02));
    put("wo", normal(dtype, {s.hidden, nq}, 4, 0.02));
    put("w1", normal(dtype, {s.ffn, s.hidden}, 5, 0.02));
    put("w3", normal(dtype, {s.ffn, s.hidden}, 6, 0.02));
    put("w2", normal(dtype, {s.hidden, s.ffn}, 7, 0.02));
    put("g1", table(dtype, {s.hidden}, [](size_t i) { return 1.0 + 0.25 * std::sin(0.1 * i); }));
    put("g2", table(dtype, {s.hidden}, [](size_t i) { return 1.0 - 0.25 * std::cos(0.07 * i); }));
    const size_t half = s.head_dim / 2;
    auto angle = [=](size_t i) { return static_cast<double>(i / half) * std::pow(s.theta, -2.0 * static_cast<double>(i % half) / s.head_dim); };
    put("cos", table(dtype, {s.seq, half}, [&](size_t i) { return std::cos(angle(i)); }));
    put("sin", table(dtype, {s.seq, half}, [&](size_t i) { return std::sin(angle(i)); }));
    put("mask", table(dtype, {s.seq, s.seq}, [&](size_t i) { return i % s.seq > i / s.seq ? -INFINITY : 0.0; }));
    put("one", table(dtype, {1}, [](size_t) { return 1.0; }));
    put("x", normal(dtype, {1, s.seq, s.hidden}, 8, 1.0));
    return w;
}

// ---- the layer, composed from the front end's operators ----------------------------------------------------------------
static Tensor rms_norm_composed(Tensor const& x, Tensor const& gain, float eps) {
    Tensor ms = mean(x * x, -1, true);
    return x * rsqrt(ms, eps) * gain;
}

// q: [1, heads, seq, head_dim], any strides.  The pairs (2i, 2i+1) turn by the position's angle.
static Tensor rope_composed(Tensor const& q, Tensor const& cs, Tensor const& sn) {
    const size_t b = q.size(0), h = q.size(1), n = q.size(2), d = q.size(3);
    Tensor qc = repack(q);
    Tensor q5 = qc.view(b, h, n, d / 2, 2);
    Tensor even = q5[range{}, range{}, range{}, range{}, 0];
    Tensor odd = q5[range{}, range{}, range{}, range{}, 1];
    Tensor re = even * cs - odd * sn;
    Tensor im = even * sn + odd * cs;
    Tensor out(q.dtype(), {b, h, n, d});
    out.initialize(q.environment());
    Tensor o5 = out.view(b, h, n, d / 2, 2);
    o5[range{}, range{}, range{}, range{}, 0] = re;
    o5[range{}, range{}, range{}, range{}, 1] = im;
    return out;
}

static Tensor softmax_composed(Tensor const& scores, bool shifted) {
    Tensor e;
    if (shifted) {
        Tensor m = max(scores, -1, true);
        e = exp(scores - m);
    } else {
        e = exp(scores);
    }
    Tensor r = rsqrt(sum(e, -1, true));
    return e * r * r;
}

static Tensor silu_composed(Tensor const& g, Tensor const& one) {
    Tensor sg = rsqrt(exp(-g) + one);   // sigmoid(g) = sg * sg
    return g * sg * sg;
}

static Tensor layer_composed(LayerShape const& s, Parameters const& w, bool shifted_softmax) {
    Tensor const& x = w.at("x");
    const size_t group = s.heads / s.kv_heads;
    Tensor xn = rms_norm_composed(x, w.at("g1"), s.eps);
    Tensor q = matmul(xn, w.at("wq").transpose());
    Tensor k = matmul(xn, w.at("wk").transpose());
    Tensor v = matmul(xn, w.at("wv").transpose());
    Tensor qh = transpose(view(q, 1, s.seq, s.heads, s.head_dim), 1, 2);
    Tensor kh = transpose(view(k, 1, s.seq, s.kv_heads, s.head_dim), 1, 2);
    Tensor vh = transpose(view(v, 1, s.seq, s.kv_heads, s.head_dim), 1, 2);
    Tensor qr = rope_composed(qh, w.at("cos"), w.at("sin"));
    Tensor kr = rope_composed(kh, w.at("cos"), w.at("sin"));
    Tensor ka = repeat(kr, static_cast<int>(group), 1);
    Tensor va = repeat(vh, static_cast<int>(group), 1);
    Tensor scores = matmul(qr, ka.transpose(-1, -2)) * static_cast<float>(1.0 / std::sqrt(static_cast<double>(s.head_dim)));
    Tensor masked = scores + w.at("mask");
    Tensor p = softmax_composed(masked, shifted_softmax);
    Tensor pv = matmul(p, va);
    Tensor heads_last = repack(transpose(pv, 1, 2));
    Tensor o = heads_last.view(1, s.seq, s.heads * s.head_dim);
    Tensor h = x + matmul(o, w.at("wo").transpose());
    Tensor hn = rms_norm_composed(h, w.at("g2"), s.eps);
    Tensor gate = matmul(hn, w.at("w1").transpose());
    Tensor up = matmul(hn, w.at("w3").transpose());
    Tensor act = silu_composed(gate, w.at("one")) * up;
    Tensor y = matmul(act, w.at("w2").transpose());
    return h + y;
}

// ---- the same layer with this backend's one-pass nodes, gate and up projections stored as one matrix ---------------------
static void pack(Parameters& w) {
    w.emplace("w13", Tensor(concatenate(w.at("w1"), w.at("w3"), 0)));
}

static Tensor layer_one_pass(LayerShape const& s, Parameters const& w) {
    Tensor const& x = w.at("x");
    const int ffn = static_cast<int>(s.ffn);
    const size_t group = s.heads / s.kv_heads;
    Tensor xn = rms_norm(x, w.at("g1"), s.eps);
    // q, k, v stay three products: a column range of a packed result cannot be seen as heads by the front end's
    // `view`, which takes contiguous tensors only (include/tannic/views.hpp:58-60)
    Tensor q = matmul(xn, w.at("wq").transpose());
    Tensor k = matmul(xn, w.at("wk").transpose());
    Tensor v = matmul(xn, w.at("wv").transpose());
    Tensor qr = rope(transpose(view(q, 1, s.seq, s.heads, s.head_dim), 1, 2), w.at("cos"), w.at("sin"));
    Tensor kr = rope(transpose(view(k, 1, s.seq, s.kv_heads, s.head_dim), 1, 2), w.at("cos"), w.at("sin"));
    Tensor vh = transpose(view(v, 1, s.seq, s.kv_heads, s.head_dim), 1, 2);
    Tensor ka = repeat(kr, static_cast<int>(group), 1);
    Tensor va = repeat(vh, static_cast<int>(group), 1);
    Tensor p = softmax(matmul(qr, ka.transpose(-1, -2)), w.at("mask"), static_cast<float>(1.0 / std::sqrt(static_cast<double>(s.head_dim))));
    Tensor pv = matmul(p, va);
    Tensor heads_last = repack(transpose(pv, 1, 2));
    Tensor o = heads_last.view(1, s.seq, s.heads * s.head_dim);
    Tensor h = x + matmul(o, w.at("wo").transpose());
    Tensor hn = rms_norm(h, w.at("g2"), s.eps);
    Tensor both = matmul(hn, w.at("w13").transpose());
    Tensor act = swiglu(both[range{}, range{}, range{0, ffn}], both[range{}, range{}, range{ffn, 2 * ffn}]);
    Tensor y = matmul(act, w.at("w2").transpose());
    return h + y;
}

// ---- helpers ---------------------------------------------------------------------------------------------------------
static bool same_bits(Tensor const& a, Tensor const& b) { return allclose(a, b, 0, 0); }

static void write_raw(std::string const& path, Tensor const& device_or_host) {
    Tensor host = std::holds_alternative<Host>(device_or_host.environment()) ? device_or_host : device_or_host.to(Host{});
    std::FILE* f = std::fopen(path.c_str(), "wb");
    if (!f) throw Exception("cannot write " + path);
    std::fwrite(host.bytes(), 1, host.nbytes(), f);
    std::fclose(f);
}

template <class Step>
static double microseconds_per_call(Step&& step, int iters) {
    for (int i = 0; i < 3; ++i) step();
    tannic_hip_device_synchronize();
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < iters; ++i) step();
    tannic_hip_device_synchronize();
    return std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count() / iters;
}

static double flop_count(LayerShape const& s) {
    const double proj = double(s.seq) * s.hidden * (s.heads + 2 * s.kv_heads) * s.head_dim + double(s.seq) * s.heads * s.head_dim * s.hidden;
    const double attn = 2.0 * s.heads * s.seq * s.seq * s.head_dim;
    const double ffn = 3.0 * s.seq * s.hidden * s.ffn;
    return 2 * (proj + attn + ffn);
}

static int report(const char* what, bool ok, std::string const& note = "") {
    std::printf("%-78s %s %s\n", what, ok ? "ok" : "FAILED", note.c_str());
    std::fflush(stdout);
    return ok ? 0 : 1;
}

static int check() {
    LayerShape s;
    s.hidden = 256; s.heads = 4; s.kv_heads = 2; s.head_dim = 64; s.ffn = 512; s.seq = 64;
    int failures = 0;
    Parameters host = parameters(s, float32, Host{});
    Parameters device = parameters(s, float32, Device());
    Tensor on_host = layer_composed(s, host, false);
    Tensor composed = layer_composed(s, device, true);
    failures += report("composed layer, float32 64 x 256: Device against the front end's Host evaluation",
                       composed.shape() == on_host.shape() && allclose(composed, on_host.to(Device()), 2e-4, 2e-4));
    Tensor unshifted = layer_composed(s, device, false);
    failures += report("... the softmax without its row maximum (the Host form), on the device", allclose(unshifted, on_host.to(Device()), 2e-4, 2e-4));
    pack(device);
    Tensor one_pass = layer_one_pass(s, device);
    failures += report("one-pass nodes and packed parameters against the composed layer", allclose(one_pass, composed, 2e-4, 2e-4));
    {
        tannic_hip::Recording recording(0);
        Tensor recorded = layer_composed(s, device, true);
        Tensor recorded_one_pass = layer_one_pass(s, device);
        recording.end();
        bool ok = true;
        for (int replay = 0; replay < 3 && ok; ++replay) {
            recording.launch();
            ok = same_bits(recorded, composed) && same_bits(recorded_one_pass, one_pass);
            Tensor between = layer_composed(s, device, true);   // eager work between the replays
            ok = ok && same_bits(between, composed);
        }
        failures += report("both forms recorded once, replayed three times: bit for bit the eager results", ok);
        // new input in the same memory
        Tensor x2 = normal(float32, {1, s.seq, s.hidden}, 99, 1.0).to(Device());
        device.at("x")[range{0, 1}] = x2;
        Tensor want = layer_composed(s, device, true);
        recording.launch();
        failures += report("... and follows new input written into x's memory", same_bits(recorded, want) && !same_bits(want, composed));
    }
    std::printf("%d checks failed\n", failures);
    return failures ? 1 : 0;
}

static int full(std::string const& dir, int iters) {
    LayerShape s;
    const auto t0 = std::chrono::steady_clock::now();
    Parameters w = parameters(s, bfloat16, Device());
    std::printf("parameters drawn and placed on the device in %.1f s\n", std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count());
    std::fflush(stdout);
    int failures = 0;
    Tensor composed = layer_composed(s, w, true);
    const double eager_us = microseconds_per_call([&] { Tensor y = layer_composed(s, w, true); }, iters);
    pack(w);
    Tensor one_pass = layer_one_pass(s, w);
    const double eager_one_pass_us = microseconds_per_call([&] { Tensor y = layer_one_pass(s, w); }, iters);
    double replay_us = 0, replay_one_pass_us = 0;
    {
        tannic_hip::Recording recording(0);
        Tensor recorded = layer_composed(s, w, true);
        recording.end();
        replay_us = microseconds_per_call([&] { recording.launch(); }, iters);
        failures += report("composed layer, bfloat16 512 x 4096: the replayed recording equals the eager result bit for bit", same_bits(recorded, composed));
    }
    {
        tannic_hip::Recording recording(0);
        Tensor recorded = layer_one_pass(s, w);
        recording.end();
        replay_one_pass_us = microseconds_per_call([&] { recording.launch(); }, iters);
        failures += report("one-pass layer: the replayed recording equals the eager result bit for bit", same_bits(recorded, one_pass));
    }
    // the two forms round differently (one rounding per row operator against one per node): the same bound as the
    // Python harness uses for this pair, 0.15 of the output's spread, is checked by the caller on the written files
    if (!dir.empty()) {
        for (const char* name : {"x", "wq", "wk", "wv", "wo", "w1", "w3", "w2", "g1", "g2", "cos", "sin", "mask"}) write_raw(dir + "/" + name + ".bin", w.at(name));
        write_raw(dir + "/composed.bin", composed);
        write_raw(dir + "/one_pass.bin", one_pass);
    }
    const double flops = flop_count(s);
    std::printf("{\"composed_eager_us\": %.1f, \"composed_replay_us\": %.1f, \"one_pass_eager_us\": %.1f, \"one_pass_replay_us\": %.1f, \"flops\": %.0f, \"iters\": %d}\n",
                eager_us, replay_us, eager_one_pass_us, replay_one_pass_us, flops, iters);
    std::printf("%d checks failed\n", failures);
    return failures ? 1 : 0;
}

int main(int argc, char** argv) {
    if (Devices::count() < 1) {
        std::printf("no device\n");
        return 2;
    }
    try {
        const std::string mode = argc > 1 ? argv[1] : "check";
        if (mode == "check") return check();
        if (mode == "full") return full(argc > 2 ? argv[2] : "", argc > 3 ? std::atoi(argv[3]) : 20);
        std::printf("usage: frontend_decoder_layer check | full [dir] [iters]\n");
        return 2;
    } catch (std::exception const& ex) {
        std::printf("exception: %s\n", ex.what());
        return 1;
    }
}

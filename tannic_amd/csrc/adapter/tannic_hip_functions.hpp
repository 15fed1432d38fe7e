// Expression nodes for the operators this backend adds to Tannic's surface: division, dtype conversion, value max / min
// over an axis, and the one-pass row operators (softmax, rms_norm, swiglu, rope).  Include it after the front end's headers in
// a program that links the `cuda::` adapter; the nodes compose with every other expression:
//
//     Tensor y = rms_norm(x, gain, 1e-5f) * 2.0f;
//     Tensor p = softmax(matmul(q, k.transpose(-1, -2)), mask, 0.0884f);
//     Tensor r = div(x, max(abs(x), -1, true));
//
// Each node follows the reference's own pattern for its kind - a functor or reducer whose `forward` allocates nothing
// itself, wrapped in the expression class that computes dtype / shape at construction and evaluates its operands into
// a fresh contiguous target (include/tannic/functions.hpp:52-57, include/tannic/reductions.hpp:88-93,
// include/tannic/operations.hpp Binary + include/tannic/tensor.hpp:358-363).  The reference's CPU backend has no twin for
// these operators, so the nodes evaluate on a Device only; on Host they throw.
#pragma once

#include <initializer_list>
#include <variant>

#include "callback.hpp"
#include "concepts.hpp"
#include "exceptions.hpp"
#include "expressions.hpp"
#include "indexing.hpp"
#include "operations.hpp"
#include "reductions.hpp"
#include "tensor.hpp"
#include "tannic_hip_adapter.hpp"

namespace tannic::hip {

// What Callback does for the reference's operators (include/tannic/callback.hpp:46-178), for any number of sources:
// every source on one device, the target allocated there, one stream popped for the call, any failure thrown.
template <class Call>
inline void on_device(std::initializer_list<const Tensor*> sources, Tensor& target, const char* who, Call&& call) {
    const Tensor& first = **sources.begin();
    if (!std::holds_alternative<Device>(first.environment())) throw Exception(std::string(who) + ": implemented by the device backend only (move the operands to a Device)");
    const int id = std::get<Device>(first.environment()).id();
    for (const Tensor* source : sources)
        if (!std::holds_alternative<Device>(source->environment()) || std::get<Device>(source->environment()).id() != id) throw Exception(std::string(who) + ": operands live in different environments");
    if (!target.is_initialized()) target.initialize(first.environment());
    device_t device{id};
    stream_t stream = pop_stream(&device);
    const status result = call(stream);
    put_stream(&device, stream);
    if (result != SUCCESS) throw Exception(std::string(who) + (result == UNSUPPORTED_DTYPE ? ": unsupported dtype" : ": rejected by the device backend (shapes or dtypes do not fit)"));
}

// ---- division and the gated activation: Binary expressions with the broadcasting and promotion of `*` ----------------
struct Division {
    void forward(Tensor const& first, Tensor const& second, Tensor& target) const {
        on_device({&first, &second}, target, "div", [&](stream_t s) { return tannic_hip::div(get_tensor(first.id()), get_tensor(second.id()), get_tensor(target.id()), s); });
    }
    constexpr static type promote(type first, type second) { return operation::promote(first, second); }
    constexpr static Shape broadcast(Shape const& first, Shape const& second) { return operation::broadcast(first, second); }
};

struct GatedActivation {   // gate / (1 + exp(-gate)) * up
    void forward(Tensor const& gate, Tensor const& up, Tensor& target) const {
        on_device({&gate, &up}, target, "swiglu", [&](stream_t s) { return tannic_hip::swiglu(get_tensor(gate.id()), get_tensor(up.id()), get_tensor(target.id()), s); });
    }
    constexpr static type promote(type first, type second) { return operation::promote(first, second); }
    constexpr static Shape broadcast(Shape const& first, Shape const& second) { return operation::broadcast(first, second); }
};

// ---- value max / min over an axis: reducers for expression::Reduction ---------------------------------------------------
template <bool LARGEST>
struct Extreme {
    int axis;
    bool keepdim;
    constexpr type reduce(type dtype) const { return dtype; }
    constexpr Shape reduce(Shape const& shape) const {
        if (shape.rank() == 0) throw Exception("Cannot reduce scalar tensors");
        Shape out;
        for (size_t dim = 0; dim < shape.rank(); ++dim) {
            if (dim != static_cast<size_t>(axis)) out.expand(shape[dim]);
            else if (keepdim) out.expand(1);
        }
        return out;
    }
    void forward(Tensor const& input, Tensor& target) const {
        on_device({&input}, target, LARGEST ? "max" : "min", [&](stream_t s) {
            return LARGEST ? tannic_hip::max(get_tensor(input.id()), get_tensor(target.id()), s, static_cast<uint8_t>(axis))
                           : tannic_hip::min(get_tensor(input.id()), get_tensor(target.id()), s, static_cast<uint8_t>(axis));
        });
    }
};

// ---- nodes whose result has the first operand's shape: conversion and the row operators ---------------------------------
// Kernel: `type result(type)` and `void forward(Tensor const&..., Tensor&) const`.
template <class Kernel, Composable... Operands>
class Rowwise : public expression::Expression<Kernel, Operands...> {
public:
    constexpr Rowwise(Kernel kernel, typename Trait<Operands>::Reference... operands)
    :   expression::Expression<Kernel, Operands...>(kernel, operands...)
    ,   dtype_(kernel.result(std::get<0>(this->operands).dtype()))
    ,   shape_(std::get<0>(this->operands).shape())
    ,   strides_(shape_) {}

    constexpr type dtype() const { return dtype_; }
    constexpr Shape const& shape() const { return shape_; }
    constexpr Strides const& strides() const { return strides_; }
    std::ptrdiff_t offset() const { return 0; }

    Tensor forward(Context const& context) const {
        Tensor target(dtype_, shape_);
        std::apply([&](auto const&... operand) { this->operation.forward(Tensor(operand.forward(context))..., target); }, this->operands);
        return target;
    }

private:
    type dtype_;
    Shape shape_;
    Strides strides_;
};

struct Conversion {
    type to;
    constexpr type result(type) const { return to; }
    void forward(Tensor const& input, Tensor& target) const {
        on_device({&input}, target, "cast", [&](stream_t s) { return tannic_hip::cast(get_tensor(input.id()), get_tensor(target.id()), s); });
    }
};

struct RootMeanSquareNorm {
    float epsilon;
    constexpr type result(type dtype) const { return dtype; }
    void forward(Tensor const& input, Tensor const& gain, Tensor& target) const {
        on_device({&input, &gain}, target, "rms_norm", [&](stream_t s) { return tannic_hip::rms_norm(get_tensor(input.id()), get_tensor(gain.id()), get_tensor(target.id()), s, epsilon); });
    }
};

struct Softmax {
    float scale;
    constexpr type result(type dtype) const { return dtype; }
    void forward(Tensor const& input, Tensor& target) const {
        on_device({&input}, target, "softmax", [&](stream_t s) { return tannic_hip::softmax(get_tensor(input.id()), nullptr, get_tensor(target.id()), s, scale); });
    }
    void forward(Tensor const& input, Tensor const& mask, Tensor& target) const {
        on_device({&input, &mask}, target, "softmax", [&](stream_t s) { return tannic_hip::softmax(get_tensor(input.id()), get_tensor(mask.id()), get_tensor(target.id()), s, scale); });
    }
};

struct RotaryEmbedding {
    constexpr type result(type dtype) const { return dtype; }
    void forward(Tensor const& input, Tensor const& cosines, Tensor const& sines, Tensor& target) const {
        on_device({&input, &cosines, &sines}, target, "rope", [&](stream_t s) {
            return tannic_hip::rope(get_tensor(input.id()), get_tensor(cosines.id()), get_tensor(sines.id()), get_tensor(target.id()), s);
        });
    }
};

}  // namespace tannic::hip

namespace tannic {

// a / b with NumPy broadcasting; the floating pairs of `*`
template <Composable Dividend, Composable Divisor>
constexpr auto div(Dividend&& dividend, Divisor&& divisor) {
    return expression::Binary<hip::Division, Dividend, Divisor>{{}, std::forward<Dividend>(dividend), std::forward<Divisor>(divisor)};
}

// gate / (1 + exp(-gate)) * up
template <Composable Gate, Composable Up>
constexpr auto swiglu(Gate&& gate, Up&& up) {
    return expression::Binary<hip::GatedActivation, Gate, Up>{{}, std::forward<Gate>(gate), std::forward<Up>(up)};
}

// largest / smallest value along an axis (`-1` for the last); the reference has the positions only (argmax, argmin)
template <Composable Source>
constexpr auto max(Source&& source, int axis, bool keepdim = false) {
    return expression::Reduction<hip::Extreme<true>, Source>{{indexing::normalize(axis, source.shape().rank()), keepdim}, std::forward<Source>(source)};
}
template <Composable Source>
constexpr auto min(Source&& source, int axis, bool keepdim = false) {
    return expression::Reduction<hip::Extreme<false>, Source>{{indexing::normalize(axis, source.shape().rank()), keepdim}, std::forward<Source>(source)};
}

// the same values in another real dtype (float to integer truncates and saturates)
template <Composable Source>
constexpr auto cast(Source&& source, type dtype) {
    return hip::Rowwise<hip::Conversion, Source>{{dtype}, std::forward<Source>(source)};
}

// x / sqrt(mean(x^2 over the last axis) + epsilon) * gain
template <Composable Source, Composable Gain>
constexpr auto rms_norm(Source&& source, Gain&& gain, float epsilon) {
    return hip::Rowwise<hip::RootMeanSquareNorm, Source, Gain>{{epsilon}, std::forward<Source>(source), std::forward<Gain>(gain)};
}

// softmax over the last axis of scale * x (+ mask: a [Q, L] table added to every [.., Q, L] slab)
template <Composable Source>
constexpr auto softmax(Source&& source, float scale = 1.0f) {
    return hip::Rowwise<hip::Softmax, Source>{{scale}, std::forward<Source>(source)};
}
template <Composable Source, Composable Mask>
constexpr auto softmax(Source&& source, Mask&& mask, float scale = 1.0f) {
    return hip::Rowwise<hip::Softmax, Source, Mask>{{scale}, std::forward<Source>(source), std::forward<Mask>(mask)};
}

// rotary embedding of x [.., n, d] by cos, sin [n, d/2]: the pair (x[2i], x[2i+1]) turns by position n's angle
template <Composable Source, Composable Cosines, Composable Sines>
constexpr auto rope(Source&& source, Cosines&& cosines, Sines&& sines) {
    return hip::Rowwise<hip::RotaryEmbedding, Source, Cosines, Sines>{{}, std::forward<Source>(source), std::forward<Cosines>(cosines), std::forward<Sines>(sines)};
}

}  // namespace tannic

// bnn::Layer (dabnn/layer.h:24-38): a named step of the network; forward()
// wraps forward_impl() and, when the net profiles, times it with HIP events
// and accumulates per layer type (the reference's BNN_BENCHMARK mode,
// dabnn/layer.cpp:16-32).
#pragma once

#include <memory>
#include <string>

#include "mat.h"

namespace bnn {

class Net;

class BNN_API Layer {
   protected:
    using NetCP = const std::weak_ptr<Net>;
    using MatCP = const std::shared_ptr<Mat>;
    using MatP = std::shared_ptr<Mat>;
    MatP mat(const std::string &name) const;
    void *stream() const;

   public:
    Layer(NetCP net, const std::string &name, const std::string &type) : net_(net), name_(name), type_(type) {}
    virtual ~Layer();

    NetCP net_;
    void forward();
    virtual void forward_impl() const = 0;
    virtual std::string to_str() const;

    std::string name_;
    std::string type_;
};

// BNN_ASSERT of the reference throws std::runtime_error (common/helper.h:69-77).
[[noreturn]] BNN_API void bnn_fail(const std::string &msg);
#define BNN_ASSERT(cond, msg)                    \
    do {                                         \
        if (!(cond)) ::bnn::bnn_fail(msg);       \
    } while (0)
// A failed C-ABI call becomes the same exception type.
BNN_API void dab_check(int rc);

}  // namespace bnn

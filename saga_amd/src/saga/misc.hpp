// -*-c++-*-
// Small utilities of the public API.  (reference: saga.hpp:590-615)
#pragma once

#include "tensor.hpp"

namespace saga {

class Publisher {
public:
    virtual ~Publisher(){};

    virtual void publish(const char *id, Tensor &t, const Dims &offset, TensorAccess *ta) = 0;

    virtual void sync() = 0;
};

std::shared_ptr<Publisher> make_tcp_publisher(int bind_port);

// monotonic microseconds
int64_t now();

std::string fmt(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

struct Barrier {
    virtual ~Barrier(){};

    virtual void wait() = 0;

    static std::shared_ptr<Barrier> make(size_t count);
};

}  // namespace saga

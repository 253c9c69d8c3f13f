// -*-c++-*-
// Engine registry: a backend registers a factory from a static constructor.
// (reference: src/engine.hpp:6-8)
#pragma once

#include <memory>

#include "saga.hpp"

namespace saga {

void registerEngineFactory(const char *name, std::shared_ptr<Engine> (*fn)(const std::shared_ptr<UI> &ui));

}  // namespace saga

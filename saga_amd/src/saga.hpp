// -*-c++-*-
// Public API of the Saga front end as built in this repository.
//
// Source compatible with the interface of the reference library (its saga.hpp): the same
// namespace, class names, members and signatures, so that programs written against the
// reference - and the hip engine in src/hip - compile against either header.  The
// declarations live in topic headers under saga/.
#pragma once

#include "saga/dims.hpp"
#include "saga/tensor.hpp"
#include "saga/graph.hpp"
#include "saga/program.hpp"
#include "saga/misc.hpp"

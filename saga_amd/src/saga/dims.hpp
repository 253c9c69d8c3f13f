// -*-c++-*-
// Dimensions and node attributes.  (reference: saga.hpp:50-116)
#pragma once

#include <assert.h>
#include <stdint.h>

#include <functional>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <variant>
#include <vector>

namespace saga {

class Context;

// Symbolic extents: resolved when a program is built (BATCH_SIZE) or when a reshape node
// infers its output (UNCHANGED keeps the input extent, REDUCE folds all remaining ones).
enum class DimParam {
    BATCH_SIZE,
    UNCHANGED,
    REDUCE,
};

struct Dim : public std::variant<int64_t, DimParam> {
    using std::variant<int64_t, DimParam>::variant;

    std::string to_string() const;

    operator int() const
    {
        const int64_t *v = std::get_if<int64_t>(&*this);
        if(v == nullptr)
            throw std::runtime_error("Unable to convert parameterized dim to scalar");
        return (int)*v;
    }

    Dim &operator++();
    Dim &operator+=(const Dim &);
};

class Dims : public std::vector<Dim> {
    using std::vector<Dim>::vector;

public:
    Dims(const std::vector<Dim> &v) : std::vector<Dim>(v) {}
    Dims(const std::vector<int> &v);

    // replaces every BATCH_SIZE extent by v
    Dims batch(int64_t v) const;
    std::vector<int64_t> i64() const;
    std::vector<int32_t> i32() const;
    // product of the extents from from_rank on
    size_t elements(size_t from_rank = 0) const;
    std::string to_string() const;
    // equal after leading extents of 1 are dropped on both sides
    bool similar(const Dims &) const;

    Dims transform(std::function<Dim(const DimParam &dp, size_t i)> fn) const;
};

struct Attribute : public std::variant<float, int, std::vector<int>, bool, Dims> {
    using std::variant<float, int, std::vector<int>, bool, Dims>::variant;

    std::string to_string() const;
};

class Attributes : public std::unordered_map<std::string, Attribute> {
public:
    using std::unordered_map<std::string, Attribute>::unordered_map;

    // value of attribute n when present AND of type T, else def
    template <typename T> T get(const std::string &n, T def) const
    {
        auto it = find(n);
        if(it == end())
            return def;
        const T *p = std::get_if<T>(&it->second);
        return p ? *p : def;
    }
};

}  // namespace saga

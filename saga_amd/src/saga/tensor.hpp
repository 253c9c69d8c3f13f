// -*-c++-*-
// Tensors as the front end sees them.  (reference: saga.hpp:121-264)
#pragma once

#include "dims.hpp"

namespace saga {

enum class TensorLayout {
    Auto,
    NHWC,
    NCHW,
};

class Tensors;

// Host-side window onto a tensor's elements.  Element coordinates are logical (N,C,H,W);
// strides() tells how they map onto data().
class TensorAccess {
protected:
    TensorAccess(){};

public:
    virtual ~TensorAccess(){};
    virtual Dims strides() = 0;
    virtual void *data() = 0;

    virtual void copyBytesFrom(const Dims &element, const void *data, size_t size) = 0;

    virtual void *getAddr(const Dims &element) { return nullptr; }
    virtual double get(const Dims &element) = 0;
    virtual void set(const Dims &element, double value) = 0;

    TensorAccess(TensorAccess const &) = delete;
    TensorAccess &operator=(TensorAccess const &) = delete;
};

class Tensor {
public:
    Tensor &operator=(Tensor const &) = delete;
    Tensor(Tensor const &) = delete;

    struct Stats {
        double min;
        double max;
        double mean;
        double stddev;
    };

    enum class DataType {
        U8,
        HALF,
        FLOAT,
        INT64,
        I32,
        I16,
    };

    static size_t DataTypeSize(DataType dt);
    static const char *DataTypeStr(DataType dt);

    virtual ~Tensor(){};

    virtual std::string info() const;

    // nullptr for tensors without backing store (pure placeholders)
    virtual std::unique_ptr<TensorAccess> access() { return nullptr; }

    virtual std::shared_ptr<Tensor> slice(const Dims &offset, const Dims &size);

    // the gradient placeholder paired with this tensor, created on demand
    virtual std::shared_ptr<Tensor> grad(bool create = true);

    // inverse of grad()
    virtual std::shared_ptr<Tensor> value() const;

    virtual void copyFrom(Tensor &t);

    // sum of squared element differences, iterating logical coordinates (layout agnostic)
    double sse(Tensor &t);

    static std::shared_ptr<Tensor> loadProtoBuf(const char *path);

    static std::shared_ptr<Tensor> load(const char *path, const std::optional<const std::string> &name);
    bool save(const char *path);

    // named lookup in named_tensors, else a generated (random normal) tensor
    static std::shared_ptr<Tensor> find(Tensor::DataType data_type, const Dims &size, double init_mean,
                                        double init_stddev, Tensors &named_tensors,
                                        const std::optional<const std::string> &name = std::nullopt);

    static std::shared_ptr<Tensor> make(Tensor::DataType data_type, const Dims &size, double init_mean,
                                        double init_stddev);

    std::shared_ptr<Tensor> toRGB(std::optional<std::pair<float, float>> range = std::nullopt);
    void print(const char *prefix, int elements_per_rank = 0);
    void print_anomaly(const char *prefix);
    void printRGB(const char *prefix, std::optional<std::pair<float, float>> range = std::nullopt);
    virtual Stats stats();
    void printStats(const char *prefix);
    std::string statsString(void);

    std::optional<const std::string> namePostfix(const std::string &postfix) const;

    const std::optional<const std::string> m_name;
    const DataType m_data_type;
    const Dims m_dims;

protected:
    Tensor(DataType data_type, const Dims &size, const std::optional<const std::string> &name = std::nullopt);
};

// row-major host tensor with storage
std::shared_ptr<Tensor> makeCPUTensor(Tensor::DataType data_type, const Dims &size,
                                      const std::optional<const std::string> &name = std::nullopt);

// placeholder without storage
std::shared_ptr<Tensor> makeTensor(Tensor::DataType data_type, const Dims &size,
                                   const std::optional<const std::string> &name = std::nullopt);

class Tensors : public std::unordered_map<std::string, std::shared_ptr<Tensor>> {
public:
    using std::unordered_map<std::string, std::shared_ptr<Tensor>>::unordered_map;

    bool has(const std::string &n) const;

    const std::shared_ptr<Tensor> operator[](const std::string &n) const;

    std::shared_ptr<Tensor> &operator[](const std::string &n);

    // x0, x1, ... until the first missing index
    std::vector<std::shared_ptr<Tensor>> getv(const std::string &n) const
    {
        std::vector<std::shared_ptr<Tensor>> v;
        for(int i = 0;; i++) {
            auto it = find(n + std::to_string(i));
            if(it == end())
                break;
            v.push_back(it->second);
        }
        return v;
    }

    void loadTensors(const char *path);

    bool saveTensors(const char *path, Context *ctx);
};

}  // namespace saga

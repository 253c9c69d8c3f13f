// Front-end tensors: dimension arithmetic, host tensors, placeholders with their gradient
// twins, generated (randomly initialised) tensors, comparison, statistics and the on-disk
// format.  Behaviour follows the reference's src/tensor.cpp (cited per function); the code
// is written for this repository.
#include <errno.h>
#include <fcntl.h>
#include <inttypes.h>
#include <limits.h>
#include <math.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <mutex>
#include <random>
#include <sstream>

#include "hosttensor.hpp"

namespace saga {

// ---------------------------------------------------------------- Dim / Dims

Dims::Dims(const std::vector<int> &v)
{
    reserve(v.size());
    for(int e : v)
        push_back((int64_t)e);
}

static int64_t &scalar_of(Dim &d, const char *what)
{
    int64_t *v = std::get_if<int64_t>(&d);
    if(v == nullptr) {
        fprintf(stderr, "Unable to %s parameterized dim\n", what);
        abort();
    }
    return *v;
}

Dim &Dim::operator++()
{
    scalar_of(*this, "++")++;
    return *this;
}

Dim &Dim::operator+=(const Dim &rhs)
{
    scalar_of(*this, "+=") += (int)rhs;
    return *this;
}

std::string Dim::to_string() const
{
    if(auto v = std::get_if<int64_t>(this))
        return std::to_string(*v);
    switch(std::get<DimParam>(*this)) {
    case DimParam::BATCH_SIZE: return "N";
    case DimParam::UNCHANGED: return "=";
    case DimParam::REDUCE: return "R";
    }
    return "?";
}

std::vector<int64_t> Dims::i64() const
{
    std::vector<int64_t> r;
    r.reserve(size());
    for(const Dim &d : *this) {
        auto v = std::get_if<int64_t>(&d);
        if(!v) {
            fprintf(stderr, "Unable to convert parameterized dim to vector<int>\n");
            abort();
        }
        r.push_back(*v);
    }
    return r;
}

std::vector<int32_t> Dims::i32() const
{
    std::vector<int32_t> r;
    for(int64_t v : i64())
        r.push_back((int32_t)v);
    return r;
}

Dims Dims::transform(std::function<Dim(const DimParam &dp, size_t i)> fn) const
{
    Dims r;
    for(size_t i = 0; i < size(); i++) {
        const Dim &d = (*this)[i];
        if(auto p = std::get_if<DimParam>(&d))
            r.push_back(fn(*p, i));
        else
            r.push_back(d);
    }
    return r;
}

// reference: src/tensor.cpp:133-139
Dims Dims::batch(int64_t n) const
{
    return transform([n](const DimParam &dp, size_t) { return dp == DimParam::BATCH_SIZE ? Dim(n) : Dim(dp); });
}

size_t Dims::elements(size_t from_rank) const
{
    size_t n = 1;
    for(size_t i = from_rank; i < size(); i++)
        n *= (size_t)(int)(*this)[i];
    return n;
}

std::string Dims::to_string() const
{
    std::string r = "[";
    for(size_t i = 0; i < size(); i++) {
        if(i)
            r += ", ";
        r += (*this)[i].to_string();
    }
    return r + "]";
}

// reference: src/tensor.cpp:184-201
bool Dims::similar(const Dims &o) const
{
    size_t a = 0, b = 0;
    while(a < size() && (*this)[a] == Dim((int64_t)1))
        a++;
    while(b < o.size() && o[b] == Dim((int64_t)1))
        b++;
    if(size() - a != o.size() - b)
        return false;
    for(; a < size(); a++, b++)
        if(!((*this)[a] == o[b]))
            return false;
    return true;
}

// ---------------------------------------------------------------- Tensor base

Tensor::Tensor(DataType data_type, const Dims &size, const std::optional<const std::string> &name)
  : m_name(name), m_data_type(data_type), m_dims(size)
{
}

size_t Tensor::DataTypeSize(DataType dt)
{
    switch(dt) {
    case DataType::U8: return 1;
    case DataType::HALF: return 2;
    case DataType::FLOAT: return 4;
    case DataType::INT64: return 8;
    case DataType::I32: return 4;
    case DataType::I16: return 2;
    }
    throw std::runtime_error("DataTypeSize: bad data type");
}

const char *Tensor::DataTypeStr(DataType dt)
{
    switch(dt) {
    case DataType::U8: return "u8";
    case DataType::HALF: return "half";
    case DataType::FLOAT: return "float";
    case DataType::INT64: return "i64";
    case DataType::I32: return "i32";
    case DataType::I16: return "i16";
    }
    return "?";
}

std::string Tensor::info() const
{
    std::string r = m_name ? "\"" + *m_name + "\"" : std::string();
    r += "<";
    r += DataTypeStr(m_data_type);
    r += ">";
    r += m_dims.to_string();
    return r;
}

std::shared_ptr<Tensor> Tensor::slice(const Dims &, const Dims &)
{
    throw std::runtime_error("slice() is not supported by this tensor: " + info());
}

std::shared_ptr<Tensor> Tensor::grad(bool) { return nullptr; }

std::shared_ptr<Tensor> Tensor::value() const { return nullptr; }

std::optional<const std::string> Tensor::namePostfix(const std::string &postfix) const
{
    if(!m_name)
        return std::nullopt;
    return *m_name + "." + postfix;
}

// Element-wise copy in logical coordinates; a source of lower rank or with extents of 1 is
// broadcast (reference: copy_tensor, src/tensor.cpp:715-966).
void Tensor::copyFrom(Tensor &t)
{
    auto dst = access();
    auto src = t.access();
    if(!dst || !src)
        throw std::runtime_error("copyFrom: tensor without storage (" + t.info() + " -> " + info() + ")");
    const size_t dr = m_dims.size(), sr = t.m_dims.size();
    if(sr > dr && t.m_dims.elements() != m_dims.elements())
        throw std::runtime_error("copyFrom: incompatible shapes " + t.info() + " -> " + info());
    const std::vector<int64_t> sext = t.m_dims.i64();
    if(sr <= dr) {
        for_each_coordinate(m_dims, [&](const Dims &c, size_t) {
            Dims sc(sr, (int64_t)0);
            for(size_t i = 0; i < sr; i++) {
                const int64_t v = (int)c[dr - sr + i];
                sc[i] = sext[i] == 1 ? (int64_t)0 : v;
            }
            dst->set(c, src->get(sc));
        });
    } else {
        // same element count, different rank: pair elements in row-major order
        std::vector<double> tmp(m_dims.elements());
        for_each_coordinate(t.m_dims, [&](const Dims &c, size_t i) { tmp[i] = src->get(c); });
        for_each_coordinate(m_dims, [&](const Dims &c, size_t i) { dst->set(c, tmp[i]); });
    }
}

// reference: src/tensor.cpp:983-1024
double Tensor::sse(Tensor &t)
{
    auto a = t.access();
    auto b = access();
    if(!a && !b)
        return 0.0;
    if(!a || !b)
        return INFINITY;
    assert(m_dims.elements() == t.m_dims.elements());
    std::vector<double> other(t.m_dims.elements());
    for_each_coordinate(t.m_dims, [&](const Dims &c, size_t i) { other[i] = a->get(c); });
    double r = 0;
    for_each_coordinate(m_dims, [&](const Dims &c, size_t i) {
        const double d = other[i] - b->get(c);
        r += d * d;
    });
    return r;
}

Tensor::Stats Tensor::stats()
{
    auto ta = access();
    if(!ta)
        return Stats{0, 0, 0, 0};
    double mn = INFINITY, mx = -INFINITY, sum = 0, sq = 0;
    const double n = (double)m_dims.elements();
    for_each_coordinate(m_dims, [&](const Dims &c, size_t) {
        const double v = ta->get(c);
        mn = std::min(mn, v);
        mx = std::max(mx, v);
        sum += v;
        sq += v * v;
    });
    const double mean = sum / n;
    const double var = std::max(0.0, sq / n - mean * mean);
    return Stats{mn, mx, mean, sqrt(var)};
}

std::string Tensor::statsString(void)
{
    const Stats s = stats();
    return fmt("{min:%f mean:%f max:%f stddev:%f}", s.min, s.mean, s.max, s.stddev);
}

void Tensor::printStats(const char *prefix) { printf("%s: %s\n", prefix, statsString().c_str()); }

void Tensor::print(const char *prefix, int elements_per_rank)
{
    printf("%s: %s\n", prefix, info().c_str());
    auto ta = access();
    if(!ta) {
        printf("%s: (no storage)\n", prefix);
        return;
    }
    const size_t rank = m_dims.size();
    const int64_t last = rank ? (int64_t)(int)m_dims[rank - 1] : 1;
    for_each_coordinate(m_dims, [&](const Dims &c, size_t) {
        if(elements_per_rank > 0)
            for(size_t i = 0; i < rank; i++)
                if((int)c[i] >= elements_per_rank)
                    return;
        const int64_t col = rank ? (int64_t)(int)c[rank - 1] : 0;
        if(col == 0) {
            printf("%s: ", prefix);
            for(size_t i = 0; i + 1 < rank; i++)
                printf("%s%d", i ? "," : "[", (int)c[i]);
            printf("%s ", rank > 1 ? "]" : "");
        }
        printf("% 1.6f ", ta->get(c));
        if(col == last - 1 || (elements_per_rank > 0 && col == elements_per_rank - 1))
            printf("\n");
    });
}

void Tensor::print_anomaly(const char *prefix)
{
    auto ta = access();
    if(!ta)
        return;
    int shown = 0;
    for_each_coordinate(m_dims, [&](const Dims &c, size_t) {
        const double v = ta->get(c);
        if(!std::isfinite(v) && shown < 16) {
            printf("%s: %s at %s\n", prefix, std::isnan(v) ? "NaN" : "Inf", c.to_string().c_str());
            shown++;
        }
    });
}

std::shared_ptr<Tensor> Tensor::toRGB(std::optional<std::pair<float, float>>)
{
    throw std::runtime_error("toRGB: image debugging helpers are not part of this build");
}

void Tensor::printRGB(const char *, std::optional<std::pair<float, float>>)
{
    throw std::runtime_error("printRGB: image debugging helpers are not part of this build");
}

// ---------------------------------------------------------------- placeholders + autograd link

static std::mutex g_autograd_mutex;

// A tensor without storage that can own a gradient twin (reference: EmptyTensor,
// src/tensor.cpp:1036-1068).
class PlaceholderTensor : public Tensor, public std::enable_shared_from_this<PlaceholderTensor> {
public:
    PlaceholderTensor(DataType dt, const Dims &size, const std::optional<const std::string> &name = std::nullopt)
      : Tensor(dt, size, name)
    {
    }

    std::shared_ptr<Tensor> grad(bool create) override
    {
        std::lock_guard<std::mutex> lk(g_autograd_mutex);
        if(!m_grad && create) {
            m_grad = std::make_shared<PlaceholderTensor>(m_data_type, m_dims, namePostfix("grad"));
            m_grad->m_owner = shared_from_this();
        }
        return m_grad;
    }

    std::shared_ptr<Tensor> value() const override
    {
        std::lock_guard<std::mutex> lk(g_autograd_mutex);
        return m_owner.lock();
    }

private:
    std::shared_ptr<PlaceholderTensor> m_grad;
    std::weak_ptr<PlaceholderTensor> m_owner;
};

std::shared_ptr<Tensor> makeTensor(Tensor::DataType data_type, const Dims &size,
                                   const std::optional<const std::string> &name)
{
    return std::make_shared<PlaceholderTensor>(data_type, size, name);
}

// ---------------------------------------------------------------- generated tensors

// Access object of a tensor whose values are drawn from N(mean, stddev) on every read;
// data() is null, which tells a backend that the tensor was auto-initialised
// (reference: GenTensorAccess, src/tensor.cpp:1079-1107; seeded from the clock there too).
class RandomAccess : public TensorAccess {
public:
    RandomAccess(size_t rank, double mean, double stddev) : m_rank(rank), m_mean(mean), m_dist(mean, stddev)
    {
        m_rng.seed((unsigned long)now());
        m_const = stddev == 0;
    }
    Dims strides() override { return Dims(m_rank, (int64_t)0); }
    void *data() override { return nullptr; }
    double get(const Dims &) override { return m_const ? m_mean : m_dist(m_rng); }
    void set(const Dims &, double) override {}
    void copyBytesFrom(const Dims &, const void *, size_t) override {}

private:
    const size_t m_rank;
    const double m_mean;
    bool m_const;
    std::normal_distribution<double> m_dist;
    std::default_random_engine m_rng;
};

class GeneratedTensor : public PlaceholderTensor {
public:
    GeneratedTensor(DataType dt, const Dims &size, const std::optional<const std::string> &name, double mean,
                    double stddev)
      : PlaceholderTensor(dt, size, name), m_mean(mean), m_stddev(stddev)
    {
    }
    std::unique_ptr<TensorAccess> access() override
    {
        return std::make_unique<RandomAccess>(m_dims.size(), m_mean, m_stddev);
    }
    std::shared_ptr<Tensor> slice(const Dims &, const Dims &size) override
    {
        return std::make_shared<GeneratedTensor>(m_data_type, size, m_name, m_mean, m_stddev);
    }
    std::string info() const override
    {
        return Tensor::info() + fmt("(mean:%g, stddev:%g)", m_mean, m_stddev);
    }

private:
    const double m_mean, m_stddev;
};

// reference: src/tensor.cpp:1142-1188
std::shared_ptr<Tensor> Tensor::find(Tensor::DataType data_type, const Dims &size, double init_mean,
                                     double init_stddev, Tensors &named_tensors,
                                     const std::optional<const std::string> &name)
{
    if(name) {
        auto it = named_tensors.find(*name);
        if(it != named_tensors.end()) {
            auto t = it->second;
            if(t->m_data_type != data_type) {
                fprintf(stderr, "Pre-initialized tensor %s datatype mismatch: Loaded:%s != Requested:%s\n",
                        name->c_str(), DataTypeStr(t->m_data_type), DataTypeStr(data_type));
                exit(1);
            }
            if(!t->m_dims.similar(size)) {
                fprintf(stderr, "Pre-initialized tensor %s dimensions mismatch: Loaded:%s != Requested:%s\n",
                        name->c_str(), t->m_dims.to_string().c_str(), size.to_string().c_str());
                exit(1);
            }
            return t;
        }
    }
    auto t = std::make_shared<GeneratedTensor>(data_type, size, name, init_mean, init_stddev);
    if(name)
        named_tensors[*name] = t;
    return t;
}

std::shared_ptr<Tensor> Tensor::make(Tensor::DataType data_type, const Dims &size, double init_mean,
                                     double init_stddev)
{
    return std::make_shared<GeneratedTensor>(data_type, size, std::nullopt, init_mean, init_stddev);
}

// ---------------------------------------------------------------- host tensors

// Malloc'ed or memory-mapped bytes shared by a CPU tensor and its slices.
struct HostBuffer {
    void *data = nullptr;
    void *map = nullptr;
    size_t map_size = 0;
    ~HostBuffer()
    {
        if(map)
            munmap(map, map_size);
        else
            free(data);
    }
};

class HostAccess : public TensorAccess {
public:
    HostAccess(Tensor::DataType dt, const std::vector<int64_t> &strides, std::shared_ptr<HostBuffer> buf, int64_t offset)
      : m_dt(dt), m_strides(strides), m_buf(buf), m_offset(offset)
    {
    }
    Dims strides() override
    {
        Dims d;
        for(auto s : m_strides)
            d.push_back(s);
        return d;
    }
    void *data() override
    {
        assert(m_offset == 0);
        return m_buf->data;
    }
    size_t index(const Dims &e) const
    {
        int64_t o = m_offset;
        for(size_t i = 0; i < e.size() && i < m_strides.size(); i++)
            o += (int64_t)(int)e[i] * m_strides[i];
        return (size_t)o;
    }
    double get(const Dims &e) override { return load_element(m_buf->data, m_dt, index(e)); }
    void set(const Dims &e, double v) override { store_element(m_buf->data, m_dt, index(e), v); }
    void *getAddr(const Dims &e) override { return (char *)m_buf->data + index(e) * Tensor::DataTypeSize(m_dt); }
    void copyBytesFrom(const Dims &e, const void *src, size_t size) override { memcpy(getAddr(e), src, size); }

private:
    const Tensor::DataType m_dt;
    const std::vector<int64_t> m_strides;
    const std::shared_ptr<HostBuffer> m_buf;
    const int64_t m_offset;
};

static std::vector<int64_t> row_major_strides(const Dims &dims)
{
    std::vector<int64_t> s(dims.size());
    int64_t acc = 1;
    for(ssize_t i = (ssize_t)dims.size() - 1; i >= 0; i--) {
        s[i] = acc;
        acc *= (int)dims[i];
    }
    return s;
}

// reference: CPUTensor, src/tensor.cpp:1300-1377
class HostTensor : public PlaceholderTensor {
public:
    HostTensor(DataType dt, const Dims &size, const std::optional<const std::string> &name)
      : PlaceholderTensor(dt, size, name), m_strides(row_major_strides(size)), m_buf(std::make_shared<HostBuffer>())
    {
        m_buf->data = calloc(std::max<size_t>(size.elements(), 1), DataTypeSize(dt));
    }
    HostTensor(DataType dt, const Dims &size, const std::vector<int64_t> &strides, std::shared_ptr<HostBuffer> buf,
               int64_t offset, const std::optional<const std::string> &name)
      : PlaceholderTensor(dt, size, name), m_strides(strides), m_buf(buf), m_offset(offset)
    {
    }
    std::unique_ptr<TensorAccess> access() override
    {
        return std::make_unique<HostAccess>(m_data_type, m_strides, m_buf, m_offset);
    }
    std::shared_ptr<Tensor> slice(const Dims &offset, const Dims &size) override
    {
        int64_t o = m_offset;
        for(size_t i = 0; i < offset.size() && i < m_strides.size(); i++)
            o += (int64_t)(int)offset[i] * m_strides[i];
        return std::make_shared<HostTensor>(m_data_type, size, m_strides, m_buf, o, namePostfix("slice"));
    }
    std::string info() const override
    {
        std::string r = Tensor::info() + "{";
        for(size_t i = 0; i < m_strides.size(); i++)
            r += (i ? ", " : "") + std::to_string(m_strides[i]);
        return r + "}";
    }

private:
    const std::vector<int64_t> m_strides;
    const std::shared_ptr<HostBuffer> m_buf;
    const int64_t m_offset = 0;
};

std::shared_ptr<Tensor> makeCPUTensor(Tensor::DataType data_type, const Dims &size,
                                      const std::optional<const std::string> &name)
{
    return std::make_shared<HostTensor>(data_type, size, name);
}

// ---------------------------------------------------------------- disk format "sagaT001"
// 8-byte magic, u32 type (0 float, 1 half), u32 rank, rank x u32 extents, row-major payload
// (reference: src/tensor.cpp:1382-1550).

struct DiskHeader {
    uint8_t magic[8];
    uint32_t type;
    uint32_t rank;
} __attribute__((packed));

std::shared_ptr<Tensor> Tensor::load(const char *path, const std::optional<const std::string> &name)
{
    const int fd = open(path, O_RDONLY);
    if(fd == -1) {
        fprintf(stderr, "Unable to open %s -- %s\n", path, strerror(errno));
        return nullptr;
    }
    struct stat st;
    if(fstat(fd, &st) || (size_t)st.st_size < sizeof(DiskHeader)) {
        fprintf(stderr, "Unable to load %s -- Not a saga tensor file\n", path);
        close(fd);
        return nullptr;
    }
    void *mem = mmap(NULL, st.st_size, PROT_READ, MAP_SHARED, fd, 0);
    close(fd);
    if(mem == MAP_FAILED) {
        fprintf(stderr, "Unable to load %s -- Out of memory\n", path);
        return nullptr;
    }
    auto buf = std::make_shared<HostBuffer>();
    buf->map = mem;
    buf->map_size = st.st_size;
    const DiskHeader *h = (const DiskHeader *)mem;
    if(memcmp(h->magic, "sagaT001", 8)) {
        fprintf(stderr, "Unable to load %s -- Not a saga tensor file\n", path);
        return nullptr;
    }
    if(h->type > 1) {
        fprintf(stderr, "Unable to load %s -- Unsupported data type:%u\n", path, h->type);
        return nullptr;
    }
    const DataType dt = h->type == 0 ? DataType::FLOAT : DataType::HALF;
    if(h->rank > 8 || (size_t)st.st_size < sizeof(DiskHeader) + h->rank * sizeof(uint32_t)) {
        fprintf(stderr, "Unable to load %s -- Bad rank or file too short\n", path);
        return nullptr;
    }
    const uint32_t *ext = (const uint32_t *)((const char *)mem + sizeof(DiskHeader));
    Dims dims;
    for(uint32_t i = 0; i < h->rank; i++)
        dims.push_back((int64_t)ext[i]);
    const size_t payload = sizeof(DiskHeader) + h->rank * sizeof(uint32_t);
    if((size_t)st.st_size < payload + dims.elements() * DataTypeSize(dt)) {
        fprintf(stderr, "Unable to load %s -- File too short\n", path);
        return nullptr;
    }
    buf->data = (char *)mem + payload;
    return std::make_shared<HostTensor>(dt, dims, row_major_strides(dims), buf, 0, name);
}

bool Tensor::save(const char *path)
{
    DiskHeader h;
    memcpy(h.magic, "sagaT001", 8);
    if(m_data_type == DataType::FLOAT)
        h.type = 0;
    else if(m_data_type == DataType::HALF)
        h.type = 1;
    else {
        fprintf(stderr, "Unable to save %s -- Unsupported data type:%d\n", path, (int)m_data_type);
        return false;
    }
    h.rank = m_dims.size();
    HostTensor copy(m_data_type, m_dims, std::nullopt);
    copy.copyFrom(*this);
    auto ta = copy.access();
    std::vector<uint32_t> ext;
    for(auto v : m_dims.i64())
        ext.push_back((uint32_t)v);
    const std::string tmp = std::string(path) + ".tmp";
    const int fd = open(tmp.c_str(), O_CREAT | O_TRUNC | O_WRONLY, 0644);
    if(fd == -1) {
        fprintf(stderr, "Unable to save %s -- %s\n", path, strerror(errno));
        return false;
    }
    const size_t bytes = m_dims.elements() * DataTypeSize(m_data_type);
    const bool ok = write(fd, &h, sizeof(h)) == (ssize_t)sizeof(h) &&
                    write(fd, ext.data(), ext.size() * 4) == (ssize_t)(ext.size() * 4) &&
                    write(fd, ta->data(), bytes) == (ssize_t)bytes;
    close(fd);
    if(!ok || rename(tmp.c_str(), path) == -1) {
        fprintf(stderr, "Unable to save %s -- %s\n", path, strerror(errno));
        unlink(tmp.c_str());
        return false;
    }
    return true;
}

}  // namespace saga

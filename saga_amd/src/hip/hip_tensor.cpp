// Device tensors, storages and host access for the hip engine
// (role of the reference's src/cuda/cuda_tensor.cpp).  Device memory is plain hipMalloc
// memory; the host sees it through explicit staging copies instead of managed memory, and
// batched tensors through pinned double buffers.
#include <immintrin.h>
#include <math.h>
#include <string.h>

#include <sstream>

#include "hip_common.hpp"

namespace saga {

// ---------------------------------------------------------------- memory

HipMemory::HipMemory(size_t bytes) : m_bytes(bytes)
{
    chkHip(hipMalloc(&m_ptr, std::max<size_t>(bytes, 256)));
    chkHip(hipMemset(m_ptr, 0, std::max<size_t>(bytes, 256)));
}

HipMemory::~HipMemory()
{
    if(m_ptr)
        (void)hipFree(m_ptr);
}

void HipScratch::alloc()
{
    if(m_mem && m_mem->m_bytes >= m_requested)
        return;
    m_mem = std::make_shared<HipMemory>(std::max<size_t>(m_requested, 4096));
}

HipStorage::HipStorage(Tensor::DataType dt, size_t elements, HipContext *ctx)
  : m_ctx(ctx)
  , m_data_type(dt)
  , m_elements(elements)
  , m_element_size(Tensor::DataTypeSize(dt))
  , m_id(ctx ? ctx->m_storage_id_gen++ : -1)
{
}

void HipStorage::rehome(const std::shared_ptr<HipMemory> &mem, void *ptr)
{
    m_memory = mem;
    m_data = ptr;
    m_in_arena = false;
    if(m_ctx)
        m_ctx->m_mem_epoch++;
}

void HipStorage::allocOwn()
{
    auto mem = std::make_shared<HipMemory>(bytes()); // zero filled
    rehome(mem, mem->m_ptr);
}

HipDoubleBuffer::HipDoubleBuffer(Tensor::DataType dt, size_t elements, HipContext *ctx) : HipStorage(dt, elements, ctx)
{
    const size_t bytes = std::max<size_t>(elements * m_element_size, 256);
    for(int i = 0; i < 2; i++) {
        chkHip(hipMalloc(&m_dev[i], bytes));
        chkHip(hipMemset(m_dev[i], 0, bytes));
        chkHip(hipHostMalloc(&m_host[i], bytes, hipHostMallocDefault));
        memset(m_host[i], 0, bytes);
    }
}

HipDoubleBuffer::~HipDoubleBuffer()
{
    for(int i = 0; i < 2; i++) {
        (void)hipFree(m_dev[i]);
        (void)hipHostFree(m_host[i]);
    }
}

void HipDoubleBuffer::uploadBack(hipStream_t st)
{
    const int b = m_index ^ 1;
    chkHip(hipMemcpyAsync(m_dev[b], m_host[b], m_elements * m_element_size, hipMemcpyHostToDevice, st));
}

void HipDoubleBuffer::downloadFront(hipStream_t st)
{
    chkHip(hipMemcpyAsync(m_host[m_index], m_dev[m_index], m_elements * m_element_size, hipMemcpyDeviceToHost, st));
}

// ---------------------------------------------------------------- element codec (host side)

static inline double host_load(const void *base, Tensor::DataType dt, size_t i)
{
    switch(dt) {
    case Tensor::DataType::U8: return ((const uint8_t *)base)[i];
    case Tensor::DataType::HALF: return _cvtsh_ss(((const uint16_t *)base)[i]);
    case Tensor::DataType::FLOAT: return ((const float *)base)[i];
    case Tensor::DataType::INT64: return (double)((const int64_t *)base)[i];
    case Tensor::DataType::I32: return ((const int32_t *)base)[i];
    case Tensor::DataType::I16: return ((const int16_t *)base)[i];
    }
    return 0;
}

static inline void host_store(void *base, Tensor::DataType dt, size_t i, double v)
{
    switch(dt) {
    case Tensor::DataType::U8: ((uint8_t *)base)[i] = (uint8_t)v; break;
    case Tensor::DataType::HALF: ((uint16_t *)base)[i] = _cvtss_sh((float)v, _MM_FROUND_TO_NEAREST_INT); break;
    case Tensor::DataType::FLOAT: ((float *)base)[i] = (float)v; break;
    case Tensor::DataType::INT64: ((int64_t *)base)[i] = (int64_t)v; break;
    case Tensor::DataType::I32: ((int32_t *)base)[i] = (int32_t)v; break;
    case Tensor::DataType::I16: ((int16_t *)base)[i] = (int16_t)v; break;
    }
}

// ---------------------------------------------------------------- layout

std::vector<int64_t> hip_strides(const Dims &dims, HipLayout layout)
{
    const size_t rank = dims.size();
    std::vector<int64_t> s(rank, 1);
    if(rank == 4 && layout == HipLayout::NHWC) {
        const int64_t C = (int)dims[1], H = (int)dims[2], W = (int)dims[3];
        s[1] = 1;
        s[3] = C;
        s[2] = W * C;
        s[0] = H * W * C;
        return s;
    }
    int64_t acc = 1;
    for(ssize_t i = (ssize_t)rank - 1; i >= 0; i--) {
        s[i] = acc;
        acc *= (int)dims[i];
    }
    return s;
}

// ---------------------------------------------------------------- HipTensor

HipTensor::HipTensor(DataType dt, const Dims &dims, HipLayout layout, HipContext *ctx,
                     const std::optional<const std::string> &name)
  : Tensor(dt, dims, name), m_strides(hip_strides(dims, layout))
{
    m_storage = std::make_shared<HipStorage>(dt, dims.elements(), ctx);
}

HipTensor::HipTensor(std::shared_ptr<HipStorage> storage, const Dims &dims, const std::vector<int64_t> &strides,
                     int64_t offset, const std::optional<const std::string> &name)
  : Tensor(storage->m_data_type, dims, name), m_storage(storage), m_strides(strides), m_offset(offset)
{
}

HipTensor::HipTensor(DataType dt, const HipTensor &like, const std::optional<const std::string> &name)
  : Tensor(dt, like.m_dims, name), m_strides(like.m_strides)
{
    // dense re-creation of `like`'s layout (an alias with a wider pitch becomes packed)
    const bool nhwc = like.m_dims.size() == 4 && like.cpacked();
    m_strides = hip_strides(like.m_dims, nhwc ? HipLayout::NHWC : HipLayout::NCHW);
    m_storage = std::make_shared<HipStorage>(dt, like.m_dims.elements(), like.m_storage->m_ctx);
}

void *HipTensor::deviceMem() const
{
    return (char *)m_storage->deviceMem() + m_offset * (int64_t)m_storage->m_element_size;
}

bool HipTensor::cpacked() const { return m_dims.size() == 4 && ((int)m_dims[1] == 1 || m_strides[1] == 1); }

bool HipTensor::rowMajor() const
{
    int64_t acc = 1;
    for(ssize_t i = (ssize_t)m_dims.size() - 1; i >= 0; i--) {
        if((int)m_dims[i] > 1 && m_strides[i] != acc)
            return false;
        acc *= (int)m_dims[i];
    }
    return true;
}

SagaTensorView HipTensor::shapeView() const
{
    if(m_storage->allocated() || m_storage->doubleBuffered())
        return view();
    HipStorage *s = m_storage.get();
    void *const keep = s->m_data;
    s->m_data = (void *)(uintptr_t)4096; // aligned placeholder, never dereferenced
    SagaTensorView v = view();
    s->m_data = keep;
    return v;
}

SagaTensorView HipTensor::view() const
{
    SagaTensorView v;
    v.ptr = deviceMem();
    v.dtype = (int)m_data_type;
    const size_t rank = m_dims.size();
    for(int i = 0; i < 4; i++) {
        v.dims[i] = 1;
        v.strides[i] = 1;
    }
    if(rank == 1) { // parameter vector [C] -> [1, C, 1, 1]
        v.dims[1] = (int)m_dims[0];
        v.strides[1] = m_strides[0];
        v.strides[0] = (int64_t)v.dims[1] * m_strides[0];
        return v;
    }
    if(rank > 4)
        throw std::runtime_error("tensors of rank > 4 are not supported: " + info());
    for(size_t i = 0; i < rank; i++) {
        v.dims[i] = (int)m_dims[i];
        v.strides[i] = m_strides[i];
    }
    return v;
}

std::string HipTensor::shortname() const
{
    std::stringstream ss;
    ss << "T" << m_storage->m_id;
    if(m_offset)
        ss << "+" << m_offset;
    return ss.str();
}

std::string HipTensor::info() const
{
    std::stringstream ss;
    ss << Tensor::info() << "{";
    for(size_t i = 0; i < m_strides.size(); i++)
        ss << (i ? ", " : "") << m_strides[i];
    ss << "}@" << shortname();
    return ss.str();
}

// Host window: the whole storage is staged to the host when the access object is created and
// written back when it is destroyed after a set().
class HipStagedAccess : public TensorAccess {
public:
    HipStagedAccess(HipTensor &t) : m_t(t), m_storage(t.m_storage)
    {
        m_bytes = m_storage->m_elements * m_storage->m_element_size;
        m_host = malloc(std::max<size_t>(m_bytes, 16));
        if(m_storage->m_ctx)
            m_storage->m_ctx->sync();
        chkHip(hipMemcpy(m_host, m_storage->deviceMem(), m_bytes, hipMemcpyDeviceToHost));
    }
    ~HipStagedAccess()
    {
        if(m_dirty) {
            chkHip(hipMemcpy(m_storage->deviceMem(), m_host, m_bytes, hipMemcpyHostToDevice));
        }
        free(m_host);
    }
    Dims strides() override
    {
        Dims d;
        for(auto s : m_t.m_strides)
            d.push_back(s);
        return d;
    }
    void *data() override { return (char *)m_host + m_t.m_offset * (int64_t)m_storage->m_element_size; }
    size_t index(const Dims &e) const
    {
        int64_t o = m_t.m_offset;
        for(size_t i = 0; i < e.size() && i < m_t.m_strides.size(); i++)
            o += (int64_t)(int)e[i] * m_t.m_strides[i];
        return (size_t)o;
    }
    double get(const Dims &e) override { return host_load(m_host, m_storage->m_data_type, index(e)); }
    void set(const Dims &e, double v) override
    {
        host_store(m_host, m_storage->m_data_type, index(e), v);
        m_dirty = true;
    }
    void *getAddr(const Dims &e) override
    {
        m_dirty = true; // the caller may write through the pointer
        return (char *)m_host + index(e) * m_storage->m_element_size;
    }
    void copyBytesFrom(const Dims &e, const void *src, size_t size) override
    {
        memcpy((char *)m_host + index(e) * m_storage->m_element_size, src, size);
        m_dirty = true;
    }

private:
    HipTensor &m_t;
    std::shared_ptr<HipStorage> m_storage;
    void *m_host = nullptr;
    size_t m_bytes = 0;
    bool m_dirty = false;
};

// Host window onto the back buffer of a batched tensor: no copies, the program moves the data.
class HipBatchAccess : public TensorAccess {
public:
    HipBatchAccess(HipTensor &t, std::shared_ptr<HipDoubleBuffer> db) : m_t(t), m_db(db) {}
    Dims strides() override
    {
        Dims d;
        for(auto s : m_t.m_strides)
            d.push_back(s);
        return d;
    }
    void *data() override { return (char *)m_db->hostBack() + m_t.m_offset * (int64_t)m_db->m_element_size; }
    size_t index(const Dims &e) const
    {
        int64_t o = m_t.m_offset;
        for(size_t i = 0; i < e.size() && i < m_t.m_strides.size(); i++)
            o += (int64_t)(int)e[i] * m_t.m_strides[i];
        return (size_t)o;
    }
    double get(const Dims &e) override { return host_load(m_db->hostBack(), m_db->m_data_type, index(e)); }
    void set(const Dims &e, double v) override { host_store(m_db->hostBack(), m_db->m_data_type, index(e), v); }
    void *getAddr(const Dims &e) override { return (char *)m_db->hostBack() + index(e) * m_db->m_element_size; }
    void copyBytesFrom(const Dims &e, const void *src, size_t size) override { memcpy(getAddr(e), src, size); }

private:
    HipTensor &m_t;
    std::shared_ptr<HipDoubleBuffer> m_db;
};

std::unique_ptr<TensorAccess> HipTensor::access()
{
    if(m_storage->doubleBuffered())
        return std::make_unique<HipBatchAccess>(*this, std::static_pointer_cast<HipDoubleBuffer>(m_storage));
    return std::make_unique<HipStagedAccess>(*this);
}

std::shared_ptr<Tensor> HipTensor::slice(const Dims &offset, const Dims &size)
{
    int64_t o = m_offset;
    for(size_t i = 0; i < offset.size() && i < m_strides.size(); i++)
        o += (int64_t)(int)offset[i] * m_strides[i];
    return std::make_shared<HipTensor>(m_storage, size, m_strides, o, namePostfix("slice"));
}

Tensor::Stats HipTensor::stats() { return Tensor::stats(); }

// Fills this tensor from a front-end tensor: a straight memcpy when type and strides agree,
// else element by element with conversion (also serves generated tensors, whose access
// object produces a fresh random value per read).
void HipTensor::copyFromHost(Tensor &src)
{
    auto ta = src.access();
    if(!ta)
        return; // placeholder without values: storage stays zero
    m_auto_initialized = ta->data() == nullptr;
    const size_t n = m_storage->m_elements;
    const size_t es = m_storage->m_element_size;
    std::vector<uint8_t> host(std::max<size_t>(n * es, 16));
    if(m_storage->m_ctx)
        m_storage->m_ctx->sync();
    chkHip(hipMemcpy(host.data(), m_storage->deviceMem(), n * es, hipMemcpyDeviceToHost));

    const size_t rank = m_dims.size(), srank = src.m_dims.size();
    if(src.m_dims.elements() != m_dims.elements())
        throw std::runtime_error("copyFromHost: element count mismatch " + src.info() + " -> " + info());
    const std::vector<int64_t> ext = m_dims.i64();
    const std::vector<int64_t> sext = src.m_dims.i64();
    const Dims sstr = ta->strides();
    const void *sdata = ta->data();
    const bool fast = sdata != nullptr && src.m_data_type == m_data_type && sstr.size() == srank;
    std::vector<int64_t> sstr64;
    if(fast)
        sstr64 = sstr.i64();
    // iterate this tensor's logical coordinates; the source is walked in row-major order of
    // ITS OWN dims (ranks may differ, e.g. {C} params lowered to {1,C})
    std::vector<int64_t> c(rank, 0), sc(srank, 0);
    Dims se(srank, (int64_t)0);
    for(size_t i = 0; i < n; i++) {
        int64_t o = m_offset;
        for(size_t j = 0; j < rank; j++)
            o += c[j] * m_strides[j];
        if(fast) {
            int64_t so = 0;
            for(size_t j = 0; j < srank; j++)
                so += sc[j] * sstr64[j];
            memcpy(host.data() + o * es, (const char *)sdata + so * es, es);
        } else {
            for(size_t j = 0; j < srank; j++)
                se[j] = sc[j];
            host_store(host.data(), m_data_type, (size_t)o, ta->get(se));
        }
        for(ssize_t j = (ssize_t)rank - 1; j >= 0; j--) {
            if(++c[j] == ext[j])
                c[j] = 0;
            else
                break;
        }
        for(ssize_t j = (ssize_t)srank - 1; j >= 0; j--) {
            if(++sc[j] == sext[j])
                sc[j] = 0;
            else
                break;
        }
    }
    if(m_storage->doubleBuffered()) {
        auto db = std::static_pointer_cast<HipDoubleBuffer>(m_storage);
        for(int i = 0; i < 2; i++) {
            memcpy(db->m_host[i], host.data(), n * es);
            chkHip(hipMemcpy(db->m_dev[i], host.data(), n * es, hipMemcpyHostToDevice));
        }
    } else {
        chkHip(hipMemcpy(m_storage->deviceMem(), host.data(), n * es, hipMemcpyHostToDevice));
    }
}

}  // namespace saga

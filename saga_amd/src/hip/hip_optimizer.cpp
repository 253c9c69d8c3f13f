// Adam optimizers of the hip engine.  Every (weight, gradient) pair of one data type is
// re-homed into ONE contiguous arena laid out [all weights | all gradients], each tensor
// padded to 16 elements, so that a single kernel launch updates the whole model
// (reference: src/cuda/cuda_optimizer.cpp:196-292; the multi-GPU reduce-scatter / all-gather
// around the update is not part of this single-GPU engine).
#include <math.h>
#include <string.h>

#include "hip_common.hpp"

namespace saga {

namespace {

constexpr double ADAM_B1 = 0.9;   // reference: src/cuda/cuda_kernels.hpp:54
constexpr double ADAM_B2 = 0.999; // reference: src/cuda/cuda_kernels.hpp:55

// where one parameter sits in the optimizer's flat arrays (elements from the start), by front-end tensor name
struct OptimizerSlot {
    std::string name;
    size_t offset, elements;
};

struct Optimizer : public HipOperation {
    HipOpArgs m_inputs, m_outputs;
    const std::shared_ptr<HipMemory> m_arena;
    const size_t m_elements; // per half of the arena
    int m_iter = 0;
    std::vector<OptimizerSlot> m_slots;
    // the fp32 state arrays, each m_elements long: m, v and - mixed precision - the master weights
    virtual std::vector<std::pair<const char *, float *>> stateArrays() = 0;
    Optimizer(const char *name, const HipOpArgs &in, const HipOpArgs &out, std::shared_ptr<HipMemory> arena,
              size_t elements)
      : HipOperation(name), m_inputs(in), m_outputs(out), m_arena(arena), m_elements(elements)
    {
    }
    HipOpArgs listInputs() const override { return m_inputs; }
    HipOpArgs listOutputs() const override { return m_outputs; }
    std::string info() const override { return fmt("%zd elements", m_elements); }
    // bias corrections and the loss scale are launch arguments that change every step
    bool graphSafe() const override { return false; }
    // w, g, m, v read and w, m, v written in fp32: 28 bytes per element; the mixed flavour moves
    // fp16 w/g and an extra fp32 master copy: also 28
    double bytes() const override { return 28.0 * m_elements; }
};

struct AdamF32 : public Optimizer {
    HipMemory m_m, m_v;
    AdamF32(const HipOpArgs &in, const HipOpArgs &out, std::shared_ptr<HipMemory> arena, size_t elements)
      : Optimizer("adam-f32", in, out, arena, elements), m_m(elements * sizeof(float)), m_v(elements * sizeof(float))
    {
    }
    std::vector<std::pair<const char *, float *>> stateArrays() override
    {
        return {{"m", (float *)m_m.m_ptr}, {"v", (float *)m_v.m_ptr}};
    }
    void exec(HipProgram &p) override
    {
        const int t = ++m_iter;
        const float b1t = 1.0 / (1.0 - pow(ADAM_B1, t)); // :79-80
        const float b2t = 1.0 / (1.0 - pow(ADAM_B2, t));
        float *w = (float *)m_arena->m_ptr;
        chkSaga(saga_hip_adam_f32(m_elements, w, w + m_elements, (float *)m_m.m_ptr, (float *)m_v.m_ptr, b1t, b2t,
                                  p.m_pc.learning_rate, p.m_pc.l2_lambda, p.m_aux, (saga_stream_t)p.m_ctx->m_stream));
    }
};

struct AdamMixed : public Optimizer {
    HipMemory m_m, m_v, m_c;
    AdamMixed(HipProgram &p, const HipOpArgs &in, const HipOpArgs &out, std::shared_ptr<HipMemory> arena,
              size_t elements)
      : Optimizer("adam-mixed", in, out, arena, elements)
      , m_m(elements * sizeof(float))
      , m_v(elements * sizeof(float))
      , m_c(elements * sizeof(float))
    {
        // fp32 master copy of the initial fp16 weights (:142-145)
        SagaTensorView src, dst;
        for(int i = 0; i < 4; i++) {
            src.dims[i] = dst.dims[i] = 1;
            src.strides[i] = dst.strides[i] = 1;
        }
        // split the flat arena into rows so that every extent fits an int32
        const size_t row = 1 << 20;
        for(size_t off = 0; off < elements; off += row) {
            const size_t n = std::min(row, elements - off);
            src.ptr = (uint16_t *)arena->m_ptr + off;
            dst.ptr = (float *)m_c.m_ptr + off;
            src.dims[1] = dst.dims[1] = (int)n;
            src.strides[0] = dst.strides[0] = (int64_t)n;
            src.dtype = SAGA_HALF;
            dst.dtype = SAGA_FLOAT;
            chkSaga(saga_hip_convert(&src, &dst, 1.0f, (saga_stream_t)p.m_ctx->m_stream));
        }
    }
    std::vector<std::pair<const char *, float *>> stateArrays() override
    {
        return {{"m", (float *)m_m.m_ptr}, {"v", (float *)m_v.m_ptr}, {"master", (float *)m_c.m_ptr}};
    }
    void exec(HipProgram &p) override
    {
        const int t = ++m_iter;
        const float b1t = 1.0 / (1.0 - pow(ADAM_B1, t));
        const float b2t = 1.0 / (1.0 - pow(ADAM_B2, t));
        uint16_t *w = (uint16_t *)m_arena->m_ptr;
        chkSaga(saga_hip_adam_mixed(m_elements, 1.0f / p.m_mp_scaling, w, w + m_elements, (float *)m_m.m_ptr,
                                    (float *)m_v.m_ptr, (float *)m_c.m_ptr, b1t, b2t, p.m_pc.learning_rate,
                                    p.m_pc.l2_lambda, p.m_aux, (saga_stream_t)p.m_ctx->m_stream));
    }
};

}  // namespace

HipOp HipProgram::createOptimizer(Tensor::DataType dt)
{
    const size_t align = 16;
    const size_t esize = Tensor::DataTypeSize(dt);
    size_t total = 0;
    for(const auto &u : m_updates) {
        const auto &w = u.second.first;
        const auto &g = u.second.second;
        if(w->m_data_type != dt)
            continue;
        if(w->m_dims != g->m_dims || w->m_data_type != g->m_data_type)
            throw std::runtime_error("optimizer: weight and gradient disagree: " + w->info() + " vs " + g->info());
        if(w->m_dims.elements() != w->m_storage->m_elements || g->m_dims.elements() != g->m_storage->m_elements)
            throw std::runtime_error("optimizer: parameter tensors must own their storage: " + w->info());
        total += (w->m_dims.elements() + align - 1) & ~(align - 1);
    }
    if(total == 0)
        return nullptr;

    auto arena = std::make_shared<HipMemory>(total * 2 * esize); // zero filled
    char *wbase = (char *)arena->m_ptr;
    char *gbase = wbase + total * esize;
    size_t at = 0;
    HipOpArgs inputs, outputs;
    std::vector<OptimizerSlot> slots;
    m_ctx->sync();
    for(const auto &u : m_updates) {
        const auto &w = u.second.first;
        const auto &g = u.second.second;
        if(w->m_data_type != dt)
            continue;
        const size_t n = w->m_dims.elements();
        void *wnew = wbase + at * esize, *gnew = gbase + at * esize;
        if(w->m_storage->m_memory != arena) { // a parameter shared with an earlier program may already live in an arena
            auto def = m_ctx->m_deferred_copy.find(w);
            if(def == m_ctx->m_deferred_copy.end()) {
                // already initialised on the device by an earlier program: carry the values over
                chkHip(hipMemcpy(wnew, w->m_storage->deviceMem(), n * esize, hipMemcpyDeviceToDevice));
                w->m_storage->rehome(arena, wnew);
            } else {
                w->m_storage->rehome(arena, wnew);
                w->copyFromHost(*def->second);
                m_ctx->m_deferred_copy.erase(def);
            }
            g->m_storage->rehome(arena, gnew);
            m_ctx->m_deferred_copy.erase(g);
        }
        inputs.push_back({"g", g});
        inputs.push_back({"w", w});
        outputs.push_back({"w", w});
        slots.push_back({u.first->m_name ? *u.first->m_name : std::string(), at, n});
        at += (n + align - 1) & ~(align - 1);
    }
    std::shared_ptr<Optimizer> opt;
    switch(dt) {
    case Tensor::DataType::FLOAT: opt = std::make_shared<AdamF32>(inputs, outputs, arena, total); break;
    case Tensor::DataType::HALF: opt = std::make_shared<AdamMixed>(*this, inputs, outputs, arena, total); break;
    default:
        throw std::runtime_error(fmt("Unsupported datatype %s in optimizer", Tensor::DataTypeStr(dt)));
    }
    opt->m_slots = std::move(slots);
    return opt;
}

// ---------------------------------------------------------------- optimizer state files
//
// The reference saves tensors only (Graph::saveTensors, src/graph.cpp:60-104), so a reloaded run restarts
// Adam's moments, bias corrections and loss scale.  This file carries them: per optimizer the step count,
// and per parameter - keyed by the front-end tensor's name, because the order of the arena follows
// pointer values and differs from process to process - the slices of m, v and the fp32 master weights.
//   "sagaO001" | f32 loss scale | u32 optimizers | { char kind[16] | i32 step | u32 arrays | u32 slots |
//   { u16 name length | name | u64 elements | arrays x f32[elements] } }

namespace {
const char OPT_MAGIC[8] = {'s', 'a', 'g', 'a', 'O', '0', '0', '1'};

template <typename V> void put(FILE *f, const V &v)
{
    if(fwrite(&v, sizeof(V), 1, f) != 1)
        throw std::runtime_error("optimizer state: write failed");
}
template <typename V> V get(FILE *f)
{
    V v;
    if(fread(&v, sizeof(V), 1, f) != 1)
        throw std::runtime_error("optimizer state: file truncated");
    return v;
}
struct FileCloser {
    FILE *f;
    ~FileCloser()
    {
        if(f)
            fclose(f);
    }
};
}  // namespace

void HipProgram::saveOptimizerState(const char *path)
{
    finalize();
    m_ctx->sync();
    FileCloser fc{fopen(path, "wb")};
    if(!fc.f)
        throw std::runtime_error(fmt("optimizer state: cannot create %s", path));
    std::vector<Optimizer *> opts;
    for(auto &op : m_ops)
        if(auto *o = dynamic_cast<Optimizer *>(op.get()))
            opts.push_back(o);
    fwrite(OPT_MAGIC, 8, 1, fc.f);
    put<float>(fc.f, m_mp_scaling);
    put<uint32_t>(fc.f, (uint32_t)opts.size());
    std::vector<float> host;
    for(Optimizer *o : opts) {
        char kind[16] = {};
        snprintf(kind, sizeof(kind), "%s", o->name().c_str());
        fwrite(kind, 16, 1, fc.f);
        auto arrays = o->stateArrays();
        put<int32_t>(fc.f, o->m_iter);
        put<uint32_t>(fc.f, (uint32_t)arrays.size());
        put<uint32_t>(fc.f, (uint32_t)o->m_slots.size());
        for(const auto &sl : o->m_slots) {
            if(sl.name.empty() || sl.name.size() > 65535)
                throw std::runtime_error("optimizer state: every trained tensor needs a name");
            put<uint16_t>(fc.f, (uint16_t)sl.name.size());
            fwrite(sl.name.data(), 1, sl.name.size(), fc.f);
            put<uint64_t>(fc.f, sl.elements);
            host.resize(sl.elements);
            for(auto &a : arrays) {
                chkHip(hipMemcpy(host.data(), a.second + sl.offset, sl.elements * sizeof(float), hipMemcpyDeviceToHost));
                if(fwrite(host.data(), sizeof(float), sl.elements, fc.f) != sl.elements)
                    throw std::runtime_error("optimizer state: write failed");
            }
        }
    }
}

void HipProgram::loadOptimizerState(const char *path)
{
    finalize();
    m_ctx->sync();
    FileCloser fc{fopen(path, "rb")};
    if(!fc.f)
        throw std::runtime_error(fmt("optimizer state: cannot open %s", path));
    char magic[8];
    if(fread(magic, 8, 1, fc.f) != 1 || memcmp(magic, OPT_MAGIC, 8))
        throw std::runtime_error(fmt("optimizer state: %s is not a sagaO001 file", path));
    const float scale = get<float>(fc.f);
    const uint32_t nopt = get<uint32_t>(fc.f);
    std::vector<Optimizer *> opts;
    for(auto &op : m_ops)
        if(auto *o = dynamic_cast<Optimizer *>(op.get()))
            opts.push_back(o);
    if(nopt != opts.size())
        throw std::runtime_error(fmt("optimizer state: file has %u optimizers, the program %zu", nopt, opts.size()));
    std::vector<float> host;
    for(uint32_t i = 0; i < nopt; i++) {
        char kind[17] = {};
        if(fread(kind, 16, 1, fc.f) != 1)
            throw std::runtime_error("optimizer state: file truncated");
        Optimizer *o = nullptr;
        for(Optimizer *c : opts)
            if(c->name() == kind)
                o = c;
        if(!o)
            throw std::runtime_error(fmt("optimizer state: the program has no %s optimizer", kind));
        auto arrays = o->stateArrays();
        const int32_t iter = get<int32_t>(fc.f);
        const uint32_t narr = get<uint32_t>(fc.f), nslots = get<uint32_t>(fc.f);
        if(narr != arrays.size() || nslots != o->m_slots.size())
            throw std::runtime_error(fmt("optimizer state: %s holds %u arrays of %u tensors, the program %zu of %zu", kind,
                                         narr, nslots, arrays.size(), o->m_slots.size()));
        for(uint32_t s = 0; s < nslots; s++) {
            const uint16_t len = get<uint16_t>(fc.f);
            std::string name(len, '\0');
            if(len && fread(&name[0], 1, len, fc.f) != len)
                throw std::runtime_error("optimizer state: file truncated");
            const uint64_t n = get<uint64_t>(fc.f);
            const OptimizerSlot *sl = nullptr;
            for(const auto &c : o->m_slots)
                if(c.name == name)
                    sl = &c;
            if(!sl || sl->elements != n)
                throw std::runtime_error(fmt("optimizer state: tensor %s (%llu elements) does not match the program",
                                             name.c_str(), (unsigned long long)n));
            host.resize(n);
            for(auto &a : arrays) {
                if(fread(host.data(), sizeof(float), n, fc.f) != n)
                    throw std::runtime_error("optimizer state: file truncated");
                chkHip(hipMemcpy(a.second + sl->offset, host.data(), n * sizeof(float), hipMemcpyHostToDevice));
            }
        }
        o->m_iter = iter;
    }
    m_mp_scaling = scale;
}

HipOps HipProgram::createOptimizers()
{
    HipOps ops;
    if(auto o = createOptimizer(Tensor::DataType::FLOAT))
        ops.push_back(o);
    if(auto o = createOptimizer(Tensor::DataType::HALF)) {
        m_mp_enabled = true;
        ops.push_back(o);
    }
    return ops;
}

}  // namespace saga

// Adam optimizers of the hip engine.  Every (weight, gradient) pair of one data type is
// re-homed into ONE contiguous arena laid out [all weights | all gradients], each tensor
// padded to 16 elements, so that a single kernel launch updates the whole model
// (reference: src/cuda/cuda_optimizer.cpp:196-292; the multi-GPU reduce-scatter / all-gather
// around the update is not part of this single-GPU engine).
#include <math.h>

#include "hip_common.hpp"

namespace saga {

namespace {

constexpr double ADAM_B1 = 0.9;   // reference: src/cuda/cuda_kernels.hpp:54
constexpr double ADAM_B2 = 0.999; // reference: src/cuda/cuda_kernels.hpp:55

struct Optimizer : public HipOperation {
    HipOpArgs m_inputs, m_outputs;
    const std::shared_ptr<HipMemory> m_arena;
    const size_t m_elements; // per half of the arena
    int m_iter = 0;
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
        at += (n + align - 1) & ~(align - 1);
    }
    switch(dt) {
    case Tensor::DataType::FLOAT: return std::make_shared<AdamF32>(inputs, outputs, arena, total);
    case Tensor::DataType::HALF: return std::make_shared<AdamMixed>(*this, inputs, outputs, arena, total);
    default:
        throw std::runtime_error(fmt("Unsupported datatype %s in optimizer", Tensor::DataTypeStr(dt)));
    }
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

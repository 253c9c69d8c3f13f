// Engine, context and program of the hip backend: node lowering driver, op-list assembly
// (forward ops, then backward ops in reverse creation order, then the optimizers), the
// accumulate-on-second-writer rule, dead-operation elimination and the run loop with
// double-buffered batched tensors and the loss-scale controller.
// Role of the reference's src/cuda/cuda_common.cpp and src/cuda/cuda_program.cpp.
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <cmath>
#include <set>
#include <sstream>
#include <unordered_map>

#include "hip_common.hpp"
// after saga.hpp: the registry header relies on its declarations
#include "engine.hpp"

namespace saga {

// ---------------------------------------------------------------- registries

static std::map<std::string, HipOpSetup> &op_table()
{
    static std::map<std::string, HipOpSetup> t;
    return t;
}

struct TransformEntry {
    int prio;
    ProgramType types;
    HipTransform fn;
};

static std::vector<TransformEntry> &transform_table()
{
    static std::vector<TransformEntry> t;
    return t;
}

void hipRegisterOp(const char *name, HipOpSetup setup) { op_table()[name] = setup; }

void hipRegisterTransform(int prio, ProgramType types, HipTransform fn)
{
    auto &t = transform_table();
    t.push_back({prio, types, fn});
    std::stable_sort(t.begin(), t.end(), [](const TransformEntry &a, const TransformEntry &b) { return a.prio < b.prio; });
}

HipOpSetup hipFindOp(const std::string &type)
{
    auto it = op_table().find(type);
    return it == op_table().end() ? nullptr : it->second;
}

Nodes hipApplyTransforms(HipProgram &p, HipProgramUnit &pu, const Nodes &nodes)
{
    Nodes cur = nodes;
    for(const auto &t : transform_table())
        if(!!(p.m_pt & t.types))
            cur = t.fn(p, pu, cur);
    return cur;
}

// ---------------------------------------------------------------- operations (generic part)

HipOpArgs HipOperation::getInputs()
{
    HipOpArgs r = listInputs();
    for(auto &o : listOutputs()) {
        float *beta = getBeta(o.second);
        if(beta && *beta != 0.0f)
            r.push_back(o);
    }
    return r;
}

std::string HipOperation::str()
{
    std::stringstream ss;
    const char *sep = "";
    for(const auto &o : getOutputs()) {
        float *beta = getBeta(o.second);
        ss << sep << (beta && *beta != 0.0f ? "+" : "") << o.first << ":" << o.second->shortname();
        sep = ", ";
    }
    ss << " = " << name() << "(";
    sep = "";
    for(const auto &i : listInputs()) {
        ss << sep << i.first << ":" << i.second->shortname();
        sep = ", ";
    }
    const std::string inf = info();
    if(!inf.empty())
        ss << ", " << inf;
    ss << ")";
    return ss.str();
}

void HipOperation::dump(FILE *out, bool full)
{
    if(!full) {
        fprintf(out, "%s\n", str().c_str());
        return;
    }
    fprintf(out, "OP: %s %s\n", name().c_str(), info().c_str());
    for(const auto &t : getInputs())
        fprintf(out, "\tI: %3s: %s\n", t.first, t.second->info().c_str());
    for(const auto &t : getOutputs())
        fprintf(out, "\tO: %3s: %s\n", t.first, t.second->info().c_str());
}

// ---------------------------------------------------------------- engine / context

class HipEngine : public Engine {
public:
    explicit HipEngine(const std::shared_ptr<UI> &ui) : m_ui(ui) {}
    // One context per process: this backend drives a single GPU
    // (the reference creates one per device, src/cuda/cuda_common.cpp:89-129).
    std::vector<std::shared_ptr<Context>> createContexts(bool) override
    {
        int count = 0;
        if(hipGetDeviceCount(&count) != hipSuccess || count < 1)
            throw std::runtime_error("hip engine: no GPU visible");
        return {std::make_shared<HipContext>(m_ui, 0)};
    }
    const std::shared_ptr<UI> m_ui;
};

static std::shared_ptr<Engine> createHipEngine(const std::shared_ptr<UI> &ui) { return std::make_shared<HipEngine>(ui); }

static void __attribute__((constructor)) registerHipEngine(void)
{
    if(getenv("SAGA_DISABLE_HIP"))
        return;
    registerEngineFactory("hip", &createHipEngine);
}

HipContext::HipContext(const std::shared_ptr<UI> &ui, int device) : m_ui(ui), m_device(device)
{
    chkHip(hipSetDevice(device));
    chkSaga(saga_hip_init(device, &m_num_cu));
    chkHip(hipStreamCreateWithFlags(&m_stream, hipStreamDefault));
    chkHip(hipStreamCreateWithFlags(&m_copy_stream, hipStreamDefault));
    hipDeviceProp_t prop;
    chkHip(hipGetDeviceProperties(&prop, device));
    m_ui->updateCell(getUiPage(), 0, 0, UI::Align::LEFT, "%s", prop.name);
    m_ui->updateCell(getUiPage(), 0, 1, UI::Align::LEFT, "Dev #%d", device);
    m_workspace.request(4096);
}

HipContext::~HipContext()
{
    if(m_stream) {
        (void)hipStreamSynchronize(m_stream);
        (void)hipStreamDestroy(m_stream);
    }
    if(m_copy_stream) {
        (void)hipStreamSynchronize(m_copy_stream);
        (void)hipStreamDestroy(m_copy_stream);
    }
}

void HipContext::reset()
{
    sync();
    m_exported.clear();
    m_tensors.clear();
    m_deferred_copy.clear();
    m_storage_id_gen = 0;
    m_program_index_gen = 0;
}

// reference: src/cuda/cuda_common.cpp:145-158
std::shared_ptr<Tensor> HipContext::resolveTensor(std::shared_ptr<Tensor> src)
{
    if(!src)
        return nullptr;
    auto it = m_tensors.find(src);
    if(it == m_tensors.end())
        return nullptr;
    m_exported.push_back(it->second->m_storage);
    // a tensor the host holds keeps its contents between steps: out of the shared arena
    // (reference: src/cuda/cuda_common.cpp:145-158)
    auto &st = it->second->m_storage;
    if(st->m_in_arena) {
        // memory of its own from here on; what the arena slot holds right now moves along
        sync();
        auto keep = st->m_memory;
        void *old = st->m_data;
        st->allocOwn();
        chkHip(hipMemcpy(st->m_data, old, st->bytes(), hipMemcpyDeviceToDevice));
    }
    return it->second;
}

// Storage reuse.  A storage qualifies when, in every finalized program that touches it, the
// first operation to touch it overwrites it (nothing is carried over from the previous step or
// from the host), the host holds no reference to it, and it has no memory of its own yet
// (weights, optimizer state and anything the host wrote have).  Two such storages may share
// addresses unless some program uses both with overlapping live ranges [first touch, last
// touch].  Placement is first-fit by decreasing size against the already placed storages that
// conflict.  The reference walks one program with a best-fit free list
// (src/cuda/cuda_analysis.cpp:472-530); planning per context instead keeps an inference and a
// training program that share activations from overwriting each other's tensors.
void HipContext::planMemory()
{
    static const bool disabled = getenv("SAGA_HIP_NO_ARENA") != nullptr;
    if(disabled)
        return;
    struct Range {
        int prog, first, last;
    };
    struct Item {
        HipStorage *s;
        size_t bytes, offset;
        std::vector<Range> ranges;
    };
    std::unordered_map<HipStorage *, Item> items;
    std::set<HipStorage *> carried;
    for(size_t pi = 0; pi < m_programs.size(); pi++) {
        const HipOps &ops = m_programs[pi]->m_ops;
        std::unordered_map<HipStorage *, Range> seen;
        for(size_t i = 0; i < ops.size(); i++) {
            auto touch = [&](const HipOpArgs &args, bool reads) {
                for(const auto &a : args) {
                    HipStorage *st = a.second->m_storage.get();
                    auto it = seen.find(st);
                    if(it == seen.end()) {
                        seen[st] = Range{(int)pi, (int)i, (int)i};
                        // a partial first write leaves the rest of the storage as it was
                        if(reads || a.second->m_dims.elements() != st->m_elements)
                            carried.insert(st);
                    } else {
                        it->second.last = (int)i;
                    }
                }
            };
            touch(ops[i]->getInputs(), true);
            touch(ops[i]->getOutputs(), false);
        }
        for(const auto &kv : seen) {
            auto &it = items[kv.first];
            it.s = kv.first;
            it.ranges.push_back(kv.second);
        }
    }
    std::set<HipStorage *> exported;
    for(const auto &e : m_exported)
        exported.insert(e.get());
    std::vector<Item *> cand;
    for(auto &kv : items) {
        HipStorage *st = kv.first;
        if(carried.count(st) || exported.count(st) || st->doubleBuffered())
            continue;
        if(st->allocated() && !st->m_in_arena)
            continue;
        kv.second.bytes = (st->bytes() + 255) & ~(size_t)255;
        cand.push_back(&kv.second);
    }
    std::sort(cand.begin(), cand.end(), [](const Item *a, const Item *b) {
        return a->bytes != b->bytes ? a->bytes > b->bytes : a->s->m_id < b->s->m_id;
    });
    auto conflict = [](const Item &a, const Item &b) {
        for(const auto &ra : a.ranges)
            for(const auto &rb : b.ranges)
                if(ra.prog == rb.prog && ra.first <= rb.last && rb.first <= ra.last)
                    return true;
        return false;
    };
    std::vector<Item *> placed;
    size_t total = 0, planned = 0;
    for(Item *it : cand) {
        std::vector<std::pair<size_t, size_t>> busy; // [begin, end) of conflicting storages
        for(Item *q : placed)
            if(conflict(*it, *q))
                busy.emplace_back(q->offset, q->offset + q->bytes);
        std::sort(busy.begin(), busy.end());
        size_t off = 0;
        for(const auto &b : busy) {
            if(off + it->bytes <= b.first)
                break;
            off = std::max(off, b.second);
        }
        it->offset = off;
        placed.push_back(it);
        total = std::max(total, off + it->bytes);
        planned += it->bytes;
    }
    if(placed.empty())
        return;
    auto arena = std::make_shared<HipMemory>(total); // zero filled once; slots are not cleared on reuse
    for(Item *it : placed) {
        it->s->rehome(arena, (char *)arena->m_ptr + it->offset);
        it->s->m_in_arena = true;
    }
    for(size_t pi = 0; pi < m_programs.size(); pi++) {
        HipProgram *pr = m_programs[pi];
        pr->m_poison_before.assign(pr->m_ops.size(), {});
        pr->m_poison_after.assign(pr->m_ops.size(), {});
        for(Item *it : placed)
            for(const auto &r : it->ranges)
                if(r.prog == (int)pi) {
                    pr->m_poison_before[r.first].push_back(it->s);
                    pr->m_poison_after[r.last].push_back(it->s);
                }
    }
    m_arena = arena;
    m_arena_bytes = total;
    m_planned_bytes = planned;
    if(getenv("SAGA_HIP_VERBOSE"))
        fprintf(stderr, "hip: arena %.1f MB holds %zu storages of %.1f MB in total\n", total / 1e6, placed.size(),
                planned / 1e6);
}

// reference: src/cuda/cuda_common.cpp:322-399
std::shared_ptr<Program> HipContext::createMultiProgram(const std::vector<ProgramSource> &sources, ProgramType pt,
                                                        const ProgramConfig &pc)
{
    chkHip(hipSetDevice(m_device));
    auto p = std::make_shared<HipProgram>(shared_from_this(), pt, pc);
    p->m_name = pt == ProgramType::INFERENCE ? "Inference" : "Training";
    m_ui->updateCell(getUiPage(), p->getUiRow(), 0, UI::Align::LEFT, "%s", p->m_name.c_str());

    float batch_sum = 0;
    for(const auto &s : sources) {
        p->addBatchedTensors(s);
        p->m_units.emplace_back();
        auto &pu = p->m_units.back();
        pu.m_batch_size = s.batch_size;
        batch_sum += s.batch_size;
        pu.m_transformed = hipApplyTransforms(*p, pu, s.graph.m_nodes);
    }
    // initial loss scale: sum of the batch sizes (src/cuda/cuda_common.cpp:339-353) unless configured
    p->m_mp_scaling = batch_sum;
#ifdef SAGA_HAS_INITIAL_LOSS_SCALE
    if(pc.initial_loss_scale > 0)
        p->m_mp_scaling = pc.initial_loss_scale;
#endif

    size_t index = 0;
    for(auto &pu : p->m_units) {
        for(const auto &n : pu.m_transformed) {
            HipOpSetup setup = hipFindOp(n->m_type);
            try {
                // the reference silently skips node types it has no operation for; here that is an error
                if(!setup)
                    throw std::runtime_error("the hip engine has no operation for this node type");
                setup(*p, pu, *n);
            } catch(const std::exception &e) {
                throw std::runtime_error(
                    fmt("Unable to create operation %s (#%zd) -- %s", n->m_type.c_str(), index, e.what()));
            }
            index++;
        }
        if(pt == ProgramType::INFERENCE && !pu.m_bwd.empty())
            throw std::runtime_error("inference program produced backward operations");
    }
    if(pt == ProgramType::TRAINING) {
        p->m_opt = p->createOptimizers();
        p->m_updates.clear();
    }
    return p;
}

// ---------------------------------------------------------------- program: lowering helpers

HipProgram::HipProgram(std::shared_ptr<HipContext> ctx, ProgramType pt, const ProgramConfig &pc)
  : m_ctx(ctx), m_index(ctx->m_program_index_gen++), m_pt(pt), m_pc(pc)
{
    chkHip(hipHostMalloc((void **)&m_aux, 4096, hipHostMallocDefault));
    memset(m_aux, 0, 4096);
}

HipProgram::~HipProgram()
{
    m_ctx->sync();
    auto &ps = m_ctx->m_programs;
    ps.erase(std::remove(ps.begin(), ps.end(), this), ps.end());
    for(auto e : m_events)
        (void)hipEventDestroy(e);
    dropGraphs();
    (void)hipHostFree(m_aux);
}

// fp16 and u8 tensors are channels-last, everything else channels-first, unless the program
// asks for one layout (reference: tensorFormat, src/cuda/cuda_program.cpp:66-90)
HipLayout HipProgram::layoutFor(Tensor::DataType dt) const
{
    switch(m_pc.tensor_layout) {
    case TensorLayout::NHWC: return HipLayout::NHWC;
    case TensorLayout::NCHW: return HipLayout::NCHW;
    case TensorLayout::Auto: break;
    }
    return (dt == Tensor::DataType::HALF || dt == Tensor::DataType::U8) ? HipLayout::NHWC : HipLayout::NCHW;
}

// reference: lower_tensor, src/cuda/cuda_program.cpp:92-120
std::shared_ptr<HipTensor> HipProgram::lower(const HipProgramUnit &pu, std::shared_ptr<Tensor> src,
                                             size_t minimum_rank)
{
    if(!src)
        return nullptr;
    auto it = m_ctx->m_tensors.find(src);
    if(it != m_ctx->m_tensors.end())
        return it->second;
    Dims dims = src->m_dims;
    if(minimum_rank > 1) {
        if(dims.size() < 2)
            dims.insert(dims.begin(), (int64_t)1);
        while(dims.size() < minimum_rank)
            dims.push_back((int64_t)1);
    }
    dims = dims.batch(pu.m_batch_size);
    auto t = std::make_shared<HipTensor>(src->m_data_type, dims, layoutFor(src->m_data_type), m_ctx.get(), src->m_name);
    m_ctx->m_deferred_copy[t] = src;
    m_ctx->m_tensors[src] = t;
    return t;
}

std::shared_ptr<HipTensor> HipProgram::lowerLike(const HipProgramUnit &pu, std::shared_ptr<Tensor> src,
                                                 const HipTensor &blueprint)
{
    auto it = m_ctx->m_tensors.find(src);
    if(it != m_ctx->m_tensors.end())
        return it->second;
    const Dims dims = src->m_dims.batch(pu.m_batch_size);
    HipLayout layout = layoutFor(src->m_data_type);
    if(dims.size() == 4 && blueprint.m_dims.size() == 4)
        layout = blueprint.cpacked() ? HipLayout::NHWC : HipLayout::NCHW;
    auto t = std::make_shared<HipTensor>(src->m_data_type, dims, layout, m_ctx.get(), src->m_name);
    m_ctx->m_deferred_copy[t] = src;
    m_ctx->m_tensors[src] = t;
    return t;
}

std::shared_ptr<HipTensor> HipProgram::lowerGrad(const HipProgramUnit &pu, std::shared_ptr<Tensor> src,
                                                 size_t minimum_rank)
{
    if(!src)
        return nullptr;
    auto g = src->grad();
    if(!g)
        return nullptr; // tensors of foreign classes may have no gradient twin
    // a gradient shares the layout of its value when that is already lowered (aliases!)
    auto vit = m_ctx->m_tensors.find(src);
    auto git = m_ctx->m_tensors.find(g);
    if(git != m_ctx->m_tensors.end())
        return git->second;
    if(vit != m_ctx->m_tensors.end() && vit->second->m_dims.size() == 4) {
        auto t = std::make_shared<HipTensor>(g->m_data_type, *vit->second, g->m_name);
        m_ctx->m_deferred_copy[t] = g;
        m_ctx->m_tensors[g] = t;
        return t;
    }
    return lower(pu, g, minimum_rank);
}

void HipProgram::upd(const std::shared_ptr<Tensor> &key, const std::shared_ptr<HipTensor> &w,
                     const std::shared_ptr<HipTensor> &g)
{
    m_updates[key] = std::make_pair(w, g);
}

// reference: addBatchedTensors, src/cuda/cuda_program.cpp:378-404
void HipProgram::addBatchedTensors(const ProgramSource &ps)
{
    for(const auto &bt : ps.batched_tensors) {
        auto src = bt.first;
        auto &slot = m_batched[src];
        if(!slot.first) {
            auto existing = m_ctx->m_tensors.find(src);
            if(existing != m_ctx->m_tensors.end() && existing->second->m_storage->doubleBuffered()) {
                slot.first = std::static_pointer_cast<HipDoubleBuffer>(existing->second->m_storage);
                m_batched_tensors[src] = existing->second;
            } else {
                const Dims dims = src->m_dims.batch(ps.batch_size);
                // The reference front end declares the classifier's loss as {1,1} although one value
                // per sample is written and read (src/node.cpp:336-337, test/test_classifier.cpp:711-716;
                // there the page granularity of managed memory absorbs it): a batched tensor's buffers
                // hold at least one element per sample.
                const size_t elements = std::max<size_t>(dims.elements(), (size_t)std::max(ps.batch_size, 1));
                auto st = std::make_shared<HipDoubleBuffer>(src->m_data_type, elements, m_ctx.get());
                auto t = std::make_shared<HipTensor>(st, dims, hip_strides(dims, layoutFor(src->m_data_type)), 0,
                                                     src->m_name);
                t->copyFromHost(*src);
                m_ctx->m_tensors[src] = t;
                m_batched_tensors[src] = t;
                slot.first = st;
            }
            slot.second = (Phase)0;
        }
        if(!(slot.second & Phase::POST) && !!(bt.second & Phase::POST))
            m_ctx->m_exported.push_back(slot.first);
        slot.second = slot.second | bt.second;
    }
}

// ---------------------------------------------------------------- finalize

// Backward liveness over the op list, treated as one iteration of a loop: a storage is needed
// at the end of the step if the host can see it or if the next step reads it before writing
// it (weights, running statistics, optimizer state).  Operations none of whose outputs are
// needed are dropped; single unneeded outputs are offered to killOutput()
// (reference: reduceLiveranges, src/cuda/cuda_analysis.cpp:328-374).
void HipProgram::eliminateDeadOps()
{
    std::set<HipStorage *> live;
    for(const auto &s : m_ctx->m_exported)
        live.insert(s.get());
    {
        std::set<HipStorage *> written;
        for(const auto &op : m_ops) {
            for(const auto &i : op->getInputs())
                if(!written.count(i.second->m_storage.get()))
                    live.insert(i.second->m_storage.get()); // read before written: carried across steps
            for(const auto &o : op->getOutputs())
                written.insert(o.second->m_storage.get());
        }
    }
    HipOps kept;
    for(auto it = m_ops.rbegin(); it != m_ops.rend(); ++it) {
        auto &op = *it;
        bool needed = false;
        for(const auto &o : op->getOutputs())
            if(live.count(o.second->m_storage.get()))
                needed = true;
        if(!needed)
            continue;
        for(const auto &o : op->getOutputs()) {
            HipStorage *s = o.second->m_storage.get();
            if(!live.count(s)) {
                op->killOutput(o.second->m_storage);
                continue;
            }
            float *beta = op->getBeta(o.second);
            const bool overwrites = !(beta && *beta != 0.0f) && o.second->m_dims.elements() == s->m_elements;
            const bool pinned =
                std::any_of(m_ctx->m_exported.begin(), m_ctx->m_exported.end(), [&](auto &e) { return e.get() == s; });
            if(overwrites && !pinned)
                live.erase(s);
        }
        for(const auto &i : op->getInputs())
            live.insert(i.second->m_storage.get());
        kept.push_back(op);
    }
    std::reverse(kept.begin(), kept.end());
    m_ops = kept;
}

// reference: finalize, src/cuda/cuda_program.cpp:406-475
void HipProgram::finalize()
{
    if(m_finalized)
        return;
    m_finalized = true;

    for(const auto &kv : m_ctx->m_deferred_copy)
        kv.first->copyFromHost(*kv.second);
    m_ctx->m_deferred_copy.clear();

    for(auto &pu : m_units) {
        m_ops.insert(m_ops.end(), pu.m_fwd.begin(), pu.m_fwd.end());
        m_ops.insert(m_ops.end(), pu.m_bwd.begin(), pu.m_bwd.end());
        m_ops.insert(m_ops.end(), pu.m_tail.begin(), pu.m_tail.end());
        pu.m_fwd.clear();
        pu.m_bwd.clear();
        pu.m_tail.clear();
    }

    // When several operations write the same tensor the results are summed: every writer after
    // the first accumulates (beta = 1).  This is how gradients that fan in (skip connections)
    // are added inside the convolution / GEMM epilogue (reference: src/cuda/cuda_program.cpp:429-453).
    // An accumulating writer reads its output, so the dead-op pass below keeps the first writer
    // whenever it keeps a later one.
    if(m_pt == ProgramType::TRAINING)
        reorder_sparse_first_writers(m_ops);
    std::set<HipTensor *> written;
    for(auto &op : m_ops) {
        for(auto &o : op->listOutputs()) {
            if(written.insert(o.second.get()).second)
                continue;
            float *beta = op->getBeta(o.second);
            if(!beta)
                throw std::runtime_error(fmt("Operation ''%s'' does not support beta for %s", op->str().c_str(), o.first));
            if(*beta == 0.0f)
                *beta = 1.0f;
        }
    }

    // optimizers read every gradient, so they keep the weight-gradient ops alive
    m_ops.insert(m_ops.end(), m_opt.begin(), m_opt.end());
    m_opt.clear();

    eliminateDeadOps();
    if(m_pt == ProgramType::TRAINING) {
        link_bn_backward(*this, m_ops);
        fuse_bn_pooling(*this, m_ops);
    }

    m_ctx->m_workspace.alloc();
    m_ctx->m_programs.push_back(this);
    m_ctx->planMemory();
}

// ---------------------------------------------------------------- run loop

void HipProgram::runCallbacks(const TensorBatchCallback &cb, long batch, Phase phase)
{
    if(!cb)
        return;
    std::unordered_map<std::shared_ptr<Tensor>, TensorAccess *> amap;
    std::vector<std::unique_ptr<TensorAccess>> keep;
    for(const auto &bt : m_batched) {
        if(!(bt.second.second & phase))
            continue;
        auto ta = m_batched_tensors[bt.first]->access();
        amap[bt.first] = ta.get();
        keep.push_back(std::move(ta));
    }
    cb(batch, *this, amap);
}

// Upload what the host wrote into the back buffers, then swap front and back.  The uploads go to the
// copy stream: the operations of the step in flight only touch the front buffers, so the transfer
// overlaps them; every caller synchronises both streams (HipContext::sync) before the next step is
// enqueued, which is when the swapped buffers are first read.
void HipProgram::flip(Phase upload_phase)
{
    for(auto &bt : m_batched) {
        if(!!(bt.second.second & upload_phase))
            bt.second.first->uploadBack(m_ctx->m_copy_stream);
        bt.second.first->flip();
    }
}

void HipProgram::checkAnomaly(HipOperation &op, const HipOpArgs &tensors, const char *what)
{
    for(const auto &t : tensors) {
        if(t.second->m_data_type != Tensor::DataType::HALF && t.second->m_data_type != Tensor::DataType::FLOAT)
            continue;
        if(t.second->m_storage->m_nonfinite_is_valid)
            continue;
        auto ta = t.second->access();
        bool bad = false;
        Dims c(t.second->m_dims.size(), (int64_t)0);
        const std::vector<int64_t> ext = t.second->m_dims.i64();
        std::vector<int64_t> cur(ext.size(), 0);
        const size_t n = t.second->m_dims.elements();
        for(size_t i = 0; i < n && !bad; i++) {
            if(!std::isfinite((double)ta->get(c)))
                bad = true;
            for(ssize_t j = (ssize_t)ext.size() - 1; j >= 0; j--) {
                if(++cur[j] == ext[j]) {
                    cur[j] = 0;
                    c[j] = (int64_t)0;
                } else {
                    c[j] = cur[j];
                    break;
                }
            }
        }
        if(bad) {
            fprintf(stderr, "\n\n *** Anomaly in tensor %s (%s)\n", t.second->info().c_str(), what);
            op.dump(stderr, true);
            // the reference aborts (src/cuda/cuda_program.cpp:163-211); a host that wants to survive the report
            // (a test, a service) asks for an exception instead
            if(getenv("SAGA_HIP_ANOMALY_THROW"))
                throw std::runtime_error(fmt("Anomaly in tensor %s (%s of %s)", t.second->info().c_str(), what,
                                             op.name().c_str()));
            abort();
        }
    }
}

void HipProgram::setProfiling(bool on)
{
    m_profiling = on;
    m_profile.clear();
}

std::vector<HipProgram::ProfileRow> HipProgram::profile() const
{
    std::vector<ProfileRow> r;
    for(const auto &kv : m_profile)
        r.push_back(kv.second);
    return r;
}

// after the step's synchronisation: turn the event pairs into per-kind totals
void HipProgram::collectProfile()
{
    if(!m_profiling || m_events.size() < m_ops.size() + 1)
        return;
    for(size_t i = 0; i < m_ops.size(); i++) {
        float ms = 0;
        if(hipEventElapsedTime(&ms, m_events[i], m_events[i + 1]) != hipSuccess)
            continue;
        // SAGA_HIP_PROFILE_PER_OP=1: one row per operation (kind#position) instead of per kind
        static const bool per_op = getenv("SAGA_HIP_PROFILE_PER_OP") != nullptr;
        const std::string key = per_op ? fmt("%s#%03zu", m_ops[i]->name().c_str(), i) : m_ops[i]->name();
        auto &row = m_profile[key];
        row.kind = key;
        row.launches++;
        row.ms += ms;
        row.flops += m_ops[i]->flops();
        row.bytes += m_ops[i]->bytes();
    }
}

// ---- HIP graphs (opt-in: SAGA_HIP_GRAPH=1)
//
// A training step of a small network is a few hundred launches of a few microseconds each.  After two
// plain steps (first-step behaviour such as adopting the batch statistics is over, every lazily allocated
// buffer exists) the operation list is cut into runs of graph-safe operations; each run is recorded from
// the stream into a graph - once per combination of front buffers, because batched tensors alternate
// between two device buffers - and replayed with a single launch.  Operations in between (loss-scaled
// classifier gradient, optimizer) run as before.  No memset nodes are recorded: no operation clears
// memory with hipMemsetAsync.  Measured on MI355X the replay is bit-identical and NOT faster (ResNet-20
// b128: 1.72 ms per step either way; ResNet-50 b256: 25.26 ms either way): the step is a chain of
// dependent kernels, and the ~7 us per link is spent on the GPU between two dependent dispatches, not on
// the host enqueueing them.  Hence off unless asked for.

bool HipProgram::graphsEnabled() const
{
    const char *e = getenv("SAGA_HIP_GRAPH"); // read per step: a test can switch within a process
    const bool on = e && *e && *e != '0';
    return on && !m_profiling && !m_pc.anomaly_detect && !m_debug && m_steps_run >= 2;
}

void HipProgram::dropGraphs()
{
    for(auto &sg : m_segments) {
        for(auto &kv : sg.exec)
            if(kv.second)
                (void)hipGraphExecDestroy(kv.second);
        sg.exec.clear();
    }
}

void HipProgram::runOpsGraphed()
{
    constexpr size_t MIN_RUN = 8; // shorter runs are not worth a graph launch
    if(m_segments.empty()) {
        size_t i = 0;
        while(i < m_ops.size()) {
            size_t j = i;
            while(j < m_ops.size() && m_ops[j]->graphSafe())
                j++;
            GraphSegment sg;
            sg.begin = i;
            if(j - i >= MIN_RUN) {
                sg.end = j;
                sg.graph = true;
            } else {
                sg.end = j < m_ops.size() ? j + 1 : j; // the short run and the operation that ended it
            }
            m_segments.push_back(sg);
            i = sg.end;
        }
        std::set<HipStorage *> seen;
        for(auto &op : m_ops)
            for(const auto &list : {op->listInputs(), op->listOutputs()})
                for(const auto &t : list) {
                    HipStorage *st = t.second->m_storage.get();
                    if(st->doubleBuffered() && seen.insert(st).second)
                        m_graph_dbufs.push_back(static_cast<HipDoubleBuffer *>(st));
                }
    }
    if(m_graph_dbufs.size() > 16) { // one recording per combination of front buffers: keep that bounded
        for(auto &op : m_ops) {
            try {
                op->exec(*this);
            } catch(const std::exception &ex) {
                throw std::runtime_error(fmt("Op %s failed -- %s", op->name().c_str(), ex.what()));
            }
        }
        return;
    }
    unsigned key = 0;
    for(size_t i = 0; i < m_graph_dbufs.size(); i++)
        key |= (unsigned)m_graph_dbufs[i]->m_index << i;
    if(m_graph_epoch != m_ctx->m_mem_epoch || m_graph_ws != m_ctx->m_workspace.ptr()) {
        dropGraphs();
        m_graph_epoch = m_ctx->m_mem_epoch;
        m_graph_ws = m_ctx->m_workspace.ptr();
    }
    hipStream_t st = m_ctx->m_stream;
    auto exec_range = [&](size_t b, size_t e) {
        for(size_t i = b; i < e; i++) {
            try {
                m_ops[i]->exec(*this);
            } catch(const std::exception &ex) {
                throw std::runtime_error(fmt("Op %s failed -- %s", m_ops[i]->name().c_str(), ex.what()));
            }
        }
    };
    for(auto &sg : m_segments) {
        if(!sg.graph) {
            exec_range(sg.begin, sg.end);
            continue;
        }
        hipGraphExec_t &ge = sg.exec[key];
        if(!ge) {
            chkHip(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
            hipGraph_t graph = nullptr;
            try {
                exec_range(sg.begin, sg.end);
            } catch(...) {
                (void)hipStreamEndCapture(st, &graph);
                if(graph)
                    (void)hipGraphDestroy(graph);
                throw;
            }
            chkHip(hipStreamEndCapture(st, &graph));
            const hipError_t e = hipGraphInstantiate(&ge, graph, nullptr, nullptr, 0);
            (void)hipGraphDestroy(graph);
            chkHip(e);
            if(getenv("SAGA_HIP_GRAPH_VERBOSE"))
                fprintf(stderr, "saga-hip: program %d recorded operations %zu..%zu into a graph (front buffers %#x)\n",
                        m_index, sg.begin, sg.end - 1, key);
        }
        chkHip(hipGraphLaunch(ge, st));
    }
}

void HipProgram::runOps(const HipOps &ops)
{
    if(&ops == &m_ops) {
        if(graphsEnabled()) {
            runOpsGraphed();
            m_steps_run++;
            return;
        }
        m_steps_run++;
    }
    if(m_profiling) {
        while(m_events.size() < ops.size() + 1) {
            hipEvent_t e;
            chkHip(hipEventCreate(&e));
            m_events.push_back(e);
        }
        chkHip(hipEventRecord(m_events[0], m_ctx->m_stream));
    }
    size_t index = 0;
    const bool poison = m_pc.anomaly_detect && &ops == &m_ops && m_poison_before.size() == ops.size();
    auto fill_nan = [&](const std::vector<HipStorage *> &list) {
        for(HipStorage *s : list)
            if(s->m_in_arena)
                chkSaga(saga_hip_fill(s->m_data, 0xff, s->bytes(), (saga_stream_t)m_ctx->m_stream));
    };
    for(const auto &op : ops) {
        if(poison)
            fill_nan(m_poison_before[index]);
        if(m_pc.anomaly_detect)
            checkAnomaly(*op, op->getInputs(), "input");
        try {
            op->exec(*this);
        } catch(const std::exception &e) {
            throw std::runtime_error(fmt("Op %s failed -- %s", op->name().c_str(), e.what()));
        }
        if(m_pc.anomaly_detect)
            checkAnomaly(*op, op->getOutputs(), "output");
        if(poison)
            fill_nan(m_poison_after[index]);
        index++;
        if(m_profiling)
            chkHip(hipEventRecord(m_events[index], m_ctx->m_stream));
    }
}

void HipProgram::prep(long, long batch_offset)
{
    finalize();
    runCallbacks(m_pc.pre_ops, 0 + batch_offset, Phase::PRE);
    flip(Phase::PRE);
    m_ctx->sync();
    m_total_samples = 0;
    m_epoch_start = now();
}

// reference: step, src/cuda/cuda_program.cpp:261-320
void HipProgram::step(long batch, long batches, long batch_offset)
{
    runOps(m_ops);
    for(auto &bt : m_batched)
        if(!!(bt.second.second & Phase::POST))
            bt.second.first->downloadFront(m_ctx->m_stream);

    // host work for the neighbouring batches overlaps the GPU work enqueued above
    if(batch > 0)
        runCallbacks(m_pc.post_ops, batch - 1 + batch_offset, Phase::POST);
    if(batch < batches - 1)
        runCallbacks(m_pc.pre_ops, batch + 1 + batch_offset, Phase::PRE);
    flip(Phase::PRE);

    for(const auto &u : m_units)
        m_total_samples += u.m_batch_size;

    m_ctx->sync(); // the only synchronisation per step
    collectProfile();

    if(m_mp_enabled) {
        // loss-scale controller (reference: src/cuda/cuda_program.cpp:295-307)
        if(m_aux->inf || m_aux->nan)
            m_mp_scaling *= 0.5;
        else if(m_aux->range > 1)
            m_mp_scaling *= 0.9;
        else
            m_mp_scaling *= 1.02;
        m_aux->range = 0;
        m_aux->inf = 0;
        m_aux->nan = 0;
    }
    const float sps = m_total_samples / (1e-6 * (now() - m_epoch_start));
    m_ctx->m_ui->updateCell(m_ctx->getUiPage(), getUiRow(), 7, UI::Align::LEFT, "%ld (%.1f/s)", (long)m_total_samples, sps);
    if(m_mp_enabled)
        m_ctx->m_ui->updateCell(m_ctx->getUiPage(), getUiRow(), 9, UI::Align::LEFT, "%.1e", m_mp_scaling);
}

void HipProgram::post(long batches, long batch_offset)
{
    runCallbacks(m_pc.post_ops, batches - 1 + batch_offset, Phase::POST);
}

ExecResult HipProgram::run(long batches, StopCheck stop_check, long batch_offset)
{
    if(batches == 0)
        return ExecResult::OK;
    if(stop_check && stop_check())
        return ExecResult::STOPPED;
    chkHip(hipSetDevice(m_ctx->m_device));
    prep(batches, batch_offset);
    for(long i = 0; i < batches; i++) {
        step(i, batches, batch_offset);
        if(stop_check && stop_check())
            return ExecResult::STOPPED;
    }
    post(batches, batch_offset);
    return ExecResult::OK;
}

void HipProgram::dump(FILE *output, bool detailed)
{
    finalize();
    fprintf(output, "\n%zd ops\n", m_ops.size());
    int index = 0;
    for(const auto &op : m_ops) {
        fprintf(output, "#%3d: ", index++);
        op->dump(output, detailed);
    }
}

bool HipProgram::dumpGraph(const char *path)
{
    finalize();
    FILE *fp = fopen(path, "w");
    if(!fp)
        return false;
    fprintf(fp, "digraph HipOps {\n");
    std::set<std::string> storages;
    int i = 0;
    for(auto &op : m_ops) {
        fprintf(fp, "node [shape=circle,label=\"%s\"]; O%d;\n", op->name().c_str(), i++);
        for(const auto &t : op->getInputs())
            storages.insert(fmt("T%d", t.second->m_storage->m_id));
        for(const auto &t : op->getOutputs())
            storages.insert(fmt("T%d", t.second->m_storage->m_id));
    }
    for(const auto &s : storages)
        fprintf(fp, "node [shape=box,label=\"%s\"]; %s;\n", s.c_str(), s.c_str());
    i = 0;
    for(auto &op : m_ops) {
        for(const auto &t : op->getInputs())
            fprintf(fp, "T%d->O%d;\n", t.second->m_storage->m_id, i);
        for(const auto &t : op->getOutputs())
            fprintf(fp, "O%d->T%d;\n", i, t.second->m_storage->m_id);
        i++;
    }
    fprintf(fp, "overlap=false\n}\n");
    fclose(fp);
    return true;
}

}  // namespace saga

// C API over the C++ front end and the hip engine, for callers without a C++ toolchain
// (the Python tests and bench.py bind it with ctypes).  Declarations: include/saga_capi.h.
#include <string.h>

#include <algorithm>
#include <mutex>

#include "saga.hpp"
#include "saga_capi.h"
#include "hip/hip_common.hpp"

using namespace saga;

namespace {

thread_local std::string g_error;

struct TensorBox {
    std::shared_ptr<Tensor> t;
};
struct NodeBox {
    std::shared_ptr<Node> n;
};
struct GraphBox {
    Graph g;
};
struct ContextBox {
    std::shared_ptr<Context> c;
};
struct ProgramBox {
    std::shared_ptr<Program> p;
};

template <typename F> int guard(F &&f)
{
    try {
        f();
        return 0;
    } catch(const std::exception &e) {
        g_error = e.what();
        return -1;
    }
}

Dims make_dims(int rank, const int64_t *dims)
{
    Dims d;
    for(int i = 0; i < rank; i++) {
        if(dims[i] == SAGA_DIM_BATCH)
            d.push_back(DimParam::BATCH_SIZE);
        else
            d.push_back(dims[i]);
    }
    return d;
}

saga_tensor_t box(std::shared_ptr<Tensor> t) { return t ? new TensorBox{t} : nullptr; }

}  // namespace

extern "C" {

const char *saga_last_error(void) { return g_error.c_str(); }

saga_tensor_t saga_tensor_create(int dtype, int rank, const int64_t *dims, const char *name, int with_storage)
{
    saga_tensor_t r = nullptr;
    guard([&] {
        const auto nm = name ? std::make_optional<const std::string>(name) : std::nullopt;
        const Dims d = make_dims(rank, dims);
        r = box(with_storage ? makeCPUTensor((Tensor::DataType)dtype, d, nm) : makeTensor((Tensor::DataType)dtype, d, nm));
    });
    return r;
}

void saga_tensor_release(saga_tensor_t t) { delete (TensorBox *)t; }

saga_tensor_t saga_tensor_grad(saga_tensor_t t)
{
    saga_tensor_t r = nullptr;
    guard([&] { r = box(((TensorBox *)t)->t->grad()); });
    return r;
}

int saga_tensor_rank(saga_tensor_t t) { return (int)((TensorBox *)t)->t->m_dims.size(); }

int saga_tensor_dtype(saga_tensor_t t) { return (int)((TensorBox *)t)->t->m_data_type; }

int saga_tensor_dims(saga_tensor_t t, int64_t *out)
{
    return guard([&] {
        const auto &d = ((TensorBox *)t)->t->m_dims;
        for(size_t i = 0; i < d.size(); i++) {
            if(auto v = std::get_if<int64_t>(&d[i]))
                out[i] = *v;
            else
                out[i] = SAGA_DIM_BATCH;
        }
    });
}

// payload is the tensor's elements in logical row-major order, in the tensor's own data type
static int transfer(saga_tensor_t tb, void *buf, size_t bytes, bool write)
{
    return guard([&] {
        auto &t = ((TensorBox *)tb)->t;
        auto ta = t->access();
        if(!ta)
            throw std::runtime_error("tensor has no storage: " + t->info());
        const size_t es = Tensor::DataTypeSize(t->m_data_type);
        const size_t n = t->m_dims.elements();
        if(bytes != n * es)
            throw std::runtime_error(fmt("payload is %zd bytes, tensor %s needs %zd", bytes, t->info().c_str(), n * es));
        const size_t rank = t->m_dims.size();
        const std::vector<int64_t> ext = t->m_dims.i64();
        const std::vector<int64_t> str = ta->strides().i64();
        char *base = (char *)ta->data();
        if(!base)
            throw std::runtime_error("tensor exposes no host memory: " + t->info());
        if(write)
            (void)ta->getAddr(Dims(rank, (int64_t)0)); // marks staged device tensors dirty
        // innermost logical dim is copied with one memcpy when it is contiguous
        const size_t inner = rank ? (size_t)ext[rank - 1] : 1;
        const bool inner_contig = rank == 0 || str[rank - 1] == 1 || inner == 1;
        std::vector<int64_t> c(rank, 0);
        const size_t outer = rank ? n / inner : 1;
        char *p = (char *)buf;
        for(size_t o = 0; o < outer; o++) {
            int64_t off = 0;
            for(size_t j = 0; j + 1 < rank; j++)
                off += c[j] * str[j];
            if(inner_contig) {
                if(write)
                    memcpy(base + off * es, p, inner * es);
                else
                    memcpy(p, base + off * es, inner * es);
                p += inner * es;
            } else {
                for(size_t i = 0; i < inner; i++, p += es) {
                    char *e = base + (off + (int64_t)i * str[rank - 1]) * es;
                    if(write)
                        memcpy(e, p, es);
                    else
                        memcpy(p, e, es);
                }
            }
            for(ssize_t j = (ssize_t)rank - 2; j >= 0; j--) {
                if(++c[j] == ext[j])
                    c[j] = 0;
                else
                    break;
            }
        }
    });
}

int saga_tensor_write(saga_tensor_t t, const void *data, size_t bytes) { return transfer(t, (void *)data, bytes, true); }

int saga_tensor_read(saga_tensor_t t, void *data, size_t bytes) { return transfer(t, data, bytes, false); }

int saga_tensor_save(saga_tensor_t t, const char *path) { return ((TensorBox *)t)->t->save(path) ? 0 : -1; }

saga_tensor_t saga_tensor_load(const char *path, const char *name)
{
    return box(Tensor::load(path, name ? std::make_optional<const std::string>(name) : std::nullopt));
}

double saga_tensor_sse(saga_tensor_t a, saga_tensor_t b)
{
    double r = -1;
    guard([&] { r = ((TensorBox *)a)->t->sse(*((TensorBox *)b)->t); });
    return r;
}

saga_graph_t saga_graph_create(void) { return new GraphBox(); }

void saga_graph_release(saga_graph_t g) { delete (GraphBox *)g; }

static Attributes make_attrs(int n, const saga_attr_t *attrs)
{
    Attributes a;
    for(int i = 0; i < n; i++) {
        switch(attrs[i].kind) {
        case SAGA_ATTR_INT: a[attrs[i].name] = (int)attrs[i].i; break;
        case SAGA_ATTR_FLOAT: a[attrs[i].name] = (float)attrs[i].f; break;
        case SAGA_ATTR_BOOL: a[attrs[i].name] = (bool)(attrs[i].i != 0); break;
        case SAGA_ATTR_INTS: a[attrs[i].name] = std::vector<int>(attrs[i].ints, attrs[i].ints + attrs[i].n_ints); break;
        case SAGA_ATTR_DIMS: {
            Dims d;
            for(int j = 0; j < attrs[i].n_ints; j++) {
                const int v = attrs[i].ints[j];
                if(v == SAGA_DIM_UNCHANGED)
                    d.push_back(DimParam::UNCHANGED);
                else if(v == SAGA_DIM_REDUCE)
                    d.push_back(DimParam::REDUCE);
                else if(v == SAGA_DIM_BATCH)
                    d.push_back(DimParam::BATCH_SIZE);
                else
                    d.push_back((int64_t)v);
            }
            a[attrs[i].name] = d;
            break;
        }
        default: throw std::runtime_error("bad attribute kind");
        }
    }
    return a;
}

saga_node_t saga_graph_add_node(saga_graph_t g, const char *type, int n_inputs, const char *const *input_names,
                                const saga_tensor_t *inputs, int n_attrs, const saga_attr_t *attrs, const char *name)
{
    saga_node_t r = nullptr;
    guard([&] {
        Tensors in;
        for(int i = 0; i < n_inputs; i++)
            in[input_names[i]] = ((TensorBox *)inputs[i])->t;
        auto n = ((GraphBox *)g)->g.addNode(type, in, make_attrs(n_attrs, attrs),
                                            name ? std::make_optional<const std::string>(name) : std::nullopt);
        r = n ? new NodeBox{n} : nullptr;
    });
    return r;
}

saga_node_t saga_graph_add_resnet_bottleneck(saga_graph_t g, saga_tensor_t input, int squeeze, int output,
                                             int downsample, const char *name)
{
    saga_node_t r = nullptr;
    guard([&] {
        r = new NodeBox{((GraphBox *)g)->g.addResNetBottleNeck(((TensorBox *)input)->t, squeeze, output, downsample != 0, name)};
    });
    return r;
}

saga_node_t saga_graph_add_resnet(saga_graph_t g, saga_tensor_t input, int output, int downsample, const char *name)
{
    saga_node_t r = nullptr;
    guard([&] { r = new NodeBox{((GraphBox *)g)->g.addResNet(((TensorBox *)input)->t, output, downsample != 0, name)}; });
    return r;
}

saga_graph_t saga_graph_load(const char *path)
{
    auto g = Graph::load(path);
    if(!g) {
        g_error = std::string("unable to load ") + path;
        return nullptr;
    }
    return new GraphBox{*g};
}

saga_tensor_t saga_tensor_load_protobuf(const char *path)
{
    auto t = Tensor::loadProtoBuf(path);
    if(!t) {
        g_error = std::string("unable to load ") + path;
        return nullptr;
    }
    return box(t);
}

// graph inputs / outputs in name order (the sets themselves have no order)
static std::vector<std::shared_ptr<Tensor>> sorted_io(saga_graph_t g, int outputs)
{
    auto &set = outputs ? ((GraphBox *)g)->g.m_outputs : ((GraphBox *)g)->g.m_inputs;
    std::vector<std::shared_ptr<Tensor>> v(set.begin(), set.end());
    std::sort(v.begin(), v.end(), [](const std::shared_ptr<Tensor> &a, const std::shared_ptr<Tensor> &b) {
        return a->m_name.value_or("") < b->m_name.value_or("");
    });
    return v;
}

int saga_graph_io_count(saga_graph_t g, int outputs) { return (int)sorted_io(g, outputs).size(); }

saga_tensor_t saga_graph_io(saga_graph_t g, int outputs, int index)
{
    const auto v = sorted_io(g, outputs);
    return index >= 0 && index < (int)v.size() ? box(v[index]) : nullptr;
}

int saga_graph_describe(saga_graph_t g, char *buf, size_t capacity)
{
    std::string out;
    auto slots = [&](const Tensors &ts) {
        std::vector<std::string> names;
        for(const auto &t : ts)
            names.push_back(t.first);
        std::sort(names.begin(), names.end());
        std::string r;
        for(const auto &n : names) {
            const auto &t = ts.find(n)->second;
            r += (r.empty() ? "" : " ") + n + "=" + (t ? t->m_name.value_or("?") + ":" + Tensor::DataTypeStr(t->m_data_type) + t->m_dims.to_string() : "null");
        }
        return r;
    };
    for(const auto &n : ((GraphBox *)g)->g.m_nodes) {
        std::vector<std::string> an;
        for(const auto &a : n->m_attributes)
            an.push_back(a.first);
        std::sort(an.begin(), an.end());
        std::string attrs;
        for(const auto &a : an)
            attrs += (attrs.empty() ? "" : " ") + a + "=" + n->m_attributes.find(a)->second.to_string();
        out += n->m_type + " | " + slots(n->m_inputs) + " | " + attrs + " | " + slots(n->m_outputs) + "\n";
    }
    if(buf && capacity) {
        const size_t c = std::min(capacity - 1, out.size());
        memcpy(buf, out.data(), c);
        buf[c] = 0;
    }
    return (int)out.size();
}

int saga_graph_node_count(saga_graph_t g) { return (int)((GraphBox *)g)->g.m_nodes.size(); }

int saga_graph_save_tensors(saga_graph_t g, const char *path, saga_context_t ctx)
{
    return ((GraphBox *)g)->g.saveTensors(path, ctx ? ((ContextBox *)ctx)->c.get() : nullptr) ? 0 : -1;
}

int saga_graph_load_tensors(saga_graph_t g, const char *path)
{
    return guard([&] { ((GraphBox *)g)->g.loadTensors(path); });
}

saga_tensor_t saga_graph_named_tensor(saga_graph_t g, const char *name)
{
    auto &nt = *((GraphBox *)g)->g.m_named_tensors;
    auto it = nt.find(name);
    return it == nt.end() ? nullptr : box(it->second);
}

void saga_node_release(saga_node_t n) { delete (NodeBox *)n; }

saga_tensor_t saga_node_output(saga_node_t n, const char *slot)
{
    auto &o = ((NodeBox *)n)->n->m_outputs;
    auto it = o.find(slot);
    return it == o.end() ? nullptr : box(it->second);
}

saga_tensor_t saga_node_input(saga_node_t n, const char *slot)
{
    auto &o = ((NodeBox *)n)->n->m_inputs;
    auto it = o.find(slot);
    return it == o.end() ? nullptr : box(it->second);
}

saga_context_t saga_context_create(void)
{
    saga_context_t r = nullptr;
    guard([&] { r = new ContextBox{createContext()}; });
    return r;
}

void saga_context_release(saga_context_t c) { delete (ContextBox *)c; }

int saga_context_reset(saga_context_t c)
{
    return guard([&] { ((ContextBox *)c)->c->reset(); });
}

saga_tensor_t saga_context_resolve(saga_context_t c, saga_tensor_t t)
{
    saga_tensor_t r = nullptr;
    guard([&] { r = box(((ContextBox *)c)->c->resolveTensor(((TensorBox *)t)->t)); });
    return r;
}

saga_program_t saga_program_create(saga_context_t c, saga_graph_t g, int batch_size, int training,
                                   const saga_program_config_t *cfg, int n_batched, const saga_tensor_t *batched,
                                   const int *phases)
{
    saga_program_t r = nullptr;
    guard([&] {
        ProgramConfig pc;
        if(cfg) {
            pc.learning_rate = cfg->learning_rate;
            pc.l2_lambda = cfg->l2_lambda;
            pc.bn_expavg = cfg->bn_expavg;
            pc.tensor_layout = (TensorLayout)cfg->tensor_layout;
            pc.anomaly_detect = cfg->anomaly_detect != 0;
            pc.disable_op_fusing = cfg->disable_op_fusing != 0;
            pc.initial_loss_scale = cfg->initial_loss_scale;
        }
        BatchedTensors bt;
        for(int i = 0; i < n_batched; i++)
            bt[((TensorBox *)batched[i])->t] = (Phase)phases[i];
        ProgramSource ps{((GraphBox *)g)->g, bt, batch_size};
        r = new ProgramBox{((ContextBox *)c)
                               ->c->createProgram(ps, training ? ProgramType::TRAINING : ProgramType::INFERENCE, pc)};
    });
    return r;
}

void saga_program_release(saga_program_t p) { delete (ProgramBox *)p; }

int saga_program_finalize(saga_program_t p)
{
    return guard([&] { ((ProgramBox *)p)->p->finalize(); });
}

int saga_program_run(saga_program_t p, long batches)
{
    int rc = 0;
    const int g = guard([&] { rc = ((ProgramBox *)p)->p->run(batches) == ExecResult::OK ? 0 : 1; });
    return g ? g : rc;
}

int saga_context_memory(saga_context_t c, size_t *arena_bytes, size_t *planned_bytes)
{
    return guard([&] {
        auto hc = std::dynamic_pointer_cast<HipContext>(((ContextBox *)c)->c);
        if(!hc)
            throw std::runtime_error("not a hip context");
        if(arena_bytes)
            *arena_bytes = hc->m_arena_bytes;
        if(planned_bytes)
            *planned_bytes = hc->m_planned_bytes;
    });
}

double saga_program_loss_scale(saga_program_t p) { return ((ProgramBox *)p)->p->getMPS(); }

static int optimizer_state(saga_program_t p, const char *path, bool save)
{
    return guard([&] {
        auto hp = std::dynamic_pointer_cast<HipProgram>(((ProgramBox *)p)->p);
        if(!hp)
            throw std::runtime_error("not a hip program");
        if(!path)
            throw std::runtime_error("no path");
        if(save)
            hp->saveOptimizerState(path);
        else
            hp->loadOptimizerState(path);
    });
}

int saga_program_save_optimizer(saga_program_t p, const char *path) { return optimizer_state(p, path, true); }
int saga_program_load_optimizer(saga_program_t p, const char *path) { return optimizer_state(p, path, false); }

int saga_program_set_profiling(saga_program_t p, int on)
{
    return guard([&] {
        auto hp = std::dynamic_pointer_cast<HipProgram>(((ProgramBox *)p)->p);
        if(!hp)
            throw std::runtime_error("not a hip program");
        hp->setProfiling(on != 0);
    });
}

int saga_program_profile(saga_program_t p, saga_profile_row_t *rows, int capacity)
{
    int n = -1;
    guard([&] {
        auto hp = std::dynamic_pointer_cast<HipProgram>(((ProgramBox *)p)->p);
        if(!hp)
            throw std::runtime_error("not a hip program");
        const auto prof = hp->profile();
        n = 0;
        for(const auto &r : prof) {
            if(n >= capacity)
                break;
            strncpy(rows[n].kind, r.kind.c_str(), sizeof(rows[n].kind) - 1);
            rows[n].kind[sizeof(rows[n].kind) - 1] = 0;
            rows[n].launches = r.launches;
            rows[n].ms = r.ms;
            rows[n].flops = r.flops;
            rows[n].bytes = r.bytes;
            n++;
        }
    });
    return n;
}

int saga_program_dump(saga_program_t p, const char *path, int detailed)
{
    return guard([&] {
        FILE *f = path ? fopen(path, "w") : stdout;
        if(!f)
            throw std::runtime_error("cannot open dump file");
        ((ProgramBox *)p)->p->dump(f, detailed != 0);
        if(path)
            fclose(f);
    });
}

}  // extern "C"

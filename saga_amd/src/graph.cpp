// Graph bookkeeping and the residual-block builders.  Block structure (layer order, names,
// v1.5 stride placement, projection rule) follows the reference's src/graph.cpp:273-425.
#include <dirent.h>
#include <errno.h>
#include <limits.h>
#include <string.h>
#include <sys/stat.h>

#include "saga.hpp"

namespace saga {

const std::shared_ptr<Tensor> Tensors::operator[](const std::string &n) const
{
    auto it = find(n);
    if(it == end())
        throw std::runtime_error{fmt("tensor-%s not found", n.c_str())};
    return it->second;
}

bool Tensors::has(const std::string &n) const { return find(n) != end(); }

std::shared_ptr<Tensor> &Tensors::operator[](const std::string &n)
{
    return std::unordered_map<std::string, std::shared_ptr<Tensor>>::operator[](n);
}

// one file per tensor, named after it (reference: src/graph.cpp:60-104)
void Tensors::loadTensors(const char *path)
{
    DIR *d = opendir(path);
    if(!d) {
        fprintf(stderr, "Unable to load tensors from %s -- %s\n", path, strerror(errno));
        return;
    }
    while(struct dirent *e = readdir(d)) {
        if(e->d_name[0] == '.')
            continue;
        const std::string file = std::string(path) + "/" + e->d_name;
        if(auto t = Tensor::load(file.c_str(), std::string(e->d_name)))
            (*this)[e->d_name] = t;
    }
    closedir(d);
}

bool Tensors::saveTensors(const char *path, Context *ctx)
{
    mkdir(path, 0777);
    for(const auto &kv : *this) {
        auto t = kv.second;
        if(ctx) {
            t = ctx->resolveTensor(t);
            if(!t)
                continue;
        }
        const std::string file = std::string(path) + "/" + kv.first;
        if(!t->save(file.c_str()))
            return false;
    }
    return true;
}

void Graph::print() const
{
    for(const auto &n : m_nodes)
        n->print();
}

std::shared_ptr<Node> Graph::addNode(const std::string &type, const Tensors &inputs, const Attributes &attributes,
                                     const std::optional<const std::string> &name)
{
    const auto made = Node::make(type, inputs, attributes, *m_named_tensors, name);
    m_nodes.insert(m_nodes.end(), made.begin(), made.end());
    return m_nodes.empty() ? nullptr : m_nodes.back();
}

std::shared_ptr<Node> Graph::addNode(const std::string &type, const std::shared_ptr<Tensor> &t,
                                     const Attributes &attributes, const std::optional<const std::string> &name)
{
    return addNode(type, Tensors{{"x", t}}, attributes, name);
}

std::shared_ptr<Node> Graph::addNode(const std::string &type, const std::shared_ptr<Node> &n,
                                     const Attributes &attributes, const std::optional<const std::string> &name)
{
    return addNode(type, n->y(), attributes, name);
}

std::shared_ptr<Node> Graph::addNode(const std::string &type, Loader loader, const Attributes &attributes)
{
    const auto made = Node::make(type, loader, attributes);
    m_nodes.insert(m_nodes.end(), made.begin(), made.end());
    return m_nodes.empty() ? nullptr : m_nodes.back();
}

// tensors consumed but never produced / produced but never consumed
std::unordered_set<std::shared_ptr<Tensor>> Graph::inputTensors() const
{
    std::unordered_set<std::shared_ptr<Tensor>> r;
    for(const auto &n : m_nodes)
        for(const auto &t : n->m_inputs)
            r.insert(t.second);
    for(const auto &n : m_nodes)
        for(const auto &t : n->m_outputs)
            r.erase(t.second);
    return r;
}

std::unordered_set<std::shared_ptr<Tensor>> Graph::outputTensors() const
{
    std::unordered_set<std::shared_ptr<Tensor>> r;
    for(const auto &n : m_nodes)
        for(const auto &t : n->m_outputs)
            r.insert(t.second);
    for(const auto &n : m_nodes)
        for(const auto &t : n->m_inputs)
            r.erase(t.second);
    return r;
}

std::pair<TensorMapping, TensorMapping> Graph::tensorMappings() const
{
    TensorMapping consumers, producers;
    for(const auto &n : m_nodes) {
        for(const auto &t : n->m_inputs)
            consumers[t.second].push_back({t.first, n});
        for(const auto &t : n->m_outputs)
            producers[t.second].push_back({t.first, n});
    }
    return {consumers, producers};
}

void Graph::loadTensors(const char *path) { m_named_tensors->loadTensors(path); }

bool Graph::saveTensors(const char *path, Context *ctx) { return m_named_tensors->saveTensors(path, ctx); }

void Graph::statsTensors(Context *ctx)
{
    if(!ctx)
        return;
    for(const auto &kv : *m_named_tensors)
        if(auto t = ctx->resolveTensor(kv.second))
            t->printStats(kv.first.c_str());
}

// ---------------------------------------------------------------- builders

std::shared_ptr<Node> Graph::addConvert(std::shared_ptr<Tensor> input, Tensor::DataType dt, float scale)
{
    return addNode("convert", input, {{"scale", scale}, {"datatype", (int)dt}});
}

std::shared_ptr<Node> Graph::addJpegDecoder(int width, int height, Tensor::DataType dt, Loader loader)
{
    auto n = addNode("jpegdecoder", loader, {{"width", width}, {"height", height}});
    return addConvert(n->y(), dt, 1 / 255.0f);
}

std::shared_ptr<Node> Graph::addSpatialTransform(std::shared_ptr<Tensor> input, std::shared_ptr<Tensor> theta,
                                                 int width, int height, bool inference)
{
    Attributes a;
    if(width > 0)
        a["width"] = width;
    if(height > 0)
        a["height"] = height;
    a["inference"] = inference;
    return addNode("spatialtransform", Tensors{{"x", input}, {"theta", theta}}, a);
}

namespace {

struct ConvSpec {
    int size, activations, stride, pad;
    const char *suffix;    // conv node name suffix
    const char *bn_suffix; // batchnorm node name suffix
    bool relu;
};

}  // namespace

// conv -> batchnorm [-> relu] chain; `extra` carries transpose / outputpad attributes
static std::shared_ptr<Node> conv_bn(Graph &g, std::shared_ptr<Tensor> x, const ConvSpec &c, const std::string &name,
                                     const Attributes &extra = {})
{
    Attributes a{{"size", c.size}, {"activations", c.activations}, {"stride", c.stride}, {"pad", c.pad}};
    for(const auto &e : extra)
        a[e.first] = e.second;
    auto n = g.addNode("conv", x, a, name + c.suffix);
    n = g.addNode("batchnorm", n->y(), {}, name + c.bn_suffix);
    if(c.relu)
        n = g.addNode("relu", n->y());
    return n;
}

static std::shared_ptr<Node> residual_tail(Graph &g, std::shared_ptr<Node> branch, std::shared_ptr<Tensor> shortcut)
{
    auto s = g.addNode("sum", Tensors{{"x0", branch->y()}, {"x1", shortcut}}, {});
    return g.addNode("relu", s->y());
}

// 1x1 squeeze, 3x3 (carries the stride: "v1.5"), 1x1 expand; 1x1 projection when the shape changes
std::shared_ptr<Node> Graph::addResNetBottleNeck(std::shared_ptr<Tensor> input, int squeeze_activations,
                                                 int output_activations, bool downsample, const std::string &name)
{
    const int st = downsample ? 2 : 1;
    auto a = conv_bn(*this, input, {1, squeeze_activations, 1, 0, "-conv-1", "-bn-1", true}, name);
    a = conv_bn(*this, a->y(), {3, squeeze_activations, st, 1, "-conv-2", "-bn-2", true}, name);
    a = conv_bn(*this, a->y(), {1, output_activations, 1, 0, "-conv-3", "-bn-3", false}, name);
    std::shared_ptr<Tensor> shortcut = input;
    if(a->y()->m_dims != input->m_dims)
        shortcut = conv_bn(*this, input, {1, output_activations, st, 0, "-conv-p", "-bn-p", false}, name)->y();
    return residual_tail(*this, a, shortcut);
}

std::shared_ptr<Node> Graph::addResNetBottleNeck_transposed(std::shared_ptr<Tensor> input, int squeeze_activations,
                                                            int output_activations, bool upsample,
                                                            const std::string &name)
{
    const int st = upsample ? 2 : 1;
    const int opad = upsample ? 1 : 0;
    const Attributes t{{"transpose", true}};
    const Attributes tp{{"transpose", true}, {"outputpad", opad}};
    auto a = conv_bn(*this, input, {1, squeeze_activations, 1, 0, "-conv-3", "-bn-3t", true}, name, t);
    a = conv_bn(*this, a->y(), {3, squeeze_activations, st, 1, "-conv-2", "-bn-2t", true}, name, tp);
    a = conv_bn(*this, a->y(), {1, output_activations, 1, 0, "-conv-1", "-bn-1t", false}, name, t);
    std::shared_ptr<Tensor> shortcut = input;
    if(a->y()->m_dims != input->m_dims) {
        // the projection keeps the conv default pad (0)
        Attributes pa{{"size", 1}, {"activations", output_activations}, {"stride", st}, {"outputpad", opad},
                      {"transpose", true}};
        auto c = addNode("conv", input, pa, name + "-conv-p");
        c = addNode("batchnorm", c->y(), {}, name + "-bn-pt");
        shortcut = c->y();
    }
    return residual_tail(*this, a, shortcut);
}

// basic block: two 3x3 convs, stride on the first
std::shared_ptr<Node> Graph::addResNet(std::shared_ptr<Tensor> input, int output_activations, bool downsample,
                                       const std::string &name)
{
    const int st = downsample ? 2 : 1;
    auto a = conv_bn(*this, input, {3, output_activations, st, 1, "-conv-1", "-bn-1", true}, name);
    a = conv_bn(*this, a->y(), {3, output_activations, 1, 1, "-conv-2", "-bn-2", false}, name);
    std::shared_ptr<Tensor> shortcut = input;
    if(a->y()->m_dims != input->m_dims)
        shortcut = conv_bn(*this, input, {1, output_activations, st, 0, "-conv-p", "-bn-p", false}, name)->y();
    return residual_tail(*this, a, shortcut);
}

}  // namespace saga

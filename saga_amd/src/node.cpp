// Node construction: implicit parameter tensors and output-shape inference per node type.
// The shape rules, attribute names and defaults, parameter names ("<node>-w", "-b"/"-bt",
// "-s", "-m", "-v") and initialisation constants follow the reference's src/node.cpp, cited
// at each rule; unknown node types are rejected with an exception.
#include <math.h>

#include <map>

#include "saga.hpp"

namespace saga {

namespace {

using Name = std::optional<const std::string>;

Name param_name(const Name &node, const char *suffix)
{
    if(!node)
        return std::nullopt;
    return *node + "-" + suffix;
}

struct NodeType {
    // shape and type of the "y" output
    std::shared_ptr<Tensor> (*infer)(const Node &n, const Name &name);
    // creates implicit inputs / extra outputs; may put helper nodes in front of n
    void (*prepare)(std::shared_ptr<Node> n, std::shared_ptr<Tensor> x, Tensors &named, Nodes &before);
};

std::shared_ptr<Tensor> same_as_x(const Node &n, const Name &name)
{
    auto x = n.m_inputs["x"];
    return makeTensor(x->m_data_type, x->m_dims, name);
}

// ---- conv (reference: src/node.cpp:44-128)
// regular:    O = 1 + (I + 2*pad - ((k-1)*dilation + 1)) / stride
// transposed: O = stride*(I-1) + outputpad + ((k-1)*dilation + 1) - 2*pad
std::shared_ptr<Tensor> conv_infer(const Node &n, const Name &name)
{
    const int stride = n.m_attributes.get("stride", 1);
    const int pad = n.m_attributes.get("pad", 0);
    const int dilation = n.m_attributes.get("dilation", 1);
    const int group = n.m_attributes.get("group", 1);
    const bool transpose = n.m_attributes.get("transpose", false);
    auto w = n.m_inputs["w"];
    auto x = n.m_inputs["x"];
    Dims out{x->m_dims[0], (int64_t)((int)w->m_dims[transpose ? 1 : 0] * group)};
    for(size_t i = 2; i < w->m_dims.size(); i++) {
        const int in = x->m_dims[i];
        const int span = ((int)w->m_dims[i] - 1) * dilation + 1;
        int o;
        if(transpose)
            o = stride * (in - 1) + n.m_attributes.get("outputpad", 0) + span - 2 * pad;
        else
            o = 1 + (in + 2 * pad - span) / stride;
        out.push_back((int64_t)o);
    }
    return makeTensor(x->m_data_type, out, name);
}

void conv_prepare(std::shared_ptr<Node> n, std::shared_ptr<Tensor> x, Tensors &named, Nodes &)
{
    if(x->m_dims.size() < 4)
        throw std::runtime_error(fmt("x-tensor rank < 4 (%s)", x->m_dims.to_string().c_str()));
    const int spatial = x->m_dims.size() - 2;
    const bool transpose = n->m_attributes.get("transpose", false);
    const int group = n->m_attributes.get("group", 1);
    auto w = n->m_inputs.has("w") ? n->m_inputs["w"] : nullptr;
    if(!w) {
        const int activations = n->m_attributes.get("activations", 1);
        const int size = n->m_attributes.get("size", 1);
        // filter dims [out, in/group, k, k]; transposed convs swap the roles of the first two
        const int in_features = (transpose ? activations : (int)x->m_dims[1]) / group;
        const int out_features = transpose ? (int)x->m_dims[1] : activations;
        Dims wd{(int64_t)out_features, (int64_t)in_features};
        double taps = 1;
        for(int i = 0; i < spatial; i++) {
            wd.push_back((int64_t)size);
            taps *= size;
        }
        // He-normal: stddev = sqrt(2 / fan_in)
        w = Tensor::find(x->m_data_type, wd, 0, sqrt(2.0 / (in_features * taps)), named, param_name(n->m_name, "w"));
        n->m_inputs["w"] = w;
    }
    if(!n->m_inputs.has("b") && n->m_attributes.get("bias", false)) {
        const int features = (int)w->m_dims[transpose ? 1 : 0] * group;
        n->m_inputs["b"] = Tensor::find(x->m_data_type, Dims{(int64_t)1, (int64_t)features}, 0, 0, named,
                                        param_name(n->m_name, transpose ? "b" : "bt"));
    }
}

// ---- batchnorm: fp32 {1,C} scale 1, bias 0, mean 0, var 1 (reference: src/node.cpp:132-162)
void batchnorm_prepare(std::shared_ptr<Node> n, std::shared_ptr<Tensor> x, Tensors &named, Nodes &)
{
    const Dims d{(int64_t)1, x->m_dims[1]};
    static const struct {
        const char *slot;
        double init;
    } params[] = {{"s", 1.0}, {"b", 0.0}, {"m", 0.0}, {"v", 1.0}};
    for(const auto &p : params) {
        if(!n->m_inputs.has(p.slot) || !n->m_inputs[p.slot])
            n->m_inputs[p.slot] =
                Tensor::find(Tensor::DataType::FLOAT, d, p.init, 0, named, param_name(n->m_name, p.slot));
    }
}

// ---- pooling: O = 1 + (I + 2*pad - size) / stride; "global" uses the input height
// (reference: src/node.cpp:166-193)
std::shared_ptr<Tensor> pooling_infer(const Node &n, const Name &name)
{
    auto x = n.m_inputs["x"];
    const int pad = n.m_attributes.get("pad", 0);
    const int stride = n.m_attributes.get("stride", 1);
    int size = n.m_attributes.get("size", 1);
    if(n.m_attributes.get("global", false)) {
        size = x->m_dims[2];
        assert((int)x->m_dims[3] == size);
    }
    const int oh = 1 + ((int)x->m_dims[2] + 2 * pad - size) / stride;
    const int ow = 1 + ((int)x->m_dims[3] + 2 * pad - size) / stride;
    return makeTensor(x->m_data_type, Dims{x->m_dims[0], x->m_dims[1], (int64_t)oh, (int64_t)ow}, name);
}

// ---- reshape: "shape" may hold UNCHANGED / REDUCE (reference: src/node.cpp:197-223)
std::shared_ptr<Tensor> reshape_infer(const Node &n, const Name &name)
{
    auto x = n.m_inputs["x"];
    auto it = n.m_attributes.find("shape");
    if(it == n.m_attributes.end())
        throw std::runtime_error{"Shape attribute missing"};
    const Dims *shape = std::get_if<Dims>(&it->second);
    if(!shape)
        throw std::runtime_error{"Shape attribute not a dimension value"};
    const Dims &in = x->m_dims;
    const Dims out = shape->transform([&](const DimParam &dp, size_t i) -> Dim {
        if(dp == DimParam::UNCHANGED)
            return in[i];
        if(dp == DimParam::REDUCE)
            return (int64_t)in.elements(i);
        return dp;
    });
    return makeTensor(x->m_data_type, out, name);
}

// ---- concat of x0, x1, ... along "axis" (default 1) (reference: src/node.cpp:227-248)
std::shared_ptr<Tensor> concat_infer(const Node &n, const Name &name)
{
    const int axis = n.m_attributes.get("axis", 1);
    const auto xs = n.m_inputs.getv("x");
    if(xs.empty())
        throw std::runtime_error("concat without inputs");
    Dims d = xs[0]->m_dims;
    for(size_t i = 1; i < xs.size(); i++)
        d[axis] += xs[i]->m_dims[axis];
    return makeTensor(xs[0]->m_data_type, d, name);
}

// ---- window (reference: src/node.cpp:252-262)
std::shared_ptr<Tensor> window_infer(const Node &n, const Name &name)
{
    auto x = n.m_inputs["x"];
    const auto shape = n.m_attributes.get("shape", std::vector<int>{});
    if(shape.size() != x->m_dims.size())
        throw std::runtime_error(
            fmt("shape rank %zd mismatches input %s", shape.size(), x->m_dims.to_string().c_str()));
    return makeTensor(x->m_data_type, Dims(shape), name);
}

// ---- fc: y is [batch, outputs] in the weights' type; w is [in,out] or (transW) [out,in];
// inputs of rank > 2 get a flattening reshape in front (reference: src/node.cpp:266-321)
std::shared_ptr<Tensor> fc_infer(const Node &n, const Name &name)
{
    auto w = n.m_inputs["w"];
    auto x = n.m_inputs["x"];
    const bool transW = n.m_attributes.get("transW", false);
    return makeTensor(w->m_data_type, Dims{x->m_dims[0], w->m_dims[transW ? 0 : 1]}, name);
}

void fc_prepare(std::shared_ptr<Node> n, std::shared_ptr<Tensor> x, Tensors &named, Nodes &before)
{
    if(x->m_dims.size() > 2) {
        auto r = std::make_shared<Node>("reshape");
        r->m_inputs["x"] = x;
        r->m_attributes["shape"] = Dims{DimParam::UNCHANGED, DimParam::REDUCE};
        x = r->inferTensor_y();
        r->m_outputs["y"] = x;
        n->m_inputs["x"] = x;
        before.push_back(r);
    }
    const bool transW = n->m_attributes.get("transW", false);
    auto w = n->m_inputs.has("w") ? n->m_inputs["w"] : nullptr;
    if(!w) {
        const int outputs = n->m_attributes.get("outputs", 1);
        const Dims d = transW ? Dims{(int64_t)outputs, x->m_dims[1]} : Dims{x->m_dims[1], (int64_t)outputs};
        w = Tensor::find(x->m_data_type, d, 0, sqrt(2.0 / (int)x->m_dims[1]), named, param_name(n->m_name, "w"));
        n->m_inputs["w"] = w;
    }
    if(!n->m_inputs.has("b") && n->m_attributes.get("bias", false)) {
        n->m_inputs["b"] = Tensor::find(x->m_data_type, Dims{w->m_dims[transW ? 0 : 1]}, 0, 0, named,
                                        param_name(n->m_name, transW ? "bt" : "b"));
    }
}

// ---- catclassifier: y = int32 labels [N,1]; extra output "loss" (reference: src/node.cpp:325-339).
// The reference declares loss as {1,1} although one value per sample is written; here it is [N].
std::shared_ptr<Tensor> catclassifier_infer(const Node &n, const Name &name)
{
    auto x = n.m_inputs["x"];
    return makeTensor(Tensor::DataType::I32, Dims{x->m_dims[0], (int64_t)1}, name);
}

void catclassifier_prepare(std::shared_ptr<Node> n, std::shared_ptr<Tensor> x, Tensors &, Nodes &)
{
    n->m_outputs["loss"] = makeTensor(Tensor::DataType::FLOAT, Dims{x->m_dims[0]}, "loss");
}

// ---- loss (L2): y like target, extra output mmss [N,4] (reference: src/node.cpp:343-359)
std::shared_ptr<Tensor> loss_infer(const Node &n, const Name &name)
{
    auto target = n.m_inputs["target"];
    return makeTensor(target->m_data_type, target->m_dims, name);
}

void loss_prepare(std::shared_ptr<Node> n, std::shared_ptr<Tensor> x, Tensors &, Nodes &)
{
    n->m_outputs["mmss"] = makeTensor(Tensor::DataType::FLOAT, Dims{x->m_dims[0], (int64_t)4});
}

// ---- sum: operands must agree in type and shape (reference: src/node.cpp:372-389)
std::shared_ptr<Tensor> sum_infer(const Node &n, const Name &name)
{
    const auto xs = n.m_inputs.getv("x");
    if(xs.empty())
        throw std::runtime_error("sum without inputs");
    auto a = xs[0];
    for(size_t i = 1; i < xs.size(); i++) {
        auto b = xs[i];
        if(a->m_data_type != b->m_data_type)
            throw std::runtime_error(fmt("x0 datatype %s != x%zu datatype %s", Tensor::DataTypeStr(a->m_data_type), i,
                                         Tensor::DataTypeStr(b->m_data_type)));
        if(a->m_dims != b->m_dims)
            throw std::runtime_error(fmt("x0 dimensions %s != x%zu dimensions %s", a->m_dims.to_string().c_str(), i,
                                         b->m_dims.to_string().c_str()));
    }
    return makeTensor(a->m_data_type, a->m_dims, name);
}

// ---- convert: "datatype" attribute is the numeric Tensor::DataType (reference: src/node.cpp:393-402)
std::shared_ptr<Tensor> convert_infer(const Node &n, const Name &name)
{
    auto x = n.m_inputs["x"];
    const int dt = n.m_attributes.get("datatype", -1);
    if(dt == -1)
        throw std::runtime_error("No target datatype given");
    return makeTensor((Tensor::DataType)dt, x->m_dims, name);
}

std::shared_ptr<Tensor> jpegdecoder_infer(const Node &n, const Name &name)
{
    const int width = n.m_attributes.get("width", 0);
    const int height = n.m_attributes.get("height", 0);
    if(width < 1)
        throw std::runtime_error("Missing or invalid width");
    if(height < 1)
        throw std::runtime_error("Missing or invalid height");
    const int channels = n.m_attributes.get("channels", 3);
    return makeTensor(Tensor::DataType::U8, Dims{(int64_t)1, (int64_t)channels, (int64_t)width, (int64_t)height},
                      name);
}

std::shared_ptr<Tensor> spatialtransform_infer(const Node &n, const Name &)
{
    auto x = n.m_inputs["x"];
    const int height = n.m_attributes.get("height", (int)x->m_dims[2]);
    const int width = n.m_attributes.get("width", (int)x->m_dims[3]);
    return makeTensor(x->m_data_type, Dims{x->m_dims[0], x->m_dims[1], (int64_t)height, (int64_t)width});
}

std::shared_ptr<Tensor> stats_infer(const Node &, const Name &)
{
    return makeTensor(Tensor::DataType::FLOAT, Dims{(int64_t)4}, "stats");
}

// node-type table (reference: src/node.cpp:446-482)
const std::map<std::string, NodeType> &node_types()
{
    static const std::map<std::string, NodeType> table = {
        {"add", {same_as_x, nullptr}},
        {"avgpool", {pooling_infer, nullptr}},
        {"batchnorm", {same_as_x, batchnorm_prepare}},
        {"catclassifier", {catclassifier_infer, catclassifier_prepare}},
        {"concat", {concat_infer, nullptr}},
        {"conv", {conv_infer, conv_prepare}},
        {"convert", {convert_infer, nullptr}},
        {"dropout", {same_as_x, nullptr}},
        {"elu", {same_as_x, nullptr}},
        {"fc", {fc_infer, fc_prepare}},
        {"jpegdecoder", {jpegdecoder_infer, nullptr}},
        {"leakyrelu", {same_as_x, nullptr}},
        {"loss", {loss_infer, loss_prepare}},
        {"maxpool", {pooling_infer, nullptr}},
        {"mul", {same_as_x, nullptr}},
        {"relu", {same_as_x, nullptr}},
        {"reshape", {reshape_infer, nullptr}},
        {"sigmoid", {same_as_x, nullptr}},
        {"softmax", {same_as_x, nullptr}},
        {"spatialtransform", {spatialtransform_infer, nullptr}},
        {"stats", {stats_infer, nullptr}},
        {"sum", {sum_infer, nullptr}},
        {"swish", {same_as_x, nullptr}},
        {"tanh", {same_as_x, nullptr}},
        {"window", {window_infer, nullptr}},
    };
    return table;
}

}  // namespace

std::shared_ptr<Tensor> Node::inferTensor_y(const std::optional<const std::string> &name)
{
    auto it = node_types().find(m_type);
    if(it == node_types().end())
        throw std::runtime_error("Unknown node type: " + m_type);
    return it->second.infer(*this, name);
}

std::string Attribute::to_string() const
{
    if(auto v = std::get_if<int>(this))
        return std::to_string(*v);
    if(auto v = std::get_if<float>(this))
        return std::to_string(*v);
    if(auto v = std::get_if<bool>(this))
        return *v ? "true" : "false";
    if(auto v = std::get_if<Dims>(this))
        return v->to_string();
    if(auto v = std::get_if<std::vector<int>>(this)) {
        std::string r = "[";
        for(size_t i = 0; i < v->size(); i++)
            r += (i ? ", " : "") + std::to_string((*v)[i]);
        return r + "]";
    }
    return "?";
}

void Node::print() const
{
    printf("%s:\n", m_type.c_str());
    for(const auto &t : m_inputs)
        printf("\t Input: %s: %s\n", t.first.c_str(), t.second ? t.second->info().c_str() : "(null)");
    for(const auto &t : m_outputs)
        printf("\tOutput: %s: %s\n", t.first.c_str(), t.second ? t.second->info().c_str() : "(null)");
    for(const auto &a : m_attributes)
        printf("\tAttrib: %s: %s\n", a.first.c_str(), a.second.to_string().c_str());
}

// reference: src/node.cpp:541-567
std::vector<std::shared_ptr<Node>> Node::make(const std::string &type, const Tensors &inputs,
                                              const Attributes &attributes, Tensors &named_tensors,
                                              const std::optional<const std::string> &name)
{
    auto it = node_types().find(type);
    if(it == node_types().end())
        throw std::runtime_error("Unknown node type: " + type);
    auto n = std::make_shared<Node>(type, name);
    n->m_inputs = inputs;
    n->m_attributes = attributes;
    Nodes before;
    if(it->second.prepare) {
        auto x = n->m_inputs.find("x");
        if(x == n->m_inputs.end())
            throw std::runtime_error("x-tensor missing");
        it->second.prepare(n, x->second, named_tensors, before);
    }
    n->m_outputs["y"] = n->inferTensor_y();
    std::vector<std::shared_ptr<Node>> r(before.begin(), before.end());
    r.push_back(n);
    return r;
}

std::vector<std::shared_ptr<Node>> Node::make(const std::string &type, Loader loader, const Attributes &attributes)
{
    auto n = std::make_shared<Node>(type);
    n->m_loader = loader;
    n->m_attributes = attributes;
    n->m_outputs["y"] = n->inferTensor_y();
    return {n};
}

std::shared_ptr<Tensor> Node::y() const { return m_outputs["y"]; }

Nodes::iterator Nodes::findSingleDownStreamNode(std::shared_ptr<Tensor> t, const std::string &type)
{
    iterator found = end();
    for(auto it = begin(); it != end(); ++it) {
        if((*it)->m_type != type)
            continue;
        for(const auto &in : (*it)->m_inputs) {
            if(in.second != t)
                continue;
            if(found != end())
                return end(); // more than one consumer
            found = it;
        }
    }
    return found;
}

}  // namespace saga

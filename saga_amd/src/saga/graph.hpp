// -*-c++-*-
// Nodes and graphs.  (reference: saga.hpp:269-403)
#pragma once

#include "tensor.hpp"

namespace saga {

typedef std::function<size_t(long batch, int n, uint8_t *data, size_t capacity)> Loader;

class Node {
public:
    Node(const std::string &type, const std::optional<const std::string> &name = std::nullopt)
      : m_type(type), m_name(name)
    {
    }

    Node(const Node &n)
      : m_type(n.m_type), m_name(n.m_name), m_inputs(n.m_inputs), m_attributes(n.m_attributes), m_outputs(n.m_outputs)
    {
    }

    const std::string m_type;
    const std::optional<const std::string> m_name;

    Tensors m_inputs;
    Attributes m_attributes;
    Tensors m_outputs;
    Loader m_loader;

    std::shared_ptr<Tensor> inferTensor_y(const std::optional<const std::string> &name = std::nullopt);
    void print() const;

    static std::vector<std::shared_ptr<Node>> make(const std::string &type, const Tensors &inputs,
                                                   const Attributes &attributes, Tensors &named_tensors,
                                                   const std::optional<const std::string> &name = std::nullopt);

    static std::vector<std::shared_ptr<Node>> make(const std::string &type, Loader loader,
                                                   const Attributes &attributes);

    std::shared_ptr<Tensor> y() const;
};

class Nodes : public std::vector<std::shared_ptr<Node>> {
public:
    using std::vector<std::shared_ptr<Node>>::vector;

    // the only node of `type` consuming t, or end()
    iterator findSingleDownStreamNode(std::shared_ptr<Tensor> t, const std::string &type);
};

typedef std::unordered_map<std::shared_ptr<Tensor>, std::vector<std::pair<std::string, std::shared_ptr<Node>>>>
    TensorMapping;

class Graph {
public:
    Graph() : m_named_tensors(std::make_shared<Tensors>()) {}

    Graph(std::shared_ptr<Tensors> named_tensors) : m_named_tensors(named_tensors) {}

    Nodes m_nodes;
    std::unordered_set<std::shared_ptr<Tensor>> m_inputs;
    std::unordered_set<std::shared_ptr<Tensor>> m_outputs;
    const std::shared_ptr<Tensors> m_named_tensors;

    std::shared_ptr<Node> addNode(const std::string &type, const std::shared_ptr<Tensor> &t,
                                  const Attributes &attributes = {},
                                  const std::optional<const std::string> &name = std::nullopt);

    std::shared_ptr<Node> addNode(const std::string &type, const std::shared_ptr<Node> &n,
                                  const Attributes &attributes = {},
                                  const std::optional<const std::string> &name = std::nullopt);

    std::shared_ptr<Node> addNode(const std::string &type, const Tensors &inputs, const Attributes &attributes = {},
                                  const std::optional<const std::string> &name = std::nullopt);

    std::shared_ptr<Node> addNode(const std::string &type, Loader loader, const Attributes &attributes);

    static std::shared_ptr<Graph> load(const char *path);

    void loadTensors(const char *path);

    bool saveTensors(const char *path, Context *p);

    void print() const;

    void statsTensors(Context *p);

    std::pair<TensorMapping, TensorMapping> tensorMappings() const;

    std::unordered_set<std::shared_ptr<Tensor>> inputTensors() const;

    std::unordered_set<std::shared_ptr<Tensor>> outputTensors() const;

    // builders
    std::shared_ptr<Node> addJpegDecoder(int width, int height, Tensor::DataType output_data_type, Loader loader);

    std::shared_ptr<Node> addConvert(std::shared_ptr<Tensor> input, Tensor::DataType dt, float scale);

    std::shared_ptr<Node> addSpatialTransform(std::shared_ptr<Tensor> input, std::shared_ptr<Tensor> theta,
                                              int output_width = -1, int output_height = -1,
                                              bool also_during_inference = false);

    std::shared_ptr<Node> addResNetBottleNeck(std::shared_ptr<Tensor> input, int squeeze_activations,
                                              int output_activations, bool downsample, const std::string &name);

    std::shared_ptr<Node> addResNetBottleNeck_transposed(std::shared_ptr<Tensor> input, int squeeze_activations,
                                                         int output_activations, bool upsample,
                                                         const std::string &name);

    std::shared_ptr<Node> addResNet(std::shared_ptr<Tensor> input, int output_activations, bool downsample,
                                    const std::string &name);
};

}  // namespace saga

// ONNX model and tensor files -> Graph / Tensor.
//
// Role of the reference's src/onnx.cpp (op mapping :298-671, graph assembly :669-748,
// Graph::load :750-775, Tensor::loadProtoBuf :777-790).  The reference parses with libprotobuf
// and generated classes; neither is available to this build, and the subset of the ONNX schema
// a loader needs is small, so the protobuf wire format is read directly: a message is a
// sequence of (field number, wire type) keys followed by a varint, a fixed 32/64-bit value or a
// length-delimited payload; nested messages and packed repeated scalars are length-delimited.
// Field numbers are those of onnx/onnx.proto3.
//
// Differences from the reference: malformed files, unknown operators and unsupported
// attribute combinations make Graph::load print the reason and return nullptr (the reference
// asserts or aborts); fp16 / u8 tensors stored in int32_data are accepted as well; FLOAT16
// BatchNormalization parameters are widened to fp32 (the batchnorm node takes fp32 parameters).
#include <fcntl.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <map>
#include <stdexcept>
#include <string>
#include <vector>

#include "saga.hpp"

namespace saga {

namespace {

// ---------------------------------------------------------------- wire format

struct Span {
    const uint8_t *p = nullptr;
    size_t n = 0;
    std::string str() const { return std::string((const char *)p, n); }
};

struct Field {
    uint32_t num = 0;
    int wire = 0;     // 0 varint, 1 fixed64, 2 length-delimited, 5 fixed32
    uint64_t v = 0;   // varint / fixed value
    Span s;           // payload of a length-delimited field
};

class Reader {
public:
    explicit Reader(Span s) : m_p(s.p), m_end(s.p + s.n) {}

    bool next(Field &f)
    {
        if(m_p >= m_end)
            return false;
        const uint64_t key = varint();
        f.num = (uint32_t)(key >> 3);
        f.wire = (int)(key & 7);
        f.v = 0;
        f.s = Span{};
        switch(f.wire) {
        case 0:
            f.v = varint();
            break;
        case 1:
            f.v = fixed(8);
            break;
        case 5:
            f.v = fixed(4);
            break;
        case 2: {
            const uint64_t len = varint();
            if(len > (uint64_t)(m_end - m_p))
                throw std::runtime_error("protobuf: length-delimited field runs past the end of its message");
            f.s = Span{m_p, (size_t)len};
            m_p += len;
            break;
        }
        default:
            throw std::runtime_error("protobuf: unsupported wire type " + std::to_string(f.wire));
        }
        return true;
    }

    uint64_t varint()
    {
        uint64_t v = 0;
        for(int shift = 0; shift < 64; shift += 7) {
            if(m_p >= m_end)
                throw std::runtime_error("protobuf: truncated varint");
            const uint8_t b = *m_p++;
            v |= (uint64_t)(b & 0x7f) << shift;
            if(!(b & 0x80))
                return v;
        }
        throw std::runtime_error("protobuf: varint longer than ten bytes");
    }

    bool done() const { return m_p >= m_end; }

private:
    uint64_t fixed(int bytes)
    {
        if(m_end - m_p < bytes)
            throw std::runtime_error("protobuf: truncated fixed-width field");
        uint64_t v = 0;
        memcpy(&v, m_p, bytes); // little endian on the wire and on the host
        m_p += bytes;
        return v;
    }

    const uint8_t *m_p, *m_end;
};

// repeated int64 / int32 / enum: one varint per field, or packed into one payload
void repeated_varint(const Field &f, std::vector<int64_t> &out)
{
    if(f.wire == 0) {
        out.push_back((int64_t)f.v);
    } else if(f.wire == 2) {
        Reader r(f.s);
        while(!r.done())
            out.push_back((int64_t)r.varint());
    } else {
        throw std::runtime_error("protobuf: repeated integer field with wire type " + std::to_string(f.wire));
    }
}

// repeated float: one fixed32 per field, or packed
void repeated_float(const Field &f, std::vector<float> &out)
{
    if(f.wire == 5) {
        float v;
        const uint32_t u = (uint32_t)f.v;
        memcpy(&v, &u, 4);
        out.push_back(v);
    } else if(f.wire == 2) {
        if(f.s.n % 4)
            throw std::runtime_error("protobuf: packed float payload is not a multiple of four bytes");
        const size_t base = out.size();
        out.resize(base + f.s.n / 4);
        memcpy(out.data() + base, f.s.p, f.s.n);
    } else {
        throw std::runtime_error("protobuf: repeated float field with wire type " + std::to_string(f.wire));
    }
}

// ---------------------------------------------------------------- the ONNX messages a loader reads

enum {
    ONNX_FLOAT = 1,
    ONNX_UINT8 = 2,
    ONNX_INT64 = 7,
    ONNX_FLOAT16 = 10,
};

enum { ATTR_FLOAT = 1, ATTR_INT = 2, ATTR_INTS = 7 };

struct TensorMsg { // TensorProto
    std::vector<int64_t> dims;
    int data_type = 0;
    std::string name;
    Span raw;
    std::vector<float> float_data;
    std::vector<int64_t> int32_data, int64_data;
    bool external = false;

    explicit TensorMsg(Span s)
    {
        Reader r(s);
        Field f;
        while(r.next(f)) {
            switch(f.num) {
            case 1: repeated_varint(f, dims); break;
            case 2: data_type = (int)f.v; break;
            case 4: repeated_float(f, float_data); break;
            case 5: repeated_varint(f, int32_data); break;
            case 7: repeated_varint(f, int64_data); break;
            case 8: name = f.s.str(); break;
            case 9: raw = f.s; break;
            case 13: external = true; break;
            case 14: external = external || f.v == 1; break;
            default: break; // segment, strings, doubles, doc_string: not used by the models in scope
            }
        }
    }
};

struct ValueInfoMsg { // ValueInfoProto -> TypeProto -> TypeProto.Tensor -> TensorShapeProto
    std::string name;
    bool has_tensor_type = false;
    bool dims_ok = true;
    int elem_type = 0;
    std::vector<int64_t> dims;

    explicit ValueInfoMsg(Span s)
    {
        Reader r(s);
        Field f;
        while(r.next(f)) {
            if(f.num == 1)
                name = f.s.str();
            else if(f.num == 2 && f.wire == 2)
                type(f.s);
        }
    }

private:
    void type(Span s)
    {
        Reader r(s);
        Field f;
        while(r.next(f)) {
            if(f.num != 1 || f.wire != 2)
                continue;
            has_tensor_type = true;
            Reader rt(f.s);
            Field ft;
            while(rt.next(ft)) {
                if(ft.num == 1)
                    elem_type = (int)ft.v;
                else if(ft.num == 2 && ft.wire == 2)
                    shape(ft.s);
            }
        }
    }

    void shape(Span s)
    {
        Reader r(s);
        Field f;
        while(r.next(f)) {
            if(f.num != 1 || f.wire != 2)
                continue;
            // a dimension holds either a value or a symbolic name (the batch size of model-zoo
            // files); a symbolic dimension counts as 1, a dimension with neither is unusable
            Reader rd(f.s);
            Field fd;
            bool have = false;
            int64_t d = 0;
            while(rd.next(fd)) {
                if(fd.num == 1 && fd.wire == 0) {
                    d = (int64_t)fd.v;
                    have = true;
                } else if(fd.num == 2 && fd.wire == 2) {
                    d = 1;
                    have = true;
                }
            }
            if(!have)
                dims_ok = false;
            dims.push_back(d);
        }
    }
};

struct NodeMsg { // NodeProto with its attributes folded into an Attributes map
    std::string op_type, name;
    std::vector<std::string> inputs, outputs;
    Attributes attribs;

    explicit NodeMsg(Span s)
    {
        Reader r(s);
        Field f;
        while(r.next(f)) {
            switch(f.num) {
            case 1: inputs.push_back(f.s.str()); break;
            case 2: outputs.push_back(f.s.str()); break;
            case 3: name = f.s.str(); break;
            case 4: op_type = f.s.str(); break;
            case 5: attribute(f.s); break;
            default: break;
            }
        }
    }

private:
    // INT, FLOAT and INTS attributes are kept; the others (strings, tensors, graphs) are not
    // used by any operator in scope (reference: src/onnx.cpp:689-706)
    void attribute(Span s)
    {
        std::string aname;
        int type = 0;
        float fv = 0;
        int64_t iv = 0;
        bool have_f = false, have_i = false;
        std::vector<int64_t> ints;
        Reader r(s);
        Field f;
        while(r.next(f)) {
            switch(f.num) {
            case 1: aname = f.s.str(); break;
            case 2: {
                const uint32_t u = (uint32_t)f.v;
                memcpy(&fv, &u, 4);
                have_f = true;
                break;
            }
            case 3: iv = (int64_t)f.v; have_i = true; break;
            case 8: repeated_varint(f, ints); break;
            case 20: type = (int)f.v; break;
            default: break;
            }
        }
        if(type == 0) // files older than IR version 2 carry no type field
            type = !ints.empty() ? ATTR_INTS : have_i ? ATTR_INT : have_f ? ATTR_FLOAT : 0;
        if(type == ATTR_INT)
            attribs[aname] = (int)iv;
        else if(type == ATTR_FLOAT)
            attribs[aname] = fv;
        else if(type == ATTR_INTS)
            attribs[aname] = std::vector<int>(ints.begin(), ints.end());
        else
            m_other.push_back(aname);
    }

public:
    std::vector<std::string> m_other; // names of attributes of other kinds (e.g. auto_pad)

    bool has_other(const char *n) const
    {
        for(const auto &o : m_other)
            if(o == n)
                return true;
        return false;
    }
};

// ---------------------------------------------------------------- file mapping

class MappedFile {
public:
    explicit MappedFile(const char *path)
    {
        const int fd = open(path, O_RDONLY);
        if(fd == -1)
            throw std::runtime_error(fmt("Failed to open protobuf file %s: %s", path, strerror(errno)));
        struct stat st;
        if(fstat(fd, &st) == -1) {
            const int e = errno;
            close(fd);
            throw std::runtime_error(fmt("Failed to stat protobuf file %s: %s", path, strerror(e)));
        }
        m_size = st.st_size;
        if(m_size) {
            m_mem = mmap(NULL, m_size, PROT_READ, MAP_PRIVATE, fd, 0);
            if(m_mem == MAP_FAILED) {
                const int e = errno;
                close(fd);
                throw std::runtime_error(fmt("Failed to map protobuf file %s: %s", path, strerror(e)));
            }
        }
        close(fd);
    }
    ~MappedFile()
    {
        if(m_mem && m_mem != MAP_FAILED)
            munmap(m_mem, m_size);
    }
    MappedFile(const MappedFile &) = delete;
    MappedFile &operator=(const MappedFile &) = delete;

    Span span() const { return Span{(const uint8_t *)m_mem, m_size}; }

private:
    void *m_mem = nullptr;
    size_t m_size = 0;
};

// ---------------------------------------------------------------- tensors

const char *onnx_type_name(int dt)
{
    static const char *names[] = {"UNDEFINED", "FLOAT", "UINT8", "INT8", "UINT16", "INT16", "INT32", "INT64", "STRING",
                                  "BOOL", "FLOAT16", "DOUBLE", "UINT32", "UINT64", "COMPLEX64", "COMPLEX128", "BFLOAT16"};
    return dt >= 0 && dt < (int)(sizeof(names) / sizeof(names[0])) ? names[dt] : "???";
}

// reference: DataType_map, src/onnx.cpp:277-294
Tensor::DataType map_type(int dt)
{
    switch(dt) {
    case ONNX_FLOAT: return Tensor::DataType::FLOAT;
    case ONNX_UINT8: return Tensor::DataType::U8;
    case ONNX_INT64: return Tensor::DataType::INT64;
    case ONNX_FLOAT16: return Tensor::DataType::HALF;
    default: throw std::runtime_error(fmt("ONNX: No mapping for data-type %s", onnx_type_name(dt)));
    }
}

Dims dims_of(const std::vector<int64_t> &v)
{
    Dims d;
    for(const int64_t e : v)
        d.push_back(e);
    return d;
}

// graph input / output declaration -> placeholder (reference: src/onnx.cpp:296-322)
std::shared_ptr<Tensor> placeholder_of(const ValueInfoMsg &vi)
{
    if(!vi.has_tensor_type || !vi.dims_ok)
        return nullptr;
    return makeTensor(map_type(vi.elem_type), dims_of(vi.dims), vi.name);
}

// initializer / tensor file -> host tensor with data (reference: src/onnx.cpp:324-354)
std::shared_ptr<Tensor> host_tensor_of(const TensorMsg &tm)
{
    if(tm.external)
        throw std::runtime_error(fmt("Unable to load %s: data stored outside the file", tm.name.c_str()));
    const auto dt = map_type(tm.data_type);
    auto t = makeCPUTensor(dt, dims_of(tm.dims), tm.name);
    auto ta = t->access();
    const size_t elements = t->m_dims.elements();
    const size_t esize = Tensor::DataTypeSize(dt);
    uint8_t *dst = (uint8_t *)ta->data();
    auto need = [&](size_t have, const char *what) {
        if(have != elements)
            throw std::runtime_error(
                fmt("Unable to load %s: %s holds %zu values for %zu elements", tm.name.c_str(), what, have, elements));
    };
    if(tm.raw.n) {
        if(tm.raw.n != elements * esize)
            throw std::runtime_error(fmt("Unable to load %s: raw_data holds %zu bytes for %zu elements of %zu bytes",
                                         tm.name.c_str(), tm.raw.n, elements, esize));
        memcpy(dst, tm.raw.p, tm.raw.n);
    } else if(!tm.float_data.empty() && dt == Tensor::DataType::FLOAT) {
        need(tm.float_data.size(), "float_data");
        memcpy(dst, tm.float_data.data(), elements * sizeof(float));
    } else if(!tm.int64_data.empty() && dt == Tensor::DataType::INT64) {
        need(tm.int64_data.size(), "int64_data");
        memcpy(dst, tm.int64_data.data(), elements * sizeof(int64_t));
    } else if(!tm.int32_data.empty() && dt == Tensor::DataType::HALF) {
        need(tm.int32_data.size(), "int32_data");
        for(size_t i = 0; i < elements; i++)
            ((uint16_t *)dst)[i] = (uint16_t)tm.int32_data[i]; // fp16 bit patterns
    } else if(!tm.int32_data.empty() && dt == Tensor::DataType::U8) {
        need(tm.int32_data.size(), "int32_data");
        for(size_t i = 0; i < elements; i++)
            dst[i] = (uint8_t)tm.int32_data[i];
    } else if(elements) {
        throw std::runtime_error(fmt("Unable to load %s: Can't load data format", tm.name.c_str()));
    }
    return t;
}

// ---------------------------------------------------------------- operators -> nodes

struct Builder {
    Graph &g;
    const NodeMsg &np;

    std::shared_ptr<Tensor> in(size_t i) const
    {
        if(i >= np.inputs.size())
            throw std::runtime_error(fmt("ONNX %s: input %zu missing", np.op_type.c_str(), i));
        auto it = g.m_named_tensors->find(np.inputs[i]);
        if(it == g.m_named_tensors->end() || !it->second)
            throw std::runtime_error(
                fmt("ONNX %s: input tensor %s is not defined", np.op_type.c_str(), np.inputs[i].c_str()));
        return it->second;
    }

    void arity(size_t lo, size_t hi) const
    {
        if(np.inputs.size() < lo || np.inputs.size() > hi)
            throw std::runtime_error(fmt("ONNX %s: %zu inputs", np.op_type.c_str(), np.inputs.size()));
    }

    void reject(bool cond, const char *what) const
    {
        if(cond)
            throw std::runtime_error(fmt("ONNX %s: %s is not supported", np.op_type.c_str(), what));
    }

    // all entries of an integer-list attribute must agree (square windows, symmetric padding)
    int uniform(const char *name, int dflt) const
    {
        const auto v = np.attribs.get(name, std::vector<int>{});
        if(v.empty())
            return dflt;
        for(int e : v)
            if(e != v[0])
                throw std::runtime_error(fmt("ONNX %s: %s must hold equal values", np.op_type.c_str(), name));
        return v[0];
    }

    std::shared_ptr<Node> finish(std::shared_ptr<Node> n) const
    {
        auto y = n->inferTensor_y(np.outputs[0]);
        (*g.m_named_tensors)[np.outputs[0]] = y;
        n->m_outputs["y"] = y;
        return n;
    }

    std::shared_ptr<Node> numbered_inputs(const char *type) const
    {
        arity(1, 1 << 20);
        auto n = std::make_shared<Node>(type);
        for(size_t i = 0; i < np.inputs.size(); i++)
            n->m_inputs["x" + std::to_string(i)] = in(i);
        return n;
    }

    std::shared_ptr<Node> unary(const char *type) const
    {
        arity(1, 1);
        auto n = std::make_shared<Node>(type);
        n->m_inputs["x"] = in(0);
        return n;
    }

    // reference: make_conv, src/onnx.cpp:373-422
    std::shared_ptr<Node> conv() const
    {
        arity(2, 3);
        auto n = std::make_shared<Node>("conv");
        n->m_inputs["x"] = in(0);
        n->m_inputs["w"] = in(1);
        if(np.inputs.size() > 2)
            n->m_inputs["b"] = in(2);
        reject(np.has_other("auto_pad"), "auto_pad");
        reject(np.attribs.get("group", 1) != 1, "group != 1");
        reject(uniform("dilations", 1) != 1, "dilation != 1");
        n->m_attributes["pad"] = uniform("pads", 0);
        n->m_attributes["stride"] = uniform("strides", 1);
        return finish(n);
    }

    // The batchnorm node takes fp32 scale / bias / mean / variance whatever the type of x (as
    // cuDNN does for the reference's backend); fp16 models store them as FLOAT16, so those
    // initializers are widened once, here, on the host.
    static std::shared_ptr<Tensor> widened(std::shared_ptr<Tensor> t)
    {
        if(t->m_data_type != Tensor::DataType::HALF)
            return t;
        auto src = t->access();
        if(!src)
            return t;
        auto w = makeCPUTensor(Tensor::DataType::FLOAT, t->m_dims, t->m_name);
        auto dst = w->access();
        const int n = (int)t->m_dims.elements();
        if(t->m_dims.size() != 1)
            throw std::runtime_error("ONNX BatchNormalization: parameters must be vectors");
        for(int i = 0; i < n; i++)
            dst->set({i}, src->get({i}));
        return w;
    }

    // reference: make_batchnorm, src/onnx.cpp:424-443
    std::shared_ptr<Node> batchnorm() const
    {
        arity(5, 5);
        auto n = std::make_shared<Node>("batchnorm");
        static const char *slots[] = {"x", "s", "b", "m", "v"};
        for(int i = 0; i < 5; i++)
            n->m_inputs[slots[i]] = i ? widened(in(i)) : in(i);
        n->m_attributes["epsilon"] = np.attribs.get("epsilon", 1e-05f);
        return finish(n);
    }

    // reference: make_pooling, src/onnx.cpp:470-523
    std::shared_ptr<Node> pooling(const char *type, bool global) const
    {
        auto n = unary(type);
        reject(np.has_other("auto_pad"), "auto_pad");
        reject(np.attribs.get("ceil_mode", 0) != 0, "ceil_mode");
        reject(uniform("dilations", 1) != 1, "dilation != 1");
        reject(np.attribs.get("storage_order", 0) != 0, "storage_order");
        if(global)
            n->m_attributes["global"] = true;
        else
            n->m_attributes["size"] = uniform("kernel_shape", 0);
        n->m_attributes["pad"] = uniform("pads", 0);
        n->m_attributes["stride"] = uniform("strides", 1);
        return finish(n);
    }

    // reference: make_mathop, src/onnx.cpp:525-537
    std::shared_ptr<Node> mathop(const char *type) const
    {
        arity(2, 2);
        auto n = std::make_shared<Node>(type);
        n->m_inputs["x"] = in(0);
        n->m_inputs["b"] = in(1);
        return finish(n);
    }

    // the target shape is an int64 initializer: 0 keeps a dimension, -1 takes what is left
    // (reference: make_reshape, src/onnx.cpp:573-598)
    std::shared_ptr<Node> reshape() const
    {
        arity(2, 2);
        auto n = std::make_shared<Node>("reshape");
        n->m_inputs["x"] = in(0);
        auto shape = in(1);
        auto ta = shape->access();
        if(!ta || shape->m_dims.size() != 1)
            throw std::runtime_error("ONNX Reshape: the shape must be a one-dimensional initializer");
        Dims a;
        for(int i = 0; i < (int)shape->m_dims[0]; i++) {
            const int64_t v = (int64_t)ta->get({i});
            if(v == 0)
                a.push_back(DimParam::UNCHANGED);
            else if(v == -1)
                a.push_back(DimParam::REDUCE);
            else if(v > 0)
                a.push_back(v);
        }
        n->m_attributes["shape"] = a;
        return finish(n);
    }

    // dimensions before `axis` stay, the rest collapse (reference: make_flatten, src/onnx.cpp:600-621)
    std::shared_ptr<Node> flatten() const
    {
        auto n = unary("reshape");
        const int rank = (int)n->m_inputs["x"]->m_dims.size();
        int axis = np.attribs.get("axis", 1);
        if(axis < 0)
            axis += rank;
        reject(axis < 0 || axis >= rank, "axis outside the tensor");
        Dims shape(axis + 1, DimParam::UNCHANGED);
        shape[axis] = DimParam::REDUCE;
        n->m_attributes["shape"] = shape;
        return finish(n);
    }

    // transB names the weights' orientation (reference: make_gemm, src/onnx.cpp:623-637)
    std::shared_ptr<Node> gemm() const
    {
        arity(3, 3);
        auto n = std::make_shared<Node>("fc");
        n->m_inputs["x"] = in(0);
        n->m_inputs["w"] = in(1);
        n->m_inputs["b"] = in(2);
        n->m_attributes["transW"] = np.attribs.get("transB", 0) ? true : false;
        return finish(n);
    }

    // reference: make_matmul, src/onnx.cpp:639-650
    std::shared_ptr<Node> matmul() const
    {
        arity(2, 2);
        auto n = std::make_shared<Node>("fc");
        n->m_inputs["x"] = in(0);
        n->m_inputs["w"] = in(1);
        return finish(n);
    }

    // the operator table (reference: src/onnx.cpp:708-743)
    std::shared_ptr<Node> build() const
    {
        if(np.outputs.size() != 1)
            throw std::runtime_error(fmt("ONNX %s: %zu outputs", np.op_type.c_str(), np.outputs.size()));
        const std::string &t = np.op_type;
        if(t == "Conv")
            return conv();
        if(t == "BatchNormalization")
            return batchnorm();
        if(t == "Relu")
            return finish(unary("relu"));
        if(t == "LeakyRelu") {
            auto n = unary("leakyrelu");
            n->m_attributes["alpha"] = np.attribs.get("alpha", 0.01f);
            return finish(n);
        }
        if(t == "MaxPool")
            return pooling("maxpool", false);
        if(t == "AveragePool")
            return pooling("avgpool", false);
        if(t == "GlobalAveragePool")
            return pooling("avgpool", true);
        if(t == "Add")
            return mathop("add");
        if(t == "Mul")
            return mathop("mul");
        if(t == "MatMul")
            return matmul();
        if(t == "Sum")
            return finish(numbered_inputs("sum"));
        if(t == "Concat")
            return finish(numbered_inputs("concat"));
        if(t == "Reshape")
            return reshape();
        if(t == "Flatten")
            return flatten();
        if(t == "Gemm")
            return gemm();
        if(t == "Softmax")
            return finish(unary("softmax"));
        if(t == "Dropout")
            return finish(unary("dropout"));
        std::string desc = "Can't handle node type " + t + " (inputs:";
        for(const auto &i : np.inputs)
            desc += " " + i;
        desc += "; outputs:";
        for(const auto &o : np.outputs)
            desc += " " + o;
        throw std::runtime_error(desc + ")");
    }
};

// GraphProto -> Graph (reference: loadgraph, src/onnx.cpp:669-748).  Declared inputs that
// also have an initializer are parameters, not graph inputs.
void load_graph(Graph &g, Span s)
{
    std::vector<Span> nodes, initializers, inputs, outputs;
    Reader r(s);
    Field f;
    while(r.next(f)) {
        if(f.wire != 2)
            continue;
        switch(f.num) {
        case 1: nodes.push_back(f.s); break;
        case 5: initializers.push_back(f.s); break;
        case 11: inputs.push_back(f.s); break;
        case 12: outputs.push_back(f.s); break;
        default: break;
        }
    }
    for(const auto &i : inputs) {
        const ValueInfoMsg vi(i);
        auto t = placeholder_of(vi);
        (*g.m_named_tensors)[vi.name] = t;
        if(t)
            g.m_inputs.insert(t);
    }
    for(const auto &i : initializers) {
        const TensorMsg tm(i);
        auto it = g.m_named_tensors->find(tm.name);
        if(it != g.m_named_tensors->end())
            g.m_inputs.erase(it->second);
        (*g.m_named_tensors)[tm.name] = host_tensor_of(tm);
    }
    for(const auto &nspan : nodes) {
        const NodeMsg np(nspan);
        g.m_nodes.push_back(Builder{g, np}.build());
    }
    for(const auto &o : outputs) {
        const ValueInfoMsg vi(o);
        auto it = g.m_named_tensors->find(vi.name);
        if(it == g.m_named_tensors->end() || !it->second)
            throw std::runtime_error("ONNX: graph output " + vi.name + " is not produced by any node");
        g.m_outputs.insert(it->second);
    }
}

}  // namespace

// reference: src/onnx.cpp:750-775
std::shared_ptr<Graph> Graph::load(const char *path)
{
    try {
        MappedFile file(path);
        Reader r(file.span());
        Field f;
        Span graph;
        bool have = false;
        while(r.next(f)) {
            if(f.num == 7 && f.wire == 2) { // ModelProto.graph
                graph = f.s;
                have = true;
            }
        }
        if(!have)
            throw std::runtime_error("no graph in the model file");
        auto g = std::make_shared<Graph>();
        load_graph(*g, graph);
        return g;
    } catch(const std::exception &e) {
        fprintf(stderr, "Unable to load %s: %s\n", path, e.what());
        return nullptr;
    }
}

// a file holding one TensorProto (the model zoo's input_0.pb / output_0.pb)
// (reference: src/onnx.cpp:777-790)
std::shared_ptr<Tensor> Tensor::loadProtoBuf(const char *path)
{
    try {
        MappedFile file(path);
        return host_tensor_of(TensorMsg(file.span()));
    } catch(const std::exception &e) {
        fprintf(stderr, "Unable to load %s: %s\n", path, e.what());
        return nullptr;
    }
}

}  // namespace saga

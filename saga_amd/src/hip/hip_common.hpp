// -*-c++-*-
// The "hip" engine: Saga's Engine / Context / Program / Tensor boundary implemented for one
// MI355X.  Takes the place of the reference's src/cuda/cuda_common.hpp, cuda_tensor.hpp and
// cuda_program.cpp; arithmetic is delegated to the C-ABI kernel library (saga_hip.h).
//
// Only the public saga.hpp and engine.hpp are used from the front end, so these sources
// also compile against the reference's own headers.
#pragma once

#include <hip/hip_runtime_api.h>

#include <map>
#include <memory>
#include <set>
#include <string>
#include <vector>

#include "saga.hpp"
#include "saga_hip.h"

namespace saga {

// HIP runtime failures are fatal, like the reference's chkCuda (src/cuda/cuda_common.hpp:32-41).
#define chkHip(expr)                                                                                      \
    do {                                                                                                  \
        hipError_t e__ = (expr);                                                                          \
        if(e__ != hipSuccess) {                                                                           \
            fprintf(stderr, "%s at %s:%d in %s: %s\n", #expr, __FILE__, __LINE__, __FUNCTION__,           \
                    hipGetErrorString(e__));                                                              \
            abort();                                                                                      \
        }                                                                                                 \
    } while(0)

// Kernel-library argument errors surface as exceptions (set-up / shape problems), like chkCUDNN.
#define chkSaga(expr)                                                                                     \
    do {                                                                                                  \
        int r__ = (expr);                                                                                 \
        if(r__ != 0)                                                                                      \
            throw std::runtime_error(fmt("%s at %s:%d: %s", #expr, __FILE__, __LINE__,                    \
                                         saga_hip_error_string(r__)));                                    \
    } while(0)

class HipContext;
class HipProgram;
class HipTensor;
struct HipOperation;

// A device allocation (possibly shared by several storages, e.g. the optimizer arena).
struct HipMemory {
    explicit HipMemory(size_t bytes);
    ~HipMemory();
    void *m_ptr = nullptr;
    size_t m_bytes = 0;
};

// Growable scratch area: ops request a size at set-up, finalize() allocates the maximum.
struct HipScratch {
    void request(size_t bytes) { m_requested = std::max(m_requested, bytes); }
    void alloc();
    void *ptr() const { return m_mem ? m_mem->m_ptr : nullptr; }
    size_t size() const { return m_mem ? m_mem->m_bytes : 0; }
    size_t m_requested = 0;
    std::shared_ptr<HipMemory> m_mem;
};

// The bytes behind one or more tensors (aliases share a storage).
class HipStorage {
public:
    HipStorage(Tensor::DataType dt, size_t elements, HipContext *ctx);
    virtual ~HipStorage() {}

    // Device memory is attached on first use: either an allocation of its own, or - for
    // storages whose contents live only within one step - a slot of the context's arena,
    // assigned by HipContext::planMemory() when a program is finalized.
    virtual void *deviceMem() const
    {
        if(!m_data)
            const_cast<HipStorage *>(this)->allocOwn();
        return m_data;
    }
    bool allocated() const { return m_data != nullptr; }
    // host staging: whole-storage copies around TensorAccess lifetimes
    virtual bool doubleBuffered() const { return false; }

    void rehome(const std::shared_ptr<HipMemory> &mem, void *ptr);
    void allocOwn();
    size_t bytes() const { return m_elements * m_element_size; }

    HipContext *const m_ctx;
    const Tensor::DataType m_data_type;
    const size_t m_elements;
    const size_t m_element_size;
    const int m_id;
    std::shared_ptr<HipMemory> m_memory;
    void *m_data = nullptr;
    bool m_in_arena = false; // m_data points into the context's arena (contents do not survive a step)
    bool m_nonfinite_is_valid = false;
};

// Batched tensors: two device buffers and two pinned host buffers.  Operations use
// device[m_index]; host callbacks see host[m_index ^ 1]
// (reference: CudaTensorStorageDoubleBuffered, src/cuda/cuda_tensor.cpp:789-954).
class HipDoubleBuffer : public HipStorage {
public:
    HipDoubleBuffer(Tensor::DataType dt, size_t elements, HipContext *ctx);
    ~HipDoubleBuffer();
    void *deviceMem() const override { return m_dev[m_index]; }
    bool doubleBuffered() const override { return true; }
    void *hostBack() const { return m_host[m_index ^ 1]; }
    void uploadBack(hipStream_t st);    // host[back] -> device[back]
    void downloadFront(hipStream_t st); // device[front] -> host[front]
    void flip() { m_index ^= 1; }
    void *m_dev[2] = {nullptr, nullptr};
    void *m_host[2] = {nullptr, nullptr};
    int m_index = 0;
};

enum class HipLayout { NCHW, NHWC };

// Device tensor.  Logical dims as in the front end (any rank up to 4); the strides, in
// elements, carry the physical layout and alias offsets
// (reference: CudaTensor, src/cuda/cuda_tensor.hpp:90-164).
class HipTensor : public Tensor {
public:
    // fresh storage in the given layout
    HipTensor(DataType dt, const Dims &dims, HipLayout layout, HipContext *ctx,
              const std::optional<const std::string> &name = std::nullopt);
    // view of existing storage
    HipTensor(std::shared_ptr<HipStorage> storage, const Dims &dims, const std::vector<int64_t> &strides,
              int64_t offset, const std::optional<const std::string> &name = std::nullopt);
    // fresh storage, same dims and strides as `like`, other data type
    HipTensor(DataType dt, const HipTensor &like, const std::optional<const std::string> &name = std::nullopt);

    std::string info() const override;
    std::unique_ptr<TensorAccess> access() override;
    std::shared_ptr<Tensor> slice(const Dims &offset, const Dims &size) override;
    Stats stats() override;

    void *deviceMem() const;
    // the 4-D view handed to the kernel library (rank < 4 is padded; rank 1 becomes [1,C,1,1])
    SagaTensorView view() const;
    // the same with a placeholder address when no memory is attached yet: for size queries at
    // set-up time, which must not trigger an allocation
    SagaTensorView shapeView() const;
    // [rows, cols] matrices for the fc path
    bool cpacked() const; // channel stride 1 (NHWC-like) for rank-4 tensors
    bool rowMajor() const;
    std::string shortname() const;

    // host -> device copy of a front-end tensor (any type / layout); values are converted
    void copyFromHost(Tensor &src);

    std::shared_ptr<HipStorage> m_storage;
    std::vector<int64_t> m_strides;
    int64_t m_offset = 0;
    bool m_auto_initialized = false;
};

std::vector<int64_t> hip_strides(const Dims &dims, HipLayout layout);

using HipOp = std::shared_ptr<HipOperation>;
using HipOps = std::vector<HipOp>;
using HipOpArgs = std::vector<std::pair<const char *, std::shared_ptr<HipTensor>>>;

// One launch (or a few) on the context's stream (reference: CudaOperation, cuda_common.hpp:323-368).
struct HipOperation {
    explicit HipOperation(const std::string &kind) : m_kind(kind) {}
    virtual ~HipOperation() {}
    virtual void exec(HipProgram &p) = 0;
    virtual HipOpArgs listInputs() const = 0;
    virtual HipOpArgs listOutputs() const = 0;
    // accumulation factor of output t (0 overwrite, 1 add) or nullptr if t cannot accumulate
    virtual float *getBeta(const std::shared_ptr<HipTensor> &t) { return nullptr; }
    // drop an output nobody reads; false if the op cannot do without it
    virtual bool killOutput(const std::shared_ptr<HipStorage> &s) { return false; }
    virtual std::string info() const { return ""; }
    // algorithmic work of one execution: floating point operations (matrix ops) and bytes that
    // must cross HBM (memory-bound ops); used for roofline accounting only
    virtual double flops() const { return 0; }
    virtual double bytes() const { return 0; }
    // false for an operation whose launches take host values that change from step to step
    // (loss scale, Adam's bias corrections): it is never recorded into a HIP graph
    virtual bool graphSafe() const { return true; }

    // inputs plus the outputs that are accumulated into
    HipOpArgs getInputs();
    HipOpArgs getOutputs() const { return listOutputs(); }
    std::string str();
    void dump(FILE *out, bool full);
    const std::string &name() const { return m_kind; }

    std::string m_kind;
};

struct HipProgram;
// hip_ops.cpp: hands the first pass of a batch norm's backward to the convolution that writes its gradient
void link_bn_backward(HipProgram &p, std::vector<std::shared_ptr<HipOperation>> &ops);
// hip_ops.cpp: a strided 1x1 backward data that writes a fan-in gradient first is moved behind the last writer
void reorder_sparse_first_writers(std::vector<std::shared_ptr<HipOperation>> &ops);
void fuse_bn_pooling(HipProgram &p, std::vector<std::shared_ptr<HipOperation>> &ops);

struct HipProgramUnit {
    Nodes m_transformed;
    int m_batch_size = 1;
    HipOps m_fwd, m_bwd, m_tail;
    void fwd(const HipOp &op) { m_fwd.push_back(op); }
    // backward ops run in reverse creation order
    void bwd(const HipOp &op) { m_bwd.insert(m_bwd.begin(), op); }
    void tail(const HipOp &op) { m_tail.push_back(op); }
};

class HipEngine;

class HipContext : public Context, public std::enable_shared_from_this<HipContext> {
public:
    HipContext(const std::shared_ptr<UI> &ui, int device);
    ~HipContext();

    std::shared_ptr<Program> createMultiProgram(const std::vector<ProgramSource> &sources, ProgramType pt,
                                                const ProgramConfig &pc) override;
    std::shared_ptr<Tensor> resolveTensor(std::shared_ptr<Tensor> t) override;
    int getId() const override { return m_device; }
    UI::Page getUiPage() const override { return (UI::Page)(UI::CTX + m_device); }
    void reset() override;
    void bindToHostThread() override { chkHip(hipSetDevice(m_device)); }

    void sync()
    {
        chkHip(hipStreamSynchronize(m_stream));
        chkHip(hipStreamSynchronize(m_copy_stream));
    }

    const std::shared_ptr<UI> m_ui;
    const int m_device;
    hipStream_t m_stream = nullptr;
    // uploads of the batched tensors' BACK buffers: they run beside the step that computes on the front buffers
    hipStream_t m_copy_stream = nullptr;
    int m_num_cu = 0;
    int m_storage_id_gen = 0;
    int m_program_index_gen = 0;

    HipScratch m_workspace;
    // bumped whenever a storage gets a new device address; recorded HIP graphs of older epochs are dropped
    uint64_t m_mem_epoch = 0;

    // front-end tensor -> device tensor, shared by all programs of this context so that
    // inference and training programs see the same weights
    std::unordered_map<std::shared_ptr<Tensor>, std::shared_ptr<HipTensor>> m_tensors;
    // device tensors whose initial values still have to be fetched from the front end
    std::unordered_map<std::shared_ptr<HipTensor>, std::shared_ptr<Tensor>> m_deferred_copy;
    // storages handed out to the host: kept by the dead-code elimination
    std::vector<std::shared_ptr<HipStorage>> m_exported;

    // ---- storage reuse (role of the reference's src/cuda/cuda_analysis.cpp:194-547)
    // Finalized programs of this context; planMemory() lays the storages that live only within a
    // step of every program that touches them into one arena, overlapping those whose live
    // ranges never intersect.
    std::vector<class HipProgram *> m_programs;
    std::shared_ptr<HipMemory> m_arena;
    size_t m_arena_bytes = 0;    // size of the arena
    size_t m_planned_bytes = 0;  // sum of the sizes of the storages laid out in it
    void planMemory();
};

class HipProgram : public Program {
public:
    HipProgram(std::shared_ptr<HipContext> ctx, ProgramType pt, const ProgramConfig &pc);
    ~HipProgram();

    void finalize() override;
    ExecResult run(long batches, StopCheck stop_check, long batch_offset) override;
    void dump(FILE *output, bool detailed) override;
    void debug(bool on) override { m_debug = on; }
    bool dumpGraph(const char *path) override;
    ProgramType getType() const override { return m_pt; }
    int getUiRow() const override { return m_index + 1; }
    double getMPS() const override { return m_mp_scaling; }

    // ---- lowering helpers used by the node set-up functions
    HipLayout layoutFor(Tensor::DataType dt) const;
    std::shared_ptr<HipTensor> lower(const HipProgramUnit &pu, std::shared_ptr<Tensor> src, size_t minimum_rank = 0);
    // like lower(), but in the layout (channels-last or not) of `blueprint`
    std::shared_ptr<HipTensor> lowerLike(const HipProgramUnit &pu, std::shared_ptr<Tensor> src,
                                         const HipTensor &blueprint);
    std::shared_ptr<HipTensor> lowerGrad(const HipProgramUnit &pu, std::shared_ptr<Tensor> src,
                                         size_t minimum_rank = 0);
    // registers a trainable parameter with its gradient
    void upd(const std::shared_ptr<Tensor> &key, const std::shared_ptr<HipTensor> &w,
             const std::shared_ptr<HipTensor> &g);

    void prep(long batches, long batch_offset);
    void step(long batch, long batches, long batch_offset);
    void post(long batches, long batch_offset);
    void runOps(const HipOps &ops);
    void addBatchedTensors(const ProgramSource &ps);
    void runCallbacks(const TensorBatchCallback &cb, long batch, Phase phase);
    void flip(Phase upload_phase);
    void eliminateDeadOps();
    void checkAnomaly(HipOperation &op, const HipOpArgs &tensors, const char *what);
    HipOps createOptimizers();
    // Adam's moments, step counts, fp32 master weights and the loss scale (hip_optimizer.cpp)
    void saveOptimizerState(const char *path);
    void loadOptimizerState(const char *path);
    HipOp createOptimizer(Tensor::DataType dt);

    const std::shared_ptr<HipContext> m_ctx;
    const int m_index;
    const ProgramType m_pt;
    const ProgramConfig m_pc;
    bool m_debug = false;
    bool m_finalized = false;
    std::string m_name;

    HipOps m_ops;
    // anomaly detection: arena storages to fill with NaN bytes before the operation that defines
    // them and after the last one that uses them (reference: m_pre_invalidate / m_post_invalidate,
    // src/cuda/cuda_analysis.cpp:486-517), indexed like m_ops
    std::vector<std::vector<HipStorage *>> m_poison_before, m_poison_after;
    HipOps m_opt;
    std::vector<HipProgramUnit> m_units;

    std::map<std::shared_ptr<Tensor>, std::pair<std::shared_ptr<HipTensor>, std::shared_ptr<HipTensor>>> m_updates;
    std::unordered_map<std::shared_ptr<Tensor>, std::pair<std::shared_ptr<HipDoubleBuffer>, Phase>> m_batched;
    std::unordered_map<std::shared_ptr<Tensor>, std::shared_ptr<HipTensor>> m_batched_tensors;

    // ---- optional per-operation timing with HIP events on the program's stream
    struct ProfileRow {
        std::string kind;
        long launches = 0;
        double ms = 0, flops = 0, bytes = 0;
    };
    void setProfiling(bool on);
    std::vector<ProfileRow> profile() const;
    bool m_profiling = false;
    std::vector<hipEvent_t> m_events;          // one per op boundary (ops + 1)
    std::map<std::string, ProfileRow> m_profile;
    void collectProfile();

    // ---- HIP graphs: runs of graph-safe operations of the step are recorded once per combination of
    // front buffers (batched tensors alternate between two device buffers) and replayed with one launch each
    struct GraphSegment {
        size_t begin = 0, end = 0; // [begin, end) of m_ops
        bool graph = false;        // false: run operation by operation
        std::map<unsigned, hipGraphExec_t> exec; // by front-buffer key
    };
    std::vector<GraphSegment> m_segments;
    std::vector<HipDoubleBuffer *> m_graph_dbufs; // every double-buffered storage the operations touch
    uint64_t m_graph_epoch = ~(uint64_t)0;
    void *m_graph_ws = nullptr;
    long m_steps_run = 0; // executions of m_ops so far
    bool graphsEnabled() const;
    void dropGraphs();
    void runOpsGraphed();

    // the operation that transposes the filters of all backward-data convolutions in one launch (hip_ops.cpp)
    std::shared_ptr<HipOperation> m_transpose_batch;

    SagaAux *m_aux = nullptr; // pinned host memory the optimizer kernels write their flags to
    float m_mp_scaling = 1.0f;
    bool m_mp_enabled = false;
    int64_t m_total_samples = 0;
    int64_t m_epoch_start = 0;
};

// node type -> lowering function; graph transforms (reference: REGISTER_CUDA_OP / _TRANSFORM)
using HipOpSetup = void (*)(HipProgram &p, HipProgramUnit &pu, const Node &n);
using HipTransform = Nodes (*)(HipProgram &p, HipProgramUnit &pu, const Nodes &nodes);
void hipRegisterOp(const char *name, HipOpSetup setup);
void hipRegisterTransform(int prio, ProgramType types, HipTransform fn);
HipOpSetup hipFindOp(const std::string &type);
Nodes hipApplyTransforms(HipProgram &p, HipProgramUnit &pu, const Nodes &nodes);

#define HIP_JOIN2(a, b) a##b
#define HIP_JOIN(a, b) HIP_JOIN2(a, b)
#define REGISTER_HIP_OP(name, setup) \
    static void __attribute__((constructor)) HIP_JOIN(hip_reg_op_, __LINE__)(void) { hipRegisterOp(name, setup); }
#define REGISTER_HIP_TRANSFORM(prio, types, fn)                                       \
    static void __attribute__((constructor)) HIP_JOIN(hip_reg_tr_, __LINE__)(void)    \
    {                                                                                 \
        hipRegisterTransform(prio, types, fn);                                        \
    }

}  // namespace saga

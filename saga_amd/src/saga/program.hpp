// -*-c++-*-
// Programs, contexts and engines: the boundary a compute backend implements.
// (reference: saga.hpp:408-585)
#pragma once

#include <stdio.h>

#include "graph.hpp"

namespace saga {

struct UI {
    virtual ~UI() {}

    enum class Align {
        LEFT,
        CENTER,
        RIGHT,
    };

    enum Page { SYS = 0, DATA = 100, CTX = 200, USER = 300 };

    virtual void updateCell(Page page, size_t row, size_t column, Align a, const char *fmt, ...)
        __attribute__((format(printf, 6, 7))) = 0;

    virtual void refresh() = 0;
};

std::shared_ptr<UI> make_tui();
std::shared_ptr<UI> make_nui();

enum class ProgramType {
    INFERENCE = 0x1,
    TRAINING = 0x2,
};

inline constexpr ProgramType operator|(ProgramType a, ProgramType b)
{
    return static_cast<ProgramType>(static_cast<int>(a) | static_cast<int>(b));
}

inline constexpr ProgramType operator&(ProgramType a, ProgramType b)
{
    return static_cast<ProgramType>(static_cast<int>(a) & static_cast<int>(b));
}

inline constexpr bool operator!(ProgramType a) { return static_cast<bool>(!static_cast<int>(a)); }

// when the host callbacks touch a batched tensor: before (PRE) or after (POST) its batch ran
enum class Phase { PRE = 0x1, POST = 0x2 };

inline constexpr Phase operator|(Phase a, Phase b)
{
    return static_cast<Phase>(static_cast<int>(a) | static_cast<int>(b));
}

inline constexpr Phase operator&(Phase a, Phase b)
{
    return static_cast<Phase>(static_cast<int>(a) & static_cast<int>(b));
}

inline constexpr bool operator!(Phase a) { return static_cast<bool>(!static_cast<int>(a)); }

typedef std::unordered_map<std::shared_ptr<Tensor>, Phase> BatchedTensors;

class Program;

typedef std::function<void(long batch, const Program &p, std::unordered_map<std::shared_ptr<Tensor>, TensorAccess *>)>
    TensorBatchCallback;

typedef std::function<bool(void)> StopCheck;

struct ProgramSource {
    const Graph &graph;

    BatchedTensors batched_tensors;

    int batch_size{1};
};

// This build adds initial_loss_scale to the reference's fields; code that must compile
// against either header tests SAGA_HAS_INITIAL_LOSS_SCALE.
#define SAGA_HAS_INITIAL_LOSS_SCALE 1

struct ProgramConfig {
    TensorBatchCallback pre_ops;

    TensorBatchCallback post_ops;

    float learning_rate{1e-4};

    // L2 regularization term
    float l2_lambda{0};

    float bn_expavg{0.1};

    TensorLayout tensor_layout{TensorLayout::Auto};

    // scan tensors for non-finite values around every operation (slow, debug only)
    bool anomaly_detect{false};

    bool disable_op_fusing{false};

    // 0 keeps the reference's rule (sum of the batch sizes) for mixed-precision programs
    float initial_loss_scale{0};
};

enum class ExecResult { OK, STOPPED };

class Program {
public:
    virtual ~Program() {}

    virtual void finalize() = 0;

    virtual ExecResult run(long batches = 1, StopCheck stop_check = nullptr, long batch_offset = 0) = 0;

    virtual void dump(FILE *output, bool detailed = false) = 0;

    virtual void debug(bool on) = 0;

    virtual bool dumpGraph(const char *path) { return false; }

    virtual ProgramType getType() const = 0;

    virtual int getUiRow() const = 0;

    // current mixed-precision loss scale
    virtual double getMPS() const = 0;
};

class Context {
public:
    virtual ~Context() {}

    virtual std::shared_ptr<Program> createMultiProgram(const std::vector<ProgramSource> &sources, ProgramType pt,
                                                        const ProgramConfig &pc) = 0;

    std::shared_ptr<Program> createProgram(const ProgramSource &ps, ProgramType pt, const ProgramConfig &pc)
    {
        return createMultiProgram({ps}, pt, pc);
    }

    // the backend's tensor standing for front-end tensor t (nullptr when t is not part of any program)
    virtual std::shared_ptr<Tensor> resolveTensor(std::shared_ptr<Tensor> t) = 0;

    virtual int getId() const = 0;

    virtual UI::Page getUiPage() const = 0;

    virtual void reset() = 0;

    virtual void bindToHostThread() = 0;
};

class Engine {
public:
    virtual ~Engine() {}

    virtual std::vector<std::shared_ptr<Context>> createContexts(bool multi = false) = 0;
};

std::shared_ptr<Engine> createEngine(const std::shared_ptr<UI> &ui);

std::shared_ptr<Context> createContext(const std::shared_ptr<UI> &ui = nullptr);

}  // namespace saga

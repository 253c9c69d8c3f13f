// Engine registry (reference: src/engine.cpp:16-39): backends register by name from static
// constructors; createEngine() takes the alphabetically first one.
#include <map>

#include "engine.hpp"

namespace saga {

typedef std::shared_ptr<Engine> (*EngineFactory)(const std::shared_ptr<UI> &ui);

static std::map<std::string, EngineFactory> &factories()
{
    static std::map<std::string, EngineFactory> m; // constructed on first use: safe from static constructors
    return m;
}

void registerEngineFactory(const char *name, EngineFactory fn) { factories()[name] = fn; }

std::shared_ptr<Engine> createEngine(const std::shared_ptr<UI> &ui)
{
    if(factories().empty())
        throw std::runtime_error("No compute engine registered");
    return factories().begin()->second(ui ? ui : make_nui());
}

std::shared_ptr<Context> createContext(const std::shared_ptr<UI> &ui)
{
    auto ctxs = createEngine(ui)->createContexts(false);
    if(ctxs.empty())
        throw std::runtime_error("Engine created no context");
    return ctxs[0];
}

}  // namespace saga

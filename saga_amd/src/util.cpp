// now(), fmt(), Barrier and the null / line UIs (reference: src/util.cpp, src/ui/nui.cpp).
#include <stdarg.h>
#include <time.h>

#include <condition_variable>
#include <mutex>

#include "saga.hpp"

namespace saga {

int64_t now()
{
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (int64_t)ts.tv_sec * 1000000LL + ts.tv_nsec / 1000;
}

std::string fmt(const char *f, ...)
{
    va_list ap, ap2;
    va_start(ap, f);
    va_copy(ap2, ap);
    const int n = vsnprintf(nullptr, 0, f, ap);
    va_end(ap);
    std::string s(n > 0 ? n : 0, '\0');
    if(n > 0)
        vsnprintf(&s[0], n + 1, f, ap2);
    va_end(ap2);
    return s;
}

namespace {

struct CountingBarrier : public Barrier {
    explicit CountingBarrier(size_t n) : m_parties(n) {}
    void wait() override
    {
        std::unique_lock<std::mutex> lk(m_mutex);
        const size_t gen = m_generation;
        if(++m_waiting == m_parties) {
            m_waiting = 0;
            m_generation++;
            m_cond.notify_all();
            return;
        }
        m_cond.wait(lk, [&] { return gen != m_generation; });
    }
    const size_t m_parties;
    size_t m_waiting = 0, m_generation = 0;
    std::mutex m_mutex;
    std::condition_variable m_cond;
};

struct NullUI : public UI {
    void updateCell(Page, size_t, size_t, Align, const char *, ...) override {}
    void refresh() override {}
};

}  // namespace

std::shared_ptr<Barrier> Barrier::make(size_t count) { return std::make_shared<CountingBarrier>(count); }

std::shared_ptr<UI> make_nui() { return std::make_shared<NullUI>(); }

// the cell-grid terminal UI is cosmetic; this build returns the null UI for it too
std::shared_ptr<UI> make_tui() { return std::make_shared<NullUI>(); }

std::shared_ptr<Publisher> make_tcp_publisher(int) { return nullptr; }

}  // namespace saga

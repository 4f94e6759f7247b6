// Named scopes around the work of the front-end, for profilers and tests that want to know what ran
// (dali/utils/scope.h, scope.cpp: Scope, DALI_SCOPE and ScopeObserver). A scope costs one test of a counter when nobody
// observes; with observers, entering and leaving one calls every observer in the order they were added.
#include "dali.h"

#include <algorithm>

namespace dali {

namespace {

struct Registry {
    int next_id = 1;
    std::vector<std::pair<int, Scope::callback_t>> enter, exit;
};

Registry& registry() {
    static Registry r;
    return r;
}

}  // namespace

bool Scope::has_observers() {
    const Registry& r = registry();
    return !r.enter.empty() || !r.exit.empty();
}

int Scope::add_observer(callback_t on_enter, callback_t on_exit) {
    Registry& r = registry();
    const int id = r.next_id++;
    if (on_enter) r.enter.emplace_back(id, std::move(on_enter));
    if (on_exit) r.exit.emplace_back(id, std::move(on_exit));
    return id;
}

void Scope::remove_observer(int id) {
    Registry& r = registry();
    auto drop = [id](std::vector<std::pair<int, callback_t>>& v) {
        v.erase(std::remove_if(v.begin(), v.end(), [id](const std::pair<int, callback_t>& e) { return e.first == id; }), v.end());
    };
    drop(r.enter);
    drop(r.exit);
}

Scope::Scope(name_t name_) : name(std::move(name_)) {
    // (a copy: an observer may add or remove observers)
    const auto observers = registry().enter;
    for (const auto& e : observers) e.second(name);
}

Scope::~Scope() {
    const auto observers = registry().exit;
    for (const auto& e : observers) {
        try {
            e.second(name);
        } catch (...) {
            // leaving a scope happens during unwinding too
        }
    }
}

ScopeObserver::ScopeObserver(callback_t on_enter_, callback_t on_exit_) : on_enter(std::move(on_enter_)), on_exit(std::move(on_exit_)) {
    id = Scope::add_observer(
        [this](Scope::name_t n) {
            state.trace.push_back(n);
            if (on_enter) on_enter(state);
        },
        [this](Scope::name_t n) {
            if (on_exit) on_exit(state);
            if (!state.trace.empty() && state.trace.back() == n) state.trace.pop_back();
        });
}

ScopeObserver::~ScopeObserver() { Scope::remove_observer(id); }

}  // namespace dali

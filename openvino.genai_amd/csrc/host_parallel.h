// Independent host work items spread over a few threads.
#pragma once

#include <algorithm>
#include <atomic>
#include <cstddef>
#include <exception>
#include <thread>
#include <vector>

namespace pa {

// Runs fn(0..count-1) over up to 16 host threads (the items must be independent); the first failure of any of them is
// rethrown after all have ended.
template <typename F>
void parallel_items(size_t count, size_t n_threads, F&& fn) {
    n_threads = std::min<size_t>({n_threads, count, 16, std::max(1u, std::thread::hardware_concurrency())});
    if (n_threads <= 1) {
        for (size_t i = 0; i < count; ++i) fn(i);
        return;
    }
    std::atomic<size_t> next{0};
    std::atomic<bool> failed{false};
    std::exception_ptr failure;
    std::vector<std::thread> pool;
    for (size_t t = 0; t < n_threads; ++t)
        pool.emplace_back([&] {
            try {
                for (size_t i = next.fetch_add(1); i < count && !failed; i = next.fetch_add(1)) fn(i);
            } catch (...) {
                if (!failed.exchange(true)) failure = std::current_exception();
            }
        });
    for (std::thread& t : pool) t.join();
    if (failed) std::rethrow_exception(failure);
}

}  // namespace pa

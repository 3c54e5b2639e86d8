// Host-side helper shared by the converters and the plan builder: a loop over
// [0, n) cut into one contiguous block per worker thread.
#pragma once
#include <algorithm>
#include <cstddef>
#include <exception>
#include <thread>
#include <vector>

namespace hspmm_host {

inline unsigned worker_count(size_t work_items, size_t min_per_worker)
{
    unsigned hw = std::thread::hardware_concurrency();
    if (hw == 0) hw = 1;
    if (hw > 16) hw = 16;
    size_t by_work = work_items / (min_per_worker ? min_per_worker : 1);
    if (by_work < 1) by_work = 1;
    return unsigned(std::min<size_t>(hw, by_work));
}

// fn(begin, end) on every block; an exception of a worker (out of memory) is rethrown
// on the calling thread once all workers are done.
template <class F>
void parallel_blocks(size_t n, size_t min_per_worker, F &&fn)
{
    const unsigned nw = worker_count(n, min_per_worker);
    if (nw <= 1) { fn(size_t(0), n); return; }
    std::vector<std::thread> th;
    std::vector<std::exception_ptr> err(nw);
    th.reserve(nw);
    for (unsigned i = 0; i < nw; ++i) {
        const size_t b = n * i / nw, e = n * (i + 1) / nw;
        th.emplace_back([&fn, &err, i, b, e] {
            try { fn(b, e); } catch (...) { err[i] = std::current_exception(); }
        });
    }
    for (auto &t : th) t.join();
    for (auto &e : err) if (e) std::rethrow_exception(e);
}

}  // namespace hspmm_host

// Host-side helpers shared by the converters and the plan builder: a loop over
// [0, n) cut into chunks that worker threads take one after the other.
#pragma once
#include <algorithm>
#include <atomic>
#include <cstddef>
#include <cstdlib>
#include <new>
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

// fn(begin, end) on chunks of `chunk` items that the workers take off a shared counter until none is left
// (work spread unevenly over [0, n) - the windows of a power-law graph: the first tenth of them holds half of
// the entries - still keeps every worker busy to the end).  An exception of a worker (out of memory) is
// rethrown on the calling thread once all workers are done.
template <class F>
void parallel_chunks(size_t n, size_t chunk, F &&fn, unsigned workers = 0)
{
    if (chunk < 1) chunk = 1;
    const unsigned nw = workers ? workers : worker_count(n, chunk);
    if (nw <= 1) { if (n) fn(size_t(0), n); return; }
    std::atomic<size_t> next{0};
    std::vector<std::thread> th;
    std::vector<std::exception_ptr> err(nw);
    th.reserve(nw);
    for (unsigned i = 0; i < nw; ++i)
        th.emplace_back([&fn, &err, &next, i, n, chunk] {
            try {
                for (size_t b = next.fetch_add(chunk); b < n; b = next.fetch_add(chunk)) fn(b, std::min(n, b + chunk));
            } catch (...) {
                err[i] = std::current_exception();
                next.store(n);                        // the others stop at their next chunk
            }
        });
    for (auto &t : th) t.join();
    for (auto &e : err) if (e) std::rethrow_exception(e);
}

// A loop over [0, n) for as many workers as have min_per_worker items each: eight chunks per worker, none
// shorter than min_per_worker.
template <class F>
void parallel_blocks(size_t n, size_t min_per_worker, F &&fn)
{
    const unsigned nw = worker_count(n, min_per_worker);
    if (nw <= 1) { fn(size_t(0), n); return; }
    const size_t pieces = size_t(nw) * 8u;
    parallel_chunks(n, std::max<size_t>(min_per_worker, (n + pieces - 1) / pieces), fn, nw);
}

// n elements that read as zero, without the single-threaded pass a std::vector spends on clearing them
// (a fifth of a second for the arrays of a large plan): the memory comes from calloc, whose fresh pages are
// zero already, and is first touched by whichever worker fills it.  Trivial element types only.
template <class T>
class ZeroedBuffer {
    T *p_ = nullptr;
    size_t n_ = 0;
public:
    ZeroedBuffer() = default;
    explicit ZeroedBuffer(size_t n) : p_(static_cast<T *>(std::calloc(n ? n : 1, sizeof(T)))), n_(n)
    {
        if (!p_) throw std::bad_alloc();
    }
    ZeroedBuffer(const ZeroedBuffer &) = delete;
    ZeroedBuffer &operator=(const ZeroedBuffer &) = delete;
    ZeroedBuffer(ZeroedBuffer &&o) noexcept : p_(o.p_), n_(o.n_) { o.p_ = nullptr; o.n_ = 0; }
    ZeroedBuffer &operator=(ZeroedBuffer &&o) noexcept
    {
        if (this != &o) { std::free(p_); p_ = o.p_; n_ = o.n_; o.p_ = nullptr; o.n_ = 0; }
        return *this;
    }
    ~ZeroedBuffer() { std::free(p_); }
    T *data() { return p_; }
    const T *data() const { return p_; }
    size_t size() const { return n_; }
    T &operator[](size_t i) { return p_[i]; }
    const T &operator[](size_t i) const { return p_[i]; }
    void swap(ZeroedBuffer &o) noexcept { std::swap(p_, o.p_); std::swap(n_, o.n_); }
};

}  // namespace hspmm_host

// Host-side helper shared by the converters and the plan builder: a loop over
// [0, n) cut into one contiguous block per worker thread.
#pragma once
#include <algorithm>
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

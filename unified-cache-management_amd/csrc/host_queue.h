// Host-side building blocks shared by the store runtimes: a countdown latch with a timed wait
// and a bounded multi-producer queue that worker threads drain until told to stop.
#pragma once

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <deque>
#include <mutex>

namespace {

using Clock = std::chrono::steady_clock;

// Counts the parts of a task that are still running (thread/latch.h of the reference).
struct Waiter {
    std::mutex m;
    std::condition_variable cv;
    int pending = 0;
    Clock::time_point start = Clock::now();
    void up()
    {
        std::lock_guard<std::mutex> lock(m);
        ++pending;
    }
    void done()
    {
        std::lock_guard<std::mutex> lock(m);
        if (pending > 0 && --pending == 0) cv.notify_all();
    }
    bool check()
    {
        std::lock_guard<std::mutex> lock(m);
        return pending == 0;
    }
    bool wait_for(size_t ms)
    {
        std::unique_lock<std::mutex> lock(m);
        return cv.wait_for(lock, std::chrono::milliseconds(ms), [this] { return pending == 0; });
    }
};

template <typename T>
class BoundedQueue {
public:
    void setup(size_t depth) { depth_ = depth; }
    bool try_push(T&& v)
    {
        {
            std::lock_guard<std::mutex> lock(m_);
            if (q_.size() >= depth_) return false;
            q_.push_back(std::move(v));
        }
        cv_.notify_one();
        return true;
    }
    void push(T&& v)
    {
        {
            std::lock_guard<std::mutex> lock(m_);
            q_.push_back(std::move(v));
        }
        cv_.notify_one();
    }
    // false once `stop` is set and the queue is empty
    bool pop(T& out, const std::atomic<bool>& stop)
    {
        std::unique_lock<std::mutex> lock(m_);
        for (;;) {
            if (!q_.empty()) {
                out = std::move(q_.front());
                q_.pop_front();
                return true;
            }
            if (stop.load()) return false;
            cv_.wait_for(lock, std::chrono::milliseconds(20));
        }
    }

private:
    std::mutex m_;
    std::condition_variable cv_;
    std::deque<T> q_;
    size_t depth_ = 1024;
};

}  // namespace

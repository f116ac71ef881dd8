// Persistent worker threads fed from one queue (mutex + condition variable), for the CPU-assisted LoRA path.
//
// Stands where the reference keeps a generic task-queue pool (csrc/tpool.hpp:18-100: workers block on a
// condition variable, enqueue() hands back a future) and runs its CPU LoRA workers as long-lived pinned
// processes (runServerCPULoRA.py:74-90).  Work arrives here as batches: n tasks that share one function,
// claimed one index at a time by whichever worker is free, so that submitting a batch of request chunks
// costs one queue entry and one wake-up, and waiting for it is one condition variable, not n futures.
#pragma once
#include <condition_variable>
#include <deque>
#include <functional>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

namespace mlora_cpu {

class TaskPool {
public:
    // A submitted batch; wait() blocks until its last task has returned.
    class Batch {
    public:
        void wait()
        {
            std::unique_lock<std::mutex> lk(mu_);
            cv_.wait(lk, [this] { return left_ == 0; });
        }
        bool done()
        {
            std::lock_guard<std::mutex> lk(mu_);
            return left_ == 0;
        }

    private:
        friend class TaskPool;
        Batch(int n, std::function<void(int)> fn) : fn_(std::move(fn)), n_(n), next_(0), left_(n) {}
        std::function<void(int)> fn_;
        const int n_;
        int next_;                      // next unclaimed index; guarded by the pool's queue mutex
        std::mutex mu_;
        std::condition_variable cv_;
        int left_;                      // tasks not yet finished; guarded by mu_
    };

    explicit TaskPool(int n_threads) : stop_(false)
    {
        if (n_threads < 1) n_threads = 1;
        workers_.reserve((size_t)n_threads);
        for (int i = 0; i < n_threads; i++) workers_.emplace_back([this] { serve(); });
    }
    TaskPool(const TaskPool &) = delete;
    TaskPool &operator=(const TaskPool &) = delete;

    // Finishes what is queued, then joins the workers.
    ~TaskPool()
    {
        {
            std::lock_guard<std::mutex> lk(mu_);
            stop_ = true;
        }
        wake_.notify_all();
        for (std::thread &t : workers_) t.join();
    }

    int threads() const { return (int)workers_.size(); }

    // Queue fn(0) .. fn(n - 1); returns at once.  fn must not throw.
    std::shared_ptr<Batch> submit(int n, std::function<void(int)> fn)
    {
        std::shared_ptr<Batch> b(new Batch(n > 0 ? n : 0, std::move(fn)));
        if (n <= 0) return b;
        {
            std::lock_guard<std::mutex> lk(mu_);
            queue_.push_back(b);
        }
        if (n == 1) wake_.notify_one();
        else wake_.notify_all();
        return b;
    }

    void run(int n, std::function<void(int)> fn) { submit(n, std::move(fn))->wait(); }

private:
    void serve()
    {
        for (;;) {
            std::shared_ptr<Batch> b;
            int idx;
            {
                std::unique_lock<std::mutex> lk(mu_);
                wake_.wait(lk, [this] { return stop_ || !queue_.empty(); });
                if (queue_.empty()) return;             // stop requested and nothing left to do
                b = queue_.front();
                idx = b->next_++;
                if (b->next_ >= b->n_) queue_.pop_front();
            }
            b->fn_(idx);
            bool last;
            {
                std::lock_guard<std::mutex> lk(b->mu_);
                last = --b->left_ == 0;
            }
            if (last) b->cv_.notify_all();
        }
    }

    std::mutex mu_;
    std::condition_variable wake_;
    std::deque<std::shared_ptr<Batch>> queue_;
    bool stop_;
    std::vector<std::thread> workers_;
};

}  // namespace mlora_cpu

// Stand-in for DAPHNE's src/runtime/local/vectorized/TaskQueues.h:27-100: a bounded queue of tasks between the
// thread that cuts a pipeline's rows into tasks and the workers that run them. A closed queue that has run empty
// hands out its end marker.
#pragma once

#include <runtime/local/vectorized/Tasks.h>

#include <condition_variable>
#include <deque>
#include <mutex>

class TaskQueue {
  public:
    virtual ~TaskQueue() = default;
    virtual void enqueueTask(Task *t) = 0;
    virtual Task *dequeueTask() = 0;
    virtual uint64_t size() = 0;
    virtual void closeInput() = 0;
};

class BlockingTaskQueue : public TaskQueue {
    std::deque<Task *> _tasks;
    std::mutex _m;
    std::condition_variable _changed;
    EOFTask _eof;
    uint64_t _capacity;
    bool _closed = false;

  public:
    explicit BlockingTaskQueue(uint64_t capacity = 100000) : _capacity(capacity ? capacity : 1) {}

    void enqueueTask(Task *t) override {
        std::unique_lock<std::mutex> lk(_m);
        _changed.wait(lk, [&] { return _tasks.size() < _capacity; });
        _tasks.push_back(t);
        lk.unlock();
        _changed.notify_all();
    }
    Task *dequeueTask() override {
        std::unique_lock<std::mutex> lk(_m);
        _changed.wait(lk, [&] { return !_tasks.empty() || _closed; });
        if (_tasks.empty())
            return &_eof;
        Task *t = _tasks.front();
        _tasks.pop_front();
        lk.unlock();
        _changed.notify_all();
        return t;
    }
    uint64_t size() override {
        std::lock_guard<std::mutex> g(_m);
        return _tasks.size();
    }
    void closeInput() override {
        {
            std::lock_guard<std::mutex> g(_m);
            _closed = true;
        }
        _changed.notify_all();
    }
};

// Stand-in for DAPHNE's src/runtime/local/vectorized/Worker.h:25-64: a thread that a derived class starts at the
// end of its constructor and that is joined when the worker goes away.
#pragma once

#include <runtime/local/vectorized/Tasks.h>

#include <memory>
#include <thread>

class Worker {
  protected:
    std::unique_ptr<std::thread> t;
    DCTX(ctx);
    explicit Worker(DCTX(dctx)) : ctx(dctx) {}

  public:
    Worker(const Worker &) = delete;
    Worker &operator=(const Worker &) = delete;
    virtual ~Worker() {
        if (t && t->joinable())
            t->join();
    }
    void join() { t->join(); }
    virtual void run() = 0;
    static bool isEOF(Task *task) { return dynamic_cast<EOFTask *>(task) != nullptr; }
};

// WorkerHIP: the thread that runs a pipeline's device tasks.
//
// The counterpart of WorkerGPU (src/runtime/local/vectorized/WorkerGPU.h:22-52): it takes tasks from one queue until
// the queue is closed and empty and runs each with the pipeline's device body (`fid`) in batches of `batchSize` rows.
// One such worker serves a device: its tasks share the device context's stream, so a second thread would only queue
// behind the first. Every entry point of the kernel library selects the context's device for the calling thread, so
// the worker needs no set-up of its own.
// A task that throws (a kernel's failed verdict, an allocation that does not fit) must not take the process down with
// it, as an exception leaving a thread would: the worker keeps the first exception for the thread that joins it
// (rethrowIfFailed) and drains the rest of its queue without running it, so that whoever fills the queue never blocks.
//
// In DAPHNE this file is src/runtime/local/vectorized/WorkerHIP.h.
#pragma once

#include <runtime/local/vectorized/TaskQueues.h>
#include <runtime/local/vectorized/Worker.h>

#include <exception>
#include <memory>
#include <thread>
#include <utility>

class WorkerHIP : public Worker {
    TaskQueue *_q;
    uint32_t _fid;
    uint32_t _batchSize;
    std::exception_ptr _failure;

  public:
    WorkerHIP(TaskQueue *tq, DCTX(dctx), uint32_t fid, uint32_t batchSize) : Worker(dctx), _q(tq), _fid(fid), _batchSize(batchSize) {
        t = std::make_unique<std::thread>(&WorkerHIP::run, this); // last: the thread sees a complete object
    }
    ~WorkerHIP() override = default;

    void run() override {
        for (Task *task = _q->dequeueTask(); !isEOF(task); task = _q->dequeueTask()) {
            if (!_failure) {
                try {
                    task->execute(_fid, _batchSize);
                } catch (...) {
                    _failure = std::current_exception();
                }
            }
            delete task;
        }
    }

    // after join(): throws what the first failing task threw
    void rethrowIfFailed() {
        if (_failure)
            std::rethrow_exception(std::exchange(_failure, nullptr));
    }
};

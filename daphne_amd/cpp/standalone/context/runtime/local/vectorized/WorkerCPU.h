// Stand-in for DAPHNE's src/runtime/local/vectorized/WorkerCPU.h:24-230 with the reference's constructor: a thread
// that runs the tasks of its queue with body `fid` until the queue is closed and empty, then those of the other
// queues in turn (the reference's sequential stealing; its other victim orders and the pinning of workers to cores
// are not reproduced).
#pragma once

#include <runtime/local/vectorized/LoadPartitioningDefs.h>
#include <runtime/local/vectorized/TaskQueues.h>
#include <runtime/local/vectorized/Worker.h>

#include <utility>
#include <vector>

class WorkerCPU : public Worker {
    std::vector<TaskQueue *> _q;
    uint32_t _fid, _batchSize;
    int _threadID, _numQueues;
    QueueTypeOption _queueMode;

  public:
    WorkerCPU(std::vector<TaskQueue *> deques, std::vector<int> /*physical_ids*/, std::vector<int> /*unique_threads*/, DCTX(dctx),
              bool /*verbose*/, uint32_t fid = 0, uint32_t batchSize = 100, int threadID = 0, int numQueues = 0,
              QueueTypeOption queueMode = QueueTypeOption::CENTRALIZED, VictimSelectionLogic = VictimSelectionLogic::SEQ,
              bool /*pinWorkers*/ = false)
        : Worker(dctx), _q(std::move(deques)), _fid(fid), _batchSize(batchSize), _threadID(threadID), _numQueues(numQueues),
          _queueMode(queueMode) {
        t = std::make_unique<std::thread>(&WorkerCPU::run, this);
    }

    void run() override {
        const int first = _queueMode == QueueTypeOption::CENTRALIZED ? 0 : _threadID % _numQueues;
        for (int k = 0; k < _numQueues; k++) {
            TaskQueue *q = _q[static_cast<size_t>((first + k) % _numQueues)];
            for (Task *task = q->dequeueTask(); !isEOF(task); task = q->dequeueTask()) {
                task->execute(_fid, _batchSize);
                delete task;
            }
        }
    }
};

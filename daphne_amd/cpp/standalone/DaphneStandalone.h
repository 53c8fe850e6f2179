// Minimal stand-ins for the parts of DAPHNE's run-time that the HIP kernel layer touches, so that this layer
// builds and is tested without the DAPHNE source tree (plain host compiler, no MLIR, no spdlog).
//
// The kernel layer (../src) includes DAPHNE's headers by their paths in DAPHNE's src/ directory. This directory
// holds a small header under each of those paths that forwards here; it is on the include path only for the
// builds of this repository. Inside DAPHNE it is left out and the real headers are found instead. Names, members
// and behaviour follow the reference so that the same kernel bodies compile against either:
//   IContext / DaphneContext            src/runtime/local/context/DaphneContext.h:40-114 (+ hip_contexts)
//   DaphneUserConfig                    src/api/cli/DaphneUserConfig.h (the fields the kernel layer reads)
//   KernelDispatchMapping, ErrorHandler src/util/KernelDispatchMapping.h, src/util/ErrorHandler.cpp:80-90
//   pre/postKernelInstrumentation       src/runtime/local/instrumentation/KernelInstrumentation.cpp:19-27
//   IAllocationDescriptor, ALLOCATION_TYPE, AllocationDescriptorHost
//                                       src/runtime/local/datastructures/IAllocationDescriptor.h:21-62
//   DataPlacement, MetaDataObject       src/runtime/local/datastructures/DataPlacement.h, MetaDataObject.{h,cpp}
//   DenseMatrix, DataObjectFactory      src/runtime/local/datastructures/DenseMatrix.{h,cpp}, DataObjectFactory.h:34-62
//
// The placement model is the reference's: a matrix owns a list of data placements (host, device 0, ...), and a
// list of the placements that hold its current contents. getValues(&descriptor) returns the pointer in the
// requested memory space, copying there first when that space is not current; the const overload leaves the
// other placements valid (addLatest), the non-const one invalidates them (setLatest). Ranges are not modelled
// ("Range support under construction", DenseMatrix.cpp:236): a placement always covers the whole buffer, and a
// view addresses into its parent's placements by offset (the reference clones the placement list per view).
#pragma once

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <map>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <vector>

// ------------------------------------------------------------------------------------------
// contexts
// ------------------------------------------------------------------------------------------
struct IContext {
    virtual ~IContext() = default;
    virtual void destroy() = 0;
};

struct DaphneUserConfig {
    bool use_hip = false;           // counterpart of use_cuda
    bool enable_statistics = false; // --statistics: kernels are timed by their dispatch id
    bool hip_fuse_any = false;      // counterpart of cuda_fuse_any (MarkCUDAOpsPass.cpp:55-72)
    bool force_hip = false;
    // HIP::vectorizedPipeline: into how many tasks the rows are cut, and how many rows a task runs per launch
    // (0: all of its rows at once)
    uint64_t hip_vect_shares = 1;
    uint64_t hip_vect_batch_rows = 0;
};

struct KernelDispatchInfo {
    std::string kernelName, fileName;
    int line = 0, column = 0;
};
// Maps the id the compiler gives every kernel call site to its name and source position.
class KernelDispatchMapping {
    std::mutex m;
    std::vector<KernelDispatchInfo> infos;

  public:
    int registerKernel(std::string name, std::string file = "", int line = 0, int column = 0) {
        std::lock_guard<std::mutex> g(m);
        infos.push_back({std::move(name), std::move(file), line, column});
        return static_cast<int>(infos.size()) - 1;
    }
    KernelDispatchInfo getKernelDispatchInfo(int kId) {
        std::lock_guard<std::mutex> g(m);
        return infos.at(static_cast<size_t>(kId));
    }
};

struct DaphneContext {
    std::vector<std::unique_ptr<IContext>> hip_contexts; // counterpart of cuda_contexts
    DaphneUserConfig config;
    KernelDispatchMapping dispatchMapping;
    // --statistics: accumulated time and call count per dispatch id
    std::mutex stats_lock;
    std::map<int, std::chrono::steady_clock::time_point> kernel_started;
    std::map<int, std::pair<uint64_t, double>> kernel_stats; // id -> (calls, seconds)

    DaphneContext() = default;
    DaphneContext(const DaphneContext &) = delete;
    ~DaphneContext() {
        for (auto &c : hip_contexts)
            c->destroy();
        hip_contexts.clear();
    }
    [[nodiscard]] const DaphneUserConfig &getUserConfig() const { return config; }
    [[nodiscard]] bool useHIP() const { return !hip_contexts.empty(); }
    [[nodiscard]] IContext *getHIPContext(size_t dev_id) const {
        if (dev_id >= hip_contexts.size())
            throw std::runtime_error("DaphneContext: no HIP context for device " + std::to_string(dev_id) +
                                     " (createHIPContext not called?)");
        return hip_contexts[dev_id].get();
    }
    void startKernelTimer(int kId) {
        std::lock_guard<std::mutex> g(stats_lock);
        kernel_started[kId] = std::chrono::steady_clock::now();
    }
    void stopKernelTimer(int kId) {
        std::lock_guard<std::mutex> g(stats_lock);
        auto &s = kernel_stats[kId];
        s.first++;
        s.second += std::chrono::duration<double>(std::chrono::steady_clock::now() - kernel_started[kId]).count();
    }
};
#define DCTX(varname) DaphneContext *varname

inline void preKernelInstrumentation(int kId, DaphneContext *ctx) {
    if (ctx->getUserConfig().enable_statistics)
        ctx->startKernelTimer(kId);
}
inline void postKernelInstrumentation(int kId, DaphneContext *ctx) {
    if (ctx->getUserConfig().enable_statistics)
        ctx->stopKernelTimer(kId);
}

struct ErrorHandler {
    static constexpr int UNREGISTERED = -1;
    // The exception a generated kernel wrapper throws: the kernel's message, prefixed with the name and the
    // source position of the call site that the dispatch id stands for.
    static std::runtime_error runtimeError(int kId, const std::string &msg, KernelDispatchMapping *kdm) {
        if (kId == UNREGISTERED)
            return std::runtime_error(msg);
        const KernelDispatchInfo kdi = kdm->getKernelDispatchInfo(kId);
        return std::runtime_error("The kernel-function " + kdi.kernelName + " failed during runtime with the following message [ " +
                                  msg + " ]\n" + kdi.fileName + ":" + std::to_string(kdi.line) + ":" + std::to_string(kdi.column));
    }
};

// ------------------------------------------------------------------------------------------
// allocation descriptors and placements
// ------------------------------------------------------------------------------------------
enum class ALLOCATION_TYPE {
    DIST_GRPC, DIST_GRPC_ASYNC, DIST_GRPC_SYNC, DIST_MPI, DIST_SPARK, GPU_CUDA, GPU_HIP, HOST, HOST_PINNED_CUDA,
    FPGA_INT, FPGA_XLX, ONEAPI, NUM_ALLOC_TYPES
};

class IAllocationDescriptor {
  public:
    virtual ~IAllocationDescriptor() = default;
    [[nodiscard]] virtual ALLOCATION_TYPE getType() const = 0;
    virtual void createAllocation(size_t size, bool zero) = 0;
    [[nodiscard]] virtual std::string getLocation() const = 0;
    virtual std::shared_ptr<std::byte> getData() = 0;
    virtual void transferTo(std::byte *src, size_t size) = 0;
    virtual void transferFrom(std::byte *dst, size_t size) = 0;
    [[nodiscard]] virtual std::unique_ptr<IAllocationDescriptor> clone() const = 0;
    virtual bool operator==(const IAllocationDescriptor *other) const = 0;
};

class AllocationDescriptorHost : public IAllocationDescriptor {
  public:
    [[nodiscard]] ALLOCATION_TYPE getType() const override { return ALLOCATION_TYPE::HOST; }
    void createAllocation(size_t, bool) override {}
    [[nodiscard]] std::string getLocation() const override { return "Host"; }
    std::shared_ptr<std::byte> getData() override { return {}; }
    void transferTo(std::byte *, size_t) override {}
    void transferFrom(std::byte *, size_t) override {}
    [[nodiscard]] std::unique_ptr<IAllocationDescriptor> clone() const override {
        return std::make_unique<AllocationDescriptorHost>(*this);
    }
    bool operator==(const IAllocationDescriptor *other) const override { return getType() == other->getType(); }
};

struct DataPlacement {
    size_t dp_id;
    std::unique_ptr<IAllocationDescriptor> allocation;
    explicit DataPlacement(std::unique_ptr<IAllocationDescriptor> a) : dp_id(next_id()++), allocation(std::move(a)) {}
    static std::atomic_size_t &next_id() {
        static std::atomic_size_t n{0};
        return n;
    }
};

class MetaDataObject {
    std::vector<std::unique_ptr<DataPlacement>> data_placements;
    std::vector<size_t> latest_version;

  public:
    std::recursive_mutex lock; // a matrix may be read by several workers at once (TasksCUDA.cpp:27 on shared inputs)
    DataPlacement *addDataPlacement(const IAllocationDescriptor *allocInfo) {
        data_placements.emplace_back(std::make_unique<DataPlacement>(allocInfo->clone()));
        return data_placements.back().get();
    }
    [[nodiscard]] DataPlacement *findDataPlacementByType(const IAllocationDescriptor *alloc_desc) const {
        for (auto &p : data_placements)
            if (p->allocation->operator==(alloc_desc))
                return p.get();
        return nullptr;
    }
    [[nodiscard]] DataPlacement *getDataPlacementByID(size_t id) const {
        for (auto &p : data_placements)
            if (p->dp_id == id)
                return p.get();
        return nullptr;
    }
    [[nodiscard]] size_t numDataPlacements() const { return data_placements.size(); }
    [[nodiscard]] bool isLatestVersion(size_t id) const {
        return std::find(latest_version.begin(), latest_version.end(), id) != latest_version.end();
    }
    void addLatest(size_t id) {
        if (!isLatestVersion(id))
            latest_version.push_back(id);
    }
    void setLatest(size_t id) {
        latest_version.clear();
        latest_version.push_back(id);
    }
    [[nodiscard]] std::vector<size_t> getLatest() const { return latest_version; }
};

// ------------------------------------------------------------------------------------------
// dense matrix
// ------------------------------------------------------------------------------------------
class Structure {
    // Structure.h:30-31, 56-70: data objects are shared by reference counting; DataObjectFactory::destroy drops
    // one reference and deletes the object with the last one.
    mutable std::atomic_size_t refCounter{1};
    friend struct DataObjectFactory;

  public:
    virtual ~Structure() = default;
    [[nodiscard]] virtual size_t getNumRows() const = 0;
    [[nodiscard]] virtual size_t getNumCols() const = 0;
    [[nodiscard]] size_t getNumItems() const { return getNumRows() * getNumCols(); }
    [[nodiscard]] virtual Structure *sliceRow(size_t rl, size_t ru) const = 0;
    [[nodiscard]] size_t getRefCounter() const { return refCounter; }
    void increaseRefCounter() const { refCounter++; }
};

template <typename ValueType> class DenseMatrix : public Structure {
    // what all views of one buffer share: the host copy (allocated on first use), the placements, the size
    struct Buffer {
        std::shared_ptr<ValueType[]> values;
        MetaDataObject mdo;
        size_t items = 0;
        [[nodiscard]] size_t bytes() const { return std::max<size_t>(items, 1) * sizeof(ValueType); }
    };
    size_t numRows, numCols, rowSkip;
    size_t view_offset = 0; // of this matrix's first element in the buffer, in elements
    bool is_view = false;
    std::shared_ptr<Buffer> buf;

    // Makes the placement that `alloc_desc` names (nullptr: host) current and returns (was already current, id,
    // pointer to the first element of the BUFFER in that space). The logic of DenseMatrix.cpp:126-234.
    std::tuple<bool, size_t, ValueType *> getValuesInternal(const IAllocationDescriptor *alloc_desc) {
        std::lock_guard<std::recursive_mutex> g(buf->mdo.lock);
        AllocationDescriptorHost host_desc;
        auto base_of = [&](DataPlacement *p) {
            return p->allocation->getType() == ALLOCATION_TYPE::HOST
                       ? buf->values.get()
                       : reinterpret_cast<ValueType *>(p->allocation->getData().get());
        };
        // the host copy first: every transfer goes through it
        auto host_current = [&]() -> DataPlacement * {
            DataPlacement *hp = buf->mdo.findDataPlacementByType(&host_desc);
            if (hp && buf->mdo.isLatestVersion(hp->dp_id))
                return hp;
            const auto latest = buf->mdo.getLatest();
            if (latest.empty())
                throw std::runtime_error("No object meta data in matrix");
            DataPlacement *src = buf->mdo.getDataPlacementByID(latest.front());
            if (!buf->values)
                buf->values = std::shared_ptr<ValueType[]>(new ValueType[std::max<size_t>(buf->items, 1)]);
            if (!hp)
                hp = buf->mdo.addDataPlacement(&host_desc);
            src->allocation->transferFrom(reinterpret_cast<std::byte *>(buf->values.get()), buf->bytes());
            buf->mdo.addLatest(hp->dp_id);
            return hp;
        };
        const IAllocationDescriptor *want = alloc_desc ? alloc_desc : &host_desc;
        DataPlacement *p = buf->mdo.findDataPlacementByType(want);
        if (p && buf->mdo.isLatestVersion(p->dp_id))
            return {true, p->dp_id, base_of(p)};
        if (want->getType() == ALLOCATION_TYPE::HOST) {
            p = host_current();
            return {true, p->dp_id, base_of(p)};
        }
        host_current();
        if (!p) {
            p = buf->mdo.addDataPlacement(want);
            p->allocation->createAllocation(buf->bytes(), false);
        }
        p->allocation->transferTo(reinterpret_cast<std::byte *>(buf->values.get()), buf->bytes());
        return {false, p->dp_id, base_of(p)};
    }

  public:
    using VT = ValueType;
    // DenseMatrix.cpp:67-87: with a descriptor the matrix lives in that memory space only (no host copy yet)
    DenseMatrix(size_t rows, size_t cols, bool zero, IAllocationDescriptor *allocInfo = nullptr)
        : numRows(rows), numCols(cols), rowSkip(cols), buf(std::make_shared<Buffer>()) {
        buf->items = rows * cols;
        DataPlacement *p;
        if (allocInfo != nullptr) {
            p = buf->mdo.addDataPlacement(allocInfo);
            p->allocation->createAllocation(buf->bytes(), zero);
        } else {
            AllocationDescriptorHost host_desc;
            buf->values = std::shared_ptr<ValueType[]>(new ValueType[std::max<size_t>(buf->items, 1)]);
            if (zero)
                std::fill(buf->values.get(), buf->values.get() + buf->items, ValueType(0));
            p = buf->mdo.addDataPlacement(&host_desc);
        }
        buf->mdo.addLatest(p->dp_id);
    }
    // view of rows [rl, ru) and columns [cl, cu) (DenseMatrix.cpp:98-115)
    DenseMatrix(const DenseMatrix *src, size_t rl, size_t ru, size_t cl, size_t cu)
        : numRows(ru - rl), numCols(cu - cl), rowSkip(src->rowSkip), view_offset(src->view_offset + rl * src->rowSkip + cl),
          is_view(true), buf(src->buf) {
        if (ru < rl || ru > src->numRows || cu < cl || cu > src->numCols)
            throw std::out_of_range("invalid arguments passed to dense matrix constructor: the view must lie inside src");
    }
    [[nodiscard]] size_t getNumRows() const override { return numRows; }
    [[nodiscard]] size_t getNumCols() const override { return numCols; }
    [[nodiscard]] size_t getRowSkip() const { return rowSkip; }
    [[nodiscard]] bool isView() const { return is_view; }
    // DenseMatrix.cpp:110-113: a view's extent in its parent's buffer
    [[nodiscard]] size_t getBufferSize() const { return (is_view ? numRows * rowSkip : numRows * numCols) * sizeof(ValueType); }

    // DenseMatrix.h:221-249
    const ValueType *getValues(const IAllocationDescriptor *alloc_desc = nullptr) const {
        auto *self = const_cast<DenseMatrix *>(this);
        std::lock_guard<std::recursive_mutex> g(buf->mdo.lock);
        auto [isLatest, id, ptr] = self->getValuesInternal(alloc_desc);
        if (!isLatest)
            buf->mdo.addLatest(id);
        return ptr + view_offset;
    }
    ValueType *getValues(IAllocationDescriptor *alloc_desc = nullptr) {
        std::lock_guard<std::recursive_mutex> g(buf->mdo.lock);
        auto [isLatest, id, ptr] = getValuesInternal(alloc_desc);
        (void)isLatest;
        buf->mdo.setLatest(id); // whoever writes here makes every other placement stale
        return ptr + view_offset;
    }
    [[nodiscard]] const MetaDataObject *getMetaDataObject() const { return &buf->mdo; }

    DenseMatrix *slice(size_t rl, size_t ru, size_t cl, size_t cu) const { return new DenseMatrix(this, rl, ru, cl, cu); }
    DenseMatrix *sliceRow(size_t rl, size_t ru) const override { return slice(rl, ru, 0, numCols); }
    DenseMatrix *sliceCol(size_t cl, size_t cu) const { return slice(0, numRows, cl, cu); }
    [[nodiscard]] ValueType get(size_t r, size_t c) const { return getValues()[r * rowSkip + c]; }
    void set(size_t r, size_t c, ValueType v) { getValues()[r * rowSkip + c] = v; }

    // test conveniences: the rows x cols values as one contiguous host vector, and back
    [[nodiscard]] std::vector<ValueType> toHost() const {
        std::vector<ValueType> v(numRows * numCols);
        const ValueType *h = getValues();
        for (size_t r = 0; r < numRows; r++)
            std::copy(h + r * rowSkip, h + r * rowSkip + numCols, v.begin() + r * numCols);
        return v;
    }
    void fromHost(const std::vector<ValueType> &v) {
        ValueType *h = getValues();
        for (size_t r = 0; r < numRows; r++)
            std::copy(v.begin() + r * numCols, v.begin() + (r + 1) * numCols, h + r * rowSkip);
    }
};

struct DataObjectFactory {
    template <class DT> static DT *create(size_t rows, size_t cols, bool zero, IAllocationDescriptor *allocInfo = nullptr) {
        return new DT(rows, cols, zero, allocInfo);
    }
    // DataObjectFactory.h:52-64: drops one reference; the last one deletes the object
    template <class DT> static void destroy(const DT *m) {
        if (!m)
            throw std::runtime_error("DataObjectFactory::destroy() must not be called with nullptr");
        if (--m->refCounter == 0)
            delete m;
    }
    template <class DT, class... Rest> static void destroy(const DT *m, const Rest *...rest) {
        destroy(m);
        destroy(rest...);
    }
};

// genGivenVals of the reference's tests (src/runtime/local/datagen/GenGivenVals.h:68): a host matrix
template <class DT> DT *genGivenVals(size_t numRows, const std::vector<typename DT::VT> &vals) {
    auto *m = DataObjectFactory::create<DT>(numRows, numRows ? vals.size() / numRows : 0, false);
    m->fromHost(vals);
    return m;
}

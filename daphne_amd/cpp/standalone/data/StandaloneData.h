// Stand-ins for the data-object side of DAPHNE's run-time, as far as the HIP kernel layer touches it:
//   IAllocationDescriptor, ALLOCATION_TYPE, AllocationDescriptorHost
//                                       src/runtime/local/datastructures/IAllocationDescriptor.h:21-62
//   DataPlacement, MetaDataObject       src/runtime/local/datastructures/DataPlacement.h, MetaDataObject.{h,cpp}
//   Structure                           src/runtime/local/datastructures/Structure.{h,cpp}
//   DenseMatrix, DataObjectFactory      src/runtime/local/datastructures/DenseMatrix.{h,cpp}, DataObjectFactory.h:34-62
//
// The placement model is the reference's, with the device-view patch of this backend applied
// (patches/0011-dense-matrix-device-views.patch), and it is kept structurally the same so that what is tested here
// holds there:
//   * Every data object has a meta-data object of its own: the placements it knows (per allocation type) and the ids
//     of those that hold its current contents.
//   * A view gets CLONES of its parent's placements, made when the view is made (Structure.cpp:24-36). A cloned
//     descriptor shares the parent's allocation; which placements are current is copied once and not kept in step
//     afterwards. Whoever slices is responsible for making the wanted placement current in the parent first.
//   * The host buffer of a view aliases its parent's host buffer at the view's first element (DenseMatrix.cpp:104-107).
//   * getValues(&descriptor) returns the pointer in the requested memory space, copying there first when that space
//     is not current. The const overload leaves the other placements valid, the non-const one makes the returned
//     placement the only current one.
// What the patch adds to the reference, and this file has as well:
//   * An inherited (cloned) placement addresses its allocation at the view's offset: a view remembers, per inherited
//     placement, where its first element lies in that allocation. In the unpatched reference such a placement yields
//     the allocation's base (DenseMatrix.cpp:176-182), i.e. row 0 of the parent for every view.
//   * Transfers between the host buffer and an inherited placement go to / come from that offset
//     (IAllocationDescriptor::transferToOffset / transferFromOffset).
//   * The non-const getValues() always invalidates the other placements (the reference skips that when the placement
//     was current already, DenseMatrix.h:262-267, so an in-place device kernel leaves a stale host copy marked current).
//   * A host read of an object that is current on a device only registers ONE host placement and marks it current.
// DAPHNE_DENSE_MATRIX_DEVICE_VIEWS tells the kernel layer that views can be handed to device kernels.
#pragma once

#include <algorithm>
#include <array>
#include <atomic>
#include <cstddef>
#include <cstdint>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

#define DAPHNE_DENSE_MATRIX_DEVICE_VIEWS 1

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
    // the same at a position `offset` bytes into the allocation; descriptors that cannot address into their
    // allocation keep these and refuse a view that does not start at the allocation's first byte
    virtual void transferToOffset(std::byte *src, size_t size, size_t offset) {
        if (offset != 0)
            throw std::runtime_error("allocation at " + getLocation() + " cannot be written at an offset");
        transferTo(src, size);
    }
    virtual void transferFromOffset(std::byte *dst, size_t size, size_t offset) {
        if (offset != 0)
            throw std::runtime_error("allocation at " + getLocation() + " cannot be read at an offset");
        transferFrom(dst, size);
    }
    [[nodiscard]] virtual std::unique_ptr<IAllocationDescriptor> clone() const = 0;
    virtual bool operator==(const IAllocationDescriptor *other) const { return getType() == other->getType(); }
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
};

struct Range; // sub-ranges of placements are "under construction" in the reference (DenseMatrix.cpp:236); always null here

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
    std::array<std::vector<std::unique_ptr<DataPlacement>>, static_cast<size_t>(ALLOCATION_TYPE::NUM_ALLOC_TYPES)> data_placements;
    std::vector<size_t> latest_version;

  public:
    DataPlacement *addDataPlacement(const IAllocationDescriptor *allocInfo, Range * = nullptr) {
        auto &of_type = data_placements[static_cast<size_t>(allocInfo->getType())];
        of_type.emplace_back(std::make_unique<DataPlacement>(allocInfo->clone()));
        return of_type.back().get();
    }
    [[nodiscard]] const std::vector<std::unique_ptr<DataPlacement>> *getDataPlacementByType(ALLOCATION_TYPE type) const {
        return &data_placements[static_cast<size_t>(type)];
    }
    [[nodiscard]] const DataPlacement *findDataPlacementByType(const IAllocationDescriptor *alloc_desc, const Range *) const {
        for (auto &p : *getDataPlacementByType(alloc_desc->getType()))
            if (p->allocation->operator==(alloc_desc))
                return p.get();
        return nullptr;
    }
    [[nodiscard]] DataPlacement *getDataPlacementByID(size_t id) const {
        for (auto &of_type : data_placements)
            for (auto &p : of_type)
                if (p->dp_id == id)
                    return p.get();
        return nullptr;
    }
    [[nodiscard]] bool isLatestVersion(size_t id) const {
        return std::find(latest_version.begin(), latest_version.end(), id) != latest_version.end();
    }
    void addLatest(size_t id) { latest_version.push_back(id); }
    void setLatest(size_t id) {
        latest_version.clear();
        latest_version.push_back(id);
    }
    [[nodiscard]] std::vector<size_t> getLatest() const { return latest_version; }
};

// ------------------------------------------------------------------------------------------
// data objects
// ------------------------------------------------------------------------------------------
struct DataObjectFactory {
    // DataObjectFactory.h:34-38: the arguments of any constructor of the data type
    template <class DT, typename... Args> static DT *create(Args... args) { return new DT(args...); }
    // DataObjectFactory.h:52-64: drops one reference; the last one deletes the object
    template <class DT> static void destroy(const DT *obj) {
        if (!obj)
            throw std::runtime_error("DataObjectFactory::destroy() must not be called with nullptr");
        bool last;
        {
            std::lock_guard<std::mutex> g(obj->refCounterMutex);
            last = --obj->refCounter == 0;
        }
        if (last)
            delete obj;
    }
    template <class DT, class... Rest> static void destroy(const DT *obj, const Rest *...rest) {
        destroy(obj);
        destroy(rest...);
    }
};

class Structure {
    mutable size_t refCounter{1};
    mutable std::mutex refCounterMutex;
    friend struct DataObjectFactory;

  protected:
    size_t row_offset{}, col_offset{}; // of a view in the object it was cut from
    size_t numRows, numCols;
    mutable std::shared_ptr<MetaDataObject> mdo;

    Structure(size_t rows, size_t cols) : numRows(rows), numCols(cols), mdo(std::make_shared<MetaDataObject>()) {}

    // Structure.cpp:24-36: one clone per placement of src, in src's order; current ones stay current
    void clone_mdo(const Structure *src) {
        for (size_t t = 0; t < static_cast<size_t>(ALLOCATION_TYPE::NUM_ALLOC_TYPES); t++)
            for (auto &p : *src->mdo->getDataPlacementByType(static_cast<ALLOCATION_TYPE>(t))) {
                DataPlacement *mine = mdo->addDataPlacement(p->allocation.get());
                if (src->mdo->isLatestVersion(p->dp_id))
                    mdo->addLatest(mine->dp_id);
            }
    }

  public:
    virtual ~Structure() = default;
    [[nodiscard]] size_t getNumRows() const { return numRows; }
    [[nodiscard]] size_t getNumCols() const { return numCols; }
    [[nodiscard]] size_t getRefCounter() const { return refCounter; }
    [[nodiscard]] MetaDataObject *getMetaDataObject() const { return mdo.get(); }
    void increaseRefCounter() const {
        std::lock_guard<std::mutex> g(refCounterMutex);
        refCounter++;
    }
    [[nodiscard]] virtual size_t getNumItems() const = 0;
    virtual Structure *sliceRow(size_t rl, size_t ru) const = 0;
    virtual Structure *sliceCol(size_t cl, size_t cu) const = 0;
    virtual Structure *slice(size_t rl, size_t ru, size_t cl, size_t cu) const = 0;
};

template <typename ValueType> class DenseMatrix : public Structure {
    const bool is_view;
    size_t rowSkip;
    std::shared_ptr<ValueType[]> values{}; // host buffer; a view's pointer is its parent's plus the view's offset
    size_t bufferSize;
    // (placement id, elements): where this object's first element lies in the allocation of an inherited placement
    std::vector<std::pair<size_t, size_t>> placementOffsets;

    [[nodiscard]] size_t offsetIn(size_t dp_id) const {
        for (auto &po : placementOffsets)
            if (po.first == dp_id)
                return po.second;
        return 0; // a placement this object made for itself starts at its first element
    }
    // after clone_mdo(src): the clones were added in src's order, so they pair up with src's placements one to one
    void inheritPlacementOffsets(const DenseMatrix *src, size_t extra) {
        for (size_t t = 0; t < static_cast<size_t>(ALLOCATION_TYPE::NUM_ALLOC_TYPES); t++) {
            auto *theirs = src->mdo->getDataPlacementByType(static_cast<ALLOCATION_TYPE>(t));
            auto *mine = mdo->getDataPlacementByType(static_cast<ALLOCATION_TYPE>(t));
            for (size_t i = 0; i < theirs->size() && i < mine->size(); i++)
                placementOffsets.emplace_back((*mine)[i]->dp_id, src->offsetIn((*theirs)[i]->dp_id) + extra);
        }
    }
    // bytes from the first to one past the last element: what a transfer of this object moves
    [[nodiscard]] size_t spanBytes() const {
        if (!is_view)
            return bufferSize;
        return numRows == 0 || numCols == 0 ? 0 : ((numRows - 1) * rowSkip + numCols) * sizeof(ValueType);
    }
    void alloc_shared_values() { values = std::shared_ptr<ValueType[]>(new ValueType[std::max<size_t>(numRows * rowSkip, 1)]); }
    [[nodiscard]] ValueType *deviceAddress(const DataPlacement *p) const {
        return reinterpret_cast<ValueType *>(p->allocation->getData().get()) + offsetIn(p->dp_id);
    }

    // Makes the placement that `alloc_desc` names (nullptr: host) hold the current contents and returns
    // (whether it did before, its id, the pointer to this object's first element there).
    std::tuple<bool, size_t, ValueType *> getValuesInternal(const IAllocationDescriptor *alloc_desc) {
        AllocationDescriptorHost hostDesc;
        const IAllocationDescriptor *want = alloc_desc ? alloc_desc : &hostDesc;
        const bool wantHost = want->getType() == ALLOCATION_TYPE::HOST;
        const DataPlacement *found = mdo->findDataPlacementByType(want, nullptr);
        if (found && mdo->isLatestVersion(found->dp_id))
            return {true, found->dp_id, wantHost ? values.get() : deviceAddress(found)};
        // everything else goes through the host buffer: bring it up to date first
        const DataPlacement *host = wantHost ? found : mdo->findDataPlacementByType(&hostDesc, nullptr);
        if (!(host && mdo->isLatestVersion(host->dp_id))) {
            const auto latest = mdo->getLatest();
            if (latest.empty())
                throw std::runtime_error("No object meta data in matrix");
            DataPlacement *current = mdo->getDataPlacementByID(latest.front());
            if (!values)
                alloc_shared_values();
            if (!host)
                host = mdo->addDataPlacement(&hostDesc);
            current->allocation->transferFromOffset(reinterpret_cast<std::byte *>(values.get()), spanBytes(),
                                                    offsetIn(current->dp_id) * sizeof(ValueType));
            mdo->addLatest(host->dp_id);
        }
        if (wantHost)
            return {true, host->dp_id, values.get()};
        if (!found) {
            DataPlacement *fresh = mdo->addDataPlacement(want);
            fresh->allocation->createAllocation(std::max<size_t>(spanBytes(), sizeof(ValueType)), false);
            found = fresh;
        }
        found->allocation->transferToOffset(reinterpret_cast<std::byte *>(values.get()), spanBytes(),
                                            offsetIn(found->dp_id) * sizeof(ValueType));
        return {false, found->dp_id, deviceAddress(found)};
    }

  public:
    using VT = ValueType;
    // DenseMatrix.cpp:67-87: with a descriptor the matrix lives in that memory space only (no host buffer yet)
    DenseMatrix(size_t maxNumRows, size_t cols, bool zero, IAllocationDescriptor *allocInfo = nullptr)
        : Structure(maxNumRows, cols), is_view(false), rowSkip(cols), bufferSize(maxNumRows * cols * sizeof(ValueType)) {
        DataPlacement *p;
        if (allocInfo != nullptr) {
            p = mdo->addDataPlacement(allocInfo);
            p->allocation->createAllocation(std::max<size_t>(bufferSize, sizeof(ValueType)), zero);
        } else {
            AllocationDescriptorHost hostDesc;
            alloc_shared_values();
            if (zero)
                std::fill(values.get(), values.get() + maxNumRows * cols, ValueType(0));
            p = mdo->addDataPlacement(&hostDesc);
        }
        mdo->addLatest(p->dp_id);
    }
    // a view of rows [rl, ru) and columns [cl, cu) of src (DenseMatrix.cpp:98-115)
    DenseMatrix(const DenseMatrix *src, int64_t rl, int64_t ru, int64_t cl, int64_t cu)
        : Structure(static_cast<size_t>(ru - rl), static_cast<size_t>(cu - cl)), is_view(true), rowSkip(src->rowSkip),
          bufferSize(static_cast<size_t>(ru - rl) * src->rowSkip * sizeof(ValueType)) {
        if (rl < 0 || ru < rl || ru > static_cast<int64_t>(src->numRows) || cl < 0 || cu < cl ||
            cu > static_cast<int64_t>(src->numCols))
            throw std::out_of_range("invalid arguments passed to dense matrix constructor: the view must lie inside src");
        row_offset = static_cast<size_t>(rl);
        col_offset = static_cast<size_t>(cl);
        const size_t first = row_offset * rowSkip + col_offset;
        if (src->values)
            values = std::shared_ptr<ValueType[]>(src->values, src->values.get() + first);
        clone_mdo(src);
        inheritPlacementOffsets(src, first);
    }
    [[nodiscard]] size_t getNumItems() const override { return numRows * numCols; }
    [[nodiscard]] size_t getRowSkip() const { return rowSkip; }
    [[nodiscard]] bool isView() const { return is_view; }
    [[nodiscard]] size_t getBufferSize() const { return bufferSize; }

    // DenseMatrix.h:221-268
    const ValueType *getValues(const IAllocationDescriptor *alloc_desc = nullptr, const Range * = nullptr) const {
        auto [isLatest, id, ptr] = const_cast<DenseMatrix *>(this)->getValuesInternal(alloc_desc);
        if (!isLatest)
            mdo->addLatest(id);
        return ptr;
    }
    ValueType *getValues(IAllocationDescriptor *alloc_desc = nullptr, const Range * = nullptr) {
        auto [isLatest, id, ptr] = getValuesInternal(alloc_desc);
        (void)isLatest;
        mdo->setLatest(id); // whoever asks for write access makes every other placement stale
        return ptr;
    }

    DenseMatrix *slice(size_t rl, size_t ru, size_t cl, size_t cu) const override {
        return DataObjectFactory::create<DenseMatrix>(this, static_cast<int64_t>(rl), static_cast<int64_t>(ru),
                                                      static_cast<int64_t>(cl), static_cast<int64_t>(cu));
    }
    DenseMatrix *sliceRow(size_t rl, size_t ru) const override { return slice(rl, ru, 0, numCols); }
    DenseMatrix *sliceCol(size_t cl, size_t cu) const override { return slice(0, numRows, cl, cu); }
    [[nodiscard]] ValueType get(size_t r, size_t c) const { return getValues()[r * rowSkip + c]; }
    void set(size_t r, size_t c, ValueType v) { getValues()[r * rowSkip + c] = v; }
};

// genGivenVals of the reference's tests (src/runtime/local/datagen/GenGivenVals.h:68): a host matrix
template <class DT> DT *genGivenVals(size_t numRows, const std::vector<typename DT::VT> &vals) {
    const size_t numCols = numRows ? vals.size() / numRows : 0;
    auto *m = DataObjectFactory::create<DT>(numRows, numCols, false);
    std::copy(vals.begin(), vals.end(), m->getValues());
    return m;
}

// AllocationDescriptorHIP: how a DAPHNE data object asks for, fills and reads back memory on a HIP device.
//
// The counterpart of AllocationDescriptorCUDA (src/runtime/local/datastructures/AllocationDescriptorCUDA.h:24-75)
// for ALLOCATION_TYPE::GPU_HIP, which the reference's enum already lists (IAllocationDescriptor.h:30). A kernel
// builds one on its stack, `AllocationDescriptorHIP alloc_desc(ctx, deviceID)`, and passes it to
// `m->getValues(&alloc_desc)` for a device pointer (the matrix uploads itself on first use and remembers the
// placement) and to `DataObjectFactory::create<DT>(rows, cols, zero, &alloc_desc)` for a result that exists on the
// device only. The buffer is shared between the context's registry and every clone of the descriptor that a
// placement holds (a view's placements are clones of its parent's, so a view addresses into its parent's buffer);
// the clone that finds itself the last holder outside the registry unregisters it. The offset forms of the
// transfers exist in IAllocationDescriptor once patches/0011-dense-matrix-device-views.patch is applied.
//
// In DAPHNE this file is src/runtime/local/datastructures/AllocationDescriptorHIP.h.
#pragma once

#include <runtime/local/context/HIPContext.h>
#include <runtime/local/datastructures/DataPlacement.h>
#include <runtime/local/datastructures/IAllocationDescriptor.h>

class AllocationDescriptorHIP : public IAllocationDescriptor {
    ALLOCATION_TYPE type = ALLOCATION_TYPE::GPU_HIP;
    uint32_t device_id{};
    DaphneContext *dctx{};
    std::shared_ptr<std::byte> data;
    size_t alloc_id{};

  public:
    AllocationDescriptorHIP() = delete;
    AllocationDescriptorHIP(DaphneContext *ctx, uint32_t device_id) : device_id(device_id), dctx(ctx) {}

    ~AllocationDescriptorHIP() override {
        // two holders left: the context's registry and this descriptor
        if (data && data.use_count() == 2) {
            try {
                HIPContext::get(dctx, device_id)->free(alloc_id);
            } catch (const std::exception &) {
                // the context is gone already: its destroy() released the device memory
            }
        }
    }

    [[nodiscard]] ALLOCATION_TYPE getType() const override { return type; }
    [[nodiscard]] std::string getLocation() const override { return std::to_string(device_id); }

    void createAllocation(size_t size, bool zero) override {
        data = HIPContext::get(dctx, device_id)->malloc(size, zero, alloc_id);
    }
    std::shared_ptr<std::byte> getData() override { return data; }

    [[nodiscard]] std::unique_ptr<IAllocationDescriptor> clone() const override {
        return std::make_unique<AllocationDescriptorHIP>(*this);
    }

    // synchronous copies, like the reference's cudaMemcpy calls
    void transferTo(std::byte *src, size_t size) override {
        if (!src)
            throw std::runtime_error("src ptr requested for transfer to device is null");
        HIP::check(dh_h2d(HIPContext::get(dctx, device_id)->raw(), data.get(), src, size));
    }
    void transferFrom(std::byte *dst, size_t size) override {
        HIP::check(dh_d2h(HIPContext::get(dctx, device_id)->raw(), dst, data.get(), size));
    }
    // the same for a view that starts `offset` bytes into the allocation it shares with its parent
    void transferToOffset(std::byte *src, size_t size, size_t offset) override {
        if (!src)
            throw std::runtime_error("src ptr requested for transfer to device is null");
        if (size != 0)
            HIP::check(dh_h2d(HIPContext::get(dctx, device_id)->raw(), data.get() + offset, src, size));
    }
    void transferFromOffset(std::byte *dst, size_t size, size_t offset) override {
        if (size != 0)
            HIP::check(dh_d2h(HIPContext::get(dctx, device_id)->raw(), dst, data.get() + offset, size));
    }

    bool operator==(const IAllocationDescriptor *other) const override {
        if (getType() == other->getType())
            return getLocation() == dynamic_cast<const AllocationDescriptorHIP *>(other)->getLocation();
        return false;
    }
};

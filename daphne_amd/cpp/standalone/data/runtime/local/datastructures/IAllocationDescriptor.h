// Stand-in for DAPHNE's src/runtime/local/datastructures/IAllocationDescriptor.h (IAllocationDescriptor, ALLOCATION_TYPE, AllocationDescriptorHost): see StandaloneData.h.
#pragma once
#include <StandaloneData.h>

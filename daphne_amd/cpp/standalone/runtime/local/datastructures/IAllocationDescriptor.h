// Stand-in for DAPHNE's src/runtime/local/datastructures/IAllocationDescriptor.h (IAllocationDescriptor, ALLOCATION_TYPE, AllocationDescriptorHost): see DaphneStandalone.h.
#pragma once
#include <DaphneStandalone.h>

// Shadows the reference's runtime/local/io/DaphneSerializer.h, which drags in the I/O layer: the tests never serialise.
#pragma once
#include <cstddef>
#include <stdexcept>
#include <vector>
template <class DT> struct DaphneSerializer {
    static size_t serialize(const DT *, std::vector<char> &) { throw std::runtime_error("serialisation is not part of this build"); }
};

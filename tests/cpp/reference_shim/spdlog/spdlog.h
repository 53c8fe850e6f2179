// Shadows spdlog/spdlog.h, which the reference's DenseMatrix.cpp includes for its debug messages and which is not
// installed here: the messages are dropped.
#pragma once
namespace spdlog {
template <typename... Args> inline void debug(Args &&...) {}
} // namespace spdlog

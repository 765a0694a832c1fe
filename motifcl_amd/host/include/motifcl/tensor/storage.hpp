// Device storage of a tensor (include/motifcl/tensor/storage.hpp:12-29 of MotifCL): one
// allocation from the library's pooled allocator, returned to the pool on destruction.
#pragma once

#include <cstddef>

namespace motifcl {

class Backend;

class Storage {
public:
    Storage() = default;
    Storage(Backend& backend, std::size_t nbytes);
    ~Storage();

    Storage(const Storage&) = delete;
    Storage& operator=(const Storage&) = delete;

    void* hip_ptr = nullptr;
    std::size_t nbytes = 0;
    bool pooled = true;
};

void clear_memory_pool();

}  // namespace motifcl

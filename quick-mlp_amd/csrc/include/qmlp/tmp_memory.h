#pragma once

#include "common.h"

#include <cstddef>

QUICKMLP_NAMESPACE_BEGIN

/**
 * RAII-style temporary device memory. If 'numBytes' is zero, no memory is
 * allocated and get() returns nullptr.
 */
class TmpMemory
{
    void* memory_;

public:
    explicit TmpMemory(size_t numBytes);
    ~TmpMemory();

    TmpMemory(const TmpMemory& other) = delete;
    TmpMemory(TmpMemory&& other) noexcept = delete;
    TmpMemory& operator=(const TmpMemory& other) = delete;
    TmpMemory& operator=(TmpMemory&& other) noexcept = delete;

    [[nodiscard]] void* get() { return memory_; }
    [[nodiscard]] const void* get() const { return memory_; }
};

QUICKMLP_NAMESPACE_END

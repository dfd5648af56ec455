// Capture of one run of a program into a device graph, and its replay.  The reference's interpreter
// launches every kernel from the host (runtime/chxvm.cc:168-236); for a network of a hundred short
// kernels the host is then the bottleneck.  A quantized-inference program does the same thing on every
// run (no control flow, no shapes that depend on data), so one run can be recorded and replayed.
#pragma once

#include <mutex>
#include <string>
#include <vector>

#include "chainerx_lite.h"

namespace chainer_compiler {
namespace runtime {

// Device blocks for the runs of one captured program.  A released block is handed out again to the next
// request it fits (the smallest such block, the oldest among equals), so runs that ask for the same sizes in
// the same order get the same addresses once the pool holds every block they need.  Blocks go back to the
// device runtime when the pool is destroyed; handles keep the pool alive.
class PoolAllocator : public chainerx::DeviceAllocator, public std::enable_shared_from_this<PoolAllocator> {
public:
    PoolAllocator() = default;
    ~PoolAllocator() override;
    std::shared_ptr<void> Allocate(size_t bytes) override;
    // frozen: a request that no free block fits fails instead of going to the device runtime
    void set_frozen(bool frozen) {
        frozen_ = frozen;
    }
    int64_t blocks_created() const {
        return static_cast<int64_t>(blocks_.size());
    }
    int64_t bytes_reserved() const {
        return bytes_reserved_;
    }

private:
    struct Block {
        void* ptr;
        size_t size;
        bool free;
    };
    void Release(size_t index);

    std::mutex mu_;
    std::vector<Block> blocks_;
    int64_t bytes_reserved_ = 0;
    bool frozen_ = false;
};

}  // namespace runtime
}  // namespace chainer_compiler

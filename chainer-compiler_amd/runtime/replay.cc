#include "replay.h"

#include "log.h"

namespace chainer_compiler {
namespace runtime {

PoolAllocator::~PoolAllocator() {
    for (Block& b : blocks_) (void)chx_hip_free(b.ptr);
}

std::shared_ptr<void> PoolAllocator::Allocate(size_t bytes) {
    const size_t want = (bytes + 255) / 256 * 256;
    size_t index = 0;
    void* ptr = nullptr;  // read under the lock: a concurrent Allocate may grow (move) the vector
    {
        std::lock_guard<std::mutex> lock(mu_);
        size_t best = blocks_.size();
        for (size_t i = 0; i < blocks_.size(); ++i)
            if (blocks_[i].free && blocks_[i].size >= want && (best == blocks_.size() || blocks_[i].size < blocks_[best].size)) best = i;
        if (best == blocks_.size()) {
            CHECK(!frozen_) << "a run that is being captured asked for " << bytes
                            << " bytes that the runs before it did not: the program does not allocate the same way on every run";
            void* p = nullptr;
            CHXVM_HIP_CALL(chx_hip_malloc(&p, want));
            blocks_.push_back(Block{p, want, false});
            bytes_reserved_ += static_cast<int64_t>(want);
        } else {
            blocks_[best].free = false;
        }
        index = best;
        ptr = blocks_[index].ptr;
    }
    std::shared_ptr<PoolAllocator> self = shared_from_this();
    return std::shared_ptr<void>(ptr, [self, index](void*) { self->Release(index); });
}

void PoolAllocator::Release(size_t index) {
    std::lock_guard<std::mutex> lock(mu_);
    blocks_[index].free = true;
}

}  // namespace runtime
}  // namespace chainer_compiler

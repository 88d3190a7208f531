// Block allocator: best-fit free blocks with address-adjacent coalescing inside large pages, and logical allocation
// streams that say who may reuse a freed block while the device may still be working on it
// (helium/src/cuda/allocator/block.rs). Pure host logic over address ranges: it never touches the device, so it is
// tested without one.
#pragma once
#include <cstddef>
#include <cstdint>
#include <map>
#include <set>
#include <unordered_map>
#include <vector>

namespace he::alloc {

using StreamId = uint64_t;  // 0: no stream
using PageId = uint32_t;

struct Block {
    PageId page = 0;
    uint64_t start = 0, size = 0;
    // Streams whose device work may still touch the block (block.rs:286-299). A free block can be handed out when the
    // set is empty, or when every member is the allocating stream or one of its ancestors: their work is over by the
    // time the new owner's work runs.
    std::set<StreamId> in_use;
    uint64_t end() const { return start + size; }
    bool overlaps(const Block& o) const { return page == o.page && start < o.end() && o.start < end(); }
};

class BlockAllocator {
public:
    PageId add_page(uint64_t size);
    // Smallest free block that fits `size` at alignment `align` and whose streams allow it; splits off what is not
    // needed on either side. Returns false when no block fits.
    bool allocate(uint64_t size, uint64_t align, StreamId stream, Block* out);
    void deallocate(Block block);
    // `parent`: a stream whose work completes before the new stream's work begins (0: none).
    StreamId begin_stream(StreamId parent);
    // The stream's device work has finished: blocks it freed become available to everyone.
    void end_stream(StreamId id);
    bool stream_is_live(StreamId id) const { return streams_.count(id) != 0; }

    size_t num_free_blocks() const { return free_.size(); }
    size_t num_streams() const { return streams_.size(); }
    uint64_t free_bytes() const;
    uint64_t largest_free_block() const { return by_size_.empty() ? 0 : by_size_.rbegin()->first; }
    // Index consistency (every free block in both indices exactly once, no two free blocks of a page overlapping or
    // mergeable, stream back-references exact); throws he::Error on a violation.
    void check_invariants() const;

private:
    using BlockId = uint64_t;
    struct Stream {
        std::set<BlockId> blocks_in_use;
        std::set<StreamId> ancestors;
    };
    void add_free_block(Block block);
    Block remove_free_block(BlockId id);
    std::unordered_map<BlockId, Block> free_;
    std::map<uint64_t, std::set<BlockId>> by_size_;
    std::vector<std::map<uint64_t, BlockId>> by_addr_;  // per page: start -> free block
    std::vector<uint64_t> page_size_;
    std::map<StreamId, Stream> streams_;
    BlockId next_block_ = 1;
    StreamId next_stream_ = 1;
};

}  // namespace he::alloc

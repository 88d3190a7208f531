#include "alloc.h"

#include <algorithm>
#include <iterator>

#include "common.h"

namespace he::alloc {

PageId BlockAllocator::add_page(uint64_t size) {
    HE_REQUIRE(size > 0, HE_ERR_INVALID, "empty page");
    const PageId page = (PageId)by_addr_.size();
    by_addr_.emplace_back();
    page_size_.push_back(size);
    Block b;
    b.page = page;
    b.start = 0;
    b.size = size;
    add_free_block(std::move(b));
    return page;
}

bool BlockAllocator::allocate(uint64_t size, uint64_t align, StreamId stream, Block* out) {
    HE_REQUIRE(size > 0 && align > 0 && (align & (align - 1)) == 0, HE_ERR_INVALID, "bad allocation request");
    const Stream* me = nullptr;
    if (stream) {
        auto it = streams_.find(stream);
        HE_REQUIRE(it != streams_.end(), HE_ERR_INVALID, "allocation in a stream that has ended");
        me = &it->second;
    }
    for (auto cls = by_size_.lower_bound(size); cls != by_size_.end(); ++cls) {
        for (BlockId id : cls->second) {
            const Block& cand = free_.at(id);
            bool allowed = true;
            for (StreamId s : cand.in_use)
                allowed = allowed && me && (s == stream || me->ancestors.count(s));
            if (!allowed) continue;
            const uint64_t offset = cand.start % align ? align - cand.start % align : 0;
            if (offset > cand.size || cand.size - offset < size) continue;
            Block b = remove_free_block(id);
            if (offset) {
                Block head = b;
                head.size = offset;
                b.start += offset;
                b.size -= offset;
                add_free_block(std::move(head));
            }
            if (b.size > size) {
                Block tail = b;
                tail.start = b.start + size;
                tail.size = b.size - size;
                b.size = size;
                add_free_block(std::move(tail));
            }
            if (stream) b.in_use.insert(stream);
            *out = std::move(b);
            return true;
        }
    }
    return false;
}

void BlockAllocator::deallocate(Block block) {
    HE_REQUIRE(block.page < by_addr_.size() && block.size > 0 && block.end() <= page_size_[block.page], HE_ERR_INVALID,
               "block does not belong to this allocator");
    add_free_block(std::move(block));
}

void BlockAllocator::add_free_block(Block block) {
    // streams that have ended no longer hold anything back
    for (auto it = block.in_use.begin(); it != block.in_use.end();)
        it = streams_.count(*it) ? std::next(it) : block.in_use.erase(it);
    // merge with the free neighbours on either side when the same streams hold them
    auto& by_addr = by_addr_[block.page];
    for (int side = 0; side < 2; side++) {
        BlockId neighbour = 0;
        if (side == 0) {
            auto it = by_addr.lower_bound(block.start);
            if (it != by_addr.begin()) neighbour = std::prev(it)->second;
        } else {
            auto it = by_addr.upper_bound(block.start);
            if (it != by_addr.end()) neighbour = it->second;
        }
        if (!neighbour) continue;
        const Block& n = free_.at(neighbour);
        const bool adjacent = n.end() == block.start || block.end() == n.start;
        if (!adjacent || n.in_use != block.in_use) continue;
        Block gone = remove_free_block(neighbour);
        const uint64_t start = std::min(block.start, gone.start), end = std::max(block.end(), gone.end());
        block.start = start;
        block.size = end - start;
    }
    const BlockId id = next_block_++;
    by_size_[block.size].insert(id);
    by_addr[block.start] = id;
    for (StreamId s : block.in_use) streams_.at(s).blocks_in_use.insert(id);
    free_.emplace(id, std::move(block));
}

Block BlockAllocator::remove_free_block(BlockId id) {
    auto it = free_.find(id);
    HE_REQUIRE(it != free_.end(), HE_ERR_INTERNAL, "free block %llu is gone", (unsigned long long)id);
    Block b = std::move(it->second);
    free_.erase(it);
    by_addr_[b.page].erase(b.start);
    auto cls = by_size_.find(b.size);
    cls->second.erase(id);
    if (cls->second.empty()) by_size_.erase(cls);
    for (StreamId s : b.in_use) {
        auto st = streams_.find(s);
        if (st != streams_.end()) st->second.blocks_in_use.erase(id);
    }
    return b;
}

StreamId BlockAllocator::begin_stream(StreamId parent) {
    Stream s;
    auto p = streams_.find(parent);
    if (parent && p != streams_.end()) {
        s.ancestors = p->second.ancestors;
        s.ancestors.insert(parent);
    }
    const StreamId id = next_stream_++;
    streams_.emplace(id, std::move(s));
    return id;
}

void BlockAllocator::end_stream(StreamId id) {
    auto it = streams_.find(id);
    HE_REQUIRE(it != streams_.end(), HE_ERR_INVALID, "stream %llu has already ended", (unsigned long long)id);
    const std::set<BlockId> held = std::move(it->second.blocks_in_use);
    streams_.erase(it);
    for (BlockId b : held) {
        // an earlier re-insertion of this loop may have merged the block away
        if (!free_.count(b)) continue;
        Block block = remove_free_block(b);
        block.in_use.erase(id);
        add_free_block(std::move(block));
    }
    for (auto& kv : streams_) kv.second.ancestors.erase(id);
}

uint64_t BlockAllocator::free_bytes() const {
    uint64_t n = 0;
    for (auto& kv : free_) n += kv.second.size;
    return n;
}

void BlockAllocator::check_invariants() const {
    size_t in_size_index = 0, in_addr_index = 0;
    for (auto& cls : by_size_) {
        HE_REQUIRE(!cls.second.empty(), HE_ERR_INTERNAL, "empty size class");
        for (BlockId id : cls.second) {
            auto it = free_.find(id);
            HE_REQUIRE(it != free_.end() && it->second.size == cls.first, HE_ERR_INTERNAL, "size index out of date");
            in_size_index++;
        }
    }
    for (PageId p = 0; p < by_addr_.size(); p++) {
        const Block* prev = nullptr;
        for (auto& kv : by_addr_[p]) {
            auto it = free_.find(kv.second);
            HE_REQUIRE(it != free_.end() && it->second.start == kv.first && it->second.page == p, HE_ERR_INTERNAL,
                       "address index out of date");
            const Block& b = it->second;
            HE_REQUIRE(b.end() <= page_size_[p], HE_ERR_INTERNAL, "free block leaves its page");
            if (prev) {
                HE_REQUIRE(prev->end() <= b.start, HE_ERR_INTERNAL, "free blocks overlap");
                HE_REQUIRE(prev->end() != b.start || prev->in_use != b.in_use, HE_ERR_INTERNAL, "unmerged neighbours");
            }
            for (StreamId s : b.in_use) {
                auto st = streams_.find(s);
                HE_REQUIRE(st != streams_.end() && st->second.blocks_in_use.count(kv.second), HE_ERR_INTERNAL,
                           "stream back-reference missing");
            }
            prev = &b;
            in_addr_index++;
        }
    }
    HE_REQUIRE(in_size_index == free_.size() && in_addr_index == free_.size(), HE_ERR_INTERNAL, "index sizes differ");
    for (auto& st : streams_)
        for (BlockId id : st.second.blocks_in_use) {
            auto it = free_.find(id);
            HE_REQUIRE(it != free_.end() && it->second.in_use.count(st.first), HE_ERR_INTERNAL, "stale stream reference");
        }
}

}  // namespace he::alloc

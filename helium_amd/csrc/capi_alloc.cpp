// C ABI of the block allocator (host logic only) and of the device pool built on it.
#include "exec.h"

struct he_block_allocator_s {
    he::alloc::BlockAllocator a;
};

namespace {
void to_c(const he::alloc::Block& b, he_block* out) {
    out->page = b.page;
    out->start = b.start;
    out->size = b.size;
    out->num_streams = 0;
    for (uint64_t s : b.in_use) {
        HE_REQUIRE(out->num_streams < 8, HE_ERR_INTERNAL, "block held by more than 8 streams");
        out->streams[out->num_streams++] = s;
    }
}
he::alloc::Block from_c(const he_block* in) {
    HE_REQUIRE(in && in->num_streams >= 0 && in->num_streams <= 8, HE_ERR_INVALID, "bad block");
    he::alloc::Block b;
    b.page = in->page;
    b.start = in->start;
    b.size = in->size;
    for (int i = 0; i < in->num_streams; i++) b.in_use.insert(in->streams[i]);
    return b;
}
}  // namespace

extern "C" {

int he_block_allocator_create(he_block_allocator_t* allocator) {
    return he::guard([&] {
        HE_REQUIRE(allocator, HE_ERR_INVALID, "bad argument");
        *allocator = new he_block_allocator_s();
    });
}
int he_block_allocator_destroy(he_block_allocator_t allocator) {
    delete allocator;
    return HE_OK;
}
int he_block_allocator_add_page(he_block_allocator_t allocator, uint64_t size, uint32_t* page) {
    return he::guard([&] {
        HE_REQUIRE(allocator && page, HE_ERR_INVALID, "bad argument");
        *page = allocator->a.add_page(size);
    });
}
int he_block_allocator_allocate(he_block_allocator_t allocator, uint64_t size, uint64_t align, uint64_t stream,
                                he_block* block, int* found) {
    return he::guard([&] {
        HE_REQUIRE(allocator && block && found, HE_ERR_INVALID, "bad argument");
        he::alloc::Block b;
        *found = allocator->a.allocate(size, align, stream, &b) ? 1 : 0;
        if (*found) to_c(b, block);
    });
}
int he_block_allocator_deallocate(he_block_allocator_t allocator, const he_block* block) {
    return he::guard([&] {
        HE_REQUIRE(allocator, HE_ERR_INVALID, "bad argument");
        allocator->a.deallocate(from_c(block));
    });
}
int he_block_allocator_begin_stream(he_block_allocator_t allocator, uint64_t parent, uint64_t* stream) {
    return he::guard([&] {
        HE_REQUIRE(allocator && stream, HE_ERR_INVALID, "bad argument");
        *stream = allocator->a.begin_stream(parent);
    });
}
int he_block_allocator_end_stream(he_block_allocator_t allocator, uint64_t stream) {
    return he::guard([&] {
        HE_REQUIRE(allocator, HE_ERR_INVALID, "bad argument");
        allocator->a.end_stream(stream);
    });
}
int he_block_allocator_stats(he_block_allocator_t allocator, uint64_t stats[4]) {
    return he::guard([&] {
        HE_REQUIRE(allocator && stats, HE_ERR_INVALID, "bad argument");
        allocator->a.check_invariants();
        stats[0] = allocator->a.num_free_blocks();
        stats[1] = allocator->a.free_bytes();
        stats[2] = allocator->a.largest_free_block();
        stats[3] = allocator->a.num_streams();
    });
}

int he_pool_begin_scope(uint64_t thread, uint64_t* scope) {
    return he::guard([&] {
        HE_REQUIRE(scope, HE_ERR_INVALID, "bad argument");
        *scope = he::exec::DevicePool::global().begin_scope(thread);
    });
}
int he_pool_end_scope(uint64_t scope) {
    return he::guard([&] { he::exec::DevicePool::global().end_scope(scope); });
}
int he_pool_allocate(size_t bytes, uint64_t scope, void** ptr, he_block* block) {
    return he::guard([&] {
        HE_REQUIRE(ptr && block, HE_ERR_INVALID, "bad argument");
        he::exec::Allocation a = he::exec::DevicePool::global().allocate(bytes, scope);
        *ptr = a.ptr;
        to_c(a.block, block);
    });
}
int he_pool_release(void* ptr, const he_block* block, uint64_t scope) {
    return he::guard([&] {
        HE_REQUIRE(ptr, HE_ERR_INVALID, "bad argument");
        he::exec::Allocation a;
        a.ptr = ptr;
        a.block = from_c(block);
        he::exec::DevicePool::global().release(a, scope, {});
    });
}

}  // extern "C"

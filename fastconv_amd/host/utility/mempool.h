// Memory pools of the layer graph, with the interface of the reference's
// utility/mempool.h:23-71 (bool returns, message on stderr), but handing out
// DEVICE memory: every pointer comes from a RangeAllocator over a block of the
// single hipMalloc'd arena.
//
//   CommonMemPool   scratch shared by all layers: each layer Request()s what it
//                   needs, Alloc() then makes ONE buffer of the largest request
//                   (layers run one after another, so they can share it), plus
//                   one buffer per numbered pool id.
//   PrivateMemPool  buffers a layer keeps for itself (transformed filters,
//                   packed weights), allocated and freed individually.
#ifndef TCNN_MEMORY_POOL_H_
#define TCNN_MEMORY_POOL_H_

#include <stdio.h>

#include <map>

#include "range_allocator.h"

#define MEMPOOL_CHECK_RETURN(var)                                            \
    {                                                                        \
        if (!(var)) {                                                        \
            fprintf(stderr, "Err in file %s line %d\n", __FILE__, __LINE__); \
            return false;                                                    \
        }                                                                    \
    }

template <typename PTR_TYPE>
class CommonMemPool {
   public:
    explicit CommonMemPool(fastconv::RangeAllocator *allocator)
        : alloc_(allocator), common_size(0), common_memory(NULL) {}
    ~CommonMemPool() {
        if (common_memory || common_size_map.size() || common_ptr_map.size()) FreeAll();
    }

    // Single common memory pool: the size grows to the largest request.
    bool Request(size_t size_byte) {
        common_size = (common_size > size_byte) ? common_size : size_byte;
        return true;
    }
    bool GetPtr(PTR_TYPE **ptr) {
        if (!common_memory) {
            fprintf(stderr, "Error: common memory not allocated.\n");
            return false;
        }
        *ptr = common_memory;
        return true;
    }
    bool Free() {
        if (common_memory) {
            alloc_->Free(common_memory);
            common_size = 0;
            common_memory = NULL;
        }
        return true;
    }

    // Multiple common pools by ID.
    bool Request(size_t size_byte, size_t id) {
        std::map<size_t, size_t>::iterator it = common_size_map.find(id);
        if (it != common_size_map.end())
            it->second = it->second > size_byte ? it->second : size_byte;
        else
            common_size_map[id] = size_byte;
        return true;
    }
    bool GetPtr(PTR_TYPE **ptr, size_t id) {
        typename std::map<size_t, PTR_TYPE *>::iterator it = common_ptr_map.find(id);
        if (it == common_ptr_map.end() || it->second == NULL) {
            fprintf(stderr, "Error: common memory id %zu not allocated.\n", id);
            return false;
        }
        *ptr = it->second;
        return true;
    }
    bool Free(size_t id) {
        std::map<size_t, size_t>::iterator it = common_size_map.find(id);
        if (it == common_size_map.end()) {
            fprintf(stderr, "Error: free common memory id %zu failed: ID doesn't exist\n", id);
            return false;
        }
        typename std::map<size_t, PTR_TYPE *>::iterator pit = common_ptr_map.find(id);
        if (pit != common_ptr_map.end()) {
            if (pit->second) alloc_->Free(pit->second);
            common_ptr_map.erase(pit);
        }
        common_size_map.erase(it);
        return true;
    }

    // Allocates the default pool at its requested size and every ID pool.
    bool Alloc() {
        if (common_memory) {
            fprintf(stderr, "Error: common memory already allocated.\n");
            return false;
        }
        if (common_size > 0) {
            common_memory = (PTR_TYPE *)alloc_->Allocate(common_size);
            if (!common_memory) {
                fprintf(stderr, "Error: cannot allocate common memory.\n");
                return false;
            }
        }
        bool ok = true;
        for (std::map<size_t, size_t>::iterator it = common_size_map.begin(); it != common_size_map.end(); ++it) {
            if (common_ptr_map.count(it->first) && common_ptr_map[it->first]) continue;
            PTR_TYPE *wptr = (PTR_TYPE *)alloc_->Allocate(it->second);
            if (!wptr) {
                fprintf(stderr, "Allocation for size %zu id %zu failed\n", it->second, it->first);
                ok = false;
                continue;
            }
            common_ptr_map[it->first] = wptr;
        }
        return ok && common_ptr_map.size() == common_size_map.size();
    }
    // Grows the default pool to at least size_byte (contents are not kept).
    bool Alloc(size_t size_byte) {
        if (size_byte > common_size || !common_memory) {
            if (common_memory) alloc_->Free(common_memory);
            common_memory = NULL;
            if (size_byte > common_size) common_size = size_byte;
            common_memory = (PTR_TYPE *)alloc_->Allocate(common_size);
            if (common_memory == NULL) return false;
        }
        return true;
    }
    bool FreeAll() {
        Free();
        for (typename std::map<size_t, PTR_TYPE *>::iterator it = common_ptr_map.begin(); it != common_ptr_map.end();
             ++it)
            if (it->second) alloc_->Free(it->second);
        common_ptr_map.clear();
        common_size_map.clear();
        return true;
    }
    void PrintStats() {
        printf("Default common pool stat: size %zu, ptr %p\n", common_size, (void *)common_memory);
        for (std::map<size_t, size_t>::iterator it = common_size_map.begin(); it != common_size_map.end(); ++it)
            printf("Pool id %zu size %zu ptr %p\n", it->first, it->second,
                   common_ptr_map.count(it->first) ? (void *)common_ptr_map[it->first] : NULL);
    }
    size_t common_bytes() const { return common_size; }

   private:
    fastconv::RangeAllocator *alloc_;
    size_t common_size;
    PTR_TYPE *common_memory;
    std::map<size_t, size_t> common_size_map;        // ID -> size
    std::map<size_t, PTR_TYPE *> common_ptr_map;     // ID -> pointer
};

template <typename PTR_TYPE>
class PrivateMemPool {
   public:
    explicit PrivateMemPool(fastconv::RangeAllocator *allocator) : alloc_(allocator) {}
    ~PrivateMemPool() {
        if (private_map.size()) FreeAll();
    }

    bool Alloc(PTR_TYPE **ptr, size_t size_byte) {
        PTR_TYPE *wptr = (PTR_TYPE *)alloc_->Allocate(size_byte);
        if (!wptr) {
            fprintf(stderr, "Allocation of size %zu failed\n", size_byte);
            *ptr = NULL;
            return false;
        }
        private_map[wptr] = size_byte;
        *ptr = wptr;
        return true;
    }
    bool GetSize(PTR_TYPE *ptr, size_t *size_byte) {
        typename std::map<PTR_TYPE *, size_t>::iterator it = private_map.find(ptr);
        if (it == private_map.end()) {
            fprintf(stderr, "Error in free private memory: ptr not found in map\n");
            return false;
        }
        *size_byte = it->second;
        return true;
    }
    bool Free(PTR_TYPE **ptr) {
        typename std::map<PTR_TYPE *, size_t>::iterator it = private_map.find(*ptr);
        if (it == private_map.end()) {
            fprintf(stderr, "Error in free private memory: ptr not found in map\n");
            return false;
        }
        alloc_->Free(it->first);
        private_map.erase(it);
        *ptr = NULL;
        return true;
    }
    bool FreeAll() {
        for (typename std::map<PTR_TYPE *, size_t>::iterator it = private_map.begin(); it != private_map.end(); ++it)
            alloc_->Free(it->first);
        private_map.clear();
        return true;
    }
    void PrintStats() {
        size_t total_mem_size = 0;
        for (typename std::map<PTR_TYPE *, size_t>::iterator it = private_map.begin(); it != private_map.end(); ++it) {
            printf("Private memory ptr %p size %zu\n", (void *)it->first, it->second);
            total_mem_size += it->second;
        }
        printf("Private memories occupy %zu bytes in %zu buffers\n", total_mem_size, private_map.size());
    }
    size_t count() const { return private_map.size(); }

   private:
    fastconv::RangeAllocator *alloc_;
    std::map<PTR_TYPE *, size_t> private_map;        // pointer -> size
};
#endif

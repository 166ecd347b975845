// Device memory for the descriptor tables of the prepared collectives: carved out of a few large
// allocations and handed back all at once (freeing device memory waits for the whole device, so it is
// kept off the path of a caller that cycles through many buffers).
//
// Blocks can be pinned: a collective recorded into a caller's HIP graph leaves kernel nodes in that
// graph whose arguments point at its tables, and the caller may replay the graph at any later time.
// A chunk with a pinned block survives Reset() with everything in it; it takes no further blocks.
//
// Header-only and free of HIP types on purpose: the memory comes from two function pointers, so the
// bookkeeping can be exercised on a machine without a GPU.
#pragma once
#include <cstddef>
#include <cstdint>
#include <vector>

namespace hcclamd {

struct TableArena {
    typedef void *(*AllocFn)(size_t bytes);   // nullptr on failure
    typedef void (*FreeFn)(void *mem);

    struct Chunk {
        char *base = nullptr;
        size_t size = 0, used = 0;
        uint32_t pinned = 0;      // pinned blocks inside
        bool sealed = false;      // survived a Reset with pinned blocks: kept as it is, takes no new blocks
    };
    std::vector<Chunk> chunks;
    AllocFn allocFn = nullptr;
    FreeFn freeFn = nullptr;
    size_t chunkBytes = size_t(4) << 20;

    // A block of `bytes` (rounded up to 256); *chunkId names the chunk for Pin().  nullptr when out of memory.
    void *Alloc(size_t bytes, uint32_t *chunkId)
    {
        bytes = (bytes + 255) & ~size_t(255);
        if (chunks.empty() || chunks.back().sealed || chunks.back().size - chunks.back().used < bytes) {
            Chunk c;
            c.size = bytes > chunkBytes ? bytes : chunkBytes;
            c.base = static_cast<char *>(allocFn(c.size));
            if (c.base == nullptr) {
                return nullptr;
            }
            chunks.push_back(c);
        }
        Chunk &c = chunks.back();
        void *out = c.base + c.used;
        c.used += bytes;
        if (chunkId != nullptr) {
            *chunkId = uint32_t(chunks.size() - 1);
        }
        return out;
    }

    // The block handed out from chunk `chunkId` must stay valid until FreeAll().
    void Pin(uint32_t chunkId)
    {
        if (chunkId < chunks.size()) {
            chunks[chunkId].pinned++;
        }
    }

    // Every block that is not in a chunk with pinned blocks becomes invalid.  One unpinned chunk is kept
    // for reuse; chunks with pinned blocks are sealed.  Chunk ids handed out before are void afterwards,
    // except that a pinned chunk's memory does not move.
    void Reset()
    {
        std::vector<Chunk> keep;
        bool spare = false;
        for (Chunk &c : chunks) {
            if (c.pinned > 0) {
                c.sealed = true;
                keep.push_back(c);
            } else if (!spare) {
                c.used = 0;
                spare = true;
                keep.push_back(c);
            } else {
                freeFn(c.base);
            }
        }
        // the reusable chunk goes last: Alloc only looks at the last chunk
        for (size_t i = 0; i + 1 < keep.size(); i++) {
            if (!keep[i].sealed) {
                Chunk t = keep[i];
                keep.erase(keep.begin() + long(i));
                keep.push_back(t);
                break;
            }
        }
        chunks.swap(keep);
    }

    void FreeAll()
    {
        for (Chunk &c : chunks) {
            freeFn(c.base);
        }
        chunks.clear();
    }

    size_t PinnedChunks() const
    {
        size_t n = 0;
        for (const Chunk &c : chunks) {
            n += c.pinned > 0 ? 1 : 0;
        }
        return n;
    }
};

}  // namespace hcclamd

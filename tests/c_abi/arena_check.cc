// Host-only check of the table arena's pinning rules (cann-hccl_amd/csrc/arena.h), compiled and run by
// tests/test_api_cpu.py: blocks of collectives recorded into a caller's graph must survive Reset().
#include <cstdio>
#include <cstdlib>
#include <set>

#include "arena.h"

static std::set<void *> live;
static void *TestAlloc(size_t n)
{
    void *p = std::malloc(n);
    live.insert(p);
    return p;
}
static void TestFree(void *p)
{
    if (live.erase(p) != 1) {
        std::printf("FAIL double or foreign free\n");
        std::exit(1);
    }
    std::free(p);
}
#define CHECK(c)                                              \
    do {                                                      \
        if (!(c)) {                                           \
            std::printf("FAIL line %d: %s\n", __LINE__, #c);  \
            return 1;                                         \
        }                                                     \
    } while (0)

int main()
{
    hcclamd::TableArena a;
    a.allocFn = TestAlloc;
    a.freeFn = TestFree;
    a.chunkBytes = 4096;
    uint32_t c0 = 99, c1 = 99, c2 = 99;
    char *b0 = static_cast<char *>(a.Alloc(1000, &c0));    // 1024 bytes of chunk 0
    char *b1 = static_cast<char *>(a.Alloc(3000, &c1));    // 3072 bytes: fills chunk 0
    char *b2 = static_cast<char *>(a.Alloc(100, &c2));     // chunk 1
    CHECK(b0 && b1 && b2 && c0 == 0 && c1 == 0 && c2 == 1 && b1 == b0 + 1024 && a.chunks.size() == 2);
    b0[0] = 'x';
    a.Pin(c0);                                             // b0 was recorded into a caller's graph
    a.Reset();
    // chunk 0 survives untouched and takes no more blocks; chunk 1 is reused from its start
    CHECK(a.chunks.size() == 2 && a.PinnedChunks() == 1 && live.size() == 2 && b0[0] == 'x');
    uint32_t c3 = 99;
    char *b3 = static_cast<char *>(a.Alloc(100, &c3));
    CHECK(b3 == b2 && (b3 < b0 || b3 >= b0 + 4096));
    // a second Reset without new pins: the pinned chunk stays, the spare chunk is kept, nothing leaks
    for (int i = 0; i < 50; i++) {
        CHECK(a.Alloc(2000, nullptr) != nullptr);
    }
    a.Reset();
    CHECK(a.chunks.size() == 2 && live.size() == 2 && b0[0] == 'x');
    // pin something in the spare chunk too: both stay, the next block comes from a fresh chunk
    uint32_t c4 = 99;
    char *b4 = static_cast<char *>(a.Alloc(64, &c4));
    a.Pin(c4);
    a.Reset();
    CHECK(a.PinnedChunks() == 2 && live.size() == 2);
    char *b5 = static_cast<char *>(a.Alloc(64, nullptr));
    CHECK(b5 != nullptr && b5 != b4 && live.size() == 3);
    // an arena without pins resets to one empty chunk
    hcclamd::TableArena plain;
    plain.allocFn = TestAlloc;
    plain.freeFn = TestFree;
    plain.chunkBytes = 4096;
    for (int i = 0; i < 10; i++) {
        CHECK(plain.Alloc(4000, nullptr) != nullptr);
    }
    CHECK(plain.chunks.size() == 10);
    plain.Reset();
    CHECK(plain.chunks.size() == 1 && plain.chunks[0].used == 0);
    plain.FreeAll();
    a.FreeAll();
    CHECK(live.empty());
    std::printf("OK\n");
    return 0;
}

// Host-only check of the repack cache's bookkeeping (ternainfer_amd/csrc/repack_cache.h): compiled with g++ and run by
// tests/test_repack_cache_policy.py.  Device memory is stood in for by malloc; `released` records what the policy let go.
#include <cstdio>
#include <cstdlib>
#include <set>

#include "../ternainfer_amd/csrc/repack_cache.h"

using namespace terna;

static std::set<void*> live;
static int releases = 0;
static void release(void* p)
{
    if (!live.count(p)) { std::printf("FAIL: released twice or never allocated\n"); std::exit(1); }
    live.erase(p);
    std::free(p);
    ++releases;
}
static void* alloc(size_t n)
{
    void* p = std::malloc(n);
    live.insert(p);
    return p;
}
#define CHECK(cond) do { if (!(cond)) { std::printf("FAIL line %d: %s\n", __LINE__, #cond); return 1; } } while (0)

struct Payload { int tag; };
static RepackKey key(int j, int n = 256, int k = 128) { return RepackKey{0, reinterpret_cast<void*>(0x1000 + 16 * j), reinterpret_cast<void*>(0x2000 + 16 * j), reinterpret_cast<void*>(0x3000 + 16 * j), n, k}; }

int main()
{
    using Cache = RepackCachePolicy<Payload>;
    Cache c(release, 300);

    // identity: device, three pointers and the shape all take part
    CHECK(c.find(key(0)) == nullptr);
    CHECK(c.make_room(100));
    Cache::Slot* s0 = c.insert(key(0), alloc(100), 100, Payload{10});
    CHECK(s0->id == 1 && c.next_id() == 2 && c.used() == 100 && c.entries() == 1);
    CHECK(c.find(key(0)) != nullptr && c.find(key(0))->payload.tag == 10);
    CHECK(c.find(key(0, 256, 192)) == nullptr);
    RepackKey other_device = key(0);
    other_device.device = 1;
    CHECK(c.find(other_device) == nullptr);

    // least recently used goes first; a find() refreshes
    c.insert(key(1), alloc(100), 100, Payload{11});
    c.insert(key(2), alloc(100), 100, Payload{12});
    CHECK(c.used() == 300 && releases == 0);
    CHECK(c.find(key(0)) != nullptr);                 // 0 is now the most recent; 1 the least
    CHECK(c.make_room(100));
    CHECK(releases == 1 && c.find(key(1)) == nullptr && c.find(key(0)) != nullptr && c.find(key(2)) != nullptr);
    c.insert(key(3), alloc(100), 100, Payload{13});
    CHECK(c.used() == 300 && c.evicted() == 1);

    // a copy larger than the limit is refused and nothing is released for it
    CHECK(!c.make_room(301) && releases == 1 && c.entries() == 3);

    // pinned copies (a captured graph holds their address) never go to make room
    c.find(key(0))->pinned = true;
    c.find(key(2))->pinned = true;
    c.find(key(3));                                   // 3 most recent, unpinned; 0 and 2 pinned
    CHECK(c.make_room(100));                          // only 3 can go
    CHECK(c.find(key(3)) == nullptr && c.find(key(0)) && c.find(key(2)) && releases == 2);
    CHECK(!c.make_room(200) && c.entries() == 2 && releases == 2);     // what remains is pinned: refused, nothing released

    // a stale unpinned copy is released; a stale pinned copy is parked until clear()
    Cache::Slot* s4 = c.insert(key(4), alloc(100), 100, Payload{14});
    const uint32_t id4 = s4->id, id0 = c.find(key(0))->id;
    CHECK(c.retire(id4) && releases == 3 && c.find(key(4)) == nullptr);
    CHECK(!c.retire(id4));                            // already gone
    CHECK(c.retire(id0) && releases == 3 && c.find(key(0)) == nullptr && c.parked_bytes() == 100 && c.used() == 100);
    CHECK(c.retired() == 2);
    // the same weight gets a fresh copy with a new id while the parked one still exists
    CHECK(c.make_room(100));
    Cache::Slot* again = c.insert(key(0), alloc(100), 100, Payload{20});
    CHECK(again->id != id0 && c.find(key(0))->payload.tag == 20);

    // lowering the limit takes effect at the next make_room
    c.set_limit(100);
    CHECK(c.used() == 200);
    CHECK(!c.make_room(100));                         // key(2) is pinned (100 bytes): no room for another 100
    c.find(key(2))->pinned = false;
    CHECK(c.make_room(100) && c.used() == 0);

    c.insert(key(5), alloc(50), 50, Payload{15});
    c.clear();
    CHECK(live.empty() && c.used() == 0 && c.entries() == 0 && c.parked_bytes() == 0);

    // workspace sizes: what the reference itself writes (decode: SPLIT_K planes of M x N int32; prefill: dense int8 N x K)
    CHECK(reference_workspace_bytes(false, 8, 2560, 2560, 7) == 4u * 8 * 2560 * 7);
    CHECK(reference_workspace_bytes(true, 256, 2560, 6912, 7) == 2560u * 6912);
    CHECK(reference_workspace_bytes(false, 8, 2560, 2560, 0) == 0);
    std::printf("repack cache policy ok\n");
    return 0;
}

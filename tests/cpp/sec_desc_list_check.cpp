// The agent's sorted list of registered regions against the orderings the reference's own
// unit tests expect of its nixlSecDescList (test/gtest/unit/descriptors/sec_desc_list.cpp:
// 86-213: batches appended, prepended, interleaved, unsorted, duplicated, with several device
// ids, and 4096 random descriptors in random batches), plus the covering-region search the
// agent builds on it (src/infra/nixl_memory_section.cpp:56-104).  Host only.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <utility>
#include <vector>

#include "agent_impl.h"

#define REQUIRE(cond)                                                              \
    do {                                                                           \
        if (!(cond)) {                                                             \
            std::fprintf(stderr, "%s:%d: %s failed\n", __FILE__, __LINE__, #cond); \
            std::exit(1);                                                          \
        }                                                                          \
    } while (0)

namespace {

constexpr size_t kLen = 64;

nixlSectionDesc
desc(uintptr_t addr, uint64_t dev = 0, size_t len = kLen) {
    return nixlSectionDesc(addr, len, dev);
}

bool
sorted(const nixlSecDescList &l) {
    for (size_t i = 1; i < l.size(); ++i)
        if (l[i] < l[i - 1]) return false;
    return true;
}

// expected = {addr, devId} in list order
void
expect(const nixlSecDescList &l, const std::vector<std::pair<uintptr_t, uint64_t>> &expected) {
    REQUIRE(l.size() == expected.size());
    REQUIRE(sorted(l));
    for (size_t i = 0; i < expected.size(); ++i)
        REQUIRE(l[i].addr == expected[i].first && l[i].devId == expected[i].second && l[i].len == kLen);
}

nixlSecDescList
make(std::initializer_list<uintptr_t> addrs) {
    nixlSecDescList l;
    std::vector<nixlSectionDesc> batch;
    for (auto a : addrs)
        batch.push_back(desc(a));
    l.add(std::move(batch));
    return l;
}

} // namespace

int
main() {
    {
        nixlSecDescList l;
        l.add({});
        REQUIRE(l.empty());
        l = make({20, 40});
        l.add({});
        expect(l, {{20, 0}, {40, 0}});
        l.add({desc(10)});
        l.add({desc(30)});
        l.add({desc(50)});
        expect(l, {{10, 0}, {20, 0}, {30, 0}, {40, 0}, {50, 0}});
    }
    {
        auto l = make({10, 20});
        l.add({desc(30), desc(40)}); // all after
        expect(l, {{10, 0}, {20, 0}, {30, 0}, {40, 0}});
        l = make({30, 40});
        l.add({desc(10), desc(20)}); // all before
        expect(l, {{10, 0}, {20, 0}, {30, 0}, {40, 0}});
        l = make({10, 30, 50});
        l.add({desc(20), desc(40)}); // interleaved
        expect(l, {{10, 0}, {20, 0}, {30, 0}, {40, 0}, {50, 0}});
        expect(make({40, 10, 30, 20}), {{10, 0}, {20, 0}, {30, 0}, {40, 0}});
        l = make({10, 20});
        l.add({desc(10), desc(20)}); // duplicates are kept
        expect(l, {{10, 0}, {10, 0}, {20, 0}, {20, 0}});
    }
    {
        nixlSecDescList l;
        l.add({desc(50, 1)});
        l.add({desc(100, 1), desc(10, 2)});
        expect(l, {{50, 1}, {100, 1}, {10, 2}});
        l.add({desc(10, 1), desc(50, 0)});
        expect(l, {{50, 0}, {10, 1}, {50, 1}, {100, 1}, {10, 2}});
        l.add({desc(10, 0), desc(75, 1), desc(200, 1), desc(20, 2)});
        expect(l, {{10, 0}, {50, 0}, {10, 1}, {50, 1}, {75, 1}, {100, 1}, {200, 1}, {10, 2}, {20, 2}});
        // covering search: inside, at the edges, across a gap, on another device
        REQUIRE(l.coveringIndex(nixlBasicDesc(75, 64, 1)) == 4);
        REQUIRE(l.coveringIndex(nixlBasicDesc(80, 16, 1)) == 4);
        REQUIRE(l.coveringIndex(nixlBasicDesc(80, 64, 1)) == -1); // runs past the region's end
        REQUIRE(l.coveringIndex(nixlBasicDesc(74, 8, 1)) == 3);   // still inside [50, 114)
        REQUIRE(l.coveringIndex(nixlBasicDesc(170, 8, 1)) == -1);
        REQUIRE(l.coveringIndex(nixlBasicDesc(75, 8, 3)) == -1);
        REQUIRE(l.indexOf(nixlBasicDesc(200, 64, 1)) == 6 && l.indexOf(nixlBasicDesc(200, 32, 1)) == -1);
        l.removeAt({0, 4, 8});
        expect(l, {{50, 0}, {10, 1}, {50, 1}, {100, 1}, {200, 1}, {10, 2}});
    }
    {
        nixlSecDescList l;
        std::mt19937 rng(42);
        std::uniform_int_distribution<uintptr_t> addr(1, 1000000);
        std::uniform_int_distribution<uint64_t> dev(0, 8);
        std::uniform_int_distribution<size_t> len(1, 64), batch_size(1, 256);
        size_t added = 0;
        while (added < 4096) {
            const size_t n = std::min(batch_size(rng), 4096 - added);
            std::vector<nixlSectionDesc> batch;
            for (size_t j = 0; j < n; ++j)
                batch.push_back(desc(addr(rng), dev(rng), len(rng)));
            l.add(std::move(batch));
            added += n;
            REQUIRE(l.size() == added && sorted(l));
        }
    }
    std::puts("OK");
    return 0;
}

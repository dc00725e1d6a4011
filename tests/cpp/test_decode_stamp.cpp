// Host-side check of the launch stamps of the decode kernel's exchange lines (csrc/glm_attn_internal.h):
// a stamp is never 0 (what a zero-filled exchange buffer holds), the launch count skips the value whose
// stamp would be, stamps of nearby launches differ, and the stamps of the static exchange memory keep the
// KV groups apart.  Built and run by tests/test_capi_cpu.py; no GPU.
#include <stdio.h>

#include <set>

#include "glm_attn_internal.h"

using namespace glm_attn;

#define CHECK(cond)                                                  \
    do {                                                             \
        if (!(cond)) {                                               \
            printf("FAILED line %d: %s\n", __LINE__, #cond);         \
            return 1;                                                \
        }                                                            \
    } while (0)

int main() {
    CHECK(decode_stamp(0) == 1u);
    // around the wrap of the 32-bit stamp: the count that would stamp 0 is never reached
    unsigned long long gen = 0xfffffffaull;
    std::set<unsigned int> seen;
    for (int i = 0; i < 16; i++) {
        CHECK(decode_stamp(gen) != 0u);
        CHECK(seen.insert(decode_stamp(gen)).second);
        const unsigned long long next = decode_next_gen(gen);
        CHECK(next > gen && next <= gen + 2);
        gen = next;
    }
    CHECK(gen > 0x100000000ull);
    // a long plain run: consecutive launches never share a stamp
    gen = 12345;
    unsigned int prev = decode_stamp(gen);
    for (int i = 0; i < 100000; i++) {
        gen = decode_next_gen(gen);
        CHECK(decode_stamp(gen) != 0u && decode_stamp(gen) != prev);
        prev = decode_stamp(gen);
    }
    // grouped stamps: never 0, the group in the upper 5 bits, 2^27 - 1 launches before a repeat
    for (int g = 0; g < 32; g++) {
        for (unsigned long long n : {0ull, 1ull, 0x7fffffeull, 0x7ffffffull, 0x8000000ull, 0xffffffffull, 0x123456789abull}) {
            const unsigned int s = decode_stamp_grouped(n, g);
            CHECK(s != 0u);
            CHECK((s >> 27) == (unsigned int)g);
            CHECK((s & 0x7ffffffu) != 0u);
        }
        CHECK(decode_stamp_grouped(5, g) != decode_stamp_grouped(6, g));
        CHECK(decode_stamp_grouped(0, g) == decode_stamp_grouped(0x7ffffffull, g));  // the period
        for (int g2 = 0; g2 < 32; g2++) {
            CHECK(g == g2 || decode_stamp_grouped(77, g) != decode_stamp_grouped(77, g2));
        }
    }
    printf("ok\n");
    return 0;
}

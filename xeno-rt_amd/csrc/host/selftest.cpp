// Self-test of the host library, meant to be built and run under the host's address and undefined-behaviour
// sanitizers: a few thousand random operations on pools and block tables against what they must keep true,
// and the packing of steps against arrays worked out by hand. Prints "host selftest ok" and exits with 0.
#include "xrt_host.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#define REQUIRE(condition)                                                                  \
    do {                                                                                    \
        if (!(condition)) {                                                                 \
            std::fprintf(stderr, "host selftest: line %d: %s failed (%s)\n", __LINE__, #condition, xrt_host_last_error()); \
            return 1;                                                                       \
        }                                                                                   \
    } while (0)

static unsigned long long state = 88172645463325252ULL;
static int draw(int below) {                       // xorshift: the same sequence everywhere
    state ^= state << 13; state ^= state >> 7; state ^= state << 17;
    return (int)(state % (unsigned long long)below);
}

int main() {
    {   // a pool hands out the lowest free item, refuses a second release, and says when it is empty
        xrt_pool* pool = xrt_pool_new(5, "slot");
        int item = -1;
        for (int want = 0; want < 5; ++want) { REQUIRE(xrt_pool_acquire(pool, &item) == XRT_HOST_OK && item == want); }
        REQUIRE(xrt_pool_acquire(pool, &item) == XRT_HOST_FULL);
        REQUIRE(xrt_pool_release(pool, 3) == XRT_HOST_OK && xrt_pool_release(pool, 1) == XRT_HOST_OK);
        REQUIRE(xrt_pool_release(pool, 3) == XRT_HOST_ERROR && xrt_pool_release(pool, 7) == XRT_HOST_ERROR);
        REQUIRE(xrt_pool_acquire(pool, &item) == XRT_HOST_OK && item == 1);
        REQUIRE(xrt_pool_n_free(pool) == 1 && xrt_pool_is_held(pool, 1) && !xrt_pool_is_held(pool, 3) && xrt_pool_check(pool) == XRT_HOST_OK);
        xrt_pool_delete(pool);
    }
    for (int window : {0, 100, 64, 1}) {   // block tables: sequences that grow, roll back and end, with and without a window
        const int n_blocks = 24, max_slots = 6, max_blocks = 10, block_tokens = 64;
        std::vector<int32_t> table((size_t)max_slots * max_blocks, -1);
        xrt_tables* tables = xrt_tables_new(n_blocks, max_slots, max_blocks, window, block_tokens, table.data());
        REQUIRE(tables != nullptr);
        std::vector<int> length((size_t)max_slots, -1);         // -1: the slot is free
        std::vector<int> added((size_t)max_blocks);
        for (int round = 0; round < 4000; ++round) {
            const int slot = draw(max_slots);
            if (length[(size_t)slot] < 0) { length[(size_t)slot] = 0; continue; }
            const int what = draw(10);
            int status = XRT_HOST_OK;
            if (what < 6) {                                       // a step: reserve, then commit or cancel
                const int longer = length[(size_t)slot] + 1 + draw(150);
                int n_added = 0;
                status = xrt_tables_grow(tables, slot, longer, added.data(), &n_added);
                if (longer > max_blocks * block_tokens) { REQUIRE(status == XRT_HOST_ERROR); }
                else if (status == XRT_HOST_OK) {
                    if (draw(4) > 0) length[(size_t)slot] = longer;
                    REQUIRE(xrt_tables_shrink_to(tables, slot, length[(size_t)slot]) == XRT_HOST_OK);
                } else {
                    REQUIRE(status == XRT_HOST_FULL);
                }
            } else if (what < 8 && window == 0) {                 // a rollback
                length[(size_t)slot] = draw(length[(size_t)slot] + 1);
                REQUIRE(xrt_tables_shrink_to(tables, slot, length[(size_t)slot]) == XRT_HOST_OK);
            } else if (what == 9) {                               // the sequence ends
                REQUIRE(xrt_tables_release_all(tables, slot) == XRT_HOST_OK);
                length[(size_t)slot] = -1;
            }
            // what every sequence holds: exactly the blocks between its window's floor and its end
            std::vector<unsigned char> held((size_t)max_slots);
            int in_use = 0;
            for (int s = 0; s < max_slots; ++s) {
                held[(size_t)s] = length[(size_t)s] >= 0;
                const int tokens = length[(size_t)s] < 0 ? 0 : length[(size_t)s];
                const int end = (tokens + block_tokens - 1) / block_tokens;
                for (int logical = 0; logical < max_blocks; ++logical) {
                    const bool has = table[(size_t)s * max_blocks + (size_t)logical] >= 0;
                    const bool must = logical < end && logical >= xrt_tables_floor(tables, s);
                    REQUIRE(has == must);
                    in_use += has;
                }
                if (window == 0) { REQUIRE(xrt_tables_floor(tables, s) == 0); }
            }
            REQUIRE(in_use == n_blocks - xrt_pool_n_free(xrt_tables_pool(tables)));
            REQUIRE(xrt_tables_check(tables, held.data()) == XRT_HOST_OK);
        }
        int low = 0, high = 0;
        xrt_tables_take_changed(tables, &low, &high);
        REQUIRE(low >= 0 && high <= max_slots && low < high);
        xrt_tables_take_changed(tables, &low, &high);
        REQUIRE(low == high);
        xrt_tables_delete(tables);
    }
    {   // a step of three sequences, padded to eight tokens
        const int slots[] = {4, 0, 2}, counts[] = {3, 1, 2}, starts[] = {10, 0, 63};
        const int tokens[] = {7, 8, 9, 5, 1, 2}, want_counts[] = {2, 0, 1}, wants[] = {0, 2, 1};
        REQUIRE(xrt_step_check(3, slots, counts, starts, tokens, want_counts, wants, 10, 65) == XRT_HOST_OK);
        REQUIRE(xrt_step_check(3, slots, counts, starts, tokens, want_counts, wants, 9, 65) == XRT_HOST_ERROR);       // token 9
        REQUIRE(xrt_step_check(3, slots, counts, starts, tokens, want_counts, wants, 10, 64) == XRT_HOST_ERROR);      // 63 + 2 tokens
        const long room = xrt_step_room(3, 6, 3, 8);
        REQUIRE(room == 3 * 8 + 3 * 3 + 1 + 3);
        std::vector<int32_t> out((size_t)room, 777);
        xrt_step_facts facts;
        REQUIRE(xrt_step_pack(3, slots, counts, starts, tokens, want_counts, wants, 8, out.data(), room - 1, &facts) == XRT_HOST_ERROR);
        REQUIRE(xrt_step_pack(3, slots, counts, starts, tokens, want_counts, wants, 8, out.data(), room, &facts) == XRT_HOST_OK);
        const int32_t want_out[] = {7, 8, 9, 5, 1, 2, 0, 0,   10, 11, 12, 0, 63, 64, 0, 0,   4, 4, 4, 0, 2, 2, -1, -1,
                                    4, 0, 2,   0, 3, 4, 6,   10, 0, 63,   0, 2, 5};
        REQUIRE(std::memcmp(out.data(), want_out, sizeof want_out) == 0);
        REQUIRE(facts.n_tokens == 8 && facts.n_rows == 3 && facts.max_count == 3 && facts.max_context == 65 && !facts.is_decode);
    }
    {   // the loop's decisions, in the reference's order, and batches that fit
        const int stops[] = {2, 5};
        int keep = -1;
        REQUIRE(xrt_loop_decide(5, stops, 2, 100, 100, 0, 1, &keep) == XRT_FINISH_STOP && keep == 0);        // a stop token wins over everything
        REQUIRE(xrt_loop_decide(7, stops, 2, 100, 100, 0, 9, &keep) == XRT_FINISH_CONTEXT && keep == 0);
        REQUIRE(xrt_loop_decide(7, stops, 2, 99, 100, 8, 9, &keep) == XRT_FINISH_LENGTH && keep == 1);
        REQUIRE(xrt_loop_decide(7, stops, 2, 99, 100, 7, 9, &keep) == XRT_GOES_ON && keep == 1);
        REQUIRE(xrt_loop_goes_on_whatever_it_draws(98, 100, 7, 9) && !xrt_loop_goes_on_whatever_it_draws(99, 100, 7, 9) &&
                !xrt_loop_goes_on_whatever_it_draws(98, 100, 8, 9));
        const int prompts[] = {60, 5, 130, 1, 64}, limits[] = {10, 200, 0, 1, 1};
        int batch_of[5];
        REQUIRE(xrt_loop_plan_batches(5, prompts, limits, 2, 64, 320, 128, batch_of) == 3);     // 128, 128, 128 (the context), 64, 128 tokens
        const int want_batches[] = {0, 0, 1, 1, 2};
        REQUIRE(std::memcmp(batch_of, want_batches, sizeof want_batches) == 0);
        REQUIRE(xrt_loop_plan_batches(5, prompts, limits, 8, 64, 100, 128, batch_of) == -1);
    }
    std::printf("host selftest ok\n");
    return 0;
}

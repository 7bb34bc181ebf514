// The host library: see xrt_host.h. Plain C++17, no GPU.
#include "xrt_host.h"

#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <functional>
#include <queue>
#include <string>
#include <unordered_set>
#include <vector>

namespace {

thread_local std::string last_error;

int fail(int code, const char* format, ...) {
    char text[512];
    va_list arguments;
    va_start(arguments, format);
    vsnprintf(text, sizeof text, format, arguments);
    va_end(arguments);
    last_error = text;
    return code;
}

}  // namespace

extern "C" const char* xrt_host_last_error(void) { return last_error.c_str(); }

// ---- pools --------------------------------------------------------------------------------------

struct xrt_pool {
    int size;
    std::string what;
    std::priority_queue<int, std::vector<int>, std::greater<int>> free_items;    // the lowest number on top
    std::vector<unsigned char> held;
};

extern "C" xrt_pool* xrt_pool_new(int size, const char* what) {
    if (size < 0) {
        fail(XRT_HOST_ERROR, "pool of %ss needs a non-negative size", what ? what : "item");
        return nullptr;
    }
    xrt_pool* pool = new xrt_pool{size, what ? what : "item", {}, std::vector<unsigned char>((size_t)size, 0)};
    for (int item = 0; item < size; ++item) pool->free_items.push(item);
    return pool;
}

extern "C" void xrt_pool_delete(xrt_pool* pool) { delete pool; }

extern "C" int xrt_pool_acquire(xrt_pool* pool, int* item) {
    if (pool->free_items.empty())
        return fail(XRT_HOST_FULL, "no free %s (all %d are in use)", pool->what.c_str(), pool->size);
    const int taken = pool->free_items.top();
    if (pool->held[(size_t)taken]) return fail(XRT_HOST_ERROR, "%s %d was on the free list while held", pool->what.c_str(), taken);
    pool->free_items.pop();
    pool->held[(size_t)taken] = 1;
    *item = taken;
    return XRT_HOST_OK;
}

extern "C" int xrt_pool_release(xrt_pool* pool, int item) {
    if (item < 0 || item >= pool->size)
        return fail(XRT_HOST_ERROR, "%s %d does not exist (pool of %d)", pool->what.c_str(), item, pool->size);
    if (!pool->held[(size_t)item])
        return fail(XRT_HOST_ERROR, "%s %d is released twice or was never acquired", pool->what.c_str(), item);
    pool->held[(size_t)item] = 0;
    pool->free_items.push(item);
    return XRT_HOST_OK;
}

extern "C" int xrt_pool_size(const xrt_pool* pool) { return pool->size; }
extern "C" int xrt_pool_n_free(const xrt_pool* pool) { return (int)pool->free_items.size(); }
extern "C" int xrt_pool_is_held(const xrt_pool* pool, int item) { return item >= 0 && item < pool->size && pool->held[(size_t)item]; }

extern "C" int xrt_pool_check(const xrt_pool* pool) {
    auto copy = pool->free_items;
    std::vector<unsigned char> is_free((size_t)pool->size, 0);
    while (!copy.empty()) {
        const int item = copy.top();
        copy.pop();
        if (item < 0 || item >= pool->size) return fail(XRT_HOST_ERROR, "%s %d on the free list does not exist", pool->what.c_str(), item);
        if (is_free[(size_t)item]) return fail(XRT_HOST_ERROR, "a %s is on the free list twice", pool->what.c_str());
        is_free[(size_t)item] = 1;
    }
    for (int item = 0; item < pool->size; ++item)
        if ((pool->held[(size_t)item] != 0) == (is_free[(size_t)item] != 0))
            return fail(XRT_HOST_ERROR, "%s %d is %s", pool->what.c_str(), item, pool->held[(size_t)item] ? "both held and free" : "lost");
    return XRT_HOST_OK;
}

// ---- block tables ---------------------------------------------------------------------------------

struct xrt_tables {
    int max_slots, max_blocks, window, block_tokens;
    int32_t* table;                      // the caller's
    xrt_pool* pool;
    std::vector<int> end, floor;         // per slot: logical blocks [floor, end) may be held
    int changed_low, changed_high;       // rows the caller has not seen yet: [low, high)
    int32_t& at(int slot, int logical) { return table[(size_t)slot * (size_t)max_blocks + (size_t)logical]; }
    int32_t at(int slot, int logical) const { return table[(size_t)slot * (size_t)max_blocks + (size_t)logical]; }
    void touch(int slot) {
        if (changed_low == changed_high) { changed_low = slot; changed_high = slot + 1; }
        else { changed_low = std::min(changed_low, slot); changed_high = std::max(changed_high, slot + 1); }
    }
    int blocks_for(int tokens) const { return (tokens + block_tokens - 1) / block_tokens; }
};

namespace {

int require_slot(const xrt_tables* tables, int slot) {
    if (slot < 0 || slot >= tables->max_slots) return fail(XRT_HOST_ERROR, "slot %d does not exist (%d slots)", slot, tables->max_slots);
    return XRT_HOST_OK;
}

int drop(xrt_tables* tables, int slot, const int* logicals, int n) {
    for (int i = 0; i < n; ++i) {
        const int logical = logicals[i];
        if (logical < 0 || logical >= tables->max_blocks) return fail(XRT_HOST_ERROR, "slot %d has no logical block %d", slot, logical);
        const int status = xrt_pool_release(tables->pool, tables->at(slot, logical));
        if (status != XRT_HOST_OK) return status;
        tables->at(slot, logical) = -1;
    }
    if (n > 0) {
        tables->touch(slot);
        int end = tables->end[(size_t)slot];
        while (end > 0 && tables->at(slot, end - 1) < 0) --end;
        tables->end[(size_t)slot] = end;
    }
    return XRT_HOST_OK;
}

}  // namespace

extern "C" xrt_tables* xrt_tables_new(int n_blocks, int max_slots, int max_blocks, int window, int block_tokens, int32_t* table) {
    if (n_blocks < 0 || max_slots <= 0 || max_blocks <= 0 || window < 0 || block_tokens <= 0 || table == nullptr) {
        fail(XRT_HOST_ERROR, "block tables: bad sizes (%d blocks, %d slots, %d blocks a sequence, window %d, %d tokens a block)",
             n_blocks, max_slots, max_blocks, window, block_tokens);
        return nullptr;
    }
    xrt_pool* pool = xrt_pool_new(n_blocks, "block");
    if (pool == nullptr) return nullptr;
    return new xrt_tables{max_slots, max_blocks, window, block_tokens, table, pool,
                          std::vector<int>((size_t)max_slots, 0), std::vector<int>((size_t)max_slots, 0), 0, 0};
}

extern "C" void xrt_tables_delete(xrt_tables* tables) {
    if (tables == nullptr) return;
    xrt_pool_delete(tables->pool);
    delete tables;
}

extern "C" xrt_pool* xrt_tables_pool(xrt_tables* tables) { return tables->pool; }

extern "C" int xrt_tables_first_needed_block(const xrt_tables* tables, int length) {
    if (tables->window == 0) return 0;
    return std::max(0, length + 1 - tables->window) / tables->block_tokens;
}

extern "C" int xrt_tables_floor(const xrt_tables* tables, int slot) {
    return slot >= 0 && slot < tables->max_slots ? tables->floor[(size_t)slot] : 0;
}

extern "C" int xrt_tables_grow(xrt_tables* tables, int slot, int new_length, int* added, int* n_added) {
    *n_added = 0;
    if (require_slot(tables, slot) != XRT_HOST_OK) return XRT_HOST_ERROR;
    const int need = tables->blocks_for(new_length);
    if (need > tables->max_blocks)
        return fail(XRT_HOST_ERROR, "sequence of %d tokens exceeds the cache's limit per sequence", new_length);
    const int start = std::max(tables->end[(size_t)slot], tables->floor[(size_t)slot]);
    int count = 0;
    for (int logical = start; logical < need; ++logical) {
        int block = -1;
        const int status = xrt_pool_acquire(tables->pool, &block);
        if (status != XRT_HOST_OK) {                           // nothing is kept of a growth that does not fit
            const std::string why = last_error;
            drop(tables, slot, added, count);
            last_error = why;
            return status;
        }
        tables->at(slot, logical) = block;
        added[count++] = logical;
    }
    if (count > 0) {
        tables->end[(size_t)slot] = need;
        tables->touch(slot);
    }
    *n_added = count;
    return XRT_HOST_OK;
}

extern "C" int xrt_tables_drop(xrt_tables* tables, int slot, const int* logicals, int n) {
    if (require_slot(tables, slot) != XRT_HOST_OK) return XRT_HOST_ERROR;
    return drop(tables, slot, logicals, n);
}

extern "C" int xrt_tables_shrink_to(xrt_tables* tables, int slot, int length) {
    if (require_slot(tables, slot) != XRT_HOST_OK) return XRT_HOST_ERROR;
    const int end = tables->end[(size_t)slot];
    std::vector<int> gone;
    for (int logical = tables->blocks_for(length); logical < end; ++logical)
        if (tables->at(slot, logical) >= 0) gone.push_back(logical);
    const int floor = xrt_tables_first_needed_block(tables, length);
    for (int logical = tables->floor[(size_t)slot]; logical < std::min(floor, end); ++logical)
        if (tables->at(slot, logical) >= 0) gone.push_back(logical);
    tables->floor[(size_t)slot] = floor;
    return drop(tables, slot, gone.data(), (int)gone.size());
}

extern "C" int xrt_tables_release_all(xrt_tables* tables, int slot) {
    if (require_slot(tables, slot) != XRT_HOST_OK) return XRT_HOST_ERROR;
    std::vector<int> gone;
    for (int logical = 0; logical < tables->end[(size_t)slot]; ++logical)
        if (tables->at(slot, logical) >= 0) gone.push_back(logical);
    const int status = drop(tables, slot, gone.data(), (int)gone.size());
    tables->floor[(size_t)slot] = 0;
    tables->end[(size_t)slot] = 0;
    return status;
}

extern "C" void xrt_tables_take_changed(xrt_tables* tables, int* low, int* high) {
    *low = tables->changed_low;
    *high = tables->changed_high;
    tables->changed_low = tables->changed_high = 0;
}

extern "C" int xrt_tables_check(const xrt_tables* tables, const unsigned char* slot_held) {
    if (xrt_pool_check(tables->pool) != XRT_HOST_OK) return XRT_HOST_ERROR;
    std::vector<unsigned char> seen((size_t)tables->pool->size, 0);
    int n_seen = 0;
    for (int slot = 0; slot < tables->max_slots; ++slot)
        for (int logical = 0; logical < tables->max_blocks; ++logical) {
            const int block = tables->at(slot, logical);
            if (block < 0) continue;
            if (!slot_held[slot]) return fail(XRT_HOST_ERROR, "free slot %d still holds block %d", slot, block);
            if (block >= tables->pool->size) return fail(XRT_HOST_ERROR, "slot %d names block %d, which does not exist", slot, block);
            if (seen[(size_t)block]) return fail(XRT_HOST_ERROR, "block %d is held by two sequences", block);
            if (!xrt_pool_is_held(tables->pool, block)) return fail(XRT_HOST_ERROR, "block %d is in a table but free in the pool", block);
            seen[(size_t)block] = 1;
            ++n_seen;
        }
    const int held = tables->pool->size - xrt_pool_n_free(tables->pool);
    if (n_seen != held) return fail(XRT_HOST_ERROR, "%d blocks are held by no sequence", held - n_seen);
    return XRT_HOST_OK;
}

// ---- a step -----------------------------------------------------------------------------------------

extern "C" long xrt_step_room(int n_sequences, long n_tokens, long n_wants, int pad_to) {
    const long padded = std::max(n_tokens, (long)pad_to);
    return 3 * padded + 3L * n_sequences + 1 + n_wants;
}

extern "C" int xrt_step_check(int n_sequences, const int* slots, const int* counts, const int* starts, const int* tokens,
                              const int* want_counts, const int* wants, int vocab, int max_context) {
    if (n_sequences <= 0) return fail(XRT_HOST_ERROR, "a step needs at least one sequence");
    std::unordered_set<int> seen;
    long token_at = 0, want_at = 0;
    for (int i = 0; i < n_sequences; ++i) {
        const int slot = slots[i], count = counts[i];
        if (!seen.insert(slot).second) return fail(XRT_HOST_ERROR, "slot %d appears twice in one step", slot);
        if (count <= 0) return fail(XRT_HOST_ERROR, "slot %d: a step needs at least one token per sequence", slot);      // llama.rs:624-626
        for (int t = 0; t < count; ++t) {                                                                                 // llama.rs:1044-1049
            const int token = tokens[token_at + t];
            if (token < 0 || token >= vocab) return fail(XRT_HOST_ERROR, "slot %d: token id %d exceeds embedding rows %d", slot, token, vocab);
        }
        for (int w = 0; w < want_counts[i]; ++w) {
            const int index = wants[want_at + w];
            if (index < 0 || index >= count)
                return fail(XRT_HOST_ERROR, "slot %d: wanted index %d is outside the %d tokens given", slot, index, count);
        }
        if ((long)starts[i] + count > max_context)
            return fail(XRT_HOST_ERROR, "slot %d: %d + %d tokens exceed the context limit %d", slot, starts[i], count, max_context);
        token_at += count;
        want_at += want_counts[i];
    }
    return XRT_HOST_OK;
}

extern "C" int xrt_step_pack(int n_sequences, const int* slots, const int* counts, const int* starts, const int* tokens,
                             const int* want_counts, const int* wants, int pad_to, int32_t* out, long room, xrt_step_facts* facts) {
    long n_tokens = 0, n_wants = 0;
    for (int i = 0; i < n_sequences; ++i) { n_tokens += counts[i]; n_wants += want_counts[i]; }
    const long padded = std::max(n_tokens, (long)pad_to);
    if (n_sequences <= 0 || padded >= (1L << 31)) return fail(XRT_HOST_ERROR, "a step of %d sequences and %ld tokens cannot be packed", n_sequences, n_tokens);
    if (room < xrt_step_room(n_sequences, n_tokens, n_wants, pad_to))
        return fail(XRT_HOST_ERROR, "a step of %ld tokens needs %ld integers, %ld given", n_tokens, xrt_step_room(n_sequences, n_tokens, n_wants, pad_to), room);
    int32_t* ids = out;
    int32_t* positions = ids + padded;
    int32_t* token_slots = positions + padded;
    int32_t* sequence_slots = token_slots + padded;
    int32_t* offsets = sequence_slots + n_sequences;
    int32_t* sequence_starts = offsets + n_sequences + 1;
    int32_t* rows = sequence_starts + n_sequences;
    long at = 0, want_at = 0, row_at = 0;
    int max_count = 0, max_context = 0, is_decode = 1;
    offsets[0] = 0;
    for (int i = 0; i < n_sequences; ++i) {
        const int count = counts[i];
        for (int t = 0; t < count; ++t) {
            ids[at + t] = tokens[at + t];
            positions[at + t] = starts[i] + t;
            token_slots[at + t] = slots[i];
        }
        for (int w = 0; w < want_counts[i]; ++w) rows[row_at++] = (int32_t)(at + wants[want_at + w]);
        want_at += want_counts[i];
        at += count;
        offsets[i + 1] = (int32_t)at;
        sequence_slots[i] = slots[i];
        sequence_starts[i] = starts[i];
        max_count = std::max(max_count, count);
        max_context = std::max(max_context, starts[i] + count);
        if (count != 1) is_decode = 0;
    }
    for (long t = n_tokens; t < padded; ++t) { ids[t] = 0; positions[t] = 0; token_slots[t] = -1; }     // padding: computed, cached nowhere
    *facts = xrt_step_facts{(int)padded, (int)n_wants, max_count, max_context, is_decode};
    return XRT_HOST_OK;
}

// ---- the generation loop's decisions -------------------------------------------------------------------

extern "C" int xrt_loop_decide(int token, const int* stops, int n_stops, int history_length, int context, int produced,
                               int max_tokens, int* keep) {
    *keep = 0;
    for (int i = 0; i < n_stops; ++i)
        if (stops[i] == token) return XRT_FINISH_STOP;                 // session.rs:117-119: neither stored nor returned
    if (history_length >= context) return XRT_FINISH_CONTEXT;           // session.rs:120-122
    *keep = 1;
    if (produced + 1 >= max_tokens) return XRT_FINISH_LENGTH;           // session.rs:115: the loop's condition
    return XRT_GOES_ON;
}

extern "C" int xrt_loop_goes_on_whatever_it_draws(int history_length, int context, int produced, int max_tokens) {
    return history_length + 1 < context && produced + 1 < max_tokens;
}

extern "C" int xrt_loop_plan_batches(int n, const int* prompt_lengths, const int* max_tokens, int batch_size, int block_tokens,
                                     long cache_tokens, int context, int* batch_of) {
    int batch = 0, in_batch = 0;
    long used = 0;
    for (int i = 0; i < n; ++i) {
        const long final_length = std::min((long)context, (long)prompt_lengths[i] + std::max(0, max_tokens[i]));
        const long need = (final_length + block_tokens - 1) / block_tokens * block_tokens;
        if (need > cache_tokens) {
            fail(XRT_HOST_ERROR, "request %d may hold %ld tokens; the cache holds %ld", i, need, cache_tokens);
            return -1;
        }
        if (in_batch > 0 && (in_batch >= batch_size || used + need > cache_tokens)) {
            ++batch;
            in_batch = 0;
            used = 0;
        }
        batch_of[i] = batch;
        ++in_batch;
        used += need;
    }
    return n > 0 ? batch + 1 : 0;
}

// C interface of the host library: the bookkeeping of the runtime that runs on the CPU, beside the kernel
// library. The reference keeps the same things in native code (crates/xrt-runtime/src/kv_cache.rs: the pages of
// a sequence, :159-176 its rollback; crates/xrt-runtime/src/session.rs:87-124: the limits and the order of
// the loop's decisions). Here: pools of numbered slots and cache blocks, the block tables of the groups of
// layer calls, the packing of a step's sequences into the arrays the kernels read, and the decisions of the
// generation loop. Nothing in this library touches the GPU. Functions that can fail return XRT_HOST_OK,
// XRT_HOST_FULL (nothing free: the caller may wait or make room) or XRT_HOST_ERROR (a use that the state does
// not allow); xrt_host_last_error() then says what was wrong. Handles are not shared between threads.
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { XRT_HOST_OK = 0, XRT_HOST_FULL = 1, XRT_HOST_ERROR = 2 };
const char* xrt_host_last_error(void);

// ---- a pool of `size` numbered items: the lowest free one is handed out, released ones are used again
typedef struct xrt_pool xrt_pool;
xrt_pool* xrt_pool_new(int size, const char* what);        // what: "slot", "block": for messages
void xrt_pool_delete(xrt_pool* pool);
int xrt_pool_acquire(xrt_pool* pool, int* item);
int xrt_pool_release(xrt_pool* pool, int item);            // an item released twice, or never acquired, is an error
int xrt_pool_size(const xrt_pool* pool);
int xrt_pool_n_free(const xrt_pool* pool);
int xrt_pool_is_held(const xrt_pool* pool, int item);
int xrt_pool_check(const xrt_pool* pool);                  // every item free once or held

// ---- the block tables of one group of layer calls: table[slot][logical block] -> physical block, -1 = none.
// `table` is the caller's memory ([max_slots][max_blocks] int32, all -1 at the start) and stays the caller's:
// the library writes it, the caller copies changed rows to the device. window 0: a sequence keeps all its
// blocks; window W: those that a query looking at the W most recent tokens (itself included) can still see.
typedef struct xrt_tables xrt_tables;
xrt_tables* xrt_tables_new(int n_blocks, int max_slots, int max_blocks, int window, int block_tokens, int32_t* table);
void xrt_tables_delete(xrt_tables* tables);
xrt_pool* xrt_tables_pool(xrt_tables* tables);             // the group's blocks (owned by the tables)
// the blocks that tokens up to new_length need; added[0 .. *n_added) are the logical blocks acquired (room:
// max_blocks). XRT_HOST_FULL leaves the sequence as it was.
int xrt_tables_grow(xrt_tables* tables, int slot, int new_length, int* added, int* n_added);
int xrt_tables_drop(xrt_tables* tables, int slot, const int* logicals, int n);
// releases what a sequence of `length` tokens no longer needs: blocks past its end, blocks out of the window
int xrt_tables_shrink_to(xrt_tables* tables, int slot, int length);
int xrt_tables_release_all(xrt_tables* tables, int slot);
int xrt_tables_first_needed_block(const xrt_tables* tables, int length);
int xrt_tables_floor(const xrt_tables* tables, int slot);  // lowest logical block the sequence may still hold
// rows [*low, *high) have changed since the last call (0, 0: none); the call forgets them
void xrt_tables_take_changed(xrt_tables* tables, int* low, int* high);
// no block held by two sequences or by none, free slots (per slot_held[max_slots]) hold nothing
int xrt_tables_check(const xrt_tables* tables, const unsigned char* slot_held);

// ---- a step: the sequences' new tokens packed one after another.
// Checks what can be checked without the cache (llama.rs:624-626 a sequence brings at least one token,
// :1044-1049 token ids below the embedding's rows; wanted places inside the tokens given; no slot twice;
// the context limit) and returns XRT_HOST_ERROR with a message, or fills
//   out = [token ids | positions | slots] (n_tokens each, padded with token 0, position 0, slot -1 up to pad_to)
//         [sequence slots (n)] [offsets (n + 1)] [starts (n)] [rows whose logits are wanted (n_rows)]
// and the facts about the step. tokens and wants are flat, counts say how many belong to each sequence.
typedef struct xrt_step_facts { int n_tokens, n_rows, max_count, max_context, is_decode; } xrt_step_facts;
long xrt_step_room(int n_sequences, long n_tokens, long n_wants, int pad_to);      // int32 elements that `out` needs
int xrt_step_check(int n_sequences, const int* slots, const int* counts, const int* starts, const int* tokens,
                   const int* want_counts, const int* wants, int vocab, int max_context);
int xrt_step_pack(int n_sequences, const int* slots, const int* counts, const int* starts, const int* tokens,
                  const int* want_counts, const int* wants, int pad_to, int32_t* out, long room, xrt_step_facts* facts);

// ---- the generation loop's decisions (session.rs:115-124, in that order: stop token, full context, keep)
enum { XRT_GOES_ON = 0, XRT_FINISH_STOP = 1, XRT_FINISH_CONTEXT = 2, XRT_FINISH_LENGTH = 3 };
// what happens to a sampled token: *keep says whether it is stored and returned; returns why the request ends, if it does
int xrt_loop_decide(int token, const int* stops, int n_stops, int history_length, int context, int produced,
                    int max_tokens, int* keep);
// whether only a stop token can end the request at the token being sampled
int xrt_loop_goes_on_whatever_it_draws(int history_length, int context, int produced, int max_tokens);
// cuts requests, in order, into batches that fit the slots and the cache: batch_of[i] is the batch of request i;
// returns the number of batches, or -1 (message) if a request alone exceeds the cache
int xrt_loop_plan_batches(int n, const int* prompt_lengths, const int* max_tokens, int batch_size, int block_tokens,
                          long cache_tokens, int context, int* batch_of);

#ifdef __cplusplus
}
#endif

// Continuous-batching scheduler above the step function.
//
// Names after the reference's (crates/spite-scheduler/src/lib.rs:55-92: SlotState,
// BatchRequest, BatchOutput, FinishReason), whose step() is unwritten (:144-152).  Here:
//  * submit() queues a request (first come, first served) or rejects it: empty prompt, a
//    prompt longer than the context limit, or one that can never fit the page pools.
//  * schedule() builds one step under `max_batch_tokens`: first one token for every
//    request that decodes, then the next portion of prompts that are under way, then new
//    requests while a slot is free and the pools hold the pages of their first portion.
//    Portions are cut to what is left of the budget, down to one token.
//  * When a running request cannot get its next page, the running request that was
//    admitted last and is not yet part of this step is preempted: its pages and slot are
//    given back, its tokens are kept, it goes to the head of the queue and is computed
//    again later.  When nothing can be preempted the portion is cut to the pages that are
//    free; a request that cannot move at all while it is the only one running fails with
//    OutOfPages.
//  * update() takes the sampled token of every request whose last position was in the
//    step, commits the cache, finishes requests (end-of-sequence and stop tokens are not
//    emitted, crates/spite-executor/src/lib.rs:671-673) and frees what they held.
#pragma once
#include <cstdint>
#include <deque>
#include <map>
#include <string>
#include <vector>

#include "cache.h"

namespace spite {

enum SlotState { SLOT_FREE = 0, SLOT_PREFILLING = 1, SLOT_GENERATING = 2, SLOT_DONE = 3 };
enum FinishReason { NOT_DONE = 0, EOS_TOKEN = 1, STOP_TOKEN = 2, MAX_TOKENS = 3,
                    CONTEXT_LIMIT = 4, OUT_OF_PAGES = 5, CANCELLED = 6 };

struct Request {
    uint64_t id = 0;
    std::vector<int32_t> tokens;     // prompt, then what was generated
    int n_prompt = 0;
    int max_tokens = 0;
    std::vector<int32_t> stop_tokens;
    int slot = -1;
    int64_t n_computed = 0;          // positions in the cache
    int n_generated = 0;
    int n_preempted = 0;
    uint64_t admit_order = 0;
    SlotState state = SLOT_FREE;
    FinishReason reason = NOT_DONE;
};

struct BatchEntry {
    uint64_t request_id;
    int slot;
    int64_t start;       // position of the first token of the portion
    int n_tokens;
    bool wants_logits;   // the portion ends at the request's last token
};

struct BatchOutput {
    uint64_t request_id;
    int32_t token;       // -1 when the step emitted nothing for the request
    bool done;
    FinishReason finish_reason;
};

class Scheduler {
public:
    Scheduler(CacheManager* cache, int max_batch_tokens, int64_t max_context,
              const std::vector<int32_t>& eos_tokens);

    // Request id (>= 1), or 0 with `error` set.
    uint64_t submit(const std::vector<int32_t>& prompt, int max_tokens,
                    const std::vector<int32_t>& stop_tokens, std::string* error);
    // The next step.  `tokens` receives the token ids of all entries, in order.
    std::vector<BatchEntry> schedule(std::vector<int32_t>* tokens);
    // `sampled` holds one token for every entry of the last schedule() with wants_logits,
    // in order.  Returns what each of those requests emitted, and requests that failed.
    std::vector<BatchOutput> update(const std::vector<int32_t>& sampled);
    bool cancel(uint64_t id);

    int n_waiting() const { return (int)waiting_.size(); }
    int n_running() const { return (int)running_.size(); }
    int active_count() const { return n_waiting() + n_running(); }
    uint64_t n_preemptions() const { return n_preemptions_; }
    const Request* find(uint64_t id) const;

private:
    void preempt(size_t running_index);
    void finish(Request& r, FinishReason why);

    CacheManager* cache_;
    int max_batch_tokens_;
    int64_t max_context_;
    std::vector<int32_t> eos_;
    uint64_t next_id_ = 1;
    uint64_t next_order_ = 1;
    uint64_t n_preemptions_ = 0;
    std::map<uint64_t, Request> requests_;     // live and finished-but-unread
    std::deque<uint64_t> waiting_;
    std::vector<uint64_t> running_;            // in order of admission
    std::vector<BatchEntry> last_batch_;
    std::vector<BatchOutput> pending_failures_;
};

}  // namespace spite

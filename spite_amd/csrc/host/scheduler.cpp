#include "scheduler.h"

#include <algorithm>
#include <set>
#include <stdexcept>

namespace spite {

Scheduler::Scheduler(CacheManager* cache, int max_batch_tokens, int64_t max_context,
                     const std::vector<int32_t>& eos_tokens)
    : cache_(cache), max_batch_tokens_(max_batch_tokens), max_context_(max_context), eos_(eos_tokens) {
    if (!cache) throw std::invalid_argument("scheduler needs a cache manager");
    if (max_batch_tokens < 1) throw std::invalid_argument("max_batch_tokens must be >= 1");
    if (max_context < 1) throw std::invalid_argument("max_context must be >= 1");
}

uint64_t Scheduler::submit(const std::vector<int32_t>& prompt, int max_tokens,
                           const std::vector<int32_t>& stop_tokens, std::string* error) {
    auto fail = [&](const std::string& m) { if (error) *error = m; return (uint64_t)0; };
    if (prompt.empty()) return fail("empty prompt");
    if (max_tokens < 0) return fail("max_tokens must be >= 0");
    if ((int64_t)prompt.size() > max_context_)
        return fail("prompt of " + std::to_string(prompt.size()) + " tokens is longer than the context limit " +
                    std::to_string(max_context_));
    for (int g = 0; g < cache_->n_groups(); ++g) {
        const int64_t need = cache_->peak_pages((int64_t)prompt.size(), max_batch_tokens_, g);
        if (need > cache_->total_pages(g))
            return fail("prompt of " + std::to_string(prompt.size()) + " tokens needs " + std::to_string(need) +
                        " pages of group " + std::to_string(g) + ", the pool has " +
                        std::to_string(cache_->total_pages(g)));
    }
    Request r;
    r.id = next_id_++;
    r.tokens = prompt;
    r.n_prompt = (int)prompt.size();
    r.max_tokens = max_tokens;
    r.stop_tokens = stop_tokens;
    requests_[r.id] = std::move(r);
    waiting_.push_back(next_id_ - 1);
    return next_id_ - 1;
}

const Request* Scheduler::find(uint64_t id) const {
    auto it = requests_.find(id);
    return it == requests_.end() ? nullptr : &it->second;
}

void Scheduler::preempt(size_t running_index) {
    Request& r = requests_[running_[running_index]];
    cache_->release(r.slot);
    r.slot = -1;
    r.n_computed = 0;
    r.state = SLOT_FREE;
    r.n_preempted += 1;
    n_preemptions_ += 1;
    waiting_.push_front(r.id);
    running_.erase(running_.begin() + running_index);
}

void Scheduler::finish(Request& r, FinishReason why) {
    if (r.slot >= 0) cache_->release(r.slot);
    r.slot = -1;
    r.state = SLOT_DONE;
    r.reason = why;
    auto it = std::find(running_.begin(), running_.end(), r.id);
    if (it != running_.end()) running_.erase(it);
    auto wt = std::find(waiting_.begin(), waiting_.end(), r.id);
    if (wt != waiting_.end()) waiting_.erase(wt);
}

std::vector<BatchEntry> Scheduler::schedule(std::vector<int32_t>* tokens) {
    std::vector<BatchEntry> batch;
    if (tokens) tokens->clear();
    int budget = max_batch_tokens_;
    std::set<uint64_t> placed;

    auto place = [&](Request& r, int n) {
        BatchEntry e;
        e.request_id = r.id;
        e.slot = r.slot;
        e.start = r.n_computed;
        e.n_tokens = n;
        e.wants_logits = r.n_computed + n == (int64_t)r.tokens.size();
        batch.push_back(e);
        if (tokens) tokens->insert(tokens->end(), r.tokens.begin() + r.n_computed, r.tokens.begin() + r.n_computed + n);
        budget -= n;
        placed.insert(r.id);
    };

    // Requests that decode first, then prompts under way; each in order of admission.
    std::vector<uint64_t> order;
    for (uint64_t id : running_)
        if ((int64_t)requests_[id].tokens.size() - requests_[id].n_computed == 1) order.push_back(id);
    for (uint64_t id : running_)
        if ((int64_t)requests_[id].tokens.size() - requests_[id].n_computed != 1) order.push_back(id);

    for (uint64_t id : order) {
        if (budget <= 0) break;
        if (std::find(running_.begin(), running_.end(), id) == running_.end()) continue;  // preempted meanwhile
        Request& r = requests_[id];
        int64_t n = std::min<int64_t>((int64_t)r.tokens.size() - r.n_computed, budget);
        while (n > 0 && !cache_->can_reserve(r.slot, n)) {
            // the running request admitted last, later than this one, not yet in the step
            int victim = -1;
            for (int i = (int)running_.size() - 1; i >= 0; --i) {
                const Request& c = requests_[running_[i]];
                if (c.id != r.id && !placed.count(c.id) && c.admit_order > r.admit_order) { victim = i; break; }
            }
            if (victim >= 0) { preempt((size_t)victim); continue; }
            // cut the portion to the pages that are free
            int64_t fit = n;
            for (int g = 0; g < cache_->n_groups(); ++g) {
                const int64_t rows = ((int64_t)cache_->table(r.slot, g).size() + cache_->free_pages(g)) * cache_->page_size();
                fit = std::min(fit, rows - r.n_computed);
            }
            n = std::max<int64_t>(fit, 0);
            if (n == 0 && placed.empty() && running_.size() == 1) {
                // alone and unable to move: no later step can help
                BatchOutput out{r.id, -1, true, OUT_OF_PAGES};
                finish(r, OUT_OF_PAGES);
                pending_failures_.push_back(out);
            }
            break;
        }
        if (n <= 0 || r.state == SLOT_DONE) continue;
        cache_->reserve(r.slot, n);
        place(r, (int)n);
    }

    // New requests, first come first served, while nothing is short.
    while (budget > 0 && !waiting_.empty() && cache_->free_slots() > 0) {
        Request& r = requests_[waiting_.front()];
        const int64_t n = std::min<int64_t>((int64_t)r.tokens.size(), budget);
        if (!cache_->can_reserve_new(n)) {
            if (running_.empty() && batch.empty()) {
                // the pools are empty of other requests and still too small for this portion:
                // take what fits, so that a chunked group can roll on
                int64_t fit = n;
                for (int g = 0; g < cache_->n_groups(); ++g)
                    fit = std::min<int64_t>(fit, (int64_t)cache_->free_pages(g) * cache_->page_size());
                if (fit < 1) break;
                r.slot = cache_->admit();
                cache_->reserve(r.slot, fit);
                r.admit_order = next_order_++;
                r.state = SLOT_PREFILLING;
                r.n_computed = 0;
                running_.push_back(r.id);
                waiting_.pop_front();
                place(r, (int)fit);
            }
            break;
        }
        r.slot = cache_->admit();
        cache_->reserve(r.slot, n);
        r.admit_order = next_order_++;
        r.state = SLOT_PREFILLING;
        r.n_computed = 0;
        running_.push_back(r.id);
        waiting_.pop_front();
        place(r, (int)n);
    }
    last_batch_ = batch;
    return batch;
}

std::vector<BatchOutput> Scheduler::update(const std::vector<int32_t>& sampled) {
    std::vector<BatchOutput> outs;
    outs.swap(pending_failures_);
    size_t k = 0;
    size_t wanted = 0;
    for (const auto& e : last_batch_) wanted += e.wants_logits;
    if (sampled.size() != wanted)
        throw std::invalid_argument("update: " + std::to_string(sampled.size()) + " tokens for " +
                                    std::to_string(wanted) + " requests that asked for one");
    for (const auto& e : last_batch_) {
        auto it = requests_.find(e.request_id);
        if (it == requests_.end() || it->second.state == SLOT_DONE) { if (e.wants_logits) ++k; continue; }
        Request& r = it->second;
        cache_->commit(r.slot, e.n_tokens);
        r.n_computed += e.n_tokens;
        if (!e.wants_logits) continue;
        const int32_t tok = sampled[k++];
        BatchOutput out{r.id, -1, false, NOT_DONE};
        if (r.n_generated >= r.max_tokens) {
            out.done = true; out.finish_reason = MAX_TOKENS;
        } else if (std::find(eos_.begin(), eos_.end(), tok) != eos_.end()) {
            out.done = true; out.finish_reason = EOS_TOKEN;
        } else if (std::find(r.stop_tokens.begin(), r.stop_tokens.end(), tok) != r.stop_tokens.end()) {
            out.done = true; out.finish_reason = STOP_TOKEN;
        } else {
            r.tokens.push_back(tok);
            r.n_generated += 1;
            r.state = SLOT_GENERATING;
            out.token = tok;
            if (r.n_generated >= r.max_tokens) { out.done = true; out.finish_reason = MAX_TOKENS; }
            else if ((int64_t)r.tokens.size() >= max_context_) { out.done = true; out.finish_reason = CONTEXT_LIMIT; }
        }
        if (out.done) finish(r, out.finish_reason);
        outs.push_back(out);
    }
    last_batch_.clear();
    for (const auto& o : outs)
        if (o.done) requests_.erase(o.request_id);
    return outs;
}

bool Scheduler::cancel(uint64_t id) {
    auto it = requests_.find(id);
    if (it == requests_.end() || it->second.state == SLOT_DONE) return false;
    finish(it->second, CANCELLED);
    requests_.erase(it);   // update() skips the entry that a step under way may still hold
    return true;
}

}  // namespace spite

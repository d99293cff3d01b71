// C interface of the host runtime (cache manager and scheduler) for the Python binding.
// Every function catches C++ exceptions; the text of the last one is kept per thread.
#include <cstring>
#include <string>
#include <vector>

#include "cache.h"
#include "scheduler.h"

using namespace spite;

static thread_local std::string g_error;
#define SP_TRY try {
#define SP_CATCH(ret) } catch (const std::exception& e) { g_error = e.what(); return ret; }

extern "C" {

const char* spite_host_last_error() { return g_error.c_str(); }
int spite_host_abi_version() { return 1; }

// ---------------------------------------------------------------- cache manager
void* spc_create(int page_size, int max_requests, int n_groups, const int* kinds, const int* spans,
                 const int* n_pages) {
    SP_TRY
    std::vector<GroupSpec> gs;
    for (int i = 0; i < n_groups; ++i) gs.push_back(GroupSpec{kinds[i], spans[i], n_pages[i]});
    return (void*)new CacheManager(page_size, max_requests, gs);
    SP_CATCH(nullptr)
}
void spc_destroy(void* c) { delete (CacheManager*)c; }
int spc_admit(void* c) { return ((CacheManager*)c)->admit(); }
int spc_take_fresh(void* c, int* out, int cap) { return ((CacheManager*)c)->take_fresh(out, cap); }
int spc_fill_step(void* c, int n, const int* slots, const int* starts, const int* counts, int g, int width,
                  int* slot_map, int* table) {
    return ((CacheManager*)c)->fill_step(n, slots, starts, counts, g, width, slot_map, table);
}
int spc_live(void* c, int slot) { return ((CacheManager*)c)->live(slot); }
long long spc_cached(void* c, int slot) { return ((CacheManager*)c)->cached(slot); }
int spc_can_reserve(void* c, int slot, long long n) { return ((CacheManager*)c)->can_reserve(slot, n); }
int spc_can_reserve_new(void* c, long long n) { return ((CacheManager*)c)->can_reserve_new(n); }
int spc_reserve(void* c, int slot, long long n) { return ((CacheManager*)c)->reserve(slot, n); }
int spc_reserve_all(void* c, int n, const int* slots, const long long* counts) {
    return ((CacheManager*)c)->reserve_all(n, slots, (const int64_t*)counts);
}
int spc_commit(void* c, int slot, long long n) { return ((CacheManager*)c)->commit(slot, n); }
int spc_release(void* c, int slot) { return ((CacheManager*)c)->release(slot); }
int spc_free_pages(void* c, int g) { return ((CacheManager*)c)->free_pages(g); }
int spc_total_pages(void* c, int g) { return ((CacheManager*)c)->total_pages(g); }
int spc_free_slots(void* c) { return ((CacheManager*)c)->free_slots(); }
long long spc_peak_pages(void* c, long long total, long long portion, int g) {
    return ((CacheManager*)c)->peak_pages(total, portion, g);
}
// Copies the block table of (slot, group) into out[0..cap); returns its length.
int spc_table(void* c, int slot, int g, int* out, int cap) {
    CacheManager* m = (CacheManager*)c;
    if (!m->live(slot)) return -2;
    const auto& t = m->table(slot, g);
    for (int i = 0; i < (int)t.size() && i < cap; ++i) out[i] = t[i];
    return (int)t.size();
}
int spc_table_len(void* c, int slot, int g) {
    CacheManager* m = (CacheManager*)c;
    return m->live(slot) ? (int)m->table(slot, g).size() : -2;
}
int spc_slot_mapping(void* c, int slot, int g, long long start, long long n, int* out) {
    CacheManager* m = (CacheManager*)c;
    if (!m->live(slot)) return -2;
    m->slot_mapping(slot, g, start, n, out);
    return 0;
}
// 0 when the books balance, else -1 and the finding in spite_host_last_error().
int spc_check(void* c) {
    std::string s = ((CacheManager*)c)->check();
    if (s.empty()) return 0;
    g_error = s;
    return -1;
}

// ---------------------------------------------------------------- scheduler
void* sps_create(void* cache, int max_batch_tokens, long long max_context, const int* eos, int n_eos) {
    SP_TRY
    return (void*)new Scheduler((CacheManager*)cache, max_batch_tokens, max_context,
                                std::vector<int32_t>(eos, eos + n_eos));
    SP_CATCH(nullptr)
}
void sps_destroy(void* s) { delete (Scheduler*)s; }
unsigned long long sps_submit(void* s, const int* prompt, int n, int max_tokens, const int* stop, int n_stop) {
    SP_TRY
    std::string err;
    uint64_t id = ((Scheduler*)s)->submit(std::vector<int32_t>(prompt, prompt + n), max_tokens,
                                          std::vector<int32_t>(stop, stop + n_stop), &err);
    if (!id) g_error = err;
    return id;
    SP_CATCH(0)
}
// Fills one row per entry; returns the number of entries, or -1 when a capacity is short.
// `n_tokens_out` receives the total number of tokens.
int sps_schedule(void* s, int cap_entries, int cap_tokens, unsigned long long* req_ids, int* slots,
                 long long* starts, int* counts, int* wants, int* tokens, int* n_tokens_out) {
    SP_TRY
    std::vector<int32_t> toks;
    auto batch = ((Scheduler*)s)->schedule(&toks);
    if ((int)batch.size() > cap_entries || (int)toks.size() > cap_tokens) {
        g_error = "schedule: caller's buffers are too small";
        return -1;
    }
    for (size_t i = 0; i < batch.size(); ++i) {
        req_ids[i] = batch[i].request_id; slots[i] = batch[i].slot; starts[i] = batch[i].start;
        counts[i] = batch[i].n_tokens; wants[i] = batch[i].wants_logits;
    }
    if (!toks.empty()) std::memcpy(tokens, toks.data(), toks.size() * sizeof(int32_t));
    *n_tokens_out = (int)toks.size();
    return (int)batch.size();
    SP_CATCH(-1)
}
int sps_update(void* s, const int* sampled, int n_sampled, int cap, unsigned long long* req_ids, int* tokens,
               int* done, int* reasons) {
    SP_TRY
    auto outs = ((Scheduler*)s)->update(std::vector<int32_t>(sampled, sampled + n_sampled));
    if ((int)outs.size() > cap) { g_error = "update: caller's buffers are too small"; return -1; }
    for (size_t i = 0; i < outs.size(); ++i) {
        req_ids[i] = outs[i].request_id; tokens[i] = outs[i].token; done[i] = outs[i].done;
        reasons[i] = outs[i].finish_reason;
    }
    return (int)outs.size();
    SP_CATCH(-1)
}
int sps_cancel(void* s, unsigned long long id) { return ((Scheduler*)s)->cancel(id); }
int sps_n_waiting(void* s) { return ((Scheduler*)s)->n_waiting(); }
int sps_n_running(void* s) { return ((Scheduler*)s)->n_running(); }
unsigned long long sps_n_preemptions(void* s) { return ((Scheduler*)s)->n_preemptions(); }
// state, slot, n_computed, n_generated, n_preempted of a live request; -1 when unknown.
int sps_request_info(void* s, unsigned long long id, long long* out5) {
    const Request* r = ((Scheduler*)s)->find(id);
    if (!r) return -1;
    out5[0] = r->state; out5[1] = r->slot; out5[2] = r->n_computed; out5[3] = r->n_generated;
    out5[4] = r->n_preempted;
    return 0;
}

}  // extern "C"

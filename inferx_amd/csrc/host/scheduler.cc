// The scheduler: all policy, no GPU.  It decides who runs, in which portions,
// and what gives when pages run out.  Part of libinferx_host.so; it drives the
// cache manager of cache.cc through that file's C interface.
//
// Policies are the reference's (src/scheduler/scheduler.cc):
//   admission   first come first served while fewer than `max_running` run; pages
//               for the whole prompt are reserved; on a shortage the request stays
//               at the head of the queue and admission stops (:294-370)
//   budget      at most `max_batch_tokens` tokens a step; sequences with one
//               pending token (decodes, last one-token portions) first, then
//               prompts in running order take min(pending, budget) (:255-291)
//   pages out   for a running sequence: the most recently admitted sequence is
//               preempted (pages back, starts over with prompt + generated tokens,
//               head of the queue); if the requester is the newest, the next
//               newest yields; if it runs alone it finishes out_of_memory
//               (:444-510, :206-229)
//   context     a sequence that would pass `max_seq_len` finishes context_limit
//   finishing   stop token (kept in the output), max_tokens, cancel (:677-758)
// Pages go back the moment a sequence finishes or is preempted (:231-245).
#include <algorithm>
#include <cstdint>
#include <deque>
#include <memory>
#include <string>
#include <vector>

extern "C" {
int ixh_cache_add(void* h, int64_t rid);
int ixh_cache_free(void* h, int64_t rid);
int ixh_cache_reserve(void* h, int64_t rid, int64_t new_len);
int ixh_cache_commit(void* h, int64_t rid, int64_t tokens);
int64_t ixh_cache_cached(void* h, int64_t rid);
int ixh_cache_contains(void* h, int64_t rid);
int ixh_cache_can_add(void* h);
}

namespace {

enum Reserve { kOk = 0, kPoolEmpty = 1, kContextFull = 2 };  // what ixh_cache_reserve returns
enum Finish { kStop = 0, kLength = 1, kCancelled = 2, kContext = 3, kOutOfMemory = 4 };

struct Seq {
  int64_t rid = 0;
  std::vector<int32_t> tokens;
  int32_t prompt_len = 0;
  int64_t max_tokens = 0, min_tokens = 0;
  std::vector<int32_t> stop;
  bool cancelled = false;
  int64_t draws = 0;  // sampled tokens so far: the counter of this request's random stream
  int64_t generated() const { return static_cast<int64_t>(tokens.size()) - prompt_len; }
};

struct Done {
  int64_t rid;
  int reason;
  std::vector<int32_t> output;
};

struct Part {  // one sequence's share of a step
  Seq* seq;
  int64_t first;
  int32_t count;
  bool samples;
};

struct Sched {
  void* cache;
  int max_running;
  int64_t max_batch_tokens, max_seq_len;
  std::deque<std::unique_ptr<Seq>> waiting;
  std::vector<std::unique_ptr<Seq>> running;
  std::vector<Done> completed;
  std::vector<Part> plan;
  bool planned = false;
  int64_t preemptions = 0;
  std::string error;

  int64_t pending(const Seq& s) const { return static_cast<int64_t>(s.tokens.size()) - ixh_cache_cached(cache, s.rid); }

  void retire(std::unique_ptr<Seq> s, int reason) {
    completed.push_back({s->rid, reason, std::vector<int32_t>(s->tokens.begin() + s->prompt_len, s->tokens.end())});
    if (ixh_cache_contains(cache, s->rid)) ixh_cache_free(cache, s->rid);
  }

  void preempt(size_t index) {
    std::unique_ptr<Seq> victim = std::move(running[index]);
    running.erase(running.begin() + static_cast<std::ptrdiff_t>(index));
    ixh_cache_free(cache, victim->rid);
    waiting.push_front(std::move(victim));
    ++preemptions;
  }

  void admit() {
    while (!waiting.empty() && static_cast<int>(running.size()) < max_running) {
      Seq& s = *waiting.front();
      if (s.cancelled || static_cast<int64_t>(s.tokens.size()) > max_seq_len) {
        const int reason = s.cancelled ? kCancelled : kOutOfMemory;
        std::unique_ptr<Seq> gone = std::move(waiting.front());
        waiting.pop_front();
        retire(std::move(gone), reason);
        continue;
      }
      if (!ixh_cache_can_add(cache)) return;
      ixh_cache_add(cache, s.rid);
      if (ixh_cache_reserve(cache, s.rid, static_cast<int64_t>(s.tokens.size())) != kOk) {
        ixh_cache_free(cache, s.rid);  // not a preemption site: it waits at the head of the queue
        return;
      }
      running.push_back(std::move(waiting.front()));
      waiting.pop_front();
    }
  }

  std::vector<int64_t> take() const {
    std::vector<int64_t> t(running.size(), 0), pend(running.size(), 0);
    int64_t budget = max_batch_tokens;
    for (size_t i = 0; i < running.size(); ++i) {
      pend[i] = pending(*running[i]);
      if (budget > 0 && pend[i] == 1) {
        t[i] = 1;
        --budget;
      }
    }
    for (size_t i = 0; i < running.size(); ++i)
      if (budget > 0 && pend[i] > 1) {
        t[i] = std::min(pend[i], budget);
        budget -= t[i];
      }
    return t;
  }

  // number of contributions (0: nothing can run), -1: called twice without a commit
  int prepare() {
    if (planned) {
      error = "prepare_step called twice without commit_step";
      return -1;
    }
    for (size_t i = 0; i < running.size();) {
      if (running[i]->cancelled) {
        std::unique_ptr<Seq> gone = std::move(running[i]);
        running.erase(running.begin() + static_cast<std::ptrdiff_t>(i));
        retire(std::move(gone), kCancelled);
      } else {
        ++i;
      }
    }
    admit();
    std::vector<int64_t> t;
    const size_t rounds = running.size() + 1;
    for (size_t round = 0; round < rounds; ++round) {
      if (running.empty()) return 0;
      t = take();
      bool replan = false;
      for (size_t i = 0; i < running.size(); ++i) {
        if (t[i] == 0) continue;
        Seq& s = *running[i];
        const int status = ixh_cache_reserve(cache, s.rid, ixh_cache_cached(cache, s.rid) + t[i]);
        if (status == kOk) continue;
        if (status == kContextFull) {
          std::unique_ptr<Seq> gone = std::move(running[i]);
          running.erase(running.begin() + static_cast<std::ptrdiff_t>(i));
          retire(std::move(gone), kContext);
        } else {
          size_t victim = running.size() - 1;
          if (victim == i) {
            if (running.size() == 1) {
              std::unique_ptr<Seq> gone = std::move(running[i]);
              running.erase(running.begin());
              retire(std::move(gone), kOutOfMemory);
              replan = true;
              break;
            }
            victim = running.size() - 2;
          }
          preempt(victim);
        }
        replan = true;
        break;
      }
      if (!replan) break;
    }
    if (running.empty()) return 0;
    plan.clear();
    for (size_t i = 0; i < running.size(); ++i) {
      if (i >= t.size() || t[i] == 0) continue;
      Seq& s = *running[i];
      const int64_t at = ixh_cache_cached(cache, s.rid);
      plan.push_back({&s, at, static_cast<int32_t>(t[i]), at + t[i] == static_cast<int64_t>(s.tokens.size())});
    }
    if (plan.empty()) return 0;
    planned = true;
    return static_cast<int>(plan.size());
  }

  int commit(const int32_t* sampled, int n) {
    if (!planned) {
      error = "commit_step without prepare_step";
      return -1;
    }
    int want = 0;
    for (const Part& p : plan) want += p.samples ? 1 : 0;
    if (n != want) {
      error = std::to_string(n) + " sampled tokens for " + std::to_string(want) + " sampling rows";
      return -2;
    }
    planned = false;
    std::vector<std::pair<Seq*, int>> finished;
    int next = 0;
    for (const Part& p : plan) {
      Seq& s = *p.seq;
      ixh_cache_commit(cache, s.rid, p.count);
      if (!p.samples) continue;
      const int32_t token = sampled[next++];
      s.tokens.push_back(token);
      ++s.draws;
      const bool is_stop = std::find(s.stop.begin(), s.stop.end(), token) != s.stop.end();
      if (is_stop && s.generated() > s.min_tokens)
        finished.push_back({&s, kStop});
      else if (s.generated() >= s.max_tokens)
        finished.push_back({&s, kLength});
    }
    plan.clear();
    for (auto& f : finished)
      for (size_t i = 0; i < running.size(); ++i)
        if (running[i].get() == f.first) {
          std::unique_ptr<Seq> gone = std::move(running[i]);
          running.erase(running.begin() + static_cast<std::ptrdiff_t>(i));
          retire(std::move(gone), f.second);
          break;
        }
    return 0;
  }

  Seq* find(int64_t rid) {
    for (auto& s : running)
      if (s->rid == rid) return s.get();
    for (auto& s : waiting)
      if (s->rid == rid) return s.get();
    return nullptr;
  }
};

Sched* S(void* h) { return static_cast<Sched*>(h); }

}  // namespace

extern "C" {

void* ixh_sched_create(void* cache, int max_running, int64_t max_batch_tokens, int64_t max_seq_len) {
  if (cache == nullptr || max_running <= 0 || max_batch_tokens <= 0 || max_seq_len <= 0) return nullptr;
  Sched* s = new Sched();
  s->cache = cache;
  s->max_running = max_running;
  s->max_batch_tokens = max_batch_tokens;
  s->max_seq_len = max_seq_len;
  return s;
}
void ixh_sched_destroy(void* h) { delete S(h); }
const char* ixh_sched_error(void* h) { return S(h)->error.c_str(); }

// 0 ok, -1 empty prompt, -2 the request is already known
int ixh_sched_add(void* h, int64_t rid, const int32_t* prompt, int n, int64_t max_tokens, int64_t min_tokens,
                  const int32_t* stop, int n_stop) {
  if (n <= 0) return -1;
  if (S(h)->find(rid) != nullptr) return -2;
  std::unique_ptr<Seq> s(new Seq());
  s->rid = rid;
  s->tokens.assign(prompt, prompt + n);
  s->prompt_len = n;
  s->max_tokens = max_tokens;
  s->min_tokens = min_tokens;
  if (n_stop > 0) s->stop.assign(stop, stop + n_stop);
  S(h)->waiting.push_back(std::move(s));
  return 0;
}
void ixh_sched_cancel(void* h, int64_t rid) {
  if (Seq* s = S(h)->find(rid)) s->cancelled = true;
}
int ixh_sched_has_work(void* h) { return (!S(h)->waiting.empty() || !S(h)->running.empty()) ? 1 : 0; }
int64_t ixh_sched_preemptions(void* h) { return S(h)->preemptions; }

int ixh_sched_prepare(void* h) { return S(h)->prepare(); }
int64_t ixh_sched_plan_tokens(void* h) {
  int64_t n = 0;
  for (const Part& p : S(h)->plan) n += p.count;
  return n;
}
// the plan of the step: per contribution the request, its first position, its number of tokens, whether its last
// row gives the next token, and (flat, `tokens` with room for ixh_sched_plan_tokens numbers) the tokens
void ixh_sched_plan(void* h, int64_t* rids, int64_t* first, int32_t* counts, int32_t* samples, int32_t* tokens) {
  size_t at = 0, i = 0;
  for (const Part& p : S(h)->plan) {
    rids[i] = p.seq->rid;
    first[i] = p.first;
    counts[i] = p.count;
    samples[i] = p.samples ? 1 : 0;
    std::copy(p.seq->tokens.begin() + p.first, p.seq->tokens.begin() + p.first + p.count, tokens + at);
    at += static_cast<size_t>(p.count);
    ++i;
  }
}
int ixh_sched_commit(void* h, const int32_t* sampled, int n) { return S(h)->commit(sampled, n); }

int ixh_sched_num_completed(void* h) { return static_cast<int>(S(h)->completed.size()); }
void ixh_sched_completed(void* h, int i, int64_t* rid, int32_t* reason, int32_t* n_out) {
  const Done& d = S(h)->completed[static_cast<size_t>(i)];
  *rid = d.rid;
  *reason = d.reason;
  *n_out = static_cast<int32_t>(d.output.size());
}
void ixh_sched_completed_tokens(void* h, int i, int32_t* out) {
  const Done& d = S(h)->completed[static_cast<size_t>(i)];
  std::copy(d.output.begin(), d.output.end(), out);
}
void ixh_sched_clear_completed(void* h) { S(h)->completed.clear(); }

// which = 0: the running sequences in order of admission, 1: the waiting ones from the head of the queue
int ixh_sched_list(void* h, int which, int64_t* out, int cap) {
  int n = 0;
  if (which == 0) {
    for (auto& s : S(h)->running)
      if (n < cap) out[n++] = s->rid;
    return static_cast<int>(S(h)->running.size());
  }
  for (auto& s : S(h)->waiting)
    if (n < cap) out[n++] = s->rid;
  return static_cast<int>(S(h)->waiting.size());
}
// 0 ok, -1 unknown request
int ixh_sched_seq_info(void* h, int64_t rid, int32_t* prompt_len, int64_t* n_tokens, int64_t* draws) {
  Seq* s = S(h)->find(rid);
  if (s == nullptr) return -1;
  *prompt_len = s->prompt_len;
  *n_tokens = static_cast<int64_t>(s->tokens.size());
  *draws = s->draws;
  return 0;
}
int ixh_sched_seq_tokens(void* h, int64_t rid, int64_t from, int32_t* out, int64_t cap) {
  Seq* s = S(h)->find(rid);
  if (s == nullptr) return -1;
  int64_t n = 0;
  for (int64_t i = from; i < static_cast<int64_t>(s->tokens.size()) && n < cap; ++i) out[n++] = s->tokens[static_cast<size_t>(i)];
  return static_cast<int>(n);
}

}  // extern "C"
